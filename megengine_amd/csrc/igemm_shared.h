// Declarations shared by the implicit-GEMM kernels (register-staged and LDS-direct variants).
#pragma once
#include "common.h"

namespace mi355 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int IG_THREADS = 256;
constexpr int IG_MAX_ENTRIES = 4096;  // k-unit table capacity (entries of 8 bytes: 32 KiB of LDS when full)

struct IgemmArgs {
    const int8_t* src;
    const int8_t* flt;
    const int32_t* bias;
    const int8_t* z;
    int8_t* dst;
    uint32_t src_bytes, flt_bytes, z_bytes, dst_bytes;
    int IH, IW, OH, OW, OHW;
    int FH, FW, T;
    int sh, sw, ph, pw;
    int OC;
    int M;            // n * oh * ow
    int kbytes;       // filter bytes per output channel
    int KC;           // 32-byte k-chunks (ceil)
    int entries;      // valid k-unit table entries (KC for NCHW32, ic/4*T for NCHW4)
    int nstages;
    int src_sn, src_scb;      // bytes: per image, per channel block
    int dst_sn, dst_scb;      // bytes: per image, per output channel block
    int z_sn;
    int tiles_m, tiles_n, tiles;
    int has_bias;
    FastDiv div_ohw, div_ow, div_t, div_fw;
    EpiParams epi;
    // filter addressing of the second-generation kernel (conv_igemm2.hip): byte offset of 16-byte half h of k-chunk kc of
    // output channel oc = oc * flt_rstride + kc * flt_kstride + 16 h.  The reference layout has (kbytes, 32); the
    // pre-processed layout [k-chunk][channel][32 bytes] has (32, 32 * padded channel count)
    int flt_rstride, flt_kstride;
    // group convolution: ocpg output channels per group, src_sg bytes between the channel blocks of two groups
    int groups, ocpg, src_sg, tiles_m_pg;
    int zslots;  // residual slots in LDS: 0 (no residual), 1 or 2
    // general epilogue (second-generation kernel): QuantizedS32 dst, full-shape bias, or scales outside the fast
    // forms' envelope.  bias_full: a.bias has the shape of dst (contiguous) and has_bias is 0.
    int general, dst_s32, bias_full;
    // planar destination (format NCHW4_NCHW, register-staged kernel): dst_f32 = dst, bias and z are Float32 tensors
    int dst_f32;
    // tile decoding of the LDS-direct kernels without run-time integer divisions (each costs ~30 scalar instructions and a
    // reciprocal on the critical path from kernel entry to the first copy): by the number of channel tiles, by the
    // channel tiles of a group, and by the tile stride of a workgroup (set by the launch code, which knows the grid)
    FastDiv div_tiles_m, div_tiles_m_pg, div_step;
    // patch-staged kernel (conv_igemm3.hip): batch size, padded row width and rows per padded image, patch pixels
    // (a multiple of 64), patch copies per wave, channel blocks of the reduction
    int NB, p_w, p_himg, pxp, pcw, cbs;
    FastDiv div_pw, div_phimg;
    int dry_run;  // host only: the launch code stops before anything is launched and reports whether the tile fits
    // residual table form (epi.zlin), host only: the 256 offsets, indexed by the residual byte as an unsigned value.  The
    // launch code of a kernel that takes the form hands them over in a kernel argument of their own (ResidualTable): a
    // kilobyte inside this struct made every launch of every kernel ~0.2 us slower.
    const float* ztab;
};

struct ResidualTable {
    float v[256];
};
struct NoResidualTable {};

struct KEntry {
    int off;    // byte offset of the k-unit relative to the pixel's (ih0, iw0) base
    int fhfw;   // fh | fw << 16 ; fh = 0x4000 marks a padding entry (never valid)
};

// 16-byte slot swizzle (S = slots per row), derived from how gfx950 serves 128-bit LDS accesses
// (measured with SQ_LDS_BANK_CONFLICT on single-wave probes):
//   ds_read_b128 : 64 banks; 4 passes over all 64 lanes; in pass k lane l reads dword (k + l/16) % 4
//   ds_write_b128: behaves as 32 banks; half-wave at a time, 4 passes; lane l writes dword (k + l/8) % 4
// MFMA fragment reads (lane -> row l%32, slot-half l/32) need, per row class (row mod 256/ROWB rows),
// distinct slots for the rows of one 16-lane group; loader writes (lane -> row l/2, half l%2) need
// disjoint slot pairs for the rows of one 8-lane group.  With r_i = bit i of the row:
template <int S>
__device__ __forceinline__ int swz(int row) {
    const int r0 = row & 1, r1 = (row >> 1) & 1, r2 = (row >> 2) & 1, r3 = (row >> 3) & 1;
    if (S == 4) return ((r1 ^ r2) << 1) | r3;
    if (S == 8) return (r1 << 2) | ((r0 ^ r2) << 1) | r3;
    if (S == 16) return r2 | (r0 << 1) | (r1 << 2) | (r3 << 3);
    return 0;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

constexpr int SENT = (int)0x80000000;  // byte offset that is out of range for every buffer (< 2 GiB)

// Residual (z) of one wave tile in the order the epilogue consumes it: POUT = 32: one 16-byte vector per 32x32 block
// (16 consecutive channels of the lane's pixel); POUT = 4: four dwords per block.
template <int MT, int NT>
struct ZRegs {
    v4i v[MT][NT];
};

// Fetches the whole wave tile's residual at once, so that a caller can issue it ahead of the epilogue
template <int POUT, int MT, int NT>
__device__ __forceinline__ void igemm_load_z(const IgemmArgs& a, ZRegs<MT, NT>& zr, int oc_w, int pix_w, int l32, int lh,
                                             int m_end = -1) {
    const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(a.z, a.z_bytes);
    if (m_end < 0) m_end = a.M;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int m = pix_w + j * 32 + l32;
        const bool pok = m < m_end;
        const uint32_t mm = pok ? m : 0;
        const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
        const int z_pix = (int)n * a.z_sn + (int)rem * POUT;
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int ocb = oc_w + i * 32;
            if (POUT == 32) {
                const int blk_off = (ocb >> 5) * a.dst_scb + lh * 16;
                zr.v[i][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_z, (pok && ocb < a.OC) ? z_pix + blk_off : SENT, 0, 0);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int oc4 = ocb + 8 * q + 4 * lh;
                    const int off = (oc4 >> 2) * a.dst_scb;
                    zr.v[i][j][q] = __builtin_amdgcn_raw_buffer_load_b32(rs_z, (pok && oc4 < a.OC) ? z_pix + off : SENT, 0, 0);
                }
            }
        }
    }
}

// ZPRE: the residual was fetched by igemm_load_z into *zr; otherwise it is loaded here, block by block
// blk_mod > 1: only the blocks b = i * NT + j with b % blk_mod == blk_rem are written (a wave of a workgroup that
// splits the reduction finishes its share of the blocks; wave-uniform)
// m_end: one past the last pixel (flattened over batch and image) this tile may write
// zt: the residual table in LDS (NL_ZLIN only)
template <int POUT, int MT, int NT, int NL, bool HZ, bool ZPRE>
__device__ __forceinline__ void igemm_epilogue(const IgemmArgs& a, v16i (&acc)[MT][NT], const ZRegs<MT, NT>* zr, int oc_w,
                                               int pix_w, int l32, int lh, int oc_end, int blk_mod, int blk_rem, int m_end,
                                               const float* zt = nullptr) {
    const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(a.z, HZ ? a.z_bytes : 0);
    // stores go through a buffer descriptor: a lane outside the tile carries the out-of-range offset and its store is
    // dropped (no branch, no 64-bit address arithmetic); the channel block's offset is wave-uniform and scalar
    const __amdgpu_buffer_rsrc_t rs_dst = make_rsrc(a.dst, a.dst_bytes);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int m = pix_w + j * 32 + l32;
        const bool pok = m < m_end;
        const uint32_t mm = pok ? m : 0;
        const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
        const int d_pix = (int)n * a.dst_sn + (int)rem * POUT;
        const int z_pix = (int)n * a.z_sn + (int)rem * POUT;
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int ocb = oc_w + i * 32;  // first channel of this 32-channel block
            if (ocb >= oc_end) continue;    // wave-uniform
            if (blk_mod > 1 && (i * NT + j) % blk_mod != blk_rem) continue;
            const v16i& c = acc[i][j];
            if (POUT == 32) {
                const int blk_off = (ocb >> 5) * a.dst_scb + lh * 16;
                uint32_t zq[4] = {0, 0, 0, 0};
                if (HZ) {
                    v4i zv;
                    if (ZPRE)
                        zv = zr->v[i][j];
                    else
                        zv = __builtin_amdgcn_raw_buffer_load_b128(rs_z, pok ? z_pix + blk_off : -1, 0, 0);
                    // stored order (16 consecutive channels per lane) -> accumulator order
                    auto s0 = __builtin_amdgcn_permlane32_swap((uint32_t)zv[0], (uint32_t)zv[1], false, false);
                    auto s1 = __builtin_amdgcn_permlane32_swap((uint32_t)zv[2], (uint32_t)zv[3], false, false);
                    zq[0] = s0[0]; zq[2] = s0[1]; zq[1] = s1[0]; zq[3] = s1[1];
                }
                uint32_t o[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if constexpr (NL == NL_ZLIN)
                        o[q] = requant4_table(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], zq[q], a.epi, zt);
                    else
                        o[q] = requant4_fast<NL, HZ>(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], zq[q], a.epi);
                }
                // accumulator order -> stored order
                auto s0 = __builtin_amdgcn_permlane32_swap(o[0], o[2], false, false);
                auto s1 = __builtin_amdgcn_permlane32_swap(o[1], o[3], false, false);
                const v4i out = {(int)s0[0], (int)s0[1], (int)s1[0], (int)s1[1]};
                __builtin_amdgcn_raw_buffer_store_b128(out, rs_dst, pok ? d_pix + lh * 16 : SENT, (ocb >> 5) * a.dst_scb, 0);
                // A vector-memory store of more than 8 bytes reads its data registers for two more cycles after it
                // issues, and the conversions that pack the next results are inline assembly, which the compiler's
                // hazard check does not look into: hold the registers (as an operand of the two wait states) until then.
                asm volatile("s_nop 1" ::"v"(out) : "memory");
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int oc4 = ocb + 8 * q + 4 * lh;  // first of 4 channels; oc is a multiple of 4
                    const bool ok = pok && oc4 < oc_end;
                    const int off = (oc4 >> 2) * a.dst_scb;
                    uint32_t zw = 0;
                    if (HZ) zw = ZPRE ? (uint32_t)zr->v[i][j][q]
                                      : (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_z, ok ? z_pix + off : -1, 0, 0);
                    uint32_t o;
                    if constexpr (NL == NL_ZLIN)
                        o = requant4_table(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], zw, a.epi, zt);
                    else
                        o = requant4_fast<NL, HZ>(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], zw, a.epi);
                    __builtin_amdgcn_raw_buffer_store_b32(o, rs_dst, ok ? d_pix + off : SENT, 0, 0);
                }
            }
        }
    }
}

// Fused requantisation + store of one wave tile (MT x NT blocks of 32 channels x 32 pixels).
// oc_end: one past the last output channel this tile may write (the layer's channel count, or the end of the tile's
// group); negative = the layer's channel count.
// zt: the kernel's LDS copy of the residual table, or null: a kernel without one never takes the table form
template <int POUT, int MT, int NT, bool ZPRE = false>
__device__ __forceinline__ void igemm_run_epilogue(const IgemmArgs& a, v16i (&acc)[MT][NT], int oc_w, int pix_w, int l32,
                                                   int lh, const ZRegs<MT, NT>* zr = nullptr, int oc_end = -1, int blk_mod = 1,
                                                   int blk_rem = 0, int m_end = -1, const float* zt = nullptr) {
    if (oc_end < 0) oc_end = a.OC;
    if (m_end < 0) m_end = a.M;
    if (zt != nullptr && a.epi.zlin) {
        igemm_epilogue<POUT, MT, NT, NL_ZLIN, true, ZPRE>(a, acc, zr, oc_w, pix_w, l32, lh, oc_end, blk_mod, blk_rem, m_end, zt);
    } else if (a.epi.lin) {
        igemm_epilogue<POUT, MT, NT, NL_LIN, false, ZPRE>(a, acc, zr, oc_w, pix_w, l32, lh, oc_end, blk_mod, blk_rem, m_end);
    } else if (a.epi.has_z) {
        switch (a.epi.nonline) {
            case NL_RELU: igemm_epilogue<POUT, MT, NT, NL_RELU, true, ZPRE>(a, acc, zr, oc_w, pix_w, l32, lh, oc_end, blk_mod, blk_rem, m_end); break;
            case NL_H_SWISH: igemm_epilogue<POUT, MT, NT, NL_H_SWISH, true, ZPRE>(a, acc, zr, oc_w, pix_w, l32, lh, oc_end, blk_mod, blk_rem, m_end); break;
            default: igemm_epilogue<POUT, MT, NT, NL_IDENTITY, true, ZPRE>(a, acc, zr, oc_w, pix_w, l32, lh, oc_end, blk_mod, blk_rem, m_end); break;
        }
    } else {
        switch (a.epi.nonline) {
            case NL_RELU: igemm_epilogue<POUT, MT, NT, NL_RELU, false, ZPRE>(a, acc, zr, oc_w, pix_w, l32, lh, oc_end, blk_mod, blk_rem, m_end); break;
            case NL_H_SWISH: igemm_epilogue<POUT, MT, NT, NL_H_SWISH, false, ZPRE>(a, acc, zr, oc_w, pix_w, l32, lh, oc_end, blk_mod, blk_rem, m_end); break;
            default: igemm_epilogue<POUT, MT, NT, NL_IDENTITY, false, ZPRE>(a, acc, zr, oc_w, pix_w, l32, lh, oc_end, blk_mod, blk_rem, m_end); break;
        }
    }
}

// General epilogue of one wave tile: every dst dtype / bias shape / scale the operator accepts, with the literal
// requantisation chain where the fast forms do not apply.  Register quad q of a 32x32 block holds channels
// ocb + 8q + 4 (lane / 32) .. + 3 of pixel lane % 32: one dword of int8 results, or 16 bytes of int32 results.
// QuantizedS32 dst: the reference accumulates in dst itself, IDENTITY stores the raw sum, the
// activations dequantise with the scale of dst (e.s_b holds it; naive/conv_bias/opr_impl.cpp:223-228,52,69-73,89-93).
template <int POUT, int MT, int NT>
__device__ __forceinline__ void igemm_epilogue_general(const IgemmArgs& a, v16i (&acc)[MT][NT], int oc_w, int pix_w, int l32,
                                                       int lh, int oc_end) {
    const bool hz = a.epi.has_z != 0;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int m = pix_w + j * 32 + l32;
        const bool pok = m < a.M;
        const uint32_t mm = pok ? m : 0;
        const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int ocb = oc_w + i * 32;
            if (ocb >= oc_end) continue;  // wave-uniform
            const v16i& c = acc[i][j];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int oc4 = ocb + 8 * q + 4 * lh;
                if (!(pok && oc4 < oc_end)) continue;
                // element offsets inside one image (dst layout) and of the image
                const int64_t in_img = (int64_t)(oc4 / POUT) * (a.OHW * POUT) + (int64_t)rem * POUT + (oc4 % POUT);
                int v[4] = {c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]};
                if (a.bias_full) {
                    const v4i b = *reinterpret_cast<const v4i*>(a.bias + (int64_t)n * ((int64_t)a.OC * a.OHW) + in_img);
                    v[0] += b[0]; v[1] += b[1]; v[2] += b[2]; v[3] += b[3];
                }
                if (a.dst_s32) {
                    v4i o = {v[0], v[1], v[2], v[3]};
                    if (hz || a.epi.nonline != NL_IDENTITY) {
                        // a residual of a QuantizedS32 dst is QuantizedS32 itself (z has the dtype of dst)
                        v4i zq = {0, 0, 0, 0};
                        if (hz) zq = *reinterpret_cast<const v4i*>(reinterpret_cast<const int*>(a.z) + (int64_t)n * a.z_sn + in_img);
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[r] = requant_s32_exact(v[r], hz, zq[r], a.epi);
                    }
                    *reinterpret_cast<v4i*>(reinterpret_cast<int*>(a.dst) + (int64_t)n * a.dst_sn + in_img) = o;
                } else {
                    uint32_t zw = 0;
                    if (hz) zw = *reinterpret_cast<const uint32_t*>(a.z + (int64_t)n * a.z_sn + in_img);
                    const uint32_t o = requant4(v[0], v[1], v[2], v[3], zw, a.epi);
                    *reinterpret_cast<uint32_t*>(a.dst + (int64_t)n * a.dst_sn + in_img) = o;
                }
            }
        }
    }
}

// Epilogue of one wave tile for a planar destination (format NCHW4_NCHW: dst, z and a full-shape bias are NCHW tensors,
// dnn/src/common/convolution.cpp:929-947).  Register quad q of a 32x32 block holds four consecutive channels of one pixel:
// four stores OHW elements apart, each contiguous over the 32 lanes of a half wave.  QuantizedS8 dst: the requantisation
// chain in whichever form the scales allow; Float32 dst: the exact sum dequantised once, then bias, z and activation in
// float (forward_bias and handle_z_inp_and_activation_naive on float tensors, dnn/src/naive/conv_bias/opr_impl.cpp:21-98).
enum { PLANAR_F32 = 0, PLANAR_S8_EXACT = 1, PLANAR_S8_FAST = 2 };
template <int MT, int NT, int KIND, int NL, bool HZ>
__device__ __forceinline__ void igemm_epilogue_planar_as(const IgemmArgs& a, v16i (&acc)[MT][NT], int oc_w, int pix_w, int l32,
                                                         int lh) {
    const bool hz = KIND == PLANAR_S8_FAST ? HZ : a.epi.has_z != 0;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int m = pix_w + j * 32 + l32;
        const bool pok = m < a.M;
        const uint32_t mm = pok ? m : 0;
        const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int ocb = oc_w + i * 32;
            const v16i& c = acc[i][j];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int oc4 = ocb + 8 * q + 4 * lh;
                const int left = pok ? a.OC - oc4 : 0;              // channels of this quad that exist (<= 0: none)
                const int64_t in_img = (int64_t)oc4 * a.OHW + rem;  // element of channel oc4 inside one image
                const int64_t full = (int64_t)n * ((int64_t)a.OC * a.OHW) + in_img;
                if (KIND == PLANAR_F32) {
                    float* dp = reinterpret_cast<float*>(a.dst) + (int64_t)n * a.dst_sn + in_img;
                    const float* zp = reinterpret_cast<const float*>(a.z) + (int64_t)n * a.z_sn + in_img;
                    const float* fb = reinterpret_cast<const float*>(a.bias);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (r < left) {
                            float v = (float)c[4 * q + r] * a.epi.s_b;
                            if (a.bias_full)
                                v = v + fb[full + (int64_t)r * a.OHW];
                            else if (a.bias)
                                v = v + fb[oc4 + r];
                            if (hz) v = v + zp[(int64_t)r * a.OHW];
                            if (a.epi.nonline == NL_RELU)
                                v = v <= 0.f ? 0.f : v;
                            else if (a.epi.nonline == NL_H_SWISH)
                                v = v * fminf(fmaxf(v + 3.f, 0.f), 6.f) * (1.f / 6.f);
                            dp[(int64_t)r * a.OHW] = v;
                        }
                    }
                } else {
                    int8_t* dp = a.dst + (int64_t)n * a.dst_sn + in_img;
                    const int8_t* zp = a.z + (int64_t)n * a.z_sn + in_img;
                    int v[4] = {c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]};
                    uint32_t zw = 0;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (r < left) {
                            if (a.bias_full) v[r] += a.bias[full + (int64_t)r * a.OHW];
                            if (hz) zw |= (uint32_t)(uint8_t)zp[(int64_t)r * a.OHW] << (8 * r);
                        }
                    }
                    const uint32_t o = KIND == PLANAR_S8_EXACT ? requant4_exact(v[0], v[1], v[2], v[3], zw, a.epi)
                                                               : requant4_fast<NL, HZ>(v[0], v[1], v[2], v[3], zw, a.epi);
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (r < left) dp[(int64_t)r * a.OHW] = (int8_t)(o >> (8 * r));
                }
            }
        }
    }
}

template <int MT, int NT>
__device__ __forceinline__ void igemm_epilogue_planar(const IgemmArgs& a, v16i (&acc)[MT][NT], int oc_w, int pix_w, int l32,
                                                      int lh) {
#define MI355_PLANAR(KIND, NL, HZ) igemm_epilogue_planar_as<MT, NT, KIND, NL, HZ>(a, acc, oc_w, pix_w, l32, lh)
    if (a.dst_f32) {
        MI355_PLANAR(PLANAR_F32, NL_IDENTITY, false);
    } else if (!a.epi.fast) {
        MI355_PLANAR(PLANAR_S8_EXACT, NL_IDENTITY, false);
    } else if (a.epi.lin) {
        MI355_PLANAR(PLANAR_S8_FAST, NL_LIN, false);
    } else if (a.epi.has_z) {
        switch (a.epi.nonline) {
            case NL_RELU: MI355_PLANAR(PLANAR_S8_FAST, NL_RELU, true); break;
            case NL_H_SWISH: MI355_PLANAR(PLANAR_S8_FAST, NL_H_SWISH, true); break;
            default: MI355_PLANAR(PLANAR_S8_FAST, NL_IDENTITY, true); break;
        }
    } else {
        switch (a.epi.nonline) {
            case NL_RELU: MI355_PLANAR(PLANAR_S8_FAST, NL_RELU, false); break;
            case NL_H_SWISH: MI355_PLANAR(PLANAR_S8_FAST, NL_H_SWISH, false); break;
            default: MI355_PLANAR(PLANAR_S8_FAST, NL_IDENTITY, false); break;
        }
    }
#undef MI355_PLANAR
}

// LDS-direct variant (conv_igemm_dma.hip): global -> LDS copies without a register stage
int igemm_dma_num_cfgs();
const char* igemm_dma_cfg_name(int cfg);
void igemm_dma_cfg_shape(int cfg, int* bm, int* bn, int* kch);
bool igemm_dma_cfg_is_pin4(int cfg);  // a 4-packed pointwise tile (NCHW4 in and out, 1x1, no padding)
int igemm_dma_first_pin4_cfg();       // the first of them (128 x 128 x 64)
int launch_igemm_dma(hipStream_t st, IgemmArgs& a, int pout, int cfg, int cu_count);

// second-generation kernel for 32-packed inputs (conv_igemm2.hip): chunk-major LDS stages, software-pipelined k-loop,
// optional pre-processed filter, group convolution
int igemm2_num_cfgs();
const char* igemm2_cfg_name(int cfg);
void igemm2_cfg_shape(int cfg, int* bm, int* bn, int* kch);
int launch_igemm2(hipStream_t st, IgemmArgs& a, int pout, int cfg, int cu_count);
// whether second-generation tile `cfg` runs this problem as itself (general epilogue instantiated, LDS fits); no launch
bool igemm2_can_run(const IgemmArgs& a, int pout, int cfg);
int igemm_first_v2_cfg();  // tile_cfg of the first second-generation tile
// pre-processed filter of the second-generation kernel: [k-chunk][channel padded to 32][32 bytes]
size_t igemm2_preprocessed_bytes(int oc, int kbytes);
int launch_igemm2_preprocess(hipStream_t st, const int8_t* flt, int8_t* out, int oc, int kbytes);

// patch-staged kernel for 32-packed inputs, filters larger than 1x1 at stride 1 (conv_igemm3.hip): same filter layouts
// (reference or pre-processed) as the second-generation kernel
int igemm3_num_cfgs();
const char* igemm3_cfg_name(int cfg);
bool igemm3_can_run(const IgemmArgs& a, int pin, int pout, int cfg);
int launch_igemm3(hipStream_t st, IgemmArgs& a, int pin, int pout, int cfg);

// weight-resident kernel for 3x3 / stride 1 / pad 1 over 32 or 64 input channels, 32-packed (conv_igemm4.hip): the
// reference filter layout only
int igemm4_num_cfgs();
const char* igemm4_cfg_name(int cfg);
bool igemm4_can_run(const IgemmArgs& a, int pin, int pout, int cfg);
int launch_igemm4(hipStream_t st, IgemmArgs& a, int pin, int pout, int cfg, int cu_count);

// streaming kernel for 4-packed pointwise layers with few input or few output channels (conv_pw4.hip)
bool pw4s_usable(const IgemmArgs& a);
int launch_pw4s(hipStream_t st, const IgemmArgs& a, int cu_count);
// the same for 32-packed pointwise layers with at most 128 input channels (tile "pw32_stream")
bool pw32s_usable(const IgemmArgs& a, int pin, int pout);
int launch_pw32s(hipStream_t st, const IgemmArgs& a, int cu_count);

}  // namespace mi355
