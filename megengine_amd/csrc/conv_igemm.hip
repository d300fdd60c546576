// Dense int8 ConvBias as an implicit GEMM on the gfx950 matrix cores.
//
//   D[oc][pixel] = sum_k  F[oc][k] * X[pixel][k]        k = (channel block, fh, fw, channel-in-block)
//
// computed with v_mfma_i32_32x32x32_i8 (A = filter rows, B = pixels, int32 accumulate) and
// requantised in registers by the fused epilogue (epilogue.h).  Activations and filters in the
// reference's NCHW4 / NCHW32 layouts already hold the 16 consecutive k-bytes an MFMA lane needs
// (NCHW32: one 16-byte run; NCHW4: four 4-byte runs), so the im2col matrix is never materialised:
// each stage gathers a BN x BK activation tile and a BM x BK filter tile straight into LDS,
// double-buffered against the MFMA loop, with an XOR swizzle on the 16-byte slots.
//
// Data layout in LDS (per stage and operand): [row][BK bytes], BK = KCH * 32, 16-byte slot s of row r
// stored at slot s ^ swz(r).  A k-chunk table {byte offset, fh, fw} for every 32-byte (NCHW32) or
// 4-byte (NCHW4) k-unit is built once per workgroup, so the loaders do no divisions.
//
// Accumulator layout of the 32x32 MFMA (lane l, register v): pixel = l % 32,
// oc = 8*(v/4) + 4*(l/32) + v%4.  NCHW4 output stores one dword (4 channels) per register quad;
// NCHW32 output first exchanges quads between lanes l and l+32 (v_permlane32_swap) so that each
// lane owns 16 consecutive channels of one pixel and stores 16 bytes.
#include "common.h"

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int IG_THREADS = 256;
constexpr int IG_MAX_ENTRIES = 2048;  // k-chunk table capacity (entries of 8 bytes)

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
    int CBI;          // input channel blocks (ic / PIN)
    int OC;
    int M;            // n * oh * ow
    int kbytes;       // filter bytes per output channel
    int KC;           // 32-byte k-chunks (ceil)
    int entries;      // valid k-unit table entries (KC for NCHW32, ic/4*T for NCHW4)
    int nstages;
    int src_sn, src_scb;      // bytes: per image, per channel block
    int dst_sn, dst_scb;      // bytes: per image, per output channel block
    int z_sn;
    int tiles_m, tiles_n;
    int has_bias;
    EpiParams epi;
};

struct KEntry {
    int off;    // byte offset of the k-unit relative to the pixel's (ih0, iw0) base
    int fhfw;   // fh | fw << 16 ; fh = 0x4000 marks a padding entry (never valid)
};

// 16-byte slot swizzle.  S = slots per row.  Rows r..r+15 read the same logical slot in one
// ds_read_b128 wavefront pass and must land in distinct 4-bank groups of the 64 banks.
template <int S>
__device__ __forceinline__ int swz(int row) {
    if (S == 4) return ((row >> 2) & 1) * 2 + ((row >> 3) & 1);
    if (S == 8) return (((row >> 1) & 3) << 1) | ((row >> 3) & 1);
    return 0;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

template <int PIN, int POUT, int BM, int BN, int WM, int WN, int KCH>
struct IgemmKernel {
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int MT = WTM / 32, NT = WTN / 32;
    static constexpr int S = KCH * 2;              // 16-byte slots per LDS row
    static constexpr int ROWB = KCH * 32;          // bytes per LDS row
    static constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB;
    static constexpr int UA = BM * S / IG_THREADS;  // 16-byte units per thread per stage
    static constexpr int UB = BN * S / IG_THREADS;
    static constexpr int LDS_BYTES = 2 * (A_BYTES + B_BYTES) + IG_MAX_ENTRIES * 8;
    static_assert(WM * WN * 64 == IG_THREADS, "4 waves");
    static_assert(UA >= 1 && UB >= 1, "tile too small for 256 loader threads");
    static_assert(MT >= 1 && NT >= 1, "wave tile");

    // unit u of an operand with R rows: half = u & 1, row = (u >> 1) % R, chunk = (u >> 1) / R
    __device__ static __forceinline__ void run(const IgemmArgs& a) {
        extern __shared__ __attribute__((aligned(16))) int8_t lds[];
        int8_t* sA = lds;
        int8_t* sB = lds + 2 * A_BYTES;
        KEntry* tab = reinterpret_cast<KEntry*>(lds + 2 * (A_BYTES + B_BYTES));

        const int t = threadIdx.x;
        const int lane = t & 63, wave = t >> 6;
        const int l32 = lane & 31, lh = lane >> 5;
        const int wm = wave / WN, wn = wave % WN;

        // ---- workgroup -> tile, XCD aware: workgroups are dealt round-robin to the 8 XCDs, so give
        // each XCD a contiguous run of tiles (neighbouring tiles share activations in that XCD's L2)
        int logical;
        {
            const int nb = gridDim.x, bid = blockIdx.x;
            const int per = nb >> 3, rem = nb & 7, x = bid & 7, i = bid >> 3;
            logical = x < rem ? x * (per + 1) + i : rem * (per + 1) + (x - rem) * per + i;
        }
        const int tile_n = logical / a.tiles_m, tile_m = logical - tile_n * a.tiles_m;
        const int oc0 = tile_m * BM, pix0 = tile_n * BN;

        // ---- k-unit table
        {
            constexpr int UNIT = PIN == 32 ? 32 : 4;
            const int cap = a.nstages * KCH * (32 / UNIT);
            for (int e = t; e < cap; e += IG_THREADS) {
                KEntry k;
                if (e < a.entries) {
                    int cb = e / a.T, tap = e - cb * a.T;
                    int fh = tap / a.FW, fw = tap - fh * a.FW;
                    k.off = cb * a.src_scb + (fh * a.IW + fw) * PIN;
                    k.fhfw = fh | (fw << 16);
                } else {
                    k.off = 0;
                    k.fhfw = 0x4000;
                }
                tab[e] = k;
            }
        }

        // ---- per-thread loader state
        // B rows handled by this thread (RB of them), fixed for the whole K loop
        constexpr int RB = BN >= 128 ? BN / 128 : 1;
        int b_base[RB], b_ih0[RB], b_iw0[RB];
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            int row = ((t >> 1) % BN) + 128 * r;
            int m = pix0 + row;
            bool ok = m < a.M;
            int mm = ok ? m : 0;
            int n = mm / a.OHW, rem = mm - n * a.OHW;
            int oh = rem / a.OW, ow = rem - oh * a.OW;
            int ih0 = oh * a.sh - a.ph, iw0 = ow * a.sw - a.pw;
            b_ih0[r] = ok ? ih0 : -0x8000;  // makes every tap fail the bounds test
            b_iw0[r] = iw0;
            b_base[r] = n * a.src_sn + (ih0 * a.IW + iw0) * PIN;
        }
        const __amdgpu_buffer_rsrc_t rs_src = make_rsrc(a.src, a.src_bytes);
        const __amdgpu_buffer_rsrc_t rs_flt = make_rsrc(a.flt, a.flt_bytes);

        v4i ra[UA], rb[UB];

        auto load_stage = [&](int s) {
            const int kc0 = s * KCH;
            // filter units
#pragma unroll
            for (int j = 0; j < UA; ++j) {
                int v = (t >> 1) + 128 * j;
                int row = v % BM, chunk = v / BM;
                int oc = oc0 + row;
                int off = oc * a.kbytes + (kc0 + chunk) * 32 + (t & 1) * 16;
                bool ok = oc < a.OC && (kc0 + chunk) < a.KC;
                ra[j] = __builtin_amdgcn_raw_buffer_load_b128(rs_flt, ok ? off : -1, 0, 0);
            }
            // activation units
#pragma unroll
            for (int j = 0; j < UB; ++j) {
                int v = (t >> 1) + 128 * j;
                int r = BN >= 128 ? (j % RB) : 0;
                int chunk = v / BN;
                if (PIN == 32) {
                    KEntry k = tab[kc0 + chunk];
                    int ih = b_ih0[r] + (k.fhfw & 0xffff), iw = b_iw0[r] + (k.fhfw >> 16);
                    bool ok = (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
                    int off = b_base[r] + k.off + (t & 1) * 16;
                    rb[j] = __builtin_amdgcn_raw_buffer_load_b128(rs_src, ok ? off : -1, 0, 0);
                } else {
                    const int e0 = (kc0 + chunk) * 8 + (t & 1) * 4;
                    v4i x;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        KEntry k = tab[e0 + i];
                        int ih = b_ih0[r] + (k.fhfw & 0xffff), iw = b_iw0[r] + (k.fhfw >> 16);
                        bool ok = (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
                        int off = b_base[r] + k.off;
                        x[i] = __builtin_amdgcn_raw_buffer_load_b32(rs_src, ok ? off : -1, 0, 0);
                    }
                    rb[j] = x;
                }
            }
        };

        auto store_stage = [&](int buf) {
#pragma unroll
            for (int j = 0; j < UA; ++j) {
                int v = (t >> 1) + 128 * j;
                int row = v % BM, chunk = v / BM;
                int slot = (chunk * 2 + (t & 1)) ^ swz<S>(row);
                *reinterpret_cast<v4i*>(sA + buf * A_BYTES + row * ROWB + slot * 16) = ra[j];
            }
#pragma unroll
            for (int j = 0; j < UB; ++j) {
                int v = (t >> 1) + 128 * j;
                int row = v % BN, chunk = v / BN;
                int slot = (chunk * 2 + (t & 1)) ^ swz<S>(row);
                *reinterpret_cast<v4i*>(sB + buf * B_BYTES + row * ROWB + slot * 16) = rb[j];
            }
        };

        // ---- accumulators, initialised with the bias of their output channel
        v16i acc[MT][NT];
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            v16i init;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                int oc = oc0 + wm * WTM + i * 32 + 8 * q + 4 * lh;
                v4i b = {0, 0, 0, 0};
                if (a.has_bias && oc < a.OC) b = *reinterpret_cast<const v4i*>(a.bias + oc);
                init[4 * q + 0] = b[0]; init[4 * q + 1] = b[1]; init[4 * q + 2] = b[2]; init[4 * q + 3] = b[3];
            }
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[i][j] = init;
        }

        __syncthreads();  // table ready
        load_stage(0);
        store_stage(0);
        __syncthreads();

        for (int s = 0; s < a.nstages; ++s) {
            const int buf = s & 1;
            const bool more = s + 1 < a.nstages;
            if (more) load_stage(s + 1);
            const int8_t* pA = sA + buf * A_BYTES;
            const int8_t* pB = sB + buf * B_BYTES;
#pragma unroll
            for (int c = 0; c < KCH; ++c) {
                v4i fa[MT], fb[NT];
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    int row = wm * WTM + i * 32 + l32;
                    int slot = (c * 2 + lh) ^ swz<S>(row);
                    fa[i] = *reinterpret_cast<const v4i*>(pA + row * ROWB + slot * 16);
                }
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    int row = wn * WTN + j * 32 + l32;
                    int slot = (c * 2 + lh) ^ swz<S>(row);
                    fb[j] = *reinterpret_cast<const v4i*>(pB + row * ROWB + slot * 16);
                }
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
            if (more) store_stage(buf ^ 1);
            __syncthreads();
        }

        // ---- epilogue
        if (a.epi.has_z) {
            switch (a.epi.nonline) {
                case NL_RELU: epilogue<NL_RELU, true>(a, acc, oc0 + wm * WTM, pix0 + wn * WTN, l32, lh); break;
                case NL_H_SWISH: epilogue<NL_H_SWISH, true>(a, acc, oc0 + wm * WTM, pix0 + wn * WTN, l32, lh); break;
                default: epilogue<NL_IDENTITY, true>(a, acc, oc0 + wm * WTM, pix0 + wn * WTN, l32, lh); break;
            }
        } else {
            switch (a.epi.nonline) {
                case NL_RELU: epilogue<NL_RELU, false>(a, acc, oc0 + wm * WTM, pix0 + wn * WTN, l32, lh); break;
                case NL_H_SWISH: epilogue<NL_H_SWISH, false>(a, acc, oc0 + wm * WTM, pix0 + wn * WTN, l32, lh); break;
                default: epilogue<NL_IDENTITY, false>(a, acc, oc0 + wm * WTM, pix0 + wn * WTN, l32, lh); break;
            }
        }
    }

    template <int NL, bool HZ>
    __device__ static __forceinline__ void epilogue(const IgemmArgs& a, v16i (&acc)[MT][NT], int oc_w, int pix_w,
                                                    int l32, int lh) {
        const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(a.z, HZ ? a.z_bytes : 0);
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int m = pix_w + j * 32 + l32;
            const bool pok = m < a.M;
            const int mm = pok ? m : 0;
            const int n = mm / a.OHW, rem = mm - n * a.OHW;
            const int d_pix = n * a.dst_sn + rem * POUT;
            const int z_pix = n * a.z_sn + rem * POUT;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const int ocb = oc_w + i * 32;  // first channel of this 32-channel block
                if (ocb >= a.OC) continue;      // wave-uniform
                const v16i& c = acc[i][j];
                if (POUT == 32) {
                    const int blk_off = (ocb >> 5) * a.dst_scb + lh * 16;
                    uint32_t zq[4] = {0, 0, 0, 0};
                    if (HZ) {
                        v4i zv = __builtin_amdgcn_raw_buffer_load_b128(rs_z, pok ? z_pix + blk_off : -1, 0, 0);
                        // stored order (16 consecutive channels per lane) -> accumulator order
                        auto s0 = __builtin_amdgcn_permlane32_swap((uint32_t)zv[0], (uint32_t)zv[1], false, false);
                        auto s1 = __builtin_amdgcn_permlane32_swap((uint32_t)zv[2], (uint32_t)zv[3], false, false);
                        zq[0] = s0[0]; zq[2] = s0[1]; zq[1] = s1[0]; zq[3] = s1[1];
                    }
                    uint32_t o[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        o[q] = requant4_fast<NL, HZ>(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], zq[q], a.epi);
                    // accumulator order -> stored order
                    auto s0 = __builtin_amdgcn_permlane32_swap(o[0], o[2], false, false);
                    auto s1 = __builtin_amdgcn_permlane32_swap(o[1], o[3], false, false);
                    u32x4 out = {s0[0], s0[1], s1[0], s1[1]};
                    if (pok) *reinterpret_cast<u32x4*>(a.dst + d_pix + blk_off) = out;
                } else {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int oc4 = ocb + 8 * q + 4 * lh;  // first of 4 channels; oc is a multiple of 4
                        const bool ok = pok && oc4 < a.OC;
                        const int off = (oc4 >> 2) * a.dst_scb;
                        uint32_t zw = 0;
                        if (HZ) zw = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_z, ok ? z_pix + off : -1, 0, 0);
                        uint32_t o = requant4_fast<NL, HZ>(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], zw, a.epi);
                        if (ok) *reinterpret_cast<uint32_t*>(a.dst + d_pix + off) = o;
                    }
                }
            }
        }
    }
};

template <int PIN, int POUT, int BM, int BN, int WM, int WN, int KCH>
__global__ __launch_bounds__(IG_THREADS) void igemm_kernel(IgemmArgs a) {
    IgemmKernel<PIN, POUT, BM, BN, WM, WN, KCH>::run(a);
}

struct TileCfg {
    const char* name;
    int bm, bn;
};
// index = tile_cfg of mi355_algo
const TileCfg kCfgs[] = {
        {"128x128", 128, 128},
        {"64x256", 64, 256},
        {"256x128", 256, 128},
        {"64x64", 64, 64},
        {"32x256", 32, 256},
};
constexpr int kNumCfgs = sizeof(kCfgs) / sizeof(kCfgs[0]);

template <int PIN, int POUT, int BM, int BN, int WM, int WN, int KCH>
int launch_one(hipStream_t st, IgemmArgs& a) {
    using K = IgemmKernel<PIN, POUT, BM, BN, WM, WN, KCH>;
    a.tiles_m = (a.OC + BM - 1) / BM;
    a.tiles_n = (a.M + BN - 1) / BN;
    a.nstages = (a.KC + KCH - 1) / KCH;
    auto kern = igemm_kernel<PIN, POUT, BM, BN, WM, WN, KCH>;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, K::LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_set = true;
    }
    const int64_t grid = (int64_t)a.tiles_m * a.tiles_n;
    if (grid <= 0 || grid > 0x7fffffff) return (int)hipErrorInvalidValue;
    const int tab_entries = a.nstages * KCH * (PIN == 32 ? 1 : 8);
    const int lds = 2 * (K::A_BYTES + K::B_BYTES) + tab_entries * 8;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(IG_THREADS), lds, st, a);
    return (int)hipGetLastError();
}

template <int PIN, int POUT>
int launch_fmt(hipStream_t st, IgemmArgs& a, int cfg) {
    switch (cfg) {
        case 0: return launch_one<PIN, POUT, 128, 128, 2, 2, 2>(st, a);
        case 1: return launch_one<PIN, POUT, 64, 256, 1, 4, 2>(st, a);
        case 2: return launch_one<PIN, POUT, 256, 128, 2, 2, 2>(st, a);
        case 3: return launch_one<PIN, POUT, 64, 64, 2, 2, 4>(st, a);
        case 4: return launch_one<PIN, POUT, 32, 256, 1, 4, 4>(st, a);
        default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace

int igemm_num_cfgs() { return kNumCfgs; }
const char* igemm_cfg_name(int cfg) { return cfg >= 0 && cfg < kNumCfgs ? kCfgs[cfg].name : "?"; }

bool igemm_usable(const ConvProblem& p) {
    const mi355_conv_desc& d = p.d;
    if (d.group != 1 || p.dw4) return false;
    if (d.format != MI355_FMT_NCHW4 && d.format != MI355_FMT_NCHW32 && d.format != MI355_FMT_NCHW4_NCHW32 &&
        d.format != MI355_FMT_NCHW32_NCHW4)
        return false;
    if (d.mode != MI355_MODE_CROSS_CORRELATION || d.dilate_h != 1 || d.dilate_w != 1) return false;
    if (d.dst_dtype != MI355_DT_QS8 || d.bias_mode == MI355_BIAS_FULL) return false;
    if (!p.epi.fast) return false;
    if (d.fh > 255 || d.fw > 255 || d.pad_h > 0xfff || d.pad_w > 0xfff || d.ih > 0x3000 || d.iw > 0x3000) return false;
    // 32-bit byte offsets and buffer descriptors
    const int64_t lim = (int64_t)1 << 31;
    const int64_t src_b = (int64_t)(d.n - 1) * p.src_sn + (int64_t)d.ic * d.ih * d.iw;
    const int64_t dst_b = (int64_t)(d.n - 1) * p.dst_sn + (int64_t)d.oc * p.oh * p.ow;
    const int64_t z_b = d.has_z ? (int64_t)(d.n - 1) * p.z_sn + (int64_t)d.oc * p.oh * p.ow : 0;
    const int64_t flt_b = (int64_t)d.oc * d.ic * d.fh * d.fw;
    if (src_b >= lim || dst_b >= lim || z_b >= lim || flt_b >= lim) return false;
    if ((int64_t)d.n * p.oh * p.ow >= lim) return false;
    const int64_t entries = p.pin == 32 ? (int64_t)(d.ic / 32) * d.fh * d.fw : (int64_t)(d.ic / 4) * d.fh * d.fw;
    // table capacity incl. the padding entries of the last stage (<= 4 chunks of 8 units)
    if (entries + 32 > IG_MAX_ENTRIES) return false;
    return true;
}

int igemm_pick_cfg(const ConvProblem& p, int cu_count) {
    const mi355_conv_desc& d = p.d;
    const int64_t M = (int64_t)d.n * p.oh * p.ow;
    const int OC = d.oc;
    if (cu_count <= 0) cu_count = 256;
    auto tiles = [&](int cfg) { return ((OC + kCfgs[cfg].bm - 1) / kCfgs[cfg].bm) * ((M + kCfgs[cfg].bn - 1) / kCfgs[cfg].bn); };
    if (OC <= 32) return 4;
    if (OC <= 64) return tiles(1) >= cu_count ? 1 : 3;
    if (OC % 256 == 0 && tiles(2) >= 2 * cu_count) return 2;
    if (tiles(0) >= cu_count) return 0;
    return 3;
}

int launch_conv_igemm(hipStream_t st, const ConvProblem& p, int cfg, const int8_t* src, const int8_t* flt,
                      const int32_t* bias, const int8_t* z, int8_t* dst) {
    const mi355_conv_desc& d = p.d;
    IgemmArgs a;
    a.src = src; a.flt = flt; a.bias = bias; a.z = z; a.dst = dst;
    a.IH = d.ih; a.IW = d.iw; a.OH = p.oh; a.OW = p.ow; a.OHW = p.oh * p.ow;
    a.FH = d.fh; a.FW = d.fw; a.T = d.fh * d.fw;
    a.sh = d.stride_h; a.sw = d.stride_w; a.ph = d.pad_h; a.pw = d.pad_w;
    a.CBI = d.ic / p.pin;
    a.OC = d.oc;
    a.M = d.n * p.oh * p.ow;
    a.kbytes = d.ic * d.fh * d.fw;
    a.KC = (a.kbytes + 31) / 32;
    a.entries = p.pin == 32 ? a.KC : (d.ic / 4) * a.T;
    a.src_sn = (int)p.src_sn;
    a.src_scb = d.ih * d.iw * p.pin;
    a.dst_sn = (int)p.dst_sn;
    a.dst_scb = p.oh * p.ow * p.pout;
    a.z_sn = (int)p.z_sn;
    a.src_bytes = (uint32_t)((int64_t)(d.n - 1) * p.src_sn + (int64_t)d.ic * d.ih * d.iw);
    a.flt_bytes = (uint32_t)((int64_t)d.oc * a.kbytes);
    a.dst_bytes = (uint32_t)((int64_t)(d.n - 1) * p.dst_sn + (int64_t)d.oc * a.OHW);
    a.z_bytes = d.has_z ? (uint32_t)((int64_t)(d.n - 1) * p.z_sn + (int64_t)d.oc * a.OHW) : 0;
    a.has_bias = d.bias_mode == MI355_BIAS_BROADCAST_CHANNEL;
    a.epi = p.epi;
    if (a.M == 0 || a.OC == 0) return 0;
    if (p.pin == 32 && p.pout == 32) return launch_fmt<32, 32>(st, a, cfg);
    if (p.pin == 4 && p.pout == 4) return launch_fmt<4, 4>(st, a, cfg);
    if (p.pin == 4 && p.pout == 32) return launch_fmt<4, 32>(st, a, cfg);
    return launch_fmt<32, 4>(st, a, cfg);
}

}  // namespace mi355
