// Channel-wise (depthwise) int8 ConvBias on channel-packed-by-4 activations.
//
// Layouts: src/dst (n, c/4, h, w, 4), filter (c/4, 1, 1, fh, fw, 4) -- the reference's NCHW44
// channel-wise filter (dnn/src/naive/convolution/helper.h:251-256, :419-424).  Every output
// needs fh*fw multiply-adds per channel and moves ~2 bytes, so the kernel is bandwidth bound:
// no matrix cores.  One thread produces 4 consecutive output pixels x 4 channels:
//   * a pixel's 4 channels arrive as one dword; the 4 per-channel products of a tap are 4
//     v_dot4_i32_i8 against the filter dword masked to one byte each (the masks are wave-uniform
//     and live in scalar registers), so no byte unpacking is needed;
//   * consecutive lanes own consecutive pixel quads: loads are coalesced dwords, the store is a
//     16-byte vector per lane (1 KiB per wavefront);
//   * all threads of a workgroup share (n, c/4), so filter and bias loads are scalar.
// That form (dw4_kernel) serves every filter size / stride.  The 3x3, stride 1 or 2 case -- every
// channel-wise layer of the MobileNet family -- has its own kernel, dw3x3_kernel, below.
#include "common.h"

namespace mi355 {
namespace {

struct DwArgs {
    const int8_t* src;
    const int8_t* flt;
    const int32_t* bias;
    const int8_t* z;
    int8_t* dst;
    int CG, IH, IW, OH, OW, QW;   // QW = quads per output row
    int FH, FW, sh, sw, ph, pw;
    int64_t src_sn, dst_sn, z_sn; // batch strides (bytes)
    int has_bias;
    int vec_ok;                   // OW % 4 == 0: 16-byte row-aligned stores and z loads
    EpiParams epi;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));

template <int F, int S>  // F = 0: runtime filter size / stride
__global__ __launch_bounds__(256) void dw4_kernel(DwArgs a) {
    const int plane = blockIdx.y;
    const int n = plane / a.CG, cg = plane - n * a.CG;
    const int quad = blockIdx.x * blockDim.x + threadIdx.x;
    if (quad >= a.OH * a.QW) return;
    const int oh = quad / a.QW, ow0 = (quad - oh * a.QW) * 4;
    const int FH = F ? F : a.FH, FW = F ? F : a.FW;
    const int sh = F ? S : a.sh, sw = F ? S : a.sw;

    const uint32_t* sp = reinterpret_cast<const uint32_t*>(a.src + n * a.src_sn) + (int64_t)cg * a.IH * a.IW;
    const uint32_t* wp = reinterpret_cast<const uint32_t*>(a.flt) + (int64_t)cg * FH * FW;

    int acc[4][4];
    {
        v4i b = {0, 0, 0, 0};
        if (a.has_bias) b = *reinterpret_cast<const v4i*>(a.bias + cg * 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[j][0] = b[0]; acc[j][1] = b[1]; acc[j][2] = b[2]; acc[j][3] = b[3];
        }
    }

    if constexpr (F != 0) {
        constexpr int COLS = F ? 3 * S + F : 1;  // input columns touched by 4 outputs
        const int iw_base = ow0 * S - a.pw;
#pragma unroll
        for (int fh = 0; fh < F; ++fh) {
            const int ih = oh * S + fh - a.ph;
            const bool rok = (unsigned)ih < (unsigned)a.IH;
            uint32_t x[COLS];
#pragma unroll
            for (int c = 0; c < COLS; ++c) {
                const int iw = iw_base + c;
                const bool ok = rok && (unsigned)iw < (unsigned)a.IW;
                x[c] = ok ? sp[ih * a.IW + iw] : 0u;
            }
#pragma unroll
            for (int fw = 0; fw < F; ++fw) {
                const uint32_t w = wp[fh * F + fw];
                const int w0 = (int)(w & 0x000000ffu), w1 = (int)(w & 0x0000ff00u), w2 = (int)(w & 0x00ff0000u),
                          w3 = (int)(w & 0xff000000u);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int xv = (int)x[j * S + fw];
                    acc[j][0] = __builtin_amdgcn_sdot4(xv, w0, acc[j][0], false);
                    acc[j][1] = __builtin_amdgcn_sdot4(xv, w1, acc[j][1], false);
                    acc[j][2] = __builtin_amdgcn_sdot4(xv, w2, acc[j][2], false);
                    acc[j][3] = __builtin_amdgcn_sdot4(xv, w3, acc[j][3], false);
                }
            }
        }
    } else {
        for (int fh = 0; fh < FH; ++fh) {
            const int ih = oh * sh + fh - a.ph;
            if ((unsigned)ih >= (unsigned)a.IH) continue;
            for (int fw = 0; fw < FW; ++fw) {
                const uint32_t w = wp[fh * FW + fw];
                const int w0 = (int)(w & 0x000000ffu), w1 = (int)(w & 0x0000ff00u), w2 = (int)(w & 0x00ff0000u),
                          w3 = (int)(w & 0xff000000u);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int iw = (ow0 + j) * sw + fw - a.pw;
                    const bool ok = (unsigned)iw < (unsigned)a.IW;
                    const int xv = ok ? (int)sp[ih * a.IW + iw] : 0;
                    acc[j][0] = __builtin_amdgcn_sdot4(xv, w0, acc[j][0], false);
                    acc[j][1] = __builtin_amdgcn_sdot4(xv, w1, acc[j][1], false);
                    acc[j][2] = __builtin_amdgcn_sdot4(xv, w2, acc[j][2], false);
                    acc[j][3] = __builtin_amdgcn_sdot4(xv, w3, acc[j][3], false);
                }
            }
        }
    }

    const int64_t row_off = (((int64_t)cg * a.OH + oh) * a.OW + ow0) * 4;
    int8_t* dp = a.dst + n * a.dst_sn + row_off;
    const int8_t* zp = a.z + n * a.z_sn + row_off;
    if (a.vec_ok) {
        u32x4 zv = {0, 0, 0, 0};
        if (a.epi.has_z) zv = *reinterpret_cast<const u32x4*>(zp);
        u32x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = requant4(acc[j][0], acc[j][1], acc[j][2], acc[j][3], zv[j], a.epi);
        *reinterpret_cast<u32x4*>(dp) = o;
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (ow0 + j < a.OW) {
                uint32_t zw = a.epi.has_z ? reinterpret_cast<const uint32_t*>(zp)[j] : 0u;
                reinterpret_cast<uint32_t*>(dp)[j] = requant4(acc[j][0], acc[j][1], acc[j][2], acc[j][3], zw, a.epi);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// 3x3, stride S in {1, 2}: one thread = 4 consecutive output pixels x R output rows x 4 channels.
//
//   * work items (image, channel quad, row strip, pixel quad) are flattened over the whole launch,
//     so 7x7 planes fill wavefronts as well as 112x112 ones; lanes run along a row, so the 16-byte
//     loads and stores of neighbouring lanes are contiguous;
//   * an input row is read once per thread as 16-byte vectors and serves up to three output rows;
//   * the 4 pixels x 4 channels block is transposed in registers (8 v_perm) so that one dword holds
//     4 consecutive pixels of ONE channel; a filter row [w0 w1 w2 0] (or shifted, [0 w0 w1 w2]) then
//     multiplies three horizontally adjacent taps with a single v_dot4: 3 dot products per output
//     instead of 9.
// ---------------------------------------------------------------------------------------------
struct Dw3Args {
    const int8_t* src;
    const int8_t* flt;
    const int32_t* bias;
    const int8_t* z;
    int8_t* dst;
    int CG, IH, IW, OH, OW, QW, OHS;  // QW = pixel quads per output row, OHS = row strips per plane
    int ph, pw;
    uint32_t items;
    uint32_t src_bytes;  // whole source tensor if it is addressable with 31-bit offsets, else 0
    int64_t src_sn, dst_sn, z_sn;
    int has_bias;
    FastDiv div_qw, div_ohs, div_cg;
    EpiParams epi;
};

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// c + dot(a, b) over four signed bytes, written to a fresh register
__device__ __forceinline__ int dot4_from(uint32_t a, int b, int c) {
    int r;
    asm("v_dot4_i32_i8 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// pixels (dwords of 4 channels) p[0..3]  ->  t[c] = {p0.c, p1.c, p2.c, p3.c}
__device__ __forceinline__ void transpose4(const uint32_t p[4], uint32_t t[4]) {
    const uint32_t a = perm(p[1], p[0], 0x05010400u), b = perm(p[1], p[0], 0x07030602u);
    const uint32_t c = perm(p[3], p[2], 0x05010400u), d = perm(p[3], p[2], 0x07030602u);
    t[0] = perm(c, a, 0x05040100u);
    t[1] = perm(c, a, 0x07060302u);
    t[2] = perm(d, b, 0x05040100u);
    t[3] = perm(d, b, 0x07060302u);
}

// 4 consecutive pixels of one input row starting at column c0 (any of them may fall outside the row)
__device__ __forceinline__ void load_px4(const uint32_t* row, int c0, int IW, bool rok, uint32_t p[4]) {
    if (rok && c0 >= 0 && c0 + 3 < IW) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(row + c0);  // needs 4-byte alignment only
        p[0] = v[0]; p[1] = v[1]; p[2] = v[2]; p[3] = v[3];
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) p[i] = (rok && (unsigned)(c0 + i) < (unsigned)IW) ? row[c0 + i] : 0u;
    }
}

template <int R, int NL, bool HZ, bool FAST>
__device__ __forceinline__ void dw3_store(const Dw3Args& a, const int (&acc)[R][4][4], int n, int cg, int oh0, int ow0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int oh = oh0 + r;
        if (oh >= a.OH) break;
        const int64_t off = (((int64_t)cg * a.OH + oh) * a.OW + ow0) * 4;
        uint32_t* dp = reinterpret_cast<uint32_t*>(a.dst + n * a.dst_sn + off);
        const uint32_t* zp = reinterpret_cast<const uint32_t*>(a.z + n * a.z_sn + off);
        const bool full = ow0 + 3 < a.OW;
        uint32_t zw[4] = {0u, 0u, 0u, 0u};
        if (FAST ? HZ : a.epi.has_z != 0) {
            if (full) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(zp);
                zw[0] = v[0]; zw[1] = v[1]; zw[2] = v[2]; zw[3] = v[3];
            } else {
#pragma unroll
                for (int x = 0; x < 4; ++x) zw[x] = ow0 + x < a.OW ? zp[x] : 0u;
            }
        }
        u32x4 o;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            if (FAST)
                o[x] = requant4_fast<NL, HZ>(acc[r][x][0], acc[r][x][1], acc[r][x][2], acc[r][x][3], zw[x], a.epi);
            else
                o[x] = requant4_exact(acc[r][x][0], acc[r][x][1], acc[r][x][2], acc[r][x][3], zw[x], a.epi);
        }
        if (full) {
            *reinterpret_cast<u32x4*>(dp) = o;
        } else {
#pragma unroll
            for (int x = 0; x < 4; ++x)
                if (ow0 + x < a.OW) dp[x] = o[x];
        }
    }
}

// EPI: the requantisation form compiled into the kernel -- 0: the one-FMA linear form, 1: RELU without a residual (multi-step
// fast form), 2: any other, chosen at run time.  BUF: input rows through bounds-checked buffer loads (tensors below
// 2 GiB, padding at most 1); otherwise pointer loads.  The two common forms of the MobileNet family get kernels that
// hold nothing else: a launch of a few microseconds should not have to fetch eight epilogues' worth of code.
template <int S, int R, int EPI, bool BUF>
__global__ __launch_bounds__(256) void dw3x3_kernel(Dw3Args a) {
    // Every kernel argument is requested in one batch of scalar loads: left alone the compiler fetches them where they
    // are first used, behind the early exit and the item decoding -- three dependent round trips to the argument
    // segment before the first vector load of a kernel whose whole life is a few microseconds.
    asm volatile("" ::"s"(a.src), "s"(a.flt), "s"(a.bias), "s"(a.z), "s"(a.dst), "s"(a.CG), "s"(a.IH), "s"(a.IW), "s"(a.OH),
                 "s"(a.OW), "s"(a.QW), "s"(a.OHS), "s"(a.ph), "s"(a.pw), "s"(a.items), "s"(a.src_bytes), "s"(a.src_sn),
                 "s"(a.dst_sn), "s"(a.z_sn), "s"(a.has_bias));
    asm volatile("" ::"s"(a.div_qw.m), "s"(a.div_qw.s1), "s"(a.div_qw.s2), "s"(a.div_ohs.m), "s"(a.div_ohs.s1),
                 "s"(a.div_ohs.s2), "s"(a.div_cg.m), "s"(a.div_cg.s1), "s"(a.div_cg.s2), "s"(a.epi.fast), "s"(a.epi.lin),
                 "s"(a.epi.has_z), "s"(a.epi.nonline), "s"(a.epi.lin_c), "s"(a.epi.lin_d), "s"(a.epi.lin_lo));
    const uint32_t item = blockIdx.x * 256u + threadIdx.x;
    if (item >= a.items) return;
    // item = ((n * CG + cg) * OHS + strip) * QW + quad
    const uint32_t i1 = fdiv(item, a.div_qw), q = item - i1 * a.QW;
    const uint32_t i2 = fdiv(i1, a.div_ohs), strip = i1 - i2 * a.OHS;
    const uint32_t n = fdiv(i2, a.div_cg), cg = i2 - n * a.CG;
    const int oh0 = (int)strip * R, ow0 = (int)q * 4;

    // The filter and the bias of this thread's channel quad are requested here and used only after the input rows
    // have been requested too (below): one round trip to memory for everything the thread reads, not two.
    uint32_t wraw[9];
    {
        const uint32_t* wp = reinterpret_cast<const uint32_t*>(a.flt) + cg * 9;
#pragma unroll
        for (int i = 0; i < 9; ++i) wraw[i] = wp[i];
    }
    // (a bounds-checked load: without a bias the buffer has no bytes and every lane reads zeros -- no branch whose join
    // would make the compiler wait for the load on the spot)
    const __amdgpu_buffer_rsrc_t rs_bias =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(a.bias), 0, a.has_bias ? a.CG * 16 : 0, 0x00020000);
    const v4i bias4 = __builtin_amdgcn_raw_buffer_load_b128(rs_bias, (int)cg * 16, 0, 0);
    int acc[R][4][4];

    const uint32_t* sp = reinterpret_cast<const uint32_t*>(a.src + n * a.src_sn) + (int64_t)cg * a.IH * a.IW;
    const int c0 = ow0 * S - a.pw;              // leftmost input column of this thread's window
    constexpr int ROWS = (R - 1) * S + 3;       // input rows touched by R output rows
    // window columns: L = c0, block T = c0+1 .. c0+4, then (S = 1) Rt = c0+5 or (S = 2) block U = c0+5 .. c0+8
    uint32_t L[ROWS], Rt[ROWS], pt[ROWS][4], pu[ROWS][4];
    const bool interior = c0 + 1 >= 0 && c0 + (S == 1 ? 4 : 8) < a.IW;
    if (BUF) {
        // Bounds-checked buffer loads with 32-bit offsets, the same straight-line code for every thread.  A row outside
        // the image, or a side column outside the row, becomes the out-of-range offset and reads zeros: nothing to
        // clamp.  The 4-pixel blocks always start inside the row (pw <= 1); where one runs past the end of the row
        // its surplus pixels (the next row's, or zeros past the tensor) are masked -- only in wavefronts that hold such
        // a thread, so whole rows of interior threads carry no masks at all.
        constexpr int OOR = (int)0x80000000;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.src), 0, a.src_bytes, 0x00020000);
        const bool lok = (unsigned)c0 < (unsigned)a.IW, rtok = (unsigned)(c0 + 5) < (unsigned)a.IW;
        const int base = (int)(n * (uint32_t)a.src_sn) + ((int)cg * a.IH * a.IW + c0) * 4;
#pragma unroll
        for (int ir = 0; ir < ROWS; ++ir) {
            const int ih = oh0 * S + ir - a.ph;
            const bool rok = (unsigned)ih < (unsigned)a.IH;
            const int ro = base + ih * a.IW * 4;
            L[ir] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, (rok && lok) ? ro : OOR, 0, 0);
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, rok ? ro + 4 : OOR, 0, 0);
            pt[ir][0] = v[0]; pt[ir][1] = v[1]; pt[ir][2] = v[2]; pt[ir][3] = v[3];
            if (S == 1) {
                Rt[ir] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, (rok && rtok) ? ro + 20 : OOR, 0, 0);
            } else {
                const u32x4 u = __builtin_amdgcn_raw_buffer_load_b128(rs, rok ? ro + 20 : OOR, 0, 0);
                pu[ir][0] = u[0]; pu[ir][1] = u[1]; pu[ir][2] = u[2]; pu[ir][3] = u[3];
            }
        }
        if (__builtin_amdgcn_ballot_w64(!interior) != 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool tok = (unsigned)(c0 + 1 + i) < (unsigned)a.IW, uok = (unsigned)(c0 + 5 + i) < (unsigned)a.IW;
#pragma unroll
                for (int ir = 0; ir < ROWS; ++ir) {
                    pt[ir][i] = tok ? pt[ir][i] : 0u;
                    if (S == 2) pu[ir][i] = uok ? pu[ir][i] : 0u;
                }
            }
        }
    } else if (interior) {
        // every vector load is in range: rows are clamped and masked afterwards, so all loads of the thread are
        // independent of any branch and go out back to back
        const bool lok = c0 >= 0, rtok = c0 + 5 < a.IW;
        const int cl = lok ? c0 : 0, cr = rtok ? c0 + 5 : 0;
#pragma unroll
        for (int ir = 0; ir < ROWS; ++ir) {
            const int ih = oh0 * S + ir - a.ph;
            const int ihc = min(max(ih, 0), a.IH - 1);
            const uint32_t* row = sp + ihc * a.IW;
            L[ir] = row[cl];
            const u32x4 v = *reinterpret_cast<const u32x4*>(row + c0 + 1);  // needs 4-byte alignment only
            pt[ir][0] = v[0]; pt[ir][1] = v[1]; pt[ir][2] = v[2]; pt[ir][3] = v[3];
            if (S == 1) {
                Rt[ir] = row[cr];
            } else {
                const u32x4 u = *reinterpret_cast<const u32x4*>(row + c0 + 5);
                pu[ir][0] = u[0]; pu[ir][1] = u[1]; pu[ir][2] = u[2]; pu[ir][3] = u[3];
            }
        }
#pragma unroll
        for (int ir = 0; ir < ROWS; ++ir) {
            const int ih = oh0 * S + ir - a.ph;
            const bool rok = (unsigned)ih < (unsigned)a.IH;
            L[ir] = (rok && lok) ? L[ir] : 0u;
#pragma unroll
            for (int i = 0; i < 4; ++i) pt[ir][i] = rok ? pt[ir][i] : 0u;
            if (S == 1) {
                Rt[ir] = (rok && rtok) ? Rt[ir] : 0u;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) pu[ir][i] = rok ? pu[ir][i] : 0u;
            }
        }
    } else {
#pragma unroll
        for (int ir = 0; ir < ROWS; ++ir) {
            const int ih = oh0 * S + ir - a.ph;
            const bool rok = (unsigned)ih < (unsigned)a.IH;
            const uint32_t* row = sp + (int64_t)ih * a.IW;
            L[ir] = (rok && (unsigned)c0 < (unsigned)a.IW) ? row[c0] : 0u;
            load_px4(row, c0 + 1, a.IW, rok, pt[ir]);
            if (S == 1)
                Rt[ir] = (rok && (unsigned)(c0 + 5) < (unsigned)a.IW) ? row[c0 + 5] : 0u;
            else
                load_px4(row, c0 + 5, a.IW, rok, pu[ir]);
        }
    }

    // filter rows per channel: wlo = {w(fh,0), w(fh,1), w(fh,2), 0}, whi = the same one byte up
    uint32_t wlo[3][4], whi[3][4];
#pragma unroll
    for (int fh = 0; fh < 3; ++fh) {
        const uint32_t w0 = wraw[fh * 3], w1 = wraw[fh * 3 + 1], w2 = wraw[fh * 3 + 2];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t t = perm(w1, w0, 0x0c0c0000u | ((4u + c) << 8) | (uint32_t)c);
            wlo[fh][c] = perm(w2, t, 0x0c000100u | ((4u + c) << 16));
            whi[fh][c] = wlo[fh][c] << 8;
        }
    }

#pragma unroll
    for (int ir = 0; ir < ROWS; ++ir) {
        uint32_t T[4], U[4] = {0u, 0u, 0u, 0u};
        transpose4(pt[ir], T);
        if (S == 2) transpose4(pu[ir], U);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            // three-tap windows of the 4 outputs, one channel: e[x] holds the taps in the bytes its filter row expects
            uint32_t e0, e1, e2, e3;
            e0 = perm(T[c], L[ir], 0x0c050400u | (uint32_t)c);               // {L.c, T0, T1, -}   -> wlo
            if (S == 1) {
                e1 = T[c];                                                     // {T0, T1, T2, -}    -> wlo
                e2 = T[c];                                                     // {-, T1, T2, T3}    -> whi
                e3 = perm(Rt[ir], T[c], 0x0003020cu | ((4u + c) << 24));       // {-, T2, T3, Rt.c}  -> whi
            } else {
                e1 = T[c];                                                     // {-, T1, T2, T3}    -> whi
                e2 = perm(U[c], T[c], 0x0c050403u);                            // {T3, U0, U1, -}    -> wlo
                e3 = U[c];                                                     // {-, U1, U2, U3}    -> whi
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int fh = ir - r * S;
                if (fh < 0 || fh > 2) continue;
                const int lo = (int)wlo[fh][c], hi = (int)whi[fh][c];
                if (fh == 0) {
                    // the first filter row of an output row starts from the bias: the three-operand form of the dot
                    // product reads it in place (the compiler's accumulate-in-place form costs a copy per accumulator)
                    acc[r][0][c] = dot4_from(e0, lo, bias4[c]);
                    acc[r][1][c] = dot4_from(e1, S == 1 ? lo : hi, bias4[c]);
                    acc[r][2][c] = dot4_from(e2, S == 1 ? hi : lo, bias4[c]);
                    acc[r][3][c] = dot4_from(e3, hi, bias4[c]);
                    continue;
                }
                acc[r][0][c] = __builtin_amdgcn_sdot4((int)e0, lo, acc[r][0][c], false);
                acc[r][1][c] = __builtin_amdgcn_sdot4((int)e1, S == 1 ? lo : hi, acc[r][1][c], false);
                acc[r][2][c] = __builtin_amdgcn_sdot4((int)e2, S == 1 ? hi : lo, acc[r][2][c], false);
                acc[r][3][c] = __builtin_amdgcn_sdot4((int)e3, hi, acc[r][3][c], false);
            }
        }
    }

    if (EPI == 0) {
        dw3_store<R, NL_LIN, false, true>(a, acc, n, cg, oh0, ow0);
    } else if (EPI == 1) {
        dw3_store<R, NL_RELU, false, true>(a, acc, n, cg, oh0, ow0);
    } else if (!a.epi.fast) {
        dw3_store<R, 0, false, false>(a, acc, n, cg, oh0, ow0);
    } else if (a.epi.lin) {
        dw3_store<R, NL_LIN, false, true>(a, acc, n, cg, oh0, ow0);
    } else if (a.epi.has_z) {
        switch (a.epi.nonline) {
            case NL_RELU: dw3_store<R, NL_RELU, true, true>(a, acc, n, cg, oh0, ow0); break;
            case NL_H_SWISH: dw3_store<R, NL_H_SWISH, true, true>(a, acc, n, cg, oh0, ow0); break;
            default: dw3_store<R, NL_IDENTITY, true, true>(a, acc, n, cg, oh0, ow0); break;
        }
    } else {
        switch (a.epi.nonline) {
            case NL_RELU: dw3_store<R, NL_RELU, false, true>(a, acc, n, cg, oh0, ow0); break;
            case NL_H_SWISH: dw3_store<R, NL_H_SWISH, false, true>(a, acc, n, cg, oh0, ow0); break;
            default: dw3_store<R, NL_IDENTITY, false, true>(a, acc, n, cg, oh0, ow0); break;
        }
    }
}

template <int S, int R>
void launch_dw3(hipStream_t st, dim3 grid, const Dw3Args& b) {
    const bool buf = b.src_bytes != 0 && b.pw <= 1;
    const int epi = !b.epi.fast ? 2 : b.epi.lin ? 0 : (!b.epi.has_z && b.epi.nonline == NL_RELU) ? 1 : 2;
    const dim3 block(256);
    if (buf) {
        if (epi == 0) hipLaunchKernelGGL((dw3x3_kernel<S, R, 0, true>), grid, block, 0, st, b);
        else if (epi == 1) hipLaunchKernelGGL((dw3x3_kernel<S, R, 1, true>), grid, block, 0, st, b);
        else hipLaunchKernelGGL((dw3x3_kernel<S, R, 2, true>), grid, block, 0, st, b);
    } else {
        hipLaunchKernelGGL((dw3x3_kernel<S, R, 2, false>), grid, block, 0, st, b);
    }
}

}  // namespace

bool depthwise_usable(const ConvProblem& p) {
    const mi355_conv_desc& d = p.d;
    if (!p.dw4) return false;
    if (d.mode != MI355_MODE_CROSS_CORRELATION || d.dilate_h != 1 || d.dilate_w != 1) return false;
    if (d.dst_dtype != MI355_DT_QS8 || d.bias_mode == MI355_BIAS_FULL) return false;
    const int64_t lim = (int64_t)1 << 31;
    if ((int64_t)d.ic * d.ih * d.iw >= lim || (int64_t)d.oc * p.oh * p.ow >= lim) return false;
    if ((int64_t)d.n * (d.ic / 4) > 65535) return false;
    return true;
}

int launch_conv_depthwise(hipStream_t st, const ConvProblem& p, const int8_t* src, const int8_t* flt,
                          const int32_t* bias, const int8_t* z, int8_t* dst) {
    const mi355_conv_desc& d = p.d;
    DwArgs a;
    a.src = src; a.flt = flt; a.bias = bias; a.z = z; a.dst = dst;
    a.CG = d.ic / 4; a.IH = d.ih; a.IW = d.iw; a.OH = p.oh; a.OW = p.ow; a.QW = (p.ow + 3) / 4;
    a.FH = d.fh; a.FW = d.fw; a.sh = d.stride_h; a.sw = d.stride_w; a.ph = d.pad_h; a.pw = d.pad_w;
    a.src_sn = p.src_sn; a.dst_sn = p.dst_sn; a.z_sn = p.z_sn;
    a.has_bias = d.bias_mode == MI355_BIAS_BROADCAST_CHANNEL;
    a.vec_ok = (p.ow % 4 == 0) && (p.dst_sn % 16 == 0) && (!d.has_z || p.z_sn % 16 == 0);
    a.epi = p.epi;
    if (d.n == 0 || p.oh == 0 || p.ow == 0) return 0;
    const bool sq = d.fh == 3 && d.fw == 3 && d.stride_h == d.stride_w && (d.stride_h == 1 || d.stride_h == 2);
    if (sq) {
        const int R = d.stride_h == 1 ? (p.oh % 4 == 0 ? 4 : 2) : (p.oh % 2 == 0 ? 2 : 1);
        Dw3Args b;
        b.src = src; b.flt = flt; b.bias = bias; b.z = z; b.dst = dst;
        b.CG = a.CG; b.IH = a.IH; b.IW = a.IW; b.OH = a.OH; b.OW = a.OW; b.QW = a.QW; b.OHS = (a.OH + R - 1) / R;
        b.ph = a.ph; b.pw = a.pw;
        b.src_sn = a.src_sn; b.dst_sn = a.dst_sn; b.z_sn = a.z_sn; b.has_bias = a.has_bias; b.epi = a.epi;
        const int64_t items = (int64_t)d.n * b.CG * b.OHS * b.QW;
        if (items < ((int64_t)1 << 31) - 256) {
            b.items = (uint32_t)items;
            const int64_t src_total = (int64_t)(d.n - 1) * p.src_sn + (int64_t)d.ic * d.ih * d.iw;
            b.src_bytes = src_total < ((int64_t)1 << 31) ? (uint32_t)src_total : 0u;
            b.div_qw = make_fastdiv(b.QW); b.div_ohs = make_fastdiv(b.OHS); b.div_cg = make_fastdiv(b.CG);
            const dim3 grid((unsigned)((items + 255) / 256));
            if (d.stride_h == 1 && R == 4)
                launch_dw3<1, 4>(st, grid, b);
            else if (d.stride_h == 1)
                launch_dw3<1, 2>(st, grid, b);
            else if (R == 2)
                launch_dw3<2, 2>(st, grid, b);
            else
                launch_dw3<2, 1>(st, grid, b);
            return (int)hipGetLastError();
        }
    }
    const int quads = a.OH * a.QW;
    const int threads = quads >= 192 ? 256 : (quads > 64 ? 128 : 64);
    dim3 grid((quads + threads - 1) / threads, d.n * a.CG), block(threads);
    hipLaunchKernelGGL((dw4_kernel<0, 0>), grid, block, 0, st, a);
    return (int)hipGetLastError();
}

}  // namespace mi355
