// First-layer int8 ConvBias on the matrix cores: NCHW4 activations with exactly 4 input channels
// (the 7x7 / stride 2 stem of ResNet, 3x3 stems of mobile networks), filter (OC, 1, FH, FW, 4).
//
// With 4 channels a filter row is FW * 4 contiguous bytes in the filter AND in the image, so the
// reduction is re-blocked as one 32-byte k-chunk per filter row: 8 taps x 4 channels, taps >= FW
// carrying zero weights.  A workgroup
//   * keeps the zero-padded weights of 64 output channels in LDS (written once per channel tile),
//   * stages the input patch of an 8 x 16 output-pixel tile in LDS once (double buffered; the next
//     tile's patch is fetched into registers while this tile is multiplied), and
//   * reads every MFMA B-fragment straight from the patch: lane (pixel, half) needs taps
//     4*half .. 4*half+3 of filter row fh = 16 contiguous patch bytes.
// The im2col matrix is never formed and each input byte is fetched from global memory about 1.5
// times (patch halo) instead of FH * FW / stride^2 times.
//
// v_mfma_i32_32x32x32_i8: A = 32 output channels, B = 32 pixels (2 output rows x 16 columns of the
// tile), accumulator layout as in conv_igemm.hip; epilogue per lane: 4 consecutive channels of one
// pixel = one dword of the NCHW4 output.
#include <atomic>

#include "common.h"

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int C4_THREADS = 256;
constexpr int C4_BM = 64;             // output channels per tile
constexpr int C4_TH = 8, C4_TW = 16;  // output pixels per tile
constexpr int C4_MAXF = 8;            // filter rows / taps per row

struct C4Args {
    const int8_t* src;
    const int8_t* flt;
    const int32_t* bias;
    const int8_t* z;
    int8_t* dst;
    int N, IH, IW, OH, OW, OC, FH, FW, ph, pw;
    int src_sn, dst_sn, z_sn;  // batch strides in bytes
    uint32_t dst_bytes, dst_bytes_z;  // extents of dst and z for the buffer descriptors
    int has_bias;
    int tiles_w, tiles_h, tiles_m, tiles;  // tile = ((mt * N + n) * tiles_h + th) * tiles_w + tw
    FastDiv div_tw, div_th, div_n;
    EpiParams epi;
};

template <int S>
struct C4Geom {
    // patch row pitch in dwords (>= 15 * S + 8); S * PWD = 32 mod 64 puts the two pixel rows of a wave's block on
    // disjoint LDS banks
    static constexpr int PWD = S == 2 ? 48 : 32;
    static constexpr int MAXROWS = (C4_TH - 1) * S + C4_MAXF;        // patch rows for the tallest filter
    static constexpr int PREG = (MAXROWS * PWD + C4_THREADS - 1) / C4_THREADS;  // patch dwords per thread
};

struct C4Tile {
    int mt, n, oh0, ow0;
};

__device__ __forceinline__ C4Tile c4_decode(const C4Args& a, int tile) {
    C4Tile r;
    const uint32_t q1 = fdiv((uint32_t)tile, a.div_tw), tw = tile - q1 * a.tiles_w;
    const uint32_t q2 = fdiv(q1, a.div_th), th = q1 - q2 * a.tiles_h;
    const uint32_t mt = fdiv(q2, a.div_n), n = q2 - mt * a.N;
    r.mt = (int)mt; r.n = (int)n; r.oh0 = (int)th * C4_TH; r.ow0 = (int)tw * C4_TW;
    return r;
}

template <int S>
__device__ __forceinline__ void c4_fetch_patch(const C4Args& a, const C4Tile& tl, int rows, int t,
                                               uint32_t (&reg)[C4Geom<S>::PREG]) {
    using G = C4Geom<S>;
    const uint32_t* sp = reinterpret_cast<const uint32_t*>(a.src + (int64_t)tl.n * a.src_sn);
    const int gy0 = tl.oh0 * S - a.ph, gx0 = tl.ow0 * S - a.pw;
#pragma unroll
    for (int j = 0; j < G::PREG; ++j) {
        const int idx = t + C4_THREADS * j;
        const int row = idx / G::PWD, col = idx - row * G::PWD;
        const int gy = gy0 + row, gx = gx0 + col;
        const bool ok = row < rows && (unsigned)gy < (unsigned)a.IH && (unsigned)gx < (unsigned)a.IW;
        reg[j] = ok ? sp[gy * a.IW + gx] : 0u;
    }
}

template <int S>
__device__ __forceinline__ void c4_store_patch(uint32_t* sP, int t, const uint32_t (&reg)[C4Geom<S>::PREG]) {
    using G = C4Geom<S>;
#pragma unroll
    for (int j = 0; j < G::PREG; ++j) {
        const int idx = t + C4_THREADS * j;
        if (idx < G::MAXROWS * G::PWD) sP[idx] = reg[j];
    }
}

// weights of channel tile mt, re-blocked to 8 taps per filter row (zeros past FW and past OC), and its bias
__device__ __forceinline__ void c4_load_weights(const C4Args& a, int mt, uint32_t* sW, int wrow_dw, int* sBias, int t) {
    const uint32_t* fp = reinterpret_cast<const uint32_t*>(a.flt);
    const int per_oc = a.FH * 8;
    for (int idx = t; idx < C4_BM * per_oc; idx += C4_THREADS) {
        const int oc = idx / per_oc, rem = idx - oc * per_oc;
        const int fh = rem >> 3, tap = rem & 7;
        const int goc = mt * C4_BM + oc;
        uint32_t v = 0u;
        if (goc < a.OC && tap < a.FW) v = fp[(goc * a.FH + fh) * a.FW + tap];
        sW[oc * wrow_dw + fh * 8 + tap] = v;
    }
    if (t < C4_BM) {
        const int goc = mt * C4_BM + t;
        sBias[t] = (a.has_bias && goc < a.OC) ? a.bias[goc] : 0;
    }
}

// dst / z byte offsets of this lane's 8 output dwords (SENT where the pixel or the channel quad is outside the tensor:
// a buffer access at that offset is dropped / returns 0, so neither loads nor stores need a branch)
__device__ __forceinline__ void c4_offsets(const C4Args& a, const C4Tile& tl, int oh, int ow, int lh, int sn, int (&off)[2][4]) {
    const bool pok = oh < a.OH && ow < a.OW;
    const int plane4 = a.OH * a.OW * 4;
    const int base = tl.n * sn + (oh * a.OW + ow) * 4;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int oc4 = tl.mt * C4_BM + i * 32 + 8 * q + 4 * lh;
            off[i][q] = (pok && oc4 < a.OC) ? base + (oc4 >> 2) * plane4 : (int)0x80000000;
        }
}

template <int NL, bool HZ>
__device__ __forceinline__ void c4_epilogue(const C4Args& a, const v16i (&acc)[2], const uint32_t (&zr)[2][4],
                                            const int (&off)[2][4], __amdgpu_buffer_rsrc_t rs_dst) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const v16i& c = acc[i];
            const uint32_t o = requant4_fast<NL, HZ>(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], zr[i][q], a.epi);
            __builtin_amdgcn_raw_buffer_store_b32(o, rs_dst, off[i][q], 0, 0);
        }
}

template <int S>
__global__ __launch_bounds__(C4_THREADS, 3) void c4_kernel(C4Args a) {
    using G = C4Geom<S>;
    __shared__ __attribute__((aligned(16))) uint32_t sW[C4_BM * (C4_MAXF * 8 + 4)];
    __shared__ __attribute__((aligned(16))) uint32_t sP[2][G::MAXROWS * G::PWD];
    __shared__ int sBias[C4_BM];

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l32 = lane & 31, lh = lane >> 5;
    const int r = l32 >> 4, c = l32 & 15;  // pixel of this lane inside the wave's 2 x 16 block
    const int wrow_dw = a.FH * 8 + 4;      // 16 bytes of padding per weight row: conflict-free 128-bit reads
    const int rows = (C4_TH - 1) * S + a.FH;

    const __amdgpu_buffer_rsrc_t rs_dst = __builtin_amdgcn_make_buffer_rsrc(a.dst, 0, a.dst_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_z =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.z), 0, a.epi.has_z ? a.dst_bytes_z : 0, 0x00020000);

    int tile = blockIdx.x;
    if (tile >= a.tiles) return;
    C4Tile tl = c4_decode(a, tile);
    uint32_t preg[G::PREG];
    c4_fetch_patch<S>(a, tl, rows, t, preg);
    c4_load_weights(a, tl.mt, sW, wrow_dw, sBias, t);
    c4_store_patch<S>(sP[0], t, preg);
    __syncthreads();

    int buf = 0;
    while (true) {
        const int next = tile + gridDim.x;
        const bool has_next = next < a.tiles;
        C4Tile tn = tl;
        if (has_next) {
            tn = c4_decode(a, next);
            c4_fetch_patch<S>(a, tn, rows, t, preg);  // in flight during the MFMAs and the epilogue
        }
        const int oh = tl.oh0 + 2 * w + r, ow = tl.ow0 + c;
        // residual of this lane's pixel, requested before the MFMAs
        int doff[2][4];
        c4_offsets(a, tl, oh, ow, lh, a.dst_sn, doff);
        uint32_t zr[2][4] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
        if (a.epi.has_z) {
            int zoff[2][4];
            c4_offsets(a, tl, oh, ow, lh, a.z_sn, zoff);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) zr[i][q] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_z, zoff[i][q], 0, 0);
        }

        v16i acc[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i b = *reinterpret_cast<const v4i*>(sBias + i * 32 + 8 * q + 4 * lh);
                acc[i][4 * q + 0] = b[0]; acc[i][4 * q + 1] = b[1]; acc[i][4 * q + 2] = b[2]; acc[i][4 * q + 3] = b[3];
            }
        const uint32_t* pb = sP[buf] + ((2 * w + r) * S) * G::PWD + c * S + 4 * lh;
        const uint32_t* wa = sW + l32 * wrow_dw + lh * 4;
        // filter rows two at a time: the fragment reads of the next row are in flight while this row multiplies
        struct Frag {
            v4i b, a0, a1;
        };
        auto frags = [&](int fh, Frag& f) __attribute__((always_inline)) {
            const uint32_t* p = pb + fh * G::PWD;
            if (S == 2) {  // c * 2 + 4 * lh is even: 8-byte aligned
                const u32x2 lo = *reinterpret_cast<const u32x2*>(p), hi = *reinterpret_cast<const u32x2*>(p + 2);
                f.b[0] = (int)lo[0]; f.b[1] = (int)lo[1]; f.b[2] = (int)hi[0]; f.b[3] = (int)hi[1];
            } else {
                f.b[0] = (int)p[0]; f.b[1] = (int)p[1]; f.b[2] = (int)p[2]; f.b[3] = (int)p[3];
            }
            f.a0 = *reinterpret_cast<const v4i*>(wa + fh * 8);
            f.a1 = *reinterpret_cast<const v4i*>(wa + 32 * wrow_dw + fh * 8);
        };
        auto mfmas = [&](const Frag& f) __attribute__((always_inline)) {
            acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.a0, f.b, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.a1, f.b, acc[1], 0, 0, 0);
        };
        Frag f0, f1;
        frags(0, f0);
        for (int fh = 0; fh < a.FH; fh += 2) {
            const bool odd = fh + 1 < a.FH;
            if (odd) frags(fh + 1, f1);
            mfmas(f0);
            if (odd) {
                if (fh + 2 < a.FH) frags(fh + 2, f0);
                mfmas(f1);
            }
        }

        // The next tile's patch goes into LDS BEFORE this tile's stores are issued: the wait for its loads then counts no
        // store (vector-memory operations are counted together and retire in order; behind the epilogue the same wait
        // stood for fifteen of this tile's sixteen stores, i.e. every tile paid the latency of its own stores).
        if (has_next) {
            if (tn.mt != tl.mt) {
                __syncthreads();  // every wave is done with the old weights
                c4_load_weights(a, tn.mt, sW, wrow_dw, sBias, t);
            }
            c4_store_patch<S>(sP[buf ^ 1], t, preg);
            __syncthreads();
        }
        if (a.epi.lin) {
            c4_epilogue<NL_LIN, false>(a, acc, zr, doff, rs_dst);
        } else if (a.epi.has_z) {
            switch (a.epi.nonline) {
                case NL_RELU: c4_epilogue<NL_RELU, true>(a, acc, zr, doff, rs_dst); break;
                case NL_H_SWISH: c4_epilogue<NL_H_SWISH, true>(a, acc, zr, doff, rs_dst); break;
                default: c4_epilogue<NL_IDENTITY, true>(a, acc, zr, doff, rs_dst); break;
            }
        } else {
            switch (a.epi.nonline) {
                case NL_RELU: c4_epilogue<NL_RELU, false>(a, acc, zr, doff, rs_dst); break;
                case NL_H_SWISH: c4_epilogue<NL_H_SWISH, false>(a, acc, zr, doff, rs_dst); break;
                default: c4_epilogue<NL_IDENTITY, false>(a, acc, zr, doff, rs_dst); break;
            }
        }
        if (!has_next) break;
        buf ^= 1;
        tile = next;
        tl = tn;
    }
}

}  // namespace

bool c4_usable(const ConvProblem& p) {
    const mi355_conv_desc& d = p.d;
    if (d.format != MI355_FMT_NCHW4 || d.group != 1 || p.dw4 || d.ic != 4) return false;
    if (d.mode != MI355_MODE_CROSS_CORRELATION || d.dilate_h != 1 || d.dilate_w != 1) return false;
    if (d.dst_dtype != MI355_DT_QS8 || d.bias_mode == MI355_BIAS_FULL || !p.epi.fast) return false;
    if (d.fh > C4_MAXF || d.fw > C4_MAXF) return false;
    if (d.stride_h != d.stride_w || (d.stride_h != 1 && d.stride_h != 2)) return false;
    if (d.pad_h > 0xfff || d.pad_w > 0xfff) return false;
    const int64_t lim = (int64_t)1 << 31;
    const int64_t src_b = (int64_t)(d.n - 1) * p.src_sn + (int64_t)4 * d.ih * d.iw;
    const int64_t dst_b = (int64_t)(d.n - 1) * p.dst_sn + (int64_t)d.oc * p.oh * p.ow;
    const int64_t z_b = d.has_z ? (int64_t)(d.n - 1) * p.z_sn + (int64_t)d.oc * p.oh * p.ow : 0;
    if (src_b >= lim || dst_b >= lim || z_b >= lim || p.src_sn >= lim || p.dst_sn >= lim || p.z_sn >= lim) return false;
    const int64_t tiles = (int64_t)((d.oc + C4_BM - 1) / C4_BM) * d.n * ((p.oh + C4_TH - 1) / C4_TH) * ((p.ow + C4_TW - 1) / C4_TW);
    return tiles > 0 && tiles < lim;
}

int launch_conv_c4(hipStream_t st, const ConvProblem& p, int cu_count, const int8_t* src, const int8_t* flt,
                   const int32_t* bias, const int8_t* z, int8_t* dst) {
    const mi355_conv_desc& d = p.d;
    C4Args a;
    a.src = src; a.flt = flt; a.bias = bias; a.z = z; a.dst = dst;
    a.N = d.n; a.IH = d.ih; a.IW = d.iw; a.OH = p.oh; a.OW = p.ow; a.OC = d.oc; a.FH = d.fh; a.FW = d.fw;
    a.ph = d.pad_h; a.pw = d.pad_w;
    a.src_sn = (int)p.src_sn; a.dst_sn = (int)p.dst_sn; a.z_sn = (int)p.z_sn;
    a.has_bias = d.bias_mode == MI355_BIAS_BROADCAST_CHANNEL;
    a.dst_bytes = (uint32_t)((int64_t)(d.n - 1) * p.dst_sn + (int64_t)d.oc * p.oh * p.ow);
    a.dst_bytes_z = d.has_z ? (uint32_t)((int64_t)(d.n - 1) * p.z_sn + (int64_t)d.oc * p.oh * p.ow) : 0;
    a.tiles_w = (p.ow + C4_TW - 1) / C4_TW;
    a.tiles_h = (p.oh + C4_TH - 1) / C4_TH;
    a.tiles_m = (d.oc + C4_BM - 1) / C4_BM;
    a.tiles = a.tiles_m * a.N * a.tiles_h * a.tiles_w;
    a.div_tw = make_fastdiv(a.tiles_w); a.div_th = make_fastdiv(a.tiles_h); a.div_n = make_fastdiv(a.N);
    a.epi = p.epi;
    if (a.tiles == 0) return 0;
    if (cu_count <= 0) cu_count = 256;
    // persistent grid: exactly as many workgroups as are resident at once (a workgroup that had to wait for a
    // slot would start its whole share of tiles late)
    static std::atomic<int> occ[2];  // zero-initialised; several threads may launch
    const int si = d.stride_h == 2 ? 1 : 0;
    if (!occ[si].load(std::memory_order_relaxed)) {
        int o = 0;
        hipError_t e = si ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&o, reinterpret_cast<const void*>(c4_kernel<2>), C4_THREADS, 0)
                          : hipOccupancyMaxActiveBlocksPerMultiprocessor(&o, reinterpret_cast<const void*>(c4_kernel<1>), C4_THREADS, 0);
        if (e != hipSuccess || o < 1) {
            (void)hipGetLastError();
            o = 1;
        }
        occ[si].store(o, std::memory_order_relaxed);
    }
    int64_t grid = (int64_t)occ[si].load(std::memory_order_relaxed) * cu_count;
    if (grid > a.tiles) grid = a.tiles;
    if (si)
        hipLaunchKernelGGL((c4_kernel<2>), dim3((unsigned)grid), dim3(C4_THREADS), 0, st, a);
    else
        hipLaunchKernelGGL((c4_kernel<1>), dim3((unsigned)grid), dim3(C4_THREADS), 0, st, a);
    return (int)hipGetLastError();
}

}  // namespace mi355
