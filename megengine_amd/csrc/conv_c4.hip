// First-layer int8 ConvBias on the matrix cores: NCHW4 activations with exactly 4 input channels
// (the 7x7 / stride 2 stem of ResNet, 3x3 stems of mobile networks), filter (OC, 1, FH, FW, 4).
//
// With 4 channels a filter row is FW * 4 contiguous bytes in the filter AND in the image, so the
// reduction is re-blocked as one 32-byte k-chunk per filter row: 8 taps x 4 channels, taps >= FW
// carrying zero weights.  A workgroup (4 waves, a persistent loop over 64-channel x 8 x 16-pixel tiles)
//   * keeps the zero-padded weights of its 64 output channels in REGISTERS, as the A fragments of all filter rows
//     (16 bytes per lane, row and 32-channel block; loaded once per channel tile),
//   * copies the input patch of each tile from global memory straight into LDS (no register stage), three tiles
//     ahead of the one being multiplied, into a ring of four patch slots, and
//   * reads every MFMA B-fragment straight from the patch: lane (pixel, half) needs taps
//     4*half .. 4*half+3 of filter row fh = 16 contiguous patch bytes.
// The im2col matrix is never formed and each input byte is fetched from global memory about 1.5
// times (patch halo) instead of FH * FW / stride^2 times.  One barrier per tile.
//
// v_mfma_i32_32x32x32_i8: A = 32 output channels, B = 32 pixels (2 output rows x 16 columns of the
// tile), accumulator layout as in conv_igemm.hip; epilogue per lane: 4 consecutive channels of one
// pixel = one dword of the NCHW4 output.
#include <atomic>

#include "lds_copy.h"

namespace mi355 {
namespace {

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
    uint32_t src_bytes, dst_bytes, dst_bytes_z;  // extents for the buffer descriptors
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
    static constexpr int MAXROWS = (C4_TH - 1) * S + C4_MAXF;                      // patch rows for the tallest filter
    static constexpr int SLOT_DW = MAXROWS * PWD + 64;  // a ring slot, in dwords
    static constexpr int NSLOT = 4;
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

// s_waitcnt vmcnt(n) for a wave-uniform n in 0 .. 63 (the count is an immediate of the instruction)
__device__ __forceinline__ void c4_wait_vmcnt(int n) {
    switch (n) {
#define C4_W1(k) case k: wait_vmcnt<k>(); break;
#define C4_W8(k) C4_W1(k) C4_W1(k + 1) C4_W1(k + 2) C4_W1(k + 3) C4_W1(k + 4) C4_W1(k + 5) C4_W1(k + 6) C4_W1(k + 7)
        C4_W8(0) C4_W8(8) C4_W8(16) C4_W8(24) C4_W8(32) C4_W8(40) C4_W8(48) C4_W8(56)
#undef C4_W8
#undef C4_W1
        default: wait_vmcnt<63>(); break;
    }
}

// Output addressing: the 8 dwords a lane stores (and the 8 residual dwords it loads) share ONE per-lane offset
// -- its pixel and lane half -- and differ by wave-uniform plane offsets, which go into the scalar offset of the
// buffer instruction.  C4Out holds the lane part (SENT when the pixel is outside the tensor: such an access is
// dropped / returns 0) and what the scalar parts are made of.
struct C4Out {
    int voff;    // (oh * OW + ow) * 4 + lh * plane4, or SENT
    int plane4;  // bytes of one 4-channel plane
    int oc0;     // first channel of the tile
    bool full;   // all 64 channels of the tile exist
};

// scalar offset of quad (i, q): batch stride * n + plane of channel oc0 + 32 * i + 8 * q (the lane half adds 4 channels)
__device__ __forceinline__ int c4_soff(const C4Out& o, int nbase, int i, int q) {
    return nbase + ((o.oc0 + 32 * i + 8 * q) >> 2) * o.plane4;
}

// per-lane offset of quad (i, q) in a channel tile that reaches past OC
__device__ __forceinline__ int c4_voff(const C4Out& o, int OC, int lh, int i, int q) {
    return (o.full || o.oc0 + 32 * i + 8 * q + 4 * lh < OC) ? o.voff : SENT;
}

constexpr int C4_VMCNT0 = 0x0f70;  // s_waitcnt vmcnt(0) with the other counters at their maxima

template <int NL, bool HZ>
__device__ __forceinline__ void c4_epilogue(const C4Args& a, const v16i (&acc)[2], const uint32_t (&zr)[2][4],
                                            const C4Out& out, int nbase, int lh, __amdgpu_buffer_rsrc_t rs_dst) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const v16i& c = acc[i];
            const uint32_t o = requant4_fast<NL, HZ>(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], zr[i][q], a.epi);
            __builtin_amdgcn_raw_buffer_store_b32(o, rs_dst, c4_voff(out, a.OC, lh, i, q), c4_soff(out, nbase, i, q), 0);
        }
}

// HZ: the launch has a residual (its registers exist only in that instantiation); FHT: the number of filter rows when it
// is 3 or 7 (no branches between the MFMAs), 0 = any number up to 8
template <int S, bool HZ, int FHT>
__global__ __launch_bounds__(C4_THREADS, FHT ? 3 : 2) void c4_kernel(C4Args a) {
    using G = C4Geom<S>;
    __shared__ __attribute__((aligned(16))) uint32_t sP[G::NSLOT * G::SLOT_DW];
    __shared__ __attribute__((aligned(16))) uint32_t sW[C4_BM * (C4_MAXF * 8 + 4)];
    __shared__ __attribute__((aligned(16))) int sBias[C4_BM];

    const int t = threadIdx.x;
    const int lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int r = l32 >> 4, c = l32 & 15;  // pixel of this lane inside the wave's 2 x 16 block
    const int FH = FHT ? FHT : a.FH;
    const int rows = (C4_TH - 1) * S + FH;

    const int first = blockIdx.x, step = gridDim.x;
    if (first >= a.tiles) return;
    const int count = (a.tiles - 1 - first) / step + 1;  // tiles of this workgroup

    const uint32_t lds_p = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)sP);
    const v4i rs_src = uniform_rsrc(a.src, a.src_bytes);
    const __amdgpu_buffer_rsrc_t rs_dst = make_rsrc(a.dst, a.dst_bytes);
    const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(a.z, HZ ? a.dst_bytes_z : 0);

    // The patch of tile k (k-th of this workgroup) goes to ring slot k & 3, one patch row per copy: lane l < PWD holds
    // column l (the other lanes are masked off and write nothing), wave w copies rows w, w + 4, ...  The row part of the
    // address is wave-uniform and travels in the scalar offset; columns outside the image and rows outside the image are
    // zero-filled by the copy itself (out-of-range lane offset).  Returns the number of copies this wave issued.
    const int ncopy = w < rows ? (rows - w + 3) >> 2 : 0;
    auto copy_patch = [&](int k) __attribute__((always_inline)) -> int {
        const C4Tile tt = c4_decode(a, first + k * step);
        const int gy0 = tt.oh0 * S - a.ph, gx = tt.ow0 * S - a.pw + lane;
        const int vcol = (unsigned)gx < (unsigned)a.IW ? gx * 4 : SENT;
        const int base = tt.n * a.src_sn;
        const uint32_t dst = lds_p + (uint32_t)((k & (G::NSLOT - 1)) * G::SLOT_DW * 4);
        if (lane < G::PWD) {
            for (int row = w; row < rows; row += 4) {
                const int gy = gy0 + row;
                const bool ok = (unsigned)gy < (unsigned)a.IH;
                lds_copy_row64x4(dst + (uint32_t)(row * G::PWD * 4), ok ? vcol : SENT, ok ? base + gy * a.IW * 4 : 0, rs_src);
            }
        }
        return ncopy;
    };

    // A fragments of every filter row: lane (l32, lh) holds taps 4 * lh .. 4 * lh + 3 of channel i * 32 + l32, zeros for
    // taps >= FW and channels >= OC.  The filter is read once per channel tile with consecutive threads on consecutive
    // dwords, re-blocked in LDS to 8 taps per row (16 bytes of padding per channel: conflict-free 128-bit reads), and
    // from there each lane takes its fragments.
    v4i wr[C4_MAXF][2];
    const int wrow_dw = FH * 8 + 4;
    auto stage_weights = [&](int mt) __attribute__((always_inline)) {
        const uint32_t* fp = reinterpret_cast<const uint32_t*>(a.flt);
        const int per_oc = FH * 8, total = C4_BM * per_oc;
        // thread indices through an opaque copy: nothing of this rarely run block is kept in registers across the tile loop
        int tid = t;
        asm volatile("" : "+v"(tid));
        constexpr int HALF = C4_BM * C4_MAXF * 8 / C4_THREADS / 2;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t v[HALF];
#pragma unroll
            for (int j = 0; j < HALF; ++j) {  // a batch of loads before the first LDS write
                const int idx = tid + C4_THREADS * (h * HALF + j);
                const int oc = idx / per_oc, rem = idx - oc * per_oc;
                const int fh = rem >> 3, tap = rem & 7;
                const int goc = mt * C4_BM + oc;
                v[j] = (idx < total && goc < a.OC && tap < a.FW) ? fp[(goc * FH + fh) * a.FW + tap] : 0u;
            }
#pragma unroll
            for (int j = 0; j < HALF; ++j) {
                const int idx = tid + C4_THREADS * (h * HALF + j);
                const int oc = idx / per_oc, rem = idx - oc * per_oc;
                if (idx < total) sW[oc * wrow_dw + rem] = v[j];
            }
        }
    };
    auto read_weights = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int fh = 0; fh < C4_MAXF; ++fh) {
            if (fh < FH) {
#pragma unroll
                for (int i = 0; i < 2; ++i) wr[fh][i] = *reinterpret_cast<const v4i*>(sW + (i * 32 + l32) * wrow_dw + fh * 8 + lh * 4);
            }
        }
    };
    auto load_bias = [&](int mt) __attribute__((always_inline)) {
        if (t < C4_BM) {
            const int goc = mt * C4_BM + t;
            sBias[t] = (a.has_bias && goc < a.OC) ? a.bias[goc] : 0;
        }
    };

    // Vector-memory loads complete in order, so "the patch of tile k has landed" is "at most as many operations outstanding
    // as COPIES were issued after its copies": were one of its copies outstanding, so would be every younger copy.  Only
    // the copies are counted (issued = copies issued so far; mk1 / mk2 / mk3 = that count right after the copies of the
    // next / second-next / third-next tile): loads and stores the compiler issues in between only make the wait
    // stricter, whatever the order in which stores complete relative to loads.
    int issued = copy_patch(0);
    int mk1 = issued, mk2 = issued, mk3 = issued;
    if (count > 1) { issued += copy_patch(1); mk1 = issued; }
    if (count > 2) { issued += copy_patch(2); mk2 = issued; }
    C4Tile tl = c4_decode(a, first);
    stage_weights(tl.mt);
    load_bias(tl.mt);
    __builtin_amdgcn_s_waitcnt(C4_VMCNT0);  // the first patches have landed (this wave's copies; the barrier covers the rest)
    __syncthreads();
    read_weights();

    for (int k = 0; k < count; ++k) {
        if (k + 3 < count) { issued += copy_patch(k + 3); mk3 = issued; }
        const int oh = tl.oh0 + 2 * w + r, ow = tl.ow0 + c;
        C4Out out;
        out.plane4 = a.OH * a.OW * 4;
        out.voff = (oh < a.OH && ow < a.OW) ? (oh * a.OW + ow) * 4 + lh * out.plane4 : SENT;
        out.oc0 = tl.mt * C4_BM;
        out.full = out.oc0 + C4_BM <= a.OC;
        // residual of this lane's pixel, requested before the MFMAs
        uint32_t zr[2][4] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
        if constexpr (HZ) {
            const int zbase = tl.n * a.z_sn;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    zr[i][q] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_z, c4_voff(out, a.OC, lh, i, q), c4_soff(out, zbase, i, q), 0);
        }

        v16i acc[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i b = *reinterpret_cast<const v4i*>(sBias + i * 32 + 8 * q + 4 * lh);
                acc[i][4 * q + 0] = b[0]; acc[i][4 * q + 1] = b[1]; acc[i][4 * q + 2] = b[2]; acc[i][4 * q + 3] = b[3];
            }
        const uint32_t* pb = sP + (k & (G::NSLOT - 1)) * G::SLOT_DW + ((2 * w + r) * S) * G::PWD + c * S + 4 * lh;
        auto frag_b = [&](int fh) __attribute__((always_inline)) -> v4i {
            const uint32_t* p = pb + fh * G::PWD;
            v4i b;
            if (S == 2) {  // c * 2 + 4 * lh is even: 8-byte aligned
                const u32x2 lo = *reinterpret_cast<const u32x2*>(p), hi = *reinterpret_cast<const u32x2*>(p + 2);
                b[0] = (int)lo[0]; b[1] = (int)lo[1]; b[2] = (int)hi[0]; b[3] = (int)hi[1];
            } else {
                b[0] = (int)p[0]; b[1] = (int)p[1]; b[2] = (int)p[2]; b[3] = (int)p[3];
            }
            return b;
        };
        // the B fragment of the next filter row is in flight while this row multiplies
        v4i fb[2];
        fb[0] = frag_b(0);
#pragma unroll
        for (int fh = 0; fh < C4_MAXF; ++fh) {
            if (fh < FH) {
                if (fh + 1 < C4_MAXF && fh + 1 < FH) fb[(fh + 1) & 1] = frag_b(fh + 1);
                acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wr[fh][0], fb[fh & 1], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wr[fh][1], fb[fh & 1], acc[1], 0, 0, 0);
            }
        }

        // One barrier per tile, before the epilogue: the next tile's patch has landed (this wave's part; the barrier
        // covers the other waves') and every wave is done with this tile's slot, which the copies issued at the top of
        // the next iteration overwrite.
        C4Tile tn = tl;
        if (k + 1 < count) {
            tn = c4_decode(a, first + (k + 1) * step);
            const int after = issued - mk1;
            c4_wait_vmcnt(after > 63 ? 63 : after);
            __syncthreads();
            if (tn.mt != tl.mt) {  // every wave has read the old bias; the old weights are dead
                stage_weights(tn.mt);
                load_bias(tn.mt);
                __syncthreads();
                read_weights();
            }
        }
        const int dbase = tl.n * a.dst_sn;
        if constexpr (HZ) {
            switch (a.epi.nonline) {
                case NL_RELU: c4_epilogue<NL_RELU, true>(a, acc, zr, out, dbase, lh, rs_dst); break;
                case NL_H_SWISH: c4_epilogue<NL_H_SWISH, true>(a, acc, zr, out, dbase, lh, rs_dst); break;
                default: c4_epilogue<NL_IDENTITY, true>(a, acc, zr, out, dbase, lh, rs_dst); break;
            }
        } else if (a.epi.lin) {
            c4_epilogue<NL_LIN, false>(a, acc, zr, out, dbase, lh, rs_dst);
        } else {
            switch (a.epi.nonline) {
                case NL_RELU: c4_epilogue<NL_RELU, false>(a, acc, zr, out, dbase, lh, rs_dst); break;
                case NL_H_SWISH: c4_epilogue<NL_H_SWISH, false>(a, acc, zr, out, dbase, lh, rs_dst); break;
                default: c4_epilogue<NL_IDENTITY, false>(a, acc, zr, out, dbase, lh, rs_dst); break;
            }
        }
        mk1 = mk2; mk2 = mk3;
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
    a.src_bytes = (uint32_t)((int64_t)(d.n - 1) * p.src_sn + (int64_t)4 * d.ih * d.iw);
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
    using Kern = void (*)(C4Args);
    static const Kern kerns[12] = {
            c4_kernel<1, false, 0>, c4_kernel<1, false, 3>, c4_kernel<1, false, 7>, c4_kernel<1, true, 0>,
            c4_kernel<1, true, 3>,  c4_kernel<1, true, 7>,  c4_kernel<2, false, 0>, c4_kernel<2, false, 3>,
            c4_kernel<2, false, 7>, c4_kernel<2, true, 0>,  c4_kernel<2, true, 3>,  c4_kernel<2, true, 7>};
    static std::atomic<int> occ[12];  // zero-initialised; several threads may launch
    const int si = (d.stride_h == 2 ? 6 : 0) + (d.has_z ? 3 : 0) + (d.fh == 3 ? 1 : d.fh == 7 ? 2 : 0);
    if (!occ[si].load(std::memory_order_relaxed)) {
        int o = 0;
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&o, reinterpret_cast<const void*>(kerns[si]), C4_THREADS, 0);
        if (e != hipSuccess || o < 1) {
            (void)hipGetLastError();
            o = 1;
        }
        occ[si].store(o, std::memory_order_relaxed);
    }
    int64_t grid = (int64_t)occ[si].load(std::memory_order_relaxed) * cu_count;
    if (grid > a.tiles) grid = a.tiles;
    hipLaunchKernelGGL(kerns[si], dim3((unsigned)grid), dim3(C4_THREADS), 0, st, a);
    return (int)hipGetLastError();
}

}  // namespace mi355
