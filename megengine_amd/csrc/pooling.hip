// QuantizedS8 Pooling forward: MAX, AVERAGE (padding counts as zeros) and AVERAGE_COUNT_EXCLUDE_PADDING over
// NCHW, NCHW4 / NCHW44 and NCHW32 tensors, with the arithmetic of the reference's naive operator
// (dnn/src/naive/pooling/opr_impl.cpp:16-36 MaxPooler, :107-127 MeanIncludeRoundedPooler for dt_qint8,
// :237-268 MeanExcludeRoundedPooler, :270-289 the window walk): the mean is roundf(float(sum) / count), one
// correctly rounded float division and a round-half-away.
//
// A pure streaming kernel.  One thread produces one vector of VB output bytes -- 16 channels of an NCHW32
// pixel (two threads per pixel), the 4 channels of an NCHW4 pixel, one NCHW element -- so that a wave's loads
// and stores cover whole, consecutive pixels.  Overlapping windows are re-read through the vector cache; HBM sees
// every input byte about once.  The window is clipped to the image up front, so the inner loops carry no
// bounds tests.  MAX compares four bytes with two packed 16-bit maxima: bytes 1 and 3 of a word are
// compared in place (as the high bytes of the two 16-bit lanes), bytes 0 and 2 after a byte shuffle.
#include "common.h"

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef short s2 __attribute__((ext_vector_type(2)));

struct PoolArgs {
    const int8_t* src;
    int8_t* dst;
    uint32_t units;  // output vectors
    int IH, IW, OH, OW, ph, pw, sh, sw, fh, fw;
    FastDiv div_ow, div_oh;
};

enum { POOL_MAX = 0, POOL_AVG = 1, POOL_AVG_EXCL = 2 };

__device__ __forceinline__ uint32_t pk_max_i16(uint32_t a, uint32_t b) {
    const s2 r = __builtin_elementwise_max(__builtin_bit_cast(s2, a), __builtin_bit_cast(s2, b));
    return __builtin_bit_cast(uint32_t, r);
}

// running maximum of the four signed bytes of a word, kept as 2 + 2 sixteen-bit lanes (byte << 8)
struct Max4 {
    uint32_t odd, even;  // bytes 1, 3 | bytes 0, 2
    __device__ __forceinline__ void init() { odd = even = 0x80008000u; }
    __device__ __forceinline__ void feed(uint32_t w) {
        odd = pk_max_i16(odd, w & 0xff00ff00u);
        even = pk_max_i16(even, __builtin_amdgcn_perm(0u, w, 0x020c000cu));  // (w << 8) & 0xff00ff00
    }
    __device__ __forceinline__ uint32_t get() const { return odd | (even >> 8); }  // the low byte of every lane is 0
};

struct Sum4 {
    int s[4];
    __device__ __forceinline__ void init() { s[0] = s[1] = s[2] = s[3] = 0; }
    __device__ __forceinline__ void feed(uint32_t w) {
        const int x = (int)w;
        s[0] += (x << 24) >> 24;
        s[1] += (x << 16) >> 24;
        s[2] += (x << 8) >> 24;
        s[3] += x >> 24;
    }
    __device__ __forceinline__ uint32_t get(float count) const {
        uint32_t r = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int v = (int)roundf((float)s[q] / count);
            r |= ((uint32_t)v & 0xffu) << (8 * q);
        }
        return r;
    }
};

template <int VB>
struct VecIO;
template <>
struct VecIO<4> {
    uint32_t w[1];
    __device__ __forceinline__ void load(const int8_t* p) { w[0] = *reinterpret_cast<const uint32_t*>(p); }
    __device__ __forceinline__ void store(int8_t* p) const { *reinterpret_cast<uint32_t*>(p) = w[0]; }
};
template <>
struct VecIO<16> {
    uint32_t w[4];
    __device__ __forceinline__ void load(const int8_t* p) {
        const v4i x = *reinterpret_cast<const v4i*>(p);
#pragma unroll
        for (int q = 0; q < 4; ++q) w[q] = (uint32_t)x[q];
    }
    __device__ __forceinline__ void store(int8_t* p) const {
        v4i o;
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = (int)w[q];
        *reinterpret_cast<v4i*>(p) = o;
    }
};

// Windows of a size known at compile time (2x2, 3x3): every tap is loaded -- from a clamped address when it falls
// outside the image -- so all loads of a thread are in flight together.  With run-time loop bounds they would be
// issued one at a time and the kernel would be bound by memory latency.
template <int PACK, int VB, int MODE, int FH, int FW>
__global__ __launch_bounds__(256) void pooling_static_kernel(PoolArgs a) {
    constexpr int UPP = PACK / VB;
    constexpr int W = VB / 4;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t u = blockIdx.x * blockDim.x + threadIdx.x; u < a.units; u += stride) {
        const uint32_t sub = UPP == 1 ? 0 : u % UPP, pix = UPP == 1 ? u : u / UPP;
        const uint32_t t = fdiv(pix, a.div_ow), ow = pix - t * a.OW;
        const uint32_t plane = fdiv(t, a.div_oh), oh = t - plane * a.OH;
        const int ih0 = (int)oh * a.sh - a.ph, iw0 = (int)ow * a.sw - a.pw;
        const int8_t* base = a.src + ((size_t)plane * a.IH * a.IW) * PACK + sub * VB;
        VecIO<VB> x[FH][FW];
        // row and column offsets once per window; a coordinate outside the image is clamped into it.  For MAX that is
        // all: the window meets the image, so the clamped tap is another tap of the same window.  The sums replace
        // such a tap by zero
        int roff[FH], coff[FW];
        bool rok[FH], cok[FW];
#pragma unroll
        for (int fh = 0; fh < FH; ++fh) {
            const int ih = ih0 + fh;
            rok[fh] = (unsigned)ih < (unsigned)a.IH;
            roff[fh] = (ih < 0 ? 0 : ih >= a.IH ? a.IH - 1 : ih) * a.IW * PACK;
        }
#pragma unroll
        for (int fw = 0; fw < FW; ++fw) {
            const int iw = iw0 + fw;
            cok[fw] = (unsigned)iw < (unsigned)a.IW;
            coff[fw] = (iw < 0 ? 0 : iw >= a.IW ? a.IW - 1 : iw) * PACK;
        }
        int inside = 0;
#pragma unroll
        for (int fh = 0; fh < FH; ++fh)
#pragma unroll
            for (int fw = 0; fw < FW; ++fw) {
                x[fh][fw].load(base + (uint32_t)(roff[fh] + coff[fw]));
                if (MODE != POOL_MAX) {
                    const bool ok = rok[fh] && cok[fw];
                    inside += ok;
                    if (!ok) {
#pragma unroll
                        for (int q = 0; q < W; ++q) x[fh][fw].w[q] = 0u;
                    }
                }
            }
        VecIO<VB> o;
        if (MODE == POOL_MAX) {
            Max4 acc[W];
#pragma unroll
            for (int q = 0; q < W; ++q) acc[q].init();
#pragma unroll
            for (int fh = 0; fh < FH; ++fh)
#pragma unroll
                for (int fw = 0; fw < FW; ++fw)
#pragma unroll
                    for (int q = 0; q < W; ++q) acc[q].feed(x[fh][fw].w[q]);
#pragma unroll
            for (int q = 0; q < W; ++q) o.w[q] = acc[q].get();
        } else {
            Sum4 acc[W];
#pragma unroll
            for (int q = 0; q < W; ++q) acc[q].init();
#pragma unroll
            for (int fh = 0; fh < FH; ++fh)
#pragma unroll
                for (int fw = 0; fw < FW; ++fw)
#pragma unroll
                    for (int q = 0; q < W; ++q) acc[q].feed(x[fh][fw].w[q]);
            const float count = MODE == POOL_AVG ? (float)(FH * FW) : (float)inside;
#pragma unroll
            for (int q = 0; q < W; ++q) o.w[q] = acc[q].get(count);
        }
        o.store(a.dst + (size_t)u * VB);
    }
}

// PACK = channel pack of the layout, VB = bytes per thread (PACK = 1: VB = 1; PACK = 4: VB = 4; PACK = 32: VB = 16)
template <int PACK, int VB, int MODE>
__global__ __launch_bounds__(256) void pooling_kernel(PoolArgs a) {
    constexpr int UPP = PACK / VB;  // threads per pixel
    constexpr int W = VB >= 4 ? VB / 4 : 1;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t u = blockIdx.x * blockDim.x + threadIdx.x; u < a.units; u += stride) {
        const uint32_t sub = UPP == 1 ? 0 : u % UPP, pix = UPP == 1 ? u : u / UPP;
        const uint32_t t = fdiv(pix, a.div_ow), ow = pix - t * a.OW;
        const uint32_t plane = fdiv(t, a.div_oh), oh = t - plane * a.OH;
        const int ih0 = (int)oh * a.sh - a.ph, iw0 = (int)ow * a.sw - a.pw;
        const int h_lo = ih0 < 0 ? -ih0 : 0, h_hi = ih0 + a.fh > a.IH ? a.IH - ih0 : a.fh;
        const int w_lo = iw0 < 0 ? -iw0 : 0, w_hi = iw0 + a.fw > a.IW ? a.IW - iw0 : a.fw;
        const int8_t* base = a.src + ((size_t)plane * a.IH * a.IW) * PACK + sub * VB;
        int8_t* out = a.dst + (size_t)u * VB;
        float count = (float)(a.fh * a.fw);
        if (MODE == POOL_AVG_EXCL) {
            const int nh = h_hi > h_lo ? h_hi - h_lo : 0, nw = w_hi > w_lo ? w_hi - w_lo : 0;
            count = (float)(nh * nw);
        }
        if (VB == 1) {
            int m = -128, s = 0;
            for (int fh = h_lo; fh < h_hi; ++fh)
                for (int fw = w_lo; fw < w_hi; ++fw) {
                    const int x = base[(size_t)(ih0 + fh) * a.IW + (iw0 + fw)];
                    m = x > m ? x : m;
                    s += x;
                }
            out[0] = MODE == POOL_MAX ? (int8_t)m : (int8_t)(int)roundf((float)s / count);
        } else if (MODE == POOL_MAX) {
            Max4 acc[W];
#pragma unroll
            for (int q = 0; q < W; ++q) acc[q].init();
            for (int fh = h_lo; fh < h_hi; ++fh) {
                const int8_t* row = base + ((size_t)(ih0 + fh) * a.IW + iw0) * PACK;
                for (int fw = w_lo; fw < w_hi; ++fw) {
                    if (VB == 16) {
                        const v4i x = *reinterpret_cast<const v4i*>(row + fw * PACK);
#pragma unroll
                        for (int q = 0; q < W; ++q) acc[q].feed((uint32_t)x[q]);
                    } else {
                        acc[0].feed(*reinterpret_cast<const uint32_t*>(row + fw * PACK));
                    }
                }
            }
            if (VB == 16) {
                v4i o;
#pragma unroll
                for (int q = 0; q < W; ++q) o[q] = (int)acc[q].get();
                *reinterpret_cast<v4i*>(out) = o;
            } else {
                *reinterpret_cast<uint32_t*>(out) = acc[0].get();
            }
        } else {
            Sum4 acc[W];
#pragma unroll
            for (int q = 0; q < W; ++q) acc[q].init();
            for (int fh = h_lo; fh < h_hi; ++fh) {
                const int8_t* row = base + ((size_t)(ih0 + fh) * a.IW + iw0) * PACK;
                for (int fw = w_lo; fw < w_hi; ++fw) {
                    if (VB == 16) {
                        const v4i x = *reinterpret_cast<const v4i*>(row + fw * PACK);
#pragma unroll
                        for (int q = 0; q < W; ++q) acc[q].feed((uint32_t)x[q]);
                    } else {
                        acc[0].feed(*reinterpret_cast<const uint32_t*>(row + fw * PACK));
                    }
                }
            }
            if (VB == 16) {
                v4i o;
#pragma unroll
                for (int q = 0; q < W; ++q) o[q] = (int)acc[q].get(count);
                *reinterpret_cast<v4i*>(out) = o;
            } else {
                *reinterpret_cast<uint32_t*>(out) = acc[0].get(count);
            }
        }
    }
}

template <int PACK, int VB, int FH, int FW>
void launch_static(hipStream_t st, const PoolArgs& a, int mode, unsigned blocks) {
    switch (mode) {
        case POOL_MAX:
            hipLaunchKernelGGL((pooling_static_kernel<PACK, VB, POOL_MAX, FH, FW>), dim3(blocks), dim3(256), 0, st, a);
            break;
        case POOL_AVG:
            hipLaunchKernelGGL((pooling_static_kernel<PACK, VB, POOL_AVG, FH, FW>), dim3(blocks), dim3(256), 0, st, a);
            break;
        default:
            hipLaunchKernelGGL((pooling_static_kernel<PACK, VB, POOL_AVG_EXCL, FH, FW>), dim3(blocks), dim3(256), 0, st, a);
            break;
    }
}

template <int PACK, int VB>
void launch_mode(hipStream_t st, const PoolArgs& a, int mode, unsigned blocks) {
    if constexpr (VB >= 4) {
        // the static kernels address a plane with 32-bit offsets
        if ((uint64_t)a.IH * (uint64_t)a.IW * PACK >= (1ull << 31)) goto generic;
        if (a.fh == 2 && a.fw == 2) return launch_static<PACK, VB, 2, 2>(st, a, mode, blocks);
        if (a.fh == 3 && a.fw == 3) return launch_static<PACK, VB, 3, 3>(st, a, mode, blocks);
    }
generic:
    switch (mode) {
        case POOL_MAX:
            hipLaunchKernelGGL((pooling_kernel<PACK, VB, POOL_MAX>), dim3(blocks), dim3(256), 0, st, a);
            break;
        case POOL_AVG:
            hipLaunchKernelGGL((pooling_kernel<PACK, VB, POOL_AVG>), dim3(blocks), dim3(256), 0, st, a);
            break;
        default:
            hipLaunchKernelGGL((pooling_kernel<PACK, VB, POOL_AVG_EXCL>), dim3(blocks), dim3(256), 0, st, a);
            break;
    }
}

}  // namespace

// pack: 1, 4 or 32; the caller has checked the descriptor (every window meets the image where the mode needs it,
// fewer than 2^31 output vectors)
int launch_pooling(hipStream_t st, const mi355_pooling_desc& d, int pack, uint32_t oh, uint32_t ow, const int8_t* src,
                   int8_t* dst, int cu_count) {
    PoolArgs a;
    a.src = src;
    a.dst = dst;
    a.IH = (int)d.ih; a.IW = (int)d.iw; a.OH = (int)oh; a.OW = (int)ow;
    a.ph = (int)d.pad_h; a.pw = (int)d.pad_w; a.sh = (int)d.stride_h; a.sw = (int)d.stride_w;
    a.fh = (int)d.window_h; a.fw = (int)d.window_w;
    a.div_ow = make_fastdiv(ow);
    a.div_oh = make_fastdiv(oh);
    const uint64_t pixels = (uint64_t)d.n * (d.c / (uint32_t)pack) * oh * ow;
    const uint64_t units = pack == 32 ? pixels * 2 : pixels;
    if (units == 0) return 0;
    a.units = (uint32_t)units;
    if (cu_count <= 0) cu_count = 256;
    uint64_t blocks = (units + 255) / 256;
    const uint64_t cap = (uint64_t)cu_count * 64;
    if (blocks > cap) blocks = cap;
    if (pack == 32)
        launch_mode<32, 16>(st, a, (int)d.mode, (unsigned)blocks);
    else if (pack == 4)
        launch_mode<4, 4>(st, a, (int)d.mode, (unsigned)blocks);
    else
        launch_mode<1, 1>(st, a, (int)d.mode, (unsigned)blocks);
    return (int)hipGetLastError();
}

}  // namespace mi355
