// RelayoutFormat kernels: NCHW <-> NCHW4 / NCHW32, NCHW4 <-> NCHW32, conv weight packing.
// Semantics: naive::RelayoutFormatImpl::exec (dnn/src/naive/relayout_format/opr_impl.cpp:486-773):
// zero-filled destination, permuted copy, per-group channel padding, optional crop on the way
// back, and for QuantizedS8 -> QuantizedS8 with different scales quantize(dequantize(x)).
//
// Two tiers:
//   * relayout_generic_kernel: one thread per destination element, any mode / element size.
//   * byte-transposing fast kernels for the int8 pure-permutation cases the conv path uses;
//     all global traffic is 16-byte vectors, fully coalesced on both sides (HBM bound).
#include "common.h"

namespace mi355 {
namespace {

struct RelayoutArgs {
    const void* src;
    void* dst;
    uint32_t mode;
    uint32_t s[7];   // src shape
    uint32_t o[7];   // dst shape
    uint32_t group;
    uint32_t elem_bytes;
    int requant;
    float s_src, s_dst;
    int64_t total;   // dst elements
};

__device__ __forceinline__ int8_t requant_s8(int8_t v, float ss, float sd) {
    float x = (float)v * ss;
    float q = x / sd;
    q = __builtin_roundf(q);
    q = fminf(fmaxf(-128.f, q), 127.f);
    return (int8_t)q;
}

__global__ __launch_bounds__(256) void relayout_generic_kernel(RelayoutArgs a) {
    int64_t di = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (di >= a.total) return;
    int64_t si = -1;
    const uint32_t g = a.group;
    switch (a.mode) {
        case MI355_RL_NCHW_NCHW4_IC_SMALL:
        case MI355_RL_NCHW_NCHW4:
        case MI355_RL_NCHW_NCHW32: {
            const int64_t p = a.o[4], C = a.s[1], H = a.s[2], W = a.s[3], CB = a.o[1];
            const int64_t gg = a.mode == MI355_RL_NCHW_NCHW4_IC_SMALL ? 1 : g;
            const int64_t icpg = C / gg, cpb = CB / gg;
            int64_t t = di;
            int64_t k = t % p; t /= p;
            int64_t w = t % W; t /= W;
            int64_t h = t % H; t /= H;
            int64_t cbg = t % CB;
            int64_t n = t / CB;
            int64_t gi = cbg / cpb, cb = cbg % cpb;
            int64_t cin = cb * p + k;
            if (cin < icpg) si = ((n * C + gi * icpg + cin) * H + h) * W + w;
            break;
        }
        case MI355_RL_NCHW4_NCHW:
        case MI355_RL_NCHW32_NCHW: {
            const int64_t p = a.s[4], CB = a.s[1], H = a.s[2], W = a.s[3], C = a.o[1];
            const int64_t ocpg = C / g, cpb = CB / g;
            int64_t t = di;
            int64_t w = t % W; t /= W;
            int64_t h = t % H; t /= H;
            int64_t c = t % C;
            int64_t n = t / C;
            int64_t gi = c / ocpg, ci = c % ocpg;
            int64_t pc = gi * cpb * p + ci;
            si = (((n * CB + pc / p) * H + h) * W + w) * p + pc % p;
            break;
        }
        case MI355_RL_NCHW_NCHW4_WEIGHT: {
            const int grp = a.o[5] ? 1 : 0;  // 6-dim dst => group
            const int64_t OC = a.s[grp], IC = a.s[grp + 1], FH = a.s[grp + 2], FW = a.s[grp + 3];
            const int64_t OCp = a.o[grp], ICb = a.o[grp + 1];
            int64_t t = di;
            int64_t k = t % 4; t /= 4;
            int64_t fw = t % FW; t /= FW;
            int64_t fh = t % FH; t /= FH;
            int64_t ib = t % ICb; t /= ICb;
            int64_t oc = t % OCp;
            int64_t gi = t / OCp;
            int64_t ic = ib * 4 + k;
            if (oc < OC && ic < IC) si = (((gi * OC + oc) * IC + ic) * FH + fh) * FW + fw;
            break;
        }
        case MI355_RL_NCHW4_NCHW32:
        case MI355_RL_NCHW32_NCHW4: {
            const int64_t ps = a.s[4], pd = a.o[4], H = a.s[2], W = a.s[3], C = (int64_t)a.s[1] * ps;
            int64_t t = di;
            int64_t k = t % pd; t /= pd;
            int64_t w = t % W; t /= W;
            int64_t h = t % H; t /= H;
            int64_t cb = t % (C / pd);
            int64_t n = t / (C / pd);
            int64_t c = cb * pd + k;
            si = (((n * (C / ps) + c / ps) * H + h) * W + w) * ps + c % ps;
            break;
        }
        default:
            break;
    }
    if (a.elem_bytes == 4) {
        reinterpret_cast<int32_t*>(a.dst)[di] = si < 0 ? 0 : reinterpret_cast<const int32_t*>(a.src)[si];
    } else {
        int8_t v = si < 0 ? (int8_t)0 : reinterpret_cast<const int8_t*>(a.src)[si];
        if (a.requant) v = requant_s8(v, a.s_src, a.s_dst);
        reinterpret_cast<int8_t*>(a.dst)[di] = v;
    }
}

// ---- 4x4 byte transpose in registers: rows r0..r3 (4 bytes each) -> columns ----
__device__ __forceinline__ void transpose4x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t& c0,
                                             uint32_t& c1, uint32_t& c2, uint32_t& c3) {
    // t01_lo = r0.b0 r1.b0 r0.b1 r1.b1 ; t01_hi = r0.b2 r1.b2 r0.b3 r1.b3
    uint32_t t01_lo = __builtin_amdgcn_perm(r1, r0, 0x05010400u);
    uint32_t t01_hi = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    uint32_t t23_lo = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
    uint32_t t23_hi = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    c0 = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x05040100u);
    c1 = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x07060302u);
    c2 = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x05040100u);
    c3 = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x07060302u);
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// NCHW -> NCHW4, int8, C % 4 == 0, HW % 16 == 0.  Thread: 4 channels x 16 pixels.
// grid.x covers (C/4) * (HW/16) work items per image, grid.y = N.
__global__ __launch_bounds__(256) void nchw_to_nchw4_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst,
                                                            uint32_t C, uint32_t HW) {
    const uint32_t pq = HW / 16;
    const uint32_t items = (C / 4) * pq;
    uint32_t it = blockIdx.x * 256 + threadIdx.x;
    if (it >= items) return;
    const uint32_t cg = it / pq, pb = it % pq;
    const int64_t img = (int64_t)blockIdx.y * C * HW;
    const int8_t* s = src + img + (int64_t)cg * 4 * HW + pb * 16;
    u32x4 r0 = *reinterpret_cast<const u32x4*>(s);
    u32x4 r1 = *reinterpret_cast<const u32x4*>(s + HW);
    u32x4 r2 = *reinterpret_cast<const u32x4*>(s + 2 * (int64_t)HW);
    u32x4 r3 = *reinterpret_cast<const u32x4*>(s + 3 * (int64_t)HW);
    int8_t* d = dst + img + ((int64_t)cg * HW + pb * 16) * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        u32x4 o;
        uint32_t c0, c1, c2, c3;
        transpose4x4(r0[j], r1[j], r2[j], r3[j], c0, c1, c2, c3);
        o[0] = c0; o[1] = c1; o[2] = c2; o[3] = c3;
        *reinterpret_cast<u32x4*>(d + j * 16) = o;
    }
}

// NCHW4 -> NCHW, int8, same constraints.
__global__ __launch_bounds__(256) void nchw4_to_nchw_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst,
                                                            uint32_t C, uint32_t HW) {
    const uint32_t pq = HW / 16;
    const uint32_t items = (C / 4) * pq;
    uint32_t it = blockIdx.x * 256 + threadIdx.x;
    if (it >= items) return;
    const uint32_t cg = it / pq, pb = it % pq;
    const int64_t img = (int64_t)blockIdx.y * C * HW;
    const int8_t* s = src + img + ((int64_t)cg * HW + pb * 16) * 4;
    u32x4 o0, o1, o2, o3;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        u32x4 v = *reinterpret_cast<const u32x4*>(s + j * 16);  // 4 pixels x 4 channels
        uint32_t c0, c1, c2, c3;
        transpose4x4(v[0], v[1], v[2], v[3], c0, c1, c2, c3);
        o0[j] = c0; o1[j] = c1; o2[j] = c2; o3[j] = c3;
    }
    int8_t* d = dst + img + (int64_t)cg * 4 * HW + pb * 16;
    *reinterpret_cast<u32x4*>(d) = o0;
    *reinterpret_cast<u32x4*>(d + HW) = o1;
    *reinterpret_cast<u32x4*>(d + 2 * (int64_t)HW) = o2;
    *reinterpret_cast<u32x4*>(d + 3 * (int64_t)HW) = o3;
}

// NCHW <-> NCHW32 through LDS.  Tile = 32 channels x 512 pixels (16 KiB).  The LDS image keeps
// the NCHW order (channel rows of 512 bytes, padded to 520 so that rows c and c+16 are 32 banks
// apart); global accesses on both sides are 16-byte vectors over contiguous runs.
constexpr int RL_TP = 512;           // pixels per tile
constexpr int RL_ROW = RL_TP + 8;    // padded channel row (bytes): 16 rows = 8320 = 32*256 + 128

__global__ __launch_bounds__(256) void nchw_to_nchw32_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst,
                                                             uint32_t CB, uint32_t HW) {
    __shared__ __attribute__((aligned(16))) int8_t sm[32 * RL_ROW];
    const uint32_t t = threadIdx.x;
    const uint32_t ptiles = (HW + RL_TP - 1) / RL_TP;
    const uint32_t cb = blockIdx.x / ptiles, pt = blockIdx.x % ptiles;
    const uint32_t p0 = pt * RL_TP;
    const int64_t img = (int64_t)blockIdx.y * CB * 32 * HW;
    // load: 32 rows x 32 vectors; thread t -> vector (t % 32), rows t/32 + 8*i
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t row = t / 32 + 8 * i, v = t % 32;
        uint32_t px = p0 + v * 16;
        u32x4 x = {0, 0, 0, 0};
        if (px < HW) x = *reinterpret_cast<const u32x4*>(src + img + ((int64_t)cb * 32 + row) * HW + px);
        *reinterpret_cast<u32x4*>(sm + row * RL_ROW + v * 16) = x;
    }
    __syncthreads();
    // item: pixel quad pq = t / 2 (4 pixels), half = t % 2 (16 channels)
    const uint32_t pq = t >> 1, half = t & 1;
    uint32_t rows[16];
#pragma unroll
    for (int k = 0; k < 16; ++k)
        rows[k] = *reinterpret_cast<const uint32_t*>(sm + (half * 16 + k) * RL_ROW + pq * 4);
    u32x4 out[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t c0, c1, c2, c3;
        transpose4x4(rows[4 * q], rows[4 * q + 1], rows[4 * q + 2], rows[4 * q + 3], c0, c1, c2, c3);
        out[0][q] = c0; out[1][q] = c1; out[2][q] = c2; out[3][q] = c3;
    }
    const uint32_t px = p0 + pq * 4;
    if (px < HW) {
        int8_t* d = dst + img + ((int64_t)cb * HW + px) * 32 + half * 16;
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(d + i * 32) = out[i];
    }
}

__global__ __launch_bounds__(256) void nchw32_to_nchw_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst,
                                                             uint32_t CB, uint32_t HW) {
    __shared__ __attribute__((aligned(16))) int8_t sm[32 * RL_ROW];
    const uint32_t t = threadIdx.x;
    const uint32_t ptiles = (HW + RL_TP - 1) / RL_TP;
    const uint32_t cb = blockIdx.x / ptiles, pt = blockIdx.x % ptiles;
    const uint32_t p0 = pt * RL_TP;
    const int64_t img = (int64_t)blockIdx.y * CB * 32 * HW;
    const uint32_t pq = t >> 1, half = t & 1;
    const uint32_t px = p0 + pq * 4;
    u32x4 in[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        in[i] = u32x4{0, 0, 0, 0};
        if (px < HW) in[i] = *reinterpret_cast<const u32x4*>(src + img + ((int64_t)cb * HW + px + i) * 32 + half * 16);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t c0, c1, c2, c3;
        // rows = pixels, bytes = channels 4q..4q+3  ->  columns = channels, bytes = pixels
        transpose4x4(in[0][q], in[1][q], in[2][q], in[3][q], c0, c1, c2, c3);
        uint32_t base = (half * 16 + 4 * q) * RL_ROW + pq * 4;
        *reinterpret_cast<uint32_t*>(sm + base) = c0;
        *reinterpret_cast<uint32_t*>(sm + base + RL_ROW) = c1;
        *reinterpret_cast<uint32_t*>(sm + base + 2 * RL_ROW) = c2;
        *reinterpret_cast<uint32_t*>(sm + base + 3 * RL_ROW) = c3;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t row = t / 32 + 8 * i, v = t % 32;
        uint32_t p = p0 + v * 16;
        if (p < HW) {
            u32x4 x = *reinterpret_cast<const u32x4*>(sm + row * RL_ROW + v * 16);
            *reinterpret_cast<u32x4*>(dst + img + ((int64_t)cb * 32 + row) * HW + p) = x;
        }
    }
}

}  // namespace

int launch_relayout(hipStream_t st, const mi355_relayout_desc& d, const uint32_t* oshape, uint32_t ondim,
                    const void* src, void* dst, bool allow_fast) {
    int64_t total = 1;
    for (uint32_t i = 0; i < ondim; ++i) total *= oshape[i];
    if (total == 0) return 0;
    const bool requant = d.elem_bytes == 1 && d.scale_src != d.scale_dst;
    const uint32_t g = d.group ? d.group : 1;
    // fast byte-permutation paths
    if (allow_fast && d.elem_bytes == 1 && !requant && g == 1 && d.shape[0] <= 65535) {
        const uint32_t N = d.shape[0];
        if (d.mode == MI355_RL_NCHW_NCHW4 || d.mode == MI355_RL_NCHW_NCHW32) {
            const uint32_t C = d.shape[1], HW = d.shape[2] * d.shape[3];
            const uint32_t p = d.mode == MI355_RL_NCHW_NCHW4 ? 4 : 32;
            if (C % p == 0 && HW % 16 == 0 && (uint64_t)C * HW < (1ull << 31)) {
                if (p == 4) {
                    uint32_t items = (C / 4) * (HW / 16);
                    hipLaunchKernelGGL(nchw_to_nchw4_kernel, dim3((items + 255) / 256, N), dim3(256), 0, st,
                                       (const int8_t*)src, (int8_t*)dst, C, HW);
                } else {
                    uint32_t ptiles = (HW + RL_TP - 1) / RL_TP;
                    hipLaunchKernelGGL(nchw_to_nchw32_kernel, dim3((C / 32) * ptiles, N), dim3(256), 0, st,
                                       (const int8_t*)src, (int8_t*)dst, C / 32, HW);
                }
                return (int)hipGetLastError();
            }
        } else if ((d.mode == MI355_RL_NCHW4_NCHW || d.mode == MI355_RL_NCHW32_NCHW) &&
                   (d.oc == 0 || d.oc == d.shape[1] * d.shape[4])) {
            const uint32_t p = d.shape[4], C = d.shape[1] * p, HW = d.shape[2] * d.shape[3];
            if (HW % 16 == 0 && (uint64_t)C * HW < (1ull << 31)) {
                if (p == 4) {
                    uint32_t items = (C / 4) * (HW / 16);
                    hipLaunchKernelGGL(nchw4_to_nchw_kernel, dim3((items + 255) / 256, N), dim3(256), 0, st,
                                       (const int8_t*)src, (int8_t*)dst, C, HW);
                } else {
                    uint32_t ptiles = (HW + RL_TP - 1) / RL_TP;
                    hipLaunchKernelGGL(nchw32_to_nchw_kernel, dim3((C / 32) * ptiles, N), dim3(256), 0, st,
                                       (const int8_t*)src, (int8_t*)dst, C / 32, HW);
                }
                return (int)hipGetLastError();
            }
        }
    }
    RelayoutArgs a;
    a.src = src; a.dst = dst; a.mode = d.mode;
    for (int i = 0; i < 7; ++i) {
        a.s[i] = i < (int)d.ndim ? d.shape[i] : 0;
        a.o[i] = i < (int)ondim ? oshape[i] : 0;
    }
    a.group = g;
    a.elem_bytes = d.elem_bytes;
    a.requant = requant ? 1 : 0;
    a.s_src = d.scale_src; a.s_dst = d.scale_dst;
    a.total = total;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffff) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(relayout_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, a);
    return (int)hipGetLastError();
}

}  // namespace mi355
