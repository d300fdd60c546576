// Stand-alone requantisation QuantizedS32 | QuantizedS8 (+ QuantizedS8) -> QuantizedS8 with the ConvBias epilogue arithmetic
// (epilogue.h): the reference's post-process pass, unary quantized ElemwiseMultiType modes and TypeCvt s32 -> s8; and
// TypeCvt between Float32 and QuantizedS8 (the quantize / dequantize at the edges of an int8 network).  Pure streaming:
// 16 bytes in (+ 4), 4 bytes out per thread step; bound by HBM (5-6 bytes per element) and by the ~10 VALU operations
// per element of the bit-exact requantisation.
#include "common.h"

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void requant_kernel(const int32_t* __restrict__ src, const int8_t* __restrict__ z,
                                                      int8_t* __restrict__ dst, uint64_t quads, uint64_t count, EpiParams e) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < quads; i += stride) {
        const v4i a = reinterpret_cast<const v4i*>(src)[i];
        const uint32_t zw = e.has_z ? reinterpret_cast<const uint32_t*>(z)[i] : 0u;
        reinterpret_cast<uint32_t*>(dst)[i] = requant4(a[0], a[1], a[2], a[3], zw, e);
    }
    // ragged tail (count % 4 elements), one thread
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        for (uint64_t j = quads * 4; j < count; ++j)
            dst[j] = (int8_t)requant_s8_exact(src[j], e.has_z != 0, e.has_z ? (int)z[j] : 0, e);
    }
}

// QuantizedS8 first operand: 16 elements per thread step (16 + 16 bytes in, 16 out; 2-3 bytes per element)
__global__ __launch_bounds__(256) void requant8_kernel(const int8_t* __restrict__ src, const int8_t* __restrict__ z,
                                                       int8_t* __restrict__ dst, uint64_t blocks16, uint64_t count, EpiParams e) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < blocks16; i += stride) {
        const v4i a = reinterpret_cast<const v4i*>(src)[i];
        v4i zv = {0, 0, 0, 0};
        if (e.has_z) zv = reinterpret_cast<const v4i*>(z)[i];
        v4i o;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int w = a[q];
            o[q] = (int)requant4((w << 24) >> 24, (w << 16) >> 24, (w << 8) >> 24, w >> 24, (uint32_t)zv[q], e);
        }
        reinterpret_cast<v4i*>(dst)[i] = o;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        for (uint64_t j = blocks16 * 16; j < count; ++j)
            dst[j] = (int8_t)requant_s8_exact((int)src[j], e.has_z != 0, e.has_z ? (int)z[j] : 0, e);
    }
}

// TypeCvt Float32 -> QuantizedS8: quantize = saturate(roundf(x / scale)), the literal divide -- the input is any float
// (infinities, NaN -> -128 through fmaxf), so the divide-free form of the epilogue has no range guarantee to stand on
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int quantize_s8(float x, float scale) {
    float v = x / scale;
    v = __builtin_roundf(v);
    v = fminf(fmaxf(-128.f, v), 127.f);
    return (int)v;
}

__global__ __launch_bounds__(256) void cvt_f32_s8_kernel(const float* __restrict__ src, int8_t* __restrict__ dst,
                                                         uint64_t quads, uint64_t count, float scale) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < quads; i += stride) {
        const v4f x = reinterpret_cast<const v4f*>(src)[i];
        reinterpret_cast<uint32_t*>(dst)[i] =
                pack4(quantize_s8(x[0], scale), quantize_s8(x[1], scale), quantize_s8(x[2], scale), quantize_s8(x[3], scale));
    }
    if (blockIdx.x == 0 && threadIdx.x == 0)
        for (uint64_t j = quads * 4; j < count; ++j) dst[j] = (int8_t)quantize_s8(src[j], scale);
}

// TypeCvt QuantizedS8 -> Float32: dequantize = float(x) * scale
__global__ __launch_bounds__(256) void cvt_s8_f32_kernel(const int8_t* __restrict__ src, float* __restrict__ dst,
                                                         uint64_t quads, uint64_t count, float scale) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < quads; i += stride) {
        const int w = reinterpret_cast<const int*>(src)[i];
        v4f o;
        o[0] = (float)((w << 24) >> 24) * scale;
        o[1] = (float)((w << 16) >> 24) * scale;
        o[2] = (float)((w << 8) >> 24) * scale;
        o[3] = (float)(w >> 24) * scale;
        reinterpret_cast<v4f*>(dst)[i] = o;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0)
        for (uint64_t j = quads * 4; j < count; ++j) dst[j] = (float)src[j] * scale;
}

unsigned stream_blocks(uint64_t steps, int cu_count) {
    if (cu_count <= 0) cu_count = 256;
    uint64_t blocks = (steps + 255) / 256;
    const uint64_t cap = (uint64_t)cu_count * 16;
    if (blocks > cap) blocks = cap;
    return blocks ? (unsigned)blocks : 1u;
}

}  // namespace

int launch_cvt_f32_s8(hipStream_t st, float scale, const float* src, int8_t* dst, uint64_t count, int cu_count) {
    if (count == 0) return 0;
    hipLaunchKernelGGL(cvt_f32_s8_kernel, dim3(stream_blocks(count / 4, cu_count)), dim3(256), 0, st, src, dst, count / 4,
                       count, scale);
    return (int)hipGetLastError();
}

int launch_cvt_s8_f32(hipStream_t st, float scale, const int8_t* src, float* dst, uint64_t count, int cu_count) {
    if (count == 0) return 0;
    hipLaunchKernelGGL(cvt_s8_f32_kernel, dim3(stream_blocks(count / 4, cu_count)), dim3(256), 0, st, src, dst, count / 4,
                       count, scale);
    return (int)hipGetLastError();
}

int launch_requant8(hipStream_t st, const EpiParams& e, const int8_t* src, const int8_t* z, int8_t* dst, uint64_t count,
                    int cu_count) {
    if (count == 0) return 0;
    const uint64_t blocks16 = count / 16;
    if (cu_count <= 0) cu_count = 256;
    uint64_t blocks = (blocks16 + 255) / 256;
    const uint64_t cap = (uint64_t)cu_count * 16;
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(requant8_kernel, dim3((unsigned)blocks), dim3(256), 0, st, src, z, dst, blocks16, count, e);
    return (int)hipGetLastError();
}

int launch_requant(hipStream_t st, const EpiParams& e, const int32_t* src, const int8_t* z, int8_t* dst, uint64_t count,
                   int cu_count) {
    if (count == 0) return 0;
    const uint64_t quads = count / 4;
    if (cu_count <= 0) cu_count = 256;
    uint64_t blocks = (quads + 255) / 256;
    const uint64_t cap = (uint64_t)cu_count * 16;
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(requant_kernel, dim3((unsigned)blocks), dim3(256), 0, st, src, z, dst, quads, count, e);
    return (int)hipGetLastError();
}

// ---- streaming probe: what a launch that only moves bytes costs on this device ----------------------------------
namespace {
typedef uint32_t u32x4p __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void stream_probe_kernel(const u32x4p* __restrict__ in, u32x4p* __restrict__ out, uint64_t nr,
                                                           uint64_t nw) {
    const uint64_t stride = (uint64_t)gridDim.x * 256;
    const uint64_t n = nr > nw ? nr : nw;
    u32x4p x = {0, 0, 0, 0};
    for (uint64_t u = (uint64_t)blockIdx.x * 256 + threadIdx.x; u < n; u += stride) {
        if (u < nr) x ^= __builtin_nontemporal_load(in + u);  // reads beyond the writes are folded in, so they stay
        if (u < nw) out[u] = x;
    }
    // keeps the reads beyond the last write alive (the host never launches a probe that reads without a byte to write)
    if (x[0] == 0x12345u && x[1] == 0x777u && x[2] == 0xabcu) out[0] = x;
}
}  // namespace

int launch_stream_probe(hipStream_t st, const void* src, uint64_t read_bytes, void* dst, uint64_t write_bytes, int cu_count) {
    const uint64_t nr = read_bytes / 16, nw = write_bytes / 16;
    if (nr == 0 && nw == 0) return 0;
    if (cu_count <= 0) cu_count = 256;
    const uint64_t units = nr > nw ? nr : nw;
    uint64_t blocks = (units + 255) / 256;
    if (blocks > (uint64_t)cu_count * 8) blocks = (uint64_t)cu_count * 8;
    hipLaunchKernelGGL(stream_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, st, reinterpret_cast<const u32x4p*>(src),
                       reinterpret_cast<u32x4p*>(dst), nr, nw);
    return (int)hipGetLastError();
}

}  // namespace mi355
