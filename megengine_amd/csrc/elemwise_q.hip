// ElemwiseMultiType quantized modes with one to three inputs (dnn/src/naive/elemwise_multi_type/opr_impl_3.cpp:11-60,
// opr_impl_4.cpp:11-66, opr_impl_5.cpp:11-45): per element, dequantize every input with its own scale, run the mode's
// float kernel (dnn/src/common/elemwise/kern_defs.cuh:166-313), quantize with dst's scale.  Streaming: four elements
// per thread step, 4- or 16-byte accesses; 2-13 bytes per element, bound by HBM.
//
// Every operation below is one individually rounded IEEE binary32 operation (the file is compiled without contraction
// and with the correctly rounded divide), in the order the reference's expressions evaluate them, so the bits of the
// result are defined; FUSE_MUL_ADD3 is a multiply followed by an add, as the reference's x86 build without FMA code
// generation computes it.  min and max are the reference's std::min / std::max: max(a, b) = a < b ? b : a.
#include "common.h"

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float std_max(float a, float b) { return a < b ? b : a; }
__device__ __forceinline__ float std_min(float a, float b) { return b < a ? b : a; }
__device__ __forceinline__ float hswish(float x) { return x * std_min(std_max(x + 3.f, 0.f), 6.f) * (1.f / 6.f); }

__device__ __forceinline__ float ew_apply(uint32_t mode, float x, float y, float z) {
    switch (mode) {
        case MI355_EW_RELU: return x <= 0.f ? 0.f : x;
        case MI355_EW_ABS: return __builtin_fabsf(x);
        case MI355_EW_CEIL: return __builtin_ceilf(x);
        case MI355_EW_FLOOR: return __builtin_floorf(x);
        case MI355_EW_NEGATE: return -x;
        case MI355_EW_ROUND: return __builtin_roundf(x);
        case MI355_EW_FAST_TANH: return x * (27.f + x * x) / (27.f + 9.f * x * x);
        case MI355_EW_H_SWISH: return hswish(x);
        case MI355_EW_ABS_GRAD: return x > 0.f ? y : -y;
        case MI355_EW_ADD: return x + y;
        case MI355_EW_FLOOR_DIV: return __builtin_floorf(x / y);
        case MI355_EW_MAX: return x > y ? x : y;
        case MI355_EW_MIN: return x < y ? x : y;
        case MI355_EW_MUL: return x * y;
        case MI355_EW_SIGMOID_GRAD: return x * (1.f - x) * y;
        case MI355_EW_SUB: return x - y;
        case MI355_EW_SWITCH_GT0: return x > 0.f ? y : 0.f;
        case MI355_EW_TANH_GRAD: return (1.f - x * x) * y;
        case MI355_EW_TRUE_DIV: return x / y;
        case MI355_EW_LT: return x < y ? 1.f : 0.f;
        case MI355_EW_LEQ: return x <= y ? 1.f : 0.f;
        case MI355_EW_EQ: return x == y ? 1.f : 0.f;
        case MI355_EW_FUSE_ADD_RELU: return (x + y) <= 0.f ? 0.f : (x + y);
        case MI355_EW_FAST_TANH_GRAD: {
            const float x2 = x * x, deno = 3.f + x2;
            return ((-48.f * x2) / deno + 27.f + x2) / (deno * 9.f) * y;
        }
        case MI355_EW_H_SWISH_GRAD: return x < -3.f ? 0.f : (x > 3.f ? y : (2.f * x + 3.f) / 6.f * y);
        case MI355_EW_FUSE_ADD_H_SWISH: return hswish(x + y);
        case MI355_EW_COND_LEQ_MOV: return x <= y ? z : 0.f;
        case MI355_EW_COND_LT_MOV: return x < y ? z : 0.f;
        case MI355_EW_FUSE_MUL_ADD3: return x * y + z;
        default: return 0.f;
    }
}

// DTypeParamImpl<dt_qint8>::quantize / <dt_qint32>::quantize (dnn/include/megdnn/dtype.h:845-853, :887-896); fmaxf drops
// a NaN, as the reference's fmax does
template <bool DST32>
__device__ __forceinline__ int ew_quantize(float r, float scale) {
    float v = r / scale;
    v = __builtin_roundf(v);
    if (DST32) return (int)fminf(fmaxf(-2147483648.f, v), 2147483520.f);
    return (int)fminf(fmaxf(-128.f, v), 127.f);
}

struct EwArgs {
    const void* src[3];
    void* dst;
    float scale[3];
    float scale_dst;
    uint64_t quads, count;
    uint32_t mode;
};

template <bool SRC32>
__device__ __forceinline__ void ew_load4(const void* p, uint64_t i, int (&v)[4]) {
    if (SRC32) {
        const v4i a = reinterpret_cast<const v4i*>(p)[i];
        v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3];
    } else {
        const int w = reinterpret_cast<const int*>(p)[i];
        v[0] = (w << 24) >> 24; v[1] = (w << 16) >> 24; v[2] = (w << 8) >> 24; v[3] = w >> 24;
    }
}

template <bool SRC32>
__device__ __forceinline__ int ew_load1(const void* p, uint64_t j) {
    return SRC32 ? reinterpret_cast<const int32_t*>(p)[j] : (int)reinterpret_cast<const int8_t*>(p)[j];
}

template <int ARITY, bool SRC32, bool DST32>
__global__ __launch_bounds__(256) void elemwise_q_kernel(EwArgs a) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.quads; i += stride) {
        int v[3][4] = {};
#pragma unroll
        for (int s = 0; s < ARITY; ++s) ew_load4<SRC32>(a.src[s], i, v[s]);
        int q[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float x = (float)v[0][e] * a.scale[0];
            const float y = ARITY > 1 ? (float)v[1][e] * a.scale[1] : 0.f;
            const float z = ARITY > 2 ? (float)v[2][e] * a.scale[2] : 0.f;
            q[e] = ew_quantize<DST32>(ew_apply(a.mode, x, y, z), a.scale_dst);
        }
        if (DST32)
            reinterpret_cast<v4i*>(a.dst)[i] = v4i{q[0], q[1], q[2], q[3]};
        else
            reinterpret_cast<uint32_t*>(a.dst)[i] =
                    (uint32_t)(q[0] & 255) | ((uint32_t)(q[1] & 255) << 8) | ((uint32_t)(q[2] & 255) << 16) | ((uint32_t)q[3] << 24);
    }
    // ragged tail (count % 4 elements), one thread
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        for (uint64_t j = a.quads * 4; j < a.count; ++j) {
            const float x = (float)ew_load1<SRC32>(a.src[0], j) * a.scale[0];
            const float y = ARITY > 1 ? (float)ew_load1<SRC32>(a.src[1], j) * a.scale[1] : 0.f;
            const float z = ARITY > 2 ? (float)ew_load1<SRC32>(a.src[2], j) * a.scale[2] : 0.f;
            const int q = ew_quantize<DST32>(ew_apply(a.mode, x, y, z), a.scale_dst);
            if (DST32)
                reinterpret_cast<int32_t*>(a.dst)[j] = q;
            else
                reinterpret_cast<int8_t*>(a.dst)[j] = (int8_t)q;
        }
    }
}

template <int ARITY>
int launch_arity(hipStream_t st, const EwArgs& a, bool src32, bool dst32, unsigned blocks) {
    if (src32) {
        if (dst32) hipLaunchKernelGGL((elemwise_q_kernel<ARITY, true, true>), dim3(blocks), dim3(256), 0, st, a);
        else hipLaunchKernelGGL((elemwise_q_kernel<ARITY, true, false>), dim3(blocks), dim3(256), 0, st, a);
    } else {
        if (dst32) hipLaunchKernelGGL((elemwise_q_kernel<ARITY, false, true>), dim3(blocks), dim3(256), 0, st, a);
        else hipLaunchKernelGGL((elemwise_q_kernel<ARITY, false, false>), dim3(blocks), dim3(256), 0, st, a);
    }
    return (int)hipGetLastError();
}

}  // namespace

// number of inputs of a served mode, 0 for a mode that is not served
int elemwise_q_arity(uint32_t mode) {
    switch (mode) {
        case MI355_EW_RELU: case MI355_EW_ABS: case MI355_EW_CEIL: case MI355_EW_FLOOR: case MI355_EW_NEGATE:
        case MI355_EW_ROUND: case MI355_EW_FAST_TANH: case MI355_EW_H_SWISH:
            return 1;
        case MI355_EW_ABS_GRAD: case MI355_EW_ADD: case MI355_EW_FLOOR_DIV: case MI355_EW_MAX: case MI355_EW_MIN:
        case MI355_EW_MUL: case MI355_EW_SIGMOID_GRAD: case MI355_EW_SUB: case MI355_EW_SWITCH_GT0:
        case MI355_EW_TANH_GRAD: case MI355_EW_TRUE_DIV: case MI355_EW_LT: case MI355_EW_LEQ: case MI355_EW_EQ:
        case MI355_EW_FUSE_ADD_RELU: case MI355_EW_FAST_TANH_GRAD: case MI355_EW_H_SWISH_GRAD:
        case MI355_EW_FUSE_ADD_H_SWISH:
            return 2;
        case MI355_EW_COND_LEQ_MOV: case MI355_EW_COND_LT_MOV: case MI355_EW_FUSE_MUL_ADD3:
            return 3;
        default:
            return 0;
    }
}

int launch_elemwise_q(hipStream_t st, const mi355_elemwise_desc& d, const void* s0, const void* s1, const void* s2, void* dst,
                      int cu_count) {
    if (d.count == 0) return 0;
    EwArgs a;
    a.src[0] = s0; a.src[1] = s1; a.src[2] = s2;
    a.dst = dst;
    for (int i = 0; i < 3; ++i) a.scale[i] = d.scale_src[i];
    a.scale_dst = d.scale_dst;
    a.quads = d.count / 4;
    a.count = d.count;
    a.mode = d.mode;
    if (cu_count <= 0) cu_count = 256;
    uint64_t blocks = (a.quads + 255) / 256;
    const uint64_t cap = (uint64_t)cu_count * 16;
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    const bool src32 = d.src_dtype == MI355_DT_QS32, dst32 = d.dst_dtype == MI355_DT_QS32;
    switch (d.arity) {
        case 1: return launch_arity<1>(st, a, src32, dst32, (unsigned)blocks);
        case 2: return launch_arity<2>(st, a, src32, dst32, (unsigned)blocks);
        case 3: return launch_arity<3>(st, a, src32, dst32, (unsigned)blocks);
        default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace mi355
