// Plain-NCHW int8 ConvBias on the MFMA kernels: algorithm MI355_NCHW_RELAYOUT_MFMA_I8.
//
// Format::NCHW is what the reference's own x86 int8 algorithms accept (dnn/src/x86/conv_bias/int8/
// algo_usable_preferred.cpp:19-37,88-108; shape rule dnn/src/common/convolution.cpp:774-801), and the CUDA backend runs
// it the same way this file does: relayout into the packed format of its tensor-core kernels, convolve, relayout back
// (dnn/src/cuda/conv_bias/conv_nchwqs8.cpp).  All intermediates live in the caller's workspace -- the first algorithm
// of this backend that reports a non-zero get_workspace_in_bytes (dnn/include/megdnn/oprs/nn.h:419-422):
//
//     [src as NCHW32, channels padded to 32][filter as (OC32, IC32/32, FH, FW, 32)][dst as NCHW32][z as NCHW32][bias, OC32]
//
// Padded input channels are zero bytes (they add nothing to a sum); padded output channels have zero filter rows and
// zero bias and are cropped by the relayout back.  The arithmetic is that of the NCHW32 kernel, which is bit-exact to
// the reference's naive path; a permutation of the operands changes no integer sum.
#include <string.h>

#include "igemm_shared.h"

namespace mi355 {
namespace {

constexpr size_t kAlign = 256;
size_t up(size_t x) { return (x + kAlign - 1) / kAlign * kAlign; }
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }  // the vector paths of the relayouts

struct NchwLayout {
    uint32_t ic32, oc32;                              // channel counts padded to whole blocks of 32
    size_t off_src, off_flt, off_dst, off_z, off_bias, total;
    ConvProblem inner;                                // the NCHW32 problem the MFMA kernel runs
};

// 16 bytes per thread
__global__ __launch_bounds__(256) void zero_fill_kernel(v4i* dst, uint64_t vecs) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < vecs) dst[i] = v4i{0, 0, 0, 0};
}

__global__ __launch_bounds__(256) void bias_pad_kernel(const int32_t* src, int32_t* dst, uint32_t oc, uint32_t oc32) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < oc32) dst[i] = i < oc ? src[i] : 0;
}

bool make_layout(const ConvProblem& p, NchwLayout* L) {
    const mi355_conv_desc& d = p.d;
    if (d.format != MI355_FMT_NCHW || p.dw4) return false;
    if (d.dst_dtype != MI355_DT_QS8 || d.bias_mode == MI355_BIAS_FULL || !p.epi.fast) return false;
    if (d.mode != MI355_MODE_CROSS_CORRELATION || d.dilate_h != 1 || d.dilate_w != 1) return false;
    // groups must be whole channel blocks on both sides: then the packed tensors of the groups are contiguous pieces of
    // the packed tensors, as the NCHW32 group kernel expects them
    if (d.group != 1 && (p.icpg % 32 || p.ocpg % 32)) return false;
    // dense batches only (a strided view would need strided relayouts)
    const int64_t src_img = (int64_t)d.ic * d.ih * d.iw, dst_img = (int64_t)d.oc * p.oh * p.ow;
    if (p.src_sn != src_img || p.dst_sn != dst_img || (d.has_z && p.z_sn != dst_img)) return false;
    if (d.n > 65535) return false;
    L->ic32 = (d.ic + 31) / 32 * 32;
    L->oc32 = (d.oc + 31) / 32 * 32;
    const size_t src_b = (size_t)d.n * L->ic32 * d.ih * d.iw, flt_b = (size_t)L->oc32 * (L->ic32 / d.group) * d.fh * d.fw;
    const size_t dst_b = (size_t)d.n * L->oc32 * p.oh * p.ow;
    size_t o = 0;
    L->off_src = o; o += up(src_b);
    L->off_flt = o; o += up(flt_b);
    L->off_dst = o; o += up(dst_b);
    L->off_z = o; o += d.has_z ? up(dst_b) : 0;
    L->off_bias = o; o += d.bias_mode == MI355_BIAS_BROADCAST_CHANNEL && L->oc32 != d.oc ? up((size_t)L->oc32 * 4) : 0;
    L->total = o;
    ConvProblem& q = L->inner;
    q = p;
    q.d.format = MI355_FMT_NCHW32;
    q.d.ic = L->ic32;
    q.d.oc = L->oc32;
    q.d.src_stride_n = q.d.dst_stride_n = q.d.z_stride_n = 0;
    q.icpg = L->ic32 / d.group;
    q.ocpg = L->oc32 / d.group;
    q.pin = q.pout = 32;
    q.dw4 = false;
    q.src_sn = (int64_t)L->ic32 * d.ih * d.iw;
    q.dst_sn = q.z_sn = (int64_t)L->oc32 * p.oh * p.ow;
    return igemm_usable(q);
}

mi355_relayout_desc rl_desc(uint32_t mode, uint32_t ndim, uint32_t s0, uint32_t s1, uint32_t s2, uint32_t s3, uint32_t s4,
                            uint32_t oc) {
    mi355_relayout_desc r;
    memset(&r, 0, sizeof(r));
    r.mode = mode;
    r.ndim = ndim;
    r.shape[0] = s0; r.shape[1] = s1; r.shape[2] = s2; r.shape[3] = s3; r.shape[4] = s4;
    r.group = 1;
    r.oc = oc;
    r.elem_bytes = 1;
    r.scale_src = r.scale_dst = 1.f;
    return r;
}

// (n, c, h, w) -> (n, ceil(c / 32), h, w, 32), zero padding past c
int to_nchw32(hipStream_t st, const void* src, void* dst, uint32_t n, uint32_t c, uint32_t h, uint32_t w) {
    const mi355_relayout_desc r = rl_desc(MI355_RL_NCHW_NCHW32, 4, n, c, h, w, 0, 0);
    const uint32_t oshape[7] = {n, (c + 31) / 32, h, w, 32, 0, 0};
    return launch_relayout(st, r, oshape, 5, src, dst, aligned16(src) && aligned16(dst));
}

}  // namespace

bool nchw_mfma_usable(const ConvProblem& p) {
    NchwLayout L;
    return make_layout(p, &L);
}

size_t nchw_mfma_workspace(const ConvProblem& p) {
    NchwLayout L;
    return make_layout(p, &L) ? L.total : 0;
}

int launch_conv_nchw_mfma(hipStream_t st, const ConvProblem& p, int cu_count, const int8_t* src, const int8_t* flt,
                          const int32_t* bias, const int8_t* z, int8_t* dst, void* workspace) {
    NchwLayout L;
    if (!make_layout(p, &L)) return (int)hipErrorInvalidValue;
    const mi355_conv_desc& d = p.d;
    if ((uint64_t)d.n * d.oc * p.oh * p.ow == 0) return 0;
    int8_t* ws = reinterpret_cast<int8_t*>(workspace);
    int8_t* src32 = ws + L.off_src;
    int8_t* flt32 = ws + L.off_flt;
    int8_t* dst32 = ws + L.off_dst;
    int8_t* z32 = d.has_z ? ws + L.off_z : nullptr;
    int rc = to_nchw32(st, src, src32, d.n, d.ic, d.ih, d.iw);
    if (rc) return rc;
    // the filter (oc, icpg, fh, fw) is an "NCHW tensor" of oc images; with groups icpg is a multiple of 32 already
    const uint32_t icpg32 = L.ic32 / d.group;
    rc = to_nchw32(st, flt, flt32, d.oc, p.icpg, d.fh, d.fw);
    if (rc) return rc;
    if (L.oc32 != d.oc) {
        // filter rows of the padded output channels (dense convolutions only: groups are whole blocks)
        const size_t row = (size_t)icpg32 * d.fh * d.fw;  // a multiple of 32 bytes
        const uint64_t vecs = (uint64_t)(L.oc32 - d.oc) * row / 16;
        hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)((vecs + 255) / 256)), dim3(256), 0, st,
                           reinterpret_cast<v4i*>(flt32 + (size_t)d.oc * row), vecs);
        rc = (int)hipGetLastError();
        if (rc) return rc;
    }
    const int32_t* bias32 = bias;
    if (d.bias_mode == MI355_BIAS_BROADCAST_CHANNEL && L.oc32 != d.oc) {
        int32_t* b = reinterpret_cast<int32_t*>(ws + L.off_bias);
        hipLaunchKernelGGL(bias_pad_kernel, dim3((L.oc32 + 255) / 256), dim3(256), 0, st, bias, b, d.oc, L.oc32);
        rc = (int)hipGetLastError();
        if (rc) return rc;
        bias32 = b;
    }
    if (d.has_z) {
        rc = to_nchw32(st, z, z32, d.n, d.oc, p.oh, p.ow);
        if (rc) return rc;
    }
    const int cfg = igemm_pick_cfg(L.inner, cu_count, false);
    rc = launch_conv_igemm(st, L.inner, cfg, cu_count, src32, flt32, bias32, z32, dst32, false);
    if (rc) return rc;
    const mi355_relayout_desc back = rl_desc(MI355_RL_NCHW32_NCHW, 5, d.n, L.oc32 / 32, p.oh, p.ow, 32, d.oc);
    const uint32_t oshape[7] = {d.n, d.oc, p.oh, p.ow, 0, 0, 0};
    return launch_relayout(st, back, oshape, 4, dst32, dst, aligned16(dst32) && aligned16(dst));
}

}  // namespace mi355
