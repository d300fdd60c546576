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
    const int quads = a.OH * a.QW;
    if (quads == 0 || d.n == 0) return 0;
    const int threads = quads >= 192 ? 256 : (quads > 64 ? 128 : 64);
    dim3 grid((quads + threads - 1) / threads, d.n * a.CG), block(threads);
    const bool sq = d.fh == 3 && d.fw == 3 && d.stride_h == d.stride_w;
    if (sq && d.stride_h == 1)
        hipLaunchKernelGGL((dw4_kernel<3, 1>), grid, block, 0, st, a);
    else if (sq && d.stride_h == 2)
        hipLaunchKernelGGL((dw4_kernel<3, 2>), grid, block, 0, st, a);
    else
        hipLaunchKernelGGL((dw4_kernel<0, 0>), grid, block, 0, st, a);
    return (int)hipGetLastError();
}

}  // namespace mi355
