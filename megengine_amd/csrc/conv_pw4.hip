// Pointwise (1x1) int8 ConvBias on 4-packed activations, NCHW4 in and out, for the two kinds of layer that a tiled
// kernel serves badly: at most 64 input channels and many output channels (the expansion layers of the MobileNet
// family: one or two MFMA k-steps, the cost is the output), and at most 32 output channels with up to 192 input
// channels (its narrow projections: a tile of 128 filter rows would be three quarters empty).
//
// A tiled implicit GEMM spends such a layer on its per-tile pipeline (stage, barrier, multiply: one k-stage per tile).
// Here nothing is staged and nothing is shared after the first barrier:
//   * a wave keeps the filter rows of its 32, 64 or 96 output channels in registers for the whole launch
//     (MFMA A fragments: lane = output channel, 16 contiguous k-bytes of its row);
//   * it walks blocks of 32 pixels; a lane's B fragment -- 16 k-bytes of its pixel = 4 channel blocks -- is four
//     coalesced dword loads (32 consecutive pixels x 4 bytes each), fetched for the NEXT block, together with its
//     residual, while this one is multiplied and requantised;
//   * accumulators start from the bias (LDS copy), the fused epilogue and the NCHW4 stores are those of the tiled
//     kernels (igemm_shared.h).
// Channel blocks past the last one, and filter bytes past the end of a row, meet zero activations.
#include <string.h>
#include <type_traits>
#include "igemm_shared.h"

namespace mi355 {
namespace {

constexpr int PW4_MAX_OC = 1024;

// HZ: the launch has a residual (its registers exist only in that instantiation)
template <int MT, int KC, bool HZ>
__global__ __launch_bounds__(256) void pw4s_kernel(IgemmArgs a, int n_ocg, int n_pb) {
    __shared__ __attribute__((aligned(16))) int sBias[PW4_MAX_OC + 96];
    const int t = threadIdx.x;
    const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l32 = lane & 31, lh = lane >> 5;

    const int gw = blockIdx.x * 4 + wave, GW = gridDim.x * 4;  // GW is a multiple of n_ocg
    const int pb0 = gw / n_ocg, ocg = gw - pb0 * n_ocg, step = GW / n_ocg;
    const int oc_w = ocg * MT * 32;
    const __amdgpu_buffer_rsrc_t rs_src = make_rsrc(a.src, a.src_bytes);
    const __amdgpu_buffer_rsrc_t rs_flt = make_rsrc(a.flt, a.flt_bytes);

    v4i fa[MT][KC];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int row = oc_w + i * 32 + l32;
#pragma unroll
        for (int kc = 0; kc < KC; ++kc)
            fa[i][kc] = __builtin_amdgcn_raw_buffer_load_b128(rs_flt, row < a.OC ? row * a.kbytes + kc * 32 + lh * 16 : SENT, 0, 0);
    }

    const int icb = a.kbytes >> 2;
    auto load_b = [&](int pb, v4i (&x)[KC]) __attribute__((always_inline)) {
        const int m = pb * 32 + l32;
        const bool ok = m < a.M;  // also false for every block past the last one
        const uint32_t mm = ok ? m : 0;
        const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
        const uint32_t oh = fdiv(rem, a.div_ow), ow = rem - oh * a.OW;
        const int pix = (int)n * a.src_sn + ((int)oh * a.sh * a.IW + (int)ow * a.sw) * 4;
#pragma unroll
        for (int kc = 0; kc < KC; ++kc)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int cb = kc * 8 + lh * 4 + i;
                x[kc][i] = __builtin_amdgcn_raw_buffer_load_b32(rs_src, (ok && cb < icb) ? pix + cb * a.src_scb : SENT, 0, 0);
            }
    };

    v4i fb[KC], nb[KC];
    ZRegs<HZ ? MT : 1, 1> zr, nz;
    load_b(pb0, fb);
    if constexpr (HZ) igemm_load_z<4, MT, 1>(a, zr, oc_w, pb0 * 32, l32, lh);
    // the bias goes to LDS after the filter rows and the first block are requested: one memory round trip before the
    // first multiply instead of two (the barrier waits for everything outstanding)
    for (int i = t; i < PW4_MAX_OC + 96; i += 256) sBias[i] = (a.has_bias && i < a.OC) ? a.bias[i] : 0;
    __syncthreads();
    for (int pb = pb0; pb < n_pb; pb += step) {
        // the next block's pixels and residual are in flight during the multiply and the epilogue
        load_b(pb + step, nb);
        if constexpr (HZ) igemm_load_z<4, MT, 1>(a, nz, oc_w, (pb + step) * 32, l32, lh);
        v16i acc[MT][1];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i b = *reinterpret_cast<const v4i*>(sBias + oc_w + i * 32 + 8 * q + 4 * lh);
                acc[i][0][4 * q + 0] = b[0]; acc[i][0][4 * q + 1] = b[1]; acc[i][0][4 * q + 2] = b[2]; acc[i][0][4 * q + 3] = b[3];
            }
#pragma unroll
        for (int kc = 0; kc < KC; ++kc)
#pragma unroll
            for (int i = 0; i < MT; ++i) acc[i][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i][kc], fb[kc], acc[i][0], 0, 0, 0);
        if constexpr (HZ)
            igemm_run_epilogue<4, MT, 1, true>(a, acc, oc_w, pb * 32, l32, lh, &zr);
        else
            igemm_run_epilogue<4, MT, 1>(a, acc, oc_w, pb * 32, l32, lh);
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) fb[kc] = nb[kc];
        if constexpr (HZ) zr = nz;
    }
}

// The same for 32-packed activations (NCHW32 in and out) with at most 128 input channels: the expanding 1x1 layers of a
// bottleneck block and its projection shortcut, whose cost is their output (and residual) stream.  A lane's B fragment
// of k-step kc is one 16-byte load -- half of its pixel's 32-byte block kc; 32 consecutive pixels are one contiguous
// kilobyte -- and the stores are the 16-byte stores of the tiled kernels.
template <int MT, int KC, bool HZ>
__global__ __launch_bounds__(256, 2) void pw32s_kernel(IgemmArgs a, int n_ocg, int n_pb,
                                                       std::conditional_t<HZ, ResidualTable, NoResidualTable> tab) {
    const int t = threadIdx.x;
    const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l32 = lane & 31, lh = lane >> 5;

    // Pixel blocks by XCD, as the tiled kernels deal out their tiles: workgroup b runs on XCD b % 8 (round-robin
    // dispatch) and each XCD takes one contiguous eighth of the pixel blocks, so that this layer finds its inputs in the
    // L2 of the XCD that wrote them and leaves its outputs where the next layer's workgroups will look for them.
    // (Grids that are no multiple of 8 n_ocg / 4 workgroups -- small problems -- interleave the blocks instead.)
    int pb_lo = 0, pb_hi = n_pb, gw = blockIdx.x * 4 + wave, GW = gridDim.x * 4;  // GW is a multiple of n_ocg
    if ((gridDim.x & 7) == 0 && ((gridDim.x >> 3) * 4) % n_ocg == 0) {
        const int x = blockIdx.x & 7, per = n_pb >> 3, rem = n_pb & 7;
        pb_lo = x * per + (x < rem ? x : rem);
        pb_hi = pb_lo + per + (x < rem ? 1 : 0);
        gw = (blockIdx.x >> 3) * 4 + wave;
        GW = (gridDim.x >> 3) * 4;
    }
    const int q0 = gw / n_ocg, ocg = gw - q0 * n_ocg, step = GW / n_ocg;
    const int pb0 = pb_lo + q0;
    const int oc_w = ocg * MT * 32;
    const __amdgpu_buffer_rsrc_t rs_src = make_rsrc(a.src, a.src_bytes);
    const __amdgpu_buffer_rsrc_t rs_flt = make_rsrc(a.flt, a.flt_bytes);
    const __amdgpu_buffer_rsrc_t rs_bias = make_rsrc(a.bias, a.has_bias ? a.OC * 4 : 0);
    // residual table form: the 256 offsets from the kernel's last argument into LDS, once per workgroup (ahead of the first
    // loads: behind them, with the barrier holding every wave until the slowest wave's loads are back, the stack is 3 us
    // slower)
    __shared__ float zt[HZ ? 256 : 1];
    if constexpr (HZ) {
        if (a.epi.zlin) zt[t] = tab.v[t];
        __syncthreads();
    }

    v4i fa[MT][KC];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int row = oc_w + i * 32 + l32;
#pragma unroll
        for (int kc = 0; kc < KC; ++kc)
            fa[i][kc] = __builtin_amdgcn_raw_buffer_load_b128(rs_flt, row < a.OC ? row * a.kbytes + kc * 32 + lh * 16 : SENT, 0, 0);
    }
    // the bias of the wave's channels, in accumulator order: the first multiply of every block takes it as its addend
    // (channels past the last one read as zero through the descriptor)
    v16i bv[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const v4i b = __builtin_amdgcn_raw_buffer_load_b128(rs_bias, (oc_w + i * 32 + 8 * q + 4 * lh) * 4, 0, 0);
            bv[i][4 * q + 0] = b[0]; bv[i][4 * q + 1] = b[1]; bv[i][4 * q + 2] = b[2]; bv[i][4 * q + 3] = b[3];
        }

    auto load_b = [&](int pb, v4i (&x)[KC]) __attribute__((always_inline)) {
        const int m = pb * 32 + l32;
        const bool ok = m < a.M;  // also false for every block past the last one
        const uint32_t mm = ok ? m : 0;
        const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
        const uint32_t oh = fdiv(rem, a.div_ow), ow = rem - oh * a.OW;
        const int pix = ok ? (int)n * a.src_sn + ((int)oh * a.sh * a.IW + (int)ow * a.sw) * 32 + lh * 16 : SENT;
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) x[kc] = __builtin_amdgcn_raw_buffer_load_b128(rs_src, pix, kc * a.src_scb, 0);
    };

    v4i fb[KC], nb[KC];
    ZRegs<HZ ? MT : 1, 1> zr, nz;
    load_b(pb0 < pb_hi ? pb0 : n_pb, fb);
    if constexpr (HZ) igemm_load_z<32, MT, 1>(a, zr, oc_w, (pb0 < pb_hi ? pb0 : n_pb) * 32, l32, lh);
    for (int pb = pb0; pb < pb_hi; pb += step) {
        // the next block's pixels and residual are in flight during the multiply and the epilogue (past the end of this
        // XCD's blocks: the block past the last one, whose lanes are all masked)
        const int nx = pb + step < pb_hi ? pb + step : n_pb;
        load_b(nx, nb);
        if constexpr (HZ) igemm_load_z<32, MT, 1>(a, nz, oc_w, nx * 32, l32, lh);
        v16i acc[MT][1];
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[i][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i][0], fb[0], bv[i], 0, 0, 0);
#pragma unroll
        for (int kc = 1; kc < KC; ++kc)
#pragma unroll
            for (int i = 0; i < MT; ++i) acc[i][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i][kc], fb[kc], acc[i][0], 0, 0, 0);
        if constexpr (HZ)
            igemm_run_epilogue<32, MT, 1, true>(a, acc, oc_w, pb * 32, l32, lh, &zr, -1, 1, 0, -1, zt);
        else
            igemm_run_epilogue<32, MT, 1>(a, acc, oc_w, pb * 32, l32, lh);
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) fb[kc] = nb[kc];
        if constexpr (HZ) zr = nz;
    }
}

template <int MT, int KC>
int launch32_mt(hipStream_t st, const IgemmArgs& a, int cu_count) {
    const int ocb = (a.OC + 31) / 32;
    const int n_ocg = (ocb + MT - 1) / MT;
    const int n_pb = (a.M + 31) / 32;
    if (cu_count <= 0) cu_count = 256;
    int64_t blocks = ((int64_t)n_pb * n_ocg + 3) / 4;
    const int64_t cap = (int64_t)cu_count * 3;  // 12 waves per CU
    if (blocks > cap) blocks = cap;
    blocks = (blocks + n_ocg - 1) / n_ocg * n_ocg;  // waves of one pixel block stay together; 4 * blocks % n_ocg == 0
    // large grids: a multiple of 8 n_ocg workgroups, which the kernel splits into one slab of pixel blocks per XCD
    if (blocks >= 16 * (int64_t)n_ocg) blocks = blocks / (8 * n_ocg) * (8 * n_ocg);
    if (a.epi.has_z) {
        ResidualTable tab;
        if (a.epi.zlin) memcpy(tab.v, a.ztab, sizeof(tab.v)); else memset(tab.v, 0, sizeof(tab.v));
        hipLaunchKernelGGL((pw32s_kernel<MT, KC, true>), dim3((unsigned)blocks), dim3(256), 0, st, a, n_ocg, n_pb, tab);
    } else {
        hipLaunchKernelGGL((pw32s_kernel<MT, KC, false>), dim3((unsigned)blocks), dim3(256), 0, st, a, n_ocg, n_pb, NoResidualTable{});
    }
    return (int)hipGetLastError();
}

template <int MT, int KC>
int launch_mt(hipStream_t st, const IgemmArgs& a, int cu_count) {
    const int ocb = (a.OC + 31) / 32;
    const int n_ocg = (ocb + MT - 1) / MT;
    const int n_pb = (a.M + 31) / 32;
    if (cu_count <= 0) cu_count = 256;
    int64_t blocks = ((int64_t)n_pb * n_ocg + 3) / 4;
    const int64_t cap = (int64_t)cu_count * 4;  // 16 waves per CU
    if (blocks > cap) blocks = cap;
    blocks = (blocks + n_ocg - 1) / n_ocg * n_ocg;  // waves of one pixel block stay together; 4 * blocks % n_ocg == 0
    if (a.epi.has_z)
        hipLaunchKernelGGL((pw4s_kernel<MT, KC, true>), dim3((unsigned)blocks), dim3(256), 0, st, a, n_ocg, n_pb);
    else
        hipLaunchKernelGGL((pw4s_kernel<MT, KC, false>), dim3((unsigned)blocks), dim3(256), 0, st, a, n_ocg, n_pb);
    return (int)hipGetLastError();
}

}  // namespace

bool pw4s_usable(const IgemmArgs& a) {
    if (a.T != 1 || a.ph != 0 || a.pw != 0 || a.OC > PW4_MAX_OC) return false;
    return a.kbytes <= 64 || (a.OC <= 32 && a.kbytes <= 192);
}

// 32-packed: pointwise without padding, dense, the fast epilogue, 32 to 128 input channels, at most 1024 output channels
bool pw32s_usable(const IgemmArgs& a, int pin, int pout) {
    return pin == 32 && pout == 32 && a.T == 1 && a.ph == 0 && a.pw == 0 && a.groups == 1 && !a.general &&
           a.OC <= PW4_MAX_OC && a.kbytes >= 32 && a.kbytes <= 128 && a.kbytes % 32 == 0;
}

int launch_pw32s(hipStream_t st, const IgemmArgs& a, int cu_count) {
    if (a.M == 0 || a.OC == 0) return 0;
    const bool one = (a.OC + 31) / 32 == 1;  // a single channel block: one block per wave
    switch (a.kbytes / 32) {
        case 1: return one ? launch32_mt<1, 1>(st, a, cu_count) : launch32_mt<2, 1>(st, a, cu_count);
        case 2: return one ? launch32_mt<1, 2>(st, a, cu_count) : launch32_mt<2, 2>(st, a, cu_count);
        case 3: return one ? launch32_mt<1, 3>(st, a, cu_count) : launch32_mt<2, 3>(st, a, cu_count);
        default: return one ? launch32_mt<1, 4>(st, a, cu_count) : launch32_mt<2, 4>(st, a, cu_count);
    }
}

int launch_pw4s(hipStream_t st, const IgemmArgs& a, int cu_count) {
    if (a.M == 0 || a.OC == 0) return 0;
    const int ocb = (a.OC + 31) / 32;
    if (ocb == 1) {  // narrow outputs (the projections): one channel block per wave, up to six k-steps
        switch ((a.kbytes + 31) / 32) {
            case 1: return launch_mt<1, 1>(st, a, cu_count);
            case 2: return launch_mt<1, 2>(st, a, cu_count);
            case 3: return launch_mt<1, 3>(st, a, cu_count);
            case 4: return launch_mt<1, 4>(st, a, cu_count);
            case 5: return launch_mt<1, 5>(st, a, cu_count);
            default: return launch_mt<1, 6>(st, a, cu_count);
        }
    }
    const bool three = ocb % 3 == 0 || ocb > 4;  // 96-channel waves unless the channel count splits evenly into 64s
    if (a.kbytes <= 32) return three ? launch_mt<3, 1>(st, a, cu_count) : launch_mt<2, 1>(st, a, cu_count);
    return three ? launch_mt<3, 2>(st, a, cu_count) : launch_mt<2, 2>(st, a, cu_count);
}

}  // namespace mi355
