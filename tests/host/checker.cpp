// Test driver for the host-side C++ operator classes (megengine_amd/host), in the manner of the
// reference's Checker<ConvBias> (dnn/test/common/checker.h, dnn/test/common/conv_bias.cpp): build
// layouts, let the operator deduce dst, run exec on the device, compare every element with the CPU
// parity checker fed from an independently written descriptor.
//
//   host_checker --cpu     layout deduction, validation errors, algorithm listing (no device needed)
//   host_checker --gpu     the above + exec cases on device 0
//
// Prints one line per case and "ALL OK" at the end; exit status 0 only when everything passed.
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <functional>
#include <string>
#include <vector>

#include "../../include/mi355_convbias.h"
#include "../../megengine_amd/host/mi355dnn.h"

extern "C" {
int oracle_convbias_s8(const mi355_conv_desc* d, const int8_t* src, const int8_t* flt, const int32_t* bias,
                       const void* z, void* dst);
int oracle_relayout_deduce(const mi355_relayout_desc* d, uint32_t* ndim, uint32_t shape[7]);
int oracle_relayout(const mi355_relayout_desc* d, const void* src, void* dst);
}

using namespace mi355dnn;
using CB = param::ConvBias;

static int g_fail = 0;
#define EXPECT(cond, ...)                        \
    do {                                         \
        if (!(cond)) {                           \
            printf("  FAIL %s:%d: ", __FILE__, __LINE__); \
            printf(__VA_ARGS__);                 \
            printf("\n");                        \
            ++g_fail;                            \
        }                                        \
    } while (0)

static uint64_t splitmix(uint64_t& s) {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static void fill_s8(std::vector<int8_t>& v, uint64_t seed, int lo, int hi) {
    for (auto& x : v) x = (int8_t)(lo + (int)(splitmix(seed) % (uint64_t)(hi - lo + 1)));
}
static void fill_s32(std::vector<int32_t>& v, uint64_t seed, int lo, int hi) {
    for (auto& x : v) x = lo + (int)(splitmix(seed) % (uint64_t)(hi - lo + 1));
}

#define HIP_OK(x)                                                        \
    do {                                                                 \
        hipError_t e_ = (x);                                             \
        if (e_ != hipSuccess) {                                          \
            printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            exit(3);                                                     \
        }                                                                \
    } while (0)

struct DevBuf {
    void* p = nullptr;
    explicit DevBuf(size_t bytes) { HIP_OK(hipMalloc(&p, bytes ? bytes : 16)); }
    ~DevBuf() { (void)hipFree(p); }
};

static bool throws(const std::function<void()>& f, int status) {
    try {
        f();
    } catch (const Error& e) {
        if (e.status() != status) printf("  (threw status %d: %s)\n", e.status(), e.what());
        return e.status() == status;
    }
    return false;
}

// ------------------------------------------------------------------ a ConvBias case
struct Case {
    const char* name;
    CB::Format fmt;
    CB::Sparse sparse;
    CB::NonlineMode nl;
    TensorShape src, flt;
    uint32_t pad, stride;
    bool has_bias, has_z;
    bool dst_s32;
    // the descriptor the CPU checker is given, written by hand for each case
    uint32_t n, ic, ih, iw, oc, fh, fw, group;
};

static std::vector<Case> cases() {
    using F = CB::Format;
    using S = CB::Sparse;
    using N = CB::NonlineMode;
    return {
        {"nchw4 dense 3x3 relu", F::NCHW4, S::DENSE, N::RELU, {2, 4, 9, 11, 4}, {24, 4, 3, 3, 4}, 1, 1, true, false, false,
         2, 16, 9, 11, 24, 3, 3, 1},
        {"nchw4 dense 1x1 z identity", F::NCHW4, S::DENSE, N::IDENTITY, {3, 8, 7, 7, 4}, {32, 8, 1, 1, 4}, 0, 1, true, true,
         false, 3, 32, 7, 7, 32, 1, 1, 1},
        {"nchw4 group 2", F::NCHW4, S::GROUP, N::RELU, {2, 4, 8, 8, 4}, {2, 8, 2, 3, 3, 4}, 1, 2, true, false, false,
         2, 16, 8, 8, 16, 3, 3, 2},
        {"nchw32 dense 3x3 hswish z", F::NCHW32, S::DENSE, N::H_SWISH, {2, 2, 10, 10, 32}, {64, 2, 3, 3, 32}, 1, 1, true,
         true, false, 2, 64, 10, 10, 64, 3, 3, 1},
        {"nchw32 1x1 s2 no bias", F::NCHW32, S::DENSE, N::IDENTITY, {2, 4, 12, 12, 32}, {32, 4, 1, 1, 32}, 0, 2, false, false,
         false, 2, 128, 12, 12, 32, 1, 1, 1},
        {"nchw32 s32 dst", F::NCHW32, S::DENSE, N::IDENTITY, {1, 1, 6, 6, 32}, {32, 1, 3, 3, 32}, 1, 1, true, false, true,
         1, 32, 6, 6, 32, 3, 3, 1},
        {"nchw4->nchw32", F::NCHW4_NCHW32, S::DENSE, N::RELU, {2, 4, 8, 8, 4}, {32, 4, 3, 3, 4}, 1, 1, true, false, false,
         2, 16, 8, 8, 32, 3, 3, 1},
        {"nchw32->nchw4", F::NCHW32_NCHW4, S::DENSE, N::RELU, {2, 1, 8, 8, 32}, {12, 1, 3, 3, 32}, 1, 1, true, false, false,
         2, 32, 8, 8, 12, 3, 3, 1},
        {"nchw4->nchw", F::NCHW4_NCHW, S::DENSE, N::RELU, {2, 4, 8, 8, 4}, {10, 4, 3, 3, 4}, 1, 1, true, true, false,
         2, 16, 8, 8, 10, 3, 3, 1},
        {"nchw dense", F::NCHW, S::DENSE, N::RELU, {2, 5, 9, 9}, {7, 5, 3, 3}, 1, 1, true, true, false,
         2, 5, 9, 9, 7, 3, 3, 1},
        // large enough for the heuristic to take the relayout + MFMA algorithm, which needs a workspace
        {"nchw dense, workspace", F::NCHW, S::DENSE, N::RELU, {4, 24, 28, 28}, {40, 24, 3, 3}, 1, 1, true, true, false,
         4, 24, 28, 28, 40, 3, 3, 1},
        {"nchw depthwise", F::NCHW, S::GROUP, N::RELU, {2, 6, 9, 9}, {6, 1, 1, 3, 3}, 1, 2, true, false, false,
         2, 6, 9, 9, 6, 3, 3, 6},
        {"nchw44 channel-wise", F::NCHW44, S::GROUP, N::RELU, {2, 3, 9, 9, 4}, {3, 1, 1, 3, 3, 4}, 1, 1, true, false, false,
         2, 12, 9, 9, 12, 3, 3, 12},
        {"nchw44 dense", F::NCHW44, S::DENSE, N::IDENTITY, {1, 2, 6, 6, 4}, {2, 2, 3, 3, 4, 4}, 1, 1, true, false, false,
         1, 8, 6, 6, 8, 3, 3, 1},
    };
}

static TensorShape bias_shape(const Case& c, const TensorShape& dst) {
    if (c.fmt == CB::Format::NCHW || c.fmt == CB::Format::NCHW4_NCHW) return {1, dst[1], 1, 1};
    return {1, dst[1], 1, 1, dst[4]};
}

static void run_conv_case(Handle* h, const Case& c, bool on_gpu) {
    printf("case: %s\n", c.name);
    fflush(stdout);
    const float s_src = 0.02f, s_flt = 0.01f, s_dst = 0.05f, s_z = 0.04f;
    auto opr = h->create_operator<ConvBiasForward>();
    opr->param().format = c.fmt;
    opr->param().sparse = c.sparse;
    opr->param().nonlineMode = c.nl;
    opr->param().pad_h = opr->param().pad_w = c.pad;
    opr->param().stride_h = opr->param().stride_w = c.stride;
    TensorLayout src(c.src, dtype::QuantizedS8(s_src)), flt(c.flt, dtype::QuantizedS8(s_flt));
    TensorLayout dst;
    dst.dtype = c.dst_s32 ? dtype::QuantizedS32(s_src * s_flt) : dtype::QuantizedS8(s_dst);
    TensorLayout none_b, none_z;
    none_b.dtype = dtype::QuantizedS32(s_src * s_flt);
    none_z.dtype = dst.dtype;
    opr->deduce_layout(src, flt, none_b, none_z, dst);

    // independent expectation of the dst shape
    mi355_conv_desc d = mi355_conv_desc();
    d.format = (uint32_t)c.fmt; d.sparse = (uint32_t)c.sparse; d.nonline = (uint32_t)c.nl; d.mode = 0;
    d.n = c.n; d.ic = c.ic; d.ih = c.ih; d.iw = c.iw; d.oc = c.oc; d.fh = c.fh; d.fw = c.fw; d.group = c.group;
    d.pad_h = d.pad_w = c.pad; d.stride_h = d.stride_w = c.stride; d.dilate_h = d.dilate_w = 1;
    d.dst_dtype = c.dst_s32 ? MI355_DT_QS32 : MI355_DT_QS8;
    d.bias_mode = c.has_bias ? MI355_BIAS_BROADCAST_CHANNEL : MI355_BIAS_NONE;
    d.has_z = c.has_z;
    d.scale_bias = s_src * s_flt; d.scale_z = c.dst_s32 ? s_src * s_flt : s_z; d.scale_dst = c.dst_s32 ? s_src * s_flt : s_dst;
    const uint32_t oh = (c.ih + 2 * c.pad - c.fh) / c.stride + 1, ow = (c.iw + 2 * c.pad - c.fw) / c.stride + 1;
    const bool plain = c.fmt == CB::Format::NCHW || c.fmt == CB::Format::NCHW4_NCHW;  // dst layout
    const uint32_t po = plain ? 1 : (c.fmt == CB::Format::NCHW32 || c.fmt == CB::Format::NCHW4_NCHW32) ? 32 : 4;
    TensorShape want = plain ? TensorShape{c.n, c.oc, oh, ow} : TensorShape{c.n, c.oc / po, oh, ow, po};
    EXPECT(dst.eq_shape(want), "deduced dst %s, expected %s", dst.to_string().c_str(), want.to_string().c_str());
    EXPECT(dst.is_contiguous(), "deduced dst must be contiguous");
    if (!c.dst_s32) EXPECT(dst.dtype == dtype::QuantizedS8(s_dst), "a named QuantizedS8 dst dtype must be kept");
    else EXPECT(dst.dtype == dtype::QuantizedS32(s_src * s_flt), "default dst dtype is QuantizedS32(s_src*s_flt)");

    TensorLayout bias = none_b, z = none_z;
    if (c.has_bias) bias = TensorLayout(bias_shape(c, dst), dtype::QuantizedS32(s_src * s_flt));
    if (c.has_z) z = TensorLayout(dst, c.dst_s32 ? dst.dtype : dtype::QuantizedS8(s_z));
    if (c.dst_s32 && c.has_z) return;  // not in the table

    size_t ws = opr->get_workspace_in_bytes(src, flt, bias, z, dst);
    auto algos = opr->get_all_algorithms_info(src, flt, bias, z, dst);
    EXPECT(!algos.empty(), "no usable algorithm");
    auto heur = opr->get_algorithm_info_heuristic(src, flt, bias, z, dst);
    bool listed = false;
    for (auto& a : algos) listed = listed || a.desc.id == heur.desc.id;
    EXPECT(listed, "heuristic algorithm %s is not in the list", heur.name.c_str());
    {
        // get_workspace_in_bytes is the C ABI's number for the heuristic's algorithm; only the plain-NCHW relayout
        // algorithm needs one
        size_t abi_ws = 0;
        mi355_algo qa;
        EXPECT(mi355_convbias_s8_query(&d, MI355_ALGO_HEURISTIC, &qa, &abi_ws) == MI355_OK && abi_ws == ws,
               "workspace: C++ %zu, C ABI %zu", ws, abi_ws);
        const bool relayout_algo = heur.name.find("NCHW_RELAYOUT") != std::string::npos;
        EXPECT((ws > 0) == relayout_algo, "workspace %zu for %s", ws, heur.name.c_str());
        if (!strcmp(c.name, "nchw dense, workspace")) EXPECT(relayout_algo, "heuristic for a large NCHW problem: %s", heur.name.c_str());
    }
    // the largest workspace any listed algorithm asks for
    size_t ws_all = ws;
    for (auto& a : algos) {
        opr->execution_policy().algo = a.desc;
        ws_all = std::max(ws_all, opr->get_workspace_in_bytes(src, flt, bias, z, dst));
    }
    opr->execution_policy().algo = AlgorithmDesc{};
    if (!on_gpu) return;

    std::vector<int8_t> hsrc(src.total_nr_elems()), hflt(flt.total_nr_elems()), hz(z.total_nr_elems());
    std::vector<int32_t> hbias(bias.total_nr_elems());
    fill_s8(hsrc, 11, -128, 127);
    fill_s8(hflt, 12, -127, 127);
    fill_s8(hz, 13, -128, 127);
    fill_s32(hbias, 14, -1000, 1000);
    const size_t dst_bytes = dst.total_nr_elems() * dst.dtype.size();
    std::vector<uint8_t> expect(dst_bytes), got(dst_bytes);
    int st = oracle_convbias_s8(&d, hsrc.data(), hflt.data(), c.has_bias ? hbias.data() : nullptr,
                                c.has_z ? hz.data() : nullptr, expect.data());
    EXPECT(st == 0, "CPU checker refused the case: %d", st);

    DevBuf dsrc(hsrc.size()), dflt(hflt.size()), dbias(hbias.size() * 4), dz(hz.size()), ddst(dst_bytes), dws(ws_all);
    HIP_OK(hipMemcpy(dsrc.p, hsrc.data(), hsrc.size(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dflt.p, hflt.data(), hflt.size(), hipMemcpyHostToDevice));
    if (c.has_bias) HIP_OK(hipMemcpy(dbias.p, hbias.data(), hbias.size() * 4, hipMemcpyHostToDevice));
    if (c.has_z) HIP_OK(hipMemcpy(dz.p, hz.data(), hz.size(), hipMemcpyHostToDevice));

    // every listed algorithm must reproduce the checker bit for bit
    for (auto& a : algos) {
        HIP_OK(hipMemset(ddst.p, 0x5a, dst_bytes));
        opr->execution_policy().algo = a.desc;
        size_t need = opr->get_workspace_in_bytes(src, flt, bias, z, dst);
        if (need > 0) {
            // check_exec's rule (dnn/src/common/conv_bias.cpp:32-37): a workspace smaller than reported is an error
            EXPECT(throws([&] {
                       opr->exec(TensorND(dsrc.p, src), TensorND(dflt.p, flt), TensorND(dbias.p, bias), TensorND(dz.p, z),
                                 TensorND(ddst.p, dst), nullptr, Workspace(dws.p, need - 1));
                   }, MI355_ERR_WORKSPACE), "%s must refuse a short workspace", a.name.c_str());
        }
        opr->exec(TensorND(dsrc.p, src), TensorND(dflt.p, flt), TensorND(dbias.p, bias), TensorND(dz.p, z),
                  TensorND(ddst.p, dst), nullptr, Workspace(dws.p, need));
        HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
        HIP_OK(hipMemcpy(got.data(), ddst.p, dst_bytes, hipMemcpyDeviceToHost));
        size_t bad = 0;
        for (size_t i = 0; i < dst_bytes; ++i) bad += got[i] != expect[i];
        EXPECT(bad == 0, "%s: %zu of %zu bytes differ from the CPU checker", a.name.c_str(), bad, dst_bytes);
    }
    printf("  %zu algorithms bit-exact (heuristic: %s)\n", algos.size(), heur.name.c_str());
}

// ------------------------------------------------------------------ validation (no device)
static void run_validation(Handle* h) {
    printf("case: validation errors\n");
    auto opr = h->create_operator<ConvBiasForward>();
    opr->param().format = CB::Format::NCHW4;
    TensorLayout src({2, 4, 8, 8, 4}, dtype::QuantizedS8(0.02f)), flt({16, 4, 3, 3, 4}, dtype::QuantizedS8(0.01f));
    TensorLayout nb, nz, dst;
    nb.dtype = dtype::QuantizedS32(0.02f * 0.01f);
    dst.dtype = dtype::QuantizedS8(0.1f);
    opr->deduce_layout(src, flt, nb, nz, dst);
    EXPECT(dst.eq_shape(TensorShape{2, 4, 6, 6, 4}), "pad 0 dst %s", dst.to_string().c_str());

    // bias scale must equal src scale * filter scale within 1e-6
    TensorLayout bad_bias({1, 4, 1, 1, 4}, dtype::QuantizedS32(0.5f));
    EXPECT(throws([&] { opr->get_workspace_in_bytes(src, flt, bad_bias, nz, dst); }, MI355_ERR_BAD_ARG),
           "bias scale mismatch must be rejected");
    // wrong bias shape
    TensorLayout bias5({1, 5, 1, 1, 4}, dtype::QuantizedS32(0.02f * 0.01f));
    EXPECT(throws([&] { opr->get_workspace_in_bytes(src, flt, bias5, nz, dst); }, MI355_ERR_SHAPE),
           "bias of the wrong shape must be rejected");
    // z must have the dst shape
    TensorLayout zbad({2, 4, 6, 5, 4}, dtype::QuantizedS8(0.1f));
    EXPECT(throws([&] { opr->get_workspace_in_bytes(src, flt, nb, zbad, dst); }, MI355_ERR_SHAPE), "z shape");
    // channel mismatch between src and filter
    TensorLayout flt_bad({16, 3, 3, 3, 4}, dtype::QuantizedS8(0.01f));
    TensorLayout d2 = dst;
    EXPECT(throws([&] { opr->deduce_layout(src, flt_bad, nb, nz, d2); }, MI355_ERR_SHAPE), "channel mismatch");
    // SIGMOID has no quantized definition
    opr->param().nonlineMode = CB::NonlineMode::SIGMOID;
    EXPECT(throws([&] { opr->deduce_layout(src, flt, nb, nz, d2); }, MI355_ERR_UNSUPPORTED), "SIGMOID");
    opr->param().nonlineMode = CB::NonlineMode::RELU;
    // dilation in a packed format
    opr->param().dilate_h = 2;
    EXPECT(throws([&] { opr->deduce_layout(src, flt, nb, nz, d2); }, MI355_ERR_UNSUPPORTED), "dilation in NCHW4");
    opr->param().dilate_h = 1;
    // unsupported format
    opr->param().format = CB::Format::NHWC;
    EXPECT(throws([&] { opr->deduce_layout(src, flt, nb, nz, d2); }, MI355_ERR_UNSUPPORTED), "NHWC");
    opr->param().format = CB::Format::NCHW4;
    // non-contiguous rows
    TensorLayout src_nc = src;
    src_nc.stride[2] += 4;
    EXPECT(throws([&] { opr->deduce_layout(src_nc, flt, nb, nz, d2); }, MI355_ERR_UNSUPPORTED), "row-strided src");
    // batch-strided src is fine
    TensorLayout src_bs = src;
    src_bs.stride[0] += 64;
    opr->deduce_layout(src_bs, flt, nb, nz, d2);
    EXPECT(d2.eq_shape(dst), "batch-strided src");
    // undersized workspace is only checked at exec; a null tensor pointer is rejected before any launch
    EXPECT(throws([&] {
               opr->exec(TensorND(nullptr, src), TensorND(nullptr, flt), TensorND(nullptr, nb), TensorND(nullptr, nz),
                         TensorND(nullptr, dst), nullptr, Workspace());
           }, MI355_ERR_BAD_ARG),
           "null pointers");
    EXPECT(std::string(opr->get_algorithm_set_name()) == "MI355_CONV_BIAS", "set name");
    EXPECT(Handle::abi_version() == MI355_CONVBIAS_ABI_VERSION, "abi version");

    // RelayoutFormat deduction against the CPU checker's rule
    auto rl = h->create_operator<RelayoutFormat>();
    struct { param::RelayoutFormat::Mode m; TensorShape s; uint32_t oc, group; } rc[] = {
        {param::RelayoutFormat::Mode::NCHW_NCHW4, {2, 7, 5, 6}, 0, 1},
        {param::RelayoutFormat::Mode::NCHW_NCHW4, {2, 12, 5, 6}, 0, 4},
        {param::RelayoutFormat::Mode::NCHW4_NCHW, {2, 2, 5, 6, 4}, 7, 1},
        {param::RelayoutFormat::Mode::NCHW_NCHW4_WEIGHT, {6, 7, 3, 3}, 0, 1},
        {param::RelayoutFormat::Mode::NCHW_NCHW4_IC_SMALL, {2, 3, 8, 8}, 0, 1},
        {param::RelayoutFormat::Mode::NCHW_NCHW32, {2, 40, 5, 6}, 0, 1},
        {param::RelayoutFormat::Mode::NCHW32_NCHW, {2, 2, 5, 6, 32}, 40, 1},
    };
    for (auto& r : rc) {
        rl->param().mode = r.m; rl->param().oc = r.oc; rl->param().group = r.group;
        TensorLayout s(r.s, dtype::QuantizedS8(1.f)), o;
        rl->deduce_layout(s, o);
        mi355_relayout_desc rd = mi355_relayout_desc();
        rd.mode = (uint32_t)r.m; rd.ndim = (uint32_t)r.s.ndim; rd.group = r.group; rd.oc = r.oc; rd.elem_bytes = 1;
        rd.scale_src = rd.scale_dst = 1.f;
        for (size_t i = 0; i < r.s.ndim; ++i) rd.shape[i] = (uint32_t)r.s[i];
        uint32_t nd, sh[7];
        int st = oracle_relayout_deduce(&rd, &nd, sh);
        bool same = st == 0 && nd == o.ndim;
        for (uint32_t i = 0; same && i < nd; ++i) same = sh[i] == o[i];
        EXPECT(same, "relayout mode %u: deduced %s", (unsigned)r.m, o.to_string().c_str());
    }
}

static void run_relayout_gpu(Handle* h) {
    printf("case: relayout exec\n");
    fflush(stdout);
    auto rl = h->create_operator<RelayoutFormat>();
    struct { param::RelayoutFormat::Mode m; TensorShape s; uint32_t oc, group; float ss, sd; } rc[] = {
        {param::RelayoutFormat::Mode::NCHW_NCHW4, {3, 7, 9, 10}, 0, 1, 1.f, 1.f},
        {param::RelayoutFormat::Mode::NCHW_NCHW4, {3, 7, 9, 10}, 0, 1, 1.f, 2.f},
        {param::RelayoutFormat::Mode::NCHW4_NCHW, {2, 2, 5, 6, 4}, 7, 1, 1.f, 1.f},
        {param::RelayoutFormat::Mode::NCHW_NCHW32, {2, 40, 15, 16}, 0, 1, 1.f, 1.f},
        {param::RelayoutFormat::Mode::NCHW32_NCHW, {2, 2, 15, 16, 32}, 40, 1, 1.f, 1.f},
    };
    for (auto& r : rc) {
        rl->param().mode = r.m; rl->param().oc = r.oc; rl->param().group = r.group;
        TensorLayout s(r.s, dtype::QuantizedS8(r.ss)), o;
        o.dtype = dtype::QuantizedS8(r.sd);
        rl->deduce_layout(s, o);
        mi355_relayout_desc rd = mi355_relayout_desc();
        rd.mode = (uint32_t)r.m; rd.ndim = (uint32_t)r.s.ndim; rd.group = r.group; rd.oc = r.oc; rd.elem_bytes = 1;
        rd.scale_src = r.ss; rd.scale_dst = r.sd;
        for (size_t i = 0; i < r.s.ndim; ++i) rd.shape[i] = (uint32_t)r.s[i];
        std::vector<int8_t> hs(s.total_nr_elems()), want(o.total_nr_elems()), got(o.total_nr_elems());
        fill_s8(hs, 21, -128, 127);
        EXPECT(oracle_relayout(&rd, hs.data(), want.data()) == 0, "checker refused relayout");
        DevBuf ds(hs.size()), dd(want.size());
        HIP_OK(hipMemcpy(ds.p, hs.data(), hs.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemset(dd.p, 0x5a, want.size()));
        rl->exec(TensorND(ds.p, s), TensorND(dd.p, o), Workspace());
        HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
        HIP_OK(hipMemcpy(got.data(), dd.p, got.size(), hipMemcpyDeviceToHost));
        EXPECT(got == want, "relayout mode %u differs from the CPU checker", (unsigned)r.m);
    }
}

// ------------------------------------------------------------------ algorithm cache (no device)
static void run_cache_roundtrip() {
    printf("case: algorithm cache save / load\n");
    AlgorithmCache& c = AlgorithmCache::instance();
    c.clear();
    mi355_conv_desc a = mi355_conv_desc(), b = mi355_conv_desc();
    a.format = MI355_FMT_NCHW32; a.n = 64; a.ic = 256; a.ih = a.iw = 14; a.oc = 256; a.fh = a.fw = 3; a.group = 1;
    a.pad_h = a.pad_w = 1; a.stride_h = a.stride_w = 1; a.dilate_h = a.dilate_w = 1; a.scale_bias = 2e-4f; a.scale_dst = 0.05f;
    b = a; b.oc = 512;
    AlgorithmCache::Result ra, rb, got;
    ra.policy.algo.id = 1; ra.policy.algo.tile_cfg = 23; ra.workspace = 0; ra.usec = 15.25f;
    rb.policy.algo.id = 0; rb.policy.algo.tile_cfg = -1; rb.workspace = 64; rb.usec = 99.5f;
    c.put(a, ra); c.put(b, rb);
    EXPECT(c.size() == 2, "two entries expected");
    const std::string path = "/tmp/mi355_algo_cache_test.txt";
    c.save(path);
    c.clear();
    EXPECT(!c.get(a, got), "cleared cache must miss");
    EXPECT(c.load(path) == 2, "two entries must come back");
    EXPECT(c.get(a, got) && got.policy.algo.id == 1 && got.policy.algo.tile_cfg == 23 && got.usec == 15.25f, "entry a");
    EXPECT(c.get(b, got) && got.policy.algo.id == 0 && got.policy.algo.tile_cfg == -1 && got.workspace == 64, "entry b");
    b.oc = 1024;
    EXPECT(!c.get(b, got), "a different problem must miss");
    // a file of another format is ignored, a missing one is an error
    FILE* f = fopen(path.c_str(), "w");
    fputs("something else\n", f);
    fclose(f);
    c.clear();
    EXPECT(c.load(path) == 0 && c.size() == 0, "foreign file must load nothing");
    EXPECT(throws([&] { c.load("/nonexistent/dir/cache.txt"); }, MI355_ERR_BAD_ARG), "missing file");
    remove(path.c_str());
    c.clear();
}

// ------------------------------------------------------------------ elementwise requantisation (GPU)
extern "C" int oracle_requant_s32_s8(const mi355_requant_desc* d, const int32_t* src, const int8_t* z, int8_t* dst);
extern "C" int oracle_requant_s8_s8(const mi355_requant_desc* d, const int8_t* src, const int8_t* z, int8_t* dst);
extern "C" int oracle_elemwise_q(const mi355_elemwise_desc* d, const void* s0, const void* s1, const void* s2, void* dst);

static void run_elemwise_gpu(Handle* h) {
    printf("case: ElemwiseMultiType quantized modes and TypeCvt\n");
    fflush(stdout);
    using EM = ElemwiseMultiType::Param::Mode;
    const size_t n = 100003;  // ragged tail
    const TensorShape shp{n};
    std::vector<int8_t> ha(n), hb(n), expect(n), got(n);
    std::vector<int32_t> ha32(n);
    fill_s8(ha, 31, -128, 127);
    fill_s8(hb, 32, -128, 127);
    fill_s32(ha32, 33, -60000, 60000);
    DevBuf da(n), db(n), da32(n * 4), dd(n);
    HIP_OK(hipMemcpy(da.p, ha.data(), n, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(db.p, hb.data(), n, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(da32.p, ha32.data(), n * 4, hipMemcpyHostToDevice));
    const float s_a = 0.031f, s_b = 0.022f, s_d = 0.047f, s_acc = 2e-4f;
    TensorLayout la(shp, dtype::QuantizedS8(s_a)), lb(shp, dtype::QuantizedS8(s_b)), ld(shp, dtype::QuantizedS8(s_d));
    TensorLayout la32(shp, dtype::QuantizedS32(s_acc));
    auto opr = h->create_operator<ElemwiseMultiType>();
    struct M { EM mode; uint32_t nl; bool binary; const char* name; };
    const M modes[] = {{EM::QADD, MI355_NL_IDENTITY, true, "QADD"}, {EM::QFUSE_ADD_RELU, MI355_NL_RELU, true, "QFUSE_ADD_RELU"},
                       {EM::QFUSE_ADD_H_SWISH, MI355_NL_H_SWISH, true, "QFUSE_ADD_H_SWISH"}, {EM::QRELU, MI355_NL_RELU, false, "QRELU"},
                       {EM::QH_SWISH, MI355_NL_H_SWISH, false, "QH_SWISH"}};
    for (int s32 = 0; s32 < 2; ++s32)
        for (auto& m : modes) {
            mi355_requant_desc d = mi355_requant_desc();
            d.nonline = m.nl; d.has_z = m.binary; d.scale_src = s32 ? s_acc : s_a; d.scale_z = s_b; d.scale_dst = s_d; d.count = n;
            int st = s32 ? oracle_requant_s32_s8(&d, ha32.data(), m.binary ? hb.data() : nullptr, expect.data())
                         : oracle_requant_s8_s8(&d, ha.data(), m.binary ? hb.data() : nullptr, expect.data());
            EXPECT(st == 0, "CPU checker refused %s", m.name);
            opr->param().mode = m.mode;
            std::vector<TensorND> src{s32 ? TensorND(da32.p, la32) : TensorND(da.p, la)};
            if (m.binary) src.push_back(TensorND(db.p, lb));
            HIP_OK(hipMemset(dd.p, 0x5a, n));
            opr->exec(src, TensorND(dd.p, ld));
            HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
            HIP_OK(hipMemcpy(got.data(), dd.p, n, hipMemcpyDeviceToHost));
            size_t bad = 0;
            for (size_t i = 0; i < n; ++i) bad += got[i] != expect[i];
            EXPECT(bad == 0, "%s (%s first operand): %zu of %zu bytes differ", m.name, s32 ? "s32" : "s8", bad, n);
        }
    // TypeCvt s32 -> s8 and the wrong arity
    {
        mi355_requant_desc d = mi355_requant_desc();
        d.nonline = MI355_NL_IDENTITY; d.scale_src = s_acc; d.scale_z = 1.f; d.scale_dst = s_d; d.count = n;
        EXPECT(oracle_requant_s32_s8(&d, ha32.data(), nullptr, expect.data()) == 0, "CPU checker refused TypeCvt");
        auto cvt = h->create_operator<TypeCvt>();
        cvt->exec(TensorND(da32.p, la32), TensorND(dd.p, ld));
        HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
        HIP_OK(hipMemcpy(got.data(), dd.p, n, hipMemcpyDeviceToHost));
        size_t bad = 0;
        for (size_t i = 0; i < n; ++i) bad += got[i] != expect[i];
        EXPECT(bad == 0, "TypeCvt: %zu bytes differ", bad);
        opr->param().mode = EM::QADD;
        EXPECT(throws([&] { opr->exec({TensorND(da.p, la)}, TensorND(dd.p, ld)); }, MI355_ERR_BAD_ARG), "QADD with one operand");
    }
    // the general entry point: modes outside the post-process chain, three operands, a QuantizedS32 destination
    {
        std::vector<int8_t> hc(n);
        fill_s8(hc, 34, -128, 127);
        DevBuf dc(n), dd32(n * 4);
        HIP_OK(hipMemcpy(dc.p, hc.data(), n, hipMemcpyHostToDevice));
        const float s_c = 0.9f;
        TensorLayout lc(shp, dtype::QuantizedS8(s_c)), ld32(shp, dtype::QuantizedS32(0.004f));
        struct G { EM mode; uint32_t ew, arity; const char* name; };
        const G gm[] = {{EM::QMUL, MI355_EW_MUL, 2, "QMUL"}, {EM::QMAX, MI355_EW_MAX, 2, "QMAX"}, {EM::QTRUE_DIV, MI355_EW_TRUE_DIV, 2, "QTRUE_DIV"},
                        {EM::QFUSE_MUL_ADD3, MI355_EW_FUSE_MUL_ADD3, 3, "QFUSE_MUL_ADD3"}, {EM::QCOND_LEQ_MOV, MI355_EW_COND_LEQ_MOV, 3, "QCOND_LEQ_MOV"},
                        {EM::QABS, MI355_EW_ABS, 1, "QABS"}, {EM::QADD, MI355_EW_ADD, 2, "QADD"}};
        std::vector<int32_t> expect32(n), got32(n);
        for (int d32 = 0; d32 < 2; ++d32)
            for (auto& m : gm) {
                mi355_elemwise_desc d = mi355_elemwise_desc();
                d.mode = m.ew; d.arity = m.arity; d.src_dtype = MI355_DT_QS8; d.dst_dtype = d32 ? MI355_DT_QS32 : MI355_DT_QS8;
                d.scale_src[0] = s_a; d.scale_src[1] = s_b; d.scale_src[2] = s_c; d.scale_dst = d32 ? 0.004f : s_d; d.count = n;
                void* want = d32 ? (void*)expect32.data() : (void*)expect.data();
                EXPECT(oracle_elemwise_q(&d, ha.data(), hb.data(), hc.data(), want) == 0, "CPU checker refused %s", m.name);
                opr->param().mode = m.mode;
                std::vector<TensorND> src{TensorND(da.p, la)};
                if (m.arity > 1) src.push_back(TensorND(db.p, lb));
                if (m.arity > 2) src.push_back(TensorND(dc.p, lc));
                if (m.mode == EM::QADD && !d32) continue;  // the chain's case, covered above
                HIP_OK(hipMemset(d32 ? dd32.p : dd.p, 0x5a, d32 ? n * 4 : n));
                opr->exec(src, d32 ? TensorND(dd32.p, ld32) : TensorND(dd.p, ld));
                HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
                size_t bad = 0;
                if (d32) {
                    HIP_OK(hipMemcpy(got32.data(), dd32.p, n * 4, hipMemcpyDeviceToHost));
                    for (size_t i = 0; i < n; ++i) bad += got32[i] != expect32[i];
                } else {
                    HIP_OK(hipMemcpy(got.data(), dd.p, n, hipMemcpyDeviceToHost));
                    for (size_t i = 0; i < n; ++i) bad += got[i] != expect[i];
                }
                EXPECT(bad == 0, "%s (%s dst): %zu of %zu elements differ", m.name, d32 ? "s32" : "s8", bad, n);
            }
        opr->param().mode = (EM)18;  // QEXP: a libm mode
        EXPECT(throws([&] { opr->exec({TensorND(da.p, la)}, TensorND(dd.p, ld)); }, MI355_ERR_UNSUPPORTED), "QEXP is refused");
    }
}

// ------------------------------------------------------------------ Pooling and float TypeCvt (GPU)
extern "C" int oracle_pooling_s8(const mi355_pooling_desc* d, const int8_t* src, int8_t* dst);
extern "C" void oracle_typecvt_f32_s8(uint64_t n, float scale, const float* src, int8_t* dst);
extern "C" void oracle_typecvt_s8_f32(uint64_t n, float scale, const int8_t* src, float* dst);
static void run_pooling_gpu(Handle* h) {
    printf("case: PoolingForward and TypeCvt Float32 <-> QuantizedS8\n");
    fflush(stdout);
    using PM = PoolingForward::Mode;
    auto opr = h->create_operator<PoolingForward>();
    opr->param().format = param::Pooling::Format::NCHW32;
    opr->param().window_h = opr->param().window_w = 3;
    opr->param().stride_h = opr->param().stride_w = 2;
    opr->param().pad_h = opr->param().pad_w = 1;
    TensorLayout src({3, 2, 15, 17, 32}, dtype::QuantizedS8(0.05f)), dst;
    opr->deduce_layout(src, dst);
    EXPECT(dst.eq_shape(TensorShape{3, 2, 8, 9, 32}) && dst.dtype == src.dtype, "pooling deduce_layout: %s", dst.to_string().c_str());
    const size_t ns = src.total_nr_elems(), nd = dst.total_nr_elems();
    std::vector<int8_t> hs(ns), expect(nd), got(nd);
    fill_s8(hs, 41, -128, 127);
    DevBuf ds(ns), dd(nd);
    HIP_OK(hipMemcpy(ds.p, hs.data(), ns, hipMemcpyHostToDevice));
    for (PM mode : {PM::MAX, PM::AVERAGE, PM::AVERAGE_COUNT_EXCLUDE_PADDING}) {
        opr->param().mode = mode;
        mi355_pooling_desc d = mi355_pooling_desc();
        d.mode = (uint32_t)mode; d.format = MI355_FMT_NCHW32; d.n = 3; d.c = 64; d.ih = 15; d.iw = 17;
        d.pad_h = d.pad_w = 1; d.stride_h = d.stride_w = 2; d.window_h = d.window_w = 3;
        EXPECT(oracle_pooling_s8(&d, hs.data(), expect.data()) == 0, "CPU checker refused pooling mode %u", (unsigned)mode);
        HIP_OK(hipMemset(dd.p, 0x5a, nd));
        opr->exec(TensorND(ds.p, src), TensorND(dd.p, dst), Workspace());
        HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
        HIP_OK(hipMemcpy(got.data(), dd.p, nd, hipMemcpyDeviceToHost));
        size_t bad = 0;
        for (size_t i = 0; i < nd; ++i) bad += got[i] != expect[i];
        EXPECT(bad == 0, "pooling mode %u: %zu of %zu bytes differ", (unsigned)mode, bad, nd);
    }
    // a window in the padding only; a dst of another dtype
    opr->param().mode = PM::MAX;
    opr->param().pad_h = 3;
    TensorLayout far;
    opr->deduce_layout(src, far);
    DevBuf dfar(far.total_nr_elems());
    EXPECT(throws([&] { opr->exec(TensorND(ds.p, src), TensorND(dfar.p, far), Workspace()); }, MI355_ERR_SHAPE),
           "window outside the image completely");
    opr->param().pad_h = 1;
    TensorLayout other(dst, dtype::QuantizedS8(0.07f));
    EXPECT(throws([&] { opr->exec(TensorND(ds.p, src), TensorND(dd.p, other), Workspace()); }, MI355_ERR_BAD_ARG), "dst scale differs");

    // TypeCvt Float32 -> QuantizedS8 -> Float32
    const size_t n = 100003;
    std::vector<float> hf(n), backf(n), expf(n);
    std::vector<int8_t> q(n), expq(n);
    for (size_t i = 0; i < n; ++i) hf[i] = ((float)((i * 2654435761u) % 20001u) - 10000.f) * 7e-4f;
    hf[0] = INFINITY; hf[1] = -INFINITY; hf[2] = NAN; hf[3] = 0.5f * 0.05f; hf[4] = -0.5f * 0.05f;
    DevBuf df(n * 4), dq(n), db(n * 4);
    HIP_OK(hipMemcpy(df.p, hf.data(), n * 4, hipMemcpyHostToDevice));
    const TensorShape shp{n};
    TensorLayout lf(shp, dtype::Float32()), lq(shp, dtype::QuantizedS8(0.05f));
    auto cvt = h->create_operator<TypeCvt>();
    cvt->exec(TensorND(df.p, lf), TensorND(dq.p, lq));
    cvt->exec(TensorND(dq.p, lq), TensorND(db.p, lf));
    HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
    HIP_OK(hipMemcpy(q.data(), dq.p, n, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(backf.data(), db.p, n * 4, hipMemcpyDeviceToHost));
    oracle_typecvt_f32_s8(n, 0.05f, hf.data(), expq.data());
    oracle_typecvt_s8_f32(n, 0.05f, expq.data(), expf.data());
    size_t bad = 0;
    for (size_t i = 0; i < n; ++i) bad += q[i] != expq[i] || memcmp(&backf[i], &expf[i], 4) != 0;
    EXPECT(bad == 0, "TypeCvt float: %zu of %zu elements differ", bad, n);
}

// ------------------------------------------------------------------ fast-run (GPU)
static void run_fast_run_gpu(Handle* h) {
    printf("case: fast-run profiling\n");
    fflush(stdout);
    AlgorithmCache::instance().clear();
    auto opr = h->create_operator<ConvBiasForward>();
    opr->param().format = CB::Format::NCHW32;
    opr->param().nonlineMode = CB::NonlineMode::RELU;
    opr->param().pad_h = opr->param().pad_w = 1;
    const float s_src = 0.02f, s_flt = 0.01f, s_dst = 0.05f;
    TensorLayout src({4, 4, 14, 14, 32}, dtype::QuantizedS8(s_src)), flt({128, 4, 3, 3, 32}, dtype::QuantizedS8(s_flt));
    TensorLayout bias({1, 4, 1, 1, 32}, dtype::QuantizedS32(s_src * s_flt)), z, dst;
    dst.dtype = dtype::QuantizedS8(s_dst);
    opr->deduce_layout(src, flt, bias, z, dst);
    std::vector<int8_t> hsrc(src.total_nr_elems()), hflt(flt.total_nr_elems());
    std::vector<int32_t> hbias(bias.total_nr_elems());
    fill_s8(hsrc, 21, -128, 127);
    fill_s8(hflt, 22, -127, 127);
    fill_s32(hbias, 23, -1000, 1000);
    mi355_conv_desc d = mi355_conv_desc();
    d.format = MI355_FMT_NCHW32; d.nonline = MI355_NL_RELU; d.n = 4; d.ic = 128; d.ih = d.iw = 14; d.oc = 128; d.fh = d.fw = 3;
    d.group = 1; d.pad_h = d.pad_w = 1; d.stride_h = d.stride_w = 1; d.dilate_h = d.dilate_w = 1;
    d.bias_mode = MI355_BIAS_BROADCAST_CHANNEL; d.scale_bias = s_src * s_flt; d.scale_z = 1.f; d.scale_dst = s_dst;
    std::vector<int8_t> expect(dst.total_nr_elems()), got(dst.total_nr_elems());
    EXPECT(oracle_convbias_s8(&d, hsrc.data(), hflt.data(), hbias.data(), nullptr, expect.data()) == 0, "CPU checker");
    DevBuf dsrc(hsrc.size()), dflt(hflt.size()), dbias(hbias.size() * 4), ddst(got.size()), dws(16);
    HIP_OK(hipMemcpy(dsrc.p, hsrc.data(), hsrc.size(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dflt.p, hflt.data(), hflt.size(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dbias.p, hbias.data(), hbias.size() * 4, hipMemcpyHostToDevice));

    auto timed = opr->profile_algorithms(TensorND(dsrc.p, src), TensorND(dflt.p, flt), TensorND(dbias.p, bias), TensorND(nullptr, z),
                                         TensorND(ddst.p, dst), Workspace(dws.p, 0), 1, 5);
    EXPECT(timed.size() >= 2, "several algorithms must have been timed, got %zu", timed.size());
    for (size_t i = 1; i < timed.size(); ++i) EXPECT(timed[i - 1].second <= timed[i].second, "results must be sorted");
    printf("  %zu algorithms timed, fastest %s %.2f us, slowest %s %.2f us\n", timed.size(), timed.front().first.name.c_str(),
           timed.front().second, timed.back().first.name.c_str(), timed.back().second);
    EXPECT(AlgorithmCache::instance().size() == 1, "the winner must be cached");

    // the PROFILE strategy takes the cached winner and must still be bit-exact
    opr->execution_policy().strategy = ExecutionPolicy::Strategy::PROFILE;
    HIP_OK(hipMemset(ddst.p, 0x5a, got.size()));
    opr->exec(TensorND(dsrc.p, src), TensorND(dflt.p, flt), TensorND(dbias.p, bias), TensorND(nullptr, z), TensorND(ddst.p, dst),
              nullptr, Workspace(dws.p, 0));
    HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
    HIP_OK(hipMemcpy(got.data(), ddst.p, got.size(), hipMemcpyDeviceToHost));
    size_t bad = 0;
    for (size_t i = 0; i < got.size(); ++i) bad += got[i] != expect[i];
    EXPECT(bad == 0, "fast-run exec: %zu bytes differ", bad);
    // a problem not seen before is profiled on first use
    AlgorithmCache::instance().clear();
    opr->exec(TensorND(dsrc.p, src), TensorND(dflt.p, flt), TensorND(dbias.p, bias), TensorND(nullptr, z), TensorND(ddst.p, dst),
              nullptr, Workspace(dws.p, 0));
    HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
    EXPECT(AlgorithmCache::instance().size() == 1, "first use under PROFILE must fill the cache");
    HIP_OK(hipMemcpy(got.data(), ddst.p, got.size(), hipMemcpyDeviceToHost));
    bad = 0;
    for (size_t i = 0; i < got.size(); ++i) bad += got[i] != expect[i];
    EXPECT(bad == 0, "fast-run first use: %zu bytes differ", bad);
    AlgorithmCache::instance().clear();
}

// weight pre-processing: deduce_preprocessed_filter_layout -> exec_preprocess -> exec with the PreprocessedFilter, the way the
// reference's OprProxy drives it (dnn/test/common/opr_proxy.h, "weight preprocess" proxies)
static void run_preprocess_gpu(Handle* h) {
    printf("case: weight pre-processing\n");
    fflush(stdout);
    const float s_src = 0.02f, s_flt = 0.01f, s_dst = 0.05f;
    for (int variant = 0; variant < 3; ++variant) {
        auto opr = h->create_operator<ConvBiasForward>();
        opr->param().format = CB::Format::NCHW32;
        opr->param().nonlineMode = variant == 1 ? CB::NonlineMode::H_SWISH : CB::NonlineMode::RELU;
        const bool pw = variant == 2;
        opr->param().pad_h = opr->param().pad_w = pw ? 0 : 1;
        opr->execution_policy().weight_preprocess = true;
        TensorLayout src({3, 4, 14, 14, 32}, dtype::QuantizedS8(s_src));
        TensorLayout flt(pw ? TensorShape{160, 4, 1, 1, 32} : TensorShape{160, 4, 3, 3, 32}, dtype::QuantizedS8(s_flt));
        TensorLayout bias({1, 5, 1, 1, 32}, dtype::QuantizedS32(s_src * s_flt)), z, dst;
        dst.dtype = dtype::QuantizedS8(s_dst);
        opr->deduce_layout(src, flt, bias, z, dst);
        std::vector<int8_t> hsrc(src.total_nr_elems()), hflt(flt.total_nr_elems());
        std::vector<int32_t> hbias(bias.total_nr_elems());
        fill_s8(hsrc, 31 + variant, -128, 127);
        fill_s8(hflt, 32 + variant, -127, 127);
        fill_s32(hbias, 33 + variant, -1000, 1000);
        mi355_conv_desc d = mi355_conv_desc();
        d.format = MI355_FMT_NCHW32; d.nonline = (uint32_t)opr->param().nonlineMode; d.n = 3; d.ic = 128; d.ih = d.iw = 14;
        d.oc = 160; d.fh = d.fw = pw ? 1 : 3; d.group = 1; d.pad_h = d.pad_w = pw ? 0 : 1; d.stride_h = d.stride_w = 1;
        d.dilate_h = d.dilate_w = 1; d.bias_mode = MI355_BIAS_BROADCAST_CHANNEL; d.scale_bias = s_src * s_flt; d.scale_z = 1.f;
        d.scale_dst = s_dst;
        std::vector<int8_t> expect(dst.total_nr_elems()), got(dst.total_nr_elems());
        EXPECT(oracle_convbias_s8(&d, hsrc.data(), hflt.data(), hbias.data(), nullptr, expect.data()) == 0, "CPU checker");
        DevBuf dsrc(hsrc.size()), dflt(hflt.size()), dbias(hbias.size() * 4), ddst(got.size()), dws(16);
        HIP_OK(hipMemcpy(dsrc.p, hsrc.data(), hsrc.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dflt.p, hflt.data(), hflt.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dbias.p, hbias.data(), hbias.size() * 4, hipMemcpyHostToDevice));

        EXPECT(opr->get_preprocess_workspace_in_bytes(src, flt, bias, z, dst) == 0, "no pre-processing workspace");
        auto layouts = opr->deduce_preprocessed_filter_layout(src, flt, bias, z, dst);
        EXPECT(layouts.size() == 1, "the heuristic for pre-processing callers must pick an algorithm with a pre-processed filter");
        if (layouts.size() != 1) return;
        EXPECT(layouts[0].total_nr_elems() >= flt.total_nr_elems(), "the re-tiled filter holds every filter byte");
        DevBuf dpre(layouts[0].total_nr_elems());
        HIP_OK(hipMemset(dpre.p, 0x77, layouts[0].total_nr_elems()));
        ConvBiasForward::PreprocessedFilter pf;
        pf.tensors.push_back(TensorND(dpre.p, layouts[0]));
        opr->exec_preprocess(src, TensorND(dflt.p, flt), TensorND(dbias.p, bias), z, dst, &pf, Workspace(dws.p, 0));
        // exec must not touch the filter any more: poison it
        HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
        HIP_OK(hipMemset(dflt.p, 0x33, hflt.size()));
        HIP_OK(hipMemset(ddst.p, 0x5a, got.size()));
        opr->exec(TensorND(dsrc.p, src), TensorND(dflt.p, flt), TensorND(dbias.p, bias), TensorND(nullptr, z), TensorND(ddst.p, dst),
                  &pf, Workspace(dws.p, 0));
        HIP_OK(hipStreamSynchronize((hipStream_t)h->stream()));
        HIP_OK(hipMemcpy(got.data(), ddst.p, got.size(), hipMemcpyDeviceToHost));
        size_t bad = 0;
        for (size_t i = 0; i < got.size(); ++i) bad += got[i] != expect[i];
        EXPECT(bad == 0, "exec with a PreprocessedFilter (variant %d): %zu bytes differ from the CPU checker", variant, bad);
        // a PreprocessedFilter with the wrong tensor count is refused
        ConvBiasForward::PreprocessedFilter empty;
        EXPECT(throws([&] { opr->exec_preprocess(src, TensorND(dflt.p, flt), TensorND(dbias.p, bias), z, dst, &empty,
                                                 Workspace(dws.p, 0)); }, MI355_ERR_BAD_ARG),
               "exec_preprocess must refuse a PreprocessedFilter without the deduced tensor");
    }
    // an algorithm that reads the reference layout only: nothing to hoist (the naive backend's answer)
    auto opr = h->create_operator<ConvBiasForward>();
    opr->param().format = CB::Format::NCHW4;
    opr->param().pad_h = opr->param().pad_w = 1;
    TensorLayout src({1, 4, 8, 8, 4}, dtype::QuantizedS8(s_src)), flt({16, 4, 3, 3, 4}, dtype::QuantizedS8(s_flt));
    TensorLayout bias({1, 4, 1, 1, 4}, dtype::QuantizedS32(s_src * s_flt)), z, dst;
    dst.dtype = dtype::QuantizedS8(s_dst);
    opr->deduce_layout(src, flt, bias, z, dst);
    EXPECT(opr->deduce_preprocessed_filter_layout(src, flt, bias, z, dst).empty(), "4-packed inputs have no pre-processed form");
}

int main(int argc, char** argv) {
    bool gpu = argc > 1 && !strcmp(argv[1], "--gpu");
    bool cpu = argc > 1 && !strcmp(argv[1], "--cpu");
    if (!gpu && !cpu) {
        printf("usage: host_checker --cpu | --gpu\n");
        return 2;
    }
    hipStream_t stream = nullptr;
    if (gpu) {
        HIP_OK(hipSetDevice(0));
        HIP_OK(hipStreamCreate(&stream));
    }
    try {
        auto handle = Handle::make(stream, 0);
        if (gpu) handle->check_device();
        run_validation(handle.get());
        run_cache_roundtrip();
        for (auto& c : cases()) run_conv_case(handle.get(), c, gpu);
        if (gpu) run_relayout_gpu(handle.get());
        if (gpu) run_elemwise_gpu(handle.get());
        if (gpu) run_pooling_gpu(handle.get());
        if (gpu) run_fast_run_gpu(handle.get());
        if (gpu) run_preprocess_gpu(handle.get());
    } catch (const Error& e) {
        printf("unexpected mi355dnn::Error %d: %s\n", e.status(), e.what());
        return 1;
    }
    if (gpu) HIP_OK(hipStreamDestroy(stream));
    if (g_fail) {
        printf("%d FAILURES\n", g_fail);
        return 1;
    }
    printf("ALL OK\n");
    return 0;
}
