// Implementation of the host-side operator classes over the C ABI.  Shape and dtype rules
// follow the reference's common layer; each block cites the rule it restates.
#include "mi355dnn.h"

#include <math.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <fstream>
#include <map>
#include <mutex>
#include <sstream>

#include "../../include/mi355_convbias.h"

namespace mi355dnn {

namespace {

[[noreturn]] void fail(int status, const std::string& msg) {
    throw Error(status, std::string(mi355_status_string(status)) + ": " + msg);
}

void check_abi(int status) {
    if (status != MI355_OK) {
        const char* m = mi355_last_error();
        throw Error(status, std::string(mi355_status_string(status)) + ": " + (m ? m : ""));
    }
}

#define HOST_ASSERT(cond, status, ...)                       \
    do {                                                     \
        if (!(cond)) {                                       \
            char buf_[512];                                  \
            snprintf(buf_, sizeof(buf_), __VA_ARGS__);       \
            fail(status, std::string(buf_) + " (" #cond ")"); \
        }                                                    \
    } while (0)

using Format = param::ConvBias::Format;

bool format_supported(Format f) {
    switch (f) {
        case Format::NCHW: case Format::NCHW4: case Format::NCHW32: case Format::NCHW44:
        case Format::NCHW4_NCHW32: case Format::NCHW32_NCHW4: case Format::NCHW4_NCHW:
            return true;
        default:
            return false;
    }
}
size_t in_pack(Format f) {
    switch (f) {
        case Format::NCHW: return 1;
        case Format::NCHW32: case Format::NCHW32_NCHW4: return 32;
        default: return 4;
    }
}
size_t out_pack(Format f) {
    switch (f) {
        case Format::NCHW: case Format::NCHW4_NCHW: return 1;
        case Format::NCHW32: case Format::NCHW4_NCHW32: return 32;
        default: return 4;
    }
}

}  // namespace

// ---------------------------------------------------------------- shapes / layouts
TensorShape::TensorShape(std::initializer_list<size_t> s) {
    if (s.size() > MAX_NDIM) fail(MI355_ERR_BAD_ARG, "too many dimensions");
    ndim = 0;
    for (size_t v : s) shape[ndim++] = v;
}
size_t TensorShape::total_nr_elems() const {
    if (!ndim) return 0;
    size_t r = 1;
    for (size_t i = 0; i < ndim; ++i) r *= shape[i];
    return r;
}
bool TensorShape::eq_shape(const TensorShape& o) const {
    if (ndim != o.ndim) return false;
    for (size_t i = 0; i < ndim; ++i)
        if (shape[i] != o.shape[i]) return false;
    return true;
}
std::string TensorShape::to_string() const {
    std::string s = "{";
    for (size_t i = 0; i < ndim; ++i) s += (i ? "," : "") + std::to_string(shape[i]);
    return s + "}";
}
TensorLayout::TensorLayout(const TensorShape& sh, DType dt) : TensorShape(sh), dtype(dt) { init_contiguous_stride(); }
void TensorLayout::init_contiguous_stride() {
    ptrdiff_t s = 1;
    for (size_t i = ndim; i-- > 0;) {
        stride[i] = s;
        s *= (ptrdiff_t)shape[i];
    }
}
bool TensorLayout::is_contiguous() const {
    ptrdiff_t s = 1;
    for (size_t i = ndim; i-- > 0;) {
        if (shape[i] != 1 && stride[i] != s) return false;
        s *= (ptrdiff_t)shape[i];
    }
    return true;
}
bool TensorLayout::is_batch_strided() const {
    ptrdiff_t s = 1;
    for (size_t i = ndim; i-- > 1;) {
        if (shape[i] != 1 && stride[i] != s) return false;
        s *= (ptrdiff_t)shape[i];
    }
    return ndim == 0 || shape[0] == 1 || stride[0] >= s;
}
size_t TensorLayout::span_bytes() const {
    if (!ndim) return 0;
    size_t last = 0;
    for (size_t i = 0; i < ndim; ++i) last += (shape[i] - 1) * (size_t)stride[i];
    return (last + 1) * dtype.size();
}

// ---------------------------------------------------------------- handle
std::unique_ptr<Handle> Handle::make(void* stream, int device) {
    return std::unique_ptr<Handle>(new Handle(stream, device));
}
int Handle::abi_version() { return mi355_abi_version(); }
void Handle::check_device() const {
    mi355_device_info info;
    check_abi(mi355_get_device_info(m_device, &info));
}

// ---------------------------------------------------------------- ConvBias
struct ConvBiasForward::Canon {
    mi355_conv_desc d;
    TensorShape dst_shape;
};

ConvBiasForward::BiasMode ConvBiasForward::bias_mode_of(const TensorLayout& bias, const TensorLayout& dst) {
    if (bias.ndim == 0) return BiasMode::NO_BIAS;
    if (bias.eq_shape(dst)) return BiasMode::BIAS;
    return BiasMode::BROADCAST_CHANNEL_BIAS;
}

void ConvBiasForward::deduce_dtype(DType src, DType filter, DType, DType, DType& dst) const {
    // dnn/src/common/convolution.cpp:545-631: s8 x s8 gives QuantizedS32(s_src * s_flt) by default and
    // accepts a caller-named QuantizedS8 of any scale
    HOST_ASSERT(src.enumv == DTypeEnum::QuantizedS8 && filter.enumv == DTypeEnum::QuantizedS8, MI355_ERR_UNSUPPORTED,
                "this backend implements QuantizedS8 x QuantizedS8 ConvBias only");
    if (dst.enumv == DTypeEnum::QuantizedS8) return;
    // NCHW4_NCHW may also dequantise into a Float32 dst (convolution.cpp:1051-1140)
    if (dst.enumv == DTypeEnum::Float32 && m_param.format == Format::NCHW4_NCHW) return;
    dst = dtype::QuantizedS32(src.scale * filter.scale);
}

void ConvBiasForward::canonize(const TensorLayout& src, const TensorLayout& filter, const TensorLayout& bias,
                               const TensorLayout& z, const TensorLayout& dst, Canon& out, bool need_dst) const {
    const Param& p = m_param;
    HOST_ASSERT(format_supported(p.format), MI355_ERR_UNSUPPORTED, "format %u is not implemented", (unsigned)p.format);
    HOST_ASSERT(p.nonlineMode != Param::NonlineMode::SIGMOID, MI355_ERR_UNSUPPORTED,
                "SIGMOID is not defined for quantized ConvBias");  // naive/conv_bias/opr_impl.cpp:79-88
    HOST_ASSERT(src.dtype.enumv == DTypeEnum::QuantizedS8 && filter.dtype.enumv == DTypeEnum::QuantizedS8,
                MI355_ERR_UNSUPPORTED, "src and filter must be QuantizedS8");
    const size_t pi = in_pack(p.format), po = out_pack(p.format);
    const bool packed = p.format != Format::NCHW;
    HOST_ASSERT(src.ndim == (packed ? 5u : 4u), MI355_ERR_SHAPE, "src %s has the wrong rank for the format",
                src.to_string().c_str());
    if (packed) HOST_ASSERT(src[4] == pi, MI355_ERR_SHAPE, "src %s: innermost axis must be %zu", src.to_string().c_str(), pi);
    HOST_ASSERT(src.is_batch_strided() && filter.is_contiguous(), MI355_ERR_UNSUPPORTED,
                "src must be contiguous within an image and filter contiguous");

    mi355_conv_desc& d = out.d;
    d = mi355_conv_desc();
    d.format = (uint32_t)p.format;
    d.sparse = (uint32_t)p.sparse;
    d.nonline = (uint32_t)p.nonlineMode;
    d.mode = (uint32_t)p.mode;
    d.pad_h = p.pad_h; d.pad_w = p.pad_w; d.stride_h = p.stride_h; d.stride_w = p.stride_w;
    d.dilate_h = p.dilate_h; d.dilate_w = p.dilate_w;
    d.n = (uint32_t)src[0];
    d.ic = (uint32_t)(src[1] * pi);
    d.ih = (uint32_t)src[2];
    d.iw = (uint32_t)src[3];

    // filter meta: dnn/src/common/convolution.cpp:33-94 (NCHW), :357-418 (NCHW4/NCHW32), :241-310 (NCHW44)
    const bool grp = p.sparse == Param::Sparse::GROUP;
    size_t g = 1, ocpg, icpg, fh, fw;
    if (p.format == Format::NCHW) {
        HOST_ASSERT(filter.ndim == (grp ? 5u : 4u), MI355_ERR_SHAPE, "filter %s: bad rank", filter.to_string().c_str());
        const size_t o = grp ? 1 : 0;
        if (grp) g = filter[0];
        ocpg = filter[o]; icpg = filter[o + 1]; fh = filter[o + 2]; fw = filter[o + 3];
    } else if (p.format == Format::NCHW44) {
        if (grp && filter.ndim == 6) {  // channel-wise: (G/4, 1, 1, FH, FW, 4)
            HOST_ASSERT(filter[1] == 1 && filter[2] == 1 && filter[5] == 4, MI355_ERR_SHAPE,
                        "filter %s is not a channel-wise NCHW44 filter", filter.to_string().c_str());
            g = filter[0] * 4; ocpg = icpg = 1; fh = filter[3]; fw = filter[4];
        } else {
            HOST_ASSERT(filter.ndim == (grp ? 7u : 6u), MI355_ERR_SHAPE, "filter %s: bad rank", filter.to_string().c_str());
            const size_t o = grp ? 1 : 0;
            if (grp) g = filter[0];
            HOST_ASSERT(filter[o + 4] == 4 && filter[o + 5] == 4, MI355_ERR_SHAPE, "filter %s: inner axes must be 4,4",
                        filter.to_string().c_str());
            ocpg = filter[o] * 4; icpg = filter[o + 1] * 4; fh = filter[o + 2]; fw = filter[o + 3];
        }
    } else {
        HOST_ASSERT(filter.ndim == (grp ? 6u : 5u), MI355_ERR_SHAPE, "filter %s: bad rank", filter.to_string().c_str());
        const size_t o = grp ? 1 : 0;
        if (grp) g = filter[0];
        HOST_ASSERT(filter[o + 4] == pi, MI355_ERR_SHAPE, "filter %s: innermost axis must be %zu",
                    filter.to_string().c_str(), pi);
        ocpg = filter[o]; icpg = filter[o + 1] * pi; fh = filter[o + 2]; fw = filter[o + 3];
        HOST_ASSERT(p.dilate_h == 1 && p.dilate_w == 1, MI355_ERR_UNSUPPORTED,
                    "dilation must be 1 for channel-packed formats");  // convolution.cpp:411-414
    }
    HOST_ASSERT(icpg * g == d.ic, MI355_ERR_SHAPE, "group %zu x icpg %zu does not match %u input channels", g, icpg, d.ic);
    d.group = (uint32_t)g;
    d.oc = (uint32_t)(ocpg * g);
    d.fh = (uint32_t)fh;
    d.fw = (uint32_t)fw;
    HOST_ASSERT(d.oc % po == 0, MI355_ERR_SHAPE, "%u output channels are not a multiple of %zu", d.oc, po);

    uint32_t oh = 0, ow = 0;
    check_abi(mi355_convbias_deduce_out(&d, &oh, &ow));
    const bool dst_packed = po != 1;
    out.dst_shape = dst_packed ? TensorShape{d.n, d.oc / po, oh, ow, po} : TensorShape{d.n, d.oc, oh, ow};

    // dtypes and the bias / z rules of dnn/src/common/conv_bias.cpp:8-133
    const float s_acc = src.dtype.scale * filter.dtype.scale;
    d.scale_bias = s_acc;
    const bool f32 = need_dst && dst.dtype.enumv == DTypeEnum::Float32;
    if (f32) {
        HOST_ASSERT(p.format == Format::NCHW4_NCHW, MI355_ERR_UNSUPPORTED, "a Float32 dst needs format NCHW4_NCHW");
        HOST_ASSERT(bias.ndim == 0 || bias.dtype.enumv == DTypeEnum::Float32, MI355_ERR_BAD_ARG,
                    "a Float32 dst takes a Float32 bias");
    } else if (bias.dtype.enumv == DTypeEnum::QuantizedS32) {
        HOST_ASSERT(fabsf(s_acc - bias.dtype.scale) < 1e-6f, MI355_ERR_BAD_ARG,
                    "bias scale %g differs from src scale * filter scale = %g", bias.dtype.scale, s_acc);
        d.scale_bias = bias.dtype.scale;
    } else {
        HOST_ASSERT(bias.ndim == 0, MI355_ERR_BAD_ARG, "bias must be QuantizedS32");
    }
    if (!need_dst) return;

    HOST_ASSERT(dst.eq_shape(out.dst_shape), MI355_ERR_SHAPE, "dst %s, expected %s", dst.to_string().c_str(),
                out.dst_shape.to_string().c_str());
    HOST_ASSERT(dst.dtype.enumv == DTypeEnum::QuantizedS8 || dst.dtype.enumv == DTypeEnum::QuantizedS32 || f32,
                MI355_ERR_UNSUPPORTED, "dst must be QuantizedS8, QuantizedS32 or (NCHW4_NCHW) Float32");
    HOST_ASSERT(dst.is_batch_strided(), MI355_ERR_UNSUPPORTED, "dst must be contiguous within an image");
    d.dst_dtype = f32 ? MI355_DT_F32 : dst.dtype.enumv == DTypeEnum::QuantizedS8 ? MI355_DT_QS8 : MI355_DT_QS32;
    d.scale_dst = dst.dtype.scale;
    switch (bias_mode_of(bias, dst)) {
        case BiasMode::NO_BIAS: d.bias_mode = MI355_BIAS_NONE; break;
        case BiasMode::BIAS: d.bias_mode = MI355_BIAS_FULL; break;
        default: {
            TensorShape want = dst_packed ? TensorShape{1, d.oc / po, 1, 1, po} : TensorShape{1, d.oc, 1, 1};
            HOST_ASSERT(bias.eq_shape(want), MI355_ERR_SHAPE, "bias %s, expected %s or the dst shape",
                        bias.to_string().c_str(), want.to_string().c_str());
            d.bias_mode = MI355_BIAS_BROADCAST_CHANNEL;
        }
    }
    if (bias.ndim) HOST_ASSERT(bias.is_contiguous(), MI355_ERR_UNSUPPORTED, "bias must be contiguous");
    d.has_z = z.ndim != 0;
    d.scale_z = 1.f;
    if (d.has_z) {
        HOST_ASSERT(z.dtype.enumv == dst.dtype.enumv, MI355_ERR_BAD_ARG, "z and dst must have the same dtype kind");
        HOST_ASSERT(z.eq_shape(dst), MI355_ERR_SHAPE, "z %s must have the dst shape %s", z.to_string().c_str(),
                    dst.to_string().c_str());
        HOST_ASSERT(z.is_batch_strided(), MI355_ERR_UNSUPPORTED, "z must be contiguous within an image");
        d.scale_z = z.dtype.scale;
        d.z_stride_n = z.stride[0];
    }
    if (f32) {  // the C ABI carries the scales of src and filter in these two fields for a Float32 dst
        d.scale_bias = src.dtype.scale;
        d.scale_z = filter.dtype.scale;
    }
    d.src_stride_n = src.is_contiguous() ? 0 : src.stride[0];
    d.dst_stride_n = dst.is_contiguous() ? 0 : dst.stride[0];
    if (d.has_z && z.is_contiguous()) d.z_stride_n = 0;
}

void ConvBiasForward::deduce_layout(const TensorLayout& src, const TensorLayout& filter, const TensorLayout& bias,
                                    const TensorLayout& z, TensorLayout& dst) const {
    Canon c;
    canonize(src, filter, bias, z, dst, c, false);
    DType dt = dst.dtype;
    deduce_dtype(src.dtype, filter.dtype, bias.dtype, z.dtype, dt);
    dst = TensorLayout(c.dst_shape, dt);
}

// ---------------------------------------------------------------- algorithm cache
struct AlgorithmCache::Impl {
    mutable std::mutex mu;
    std::map<std::string, Result> map;
    static std::string key_of(const mi355_conv_desc& d) {
        return std::string(reinterpret_cast<const char*>(&d), sizeof(d));
    }
};
AlgorithmCache& AlgorithmCache::instance() {
    static AlgorithmCache c;
    return c;
}
AlgorithmCache::Impl& AlgorithmCache::impl() const {
    static Impl i;
    return i;
}
void AlgorithmCache::put(const mi355_conv_desc& key, const Result& r) {
    Impl& i = impl();
    std::lock_guard<std::mutex> lk(i.mu);
    i.map[Impl::key_of(key)] = r;
}
bool AlgorithmCache::get(const mi355_conv_desc& key, Result& r) const {
    Impl& i = impl();
    std::lock_guard<std::mutex> lk(i.mu);
    auto it = i.map.find(Impl::key_of(key));
    if (it == i.map.end()) return false;
    r = it->second;
    return true;
}
void AlgorithmCache::clear() {
    Impl& i = impl();
    std::lock_guard<std::mutex> lk(i.mu);
    i.map.clear();
}
size_t AlgorithmCache::size() const {
    Impl& i = impl();
    std::lock_guard<std::mutex> lk(i.mu);
    return i.map.size();
}
void AlgorithmCache::save(const std::string& path) const {
    Impl& i = impl();
    std::lock_guard<std::mutex> lk(i.mu);
    std::ofstream f(path, std::ios::trunc);
    if (!f) fail(MI355_ERR_BAD_ARG, "cannot write the algorithm cache to " + path);
    f << "mi355-algorithm-cache 1 " << sizeof(mi355_conv_desc) << " " << mi355_abi_version() << "\n";
    static const char* hex = "0123456789abcdef";
    for (auto& kv : i.map) {
        for (unsigned char ch : kv.first) f << hex[ch >> 4] << hex[ch & 15];
        f << ' ' << kv.second.policy.algo.id << ' ' << kv.second.policy.algo.tile_cfg << ' ' << kv.second.workspace << ' '
          << kv.second.usec << "\n";
    }
}
size_t AlgorithmCache::load(const std::string& path) {
    std::ifstream f(path);
    if (!f) fail(MI355_ERR_BAD_ARG, "cannot read the algorithm cache from " + path);
    std::string magic;
    size_t ver = 0, desc_bytes = 0;
    int abi = 0;
    f >> magic >> ver >> desc_bytes >> abi;
    // a cache written for another descriptor layout or ABI revision names algorithms this library may not have
    if (magic != "mi355-algorithm-cache" || ver != 1 || desc_bytes != sizeof(mi355_conv_desc) || abi != mi355_abi_version())
        return 0;
    Impl& i = impl();
    std::lock_guard<std::mutex> lk(i.mu);
    size_t n = 0;
    std::string hexkey;
    Result r;
    while (f >> hexkey >> r.policy.algo.id >> r.policy.algo.tile_cfg >> r.workspace >> r.usec) {
        if (hexkey.size() != 2 * sizeof(mi355_conv_desc)) continue;
        std::string key(sizeof(mi355_conv_desc), '\0');
        bool ok = true;
        for (size_t b = 0; b < key.size() && ok; ++b) {
            auto nib = [&](char ch) -> int {
                if (ch >= '0' && ch <= '9') return ch - '0';
                if (ch >= 'a' && ch <= 'f') return ch - 'a' + 10;
                ok = false;
                return 0;
            };
            key[b] = (char)((nib(hexkey[2 * b]) << 4) | nib(hexkey[2 * b + 1]));
        }
        if (!ok || r.policy.algo.id < 0 || r.policy.algo.id >= mi355_convbias_algo_count() ||
            r.policy.algo.tile_cfg >= mi355_igemm_tile_count())
            continue;
        i.map[key] = r;
        ++n;
    }
    return n;
}

static mi355_algo resolve_algo(const mi355_conv_desc& d, const ExecutionPolicy& pol, size_t* ws) {
    // fast-run: a recorded winner replaces the heuristic
    AlgorithmCache::Result hit;
    if (!pol.valid() && pol.strategy == ExecutionPolicy::Strategy::PROFILE && AlgorithmCache::instance().get(d, hit)) {
        mi355_algo a;
        check_abi(mi355_convbias_s8_query(&d, hit.policy.algo.id, &a, ws));
        if (hit.policy.algo.tile_cfg >= 0) a.tile_cfg = hit.policy.algo.tile_cfg;
        return a;
    }
    mi355_algo a;
    const int heur = pol.weight_preprocess ? MI355_ALGO_HEURISTIC_PREPROCESS : MI355_ALGO_HEURISTIC;
    check_abi(mi355_convbias_s8_query(&d, pol.valid() ? pol.algo.id : heur, &a, ws));
    if (pol.valid() && pol.algo.tile_cfg >= 0) {
        if (pol.algo.tile_cfg >= mi355_igemm_tile_count()) fail(MI355_ERR_ALGO, "unknown tile configuration");
        a.tile_cfg = pol.algo.tile_cfg;
    }
    return a;
}

size_t ConvBiasForward::get_workspace_in_bytes(const TensorLayout& src, const TensorLayout& filter,
                                               const TensorLayout& bias, const TensorLayout& z,
                                               const TensorLayout& dst, const PreprocessedFilter*) const {
    Canon c;
    canonize(src, filter, bias, z, dst, c, true);
    size_t ws = 0;
    resolve_algo(c.d, m_policy, &ws);
    return ws;
}

std::vector<TensorLayout> ConvBiasForward::deduce_preprocessed_filter_layout(const TensorLayout& src,
                                                                             const TensorLayout& filter,
                                                                             const TensorLayout& bias, const TensorLayout& z,
                                                                             const TensorLayout& dst) const {
    Canon c;
    canonize(src, filter, bias, z, dst, c, true);
    size_t ws = 0, bytes = 0;
    mi355_algo a = resolve_algo(c.d, m_policy, &ws);
    check_abi(mi355_convbias_s8_preprocess_size(&c.d, &a, &bytes));
    if (bytes == 0) return {};
    return {TensorLayout(TensorShape{bytes}, dtype::Int8())};
}

void ConvBiasForward::exec_preprocess(const TensorLayout& src_layout, const TensorND& filter, const TensorND& bias,
                                      const TensorLayout& z_layout, const TensorLayout& dst_layout,
                                      PreprocessedFilter* pf, const Workspace&) {
    HOST_ASSERT(pf != nullptr, MI355_ERR_BAD_ARG, "null PreprocessedFilter");
    Canon c;
    canonize(src_layout, filter.layout, bias.layout, z_layout, dst_layout, c, true);
    size_t ws = 0, bytes = 0;
    mi355_algo a = resolve_algo(c.d, m_policy, &ws);
    pf->algorithm = AlgorithmDesc{a.id, a.tile_cfg};
    check_abi(mi355_convbias_s8_preprocess_size(&c.d, &a, &bytes));
    if (bytes == 0) {
        HOST_ASSERT(pf->tensors.empty(), MI355_ERR_BAD_ARG, "this algorithm has no pre-processed tensors");
        return;
    }
    HOST_ASSERT(pf->tensors.size() == 1 && pf->tensors[0].raw_ptr && pf->tensors[0].layout.total_nr_elems() >= bytes,
                MI355_ERR_BAD_ARG, "PreprocessedFilter needs the one tensor of deduce_preprocessed_filter_layout (%zu bytes)",
                bytes);
    HOST_ASSERT(filter.raw_ptr, MI355_ERR_BAD_ARG, "null filter");
    check_abi(mi355_convbias_s8_preprocess(m_handle->stream(), &c.d, &a, (const int8_t*)filter.raw_ptr,
                                           pf->tensors[0].raw_ptr, pf->tensors[0].layout.total_nr_elems()));
}

void ConvBiasForward::exec(const TensorND& src, const TensorND& filter, const TensorND& bias, const TensorND& z,
                           const TensorND& dst, const PreprocessedFilter* pf, const Workspace& workspace) {
    if (pf && !pf->tensors.empty()) {
        // the artefact was made for pf->algorithm: run exactly that one
        Canon c;
        canonize(src.layout, filter.layout, bias.layout, z.layout, dst.layout, c, true);
        HOST_ASSERT(src.raw_ptr && dst.raw_ptr && pf->tensors[0].raw_ptr, MI355_ERR_BAD_ARG, "null tensor pointer");
        size_t ws = 0;
        mi355_algo a;
        check_abi(mi355_convbias_s8_query(&c.d, pf->algorithm.id, &a, &ws));
        if (pf->algorithm.tile_cfg >= 0) a.tile_cfg = pf->algorithm.tile_cfg;
        HOST_ASSERT(workspace.size >= ws, MI355_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace.size, ws);
        check_abi(mi355_convbias_s8_exec_preprocessed(m_handle->stream(), &c.d, &a, (const int8_t*)src.raw_ptr,
                                                      pf->tensors[0].raw_ptr, pf->tensors[0].layout.total_nr_elems(),
                                                      bias.layout.ndim ? (const int32_t*)bias.raw_ptr : nullptr,
                                                      z.layout.ndim ? (const int8_t*)z.raw_ptr : nullptr, dst.raw_ptr,
                                                      workspace.raw_ptr, workspace.size));
        return;
    }
    Canon c;
    canonize(src.layout, filter.layout, bias.layout, z.layout, dst.layout, c, true);
    HOST_ASSERT(src.raw_ptr && filter.raw_ptr && dst.raw_ptr, MI355_ERR_BAD_ARG, "null tensor pointer");
    if (!m_policy.valid() && m_policy.strategy == ExecutionPolicy::Strategy::PROFILE) {
        AlgorithmCache::Result hit;
        if (!AlgorithmCache::instance().get(c.d, hit)) profile_algorithms(src, filter, bias, z, dst, workspace);
    }
    size_t ws = 0;
    mi355_algo a = resolve_algo(c.d, m_policy, &ws);
    HOST_ASSERT(workspace.size >= ws, MI355_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace.size, ws);
    check_abi(mi355_convbias_s8_exec(m_handle->stream(), &c.d, &a, (const int8_t*)src.raw_ptr,
                                     (const int8_t*)filter.raw_ptr,
                                     bias.layout.ndim ? (const int32_t*)bias.raw_ptr : nullptr,
                                     z.layout.ndim ? (const int8_t*)z.raw_ptr : nullptr, dst.raw_ptr,
                                     workspace.raw_ptr, workspace.size));
}

std::vector<AlgorithmInfo> ConvBiasForward::get_all_algorithms_info(const TensorLayout& src, const TensorLayout& filter,
                                                                    const TensorLayout& bias, const TensorLayout& z,
                                                                    const TensorLayout& dst) const {
    Canon c;
    canonize(src, filter, bias, z, dst, c, true);
    std::vector<AlgorithmInfo> r;
    for (int id = 0; id < mi355_convbias_algo_count(); ++id) {
        if (mi355_convbias_algo_usable(&c.d, id) != MI355_OK) continue;
        const std::string base = mi355_convbias_algo_name(id);
        r.push_back(AlgorithmInfo{AlgorithmDesc{id, -1}, base, true});
        if (base.find("IGEMM") != std::string::npos)
            for (int t = 0; t < mi355_igemm_tile_count(); ++t)
                if (mi355_igemm_tile_usable(&c.d, t) == MI355_OK)  // one kernel, one name
                    r.push_back(AlgorithmInfo{AlgorithmDesc{id, t}, base + ":" + mi355_igemm_tile_name(t), true});
    }
    return r;
}

std::vector<std::pair<AlgorithmInfo, float>> ConvBiasForward::profile_algorithms(
        const TensorND& src, const TensorND& filter, const TensorND& bias, const TensorND& z, const TensorND& dst,
        const Workspace& workspace, int warmup, int iters) {
    Canon c;
    canonize(src.layout, filter.layout, bias.layout, z.layout, dst.layout, c, true);
    HOST_ASSERT(src.raw_ptr && filter.raw_ptr && dst.raw_ptr, MI355_ERR_BAD_ARG, "null tensor pointer");
    std::vector<std::pair<AlgorithmInfo, float>> timed;
    for (auto& info : get_all_algorithms_info(src.layout, filter.layout, bias.layout, z.layout, dst.layout)) {
        size_t ws = 0;
        mi355_algo a;
        if (mi355_convbias_s8_query(&c.d, info.desc.id, &a, &ws) != MI355_OK || ws > workspace.size) continue;
        if (info.desc.tile_cfg >= 0) a.tile_cfg = info.desc.tile_cfg;
        float us = 0.f;
        // an algorithm that cannot take these tensors (alignment) is skipped, not fatal
        if (mi355_convbias_s8_profile(m_handle->stream(), &c.d, &a, (const int8_t*)src.raw_ptr,
                                      (const int8_t*)filter.raw_ptr,
                                      bias.layout.ndim ? (const int32_t*)bias.raw_ptr : nullptr,
                                      z.layout.ndim ? (const int8_t*)z.raw_ptr : nullptr, dst.raw_ptr, workspace.raw_ptr,
                                      workspace.size, warmup, iters, &us) != MI355_OK)
            continue;
        timed.emplace_back(info, us);
    }
    HOST_ASSERT(!timed.empty(), MI355_ERR_ALGO, "no algorithm could be profiled");
    std::stable_sort(timed.begin(), timed.end(), [](const auto& x, const auto& y) { return x.second < y.second; });
    AlgorithmCache::Result best;
    best.policy.algo = timed.front().first.desc;
    best.usec = timed.front().second;
    AlgorithmCache::instance().put(c.d, best);
    return timed;
}

AlgorithmInfo ConvBiasForward::get_algorithm_info_heuristic(const TensorLayout& src, const TensorLayout& filter,
                                                            const TensorLayout& bias, const TensorLayout& z,
                                                            const TensorLayout& dst, size_t workspace_limit) const {
    Canon c;
    canonize(src, filter, bias, z, dst, c, true);
    size_t ws = 0;
    mi355_algo a;
    check_abi(mi355_convbias_s8_query(&c.d, MI355_ALGO_HEURISTIC, &a, &ws));
    HOST_ASSERT(ws <= workspace_limit, MI355_ERR_WORKSPACE, "no algorithm within the workspace limit of %zu bytes",
                workspace_limit);
    std::string name = mi355_convbias_algo_name(a.id);
    if (name.find("IGEMM") != std::string::npos && a.tile_cfg >= 0) name += std::string(":") + mi355_igemm_tile_name(a.tile_cfg);
    return AlgorithmInfo{AlgorithmDesc{a.id, a.tile_cfg}, name, true};
}

// ---------------------------------------------------------------- RelayoutFormat
static mi355_relayout_desc relayout_desc(const param::RelayoutFormat& p, const TensorLayout& src, const DType& dst_dt) {
    mi355_relayout_desc d = mi355_relayout_desc();
    d.mode = (uint32_t)p.mode;
    d.ndim = (uint32_t)src.ndim;
    for (size_t i = 0; i < src.ndim; ++i) d.shape[i] = (uint32_t)src[i];
    d.group = p.group ? p.group : 1;
    d.oc = p.oc;
    d.elem_bytes = (uint32_t)src.dtype.size();
    d.scale_src = src.dtype.enumv == DTypeEnum::QuantizedS8 ? src.dtype.scale : 1.f;
    d.scale_dst = dst_dt.enumv == DTypeEnum::QuantizedS8 ? dst_dt.scale : d.scale_src;
    return d;
}

void RelayoutFormat::deduce_layout(const TensorLayout& src, TensorLayout& dst) const {
    mi355_relayout_desc d = relayout_desc(m_param, src, src.dtype);
    uint32_t nd = 0, sh[7];
    check_abi(mi355_relayout_deduce(&d, &nd, sh));
    TensorShape s;
    s.ndim = nd;
    for (uint32_t i = 0; i < nd; ++i) s.shape[i] = sh[i];
    // an unset dst dtype inherits the src dtype (relayout_format.cpp deduce_layout)
    DType dt = (dst.ndim == 0 && dst.dtype == DType()) ? src.dtype : dst.dtype;
    if (dt.size() != src.dtype.size()) dt = src.dtype;
    dst = TensorLayout(s, dt);
}

void RelayoutFormat::exec(const TensorND& src, const TensorND& dst, const Workspace&) {
    HOST_ASSERT(src.layout.is_contiguous() && dst.layout.is_contiguous(), MI355_ERR_UNSUPPORTED,
                "relayout takes contiguous tensors");
    HOST_ASSERT(src.layout.dtype.size() == dst.layout.dtype.size(), MI355_ERR_BAD_ARG, "element sizes differ");
    mi355_relayout_desc d = relayout_desc(m_param, src.layout, dst.layout.dtype);
    uint32_t nd = 0, sh[7];
    check_abi(mi355_relayout_deduce(&d, &nd, sh));
    TensorShape want;
    want.ndim = nd;
    for (uint32_t i = 0; i < nd; ++i) want.shape[i] = sh[i];
    HOST_ASSERT(dst.layout.eq_shape(want), MI355_ERR_SHAPE, "dst %s, expected %s", dst.layout.to_string().c_str(),
                want.to_string().c_str());
    HOST_ASSERT(src.raw_ptr && dst.raw_ptr, MI355_ERR_BAD_ARG, "null tensor pointer");
    check_abi(mi355_relayout_exec(m_handle->stream(), &d, src.raw_ptr, dst.raw_ptr));
}

// ---------------------------------------------------------------- elementwise requantisation
static void requant_exec(Handle* h, uint32_t nonline, const TensorND& a, const TensorND* b, const TensorND& dst) {
    HOST_ASSERT(dst.layout.dtype.enumv == DTypeEnum::QuantizedS8, MI355_ERR_UNSUPPORTED, "dst must be QuantizedS8");
    HOST_ASSERT(a.layout.dtype.enumv == DTypeEnum::QuantizedS8 || a.layout.dtype.enumv == DTypeEnum::QuantizedS32,
                MI355_ERR_UNSUPPORTED, "the first operand must be QuantizedS8 or QuantizedS32");
    HOST_ASSERT(a.layout.eq_shape(dst.layout) && a.layout.is_contiguous() && dst.layout.is_contiguous(), MI355_ERR_SHAPE,
                "operands must be contiguous and of the dst shape %s", dst.layout.to_string().c_str());
    mi355_requant_desc d = mi355_requant_desc();
    d.nonline = nonline;
    d.scale_src = a.layout.dtype.scale;
    d.scale_dst = dst.layout.dtype.scale;
    d.scale_z = 1.f;
    d.count = dst.layout.total_nr_elems();
    const int8_t* zp = nullptr;
    if (b) {
        HOST_ASSERT(b->layout.dtype.enumv == DTypeEnum::QuantizedS8, MI355_ERR_UNSUPPORTED,
                    "the second operand must be QuantizedS8");
        HOST_ASSERT(b->layout.eq_shape(dst.layout) && b->layout.is_contiguous(), MI355_ERR_SHAPE,
                    "operands must be contiguous and of the dst shape %s", dst.layout.to_string().c_str());
        d.has_z = 1;
        d.scale_z = b->layout.dtype.scale;
        zp = (const int8_t*)b->raw_ptr;
        HOST_ASSERT(zp, MI355_ERR_BAD_ARG, "null tensor pointer");
    }
    HOST_ASSERT(a.raw_ptr && dst.raw_ptr, MI355_ERR_BAD_ARG, "null tensor pointer");
    if (a.layout.dtype.enumv == DTypeEnum::QuantizedS32)
        check_abi(mi355_requant_s32_s8_exec(h->stream(), &d, (const int32_t*)a.raw_ptr, zp, (int8_t*)dst.raw_ptr));
    else
        check_abi(mi355_requant_s8_s8_exec(h->stream(), &d, (const int8_t*)a.raw_ptr, zp, (int8_t*)dst.raw_ptr));
}

void ElemwiseMultiType::exec(const std::vector<TensorND>& src, const TensorND& dst) {
    using Mode = Param::Mode;
    // Q-mode -> the Elemwise::Mode whose float kernel it runs and its number of operands (the ON_QUANTIZED_MODE table,
    // dnn/src/common/elemwise_multi_type/opr_impl_helper.cpp:6-11,:53-111)
    struct Row { Mode q; uint32_t ew, arity; };
    static const Row kRows[] = {
            {Mode::QADD, MI355_EW_ADD, 2}, {Mode::QFUSE_ADD_RELU, MI355_EW_FUSE_ADD_RELU, 2}, {Mode::QMUL, MI355_EW_MUL, 2},
            {Mode::QMIN, MI355_EW_MIN, 2}, {Mode::QMAX, MI355_EW_MAX, 2}, {Mode::QSUB, MI355_EW_SUB, 2},
            {Mode::QTRUE_DIV, MI355_EW_TRUE_DIV, 2}, {Mode::QRELU, MI355_EW_RELU, 1}, {Mode::QABS, MI355_EW_ABS, 1},
            {Mode::QFUSE_MUL_ADD3, MI355_EW_FUSE_MUL_ADD3, 3}, {Mode::QFAST_TANH, MI355_EW_FAST_TANH, 1},
            {Mode::QNEGATE, MI355_EW_NEGATE, 1}, {Mode::QCEIL, MI355_EW_CEIL, 1}, {Mode::QFLOOR, MI355_EW_FLOOR, 1},
            {Mode::QROUND, MI355_EW_ROUND, 1}, {Mode::QABS_GRAD, MI355_EW_ABS_GRAD, 2}, {Mode::QFLOOR_DIV, MI355_EW_FLOOR_DIV, 2},
            {Mode::QSIGMOID_GRAD, MI355_EW_SIGMOID_GRAD, 2}, {Mode::QSWITCH_GT0, MI355_EW_SWITCH_GT0, 2},
            {Mode::QTANH_GRAD, MI355_EW_TANH_GRAD, 2}, {Mode::QLT, MI355_EW_LT, 2}, {Mode::QLEQ, MI355_EW_LEQ, 2},
            {Mode::QEQ, MI355_EW_EQ, 2}, {Mode::QFAST_TANH_GRAD, MI355_EW_FAST_TANH_GRAD, 2},
            {Mode::QCOND_LEQ_MOV, MI355_EW_COND_LEQ_MOV, 3}, {Mode::QH_SWISH, MI355_EW_H_SWISH, 1},
            {Mode::QFUSE_ADD_H_SWISH, MI355_EW_FUSE_ADD_H_SWISH, 2}, {Mode::QH_SWISH_GRAD, MI355_EW_H_SWISH_GRAD, 2},
            {Mode::QCOND_LT_MOV, MI355_EW_COND_LT_MOV, 3},
    };
    const Row* row = nullptr;
    for (const Row& r : kRows)
        if (r.q == m_param.mode) row = &r;
    if (!row) fail(MI355_ERR_UNSUPPORTED, "ElemwiseMultiType mode " + std::to_string((unsigned)m_param.mode) + " is not implemented");
    HOST_ASSERT(src.size() == row->arity, MI355_ERR_BAD_ARG, "mode takes %u operands, got %zu", row->arity, src.size());
    // the requantisation kernels (proved divide-free forms) take the modes of the ConvBias post-process on their
    // operand types: first operand QuantizedS8 / QuantizedS32, second QuantizedS8, dst QuantizedS8
    uint32_t nl = 0;
    bool chain = true;
    switch (m_param.mode) {
        case Mode::QADD: nl = MI355_NL_IDENTITY; break;
        case Mode::QFUSE_ADD_RELU: case Mode::QRELU: nl = MI355_NL_RELU; break;
        case Mode::QFUSE_ADD_H_SWISH: case Mode::QH_SWISH: nl = MI355_NL_H_SWISH; break;
        default: chain = false;
    }
    if (chain && dst.layout.dtype.enumv == DTypeEnum::QuantizedS8 &&
        (row->arity == 1 || src[1].layout.dtype.enumv == DTypeEnum::QuantizedS8))
        return requant_exec(m_handle, nl, src[0], row->arity == 2 ? &src[1] : nullptr, dst);
    auto code = [](DTypeEnum e) -> uint32_t {
        if (e == DTypeEnum::QuantizedS8) return MI355_DT_QS8;
        if (e == DTypeEnum::QuantizedS32) return MI355_DT_QS32;
        fail(MI355_ERR_UNSUPPORTED, "quantized elemwise takes QuantizedS8 or QuantizedS32 tensors");
        return 0;
    };
    mi355_elemwise_desc d = mi355_elemwise_desc();
    d.mode = row->ew;
    d.arity = row->arity;
    d.src_dtype = code(src[0].layout.dtype.enumv);
    d.dst_dtype = code(dst.layout.dtype.enumv);
    d.scale_dst = dst.layout.dtype.scale;
    d.count = dst.layout.total_nr_elems();
    HOST_ASSERT(dst.layout.is_contiguous() && dst.raw_ptr, MI355_ERR_BAD_ARG, "dst must be contiguous and non-null");
    const void* p[3] = {nullptr, nullptr, nullptr};
    for (uint32_t i = 0; i < row->arity; ++i) {
        // the operands share one dtype (dnn/src/naive/elemwise_multi_type/opr_impl_4.cpp:14-16)
        HOST_ASSERT(src[i].layout.dtype.enumv == src[0].layout.dtype.enumv, MI355_ERR_BAD_ARG, "operand %u has another dtype", i);
        HOST_ASSERT(src[i].layout.eq_shape(dst.layout) && src[i].layout.is_contiguous(), MI355_ERR_SHAPE,
                    "operands must be contiguous and of the dst shape %s", dst.layout.to_string().c_str());
        HOST_ASSERT(src[i].raw_ptr, MI355_ERR_BAD_ARG, "null tensor pointer");
        d.scale_src[i] = src[i].layout.dtype.scale;
        p[i] = src[i].raw_ptr;
    }
    check_abi(mi355_elemwise_q_exec(m_handle->stream(), &d, p[0], p[1], p[2], dst.raw_ptr));
}

void TypeCvt::exec(const TensorND& src, const TensorND& dst) {
    const DTypeEnum se = src.layout.dtype.enumv, de = dst.layout.dtype.enumv;
    const bool quantize = se == DTypeEnum::Float32 && de == DTypeEnum::QuantizedS8;
    const bool dequantize = se == DTypeEnum::QuantizedS8 && de == DTypeEnum::Float32;
    if (!quantize && !dequantize) return requant_exec(m_handle, MI355_NL_IDENTITY, src, nullptr, dst);
    HOST_ASSERT(src.layout.eq_shape(dst.layout) && src.layout.is_contiguous() && dst.layout.is_contiguous(), MI355_ERR_SHAPE,
                "operands must be contiguous and of the dst shape %s", dst.layout.to_string().c_str());
    HOST_ASSERT(src.raw_ptr && dst.raw_ptr, MI355_ERR_BAD_ARG, "null tensor pointer");
    const uint64_t n = dst.layout.total_nr_elems();
    if (quantize)
        check_abi(mi355_typecvt_f32_s8_exec(m_handle->stream(), n, dst.layout.dtype.scale,
                                            static_cast<const float*>(src.raw_ptr), static_cast<int8_t*>(dst.raw_ptr)));
    else
        check_abi(mi355_typecvt_s8_f32_exec(m_handle->stream(), n, src.layout.dtype.scale,
                                            static_cast<const int8_t*>(src.raw_ptr), static_cast<float*>(dst.raw_ptr)));
}

// ---------------------------------------------------------------- pooling
static mi355_pooling_desc pooling_desc(const param::Pooling& p, const TensorLayout& src) {
    using F = param::Pooling::Format;
    uint32_t pack = 0;
    switch (p.format) {
        case F::NCHW: pack = 1; break;
        case F::NCHW4:
        case F::NCHW44: pack = 4; break;
        case F::NCHW32: pack = 32; break;
        default: HOST_ASSERT(false, MI355_ERR_UNSUPPORTED, "invalid pooling format %u", (unsigned)p.format);
    }
    HOST_ASSERT(src.ndim == (pack == 1 ? 4u : 5u), MI355_ERR_SHAPE, "src %s does not fit the format", src.to_string().c_str());
    HOST_ASSERT(pack == 1 || src[4] == pack, MI355_ERR_SHAPE, "src %s: innermost axis must be %u", src.to_string().c_str(), pack);
    mi355_pooling_desc d = mi355_pooling_desc();
    d.mode = (uint32_t)p.mode;
    d.format = (uint32_t)p.format;
    d.n = (uint32_t)src[0];
    d.c = (uint32_t)(src[1] * pack);
    d.ih = (uint32_t)src[2];
    d.iw = (uint32_t)src[3];
    d.pad_h = p.pad_h; d.pad_w = p.pad_w; d.stride_h = p.stride_h; d.stride_w = p.stride_w;
    d.window_h = p.window_h; d.window_w = p.window_w;
    return d;
}

void PoolingForward::deduce_layout(const TensorLayout& src, TensorLayout& dst) const {
    const mi355_pooling_desc d = pooling_desc(m_param, src);
    uint32_t oh = 0, ow = 0;
    check_abi(mi355_pooling_deduce_out(&d, &oh, &ow));
    TensorShape s = src;
    s.shape[2] = oh;
    s.shape[3] = ow;
    dst = TensorLayout(s, src.dtype);
}

void PoolingForward::exec(const TensorND& src, const TensorND& dst, const Workspace&) {
    HOST_ASSERT(src.layout.dtype.enumv == DTypeEnum::QuantizedS8, MI355_ERR_UNSUPPORTED, "pooling takes QuantizedS8 tensors");
    HOST_ASSERT(src.layout.dtype == dst.layout.dtype, MI355_ERR_BAD_ARG, "src and dst dtypes differ");
    HOST_ASSERT(src.layout.is_contiguous() && dst.layout.is_contiguous(), MI355_ERR_UNSUPPORTED, "pooling takes contiguous tensors");
    TensorLayout want;
    deduce_layout(src.layout, want);
    HOST_ASSERT(dst.layout.eq_shape(want), MI355_ERR_SHAPE, "dst %s, expected %s", dst.layout.to_string().c_str(),
                want.to_string().c_str());
    HOST_ASSERT(src.raw_ptr && dst.raw_ptr, MI355_ERR_BAD_ARG, "null tensor pointer");
    const mi355_pooling_desc d = pooling_desc(m_param, src.layout);
    check_abi(mi355_pooling_s8_exec(m_handle->stream(), &d, static_cast<const int8_t*>(src.raw_ptr),
                                    static_cast<int8_t*>(dst.raw_ptr)));
}

}  // namespace mi355dnn
