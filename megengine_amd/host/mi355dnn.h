// Host-side C++ operator interface over the MI355X ConvBias / RelayoutFormat kernels.
//
// This is the class-level surface a MegDNN backend exposes for the quantized-int8 ConvBias path,
// restated over the C ABI of include/mi355_convbias.h.  Names, argument meaning and error
// behaviour follow the reference interface so that a maintainer can map one onto the other:
//
//   TensorShape / TensorLayout / TensorND / Workspace   dnn/include/megdnn/basic_types.h:86-300, :462-530
//   DType (QuantizedS8 / QuantizedS32 with a scale)     dnn/include/megdnn/dtype.h:835-898
//   param::ConvBias, param::RelayoutFormat              dnn/scripts/opr_param_defs.py:5-35, :96-113, :199-215, :1069-1111
//   Handle::create_operator<Opr>()                      dnn/include/megdnn/handle.h:17-28, :96-160
//   ConvBiasForward                                     dnn/include/megdnn/oprs/nn.h:358-536
//   RelayoutFormat                                      dnn/include/megdnn/oprs/general.h:1348-1373
//   Algorithm / ExecutionPolicy                         dnn/include/megdnn/oprs/base.h:89-287, :323-329, :545-615
//   Error                                               megdnn_error via megdnn_throw, dnn/include/megdnn/basic_types.h:21-58
//
// Operators never allocate device memory and do not own the stream; exec() is asynchronous
// with respect to the host and ordered on the handle's stream.  Every failed check throws
// mi355dnn::Error (the counterpart of megdnn_throw), carrying the C ABI's status and message.
#pragma once
#include <stddef.h>
#include <stdint.h>

#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

struct mi355_conv_desc;  // include/mi355_convbias.h

namespace mi355dnn {

class Error : public std::runtime_error {
public:
    Error(int status, const std::string& msg) : std::runtime_error(msg), m_status(status) {}
    int status() const { return m_status; }

private:
    int m_status;
};

// ---- dtypes on this path
enum class DTypeEnum : uint32_t { QuantizedS8 = 0, QuantizedS32 = 1, Int8 = 2, Int32 = 3, Float32 = 4 };

struct DType {
    DTypeEnum enumv = DTypeEnum::QuantizedS8;
    float scale = 1.f;  // meaningful for the quantized types only
    size_t size() const { return enumv == DTypeEnum::QuantizedS8 || enumv == DTypeEnum::Int8 ? 1 : 4; }
    bool operator==(const DType& o) const { return enumv == o.enumv && scale == o.scale; }
};
namespace dtype {
inline DType QuantizedS8(float scale) { return DType{DTypeEnum::QuantizedS8, scale}; }
inline DType QuantizedS32(float scale) { return DType{DTypeEnum::QuantizedS32, scale}; }
inline DType Int8() { return DType{DTypeEnum::Int8, 1.f}; }
inline DType Int32() { return DType{DTypeEnum::Int32, 1.f}; }
inline DType Float32() { return DType{DTypeEnum::Float32, 1.f}; }
}  // namespace dtype

// ---- shapes and layouts (strides in elements, as in the reference)
struct TensorShape {
    static constexpr size_t MAX_NDIM = 7;
    size_t shape[MAX_NDIM] = {0, 0, 0, 0, 0, 0, 0};
    size_t ndim = 0;
    TensorShape() = default;
    TensorShape(std::initializer_list<size_t> s);
    size_t total_nr_elems() const;
    bool eq_shape(const TensorShape& o) const;
    std::string to_string() const;
    size_t& operator[](size_t i) { return shape[i]; }
    size_t operator[](size_t i) const { return shape[i]; }
};

struct TensorLayout : TensorShape {
    ptrdiff_t stride[MAX_NDIM] = {0, 0, 0, 0, 0, 0, 0};
    DType dtype;
    TensorLayout() = default;
    TensorLayout(const TensorShape& shape, DType dt);  // contiguous
    void init_contiguous_stride();
    bool is_contiguous() const;
    // contiguous in every axis but the first (a batch-strided view)
    bool is_batch_strided() const;
    size_t span_bytes() const;
};

struct TensorND {
    TensorLayout layout;
    void* raw_ptr = nullptr;  // DEVICE pointer
    TensorND() = default;
    TensorND(void* p, const TensorLayout& l) : layout(l), raw_ptr(p) {}
};

struct Workspace {
    void* raw_ptr = nullptr;
    size_t size = 0;
    Workspace() = default;
    Workspace(void* p, size_t s) : raw_ptr(p), size(s) {}
};

// ---- params (enumerator values are the reference's)
namespace param {
struct ConvBias {
    enum class NonlineMode : uint32_t { IDENTITY = 0, RELU = 1, SIGMOID = 2, H_SWISH = 3 };
    enum class Mode : uint32_t { CROSS_CORRELATION = 0, CONVOLUTION = 1 };
    enum class Sparse : uint32_t { DENSE = 0, GROUP = 1 };
    enum class Format : uint32_t {
        NCHW = 0, NHWC = 1, NHWCD4 = 2, NCHW4 = 3, NCHW8 = 4, NCHW32 = 5, NCHW88 = 6, NCHW44 = 7,
        NCHW44_DOT = 8, NCHW4_NCHW32 = 9, NCHW32_NCHW4 = 10, NCHW4_NCHW = 11, CHWN4 = 15, NCHW64 = 16,
        NCHW4_NHWC = 17
    };
    enum class ComputeMode : uint32_t { DEFAULT = 0, FLOAT32 = 1 };
    NonlineMode nonlineMode = NonlineMode::IDENTITY;
    Mode mode = Mode::CROSS_CORRELATION;
    Sparse sparse = Sparse::DENSE;
    Format format = Format::NCHW;
    uint32_t pad_h = 0, pad_w = 0, stride_h = 1, stride_w = 1, dilate_h = 1, dilate_w = 1;
    ComputeMode compute_mode = ComputeMode::DEFAULT;
};

struct RelayoutFormat {
    enum class Mode : uint32_t {
        NCHW_NCHW4_IC_SMALL = 22, NCHW_NCHW4 = 24, NCHW4_NCHW = 25, NCHW_NCHW4_WEIGHT = 26,
        // additions of this backend: the reference reaches NCHW32 through reshape + dimshuffle
        NCHW_NCHW32 = 32, NCHW32_NCHW = 33, NCHW4_NCHW32 = 34, NCHW32_NCHW4 = 35
    };
    Mode mode = Mode::NCHW_NCHW4;
    uint32_t oc = 0;
    uint32_t group = 1;
};
// param::Pooling (dnn/scripts/opr_param_defs.py:233-254); Format shares the ConvBias enumerators
struct Pooling {
    enum class Mode : uint32_t { MAX = 0, AVERAGE = 1, AVERAGE_COUNT_EXCLUDE_PADDING = 2 };
    using Format = ConvBias::Format;
    Mode mode = Mode::MAX;
    uint32_t pad_h = 0, pad_w = 0, stride_h = 2, stride_w = 2, window_h = 2, window_w = 2;
    Format format = Format::NCHW;
};
}  // namespace param

// ---- algorithms
struct AlgorithmDesc {
    int32_t id = -1;        // kernel family (index into the C ABI's algorithm list)
    int32_t tile_cfg = -1;  // tile shape for the implicit-GEMM family, -1 = heuristic
    bool operator==(const AlgorithmDesc& o) const { return id == o.id && tile_cfg == o.tile_cfg; }
};
struct AlgorithmInfo {
    AlgorithmDesc desc;
    std::string name;
    bool is_reproducible = true;  // every kernel here is deterministic (no atomics, fixed order)
};
struct ExecutionPolicy {
    // HEURISTIC: the backend's rule table.  PROFILE: fast-run -- the first exec of a problem times every usable
    // algorithm and tile on the caller's tensors, later ones take the winner from AlgorithmCache.
    enum class Strategy : uint32_t { HEURISTIC = 0, PROFILE = 1 };
    AlgorithmDesc algo;  // id >= 0: use exactly this one, whatever the strategy
    Strategy strategy = Strategy::HEURISTIC;
    // the caller runs exec_preprocess once and hands exec the PreprocessedFilter (the reference's weight_preprocess
    // graph option): the heuristic may then choose an algorithm that is fastest only with its pre-processed filter
    bool weight_preprocess = false;
    bool valid() const { return algo.id >= 0; }
};

// Winners of profiling runs, keyed by the flat problem descriptor: megdnn::AlgorithmCache
// (dnn/include/megdnn/algorithm_cache.h:12-80) with the persistence the reference keeps in its PersistentCache
// (src/core/include/megbrain/utils/persistent_cache.h): one text line per problem.
class AlgorithmCache {
public:
    struct Result {
        ExecutionPolicy policy;
        size_t workspace = 0;
        float usec = 0.f;  // measured time of the winner
    };
    static AlgorithmCache& instance();
    void put(const mi355_conv_desc& key, const Result& r);
    bool get(const mi355_conv_desc& key, Result& r) const;
    void clear();
    size_t size() const;
    // text file: "<descriptor bytes in hex> <algorithm id> <tile> <workspace> <microseconds>" per line
    void save(const std::string& path) const;
    size_t load(const std::string& path);  // returns the number of entries read; unknown lines are skipped

private:
    AlgorithmCache() = default;
    struct Impl;
    Impl& impl() const;
};

class Handle;

class OperatorBase {
public:
    explicit OperatorBase(Handle* h) : m_handle(h) {}
    virtual ~OperatorBase() = default;
    Handle* handle() const { return m_handle; }
    virtual bool is_thread_safe() const { return false; }

protected:
    Handle* m_handle;
};

class ConvBiasForward : public OperatorBase {
public:
    using Param = param::ConvBias;
    enum class BiasMode : uint32_t { NO_BIAS = 0, BROADCAST_CHANNEL_BIAS, BIAS };
    // the tensors that exec_preprocess filled for `algorithm` (megdnn::detail::PreprocessedFilter,
    // dnn/include/megdnn/oprs/nn.h:47-52); exec uses them instead of the filter
    struct PreprocessedFilter {
        AlgorithmDesc algorithm;
        std::vector<TensorND> tensors;
    };

    explicit ConvBiasForward(Handle* h) : OperatorBase(h) {}
    Param& param() { return m_param; }
    const Param& param() const { return m_param; }
    ExecutionPolicy& execution_policy() { return m_policy; }
    const ExecutionPolicy& execution_policy() const { return m_policy; }

    // dst dtype for s8 x s8: QuantizedS32(src.scale * filter.scale) unless dst already names
    // QuantizedS8 (any scale) or QuantizedS32
    void deduce_dtype(DType src, DType filter, DType bias, DType z, DType& dst) const;
    void deduce_layout(const TensorLayout& src, const TensorLayout& filter, const TensorLayout& bias,
                       const TensorLayout& z, TensorLayout& dst) const;
    size_t get_workspace_in_bytes(const TensorLayout& src, const TensorLayout& filter, const TensorLayout& bias,
                                  const TensorLayout& z, const TensorLayout& dst,
                                  const PreprocessedFilter* preprocessed_filter = nullptr) const;
    // bias / z absent: layout.ndim == 0 (the pointer is then ignored)
    void exec(const TensorND& src, const TensorND& filter, const TensorND& bias, const TensorND& z,
              const TensorND& dst, const PreprocessedFilter* preprocessed_filter, const Workspace& workspace);

    // Weight pre-processing (dnn/include/megdnn/oprs/nn.h:400-447).  The artefact belongs to the algorithm the
    // execution policy resolves to for these layouts: one Int8 tensor (the filter re-tiled for that kernel's copies),
    // or no tensor at all when the algorithm reads the reference layout only -- then exec_preprocess does nothing
    // and exec ignores an empty PreprocessedFilter, as the reference's naive backend does.  No workspace is needed.
    size_t get_preprocess_workspace_in_bytes(const TensorLayout&, const TensorLayout&, const TensorLayout&,
                                             const TensorLayout&, const TensorLayout&) const { return 0; }
    std::vector<TensorLayout> deduce_preprocessed_filter_layout(const TensorLayout& src, const TensorLayout& filter,
                                                                const TensorLayout& bias, const TensorLayout& z,
                                                                const TensorLayout& dst) const;
    void exec_preprocess(const TensorLayout& src_layout, const TensorND& filter, const TensorND& bias,
                         const TensorLayout& z_layout, const TensorLayout& dst_layout,
                         PreprocessedFilter* preprocessed_filter, const Workspace& workspace);

    // algorithm surface
    std::vector<AlgorithmInfo> get_all_algorithms_info(const TensorLayout& src, const TensorLayout& filter,
                                                       const TensorLayout& bias, const TensorLayout& z,
                                                       const TensorLayout& dst) const;
    AlgorithmInfo get_algorithm_info_heuristic(const TensorLayout& src, const TensorLayout& filter,
                                               const TensorLayout& bias, const TensorLayout& z,
                                               const TensorLayout& dst,
                                               size_t workspace_limit_in_bytes = SIZE_MAX) const;
    const char* get_algorithm_set_name() const { return "MI355_CONV_BIAS"; }
    // fast-run: times every usable algorithm (every tile of the implicit-GEMM family) on these tensors, fastest first,
    // and records the winner in AlgorithmCache.  Overwrites dst; synchronises the handle's stream.
    std::vector<std::pair<AlgorithmInfo, float>> profile_algorithms(const TensorND& src, const TensorND& filter,
                                                                    const TensorND& bias, const TensorND& z,
                                                                    const TensorND& dst, const Workspace& workspace,
                                                                    int warmup = 2, int iters = 10);
    static BiasMode bias_mode_of(const TensorLayout& bias, const TensorLayout& dst);

private:
    struct Canon;  // filled descriptor + bookkeeping
    void canonize(const TensorLayout& src, const TensorLayout& filter, const TensorLayout& bias,
                  const TensorLayout& z, const TensorLayout& dst, Canon& out, bool need_dst) const;
    Param m_param;
    ExecutionPolicy m_policy;
};
using ConvBias = ConvBiasForward;

class RelayoutFormat : public OperatorBase {
public:
    using Param = param::RelayoutFormat;
    explicit RelayoutFormat(Handle* h) : OperatorBase(h) {}
    Param& param() { return m_param; }
    const Param& param() const { return m_param; }
    void deduce_layout(const TensorLayout& src, TensorLayout& dst) const;
    size_t get_workspace_in_bytes(const TensorLayout&, const TensorLayout&) const { return 0; }
    void exec(const TensorND& src, const TensorND& dst, const Workspace& workspace);

private:
    Param m_param;
};

// The quantized modes of megdnn::ElemwiseMultiType (dnn/include/megdnn/oprs/nn_int.h:12): dst = quantize(mode(
// dequantize(a) [, dequantize(b) [, dequantize(c)]])), operands QuantizedS8 or QuantizedS32 of one dtype, dst
// QuantizedS8 or QuantizedS32, contiguous tensors of one shape.  The modes whose float kernel calls the C math library
// (QEXP, QSIGMOID, QTANH, QPOW ...) are MI355_ERR_UNSUPPORTED: their bits belong to the host's libm.
class ElemwiseMultiType : public OperatorBase {
public:
    struct Param {
        // values of param::ElemwiseMultiType::Mode (dnn/scripts/opr_param_defs.py:479-540)
        enum class Mode : uint32_t {
            QADD = 6, QFUSE_ADD_RELU = 7, QMUL = 8, QMIN = 9, QMAX = 10, QSUB = 11, QTRUE_DIV = 12, QRELU = 15, QABS = 16,
            QFUSE_MUL_ADD3 = 20, QFAST_TANH = 21, QNEGATE = 22, QCEIL = 25, QFLOOR = 28, QROUND = 32, QABS_GRAD = 37,
            QFLOOR_DIV = 38, QSIGMOID_GRAD = 40, QSWITCH_GT0 = 41, QTANH_GRAD = 42, QLT = 43, QLEQ = 44, QEQ = 45,
            QFAST_TANH_GRAD = 48, QCOND_LEQ_MOV = 50, QH_SWISH = 51, QFUSE_ADD_H_SWISH = 52, QH_SWISH_GRAD = 53,
            QCOND_LT_MOV = 57
        };
        Mode mode = Mode::QADD;
    };
    explicit ElemwiseMultiType(Handle* h) : OperatorBase(h) {}
    Param& param() { return m_param; }
    const Param& param() const { return m_param; }
    // src: as many tensors as the mode has operands
    void exec(const std::vector<TensorND>& src, const TensorND& dst);

private:
    Param m_param;
};

// megdnn::PoolingForward (dnn/include/megdnn/oprs/nn.h, class PoolingForward) on QuantizedS8 tensors in NCHW, NCHW4,
// NCHW44 or NCHW32; dst has the dtype of src (dnn/src/common/pooling.cpp:129-140).
class PoolingForward : public OperatorBase {
public:
    using Param = param::Pooling;
    using Mode = Param::Mode;
    explicit PoolingForward(Handle* h) : OperatorBase(h) {}
    Param& param() { return m_param; }
    const Param& param() const { return m_param; }
    void deduce_layout(const TensorLayout& src, TensorLayout& dst) const;
    size_t get_workspace_in_bytes(const TensorLayout&, const TensorLayout&) const { return 0; }
    void exec(const TensorND& src, const TensorND& dst, const Workspace& workspace);

private:
    Param m_param;
};
using Pooling = PoolingForward;

// megdnn::TypeCvt (dnn/include/megdnn/oprs/general.h:890) for QuantizedS32 / QuantizedS8 -> QuantizedS8 and between
// Float32 and QuantizedS8
class TypeCvt : public OperatorBase {
public:
    explicit TypeCvt(Handle* h) : OperatorBase(h) {}
    void exec(const TensorND& src, const TensorND& dst);
};

// One handle <-> one device and one stream; the caller keeps ownership of the stream.
class Handle {
public:
    // stream: a hipStream_t (nullptr = the null stream); device: HIP device ordinal
    static std::unique_ptr<Handle> make(void* stream, int device = 0);
    template <typename Opr>
    std::unique_ptr<Opr> create_operator() {
        return std::unique_ptr<Opr>(new Opr(this));
    }
    void* stream() const { return m_stream; }
    int device() const { return m_device; }
    // checks that the device exists and is gfx950; throws Error otherwise
    void check_device() const;
    static int abi_version();

private:
    Handle(void* stream, int device) : m_stream(stream), m_device(device) {}
    void* m_stream;
    int m_device;
};

}  // namespace mi355dnn
