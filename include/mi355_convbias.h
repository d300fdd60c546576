/*
 * mi355_convbias.h -- C ABI of the MI355X (gfx950) quantized ConvBias / RelayoutFormat path.
 *
 * This is the boundary a MegDNN handle backend binds: plain C types, caller-owned
 * device pointers, no allocation, no exceptions.  Every entry point returns an
 * mi355_status; the C++ operator classes turn a non-zero status into megdnn_throw.
 *
 * Reference interfaces each entry point stands in for (paths relative to the
 * MegEngine tree):
 *   mi355_conv_desc            <- param::ConvBias (dnn/scripts/opr_param_defs.py:199-215)
 *                                 + ConvolutionBase::CanonizedFilterMeta
 *                                 (dnn/include/megdnn/oprs/nn.h:82-135)
 *                                 + the QuantizedS8/QuantizedS32 dtype scales
 *                                 (dnn/include/megdnn/dtype.h:835-898)
 *   mi355_convbias_s8_query    <- ConvBiasForward::get_workspace_in_bytes
 *                                 (dnn/include/megdnn/oprs/nn.h:419-422) and
 *                                 get_algorithm_heuristic (dnn/include/megdnn/oprs/base.h:595-614)
 *   mi355_convbias_s8_exec     <- ConvBiasForward::exec (dnn/include/megdnn/oprs/nn.h:381-385),
 *                                 arithmetic of naive::ConvBiasForwardImpl::exec
 *                                 (dnn/src/naive/conv_bias/opr_impl.cpp:211-292)
 *   mi355_convbias_algo_*      <- MultiAlgoOpr::get_all_algorithms / Algorithm::name
 *                                 (dnn/include/megdnn/oprs/base.h:545-615)
 *   mi355_convbias_s8_profile  <- the timed trial run of the fast-run algorithm chooser (src/rdnn/impl/algo_chooser.cpp)
 *   mi355_requant_s32_s8_exec  <- the ConvBias post-process as its own pass, handle_z_inp_and_activation_naive
 *                                 (dnn/src/naive/conv_bias/opr_impl.cpp:21-98); without z that is the unary
 *                                 ElemwiseMultiType Q<mode> s32 -> s8 (dnn/src/naive/elemwise_multi_type/
 *                                 opr_impl.h:47-68, opr_impl_3.cpp:12-59) or TypeCvt s32 -> s8
 *                                 (dnn/src/naive/type_cvt/opr_impl.cpp:24-56)
 *   mi355_requant_s8_s8_exec   <- ElemwiseMultiType binary quantized modes on two QuantizedS8 tensors
 *                                 (dnn/src/naive/elemwise_multi_type/opr_impl.h:88-116, opr_impl_4.cpp:11-60)
 *   mi355_elemwise_q_exec      <- ElemwiseMultiType::on_quantized_mode, one to three inputs, every libm-free mode
 *                                 (opr_impl_3.cpp:11-60, opr_impl_4.cpp:11-66, opr_impl_5.cpp:11-45)
 *   mi355_relayout_exec        <- RelayoutFormat::exec (dnn/include/megdnn/oprs/general.h:1353-1359),
 *                                 arithmetic of naive::RelayoutFormatImpl::exec
 *                                 (dnn/src/naive/relayout_format/opr_impl.cpp:486-773)
 *   mi355_status_string        <- ErrorHandler::on_megdnn_error message path
 *                                 (dnn/include/megdnn/basic_types.h:21-58)
 */
#ifndef MI355_CONVBIAS_H_
#define MI355_CONVBIAS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_CONVBIAS_ABI_VERSION 1

typedef enum mi355_status {
    MI355_OK = 0,
    MI355_ERR_BAD_ARG = 1,       /* null pointer / malformed descriptor */
    MI355_ERR_UNSUPPORTED = 2,   /* legal megdnn request this backend does not cover */
    MI355_ERR_SHAPE = 3,         /* shapes inconsistent (channel/group/pack mismatch) */
    MI355_ERR_WORKSPACE = 4,     /* workspace smaller than query() reported */
    MI355_ERR_LAUNCH = 5,        /* HIP launch or runtime error */
    MI355_ERR_NO_DEVICE = 6,     /* no gfx950 device visible */
    MI355_ERR_ALGO = 7           /* algorithm id unknown or not usable for this descriptor */
} mi355_status;

/* values of param::ConvBias::Format (opr_param_defs.py:96-113) */
enum {
    MI355_FMT_NCHW = 0,
    MI355_FMT_NCHW4 = 3,
    MI355_FMT_NCHW32 = 5,
    MI355_FMT_NCHW44 = 7,
    MI355_FMT_NCHW4_NCHW32 = 9,
    MI355_FMT_NCHW32_NCHW4 = 10,
    MI355_FMT_NCHW4_NCHW = 11
};
/* param::ConvBias::NonlineMode (opr_param_defs.py:5-35); SIGMOID (2) is rejected for
 * quantized data exactly as naive does (conv_bias/opr_impl.cpp:79-88). */
enum { MI355_NL_IDENTITY = 0, MI355_NL_RELU = 1, MI355_NL_SIGMOID = 2, MI355_NL_H_SWISH = 3 };
/* param::ConvBias::Mode */
enum { MI355_MODE_CROSS_CORRELATION = 0, MI355_MODE_CONVOLUTION = 1 };
/* param::ConvBias::Sparse */
enum { MI355_SPARSE_DENSE = 0, MI355_SPARSE_GROUP = 1 };
/* ConvBiasForward::BiasMode (nn.h:449-453) */
enum { MI355_BIAS_NONE = 0, MI355_BIAS_BROADCAST_CHANNEL = 1, MI355_BIAS_FULL = 2 };
/* dst dtype */
enum { MI355_DT_QS8 = 0, MI355_DT_QS32 = 1, MI355_DT_F32 = 2 /* Float32 dst: NCHW4_NCHW only */ };

/*
 * One ConvBias problem.  Channel counts are LOGICAL channels (ic = group * icpg,
 * oc = group * ocpg); packed formats store ic/4 or ic/32 blocks.
 *
 * Tensor layouts (all int8 unless noted, innermost dimension last):
 *   NCHW    src (n, ic, ih, iw)        filter (oc, ic, fh, fw) | (g, ocpg, icpg, fh, fw)
 *   NCHW4   src (n, ic/4, ih, iw, 4)   filter (oc, ic/4, fh, fw, 4) | (g, ocpg, icpg/4, fh, fw, 4)
 *   NCHW32  same with 32
 *   NCHW44  src (n, ic/4, ih, iw, 4)   filter dense (oc/4, ic/4, fh, fw, 4ic, 4oc),
 *           group (g, ocpg/4, icpg/4, fh, fw, 4ic, 4oc), channel-wise (g/4, 1, 1, fh, fw, 4)
 *   NCHW4 with sparse=GROUP and icpg == ocpg == 1 is accepted as an extension and uses the
 *   NCHW44 channel-wise filter layout (g/4, 1, 1, fh, fw, 4); the reference cannot express
 *   icpg < 4 under Format::NCHW4 (dnn/src/common/convolution.cpp:392-407).
 *   NCHW4_NCHW32 / NCHW32_NCHW4: src+filter in the first pack, dst/bias in the second.
 *   NCHW4_NCHW: src+filter NCHW4, dst/bias/z NCHW (dnn/src/common/convolution.cpp:929-947).  Its dst may also be
 *   Float32 (MI355_DT_F32; check_or_deduce_dtype_fwd, dnn/src/common/convolution.cpp:1051-1140): then bias and z are
 *   Float32 too (passed through the typed pointers of exec by a cast, as the int32 z of a QuantizedS32 dst is),
 *   scale_bias holds the scale of src, scale_z the scale of filter, scale_dst is ignored, and the result is
 *   act(sum(dequantize(s) * dequantize(f)) + bias + z) in float (StrategyFwd::on for qint8 -> float,
 *   dnn/src/naive/convolution/helper.h:59-66).  Float accumulation order is not part of the contract: the kernel
 *   accumulates exactly in int32 and scales once; agreement with the reference's float running sum is to 1e-3
 *   relative, the tolerance of its own checker.
 *   bias: int32, (1, oc, 1, 1) / (1, oc/p, 1, 1, p) of the dst pack, or the full dst shape.
 *   z:    dst dtype and shape, own scale.
 * src/dst/z may have a non-contiguous batch dimension: *_stride_n are in elements, 0 = dense.
 * dst may be the very buffer of z (same address, same batch stride, same dtype): every kernel reads the residual of an
 * output element in the thread that writes that element, before the write, so the output replaces the residual in
 * place.  Any other overlap of dst with an input is undefined.
 */
typedef struct mi355_conv_desc {
    uint32_t format;
    uint32_t sparse;
    uint32_t nonline;
    uint32_t mode;
    uint32_t n, ic, ih, iw;
    uint32_t oc, fh, fw;
    uint32_t group;
    uint32_t pad_h, pad_w, stride_h, stride_w, dilate_h, dilate_w;
    uint32_t dst_dtype;
    uint32_t bias_mode;
    uint32_t has_z;
    float scale_bias; /* scale stored on the bias dtype (QuantizedS32), used even when bias is absent */
    float scale_z;
    float scale_dst;
    int64_t src_stride_n, dst_stride_n, z_stride_n;
} mi355_conv_desc;

/* Opaque-ish algorithm choice: id indexes the static algorithm table; the tile fields are
 * filled by query() and must be passed back unchanged. */
typedef struct mi355_algo {
    int32_t id;
    int32_t tile_cfg;
    uint64_t reserved;
} mi355_algo;

#define MI355_ALGO_HEURISTIC (-1)
/* the heuristic for a caller that will pre-process the filter for the algorithm it is given (the reference's
 * weight_preprocess graph option): it may prefer an algorithm that is fastest only with its pre-processed filter */
#define MI355_ALGO_HEURISTIC_PREPROCESS (-2)
/* bit of mi355_algo.reserved, set by query() when the heuristic chose the algorithm: exec() may then replace it by
 * the generic kernel when a tensor is not aligned for the tiled kernels (the reference accepts any pointer); an
 * algorithm requested by id is never replaced, exec() reports MI355_ERR_ALGO instead. */
#define MI355_ALGO_FLAG_HEURISTIC 1ull

/* ---- library / device ---- */
int mi355_abi_version(void);
const char* mi355_status_string(int status);
/* last error text of the calling thread (HIP error string, failed check) */
const char* mi355_last_error(void);

typedef struct mi355_device_info {
    int32_t device;
    int32_t compute_units;
    int32_t clock_khz;
    int32_t lds_bytes_per_cu;
    int64_t hbm_bytes;
    char arch[32];
    char name[96];
} mi355_device_info;
int mi355_get_device_info(int device, mi355_device_info* out);

/* A measuring stick, not an operator: launches one plain streaming kernel on `stream` that reads read_bytes from src and
 * writes write_bytes to dst in 16-byte accesses (buffers 16-byte aligned, counts multiples of 16; the bytes written are
 * a function of the bytes read; a probe that reads must write at least 16 bytes, which is what keeps its loads).  A chain of such launches with the byte counts of a network's layers shows what the
 * launches and the memory traffic alone cost on this device, which is what bench.py reports beside the data-sheet
 * roofline.  No counterpart in the reference. */
int mi355_stream_probe(void* stream, const void* src, uint64_t read_bytes, void* dst, uint64_t write_bytes);

/* ---- ConvBias ---- */
/* output spatial size: floor((i + 2p - ((f-1)d+1)) / s) + 1  (dnn/src/common/utils.cpp:130-138) */
int mi355_convbias_deduce_out(const mi355_conv_desc* d, uint32_t* oh, uint32_t* ow);

/* number of algorithms in the static table, their names ("MI355_IGEMM_MFMA_I8", ...) */
int mi355_convbias_algo_count(void);
const char* mi355_convbias_algo_name(int id);
/* MI355_OK if algorithm `id` can run descriptor `d` */
int mi355_convbias_algo_usable(const mi355_conv_desc* d, int id);

/* Validate d, pick an algorithm (algo_request = MI355_ALGO_HEURISTIC, MI355_ALGO_HEURISTIC_PREPROCESS or a table
 * id) and report the workspace it needs. */
int mi355_convbias_s8_query(const mi355_conv_desc* d, int algo_request, mi355_algo* algo_out,
                            size_t* workspace_bytes);

/* Launch on `stream` (a hipStream_t; NULL = default stream).  Asynchronous. */
int mi355_convbias_s8_exec(void* stream, const mi355_conv_desc* d, const mi355_algo* algo,
                           const int8_t* src, const int8_t* filter, const int32_t* bias,
                           const int8_t* z, void* dst, void* workspace, size_t workspace_bytes);

/* exec for callers that cannot allocate a workspace -- code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference (its operators always take the caller's Workspace).  Same
 * arguments, algorithms and results as mi355_convbias_s8_exec, minus the workspace: the algorithms that need one (plain
 * NCHW through relayout + MFMA) use an array of MI355_STATIC_WORKSPACE_BYTES that is part of the library's own device
 * image, one per GPU, held from the first use of the library on that GPU until the process ends.  The call allocates
 * nothing (no hipMalloc / hipFree, no allocating library routine); the first call on a device looks the array's address
 * up once (not under stream capture: make one call per device before capturing).  An algorithm that needs more than the
 * array holds is MI355_ERR_WORKSPACE; without an algorithm the heuristic only considers what fits.  All calls on one
 * GPU share the one array: calls that overlap in time on the same GPU (different streams, different threads) race --
 * serialise them, or give all but one a workspace of their own through mi355_convbias_s8_exec.  Nothing in the array
 * needs to survive between calls, and nothing in it is assumed to be zero. */
#define MI355_STATIC_WORKSPACE_BYTES (32u << 20)
size_t mi355_static_workspace_bytes(void);
int mi355_convbias_s8_exec_static_workspace(void* stream, const mi355_conv_desc* d, const mi355_algo* algo,
                                            const int8_t* src, const int8_t* filter, const int32_t* bias,
                                            const int8_t* z, void* dst);

/* Weight pre-processing: ConvBiasForward::deduce_preprocessed_filter_layout / get_preprocess_workspace_in_bytes /
 * exec_preprocess and the PreprocessedFilter argument of exec (dnn/include/megdnn/oprs/nn.h:381-385,400-447; CUDA
 * precedent dnn/src/cuda/conv_bias/implicit_gemm_int8_nchw32_imma.cpp:164-198: the filter re-ordered once for the
 * kernel, outside exec).  The artefact belongs to ONE algorithm (pass the mi355_algo of query(), tile included):
 *   _preprocess_size   bytes of its one pre-processed tensor; 0 when the algorithm reads the reference layout only
 *                      (then _preprocess does nothing, like the reference's naive backend, and exec takes the filter);
 *   _preprocess        writes it from the filter in the reference layout (asynchronous on `stream`, no workspace);
 *   _exec_preprocessed exec with that tensor in place of the filter.
 * Today the second-generation MFMA tiles ("v2_*") on 32-packed inputs have one: the filter as
 * [32-byte k-chunk][output channel, padded to a multiple of 32][32 bytes], so that every global -> LDS copy of the
 * kernel moves one contiguous kilobyte. */
int mi355_convbias_s8_preprocess_size(const mi355_conv_desc* d, const mi355_algo* algo, size_t* bytes);
int mi355_convbias_s8_preprocess(void* stream, const mi355_conv_desc* d, const mi355_algo* algo, const int8_t* filter,
                                 void* preprocessed, size_t preprocessed_bytes);
int mi355_convbias_s8_exec_preprocessed(void* stream, const mi355_conv_desc* d, const mi355_algo* algo, const int8_t* src,
                                        const void* preprocessed, size_t preprocessed_bytes, const int32_t* bias,
                                        const int8_t* z, void* dst, void* workspace, size_t workspace_bytes);

/* Profiling primitive of a fast-run chooser (the role of rdnn::AlgoChooser's timed trial runs over
 * get_all_algorithms_info_safe, src/rdnn/impl/algo_chooser.cpp; dnn/include/megdnn/oprs/base.h:545-615): `warmup`
 * untimed and `iters` timed launches of ONE algorithm, bracketed by HIP events on `stream`; *avg_usec receives the
 * average time of a launch.  Synchronises the stream and overwrites dst; allocates no device memory. */
int mi355_convbias_s8_profile(void* stream, const mi355_conv_desc* d, const mi355_algo* algo,
                              const int8_t* src, const int8_t* filter, const int32_t* bias, const int8_t* z,
                              void* dst, void* workspace, size_t workspace_bytes, int warmup, int iters,
                              float* avg_usec);

/* tile configurations of the MFMA implicit-GEMM algorithm (values of mi355_algo.tile_cfg) */
int mi355_igemm_tile_count(void);
const char* mi355_igemm_tile_name(int tile_cfg);
/* MI355_OK if the MFMA algorithm runs descriptor `d` on exactly this tile (AlgoBase::is_available of the reference's
 * algorithm packs, dnn/src/cuda/conv_bias/algo.h: each tile is one algorithm there too).  A tile can be unavailable
 * for a packing (the LDS-direct tiles need 32-packed inputs), a dst dtype or bias shape (two tiles carry the general
 * epilogue) or a residual (ring + residual slot beyond the LDS of a CU).  exec() with such a tile: MI355_ERR_ALGO when the
 * caller named it, the tile that can run when the heuristic did (MI355_ALGO_FLAG_HEURISTIC). */
int mi355_igemm_tile_usable(const mi355_conv_desc* d, int tile_cfg);

/* The requantisation without z, dst = quantize_s8(act(float(sfb) * scale_bias)) with act IDENTITY or RELU
 * (dnn/src/naive/conv_bias/opr_impl.cpp:52,69-73,89-93; dnn/include/megdnn/dtype.h:845-853), is a step
 * function of the integer sfb.  When the library has proved that one fused multiply-add reproduces it on
 * every int32, dst = floor(min(max(fma(float(sfb), c, d), lo), 127.5)) with lo = 0 (RELU) or -128, its
 * kernels use that form.  Returns 1 and writes (c, d) if it has such a proof for these scales, 0 if not
 * (the kernels then run the multi-step form), a negative mi355_status on a bad argument.  Diagnostic:
 * no counterpart in the reference. */
int mi355_epilogue_linear_form(float scale_bias, float scale_dst, uint32_t nonline, float* c, float* d);

/* With a residual the same requantisation, dst = quantize_s8(act(float(sfb) * scale_bias + float(z) * scale_z)) with act
 * IDENTITY or RELU (dnn/src/naive/conv_bias/opr_impl.cpp:21-98), is a step function of the integer sfb for each of the
 * 256 values of the residual byte z.  When the library has proved, for every z and every int32 sfb, that
 *     dst = floor(min(max(fma(float(sfb), c, table[z & 255]), lo), 127.5))         lo = 0 (RELU) or -128
 * reproduces it, the kernels that hold the table in LDS use that form (five vector instructions and a table read per
 * output instead of nine).  Returns 1 and writes c and the 256 offsets (indexed by the residual byte as an unsigned
 * value) if it has such a proof for these scales -- it has none where scale_bias / scale_dst is below about 3e-3 --
 * 0 if not (the kernels then run the multi-step form), a negative mi355_status on a bad argument.  The first call for
 * a scale triple costs about a millisecond of host time.  Diagnostic: no counterpart in the reference. */
int mi355_epilogue_residual_table(float scale_bias, float scale_z, float scale_dst, uint32_t nonline, float* c,
                                  float* table);

/* The division r / scale_dst of the requantisation (dnn/include/megdnn/dtype.h:846) runs in the tiled kernels as
 *     t = r * y_lo;  q = fma(r, y_hi, t)          y_hi = RN(1 / scale_dst),  y_lo = RN(1 / scale_dst - y_hi)
 * -- a quotient at most one ulp from the correctly rounded one, which can change a result only next to a rounding
 * boundary of roundf.  The library uses it for a dst scale only after it has evaluated this form and the literal chain
 * (IEEE divide, roundf, clamp) on every float around every such boundary and found them equal; other scales run the
 * literal chain.  Returns 1 and the two parts of the reciprocal if the scale has passed, 0 if not, a negative
 * mi355_status on a bad argument.  Diagnostic: no counterpart in the reference. */
int mi355_epilogue_quotient_form(float scale_dst, float* y_hi, float* y_lo);

/* ---- RelayoutFormat ---- */
/* param::RelayoutFormat::Mode values (opr_param_defs.py:1069-1111); 32/33 and 34/35 are
 * extensions of this backend (the reference has no NCHW32 relayout mode). */
enum {
    MI355_RL_NCHW_NCHW4_IC_SMALL = 22,
    MI355_RL_NCHW_NCHW4 = 24,
    MI355_RL_NCHW4_NCHW = 25,
    MI355_RL_NCHW_NCHW4_WEIGHT = 26,
    MI355_RL_NCHW_NCHW32 = 32,
    MI355_RL_NCHW32_NCHW = 33,
    MI355_RL_NCHW4_NCHW32 = 34,
    MI355_RL_NCHW32_NCHW4 = 35
};

typedef struct mi355_relayout_desc {
    uint32_t mode;
    uint32_t ndim;         /* src ndim */
    uint32_t shape[7];     /* src shape */
    uint32_t group;        /* param.group (>= 1) */
    uint32_t oc;           /* param.oc (0 = keep all channels) */
    uint32_t elem_bytes;   /* 1 (int8) or 4 (int32/float32: pure permutation) */
    float scale_src;       /* QuantizedS8 scales; equal scales = pure byte permutation */
    float scale_dst;
} mi355_relayout_desc;

/* dst shape for the descriptor (dnn/src/common/relayout_format.cpp:7-296) */
int mi355_relayout_deduce(const mi355_relayout_desc* d, uint32_t* ndim, uint32_t shape[7]);
int mi355_relayout_exec(void* stream, const mi355_relayout_desc* d, const void* src, void* dst);

/* ---- stand-alone requantisation: dst[i] = quantize_s8(act(dequant_s32(src[i]) [+ dequant_s8(z[i])]), scale_dst) ----
 * The reference runs this as a separate pass over a QuantizedS32 convolution result
 * (handle_z_inp_and_activation_naive, naive/conv_bias/opr_impl.cpp:21-98), and a graph that keeps a convolution with
 * dst_dtype QuantizedS32 apart from its activation runs the same arithmetic as operators of its own: the unary
 * ElemwiseMultiType quantized modes QRELU / QH_SWISH from QuantizedS32 to QuantizedS8 (has_z = 0), and TypeCvt
 * QuantizedS32 -> QuantizedS8 (nonline IDENTITY, has_z = 0).  With has_z the chain is the post-process's own
 * TypeCvt -> float ADD -> activation -> TypeCvt.  Tensors are contiguous; src and dst need 16- and 4-byte alignment. */
typedef struct mi355_requant_desc {
    uint32_t nonline;   /* MI355_NL_* (no SIGMOID) */
    uint32_t has_z;
    float scale_src;    /* scale of the QuantizedS32 input */
    float scale_z;      /* scale of the QuantizedS8 second input */
    float scale_dst;
    uint32_t reserved;
    uint64_t count;     /* elements */
} mi355_requant_desc;
int mi355_requant_s32_s8_exec(void* stream, const mi355_requant_desc* d, const int32_t* src, const int8_t* z, int8_t* dst);
/* The same with a QuantizedS8 first operand (scale_src is its scale): the binary quantized modes of ElemwiseMultiType
 * on two QuantizedS8 tensors -- QADD (IDENTITY), QFUSE_ADD_RELU, QFUSE_ADD_H_SWISH: quantize(mode(dequantize(a),
 * dequantize(b))), dnn/src/naive/elemwise_multi_type/opr_impl.h:88-116, opr_impl_4.cpp:11-60, kernels
 * dnn/src/common/elemwise/kern_defs.cuh:52-55,:234,:268 -- and with has_z = 0 the unary QRELU / QH_SWISH and the
 * rescaling TypeCvt QuantizedS8 -> QuantizedS8.  The residual add of a network whose fuser left it outside ConvBias.
 * All three tensors need 16-byte alignment. */
int mi355_requant_s8_s8_exec(void* stream, const mi355_requant_desc* d, const int8_t* src, const int8_t* z, int8_t* dst);

/* ---- ElemwiseMultiType quantized modes in general: dst = quantize(mode(dequantize(a) [, dequantize(b) [, dequantize(c)]])) ----
 * ElemwiseMultiType::on_quantized_mode for one, two and three inputs (dnn/src/naive/elemwise_multi_type/opr_impl_3.cpp:
 * 11-60, opr_impl_4.cpp:11-66, opr_impl_5.cpp:11-45; the per-element drivers opr_impl.h:45-66, :88-116, :142-175):
 * every input is dequantized with its own scale (float(x) * scale, dnn/include/megdnn/dtype.h:854,:897), the float
 * kernel of the mode runs on the floats (dnn/src/common/elemwise/kern_defs.cuh:166-313), the result is quantized with
 * dst's scale (dtype.h:845-853 for QuantizedS8; :887-896 for QuantizedS32, which saturates at 2147483520).  The inputs
 * share one dtype (opr_impl_4.cpp:14-16), QuantizedS8 or QuantizedS32; dst is QuantizedS8 or QuantizedS32.
 * `mode` carries the reference's Elemwise::Mode enumerator values (dnn/scripts/opr_param_defs.py:341-455).  Served are
 * the modes whose float kernel is made of individually rounded IEEE operations, so that the result is defined bit for
 * bit; the modes that call the C math library (ACOS ASIN COS EXP EXPM1 LOG LOG1P SIGMOID SIN TANH ERF* POW LOG_SUM_EXP
 * FUSE_ADD_SIGMOID FUSE_ADD_TANH ATAN2 MOD) return MI355_ERR_UNSUPPORTED: their bits are a property of the host's libm.
 * The comparison modes produce 1.0f / 0.0f before the quantization, as the reference's float kernels do.
 * Contiguous tensors of `count` elements; QuantizedS8 tensors need 4-byte, QuantizedS32 tensors 16-byte alignment. */
enum {
    MI355_EW_RELU = 0, MI355_EW_ABS = 1, MI355_EW_CEIL = 4, MI355_EW_FLOOR = 8, MI355_EW_NEGATE = 11,
    MI355_EW_ABS_GRAD = 15, MI355_EW_ADD = 16, MI355_EW_FLOOR_DIV = 17, MI355_EW_MAX = 18, MI355_EW_MIN = 19,
    MI355_EW_MUL = 21, MI355_EW_SIGMOID_GRAD = 23, MI355_EW_SUB = 24, MI355_EW_SWITCH_GT0 = 25, MI355_EW_TANH_GRAD = 26,
    MI355_EW_TRUE_DIV = 27, MI355_EW_LT = 29, MI355_EW_LEQ = 30, MI355_EW_EQ = 31, MI355_EW_COND_LEQ_MOV = 34,
    MI355_EW_FUSE_MUL_ADD3 = 35, MI355_EW_FUSE_ADD_RELU = 37, MI355_EW_FAST_TANH = 40, MI355_EW_FAST_TANH_GRAD = 41,
    MI355_EW_ROUND = 42, MI355_EW_H_SWISH = 49, MI355_EW_H_SWISH_GRAD = 50, MI355_EW_FUSE_ADD_H_SWISH = 51,
    MI355_EW_COND_LT_MOV = 60
};
typedef struct mi355_elemwise_desc {
    uint32_t mode;        /* MI355_EW_* */
    uint32_t arity;       /* 1, 2 or 3: must be the mode's */
    uint32_t src_dtype;   /* MI355_DT_QS8 or MI355_DT_QS32, shared by the inputs */
    uint32_t dst_dtype;   /* MI355_DT_QS8 or MI355_DT_QS32 */
    float scale_src[3];
    float scale_dst;
    uint64_t count;       /* elements */
} mi355_elemwise_desc;
int mi355_elemwise_q_exec(void* stream, const mi355_elemwise_desc* d, const void* src0, const void* src1, const void* src2,
                          void* dst);

/* TypeCvt between Float32 and QuantizedS8, the quantize / dequantize at the two ends of an int8 network
 * (dnn/src/naive/type_cvt/opr_impl.cpp:24-56): Float32 -> QuantizedS8 is DTypeParamImpl<dt_qint8>::quantize =
 * saturate(roundf(x / scale)) (dnn/include/megdnn/dtype.h:845-853; NaN -> -128), QuantizedS8 -> Float32 is
 * float(x) * scale (dtype.h:854).  Contiguous tensors; the float side needs 16-byte, the int8 side 4-byte alignment. */
int mi355_typecvt_f32_s8_exec(void* stream, uint64_t count, float scale_dst, const float* src, int8_t* dst);
int mi355_typecvt_s8_f32_exec(void* stream, uint64_t count, float scale_src, const int8_t* src, float* dst);

/* ---- Pooling forward on QuantizedS8 (src and dst share one scale: the stored bytes are pooled) ----
 * megdnn::PoolingForward (dnn/include/megdnn/oprs/nn.h PoolingForward::exec; param::Pooling,
 * dnn/scripts/opr_param_defs.py:233-254) with the naive arithmetic (dnn/src/naive/pooling/opr_impl.cpp:16-36,
 * :107-127, :237-289): MAX over the part of the window inside the image; AVERAGE = roundf(float(sum) / (window_h *
 * window_w)), padding counted as zeros; AVERAGE_COUNT_EXCLUDE_PADDING = roundf(float(sum) / float(elements inside)).
 * format: MI355_FMT_NCHW, MI355_FMT_NCHW4, MI355_FMT_NCHW44 or MI355_FMT_NCHW32 (c a multiple of the pack).
 * Output size (dnn/src/common/pooling.cpp:7-125): (i + 2 * pad - window) / stride + 1.  A window that lies outside
 * the image completely is an error for MAX and AVERAGE_COUNT_EXCLUDE_PADDING, as in the reference (its message:
 * "The pooling window lies outside completely").  NCHW4 tensors need 4-byte, NCHW32 tensors 16-byte alignment. */
enum { MI355_POOL_MAX = 0, MI355_POOL_AVERAGE = 1, MI355_POOL_AVERAGE_COUNT_EXCLUDE_PADDING = 2 };
typedef struct mi355_pooling_desc {
    uint32_t mode;     /* MI355_POOL_* */
    uint32_t format;   /* MI355_FMT_* */
    uint32_t n, c, ih, iw;
    uint32_t pad_h, pad_w, stride_h, stride_w, window_h, window_w;
} mi355_pooling_desc;
int mi355_pooling_deduce_out(const mi355_pooling_desc* d, uint32_t* oh, uint32_t* ow);
int mi355_pooling_s8_exec(void* stream, const mi355_pooling_desc* d, const int8_t* src, int8_t* dst);

#ifdef __cplusplus
}
#endif
#endif /* MI355_CONVBIAS_H_ */
