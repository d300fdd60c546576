/*
 * convbias_oracle.c -- CPU restatement of MegDNN's naive quantized ConvBias,
 * RelayoutFormat, the requantising elementwise operators and QuantizedS8 Pooling.  TEST INFRASTRUCTURE ONLY: the parity checker for tests/, the smoke
 * check and the bench's cpu_baseline leg.  Nothing in the product library links, calls
 * or falls back to this file.
 *
 * Build with:  gcc -O2 -ffp-contract=off -fno-fast-math  (every float op below must be a
 * separately rounded IEEE binary32 operation).
 *
 * Each function cites the reference code it follows (paths relative to the MegEngine tree).
 * Pinning of each function (what independent evidence fixes it) is listed in oracle/README.md
 * and exercised by tests/test_oracle_*.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/mi355_convbias.h"

/* ------------------------------------------------------------------------------------ */
/* scalar pieces                                                                         */
/* ------------------------------------------------------------------------------------ */

/* DTypeParamImpl<dt_qint8>::quantize, dnn/include/megdnn/dtype.h:845-853:
 * true division, roundf (ties away from zero), fmax before fmin so NaN -> -128. */
int8_t oracle_quantize_s8(float x, float scale) {
    float v = x / scale;
    v = roundf(v);
    v = fminf(fmaxf(-128.f, v), 127.f);
    return (int8_t)v;
}

/* DTypeParamImpl<dt_qint32>::quantize, dtype.h:878-890 */
int32_t oracle_quantize_s32(float x, float scale) {
    float v = x / scale;
    v = roundf(v);
    v = fminf(fmaxf(-2147483648.f, v), 2147483520.f);
    return (int32_t)v;
}

/* dequantize: int -> float conversion (round to nearest even) then one multiply,
 * dtype.h:854 (s8) and :897 (s32) */
float oracle_dequantize_s8(int8_t v, float scale) { return (float)v * scale; }
float oracle_dequantize_s32(int32_t v, float scale) { return (float)v * scale; }

/* activation on float, dnn/src/common/elemwise/kern_defs.cuh:176 (RELU), :203 (H_SWISH).
 * H_SWISH is ((x * clamp(x + 3, 0, 6)) * (1/6)) with 1.f/6.f rounded once. */
float oracle_activation(float x, int nonline) {
    switch (nonline) {
        case MI355_NL_RELU:
            return x <= 0.f ? 0.f : x;
        case MI355_NL_H_SWISH: {
            float t = x + 3.f;
            t = t > 0.f ? t : 0.f;      /* max(x + 3, 0.f) */
            t = t < 6.f ? t : 6.f;      /* min(., 6.f)     */
            float r = x * t;
            return r * (1.f / 6.f);
        }
        default:
            return x;
    }
}

/* handle_z_inp_and_activation_naive, dnn/src/naive/conv_bias/opr_impl.cpp:21-98, applied to
 * one element.  sfb is the int32 conv+bias value carried in the bias dtype (scale s_bias).
 *   with z   : TypeCvt s32->f32 (:45), TypeCvt z->f32 (:46), float ADD (:48-50),
 *              float activation (:60-68), TypeCvt f32 -> dst (:67 / :89-93)
 *   without z: ElemwiseMultiType Q<mode> s32->dst (:69-73) or TypeCvt (:89-93); both are
 *              quantize(act(dequantize(sfb))) (naive/elemwise_multi_type/opr_impl.h:47-68,
 *              naive/type_cvt/opr_impl.cpp:24-56)
 */
float oracle_epilogue_float(int32_t sfb, float s_bias, int has_z, float zf, int nonline) {
    float r = oracle_dequantize_s32(sfb, s_bias);
    if (has_z) r = r + zf;
    return oracle_activation(r, nonline);
}

int8_t oracle_epilogue_s8(int32_t sfb, float s_bias, int has_z, int8_t z, float s_z, int nonline,
                          float s_dst) {
    float zf = has_z ? oracle_dequantize_s8(z, s_z) : 0.f;
    return oracle_quantize_s8(oracle_epilogue_float(sfb, s_bias, has_z, zf, nonline), s_dst);
}

int32_t oracle_epilogue_s32(int32_t sfb, float s_bias, int has_z, int32_t z, float s_z, int nonline,
                            float s_dst) {
    float zf = has_z ? oracle_dequantize_s32(z, s_z) : 0.f;
    return oracle_quantize_s32(oracle_epilogue_float(sfb, s_bias, has_z, zf, nonline), s_dst);
}

/* The post-process as a stand-alone pass over n elements (handle_z_inp_and_activation_naive,
 * naive/conv_bias/opr_impl.cpp:21-98); without z it is the unary ElemwiseMultiType Q<mode> s32 -> s8
 * (naive/elemwise_multi_type/opr_impl.h:47-68, opr_impl_3.cpp:12-59) or TypeCvt s32 -> s8
 * (naive/type_cvt/opr_impl.cpp:24-56).  Same scalar chain as oracle_epilogue_s8. */
int oracle_requant_s32_s8(const mi355_requant_desc* d, const int32_t* src, const int8_t* z, int8_t* dst) {
    if (d->nonline == MI355_NL_SIGMOID || d->nonline > MI355_NL_H_SWISH) return MI355_ERR_UNSUPPORTED;
    const int64_t n = (int64_t)d->count;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        dst[i] = oracle_epilogue_s8(src[i], d->scale_src, d->has_z != 0, d->has_z ? z[i] : 0, d->scale_z, (int)d->nonline,
                                    d->scale_dst);
    return MI355_OK;
}

/* Binary quantized ElemwiseMultiType modes on two QuantizedS8 tensors (ADD, FUSE_ADD_RELU, FUSE_ADD_H_SWISH) and the
 * unary ones without z: dst = quantize(mode(dequantize(a), dequantize(b))), naive/elemwise_multi_type/opr_impl.h:88-116;
 * the float kernels (common/elemwise/kern_defs.cuh:52-55 fuse_add_hswish, :234 ADD, :268 FUSE_ADD_RELU) are the
 * activation chain of oracle_epilogue_s8 applied to dequantize(a) + dequantize(b). */
int oracle_requant_s8_s8(const mi355_requant_desc* d, const int8_t* src, const int8_t* z, int8_t* dst) {
    if (d->nonline == MI355_NL_SIGMOID || d->nonline > MI355_NL_H_SWISH) return MI355_ERR_UNSUPPORTED;
    const int64_t n = (int64_t)d->count;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        dst[i] = oracle_epilogue_s8((int32_t)src[i], d->scale_src, d->has_z != 0, d->has_z ? z[i] : 0, d->scale_z,
                                    (int)d->nonline, d->scale_dst);
    return MI355_OK;
}

/* The float kernels of the quantized elemwise modes that use no libm function, transcribed expression by expression
 * from dnn/src/common/elemwise/kern_defs.cuh (unary :166-208, binary :229-295, ternary :311-313; fast_tanh :44-46,
 * fuse_add_hswish :52-55, fast_tanh_grad :57-61).  min / max there are std::min / std::max: max(a, b) = a < b ? b : a.
 * x * y + z is a multiply and an add (this file is built with -ffp-contract=off), what an x86-64 build of the
 * reference without FMA code generation evaluates.  Returns 0 for a mode outside the table (*ok = 0). */
static float omax(float a, float b) { return a < b ? b : a; }
static float omin(float a, float b) { return b < a ? b : a; }
static float oracle_elemwise_float(uint32_t mode, float x, float y, float z, int* ok) {
    *ok = 1;
    switch (mode) {
        case MI355_EW_RELU: return x <= 0.f ? 0.f : x;                                    /* :176 */
        case MI355_EW_ABS: return fabsf(x);                                               /* :182 */
        case MI355_EW_CEIL: return ceilf(x);                                              /* :187 */
        case MI355_EW_FLOOR: return floorf(x);                                            /* :191 */
        case MI355_EW_NEGATE: return -x;                                                  /* :166 */
        case MI355_EW_ROUND: return roundf(x);                                            /* :198 */
        case MI355_EW_FAST_TANH: return x * (27.f + x * x) / (27.f + 9.f * x * x);        /* :44-46 */
        case MI355_EW_H_SWISH: return x * omin(omax(x + 3, 0.f), 6.f) * (1.f / 6.f);      /* :203 */
        case MI355_EW_ABS_GRAD: return x > 0.f ? y : -y;                                  /* :230 */
        case MI355_EW_ADD: return x + y;                                                  /* :234 */
        case MI355_EW_FLOOR_DIV: return floorf(x / y);                                    /* :259 */
        case MI355_EW_MAX: return x > y ? x : y;                                          /* :235 */
        case MI355_EW_MIN: return x < y ? x : y;                                          /* :236 */
        case MI355_EW_MUL: return x * y;                                                  /* :237 */
        case MI355_EW_SIGMOID_GRAD: return x * (1.f - x) * y;                             /* :242 */
        case MI355_EW_SUB: return x - y;                                                  /* :243 */
        case MI355_EW_SWITCH_GT0: return x > 0.f ? y : 0.f;                               /* :246 */
        case MI355_EW_TANH_GRAD: return (1.f - x * x) * y;                                /* :250 */
        case MI355_EW_TRUE_DIV: return x / y;                                             /* :280 */
        case MI355_EW_LT: return (float)(x < y);                                          /* :251 */
        case MI355_EW_LEQ: return (float)(x <= y);                                        /* :252 */
        case MI355_EW_EQ: return (float)(x == y);                                         /* :253 */
        case MI355_EW_FUSE_ADD_RELU: return (x + y) <= 0.f ? 0.f : (x + y);               /* :268 */
        case MI355_EW_FAST_TANH_GRAD: {                                                   /* :57-61 */
            float x_pow2 = x * x;
            float deno = 3.f + x_pow2;
            return ((-48.f * x_pow2) / deno + 27.f + x_pow2) / (deno * 9.f) * y;
        }
        case MI355_EW_H_SWISH_GRAD:                                                       /* :287-290 */
            return x < -3.f ? 0.f : (x > 3.f ? y : (2.f * x + 3.f) / 6.f * y);
        case MI355_EW_FUSE_ADD_H_SWISH: {                                                 /* :52-55 */
            float t = x + y;
            return t * omin(omax(t + 3, 0.f), 6.f) * (1.f / 6.f);
        }
        case MI355_EW_COND_LEQ_MOV: return x <= y ? z : 0.f;                              /* :311 */
        case MI355_EW_COND_LT_MOV: return x < y ? z : 0.f;                                /* :312 */
        case MI355_EW_FUSE_MUL_ADD3: return x * y + z;                                    /* :313 */
        default: *ok = 0; return 0.f;
    }
}

/* ElemwiseMultiType::on_quantized_mode, naive: dst = dst_param.quantize(KernImpl::apply(param0.dequantize(a), ...))
 * (dnn/src/naive/elemwise_multi_type/opr_impl.h:45-66 one input, :88-116 two, :142-175 three); dequantize =
 * float(x) * scale (dtype.h:854, :897).  Inputs share one dtype; src and dst are int8 or int32 arrays. */
int oracle_elemwise_q(const mi355_elemwise_desc* d, const void* s0, const void* s1, const void* s2, void* dst) {
    int ok;
    (void)oracle_elemwise_float(d->mode, 0.f, 0.f, 0.f, &ok);
    if (!ok) return MI355_ERR_UNSUPPORTED;
    if (d->arity < 1 || d->arity > 3) return MI355_ERR_BAD_ARG;
    const void* src[3] = {s0, s1, s2};
    const int s32 = d->src_dtype == MI355_DT_QS32, d32 = d->dst_dtype == MI355_DT_QS32;
    for (uint64_t i = 0; i < d->count; ++i) {
        float v[3] = {0.f, 0.f, 0.f};
        for (uint32_t k = 0; k < d->arity; ++k)
            v[k] = (s32 ? (float)((const int32_t*)src[k])[i] : (float)((const int8_t*)src[k])[i]) * d->scale_src[k];
        const float r = oracle_elemwise_float(d->mode, v[0], v[1], v[2], &ok);
        if (d32)
            ((int32_t*)dst)[i] = oracle_quantize_s32(r, d->scale_dst);
        else
            ((int8_t*)dst)[i] = oracle_quantize_s8(r, d->scale_dst);
    }
    return MI355_OK;
}

/* TypeCvt Float32 <-> QuantizedS8 over n elements (naive/type_cvt/opr_impl.cpp:24-56: quantize / dequantize of
 * dtype.h:845-854, the scalar functions above) */
void oracle_typecvt_f32_s8(uint64_t n, float scale, const float* src, int8_t* dst) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = oracle_quantize_s8(src[i], scale);
}
void oracle_typecvt_s8_f32(uint64_t n, float scale, const int8_t* src, float* dst) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = oracle_dequantize_s8(src[i], scale);
}

/* ------------------------------------------------------------------------------------ */
/* Pooling forward on dt_qint8                                                           */
/* ------------------------------------------------------------------------------------ */

/* element index of (n, c, h, w): the IdxGetters of dnn/src/naive/pooling/opr_impl.cpp:129-186
 * (NCHW :129-135, NCHW4 :153-159, NCHW44 :168-175, NCHW32 :185-191) */
static size_t pool_idx(int pack, size_t n, size_t c, size_t h, size_t w, size_t C, size_t H, size_t W) {
    if (pack == 1) return ((n * C + c) * H + h) * W + w;
    return (((n * (C / (size_t)pack) + c / (size_t)pack) * H + h) * W + w) * (size_t)pack + c % (size_t)pack;
}

/* pooling_forward_impl (naive/pooling/opr_impl.cpp:270-289) with the dt_qint8 poolers: MaxPooler (:16-36),
 * MeanIncludePooler<dt_qint8> = MeanIncludeRoundedPooler (:107-127: round(float(sum) / count), count = window),
 * MeanExcludePooler<dt_qint8> = MeanExcludeRoundedPooler (:237-268: count = elements fed).  The bounds test uses the
 * reference's unsigned wrap-around (ih = -PH + oh * SH + fh as size_t, valid when < IH).  A window without a
 * valid element makes MAX and the excluding mean throw: status MI355_ERR_SHAPE here. */
int oracle_pooling_s8(const mi355_pooling_desc* d, const int8_t* src, int8_t* dst) {
    int pack;
    switch (d->format) {
        case MI355_FMT_NCHW: pack = 1; break;
        case MI355_FMT_NCHW4:
        case MI355_FMT_NCHW44: pack = 4; break;
        case MI355_FMT_NCHW32: pack = 32; break;
        default: return MI355_ERR_UNSUPPORTED;
    }
    if (d->mode > MI355_POOL_AVERAGE_COUNT_EXCLUDE_PADDING) return MI355_ERR_UNSUPPORTED;
    const size_t N = d->n, C = d->c, IH = d->ih, IW = d->iw;
    const size_t PH = d->pad_h, PW = d->pad_w, SH = d->stride_h, SW = d->stride_w, FH = d->window_h, FW = d->window_w;
    if (C % (size_t)pack || !FH || !FW || !SH || !SW || IH + 2 * PH < FH || IW + 2 * PW < FW) return MI355_ERR_SHAPE;
    const size_t OH = (IH + 2 * PH - FH) / SH + 1, OW = (IW + 2 * PW - FW) / SW + 1;
    int status = MI355_OK;
#pragma omp parallel for collapse(2) schedule(static)
    for (size_t n = 0; n < N; ++n)
        for (size_t c = 0; c < C; ++c)
            for (size_t oh = 0; oh < OH; ++oh)
                for (size_t ow = 0; ow < OW; ++ow) {
                    int8_t best = INT8_MIN;
                    int32_t sum = 0;
                    size_t fed = 0;
                    for (size_t fh = 0; fh < FH; ++fh)
                        for (size_t fw = 0; fw < FW; ++fw) {
                            const size_t ih = -PH + oh * SH + fh, iw = -PW + ow * SW + fw;
                            if (ih < IH && iw < IW) {
                                const int8_t x = src[pool_idx(pack, n, c, ih, iw, C, IH, IW)];
                                best = best > x ? best : x;
                                sum += (int32_t)x;
                                ++fed;
                            }
                        }
                    int8_t r;
                    if (d->mode == MI355_POOL_AVERAGE) {
                        const int32_t count = (int32_t)(FH * FW);
                        r = (int8_t)roundf((float)sum / count);
                    } else if (!fed) {
                        status = MI355_ERR_SHAPE;
                        r = 0;
                    } else if (d->mode == MI355_POOL_MAX) {
                        r = best;
                    } else {
                        r = (int8_t)roundf((float)sum / fed);
                    }
                    dst[pool_idx(pack, n, c, oh, ow, C, OH, OW)] = r;
                }
    return status;
}

/* infer_conv_shape, dnn/src/common/utils.cpp:130-138 */
static uint32_t out_size(uint32_t i, uint32_t f, uint32_t d, uint32_t s, uint32_t p) {
    uint32_t df = (f - 1) * d + 1;
    return (i + 2 * p - df) / s + 1;
}

/* ------------------------------------------------------------------------------------ */
/* addressing (naive/convolution/helper.h:292-381 activations, :383-463 filters)         */
/* ------------------------------------------------------------------------------------ */

static int in_pack(uint32_t fmt) {
    switch (fmt) {
        case MI355_FMT_NCHW: return 1;
        case MI355_FMT_NCHW4: case MI355_FMT_NCHW44: case MI355_FMT_NCHW4_NCHW32: case MI355_FMT_NCHW4_NCHW: return 4;
        default: return 32;
    }
}
static int out_pack(uint32_t fmt) {
    switch (fmt) {
        case MI355_FMT_NCHW: case MI355_FMT_NCHW4_NCHW: return 1;
        case MI355_FMT_NCHW4: case MI355_FMT_NCHW44: case MI355_FMT_NCHW32_NCHW4: return 4;
        default: return 32;
    }
}

/* offset of logical element (n, c, h, w) in a (N, C/p, H, W, p) tensor, p = 1 gives NCHW */
static int64_t act_off(int64_t stride_n, int p, int64_t C, int64_t H, int64_t W, int64_t n, int64_t c,
                       int64_t h, int64_t w) {
    int64_t sn = stride_n ? stride_n : C * H * W;
    return n * sn + (c / p) * (H * W * p) + h * (W * p) + w * p + (c % p);
}

/* true when the descriptor is the channel-wise packed-by-4 case (NCHW44 "chan" filter
 * (g/4,1,1,fh,fw,4), helper.h:419-424), also accepted under Format::NCHW4 as an extension */
static int is_dw4(const mi355_conv_desc* d, uint32_t icpg, uint32_t ocpg) {
    return (d->format == MI355_FMT_NCHW44 || d->format == MI355_FMT_NCHW4) && d->group > 1 &&
           icpg == 1 && ocpg == 1;
}

static int64_t flt_off(const mi355_conv_desc* d, uint32_t icpg, uint32_t ocpg, uint32_t g, uint32_t oc_in_g,
                       uint32_t ic_in_g, uint32_t fh, uint32_t fw) {
    const int64_t FH = d->fh, FW = d->fw;
    if (is_dw4(d, icpg, ocpg)) {
        /* FS_SPATIAL = 4, FS_IC = FH*FW*4, FS_OC = FS_IC, FS_G = FS_OC   (helper.h:251-256) */
        return (int64_t)(g / 4) * (FH * FW * 4) + (fh * FW + fw) * 4 + (g % 4);
    }
    switch (d->format) {
        case MI355_FMT_NCHW: {
            /* g, oc, ic, fh, fw: FS_IC = FH*FW, FS_OC = FS_IC*icpg, FS_G = FS_OC*ocpg (:217-221) */
            int64_t FS_OC = FH * FW * icpg, FS_G = FS_OC * ocpg;
            return g * FS_G + oc_in_g * FS_OC + ic_in_g * (FH * FW) + fh * FW + fw;
        }
        case MI355_FMT_NCHW44: {
            /* normal case: FS_SPATIAL = 16, FS_IC = FH*FW*16, FS_OC = FS_IC*icpg/4,
             * FS_G = FS_OC*ocpg/4 (:257-262); element (:425-430) */
            int64_t FS_SP = 16, FS_IC = FH * FW * FS_SP, FS_OC = FS_IC * icpg / 4, FS_G = FS_OC * ocpg / 4;
            return g * FS_G + (oc_in_g / 4) * FS_OC + (ic_in_g / 4) * FS_IC + (fh * FW + fw) * FS_SP +
                   (ic_in_g % 4) * 4 + (oc_in_g % 4);
        }
        default: {
            /* NCHW4 / NCHW32 / mixed: (:385-401) */
            int p = in_pack(d->format);
            int64_t FS_OC = FH * FW * icpg, FS_G = FS_OC * ocpg;
            return g * FS_G + oc_in_g * FS_OC + (ic_in_g / p) * (FH * FW * p) + (fh * FW + fw) * p +
                   (ic_in_g % p);
        }
    }
}

/* ------------------------------------------------------------------------------------ */
/* ConvBias                                                                              */
/* ------------------------------------------------------------------------------------ */

static int check_desc(const mi355_conv_desc* d, uint32_t* icpg, uint32_t* ocpg) {
    if (!d || !d->group || !d->n || !d->fh || !d->fw || !d->stride_h || !d->stride_w) return MI355_ERR_BAD_ARG;
    if (d->sparse == MI355_SPARSE_DENSE && d->group != 1) return MI355_ERR_SHAPE;
    if (d->ic % d->group || d->oc % d->group) return MI355_ERR_SHAPE;
    *icpg = d->ic / d->group;
    *ocpg = d->oc / d->group;
    int pi = in_pack(d->format), po = out_pack(d->format);
    if (d->format != MI355_FMT_NCHW && (d->dilate_h != 1 || d->dilate_w != 1))
        return MI355_ERR_SHAPE; /* convolution.cpp:411-414 */
    if (!is_dw4(d, *icpg, *ocpg)) {
        if (*icpg % pi) return MI355_ERR_SHAPE;
        if (d->format == MI355_FMT_NCHW44 && (*ocpg % 4)) return MI355_ERR_SHAPE;
    } else if (d->group % 4) {
        return MI355_ERR_SHAPE;
    }
    if (d->oc % po) return MI355_ERR_SHAPE;
    if (d->nonline == MI355_NL_SIGMOID || d->nonline > MI355_NL_H_SWISH) return MI355_ERR_UNSUPPORTED;
    if (d->has_z && (d->format == MI355_FMT_NCHW4_NCHW32 || d->format == MI355_FMT_NCHW32_NCHW4))
        return MI355_ERR_SHAPE; /* common/conv_bias.cpp:127-129 */
    {
        uint32_t dfh = (d->fh - 1) * d->dilate_h + 1, dfw = (d->fw - 1) * d->dilate_w + 1;
        if (d->ih + 2 * d->pad_h < dfh || d->iw + 2 * d->pad_w < dfw) return MI355_ERR_SHAPE;
    }
    return MI355_OK;
}

/* one output element of naive compute2d (helper.h:466-502): the fh/fw/ic loops with zero
 * padding by skipping out-of-range taps and int32 wraparound accumulation. */
static int32_t acc_one(const mi355_conv_desc* d, uint32_t icpg, uint32_t ocpg, const int8_t* src, const int8_t* flt,
                       uint32_t n, uint32_t oc, uint32_t oh, uint32_t ow) {
    const int pi = in_pack(d->format);
    /* should_flip (helper.h:285-290): h_offset += dilated_spatial - 1, dilation negated */
    int h_offset = -(int)d->pad_h, w_offset = -(int)d->pad_w;
    int dh = (int)d->dilate_h, dw = (int)d->dilate_w;
    if (d->mode == MI355_MODE_CONVOLUTION) {
        h_offset += (int)((d->fh - 1) * d->dilate_h);
        w_offset += (int)((d->fw - 1) * d->dilate_w);
        dh = -dh;
        dw = -dw;
    }
    const uint32_t g = oc / ocpg, oc_in_g = oc % ocpg; /* GroupCounter, helper.h:12-24 */
    int32_t acc = 0;                                    /* StrategyFwd::init_dval, helper.h:37-40 */
    for (uint32_t fh = 0; fh < d->fh; ++fh)
        for (uint32_t fw = 0; fw < d->fw; ++fw) {
            int64_t ih = (int64_t)d->stride_h * oh + (int64_t)fh * dh + h_offset;
            int64_t iw = (int64_t)d->stride_w * ow + (int64_t)fw * dw + w_offset;
            if (ih < 0 || ih >= (int64_t)d->ih || iw < 0 || iw >= (int64_t)d->iw) continue;
            for (uint32_t ic = 0; ic < icpg; ++ic) {
                int32_t s = src[act_off(d->src_stride_n, pi, d->ic, d->ih, d->iw, n, (int64_t)g * icpg + ic, ih, iw)];
                int32_t f = flt[flt_off(d, icpg, ocpg, g, oc_in_g, ic, fh, fw)];
                /* StrategyFwd::on for qint8: int32 multiply-add with wraparound (helper.h:67-74) */
                acc = (int32_t)((uint32_t)acc + (uint32_t)(s * f));
            }
        }
    return acc;
}

/* integer part: naive compute2d + bias add (helper.h:732-803), writes the int32 "sfb" tensor in
 * dst layout (shape and pack of dst, dense batch). */
int oracle_convbias_s8_acc(const mi355_conv_desc* d, const int8_t* src, const int8_t* flt, const int32_t* bias,
                           int32_t* sfb) {
    uint32_t icpg, ocpg;
    int st = check_desc(d, &icpg, &ocpg);
    if (st) return st;
    const int po = out_pack(d->format);
    const uint32_t OH = out_size(d->ih, d->fh, d->dilate_h, d->stride_h, d->pad_h);
    const uint32_t OW = out_size(d->iw, d->fw, d->dilate_w, d->stride_w, d->pad_w);
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t n = 0; n < d->n; ++n) {
        for (uint32_t oc = 0; oc < d->oc; ++oc) {
            for (uint32_t oh = 0; oh < OH; ++oh)
                for (uint32_t ow = 0; ow < OW; ++ow) {
                    int32_t acc = acc_one(d, icpg, ocpg, src, flt, n, oc, oh, ow);
                    int64_t o = act_off(0, po, d->oc, OH, OW, n, oc, oh, ow);
                    if (d->bias_mode == MI355_BIAS_BROADCAST_CHANNEL)
                        acc = (int32_t)((uint32_t)acc + (uint32_t)bias[oc]); /* bias is linear in channel */
                    else if (d->bias_mode == MI355_BIAS_FULL)
                        acc = (int32_t)((uint32_t)acc + (uint32_t)bias[o]);
                    sfb[o] = acc;
                }
        }
    }
    return MI355_OK;
}

/* The operator evaluated at `count` chosen output elements only (for spot checks at sizes where
 * the whole tensor would take too long).  idx[i] is a linear index into the dense dst tensor
 * (n, oc/p, oh, ow, p); QuantizedS8 dst only.  z is addressed with z_stride_n. */
int oracle_convbias_s8_points(const mi355_conv_desc* d, const int8_t* src, const int8_t* flt, const int32_t* bias,
                              const int8_t* z, const int64_t* idx, int64_t count, int8_t* out) {
    uint32_t icpg, ocpg;
    int st = check_desc(d, &icpg, &ocpg);
    if (st) return st;
    if (d->dst_dtype != MI355_DT_QS8) return MI355_ERR_UNSUPPORTED;
    const int po = out_pack(d->format);
    const int64_t OH = out_size(d->ih, d->fh, d->dilate_h, d->stride_h, d->pad_h);
    const int64_t OW = out_size(d->iw, d->fw, d->dilate_w, d->stride_w, d->pad_w);
    const int64_t per_n = (int64_t)d->oc * OH * OW;
    const int64_t zsn = d->z_stride_n ? d->z_stride_n : per_n;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < count; ++i) {
        int64_t t = idx[i];
        int64_t n = t / per_n, r = t % per_n;
        int64_t k = r % po, q = r / po;
        int64_t ow = q % OW;
        q /= OW;
        int64_t oh = q % OH, ocb = q / OH;
        uint32_t oc = (uint32_t)(ocb * po + k);
        int32_t acc = acc_one(d, icpg, ocpg, src, flt, (uint32_t)n, oc, (uint32_t)oh, (uint32_t)ow);
        if (d->bias_mode == MI355_BIAS_BROADCAST_CHANNEL)
            acc = (int32_t)((uint32_t)acc + (uint32_t)bias[oc]);
        else if (d->bias_mode == MI355_BIAS_FULL)
            acc = (int32_t)((uint32_t)acc + (uint32_t)bias[t]);
        int8_t zv = d->has_z ? z[n * zsn + r] : 0;
        out[i] = oracle_epilogue_s8(acc, d->scale_bias, d->has_z, zv, d->scale_z, d->nonline, d->scale_dst);
    }
    return MI355_OK;
}

/* full operator: naive::ConvBiasForwardImpl::exec (conv_bias/opr_impl.cpp:211-292) */
/* Float32 dst (NCHW4_NCHW): StrategyFwd::on for (qint8, qint8) -> float, helper.h:59-66: every product is
 * dequantize(s) * dequantize(f) in float, added to a float running sum in the loop order of compute2d (fh, fw, ic;
 * padded taps skipped, helper.h:466-502); then the bias (float add, helper.h:732-760), z (Elemwise ADD) and the float
 * activation (naive/conv_bias/opr_impl.cpp:21-98).  scale_bias / scale_z of the descriptor hold the scales of src and
 * filter. */
static int oracle_convbias_s8_f32(const mi355_conv_desc* d, uint32_t icpg, uint32_t ocpg, const int8_t* src,
                                  const int8_t* flt, const float* bias, const float* z, float* dst) {
    if (d->format != MI355_FMT_NCHW4_NCHW) return MI355_ERR_UNSUPPORTED;
    const uint32_t OH = out_size(d->ih, d->fh, d->dilate_h, d->stride_h, d->pad_h);
    const uint32_t OW = out_size(d->iw, d->fw, d->dilate_w, d->stride_w, d->pad_w);
    const int64_t per_n = (int64_t)d->oc * OH * OW;
    const int64_t dsn = d->dst_stride_n ? d->dst_stride_n : per_n;
    const int64_t zsn = d->z_stride_n ? d->z_stride_n : per_n;
    const float ss = d->scale_bias, sf = d->scale_z;
    int h_offset = -(int)d->pad_h, w_offset = -(int)d->pad_w;
    int dh = 1, dw = 1;
    if (d->mode == MI355_MODE_CONVOLUTION) {
        h_offset += (int)(d->fh - 1);
        w_offset += (int)(d->fw - 1);
        dh = dw = -1;
    }
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t n = 0; n < d->n; ++n)
        for (uint32_t oc = 0; oc < d->oc; ++oc) {
            const uint32_t g = oc / ocpg, oc_in_g = oc % ocpg;
            for (uint32_t oh = 0; oh < OH; ++oh)
                for (uint32_t ow = 0; ow < OW; ++ow) {
                    float dval = 0.f;
                    for (uint32_t fh = 0; fh < d->fh; ++fh)
                        for (uint32_t fw = 0; fw < d->fw; ++fw) {
                            int64_t ih = (int64_t)d->stride_h * oh + (int64_t)fh * dh + h_offset;
                            int64_t iw = (int64_t)d->stride_w * ow + (int64_t)fw * dw + w_offset;
                            if (ih < 0 || ih >= (int64_t)d->ih || iw < 0 || iw >= (int64_t)d->iw) continue;
                            for (uint32_t ic = 0; ic < icpg; ++ic) {
                                float s = (float)src[act_off(d->src_stride_n, 4, d->ic, d->ih, d->iw, n,
                                                             (int64_t)g * icpg + ic, ih, iw)] * ss;
                                float f = (float)flt[flt_off(d, icpg, ocpg, g, oc_in_g, ic, fh, fw)] * sf;
                                float prod = s * f;
                                dval = dval + prod;
                            }
                        }
                    const int64_t i = ((int64_t)oc * OH + oh) * OW + ow;
                    if (d->bias_mode == MI355_BIAS_BROADCAST_CHANNEL)
                        dval = dval + bias[oc];
                    else if (d->bias_mode == MI355_BIAS_FULL)
                        dval = dval + bias[(int64_t)n * per_n + i];
                    if (d->has_z) dval = dval + z[n * zsn + i];
                    dst[n * dsn + i] = oracle_activation(dval, (int)d->nonline);
                }
        }
    return MI355_OK;
}

int oracle_convbias_s8(const mi355_conv_desc* d, const int8_t* src, const int8_t* flt, const int32_t* bias,
                       const void* z, void* dst) {
    uint32_t icpg, ocpg;
    int st = check_desc(d, &icpg, &ocpg);
    if (st) return st;
    if (d->dst_dtype == MI355_DT_F32)
        return oracle_convbias_s8_f32(d, icpg, ocpg, src, flt, (const float*)bias, (const float*)z, (float*)dst);
    const int po = out_pack(d->format);
    const uint32_t OH = out_size(d->ih, d->fh, d->dilate_h, d->stride_h, d->pad_h);
    const uint32_t OW = out_size(d->iw, d->fw, d->dilate_w, d->stride_w, d->pad_w);
    const int64_t per_n = (int64_t)d->oc * OH * OW;
    int32_t* sfb = (int32_t*)malloc(sizeof(int32_t) * (size_t)per_n * d->n);
    if (!sfb) return MI355_ERR_BAD_ARG;
    st = oracle_convbias_s8_acc(d, src, flt, bias, sfb);
    if (st) {
        free(sfb);
        return st;
    }
    const int64_t dsn = d->dst_stride_n ? d->dst_stride_n : per_n;
    const int64_t zsn = d->z_stride_n ? d->z_stride_n : per_n;
    (void)po;
    for (uint32_t n = 0; n < d->n; ++n)
        for (int64_t i = 0; i < per_n; ++i) {
            int32_t v = sfb[n * per_n + i];
            if (d->dst_dtype == MI355_DT_QS8) {
                int8_t zv = d->has_z ? ((const int8_t*)z)[n * zsn + i] : 0;
                ((int8_t*)dst)[n * dsn + i] =
                        oracle_epilogue_s8(v, d->scale_bias, d->has_z, zv, d->scale_z, d->nonline, d->scale_dst);
            } else {
                /* QuantizedS32 dst: bias and dst have the same dtype enum, so the reference accumulates straight into
                 * dst (sfb = dst, naive/conv_bias/opr_impl.cpp:223-228).  IDENTITY without z then leaves the raw sum
                 * where it is (res.raw_ptr() == dst.raw_ptr(), :52,:89-93): no float round trip, the scales are not
                 * used.  Every other case dequantises that tensor with ITS dtype, i.e. with the scale of dst (:44-46 TypeCvt
                 * of conv_bias_tensor = dst; :69-73 ElemwiseMultiType reads param0 from the dtype of res = dst,
                 * naive/elemwise_multi_type/opr_impl.h:54-60), never with the scale of the bias tensor. */
                if (d->nonline == MI355_NL_IDENTITY && !d->has_z) {
                    ((int32_t*)dst)[n * dsn + i] = v;
                } else {
                    int32_t zv = d->has_z ? ((const int32_t*)z)[n * zsn + i] : 0;
                    ((int32_t*)dst)[n * dsn + i] =
                            oracle_epilogue_s32(v, d->scale_dst, d->has_z, zv, d->scale_z, d->nonline, d->scale_dst);
                }
            }
        }
    free(sfb);
    return MI355_OK;
}

/* ------------------------------------------------------------------------------------ */
/* RelayoutFormat                                                                        */
/* ------------------------------------------------------------------------------------ */

static uint32_t cdiv(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

/* dst shapes: dnn/src/common/relayout_format.cpp:19-27 (IC_SMALL), :209-220 (NCHW_NCHW4),
 * :221-242 (WEIGHT), :243-251 (NCHW4_NCHW).  The NCHW32 modes are this backend's extension,
 * defined as the same rules with pack 32 (NCHW<->NCHW32) or as the channel-preserving
 * re-blocking (NCHW4<->NCHW32), cf. from_nchw4_to_nchw32 in dnn/test/naive/conv_bias.cpp:222-269. */
int oracle_relayout_deduce(const mi355_relayout_desc* d, uint32_t* ndim, uint32_t shape[7]) {
    const uint32_t* s = d->shape;
    uint32_t g = d->group ? d->group : 1;
    switch (d->mode) {
        case MI355_RL_NCHW_NCHW4_IC_SMALL:
            if (d->ndim != 4 || s[1] > 4) return MI355_ERR_SHAPE;
            *ndim = 5; shape[0] = s[0]; shape[1] = cdiv(s[1], 4); shape[2] = s[2]; shape[3] = s[3]; shape[4] = 4;
            return MI355_OK;
        case MI355_RL_NCHW_NCHW4:
        case MI355_RL_NCHW_NCHW32: {
            uint32_t p = d->mode == MI355_RL_NCHW_NCHW4 ? 4 : 32;
            if (d->ndim != 4 || s[1] % g) return MI355_ERR_SHAPE;
            *ndim = 5; shape[0] = s[0]; shape[1] = g * cdiv(s[1] / g, p); shape[2] = s[2]; shape[3] = s[3];
            shape[4] = p;
            return MI355_OK;
        }
        case MI355_RL_NCHW4_NCHW:
        case MI355_RL_NCHW32_NCHW: {
            uint32_t p = d->mode == MI355_RL_NCHW4_NCHW ? 4 : 32;
            if (d->ndim != 5 || s[4] != p) return MI355_ERR_SHAPE;
            uint32_t c = d->oc ? d->oc : s[1] * p;
            if (c % g || c > s[1] * p) return MI355_ERR_SHAPE;
            if (g * cdiv(c / g, p) != s[1]) return MI355_ERR_SHAPE;
            *ndim = 4; shape[0] = s[0]; shape[1] = c; shape[2] = s[2]; shape[3] = s[3];
            return MI355_OK;
        }
        case MI355_RL_NCHW_NCHW4_WEIGHT:
            if (d->ndim == 4) {
                *ndim = 5; shape[0] = cdiv(s[0], 4) * 4; shape[1] = cdiv(s[1], 4); shape[2] = s[2];
                shape[3] = s[3]; shape[4] = 4;
                return MI355_OK;
            } else if (d->ndim == 5) {
                *ndim = 6; shape[0] = s[0]; shape[1] = cdiv(s[1], 4) * 4; shape[2] = cdiv(s[2], 4);
                shape[3] = s[3]; shape[4] = s[4]; shape[5] = 4;
                return MI355_OK;
            }
            return MI355_ERR_SHAPE;
        case MI355_RL_NCHW4_NCHW32:
            if (d->ndim != 5 || s[4] != 4 || s[1] % 8) return MI355_ERR_SHAPE;
            *ndim = 5; shape[0] = s[0]; shape[1] = s[1] / 8; shape[2] = s[2]; shape[3] = s[3]; shape[4] = 32;
            return MI355_OK;
        case MI355_RL_NCHW32_NCHW4:
            if (d->ndim != 5 || s[4] != 32) return MI355_ERR_SHAPE;
            *ndim = 5; shape[0] = s[0]; shape[1] = s[1] * 8; shape[2] = s[2]; shape[3] = s[3]; shape[4] = 4;
            return MI355_OK;
        default:
            return MI355_ERR_UNSUPPORTED;
    }
}

/* naive::RelayoutFormatImpl::exec (naive/relayout_format/opr_impl.cpp:486-773): dst is
 * cleared, the (zero-padded) source is permuted, and for QuantizedS8 -> QuantizedS8 every
 * copied element goes through quantize_dst(dequantize_src(x)) (do_copy_diff_q8_q8, :255-265). */
static void put(const mi355_relayout_desc* d, void* dst, int64_t di, const void* src, int64_t si) {
    if (d->elem_bytes == 4) {
        ((int32_t*)dst)[di] = si < 0 ? 0 : ((const int32_t*)src)[si];
    } else {
        int8_t v = si < 0 ? 0 : ((const int8_t*)src)[si];
        if (d->scale_src != d->scale_dst) v = oracle_quantize_s8(oracle_dequantize_s8(v, d->scale_src), d->scale_dst);
        ((int8_t*)dst)[di] = v;
    }
}

int oracle_relayout(const mi355_relayout_desc* d, const void* src, void* dst) {
    uint32_t ondim, os[7];
    int st = oracle_relayout_deduce(d, &ondim, os);
    if (st) return st;
    const uint32_t* s = d->shape;
    const uint32_t g = d->group ? d->group : 1;
    switch (d->mode) {
        case MI355_RL_NCHW_NCHW4_IC_SMALL:
        case MI355_RL_NCHW_NCHW4:
        case MI355_RL_NCHW_NCHW32: {
            /* dst[n][gi*cpb + cb][h][w][k] = src[n][gi*icpg + cb*p + k][h][w], zero when
             * cb*p + k >= icpg (per-group padding, relayout_format.cpp:458-473) */
            const int64_t p = os[4], N = s[0], C = s[1], H = s[2], W = s[3];
            const int64_t gg = d->mode == MI355_RL_NCHW_NCHW4_IC_SMALL ? 1 : g;
            const int64_t icpg = C / gg, cpb = os[1] / gg;
            for (int64_t n = 0; n < N; ++n)
                for (int64_t gi = 0; gi < gg; ++gi)
                    for (int64_t cb = 0; cb < cpb; ++cb)
                        for (int64_t h = 0; h < H; ++h)
                            for (int64_t w = 0; w < W; ++w)
                                for (int64_t k = 0; k < p; ++k) {
                                    int64_t cin = cb * p + k;
                                    int64_t di = (((n * os[1] + gi * cpb + cb) * H + h) * W + w) * p + k;
                                    int64_t si = cin < icpg ? ((n * C + gi * icpg + cin) * H + h) * W + w : -1;
                                    put(d, dst, di, src, si);
                                }
            return MI355_OK;
        }
        case MI355_RL_NCHW4_NCHW:
        case MI355_RL_NCHW32_NCHW: {
            /* inverse with optional crop: dst channel c = gi*ocpg + ci reads packed channel
             * gi*cpb*p + ci (extract_from_workspace, naive :761-769) */
            const int64_t p = s[4], N = s[0], CB = s[1], H = s[2], W = s[3], C = os[1];
            const int64_t ocpg = C / g, cpb = CB / g;
            for (int64_t n = 0; n < N; ++n)
                for (int64_t c = 0; c < C; ++c) {
                    int64_t gi = c / ocpg, ci = c % ocpg;
                    int64_t pc = gi * cpb * p + ci;
                    for (int64_t h = 0; h < H; ++h)
                        for (int64_t w = 0; w < W; ++w) {
                            int64_t si = (((n * CB + pc / p) * H + h) * W + w) * p + pc % p;
                            int64_t di = ((n * C + c) * H + h) * W + w;
                            put(d, dst, di, src, si);
                        }
                }
            return MI355_OK;
        }
        case MI355_RL_NCHW_NCHW4_WEIGHT: {
            /* dense (OC,IC,FH,FW) -> (ceil4(OC), ceil(IC/4), FH, FW, 4); group adds a leading
             * G and pads per group (relayout_format.cpp:221-242, :474-503) */
            const int grp = d->ndim == 5;
            const int64_t G = grp ? s[0] : 1, OC = s[grp], IC = s[grp + 1], FH = s[grp + 2], FW = s[grp + 3];
            const int64_t OCp = (OC + 3) / 4 * 4, ICb = (IC + 3) / 4;
            for (int64_t gi = 0; gi < G; ++gi)
                for (int64_t oc = 0; oc < OCp; ++oc)
                    for (int64_t ib = 0; ib < ICb; ++ib)
                        for (int64_t fh = 0; fh < FH; ++fh)
                            for (int64_t fw = 0; fw < FW; ++fw)
                                for (int64_t k = 0; k < 4; ++k) {
                                    int64_t ic = ib * 4 + k;
                                    int64_t di = ((((gi * OCp + oc) * ICb + ib) * FH + fh) * FW + fw) * 4 + k;
                                    int64_t si = (oc < OC && ic < IC)
                                                         ? (((gi * OC + oc) * IC + ic) * FH + fh) * FW + fw
                                                         : -1;
                                    put(d, dst, di, src, si);
                                }
            return MI355_OK;
        }
        case MI355_RL_NCHW4_NCHW32:
        case MI355_RL_NCHW32_NCHW4: {
            /* channel c keeps its position: (c/ps, h, w, c%ps) -> (c/pd, h, w, c%pd) */
            const int64_t ps = s[4], pd = os[4], N = s[0], H = s[2], W = s[3], C = (int64_t)s[1] * ps;
            for (int64_t n = 0; n < N; ++n)
                for (int64_t c = 0; c < C; ++c)
                    for (int64_t h = 0; h < H; ++h)
                        for (int64_t w = 0; w < W; ++w) {
                            int64_t si = (((n * (C / ps) + c / ps) * H + h) * W + w) * ps + c % ps;
                            int64_t di = (((n * (C / pd) + c / pd) * H + h) * W + w) * pd + c % pd;
                            put(d, dst, di, src, si);
                        }
            return MI355_OK;
        }
        default:
            return MI355_ERR_UNSUPPORTED;
    }
}

/* ------------------------------------------------------------------------------------ */
/* helpers for tests of the device epilogue's division scheme                            */
/* ------------------------------------------------------------------------------------ */

/* Division by a constant without a hardware divide, in its correctly rounded form: with y_hi = RN(1/b),
 * y_lo = RN(1/b - y_hi),
 *   q0 = fma(a, y_hi, a * y_lo)   (faithful quotient)
 *   r  = fma(-q0, b, a)           (exact residual)
 *   q  = fma(r, y_hi, q0)         (correctly rounded a / b)
 * This host copy lets a CPU test sweep it against the C '/' operator.  The device epilogue runs the cheaper variant
 * q0 = a * y_hi (a faithful quotient, not always the correctly rounded one), which is checked differently: at every
 * rounding boundary of the final roundf, per dst scale (tests/test_epilogue_quotient.py and the library's own proof). */
float oracle_fastdiv(float a, float b, float y_hi, float y_lo) {
    float t = a * y_lo;
    float q0 = fmaf(a, y_hi, t);
    float r = fmaf(-q0, b, a);
    return fmaf(r, y_hi, q0);
}

/* returns the number of mismatches of the fast division against a / b over `count`
 * numerators starting at bit pattern `start_bits` with stride `step` (numerators whose true
 * quotient is outside [-lim, lim] only need to agree after clamping to [-129, 129]). */
uint64_t oracle_fastdiv_sweep(float b, uint32_t start_bits, uint32_t step, uint64_t count, float* first_bad) {
    double inv = 1.0 / (double)b;
    float y_hi = (float)inv;
    float y_lo = (float)(inv - (double)y_hi);
    uint64_t bad = 0;
    uint32_t bits = start_bits;
    for (uint64_t i = 0; i < count; ++i, bits += step) {
        float a;
        memcpy(&a, &bits, 4);
        if (!(fabsf(a) < 3.0e38f)) continue;
        float want = a / b;
        float got = oracle_fastdiv(a, b, y_hi, y_lo);
        if (fabsf(want) > 129.f) {
            float cw = fminf(fmaxf(want, -129.f), 129.f), cg = fminf(fmaxf(got, -129.f), 129.f);
            if (cw != cg) {
                if (!bad && first_bad) *first_bad = a;
                ++bad;
            }
        } else if (want != got && !(fabsf(want) < 1e-30f && fabsf(got) < 1e-30f)) {
            if (!bad && first_bad) *first_bad = a;
            ++bad;
        }
    }
    return bad;
}

/* device rounding scheme: clamp, then truncate(q + copysign(pred(0.5), q)); must equal
 * roundf + clamp for every float.  Sweeps all bit patterns in [lo_bits, hi_bits]. */
uint64_t oracle_round_sweep(uint32_t lo_bits, uint32_t hi_bits, float* first_bad) {
    uint64_t bad = 0;
    const float half_pred = 0.49999997f;
    for (uint64_t b = lo_bits; b <= hi_bits; ++b) {
        uint32_t bits = (uint32_t)b;
        float q;
        memcpy(&q, &bits, 4);
        float want = fminf(fmaxf(-128.f, roundf(q)), 127.f);
        float c = fminf(fmaxf(-128.f, q), 127.f);
        float t = c + copysignf(half_pred, c);
        int got = (int)t; /* truncation toward zero */
        if (q != q) continue;
        if ((int)want != got) {
            if (!bad && first_bad) *first_bad = q;
            ++bad;
        }
    }
    return bad;
}
