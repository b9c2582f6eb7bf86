/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement ("port") of the arithmetic of MegCC's generated
 * x86/BAREMETAL kernels for the conv / matmul / pooling / elemwise / typecvt / relayout / concat
 * path. It exists to check the gfx950 kernels and to serve as bench.py's cpu_baseline leg; nothing
 * in the product library includes, links or calls it.
 *
 * Every function cites the generator it restates (paths relative to the MegCC tree,
 * compiler/lib/KernelGen/...). Integer accumulation is exact, so loop order is free there; every
 * *float* expression keeps the reference's operand order and is compiled with
 * -ffp-contract=off -fno-fast-math (see oracle/Makefile) so that no FMA or re-association can
 * change a result.
 *
 * Pinning: tests/test_oracle.py runs each function against the reference's own generated C
 * (oracle/_ref/libmegcc_ref.so, built by `make ref` where the reference tree exists) and against
 * the fixtures under tests/golden/ that were produced from it. Functions without such a check:
 * none.  Known limit: `int r = roundf(x)` for |x| >= 2^31 is undefined behaviour in the
 * reference (BareMetal/Activation.cpp:50); it is unreachable with int8 data and sane scales and is
 * not restated.
 *
 * Threads: orc_set_threads(n) lets the *tests* spread the outer loop over n cores; the default
 * and the cpu_baseline use 1 (the reference runtime is single-threaded).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

static int g_threads = 1;
void orc_set_threads(int n) {
    g_threads = n < 1 ? 1 : n;
}

enum { FMT_NCHW = 0, FMT_NCHW44 = 1, FMT_NCHW_NCHW44 = 2 };
enum { ACT_IDENTITY = 0, ACT_RELU = 1, ACT_H_SWISH = 2, ACT_SIGMOID = 3 };

/* BareMetal/Activation.cpp:9-42 -- the helper functions the generator pastes in front of a
 * kernel; `min`/`max` there are `a > b ? b : a` and `a > b ? a : b`. */
static inline float act_apply(int act, float x) {
    switch (act) {
        case ACT_RELU:
            return x > 0 ? x : 0;
        case ACT_H_SWISH: {
            float t = x + 3;
            float mx = t > 0.f ? t : 0.f;
            float mn = mx > 6.f ? 6.f : mx;
            return x * mn * (1.f / 6.f);
        }
        case ACT_SIGMOID:
            return 1.f / (expf(-x) + 1.f);
        default:
            return x;
    }
}

/* BareMetal/Activation.cpp:47-56 fp32_to_int8 */
static inline int8_t fp32_to_int8(float src) {
    int res = roundf(src);
    res = res > 127 ? 127 : res;
    res = res < -128 ? -128 : res;
    return (int8_t)res;
}

/* element offset of (n, c, h, w): BareMetal/FormatHelper.cpp:12-36 on a contiguous tensor */
static inline size_t off_nchw(int C, int H, int W, int n, int c, int h, int w) {
    return (((size_t)n * C + c) * H + h) * W + w;
}
static inline size_t off_nchw44(int C, int H, int W, int n, int c, int h, int w) {
    return ((((size_t)n * (C / 4) + c / 4) * H + h) * W + w) * 4 + (c % 4);
}

/* filter offset: BareMetal/ConvKernel.cpp:48-76 (strides) and :78-113 (address) */
static inline size_t flt_off(
        int fmt, int group_conv, int g, int oc, int ic, int fh, int fw, int ocpg, int icpg,
        int FH, int FW) {
    if (fmt == FMT_NCHW) {
        /* [G,] OCpg, ICpg, FH, FW */
        return ((((size_t)g * ocpg + oc) * icpg + ic) * FH + fh) * FW + fw;
    } else if (fmt == FMT_NCHW_NCHW44) {
        /* OC/4, FH, FW, IC, 4oc */
        return ((((size_t)(oc / 4) * FH + fh) * FW + fw) * icpg + ic) * 4 + (oc % 4);
    } else if (!group_conv) {
        /* OC/4, IC/4, FH, FW, 4ic, 4oc */
        return (((((size_t)(oc / 4) * (icpg / 4) + ic / 4) * FH + fh) * FW + fw) * 4 + (ic % 4)) *
                       4 +
               (oc % 4);
    } else {
        /* channel-wise: G/4, 1, 1, FH, FW, 4 */
        return (((size_t)(g / 4) * FH + fh) * FW + fw) * 4 + (g % 4);
    }
}

/* BareMetal::ConvGeneral, qsi8 x qsi8 (+qsi32 bias) -> qsi8:
 * BareMetal/ConvKernel.cpp:305-344 (loops, `uint32 idx < ih` zero padding), :374-380 (bias added
 * to the int accumulator), BareMetal/Activation.cpp:105-114 (dval*scale*flt_scale/dst_scale,
 * activation applied to the fully scaled value, then fp32_to_int8).
 * groups == 1: DENSE; groups > 1: GROUP with ocpg = OC/groups, icpg = IC/groups. */
void orc_conv_q8(
        const int8_t* src, const int8_t* flt, const int32_t* bias, int8_t* dst, int fmt,
        int groups, int N, int IC, int IH, int IW, int OC, int OH, int OW, int FH, int FW, int SH,
        int SW, int PH, int PW, int DH, int DW, int act, float scale, float flt_scale,
        float dst_scale) {
    const int ocpg = OC / groups, icpg = IC / groups;
    const int src44 = (fmt == FMT_NCHW44);
    const int dst44 = (fmt != FMT_NCHW);
    const int is_group = groups > 1;
    const long total = (long)N * OC;
#pragma omp parallel for schedule(dynamic) num_threads(g_threads) if (g_threads > 1)
    for (long job = 0; job < total; ++job) {
        const int n = (int)(job / OC), oc = (int)(job % OC);
        const int g = oc / ocpg, ocl = oc % ocpg;
        for (int oh = 0; oh < OH; ++oh)
            for (int ow = 0; ow < OW; ++ow) {
                int dval = 0;
                for (int fh = 0; fh < FH; ++fh)
                    for (int fw = 0; fw < FW; ++fw) {
                        uint32_t ih = (uint32_t)(oh * SH + fh * DH - PH);
                        uint32_t iw = (uint32_t)(ow * SW + fw * DW - PW);
                        if (ih < (uint32_t)IH && iw < (uint32_t)IW) {
                            for (int icl = 0; icl < icpg; ++icl) {
                                int ic = g * icpg + icl;
                                int sval = src44 ? src[off_nchw44(IC, IH, IW, n, ic, ih, iw)]
                                                 : src[off_nchw(IC, IH, IW, n, ic, ih, iw)];
                                int fval = flt[flt_off(
                                        fmt, is_group, g, ocl, icl, fh, fw, ocpg, icpg, FH, FW)];
                                dval += sval * fval;
                            }
                        }
                    }
                if (bias)
                    dval += bias[oc];
                size_t o = dst44 ? off_nchw44(OC, OH, OW, n, oc, oh, ow)
                                 : off_nchw(OC, OH, OW, n, oc, oh, ow);
                dst[o] = fp32_to_int8(act_apply(act, dval * scale * flt_scale / dst_scale));
            }
    }
}

/* Same template with acc_specifier = "float" (BareMetal/ConvKernel.cpp:199-207): accumulation
 * order fh -> fw -> ic, bias added last, activation on the sum. The kernel MegCC actually selects
 * for f32 NCHW DENSE on x86 is GI im2col + 4x12 GEMM (GeneralIntrinsic/ConvKernel/Fp32Im2col.cpp:
 * 88-218), which sums in a different order; the two agree to ~1e-6 relative and the product is
 * held to 1e-4 against either. */
void orc_conv_f32(
        const float* src, const float* flt, const float* bias, float* dst, int fmt, int groups,
        int N, int IC, int IH, int IW, int OC, int OH, int OW, int FH, int FW, int SH, int SW,
        int PH, int PW, int DH, int DW, int act) {
    const int ocpg = OC / groups, icpg = IC / groups;
    const int src44 = (fmt == FMT_NCHW44);
    const int dst44 = (fmt != FMT_NCHW);
    const int is_group = groups > 1;
    const long total = (long)N * OC;
#pragma omp parallel for schedule(dynamic) num_threads(g_threads) if (g_threads > 1)
    for (long job = 0; job < total; ++job) {
        const int n = (int)(job / OC), oc = (int)(job % OC);
        const int g = oc / ocpg, ocl = oc % ocpg;
        for (int oh = 0; oh < OH; ++oh)
            for (int ow = 0; ow < OW; ++ow) {
                float dval = 0;
                for (int fh = 0; fh < FH; ++fh)
                    for (int fw = 0; fw < FW; ++fw) {
                        uint32_t ih = (uint32_t)(oh * SH + fh * DH - PH);
                        uint32_t iw = (uint32_t)(ow * SW + fw * DW - PW);
                        if (ih < (uint32_t)IH && iw < (uint32_t)IW) {
                            for (int icl = 0; icl < icpg; ++icl) {
                                int ic = g * icpg + icl;
                                float sval = src44 ? src[off_nchw44(IC, IH, IW, n, ic, ih, iw)]
                                                   : src[off_nchw(IC, IH, IW, n, ic, ih, iw)];
                                float fval = flt[flt_off(
                                        fmt, is_group, g, ocl, icl, fh, fw, ocpg, icpg, FH, FW)];
                                dval += sval * fval;
                            }
                        }
                    }
                if (bias)
                    dval += bias[oc];
                size_t o = dst44 ? off_nchw44(OC, OH, OW, n, oc, oh, ow)
                                 : off_nchw(OC, OH, OW, n, oc, oh, ow);
                dst[o] = act_apply(act, dval);
            }
    }
}

/* f32 MatrixMul, row-major, no bias. BareMetal/MatrixMul.cpp:25-120 (naive m,n,k loops) --
 * GI 4x12 (GeneralIntrinsic/MatMulKernel/Fp32MatMulM4N12.cpp) and gevm
 * (GeneralIntrinsic/MatMulKernel/Fp32Gevm.cpp:50-91) differ only in summation order. */
void orc_matmul_f32(
        const float* A, const float* B, float* C, int M, int N, int K, int lda, int ldb, int ldc,
        int trans_a, int trans_b) {
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float acc = 0.f;
            for (int k = 0; k < K; ++k) {
                float a = trans_a ? A[(size_t)k * lda + m] : A[(size_t)m * lda + k];
                float b = trans_b ? B[(size_t)n * ldb + k] : B[(size_t)k * ldb + n];
                acc += a * b;
            }
            C[(size_t)m * ldc + n] = acc;
        }
}

enum { POOL_MAX = 0, POOL_AVG = 1, POOL_AVG_EXCL = 2 };

/* qsi8 pooling.
 * NCHW  : BareMetal/Pooling.cpp:84-148,219-245 -- MAX over in-bounds taps starting from -128;
 *         AVERAGE `sum = roundf((float)sum / (wh*ww))`, COUNT_EXCLUDE_PADDING `/ count`; the int
 *         is stored to int8 without a clamp.
 * NCHW44: GeneralIntrinsic/PoolingKernel/QInt8PoolingNCHW44.cpp:34-113 -- AVERAGE is
 *         `float count_div = 1.0 / window_count;` then saturate(round((float)sum * count_div))
 *         (the non-SSE4.2 branch of GiCvtFromFloat32ToInt8, immigration/include/gi_int.h:
 *         1145-1160: round(), clamp to [-128,127]). */
void orc_pool_q8(
        const int8_t* src, int8_t* dst, int fmt, int mode, int N, int C, int IH, int IW, int OH,
        int OW, int WH, int WW, int SH, int SW, int PH, int PW) {
    const long total = (long)N * C;
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1)
    for (long job = 0; job < total; ++job) {
        const int n = (int)(job / C), c = (int)(job % C);
        for (int oh = 0; oh < OH; ++oh)
            for (int ow = 0; ow < OW; ++ow) {
                int8_t res = -128;
                int sum = 0, count = 0;
                for (int fh = 0; fh < WH; ++fh)
                    for (int fw = 0; fw < WW; ++fw) {
                        uint32_t ih = (uint32_t)(-PH + oh * SH + fh);
                        uint32_t iw = (uint32_t)(-PW + ow * SW + fw);
                        if (ih < (uint32_t)IH && iw < (uint32_t)IW) {
                            int8_t v = fmt == FMT_NCHW44
                                             ? src[off_nchw44(C, IH, IW, n, c, ih, iw)]
                                             : src[off_nchw(C, IH, IW, n, c, ih, iw)];
                            res = res > v ? res : v;
                            sum += v;
                            ++count;
                        }
                    }
                int8_t out;
                if (mode == POOL_MAX) {
                    out = res;
                } else if (fmt == FMT_NCHW44) {
                    uint32_t window_count = mode == POOL_AVG ? (uint32_t)(WH * WW) : (uint32_t)count;
                    float count_div = 1.0 / window_count;
                    double r = round((float)sum * count_div);
                    r = r > 127 ? 127 : r;
                    r = r < -128 ? -128 : r;
                    out = (int8_t)r;
                } else {
                    int s = mode == POOL_AVG ? (int)roundf((float)sum / (WH * WW))
                                             : (int)roundf((float)sum / count);
                    out = (int8_t)s;
                }
                size_t o = fmt == FMT_NCHW44 ? off_nchw44(C, OH, OW, n, c, oh, ow)
                                             : off_nchw(C, OH, OW, n, c, oh, ow);
                dst[o] = out;
            }
    }
}

enum { Q_ADD = 0, Q_FUSE_ADD_RELU = 1, Q_MUL = 2, Q_RELU = 3 };

/* BareMetal/ElemwiseMultiType.cpp:16-55 (expressions) and :102-213 (three broadcast cases).
 * bcast: 0 same shape, 1 b is one element, 2 b is [1,C,1,1..] against a = [outer,C,inner]. */
void orc_multitype_q8(
        const int8_t* a, const int8_t* b, int8_t* dst, int mode, size_t n, int bcast, int C,
        size_t inner, float scale_0, float scale_1, float scale_dst) {
    float scale_div = 1.f / scale_dst;
    float scale_mul = scale_0 * scale_1 * scale_div;
    for (size_t i = 0; i < n; ++i) {
        int8_t val_0 = a[i];
        int8_t val_1 = 0;
        if (mode != Q_RELU)
            val_1 = bcast == 0 ? b[i] : bcast == 1 ? b[0] : b[(i / inner) % C];
        int8_t out;
        if (mode == Q_ADD) {
            out = fp32_to_int8((scale_0 * val_0 + scale_1 * val_1) * scale_div);
        } else if (mode == Q_FUSE_ADD_RELU) {
            float val0 = scale_0 * val_0;
            float val1 = scale_1 * val_1;
            out = fp32_to_int8(((val0 + val1) > 0 ? (val0 + val1) : 0) * scale_div);
        } else if (mode == Q_MUL) {
            out = fp32_to_int8(val_0 * val_1 * scale_mul);
        } else {
            out = fp32_to_int8(((scale_0 * val_0) > 0 ? (scale_0 * val_0) : 0) * scale_div);
        }
        dst[i] = out;
    }
}

/* GeneralIntrinsic/Typecvt.cpp:227-295: `scale = src_scale/dst_scale` with 1 substituted on a float
 * side, then x*scale; the 16-wide body and the scalar tail round identically on a host without
 * SSE4.2 (gi_int.h:1145-1160 round() vs roundf(), both half away from zero; both clamp). */
static inline int8_t sat_q8(float v) {
    int d = roundf(v);
    d = d >= 127 ? 127 : d;
    d = d <= -128 ? -128 : d;
    return (int8_t)d;
}
void orc_typecvt_f32_q8(const float* src, int8_t* dst, size_t n, float dst_scale) {
    float scale = 1.f / dst_scale;
    for (size_t i = 0; i < n; ++i)
        dst[i] = sat_q8(src[i] * scale);
}
void orc_typecvt_q8_f32(const int8_t* src, float* dst, size_t n, float src_scale) {
    float scale = src_scale / 1.f;
    for (size_t i = 0; i < n; ++i)
        dst[i] = src[i] * scale;
}
void orc_typecvt_q8_q8(const int8_t* src, int8_t* dst, size_t n, float src_scale, float dst_scale) {
    float scale = src_scale / dst_scale;
    for (size_t i = 0; i < n; ++i)
        dst[i] = sat_q8(src[i] * scale);
}
/* BareMetal/Typecvt.cpp:43-105: qsi32 -> qsi8 is `staturate(val * src_scale / dst_scale)` */
void orc_typecvt_q32_q8(
        const int32_t* src, int8_t* dst, size_t n, float src_scale, float dst_scale) {
    for (size_t i = 0; i < n; ++i)
        dst[i] = sat_q8(src[i] * src_scale / dst_scale);
}

enum {
    EW_RELU = 0,
    EW_EXP = 1,
    EW_SIGMOID = 2,
    EW_H_SWISH = 3,
    EW_NEGATE = 4,
    EW_ADD = 16,
    EW_SUB = 17,
    EW_MUL = 18,
    EW_TRUE_DIV = 19,
    EW_MAX = 20,
    EW_MIN = 21,
    EW_FUSE_ADD_RELU = 22
};

/* f32 elementwise, BareMetal/ElemwiseKernel.cpp:35-110 expressions.
 * bcast: 0 same shape, 1 scalar b, 2 b indexed by (i / inner) % C, i.e. [1,C,1,1] or a trailing
 * vector when inner == 1. */
void orc_elemwise_f32(
        const float* a, const float* b, float* dst, int mode, size_t n, int bcast, int C,
        size_t inner) {
    for (size_t i = 0; i < n; ++i) {
        float x = a[i], y = 0.f, r;
        if (mode >= EW_ADD)
            y = bcast == 0 ? b[i] : bcast == 1 ? b[0] : b[(i / inner) % C];
        switch (mode) {
            case EW_RELU:
                r = x > 0 ? x : 0;
                break;
            case EW_EXP:
                r = expf(x);
                break;
            case EW_SIGMOID:
                r = 1.f / (1.f + expf(-x));
                break;
            case EW_H_SWISH: {
                float t = x + 3.f;
                t = t > 6.f ? 6.f : t;
                t = t < 0.f ? 0.f : t;
                r = x * t / 6.f;
                break;
            }
            case EW_NEGATE:
                r = -x;
                break;
            case EW_ADD:
                r = x + y;
                break;
            case EW_SUB:
                r = x - y;
                break;
            case EW_MUL:
                r = x * y;
                break;
            case EW_TRUE_DIV:
                r = x / y;
                break;
            case EW_MAX:
                r = x > y ? x : y;
                break;
            case EW_MIN:
                r = x < y ? x : y;
                break;
            default: /* FUSE_ADD_RELU */
                r = (x + y) > 0 ? (x + y) : 0;
                break;
        }
        dst[i] = r;
    }
}

enum { RED_SUM = 0, RED_MEAN = 1, RED_MAX = 2, RED_MIN = 3, RED_PRODUCT = 4, RED_SUM_SQR = 5 };

/* BareMetal/Reduce.cpp:11-72,98-131: view as [A,B,C], reduce over B in ascending j; start value
 * lowest / highest float for MAX / MIN, 1 for PRODUCT, else 0; MEAN divides the sum by B. */
void orc_reduce_f32(const float* src, float* dst, int mode, int A, int B, int C) {
    for (int i = 0; i < A; ++i)
        for (int k = 0; k < C; ++k) {
            float acc = mode == RED_MAX       ? -__FLT_MAX__
                        : mode == RED_MIN     ? __FLT_MAX__
                        : mode == RED_PRODUCT ? 1.f
                                              : 0.f;
            for (int j = 0; j < B; ++j) {
                float v = src[((size_t)i * B + j) * C + k];
                if (mode == RED_MAX)
                    acc = acc > v ? acc : v;
                else if (mode == RED_MIN)
                    acc = acc < v ? acc : v;
                else if (mode == RED_PRODUCT)
                    acc = acc * v;
                else if (mode == RED_SUM_SQR)
                    acc = acc + (v * v);
                else
                    acc = acc + v;
            }
            dst[(size_t)i * C + k] = mode == RED_MEAN ? acc / B : acc;
        }
}

/* Relayout: BareMetal/Relayout.cpp:83-91 (the "fallback to naive" loop, which every faster
 * branch of that kernel must agree with) over the odometers of Common/Relayout.h:18-40:
 * element k, counted in the row-major order of each side's own dims, goes from
 * src[sum idx_s * sstride] to dst[sum idx_d * dstride]. Offsets are in elements of `es` bytes and
 * relative to the first element of each view. */
void orc_relayout(
        const void* src, int snd, const int64_t* sdims, const int64_t* sstr, void* dst, int dnd,
        const int64_t* ddims, const int64_t* dstr, int es) {
    int64_t sidx[8] = {0}, didx[8] = {0};
    int64_t total = 1;
    for (int i = 0; i < snd; ++i)
        total *= sdims[i];
    int64_t so = 0, doff = 0;
    for (int64_t k = 0; k < total; ++k) {
        memcpy((char*)dst + doff * es, (const char*)src + so * es, (size_t)es);
        for (int i = snd - 1; i >= 0; --i) {
            if (++sidx[i] < sdims[i]) {
                so += sstr[i];
                break;
            }
            sidx[i] = 0;
            so -= (sdims[i] - 1) * sstr[i];
        }
        for (int i = dnd - 1; i >= 0; --i) {
            if (++didx[i] < ddims[i]) {
                doff += dstr[i];
                break;
            }
            didx[i] = 0;
            doff -= (ddims[i] - 1) * dstr[i];
        }
    }
}

/* Concat of dense tensors, BareMetal/Concat.cpp:35-61: input i, viewed as [outer, len_i * inner],
 * lands in the output [outer, sum(len) * inner] at column (len of the inputs before it) * inner. */
void orc_concat(
        const void* const* srcs, const int64_t* lens, int nr, void* dst, int64_t outer,
        int64_t inner, int es) {
    int64_t all = 0;
    for (int i = 0; i < nr; ++i)
        all += lens[i];
    int64_t at = 0;
    for (int i = 0; i < nr; ++i) {
        for (int64_t o = 0; o < outer; ++o)
            for (int64_t j = 0; j < lens[i] * inner; ++j)
                memcpy((char*)dst + ((o * all + at) * inner + j) * es,
                       (const char*)srcs[i] + (o * lens[i] * inner + j) * es, (size_t)es);
        at += lens[i];
    }
}

/* Resize, f32. Common/Resize.h:16-40 (get_coord), :42-101 (LINEAR body, NCHW / NCHW44 through
 * get_offset :209-225), :158-175 (NEAREST, strided NCHW source). scale = (float)O / I. */
static void orc_resize_coord(float scale, int size, int idx, float* a0, int* i0, float* a1, int* i1) {
    if (size == 1) {
        *a0 = 1.f; *i0 = 0; *a1 = 0.f; *i1 = 0;
        return;
    }
    float alpha = (idx + 0.5f) / scale - 0.5f;
    int origin = (int)floorf(alpha);
    alpha -= origin;
    if (origin < 0) {
        origin = 0;
        alpha = 0;
    } else if (origin + 1 >= size) {
        origin = size - 2;
        alpha = 1;
    }
    *a0 = 1 - alpha; *i0 = origin; *a1 = alpha; *i1 = origin + 1;
}

static size_t orc_resize_off(int pack4, size_t h, size_t w, size_t c, size_t H, size_t W) {
    return pack4 ? ((((c >> 2) * H * W + h * W + w) << 2) + (c & 3)) : c * H * W + h * W + w;
}

/* C counts channels (4 * dims[1] for NCHW44) */
void orc_resize_linear_f32(
        const float* src, float* dst, int N, int C, int IH, int IW, int OH, int OW, int pack4) {
    const float scale_h = (float)OH / IH, scale_w = (float)OW / IW;
    for (int n = 0; n < N; ++n) {
        for (int c = 0; c < C; ++c)
            for (int oh = 0; oh < OH; ++oh) {
                int ih0, ih1;
                float ah0, ah1;
                orc_resize_coord(scale_h, IH, oh, &ah0, &ih0, &ah1, &ih1);
                for (int ow = 0; ow < OW; ++ow) {
                    int iw0, iw1;
                    float aw0, aw1;
                    orc_resize_coord(scale_w, IW, ow, &aw0, &iw0, &aw1, &iw1);
                    dst[orc_resize_off(pack4, oh, ow, c, OH, OW)] =
                            src[orc_resize_off(pack4, ih0, iw0, c, IH, IW)] * ah0 * aw0 +
                            src[orc_resize_off(pack4, ih0, iw1, c, IH, IW)] * ah0 * aw1 +
                            src[orc_resize_off(pack4, ih1, iw0, c, IH, IW)] * ah1 * aw0 +
                            src[orc_resize_off(pack4, ih1, iw1, c, IH, IW)] * ah1 * aw1;
                }
            }
        src += (size_t)C * IH * IW;
        dst += (size_t)C * OH * OW;
    }
}

/* source strides in elements; dense NCHW destination */
void orc_resize_nearest_f32(
        const float* src, float* dst, int N, int C, int IH, int IW, int OH, int OW, int64_t s_n,
        int64_t s_c, int64_t s_h, int64_t s_w) {
    const float scale_h = (float)OH / IH, scale_w = (float)OW / IW;
    for (int n = 0; n < N; ++n) {
        for (int oh = 0; oh < OH; ++oh)
            for (int ow = 0; ow < OW; ++ow) {
                int ih = (int)(oh / scale_h), iw = (int)(ow / scale_w);
                ih = ih < IH - 1 ? ih : IH - 1;
                iw = iw < IW - 1 ? iw : IW - 1;
                for (int c = 0; c < C; ++c)
                    dst[(size_t)c * OH * OW + (size_t)oh * OW + ow] = src[c * s_c + ih * s_h + iw * s_w];
            }
        src += s_n;
        dst += (size_t)C * OH * OW;
    }
}

/* Fused f32 elementwise chain, BareMetal/FusedElemwiseKernel.cpp:32-113 (expressions), :159-219
 * (operand reads), :390-413 (loop). prog: per step {mode, nr_arg, arg0..arg3}; value k < nr_input
 * is input k, value nr_input + j the result of step j; the last result is stored.
 * types: 0 VECTOR, 1 SCALAR, 2 BCAST101, 3 BCAST101x4 (Common/ElemwiseCommon.h:8-15). */
enum {
    EW_ABS = 5, EW_LOG = 6, EW_SILU = 7, EW_ROUND = 8, EW_LT = 23, EW_LEQ = 24, EW_EQ = 25,
    EW_FLOOR_DIV = 26, EW_FUSE_ADD_SIGMOID = 27, EW_FUSE_ADD_TANH = 28, EW_FUSE_MUL_ADD3 = 32,
    EW_FUSE_MUL_ADD4 = 33
};

static float orc_fused_clip(float val, float min, float max) {
    if (val < min)
        val = min;
    if (val > max)
        val = max;
    return val;
}

void orc_fused_elemwise_f32(
        const int* prog, int nr_input, int nr_step, const float* const* in, const int* types,
        float* dst, size_t n, size_t stride1, size_t dims1) {
    float v[64];
    for (size_t i = 0; i < n; ++i) {
        const size_t ch = (i / stride1) % dims1;
        for (int k = 0; k < nr_input; ++k)
            v[k] = types[k] == 0   ? in[k][i]
                   : types[k] == 1 ? in[k][0]
                   : types[k] == 2 ? in[k][ch]
                                   : in[k][ch * 4 + i % 4];
        float r = 0.f;
        for (int j = 0; j < nr_step; ++j) {
            const int* s = prog + 6 * j;
            const float a = v[s[2]], b = s[1] > 1 ? v[s[3]] : 0.f, c = s[1] > 2 ? v[s[4]] : 0.f,
                        d = s[1] > 3 ? v[s[5]] : 0.f;
            switch (s[0]) {
                case EW_RELU: r = a > 0 ? a : 0; break;
                case EW_EXP: r = expf(a); break;
                case EW_SIGMOID: r = 1 / (1 + expf(-a)); break;
                case EW_NEGATE: r = -a; break;
                case EW_ROUND: r = roundf(a); break;
                case EW_H_SWISH: r = a * orc_fused_clip(a + 3, 0, 6) / 6; break;
                case EW_ABS: r = a > 0 ? a : -a; break;
                case EW_LOG: r = logf(a); break;
                case EW_SILU: r = a / (1 + expf(-a)); break;
                case EW_ADD: r = a + b; break;
                case EW_SUB: r = a - b; break;
                case EW_MUL: r = a * b; break;
                case EW_TRUE_DIV: r = a / b; break;
                case EW_FUSE_ADD_RELU: r = (a + b) > 0 ? (a + b) : 0; break;
                case EW_FUSE_ADD_SIGMOID: r = 1.f / (1.f + expf(-(a + b))); break;
                case EW_FUSE_ADD_TANH: r = (float)tanh(a + b); break;
                case EW_MAX: r = a > b ? a : b; break;
                case EW_MIN: r = a < b ? a : b; break;
                case EW_LT: r = (a < b); break;
                case EW_LEQ: r = (a <= b); break;
                case EW_EQ: r = (a == b); break;
                case EW_FLOOR_DIV: r = floorf(a / b); break;
                case EW_FUSE_MUL_ADD3: r = a * b + c; break;
                default: r = a * b + c * d; break; /* FUSE_MUL_ADD4 */
            }
            v[nr_input + j] = r;
        }
        dst[i] = r;
    }
}
