// Bandwidth-bound elementwise kernels: quantized ElemwiseMultiType, TypeCvt and f32 Elemwise.
// One thread moves 16 bytes of the narrowest operand per iteration (uint4 / float4 vectors) when
// the pointers are 16-byte aligned and no per-channel broadcast is involved; a scalar variant of
// the same code covers the ragged tail, unaligned tensors and the [1,C,1,1] broadcast.
//
// Float expressions are those of the reference, operand for operand:
//   QADD            fp32_to_int8((s0*a + s1*b) * (1.f/sd))          BareMetal/ElemwiseMultiType.cpp:39-41
//   QFUSE_ADD_RELU  v0=s0*a; v1=s1*b; fp32_to_int8(max(v0+v1,0) * (1.f/sd))              :42-46
//   QMUL            fp32_to_int8((a*b) * (s0*s1*(1.f/sd)))   (a*b is an int product)     :47-50,159
//   QRELU           fp32_to_int8(max(s0*a,0) * (1.f/sd))                                 :28-31
//   typecvt (GI)    x * (src_scale/dst_scale), roundf, clamp    GeneralIntrinsic/Typecvt.cpp:173-190,262-281
//   typecvt q32->q8 x * src_scale / dst_scale, roundf, clamp    BareMetal/Typecvt.cpp:43-105
#include "common.h"
#include "epilogue.h"
#include "fastdiv.h"

namespace mg {

enum { BC_NONE = 0, BC_SCALAR = 1, BC_CHANNEL = 2 };

struct EwArgs {
    const void* a;
    const void* b;
    void* d;
    size_t n;
    int bcast;
    int C;
    size_t inner;
    float s0, s1, sdiv, smul;
};

template <int MODE>
__device__ __forceinline__ int multitype_one(int a, int b, const EwArgs& p) {
    if (MODE == MEGCC_Q_ADD) {
        return fp32_to_int8((p.s0 * (float)a + p.s1 * (float)b) * p.sdiv);
    } else if (MODE == MEGCC_Q_FUSE_ADD_RELU) {
        float v0 = p.s0 * (float)a;
        float v1 = p.s1 * (float)b;
        return fp32_to_int8(((v0 + v1) > 0 ? (v0 + v1) : 0) * p.sdiv);
    } else if (MODE == MEGCC_Q_MUL) {
        return fp32_to_int8((float)(a * b) * p.smul);
    } else {
        return fp32_to_int8(((p.s0 * (float)a) > 0 ? (p.s0 * (float)a) : 0) * p.sdiv);
    }
}

template <int MODE, bool VEC>
__global__ void __launch_bounds__(256) multitype_kernel(EwArgs p) {
    const int8_t* a = (const int8_t*)p.a;
    const int8_t* b = (const int8_t*)p.b;
    int8_t* d = (int8_t*)p.d;
    const size_t tid = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * blockDim.x;
    size_t done = 0;
    if (VEC) {
        const size_t nvec = p.n / 16;
        const int bs = (MODE != MEGCC_Q_RELU && p.bcast == BC_SCALAR) ? b[0] : 0;
        for (size_t i = tid; i < nvec; i += nthreads) {
            uint4 va = ((const uint4*)a)[i];
            uint4 vb = make_uint4(0, 0, 0, 0);
            if (MODE != MEGCC_Q_RELU && p.bcast == BC_NONE)
                vb = ((const uint4*)b)[i];
            uint32_t wa[4] = {va.x, va.y, va.z, va.w};
            uint32_t wb[4] = {vb.x, vb.y, vb.z, vb.w};
            uint32_t wo[4];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                int o[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    int y = p.bcast == BC_SCALAR ? bs : sbyte(wb[w], c);
                    o[c] = multitype_one<MODE>(sbyte(wa[w], c), y, p);
                }
                wo[w] = pack4(o[0], o[1], o[2], o[3]);
            }
            ((uint4*)d)[i] = make_uint4(wo[0], wo[1], wo[2], wo[3]);
        }
        done = nvec * 16;
    }
    for (size_t i = done + tid; i < p.n; i += nthreads) {
        int y = 0;
        if (MODE != MEGCC_Q_RELU)
            y = p.bcast == BC_NONE ? b[i] : p.bcast == BC_SCALAR ? b[0] : b[(i / p.inner) % p.C];
        d[i] = (int8_t)multitype_one<MODE>(a[i], y, p);
    }
}

template <int MODE>
__device__ __forceinline__ float ew_one(float x, float y) {
    switch (MODE) {
        case MEGCC_EW_RELU: return x > 0 ? x : 0;
        case MEGCC_EW_EXP: return expf(x);
        case MEGCC_EW_SIGMOID: return 1.f / (1.f + expf(-x));
        case MEGCC_EW_H_SWISH: {
            float t = x + 3.f;
            t = t < 0.f ? 0.f : t;
            t = t > 6.f ? 6.f : t;
            return x * t / 6.f;
        }
        case MEGCC_EW_NEGATE: return -x;
        case MEGCC_EW_ADD: return x + y;
        case MEGCC_EW_SUB: return x - y;
        case MEGCC_EW_MUL: return x * y;
        case MEGCC_EW_TRUE_DIV: return x / y;
        case MEGCC_EW_MAX: return x > y ? x : y;
        case MEGCC_EW_MIN: return x < y ? x : y;
        default: return (x + y) > 0 ? (x + y) : 0;  // FUSE_ADD_RELU
    }
}

// f32 elementwise over the broadcast of two dense operands (GetBinaryBcastType of the reference,
// Common/ElemwiseCommon.cpp:47-127: VEC_VEC, VEC_SCALAR, VEC_BCAST101, VEC_BCAST101xX,
// VEC_BCAST111C, VEC_BV, VEC_BCAST110, their mirrored forms and NAIVE are all one index rule
// here). The host right-aligns the operand shapes against the output's, gives broadcast dims the
// stride 0 and merges neighbouring dims that both operands walk densely (or both broadcast), so
// the common cases arrive with 1-3 dims: [n], [rows, N] + [N], [outer, C, inner] * [C].
// A work item is one output element, or 4 neighbours of the innermost dim (one 16-byte access per
// dense operand, one scalar load per broadcast one).
constexpr int EW_MAX_DIM = MAX_DIM;
struct EwBcastArgs {
    const float* a;
    const float* b;
    float* d;
    size_t items;            // work items
    int nd;                  // merged dims, dims[nd - 1] innermost
    FastDiv div[EW_MAX_DIM]; // extents (innermost: in work items)
    int sa[EW_MAX_DIM], sb[EW_MAX_DIM];  // element strides; innermost 0 or 1
};

template <int MODE, int ND, bool VEC>
__global__ void __launch_bounds__(256) elemwise_f32_bcast_kernel(EwBcastArgs p) {
    constexpr bool binary = MODE >= MEGCC_EW_ADD;
    constexpr int W = VEC ? 4 : 1;
    const size_t tid = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * blockDim.x;
    for (size_t item = tid; item < p.items; item += nthreads) {
        size_t oa, ob;
        if (ND == 1) {
            oa = item * W * p.sa[0];
            ob = item * W * p.sb[0];
        } else {
            // (more than one dim: the host keeps the element count below 2^31)
            uint32_t k = (uint32_t)item;
            uint32_t q = fdiv(k, p.div[p.nd - 1]);
            const uint32_t in = (k - q * p.div[p.nd - 1].d) * W;
            oa = (size_t)in * p.sa[p.nd - 1];
            ob = (size_t)in * p.sb[p.nd - 1];
            k = q;
#pragma unroll
            for (int i = (ND < EW_MAX_DIM ? ND : EW_MAX_DIM) - 2; i >= 1; --i) {
                if (ND < EW_MAX_DIM || i < p.nd - 1) {
                    q = fdiv(k, p.div[i]);
                    const uint32_t r = k - q * p.div[i].d;
                    oa += (size_t)r * p.sa[i];
                    ob += (size_t)r * p.sb[i];
                    k = q;
                }
            }
            oa += (size_t)k * p.sa[0];
            ob += (size_t)k * p.sb[0];
        }
        const int li = ND == 1 ? 0 : p.nd - 1;
        if (VEC) {
            float4 x, y = make_float4(0.f, 0.f, 0.f, 0.f);
            if (p.sa[li]) {
                x = *(const float4*)(p.a + oa);
            } else {
                const float v = p.a[oa];
                x = make_float4(v, v, v, v);
            }
            if (binary) {
                if (p.sb[li]) {
                    y = *(const float4*)(p.b + ob);
                } else {
                    const float v = p.b[ob];
                    y = make_float4(v, v, v, v);
                }
            }
            float4 r;
            r.x = ew_one<MODE>(x.x, y.x);
            r.y = ew_one<MODE>(x.y, y.y);
            r.z = ew_one<MODE>(x.z, y.z);
            r.w = ew_one<MODE>(x.w, y.w);
            ((float4*)p.d)[item] = r;
        } else {
            p.d[item] = ew_one<MODE>(p.a[oa], binary ? p.b[ob] : 0.f);
        }
    }
}

enum { CVT_F32_Q8 = 0, CVT_Q8_F32 = 1, CVT_Q8_Q8 = 2, CVT_Q32_Q8 = 3 };

template <int KIND, bool VEC>
__global__ void __launch_bounds__(256) typecvt_kernel(
        const void* __restrict__ src, void* __restrict__ dst, size_t n, float scale,
        float src_scale, float dst_scale) {
    const size_t tid = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * blockDim.x;
    size_t done = 0;
    if (VEC) {
        const size_t nvec = n / 16;
        for (size_t i = tid; i < nvec; i += nthreads) {
            if (KIND == CVT_F32_Q8) {
                uint32_t wo[4];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    float4 x = ((const float4*)src)[i * 4 + w];
                    wo[w] = pack4(fp32_to_int8(x.x * scale), fp32_to_int8(x.y * scale),
                                  fp32_to_int8(x.z * scale), fp32_to_int8(x.w * scale));
                }
                ((uint4*)dst)[i] = make_uint4(wo[0], wo[1], wo[2], wo[3]);
            } else if (KIND == CVT_Q32_Q8) {
                uint32_t wo[4];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    int4 x = ((const int4*)src)[i * 4 + w];
                    wo[w] = pack4(fp32_to_int8((float)x.x * src_scale / dst_scale),
                                  fp32_to_int8((float)x.y * src_scale / dst_scale),
                                  fp32_to_int8((float)x.z * src_scale / dst_scale),
                                  fp32_to_int8((float)x.w * src_scale / dst_scale));
                }
                ((uint4*)dst)[i] = make_uint4(wo[0], wo[1], wo[2], wo[3]);
            } else {
                uint4 v = ((const uint4*)src)[i];
                uint32_t wi[4] = {v.x, v.y, v.z, v.w};
                if (KIND == CVT_Q8_F32) {
#pragma unroll
                    for (int w = 0; w < 4; ++w)
                        ((float4*)dst)[i * 4 + w] = make_float4(
                                (float)sbyte(wi[w], 0) * scale, (float)sbyte(wi[w], 1) * scale,
                                (float)sbyte(wi[w], 2) * scale, (float)sbyte(wi[w], 3) * scale);
                } else {
                    uint32_t wo[4];
#pragma unroll
                    for (int w = 0; w < 4; ++w)
                        wo[w] = pack4(fp32_to_int8((float)sbyte(wi[w], 0) * scale),
                                      fp32_to_int8((float)sbyte(wi[w], 1) * scale),
                                      fp32_to_int8((float)sbyte(wi[w], 2) * scale),
                                      fp32_to_int8((float)sbyte(wi[w], 3) * scale));
                    ((uint4*)dst)[i] = make_uint4(wo[0], wo[1], wo[2], wo[3]);
                }
            }
        }
        done = nvec * 16;
    }
    for (size_t i = done + tid; i < n; i += nthreads) {
        if (KIND == CVT_F32_Q8)
            ((int8_t*)dst)[i] = (int8_t)fp32_to_int8(((const float*)src)[i] * scale);
        else if (KIND == CVT_Q8_F32)
            ((float*)dst)[i] = (float)((const int8_t*)src)[i] * scale;
        else if (KIND == CVT_Q8_Q8)
            ((int8_t*)dst)[i] = (int8_t)fp32_to_int8((float)((const int8_t*)src)[i] * scale);
        else
            ((int8_t*)dst)[i] =
                    (int8_t)fp32_to_int8((float)((const int32_t*)src)[i] * src_scale / dst_scale);
    }
}

static unsigned grid_for(size_t work_items) {
    size_t b = (work_items + 255) / 256;
    if (b < 1)
        b = 1;
    if (b > (1u << 16) * 16)
        b = (1u << 16) * 16;
    return (unsigned)b;
}

static bool aligned16(const void* p) {
    return ((uintptr_t)p & 15) == 0;
}

// Classifies operand b against a: same shape, one element, or per-channel [1,C,1,1..]
// (BareMetal/ElemwiseMultiType.cpp:76-92); for f32 also a trailing vector [N] against [..,N].
static TinyNNStatus classify_bcast(const Tensor* a, const Tensor* b, EwArgs* p, const char* who) {
    size_t na = nr_elem(a->layout), nb = nr_elem(b->layout);
    p->C = 1;
    p->inner = 1;
    if (na == nb) {
        p->bcast = BC_NONE;
    } else if (nb == 1) {
        p->bcast = BC_SCALAR;
    } else if (
            a->layout.nr_dim == b->layout.nr_dim && a->layout.nr_dim > 2 &&
            a->layout.dims[1] == b->layout.dims[1] && nb == b->layout.dims[1]) {
        p->bcast = BC_CHANNEL;
        p->C = a->layout.dims[1];
        for (int i = 2; i < a->layout.nr_dim; ++i)
            p->inner *= a->layout.dims[i];
    } else if (nb == a->layout.dims[a->layout.nr_dim - 1] &&
               b->layout.dims[b->layout.nr_dim - 1] == nb) {
        p->bcast = BC_CHANNEL;
        p->C = (int)nb;
        p->inner = 1;
    } else if (a->layout.nr_dim == 2 && b->layout.nr_dim == 2 &&
               b->layout.dims[0] == a->layout.dims[0] && b->layout.dims[1] == 1) {
        // [A,N] op [A,1]: one value per row (softmax: x - max, e / sum)
        p->bcast = BC_CHANNEL;
        p->C = a->layout.dims[0];
        p->inner = a->layout.dims[1];
    } else {
        return fail(TinyNN_ERROR_INVALID_LAYOUT, "%s: unsupported broadcast", who);
    }
    return TinyNN_SUCCESS;
}

}  // namespace mg

using namespace mg;

#define MG_LAUNCH_EW(KERNEL, MODE, vec, work, args)                                        \
    do {                                                                                   \
        if (vec)                                                                           \
            hipLaunchKernelGGL((KERNEL<MODE, true>), dim3(grid_for(work)), dim3(256), 0,   \
                               stream(), args);                                            \
        else                                                                               \
            hipLaunchKernelGGL((KERNEL<MODE, false>), dim3(grid_for(work)), dim3(256), 0,  \
                               stream(), args);                                            \
    } while (0)

extern "C" TinyNNStatus megcc_gfx950_elemwise_multitype(
        const MegccMultiTypeMode* mode, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace*, const RuntimeOpt*) {
    MG_REQUIRE(mode, TinyNN_ERROR_NULL_PTR, "elemwise_multitype: NULL mode");
    const bool unary = *mode == MEGCC_Q_RELU;
    TinyNNStatus st = check_io(inputs, nr_input, unary ? 1 : 2, unary ? 1 : 2, outputs, nr_output,
                               "elemwise_multitype");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor* a = inputs[0];
    const Tensor* b = unary ? nullptr : inputs[1];
    const Tensor* d = outputs[0];
    MG_REQUIRE(is_q8(a) && (!b || is_q8(b)) && is_q8(d), TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "elemwise_multitype: only qsi8 operands are implemented");
    MG_REQUIRE(is_contiguous(a->layout) && (!b || is_contiguous(b->layout)) &&
                       is_contiguous(d->layout) && nr_elem(d->layout) == nr_elem(a->layout),
               TinyNN_ERROR_INVALID_LAYOUT, "elemwise_multitype: expects contiguous tensors");
    EwArgs p;
    p.a = a->ptr;
    p.b = b ? b->ptr : nullptr;
    p.d = d->ptr;
    p.n = nr_elem(a->layout);
    p.bcast = BC_NONE;
    p.C = 1;
    p.inner = 1;
    if (b) {
        st = classify_bcast(a, b, &p, "elemwise_multitype");
        if (st != TinyNN_SUCCESS)
            return st;
    }
    p.s0 = a->dtype.param.scale;
    p.s1 = b ? b->dtype.param.scale : 0.f;
    p.sdiv = 1.f / d->dtype.param.scale;
    p.smul = p.s0 * p.s1 * p.sdiv;
    if (p.n == 0)
        return TinyNN_SUCCESS;
    const bool vec = p.bcast != BC_CHANNEL && aligned16(p.a) && aligned16(p.d) &&
                     (p.bcast != BC_NONE || !b || aligned16(p.b));
    const size_t work = vec ? p.n / 16 + 16 : p.n;
    switch (*mode) {
        case MEGCC_Q_ADD: MG_LAUNCH_EW(multitype_kernel, MEGCC_Q_ADD, vec, work, p); break;
        case MEGCC_Q_FUSE_ADD_RELU: MG_LAUNCH_EW(multitype_kernel, MEGCC_Q_FUSE_ADD_RELU, vec, work, p); break;
        case MEGCC_Q_MUL: MG_LAUNCH_EW(multitype_kernel, MEGCC_Q_MUL, vec, work, p); break;
        case MEGCC_Q_RELU: MG_LAUNCH_EW(multitype_kernel, MEGCC_Q_RELU, vec, work, p); break;
        default: return fail(TinyNN_ERROR_NO_IMPLEMENT, "elemwise_multitype: mode %d", (int)*mode);
    }
    return check_launch("elemwise_multitype");
}

namespace {

// Right-aligns `t` against the output dims `od[0..nd)`; fills element strides (0 where the operand
// has extent 1 and the output more). False when the shapes do not broadcast.
bool bcast_strides(const Tensor* t, const uint32_t* od, int nd, long* stride) {
    const Layout& l = t->layout;
    if (l.nr_dim > nd)
        return false;
    long dense = 1;
    for (int i = nd - 1; i >= 0; --i) {
        const int j = i - (nd - l.nr_dim);
        const uint32_t ext = j >= 0 ? l.dims[j] : 1;
        if (ext == od[i]) {
            stride[i] = ext == 1 ? 0 : dense;
        } else if (ext == 1) {
            stride[i] = 0;
        } else {
            return false;
        }
        dense *= ext;
    }
    return true;
}

template <int MODE>
void launch_elemwise_bcast(const EwBcastArgs& p, bool vec) {
    const dim3 grid(grid_for(p.items)), block(256);
#define MG_EW_ND(ND)                                                                              \
    do {                                                                                          \
        if (vec)                                                                                  \
            hipLaunchKernelGGL((elemwise_f32_bcast_kernel<MODE, ND, true>), grid, block, 0,       \
                               stream(), p);                                                      \
        else                                                                                      \
            hipLaunchKernelGGL((elemwise_f32_bcast_kernel<MODE, ND, false>), grid, block, 0,      \
                               stream(), p);                                                      \
    } while (0)
    if (p.nd == 1)
        MG_EW_ND(1);
    else if (MODE < MEGCC_EW_ADD)
        return;  // (a unary operator has one dense operand: always one dim)
    else if (p.nd == 2)
        MG_EW_ND(2);
    else if (p.nd == 3)
        MG_EW_ND(3);
    else
        MG_EW_ND(EW_MAX_DIM);
#undef MG_EW_ND
}

}  // namespace

extern "C" TinyNNStatus megcc_gfx950_elemwise(
        const MegccElemwiseMode* mode, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace*, const RuntimeOpt*) {
    MG_REQUIRE(mode, TinyNN_ERROR_NULL_PTR, "elemwise: NULL mode");
    const bool binary = *mode >= MEGCC_EW_ADD;
    TinyNNStatus st = check_io(inputs, nr_input, binary ? 2 : 1, binary ? 2 : 1, outputs,
                               nr_output, "elemwise");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor* a = inputs[0];
    const Tensor* b = binary ? inputs[1] : nullptr;
    const Tensor* d = outputs[0];
    MG_REQUIRE(is_f32(a) && (!b || is_f32(b)) && is_f32(d), TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "elemwise: only f32 is implemented");
    MG_REQUIRE(is_contiguous(a->layout) && (!b || is_contiguous(b->layout)) &&
                       is_contiguous(d->layout),
               TinyNN_ERROR_INVALID_LAYOUT, "elemwise: expects contiguous tensors");
    const int nd0 = d->layout.nr_dim;
    MG_REQUIRE(nd0 >= 1 && nd0 <= MAX_DIM, TinyNN_ERROR_INVALID_LAYOUT, "elemwise: %d dims", nd0);
    uint32_t od[MAX_DIM];
    long sa[MAX_DIM], sb[MAX_DIM];
    for (int i = 0; i < nd0; ++i)
        od[i] = d->layout.dims[i];
    const size_t n = nr_elem(d->layout);
    MG_REQUIRE(bcast_strides(a, od, nd0, sa) && (!b || bcast_strides(b, od, nd0, sb)),
               TinyNN_ERROR_INVALID_LAYOUT,
               "elemwise: operand shapes do not broadcast to the output's");
    // the output is the broadcast of the operands, not more
    for (int i = 0; i < nd0; ++i)
        MG_REQUIRE(od[i] == 1 || sa[i] != 0 || (b && sb[i] != 0), TinyNN_ERROR_INVALID_LAYOUT,
                   "elemwise: output dim %d (%u) is larger than both operands'", i, od[i]);
    if (n == 0)
        return TinyNN_SUCCESS;
    if (!b)
        for (int i = 0; i < nd0; ++i)
            sb[i] = sa[i];
    // drop dims of extent 1, merge neighbours that both operands walk as one dense (or one
    // broadcast) run
    uint32_t md[MAX_DIM];
    long ma[MAX_DIM], mb[MAX_DIM];
    int nd = 0;
    for (int i = 0; i < nd0; ++i) {
        if (od[i] == 1)
            continue;
        if (nd > 0 && ma[nd - 1] == sa[i] * (long)od[i] && mb[nd - 1] == sb[i] * (long)od[i]) {
            md[nd - 1] *= od[i];
            ma[nd - 1] = sa[i];
            mb[nd - 1] = sb[i];
        } else {
            md[nd] = od[i];
            ma[nd] = sa[i];
            mb[nd] = sb[i];
            ++nd;
        }
    }
    if (nd == 0) {
        md[0] = 1;
        ma[0] = mb[0] = 1;
        nd = 1;
    }
    MG_REQUIRE(nd == 1 || n < (1u << 31), TinyNN_ERROR_OUT_OF_RANGE,
               "elemwise: a broadcast over %zu elements is beyond the 32-bit index range", n);
    EwBcastArgs p = {};
    p.a = (const float*)a->ptr;
    p.b = b ? (const float*)b->ptr : nullptr;
    p.d = (float*)d->ptr;
    p.nd = nd;
    // 16-byte accesses: whole groups of 4 along the innermost dim, aligned bases; the outer
    // strides of an operand that is dense along it are multiples of its extent
    const bool vec = (md[nd - 1] & 3) == 0 && aligned16(p.d) && (ma[nd - 1] == 0 || aligned16(p.a)) &&
                     (!b || mb[nd - 1] == 0 || aligned16(p.b));
    bool outer_ok = true;
    for (int i = 0; i < nd - 1; ++i)
        outer_ok = outer_ok && (ma[nd - 1] == 0 || (ma[i] & 3) == 0) && (mb[nd - 1] == 0 || (mb[i] & 3) == 0);
    const bool v4 = vec && outer_ok;
    for (int i = 0; i < nd; ++i) {
        p.div[i] = make_fastdiv(i == nd - 1 && v4 ? md[i] / 4 : md[i]);
        p.sa[i] = (int)ma[i];
        p.sb[i] = (int)mb[i];
    }
    p.items = v4 ? n / 4 : n;
    switch (*mode) {
#define MG_CASE(M) case M: launch_elemwise_bcast<M>(p, v4); break;
        MG_CASE(MEGCC_EW_RELU)
        MG_CASE(MEGCC_EW_EXP)
        MG_CASE(MEGCC_EW_SIGMOID)
        MG_CASE(MEGCC_EW_H_SWISH)
        MG_CASE(MEGCC_EW_NEGATE)
        MG_CASE(MEGCC_EW_ADD)
        MG_CASE(MEGCC_EW_SUB)
        MG_CASE(MEGCC_EW_MUL)
        MG_CASE(MEGCC_EW_TRUE_DIV)
        MG_CASE(MEGCC_EW_MAX)
        MG_CASE(MEGCC_EW_MIN)
        MG_CASE(MEGCC_EW_FUSE_ADD_RELU)
#undef MG_CASE
        default: return fail(TinyNN_ERROR_NO_IMPLEMENT, "elemwise: mode %d", (int)*mode);
    }
    note_kernel("elemwise_f32_bcast", nd, v4 ? 4 : 1);
    return check_launch("elemwise");
}

extern "C" TinyNNStatus megcc_gfx950_typecvt(
        Tensor** inputs, int nr_input, Tensor** outputs, int nr_output, const Workspace*,
        const RuntimeOpt*) {
    TinyNNStatus st = check_io(inputs, nr_input, 1, 1, outputs, nr_output, "typecvt");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor* s = inputs[0];
    const Tensor* d = outputs[0];
    MG_REQUIRE(is_contiguous(s->layout) && is_contiguous(d->layout) &&
                       nr_elem(s->layout) == nr_elem(d->layout),
               TinyNN_ERROR_INVALID_LAYOUT, "typecvt: expects contiguous tensors of equal size");
    const size_t n = nr_elem(s->layout);
    float src_scale = s->dtype.param.scale, dst_scale = d->dtype.param.scale;
    int kind;
    if (is_f32(s) && d->dtype.type_enum == TinyNN_QINT8) {
        kind = CVT_F32_Q8;
        src_scale = 1.f;
    } else if (s->dtype.type_enum == TinyNN_QINT8 && is_f32(d)) {
        kind = CVT_Q8_F32;
        dst_scale = 1.f;
    } else if (s->dtype.type_enum == TinyNN_QINT8 && d->dtype.type_enum == TinyNN_QINT8) {
        kind = CVT_Q8_Q8;
    } else if (s->dtype.type_enum == TinyNN_QINT32 && d->dtype.type_enum == TinyNN_QINT8) {
        kind = CVT_Q32_Q8;
    } else {
        return fail(TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE, "typecvt: %d -> %d is not implemented",
                    (int)s->dtype.type_enum, (int)d->dtype.type_enum);
    }
    MG_REQUIRE(src_scale > 0 && dst_scale > 0, TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "typecvt: scales must be positive");
    if (n == 0)
        return TinyNN_SUCCESS;
    const float scale = src_scale / dst_scale;  // host IEEE division, as the generated C does once
    const bool vec = aligned16(s->ptr) && aligned16(d->ptr);
    const size_t work = vec ? n / 16 + 16 : n;
#define MG_CVT(K)                                                                              \
    case K:                                                                                    \
        if (vec)                                                                               \
            hipLaunchKernelGGL((typecvt_kernel<K, true>), dim3(grid_for(work)), dim3(256), 0,  \
                               stream(), s->ptr, d->ptr, n, scale, src_scale, dst_scale);      \
        else                                                                                   \
            hipLaunchKernelGGL((typecvt_kernel<K, false>), dim3(grid_for(work)), dim3(256), 0, \
                               stream(), s->ptr, d->ptr, n, scale, src_scale, dst_scale);      \
        break;
    switch (kind) {
        MG_CVT(CVT_F32_Q8)
        MG_CVT(CVT_Q8_F32)
        MG_CVT(CVT_Q8_Q8)
        default:
        MG_CVT(CVT_Q32_Q8)
    }
#undef MG_CVT
    return check_launch("typecvt");
}
