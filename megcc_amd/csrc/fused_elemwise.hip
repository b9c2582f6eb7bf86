// Fused chain of f32 elementwise steps in one pass over memory: what MegCC's elemwise fusion
// hands to FusedElemwiseKernel (BareMetal/FusedElemwiseKernel.cpp:270-423; expressions :32-113;
// operand kinds Common/ElemwiseCommon.cpp:7-45, reads :159-219). The reference generates C for
// each chain; here the chain travels as a small program in the kernel arguments and every thread
// interprets it - the steps are the same for all lanes, so the interpreter's branches are uniform
// and cost a few scalar instructions per step.
// Bound: HBM, 4 B per VECTOR input + 4 B out per element.
#include "common.h"

namespace mg {
namespace {

enum { FT_VECTOR = 0, FT_SCALAR = 1, FT_BCAST101 = 2, FT_BCAST101x4 = 3 };

struct FusedArgs {
    const float* in[MEGCC_FUSED_MAX_INPUTS];
    int type[MEGCC_FUSED_MAX_INPUTS];
    float* dst;
    unsigned n;
    unsigned stride1, dims1;  // of the output: channel = (i / stride1) % dims1
    MegccFusedElemwiseAttr prog;
};

__device__ __forceinline__ float fused_step(int mode, float a, float b, float c, float d) {
    switch (mode) {
        case MEGCC_EW_RELU: return a > 0 ? a : 0;
        case MEGCC_EW_EXP: return expf(a);
        case MEGCC_EW_SIGMOID: return 1.f / (1.f + expf(-a));
        case MEGCC_EW_NEGATE: return -a;
        case MEGCC_EW_ROUND: return roundf(a);
        case MEGCC_EW_H_SWISH: {
            float t = a + 3.f;
            t = t < 0.f ? 0.f : t;
            t = t > 6.f ? 6.f : t;
            return a * t / 6.f;
        }
        case MEGCC_EW_ABS: return a > 0 ? a : -a;
        case MEGCC_EW_LOG: return logf(a);
        case MEGCC_EW_SILU: return a / (1.f + expf(-a));
        case MEGCC_EW_ADD: return a + b;
        case MEGCC_EW_SUB: return a - b;
        case MEGCC_EW_MUL: return a * b;
        case MEGCC_EW_TRUE_DIV: return a / b;
        case MEGCC_EW_FUSE_ADD_RELU: return (a + b) > 0 ? (a + b) : 0;
        case MEGCC_EW_FUSE_ADD_SIGMOID: return 1.f / (1.f + expf(-(a + b)));
        case MEGCC_EW_FUSE_ADD_TANH: return tanhf(a + b);
        case MEGCC_EW_MAX: return a > b ? a : b;
        case MEGCC_EW_MIN: return a < b ? a : b;
        case MEGCC_EW_LT: return a < b ? 1.f : 0.f;
        case MEGCC_EW_LEQ: return a <= b ? 1.f : 0.f;
        case MEGCC_EW_EQ: return a == b ? 1.f : 0.f;
        case MEGCC_EW_FLOOR_DIV: return floorf(a / b);
        case MEGCC_EW_FUSE_MUL_ADD3: return a * b + c;
        default: return a * b + c * d;  // FUSE_MUL_ADD4
    }
}

__device__ __forceinline__ float4 fused_step4(int mode, float4 a, float4 b, float4 c, float4 d) {
    float4 r;
#define MG_F4(M)                                  \
    case M:                                       \
        r.x = fused_step(M, a.x, b.x, c.x, d.x);  \
        r.y = fused_step(M, a.y, b.y, c.y, d.y);  \
        r.z = fused_step(M, a.z, b.z, c.z, d.z);  \
        r.w = fused_step(M, a.w, b.w, c.w, d.w);  \
        break;
    switch (mode) {  // the same for all lanes: one branch per step, then straight-line code
        MG_F4(MEGCC_EW_RELU) MG_F4(MEGCC_EW_EXP) MG_F4(MEGCC_EW_SIGMOID) MG_F4(MEGCC_EW_NEGATE)
        MG_F4(MEGCC_EW_ROUND) MG_F4(MEGCC_EW_H_SWISH) MG_F4(MEGCC_EW_ABS) MG_F4(MEGCC_EW_LOG)
        MG_F4(MEGCC_EW_SILU) MG_F4(MEGCC_EW_ADD) MG_F4(MEGCC_EW_SUB) MG_F4(MEGCC_EW_MUL)
        MG_F4(MEGCC_EW_TRUE_DIV) MG_F4(MEGCC_EW_FUSE_ADD_RELU) MG_F4(MEGCC_EW_FUSE_ADD_SIGMOID)
        MG_F4(MEGCC_EW_FUSE_ADD_TANH) MG_F4(MEGCC_EW_MAX) MG_F4(MEGCC_EW_MIN) MG_F4(MEGCC_EW_LT)
        MG_F4(MEGCC_EW_LEQ) MG_F4(MEGCC_EW_EQ) MG_F4(MEGCC_EW_FLOOR_DIV) MG_F4(MEGCC_EW_FUSE_MUL_ADD3)
        default:
            r.x = fused_step(MEGCC_EW_FUSE_MUL_ADD4, a.x, b.x, c.x, d.x);
            r.y = fused_step(MEGCC_EW_FUSE_MUL_ADD4, a.y, b.y, c.y, d.y);
            r.z = fused_step(MEGCC_EW_FUSE_MUL_ADD4, a.z, b.z, c.z, d.z);
            r.w = fused_step(MEGCC_EW_FUSE_MUL_ADD4, a.w, b.w, c.w, d.w);
            break;
    }
#undef MG_F4
    return r;
}

// One thread = 4 neighbouring elements (16-byte accesses when `vec`: every same-size operand and
// the output 16-byte aligned, n a multiple of 4). The value table lives in LDS, one float4
// column per thread and only as many rows as the chain has values: a register array indexed by
// run-time value numbers ends up in scratch memory.
template <bool VEC>
__global__ void __launch_bounds__(256) fused_elemwise_kernel(FusedArgs q) {
    extern __shared__ float4 fused_lds[];
    const unsigned g = blockIdx.x * blockDim.x + threadIdx.x;
    const unsigned i0 = g * 4;
    if (i0 >= q.n)
        return;
    float4* const val = fused_lds + threadIdx.x;  // value k at val[k * blockDim.x]
    const unsigned vs = blockDim.x;
    for (int k = 0; k < q.prog.nr_input; ++k) {
        const float* p = q.in[k];
        const int ty = q.type[k];
        float e[4];
        if (ty == FT_SCALAR) {
            e[0] = e[1] = e[2] = e[3] = p[0];
        } else if (ty == FT_VECTOR && VEC) {
            const float4 x = *(const float4*)(p + i0);
            e[0] = x.x; e[1] = x.y; e[2] = x.z; e[3] = x.w;
        } else if (VEC && ty != FT_VECTOR && (q.stride1 & 3) == 0) {
            // the 4 elements lie in one channel
            const unsigned ch = (i0 / q.stride1) % q.dims1;
            if (ty == FT_BCAST101) {
                e[0] = e[1] = e[2] = e[3] = p[ch];
            } else {
                const float4 x = *(const float4*)(p + ch * 4);
                e[0] = x.x; e[1] = x.y; e[2] = x.z; e[3] = x.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const unsigned i = min(i0 + j, q.n - 1);
                const unsigned ch = (i / q.stride1) % q.dims1;
                e[j] = ty == FT_VECTOR ? p[i] : ty == FT_BCAST101 ? p[ch] : p[ch * 4 + (i & 3)];
            }
        }
        val[k * vs] = make_float4(e[0], e[1], e[2], e[3]);
    }
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < q.prog.nr_step; ++j) {
        const MegccFusedStep& s = q.prog.step[j];
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
        const float4 a = val[s.arg[0] * vs];
        const float4 b = s.nr_arg > 1 ? val[s.arg[1] * vs] : zero;
        const float4 c = s.nr_arg > 2 ? val[s.arg[2] * vs] : zero;
        const float4 d = s.nr_arg > 3 ? val[s.arg[3] * vs] : zero;
        r = fused_step4(s.mode, a, b, c, d);
        val[(q.prog.nr_input + j) * vs] = r;
    }
    if (VEC) {
        *(float4*)(q.dst + i0) = r;
    } else {
        const float e[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (i0 + j < q.n)
                q.dst[i0 + j] = e[j];
    }
}

int step_arity(int mode) {
    switch (mode) {
        case MEGCC_EW_RELU: case MEGCC_EW_EXP: case MEGCC_EW_SIGMOID: case MEGCC_EW_NEGATE:
        case MEGCC_EW_ROUND: case MEGCC_EW_H_SWISH: case MEGCC_EW_ABS: case MEGCC_EW_LOG:
        case MEGCC_EW_SILU:
            return 1;
        case MEGCC_EW_ADD: case MEGCC_EW_SUB: case MEGCC_EW_MUL: case MEGCC_EW_TRUE_DIV:
        case MEGCC_EW_FUSE_ADD_RELU: case MEGCC_EW_FUSE_ADD_SIGMOID: case MEGCC_EW_FUSE_ADD_TANH:
        case MEGCC_EW_MAX: case MEGCC_EW_MIN: case MEGCC_EW_LT: case MEGCC_EW_LEQ: case MEGCC_EW_EQ:
        case MEGCC_EW_FLOOR_DIV:
            return 2;
        case MEGCC_EW_FUSE_MUL_ADD3: return 3;
        case MEGCC_EW_FUSE_MUL_ADD4: return 4;
        default: return 0;
    }
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" TinyNNStatus megcc_gfx950_fused_elemwise(
        const MegccFusedElemwiseAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace*, const RuntimeOpt*) {
    MG_REQUIRE(attr, TinyNN_ERROR_NULL_PTR, "fused_elemwise: NULL attr");
    MG_REQUIRE(attr->nr_input >= 1 && attr->nr_input <= MEGCC_FUSED_MAX_INPUTS && attr->nr_step >= 1 &&
                       attr->nr_step <= MEGCC_FUSED_MAX_STEPS,
               TinyNN_ERROR_OUT_OF_RANGE, "fused_elemwise: %d inputs, %d steps", attr->nr_input,
               attr->nr_step);
    TinyNNStatus st = check_io(inputs, nr_input, attr->nr_input, attr->nr_input, outputs, nr_output,
                               "fused_elemwise");
    if (st != TinyNN_SUCCESS)
        return st;
    // every step reads values that exist before it
    for (int j = 0; j < attr->nr_step; ++j) {
        const MegccFusedStep& s = attr->step[j];
        MG_REQUIRE(step_arity(s.mode) != 0 && s.nr_arg == step_arity(s.mode), TinyNN_ERROR_OUT_OF_RANGE,
                   "fused_elemwise: step %d has mode %d with %d operands", j, (int)s.mode, s.nr_arg);
        for (int a = 0; a < s.nr_arg; ++a)
            MG_REQUIRE(s.arg[a] >= 0 && s.arg[a] < attr->nr_input + j, TinyNN_ERROR_OUT_OF_RANGE,
                       "fused_elemwise: step %d reads value %d before it exists", j, s.arg[a]);
    }
    const Tensor* d = outputs[0];
    const Layout& dl = d->layout;
    MG_REQUIRE(is_f32(d) && is_contiguous(dl), TinyNN_ERROR_INVALID_LAYOUT,
               "fused_elemwise: the output must be a dense f32 tensor");
    const size_t n = nr_elem(dl);
    if (n == 0)
        return TinyNN_SUCCESS;
    MG_REQUIRE(n < (1ull << 32), TinyNN_ERROR_OUT_OF_RANGE, "fused_elemwise: tensor too large");
    FusedArgs q = {};
    q.dst = (float*)d->ptr;
    q.n = (unsigned)n;
    q.stride1 = 1;
    q.dims1 = 1;
    if (dl.nr_dim >= 2) {
        q.dims1 = dl.dims[1];
        size_t inner = 1;
        for (int i = 2; i < dl.nr_dim; ++i)
            inner *= dl.dims[i];
        q.stride1 = (unsigned)inner;
    }
    q.prog = *attr;
    for (int k = 0; k < nr_input; ++k) {
        const Tensor* t = inputs[k];
        const Layout& l = t->layout;
        MG_REQUIRE(is_f32(t), TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE, "fused_elemwise: input %d is not f32", k);
        const size_t ne = nr_elem(l);
        int type;
        if (ne == n) {
            type = FT_VECTOR;
            MG_REQUIRE(is_contiguous(l), TinyNN_ERROR_INVALID_LAYOUT, "fused_elemwise: input %d is strided", k);
        } else if (ne == 1) {
            type = FT_SCALAR;
        } else if (dl.nr_dim >= 4 && l.nr_dim == 4 && l.dims[0] == 1 && l.dims[2] == 1 && l.dims[3] == 1 &&
                   l.dims[1] == dl.dims[1] && l.nr_dim == dl.nr_dim) {
            type = FT_BCAST101;
        } else if (dl.nr_dim == 5 && l.nr_dim == 5 && l.dims[0] == 1 && l.dims[2] == 1 && l.dims[3] == 1 &&
                   l.dims[4] == 4 && dl.dims[4] == 4 && l.dims[1] == dl.dims[1]) {
            type = FT_BCAST101x4;
        } else {
            return fail(TinyNN_ERROR_INVALID_LAYOUT,
                        "fused_elemwise: input %d is neither of the output's size, a scalar, "
                        "[1,C,1,1] nor [1,C,1,1,4]", k);
        }
        q.in[k] = (const float*)t->ptr;
        q.type[k] = type;
    }
    bool vec = (n & 3) == 0 && ((uintptr_t)q.dst & 15) == 0;
    for (int k = 0; k < nr_input; ++k)
        vec = vec && (q.type[k] == FT_SCALAR || q.type[k] == FT_BCAST101 || ((uintptr_t)q.in[k] & 15) == 0);
    // LDS: 16 B per value and thread; long chains run with smaller workgroups (at most 48 KB)
    const int values = attr->nr_input + attr->nr_step;
    const unsigned threads = values <= 12 ? 256 : 128;
    const size_t lds = (size_t)values * threads * sizeof(float4);
    const dim3 grid((unsigned)((n + threads * 4 - 1) / (threads * 4)));
    if (vec)
        hipLaunchKernelGGL(fused_elemwise_kernel<true>, grid, dim3(threads), lds, stream(), q);
    else
        hipLaunchKernelGGL(fused_elemwise_kernel<false>, grid, dim3(threads), lds, stream(), q);
    return check_launch("fused_elemwise");
}
