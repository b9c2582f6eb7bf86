// f32 reduction over one axis of a contiguous tensor viewed as [A,B,C]
// (BareMetal/Reduce.cpp:98-131). Used by the softmax tail (MAX and SUM over the class axis).
// C == 1 : one 256-thread workgroup per output, wavefront shuffles + one LDS exchange.
// C  > 1 : one thread per output, lanes walk C (coalesced), serial over B.
// The summation order differs from the reference's ascending loop; f32 results are held to the
// 1e-4 tolerance, not bit-exactness.
#include <float.h>

#include "common.h"

namespace mg {

template <int MODE>
__device__ __forceinline__ float red_init() {
    return MODE == MEGCC_REDUCE_MAX       ? -FLT_MAX
           : MODE == MEGCC_REDUCE_MIN     ? FLT_MAX
           : MODE == MEGCC_REDUCE_PRODUCT ? 1.f
                                          : 0.f;
}
// an element on its way into the reduction (SUM_SQR squares it once; partial sums then add)
template <int MODE>
__device__ __forceinline__ float red_in(float v) {
    return MODE == MEGCC_REDUCE_SUM_SQR ? v * v : v;
}
template <int MODE>
__device__ __forceinline__ float red_op(float a, float b) {
    return MODE == MEGCC_REDUCE_MAX       ? (a > b ? a : b)
           : MODE == MEGCC_REDUCE_MIN     ? (a < b ? a : b)
           : MODE == MEGCC_REDUCE_PRODUCT ? a * b
                                          : a + b;
}

template <int MODE>
__global__ void __launch_bounds__(256) reduce_rows_kernel(
        const float* __restrict__ src, float* __restrict__ dst, int B) {
    __shared__ float part[4];
    const float* row = src + (size_t)blockIdx.x * B;
    float acc = red_init<MODE>();
    for (int j = threadIdx.x; j < B; j += 256)
        acc = red_op<MODE>(acc, red_in<MODE>(row[j]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        acc = red_op<MODE>(acc, __shfl_down(acc, off, 64));
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = red_op<MODE>(red_op<MODE>(part[0], part[1]), red_op<MODE>(part[2], part[3]));
        dst[blockIdx.x] = MODE == MEGCC_REDUCE_MEAN ? r / (float)B : r;
    }
}

template <int MODE>
__global__ void __launch_bounds__(256) reduce_strided_kernel(
        const float* __restrict__ src, float* __restrict__ dst, size_t total, int B, int C) {
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    if (i >= total)
        return;
    size_t a = i / C, k = i - a * C;
    const float* p = src + a * B * C + k;
    float acc = red_init<MODE>();
    for (int j = 0; j < B; ++j)
        acc = red_op<MODE>(acc, red_in<MODE>(p[(size_t)j * C]));
    dst[i] = MODE == MEGCC_REDUCE_MEAN ? acc / (float)B : acc;
}

template <int MODE>
static void launch_reduce(const float* s, float* d, int A, int B, int C) {
    if (C == 1) {
        hipLaunchKernelGGL(reduce_rows_kernel<MODE>, dim3(A), dim3(256), 0, stream(), s, d, B);
    } else {
        size_t total = (size_t)A * C;
        hipLaunchKernelGGL(reduce_strided_kernel<MODE>, dim3(ceil_div(total, 256)), dim3(256), 0,
                           stream(), s, d, total, B, C);
    }
}

}  // namespace mg

using namespace mg;

extern "C" TinyNNStatus megcc_gfx950_reduce(
        const MegccReduceAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace*, const RuntimeOpt*) {
    MG_REQUIRE(attr, TinyNN_ERROR_NULL_PTR, "reduce: NULL attr");
    TinyNNStatus st = check_io(inputs, nr_input, 1, 1, outputs, nr_output, "reduce");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor* s = inputs[0];
    const Tensor* d = outputs[0];
    MG_REQUIRE(is_f32(s) && is_f32(d), TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "reduce: only f32 is implemented");
    MG_REQUIRE(is_contiguous(s->layout) && is_contiguous(d->layout), TinyNN_ERROR_INVALID_LAYOUT,
               "reduce: expects contiguous tensors");
    MG_REQUIRE(attr->axis >= 0 && attr->axis < s->layout.nr_dim, TinyNN_ERROR_OUT_OF_RANGE,
               "reduce: axis %d of a %d-d tensor", attr->axis, s->layout.nr_dim);
    size_t A = 1, C = 1;
    for (int i = 0; i < attr->axis; ++i)
        A *= s->layout.dims[i];
    int B = s->layout.dims[attr->axis];
    for (int i = attr->axis + 1; i < s->layout.nr_dim; ++i)
        C *= s->layout.dims[i];
    MG_REQUIRE(nr_elem(d->layout) == A * C, TinyNN_ERROR_INVALID_LAYOUT,
               "reduce: destination has %zu elements, expected %zu", nr_elem(d->layout), A * C);
    MG_REQUIRE(A < (1u << 31) && C < (1u << 31), TinyNN_ERROR_OUT_OF_RANGE, "reduce: too large");
    if (A * C == 0)
        return TinyNN_SUCCESS;
    MG_REQUIRE(B > 0, TinyNN_ERROR_OUT_OF_RANGE, "reduce: empty axis");
    const float* sp = (const float*)s->ptr;
    float* dp = (float*)d->ptr;
    switch (attr->mode) {
        case MEGCC_REDUCE_SUM: launch_reduce<MEGCC_REDUCE_SUM>(sp, dp, (int)A, B, (int)C); break;
        case MEGCC_REDUCE_MEAN: launch_reduce<MEGCC_REDUCE_MEAN>(sp, dp, (int)A, B, (int)C); break;
        case MEGCC_REDUCE_MAX: launch_reduce<MEGCC_REDUCE_MAX>(sp, dp, (int)A, B, (int)C); break;
        case MEGCC_REDUCE_MIN: launch_reduce<MEGCC_REDUCE_MIN>(sp, dp, (int)A, B, (int)C); break;
        case MEGCC_REDUCE_PRODUCT: launch_reduce<MEGCC_REDUCE_PRODUCT>(sp, dp, (int)A, B, (int)C); break;
        case MEGCC_REDUCE_SUM_SQR: launch_reduce<MEGCC_REDUCE_SUM_SQR>(sp, dp, (int)A, B, (int)C); break;
        default: return fail(TinyNN_ERROR_NO_IMPLEMENT, "reduce: mode %d", (int)attr->mode);
    }
    note_kernel(C == 1 ? "reduce_rows" : "reduce_strided", attr->mode);
    return check_launch("reduce");
}
