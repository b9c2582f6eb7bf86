// Soft-max over the last axis of a [rows, n] tensor in one kernel.
//
// MegCC has no soft-max kernel: its importer decomposes opr::Softmax into five operators - Reduce
// MAX over the axis, SUB, EXP, Reduce SUM, TRUE_DIV (compiler/lib/Target/MGB/importer.cpp:987-1016)
// - and a classifier usually dequantises its logits first (typecvt qsi8 -> f32). On this chip a
// kernel boundary costs 3-5 us whatever the kernel does (each of the 8 XCDs has its own L2, so
// every kernel ends with a write-back and starts cold), i.e. ~25 us for 0.5 MB of data. This kernel
// computes the same expressions in the same order per element - x = (float)q * scale for a qsi8
// source (GeneralIntrinsic/Typecvt.cpp:262-281), m = max x, e = expf(x - m), s = sum e, e / s - with
// one workgroup per row and the row in registers; only the order of the additions in s differs
// from the reference's ascending loop (BareMetal/Reduce.cpp:98-131), as it does in reduce.hip.
// The model runtime substitutes it for that operator chain (model.cpp); the five kernels stay
// available under their own symbols.
#include <float.h>

#include "common.h"

namespace mg {

static constexpr int SM_MAX_PER_THREAD = 16;  // rows of up to 4096 elements

template <typename T>
__global__ void __launch_bounds__(256) softmax_rows_kernel(
        const T* __restrict__ src, float* __restrict__ dst, int n, float scale) {
    __shared__ float part[4];
    const T* row = src + (size_t)blockIdx.x * n;
    float* out = dst + (size_t)blockIdx.x * n;
    const int tid = threadIdx.x;
    float x[SM_MAX_PER_THREAD];
    float mx = -FLT_MAX;
#pragma unroll
    for (int k = 0; k < SM_MAX_PER_THREAD; ++k) {
        const int j = tid + k * 256;
        if (j < n) {
            x[k] = sizeof(T) == 1 ? (float)row[j] * scale : (float)row[j];
            mx = x[k] > mx ? x[k] : mx;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(mx, off, 64);
        mx = o > mx ? o : mx;
    }
    if ((tid & 63) == 0)
        part[tid >> 6] = mx;
    __syncthreads();
    {
        const float a = part[0] > part[1] ? part[0] : part[1], b = part[2] > part[3] ? part[2] : part[3];
        mx = a > b ? a : b;
    }
    __syncthreads();
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < SM_MAX_PER_THREAD; ++k) {
        const int j = tid + k * 256;
        if (j < n) {
            x[k] = expf(x[k] - mx);
            sum += x[k];
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        sum += __shfl_xor(sum, off, 64);
    if ((tid & 63) == 0)
        part[tid >> 6] = sum;
    __syncthreads();
    sum = (part[0] + part[1]) + (part[2] + part[3]);
#pragma unroll
    for (int k = 0; k < SM_MAX_PER_THREAD; ++k) {
        const int j = tid + k * 256;
        if (j < n)
            out[j] = x[k] / sum;
    }
}

}  // namespace mg

using namespace mg;

extern "C" int megcc_gfx950_softmax_max_columns(void) {
    return 256 * SM_MAX_PER_THREAD;
}

extern "C" TinyNNStatus megcc_gfx950_softmax(
        Tensor** inputs, int nr_input, Tensor** outputs, int nr_output, const Workspace*,
        const RuntimeOpt*) {
    TinyNNStatus st = check_io(inputs, nr_input, 1, 1, outputs, nr_output, "softmax");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor* s = inputs[0];
    const Tensor* d = outputs[0];
    MG_REQUIRE((is_f32(s) || is_q8(s)) && is_f32(d), TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "softmax: f32 or qsi8 in, f32 out");
    MG_REQUIRE(is_contiguous(s->layout) && is_contiguous(d->layout) &&
                       nr_elem(s->layout) == nr_elem(d->layout),
               TinyNN_ERROR_INVALID_LAYOUT, "softmax: expects contiguous tensors of one size");
    // the rows are those of the destination (a dequantised source may still carry the [N,C,1,1]
    // shape of the layer that produced it)
    MG_REQUIRE(d->layout.nr_dim >= 1, TinyNN_ERROR_INVALID_LAYOUT, "softmax: destination without dims");
    const int n = (int)d->layout.dims[d->layout.nr_dim - 1];
    MG_REQUIRE(n >= 1 && n <= 256 * SM_MAX_PER_THREAD, TinyNN_ERROR_OUT_OF_RANGE,
               "softmax: rows of %d elements (at most %d)", n, 256 * SM_MAX_PER_THREAD);
    const size_t rows = nr_elem(s->layout) / (size_t)n;
    MG_REQUIRE(rows < (1u << 31), TinyNN_ERROR_OUT_OF_RANGE, "softmax: too many rows");
    if (rows == 0)
        return TinyNN_SUCCESS;
    if (is_q8(s))
        hipLaunchKernelGGL(softmax_rows_kernel<int8_t>, dim3((unsigned)rows), dim3(256), 0, stream(),
                           (const int8_t*)s->ptr, (float*)d->ptr, n, s->dtype.param.scale);
    else
        hipLaunchKernelGGL(softmax_rows_kernel<float>, dim3((unsigned)rows), dim3(256), 0, stream(),
                           (const float*)s->ptr, (float*)d->ptr, n, 1.f);
    note_kernel("softmax_rows", is_q8(s) ? 1 : 4);
    return check_launch("softmax");
}
