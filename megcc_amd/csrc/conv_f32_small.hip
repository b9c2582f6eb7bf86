// f32 NCHW dense convolution for SMALL layers (a few tens of MFLOP: the batch-1 first layers of a
// float model, e.g. 32 -> 32 channels on 56 x 56): one launch, no matrix cores, no split-K. A wave
// owns 64 output pixels and 2 output channels; the filter rows of its 2 channels are read through
// wave-uniform addresses (one cache line per load), the input pixels coalesced along the row;
// about a wave per SIMD for such a layer, so the whole thing is launch + a few microseconds. The
// tiled implicit GEMM needs a split over K and a second (reduce) launch to fill the chip here.
// Summation order: input channel, filter row, filter column ascending, then the bias
// (GeneralIntrinsic/ConvKernel/Fp32Im2col.cpp:88-218 accumulates in GEMM order; f32 results are
// held to the 1e-4 tolerance, not to bit equality).
#include "common.h"
#include "conv_geom.h"
#include "epilogue.h"

namespace mg {

static constexpr int CS_OCW = 2;  // output channels per wave

__device__ __forceinline__ float cs_act(int act, float x) {
    switch (act) {
        case MEGCC_NONLINE_RELU: return act_apply<MEGCC_NONLINE_RELU>(x);
        case MEGCC_NONLINE_H_SWISH: return act_apply<MEGCC_NONLINE_H_SWISH>(x);
        case MEGCC_NONLINE_SIGMOID: return act_apply<MEGCC_NONLINE_SIGMOID>(x);
        default: return x;
    }
}

template <int FH, int FW>
__global__ void __launch_bounds__(256) conv_f32_small_kernel(
        ConvGeom g, const float* __restrict__ src, const float* __restrict__ flt,
        const float* __restrict__ bias, float* __restrict__ dst) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ohw = g.oh * g.ow;
    const int P = g.n * ohw;
    const int p = blockIdx.x * 64 + lane;
    // wave-uniform, and told so: the filter rows are then read through the scalar cache
    const int oc0 = __builtin_amdgcn_readfirstlane((blockIdx.y * 4 + wave) * CS_OCW);
    if (oc0 >= g.oc)
        return;
    const int pp = p < P ? p : P - 1;  // lanes beyond the end repeat the last pixel, store nothing
    const int n = pp / ohw, r = pp - n * ohw;
    const int oh = r / g.ow, ow = r - oh * g.ow;
    const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
    const float* img = src + (size_t)n * g.ic * g.ih * g.iw;
    const int K = g.ic * FH * FW;
    const float* w0 = flt + (size_t)oc0 * K;
    const bool two = oc0 + 1 < g.oc;
    const float* w1 = two ? w0 + K : w0;
    // taps inside the image, one bit per (fh, fw)
    unsigned valid = 0;
#pragma unroll
    for (int fh = 0; fh < FH; ++fh)
#pragma unroll
        for (int fw = 0; fw < FW; ++fw) {
            const unsigned ih = (unsigned)(ih0 + fh * g.dh), iw = (unsigned)(iw0 + fw * g.dw);
            if (ih < (unsigned)g.ih && iw < (unsigned)g.iw)
                valid |= 1u << (fh * FW + fw);
        }
    float a0 = 0.f, a1 = 0.f;
#pragma unroll 4
    for (int ic = 0; ic < g.ic; ++ic) {
        const float* plane = img + (size_t)ic * g.ih * g.iw;
        float x[FH * FW];
#pragma unroll
        for (int fh = 0; fh < FH; ++fh)
#pragma unroll
            for (int fw = 0; fw < FW; ++fw) {
                const int t = fh * FW + fw;
                x[t] = (valid >> t) & 1 ? plane[(ih0 + fh * g.dh) * g.iw + iw0 + fw * g.dw] : 0.f;
            }
#pragma unroll
        for (int t = 0; t < FH * FW; ++t) {
            a0 += x[t] * w0[ic * FH * FW + t];
            a1 += x[t] * w1[ic * FH * FW + t];
        }
    }
    if (p < P) {
        float* o = dst + ((size_t)n * g.oc + oc0) * ohw + r;
        o[0] = cs_act(g.act, a0 + (bias ? bias[oc0] : 0.f));
        if (two)
            o[ohw] = cs_act(g.act, a1 + (bias ? bias[oc0 + 1] : 0.f));
    }
}

// 3x3 and 1x1 f32 NCHW dense layers of at most 2^27 multiply-adds
bool conv_f32_small_supported(const ConvGeom& g) {
    const long P = (long)g.n * g.oh * g.ow;
    const long macs = P * g.oc * g.ic * g.fh * g.fw;
    return g.fmt == MEGCC_FMT_NCHW && g.groups == 1 && ((g.fh == 3 && g.fw == 3) || (g.fh == 1 && g.fw == 1)) &&
           P >= 1 && P < (1L << 30) && macs <= (1L << 27) && g.oc >= 1 &&
           (long)g.n * g.ic * g.ih * g.iw < (1L << 31) && P * g.oc < (1L << 31);
}

TinyNNStatus conv_f32_small_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    const long P = (long)g.n * g.oh * g.ow;
    const dim3 grid((unsigned)((P + 63) / 64), (unsigned)((g.oc + 4 * CS_OCW - 1) / (4 * CS_OCW)));
    if (g.fh == 3)
        hipLaunchKernelGGL((conv_f32_small_kernel<3, 3>), grid, dim3(256), 0, stream(), g, (const float*)src,
                           (const float*)flt, (const float*)bias, (float*)dst);
    else
        hipLaunchKernelGGL((conv_f32_small_kernel<1, 1>), grid, dim3(256), 0, stream(), g, (const float*)src,
                           (const float*)flt, (const float*)bias, (float*)dst);
    return check_launch("conv_f32_small");
}

}  // namespace mg
