// f32 NCHW dense convolution for SMALL layers (a few tens of MFLOP: the batch-1 first layers of a
// float model, e.g. 32 -> 32 channels on 56 x 56): one launch, no matrix cores, no split-K. A
// workgroup owns 64 output pixels and 2 output channels, each of its 4 waves a quarter of the input
// channels; the filter rows of its 2 channels are read through
// wave-uniform addresses (one cache line per load), the input pixels coalesced along the row;
// about a wave per SIMD for such a layer, so the whole thing is launch + a few microseconds. The
// tiled implicit GEMM needs a split over K and a second (reduce) launch to fill the chip here.
// Summation order: four slices of the input channels, each input channel, filter row, filter column
// ascending; the partial sums in slice order; then the bias
// (GeneralIntrinsic/ConvKernel/Fp32Im2col.cpp:88-218 accumulates in GEMM order; f32 results are
// held to the 1e-4 tolerance, not to bit equality).
#include "common.h"
#include "conv_geom.h"
#include "epilogue.h"

namespace mg {

static constexpr int CS_OCW = 2;  // output channels per wave
static constexpr int CS_ICS = 4;  // input channels whose taps are in flight together
static constexpr int CS_SLICES = 4;  // waves of a workgroup = slices of the input channels

__device__ __forceinline__ float cs_act(int act, float x) {
    switch (act) {
        case MEGCC_NONLINE_RELU: return act_apply<MEGCC_NONLINE_RELU>(x);
        case MEGCC_NONLINE_H_SWISH: return act_apply<MEGCC_NONLINE_H_SWISH>(x);
        case MEGCC_NONLINE_SIGMOID: return act_apply<MEGCC_NONLINE_SIGMOID>(x);
        default: return x;
    }
}

template <int FH, int FW>
__global__ void __launch_bounds__(64 * CS_SLICES) conv_f32_small_kernel(
        ConvGeom g, const float* __restrict__ src, const float* __restrict__ flt,
        const float* __restrict__ bias, float* __restrict__ dst) {
    __shared__ float red[CS_SLICES][CS_OCW][64];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ohw = g.oh * g.ow;
    const int P = g.n * ohw;
    const int p = blockIdx.x * 64 + lane;
    // wave-uniform: the filter rows are read through the scalar cache
    const int oc0 = blockIdx.y * CS_OCW;
    // The workgroup's waves share the 64 pixels x 2 channels and split the input channels:
    // a wave's loop is a chain of dependent round trips (taps, then filter rows, per step of
    // CS_ICS channels), and a quarter of the channels is a quarter of the chain (eight slices measured no better: 7.2 us against 6.9).
    const int icq = (g.ic + CS_SLICES - 1) / CS_SLICES;
    const int ic_begin = min(wave * icq, g.ic), ic_end = min(ic_begin + icq, g.ic);
    const int pp = p < P ? p : P - 1;  // lanes beyond the end repeat the last pixel, store nothing
    const int n = pp / ohw, r = pp - n * ohw;
    const int oh = r / g.ow, ow = r - oh * g.ow;
    const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
    const float* img = src + (size_t)n * g.ic * g.ih * g.iw;
    const int K = g.ic * FH * FW;
    const float* w0 = flt + (size_t)oc0 * K;
    const bool two = oc0 + 1 < g.oc;
    const float* w1 = two ? w0 + K : w0;
    // taps inside the image, one bit per (fh, fw), and each tap's offset in its plane. A tap
    // outside reads element 0 of the plane and is replaced by 0 after the load: a load under a
    // condition makes the compiler wait for every outstanding load at the join, and the 9 loads of
    // a channel were 9 dependent cache round trips (288 of them for 32 channels: 12 us).
    unsigned valid = 0;
    int off[FH * FW];
#pragma unroll
    for (int fh = 0; fh < FH; ++fh)
#pragma unroll
        for (int fw = 0; fw < FW; ++fw) {
            const unsigned ih = (unsigned)(ih0 + fh * g.dh), iw = (unsigned)(iw0 + fw * g.dw);
            const bool in = ih < (unsigned)g.ih && iw < (unsigned)g.iw;
            valid |= (unsigned)in << (fh * FW + fw);
            off[fh * FW + fw] = in ? (int)(ih * g.iw + iw) : 0;
        }
    float a0 = 0.f, a1 = 0.f;
    // the taps of CS_ICS channels are requested together (a channel beyond the last repeats the
    // last one and contributes zeros; no branch around the products, or their loads would be moved
    // into it, next to their use)
    for (int ic0 = ic_begin; ic0 < ic_end; ic0 += CS_ICS) {
        float x[CS_ICS][FH * FW];
#pragma unroll
        for (int u = 0; u < CS_ICS; ++u) {
            const float* plane = img + (size_t)min(ic0 + u, ic_end - 1) * g.ih * g.iw;
#pragma unroll
            for (int t = 0; t < FH * FW; ++t)
                x[u][t] = plane[off[t]];
        }
#pragma unroll
        for (int u = 0; u < CS_ICS; ++u) {
            const int ic = min(ic0 + u, ic_end - 1);
            const unsigned live = ic0 + u < ic_end ? valid : 0u;
#pragma unroll
            for (int t = 0; t < FH * FW; ++t) {
                const float xt = (live >> t) & 1 ? x[u][t] : 0.f;
                a0 += xt * w0[ic * FH * FW + t];
                a1 += xt * w1[ic * FH * FW + t];
            }
        }
    }
    red[wave][0][lane] = a0;
    red[wave][1][lane] = a1;
    __syncthreads();
    // waves 0 and 1 finish channel oc0 and oc0 + 1: the partial sums in slice order, the bias
    if (wave < CS_OCW && p < P && oc0 + wave < g.oc) {
        float v = red[0][wave][lane];
#pragma unroll
        for (int w = 1; w < CS_SLICES; ++w)
            v += red[w][wave][lane];
        dst[((size_t)n * g.oc + oc0 + wave) * ohw + r] = cs_act(g.act, v + (bias ? bias[oc0 + wave] : 0.f));
    }
}

// 3x3 and 1x1 f32 NCHW dense layers of at most 2^27 multiply-adds
bool conv_f32_small_supported(const ConvGeom& g) {
    const long P = (long)g.n * g.oh * g.ow;
    const long macs = P * g.oc * g.ic * g.fh * g.fw;
    return g.fmt == MEGCC_FMT_NCHW && g.groups == 1 && ((g.fh == 3 && g.fw == 3) || (g.fh == 1 && g.fw == 1)) &&
           P >= 1 && P < (1L << 30) && macs <= (1L << 27) && g.oc >= 1 && g.oc <= 65535 * CS_OCW &&
           (long)g.n * g.ic * g.ih * g.iw < (1L << 31) && P * g.oc < (1L << 31);
}

TinyNNStatus conv_f32_small_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    const long P = (long)g.n * g.oh * g.ow;
    const dim3 grid((unsigned)((P + 63) / 64), (unsigned)((g.oc + CS_OCW - 1) / CS_OCW));
    if (g.fh == 3)
        hipLaunchKernelGGL((conv_f32_small_kernel<3, 3>), grid, dim3(64 * CS_SLICES), 0, stream(), g, (const float*)src,
                           (const float*)flt, (const float*)bias, (float*)dst);
    else
        hipLaunchKernelGGL((conv_f32_small_kernel<1, 1>), grid, dim3(64 * CS_SLICES), 0, stream(), g, (const float*)src,
                           (const float*)flt, (const float*)bias, (float*)dst);
    return check_launch("conv_f32_small");
}

}  // namespace mg
