// Direct (one thread per output) convolution kernels. They cover every layout / sparsity /
// stride / dilation combination of BareMetal::ConvGeneral (BareMetal/ConvKernel.cpp:305-344) and
// are the implementation of the cases that have no specialised kernel: qsi8 NCHW with spatial
// extent, the NCHW->NCHW44 first layer (IC = 3), NCHW depthwise, dilated convolutions, and f32 in
// the NCHW44 / GROUP layouts. Dense qsi8 NCHW44 and FullyConnected run on conv_mfma_i8.hip, NCHW44
// depthwise on dwconv.hip, f32 NCHW dense on gemm_f32.hip.
#include "common.h"
#include "conv_geom.h"
#include "epilogue.h"

namespace mg {

// element offsets, BareMetal/FormatHelper.cpp:12-36 on contiguous tensors
__device__ __forceinline__ size_t off_nchw(int C, int H, int W, int n, int c, int h, int w) {
    return (((size_t)n * C + c) * H + h) * W + w;
}
__device__ __forceinline__ size_t off_nchw44(int C, int H, int W, int n, int c, int h, int w) {
    return ((((size_t)n * (C >> 2) + (c >> 2)) * H + h) * W + w) * 4 + (c & 3);
}

// filter offsets, BareMetal/ConvKernel.cpp:48-113
__device__ __forceinline__ size_t flt_off(
        const ConvGeom& g, int grp, int ocl, int icl, int fh, int fw, int ocpg, int icpg) {
    if (g.fmt == MEGCC_FMT_NCHW) {
        return ((((size_t)grp * ocpg + ocl) * icpg + icl) * g.fh + fh) * g.fw + fw;
    } else if (g.fmt == MEGCC_FMT_NCHW_NCHW44) {
        return ((((size_t)(ocl >> 2) * g.fh + fh) * g.fw + fw) * icpg + icl) * 4 + (ocl & 3);
    } else if (g.groups == 1) {
        return (((((size_t)(ocl >> 2) * (icpg >> 2) + (icl >> 2)) * g.fh + fh) * g.fw + fw) * 4 +
                (icl & 3)) * 4 + (ocl & 3);
    } else {
        return (((size_t)(grp >> 2) * g.fh + fh) * g.fw + fw) * 4 + (grp & 3);
    }
}

template <typename T, typename ACC>
__device__ __forceinline__ ACC conv_point(
        const ConvGeom& g, const T* __restrict__ src, const T* __restrict__ flt, int n, int oc,
        int oh, int ow) {
    const int ocpg = g.oc / g.groups, icpg = g.ic / g.groups;
    const int grp = oc / ocpg, ocl = oc - grp * ocpg;
    const bool src44 = g.fmt == MEGCC_FMT_NCHW44;
    ACC acc = 0;
    for (int fh = 0; fh < g.fh; ++fh) {
        unsigned ih = (unsigned)(oh * g.sh + fh * g.dh - g.ph);
        if (ih >= (unsigned)g.ih)
            continue;
        for (int fw = 0; fw < g.fw; ++fw) {
            unsigned iw = (unsigned)(ow * g.sw + fw * g.dw - g.pw);
            if (iw >= (unsigned)g.iw)
                continue;
            for (int icl = 0; icl < icpg; ++icl) {
                int ic = grp * icpg + icl;
                ACC s = src44 ? (ACC)src[off_nchw44(g.ic, g.ih, g.iw, n, ic, ih, iw)]
                              : (ACC)src[off_nchw(g.ic, g.ih, g.iw, n, ic, ih, iw)];
                ACC f = (ACC)flt[flt_off(g, grp, ocl, icl, fh, fw, ocpg, icpg)];
                acc += s * f;
            }
        }
    }
    return acc;
}

template <int ACT>
__global__ void __launch_bounds__(256) conv_direct_q8(
        ConvGeom g, const int8_t* __restrict__ src, const int8_t* __restrict__ flt,
        const int32_t* __restrict__ bias, int8_t* __restrict__ dst) {
    const size_t total = (size_t)g.n * g.oc * g.oh * g.ow;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        int n, oc, oh, ow;
        size_t r = i;
        if (g.fmt == MEGCC_FMT_NCHW) {
            ow = r % g.ow; r /= g.ow;
            oh = r % g.oh; r /= g.oh;
            oc = r % g.oc; n = (int)(r / g.oc);
        } else {
            int o4 = r & 3; r >>= 2;
            ow = r % g.ow; r /= g.ow;
            oh = r % g.oh; r /= g.oh;
            int c4 = r % (g.oc >> 2); n = (int)(r / (g.oc >> 2));
            oc = c4 * 4 + o4;
        }
        int acc = conv_point<int8_t, int>(g, src, flt, n, oc, oh, ow);
        if (bias)
            acc += bias[oc];
        dst[i] = (int8_t)requant_conv<ACT>(acc, g.s_src, g.s_flt, g.s_dst);
    }
}

template <int ACT>
__global__ void __launch_bounds__(256) conv_direct_f32(
        ConvGeom g, const float* __restrict__ src, const float* __restrict__ flt,
        const float* __restrict__ bias, float* __restrict__ dst) {
    const size_t total = (size_t)g.n * g.oc * g.oh * g.ow;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        int n, oc, oh, ow;
        size_t r = i;
        if (g.fmt == MEGCC_FMT_NCHW) {
            ow = r % g.ow; r /= g.ow;
            oh = r % g.oh; r /= g.oh;
            oc = r % g.oc; n = (int)(r / g.oc);
        } else {
            int o4 = r & 3; r >>= 2;
            ow = r % g.ow; r /= g.ow;
            oh = r % g.oh; r /= g.oh;
            int c4 = r % (g.oc >> 2); n = (int)(r / (g.oc >> 2));
            oc = c4 * 4 + o4;
        }
        float acc = conv_point<float, float>(g, src, flt, n, oc, oh, ow);
        if (bias)
            acc += bias[oc];
        dst[i] = act_apply<ACT>(acc);
    }
}

template <int ACT>
static void launch_q8(const ConvGeom& g, const void* s, const void* f, const void* b, void* d) {
    size_t total = (size_t)g.n * g.oc * g.oh * g.ow;
    unsigned blocks = (unsigned)((total + 255) / 256);
    if (blocks > 65536u * 4)
        blocks = 65536u * 4;
    hipLaunchKernelGGL(conv_direct_q8<ACT>, dim3(blocks), dim3(256), 0, stream(), g,
                       (const int8_t*)s, (const int8_t*)f, (const int32_t*)b, (int8_t*)d);
}
template <int ACT>
static void launch_f32(const ConvGeom& g, const void* s, const void* f, const void* b, void* d) {
    size_t total = (size_t)g.n * g.oc * g.oh * g.ow;
    unsigned blocks = (unsigned)((total + 255) / 256);
    if (blocks > 65536u * 4)
        blocks = 65536u * 4;
    hipLaunchKernelGGL(conv_direct_f32<ACT>, dim3(blocks), dim3(256), 0, stream(), g,
                       (const float*)s, (const float*)f, (const float*)b, (float*)d);
}

TinyNNStatus conv_direct_launch(
        const ConvGeom& g, bool is_float, const void* src, const void* flt, const void* bias,
        void* dst) {
    if ((size_t)g.n * g.oc * g.oh * g.ow == 0)
        return TinyNN_SUCCESS;
#define MG_ACT_SWITCH(fn)                                         \
    switch (g.act) {                                              \
        case MEGCC_NONLINE_IDENTITY: fn<MEGCC_NONLINE_IDENTITY>(g, src, flt, bias, dst); break; \
        case MEGCC_NONLINE_RELU: fn<MEGCC_NONLINE_RELU>(g, src, flt, bias, dst); break;         \
        case MEGCC_NONLINE_H_SWISH: fn<MEGCC_NONLINE_H_SWISH>(g, src, flt, bias, dst); break;   \
        default: fn<MEGCC_NONLINE_SIGMOID>(g, src, flt, bias, dst); break;                      \
    }
    if (is_float) {
        MG_ACT_SWITCH(launch_f32)
    } else {
        MG_ACT_SWITCH(launch_q8)
    }
#undef MG_ACT_SWITCH
    return check_launch("conv_direct");
}

}  // namespace mg
