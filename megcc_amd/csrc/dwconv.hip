// qsi8 depthwise (channel-wise GROUP) convolution in NCHW44: one thread per output dword, i.e. the
// 4 channels of one pixel. The tensor is [N, C/4, H, W, 4] and the filter [C/4, 1, 1, FH, FW, 4]
// (BareMetal/ConvKernel.cpp:62-64,100-101), so a pixel's 4 channels and a tap's 4 weights are one
// aligned dword each; consecutive lanes walk W, which makes every load and the store coalesced.
// Bandwidth-bound (18 int ops per byte moved): no MFMA. Same accumulator and epilogue as the
// reference's generic loop (ConvKernel.cpp:305-344,374-380).
#include "common.h"
#include "conv_geom.h"
#include "epilogue.cuh"

namespace mg {

template <int ACT>
__global__ void __launch_bounds__(256) dwconv44_q8_kernel(
        ConvGeom g, RequantFast rq, const uint32_t* __restrict__ src, const uint32_t* __restrict__ flt,
        const int32_t* __restrict__ bias, uint32_t* __restrict__ dst) {
    const int c4n = g.oc >> 2;
    const size_t total = (size_t)g.n * c4n * g.oh * g.ow;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i;
        int ow = r % g.ow; r /= g.ow;
        int oh = r % g.oh; r /= g.oh;
        int c4 = r % c4n;
        int n = (int)(r / c4n);
        int acc[4] = {0, 0, 0, 0};
        const uint32_t* plane = src + ((size_t)n * c4n + c4) * g.ih * g.iw;
        const uint32_t* w = flt + (size_t)c4 * g.fh * g.fw;
        for (int fh = 0; fh < g.fh; ++fh) {
            unsigned ih = (unsigned)(oh * g.sh + fh * g.dh - g.ph);
            if (ih >= (unsigned)g.ih)
                continue;
            for (int fw = 0; fw < g.fw; ++fw) {
                unsigned iw = (unsigned)(ow * g.sw + fw * g.dw - g.pw);
                if (iw >= (unsigned)g.iw)
                    continue;
                uint32_t s = plane[ih * g.iw + iw];
                uint32_t f = w[fh * g.fw + fw];
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    acc[c] += sbyte(s, c) * sbyte(f, c);
            }
        }
        int o[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int a = acc[c] + (bias ? bias[c4 * 4 + c] : 0);
            if (ACT < 0)
                o[c] = requant_conv_rt(g.act, a, g.s_src, g.s_flt, g.s_dst);
            else
                o[c] = requant_conv_fast<(ACT < 0 ? 0 : ACT)>(a, rq);
        }
        dst[i] = pack4(o[0], o[1], o[2], o[3]);
    }
}

bool dwconv44_supported(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups > 1 && g.groups == g.ic && g.ic == g.oc &&
           (g.ic & 3) == 0;
}

TinyNNStatus dwconv44_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    size_t total = (size_t)g.n * (g.oc >> 2) * g.oh * g.ow;
    if (total == 0)
        return TinyNN_SUCCESS;
    unsigned blocks = (unsigned)((total + 255) / 256);
    if (blocks > 65536u * 8)
        blocks = 65536u * 8;
    const RequantFast rq = make_requant_fast(g.s_src, g.s_flt, g.s_dst);
    auto kern = g.act == MEGCC_NONLINE_IDENTITY ? dwconv44_q8_kernel<MEGCC_NONLINE_IDENTITY>
              : g.act == MEGCC_NONLINE_RELU     ? dwconv44_q8_kernel<MEGCC_NONLINE_RELU>
                                                : dwconv44_q8_kernel<-1>;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), 0, stream(), g, rq, (const uint32_t*)src,
                       (const uint32_t*)flt, (const int32_t*)bias, (uint32_t*)dst);
    return check_launch("dwconv44_q8");
}

}  // namespace mg
