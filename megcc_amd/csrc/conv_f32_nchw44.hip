// f32 layers in the NCHW44 layout that are bound by memory traffic, not by arithmetic:
//   * channel-wise (depthwise) 3x3 / 5x5 / any square window, stride 1 or 2, any padding:
//     GeneralIntrinsic::ChannelWiseFloatMk4, `GI_chanwise_kernel_conv2d_<k>x<k>_NCHW44_GROUP_...`
//     (GeneralIntrinsic/ConvKernel/Fp32ChannelWiseMk4.cpp:326-356), and
//   * the first layer of a network, NCHW source -> NCHW44 result, 1..4 input channels:
//     GeneralIntrinsic::ConvFloatNCHWNCHW44, `GI_kernel_conv2d_..._nchw_nchw44_oc<n>_ic<n>`
//     (GeneralIntrinsic/ConvKernel/Fp32ConvNchwNchw44.cpp:12-55).
// In NCHW44 the four channels of a pixel are one float4, so both kernels move whole 16-byte words
// and multiply on the vector ALU (2 to 9.4 K multiply-adds per 16 bytes written - below what the
// memory system needs for those bytes except for the 7x7 stems). Sums are formed tap by tap in the
// order fh, fw(, ic); the reference's kernels vectorise over the same four channels, results agree
// to rounding (held to 1e-4).
#include "common.h"
#include "conv_geom.h"
#include "epilogue.h"

namespace mg {

static __device__ __forceinline__ float f32_act(int act, float x) {
    switch (act) {
        case MEGCC_NONLINE_RELU: return act_apply<MEGCC_NONLINE_RELU>(x);
        case MEGCC_NONLINE_H_SWISH: return act_apply<MEGCC_NONLINE_H_SWISH>(x);
        case MEGCC_NONLINE_SIGMOID: return act_apply<MEGCC_NONLINE_SIGMOID>(x);
        default: return x;
    }
}

// ---- channel-wise ------------------------------------------------------------------------------
// A workgroup makes DW_TH x DW_TW output pixels of one (image, channel group) plane. The input
// pixels under them - ((DW_TH - 1) S + K) x ((DW_TW - 1) S + K) float4 - are staged in LDS with
// coalesced 16-byte loads (a pixel outside the image is loaded from a clamped address and stored
// as zero: no load sits under a branch), then every thread reads its K x K window from LDS
// (16-byte reads, consecutive lanes = consecutive words for stride 1). The K x K filter words of
// the plane are the same for the whole workgroup and come through the scalar cache.
static constexpr int DW_TH = 4, DW_TW = 64;

template <int K, int S>
__global__ void __launch_bounds__(DW_TH * DW_TW) dwconv44_f32_kernel(
        ConvGeom g, const float4* __restrict__ src, const float4* __restrict__ flt,
        const float4* __restrict__ bias, float4* __restrict__ dst, int col_tiles, int row_tiles) {
    constexpr int IN_H = (DW_TH - 1) * S + K, IN_W = (DW_TW - 1) * S + K;
    __shared__ float4 tile[IN_H][IN_W];
    const int tid = threadIdx.x;
    // blockIdx.x = (plane * row_tiles + row tile) * col_tiles + col tile
    const int ct = blockIdx.x % col_tiles, rest = blockIdx.x / col_tiles;
    const int rt = rest % row_tiles, plane = rest / row_tiles;  // plane = n * C/4 + channel group
    const int cg = plane % (g.ic >> 2);
    const int oh0 = rt * DW_TH, ow0 = ct * DW_TW;
    const int ih0 = oh0 * S - g.ph, iw0 = ow0 * S - g.pw;
    const float4* const in = src + (size_t)plane * g.ih * g.iw;
    for (int i = tid; i < IN_H * IN_W; i += DW_TH * DW_TW) {
        const int r = i / IN_W, c = i - r * IN_W;
        const int ih = ih0 + r, iw = iw0 + c;
        const bool ok = (unsigned)ih < (unsigned)g.ih && (unsigned)iw < (unsigned)g.iw;
        const int ihc = min(max(ih, 0), g.ih - 1), iwc = min(max(iw, 0), g.iw - 1);
        const float4 v = in[(size_t)ihc * g.iw + iwc];
        tile[r][c] = ok ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();
    const int ty = tid / DW_TW, tx = tid - ty * DW_TW;
    const int oh = oh0 + ty, ow = ow0 + tx;
    const float4* const w = flt + (size_t)cg * K * K;
    float4 acc = bias ? bias[cg] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int fh = 0; fh < K; ++fh)
#pragma unroll
        for (int fw = 0; fw < K; ++fw) {
            const float4 x = tile[ty * S + fh][tx * S + fw];
            const float4 f = w[fh * K + fw];
            acc.x += x.x * f.x;
            acc.y += x.y * f.y;
            acc.z += x.z * f.z;
            acc.w += x.w * f.w;
        }
    if (oh < g.oh && ow < g.ow) {
        acc.x = f32_act(g.act, acc.x);
        acc.y = f32_act(g.act, acc.y);
        acc.z = f32_act(g.act, acc.z);
        acc.w = f32_act(g.act, acc.w);
        dst[((size_t)plane * g.oh + oh) * g.ow + ow] = acc;
    }
}

bool dwconv44_f32_supported(const ConvGeom& g) {
    const long planes = (long)g.n * (g.ic >> 2);
    const long blocks = planes * ((g.oh + DW_TH - 1) / DW_TH) * ((g.ow + DW_TW - 1) / DW_TW);
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups == g.ic && g.ic == g.oc && g.groups > 1 && (g.ic & 3) == 0 &&
           g.fh == g.fw && (g.fh == 3 || g.fh == 5) && g.sh == g.sw && (g.sh == 1 || g.sh == 2) && g.dh == 1 &&
           g.dw == 1 && g.oh >= 1 && g.ow >= 1 && g.ih >= 1 && g.iw >= 1 && blocks >= 1 && blocks < (1L << 31) &&
           (long)g.n * g.ic * g.ih * g.iw < (1L << 31) && (long)g.n * g.oc * g.oh * g.ow < (1L << 31);
}

TinyNNStatus dwconv44_f32_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    const int col_tiles = (g.ow + DW_TW - 1) / DW_TW, row_tiles = (g.oh + DW_TH - 1) / DW_TH;
    const dim3 grid((unsigned)((long)g.n * (g.ic >> 2) * row_tiles * col_tiles));
#define MG_DW_F32(K, S)                                                                                      \
    hipLaunchKernelGGL((dwconv44_f32_kernel<K, S>), grid, dim3(DW_TH * DW_TW), 0, stream(), g,               \
                       (const float4*)src, (const float4*)flt, (const float4*)bias, (float4*)dst, col_tiles, \
                       row_tiles)
    if (g.fh == 3 && g.sh == 1)
        MG_DW_F32(3, 1);
    else if (g.fh == 3)
        MG_DW_F32(3, 2);
    else if (g.sh == 1)
        MG_DW_F32(5, 1);
    else
        MG_DW_F32(5, 2);
#undef MG_DW_F32
    return check_launch("dwconv44_f32");
}

// ---- first layer: NCHW source, NCHW44 result ------------------------------------------------------
// A thread makes one output pixel for up to FL_OCG groups of 4 output channels (blockIdx.y walks
// further groups): the IC * K * K source values under the pixel are loaded once (clamped address,
// zero where the tap is padding; consecutive lanes = consecutive output pixels of a row, so a
// wave-load is one stretch of a source row) and each meets FL_OCG filter words [4 oc] that are the
// same for the whole workgroup (scalar cache). Filter layout: [OC/4][FH][FW][IC][4 oc]
// (BareMetal/ConvKernel.cpp:53-57, the layout the reference's own first-layer kernel re-packs from).
static constexpr int FL_OCG = 8;

template <int K>
__global__ void __launch_bounds__(256) conv_first_f32_kernel(
        ConvGeom g, const float* __restrict__ src, const float4* __restrict__ flt,
        const float4* __restrict__ bias, float4* __restrict__ dst, int pix_blocks) {
    const int n = blockIdx.x / pix_blocks, pb = blockIdx.x - n * pix_blocks;
    const int ohw = g.oh * g.ow;
    const int p = pb * 256 + threadIdx.x;
    const int pc = min(p, ohw - 1);  // (surplus lanes of the last block repeat the last pixel)
    const int oh = pc / g.ow, ow = pc - oh * g.ow;
    const int og0 = blockIdx.y * FL_OCG, ogs = g.oc >> 2;
    float4 acc[FL_OCG];
#pragma unroll
    for (int j = 0; j < FL_OCG; ++j)
        acc[j] = bias && og0 + j < ogs ? bias[og0 + j] : make_float4(0.f, 0.f, 0.f, 0.f);
    const float* const in = src + (size_t)n * g.ic * g.ih * g.iw;
    for (int ic = 0; ic < g.ic; ++ic) {
        float x[K * K];
#pragma unroll
        for (int fh = 0; fh < K; ++fh)
#pragma unroll
            for (int fw = 0; fw < K; ++fw) {
                const int ih = oh * g.sh + fh - g.ph, iw = ow * g.sw + fw - g.pw;
                const bool ok = (unsigned)ih < (unsigned)g.ih && (unsigned)iw < (unsigned)g.iw;
                const int ihc = min(max(ih, 0), g.ih - 1), iwc = min(max(iw, 0), g.iw - 1);
                const float v = in[((size_t)ic * g.ih + ihc) * g.iw + iwc];
                x[fh * K + fw] = ok ? v : 0.f;
            }
#pragma unroll
        for (int j = 0; j < FL_OCG; ++j) {
            // (groups beyond OC / 4 read the last group's filter words; their sums are not stored)
            const float4* const w = flt + ((size_t)min(og0 + j, ogs - 1) * K * K) * g.ic + ic;
#pragma unroll
            for (int t = 0; t < K * K; ++t) {
                const float4 f = w[(size_t)t * g.ic];
                acc[j].x += x[t] * f.x;
                acc[j].y += x[t] * f.y;
                acc[j].z += x[t] * f.z;
                acc[j].w += x[t] * f.w;
            }
        }
    }
    if (p < ohw) {
#pragma unroll
        for (int j = 0; j < FL_OCG; ++j)
            if (og0 + j < ogs) {
                float4 r = acc[j];
                r.x = f32_act(g.act, r.x);
                r.y = f32_act(g.act, r.y);
                r.z = f32_act(g.act, r.z);
                r.w = f32_act(g.act, r.w);
                dst[((size_t)n * ogs + og0 + j) * ohw + p] = r;
            }
    }
}

bool conv_first_f32_supported(const ConvGeom& g) {
    const long ohw = (long)g.oh * g.ow;
    return g.fmt == MEGCC_FMT_NCHW_NCHW44 && g.groups == 1 && g.ic >= 1 && g.ic <= 4 && (g.oc & 3) == 0 &&
           g.oc >= 4 && g.fh == g.fw && (g.fh == 3 || g.fh == 5 || g.fh == 7) && g.dh == 1 && g.dw == 1 &&
           g.sh >= 1 && g.sw >= 1 && ohw >= 1 && ohw < (1L << 30) && (ohw + 255) / 256 * g.n < (1L << 31) &&
           (g.oc / 4 + FL_OCG - 1) / FL_OCG <= 65535 && (long)g.n * g.ic * g.ih * g.iw < (1L << 31) &&
           (long)g.n * g.oc * ohw < (1L << 31);
}

TinyNNStatus conv_first_f32_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    const int pix_blocks = (g.oh * g.ow + 255) / 256;
    const dim3 grid((unsigned)(pix_blocks * g.n), (unsigned)((g.oc / 4 + FL_OCG - 1) / FL_OCG));
#define MG_FIRST_F32(K)                                                                                     \
    hipLaunchKernelGGL((conv_first_f32_kernel<K>), grid, dim3(256), 0, stream(), g, (const float*)src,      \
                       (const float4*)flt, (const float4*)bias, (float4*)dst, pix_blocks)
    if (g.fh == 3)
        MG_FIRST_F32(3);
    else if (g.fh == 5)
        MG_FIRST_F32(5);
    else
        MG_FIRST_F32(7);
#undef MG_FIRST_F32
    return check_launch("conv_first_f32");
}

}  // namespace mg
