// Dense qsi8 NCHW44 convolution of any filter size, stride and dilation on the 4-way int8 dot
// product (v_dot4_i32_i8): the implementation of what the matrix-core kernels do not take - more
// than 9 taps (5x5, 7x7), or a filter that did not go through the init step. Same loop nest and
// epilogue as BareMetal/ConvKernel.cpp:305-344,374-380 on src [N,C/4,H,W,4] and filter
// [OC/4,IC/4,FH,FW,4 ic,4 oc] (:58-64,95-99).
//   * a thread owns one output pixel x OCB groups of 4 output channels; a pixel's 4 input channels
//     are one dword = one operand of the dot product;
//   * the 16 filter bytes of an (ic group, tap, oc group) are the same for the whole workgroup:
//     they arrive through the scalar cache (loads only) and are transposed from [ic][oc] to
//     [oc][ic] by 6 byte permutes;
//   * 12 vector instructions per 16 MACs and lane; no LDS, no staging. About 25x the
//     one-output-per-thread kernel, far below the matrix cores - a fallback, not a fast path.
#include "common.h"
#include "conv_geom.h"
#include "epilogue.h"

namespace mg {

struct Dot4Params {
    const uint32_t* src;
    const int8_t* flt;
    const int32_t* bias;
    uint32_t* dst;
    ConvGeom g;
    int ic4, oc4;
};

template <int OCB>
__global__ void __launch_bounds__(256) conv_dot4_kernel(Dot4Params q) {
    const ConvGeom& g = q.g;
    const int p = blockIdx.x * 256 + threadIdx.x;
    const int npix = g.oh * g.ow;
    const bool live = p < npix;
    const int pc = live ? p : npix - 1;
    const int oh = pc / g.ow, ow = pc - oh * g.ow;
    const int o0 = blockIdx.y * OCB, n = blockIdx.z;
    int acc[OCB][4];
#pragma unroll
    for (int b = 0; b < OCB; ++b)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[b][j] = (q.bias && o0 + b < q.oc4) ? q.bias[(o0 + b) * 4 + j] : 0;
    const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
    for (int c4 = 0; c4 < q.ic4; ++c4) {
        const uint32_t* plane = q.src + ((size_t)n * q.ic4 + c4) * g.ih * g.iw;
        for (int fh = 0; fh < g.fh; ++fh) {
            const int ih = ih0 + fh * g.dh;
            const bool rowok = (unsigned)ih < (unsigned)g.ih;
            for (int fw = 0; fw < g.fw; ++fw) {
                const int iw = iw0 + fw * g.dw;
                const bool ok = rowok && (unsigned)iw < (unsigned)g.iw;
                const int s = ok ? (int)plane[ih * g.iw + iw] : 0;
#pragma unroll
                for (int b = 0; b < OCB; ++b) {
                    if (o0 + b >= q.oc4)  // the same for the whole workgroup
                        break;
                    const uint4 f = *(const uint4*)(q.flt + ((((size_t)(o0 + b) * q.ic4 + c4) * g.fh + fh) * g.fw + fw) * 16);
                    // f.x .. f.w = input channel 0 .. 3, bytes = output channel 0 .. 3: transpose
                    const uint32_t lo = __builtin_amdgcn_perm(f.y, f.x, 0x05010400);   // x0 y0 x1 y1
                    const uint32_t hi = __builtin_amdgcn_perm(f.w, f.z, 0x05010400);   // z0 w0 z1 w1
                    const uint32_t lo2 = __builtin_amdgcn_perm(f.y, f.x, 0x07030602);  // x2 y2 x3 y3
                    const uint32_t hi2 = __builtin_amdgcn_perm(f.w, f.z, 0x07030602);
                    acc[b][0] = __builtin_amdgcn_sdot4(s, (int)__builtin_amdgcn_perm(hi, lo, 0x05040100), acc[b][0], false);
                    acc[b][1] = __builtin_amdgcn_sdot4(s, (int)__builtin_amdgcn_perm(hi, lo, 0x07060302), acc[b][1], false);
                    acc[b][2] = __builtin_amdgcn_sdot4(s, (int)__builtin_amdgcn_perm(hi2, lo2, 0x05040100), acc[b][2], false);
                    acc[b][3] = __builtin_amdgcn_sdot4(s, (int)__builtin_amdgcn_perm(hi2, lo2, 0x07060302), acc[b][3], false);
                }
            }
        }
    }
    if (!live)
        return;
#pragma unroll
    for (int b = 0; b < OCB; ++b) {
        if (o0 + b >= q.oc4)
            break;
        int r[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            r[j] = requant_conv_rt(g.act, acc[b][j], g.s_src, g.s_flt, g.s_dst);
        q.dst[((size_t)n * q.oc4 + o0 + b) * npix + p] = pack4_perm(r[0], r[1], r[2], r[3]);
    }
}

bool conv_dot4_supported(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups == 1 && (g.ic & 3) == 0 && (g.oc & 3) == 0 && g.ic >= 4 &&
           g.oc >= 4 && (long)g.ih * g.iw < (1L << 31) && (long)g.oh * g.ow < (1L << 31) - 256 &&
           g.n <= 65535 && (g.oc / 4 + 1) / 2 <= 65535;
}

TinyNNStatus conv_dot4_launch(const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    Dot4Params q = {};
    q.src = (const uint32_t*)src;
    q.flt = (const int8_t*)flt;
    q.bias = (const int32_t*)bias;
    q.dst = (uint32_t*)dst;
    q.g = g;
    q.ic4 = g.ic / 4;
    q.oc4 = g.oc / 4;
    const unsigned tiles = (unsigned)(((long)g.oh * g.ow + 255) / 256);
    // two groups of output channels per thread halve the activation loads; one when that would
    // leave too few workgroups
    if ((long)tiles * ((q.oc4 + 1) / 2) * g.n >= 2L * num_cus())
        hipLaunchKernelGGL(conv_dot4_kernel<2>, dim3(tiles, (q.oc4 + 1) / 2, g.n), dim3(256), 0, stream(), q);
    else
        hipLaunchKernelGGL(conv_dot4_kernel<1>, dim3(tiles, q.oc4, g.n), dim3(256), 0, stream(), q);
    return check_launch("conv_dot4");
}

}  // namespace mg
