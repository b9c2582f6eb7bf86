// qsi8 first-layer convolution: NCHW input with 3 channels -> NCHW44 output, 3x3, stride 2, pad 1
// (the "hybrid" format NCHW_NCHW44 of MegCC's nchw44 layout pass; filter [OC/4, FH, FW, IC, 4oc],
// same loop nest and epilogue as BareMetal/ConvKernel.cpp:305-344,374-380).
//
// K = 27 is far too short for the matrix cores and the layer moves 3.7 bytes per MAC-quad, so
// this is a VALU kernel built around v_dot4_i32_i8:
//   * one thread = two horizontally adjacent output pixels (ow even) x all output channels. With
//     stride 2 and pad 1 the two pixels need input columns 4k-1 .. 4k+3 of three rows per channel:
//     the last byte of one aligned dword and the whole next one, so every load is an aligned dword
//     and consecutive lanes read consecutive dwords;
//   * per (channel, filter row) the 3 taps of a pixel are one dword (v_alignbyte / shift), the
//     matching weights one dword (w0, w1, w2, 0): 9 dot4 per pixel and output channel;
//   * weights are re-packed once per workgroup into LDS as [oc/4][ic*3+fh][4 oc] dwords and read
//     back as wave-wide broadcasts; bias and the 8 results of an oc group stay in registers and
//     leave as one 8-byte store (pixels ow, ow+1 of one NCHW44 plane).
// Only the top row and the left column can be padding for even IH, IW.
#include "common.h"
#include "conv_geom.h"
#include "epilogue.h"

namespace mg {

static constexpr int CF_THREADS = 256;
static constexpr int CF_MAX_OC = 128;
typedef int cf_v4i __attribute__((ext_vector_type(4)));

template <int ACT>
__global__ void __launch_bounds__(CF_THREADS) conv_first_q8_kernel(
        ConvGeom g, RequantFast rq, const int8_t* __restrict__ src, const int8_t* __restrict__ flt,
        const int32_t* __restrict__ bias, uint32_t* __restrict__ dst, int total_pairs,
        RequantTable table) {
    __shared__ __attribute__((aligned(16))) int wlds[CF_MAX_OC * 9];
    __shared__ __attribute__((aligned(16))) int blds[CF_MAX_OC];
    __shared__ int tbl[REQUANT_TABLE_ENTRIES];
    if (ACT >= 0)
        tbl[threadIdx.x] = table.t[threadIdx.x];
    const int oc4n = g.oc >> 2;
    // packed weight dword (g4, row = ic*3 + fh, o): bytes fw = 0, 1, 2 and a zero
    for (int i = threadIdx.x; i < g.oc * 9; i += CF_THREADS) {
        const int o = i & 3, row = (i >> 2) % 9, g4 = (i >> 2) / 9;
        const int ic = row / 3, fh = row - ic * 3;
        uint32_t w = 0;
#pragma unroll
        for (int fw = 0; fw < 3; ++fw) {
            const int8_t v = flt[((((size_t)g4 * 3 + fh) * 3 + fw) * 3 + ic) * 4 + o];
            w |= (uint32_t)(uint8_t)v << (8 * fw);
        }
        wlds[i] = (int)w;
    }
    for (int i = threadIdx.x; i < g.oc; i += CF_THREADS)
        blds[i] = bias ? bias[i] : 0;
    __syncthreads();

    const int ow2n = g.ow >> 1;
    const int iw4 = g.iw >> 2;  // dwords per input row
    for (int p = blockIdx.x * CF_THREADS + threadIdx.x; p < total_pairs; p += gridDim.x * CF_THREADS) {
        int r = p;
        const int ow2 = r % ow2n; r /= ow2n;
        const int oh = r % g.oh;
        const int n = r / g.oh;
        // x[row][0 / 1]: the 3 taps of pixel ow = 2*ow2 / 2*ow2 + 1 in (channel, filter row) `row`
        int xa[9], xb[9];
        const uint32_t* img = (const uint32_t*)(src + (size_t)n * 3 * g.ih * g.iw);
#pragma unroll
        for (int ic = 0; ic < 3; ++ic) {
#pragma unroll
            for (int fh = 0; fh < 3; ++fh) {
                const int ih = 2 * oh - 1 + fh;
                uint32_t cur = 0, prev = 0;
                if ((unsigned)ih < (unsigned)g.ih) {
                    const uint32_t* rowp = img + ((size_t)ic * g.ih + ih) * iw4;
                    cur = rowp[ow2];
                    if (ow2 > 0)
                        prev = rowp[ow2 - 1];
                }
                xa[ic * 3 + fh] = (int)__builtin_amdgcn_alignbyte(cur, prev, 3);  // prev.b3 cur.b0 cur.b1 (cur.b2)
                xb[ic * 3 + fh] = (int)(cur >> 8);                                // cur.b1 cur.b2 cur.b3 0
            }
        }
        uint32_t* out = dst + ((size_t)n * oc4n * g.oh + oh) * g.ow + 2 * ow2;
        for (int g4 = 0; g4 < oc4n; ++g4) {
            const cf_v4i bv = *(const cf_v4i*)(blds + g4 * 4);
            int a[4] = {bv[0], bv[1], bv[2], bv[3]}, b[4] = {bv[0], bv[1], bv[2], bv[3]};
#pragma unroll
            for (int row = 0; row < 9; ++row) {
                const cf_v4i w = *(const cf_v4i*)(wlds + (g4 * 9 + row) * 4);
#pragma unroll
                for (int o = 0; o < 4; ++o) {
                    a[o] = __builtin_amdgcn_sdot4(xa[row], w[o], a[o], false);
                    b[o] = __builtin_amdgcn_sdot4(xb[row], w[o], b[o], false);
                }
            }
            int ra[4], rb[4];
#pragma unroll
            for (int o = 0; o < 4; ++o) {
                if (ACT < 0) {
                    ra[o] = requant_conv_rt(g.act, a[o], g.s_src, g.s_flt, g.s_dst);
                    rb[o] = requant_conv_rt(g.act, b[o], g.s_src, g.s_flt, g.s_dst);
                } else {
                    ra[o] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(a[o], rq.c, tbl);
                    rb[o] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(b[o], rq.c, tbl);
                }
            }
            uint2 v;
            v.x = pack4_perm(ra[0], ra[1], ra[2], ra[3]);
            v.y = pack4_perm(rb[0], rb[1], rb[2], rb[3]);
            *(uint2*)(out + (size_t)g4 * g.oh * g.ow) = v;
        }
    }
}

bool conv_first_supported(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW_NCHW44 && g.groups == 1 && g.ic == 3 && g.fh == 3 && g.fw == 3 &&
           g.sh == 2 && g.sw == 2 && g.ph == 1 && g.pw == 1 && g.dh == 1 && g.dw == 1 &&
           (g.iw & 3) == 0 && (g.ih & 1) == 0 && (g.oc & 3) == 0 && g.oc <= CF_MAX_OC &&
           g.ow * 2 == g.iw && g.oh * 2 == g.ih &&
           (long)g.n * g.oh * g.ow < (1L << 31);
}

TinyNNStatus conv_first_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    const long pairs = (long)g.n * g.oh * (g.ow / 2);
    if (pairs == 0)
        return TinyNN_SUCCESS;
    long blocks = (pairs + CF_THREADS - 1) / CF_THREADS;
    if (blocks > 256 * 16)
        blocks = 256 * 16;
    const RequantFast rq = make_requant_fast(g.s_src, g.s_flt, g.s_dst);
    // exact thresholds for the monotone activations; anything else (and extreme scales)
    // evaluates the literal sequence per output
    const bool tab = (g.act == MEGCC_NONLINE_IDENTITY || g.act == MEGCC_NONLINE_RELU) &&
                     requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    static const RequantTable no_table = {};
    const RequantTable& table = tab ? requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst) : no_table;
    auto kern = tab && g.act == MEGCC_NONLINE_IDENTITY ? conv_first_q8_kernel<MEGCC_NONLINE_IDENTITY>
              : tab && g.act == MEGCC_NONLINE_RELU     ? conv_first_q8_kernel<MEGCC_NONLINE_RELU>
                                                       : conv_first_q8_kernel<-1>;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(CF_THREADS), 0, stream(), g, rq,
                       (const int8_t*)src, (const int8_t*)flt, (const int32_t*)bias, (uint32_t*)dst,
                       (int)pairs, table);
    return check_launch("conv_first_q8");
}

}  // namespace mg
