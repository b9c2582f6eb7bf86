// qsi8 depthwise (channel-wise GROUP) convolution in NCHW44: one thread per output dword, i.e. the
// 4 channels of one pixel. The tensor is [N, C/4, H, W, 4] and the filter [C/4, 1, 1, FH, FW, 4]
// (BareMetal/ConvKernel.cpp:62-64,100-101), so a pixel's 4 channels and a tap's 4 weights are one
// aligned dword each; consecutive lanes walk W, which makes every load and the store coalesced.
// Bandwidth-bound (18 int ops per byte moved): no MFMA. Same accumulator and epilogue as the
// reference's generic loop (ConvKernel.cpp:305-344,374-380).
#include <stdlib.h>

#include "common.h"
#include "conv_geom.h"
#include "conv_mfma_i8.h"
#include "epilogue.h"

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


// ---- 3x3, pad 1, stride 1 or 2 -----------------------------------------------------------------
// One thread = 4 horizontally adjacent output pixels x the 4 channels of one NCHW44 plane group.
// The pixels of an input row arrive as aligned 16-byte loads (4 pixels x 4 channels); a 4x4 byte
// transpose (8 v_perm) turns them into one dword per channel holding 4 consecutive pixels, so the
// three horizontal taps of an output pixel are adjacent bytes of one dword (a v_perm / shift away)
// and meet the weights (w0, w1, w2, 0) of that channel and filter row in ONE v_dot4_i32_i8.
// All loads are buffer loads: rows above / below the image, the left and right neighbour column
// and anything past the end of the tensor use an out-of-range offset and read as zero, so padding
// needs no branches; pixels past the end of a ragged row are masked after the transpose.
typedef unsigned dw_v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void transpose4x4(const dw_v4u p, unsigned (&t)[4]) {
    const unsigned lo01 = __builtin_amdgcn_perm(p[1], p[0], 0x05010400u);
    const unsigned hi01 = __builtin_amdgcn_perm(p[1], p[0], 0x07030602u);
    const unsigned lo23 = __builtin_amdgcn_perm(p[3], p[2], 0x05010400u);
    const unsigned hi23 = __builtin_amdgcn_perm(p[3], p[2], 0x07030602u);
    t[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    t[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    t[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    t[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

// Two vertically adjacent output rows per thread: their 3 + 3 input rows overlap (4 distinct rows
// for stride 1, 5 for stride 2), so a row is loaded and transposed once for both, and the weights
// are rearranged once for 32 outputs.
// RAGGED: the input width is not a multiple of the pixels a thread loads per row (4, or 8 with
// stride 2), so the loads of the last group run into the next row and are masked.
// FUSE: what follows the requantised outputs. 0: they are stored. 1 / 2 (R = 2 only): a 2x2 stride-2
// maximum pooling over them and QADD / QFUSE_ADD_RELU of the pooled value with `other` follow in
// registers (BareMetal/Pooling.cpp, BareMetal/ElemwiseMultiType.cpp:39-48: the same float sequence
// as elemwise.hip); the thread's 2 rows x 4 pixels are two pooling windows, and what it stores is
// 2 pixels of the final tensor - the depthwise result and the pooled one never reach memory.
struct DwChain {
    const uint32_t* other;  // the second operand of the addition: [N][C/4][poh][pow] dwords
    int poh, pow;           // extent of the pooled tensor: floor(OH / 2), floor(OW / 2)
    float s_a, s_b, sdiv;   // scale of the pooled operand, of `other`, 1 / scale of the result
};

template <int S, int ACT, int R, bool RAGGED, int FUSE = 0>
__global__ void __launch_bounds__(256) dwconv44_3x3_kernel(
        ConvGeom g, RequantFast rq, const uint32_t* __restrict__ src, const uint32_t* __restrict__ flt,
        const int32_t* __restrict__ bias, uint32_t* __restrict__ dst, int total, int src_bytes,
        FastDiv d_ogn, FastDiv d_ohn, FastDiv d_c4n, RequantTable table, DwChain fz) {
    static_assert(FUSE == 0 || R == 2, "a pooling window is two output rows");
    __shared__ int tbl[REQUANT_TABLE_ENTRIES];
    if (ACT >= 0) {
        tbl[threadIdx.x] = table.t[threadIdx.x];
        __syncthreads();
    }
    constexpr int ROWS = (R - 1) * S + 3;   // input rows they need
    const int c4n = g.oc >> 2;
    const int ogn = (g.ow + 3) >> 2;  // groups of 4 output pixels per row
    const int ohn = (g.oh + R - 1) / R;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, src_bytes, 0x00020000);
    const int OOB = (int)0x80000000u;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
        // i = ((n * c4n + c4) * ohn + row group) * ogn + pixel group; divisions by multiplication
        const int r1 = fdiv(i, d_ogn), og = i - r1 * ogn;
        const int r2 = fdiv(r1, d_ohn), oh = (r1 - r2 * ohn) * R;
        const int n = fdiv(r2, d_c4n), c4 = r2 - n * c4n;
        const int plane_off = ((n * c4n + c4) * g.ih) * g.iw * 4;  // bytes
        // weights: per filter row one dword per channel = (w(fw=0), w(fw=1), w(fw=2), 0)
        unsigned wq[3][4], ws[3][4];  // ws: (0, w0, w1, w2), for the odd outputs of stride 2
#pragma unroll
        for (int fh = 0; fh < 3; ++fh) {
            const uint32_t* f = flt + (size_t)c4 * 9 + fh * 3;
            const dw_v4u fv = {f[0], f[1], f[2], 0u};
            transpose4x4(fv, wq[fh]);
#pragma unroll
            for (int c = 0; c < 4; ++c)
                ws[fh][c] = wq[fh][c] << 8;
        }
        // FUSE: the second operand of the addition for the thread's two pooled pixels, requested before
        // the input rows (a load issued where its value is needed would wait a round trip to memory)
        uint32_t other4[2] = {0u, 0u};
        if (FUSE) {
            const int py = oh >> 1;  // (oh is even: R = 2)
            if (py < fz.poh) {
                const size_t row = ((size_t)(n * c4n + c4) * fz.poh + py) * fz.pow;
#pragma unroll
                for (int k = 0; k < 2; ++k)
                    if (og * 2 + k < fz.pow)
                        other4[k] = fz.other[row + og * 2 + k];
            }
        }
        int acc[R * 16];  // [row][pixel][channel]
        {
            int b4[4] = {0, 0, 0, 0};
            if (bias) {
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    b4[c] = bias[c4 * 4 + c];
            }
#pragma unroll
            for (int e = 0; e < R * 16; ++e)
                acc[e] = b4[e & 3];
        }
        const int iw0 = og * 4 * S;   // first input pixel of the aligned loads
        const int left = g.iw - iw0;  // valid pixels from iw0 on
#pragma unroll
        for (int ir = 0; ir < ROWS; ++ir) {
            const int ih = oh * S - 1 + ir;
            const bool row_ok = (unsigned)ih < (unsigned)g.ih;
            const int row_off = plane_off + ih * g.iw * 4;
            // left neighbour pixel (iw0 - 1), pixel-major dword
            const unsigned pv = __builtin_amdgcn_raw_buffer_load_b32(
                    rs, row_ok && iw0 > 0 ? row_off + (iw0 - 1) * 4 : OOB, 0, 0);
            dw_v4u l0 = __builtin_amdgcn_raw_buffer_load_b128(rs, row_ok ? row_off + iw0 * 4 : OOB, 0, 0);
            // pixels past the end of the row belong to the next row: zero them
            if (RAGGED) {
#pragma unroll
                for (int k = 1; k < 4; ++k)
                    l0[k] = k < left ? l0[k] : 0u;
            }
            unsigned t0[4];
            transpose4x4(l0, t0);
            // the four 3-pixel windows of each channel in this input row
            unsigned win[4][4];  // [pixel][channel]
            if (S == 1) {
                const unsigned nx = __builtin_amdgcn_raw_buffer_load_b32(
                        rs, row_ok && left > 4 ? row_off + (iw0 + 4) * 4 : OOB, 0, 0);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    win[0][c] = __builtin_amdgcn_perm(t0[c], pv, 0x06050400u | c);
                    win[1][c] = t0[c];
                    win[2][c] = t0[c] >> 8;
                    win[3][c] = __builtin_amdgcn_perm(nx, t0[c], 0x0c000302u | ((4u + c) << 16));
                }
            } else {
                dw_v4u l1 = __builtin_amdgcn_raw_buffer_load_b128(
                        rs, row_ok && left > 4 ? row_off + (iw0 + 4) * 4 : OOB, 0, 0);
                if (RAGGED) {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        l1[k] = k + 4 < left ? l1[k] : 0u;
                }
                unsigned t1[4];
                transpose4x4(l1, t1);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    // outputs 1 and 3 read bytes 1-3 of t0 / t1: they meet the weights moved up a
                    // byte (SHIFTED below) instead of being shifted themselves
                    win[0][c] = __builtin_amdgcn_perm(t0[c], pv, 0x06050400u | c);
                    win[1][c] = t0[c];
                    win[2][c] = __builtin_amdgcn_alignbyte(t1[c], t0[c], 3);
                    win[3][c] = t1[c];
                }
            }
            // input row ir is filter row ir - orow * S of output row orow
#pragma unroll
            for (int orow = 0; orow < R; ++orow) {
                const int fh = ir - orow * S;
                if (fh < 0 || fh > 2)
                    continue;
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        acc[orow * 16 + j * 4 + c] = __builtin_amdgcn_sdot4(
                                (int)win[j][c], (int)(S == 2 && (j & 1) ? ws[fh][c] : wq[fh][c]),
                                acc[orow * 16 + j * 4 + c], false);
            }
        }
        if (FUSE && ACT >= 0) {
            // with the threshold table the requantisation is a non-decreasing function of the
            // accumulator, so max F(a_i) = F(max a_i): pool the int32 accumulators first and requantise
            // 8 instead of 32 values (the pooled ones land where the code below looks for window k:
            // row 0, pixel 2 * k; the other three places get the same value)
            int m[8], f[8];
#pragma unroll
            for (int k = 0; k < 2; ++k)
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    m[k * 4 + c] = max(max(acc[(2 * k) * 4 + c], acc[(2 * k + 1) * 4 + c]),
                                       max(acc[16 + (2 * k) * 4 + c], acc[16 + (2 * k + 1) * 4 + c]));
            if (rq.aff_d != 0.f) {  // (uniform; one branch around all eight)
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    f[i] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(m[i], rq.aff_c, rq.aff_d);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    f[i] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(m[i], rq.c, tbl);
            }
#pragma unroll
            for (int k = 0; k < 2; ++k)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    acc[(2 * k) * 4 + c] = acc[(2 * k + 1) * 4 + c] = f[k * 4 + c];
                    acc[16 + (2 * k) * 4 + c] = acc[16 + (2 * k + 1) * 4 + c] = f[k * 4 + c];
                }
        } else if (ACT < 0) {
#pragma unroll
            for (int e = 0; e < R * 16; ++e)
                acc[e] = requant_conv_rt(g.act, acc[e], g.s_src, g.s_flt, g.s_dst);
        } else if (rq.aff_d != 0.f) {  // (uniform)
#pragma unroll
            for (int e = 0; e < R * 16; ++e)
                acc[e] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(acc[e], rq.aff_c, rq.aff_d);
        } else {
#pragma unroll
            for (int e = 0; e < R * 16; ++e)
                acc[e] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(acc[e], rq.c, tbl);
        }
        if (FUSE) {
            const int py = oh >> 1;  // (oh is even: R = 2)
            if (py < fz.poh) {
                const size_t row = ((size_t)(n * c4n + c4) * fz.poh + py) * fz.pow;
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    const int px = og * 2 + k;
                    if (px >= fz.pow)
                        break;
                    const uint32_t b4 = other4[k];
                    int r[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const int m0 = max(acc[(2 * k) * 4 + c], acc[(2 * k + 1) * 4 + c]);
                        const int m1 = max(acc[16 + (2 * k) * 4 + c], acc[16 + (2 * k + 1) * 4 + c]);
                        const float v0 = fz.s_a * (float)max(m0, m1);
                        const float v1 = fz.s_b * (float)sbyte(b4, c);
                        const float sum = v0 + v1;
                        r[c] = fp32_to_int8((FUSE == 2 ? (sum > 0 ? sum : 0) : sum) * fz.sdiv);
                    }
                    dst[row + px] = pack4_perm(r[0], r[1], r[2], r[3]);
                }
            }
            continue;
        }
#pragma unroll
        for (int orow = 0; orow < R; ++orow) {
            if (oh + orow >= g.oh)
                break;
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                o[j] = pack4_perm(acc[orow * 16 + j * 4], acc[orow * 16 + j * 4 + 1],
                                  acc[orow * 16 + j * 4 + 2], acc[orow * 16 + j * 4 + 3]);
            uint32_t* out = dst + ((size_t)(n * c4n + c4) * g.oh + oh + orow) * g.ow + og * 4;
            if (og * 4 + 4 <= g.ow && (g.ow & 3) == 0) {
                *(uint4*)out = make_uint4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (og * 4 + j < g.ow)
                        out[j] = o[j];
            }
        }
    }
}

static bool dwconv44_3x3_ok(const ConvGeom& g, const void* src, const void* dst) {
    const long src_bytes = (long)g.n * g.ic * g.ih * g.iw;
    const long groups4 = (long)g.n * (g.oc >> 2) * g.oh * ((g.ow + 3) / 4);
    return g.fh == 3 && g.fw == 3 && g.ph == 1 && g.pw == 1 && g.dh == 1 && g.dw == 1 &&
           g.sh == g.sw && (g.sh == 1 || g.sh == 2) &&
           ((uintptr_t)src & 3) == 0 && ((uintptr_t)dst & 15) == 0 && src_bytes < (1L << 31) && groups4 < (1L << 31) &&
           (long)g.n * g.oc * g.oh * g.ow < (1L << 31);
}

// ---- depthwise 3x3 -> 2x2 stride-2 maximum pooling -> QADD / QFUSE_ADD_RELU as one kernel ------------
// (g.s_dst is the scale of the depthwise result, which the pooling keeps; `other` has the extent of the
//  pooled tensor)
bool dwconv44_chain_supported(const ConvGeom& g, const void* src, const void* other, const void* dst) {
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups > 1 && g.groups == g.ic && g.ic == g.oc && (g.ic & 3) == 0 &&
           dwconv44_3x3_ok(g, src, dst) && ((uintptr_t)other & 3) == 0 && g.oh >= 2 && g.ow >= 2;
}

bool dwconv44_mfma_chain_supported(const ConvGeom& g, const void* src, const void* dst);
TinyNNStatus dwconv44_mfma_chain_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, const void* other, void* dst,
        bool relu_after_add, float s_other, float s_out);

TinyNNStatus dwconv44_chain_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, const void* other, void* dst,
        bool relu_after_add, float s_other, float s_out) {
    // stride 1: the multiply-adds on the matrix cores, as for the layer on its own
    if (dwconv44_mfma_chain_supported(g, src, dst) && !options().no_dwmfma && !options().dw_generic)
        return dwconv44_mfma_chain_launch(g, src, flt, bias, other, dst, relu_after_add, s_other, s_out);
    constexpr int R = 2;
    const int groups4 = (int)((long)g.n * (g.oc >> 2) * ((g.oh + R - 1) / R) * ((g.ow + 3) / 4));
    if (groups4 == 0)
        return TinyNN_SUCCESS;
    const unsigned nb = (unsigned)((groups4 + 255) / 256);
    RequantFast rq3 = make_requant_fast(g.s_src, g.s_flt, g.s_dst);
    const bool tab = (g.act == MEGCC_NONLINE_IDENTITY || g.act == MEGCC_NONLINE_RELU) &&
                     requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    static const RequantTable no_table = {};
    const RequantTable& table = tab ? requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst) : no_table;
    const RequantAffine aff = requant_affine_pick(tab, g.act, g.s_src, g.s_flt, g.s_dst);
    rq3.aff_c = aff.c;
    rq3.aff_d = aff.d;
    DwChain fz;
    fz.other = (const uint32_t*)other;
    fz.poh = g.oh / 2;
    fz.pow = g.ow / 2;
    fz.s_a = g.s_dst;
    fz.s_b = s_other;
    fz.sdiv = 1.f / s_out;
    void (*k)(ConvGeom, RequantFast, const uint32_t*, const uint32_t*, const int32_t*, uint32_t*, int, int, FastDiv,
              FastDiv, FastDiv, RequantTable, DwChain);
#define MG_DWC_ACT(S_, G_, F_)                                                                             \
    (tab && g.act == MEGCC_NONLINE_IDENTITY ? dwconv44_3x3_kernel<S_, MEGCC_NONLINE_IDENTITY, 2, G_, F_>     \
     : tab && g.act == MEGCC_NONLINE_RELU   ? dwconv44_3x3_kernel<S_, MEGCC_NONLINE_RELU, 2, G_, F_>         \
                                            : dwconv44_3x3_kernel<S_, -1, 2, G_, F_>)
#define MG_DWC_PICK(S_, G_) (relu_after_add ? MG_DWC_ACT(S_, G_, 2) : MG_DWC_ACT(S_, G_, 1))
    const bool ragged = (g.iw % (4 * g.sh)) != 0;
    if (g.sh == 1)
        k = ragged ? MG_DWC_PICK(1, true) : MG_DWC_PICK(1, false);
    else
        k = ragged ? MG_DWC_PICK(2, true) : MG_DWC_PICK(2, false);
#undef MG_DWC_PICK
#undef MG_DWC_ACT
    hipLaunchKernelGGL(k, dim3(nb), dim3(256), 0, stream(), g, rq3, (const uint32_t*)src, (const uint32_t*)flt,
                       (const int32_t*)bias, (uint32_t*)dst, groups4, (int)((long)g.n * g.ic * g.ih * g.iw),
                       make_fastdiv((g.ow + 3) / 4), make_fastdiv((g.oh + R - 1) / R), make_fastdiv(g.oc >> 2), table,
                       fz);
    return check_launch("dwconv44_chain");
}

bool dwconv44_supported(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups > 1 && g.groups == g.ic && g.ic == g.oc &&
           (g.ic & 3) == 0;
}

bool dwconv44_mfma_supported(const ConvGeom& g, const void* src, const void* dst);
TinyNNStatus dwconv44_mfma_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst);

// the matrix-core kernel (dwconv_mfma.hip) for stride 1, where the vector ALU is the limit
static bool use_mfma(const ConvGeom& g, const void* src, const void* dst) {
    return dwconv44_mfma_supported(g, src, dst) && !options().no_dwmfma && !options().dw_generic;
}

// which kernel dwconv44_launch picks: (pixels per thread and row) << 4 | rows per thread
static int dwconv44_shape(const ConvGeom& g, const void* src, const void* dst) {
    if (!dwconv44_3x3_ok(g, src, dst) || options().dw_generic)
        return 1 << 4 | 1;
    return 4 << 4 | (g.sh == 1 && g.oh >= 28 ? 2 : 1);
}

// records the kernel dwconv44_launch runs for this layer
void dwconv44_note(const ConvGeom& g, const void* src, const void* dst) {
    if (use_mfma(g, src, dst))
        note_kernel("dwconv44_mfma");
    else  // pixels per thread and row (4: the 3x3 kernels, 1: the generic one), rows per thread
        note_kernel("dwconv44", dwconv44_shape(g, src, dst) >> 4, dwconv44_shape(g, src, dst) & 15);
}

TinyNNStatus dwconv44_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    size_t total = (size_t)g.n * (g.oc >> 2) * g.oh * g.ow;
    if (total == 0)
        return TinyNN_SUCCESS;
    if (use_mfma(g, src, dst))
        return dwconv44_mfma_launch(g, src, flt, bias, dst);
    const int shape = dwconv44_shape(g, src, dst);
    if (shape >> 4 == 4) {
        // one thread per R output rows x 4 output pixels x 4 channels
        // (two rows share input rows and the weight set-up: measured faster for stride 1 on
        // large planes only)
        const int R = shape & 15;
        const int groups4 = (int)((long)g.n * (g.oc >> 2) * ((g.oh + R - 1) / R) * ((g.ow + 3) / 4));
        unsigned nb = (unsigned)((groups4 + 255) / 256);
        RequantFast rq3 = make_requant_fast(g.s_src, g.s_flt, g.s_dst);
        void (*k3)(ConvGeom, RequantFast, const uint32_t*, const uint32_t*, const int32_t*, uint32_t*, int, int,
                   FastDiv, FastDiv, FastDiv, RequantTable, DwChain);
        // exact thresholds for the monotone activations; anything else (and extreme scales)
        // evaluates the literal sequence per output
        const bool tab = requant_table_act(g.act) && requant_table_ok(g.s_src, g.s_flt, g.s_dst);
        static const RequantTable no_table = {};
        const RequantTable& table = tab ? requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst) : no_table;
        const RequantAffine aff = requant_affine_pick(tab, g.act, g.s_src, g.s_flt, g.s_dst);
        rq3.aff_c = aff.c;
        rq3.aff_d = aff.d;
#define MG_DW_PICK(S_, R_, G_)                                                                      \
    (tab && g.act == MEGCC_NONLINE_IDENTITY ? dwconv44_3x3_kernel<S_, MEGCC_NONLINE_IDENTITY, R_, G_> \
     : tab && g.act == MEGCC_NONLINE_RELU   ? dwconv44_3x3_kernel<S_, MEGCC_NONLINE_RELU, R_, G_>     \
     : tab && g.act == MEGCC_NONLINE_H_SWISH ? dwconv44_3x3_kernel<S_, MEGCC_NONLINE_H_SWISH, R_, G_> \
                                            : dwconv44_3x3_kernel<S_, -1, R_, G_>)
        const bool ragged = (g.iw % (4 * g.sh)) != 0;
        if (g.sh == 1 && R == 2)
            k3 = ragged ? MG_DW_PICK(1, 2, true) : MG_DW_PICK(1, 2, false);
        else if (g.sh == 1)
            k3 = ragged ? MG_DW_PICK(1, 1, true) : MG_DW_PICK(1, 1, false);
        else
            k3 = ragged ? MG_DW_PICK(2, 1, true) : MG_DW_PICK(2, 1, false);
#undef MG_DW_PICK
        hipLaunchKernelGGL(k3, dim3(nb), dim3(256), 0, stream(), g, rq3, (const uint32_t*)src,
                           (const uint32_t*)flt, (const int32_t*)bias, (uint32_t*)dst, groups4,
                           (int)((long)g.n * g.ic * g.ih * g.iw), make_fastdiv((g.ow + 3) / 4),
                           make_fastdiv((g.oh + R - 1) / R), make_fastdiv(g.oc >> 2), table, DwChain{});
        return check_launch("dwconv44_3x3");
    }
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
