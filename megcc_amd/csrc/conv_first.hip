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
#include "fastdiv.h"

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

// The same layer with 32 or 64 output channels on the matrix cores. K = 27 is short, but what the
// v_dot4 kernel above spends per output - 9 dot products next to the 10 instructions of the exact
// requantisation - is what an MFMA saves: here the reduction index is k = 4 * (ic * 3 + fh) + fw with a
// zero weight at fw = 3, so a lane's 16 K-bytes of the B operand are the 4 bytes at input columns
// 2 * ox - 1 .. 2 * ox + 2 of four (channel, filter row) pairs = four dword loads from byte addresses,
// no byte is moved by hand; 9 pairs x 4 bytes = 36 > 32, so a second MFMA takes the ninth pair.
// A lane's loads stay inside their image row: the first column loads one byte to the right and shifts
// (its byte 0 is the left padding), the last column one byte to the left.
typedef int cfm_v4i __attribute__((ext_vector_type(4)));
typedef int cfm_v16i __attribute__((ext_vector_type(16)));

struct ConvFirstMfmaParams {
    const int8_t* src;
    const int8_t* flt;
    const int32_t* bias;
    uint32_t* dst;
    int src_bytes;
    int N, IH, IW, OH, OW, OHW, P, tiles, OC;
    int act;
    float s_src, s_flt, s_dst, c;
    float aff_c, aff_d;  // requantisation by one fused multiply-add (epilogue.h); aff_d == 0: table
    FastDiv dOW, dOHW;
    RequantTable table;
};

template <int MT, int ACT>
__global__ void __launch_bounds__(256) conv_first_mfma_kernel(ConvFirstMfmaParams q) {
    __shared__ int tbl[REQUANT_TABLE_ENTRIES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int col = lane & 31, kg = lane >> 5;
    if (ACT >= 0) {
        tbl[tid] = q.table.t[tid];
        __syncthreads();
    }
    // ---- filter rows of this lane's output channels: A1 = pairs 4 * kg .. 4 * kg + 3, A2 = pair 8
    auto weight_dword = [&](int oc, int pair) {
        const int ic = pair / 3, fh = pair - ic * 3;
        uint32_t w = 0;
#pragma unroll
        for (int fw = 0; fw < 3; ++fw)
            w |= (uint32_t)(uint8_t)q.flt[((((size_t)(oc >> 2) * 3 + fh) * 3 + fw) * 3 + ic) * 4 + (oc & 3)] << (8 * fw);
        return (int)w;
    };
    cfm_v4i A1[MT], A2[MT];
    int biasv[MT][4][4];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
        const int oc = mi * 32 + col;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            A1[mi][j] = weight_dword(oc, 4 * kg + j);
        A2[mi] = cfm_v4i{kg == 0 ? weight_dword(oc, 8) : 0, 0, 0, 0};
        // accumulator register e is channel 8 * (e / 4) + 4 * kg + e % 4 of the row tile
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4)
#pragma unroll
            for (int k = 0; k < 4; ++k)
                biasv[mi][e4][k] = q.bias ? q.bias[mi * 32 + e4 * 8 + kg * 4 + k] : 0;
    }
    // byte offset of this lane's pairs inside an image, relative to (row 2 * oy - 1, column 2 * ox - 1)
    int pair_off[4];
    bool pair_top[4];  // the pair's filter row is 0: above the image when oy == 0
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int pair = 4 * kg + j, ic = pair / 3, fh = pair - ic * 3;
        pair_off[j] = (ic * q.IH + fh) * q.IW;
        pair_top[j] = fh == 0;
    }
    const int pair8_off = (2 * q.IH + 2) * q.IW;  // channel 2, filter row 2
    const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void*)q.src, 0, q.src_bytes, 0x00020000);
    const int OOB = (int)0x80000000u;
    const int oc4n = q.OC >> 2;

    const int gw = blockIdx.x * 4 + (tid >> 6), nw = gridDim.x * 4;
    // operands of a tile (requested one tile ahead: the loads fly during the epilogue before them)
    struct Tile {
        cfm_v4i B1, B2;
        int obase;
        bool ok, first, last;
    };
    auto request = [&](int t) __attribute__((always_inline)) {
        Tile r;
        const int p = t * 32 + col;
        r.ok = t < q.tiles && p < q.P;
        const int n = fdiv(p, q.dOHW), rem = p - n * q.OHW;
        const int oy = fdiv(rem, q.dOW), ox = rem - oy * q.OW;
        // first column: load from column 0 and shift one byte up (byte 0 = padding);
        // last column: load from column 2 * ox - 2 and shift one byte down (its byte 3 has weight 0)
        r.first = ox == 0;
        r.last = 2 * ox + 2 >= q.IW;
        const int base = n * 3 * q.IH * q.IW + (2 * oy - 1) * q.IW + 2 * ox - 1 + (r.first ? 1 : r.last ? -1 : 0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool row_ok = r.ok && !(pair_top[j] && oy == 0);
            r.B1[j] = (int)__builtin_amdgcn_raw_buffer_load_b32(rs, row_ok ? base + pair_off[j] : OOB, 0, 0);
        }
        r.B2 = cfm_v4i{(int)__builtin_amdgcn_raw_buffer_load_b32(rs, r.ok && kg == 0 ? base + pair8_off : OOB, 0, 0), 0, 0, 0};
        r.obase = n * oc4n * q.OHW + rem;
        return r;
    };
    Tile next = request(gw);
    for (int t = gw; t < q.tiles; t += nw) {
        const Tile cur = next;
        auto fix = [&](int v) { return (int)(cur.first ? (unsigned)v << 8 : cur.last ? (unsigned)v >> 8 : (unsigned)v); };
        cfm_v4i B1, B2 = {fix(cur.B2[0]), 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            B1[j] = fix(cur.B1[j]);
        cfm_v16i acc[MT];
#pragma unroll
        for (int mi = 0; mi < MT; ++mi) {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[mi][e] = biasv[mi][e >> 2][e & 3];
            acc[mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(A1[mi], B1, acc[mi], 0, 0, 0);
            acc[mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(A2[mi], B2, acc[mi], 0, 0, 0);
        }
        next = request(t + nw);
#pragma unroll
        for (int mi = 0; mi < MT; ++mi) {
            int r[16];
            if (ACT >= 0 && q.aff_d != 0.f) {  // (uniform)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    r[e] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(acc[mi][e], q.aff_c, q.aff_d);
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    if (ACT < 0)
                        r[e] = requant_conv_rt(q.act, acc[mi][e], q.s_src, q.s_flt, q.s_dst);
                    else
                        r[e] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(acc[mi][e], q.c, tbl);
                }
            }
            if (cur.ok) {
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4)
                    q.dst[cur.obase + (mi * 8 + e4 * 2 + kg) * q.OHW] =
                            pack4_perm(r[e4 * 4], r[e4 * 4 + 1], r[e4 * 4 + 2], r[e4 * 4 + 3]);
            }
        }
    }
}

static bool conv_first_mfma_ok(const ConvGeom& g) {
    return (g.oc == 32 || g.oc == 64) && g.iw >= 4 && (long)g.n * 3 * g.ih * g.iw < (1L << 31) &&
           (long)g.n * g.oc * g.oh * g.ow < (1L << 31) && !options().no_firstmfma;
}

static TinyNNStatus conv_first_mfma_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    ConvFirstMfmaParams q = {};
    q.src = (const int8_t*)src;
    q.flt = (const int8_t*)flt;
    q.bias = (const int32_t*)bias;
    q.dst = (uint32_t*)dst;
    q.src_bytes = (int)((long)g.n * 3 * g.ih * g.iw);
    q.N = g.n; q.IH = g.ih; q.IW = g.iw; q.OH = g.oh; q.OW = g.ow;
    q.OHW = g.oh * g.ow;
    q.P = g.n * q.OHW;
    q.tiles = (q.P + 31) / 32;
    q.OC = g.oc;
    q.act = g.act;
    q.s_src = g.s_src; q.s_flt = g.s_flt; q.s_dst = g.s_dst;
    q.c = make_requant_fast(g.s_src, g.s_flt, g.s_dst).c;
    q.dOW = make_fastdiv(q.OW);
    q.dOHW = make_fastdiv(q.OHW);
    const bool tab = requant_table_act(g.act) && requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    if (tab)
        q.table = requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst);
    const int act = tab ? g.act : -1;
    const RequantAffine aff = requant_affine_pick(tab, g.act, g.s_src, g.s_flt, g.s_dst);
    q.aff_c = aff.c;
    q.aff_d = aff.d;
    const void* kern;
#define MG_CFM(MT_)                                                                                     \
    (act == MEGCC_NONLINE_IDENTITY ? (const void*)conv_first_mfma_kernel<MT_, MEGCC_NONLINE_IDENTITY>     \
     : act == MEGCC_NONLINE_RELU   ? (const void*)conv_first_mfma_kernel<MT_, MEGCC_NONLINE_RELU>         \
     : act == MEGCC_NONLINE_H_SWISH ? (const void*)conv_first_mfma_kernel<MT_, MEGCC_NONLINE_H_SWISH>     \
                                   : (const void*)conv_first_mfma_kernel<MT_, -1>)
    kern = g.oc == 32 ? MG_CFM(1) : MG_CFM(2);
#undef MG_CFM
    long blocks = (q.tiles + 3) / 4;
    const long cap = (long)num_cus() * 8;
    if (blocks > cap)
        blocks = cap;
    void* args[] = {&q};
    hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(256), args, 0, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_first_mfma: %s", hipGetErrorString(e));
    return check_launch("conv_first_mfma");
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
    if (conv_first_mfma_ok(g)) {
        note_kernel("conv_first_mfma", g.oc / 32);
        return conv_first_mfma_launch(g, src, flt, bias, dst);
    }
    long blocks = (pairs + CF_THREADS - 1) / CF_THREADS;
    if (blocks > 256 * 16)
        blocks = 256 * 16;
    const RequantFast rq = make_requant_fast(g.s_src, g.s_flt, g.s_dst);
    // exact thresholds for the monotone activations; anything else (and extreme scales)
    // evaluates the literal sequence per output
    const bool tab = requant_table_act(g.act) && requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    static const RequantTable no_table = {};
    const RequantTable& table = tab ? requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst) : no_table;
    auto kern = tab && g.act == MEGCC_NONLINE_IDENTITY ? conv_first_q8_kernel<MEGCC_NONLINE_IDENTITY>
              : tab && g.act == MEGCC_NONLINE_RELU     ? conv_first_q8_kernel<MEGCC_NONLINE_RELU>
              : tab && g.act == MEGCC_NONLINE_H_SWISH  ? conv_first_q8_kernel<MEGCC_NONLINE_H_SWISH>
                                                       : conv_first_q8_kernel<-1>;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(CF_THREADS), 0, stream(), g, rq,
                       (const int8_t*)src, (const int8_t*)flt, (const int32_t*)bias, (uint32_t*)dst,
                       (int)pairs, table);
    return check_launch("conv_first_q8");
}

}  // namespace mg
