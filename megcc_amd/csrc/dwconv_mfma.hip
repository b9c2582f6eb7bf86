// qsi8 depthwise 3x3 (pad 1, stride 1), 5x5 (pad 2) and 7x7 (pad 3, both stride 1 or 2) in NCHW44 on
// the matrix cores. The text below describes the 3x3 case; an F x F filter with pad F / 2 has F
// filter rows, filter columns 0 .. F - 1 in the band, and still fits the same S + 1 aligned K steps
// (a group of 8 output pixels from x0 on reads input pixels S*x0 - F/2 .. S*x0 + 7*S + F/2, all of
// them inside S*x0 - 4 .. S*x0 + 8*S + 3 while F/2 <= 3).
//
// A depthwise layer moves two bytes per output and has to requantise every output exactly, which
// costs 7 vector instructions and a table look-up (epilogue.h). Done with v_dot4 the multiply-adds
// and the byte shuffling in front of them cost another 10 vector instructions per output, and the
// layer is bound by the vector ALU at a third of the memory rate. Here the multiply-adds go to the
// MFMA unit, which is otherwise idle, as a product with a banded matrix:
//
//   for one group of 4 channels (one NCHW44 plane set) and one filter row dy,
//     D[(px, ch), col] += A_dy[(px, ch), (ipx, ich)] * B_dy[(ipx, ich), col]
//   * a column is one group of 8 consecutive output pixels (image n, row y, pixels 8b .. 8b + 7)
//     of the plane set; the 32 columns of a tile are 32 consecutive groups in (n, y, b) order,
//     i.e. they walk along the rows;
//   * K = 32 bytes = 8 consecutive input pixels x 4 channels exactly as they lie in memory, so the
//     B operand of lane (col, K-half) is ONE aligned 16-byte load from input row y*S - 1 + dy, and
//     the 64 lanes of a K step read one contiguous kilobyte (stride 1: column c + 1 continues
//     where column c ends): no transposes, no shuffles, fully coalesced; rows above / below the
//     image and pixel groups left / right of it are loaded with an out-of-range buffer offset and
//     read as zero, which is the padding;
//   * M = 32 = 8 output pixels x 4 channels; A_dy holds weight w[dy][fw][ch] where ich == ch and
//     fw = ipx - (S * px - 1) is the filter column that connects input pixel ipx with output
//     pixel px (0 <= fw <= 2), zero elsewhere. It only depends on the DISTANCE between the K
//     step's first pixel and the tile's first pixel, so S + 1 matrices per filter row serve every
//     tile of the layer; a wave builds them once from the 36 weight bytes of its plane set and
//     keeps them in registers.
//   A group of 8 output pixels from x0 on needs input pixels S*x0 - 1 .. S*x0 + 7*S + 1: S + 1
//   aligned K steps of 8 pixels starting at S*x0 - 4, i.e. 3 * (S + 1) MFMAs per tile of
//   32 groups x 8 pixels x 4 channels. The accumulators start from the bias through the MFMA's C
//   operand.
//
// The 1/32 utilisation of the band is irrelevant: 3 * (S + 1) MFMAs per 1024 outputs is 0.2
// cycles per output and SIMD, against 28 cycles for the exact epilogue.
//
// Accumulator register e of lane (col, h) is output pixel 2 * (e / 4) + h, channel e % 4: four
// consecutive registers pack into the NCHW44 dword of one pixel, and two v_permlane32_swap hand the
// odd pixels of the lower half wave to the upper one and back, after which every lane owns 4
// consecutive pixels = one 16-byte store, the 64 stores of a wave again one contiguous kilobyte.
//
// Same arithmetic as the reference's loop (BareMetal/ConvKernel.cpp:305-344,374-380): int32
// accumulators over the in-bounds taps plus the bias, then the exact requantisation (epilogue.h).
#include "common.h"
#include "conv_geom.h"
#include "conv_mfma_i8.h"
#include "epilogue.h"

namespace mg {

struct DwMfmaParams {
    const uint32_t* src;
    const uint32_t* flt;   // [C/4][F][F] dwords of 4 channel bytes
    const int32_t* bias;   // or nullptr
    uint32_t* dst;
    int src_bytes;
    int c4n, ih, iw, oh, ow;
    int dst_bytes;
    int ohp;               // ceil(OH / R): row groups per image
    int cols;              // N * ohp * xblocks: (row group, 8 output pixels) pairs per plane set
    int xblocks;           // ceil(OW / 8)
    int tiles;             // per plane set: ceil(cols / 32)
    int act;
    float s_src, s_flt, s_dst, c;
    float aff_c, aff_d;   // requantisation by one fused multiply-add (epilogue.h); aff_d == 0: table
    FastDiv d_ohp, d_xb;  // division by ohp, by xblocks
    // FUSE: the second operand of the addition that follows the pooling ([N][C/4][poh][pow] dwords), the
    // extent of the pooled tensor, the scales of the pooled operand and of `other`, 1 / the result's
    const uint32_t* other;
    int poh, pow;
    float s_a, s_b, sdiv;
    RequantTable table;
};

struct DwMfmaChain {
    const void* other;
    bool relu_after_add;
    float s_other, s_out;
};

typedef unsigned dwm_v2u __attribute__((ext_vector_type(2)));
typedef unsigned dw_v4u __attribute__((ext_vector_type(4)));
// R: output rows per lane and tile (2 share input rows and index arithmetic but need 200 registers:
// measured 15.3 us against 14.9 us with 1 on N=64 C=32 112x112; the layer on its own uses 1).
// FUSE (3x3 stride 1 with R = 2 only): 1 / 2 = a 2x2 stride-2 maximum pooling of the requantised
// outputs and QADD / QFUSE_ADD_RELU of the pooled value with q.other follow in registers (the same
// float sequence as elemwise.hip, BareMetal/ElemwiseMultiType.cpp:39-48). A lane's 2 rows x 4 pixels
// are the halves of four pooling windows whose other halves the lane 32 further on holds: after the
// vertical maximum the same two v_permlane32_swap that prepare the 16-byte stores of the plain
// kernel hand each lane both halves of two windows; it stores 2 pixels of the final tensor.

// S: stride (only 1 is instantiated: with stride 2 the layer reads four bytes per byte written and
// the v_dot4 kernel of dwconv.hip already runs at the rate of a copy - measured 7.8 us against
// 9.8 us for this one on N=64 C=32 112x112). RAGGED: IW is not a multiple of 4, so the last 16-byte load of a row runs into the
// next row and is masked. ACT: IDENTITY / RELU / H_SWISH use the threshold table, -1 evaluates the literal
// sequence with the run-time activation. F: filter rows = filter columns (3, 5 or 7; pad F / 2).
template <int S, bool RAGGED, int ACT, int F = 3, int R = 1, int FUSE = 0>
__global__ void __launch_bounds__(256) dwconv44_mfma_kernel(DwMfmaParams q) {
    static_assert(FUSE == 0 || (R == 2 && S == 1 && F == 3), "a pooling window is two output rows");
    static_assert(F == 3 || F == 5 || F == 7, "the band must fit S + 1 K steps: pad <= 3");
    constexpr int PAD = F / 2;
    constexpr int NS = S + 1;            // K steps a group of 8 output pixels reads
    constexpr int IR = (R - 1) * S + F;  // input rows they read
    __shared__ int tbl[REQUANT_TABLE_ENTRIES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int col_l = lane & 31, kg = lane >> 5;
    // Workgroups are handed to the 8 XCDs in turn and every XCD has an L2 of its own: workgroup b
    // takes the place b % 8 * (blocks / 8) + b / 8 in tile order, so that an XCD walks a contiguous
    // eighth of the tiles and the input rows that neighbouring tiles share are fetched into one
    // L2 instead of two or three.
    const int nb = gridDim.x;
    const int lb = (nb & 7) == 0 ? (blockIdx.x & 7) * (nb >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    // wave -> (plane set, a run of consecutive tiles): the grid holds a multiple of c4n waves. A
    // tile is 256 output pixels along the rows - 2.3 rows of a 112-pixel map - and reads one row
    // more above and below, which the tile after it reads again: walking its run tile by tile, a
    // wave finds those rows in its XCD's L2 two microseconds after it fetched them. (Tiles dealt
    // round-robin to the waves of a plane set left the re-read to another wave at another time:
    // on N=64 C=512 112x112, whose 411 MB no cache holds, 1.82 times the input came from HBM.)
    const int gw = lb * 4 + __builtin_amdgcn_readfirstlane(tid >> 6);  // (scalar: the plane set's weights and bias come through the scalar cache)
    const int nw = gridDim.x * 4;
    const int c4 = gw % q.c4n;
    // (runs of floor(tiles / waves) tiles, the first tiles % waves of them one longer: with runs of
    //  the rounded-up length the last waves of a plane set had nothing to do - an eighth of them on
    //  N=64 C=32 112x112, which cost that layer 5 % and its fused chain 14 %)
    const int wps = nw / q.c4n;                     // waves per plane set
    const int wi = gw / q.c4n;                      // this wave's place among them
    const int run_q = q.tiles / wps, run_r = q.tiles - run_q * wps;
    const int t_begin = wi * run_q + min(wi, run_r);
    const int t_end = t_begin + run_q + (wi < run_r ? 1 : 0);

    const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void*)q.src, 0, q.src_bytes, 0x00020000);
    const int OOB = (int)0x80000000u;

    const __amdgpu_buffer_rsrc_t rd =
            __builtin_amdgcn_make_buffer_rsrc((void*)q.dst, 0, q.dst_bytes, 0x00020000);
    // where a lane's results go: byte offset of its 4 pixels in output row y, pixels left in the
    // row (<= 0: nothing to store), rows left in the image
    struct Where {
        int off, left, rows;
        // FUSE: dword index of the lane's first pooled pixel in `other` / the result, how many of its 2
        // pixels exist, and the second operand's 2 dwords (requested with the tile's rows: a load
        // issued where its value is needed would put a round trip to memory behind every tile)
        int pidx, pleft;
        uint32_t b4[2];
    };
    // requests the B operands of a tile: NS aligned 16-byte loads for each of the IR input rows
    auto request = [&](int tile, v4i (&B)[IR][NS]) __attribute__((always_inline)) -> Where {
        const int col = tile * 32 + col_l;
        const bool col_ok = col < q.cols && tile < q.tiles;
        const int rg = fdiv(col, q.d_xb), x0 = (col - rg * q.xblocks) * 8;
        const int n = fdiv(rg, q.d_ohp), y = (rg - n * q.ohp) * R;
        const int pset = n * q.c4n + c4;
        const int base = pset * q.ih * q.iw;   // first pixel of the input plane set
        const int ix0 = S * x0 - 4 + 4 * kg;   // this lane's first input pixel of K step 0
#pragma unroll
        for (int ir = 0; ir < IR; ++ir) {
            const int iy = y * S - PAD + ir;
            const bool row_ok = col_ok && (unsigned)iy < (unsigned)q.ih;
            const int row_off = base + __mul24(iy, q.iw);
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const int ix = ix0 + 8 * s;
                const bool ok = row_ok && (unsigned)ix < (unsigned)q.iw;
                B[ir][s] = __builtin_bit_cast(
                        v4i, __builtin_amdgcn_raw_buffer_load_b128(rs, ok ? (row_off + ix) * 4 : OOB, 0, 0));
                if (RAGGED) {
#pragma unroll
                    for (int j = 1; j < 4; ++j)
                        B[ir][s][j] = ix + j < q.iw ? B[ir][s][j] : 0;
                }
            }
        }
        Where w;
        const int xo = x0 + 4 * kg;  // after the exchange this lane stores pixels xo .. xo + 3
        w.off = ((pset * q.oh + y) * q.ow + xo) * 4;
        w.left = col_ok ? q.ow - xo : 0;
        w.rows = q.oh - y;
        if constexpr (FUSE != 0) {
            const int py = rg - n * q.ohp;  // (R = 2: row group = pooled row)
            const int px0 = (x0 >> 1) + 2 * kg;
            w.pidx = (pset * q.poh + py) * q.pow + px0;
            w.pleft = col_ok && py < q.poh ? q.pow - px0 : 0;
#pragma unroll
            for (int k = 0; k < 2; ++k)
                w.b4[k] = w.pleft > k ? q.other[w.pidx + k] : 0u;
        }
        return w;
    };

    // Order of the set-up: threshold table to LDS (one barrier), then the first tile's rows are
    // requested, then the banded matrices are built while those loads fly. (Requesting the rows
    // before the table copy made the barrier wait for them: 5 - 8 % slower on 14 x 14 and 112 x 112
    // maps alike.)
    v4i B[IR][NS];
    int tile = t_begin;
    if (ACT >= 0) {
        tbl[tid] = q.table.t[tid];
        __syncthreads();
    }
    Where next = request(tile < t_end ? tile : q.tiles, B);
    // ---- the banded weight matrices of this plane set -------------------------------------------
    // row m = lane & 31 = (output pixel m / 4, channel m % 4); the lane's 16 K bytes are input
    // pixels 4 * kg + j (j = 0..3) of the K step, 4 channel bytes each. K step s starts 4 pixels
    // left of S * x0, so input pixel (s, j) meets output pixel px through filter column
    // fw = 8 * s + 4 * kg + j - 4 - S * px + PAD.
    v4i A[F][NS];
    {
        const int px = col_l >> 2, ch = col_l & 3;
        const unsigned keep = 0xffu << (8 * ch);
        const uint32_t* w = q.flt + (size_t)c4 * (F * F);
#pragma unroll
        for (int dy = 0; dy < F; ++dy) {
            unsigned wr[F];
#pragma unroll
            for (int k = 0; k < F; ++k)
                wr[k] = w[dy * F + k] & keep;
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int fw = 8 * s + 4 * kg + j - 4 + PAD - S * px;
                    unsigned v = 0;
#pragma unroll
                    for (int k = 0; k < F; ++k)
                        v = fw == k ? wr[k] : v;
                    A[dy][s][j] = (int)v;
                }
        }
    }
    v16i biasv;
    {
        int b4[4] = {0, 0, 0, 0};
        if (q.bias) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                b4[c] = q.bias[c4 * 4 + c];
        }
#pragma unroll
        for (int e = 0; e < 16; ++e)
            biasv[e] = b4[e & 3];
    }
    for (; tile < t_end; ++tile) {
        const Where cur = next;
        v16i acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            acc[r] = biasv;
#pragma unroll
            for (int dy = 0; dy < F; ++dy)
#pragma unroll
                for (int s = 0; s < NS; ++s)
                    acc[r] = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[dy][s], B[r * S + dy][s], acc[r], 0, 0, 0);
        }
        // the operands are consumed: the next tile's loads fly while this one is requantised
        // (past the last tile every offset is out of range and nothing is fetched)
        next = request(tile + 1 < t_end ? tile + 1 : q.tiles, B);
        if constexpr (FUSE != 0) {
            // ---- pool, requantise, add, store ----------------------------------------------------
            // With the threshold table the requantisation F is a non-decreasing function of the
            // accumulator (epilogue.h), so max F(a_i) = F(max a_i): the maximum is taken over the
            // int32 accumulators and 8 instead of 32 values per lane are requantised. The literal
            // sequence (SIGMOID, extreme scales) requantises first.
            int pooled[2][4];  // [window of this lane][channel], requantised
            if (ACT >= 0) {
                int v[16];  // vertical maximum: pixel 2 * (e / 4) + kg, channel e % 4
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    v[e] = max(acc[0][e], acc[1][e]);
                // lower half wave: both halves of windows 0 and 1; upper: of windows 2 and 3
                int w0[4], w1[4];  // the windows' maxima over the accumulators
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const dwm_v2u s02 = __builtin_amdgcn_permlane32_swap((unsigned)v[c], (unsigned)v[8 + c], false, false);
                    const dwm_v2u s13 = __builtin_amdgcn_permlane32_swap((unsigned)v[4 + c], (unsigned)v[12 + c], false, false);
                    w0[c] = max((int)s02[0], (int)s02[1]);
                    w1[c] = max((int)s13[0], (int)s13[1]);
                }
                // (one uniform branch around all eight, so that the look-ups of the table form stay in
                //  flight together)
                if (q.aff_d != 0.f) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        pooled[0][c] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(w0[c], q.aff_c, q.aff_d);
                        pooled[1][c] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(w1[c], q.aff_c, q.aff_d);
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        pooled[0][c] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(w0[c], q.c, tbl);
                        pooled[1][c] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(w1[c], q.c, tbl);
                    }
                }
            } else {
                unsigned d[4];  // vertical maximum of pixel 2 * j + kg, 4 requantised channel bytes
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    int o[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        o[c] = max(requant_conv_rt(q.act, acc[0][4 * j + c], q.s_src, q.s_flt, q.s_dst),
                                   requant_conv_rt(q.act, acc[1][4 * j + c], q.s_src, q.s_flt, q.s_dst));
                    d[j] = pack4_perm(o[0], o[1], o[2], o[3]);
                }
                const dwm_v2u s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
                const dwm_v2u s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    pooled[0][c] = max(sbyte(s02[0], c), sbyte(s02[1], c));
                    pooled[1][c] = max(sbyte(s13[0], c), sbyte(s13[1], c));
                }
            }
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const bool ok = cur.pleft > k;
                const uint32_t b4 = cur.b4[k];
                int r4[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float v0 = q.s_a * (float)pooled[k][c];
                    const float v1 = q.s_b * (float)sbyte(b4, c);
                    const float sum = v0 + v1;
                    r4[c] = fp32_to_int8((FUSE == 2 ? (sum > 0 ? sum : 0) : sum) * q.sdiv);
                }
                if (ok)
                    q.dst[cur.pidx + k] = pack4_perm(r4[0], r4[1], r4[2], r4[3]);
            }
            continue;
        }
        // ---- requantise, pack, exchange, store ---------------------------------------------------
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int o[16];
            if (ACT < 0) {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    o[e] = requant_conv_rt(q.act, acc[r][e], q.s_src, q.s_flt, q.s_dst);
            } else if (q.aff_d != 0.f) {  // (uniform)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    o[e] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(acc[r][e], q.aff_c, q.aff_d);
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    o[e] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(acc[r][e], q.c, tbl);
            }
            unsigned d[4];  // pixel 2 * j + kg
#pragma unroll
            for (int j = 0; j < 4; ++j)
                d[j] = pack4_perm(o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]);
            // lower half wave: pixels 0 2 4 6, upper: 1 3 5 7  ->  lower 0 1 2 3, upper 4 5 6 7
            const dwm_v2u s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
            const dwm_v2u s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
            const dw_v4u px4 = {s02[0], s02[1], s13[0], s13[1]};
            const int left = r < cur.rows ? cur.left : 0;
            const int off = cur.off + r * q.ow * 4;
            if ((q.ow & 3) == 0) {
                __builtin_amdgcn_raw_buffer_store_b128(px4, rd, left >= 4 ? off : OOB, 0, 0);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    __builtin_amdgcn_raw_buffer_store_b32(px4[j], rd, left > j ? off + 4 * j : OOB, 0, 0);
            }
        }
    }
}

bool dwconv44_mfma_supported(const ConvGeom& g, const void* src, const void* dst) {
    const long src_bytes = (long)g.n * g.ic * g.ih * g.iw;
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups > 1 && g.groups == g.ic && g.ic == g.oc &&
           (g.ic & 3) == 0 && g.fh == g.fw && (g.fh == 3 || g.fh == 5 || g.fh == 7) && g.ph == g.fh / 2 &&
           g.pw == g.fw / 2 && g.dh == 1 && g.dw == 1 && g.sh == g.sw &&
           (g.sh == 1 || (g.sh == 2 && g.fh > 3)) && ((uintptr_t)src & 15) == 0 &&
           ((uintptr_t)dst & 15) == 0 && src_bytes < (1L << 31) &&
           (long)g.n * g.oc * g.oh * g.ow < (1L << 31) && (long)g.n * g.oh * ((g.ow + 7) / 8) < (1L << 30) && (long)g.ih * g.iw < (1L << 24);
}

// chain: the pooling + addition that follow (FUSE), or NULL
static TinyNNStatus dwconv44_mfma_run(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst, const DwMfmaChain* chain) {
    const int rows = chain ? 2 : 1;
    DwMfmaParams q = {};
    if (chain) {
        q.other = (const uint32_t*)chain->other;
        q.poh = g.oh / 2;
        q.pow = g.ow / 2;
        q.s_a = g.s_dst;
        q.s_b = chain->s_other;
        q.sdiv = 1.f / chain->s_out;
    }
    q.src = (const uint32_t*)src;
    q.flt = (const uint32_t*)flt;
    q.bias = (const int32_t*)bias;
    q.dst = (uint32_t*)dst;
    q.src_bytes = (int)((long)g.n * g.ic * g.ih * g.iw);
    q.c4n = g.ic >> 2;
    q.ih = g.ih;
    q.iw = g.iw;
    q.oh = g.oh;
    q.ow = g.ow;
    q.dst_bytes = chain ? (int)((long)g.n * g.oc * (g.oh / 2) * (g.ow / 2)) : (int)((long)g.n * g.oc * g.oh * g.ow);
    q.xblocks = (g.ow + 7) / 8;
    q.ohp = (g.oh + rows - 1) / rows;
    q.cols = g.n * q.ohp * q.xblocks;
    q.tiles = (q.cols + 31) / 32;
    q.act = g.act;
    q.s_src = g.s_src;
    q.s_flt = g.s_flt;
    q.s_dst = g.s_dst;
    q.c = make_requant_fast(g.s_src, g.s_flt, g.s_dst).c;
    q.d_ohp = make_fastdiv(q.ohp);
    q.d_xb = make_fastdiv(q.xblocks);
    if ((long)q.tiles * q.c4n == 0)
        return TinyNN_SUCCESS;
    const bool tab = requant_table_act(g.act) && requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    if (tab)
        q.table = requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst);
    const int act = tab ? g.act : -1;
    // (the chain kernel has no table instantiation for H_SWISH: the pair is only asked for where one runs)
    const RequantAffine aff = requant_affine_pick(tab, g.act, g.s_src, g.s_flt, g.s_dst);
    q.aff_c = aff.c;
    q.aff_d = aff.d;
    const bool ragged = (g.iw & 3) != 0;
    const void* kern = nullptr;
#define MG_DWM_ACT(S_, R_, F_)                                                                        \
    (act == MEGCC_NONLINE_IDENTITY ? (const void*)dwconv44_mfma_kernel<S_, R_, MEGCC_NONLINE_IDENTITY, F_> \
     : act == MEGCC_NONLINE_RELU   ? (const void*)dwconv44_mfma_kernel<S_, R_, MEGCC_NONLINE_RELU, F_>     \
     : act == MEGCC_NONLINE_H_SWISH ? (const void*)dwconv44_mfma_kernel<S_, R_, MEGCC_NONLINE_H_SWISH, F_> \
                                   : (const void*)dwconv44_mfma_kernel<S_, R_, -1, F_>)
#define MG_DWM_F(S_, F_) (ragged ? MG_DWM_ACT(S_, true, F_) : MG_DWM_ACT(S_, false, F_))
    if (chain) {
        // (IDENTITY / RELU through the table, anything else the literal sequence)
        const int a2 = act == MEGCC_NONLINE_H_SWISH ? -1 : act;
#define MG_DWM_CHAIN(R_, FZ_)                                                                                  \
    (a2 == MEGCC_NONLINE_IDENTITY ? (const void*)dwconv44_mfma_kernel<1, R_, MEGCC_NONLINE_IDENTITY, 3, 2, FZ_> \
     : a2 == MEGCC_NONLINE_RELU   ? (const void*)dwconv44_mfma_kernel<1, R_, MEGCC_NONLINE_RELU, 3, 2, FZ_>     \
                                  : (const void*)dwconv44_mfma_kernel<1, R_, -1, 3, 2, FZ_>)
        if (chain->relu_after_add)
            kern = ragged ? MG_DWM_CHAIN(true, 2) : MG_DWM_CHAIN(false, 2);
        else
            kern = ragged ? MG_DWM_CHAIN(true, 1) : MG_DWM_CHAIN(false, 1);
#undef MG_DWM_CHAIN
    } else if (g.fh == 3)
        kern = MG_DWM_F(1, 3);
    else if (g.fh == 5)
        kern = g.sh == 1 ? MG_DWM_F(1, 5) : MG_DWM_F(2, 5);
    else
        kern = g.sh == 1 ? MG_DWM_F(1, 7) : MG_DWM_F(2, 7);
#undef MG_DWM_F
#undef MG_DWM_ACT
    // one wave per (plane set, tile) while they are all resident at once, otherwise as many
    // waves as are resident, each walking over the tiles of its plane set; the wave count is a
    // multiple of the plane sets and of the 4 waves of a workgroup
    const long items = (long)q.tiles * q.c4n;
    const long cap = (long)num_cus() * 16;
    long per_set = items <= cap ? q.tiles : cap / q.c4n;
    if (per_set < 1)
        per_set = 1;
    long waves = per_set * q.c4n;
    while (waves & 3) {  // (c4n odd: add whole rounds of plane sets until workgroups are full)
        waves += q.c4n;
    }
    void* args[] = {&q};
    hipError_t e = hipLaunchKernel(kern, dim3((unsigned)(waves / 4)), dim3(256), args, 0, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "dwconv44_mfma: %s", hipGetErrorString(e));
    return check_launch("dwconv44_mfma");
}

TinyNNStatus dwconv44_mfma_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    return dwconv44_mfma_run(g, src, flt, bias, dst, nullptr);
}

// 3x3 stride 1 -> max-pool 2x2 stride 2 -> QADD / QFUSE_ADD_RELU in one kernel (g.s_dst: the scale of
// the depthwise result; dst and other: [N][C/4][OH / 2][OW / 2][4])
bool dwconv44_mfma_chain_supported(const ConvGeom& g, const void* src, const void* dst) {
    return dwconv44_mfma_supported(g, src, dst) && g.fh == 3 && g.sh == 1 && g.oh >= 2 && g.ow >= 2;
}
TinyNNStatus dwconv44_mfma_chain_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, const void* other, void* dst,
        bool relu_after_add, float s_other, float s_out) {
    const DwMfmaChain chain = {other, relu_after_add, s_other, s_out};
    return dwconv44_mfma_run(g, src, flt, bias, dst, &chain);
}

}  // namespace mg
