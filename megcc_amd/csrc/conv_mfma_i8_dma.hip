// qsi8 implicit-GEMM convolution for large layers, third generation (same arithmetic and packed
// filter as conv_mfma_i8.hip): every byte reaches LDS by LDS-direct loads, so no wave spends
// registers, VALU work or LDS-write instructions on data movement.
//
//   * filter tile of a stage (taps x 128 oc x 32 ic): 16-byte global->LDS loads, 1 KB per wave-load;
//   * activation patch of a stage: dword buffer->LDS loads. Lane l of a wave-load fetches plane
//     (l & 3) of patch slot (l >> 2): the 64 dwords land as 16 consecutive 16-byte words, which is
//     exactly the LDS layout [sub-chunk][16-channel half][virtual pixel][16 bytes] the MFMA operand
//     reads want (consecutive lanes -> consecutive words, a tap = a wave-uniform byte offset).
//     Padding pixels use an offset beyond the buffer's num_records: the hardware range check
//     returns zero for them, so padding costs nothing;
//   * three LDS stage buffers; the loads of stage g+2 are issued at the start of stage g and waited
//     for (s_waitcnt vmcnt, loads return in order) at the end of stage g+1; one barrier per stage.
//     The stage counter runs across the 256-pixel sub-tiles of the workgroup's pixel range.
//
// One workgroup = 8 waves (2 x 4) on a 128 oc x 256 pixel tile, 64 accumulators per lane. The
// loads of the next sub-tile's first stages are already in flight while a sub-tile's epilogue runs.
//
// Requantisation uses the exact threshold table (epilogue.h) built once per workgroup.
#include <stdlib.h>

#include "conv_mfma_i8.h"

namespace mg {

static constexpr int ACT_RT = -1;

// FH x FW taps, KS 32-channel sub-chunks per stage, LMAX patch slots (compile time, so that the
// number of loads per stage is a constant the vmcnt waits can be written for).
// FC: dst is row-major [pixel][oc] (qsi8 FullyConnected as a 1x1 NCHW convolution on [M,K,1,1]).
// MT: 32-row MFMA tiles per wave along oc; the workgroup tile is 64 * MT output channels.
// DM_NBUF: LDS stage buffers; the loads of stage g + DM_NBUF - 1 are issued at the start of stage g.
// More, smaller stages keep more loads in flight per byte of LDS and push the (in-order) wait for
// the previous sub-tile's output stores further back: what bandwidth-bound 1x1 layers need.
// WGM: waves along oc (1 or 2; 4 waves along pixels). WGM = 1 gives 256-thread workgroups of which
// two share a CU (launch bound 2): their phases drift apart, so one's epilogue, barrier and load
// waits overlap the other's MFMAs.
// BPC: workgroups per CU the register budget is set for.
// NT: 32-pixel MFMA tiles per wave along pixels; the workgroup sub-tile is 128 * NT pixels. NT = 4
// reads 0.75 KB of LDS per MFMA instead of 1 KB (the 2 x 2 wave tile keeps the LDS port as busy as
// the matrix core).
// PM: plane-major activation patch for 3x3 stride-1 layers whose rows are a multiple of 4 pixels:
// the activation loads are 16 bytes per lane as well (the cost of LDS-direct loads goes with their
// number, not their bytes). Slot space = VW = round_up(IW + PW, 4) slots per padded image row,
// image column x at slot x, so the left padding of a row is the tail of the row before; a patch
// starts at a multiple of 4 and every group of 4 slots is 4 neighbouring pixels of one plane or 4
// padding slots (offset beyond num_records -> zeros). LDS holds [plane][slot][4 bytes], a
// wave-load = 256 consecutive slots of one plane, and the MFMA B operand (16 channels = 4 planes)
// is read as four dwords LMAX * 4 bytes apart (two ds_read2st64_b32).
// FCB: FullyConnected with K a multiple of 128 and a 16-byte aligned source: the rows of the
// activation matrix are contiguous in K, so the B tile comes in with 16-byte loads as well - a
// wave-load is 8 rows x 128 bytes = 8 full cache lines. LDS then holds a pixel's 128 bytes of a
// stage together; the eight 16-byte pieces of a row are stored at piece ^ (row & 7) (the load
// fetches the matching piece), which keeps the MFMA operand reads of 8 consecutive rows on
// different banks.
// RS: row split for filters of more than 9 taps (5x5, 7x7): FH = 1 here, a stage is ONE filter row
// (q.FH of them) of one 32-channel chunk - the packed filter keeps the taps of a chunk together, so
// stage chunk * q.FH + fh finds its FW taps at the same place as a stage of an FW-tap filter would;
// its patch is the patch of filter row 0 moved down by fh * DH image rows, with the rows that fall
// off the image read as zeros (every load remembers the image row it fetches for filter row 0).
template <int FH, int FW, int KS, int LMAX, int ACT, bool FC, int MT, int DM_NBUF, int WGM, int BPC, int NT, bool FCB, bool PM, bool RS = false>
__global__ void __launch_bounds__(256 * WGM, BPC) conv_mfma_i8_dma_kernel(MfmaParams q) {
    static_assert(!FCB || (FC && KS == 4 && FH * FW == 1), "FCB: FullyConnected, 128 channels per stage");
    static_assert(!RS || (FH == 1 && KS == 1 && !FC && !FCB && !PM), "RS: one filter row of one chunk per stage");
    constexpr int WGN = 4;
    constexpr int FC_STAGE_ROW = 80, FC_STAGE_BYTES = 32 * FC_STAGE_ROW;  // (FCB: a wave's staging rows)
    constexpr int DM_BNP = 32 * NT * WGN;
    constexpr int DM_WAVES = WGM * WGN, DM_THREADS = 64 * DM_WAVES;
    constexpr int DM_BM = 32 * MT * WGM;
    constexpr int TAPS = FH * FW;
    constexpr int TS = TAPS * KS;
    constexpr int A_BYTES = TS * DM_BM * KROW;
    constexpr int A_CHUNKS = A_BYTES / 1024;
    constexpr int A_PER_WAVE = (A_CHUNKS + DM_WAVES - 1) / DM_WAVES;
    constexpr int B_BYTES = KS * 2 * LMAX * 16;
    constexpr int B_WL = B_BYTES / (FCB || PM ? 1024 : 256);
    static_assert(B_WL % DM_WAVES == 0 && LMAX % 16 == 0, "whole wave-loads");
    static_assert(!PM || (!FC && LMAX % 256 == 0), "PM: planes of whole 1 KB wave-loads");
    constexpr int PM_PARTS = LMAX / 256;  // wave-loads per plane
    static_assert(!FCB || LMAX == 32 * NT * 4, "FCB: one LDS row per pixel of the sub-tile");
    constexpr int B_PER_WAVE = B_WL / DM_WAVES;
    constexpr int LW = LMAX / 16;  // wave-loads per (sub-chunk, half)
    constexpr int N_DMA = A_PER_WAVE + B_PER_WAVE;
    constexpr int BUF_BYTES = A_BYTES + B_BYTES;
    constexpr int N_FLIGHT = N_DMA * (DM_NBUF - 2);  // loads allowed in flight at a stage's end
    static_assert(N_FLIGHT < 64 && DM_NBUF >= 2, "vmcnt range");

    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    int* const rq_table = (int*)(lds + DM_NBUF * BUF_BYTES);
    int* const bias_lds = rq_table + REQUANT_TABLE_ENTRIES;

    // (the wave index through readfirstlane: everything derived from it - which chunks a wave loads,
    //  ring positions, the column count of a ragged sub-tile, the stage counters updated under it -
    //  then lives in scalar registers and branches are scalar)
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned lds0 = __builtin_amdgcn_readfirstlane(lds_address(lds));
    // (waves w and w + 4 share a SIMD: give them different pixel columns, so that the wave with
    //  one column more in a ragged sub-tile does not meet its twin on the same SIMD)
    const int wm = wave / WGN, wn = (wave + wm) % WGN, kg = lane >> 5;
    // (FCB: both operands are matrices of many panels, so each XCD gets a compact rectangle of
    //  tiles; for convolutions the order made no difference - two or four channel tiles per range)
    int tile_x = blockIdx.x, tile_y = blockIdx.y;
    if constexpr (FCB)
        xcd_tile(q.xo, blockIdx.x, blockIdx.y, gridDim.x, gridDim.y, tile_x, tile_y);
    const int oc0 = tile_y * DM_BM;
    const int range0 = tile_x * q.range_len;
    const int range1 = min(range0 + q.range_len, q.P);
    const int stages = q.stages;
    const int n_tiles = (range1 - range0 + DM_BNP - 1) / DM_BNP;
    const int G = n_tiles * stages;

    // ---- once per workgroup: requantisation thresholds and the bias slice of this oc tile
    if constexpr (ACT != ACT_RT) {
        if (tid < REQUANT_TABLE_ENTRIES)
            rq_table[tid] = kernarg_rq_table(tid);
    }
    for (int i = tid; i < DM_BM; i += DM_THREADS)
        bias_lds[i] = (q.bias && oc0 + i < q.OC) ? q.bias[oc0 + i] : 0;

    // ---- load side ---------------------------------------------------------------------------
    v4u src_rsrc = make_raw_buffer(q.src, (unsigned)q.src_bytes);
#pragma unroll
    for (int i = 0; i < 4; ++i)
        src_rsrc[i] = __builtin_amdgcn_readfirstlane(src_rsrc[i]);
    // filter: chunk c = wave + 8a (wrapped: the surplus loads repeat a chunk, same bytes to the
    // same place), c = (DM_BM / 32) * tap-step + 1 KB part
    int a_chunk[A_PER_WAVE];  // wave-uniform
#pragma unroll
    for (int a = 0; a < A_PER_WAVE; ++a) {
        a_chunk[a] = (wave + a * DM_WAVES) % A_CHUNKS;
    }
    const int lane16 = lane * 16;
    // activations: wave-load u = wave + 8j covers 16 slots of (sub-chunk, half) u / LW; this lane
    // fetches plane (lane & 3) of slot (u % LW) * 16 + (lane >> 2). b_goff = byte offset of that
    // dword in the first plane group of a stage, or 2^31 (out of range -> zero) for padding.
    unsigned b_goff[B_PER_WAVE];
    int b_ih[RS ? B_PER_WAVE : 1];  // RS: image row of the load for filter row 0 (far below 0: never valid)
    constexpr int NEVER = -0x40000000;
    // PM: first slot of a sub-tile's patch. Slot space = rows of VW (a multiple of 4) slots per
    // padded image row, image column x at slot x: the left padding of a row is the tail of the
    // row before it. The patch starts PW slots before the first pixel's window, rounded down to 4.
    auto pm_base = [&](int p0) __attribute__((always_inline)) {
        return (vp_of(q, p0) - q.PW) & ~3;  // (arithmetic: also right below zero)
    };
    auto describe = [&](int p0) __attribute__((always_inline)) {
        if constexpr (FCB) {
            // wave-load u covers rows 8u .. 8u + 7; rows beyond the matrix repeat the last one
            // (their columns of the product are never stored)
            static_for<B_PER_WAVE>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const int u = wave + j * DM_WAVES;
                const int row = min(p0 + u * 8 + (lane >> 3), q.P - 1);
                b_goff[j] = (unsigned)row * (unsigned)q.image_stride + (((lane & 7) ^ (lane >> 3)) << 4);
            });
            return;
        }
        if constexpr (PM) {
            // wave-load u = plane u / PM_PARTS, slots (u % PM_PARTS) * 256 + 4 * lane .. + 3: four
            // neighbours of one image row (rows are 4-aligned in slot space) or four padding slots
            const int vbase = pm_base(p0);
            // slots the sub-tile's windows reach; the rest of the LMAX slots is not fetched
            const int L = vp_of(q, min(p0 + DM_BNP, range1) - 1) - q.PW +
                          ((FH - 1) * q.DH) * q.VW + (FW - 1) * q.DW - vbase + 1;
            static_for<B_PER_WAVE>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const int u = wave + j * DM_WAVES;
                const int pl = u / PM_PARTS;
                const int slot = (u - pl * PM_PARTS) * 256 + lane * 4;
                const int vs = vbase + slot;
                unsigned off = 0x80000000u;
                if (vs >= 0 && slot < L) {
                    const int v = fdiv(vs, q.dVW), vc = vs - v * q.VW;
                    const int n = fdiv(v, q.dVH), ih = v - n * q.VH - q.PH;
                    if (n < q.N && (unsigned)ih < (unsigned)q.IH && vc < q.IW)
                        off = n * q.image_stride + ih * q.row_stride + vc * q.pix_stride +
                              pl * q.plane_stride;
                }
                b_goff[j] = off;
            });
            return;
        }
        const int plast = min(p0 + DM_BNP, range1) - 1;
        const int vp0 = vp_of(q, p0);
        const int L = vp_of(q, plast) + ((FH - 1) * q.DH) * q.VW + (FW - 1) * q.DW - vp0 + 1;
        static_for<B_PER_WAVE>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int u = wave + j * DM_WAVES;
            const int kh = u / LW, slot = (u - kh * LW) * 16 + (lane >> 2);
            unsigned off = 0x80000000u;
            if constexpr (RS)
                b_ih[j] = NEVER;
            if (slot < L) {
                const int vp = vp0 + slot;
                const int v = fdiv(vp, q.dVW), vc = vp - v * q.VW;
                const int n = fdiv(v, q.dVH), vh = v - n * q.VH;
                const int ih = vh - q.PH, iw = vc - q.PW;
                if constexpr (RS) {
                    // (the offset of filter row 0 also where that row is above the image: issue()
                    //  adds fh * DH rows and checks the row it lands on)
                    if (n < q.N && (unsigned)iw < (unsigned)q.IW) {
                        b_ih[j] = ih;
                        off = (unsigned)(n * q.image_stride + ih * q.row_stride + iw * q.pix_stride +
                                         ((kh >> 1) * 8 + (kh & 1) * 4 + (lane & 3)) * q.plane_stride);
                    }
                } else if (n < q.N && (unsigned)ih < (unsigned)q.IH && (unsigned)iw < (unsigned)q.IW)
                    off = n * q.image_stride + ih * q.row_stride + iw * q.pix_stride +
                          ((kh >> 1) * 8 + (kh & 1) * 4 + (lane & 3)) * q.plane_stride;
            }
            b_goff[j] = off;
        });
    };
    int lp0 = range0, lst = 0, lbuf = 0;  // load cursor: sub-tile, stage in it, LDS buffer
    int lfh = 0, lchunk = 0;              // RS: filter row and chunk of stage lst
    describe(lp0);
    auto issue = [&](int bufidx) __attribute__((always_inline)) {
        const unsigned buf = lds0 + bufidx * BUF_BYTES;  // (LDS byte address, scalar)
        const int8_t* abase = q.wp + ((size_t)lst * TS * q.OCP + oc0) * KROW;
#pragma unroll
        for (int a = 0; a < A_PER_WAVE; ++a)
            dma_global_saddr_b128(abase + ((size_t)(a_chunk[a] / (DM_BM / 32)) * q.OCP * KROW +
                                           (a_chunk[a] % (DM_BM / 32)) * 1024),
                                  lane16, buf + a_chunk[a] * 1024);
        const unsigned poff = RS ? (unsigned)(lchunk * 8) * (unsigned)q.plane_stride +
                                           (unsigned)(lfh * q.DH) * (unsigned)q.row_stride
                                 : (unsigned)(lst * KS * 8) * (unsigned)q.plane_stride;
        static_for<B_PER_WAVE>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int u = wave + j * DM_WAVES;
            if constexpr (FCB)
                dma_global_b128(q.src + (b_goff[j] + poff), buf + A_BYTES + u * 1024);
            else if constexpr (PM)
                dma_buffer_b128(src_rsrc, b_goff[j] + poff, buf + A_BYTES + u * 1024);
            else if constexpr (RS)
                dma_buffer_b32(src_rsrc,
                               (unsigned)(b_ih[j] + lfh * q.DH) < (unsigned)q.IH ? b_goff[j] + poff : 0x80000000u,
                               buf + A_BYTES + u * 256);
            else
                dma_buffer_b32(src_rsrc, b_goff[j] + poff, buf + A_BYTES + u * 256);
        });
        if constexpr (RS) {
            if (++lfh == q.FH) {
                lfh = 0;
                ++lchunk;
            }
        }
        if (++lst == stages) {
            lst = 0;
            lchunk = 0;  // (lfh is 0 here: the stages of a sub-tile are whole chunks)
            lp0 += DM_BNP;
            if (lp0 < range1)
                describe(lp0);
        }
        lbuf = lbuf == DM_NBUF - 1 ? 0 : lbuf + 1;
    };

    // ---- compute side ------------------------------------------------------------------------
    int a_off[MT];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
        int r = (wm * MT + mi) * 32 + (lane & 31);
        a_off[mi] = r * KROW + (((kg ^ (r >> 3)) & 1) << 4);
    }

    v16i acc[MT][NT];

    // Epilogue of one 32 oc x 32 pixel MFMA tile (16 outputs per lane = 4 NCHW44 dwords), written
    // as one straight-line block so that its 4 bias reads and 16 table look-ups are in flight
    // together. ob: dword index in dst of this lane's pixel in oc-group 0 (-1: lane beyond the
    // sub-tile, -2: whole 32-pixel column beyond it, wave-uniform).
    // the 16 requantised outputs of this lane in tile (mi, ni)
    auto requant_tile = [&](auto mic, auto nic, int (&r)[16], const int* tbl) __attribute__((always_inline)) {
        constexpr int mi = decltype(mic)::value, ni = decltype(nic)::value;
        if constexpr (ACT == ACT_RT) {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                r[e] = requant_conv_rt(q.act, acc[mi][ni][e], q.s_src, q.s_flt, q.s_dst);
        } else if (ACT != MEGCC_NONLINE_H_SWISH && q.rq.aff_d != 0.f) {  // (uniform)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                r[e] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(acc[mi][ni][e], q.rq.aff_c, q.rq.aff_d);
        } else {
            int m[16], t[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                m[e] = requant_table_candidate<ACT>(acc[mi][ni][e], q.rq.c);
                t[e] = tbl[m[e] + 128];
            }
#pragma unroll
            for (int e = 0; e < 16; ++e)
                r[e] = m[e] + (acc[mi][ni][e] > t[e] ? 1 : 0);
        }
    };
    // (FC, dst_fc >= 2) the lane's 16 bytes of tile (mi, ni): channels 16 kg .. + 15 of the tile, row =
    // the lane's column. A lane's four dwords are channels 8 e4 + 4 kg .. + 3, so lanes l and l + 32
    // (same row, the two K-halves) together own 32 consecutive bytes; two v_permlane32_swap give the
    // lower lane the first 16 of them and the upper lane the rest.
    auto fc_piece = [&](auto mic, auto nic, const int* tbl) __attribute__((always_inline)) -> v4u {
        typedef unsigned v2u_t __attribute__((ext_vector_type(2)));
        int r[16];
        requant_tile(mic, nic, r, tbl);
        uint32_t w[4];
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4)
            w[e4] = pack4_perm(r[e4 * 4], r[e4 * 4 + 1], r[e4 * 4 + 2], r[e4 * 4 + 3]);
        const v2u_t s02 = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
        const v2u_t s13 = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
        return v4u{s02[0], s02[1], s13[0], s13[1]};
    };
    auto emit_tile = [&](auto mic, auto nic, const int ob, const int* tbl) __attribute__((always_inline)) {
        constexpr int mi = decltype(mic)::value;
        if (ob < -1)
            return;
        const int ocl = (wm * MT + mi) * 32 + kg * 4;
        if constexpr (FC) {
            // Row-major [row][OC] output with whole 32-channel tiles and 16-byte alignment: one 16-byte
            // store per lane instead of four dword stores 4096 bytes apart from their neighbours' (the
            // dword stores were half of the 4096 x 4096 x 4096 layer's time).
            if (q.dst_fc >= 2) {  // (uniform)
                const v4u px = fc_piece(mic, nic, tbl);
                if (ob >= 0 && oc0 + (wm * MT + mi) * 32 < q.OC)  // (whole tiles: OC is a multiple of 32)
                    *(v4u*)(q.dst + (size_t)ob * q.OC + oc0 + (wm * MT + mi) * 32 + kg * 16) = px;
                return;
            }
        }
        int r[16];
        requant_tile(mic, nic, r, tbl);
        if (ob >= 0) {
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int oc = oc0 + ocl + e4 * 8;
                if (oc >= q.OC)
                    continue;
                const uint32_t w = pack4_perm(r[e4 * 4], r[e4 * 4 + 1], r[e4 * 4 + 2], r[e4 * 4 + 3]);
                if constexpr (!FC) {
                    // scalar base (channel group) + 32-bit lane offset (pixel and K-half's plane)
                    int8_t* const base =
                            q.dst + ((size_t)(((oc0 >> 2) + (wm * MT + mi) * 8 + e4 * 2) * q.OHW) << 2);
                    *(uint32_t*)(base + ((unsigned)ob << 2)) = w;
                } else {  // ob = pixel (row of the output matrix)
                    int8_t* o = q.dst + (size_t)ob * q.OC + oc;
                    if ((q.OC & 3) == 0) {
                        *(uint32_t*)o = w;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (oc + e < q.OC)
                                o[e] = (int8_t)(w >> (8 * e));
                    }
                }
            }
        }
    };

    // ---- prologue: DM_NBUF - 1 stages in flight, the first one landed
#pragma unroll
    for (int i = 0; i < DM_NBUF - 1; ++i)
        if (i < G)
            issue(i);
    if (G >= DM_NBUF - 1)
        wait_vmcnt<N_FLIGHT>();
    else
        wait_vmcnt<0>();
    lds_barrier();

    int g = 0, cbuf = 0;
    for (int p0 = range0; p0 < range1; p0 += DM_BNP) {
        const int plast = min(p0 + DM_BNP, range1) - 1;
        const int vp0 = PM ? pm_base(p0) + q.PW : vp_of(q, p0);
        int b_byte[NT];  // LDS byte offset of this lane's 16 channels at tap (0,0)
        int cur_o[NT];
        int cols = 0;    // wave-uniform: 32-pixel columns of this wave with pixels of the sub-tile
#pragma unroll
        for (int ni = 0; ni < NT; ++ni) {
            // columns are dealt round-robin to the 4 pixel waves, so a partial sub-tile keeps
            // all of them busy
            const int pc = p0 + (ni * WGN + wn) * 32;
            const int p = pc + (lane & 31);
            if constexpr (FCB)
                b_byte[ni] = p - p0;  // LDS row of this lane's pixel
            else if constexpr (PM)  // dword of the pixel in the lane's first plane
                b_byte[ni] = (kg * 4 * LMAX + (p <= plast ? vp_of(q, p) - vp0 : 0)) * 4;
            else
                b_byte[ni] = (kg * LMAX + (p <= plast ? vp_of(q, p) - vp0 : 0)) * 16;
            cols += pc <= plast ? 1 : 0;
            const int pn = (int)fdiv(p, q.dOHW);
            cur_o[ni] = pc > plast ? -2
                        : p > plast ? -1
                        : FC        ? p
                                    : pn * (q.OC >> 2) * q.OHW + (p - pn * q.OHW) + kg * q.OHW;
        }
        // the accumulators start from the bias of their output channel (register e of a tile:
        // channel 8 * (e / 4) + 4 * kg + e % 4)
#pragma unroll
        for (int mi = 0; mi < MT; ++mi) {
            v4i bv[4];
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4)
                bv[e4] = *(const v4i*)(bias_lds + (wm * MT + mi) * 32 + kg * 4 + e4 * 8);
#pragma unroll
            for (int ni = 0; ni < NT; ++ni)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[mi][ni][e] = bv[e / 4][e % 4];
        }

        auto stage_body = [&](auto cols_c, const int8_t* bufA, int dma_buf) __attribute__((always_inline)) {
            constexpr int COLS = decltype(cols_c)::value;
            if (g + DM_NBUF - 1 < G)
                issue(dma_buf);
            const int8_t* bufB = bufA + A_BYTES;
            if constexpr (COLS > 0) {
                v4i fa[2][MT], fb[2][NT];
                auto fetch = [&](auto tc) __attribute__((always_inline)) {
                    constexpr int t = decltype(tc)::value;
                    constexpr int ks = t / TAPS, tap = t % TAPS;
                    constexpr int fh = tap / FW, fw = tap % FW;
                    const int tap_off = fh * q.DH * q.VW + fw * q.DW;
#pragma unroll
                    for (int mi = 0; mi < MT; ++mi)
                        fa[t & 1][mi] = *(const v4i*)(bufA + t * (DM_BM * KROW) + a_off[mi]);
#pragma unroll
                    for (int ni = 0; ni < COLS; ++ni) {
                        if constexpr (FCB)
                            fb[t & 1][ni] = *(const v4i*)(bufB + b_byte[ni] * 128 +
                                                          (((ks * 2 + kg) ^ (b_byte[ni] & 7)) << 4));
                        else if constexpr (PM) {
                            const int8_t* b0 = bufB + ks * (8 * LMAX * 4) + b_byte[ni] + tap_off * 4;
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                fb[t & 1][ni][i] = *(const int*)(b0 + i * (LMAX * 4));
                        } else
                            fb[t & 1][ni] = *(const v4i*)(bufB + ks * (2 * LMAX * 16) + b_byte[ni] +
                                                          tap_off * 16);
                    }
                };
                fetch(std::integral_constant<int, 0>{});
                static_for<TS>([&](auto tc) {
                    constexpr int t = decltype(tc)::value;
                    if constexpr (t + 1 < TS)
                        fetch(std::integral_constant<int, t + 1>{});
                    // keep the compiler from sinking these reads below the MFMAs of step t
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ni = 0; ni < COLS; ++ni)
#pragma unroll
                        for (int mi = 0; mi < MT; ++mi)
                            acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                    fa[t & 1][mi], fb[t & 1][ni], acc[mi][ni], 0, 0, 0);
                });
            }
        };
        auto run_stages = [&](auto cols_c) __attribute__((always_inline)) {
            for (int st = 0; st < stages; ++st, ++g) {
                stage_body(cols_c, lds + cbuf * BUF_BYTES, lbuf);
                // stage g+1 must have landed; the DM_NBUF - 2 stages issued after it may be in
                // flight (stores issued in between only make the wait longer, never shorter)
                if (g + DM_NBUF - 1 < G)
                    wait_vmcnt<N_FLIGHT>();
                else
                    wait_vmcnt<0>();
                lds_barrier();
                cbuf = cbuf == DM_NBUF - 1 ? 0 : cbuf + 1;
            }
        };
        static_for<NT + 1>([&](auto cc) {
            if (cols == decltype(cc)::value)
                run_stages(cc);
        });

        if constexpr (FCB && MT == 4) {  // (the 256-channel tile: its two stage buffers leave room for the staging area)
            // dst_fc == 3: the rows leave through a staging area in LDS (this wave's own 32 rows x 64
            // bytes, rows 80 bytes apart): the lanes park the 16-byte pieces of two neighbouring tiles
            // and read them back four lanes to a row, so that a store instruction writes 64 contiguous
            // bytes of each of 16 rows instead of 32 bytes of each of 32.
            if (q.dst_fc == 3) {  // (uniform)
                int8_t* const stage = (int8_t*)(bias_lds + (DM_BM > 128 ? DM_BM : 128)) + wave * FC_STAGE_BYTES;
                static_for<NT>([&](auto nic) {
                    constexpr int ni = decltype(nic)::value;
                    if (cur_o[ni] < -1)
                        return;
                    const int row0 = p0 + (ni * WGN + wn) * 32;  // first row of this 32-row column
                    static_for<MT / 2>([&](auto hc) {
                        constexpr int h = decltype(hc)::value;
                        const v4u pa = fc_piece(std::integral_constant<int, 2 * h>{}, nic, rq_table);
                        const v4u pb = fc_piece(std::integral_constant<int, 2 * h + 1>{}, nic, rq_table);
                        *(v4u*)(stage + (lane & 31) * FC_STAGE_ROW + kg * 16) = pa;
                        *(v4u*)(stage + (lane & 31) * FC_STAGE_ROW + 32 + kg * 16) = pb;
                        const int ocb = oc0 + (wm * MT + 2 * h) * 32;  // (64 channels from here on)
#pragma unroll
                        for (int it = 0; it < 2; ++it) {
                            const int rr = (lane >> 2) + 16 * it, piece = lane & 3;
                            const v4u v = *(const v4u*)(stage + rr * FC_STAGE_ROW + piece * 16);
                            if (row0 + rr <= plast && ocb + piece * 16 < q.OC)
                                *(v4u*)(q.dst + (size_t)(row0 + rr) * q.OC + ocb + piece * 16) = v;
                        }
                    });
                });
                continue;
            }
        }
        static_for<MT>([&](auto mic) {
            static_for<NT>([&](auto nic) { emit_tile(mic, nic, cur_o[decltype(nic)::value], rq_table); });
        });
    }
}

// ---- configurations --------------------------------------------------------------------------
template <int FH, int FW, int KS, int LMAX, bool FC, int MT = 2, int DM_NBUF = 3, int WGM = 2, int BPC = 1, int NT = 2, bool FCB = false, bool PM = false>
static PipeConfig make_dma_config(int act, bool table_ok);

// row-split configurations (filters of more than 9 taps): 64 * MT oc x 128 * NT px, FW taps per stage
template <int FW, int LMAX, int MT, int DM_NBUF, int NT>
static PipeConfig make_rs_config(int act, bool table_ok) {
    PipeConfig c;
    c.bm = 64 * MT;
    c.bn = 128 * NT;
    c.ks = 1;
    c.threads = 512;
    c.nbuf = DM_NBUF;
    c.blocks_per_cu = 1;
    c.a_bytes = FW * c.bm * KROW;
    c.fixed_lmax = LMAX;
    c.rs = 1;
    c.extra_lds = REQUANT_TABLE_ENTRIES * 4 + 128 * 4;
    c.kernel = (const void*)conv_mfma_i8_dma_kernel<1, FW, 1, LMAX, ACT_RT, false, MT, DM_NBUF, 2, 1, NT, false, false, true>;
    if (act == MEGCC_NONLINE_IDENTITY && table_ok)
        c.kernel = (const void*)conv_mfma_i8_dma_kernel<1, FW, 1, LMAX, MEGCC_NONLINE_IDENTITY, false, MT, DM_NBUF, 2, 1, NT, false, false, true>;
    else if (act == MEGCC_NONLINE_RELU && table_ok)
        c.kernel = (const void*)conv_mfma_i8_dma_kernel<1, FW, 1, LMAX, MEGCC_NONLINE_RELU, false, MT, DM_NBUF, 2, 1, NT, false, false, true>;
    else if (act == MEGCC_NONLINE_H_SWISH && table_ok)
        c.kernel = (const void*)conv_mfma_i8_dma_kernel<1, FW, 1, LMAX, MEGCC_NONLINE_H_SWISH, false, MT, DM_NBUF, 2, 1, NT, false, false, true>;
    return c;
}

template <int FH, int FW, int KS, int LMAX, bool FC, int MT, int DM_NBUF, int WGM, int BPC, int NT, bool FCB, bool PM>
static PipeConfig make_dma_config(int act, bool table_ok) {
    constexpr int DM_BM = 32 * MT * WGM;
    PipeConfig c;
    c.bm = DM_BM;
    c.bn = 128 * NT;
    c.ks = KS;
    c.threads = 256 * WGM;
    c.nbuf = DM_NBUF;
    c.blocks_per_cu = BPC;
    c.a_bytes = FH * FW * KS * c.bm * KROW;
    c.fixed_lmax = LMAX;
    c.pm = PM ? 1 : 0;
    c.extra_lds = REQUANT_TABLE_ENTRIES * 4 + (DM_BM > 128 ? DM_BM : 128) * 4 +
                  (FCB && MT == 4 ? 4 * WGM * 32 * 80 : 0);  // (32 rows x 80 bytes of staging per wave)
    c.fcb = FCB ? 1 : 0;
    c.kernel = (const void*)conv_mfma_i8_dma_kernel<FH, FW, KS, LMAX, ACT_RT, FC, MT, DM_NBUF, WGM, BPC, NT, FCB, PM>;
    if (act == MEGCC_NONLINE_IDENTITY && table_ok)
        c.kernel = (const void*)conv_mfma_i8_dma_kernel<FH, FW, KS, LMAX, MEGCC_NONLINE_IDENTITY, FC, MT, DM_NBUF, WGM, BPC, NT, FCB, PM>;
    else if (act == MEGCC_NONLINE_RELU && table_ok)
        c.kernel = (const void*)conv_mfma_i8_dma_kernel<FH, FW, KS, LMAX, MEGCC_NONLINE_RELU, FC, MT, DM_NBUF, WGM, BPC, NT, FCB, PM>;
    if constexpr (!FC) {  // (FullyConnected with H_SWISH keeps the literal sequence)
        if (act == MEGCC_NONLINE_H_SWISH && table_ok)
            c.kernel = (const void*)conv_mfma_i8_dma_kernel<FH, FW, KS, LMAX, MEGCC_NONLINE_H_SWISH, FC, MT, DM_NBUF, WGM, BPC, NT, FCB, PM>;
    }
    return c;
}

// 3x3 and 1x1 NCHW44 layers and FullyConnected with at least 128 output channels (64 for the 1x1
// with 32 input channels) and enough pixels. 1x1: 128 input channels per stage (64 / 32 when
// IC <= 64 / 32).
// variant 0: 512-pixel sub-tiles (3x3 only, two stage buffers); variant 1: 256-pixel sub-tiles;
// variants 2 / 3: variant 0 with the plane-major patch of 768 / 1024 slots.
bool conv_mfma_dma_config(const ConvGeom& g, bool fc, int variant, bool b128_ok, PipeConfig* c) {
    const long P = (long)g.n * g.oh * g.ow;
    const bool k3 = g.fh == 3 && g.fw == 3, k1 = g.fh == 1 && g.fw == 1;
    if (variant == 8 || variant == 9) {
        // square filters of 5 or 7 columns, one filter row per stage: variant 8 with 256-pixel sub-tiles
        // and three buffers of 512 patch slots (stride 1), variant 9 with 128-pixel sub-tiles and two
        // buffers of 1024 slots (stride 2, wide rows, dilation)
        if (fc || g.fmt != MEGCC_FMT_NCHW44 || !(g.fw == 5 || g.fw == 7) || g.fh != g.fw || g.oc < 32 ||
            P < 2048 || (long)g.n * g.oc * g.oh * g.ow >= (1L << 31))
            return false;
        const bool okt = requant_table_ok(g.s_src, g.s_flt, g.s_dst);
        const bool wide = g.oc >= 128;
        if (variant == 8)
            *c = g.fw == 5 ? (wide ? make_rs_config<5, 512, 2, 3, 2>(g.act, okt) : make_rs_config<5, 512, 1, 3, 2>(g.act, okt))
                           : (wide ? make_rs_config<7, 512, 2, 3, 2>(g.act, okt) : make_rs_config<7, 512, 1, 3, 2>(g.act, okt));
        else
            *c = g.fw == 5 ? (wide ? make_rs_config<5, 1024, 2, 2, 1>(g.act, okt) : make_rs_config<5, 1024, 1, 2, 1>(g.act, okt))
                           : (wide ? make_rs_config<7, 1024, 2, 2, 1>(g.act, okt) : make_rs_config<7, 1024, 1, 2, 1>(g.act, okt));
        return true;
    }
    if (g.fh * g.fw > MAX_TAPS_STAGE)
        return false;
    if (variant == 6 || variant == 7) {
        // small 3x3 layers (batch 1): 32 oc x 128 px tiles of four waves, one 32 x 32 MFMA tile
        // each, so that a few thousand pixels still give every CU a workgroup; variant 6 with the
        // plane-major patch
        // (only while the 128-channel tiles of the other variants would get fewer than 32 pixels per
        //  CU: above that, half-filled 256-pixel tiles on part of the CUs are faster - N=3,
        //  128->128, 56x56: 8.9 against 9.3 us, N=2, 256->256: 13.1 against 14.5 us; below, N=2,
        //  128->128: 6.1 against 8.8 us; layers under 4096 pixels keep these tiles up to 64 per CU)
        if (!k3 || fc || g.fmt != MEGCC_FMT_NCHW44 || P < 512 ||
            P * ((g.oc + 127) / 128) >= (P >= 4096 ? 32L : 64L) * num_cus() || g.oc < 32 || (g.ic & 31) ||
            (long)g.n * g.oc * g.oh * g.ow >= (1L << 31))
            return false;
        const bool okt = requant_table_ok(g.s_src, g.s_flt, g.s_dst);
        if (variant == 6) {
            if (g.sw != 1 || (g.iw & 3) || !b128_ok ||
                ((long)g.n * (g.ih + 2 * g.ph) + 2L * g.fh * g.dh) * (g.iw + g.pw + 3) >= (1L << 31))
                return false;
            *c = make_dma_config<3, 3, 1, 512, false, 1, 3, 1, 1, 1, false, true>(g.act, okt);
        } else {
            *c = make_dma_config<3, 3, 1, 384, false, 1, 3, 1, 1, 1>(g.act, okt);
        }
        return true;
    }
    if (!(k3 || k1) || !(g.fmt == MEGCC_FMT_NCHW44 || fc) || g.oc < 64 || P < 2048)
        return false;
    if (g.oc < 128 && !(k1 && !fc && g.ic <= 32) && !k3)
        return false;  // 64-channel tiles: 3x3 layers and the 1x1 with 32 input channels
    if ((long)g.n * g.oc * g.oh * g.ow >= (1L << 31))
        return false;  // 32-bit output offsets
    const bool ok = requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    // measured slower on the 256-channel 56x56 layer (91 us): two 256-thread workgroups per CU
    // with 64-channel tiles and two buffers (100 us), four waves of 128 oc x 64 pixels (107 us)
    if (variant == 2 || variant == 3) {
        // plane-major patch, 16-byte activation loads: needs whole 16-byte groups per image row
        if (!k3 || g.sw != 1 || (g.iw & 3) || !b128_ok || fc ||
            ((long)g.n * (g.ih + 2 * g.ph) + 2L * g.fh * g.dh) * (g.iw + g.pw + 3) >= (1L << 31))
            return false;
        // 768 slots hold a 512-pixel sub-tile of rows up to ~60 slots inside one image; a sub-tile
        // that crosses into the next image also spans the padding rows between them
        if (g.oc < 128 && variant == 2)
            *c = make_dma_config<3, 3, 1, 768, false, 1, 2, 2, 1, 4, false, true>(g.act, ok);
        else if (g.oc < 128)
            *c = make_dma_config<3, 3, 1, 1024, false, 1, 2, 2, 1, 4, false, true>(g.act, ok);
        else if (variant == 2)
            *c = make_dma_config<3, 3, 1, 768, false, 2, 2, 2, 1, 4, false, true>(g.act, ok);
        else
            *c = make_dma_config<3, 3, 1, 1024, false, 2, 2, 2, 1, 4, false, true>(g.act, ok);
        return true;
    }
    if (variant == 4) {  // variant 1 (256-pixel sub-tiles, three buffers) with the plane-major patch
        if (!k3 || g.sw != 1 || (g.iw & 3) || !b128_ok || fc ||
            ((long)g.n * (g.ih + 2 * g.ph) + 2L * g.fh * g.dh) * (g.iw + g.pw + 3) >= (1L << 31))
            return false;
        if (g.oc < 128)
            *c = make_dma_config<3, 3, 1, 512, false, 1, 3, 2, 1, 2, false, true>(g.act, ok);
        else
            *c = make_dma_config<3, 3, 1, 512, false, 2, 3, 2, 1, 2, false, true>(g.act, ok);
        return true;
    }
    // 3x3 with stride 2 (down-sampling layers): the patch of a sub-tile holds four input pixels per
    // output pixel, so the sub-tiles are smaller and the patches longer - 256 pixels in 1280 slots
    // for large layers (variant 0), 128 pixels in 768 slots otherwise (variant 1). N=64, 128->128,
    // 56x56: 17.1 us (the one-stage kernel: 29.4); 256->256, 28x28: 16.9 (36.9); 512->512, 14x14:
    // 24.9 (40.9).
    const bool k3s2 = k3 && g.sh == 2 && g.sw == 2 && !fc;
    if (k3s2 && (variant == 0 || variant == 1)) {
        if (g.oc < 128 || (variant == 0 && P < 32768))
            return false;
        if (variant == 0)
            *c = make_dma_config<3, 3, 1, 1280, false, 2, 2>(g.act, ok);
        else
            *c = make_dma_config<3, 3, 1, 768, false, 2, 2, 2, 1, 1>(g.act, ok);
        return true;
    }
    if (variant == 0) {
        if (!k3)
            return false;
        if (g.oc < 128)  // 64 oc x 512 px: each wave 32 oc x 128 px
            *c = make_dma_config<3, 3, 1, 768, false, 1, 2, 2, 1, 4>(g.act, ok);
        else
            *c = make_dma_config<3, 3, 1, 768, false, 2, 2, 2, 1, 4>(g.act, ok);
        return true;
    }
    if (k3 && g.oc < 128)
        *c = make_dma_config<3, 3, 1, 512, false, 1>(g.act, ok);
    else if (k3)
        *c = make_dma_config<3, 3, 1, 512, false>(g.act, ok);
    else if (fc && (g.ic & 127) == 0 && b128_ok && g.oc >= 256)
        // 256 x 256 tile, each wave 128 oc x 64 rows (4 x 2 MFMA tiles: 0.75 KB of LDS per MFMA;
        // measured 86 us on 4096^3 against 105 us with the 128 x 256 tile)
        *c = make_dma_config<1, 1, 4, 256, true, 4, 2, 2, 1, 2, true>(g.act, ok);
    else if (fc && (g.ic & 127) == 0 && b128_ok)
        *c = make_dma_config<1, 1, 4, 256, true, 2, 3, 2, 1, 2, true>(g.act, ok);
    else if (fc)
        *c = make_dma_config<1, 1, 4, 256, true>(g.act, ok);
    else if (g.oc < 128)
        *c = make_dma_config<1, 1, 1, 256, false, 1, 8>(g.act, ok);
    else if (g.ic <= 128)
        *c = make_dma_config<1, 1, 2, 256, false, 2, 6>(g.act, ok);

    else
        *c = make_dma_config<1, 1, 4, 256, false>(g.act, ok);
    return true;
}

}  // namespace mg
