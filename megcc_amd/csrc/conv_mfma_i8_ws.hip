// Wave-specialised variant of the qsi8 implicit-GEMM convolution (same arithmetic, packed filter
// and LDS row layout as conv_mfma_i8.hip / conv_mfma_i8_wide.hip) for large NCHW44 layers.
//
// In the symmetric kernels every wave alternates between issuing global loads, writing LDS and
// feeding the matrix cores, and the workgroup barrier keeps all waves in the same phase: while
// loads are issued the MFMA pipes idle. Here the two jobs belong to different waves of one
// workgroup, so the hardware interleaves them on every SIMD:
//
//   waves 0..7  (consumers, 2 x 4 over a 128 oc x 256 pixel tile, 64 accumulators per lane):
//               LDS reads + MFMA of stage k out of buffer k % 3, then the requantising epilogue;
//   waves 8..11 (producers): during step k they start the filter loads of stage k+2, straight
//               into LDS buffer (k+2) % 3 with 16-byte LDS-direct loads (no registers, no LDS
//               write instructions), and the activation loads of stage k+3 into registers, and
//               scatter the activations of stage k+1 (loaded two steps earlier) into buffer
//               (k+1) % 3 as rows of 32 channels per virtual pixel.
//
// One workgroup barrier per step. The stage counter runs across the
// sub-tiles of a workgroup's pixel range, so the producers are already fetching the next sub-tile
// while the consumers run the epilogue of the current one.
//
// LDS layout of the activation patch: [sub-chunk][16-channel half][virtual pixel][16 bytes], i.e.
// the lanes of an MFMA operand read (consecutive pixels, one half) touch consecutive 16-byte
// words, and a tap is a wave-uniform address offset. The gather takes 4 dwords (4 planes of one
// pixel) per 16-byte word: every LDS write is one conflict-free 16-byte store and padding is a
// zero written in place.
#include <stdlib.h>

#include "conv_mfma_i8.h"

namespace mg {

static constexpr int ACT_RT = -1;
static constexpr int WS_CONSUMERS = 512;  // threads
static constexpr int WS_PRODUCERS = 256;
static constexpr int WS_THREADS = WS_CONSUMERS + WS_PRODUCERS;
static constexpr int WS_NBUF = 3;
static constexpr int WS_BM = 128, WS_BNP = 256;

struct WsTile {  // activation patch of one sub-tile
    int vp0, L, v_first, rows, slot_base;
};

// DBG (development builds only, -DMG_WS_DEBUG): bit mask of parts left out for timing experiments
template <int FH, int FW, int KS, int ACT, int MAXB, int DBG = 0>
__global__ void __launch_bounds__(WS_THREADS) conv_mfma_i8_ws_kernel(MfmaParams q) {
    constexpr int MT = 2, NT = 2, WGN = 4;
    constexpr int TAPS = FH * FW;
    constexpr int TS = TAPS * KS;
    constexpr int A_BYTES = TS * WS_BM * KROW;
    constexpr int A_LOADS = A_BYTES / 1024 / (WS_PRODUCERS / 64);  // LDS-direct loads per wave
    static_assert(A_BYTES % (1024 * (WS_PRODUCERS / 64)) == 0, "whole 1 KB chunks per wave");

    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    const int b_bytes = KS * q.Lmax * KROW;
    const int buf_bytes = A_BYTES + b_bytes;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int oc0 = blockIdx.y * WS_BM;
    const int range0 = blockIdx.x * q.range_len;
    const int range1 = min(range0 + q.range_len, q.P);
    const int stages = q.stages;

    auto make_tile = [&](int p0) {
        WsTile t;
        const int plast = min(p0 + WS_BNP, range1) - 1;
        t.vp0 = vp_of(q, p0);
        t.L = vp_of(q, plast) + ((FH - 1) * q.DH) * q.VW + (FW - 1) * q.DW - t.vp0 + 1;
        t.v_first = fdiv(t.vp0, q.dVW);
        t.rows = (int)fdiv(t.vp0 + t.L - 1, q.dVW) - t.v_first + 1;
        t.slot_base = q.PW - (t.vp0 - t.v_first * q.VW);
        return t;
    };

    if (wave >= WS_CONSUMERS / 64) {
        // =================================== producers ===================================
        const int ptid = tid - WS_CONSUMERS, pwave = wave - WS_CONSUMERS / 64;
        const int n_tiles = (range1 - range0 + WS_BNP - 1) / WS_BNP;
        const int G = n_tiles * stages;

        // gather item j of this thread: (patch slot, 16-channel half of its 32-channel row,
        // sub-chunk) = one 16-byte LDS row half, filled from 4 dword loads (4 planes of one pixel).
        // LDS offset and first plane are the same for every sub-tile; only the source offset of
        // the pixel (-1: padding, zero filled) depends on the sub-tile.
        int d_loff[MAXB], d_plane[MAXB];
#pragma unroll
        for (int j = 0; j < MAXB; ++j) {
            const int i = ptid + j * WS_PRODUCERS;
            const int h = fdiv(i, q.dL), slot = i - h * q.Lmax;  // h = ks*2 + half
            d_loff[j] = h < 2 * KS ? A_BYTES + (h * q.Lmax + slot) * 16 : -1;
            d_plane[j] = (h >> 1) * 8 + (h & 1) * 4;
        }
        auto describe = [&](const WsTile& t, int (&goff)[MAXB]) {
#pragma unroll
            for (int j = 0; j < MAXB; ++j) {
                const int i = ptid + j * WS_PRODUCERS;
                const int h = fdiv(i, q.dL), slot = i - h * q.Lmax;
                goff[j] = -1;
                if (slot < t.L && d_loff[j] >= 0) {
                    const int vp = t.vp0 + slot;
                    const int v = fdiv(vp, q.dVW), vc = vp - v * q.VW;
                    const int n = fdiv(v, q.dVH), vh = v - n * q.VH;
                    const int ih = vh - q.PH, iw = vc - q.PW;
                    if (n < q.N && (unsigned)ih < (unsigned)q.IH && (unsigned)iw < (unsigned)q.IW)
                        goff[j] = n * q.image_stride + ih * q.row_stride + iw * q.pix_stride;
                }
            }
        };

        // Loads return in issue order. Per step k the producers issue the filter loads of stage
        // k+2 (L2 hits: one step is enough) and then the activation loads of stage k+3 (first
        // touch of the data, HBM latency: two steps, kept in a ring of three register sets), then
        // wait for everything older than these and scatter the activations of stage k+1.
        v4i rb[3][MAXB];
        int gset[3][MAXB];  // source offsets the loads of each register set were made with
        int bp0 = range0, bst = 0;  // activation loads: sub-tile and stage in it
        int ast = 0, abuf = 0;      // filter loads: stage in the sub-tile, LDS buffer
        int sbuf = 0;               // LDS buffer of the next scatter
        int bgoff[MAXB];
        describe(make_tile(bp0), bgoff);

        auto issue_a = [&]() {
            int8_t* buf = lds + abuf * buf_bytes;
            // TS taps x 128 rows x 32 bytes, 1 KB (32 rows) per wave-load
            if constexpr (!(DBG & 4))
#pragma unroll
            for (int a = 0; a < A_LOADS; ++a) {
                const int c = pwave + a * (WS_PRODUCERS / 64);
                const int t = c >> 2, part = c & 3;
                const int8_t* g = q.wp + ((size_t)(ast * TS + t) * q.OCP + oc0) * KROW + part * 1024 +
                                  lane * 16;
                __builtin_amdgcn_global_load_lds(MG_GLOBAL_PTR(g), MG_LDS_PTR(buf + c * 1024), 16, 0, 0);
            }
            ast = ast + 1 == stages ? 0 : ast + 1;
            abuf = abuf == WS_NBUF - 1 ? 0 : abuf + 1;
        };
        auto issue_b = [&](auto set_c) {
            constexpr int S = decltype(set_c)::value;
            // always 4 * MAXB loads (padding items read pixel 0 and are zeroed when they are
            // written), so that the number of loads per stage is fixed. Planes past the last one
            // are clamped: they meet zero filter rows.
            const int plane0 = bst * KS * 8, last = q.C4 - 1;
            if constexpr (!(DBG & 8))
#pragma unroll
            for (int j = 0; j < MAXB; ++j) {
                gset[S][j] = bgoff[j];
                const int8_t* g = q.src + (bgoff[j] >= 0 ? bgoff[j] : 0);
                const int pl = plane0 + d_plane[j];
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    rb[S][j][c] = *(const int*)(g + (size_t)min(pl + c, last) * q.plane_stride);
            }
            if (++bst == stages) {
                bst = 0;
                bp0 += WS_BNP;
                if (bp0 < range1)
                    describe(make_tile(bp0), bgoff);
            }
        };
        auto scatter = [&](auto set_c) {
            constexpr int S = decltype(set_c)::value;
            int8_t* buf = lds + sbuf * buf_bytes;
            if constexpr (!(DBG & 16))
#pragma unroll
            for (int j = 0; j < MAXB; ++j)
                if (d_loff[j] >= 0)
                    *(v4i*)(buf + d_loff[j]) = gset[S][j] >= 0 ? rb[S][j] : v4i{0, 0, 0, 0};
            sbuf = sbuf == WS_NBUF - 1 ? 0 : sbuf + 1;
        };
        // step k = -3 .. G-1, register set S = (k + 3) % 3
        auto step = [&](int k, auto set_c) {
            constexpr int S = decltype(set_c)::value;
            if (k + 2 >= 0 && k + 2 < G)
                issue_a();
            if (k + 3 < G)
                issue_b(std::integral_constant<int, S>{});
            if (k + 1 >= 0 && k + 1 < G) {
                // allowed to be in flight: activations of stage k+2, filter of k+2, activations of k+3
                if constexpr (DBG & 64)
                    wait_vmcnt<63>();
                else if (k + 3 < G)
                    wait_vmcnt<A_LOADS + 8 * MAXB>();
                else if (k + 2 < G)
                    wait_vmcnt<A_LOADS + 4 * MAXB>();
                else
                    wait_vmcnt<0>();
                scatter(std::integral_constant<int, (S + 1) % 3>{});
            }
            lds_barrier();
        };
        for (int k = -3; k < G; k += 3) {
            step(k, std::integral_constant<int, 0>{});
            if (k + 1 < G)
                step(k + 1, std::integral_constant<int, 1>{});
            if (k + 2 < G)
                step(k + 2, std::integral_constant<int, 2>{});
        }
        return;
    }

    // ===================================== consumers =====================================
    const int wm = wave / WGN, wn = wave % WGN;
    const int kg = lane >> 5;
    int a_off[MT];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
        int r = (wm * MT + mi) * 32 + (lane & 31);
        a_off[mi] = r * KROW + (((kg ^ (r >> 3)) & 1) << 4);
    }
    // requantisation thresholds, one entry per consumer thread (hidden behind the first loads)
    int* const rq_table = (int*)(lds + WS_NBUF * buf_bytes);
    if constexpr (ACT != ACT_RT) {
        if (tid < REQUANT_TABLE_ENTRIES)
            rq_table[tid] = kernarg_rq_table(tid);
    }
    lds_barrier();  // step -3
    lds_barrier();  // step -2
    lds_barrier();  // step -1: stage 0 is in buffer 0
    int cbuf = 0;
    for (int p0 = range0; p0 < range1; p0 += WS_BNP) {
        const int plast = min(p0 + WS_BNP, range1) - 1;
        const int vp0 = vp_of(q, p0);
        int b_byte[NT];  // LDS byte offset of this lane's 16 channels at tap (0,0)
        bool col_on[NT];  // wave-uniform: the 32-pixel column has pixels of this sub-tile
#pragma unroll
        for (int ni = 0; ni < NT; ++ni) {
            const int pc = p0 + (wn * NT + ni) * 32;
            const int p = pc + (lane & 31);
            b_byte[ni] = (kg * q.Lmax + (p <= plast ? vp_of(q, p) - vp0 : 0)) * 16;
            col_on[ni] = pc <= plast;
        }
        v16i acc[MT][NT];
#pragma unroll
        for (int mi = 0; mi < MT; ++mi)
#pragma unroll
            for (int ni = 0; ni < NT; ++ni)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[mi][ni][e] = 0;

        // one stage = TS (tap, sub-chunk) steps; the LDS reads of step t+1 are issued before the
        // MFMAs of step t. COLS: 32-pixel columns of this wave that hold pixels (ragged last
        // sub-tile), wave-uniform.
        auto run_stages = [&](auto cols_c) {
            constexpr int COLS = decltype(cols_c)::value;
            for (int st = 0; st < stages; ++st) {
                const int8_t* bufA = lds + cbuf * buf_bytes;
                const int8_t* bufB = bufA + A_BYTES;
                v4i fa[2][MT], fb[2][NT];
                auto fetch = [&](auto tc) {
                    constexpr int t = decltype(tc)::value;
                    constexpr int ks = t / TAPS, tap = t % TAPS;
                    constexpr int fh = tap / FW, fw = tap % FW;
                    const int tap_off = fh * q.DH * q.VW + fw * q.DW;
                    if constexpr (DBG & 2) {
                        fa[t & 1][0] = fa[t & 1][1] = v4i{a_off[0], t, 2, 3};
                        fb[t & 1][0] = fb[t & 1][1] = v4i{b_byte[0], t, 5, 6};
                        (void)tap_off;
                        return;
                    }
#pragma unroll
                    for (int mi = 0; mi < MT; ++mi)
                        fa[t & 1][mi] = *(const v4i*)(bufA + t * (WS_BM * KROW) + a_off[mi]);
#pragma unroll
                    for (int ni = 0; ni < COLS; ++ni)
                        fb[t & 1][ni] = *(const v4i*)(bufB + ks * (q.Lmax * KROW) + b_byte[ni] + tap_off * 16);
                };
                if (COLS > 0) {
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
                            for (int mi = 0; mi < MT; ++mi) {
                                if constexpr (DBG & 1)
                                    acc[mi][ni][0] += fa[t & 1][mi][0] + fb[t & 1][ni][1];
                                else
                                    acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                            fa[t & 1][mi], fb[t & 1][ni], acc[mi][ni], 0, 0, 0);
                            }
                    });
                }
                lds_barrier();
                cbuf = cbuf == WS_NBUF - 1 ? 0 : cbuf + 1;
            }
        };
        if (col_on[1])
            run_stages(std::integral_constant<int, 2>{});
        else if (col_on[0])
            run_stages(std::integral_constant<int, 1>{});
        else
            run_stages(std::integral_constant<int, 0>{});

        // ---- epilogue. Register e of a 32x32 tile holds row 8*(e/4) + 4*(lane/32) + e%4, column
        //      lane%32: 4 consecutive registers = 4 consecutive oc of one pixel = one NCHW44 dword.
        int pix_n[NT], pix_rem[NT];
#pragma unroll
        for (int ni = 0; ni < NT; ++ni) {
            const int p = p0 + (wn * NT + ni) * 32 + (lane & 31);
            pix_n[ni] = p <= plast ? (int)fdiv(p, q.dOHW) : -1;
            pix_rem[ni] = p - pix_n[ni] * q.OHW;
        }
        if constexpr (DBG & 32) {
            if (acc[0][0][0] + acc[1][0][0] + acc[0][1][0] + acc[1][1][0] == 0x12345678)
                q.dst[0] = 1;
            continue;
        }
        static_for<MT * 4>([&](auto mc) {
            constexpr int mi = decltype(mc)::value / 4, e4 = decltype(mc)::value % 4;
            const int oc = oc0 + (wm * MT + mi) * 32 + e4 * 8 + kg * 4;
            int bv[4] = {0, 0, 0, 0};
            if (q.bias) {
                if (oc + 3 < q.OC && q.bias_vec4) {
                    const int4 t4 = *(const int4*)(q.bias + oc);
                    bv[0] = t4.x; bv[1] = t4.y; bv[2] = t4.z; bv[3] = t4.w;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (oc + e < q.OC)
                            bv[e] = q.bias[oc + e];
                }
            }
            static_for<NT>([&](auto nc) {
                constexpr int ni = decltype(nc)::value;
                if (!col_on[ni])
                    return;
                int r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int a = acc[mi][ni][e4 * 4 + e] + bv[e];
                    if constexpr (ACT == ACT_RT)
                        r[e] = requant_conv_rt(q.act, a, q.s_src, q.s_flt, q.s_dst);
                    else
                        r[e] = requant_conv_table<ACT>(a, q.rq.c, rq_table);
                }
                if (pix_n[ni] >= 0 && oc < q.OC) {
                    size_t o = ((size_t)pix_n[ni] * (q.OC >> 2) + (oc >> 2)) * q.OHW + pix_rem[ni];
                    ((uint32_t*)q.dst)[o] = pack4_perm(r[0], r[1], r[2], r[3]);
                }
            });
        });
    }
}

// ---- configurations --------------------------------------------------------------------------
#ifdef MG_WS_DEBUG
template <int... D>
static const void* ws_debug_kernel(int dbg, std::integer_sequence<int, D...>) {
    const void* k = nullptr;
    ((dbg == D ? (k = (const void*)conv_mfma_i8_ws_kernel<3, 3, 1, MEGCC_NONLINE_RELU, 4, D>) : k), ...);
    return k;
}
#endif

template <int FH, int FW, int KS, int MAXB>
static PipeConfig make_ws_config(int act, bool table_ok) {
    PipeConfig c;
    c.bm = WS_BM;
    c.bn = WS_BNP;
    c.ks = KS;
    c.maxb = MAXB;
    c.g4 = 0;
    c.threads = WS_THREADS;
    c.gather_threads = WS_PRODUCERS;
    c.nbuf = WS_NBUF;
    c.blocks_per_cu = 1;
    c.a_bytes = FH * FW * KS * c.bm * KROW;
    c.extra_lds = REQUANT_TABLE_ENTRIES * 4;
    c.fixed_lmax = 0;
    if (act == MEGCC_NONLINE_IDENTITY && table_ok)
        c.kernel = (const void*)conv_mfma_i8_ws_kernel<FH, FW, KS, MEGCC_NONLINE_IDENTITY, MAXB>;
    else if (act == MEGCC_NONLINE_RELU && table_ok)
        c.kernel = (const void*)conv_mfma_i8_ws_kernel<FH, FW, KS, MEGCC_NONLINE_RELU, MAXB>;
    else
        c.kernel = (const void*)conv_mfma_i8_ws_kernel<FH, FW, KS, ACT_RT, MAXB>;
#ifdef MG_WS_DEBUG
    if (getenv("MEGCC_WS_DBG"))
        c.kernel = ws_debug_kernel(atoi(getenv("MEGCC_WS_DBG")), std::make_integer_sequence<int, 128>{});
#endif
    return c;
}

// NCHW44 3x3 layers with at least 128 output channels
bool conv_mfma_ws_config(const ConvGeom& g, bool g4_ok, PipeConfig* c) {
    const long P = (long)g.n * g.oh * g.ow;
    (void)g4_ok;
    if (!(g.fh == 3 && g.fw == 3) || g.fmt != MEGCC_FMT_NCHW44 || g.oc < 128 || P < 8192)
        return false;
    *c = make_ws_config<3, 3, 1, 4>(g.act, requant_table_ok(g.s_src, g.s_flt, g.s_dst));
    return true;
}

}  // namespace mg
