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
//   waves 8..11 (producers): during step k they start the global loads of stage k+2 -- the
//               filter tile straight into LDS buffer (k+2) % 3 with 16-byte LDS-direct loads (no
//               registers, no LDS write instructions), the activation patch into registers --
//               and scatter the patch of stage k+1 (loaded one step earlier) into buffer
//               (k+1) % 3 as rows of 32 channels per virtual pixel.
//
// One workgroup barrier per step. A load has two steps to arrive. The stage counter runs across the
// sub-tiles of a workgroup's pixel range, so the producers are already fetching the next sub-tile
// while the consumers run the epilogue of the current one.
//
// The activation gather takes 4 dwords (4 planes of one pixel) per 16-byte LDS row half, so every
// LDS write is one conflict-free 16-byte store and padding is a zero written in place.
#include "conv_mfma_i8.h"

namespace mg {

static constexpr int ACT_RT = -1;
static constexpr int WS_CONSUMERS = 512;  // threads
static constexpr int WS_PRODUCERS = 256;
static constexpr int WS_THREADS = WS_CONSUMERS + WS_PRODUCERS;
static constexpr int WS_NBUF = 3;
static constexpr int WS_BM = 128, WS_BNP = 256;

#define MG_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define MG_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt = bits 3:0 and
// 15:14, expcnt = 6:4, lgkmcnt = 11:8)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

struct WsTile {  // activation patch of one sub-tile
    int vp0, L, v_first, rows, slot_base;
};

template <int FH, int FW, int KS, int ACT, int MAXB>
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
            d_loff[j] = h < 2 * KS ? A_BYTES + (h >> 1) * (q.Lmax * KROW) + slot * KROW +
                                             (((h ^ (slot >> 3)) & 1) << 4)
                                   : -1;
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

        v4i rb[2][MAXB];
        // cursors: (sub-tile, stage in it) of the stage being loaded and of the one being scattered
        int ip0 = range0, ist = 0, sp0 = range0, sst = 0;
        int igoff[MAXB], sgoff[MAXB];
        describe(make_tile(ip0), igoff);
#pragma unroll
        for (int j = 0; j < MAXB; ++j)
            sgoff[j] = igoff[j];
        int ibuf = 0, sbuf = 0;

        auto issue = [&](auto set_c) {
            constexpr int S = decltype(set_c)::value;
            int8_t* buf = lds + ibuf * buf_bytes;
            // filter: TS taps x 128 rows x 32 bytes, 1 KB (32 rows) per wave-load
#pragma unroll
            for (int a = 0; a < A_LOADS; ++a) {
                const int c = pwave + a * (WS_PRODUCERS / 64);
                const int t = c >> 2, part = c & 3;
                const int8_t* g = q.wp + ((size_t)(ist * TS + t) * q.OCP + oc0) * KROW + part * 1024 +
                                  lane * 16;
                __builtin_amdgcn_global_load_lds(MG_GLOBAL_PTR(g), MG_LDS_PTR(buf + c * 1024), 16, 0, 0);
            }
            // activations: always 4 * MAXB loads (padding items read pixel 0 and are zeroed when
            // they are written), so that the number of loads per stage is fixed. Planes past the
            // last one are clamped: they meet zero filter rows.
            const int plane0 = ist * KS * 8, last = q.C4 - 1;
#pragma unroll
            for (int j = 0; j < MAXB; ++j) {
                const int8_t* g = q.src + (igoff[j] >= 0 ? igoff[j] : 0);
                const int pl = plane0 + d_plane[j];
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    rb[S][j][c] = *(const int*)(g + (size_t)min(pl + c, last) * q.plane_stride);
            }
            if (++ist == stages) {
                ist = 0;
                ip0 += WS_BNP;
                if (ip0 < range1)
                    describe(make_tile(ip0), igoff);
            }
            ibuf = ibuf == WS_NBUF - 1 ? 0 : ibuf + 1;
        };
        auto scatter = [&](auto set_c) {
            constexpr int S = decltype(set_c)::value;
            int8_t* buf = lds + sbuf * buf_bytes;
#pragma unroll
            for (int j = 0; j < MAXB; ++j)
                if (d_loff[j] >= 0)
                    *(v4i*)(buf + d_loff[j]) = sgoff[j] >= 0 ? rb[S][j] : v4i{0, 0, 0, 0};
            if (++sst == stages) {
                sst = 0;
                sp0 += WS_BNP;
                if (sp0 < range1)
                    describe(make_tile(sp0), sgoff);
            }
            sbuf = sbuf == WS_NBUF - 1 ? 0 : sbuf + 1;
        };
        // step k (k = -2 .. G-1): start stage k+2, finish stage k+1, barrier
        auto step = [&](int k, auto set_c) {
            constexpr int S = decltype(set_c)::value;
            const bool more = k + 2 < G;
            if (more)
                issue(std::integral_constant<int, S>{});
            if (k + 1 >= 0 && k + 1 < G) {
                // everything but the loads just issued has arrived (loads return in order)
                if (more)
                    wait_vmcnt<A_LOADS + 4 * MAXB>();
                else
                    wait_vmcnt<0>();
                scatter(std::integral_constant<int, S ^ 1>{});
            }
            lds_barrier();
        };
        for (int k = -2; k < G; k += 2) {
            step(k, std::integral_constant<int, 0>{});
            if (k + 1 < G)
                step(k + 1, std::integral_constant<int, 1>{});
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
    lds_barrier();  // step -2
    lds_barrier();  // step -1: stage 0 is in buffer 0
    int cbuf = 0;
    for (int p0 = range0; p0 < range1; p0 += WS_BNP) {
        const int plast = min(p0 + WS_BNP, range1) - 1;
        const int vp0 = vp_of(q, p0);
        int b_slot[NT];
        bool col_on[NT];  // wave-uniform: the 32-pixel column has pixels of this sub-tile
#pragma unroll
        for (int ni = 0; ni < NT; ++ni) {
            const int pc = p0 + (wn * NT + ni) * 32;
            const int p = pc + (lane & 31);
            b_slot[ni] = p <= plast ? vp_of(q, p) - vp0 : 0;
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
#pragma unroll
                    for (int mi = 0; mi < MT; ++mi)
                        fa[t & 1][mi] = *(const v4i*)(bufA + t * (WS_BM * KROW) + a_off[mi]);
#pragma unroll
                    for (int ni = 0; ni < COLS; ++ni) {
                        const int s = b_slot[ni] + tap_off;
                        fb[t & 1][ni] = *(const v4i*)(bufB + ks * (q.Lmax * KROW) + s * KROW +
                                                      (((kg ^ (s >> 3)) & 1) << 4));
                    }
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
                            for (int mi = 0; mi < MT; ++mi)
                                acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                        fa[t & 1][mi], fb[t & 1][ni], acc[mi][ni], 0, 0, 0);
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
                int r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int a = acc[mi][ni][e4 * 4 + e] + bv[e];
                    if constexpr (ACT == ACT_RT)
                        r[e] = requant_conv_rt(q.act, a, q.s_src, q.s_flt, q.s_dst);
                    else
                        r[e] = requant_conv_fast<ACT>(a, q.rq);
                }
                if (pix_n[ni] >= 0 && oc < q.OC) {
                    size_t o = ((size_t)pix_n[ni] * (q.OC >> 2) + (oc >> 2)) * q.OHW + pix_rem[ni];
                    ((uint32_t*)q.dst)[o] = pack4(r[0], r[1], r[2], r[3]);
                }
            });
        });
    }
}

// ---- configurations --------------------------------------------------------------------------
template <int FH, int FW, int KS, int MAXB>
static PipeConfig make_ws_config(int act) {
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
    if (act == MEGCC_NONLINE_IDENTITY)
        c.kernel = (const void*)conv_mfma_i8_ws_kernel<FH, FW, KS, MEGCC_NONLINE_IDENTITY, MAXB>;
    else if (act == MEGCC_NONLINE_RELU)
        c.kernel = (const void*)conv_mfma_i8_ws_kernel<FH, FW, KS, MEGCC_NONLINE_RELU, MAXB>;
    else
        c.kernel = (const void*)conv_mfma_i8_ws_kernel<FH, FW, KS, ACT_RT, MAXB>;
    return c;
}

// NCHW44 3x3 layers with at least 128 output channels
bool conv_mfma_ws_config(const ConvGeom& g, bool g4_ok, PipeConfig* c) {
    const long P = (long)g.n * g.oh * g.ow;
    (void)g4_ok;
    if (!(g.fh == 3 && g.fw == 3) || g.fmt != MEGCC_FMT_NCHW44 || g.oc < 128 || P < 8192)
        return false;
    *c = make_ws_config<3, 3, 1, 4>(g.act);
    return true;
}

}  // namespace mg
