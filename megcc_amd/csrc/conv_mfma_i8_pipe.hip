// Software-pipelined variant of the qsi8 implicit-GEMM convolution for large shapes
// (same arithmetic, packed filter and LDS layouts as conv_mfma_i8.hip).
//
// One workgroup of 4 waves owns a tile of BM output channels x BN pixels with BM x BN up to
// 256 x 256; every wave keeps MT x NT accumulator tiles of 32x32 int32 (up to 4 x 4 = 256
// registers), so each 16-byte operand fetched from LDS feeds 4 MFMAs and LDS traffic stays at
// half of what the matrix cores could consume.
//
// The K loop runs over "steps" = (ic-chunk of 32, tap). Per step the filter contributes one
// BM x 32-byte tile (8 KB at BM = 256) that is streamed through a ring of 3 LDS slots:
//     global -> registers   issued 2 + PD steps ahead  (PD register sets hide the L2 latency)
//     registers -> LDS      2 steps ahead
//     LDS -> MFMA operands  1 step ahead, into the second half of a register double buffer,
//                           interleaved with the MFMAs of the current step
// so that only one workgroup barrier per step is needed and nothing the matrix cores wait for is
// younger than one full step (16 MFMAs = 512 cycles per wave at the 256 x 256 tile).
// The activation patch (tile + halo, all taps) changes once per ic-chunk stage; it is gathered from
// the NCHW44 planes at the first step of the previous stage and written to the other half of a
// double buffer two steps before that stage ends.
// Barriers are "LDS only": s_waitcnt lgkmcnt(0) + s_barrier, so global loads stay in flight
// across them.
#include <utility>

#include "conv_mfma_i8.h"

namespace mg {

// compile-time loop: f(std::integral_constant<int, 0>) ... f(<N-1>), so that every register-array
// index derived from the counter is a constant whatever the unroller decides
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// workgroup barrier that orders LDS traffic only (no wait for outstanding global loads)
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

static constexpr int ACT_RUNTIME = -1;

// ACT: MEGCC_NONLINE_IDENTITY / MEGCC_NONLINE_RELU compile the epilogue for that activation;
// ACT_RUNTIME selects by q.act per element (H_SWISH, SIGMOID).
template <int WGM, int WGN, int MT, int NT, int FH, int FW, int KS, int PD, int MAXB, int ACT, int MINB>
__global__ void __launch_bounds__(THREADS, MINB) conv_mfma_i8_pipe_kernel(MfmaParams q) {
    constexpr int BM = WGM * MT * 32;
    constexpr int BNP = WGN * NT * 32;
    constexpr int TAPS = FH * FW;
    constexpr int TS = TAPS * KS;  // steps per stage
    constexpr int RING = 3;
    constexpr int A_TILE = BM * KROW;
    constexpr int A_CHUNKS = A_TILE / 16;
    constexpr int A_ITEMS = (A_CHUNKS + THREADS - 1) / THREADS;
    static_assert(TS % PD == 0, "register-set index must be static");
    static_assert(WGM * WGN == 4, "4 waves");

    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    int8_t* ringA = lds;
    const int b_buf_bytes = KS * q.Lmax * KROW;
    int8_t* ldsB = lds + RING * A_TILE;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int oc0 = blockIdx.y * BM;
    const int kg = lane >> 5;
    const int S = q.stages * TS;  // total steps

    int a_off[MT];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
        int r = (wm * MT + mi) * 32 + (lane & 31);
        a_off[mi] = r * KROW + (((kg ^ (r >> 3)) & 1) << 4);
    }

    // this workgroup's share of the pixels, walked in sub-tiles of BNP
    const int range0 = blockIdx.x * q.range_len;
    const int range1 = min(range0 + q.range_len, q.P);

    for (int p0 = range0; p0 < range1; p0 += BNP) {
        const int plast = min(p0 + BNP, range1) - 1;
        const int vp0 = vp_of(q, p0);
        const int L = vp_of(q, plast) + ((FH - 1) * q.DH) * q.VW + (FW - 1) * q.DW - vp0 + 1;

        // ---- gather items of this thread (see conv_mfma_i8.hip)
        int b_goff[MAXB], b_loff[MAXB], b_plane[MAXB];
        const int n_items = 2 * KS * q.Lmax;
#pragma unroll
        for (int j = 0; j < MAXB; ++j) {
            int i = tid + j * THREADS;
            b_goff[j] = -1;
            b_loff[j] = -1;
            b_plane[j] = 0;
            if (i < n_items) {
                int h = fdiv(i, q.dL), slot = i - h * q.Lmax;
                b_loff[j] = (h >> 1) * (q.Lmax * KROW) + slot * KROW + (((h ^ (slot >> 3)) & 1) << 4);
                b_plane[j] = (h >> 1) * 8 + (h & 1) * 4;
                if (slot < L) {
                    int vp = vp0 + slot;
                    int v = fdiv(vp, q.dVW), vc = vp - v * q.VW;
                    int n = fdiv(v, q.dVH), vh = v - n * q.VH;
                    int ih = vh - q.PH, iw = vc - q.PW;
                    if (n < q.N && (unsigned)ih < (unsigned)q.IH && (unsigned)iw < (unsigned)q.IW)
                        b_goff[j] = n * q.image_stride + ih * q.row_stride + iw * q.pix_stride;
                }
            }
        }
        int b_slot[NT];
#pragma unroll
        for (int ni = 0; ni < NT; ++ni) {
            int p = p0 + (wn * NT + ni) * 32 + (lane & 31);
            b_slot[ni] = p <= plast ? vp_of(q, p) - vp0 : 0;
        }

        v16i acc[MT][NT];
#pragma unroll
        for (int mi = 0; mi < MT; ++mi)
#pragma unroll
            for (int ni = 0; ni < NT; ++ni)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[mi][ni][e] = 0;

        v4i ra[PD][A_ITEMS];
        v4i rb[MAXB];
        v4i fa[2][MT], fb[2][NT];

        // filter tile of step x: global -> registers (set x % PD)
        auto load_a = [&](int x, v4i (&r)[A_ITEMS]) {
            const int8_t* base = q.wp + ((size_t)x * q.OCP + oc0) * KROW;
#pragma unroll
            for (int j = 0; j < A_ITEMS; ++j) {
                int c = tid + j * THREADS;
                if (A_CHUNKS % THREADS == 0 || c < A_CHUNKS)
                    r[j] = *(const v4i*)(base + c * 16);
            }
        };
        auto store_a = [&](int x, const v4i (&r)[A_ITEMS]) {
            int8_t* dst = ringA + (x % RING) * A_TILE;
#pragma unroll
            for (int j = 0; j < A_ITEMS; ++j) {
                int c = tid + j * THREADS;
                if (A_CHUNKS % THREADS == 0 || c < A_CHUNKS)
                    *(v4i*)(dst + c * 16) = r[j];
            }
        };
        auto load_b = [&](int st) {
            const int plane0 = st * KS * 8;
            const int last = q.C4 - 1;
#pragma unroll
            for (int j = 0; j < MAXB; ++j) {
                // branch-free: padding pixels read pixel 0 and are zeroed by a select; planes past
                // the last one are clamped (they meet zero filter rows: their value is irrelevant)
                const bool ok = b_goff[j] >= 0;
                const int8_t* g = q.src + (ok ? b_goff[j] : 0);
                const int pl = plane0 + b_plane[j];
                v4i v;
                v[0] = *(const int*)(g + (size_t)min(pl + 0, last) * q.plane_stride);
                v[1] = *(const int*)(g + (size_t)min(pl + 1, last) * q.plane_stride);
                v[2] = *(const int*)(g + (size_t)min(pl + 2, last) * q.plane_stride);
                v[3] = *(const int*)(g + (size_t)min(pl + 3, last) * q.plane_stride);
                rb[j] = ok ? v : v4i{0, 0, 0, 0};
            }
        };
        auto store_b = [&](int st) {
            int8_t* dst = ldsB + (st & 1) * b_buf_bytes;
#pragma unroll
            for (int j = 0; j < MAXB; ++j)
                if (b_loff[j] >= 0)
                    *(v4i*)(dst + b_loff[j]) = rb[j];
        };
        // MFMA operands of step (st, t): LDS -> registers
        auto load_frags = [&](int st, int t, int x, v4i (&a)[MT], v4i (&b)[NT]) {
            const int ks = t / TAPS, tap = t % TAPS;
            const int fh = tap / FW, fw = tap % FW;
            const int tap_off = fh * q.DH * q.VW + fw * q.DW;
            const int8_t* as = ringA + (x % RING) * A_TILE;
            const int8_t* bs = ldsB + (st & 1) * b_buf_bytes + ks * (q.Lmax * KROW);
#pragma unroll
            for (int ni = 0; ni < NT; ++ni) {
                int s = b_slot[ni] + tap_off;
                b[ni] = *(const v4i*)(bs + s * KROW + (((kg ^ (s >> 3)) & 1) << 4));
            }
#pragma unroll
            for (int mi = 0; mi < MT; ++mi)
                a[mi] = *(const v4i*)(as + a_off[mi]);
        };

        // ---- prologue: steps 0 and 1 of the filter and stage 0 of the patch into LDS,
        //      steps 2 .. 2+PD-1 of the filter into the register sets
        lds_barrier();  // the previous sub-tile's last operands have been consumed
        load_b(0);
        load_a(0, ra[0]);
        if (1 < S)
            load_a(1, ra[1 % PD]);
        store_a(0, ra[0]);
        if (1 < S)
            store_a(1, ra[1 % PD]);
        store_b(0);
#pragma unroll
        for (int d = 0; d < PD; ++d)
            if (2 + d < S)
                load_a(2 + d, ra[(2 + d) % PD]);
        lds_barrier();
        load_frags(0, 0, 0, fa[0], fb[0]);

        for (int st = 0; st < q.stages; ++st) {
            static_for<TS>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                const int x = st * TS + t;  // this step
                constexpr int cur = t & 1, nxt = cur ^ 1;
                // 1. filter tile two steps ahead: registers -> LDS, then refill that register set
                if (x + 2 < S) {
                    store_a(x + 2, ra[(t + 2) % PD]);
                    if (x + 2 + PD < S)
                        load_a(x + 2 + PD, ra[(t + 2) % PD]);
                }
                // 2. patch of the next stage
                if (t == 0 && st + 1 < q.stages)
                    load_b(st + 1);
                if (t == (TS >= 2 ? TS - 2 : 0) && st + 1 < q.stages)
                    store_b(st + 1);
                // 3. operands of the next step (visible since the barrier of the previous step)
                if (x + 1 < S) {
                    constexpr int nt = (t + 1) % TS;
                    const int nst = st + (t + 1 == TS ? 1 : 0);
                    load_frags(nst, nt, x + 1, fa[nxt], fb[nxt]);
                }
                // 4. this step's MFMAs
#pragma unroll
                for (int mi = 0; mi < MT; ++mi)
#pragma unroll
                    for (int ni = 0; ni < NT; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                fa[cur][mi], fb[cur][ni], acc[mi][ni], 0, 0, 0);
                lds_barrier();
            });
            if (TS & 1) {
                // odd number of steps per stage: the operands prefetched for the next stage's
                // first step sit in buffer 1, the unrolled body expects them in buffer 0
#pragma unroll
                for (int mi = 0; mi < MT; ++mi)
                    fa[0][mi] = fa[1][mi];
#pragma unroll
                for (int ni = 0; ni < NT; ++ni)
                    fb[0][ni] = fb[1][ni];
            }
        }

        // ---- epilogue. Register e of a 32x32 tile holds row 8*(e/4) + 4*(lane/32) + e%4, column
        //      lane%32: 4 consecutive registers = 4 consecutive oc of one pixel = one NCHW44
        //      dword. All bias values of the lane's rows are fetched first; the per-element code
        //      is straight-line (the activation is a template parameter).
        int bv[MT * 4][4];
#pragma unroll
        for (int g4 = 0; g4 < MT * 4; ++g4) {
            const int oc = oc0 + (wm * MT + g4 / 4) * 32 + (g4 % 4) * 8 + kg * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                bv[g4][e] = 0;
            if (q.bias) {
                if (oc + 3 < q.OC && q.bias_vec4) {
                    const int4 t4 = *(const int4*)(q.bias + oc);
                    bv[g4][0] = t4.x; bv[g4][1] = t4.y; bv[g4][2] = t4.z; bv[g4][3] = t4.w;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (oc + e < q.OC)
                            bv[g4][e] = q.bias[oc + e];
                }
            }
        }
        static_for<NT>([&](auto nc) {
            constexpr int ni = decltype(nc)::value;
            const int p = p0 + (wn * NT + ni) * 32 + (lane & 31);
            if (p <= plast) {
                const int n = fdiv(p, q.dOHW), rem = p - n * q.OHW;
                uint32_t* out44 = (uint32_t*)q.dst + (size_t)n * (q.OC >> 2) * q.OHW + rem;
                static_for<MT * 4>([&](auto mc) {
                    constexpr int g4 = decltype(mc)::value;
                    constexpr int mi = g4 / 4, e4 = g4 % 4;
                    const int oc = oc0 + (wm * MT + mi) * 32 + e4 * 8 + kg * 4;
                    int r[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int a = acc[mi][ni][e4 * 4 + e] + bv[g4][e];
                        if (ACT == ACT_RUNTIME)
                            r[e] = requant_conv_rt(q.act, a, q.s_src, q.s_flt, q.s_dst);
                        else
                            r[e] = requant_conv<ACT>(a, q.s_src, q.s_flt, q.s_dst);
                    }
                    if (!q.dst_fc) {
                        if (oc < q.OC)
                            out44[(size_t)(oc >> 2) * q.OHW] = pack4(r[0], r[1], r[2], r[3]);
                    } else {
                        int8_t* o = q.dst + (size_t)p * q.OC + oc;
                        if ((q.OC & 3) == 0) {
                            if (oc < q.OC)
                                *(uint32_t*)o = pack4(r[0], r[1], r[2], r[3]);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (oc + e < q.OC)
                                    o[e] = (int8_t)r[e];
                        }
                    }
                });
            }
        });
    }
}

// ---- configurations --------------------------------------------------------------------------
template <int WGM, int WGN, int MT, int NT, int FH, int FW, int KS, int PD, int MAXB, int MINB>
static PipeConfig make_config(int act) {
    PipeConfig c;
    c.bm = WGM * MT * 32;
    c.bn = WGN * NT * 32;
    c.ks = KS;
    c.maxb = MAXB;
    c.blocks_per_cu = MINB;
    if (act == MEGCC_NONLINE_IDENTITY)
        c.kernel = (const void*)conv_mfma_i8_pipe_kernel<WGM, WGN, MT, NT, FH, FW, KS, PD, MAXB,
                                                         MEGCC_NONLINE_IDENTITY, MINB>;
    else if (act == MEGCC_NONLINE_RELU)
        c.kernel = (const void*)conv_mfma_i8_pipe_kernel<WGM, WGN, MT, NT, FH, FW, KS, PD, MAXB,
                                                         MEGCC_NONLINE_RELU, MINB>;
    else
        c.kernel = (const void*)conv_mfma_i8_pipe_kernel<WGM, WGN, MT, NT, FH, FW, KS, PD, MAXB,
                                                         ACT_RUNTIME, MINB>;
    return c;
}

// Picks the tile for (filter size, oc); returns false when the shape is better served by the
// one-stage kernel (small problems, filter sizes other than 1x1 and 3x3).
bool conv_mfma_pipe_config(const ConvGeom& g, PipeConfig* c) {
    const long P = (long)g.n * g.oh * g.ow;
    const bool k3 = g.fh == 3 && g.fw == 3, k1 = g.fh == 1 && g.fw == 1;
    if (!(k3 || k1) || g.oc < 128 || P < 8192)
        return false;
    // 128 oc x 256 pixels per workgroup, 128 accumulator registers per lane, 2 workgroups per CU
    *c = k3 ? make_config<2, 2, 2, 4, 3, 3, 1, 3, 4, 2>(g.act)
            : make_config<2, 2, 2, 4, 1, 1, 4, 4, 8, 2>(g.act);
    return true;
}

TinyNNStatus conv_mfma_pipe_launch(const PipeConfig& c, MfmaParams q) {
    const size_t lds = (size_t)3 * c.bm * KROW + 2 * (size_t)c.ks * q.Lmax * KROW;
    MG_REQUIRE(lds <= 160 * 1024, TinyNN_ERROR_OUT_OF_RANGE, "conv_mfma_pipe: %zu bytes of LDS", lds);
    MG_REQUIRE(2L * c.ks * q.Lmax <= (long)c.maxb * THREADS, TinyNN_ERROR_OUT_OF_RANGE,
               "conv_mfma_pipe: patch of %d slots exceeds the gather registers", q.Lmax);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(c.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_mfma_pipe: LDS attribute: %s",
                   hipGetErrorString(e));
    }
    dim3 grid((q.P + q.range_len - 1) / q.range_len, (q.OC + c.bm - 1) / c.bm);
    void* args[] = {&q};
    hipError_t e = hipLaunchKernel(c.kernel, grid, dim3(THREADS), args, lds, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_mfma_pipe: launch: %s", hipGetErrorString(e));
    return check_launch("conv_mfma_i8_pipe");
}

}  // namespace mg
