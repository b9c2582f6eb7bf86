// Wide-tile variant of the qsi8 implicit-GEMM convolution for large shapes (same arithmetic,
// packed filter and LDS layouts as conv_mfma_i8.hip).
//
// Why a second kernel: the filter and activation tiles reach LDS through the CU's vector memory
// path, which moves 64 bytes per clock, while the four matrix cores of a CU consume a
// 128 oc x 128 pixel x 32 ic step in 128 clocks. A 128 x 128 tile therefore needs 42 bytes/clock
// of L2->LDS traffic to keep the MFMAs busy (two thirds of what the path can deliver, measured as
// the limiter of conv_mfma_i8.hip on 256-channel layers); a 128 x 256 tile needs 21.
//
// One workgroup = 8 waves (2 per SIMD) in a 2 x 4 grid over a 128 oc x 256 pixel tile, 64 int32
// accumulators per lane, so the register budget of two waves per SIMD holds without spilling.
// LDS is double buffered per ic-chunk stage (filter: all taps of the stage; activations: the
// tile's pixels + halo): while stage s is multiplied out of buffer s&1, the global loads of stage
// s+1 are in flight into registers and are written to the other buffer at the end of the stage.
// One workgroup barrier per stage, and it orders LDS traffic only (s_waitcnt lgkmcnt(0) +
// s_barrier), so the loads of the next stage stay in flight across it.
//
// Work distribution: the pixels are cut into as many contiguous ranges as there are workgroup
// slots on the chip (CUs / oc-tiles), each workgroup walks its range in sub-tiles of 256 pixels:
// the whole grid is resident at once and all CUs finish together instead of leaving a partial
// last round.
#include "conv_mfma_i8.h"

namespace mg {

static constexpr int ACT_RT = -1;
static constexpr int WTHREADS = 512;

// FH x FW: 3x3 or 1x1 (taps unrolled); KS: 32-channel sub-chunks per stage.
// ACT: MEGCC_NONLINE_IDENTITY / _RELU compile the epilogue for that activation, ACT_RT selects by
// q.act per element.
//
// G4 selects how the activation patch is gathered from the NCHW44 planes:
//   G4 = false: one dword (4 channels of one pixel) per lane and load, 4 loads -> one 16-byte LDS
//               write; works for any layout the one-stage kernel accepts.
//   G4 = true : one 16-byte load = 4 horizontally adjacent pixels x 4 channels of one plane,
//               scattered as four dword LDS writes (a quarter of the load instructions); needs
//               IW % 4 == 0 and a 16-byte aligned source. Padding slots are never written by
//               the gather: they are zeroed once per sub-tile.
template <int WGM, int WGN, int MT, int NT, int FH, int FW, int KS, int ACT, bool G4, int MAXB>
__global__ void __launch_bounds__(WTHREADS) conv_mfma_i8_wide_kernel(MfmaParams q) {
    constexpr int BM = WGM * MT * 32;
    constexpr int BNP = WGN * NT * 32;
    constexpr int TAPS = FH * FW;
    constexpr int TS = TAPS * KS;
    constexpr int A_BYTES = TS * BM * KROW;
    constexpr int A_CHUNKS = A_BYTES / 16;
    constexpr int A_ITEMS = (A_CHUNKS + WTHREADS - 1) / WTHREADS;
    static_assert(WGM * WGN * 64 == WTHREADS, "8 waves");

    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    const int b_bytes = KS * q.Lmax * KROW;
    const int buf_bytes = A_BYTES + b_bytes;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int oc0 = blockIdx.y * BM;
    const int kg = lane >> 5;

    int a_off[MT];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
        int r = (wm * MT + mi) * 32 + (lane & 31);
        a_off[mi] = r * KROW + (((kg ^ (r >> 3)) & 1) << 4);
    }

    const int range0 = blockIdx.x * q.range_len;
    const int range1 = min(range0 + q.range_len, q.P);

    for (int p0 = range0; p0 < range1; p0 += BNP) {
        const int plast = min(p0 + BNP, range1) - 1;
        const int vp0 = vp_of(q, p0);
        const int L = vp_of(q, plast) + ((FH - 1) * q.DH) * q.VW + (FW - 1) * q.DW - vp0 + 1;

        // ---- gather items of this thread
        int b_goff[MAXB], b_loff[MAXB], b_plane[MAXB];
        if (!G4) {
            // (patch slot, 16-byte half of a 32-channel row, sub-chunk), see conv_mfma_i8.hip
            const int n_items = 2 * KS * q.Lmax;
#pragma unroll
            for (int j = 0; j < MAXB; ++j) {
                int i = tid + j * WTHREADS;
                b_goff[j] = -1;
                b_loff[j] = -1;
                b_plane[j] = 0;
                if (i < n_items) {
                    int h = fdiv(i, q.dL), slot = i - h * q.Lmax;
                    b_loff[j] = A_BYTES + (h >> 1) * (q.Lmax * KROW) + slot * KROW +
                                (((h ^ (slot >> 3)) & 1) << 4);
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
        } else {
            // (plane of the stage, patch row, group of 4 pixels): b_goff = byte offset of the
            // group in plane 0 (-1: no such item / padding row), b_loff = patch slot of its first
            // pixel (may be negative at the ragged start of the patch), b_plane = plane in stage
            const int v_first = fdiv(vp0, q.dVW);
            const int rows = (int)fdiv(vp0 + L - 1, q.dVW) - v_first + 1;
            const int slot_base = q.PW - (vp0 - v_first * q.VW);
#pragma unroll
            for (int j = 0; j < MAXB; ++j) {
                int i = tid + j * WTHREADS;
                int pl = fdiv(i, q.dRG), rem = i - pl * q.RG;
                int r = fdiv(rem, q.dG), g4 = rem - r * q.G;
                b_goff[j] = -1;
                b_plane[j] = pl;
                b_loff[j] = r * q.VW + slot_base + 4 * g4;
                if (pl < KS * 8 && r < rows) {
                    int v = v_first + r;
                    int n = fdiv(v, q.dVH), vh = v - n * q.VH;
                    int ih = vh - q.PH;
                    if (n < q.N && (unsigned)ih < (unsigned)q.IH)
                        b_goff[j] = n * q.image_stride + ih * q.row_stride + g4 * 16;
                }
            }
            // padding slots stay zero for the whole sub-tile, in both buffers
            const v4i zero = {0, 0, 0, 0};
            for (int i = tid; i < b_bytes / 16; i += WTHREADS) {
                *(v4i*)(lds + A_BYTES + i * 16) = zero;
                *(v4i*)(lds + buf_bytes + A_BYTES + i * 16) = zero;
            }
            lds_barrier();
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

        v4i ra[A_ITEMS];
        v4i rb[MAXB];

        auto prefetch = [&](int st) {
#pragma unroll
            for (int j = 0; j < A_ITEMS; ++j) {
                int i = tid + j * WTHREADS;
                if (A_CHUNKS % WTHREADS == 0 || i < A_CHUNKS) {
                    int t = i / (BM * 2), c = i - t * (BM * 2);
                    ra[j] = *(const v4i*)(q.wp + ((size_t)(st * TS + t) * q.OCP + oc0) * KROW + c * 16);
                }
            }
            const int plane0 = st * KS * 8;
            const int last = q.C4 - 1;
#pragma unroll
            for (int j = 0; j < MAXB; ++j) {
                if (G4) {
                    // planes past the last one are clamped: they meet zero filter rows
                    if (b_goff[j] >= 0)
                        rb[j] = *(const v4i*)(q.src + b_goff[j] +
                                                   (size_t)min(plane0 + b_plane[j], last) * q.plane_stride);
                } else {
                    // whole waves have no item j (wave-uniform branch); inside an item the loads
                    // are branch-free: padding pixels read pixel 0 and are zeroed by a select
                    if (b_loff[j] < 0)
                        continue;
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
            }
        };
        auto stage_to_lds = [&](int st) {
            int8_t* buf = lds + (st & 1) * buf_bytes;
#pragma unroll
            for (int j = 0; j < A_ITEMS; ++j) {
                int i = tid + j * WTHREADS;
                if (A_CHUNKS % WTHREADS == 0 || i < A_CHUNKS)
                    *(v4i*)(buf + i * 16) = ra[j];
            }
#pragma unroll
            for (int j = 0; j < MAXB; ++j) {
                if (G4) {
                    if (b_goff[j] >= 0) {
                        const int pl = b_plane[j];
                        int8_t* row = buf + A_BYTES + (pl >> 3) * (q.Lmax * KROW) + (pl & 3) * 4;
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const int slot = b_loff[j] + k;
                            if ((unsigned)slot < (unsigned)L)
                                *(int*)(row + slot * KROW + ((((pl >> 2) ^ (slot >> 3)) & 1) << 4)) =
                                        rb[j][k];
                        }
                    }
                } else if (b_loff[j] >= 0) {
                    *(v4i*)(buf + b_loff[j]) = rb[j];
                }
            }
        };
        auto compute = [&](int st) {
            const int8_t* bufA = lds + (st & 1) * buf_bytes;
            const int8_t* bufB = bufA + A_BYTES;
            static_for<TS>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                constexpr int ks = t / TAPS, tap = t % TAPS;
                constexpr int fh = tap / FW, fw = tap % FW;
                const int tap_off = fh * q.DH * q.VW + fw * q.DW;
                v4i a[MT], b[NT];
#pragma unroll
                for (int mi = 0; mi < MT; ++mi)
                    a[mi] = *(const v4i*)(bufA + t * (BM * KROW) + a_off[mi]);
#pragma unroll
                for (int ni = 0; ni < NT; ++ni) {
                    int s = b_slot[ni] + tap_off;
                    b[ni] = *(const v4i*)(bufB + ks * (q.Lmax * KROW) + s * KROW +
                                          (((kg ^ (s >> 3)) & 1) << 4));
                }
#pragma unroll
                for (int mi = 0; mi < MT; ++mi)
#pragma unroll
                    for (int ni = 0; ni < NT; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                a[mi], b[ni], acc[mi][ni], 0, 0, 0);
            });
        };
        prefetch(0);
        stage_to_lds(0);
        lds_barrier();

        for (int st = 0; st < q.stages; ++st) {
            if (st + 1 < q.stages)
                prefetch(st + 1);
            compute(st);
            if (st + 1 < q.stages)
                stage_to_lds(st + 1);
            lds_barrier();
        }

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
                    if (!q.dst_fc) {
                        size_t o = ((size_t)pix_n[ni] * (q.OC >> 2) + (oc >> 2)) * q.OHW + pix_rem[ni];
                        ((uint32_t*)q.dst)[o] = pack4(r[0], r[1], r[2], r[3]);
                    } else {
                        const int p = p0 + (wn * NT + ni) * 32 + (lane & 31);
                        int8_t* o = q.dst + (size_t)p * q.OC + oc;
                        if ((q.OC & 3) == 0) {
                            *(uint32_t*)o = pack4(r[0], r[1], r[2], r[3]);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (oc + e < q.OC)
                                    o[e] = (int8_t)r[e];
                        }
                    }
                }
            });
        });
    }
}

// ---- configurations --------------------------------------------------------------------------
template <int WGM, int WGN, int MT, int NT, int FH, int FW, int KS, bool G4, int MAXB>
static PipeConfig make_config(int act) {
    PipeConfig c;
    c.bm = WGM * MT * 32;
    c.bn = WGN * NT * 32;
    c.ks = KS;
    c.maxb = MAXB;
    c.g4 = G4;
    c.threads = WTHREADS;
    c.gather_threads = WTHREADS;
    c.nbuf = 2;
    c.extra_lds = 0;
    c.fixed_lmax = 0;
    c.blocks_per_cu = 1;
    c.a_bytes = FH * FW * KS * c.bm * KROW;
    if (act == MEGCC_NONLINE_IDENTITY)
        c.kernel = (const void*)conv_mfma_i8_wide_kernel<WGM, WGN, MT, NT, FH, FW, KS,
                                                         MEGCC_NONLINE_IDENTITY, G4, MAXB>;
    else if (act == MEGCC_NONLINE_RELU)
        c.kernel = (const void*)conv_mfma_i8_wide_kernel<WGM, WGN, MT, NT, FH, FW, KS,
                                                         MEGCC_NONLINE_RELU, G4, MAXB>;
    else
        c.kernel = (const void*)conv_mfma_i8_wide_kernel<WGM, WGN, MT, NT, FH, FW, KS, ACT_RT, G4, MAXB>;
    return c;
}

// Picks the tile for (filter size, oc); returns false when the shape is better served by the
// one-stage kernel (small problems, filter sizes other than 1x1 and 3x3). `g4_ok`: the source
// allows 16-byte gathers (NCHW44, IW % 4 == 0, 16-byte aligned).
bool conv_mfma_pipe_config(const ConvGeom& g, bool g4_ok, PipeConfig* c) {
    const long P = (long)g.n * g.oh * g.ow;
    const bool k3 = g.fh == 3 && g.fw == 3, k1 = g.fh == 1 && g.fw == 1;
    if (!(k3 || k1) || g.oc < 128 || P < 8192)
        return false;
    if (k3)
        *c = g4_ok ? make_config<2, 4, 2, 2, 3, 3, 1, true, 3>(g.act)
                   : make_config<2, 4, 2, 2, 3, 3, 1, false, 2>(g.act);
    else
        *c = g4_ok ? make_config<2, 4, 2, 2, 1, 1, 4, true, 7>(g.act)
                   : make_config<2, 4, 2, 2, 1, 1, 4, false, 4>(g.act);
    return true;
}

TinyNNStatus conv_mfma_pipe_launch(const PipeConfig& c, MfmaParams q) {
    const size_t lds = c.nbuf * ((size_t)c.a_bytes + (size_t)c.ks * q.Lmax * KROW) + c.extra_lds;
    MG_REQUIRE(lds <= 160 * 1024, TinyNN_ERROR_OUT_OF_RANGE, "conv_mfma_wide: %zu bytes of LDS", lds);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(c.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_mfma_wide: LDS attribute: %s",
                   hipGetErrorString(e));
    }
    dim3 grid((q.P + q.range_len - 1) / q.range_len, (q.OC + c.bm - 1) / c.bm);
    void* args[] = {&q};
    hipError_t e = hipLaunchKernel(c.kernel, grid, dim3(c.threads), args, lds, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_mfma_wide: launch: %s", hipGetErrorString(e));
    return check_launch("conv_mfma_i8_wide");
}

}  // namespace mg
