// qsi8 dense convolution / FullyConnected as an implicit GEMM on the gfx950 matrix cores
// (v_mfma_i32_32x32x32_i8): rows = output channels, columns = output pixels, K = (tap, ic).
//
// Replaces, for format NCHW44 + sparse DENSE and for the 1x1 NCHW convolution on [M,K,1,1] that
// MegCC uses as quantized FullyConnected, the scalar seven-deep loop of BareMetal::ConvGeneral
// (compiler/lib/KernelGen/BareMetal/ConvKernel.cpp:305-344). int8 x int8 products are summed
// exactly in int32, so any summation order gives the reference's accumulator; the epilogue is the
// reference's float sequence (epilogue.h).
//
// Data movement per workgroup (256 threads = 4 waves in a 2x2 grid, tile BM oc x 128 pixels):
//   * the filter is pre-packed once by the _init entry point into rows of 32 consecutive input
//     channels per (ic-chunk, tap, oc): a tile is a straight 16-byte-vector copy into LDS;
//   * the activations needed by ALL taps of the tile (the tile's pixels plus their halo, in a
//     zero-padded "virtual" image) are gathered once per ic-chunk from the NCHW44 planes into LDS
//     rows of 32 channels per pixel -- im2col happens only as an LDS address offset per tap, and
//     padding is a predicated zero at load time, so there is no workspace and no 9x re-read;
//   * both LDS tiles swap the two 16-byte halves of a row on every other group of 8 rows, which
//     makes the 64-lane ds_read_b128 of an MFMA operand (stride 32 bytes between lanes) hit every
//     bank once;
//   * the MFMA result layout (lane = pixel, 4 consecutive registers = 4 consecutive oc) is exactly
//     one NCHW44 dword per pixel, so 32 lanes store 128 contiguous bytes.
#include <stdlib.h>

#include <array>
#include <map>
#include <mutex>

#include "conv_mfma_i8.h"

namespace mg {

static constexpr int ACT_RUNTIME = -1;

// ACT: MEGCC_NONLINE_IDENTITY / MEGCC_NONLINE_RELU compile the epilogue for that activation;
// ACT_RUNTIME selects by q.act per element (H_SWISH, SIGMOID).
template <int BM, int ACT>
__global__ void __launch_bounds__(THREADS) conv_mfma_i8_kernel(MfmaParams q) {
    constexpr int WM = BM / 2;          // rows per wave
    constexpr int MT = WM / 32;         // 32x32 tiles per wave along oc
    constexpr int NT = 2;               // 64 pixels per wave
    constexpr int A_ROW_CHUNKS = BM * 2;  // 16-byte chunks per tap
    constexpr int MAX_A_ITEMS = (MAX_TAPS_STAGE * A_ROW_CHUNKS + THREADS - 1) / THREADS;

    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    const int taps_stage = q.taps * q.KS;
    int8_t* ldsA = lds;
    int8_t* ldsB = lds + taps_stage * BM * KROW;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int p0 = blockIdx.x * BN, oc0 = blockIdx.y * BM;
    const int plast = min(p0 + BN, q.P) - 1;
    const int vp0 = vp_of(q, p0);
    const int L = vp_of(q, plast) + ((q.FH - 1) * q.DH) * q.VW + (q.FW - 1) * q.DW - vp0 + 1;

    // ---- gather items of this thread: (patch slot, 16-byte half of a 32-channel row, sub-chunk)
    int b_goff[MAX_B_ITEMS];   // byte offset of the pixel in plane 0 of its image, -1 = zero fill
    int b_loff[MAX_B_ITEMS];   // LDS byte offset of the 16-byte destination, -1 = no item
    int b_plane[MAX_B_ITEMS];  // first of the 4 planes, relative to the stage
    const int n_items = 2 * q.KS * q.Lmax;
#pragma unroll
    for (int j = 0; j < MAX_B_ITEMS; ++j) {
        int i = tid + j * THREADS;
        b_goff[j] = -1;
        b_loff[j] = -1;
        b_plane[j] = 0;
        if (i < n_items) {
            int h = fdiv(i, q.dL), slot = i - h * q.Lmax;  // h = ks*2 + half
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

    // ---- MFMA operand addresses of this lane
    const int kg = lane >> 5;  // which 16 of the 32 K values this lane feeds
    int a_off[MT];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
        int r = wm * WM + mi * 32 + (lane & 31);
        a_off[mi] = r * KROW + (((kg ^ (r >> 3)) & 1) << 4);
    }
    int b_slot[NT];
#pragma unroll
    for (int ni = 0; ni < NT; ++ni) {
        int p = p0 + wn * 64 + ni * 32 + (lane & 31);
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

    v4i ra[MAX_A_ITEMS];
    v4i rb[MAX_B_ITEMS];
    const int a_items = taps_stage * A_ROW_CHUNKS;  // 16-byte chunks of filter per stage

    auto prefetch = [&](int st) {
#pragma unroll
        for (int j = 0; j < MAX_A_ITEMS; ++j) {
            int i = tid + j * THREADS;
            if (i < a_items) {
                int t = i / A_ROW_CHUNKS, c = i - t * A_ROW_CHUNKS;
                const int8_t* g = q.wp + ((size_t)(st * taps_stage + t) * q.OCP + oc0) * KROW + c * 16;
                ra[j] = *(const v4i*)g;
            }
        }
        const int plane0 = st * q.KS * 8;
#pragma unroll
        for (int j = 0; j < MAX_B_ITEMS; ++j) {
            v4i v = {0, 0, 0, 0};
            if (b_goff[j] >= 0) {
                int pl = plane0 + b_plane[j];
                const int8_t* g = q.src + b_goff[j] + (size_t)pl * q.plane_stride;
                // planes past the last one meet zero filter rows, so their value is irrelevant;
                // they are only kept from reading out of bounds
                if (pl + 0 < q.C4) v[0] = *(const int*)(g);
                if (pl + 1 < q.C4) v[1] = *(const int*)(g + q.plane_stride);
                if (pl + 2 < q.C4) v[2] = *(const int*)(g + 2 * q.plane_stride);
                if (pl + 3 < q.C4) v[3] = *(const int*)(g + 3 * q.plane_stride);
            }
            rb[j] = v;
        }
    };

    const int st_begin = blockIdx.z * q.sps, st_end = min(q.stages, st_begin + q.sps);
    if (st_begin < st_end)
        prefetch(st_begin);
    for (int st = st_begin; st < st_end; ++st) {
        __syncthreads();
#pragma unroll
        for (int j = 0; j < MAX_A_ITEMS; ++j) {
            int i = tid + j * THREADS;
            if (i < a_items)
                *(v4i*)(ldsA + i * 16) = ra[j];
        }
#pragma unroll
        for (int j = 0; j < MAX_B_ITEMS; ++j)
            if (b_loff[j] >= 0)
                *(v4i*)(ldsB + b_loff[j]) = rb[j];
        __syncthreads();
        if (st + 1 < st_end)
            prefetch(st + 1);

        for (int ks = 0; ks < q.KS; ++ks) {
            const int8_t* bks = ldsB + ks * (q.Lmax * KROW);
            int t = ks * q.taps;
            for (int fh = 0; fh < q.FH; ++fh) {
                for (int fw = 0; fw < q.FW; ++fw, ++t) {
                    const int tap_off = fh * q.DH * q.VW + fw * q.DW;
                    v4i a[MT], b[NT];
#pragma unroll
                    for (int mi = 0; mi < MT; ++mi)
                        a[mi] = *(const v4i*)(ldsA + t * (BM * KROW) + a_off[mi]);
#pragma unroll
                    for (int ni = 0; ni < NT; ++ni) {
                        int s = b_slot[ni] + tap_off;
                        b[ni] = *(const v4i*)(bks + s * KROW + (((kg ^ (s >> 3)) & 1) << 4));
                    }
#pragma unroll
                    for (int mi = 0; mi < MT; ++mi)
#pragma unroll
                        for (int ni = 0; ni < NT; ++ni)
                            acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                    a[mi], b[ni], acc[mi][ni], 0, 0, 0);
                }
            }
        }
    }

    // ---- epilogue: register e of a 32x32 tile holds row 8*(e/4) + 4*(lane/32) + e%4, col lane%32.
    //      The 4 bias values of a register group are fetched once and reused for all pixels.
    if (q.split > 1) {
        const int ocs = (q.OC + 3) & ~3;
#pragma unroll
        for (int mi = 0; mi < MT; ++mi)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int oc = oc0 + wm * WM + mi * 32 + e4 * 8 + kg * 4;
                if (oc >= q.OC)
                    continue;
#pragma unroll
                for (int ni = 0; ni < NT; ++ni) {
                    const int p = p0 + wn * 64 + ni * 32 + (lane & 31);
                    if (p <= plast)
                        *(int4*)(q.partial + ((size_t)blockIdx.z * q.P + p) * ocs + oc) =
                                make_int4(acc[mi][ni][e4 * 4], acc[mi][ni][e4 * 4 + 1],
                                          acc[mi][ni][e4 * 4 + 2], acc[mi][ni][e4 * 4 + 3]);
                }
            }
        return;
    }
    int pix_n[NT], pix_rem[NT];
#pragma unroll
    for (int ni = 0; ni < NT; ++ni) {
        const int p = p0 + wn * 64 + ni * 32 + (lane & 31);
        pix_n[ni] = p <= plast ? (int)fdiv(p, q.dOHW) : -1;
        pix_rem[ni] = p - pix_n[ni] * q.OHW;
    }
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
            const int oc = oc0 + wm * WM + mi * 32 + e4 * 8 + kg * 4;
            if (oc < q.OC) {
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
#pragma unroll
                for (int ni = 0; ni < NT; ++ni) {
                    if (pix_n[ni] >= 0) {
                        int r[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int a = acc[mi][ni][e4 * 4 + e] + bv[e];
                            if constexpr (ACT == ACT_RUNTIME)
                                r[e] = requant_conv_rt(q.act, a, q.s_src, q.s_flt, q.s_dst);
                            else
                                r[e] = requant_conv_fast<ACT>(a, q.rq);
                        }
                        if (!q.dst_fc) {
                            size_t o = ((size_t)pix_n[ni] * (q.OC >> 2) + (oc >> 2)) * q.OHW + pix_rem[ni];
                            ((uint32_t*)q.dst)[o] = pack4(r[0], r[1], r[2], r[3]);
                        } else {
                            const int p = p0 + wn * 64 + ni * 32 + (lane & 31);
                            int8_t* o = q.dst + (size_t)p * q.OC + oc;
                            if (((q.OC & 3) == 0)) {
                                *(uint32_t*)o = pack4(r[0], r[1], r[2], r[3]);
                            } else {
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    if (oc + e < q.OC)
                                        o[e] = (int8_t)r[e];
                            }
                        }
                    }
                }
            }
        }
    }
}

// ---- split-K: sum the partial accumulators, then bias + requantise + store -----------------
__global__ void __launch_bounds__(256) conv_mfma_reduce_kernel(MfmaParams q) {
    const int ocs = (q.OC + 3) & ~3, oc4n = ocs >> 2;
    const size_t total = (size_t)q.P * oc4n;
    for (size_t i = blockIdx.x * (size_t)256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const int p = (int)(i / oc4n), oc = (int)(i - (size_t)p * oc4n) * 4;
        int a[4] = {0, 0, 0, 0};
#pragma unroll 8
        for (int z = 0; z < q.split; ++z) {
            const int4 v = *(const int4*)(q.partial + ((size_t)z * q.P + p) * ocs + oc);
            a[0] += v.x; a[1] += v.y; a[2] += v.z; a[3] += v.w;
        }
        int r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int b = (q.bias && oc + e < q.OC) ? q.bias[oc + e] : 0;
            r[e] = requant_conv_rt(q.act, a[e] + b, q.s_src, q.s_flt, q.s_dst);
        }
        if (!q.dst_fc) {
            const int n = (int)fdiv(p, q.dOHW), rem = p - n * q.OHW;
            ((uint32_t*)q.dst)[((size_t)n * (q.OC >> 2) + (oc >> 2)) * q.OHW + rem] =
                    pack4(r[0], r[1], r[2], r[3]);
        } else {
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
}

// Split factor of the one-stage kernel for layers with few output pixels and a long K
// (FullyConnected at small batch, the last pointwise layers): a pure function of the shape, shared
// by the _workspace entry point, the generated shims and the launch.
// oc tile of the one-stage kernel: 64 rows when 128-row tiles would leave most of the chip idle
static int conv_mfma_bm(const ConvGeom& g) {
    const long P = (long)g.n * g.oh * g.ow;
    return g.oc <= 64 || ((P + 127) / 128) * ((g.oc + 127) / 128) < 64 ? 64 : 128;
}

static int conv_mfma_split(const ConvGeom& g) {
    const long P = (long)g.n * g.oh * g.ow;
    const int taps = g.fh * g.fw;
    const int ks = taps <= 2 ? 4 : taps <= 4 ? 2 : 1;
    const long chunks = (g.ic + 31) / 32, stages = (chunks + ks - 1) / ks;
    const long bm = conv_mfma_bm(g);
    const long tiles = ((P + 127) / 128) * ((g.oc + bm - 1) / bm);
    if (tiles >= 128 || stages < 2)
        return 1;
    long s = (512 + tiles - 1) / tiles;
    if (s > stages)
        s = stages;
    if (s > 16)
        s = 16;
    return s < 2 ? 1 : (int)s;
}

size_t conv_mfma_workspace_bytes(const ConvGeom& g) {
    const int s = conv_mfma_split(g);
    const long P = (long)g.n * g.oh * g.ow;
    return s > 1 ? (size_t)s * P * ((g.oc + 3) & ~3) * sizeof(int32_t) : 0;
}

// ---- filter packing ---------------------------------------------------------------------
// packed[(chunk*taps + tap)*OCP + oc][pos], pos in 0..31 holds input channel
// chunk*32 + (pos ^ 16*((oc>>3)&1)); zero beyond IC / OC.
__global__ void __launch_bounds__(256) pack_filter_kernel(
        const int8_t* __restrict__ flt, int8_t* __restrict__ out, size_t total, int taps, int FW,
        int OC, int OCP, int IC, int fmt) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        int pos = i & 31;
        size_t r = i >> 5;
        int oc = r % OCP;
        r /= OCP;
        int tap = r % taps;
        int chunk = (int)(r / taps);
        int ic = chunk * 32 + (pos ^ (((oc >> 3) & 1) << 4));
        int8_t v = 0;
        if (oc < OC && ic < IC) {
            int fh = tap / FW, fw = tap - fh * FW;
            int FH = taps / FW;
            size_t o;
            if (fmt == MEGCC_FMT_NCHW44)  // [OC/4][IC/4][FH][FW][4 ic][4 oc]
                o = (((((size_t)(oc >> 2) * (IC >> 2) + (ic >> 2)) * FH + fh) * FW + fw) * 4 +
                     (ic & 3)) * 4 + (oc & 3);
            else  // NCHW [OC][IC][FH][FW]
                o = (((size_t)oc * IC + ic) * FH + fh) * FW + fw;
            v = flt[o];
        }
        out[i] = v;
    }
}

static int round_up(int a, int b) {
    return (a + b - 1) / b * b;
}

static bool is_fc(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW && g.ih == 1 && g.iw == 1 && g.fh == 1 && g.fw == 1 &&
           g.oh == 1 && g.ow == 1 && g.ph == 0 && g.pw == 0;
}

static int choose_ks(int taps) {
    return taps <= 2 ? 4 : taps <= 4 ? 2 : 1;
}

struct TilePlan {
    int Lmax;
    int VW, VH;
    int rows_max;  // most virtual rows any patch touches
};

// largest patch any tile of `bn` pixels needs; mirrors vp_of() / L in the kernels
static TilePlan plan_tiles_uncached(const ConvGeom& g, int bn, long range_len, int pm);

// The plan walks over every tile of the layer: kept per geometry, so that a launch costs the host
// a map look-up and not a loop over the tensor.
static TilePlan plan_tiles(const ConvGeom& g, int bn = BN, long range_len = 0, int pm = 0) {
    typedef std::array<long, 16> Key;
    static std::map<Key, TilePlan> cache;
    static std::mutex lock;
    const Key key = {g.n, g.ih, g.iw, g.oh, g.ow, g.fh, g.fw, g.sh, g.sw, g.ph, g.pw, g.dh, g.dw,
                     bn, range_len, pm};
    std::lock_guard<std::mutex> guard(lock);
    auto it = cache.find(key);
    if (it != cache.end())
        return it->second;
    if (cache.size() > 4096)
        cache.clear();
    return cache[key] = plan_tiles_uncached(g, bn, range_len, pm);
}

// pm: the slot space of the plane-major patch (rows padded on the right only, to a multiple of 4;
// a patch starts pw slots before its first window, rounded down to 4)
static TilePlan plan_tiles_uncached(const ConvGeom& g, int bn, long range_len, int pm) {
    TilePlan t;
    t.VW = pm ? round_up(g.iw + g.pw, 4) : g.iw + 2 * g.pw;
    t.VH = g.ih + 2 * g.ph;
    long P = (long)g.n * g.oh * g.ow;
    auto vp = [&](long p) {
        long gi = p / g.ow, ow = p % g.ow;
        long n = gi / g.oh, oh = gi % g.oh;
        return (n * t.VH + oh * g.sh) * t.VW + ow * g.sw;
    };
    long lmax = 1, rmax = 1;
    if (range_len <= 0)
        range_len = P;
    for (long r0 = 0; r0 < P; r0 += range_len)
    for (long p0 = r0; p0 < (r0 + range_len < P ? r0 + range_len : P); p0 += bn) {
        long r1 = r0 + range_len < P ? r0 + range_len : P;
        long pl = (p0 + bn < r1 ? p0 + bn : r1) - 1;
        long L = vp(pl) + (long)(g.fh - 1) * g.dh * t.VW + (g.fw - 1) * g.dw - vp(p0) + 1;
        if (pm)
            L += (vp(p0) - g.pw) & 3;  // the slots between the rounded-down start and the window
        if (L > lmax)
            lmax = L;
        long rows = (vp(p0) + L - 1) / t.VW - vp(p0) / t.VW + 1;
        if (rows > rmax)
            rmax = rows;
    }
    t.Lmax = round_up((int)(lmax > (1 << 20) ? (1 << 20) : lmax), 64);
    t.rows_max = (int)rmax;
    return t;
}

static bool pick_dma(const ConvGeom& g, bool b128_ok, PipeConfig* pc, TilePlan* t, long* range_len, int* picked);

bool conv_mfma_supported(const ConvGeom& g) {
    if (g.groups != 1)
        return false;
    bool fc = is_fc(g);
    if (!(g.fmt == MEGCC_FMT_NCHW44 || fc))
        return false;
    if (g.ic & 3)
        return false;
    if (g.fmt == MEGCC_FMT_NCHW44 && (g.oc & 3))
        return false;
    if (g.fh * g.fw > MAX_TAPS_STAGE) {
        // only the row-split variants of the LDS-direct kernel (no one-stage fallback: that kernel
        // keeps every tap of a chunk in LDS and registers)
        PipeConfig pc;
        TilePlan t;
        long range_len = 0;
        int picked = -1;
        const long slots = ((long)g.n * (g.ih + 2 * g.ph) + 2L * g.fh * g.dh) * (g.iw + 2 * g.pw);
        return (long)g.n * g.ic * g.ih * g.iw < (1L << 31) && slots < (1L << 31) &&
               (long)g.n * g.oh * g.ow < (1L << 31) - 512 && pick_dma(g, false, &pc, &t, &range_len, &picked);
    }
    long P = (long)g.n * g.oh * g.ow;
    long src_bytes = (long)g.n * g.ic * g.ih * g.iw;
    long vmax = ((long)g.n * (g.ih + 2 * g.ph) + 2L * g.fh * g.dh) * (g.iw + 2 * g.pw);
    if (P <= 0 || P >= (1L << 31) - BN || src_bytes >= (1L << 31) || vmax >= (1L << 31))
        return false;
    TilePlan t = plan_tiles(g);
    int ks = choose_ks(g.fh * g.fw);
    if (2L * ks * t.Lmax > (long)MAX_B_ITEMS * THREADS)
        return false;
    return true;
}

size_t conv_mfma_packed_bytes(const ConvGeom& g) {
    int taps = g.fh * g.fw, ks = choose_ks(taps);
    (void)ks;
    int chunks = round_up((g.ic + 31) / 32, CHUNK_PAD);
    // (pointwise layers of 257 .. 512 input channels: the streaming kernel reads 16 chunks)
    if (taps == 1 && chunks > 8 && chunks < 16)
        chunks = 16;
    return (size_t)chunks * taps * round_up(g.oc, OC_PAD) * KROW;
}

TinyNNStatus conv_mfma_pack(const ConvGeom& g, const void* flt, void* packed) {
    size_t total = conv_mfma_packed_bytes(g);
    unsigned blocks = (unsigned)((total + 255) / 256);
    if (blocks > 65536u)
        blocks = 65536u;
    hipLaunchKernelGGL(pack_filter_kernel, dim3(blocks), dim3(256), 0, stream(),
                       (const int8_t*)flt, (int8_t*)packed, total, g.fh * g.fw, g.fw, g.oc,
                       round_up(g.oc, OC_PAD), g.ic, g.fmt);
    return check_launch("pack_filter");
}

bool conv_mfma_dma_config(const ConvGeom& g, bool fc, int variant, bool b128_ok, PipeConfig* c);

// launches a configuration of the LDS-direct kernel (conv_mfma_i8_dma.hip): one workgroup per
// pixel range and output-channel tile, the whole grid resident at once
static TinyNNStatus conv_mfma_pipe_launch(const PipeConfig& c, MfmaParams q) {
    const size_t lds = c.nbuf * ((size_t)c.a_bytes + (size_t)c.ks * q.Lmax * KROW) + c.extra_lds;
    MG_REQUIRE(lds <= 160 * 1024, TinyNN_ERROR_OUT_OF_RANGE, "conv_mfma_i8_dma: %zu bytes of LDS", lds);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(c.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_mfma_i8_dma: LDS attribute: %s",
                   hipGetErrorString(e));
    }
    dim3 grid((q.P + q.range_len - 1) / q.range_len, (q.OC + c.bm - 1) / c.bm);
    void* args[] = {&q};
    hipError_t e = hipLaunchKernel(c.kernel, grid, dim3(c.threads), args, lds, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_mfma_i8_dma: launch: %s", hipGetErrorString(e));
    return check_launch("conv_mfma_i8_dma");
}



int fc_stream_split(const ConvGeom& g, const void* src, size_t ws_bytes, int max_split);
TinyNNStatus fc_stream_launch(
        const ConvGeom& g, const void* src, const void* packed, int32_t* partial, int split);
bool fc_one_supported(const ConvGeom& g, const void* src);
TinyNNStatus fc_one_launch(
        const ConvGeom& g, const void* src, const void* packed, const void* bias, void* dst);
bool fc_gevm_q8_supported(const ConvGeom& g);
TinyNNStatus fc_gevm_q8_launch(
        const ConvGeom& g, const void* src, const void* packed, const void* bias, void* dst);
bool conv_pw_stream_supported(const ConvGeom& g);
TinyNNStatus conv_pw_stream_launch(
        const ConvGeom& g, const void* src, const void* packed, const void* bias, void* dst);

// Picks the variant of the LDS-direct kernel for this layer (in order of preference; development
// switches skip one) and the pixel range per workgroup; false: none of them takes the layer.
static bool pick_dma(const ConvGeom& g, bool b128_ok, PipeConfig* pc, TilePlan* t, long* range_len, int* picked) {
    bool pipe = false;
    // variants of the LDS-direct kernel in order of preference (see conv_mfma_dma_config); a
    // layer none of them takes runs on the one-stage kernel below
    // (8, 9: one filter row per stage, the only ones that take filters of more than 9 taps)
    static const int kDmaVariants[] = {6, 7, 2, 3, 0, 4, 1, 8, 9};
    const Options& opt = options();
    const bool dma_off[] = {opt.no_small, opt.no_small, opt.no_pm768, opt.no_pm,
                            opt.no_dma512, opt.no_pm256, opt.no_dma, opt.no_rowsplit, opt.no_rowsplit};
    constexpr int N_DMA_VARIANTS = 9;
    for (int cand = 0; cand < N_DMA_VARIANTS && !pipe; ++cand) {
        const int v = kDmaVariants[cand];
        const bool have = !opt.no_dma && !dma_off[cand] && !((v == 2 || v == 4 || v == 6) && opt.no_pm) &&
                          conv_mfma_dma_config(g, is_fc(g), v, b128_ok, pc);
        if (!have)
            continue;
        *picked = v;
        // one pixel range per free workgroup slot, so that the whole grid is resident at once and
        // every CU finishes at the same time (no partial last round)
        const long P = (long)g.n * g.oh * g.ow;
        const long slots = (long)num_cus() * pc->blocks_per_cu;
        const long oc_tiles = (g.oc + pc->bm - 1) / pc->bm;
        long ranges = slots / oc_tiles > 0 ? slots / oc_tiles : 1;
        (*range_len) = ((P + ranges - 1) / ranges + 31) / 32 * 32;
        if ((*range_len) < pc->bn / 2) {  // too few pixels per workgroup for the tile
            if (pc->bm == 32)
                (*range_len) = pc->bn;  // the small-layer tiles: one tile per workgroup, not every CU busy
            else if (pc->bn <= 256 && (P >= 4096 || (g.fh == 1 && g.fw == 1 && P >= 2048)))
                // between the small-layer tiles and a full grid of 256- / 128-pixel tiles: half-filled
                // tiles on part of the CUs (N=6, 128->128, 56x56: 9.4 us; the one-stage kernel
                // these layers fell to: 20.8 us)
                (*range_len) = pc->bn / 2;
            else
                continue;
        }
        ConvGeom gp = g;  // (row split: a stage's patch spans the windows of ONE filter row)
        if (pc->rs)
            gp.fh = 1;
        *t = plan_tiles(gp, pc->bn, (*range_len), pc->pm);
        if (pc->fixed_lmax) {
            if (t->Lmax > pc->fixed_lmax)
                continue;
            t->Lmax = pc->fixed_lmax;
        }
        pipe = ((long)pc->nbuf * (pc->a_bytes + (long)pc->ks * t->Lmax * KROW) + pc->extra_lds) * pc->blocks_per_cu <= 160 * 1024;
    }
    return pipe;
}

TinyNNStatus conv_mfma_launch(
        const ConvGeom& g, const void* src, const void* packed, const void* bias, void* dst,
        const Workspace* ws) {
    // pointwise layers with few input channels: the streaming kernel (conv_pw_stream.hip)
    if (conv_pw_stream_supported(g) && !options().no_pws)
        return conv_pw_stream_launch(g, src, packed, bias, dst);  // (notes its own variant)
    // FullyConnected with at most 4 rows: one pass over the weights (fc_gevm_q8.hip)
    if (is_fc(g) && fc_gevm_q8_supported(g) && !options().no_gevm) {
        note_kernel("fc_gevm_q8");
        return fc_gevm_q8_launch(g, src, packed, bias, dst);
    }
    // FullyConnected with at most 64 rows: one launch, K slices meet inside the workgroup
    // (fc_stream.hip). A long K under few output channels is a handful of workgroups with hundreds
    // of KB each: that shape stays with the K slices in separate workgroups below, if it has the
    // workspace for them.
    const bool few_long = g.ic > 8192 && g.oc < 4096 && ws && ws->ptr;
    if (is_fc(g) && fc_one_supported(g, src) && !few_long && !options().no_fcone && !options().no_fcs) {
        return fc_one_launch(g, src, packed, bias, dst);
    }
    MfmaParams q = {};
    PipeConfig pc;
    const bool b128_ok = ((uintptr_t)src & 15) == 0 && !options().no_fcb;
    long range_len = 0;
    TilePlan t;
    int picked = -1;  // variant of the LDS-direct kernel
    const bool pipe = pick_dma(g, b128_ok, &pc, &t, &range_len, &picked);
    if (!pipe) {
        range_len = 0;
        t = plan_tiles(g, BN);
    }
    q.range_len = (int)range_len;
    bool fc = is_fc(g);
    q.src = (const int8_t*)src;
    q.src_bytes = (int)((long)g.n * g.ic * g.ih * g.iw);
    q.wp = (const int8_t*)packed;
    q.bias = (const int32_t*)bias;
    q.dst = (int8_t*)dst;
    q.N = g.n;
    q.OH = g.oh;
    q.OW = g.ow;
    q.OHW = g.oh * g.ow;
    q.P = g.n * q.OHW;
    q.OC = g.oc;
    q.OCP = round_up(g.oc, OC_PAD);
    q.C4 = g.ic / 4;
    q.taps = g.fh * g.fw;
    q.FH = g.fh;
    q.FW = g.fw;
    q.KS = pipe ? pc.ks : choose_ks(q.taps);
    q.stages = round_up((g.ic + 31) / 32, q.KS) / q.KS;
    if (pipe && pc.rs)
        q.stages *= g.fh;  // one stage per (chunk, filter row)
    MG_REQUIRE(pipe || q.taps <= MAX_TAPS_STAGE, TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "conv_mfma: %d taps and no row-split variant takes the layer", q.taps);
    q.VW = t.VW;
    q.VH = t.VH;
    q.IH = g.ih;
    q.IW = g.iw;
    q.PH = g.ph;
    q.PW = g.pw;
    q.SH = g.sh;
    q.SW = g.sw;
    q.DH = g.dh;
    q.DW = g.dw;
    if (fc) {
        q.image_stride = g.ic;
        q.plane_stride = 4;
        q.row_stride = 0;
        q.pix_stride = 0;
    } else {
        q.image_stride = g.ic * g.ih * g.iw;
        q.plane_stride = g.ih * g.iw * 4;
        q.row_stride = g.iw * 4;
        q.pix_stride = 4;
    }
    q.Lmax = t.Lmax;
    q.dst_fc = fc ? ((g.oc & 31) == 0 && ((uintptr_t)dst & 15) == 0 ? 2 : 1) : 0;
    q.bias_vec4 = bias && ((uintptr_t)bias & 15) == 0;
    q.act = g.act;
    q.s_src = g.s_src;
    q.s_flt = g.s_flt;
    q.s_dst = g.s_dst;
    q.rq = make_requant_fast(g.s_src, g.s_flt, g.s_dst);
    if (pipe && requant_table_act(g.act) && !(fc && g.act == MEGCC_NONLINE_H_SWISH) &&
        requant_table_ok(g.s_src, g.s_flt, g.s_dst))
        q.rq_table = requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst);
    q.dOW = make_fastdiv(q.OW);
    q.dOH = make_fastdiv(q.OH);
    q.dVW = make_fastdiv(q.VW);
    q.dVH = make_fastdiv(q.VH);
    q.dL = make_fastdiv(q.Lmax);
    q.dOHW = make_fastdiv(q.OHW);

    q.split = 1;
    q.sps = q.stages;
    q.partial = nullptr;
    if (pipe) {
        // (FullyConnected tiles: each XCD a compact rectangle of the tile grid, common.h)
        q.xo = pc.fcb && !options().no_xcdorder
                       ? make_xcd_order((q.P + q.range_len - 1) / q.range_len, (q.OC + pc.bm - 1) / pc.bm)
                       : XcdOrder{0};
        if (pc.fcb && pc.bm == 256 && q.dst_fc == 2)
            q.dst_fc = 3;  // rows leave through the kernel's staging area in LDS
        note_kernel(q.xo.w ? "conv_mfma_i8_dma_xo" : "conv_mfma_i8_dma", picked,
                    pc.bm, pc.bn, q.Lmax, pc.ks);
        const RequantAffine aff = requant_affine_pick(
                requant_table_act(g.act) && requant_table_ok(g.s_src, g.s_flt, g.s_dst), g.act, g.s_src, g.s_flt,
                g.s_dst);
        q.rq.aff_c = aff.c;
        q.rq.aff_d = aff.d;
        return conv_mfma_pipe_launch(pc, q);
    }
    const int split = conv_mfma_split(g);
    // FullyConnected with few rows: stream the weights (fc_stream.hip), finish with the reduce
    // kernel below
    if (fc && split > 1 && ws && ws->ptr && ((uintptr_t)ws->ptr & 15) == 0 && !options().no_fcs) {
        const int fs = fc_stream_split(g, src, ws->size, split);
        if (fs > 0) {
            note_kernel("fc_stream", fs);
            TinyNNStatus st = fc_stream_launch(g, src, packed, (int32_t*)ws->ptr, fs);
            if (st != TinyNN_SUCCESS)
                return st;
            q.split = fs;
            q.partial = (int32_t*)ws->ptr;
            const size_t total = (size_t)q.P * ((q.OC + 3) / 4);
            unsigned blocks = (unsigned)((total + 255) / 256);
            hipLaunchKernelGGL(conv_mfma_reduce_kernel, dim3(blocks > 4096 ? 4096 : blocks), dim3(256),
                               0, stream(), q);
            return check_launch("conv_mfma_reduce");
        }
    }
    if (split > 1 && ws && ws->ptr && ws->size >= conv_mfma_workspace_bytes(g) &&
        ((uintptr_t)ws->ptr & 15) == 0) {
        // equal slices of whole stages; no slice may start at or beyond the last stage (it would
        // fetch filter rows past the packed buffer), so the slice count follows from the slice
        // length: 8 stages asked in 6 slices are 4 slices of 2
        q.sps = (q.stages + split - 1) / split;
        q.split = (q.stages + q.sps - 1) / q.sps;
        q.partial = (int32_t*)ws->ptr;
    }

    const int bm = conv_mfma_bm(g);
    note_kernel("conv_mfma_i8", bm, q.split);
    const size_t lds = (size_t)q.taps * q.KS * bm * KROW + (size_t)q.KS * q.Lmax * KROW;
    MG_REQUIRE(lds <= 160 * 1024, TinyNN_ERROR_OUT_OF_RANGE, "conv_mfma: %zu bytes of LDS", lds);
    dim3 grid((q.P + BN - 1) / BN, (g.oc + bm - 1) / bm, q.split);
    void (*kern)(MfmaParams);
    if (g.act == MEGCC_NONLINE_IDENTITY)
        kern = bm == 64 ? conv_mfma_i8_kernel<64, MEGCC_NONLINE_IDENTITY>
                        : conv_mfma_i8_kernel<128, MEGCC_NONLINE_IDENTITY>;
    else if (g.act == MEGCC_NONLINE_RELU)
        kern = bm == 64 ? conv_mfma_i8_kernel<64, MEGCC_NONLINE_RELU>
                        : conv_mfma_i8_kernel<128, MEGCC_NONLINE_RELU>;
    else
        kern = bm == 64 ? conv_mfma_i8_kernel<64, ACT_RUNTIME> : conv_mfma_i8_kernel<128, ACT_RUNTIME>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(
                (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_mfma: LDS attribute: %s",
                   hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, grid, dim3(THREADS), lds, stream(), q);
    if (q.split > 1) {
        const size_t total = (size_t)q.P * ((q.OC + 3) / 4);
        unsigned blocks = (unsigned)((total + 255) / 256);
        hipLaunchKernelGGL(conv_mfma_reduce_kernel, dim3(blocks > 4096 ? 4096 : blocks), dim3(256), 0,
                           stream(), q);
    }
    return check_launch("conv_mfma_i8");
}

}  // namespace mg
