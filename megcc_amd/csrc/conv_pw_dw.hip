// qsi8 NCHW44: a pointwise (1x1, stride 1) convolution and the channel-wise 3x3 convolution that reads
// its result, as ONE kernel, for small images.
//
// On 14 x 14 and 7 x 7 images both layers of such a pair are far too short to fill the chip for
// long: each costs a launch, a pipeline fill and a trip of the tensor in between through memory.
// Here a workgroup owns one image and a slice of OCS output channels and keeps everything in LDS:
//   0. the slice's rows of the packed pointwise filter (IC x OCS bytes), both threshold tables and
//      both bias slices go to LDS; the area of the intermediate image is cleared;
//   1. pointwise: a wave takes (32-pixel tile, 32-channel tile) jobs. The MFMA's A operand is the
//      activations - lane (pixel l & 31, K-half l >> 5) needs 16 consecutive channels = one dword
//      from each of 4 consecutive NCHW44 planes, straight from global memory - and its B operand the
//      filter rows from LDS, so D[pixel][channel] leaves 4 consecutive pixels of ONE channel in 4
//      consecutive accumulator registers: after the requantisation they are one dword of a
//      channel-planar image. A tile is 32 / P rows of P pixels, P the power of two above the width,
//      so that dword never crosses a row; pixels beyond the width are cleared. The planes keep one
//      cleared row above and below and at least one cleared column right of every row, which is
//      all the padding the 3x3 window needs;
//   2. channel-wise 3x3 on those planes: a thread owns 4 channels and walks over groups of 4
//      output pixels of a row; per channel and filter row three aligned dwords give the windows
//      (two v_alignbyte), the taps (w0, w1, w2, 0) and (0, w0, w1, w2) go through v_dot4; the 4 x 4
//      results are requantised, transposed back to NCHW44 and stored 16 bytes at a time.
// Both requantisations are the library's exact ones (threshold table, or the proven fused
// multiply-add), so the result is bit for bit what the two kernels give in sequence.
// Reference loops: BareMetal/ConvKernel.cpp:305-344 (dense) and the GROUP branch of the same.
#include "conv_mfma_i8.h"

namespace mg {

static constexpr int PWDW_THREADS = 512;

struct PwDwParams {
    const int8_t* src;       // [N][IC/4][H][W][4]
    const int8_t* wp;        // packed pointwise filter [IC/32][OCP][32]
    const int32_t* pw_bias;  // or NULL
    const uint32_t* dw_flt;  // [OC/4][3][3][4]
    const int32_t* dw_bias;  // or NULL
    uint32_t* dst;           // [N][OC/4][OH][OW][4]
    int src_bytes;
    int IC4, H, W, HW, OH, OW, OC4, OCP;
    int lgP;           // rows of the intermediate planes are 1 << lgP bytes
    int tiles;         // 32-pixel tiles of an image: ceil(H / (32 >> lgP))
    int XQ;            // groups of 4 output pixels per row
    int items;         // OH * XQ
    int plane_stride;  // bytes, an odd number of dwords
    int slices;        // OC / OCS
    int pw_lo, dw_lo;  // lowest output: 0 with RELU, -128 else
    float pw_c, pw_ac, pw_ad, dw_c, dw_ac, dw_ad;  // a?_ad != 0: requantisation by multiply-add
    FastDiv dXQ;
    RequantTable pw_table, dw_table;
};

__device__ __forceinline__ int pwdw_kernarg(int byte_offset) {
    typedef const __attribute__((address_space(4))) char* kptr;
    const kptr base = (kptr)__builtin_amdgcn_kernarg_segment_ptr();
    return *(const __attribute__((address_space(4))) int*)(base + byte_offset);
}

__device__ __forceinline__ int pwdw_med3(int x, int lo, int hi) {
    return min(max(x, lo), hi);
}
__device__ __forceinline__ int pwdw_requant_table(int acc, float c, int lo, const int* tbl) {
    const int m = pwdw_med3(cvt_floor_i32((float)acc * c), lo, 126);
    return m + (acc > tbl[m + 128] ? 1 : 0);
}
__device__ __forceinline__ int pwdw_requant_affine(int acc, float c, float d, int lo) {
    return pwdw_med3(cvt_floor_i32(__builtin_fmaf((float)acc, c, d)), lo, 127);
}

typedef unsigned v4u_a4 __attribute__((ext_vector_type(4), aligned(4)));

// bytes `i` of a, b, c -> (a_i, b_i, c_i, 0)
__device__ __forceinline__ uint32_t pwdw_taps(uint32_t a, uint32_t b, uint32_t c, int i) {
    return ((a >> (8 * i)) & 0xffu) | (((b >> (8 * i)) & 0xffu) << 8) | (((c >> (8 * i)) & 0xffu) << 16);
}

// KC: 32-channel chunks of the pointwise layer (IC = 32 * KC). OCS: output channels per workgroup.
// S: stride of the channel-wise layer. JT: 32-channel tiles per pointwise job - all of the slice's
// when the image has enough 32-pixel tiles to occupy the waves (the activations are then fetched
// once), one when it has only a few.
template <int KC, int OCS, int S, int JT>
__global__ void __launch_bounds__(PWDW_THREADS) conv_pw_dw_kernel(PwDwParams q) {
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    constexpr int OT = OCS / 32 / JT;         // pointwise jobs per 32-pixel tile
    constexpr int NW = PWDW_THREADS / 64;     // waves
    int8_t* const flt = lds;                                      // KC * OCS * 32
    int* const tbl_pw = (int*)(flt + KC * OCS * KROW);            // 256
    int* const tbl_dw = tbl_pw + REQUANT_TABLE_ENTRIES;           // 256
    int* const bias_pw = tbl_dw + REQUANT_TABLE_ENTRIES;          // OCS
    int* const bias_dw = bias_pw + OCS;                           // OCS
    int8_t* const planes = (int8_t*)(bias_dw + OCS);              // OCS * plane_stride + 16
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, kg = lane >> 5;
    const int n = blockIdx.x / q.slices;
    const int oc0 = (blockIdx.x - n * q.slices) * OCS;
    const int P = 1 << q.lgP, rpt = 32 >> q.lgP;

    const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void*)q.src, 0, q.src_bytes, 0x00020000);
    const int jobs = q.tiles * OT;
    // the A operand of a job: this lane's pixel (row col >> lgP, column col & (P - 1)) of tile t,
    // planes c * 8 + kg * 4 + j; a wave keeps a ring of R chunks in flight, the next job's first
    // chunks behind the current job's last
    constexpr int R = KC < 8 ? KC : 8;
    auto job_base = [&](int job) __attribute__((always_inline)) -> unsigned {
        const int t = job / OT;
        const int y = t * rpt + (col >> q.lgP), x = col & (P - 1);
        return job < jobs && y < q.H && x < q.W
                       ? (unsigned)((((n * q.IC4 + kg * 4) * q.HW) + y * q.W + x) * 4)
                       : 0x80000000u;
    };
    auto load_chunk = [&](unsigned base, int c, v4i& dst) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            dst[j] = (int)__builtin_amdgcn_raw_buffer_load_b32(
                    rs, (int)(base + (unsigned)((c * 8 + j) * q.HW * 4)), 0, 0);
    };
    // ---- 0. filter slice, tables, bias; clear the planes -----------------------------------------
    // Loads return in the order they were issued and the barrier below waits for the filter: the
    // tables and biases go first, then the filter, then the first job's activations (which are
    // still in flight while the LDS is written).
    const int tbl_word = tid < REQUANT_TABLE_ENTRIES
                                 ? pwdw_kernarg((int)offsetof(PwDwParams, pw_table) + 4 * tid)
                                 : pwdw_kernarg((int)offsetof(PwDwParams, dw_table) + 4 * (tid - REQUANT_TABLE_ENTRIES));
    int bias_word = 0;
    if (tid < OCS)
        bias_word = q.pw_bias ? q.pw_bias[oc0 + tid] : 0;
    else if (tid < 2 * OCS)
        bias_word = q.dw_bias ? q.dw_bias[oc0 + tid - OCS] : 0;
    constexpr int PIECES = KC * OCS * 2;  // 16-byte pieces of the slice
    constexpr int PPT = (PIECES + PWDW_THREADS - 1) / PWDW_THREADS;  // per thread
    static_assert(PIECES % PWDW_THREADS == 0 || PIECES < PWDW_THREADS, "whole rounds, or part of one");
    v4i piece[PPT];
#pragma unroll
    for (int k = 0; k < PPT; ++k) {
        const int idx = tid + k * PWDW_THREADS;
        const int c = idx / (OCS * 2), r = idx - c * (OCS * 2);
        if (PIECES % PWDW_THREADS == 0 || idx < PIECES)
            piece[k] = *(const v4i*)(q.wp + ((size_t)c * q.OCP + oc0) * KROW + r * 16);
    }
    v4i ring[R];
    unsigned base = job_base(wave);
#pragma unroll
    for (int c = 0; c < R; ++c)
        load_chunk(base, c, ring[c]);
    {
        const int plane_bytes = OCS * q.plane_stride + 16;  // (a multiple of 16 by construction)
        for (int i = tid * 16; i < plane_bytes; i += PWDW_THREADS * 16)
            *(v4i*)(planes + i) = v4i{0, 0, 0, 0};
        tbl_pw[tid] = tbl_word;  // (tbl_dw follows tbl_pw)
        if (tid < 2 * OCS)
            bias_pw[tid] = bias_word;  // (bias_dw follows bias_pw)
#pragma unroll
        for (int k = 0; k < PPT; ++k)
            if (PIECES % PWDW_THREADS == 0 || tid + k * PWDW_THREADS < PIECES)
                *(v4i*)(flt + (tid + k * PWDW_THREADS) * 16) = piece[k];
    }
    __syncthreads();

    // ---- 1. pointwise -----------------------------------------------------------------------------
    for (int job = wave; job < jobs; job += NW) {
        const unsigned next_base = job_base(job + NW);
        const int t = job / OT, ot = (job - t * OT) * JT;
        v16i acc[JT], acc1 = {};
        const int8_t* frow[JT];
#pragma unroll
        for (int jt = 0; jt < JT; ++jt) {
            const int ocl = (ot + jt) * 32 + col;
            const int b = bias_pw[ocl];
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[jt][e] = b;
            frow[jt] = flt + ocl * KROW + (((kg ^ (ocl >> 3)) & 1) << 4);
        }
        static_for<KC>([&](auto cc) {
            constexpr int c = decltype(cc)::value;
            if (JT == 1) {
                // two accumulator chains (even and odd chunks) keep the matrix core busy between them
                const v4i f = *(const v4i*)(frow[0] + c * (OCS * KROW));
                if (c & 1)
                    acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[c % R], f, acc1, 0, 0, 0);
                else
                    acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[c % R], f, acc[0], 0, 0, 0);
            } else {
#pragma unroll
                for (int jt = 0; jt < JT; ++jt) {
                    const v4i f = *(const v4i*)(frow[jt] + c * (OCS * KROW));
                    acc[jt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[c % R], f, acc[jt], 0, 0, 0);
                }
            }
            if (c + R < KC)
                load_chunk(base, c + R, ring[c % R]);
            else
                load_chunk(next_base, c + R - KC, ring[c % R]);
        });
        base = next_base;
        if (JT == 1)
            acc[0] += acc1;
#pragma unroll
        for (int jt = 0; jt < JT; ++jt) {
            int r[16];
            if (q.pw_ad != 0.f) {  // (uniform)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    r[e] = pwdw_requant_affine(acc[jt][e], q.pw_ac, q.pw_ad, q.pw_lo);
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    r[e] = pwdw_requant_table(acc[jt][e], q.pw_c, q.pw_lo, tbl_pw);
            }
            int8_t* const plane = planes + ((ot + jt) * 32 + col) * q.plane_stride + 4;
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                // registers 4 e4 .. 4 e4 + 3: pixels 8 e4 + 4 kg + (0..3) of the tile
                const int m0 = 8 * e4 + 4 * kg;
                const int y = t * rpt + (m0 >> q.lgP), x0 = m0 & (P - 1);
                const int left = q.W - x0;  // pixels of this dword inside the row
                uint32_t w = pack4_perm(r[4 * e4], r[4 * e4 + 1], r[4 * e4 + 2], r[4 * e4 + 3]);
                if (left < 4)
                    w &= (1u << (8 * max(left, 0))) - 1u;
                if (y < q.H && left > 0)
                    *(uint32_t*)(plane + (y + 1) * P + x0) = w;
            }
        }
    }
    __syncthreads();

    // ---- 2. channel-wise 3x3 ----------------------------------------------------------------------
    constexpr int Q4 = OCS / 4;                // channel quads of the slice
    constexpr int SL = PWDW_THREADS / Q4;      // threads per quad
    const int c4 = tid / SL, slot = tid - c4 * SL;
    uint32_t wq[3][4], ws[3][4];
    {
        const uint32_t* f = q.dw_flt + (size_t)(oc0 / 4 + c4) * 9;
#pragma unroll
        for (int dy = 0; dy < 3; ++dy) {
            const uint32_t f0 = f[dy * 3], f1 = f[dy * 3 + 1], f2 = f[dy * 3 + 2];
#pragma unroll
            for (int ch = 0; ch < 4; ++ch) {
                wq[dy][ch] = pwdw_taps(f0, f1, f2, ch);
                ws[dy][ch] = wq[dy][ch] << 8;
            }
        }
    }
    int bias4[4];
#pragma unroll
    for (int ch = 0; ch < 4; ++ch)
        bias4[ch] = bias_dw[c4 * 4 + ch];
    const int8_t* const quad = planes + (c4 * 4) * q.plane_stride + 4;
    uint32_t* const out_plane = q.dst + (size_t)(n * q.OC4 + oc0 / 4 + c4) * (q.OH * q.OW);
    for (int s = slot; s < q.items; s += SL) {
        const int oy = fdiv(s, q.dXQ), xq = s - oy * q.XQ;
        int acc[4][4];
#pragma unroll
        for (int ch = 0; ch < 4; ++ch)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[ch][j] = bias4[ch];
#pragma unroll
        for (int dy = 0; dy < 3; ++dy) {
            // plane row (input row + 1) = oy * S - 1 + dy + 1
            const int8_t* const row = quad + (oy * S + dy) * P + xq * (4 * S);
#pragma unroll
            for (int ch = 0; ch < 4; ++ch) {
                const int8_t* const p = row + ch * q.plane_stride;
                const uint32_t l = *(const uint32_t*)(p - 4), a = *(const uint32_t*)p,
                               b = *(const uint32_t*)(p + 4);
                uint32_t w0, w1, w2, w3;
                if (S == 1) {
                    w0 = w1 = __builtin_amdgcn_alignbyte(a, l, 3);  // x-1 x x+1 x+2
                    w2 = w3 = __builtin_amdgcn_alignbyte(b, a, 1);  // x+1 .. x+4
                } else {
                    w0 = __builtin_amdgcn_alignbyte(a, l, 3);  // 2x-1 2x 2x+1
                    w1 = a;                                    // . 2x+1 2x+2 2x+3
                    w2 = __builtin_amdgcn_alignbyte(b, a, 3);  // 2x+3 2x+4 2x+5
                    w3 = b;                                    // . 2x+5 2x+6 2x+7
                }
                acc[ch][0] = __builtin_amdgcn_sdot4((int)w0, (int)wq[dy][ch], acc[ch][0], false);
                acc[ch][1] = __builtin_amdgcn_sdot4((int)w1, (int)ws[dy][ch], acc[ch][1], false);
                acc[ch][2] = __builtin_amdgcn_sdot4((int)w2, (int)wq[dy][ch], acc[ch][2], false);
                acc[ch][3] = __builtin_amdgcn_sdot4((int)w3, (int)ws[dy][ch], acc[ch][3], false);
            }
        }
        int r[4][4];
        if (q.dw_ad != 0.f) {  // (uniform)
#pragma unroll
            for (int ch = 0; ch < 4; ++ch)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    r[ch][j] = pwdw_requant_affine(acc[ch][j], q.dw_ac, q.dw_ad, q.dw_lo);
        } else {
#pragma unroll
            for (int ch = 0; ch < 4; ++ch)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    r[ch][j] = pwdw_requant_table(acc[ch][j], q.dw_c, q.dw_lo, tbl_dw);
        }
        v4u o;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            o[j] = pack4_perm(r[0][j], r[1][j], r[2][j], r[3][j]);
        uint32_t* const d = out_plane + oy * q.OW + 4 * xq;
        if (4 * xq + 3 < q.OW) {
            *(v4u_a4*)d = o;  // (one 16-byte store; rows of e.g. 14 pixels leave it dword-aligned only)
        } else {
#pragma unroll
            for (int j = 0; j < 3; ++j)
                if (4 * xq + j < q.OW)
                    d[j] = o[j];
        }
    }
}

static int pwdw_lgp(int w) {
    int lg = 3;
    while ((1 << lg) < w + 1)
        ++lg;
    return lg;
}
static int pwdw_plane_stride(int h, int w) {
    int bytes = 4 + (h + 2) * (1 << pwdw_lgp(w)) + 4;  // a cleared dword in front and behind
    if (((bytes >> 2) & 1) == 0)
        bytes += 4;  // an odd number of dwords: the planes of 32 lanes start in 32 different banks
    return bytes;
}
// Channels per workgroup. Two workgroups fit a CU while one stays under half the LDS and 128 vector
// registers, and the three phases of one then overlap the other's: 64 channels do (a pointwise job
// then holds 2 x 16 accumulators); 128 only for images of a few 32-pixel tiles, where a job is one
// 32-channel tile and 128 channels give every wave one.
static size_t pwdw_lds_bytes(const ConvGeom& pw, int ocs);
static int pwdw_tiles(const ConvGeom& pw) {
    const int rpt = 32 >> pwdw_lgp(pw.iw);
    return (pw.ih + rpt - 1) / rpt;
}
static int pwdw_slice(const ConvGeom& pw) {
    if ((pw.oc & 127) == 0 && pwdw_tiles(pw) < 6 && pwdw_lds_bytes(pw, 128) <= 80 * 1024)
        return 128;
    // a batch that leaves CUs without a workgroup at 64 channels: 32; also when 64 planes of a large
    // image do not fit the LDS (32 always do: at most 64 rows of 32 bytes and 512 input channels)
    return (long)pw.n * (pw.oc / 64) < 256 || pwdw_lds_bytes(pw, 64) > 160 * 1024 ? 32 : 64;
}
static size_t pwdw_lds_bytes(const ConvGeom& pw, int ocs) {
    return (size_t)pw.ic * ocs + 2 * REQUANT_TABLE_ENTRIES * 4 + 2 * ocs * 4 +
           ((size_t)ocs * pwdw_plane_stride(pw.ih, pw.iw) + 16 + 15) / 16 * 16;
}

// pw: the pointwise layer (its s_dst is the scale of the tensor in between); dw: the channel-wise one
bool conv_pw_dw_supported(const ConvGeom& pw, const ConvGeom& dw, const void* src, const void* dst) {
    auto act_ok = [](const ConvGeom& g) {
        return (g.act == MEGCC_NONLINE_IDENTITY || g.act == MEGCC_NONLINE_RELU) &&
               requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    };
    if (!(pw.fmt == MEGCC_FMT_NCHW44 && pw.groups == 1 && pw.fh == 1 && pw.fw == 1 && pw.sh == 1 && pw.sw == 1 &&
          pw.ph == 0 && pw.pw == 0 && (pw.ic == 128 || pw.ic == 256 || pw.ic == 512) && (pw.oc & 63) == 0 &&
          pw.oc > 0 && pw.n > 0))
        return false;
    if (!(dw.fmt == MEGCC_FMT_NCHW44 && dw.groups == dw.ic && dw.ic == dw.oc && dw.oc == pw.oc && dw.n == pw.n &&
          dw.ih == pw.oh && dw.iw == pw.ow && dw.fh == 3 && dw.fw == 3 && dw.ph == 1 && dw.pw == 1 && dw.dh == 1 &&
          dw.dw == 1 && dw.sh == dw.sw && (dw.sh == 1 || dw.sh == 2) && dw.oh > 0 && dw.ow > 0))
        return false;
    if (!(pw.iw >= 4 && pw.iw <= 31 && pw.ih >= 1 && pw.ih <= 64 && act_ok(pw) && act_ok(dw)))
        return false;
    if (pwdw_lds_bytes(pw, pwdw_slice(pw)) > 160 * 1024)
        return false;
    return ((uintptr_t)src & 3) == 0 && ((uintptr_t)dst & 3) == 0 &&
           (long)pw.n * pw.ic * pw.ih * pw.iw < (1L << 31) && (long)dw.n * dw.oc * dw.oh * dw.ow < (1L << 31) &&
           (long)pw.n * (pw.oc / 64) < (1L << 31);
}

TinyNNStatus conv_pw_dw_launch(
        const ConvGeom& pw, const ConvGeom& dw, const void* src, const void* packed, const void* pw_bias,
        const void* dw_flt, const void* dw_bias, void* dst) {
    PwDwParams q = {};
    q.src = (const int8_t*)src;
    q.wp = (const int8_t*)packed;
    q.pw_bias = (const int32_t*)pw_bias;
    q.dw_flt = (const uint32_t*)dw_flt;
    q.dw_bias = (const int32_t*)dw_bias;
    q.dst = (uint32_t*)dst;
    q.src_bytes = (int)((long)pw.n * pw.ic * pw.ih * pw.iw);
    q.IC4 = pw.ic >> 2;
    q.H = pw.ih;
    q.W = pw.iw;
    q.HW = pw.ih * pw.iw;
    q.OH = dw.oh;
    q.OW = dw.ow;
    q.OC4 = pw.oc >> 2;
    q.OCP = (pw.oc + OC_PAD - 1) / OC_PAD * OC_PAD;
    q.lgP = pwdw_lgp(pw.iw);
    const int rpt = 32 >> q.lgP;
    q.tiles = (pw.ih + rpt - 1) / rpt;
    q.XQ = (dw.ow + 3) / 4;
    q.items = dw.oh * q.XQ;
    q.dXQ = make_fastdiv(q.XQ);
    q.plane_stride = pwdw_plane_stride(pw.ih, pw.iw);
    const int ocs = pwdw_slice(pw);
    q.slices = pw.oc / ocs;
    q.pw_lo = pw.act == MEGCC_NONLINE_RELU ? 0 : -128;
    q.dw_lo = dw.act == MEGCC_NONLINE_RELU ? 0 : -128;
    q.pw_c = make_requant_fast(pw.s_src, pw.s_flt, pw.s_dst).c;
    q.dw_c = make_requant_fast(dw.s_src, dw.s_flt, dw.s_dst).c;
    q.pw_table = requant_table_for(pw.act, pw.s_src, pw.s_flt, pw.s_dst);
    q.dw_table = requant_table_for(dw.act, dw.s_src, dw.s_flt, dw.s_dst);
    const RequantAffine a0 = requant_affine_pick(true, pw.act, pw.s_src, pw.s_flt, pw.s_dst);
    const RequantAffine a1 = requant_affine_pick(true, dw.act, dw.s_src, dw.s_flt, dw.s_dst);
    q.pw_ac = a0.c;
    q.pw_ad = a0.d;
    q.dw_ac = a1.c;
    q.dw_ad = a1.d;
    note_requant_affine(a0.d != 0.f && a1.d != 0.f);  // (the kernel's name says so when both layers use it)
    const int kc = pw.ic / 32;
    // enough 32-pixel tiles for every wave: a job takes the whole slice (64 channels then, see pwdw_slice)
    const bool whole = q.tiles >= 6;
    const void* kern = nullptr;
#define MG_PWDW_PICK(KC_, OCS_, JT_)                                          \
    (dw.sh == 1 ? (const void*)conv_pw_dw_kernel<KC_, OCS_, 1, JT_> : (const void*)conv_pw_dw_kernel<KC_, OCS_, 2, JT_>)
    if (ocs == 128)
        kern = kc == 4 ? MG_PWDW_PICK(4, 128, 1) : kc == 8 ? MG_PWDW_PICK(8, 128, 1) : MG_PWDW_PICK(16, 128, 1);
    else if (ocs == 32)
        kern = kc == 4 ? MG_PWDW_PICK(4, 32, 1) : kc == 8 ? MG_PWDW_PICK(8, 32, 1) : MG_PWDW_PICK(16, 32, 1);
    else if (whole)
        kern = kc == 4 ? MG_PWDW_PICK(4, 64, 2) : kc == 8 ? MG_PWDW_PICK(8, 64, 2) : MG_PWDW_PICK(16, 64, 2);
    else
        kern = kc == 4 ? MG_PWDW_PICK(4, 64, 1) : kc == 8 ? MG_PWDW_PICK(8, 64, 1) : MG_PWDW_PICK(16, 64, 1);
#undef MG_PWDW_PICK
    const size_t lds = pwdw_lds_bytes(pw, ocs);
    MG_REQUIRE(lds <= 160 * 1024, TinyNN_ERROR_OUT_OF_RANGE, "conv_pw_dw: %zu bytes of LDS", lds);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_pw_dw: LDS attribute: %s", hipGetErrorString(e));
    }
    void* args[] = {&q};
    hipError_t e = hipLaunchKernel(
            kern, dim3((unsigned)(pw.n * q.slices)), dim3(PWDW_THREADS), args, lds, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_pw_dw: launch: %s", hipGetErrorString(e));
    return check_launch("conv_pw_dw");
}

}  // namespace mg
