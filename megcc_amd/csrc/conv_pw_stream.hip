// qsi8 pointwise (1x1, stride 1) NCHW44 convolution with few input channels: a streaming kernel.
//
// With K = IC <= 512 a pointwise layer does one to sixteen MFMAs per 32 x 32 output tile and then
// requantises 16 outputs per lane: the layer is bound by HBM and by the epilogue's vector
// instructions, not by the matrix cores, and any staging through LDS (barriers, stage buffers,
// one workgroup per CU) only adds latency. So nothing is staged:
//   * a wave owns 64 output channels (32 with 512 input channels) and keeps their filter rows in
//     registers for its whole life (MFMA row tiles x IC/32 K-chunks x 4 VGPRs, read once from the
//     packed filter);
//   * it walks over 32-pixel tiles; the MFMA B operand of a tile is exactly what NCHW44 holds per
//     lane - lane (pixel l & 31, K-half l >> 5) needs 16 consecutive channels = one dword from
//     each of 4 consecutive channel planes - so it is loaded straight from global memory, 128
//     contiguous bytes per plane and half wave, the next tile's loads issued before the current
//     tile's MFMAs;
//   * results leave like in the tiled kernels: 4 consecutive accumulator registers are the 4
//     channels of one NCHW44 dword, 32 lanes store 128 contiguous bytes.
// Waves never synchronise after the set-up (threshold table and bias to LDS), so any number of
// them can be resident and the memory latency is hidden by occupancy.
//
// Same arithmetic as the other qsi8 kernels: int32 accumulators starting from the bias, exact
// requantisation by threshold table (epilogue.h). Reference loop: BareMetal/ConvKernel.cpp:305-344.
#include <stdlib.h>

#include <map>
#include <mutex>

#include "conv_mfma_i8.h"

namespace mg {

static constexpr int PW_THREADS = 256;
static constexpr int PW_MAX_OC = 1024;

struct PwParams {
    const int8_t* src;
    const int8_t* wp;  // packed filter [IC/32][OCP][32], 16-byte halves swapped when (oc >> 3) & 1
    const int32_t* bias;
    uint32_t* dst;
    int src_bytes;
    int IC4;           // input channel planes (IC / 4)
    int P, OHW, OC, OCP;
    int tiles;         // ceil(P / 32)
    int groups;        // OC / channels per wave
    int image_stride;  // bytes
    int plane_stride;  // bytes
    int act;
    float s_src, s_flt, s_dst, c;
    float aff_c, aff_d;  // requantisation by one fused multiply-add (epilogue.h); aff_d == 0: table
    FastDiv dOHW;
    RequantTable table;
};

__device__ __forceinline__ int pw_kernarg_table(int i) {
    typedef const __attribute__((address_space(4))) char* kptr;
    const kptr base = (kptr)__builtin_amdgcn_kernarg_segment_ptr();
    return *(const __attribute__((address_space(4))) int*)(base + offsetof(PwParams, table) + 4 * i);
}

// KC: 32-channel K chunks (IC = 32 * KC). ACT: IDENTITY / RELU use the table, -1 evaluates the
// literal sequence with the run-time activation.
// MT: 32-channel MFMA row tiles per wave (a wave owns 32 * MT output channels).
// RG: ragged channel counts - IC below 32 * KC (the planes beyond IC are not fetched: out-of-range
// offset, zeros; the packed filter holds zeros there too) and / or OC no multiple of 32 * MT (the last
// wave's surplus channels are computed from zero filter rows and not stored).
template <int KC, int MT, int ACT, bool RG = false>
__global__ void __launch_bounds__(PW_THREADS) conv_pw_stream_kernel(PwParams q) {
    __shared__ int tbl[REQUANT_TABLE_ENTRIES];
    __shared__ __attribute__((aligned(16))) int bias_lds[PW_MAX_OC];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, kg = lane >> 5;
    // wave -> (64-channel group, first tile, tile step); the grid holds a multiple of `groups` waves
    const int gw = blockIdx.x * (PW_THREADS / 64) + wave;
    const int nw = gridDim.x * (PW_THREADS / 64);
    const int og = gw % q.groups;
    // each wave walks a contiguous run of tiles: its loads and stores stream through every
    // channel plane in address order
    const int per = (q.tiles + nw / q.groups - 1) / (nw / q.groups);
    int t = (gw / q.groups) * per;
    const int tend = min(t + per, q.tiles);

    v4i A[MT][KC];
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) {
        const int oc = og * (32 * MT) + mi * 32 + col;
#pragma unroll
        for (int c = 0; c < KC; ++c)
            A[mi][c] = *(const v4i*)(q.wp + ((size_t)c * q.OCP + oc) * KROW + (((kg ^ (oc >> 3)) & 1) << 4));
    }

    const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void*)q.src, 0, q.src_bytes, 0x00020000);
    // ---- B operand: a ring of RING 32-channel chunks in flight per wave ------------------------
    // The memory latency is several times the time a tile takes, so chunks are requested RING
    // positions ahead of their MFMA in the sequence (tile, chunk) -> tile * KC + chunk: four tiles
    // ahead with 32 input channels, half a tile with 512. The loop is unrolled over U tiles so that
    // every ring slot and every "which tile, which chunk" below is a compile-time constant.
    constexpr int RING = KC == 1 ? 4 : KC == 2 ? 6 : KC >= 16 ? 16 : 8;
    constexpr int U = RING > KC ? RING / KC : 1;           // tiles per unrolled step
    constexpr int AHEAD = (RING + KC - 1) / KC;            // tiles a request can be ahead
    static_assert(RING % KC == 0 || KC % RING == 0, "slots repeat every U tiles");
    static_assert(4 * (KC * MT + RING) <= 192, "filter rows and chunks in flight must fit the registers");
    // byte offset of a tile's pixel in plane 0, or out of range (reads as zero) beyond the
    // wave's run / the last pixel
    auto tile_base = [&](int tile) __attribute__((always_inline)) -> unsigned {
        const int p = tile * 32 + col;
        const int n = fdiv(p, q.dOHW);
        return tile < tend && p < q.P
                       ? (unsigned)(n * q.image_stride + (p - n * q.OHW) * 4 + kg * 4 * q.plane_stride)
                       : 0x80000000u;
    };
    const int planes_left = q.IC4 - 4 * kg;  // RG: this lane reads plane c * 8 + j while that is below
    auto load_chunk = [&](unsigned base, int c, v4i& dst) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            unsigned off = base + (unsigned)((c * 8 + j) * q.plane_stride);
            if (RG)
                off = c * 8 + j < planes_left ? off : 0x80000000u;
            dst[j] = (int)__builtin_amdgcn_raw_buffer_load_b32(rs, (int)off, 0, 0);
        }
    };

    v4i ring[RING];
    static_for<RING>([&](auto sc) {
        constexpr int s = decltype(sc)::value;
        load_chunk(tile_base(t + s / KC), s % KC, ring[s]);
    });

    // threshold table and bias to LDS while those loads are in flight
    if (ACT >= 0)
        tbl[tid] = pw_kernarg_table(tid);
    for (int i = tid; i < (RG ? q.groups * (32 * MT) : q.OC); i += PW_THREADS)
        bias_lds[i] = q.bias && i < q.OC ? q.bias[i] : 0;
    __syncthreads();

    for (; t < tend; t += U) {
        unsigned base[U + AHEAD];  // of tiles t, t + 1, ...: the targets of this step's requests
        static_for<U + AHEAD>([&](auto kc) {
            constexpr int k = decltype(kc)::value;
            base[k] = tile_base(t + k);
        });
        static_for<U>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            const int tile = t + u;
            if (tile < tend) {
                v16i acc[MT];
#pragma unroll
                for (int mi = 0; mi < MT; ++mi) {
                    // register e of a tile: channel 8 * (e / 4) + 4 * kg + e % 4
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4) {
                        const v4i bv = *(const v4i*)(bias_lds + og * (32 * MT) + mi * 32 + e4 * 8 + kg * 4);
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            acc[mi][e4 * 4 + k] = bv[k];
                    }
                }
                static_for<KC>([&](auto cc) {
                    constexpr int c = decltype(cc)::value;
                    constexpr int s = u * KC + c, slot = s % RING;
#pragma unroll
                    for (int mi = 0; mi < MT; ++mi)
                        acc[mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[mi][c], ring[slot], acc[mi], 0, 0, 0);
                    // the slot is free again: request the chunk RING positions ahead
                    load_chunk(base[(s + RING) / KC], (s + RING) % KC, ring[slot]);
                });

                const int p = tile * 32 + col;
                const bool ok = p < q.P;
                const int n = fdiv(p, q.dOHW);
                const int obase = n * (q.OC >> 2) * q.OHW + (p - n * q.OHW);
#pragma unroll
                for (int mi = 0; mi < MT; ++mi) {
                    if (RG && (og * MT + mi) * 32 >= q.OC)  // (wave-uniform: a tile of surplus channels)
                        continue;
                    int r[16];
                    if (ACT < 0) {
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            r[e] = requant_conv_rt(q.act, acc[mi][e], q.s_src, q.s_flt, q.s_dst);
                    } else if (q.aff_d != 0.f) {  // (uniform)
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            r[e] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(acc[mi][e], q.aff_c, q.aff_d);
                    } else {
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            r[e] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(acc[mi][e], q.c, tbl);
                    }
                    if (ok) {
#pragma unroll
                        for (int e4 = 0; e4 < 4; ++e4) {
                            const int oc4 = og * (8 * MT) + mi * 8 + e4 * 2 + kg;
                            if (!RG || oc4 * 4 < q.OC)
                                q.dst[obase + oc4 * q.OHW] =
                                        pack4_perm(r[e4 * 4], r[e4 * 4 + 1], r[e4 * 4 + 2], r[e4 * 4 + 3]);
                        }
                    }
                }
            }
        });
    }
}


// The same layer with the activation tile SHARED by the four waves of a workgroup (512 input
// channels): the waves own four neighbouring 32-channel groups and the same run of pixel tiles; the
// MFMA B operand of a tile does not depend on the channel group, so each wave fetches a quarter
// of a tile's 16 chunks (16 dword loads instead of 64) and parks them in LDS exactly as the lanes
// will read them back (chunk c, lane l at c * 1 KB + l * 16: consecutive lanes, consecutive 16-byte
// words, no bank conflicts). Two LDS tiles: the chunks of tile t + 1 are requested before tile t
// is computed and written after it, one barrier per tile. A quarter of the L2 traffic and of the
// load instructions of the streaming form.
template <int KC, int ACT>
__global__ void __launch_bounds__(PW_THREADS) conv_pw_share_kernel(PwParams q) {
    static_assert(KC % 4 == 0, "a quarter of the chunks per wave");
    constexpr int CW = KC / 4;  // chunks a wave fetches per tile
    __shared__ int tbl[REQUANT_TABLE_ENTRIES];
    __shared__ __attribute__((aligned(16))) int bias_lds[PW_MAX_OC];
    __shared__ __attribute__((aligned(16))) int8_t btile[2][KC * 1024];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, kg = lane >> 5;
    // workgroup -> (block of 4 channel groups, run of tiles)
    const int gblocks = q.groups >> 2;
    const int gb = blockIdx.x % gblocks;
    const int runs = gridDim.x / gblocks;
    const int og = gb * 4 + wave;
    const int per = (q.tiles + runs - 1) / runs;
    const int t0 = (blockIdx.x / gblocks) * per;
    const int tend = min(t0 + per, q.tiles);

    v4i A[KC];
    {
        const int oc = og * 32 + col;
#pragma unroll
        for (int c = 0; c < KC; ++c)
            A[c] = *(const v4i*)(q.wp + ((size_t)c * q.OCP + oc) * KROW + (((kg ^ (oc >> 3)) & 1) << 4));
    }
    const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void*)q.src, 0, q.src_bytes, 0x00020000);
    auto tile_base = [&](int tile) __attribute__((always_inline)) -> unsigned {
        const int p = tile * 32 + col;
        const int n = fdiv(p, q.dOHW);
        return tile < tend && p < q.P
                       ? (unsigned)(n * q.image_stride + (p - n * q.OHW) * 4 + kg * 4 * q.plane_stride)
                       : 0x80000000u;
    };
    // this wave's chunks wave * CW .. + CW - 1 of `tile`
    auto request = [&](int tile, v4i (&r)[CW]) __attribute__((always_inline)) {
        const unsigned base = tile_base(tile);
#pragma unroll
        for (int k = 0; k < CW; ++k)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                r[k][j] = (int)__builtin_amdgcn_raw_buffer_load_b32(
                        rs, (int)(base + (unsigned)(((wave * CW + k) * 8 + j) * q.plane_stride)), 0, 0);
    };
    auto park = [&](int buf, const v4i (&r)[CW]) __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < CW; ++k)
            *(v4i*)(btile[buf] + (wave * CW + k) * 1024 + lane * 16) = r[k];
    };

    v4i nxt[CW];
    request(t0, nxt);
    if (ACT >= 0)
        tbl[tid] = pw_kernarg_table(tid);
    for (int i = tid; i < q.OC; i += PW_THREADS)
        bias_lds[i] = q.bias ? q.bias[i] : 0;
    park(0, nxt);
    __syncthreads();

    for (int t = t0, buf = 0; t < tend; ++t, buf ^= 1) {
        if (t + 1 < tend)
            request(t + 1, nxt);
        v16i acc;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
            const v4i bv = *(const v4i*)(bias_lds + og * 32 + e4 * 8 + kg * 4);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                acc[e4 * 4 + k] = bv[k];
        }
        // two accumulator chains (even and odd chunks): a dependent MFMA can only issue when the one
        // before it has left the pipe, two chains keep the matrix core busy between them
        v16i acc1 = {};
#pragma unroll
        for (int c = 0; c < KC; c += 2) {
            const v4i b0 = *(const v4i*)(btile[buf] + c * 1024 + lane * 16);
            const v4i b1 = *(const v4i*)(btile[buf] + (c + 1) * 1024 + lane * 16);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[c], b0, acc, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[c + 1], b1, acc1, 0, 0, 0);
        }
        acc += acc1;
        const int p = t * 32 + col;
        const bool ok = p < q.P;
        const int n = fdiv(p, q.dOHW);
        const int obase = n * (q.OC >> 2) * q.OHW + (p - n * q.OHW);
        int r[16];
        if (ACT < 0) {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                r[e] = requant_conv_rt(q.act, acc[e], q.s_src, q.s_flt, q.s_dst);
        } else if (q.aff_d != 0.f) {  // (uniform)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                r[e] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(acc[e], q.aff_c, q.aff_d);
        } else {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                r[e] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(acc[e], q.c, tbl);
        }
        if (ok) {
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int oc4 = og * 8 + e4 * 2 + kg;
                q.dst[obase + oc4 * q.OHW] = pack4_perm(r[e4 * 4], r[e4 * 4 + 1], r[e4 * 4 + 2], r[e4 * 4 + 3]);
            }
        }
        if (t + 1 < tend)
            park(buf ^ 1, nxt);
        __syncthreads();
    }
}

// workgroups of `kern` one CU holds at a time
static int pw_resident_blocks(const void* kern) {
    static std::map<const void*, int> cache;
    static std::mutex lock;
    std::lock_guard<std::mutex> guard(lock);
    auto it = cache.find(kern);
    if (it != cache.end())
        return it->second;
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, PW_THREADS, 0) != hipSuccess || n < 1)
        n = 2;
    return cache[kern] = n;
}

bool conv_pw_stream_supported(const ConvGeom& g) {
    const long P = (long)g.n * g.oh * g.ow;
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups == 1 && g.fh == 1 && g.fw == 1 && g.sh == 1 &&
           g.sw == 1 && g.ph == 0 && g.pw == 0 && (g.ic & 3) == 0 && (g.oc & 3) == 0 && (g.ic <= 512 ||
            // (1024: layers too small for the LDS-staged kernel, where one round trip wins, and the
            //  workgroup-shared form up to a few thousand pixels)
            (g.ic == 1024 && (P < 2048 || (P <= 4096 && (g.oc & 127) == 0 && !options().no_pwshare &&
                                         (P + 31) / 32 * (g.oc / 128) >= 256)))) &&
           ((g.oc & 63) == 0 || g.ic <= 512) && g.oc <= PW_MAX_OC && P >= 32 &&
           (long)g.n * g.ic * g.ih * g.iw < (1L << 31) && P * g.oc < (1L << 31);
}

TinyNNStatus conv_pw_stream_launch(
        const ConvGeom& g, const void* src, const void* packed, const void* bias, void* dst) {
    PwParams q = {};
    q.src = (const int8_t*)src;
    q.wp = (const int8_t*)packed;
    q.bias = (const int32_t*)bias;
    q.dst = (uint32_t*)dst;
    q.src_bytes = (int)((long)g.n * g.ic * g.ih * g.iw);
    q.OHW = g.oh * g.ow;
    q.P = g.n * q.OHW;
    q.OC = g.oc;
    q.OCP = (g.oc + OC_PAD - 1) / OC_PAD * OC_PAD;
    q.tiles = (q.P + 31) / 32;
    q.IC4 = g.ic >> 2;
    // (ragged channel counts: IC below the next power of two of 32-channel chunks, OC no multiple of
    //  a wave's 64 / 32 channels)
    const int chunks = (g.ic + 31) / 32;
    const int kc = chunks <= 1 ? 1 : chunks <= 2 ? 2 : chunks <= 4 ? 4 : chunks <= 8 ? 8 : chunks <= 16 ? 16 : 32;
    const int per_wave = kc > 8 ? 32 : 64;
    const bool ragged = g.ic != kc * 32 || g.oc % per_wave != 0;
    q.groups = (g.oc + per_wave - 1) / per_wave;
    q.image_stride = g.ic * q.OHW;
    q.plane_stride = q.OHW * 4;
    q.act = g.act;
    q.s_src = g.s_src;
    q.s_flt = g.s_flt;
    q.s_dst = g.s_dst;
    q.c = make_requant_fast(g.s_src, g.s_flt, g.s_dst).c;
    q.dOHW = make_fastdiv(q.OHW);
    const bool tab = requant_table_act(g.act) && requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    if (tab)
        q.table = requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst);
    const int act = tab ? g.act : -1;

    const void* kern = nullptr;
#define MG_PW_PICK_RG(KC_, MT_, RG_)                                                                      \
    (act == MEGCC_NONLINE_IDENTITY ? (const void*)conv_pw_stream_kernel<KC_, MT_, MEGCC_NONLINE_IDENTITY, RG_> \
     : act == MEGCC_NONLINE_RELU   ? (const void*)conv_pw_stream_kernel<KC_, MT_, MEGCC_NONLINE_RELU, RG_>     \
     : act == MEGCC_NONLINE_H_SWISH ? (const void*)conv_pw_stream_kernel<KC_, MT_, MEGCC_NONLINE_H_SWISH, RG_> \
                                   : (const void*)conv_pw_stream_kernel<KC_, MT_, -1, RG_>)
#define MG_PW_PICK(KC_, MT_) (ragged ? MG_PW_PICK_RG(KC_, MT_, true) : MG_PW_PICK_RG(KC_, MT_, false))
    switch (kc) {
        case 1: kern = MG_PW_PICK(1, 2); break;
        case 2: kern = MG_PW_PICK(2, 2); break;
        case 4: kern = MG_PW_PICK(4, 2); break;
        case 8: kern = MG_PW_PICK(8, 2); break;
        case 16: kern = MG_PW_PICK(16, 1); break;  // 512 input channels: 32 output channels per wave
        default: kern = MG_PW_PICK_RG(32, 1, false); break;  // 1024: the filter rows fill half the registers
    }
#undef MG_PW_PICK
#undef MG_PW_PICK_RG

    // 512 input channels and more tiles than resident waves: the workgroup-shared form
    if ((g.ic == 512 || g.ic == 1024) && !ragged && (q.groups & 3) == 0 && !options().no_pwshare) {
#define MG_PWS_PICK(KC_)                                                                                  \
    (act == MEGCC_NONLINE_IDENTITY ? (const void*)conv_pw_share_kernel<KC_, MEGCC_NONLINE_IDENTITY>         \
     : act == MEGCC_NONLINE_RELU   ? (const void*)conv_pw_share_kernel<KC_, MEGCC_NONLINE_RELU>             \
     : act == MEGCC_NONLINE_H_SWISH ? (const void*)conv_pw_share_kernel<KC_, MEGCC_NONLINE_H_SWISH>         \
                                   : (const void*)conv_pw_share_kernel<KC_, -1>)
        const void* sk = g.ic == 512 ? MG_PWS_PICK(16) : MG_PWS_PICK(32);
#undef MG_PWS_PICK
        const long gblocks = q.groups / 4;
        const long capb = (long)num_cus() * pw_resident_blocks(sk);
        if ((long)q.tiles * gblocks >= capb / 2) {
            long runs = capb / gblocks;
            if (runs > q.tiles)
                runs = q.tiles;
            if (runs < 1)
                runs = 1;
            void* sargs[] = {&q};
            note_kernel("conv_pw_share", g.ic / 32);
            const RequantAffine aff = requant_affine_pick(tab, g.act, g.s_src, g.s_flt, g.s_dst);
            q.aff_c = aff.c;
            q.aff_d = aff.d;
            hipError_t e = hipLaunchKernel(sk, dim3((unsigned)(runs * gblocks)), dim3(PW_THREADS), sargs, 0, stream());
            MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_pw_share: %s", hipGetErrorString(e));
            return check_launch("conv_pw_share");
        }
    }
    // waves: a multiple of `groups`; one per (tile, channel group) while they are all resident at
    // once - a small layer is then one memory round trip - and never more than are resident (every
    // wave pays the set-up once and then streams over its tiles)
    const long items = (long)q.tiles * q.groups;
    const long cap = (long)num_cus() * 4 * pw_resident_blocks(kern);
    long waves = items < cap ? items : cap;
    long gcd = q.groups, rest = 4;  // unit = lcm(groups, waves per workgroup)
    while (rest) {
        const long r = gcd % rest;
        gcd = rest;
        rest = r;
    }
    const long unit = (long)q.groups * 4 / gcd;
    waves = (waves + unit - 1) / unit * unit;
    const unsigned blocks = (unsigned)(waves / 4);

    note_kernel("conv_pw_stream", kc, ragged);
    const RequantAffine aff = requant_affine_pick(tab, g.act, g.s_src, g.s_flt, g.s_dst);
    q.aff_c = aff.c;
    q.aff_d = aff.d;
    void* args[] = {&q};
    hipError_t e = hipLaunchKernel(kern, dim3(blocks), dim3(PW_THREADS), args, 0, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_pw_stream: %s", hipGetErrorString(e));
    return check_launch("conv_pw_stream");
}

}  // namespace mg
