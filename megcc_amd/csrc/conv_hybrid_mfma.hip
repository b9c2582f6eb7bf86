// qsi8 NCHW -> NCHW44 ("hybrid" first layer) convolution for any filter up to 8 x 8, stride 1 or 2,
// 1..4 input channels - the 7x7 stride-2 stem of ResNet-like networks, 5x5 and stride-1 3x3
// stems. Filter [OC/4, FH, FW, IC, 4 oc], same loop nest and epilogue as
// BareMetal/ConvKernel.cpp:305-344,374-380 (format detection :115-127).
//
// K = IC * FH * FW is at most 147 here, too short for a staged GEMM but long enough that the
// per-tap VALU kernel of the 3x3 case would spend thousands of instructions per pixel. So the
// reduction index is re-ordered to make the matrix cores usable without an im2col:
//     k' = (ic * FH + fh) * 8 + fw          (fw padded to 8, zero weights in the padding)
// A lane's 16 K-bytes of an MFMA B operand are then two (ic, fh) rows x 8 consecutive input
// columns: 8 bytes that lie next to each other in an LDS copy of the input rows under a strip of
// output pixels. They are read as the three aligned dwords around them and shifted into place.
//   * a workgroup walks over strips of 128 output pixels x R consecutive output rows (a wave: 32
//     pixels x all output channels, one output row after the other); per strip the
//     IC * (FH + (R - 1) * S) input row pieces go to LDS once, zero where the image ends - padding
//     costs nothing later, and neighbouring output rows share most of their input rows;
//   * the filter is copied to LDS with coalesced loads and re-ordered there to k' once per
//     workgroup ([chunk of 32 k'][oc][32 bytes]); every wave then keeps its MFMA A operands (all
//     chunks x output-channel tiles) in registers;
//   * accumulators start from the bias, exact requantisation by threshold table, 4 consecutive
//     accumulator registers = one NCHW44 dword, 32 lanes store 128 contiguous bytes.
#include <algorithm>
#include <map>
#include <mutex>

#include "common.h"
#include "conv_geom.h"
#include "conv_mfma_i8.h"
#include "epilogue.h"

namespace mg {

static constexpr int CH_MAX_OC = 128;    // output channels (4 MFMA row tiles)
static constexpr int CH_MAX_ROWS = 32;   // IC * FH
static constexpr int CH_MAX_CHUNKS = CH_MAX_ROWS / 4;
static constexpr int CH_STRIP = 128;     // output pixels per strip
static constexpr int CH_FILL = 16;       // patch dwords a thread has in flight
static constexpr int CH_THREADS = 256;

struct ChParams {
    const int8_t* src;
    const int8_t* flt;
    const int32_t* bias;
    uint32_t* dst;
    int N, IC, IH, IW, OC, OH, OW, FH, FW, PH, PW;
    int rows;    // IC * FH
    int chunks;  // ceil(rows / 4)
    int octiles; // ceil(OC / 32)
    int pitch;   // bytes per LDS row: (CH_STRIP - 1) * S + 8, rounded up to 4
    int strips;  // per output row
    int R;       // output rows per item
    int RP;      // input rows per channel under R output rows: FH + (R - 1) * S
    int ohg;     // ceil(OH / R)
    int items;   // N * ohg * strips
    int fbytes;  // OC * FH * FW * IC
    int src_bytes;
    float inv_pitch4, inv_rp;  // 4 / pitch, 1 / RP
    int act;
    float s_src, s_flt, s_dst, c;
    float aff_c, aff_d;  // requantisation by one fused multiply-add (epilogue.h); aff_d == 0: table
    RequantTable table;
};

__device__ __forceinline__ int ch_kernarg_table(int i) {
    typedef const __attribute__((address_space(4))) char* kptr;
    const kptr base = (kptr)__builtin_amdgcn_kernarg_segment_ptr();
    return *(const __attribute__((address_space(4))) int*)(base + offsetof(ChParams, table) + 4 * i);
}

// S: stride. ACT: IDENTITY / RELU use the table, -1 the literal sequence. OT: MFMA row tiles (OC <= 32 * OT).
template <int S, int ACT, int OT>
__global__ void __launch_bounds__(CH_THREADS, OT == 1 ? 3 : 2) conv_hybrid_mfma_kernel(ChParams q) {
    extern __shared__ __attribute__((aligned(16))) int8_t ch_lds[];
    __shared__ int tbl[REQUANT_TABLE_ENTRIES];
    __shared__ __attribute__((aligned(16))) int bias_lds[CH_MAX_OC];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, kg = lane >> 5;
    const int ocp = OT * 32;
    int8_t* const wl = ch_lds;                              // [chunk][ocp][32]
    int8_t* const patch = ch_lds + q.chunks * ocp * 32;     // [IC][RP][pitch]; first the raw filter

    // ---- once per workgroup: filter in k' order, bias, thresholds, row offsets ------------------
    for (int i = tid; i < (q.fbytes >> 2); i += CH_THREADS)
        ((uint32_t*)patch)[i] = ((const uint32_t*)q.flt)[i];
    if (ACT >= 0 && tid < REQUANT_TABLE_ENTRIES)
        tbl[tid] = ch_kernarg_table(tid);
    for (int i = tid; i < ocp; i += CH_THREADS)
        bias_lds[i] = (q.bias && i < q.OC) ? q.bias[i] : 0;
    // k' row r = (ic, fh) lies in patch row ic * RP + fh (+ S per output row); rows beyond IC * FH
    // are multiplied by zero weights: any patch bytes do. Lane r of every wave keeps the offset of
    // row r; the chunk loop fetches its four rows with v_readlane.
    int rtab;
    {
        const int r = lane & 31, ic = r / q.FH;
        rtab = r < q.rows ? (ic * q.RP + r - ic * q.FH) * q.pitch : 0;
    }
    __syncthreads();
    // a thread makes 4 bytes of wl: one oc, one (ic, fh), fw0 .. fw0 + 3
    for (int i = tid; i < q.chunks * ocp * 8; i += CH_THREADS) {
        const int b4 = i & 7, oc = (i >> 3) % ocp, chunk = (i >> 3) / ocp;
        const int r = chunk * 4 + (b4 >> 1), fw0 = (b4 & 1) * 4;
        uint32_t v = 0;
        if (oc < q.OC && r < q.rows) {
            const int ic = r / q.FH, fh = r - ic * q.FH;
            const uint8_t* f = (const uint8_t*)patch +
                               ((((oc >> 2) * q.FH + fh) * q.FW + fw0) * q.IC + ic) * 4 + (oc & 3);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (fw0 + j < q.FW)
                    v |= (uint32_t)f[j * q.IC * 4] << (8 * j);
        }
        ((uint32_t*)wl)[i] = v;
    }
    __syncthreads();  // the raw filter is overwritten by the first patch

    // this wave's MFMA A operands (filter rows of all chunks) stay in registers
    // (up to 64 output channels; with more they would not fit and are read from LDS per use)
    constexpr bool AREG = OT <= 2;
    const int8_t* const wa = wl + col * 32 + kg * 16;
    v4i areg[AREG ? OT : 1][AREG ? CH_MAX_CHUNKS : 1];
    if (AREG) {
#pragma unroll
        for (int c = 0; c < CH_MAX_CHUNKS; ++c)
#pragma unroll
            for (int t = 0; t < OT; ++t)
                areg[t][c] = c < q.chunks ? *(const v4i*)(wa + (c * ocp + t * 32) * 32) : v4i{0, 0, 0, 0};
    }
    const int ohw = q.OH * q.OW;
    const int pitch4 = q.pitch >> 2;
    // ---- the input rows under a strip -> LDS (zero outside the image) -----------------------------
    // Element e = 4 columns of one patch row = one dword load from the byte address of its first
    // column (any alignment; rows outside the image get the out-of-range offset and read as zero);
    // the bytes left and right of the image row, which the load took from the neighbouring rows, are
    // masked. A dword that would start before the tensor or run past its end - the range check would
    // cut it off - is loaded from the nearest address inside and shifted into place. A thread takes
    // elements tid, tid + 256, ... and has CH_FILL of them in flight: a round trip to memory takes
    // microseconds while the chip writes at full rate, an item should need one or two.
    const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void*)q.src, 0, q.src_bytes, 0x00020000);
    const int total = q.IC * q.RP * pitch4;
    for (int item = blockIdx.x; item < q.items; item += gridDim.x) {
        const int sx = item % q.strips, grp = item / q.strips;
        const int n = grp / q.ohg, oh0 = (grp - n * q.ohg) * q.R;
        const int ow0 = sx * CH_STRIP;
        const int ih0 = oh0 * S - q.PH, iw0 = ow0 * S - q.PW;
        const int nout = min(q.R, q.OH - oh0);
        const int need = (nout - 1) * S + q.FH;  // rows per channel that the nout output rows read
        for (int e0 = tid; e0 < total; e0 += 256 * CH_FILL) {
            // where element e comes from: byte offset in the tensor, first column, wanted at all
            auto element = [&](int e, int& off, int& iw) __attribute__((always_inline)) -> bool {
                // e / pitch4 and row / RP by float: (x + 0.5) / d is at least 0.5 / d away from an
                // integer, far more than the rounding error for these small numbers
                const int prow = (int)(((float)e + 0.5f) * q.inv_pitch4);
                const int c4 = e - prow * pitch4;
                const int ic = (int)(((float)prow + 0.5f) * q.inv_rp);
                const int j = prow - ic * q.RP;
                const int ih = ih0 + j;
                iw = iw0 + c4 * 4;
                off = (n * q.IC + ic) * q.IH * q.IW + ih * q.IW + iw;
                return e < total && (unsigned)ih < (unsigned)q.IH && j < need && iw > -4 && iw < q.IW;
            };
            uint32_t d[CH_FILL];
#pragma unroll
            for (int u = 0; u < CH_FILL; ++u) {
                int off, iw;
                const bool want = element(e0 + u * 256, off, iw);
                d[u] = __builtin_amdgcn_raw_buffer_load_b32(
                        rs, want ? min(max(off, 0), q.src_bytes - 4) : (int)0x80000000u, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < CH_FILL; ++u) {
                int off, iw;
                (void)element(e0 + u * 256, off, iw);  // (again: cheaper than keeping it per load in flight)
                const int sh = off - min(max(off, 0), q.src_bytes - 4);  // -3 .. 3, 0 except at the tensor's ends
                const uint32_t v = sh > 0 ? d[u] >> (8 * sh) : d[u] << (-8 * sh);
                uint32_t keep = 0;
#pragma unroll
                for (int bb = 0; bb < 4; ++bb)
                    keep |= (unsigned)(iw + bb) < (unsigned)q.IW ? 0xffu << (8 * bb) : 0u;
                if (e0 + u * 256 < total)
                    ((uint32_t*)patch)[e0 + u * 256] = v & keep;
            }
        }
        lds_barrier();

        const int px = wave * 32 + col;          // pixel of the strip
        const int ow = ow0 + px;
        for (int orow = 0; orow < nout; ++orow) {
        const int oh = oh0 + orow;
        // ---- this wave's 32 pixels x all output channels
        v16i acc[OT];
#pragma unroll
        for (int t = 0; t < OT; ++t)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const v4i bv = *(const v4i*)(bias_lds + t * 32 + e4 * 8 + kg * 4);
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    acc[t][e4 * 4 + k] = bv[k];
            }
        // its window starts at byte px * S of every row: read as three aligned dwords from the dword
        // below it and shifted into place (lanes that share a dword get it by broadcast; reads of
        // two or eight single bytes kept the LDS pipe busy for 70 % of the kernel)
        const int woff = px * S + orow * S * q.pitch;
        const int wsh = woff & 3;
        const int8_t* pb = patch + (woff & ~3);
        // lane's K-bytes of a chunk: rows chunk * 4 + 2 kg, + 1; 8 columns each
        auto load_b = [&](int chunk) __attribute__((always_inline)) {
            const int r0 = __builtin_amdgcn_readlane(rtab, chunk * 4), r1 = __builtin_amdgcn_readlane(rtab, chunk * 4 + 1);
            const int r2 = __builtin_amdgcn_readlane(rtab, chunk * 4 + 2), r3 = __builtin_amdgcn_readlane(rtab, chunk * 4 + 3);
            const int ro[2] = {kg ? r2 : r0, kg ? r3 : r1};
            v4i b;
#pragma unroll
            for (int rr = 0; rr < 2; ++rr) {
                const uint32_t* p = (const uint32_t*)(pb + ro[rr]);
                const uint32_t d0 = p[0], d1 = p[1], d2 = p[2];
                b[rr * 2] = (int)__builtin_amdgcn_alignbyte(d1, d0, wsh);
                b[rr * 2 + 1] = (int)__builtin_amdgcn_alignbyte(d2, d1, wsh);
            }
            return b;
        };
        // all chunks' operands first, then the MFMAs against the filter rows kept in registers; one
        // straight-line copy per chunk count (the count is uniform)
        static_for<CH_MAX_CHUNKS>([&](auto ncc) {
            constexpr int NC = decltype(ncc)::value + 1;
            if (q.chunks == NC) {
                v4i b[NC];
#pragma unroll
                for (int c = 0; c < NC; ++c)
                    b[c] = load_b(c);
#pragma unroll
                for (int c = 0; c < NC; ++c)
#pragma unroll
                    for (int t = 0; t < OT; ++t)
                        acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                AREG ? areg[AREG ? t : 0][AREG ? c : 0] : *(const v4i*)(wa + (c * ocp + t * 32) * 32),
                                b[c], acc[t], 0, 0, 0);
            }
        });

        // ---- epilogue: register e of a tile = channel 8 * (e / 4) + 4 * kg + e % 4, pixel = col
        const int obase = (n * (q.OC >> 2)) * ohw + oh * q.OW + ow;
#pragma unroll
        for (int t = 0; t < OT; ++t) {
            int r[16];
            if (ACT < 0) {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    r[e] = requant_conv_rt(q.act, acc[t][e], q.s_src, q.s_flt, q.s_dst);
            } else if (q.aff_d != 0.f) {  // (uniform)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    r[e] = requant_conv_affine<(ACT == MEGCC_NONLINE_RELU ? ACT : 0)>(acc[t][e], q.aff_c, q.aff_d);
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    r[e] = requant_conv_table<(ACT < 0 ? 0 : ACT)>(acc[t][e], q.c, tbl);
            }
            if (ow < q.OW) {
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    const int oc4 = t * 8 + e4 * 2 + kg;
                    if (oc4 * 4 < q.OC)
                        q.dst[obase + oc4 * ohw] =
                                pack4_perm(r[e4 * 4], r[e4 * 4 + 1], r[e4 * 4 + 2], r[e4 * 4 + 3]);
                }
            }
        }
        }
        lds_barrier();  // the patch is rewritten for the next item
    }
}

bool conv_hybrid_mfma_supported(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW_NCHW44 && g.groups == 1 && g.ic >= 1 && g.ic <= 4 && g.fh >= 1 &&
           g.fw >= 1 && g.fw <= 8 && g.ic * g.fh <= CH_MAX_ROWS && g.sh == g.sw && (g.sh == 1 || g.sh == 2) &&
           g.dh == 1 && g.dw == 1 && (g.oc & 3) == 0 && g.oc >= 4 && g.oc <= CH_MAX_OC &&
           (long)g.n * g.ic * g.ih * g.iw < (1L << 31) && (long)g.n * g.ic * g.ih * g.iw >= 4 &&
           (long)g.n * g.oc * g.oh * g.ow < (1L << 31) &&
           (long)g.n * g.oh * ((g.ow + CH_STRIP - 1) / CH_STRIP) < (1L << 31);
}

TinyNNStatus conv_hybrid_mfma_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst) {
    ChParams q = {};
    q.src = (const int8_t*)src;
    q.flt = (const int8_t*)flt;
    q.bias = (const int32_t*)bias;
    q.dst = (uint32_t*)dst;
    q.N = g.n; q.IC = g.ic; q.IH = g.ih; q.IW = g.iw;
    q.OC = g.oc; q.OH = g.oh; q.OW = g.ow;
    q.FH = g.fh; q.FW = g.fw; q.PH = g.ph; q.PW = g.pw;
    q.rows = g.ic * g.fh;
    q.chunks = (q.rows + 3) / 4;
    q.octiles = (g.oc + 31) / 32;
    q.pitch = ((CH_STRIP - 1) * g.sh + 8 + 3) & ~3;
    q.strips = (g.ow + CH_STRIP - 1) / CH_STRIP;
    // up to 16 output rows per item share their input rows in LDS and one round trip to memory
    // (stride-1 stems: 102 us with 4 rows, 68 us with 16 on N=64 3->32 3x3 224x224); fewer when the
    // problem is too small to give every CU four items otherwise
    q.R = 16;
    while (q.R > 1 && (long)g.n * ((g.oh + q.R - 1) / q.R) * q.strips < 4L * num_cus())
        q.R >>= 1;
    q.src_bytes = (int)((long)g.n * g.ic * g.ih * g.iw);
    q.RP = g.fh + (q.R - 1) * g.sh;
    q.ohg = (g.oh + q.R - 1) / q.R;
    q.items = g.n * q.ohg * q.strips;
    q.fbytes = g.oc * g.fh * g.fw * g.ic;
    q.inv_pitch4 = 4.f / (float)q.pitch;
    q.inv_rp = 1.f / (float)q.RP;
    q.act = g.act;
    q.s_src = g.s_src; q.s_flt = g.s_flt; q.s_dst = g.s_dst;
    q.c = make_requant_fast(g.s_src, g.s_flt, g.s_dst).c;
    const bool tab = (g.act == MEGCC_NONLINE_IDENTITY || g.act == MEGCC_NONLINE_RELU) &&
                     requant_table_ok(g.s_src, g.s_flt, g.s_dst);
    if (tab)
        q.table = requant_table_for(g.act, g.s_src, g.s_flt, g.s_dst);
    const int act = tab ? g.act : -1;
    const RequantAffine aff = requant_affine_pick(tab, g.act, g.s_src, g.s_flt, g.s_dst);
    q.aff_c = aff.c;
    q.aff_d = aff.d;
    const void* kern = nullptr;
#define MG_CH_PICK(S_, OT_)                                                                             \
    (act == MEGCC_NONLINE_IDENTITY ? (const void*)conv_hybrid_mfma_kernel<S_, MEGCC_NONLINE_IDENTITY, OT_> \
     : act == MEGCC_NONLINE_RELU   ? (const void*)conv_hybrid_mfma_kernel<S_, MEGCC_NONLINE_RELU, OT_>     \
                                   : (const void*)conv_hybrid_mfma_kernel<S_, -1, OT_>)
    const int ot = q.octiles;
    if (g.sh == 1)
        kern = ot == 1 ? MG_CH_PICK(1, 1) : ot == 2 ? MG_CH_PICK(1, 2) : ot == 3 ? MG_CH_PICK(1, 3) : MG_CH_PICK(1, 4);
    else
        kern = ot == 1 ? MG_CH_PICK(2, 1) : ot == 2 ? MG_CH_PICK(2, 2) : ot == 3 ? MG_CH_PICK(2, 3) : MG_CH_PICK(2, 4);
#undef MG_CH_PICK
    // (+ 16: the aligned three-dword reads of a window may touch the dword behind the last row)
    const size_t lds = (size_t)q.chunks * ot * 32 * 32 +
                       std::max((size_t)g.ic * q.RP * q.pitch, (size_t)q.fbytes) + 16;

    // as many workgroups as are resident at once: the filter set-up is paid once per workgroup
    static std::map<std::pair<const void*, size_t>, int> per_cu;
    static std::mutex lock;
    int blocks_per_cu;
    {
        std::lock_guard<std::mutex> guard(lock);
        auto key = std::make_pair(kern, lds);
        auto it = per_cu.find(key);
        if (it == per_cu.end()) {
            if (lds > 48 * 1024)
                MG_REQUIRE(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) ==
                                   hipSuccess,
                           TinyNN_ERROR_RUNTIME, "conv_hybrid_mfma: LDS attribute");
            int nb = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kern, CH_THREADS, lds) != hipSuccess || nb < 1)
                nb = 1;
            it = per_cu.emplace(key, nb).first;
        }
        blocks_per_cu = it->second;
    }
    // every CU gets the same number of workgroups (they take items in turn, so every CU gets the same
    // number of items, give or take one); a grid trimmed to equal shares per WORKGROUP left a third
    // of the CUs with one workgroup more than the rest
    long blocks = (long)num_cus() * blocks_per_cu;
    if (blocks > q.items)
        blocks = q.items;
    void* args[] = {&q};
    hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(CH_THREADS), args, lds, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "conv_hybrid_mfma: %s", hipGetErrorString(e));
    return check_launch("conv_hybrid_mfma");
}

}  // namespace mg
