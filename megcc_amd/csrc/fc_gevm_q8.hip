// qsi8 FullyConnected with at most 4 rows (batch 1 .. 4): one pass over the packed weights in ONE
// launch, no matrix cores. A lane owns one output channel, the 16 waves of a workgroup own 16
// interleaved slices of K; every lane requests its 32-byte filter rows (two 16-byte loads per
// 32-channel chunk, in logical order whatever the packed layout's half swap) before it uses the
// first one, multiplies them with the activations (copied to LDS once, read as broadcasts) by
// v_dot4, and the 16 partial sums of a channel meet in LDS. Integer sums: exact in any order. The
// epilogue is the reference's literal sequence (bias, scale, activation, roundf, saturate;
// BareMetal/ConvKernel.cpp:305-344,374-380 on the [M,K,1,1] x [N,K,1,1] layer).
#include "conv_geom.h"
#include "conv_mfma_i8.h"
#include "epilogue.h"

namespace mg {

struct FcGevmArgs {
    const int8_t* src;    // [M][K]
    const int8_t* wp;     // packed filter [chunk][OCP][32], 16-byte halves swapped when (oc >> 3) & 1
    const int32_t* bias;  // [OC] or NULL
    int8_t* dst;          // [M][OC]
    int K, OC, OCP, nchunks;
    int act;
    float s_src, s_flt, s_dst;
};

static constexpr int FG_SLICES = 16, FG_PRE = 2;

template <int M>
__global__ void __launch_bounds__(64 * FG_SLICES) fc_gevm_q8_kernel(FcGevmArgs q) {
    extern __shared__ __attribute__((aligned(16))) int fg_lds[];
    const int tid = threadIdx.x, lane = tid & 63, sl = tid >> 6;
    const int kpad = q.nchunks * 32;
    int8_t* const act = (int8_t*)fg_lds;                 // [M][kpad], zero beyond K
    int* const red = fg_lds + (M * kpad) / 4;            // [slice][M][64]
    // The first 1024 bytes of the activations, then the filter rows: all loads of the common case
    // (M * K <= 1024) are unconditional and go out together.
    const int first_m = tid / kpad, first_k = tid - first_m * kpad;
    const bool first_ok = tid < M * kpad && first_k < q.K;
    const int8_t first = q.src[first_ok ? (size_t)first_m * q.K + first_k : 0];
    // The filter rows of the slice's first FG_PRE chunks are requested before the activations are
    // staged: they do not depend on LDS, and behind the barrier they would be a second memory
    // round trip of a kernel that is little more than one. (Unconditional loads: a chunk beyond the
    // end reads the last chunk again and is not used.)
    const int oc = blockIdx.x * 64 + lane;  // < OCP: rows beyond OC are zero in the packed filter
    const int sw = ((oc >> 3) & 1) << 4;
    const int8_t* row = q.wp + (size_t)oc * KROW;
    const size_t cstep = (size_t)q.OCP * KROW;
    v4i pre[FG_PRE][2];
#pragma unroll
    for (int i = 0; i < FG_PRE; ++i) {
        const int8_t* r = row + (size_t)min(sl + i * FG_SLICES, q.nchunks - 1) * cstep;
        pre[i][0] = *(const v4i*)(r + sw);
        pre[i][1] = *(const v4i*)(r + (sw ^ 16));
    }
    __builtin_amdgcn_sched_barrier(0);
    // (every thread stores, the surplus ones into a byte of `red` that is written again later: a
    //  store under a condition would take its load with it, behind the filter rows)
    *(tid < M * kpad ? act + tid : (int8_t*)red) = first_ok ? first : (int8_t)0;
    for (int i = tid + 64 * FG_SLICES; i < M * kpad; i += 64 * FG_SLICES) {
        const int m = i / kpad, k = i - m * kpad;
        act[i] = k < q.K ? q.src[(size_t)m * q.K + k] : (int8_t)0;
    }
    __syncthreads();

    int acc[M];
#pragma unroll
    for (int m = 0; m < M; ++m)
        acc[m] = 0;
#pragma unroll
    for (int i = 0; i < FG_PRE; ++i) {
        const int c = sl + i * FG_SLICES;
        if (c < q.nchunks) {
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const v4i a0 = *(const v4i*)(act + m * kpad + c * 32);
                const v4i a1 = *(const v4i*)(act + m * kpad + c * 32 + 16);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[m] = __builtin_amdgcn_sdot4(pre[i][0][j], a0[j], acc[m], false);
                    acc[m] = __builtin_amdgcn_sdot4(pre[i][1][j], a1[j], acc[m], false);
                }
            }
        }
    }
#pragma unroll 4
    for (int c = sl + FG_PRE * FG_SLICES; c < q.nchunks; c += FG_SLICES) {
        const int8_t* r = row + (size_t)c * cstep;
        const v4i w0 = *(const v4i*)(r + sw), w1 = *(const v4i*)(r + (sw ^ 16));
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const v4i a0 = *(const v4i*)(act + m * kpad + c * 32);
            const v4i a1 = *(const v4i*)(act + m * kpad + c * 32 + 16);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[m] = __builtin_amdgcn_sdot4(w0[j], a0[j], acc[m], false);
                acc[m] = __builtin_amdgcn_sdot4(w1[j], a1[j], acc[m], false);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < M; ++m)
        red[(sl * M + m) * 64 + lane] = acc[m];
    __syncthreads();
    if (tid < M * 64) {
        const int m = tid >> 6;
        int s = 0;
#pragma unroll
        for (int g = 0; g < FG_SLICES; ++g)
            s += red[(g * M + m) * 64 + lane];
        if (oc < q.OC) {
            if (q.bias)
                s += q.bias[oc];
            q.dst[(size_t)m * q.OC + oc] = (int8_t)requant_conv_rt(q.act, s, q.s_src, q.s_flt, q.s_dst);
        }
    }
}

static size_t fc_gevm_lds(int m, int nchunks) {
    return (size_t)m * nchunks * 32 + (size_t)FG_SLICES * m * 64 * 4;
}

// FullyConnected ([M,K,1,1] x [N,K,1,1]) with M <= 4 whose activations fit LDS
bool fc_gevm_q8_supported(const ConvGeom& g) {
    const int nchunks = (g.ic + 31) / 32;
    return g.n >= 1 && g.n <= 4 && g.ic >= 1 && g.oc >= 1 && fc_gevm_lds(g.n, nchunks) <= 64 * 1024;
}

TinyNNStatus fc_gevm_q8_launch(
        const ConvGeom& g, const void* src, const void* packed, const void* bias, void* dst) {
    FcGevmArgs q;
    q.src = (const int8_t*)src;
    q.wp = (const int8_t*)packed;
    q.bias = (const int32_t*)bias;
    q.dst = (int8_t*)dst;
    q.K = g.ic;
    q.OC = g.oc;
    q.OCP = (g.oc + OC_PAD - 1) / OC_PAD * OC_PAD;
    q.nchunks = (g.ic + 31) / 32;  // (the packed filter holds at least this many, zero-padded)
    q.act = g.act;
    q.s_src = g.s_src;
    q.s_flt = g.s_flt;
    q.s_dst = g.s_dst;
    const size_t lds = fc_gevm_lds(g.n, q.nchunks);
    void (*kern)(FcGevmArgs) = g.n == 1   ? fc_gevm_q8_kernel<1>
                               : g.n == 2 ? fc_gevm_q8_kernel<2>
                               : g.n == 3 ? fc_gevm_q8_kernel<3>
                                          : fc_gevm_q8_kernel<4>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "fc_gevm_q8: LDS attribute: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, dim3((g.oc + 63) / 64), dim3(64 * FG_SLICES), lds, stream(), q);
    return check_launch("fc_gevm_q8");
}

}  // namespace mg
