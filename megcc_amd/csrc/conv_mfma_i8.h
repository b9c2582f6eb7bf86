// Definitions shared by the two qsi8 MFMA convolution kernels (conv_mfma_i8.hip: one stage at a time,
// any shape; conv_mfma_i8_wide.hip and conv_mfma_i8_ws.hip: pipelined, large shapes).
#pragma once
#include <utility>

#include "common.h"
#include "conv_geom.h"
#include "epilogue.cuh"

namespace mg {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

static constexpr int BN = 128;       // pixels per workgroup
static constexpr int THREADS = 256;  // 4 waves
static constexpr int KROW = 32;      // input channels per LDS row = K of one MFMA
static constexpr int MAX_TAPS_STAGE = 9;
static constexpr int MAX_B_ITEMS = 8;  // 16-byte gather items per thread per stage
static constexpr int OC_PAD = 256;   // packed filter rows are padded to the largest oc tile
static constexpr int CHUNK_PAD = 4;  // ... and ic chunks to the largest sub-chunk count per stage

// unsigned division by a run-time constant: q = (x * mul) >> (32 + shift), exact for x < 2^31
struct FastDiv {
    uint32_t mul, shift, d;
};
static inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    if (d == 1) {
        f.mul = 0;
        f.shift = 0;
        return f;
    }
    uint32_t s = 0;
    while ((1u << s) < d)
        ++s;  // ceil(log2 d)
    uint64_t m = ((uint64_t(1) << (32 + s - 1)) + d - 1) / d;  // fits 32 bits for x < 2^31
    f.mul = (uint32_t)m;
    f.shift = s - 1;
    return f;
}
__device__ __forceinline__ uint32_t fdiv(uint32_t x, const FastDiv& f) {
    return f.d == 1 ? x : (__umulhi(x, f.mul) >> f.shift);
}

struct MfmaParams {
    const int8_t* src;
    const int8_t* wp;
    const int32_t* bias;
    int8_t* dst;
    int P, OH, OW, OHW, N;
    int OC, OCP, C4;
    int stages, KS, taps, FH, FW;
    int VW, VH, IH, IW, PH, PW, SH, SW, DH, DW;
    int image_stride, plane_stride, row_stride, pix_stride;  // bytes
    int Lmax;    // LDS patch slots (multiple of 64)
    int dst_fc;  // 0: NCHW44, 1: [P][OC] row-major
    int bias_vec4;  // bias pointer is 16-byte aligned
    int range_len;  // pixels per workgroup of the pipelined kernel (multiple of 32)
    int act;
    float s_src, s_flt, s_dst;
    RequantFast rq;
    FastDiv dOW, dOH, dVW, dVH, dL, dOHW;
    int G, RG;       // 16-byte gather: pixel groups per row, groups per plane of the largest patch
    FastDiv dG, dRG;
};

// virtual pixel index of output pixel p at tap (0,0): rows of the zero-padded images stacked
__device__ __forceinline__ int vp_of(const MfmaParams& q, int p) {
    int g = fdiv(p, q.dOW), ow = p - g * q.OW;
    int n = fdiv(g, q.dOH), oh = g - n * q.OH;
    return (n * q.VH + oh * q.SH) * q.VW + ow * q.SW;
}


// compile-time loop: f(std::integral_constant<int, 0>) ... f(<N-1>)
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

struct PipeConfig {
    int bm, bn, ks, maxb, blocks_per_cu, threads, a_bytes, g4;
    int gather_threads;  // threads that share the activation gather (maxb items each)
    int nbuf;            // LDS stage buffers
    int extra_lds;       // bytes of LDS beyond the stage buffers
    const void* kernel;
};

}  // namespace mg
