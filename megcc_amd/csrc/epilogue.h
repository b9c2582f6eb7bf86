// Device-side arithmetic shared by every kernel that produces qsi8: the exact float sequence of
// the reference's generated C, so that outputs are bit-identical.
//
//   conv / FullyConnected : fp32_to_int8(act((float)acc * src_scale * flt_scale / dst_scale))
//                           (BareMetal/Activation.cpp:47-56,105-114; ConvKernel.cpp:374-380)
//   fp32_to_int8          : int r = roundf(x); clamp to [-128,127]   (half away from zero)
//
// Built with -ffp-contract=off: no multiply may fuse with a following add, and the division is the
// correctly rounded IEEE one (hipcc's default for fp32 `/`); int->float conversion rounds to
// nearest even exactly like the host's cvtsi2ss.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "megcc_gfx950.h"

namespace mg {

template <int ACT>
__host__ __device__ __forceinline__ float act_apply(float x) {
    if (ACT == MEGCC_NONLINE_RELU) {
        return x > 0 ? x : 0;
    } else if (ACT == MEGCC_NONLINE_H_SWISH) {
        // res * min(max(res + 3, 0.f), 6.f) * (1.f / 6.f) with the generated min/max helpers
        float t = x + 3;
        float mx = t > 0.f ? t : 0.f;
        float mn = mx > 6.f ? 6.f : mx;
        return x * mn * (1.f / 6.f);
    } else if (ACT == MEGCC_NONLINE_SIGMOID) {
        return 1.f / (expf(-x) + 1.f);
    }
    return x;
}

__host__ __device__ __forceinline__ int fp32_to_int8(float v) {
    // (clamped as a float: the conversion of an out-of-range float is the saturating one on the
    //  device but not on the host, where the threshold tables are built)
    float r = roundf(v);
    r = r > 127.f ? 127.f : r;
    r = r < -128.f ? -128.f : r;
    return (int)r;
}

// acc already includes the int32 bias.
template <int ACT>
__host__ __device__ __forceinline__ int requant_conv(int acc, float s_src, float s_flt, float s_dst) {
    float v = (float)acc * s_src * s_flt / s_dst;
    return fp32_to_int8(act_apply<ACT>(v));
}

// ---- exact requantisation at a third of the instructions ---------------------------------------
// For IDENTITY and RELU the int8 result only depends on which integer the scaled value rounds to,
// so it can be taken from ONE multiply by c = fl(fl(s_src*s_flt)/s_dst) whenever that product is
// safely away from a rounding boundary:
//     v = fl(fl(fl(a*s_src)*s_flt)/s_dst)  (the reference, three roundings)
//     g = fl(a*c)                          (three roundings too, c is computed on the host)
// both are within 3*2^-24 relative of the real quotient, so |v - g| <= 6*2^-24*|v| < 2^-14 for
// |v| < 129. If the distance of g to the nearest integer r is below 0.5 - 2^-13, v rounds (half
// away from zero, like roundf) to the same r; beyond +-129 both clamp. Only lanes closer than
// 2^-13 to a tie (about one in 4000; exact ties included) take the reference's own sequence.
// RELU commutes with the rounding: roundf(max(v,0)) == max(roundf(v),0).
struct RequantFast {
    float c;       // fl(fl(s_src*s_flt)/s_dst); 0 disables the fast path (extreme scales)
    float s_src, s_flt, s_dst;
    float aff_c, aff_d;  // requant_conv_affine's pair when the launch picked one (below); aff_d == 0: none
};

// host side: c, or 0 when a scale is so extreme that the error bound above does not hold
static inline RequantFast make_requant_fast(float s_src, float s_flt, float s_dst) {
    RequantFast q;
    q.s_src = s_src;
    q.s_flt = s_flt;
    q.s_dst = s_dst;
    const float p = s_src * s_flt;
    const float c = p / s_dst;
    auto mid = [](float x) { return x > 1e-30f && x < 1e30f; };
    const bool sane = mid(s_src) && mid(s_flt) && mid(p) && mid(s_dst) && mid(c);
    q.c = sane ? c : 0.f;
    q.aff_c = q.aff_d = 0.f;
    return q;
}

template <int ACT>
__device__ __forceinline__ int requant_conv_fast(int acc, const RequantFast& q) {
    static_assert(ACT == MEGCC_NONLINE_IDENTITY || ACT == MEGCC_NONLINE_RELU, "monotone only");
    const float a = (float)acc;
    const float g = a * q.c;
    const float r = __builtin_rintf(g);  // nearest, ties to even: ties never use this result
    const float d = __builtin_fabsf(g - r);
    int out;
    if (__builtin_expect((!(d <= 0.5f - 0x1p-13f) && __builtin_fabsf(g) < 129.f) || q.c == 0.f, 0)) {
        out = requant_conv<ACT>(acc, q.s_src, q.s_flt, q.s_dst);
    } else {
        int i = (int)r;  // saturating conversion
        const int lo = ACT == MEGCC_NONLINE_RELU ? 0 : -128;
        out = i < lo ? lo : (i > 127 ? 127 : i);
    }
    return out;
}

// run-time activation selector (a uniform branch) for kernels that are not templated on it
__device__ __forceinline__ int requant_conv_rt(int act, int acc, float s0, float s1, float s2) {
    switch (act) {
        case MEGCC_NONLINE_RELU:
            return requant_conv<MEGCC_NONLINE_RELU>(acc, s0, s1, s2);
        case MEGCC_NONLINE_H_SWISH:
            return requant_conv<MEGCC_NONLINE_H_SWISH>(acc, s0, s1, s2);
        case MEGCC_NONLINE_SIGMOID:
            return requant_conv<MEGCC_NONLINE_SIGMOID>(acc, s0, s1, s2);
        default:
            return requant_conv<MEGCC_NONLINE_IDENTITY>(acc, s0, s1, s2);
    }
}

// ---- exact requantisation by threshold table ---------------------------------------------------
// For a monotone activation (IDENTITY, RELU) the reference's F(acc) = fp32_to_int8(act(acc * s_src
// * s_flt / s_dst)) is a non-decreasing step function of the integer accumulator, so it is fully
// described by 255 thresholds T[j] = max{a : F(a) < j}, j = -127..127:  F(a) = lo + #{j : a > T[j]}.
// The table is built with the reference's literal float sequence (binary search over int32) - on
// the host, once per (activation, scales) and cached, since x86-64 SSE arithmetic and the device's
// are the same IEEE operations; it travels to the kernel as an argument and each workgroup copies
// it to LDS. A kernel then needs only ONE estimate per output:
// with g = fl((float)a * c), c = fl(fl(s_src*s_flt)/s_dst), the true value is within 2^-14 of g
// while |g| < 129, so F(a) is floor(g) or floor(g)+1 (clamped), and the table decides which:
//     m = clamp(floor(g), lo, 126);   F(a) = m + (a > T[m + 1])
// No rounding-mode reasoning, no near-tie special case, bit-exact by construction.
static constexpr int REQUANT_TABLE_ENTRIES = 256;  // entry j + 127, last one unused

// entry `idx` (0..254) of the table: a handful of evaluations of the literal sequence (32 when
// the estimate from c is useless)
template <int ACT>
__host__ __device__ __forceinline__ int requant_threshold(int idx, float s_src, float s_flt, float s_dst, float c) {
    const int j = idx - 127;
    auto below = [&](long long a) { return requant_conv<ACT>((int)a, s_src, s_flt, s_dst) < j; };
    long long lo = INT32_MIN, hi = INT32_MAX;
    if (!below(lo))
        return INT32_MIN;  // F never drops below j: entry not used (j <= lowest output)
    // the threshold is next to (j - 0.5) / c: try a bracket of +-8 around it first
    if (c > 0.f) {
        const float est = ((float)j - 0.5f) / c;
        if (est > -2.0e9f && est < 2.0e9f) {
            const long long e = (long long)est;
            if (below(e - 8) && !below(e + 8)) {
                lo = e - 8;
                hi = e + 7;
            }
        }
    }
    while (lo < hi) {  // invariant: F(lo) < j, F(hi + 1) >= j or hi == INT32_MAX
        const long long mid = lo + (hi - lo + 1) / 2;
        if (below(mid))
            lo = mid;
        else
            hi = mid - 1;
    }
    return (int)lo;
}

// (int)floorf(x) in one instruction (saturating like the plain conversion)
__device__ __forceinline__ int cvt_floor_i32(float x) {
    int r;
    asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}

struct RequantTable {
    int t[REQUANT_TABLE_ENTRIES];
};

// H_SWISH joins the monotone activations: the reference applies it to the value already divided by
// the output scale, h(v) = v * min(max(v + 3, 0), 6) * (1/6), so its dip (-0.375 at v = -1.5) never
// reaches -0.5 and F is 0 for every v < 0; for v >= 0 both factors grow with v and every float
// rounding keeps the order, so F is a non-decreasing step function from 0 to 127 and the same table
// describes it exactly. The estimate is h(g) itself: |h(g) - h(v)| <= 1.5 * 2^-14, far inside the
// quarter that the look-up tolerates (m = floor(h(g) + 0.25), F = m or m + 1).
static inline bool requant_table_act(int act) {
    return act == MEGCC_NONLINE_IDENTITY || act == MEGCC_NONLINE_RELU || act == MEGCC_NONLINE_H_SWISH;
}

// host: the table for (act in {IDENTITY, RELU, H_SWISH}, scales); the reference stays valid for the
// life of the process (requant_table.hip)
const RequantTable& requant_table_for(int act, float s_src, float s_flt, float s_dst);

// the lower candidate m (clamped to [lowest output, 126]) of the output for accumulator acc
template <int ACT>
__device__ __forceinline__ int requant_table_candidate(int acc, float c) {
    static_assert(ACT == MEGCC_NONLINE_IDENTITY || ACT == MEGCC_NONLINE_RELU || ACT == MEGCC_NONLINE_H_SWISH,
                  "monotone only");
    constexpr int LO = ACT == MEGCC_NONLINE_IDENTITY ? -128 : 0;
    float g = (float)acc * c;
    if (ACT == MEGCC_NONLINE_H_SWISH) {
        const float t = __builtin_fminf(__builtin_fmaxf(g + 3.f, 0.f), 6.f);
        g = __builtin_fmaf(g * t, 1.f / 6.f, 0.25f);
    }
    const int m = cvt_floor_i32(g);  // saturating conversion
    return m < LO ? LO : (m > 126 ? 126 : m);
}

// table: pointer to entry 0 (LDS)
template <int ACT>
__device__ __forceinline__ int requant_conv_table(int acc, float c, const int* table) {
    const int m = requant_table_candidate<ACT>(acc, c);
    return m + (acc > table[m + 128] ? 1 : 0);
}

// ---- exact requantisation by ONE fused multiply-add, where the host can prove it ----------------
// The table look-up costs 7-8 vector instructions and an LDS read per output, and layers with few
// multiply-adds per output (pointwise with 32..128 input channels, depthwise) are bound by exactly
// that. For IDENTITY and RELU the candidate
//     F'(a) = clamp(floor(fma((float)a, c', d)), lo, 127)
// is a non-decreasing step function of a like F itself, so F' == F on all of int32 iff the two
// agree on both sides of every step of F - 2 x 255 evaluations. The host looks for a pair (c', d)
// near (c, 0.5) that passes that check against the reference's literal float sequence (for each
// c' within a few ulps of c the feasible d form an interval; its middle is then verified with the
// exact fmaf) and caches the answer per (activation, scales). Scales with exact ties whose
// roundings land on either side (0.02 * 0.01 / 0.05 ...) have no such pair and keep the table;
// calibrated scales of real networks almost always have one. 4 instructions per output, no LDS.
struct RequantAffine {
    float c, d;  // d == 0: no exact pair exists (or the activation is not IDENTITY / RELU)
};
RequantAffine requant_affine_for(int act, float s_src, float s_flt, float s_dst);
// what a launch uses: the pair (and the launch is noted as "+affine") when `table` - the kernel is the
// table instantiation for IDENTITY / RELU - and the switch "noaffine" is off; else d == 0. Call it
// after note_kernel().
RequantAffine requant_affine_pick(bool table, int act, float s_src, float s_flt, float s_dst);

template <int ACT>
__host__ __device__ __forceinline__ int requant_affine_lo() {
    return ACT == MEGCC_NONLINE_RELU ? 0 : -128;
}
template <int ACT>
__device__ __forceinline__ int requant_conv_affine(int acc, float c, float d) {
    constexpr int LO = ACT == MEGCC_NONLINE_RELU ? 0 : -128;
    const int m = cvt_floor_i32(__builtin_fmaf((float)acc, c, d));  // saturating conversion
    return m < LO ? LO : (m > 127 ? 127 : m);
}

// host side: the estimate above is valid (else kernels use the literal sequence per element)
static inline bool requant_table_ok(float s_src, float s_flt, float s_dst) {
    const RequantFast q = make_requant_fast(s_src, s_flt, s_dst);
    return q.c != 0.f && q.c * 2147483648.f > 1000.f;
}

// bytes 0 of a, b, c, d -> one dword
__device__ __forceinline__ uint32_t pack4_perm(int a, int b, int c, int d) {
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
           ((uint32_t)(d & 0xff) << 24);
}

__device__ __forceinline__ int sbyte(uint32_t w, int i) {
    return (int)(int8_t)(w >> (8 * i));
}

}  // namespace mg
