// Unsigned division by a run-time constant, for index arithmetic in kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mg {

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

}  // namespace mg
