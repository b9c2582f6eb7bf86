// f32 matrix product with at most 4 rows (gevm_f32.hip).
#pragma once
#include "common.h"

namespace mg {

struct GevmArgs {
    const float* A;  // a(m, k) = A[m * a_rs + k * a_cs]
    const float* B;  // b(k, n) = B[k * b_rs + n * b_cs], one of the two strides is 1
    float* C;        // c(m, n) = C[m * ldc + n]
    int M, N, K;
    long a_rs, a_cs, b_rs, b_cs, ldc;
};

bool gevm_f32_supported(const GevmArgs& q);
TinyNNStatus gevm_f32_launch(const GevmArgs& q);

}  // namespace mg
