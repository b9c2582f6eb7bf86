// f32 MatMul with at most 4 rows (C[M,N] = A[M,K] * B, M <= 4): the reference's gevm / gemv case
// (GeneralIntrinsic/MatMulKernel/Fp32Gevm.cpp:50-119 for M <= 4, BareMetal/MatrixMul.cpp:43-120).
// The layer is ONE pass over B, a few MB: what counts is that every byte of B is requested at
// once - the whole matrix is smaller than the bandwidth-latency product of the chip - and that it
// is one launch. No matrix cores (2 flops per 4 bytes of B).
//   * B row-major [K,N] (not transposed): a workgroup owns 16 columns, a thread 4 of them (one
//     16-byte load per row) and the rows k = kg, kg + 64, ...; the 64 partial sums of a column meet
//     in LDS and are added in a fixed order.
//   * B transposed [N,K]: a wave owns 4 rows of B (= 4 outputs), a lane 16-byte pieces of them
//     along K; the lanes' partial sums meet by wavefront shuffles in a fixed order.
// The order of the additions differs from the reference's ascending k; f32 results are held to the
// 1e-4 tolerance like the tiled GEMM, not to bit equality.
#include "common.h"
#include "gevm_f32.h"

namespace mg {
namespace {

constexpr int GV_UNROLL = 8;  // rows (or 16-byte pieces) requested before the first one is used

// B[k, n] at B + k * b_rs + n (rows contiguous). VEC: 16-byte loads are possible (base, row stride
// and N allow it); otherwise the 4 columns are read one by one and checked against N.
template <int M, bool VEC>
__global__ void __launch_bounds__(256) gevm_f32_cols_kernel(GevmArgs q) {
    __shared__ float red[64][M][17];
    const int tid = threadIdx.x, cg = tid & 3, kg = tid >> 2;
    const int n0 = blockIdx.x * 16 + cg * 4;
    float acc[M][4];
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[m][j] = 0.f;
    if (n0 < q.N) {
        for (int k0 = kg; k0 < q.K; k0 += 64 * GV_UNROLL) {
            // No load stands under a condition (the compiler would wait for every outstanding
            // load at each join, one round trip per row): rows beyond K read row K - 1, columns
            // beyond N column N - 1, and their products are replaced by 0.
            float b[GV_UNROLL][4], a[GV_UNROLL][M];
#pragma unroll
            for (int u = 0; u < GV_UNROLL; ++u) {
                const int k = min(k0 + u * 64, q.K - 1);
                const float* p = q.B + (size_t)k * q.b_rs + n0;
                if (VEC) {
                    const float4 v = *(const float4*)p;
                    b[u][0] = v.x; b[u][1] = v.y; b[u][2] = v.z; b[u][3] = v.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        b[u][j] = p[min(j, q.N - 1 - n0)];
                }
#pragma unroll
                for (int m = 0; m < M; ++m)
                    a[u][m] = q.A[(size_t)m * q.a_rs + (size_t)k * q.a_cs];
            }
#pragma unroll
            for (int u = 0; u < GV_UNROLL; ++u) {
                const bool ok = k0 + u * 64 < q.K;
#pragma unroll
                for (int m = 0; m < M; ++m)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[m][j] += ok ? a[u][m] * b[u][j] : 0.f;
            }
        }
    }
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            red[kg][m][cg * 4 + j] = acc[m][j];
    __syncthreads();
    // thread (m, column) adds the 64 partial sums in ascending kg
    if (tid < M * 16) {
        const int m = tid >> 4, c = tid & 15, n = blockIdx.x * 16 + c;
        if (n < q.N) {
            float s = 0.f;
#pragma unroll 8
            for (int g = 0; g < 64; ++g)
                s += red[g][m][c];
            q.C[(size_t)m * q.ldc + n] = s;
        }
    }
}

// B[k, n] at B + n * b_cs + k (B stored transposed, rows of K contiguous)
template <int M, bool VEC>
__global__ void __launch_bounds__(256) gevm_f32_rows_kernel(GevmArgs q) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * 4 + wave) * 4;  // this wave's 4 outputs
    if (n0 >= q.N)
        return;
    float acc[M][4];
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            acc[m][r] = 0.f;
    for (int k0 = lane * 4; k0 < q.K; k0 += 256 * 2) {
        // (no load under a condition, as above: rows beyond N read row N - 1, elements beyond K
        //  element K - 1, and their products are replaced by 0)
        float b[2][4][4], a[2][M][4];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int k = k0 + u * 256;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float* row = q.B + (size_t)min(n0 + r, q.N - 1) * q.b_cs;
                if (VEC) {  // K % 4 == 0: a piece is whole or beyond K
                    const float4 v = *(const float4*)(row + min(k, q.K - 4));
                    b[u][r][0] = v.x; b[u][r][1] = v.y; b[u][r][2] = v.z; b[u][r][3] = v.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        b[u][r][j] = row[min(k + j, q.K - 1)];
                }
            }
#pragma unroll
            for (int m = 0; m < M; ++m)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    a[u][m][j] = q.A[(size_t)m * q.a_rs + (size_t)min(k + j, q.K - 1) * q.a_cs];
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int k = k0 + u * 256;
#pragma unroll
            for (int m = 0; m < M; ++m)
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[m][r] += k + j < q.K ? a[u][m][j] * b[u][r][j] : 0.f;
        }
    }
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float s = acc[m][r];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1)
                s += __shfl_down(s, off, 64);
            if (lane == 0 && n0 + r < q.N)
                q.C[(size_t)m * q.ldc + n0 + r] = s;
        }
}

template <bool VEC>
void launch_cols(const GevmArgs& q) {
    const dim3 grid((q.N + 15) / 16);
    switch (q.M) {
        case 1: hipLaunchKernelGGL((gevm_f32_cols_kernel<1, VEC>), grid, dim3(256), 0, stream(), q); break;
        case 2: hipLaunchKernelGGL((gevm_f32_cols_kernel<2, VEC>), grid, dim3(256), 0, stream(), q); break;
        case 3: hipLaunchKernelGGL((gevm_f32_cols_kernel<3, VEC>), grid, dim3(256), 0, stream(), q); break;
        default: hipLaunchKernelGGL((gevm_f32_cols_kernel<4, VEC>), grid, dim3(256), 0, stream(), q); break;
    }
}

template <bool VEC>
void launch_rows(const GevmArgs& q) {
    const dim3 grid((q.N + 15) / 16);
    switch (q.M) {
        case 1: hipLaunchKernelGGL((gevm_f32_rows_kernel<1, VEC>), grid, dim3(256), 0, stream(), q); break;
        case 2: hipLaunchKernelGGL((gevm_f32_rows_kernel<2, VEC>), grid, dim3(256), 0, stream(), q); break;
        case 3: hipLaunchKernelGGL((gevm_f32_rows_kernel<3, VEC>), grid, dim3(256), 0, stream(), q); break;
        default: hipLaunchKernelGGL((gevm_f32_rows_kernel<4, VEC>), grid, dim3(256), 0, stream(), q); break;
    }
}

}  // namespace

bool gevm_f32_supported(const GevmArgs& q) {
    return q.M >= 1 && q.M <= 4 && q.N >= 1 && q.K >= 1 && (q.b_cs == 1 || q.b_rs == 1);
}

TinyNNStatus gevm_f32_launch(const GevmArgs& q) {
    const bool aligned = ((uintptr_t)q.B & 15) == 0;
    if (q.b_cs == 1) {  // rows of B run along n
        if (aligned && (q.b_rs & 3) == 0 && (q.N & 3) == 0)
            launch_cols<true>(q);
        else
            launch_cols<false>(q);
    } else {  // rows of B run along k
        if (aligned && (q.b_cs & 3) == 0 && (q.K & 3) == 0)
            launch_rows<true>(q);
        else
            launch_rows<false>(q);
    }
    return check_launch("gevm_f32");
}

}  // namespace mg
