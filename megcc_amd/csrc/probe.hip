// Measurement aid, not an operator: how fast do this chip's matrix cores run v_mfma_i32_32x32x32_i8
// back to back when NOTHING else happens - operands in registers, no loads, no LDS, no epilogue,
// every SIMD the same number of MFMAs? The answer depends on the operand VALUES: the board is
// power-limited, and uniform random int8 operands (the reference benchmark's distribution,
// compiler/test/kernel/opr/arm/benchmark_conv.cpp:198) toggle the multipliers far more than zeros or
// small values do. bench.py --workload mfma_only reports it next to the published peak.
//
// Built into a library of its own (libmegcc_bench_probe.so) that only bench.py and one test load:
// the product library neither contains nor exports it. Self-contained: its own stream-less
// launches on the null stream, no dependency on the product's sources.
#include <hip/hip_runtime.h>
#include <stdlib.h>

#include <vector>

namespace {

typedef int probe_v4i __attribute__((ext_vector_type(4)));
typedef int probe_v16i __attribute__((ext_vector_type(16)));

// 8 waves per workgroup = 2 per SIMD, 8 independent accumulators per wave; a / b: 4 + 4 operand
// registers per lane, taken from `ops` once
__global__ void __launch_bounds__(512) probe_mfma_kernel(
        const probe_v4i* __restrict__ ops, int* __restrict__ out, int iters, int nvar) {
    const int tid = blockIdx.x * 512 + threadIdx.x;
    probe_v4i a[4], b[4];
    for (int i = 0; i < 4; ++i) {
        a[i] = ops[(tid * 8 + i) % nvar];
        b[i] = ops[(tid * 8 + 4 + i) % nvar];
    }
    probe_v16i acc[8] = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < 8; ++k)
            acc[k] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[k & 3], b[(k + it) & 3], acc[k], 0, 0, 0);
    }
    int s = 0;
    for (int k = 0; k < 8; ++k)
        for (int e = 0; e < 16; ++e)
            s += acc[k][e];
    if (s == 0x12345678)  // (keeps the accumulators alive; practically never true)
        out[tid] = s;
}

}  // namespace

// operand_kind 0: zeros; 1: uniform random int8 in [-127, 127]; 2: activations max(0, x) with x normal
// (sigma 20) against weights normal (sigma 30), both clipped to int8. Runs `launches` launches of one
// workgroup per CU with `mfma_per_simd` MFMAs per SIMD each (after as many untimed ones) and
// returns the average time of a launch in microseconds and the MFMAs a launch issued.
// Status: 0 = measured, 1 = bad argument, 2 = device memory, 3 = a HIP call failed.
extern "C" int megcc_bench_probe_mfma_i8(
        int operand_kind, int mfma_per_simd, int launches, double* us_per_launch, double* mfma_per_launch) {
    if (!(us_per_launch && mfma_per_launch && launches > 0 && mfma_per_simd >= 16 && operand_kind >= 0 &&
          operand_kind <= 2))
        return 1;
    const int nvar = 1 << 16;
    std::vector<int> h((size_t)nvar * 4);
    unsigned long long state = 88172645463325252ull;
    auto next = [&]() {  // xorshift64
        state ^= state << 13;
        state ^= state >> 7;
        state ^= state << 17;
        return state;
    };
    auto normal = [&](double sigma) {  // sum of 12 uniforms
        double s = 0;
        for (int i = 0; i < 12; ++i)
            s += (double)(next() >> 11) / 9007199254740992.0;
        return (s - 6.0) * sigma;
    };
    for (size_t i = 0; i < h.size(); ++i) {
        unsigned w = 0;
        for (int k = 0; k < 4; ++k) {
            int v = 0;
            if (operand_kind == 1) {
                v = (int)(next() % 255) - 127;
            } else if (operand_kind == 2) {
                // (operands a and b of a lane come from alternating groups of 4 entries of 16 bytes)
                const bool is_weight = ((i / 4) / 4) & 1;
                double x = is_weight ? normal(30) : normal(20);
                if (!is_weight && x < 0)
                    x = 0;
                v = (int)(x < -127 ? -127 : x > 127 ? 127 : x);
            }
            w |= (unsigned)(v & 0xff) << (8 * k);
        }
        h[i] = (int)w;
    }
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return 3;
    const int iters = (mfma_per_simd / 2 + 7) / 8;  // 2 waves per SIMD, 8 MFMAs per iteration
    void* d = nullptr;
    void* out = nullptr;
    if (hipMalloc(&d, (size_t)nvar * 16) != hipSuccess)
        return 2;
    if (hipMalloc(&out, (size_t)cus * 512 * 4) != hipSuccess) {
        (void)hipFree(d);
        return 2;
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int st = 0;
    float ms = 0;
    hipStream_t strm = nullptr;  // the null stream
    if (hipMemcpy(d, h.data(), (size_t)nvar * 16, hipMemcpyHostToDevice) != hipSuccess ||
        hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        st = 3;
    } else {
        for (int w = 0; w < launches; ++w)
            hipLaunchKernelGGL(probe_mfma_kernel, dim3(cus), dim3(512), 0, strm, (const probe_v4i*)d, (int*)out,
                               iters, nvar);
        (void)hipEventRecord(e0, strm);
        for (int w = 0; w < launches; ++w)
            hipLaunchKernelGGL(probe_mfma_kernel, dim3(cus), dim3(512), 0, strm, (const probe_v4i*)d, (int*)out,
                               iters, nvar);
        (void)hipEventRecord(e1, strm);
        if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
            st = 3;
    }
    if (e0)
        (void)hipEventDestroy(e0);
    if (e1)
        (void)hipEventDestroy(e1);
    (void)hipFree(d);
    (void)hipFree(out);
    if (st)
        return st;
    *us_per_launch = (double)ms / launches * 1e3;
    *mfma_per_launch = (double)cus * 8 * 8 * iters;
    return 0;
}
