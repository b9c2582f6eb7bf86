// Stand-in for <hip/hip_runtime.h> used by tests/host_audit/audit.cpp ONLY: it lets the library's
// own kernel sources (megcc_amd/csrc/*.hip, included as they are) be compiled as plain host C++
// and run one GPU thread after the other, so that every address a kernel computes is dereferenced
// on the host, on buffers fenced by inaccessible pages. Values do not matter here - threads do not
// see each other's LDS writes, matrix-core and cross-lane builtins return an operand - only the
// index arithmetic is exercised, and that arithmetic never depends on loaded values in the
// audited kernels.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>

#define MG_HOST_AUDIT 1
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__
#define __launch_bounds__(...)

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint3_ {
    unsigned x, y, z;
};
inline thread_local uint3_ threadIdx, blockIdx;
inline thread_local dim3 blockDim, gridDim;

struct float4 {
    float x, y, z, w;
} __attribute__((aligned(16)));
inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
struct float2 {
    float x, y;
} __attribute__((aligned(8)));
inline float2 make_float2(float x, float y) { return float2{x, y}; }
struct int4 {
    int x, y, z, w;
} __attribute__((aligned(16)));
struct int2 {
    int x, y;
} __attribute__((aligned(8)));
struct uint4 {
    unsigned x, y, z, w;
} __attribute__((aligned(16)));
struct uint2 {
    unsigned x, y;
} __attribute__((aligned(8)));

using std::max;
using std::min;
inline int min(int a, unsigned b) { return a < (int)b ? a : (int)b; }
inline long min(long a, int b) { return a < b ? a : (long)b; }
inline long max(long a, int b) { return a > b ? a : (long)b; }

typedef int hipError_t;
typedef void* hipStream_t;
enum { hipSuccess = 0, hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
inline const char* hipGetErrorString(hipError_t) { return "host audit"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, int, int) { return hipSuccess; }

inline void __syncthreads() {}
template <typename T>
inline T __shfl_down(T v, int, int = 64) { return v; }
template <typename T>
inline T __shfl_xor(T v, int, int = 64) { return v; }
template <typename T>
inline T __shfl(T v, int, int = 64) { return v; }
inline unsigned __umulhi(unsigned a, unsigned b) { return (unsigned)(((unsigned long long)a * b) >> 32); }

#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) (c)
#define __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, x, y, z) (c)
#define __builtin_amdgcn_sdot4(a, b, c, clamp) (c)
#define __builtin_amdgcn_perm(a, b, sel) ((a) ^ (b) ^ (sel))
#define __builtin_amdgcn_s_barrier() ((void)0)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_fence(...) ((void)0)
#define __builtin_amdgcn_kernarg_segment_ptr() ((const char*)0)

// every block, every thread, one after the other
template <typename K, typename... Args>
inline void host_audit_launch(K kernel, dim3 grid, dim3 block, Args... args) {
    gridDim = grid;
    blockDim = block;
    for (unsigned bz = 0; bz < grid.z; ++bz)
        for (unsigned by = 0; by < grid.y; ++by)
            for (unsigned bx = 0; bx < grid.x; ++bx) {
                blockIdx = uint3_{bx, by, bz};
                for (unsigned tz = 0; tz < block.z; ++tz)
                    for (unsigned ty = 0; ty < block.y; ++ty)
                        for (unsigned tx = 0; tx < block.x; ++tx) {
                            threadIdx = uint3_{tx, ty, tz};
                            kernel(args...);
                        }
            }
}
#define hipLaunchKernelGGL(kernel, grid, block, lds_bytes, strm, ...) \
    host_audit_launch(kernel, dim3(grid), dim3(block), __VA_ARGS__)
