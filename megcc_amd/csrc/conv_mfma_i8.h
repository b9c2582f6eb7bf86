// Definitions shared by the qsi8 MFMA convolution kernels (conv_mfma_i8.hip: one stage at a time,
// any shape; conv_mfma_i8_dma.hip: LDS-direct loads, pipelined, large shapes).
#pragma once
#include <stddef.h>
#include <utility>

#include "common.h"
#include "conv_geom.h"
#include "epilogue.h"
#include "fastdiv.h"

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

struct MfmaParams {
    const int8_t* src;
    int src_bytes;
    const int8_t* wp;
    const int32_t* bias;
    int8_t* dst;
    int P, OH, OW, OHW, N;
    int OC, OCP, C4;
    int stages, KS, taps, FH, FW;
    int VW, VH, IH, IW, PH, PW, SH, SW, DH, DW;
    int image_stride, plane_stride, row_stride, pix_stride;  // bytes
    int Lmax;    // LDS patch slots (multiple of 64)
    int dst_fc;  // 0: NCHW44, 1: [P][OC] row-major, 2: the same with OC a multiple of 32 and a 16-byte aligned base,
                 // 3: 2 and the LDS-direct kernel's FullyConnected tile (rows leave through LDS)
    int bias_vec4;  // bias pointer is 16-byte aligned
    int range_len;  // pixels per workgroup of the pipelined kernel (multiple of 32)
    int act;
    float s_src, s_flt, s_dst;
    RequantFast rq;
    // split-K of the one-stage kernel: blockIdx.z handles stages [z*sps, (z+1)*sps) and writes raw
    // int32 sums to partial[z][P][round_up(OC,4)]; conv_mfma_reduce_kernel finishes
    int split, sps;
    int32_t* partial;
    XcdOrder xo;  // FullyConnected tiles of the LDS-direct kernel: tile order (set at launch)
    FastDiv dOW, dOH, dVW, dVH, dL, dOHW;
    // exact requantisation thresholds for IDENTITY / RELU (built on the host, epilogue.h); only
    // the kernels that look outputs up in LDS read it
    RequantTable rq_table;
};

// Entry i of the threshold table of a kernel whose ONLY argument is an MfmaParams, read straight
// from the kernel-argument segment (indexing the by-value struct with a run-time index can make
// the compiler copy all of it to scratch).
__device__ __forceinline__ int kernarg_rq_table(int i) {
    typedef const __attribute__((address_space(4))) char* kptr;
    const kptr base = (kptr)__builtin_amdgcn_kernarg_segment_ptr();
    return *(const __attribute__((address_space(4))) int*)(base + offsetof(MfmaParams, rq_table) + 4 * i);
}

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

#define MG_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define MG_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt = bits 3:0 and
// 15:14, expcnt = 6:4, lgkmcnt = 11:8)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// LDS-direct loads written as inline assembly: the compiler's wait-count pass treats the builtin
// forms as possible LDS accesses of unknown order and then drains the LDS counter (lgkmcnt(0)) at
// every operand wait of the MFMA loop. These are invisible to it; completion is tracked by hand with
// wait_vmcnt(). `lds_addr` (byte address in LDS of lane 0's data) must be wave-uniform; lane l's
// data lands at lds_addr + l * size.
typedef unsigned v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ unsigned lds_address(const void* p) {
    return (unsigned)(size_t)MG_LDS_PTR(p);
}
__device__ __forceinline__ void dma_global_b128(const void* gptr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_addr))
                 : "memory");
}
// the same with a scalar base address and a 32-bit lane offset (no 64-bit address per lane)
__device__ __forceinline__ void dma_global_saddr_b128(const void* sbase, unsigned voffset, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voffset), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane(lds_addr))
                 : "memory");
}
// raw buffer (stride 0): offsets at or beyond num_records read as zero
__device__ __forceinline__ v4u make_raw_buffer(const void* base, unsigned num_records) {
    const unsigned long long a = (unsigned long long)base;
    v4u r;
    r[0] = (unsigned)a;
    r[1] = (unsigned)(a >> 32) & 0xffffu;
    r[2] = num_records;
    r[3] = 0x00020000u;
    return r;
}
__device__ __forceinline__ void dma_buffer_b32(v4u rsrc, unsigned voffset, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tbuffer_load_dword %0, %1, 0 offen lds"
                 :
                 : "v"(voffset), "s"(rsrc), "s"(__builtin_amdgcn_readfirstlane(lds_addr))
                 : "memory");
}

// 16 bytes per lane from a raw buffer straight into LDS (64 lanes -> 1 KB at lds_addr); offsets at
// or beyond num_records read as zero
__device__ __forceinline__ void dma_buffer_b128(v4u rsrc, unsigned voffset, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, 0 offen lds"
                 :
                 : "v"(voffset), "s"(rsrc), "s"(__builtin_amdgcn_readfirstlane(lds_addr))
                 : "memory");
}

struct PipeConfig {
    int bm, bn, ks, blocks_per_cu, threads, a_bytes;
    int nbuf;            // LDS stage buffers
    int extra_lds;       // bytes of LDS beyond the stage buffers
    int fixed_lmax;      // patch slots compiled into the kernel (0: run-time Lmax)
    int pm = 0;          // plane-major activation patch (virtual rows padded to a multiple of 4)
    int rs = 0;          // a stage is ONE filter row of a 32-channel chunk (filters of more than 9 taps)
    int fcb = 0;         // FullyConnected with 16-byte activation loads (K a multiple of 128)
    const void* kernel;
};

}  // namespace mg
