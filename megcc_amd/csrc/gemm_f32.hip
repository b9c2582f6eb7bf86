// f32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32), shared by
//   * MatrixMul C = op(A) op(B)   (GeneralIntrinsic/MatMulKernel/Fp32MatMulM4N12.cpp:9-158,
//                                  Fp32Gevm.cpp:50-119, BareMetal/MatrixMul.cpp:25-120), and
//   * f32 NCHW dense convolution as an implicit GEMM: rows = oc, columns = output pixels,
//     K = (ic, fh, fw) (GeneralIntrinsic/ConvKernel/Fp32Im2col.cpp:88-218 does the same product
//     through an explicit im2col + pack into workspace; here the gather happens while the B tile
//     is staged into LDS, so there is no workspace), bias + activation fused into the store.
// Workgroup: 256 threads, four waves of 64 x 64 outputs each: tile 128 x 128 x 16 (2 x 2 waves) or,
// for problems with at most 64 rows (GEVM, batch-64 FullyConnected, convolutions with few output
// channels), 64 x 256 x 16 (1 x 4 waves) so that no wave multiplies rows that do not exist. LDS
// tiles are K-major with the row padded by 4 floats so both the staging writes and the MFMA
// operand reads are bank-conflict free.
// fp32 sums are formed in a different order from the reference's 4x12 micro-kernel; results are
// held to 1e-4 relative, not bit-exactness. A float32 running sum over thousands of products
// drifts from the exact value by more than that (K = 4096, values in [-1, 1]: 1.1e-4 on the worst
// of 16 M outputs), so a workgroup whose K range is longer than 1024 (LONGK) closes its running
// sums every 512 steps of K into a second set of registers: 3e-5 at K = 4096.
#include "common.h"
#include "gevm_f32.h"
#include "conv_geom.h"
#include "epilogue.h"

namespace mg {

typedef float v16f __attribute__((ext_vector_type(16)));

static constexpr int GBM = 128, GBN = 128, GBK = 16, GPAD = 4;

struct GemmArgs {
    const float* A;
    const float* B;
    float* C;
    const float* bias;
    int M, N, K;
    long a_rs, a_cs;  // element strides of A(m,k)
    long b_rs, b_cs;  // element strides of B(k,n)  (matmul only)
    long ldc;
    int act;
    ConvGeom g;  // convolution only
    int is_conv;
    // split-K: blockIdx.z handles k in [z*kchunk, (z+1)*kchunk) and writes its partial sums to
    // partial[z][M][N]; gemm_f32_reduce_kernel adds them in z order (deterministic) and stores
    int split, kchunk;
    float* partial;
    XcdOrder xo;  // tile order (set at launch from the grid)
};

__device__ __forceinline__ float act_rt(int act, float x) {
    switch (act) {
        case MEGCC_NONLINE_RELU: return act_apply<MEGCC_NONLINE_RELU>(x);
        case MEGCC_NONLINE_H_SWISH: return act_apply<MEGCC_NONLINE_H_SWISH>(x);
        case MEGCC_NONLINE_SIGMOID: return act_apply<MEGCC_NONLINE_SIGMOID>(x);
        default: return x;
    }
}

// B(k, p) of the implicit GEMM: source pixel of output pixel p under filter tap k
// (ok: the tap lies on the image; otherwise element 0 is read and the caller discards it)
__device__ __forceinline__ float conv_b(const GemmArgs& q, int k, int p, bool& ok) {
    const ConvGeom& g = q.g;
    int taps = g.fh * g.fw;
    int ic = k / taps, t = k - ic * taps;
    int fh = t / g.fw, fw = t - fh * g.fw;
    int ohw = g.oh * g.ow;
    int n = p / ohw, r = p - n * ohw;
    int oh = r / g.ow, ow = r - oh * g.ow;
    unsigned ih = (unsigned)(oh * g.sh + fh * g.dh - g.ph);
    unsigned iw = (unsigned)(ow * g.sw + fw * g.dw - g.pw);
    ok = ih < (unsigned)g.ih && iw < (unsigned)g.iw;
    return q.B[ok ? (((size_t)n * g.ic + ic) * g.ih + ih) * g.iw + iw : 0];
}

// A_KFAST: A(m,k) has k contiguous (row-major, not transposed) -> lanes walk k when staging.
// B_NFAST: B(k,n) has n contiguous -> lanes walk n.
template <bool A_KFAST, bool B_NFAST, bool CONV, int BM, bool LONGK = false>
__global__ void __launch_bounds__(256) gemm_f32_kernel(GemmArgs q) {
    constexpr int KSEG = 512;  // LONGK: steps of K per running sum
    constexpr int BN = GBM * GBN / BM;  // 128 x 128 or 64 x 256
    constexpr int A_IT = BM / 16, B_IT = BN / 16;
    // LDS is double buffered: the global loads of step k+1 are in flight (in registers) while
    // step k is multiplied out of the other buffer; one barrier per step.
    __shared__ __attribute__((aligned(16))) float As[2][GBK][BM + GPAD];
    __shared__ __attribute__((aligned(16))) float Bs[2][GBK][BN + GPAD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = BM == 128 ? wave >> 1 : 0, wn = BM == 128 ? wave & 1 : wave;
    // (each XCD owns a compact rectangle of tiles: with the plain order every XCD fetched every
    //  row panel of A - 3.7 times the matrices' bytes from memory for 4096 x 4096 x 4096)
    int tile_x, tile_y;
    xcd_tile(q.xo, blockIdx.x, blockIdx.y, gridDim.x, gridDim.y, tile_x, tile_y);
    const int m0 = tile_y * BM, n0 = tile_x * BN;

    v16f acc[2][2], tot[LONGK ? 2 : 1][LONGK ? 2 : 1];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0.f;
                if (LONGK)
                    tot[i][j][e] = 0.f;
            }

    const int k_begin = blockIdx.z * q.kchunk;
    const int k_end = min(q.K, k_begin + q.kchunk);
    float ra[A_IT], rb[B_IT];
    // MatrixMul tiles that lie inside the matrices are staged with 16-byte loads along each
    // operand's contiguous axis and no range checks: the checked element-wise loads below are some
    // 350 instructions per stage, issued while the matrix cores have nothing queued.
    constexpr bool VEC = !CONV;
    bool vec_tile = false;
    if (VEC)  // the strides of the non-contiguous axes: rows of 4n floats from a 16-byte base
        vec_tile = m0 + BM <= q.M && n0 + BN <= q.N &&
                   (((A_KFAST ? q.a_rs : q.a_cs) | (B_NFAST ? q.b_rs : q.b_cs)) & 3) == 0 &&
                   (((uintptr_t)q.A | (uintptr_t)q.B) & 15) == 0;
    // thread -> (row along the strided axis, first of 4 elements along the contiguous axis) of a
    // tile of `fast` contiguous elements per row
    auto vec_pos = [&](int fast, int it, int& slow_i, int& fast_i) {
        slow_i = tid / (fast / 4) + it * (1024 / fast);
        fast_i = (tid % (fast / 4)) * 4;
    };
    auto load_tiles_vec = [&](int k0) {
#pragma unroll
        for (int it = 0; it < A_IT / 4; ++it) {
            int m, k;
            if (A_KFAST)
                vec_pos(GBK, it, m, k);
            else
                vec_pos(BM, it, k, m);
            const float4 v =
                    *(const float4*)(q.A + (size_t)(m0 + m) * q.a_rs + (size_t)(k0 + k) * q.a_cs);
            ra[4 * it] = v.x, ra[4 * it + 1] = v.y, ra[4 * it + 2] = v.z, ra[4 * it + 3] = v.w;
        }
#pragma unroll
        for (int it = 0; it < B_IT / 4; ++it) {
            int k, n;
            if (B_NFAST)
                vec_pos(BN, it, k, n);
            else
                vec_pos(GBK, it, n, k);
            const float4 v =
                    *(const float4*)(q.B + (size_t)(k0 + k) * q.b_rs + (size_t)(n0 + n) * q.b_cs);
            rb[4 * it] = v.x, rb[4 * it + 1] = v.y, rb[4 * it + 2] = v.z, rb[4 * it + 3] = v.w;
        }
    };
    auto store_tiles_vec = [&](int buf) {
#pragma unroll
        for (int it = 0; it < A_IT / 4; ++it) {
            int m, k;
            if (A_KFAST) {
                vec_pos(GBK, it, m, k);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    As[buf][k + j][m] = ra[4 * it + j];
            } else {
                vec_pos(BM, it, k, m);
                *(float4*)&As[buf][k][m] =
                        make_float4(ra[4 * it], ra[4 * it + 1], ra[4 * it + 2], ra[4 * it + 3]);
            }
        }
#pragma unroll
        for (int it = 0; it < B_IT / 4; ++it) {
            int k, n;
            if (B_NFAST) {
                vec_pos(BN, it, k, n);
                *(float4*)&Bs[buf][k][n] =
                        make_float4(rb[4 * it], rb[4 * it + 1], rb[4 * it + 2], rb[4 * it + 3]);
            } else {
                vec_pos(GBK, it, n, k);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    Bs[buf][k + j][n] = rb[4 * it + j];
            }
        }
    };
    // implicit GEMM: with B_NFAST a thread stages the same output pixel in every K step, so its
    // image / row / column are worked out once
    // (a column beyond N takes the last column's pixel: its loads are issued like all others,
    //  unconditionally, and must stay inside the tensor; its values are never stored)
    const int cn = min(n0 + tid % BN, q.N - 1);
    long c_img = 0;
    int c_ih0 = 0, c_iw0 = 0;
    float c_inv_taps = 0.f, c_inv_fw = 0.f;
    if (CONV) {
        const ConvGeom& g = q.g;
        const int ohw = g.oh * g.ow;
        const int n = cn / ohw, r = cn - n * ohw;
        const int oh = r / g.ow, ow = r - oh * g.ow;
        c_img = (long)n * g.ic * g.ih * g.iw;
        c_ih0 = oh * g.sh - g.ph;
        c_iw0 = ow * g.sw - g.pw;
        c_inv_taps = 1.f / (float)(g.fh * g.fw);
        c_inv_fw = 1.f / (float)g.fw;
    }
    // B(k, cn): the quotients are exact for k below 2^22 (k + 0.5 keeps them off the boundaries)
    auto conv_b_col = [&](int k, bool& ok) __attribute__((always_inline)) -> float {
        const ConvGeom& g = q.g;
        const int taps = g.fh * g.fw;
        const int ic = (int)(((float)k + 0.5f) * c_inv_taps), t = k - ic * taps;
        const int fh = (int)(((float)t + 0.5f) * c_inv_fw), fw = t - fh * g.fw;
        const unsigned ih = (unsigned)(c_ih0 + fh * g.dh), iw = (unsigned)(c_iw0 + fw * g.dw);
        ok = ih < (unsigned)g.ih && iw < (unsigned)g.iw;
        return q.B[ok ? c_img + ((size_t)ic * g.ih + ih) * g.iw + iw : 0];
    };
    // Loads that are out of range read element 0 instead, and the value is replaced by 0 when it is
    // written to LDS (the range test is repeated there; a convolution keeps one bit per element of
    // the stage in flight, tap_ok, for what the gather found). A load under a branch makes the
    // compiler wait for every outstanding load at the join, and a select right after the load
    // waits for that load: either turns the loads of a stage into as many round trips.
    unsigned tap_bits = 0;
    // stage A tile (BM x GBK) and B tile (GBK x BN): BM / 16 and BN / 16 elements per thread
    auto load_tiles = [&](int k0) {
        if (VEC && vec_tile && k0 + GBK <= k_end) {
            load_tiles_vec(k0);
            return;
        }
#pragma unroll
        for (int it = 0; it < A_IT; ++it) {
            int m, k;
            if (A_KFAST) {
                k = tid & 15;
                m = (tid >> 4) + it * 16;
            } else {
                m = tid % BM;
                k = tid / BM + it * (256 / BM);
            }
            const bool ok = m0 + m < q.M && k0 + k < k_end;
            ra[it] = q.A[ok ? (size_t)(m0 + m) * q.a_rs + (size_t)(k0 + k) * q.a_cs : 0];
        }
#pragma unroll
        for (int it = 0; it < B_IT; ++it) {
            int n, k;
            if (B_NFAST) {
                n = tid % BN;
                k = tid / BN + it * (256 / BN);
            } else {
                k = tid & 15;
                n = (tid >> 4) + it * 16;
            }
            const bool ok = n0 + n < q.N && k0 + k < k_end;
            bool tap_ok = true;
            if (CONV && B_NFAST)
                rb[it] = conv_b_col(min(k0 + k, k_end - 1), tap_ok);
            else if (CONV)
                rb[it] = conv_b(q, min(k0 + k, k_end - 1), min(n0 + n, q.N - 1), tap_ok);
            else
                rb[it] = q.B[ok ? (size_t)(k0 + k) * q.b_rs + (size_t)(n0 + n) * q.b_cs : 0];
            if (CONV)
                tap_bits = (tap_bits & ~(1u << it)) | ((unsigned)tap_ok << it);
        }
    };
    auto store_tiles = [&](int buf, int k0) {
        if (VEC && vec_tile && k0 + GBK <= k_end) {
            store_tiles_vec(buf);
            return;
        }
#pragma unroll
        for (int it = 0; it < A_IT; ++it) {
            const int k = A_KFAST ? tid & 15 : tid / BM + it * (256 / BM);
            const int m = A_KFAST ? (tid >> 4) + it * 16 : tid % BM;
            As[buf][k][m] = m0 + m < q.M && k0 + k < k_end ? ra[it] : 0.f;
        }
#pragma unroll
        for (int it = 0; it < B_IT; ++it) {
            const int k = B_NFAST ? tid / BN + it * (256 / BN) : tid & 15;
            const int n = B_NFAST ? tid % BN : (tid >> 4) + it * 16;
            const bool ok = n0 + n < q.N && k0 + k < k_end && (!CONV || ((tap_bits >> it) & 1));
            Bs[buf][k][n] = ok ? rb[it] : 0.f;
        }
    };
    if (k_begin < k_end) {
        load_tiles(k_begin);
        store_tiles(0, k_begin);
    }
    __syncthreads();
    int buf = 0;
    for (int k0 = k_begin; k0 < k_end; k0 += GBK, buf ^= 1) {
        const bool more = k0 + GBK < k_end;
        if (more)
            load_tiles(k0 + GBK);
#pragma unroll
        for (int kk = 0; kk < GBK; kk += 2) {
            const int k = kk + (lane >> 5);
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                a[i] = As[buf][k][wm * 64 + i * 32 + (lane & 31)];
#pragma unroll
            for (int j = 0; j < 2; ++j)
                b[j] = Bs[buf][k][wn * 64 + j * 32 + (lane & 31)];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (LONGK && ((k0 - k_begin) / GBK) % (KSEG / GBK) == KSEG / GBK - 1) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        tot[i][j][e] += acc[i][j][e];
                        acc[i][j][e] = 0.f;
                    }
        }
        if (more)
            store_tiles(buf ^ 1, k0 + GBK);
        __syncthreads();
    }
    if (LONGK) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[i][j][e] += tot[i][j][e];
    }

    // register e of a tile: row 8*(e/4) + 4*(lane/32) + e%4, column lane%32
    // The bias of the thread's 32 rows, requested at once and without a branch around the load (a
    // load under `if (bias)` per element makes 64 dependent round trips of the epilogue: 35 us for a
    // 1x1 layer whose multiplication takes 10).
    float bv[2][16];
    if (CONV && q.split == 1) {
        const float* bp = q.bias ? q.bias : q.A;  // (any readable floats: discarded below)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                bv[i][e] = bp[min(m, q.M - 1)];
            }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                bv[i][e] = q.bias ? bv[i][e] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = n0 + wn * 64 + j * 32 + (lane & 31);
        if (n >= q.N)
            continue;
        size_t col_off;
        int img = 0, rem = 0;
        if (CONV) {
            int ohw = q.g.oh * q.g.ow;
            img = n / ohw;
            rem = n - img * ohw;
            col_off = 0;
        } else {
            col_off = n;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (m >= q.M)
                    continue;
                float v = acc[i][j][e];
                if (q.split > 1) {
                    q.partial[((size_t)blockIdx.z * q.M + m) * q.N + n] = v;
                } else if (CONV) {
                    v = act_rt(q.act, v + bv[i][e]);
                    q.C[((size_t)img * q.M + m) * (q.g.oh * q.g.ow) + rem] = v;
                } else {
                    q.C[(size_t)m * q.ldc + col_off] = v;
                }
            }
    }
}

// sums the split-K partials in a fixed order (z ascending) and stores like the unsplit kernel
// would. V = 4: four neighbouring columns per thread, 16-byte loads and stores (the host checks
// that rows, images and pointers allow it).
template <int V>
__global__ void __launch_bounds__(256) gemm_f32_reduce_kernel(GemmArgs q) {
    const size_t total = (size_t)q.M * q.N / V;
    const int ohw = q.g.oh * q.g.ow;
    for (size_t i = blockIdx.x * (size_t)256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const size_t e = i * V;
        const int m = (int)(e / q.N), n = (int)(e - (size_t)m * q.N);
        float v[V];
#pragma unroll
        for (int c = 0; c < V; ++c)
            v[c] = 0.f;
#pragma unroll 4
        for (int z = 0; z < q.split; ++z) {  // (the loads of 4 slices go out together)
            const float* p = q.partial + (size_t)z * q.M * q.N + e;
            if (V == 4) {
                const float4 t = *(const float4*)p;
                v[0] += t.x, v[1 % V] += t.y, v[2 % V] += t.z, v[3 % V] += t.w;
            } else {
                v[0] += *p;
            }
        }
        float* out;
        if (q.is_conv) {
            const float b = q.bias ? q.bias[m] : 0.f;
#pragma unroll
            for (int c = 0; c < V; ++c)
                v[c] = act_rt(q.act, v[c] + b);
            const int img = n / ohw, rem = n - img * ohw;
            out = q.C + ((size_t)img * q.M + m) * ohw + rem;
        } else {
            out = q.C + (size_t)m * q.ldc + n;
        }
        if (V == 4)
            *(float4*)out = make_float4(v[0], v[1 % V], v[2 % V], v[3 % V]);
        else
            *out = v[0];
    }
}

// Split factor for problems with too few 128 x 128 tiles to fill the chip (skinny M: GEVM,
// batch-64 FullyConnected, the small f32 convolution). A pure function of the shape, so that the
// _workspace entry point and the kernel agree.
static int gemm_split(long M, long N, long K, bool conv) {
    // (at most 64 rows: 64 x 256 tiles)
    const long tiles = M <= 64 ? (N + 255) / 256 : ((M + GBM - 1) / GBM) * ((N + GBN - 1) / GBN);
    if (tiles >= 192 || K < 128)
        return 1;
    // Every split writes M x N partial sums. A MatrixMul of few rows is best at one workgroup per
    // CU (64 x 4096 x 4096: 37 us with 16 slices, 40 us with 32); the implicit GEMM spends more of a
    // stage on its gather and gains from a second workgroup per CU that multiplies meanwhile
    // (N=8, 64 -> 64, 56 x 56, 3x3: 74 us with 3 slices, 64 us with 6; 118 us unsplit).
    long s = ((M <= 64 && !conv ? 256 : 512) + tiles - 1) / tiles;
    const long max_s = K / 64;
    if (s > max_s)
        s = max_s;
    if (s > 64)
        s = 64;
    return s < 2 ? 1 : (int)s;
}

size_t gemm_f32_workspace_bytes(long M, long N, long K, bool conv) {
    const int s = gemm_split(M, N, K, conv);
    return s > 1 ? (size_t)s * M * N * sizeof(float) : 0;
}

// chooses the split for (q.M, q.N, q.K) if the workspace can hold the partials
static void gemm_plan_split(GemmArgs& q, const Workspace* ws) {
    q.split = 1;
    q.kchunk = (q.K + GBK - 1) / GBK * GBK;
    q.partial = nullptr;
    const int s = gemm_split(q.M, q.N, q.K, q.is_conv != 0);
    if (s > 1 && ws && ws->ptr && ws->size >= gemm_f32_workspace_bytes(q.M, q.N, q.K, q.is_conv != 0) &&
        ((uintptr_t)ws->ptr & 3) == 0) {
        q.split = s;
        q.kchunk = ((q.K + s - 1) / s + GBK - 1) / GBK * GBK;
        q.partial = (float*)ws->ptr;
    }
}

static void gemm_launch_reduce(const GemmArgs& q) {
    // four columns per thread: they must share a row (and an image), and every address a multiple
    // of 16 bytes
    const bool v4 = (q.N & 3) == 0 && (((uintptr_t)q.partial | (uintptr_t)q.C) & 15) == 0 &&
                    (q.is_conv ? (q.g.oh * q.g.ow & 3) == 0 : (q.ldc & 3) == 0);
    const size_t total = (size_t)q.M * q.N / (v4 ? 4 : 1);
    unsigned blocks = (unsigned)((total + 255) / 256);
    if (blocks > 8192)
        blocks = 8192;
    if (v4)
        hipLaunchKernelGGL(gemm_f32_reduce_kernel<4>, dim3(blocks), dim3(256), 0, stream(), q);
    else
        hipLaunchKernelGGL(gemm_f32_reduce_kernel<1>, dim3(blocks), dim3(256), 0, stream(), q);
}

bool conv_f32_gemm_supported(const ConvGeom& g) {
    long P = (long)g.n * g.oh * g.ow;
    return g.fmt == MEGCC_FMT_NCHW && g.groups == 1 && P < (1L << 31) &&
           (long)g.ic * g.fh * g.fw < (1L << 31);
}

size_t conv_f32_gemm_workspace_bytes(const ConvGeom& g) {
    return gemm_f32_workspace_bytes(g.oc, (long)g.n * g.oh * g.ow, (long)g.ic * g.fh * g.fw, true);
}

TinyNNStatus conv_f32_gemm_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, void* dst,
        const Workspace* ws) {
    GemmArgs q;
    q.A = (const float*)flt;  // [OC][IC*FH*FW]
    q.B = (const float*)src;
    q.C = (float*)dst;
    q.bias = (const float*)bias;
    q.M = g.oc;
    q.N = g.n * g.oh * g.ow;
    q.K = g.ic * g.fh * g.fw;
    q.a_rs = q.K;
    q.a_cs = 1;
    q.b_rs = q.b_cs = 0;
    q.ldc = 0;
    q.act = g.act;
    q.g = g;
    q.is_conv = 1;
    if (q.M == 0 || q.N == 0)
        return TinyNN_SUCCESS;
    gemm_plan_split(q, ws);
    const bool longk = q.kchunk > 1024;
    if (q.M <= 64 && (long)((q.N + 255) / 256) * q.split >= 128) {
        dim3 grid((q.N + 255) / 256, 1, q.split);
        q.xo = options().no_xcdorder ? XcdOrder{0} : make_xcd_order((int)grid.x, (int)grid.y);
        if (longk)
            hipLaunchKernelGGL((gemm_f32_kernel<true, true, true, 64, true>), grid, dim3(256), 0, stream(), q);
        else
            hipLaunchKernelGGL((gemm_f32_kernel<true, true, true, 64>), grid, dim3(256), 0, stream(), q);
    } else {
        dim3 grid((q.N + GBN - 1) / GBN, (q.M + GBM - 1) / GBM, q.split);
        q.xo = options().no_xcdorder ? XcdOrder{0} : make_xcd_order((int)grid.x, (int)grid.y);
        if (longk)
            hipLaunchKernelGGL((gemm_f32_kernel<true, true, true, 128, true>), grid, dim3(256), 0, stream(), q);
        else
            hipLaunchKernelGGL((gemm_f32_kernel<true, true, true, 128>), grid, dim3(256), 0, stream(), q);
    }
    if (q.split > 1)
        gemm_launch_reduce(q);
    return check_launch("conv_f32_gemm");
}

}  // namespace mg

using namespace mg;

extern "C" TinyNNStatus megcc_gfx950_matmul(
        const MegccMatMulAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace* ws, const RuntimeOpt*) {
    MG_REQUIRE(attr, TinyNN_ERROR_NULL_PTR, "matmul: NULL attr");
    TinyNNStatus st = check_io(inputs, nr_input, 2, 2, outputs, nr_output, "matmul");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor *a = inputs[0], *b = inputs[1], *c = outputs[0];
    // the reference has no quantized MatrixMul for row-major operands on this arch
    // (BareMetal/MatrixMul.cpp:13-23 is f32/f16 only); a qsi8 FullyConnected is a 1x1 conv
    MG_REQUIRE(is_f32(a) && is_f32(b) && is_f32(c), TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "matmul: only f32 is implemented (quantized FullyConnected goes through conv2d)");
    MG_REQUIRE(a->layout.nr_dim == 2 && b->layout.nr_dim == 2 && c->layout.nr_dim == 2,
               TinyNN_ERROR_INVALID_LAYOUT, "matmul: expects 2-d tensors");
    MG_REQUIRE(a->layout.stride[1] == 1 && b->layout.stride[1] == 1 && c->layout.stride[1] == 1,
               TinyNN_ERROR_INVALID_LAYOUT, "matmul: innermost stride must be 1");
    GemmArgs q;
    const int ta = attr->transpose_a != 0, tb = attr->transpose_b != 0;
    q.M = c->layout.dims[0];
    q.N = c->layout.dims[1];
    q.K = ta ? a->layout.dims[0] : a->layout.dims[1];
    MG_REQUIRE((int)(ta ? a->layout.dims[1] : a->layout.dims[0]) == q.M &&
                       (int)(tb ? b->layout.dims[1] : b->layout.dims[0]) == q.K &&
                       (int)(tb ? b->layout.dims[0] : b->layout.dims[1]) == q.N,
               TinyNN_ERROR_INVALID_LAYOUT, "matmul: shapes do not agree");
    const long lda = a->layout.stride[0], ldb = b->layout.stride[0];
    // rows may be padded (a leading dimension larger than the row), never overlapping or reversed
    MG_REQUIRE((a->layout.dims[0] <= 1 || lda >= (long)a->layout.dims[1]) &&
                       (b->layout.dims[0] <= 1 || ldb >= (long)b->layout.dims[1]) &&
                       (c->layout.dims[0] <= 1 || c->layout.stride[0] >= (long)c->layout.dims[1]),
               TinyNN_ERROR_INVALID_LAYOUT, "matmul: a leading stride is shorter than its row");
    q.A = (const float*)a->ptr;
    q.B = (const float*)b->ptr;
    q.C = (float*)c->ptr;
    q.bias = nullptr;
    q.a_rs = ta ? 1 : lda;
    q.a_cs = ta ? lda : 1;
    q.b_rs = tb ? 1 : ldb;
    q.b_cs = tb ? ldb : 1;
    q.ldc = c->layout.stride[0];
    q.act = 0;
    q.is_conv = 0;
    if (q.M == 0 || q.N == 0)
        return TinyNN_SUCCESS;
    if (q.M <= 4 && q.K > 0 && !options().no_gevm) {  // the reference's gevm case: one pass over B
        const GevmArgs v = {q.A, q.B, q.C, q.M, q.N, q.K, q.a_rs, q.a_cs, q.b_rs, q.b_cs, q.ldc};
        if (gevm_f32_supported(v)) {
            note_kernel("gevm_f32");
            return gevm_f32_launch(v);
        }
    }
    gemm_plan_split(q, ws);
    // 64 x 256 tiles when they still give every CU a workgroup
    const bool skinny = q.M <= 64 && (long)((q.N + 255) / 256) * q.split >= 128;
    dim3 grid(skinny ? (q.N + 255) / 256 : (q.N + GBN - 1) / GBN, skinny ? 1 : (q.M + GBM - 1) / GBM,
              q.split);
    q.xo = options().no_xcdorder ? XcdOrder{0} : make_xcd_order((int)grid.x, (int)grid.y);
    note_kernel("gemm_f32", skinny ? 64 : 128, q.split, q.kchunk > 1024, q.xo.w);
    const bool longk = q.kchunk > 1024;
#define MG_GEMM_LAUNCH(AK, BN_)                                                                  \
    do {                                                                                         \
        if (skinny && longk)                                                                     \
            hipLaunchKernelGGL((gemm_f32_kernel<AK, BN_, false, 64, true>), grid, dim3(256), 0,  \
                               stream(), q);                                                     \
        else if (skinny)                                                                         \
            hipLaunchKernelGGL((gemm_f32_kernel<AK, BN_, false, 64>), grid, dim3(256), 0,        \
                               stream(), q);                                                     \
        else if (longk)                                                                          \
            hipLaunchKernelGGL((gemm_f32_kernel<AK, BN_, false, 128, true>), grid, dim3(256), 0, \
                               stream(), q);                                                     \
        else                                                                                     \
            hipLaunchKernelGGL((gemm_f32_kernel<AK, BN_, false, 128>), grid, dim3(256), 0,       \
                               stream(), q);                                                     \
    } while (0)
    if (!ta && !tb)
        MG_GEMM_LAUNCH(true, true);
    else if (!ta && tb)
        MG_GEMM_LAUNCH(true, false);
    else if (ta && !tb)
        MG_GEMM_LAUNCH(false, true);
    else
        MG_GEMM_LAUNCH(false, false);
#undef MG_GEMM_LAUNCH
    if (q.split > 1)
        gemm_launch_reduce(q);
    return check_launch("matmul");
}

// Tiles are staged straight from the operands (the reference packs A and B into workspace,
// GeneralIntrinsic/MatMulKernel/Fp32MatMulM4N12.cpp:47-66); the only scratch is the split-K partial
// sums of skinny problems. Without it (NULL or short workspace) the kernel runs unsplit.
extern "C" TinyNNStatus megcc_gfx950_matmul_workspace(
        const MegccMatMulAttr* attr, Tensor** inputs, int nr_input, int, size_t* workspace) {
    MG_REQUIRE(workspace, TinyNN_ERROR_NULL_PTR, "matmul_workspace: NULL size");
    *workspace = 0;
    if (!attr || !inputs || nr_input < 2 || !inputs[0] || !inputs[1] ||
        inputs[0]->layout.nr_dim != 2 || inputs[1]->layout.nr_dim != 2)
        return TinyNN_SUCCESS;
    const Tensor *a = inputs[0], *b = inputs[1];
    const int ta = attr->transpose_a != 0, tb = attr->transpose_b != 0;
    const long M = ta ? a->layout.dims[1] : a->layout.dims[0];
    const long K = ta ? a->layout.dims[0] : a->layout.dims[1];
    const long N = tb ? b->layout.dims[0] : b->layout.dims[1];
    *workspace = gemm_f32_workspace_bytes(M, N, K, false);
    return TinyNN_SUCCESS;
}
