// qsi8 FullyConnected with few rows (M <= 64): the layer is one pass over the weight matrix, so it
// is bound by how fast the weights stream from HBM, and everything is arranged around that.
//   * a wave owns 32 output channels and a slice of K; its MFMA A operand is the packed filter as
//     it lies (one contiguous KB per wave and 32-channel chunk), fetched straight into registers
//     through a ring of 16 chunks in flight - far more than the
//     bandwidth-latency product;
//   * the activation slice of the workgroup (M rows x the K slice, at most 64 KB) is copied to LDS
//     once, rows of 128 bytes with their 16-byte pieces at piece ^ (row & 7) so that the B-operand
//     reads of 8 consecutive rows hit different banks;
//   * K is split so that about a thousand waves exist; every slice writes its int32 sums to the
//     workspace ([slice][row][oc]) and conv_mfma_reduce_kernel adds them in a fixed order, adds
//     the bias and requantises: integer sums, so the result does not depend on the split.
// Reference loop: BareMetal/ConvKernel.cpp:305-344 on the [M,K,1,1] x [N,K,1,1] layer.
#include "conv_mfma_i8.h"

namespace mg {

struct FcsParams {
    const int8_t* src;
    const int8_t* wp;  // packed filter [K/32][OCP][32], 16-byte halves swapped when (oc >> 3) & 1
    int32_t* partial;  // [split][M][ocs]
    int M, K, OCP, ocs;
    int kslice;        // bytes of K per slice (multiple of 128)
    int oc_tiles;      // ceil(ocs / 32)
};

static constexpr int FCS_RING = 16;

template <int NT>
__global__ void __launch_bounds__(256) fc_stream_kernel(FcsParams q) {
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    constexpr int ROWS = 32 * NT;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, kg = lane >> 5;
    const int z = blockIdx.y, k0 = z * q.kslice;
    const int oct = blockIdx.x * 4 + wave;
    const int nchunks = q.kslice >> 5;
    const bool work = oct < q.oc_tiles;

    // filter chunks: start streaming before anything else
    const int oc = oct * 32 + col;
    const int8_t* arow = q.wp + ((size_t)(k0 >> 5) * q.OCP + oc) * KROW + (((kg ^ (oc >> 3)) & 1) << 4);
    const size_t astep = (size_t)q.OCP * KROW;
    v4i ring[FCS_RING];
    static_for<FCS_RING>([&](auto sc) {
        constexpr int s = decltype(sc)::value;
        ring[s] = work && s < nchunks ? *(const v4i*)(arow + s * astep) : v4i{0, 0, 0, 0};
    });

    // activation slice -> LDS
    const int pieces = q.kslice >> 4;  // 16-byte pieces per row
    for (int i = tid; i < ROWS * pieces; i += 256) {
        const int row = i / pieces, pc = i - row * pieces;
        v4i v = {0, 0, 0, 0};
        if (row < q.M)
            v = *(const v4i*)(q.src + (size_t)row * q.K + k0 + pc * 16);
        *(v4i*)(lds + ((pc >> 3) * ROWS + row) * 128 + (((pc & 7) ^ (row & 7)) << 4)) = v;
    }
    __syncthreads();
    if (!work)
        return;

    v16i acc[NT];
#pragma unroll
    for (int ni = 0; ni < NT; ++ni)
#pragma unroll
        for (int e = 0; e < 16; ++e)
            acc[ni][e] = 0;
    for (int c0 = 0; c0 < nchunks; c0 += FCS_RING) {
        static_for<FCS_RING>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            const int c = c0 + s;
            if (c < nchunks) {
                const v4i a = ring[s];
                if (c + FCS_RING < nchunks)
                    ring[s] = *(const v4i*)(arow + (size_t)(c + FCS_RING) * astep);
                const int piece = (c & 3) * 2 + kg;
#pragma unroll
                for (int ni = 0; ni < NT; ++ni) {
                    const int row = ni * 32 + col;
                    const v4i b = *(const v4i*)(lds + ((c >> 2) * ROWS + row) * 128 +
                                                ((piece ^ (row & 7)) << 4));
                    acc[ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[ni], 0, 0, 0);
                }
            }
        });
    }
    // register e of a tile: channel 8 * (e / 4) + 4 * kg + e % 4 of this wave's 32, row = lane's
#pragma unroll
    for (int ni = 0; ni < NT; ++ni) {
        const int row = ni * 32 + col;
        if (row < q.M) {
            int32_t* out = q.partial + ((size_t)z * q.M + row) * q.ocs + oct * 32 + kg * 4;
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4)
                if (oct * 32 + e4 * 8 + kg * 4 < q.ocs)
                    *(v4i*)(out + e4 * 8) = v4i{acc[ni][e4 * 4], acc[ni][e4 * 4 + 1],
                                                acc[ni][e4 * 4 + 2], acc[ni][e4 * 4 + 3]};
        }
    }
}

// M <= 64 rows, K a multiple of 128, 16-byte aligned operands. Returns the number of K slices (0:
// not for this kernel) for a workspace that holds `ws_bytes`.
int fc_stream_split(const ConvGeom& g, const void* src, size_t ws_bytes, int max_split) {
    if (g.n > 64 || g.n < 1 || (g.ic & 127) || ((uintptr_t)src & 15) || g.oc < 32)
        return 0;
    const int ocs = (g.oc + 3) & ~3;
    const int oc_tiles = (ocs + 31) / 32;
    long s = (1024 + oc_tiles - 1) / oc_tiles;
    if (s > g.ic / 128)
        s = g.ic / 128;
    if (s > max_split)
        s = max_split;
    // the slice of the activations must fit LDS: 64 KB
    const int rows = g.n <= 32 ? 32 : 64;
    while (s < g.ic / 128 && (long)rows * (g.ic / s) > 64 * 1024)
        ++s;
    while (g.ic % (s * 128) && s > 1)
        --s;  // equal slices of whole 128-byte blocks
    if (g.ic % (s * 128) || (long)rows * (g.ic / s) > 64 * 1024)
        return 0;
    if ((size_t)s * g.n * ocs * sizeof(int32_t) > ws_bytes)
        return 0;
    return (int)s;
}

TinyNNStatus fc_stream_launch(
        const ConvGeom& g, const void* src, const void* packed, int32_t* partial, int split) {
    FcsParams q;
    q.src = (const int8_t*)src;
    q.wp = (const int8_t*)packed;
    q.partial = partial;
    q.M = g.n;
    q.K = g.ic;
    q.OCP = (g.oc + OC_PAD - 1) / OC_PAD * OC_PAD;
    q.ocs = (g.oc + 3) & ~3;
    q.kslice = g.ic / split;
    q.oc_tiles = (q.ocs + 31) / 32;
    const int rows = g.n <= 32 ? 32 : 64;
    const size_t lds = (size_t)rows * q.kslice;
    auto kern = rows == 32 ? fc_stream_kernel<1> : fc_stream_kernel<2>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "fc_stream: LDS attribute: %s",
                   hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, dim3((q.oc_tiles + 3) / 4, split), dim3(256), lds, stream(), q);
    return check_launch("fc_stream");
}

}  // namespace mg
