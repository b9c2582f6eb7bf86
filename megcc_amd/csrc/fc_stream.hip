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

// ---- one launch: the K slices of a 32-channel tile meet inside the workgroup ------------------
// The split above costs a second launch and a round trip of the int32 partial sums through memory
// (8 slices of 64 x 4096 sums are half the bytes of the weights themselves). Here a workgroup of 8
// waves owns 32 output channels for the whole of K: wave w multiplies the 128-byte blocks
// w, w + 8, ... of K, with every one of its filter chunks (up to 16 KB) requested before the first
// is used, so a 64 x 4096 x 4096 layer is one memory round trip of 128 KB per workgroup; its
// activations come from L2 (every workgroup reads the same rows), one block ahead. The eight accumulator sets meet in LDS, and the reference's
// epilogue (bias, requantisation, activation: BareMetal/ConvKernel.cpp:327-344) runs once.
struct FcOneParams {
    const int8_t* src;
    const int8_t* wp;  // packed filter, as above
    const int32_t* bias;
    int8_t* dst;  // [M][OC]
    int M, K, OC, OCP, act;
    float s_src, s_flt, s_dst;
};

static constexpr int FO_WAVES = 8, FO_RING = 16;

template <int NT>
__global__ void __launch_bounds__(64 * FO_WAVES) fc_one_kernel(FcOneParams q) {
    __shared__ int32_t red[FO_WAVES][NT * 16][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, kg = lane >> 5;
    const int oct = blockIdx.x, oc = oct * 32 + col;
    const int row0 = blockIdx.y * (32 * NT);  // first row of this workgroup
    // chunk j of this wave is chunk (j & 3) of its (j >> 2)-th 128-byte block of K
    const int blocks = q.K >> 7;
    const int nj = wave < blocks ? ((blocks - wave + FO_WAVES - 1) / FO_WAVES) * 4 : 0;
    const size_t astep = (size_t)q.OCP * KROW;
    const int8_t* arow = q.wp + ((size_t)(wave * 4) * q.OCP + oc) * KROW + (((kg ^ (oc >> 3)) & 1) << 4);
    auto a_at = [&](int j) { return *(const v4i*)(arow + (size_t)((j >> 2) * (4 * FO_WAVES) + (j & 3)) * astep); };
    // activations: the wave's 128-byte blocks of K, whole lines at a time (8 lanes per row), through
    // a staging area of its own: rows of 128 bytes with their 16-byte pieces at piece ^ (row & 7),
    // so that the B-operand reads of 8 consecutive rows hit different banks. The area is the wave's
    // slot of `red`: it is free again when the wave's last product has been issued.
    constexpr int AL = 4 * NT;  // loads per lane and block: rows 8 i + lane / 8
    int8_t* stage = (int8_t*)&red[wave][0][0];
    const int srow = lane >> 3, apc = lane & 7, nb = nj >> 2;
    const int8_t* asrc = q.src + (size_t)(row0 + srow) * q.K + wave * 128 + apc * 16;
    v4i areg[2][AL];  // two blocks ahead: a block is one L2 round trip
    auto act_load = [&](int blk, auto par) {
#pragma unroll
        for (int i = 0; i < AL; ++i)
            areg[decltype(par)::value][i] = row0 + i * 8 + srow < q.M
                            ? *(const v4i*)(asrc + (size_t)(i * 8) * q.K + (size_t)blk * (128 * FO_WAVES))
                            : v4i{0, 0, 0, 0};
    };
    auto act_store = [&](auto par) {
#pragma unroll
        for (int i = 0; i < AL; ++i)
            *(v4i*)(stage + (i * 8 + srow) * 128 + ((apc ^ srow) << 4)) = areg[decltype(par)::value][i];
    };
    if (nb > 0)
        act_load(0, std::integral_constant<int, 0>{});
    if (nb > 1)
        act_load(1, std::integral_constant<int, 1>{});
    v4i ring[FO_RING];
    static_for<FO_RING>([&](auto sc) {
        constexpr int s = decltype(sc)::value;
        ring[s] = s < nj ? a_at(s) : v4i{0, 0, 0, 0};
    });
    v16i acc[NT];
#pragma unroll
    for (int ni = 0; ni < NT; ++ni)
#pragma unroll
        for (int e = 0; e < 16; ++e)
            acc[ni][e] = 0;
    for (int j0 = 0; j0 < nj; j0 += FO_RING) {
        static_for<FO_RING / 4>([&](auto bc) {
            constexpr int bb = decltype(bc)::value;
            const int blk = (j0 >> 2) + bb;
            if (blk < nb) {
                constexpr std::integral_constant<int, bb & 1> par{};
                act_store(par);  // (LDS operations of one wave execute in order)
                if (blk + 2 < nb)
                    act_load(blk + 2, par);
                static_for<4>([&](auto cc_) {
                    constexpr int cc = decltype(cc_)::value, s = bb * 4 + cc;
                    const int j = j0 + s;
                    const v4i a = ring[s];
                    if (j + FO_RING < nj)
                        ring[s] = a_at(j + FO_RING);
#pragma unroll
                    for (int ni = 0; ni < NT; ++ni) {
                        const int row = ni * 32 + col;
                        const v4i b = *(const v4i*)(stage + row * 128 + (((cc * 2 + kg) ^ (row & 7)) << 4));
                        acc[ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[ni], 0, 0, 0);
                    }
                });
            }
        });
    }
#pragma unroll
    for (int ni = 0; ni < NT; ++ni)
#pragma unroll
        for (int e = 0; e < 16; ++e)
            red[wave][ni * 16 + e][lane] = acc[ni][e];
    __syncthreads();
    // thread -> (row half ni, register quad e4, lane): registers 4 e4 .. 4 e4 + 3 of a lane are the
    // channels 8 e4 + 4 kg .. + 3 of the tile for row ni * 32 + col
    const int grp = tid >> 6;
    if (grp >= NT * 4)
        return;
    const int ni = grp >> 2, e4 = grp & 3;
    const int row = row0 + ni * 32 + col, ocb = oct * 32 + e4 * 8 + kg * 4;
    if (row >= q.M || ocb >= q.OC)
        return;
    int r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        int sum = 0;
#pragma unroll
        for (int w = 0; w < FO_WAVES; ++w)
            sum += red[w][ni * 16 + e4 * 4 + e][lane];
        const int b = (q.bias && ocb + e < q.OC) ? q.bias[ocb + e] : 0;
        r[e] = requant_conv_rt(q.act, sum + b, q.s_src, q.s_flt, q.s_dst);
    }
    int8_t* o = q.dst + (size_t)row * q.OC + ocb;
    if ((q.OC & 3) == 0) {
        *(uint32_t*)o = pack4(r[0], r[1], r[2], r[3]);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (ocb + e < q.OC)
                o[e] = (int8_t)r[e];
    }
}

// The same workgroup for K <= 4096 (at most NB = 4 blocks of K per wave) and 32 rows: every global
// load of the wave - its activations and its filter chunks - is issued at the top, without a
// condition. A load that is issued under a condition (a prefetch inside `if (block + 2 < blocks)`,
// a row test around the load) leaves the compiler unable to count how many loads are outstanding
// behind an earlier one, and it then waits for ALL of them before the first use: each prefetch
// became a round trip of its own. Here a wave with fewer blocks than NB, or none, fetches a block it
// has a right to read again and multiplies it with zeros; rows beyond M read row M - 1 and are
// zeroed on their way into LDS.
template <int NB>
__global__ void __launch_bounds__(64 * FO_WAVES) fc_one32_kernel(FcOneParams q) {
    __shared__ int32_t red[FO_WAVES][16][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, kg = lane >> 5;
    const int oct = blockIdx.x, oc = oct * 32 + col;
    const int row0 = blockIdx.y * 32;
    const int blocks = q.K >> 7;
    const int myb = wave < blocks ? (blocks - wave + FO_WAVES - 1) / FO_WAVES : 0;  // <= NB
    const int wv = myb ? wave : 0;
    const size_t astep = (size_t)q.OCP * KROW;
    const int8_t* arow = q.wp + ((size_t)(wv * 4) * q.OCP + oc) * KROW + (((kg ^ (oc >> 3)) & 1) << 4);
    int8_t* stage = (int8_t*)&red[wave][0][0];  // 4 KB: 32 rows of 128 bytes, pieces at piece ^ (row & 7)
    const int srow = lane >> 3, apc = lane & 7;
    v4i areg[NB][4], ring[NB * 4];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int bc = b < myb ? b : 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = min(row0 + i * 8 + srow, q.M - 1);
            areg[b][i] = *(const v4i*)(q.src + (size_t)row * q.K + (wv + FO_WAVES * bc) * 128 + apc * 16);
        }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int bc = b < myb ? b : 0;
#pragma unroll
        for (int cc = 0; cc < 4; ++cc)
            ring[b * 4 + cc] = *(const v4i*)(arow + (size_t)(bc * (4 * FO_WAVES) + cc) * astep);
    }
    // (the scheduler otherwise moves each load down to a few instructions before its use)
    __builtin_amdgcn_sched_barrier(0);
    v16i acc;
#pragma unroll
    for (int e = 0; e < 16; ++e)
        acc[e] = 0;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool ok = row0 + i * 8 + srow < q.M && b < myb;
            v4i v = areg[b][i];
            v.x = ok ? v.x : 0, v.y = ok ? v.y : 0, v.z = ok ? v.z : 0, v.w = ok ? v.w : 0;
            *(v4i*)(stage + (i * 8 + srow) * 128 + ((apc ^ srow) << 4)) = v;  // (a wave's LDS operations execute in order)
        }
        // (no `if (b < myb)` here: the compiler would sink the block's filter loads into it, next to
        //  their use, one round trip each; a block the wave does not own multiplies zeros)
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            const v4i bo = *(const v4i*)(stage + col * 128 + (((cc * 2 + kg) ^ (col & 7)) << 4));
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[b * 4 + cc], bo, acc, 0, 0, 0);
        }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e)
        red[wave][e][lane] = acc[e];
    __syncthreads();
    const int e4 = tid >> 6;
    if (e4 >= 4)
        return;
    const int row = row0 + col, ocb = oct * 32 + e4 * 8 + kg * 4;
    if (row >= q.M || ocb >= q.OC)
        return;
    int bias[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
        bias[e] = q.bias ? q.bias[min(ocb + e, q.OC - 1)] : 0;
    int r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        int sum = 0;
#pragma unroll
        for (int w = 0; w < FO_WAVES; ++w)
            sum += red[w][e4 * 4 + e][lane];
        r[e] = requant_conv_rt(q.act, sum + bias[e], q.s_src, q.s_flt, q.s_dst);
    }
    int8_t* o = q.dst + (size_t)row * q.OC + ocb;
    if ((q.OC & 3) == 0) {
        *(uint32_t*)o = pack4(r[0], r[1], r[2], r[3]);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (ocb + e < q.OC)
                o[e] = (int8_t)r[e];
    }
}

// M <= 64 rows, K a multiple of 128, 16-byte aligned activations
bool fc_one_supported(const ConvGeom& g, const void* src) {
    return g.n >= 1 && g.n <= 64 && g.ic >= 128 && (g.ic & 127) == 0 && ((uintptr_t)src & 15) == 0 &&
           g.oc >= 1;
}

TinyNNStatus fc_one_launch(
        const ConvGeom& g, const void* src, const void* packed, const void* bias, void* dst) {
    FcOneParams q;
    q.src = (const int8_t*)src;
    q.wp = (const int8_t*)packed;
    q.bias = (const int32_t*)bias;
    q.dst = (int8_t*)dst;
    q.M = g.n;
    q.K = g.ic;
    q.OC = g.oc;
    q.OCP = (g.oc + OC_PAD - 1) / OC_PAD * OC_PAD;
    q.act = g.act;
    q.s_src = g.s_src;
    q.s_flt = g.s_flt;
    q.s_dst = g.s_dst;
    const int oc_tiles = (g.oc + 31) / 32;
    // 33..64 rows: two workgroups of 32 rows per channel tile while that still is one workgroup per
    // CU - what a CU pulls through its L2 port (its share of the weights + the activations of its
    // rows) bounds the kernel: 64 x 4096 x 4096 8.1 -> 6.6 us. (With a multiple of 8 channel tiles the
    // two are on the same XCD: the weights still leave HBM once.)
    const bool rows32 = g.n <= 32 || oc_tiles * 2 <= num_cus();
    const int nb = rows32 && g.ic <= 4096 ? (g.ic / 128 + FO_WAVES - 1) / FO_WAVES : 0;  // blocks per wave
    note_kernel("fc_one", rows32 ? 32 : 64, nb);
    const dim3 grid32(oc_tiles, (g.n + 31) / 32), block(64 * FO_WAVES);
    if (nb == 1)
        hipLaunchKernelGGL(fc_one32_kernel<1>, grid32, block, 0, stream(), q);
    else if (nb == 2)
        hipLaunchKernelGGL(fc_one32_kernel<2>, grid32, block, 0, stream(), q);
    else if (nb >= 3)
        hipLaunchKernelGGL(fc_one32_kernel<4>, grid32, block, 0, stream(), q);
    else if (rows32)
        hipLaunchKernelGGL(fc_one_kernel<1>, dim3(oc_tiles, (g.n + 31) / 32), dim3(64 * FO_WAVES), 0, stream(), q);
    else
        hipLaunchKernelGGL(fc_one_kernel<2>, dim3(oc_tiles), dim3(64 * FO_WAVES), 0, stream(), q);
    return check_launch("fc_one");
}

}  // namespace mg
