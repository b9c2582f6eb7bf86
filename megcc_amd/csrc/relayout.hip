// Relayout and Concat: copies between strided views.
//
// Relayout (compiler/lib/KernelGen/BareMetal/Relayout.cpp:13-101, helpers in
// KernelGen/Common/Relayout.h:10-80): source and destination hold the same number of elements of
// the same dtype; each side is walked in the row-major order of its OWN dims with its OWN strides
// (in elements, negative and zero source strides allowed), and the k-th element of the source is
// written to the k-th element of the destination. The reference collapses each layout, memcpy's
// when both are dense, and otherwise walks the two iterators on one core.
//
// Concat (BareMetal/Concat.cpp:14-76): input i is copied into the slice of the output that starts
// at sum(dims[axis] of the inputs before it) along `axis`; it is the same strided copy once per
// input.
//
// Here one copy is planned on the host in four steps and runs as one kernel:
//   1. each side is collapsed (extent-1 dims dropped, neighbours merged when
//      stride[i] == dims[i+1] * stride[i+1]);
//   2. the two sides are brought to one index space: equal collapsed dims are taken as they are,
//      a dense side takes the dims of the other one; what is left (two differently shaped strided
//      views) runs on the two-decomposition kernel below;
//   3. in the common space dims are merged again when both sides allow it, ordered by falling
//      |destination stride| (any order of the dims copies the same elements), and, when the last
//      dim is dense on both sides, the element is widened to 2/4/8/16 bytes as far as extents,
//      strides and addresses allow;
//   4. kernel choice: `relayout_rows_kernel` (one thread per element, the destination's densest
//      dim across lanes) unless the source's dense dim is another one than the destination's -
//      then `relayout_tile_kernel` moves 4096-element tiles of those two dims through LDS so that
//      both the reads and the writes of a wavefront are runs of consecutive addresses.
// HBM-bound: algorithmic traffic is one read and one write of every element.
#include <algorithm>
#include <vector>

#include "common.h"
#include "fastdiv.h"

namespace mg {
namespace {

constexpr int RL_MAX_DIM = MAX_DIM;

struct Dim {
    uint32_t extent;
    long long ss, ds;  // strides in elements
};

struct RowsParams {
    int nd;  // >= 1
    FastDiv div[RL_MAX_DIM];
    long long ss[RL_MAX_DIM], ds[RL_MAX_DIM];
    uint32_t total;
};

// One thread per element of the common index space, last dim fastest.
template <typename T>
__global__ void __launch_bounds__(256) relayout_rows_kernel(
        const T* __restrict__ src, T* __restrict__ dst, const RowsParams p) {
    uint32_t k = blockIdx.x * 256u + threadIdx.x;
    if (k >= p.total)
        return;
    long long so = 0, doff = 0;
#pragma unroll
    for (int i = RL_MAX_DIM - 1; i >= 0; --i) {
        if (i < p.nd) {
            uint32_t q = fdiv(k, p.div[i]);
            uint32_t r = k - q * p.div[i].d;
            so += (long long)r * p.ss[i];
            doff += (long long)r * p.ds[i];
            k = q;
        }
    }
    dst[doff] = src[so];
}

struct PairParams {
    int snd, dnd;
    FastDiv sdiv[RL_MAX_DIM], ddiv[RL_MAX_DIM];
    long long ss[RL_MAX_DIM], ds[RL_MAX_DIM];
    uint32_t total;
};

// Two strided views with different dims: the element number is decomposed once per side.
template <typename T>
__global__ void __launch_bounds__(256) relayout_pair_kernel(
        const T* __restrict__ src, T* __restrict__ dst, const PairParams p) {
    const uint32_t k0 = blockIdx.x * 256u + threadIdx.x;
    if (k0 >= p.total)
        return;
    long long so = 0, doff = 0;
    uint32_t k = k0;
#pragma unroll
    for (int i = RL_MAX_DIM - 1; i >= 0; --i) {
        if (i < p.snd) {
            uint32_t q = fdiv(k, p.sdiv[i]);
            so += (long long)(k - q * p.sdiv[i].d) * p.ss[i];
            k = q;
        }
    }
    k = k0;
#pragma unroll
    for (int i = RL_MAX_DIM - 1; i >= 0; --i) {
        if (i < p.dnd) {
            uint32_t q = fdiv(k, p.ddiv[i]);
            doff += (long long)(k - q * p.ddiv[i].d) * p.ds[i];
            k = q;
        }
    }
    dst[doff] = src[so];
}

constexpr int TILE_ELEMS = 4096;

struct TileParams {
    // dims [0, nb) are the batch dims; A is the dim the source is dense in, B the one the
    // destination is dense in
    int nb;
    FastDiv div[RL_MAX_DIM];
    long long ss[RL_MAX_DIM], ds[RL_MAX_DIM];
    uint32_t ext_a, ext_b;
    long long sa, sb, da, db;
    uint32_t ta, tb;        // tile extents, powers of two, ta * tb <= TILE_ELEMS
    uint32_t tile_elems;
    uint32_t row;           // LDS row length, ta + padding
    uint32_t log_ta, log_tb;
    FastDiv tiles_a, tiles_b;  // number of tiles along A and B
};

// A block moves one ta x tb tile: reads walk A across lanes, writes walk B across lanes. The LDS
// copy is [b][a] with padded rows, so that the column reads of the write phase fall into
// different banks.
template <typename T>
__global__ void __launch_bounds__(256) relayout_tile_kernel(
        const T* __restrict__ src, T* __restrict__ dst, const TileParams p) {
    __shared__ T tile[TILE_ELEMS + TILE_ELEMS / 4 + 64];
    uint32_t blk = blockIdx.x;
    uint32_t q = fdiv(blk, p.tiles_b);
    const uint32_t b0 = (blk - q * p.tiles_b.d) << p.log_tb;
    blk = q;
    q = fdiv(blk, p.tiles_a);
    const uint32_t a0 = (blk - q * p.tiles_a.d) << p.log_ta;
    blk = q;
    long long so = 0, doff = 0;
#pragma unroll
    for (int i = RL_MAX_DIM - 1; i >= 0; --i) {
        if (i < p.nb) {
            q = fdiv(blk, p.div[i]);
            const uint32_t r = blk - q * p.div[i].d;
            so += (long long)r * p.ss[i];
            doff += (long long)r * p.ds[i];
            blk = q;
        }
    }
    // (the launcher has checked that offsets inside one tile fit 32 bits)
    src += so + (long long)a0 * p.sa + (long long)b0 * p.sb;
    dst += doff + (long long)a0 * p.da + (long long)b0 * p.db;
    const int sa = (int)p.sa, sb = (int)p.sb, da = (int)p.da, db = (int)p.db;
    const uint32_t na = min(p.ta, p.ext_a - a0), nb = min(p.tb, p.ext_b - b0);
    const uint32_t row = p.row;
#pragma unroll 4
    for (uint32_t e = threadIdx.x; e < p.tile_elems; e += 256) {
        const uint32_t a = e & (p.ta - 1), b = e >> p.log_ta;
        if (a < na && b < nb)
            tile[b * row + a] = src[(int)a * sa + (int)b * sb];
    }
    __syncthreads();
#pragma unroll 4
    for (uint32_t e = threadIdx.x; e < p.tile_elems; e += 256) {
        const uint32_t b = e & (p.tb - 1), a = e >> p.log_tb;
        if (a < na && b < nb)
            dst[(int)a * da + (int)b * db] = tile[b * row + a];
    }
}

struct Tile4Params {
    int nb;
    FastDiv div[RL_MAX_DIM];
    long long ss[RL_MAX_DIM], ds[RL_MAX_DIM];
    uint32_t ext_a, ext_b;  // bytes, multiples of 4
    long long sb, da;       // source stride of B, destination stride of A (sa == db == 1)
    uint32_t log_ta4, log_tb4;  // tile extents in units of 4 bytes
    FastDiv tiles_a, tiles_b;
};

constexpr int TILE4_WORDS = 4096;  // 16 KB of bytes per tile

// The byte transpose: every thread loads 4 rows of 4 consecutive source bytes as dwords,
// transposes the 4 x 4 bytes in registers and parks the 4 resulting dwords (4 consecutive
// destination bytes each) in LDS, plane i = a % 4, [a / 4][b / 4] with odd row length; the write
// phase reads them back with B across lanes. All global and LDS accesses are dwords.
__global__ void __launch_bounds__(256) relayout_tile_b4_kernel(
        const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, const Tile4Params p) {
    __shared__ uint32_t tile[2 * TILE4_WORDS];
    uint32_t blk = blockIdx.x;
    uint32_t q = fdiv(blk, p.tiles_b);
    const uint32_t b0 = (blk - q * p.tiles_b.d) << (p.log_tb4 + 2);
    blk = q;
    q = fdiv(blk, p.tiles_a);
    const uint32_t a0 = (blk - q * p.tiles_a.d) << (p.log_ta4 + 2);
    blk = q;
    long long so = 0, doff = 0;
#pragma unroll
    for (int i = RL_MAX_DIM - 1; i >= 0; --i) {
        if (i < p.nb) {
            q = fdiv(blk, p.div[i]);
            const uint32_t r = blk - q * p.div[i].d;
            so += (long long)r * p.ss[i];
            doff += (long long)r * p.ds[i];
            blk = q;
        }
    }
    src += so + a0 + (long long)b0 * p.sb;
    dst += doff + (long long)a0 * p.da + b0;
    const int sb = (int)p.sb, da = (int)p.da;
    const uint32_t ta4 = 1u << p.log_ta4, tb4 = 1u << p.log_tb4;
    const uint32_t na4 = min(ta4, (p.ext_a - a0) >> 2), nb4 = min(tb4, (p.ext_b - b0) >> 2);
    const uint32_t row = tb4 + 1, plane = ta4 * row;
    const uint32_t items = ta4 << p.log_tb4;
    for (uint32_t e = threadIdx.x; e < items; e += 256) {
        const uint32_t a4 = e & (ta4 - 1), b4 = e >> p.log_ta4;
        if (a4 < na4 && b4 < nb4) {
            const uint8_t* s = src + (int)(4 * a4) + (int)(4 * b4) * sb;
            const uint32_t w0 = *(const uint32_t*)s, w1 = *(const uint32_t*)(s + sb),
                           w2 = *(const uint32_t*)(s + 2 * sb), w3 = *(const uint32_t*)(s + 3 * sb);
            uint32_t* t = tile + a4 * row + b4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                t[i * plane] = ((w0 >> (8 * i)) & 0xff) | (((w1 >> (8 * i)) & 0xff) << 8) |
                               (((w2 >> (8 * i)) & 0xff) << 16) | (((w3 >> (8 * i)) & 0xff) << 24);
        }
    }
    __syncthreads();
    for (uint32_t e = threadIdx.x; e < 4 * items; e += 256) {
        const uint32_t b4 = e & (tb4 - 1), a = e >> p.log_tb4;
        if (a < 4 * na4 && b4 < nb4)
            *(uint32_t*)(dst + (int)a * da + (int)(4 * b4)) =
                    tile[(a & 3) * plane + (a >> 2) * row + b4];
    }
}

long long iabs(long long v) {
    return v < 0 ? -v : v;
}

// step 1 of the plan (the reference's collapse_contiguous): (extent, stride) pairs
std::vector<std::pair<uint32_t, long long>> collapse(const Layout& l) {
    std::vector<std::pair<uint32_t, long long>> out;
    for (int i = 0; i < l.nr_dim; ++i) {
        if (l.dims[i] == 1)
            continue;
        if (!out.empty() && out.back().second == (long long)l.dims[i] * l.stride[i]) {
            out.back().first *= l.dims[i];
            out.back().second = l.stride[i];
        } else {
            out.emplace_back(l.dims[i], (long long)l.stride[i]);
        }
    }
    return out;
}

bool dense(const std::vector<std::pair<uint32_t, long long>>& c) {
    return c.empty() || (c.size() == 1 && c[0].second == 1);
}

// row-major strides for `dims` (the dense side reshaped to the other side's dims)
void reshape_dense(const std::vector<std::pair<uint32_t, long long>>& like,
                   std::vector<long long>* strides) {
    strides->assign(like.size(), 1);
    long long s = 1;
    for (int i = (int)like.size() - 1; i >= 0; --i) {
        (*strides)[i] = s;
        s *= like[i].first;
    }
}

template <typename T>
void launch_rows(const void* src, void* dst, const std::vector<Dim>& d, uint32_t total) {
    RowsParams p = {};
    p.nd = (int)d.size();
    for (int i = 0; i < p.nd; ++i) {
        p.div[i] = make_fastdiv(d[i].extent);
        p.ss[i] = d[i].ss;
        p.ds[i] = d[i].ds;
    }
    p.total = total;
    hipLaunchKernelGGL(relayout_rows_kernel<T>, dim3(ceil_div(total, 256)), dim3(256), 0, stream(),
                       (const T*)src, (T*)dst, p);
}

uint32_t log2_ceil(uint32_t v) {
    uint32_t s = 0;
    while ((1u << s) < v)
        ++s;
    return s;
}

// Tile extent 2^k, floor <= k <= most, that wastes the least of the last tile of `extent`
// (the largest one among equals).
uint32_t best_log_tile(uint32_t extent, uint32_t most, uint32_t floor) {
    uint32_t best = most;
    size_t best_cover = (size_t)ceil_div(extent, 1u << most) << most;
    for (uint32_t k = most; k > floor; --k) {
        const size_t cover = (size_t)ceil_div(extent, 1u << (k - 1)) << (k - 1);
        if (cover < best_cover) {
            best_cover = cover;
            best = k - 1;
        }
    }
    return best;
}

template <typename T>
bool launch_tile(const void* src, void* dst, const std::vector<Dim>& d, int ia) {
    const int ib = (int)d.size() - 1;
    TileParams p = {};
    size_t batch = 1;
    for (int i = 0; i < (int)d.size(); ++i) {
        if (i == ia || i == ib)
            continue;
        p.div[p.nb] = make_fastdiv(d[i].extent);
        p.ss[p.nb] = d[i].ss;
        p.ds[p.nb] = d[i].ds;
        ++p.nb;
        batch *= d[i].extent;
    }
    p.ext_a = d[ia].extent;
    p.ext_b = d[ib].extent;
    p.sa = d[ia].ss; p.da = d[ia].ds;
    p.sb = d[ib].ss; p.db = d[ib].ds;
    // square tiles unless one of the two dims is short; a tile is never larger than the two
    // extents need (the padded LDS copy, tb rows of at most ta + 32 elements, stays inside the array:
    // tb * pad is 64 for ta >= 32 and the whole tile is small otherwise)
    const uint32_t la = std::max(log2_ceil(p.ext_a), 2u), lb = std::max(log2_ceil(p.ext_b), 1u);
    p.log_ta = std::min(la, 6u);
    p.log_tb = std::min(lb, 12 - p.log_ta);
    p.log_ta = std::min(la, 12 - p.log_tb);
    if (p.log_ta > 8)
        p.log_ta = best_log_tile(p.ext_a, p.log_ta, 8);
    else if (p.log_tb > 8)
        p.log_tb = best_log_tile(p.ext_b, p.log_tb, 8);
    p.ta = 1u << p.log_ta;
    p.tb = 1u << p.log_tb;
    p.tile_elems = p.ta * p.tb;
    // The write phase reads LDS with B across lanes: 64 / tb values of A per wavefront when the
    // tile is narrow. The row length makes those tb * (64 / tb) dwords fall into distinct banks
    // (twice each of the 32, the least 64 lanes can do): row = 64 / tb (mod 32), at least ta + 1.
    uint32_t pad = 1;
    if (p.tb < 64)
        pad = ((64 / p.tb) + 32 - p.ta % 32) % 32;
    if (pad == 0)
        pad = 32;
    p.row = p.ta + pad;
    const size_t na = ceil_div(p.ext_a, p.ta), nb = ceil_div(p.ext_b, p.tb);
    p.tiles_a = make_fastdiv((uint32_t)na);
    p.tiles_b = make_fastdiv((uint32_t)nb);
    const size_t blocks = batch * na * nb;
    const long long lim = 1ll << 31;
    if (blocks >= (1u << 31) || p.ta * iabs(p.sa) + p.tb * iabs(p.sb) >= lim ||
        p.ta * iabs(p.da) + p.tb * iabs(p.db) >= lim)
        return false;
    hipLaunchKernelGGL(relayout_tile_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream(),
                       (const T*)src, (T*)dst, p);
    return true;
}

// The dword version of the tile kernel for 1-byte elements; false when an extent, a stride or an
// address is not a multiple of 4 or a direction is reversed.
bool launch_tile_b4(const void* src, void* dst, const std::vector<Dim>& d, int ia) {
    const int ib = (int)d.size() - 1;
    if (d[ia].ss != 1 || d[ib].ds != 1 || d[ia].extent % 4 || d[ib].extent % 4 ||
        d[ia].ds % 4 || d[ib].ss % 4 || (uintptr_t)src % 4 || (uintptr_t)dst % 4)
        return false;
    Tile4Params p = {};
    size_t batch = 1;
    for (int i = 0; i < (int)d.size(); ++i) {
        if (i == ia || i == ib)
            continue;
        if (d[i].ss % 4 || d[i].ds % 4)
            return false;
        p.div[p.nb] = make_fastdiv(d[i].extent);
        p.ss[p.nb] = d[i].ss;
        p.ds[p.nb] = d[i].ds;
        ++p.nb;
        batch *= d[i].extent;
    }
    p.ext_a = d[ia].extent;
    p.ext_b = d[ib].extent;
    p.sb = d[ib].ss;
    p.da = d[ia].ds;
    // 128 x 128 bytes unless one of the two dims is short (ta4 * tb4 <= TILE4_WORDS / 4, so the
    // 4 padded planes, 4 * ta4 * (tb4 + 1) dwords, fit the array)
    const uint32_t la = log2_ceil(p.ext_a / 4), lb = log2_ceil(p.ext_b / 4);
    p.log_ta4 = std::min(la, 5u);
    p.log_tb4 = std::min(lb, 10 - p.log_ta4);
    p.log_ta4 = std::min(la, 10 - p.log_tb4);
    const uint32_t ta = 4u << p.log_ta4, tb = 4u << p.log_tb4;
    const size_t na = ceil_div(p.ext_a, ta), nb = ceil_div(p.ext_b, tb);
    p.tiles_a = make_fastdiv((uint32_t)na);
    p.tiles_b = make_fastdiv((uint32_t)nb);
    const size_t blocks = batch * na * nb;
    const long long lim = 1ll << 31;
    if (blocks >= (1u << 31) || ta + tb * iabs(p.sb) >= lim || ta * iabs(p.da) + tb >= lim)
        return false;
    hipLaunchKernelGGL(relayout_tile_b4_kernel, dim3((unsigned)blocks), dim3(256), 0, stream(),
                       (const uint8_t*)src, (uint8_t*)dst, p);
    return true;
}

template <typename T>
void launch_pair(const void* src, void* dst,
                 const std::vector<std::pair<uint32_t, long long>>& s,
                 const std::vector<std::pair<uint32_t, long long>>& d, uint32_t total) {
    PairParams p = {};
    p.snd = (int)s.size();
    p.dnd = (int)d.size();
    for (int i = 0; i < p.snd; ++i) {
        p.sdiv[i] = make_fastdiv(s[i].first);
        p.ss[i] = s[i].second;
    }
    for (int i = 0; i < p.dnd; ++i) {
        p.ddiv[i] = make_fastdiv(d[i].first);
        p.ds[i] = d[i].second;
    }
    p.total = total;
    hipLaunchKernelGGL(relayout_pair_kernel<T>, dim3(ceil_div(total, 256)), dim3(256), 0, stream(),
                       (const T*)src, (T*)dst, p);
}

struct alignas(8) B8 {
    uint32_t v[2];
};
struct alignas(16) B16 {
    uint32_t v[4];
};

#define RL_BY_SIZE(es, CALL)                                                            \
    switch (es) {                                                                       \
        case 1: CALL(uint8_t); break;                                                   \
        case 2: CALL(uint16_t); break;                                                  \
        case 4: CALL(uint32_t); break;                                                  \
        case 8: CALL(B8); break;                                                        \
        default: CALL(B16); break;                                                      \
    }

}  // namespace

// Copies `src` (layout sl) to `dst` (layout dl), elements of `es` bytes. Both layouts hold the
// same number of elements. Launches at most one kernel or one device-to-device copy.
TinyNNStatus strided_copy(
        const void* src, const Layout& sl, void* dst, const Layout& dl, size_t es,
        const char* who) {
    const size_t es0 = es;
    const size_t total = nr_elem(sl);
    MG_REQUIRE(total == nr_elem(dl), TinyNN_ERROR_INVALID_LAYOUT,
               "%s: source has %zu elements, destination %zu", who, total, nr_elem(dl));
    if (total == 0)
        return TinyNN_SUCCESS;
    MG_REQUIRE(total < (1u << 31), TinyNN_ERROR_OUT_OF_RANGE, "%s: %zu elements", who, total);
    auto sc = collapse(sl), dc = collapse(dl);
    for (auto& d : dc)
        MG_REQUIRE(d.second != 0, TinyNN_ERROR_INVALID_LAYOUT,
                   "%s: destination stride 0 over %u elements", who, d.first);
    if (dense(sc) && dense(dc)) {
        if (hipMemcpyAsync(dst, src, total * es, hipMemcpyDeviceToDevice, stream()) != hipSuccess)
            return fail(TinyNN_ERROR_RUNTIME, "%s: device copy failed", who);
        return TinyNN_SUCCESS;
    }

    // step 2
    std::vector<Dim> dims;
    bool common = false;
    if (sc.size() == dc.size()) {
        common = true;
        for (size_t i = 0; i < sc.size(); ++i)
            common = common && sc[i].first == dc[i].first;
        if (common)
            for (size_t i = 0; i < sc.size(); ++i)
                dims.push_back({sc[i].first, sc[i].second, dc[i].second});
    }
    if (!common && (dense(sc) || dense(dc))) {
        std::vector<long long> st;
        if (dense(sc)) {
            reshape_dense(dc, &st);
            for (size_t i = 0; i < dc.size(); ++i)
                dims.push_back({dc[i].first, st[i], dc[i].second});
        } else {
            reshape_dense(sc, &st);
            for (size_t i = 0; i < sc.size(); ++i)
                dims.push_back({sc[i].first, sc[i].second, st[i]});
        }
        common = true;
    }
    if (!common) {
#define CALL(T) launch_pair<T>(src, dst, sc, dc, (uint32_t)total)
        RL_BY_SIZE(es, CALL)
#undef CALL
        return check_launch(who);
    }

    // step 3: merge, order, widen
    {
        std::vector<Dim> m;
        for (const Dim& d : dims) {
            if (!m.empty() && m.back().ss == (long long)d.extent * d.ss &&
                m.back().ds == (long long)d.extent * d.ds) {
                m.back().extent *= d.extent;
                m.back().ss = d.ss;
                m.back().ds = d.ds;
            } else {
                m.push_back(d);
            }
        }
        dims.swap(m);
    }
    std::stable_sort(dims.begin(), dims.end(),
                     [](const Dim& a, const Dim& b) { return iabs(a.ds) > iabs(b.ds); });
    uint32_t n = (uint32_t)total;
    Dim& last = dims.back();
    if (last.ss == 1 && last.ds == 1) {
        while (es < 16) {
            bool ok = last.extent % 2 == 0 && (uintptr_t)src % (2 * es) == 0 &&
                      (uintptr_t)dst % (2 * es) == 0;
            for (size_t i = 0; ok && i + 1 < dims.size(); ++i)
                ok = dims[i].ss % 2 == 0 && dims[i].ds % 2 == 0;
            if (!ok)
                break;
            last.extent /= 2;
            for (size_t i = 0; i + 1 < dims.size(); ++i) {
                dims[i].ss /= 2;
                dims[i].ds /= 2;
            }
            es *= 2;
            n /= 2;
        }
    }

    // The plan must touch exactly the address range the caller's layouts describe.
    {
        long long lo[4] = {0, 0, 0, 0}, hi[4] = {0, 0, 0, 0};
        auto widen = [](long long stride, uint32_t extent, long long* l, long long* h) {
            (stride < 0 ? *l : *h) += stride * (long long)(extent - 1);
        };
        for (const Dim& d : dims) {
            widen(d.ss, d.extent, &lo[0], &hi[0]);
            widen(d.ds, d.extent, &lo[1], &hi[1]);
        }
        for (auto& d : sc)
            widen(d.second, d.first, &lo[2], &hi[2]);
        for (auto& d : dc)
            widen(d.second, d.first, &lo[3], &hi[3]);
        const long long w = (long long)(es / es0);
        MG_REQUIRE(lo[0] * w == lo[2] && (hi[0] + 1) * w == hi[2] + 1 && lo[1] * w == lo[3] &&
                           (hi[1] + 1) * w == hi[3] + 1,
                   TinyNN_ERROR_RUNTIME, "%s: internal error, plan leaves the tensors' extent", who);
    }

    // step 4
    int ia = -1;
    if (iabs(last.ds) == 1 && iabs(last.ss) != 1) {
        for (int i = 0; i + 1 < (int)dims.size(); ++i)
            if (iabs(dims[i].ss) == 1 && dims[i].extent >= 2 && (ia < 0 || dims[i].extent > dims[ia].extent))
                ia = i;
    }
    if (ia >= 0 && last.extent >= 2) {  // (es is still the dtype's size: nothing was widened)
        bool done = false;
        switch (es) {
            case 1:
                done = launch_tile_b4(src, dst, dims, ia) ||
                       launch_tile<uint8_t>(src, dst, dims, ia);
                break;
            case 2: done = launch_tile<uint16_t>(src, dst, dims, ia); break;
            case 4: done = launch_tile<uint32_t>(src, dst, dims, ia); break;
            default: break;
        }
        if (done)
            return check_launch(who);
    }
#define CALL(T) launch_rows<T>(src, dst, dims, n)
    RL_BY_SIZE(es, CALL)
#undef CALL
    return check_launch(who);
}

}  // namespace mg

using namespace mg;

extern "C" TinyNNStatus megcc_gfx950_relayout(
        Tensor** inputs, int nr_input, Tensor** outputs, int nr_output, const Workspace*,
        const RuntimeOpt*) {
    TinyNNStatus st = check_io(inputs, nr_input, 1, 1, outputs, nr_output, "relayout");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor* s = inputs[0];
    const Tensor* d = outputs[0];
    MG_REQUIRE(s->dtype.type_enum == d->dtype.type_enum, TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "relayout: source dtype %d, destination dtype %d", (int)s->dtype.type_enum,
               (int)d->dtype.type_enum);
    MG_REQUIRE(s->layout.nr_dim >= 0 && s->layout.nr_dim <= MAX_DIM && d->layout.nr_dim >= 0 &&
                       d->layout.nr_dim <= MAX_DIM,
               TinyNN_ERROR_INVALID_LAYOUT, "relayout: bad number of dims");
    return strided_copy(s->ptr, s->layout, d->ptr, d->layout, dtype_size(s), "relayout");
}

extern "C" TinyNNStatus megcc_gfx950_concat(
        const int* axis_ptr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace*, const RuntimeOpt*) {
    MG_REQUIRE(axis_ptr, TinyNN_ERROR_NULL_PTR, "concat: NULL attr");
    TinyNNStatus st = check_io(inputs, nr_input, 1, 1 << 20, outputs, nr_output, "concat");
    if (st != TinyNN_SUCCESS)
        return st;
    const int axis = *axis_ptr;
    const Tensor* out = outputs[0];
    const Layout& ol = out->layout;
    MG_REQUIRE(ol.nr_dim >= 1 && ol.nr_dim <= MAX_DIM && axis >= 0 && axis < ol.nr_dim,
               TinyNN_ERROR_OUT_OF_RANGE, "concat: axis %d of a %d-d tensor", axis, ol.nr_dim);
    const size_t es = dtype_size(out);
    size_t along = 0;
    for (int i = 0; i < nr_input; ++i) {
        const Tensor* in = inputs[i];
        MG_REQUIRE(in->dtype.type_enum == out->dtype.type_enum, TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
                   "concat: input %d has dtype %d, output %d", i, (int)in->dtype.type_enum,
                   (int)out->dtype.type_enum);
        MG_REQUIRE(in->layout.nr_dim == ol.nr_dim, TinyNN_ERROR_INVALID_LAYOUT,
                   "concat: input %d has %d dims, output %d", i, in->layout.nr_dim, ol.nr_dim);
        for (int j = 0; j < ol.nr_dim; ++j)
            MG_REQUIRE(j == axis || in->layout.dims[j] == ol.dims[j], TinyNN_ERROR_INVALID_LAYOUT,
                       "concat: input %d dim %d is %u, output has %u", i, j, in->layout.dims[j],
                       ol.dims[j]);
        along += in->layout.dims[axis];
    }
    MG_REQUIRE(along == ol.dims[axis], TinyNN_ERROR_INVALID_LAYOUT,
               "concat: inputs add up to %zu along axis %d, output has %u", along, axis,
               ol.dims[axis]);
    size_t at = 0;
    for (int i = 0; i < nr_input; ++i) {
        const Tensor* in = inputs[i];
        Layout slice = ol;
        slice.dims[axis] = in->layout.dims[axis];
        char* p = (char*)out->ptr + (long long)at * ol.stride[axis] * (long long)es;
        st = strided_copy(in->ptr, in->layout, p, slice, es, "concat");
        if (st != TinyNN_SUCCESS)
            return st;
        at += in->layout.dims[axis];
    }
    return TinyNN_SUCCESS;
}
