// qsi8 pooling, bandwidth-bound, no MFMA.
//   NCHW   : BareMetal::PoolingKernel (BareMetal/Pooling.cpp:84-148,219-245): MAX of the in-bounds
//            taps starting from -128; AVERAGE roundf((float)sum / (wh*ww)); COUNT_EXCLUDE_PADDING
//            roundf((float)sum / count); stored without clamp.
//   NCHW44 : GeneralIntrinsic::PoolingNchw44QInt8 (GeneralIntrinsic/PoolingKernel/
//            QInt8PoolingNCHW44.cpp:34-113): AVERAGE is saturate(round((float)sum * count_div)) with
//            `float count_div = 1.0 / window_count` (a double quotient rounded to float).
// NCHW44: one thread per output dword (4 channels of a pixel), lanes walk W -> coalesced dwords.
// NCHW  : four outputs of a row per thread for the common windows, else one thread per output byte.
#include "common.h"
#include "epilogue.h"
#include "fastdiv.h"

namespace mg {

struct PoolGeom {
    int n, c, ih, iw, oh, ow;
    int wh, ww, sh, sw, ph, pw;
    int mode;
    float count_div;  // 1.0 / (wh*ww) rounded to float, for NCHW44 AVERAGE
};

__global__ void __launch_bounds__(256) pool44_q8_kernel(
        PoolGeom g, const uint32_t* __restrict__ src, uint32_t* __restrict__ dst) {
    const int c4n = g.c >> 2;
    const size_t total = (size_t)g.n * c4n * g.oh * g.ow;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i;
        int ow = r % g.ow; r /= g.ow;
        int oh = r % g.oh; r /= g.oh;
        const uint32_t* plane = src + r * g.ih * g.iw;
        int mx[4] = {-128, -128, -128, -128};
        int sum[4] = {0, 0, 0, 0};
        int count = 0;
        for (int fh = 0; fh < g.wh; ++fh) {
            unsigned ih = (unsigned)(oh * g.sh + fh - g.ph);
            if (ih >= (unsigned)g.ih)
                continue;
            for (int fw = 0; fw < g.ww; ++fw) {
                unsigned iw = (unsigned)(ow * g.sw + fw - g.pw);
                if (iw >= (unsigned)g.iw)
                    continue;
                uint32_t v = plane[ih * g.iw + iw];
                ++count;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    int b = sbyte(v, c);
                    mx[c] = max(mx[c], b);
                    sum[c] += b;
                }
            }
        }
        int o[4];
        if (g.mode == MEGCC_POOL_MAX) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                o[c] = mx[c];
        } else {
            float div = g.mode == MEGCC_POOL_AVERAGE ? g.count_div : (float)(1.0 / (double)(uint32_t)count);
#pragma unroll
            for (int c = 0; c < 4; ++c)
                o[c] = fp32_to_int8((float)sum[c] * div);
        }
        dst[i] = pack4(o[0], o[1], o[2], o[3]);
    }
}

// NCHW44, square windows of the common widths and strides, rows a multiple of 4 pixels: a thread
// makes 4 neighbouring output pixels of a row = one 16-byte store. Their windows cover 3 * SW + WW
// input pixels of each window row, fetched as the aligned 16-byte groups of 4 pixels that contain
// them (a third of the loads of one dword per tap, and neighbouring lanes 32 or 16 bytes apart
// instead of every lane on its own stretch; with a row length that is a multiple of 4 a group lies
// inside the row or outside, so the left / right padding is a group that is not loaded). A
// pixel's 4 channel bytes are split into even and odd bytes as packed 16-bit halves, the window
// rows are combined column by column with packed max / add, then the WW columns of each output,
// and one v_perm puts the bytes back together (MAX). PW: the horizontal padding, which fixes where
// the span starts inside its first group.
typedef short pool44_s2 __attribute__((ext_vector_type(2)));
typedef unsigned pool44_v4u __attribute__((ext_vector_type(4)));

template <int WW, int SW, int PW, bool IS_MAX>
__global__ void __launch_bounds__(256) pool44_rows_kernel(
        PoolGeom g, const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, unsigned total, int owg,
        FastDiv d_owg, FastDiv d_oh, int vec_store) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;  // (plane set, oh, group of 4 ow)
    if (i >= total)
        return;
    const unsigned row = fdiv(i, d_owg), q = i - row * (unsigned)owg;
    const unsigned plane = fdiv(row, d_oh), oh = row - plane * (unsigned)g.oh;
    const int ow0 = (int)q * 4;
    const int nvalid = min(4, g.ow - ow0);
    constexpr int SPAN = 3 * SW + WW;
    constexpr int SH = (4 - (PW & 3)) & 3;     // span pixel 0 inside its group of 4
    constexpr int NCH = (SH + SPAN + 3) / 4;   // groups of 4 pixels per window row
    const int s = ow0 * SW - PW;               // input column of span pixel 0
    const int c0 = s - SH;                     // first column of the first group (a multiple of 4)
    const uint32_t* const in_plane = src + (size_t)plane * g.ih * g.iw;
    const short init = IS_MAX ? -128 : 0;
    const unsigned neutral = IS_MAX ? 0x80808080u : 0u;
    int rows = 0;
    uint32_t d[WW][NCH * 4];
#pragma unroll
    for (int fh = 0; fh < WW; ++fh) {
        const unsigned ih = (unsigned)((int)oh * g.sh + fh - g.ph);
        const bool row_ok = ih < (unsigned)g.ih;
        rows += row_ok ? 1 : 0;
        const uint32_t* in_row = in_plane + (size_t)(row_ok ? ih : 0u) * g.iw;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const bool ok = row_ok && (unsigned)(c0 + 4 * c) < (unsigned)g.iw;
            pool44_v4u v = {neutral, neutral, neutral, neutral};
            if (ok)
                v = *(const pool44_v4u*)(in_row + c0 + 4 * c);
            d[fh][4 * c] = v.x;
            d[fh][4 * c + 1] = v.y;
            d[fh][4 * c + 2] = v.z;
            d[fh][4 * c + 3] = v.w;
        }
    }
    pool44_s2 ev[SPAN], od[SPAN];  // channels 0 / 2 and 1 / 3 of each span column, combined over the rows
#pragma unroll
    for (int j = 0; j < SPAN; ++j)
        ev[j] = od[j] = pool44_s2{init, init};
#pragma unroll
    for (int fh = 0; fh < WW; ++fh)
#pragma unroll
        for (int j = 0; j < SPAN; ++j) {
            const pool44_s2 w = __builtin_bit_cast(pool44_s2, d[fh][j + SH]);
            const pool44_s2 e = (w << 8) >> 8, odd = w >> 8;
            ev[j] = IS_MAX ? __builtin_elementwise_max(ev[j], e) : ev[j] + e;
            od[j] = IS_MAX ? __builtin_elementwise_max(od[j], odd) : od[j] + odd;
        }
    uint32_t out[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        pool44_s2 e = ev[k * SW], o = od[k * SW];
#pragma unroll
        for (int fw = 1; fw < WW; ++fw) {
            e = IS_MAX ? __builtin_elementwise_max(e, ev[k * SW + fw]) : e + ev[k * SW + fw];
            o = IS_MAX ? __builtin_elementwise_max(o, od[k * SW + fw]) : o + od[k * SW + fw];
        }
        if (IS_MAX) {
            // bytes: e.lo, o.lo, e.hi, o.hi
            out[k] = __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, o), __builtin_bit_cast(unsigned, e), 0x06020400u);
        } else {
            float div = g.count_div;
            if (g.mode != MEGCC_POOL_AVERAGE) {
                const int x0 = s + k * SW;
                const int cols = min(g.iw, x0 + WW) - max(0, x0);
                div = (float)(1.0 / (double)(uint32_t)max(rows * cols, 1));
            }
            out[k] = pack4(fp32_to_int8((float)(int)e[0] * div), fp32_to_int8((float)(int)o[0] * div),
                           fp32_to_int8((float)(int)e[1] * div), fp32_to_int8((float)(int)o[1] * div));
        }
    }
    uint32_t* o = dst + ((size_t)plane * g.oh + oh) * g.ow + ow0;
    if (vec_store && nvalid == 4) {
        *(pool44_v4u*)o = pool44_v4u{out[0], out[1], out[2], out[3]};
    } else {
        for (int k = 0; k < nvalid; ++k)
            o[k] = out[k];
    }
}

// NCHW44, one output pixel per plane (global pooling, e.g. the 7x7 average in front of a
// classifier): 8 lanes per plane group instead of one thread, so that a wave reads 8 consecutive
// planes as one contiguous stretch; integer max / sum are combined across the 8 lanes, the last
// step is the same expression as above.
__global__ void __launch_bounds__(256) pool44_global_q8_kernel(
        PoolGeom g, const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, int planes) {
    const int sub = threadIdx.x & 7;
    const int hw = g.ih * g.iw;
    const bool is_max = g.mode == MEGCC_POOL_MAX;
    for (int pl = (blockIdx.x * 256 + threadIdx.x) >> 3; pl < planes; pl += gridDim.x * 32) {
        const uint32_t* plane = src + (size_t)pl * hw;
        int v4[4] = {is_max ? -128 : 0, is_max ? -128 : 0, is_max ? -128 : 0, is_max ? -128 : 0};
        for (int i = sub; i < hw; i += 8) {
            const uint32_t v = plane[i];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int b = sbyte(v, c);
                v4[c] = is_max ? max(v4[c], b) : v4[c] + b;
            }
        }
#pragma unroll
        for (int off = 4; off > 0; off >>= 1) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int o = __shfl_xor(v4[c], off, 64);
                v4[c] = is_max ? max(v4[c], o) : v4[c] + o;
            }
        }
        if (sub == 0) {
            int o[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (is_max)
                    o[c] = v4[c];
                else if (g.mode == MEGCC_POOL_AVERAGE)
                    o[c] = fp32_to_int8((float)v4[c] * g.count_div);
                else
                    o[c] = fp32_to_int8((float)v4[c] * (float)(1.0 / (double)(uint32_t)hw));
            }
            dst[pl] = pack4(o[0], o[1], o[2], o[3]);
        }
    }
}

__global__ void __launch_bounds__(256) pool_nchw_q8_kernel(
        PoolGeom g, const int8_t* __restrict__ src, int8_t* __restrict__ dst) {
    const size_t total = (size_t)g.n * g.c * g.oh * g.ow;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i;
        int ow = r % g.ow; r /= g.ow;
        int oh = r % g.oh; r /= g.oh;
        const int8_t* plane = src + r * g.ih * g.iw;
        int mx = -128, sum = 0, count = 0;
        for (int fh = 0; fh < g.wh; ++fh) {
            unsigned ih = (unsigned)(oh * g.sh + fh - g.ph);
            if (ih >= (unsigned)g.ih)
                continue;
            for (int fw = 0; fw < g.ww; ++fw) {
                unsigned iw = (unsigned)(ow * g.sw + fw - g.pw);
                if (iw >= (unsigned)g.iw)
                    continue;
                int b = plane[ih * g.iw + iw];
                mx = max(mx, b);
                sum += b;
                ++count;
            }
        }
        int o;
        if (g.mode == MEGCC_POOL_MAX)
            o = mx;
        else if (g.mode == MEGCC_POOL_AVERAGE)
            o = (int)roundf((float)sum / (float)(g.wh * g.ww));
        else
            o = (int)roundf((float)sum / (float)count);
        dst[i] = (int8_t)o;
    }
}

// NCHW, any mode, square windows of the common widths and strides: a thread makes 4 neighbouring
// outputs of a row. Their windows cover 3 * SW + WW consecutive bytes of each input row, which are
// fetched as the aligned dwords that contain them (only dwords that hold at least one byte of the
// row: an aligned dword with a byte of the tensor in it lies inside the tensor's page) and shifted
// into place with v_alignbyte; bytes left or right of the row (padding, outputs beyond the row's
// end) are replaced by the neutral value through a per-thread byte mask, so that there is ONE code
// path and no divergence at the borders. The window ROWS are combined first, on whole dwords: a
// dword of 4 signed bytes is split into its even and its odd bytes as packed 16-bit halves (as in
// max4_bytes below) and the rows meet in packed max / add (a column sum of up to 255 bytes fits 16
// bits); only then the WW columns of each output are picked out of the combined row at
// compile-time positions. All loads of a thread are in flight together.
typedef short pool_s2 __attribute__((ext_vector_type(2)));

template <int WW, int SW, bool IS_MAX>
__global__ void __launch_bounds__(256) pool_nchw_rows_kernel(
        PoolGeom g, const int8_t* __restrict__ src, int8_t* __restrict__ dst, unsigned total, int owg,
        FastDiv d_owg, FastDiv d_oh, int dword_store) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;  // (plane, oh, group of 4 ow)
    if (i >= total)
        return;
    const unsigned row = fdiv(i, d_owg), q = i - row * (unsigned)owg;
    const unsigned plane = fdiv(row, d_oh), oh = row - plane * (unsigned)g.oh;
    const int ow0 = (int)q * 4;
    const int nvalid = min(4, g.ow - ow0);
    constexpr int SPAN = 3 * SW + WW;
    constexpr int NA = (SPAN + 3) / 4;  // dwords of the shifted span
    const int s = ow0 * SW - g.pw;      // input column of span byte 0
    // span bytes lo .. hi - 1 lie inside the row
    const int lo = max(0, -s), hi = min(SPAN, g.iw - s);
    unsigned keep[NA];  // 0xff for every byte of span dword k that lies inside the row
#pragma unroll
    for (int k = 0; k < NA; ++k) {
        const int b0 = min(max(lo - 4 * k, 0), 4), b1 = min(max(hi - 4 * k, 0), 4);
        const unsigned below1 = b1 >= 4 ? 0xffffffffu : (1u << (8 * b1)) - 1u;
        const unsigned below0 = b0 >= 4 ? 0xffffffffu : (1u << (8 * b0)) - 1u;
        keep[k] = below1 & ~below0;
    }
    const int8_t* const in_plane = src + (size_t)plane * g.ih * g.iw;
    const unsigned neutral = IS_MAX ? 0x80808080u : 0u;
    int rows = 0;
    uint32_t d[WW][NA + 1];
    unsigned shift[WW];
    bool row_ok[WW];
#pragma unroll
    for (int fh = 0; fh < WW; ++fh) {
        const unsigned ih = (unsigned)((int)oh * g.sh + fh - g.ph);
        row_ok[fh] = ih < (unsigned)g.ih && hi > lo;
        rows += ih < (unsigned)g.ih ? 1 : 0;
        const int8_t* a = in_plane + (ptrdiff_t)(row_ok[fh] ? ih : 0u) * g.iw + s;
        const int sh = (int)((uintptr_t)a & 3u);
        shift[fh] = (unsigned)sh;
        const uint32_t* p0 = (const uint32_t*)(a - sh);
        // loaded dword k holds span bytes 4k - sh .. 4k - sh + 3
#pragma unroll
        for (int k = 0; k <= NA; ++k)
            d[fh][k] = row_ok[fh] && 4 * k - sh + 3 >= lo && 4 * k - sh < hi ? p0[k] : 0u;
    }
    pool_s2 ev[NA], od[NA];  // bytes 0 / 2 and 1 / 3 of each span dword, combined over the rows
    const short init = IS_MAX ? -128 : 0;
#pragma unroll
    for (int k = 0; k < NA; ++k)
        ev[k] = od[k] = pool_s2{init, init};
#pragma unroll
    for (int fh = 0; fh < WW; ++fh) {
        if (!row_ok[fh])
            continue;
#pragma unroll
        for (int k = 0; k < NA; ++k) {
            unsigned v = __builtin_amdgcn_alignbyte(d[fh][k + 1], d[fh][k], shift[fh]);
            v = (v & keep[k]) | (neutral & ~keep[k]);
            const pool_s2 w = __builtin_bit_cast(pool_s2, v);
            const pool_s2 e = (w << 8) >> 8, odd = w >> 8;
            ev[k] = IS_MAX ? __builtin_elementwise_max(ev[k], e) : ev[k] + e;
            od[k] = IS_MAX ? __builtin_elementwise_max(od[k], odd) : od[k] + odd;
        }
    }
    int o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        int acc = IS_MAX ? -128 : 0;
#pragma unroll
        for (int fw = 0; fw < WW; ++fw) {
            const int j = k * SW + fw;  // byte of the span
            const int v = (j & 1) ? (int)od[j >> 2][(j >> 1) & 1] : (int)ev[j >> 2][(j >> 1) & 1];
            acc = IS_MAX ? max(acc, v) : acc + v;
        }
        if (IS_MAX) {
            o[k] = acc;
        } else if (g.mode == MEGCC_POOL_AVERAGE) {
            o[k] = (int)roundf((float)acc / (float)(g.wh * g.ww));
        } else {
            // taps inside the image: `rows` window rows x the window columns inside the row
            const int c0 = s + k * SW;
            const int cols = min(g.iw, c0 + WW) - max(0, c0);
            o[k] = (int)roundf((float)acc / (float)(rows * cols));
        }
    }
    int8_t* out = dst + ((size_t)plane * g.oh + oh) * g.ow + ow0;
    if (dword_store && nvalid == 4) {
        *(uint32_t*)out = pack4(o[0], o[1], o[2], o[3]);
    } else {
        for (int k = 0; k < nvalid; ++k)
            out[k] = (int8_t)o[k];
    }
}

// MAX 2x2 stride 2 without padding on NCHW (kernel_pooling_MAX_NCHW_p0x0_s2x2_w2x2_qsi8qsi8): a
// thread makes 4 neighbouring outputs of a row = one dword, from 8 bytes of each of the two input
// rows (two 8-byte loads instead of 16 single bytes). Needs IW % 8 == 0 and aligned tensors.
__global__ void __launch_bounds__(256) pool_nchw_max2x2_kernel(
        const uint2* __restrict__ src, uint32_t* __restrict__ dst, unsigned total, int oh_n, int ow4) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;  // (plane, oh, group of 4 ow)
    if (i >= total)
        return;
    const unsigned row = i / (unsigned)ow4, q = i - row * (unsigned)ow4;
    const unsigned plane = row / (unsigned)oh_n, oh = row - plane * (unsigned)oh_n;
    // input row = ow4 groups of 8 bytes; rows 2 oh and 2 oh + 1 of the plane
    const size_t in = ((size_t)plane * oh_n * 2 + oh * 2) * ow4 + q;
    const uint2 a = src[in], b = src[in + ow4];
    int o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t wa = k < 2 ? a.x : a.y, wb = k < 2 ? b.x : b.y;
        const int c = (k & 1) * 2;
        o[k] = max(max(sbyte(wa, c), sbyte(wa, c + 1)), max(sbyte(wb, c), sbyte(wb, c + 1)));
    }
    dst[i] = pack4(o[0], o[1], o[2], o[3]);
}

// MAX 2x2 stride 2 without padding on NCHW44 (the pooling of the depthwise -> pool -> add chain):
// a thread makes 4 neighbouring output pixels = one 16-byte store from 8 input pixels of each of
// the two input rows (four 16-byte loads). The maximum per channel byte is taken on packed 16-bit
// halves: a dword of 4 signed bytes is split into its even bytes (shift left, arithmetic shift
// right, both packed) and its odd bytes (arithmetic shift right), the four window positions meet
// in v_pk_max_i16, and one v_perm puts the low bytes of the two results back together:
// 20 vector instructions per output dword instead of 40 byte extractions and maxima, and no
// division in the index arithmetic beyond two by run-time constants. Needs IW % 8 == 0.
typedef unsigned pool_v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned max4_bytes(unsigned a, unsigned b, unsigned c, unsigned d) {
    auto even = [](unsigned v) { return (__builtin_bit_cast(pool_s2, v) << 8) >> 8; };
    auto odd = [](unsigned v) { return __builtin_bit_cast(pool_s2, v) >> 8; };
    const pool_s2 e = __builtin_elementwise_max(__builtin_elementwise_max(even(a), even(b)),
                                                __builtin_elementwise_max(even(c), even(d)));
    const pool_s2 o = __builtin_elementwise_max(__builtin_elementwise_max(odd(a), odd(b)),
                                                __builtin_elementwise_max(odd(c), odd(d)));
    // bytes: e.lo, o.lo, e.hi, o.hi
    return __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, o), __builtin_bit_cast(unsigned, e), 0x06020400u);
}

__global__ void __launch_bounds__(256) pool44_max2x2_kernel(
        const pool_v4u* __restrict__ src, pool_v4u* __restrict__ dst, unsigned total, FastDiv d_ow4,
        int ow4) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;  // (plane set, oh, group of 4 ow)
    if (i >= total)
        return;
    const unsigned row = fdiv(i, d_ow4), q = i - row * (unsigned)ow4;
    // an input row is 2 * ow4 16-byte words; output row `row` (over all plane sets: IH = 2 * OH)
    // reads input rows 2 * row and 2 * row + 1
    const size_t in = (size_t)row * 4 * ow4 + 2 * q;
    const pool_v4u a0 = src[in], a1 = src[in + 1], b0 = src[in + 2 * ow4], b1 = src[in + 2 * ow4 + 1];
    pool_v4u o;
    o[0] = max4_bytes(a0[0], a0[1], b0[0], b0[1]);
    o[1] = max4_bytes(a0[2], a0[3], b0[2], b0[3]);
    o[2] = max4_bytes(a1[0], a1[1], b1[0], b1[1]);
    o[3] = max4_bytes(a1[2], a1[3], b1[2], b1[3]);
    dst[i] = o;
}

}  // namespace mg

using namespace mg;

extern "C" TinyNNStatus megcc_gfx950_pooling(
        const MegccPoolAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace*, const RuntimeOpt*) {
    MG_REQUIRE(attr, TinyNN_ERROR_NULL_PTR, "pooling: NULL attr");
    TinyNNStatus st = check_io(inputs, nr_input, 1, 1, outputs, nr_output, "pooling");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor* src = inputs[0];
    const Tensor* dst = outputs[0];
    MG_REQUIRE(is_q8(src) && is_q8(dst), TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "pooling: only qsi8 -> qsi8 is implemented");
    // "quant pooling only support same scale" (BareMetal/Pooling.cpp:22-27)
    MG_REQUIRE(src->dtype.param.scale == dst->dtype.param.scale, TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "pooling: source and destination scales differ");
    const bool f44 = attr->format == MEGCC_FMT_NCHW44;
    MG_REQUIRE(f44 || attr->format == MEGCC_FMT_NCHW, TinyNN_ERROR_NO_IMPLEMENT,
               "pooling: format %d", (int)attr->format);
    const int want_dim = f44 ? 5 : 4;
    MG_REQUIRE(src->layout.nr_dim == want_dim && dst->layout.nr_dim == want_dim &&
                       is_contiguous(src->layout) && is_contiguous(dst->layout),
               TinyNN_ERROR_INVALID_LAYOUT, "pooling: expects contiguous %d-d tensors", want_dim);
    PoolGeom g;
    g.n = src->layout.dims[0];
    g.c = src->layout.dims[1] * (f44 ? 4 : 1);
    g.ih = src->layout.dims[2];
    g.iw = src->layout.dims[3];
    g.oh = dst->layout.dims[2];
    g.ow = dst->layout.dims[3];
    g.wh = attr->window_h; g.ww = attr->window_w;
    g.sh = attr->stride_h; g.sw = attr->stride_w;
    g.ph = attr->pad_h; g.pw = attr->pad_w;
    g.mode = attr->mode;
    MG_REQUIRE(g.wh > 0 && g.ww > 0 && g.sh > 0 && g.sw > 0, TinyNN_ERROR_OUT_OF_RANGE,
               "pooling: empty window or stride");
    MG_REQUIRE(dst->layout.dims[0] == (uint32_t)g.n && dst->layout.dims[1] == src->layout.dims[1] &&
                       g.oh == (g.ih + 2 * g.ph - g.wh) / g.sh + 1 &&
                       g.ow == (g.iw + 2 * g.pw - g.ww) / g.sw + 1,
               TinyNN_ERROR_INVALID_LAYOUT, "pooling: destination shape does not match");
    g.count_div = (float)(1.0 / (double)(uint32_t)(g.wh * g.ww));
    size_t total = (size_t)g.n * g.c * g.oh * g.ow;
    if (total == 0)
        return TinyNN_SUCCESS;
    if (f44) {
        MG_REQUIRE(((uintptr_t)src->ptr & 3) == 0 && ((uintptr_t)dst->ptr & 3) == 0,
                   TinyNN_ERROR_INVALID_LAYOUT, "pooling: NCHW44 tensors must be 4-byte aligned");
        const long planes = (long)g.n * (g.c / 4);
        if (g.oh == 1 && g.ow == 1 && g.ph == 0 && g.pw == 0 && g.wh == g.ih && g.ww == g.iw &&
            g.ih * g.iw >= 16 && planes < (1L << 30)) {
            unsigned blocks = min(ceil_div((size_t)planes, 32), 1u << 16);
            hipLaunchKernelGGL(pool44_global_q8_kernel, dim3(blocks), dim3(256), 0, stream(), g,
                               (const uint32_t*)src->ptr, (uint32_t*)dst->ptr, (int)planes);
            return check_launch("pooling");
        }
        if (g.mode == MEGCC_POOL_MAX && g.wh == 2 && g.ww == 2 && g.sh == 2 && g.sw == 2 && g.ph == 0 &&
            g.pw == 0 && (g.iw & 7) == 0 && (g.ih & 1) == 0 && ((uintptr_t)src->ptr & 15) == 0 &&
            ((uintptr_t)dst->ptr & 15) == 0 && total / 16 < (1ull << 31)) {
            const unsigned items = (unsigned)(total / 16);  // 4 pixels x 4 channels each
            hipLaunchKernelGGL(pool44_max2x2_kernel, dim3((items + 255) / 256), dim3(256), 0, stream(),
                               (const pool_v4u*)src->ptr, (pool_v4u*)dst->ptr, items,
                               make_fastdiv(g.ow / 4), g.ow / 4);
            note_kernel("pool44_max2x2");
            return check_launch("pooling");
        }
        {
            // four output pixels of a row per thread for the common window widths and strides
            const int owg = (g.ow + 3) / 4;
            const size_t items = (size_t)planes * g.oh * owg;
            void (*rk)(PoolGeom, const uint32_t*, uint32_t*, unsigned, int, FastDiv, FastDiv, int) = nullptr;
            const bool mx = g.mode == MEGCC_POOL_MAX;
#define MG_POOL44_ROWS(W_, S_)                                                                        \
    (g.pw == 0   ? (mx ? pool44_rows_kernel<W_, S_, 0, true> : pool44_rows_kernel<W_, S_, 0, false>)     \
     : g.pw == 1 ? (mx ? pool44_rows_kernel<W_, S_, 1, true> : pool44_rows_kernel<W_, S_, 1, false>)     \
                 : nullptr)
            if (g.ww == 3 && g.sw == 2)
                rk = MG_POOL44_ROWS(3, 2);
            else if (g.ww == 2 && g.sw == 2)
                rk = MG_POOL44_ROWS(2, 2);
            else if (g.ww == 3 && g.sw == 1)
                rk = MG_POOL44_ROWS(3, 1);
            else if (g.ww == 2 && g.sw == 1)
                rk = MG_POOL44_ROWS(2, 1);
#undef MG_POOL44_ROWS
            if (rk && !options().no_poolrows && g.wh == g.ww && g.ow >= 4 && (g.iw & 3) == 0 &&
                ((uintptr_t)src->ptr & 15) == 0 && items < (1ull << 31) &&
                (size_t)planes * g.oh < (1ull << 31)) {
                const int vec_store = ((uintptr_t)dst->ptr & 15) == 0 && (g.ow & 3) == 0;
                hipLaunchKernelGGL(rk, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream(), g,
                                   (const uint32_t*)src->ptr, (uint32_t*)dst->ptr, (unsigned)items, owg,
                                   make_fastdiv(owg), make_fastdiv(g.oh), vec_store);
                note_kernel("pool44_rows", g.ww, g.sw);
                return check_launch("pooling");
            }
        }
        unsigned blocks = min(ceil_div(total / 4, 256), 1u << 20);
        hipLaunchKernelGGL(pool44_q8_kernel, dim3(blocks), dim3(256), 0, stream(), g,
                           (const uint32_t*)src->ptr, (uint32_t*)dst->ptr);
    } else if (g.mode == MEGCC_POOL_MAX && g.wh == 2 && g.ww == 2 && g.sh == 2 && g.sw == 2 && g.ph == 0 &&
               g.pw == 0 && (g.iw & 7) == 0 && (g.ih & 1) == 0 && ((uintptr_t)src->ptr & 7) == 0 &&
               ((uintptr_t)dst->ptr & 3) == 0 && total / 4 < (1ull << 32)) {
        const unsigned items = (unsigned)(total / 4);
        hipLaunchKernelGGL(pool_nchw_max2x2_kernel, dim3((items + 255) / 256), dim3(256), 0, stream(),
                           (const uint2*)src->ptr, (uint32_t*)dst->ptr, items, g.oh, g.ow / 4);
    } else {
        // four outputs of a row per thread for the common window widths and strides
        const int owg = (g.ow + 3) / 4;
        const size_t items = (size_t)g.n * g.c * g.oh * owg;
        void (*rows_kernel)(PoolGeom, const int8_t*, int8_t*, unsigned, int, FastDiv, FastDiv, int) = nullptr;
        const bool mx = g.mode == MEGCC_POOL_MAX;
#define MG_POOL_ROWS(W_, S_) (mx ? pool_nchw_rows_kernel<W_, S_, true> : pool_nchw_rows_kernel<W_, S_, false>)
        if (g.ww == 3 && g.sw == 2)
            rows_kernel = MG_POOL_ROWS(3, 2);
        else if (g.ww == 2 && g.sw == 2)
            rows_kernel = MG_POOL_ROWS(2, 2);
        else if (g.ww == 3 && g.sw == 1)
            rows_kernel = MG_POOL_ROWS(3, 1);
        else if (g.ww == 2 && g.sw == 1)
            rows_kernel = MG_POOL_ROWS(2, 1);
        else if (g.ww == 5 && g.sw == 1)
            rows_kernel = MG_POOL_ROWS(5, 1);
#undef MG_POOL_ROWS
        if (rows_kernel && !options().no_poolrows && g.ow >= 8 && g.wh == g.ww && items < (1ull << 31) && (size_t)g.n * g.c * g.oh < (1ull << 31)) {
            const int dword_store = ((uintptr_t)dst->ptr & 3) == 0 && (g.ow & 3) == 0;
            hipLaunchKernelGGL(rows_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream(), g,
                               (const int8_t*)src->ptr, (int8_t*)dst->ptr, (unsigned)items, owg,
                               make_fastdiv(owg), make_fastdiv(g.oh), dword_store);
            note_kernel("pool_nchw_rows", g.ww, g.sw);
            return check_launch("pooling");
        }
        unsigned blocks = min(ceil_div(total, 256), 1u << 20);
        hipLaunchKernelGGL(pool_nchw_q8_kernel, dim3(blocks), dim3(256), 0, stream(), g,
                           (const int8_t*)src->ptr, (int8_t*)dst->ptr);
    }
    return check_launch("pooling");
}
