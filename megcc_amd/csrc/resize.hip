// f32 Resize: bilinear (NCHW, NCHW44) and nearest (NCHW, strided source).
// Reference: Common/Resize.h:16-40 (coordinates), :42-101 (LINEAR body), :158-175 (NEAREST),
// :209-225 (offsets); GeneralIntrinsic/Resize.cpp:13-33 and BareMetal/Resize.cpp:15-35 pick them.
//
// One thread per 4 neighbouring outputs of a row (NCHW, one 16-byte store) or per pixel of 4
// channels (NCHW44, 16-byte accesses); the work is one pass over the output with gathered reads
// that mostly hit cache, so the kernels are plain. The arithmetic keeps the reference's order -
// (idx + 0.5f) / scale - 0.5f, ((v * ah) * aw) summed left to right - and the library is built
// with -ffp-contract=off (no fused multiply-adds, every product and sum rounded), so the results
// are the reference's bit for bit, not only within the f32 tolerance.
#include "common.h"

namespace mg {
namespace {

struct ResizeArgs {
    const float* src;
    float* dst;
    int planes;  // N * C (NCHW44: N * C / 4)
    int IH, IW, OH, OW;
    float scale_h, scale_w;
    long long s_n, s_c, s_h, s_w;  // NEAREST: source strides in elements
    int C;
    unsigned items;   // work items of the launch
    int vec_store;    // NCHW: rows of the destination take 16-byte stores
};

__device__ __forceinline__ void resize_coord(float scale, int size, int idx, float& a0, int& i0, float& a1, int& i1) {
    if (size == 1) {
        a0 = 1.f; i0 = 0; a1 = 0.f; i1 = 0;
        return;
    }
    float alpha = __fsub_rn(__fdiv_rn(__fadd_rn((float)idx, 0.5f), scale), 0.5f);
    int origin = (int)floorf(alpha);
    alpha = __fsub_rn(alpha, (float)origin);
    if (origin < 0) {
        origin = 0;
        alpha = 0.f;
    } else if (origin + 1 >= size) {
        origin = size - 2;
        alpha = 1.f;
    }
    a0 = __fsub_rn(1.f, alpha); i0 = origin; a1 = alpha; i1 = origin + 1;
}

__device__ __forceinline__ float resize_mix(float v00, float v01, float v10, float v11, float ah0, float ah1, float aw0, float aw1) {
    const float t0 = __fmul_rn(__fmul_rn(v00, ah0), aw0);
    const float t1 = __fmul_rn(__fmul_rn(v01, ah0), aw1);
    const float t2 = __fmul_rn(__fmul_rn(v10, ah1), aw0);
    const float t3 = __fmul_rn(__fmul_rn(v11, ah1), aw1);
    return __fadd_rn(__fadd_rn(__fadd_rn(t0, t1), t2), t3);
}

// Work item of the NCHW kernels: 4 neighbouring outputs of one row (one 16-byte store when the
// rows allow it), so the row coordinates and the index arithmetic are paid once per 4 outputs.
__device__ __forceinline__ bool resize_item(const ResizeArgs& q, unsigned& plane, int& oh, int& ow0) {
    const unsigned groups = (unsigned)(q.OW + 3) >> 2;
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i >= q.items)
        return false;
    const unsigned t = i / groups;
    ow0 = (int)(i - t * groups) * 4;
    plane = t / (unsigned)q.OH;
    oh = (int)(t - plane * (unsigned)q.OH);
    return true;
}

__device__ __forceinline__ void resize_store4(const ResizeArgs& q, size_t at, int ow0, const float (&r)[4]) {
    if (q.vec_store) {
        *(float4*)(q.dst + at) = make_float4(r[0], r[1], r[2], r[3]);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (ow0 + j < q.OW)
                q.dst[at + j] = r[j];
    }
}

// TAB: the column coordinates (one correctly rounded division each) are computed once per
// workgroup into LDS instead of once per output; for rows longer than RESIZE_TAB every thread
// computes its own.
constexpr int RESIZE_TAB = 2048;

// PAIR: the source is at least 2 wide, so the right-hand column is always the left-hand one + 1
// (get_coord) and shares its address.
template <bool TAB, bool PAIR>
__global__ void __launch_bounds__(256) resize_linear_nchw_kernel(ResizeArgs q) {
    __shared__ float aw_tab[TAB ? RESIZE_TAB : 1];
    __shared__ int iw_tab[TAB ? RESIZE_TAB : 1];
    if (TAB) {
        for (int ow = threadIdx.x; ow < q.OW; ow += 256) {
            float aw0, aw1;
            int iw0, iw1;
            resize_coord(q.scale_w, q.IW, ow, aw0, iw0, aw1, iw1);
            aw_tab[ow] = aw1;
            iw_tab[ow] = iw0 | (iw1 - iw0) << 30;  // iw1 = iw0 + 1, or both 0 for a 1-wide source
        }
        __syncthreads();
    }
    unsigned plane;
    int oh, ow0;
    if (!resize_item(q, plane, oh, ow0))
        return;
    float ah0, ah1;
    int ih0, ih1;
    resize_coord(q.scale_h, q.IH, oh, ah0, ih0, ah1, ih1);
    const float* s = q.src + (size_t)plane * q.IH * q.IW;
    const int row0 = ih0 * q.IW, row1 = ih1 * q.IW;  // a plane has fewer than 2^31 elements
    float r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int ow = min(ow0 + j, q.OW - 1);
        float aw0, aw1;
        int iw0, iw1;
        if (TAB) {
            const int packed = iw_tab[ow];
            aw1 = aw_tab[ow];
            iw0 = packed & 0x3fffffff;
            iw1 = iw0 + (packed >> 30);
            // 1 - alpha as in get_coord; a 1-wide source has the weights (1, 0)
            aw0 = q.IW == 1 ? 1.f : __fsub_rn(1.f, aw1);
        } else {
            resize_coord(q.scale_w, q.IW, ow, aw0, iw0, aw1, iw1);
        }
        const float* p0 = s + (row0 + iw0);
        const float* p1 = s + (row1 + iw0);
        if (PAIR)
            r[j] = resize_mix(p0[0], p0[1], p1[0], p1[1], ah0, ah1, aw0, aw1);
        else
            r[j] = resize_mix(p0[0], p0[iw1 - iw0], p1[0], p1[iw1 - iw0], ah0, ah1, aw0, aw1);
    }
    resize_store4(q, ((size_t)plane * q.OH + oh) * q.OW + ow0, ow0, r);
}

// element = float4 = the 4 channels of a pixel
__global__ void __launch_bounds__(256) resize_linear_nchw44_kernel(ResizeArgs q) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i >= q.items)
        return;
    const unsigned t = i / (unsigned)q.OW;
    const int ow = (int)(i - t * (unsigned)q.OW);
    const unsigned plane = t / (unsigned)q.OH;
    const int oh = (int)(t - plane * (unsigned)q.OH);
    float ah0, ah1, aw0, aw1;
    int ih0, ih1, iw0, iw1;
    resize_coord(q.scale_h, q.IH, oh, ah0, ih0, ah1, ih1);
    resize_coord(q.scale_w, q.IW, ow, aw0, iw0, aw1, iw1);
    const float4* s4 = (const float4*)q.src + (size_t)plane * q.IH * q.IW;
    const float4 a = s4[ih0 * q.IW + iw0], b = s4[ih0 * q.IW + iw1];
    const float4 c = s4[ih1 * q.IW + iw0], d = s4[ih1 * q.IW + iw1];
    float4 r;
    r.x = resize_mix(a.x, b.x, c.x, d.x, ah0, ah1, aw0, aw1);
    r.y = resize_mix(a.y, b.y, c.y, d.y, ah0, ah1, aw0, aw1);
    r.z = resize_mix(a.z, b.z, c.z, d.z, ah0, ah1, aw0, aw1);
    r.w = resize_mix(a.w, b.w, c.w, d.w, ah0, ah1, aw0, aw1);
    ((float4*)q.dst)[i] = r;
}

__global__ void __launch_bounds__(256) resize_nearest_kernel(ResizeArgs q) {
    unsigned plane;
    int oh, ow0;
    if (!resize_item(q, plane, oh, ow0))
        return;
    const unsigned n = plane / (unsigned)q.C;
    const int c = (int)(plane - n * (unsigned)q.C);
    const int ih = min((int)__fdiv_rn((float)oh, q.scale_h), q.IH - 1);
    const float* row = q.src + (long long)n * q.s_n + c * q.s_c + ih * q.s_h;
    float r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int ow = min(ow0 + j, q.OW - 1);
        const int iw = min((int)__fdiv_rn((float)ow, q.scale_w), q.IW - 1);
        r[j] = row[iw * q.s_w];
    }
    resize_store4(q, ((size_t)plane * q.OH + oh) * q.OW + ow0, ow0, r);
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" TinyNNStatus megcc_gfx950_resize(
        const MegccResizeAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace*, const RuntimeOpt*) {
    MG_REQUIRE(attr, TinyNN_ERROR_NULL_PTR, "resize: NULL attr");
    // the operator carries its target shape as a second input; the kernels never read it
    TinyNNStatus st = check_io(inputs, nr_input, 1, 2, outputs, nr_output, "resize");
    if (st != TinyNN_SUCCESS)
        return st;
    const Tensor* s = inputs[0];
    const Tensor* d = outputs[0];
    MG_REQUIRE(is_f32(s) && is_f32(d), TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE, "resize: f32 only");
    const bool linear = attr->imode == MEGCC_IMODE_LINEAR;
    const bool p4 = attr->format == MEGCC_FMT_NCHW44;
    MG_REQUIRE(linear || attr->imode == MEGCC_IMODE_NEAREST, TinyNN_ERROR_OUT_OF_RANGE,
               "resize: imode %d", (int)attr->imode);
    MG_REQUIRE(attr->format == MEGCC_FMT_NCHW || (p4 && linear), TinyNN_ERROR_OUT_OF_RANGE,
               "resize: format %d with imode %d", (int)attr->format, (int)attr->imode);
    const Layout& sl = s->layout;
    const Layout& dl = d->layout;
    const int nd = p4 ? 5 : 4;
    MG_REQUIRE(sl.nr_dim == nd && dl.nr_dim == nd, TinyNN_ERROR_INVALID_LAYOUT,
               "resize: %d-d source, %d-d destination, want %d", sl.nr_dim, dl.nr_dim, nd);
    MG_REQUIRE(sl.dims[0] == dl.dims[0] && sl.dims[1] == dl.dims[1] &&
                       (!p4 || (sl.dims[4] == 4 && dl.dims[4] == 4)),
               TinyNN_ERROR_INVALID_LAYOUT, "resize: batch / channel extents differ");
    MG_REQUIRE(is_contiguous(dl) && (!linear || is_contiguous(sl)), TinyNN_ERROR_INVALID_LAYOUT,
               "resize: strided %s", is_contiguous(dl) ? "source of a LINEAR resize" : "destination");
    const size_t out_elems = nr_elem(dl);
    if (out_elems == 0)
        return TinyNN_SUCCESS;
    MG_REQUIRE(nr_elem(sl) > 0, TinyNN_ERROR_INVALID_LAYOUT, "resize: empty source");
    MG_REQUIRE(out_elems < (1ull << 40) && nr_elem(sl) < (1ull << 40), TinyNN_ERROR_OUT_OF_RANGE,
               "resize: tensor too large");
    ResizeArgs q = {};
    q.src = (const float*)s->ptr;
    q.dst = (float*)d->ptr;
    q.C = (int)sl.dims[1];
    q.planes = (int)(sl.dims[0] * sl.dims[1]);
    q.IH = (int)sl.dims[2]; q.IW = (int)sl.dims[3];
    q.OH = (int)dl.dims[2]; q.OW = (int)dl.dims[3];
    q.scale_h = (float)q.OH / q.IH;
    q.scale_w = (float)q.OW / q.IW;
    // work items: a pixel of 4 channels (NCHW44) or 4 neighbouring outputs of a row (NCHW)
    const size_t items = p4 ? out_elems / 4 : (size_t)q.planes * q.OH * (((size_t)q.OW + 3) / 4);
    MG_REQUIRE(items < (1ull << 31) && nr_elem(sl) < (1ull << 31) * (p4 ? 4 : 1),
               TinyNN_ERROR_OUT_OF_RANGE, "resize: tensor too large");
    q.items = (unsigned)items;
    q.vec_store = !p4 && (q.OW & 3) == 0 && ((uintptr_t)q.dst & 15) == 0;
    const dim3 grid((unsigned)((items + 255) / 256));
    if (linear) {
        if (p4) {
            MG_REQUIRE(((uintptr_t)q.src & 15) == 0 && ((uintptr_t)q.dst & 15) == 0,
                       TinyNN_ERROR_INVALID_LAYOUT, "resize: NCHW44 tensors must be 16-byte aligned");
            hipLaunchKernelGGL(resize_linear_nchw44_kernel, grid, dim3(256), 0, stream(), q);
        } else {
            const bool tab = q.OW <= RESIZE_TAB, pair = q.IW >= 2;
            const void* kern = tab ? (pair ? (const void*)resize_linear_nchw_kernel<true, true>
                                           : (const void*)resize_linear_nchw_kernel<true, false>)
                                   : (pair ? (const void*)resize_linear_nchw_kernel<false, true>
                                           : (const void*)resize_linear_nchw_kernel<false, false>);
            void* args[] = {&q};
            MG_REQUIRE(hipLaunchKernel(kern, grid, dim3(256), args, 0, stream()) == hipSuccess,
                       TinyNN_ERROR_RUNTIME, "resize: launch failed");
        }
    } else {
        long long lo, hi;
        MG_REQUIRE(view_span(sl, &lo, &hi), TinyNN_ERROR_INVALID_LAYOUT, "resize: bad source strides");
        q.s_n = sl.stride[0]; q.s_c = sl.stride[1]; q.s_h = sl.stride[2]; q.s_w = sl.stride[3];
        hipLaunchKernelGGL(resize_nearest_kernel, grid, dim3(256), 0, stream(), q);
    }
    return check_launch("resize");
}
