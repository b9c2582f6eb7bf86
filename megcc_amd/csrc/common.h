// Shared host-side helpers of libmegcc_gfx950.so: error reporting, the library stream, Tensor
// inspection. Host code, plus the tile-order helper the tiled kernels share; the other device helpers live in epilogue.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "megcc_gfx950.h"

namespace mg {

// One stream for every launch and copy, default priority, created on first use.
hipStream_t stream();
// The library stream itself, whatever stream() currently answers.
hipStream_t main_stream();
// While `on`, stream() answers `s` on this thread: the model runtime launches the last operators of a
// forward on a second stream this way (model.cpp). The kernels' launch code is unchanged.
void set_stream_override(hipStream_t s, bool on);
// Streams megcc_gfx950_wait() synchronises besides the library stream.
void register_aux_stream(hipStream_t s);
void unregister_aux_stream(hipStream_t s);

// Compute units of the current device (256 when the query fails).
int num_cus();

// Records a message for megcc_gfx950_last_error() and returns `st`.
TinyNNStatus fail(TinyNNStatus st, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define MG_REQUIRE(cond, st, ...)          \
    do {                                   \
        if (!(cond))                       \
            return ::mg::fail(st, __VA_ARGS__); \
    } while (0)

// Tile order of a 2-D grid of gx x gy workgroups for the chip's eight XCDs. Workgroups are handed to
// the XCDs in turn (workgroup i runs on XCD i % 8) and every XCD has an L2 of its own, so with the
// plain order each XCD touches every row panel of one operand. Here workgroup i takes place
// (i % 8) * (gx * gy / 8) + i / 8 in an order that walks the grid in strips of `w` columns, row by
// row inside a strip: the eighth of the tiles one XCD owns is then a compact rectangle and each
// operand panel is fetched by the one or two XCDs that need it. w = 0 (or a tile count that is no
// multiple of 8) keeps the plain order. Any w >= 1 gives a bijection.
struct XcdOrder {
    int w;
};
inline XcdOrder make_xcd_order(int gx, int gy) {
    const long nb = (long)gx * gy;
    if (nb < 64 || (nb & 7) != 0)
        return {0};
    // w ~ sqrt(tiles per XCD / 2): the half of its share an XCD has resident at a time is about square
    // (a round of workgroups streams its panels through the 4 MB L2 once; the next round starts over)
    int w = 1;
    while ((long)w * w * 8 <= nb / 8)
        w *= 2;
    return {w < gx ? w : gx};
}
__device__ __forceinline__ void xcd_tile(XcdOrder o, int bx, int by, int gx, int gy, int& tx, int& ty) {
    tx = bx;
    ty = by;
    if (o.w == 0)
        return;
    const int nb = gx * gy, lb = by * gx + bx;
    const int place = (lb & 7) * (nb >> 3) + (lb >> 3);
    const int strip = place / (o.w * gy), rem = place - strip * (o.w * gy);
    const int w = min(o.w, gx - strip * o.w);
    ty = rem / w;
    tx = strip * o.w + rem - ty * w;
}

// Kernel-selection overrides: each one takes a kernel (or a variant of one) out of the dispatch so
// that the regression tests can reach the kernels that serve the shapes behind it. Read from the
// environment (MEGCC_NOPWS=1, ...) ONCE, when the library first consults them; later changes go
// through megcc_gfx950_set_option(). Nothing on a launch path scans the environment.
struct Options {
    bool no_pws, no_gevm, no_fcb, no_small, no_pm768, no_pm, no_dma512, no_pm256, no_dma, no_fcs, no_pwshare, no_hybrid, no_dot4, no_f32small, dw_generic, no_dwmfma, no_dwnchw, no_fuse_softmax, no_graph, no_poolrows, no_firstmfma, no_rowsplit, no_fuse_chain, no_fuse_pwdw, fuse_pwdw, no_fcone, no_xcdorder, no_affine, no_pipeline;
};
Options& options();

// Which kernel variant the most recent dispatch on this thread selected: `name` (a string literal)
// and up to five numbers that identify the instantiation; megcc_gfx950_last_kernel() formats them.
void note_kernel(const char* name, int a = -1, int b = -1, int c = -1, int d = -1, int e = -1);

// A kernel that requantises by the proven fused multiply-add (epilogue.h) says so after its
// note_kernel(): megcc_gfx950_last_kernel() then ends in "+affine".
void note_requant_affine(bool on);

// conv_api.hip: looks up the address of the static scratch array of
// megcc_gfx950_conv2d_noalloc on the current device (once per device; later calls return at once).
TinyNNStatus noalloc_scratch_setup();

// After a kernel launch: surfaces launch-configuration errors as TinyNN_ERROR_RUNTIME.
TinyNNStatus check_launch(const char* what);

// relayout.hip: copies `src` (layout sl) to `dst` (layout dl), elements of `es` bytes; one launch.
TinyNNStatus strided_copy(
        const void* src, const Layout& sl, void* dst, const Layout& dl, size_t es, const char* who);

inline size_t nr_elem(const Layout& l) {
    size_t n = 1;
    for (int i = 0; i < l.nr_dim; ++i)
        n *= l.dims[i];
    return n;
}

// Dense row-major strides (dims of extent 1 may carry any stride).
inline bool is_contiguous(const Layout& l) {
    long expect = 1;
    for (int i = l.nr_dim - 1; i >= 0; --i) {
        if (l.dims[i] != 1 && l.stride[i] != expect)
            return false;
        expect *= l.dims[i];
    }
    return true;
}

// Lowest and highest element offset a layout touches, relative to its first element; false when
// it has no elements.
inline bool view_span(const Layout& l, long long* lo, long long* hi) {
    *lo = *hi = 0;
    for (int i = 0; i < l.nr_dim; ++i) {
        if (l.dims[i] == 0)
            return false;
        const long long reach = (long long)(l.dims[i] - 1) * l.stride[i];
        (reach < 0 ? *lo : *hi) += reach;
    }
    return true;
}

inline bool is_q8(const Tensor* t) {
    return t->dtype.type_enum == TinyNN_QINT8 || t->dtype.type_enum == TinyNN_INT8;
}
inline bool is_q32(const Tensor* t) {
    return t->dtype.type_enum == TinyNN_QINT32 || t->dtype.type_enum == TinyNN_INT;
}
inline bool is_f32(const Tensor* t) {
    return t->dtype.type_enum == TinyNN_FLOAT;
}
inline size_t dtype_size(const Tensor* t) {
    switch (t->dtype.type_enum) {
        case TinyNN_FLOAT:
        case TinyNN_INT:
        case TinyNN_QINT32:
            return 4;
        case TinyNN_FLOAT16:
        case TinyNN_INT16:
            return 2;
        default:
            return 1;
    }
}

inline unsigned ceil_div(size_t a, size_t b) {
    return (unsigned)((a + b - 1) / b);
}

// NULL / pointer checks shared by every entry point (the reference kernels TINYNN_ASSERT these).
TinyNNStatus check_io(
        Tensor** inputs, int nr_input, int want_in_min, int want_in_max, Tensor** outputs,
        int nr_output, const char* who);

}  // namespace mg
