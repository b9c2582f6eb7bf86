// ConvBias entry points: derive the geometry from the Tensor layouts exactly as the reference's
// generated kernel does at run time (BareMetal/ConvKernel.cpp:262-287), validate what that kernel
// would TINYNN_ASSERT, and route to the kernel for the case:
//   qsi8 NCHW44 DENSE, qsi8 FullyConnected (1x1 NCHW on [M,K,1,1])  -> conv_mfma_i8.hip
//   qsi8 NCHW44 depthwise                                           -> dwconv.hip
//   qsi8 3-channel NCHW -> NCHW44 3x3 stride 2 (first layer)        -> conv_first.hip
//   qsi8 NCHW -> NCHW44, other filters up to 8x8, stride 1 / 2       -> conv_hybrid_mfma.hip
//   qsi8 NCHW44 dense, anything else (5x5, 7x7, filter not packed)   -> conv_dot4.hip
//   f32 NCHW DENSE                                                  -> gemm_f32.hip
//   everything else ConvGeneral accepts                             -> conv_direct.hip
#include <mutex>

#include "common.h"
#include "conv_geom.h"

namespace mg {
bool conv_mfma_supported(const ConvGeom& g);
size_t conv_mfma_packed_bytes(const ConvGeom& g);
TinyNNStatus conv_mfma_pack(const ConvGeom& g, const void* flt, void* packed);
TinyNNStatus conv_mfma_launch(const ConvGeom&, const void*, const void*, const void*, void*,
                              const Workspace*);
size_t conv_mfma_workspace_bytes(const ConvGeom& g);
bool conv_hybrid_mfma_supported(const ConvGeom& g);
TinyNNStatus conv_hybrid_mfma_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool conv_dot4_supported(const ConvGeom& g);
TinyNNStatus conv_dot4_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool conv_first_supported(const ConvGeom& g);
TinyNNStatus conv_first_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool dwconv44_supported(const ConvGeom& g);
TinyNNStatus dwconv44_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool dwconv44_chain_supported(const ConvGeom& g, const void* src, const void* other, const void* dst);
TinyNNStatus dwconv44_chain_launch(
        const ConvGeom& g, const void* src, const void* flt, const void* bias, const void* other, void* dst,
        bool relu_after_add, float s_other, float s_out);
void dwconv44_note(const ConvGeom&, const void* src, const void* dst);
bool dwconv_nchw_supported(const ConvGeom& g, const void* src, const void* dst);
TinyNNStatus dwconv_nchw_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool conv_f32_small_supported(const ConvGeom& g);
TinyNNStatus conv_f32_small_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool dwconv44_f32_supported(const ConvGeom&);
TinyNNStatus dwconv44_f32_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool conv_first_f32_supported(const ConvGeom&);
TinyNNStatus conv_first_f32_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool conv_f32_gemm_supported(const ConvGeom& g);
TinyNNStatus conv_f32_gemm_launch(const ConvGeom&, const void*, const void*, const void*, void*,
                                  const Workspace*);
size_t conv_f32_gemm_workspace_bytes(const ConvGeom& g);
TinyNNStatus conv_direct_launch(const ConvGeom&, bool, const void*, const void*, const void*, void*);
bool conv_pw_dw_supported(const ConvGeom& pw, const ConvGeom& dw, const void* src, const void* dst);
TinyNNStatus conv_pw_dw_launch(
        const ConvGeom& pw, const ConvGeom& dw, const void* src, const void* packed, const void* pw_bias,
        const void* dw_flt, const void* dw_bias, void* dst);

// A filter that went through megcc_gfx950_conv2d_init is a 1-d byte tensor.
static bool is_packed_filter(const Tensor* flt) {
    return flt->layout.nr_dim == 1;
}

// Fills `g` from (attr, src, filter, dst). `dst` may be NULL (init / workspace time): the output
// extent is then computed from the convolution formula.
static TinyNNStatus make_geom(
        const MegccConvAttr* a, const Tensor* src, const Tensor* flt, const Tensor* dst,
        bool filter_is_packed, int oc_hint, ConvGeom* g) {
    const int fmt = a->format;
    MG_REQUIRE(fmt == MEGCC_FMT_NCHW || fmt == MEGCC_FMT_NCHW44 || fmt == MEGCC_FMT_NCHW_NCHW44,
               TinyNN_ERROR_NO_IMPLEMENT, "conv2d: format %d", fmt);
    const int src_dims = fmt == MEGCC_FMT_NCHW44 ? 5 : 4;
    MG_REQUIRE(src->layout.nr_dim == src_dims && is_contiguous(src->layout),
               TinyNN_ERROR_INVALID_LAYOUT, "conv2d: source must be a contiguous %d-d tensor",
               src_dims);
    MG_REQUIRE(a->kernel_h && a->kernel_w && a->stride_h && a->stride_w && a->dilate_h &&
                       a->dilate_w,
               TinyNN_ERROR_OUT_OF_RANGE, "conv2d: zero kernel / stride / dilation");
    const int ic_ratio = fmt == MEGCC_FMT_NCHW44 ? 4 : 1;
    const int oc_ratio = fmt == MEGCC_FMT_NCHW ? 1 : 4;
    g->fmt = fmt;
    g->act = a->nonline;
    g->has_bias = a->with_bias;
    g->n = src->layout.dims[0];
    g->ic = src->layout.dims[1] * ic_ratio;
    g->ih = src->layout.dims[2];
    g->iw = src->layout.dims[3];
    g->fh = a->kernel_h; g->fw = a->kernel_w;
    g->sh = a->stride_h; g->sw = a->stride_w;
    g->ph = a->pad_h; g->pw = a->pad_w;
    g->dh = a->dilate_h; g->dw = a->dilate_w;
    if (dst) {
        const int dst_dims = fmt == MEGCC_FMT_NCHW ? 4 : 5;
        MG_REQUIRE(dst->layout.nr_dim == dst_dims && is_contiguous(dst->layout),
                   TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: destination must be a contiguous %d-d tensor", dst_dims);
        g->oc = dst->layout.dims[1] * oc_ratio;
        g->oh = dst->layout.dims[2];
        g->ow = dst->layout.dims[3];
        MG_REQUIRE(dst->layout.dims[0] == (uint32_t)g->n, TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: batch of source and destination differ");
    } else {
        g->oc = oc_hint;
        g->oh = g->ow = -1;
    }
    const int eh = g->dh * (g->fh - 1) + 1, ew = g->dw * (g->fw - 1) + 1;
    const int want_oh = g->ih + 2 * g->ph >= eh ? (g->ih + 2 * g->ph - eh) / g->sh + 1 : 0;
    const int want_ow = g->iw + 2 * g->pw >= ew ? (g->iw + 2 * g->pw - ew) / g->sw + 1 : 0;
    if (dst)
        MG_REQUIRE(g->oh == want_oh && g->ow == want_ow, TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: destination is %dx%d, the convolution yields %dx%d", g->oh, g->ow,
                   want_oh, want_ow);
    g->oh = want_oh;
    g->ow = want_ow;

    // group count and filter shape (BareMetal/ConvKernel.cpp:209-236, 48-76)
    g->groups = 1;
    if (!filter_is_packed) {
        const Layout& fl = flt->layout;
        if (a->sparse == MEGCC_SPARSE_GROUP) {
            MG_REQUIRE(fmt != MEGCC_FMT_NCHW_NCHW44, TinyNN_ERROR_NO_IMPLEMENT,
                       "conv2d: NCHW->NCHW44 is DENSE only");
            g->groups = fl.dims[0] * (fmt == MEGCC_FMT_NCHW44 ? 4 : 1);
        }
        if (!dst && a->sparse == MEGCC_SPARSE_DENSE) {
            g->oc = fl.dims[0] * oc_ratio;
        } else if (!dst) {
            g->oc = fmt == MEGCC_FMT_NCHW ? fl.dims[0] * fl.dims[1] : g->groups;
        }
        MG_REQUIRE(g->groups > 0 && g->oc % g->groups == 0 && g->ic % g->groups == 0,
                   TinyNN_ERROR_INVALID_LAYOUT, "conv2d: %d groups do not divide ic=%d / oc=%d",
                   g->groups, g->ic, g->oc);
        const int ocpg = g->oc / g->groups, icpg = g->ic / g->groups;
        size_t want;
        if (fmt == MEGCC_FMT_NCHW44 && a->sparse == MEGCC_SPARSE_GROUP) {
            MG_REQUIRE(ocpg == 1 && icpg == 1, TinyNN_ERROR_NO_IMPLEMENT,
                       "conv2d: NCHW44 GROUP is implemented for channel-wise filters only");
            want = (size_t)g->groups * g->fh * g->fw;
        } else {
            want = (size_t)g->groups * ocpg * icpg * g->fh * g->fw;
        }
        MG_REQUIRE(nr_elem(fl) == want && is_contiguous(fl), TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: filter has %zu elements, expected %zu", nr_elem(fl), want);
    } else {
        MG_REQUIRE(a->sparse == MEGCC_SPARSE_DENSE, TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: packed filter with a GROUP convolution");
    }
    if (fmt != MEGCC_FMT_NCHW)
        MG_REQUIRE(g->oc % 4 == 0, TinyNN_ERROR_INVALID_LAYOUT, "conv2d: oc %% 4 != 0");
    g->s_src = src->dtype.param.scale;
    g->s_flt = flt->dtype.param.scale;
    g->s_dst = dst ? dst->dtype.param.scale : 1.f;
    return TinyNN_SUCCESS;
}

static bool aligned4(const void* p) {
    return ((uintptr_t)p & 3) == 0;
}
static bool aligned16(const void* p) {
    return ((uintptr_t)p & 15) == 0;
}

// A 1x1 convolution with a stride (the projection shortcut of ResNet-like networks) reads one
// input pixel per output pixel: it is the stride-1 pointwise convolution of the sub-sampled
// input. The pixels it keeps are gathered into the workspace by one strided copy (4-byte
// elements = a pixel's 4 channels), then the pointwise kernels run on dense data.
static bool strided_pointwise(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups == 1 && g.fh == 1 && g.fw == 1 && g.ph == 0 &&
           g.pw == 0 && (g.sh > 1 || g.sw > 1) && (g.ic & 3) == 0;
}
static ConvGeom subsampled(const ConvGeom& g) {
    ConvGeom s = g;
    s.ih = g.oh;
    s.iw = g.ow;
    s.sh = s.sw = 1;
    return s;
}
static size_t round_up256(size_t v) {
    return (v + 255) & ~(size_t)255;
}
// workspace = [partial sums of the stride-1 kernel, rounded up to 256 B][gathered pixels]
static size_t gather_bytes(const ConvGeom& g) {
    return (size_t)g.n * g.ic * g.oh * g.ow;
}

// A dense qsi8 convolution with spatial extent on plain NCHW tensors (a model compiled without
// the NCHW44 layout pass): the matrix-core kernels want 4 channels per pixel next to each other,
// so the layer runs as relayout NCHW -> NCHW44 into the workspace, the NCHW44 kernel, relayout
// back. The filter [OC][IC][FH][FW] packs into the same tiles as an NCHW44 one; the bias layouts
// are the same bytes.
static bool nchw_spatial(const ConvGeom& g) {
    // (at most 9 taps: the generated workspace function sizes the copies for those filters only)
    return g.fmt == MEGCC_FMT_NCHW && g.groups == 1 && g.fh * g.fw <= 9 &&
           !(g.ih == 1 && g.iw == 1 && g.fh == 1 && g.fw == 1);
}
// (channel counts that are no multiple of 4 are padded: the packed filter holds zeros for channels
//  beyond IC / OC anyway, so what the padding lanes of the NCHW44 copies hold does not matter)
static int round_up4(int v) {
    return (v + 3) & ~3;
}
static ConvGeom as_nchw44(const ConvGeom& g) {
    ConvGeom s = g;
    s.fmt = MEGCC_FMT_NCHW44;
    s.ic = round_up4(g.ic);
    s.oc = round_up4(g.oc);
    return s;
}
// workspace of the detour: [inner kernel's][input copy][output copy][bias copy when OC % 4 != 0]
static size_t nchw_spatial_bytes(const ConvGeom& g, size_t inner) {
    const ConvGeom g1 = as_nchw44(g);
    return round_up256(inner) + round_up256((size_t)g.n * g1.ic * g.ih * g.iw) +
           round_up256((size_t)g.n * g1.oc * g.oh * g.ow) + (g1.oc != g.oc ? round_up256((size_t)g1.oc * 4) : 0);
}
// Channel-wise (depthwise) qsi8 convolution on plain NCHW tensors: the same detour around the
// NCHW44 depthwise kernel; the filter [G,1,1,FH,FW] becomes [G/4,1,1,FH,FW,4] by a third, tiny
// relayout. Workspace = [input copy, 256][output copy, 256][filter].
static bool nchw_depthwise(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW && g.groups > 1 && g.groups == g.ic && g.ic == g.oc && (g.ic & 3) == 0 &&
           (long)g.n * g.ic * g.ih * g.iw < (1L << 31) && (long)g.n * g.oc * g.oh * g.ow < (1L << 31);
}
static size_t nchw_depthwise_bytes(const ConvGeom& g) {
    return round_up256((size_t)g.n * g.ic * g.ih * g.iw) + round_up256((size_t)g.n * g.oc * g.oh * g.ow) +
           (size_t)g.ic * g.fh * g.fw;
}
// [N, C/4, H, W, 4] view (byte strides = element strides) of an NCHW int8 tensor, and the dense one
static void nchw44_views(int n, int c, int h, int w, Layout* view, Layout* dense) {
    view->nr_dim = dense->nr_dim = 5;
    const uint32_t d[5] = {(uint32_t)n, (uint32_t)(c / 4), (uint32_t)h, (uint32_t)w, 4u};
    const int vs[5] = {c * h * w, 4 * h * w, w, 1, h * w};
    const int ds[5] = {c * h * w, 4 * h * w, 4 * w, 4, 1};
    for (int i = 0; i < 5; ++i) {
        view->dims[i] = dense->dims[i] = d[i];
        view->stride[i] = vs[i];
        dense->stride[i] = ds[i];
    }
}
// f32 dense layers in NCHW44 (the layout MegCC gives fp32 models on ARM): the implicit-GEMM kernel
// works on NCHW, so the layer runs as relayout NCHW44 -> NCHW into the workspace, that kernel,
// relayout back; the filter [OC/4][IC/4][FH][FW][4 ic][4 oc] becomes [OC][IC][FH][FW] by a third,
// small relayout. The bias layouts are the same bytes.
static bool f32_nchw44_dense(const ConvGeom& g) {
    return g.fmt == MEGCC_FMT_NCHW44 && g.groups == 1 && (g.ic & 3) == 0 && (g.oc & 3) == 0;
}
static ConvGeom as_nchw(const ConvGeom& g) {
    ConvGeom s = g;
    s.fmt = MEGCC_FMT_NCHW;
    return s;
}
// workspace of that detour: [inner kernel's][input copy][output copy][filter copy]
static size_t f32_nchw44_bytes(const ConvGeom& g, size_t inner) {
    return round_up256(inner) + round_up256((size_t)g.n * g.ic * g.ih * g.iw * 4) +
           round_up256((size_t)g.n * g.oc * g.oh * g.ow * 4) + round_up256((size_t)g.oc * g.ic * g.fh * g.fw * 4);
}
// NCHW tensor with c channels <-> NCHW44 tensor with round_up4(c) channels: the whole groups of 4
// in one copy, the last group's c % 4 channels in a second (its other lanes are not touched)
static TinyNNStatus nchw_nchw44_copy(
        bool to44, const void* from, void* to, int n, int c, int h, int w, const char* what) {
    const int c1 = round_up4(c), full = c & ~3, rem = c - full;
    const char* nchw = (const char*)(to44 ? from : to);
    const char* n44 = (const char*)(to44 ? to : from);
    for (int part = 0; part < 2; ++part) {
        const int groups = part == 0 ? full / 4 : 1, lanes = part == 0 ? 4 : rem;
        if (groups == 0 || lanes == 0)
            continue;
        Layout view = {}, dense = {};
        view.nr_dim = dense.nr_dim = 5;
        const uint32_t d[5] = {(uint32_t)n, (uint32_t)groups, (uint32_t)h, (uint32_t)w, (uint32_t)lanes};
        const int vs[5] = {c * h * w, 4 * h * w, w, 1, h * w};
        const int ds[5] = {c1 * h * w, 4 * h * w, 4 * w, 4, 1};
        for (int i = 0; i < 5; ++i) {
            view.dims[i] = dense.dims[i] = d[i];
            view.stride[i] = vs[i];
            dense.stride[i] = ds[i];
        }
        const size_t off = part == 0 ? 0 : (size_t)full * h * w;  // first byte of the last group in both
        TinyNNStatus st = to44 ? strided_copy(nchw + off, view, (char*)n44 + off, dense, 1, what)
                               : strided_copy(n44 + off, dense, (char*)nchw + off, view, 1, what);
        if (st != TinyNN_SUCCESS)
            return st;
    }
    return TinyNN_SUCCESS;
}

// ---- scratch memory of megcc_gfx950_conv2d_noalloc ---------------------------------------------
// One array per GPU, placed by the loader when the code object is loaded on that GPU; it holds
// whatever the last call left in it. In host code its NAME is only a handle for
// hipGetSymbolAddress: every use of the memory goes through the per-device address that call
// returns.
static __device__ __align__(256) unsigned char scratch[MEGCC_GFX950_NOALLOC_SCRATCH_BYTES];

static constexpr int MAX_GPUS = 64;
static void* g_scratch_ptr[MAX_GPUS];  // address of `scratch` on device i, once asked for
static std::mutex g_scratch_lock;

// Address of the current device's copy of `scratch` (asked for once per device).
static TinyNNStatus scratch_of_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    MG_REQUIRE(e == hipSuccess && dev >= 0 && dev < MAX_GPUS, TinyNN_ERROR_RUNTIME,
               "conv2d_noalloc: no current HIP device (%s)", hipGetErrorString(e));
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        MG_REQUIRE(e == hipSuccess && p, TinyNN_ERROR_RUNTIME,
                   "conv2d_noalloc: address of the scratch array on device %d: %s", dev,
                   hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return TinyNN_SUCCESS;
}

TinyNNStatus noalloc_scratch_setup() {
    void* p = nullptr;
    return scratch_of_current_device(&p);
}

// Scratch bytes the kernels of this layer take from the workspace (what
// megcc_gfx950_conv2d_workspace reports before the filter is packed).
static size_t conv2d_scratch_bytes(const ConvGeom& g, bool q8, bool f32, bool packed) {
    if (packed && q8 && strided_pointwise(g) && conv_mfma_supported(subsampled(g)))
        return round_up256(conv_mfma_workspace_bytes(subsampled(g))) + gather_bytes(g);
    if (packed && q8 && nchw_spatial(g) && conv_mfma_supported(as_nchw44(g)))
        return nchw_spatial_bytes(g, conv_mfma_workspace_bytes(as_nchw44(g)));
    if (packed && q8 && conv_mfma_supported(g))
        return conv_mfma_workspace_bytes(g);
    if (!packed && q8 && nchw_depthwise(g) && dwconv44_supported(as_nchw44(g)))
        return nchw_depthwise_bytes(g);
    if (f32 && !(conv_f32_small_supported(g) && !options().no_f32small) && conv_f32_gemm_supported(g))
        return conv_f32_gemm_workspace_bytes(g);
    if (f32 && f32_nchw44_dense(g) && conv_f32_gemm_supported(as_nchw(g)))
        return f32_nchw44_bytes(g, conv_f32_gemm_workspace_bytes(as_nchw(g)));
    return 0;
}

}  // namespace mg

using namespace mg;

// `workspace` from the caller, or (static_scratch) the library's own array of the current GPU.
static TinyNNStatus conv2d_run(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, bool static_scratch) {
    MG_REQUIRE(attr, TinyNN_ERROR_NULL_PTR, "conv2d: NULL attr");
    const int want_in = attr->with_bias ? 3 : 2;
    // the test harness of the reference passes an extra empty `z` operand after the bias
    TinyNNStatus st = check_io(inputs, nr_input < want_in ? nr_input : want_in, want_in, want_in,
                               outputs, nr_output, "conv2d");
    if (st != TinyNN_SUCCESS)
        return st;
    MG_REQUIRE(nr_input <= want_in + 1, TinyNN_ERROR_OUT_OF_RANGE, "conv2d: %d inputs", nr_input);
    const Tensor *src = inputs[0], *flt = inputs[1], *dst = outputs[0];
    const Tensor* bias = attr->with_bias ? inputs[2] : nullptr;
    const bool q8 = is_q8(src) && is_q8(flt) && is_q8(dst) && (!bias || is_q32(bias));
    const bool f32 = is_f32(src) && is_f32(flt) && is_f32(dst) && (!bias || is_f32(bias));
    MG_REQUIRE(q8 || f32, TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
               "conv2d: operands must be qsi8,qsi8[,qsi32]->qsi8 or all f32");
    const bool packed = is_packed_filter(flt);
    ConvGeom g;
    st = make_geom(attr, src, flt, dst, packed, 0, &g);
    if (st != TinyNN_SUCCESS)
        return st;
    if (bias) {
        MG_REQUIRE(nr_elem(bias->layout) == (size_t)g.oc && is_contiguous(bias->layout),
                   TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: bias must be per output channel (%zu elements, oc=%d)",
                   nr_elem(bias->layout), g.oc);
        if (q8) {
            // ConvGeneral::IsAvailable, BareMetal/ConvKernel.cpp:37-42
            float d = g.s_src * g.s_flt - bias->dtype.param.scale;
            MG_REQUIRE((d < 0 ? -d : d) < 1e-5f, TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE,
                       "conv2d: bias scale %g != src scale * filter scale %g",
                       bias->dtype.param.scale, g.s_src * g.s_flt);
        }
    }
    if (q8)
        MG_REQUIRE(g.s_dst > 0.f, TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE, "conv2d: dst scale <= 0");
    const void* b = bias ? bias->ptr : nullptr;
    if ((size_t)g.n * g.oc * g.oh * g.ow == 0)
        return TinyNN_SUCCESS;
    Workspace own = {nullptr, 0, 0};
    if (static_scratch) {
        // (the native kernel for channel-wise NCHW layers needs none)
        const bool native_dw = q8 && dwconv_nchw_supported(g, src->ptr, dst->ptr) && !options().no_dwnchw;
        const size_t need = native_dw ? 0 : conv2d_scratch_bytes(g, q8, f32, packed);
        // Only two paths cannot run without their scratch: a strided 1x1 layer (gathered pixels) and
        // a dense layer on plain NCHW tensors (NCHW44 copies), both behind a packed filter. Every
        // other request is an optimisation (split-K partial sums, relayout detours) that
        // megcc_gfx950_conv2d also does without when it gets no workspace: same result, other kernel.
        const bool strict = packed && q8 &&
                            ((strided_pointwise(g) && conv_mfma_supported(subsampled(g))) ||
                             (nchw_spatial(g) && conv_mfma_supported(as_nchw44(g))));
        MG_REQUIRE(need <= (size_t)MEGCC_GFX950_NOALLOC_SCRATCH_BYTES || !strict, TinyNN_ERROR_OUT_OF_RANGE,
                   "conv2d_noalloc: this layer needs %zu bytes of scratch memory, the static "
                   "buffer holds %zu; call megcc_gfx950_conv2d with a workspace instead",
                   need, (size_t)MEGCC_GFX950_NOALLOC_SCRATCH_BYTES);
        if (need && need <= (size_t)MEGCC_GFX950_NOALLOC_SCRATCH_BYTES) {
            st = scratch_of_current_device(&own.ptr);
            if (st != TinyNN_SUCCESS)
                return st;
            own.size = need;
        }
        workspace = &own;
    }

    if (packed && q8 && strided_pointwise(g) && conv_mfma_supported(subsampled(g))) {
        const ConvGeom g1 = subsampled(g);
        MG_REQUIRE(nr_elem(flt->layout) == conv_mfma_packed_bytes(g1), TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: packed filter has %zu bytes, expected %zu", nr_elem(flt->layout),
                   conv_mfma_packed_bytes(g1));
        MG_REQUIRE(aligned4(src->ptr) && aligned4(dst->ptr) && aligned16(flt->ptr) && (!b || aligned4(b)),
                   TinyNN_ERROR_INVALID_LAYOUT, "conv2d: misaligned operand");
        const size_t inner = round_up256(conv_mfma_workspace_bytes(g1));
        MG_REQUIRE(workspace && workspace->ptr && workspace->size >= inner + gather_bytes(g) &&
                           aligned16(workspace->ptr),
                   TinyNN_ERROR_OUT_OF_RANGE,
                   "conv2d: a strided 1x1 convolution needs %zu bytes of workspace",
                   inner + gather_bytes(g));
        void* gathered = (char*)workspace->ptr + inner;
        Layout from = {}, to = {};
        from.nr_dim = to.nr_dim = 3;  // [N * C/4, OH, OW] of 4-byte pixels
        from.dims[0] = to.dims[0] = (uint32_t)(g.n * (g.ic / 4));
        from.dims[1] = to.dims[1] = (uint32_t)g.oh;
        from.dims[2] = to.dims[2] = (uint32_t)g.ow;
        from.stride[0] = g.ih * g.iw; from.stride[1] = g.sh * g.iw; from.stride[2] = g.sw;
        to.stride[0] = g.oh * g.ow; to.stride[1] = g.ow; to.stride[2] = 1;
        st = strided_copy(src->ptr, from, gathered, to, 4, "conv2d (gather of a strided 1x1)");
        if (st != TinyNN_SUCCESS)
            return st;
        Workspace sub = {workspace->ptr, inner, 0};
        return conv_mfma_launch(g1, gathered, flt->ptr, b, dst->ptr, &sub);
    }
    if (packed && q8 && nchw_spatial(g) && conv_mfma_supported(as_nchw44(g))) {
        const ConvGeom g1 = as_nchw44(g);
        MG_REQUIRE(nr_elem(flt->layout) == conv_mfma_packed_bytes(g1), TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: packed filter has %zu bytes, expected %zu", nr_elem(flt->layout),
                   conv_mfma_packed_bytes(g1));
        MG_REQUIRE(aligned16(flt->ptr) && (!b || aligned4(b)), TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: misaligned operand");
        const size_t inner = round_up256(conv_mfma_workspace_bytes(g1));
        const size_t in44 = round_up256((size_t)g.n * g1.ic * g.ih * g.iw);
        const size_t out44 = round_up256((size_t)g.n * g1.oc * g.oh * g.ow);
        const size_t need = nchw_spatial_bytes(g, conv_mfma_workspace_bytes(g1));
        MG_REQUIRE(workspace && workspace->ptr && workspace->size >= need && aligned16(workspace->ptr),
                   TinyNN_ERROR_OUT_OF_RANGE, "conv2d: a dense NCHW convolution needs %zu bytes of workspace",
                   need);
        MG_REQUIRE((long)g.n * g1.ic * g.ih * g.iw < (1L << 31) && (long)g.n * g1.oc * g.oh * g.ow < (1L << 31),
                   TinyNN_ERROR_OUT_OF_RANGE, "conv2d: tensor too large");
        char* src44 = (char*)workspace->ptr + inner;
        char* dst44 = src44 + in44;
        st = nchw_nchw44_copy(true, src->ptr, src44, g.n, g.ic, g.ih, g.iw, "conv2d (NCHW -> NCHW44)");
        if (st != TinyNN_SUCCESS)
            return st;
        const void* b1 = b;
        if (b && g1.oc != g.oc) {
            // the kernel reads a bias per (padded) output channel: a copy it may read to the end
            Layout bl = {};
            bl.nr_dim = 1;
            bl.dims[0] = (uint32_t)g.oc;
            bl.stride[0] = 1;
            st = strided_copy(b, bl, dst44 + out44, bl, 4, "conv2d (bias)");
            if (st != TinyNN_SUCCESS)
                return st;
            b1 = dst44 + out44;
        }
        Workspace sub = {workspace->ptr, inner, 0};
        st = conv_mfma_launch(g1, src44, flt->ptr, b1, dst44, &sub);
        if (st != TinyNN_SUCCESS)
            return st;
        return nchw_nchw44_copy(false, dst44, dst->ptr, g.n, g.oc, g.oh, g.ow, "conv2d (NCHW44 -> NCHW)");
    }
    if (packed) {
        MG_REQUIRE(q8 && conv_mfma_supported(g), TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: a packed filter was passed to a convolution the MFMA kernel does not cover");
        MG_REQUIRE(nr_elem(flt->layout) == conv_mfma_packed_bytes(g), TinyNN_ERROR_INVALID_LAYOUT,
                   "conv2d: packed filter has %zu bytes, expected %zu", nr_elem(flt->layout),
                   conv_mfma_packed_bytes(g));
        MG_REQUIRE(aligned4(src->ptr) && aligned4(dst->ptr) && aligned16(flt->ptr) &&
                           (!b || aligned4(b)),
                   TinyNN_ERROR_INVALID_LAYOUT, "conv2d: misaligned operand");
        return conv_mfma_launch(g, src->ptr, flt->ptr, b, dst->ptr, workspace);
    }
    // channel-wise 3x3 on plain NCHW planes whose rows are a multiple of 4 pixels: native kernel
    if (q8 && dwconv_nchw_supported(g, src->ptr, dst->ptr) && !options().no_dwnchw) {
        note_kernel("dwconv_nchw", g.sh);
        return dwconv_nchw_launch(g, src->ptr, flt->ptr, b, dst->ptr);
    }
    if (q8 && nchw_depthwise(g) && dwconv44_supported(as_nchw44(g)) && workspace && workspace->ptr &&
        workspace->size >= nchw_depthwise_bytes(g) && aligned16(workspace->ptr)) {
        const ConvGeom g1 = as_nchw44(g);
        char* src44 = (char*)workspace->ptr;
        char* dst44 = src44 + round_up256((size_t)g.n * g.ic * g.ih * g.iw);
        char* flt44 = dst44 + round_up256((size_t)g.n * g.oc * g.oh * g.ow);
        Layout view, dense;
        nchw44_views(g.n, g.ic, g.ih, g.iw, &view, &dense);
        st = strided_copy(src->ptr, view, src44, dense, 1, "conv2d (NCHW -> NCHW44)");
        if (st != TinyNN_SUCCESS)
            return st;
        const int taps = g.fh * g.fw;
        Layout fv = {}, fd = {};  // [G/4, taps, 4]: channel c = 4 * group + lane
        fv.nr_dim = fd.nr_dim = 3;
        fv.dims[0] = fd.dims[0] = (uint32_t)(g.ic / 4);
        fv.dims[1] = fd.dims[1] = (uint32_t)taps;
        fv.dims[2] = fd.dims[2] = 4;
        fv.stride[0] = 4 * taps; fv.stride[1] = 1; fv.stride[2] = taps;
        fd.stride[0] = 4 * taps; fd.stride[1] = 4; fd.stride[2] = 1;
        st = strided_copy(flt->ptr, fv, flt44, fd, 1, "conv2d (depthwise filter -> NCHW44)");
        if (st != TinyNN_SUCCESS)
            return st;
        note_kernel("dwconv44 between NCHW relayouts");
        st = dwconv44_launch(g1, src44, flt44, b, dst44);
        if (st != TinyNN_SUCCESS)
            return st;
        nchw44_views(g.n, g.oc, g.oh, g.ow, &view, &dense);
        return strided_copy(dst44, dense, dst->ptr, view, 1, "conv2d (NCHW44 -> NCHW)");
    }
    if (q8 && dwconv44_supported(g) && aligned4(src->ptr) && aligned4(flt->ptr) &&
        aligned4(dst->ptr)) {
        dwconv44_note(g, src->ptr, dst->ptr);
        return dwconv44_launch(g, src->ptr, flt->ptr, b, dst->ptr);
    }
    if (q8 && conv_first_supported(g) && aligned4(src->ptr) && aligned4(dst->ptr) && (!b || aligned4(b))) {
        note_kernel("conv_first_q8");
        return conv_first_launch(g, src->ptr, flt->ptr, b, dst->ptr);
    }
    if (q8 && conv_hybrid_mfma_supported(g) && aligned4(dst->ptr) && aligned4(flt->ptr) && (!b || aligned4(b)) &&
        !options().no_hybrid) {
        note_kernel("conv_hybrid_mfma");
        return conv_hybrid_mfma_launch(g, src->ptr, flt->ptr, b, dst->ptr);
    }
    if (q8 && conv_dot4_supported(g) && aligned4(src->ptr) && aligned4(dst->ptr) && aligned16(flt->ptr) &&
        (!b || aligned4(b)) && !options().no_dot4) {
        note_kernel("conv_dot4");
        return conv_dot4_launch(g, src->ptr, flt->ptr, b, dst->ptr);
    }
    if (f32 && f32_nchw44_dense(g) && conv_f32_gemm_supported(as_nchw(g)) && workspace && workspace->ptr &&
        aligned16(workspace->ptr) &&
        workspace->size >= f32_nchw44_bytes(g, conv_f32_gemm_workspace_bytes(as_nchw(g)))) {
        const ConvGeom g1 = as_nchw(g);
        const size_t inner = round_up256(conv_f32_gemm_workspace_bytes(g1));
        char* src_nchw = (char*)workspace->ptr + inner;
        char* dst_nchw = src_nchw + round_up256((size_t)g.n * g.ic * g.ih * g.iw * 4);
        char* flt_nchw = dst_nchw + round_up256((size_t)g.n * g.oc * g.oh * g.ow * 4);
        Layout view, dense;
        nchw44_views(g.n, g.ic, g.ih, g.iw, &view, &dense);
        st = strided_copy(src->ptr, dense, src_nchw, view, 4, "conv2d (f32 NCHW44 -> NCHW)");
        if (st != TinyNN_SUCCESS)
            return st;
        const int taps = g.fh * g.fw;
        Layout fs = {}, fd = {};  // [OC/4][IC/4][taps][4 ic][4 oc] -> oc = 4 * og + o, ic = 4 * ig + i
        fs.nr_dim = fd.nr_dim = 5;
        const uint32_t fdim[5] = {(uint32_t)(g.oc / 4), (uint32_t)(g.ic / 4), (uint32_t)taps, 4u, 4u};
        const int fss[5] = {(g.ic / 4) * taps * 16, taps * 16, 16, 4, 1};
        const int fds[5] = {4 * g.ic * taps, 4 * taps, 1, taps, g.ic * taps};
        for (int i = 0; i < 5; ++i) {
            fs.dims[i] = fd.dims[i] = fdim[i];
            fs.stride[i] = fss[i];
            fd.stride[i] = fds[i];
        }
        st = strided_copy(flt->ptr, fs, flt_nchw, fd, 4, "conv2d (f32 NCHW44 filter -> NCHW)");
        if (st != TinyNN_SUCCESS)
            return st;
        note_kernel("conv_f32_gemm between NCHW44 relayouts");
        Workspace sub = {workspace->ptr, inner, 0};
        st = conv_f32_gemm_launch(g1, src_nchw, flt_nchw, b, dst_nchw, &sub);
        if (st != TinyNN_SUCCESS)
            return st;
        nchw44_views(g.n, g.oc, g.oh, g.ow, &view, &dense);
        return strided_copy(dst_nchw, view, dst->ptr, dense, 4, "conv2d (f32 NCHW -> NCHW44)");
    }
    if (f32 && conv_f32_small_supported(g) && !options().no_f32small) {
        note_kernel("conv_f32_small");
        return conv_f32_small_launch(g, src->ptr, flt->ptr, b, dst->ptr);
    }
    if (f32 && conv_f32_gemm_supported(g)) {
        note_kernel("conv_f32_gemm");
        return conv_f32_gemm_launch(g, src->ptr, flt->ptr, b, dst->ptr, workspace);
    }
    if (f32 && dwconv44_f32_supported(g) && aligned16(src->ptr) && aligned16(flt->ptr) && aligned16(dst->ptr) &&
        (!b || aligned16(b))) {
        note_kernel("dwconv44_f32", g.fh, g.sh);
        return dwconv44_f32_launch(g, src->ptr, flt->ptr, b, dst->ptr);
    }
    if (f32 && conv_first_f32_supported(g) && aligned4(src->ptr) && aligned16(flt->ptr) && aligned16(dst->ptr) &&
        (!b || aligned16(b))) {
        note_kernel("conv_first_f32", g.fh, g.sh);
        return conv_first_f32_launch(g, src->ptr, flt->ptr, b, dst->ptr);
    }
    note_kernel("conv_direct");
    return conv_direct_launch(g, f32, src->ptr, flt->ptr, b, dst->ptr);
}

extern "C" TinyNNStatus megcc_gfx950_conv2d(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, const RuntimeOpt*) {
    return conv2d_run(attr, inputs, nr_input, outputs, nr_output, workspace, false);
}

extern "C" TinyNNStatus megcc_gfx950_conv2d_noalloc(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const RuntimeOpt*) {
    return conv2d_run(attr, inputs, nr_input, outputs, nr_output, nullptr, true);
}

extern "C" TinyNNStatus megcc_gfx950_conv2d_init(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, Tensor* out_weights,
        int* nr_out_weight, const RuntimeOpt*) {
    MG_REQUIRE(attr && inputs && nr_input >= 2 && inputs[0] && inputs[1], TinyNN_ERROR_NULL_PTR,
               "conv2d_init: NULL argument");
    const Tensor *src = inputs[0], *flt = inputs[1];
    ConvGeom g;
    bool pack = false;
    if (is_q8(src) && is_q8(flt) && attr->sparse == MEGCC_SPARSE_DENSE &&
        !is_packed_filter(flt)) {
        TinyNNStatus st = make_geom(attr, src, flt, nullptr, false, 0, &g);
        if (st != TinyNN_SUCCESS)
            return st;
        if (strided_pointwise(g))
            g = subsampled(g);
        // (an NCHW filter packs into the tiles of the NCHW44 kernel: conv_mfma_pack reads g.fmt)
        pack = nchw_spatial(g) ? conv_mfma_supported(as_nchw44(g)) : conv_mfma_supported(g);
    }
    if (!out_weights) {  // phase 1: how many
        MG_REQUIRE(nr_out_weight, TinyNN_ERROR_NULL_PTR, "conv2d_init: both outputs NULL");
        *nr_out_weight = pack ? 1 : 0;
        return TinyNN_SUCCESS;
    }
    if (!pack) {
        if (nr_out_weight)
            *nr_out_weight = 0;
        return TinyNN_SUCCESS;
    }
    if (!nr_out_weight) {  // phase 2: describe
        out_weights->layout.nr_dim = 1;
        out_weights->layout.dims[0] = (uint32_t)conv_mfma_packed_bytes(g);
        out_weights->layout.stride[0] = 1;
        out_weights->layout.format = flt->layout.format;
        out_weights->dtype = flt->dtype;
        out_weights->name = flt->name;  // identity by name pointer: runtime/src/init.c:64,88
        return TinyNN_SUCCESS;
    }
    // phase 3: transform into the caller-allocated device buffer
    MG_REQUIRE(out_weights->ptr && flt->ptr, TinyNN_ERROR_NULL_PTR, "conv2d_init: NULL weight");
    MG_REQUIRE(aligned16(out_weights->ptr), TinyNN_ERROR_INVALID_LAYOUT,
               "conv2d_init: processed weight must be 16-byte aligned");
    *nr_out_weight = 1;
    return conv_mfma_pack(g, flt->ptr, out_weights->ptr);
}

// im2col never leaves LDS, so the quantized kernels need no scratch; the f32 implicit GEMM asks
// for room for split-K partial sums when the layer has too few tiles to fill the chip.
extern "C" TinyNNStatus megcc_gfx950_conv2d_workspace(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, int, size_t* workspace) {
    MG_REQUIRE(workspace, TinyNN_ERROR_NULL_PTR, "conv2d_workspace: NULL size");
    *workspace = 0;
    if (!attr || !inputs || nr_input < 2 || !inputs[0] || !inputs[1])
        return TinyNN_SUCCESS;
    const Tensor *src = inputs[0], *flt = inputs[1];
    ConvGeom g;
    if (is_f32(src) && is_f32(flt)) {
        if (make_geom(attr, src, flt, nullptr, false, 0, &g) == TinyNN_SUCCESS) {
            if (conv_f32_gemm_supported(g))
                *workspace = conv_f32_gemm_workspace_bytes(g);
            else if (attr->sparse == MEGCC_SPARSE_DENSE && f32_nchw44_dense(g) && conv_f32_gemm_supported(as_nchw(g)))
                *workspace = f32_nchw44_bytes(g, conv_f32_gemm_workspace_bytes(as_nchw(g)));
        }
    } else if (is_q8(src) && is_q8(flt) && attr->sparse == MEGCC_SPARSE_GROUP) {
        if (make_geom(attr, src, flt, nullptr, false, 0, &g) == TinyNN_SUCCESS && nchw_depthwise(g))
            *workspace = nchw_depthwise_bytes(g);
    } else if (is_q8(src) && is_q8(flt) && attr->sparse == MEGCC_SPARSE_DENSE &&
               !is_packed_filter(flt)) {
        // split-K partial sums of the one-stage MFMA kernel (few pixels, long K)
        if (make_geom(attr, src, flt, nullptr, false, 0, &g) == TinyNN_SUCCESS) {
            if (strided_pointwise(g) && conv_mfma_supported(subsampled(g)))
                *workspace = round_up256(conv_mfma_workspace_bytes(subsampled(g))) + gather_bytes(g);
            else if (nchw_spatial(g) && conv_mfma_supported(as_nchw44(g)))
                *workspace = nchw_spatial_bytes(g, conv_mfma_workspace_bytes(as_nchw44(g)));
            else if (conv_mfma_supported(g))
                *workspace = conv_mfma_workspace_bytes(g);
        }
    }
    return TinyNN_SUCCESS;
}

// ---- depthwise 3x3 -> max-pool 2x2 s2 -> QADD / QFUSE_ADD_RELU as one operator --------------------
// Fills `g` (the depthwise layer; its s_dst is the scale between the operators) and checks the
// operands; `why` gets the reason when they are not what the kernel takes.
static bool dw_pool_add_geom(
        const MegccDwPoolAddAttr* a, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output, ConvGeom* g,
        const Tensor** other_out, const char** why) {
    *why = "NULL argument";
    if (!a || !inputs || !outputs || nr_output != 1 || !outputs[0])
        return false;
    const int want_in = a->conv.with_bias ? 4 : 3;
    *why = "inputs: source, filter, [bias,] second operand of the addition";
    if (nr_input != want_in)
        return false;
    for (int i = 0; i < nr_input; ++i)
        if (!inputs[i])
            return false;
    const Tensor *src = inputs[0], *flt = inputs[1], *bias = a->conv.with_bias ? inputs[2] : nullptr;
    const Tensor *other = inputs[want_in - 1], *dst = outputs[0];
    *why = "operands must be qsi8 (bias qsi32)";
    if (!is_q8(src) || !is_q8(flt) || !is_q8(other) || !is_q8(dst) || (bias && !is_q32(bias)))
        return false;
    *why = "conv: NCHW44 GROUP 3x3, pad 1, stride 1 or 2; pool: MAX 2x2 stride 2 pad 0 NCHW44; mode: QADD or QFUSE_ADD_RELU";
    if (a->conv.format != MEGCC_FMT_NCHW44 || a->conv.sparse != MEGCC_SPARSE_GROUP || a->pool.format != MEGCC_FMT_NCHW44 ||
        a->pool.mode != MEGCC_POOL_MAX || a->pool.window_h != 2 || a->pool.window_w != 2 || a->pool.stride_h != 2 ||
        a->pool.stride_w != 2 || a->pool.pad_h != 0 || a->pool.pad_w != 0 ||
        !(a->mode == MEGCC_Q_ADD || a->mode == MEGCC_Q_FUSE_ADD_RELU) || !(a->mid_scale > 0.f))
        return false;
    *why = "filter / source layout";
    if (is_packed_filter(flt) || make_geom(&a->conv, src, flt, nullptr, false, 0, g) != TinyNN_SUCCESS)
        return false;
    g->s_dst = a->mid_scale;
    *why = "bias must be per channel";
    if (bias && !(nr_elem(bias->layout) == (size_t)g->oc && is_contiguous(bias->layout)))
        return false;
    *why = "second operand and result must be contiguous [N, C/4, OH/2, OW/2, 4] tensors";
    const uint32_t want[5] = {(uint32_t)g->n, (uint32_t)(g->oc / 4), (uint32_t)(g->oh / 2), (uint32_t)(g->ow / 2), 4u};
    for (const Tensor* t : {other, dst}) {
        if (t->layout.nr_dim != 5 || !is_contiguous(t->layout))
            return false;
        for (int i = 0; i < 5; ++i)
            if (t->layout.dims[i] != want[i])
                return false;
    }
    *why = "alignment, extent or window the kernel does not take";
    if (!dwconv44_chain_supported(*g, src->ptr, other->ptr, dst->ptr) || !aligned4(flt->ptr) ||
        (bias && !aligned4(bias->ptr)))
        return false;
    *other_out = other;
    return true;
}

extern "C" int megcc_gfx950_dw_pool_add_supported(
        const MegccDwPoolAddAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output) {
    ConvGeom g;
    const Tensor* other = nullptr;
    const char* why = "";
    return dw_pool_add_geom(attr, inputs, nr_input, outputs, nr_output, &g, &other, &why) ? 1 : 0;
}

extern "C" TinyNNStatus megcc_gfx950_dw_pool_add(
        const MegccDwPoolAddAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace*, const RuntimeOpt*) {
    ConvGeom g;
    const Tensor* other = nullptr;
    const char* why = "";
    MG_REQUIRE(dw_pool_add_geom(attr, inputs, nr_input, outputs, nr_output, &g, &other, &why),
               TinyNN_ERROR_INVALID_LAYOUT, "dw_pool_add: %s", why);
    note_kernel("dwconv44_chain", g.sh, attr->mode == MEGCC_Q_FUSE_ADD_RELU);
    return dwconv44_chain_launch(
            g, inputs[0]->ptr, inputs[1]->ptr, attr->conv.with_bias ? inputs[2]->ptr : nullptr, other->ptr,
            outputs[0]->ptr, attr->mode == MEGCC_Q_FUSE_ADD_RELU, other->dtype.param.scale,
            outputs[0]->dtype.param.scale);
}

// ---- pointwise 1x1 -> channel-wise 3x3 as one operator -------------------------------------------
// Fills the two layers' geometries (pw.s_dst = dw.s_src = the scale in between) and checks the
// operands; `why` gets the reason when they are not what the kernel takes.
struct PwDwOperands {
    const Tensor *src, *packed, *pw_bias, *dw_flt, *dw_bias, *dst;
};
static bool pw_dw_geom(
        const MegccPwDwAttr* a, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output, ConvGeom* pw,
        ConvGeom* dw, PwDwOperands* t, const char** why) {
    *why = "NULL argument";
    if (!a || !inputs || !outputs || nr_output != 1 || !outputs[0])
        return false;
    *why = "inputs: source, packed pointwise filter, [pointwise bias,] channel-wise filter [, channel-wise bias]";
    if (nr_input != 3 + (a->pw.with_bias ? 1 : 0) + (a->dw.with_bias ? 1 : 0))
        return false;
    for (int i = 0; i < nr_input; ++i)
        if (!inputs[i])
            return false;
    int k = 0;
    t->src = inputs[k++];
    t->packed = inputs[k++];
    t->pw_bias = a->pw.with_bias ? inputs[k++] : nullptr;
    t->dw_flt = inputs[k++];
    t->dw_bias = a->dw.with_bias ? inputs[k++] : nullptr;
    t->dst = outputs[0];
    *why = "operands must be qsi8 (biases qsi32)";
    if (!is_q8(t->src) || !is_q8(t->packed) || !is_q8(t->dw_flt) || !is_q8(t->dst) ||
        (t->pw_bias && !is_q32(t->pw_bias)) || (t->dw_bias && !is_q32(t->dw_bias)))
        return false;
    *why = "pw: NCHW44 DENSE 1x1 with the filter from megcc_gfx950_conv2d_init; dw: NCHW44 GROUP 3x3";
    if (a->pw.format != MEGCC_FMT_NCHW44 || a->pw.sparse != MEGCC_SPARSE_DENSE || a->dw.format != MEGCC_FMT_NCHW44 ||
        a->dw.sparse != MEGCC_SPARSE_GROUP || !is_packed_filter(t->packed) || is_packed_filter(t->dw_flt) ||
        !(a->mid_scale > 0.f) || t->dw_flt->layout.nr_dim < 1)
        return false;
    *why = "source / filter / destination layout";
    const int oc = (int)t->dw_flt->layout.dims[0] * 4;
    if (make_geom(&a->pw, t->src, t->packed, nullptr, true, oc, pw) != TinyNN_SUCCESS || pw->oh <= 0 || pw->ow <= 0)
        return false;
    pw->s_dst = a->mid_scale;
    Tensor mid = {};
    mid.dtype.type_enum = TinyNN_QINT8;
    mid.dtype.param.scale = a->mid_scale;
    mid.layout.nr_dim = 5;
    const uint32_t md[5] = {(uint32_t)pw->n, (uint32_t)(oc / 4), (uint32_t)pw->oh, (uint32_t)pw->ow, 4u};
    int stride = 1;
    for (int i = 4; i >= 0; --i) {
        mid.layout.dims[i] = md[i];
        mid.layout.stride[i] = stride;
        stride *= (int)md[i];
    }
    if (make_geom(&a->dw, &mid, t->dw_flt, t->dst, false, 0, dw) != TinyNN_SUCCESS)
        return false;
    *why = "packed filter size";
    if (!conv_mfma_supported(*pw) || nr_elem(t->packed->layout) != conv_mfma_packed_bytes(*pw))
        return false;
    *why = "biases must be per channel, with the scale source scale * filter scale";
    for (const Tensor* b : {t->pw_bias, t->dw_bias}) {
        if (!b)
            continue;
        if (!(nr_elem(b->layout) == (size_t)oc && is_contiguous(b->layout) && aligned4(b->ptr)))
            return false;
        // ConvGeneral::IsAvailable, BareMetal/ConvKernel.cpp:37-42
        const ConvGeom& g = b == t->pw_bias ? *pw : *dw;
        const float d = g.s_src * g.s_flt - b->dtype.param.scale;
        if (!((d < 0 ? -d : d) < 1e-5f))
            return false;
    }
    *why = "shape, activation, alignment or extent the kernel does not take";
    return conv_pw_dw_supported(*pw, *dw, t->src->ptr, t->dst->ptr) && aligned16(t->packed->ptr) &&
           aligned4(t->dw_flt->ptr);
}

extern "C" int megcc_gfx950_pw_dw_supported(
        const MegccPwDwAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output) {
    ConvGeom pw, dw;
    PwDwOperands t;
    const char* why = "";
    return pw_dw_geom(attr, inputs, nr_input, outputs, nr_output, &pw, &dw, &t, &why) ? 1 : 0;
}

extern "C" TinyNNStatus megcc_gfx950_pw_dw(
        const MegccPwDwAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace*, const RuntimeOpt*) {
    ConvGeom pw, dw;
    PwDwOperands t;
    const char* why = "";
    MG_REQUIRE(pw_dw_geom(attr, inputs, nr_input, outputs, nr_output, &pw, &dw, &t, &why),
               TinyNN_ERROR_INVALID_LAYOUT, "pw_dw: %s", why);
    note_kernel("conv_pw_dw", pw.ic / 32, dw.sh);
    return conv_pw_dw_launch(
            pw, dw, t.src->ptr, t.packed->ptr, t.pw_bias ? t.pw_bias->ptr : nullptr, t.dw_flt->ptr,
            t.dw_bias ? t.dw_bias->ptr : nullptr, t.dst->ptr);
}
