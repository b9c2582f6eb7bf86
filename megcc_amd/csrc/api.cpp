// Dispatch by the reference's generated kernel symbol. The symbol grammar is the one KernelGen
// builds in GetKernelSymbol():
//   conv     BareMetal/ConvKernel.cpp:144-176, GeneralIntrinsic/ConvKernel/Fp32Im2col.cpp:88-118
//   pooling  BareMetal/Pooling.cpp:31-44, GeneralIntrinsic/PoolingKernel/QInt8PoolingNCHW44.cpp:25-31
//   multitype BareMetal/ElemwiseMultiType.cpp:94-100
//   elemwise BareMetal/ElemwiseKernel.cpp:433-439 (GI_ variants carry extra suffixes)
//   typecvt  BareMetal/Typecvt.cpp:36-41, GeneralIntrinsic/Typecvt.cpp:36-41
//   reduce   BareMetal/Reduce.cpp:82-90, GeneralIntrinsic/Reduce.cpp:615-623
//   matmul   BareMetal/MatrixMul.cpp:26-41, GeneralIntrinsic/MatMulKernel (4x12, gevm)
#include <stdio.h>
#include <string.h>

#include <string>

#include "common.h"

using namespace mg;

namespace {

bool starts_with(const std::string& s, const char* p) {
    return s.compare(0, strlen(p), p) == 0;
}
bool ends_with(const std::string& s, const char* p) {
    size_t n = strlen(p);
    return s.size() >= n && s.compare(s.size() - n, n, p) == 0;
}
// removes prefix p from s if present
bool eat(std::string& s, const char* p) {
    if (!starts_with(s, p))
        return false;
    s.erase(0, strlen(p));
    return true;
}

bool parse_nonline(const std::string& s, MegccNonline* out) {
    if (s.empty() || s == "IDENTITY") {
        *out = MEGCC_NONLINE_IDENTITY;
    } else if (s == "RELU") {
        *out = MEGCC_NONLINE_RELU;
    } else if (s == "H_SWISH") {
        *out = MEGCC_NONLINE_H_SWISH;
    } else if (s == "SIGMOID") {
        *out = MEGCC_NONLINE_SIGMOID;
    } else {
        return false;
    }
    return true;
}

bool parse_conv(std::string s, MegccConvAttr* a) {
    // the names of the f32 NCHW44 kernels the reference picks (GeneralIntrinsic/ConvKernel):
    //   GI_kernel_conv2d_<k>x<k>_NCHW44_DENSE_p.._s.._d.._<io>[_bias][_NONLINE]_winograd_f23
    //       ... _winograd_f43_fp32 / _winograd_f63_fp32   (Fp32WinogradNchw44.cpp:83,157,231; F63
    //       is the registry's first choice for 3x3 stride 1, GeneralIntrinsic/KernelPack.cpp:54-56)
    //   GI_kernel_conv2d_conv1x1_NCHW44_1x1_DENSE_p.._s.._d..[_bias][_NONLINE]
    //   GI_kernel_conv2d_<k>x<k>_NCHW44_DENSE_..._<io>[_bias][_NONLINE]_nchw_nchw44_oc<n>_ic<n>
    //       (first layer: 4-dim source, 5-dim result; Fp32ConvNchwNchw44.cpp:37-55)
    //   GI_chanwise_kernel_conv2d_<k>x<k>_NCHW44_GROUP_..._<io>[_bias][_NONLINE]
    //       (ConvKernel.h:24-32,63-65)
    bool first_layer = false;
    for (const char* w : {"_winograd_f23", "_winograd_f43_fp32", "_winograd_f63_fp32"})
        if (ends_with(s, w)) {
            s.erase(s.size() - strlen(w));
            if (!eat(s, "GI_"))
                return false;
        }
    {
        const size_t at = s.rfind("_nchw_nchw44_oc");
        unsigned oc, ic;
        int used = 0;
        if (at != std::string::npos && sscanf(s.c_str() + at, "_nchw_nchw44_oc%u_ic%u%n", &oc, &ic, &used) == 2 &&
            at + used == s.size()) {
            s.erase(at);
            if (!eat(s, "GI_"))
                return false;
            first_layer = true;
        }
    }
    if (eat(s, "GI_chanwise_")) {
        if (s.find("_NCHW44_GROUP_") == std::string::npos)
            return false;
    }
    if (eat(s, "GI_kernel_conv2d_conv1x1_")) {
        const bool f44 = eat(s, "NCHW44_");
        if (!f44 && !eat(s, "NCHW_"))
            return false;
        if (!eat(s, "1x1_"))
            return false;
        s = std::string("kernel_conv2d_1x1_") + (f44 ? "NCHW44_" : "NCHW_") + s;
        // (no operand types in this name: put them where the common form has them)
        size_t d = s.find("_d");
        if (d == std::string::npos)
            return false;
        size_t e = s.find('_', d + 1);
        s.insert(e == std::string::npos ? s.size() : e, "_f32f32f32f32");
    }
    const bool gi = eat(s, "GI_kernel_conv2d_im2col_");
    if (!gi && !eat(s, "kernel_conv2d_"))
        return false;
    unsigned kh, kw;
    int used = 0;
    if (sscanf(s.c_str(), "%ux%u_%n", &kh, &kw, &used) != 2)
        return false;
    s.erase(0, used);
    if (eat(s, "NCHW_NCHW44_"))
        a->format = MEGCC_FMT_NCHW_NCHW44;
    else if (eat(s, "NCHW44_"))
        a->format = first_layer ? MEGCC_FMT_NCHW_NCHW44 : MEGCC_FMT_NCHW44;
    else if (eat(s, "NCHW_"))
        a->format = MEGCC_FMT_NCHW;
    else
        return false;
    if (first_layer && a->format != MEGCC_FMT_NCHW_NCHW44)
        return false;
    if (eat(s, "DENSE_"))
        a->sparse = MEGCC_SPARSE_DENSE;
    else if (eat(s, "GROUP_"))
        a->sparse = MEGCC_SPARSE_GROUP;
    else
        return false;
    unsigned ph, pw, sh, sw, dh, dw;
    if (sscanf(s.c_str(), "p%ux%u_s%ux%u_d%ux%u%n", &ph, &pw, &sh, &sw, &dh, &dw, &used) != 6)
        return false;
    s.erase(0, used);
    a->kernel_h = kh; a->kernel_w = kw;
    a->pad_h = ph; a->pad_w = pw;
    a->stride_h = sh; a->stride_w = sw;
    a->dilate_h = dh; a->dilate_w = dw;
    if (gi) {
        // "[_bias][_NONLINE]f32"
        if (!ends_with(s, "f32"))
            return false;
        s.erase(s.size() - 3);
    } else {
        // "_<io>[_bias][_NONLINE]"
        if (!eat(s, "_"))
            return false;
        size_t us = s.find('_');
        s.erase(0, us == std::string::npos ? s.size() : us);
    }
    a->with_bias = eat(s, "_bias") ? 1 : 0;
    if (!s.empty() && s[0] == '_')
        s.erase(0, 1);
    return parse_nonline(s, &a->nonline);
}

bool parse_pool(std::string s, MegccPoolAttr* a) {
    eat(s, "GI_");
    if (!eat(s, "kernel_pooling_"))
        return false;
    if (eat(s, "AVERAGE_COUNT_EXCLUDE_PADDING_"))
        a->mode = MEGCC_POOL_AVERAGE_COUNT_EXCLUDE_PADDING;
    else if (eat(s, "AVERAGE_"))
        a->mode = MEGCC_POOL_AVERAGE;
    else if (eat(s, "MAX_"))
        a->mode = MEGCC_POOL_MAX;
    else
        return false;
    if (eat(s, "NCHW44_"))
        a->format = MEGCC_FMT_NCHW44;
    else if (eat(s, "NCHW_"))
        a->format = MEGCC_FMT_NCHW;
    else
        return false;
    unsigned ph, pw, sh, sw, wh, ww;
    if (sscanf(s.c_str(), "p%ux%u_s%ux%u_w%ux%u", &ph, &pw, &sh, &sw, &wh, &ww) != 6)
        return false;
    a->pad_h = ph; a->pad_w = pw;
    a->stride_h = sh; a->stride_w = sw;
    a->window_h = wh; a->window_w = ww;
    return true;
}

struct ModeName {
    const char* name;
    int value;
};

// longest names first so that e.g. FUSE_ADD_RELU is not read as a prefix of something shorter
const ModeName kElemwise[] = {
        {"FUSE_ADD_RELU", MEGCC_EW_FUSE_ADD_RELU}, {"TRUE_DIV", MEGCC_EW_TRUE_DIV},
        {"H_SWISH", MEGCC_EW_H_SWISH},             {"SIGMOID", MEGCC_EW_SIGMOID},
        {"NEGATE", MEGCC_EW_NEGATE},               {"RELU", MEGCC_EW_RELU},
        {"EXP", MEGCC_EW_EXP},                     {"ADD", MEGCC_EW_ADD},
        {"SUB", MEGCC_EW_SUB},                     {"MUL", MEGCC_EW_MUL},
        {"MAX", MEGCC_EW_MAX},                     {"MIN", MEGCC_EW_MIN},
};
const ModeName kMultiType[] = {
        {"QFUSE_ADD_RELU", MEGCC_Q_FUSE_ADD_RELU},
        {"QADD", MEGCC_Q_ADD},
        {"QMUL", MEGCC_Q_MUL},
        {"QRELU", MEGCC_Q_RELU},
};
const ModeName kReduce[] = {
        {"SUM_SQR", MEGCC_REDUCE_SUM_SQR},
        {"PRODUCT", MEGCC_REDUCE_PRODUCT},
        {"SUM", MEGCC_REDUCE_SUM},
        {"MEAN", MEGCC_REDUCE_MEAN},
        {"MAX", MEGCC_REDUCE_MAX},
        {"MIN", MEGCC_REDUCE_MIN},
};

template <size_t N>
bool eat_mode(std::string& s, const ModeName (&table)[N], int* value) {
    for (size_t i = 0; i < N; ++i) {
        std::string key = std::string(table[i].name) + "_";
        if (starts_with(s, key.c_str())) {
            s.erase(0, key.size());
            *value = table[i].value;
            return true;
        }
    }
    return false;
}

}  // namespace

extern "C" TinyNNStatus megcc_gfx950_parse_symbol(const char* symbol, MegccKernelDesc* desc) {
    MG_REQUIRE(symbol && desc, TinyNN_ERROR_NULL_PTR, "parse_symbol: NULL argument");
    memset(desc, 0, sizeof(*desc));
    std::string s(symbol);
    int v = 0;
    if (starts_with(s, "kernel_conv2d_") || starts_with(s, "GI_kernel_conv2d_") ||
        starts_with(s, "GI_chanwise_kernel_conv2d_")) {
        if (parse_conv(s, &desc->attr.conv)) {
            desc->kind = MEGCC_KERN_CONV;
            return TinyNN_SUCCESS;
        }
    } else if (starts_with(s, "kernel_pooling_") || starts_with(s, "GI_kernel_pooling_")) {
        if (parse_pool(s, &desc->attr.pool)) {
            desc->kind = MEGCC_KERN_POOLING;
            return TinyNN_SUCCESS;
        }
    } else if (eat(s, "kernel_elementwise_multitype_")) {
        if (eat_mode(s, kMultiType, &v)) {
            desc->kind = MEGCC_KERN_ELEMWISE_MULTITYPE;
            desc->attr.multitype = (MegccMultiTypeMode)v;
            return TinyNN_SUCCESS;
        }
    } else if (eat(s, "GI_kernel_elementwise_") || eat(s, "kernel_elementwise_")) {
        if (eat_mode(s, kElemwise, &v) && s.find("f32") != std::string::npos) {
            desc->kind = MEGCC_KERN_ELEMWISE;
            desc->attr.elemwise = (MegccElemwiseMode)v;
            return TinyNN_SUCCESS;
        }
    } else if (eat(s, "GI_kernel_typecvt_") || eat(s, "kernel_typecvt_")) {
        if (s == "f32qsi8" || s == "qsi8f32" || s == "qsi8qsi8" || s == "qsi32qsi8") {
            desc->kind = MEGCC_KERN_TYPECVT;
            return TinyNN_SUCCESS;
        }
    } else if (eat(s, "GI_kernel_reduce_") || eat(s, "kernel_reduce_")) {
        // GI: <MODE>_<data_type>_<dtype>_a<axis>   BareMetal: <MODE>_<data_type>_a<axis>_<io>
        if (eat_mode(s, kReduce, &v)) {
            size_t p = s.find("_a");
            int axis = -1;
            if (p != std::string::npos && sscanf(s.c_str() + p, "_a%d", &axis) == 1 && axis >= 0 &&
                s.find("f32") != std::string::npos) {
                desc->kind = MEGCC_KERN_REDUCE;
                desc->attr.reduce.mode = (MegccReduceMode)v;
                desc->attr.reduce.axis = axis;
                return TinyNN_SUCCESS;
            }
        }
    } else if (eat(s, "GI_kernel_relayout_") || eat(s, "kernel_relayout_")) {
        if (s == "f32" || s == "qsi8" || s == "si8" || s == "i8" || s == "ui8" || s == "qsi32" ||
            s == "i32" || s == "i16" || s == "ui16" || s == "f16") {
            desc->kind = MEGCC_KERN_RELAYOUT;
            return TinyNN_SUCCESS;
        }
    } else if (eat(s, "GI_kernel_resize_linear_") || eat(s, "kernel_resize_linear_")) {
        // <format>_<imode>_f32
        const bool p4 = eat(s, "NCHW44_");
        if (p4 || eat(s, "NCHW_")) {
            const bool linear = eat(s, "LINEAR_");
            if ((linear || (!p4 && eat(s, "NEAREST_"))) && s == "f32") {
                desc->kind = MEGCC_KERN_RESIZE;
                desc->attr.resize.format = p4 ? MEGCC_FMT_NCHW44 : MEGCC_FMT_NCHW;
                desc->attr.resize.imode = linear ? MEGCC_IMODE_LINEAR : MEGCC_IMODE_NEAREST;
                return TinyNN_SUCCESS;
            }
        }
    } else if (eat(s, "kernel_concat_byte_")) {
        int bytes = 0, axis = -1;
        char tail = 0;
        if (sscanf(s.c_str(), "%d_axis_%d%c", &bytes, &axis, &tail) == 2 &&
            (bytes == 1 || bytes == 2 || bytes == 4) && axis >= 0 && axis < MAX_DIM) {
            desc->kind = MEGCC_KERN_CONCAT;
            desc->attr.concat_axis = axis;
            return TinyNN_SUCCESS;
        }
    } else if (eat(s, "GI_kernel_fp32_matmul_4x12_") || eat(s, "GI_kernel_gevm_") ||
               eat(s, "GI_kernel_gemv_") || eat(s, "kernel_matmul_")) {
        if (s.size() >= 2 && (s[0] == 'n' || s[0] == 't') && (s[1] == 'n' || s[1] == 't') &&
            (s.size() == 2 || s.substr(2) == "_f32")) {
            desc->kind = MEGCC_KERN_MATMUL;
            desc->attr.matmul.transpose_a = s[0] == 't';
            desc->attr.matmul.transpose_b = s[1] == 't';
            return TinyNN_SUCCESS;
        }
    }
    return fail(TinyNN_ERROR_NO_FOUND, "parse_symbol: '%s' is not a kernel of this library", symbol);
}

extern "C" TinyNNStatus megcc_gfx950_call(
        const MegccKernelDesc* d, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* ws, const RuntimeOpt* opt) {
    MG_REQUIRE(d, TinyNN_ERROR_NULL_PTR, "call: NULL descriptor");
    switch (d->kind) {
        case MEGCC_KERN_CONV:
            return megcc_gfx950_conv2d(&d->attr.conv, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_MATMUL:
            return megcc_gfx950_matmul(&d->attr.matmul, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_POOLING:
            return megcc_gfx950_pooling(&d->attr.pool, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_ELEMWISE_MULTITYPE:
            return megcc_gfx950_elemwise_multitype(&d->attr.multitype, inputs, nr_input, outputs,
                                                   nr_output, ws, opt);
        case MEGCC_KERN_ELEMWISE:
            return megcc_gfx950_elemwise(&d->attr.elemwise, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_TYPECVT:
            return megcc_gfx950_typecvt(inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_REDUCE:
            return megcc_gfx950_reduce(&d->attr.reduce, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_RELAYOUT:
            return megcc_gfx950_relayout(inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_RESIZE:
            return megcc_gfx950_resize(&d->attr.resize, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_FUSED_ELEMWISE:
            return megcc_gfx950_fused_elemwise(&d->attr.fused, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_SOFTMAX:
            return megcc_gfx950_softmax(inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_DW_POOL_ADD:
            return megcc_gfx950_dw_pool_add(&d->attr.dw_pool_add, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_PW_DW:
            return megcc_gfx950_pw_dw(&d->attr.pw_dw, inputs, nr_input, outputs, nr_output, ws, opt);
        case MEGCC_KERN_CONCAT:
            return megcc_gfx950_concat(&d->attr.concat_axis, inputs, nr_input, outputs, nr_output,
                                       ws, opt);
        default:
            return fail(TinyNN_ERROR_NO_FOUND, "call: unknown kernel kind %d", (int)d->kind);
    }
}

extern "C" TinyNNStatus megcc_gfx950_call_init(
        const MegccKernelDesc* d, Tensor** inputs, int nr_input, Tensor* out_weights,
        int* nr_out_weight, const RuntimeOpt* opt) {
    MG_REQUIRE(d, TinyNN_ERROR_NULL_PTR, "call_init: NULL descriptor");
    if (d->kind == MEGCC_KERN_CONV)
        return megcc_gfx950_conv2d_init(&d->attr.conv, inputs, nr_input, out_weights, nr_out_weight, opt);
    // default InitFunc of the reference: no processed weights (KernelGen.h:97-106)
    if (nr_out_weight)
        *nr_out_weight = 0;
    return TinyNN_SUCCESS;
}

extern "C" TinyNNStatus megcc_gfx950_call_workspace(
        const MegccKernelDesc* d, Tensor** inputs, int nr_input, int nr_thread, size_t* workspace) {
    MG_REQUIRE(d && workspace, TinyNN_ERROR_NULL_PTR, "call_workspace: NULL argument");
    if (d->kind == MEGCC_KERN_CONV)
        return megcc_gfx950_conv2d_workspace(&d->attr.conv, inputs, nr_input, nr_thread, workspace);
    if (d->kind == MEGCC_KERN_MATMUL)
        return megcc_gfx950_matmul_workspace(&d->attr.matmul, inputs, nr_input, nr_thread, workspace);
    *workspace = 0;  // the other kernels of this library need no scratch memory
    return TinyNN_SUCCESS;
}
