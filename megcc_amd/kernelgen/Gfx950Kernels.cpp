// KernelFunc implementations of the gfx950 target: availability rules, kernel symbols and the
// emitted C shims. Symbol construction follows the reference's GetKernelSymbol() of the kernel
// its x86 (Arch::BAREMETAL) registry selects for the same context:
//   conv      BareMetal/ConvKernel.cpp:144-176 (ConvImpl), NCHW_NCHW44 detection :115-127
//   pooling   BareMetal/Pooling.cpp:31-44; NCHW44 qsi8 comes from GI with
//             "_<io>_fallback" appended (GeneralIntrinsic/PoolingKernel/QInt8PoolingNCHW44.cpp:25-31)
//   multitype BareMetal/ElemwiseMultiType.cpp:94-100
//   typecvt   GeneralIntrinsic/Typecvt.cpp:36-41 (q8<->f32, q8->q8), BareMetal/Typecvt.cpp:36-41
//   elemwise  BareMetal/ElemwiseKernel.cpp:433-439
//   reduce    BareMetal/Reduce.cpp:82-90
//   matmul    BareMetal/MatrixMul.cpp:26-41
//   resize    GeneralIntrinsic/Resize.cpp:25-33 (LINEAR), BareMetal/Resize.cpp:27-35 (NEAREST)
//   relayout  GeneralIntrinsic/Relayout.cpp:43-48 (first in the x86 list for 1/2/4-byte dtypes)
//   concat    BareMetal/Concat.cpp:14-22
// (for f32 conv / matmul / elemwise / reduce the x86 registry prefers GI variants whose names
// carry tiling details; the BAREMETAL template's name is used for those, and the run-time library
// also resolves the GI spellings.)
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <sstream>

#include "KernelGen.h"

namespace megcc_gfx950 {

#ifndef MEGCC_GFX950_IN_TREE
// ---- TContext mirror ---------------------------------------------------------------------------
static void missing(const std::string& k) {
    fprintf(stderr, "not find CCAttr %s\n", k.c_str());
    abort();  // TContext.h:224-231 aborts as well
}
std::string TContext::getAttrStr(const std::string& k) const {
    auto it = m_str.find(k);
    if (it == m_str.end())
        missing(k);
    return it->second;
}
int64_t TContext::get_int(const std::string& k) const {
    auto it = m_int.find(k);
    if (it == m_int.end())
        missing(k);
    return it->second;
}
CCOperand TContext::getAttrOprand(const std::string& k) const {
    auto it = m_op.find(k);
    if (it == m_op.end())
        missing(k);
    return it->second;
}

// KernelGen.cpp:130-153
static const char* kCall =
        "(Tensor** inputs, int nr_input, Tensor** outputs, int nr_output, "
        "const Workspace* workspace, const RuntimeOpt* opt)";
static const char* kInitCall =
        "(Tensor** inputs, int nr_input, Tensor* out_weights, int* nr_out_weight, "
        "const RuntimeOpt* opt)";
static const char* kWorkspaceCall =
        "(Tensor** inputs, int nr_input, int nr_thread, size_t* workspace)";

std::string KernelFuncBase::GetKernelSignature(TContext* c) const {
    return GetKernelSymbol(c) + kCall;
}
std::string KernelFuncBase::GetInitSignature(TContext* c) const {
    return GetInitSymbol(c) + kInitCall;
}
std::string KernelFuncBase::GetWorkspaceSignature(TContext* c) const {
    return GetWorkspaceSymbol(c) + kWorkspaceCall;
}
// defaults of KernelGen.h:97-124: no processed weights, no workspace
std::string KernelFuncBase::GetInitBody(TContext* c) const {
    return "TinyNNStatus " + GetInitSignature(c) +
           " {\n    if (nr_out_weight) *nr_out_weight = 0;\n    return TinyNN_SUCCESS;\n}\n";
}
std::string KernelFuncBase::GetWorkspaceBody(TContext* c) const {
    return "TinyNNStatus " + GetWorkspaceSignature(c) +
           " {\n    *workspace = 0;\n    return TinyNN_SUCCESS;\n}\n";
}
#endif

namespace {

static std::string split_body(bool conv) {
    return std::string(
        "    /* room for the split-K partial sums of problems with too few 128 x 128 tiles (64 x 256\n"
        "       for at most 64 rows) to fill the chip; the same formula as the library (gemm_f32.hip, gemm_split) */\n"
        "    long tiles = M <= 64 ? (N + 255) / 256 : ((M + 127) / 128) * ((N + 127) / 128), s = 1;\n"
        "    if (tiles < 192 && K >= 128) {\n"
        "        s = (") + (conv ? "512" : "(M <= 64 ? 256 : 512)") + std::string(" + tiles - 1) / tiles;\n"
        "        if (s > K / 64) s = K / 64;\n"
        "        if (s > 64) s = 64;\n"
        "        if (s < 2) s = 1;\n"
        "    }\n"
        "    *workspace = s > 1 ? (size_t)s * M * N * 4 : 0;\n"
        "    return TinyNN_SUCCESS;\n}\n");
}


// ---- dtype helpers (Utils/Utils.h:41-140, Utils/SymbolHelper.h:9-23) ---------------------------
std::string valid_dtype(const std::string& d) {
    size_t p = d.find('<');
    return p == std::string::npos ? d : d.substr(0, p);
}
bool is_q(const std::string& d, int bits) {
    return valid_dtype(d) == "qsi" + std::to_string(bits);
}
bool is_f32(const std::string& d) {
    return d == "f32";
}
std::string io_str(TContext* c) {
    std::string s;
    for (int i = 0; i < c->getAttrInt("nr_operands"); ++i)
        s += valid_dtype(c->getAttrOprand("operand:" + std::to_string(i)).dtype);
    return s;
}
size_t nr_elem(const CCOperand& o) {
    size_t n = o.shape.empty() ? 0 : 1;
    for (size_t d : o.shape)
        n *= d;
    return n;
}

const char* kHeader = "#include \"megcc_gfx950.h\"\n";

std::string kernel_def(const KernelFuncBase* k, TContext* c, const std::string& attr_decl,
                       const std::string& call) {
    std::stringstream ss;
    ss << "TinyNNStatus " << k->GetKernelSignature(c) << " {\n"
       << attr_decl << "    return " << call << ";\n}\n";
    return ss.str();
}

// ---- ConvBias ----------------------------------------------------------------------------------
// Common/ConvKernel.h:10-13 is_bias
bool conv_is_bias(TContext* c) {
    return c->getAttrInt("nr_operands") > 3 && !c->getAttrOprand("operand:2").shape.empty();
}
// BareMetal/ConvKernel.cpp:115-127 get_format
std::string conv_format(TContext* c) {
    std::string f = c->getAttrStr("format");
    if (f == "NCHW44" && c->getAttrOprand("operand:0").shape.size() == 4)
        return "NCHW_NCHW44";
    return f;
}
std::string conv_nonline(TContext* c) {
    return c->haveAttr("nonlineMode") ? c->getAttrStr("nonlineMode") : "IDENTITY";
}

struct ConvKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        const std::string fmt = conv_format(c), sparse = c->getAttrStr("sparse");
        if (!(fmt == "NCHW" || fmt == "NCHW44" || fmt == "NCHW_NCHW44") ||
            c->getAttrStr("mode") != "CROSS_CORRELATION" || c->getAttrInt("nr_operands") < 3)
            return false;
        const auto src = c->getAttrOprand("operand:0"), flt = c->getAttrOprand("operand:1");
        const auto op2 = c->getAttrOprand("operand:2");
        const bool f32 = is_f32(src.dtype) && is_f32(flt.dtype) && is_f32(op2.dtype);
        // the reference wants operand:2 to be qsi32, i.e. a qsi8 conv always has a bias
        // (BareMetal/ConvKernel.cpp:25-29), and |src*flt - bias scale| < 1e-5 (:37-42)
        bool q8 = is_q(src.dtype, 8) && is_q(flt.dtype, 8) && is_q(op2.dtype, 32);
        if (q8 && conv_is_bias(c))
            q8 = std::fabs(src.scale * flt.scale - op2.scale) < 1e-5;
        if (!(f32 || q8))
            return false;
        const std::string nl = conv_nonline(c);
        if (!(nl == "IDENTITY" || nl == "RELU" || nl == "H_SWISH" || nl == "SIGMOID"))
            return false;
        // bias must be per channel (Common/ConvKernel.h:15-30)
        if (conv_is_bias(c)) {
            const auto dst = c->getAttrOprand("operand:" + std::to_string(c->getAttrInt("nr_operands") - 1));
            size_t oc = dst.shape.size() == 5 ? dst.shape[1] * 4 : dst.shape[1];
            if (nr_elem(op2) != oc)
                return false;
        }
        if (sparse == "GROUP") {
            if (fmt == "NCHW_NCHW44")
                return false;
            // NCHW44 GROUP: channel-wise filters [G/4,1,1,FH,FW,4] only
            if (fmt == "NCHW44" && flt.shape.size() != 6)
                return false;
        } else if (sparse != "DENSE") {
            return false;
        }
        return true;
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)
            return "kernel_conv2d";
        std::stringstream ss;
        ss << "kernel_conv2d_" << c->getAttrUInt("kernel_h") << "x" << c->getAttrUInt("kernel_w")
           << "_" << conv_format(c) << "_" << c->getAttrStr("sparse") << "_p"
           << c->getAttrUInt("pad_h") << "x" << c->getAttrUInt("pad_w") << "_s"
           << c->getAttrUInt("stride_h") << "x" << c->getAttrUInt("stride_w") << "_d"
           << c->getAttrUInt("dilate_h") << "x" << c->getAttrUInt("dilate_w") << "_" << io_str(c);
        if (conv_is_bias(c))
            ss << "_bias";
        if (conv_nonline(c) != "IDENTITY")
            ss << "_" << conv_nonline(c);
        return ss.str();
    }
    std::string attr_decl(TContext* c) const {
        const std::string fmt = conv_format(c);
        std::stringstream ss;
        ss << "    static const MegccConvAttr attr = {" << c->getAttrUInt("kernel_h") << ", "
           << c->getAttrUInt("kernel_w") << ", " << c->getAttrUInt("stride_h") << ", "
           << c->getAttrUInt("stride_w") << ", " << c->getAttrUInt("pad_h") << ", "
           << c->getAttrUInt("pad_w") << ", " << c->getAttrUInt("dilate_h") << ", "
           << c->getAttrUInt("dilate_w") << ", MEGCC_FMT_" << fmt << ", MEGCC_SPARSE_"
           << c->getAttrStr("sparse") << ", MEGCC_NONLINE_" << conv_nonline(c) << ", "
           << (conv_is_bias(c) ? 1 : 0) << "};\n";
        return ss.str();
    }
    std::string GetKernelBody(TContext* c) const override {
        return kHeader + kernel_def(this, c, attr_decl(c),
                                    "megcc_gfx950_conv2d(&attr, inputs, nr_input, outputs, "
                                    "nr_output, workspace, opt)");
    }
    // the filter repack for the MFMA kernel happens at model load through the 3-phase protocol
    std::string GetInitBody(TContext* c) const override {
        return "TinyNNStatus " + GetInitSignature(c) + " {\n" + attr_decl(c) +
               "    return megcc_gfx950_conv2d_init(&attr, inputs, nr_input, out_weights, "
               "nr_out_weight, opt);\n}\n";
    }
    // plain C, no external call: the compiler may evaluate it at compile time
    // (compiler/lib/KernelGen/Jit/JitExe.cpp:67-123 forbids externs in workspace bodies).
    // Quantized kernels need none (im2col stays in LDS); the f32 implicit GEMM may split K.
    std::string GetWorkspaceBody(TContext* c) const override {
        const bool f32 = is_f32(c->getAttrOprand("operand:0").dtype);
        const std::string fmt = conv_format(c);
        const bool dense = c->getAttrStr("sparse") == "DENSE";
        const unsigned taps = c->getAttrUInt("kernel_h") * c->getAttrUInt("kernel_w");
        const bool q8_mfma = !f32 && dense && (fmt == "NCHW44" || fmt == "NCHW") && taps <= 9;
        if (!f32 && !dense && fmt == "NCHW") {
            // channel-wise on plain NCHW: NCHW44 copies of input, output and filter (conv_api.hip)
            std::stringstream ss;
            ss << "TinyNNStatus " << GetWorkspaceSignature(c) << " {\n"
               << "    const Layout src = inputs[0]->layout, flt = inputs[1]->layout;\n"
               << "    const long eh = " << c->getAttrUInt("dilate_h") << " * (" << c->getAttrUInt("kernel_h")
               << " - 1) + 1, ew = " << c->getAttrUInt("dilate_w") << " * (" << c->getAttrUInt("kernel_w")
               << " - 1) + 1;\n"
               << "    const long ih = src.dims[2] + 2 * " << c->getAttrUInt("pad_h")
               << ", iw = src.dims[3] + 2 * " << c->getAttrUInt("pad_w") << ";\n"
               << "    const long oh = ih >= eh ? (ih - eh) / " << c->getAttrUInt("stride_h")
               << " + 1 : 0, ow = iw >= ew ? (iw - ew) / " << c->getAttrUInt("stride_w") << " + 1 : 0;\n"
               << "    const long n = src.dims[0], ch = src.dims[1];\n"
               << "    const long in = n * ch * src.dims[2] * src.dims[3], out = n * ch * oh * ow;\n"
               << "    *workspace = 0;\n"
               << "    /* one output channel per input channel, a multiple of 4 of them */\n"
               << "    if (flt.nr_dim == 5 && flt.dims[0] == ch && flt.dims[1] == 1 && flt.dims[2] == 1 && (ch & 3) == 0 &&\n"
               << "        in < (1L << 31) && out < (1L << 31))\n"
               << "        *workspace = ((size_t)(in + 255) & ~(size_t)255) + ((size_t)(out + 255) & ~(size_t)255) + (size_t)ch * "
               << taps << ";\n"
               << "    return TinyNN_SUCCESS;\n}\n";
            return ss.str();
        }
        if (f32 && fmt == "NCHW44" && dense) {
            // f32 dense NCHW44 runs as relayout -> NCHW implicit GEMM -> relayout (conv_api.hip): the
            // GEMM's split-K room, then NCHW copies of input, output and filter
            std::stringstream ss;
            ss << "TinyNNStatus " << GetWorkspaceSignature(c) << " {\n"
               << "    const Layout src = inputs[0]->layout, flt = inputs[1]->layout;\n"
               << "    const long eh = " << c->getAttrUInt("dilate_h") << " * (" << c->getAttrUInt("kernel_h")
               << " - 1) + 1, ew = " << c->getAttrUInt("dilate_w") << " * (" << c->getAttrUInt("kernel_w")
               << " - 1) + 1;\n"
               << "    const long ih = src.dims[2] + 2 * " << c->getAttrUInt("pad_h")
               << ", iw = src.dims[3] + 2 * " << c->getAttrUInt("pad_w") << ";\n"
               << "    const long oh = ih >= eh ? (ih - eh) / " << c->getAttrUInt("stride_h")
               << " + 1 : 0, ow = iw >= ew ? (iw - ew) / " << c->getAttrUInt("stride_w") << " + 1 : 0;\n"
               << "    const long ic = (long)src.dims[1] * 4, oc = (long)flt.dims[0] * 4;\n"
               << "    const long M = oc, N = (long)src.dims[0] * oh * ow, K = ic * " << taps << ";\n"
               << "    long tiles = M <= 64 ? (N + 255) / 256 : ((M + 127) / 128) * ((N + 127) / 128), s = 1;\n"
               << "    if (tiles < 192 && K >= 128) {\n"
               << "        s = (512 + tiles - 1) / tiles;\n"
               << "        if (s > K / 64) s = K / 64;\n"
               << "        if (s > 64) s = 64;\n"
               << "        if (s < 2) s = 1;\n"
               << "    }\n"
               << "    *workspace = 0;\n"
               << "    if (N < (1L << 31) && K < (1L << 31))\n"
               << "        *workspace = (((s > 1 ? (size_t)s * M * N * 4 : 0) + 255) & ~(size_t)255) +\n"
               << "                     (((size_t)src.dims[0] * ic * src.dims[2] * src.dims[3] * 4 + 255) & ~(size_t)255) +\n"
               << "                     (((size_t)N * oc * 4 + 255) & ~(size_t)255) +\n"
               << "                     (((size_t)oc * K * 4 + 255) & ~(size_t)255);\n"
               << "    return TinyNN_SUCCESS;\n}\n";
            return ss.str();
        }
        if (!(f32 && fmt == "NCHW" && dense) && !q8_mfma)
            return "TinyNNStatus " + GetWorkspaceSignature(c) +
                   " {\n    *workspace = 0;\n    return TinyNN_SUCCESS;\n}\n";
        std::stringstream ss;
        ss << "TinyNNStatus " << GetWorkspaceSignature(c) << " {\n"
           << "    const Layout src = inputs[0]->layout, flt = inputs[1]->layout;\n"
           << "    const long eh = " << c->getAttrUInt("dilate_h") << " * (" << c->getAttrUInt("kernel_h")
           << " - 1) + 1, ew = " << c->getAttrUInt("dilate_w") << " * (" << c->getAttrUInt("kernel_w")
           << " - 1) + 1;\n"
           << "    const long ih = src.dims[2] + 2 * " << c->getAttrUInt("pad_h")
           << ", iw = src.dims[3] + 2 * " << c->getAttrUInt("pad_w") << ";\n"
           << "    const long oh = ih >= eh ? (ih - eh) / " << c->getAttrUInt("stride_h")
           << " + 1 : 0, ow = iw >= ew ? (iw - ew) / " << c->getAttrUInt("stride_w") << " + 1 : 0;\n"
           ;
        if (f32) {
            ss << "    const long M = flt.dims[0], N = (long)src.dims[0] * oh * ow, K = (long)src.dims[1] * "
               << c->getAttrUInt("kernel_h") << " * " << c->getAttrUInt("kernel_w") << ";\n"
               << split_body(true);
            return ss.str();
        }
        // qsi8 dense / FullyConnected: split-K partial sums of the one-stage MFMA kernel
        // (conv_mfma_i8.hip, conv_mfma_split); it covers NCHW44 and the 1x1 NCHW on [M,K,1,1]
        const int r = fmt == "NCHW44" ? 4 : 1;
        const int ks = taps <= 2 ? 4 : taps <= 4 ? 2 : 1;
        ss << "    const long P = (long)src.dims[0] * oh * ow, oc = (long)flt.dims[0] * " << r
           << ", ic = (long)src.dims[1] * " << r << ";\n";
        // NCHW with spatial extent runs as relayout -> NCHW44 kernel -> relayout (conv_api.hip): both
        // NCHW44 copies live in the workspace, after the split-K room, their channel counts padded to
        // a multiple of 4 (then the bias gets a padded copy too)
        if (fmt == "NCHW")
            ss << "    const int spatial = !(src.dims[2] == 1 && src.dims[3] == 1 && " << taps << " == 1);\n"
               << "    const long icp = spatial ? (ic + 3) & ~3L : ic, ocp = spatial ? (oc + 3) & ~3L : oc;\n";
        else
            ss << "    const long icp = ic, ocp = oc;\n";
        ss << "    *workspace = 0;\n"
           << "    if ((icp & 3) == 0 && P > 0) {\n"
           << "        const long stages = ((icp + 31) / 32 + " << ks - 1 << ") / " << ks << ";\n"
           << "        const long bm = ocp <= 64 || ((P + 127) / 128) * ((ocp + 127) / 128) < 64 ? 64 : 128;\n"
           << "        const long tiles = ((P + 127) / 128) * ((ocp + bm - 1) / bm);\n"
           << "        long s = 1;\n"
           << "        if (tiles < 128 && stages >= 2) {\n"
           << "            s = (512 + tiles - 1) / tiles;\n"
           << "            if (s > stages) s = stages;\n"
           << "            if (s > 16) s = 16;\n"
           << "        }\n"
           << "        if (s > 1) *workspace = (size_t)s * P * ((ocp + 3) & ~3L) * 4;\n";
        // a strided 1x1 convolution first gathers the pixels it keeps (conv_api.hip)
        if (fmt == "NCHW44" && taps == 1 && c->getAttrUInt("pad_h") == 0 && c->getAttrUInt("pad_w") == 0 &&
            (c->getAttrUInt("stride_h") > 1 || c->getAttrUInt("stride_w") > 1))
            ss << "        *workspace = ((*workspace + 255) & ~(size_t)255) + (size_t)P * ic;\n";
        if (fmt == "NCHW")
            ss << "        if (spatial)\n"
               << "            *workspace = ((*workspace + 255) & ~(size_t)255) +\n"
               << "                         (((size_t)src.dims[0] * icp * src.dims[2] * src.dims[3] + 255) & ~(size_t)255) +\n"
               << "                         (((size_t)P * ocp + 255) & ~(size_t)255) +\n"
               << "                         (ocp != oc ? (((size_t)ocp * 4 + 255) & ~(size_t)255) : 0);\n";
        ss << "    }\n"
           << "    return TinyNN_SUCCESS;\n}\n";
        return ss.str();
    }
};

// ---- Pooling -----------------------------------------------------------------------------------
struct PoolingKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        const std::string fmt = c->getAttrStr("format"), mode = c->getAttrStr("mode");
        const auto src = c->getAttrOprand("operand:0"), dst = c->getAttrOprand("operand:1");
        if (!(fmt == "NCHW" || fmt == "NCHW44"))
            return false;
        if (!(mode == "MAX" || mode == "AVERAGE" || mode == "AVERAGE_COUNT_EXCLUDE_PADDING"))
            return false;
        // "quant pooling only support same scale" (BareMetal/Pooling.cpp:22-27)
        return is_q(src.dtype, 8) && is_q(dst.dtype, 8) && src.scale == dst.scale;
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_pooling";
        std::stringstream ss;
        const bool f44 = c->getAttrStr("format") == "NCHW44";
        ss << (f44 ? "GI_" : "") << "kernel_pooling_" << c->getAttrStr("mode") << "_"
           << c->getAttrStr("format") << "_p" << c->getAttrInt("pad_h") << "x"
           << c->getAttrInt("pad_w") << "_s" << c->getAttrInt("stride_h") << "x"
           << c->getAttrInt("stride_w") << "_w" << c->getAttrInt("window_h") << "x"
           << c->getAttrInt("window_w") << "_" << io_str(c);
        if (f44)
            ss << "_" << io_str(c) << "_fallback";
        return ss.str();
    }
    std::string GetKernelBody(TContext* c) const override {
        std::stringstream a;
        a << "    static const MegccPoolAttr attr = {" << c->getAttrInt("window_h") << ", "
          << c->getAttrInt("window_w") << ", " << c->getAttrInt("stride_h") << ", "
          << c->getAttrInt("stride_w") << ", " << c->getAttrInt("pad_h") << ", "
          << c->getAttrInt("pad_w") << ", MEGCC_FMT_" << c->getAttrStr("format")
          << ", MEGCC_POOL_" << c->getAttrStr("mode") << "};\n";
        return kHeader + kernel_def(this, c, a.str(),
                                    "megcc_gfx950_pooling(&attr, inputs, nr_input, outputs, "
                                    "nr_output, workspace, opt)");
    }
};

// ---- ElemwiseMultiType -------------------------------------------------------------------------
struct ElemwiseMultiTypeKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        const std::string mode = c->getAttrStr("mode");
        const int n = c->getAttrInt("nr_operands");
        for (int i = 0; i < n; ++i)
            if (!is_q(c->getAttrOprand("operand:" + std::to_string(i)).dtype, 8))
                return false;
        if (n == 2)
            return mode == "QRELU";
        if (n != 3 || !(mode == "QADD" || mode == "QFUSE_ADD_RELU" || mode == "QMUL"))
            return false;
        // broadcast modes of BareMetal/ElemwiseMultiType.cpp:76-92
        const auto a = c->getAttrOprand("operand:0"), b = c->getAttrOprand("operand:1");
        const size_t nb = nr_elem(b);
        return a.shape == b.shape || nb == 1 ||
               (a.shape.size() == b.shape.size() && a.shape.size() > 2 &&
                a.shape[1] == b.shape[1] && nb == b.shape[1]);
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_elementwise_multitype";
        return "kernel_elementwise_multitype_" + c->getAttrStr("mode") + "_" + io_str(c);
    }
    std::string GetKernelBody(TContext* c) const override {
        std::string m = c->getAttrStr("mode").substr(1);  // QADD -> ADD
        return kHeader +
               kernel_def(this, c, "    static const MegccMultiTypeMode mode = MEGCC_Q_" + m + ";\n",
                          "megcc_gfx950_elemwise_multitype(&mode, inputs, nr_input, outputs, "
                          "nr_output, workspace, opt)");
    }
};

// ---- Elemwise (f32) ----------------------------------------------------------------------------
struct ElemwiseKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        static const char* unary[] = {"RELU", "EXP", "SIGMOID", "H_SWISH", "NEGATE"};
        static const char* binary[] = {"ADD", "SUB", "MUL", "TRUE_DIV", "MAX", "MIN", "FUSE_ADD_RELU"};
        const std::string mode = c->getAttrStr("mode");
        const int n = c->getAttrInt("nr_operands");
        for (int i = 0; i < n; ++i)
            if (!is_f32(c->getAttrOprand("operand:" + std::to_string(i)).dtype))
                return false;
        bool ok = false;
        if (n == 2)
            for (auto u : unary)
                ok |= mode == u;
        if (n == 3)
            for (auto b : binary)
                ok |= mode == b;
        return ok;
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_elementwise";
        return "kernel_elementwise_" + c->getAttrStr("mode") + "_" + io_str(c);
    }
    std::string GetKernelBody(TContext* c) const override {
        return kHeader + kernel_def(this, c,
                                    "    static const MegccElemwiseMode mode = MEGCC_EW_" +
                                            c->getAttrStr("mode") + ";\n",
                                    "megcc_gfx950_elemwise(&mode, inputs, nr_input, outputs, "
                                    "nr_output, workspace, opt)");
    }
};

// ---- TypeCvt -----------------------------------------------------------------------------------
struct TypeCvtKernel : KernelFuncBase {
    static std::string pair(TContext* c) {
        return valid_dtype(c->getAttrOprand("operand:0").dtype) +
               valid_dtype(c->getAttrOprand("operand:1").dtype);
    }
    bool IsAvailable(TContext* c) const override {
        const std::string p = pair(c);
        if (!(p == "f32qsi8" || p == "qsi8f32" || p == "qsi8qsi8" || p == "qsi32qsi8"))
            return false;
        const auto s = c->getAttrOprand("operand:0"), d = c->getAttrOprand("operand:1");
        return (is_f32(s.dtype) || s.scale > 0) && (is_f32(d.dtype) || d.scale > 0);
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_typecvt";
        const std::string p = pair(c);
        return std::string(p == "qsi32qsi8" ? "" : "GI_") + "kernel_typecvt_" + p;
    }
    std::string GetKernelBody(TContext* c) const override {
        return kHeader + kernel_def(this, c, "",
                                    "megcc_gfx950_typecvt(inputs, nr_input, outputs, nr_output, "
                                    "workspace, opt)");
    }
};

// ---- Reduce (f32) ------------------------------------------------------------------------------
struct ReduceKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        const std::string mode = c->getAttrStr("mode");
        return c->getAttrStr("data_type") == "DEFAULT" &&
               is_f32(c->getAttrOprand("operand:0").dtype) &&
               (mode == "SUM" || mode == "MEAN" || mode == "MAX" || mode == "MIN" ||
                mode == "PRODUCT" || mode == "SUM_SQR");
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_reduce";
        std::stringstream ss;
        ss << "kernel_reduce_" << c->getAttrStr("mode") << "_" << c->getAttrStr("data_type")
           << "_a" << c->getAttrInt("axis") << "_" << io_str(c);
        return ss.str();
    }
    std::string GetKernelBody(TContext* c) const override {
        std::stringstream a;
        a << "    static const MegccReduceAttr attr = {MEGCC_REDUCE_" << c->getAttrStr("mode")
          << ", " << c->getAttrInt("axis") << "};\n";
        return kHeader + kernel_def(this, c, a.str(),
                                    "megcc_gfx950_reduce(&attr, inputs, nr_input, outputs, "
                                    "nr_output, workspace, opt)");
    }
};

// ---- Relayout / Concat (dtypes of 1, 2 and 4 bytes) --------------------------------------------
// Utils/Utils.h:41-84 get_dtype_size
int dtype_bytes(const std::string& d) {
    const std::string v = valid_dtype(d);
    if (v == "f32" || v == "i32" || v == "qsi32")
        return 4;
    if (v == "f16" || v == "i16" || v == "ui16")
        return 2;
    if (v == "i8" || v == "si8" || v == "ui8" || v == "qsi8")
        return 1;
    return 0;
}

struct RelayoutKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        const std::string d = c->getAttrOprand("operand:0").dtype;
        return dtype_bytes(d) != 0 && d == c->getAttrOprand("operand:1").dtype;
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "GI_kernel_relayout";
        return "GI_kernel_relayout_" + valid_dtype(c->getAttrOprand("operand:0").dtype);
    }
    std::string GetKernelBody(TContext* c) const override {
        return kHeader + kernel_def(this, c, "",
                                    "megcc_gfx950_relayout(inputs, nr_input, outputs, nr_output, "
                                    "workspace, opt)");
    }
};

struct ConcatKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        return dtype_bytes(c->getAttrOprand("operand:0").dtype) != 0 && c->getAttrInt("axis") >= 0;
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_concat";
        std::stringstream ss;
        ss << "kernel_concat_byte_" << dtype_bytes(c->getAttrOprand("operand:0").dtype) << "_axis_"
           << c->getAttrInt("axis");
        return ss.str();
    }
    std::string GetKernelBody(TContext* c) const override {
        std::stringstream a;
        a << "    static const int axis = " << c->getAttrInt("axis") << ";\n";
        return kHeader + kernel_def(this, c, a.str(),
                                    "megcc_gfx950_concat(&axis, inputs, nr_input, outputs, "
                                    "nr_output, workspace, opt)");
    }
};

// ---- Resize (f32; GeneralIntrinsic/Resize.cpp:13-33 for LINEAR, BareMetal/Resize.cpp:15-35) ----
struct ResizeKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        const std::string imode = c->getAttrStr("imode"), fmt = c->getAttrStr("format");
        return is_f32(c->getAttrOprand("operand:0").dtype) &&
               ((imode == "LINEAR" && (fmt == "NCHW" || fmt == "NCHW44")) ||
                (imode == "NEAREST" && fmt == "NCHW"));
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_resize_linear";
        const std::string imode = c->getAttrStr("imode");
        return std::string(imode == "LINEAR" ? "GI_" : "") + "kernel_resize_linear_" +
               c->getAttrStr("format") + "_" + imode + "_" + c->getAttrOprand("operand:0").dtype;
    }
    std::string GetKernelBody(TContext* c) const override {
        std::stringstream a;
        a << "    static const MegccResizeAttr attr = {MEGCC_FMT_" << c->getAttrStr("format")
          << ", MEGCC_IMODE_" << c->getAttrStr("imode") << "};\n";
        return kHeader + kernel_def(this, c, a.str(),
                                    "megcc_gfx950_resize(&attr, inputs, nr_input, outputs, "
                                    "nr_output, workspace, opt)");
    }
};

// ---- FusedElemwise (f32): the chain "modes:<i>" = "<operands...>,<MODE>,<result>" becomes a
// constant MegccFusedElemwiseAttr in the shim (names I<k> / O<j> resolved to value numbers). The
// symbol follows BareMetal/FusedElemwiseKernel.cpp:293-317; like the reference's it names only
// modes and operand kinds, so - unlike every other operator - the library cannot rebuild the attr
// from it: the shim is the only carrier.
struct FusedElemwiseKernel : KernelFuncBase {
    static std::vector<std::string> split(const std::string& s) {
        std::vector<std::string> out;
        std::stringstream ss(s);
        std::string item;
        while (std::getline(ss, item, ','))
            out.push_back(item);
        return out;
    }
    static const char* mode_enum(const std::string& m) {
        static const char* const known[] = {
                "RELU", "EXP", "SIGMOID", "H_SWISH", "NEGATE", "ABS", "LOG", "SILU", "ROUND", "ADD",
                "SUB", "MUL", "TRUE_DIV", "MAX", "MIN", "FUSE_ADD_RELU", "LT", "LEQ", "EQ",
                "FLOOR_DIV", "FUSE_ADD_SIGMOID", "FUSE_ADD_TANH", "FUSE_MUL_ADD3", "FUSE_MUL_ADD4"};
        for (const char* k : known)
            if (m == k)
                return k;
        return nullptr;
    }
    // 0 VECTOR, 1 SCALAR, 2 BCAST101, 3 BCAST101xX, 4 unknown (Common/ElemwiseCommon.cpp:7-45)
    static int tensor_type(const CCOperand& dst, const CCOperand& op) {
        size_t n = 1, m = 1;
        for (size_t d : dst.shape)
            n *= d;
        for (size_t d : op.shape)
            m *= d;
        if (n == m)
            return 0;
        if (m == 1)
            return 1;
        const auto& s = op.shape;
        if (dst.shape.size() >= 4 && s.size() == 4 && s[0] == 1 && s[2] == 1 && s[3] == 1)
            return 2;
        if (dst.shape.size() >= 4 && s.size() == 5 && s[0] == 1 && s[2] == 1 && s[3] == 1 && s[4] == 4)
            return 3;
        return 4;
    }
    bool IsAvailable(TContext* c) const override {
        const int steps = c->getAttrInt("modes:size"), nr = c->getAttrInt("nr_operands");
        if (steps < 1 || steps > 16 || nr < 2 || nr > 9)
            return false;
        const CCOperand dst = c->getAttrOprand("operand:" + std::to_string(nr - 1));
        for (int i = 0; i < nr; ++i) {
            const CCOperand op = c->getAttrOprand("operand:" + std::to_string(i));
            if (!is_f32(op.dtype) || tensor_type(dst, op) == 4)
                return false;
        }
        for (int j = 0; j < steps; ++j) {
            const auto parts = split(c->getAttrStr("modes:" + std::to_string(j)));
            if (parts.size() < 3 || parts.size() > 6 || !mode_enum(parts[parts.size() - 2]))
                return false;
            for (size_t a = 0; a + 2 < parts.size(); ++a) {
                const std::string& nm = parts[a];
                if (nm.size() < 2 || (nm[0] != 'I' && nm[0] != 'O'))
                    return false;
                const int k = std::atoi(nm.c_str() + 1);
                if ((nm[0] == 'I' && k >= nr - 1) || (nm[0] == 'O' && k >= j))
                    return false;
            }
        }
        return true;
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_fused_elemwise";
        const int steps = c->getAttrInt("modes:size"), nr = c->getAttrInt("nr_operands");
        const CCOperand dst = c->getAttrOprand("operand:" + std::to_string(nr - 1));
        std::stringstream ss;
        ss << "kernel_naive_fused_elementwise";
        for (int j = 0; j < steps; ++j) {
            const auto parts = split(c->getAttrStr("modes:" + std::to_string(j)));
            ss << "_" << parts[parts.size() - 2];
        }
        for (int i = 0; i < nr; ++i)
            ss << "_tensortype" << tensor_type(dst, c->getAttrOprand("operand:" + std::to_string(i)));
        ss << "_";
        for (int i = 0; i < nr; ++i)
            ss << valid_dtype(c->getAttrOprand("operand:" + std::to_string(i)).dtype);
        return ss.str();
    }
    std::string GetKernelBody(TContext* c) const override {
        const int steps = c->getAttrInt("modes:size"), nr_in = c->getAttrInt("nr_operands") - 1;
        std::stringstream a;
        a << "    static const MegccFusedElemwiseAttr attr = {" << nr_in << ", " << steps << ", {\n";
        for (int j = 0; j < steps; ++j) {
            const auto parts = split(c->getAttrStr("modes:" + std::to_string(j)));
            const size_t n = parts.size() - 2;
            a << "        {MEGCC_EW_" << parts[n] << ", " << n << ", {";
            for (size_t k = 0; k < 4; ++k) {
                int v = 0;
                if (k < n)
                    v = std::atoi(parts[k].c_str() + 1) + (parts[k][0] == 'O' ? nr_in : 0);
                a << v << (k < 3 ? ", " : "");
            }
            a << "}},\n";
        }
        a << "    }};\n";
        return kHeader + kernel_def(this, c, a.str(),
                                    "megcc_gfx950_fused_elemwise(&attr, inputs, nr_input, outputs, "
                                    "nr_output, workspace, opt)");
    }
};

// ---- MatrixMul (f32) ---------------------------------------------------------------------------
struct MatrixMulKernel : KernelFuncBase {
    bool IsAvailable(TContext* c) const override {
        for (int i = 0; i < 3; ++i)
            if (!is_f32(c->getAttrOprand("operand:" + std::to_string(i)).dtype))
                return false;
        return c->getAttrStr("format") == "DEFAULT" &&
               (!c->haveAttr("compute_mode") || c->getAttrStr("compute_mode") == "DEFAULT");
    }
    std::string GetKernelSymbol(TContext* c) const override {
        if (!c)  // name filtering without a context (KernelGen.cpp:49-53)
            return "kernel_matmul";
        return std::string("kernel_matmul_") + (c->getAttrBool("transposeA") ? "t" : "n") +
               (c->getAttrBool("transposeB") ? "t" : "n") + "_" +
               c->getAttrOprand("operand:0").dtype;
    }
    std::string GetKernelBody(TContext* c) const override {
        std::stringstream a;
        a << "    static const MegccMatMulAttr attr = {" << (c->getAttrBool("transposeA") ? 1 : 0)
          << ", " << (c->getAttrBool("transposeB") ? 1 : 0) << "};\n";
        return kHeader + kernel_def(this, c, a.str(),
                                    "megcc_gfx950_matmul(&attr, inputs, nr_input, outputs, "
                                    "nr_output, workspace, opt)");
    }
    std::string GetWorkspaceBody(TContext* c) const override {
        const bool ta = c->getAttrBool("transposeA"), tb = c->getAttrBool("transposeB");
        std::stringstream ss;
        ss << "TinyNNStatus " << GetWorkspaceSignature(c) << " {\n"
           << "    const Layout a = inputs[0]->layout, b = inputs[1]->layout;\n"
           << "    const long M = a.dims[" << (ta ? 1 : 0) << "], K = a.dims[" << (ta ? 0 : 1)
           << "], N = b.dims[" << (tb ? 0 : 1) << "];\n"
           << split_body(false);
        return ss.str();
    }
};

}  // namespace

std::vector<const KernelFuncBase*> Gfx950KernelPack::GetKernel(KernType type) {
    static const ConvKernel conv;
    static const PoolingKernel pool;
    static const ElemwiseMultiTypeKernel multitype;
    static const ElemwiseKernel elemwise;
    static const TypeCvtKernel typecvt;
    static const ReduceKernel reduce;
    static const MatrixMulKernel matmul;
    static const RelayoutKernel relayout;
    static const ConcatKernel concat;
    static const ResizeKernel resize;
    static const FusedElemwiseKernel fused;
    switch (type) {
        case KernType::ConvKernel: return {&conv};
        case KernType::PoolingKernel: return {&pool};
        case KernType::ElemwiseMultiKernel: return {&multitype};
        case KernType::ElemwiseKernel: return {&elemwise};
        case KernType::TypeCvtKernel: return {&typecvt};
        case KernType::ReduceKernel: return {&reduce};
        case KernType::MatrixMulKernel: return {&matmul};
        case KernType::RelayoutKernel: return {&relayout};
        case KernType::ConcatKernel: return {&concat};
        case KernType::ResizeKernel: return {&resize};
        case KernType::FusedElemwiseKernel: return {&fused};
        default: return {};
    }
}

std::string ReferenceSymbol(KernType type, TContext* context) {
    for (auto* k : Gfx950KernelPack::GetKernel(type))
        if (k->IsAvailable(context))
            return k->GetKernelSymbol(context);
    return "";
}

}  // namespace megcc_gfx950
