/*
 * megcc_gfx950.h -- C ABI of libmegcc_gfx950.so: MI355X (gfx950) implementations of the
 * per-operator kernels MegCC's KernelGen emits and its TinyNN VM calls.
 *
 * Boundary being replaced (all citations relative to the MegCC tree):
 *   - every generated kernel has the uniform signature
 *         TinyNNStatus S(Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
 *                        const Workspace* workspace, const RuntimeOpt* opt);
 *     with companions S_init / S_workspace (runtime/src/data_struct.h:131-153, emitted by
 *     compiler/lib/KernelGen/KernelGen.cpp:130-153) and is called from execute_single_opr
 *     (runtime/src/vm/op.c:161-163) and init_model_weights (runtime/src/init.c:29-131).
 *   - everything that is *not* a run-time tensor (window, stride, padding, layout format,
 *     activation ...) is baked into the generated symbol S at compile time. Here those
 *     attributes travel in a small constant "attr" struct placed in front of the uniform
 *     argument list; the KernelGen target for this arch emits, per symbol S, a three-line C
 *     shim `S(...) { static const MegccConvAttr a = {...}; return megcc_gfx950_conv2d(&a, ...); }`.
 *
 * All Tensor.ptr / Workspace.ptr / out_weights->ptr are DEVICE pointers obtained through the
 * Device.malloc hook installed by megcc_gfx950_init_device(). Kernels are launched
 * asynchronously on one library-owned stream, in call order; results are visible to the host
 * after megcc_gfx950_wait() or a megcc_gfx950_memcpy_d2h().
 *
 * There is no CPU fallback anywhere in the library: an operator / layout / dtype combination that
 * has no gfx950 kernel returns TinyNN_ERROR_NO_IMPLEMENT.
 */
#ifndef MEGCC_GFX950_H
#define MEGCC_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Run-time ABI types. Field order, widths and enum values are those of
 * runtime/src/tinynn.h:7-54, runtime/src/device.h:8-21 and runtime/src/data_struct.h:12-59 so
 * that a Tensor built by the TinyNN runtime can be handed over unchanged. When the reference's
 * own data_struct.h has been included first, its definitions are used instead.
 * ---------------------------------------------------------------------------------------- */
#ifndef DATA_STRUCT_H

#define MAX_DIM (7)

typedef enum {
    TinyNN_SUCCESS = 0,
    TinyNN_ERROR_NULL_PTR = 1,
    TinyNN_ERROR_STANDER = 2,
    TinyNN_ERROR_RUNTIME = 3,
    TinyNN_ERROR_OUT_OF_RANGE = 4,
    TinyNN_ERROR_NO_FOUND = 5,
    TinyNN_ERROR_NO_IMPLEMENT = 6,
    TinyNN_ERROR_MODEL_PARSE = 7,
    TinyNN_ERROR_OPEN_FILE_ERROR = 8,
    TinyNN_ERROR_MEMORY_MALLOC = 9,
    TinyNN_ERROR_UNSUPPORTED_INSTRUCTION_TYPE = 10,
    TinyNN_ERROR_UNSUPPORTED_DTYPE_TYPE = 11,
    TinyNN_ERROR_INVALID_LAYOUT = 12,
    TinyNN_ERROR = 13
} TinyNNStatus;

typedef enum {
    TinyNN_FLOAT = 0,
    TinyNN_FLOAT16 = 1,
    TinyNN_INT = 2,
    TinyNN_INT8 = 3,
    TinyNN_INT16 = 4,
    TinyNN_UINT8 = 5,
    TinyNN_QINT8 = 100,
    TinyNN_QINT32 = 101,
    TinyNN_QUINT8 = 102
} TinyNNDType;

typedef enum { TinyNN_NCHW = 0, TinyNN_NHWC, TinyNN_NCHW4, TinyNN_NCHW8, TinyNN_OIHW } TinyNNFormat;

typedef enum {
    TinyNN_BARE_METAL = 0,
    TinyNN_ARM64,
    TinyNN_ARM32,
    TinyNN_ARM64_V82,
    TinyNN_ARM32_V82,
    TinyNN_OPENCL_MALI,
    TinyNN_WEB_ASSEMBLY
} TinyNNDevice;

typedef struct {
    int alignment;
    TinyNNDevice device_type;
    void* (*malloc)(size_t length);
    void (*free)(void* ptr);
} Device;

typedef struct RuntimeOpt {
    const Device* device;
} RuntimeOpt;

typedef struct {
    float scale;
    uint8_t zero_point;
} DTypeParam;

typedef struct {
    TinyNNDType type_enum;
    DTypeParam param;
} DType;

typedef struct {
    int nr_dim;
    uint32_t dims[MAX_DIM];
    int stride[MAX_DIM]; /* in elements */
    TinyNNFormat format;
} Layout;

typedef struct Tensor {
    char* name;
    DType dtype;
    Layout layout;
    void* ptr;
    size_t offset;
    int use_count;
    int is_weight;
    int is_dynamic;
    uint32_t checksum;
    size_t size;
    int is_shared;
    int is_input;
} Tensor;

typedef struct {
    void* ptr;
    size_t size;
    size_t offset;
} Workspace;

#endif /* DATA_STRUCT_H */

/* Value of Device.device_type reported by megcc_gfx950_init_device(): the next free slot after
 * runtime/src/tinynn.h:46-54 (TinyNN_WEB_ASSEMBLY = 6). */
#define TinyNN_GFX950 ((TinyNNDevice)7)

/* ------------------------------------------------------------------------------------------
 * Compile-time attributes (what the reference bakes into the kernel symbol).
 * ---------------------------------------------------------------------------------------- */
typedef enum {
    MEGCC_FMT_NCHW = 0,        /* "NCHW"  : [N,C,H,W]                                      */
    MEGCC_FMT_NCHW44 = 1,      /* "NCHW44": [N,C/4,H,W,4]                                  */
    MEGCC_FMT_NCHW_NCHW44 = 2  /* "NCHW44" with a 4-D source: NCHW in, NCHW44 out (first layer) */
} MegccFormat;

typedef enum { MEGCC_SPARSE_DENSE = 0, MEGCC_SPARSE_GROUP = 1 } MegccSparse;

typedef enum {
    MEGCC_NONLINE_IDENTITY = 0,
    MEGCC_NONLINE_RELU = 1,
    MEGCC_NONLINE_H_SWISH = 2,
    MEGCC_NONLINE_SIGMOID = 3
} MegccNonline;

/* ConvBias attributes: the keys KernelMaterialization hands to KernelGen
 * (compiler/test/kernel/common/src/cc_fill_attr.cpp:253-274). */
typedef struct {
    uint32_t kernel_h, kernel_w;
    uint32_t stride_h, stride_w;
    uint32_t pad_h, pad_w;
    uint32_t dilate_h, dilate_w;
    MegccFormat format;
    MegccSparse sparse;
    MegccNonline nonline;
    int with_bias; /* Common/ConvKernel.h:10-13 "is_bias" */
} MegccConvAttr;

typedef enum {
    MEGCC_POOL_MAX = 0,
    MEGCC_POOL_AVERAGE = 1,
    MEGCC_POOL_AVERAGE_COUNT_EXCLUDE_PADDING = 2
} MegccPoolMode;

/* cc_fill_attr.cpp:276-292 */
typedef struct {
    uint32_t window_h, window_w;
    uint32_t stride_h, stride_w;
    uint32_t pad_h, pad_w;
    MegccFormat format; /* NCHW or NCHW44 */
    MegccPoolMode mode;
} MegccPoolAttr;

/* cc_fill_attr.cpp:304-317; only format DEFAULT (row-major) is on this path */
typedef struct {
    int transpose_a;
    int transpose_b;
} MegccMatMulAttr;

typedef enum {
    MEGCC_Q_ADD = 0,
    MEGCC_Q_FUSE_ADD_RELU = 1,
    MEGCC_Q_MUL = 2,
    MEGCC_Q_RELU = 3
} MegccMultiTypeMode;

typedef enum {
    MEGCC_EW_RELU = 0,
    MEGCC_EW_EXP = 1,
    MEGCC_EW_SIGMOID = 2,
    MEGCC_EW_H_SWISH = 3,
    MEGCC_EW_NEGATE = 4,
    MEGCC_EW_ADD = 16,
    MEGCC_EW_SUB = 17,
    MEGCC_EW_MUL = 18,
    MEGCC_EW_TRUE_DIV = 19,
    MEGCC_EW_MAX = 20,
    MEGCC_EW_MIN = 21,
    MEGCC_EW_FUSE_ADD_RELU = 22,
    /* the modes below exist only as steps of a fused elementwise program */
    MEGCC_EW_ABS = 5,
    MEGCC_EW_LOG = 6,
    MEGCC_EW_SILU = 7,
    MEGCC_EW_ROUND = 8,
    MEGCC_EW_LT = 23,
    MEGCC_EW_LEQ = 24,
    MEGCC_EW_EQ = 25,
    MEGCC_EW_FLOOR_DIV = 26,
    MEGCC_EW_FUSE_ADD_SIGMOID = 27,
    MEGCC_EW_FUSE_ADD_TANH = 28,
    MEGCC_EW_FUSE_MUL_ADD3 = 32, /* a * b + c         */
    MEGCC_EW_FUSE_MUL_ADD4 = 33  /* a * b + c * d     */
} MegccElemwiseMode;

typedef enum {
    MEGCC_REDUCE_SUM = 0,
    MEGCC_REDUCE_MEAN = 1,
    MEGCC_REDUCE_MAX = 2,
    MEGCC_REDUCE_MIN = 3,
    MEGCC_REDUCE_PRODUCT = 4,
    MEGCC_REDUCE_SUM_SQR = 5
} MegccReduceMode;

typedef struct {
    MegccReduceMode mode;
    int axis;
} MegccReduceAttr;

/* A fused chain of f32 elementwise steps: the "modes:<i>" attributes of FusedElemwiseKernel
 * ("I0,I1,ADD,O0", "O0,I2,MUL,D", ...: BareMetal/FusedElemwiseKernel.cpp:126-153,286-306) with the
 * names resolved to value numbers. Value k < nr_input is input k; value nr_input + j is the
 * result of step j; the result of the last step is the output. */
#define MEGCC_FUSED_MAX_STEPS 16
#define MEGCC_FUSED_MAX_INPUTS 8
typedef struct {
    MegccElemwiseMode mode;
    int nr_arg;  /* 1..4 */
    int arg[4];  /* value numbers */
} MegccFusedStep;

typedef struct {
    int nr_input;
    int nr_step;
    MegccFusedStep step[MEGCC_FUSED_MAX_STEPS];
} MegccFusedElemwiseAttr;

/* "imode" of Resize (names as in the kernel symbol) */
typedef enum { MEGCC_IMODE_NEAREST = 0, MEGCC_IMODE_LINEAR = 1 } MegccInterpMode;

typedef struct {
    MegccFormat format; /* NCHW, or NCHW44 (LINEAR only) */
    MegccInterpMode imode;
} MegccResizeAttr;

/* ------------------------------------------------------------------------------------------
 * Operator entry points. After the attr pointer the argument lists are exactly KernelFunc /
 * InitFunc / WorkspaceFunc of runtime/src/data_struct.h:131-153.
 * ---------------------------------------------------------------------------------------- */

/* ConvBias. Replaces BareMetal::ConvGeneral (compiler/lib/KernelGen/BareMetal/ConvKernel.cpp:
 * 178-389) for qsi8 x qsi8 (+qsi32 bias) -> qsi8 and f32, formats NCHW / NCHW44 / NCHW->NCHW44,
 * DENSE and GROUP, and GeneralIntrinsic::ConvIm2colFloat (GeneralIntrinsic/ConvKernel/
 * Fp32Im2col.cpp:88-218) for f32 NCHW DENSE.
 * inputs = {src, filter[, bias]}, outputs = {dst}. qsi8 results are bit-identical with the
 * reference: int32 accumulate, + int32 bias, (float)acc * src_scale * flt_scale / dst_scale in
 * IEEE fp32, activation, roundf, saturate (BareMetal/Activation.cpp:47-56,105-114). */
TinyNNStatus megcc_gfx950_conv2d(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, const RuntimeOpt* opt);
/* Three-phase weight pre-processing protocol of Utils/StringTemplate.cpp:106-135 /
 * runtime/src/init.c:94-131: (out_weights==NULL) -> *nr_out_weight = number of processed weights;
 * (nr_out_weight==NULL) -> fill out_weights[i].layout/dtype/name; both non-NULL -> write the
 * processed weights into out_weights[i].ptr (device memory allocated by the caller). Dense qsi8
 * NCHW44 / NCHW convolutions that run on the MFMA kernel repack the filter into K-major 32-byte
 * rows; every other case reports 0 processed weights. */
TinyNNStatus megcc_gfx950_conv2d_init(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, Tensor* out_weights,
        int* nr_out_weight, const RuntimeOpt* opt);
/* Scratch bytes of the layer; MUST be queried (with the unpacked filter, before the init protocol
 * replaces it, as the compiler does) and handed to megcc_gfx950_conv2d. Padding and im2col are
 * folded into the LDS loads (the reference's optimised paths copy a padded source into workspace,
 * e.g. GeneralIntrinsic/ConvKernel/Im2colCommon.cpp:326-377), so most layers report 0; these do
 * not:
 *   - dense qsi8 layers with few output pixels and a long K (batch-1 layers, FullyConnected with
 *     up to 64 rows) and skinny f32 layers: int32 / f32 partial sums of a split of K. Without the
 *     workspace the layer still runs, unsplit and slower;
 *   - a 1x1 NCHW44 convolution with a stride: the gathered pixels. REQUIRED: without it the call
 *     returns TinyNN_ERROR_OUT_OF_RANGE (the filter was packed for the gathered geometry);
 *   - a dense qsi8 convolution on plain NCHW tensors: both NCHW44 copies. REQUIRED likewise;
 *   - a channel-wise qsi8 convolution on plain NCHW tensors: both NCHW44 copies and the filter.
 *     Without it the layer runs on the generic one-output-per-thread kernel.
 * Plain C semantics, no side effects, so the compiler may evaluate it at compile time as
 * compiler/lib/KernelGen/Jit/JitExe.cpp:67-123 does. */
TinyNNStatus megcc_gfx950_conv2d_workspace(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, int nr_thread,
        size_t* workspace);

/* megcc_gfx950_conv2d without the workspace argument and without any allocation. No counterpart
 * in the reference (its kernels get their scratch from the VM's arena); it is for callers that
 * cannot allocate or plan a workspace: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc. The scratch the layer's kernels need (split-K partial sums,
 * gathered pixels, NCHW44 copies: see megcc_gfx950_conv2d_workspace) lives in a static device
 * array of MEGCC_GFX950_NOALLOC_SCRATCH_BYTES that each GPU the library runs on holds until the
 * process ends. A layer whose REQUIRED scratch (the strided 1x1 and dense plain-NCHW cases of
 * megcc_gfx950_conv2d_workspace) exceeds the array returns TinyNN_ERROR_OUT_OF_RANGE (use
 * megcc_gfx950_conv2d); a layer whose optional scratch exceeds it runs as megcc_gfx950_conv2d runs
 * it without a workspace (unsplit, or on the generic kernel: qsi8 results identical, f32 results
 * within the 1e-4 tolerance of another summation order). `inputs[1]` is the filter as the init protocol left it. Every call on a
 * GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race.
 * Nothing in the array has to start at zero - every byte a kernel reads was written by an
 * earlier kernel of the same call. Calls no hipMalloc / hipFree; the array's address is looked
 * up at megcc_gfx950_init_device() or, failing that, on the first call on a device - so a caller
 * that captures this entry point into a HIP graph calls megcc_gfx950_init_device() (or this entry
 * point once) on the device BEFORE the capture begins: the look-up is not a stream operation. */
#define MEGCC_GFX950_NOALLOC_SCRATCH_BYTES (32u << 20)
TinyNNStatus megcc_gfx950_conv2d_noalloc(
        const MegccConvAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const RuntimeOpt* opt);

/* f32 MatrixMul, row-major, C = op(A) * op(B), no bias. Replaces GeneralIntrinsic::
 * Fp32MatMulM4N12 (GeneralIntrinsic/MatMulKernel/Fp32MatMulM4N12.cpp:9-158), Fp32GevmKernel
 * (GeneralIntrinsic/MatMulKernel/Fp32Gevm.cpp:50-119) and BareMetal::MatrixMulKernel
 * (BareMetal/MatrixMul.cpp:13-120). Leading dimensions are layout.stride[0].
 * (The reference has no qsi8 MatrixMul on this arch: a quantized FullyConnected is the 1x1 NCHW
 * convolution above on [M,K,1,1] x [N,K,1,1].) */
TinyNNStatus megcc_gfx950_matmul(
        const MegccMatMulAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace* workspace, const RuntimeOpt* opt);
TinyNNStatus megcc_gfx950_matmul_workspace(
        const MegccMatMulAttr* attr, Tensor** inputs, int nr_input, int nr_thread,
        size_t* workspace);

/* Pooling qsi8 / f32. Replaces BareMetal::PoolingKernel (BareMetal/Pooling.cpp:166-273, NCHW) and
 * GeneralIntrinsic::PoolingNchw44QInt8 (GeneralIntrinsic/PoolingKernel/QInt8PoolingNCHW44.cpp:
 * 116-216, NCHW44). inputs = {src}, outputs = {dst}. */
TinyNNStatus megcc_gfx950_pooling(
        const MegccPoolAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, const RuntimeOpt* opt);

/* Quantized elementwise QADD / QFUSE_ADD_RELU / QMUL (inputs = {a, b}) and QRELU (inputs = {a});
 * b may equal a in shape, be [1,C,1,1...] or a single element. Replaces
 * BareMetal::ElemwiseMultiTypeKernel (BareMetal/ElemwiseMultiType.cpp:16-213). */
TinyNNStatus megcc_gfx950_elemwise_multitype(
        const MegccMultiTypeMode* mode, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace* workspace, const RuntimeOpt* opt);

/* f32 elementwise, unary (inputs = {a}) or binary (inputs = {a, b}) over the broadcast of the two
 * operand shapes: shapes are aligned at their last dim, an extent of 1 stretches, the output has
 * the broadcast shape. That covers every operand pairing the reference names
 * (Common/ElemwiseCommon.cpp:47-127: VEC_VEC, VEC_SCALAR, VEC_BCAST101, VEC_BCAST101xX,
 * VEC_BCAST111C - [M,N] + [N], the FullyConnected bias -, VEC_BV, VEC_BCAST110, their mirrored
 * forms and NAIVE). More than one merged dim: fewer than 2^31 elements. Replaces
 * GeneralIntrinsic::ElemwiseKernel
 * (GeneralIntrinsic/Elemwise/Elemwise.cpp:10-36) / BareMetal::ElmwiseKernel
 * (BareMetal/ElemwiseKernel.cpp:35-66,413-431). */
TinyNNStatus megcc_gfx950_elemwise(
        const MegccElemwiseMode* mode, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace* workspace, const RuntimeOpt* opt);

/* TypeCvt f32->qsi8, qsi8->f32, qsi8->qsi8 (GeneralIntrinsic/Typecvt.cpp:71-295: one premultiplied
 * scale = src_scale/dst_scale) and qsi32->qsi8 (BareMetal/Typecvt.cpp:43-105: val*src/dst).
 * Directions are taken from the tensors' dtype; no attr. */
TinyNNStatus megcc_gfx950_typecvt(
        Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, const RuntimeOpt* opt);

/* f32 reduce over one axis of a contiguous tensor viewed as [A,B,C] (BareMetal/Reduce.cpp:73-134,
 * GeneralIntrinsic/Reduce.cpp:605-613). */
TinyNNStatus megcc_gfx950_reduce(
        const MegccReduceAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace* workspace, const RuntimeOpt* opt);

/* Relayout: copy between two strided views of the same dtype and element count (dimshuffle,
 * subtensor copies, NCHW <-> NCHW4 changes). Each side is walked in row-major order of its own
 * dims with its own strides (elements; negative strides and stride-0 sources allowed); element k
 * of the source becomes element k of the destination. Replaces BareMetal::RelayoutKernel
 * (BareMetal/Relayout.cpp:13-101, Common/Relayout.h:10-80; symbol kernel_relayout_<dtype>) and
 * GeneralIntrinsic::RelayoutKernel (GeneralIntrinsic/Relayout.cpp:27-48, GI_kernel_relayout_<dtype>).
 * inputs = {src}, outputs = {dst}; dtypes of 1, 2 and 4 bytes. */
TinyNNStatus megcc_gfx950_relayout(
        Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, const RuntimeOpt* opt);

/* Concat along *axis: input i goes to the slice of the output that starts where the inputs
 * before it end. Inputs and output may be strided. Replaces BareMetal::ConcatKernel
 * (BareMetal/Concat.cpp:14-76; symbol kernel_concat_byte_<dtype bytes>_axis_<axis>). */
TinyNNStatus megcc_gfx950_concat(
        const int* axis, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, const RuntimeOpt* opt);

/* f32 Resize of the two spatial dims: inputs = {src [N,C,IH,IW] or [N,C/4,IH,IW,4] (, target
 * shape: never read)}, outputs = {dst with OH, OW}. LINEAR: half-pixel centres, edges clamped,
 * dense tensors; NEAREST: floor(o / (O / I)), the source is read through its strides. Replaces
 * GeneralIntrinsic::ResizeKernel (GeneralIntrinsic/Resize.cpp:13-83,
 * GI_kernel_resize_linear_<fmt>_LINEAR_f32) and BareMetal::ResizeKernel (BareMetal/Resize.cpp:15-106,
 * kernel_resize_linear_<fmt>_<imode>_f32); arithmetic of Common/Resize.h:16-175. */
TinyNNStatus megcc_gfx950_resize(
        const MegccResizeAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace* workspace, const RuntimeOpt* opt);

/* Fused f32 elementwise chain over a dense output: inputs = the attr's nr_input tensors, each
 * either of the output's element count, a single element, [1,C,1,1] under a >= 4-d output or
 * [1,C,1,1,4] under a 5-d one (Common/ElemwiseCommon.cpp:7-45; reads as in
 * BareMetal/FusedElemwiseKernel.cpp:159-219). Replaces BareMetal::FusedElmwiseKernel
 * (BareMetal/FusedElemwiseKernel.cpp:270-423, kernel_naive_fused_elementwise_*) and
 * GeneralIntrinsic::FusedElmwiseKernel (GeneralIntrinsic/FusedElemwiseKernel.cpp:680-726,
 * kernel_gi_fused_elementwise_*). The reference's symbol names only the modes and operand kinds,
 * not which value feeds which step, so this operator cannot be reached through
 * megcc_gfx950_parse_symbol: the KernelGen shim carries the attr. */
TinyNNStatus megcc_gfx950_fused_elemwise(
        const MegccFusedElemwiseAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace* workspace, const RuntimeOpt* opt);

/* ------------------------------------------------------------------------------------------
 * Dispatch by the reference's kernel symbol: lets a caller that only knows the generated name
 * (e.g. "kernel_conv2d_3x3_NCHW44_DENSE_p1x1_s1x1_d1x1_qsi8qsi8qsi32qsi8_bias_RELU",
 * BareMetal/ConvKernel.cpp:144-176; "kernel_pooling_MAX_NCHW_p0x0_s2x2_w2x2_qsi8qsi8",
 * BareMetal/Pooling.cpp:31-44; GI_* aliases of the same operators) reach the entry points above.
 * ---------------------------------------------------------------------------------------- */
typedef enum {
    MEGCC_KERN_CONV = 1,
    MEGCC_KERN_MATMUL = 2,
    MEGCC_KERN_POOLING = 3,
    MEGCC_KERN_ELEMWISE_MULTITYPE = 4,
    MEGCC_KERN_ELEMWISE = 5,
    MEGCC_KERN_TYPECVT = 6,
    MEGCC_KERN_REDUCE = 7,
    MEGCC_KERN_RELAYOUT = 8,
    MEGCC_KERN_CONCAT = 9,
    MEGCC_KERN_RESIZE = 10,
    MEGCC_KERN_FUSED_ELEMWISE = 11, /* never produced by parse_symbol; a caller fills the attr */
    MEGCC_KERN_SOFTMAX = 12,        /* never produced by parse_symbol either: see megcc_gfx950_softmax */
    MEGCC_KERN_DW_POOL_ADD = 13,    /* nor this one: see megcc_gfx950_dw_pool_add */
    MEGCC_KERN_PW_DW = 14           /* nor this one: see megcc_gfx950_pw_dw */
} MegccKernelKind;

/* A channel-wise 3x3 convolution, the 2x2 stride-2 maximum pooling of its result and the quantised
 * addition of the pooled tensor with a second operand, as one operator (megcc_gfx950_dw_pool_add):
 * the attributes of the three operators and the scale of the two tensors between them (the pooling
 * keeps its input's scale, BareMetal/Pooling.cpp:22-27). */
typedef struct {
    MegccConvAttr conv;
    MegccPoolAttr pool;
    MegccMultiTypeMode mode; /* MEGCC_Q_ADD or MEGCC_Q_FUSE_ADD_RELU */
    float mid_scale;
} MegccDwPoolAddAttr;

/* A pointwise (1x1) convolution and the channel-wise 3x3 convolution of its result as one operator
 * (megcc_gfx950_pw_dw): the attributes of the two and the scale of the tensor between them. */
typedef struct {
    MegccConvAttr pw;
    MegccConvAttr dw;
    float mid_scale;
} MegccPwDwAttr;

typedef struct {
    MegccKernelKind kind;
    union {
        MegccConvAttr conv;
        MegccMatMulAttr matmul;
        MegccPoolAttr pool;
        MegccMultiTypeMode multitype;
        MegccElemwiseMode elemwise;
        MegccReduceAttr reduce;
        int concat_axis;
        MegccResizeAttr resize;
        MegccFusedElemwiseAttr fused;
        MegccDwPoolAddAttr dw_pool_add;
        MegccPwDwAttr pw_dw;
    } attr;
} MegccKernelDesc;

/* Depthwise 3x3 -> max-pool 2x2 stride 2 -> QADD / QFUSE_ADD_RELU in ONE kernel. MegCC emits three
 * kernels for this chain (kernel_conv2d_3x3_NCHW44_GROUP_..., kernel_pooling_MAX_NCHW44_p0x0_s2x2_w2x2_...,
 * kernel_elementwise_multitype_...: BareMetal/ConvKernel.cpp:144-176, BareMetal/Pooling.cpp:31-44,
 * BareMetal/ElemwiseMultiType.cpp:39-48); all three are bound by memory traffic, and two thirds of
 * that traffic is the depthwise result written and read back and the pooled tensor written and read
 * back. Here a thread keeps the 2 x 4 depthwise outputs of two pooling windows in registers, takes
 * the maxima, adds the second operand and stores 2 pixels of the final tensor. The model runtime
 * (megcc_gfx950_model_finalize) launches this entry point instead of the three kernels when the
 * tensors between them have no other reader; the three kernels stay available under their symbols.
 * qsi8 NCHW44 only; conv: GROUP (channel-wise) 3x3, pad 1, stride 1 or 2, dilation 1, any
 * activation; pool: MAX, window 2x2, stride 2, pad 0. inputs: source, filter, bias (when conv has
 * one), second operand of the addition (shape of the pooled tensor); outputs[0]: the sum. Bit-identical
 * to the three kernels run in sequence. megcc_gfx950_dw_pool_add_supported returns 1 for operands
 * this entry point takes. */
TinyNNStatus megcc_gfx950_dw_pool_add(
        const MegccDwPoolAddAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, const RuntimeOpt* opt);
int megcc_gfx950_dw_pool_add_supported(
        const MegccDwPoolAddAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output);

/* Pointwise 1x1 convolution -> channel-wise 3x3 convolution in ONE kernel, for images of at most 31
 * pixels a row. MegCC emits two kernels for the pair (kernel_conv2d_1x1_NCHW44_DENSE_... and
 * kernel_conv2d_3x3_NCHW44_GROUP_..., BareMetal/ConvKernel.cpp:144-176, loops :305-344); on the 14 x 14
 * and 7 x 7 images at the end of a MobileNet each of them is over before the chip is filled, so
 * their cost is launches and the trip of the tensor in between through memory. Here a workgroup
 * owns one image and 64 or 128 output channels, keeps its slice of the pointwise filter and the
 * pointwise result (channel-planar, zero border included) in LDS and runs the 3x3 window from
 * there. The model runtime launches this entry point instead of the two kernels when nothing else
 * reads the tensor between them; the two kernels stay available under their symbols.
 * qsi8 NCHW44 only. pw: DENSE 1x1, stride 1, pad 0, 128 / 256 / 512 input channels, output
 * channels a multiple of 64; dw: GROUP (channel-wise) 3x3, pad 1, stride 1 or 2, dilation 1; both with
 * IDENTITY or RELU; image width 4..31. inputs: source, the pointwise filter as megcc_gfx950_conv2d_init
 * returns it for `pw`, pointwise bias (when pw has one), channel-wise filter, channel-wise bias (when dw
 * has one); outputs[0]: the channel-wise layer's result. Bit-identical to the two kernels run in
 * sequence. megcc_gfx950_pw_dw_supported returns 1 for operands this entry point takes. */
TinyNNStatus megcc_gfx950_pw_dw(
        const MegccPwDwAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output,
        const Workspace* workspace, const RuntimeOpt* opt);
int megcc_gfx950_pw_dw_supported(
        const MegccPwDwAttr* attr, Tensor** inputs, int nr_input, Tensor** outputs, int nr_output);

/* Soft-max over the last axis in ONE kernel. MegCC has no such kernel: its importer decomposes
 * opr::Softmax into Reduce MAX -> SUB -> EXP -> Reduce SUM -> TRUE_DIV
 * (compiler/lib/Target/MGB/importer.cpp:987-1016), five kernel calls per forward, usually behind a
 * typecvt qsi8 -> f32. A kernel boundary costs 3-5 us on this chip, so the model runtime
 * (megcc_gfx950_model_finalize) replaces that operator chain - and the typecvt in front of it, when
 * nothing else reads its result - by this entry point; the five kernels stay available under their
 * own symbols. inputs[0]: f32, or qsi8 (dequantised with its scale first, as
 * GI_kernel_typecvt_qsi8f32 does); outputs[0]: f32 with as many elements, its last axis is the
 * soft-max axis; rows of at most
 * megcc_gfx950_softmax_max_columns() elements; same expressions per element as the five kernels,
 * only the order of the additions of a row's sum differs (results within 1e-6 relative). */
TinyNNStatus megcc_gfx950_softmax(
        Tensor** inputs, int nr_input, Tensor** outputs, int nr_output, const Workspace* workspace,
        const RuntimeOpt* opt);
int megcc_gfx950_softmax_max_columns(void);

/* TinyNN_ERROR_NO_FOUND when the symbol is not one of this path's operators. */
TinyNNStatus megcc_gfx950_parse_symbol(const char* symbol, MegccKernelDesc* desc);
TinyNNStatus megcc_gfx950_call(
        const MegccKernelDesc* desc, Tensor** inputs, int nr_input, Tensor** outputs,
        int nr_output, const Workspace* workspace, const RuntimeOpt* opt);
TinyNNStatus megcc_gfx950_call_init(
        const MegccKernelDesc* desc, Tensor** inputs, int nr_input, Tensor* out_weights,
        int* nr_out_weight, const RuntimeOpt* opt);
TinyNNStatus megcc_gfx950_call_workspace(
        const MegccKernelDesc* desc, Tensor** inputs, int nr_input, int nr_thread,
        size_t* workspace);

/* ------------------------------------------------------------------------------------------
 * Device seam: what runtime/src/device.c:29-43 (init_device) and the Lite C API's staging points
 * (runtime/src/lite/tensor.c:93-112 LITE_reset_tensor_memory, lite/network.c:229-232 LITE_wait)
 * need from a GPU device.
 * ---------------------------------------------------------------------------------------- */
/* Fills alignment (256), device_type and the HBM malloc/free hooks. */
TinyNNStatus megcc_gfx950_init_device(Device* device);
/* The hooks themselves (plain hipMalloc/hipFree: the TinyNN runtime asks for ONE arena per model,
 * runtime/src/init.c:437-487, plus one block per weight). */
void* megcc_gfx950_malloc(size_t length);
void megcc_gfx950_free(void* ptr);
/* Stream-ordered copies on the library stream (input staging / output fetch). d2h waits. */
TinyNNStatus megcc_gfx950_memcpy_h2d(void* dst_device, const void* src_host, size_t length);
TinyNNStatus megcc_gfx950_memcpy_d2h(void* dst_host, const void* src_device, size_t length);
TinyNNStatus megcc_gfx950_memset(void* dst_device, int value, size_t length);
/* Blocks until every kernel launched so far has finished (LITE_wait). */
TinyNNStatus megcc_gfx950_wait(void);
/* The hipStream_t all kernels are launched on, for callers that time with HIP events. */
void* megcc_gfx950_stream(void);
/* Text of the most recent error on the calling thread ("" if none). */
const char* megcc_gfx950_last_error(void);
/* Diagnostics (no counterpart in the reference, whose kernel choice is fixed at compile time):
 * which kernel variant the calling thread's most recent operator call selected, as
 * "<kernel>[:n,n,...]" (e.g. "conv_mfma_i8_dma:3,128,512,1024" = variant, oc tile, pixel
 * sub-tile, patch slots); "+affine" at the end: the kernel requantised by the one fused multiply-add
 * the host proved exact for the layer's scales instead of the threshold table. The text lives until
 * the thread's next call of this function. */
const char* megcc_gfx950_last_kernel(void);
/* Diagnostics (no counterpart in the reference): the constants of the one-multiply-add
 * requantisation for a convolution's activation and scales, as the qsi8 kernels would use them:
 * out = clamp(floor(fma((float)acc, *c, *d)), activation's lowest output, 127) equals the
 * reference's fp32_to_int8(act(acc * s_src * s_flt / s_dst)) (BareMetal/Activation.cpp:47-56,
 * 105-114) for EVERY int32 accumulator. Returns 1 and the pair when the host search finds one
 * (IDENTITY / RELU only), else 0 - such layers requantise by threshold table. Host arithmetic only:
 * needs no device. */
int megcc_gfx950_requant_affine(int nonline_mode, float s_src, float s_flt, float s_dst, float* c, float* d);
/* Kernel-selection overrides, for regression tests of kernels that un-switched shapes only reach
 * through a fallback: "nopws", "nogevm", "nofcb", "nosmall", "nopm768", "nopm", "nodma512",
 * "nopm256", "nodma", "nofcs", "nopwshare", "nohybrid", "nodot4", "nof32small",
 * "dw_generic", "nodwmfma", "nodwnchw", "nofusesoftmax", "nopoolrows", "nofirstmfma", "norowsplit", "nofusechain", "nofusepwdw", "fusepwdw", "nofcone", "noxcdorder", "noaffine", "nopipeline", "no_graph"; value 1 takes the kernel out
 * of the dispatch, 0 puts it back ("fusepwdw": 1 makes the model runtime take the one-kernel form of a
 * pointwise / channel-wise pair wherever it applies instead of timing both forms). The
 * same names in capitals behind MEGCC_ are read from the environment once, at first use.
 * Unknown names return TinyNN_ERROR_NO_FOUND. */
TinyNNStatus megcc_gfx950_set_option(const char* name, int value);

/* ------------------------------------------------------------------------------------------
 * In-memory model runtime: MegCC's static memory plan on one HBM arena. The calls mirror what the
 * TinyNN runtime does with a parsed `.tiny` model -- tensors with offsets into one buffer, weights,
 * a list of Opr instructions (runtime/schema/model.fbs:63-124) -- for a caller that builds the
 * model in memory the way runtime/test/common/common.h:46-123 does:
 *   add_* / add_opr   describe tensors, weights (uploaded to HBM at once) and instructions; an
 *                     instruction names its kernel by the generated symbol
 *   add_alias         a MemForward / reshape view sharing another tensor's memory
 *   finalize          liveness -> offsets (the [def, last use] intervals of
 *                     compiler/lib/Dialect/Kernel/Transforms/StaticMemoryPlanning.cpp:88-96), one
 *                     Device.malloc for the arena (runtime/src/init.c:437-487), three-phase kernel
 *                     init on the weights (init.c:29-131)
 *   set_input         LITE_reset_tensor_memory + staging copy (runtime/src/lite/tensor.c:93-112)
 *   forward           LITE_forward: one asynchronous launch per Opr (lite/network.c:171-227)
 *   get_output        waits, then copies back (LITE_get_tensor_memory)
 * Tensor ids are the return values of the add_* calls (-1 on error).
 * ---------------------------------------------------------------------------------------- */
void* megcc_gfx950_model_create(void);
void megcc_gfx950_model_destroy(void* model);
int megcc_gfx950_model_add_tensor(
        void* model, const char* name, int nr_dim, const uint32_t* dims, TinyNNDType dtype,
        float scale);
int megcc_gfx950_model_add_weight(
        void* model, const char* name, int nr_dim, const uint32_t* dims, TinyNNDType dtype,
        float scale, const void* host_data);
int megcc_gfx950_model_add_alias(
        void* model, const char* name, int of_tensor, int nr_dim, const uint32_t* dims);
/* A strided window into `of_tensor`: dims and strides (in elements, may be negative or 0) of the
 * view, whose first element lies offset_bytes after the start of `of_tensor`. This is what a
 * MemForward instruction of type SUBTENSOR or DIMSHUFFLE leaves behind (runtime/schema/
 * model.fbs:119-140, runtime/src/vm/memforward.c:43-53); operators that take strided tensors
 * (Relayout, Concat, MatMul row strides) read it as it is. -1 when an element would lie outside
 * of_tensor. */
int megcc_gfx950_model_add_view(
        void* model, const char* name, int of_tensor, int nr_dim, const uint32_t* dims,
        const int* strides, size_t offset_bytes);
TinyNNStatus megcc_gfx950_model_add_opr(
        void* model, const char* symbol, const int* inputs, int nr_input, const int* outputs,
        int nr_output);
/* The same with the operator given as a filled MegccKernelDesc instead of its symbol: for the one
 * operator whose reference symbol does not determine it (fused elementwise chains; `name` is
 * only a label). What runtime/src/vm/op.c:161-163 does with a function pointer taken from the
 * generated kernel table. */
TinyNNStatus megcc_gfx950_model_add_opr_desc(
        void* model, const MegccKernelDesc* desc, const char* name, const int* inputs, int nr_input,
        const int* outputs, int nr_output);
TinyNNStatus megcc_gfx950_model_mark_io(void* model, int tensor, int is_output);
/* The compiler's static memory plan for a model built in memory: offsets[i] = byte offset of
 * tensor i in one arena of arena_bytes bytes (entries of weights, model inputs and views are
 * ignored), what a `.tiny` file carries as Tensor.offset / DeviceModel.tensor_memory
 * (runtime/schema/model.fbs:63-124, used by runtime/src/init.c:437-487). finalize then keeps these
 * offsets instead of planning. TinyNN_ERROR_INVALID_LAYOUT for an offset that is not a multiple of
 * the device alignment or a tensor that leaves the arena. Call after the last add_* / mark_io. */
TinyNNStatus megcc_gfx950_model_set_plan(
        void* model, const size_t* offsets, int nr_tensor, size_t arena_bytes);
TinyNNStatus megcc_gfx950_model_finalize(void* model);
/* No counterpart in the reference (its VM runs one kernel per Opr, synchronously): the number of
 * kernels one forward launches (an operator chain that runs as one kernel counts once; a chain is
 * only replaced when its result shares no byte with anything the one kernel reads), and how they
 * are launched: 1 = HIP-graph replay, -1 = one launch per kernel, 0 = still measuring. The first ten
 * forwards of a model with at least 5 kernels measure: 2 + 3 and 7 + 8 are pairs of plain-launch
 * forwards between two events on the library stream, 5 + 6 and 9 + 10 pairs of replays (4 captures);
 * the second forward of a pair blocks the host until both are done. A pair's cost is the time on
 * the device from the end of its first forward to the end of its second - the first forward's last
 * operators overlapping the second one's first where plain launches allow it
 * (megcc_gfx950_model_join below) - or the time the host took to enqueue the second forward,
 * whichever is longer: what limits back-to-back forwards. *eager_ms /
 * *graph_ms receive the lower of the two pairs each, -1 when not measured; the replay is kept when
 * it is at least 2 % faster. Every other forward is asynchronous. */
int megcc_gfx950_model_nr_kernel(void* model);
int megcc_gfx950_model_launch_mode(void* model, float* eager_ms, float* graph_ms);
size_t megcc_gfx950_model_arena_bytes(void* model);
void* megcc_gfx950_model_tensor_ptr(void* model, int tensor);
TinyNNStatus megcc_gfx950_model_set_input(void* model, int tensor, const void* host, size_t bytes);
TinyNNStatus megcc_gfx950_model_get_output(void* model, int tensor, void* host, size_t bytes);
TinyNNStatus megcc_gfx950_model_forward(void* model);
/* No counterpart in the reference either. With plain launches (launch mode -1) the last operators
 * of a forward - the longest suffix estimated to take no longer than the operators before it - are
 * launched on a second stream, ordered behind the rest by an event, so that they
 * overlap the first operators of the NEXT forward, which do not depend on them (the runtime's own
 * memory plan gives what they touch bytes of its own; under any other plan the next forward waits
 * for them before it writes bytes they use). megcc_gfx950_wait(), megcc_gfx950_model_get_output()
 * and megcc_gfx950_model_set_input() (for an input those operators read) take that into account.
 * A caller that orders work of its own on megcc_gfx950_stream() behind a forward - an event, a
 * copy - calls megcc_gfx950_model_join() first: it makes the library stream wait (on the device,
 * not the host) for everything the model's forwards have launched. Switch "nopipeline"
 * (MEGCC_NOPIPELINE=1) keeps every operator on the library stream. */
TinyNNStatus megcc_gfx950_model_join(void* model);
/* how many of megcc_gfx950_model_nr_kernel's kernels those last operators are (0: none) */
int megcc_gfx950_model_nr_tail_kernel(void* model);
/* megcc_gfx950_model_get_output without the host waiting: the copy is enqueued behind the forward
 * that produced the tensor (on the second stream when that forward's last operators are there) and
 * the bytes are in `host` - pinned memory, for the copy to be asynchronous - after
 * megcc_gfx950_wait(). The loop forward(i), get_output_async(i), set_input(i + 1), forward(i + 1)
 * keeps forward i's last operators overlapped with forward i + 1's first, which the blocking call
 * cannot: the host would not enqueue forward i + 1 before forward i is over. */
TinyNNStatus megcc_gfx950_model_get_output_async(void* model, int tensor, void* host, size_t bytes);
int megcc_gfx950_model_nr_opr(void* model);
/* one instruction only: per-layer timing / tensor dumps (the TINYNN_PROFILE_KERNEL and
 * TINYNN_DUMP_TENSOR hooks of runtime/src/lite/network.c:187-224) */
TinyNNStatus megcc_gfx950_model_run_opr(void* model, int index);

/* `.tiny` model files (the FlatBuffers binary of runtime/schema/model.fbs written by the MegCC
 * compiler, compiler/lib/Target/TinyNN/exporter.cpp).
 * model_load replaces LITE_load_model_from_mem -> parse_model (runtime/src/parse.c:423-560,
 * per-instruction loaders runtime/src/vm/op.c:11-65 and vm/memforward.c:24-41) plus
 * init_model_weights / init_model_memory (runtime/src/init.c): weights go to HBM (fp16-compressed
 * fp32 weights are widened like parse.c:232-263), tensors sit at the offsets of the file's static
 * memory plan inside one arena of tensor_memory bytes, model inputs get device buffers of their
 * own, every Opr instruction is bound by its kernel symbol (Opr.type) to the gfx950 kernel of the
 * same name, MemForward instructions become views. The device model used is the one compiled for
 * this device (Device value 7, appended to the schema's enum) or else the BARE_METAL one.
 * Tensor ids of the loaded model = index in the file's tensor_pool; weight j = nr_tensor + j.
 * Errors: TinyNN_ERROR_MODEL_PARSE for a truncated / inconsistent file (the reference traps),
 * TinyNN_ERROR_NO_FOUND when no usable device model or no gfx950 kernel for a symbol,
 * TinyNN_ERROR_UNSUPPORTED_INSTRUCTION_TYPE for instructions other than Opr and MemForward,
 * TinyNN_ERROR_NO_IMPLEMENT for dynamic tensors. The buffer may be freed after the call.
 *
 * tiny_describe writes one text line per weight, tensor and instruction of the file (every field
 * the loader reads); *needed receives the length including the NUL. Host code only. */
TinyNNStatus megcc_gfx950_model_load(const void* buffer, size_t size, void** model);
TinyNNStatus megcc_gfx950_tiny_describe(
        const void* buffer, size_t size, char* text, size_t capacity, size_t* needed);

/* The static memory plan by itself: interval i is alive during time steps [begin[i], end[i]) and
 * needs size[i] bytes; offset[i] receives its place in one arena of *arena_bytes bytes, every
 * offset a multiple of `alignment` (a power of two). Replaces, with identical offsets and arena
 * size, StaticMemAlloc::make(PUSHDOWN) + add() + alignment() + solve() + get_start_addr() /
 * tot_alloc() / tot_alloc_lower_bound() of compiler/lib/Dialect/Kernel/Transforms/migrate/
 * static_mem_alloc.h:12-87 as driven by Transforms/StaticMemoryPlanning.cpp:34-96 (time step =
 * operator index, end = last use + 1). Host code only, no GPU needed. lower_bound may be NULL.
 * TinyNN_ERROR_INVALID_LAYOUT for a bad alignment or an interval with begin >= end (the reference
 * asserts on both). Overwrite specs (add_overwrite_spec) are not offered: that pass never adds
 * one. */
TinyNNStatus megcc_gfx950_plan_memory(
        size_t nr_interval, const size_t* begin, const size_t* end, const size_t* size,
        size_t alignment, size_t* offset, size_t* arena_bytes, size_t* lower_bound);

#ifdef __cplusplus
}
#endif
#endif /* MEGCC_GFX950_H */
