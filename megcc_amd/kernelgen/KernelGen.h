// KernelGen target for gfx950: the compile-time half of the drop-in boundary.
//
// MegCC selects and emits kernels through `KernelGen::KernelFunc` objects returned by
// `KernelPack::GetKernel(KernType, Arch)` (compiler/include/compiler/KernelGen/KernelGen.h:75-136,
// 160-197; candidate order = priority, first IsAvailable() wins,
// compiler/lib/Dialect/Kernel/Transforms/KernelMaterialization.cpp:212-276). This target keeps
// that interface -- same method names, same attribute keys, same kernel symbols -- but where the
// reference's templates emit the loop nest itself, these emit a few lines of C that fix the
// operator's compile-time attributes in a constant struct and forward the uniform
// (Tensor**, int, Tensor**, int, const Workspace*, const RuntimeOpt*) call to the hand-written
// HIP kernels behind libmegcc_gfx950.so (include/megcc_gfx950.h).
//
// The attribute bag is MegCC's `TContext` (compiler/include/compiler/Common/TContext.h:177-243).
// Inside a MegCC tree (this file and Gfx950Kernels.cpp dropped into compiler/lib/KernelGen/Gfx950/,
// where "compiler/KernelGen/KernelGen.h" is on the include path, or MEGCC_GFX950_IN_TREE defined)
// the reference's own headers are used and the classes below derive from its KernelFunc.
// Stand-alone (this repository: tests, the kernelgen tool) a minimal mirror with the same method
// names is declared here.
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#if !defined(MEGCC_GFX950_IN_TREE) && defined(__has_include)
#if __has_include("compiler/KernelGen/KernelGen.h")
#define MEGCC_GFX950_IN_TREE 1
#endif
#endif

#ifdef MEGCC_GFX950_IN_TREE
#include "compiler/KernelGen/KernelGen.h"
namespace megcc_gfx950 {
using megcc::CCOperand;
using megcc::TContext;
using KernelFuncBase = megcc::KernelGen::KernelFunc;
using KernType = megcc::KernelGen::KernelPack::KernType;
}  // namespace megcc_gfx950
#else
namespace megcc_gfx950 {

// operand description: TContext.h:12-47
struct CCOperand {
    std::vector<size_t> shape;
    std::string dtype;  // "f32", "si8", "i32", "qsi8<bits:scale>", "qsi32<bits:scale>"
    float scale = -1.f;
};

// the subset of TContext the conv / matmul / pooling / elemwise / typecvt / reduce templates read
class TContext {
public:
    void setAttr(const std::string& k, const std::string& v) { m_str[k] = v; }
    void setAttr(const std::string& k, const char* v) { m_str[k] = v; }
    void setAttr(const std::string& k, int64_t v) { m_int[k] = v; }
    void setAttr(const std::string& k, bool v) { m_int[k] = v; }
    void setAttr(const std::string& k, const CCOperand& v) { m_op[k] = v; }
    bool haveAttr(const std::string& k) const {
        return m_str.count(k) || m_int.count(k) || m_op.count(k);
    }
    std::string getAttrStr(const std::string& k) const;
    int32_t getAttrInt(const std::string& k) const { return (int32_t)get_int(k); }
    uint32_t getAttrUInt(const std::string& k) const { return (uint32_t)get_int(k); }
    bool getAttrBool(const std::string& k) const { return get_int(k) != 0; }
    CCOperand getAttrOprand(const std::string& k) const;

private:
    int64_t get_int(const std::string& k) const;
    std::unordered_map<std::string, std::string> m_str;
    std::unordered_map<std::string, int64_t> m_int;
    std::unordered_map<std::string, CCOperand> m_op;
};

// KernelGen.h:75-136
struct KernelFuncBase {
    virtual ~KernelFuncBase() = default;
    virtual bool IsAvailable(TContext* context) const = 0;
    virtual std::string GetKernelSymbol(TContext* context) const = 0;
    virtual std::string GetKernelSignature(TContext* context) const;
    virtual std::string GetKernelBody(TContext* context) const = 0;
    virtual std::string GetInitSymbol(TContext* context) const {
        return GetKernelSymbol(context) + "_init";
    }
    virtual std::string GetInitSignature(TContext* context) const;
    virtual std::string GetInitBody(TContext* context) const;
    virtual std::string GetWorkspaceSymbol(TContext* context) const {
        return GetKernelSymbol(context) + "_workspace";
    }
    virtual std::string GetWorkspaceSignature(TContext* context) const;
    virtual std::string GetWorkspaceBody(TContext* context) const;
};

// KernelGen.h:160-194 (the kernel types on this path)
enum class KernType {
    Unknow = 0,
    ConvKernel,
    ElemwiseKernel,
    ElemwiseMultiKernel,
    PoolingKernel,
    MatrixMulKernel,
    RelayoutKernel = 7,
    ReduceKernel = 8,
    TypeCvtKernel = 13,
    ResizeKernel = 19,
    ConcatKernel = 25,
    FusedElemwiseKernel = 28,
};

}  // namespace megcc_gfx950
#endif

namespace megcc_gfx950 {

// What `KernelPack::GetKernel(kernel_type, Arch::GFX950)` returns: ordered candidates, first
// available wins. Unlike the other non-BAREMETAL arches no BAREMETAL kernels are appended
// (compiler/lib/Dialect/Kernel/Transforms/KernelTemplate.cpp:128-135): an operator without a
// gfx950 kernel is a compile-time error, never a silent CPU fallback.
struct Gfx950KernelPack {
    static std::vector<const KernelFuncBase*> GetKernel(KernType kernel_type);
};

// kernel symbol MegCC's own x86 registry generates for the same context (the dedup key of
// KernelTemplate.cpp:60-62): the shims keep these names so that models, dumps and the tests can
// address a kernel by the name they already know
std::string ReferenceSymbol(KernType type, TContext* context);

}  // namespace megcc_gfx950
