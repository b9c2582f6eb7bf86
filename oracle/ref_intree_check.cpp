// TEST INFRASTRUCTURE ONLY -- never linked into or called by the product library.
//
// The gfx950 KernelGen target (megcc_amd/kernelgen/Gfx950Kernels.cpp) built in-tree, i.e.
// deriving from the reference's own KernelGen::KernelFunc
// (compiler/include/compiler/KernelGen/KernelGen.h:75-136) and reading the reference's own
// TContext (compiler/include/compiler/Common/TContext.h:177-243), linked with the reference's
// KernelGen registry compiled from the sources where they lie (oracle/Makefile) - except
// KernelGen.h / KernelGen.cpp, of which scratch copies with
// megcc_amd/upstream/kernelgen_arch_gfx950.patch applied are compiled, so that every pack below
// comes from the reference's own KernelPack::GetKernel(type, Arch::GFX950). For every line
// of a spec file (format: oracle/ref_dump.cpp) it checks what that registry branch relies on:
//   1. a gfx950 kernel is available for the context, through the reference's CodeGenContext;
//   2. its symbol is the symbol of an available kernel of the reference's Arch::BAREMETAL list
//      for the same context ("first" = the one the x86 build would select, "later" = a lower
//      priority BAREMETAL template; the run-time library resolves both spellings);
//   3. kernel / init / workspace texts and signatures are produced without touching a missing
//      attribute (the reference's TContext aborts on one);
//   4. the workspace function's text is self-contained C: the compiler JIT-compiles and runs it
//      at model-compile time (compiler/lib/KernelGen/Jit/JitExe.cpp), where the GPU library is
//      not loaded, so it may not call into it.
// And once per kernel type: GetKernelSymbol(nullptr) returns without crashing, since the exporter
// calls it with a null context to filter kernels by name (KernelGen.cpp:49-53).
// Prints one line per spec line and a summary; exit status 0 only if every check held.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "compiler/Common/Logger.h"
#include "compiler/Common/TContext.h"
#include "compiler/KernelGen/KernelGen.h"

#include "../megcc_amd/kernelgen/KernelGen.h"

using namespace megcc;
using KT = KernelGen::KernelPack::KernType;

static const std::map<std::string, KT> kTypes = {
        {"ConvKernel", KT::ConvKernel},
        {"ElemwiseKernel", KT::ElemwiseKernel},
        {"ElemwiseMultiKernel", KT::ElemwiseMultiKernel},
        {"PoolingKernel", KT::PoolingKernel},
        {"MatrixMulKernel", KT::MatrixMulKernel},
        {"ReduceKernel", KT::ReduceKernel},
        {"TypeCvtKernel", KT::TypeCvtKernel},
        {"RelayoutKernel", KT::RelayoutKernel},
        {"ConcatKernel", KT::ConcatKernel},
        {"ResizeKernel", KT::ResizeKernel},
        {"FusedElemwiseKernel", KT::FusedElemwiseKernel},
};

static CCOperand parse_operand(const std::string& v) {
    CCOperand op;
    size_t p0 = v.find('|');
    std::string shape = v.substr(0, p0);
    std::string rest = p0 == std::string::npos ? "" : v.substr(p0 + 1);
    size_t p1 = rest.find('|');
    std::string dtype = rest.substr(0, p1);
    std::string scale = p1 == std::string::npos ? "" : rest.substr(p1 + 1);
    if (!shape.empty()) {
        std::stringstream ss(shape);
        std::string tok;
        while (std::getline(ss, tok, 'x'))
            op.shape.push_back(std::stoull(tok));
    }
    if (dtype == "qsi8" || dtype == "qsi32") {
        float s = std::stof(scale);
        uint32_t bits;
        std::memcpy(&bits, &s, 4);
        std::stringstream ds;
        ds << dtype << "<" << bits << ":" << s << ">";
        op.dtype = ds.str();
        op.scale = s;
    } else {
        op.dtype = dtype;
    }
    return op;
}

static bool available(const KernelGen::KernelFunc* k, TContext* ctx) {
    try {
        return k->IsAvailable(ctx);
    } catch (...) {
        return false;
    }
}

int main(int argc, char** argv) {
    if (argc != 2) {
        fprintf(stderr, "usage: %s <spec-file>\n", argv[0]);
        return 2;
    }
    megcc::setAssertThrow(true);
    int bad = 0, n_first = 0, n_later = 0, n_lines = 0;
    for (auto& kv : kTypes) {
        for (auto* k : KernelGen::KernelPack::GetKernel(kv.second, KernelGen::Arch::GFX950).first) {
            std::string s = k->GetKernelSymbol(nullptr);
            if (s.empty()) {
                printf("FAIL %s: empty symbol for a null context\n", kv.first.c_str());
                ++bad;
            }
        }
    }
    std::ifstream spec(argv[1]);
    std::string line;
    int line_no = 0;
    while (std::getline(spec, line)) {
        ++line_no;
        if (line.empty() || line[0] == '#')
            continue;
        std::stringstream ls(line);
        std::string type_name, kvs, label = std::to_string(line_no);
        ls >> type_name;
        auto it = kTypes.find(type_name);
        if (it == kTypes.end()) {
            fprintf(stderr, "line %d: unknown kernel type %s\n", line_no, type_name.c_str());
            return 2;
        }
        std::unordered_map<std::string, CCAttr> attrs;
        while (ls >> kvs) {
            if (kvs[0] == '@') {
                label = kvs.substr(1);
                continue;
            }
            size_t eq = kvs.find('=');
            std::string key = kvs.substr(0, eq), val = kvs.substr(eq + 3);
            switch (kvs[eq + 1]) {
                case 's': attrs[key] = CCAttr(val); break;
                case 'u': attrs[key] = CCAttr((uint32_t)std::stoul(val)); break;
                case 'i': attrs[key] = CCAttr((int32_t)std::stol(val)); break;
                case 'b': attrs[key] = CCAttr((bool)(val == "1")); break;
                case 'o': attrs[key] = CCAttr(parse_operand(val)); break;
                default: fprintf(stderr, "line %d: bad attr %s\n", line_no, kvs.c_str()); return 2;
            }
        }
        ++n_lines;
        CodeGenContext ctx(attrs);
        // what the x86 build offers for this context, in priority order
        std::vector<std::string> ref_syms;
        for (auto* k : KernelGen::KernelPack::GetKernel(it->second, KernelGen::Arch::BAREMETAL).first)
            if (available(k, &ctx))
                ref_syms.push_back(k->GetKernelSymbol(&ctx));
        const KernelGen::KernelFunc* mine = nullptr;
        for (auto* k : KernelGen::KernelPack::GetKernel(it->second, KernelGen::Arch::GFX950).first)
            if (available(k, &ctx)) {
                mine = k;
                break;
            }
        if (!mine) {
            printf("FAIL %s: no gfx950 kernel is available\n", label.c_str());
            ++bad;
            continue;
        }
        const std::string sym = mine->GetKernelSymbol(&ctx);
        int where = -1;
        for (size_t i = 0; i < ref_syms.size(); ++i)
            if (ref_syms[i] == sym) {
                where = (int)i;
                break;
            }
        const std::string body = mine->GetKernelBody(&ctx), init = mine->GetInitBody(&ctx),
                          ws = mine->GetWorkspaceBody(&ctx);
        const bool sigs = mine->GetKernelSignature(&ctx).find(sym + "(") == 0 &&
                          mine->GetInitSignature(&ctx).find(sym + "_init(") == 0 &&
                          mine->GetWorkspaceSignature(&ctx).find(sym + "_workspace(") == 0;
        const bool ws_alone = ws.find("megcc_gfx950") == std::string::npos &&
                              ws.find("extern") == std::string::npos &&
                              ws.find("#include") == std::string::npos;
        const bool texts = body.find(sym) != std::string::npos &&
                           init.find(sym + "_init") != std::string::npos &&
                           ws.find(sym + "_workspace") != std::string::npos;
        const bool ok = where >= 0 && sigs && ws_alone && texts;
        if (where == 0)
            ++n_first;
        else if (where > 0)
            ++n_later;
        if (!ok)
            ++bad;
        printf("%s %s %s %s%s%s%s\n", ok ? "ok" : "FAIL", label.c_str(), sym.c_str(),
               where == 0  ? "first"
               : where > 0 ? "later"
                           : "not-a-reference-symbol",
               sigs ? "" : " bad-signature", ws_alone ? "" : " workspace-text-not-self-contained",
               texts ? "" : " text-without-symbol");
        if (where < 0)
            for (auto& s : ref_syms)
                printf("     reference offers %s\n", s.c_str());
    }
    printf("SUMMARY lines=%d first=%d later=%d failed=%d\n", n_lines, n_first, n_later, bad);
    return bad ? 1 : 0;
}
