// TEST INFRASTRUCTURE ONLY -- never linked into or called by the product library.
//
// What MegCC's compiler does for a model once `Arch::GFX950` exists, minus MLIR: for every line of
// a spec file (format: oracle/ref_dump.cpp) the reference's OWN registry - its KernelGen.cpp with
// megcc_amd/upstream/kernelgen_arch_gfx950.patch applied to a scratch copy, compiled and linked with
// the rest of compiler/lib/KernelGen where it lies - is asked for
// KernelPack::GetKernel(type, Arch::GFX950), the first candidate whose IsAvailable() holds is taken
// (the rule of KernelMaterialization.cpp:229), and the files the TinyNN exporter would write are
// written (compiler/lib/Target/TinyNN/KernelExporter.cpp:15-66,79-88,190-216):
//   <outdir>/<symbol>.c     #include "kernels.h" + kernel, init and workspace text of one kernel
//   <outdir>/kernels.h      NR_KERNELS / NR_INIT / NR_WORKSPACE / NR_DEDUCE_SHAPE, the four tables,
//                           one declaration per function
//   <outdir>/kernels.c      the tables and load_kernel_init_function() filling them
//   <outdir>/kernel_ids.txt "<symbol> <kernel_id> <init_id> <workspace_id>" per distinct kernel: the
//                           numbers an Opr of a `.tiny` file carries (Opr.kernel_id / init_id /
//                           workspace_id, runtime/schema/model.fbs, read by runtime/src/vm/op.c:15-22)
//   <outdir>/runtime_inst_switch.h  the instruction types a static-shape model uses (Opr is always
//                           built in; MEMFORWARD for its reshape / sub-tensor views)
//   <outdir>/manifest.txt   "<label> <symbol>" per spec line
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

struct Exported {
    std::string symbol, kernel_sig, init_sig, workspace_sig, init_sym, workspace_sym;
};

int main(int argc, char** argv) {
    if (argc != 3) {
        fprintf(stderr, "usage: %s <spec-file> <outdir>\n", argv[0]);
        return 2;
    }
    megcc::setAssertThrow(true);
    std::ifstream spec(argv[1]);
    const std::string outdir = argv[2];
    std::ofstream manifest(outdir + "/manifest.txt");
    std::vector<Exported> kernels;
    std::map<std::string, int> index;
    std::string line;
    int line_no = 0, fail = 0;
    while (std::getline(spec, line)) {
        ++line_no;
        if (line.empty() || line[0] == '#')
            continue;
        std::stringstream ls(line);
        std::string type_name, kv, label = std::to_string(line_no);
        ls >> type_name;
        auto it = kTypes.find(type_name);
        if (it == kTypes.end()) {
            fprintf(stderr, "line %d: unknown kernel type %s\n", line_no, type_name.c_str());
            return 2;
        }
        std::unordered_map<std::string, CCAttr> attrs;
        while (ls >> kv) {
            if (kv[0] == '@') {
                label = kv.substr(1);
                continue;
            }
            size_t eq = kv.find('=');
            std::string key = kv.substr(0, eq), val = kv.substr(eq + 3);
            switch (kv[eq + 1]) {
                case 's': attrs[key] = CCAttr(val); break;
                case 'u': attrs[key] = CCAttr((uint32_t)std::stoul(val)); break;
                case 'i': attrs[key] = CCAttr((int32_t)std::stol(val)); break;
                case 'b': attrs[key] = CCAttr((bool)(val == "1")); break;
                case 'o': attrs[key] = CCAttr(parse_operand(val)); break;
                default:
                    fprintf(stderr, "line %d: bad attr %s\n", line_no, kv.c_str());
                    return 2;
            }
        }
        CodeGenContext ctx(attrs);
        // the one call this driver exists for: the reference's registry, the new Arch
        auto pack = KernelGen::KernelPack::GetKernel(it->second, KernelGen::Arch::GFX950).first;
        const KernelGen::KernelFunc* chosen = nullptr;
        for (auto* k : pack) {
            bool ok = false;
            try {
                ok = k->IsAvailable(&ctx);
            } catch (...) {
            }
            if (ok) {
                chosen = k;
                break;
            }
        }
        if (!chosen) {
            fprintf(stderr, "line %d: Arch::GFX950 has no kernel (%s)\n", line_no, line.c_str());
            manifest << label << " NONE\n";
            ++fail;
            continue;
        }
        const std::string sym = chosen->GetKernelSymbol(&ctx);
        manifest << label << " " << sym << "\n";
        if (index.count(sym))
            continue;
        index[sym] = (int)kernels.size();
        Exported e;
        e.symbol = sym;
        e.kernel_sig = chosen->GetKernelSignature(&ctx);
        e.init_sig = chosen->GetInitSignature(&ctx);
        e.workspace_sig = chosen->GetWorkspaceSignature(&ctx);
        e.init_sym = chosen->GetInitSymbol(&ctx);
        e.workspace_sym = chosen->GetWorkspaceSymbol(&ctx);
        kernels.push_back(e);
        std::ofstream f(outdir + "/" + sym + ".c");
        f << "// this file should be generated by MegCC\n\n#include \"kernels.h\"\n\n"
          << chosen->GetKernelBody(&ctx) << "\n\n"
          << chosen->GetInitBody(&ctx) << "\n\n"
          << chosen->GetWorkspaceBody(&ctx) << "\n";
    }
    const std::string ret = KernelGen::GenCommonRet();
    {
        std::ofstream h(outdir + "/kernels.h");
        h << "// this file should be generated by MegCC\n#ifndef KERNEL_H\n#define KERNEL_H\n\n"
             "#include \"data_struct.h\"\n#include \"stdint.h\"\n#include \"string.h\"\n\n"
          << "#define NR_KERNELS (" << kernels.size() << ")\n#define NR_INIT (" << kernels.size()
          << ")\n#define NR_DEDUCE_SHAPE (1)\n#define NR_WORKSPACE (" << kernels.size() << ")\n\n"
          << "#define KERNEL_MARK_USDED_VAR(x) (void)(x);\n\n"
             "extern KernelFunc kernels[NR_KERNELS];\n\nextern InitFunc init_kernels[NR_INIT];\n"
             "extern WorkspaceFunc workspace_func[NR_WORKSPACE];\n"
             "extern DeduceFunc deduce_func[NR_DEDUCE_SHAPE];\n//! declare all the kernel here in C\n\n";
        for (auto& e : kernels)
            h << ret << " " << e.kernel_sig << ";\n";
        for (auto& e : kernels)
            h << ret << " " << e.init_sig << ";\n";
        for (auto& e : kernels)
            h << ret << " " << e.workspace_sig << ";\n";
        h << "\nvoid load_kernel_init_function();\n\n#endif\n";
    }
    {
        std::ofstream c(outdir + "/kernels.c"), ids(outdir + "/kernel_ids.txt");
        c << "// this file should be generated by MegCC\n\n#include \"kernels.h\"\n\n"
             "KernelFunc kernels[NR_KERNELS];\nInitFunc init_kernels[NR_INIT];\n"
             "WorkspaceFunc workspace_func[NR_WORKSPACE];\nDeduceFunc deduce_func[NR_DEDUCE_SHAPE];\n\n"
             "//! not thread safe\nvoid load_kernel_init_function() {\n    static int done = 0;\n"
             "    if (done) {\n        return ;\n    }\n";
        for (size_t i = 0; i < kernels.size(); ++i) {
            c << "    kernels[" << i << "] = " << kernels[i].symbol << ";\n"
              << "    init_kernels[" << i << "] = " << kernels[i].init_sym << ";\n"
              << "    workspace_func[" << i << "] = " << kernels[i].workspace_sym << ";\n";
            ids << kernels[i].symbol << " " << i << " " << i << " " << i << "\n";
        }
        c << "    done = 1;\n    return ;\n}\n";
    }
    {
        std::ofstream sw(outdir + "/runtime_inst_switch.h");
        sw << "// this file should be generated by MegCC\n#define ENABLE_INST_MEMFORWARD 1 \n";
    }
    fprintf(stderr, "Arch::GFX950: %zu kernels exported%s\n", kernels.size(),
            fail ? ", SOME LINES HAD NONE" : "");
    return fail ? 1 : 0;
}
