// TEST INFRASTRUCTURE ONLY -- never linked into or called by the product library.
//
// Driver around the *reference's own* KernelGen registry (compiled from the sources where they
// lie under /root/reference by oracle/Makefile; nothing of the reference is copied here).
// For every line of a spec file it builds a CodeGenContext, asks
// KernelPack::GetKernel(type, Arch::BAREMETAL) for the ordered candidate list
// (compiler/lib/KernelGen/KernelGen.cpp:100-125), takes the first candidate whose IsAvailable()
// holds -- the same selection rule as KernelMaterialization.cpp:229 -- and writes the C text the
// reference generates for it (kernel + init + workspace, internal helper kernels in files of
// their own, as compiler/lib/Target/TinyNN/KernelExporter.cpp:190-216 does).
//
// Spec line:   <KernType> [@label] <key>=<t>:<value> ...
//   t = s string | u uint32 | i int32 | b bool | o operand "d0xd1x...|dtype|scale"
//   dtype: f32 | i32 | si8 | qsi8 | qsi32   (q types get the "<bits:scale>" suffix the
//   compiler writes, compiler/test/kernel/common/src/cc_proxy_utils.h:37-68)
// Output: <outdir>/<symbol>.c per distinct symbol, <outdir>/manifest.txt ("<label> <symbol>",
// label = line number when the line carries none).
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iostream>
#include <map>
#include <set>
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
    // "1x16x56x56x4|qsi8|0.02"
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

static void write_file(const std::string& path, const std::string& text) {
    std::ofstream f(path);
    f << text;
}

int main(int argc, char** argv) {
    if (argc != 3) {
        fprintf(stderr, "usage: %s <spec-file> <outdir>\n", argv[0]);
        return 2;
    }
    megcc::setAssertThrow(true);
    std::ifstream spec(argv[1]);
    std::string outdir = argv[2];
    std::ofstream manifest(outdir + "/manifest.txt");
    std::set<std::string> written;
    std::string line;
    int line_no = 0, fail = 0;
    while (std::getline(spec, line)) {
        ++line_no;
        if (line.empty() || line[0] == '#')
            continue;
        std::stringstream ls(line);
        std::string type_name, kv;
        ls >> type_name;
        auto it = kTypes.find(type_name);
        if (it == kTypes.end()) {
            fprintf(stderr, "line %d: unknown kernel type %s\n", line_no, type_name.c_str());
            return 2;
        }
        std::unordered_map<std::string, CCAttr> attrs;
        std::string label = std::to_string(line_no);
        while (ls >> kv) {
            if (kv[0] == '@') {
                label = kv.substr(1);
                continue;
            }
            size_t eq = kv.find('=');
            std::string key = kv.substr(0, eq);
            char t = kv[eq + 1];
            std::string val = kv.substr(eq + 3);
            switch (t) {
                case 's':
                    attrs[key] = CCAttr(val);
                    break;
                case 'u':
                    attrs[key] = CCAttr((uint32_t)std::stoul(val));
                    break;
                case 'i':
                    attrs[key] = CCAttr((int32_t)std::stol(val));
                    break;
                case 'b':
                    attrs[key] = CCAttr((bool)(val == "1"));
                    break;
                case 'o':
                    attrs[key] = CCAttr(parse_operand(val));
                    break;
                default:
                    fprintf(stderr, "line %d: bad attr %s\n", line_no, kv.c_str());
                    return 2;
            }
        }
        CodeGenContext ctx(attrs);
        auto kernels =
                KernelGen::KernelPack::GetKernel(it->second, KernelGen::Arch::BAREMETAL).first;
        const KernelGen::KernelFunc* chosen = nullptr;
        for (auto* k : kernels) {
            bool ok = false;
            try {
                ok = k->IsAvailable(&ctx);
            } catch (...) {
                ok = false;
            }
            if (ok) {
                chosen = k;
                break;
            }
        }
        if (!chosen) {
            fprintf(stderr, "line %d: no available kernel (%s)\n", line_no, line.c_str());
            manifest << label << " NONE\n";
            ++fail;
            continue;
        }
        std::string sym = chosen->GetKernelSymbol(&ctx);
        manifest << label << " " << sym << "\n";
        if (written.insert(sym).second) {
            std::stringstream body;
            body << "#include <data_struct.h>\n";
            body << chosen->GetBodyGuardBegin(&ctx) << "\n";
            body << chosen->GetKernelBody(&ctx) << "\n";
            body << chosen->GetInitBody(&ctx) << "\n";
            body << chosen->GetWorkspaceBody(&ctx) << "\n";
            body << chosen->GetBodyGuardEnd(&ctx) << "\n";
            write_file(outdir + "/" + sym + ".c", body.str());
            for (auto& dep : chosen->GetDependInternalSymbol(&ctx)) {
                if (written.insert(dep.kernel_symbol).second) {
                    write_file(
                            outdir + "/" + dep.kernel_symbol + ".c",
                            dep.guard_begin + "\n" + dep.kernel_body + "\n" + dep.guard_end +
                                    "\n");
                }
            }
        }
    }
    return fail ? 1 : 0;
}
