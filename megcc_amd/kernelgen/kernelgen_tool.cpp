// kernelgen_tool <spec-file> <outdir>
//
// Stand-alone driver of the gfx950 KernelGen target, the counterpart of MegCC's kernel_exporter
// (compiler/tools/kernel_exporter/exporter_imp.cpp:40-100): every line of the spec file is one
// operator's attribute bag (the keys KernelMaterialization.cpp:70-158 passes to KernelGen); the
// first available candidate of Gfx950KernelPack::GetKernel is asked for its symbol and its
// kernel / init / workspace bodies, which are written to <outdir>/<symbol>.c, and
// "<label> <symbol>" is appended to <outdir>/manifest.txt ("<label> NONE" when no kernel of this
// target is available).
//
// Spec line:  <KernType> [@label] <key>=<t>:<value> ...
//   t = s string | u uint32 | i int32 | b bool | o operand "d0xd1x..|dtype|scale"
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iostream>
#include <map>
#include <set>
#include <sstream>

#include "KernelGen.h"

using namespace megcc_gfx950;

static CCOperand parse_operand(const std::string& v) {
    CCOperand op;
    size_t p0 = v.find('|');
    std::string shape = v.substr(0, p0);
    std::string rest = p0 == std::string::npos ? "" : v.substr(p0 + 1);
    size_t p1 = rest.find('|');
    std::string dtype = rest.substr(0, p1);
    std::string scale = p1 == std::string::npos ? "" : rest.substr(p1 + 1);
    std::stringstream ss(shape);
    std::string tok;
    while (std::getline(ss, tok, 'x'))
        if (!tok.empty())
            op.shape.push_back(std::stoull(tok));
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

int main(int argc, char** argv) {
    static const std::map<std::string, KernType> types = {
            {"ConvKernel", KernType::ConvKernel},
            {"ElemwiseKernel", KernType::ElemwiseKernel},
            {"ElemwiseMultiKernel", KernType::ElemwiseMultiKernel},
            {"PoolingKernel", KernType::PoolingKernel},
            {"MatrixMulKernel", KernType::MatrixMulKernel},
            {"ReduceKernel", KernType::ReduceKernel},
            {"TypeCvtKernel", KernType::TypeCvtKernel},
            {"RelayoutKernel", KernType::RelayoutKernel},
            {"ConcatKernel", KernType::ConcatKernel},
            {"ResizeKernel", KernType::ResizeKernel},
            {"FusedElemwiseKernel", KernType::FusedElemwiseKernel},
    };
    if (argc == 2 && std::string(argv[1]) == "--null-symbols") {
        // what every kernel answers to the exporter's name filter, which has no context
        for (auto& t : types)
            for (auto* k : Gfx950KernelPack::GetKernel(t.second))
                printf("%s\n", k->GetKernelSymbol(nullptr).c_str());
        return 0;
    }
    if (argc != 3) {
        fprintf(stderr, "usage: %s <spec-file> <outdir> | --null-symbols\n", argv[0]);
        return 2;
    }
    std::ifstream spec(argv[1]);
    if (!spec) {
        fprintf(stderr, "cannot read %s\n", argv[1]);
        return 2;
    }
    const std::string outdir = argv[2];
    std::ofstream manifest(outdir + "/manifest.txt");
    std::set<std::string> written;
    std::string line;
    int line_no = 0;
    while (std::getline(spec, line)) {
        ++line_no;
        if (line.empty() || line[0] == '#')
            continue;
        std::stringstream ls(line);
        std::string type_name, kv, label = std::to_string(line_no);
        ls >> type_name;
        auto it = types.find(type_name);
        if (it == types.end()) {
            fprintf(stderr, "line %d: unknown kernel type %s\n", line_no, type_name.c_str());
            return 2;
        }
        TContext ctx;
        while (ls >> kv) {
            if (kv[0] == '@') {
                label = kv.substr(1);
                continue;
            }
            size_t eq = kv.find('=');
            if (eq == std::string::npos || eq + 2 >= kv.size() || kv[eq + 2] != ':') {
                fprintf(stderr, "line %d: bad attribute %s\n", line_no, kv.c_str());
                return 2;
            }
            const std::string key = kv.substr(0, eq), val = kv.substr(eq + 3);
            switch (kv[eq + 1]) {
                case 's': ctx.setAttr(key, val); break;
                case 'u':
                case 'i': ctx.setAttr(key, (int64_t)std::stoll(val)); break;
                case 'b': ctx.setAttr(key, val == "1"); break;
                case 'o': ctx.setAttr(key, parse_operand(val)); break;
                default:
                    fprintf(stderr, "line %d: bad attribute type in %s\n", line_no, kv.c_str());
                    return 2;
            }
        }
        const KernelFuncBase* chosen = nullptr;
        for (auto* k : Gfx950KernelPack::GetKernel(it->second))
            if (k->IsAvailable(&ctx)) {
                chosen = k;
                break;
            }
        if (!chosen) {
            manifest << label << " NONE\n";
            continue;
        }
        const std::string sym = chosen->GetKernelSymbol(&ctx);
        manifest << label << " " << sym << "\n";
        if (written.insert(sym).second) {
            std::ofstream f(outdir + "/" + sym + ".c");
            f << "// generated by the gfx950 KernelGen target\n"
              << chosen->GetKernelBody(&ctx) << "\n"
              << chosen->GetInitBody(&ctx) << "\n"
              << chosen->GetWorkspaceBody(&ctx) << "\n";
        }
    }
    return 0;
}
