// Host-side bounds audit of kernels that load unconditionally from clamped indices.
//
// Linked with the library's OWN kernel sources (gemm_f32.hip, gevm_f32.hip, conv_f32_small.hip,
// fc_stream.hip, fc_gevm_q8.hip) compiled as host C++ against tests/host_audit/hip/hip_runtime.h,
// where a launch runs every thread of every workgroup one after the other on the CPU. The operand
// buffers are fenced: each sits at the very end (then, in a second pass, at the very start) of a
// mapping whose neighbouring page is inaccessible, so a load or store one element outside a tensor
// ends the process with SIGSEGV instead of reading a stray value. Nothing here restates an index
// formula: the addresses dereferenced are the ones the kernels compute.
//
// stdin: one case per line, stdout: "ok <line>" per case; exit status 0 when all of them ran.
//   mm     M K N ta tb lda_pad ldb_pad ws     f32 MatMul through megcc_gfx950_matmul (gemm / gevm); ws = 1: with split-K room
//   conv   n ic ih iw oc k s p d bias ws      f32 NCHW convolution through the implicit GEMM
//   small  n ic ih iw oc k s p d bias         f32 NCHW convolution through conv_f32_small (k = 1 or 3)
//   dwf32  n c ih iw k s p bias               f32 channel-wise layer in NCHW44
//   first  n ic ih iw oc k s p bias           f32 first layer, NCHW source -> NCHW44 result
//   fcone  M K OC packed_bytes bias           qsi8 FullyConnected, M <= 64, one launch
//   fcgevm M K OC packed_bytes bias           qsi8 FullyConnected, M <= 4
#include <hip/hip_runtime.h>
#include <signal.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <sys/mman.h>
#include <unistd.h>

#include <sstream>
#include <string>
#include <vector>

#include "common.h"
#include "conv_geom.h"
#include "gevm_f32.h"

namespace mg {
// what the kernel sources expect from the rest of the library
hipStream_t stream() { return nullptr; }
int num_cus() { return 256; }
TinyNNStatus fail(TinyNNStatus st, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vfprintf(stderr, fmt, ap);
    va_end(ap);
    fputc('\n', stderr);
    return st;
}
Options& options() {
    static Options o = {};
    return o;
}
void note_kernel(const char*, int, int, int, int, int) {}
TinyNNStatus check_launch(const char*) { return TinyNN_SUCCESS; }
TinyNNStatus check_io(Tensor** in, int nin, int lo, int hi, Tensor** out, int nout, const char* who) {
    if (!in || !out || nin < lo || nin > hi || nout != 1)
        return fail(TinyNN_ERROR_OUT_OF_RANGE, "%s: operand count", who);
    return TinyNN_SUCCESS;
}
// dynamic LDS of fc_stream.hip / fc_gevm_q8.hip (`extern __shared__ ... name[]`)
__attribute__((aligned(16))) int8_t lds[160 * 1024];
__attribute__((aligned(16))) int fg_lds[40 * 1024];

size_t gemm_f32_workspace_bytes(long M, long N, long K, bool conv);
size_t conv_f32_gemm_workspace_bytes(const ConvGeom& g);
TinyNNStatus conv_f32_gemm_launch(const ConvGeom&, const void*, const void*, const void*, void*, const Workspace*);
bool conv_f32_small_supported(const ConvGeom& g);
TinyNNStatus conv_f32_small_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool dwconv44_f32_supported(const ConvGeom&);
TinyNNStatus dwconv44_f32_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool conv_first_f32_supported(const ConvGeom&);
TinyNNStatus conv_first_f32_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool fc_one_supported(const ConvGeom& g, const void* src);
TinyNNStatus fc_one_launch(const ConvGeom&, const void*, const void*, const void*, void*);
bool fc_gevm_q8_supported(const ConvGeom& g);
TinyNNStatus fc_gevm_q8_launch(const ConvGeom&, const void*, const void*, const void*, void*);
}  // namespace mg

extern "C" TinyNNStatus megcc_gfx950_matmul(
        const MegccMatMulAttr*, Tensor**, int, Tensor**, int, const Workspace*, const RuntimeOpt*);

static std::string g_case;
static void on_fault(int, siginfo_t* info, void*) {
    char buf[512];
    int n = snprintf(buf, sizeof(buf), "OUT OF BOUNDS: access at %p while running: %s\n", info->si_addr,
                     g_case.c_str());
    (void)!write(2, buf, n);
    _exit(3);
}

// `bytes` usable bytes whose end (at_end) or start touches an inaccessible page
struct Fenced {
    void* map = nullptr;
    size_t map_bytes = 0;
    char* ptr = nullptr;
    Fenced(size_t bytes, bool at_end, size_t align) {
        const size_t page = 4096, body = (bytes + page - 1) / page * page + page;
        map_bytes = body + 2 * page;
        map = mmap(nullptr, map_bytes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
        if (map == MAP_FAILED) {
            perror("mmap");
            exit(2);
        }
        char* base = (char*)map;
        mprotect(base, page, PROT_NONE);
        mprotect(base + page + body, page, PROT_NONE);
        if (at_end) {
            // the last byte right below the fence, moved down only as far as `align` demands
            size_t start = page + body - bytes;
            start -= start % align;
            ptr = base + start;
        } else {
            ptr = base + page;
        }
        memset(ptr, 1, bytes);
    }
    ~Fenced() { munmap(map, map_bytes); }
};

static Tensor tensor2d(void* p, int rows, int cols, long ld) {
    Tensor t;
    memset(&t, 0, sizeof(t));
    t.ptr = p;
    t.dtype.type_enum = TinyNN_FLOAT;
    t.layout.nr_dim = 2;
    t.layout.dims[0] = rows;
    t.layout.dims[1] = cols;
    t.layout.stride[0] = (int)ld;
    t.layout.stride[1] = 1;
    return t;
}

static bool run_case(const std::string& line, bool at_end) {
    using namespace mg;
    std::stringstream ss(line);
    std::string kind;
    ss >> kind;
    if (kind == "mm") {
        int M, K, N, ta, tb, pa, pb, ws;
        ss >> M >> K >> N >> ta >> tb >> pa >> pb >> ws;
        const int ar = ta ? K : M, ac = ta ? M : K, br = tb ? N : K, bc = tb ? K : N;
        const long lda = ac + pa, ldb = bc + pb;
        // a padded last row ends with its last element, not with its padding
        Fenced A(((size_t)(ar - 1) * lda + ac) * 4, at_end, 16), B(((size_t)(br - 1) * ldb + bc) * 4, at_end, 16),
                Cm((size_t)M * N * 4, at_end, 16);
        const size_t wsb = ws ? gemm_f32_workspace_bytes(M, N, K, false) : 0;
        Fenced W(wsb ? wsb : 16, at_end, 16);
        Tensor a = tensor2d(A.ptr, ar, ac, lda), b = tensor2d(B.ptr, br, bc, ldb), c = tensor2d(Cm.ptr, M, N, N);
        Tensor *in[2] = {&a, &b}, *out[1] = {&c};
        MegccMatMulAttr attr;
        memset(&attr, 0, sizeof(attr));
        attr.transpose_a = ta;
        attr.transpose_b = tb;
        Workspace w = {wsb ? W.ptr : nullptr, wsb, 0};
        return megcc_gfx950_matmul(&attr, in, 2, out, 1, &w, nullptr) == TinyNN_SUCCESS;
    }
    if (kind == "conv" || kind == "small") {
        ConvGeom g;
        memset(&g, 0, sizeof(g));
        int k, s, p, d, bias, ws = 0;
        ss >> g.n >> g.ic >> g.ih >> g.iw >> g.oc >> k >> s >> p >> d >> bias;
        if (kind == "conv")
            ss >> ws;
        g.fh = g.fw = k, g.sh = g.sw = s, g.ph = g.pw = p, g.dh = g.dw = d;
        g.oh = (g.ih + 2 * p - (d * (k - 1) + 1)) / s + 1;
        g.ow = (g.iw + 2 * p - (d * (k - 1) + 1)) / s + 1;
        g.groups = 1, g.fmt = MEGCC_FMT_NCHW, g.act = MEGCC_NONLINE_RELU, g.has_bias = bias;
        Fenced src((size_t)g.n * g.ic * g.ih * g.iw * 4, at_end, 16), flt((size_t)g.oc * g.ic * k * k * 4, at_end, 16),
                b((size_t)g.oc * 4, at_end, 4), dst((size_t)g.n * g.oc * g.oh * g.ow * 4, at_end, 16);
        if (kind == "small") {
            if (!conv_f32_small_supported(g)) {
                fprintf(stderr, "not a conv_f32_small layer: %s\n", line.c_str());
                return false;
            }
            return conv_f32_small_launch(g, src.ptr, flt.ptr, bias ? b.ptr : nullptr, dst.ptr) == TinyNN_SUCCESS;
        }
        const size_t wsb = ws ? conv_f32_gemm_workspace_bytes(g) : 0;
        Fenced W(wsb ? wsb : 16, at_end, 16);
        Workspace w = {wsb ? W.ptr : nullptr, wsb, 0};
        return conv_f32_gemm_launch(g, src.ptr, flt.ptr, bias ? b.ptr : nullptr, dst.ptr, &w) == TinyNN_SUCCESS;
    }
    if (kind == "dwf32" || kind == "first") {
        ConvGeom g;
        memset(&g, 0, sizeof(g));
        int k, s, p, bias;
        ss >> g.n >> g.ic >> g.ih >> g.iw;
        if (kind == "first")
            ss >> g.oc;
        else
            g.oc = g.ic;
        ss >> k >> s >> p >> bias;
        g.fh = g.fw = k, g.sh = g.sw = s, g.ph = g.pw = p, g.dh = g.dw = 1;
        g.oh = (g.ih + 2 * p - k) / s + 1;
        g.ow = (g.iw + 2 * p - k) / s + 1;
        g.groups = kind == "first" ? 1 : g.ic;
        g.fmt = kind == "first" ? MEGCC_FMT_NCHW_NCHW44 : MEGCC_FMT_NCHW44;
        g.act = MEGCC_NONLINE_H_SWISH, g.has_bias = bias;
        const size_t taps = (size_t)k * k * (kind == "first" ? (size_t)g.ic * g.oc : (size_t)g.ic);
        Fenced src((size_t)g.n * g.ic * g.ih * g.iw * 4, at_end, 16), flt(taps * 4, at_end, 16),
                b((size_t)g.oc * 4, at_end, 16), dst((size_t)g.n * g.oc * g.oh * g.ow * 4, at_end, 16);
        if (kind == "first") {
            if (!conv_first_f32_supported(g)) {
                fprintf(stderr, "not a conv_first_f32 layer: %s\n", line.c_str());
                return false;
            }
            return conv_first_f32_launch(g, src.ptr, flt.ptr, bias ? b.ptr : nullptr, dst.ptr) == TinyNN_SUCCESS;
        }
        if (!dwconv44_f32_supported(g)) {
            fprintf(stderr, "not a dwconv44_f32 layer: %s\n", line.c_str());
            return false;
        }
        return dwconv44_f32_launch(g, src.ptr, flt.ptr, bias ? b.ptr : nullptr, dst.ptr) == TinyNN_SUCCESS;
    }
    if (kind == "fcone" || kind == "fcgevm") {
        ConvGeom g;
        memset(&g, 0, sizeof(g));
        long packed;
        int bias;
        ss >> g.n >> g.ic >> g.oc >> packed >> bias;
        g.ih = g.iw = g.oh = g.ow = g.fh = g.fw = g.sh = g.sw = g.dh = g.dw = 1;
        g.groups = 1, g.fmt = MEGCC_FMT_NCHW, g.act = MEGCC_NONLINE_RELU, g.has_bias = bias;
        g.s_src = g.s_flt = 0.01f, g.s_dst = 0.1f;
        Fenced src((size_t)g.n * g.ic, at_end, 16), wp((size_t)packed, at_end, 16), b((size_t)g.oc * 4, at_end, 4),
                dst((size_t)g.n * g.oc, at_end, g.oc % 4 ? 1 : 4);
        if (kind == "fcone") {
            if (!fc_one_supported(g, src.ptr)) {
                fprintf(stderr, "not an fc_one layer: %s\n", line.c_str());
                return false;
            }
            return fc_one_launch(g, src.ptr, wp.ptr, bias ? b.ptr : nullptr, dst.ptr) == TinyNN_SUCCESS;
        }
        if (!fc_gevm_q8_supported(g)) {
            fprintf(stderr, "not an fc_gevm_q8 layer: %s\n", line.c_str());
            return false;
        }
        return fc_gevm_q8_launch(g, src.ptr, wp.ptr, bias ? b.ptr : nullptr, dst.ptr) == TinyNN_SUCCESS;
    }
    fprintf(stderr, "unknown case kind: %s\n", line.c_str());
    return false;
}

int main() {
    struct sigaction sa;
    memset(&sa, 0, sizeof(sa));
    sa.sa_sigaction = on_fault;
    sa.sa_flags = SA_SIGINFO;
    sigaction(SIGSEGV, &sa, nullptr);
    sigaction(SIGBUS, &sa, nullptr);
    char buf[512];
    int n = 0;
    while (fgets(buf, sizeof(buf), stdin)) {
        std::string line(buf);
        while (!line.empty() && (line.back() == '\n' || line.back() == ' '))
            line.pop_back();
        if (line.empty() || line[0] == '#')
            continue;
        for (int at_end = 1; at_end >= 0; --at_end) {
            g_case = line + (at_end ? "  [buffers end at a fence]" : "  [buffers start at a fence]");
            if (!run_case(line, at_end != 0)) {
                fprintf(stderr, "FAILED: %s\n", g_case.c_str());
                return 1;
            }
        }
        printf("ok %s\n", line.c_str());
        fflush(stdout);
        ++n;
    }
    printf("audited %d cases\n", n);
    return 0;
}
