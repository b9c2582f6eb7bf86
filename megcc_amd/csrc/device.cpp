// Device seam: the hooks a TinyNN `Device` needs from a GPU (runtime/src/device.c:29-43 fills the
// same struct for the CPU), the staging copies of the Lite API, the library stream and the
// per-thread error text.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <vector>

#include "common.h"
#include "epilogue.h"

namespace mg {

static hipStream_t g_stream = nullptr;
static std::once_flag g_stream_once;
static thread_local char g_error[512] = "";

namespace {
struct OptionName {
    const char* name;  // option name; the environment variable is MEGCC_<NAME in capitals>
    bool Options::*field;
};
const OptionName kOptions[] = {
        {"nopws", &Options::no_pws},         {"nogevm", &Options::no_gevm},
        {"nofcb", &Options::no_fcb},         {"nosmall", &Options::no_small},
        {"nopm768", &Options::no_pm768},     {"nopm", &Options::no_pm},
        {"nodma512", &Options::no_dma512},   {"nopm256", &Options::no_pm256},
        {"nodma", &Options::no_dma},         {"nofcs", &Options::no_fcs},
        {"nopwshare", &Options::no_pwshare}, {"nohybrid", &Options::no_hybrid},
        {"nodot4", &Options::no_dot4},       {"nof32small", &Options::no_f32small},
        {"dw_generic", &Options::dw_generic}, {"no_graph", &Options::no_graph},
        {"nodwmfma", &Options::no_dwmfma},   {"nodwnchw", &Options::no_dwnchw},
        {"nofusesoftmax", &Options::no_fuse_softmax}, {"nopoolrows", &Options::no_poolrows}, {"nofirstmfma", &Options::no_firstmfma}, {"norowsplit", &Options::no_rowsplit}, {"nofusechain", &Options::no_fuse_chain}, {"nofusepwdw", &Options::no_fuse_pwdw}, {"fusepwdw", &Options::fuse_pwdw}, {"nofcone", &Options::no_fcone}, {"noxcdorder", &Options::no_xcdorder}, {"noaffine", &Options::no_affine}, {"nopipeline", &Options::no_pipeline},
};
struct KernelNote {
    const char* name;
    int v[5];
};
thread_local KernelNote g_note = {"", {-1, -1, -1, -1, -1}};
thread_local char g_note_text[160];
thread_local bool g_note_affine = false;  // the noted kernel requantises by the proven multiply-add
}  // namespace

Options& options() {
    static Options opt = [] {
        Options o = {};
        for (const OptionName& n : kOptions) {
            char env[48] = "MEGCC_";
            size_t k = strlen(env);
            for (const char* c = n.name; *c && k + 1 < sizeof(env); ++c)
                env[k++] = (*c >= 'a' && *c <= 'z') ? (char)(*c - 'a' + 'A') : *c;
            env[k] = 0;
            const char* v = getenv(env);
            o.*(n.field) = v && *v && strcmp(v, "0") != 0;
        }
        return o;
    }();
    return opt;
}

void note_kernel(const char* name, int a, int b, int c, int d, int e) {
    g_note.name = name;
    g_note.v[0] = a;
    g_note.v[1] = b;
    g_note.v[2] = c;
    g_note.v[3] = d;
    g_note.v[4] = e;
    g_note_affine = false;
}

void note_requant_affine(bool on) {
    g_note_affine = on;
}

static thread_local hipStream_t g_stream_override = nullptr;
static thread_local bool g_stream_override_on = false;
static std::mutex g_aux_lock;
static std::vector<hipStream_t> g_aux_streams;

hipStream_t main_stream() {
    std::call_once(g_stream_once, [] {
        if (hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking) != hipSuccess)
            g_stream = nullptr;  // falls back to the null stream; launches still work
    });
    return g_stream;
}

hipStream_t stream() {
    return g_stream_override_on ? g_stream_override : main_stream();
}

void set_stream_override(hipStream_t s, bool on) {
    g_stream_override = s;
    g_stream_override_on = on;
}

void register_aux_stream(hipStream_t s) {
    std::lock_guard<std::mutex> guard(g_aux_lock);
    g_aux_streams.push_back(s);
}

void unregister_aux_stream(hipStream_t s) {
    std::lock_guard<std::mutex> guard(g_aux_lock);
    for (size_t i = 0; i < g_aux_streams.size(); ++i)
        if (g_aux_streams[i] == s) {
            g_aux_streams.erase(g_aux_streams.begin() + (long)i);
            break;
        }
}

TinyNNStatus fail(TinyNNStatus st, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return st;
}

TinyNNStatus check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(TinyNN_ERROR_RUNTIME, "%s: launch failed: %s", what, hipGetErrorString(e));
    return TinyNN_SUCCESS;
}

int num_cus() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            n = prop.multiProcessorCount;
        if (n <= 0)
            n = 256;
    }
    return n;
}

TinyNNStatus check_io(
        Tensor** inputs, int nr_input, int want_in_min, int want_in_max, Tensor** outputs,
        int nr_output, const char* who) {
    MG_REQUIRE(inputs && outputs, TinyNN_ERROR_NULL_PTR, "%s: NULL tensor list", who);
    MG_REQUIRE(nr_input >= want_in_min && nr_input <= want_in_max, TinyNN_ERROR_OUT_OF_RANGE,
               "%s: %d inputs, expected %d..%d", who, nr_input, want_in_min, want_in_max);
    MG_REQUIRE(nr_output == 1, TinyNN_ERROR_OUT_OF_RANGE, "%s: %d outputs, expected 1", who,
               nr_output);
    for (int i = 0; i < nr_input; ++i)
        MG_REQUIRE(inputs[i] && inputs[i]->ptr, TinyNN_ERROR_NULL_PTR, "%s: input %d is NULL", who, i);
    MG_REQUIRE(outputs[0] && outputs[0]->ptr, TinyNN_ERROR_NULL_PTR, "%s: output is NULL", who);
    return TinyNN_SUCCESS;
}

}  // namespace mg

using namespace mg;

extern "C" {

void* megcc_gfx950_malloc(size_t length) {
    void* p = nullptr;
    if (length == 0)
        length = 1;
    if (hipMalloc(&p, length) != hipSuccess) {
        fail(TinyNN_ERROR_MEMORY_MALLOC, "hipMalloc(%zu) failed", length);
        return nullptr;
    }
    return p;
}

void megcc_gfx950_free(void* ptr) {
    if (ptr)
        (void)hipFree(ptr);
}

TinyNNStatus megcc_gfx950_init_device(Device* device) {
    MG_REQUIRE(device, TinyNN_ERROR_NULL_PTR, "init_device: NULL device");
    int n = 0;
    MG_REQUIRE(hipGetDeviceCount(&n) == hipSuccess && n > 0, TinyNN_ERROR_RUNTIME,
               "init_device: no HIP device");
    // (so that a first megcc_gfx950_conv2d_noalloc call under stream capture has nothing to set up)
    TinyNNStatus st = noalloc_scratch_setup();
    if (st != TinyNN_SUCCESS)
        return st;
    device->alignment = 256;
    device->device_type = TinyNN_GFX950;
    device->malloc = megcc_gfx950_malloc;
    device->free = megcc_gfx950_free;
    return TinyNN_SUCCESS;
}

TinyNNStatus megcc_gfx950_memcpy_h2d(void* dst, const void* src, size_t length) {
    MG_REQUIRE(dst && src, TinyNN_ERROR_NULL_PTR, "memcpy_h2d: NULL pointer");
    hipError_t e = hipMemcpyAsync(dst, src, length, hipMemcpyHostToDevice, stream());
    // pageable source: the copy is staged before the call returns, so `src` may be reused
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "memcpy_h2d: %s", hipGetErrorString(e));
    return TinyNN_SUCCESS;
}

TinyNNStatus megcc_gfx950_memcpy_d2h(void* dst, const void* src, size_t length) {
    MG_REQUIRE(dst && src, TinyNN_ERROR_NULL_PTR, "memcpy_d2h: NULL pointer");
    hipError_t e = hipMemcpyAsync(dst, src, length, hipMemcpyDeviceToHost, stream());
    if (e == hipSuccess)
        e = hipStreamSynchronize(stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "memcpy_d2h: %s", hipGetErrorString(e));
    return TinyNN_SUCCESS;
}

TinyNNStatus megcc_gfx950_memset(void* dst, int value, size_t length) {
    MG_REQUIRE(dst, TinyNN_ERROR_NULL_PTR, "memset: NULL pointer");
    hipError_t e = hipMemsetAsync(dst, value, length, stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "memset: %s", hipGetErrorString(e));
    return TinyNN_SUCCESS;
}

TinyNNStatus megcc_gfx950_wait(void) {
    hipError_t e = hipStreamSynchronize(main_stream());
    MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "wait: %s", hipGetErrorString(e));
    // (the streams on which models run the last operators of their forwards)
    std::vector<hipStream_t> aux;
    {
        std::lock_guard<std::mutex> guard(g_aux_lock);
        aux = g_aux_streams;
    }
    for (hipStream_t s : aux) {
        e = hipStreamSynchronize(s);
        MG_REQUIRE(e == hipSuccess, TinyNN_ERROR_RUNTIME, "wait: %s", hipGetErrorString(e));
    }
    return TinyNN_SUCCESS;
}

void* megcc_gfx950_stream(void) {
    return (void*)main_stream();
}

const char* megcc_gfx950_last_error(void) {
    return g_error;
}

const char* megcc_gfx950_last_kernel(void) {
    int n = snprintf(g_note_text, sizeof(g_note_text), "%s", g_note.name);
    for (int i = 0; i < 5 && g_note.v[i] != -1 && n > 0 && n < (int)sizeof(g_note_text); ++i)
        n += snprintf(g_note_text + n, sizeof(g_note_text) - n, "%c%d", i ? ',' : ':', g_note.v[i]);
    if (g_note_affine && n > 0 && n < (int)sizeof(g_note_text))
        snprintf(g_note_text + n, sizeof(g_note_text) - n, "+affine");
    return g_note_text;
}

int megcc_gfx950_requant_affine(int nonline_mode, float s_src, float s_flt, float s_dst, float* c, float* d) {
    const RequantAffine a = requant_affine_for(nonline_mode, s_src, s_flt, s_dst);
    if (c)
        *c = a.c;
    if (d)
        *d = a.d;
    return a.d != 0.f;
}

TinyNNStatus megcc_gfx950_set_option(const char* name, int value) {
    MG_REQUIRE(name, TinyNN_ERROR_NULL_PTR, "set_option: NULL name");
    for (const OptionName& n : kOptions)
        if (strcmp(n.name, name) == 0) {
            options().*(n.field) = value != 0;
            return TinyNN_SUCCESS;
        }
    return fail(TinyNN_ERROR_NO_FOUND, "set_option: unknown option '%s'", name);
}

}  // extern "C"
