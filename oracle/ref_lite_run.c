/* TEST INFRASTRUCTURE ONLY -- never linked into or called by the product library.
 *
 * A caller of MegCC's TinyNN runtime that knows nothing about GPUs: the public LITE C API
 * (runtime/include/lite-c/network_c.h, tensor_c.h), host buffers in and out. Linked by
 * oracle/Makefile with the reference's OWN runtime sources (runtime/src: parse.c, init.c, vm.c,
 * vm/<all>.c, lite/<all>.c, ...) compiled from where they lie, with
 * megcc_amd/upstream/runtime_device_gfx950.patch applied to scratch copies of the files it touches,
 * the kernel tables written by oracle/ref_gfx950_export.cpp, and libmegcc_gfx950.so. The whole
 * reference call stack - LITE_load_model_from_path -> parse_model -> init_model_weights (three
 * phase kernel init) -> init_model_memory -> LITE_forward -> vm_instruction_call ->
 * execute_single_opr -> kernels[id](...) - then runs on the GPU.
 *
 * usage: ref_lite_run <model.tiny> <forwards> <in_0.bin> ... -- <out_0.bin> ...
 * Inputs and outputs in the model's own order; every forward re-stages the inputs. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "lite-c/common_enum_c.h"
#include "lite-c/network_c.h"
#include "lite-c/tensor_c.h"

#define CHECK(call)                                                        \
    do {                                                                   \
        int st_ = (call);                                                  \
        if (st_ != 0) {                                                    \
            fprintf(stderr, "ref_lite_run: %s -> status %d\n", #call, st_); \
            return 1;                                                      \
        }                                                                  \
    } while (0)

static void* read_file(const char* path, size_t want) {
    FILE* f = fopen(path, "rb");
    if (!f)
        return NULL;
    void* p = malloc(want ? want : 1);
    size_t got = fread(p, 1, want, f);
    int more = fgetc(f) != EOF;
    fclose(f);
    if (got != want || more) {
        free(p);
        return NULL;
    }
    return p;
}

int main(int argc, char** argv) {
    if (argc < 4) {
        fprintf(stderr, "usage: %s <model.tiny> <forwards> <in.bin>... -- <out.bin>...\n", argv[0]);
        return 2;
    }
    const int forwards = atoi(argv[2]);
    int sep = 3;
    while (sep < argc && strcmp(argv[sep], "--"))
        ++sep;
    const int nr_in_files = sep - 3, nr_out_files = argc - sep - 1;

    LiteNetwork net;
    CHECK(LITE_make_network(&net, *default_config(), *default_network_io()));
    CHECK(LITE_load_model_from_path(net, argv[1]));

    size_t nr_in = 0, nr_out = 0;
    CHECK(LITE_get_all_input_name(net, &nr_in, NULL));
    CHECK(LITE_get_all_output_name(net, &nr_out, NULL));
    if ((int)nr_in != nr_in_files || (int)nr_out != nr_out_files) {
        fprintf(stderr, "ref_lite_run: the model has %zu inputs and %zu outputs, %d and %d files given\n",
                nr_in, nr_out, nr_in_files, nr_out_files);
        return 2;
    }
    const char** in_names = (const char**)malloc(sizeof(char*) * (nr_in + 1));
    const char** out_names = (const char**)malloc(sizeof(char*) * (nr_out + 1));
    CHECK(LITE_get_all_input_name(net, NULL, in_names));
    CHECK(LITE_get_all_output_name(net, NULL, out_names));

    void** in_data = (void**)calloc(nr_in + 1, sizeof(void*));
    size_t* in_bytes = (size_t*)calloc(nr_in + 1, sizeof(size_t));
    LiteTensor* in_t = (LiteTensor*)calloc(nr_in + 1, sizeof(LiteTensor));
    for (size_t i = 0; i < nr_in; ++i) {
        CHECK(LITE_get_io_tensor(net, in_names[i], LITE_INPUT, &in_t[i]));
        CHECK(LITE_get_tensor_total_size_in_byte(in_t[i], &in_bytes[i]));
        in_data[i] = read_file(argv[3 + i], in_bytes[i]);
        if (!in_data[i]) {
            fprintf(stderr, "ref_lite_run: %s does not hold the %zu bytes of input %s\n", argv[3 + i],
                    in_bytes[i], in_names[i]);
            return 2;
        }
    }
    for (int it = 0; it < forwards; ++it) {
        for (size_t i = 0; i < nr_in; ++i)
            CHECK(LITE_reset_tensor_memory(in_t[i], in_data[i], in_bytes[i]));
        CHECK(LITE_forward(net));
        CHECK(LITE_wait(net));
    }
    for (size_t i = 0; i < nr_out; ++i) {
        LiteTensor t;
        size_t bytes = 0;
        void* data = NULL;
        CHECK(LITE_get_io_tensor(net, out_names[i], LITE_OUTPUT, &t));
        CHECK(LITE_get_tensor_total_size_in_byte(t, &bytes));
        CHECK(LITE_get_tensor_memory(t, &data));
        FILE* f = fopen(argv[sep + 1 + i], "wb");
        if (!f || fwrite(data, 1, bytes, f) != bytes) {
            fprintf(stderr, "ref_lite_run: cannot write %s\n", argv[sep + 1 + i]);
            return 1;
        }
        fclose(f);
        printf("output %s: %zu bytes\n", out_names[i], bytes);
    }
    CHECK(LITE_destroy_network(net));
    return 0;
}
