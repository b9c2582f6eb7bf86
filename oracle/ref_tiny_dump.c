/* TEST INFRASTRUCTURE ONLY. Prints what the REFERENCE's own generated FlatBuffers reader
 * (runtime/src/cheader/model_reader.h over runtime/flatcc/include, both header-only and used where
 * they lie) sees in a `.tiny` file, one line per object, in the same text format as the product's
 * reader (megcc_gfx950_tiny_describe). The accessors are the ones runtime/src/parse.c:110-355,
 * vm/op.c:11-65 and vm/memforward.c:24-41 call.
 *
 *     ref_tiny_dump model.tiny > model.txt
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "model_reader.h"

#undef ns
#define ns(x) FLATBUFFERS_WRAP_NAMESPACE(MegCC, x)

static void put_ints(const char* key, flatbuffers_int32_vec_t v) {
    size_t n = v ? flatbuffers_int32_vec_len(v) : 0;
    printf(" %s=[", key);
    for (size_t i = 0; i < n; ++i)
        printf(i ? ",%d" : "%d", flatbuffers_int32_vec_at(v, i));
    printf("]");
}

static void put_typed(ns(DType_table_t) d, ns(Layout_table_t) l) {
    int type = 0, zero = 0, format = 0;
    float scale = 1.0f;
    if (d) {
        type = ns(DType_type(d));
        if (ns(DType_param_is_present(d))) {
            ns(DTypeParam_table_t) p = ns(DType_param(d));
            scale = ns(DTypeParam_scale(p));
            zero = ns(DTypeParam_zero_point(p));
        }
    }
    printf(" dtype=%d scale=%.9g zero_point=%d", type, scale, zero);
    put_ints("dims", l ? ns(Layout_dims(l)) : 0);
    put_ints("stride", l ? ns(Layout_stride(l)) : 0);
    if (l)
        format = ns(Layout_format(l));
    printf(" format=%d", format);
}

static const char* str(flatbuffers_string_t s) {
    return s ? s : "";
}

int main(int argc, char** argv) {
    if (argc != 2) {
        fprintf(stderr, "usage: %s model.tiny\n", argv[0]);
        return 2;
    }
    FILE* f = fopen(argv[1], "rb");
    if (!f) {
        perror(argv[1]);
        return 2;
    }
    fseek(f, 0, SEEK_END);
    long size = ftell(f);
    fseek(f, 0, SEEK_SET);
    void* buffer = aligned_alloc(64, (size + 63) / 64 * 64);
    if (fread(buffer, 1, size, f) != (size_t)size)
        return 2;
    fclose(f);

    ns(Model_table_t) model = ns(Model_as_root(buffer));
    if (!model)
        return 1;
    ns(Weight_vec_t) weights = ns(Model_weight_pool(model));
    ns(DeviceModel_vec_t) dms = ns(Model_device_models(model));
    size_t nw = weights ? ns(Weight_vec_len(weights)) : 0, nd = dms ? ns(DeviceModel_vec_len(dms)) : 0;
    printf("model name=%s model_id=%llu const_shape=%d weights=%zu device_models=%zu\n",
           str(ns(Model_name(model))), (unsigned long long)ns(Model_model_id(model)),
           ns(Model_const_shape(model)) ? 1 : 0, nw, nd);
    for (size_t i = 0; i < nw; ++i) {
        ns(Weight_table_t) w = ns(Weight_vec_at(weights, i));
        flatbuffers_int8_vec_t data = ns(Weight_data(w));
        size_t bytes = data ? flatbuffers_int8_vec_len(data) : 0;
        uint64_t h = 1469598103934665603ull;
        for (size_t k = 0; k < bytes; ++k)
            h = (h ^ (uint8_t)flatbuffers_int8_vec_at(data, k)) * 1099511628211ull;
        printf("weight %zu name=%s", i, str(ns(Weight_name(w))));
        put_typed(ns(Weight_dtype(w)), ns(Weight_layout(w)));
        printf(" use_count=%d checksum=%u compressed=%d bytes=%zu fnv=%016llx\n",
               ns(Weight_use_count(w)), ns(Weight_checksum(w)), ns(Weight_compressed(w)) ? 1 : 0,
               bytes, (unsigned long long)h);
    }
    for (size_t i = 0; i < nd; ++i) {
        ns(DeviceModel_table_t) d = ns(DeviceModel_vec_at(dms, i));
        ns(Tensor_vec_t) tensors = ns(DeviceModel_tensor_pool(d));
        ns(Instruction_union_vec_t) insts = ns(DeviceModel_instructions_union(d));
        size_t nt = tensors ? ns(Tensor_vec_len(tensors)) : 0;
        size_t ni = ns(Instruction_union_vec_len(insts));
        printf("device_model %zu device=%d tensors=%zu instructions=%zu tensor_memory=%llu", i,
               (int)ns(DeviceModel_device(d)), nt, ni,
               (unsigned long long)ns(DeviceModel_tensor_memory(d)));
        put_ints("inputs", ns(DeviceModel_inputs(d)));
        put_ints("outputs", ns(DeviceModel_outputs(d)));
        put_ints("weight_outputs", ns(DeviceModel_weight_outputs(d)));
        flatbuffers_string_vec_t names = ns(DeviceModel_weight_outputs_name(d));
        size_t nn = names ? flatbuffers_string_vec_len(names) : 0;
        printf(" weight_output_names=[");
        for (size_t k = 0; k < nn; ++k)
            printf(k ? ",%s" : "%s", flatbuffers_string_vec_at(names, k));
        printf("]\n");
        for (size_t k = 0; k < nt; ++k) {
            ns(Tensor_table_t) t = ns(Tensor_vec_at(tensors, k));
            printf("tensor %zu name=%s", k, str(ns(Tensor_name(t))));
            put_typed(ns(Tensor_dtype(t)), ns(Tensor_layout(t)));
            printf(" offset=%lld dynamic=%d use_count=%d\n", (long long)ns(Tensor_offset(t)),
                   ns(Tensor_dynamic(t)) ? 1 : 0, ns(Tensor_use_count(t)));
        }
        for (size_t k = 0; k < ni; ++k) {
            ns(Instruction_union_t) u = ns(Instruction_union_vec_at(insts, k));
            if (u.type == ns(Instruction_Opr)) {
                ns(Opr_table_t) o = (ns(Opr_table_t))u.value;
                printf("inst %zu Opr name=%s type=%s", k, str(ns(Opr_name(o))), str(ns(Opr_type(o))));
                put_ints("inputs", ns(Opr_inputs(o)));
                flatbuffers_int8_vec_t ty = (flatbuffers_int8_vec_t)ns(Opr_input_types(o));
                size_t nty = ty ? flatbuffers_int8_vec_len(ty) : 0;
                printf(" input_types=[");
                for (size_t j = 0; j < nty; ++j)
                    printf(j ? ",%d" : "%d", (int)flatbuffers_int8_vec_at(ty, j));
                printf("]");
                put_ints("outputs", ns(Opr_outputs(o)));
                ns(Workspace_table_t) ws = ns(Opr_workspace(o));
                printf(" ws_size=%lld ws_offset=%lld init_id=%d kernel_id=%d workspace_id=%d deduce_id=%d\n",
                       ws ? (long long)ns(Workspace_size(ws)) : 0LL,
                       ws ? (long long)ns(Workspace_offset(ws)) : 0LL, ns(Opr_init_id(o)),
                       ns(Opr_kernel_id(o)), ns(Opr_workspace_id(o)), ns(Opr_deduce_id(o)));
            } else if (u.type == ns(Instruction_MemForward)) {
                ns(MemForward_table_t) m = (ns(MemForward_table_t))u.value;
                printf("inst %zu MemForward input=%d output=%d offset=%d type=%d\n", k,
                       ns(MemForward_input(m)), ns(MemForward_output(m)), ns(MemForward_offset(m)),
                       (int)ns(MemForward_type(m)));
            } else if (u.type == ns(Instruction_DevMemAlloc)) {
                printf("inst %zu DevMemAlloc tensor=%d\n", k,
                       ns(DevMemAlloc_tensor((ns(DevMemAlloc_table_t))u.value)));
            } else if (u.type == ns(Instruction_DevMemFree)) {
                printf("inst %zu DevMemFree tensor=%d\n", k,
                       ns(DevMemFree_tensor((ns(DevMemFree_table_t))u.value)));
            } else {
                printf("inst %zu kind=%d\n", k, (int)u.type);
            }
        }
    }
    free(buffer);
    return 0;
}
