// Reader for MegCC's `.tiny` model files (a FlatBuffers binary of runtime/schema/model.fbs).
// Everything is copied out of the file into plain structs after bounds checks, so a truncated or
// hostile file ends in an error message, never in an out-of-range read.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace mg {
namespace tiny {

// values of the schema's enums (runtime/schema/model.fbs)
enum : int {
    DT_Float32 = 0, DT_Float16 = 1, DT_Int32 = 2, DT_Int8 = 3, DT_Int16 = 4, DT_Uint8 = 5,
    DT_QInt8 = 100, DT_QInt32 = 101, DT_QUint8 = 102,
};
enum : int {
    DEV_BARE_METAL = 0, DEV_ARM64, DEV_ARM32, DEV_ARM64_V82, DEV_ARM32_V82, DEV_OPENCL_MALI,
    DEV_WEB_ASSEMBLY,
    DEV_GFX950  // the value a compiler with the gfx950 target appends to the list
};
enum : int { INST_Opr = 1, INST_DevMemAlloc = 2, INST_DevMemFree = 3, INST_MemForward = 4, INST_END = 18 };
enum : int { TT_TENSOR = 0, TT_WEIGHT = 1 };

struct DType {
    int type = 0;
    float scale = 1.0f;  // schema default
    int zero_point = 0;
    bool has_param = false;
};

struct Layout {
    std::vector<int32_t> dims, stride;
    int format = 0;
};

struct TensorInfo {
    DType dtype;
    Layout layout;
    int64_t offset = 0;
    bool dynamic = false;
    int32_t use_count = 0;
    std::string name;
};

struct WeightInfo {
    DType dtype;
    Layout layout;
    int32_t use_count = 0;
    const int8_t* data = nullptr;  // points into the file buffer
    size_t data_bytes = 0;
    std::string name;
    uint32_t checksum = 0;
    bool compressed = false;
};

struct Instruction {
    int kind = 0;  // INST_*
    // Opr
    std::string name, type;
    std::vector<int32_t> inputs, outputs;
    std::vector<int8_t> input_types;
    int64_t ws_size = 0, ws_offset = 0;
    int32_t init_id = -1, kernel_id = 0, workspace_id = -1, deduce_id = -1;
    // MemForward
    int32_t fwd_input = 0, fwd_output = 0, fwd_offset = 0;
    int fwd_type = 0;
    // DevMemAlloc / DevMemFree
    int32_t mem_tensor = 0;
};

struct DeviceModelInfo {
    int device = 0;
    std::vector<TensorInfo> tensors;
    std::vector<Instruction> instructions;
    uint64_t tensor_memory = 0;
    std::vector<int32_t> inputs, outputs, weight_outputs;
    std::vector<std::string> weight_output_names;
};

struct ModelInfo {
    std::vector<WeightInfo> weights;
    std::vector<DeviceModelInfo> device_models;
    bool const_shape = false;
    std::string name;
    uint64_t model_id = 0;
};

// Parses `size` bytes at `buffer`. On failure returns false and explains in *error.
bool read_model(const void* buffer, size_t size, ModelInfo* out, std::string* error);

// One line per object, every field of the tables this runtime understands: the text the tests
// compare with what the reference's own generated reader sees in the same file.
std::string describe(const ModelInfo& m);

}  // namespace tiny
}  // namespace mg
