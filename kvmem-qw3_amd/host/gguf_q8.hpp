// GGUF v3 container reader for the tensors this path consumes, and the step from a
// Q8_0 tensor in the file to a device-resident split-plane weight.
//
// Declares the part of the reference's reader interface that the weight loader uses
// (include/qw3/gguf.hpp:13-78): same class and member names, and a std::runtime_error
// under the same conditions as the reference's reader (src/gguf.cpp:205-392:
// unreadable or empty file, wrong magic, version != 3, a file that ends inside the
// header, tensor rank above 8, a tensor outside the file, a block type that does not
// divide into whole blocks); the implementation and its messages are this library's
// own.  The tokenizer/model-info helpers of the
// reference's class are outside this path and absent.  The file is mapped
// read-only; tensor data is handed to the backend straight from the mapping, as
// the reference's model source does (src/model_source.cpp:108-127).
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "hip_q8_backend.hpp"

namespace qw3 {

enum class GgufValueType : uint32_t {
    Uint8 = 0, Int8 = 1, Uint16 = 2, Int16 = 3, Uint32 = 4, Int32 = 5, Float32 = 6,
    Bool = 7, String = 8, Array = 9, Uint64 = 10, Int64 = 11, Float64 = 12,
};

struct GgufValue {
    GgufValueType type{};
    std::string string_value;
    std::vector<std::string> string_array;   // arrays of strings only; other arrays are skipped
    uint64_t unsigned_value = 0;
    int64_t signed_value = 0;
    double float_value = 0.0;
    bool bool_value = false;
};

struct GgufTensorInfo {
    std::string name;
    std::vector<uint64_t> dims;   // dims[0] is the contiguous one: cols of a weight
    uint32_t type = 0;            // ggml type id; 8 = Q8_0, 0 = F32
    uint64_t rel_offset = 0;
    uint64_t abs_offset = 0;
    uint64_t elements = 0;
    uint64_t bytes = 0;
};

class GgufFile {
public:
    explicit GgufFile(const std::string &path);
    ~GgufFile();
    GgufFile(const GgufFile &) = delete;
    GgufFile &operator=(const GgufFile &) = delete;

    const std::string &path() const;
    uint64_t size() const;
    const uint8_t *data() const;
    uint32_t version() const;
    uint32_t alignment() const;
    uint64_t tensor_data_offset() const;
    const std::unordered_map<std::string, GgufValue> &metadata() const;
    const std::vector<GgufTensorInfo> &tensors() const;
    const GgufTensorInfo *find_tensor(const std::string &name) const;

private:
    struct Impl;
    std::unique_ptr<Impl> impl_;
};

std::string gguf_tensor_type_name(uint32_t type);
// Bytes of `elements` values of a ggml type (0 for a type this reader does not size);
// throws when a block-quantized type does not divide into whole blocks.
uint64_t gguf_tensor_type_size(uint32_t type, uint64_t elements);

// rows / cols of a tensor as the weight loader sees them (src/qwen_weights.cpp:12-22):
// cols = dims[0], rows = product of the others.
uint64_t gguf_tensor_rows(const GgufTensorInfo &t);
uint64_t gguf_tensor_cols(const GgufTensorInfo &t);

// Uploads the named Q8_0 tensor (interleaved 34-byte blocks in the file) as a
// split-plane device weight (src/qwen_weights.cpp:287-297).  nullptr when the tensor
// is missing, is not Q8_0 or the upload fails.
std::unique_ptr<DeviceWeight> gguf_upload_q8_0(HipQ8Backend &backend, const GgufFile &file, const std::string &name);

}  // namespace qw3
