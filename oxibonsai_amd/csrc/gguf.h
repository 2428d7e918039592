// gguf.h — read-only view of a GGUF file (versions 2 and 3), host code only.
//
// Follows the reference's reader (crates/oxibonsai-core/src/gguf/reader.rs:11-80, header.rs, metadata.rs,
// tensor_info.rs): little-endian header {magic 0x46554747, version, tensor count, metadata count}, metadata
// key/value pairs, tensor infos {name, dims, type id, offset}, then the tensor data section, which starts at the
// next multiple of `general.alignment` (default 32); tensor offsets count from there.  The file is memory-mapped;
// tensor data is never copied by the parser.
#pragma once
#include <stddef.h>
#include <stdint.h>

#include <map>
#include <string>
#include <vector>

namespace oxb {

enum GgufTensorType : uint32_t {  // crates/oxibonsai-core/src/gguf/types.rs:17-44 (the ids this tier consumes)
    GGUF_F32 = 0,
    GGUF_F16 = 1,
    GGUF_Q1_0_G128 = 41,
    GGUF_TQ2_0_G128 = 42,
};

struct GgufValue {
    uint32_t type = 0;  // GgufValueType id (types.rs:161-175); arrays keep only their element type and count
    uint64_t u = 0;     // unsigned integers, bool
    int64_t i = 0;      // signed integers
    double f = 0.0;     // floats
    std::string s;
    uint32_t elem_type = 0;
    uint64_t count = 0;
};

struct GgufTensor {
    std::string name;
    std::vector<uint64_t> shape;  // GGUF order: shape[0] = in features (k), shape[1] = out features (rows)
    uint32_t type = 0;
    uint64_t offset = 0;          // from the start of the data section
    const uint8_t* data = nullptr;
    uint64_t bytes = 0;
};

class GgufFile {
public:
    GgufFile() = default;
    ~GgufFile();
    GgufFile(const GgufFile&) = delete;
    GgufFile& operator=(const GgufFile&) = delete;

    // Maps and parses the file; on failure returns false and leaves the reason in err.
    bool open(const char* path, std::string* err);

    uint32_t version = 0, alignment = 32;
    uint64_t n_tensors = 0, n_kv = 0;
    size_t data_offset = 0;
    std::map<std::string, GgufValue> meta;
    std::map<std::string, GgufTensor> tensors;

    const GgufTensor* find(const std::string& name) const;
    // Typed metadata access with the reference's conversions (metadata.rs:28-66): u32 from Uint32 / Uint64 / Int32
    // when it fits, f32 from Float32 / Float64.
    bool get_u32(const std::string& key, uint32_t* out) const;
    bool get_f32(const std::string& key, float* out) const;
    bool get_str(const std::string& key, std::string* out) const;

private:
    const uint8_t* base_ = nullptr;
    size_t size_ = 0;
    int fd_ = -1;
};

// Bytes of a tensor of `elements` values of the given type, or 0 for a type this tier does not read
// (types.rs block_size / block_bytes; tensor_info.rs:37-44).
uint64_t gguf_tensor_bytes(uint32_t type, uint64_t elements);

}  // namespace oxb
