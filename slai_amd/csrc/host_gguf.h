// GGUF container parser: the host-side mirror of crates/slai/src/gguf.rs.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace slai {

// gguf.rs:240-255 `GgufMetadataValue` (+ :197-212 for arrays: only type/length/offset are kept;
// string arrays are materialised because the tokenizer-free decode path only needs their length,
// gguf.rs:292-298).
struct GgufMetaValue {
    uint32_t type = 0;       // 0..12, gguf.rs:385-416
    uint64_t u = 0;          // unsigned / bool
    int64_t i = 0;           // signed
    double f = 0.0;          // F32 / F64
    std::string s;           // String
    uint32_t arr_type = 0;   // Array: element type
    uint64_t arr_len = 0;    // Array: element count
    uint64_t arr_offset = 0; // Array: file offset of the first element
};

// gguf.rs:333-345 `GgufTensor`; data stays in the caller's byte slice (no per-element copies).
struct GgufTensorInfo {
    std::string name;
    uint64_t dims[4] = {1, 1, 1, 1};  // [nrows, ncols, nmats, ncubes] after the swap of gguf.rs:581
    uint32_t ndims = 0;
    uint32_t type = 0;                // ggml type tag, gguf.rs:75-107
    uint64_t offset = 0;              // absolute (gguf.rs:598)
    uint64_t nbytes = 0;              // 0 for types without a loader (gguf.rs:674)
};

struct Gguf {
    const uint8_t *bytes = nullptr;
    size_t len = 0;
    uint32_t version = 0, alignment = 32;
    uint64_t data_start = 0;
    std::map<std::string, GgufMetaValue> metadata;
    std::vector<GgufTensorInfo> tensors;
    std::map<std::string, size_t> tensor_index;

    // gguf.rs:504-524 `Gguf::from_bytes`.  Returns 0 or SLAI_E_PARSE with a message in `err`
    // (IncorrectMagicNumber :30, UnsupportedMetadataValueType :32, UnsupportedTensorType :34;
    // truncation, which panics in the reference :722, is reported as an error).
    int parse(const uint8_t *data, size_t n, std::string &err);
    const GgufTensorInfo *find(const std::string &name) const;
    const GgufMetaValue *meta(const std::string &key) const;
};

}  // namespace slai

// `map` is set when the handle owns a read-only mapping of the file (slai_gguf_open_file)
struct slai_gguf {
    slai::Gguf g;
    void *map = nullptr;
    size_t map_len = 0;
};
