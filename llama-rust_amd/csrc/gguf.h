// GGUF v3 container: the reader and writer the host decode and the synthetic-model
// generator use.  Same container rules as the reference's module
// (langtax/src/gguf.rs:64-68 magic, version 3, default alignment 32;
// :626-702 writer; :728-828 parser): little-endian, i64 tensor and key counts,
// strings as u64 length + bytes, tensor offsets relative to the aligned start of
// the data section, every tensor start aligned.
#pragma once
#include <cstdint>
#include <cstdio>
#include <functional>
#include <map>
#include <string>
#include <vector>

namespace nh {
namespace gguf {

enum KvType : int32_t {
    KV_U8 = 0, KV_I8 = 1, KV_U16 = 2, KV_I16 = 3, KV_U32 = 4, KV_I32 = 5, KV_F32 = 6, KV_BOOL = 7,
    KV_STRING = 8, KV_ARRAY = 9, KV_U64 = 10, KV_I64 = 11, KV_F64 = 12,
};

struct Kv {
    int32_t type = KV_U32;
    uint64_t u = 0;   // unsigned and bool payloads
    int64_t i = 0;    // signed payloads
    double f = 0.0;   // F32 / F64 payloads
    std::string s;    // STRING payload
    int32_t elem = KV_U32;  // ARRAY: element type
    std::vector<Kv> items;  // ARRAY: elements

    static Kv u32(uint32_t v) { Kv k; k.type = KV_U32; k.u = v; return k; }
    static Kv f32(float v) { Kv k; k.type = KV_F32; k.f = v; return k; }
    static Kv str(const std::string &v) { Kv k; k.type = KV_STRING; k.s = v; return k; }
    static Kv boolean(bool v) { Kv k; k.type = KV_BOOL; k.u = v; return k; }
};

struct TensorInfo {
    std::string name;
    uint32_t type = 0;            // ggml type id
    std::vector<uint64_t> shape;  // ggml order: shape[0] is the contiguous (column) dimension
    size_t start = 0, end = 0;    // byte range in the file
};

// Bytes and elements of one block of a ggml type this build handles; false for the others.
bool type_layout(uint32_t ggml_type, size_t *block_bytes, size_t *block_elems);

struct File {
    const uint8_t *data = nullptr;
    size_t size = 0;
    size_t alignment = 32;
    std::map<std::string, Kv> kv;
    std::vector<TensorInfo> tensors;
    std::map<std::string, size_t> by_name;

    const TensorInfo *tensor(const std::string &name) const;
    bool kv_u32(const std::string &key, uint32_t *out) const;  // U32 only, like the reference's kv_u32
    bool kv_f32(const std::string &key, float *out) const;
    bool kv_str(const std::string &key, std::string *out) const;
};

// Parses `bytes` (which must outlive `out`).  Error texts follow the reference's GgufError
// variants: "bad magic", "unsupported version N", "truncated", "bad shape", "unsupported ggml type N".
bool parse(const uint8_t *bytes, size_t size, File *out, std::string *err);

struct TensorWrite {
    std::string name;
    uint32_t type = 0;
    std::vector<uint64_t> shape;
    size_t nbytes = 0;
    const uint8_t *data = nullptr;                    // either the bytes themselves ...
    std::function<void(uint8_t *dst)> fill;           // ... or a producer called with an nbytes buffer
};

// Streams a GGUF v3 file: header, keys in the given order, tensor infos, padding, tensor data.
bool write(FILE *f, const std::vector<std::pair<std::string, Kv>> &kv, const std::vector<TensorWrite> &tensors,
           std::string *err);

}  // namespace gguf
}  // namespace nh
