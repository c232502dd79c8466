// GGUF v3 reader and writer (see gguf.h).
#include "gguf.h"

#include <cstring>

namespace nh {
namespace gguf {

bool type_layout(uint32_t t, size_t *block_bytes, size_t *block_elems) {
    size_t b = 0, k = 0;
    switch (t) {  // langtax/src/quant.rs:87-163 block constants
    case 0: b = 4; k = 1; break;       // F32
    case 1: b = 2; k = 1; break;       // F16
    case 2: b = 18; k = 32; break;     // Q4_0
    case 6: b = 22; k = 32; break;     // Q5_0
    case 7: b = 24; k = 32; break;     // Q5_1
    case 8: b = 34; k = 32; break;     // Q8_0
    case 12: b = 144; k = 256; break;  // Q4_K
    case 14: b = 210; k = 256; break;  // Q6_K
    default: return false;
    }
    if (block_bytes) *block_bytes = b;
    if (block_elems) *block_elems = k;
    return true;
}

const TensorInfo *File::tensor(const std::string &name) const {
    auto it = by_name.find(name);
    return it == by_name.end() ? nullptr : &tensors[it->second];
}
bool File::kv_u32(const std::string &key, uint32_t *out) const {
    auto it = kv.find(key);
    if (it == kv.end() || it->second.type != KV_U32) return false;
    *out = (uint32_t)it->second.u;
    return true;
}
bool File::kv_f32(const std::string &key, float *out) const {
    auto it = kv.find(key);
    if (it == kv.end() || it->second.type != KV_F32) return false;
    *out = (float)it->second.f;
    return true;
}
bool File::kv_str(const std::string &key, std::string *out) const {
    auto it = kv.find(key);
    if (it == kv.end() || it->second.type != KV_STRING) return false;
    *out = it->second.s;
    return true;
}

namespace {

struct Reader {
    const uint8_t *p;
    size_t n, pos = 0;
    bool ok = true;
    const uint8_t *take(size_t k) {
        if (!ok || k > n - pos) {
            ok = false;
            return nullptr;
        }
        const uint8_t *r = p + pos;
        pos += k;
        return r;
    }
    template <typename T> T get() {
        T v{};
        if (const uint8_t *r = take(sizeof(T))) std::memcpy(&v, r, sizeof(T));
        return v;
    }
    std::string str() {
        const uint64_t len = get<uint64_t>();
        if (!ok || len > n - pos) {
            ok = false;
            return {};
        }
        const uint8_t *r = take((size_t)len);
        return r ? std::string(reinterpret_cast<const char *>(r), (size_t)len) : std::string();
    }
};

bool read_value(Reader &r, int32_t ty, Kv *out, int depth, std::string *err) {
    out->type = ty;
    switch (ty) {
    case KV_U8: out->u = r.get<uint8_t>(); break;
    case KV_I8: out->i = r.get<int8_t>(); break;
    case KV_U16: out->u = r.get<uint16_t>(); break;
    case KV_I16: out->i = r.get<int16_t>(); break;
    case KV_U32: out->u = r.get<uint32_t>(); break;
    case KV_I32: out->i = r.get<int32_t>(); break;
    case KV_F32: out->f = r.get<float>(); break;
    case KV_BOOL: out->u = r.get<uint8_t>() != 0; break;
    case KV_STRING: out->s = r.str(); break;
    case KV_U64: out->u = r.get<uint64_t>(); break;
    case KV_I64: out->i = r.get<int64_t>(); break;
    case KV_F64: out->f = r.get<double>(); break;
    case KV_ARRAY: {
        out->elem = r.get<int32_t>();
        const uint64_t n = r.get<uint64_t>();
        // every element takes at least one byte of what is left; the vector grows with the elements
        // actually read, so a huge count in a short file cannot reserve memory up front
        if (!r.ok || depth > 4 || n > r.n - r.pos) {
            *err = "truncated";
            return false;
        }
        out->items.clear();
        out->items.reserve((size_t)(n < 4096 ? n : 4096));
        for (uint64_t i = 0; i < n; i++) {
            Kv it;
            if (!read_value(r, out->elem, &it, depth + 1, err)) return false;
            out->items.push_back(std::move(it));
        }
        break;
    }
    default: *err = "unsupported metadata type " + std::to_string(ty); return false;
    }
    if (!r.ok) {
        *err = "truncated";
        return false;
    }
    return true;
}

size_t align_up(size_t n, size_t a) { return (n + a - 1) / a * a; }

}  // namespace

bool parse(const uint8_t *bytes, size_t size, File *out, std::string *err) {
    Reader r{bytes, size};
    const uint8_t *magic = r.take(4);
    if (!magic) return *err = "truncated", false;
    if (std::memcmp(magic, "GGUF", 4) != 0) return *err = "bad magic", false;
    const uint32_t version = r.get<uint32_t>();
    if (!r.ok) return *err = "truncated", false;
    if (version != 3) return *err = "unsupported version " + std::to_string(version), false;
    const int64_t n_tensors = r.get<int64_t>(), n_kv = r.get<int64_t>();
    if (!r.ok || n_tensors < 0 || n_kv < 0) return *err = "truncated", false;

    out->data = bytes;
    out->size = size;
    out->kv.clear();
    out->tensors.clear();
    out->by_name.clear();
    for (int64_t i = 0; i < n_kv; i++) {
        std::string key = r.str();
        const int32_t ty = r.get<int32_t>();
        if (!r.ok) return *err = "truncated", false;
        Kv v;
        if (!read_value(r, ty, &v, 0, err)) return false;
        out->kv[key] = std::move(v);  // last write wins
    }
    out->alignment = 32;
    uint32_t al = 0;
    if (out->kv_u32("general.alignment", &al) && al > 0) out->alignment = al;

    struct Raw {
        std::string name;
        std::vector<uint64_t> shape;
        int32_t type;
        uint64_t offset;
    };
    std::vector<Raw> raw;
    for (int64_t i = 0; i < n_tensors; i++) {
        Raw t;
        t.name = r.str();
        const uint32_t n_dims = r.get<uint32_t>();
        if (!r.ok) return *err = "truncated", false;
        if (n_dims == 0 || n_dims > 4) return *err = "bad shape", false;
        for (uint32_t d = 0; d < n_dims; d++) {
            const int64_t v = r.get<int64_t>();
            if (!r.ok) return *err = "truncated", false;
            if (v <= 0) return *err = "bad shape", false;
            t.shape.push_back((uint64_t)v);
        }
        t.type = r.get<int32_t>();
        t.offset = r.get<uint64_t>();
        if (!r.ok) return *err = "truncated", false;
        raw.push_back(std::move(t));
    }
    const size_t data_start = align_up(r.pos, out->alignment);
    for (auto &t : raw) {
        size_t block = 0, k = 0;
        if (t.type < 0 || !type_layout((uint32_t)t.type, &block, &k))
            return *err = "unsupported ggml type " + std::to_string(t.type), false;
        uint64_t n_el = 1;
        for (uint64_t d : t.shape) {
            if (d != 0 && n_el > UINT64_MAX / d) return *err = "bad shape", false;
            n_el *= d;
        }
        // rows are whole blocks (the row dequantizers and the device kernels walk a row block by block)
        if (t.shape[0] % k != 0) return *err = "bad shape", false;
        const uint64_t n_blocks = n_el / k;
        if (n_blocks > UINT64_MAX / block) return *err = "bad shape", false;
        const uint64_t nbytes = n_blocks * block;
        if (t.offset > size || data_start > size - (size_t)t.offset) return *err = "truncated", false;
        const size_t start = data_start + (size_t)t.offset;
        if (nbytes > size - start) return *err = "truncated", false;
        TensorInfo info;
        info.name = t.name;
        info.type = (uint32_t)t.type;
        info.shape = t.shape;
        info.start = start;
        info.end = start + (size_t)nbytes;
        out->by_name[info.name] = out->tensors.size();
        out->tensors.push_back(std::move(info));
    }
    return true;
}

namespace {

struct Buf {
    std::vector<uint8_t> b;
    template <typename T> void put(T v) {
        const size_t at = b.size();
        b.resize(at + sizeof(T));
        std::memcpy(b.data() + at, &v, sizeof(T));
    }
    void str(const std::string &s) {
        put<uint64_t>(s.size());
        b.insert(b.end(), s.begin(), s.end());
    }
};

bool put_value(Buf &o, const Kv &v, std::string *err) {
    switch (v.type) {
    case KV_U8: o.put<uint8_t>((uint8_t)v.u); break;
    case KV_I8: o.put<int8_t>((int8_t)v.i); break;
    case KV_U16: o.put<uint16_t>((uint16_t)v.u); break;
    case KV_I16: o.put<int16_t>((int16_t)v.i); break;
    case KV_U32: o.put<uint32_t>((uint32_t)v.u); break;
    case KV_I32: o.put<int32_t>((int32_t)v.i); break;
    case KV_F32: o.put<float>((float)v.f); break;
    case KV_BOOL: o.put<uint8_t>(v.u ? 1 : 0); break;
    case KV_STRING: o.str(v.s); break;
    case KV_U64: o.put<uint64_t>(v.u); break;
    case KV_I64: o.put<int64_t>(v.i); break;
    case KV_F64: o.put<double>(v.f); break;
    case KV_ARRAY:
        o.put<int32_t>(v.elem);
        o.put<uint64_t>(v.items.size());
        for (const Kv &it : v.items) {
            if (it.type != v.elem) return *err = "array element of another type", false;
            if (!put_value(o, it, err)) return false;
        }
        break;
    default: *err = "unsupported metadata type " + std::to_string(v.type); return false;
    }
    return true;
}

}  // namespace

bool write(FILE *f, const std::vector<std::pair<std::string, Kv>> &kv, const std::vector<TensorWrite> &tensors,
           std::string *err) {
    const size_t alignment = 32;
    std::vector<uint64_t> offsets;
    size_t off = 0;
    for (const TensorWrite &t : tensors) {
        size_t block = 0, k = 0;
        if (!type_layout(t.type, &block, &k)) return *err = "unsupported ggml type " + std::to_string(t.type), false;
        uint64_t n_el = 1;
        for (uint64_t d : t.shape) n_el *= d;
        if (t.shape.empty() || t.shape.size() > 4 || n_el % k != 0 || n_el / k * block != t.nbytes)
            return *err = "bad shape for " + t.name, false;
        off = align_up(off, alignment);
        offsets.push_back(off);
        off += t.nbytes;
    }
    Buf h;
    h.b.insert(h.b.end(), {'G', 'G', 'U', 'F'});
    h.put<uint32_t>(3);
    h.put<int64_t>((int64_t)tensors.size());
    h.put<int64_t>((int64_t)kv.size());
    for (const auto &e : kv) {
        h.str(e.first);
        h.put<int32_t>(e.second.type);
        if (!put_value(h, e.second, err)) return false;
    }
    for (size_t i = 0; i < tensors.size(); i++) {
        h.str(tensors[i].name);
        h.put<uint32_t>((uint32_t)tensors[i].shape.size());
        for (uint64_t d : tensors[i].shape) h.put<int64_t>((int64_t)d);
        h.put<int32_t>((int32_t)tensors[i].type);
        h.put<uint64_t>(offsets[i]);
    }
    h.b.resize(align_up(h.b.size(), alignment), 0);
    if (std::fwrite(h.b.data(), 1, h.b.size(), f) != h.b.size()) return *err = "write failed", false;
    size_t cursor = 0;
    std::vector<uint8_t> scratch;
    const uint8_t zeros[32] = {0};
    for (size_t i = 0; i < tensors.size(); i++) {
        const size_t pad = (size_t)offsets[i] - cursor;
        if (pad && std::fwrite(zeros, 1, pad, f) != pad) return *err = "write failed", false;
        const uint8_t *src = tensors[i].data;
        if (!src) {
            if (!tensors[i].fill) return *err = "tensor without data: " + tensors[i].name, false;
            scratch.resize(tensors[i].nbytes);
            tensors[i].fill(scratch.data());
            src = scratch.data();
        }
        if (std::fwrite(src, 1, tensors[i].nbytes, f) != tensors[i].nbytes) return *err = "write failed", false;
        cursor = (size_t)offsets[i] + tensors[i].nbytes;
    }
    return true;
}

}  // namespace gguf
}  // namespace nh
