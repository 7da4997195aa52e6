// GGUF container reader (host only): header, metadata and tensor directory of a
// file mapped read-only, with tensor types kept as raw ids so that types outside
// the common table (MXFP4 = 39, IQ2_XXS = 16) survive parsing.
//
// Behaviour follows the reference's tolerant header reader
// (reference: src/gguf_ext.rs:33-59 limits, :293-398 value reader, :400-480
// read_header, :483-512 type_size_bytes):
//   - versions 1..3; lengths are u32 in version 1 and u64 after;
//   - tensor and metadata counts above 2^24 are refused before anything is stored;
//   - a string may claim at most 2^24 bytes and never more than the bytes left;
//     trailing NUL bytes are dropped and the bytes are otherwise kept as they are;
//   - an array may claim at most 2^24 elements; arrays nest to depth 64;
//   - a tensor has at most 8 dimensions, stored fastest first and reversed here
//     into row-major order;
//   - general.alignment (any integer type up to 32 bits, not negative) must be a
//     power of two, default 32; tensor data starts at the next multiple of it.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace jq {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;  // "GGUF" read as a little-endian word
constexpr uint64_t GGUF_DEFAULT_ALIGNMENT = 32;
constexpr uint64_t GGUF_MAX_COUNT = 1ull << 24;
constexpr uint64_t GGUF_MAX_STRING = 1ull << 24;
constexpr uint64_t GGUF_MAX_ARRAY = 1ull << 24;
constexpr int GGUF_MAX_DEPTH = 64;

// Bytes of `elems` elements of a raw GGUF type id; false for an unknown id or a
// count that is not a whole number of blocks (reference: src/gguf_ext.rs:483-512).
inline bool gguf_type_size_bytes(uint32_t dtype, uint64_t elems, uint64_t *out) {
    uint64_t blck, bytes;
    switch (dtype) {
    case 0: blck = 1; bytes = 4; break;      // F32
    case 1: blck = 1; bytes = 2; break;      // F16
    case 30: blck = 1; bytes = 2; break;     // BF16
    case 2: blck = 32; bytes = 18; break;    // Q4_0
    case 3: blck = 32; bytes = 20; break;    // Q4_1
    case 6: blck = 32; bytes = 22; break;    // Q5_0
    case 7: blck = 32; bytes = 24; break;    // Q5_1
    case 8: blck = 32; bytes = 34; break;    // Q8_0
    case 9: blck = 32; bytes = 36; break;    // Q8_1
    case 10: blck = 256; bytes = 84; break;  // Q2_K
    case 11: blck = 256; bytes = 110; break; // Q3_K
    case 12: blck = 256; bytes = 144; break; // Q4_K
    case 13: blck = 256; bytes = 176; break; // Q5_K
    case 14: blck = 256; bytes = 210; break; // Q6_K
    case 15: blck = 256; bytes = 292; break; // Q8_K
    case 26: blck = 1; bytes = 4; break;     // I32
    case 16: blck = 256; bytes = 66; break;  // IQ2_XXS
    case 39: blck = 32; bytes = 17; break;   // MXFP4
    default: return false;
    }
    if (elems % blck != 0) return false;
    *out = elems / blck * bytes;
    return true;
}

// One metadata value.  Scalars keep their GGUF value type (0..12); arrays keep
// their elements.
struct GgufValue {
    uint32_t type = 0;
    uint64_t u = 0;    // unsigned integers and bool
    int64_t i = 0;     // signed integers
    double f = 0.0;    // F32 / F64
    std::string s;     // string
    std::vector<GgufValue> items;  // array
};

struct GgufTensor {
    std::string name;
    uint32_t dtype = 0;
    std::vector<uint64_t> dims;  // row-major (slowest first)
    uint64_t offset = 0;         // from tensor_data_offset
    uint64_t elem_count() const {
        uint64_t e = 1;
        for (uint64_t d : dims) e *= d;
        return e;
    }
};

struct Gguf {
    uint32_t version = 0;
    std::map<std::string, GgufValue> metadata;
    std::vector<GgufTensor> tensors;            // in file order
    std::map<std::string, size_t> by_name;      // a repeated name keeps the last entry, as a map insert would
    uint64_t tensor_data_offset = 0;
    // the bytes: either a private read-only mapping of a file or a caller's buffer (header-only parse)
    const uint8_t *base = nullptr;
    uint64_t size = 0;
    bool mapped = false;
    std::vector<uint8_t> owned;  // the copy behind `base` when the header came from a caller's buffer

    ~Gguf() {
        if (mapped && base) munmap((void *)base, size);
    }

    const GgufValue *find(const std::string &key) const {
        auto it = metadata.find(key);
        return it == metadata.end() ? nullptr : &it->second;
    }
    // Integer of any width up to 32 bits that is not negative.
    bool meta_u32(const std::string &key, uint32_t *out) const {
        const GgufValue *v = find(key);
        if (!v) return false;
        switch (v->type) {
        case 0: case 2: case 4: *out = (uint32_t)v->u; return true;
        case 1: case 3: case 5:
            if (v->i < 0) return false;
            *out = (uint32_t)v->i;
            return true;
        default: return false;
        }
    }
    bool meta_f32(const std::string &key, float *out) const {
        const GgufValue *v = find(key);
        if (!v || v->type != 6) return false;
        *out = (float)v->f;
        return true;
    }
    bool meta_bool(const std::string &key, bool *out) const {
        const GgufValue *v = find(key);
        if (!v || v->type != 7) return false;
        *out = v->u != 0;
        return true;
    }
    const std::string *meta_str(const std::string &key) const {
        const GgufValue *v = find(key);
        return v && v->type == 8 ? &v->s : nullptr;
    }
    const GgufTensor *tensor(const std::string &name) const {
        auto it = by_name.find(name);
        return it == by_name.end() ? nullptr : &tensors[it->second];
    }
    // The tensor's bytes inside the mapping, or an explanation.  The range check is the
    // reference's borrow check (reference: src/mmap_tensor.rs:105-123): sizes that overflow or
    // run past the end of the file are refused.
    bool tensor_bytes(const GgufTensor &t, const uint8_t **data, uint64_t *nbytes, std::string *err) const {
        uint64_t sz;
        if (!gguf_type_size_bytes(t.dtype, t.elem_count(), &sz)) {
            *err = "tensor `" + t.name + "`: type id " + std::to_string(t.dtype) + " with " +
                   std::to_string(t.elem_count()) + " elements has no known size";
            return false;
        }
        uint64_t begin = tensor_data_offset + t.offset;
        if (begin < tensor_data_offset || begin + sz < begin || begin + sz > size) {
            *err = "tensor `" + t.name + "`: bytes [" + std::to_string(begin) + ", +" + std::to_string(sz) +
                   ") run past the " + std::to_string(size) + " bytes of the file";
            return false;
        }
        *data = base + begin;
        *nbytes = sz;
        return true;
    }
};

namespace gguf_detail {

struct Reader {
    const uint8_t *p;
    uint64_t size, pos = 0;
    uint32_t version = 0;
    std::string err;

    bool fail(const std::string &msg) {
        if (err.empty()) err = "GGUF header: " + msg;
        return false;
    }
    bool take(void *dst, uint64_t n) {
        if (n > size - pos) return fail("failed to fill whole buffer");
        memcpy(dst, p + pos, n);
        pos += n;
        return true;
    }
    bool u32(uint32_t *v) { return take(v, 4); }
    bool u64(uint64_t *v) { return take(v, 8); }
    bool len(uint64_t *v) {
        if (version == 1) {
            uint32_t w;
            if (!u32(&w)) return false;
            *v = w;
            return true;
        }
        return u64(v);
    }
    bool string(std::string *out) {
        uint64_t n;
        if (!len(&n)) return false;
        if (n > GGUF_MAX_STRING)
            return fail("string of " + std::to_string(n) + " bytes exceeds max " + std::to_string(GGUF_MAX_STRING));
        if (n > size - pos)
            return fail("string of " + std::to_string(n) + " bytes exceeds the " + std::to_string(size - pos) +
                        " bytes remaining in the stream");
        out->assign((const char *)p + pos, n);
        pos += n;
        while (!out->empty() && out->back() == '\0') out->pop_back();
        return true;
    }
    bool value(uint32_t ty, int depth, GgufValue *v) {
        if (depth > GGUF_MAX_DEPTH) return fail("value nesting depth exceeds max " + std::to_string(GGUF_MAX_DEPTH));
        v->type = ty;
        switch (ty) {
        case 0: { uint8_t x; if (!take(&x, 1)) return false; v->u = x; return true; }
        case 1: { int8_t x; if (!take(&x, 1)) return false; v->i = x; return true; }
        case 2: { uint16_t x; if (!take(&x, 2)) return false; v->u = x; return true; }
        case 3: { int16_t x; if (!take(&x, 2)) return false; v->i = x; return true; }
        case 4: { uint32_t x; if (!take(&x, 4)) return false; v->u = x; return true; }
        case 5: { int32_t x; if (!take(&x, 4)) return false; v->i = x; return true; }
        case 6: { float x; if (!take(&x, 4)) return false; v->f = x; return true; }
        case 7: { uint8_t x; if (!take(&x, 1)) return false; v->u = x != 0; return true; }
        case 8: return string(&v->s);
        case 9: {
            uint32_t elem_ty;
            uint64_t n;
            if (!u32(&elem_ty) || !len(&n)) return false;
            if (n > GGUF_MAX_ARRAY)
                return fail("array of " + std::to_string(n) + " elements exceeds max " + std::to_string(GGUF_MAX_ARRAY));
            // nothing is reserved for the claimed count: the vector grows as elements arrive
            for (uint64_t i = 0; i < n; i++) {
                v->items.emplace_back();
                if (!value(elem_ty, depth + 1, &v->items.back())) return false;
            }
            return true;
        }
        case 10: { uint64_t x; if (!take(&x, 8)) return false; v->u = x; return true; }
        case 11: { int64_t x; if (!take(&x, 8)) return false; v->i = x; return true; }
        case 12: { double x; if (!take(&x, 8)) return false; v->f = x; return true; }
        default: return fail("unknown metadata value type " + std::to_string(ty));
        }
    }
};

}  // namespace gguf_detail

// Parses the header found in `bytes`; on failure returns null and sets *err.
inline std::unique_ptr<Gguf> gguf_parse(const uint8_t *bytes, uint64_t size, std::string *err) {
    gguf_detail::Reader rd{bytes, size};
    auto g = std::make_unique<Gguf>();
    auto bail = [&]() -> std::unique_ptr<Gguf> {
        *err = rd.err;
        return nullptr;
    };
    uint32_t magic;
    if (!rd.u32(&magic)) return bail();
    if (magic != GGUF_MAGIC) {
        rd.fail("not a GGUF file (bad magic)");
        return bail();
    }
    uint32_t version;
    if (!rd.u32(&version)) return bail();
    if (version < 1 || version > 3) {
        rd.fail("unsupported GGUF version " + std::to_string(version));
        return bail();
    }
    rd.version = g->version = version;
    uint64_t tensor_count, kv_count;
    if (!rd.len(&tensor_count) || !rd.len(&kv_count)) return bail();
    if (tensor_count > GGUF_MAX_COUNT || kv_count > GGUF_MAX_COUNT) {
        rd.fail("implausible tensor/metadata count");
        return bail();
    }
    for (uint64_t i = 0; i < kv_count; i++) {
        std::string key;
        uint32_t ty;
        GgufValue v;
        if (!rd.string(&key) || !rd.u32(&ty) || !rd.value(ty, 0, &v)) return bail();
        g->metadata[key] = std::move(v);
    }
    for (uint64_t i = 0; i < tensor_count; i++) {
        GgufTensor t;
        uint32_t n_dims;
        if (!rd.string(&t.name) || !rd.u32(&n_dims)) return bail();
        if (n_dims > 8) {
            rd.fail("tensor `" + t.name + "` claims " + std::to_string(n_dims) + " dimensions");
            return bail();
        }
        t.dims.resize(n_dims);
        for (uint32_t d = 0; d < n_dims; d++)
            if (!rd.len(&t.dims[n_dims - 1 - d])) return bail();
        if (!rd.u32(&t.dtype) || !rd.u64(&t.offset)) return bail();
        g->by_name[t.name] = g->tensors.size();
        g->tensors.push_back(std::move(t));
    }
    uint64_t alignment = GGUF_DEFAULT_ALIGNMENT;
    if (const GgufValue *a = g->find("general.alignment")) {
        switch (a->type) {
        case 0: case 2: case 4: alignment = a->u; break;
        case 1: case 3: case 5:
            if (a->i >= 0) alignment = (uint64_t)a->i;
            break;
        default: break;
        }
    }
    if (alignment == 0 || (alignment & (alignment - 1)) != 0) {
        rd.fail("invalid general.alignment " + std::to_string(alignment));
        return bail();
    }
    g->tensor_data_offset = (rd.pos + alignment - 1) / alignment * alignment;
    g->base = bytes;
    g->size = size;
    return g;
}

// Maps the file read-only and parses its header.  The mapping lives as long as the object.
inline std::unique_ptr<Gguf> gguf_open(const char *path, std::string *err) {
    int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) {
        *err = std::string("cannot open `") + path + "`: " + strerror(errno);
        return nullptr;
    }
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        *err = std::string("cannot size `") + path + "`";
        close(fd);
        return nullptr;
    }
    void *map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED) {
        *err = std::string("cannot map `") + path + "`: " + strerror(errno);
        return nullptr;
    }
    auto g = gguf_parse((const uint8_t *)map, (uint64_t)st.st_size, err);
    if (!g) {
        munmap(map, (size_t)st.st_size);
        return nullptr;
    }
    g->mapped = true;
    return g;
}

}  // namespace jq
