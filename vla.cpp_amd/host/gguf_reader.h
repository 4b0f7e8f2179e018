// GGUF file reader with the interface the reference's model loaders use
// (struct gguf_reader, src/gguf_reader.h:33-216): typed metadata getters that return a
// zero value and print to stderr instead of aborting, tensor metadata by name, raw and
// fp32 reads, conversion to a resident type with the Gemma "+1" norm option, and row
// fetches from an embedding matrix left on disk.  The reference wraps ggml's gguf library;
// this is a self-contained parser of the published container format (versions 2 and 3):
//
//   "GGUF" | u32 version | u64 n_tensors | u64 n_kv
//   n_kv x    { string key | u32 value type | value }
//   n_tensors x { string name | u32 n_dims | u64 dims[n_dims] (ne0 innermost) | u32 ggml type | u64 offset }
//   padding to general.alignment (default 32) | tensor data (offsets relative to here)
//   string = u64 length + bytes; array value = u32 element type | u64 count | elements.
//
// Every length read from the file is checked against the file size before it is used.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace vla {

// ggml tensor types by their on-disk numbers (the subset with a fixed block size).
enum gguf_tensor_type : uint32_t {
    GGUF_T_F32 = 0, GGUF_T_F16 = 1, GGUF_T_Q4_0 = 2, GGUF_T_Q4_1 = 3, GGUF_T_Q5_0 = 6, GGUF_T_Q5_1 = 7, GGUF_T_Q8_0 = 8,
    GGUF_T_Q8_1 = 9, GGUF_T_Q2_K = 10, GGUF_T_Q3_K = 11, GGUF_T_Q4_K = 12, GGUF_T_Q5_K = 13, GGUF_T_Q6_K = 14,
    GGUF_T_Q8_K = 15, GGUF_T_I8 = 24, GGUF_T_I16 = 25, GGUF_T_I32 = 26, GGUF_T_I64 = 27, GGUF_T_F64 = 28, GGUF_T_BF16 = 30,
};

// Metadata value types by their on-disk numbers.
enum gguf_kv_type : uint32_t {
    GGUF_KV_U8 = 0, GGUF_KV_I8 = 1, GGUF_KV_U16 = 2, GGUF_KV_I16 = 3, GGUF_KV_U32 = 4, GGUF_KV_I32 = 5, GGUF_KV_F32 = 6,
    GGUF_KV_BOOL = 7, GGUF_KV_STRING = 8, GGUF_KV_ARRAY = 9, GGUF_KV_U64 = 10, GGUF_KV_I64 = 11, GGUF_KV_F64 = 12,
};

struct gguf_tensor_meta {
    std::string name;
    uint32_t type = 0;
    int n_dims = 0;
    int64_t ne[4] = {1, 1, 1, 1};  // ne[0] is the contiguous dimension
    uint64_t offset = 0;           // relative to the data section
    uint64_t nbytes = 0;           // 0 when the type's block size is unknown
    int64_t nelements() const { return ne[0] * ne[1] * ne[2] * ne[3]; }
};

struct gguf_kv {
    uint32_t type = 0;
    uint64_t bits = 0;  // scalars, as stored (little-endian, zero-extended)
    std::string s;      // GGUF_KV_STRING
    uint32_t elem_type = 0;
    uint64_t count = 0;
    std::vector<uint8_t> raw;         // numeric arrays, packed as in the file
    std::vector<std::string> strs;    // string arrays
};

inline bool gguf_type_block(uint32_t type, int* block_elems, int* block_bytes) {
    switch (type) {
        case GGUF_T_F32: *block_elems = 1; *block_bytes = 4; return true;
        case GGUF_T_F16: case GGUF_T_BF16: case GGUF_T_I16: *block_elems = 1; *block_bytes = 2; return true;
        case GGUF_T_I8: *block_elems = 1; *block_bytes = 1; return true;
        case GGUF_T_I32: *block_elems = 1; *block_bytes = 4; return true;
        case GGUF_T_I64: case GGUF_T_F64: *block_elems = 1; *block_bytes = 8; return true;
        case GGUF_T_Q4_0: *block_elems = 32; *block_bytes = 18; return true;
        case GGUF_T_Q4_1: *block_elems = 32; *block_bytes = 20; return true;
        case GGUF_T_Q5_0: *block_elems = 32; *block_bytes = 22; return true;
        case GGUF_T_Q5_1: *block_elems = 32; *block_bytes = 24; return true;
        case GGUF_T_Q8_0: *block_elems = 32; *block_bytes = 34; return true;
        case GGUF_T_Q8_1: *block_elems = 32; *block_bytes = 36; return true;
        case GGUF_T_Q2_K: *block_elems = 256; *block_bytes = 84; return true;
        case GGUF_T_Q3_K: *block_elems = 256; *block_bytes = 110; return true;
        case GGUF_T_Q4_K: *block_elems = 256; *block_bytes = 144; return true;
        case GGUF_T_Q5_K: *block_elems = 256; *block_bytes = 176; return true;
        case GGUF_T_Q6_K: *block_elems = 256; *block_bytes = 210; return true;
        case GGUF_T_Q8_K: *block_elems = 256; *block_bytes = 292; return true;
        default: return false;
    }
}

inline float gguf_half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const int exp = (h >> 10) & 0x1f;
    const uint32_t man = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else {  // subnormal half: value = man * 2^-24
            const float v = std::ldexp((float)man, -24);
            std::memcpy(&u, &v, 4);
            u |= sign;
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((uint32_t)(exp - 15 + 127) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// fp32 -> bf16, round to nearest even, NaN kept quiet (what ggml_fp32_to_bf16_row does in
// the reference's read_convert, src/gguf_reader.h:175-178).
inline uint16_t gguf_float_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 64);
    return (uint16_t)((u + (0x7fffu + ((u >> 16) & 1))) >> 16);
}

struct gguf_reader {
    const char* arch = "vla";
    FILE* fp = nullptr;
    uint32_t version = 0;
    uint64_t file_size = 0;
    size_t data_off = 0;
    uint32_t alignment = 32;
    std::map<std::string, gguf_kv> kv;
    std::vector<gguf_tensor_meta> tensors;
    std::map<std::string, size_t> index;

    explicit gguf_reader(const char* arch_ = "vla") : arch(arch_) {}
    ~gguf_reader() {
        if (fp) std::fclose(fp);
    }
    gguf_reader(const gguf_reader&) = delete;
    gguf_reader& operator=(const gguf_reader&) = delete;

    bool open(const std::string& path) {
        fp = std::fopen(path.c_str(), "rb");
        if (!fp) {
            std::fprintf(stderr, "vla(%s): fopen failed for %s\n", arch, path.c_str());
            return false;
        }
        if (fseeko(fp, 0, SEEK_END) != 0) return fail(path, "seek failed");
        file_size = (uint64_t)ftello(fp);
        if (fseeko(fp, 0, SEEK_SET) != 0) return fail(path, "seek failed");
        char magic[4];
        uint64_t n_tensors = 0, n_kv = 0;
        if (!rd(magic, 4) || std::memcmp(magic, "GGUF", 4) != 0) return fail(path, "not a GGUF file");
        if (!rd(&version, 4) || (version != 2 && version != 3)) return fail(path, "unsupported GGUF version");
        if (!rd(&n_tensors, 8) || !rd(&n_kv, 8)) return fail(path, "truncated header");
        // each record takes at least 12 bytes (kv) / 24 bytes (tensor info) of the file
        if (n_kv > file_size / 12 || n_tensors > file_size / 24) return fail(path, "implausible record counts");
        for (uint64_t i = 0; i < n_kv; ++i) {
            std::string key;
            gguf_kv v;
            if (!rd_str(key) || !rd(&v.type, 4) || !rd_value(v)) return fail(path, "truncated or malformed metadata");
            kv[key] = std::move(v);
        }
        auto al = kv.find("general.alignment");
        if (al != kv.end() && al->second.type == GGUF_KV_U32) alignment = (uint32_t)al->second.bits;
        if (alignment == 0 || (alignment & (alignment - 1)) != 0) return fail(path, "general.alignment is not a power of two");
        tensors.resize((size_t)n_tensors);
        for (gguf_tensor_meta& t : tensors) {
            uint32_t nd = 0;
            if (!rd_str(t.name) || !rd(&nd, 4) || nd < 1 || nd > 4) return fail(path, "malformed tensor record");
            t.n_dims = (int)nd;
            uint64_t ne_total = 1;
            for (uint32_t d = 0; d < nd; ++d) {
                uint64_t e = 0;
                if (!rd(&e, 8) || e == 0 || e > (uint64_t)INT64_MAX / ne_total) return fail(path, "malformed tensor shape");
                t.ne[d] = (int64_t)e;
                ne_total *= e;
            }
            if (!rd(&t.type, 4) || !rd(&t.offset, 8)) return fail(path, "truncated tensor record");
            int be = 0, bb = 0;
            if (gguf_type_block(t.type, &be, &bb)) {
                if (t.ne[0] % be != 0) return fail(path, "row length is not a multiple of the type's block");
                t.nbytes = ne_total / (uint64_t)be * (uint64_t)bb;
            }
            if (index.count(t.name)) return fail(path, "duplicate tensor name");
            index[t.name] = (size_t)(&t - tensors.data());
        }
        const uint64_t pos = (uint64_t)ftello(fp);
        data_off = (size_t)((pos + alignment - 1) / alignment * alignment);
        for (const gguf_tensor_meta& t : tensors) {
            if (t.offset % alignment != 0 || t.offset > file_size || data_off + t.offset > file_size ||
                t.nbytes > file_size - data_off - t.offset)
                return fail(path, ("tensor " + t.name + " lies outside the file").c_str());
        }
        return true;
    }

    bool has(const char* k) const { return kv.count(k) != 0; }

    // A key of another type prints a message and reads as absent: the caller gets the
    // zero value instead of an abort (src/gguf_reader.h:74-87).
    const gguf_kv* typed_key(const char* k, uint32_t want) const {
        auto it = kv.find(k);
        if (it == kv.end()) return nullptr;
        if (it->second.type != want) {
            std::fprintf(stderr, "vla(%s): key %s has unexpected type %d\n", arch, k, (int)it->second.type);
            return nullptr;
        }
        return &it->second;
    }
    uint32_t u32(const char* k) const {
        const gguf_kv* v = typed_key(k, GGUF_KV_U32);
        return v ? (uint32_t)v->bits : 0u;
    }
    float f32(const char* k) const {
        const gguf_kv* v = typed_key(k, GGUF_KV_F32);
        if (!v) return 0.f;
        const uint32_t u = (uint32_t)v->bits;
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
    double f64(const char* k) const {
        const gguf_kv* v = typed_key(k, GGUF_KV_F64);
        if (!v) return 0.0;
        double d;
        std::memcpy(&d, &v->bits, 8);
        return d;
    }
    std::string str(const char* k) const {
        const gguf_kv* v = typed_key(k, GGUF_KV_STRING);
        return v ? v->s : std::string();
    }
    const gguf_tensor_meta* meta(const char* name) const {
        auto it = index.find(name);
        return it == index.end() ? nullptr : &tensors[it->second];
    }

    // cap must equal the tensor's size in the file (src/gguf_reader.h:116-137).
    bool read_raw(const char* name, void* buf, size_t cap) {
        const gguf_tensor_meta* t = meta(name);
        if (!t) {
            std::fprintf(stderr, "vla(%s): missing tensor %s\n", arch, name);
            return false;
        }
        if (t->nbytes == 0 || t->nbytes != cap) {
            std::fprintf(stderr, "vla(%s): tensor %s is %zu bytes, caller expects %zu\n", arch, name, (size_t)t->nbytes, cap);
            return false;
        }
        if (fseeko(fp, (off_t)(data_off + t->offset), SEEK_SET) != 0) return false;
        return std::fread(buf, 1, cap, fp) == cap;
    }

    // F32, BF16 (and F16) tensors widened to fp32; empty on failure (src/gguf_reader.h:139-149).
    std::vector<float> read_f32(const char* name) {
        const gguf_tensor_meta* t = meta(name);
        if (!t) {
            std::fprintf(stderr, "vla(%s): missing tensor %s\n", arch, name);
            return {};
        }
        // (the type first: only for the types sized at open() is the element count known to fit
        // the file; a record of an unknown type may declare any shape)
        if (t->type != GGUF_T_F32 && t->type != GGUF_T_BF16 && t->type != GGUF_T_F16) {
            std::fprintf(stderr, "vla(%s): tensor %s unsupported type %d\n", arch, name, (int)t->type);
            return {};
        }
        const size_t n = (size_t)t->nelements();
        std::vector<float> out(n);
        if (t->type == GGUF_T_F32) {
            if (!read_raw(name, out.data(), n * 4)) return {};
        } else if (t->type == GGUF_T_BF16 || t->type == GGUF_T_F16) {
            std::vector<uint16_t> tmp(n);
            if (!read_raw(name, tmp.data(), n * 2)) return {};
            for (size_t i = 0; i < n; ++i) out[i] = widen16(tmp[i], t->type);
        } else {
            std::fprintf(stderr, "vla(%s): tensor %s unsupported type %d\n", arch, name, (int)t->type);
            return {};
        }
        return out;
    }

    // Bytes of the tensor in the resident type `target`: F32 / BF16 convert (gemma_norm adds
    // 1.0 per weight first), any other target passes the file's bytes through
    // (src/gguf_reader.h:151-181).
    std::vector<uint8_t> read_convert(const char* name, uint32_t target, bool gemma_norm = false) {
        if (target != GGUF_T_F32 && target != GGUF_T_BF16) {
            if (gemma_norm) {
                std::fprintf(stderr, "vla(%s): %s needs the Gemma norm +1 but the target type is packed\n", arch, name);
                return {};
            }
            const gguf_tensor_meta* t = meta(name);
            if (!t) {
                std::fprintf(stderr, "vla(%s): missing tensor %s\n", arch, name);
                return {};
            }
            std::vector<uint8_t> o((size_t)t->nbytes);
            if (o.empty() || !read_raw(name, o.data(), o.size())) return {};
            return o;
        }
        std::vector<float> f = read_f32(name);
        if (f.empty()) return {};
        if (gemma_norm)
            for (float& v : f) v += 1.0f;
        std::vector<uint8_t> o(f.size() * (target == GGUF_T_F32 ? 4 : 2));
        if (target == GGUF_T_F32) {
            std::memcpy(o.data(), f.data(), o.size());
        } else {
            uint16_t* d = reinterpret_cast<uint16_t*>(o.data());
            for (size_t i = 0; i < f.size(); ++i) d[i] = gguf_float_to_bf16(f[i]);
        }
        return o;
    }

    // Rows of a 2-D F32 / BF16 (or F16) matrix left on disk, e.g. token embeddings
    // (src/gguf_reader.h:183-215).
    bool fetch_rows_f32(const char* name, const std::vector<int32_t>& row_ids, float* dst, int64_t cols) {
        const gguf_tensor_meta* t = meta(name);
        if (!t || t->ne[0] != cols || t->ne[2] != 1 || t->ne[3] != 1) {
            std::fprintf(stderr, "vla(%s): %s shape unfit for row-fetch\n", arch, name);
            return false;
        }
        if (t->type != GGUF_T_F32 && t->type != GGUF_T_BF16 && t->type != GGUF_T_F16) {
            std::fprintf(stderr, "vla(%s): %s type %d not f32/bf16 for row-fetch\n", arch, name, (int)t->type);
            return false;
        }
        const size_t elsz = t->type == GGUF_T_F32 ? 4u : 2u, rb = (size_t)cols * elsz;
        std::vector<uint8_t> row(rb);
        for (size_t k = 0; k < row_ids.size(); ++k) {
            const int32_t r = row_ids[k];
            if (r < 0 || r >= t->ne[1]) {
                std::fprintf(stderr, "vla(%s): row %d out of range for %s\n", arch, r, name);
                return false;
            }
            if (fseeko(fp, (off_t)(data_off + t->offset + (size_t)r * rb), SEEK_SET) != 0) return false;
            if (std::fread(row.data(), 1, rb, fp) != rb) return false;
            if (elsz == 4) {
                std::memcpy(dst + k * cols, row.data(), rb);
            } else {
                const uint16_t* s = reinterpret_cast<const uint16_t*>(row.data());
                for (int64_t c = 0; c < cols; ++c) dst[k * cols + c] = widen16(s[c], t->type);
            }
        }
        return true;
    }

  private:
    static float widen16(uint16_t h, uint32_t type) {
        if (type == GGUF_T_F16) return gguf_half_to_float(h);
        const uint32_t u = (uint32_t)h << 16;
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
    bool fail(const std::string& path, const char* why) {
        std::fprintf(stderr, "vla(%s): %s: %s\n", arch, path.c_str(), why);
        if (fp) std::fclose(fp);
        fp = nullptr;
        kv.clear();
        tensors.clear();
        index.clear();
        return false;
    }
    bool rd(void* dst, size_t n) { return std::fread(dst, 1, n, fp) == n; }
    uint64_t remaining() const { return file_size - (uint64_t)ftello(fp); }
    bool rd_str(std::string& s) {
        uint64_t len = 0;
        if (!rd(&len, 8) || len > remaining()) return false;
        s.resize((size_t)len);
        return len == 0 || rd(&s[0], (size_t)len);
    }
    static int scalar_size(uint32_t type) {
        switch (type) {
            case GGUF_KV_U8: case GGUF_KV_I8: case GGUF_KV_BOOL: return 1;
            case GGUF_KV_U16: case GGUF_KV_I16: return 2;
            case GGUF_KV_U32: case GGUF_KV_I32: case GGUF_KV_F32: return 4;
            case GGUF_KV_U64: case GGUF_KV_I64: case GGUF_KV_F64: return 8;
            default: return 0;
        }
    }
    bool rd_value(gguf_kv& v) {
        if (v.type == GGUF_KV_STRING) return rd_str(v.s);
        if (v.type == GGUF_KV_ARRAY) {
            if (!rd(&v.elem_type, 4) || !rd(&v.count, 8)) return false;
            if (v.elem_type == GGUF_KV_STRING) {
                if (v.count > remaining() / 8) return false;
                v.strs.resize((size_t)v.count);
                for (std::string& s : v.strs)
                    if (!rd_str(s)) return false;
                return true;
            }
            const int es = scalar_size(v.elem_type);  // nested arrays are not part of any file read here
            if (es == 0 || v.count > remaining() / (uint64_t)es) return false;
            v.raw.resize((size_t)v.count * es);
            return v.raw.empty() || rd(v.raw.data(), v.raw.size());
        }
        const int es = scalar_size(v.type);
        return es != 0 && rd(&v.bits, (size_t)es);
    }
};

}  // namespace vla
