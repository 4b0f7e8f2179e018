// proto3 wire codec for the two messages of the reference's serving protocol
// (src/serving/vla.proto): PredictRequest is parsed, PredictResponse is written (and both
// the other way round for clients and tests).  The encoding rules are protobuf's published
// ones: a field is (number << 3 | wire type) as a varint, wire type 0 = varint, 1 = 64-bit,
// 2 = length-delimited, 5 = 32-bit; repeated scalars arrive packed (one length-delimited
// run) or one element per field, and both must be accepted; unknown fields are skipped;
// default values are not written; fields are written in field-number order, which is what
// the protobuf libraries emit, so frames compare equal byte for byte.
#pragma once

#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace vla {
namespace wire {

struct Reader {
    const uint8_t* p;
    const uint8_t* end;
    bool ok = true;
    Reader(const uint8_t* b, size_t n) : p(b), end(b + n) {}
    bool done() const { return p >= end; }
    uint64_t varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 64; shift += 7) {
            if (p >= end) break;
            const uint8_t b = *p++;
            v |= (uint64_t)(b & 0x7f) << shift;
            if (!(b & 0x80)) return v;
        }
        ok = false;
        return 0;
    }
    uint32_t fixed32() {
        if (end - p < 4) {
            ok = false;
            return 0;
        }
        uint32_t v;
        std::memcpy(&v, p, 4);
        p += 4;
        return v;
    }
    Reader sub() {  // a length-delimited payload
        const uint64_t n = varint();
        if (!ok || n > (uint64_t)(end - p)) {
            ok = false;
            return Reader(p, 0);
        }
        Reader r(p, (size_t)n);
        p += n;
        return r;
    }
    void skip(int wt) {
        switch (wt) {
            case 0: varint(); break;
            case 1: if (end - p < 8) ok = false; else p += 8; break;
            case 2: sub(); break;
            case 5: fixed32(); break;
            default: ok = false;  // groups (3, 4) are not part of proto3
        }
    }
};

// repeated float: packed run (wire type 2) or a single fixed32 (wire type 5)
inline bool read_floats(Reader& r, int wt, std::vector<float>& out) {
    if (wt == 5) {
        const uint32_t u = r.fixed32();
        float f;
        std::memcpy(&f, &u, 4);
        out.push_back(f);
        return r.ok;
    }
    if (wt != 2) return false;
    Reader s = r.sub();
    if (!r.ok || (s.end - s.p) % 4 != 0) return false;
    const size_t n = (size_t)(s.end - s.p) / 4, at = out.size();
    out.resize(at + n);
    if (n) std::memcpy(out.data() + at, s.p, n * 4);
    return true;
}

// repeated (u)int32: packed varints or a single varint; int32 is the low 32 bits of the
// (sign-extended) 64-bit varint
template <typename T>
inline bool read_ints(Reader& r, int wt, std::vector<T>& out) {
    if (wt == 0) {
        out.push_back((T)(uint32_t)r.varint());
        return r.ok;
    }
    if (wt != 2) return false;
    Reader s = r.sub();
    if (!r.ok) return false;
    while (!s.done()) {
        out.push_back((T)(uint32_t)s.varint());
        if (!s.ok) return false;
    }
    return true;
}

struct PredictRequest {
    int n_images = 0;  // Image messages are counted, not decoded (no vision tower here)
    std::vector<int32_t> lang_tokens;
    std::vector<float> state, noise, precomputed_img_emb;
    uint64_t request_id = 0;
    uint32_t precomputed_img_emb_n_views = 0;
    std::vector<uint32_t> attention_mask;
};

inline bool parse_request(const uint8_t* buf, size_t n, PredictRequest& q) {
    Reader r(buf, n);
    while (!r.done()) {
        const uint64_t key = r.varint();
        if (!r.ok) return false;
        const int wt = (int)(key & 7);
        bool good = true;
        switch (key >> 3) {
            case 1: if (wt != 2) return false; r.sub(); ++q.n_images; break;
            case 2: good = read_ints(r, wt, q.lang_tokens); break;
            case 3: good = read_floats(r, wt, q.state); break;
            case 4: good = read_floats(r, wt, q.noise); break;
            case 5: if (wt != 0) return false; q.request_id = r.varint(); break;
            case 6: good = read_floats(r, wt, q.precomputed_img_emb); break;
            case 7: if (wt != 0) return false; q.precomputed_img_emb_n_views = (uint32_t)r.varint(); break;
            case 8: good = read_ints(r, wt, q.attention_mask); break;
            case 0: return false;
            default: r.skip(wt);
        }
        if (!good || !r.ok) return false;
    }
    return true;
}

struct Writer {
    std::string out;
    void varint(uint64_t v) {
        while (v >= 0x80) {
            out.push_back((char)(v | 0x80));
            v >>= 7;
        }
        out.push_back((char)v);
    }
    void key(int field, int wt) { varint((uint64_t)field << 3 | (uint64_t)wt); }
    void u64(int field, uint64_t v) {
        if (v) {
            key(field, 0);
            varint(v);
        }
    }
    void f32(int field, float v) {
        uint32_t u;
        std::memcpy(&u, &v, 4);
        if (u) {  // proto3 skips +0.0 only; -0.0 has a set sign bit and is written
            key(field, 5);
            out.append((const char*)&u, 4);
        }
    }
    void floats(int field, const float* v, size_t n) {
        if (n) {
            key(field, 2);
            varint(n * 4);
            out.append((const char*)v, n * 4);
        }
    }
    template <typename T>
    void ints(int field, const T* v, size_t n) {  // packed; int32 sign-extends to 64 bits
        if (!n) return;
        Writer body;
        for (size_t i = 0; i < n; ++i) body.varint((uint64_t)(int64_t)v[i]);
        key(field, 2);
        varint(body.out.size());
        out += body.out;
    }
    void str(int field, const std::string& s) {
        if (!s.empty()) {
            key(field, 2);
            varint(s.size());
            out += s;
        }
    }
};

struct PredictResponse {
    uint64_t request_id = 0;
    std::vector<float> action_chunk;
    uint32_t chunk_size = 0, action_dim = 0;
    float ms_total = 0.f, ms_inference = 0.f, ms_prefill = 0.f, ms_denoise = 0.f, ms_vision = 0.f;
    std::string error;
};

inline std::string encode_response(const PredictResponse& r) {
    Writer w;
    w.u64(1, r.request_id);
    w.floats(2, r.action_chunk.data(), r.action_chunk.size());
    w.u64(3, r.chunk_size);
    w.u64(4, r.action_dim);
    w.f32(5, r.ms_total);
    w.f32(6, r.ms_inference);
    w.str(7, r.error);
    w.f32(8, r.ms_prefill);
    w.f32(9, r.ms_denoise);
    w.f32(10, r.ms_vision);
    return w.out;
}

inline bool parse_response(const uint8_t* buf, size_t n, PredictResponse& q) {
    Reader r(buf, n);
    auto f = [&](float& dst, int wt) {
        if (wt != 5) return false;
        const uint32_t u = r.fixed32();
        std::memcpy(&dst, &u, 4);
        return r.ok;
    };
    while (!r.done()) {
        const uint64_t key = r.varint();
        if (!r.ok) return false;
        const int wt = (int)(key & 7);
        bool good = true;
        switch (key >> 3) {
            case 1: if (wt != 0) return false; q.request_id = r.varint(); break;
            case 2: good = read_floats(r, wt, q.action_chunk); break;
            case 3: if (wt != 0) return false; q.chunk_size = (uint32_t)r.varint(); break;
            case 4: if (wt != 0) return false; q.action_dim = (uint32_t)r.varint(); break;
            case 5: good = f(q.ms_total, wt); break;
            case 6: good = f(q.ms_inference, wt); break;
            case 7: {
                if (wt != 2) return false;
                Reader s = r.sub();
                if (r.ok) q.error.assign((const char*)s.p, (size_t)(s.end - s.p));
                break;
            }
            case 8: good = f(q.ms_prefill, wt); break;
            case 9: good = f(q.ms_denoise, wt); break;
            case 10: good = f(q.ms_vision, wt); break;
            case 0: return false;
            default: r.skip(wt);
        }
        if (!good || !r.ok) return false;
    }
    return true;
}

inline std::string encode_request(const PredictRequest& q) {
    Writer w;
    w.ints(2, q.lang_tokens.data(), q.lang_tokens.size());
    w.floats(3, q.state.data(), q.state.size());
    w.floats(4, q.noise.data(), q.noise.size());
    w.u64(5, q.request_id);
    w.floats(6, q.precomputed_img_emb.data(), q.precomputed_img_emb.size());
    w.u64(7, q.precomputed_img_emb_n_views);
    w.ints(8, q.attention_mask.data(), q.attention_mask.size());
    return w.out;
}

}  // namespace wire
}  // namespace vla
