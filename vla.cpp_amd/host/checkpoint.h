// Weight container the model builders read.  Filled either from a "VLAW" file (the flat
// container written by vla.cpp_amd/checkpoint.py) or in memory by the GGUF importer
// (gguf_import.cpp), which maps the reference's tensor names (src/models/*.cpp) onto the
// names used here.  VLAW layout:
//
//   bytes 0..7   "VLAW0001"
//   bytes 8..15  header length H (little-endian uint64)
//   H bytes      text header, one record per line:
//                  K <key> <value>
//                  T <name> <dtype> <ndim> <d0> [<d1> ...] <offset> <nbytes>
//   data         starts at the next multiple of 64 after the header; tensor
//                offsets are relative to it.  dtype in {f32, bf16, i8, u8, i32}.
//
// Written by vla.cpp_amd/checkpoint.py.
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <mutex>
#include <string>
#include <vector>

namespace vla {

// Rows of a matrix that stays on disk and is read per request: the token embeddings of a
// 257k-row vocabulary are 2 GB as fp32, and one observation uses a few dozen rows (the
// reference fetches them the same way, fetch_rows_f32, src/models/pi0.cpp:530-534).
struct RowSource {
    int64_t rows = 0, cols = 0;
    virtual ~RowSource() = default;
    // dst receives ids.size() x cols floats; false on an id outside [0, rows) or a read error.
    // Callers on several threads (a batch's observations are staged in parallel) go through
    // fetch_locked: an implementation reads through one file handle.
    virtual bool fetch(const std::vector<int32_t>& ids, float* dst) = 0;
    bool fetch_locked(const std::vector<int32_t>& ids, float* dst) {
        std::lock_guard<std::mutex> hold(mu_);
        return fetch(ids, dst);
    }

  private:
    std::mutex mu_;
};

inline size_t ckpt_dtype_size(const std::string& dt) {
    if (dt == "f32" || dt == "i32") return 4;
    if (dt == "bf16") return 2;
    if (dt == "i8" || dt == "u8") return 1;
    return 0;
}

struct CkptTensor {
    std::string dtype;
    std::vector<int64_t> shape;
    size_t offset = 0, nbytes = 0;
    int64_t numel() const {
        int64_t n = 1;
        for (int64_t d : shape) n *= d;
        return n;
    }
};

class Checkpoint {
  public:
    Checkpoint() = default;  // empty; filled with set_key / add_tensor

    void set_key(const std::string& k, const std::string& v) { kv_[k] = v; }
    void set_key(const std::string& k, int64_t v) { kv_[k] = std::to_string(v); }
    void set_key(const std::string& k, double v) {
        char buf[64];
        std::snprintf(buf, sizeof(buf), "%.17g", v);
        kv_[k] = buf;
    }
    // Appends a tensor (bytes copied, 64-byte aligned); dtype as in the VLAW header.
    void add_tensor(const std::string& name, const std::string& dtype, const std::vector<int64_t>& shape, const void* bytes,
                    size_t nbytes) {
        CkptTensor t;
        t.dtype = dtype;
        t.shape = shape;
        t.offset = (blob_.size() + 63) / 64 * 64;
        t.nbytes = nbytes;
        blob_.resize(t.offset + nbytes);
        if (nbytes) std::memcpy(blob_.data() + t.offset, bytes, nbytes);
        tensors_[name] = t;
    }
    void add_f32(const std::string& name, const std::vector<int64_t>& shape, const std::vector<float>& v) {
        add_tensor(name, "f32", shape, v.data(), v.size() * sizeof(float));
    }

    explicit Checkpoint(const std::string& path) {
        FILE* f = std::fopen(path.c_str(), "rb");
        if (!f) throw std::runtime_error("vla: cannot open checkpoint " + path);
        std::fseek(f, 0, SEEK_END);
        const long sz = std::ftell(f);
        std::fseek(f, 0, SEEK_SET);
        blob_.resize((size_t)sz);
        const size_t got = std::fread(blob_.data(), 1, (size_t)sz, f);
        std::fclose(f);
        if (got != (size_t)sz || sz < 16 || std::string(blob_.data(), 8) != "VLAW0001")
            throw std::runtime_error("vla: " + path + " is not a VLAW0001 checkpoint");
        uint64_t hlen = 0;
        std::memcpy(&hlen, blob_.data() + 8, 8);
        if (hlen > (uint64_t)sz - 16) throw std::runtime_error("vla: truncated checkpoint header");
        data_ = (16 + (size_t)hlen + 63) / 64 * 64;
        if (data_ > blob_.size()) data_ = blob_.size();
        std::istringstream hs(std::string(blob_.data() + 16, (size_t)hlen));
        std::string line;
        while (std::getline(hs, line)) {
            std::istringstream ls(line);
            std::string tag;
            ls >> tag;
            if (tag == "K") {
                std::string k, v;
                ls >> k >> v;
                kv_[k] = v;
            } else if (tag == "T") {
                std::string name;
                CkptTensor t;
                int ndim = 0;
                ls >> name >> t.dtype >> ndim;
                if (!ls || ndim < 0 || ndim > 8) throw std::runtime_error("vla: tensor " + name + " has a malformed record");
                t.shape.resize((size_t)ndim);
                int64_t numel = 1;
                for (int i = 0; i < ndim; ++i) {
                    ls >> t.shape[i];
                    if (!ls || t.shape[i] <= 0 || t.shape[i] > ((int64_t)1 << 40) / numel)
                        throw std::runtime_error("vla: tensor " + name + " has a malformed shape");
                    numel *= t.shape[i];
                }
                ls >> t.offset >> t.nbytes;
                const size_t room = blob_.size() - data_;  // data_ <= blob_.size() was checked above
                const size_t es = ckpt_dtype_size(t.dtype);
                if (!ls || es == 0 || t.offset > room || t.nbytes > room - t.offset)
                    throw std::runtime_error("vla: tensor " + name + " lies outside the checkpoint");
                if (t.nbytes != (size_t)numel * es)
                    throw std::runtime_error("vla: tensor " + name + " declares " + std::to_string(t.nbytes) + " bytes for " +
                                             std::to_string(numel) + " " + t.dtype + " elements");
                tensors_[name] = t;
            }
        }
    }

    bool has(const std::string& name) const { return tensors_.count(name) != 0; }
    const CkptTensor& info(const std::string& name) const {
        auto it = tensors_.find(name);
        if (it == tensors_.end()) throw std::runtime_error("vla: checkpoint has no tensor " + name);
        return it->second;
    }
    const void* data(const std::string& name) const { return blob_.data() + data_ + info(name).offset; }
    // info(name), after checking that the tensor has exactly this shape: a file whose tensors
    // do not match its own configuration must fail at load, not as an out-of-bounds read on
    // the device.
    const CkptTensor& expect(const std::string& name, const std::vector<int64_t>& shape) const {
        const CkptTensor& t = info(name);
        auto squeeze = [](const std::vector<int64_t>& v) {  // [1, W] and [W] name the same vector
            std::vector<int64_t> o;
            for (int64_t d : v)
                if (d != 1) o.push_back(d);
            return o;
        };
        if (squeeze(t.shape) != squeeze(shape)) {
            std::string got, want;
            for (int64_t d : t.shape) got += (got.empty() ? "" : " x ") + std::to_string(d);
            for (int64_t d : shape) want += (want.empty() ? "" : " x ") + std::to_string(d);
            throw std::runtime_error("vla: checkpoint tensor " + name + " is [" + got + "], expected [" + want + "]");
        }
        return t;
    }

    // A matrix left on disk (see RowSource); the model keeps the pointer after the
    // checkpoint object is gone.
    void set_row_source(const std::string& name, std::shared_ptr<RowSource> src) { rows_[name] = std::move(src); }
    std::shared_ptr<RowSource> row_source(const std::string& name) const {
        auto it = rows_.find(name);
        return it == rows_.end() ? nullptr : it->second;
    }

    // Tensor as fp32 on the host (bf16 widened exactly).
    std::vector<float> f32(const std::string& name) const {
        const CkptTensor& t = info(name);
        std::vector<float> out((size_t)t.numel());
        if (t.dtype == "f32") {
            std::memcpy(out.data(), data(name), out.size() * 4);
        } else if (t.dtype == "bf16") {
            const uint16_t* p = (const uint16_t*)data(name);
            for (size_t i = 0; i < out.size(); ++i) {
                uint32_t u = ((uint32_t)p[i]) << 16;
                std::memcpy(&out[i], &u, 4);
            }
        } else {
            throw std::runtime_error("vla: tensor " + name + " is not floating point");
        }
        return out;
    }

    std::string str(const std::string& key) const {
        auto it = kv_.find(key);
        if (it == kv_.end()) throw std::runtime_error("vla: checkpoint has no key " + key);
        return it->second;
    }
    bool has_key(const std::string& key) const { return kv_.count(key) != 0; }
    int64_t i64(const std::string& key) const { return std::stoll(str(key)); }
    int64_t i64(const std::string& key, int64_t dflt) const { return has_key(key) ? i64(key) : dflt; }
    double f64(const std::string& key) const { return std::stod(str(key)); }
    double f64(const std::string& key, double dflt) const { return has_key(key) ? f64(key) : dflt; }

  private:
    std::vector<char> blob_;
    size_t data_ = 0;
    std::map<std::string, std::string> kv_;
    std::map<std::string, CkptTensor> tensors_;
    std::map<std::string, std::shared_ptr<RowSource>> rows_;
};

// GGUF input (gguf_import.cpp): true when the file starts with the GGUF magic; import_gguf
// reads the tensors on the action-expert path under the reference's names and throws
// std::runtime_error on a file it cannot use.
bool is_gguf_file(const std::string& path);
Checkpoint import_gguf(const std::string& path);

}  // namespace vla
