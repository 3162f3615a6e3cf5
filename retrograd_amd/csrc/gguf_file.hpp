// GGUF v3 container access for the engine: a read-only mapping, the metadata
// the decode step needs and a name -> tensor index. Layout as written by the
// reference's fixture generators (scripts/gen-tiny-fixture.py:343-374) and by
// llama.cpp's converters: header, key/values, tensor table, aligned payloads.
#pragma once

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "transcode.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace retro {

struct TensorInfo {
    std::string name;
    int n_dims = 0;
    int64_t ne[4] = {1, 1, 1, 1};
    int type = 0;
    const uint8_t * data = nullptr;
    size_t nbytes = 0;
};

struct MetaValue {
    enum Kind { NONE, INT, FLOAT, STRING, INT_ARRAY, FLOAT_ARRAY, STRING_ARRAY } kind = NONE;
    int64_t i = 0;
    double f = 0.0;
    std::string s;
    std::vector<int64_t> ia;
    std::vector<double> fa;
    std::vector<std::string> sa;
};

class GgufFile {
public:
    explicit GgufFile(const std::string & path) : path_(path) {
        fd_ = ::open(path.c_str(), O_RDONLY);
        if (fd_ < 0) throw std::runtime_error("cannot open " + path);
        struct stat st {};
        if (::fstat(fd_, &st) != 0 || st.st_size < 24) {
            ::close(fd_);
            throw std::runtime_error("cannot read " + path);
        }
        size_ = (size_t)st.st_size;
        void * p = ::mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
        if (p == MAP_FAILED) {
            ::close(fd_);
            throw std::runtime_error("cannot map " + path);
        }
        map_ = (const uint8_t *)p;
        try {
            read_all();
        } catch (...) {
            ::munmap((void *)map_, size_);
            ::close(fd_);
            throw;
        }
    }
    ~GgufFile() {
        if (map_) ::munmap((void *)map_, size_);
        if (fd_ >= 0) ::close(fd_);
    }
    GgufFile(const GgufFile &) = delete;
    GgufFile & operator=(const GgufFile &) = delete;

    const std::string & path() const { return path_; }
    size_t file_size() const { return size_; }
    // Bytes of all tensor payloads: what llama_model_size reports for a file
    // whose tensors are all loaded.
    uint64_t tensor_bytes() const { return tensor_bytes_; }
    // Rewrites every tensor of a type Q8_0 holds exactly (transcode.hpp) as Q8_0 rows in memory of this object:
    // the loader then sees a Q8_0 tensor. tensor_bytes() keeps reporting the file's own sizes.
    void rewrite_as_q8_0() {
        for (TensorInfo & t : tensors_) {
            if (!q8_0_holds(t.type)) continue;
            size_t elems = 1;
            for (int d = 0; d < t.n_dims; ++d) elems *= (size_t)t.ne[d];
            owned_.emplace_back(elems / 32 * 34);
            to_q8_0(t.type, t.data, elems, owned_.back().data());
            t.type = GT_Q8_0;
            t.data = owned_.back().data();
            t.nbytes = owned_.back().size();
        }
    }
    // Frees what rewrite_as_q8_0 allocated; the rewritten tensors must not be read afterwards.
    void drop_rewritten() { owned_.clear(); owned_.shrink_to_fit(); }
    const std::vector<TensorInfo> & tensors() const { return tensors_; }
    const TensorInfo * find(const std::string & name) const {
        auto it = by_name_.find(name);
        return it == by_name_.end() ? nullptr : &tensors_[it->second];
    }
    const TensorInfo & require(const std::string & name) const {
        const TensorInfo * t = find(name);
        if (!t) throw std::runtime_error("model is missing tensor " + name);
        return *t;
    }
    const MetaValue * meta(const std::string & key) const {
        auto it = meta_.find(key);
        return it == meta_.end() ? nullptr : &it->second;
    }
    int64_t get_int(const std::string & key, int64_t dflt) const {
        const MetaValue * v = meta(key);
        if (!v) return dflt;
        if (v->kind == MetaValue::INT) return v->i;
        if (v->kind == MetaValue::FLOAT) return (int64_t)v->f;
        return dflt;
    }
    int64_t need_int(const std::string & key) const {
        const MetaValue * v = meta(key);
        if (!v || v->kind != MetaValue::INT) throw std::runtime_error("model is missing metadata " + key);
        return v->i;
    }
    double get_float(const std::string & key, double dflt) const {
        const MetaValue * v = meta(key);
        if (!v) return dflt;
        if (v->kind == MetaValue::FLOAT) return v->f;
        if (v->kind == MetaValue::INT) return (double)v->i;
        return dflt;
    }
    std::string get_string(const std::string & key, const std::string & dflt = "") const {
        const MetaValue * v = meta(key);
        return v && v->kind == MetaValue::STRING ? v->s : dflt;
    }

private:
    struct Cursor {
        const uint8_t * p;
        const uint8_t * end;
        template <typename T> T take() {
            if ((size_t)(end - p) < sizeof(T)) throw std::runtime_error("truncated GGUF header");
            T v;
            std::memcpy(&v, p, sizeof(T));
            p += sizeof(T);
            return v;
        }
        std::string take_string() {
            const uint64_t n = take<uint64_t>();
            if ((uint64_t)(end - p) < n) throw std::runtime_error("truncated GGUF string");
            std::string s((const char *)p, (size_t)n);
            p += n;
            return s;
        }
    };

    static bool scalar(Cursor & c, uint32_t type, MetaValue & out) {
        switch (type) {
            case 0: out.kind = MetaValue::INT; out.i = c.take<uint8_t>(); return true;
            case 1: out.kind = MetaValue::INT; out.i = c.take<int8_t>(); return true;
            case 2: out.kind = MetaValue::INT; out.i = c.take<uint16_t>(); return true;
            case 3: out.kind = MetaValue::INT; out.i = c.take<int16_t>(); return true;
            case 4: out.kind = MetaValue::INT; out.i = c.take<uint32_t>(); return true;
            case 5: out.kind = MetaValue::INT; out.i = c.take<int32_t>(); return true;
            case 6: out.kind = MetaValue::FLOAT; out.f = c.take<float>(); return true;
            case 7: out.kind = MetaValue::INT; out.i = c.take<uint8_t>() ? 1 : 0; return true;
            case 8: out.kind = MetaValue::STRING; out.s = c.take_string(); return true;
            case 10: out.kind = MetaValue::INT; out.i = (int64_t)c.take<uint64_t>(); return true;
            case 11: out.kind = MetaValue::INT; out.i = c.take<int64_t>(); return true;
            case 12: out.kind = MetaValue::FLOAT; out.f = c.take<double>(); return true;
            default: return false;
        }
    }

    static size_t payload_bytes(const TensorInfo & t) {
        int64_t elems = 1, block = 1, bytes = 0;
        switch (t.type) {
            case 0: block = 1; bytes = 4; break;
            case 1: case 30: block = 1; bytes = 2; break;
            case 8: block = 32; bytes = 34; break;
            case 12: block = 256; bytes = 144; break;
            case 39: block = 32; bytes = 17; break;
            // other ggml types are carried through unparsed; the engine refuses them at load
            case 2: block = 32; bytes = 18; break;
            case 3: block = 32; bytes = 20; break;
            case 6: block = 32; bytes = 22; break;
            case 7: block = 32; bytes = 24; break;
            case 10: block = 256; bytes = 84; break;
            case 11: block = 256; bytes = 110; break;
            case 13: block = 256; bytes = 176; break;
            case 14: block = 256; bytes = 210; break;
            case 20: block = 32; bytes = 18; break;
            case 23: block = 256; bytes = 136; break;
            default: return 0;
        }
        for (int d = 0; d < t.n_dims; ++d) {
            if (t.ne[d] <= 0) throw std::runtime_error("tensor " + t.name + " has a dimension that is not positive");
            if (elems > ((int64_t)1 << 46) / t.ne[d]) throw std::runtime_error("tensor " + t.name + " is larger than any file");
            elems *= t.ne[d];
        }
        if (t.ne[0] % block != 0) throw std::runtime_error("tensor " + t.name + " has rows that are not whole blocks of its type");
        return (size_t)(elems / block * bytes);
    }

    void read_all() {
        Cursor c{map_, map_ + size_};
        if (c.take<uint32_t>() != 0x46554747u) throw std::runtime_error(path_ + " is not a GGUF file");
        const uint32_t version = c.take<uint32_t>();
        if (version < 2 || version > 3) throw std::runtime_error("unsupported GGUF version");
        const uint64_t n_tensors = c.take<uint64_t>();
        const uint64_t n_kv = c.take<uint64_t>();
        // every key/value takes at least 12 bytes of the file and every tensor entry at least 24
        if (n_kv > size_ / 12 || n_tensors > size_ / 24) throw std::runtime_error(path_ + ": the GGUF header counts more entries than the file can hold");
        for (uint64_t k = 0; k < n_kv; ++k) {
            std::string key = c.take_string();
            const uint32_t type = c.take<uint32_t>();
            MetaValue v;
            if (type == 9) {
                const uint32_t et = c.take<uint32_t>();
                const uint64_t n = c.take<uint64_t>();
                if (n > (uint64_t)(c.end - c.p)) throw std::runtime_error("truncated GGUF array for key " + key);
                v.kind = et == 8 ? MetaValue::STRING_ARRAY : ((et == 6 || et == 12) ? MetaValue::FLOAT_ARRAY : MetaValue::INT_ARRAY);
                for (uint64_t i = 0; i < n; ++i) {
                    MetaValue e;
                    if (!scalar(c, et, e)) throw std::runtime_error("unsupported GGUF array element type");
                    if (et == 8) v.sa.push_back(std::move(e.s));
                    else if (e.kind == MetaValue::FLOAT) v.fa.push_back(e.f);
                    else v.ia.push_back(e.i);
                }
            } else if (!scalar(c, type, v)) {
                throw std::runtime_error("unsupported GGUF value type for key " + key);
            }
            meta_.emplace(std::move(key), std::move(v));
        }
        tensors_.resize((size_t)n_tensors);
        std::vector<uint64_t> offsets((size_t)n_tensors);
        for (size_t i = 0; i < tensors_.size(); ++i) {
            TensorInfo & t = tensors_[i];
            t.name = c.take_string();
            t.n_dims = (int)c.take<uint32_t>();
            if (t.n_dims < 1 || t.n_dims > 4) throw std::runtime_error("tensor " + t.name + " has a bad rank");
            for (int d = 0; d < t.n_dims; ++d) t.ne[d] = (int64_t)c.take<uint64_t>();
            t.type = (int)c.take<uint32_t>();
            offsets[i] = c.take<uint64_t>();
        }
        const int64_t align_field = get_int("general.alignment", 32);
        if (align_field < 1 || align_field > (1 << 20) || (align_field & (align_field - 1)) != 0)
            throw std::runtime_error(path_ + ": general.alignment must be a power of two");
        const uint64_t align = (uint64_t)align_field;
        const uint64_t header = (uint64_t)(c.p - map_);
        const uint64_t data0 = (header + align - 1) / align * align;
        if (data0 > size_) throw std::runtime_error(path_ + ": the tensor data starts past the end of the file");
        const uint64_t room = size_ - data0;
        for (size_t i = 0; i < tensors_.size(); ++i) {
            TensorInfo & t = tensors_[i];
            t.nbytes = payload_bytes(t);
            // compared without sums, which a huge offset would wrap
            if (offsets[i] > room || t.nbytes > room - offsets[i]) throw std::runtime_error("tensor " + t.name + " runs past the file");
            t.data = map_ + data0 + offsets[i];
            by_name_[t.name] = i;
            tensor_bytes_ += t.nbytes;
        }
    }

    std::string path_;
    int fd_ = -1;
    size_t size_ = 0;
    const uint8_t * map_ = nullptr;
    std::unordered_map<std::string, MetaValue> meta_;
    std::vector<TensorInfo> tensors_;
    std::unordered_map<std::string, size_t> by_name_;
    uint64_t tensor_bytes_ = 0;
    std::vector<std::vector<uint8_t>> owned_;
};

}  // namespace retro
