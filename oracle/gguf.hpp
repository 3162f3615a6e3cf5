// TEST INFRASTRUCTURE - CPU oracle, never linked into or called by the product.
//
// Minimal GGUF v3 reader: the container the reference's fixture generators
// write (scripts/gen-tiny-fixture.py:265-374 - header "GGUF", version 3,
// tensor count, kv count; typed key/values; tensor table of name, n_dims,
// ne[], type, offset; data aligned to general.alignment, default 32).
// Pinned by tests/test_gguf_fixture.py: files written to the reference's
// published sha256 digests (tests/fixtures/TINY_*_FIXTURE.toml) are parsed
// back by this reader.
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace oracle {

struct gguf_tensor {
    std::string name;
    std::vector<uint64_t> ne;   // fastest dimension first
    uint32_t type = 0;
    uint64_t offset = 0;        // relative to the data section
    const uint8_t * data = nullptr;
};

struct gguf_value {
    uint32_t type = 0;          // GGUF value type
    uint64_t u = 0;             // integers / bool
    double f = 0.0;             // floats
    std::string s;              // strings
    uint32_t arr_type = 0;
    uint64_t arr_n = 0;
    std::vector<std::string> arr_s;
    std::vector<double> arr_f;  // numeric arrays, widened
};

class gguf_file {
public:
    explicit gguf_file(const std::string & path) {
        fd_ = ::open(path.c_str(), O_RDONLY);
        if (fd_ < 0) throw std::runtime_error("oracle: cannot open " + path);
        struct stat st {};
        if (fstat(fd_, &st) != 0) throw std::runtime_error("oracle: cannot stat " + path);
        size_ = (size_t)st.st_size;
        base_ = (const uint8_t *)mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
        if (base_ == MAP_FAILED) throw std::runtime_error("oracle: cannot map " + path);
        parse();
    }
    ~gguf_file() {
        if (base_ && base_ != MAP_FAILED) munmap((void *)base_, size_);
        if (fd_ >= 0) ::close(fd_);
    }
    gguf_file(const gguf_file &) = delete;
    gguf_file & operator=(const gguf_file &) = delete;

    const gguf_tensor * find(const std::string & name) const {
        auto it = index_.find(name);
        return it == index_.end() ? nullptr : &tensors[it->second];
    }
    const gguf_tensor & need(const std::string & name) const {
        const gguf_tensor * t = find(name);
        if (!t) throw std::runtime_error("oracle: missing tensor " + name);
        return *t;
    }
    bool has(const std::string & key) const { return kv.count(key) != 0; }
    uint64_t u(const std::string & key) const { return at(key).u; }
    double f(const std::string & key) const { return at(key).f; }
    const std::string & s(const std::string & key) const { return at(key).s; }
    uint64_t u_or(const std::string & key, uint64_t dflt) const { return has(key) ? u(key) : dflt; }
    double f_or(const std::string & key, double dflt) const { return has(key) ? f(key) : dflt; }
    const gguf_value & at(const std::string & key) const {
        auto it = kv.find(key);
        if (it == kv.end()) throw std::runtime_error("oracle: missing metadata key " + key);
        return it->second;
    }
    size_t file_size() const { return size_; }

    std::map<std::string, gguf_value> kv;
    std::vector<gguf_tensor> tensors;

private:
    template <typename T> T rd() {
        if (pos_ + sizeof(T) > size_) throw std::runtime_error("oracle: truncated gguf");
        T v;
        std::memcpy(&v, base_ + pos_, sizeof(T));
        pos_ += sizeof(T);
        return v;
    }
    std::string rd_str() {
        const uint64_t n = rd<uint64_t>();
        if (pos_ + n > size_) throw std::runtime_error("oracle: truncated gguf string");
        std::string s((const char *)base_ + pos_, n);
        pos_ += n;
        return s;
    }
    void rd_scalar(uint32_t type, gguf_value & v) {
        switch (type) {
            case 0: v.u = rd<uint8_t>(); break;
            case 1: v.u = (uint64_t)(int64_t)rd<int8_t>(); break;
            case 2: v.u = rd<uint16_t>(); break;
            case 3: v.u = (uint64_t)(int64_t)rd<int16_t>(); break;
            case 4: v.u = rd<uint32_t>(); break;
            case 5: v.u = (uint64_t)(int64_t)rd<int32_t>(); break;
            case 6: v.f = rd<float>(); break;
            case 7: v.u = rd<uint8_t>() != 0; break;
            case 8: v.s = rd_str(); break;
            case 10: v.u = rd<uint64_t>(); break;
            case 11: v.u = (uint64_t)rd<int64_t>(); break;
            case 12: v.f = rd<double>(); break;
            default: throw std::runtime_error("oracle: unknown gguf value type");
        }
        if (type != 6 && type != 12 && type != 8) v.f = (double)(int64_t)v.u;
    }
    void parse() {
        if (rd<uint32_t>() != 0x46554747u) throw std::runtime_error("oracle: not a GGUF file");
        const uint32_t version = rd<uint32_t>();
        if (version != 3 && version != 2) throw std::runtime_error("oracle: unsupported GGUF version");
        const uint64_t n_tensors = rd<uint64_t>();
        const uint64_t n_kv = rd<uint64_t>();
        for (uint64_t i = 0; i < n_kv; ++i) {
            const std::string key = rd_str();
            gguf_value v;
            v.type = rd<uint32_t>();
            if (v.type == 9) {
                v.arr_type = rd<uint32_t>();
                v.arr_n = rd<uint64_t>();
                for (uint64_t j = 0; j < v.arr_n; ++j) {
                    gguf_value e;
                    rd_scalar(v.arr_type, e);
                    if (v.arr_type == 8) v.arr_s.push_back(std::move(e.s));
                    else v.arr_f.push_back(e.f);
                }
            } else {
                rd_scalar(v.type, v);
            }
            kv.emplace(key, std::move(v));
        }
        tensors.resize(n_tensors);
        for (auto & t : tensors) {
            t.name = rd_str();
            const uint32_t nd = rd<uint32_t>();
            t.ne.resize(nd);
            for (auto & d : t.ne) d = rd<uint64_t>();
            t.type = rd<uint32_t>();
            t.offset = rd<uint64_t>();
        }
        const uint64_t align = u_or("general.alignment", 32);
        const size_t data0 = (pos_ + align - 1) / align * align;
        for (size_t i = 0; i < tensors.size(); ++i) {
            tensors[i].data = base_ + data0 + tensors[i].offset;
            index_[tensors[i].name] = i;
        }
    }

    int fd_ = -1;
    size_t size_ = 0;
    size_t pos_ = 0;
    const uint8_t * base_ = nullptr;
    std::map<std::string, size_t> index_;
};

}  // namespace oracle
