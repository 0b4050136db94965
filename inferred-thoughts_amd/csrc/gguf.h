// Memory-mapped GGUF v3 reader: metadata needed by the qwen35moe loader and the
// tensor table.  Container facts follow /root/reference src/gguf/mod.rs:143-296 and
// src/gguf/metadata.rs:131-205 (value type codes, u64 string lengths, tensor dims
// as i64 in ggml order, data blob aligned to general.alignment, default 32;
// duplicate tensor names are rejected).
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <variant>
#include <vector>

namespace itg {

struct Tensor {
    std::string name;
    std::vector<uint64_t> dims;  // ggml order: dims[0] is the row length
    uint32_t ty = 0;
    uint64_t offset = 0;  // relative to the data blob
    // the product of the dims; false when it does not fit 64 bits (a corrupt or hostile file)
    bool n_elems_checked(uint64_t* out) const {
        uint64_t n = 1;
        for (auto d : dims)
            if (__builtin_mul_overflow(n, d, &n)) return false;
        *out = n;
        return true;
    }
    uint64_t n_elems() const {  // of a tensor File::open has accepted
        uint64_t n = 1;
        for (auto d : dims) n *= d;
        return n;
    }
};

using Value = std::variant<uint64_t, int64_t, double, bool, std::string, std::vector<int32_t>>;

class File {
  public:
    ~File();
    bool open(const std::string& path, std::string* err);
    const Tensor* tensor(const std::string& name) const;
    const uint8_t* bytes(const Tensor& t) const { return base_ + data_start_ + t.offset; }
    // unsigned getters accept any integer width (metadata.rs:313-330)
    bool get_uint(const std::string& key, uint64_t* out) const;
    bool get_float(const std::string& key, float* out) const;
    bool get_string(const std::string& key, std::string* out) const;
    const std::vector<int32_t>* get_i32_array(const std::string& key) const;
    size_t size() const { return size_; }
    const uint8_t* base() const { return base_; }   // where the file is mapped
    const std::vector<Tensor>& tensors() const { return tensors_; }

  private:
    int fd_ = -1;
    const uint8_t* base_ = nullptr;
    size_t size_ = 0, data_start_ = 0;
    std::unordered_map<std::string, Value> meta_;
    std::vector<Tensor> tensors_;
    std::unordered_map<std::string, size_t> by_name_;
};

// bytes of `n` elements of a ggml type; 0 when unsupported or not whole blocks
// (src/gguf/types.rs:143-210)
uint64_t type_bytes(uint32_t ty, uint64_t n);
// the same with the multiplication checked: false when the byte count does not fit 64 bits
bool type_bytes_checked(uint32_t ty, uint64_t n, uint64_t* out);

}  // namespace itg
