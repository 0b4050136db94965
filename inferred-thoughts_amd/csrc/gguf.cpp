#include "gguf.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>

namespace itg {

uint64_t type_bytes(uint32_t ty, uint64_t n) {
    switch (ty) {
        case 0: return n * 4;                           // F32
        case 1: case 30: return n * 2;                  // F16, BF16
        case 8: return n % 32 ? 0 : n / 32 * 34;        // Q8_0
        case 40: return n % 64 ? 0 : n / 64 * 36;       // NVFP4
        default: return 0;
    }
}

bool type_bytes_checked(uint32_t ty, uint64_t n, uint64_t* out) {
    switch (ty) {
        case 0: return !__builtin_mul_overflow(n, (uint64_t)4, out);
        case 1: case 30: return !__builtin_mul_overflow(n, (uint64_t)2, out);
        default: *out = type_bytes(ty, n); return true;  // block formats shrink: n / 32 * 34 and n / 64 * 36 cannot wrap
    }
}

namespace {
struct Reader {
    const uint8_t* p;
    const uint8_t* end;
    bool ok = true;
    template <class T>
    T take() {
        T v{};
        if ((size_t)(end - p) < sizeof(T)) {
            ok = false;
            return v;
        }
        memcpy(&v, p, sizeof(T));
        p += sizeof(T);
        return v;
    }
    std::string str() {
        uint64_t n = take<uint64_t>();
        if (!ok || (uint64_t)(end - p) < n) {
            ok = false;
            return {};
        }
        std::string s((const char*)p, (size_t)n);
        p += n;
        return s;
    }
    void skip(uint64_t n) {
        if ((uint64_t)(end - p) < n) ok = false;
        else p += n;
    }
};

size_t width_of(uint32_t vt) {
    switch (vt) {
        case 0: case 1: case 7: return 1;
        case 2: case 3: return 2;
        case 4: case 5: case 6: return 4;
        case 10: case 11: case 12: return 8;
        default: return 0;
    }
}

bool read_scalar(Reader& r, uint32_t vt, Value* out) {
    switch (vt) {
        case 0: *out = (uint64_t)r.take<uint8_t>(); return r.ok;
        case 1: *out = (int64_t)r.take<int8_t>(); return r.ok;
        case 2: *out = (uint64_t)r.take<uint16_t>(); return r.ok;
        case 3: *out = (int64_t)r.take<int16_t>(); return r.ok;
        case 4: *out = (uint64_t)r.take<uint32_t>(); return r.ok;
        case 5: *out = (int64_t)r.take<int32_t>(); return r.ok;
        case 6: *out = (double)r.take<float>(); return r.ok;
        case 7: *out = r.take<uint8_t>() != 0; return r.ok;
        case 8: *out = r.str(); return r.ok;
        case 10: *out = r.take<uint64_t>(); return r.ok;
        case 11: *out = r.take<int64_t>(); return r.ok;
        case 12: *out = r.take<double>(); return r.ok;
        default: return false;
    }
}
}  // namespace

File::~File() {
    if (base_) munmap((void*)base_, size_);
    if (fd_ >= 0) close(fd_);
}

bool File::open(const std::string& path, std::string* err) {
    auto bad = [&](const std::string& m) {
        if (err) *err = path + ": " + m;
        return false;
    };
    fd_ = ::open(path.c_str(), O_RDONLY);
    if (fd_ < 0) return bad("cannot open");
    struct stat st;
    if (fstat(fd_, &st) != 0) return bad("cannot stat");
    size_ = (size_t)st.st_size;
    if (size_ < 24) return bad("too short to be a GGUF file");
    void* m = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
    if (m == MAP_FAILED) return bad("mmap failed");
    base_ = (const uint8_t*)m;
    Reader r{base_, base_ + size_};
    if (memcmp(r.p, "GGUF", 4) != 0) return bad("bad magic");
    r.p += 4;
    uint32_t version = r.take<uint32_t>();
    if (version != 3) return bad("unsupported GGUF version " + std::to_string(version));
    int64_t n_tensors = r.take<int64_t>();
    int64_t n_kv = r.take<int64_t>();
    if (n_tensors < 0 || n_kv < 0) return bad("negative counts");
    for (int64_t i = 0; i < n_kv; i++) {
        std::string key = r.str();
        uint32_t vt = r.take<uint32_t>();
        if (!r.ok) return bad("truncated metadata");
        if (vt == 9) {
            uint32_t et = r.take<uint32_t>();
            uint64_t n = r.take<uint64_t>();
            if (et == 5) {
                std::vector<int32_t> v;
                if (n > (uint64_t)(r.end - r.p) / 4) return bad("array longer than the file at " + key);
                for (uint64_t k = 0; k < n && r.ok; k++) v.push_back(r.take<int32_t>());
                meta_[key] = std::move(v);
            } else if (et == 8) {
                for (uint64_t k = 0; k < n && r.ok; k++) r.str();
            } else {
                size_t w = width_of(et);
                if (w == 0) return bad("unknown array element type at " + key);
                uint64_t bytes = 0;
                if (__builtin_mul_overflow((uint64_t)w, n, &bytes)) return bad("array length overflows at " + key);
                r.skip(bytes);
            }
        } else {
            Value v;
            if (!read_scalar(r, vt, &v)) return bad("unknown value type at " + key);
            meta_[key] = std::move(v);
        }
        if (!r.ok) return bad("truncated metadata at " + key);
    }
    for (int64_t i = 0; i < n_tensors; i++) {
        Tensor t;
        t.name = r.str();
        uint32_t nd = r.take<uint32_t>();
        if (!r.ok || nd > 4) return bad("bad tensor entry");
        for (uint32_t d = 0; d < nd; d++) t.dims.push_back((uint64_t)r.take<int64_t>());
        t.ty = r.take<uint32_t>();
        t.offset = r.take<uint64_t>();
        if (!r.ok) return bad("truncated tensor table");
        if (by_name_.count(t.name)) return bad("duplicate tensor " + t.name);
        by_name_[t.name] = tensors_.size();
        tensors_.push_back(std::move(t));
    }
    uint64_t align = 32;
    get_uint("general.alignment", &align);
    if (align == 0) return bad("zero alignment");
    if (align > (1ull << 30)) return bad("implausible alignment");
    const uint64_t pos = (uint64_t)(r.p - base_);
    uint64_t start = 0;
    if (__builtin_add_overflow(pos, align - 1, &start)) return bad("header end overflows");
    start = start / align * align;
    if (start > size_) return bad("the data blob starts past the end of the file");
    data_start_ = (size_t)start;
    const uint64_t blob = size_ - data_start_;
    // Every size below comes from the file: each product and sum is checked, so that a huge dimension or offset
    // cannot wrap round into a small number that passes the bounds test and later indexes outside the mapping.
    for (const Tensor& t : tensors_) {
        uint64_t n = 0, nb = 0;
        if (!t.n_elems_checked(&n)) return bad("tensor " + t.name + ": element count overflows");
        if (!type_bytes_checked(t.ty, n, &nb)) return bad("tensor " + t.name + ": byte size overflows");
        if (nb == 0 && n != 0) return bad("tensor " + t.name + " has an unsupported type or partial blocks");
        if (t.dims.empty() || (t.ty == 8 && t.dims[0] % 32) || (t.ty == 40 && t.dims[0] % 64))
            return bad("tensor " + t.name + ": row length is not a whole number of blocks");
        if (t.offset % align) return bad("tensor " + t.name + " is misaligned");
        if (t.offset > blob || nb > blob - t.offset) return bad("tensor " + t.name + " runs past the end of the file");
    }
    return true;
}

const Tensor* File::tensor(const std::string& name) const {
    auto it = by_name_.find(name);
    return it == by_name_.end() ? nullptr : &tensors_[it->second];
}

bool File::get_uint(const std::string& key, uint64_t* out) const {
    auto it = meta_.find(key);
    if (it == meta_.end()) return false;
    if (auto u = std::get_if<uint64_t>(&it->second)) {
        *out = *u;
        return true;
    }
    return false;
}
bool File::get_float(const std::string& key, float* out) const {
    auto it = meta_.find(key);
    if (it == meta_.end()) return false;
    if (auto d = std::get_if<double>(&it->second)) {
        *out = (float)*d;
        return true;
    }
    return false;
}
bool File::get_string(const std::string& key, std::string* out) const {
    auto it = meta_.find(key);
    if (it == meta_.end()) return false;
    if (auto s = std::get_if<std::string>(&it->second)) {
        *out = *s;
        return true;
    }
    return false;
}
const std::vector<int32_t>* File::get_i32_array(const std::string& key) const {
    auto it = meta_.find(key);
    if (it == meta_.end()) return nullptr;
    return std::get_if<std::vector<int32_t>>(&it->second);
}

}  // namespace itg
