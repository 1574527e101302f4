// GGUF v3 reader / writer.  See gguf.h for the reference lines followed.
#include "gguf.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdio>
#include <cstring>

#include "cera_host.h"

namespace cera {
namespace {

constexpr uint32_t GGUF_MAGIC = 0x46554747;  // "GGUF" little-endian, gguf.rs:18

struct Cursor {
    const uint8_t* p;
    uint64_t n, pos = 0;
    bool fail = false;
    std::string why;

    bool take(void* dst, uint64_t len, const char* what) {
        if (fail) return false;
        if (len > n - pos) {
            fail = true;
            why = std::string("unexpected end of file reading ") + what;
            return false;
        }
        std::memcpy(dst, p + pos, len);
        pos += len;
        return true;
    }
    template <class T>
    T num(const char* what) {
        T v{};
        take(&v, sizeof(T), what);
        return v;
    }
    std::string str() {
        uint64_t len = num<uint64_t>("string length");
        if (fail) return {};
        if (len >= 1000000) {  // gguf.rs:221
            fail = true;
            why = "string too long: " + std::to_string(len);
            return {};
        }
        std::string s(len, '\0');
        take(s.data(), len, "string");
        return s;
    }
    GgufValue value(uint32_t type, int depth) {
        GgufValue v;
        v.type = type;
        switch (type) {
            case GGUF_U8: v.u = num<uint8_t>("u8"); break;
            case GGUF_I8: v.i = num<int8_t>("i8"); break;
            case GGUF_U16: v.u = num<uint16_t>("u16"); break;
            case GGUF_I16: v.i = num<int16_t>("i16"); break;
            case GGUF_U32: v.u = num<uint32_t>("u32"); break;
            case GGUF_I32: v.i = num<int32_t>("i32"); break;
            case GGUF_U64: v.u = num<uint64_t>("u64"); break;
            case GGUF_I64: v.i = num<int64_t>("i64"); break;
            case GGUF_F32: v.f = num<float>("f32"); break;
            case GGUF_F64: v.f = num<double>("f64"); break;
            case GGUF_BOOL: v.u = num<uint8_t>("bool") != 0; break;
            case GGUF_STRING: v.s = str(); break;
            case GGUF_ARRAY: {
                v.elem_type = num<uint32_t>("array element type");
                uint64_t count = num<uint64_t>("array length");
                if (fail) break;
                if (depth > 4 || count > n - pos) {  // every element takes at least a byte
                    fail = true;
                    why = "array too long or nested too deep";
                    break;
                }
                v.arr.reserve(count);
                for (uint64_t i = 0; i < count && !fail; ++i) v.arr.push_back(value(v.elem_type, depth + 1));
                break;
            }
            default:
                fail = true;
                why = "unknown GGUF metadata value type " + std::to_string(type);
        }
        return v;
    }
};

// elements per block / bytes per block for the types this backend can size
// (gguf.rs:259-278 maps the same set; everything else is listed with size 0)
bool type_block(uint32_t t, uint64_t* elems, uint64_t* bytes) {
    switch (t) {
        case CERA_TYPE_F32: *elems = 1; *bytes = 4; return true;
        case CERA_TYPE_F16: case CERA_TYPE_BF16: *elems = 1; *bytes = 2; return true;
        case 26 /* I32 */: *elems = 1; *bytes = 4; return true;
        case CERA_TYPE_Q4_0: *elems = 32; *bytes = 18; return true;
        case CERA_TYPE_Q4_1: *elems = 32; *bytes = 20; return true;
        case CERA_TYPE_Q8_0: *elems = 32; *bytes = 34; return true;
        case CERA_TYPE_Q4_K: *elems = 256; *bytes = 144; return true;
        case CERA_TYPE_Q5_K: *elems = 256; *bytes = 176; return true;
        case CERA_TYPE_Q6_K: *elems = 256; *bytes = 210; return true;
        default: return false;
    }
}

bool mul_overflow(uint64_t a, uint64_t b, uint64_t* out) { return __builtin_mul_overflow(a, b, out); }

void put(std::vector<uint8_t>& o, const void* p, size_t n) {
    const uint8_t* b = static_cast<const uint8_t*>(p);
    o.insert(o.end(), b, b + n);
}
template <class T>
void put_num(std::vector<uint8_t>& o, T v) { put(o, &v, sizeof(T)); }
void put_str(std::vector<uint8_t>& o, const std::string& s) {
    put_num<uint64_t>(o, s.size());
    put(o, s.data(), s.size());
}
void put_value(std::vector<uint8_t>& o, const GgufValue& v, bool with_tag) {
    if (with_tag) put_num<uint32_t>(o, v.type);
    switch (v.type) {
        case GGUF_U8: put_num<uint8_t>(o, static_cast<uint8_t>(v.u)); break;
        case GGUF_I8: put_num<int8_t>(o, static_cast<int8_t>(v.i)); break;
        case GGUF_U16: put_num<uint16_t>(o, static_cast<uint16_t>(v.u)); break;
        case GGUF_I16: put_num<int16_t>(o, static_cast<int16_t>(v.i)); break;
        case GGUF_U32: put_num<uint32_t>(o, static_cast<uint32_t>(v.u)); break;
        case GGUF_I32: put_num<int32_t>(o, static_cast<int32_t>(v.i)); break;
        case GGUF_U64: put_num<uint64_t>(o, v.u); break;
        case GGUF_I64: put_num<int64_t>(o, v.i); break;
        case GGUF_F32: put_num<float>(o, static_cast<float>(v.f)); break;
        case GGUF_F64: put_num<double>(o, v.f); break;
        case GGUF_BOOL: put_num<uint8_t>(o, v.u ? 1 : 0); break;
        case GGUF_STRING: put_str(o, v.s); break;
        case GGUF_ARRAY:
            put_num<uint32_t>(o, v.elem_type);
            put_num<uint64_t>(o, v.arr.size());
            for (const GgufValue& e : v.arr) put_value(o, e, false);
            break;
        default: break;
    }
}

}  // namespace

GgufFile::~GgufFile() {
    if (mapped_ && data_) munmap(const_cast<uint8_t*>(data_), size_);
}

std::unique_ptr<GgufFile> GgufFile::open(const std::string& path, std::string* err) {
    auto fail = [&](const std::string& m) {
        if (err) *err = m;
        return std::unique_ptr<GgufFile>();
    };
    int fd = ::open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) return fail("cannot open " + path + ": " + std::strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        ::close(fd);
        return fail("cannot stat " + path + " (or empty file)");
    }
    void* m = mmap(nullptr, static_cast<size_t>(st.st_size), PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (m == MAP_FAILED) return fail("mmap failed for " + path + ": " + std::strerror(errno));
    std::unique_ptr<GgufFile> g(new GgufFile());
    g->data_ = static_cast<const uint8_t*>(m);
    g->size_ = static_cast<uint64_t>(st.st_size);
    g->mapped_ = true;
    if (!g->parse(err)) return nullptr;
    return g;
}

std::unique_ptr<GgufFile> GgufFile::from_bytes(std::vector<uint8_t> bytes, std::string* err) {
    std::unique_ptr<GgufFile> g(new GgufFile());
    g->owned_ = std::move(bytes);
    g->data_ = g->owned_.data();
    g->size_ = g->owned_.size();
    if (!g->parse(err)) return nullptr;
    return g;
}

bool GgufFile::parse(std::string* err) {
    auto fail = [&](const std::string& m) {
        if (err) *err = m;
        return false;
    };
    if (size_ < 24) return fail("GGUF buffer too small (" + std::to_string(size_) + " bytes; need at least 24 for the header)");
    Cursor c{data_, size_};
    uint32_t magic = c.num<uint32_t>("magic");
    if (magic != GGUF_MAGIC) {
        char buf[64];
        std::snprintf(buf, sizeof buf, "not a GGUF file (magic: 0x%08X, expected 0x%08X)", magic, GGUF_MAGIC);
        return fail(buf);
    }
    uint32_t version = c.num<uint32_t>("version");
    if (version != 3) return fail("unsupported GGUF version " + std::to_string(version) + " (expected 3)");
    uint64_t tensor_count = c.num<uint64_t>("tensor count");
    uint64_t kv_count = c.num<uint64_t>("kv count");
    for (uint64_t i = 0; i < kv_count && !c.fail; ++i) {
        std::string key = c.str();
        uint32_t type = c.num<uint32_t>("value type");
        if (c.fail) break;
        GgufValue v = c.value(type, 0);
        if (!c.fail) metadata_[key] = std::move(v);  // a repeated key keeps the last value, like HashMap::insert
    }
    if (c.fail) return fail(c.why);

    struct Raw { std::string name; std::vector<uint64_t> shape; uint32_t type; uint64_t offset; };
    std::vector<Raw> raw;
    for (uint64_t i = 0; i < tensor_count && !c.fail; ++i) {
        Raw r;
        r.name = c.str();
        uint32_t n_dims = c.num<uint32_t>("n_dims");
        if (c.fail) break;
        if (n_dims > 8) return fail("tensor " + r.name + " has too many dimensions: " + std::to_string(n_dims));
        for (uint32_t d = 0; d < n_dims; ++d) r.shape.push_back(c.num<uint64_t>("dimension"));
        r.type = c.num<uint32_t>("tensor type");
        r.offset = c.num<uint64_t>("tensor offset");
        raw.push_back(std::move(r));
    }
    if (c.fail) return fail(c.why);

    uint64_t alignment = 32;
    auto a = metadata_.find("general.alignment");
    if (a != metadata_.end() && a->second.type == GGUF_U32) alignment = a->second.u;
    if (alignment == 0 || alignment > 1024 * 1024) return fail("invalid GGUF alignment: " + std::to_string(alignment));
    uint64_t header_end = c.pos;
    data_offset_ = (header_end + alignment - 1) / alignment * alignment;

    for (Raw& r : raw) {
        TensorInfo t;
        t.name = r.name;
        t.shape = r.shape;
        t.ggml_type = r.type;
        uint64_t elems = 1, bytes = 0, numel = 1;
        if (type_block(r.type, &elems, &bytes)) {
            for (uint64_t d : r.shape)
                if (mul_overflow(numel, d, &numel)) return fail("tensor " + r.name + " numel overflow");
            if (numel % elems)
                return fail("tensor element count " + std::to_string(numel) + " is not divisible by block size " +
                            std::to_string(elems));
            if (mul_overflow(numel / elems, bytes, &t.size_bytes)) return fail("tensor " + r.name + " size overflow");
        }
        if (__builtin_add_overflow(data_offset_, r.offset, &t.offset)) return fail("tensor " + r.name + " offset overflow");
        if (t.size_bytes) {
            uint64_t end;
            if (__builtin_add_overflow(t.offset, t.size_bytes, &end)) return fail("tensor " + r.name + " end offset overflow");
            if (end > size_)
                return fail("tensor " + r.name + " extends beyond file (offset=" + std::to_string(t.offset) +
                            ", size=" + std::to_string(t.size_bytes) + ", file_size=" + std::to_string(size_) + ")");
        }
        tensors_[r.name] = std::move(t);
    }
    return true;
}

std::optional<uint32_t> GgufFile::get_u32(const std::string& key) const {
    auto it = metadata_.find(key);
    if (it == metadata_.end() || it->second.type != GGUF_U32) return std::nullopt;
    return static_cast<uint32_t>(it->second.u);
}
std::optional<float> GgufFile::get_f32(const std::string& key) const {
    auto it = metadata_.find(key);
    if (it == metadata_.end() || it->second.type != GGUF_F32) return std::nullopt;
    return static_cast<float>(it->second.f);
}
std::optional<std::string> GgufFile::get_str(const std::string& key) const {
    auto it = metadata_.find(key);
    if (it == metadata_.end() || it->second.type != GGUF_STRING) return std::nullopt;
    return it->second.s;
}
std::optional<bool> GgufFile::get_bool(const std::string& key) const {
    auto it = metadata_.find(key);
    if (it == metadata_.end() || it->second.type != GGUF_BOOL) return std::nullopt;
    return it->second.u != 0;
}

const TensorInfo* GgufFile::tensor(const std::string& name) const {
    auto it = tensors_.find(name);
    return it == tensors_.end() ? nullptr : &it->second;
}

bool GgufFile::tensor_to_f32(const std::string& name, std::vector<float>* out, std::string* err) const {
    const TensorInfo* t = tensor(name);
    if (!t) {
        if (err) *err = "tensor not found: " + name;
        return false;
    }
    if (!t->size_bytes) {
        if (err) *err = "tensor " + name + " has unsupported GGML type " + std::to_string(t->ggml_type);
        return false;
    }
    const uint8_t* p = data_ + t->offset;
    if (t->ggml_type == CERA_TYPE_F32) {
        out->resize(t->size_bytes / 4);
        std::memcpy(out->data(), p, t->size_bytes);
        return true;
    }
    if (t->ggml_type == CERA_TYPE_F16 || t->ggml_type == CERA_TYPE_BF16) {
        uint64_t n = t->size_bytes / 2;
        out->resize(n);
        for (uint64_t i = 0; i < n; ++i) {
            uint16_t h;
            std::memcpy(&h, p + 2 * i, 2);
            if (t->ggml_type == CERA_TYPE_F16) {
                (*out)[i] = cera_f16_to_f32(h);
            } else {
                uint32_t w = static_cast<uint32_t>(h) << 16;
                std::memcpy(&(*out)[i], &w, 4);
            }
        }
        return true;
    }
    if (err) *err = "tensor " + name + " is quantized (type " + std::to_string(t->ggml_type) + "); an f32/f16/bf16 vector was expected";
    return false;
}

bool resolve_weight(const GgufFile& g, const std::string& name, WeightRef* out, std::string* err) {
    const TensorInfo* t = g.tensor(name);
    if (!t) {
        if (err) *err = "tensor not found: " + name;
        return false;
    }
    if (!t->size_bytes) {
        if (err) *err = "tensor " + name + " has unsupported GGML type " + std::to_string(t->ggml_type) + " -- cannot run this file";
        return false;
    }
    out->start = t->offset;
    out->size = t->size_bytes;
    out->ggml_type = t->ggml_type;
    out->k = t->shape.empty() ? 1 : t->shape[0];
    out->m = t->shape.size() > 1 ? t->shape[1] : 1;
    return true;
}

size_t GgufWriter::add_tensor(const std::string& name, const std::vector<uint64_t>& dims, uint32_t ggml_type,
                              uint64_t size_bytes) {
    uint64_t off = (next_offset_ + alignment_ - 1) / alignment_ * alignment_;
    next_offset_ = off + size_bytes;
    tensors_.push_back(Meta{name, dims, ggml_type, off, size_bytes});
    return tensors_.size() - 1;
}

std::vector<uint8_t> GgufWriter::header_bytes() const {
    std::vector<uint8_t> o;
    put(o, "GGUF", 4);
    put_num<uint32_t>(o, 3);
    put_num<uint64_t>(o, tensors_.size());
    put_num<uint64_t>(o, metadata_.size());
    for (const auto& kv : metadata_) {
        put_str(o, kv.first);
        put_value(o, kv.second, true);
    }
    for (const Meta& t : tensors_) {
        put_str(o, t.name);
        put_num<uint32_t>(o, static_cast<uint32_t>(t.dims.size()));
        for (uint64_t d : t.dims) put_num<uint64_t>(o, d);
        put_num<uint32_t>(o, t.ggml_type);
        put_num<uint64_t>(o, t.offset);
    }
    while (o.size() % alignment_) o.push_back(0);
    return o;
}

int GgufWriter::open_out(const std::string& path, std::string* err) const {
    int fd = ::open(path.c_str(), O_WRONLY | O_CREAT | O_TRUNC | O_CLOEXEC, 0644);
    if (fd < 0 && err) *err = "cannot create " + path + ": " + std::strerror(errno);
    return fd;
}
void GgufWriter::close_out(int fd) const { ::close(fd); }
bool GgufWriter::write_all(int fd, const void* p, uint64_t n, std::string* err) const {
    const uint8_t* b = static_cast<const uint8_t*>(p);
    while (n) {
        ssize_t w = ::write(fd, b, n > (1u << 30) ? (1u << 30) : n);
        if (w < 0) {
            if (errno == EINTR) continue;
            if (err) *err = std::string("write failed: ") + std::strerror(errno);
            return false;
        }
        b += w;
        n -= static_cast<uint64_t>(w);
    }
    return true;
}

}  // namespace cera
