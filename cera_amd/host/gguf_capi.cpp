// C face of the GGUF reader / writer for callers without C++ (the ctypes tests).
#include <algorithm>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "cera_host.h"
#include "gguf.h"

struct cera_gguf {
    std::unique_ptr<cera::GgufFile> file;
    std::vector<const std::string*> names;  // sorted (map order)
};

struct cera_gguf_writer {
    cera::GgufWriter w;
    std::vector<const void*> data;
    explicit cera_gguf_writer(uint32_t a) : w(a) {}
};

namespace {
void set_err(char* err, uint64_t n, const std::string& m) {
    if (!err || !n) return;
    std::strncpy(err, m.c_str(), n - 1);
    err[n - 1] = 0;
}
cera_gguf* wrap(std::unique_ptr<cera::GgufFile> f) {
    if (!f) return nullptr;
    cera_gguf* g = new cera_gguf();
    g->file = std::move(f);
    for (const auto& kv : g->file->tensors()) g->names.push_back(&kv.first);
    return g;
}
}  // namespace

extern "C" {

cera_gguf* cera_gguf_open(const char* path, char* err, uint64_t err_len) {
    if (!path) { set_err(err, err_len, "null path"); return nullptr; }
    std::string e;
    cera_gguf* g = wrap(cera::GgufFile::open(path, &e));
    if (!g) set_err(err, err_len, e);
    return g;
}
cera_gguf* cera_gguf_from_bytes(const void* bytes, uint64_t n, char* err, uint64_t err_len) {
    std::string e;
    const uint8_t* b = static_cast<const uint8_t*>(bytes);
    cera_gguf* g = wrap(cera::GgufFile::from_bytes(std::vector<uint8_t>(b, b + (b ? n : 0)), &e));
    if (!g) set_err(err, err_len, e);
    return g;
}
void cera_gguf_close(cera_gguf* g) { delete g; }

int cera_gguf_get_u32(const cera_gguf* g, const char* key, uint32_t* out) {
    auto v = g->file->get_u32(key);
    if (v && out) *out = *v;
    return v ? 1 : 0;
}
int cera_gguf_get_f32(const cera_gguf* g, const char* key, float* out) {
    auto v = g->file->get_f32(key);
    if (v && out) *out = *v;
    return v ? 1 : 0;
}
int64_t cera_gguf_get_str(const cera_gguf* g, const char* key, char* out, uint64_t out_len) {
    auto v = g->file->get_str(key);
    if (!v) return -1;
    if (out && out_len) {
        uint64_t n = std::min<uint64_t>(out_len - 1, v->size());
        std::memcpy(out, v->data(), n);
        out[n] = 0;
    }
    return static_cast<int64_t>(v->size());
}
uint64_t cera_gguf_data_offset(const cera_gguf* g) { return g->file->data_offset(); }
uint64_t cera_gguf_n_tensors(const cera_gguf* g) { return g->names.size(); }
const char* cera_gguf_tensor_name(const cera_gguf* g, uint64_t i) {
    return i < g->names.size() ? g->names[i]->c_str() : nullptr;
}
int cera_gguf_tensor(const cera_gguf* g, const char* name, cera_gguf_tensor_info* out) {
    const cera::TensorInfo* t = g->file->tensor(name);
    if (!t) return 0;
    if (out) {
        std::memset(out, 0, sizeof *out);
        out->ggml_type = t->ggml_type;
        out->n_dims = static_cast<uint32_t>(t->shape.size());
        for (size_t i = 0; i < t->shape.size() && i < 8; ++i) out->dims[i] = t->shape[i];
        out->offset = t->offset;
        out->size_bytes = t->size_bytes;
        out->data = g->file->tensor_data(*t);
    }
    return 1;
}

cera_gguf_writer* cera_gguf_writer_new(uint32_t alignment) {
    return alignment ? new cera_gguf_writer(alignment) : nullptr;
}
void cera_gguf_writer_free(cera_gguf_writer* w) { delete w; }
void cera_gguf_writer_add_u32(cera_gguf_writer* w, const char* key, uint32_t v) {
    w->w.add_metadata(key, cera::GgufValue::u32(v));
}
void cera_gguf_writer_add_f32(cera_gguf_writer* w, const char* key, float v) {
    w->w.add_metadata(key, cera::GgufValue::f32(v));
}
void cera_gguf_writer_add_str(cera_gguf_writer* w, const char* key, const char* v) {
    w->w.add_metadata(key, cera::GgufValue::str(v ? v : ""));
}
void cera_gguf_writer_add_tensor(cera_gguf_writer* w, const char* name, const uint64_t* dims, uint32_t n_dims,
                                 uint32_t ggml_type, const void* data, uint64_t size_bytes) {
    w->w.add_tensor(name, std::vector<uint64_t>(dims, dims + n_dims), ggml_type, size_bytes);
    w->data.push_back(data);
}
int cera_gguf_writer_write(cera_gguf_writer* w, const char* path, char* err, uint64_t err_len) {
    std::string e;
    static const uint8_t empty = 0;
    bool ok = w->w.write_file(
        path, [&](size_t i) -> const void* { return w->w.tensor_size(i) ? w->data[i] : &empty; }, &e);
    if (!ok) set_err(err, err_len, e);
    return ok ? 0 : -1;
}

}  // extern "C"
