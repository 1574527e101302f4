// GGUF v3 container: a reader over an mmap (or an owned buffer) and a writer.
//
// Mirrors cera's format layer: the reader follows GgufFile::from_backing
// (cera/src/gguf.rs:409-568: magic, version 3 only, KV table, tensor infos,
// data section aligned to `general.alignment` (default 32), tensor offsets
// relative to it), the typed getters (:578-672) accept exactly one value type
// each, and the writer follows GgufWriter::write_header_and_tensor_info /
// write_tensor_data (cera/src/convert/writer.rs:205-276).
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <optional>
#include <string>
#include <utility>
#include <vector>

namespace cera {

// metadata value type ids, cera/src/gguf.rs:20-33
enum GgufValueType : uint32_t {
    GGUF_U8 = 0, GGUF_I8 = 1, GGUF_U16 = 2, GGUF_I16 = 3, GGUF_U32 = 4, GGUF_I32 = 5, GGUF_F32 = 6,
    GGUF_BOOL = 7, GGUF_STRING = 8, GGUF_ARRAY = 9, GGUF_U64 = 10, GGUF_I64 = 11, GGUF_F64 = 12
};

struct GgufValue {
    uint32_t type = GGUF_U32;
    uint64_t u = 0;   // unsigned integers and bool
    int64_t i = 0;    // signed integers
    double f = 0.0;   // f32 / f64
    std::string s;
    uint32_t elem_type = GGUF_U32;  // arrays only
    std::vector<GgufValue> arr;

    static GgufValue u32(uint32_t v) { GgufValue g; g.type = GGUF_U32; g.u = v; return g; }
    static GgufValue f32(float v) { GgufValue g; g.type = GGUF_F32; g.f = v; return g; }
    static GgufValue str(std::string v) { GgufValue g; g.type = GGUF_STRING; g.s = std::move(v); return g; }
    static GgufValue boolean(bool v) { GgufValue g; g.type = GGUF_BOOL; g.u = v; return g; }
};

struct TensorInfo {
    std::string name;
    std::vector<uint64_t> shape;  // GGUF order: shape[0] is the inner (row) dimension
    uint32_t ggml_type = 0;
    uint64_t offset = 0;      // absolute offset in the file
    uint64_t size_bytes = 0;  // 0: a type this build cannot size (listed, not loadable)
};

class GgufFile {
public:
    // nullptr + *err on any malformed input; never throws.
    static std::unique_ptr<GgufFile> open(const std::string& path, std::string* err);
    static std::unique_ptr<GgufFile> from_bytes(std::vector<uint8_t> bytes, std::string* err);
    ~GgufFile();
    GgufFile(const GgufFile&) = delete;
    GgufFile& operator=(const GgufFile&) = delete;

    std::optional<uint32_t> get_u32(const std::string& key) const;
    std::optional<float> get_f32(const std::string& key) const;
    std::optional<std::string> get_str(const std::string& key) const;
    std::optional<bool> get_bool(const std::string& key) const;

    const TensorInfo* tensor(const std::string& name) const;
    // pointer into the mapping; nullptr if the tensor is absent or unsizable
    const uint8_t* tensor_data(const TensorInfo& t) const { return t.size_bytes ? data_ + t.offset : nullptr; }
    // F32 / F16 / BF16 tensors as f32 (norm weights, biases, rope_freqs); false + *err otherwise
    bool tensor_to_f32(const std::string& name, std::vector<float>* out, std::string* err) const;

    const std::map<std::string, GgufValue>& metadata() const { return metadata_; }
    const std::map<std::string, TensorInfo>& tensors() const { return tensors_; }
    uint64_t data_offset() const { return data_offset_; }
    uint64_t file_size() const { return size_; }

private:
    GgufFile() = default;
    bool parse(std::string* err);
    std::map<std::string, GgufValue> metadata_;
    std::map<std::string, TensorInfo> tensors_;
    const uint8_t* data_ = nullptr;
    uint64_t size_ = 0;
    uint64_t data_offset_ = 0;
    bool mapped_ = false;
    std::vector<uint8_t> owned_;
};

// Resolved weight: cera/src/model/transformer.rs:127-139 (WeightRef) and
// :187-231 (resolve_weight): k = shape[0] (row length), m = shape[1] or 1.
struct WeightRef {
    uint64_t start = 0, size = 0;
    uint32_t ggml_type = 0;
    uint64_t m = 0, k = 0;
};
bool resolve_weight(const GgufFile& g, const std::string& name, WeightRef* out, std::string* err);

class GgufWriter {
public:
    explicit GgufWriter(uint32_t alignment = 32) : alignment_(alignment) {}
    void add_metadata(const std::string& key, GgufValue v) { metadata_.emplace_back(key, std::move(v)); }
    // Registers a tensor; its offset (relative to the data section) is the running
    // aligned total, like GgufWriter::add_tensor_info (writer.rs:170-203).
    // Returns the tensor's index.  `dims` in GGUF order (inner dimension first).
    size_t add_tensor(const std::string& name, const std::vector<uint64_t>& dims, uint32_t ggml_type,
                      uint64_t size_bytes);
    // Header + KV + tensor table + padding to the data boundary.
    std::vector<uint8_t> header_bytes() const;
    // Whole file into `path`: header, then each tensor's payload from `payload(i)`
    // (must return size_bytes bytes) followed by its alignment padding.
    template <class F>
    bool write_file(const std::string& path, F&& payload, std::string* err) const;
    uint64_t tensor_size(size_t i) const { return tensors_[i].size_bytes; }
    size_t n_tensors() const { return tensors_.size(); }
    uint32_t alignment() const { return alignment_; }

private:
    bool write_all(int fd, const void* p, uint64_t n, std::string* err) const;
    int open_out(const std::string& path, std::string* err) const;
    void close_out(int fd) const;
    struct Meta { std::string name; std::vector<uint64_t> dims; uint32_t ggml_type; uint64_t offset, size_bytes; };
    uint32_t alignment_;
    uint64_t next_offset_ = 0;
    std::vector<std::pair<std::string, GgufValue>> metadata_;
    std::vector<Meta> tensors_;
};

template <class F>
bool GgufWriter::write_file(const std::string& path, F&& payload, std::string* err) const {
    int fd = open_out(path, err);
    if (fd < 0) return false;
    std::vector<uint8_t> head = header_bytes();
    bool ok = write_all(fd, head.data(), head.size(), err);
    static const uint8_t zeros[4096] = {0};
    for (size_t i = 0; ok && i < tensors_.size(); ++i) {
        const void* p = payload(i);
        ok = p != nullptr && write_all(fd, p, tensors_[i].size_bytes, err);
        uint64_t rem = tensors_[i].size_bytes % alignment_;
        uint64_t pad = rem ? alignment_ - rem : 0;
        while (ok && pad) {
            uint64_t n = pad < sizeof(zeros) ? pad : sizeof(zeros);
            ok = write_all(fd, zeros, n, err);
            pad -= n;
        }
        if (!p && err) *err = "no payload for tensor " + tensors_[i].name;
    }
    close_out(fd);
    return ok;
}

}  // namespace cera
