// Bounded GGUF reader: header, key/value table and tensor directory; tensor data is mapped, never copied.
//
// Container rules follow mesh-client/src/models/gguf.rs (magic "GGUF", version >= 2, signed 64-bit
// counts capped at 1e6 :4-9,96-112; value types 0..12 :21-35; strings and arrays length-capped, array
// nesting capped at 64; tensor info = name, n_dims <= 8, u64 dims, u32 type, u64 offset :432-460; data section
// starts at the next multiple of general.alignment, default 32 :422-430,498) and the tensor-by-name lookup of
// rpc_server::set_tensor_gguf (third_party/llama.cpp/patches/0001-rpc-optimize-local-GGUF-tensor-loading.patch:179-266:
// file offset = data offset + tensor offset, whole-tensor read, bounds-checked).
#pragma once

#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace mesh {

struct GgufTensorInfo {
    std::string name;
    uint32_t n_dims = 0;
    uint64_t ne[4] = {1, 1, 1, 1};   // ne[0] is the contiguous (row) dimension
    uint32_t type = 0;               // ggml type id
    uint64_t offset = 0;             // relative to the data section
    uint64_t nbytes = 0;             // ggml_nbytes, 0 if the type is unknown to this build
};

struct GgufValue {
    enum Kind { NONE, UINT, INT, FLOAT, BOOL, STRING } kind = NONE;
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0.0;
    std::string s;
};

class GgufFile {
  public:
    GgufFile() = default;
    ~GgufFile();
    GgufFile(const GgufFile &) = delete;
    GgufFile &operator=(const GgufFile &) = delete;

    // 0 or a negative mesh_status (message in mesh_last_error)
    int open(const char *path);

    uint32_t version() const { return version_; }
    uint32_t alignment() const { return alignment_; }
    uint64_t data_offset() const { return data_offset_; }
    uint64_t file_size() const { return size_; }
    const std::vector<GgufTensorInfo> &tensors() const { return tensors_; }
    const GgufTensorInfo *find(const std::string &name) const;
    // pointer to the tensor's bytes inside the mapping, or nullptr if it would leave the file
    const uint8_t *data(const GgufTensorInfo &t) const;

    bool has(const std::string &key) const { return kv_.count(key) != 0; }
    // scalar lookups; arrays are skipped at parse time and never stored
    bool get_u32(const std::string &key, uint32_t &out) const;
    bool get_f32(const std::string &key, float &out) const;
    bool get_str(const std::string &key, std::string &out) const;

  private:
    int fd_ = -1;
    const uint8_t *map_ = nullptr;
    uint64_t size_ = 0;
    uint32_t version_ = 0;
    uint32_t alignment_ = 32;
    uint64_t data_offset_ = 0;
    std::vector<GgufTensorInfo> tensors_;
    std::map<std::string, size_t> index_;
    std::map<std::string, GgufValue> kv_;
};

}  // namespace mesh
