// See gguf.hpp.  Host-only; parses from the read-only mapping with explicit bounds on every read.

#include "gguf.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstring>

#include "mesh_common.hpp"

namespace mesh {

namespace {

constexpr uint64_t MAX_STRING_BYTES = 1000000;
constexpr uint64_t MAX_ARRAY_ELEMENTS = 1000000;
constexpr uint32_t MAX_ARRAY_DEPTH = 64;
constexpr uint32_t MAX_TENSOR_DIMS = 8;
constexpr int64_t MAX_KV_COUNT = 1000000;
constexpr int64_t MAX_TENSOR_COUNT = 1000000;

enum : uint32_t { T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64, T_COUNT };

struct Cursor {
    const uint8_t *p;
    uint64_t size;
    uint64_t pos = 0;
    const char *err = nullptr;

    bool need(uint64_t n) {
        if (err) return false;
        if (n > size - pos) { err = "unexpected end of file"; return false; }
        return true;
    }
    template <typename T> T rd() {
        T v{};
        if (need(sizeof(T))) { memcpy(&v, p + pos, sizeof(T)); pos += sizeof(T); }
        return v;
    }
    std::string str() {
        const uint64_t n = rd<uint64_t>();
        if (err) return {};
        if (n > MAX_STRING_BYTES) { err = "string too long"; return {}; }
        if (!need(n)) return {};
        std::string s(reinterpret_cast<const char *>(p + pos), (size_t)n);
        pos += n;
        return s;
    }
};

size_t fixed_size(uint32_t t) {
    switch (t) {
        case T_U8: case T_I8: case T_BOOL: return 1;
        case T_U16: case T_I16: return 2;
        case T_U32: case T_I32: case T_F32: return 4;
        case T_U64: case T_I64: case T_F64: return 8;
        default: return 0;
    }
}

void skip_value(Cursor &c, uint32_t type, uint32_t depth) {
    if (c.err) return;
    if (type >= T_COUNT) { c.err = "unknown value type"; return; }
    if (type == T_STR) { (void)c.str(); return; }
    if (type == T_ARR) {
        if (depth >= MAX_ARRAY_DEPTH) { c.err = "array nesting too deep"; return; }
        const uint32_t et = c.rd<uint32_t>();
        const uint64_t n = c.rd<uint64_t>();
        if (c.err) return;
        if (et >= T_COUNT) { c.err = "unknown array element type"; return; }
        if (n > MAX_ARRAY_ELEMENTS) { c.err = "array too long"; return; }
        const size_t fs = fixed_size(et);
        if (fs) { if (c.need(fs * n)) c.pos += fs * n; return; }
        for (uint64_t i = 0; i < n && !c.err; ++i) skip_value(c, et, depth + 1);
        return;
    }
    const size_t fs = fixed_size(type);
    if (c.need(fs)) c.pos += fs;
}

GgufValue read_scalar(Cursor &c, uint32_t type) {
    GgufValue v;
    switch (type) {
        case T_U8: v.kind = GgufValue::UINT; v.u = c.rd<uint8_t>(); break;
        case T_U16: v.kind = GgufValue::UINT; v.u = c.rd<uint16_t>(); break;
        case T_U32: v.kind = GgufValue::UINT; v.u = c.rd<uint32_t>(); break;
        case T_U64: v.kind = GgufValue::UINT; v.u = c.rd<uint64_t>(); break;
        case T_I8: v.kind = GgufValue::INT; v.i = c.rd<int8_t>(); break;
        case T_I16: v.kind = GgufValue::INT; v.i = c.rd<int16_t>(); break;
        case T_I32: v.kind = GgufValue::INT; v.i = c.rd<int32_t>(); break;
        case T_I64: v.kind = GgufValue::INT; v.i = c.rd<int64_t>(); break;
        case T_F32: v.kind = GgufValue::FLOAT; v.f = c.rd<float>(); break;
        case T_F64: v.kind = GgufValue::FLOAT; v.f = c.rd<double>(); break;
        case T_BOOL: v.kind = GgufValue::BOOL; v.u = c.rd<uint8_t>() != 0; break;
        case T_STR: v.kind = GgufValue::STRING; v.s = c.str(); break;
        default: skip_value(c, type, 0); break;
    }
    return v;
}

}  // namespace

GgufFile::~GgufFile() {
    if (map_) munmap(const_cast<uint8_t *>(map_), size_);
    if (fd_ >= 0) close(fd_);
}

int GgufFile::open(const char *path) {
    if (!path) return fail(MESH_ERR_INVALID, "gguf: null path");
    fd_ = ::open(path, O_RDONLY | O_CLOEXEC);
    if (fd_ < 0) return fail(MESH_ERR_IO, "gguf: cannot open '%s': %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd_, &st) != 0) return fail(MESH_ERR_IO, "gguf: fstat('%s') failed: %s", path, strerror(errno));
    size_ = (uint64_t)st.st_size;
    if (size_ < 24) return fail(MESH_ERR_FORMAT, "gguf: '%s' is too short to be a GGUF file", path);
    void *m = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
    if (m == MAP_FAILED) return fail(MESH_ERR_IO, "gguf: mmap('%s') failed: %s", path, strerror(errno));
    map_ = static_cast<const uint8_t *>(m);

    Cursor c{map_, size_};
    if (memcmp(map_, "GGUF", 4) != 0) return fail(MESH_ERR_FORMAT, "gguf: '%s' has no GGUF magic", path);
    c.pos = 4;
    version_ = c.rd<uint32_t>();
    if (version_ < 2) return fail(MESH_ERR_FORMAT, "gguf: version %u is not supported (need >= 2)", version_);
    const int64_t n_tensors = c.rd<int64_t>();
    const int64_t n_kv = c.rd<int64_t>();
    if (n_tensors < 0 || n_tensors > MAX_TENSOR_COUNT) return fail(MESH_ERR_FORMAT, "gguf: tensor count %lld out of range", (long long)n_tensors);
    if (n_kv < 0 || n_kv > MAX_KV_COUNT) return fail(MESH_ERR_FORMAT, "gguf: KV count %lld out of range", (long long)n_kv);

    for (int64_t i = 0; i < n_kv; ++i) {
        std::string key = c.str();
        const uint32_t type = c.rd<uint32_t>();
        if (c.err) break;
        if (type >= T_COUNT) { c.err = "unknown value type"; break; }
        GgufValue v = read_scalar(c, type);
        if (c.err) break;
        if (v.kind != GgufValue::NONE) kv_[key] = std::move(v);
    }
    if (c.err) return fail(MESH_ERR_FORMAT, "gguf: bad key/value table in '%s': %s", path, c.err);

    uint32_t al = 32;
    if (get_u32("general.alignment", al)) alignment_ = al ? al : 1;

    tensors_.reserve((size_t)n_tensors);
    for (int64_t i = 0; i < n_tensors; ++i) {
        GgufTensorInfo t;
        t.name = c.str();
        t.n_dims = c.rd<uint32_t>();
        if (c.err) break;
        if (t.n_dims > MAX_TENSOR_DIMS) { c.err = "too many tensor dimensions"; break; }
        uint64_t nelem = 1;
        bool overflow = false;
        for (uint32_t d = 0; d < t.n_dims; ++d) {
            const uint64_t ne = c.rd<uint64_t>();
            if (d < 4) t.ne[d] = ne;
            else if (ne != 1) overflow = true;      // this build handles at most 4 real dimensions
            if (ne != 0 && nelem > UINT64_MAX / ne) overflow = true;
            else nelem *= ne;
        }
        t.type = c.rd<uint32_t>();
        t.offset = c.rd<uint64_t>();
        if (c.err) break;
        const int64_t be = block_elems((int)t.type);
        if (!overflow && be > 0 && t.ne[0] % (uint64_t)be == 0) {
            const uint64_t blocks = nelem / (uint64_t)be;
            const uint64_t bb = (uint64_t)block_bytes((int)t.type);
            if (blocks <= UINT64_MAX / bb) t.nbytes = blocks * bb;
        }
        index_[t.name] = tensors_.size();
        tensors_.push_back(std::move(t));
    }
    if (c.err) return fail(MESH_ERR_FORMAT, "gguf: bad tensor directory in '%s': %s", path, c.err);

    const uint64_t a = alignment_;
    data_offset_ = c.pos % a ? c.pos + (a - c.pos % a) : c.pos;
    return MESH_OK;
}

const GgufTensorInfo *GgufFile::find(const std::string &name) const {
    auto it = index_.find(name);
    return it == index_.end() ? nullptr : &tensors_[it->second];
}

const uint8_t *GgufFile::data(const GgufTensorInfo &t) const {
    if (t.nbytes == 0 || data_offset_ > size_) return nullptr;
    const uint64_t avail = size_ - data_offset_;
    if (t.offset > avail || t.nbytes > avail - t.offset) return nullptr;
    return map_ + data_offset_ + t.offset;
}

bool GgufFile::get_u32(const std::string &key, uint32_t &out) const {
    auto it = kv_.find(key);
    if (it == kv_.end()) return false;
    const GgufValue &v = it->second;
    if (v.kind == GgufValue::UINT || v.kind == GgufValue::BOOL) {
        if (v.u > UINT32_MAX) return false;
        out = (uint32_t)v.u;
        return true;
    }
    if (v.kind == GgufValue::INT) {
        if (v.i < 0 || v.i > (int64_t)UINT32_MAX) return false;   // negative where unsigned expected
        out = (uint32_t)v.i;
        return true;
    }
    return false;
}

bool GgufFile::get_f32(const std::string &key, float &out) const {
    auto it = kv_.find(key);
    if (it == kv_.end()) return false;
    const GgufValue &v = it->second;
    if (v.kind == GgufValue::FLOAT) { out = (float)v.f; return true; }
    if (v.kind == GgufValue::UINT) { out = (float)v.u; return true; }
    if (v.kind == GgufValue::INT) { out = (float)v.i; return true; }
    return false;
}

bool GgufFile::get_str(const std::string &key, std::string &out) const {
    auto it = kv_.find(key);
    if (it == kv_.end() || it->second.kind != GgufValue::STRING) return false;
    out = it->second.s;
    return true;
}

}  // namespace mesh
