// Just enough protobuf wire format for the plugin protocol's envelopes: varints, length-delimited fields, and a reader
// that walks a message's fields.  Message and field numbers are those of mesh-llm/proto/plugin.proto (package
// meshllm.plugin.v1); plugin_main.cpp names the ones it uses.
#pragma once

#include <cstdint>
#include <string>

namespace mesh_plugin {

class PbWriter {
  public:
    void varint(uint64_t v) {
        while (v >= 0x80) {
            out_.push_back((char)((v & 0x7F) | 0x80));
            v >>= 7;
        }
        out_.push_back((char)v);
    }
    void tag(uint32_t field, uint32_t wire) { varint(((uint64_t)field << 3) | wire); }
    // proto3 scalars: zero / empty values are not written
    void u64(uint32_t field, uint64_t v) { if (v) { tag(field, 0); varint(v); } }
    void boolean(uint32_t field, bool v) { if (v) { tag(field, 0); varint(1); } }
    void str(uint32_t field, const std::string &v) { if (!v.empty()) bytes(field, v); }
    // sub-messages and `optional` fields: written even when empty
    void bytes(uint32_t field, const std::string &v) {
        tag(field, 2);
        varint(v.size());
        out_.append(v);
    }
    const std::string &data() const { return out_; }

  private:
    std::string out_;
};

// Iterates the fields of one message.  next() returns false at the end or on malformed input (ok() tells which).
class PbReader {
  public:
    PbReader(const char *p, size_t n) : p_(p), end_(p + n) {}
    explicit PbReader(const std::string &s) : PbReader(s.data(), s.size()) {}
    bool next() {
        if (p_ >= end_) return false;
        uint64_t key;
        if (!varint(&key)) return fail();
        field = (uint32_t)(key >> 3);
        wire = (uint32_t)(key & 7);
        switch (wire) {
            case 0: return varint(&value) || fail();
            case 1: return skip(8) || fail();
            case 5: return skip(4) || fail();
            case 2: {
                uint64_t n;
                if (!varint(&n) || n > (uint64_t)(end_ - p_)) return fail();
                chunk.assign(p_, (size_t)n);
                p_ += n;
                return true;
            }
            default: return fail();
        }
    }
    bool ok() const { return ok_; }
    uint32_t field = 0, wire = 0;
    uint64_t value = 0;        // wire type 0
    std::string chunk;         // wire type 2

  private:
    bool varint(uint64_t *out) {
        uint64_t v = 0;
        for (int shift = 0; shift < 64 && p_ < end_; shift += 7) {
            const uint8_t b = (uint8_t)*p_++;
            v |= (uint64_t)(b & 0x7F) << shift;
            if (!(b & 0x80)) {
                *out = v;
                return true;
            }
        }
        return false;
    }
    bool skip(size_t n) {
        if ((size_t)(end_ - p_) < n) return false;
        p_ += n;
        return true;
    }
    bool fail() {
        ok_ = false;
        p_ = end_;
        return false;
    }
    const char *p_, *end_;
    bool ok_ = true;
};

}  // namespace mesh_plugin
