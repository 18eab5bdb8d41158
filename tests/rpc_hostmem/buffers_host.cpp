// Host-memory stand-in for the RPC server's HBM buffers, so that the protocol tests run on a machine without a GPU.
// Test infrastructure only: the product binary links mesh-llm_amd/csrc/rpc/rpc_buffers_hip.cpp instead.

#include <cstdlib>
#include <cstring>

#include "rpc_buffers.hpp"

namespace mesh_rpc {

namespace {

class HostBuffers final : public BufferBackend {
  public:
    int device_count() override { return 2; }                      // two, so that device indices are exercised
    std::string device_name(int dev) override { return "ROCm" + std::to_string(dev); }
    std::string device_description(int) override { return "host memory stand-in"; }
    bool device_memory(int, uint64_t *free_bytes, uint64_t *total_bytes) override {
        *total_bytes = (uint64_t)8 << 30;
        *free_bytes = *total_bytes - used_;
        return true;
    }
    uint64_t alignment() override { return 256; }
    uint64_t max_size(int) override { return (uint64_t)8 << 30; }
    void *alloc(int, uint64_t size) override {
        if (size > ((uint64_t)1 << 30)) return nullptr;             // "out of memory" for the failure test
        void *p = nullptr;
        if (posix_memalign(&p, 256, size ? size : 1) != 0) return nullptr;
        memset(p, 0xCD, size);
        used_ += size;
        return p;
    }
    void release(int, void *base) override { free(base); }
    bool upload(int, void *dst, const void *src, uint64_t n) override { memcpy(dst, src, n); return true; }
    bool download(int, void *dst, const void *src, uint64_t n) override { memcpy(dst, src, n); return true; }
    bool fill(int, void *dst, uint8_t v, uint64_t n) override { memset(dst, v, n); return true; }
    bool copy(int, void *dst, const void *src, uint64_t n) override { memmove(dst, src, n); return true; }

  private:
    uint64_t used_ = 0;
};

}  // namespace

BufferBackend *buffer_backend() {
    static HostBuffers b;
    return &b;
}

}  // namespace mesh_rpc
