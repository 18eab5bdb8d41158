// HBM buffers of the RPC server: hipMalloc / hipMemcpy on the GPU the buffer was allocated on.

#include <hip/hip_runtime.h>

#include <cstdio>

#include "rpc_buffers.hpp"

namespace mesh_rpc {

namespace {

class HipBuffers final : public BufferBackend {
  public:
    int device_count() override {
        int n = 0;
        return hipGetDeviceCount(&n) == hipSuccess ? n : 0;
    }
    std::string device_name(int dev) override { return "ROCm" + std::to_string(dev); }
    std::string device_description(int dev) override {
        hipDeviceProp_t p;
        if (hipGetDeviceProperties(&p, dev) != hipSuccess) return "unknown";
        return p.name;
    }
    bool device_memory(int dev, uint64_t *free_bytes, uint64_t *total_bytes) override {
        size_t f = 0, t = 0;
        if (!use(dev) || hipMemGetInfo(&f, &t) != hipSuccess) return false;
        *free_bytes = f;
        *total_bytes = t;
        return true;
    }
    uint64_t alignment() override { return 256; }          // hipMalloc returns at least this; tensors inside a buffer start on it
    uint64_t max_size(int dev) override {
        hipDeviceProp_t p;
        return hipGetDeviceProperties(&p, dev) == hipSuccess ? (uint64_t)p.totalGlobalMem : 0;
    }
    void *alloc(int dev, uint64_t size) override {
        void *p = nullptr;
        if (!use(dev) || hipMalloc(&p, size ? size : 1) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        return p;
    }
    void release(int dev, void *base) override {
        if (use(dev)) (void)hipFree(base);
    }
    bool upload(int dev, void *dst, const void *host_src, uint64_t size) override {
        return use(dev) && hipMemcpy(dst, host_src, size, hipMemcpyHostToDevice) == hipSuccess;
    }
    bool download(int dev, void *host_dst, const void *src, uint64_t size) override {
        return use(dev) && hipMemcpy(host_dst, src, size, hipMemcpyDeviceToHost) == hipSuccess;
    }
    bool fill(int dev, void *dst, uint8_t value, uint64_t size) override {
        return use(dev) && hipMemset(dst, value, size) == hipSuccess && hipDeviceSynchronize() == hipSuccess;
    }
    bool copy(int dev, void *dst, const void *src, uint64_t size) override {
        return use(dev) && hipMemcpy(dst, src, size, hipMemcpyDeviceToDevice) == hipSuccess;
    }

  private:
    static bool use(int dev) { return hipSetDevice(dev) == hipSuccess; }    // the current device is per thread
};

}  // namespace

BufferBackend *buffer_backend() {
    static HipBuffers b;
    return &b;
}

}  // namespace mesh_rpc
