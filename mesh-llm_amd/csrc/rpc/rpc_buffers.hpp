// Device memory behind the RPC server's buffers: what ggml_backend_buft_alloc_buffer / ggml_backend_tensor_set /
// ggml_backend_tensor_get / ggml_backend_buffer_clear / ggml_backend_dev_memory are to the reference's rpc_server
// (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:340-470).  The product binary links the
// HIP implementation (rpc_buffers_hip.cpp); the protocol tests on machines without a GPU link a host-memory stand-in.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>

namespace mesh_rpc {

class BufferBackend {
  public:
    virtual ~BufferBackend() = default;
    virtual int device_count() = 0;
    virtual std::string device_name(int dev) = 0;          // "ROCm0": what `-d` takes and the device probe lists
    virtual std::string device_description(int dev) = 0;
    virtual bool device_memory(int dev, uint64_t *free_bytes, uint64_t *total_bytes) = 0;
    virtual uint64_t alignment() = 0;
    virtual uint64_t max_size(int dev) = 0;
    // allocations live on device `dev`; the pointer value is the address clients put into tensor descriptors
    virtual void *alloc(int dev, uint64_t size) = 0;
    virtual void release(int dev, void *base) = 0;
    virtual bool upload(int dev, void *dst, const void *host_src, uint64_t size) = 0;
    virtual bool download(int dev, void *host_dst, const void *src, uint64_t size) = 0;
    virtual bool fill(int dev, void *dst, uint8_t value, uint64_t size) = 0;
    virtual bool copy(int dev, void *dst, const void *src, uint64_t size) = 0;
};

// one per process; defined by whichever implementation is linked
BufferBackend *buffer_backend();

}  // namespace mesh_rpc
