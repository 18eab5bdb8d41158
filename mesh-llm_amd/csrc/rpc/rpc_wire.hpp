// Wire format of the ggml RPC protocol, version 4.1.0, as spoken by the reference's patched rpc-server.
//
//   request : | cmd u8 | size u64 LE | payload[size] |
//   response: | size u64 LE | payload[size] |           (commands with a reply; SET_TENSOR has none)
//
// Command numbering, the packed 296-byte tensor descriptor and the peer-transfer messages follow
// third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:1042-1148 (its self-contained test client
// restates them), SET_TENSOR_GGUF follows patches/0001-rpc-optimize-local-GGUF-tensor-loading.patch:56-63.  The remaining
// messages (alignment, max size, clear, hash, copy, alloc size, device memory, device count) belong to the un-vendored
// upstream ggml/src/ggml-rpc/ggml-rpc.cpp of llama.cpp@45155597; the patches show them only in use
// (patches/0001:110-138 get_alloc_size request = device, tensor, srcs[]; patches/0002:1990 device_count;
// patches/0002:391 buffer_clear = remote_ptr, value), and they are restated here from the protocol's published layout.
#pragma once

#include <cstdint>

namespace mesh_rpc {

constexpr uint8_t PROTO_MAJOR = 4, PROTO_MINOR = 1, PROTO_PATCH = 0;   // minor >= 1 announces the peer commands (patches/0002:25-28)

constexpr int MAX_DIMS = 4, MAX_SRC = 10, MAX_OP_PARAMS = 64, MAX_NAME = 64, CONN_CAPS_SIZE = 24;

enum Cmd : uint8_t {
    CMD_ALLOC_BUFFER = 0,
    CMD_GET_ALIGNMENT,
    CMD_GET_MAX_SIZE,
    CMD_BUFFER_GET_BASE,
    CMD_FREE_BUFFER,
    CMD_BUFFER_CLEAR,
    CMD_SET_TENSOR,
    CMD_SET_TENSOR_HASH,
    CMD_GET_TENSOR,
    CMD_COPY_TENSOR,
    CMD_GRAPH_COMPUTE,
    CMD_GET_DEVICE_MEMORY,
    CMD_INIT_TENSOR,
    CMD_GET_ALLOC_SIZE,
    CMD_HELLO,
    CMD_DEVICE_COUNT,
    CMD_GRAPH_RECOMPUTE,
    CMD_SET_TENSOR_GGUF,
    CMD_REGISTER_PEER,          // 18, the value mesh-llm's tunnel rewrites (mesh-llm/src/network/rewrite.rs:30)
    CMD_PUSH_TENSOR_TO_PEER,
    CMD_PEER_TENSOR_DATA,
    CMD_COUNT,
};

#pragma pack(push, 1)

struct Tensor {
    uint64_t id;
    uint32_t type;
    uint64_t buffer;                              // handle returned by ALLOC_BUFFER, 0 = no buffer
    uint32_t ne[MAX_DIMS];
    uint32_t nb[MAX_DIMS];
    uint32_t op;
    int32_t op_params[MAX_OP_PARAMS / sizeof(int32_t)];
    int32_t flags;
    uint64_t src[MAX_SRC];
    uint64_t view_src;
    uint64_t view_offs;
    uint64_t data;                                // device address inside the buffer
    char name[MAX_NAME];
    char padding[4];
};
static_assert(sizeof(Tensor) == 296, "rpc_tensor is 296 bytes on the wire");

struct HelloReq { uint8_t conn_caps[CONN_CAPS_SIZE]; };
struct HelloRsp { uint8_t major, minor, patch, padding; uint8_t conn_caps[CONN_CAPS_SIZE]; };
struct DeviceCountRsp { uint32_t device_count; };
struct AllocBufferReq { uint32_t device; uint64_t size; };
struct AllocBufferRsp { uint64_t remote_ptr, remote_size; };
struct GetAlignmentReq { uint32_t device; };
struct GetAlignmentRsp { uint64_t alignment; };
struct GetMaxSizeReq { uint32_t device; };
struct GetMaxSizeRsp { uint64_t max_size; };
struct BufferGetBaseReq { uint64_t remote_ptr; };
struct BufferGetBaseRsp { uint64_t base_ptr; };
struct FreeBufferReq { uint64_t remote_ptr; };
struct BufferClearReq { uint64_t remote_ptr; uint8_t value; };
struct SetTensorHashReq { Tensor tensor; uint64_t offset, hash; };
struct SetTensorHashRsp { uint8_t result; };
struct GetTensorReq { Tensor tensor; uint64_t offset, size; };
struct CopyTensorReq { Tensor src, dst; };
struct CopyTensorRsp { uint8_t result; };
struct InitTensorReq { Tensor tensor; };
struct GetAllocSizeReq { uint32_t device; Tensor tensor; Tensor srcs[MAX_SRC]; };
struct GetAllocSizeRsp { uint64_t alloc_size; };
struct GetDeviceMemoryReq { uint32_t device; };
struct GetDeviceMemoryRsp { uint64_t free_mem, total_mem; };
struct GraphRecomputeReq { uint32_t device; };
struct SetTensorGgufReq { Tensor tensor; uint64_t offset; };
struct SetTensorGgufRsp { uint8_t result; };
struct RegisterPeerReq { uint32_t peer_id; char endpoint[128]; };
struct RegisterPeerRsp { uint8_t result; };
struct PushTensorToPeerReq { uint32_t peer_id; Tensor src, dst; uint64_t offset, size; };
struct PushTensorToPeerRsp { uint8_t result; };

#pragma pack(pop)

static_assert(sizeof(HelloRsp) == 28 && sizeof(AllocBufferReq) == 12 && sizeof(RegisterPeerReq) == 132 &&
              sizeof(PushTensorToPeerReq) == 4 + 2 * 296 + 16 && sizeof(GetTensorReq) == 312, "packed message sizes");

// ggml type ids that can appear in a tensor descriptor: elements per block and bytes per block (0 = unknown to this build)
struct TypeTraits { uint32_t block_elems, block_bytes; };
inline TypeTraits type_traits(uint32_t type) {
    switch (type) {
        case 0: return {1, 4};        // F32
        case 1: return {1, 2};        // F16
        case 2: return {32, 18};      // Q4_0
        case 3: return {32, 20};      // Q4_1
        case 6: return {32, 22};      // Q5_0
        case 7: return {32, 24};      // Q5_1
        case 8: return {32, 34};      // Q8_0
        case 9: return {32, 36};      // Q8_1
        case 10: return {256, 84};    // Q2_K
        case 11: return {256, 110};   // Q3_K
        case 12: return {256, 144};   // Q4_K
        case 13: return {256, 176};   // Q5_K
        case 14: return {256, 210};   // Q6_K
        case 15: return {256, 292};   // Q8_K
        case 24: return {1, 1};       // I8
        case 25: return {1, 2};       // I16
        case 26: return {1, 4};       // I32
        case 27: return {1, 8};       // I64
        case 28: return {1, 8};       // F64
        case 30: return {1, 2};       // BF16
        default: return {0, 0};
    }
}

// ggml_nbytes of a descriptor: the span from its first to one past its last byte; 0 if the type is unknown
inline uint64_t tensor_nbytes(const Tensor &t) {
    const TypeTraits tt = type_traits(t.type);
    if (!tt.block_elems) return 0;
    for (int i = 0; i < MAX_DIMS; ++i)
        if (t.ne[i] == 0) return 0;
    uint64_t n;
    if (tt.block_elems == 1) {
        n = tt.block_bytes;
        for (int i = 0; i < MAX_DIMS; ++i) n += (uint64_t)(t.ne[i] - 1) * t.nb[i];
    } else {
        n = (uint64_t)t.ne[0] * t.nb[0] / tt.block_elems;
        for (int i = 1; i < MAX_DIMS; ++i) n += (uint64_t)(t.ne[i] - 1) * t.nb[i];
    }
    return n;
}

}  // namespace mesh_rpc
