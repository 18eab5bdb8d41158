// GRAPH_COMPUTE / GRAPH_RECOMPUTE of the ggml RPC protocol: what rpc_server::graph_compute deserialises and hands to
// ggml_backend_graph_compute in the reference (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:
// 443-451; the stored graph a RECOMPUTE replays: patches/0001-rpc-optimize-local-GGUF-tensor-loading.patch:163-174).
//
// This build has no general graph interpreter.  The one graph a mesh-llm worker is sent is the decoder sub-graph of its
// contiguous layer range; it is recognised by the GGUF names of the weight tensors it multiplies with (the same names
// SET_TENSOR_GGUF loads by, patches/0001:179-266) and run as ONE stage decode call over the tensors' device memory.  Any
// other graph is refused, and a refused request ends the connection with a logged reason, as a failing request does in
// the reference.
#pragma once

#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "rpc_wire.hpp"

namespace mesh_rpc {

// payload of GRAPH_COMPUTE: | device u32 | n_nodes u32 | node ids u64[n_nodes] | n_tensors u32 | rpc_tensor[n_tensors] |
// (rpc_tensor: patches/0002:1070-1085; the ids are the client's tensor addresses)
struct ParsedGraph {
    uint32_t device = 0;
    std::vector<uint64_t> nodes;                       // evaluation order
    std::vector<Tensor> tensors;                       // nodes and leaves
    std::unordered_map<uint64_t, size_t> index;        // id -> position in `tensors`
    const Tensor *find(uint64_t id) const {
        auto it = index.find(id);
        return it == index.end() ? nullptr : &tensors[it->second];
    }
};

// false with `why` set: truncated or oversized payload, duplicate ids, a node or source id without a descriptor
bool parse_graph(const uint8_t *data, size_t size, ParsedGraph *out, std::string *why);

// What a recognised layer-range graph asks for.
struct StagePlan {
    int layer_begin = 0, layer_end = 0;                // [begin, end) by the blk.{i}.* names
    int n_tokens = 0;
    uint32_t n_embd = 0;
    Tensor input;                                      // f32 [n_embd, n_tokens]: the hidden state entering the range
    Tensor positions;                                  // i32 [n_tokens]
    Tensor output;                                     // the graph's last node: f32 [n_embd, n_tokens], or [n_vocab, n_tokens] logits
    bool logits = false;
    int n_ctx = 0;                                     // cache positions per sequence, from the cache tensors' shape; 0 = not in the graph
    uint32_t k_type = 1, v_type = 1;                   // ggml types of the cache tensors (f16 when the graph shows none)
};

// false with `why` set when the graph is not the decoder sub-graph of one contiguous layer range of a llama / qwen2 /
// qwen3 / qwen3moe model, or uses something the stage has no kernel for.
bool recognise_layer_range(const ParsedGraph &g, StagePlan *plan, std::string *why);

// Runs a plan on the device that holds the tensors.  The product binary links the stage library's runner
// (rpc_graph_runner.cpp); the protocol tests on machines without a GPU link a stand-in.
class GraphRunner {
  public:
    virtual ~GraphRunner() = default;
    // device: backend device index; gguf_path: the server's --gguf file (the hyper-parameters and the stage's own weight
    // layout come from it).  false with `why` set on failure.
    virtual bool run(int device, const std::string &gguf_path, const StagePlan &plan, std::string *why) = 0;
};
GraphRunner *graph_runner();

}  // namespace mesh_rpc
