// Stand-in for the stage library's graph runner, so that graph parsing, recognition, replay and failure behaviour of the
// RPC server are testable on a machine without a GPU.  Test infrastructure only: the product binary links
// mesh-llm_amd/csrc/rpc/rpc_graph_runner.cpp, which runs the stage's kernels.
//
// "Runs" a recognised plan over host memory: result[t][i] = input[t][i % n_embd] + positions[t] + 100 * layer_begin +
// 10000 * layer_end, which lets a test see which graph ran, on which data, and that a replay read fresh inputs.

#include <cstring>

#include "rpc_graph.hpp"

namespace mesh_rpc {

namespace {

class HostRunner final : public GraphRunner {
  public:
    bool run(int, const std::string &gguf_path, const StagePlan &plan, std::string *why) override {
        if (gguf_path.empty()) {
            if (why) *why = "graph execution needs the model file: start the server with --gguf PATH";
            return false;
        }
        const float *in = reinterpret_cast<const float *>((uintptr_t)plan.input.data);
        const int32_t *pos = reinterpret_cast<const int32_t *>((uintptr_t)plan.positions.data);
        float *out = reinterpret_cast<float *>((uintptr_t)plan.output.data);
        const uint32_t rows = plan.output.ne[0];
        for (int t = 0; t < plan.n_tokens; ++t)
            for (uint32_t i = 0; i < rows; ++i)
                out[(size_t)t * rows + i] = in[(size_t)t * plan.n_embd + i % plan.n_embd] + (float)pos[t] + 100.f * plan.layer_begin + 10000.f * plan.layer_end;
        return true;
    }
};

}  // namespace

GraphRunner *graph_runner() {
    static HostRunner r;
    return &r;
}

}  // namespace mesh_rpc
