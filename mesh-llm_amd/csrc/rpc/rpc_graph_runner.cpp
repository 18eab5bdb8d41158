// Runs a recognised layer-range graph as one call of the stage library (mesh_stage_decode_dev over the tensors' device
// memory): where the reference hands the deserialised graph to ggml_backend_graph_compute
// (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451).
//
// The stage is opened from the server's --gguf file on first use of a layer range (the launcher passes the same file to
// rpc-server and to llama-server, mesh-llm/src/inference/launch.rs:920-932): hyper-parameters come from the file's
// metadata, and the weights are kept a second time in the mat-vec kernels' tiled layout, beside the row-major bytes the
// client placed in its RPC buffers.  The key / value cache is the stage session's own (cache slot = position, one
// sequence); the cache tensors the client allocated only tell its depth and row types.

#include <cstdarg>
#include <cstdio>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "../../../include/mesh_stage.h"
#include "rpc_buffers.hpp"
#include "rpc_graph.hpp"

namespace mesh_rpc {

namespace {

class StageRunner final : public GraphRunner {
  public:
    ~StageRunner() override {
        for (auto &kv : entries_) {
            if (kv.second.session) mesh_stage_session_free(kv.second.session);
            if (kv.second.stage) mesh_stage_close(kv.second.stage);
        }
    }

    bool run(int device, const std::string &gguf_path, const StagePlan &plan, std::string *why) override {
        if (gguf_path.empty()) return fail(why, "graph execution needs the model file: start the server with --gguf PATH");
        std::lock_guard<std::mutex> lk(mu_);
        const Key key{device, plan.layer_begin, plan.layer_end, (int)plan.k_type, (int)plan.v_type};
        Entry &e = entries_[key];
        const int n_ctx = plan.n_ctx > 0 ? plan.n_ctx : 4096;
        if (!e.stage || e.n_batch < plan.n_tokens || e.n_ctx < n_ctx) {
            // first use of this range, or a call larger than the stage was opened for: (re)open
            if (e.session) mesh_stage_session_free(e.session);
            if (e.stage) mesh_stage_close(e.stage);
            e = Entry{};
            const std::string dev_name = "ROCm" + std::to_string(device);
            mesh_stage_opts o{};
            o.device = dev_name.c_str();
            o.n_ctx = n_ctx;
            o.n_seq_max = 1;
            o.n_batch_max = plan.n_tokens > 512 ? plan.n_tokens : 512;      // llama-server's default micro-batch
            o.kv_type = (int)plan.k_type;
            o.kv_type_v = (int)plan.v_type;
            if (mesh_stage_open(gguf_path.c_str(), plan.layer_begin, plan.layer_end, &o, &e.stage) != MESH_OK ||
                mesh_stage_session_new(e.stage, &e.session) != MESH_OK) {
                const std::string msg = mesh_last_error();
                if (e.stage) mesh_stage_close(e.stage);
                entries_.erase(key);
                return fail(why, "cannot open layers [%d, %d) of %s as a stage: %s", plan.layer_begin, plan.layer_end, gguf_path.c_str(), msg.c_str());
            }
            e.n_batch = o.n_batch_max;
            e.n_ctx = n_ctx;
            mesh_model_info info{};
            if (mesh_stage_info(e.stage, &info) == MESH_OK) e.n_embd = info.n_embd;
            fprintf(stderr, "[rpc-server] graph execution: layers [%d, %d) of %s opened as a stage (%zu weight bytes, context %d)\n", plan.layer_begin,
                    plan.layer_end, gguf_path.c_str(), mesh_stage_weight_bytes(e.stage), n_ctx);
        }
        if (e.n_embd != plan.n_embd) return fail(why, "the graph's hidden state has %u rows, the model file says %u", plan.n_embd, e.n_embd);
        std::vector<int32_t> pos((size_t)plan.n_tokens);
        if (!buffer_backend()->download(device, pos.data(), reinterpret_cast<const void *>((uintptr_t)plan.positions.data), pos.size() * sizeof(int32_t)))
            return fail(why, "cannot read the positions");
        mesh_batch batch{plan.n_tokens, pos.data(), nullptr};
        const size_t out_cap = (size_t)tensor_nbytes(plan.output);
        size_t out_len = 0;
        const int rc = mesh_stage_decode_dev(e.session, &batch, reinterpret_cast<const void *>((uintptr_t)plan.input.data), MESH_F32,
                                             reinterpret_cast<void *>((uintptr_t)plan.output.data), plan.logits ? MESH_LOGITS : MESH_F32, out_cap, &out_len);
        if (rc != MESH_OK || mesh_session_synchronize(e.session) != MESH_OK) return fail(why, "stage decode of %d tokens failed: %s", plan.n_tokens, mesh_last_error());
        if (out_len != out_cap) return fail(why, "the stage wrote %zu bytes, the graph's result tensor holds %zu", out_len, out_cap);
        return true;
    }

  private:
    using Key = std::tuple<int, int, int, int, int>;
    struct Entry {
        mesh_stage *stage = nullptr;
        mesh_session *session = nullptr;
        int n_batch = 0, n_ctx = 0;
        uint32_t n_embd = 0;
    };
    static bool fail(std::string *why, const char *fmt, ...) __attribute__((format(printf, 2, 3))) {
        char buf[640];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        if (why) *why = buf;
        return false;
    }
    std::mutex mu_;
    std::map<Key, Entry> entries_;
};

}  // namespace

GraphRunner *graph_runner() {
    static StageRunner r;
    return &r;
}

}  // namespace mesh_rpc
