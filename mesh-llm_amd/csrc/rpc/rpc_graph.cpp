// Deserialisation of GRAPH_COMPUTE payloads and recognition of the one graph this build runs: the decoder sub-graph of a
// contiguous layer range.  See rpc_graph.hpp.

#include "rpc_graph.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>

#include "ggml_ops.hpp"

namespace mesh_rpc {

namespace {

constexpr uint32_t TYPE_F32 = 0, TYPE_F16 = 1, TYPE_Q4_0 = 2, TYPE_Q8_0 = 8, TYPE_I32 = 26;
// a graph of a 64-layer range has a few thousand tensors; anything far beyond that is not a decoder sub-graph
constexpr uint32_t MAX_NODES = 1u << 20, MAX_TENSORS = 1u << 20;

std::string tensor_name(const Tensor &t) { return std::string(t.name, strnlen(t.name, MAX_NAME)); }

// The scheduler names the copy of a tensor that crosses into another backend "<backend>#<name>#<copy>"; the name proper is
// what lies between the first and the last '#'.  (patches/0001:78-79 skips such names for the local-GGUF load for the same
// reason: they are not GGUF tensors.)
std::string base_name(const std::string &n) {
    const size_t a = n.find('#'), b = n.rfind('#');
    if (a == std::string::npos || a == b) return n;
    return n.substr(a + 1, b - a - 1);
}

bool starts_with(const std::string &s, const char *p) { return s.compare(0, strlen(p), p) == 0; }

bool set_why(std::string *why, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
bool set_why(std::string *why, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (why) *why = buf;
    return false;
}

uint64_t n_elements(const Tensor &t) { return (uint64_t)t.ne[0] * t.ne[1] * t.ne[2] * t.ne[3]; }

// "blk.<i>.<rest>" -> (i, rest)
bool split_blk(const std::string &name, int *layer, std::string *rest) {
    if (!starts_with(name, "blk.")) return false;
    size_t p = 4;
    if (p >= name.size() || name[p] < '0' || name[p] > '9') return false;
    long v = 0;
    while (p < name.size() && name[p] >= '0' && name[p] <= '9' && v < 100000) v = v * 10 + (name[p++] - '0');
    if (p >= name.size() || name[p] != '.') return false;
    *layer = (int)v;
    *rest = name.substr(p + 1);
    return true;
}

}  // namespace

bool parse_graph(const uint8_t *data, size_t size, ParsedGraph *out, std::string *why) {
    *out = ParsedGraph{};
    size_t at = 0;
    auto take = [&](void *dst, size_t n) {
        if (size - at < n) return false;
        memcpy(dst, data + at, n);
        at += n;
        return true;
    };
    uint32_t n_nodes = 0, n_tensors = 0;
    if (!take(&out->device, 4) || !take(&n_nodes, 4)) return set_why(why, "payload of %zu bytes is shorter than its header", size);
    if (n_nodes == 0 || n_nodes > MAX_NODES) return set_why(why, "%u nodes", n_nodes);
    if ((size - at) / sizeof(uint64_t) < n_nodes) return set_why(why, "payload ends inside the list of %u node ids", n_nodes);
    out->nodes.resize(n_nodes);
    (void)take(out->nodes.data(), (size_t)n_nodes * sizeof(uint64_t));
    if (!take(&n_tensors, 4)) return set_why(why, "payload ends before the tensor count");
    if (n_tensors == 0 || n_tensors > MAX_TENSORS) return set_why(why, "%u tensors", n_tensors);
    if (size - at != (size_t)n_tensors * sizeof(Tensor))
        return set_why(why, "%zu bytes follow the tensor count, %u descriptors of %zu bytes were announced", size - at, n_tensors, sizeof(Tensor));
    out->tensors.resize(n_tensors);
    (void)take(out->tensors.data(), (size_t)n_tensors * sizeof(Tensor));
    out->index.reserve(n_tensors);
    for (size_t i = 0; i < out->tensors.size(); ++i) {
        const uint64_t id = out->tensors[i].id;
        if (id == 0) return set_why(why, "descriptor %zu has id 0", i);
        if (!out->index.emplace(id, i).second) return set_why(why, "two descriptors share id 0x%llx", (unsigned long long)id);
    }
    for (uint64_t id : out->nodes)
        if (!out->find(id)) return set_why(why, "node 0x%llx has no descriptor", (unsigned long long)id);
    for (const Tensor &t : out->tensors) {
        for (int s = 0; s < MAX_SRC; ++s)
            if (t.src[s] && !out->find(t.src[s])) return set_why(why, "source %d of '%s' has no descriptor", s, tensor_name(t).c_str());
        if (t.view_src && !out->find(t.view_src)) return set_why(why, "the view source of '%s' has no descriptor", tensor_name(t).c_str());
    }
    return true;
}

bool recognise_layer_range(const ParsedGraph &g, StagePlan *plan, std::string *why) {
    *plan = StagePlan{};
    // ---- the weights, by GGUF name
    static const char *const required[] = {"attn_norm.weight", "attn_q.weight", "attn_k.weight", "attn_v.weight", "attn_output.weight", "ffn_norm.weight"};
    static const char *const dense[] = {"ffn_gate.weight", "ffn_up.weight", "ffn_down.weight"};
    static const char *const experts[] = {"ffn_gate_inp.weight", "ffn_gate_exps.weight", "ffn_up_exps.weight", "ffn_down_exps.weight"};
    static const char *const optional[] = {"attn_q.bias", "attn_k.bias", "attn_v.bias", "attn_q_norm.weight", "attn_k_norm.weight"};
    std::map<int, std::map<std::string, const Tensor *>> layers;
    const Tensor *output_w = nullptr, *output_norm = nullptr;
    std::set<uint64_t> used;            // ids that some node reads
    for (const Tensor &t : g.tensors)
        for (int s = 0; s < MAX_SRC; ++s)
            if (t.src[s]) used.insert(t.src[s]);
    for (const Tensor &t : g.tensors) {
        if (t.op != GGML_OP_NONE) continue;
        const std::string name = tensor_name(t);
        int il;
        std::string rest;
        if (split_blk(name, &il, &rest)) {
            bool known = false;
            for (const char *k : required) known = known || rest == k;
            for (const char *k : dense) known = known || rest == k;
            for (const char *k : experts) known = known || rest == k;
            for (const char *k : optional) known = known || rest == k;
            if (!known) return set_why(why, "tensor '%s': the stage has no kernel for this weight", name.c_str());
            if (!used.count(t.id)) return set_why(why, "weight '%s' is in the graph but no node reads it", name.c_str());
            layers[il][rest] = &t;
        } else if (name == "output.weight") {
            output_w = &t;
        } else if (name == "output_norm.weight") {
            output_norm = &t;
        } else if (name == "token_embd.weight") {
            if (!output_w) output_w = &t;          // tied output projection (or an embedding lookup, refused below by the input search)
        } else if (starts_with(name, "rope_freqs")) {
            return set_why(why, "tensor '%s': rope frequency factors are not supported", name.c_str());
        }
    }
    if (layers.empty()) return set_why(why, "no blk.{i}.* weight in the graph: not a decoder layer sub-graph (%zu nodes, first op %u %s)", g.nodes.size(),
                                       g.find(g.nodes[0])->op, ggml_op_name_guess(g.find(g.nodes[0])->op));
    const int b = layers.begin()->first, e = layers.rbegin()->first + 1;
    if ((int)layers.size() != e - b) return set_why(why, "the graph names layers %d..%d but only %zu of them: not one contiguous range", b, e - 1, layers.size());
    for (const auto &kv : layers) {
        for (const char *k : required)
            if (!kv.second.count(k)) return set_why(why, "layer %d lacks blk.%d.%s", kv.first, kv.first, k);
        int n_dense = 0, n_exp = 0;
        for (const char *k : dense) n_dense += (int)kv.second.count(k);
        for (const char *k : experts) n_exp += (int)kv.second.count(k);
        if (!((n_dense == 3 && n_exp == 0) || (n_dense == 0 && n_exp == 4)))
            return set_why(why, "layer %d has neither a whole dense nor a whole mixture-of-experts feed-forward block", kv.first);
    }
    const Tensor &an = *layers.begin()->second.at("attn_norm.weight");
    const Tensor &wk = *layers.begin()->second.at("attn_k.weight");
    if (an.type != TYPE_F32 || an.ne[0] == 0) return set_why(why, "blk.%d.attn_norm.weight is not an f32 vector", b);
    plan->layer_begin = b;
    plan->layer_end = e;
    plan->n_embd = an.ne[0];

    // ---- the hidden state entering the range: the one f32 leaf [n_embd, T] that is neither a weight nor a cache
    const Tensor *input = nullptr;
    int n_inputs = 0;
    for (const Tensor &t : g.tensors) {
        if (t.op != GGML_OP_NONE || t.view_src || t.type != TYPE_F32 || t.ne[0] != plan->n_embd || t.ne[2] != 1 || t.ne[3] != 1) continue;
        const std::string name = tensor_name(t), bn = base_name(name);
        int il;
        std::string rest;
        if (split_blk(name, &il, &rest) || starts_with(name, "output") || starts_with(name, "token_embd") || starts_with(bn, "cache_")) continue;
        if (!used.count(t.id)) continue;
        input = &t;
        ++n_inputs;
    }
    if (n_inputs != 1) return set_why(why, "%d candidates for the hidden-state input (f32 leaves of %u rows): cannot tell what enters layer %d", n_inputs, plan->n_embd, b);
    plan->input = *input;
    plan->n_tokens = (int)input->ne[1];
    if (plan->n_tokens <= 0) return set_why(why, "the hidden-state input holds no token");

    // ---- positions
    const Tensor *pos = nullptr;
    for (const Tensor &t : g.tensors) {
        if (t.op != GGML_OP_NONE || t.type != TYPE_I32) continue;
        if (base_name(tensor_name(t)) == "inp_pos") {
            if (pos) return set_why(why, "two position inputs");
            pos = &t;
        }
    }
    if (!pos) return set_why(why, "no position input (inp_pos) among the leaves");
    if (n_elements(*pos) != (uint64_t)plan->n_tokens)
        return set_why(why, "%llu positions for %d tokens (multi-section rope is not supported)", (unsigned long long)n_elements(*pos), plan->n_tokens);
    plan->positions = *pos;

    // ---- the result: the graph's last node
    const Tensor &out = *g.find(g.nodes.back());
    if (out.type != TYPE_F32 || out.ne[2] != 1 || out.ne[3] != 1) return set_why(why, "the last node '%s' is not an f32 matrix", tensor_name(out).c_str());
    if (out.ne[0] == plan->n_embd && !output_w) {
        plan->logits = false;
    } else if (output_w && output_norm && out.ne[0] == output_w->ne[1]) {
        plan->logits = true;
    } else {
        return set_why(why, "the last node '%s' has %u rows: neither the hidden state (%u) nor logits of an output projection in the graph",
                       tensor_name(out).c_str(), out.ne[0], plan->n_embd);
    }
    if ((int)out.ne[1] != plan->n_tokens)
        return set_why(why, "the last node holds %u of the %d tokens (output row selection is not supported: ask for every token's result)", out.ne[1], plan->n_tokens);
    plan->output = out;

    // ---- the cache the client allocated: its row types and depth tell how to size the stage's own
    const uint64_t kd = wk.ne[1];
    for (const Tensor &t : g.tensors) {
        if (t.op != GGML_OP_NONE || t.view_src) continue;
        const std::string bn = base_name(tensor_name(t));
        const bool is_k = starts_with(bn, "cache_k_l"), is_v = starts_with(bn, "cache_v_l");
        if (!is_k && !is_v) continue;
        if (t.type != TYPE_F16 && t.type != TYPE_Q8_0 && t.type != TYPE_Q4_0) return set_why(why, "cache tensor '%s' has type %u (f16, q8_0 and q4_0 are supported)", bn.c_str(), t.type);
        (is_k ? plan->k_type : plan->v_type) = t.type;
        if (kd && n_elements(t) % kd == 0) {
            const uint64_t depth = n_elements(t) / kd;
            if (depth > 0 && depth < (1u << 24)) plan->n_ctx = (int)depth;
        }
    }
    return true;
}

}  // namespace mesh_rpc
