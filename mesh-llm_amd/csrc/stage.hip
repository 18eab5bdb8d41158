// The pipeline-stage executor: loads layers [begin, end) of a GGUF model into HBM and runs them over a batch of
// token activations, keeping a stage-local f16 KV cache per session.
//
// It does, in one process and on one GPU, what a mesh-llm worker does today through llama.cpp RPC:
//   * weight load by tensor name from the local GGUF  -- rpc_server::set_tensor_gguf,
//     third_party/llama.cpp/patches/0001-rpc-optimize-local-GGUF-tensor-loading.patch:179-266
//   * the per-layer graph  rms_norm -> q,k,v -> rope -> kv store -> attention -> o (+residual) -> rms_norm ->
//     gate,up -> silu*mul -> down (+residual)  -- rpc_server::graph_compute, patches/0002-...:443-451
//   * boundary hand-off of the hidden state -- push_tensor_to_peer, patches/0002-...:544-622 (packed here).

#include "stage.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "attn.hpp"
#include "gemm.hpp"
#include "gemv.hpp"
#include "moe.hpp"

namespace mesh {

int act_pack_dev(int fmt, const float *src, void *dst, int64_t n, hipStream_t stream);
int act_unpack_dev(int fmt, const void *src, float *dst, int64_t n, hipStream_t stream);
int dequantize_dev(int type, const void *src, float *dst, int64_t n, hipStream_t stream);

// ------------------------------------------------------------------------------------------------ hparams
int hparams_from_gguf(const GgufFile &g, HParams &hp) {
    if (!g.get_str("general.architecture", hp.arch)) return fail(MESH_ERR_FORMAT, "gguf: general.architecture missing");
    const std::string &a = hp.arch;
    if (a != "llama" && a != "qwen2" && a != "qwen3" && a != "qwen3moe")
        return fail(MESH_ERR_UNSUPPORTED, "architecture '%s' is not supported (llama, qwen2, qwen3, qwen3moe are)", a.c_str());
    auto need = [&](const char *suffix, uint32_t &out) -> int {
        if (!g.get_u32(a + suffix, out)) return fail(MESH_ERR_FORMAT, "gguf: key %s%s missing or not an unsigned integer", a.c_str(), suffix);
        return MESH_OK;
    };
    int rc;
    if ((rc = need(".block_count", hp.n_layer)) || (rc = need(".embedding_length", hp.n_embd)) ||
        (rc = need(".attention.head_count", hp.n_head)))
        return rc;
    hp.n_head_kv = hp.n_head;
    g.get_u32(a + ".attention.head_count_kv", hp.n_head_kv);
    g.get_u32(a + ".feed_forward_length", hp.n_ff);
    g.get_u32(a + ".vocab_size", hp.n_vocab);
    if (hp.n_head == 0 || hp.n_head_kv == 0 || hp.n_head % hp.n_head_kv) return fail(MESH_ERR_FORMAT, "gguf: head counts %u/%u inconsistent", hp.n_head, hp.n_head_kv);
    hp.head_dim = hp.n_embd / hp.n_head;
    g.get_u32(a + ".attention.key_length", hp.head_dim);
    hp.n_rot = hp.head_dim;
    g.get_u32(a + ".rope.dimension_count", hp.n_rot);
    g.get_f32(a + ".attention.layer_norm_rms_epsilon", hp.rms_eps);
    g.get_f32(a + ".rope.freq_base", hp.rope_freq_base);
    g.get_u32(a + ".expert_count", hp.n_expert);
    g.get_u32(a + ".expert_used_count", hp.n_expert_used);
    g.get_u32(a + ".expert_feed_forward_length", hp.n_ff_exp);
    hp.rope_mode = (a == "llama") ? ROPE_NORM : ROPE_NEOX;
    // Frequency scaling (linear / yarn keys, or the per-frequency factors tensor of Llama-3.1 files) would change every
    // rotation angle; no kernel here applies it, so such a file is refused instead of decoded with unscaled angles.
    {
        std::string scaling;
        if (g.get_str(a + ".rope.scaling.type", scaling) && !scaling.empty() && scaling != "none")
            return fail(MESH_ERR_UNSUPPORTED, "gguf: rope scaling type '%s' is not supported", scaling.c_str());
        if (g.find("rope_freqs.weight")) return fail(MESH_ERR_UNSUPPORTED, "gguf: rope frequency factors (rope_freqs.weight) are not supported");
    }
    if (hp.n_layer == 0 || hp.n_embd == 0 || hp.head_dim == 0) return fail(MESH_ERR_FORMAT, "gguf: zero-sized model dimensions");
    if (hp.n_rot > hp.head_dim || hp.n_rot % 2) return fail(MESH_ERR_FORMAT, "gguf: rope dimension count %u does not fit head_dim %u", hp.n_rot, hp.head_dim);
    if (a == "qwen3moe" && (hp.n_expert == 0 || hp.n_expert_used == 0 || hp.n_expert_used > hp.n_expert))
        return fail(MESH_ERR_FORMAT, "gguf: qwen3moe without a usable expert_count / expert_used_count");
    return MESH_OK;
}


// ------------------------------------------------------------------------------------------------ loading
namespace {

struct Loader {
    const GgufFile &g;
    mesh_stage &st;
    void *staging = nullptr;
    size_t staging_bytes = 0;
    bool gemm_layout = false;      // also keep K-quant projection matrices in the prefill GEMM's layout

    ~Loader() { if (staging) (void)hipFree(staging); }

    int dev_alloc(void **p, size_t bytes) {
        hipError_t e = hipMalloc(p, bytes ? bytes : 16);
        if (e != hipSuccess) return fail(e == hipErrorOutOfMemory ? MESH_ERR_NOMEM : MESH_ERR_DEVICE, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        st.allocations.push_back(*p);
        return MESH_OK;
    }

    // Loads tensor `name` into `out`.  want_K / want_M < 0 skip that check.  required=false: absent is fine.
    int load(const std::string &name, DevTensor &out, int64_t want_K, int64_t want_M, int64_t want_E, bool required,
             bool tile, bool f32_only) {
        const GgufTensorInfo *ti = g.find(name);
        if (!ti) return required ? fail(MESH_ERR_FORMAT, "gguf: tensor '%s' not found", name.c_str()) : MESH_OK;
        const int64_t K = (int64_t)ti->ne[0], M = (int64_t)ti->ne[1], E = (int64_t)ti->ne[2];
        if (ti->ne[3] != 1 || (want_K >= 0 && K != want_K) || (want_M >= 0 && M != want_M) || (want_E >= 0 && E != want_E))
            return fail(MESH_ERR_FORMAT, "gguf: tensor '%s' has shape [%lld,%lld,%lld], expected [%lld,%lld,%lld]", name.c_str(),
                        (long long)K, (long long)M, (long long)E, (long long)want_K, (long long)want_M, (long long)want_E);
        if (block_elems((int)ti->type) < 0)
            return fail(MESH_ERR_UNSUPPORTED, "gguf: tensor '%s' has ggml type %u, which this build has no kernel for", name.c_str(), ti->type);
        if (f32_only && ti->type != MESH_F32) return fail(MESH_ERR_UNSUPPORTED, "gguf: tensor '%s' must be F32 (is type %u)", name.c_str(), ti->type);
        const uint8_t *src = g.data(*ti);
        if (!src) return fail(MESH_ERR_FORMAT, "gguf: tensor '%s' (%llu bytes at offset %llu) lies outside the file", name.c_str(),
                              (unsigned long long)ti->nbytes, (unsigned long long)ti->offset);
        out.type = (int)ti->type;
        out.K = K; out.M = M; out.E = E;
        out.tiled = tile && type_is_tiled(out.type);
        st.weight_bytes += ti->nbytes;
        int rc;
        if (!out.tiled) {
            out.bytes = ti->nbytes;
            if ((rc = dev_alloc(&out.data, out.bytes)) != MESH_OK) return rc;
            MESH_HIP_TRY(hipMemcpy(out.data, src, out.bytes, hipMemcpyHostToDevice));
            return MESH_OK;
        }
        const size_t per_e = (size_t)tiled_bytes(out.type, M, K);
        const size_t src_per_e = (size_t)(M * row_bytes(out.type, K));
        out.bytes = per_e * (size_t)E;
        if ((rc = dev_alloc(&out.data, out.bytes)) != MESH_OK) return rc;
        if (staging_bytes < ti->nbytes) {
            if (staging) (void)hipFree(staging);
            staging = nullptr;
            hipError_t e = hipMalloc(&staging, ti->nbytes);
            if (e != hipSuccess) { staging_bytes = 0; return fail(MESH_ERR_NOMEM, "hipMalloc(%llu) for load staging failed", (unsigned long long)ti->nbytes); }
            staging_bytes = ti->nbytes;
        }
        MESH_HIP_TRY(hipMemcpy(staging, src, ti->nbytes, hipMemcpyHostToDevice));
        for (int64_t e = 0; e < E; ++e) {
            rc = repack_tiled(out.type, static_cast<const uint8_t *>(staging) + e * src_per_e,
                              static_cast<uint8_t *>(out.data) + e * per_e, M, K, nullptr);
            if (rc != MESH_OK) return rc;
        }
        MESH_HIP_TRY(hipDeviceSynchronize());
        return MESH_OK;
    }

    static bool packable(const DevTensor &t) { return t.present() && t.tiled && t.E == 1 && gemm_packed_bytes(t.type, t.M, t.K) > 0; }
    // GEMM-layout copies of n matrices back to back in one buffer (every matrix but the last must be a whole number
    // of 128-row blocks for the buffer to serve one launch; the caller checks that before relying on it)
    int pack_group(DevTensor *const *ts, int n) {
        size_t total = 0;
        for (int i = 0; i < n; ++i) total += gemm_packed_bytes(ts[i]->type, ts[i]->M, ts[i]->K);
        void *buf = nullptr;
        int rc;
        if ((rc = dev_alloc(&buf, total)) != MESH_OK) return rc;
        size_t off = 0;
        for (int i = 0; i < n; ++i) {
            ts[i]->gemm = static_cast<uint8_t *>(buf) + off;
            if ((rc = gemm_pack(ts[i]->type, ts[i]->data, ts[i]->gemm, ts[i]->M, ts[i]->K, nullptr)) != MESH_OK) return rc;
            off += gemm_packed_bytes(ts[i]->type, ts[i]->M, ts[i]->K);
        }
        st.gemm_layout_bytes += total;
        MESH_HIP_TRY(hipDeviceSynchronize());
        return MESH_OK;
    }
    // the dense projections of a layer
    int pack_layer(LayerWeights &L) {
        if (!gemm_layout) return MESH_OK;
        int rc;
        auto same = [](const DevTensor &a, const DevTensor &b) { return a.type == b.type && a.K == b.K; };
        DevTensor *q = &L.wq, *k = &L.wk, *v = &L.wv, *o = &L.wo, *g = &L.w_gate, *u = &L.w_up, *d = &L.w_down;
        if (packable(*q) && packable(*k) && same(*q, *k) && q->M % 128 == 0) {
            const bool three = packable(*v) && same(*q, *v) && k->M % 128 == 0;
            DevTensor *grp[3] = {q, k, v};
            if ((rc = pack_group(grp, three ? 3 : 2)) != MESH_OK) return rc;
            L.qkv_fused = three ? 3 : 2;
            if (!three && packable(*v) && (rc = pack_group(&v, 1)) != MESH_OK) return rc;
        } else {
            for (DevTensor *t : {q, k, v})
                if (packable(*t) && (rc = pack_group(&t, 1)) != MESH_OK) return rc;
        }
        for (DevTensor *t : {o, d})
            if (packable(*t) && (rc = pack_group(&t, 1)) != MESH_OK) return rc;
        if (packable(*g) && packable(*u) && same(*g, *u) && g->M == u->M) {
            const size_t pb = gemm_packed_pair_bytes(g->type, g->M, g->K);
            if ((rc = dev_alloc(&L.gate_up_gemm, pb)) != MESH_OK) return rc;
            if ((rc = gemm_pack_pair(g->type, g->data, u->data, L.gate_up_gemm, g->M, g->K, nullptr)) != MESH_OK) return rc;
            st.gemm_layout_bytes += pb;
            MESH_HIP_TRY(hipDeviceSynchronize());
        } else {
            for (DevTensor *t : {g, u})
                if (packable(*t) && (rc = pack_group(&t, 1)) != MESH_OK) return rc;
        }
        return MESH_OK;
    }
    // the expert matrices of a mixture-of-experts layer, for prefill chunks (expert launches of the large-tile GEMM): every
    // expert's gate / up pair and down projection in the GEMM layout, experts back to back
    int pack_experts(LayerWeights &L) {
        if (!gemm_layout) return MESH_OK;
        const DevTensor &g = L.gate_exps, &u = L.up_exps, &d = L.down_exps;
        if (!g.present() || !g.tiled || !u.tiled || !d.tiled || g.type != u.type || g.M != u.M || g.K != u.K || g.M % 64 || g.E != u.E || g.E != d.E) return MESH_OK;
        const size_t pair_b = gemm_packed_pair_bytes(g.type, g.M, g.K), down_b = gemm_packed_bytes(d.type, d.M, d.K);
        if (!pair_b || !down_b) return MESH_OK;
        int rc;
        if ((rc = dev_alloc(&L.exps_gate_up_gemm, pair_b * (size_t)g.E)) != MESH_OK || (rc = dev_alloc(&L.exps_down_gemm, down_b * (size_t)g.E)) != MESH_OK) return rc;
        const size_t g_e = tiled_bytes(g.type, g.M, g.K), d_e = tiled_bytes(d.type, d.M, d.K);
        for (int64_t e = 0; e < g.E; ++e) {
            if ((rc = gemm_pack_pair(g.type, static_cast<const uint8_t *>(g.data) + e * g_e, static_cast<const uint8_t *>(u.data) + e * g_e,
                                     static_cast<uint8_t *>(L.exps_gate_up_gemm) + e * pair_b, g.M, g.K, nullptr)) != MESH_OK ||
                (rc = gemm_pack(d.type, static_cast<const uint8_t *>(d.data) + e * d_e, static_cast<uint8_t *>(L.exps_down_gemm) + e * down_b, d.M, d.K, nullptr)) != MESH_OK)
                return rc;
        }
        L.exps_gate_up_stride = pair_b;
        L.exps_down_stride = down_b;
        st.gemm_layout_bytes += (pair_b + down_b) * (size_t)g.E;
        MESH_HIP_TRY(hipDeviceSynchronize());
        return MESH_OK;
    }
};

}  // namespace

int stage_open(const char *path, int layer_begin, int layer_end, const mesh_stage_opts *opts, mesh_stage **out) {
    if (!path || !out) return fail(MESH_ERR_INVALID, "mesh_stage_open: null argument");
    *out = nullptr;
    GgufFile g;
    int rc = g.open(path);
    if (rc != MESH_OK) return rc;
    std::unique_ptr<mesh_stage> st(new mesh_stage());
    if ((rc = hparams_from_gguf(g, st->hp)) != MESH_OK) return rc;
    const HParams &hp = st->hp;
    if (layer_end < 0) layer_end = (int)hp.n_layer;
    if (layer_begin < 0 || layer_begin >= layer_end || layer_end > (int)hp.n_layer)
        return fail(MESH_ERR_INVALID, "mesh_stage_open: layer range [%d,%d) does not fit a %u-layer model", layer_begin, layer_end, hp.n_layer);
    st->layer_begin = layer_begin;
    st->layer_end = layer_end;
    if ((rc = tuning_process_default(st->tune)) != MESH_OK) return rc;
    if (opts && opts->tuning && (rc = tuning_parse(st->tune, opts->tuning, "mesh_stage_opts.tuning")) != MESH_OK) return rc;
    st->n_ctx = opts && opts->n_ctx > 0 ? opts->n_ctx : 4096;
    st->n_seq_max = opts && opts->n_seq_max > 0 ? opts->n_seq_max : 1;
    st->n_batch_max = opts && opts->n_batch_max > 0 ? opts->n_batch_max : 512;
    st->k_type = opts && opts->kv_type ? opts->kv_type : MESH_F16;
    st->v_type = opts && opts->kv_type_v ? opts->kv_type_v : (st->k_type == MESH_F16 ? MESH_F16 : MESH_Q4_0);
    if (!kv_pair_supported(st->k_type, st->v_type))
        return fail(MESH_ERR_UNSUPPORTED, "mesh_stage_open: KV cache types %d/%d not supported (f16/f16, q8_0/q4_0 and q4_0/q4_0 are)", st->k_type, st->v_type);
    if (opts && opts->device && opts->device[0]) {
        if ((rc = mesh_device_select(opts->device)) != MESH_OK) return rc;
    }
    if (mesh_device_count() < 1) return fail(MESH_ERR_DEVICE, "mesh_stage_open: no GPU available");
    MESH_HIP_TRY(hipGetDevice(&st->device));
    if (hp.head_dim != 64 && hp.head_dim != 128)
        return fail(MESH_ERR_UNSUPPORTED, "mesh_stage_open: head_dim %u has no attention kernel (64 and 128 do)", hp.head_dim);

    Loader ld{g, *st};
    // stages that can be handed prefill-sized calls keep a GEMM-layout copy of their projections (gemm_layout=0: no
    // copy, the GEMM reads the mat-vec tiles)
    ld.gemm_layout = st->n_batch_max >= st->tune.gemm_min_tokens && st->tune.gemm_layout;
    const int64_t E = hp.n_embd, QD = (int64_t)hp.n_head * hp.head_dim, KD = (int64_t)hp.n_head_kv * hp.head_dim;
    const bool moe = hp.arch == "qwen3moe";
    st->layers.resize((size_t)(layer_end - layer_begin));
    int64_t n_expert_file = -1;
    for (int il = layer_begin; il < layer_end; ++il) {
        LayerWeights &L = st->layers[(size_t)(il - layer_begin)];
        const std::string p = "blk." + std::to_string(il) + ".";
        if ((rc = ld.load(p + "attn_norm.weight", L.attn_norm, E, 1, 1, true, false, true)) ||
            (rc = ld.load(p + "attn_q.weight", L.wq, E, QD, 1, true, true, false)) ||
            (rc = ld.load(p + "attn_k.weight", L.wk, E, KD, 1, true, true, false)) ||
            (rc = ld.load(p + "attn_v.weight", L.wv, E, KD, 1, true, true, false)) ||
            (rc = ld.load(p + "attn_output.weight", L.wo, QD, E, 1, true, true, false)) ||
            (rc = ld.load(p + "attn_q.bias", L.bq, QD, 1, 1, false, false, true)) ||
            (rc = ld.load(p + "attn_k.bias", L.bk, KD, 1, 1, false, false, true)) ||
            (rc = ld.load(p + "attn_v.bias", L.bv, KD, 1, 1, false, false, true)) ||
            (rc = ld.load(p + "attn_q_norm.weight", L.q_norm, hp.head_dim, 1, 1, false, false, true)) ||
            (rc = ld.load(p + "attn_k_norm.weight", L.k_norm, hp.head_dim, 1, 1, false, false, true)) ||
            (rc = ld.load(p + "ffn_norm.weight", L.ffn_norm, E, 1, 1, true, false, true)))
            return rc;
        if (moe && (rc = ld.pack_layer(L)) != MESH_OK) return rc;       // (its attention projections)
        if (!moe) {
            if (hp.n_ff == 0) return fail(MESH_ERR_FORMAT, "gguf: feed_forward_length missing");
            if ((rc = ld.load(p + "ffn_gate.weight", L.w_gate, E, hp.n_ff, 1, true, true, false)) ||
                (rc = ld.load(p + "ffn_up.weight", L.w_up, E, hp.n_ff, 1, true, true, false)) ||
                (rc = ld.load(p + "ffn_down.weight", L.w_down, hp.n_ff, E, 1, true, true, false)))
                return rc;
            if ((rc = ld.pack_layer(L)) != MESH_OK) return rc;
        } else {
            const GgufTensorInfo *gi = g.find(p + "ffn_gate_inp.weight");
            if (!gi) return fail(MESH_ERR_FORMAT, "gguf: tensor '%sffn_gate_inp.weight' not found", p.c_str());
            const int64_t ne = (int64_t)gi->ne[1];     // experts present in this file (a shard has fewer than the model)
            const int64_t ffe = hp.n_ff_exp;
            if (ffe == 0) return fail(MESH_ERR_FORMAT, "gguf: expert_feed_forward_length missing");
            // the session sizes its routing buffers by the first layer's count, and one lane of the router holds at
            // most MOE_EXPERTS_MAX / 64 experts
            if (n_expert_file < 0) n_expert_file = ne;
            if (ne != n_expert_file || ne < (int64_t)hp.n_expert_used || ne > MOE_EXPERTS_MAX)
                return fail(MESH_ERR_FORMAT, "gguf: layer %d routes over %lld experts (first layer %lld, %u used per token, at most %d supported)", il,
                            (long long)ne, (long long)n_expert_file, hp.n_expert_used, MOE_EXPERTS_MAX);
            if ((rc = ld.load(p + "ffn_gate_inp.weight", L.gate_inp, E, ne, 1, true, false, false)) ||
                (rc = ld.load(p + "ffn_gate_exps.weight", L.gate_exps, E, ffe, ne, true, true, false)) ||
                (rc = ld.load(p + "ffn_up_exps.weight", L.up_exps, E, ffe, ne, true, true, false)) ||
                (rc = ld.load(p + "ffn_down_exps.weight", L.down_exps, ffe, E, ne, true, true, false)))
                return rc;
            if ((rc = ld.pack_experts(L)) != MESH_OK) return rc;
        }
    }
    if (layer_begin == 0) {
        if ((rc = ld.load("token_embd.weight", st->tok_embd, E, -1, 1, false, false, false)) != MESH_OK) return rc;
    }
    if (layer_end == (int)hp.n_layer) {
        if ((rc = ld.load("output_norm.weight", st->output_norm, E, 1, 1, false, false, true)) != MESH_OK) return rc;
        if (g.find("output.weight")) {
            if ((rc = ld.load("output.weight", st->output, E, -1, 1, true, true, false)) != MESH_OK) return rc;
        } else if (st->output_norm.present() && g.find("token_embd.weight")) {
            // tied embeddings: the output projection is token_embd
            if ((rc = ld.load("token_embd.weight", st->output, E, -1, 1, true, true, false)) != MESH_OK) return rc;
        }
    }
    // inverse frequencies by ggml's f32 recurrence: theta_i = theta_{i-1} * base^(-2/n_rot)
    {
        std::vector<float> inv(hp.n_rot / 2);
        const float theta_scale = powf(hp.rope_freq_base, -2.0f / (float)hp.n_rot);
        float th = 1.0f;
        for (size_t i = 0; i < inv.size(); ++i) { inv[i] = th; th *= theta_scale; }
        void *p = nullptr;
        if ((rc = ld.dev_alloc(&p, inv.size() * sizeof(float))) != MESH_OK) return rc;
        st->rope_inv_freq = static_cast<float *>(p);
        MESH_HIP_TRY(hipMemcpy(p, inv.data(), inv.size() * sizeof(float), hipMemcpyHostToDevice));
    }
    MESH_HIP_TRY(hipDeviceSynchronize());
    *out = st.release();
    return MESH_OK;
}

static int sess_alloc(mesh_session *s, void **p, size_t bytes);
static bool layer_is_kquant_dense(const LayerWeights &L);

// ------------------------------------------------------------------------------------------------ session
static int sess_alloc(mesh_session *s, void **p, size_t bytes) {
    hipError_t e = hipMalloc(p, bytes ? bytes : 16);
    if (e != hipSuccess) return fail(e == hipErrorOutOfMemory ? MESH_ERR_NOMEM : MESH_ERR_DEVICE, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    s->allocations.push_back(*p);
    return MESH_OK;
}

constexpr int ATTN_SPLITS_MAX = ATTN_SPLITS_CAP;
constexpr int ATTN_PART_ROWS_MIN = 512;     // rows of (token, split) the partial buffers always hold
constexpr int META_SLOTS = 8;
constexpr int LOGITS_TOKENS_MAX = MESH_LOGITS_TOKENS_MAX;        // logits rows the host-pointer entry point stages per call
// Mixture of experts: calls with at least moe_gemm_min_pairs (token, slot) pairs per expert on average run the expert
// products as tiles of the large-tile GEMM (measured against the other kernels on a 64-expert shard with top-8 routing,
// four layers: 0.607 against 0.659 ms at 4 pairs per expert, 0.536 against 0.485 at 2).  Below that the mat-vec kernel;
// the 16-pair integer matrix-core kernel covers stages without GEMM-layout copies of the experts.
#define PREFILL_MIN_TOKENS (s->tune.gemm_min_tokens)
#define MOE_GEMM_MIN_PAIRS_PER_EXPERT ((size_t)s->tune.moe_gemm_min_pairs)

int session_new(mesh_stage *st, mesh_session **out) {
    if (!st || !out) return fail(MESH_ERR_INVALID, "mesh_stage_session_new: null argument");
    *out = nullptr;
    MESH_HIP_TRY(hipSetDevice(st->device));
    std::unique_ptr<mesh_session> s(new mesh_session());
    s->stage = st;
    const HParams &hp = st->hp;
    const size_t nl = st->layers.size(), B = (size_t)st->n_batch_max;
    MESH_HIP_TRY(hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking));
    s->tune = st->tune;
    const size_t kv_rows = (size_t)st->n_seq_max * hp.n_head_kv * (size_t)st->n_ctx;
    s->k_layer_bytes = kv_rows * (size_t)kv_row_bytes(st->k_type, (int)hp.head_dim);
    s->v_layer_bytes = kv_rows * (size_t)kv_row_bytes(st->v_type, (int)hp.head_dim);
    int rc;
    void *p = nullptr;
    if ((rc = sess_alloc(s.get(), &p, nl * s->k_layer_bytes)) != MESH_OK) return rc;
    s->kcache = static_cast<uint8_t *>(p);
    if ((rc = sess_alloc(s.get(), &p, nl * s->v_layer_bytes)) != MESH_OK) return rc;
    s->vcache = static_cast<uint8_t *>(p);
    MESH_HIP_TRY(hipMemsetAsync(s->kcache, 0, nl * s->k_layer_bytes, s->stream));
    MESH_HIP_TRY(hipMemsetAsync(s->vcache, 0, nl * s->v_layer_bytes, s->stream));
    const size_t QD = (size_t)hp.n_head * hp.head_dim, KD = (size_t)hp.n_head_kv * hp.head_dim;
    const size_t ff = std::max<size_t>(hp.n_ff, (size_t)hp.n_ff_exp * std::max<uint32_t>(hp.n_expert_used, 1));
    auto fbuf = [&](float **dst, size_t n) -> int {
        void *q = nullptr;
        int r = sess_alloc(s.get(), &q, n * sizeof(float));
        *dst = static_cast<float *>(q);
        return r;
    };
    const size_t part_rows = std::max<size_t>(B, ATTN_PART_ROWS_MIN);
    s->attn_part_rows = part_rows;
    if ((rc = fbuf(&s->x, B * hp.n_embd)) || (rc = fbuf(&s->q, B * QD)) || (rc = fbuf(&s->k, B * KD)) ||
        (rc = fbuf(&s->v, B * KD)) || (rc = fbuf(&s->attn, B * QD)) || (rc = fbuf(&s->ffn, B * ff)) ||
        (rc = fbuf(&s->attn_part, part_rows * QD)) || (rc = fbuf(&s->attn_ml, part_rows * hp.n_head * 2)))
        return rc;
    if ((rc = sess_alloc(s.get(), &p, 256)) != MESH_OK) return rc;
    s->f16_sat = static_cast<unsigned *>(p);
    MESH_HIP_TRY(hipMemsetAsync(p, 0, 256, s->stream));
    if (hp.n_ff && hp.n_ff % QK_K == 0) {
        if ((rc = sess_alloc(s.get(), &p, xq_bytes((int)hp.n_ff))) != MESH_OK) return rc;
        s->ffn_xq = static_cast<uint8_t *>(p);
    }
    // (either skinny kernel may be picked per call, so the buffers are there from the smaller of their thresholds on)
    const int skinny_alloc_from = s->tune.skinny_min_tokens > 0 ? s->tune.skinny_min_tokens : 4;
    if (B >= (size_t)std::min(PREFILL_MIN_TOKENS, skinny_alloc_from)) {
        const size_t B16 = (B + 15) / 16 * 16;       // the skinny GEMM reads whole blocks of 16 tokens
        if ((rc = sess_alloc(s.get(), &p, B16 * std::max<size_t>(hp.n_embd, QD) * 2)) != MESH_OK) return rc;
        s->xn16 = static_cast<uint16_t *>(p);
        MESH_HIP_TRY(hipMemsetAsync(p, 0, B16 * std::max<size_t>(hp.n_embd, QD) * 2, s->stream));     // unused token columns stay finite
        {
            // q16 activations of the skinny GEMM (calls below the large-tile GEMM's token count), widest projection input
            // (mixture-of-experts stages also run their prefill expert products from this layout: every token)
            const size_t tok = hp.n_expert ? B : std::min<size_t>(B, (size_t)std::max(16, PREFILL_MIN_TOKENS - 1));
            s->xq_tokens = tok;
            const size_t kmax = std::max<size_t>(std::max<size_t>(hp.n_embd, QD), hp.n_ff);
            size_t bytes = (tok + 15) / 16 * q16_block_bytes((int)((kmax + 255) / 256 * 256));
            // mixture of experts: the down projections read one row of n_ff_exp per (token, slot) pair
            if (hp.n_expert) bytes = std::max(bytes, (tok * hp.n_expert_used + 15) / 16 * q16_block_bytes((int)((hp.n_ff_exp + 255) / 256 * 256)));
            if ((rc = sess_alloc(s.get(), &p, bytes)) != MESH_OK) return rc;
            s->xq = static_cast<uint8_t *>(p);
        }
        if (st->k_type != MESH_F16 && hp.head_dim == 128 && B >= 128) {
            // f16 copy of one sequence's K and V rows of one layer: a long prefill chunk decodes the quantised cache once
            // per layer into it (attn.hpp: chunk_kv16).  Zeroed, so that rows past a chunk's last key are finite.
            const size_t bytes = 2 * (size_t)hp.n_head_kv * st->n_ctx * hp.head_dim * 2;
            if ((rc = sess_alloc(s.get(), &p, bytes)) != MESH_OK) return rc;
            s->chunk_kv16 = static_cast<uint16_t *>(p);
            MESH_HIP_TRY(hipMemsetAsync(p, 0, bytes, s->stream));
        }
        if (hp.n_ff > 0) {
            // (two blocks of 16 tokens: the hand-over is for calls the skinny GEMM takes in one launch)
            if ((rc = sess_alloc(s.get(), &p, SKINNY_F16_NORM_TOKENS_MAX * (size_t)hp.n_embd * 2)) != MESH_OK) return rc;
            s->norm16 = static_cast<uint16_t *>(p);
            MESH_HIP_TRY(hipMemsetAsync(p, 0, SKINNY_F16_NORM_TOKENS_MAX * (size_t)hp.n_embd * 2, s->stream));
            if ((rc = fbuf(&s->norm_part, (size_t)SKINNY_F16_NORM_PARTS_MAX * SKINNY_F16_NORM_TOKENS_MAX)) != MESH_OK) return rc;
            if ((rc = sess_alloc(s.get(), &p, B16 * (size_t)hp.n_ff * 2)) != MESH_OK) return rc;
            s->ffn16 = static_cast<uint16_t *>(p);
            if ((rc = fbuf(&s->ffn_up, B * (size_t)hp.n_ff)) != MESH_OK) return rc;
        }
        if (B >= (size_t)PREFILL_MIN_TOKENS) {
            // a split launch holds at most one 128 x 128 f32 tile per CU: 16.8 MB on 256 CUs
            s->gemm_part_bytes = (size_t)32 << 20;
            if ((rc = sess_alloc(s.get(), &p, s->gemm_part_bytes)) != MESH_OK) return rc;
            s->gemm_part = static_cast<float *>(p);
        }
    }
    if (hp.n_expert_used > 0 && !st->layers.empty() && st->layers[0].gate_inp.present()) {
        const size_t ne = (size_t)st->layers[0].gate_inp.M, k = hp.n_expert_used;
        if ((rc = fbuf(&s->moe_logits, B * ne)) || (rc = fbuf(&s->moe_w, B * k)) || (rc = fbuf(&s->moe_out, B * k * hp.n_embd)) ||
            (rc = fbuf(&s->expert_mask, ne)))
            return rc;
        if ((rc = sess_alloc(s.get(), &p, B * k * sizeof(int32_t))) != MESH_OK) return rc;
        s->moe_ids = static_cast<int32_t *>(p);
        // work items: 4 pairs each for the mat-vec kernel, 16 for the matrix-core one; the buffer fits either
        const size_t items = (size_t)std::max(moe_max_items((int)(B * k), (int)ne) * MOE_ITEM_INTS,
                                              moe_max_items((int)(B * k), (int)ne, SKINNY_ITEM_PAIRS) * moe_item_ints(SKINNY_ITEM_PAIRS)) / MOE_ITEM_INTS + 1;
        // (+ the item count, + the arrival counter of the router launch whose last workgroup routes and groups)
        if ((rc = sess_alloc(s.get(), &p, (items * MOE_ITEM_INTS + 2) * sizeof(int32_t))) != MESH_OK) return rc;
        s->moe_items = static_cast<int32_t *>(p);
        s->moe_n_items = s->moe_items + items * MOE_ITEM_INTS;
        s->moe_arrive = reinterpret_cast<int *>(s->moe_n_items + 1);
        MESH_HIP_TRY(hipMemsetAsync(s->moe_items, 0, (items * MOE_ITEM_INTS + 2) * sizeof(int32_t), s->stream));
        MESH_HIP_TRY(hipMemsetAsync(s->expert_mask, 0, ne * sizeof(float), s->stream));
        if (st->layers[0].exps_gate_up_gemm && s->xn16 && B * k >= MOE_GEMM_MIN_PAIRS_PER_EXPERT * ne) {
            // prefill chunks: the pairs sorted by expert, their inputs / SwiGLU outputs in the k8-major f16 layout and their
            // down-projection rows, all indexed by slot (moe.hpp: moe_sort)
            const size_t slots = (size_t)moe_sort_slots((int)(B * k), (int)ne), tiles = (size_t)moe_sort_max_tiles((int)(B * k), (int)ne);
            const size_t pairs4 = (B * k + 3) / 4 * 4;
            if ((rc = sess_alloc(s.get(), &p, (pairs4 + slots + 4 * tiles + 4) * sizeof(int32_t))) != MESH_OK) return rc;
            s->moe_sorted.slot_of_pair = static_cast<int32_t *>(p);
            s->moe_sorted.pair_of_slot = s->moe_sorted.slot_of_pair + pairs4;
            s->moe_sorted.tiles = s->moe_sorted.pair_of_slot + slots;           // (a multiple of 16 ints in: 16-byte aligned)
            s->moe_sorted.counts = s->moe_sorted.tiles + 4 * tiles;
            if ((rc = sess_alloc(s.get(), &p, slots * hp.n_embd * 2)) != MESH_OK) return rc;
            s->moe_x16 = static_cast<uint16_t *>(p);
            if ((rc = sess_alloc(s.get(), &p, slots * (size_t)hp.n_ff_exp * 2)) != MESH_OK) return rc;
            s->moe_ffn16 = static_cast<uint16_t *>(p);
            if ((rc = fbuf(&s->moe_out_slots, slots * hp.n_embd)) != MESH_OK) return rc;
            MESH_HIP_TRY(hipMemsetAsync(s->moe_x16, 0, slots * hp.n_embd * 2, s->stream));          // unused slots stay finite
            MESH_HIP_TRY(hipMemsetAsync(s->moe_ffn16, 0, slots * (size_t)hp.n_ff_exp * 2, s->stream));
        }
    }
    if ((rc = sess_alloc(s.get(), &p, 3 * B * sizeof(int32_t))) != MESH_OK) return rc;
    s->d_pos = static_cast<int32_t *>(p);
    s->d_seq = s->d_pos + B;
    s->d_tok = s->d_seq + B;
    MESH_HIP_TRY(hipHostMalloc(reinterpret_cast<void **>(&s->h_meta), META_SLOTS * 3 * B * sizeof(int32_t), hipHostMallocDefault));
    memset(s->h_meta, 0, META_SLOTS * 3 * B * sizeof(int32_t));
    // staging for packed in/out of the host-pointer entry point: f32 rows of n_embd in; the same or logits rows out
    // (logits of at most LOGITS_TOKENS_MAX tokens per call: a row of a 152k vocabulary is 0.6 MB)
    s->io_stage_bytes = B * (size_t)hp.n_embd * sizeof(float);
    s->io_out_bytes = std::max(s->io_stage_bytes, st->output.present() ? std::min<size_t>(B, LOGITS_TOKENS_MAX) * (size_t)st->output.M * sizeof(float) : 0);
    if ((rc = sess_alloc(s.get(), &s->io_stage, s->io_stage_bytes + s->io_out_bytes)) != MESH_OK) return rc;
    MESH_HIP_TRY(hipHostMalloc(&s->h_io, s->io_stage_bytes + s->io_out_bytes, hipHostMallocDefault));
    MESH_HIP_TRY(hipStreamSynchronize(s->stream));
    *out = s.release();
    return MESH_OK;
}

// ------------------------------------------------------------------------------------------------ decode
static GemvMat mat_of(const DevTensor &w, float *y, int ldy, const DevTensor *bias) {
    GemvMat m;
    m.W = w.data; m.type = w.type; m.M = (int)w.M; m.y = y; m.ldy = ldy;
    m.bias = bias && bias->present() ? static_cast<const float *>(bias->data) : nullptr;
    return m;
}

// Batches of at least attn_mma_min_tokens tokens take the matrix-core decode attention (Q and the probabilities rounded
// to f16; faster at every batch size, so the default is 1).  Callers that want the all-f32 vector-ALU kernel at small
// batches raise it.
// quantised: the cache rows are q8_0 / q4_0
static int attn_splits_for(const Tuning &tune, int T, int n_kv, int max_keys, bool quantised) {
    // One workgroup per compute unit (256 on gfx950) measured best from batch 1 to 16 with f16 rows, which that many
    // workgroups stream at the memory's rate.  Quantised rows are bound by the instructions that decode them, and two
    // workgroups per CU hide each other's waits: 3-7% of the step at batch 8-32 (Qwen2.5-32B shape, q8_0 / q4_0 cache:
    // 9.86 -> 9.18 ms at batch 32, which otherwise runs unsplit); four per CU lose again, and so do 64 splits of a single
    // token's walk (from 64 (token, KV head) pairs on).
    // (attn_split_target: the workgroup count aimed at, for experiments)
    const int forced = tune.attn_split_target;
    const int target = forced ? forced : (quantised && T * n_kv >= 64) ? 512 : 256;
    int s = target / std::max(1, T * n_kv);
    s = std::min(s, (max_keys + 63) / 64);
    return std::max(1, std::min(s, ATTN_SPLITS_MAX));
}

// ---- optional timing -----------------------------------------------------------------------------
// A ProfScope names the kernel class of the launches made while it lives; launch_timer() (mesh_common.hpp) hands each of
// them an event pair of the session, which profile_collect reads back.
namespace {
thread_local mesh_session *t_prof_session = nullptr;
thread_local int t_prof_kind = 0;
}  // namespace

LaunchTimer launch_timer() {
    LaunchTimer t;
    mesh_session *s = t_prof_session;
    if (!s) return t;
    if (s->prof_used + 2 > s->prof_events.size()) {
        for (int i = 0; i < 2; ++i) {
            hipEvent_t e;
            if (hipEventCreate(&e) != hipSuccess) { (void)hipGetLastError(); return t; }
            s->prof_events.push_back(e);
        }
    }
    s->prof_kinds.push_back(t_prof_kind);
    t.start = s->prof_events[s->prof_used];
    t.stop = s->prof_events[s->prof_used + 1];
    s->prof_used += 2;
    return t;
}

struct ProfScope {
    mesh_session *prev_s;
    int prev_kind;
    ProfScope(mesh_session *ses, int kind) : prev_s(t_prof_session), prev_kind(t_prof_kind) {
        if (ses->profile) { t_prof_session = ses; t_prof_kind = kind; }
    }
    ~ProfScope() { t_prof_session = prev_s; t_prof_kind = prev_kind; }
};

int profile_collect(mesh_session *s) {
    MESH_HIP_TRY(hipStreamSynchronize(s->stream));
    for (size_t i = 0; i + 1 < s->prof_used && i / 2 < s->prof_kinds.size(); i += 2) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, s->prof_events[i], s->prof_events[i + 1]) == hipSuccess) {
            s->prof_ms[s->prof_kinds[i / 2]] += ms;
            s->prof_launches[s->prof_kinds[i / 2]] += 1;
        } else {
            (void)hipGetLastError();
        }
    }
    s->prof_used = 0;
    s->prof_kinds.clear();
    return MESH_OK;
}

static bool layer_attn_is_kquant(const LayerWeights &L) {
    const DevTensor *w[] = {&L.wq, &L.wk, &L.wv, &L.wo};
    for (const DevTensor *t : w)
        if (!t->present() || !t->tiled) return false;
    return true;
}
static bool layer_is_kquant_dense(const LayerWeights &L) {
    const DevTensor *w[] = {&L.w_gate, &L.w_up, &L.w_down};
    for (const DevTensor *t : w)
        if (!t->present() || !t->tiled) return false;
    return layer_attn_is_kquant(L);
}

static GemmArgs gemm_of(const DevTensor &w, const uint16_t *x16, int ldx, int T, float *y, int ldy, const DevTensor *bias) {
    GemmArgs g;
    g.W = w.data; g.Wp = w.gemm; g.type = w.type; g.M = (int)w.M; g.K = (int)w.K; g.T = T;
    g.X = reinterpret_cast<const _Float16 *>(x16); g.ldx = ldx; g.Y = y; g.ldy = ldy;
    g.bias = bias && bias->present() ? static_cast<const float *>(bias->data) : nullptr;
    return g;
}

// One layer over many tokens: norms and activations are materialised in f16 and every projection is an MFMA GEMM.
// One dense K-quant layer over f16 activations on the matrix cores: `skinny` selects the batched-decode GEMM (few
// tokens, weight-streaming bound) instead of the large-tile prefill GEMM.
// attn_only: stop after the attention block (x += Wo . attention); the caller runs the feed-forward part.
static int run_layer_prefill(mesh_session *s, const LayerWeights &L, size_t il, int T, int max_keys, bool skinny, bool attn_only) {
    mesh_stage *st = s->stage;
    const HParams &hp = st->hp;
    hipStream_t stream = s->stream;
    const int E = (int)hp.n_embd, QD = (int)(hp.n_head * hp.head_dim), KD = (int)(hp.n_head_kv * hp.head_dim), FF = (int)hp.n_ff;
    _Float16 *xn = reinterpret_cast<_Float16 *>(s->xn16), *f16ffn = reinterpret_cast<_Float16 *>(s->ffn16);
    int rc;
    bool rope_fused = false, attn_is_k8 = false, ffn_norm_fused = false;
    const bool k8 = skinny || s->tune.gemm_xdirect;      // activations in the k8-major layout (both GEMMs can read it)
    // the batched-decode GEMM on the f16 matrix cores (k8-major f16 activations) instead of the integer ones (q16 activations);
    // a mixture-of-experts stage keeps the integer kernel, whose activation layout its expert launches share
    const bool sk16 = skinny && s->tune.skinny_f16 && L.w_gate.present() && f16ffn;
    const bool sk8 = skinny && !sk16;
    auto gemm_k8 = [&](GemmArgs g) { g.x_k8 = k8; g.part = s->tune.gemm_splitk ? s->gemm_part : nullptr; g.part_bytes = s->gemm_part_bytes; g.sat = s->f16_sat; g.big_tile = s->tune.gemm_big; g.narrow_tile = s->tune.gemm_narrow; return g; };
    auto rope_of = [&]() {
        GemvRope r;
        r.pos = s->d_pos; r.seq = s->d_seq; r.inv_freq = st->rope_inv_freq;
        r.kcache = reinterpret_cast<uint16_t *>(s->kcache + il * s->k_layer_bytes);
        r.vcache = reinterpret_cast<uint16_t *>(s->vcache + il * s->v_layer_bytes);
        r.head_dim = (int)hp.head_dim; r.n_rot = (int)hp.n_rot; r.n_kv = (int)hp.n_head_kv; r.n_ctx = st->n_ctx;
        return r;
    };
    // f16 skinny GEMM, calls it takes in one launch: the two RMS norms of the layer ride in the launches around them.  The output
    // projection and the down projection also write their result times the next norm's weight as f16 (norm16) and the sums
    // of squares their workgroups saw; q/k/v and gate/up read that and divide their products by the token's rms.
    const bool nf = sk16 && T <= SKINNY_F16_NORM_TOKENS_MAX && s->tune.skinny_norm_fused && s->norm16 && s->norm_part && E % 8 == 0;
    _Float16 *const nx = reinterpret_cast<_Float16 *>(s->norm16);
    const bool norm_ready = nf && s->norm_layer == (int)il;
    s->norm_layer = -1;
    {
        ProfScope ps(s, MESH_PROF_PREP);
        if (norm_ready) rc = MESH_OK;                        // the previous layer's down projection has left them in norm16
        else if (sk8 && s->xq_layer == (int)il) rc = MESH_OK;     // the previous layer's combine step has left them in s->xq
        else if (sk8) rc = quant16_k8(s->x, static_cast<const float *>(L.attn_norm.data), hp.rms_eps, T, E, s->xq, stream);
        else if (k8) rc = rmsnorm_f16_k8(s->x, static_cast<const float *>(L.attn_norm.data), hp.rms_eps, T, E, xn, stream, s->f16_sat);
        else rc = rmsnorm_f16(s->x, static_cast<const float *>(L.attn_norm.data), hp.rms_eps, T, E, xn, E, stream, s->f16_sat);
    }
    if (rc != MESH_OK) return rc;
    if (sk16) {
        SkinnyF16Args qa;
        qa.n_mat = 3;
        qa.mat[0] = mat_of(L.wq, s->q, QD, &L.bq);
        qa.mat[1] = mat_of(L.wk, s->k, KD, &L.bk);
        qa.mat[2] = mat_of(L.wv, s->v, KD, &L.bv);
        qa.x = xn; qa.K = E; qa.T = T;
        qa.pair_launch = s->tune.skinny_pair != 0;
        if (norm_ready) {
            qa.x = nx;
            qa.norm_in.part = s->norm_part; qa.norm_in.n_parts = s->norm_parts; qa.norm_in.eps = hp.rms_eps;
        }
        if (s->tune.gemv_rope && hp.rope_mode == ROPE_MODE_NORM && st->k_type == MESH_F16 && st->v_type == MESH_F16 && !L.q_norm.present() &&
            !L.k_norm.present() && hp.head_dim % 2 == 0 && hp.n_rot % 2 == 0) {
            qa.rope = rope_of();
            qa.kind[0] = GEMV_KIND_Q; qa.kind[1] = GEMV_KIND_K; qa.kind[2] = GEMV_KIND_V;
            rope_fused = true;
        }
        ProfScope ps(s, MESH_PROF_GEMV);
        if ((rc = gemm_skinny_f16(qa, stream)) != MESH_OK) return rc;
    } else if (skinny) {
        SkinnyArgs qa;
        qa.n_mat = 3;
        qa.mat[0] = mat_of(L.wq, s->q, QD, &L.bq);
        qa.mat[1] = mat_of(L.wk, s->k, KD, &L.bk);
        qa.mat[2] = mat_of(L.wv, s->v, KD, &L.bv);
        qa.xq = s->xq; qa.K = E; qa.T = T;
        qa.pair_launch = s->tune.skinny_pair != 0;
        if (s->tune.gemv_rope && hp.rope_mode == ROPE_MODE_NORM && st->k_type == MESH_F16 && st->v_type == MESH_F16 && !L.q_norm.present() &&
            !L.k_norm.present() && hp.head_dim % 2 == 0 && hp.n_rot % 2 == 0) {
            qa.rope.pos = s->d_pos; qa.rope.seq = s->d_seq; qa.rope.inv_freq = st->rope_inv_freq;
            qa.rope.kcache = reinterpret_cast<uint16_t *>(s->kcache + il * s->k_layer_bytes);
            qa.rope.vcache = reinterpret_cast<uint16_t *>(s->vcache + il * s->v_layer_bytes);
            qa.rope.head_dim = (int)hp.head_dim; qa.rope.n_rot = (int)hp.n_rot; qa.rope.n_kv = (int)hp.n_head_kv; qa.rope.n_ctx = st->n_ctx;
            qa.kind[0] = GEMV_KIND_Q; qa.kind[1] = GEMV_KIND_K; qa.kind[2] = GEMV_KIND_V;
            rope_fused = true;
        }
        ProfScope ps(s, MESH_PROF_GEMV);
        if ((rc = gemm_skinny(qa, stream)) != MESH_OK) return rc;
    } else {
        ProfScope ps(s, MESH_PROF_GEMV);
        if (L.qkv_fused >= 2 && s->tune.gemm_fused) {
            // q, k (and v when it is of the same K-quant type) as one launch over their back-to-back GEMM-layout copies
            const DevTensor *w[3] = {&L.wq, &L.wk, &L.wv}, *b[3] = {&L.bq, &L.bk, &L.bv};
            float *y[3] = {s->q, s->k, s->v};
            GemmArgs g = gemm_k8(gemm_of(L.wq, s->xn16, E, T, s->q, QD, nullptr));
            g.n_seg = L.qkv_fused;
            g.M = 0;
            for (int i = 0; i < g.n_seg; ++i) {
                g.seg_begin[i] = g.M / 128;
                g.seg_M[i] = (int)w[i]->M; g.seg_ldy[i] = (int)w[i]->M; g.seg_Y[i] = y[i];
                g.seg_bias[i] = b[i]->present() ? static_cast<const float *>(b[i]->data) : nullptr;
                g.M += (int)w[i]->M;
            }
            GemmArgs gv = gemm_k8(gemm_of(L.wv, s->xn16, E, T, s->v, KD, &L.bv));
            // RoPE and the KV append ride in the second kernel of split launches (both launches must be split)
            if (s->tune.gemv_rope && hp.rope_mode == ROPE_MODE_NORM && st->k_type == MESH_F16 && st->v_type == MESH_F16 && !L.q_norm.present() &&
                !L.k_norm.present() && hp.head_dim % 4 == 0 && hp.n_rot % 2 == 0 && gemm_split_count(g) > 1 &&
                (L.qkv_fused == 3 || gemm_split_count(gv) > 1)) {
                GemvRope r;
                r.pos = s->d_pos; r.seq = s->d_seq; r.inv_freq = st->rope_inv_freq;
                r.kcache = reinterpret_cast<uint16_t *>(s->kcache + il * s->k_layer_bytes);
                r.vcache = reinterpret_cast<uint16_t *>(s->vcache + il * s->v_layer_bytes);
                r.head_dim = (int)hp.head_dim; r.n_rot = (int)hp.n_rot; r.n_kv = (int)hp.n_head_kv; r.n_ctx = st->n_ctx;
                g.rope = r; gv.rope = r;
                g.kind[0] = GEMV_KIND_Q; g.kind[1] = GEMV_KIND_K; g.kind[2] = GEMV_KIND_V;
                gv.kind[0] = GEMV_KIND_V;
                rope_fused = true;
            }
            if ((rc = gemm_kquant(g, stream)) != MESH_OK) return rc;
            if (L.qkv_fused == 2 && (rc = gemm_kquant(gv, stream)) != MESH_OK) return rc;
        } else {
        if ((rc = gemm_kquant(gemm_k8(gemm_of(L.wq, s->xn16, E, T, s->q, QD, &L.bq)), stream)) != MESH_OK) return rc;
        if ((rc = gemm_kquant(gemm_k8(gemm_of(L.wk, s->xn16, E, T, s->k, KD, &L.bk)), stream)) != MESH_OK) return rc;
        if ((rc = gemm_kquant(gemm_k8(gemm_of(L.wv, s->xn16, E, T, s->v, KD, &L.bv)), stream)) != MESH_OK) return rc;
        }
    }
    RopeKvArgs ra;
    ra.q = s->q; ra.k = s->k; ra.v = s->v;
    ra.kcache = s->kcache + il * s->k_layer_bytes;
    ra.vcache = s->vcache + il * s->v_layer_bytes;
    ra.k_type = st->k_type; ra.v_type = st->v_type;
    ra.pos = s->d_pos; ra.seq = s->d_seq; ra.inv_freq = st->rope_inv_freq;
    ra.q_norm = L.q_norm.present() ? static_cast<const float *>(L.q_norm.data) : nullptr;
    ra.k_norm = L.k_norm.present() ? static_cast<const float *>(L.k_norm.data) : nullptr;
    ra.eps = hp.rms_eps;
    ra.n_head = (int)hp.n_head; ra.n_kv = (int)hp.n_head_kv; ra.head_dim = (int)hp.head_dim;
    ra.n_rot = (int)hp.n_rot; ra.rope_mode = (int)hp.rope_mode; ra.n_ctx = st->n_ctx;
    if (!rope_fused) {
        ProfScope ps(s, MESH_PROF_ROPE);
        if ((rc = rope_kv(ra, T, stream)) != MESH_OK) return rc;
    }
    AttnArgs aa;
    aa.q = s->q; aa.kcache = ra.kcache; aa.vcache = ra.vcache; aa.k_type = st->k_type; aa.v_type = st->v_type; aa.pos = s->d_pos; aa.seq = s->d_seq;
    aa.part = s->attn_part; aa.ml = s->attn_ml; aa.out = s->attn;
    aa.scale = 1.0f / sqrtf((float)hp.head_dim);
    aa.n_head = (int)hp.n_head; aa.n_kv = (int)hp.n_head_kv; aa.group = (int)(hp.n_head / hp.n_head_kv);
    aa.head_dim = (int)hp.head_dim; aa.n_ctx = st->n_ctx;
    aa.n_splits = T < 64 ? attn_splits_for(s->tune, T, (int)hp.n_head_kv, max_keys, st->k_type != MESH_F16) : 1;     // a batch of decode steps still splits the long KV
    {
        ProfScope ps(s, MESH_PROF_ATTN);
        if (!skinny && s->chunk_pos0 >= 0 && hp.head_dim == 128) {
            if (k8) { aa.out16_k8 = xn; attn_is_k8 = true; }          // straight into the output projection's input layout
            aa.chunk_kv16 = s->tune.chunk_kv16 ? reinterpret_cast<_Float16 *>(s->chunk_kv16) : nullptr;     // 0: every query tile decodes the quantised rows itself
            aa.part_rows = s->tune.attn_chunk_ksplit ? s->attn_part_rows : 0;
            rc = attention_chunk(aa, T, s->chunk_pos0, s->chunk_seq, stream);
        }
        else if (T >= s->tune.attn_mma_min_tokens && attention_mma_supported(aa)) {
            // straight into the output projection's input layout
            if (sk8) { aa.out_q16 = s->xq; attn_is_k8 = true; }
            else if (k8) { aa.out16_k8 = xn; attn_is_k8 = true; }
            rc = attention_mma(aa, T, stream);
        } else rc = attention(aa, T, stream);
    }
    if (rc != MESH_OK) return rc;
    {
        ProfScope ps(s, MESH_PROF_PREP);
        if (attn_is_k8) rc = MESH_OK;
        else if (sk8) rc = quant16_k8(s->attn, nullptr, 0.f, T, QD, s->xq, stream);
        else if (k8) rc = pack_f16_k8(s->attn, T, QD, xn, stream, s->f16_sat);
        else rc = act_pack_dev(MESH_F16, s->attn, s->xn16, (int64_t)T * QD, stream);
    }
    if (rc != MESH_OK) return rc;
    if (sk16) {
        SkinnyF16Args oa;
        oa.n_mat = 1;
        oa.mat[0] = mat_of(L.wo, s->x, E, nullptr);
        oa.x = xn; oa.K = QD; oa.T = T;
        oa.residual = s->x; oa.ldres = E; oa.epi = EPI_RESIDUAL;
        oa.sat = s->f16_sat;
        ffn_norm_fused = nf && !attn_only && gemm_skinny_f16_workgroups(oa) >= 1 && gemm_skinny_f16_workgroups(oa) <= SKINNY_F16_NORM_PARTS_MAX;
        if (ffn_norm_fused) {
            oa.norm_out.norm_w = static_cast<const float *>(L.ffn_norm.data); oa.norm_out.x16 = nx; oa.norm_out.part = s->norm_part;
            s->norm_parts = gemm_skinny_f16_workgroups(oa);
        }
        ProfScope ps(s, MESH_PROF_GEMV);
        if ((rc = gemm_skinny_f16(oa, stream)) != MESH_OK) return rc;
    } else if (skinny) {
        SkinnyArgs oa;
        oa.n_mat = 1;
        oa.mat[0] = mat_of(L.wo, s->x, E, nullptr);
        oa.xq = s->xq; oa.K = QD; oa.T = T;
        oa.residual = s->x; oa.ldres = E; oa.epi = EPI_RESIDUAL;
        ProfScope ps(s, MESH_PROF_GEMV);
        if ((rc = gemm_skinny(oa, stream)) != MESH_OK) return rc;
    } else {
        ProfScope ps(s, MESH_PROF_GEMV);
        GemmArgs go = gemm_k8(gemm_of(L.wo, s->xn16, QD, T, s->x, E, nullptr));
        go.residual = s->x; go.ldres = E;
        if ((rc = gemm_kquant(go, stream)) != MESH_OK) return rc;
    }
    if (attn_only) return MESH_OK;
    {
        ProfScope ps(s, MESH_PROF_PREP);
        if (ffn_norm_fused) rc = MESH_OK;
        else if (sk8) rc = quant16_k8(s->x, static_cast<const float *>(L.ffn_norm.data), hp.rms_eps, T, E, s->xq, stream);
        else if (k8) rc = rmsnorm_f16_k8(s->x, static_cast<const float *>(L.ffn_norm.data), hp.rms_eps, T, E, xn, stream, s->f16_sat);
        else rc = rmsnorm_f16(s->x, static_cast<const float *>(L.ffn_norm.data), hp.rms_eps, T, E, xn, E, stream, s->f16_sat);
    }
    if (rc != MESH_OK) return rc;
    if (sk16) {
        // gate and up in one pass with the SwiGLU epilogue, written as f16 straight into the down projection's input
        SkinnyF16Args ga;
        ga.n_mat = 2;
        ga.mat[0] = mat_of(L.w_gate, nullptr, FF, nullptr);
        ga.mat[1] = mat_of(L.w_up, nullptr, FF, nullptr);
        ga.x = xn; ga.K = E; ga.T = T; ga.epi = EPI_SWIGLU;
        ga.y16 = f16ffn;
        ga.sat = s->f16_sat;
        if (ffn_norm_fused) {
            ga.x = nx;
            ga.norm_in.part = s->norm_part; ga.norm_in.n_parts = s->norm_parts; ga.norm_in.eps = hp.rms_eps;
        }
        SkinnyF16Args da;
        da.n_mat = 1;
        da.mat[0] = mat_of(L.w_down, s->x, E, nullptr);
        da.x = f16ffn; da.K = FF; da.T = T;
        da.residual = s->x; da.ldres = E; da.epi = EPI_RESIDUAL;
        da.sat = s->f16_sat;
        // the next layer's attention norm, when that layer takes this path too
        const LayerWeights *Ln = il + 1 < st->layers.size() ? &st->layers[il + 1] : nullptr;
        const bool next_fused = nf && Ln && layer_is_kquant_dense(*Ln) && Ln->w_gate.type == Ln->w_up.type &&
                                gemm_skinny_f16_workgroups(da) >= 1 && gemm_skinny_f16_workgroups(da) <= SKINNY_F16_NORM_PARTS_MAX;
        ProfScope ps(s, MESH_PROF_GEMV);
        if ((rc = gemm_skinny_f16(ga, stream)) != MESH_OK) return rc;
        if (next_fused) {
            da.norm_out.norm_w = static_cast<const float *>(Ln->attn_norm.data); da.norm_out.x16 = nx; da.norm_out.part = s->norm_part;
        }
        if ((rc = gemm_skinny_f16(da, stream)) != MESH_OK) return rc;
        if (next_fused) { s->norm_parts = gemm_skinny_f16_workgroups(da); s->norm_layer = (int)il + 1; }
        return MESH_OK;
    }
    if (skinny) {
        // gate and up in one pass with the SwiGLU epilogue; its f32 output is quantised for the down projection
        SkinnyArgs ga;
        ga.n_mat = 2;
        ga.mat[0] = mat_of(L.w_gate, s->ffn, FF, nullptr);
        ga.mat[1] = mat_of(L.w_up, nullptr, FF, nullptr);
        ga.xq = s->xq; ga.K = E; ga.T = T; ga.epi = EPI_SWIGLU;
        SkinnyArgs da;
        da.n_mat = 1;
        da.mat[0] = mat_of(L.w_down, s->x, E, nullptr);
        da.xq = s->xq; da.K = FF; da.T = T;
        da.residual = s->x; da.ldres = E; da.epi = EPI_RESIDUAL;
        { ProfScope ps(s, MESH_PROF_GEMV); rc = gemm_skinny(ga, stream); }
        if (rc != MESH_OK) return rc;
        { ProfScope ps(s, MESH_PROF_PREP); rc = quant16_k8(s->ffn, nullptr, 0.f, T, FF, s->xq, stream); }
        if (rc != MESH_OK) return rc;
        ProfScope ps(s, MESH_PROF_GEMV);
        return gemm_skinny(da, stream);
    }
    if (L.gate_up_gemm && k8 && s->tune.gemm_fused) {
        // gate and up as one launch whose epilogue writes f16(silu(gate) * up) straight into the down projection's input
        ProfScope ps(s, MESH_PROF_GEMV);
        GemmArgs g = gemm_k8(gemm_of(L.w_gate, s->xn16, E, T, nullptr, FF, nullptr));
        g.Wp = L.gate_up_gemm;
        g.y16_k8 = f16ffn;
        if ((rc = gemm_kquant(g, stream)) != MESH_OK) return rc;
    } else {
        // (without the pair copy each matrix may still have its own GEMM-layout copy, or none)
        {
            ProfScope ps(s, MESH_PROF_GEMV);
            if ((rc = gemm_kquant(gemm_k8(gemm_of(L.w_gate, s->xn16, E, T, s->ffn, FF, nullptr)), stream)) != MESH_OK) return rc;
            if ((rc = gemm_kquant(gemm_k8(gemm_of(L.w_up, s->xn16, E, T, s->ffn_up, FF, nullptr)), stream)) != MESH_OK) return rc;
        }
        {
            ProfScope ps(s, MESH_PROF_PREP);
            if (k8) rc = swiglu_f16_k8(s->ffn, s->ffn_up, T, FF, f16ffn, stream, s->f16_sat);
            else rc = swiglu_f16(s->ffn, s->ffn_up, f16ffn, (int64_t)T * FF, stream, s->f16_sat);
        }
        if (rc != MESH_OK) return rc;
    }
    {
        ProfScope ps(s, MESH_PROF_GEMV);
        GemmArgs gd = gemm_k8(gemm_of(L.w_down, s->ffn16, FF, T, s->x, E, nullptr));
        gd.residual = s->x; gd.ldres = E;
        if ((rc = gemm_kquant(gd, stream)) != MESH_OK) return rc;
    }
    return MESH_OK;
}

// Runs the layers over the T token rows already in s->x.  pos/seq are on the device in s->d_pos / s->d_seq.
static int run_layers(mesh_session *s, int T, int max_keys) {
    mesh_stage *st = s->stage;
    const HParams &hp = st->hp;
    hipStream_t stream = s->stream;
    const int E = (int)hp.n_embd, QD = (int)(hp.n_head * hp.head_dim), KD = (int)(hp.n_head_kv * hp.head_dim);
    int rc;
    s->xq_layer = -1;
    s->norm_layer = -1;
    // a mixture-of-experts layer whose attention block runs on the batched-decode (integer matrix-core) path
    auto moe_attn_skinny = [&](const LayerWeights &Ln) {
        return !Ln.w_gate.present() && T >= std::min(PREFILL_MIN_TOKENS, s->tune.skinny_from()) && T < PREFILL_MIN_TOKENS && s->xn16 && layer_attn_is_kquant(Ln) &&
               hp.n_embd % 256 == 0 && (hp.n_head * hp.head_dim) % 256 == 0;
    };
    // the combine step at the end of a mixture-of-experts layer; when the next layer starts by quantising the new hidden
    // state for its projections, the same launch does that too (the same bits) and the layer finds them in s->xq
    auto combine = [&](size_t il, int top_k) {
        if (s->tune.moe_fuse_quant && il + 1 < st->layers.size() && moe_attn_skinny(st->layers[il + 1]) && moe_combine_quant16_supported(E)) {
            const int r = moe_combine_quant16(s->x, s->moe_out, s->moe_w, T, E, top_k, static_cast<const float *>(st->layers[il + 1].attn_norm.data), hp.rms_eps,
                                              s->xq, stream);
            if (r == MESH_OK) s->xq_layer = (int)il + 1;
            return r;
        }
        return moe_combine(s->x, s->moe_out, s->moe_w, T, E, top_k, stream);
    };
    for (size_t il = 0; il < st->layers.size(); ++il) {
        const LayerWeights &L = st->layers[il];
        if (T >= std::min(PREFILL_MIN_TOKENS, s->tune.skinny_from()) && s->xn16 && layer_is_kquant_dense(L) && hp.n_embd % 8 == 0 && hp.n_ff % 8 == 0) {
            // batches of decode steps of up to 32 tokens stay on the f16 skinny GEMM, two blocks of 16 columns per pass over
            // the weights (a prefill chunk of that length goes to the large-tile GEMM and the chunk attention)
            const bool wide = T >= PREFILL_MIN_TOKENS && T <= 32 && s->tune.skinny_f16 && s->tune.skinny_f16_wide && s->ffn16 && s->chunk_pos0 < 0;
            const bool skinny = (T < PREFILL_MIN_TOKENS || wide) && hp.n_embd % 256 == 0 && hp.n_ff % 256 == 0 && (hp.n_head * hp.head_dim) % 256 == 0 &&
                                L.w_gate.type == L.w_up.type;
            if (skinny || T >= PREFILL_MIN_TOKENS) {
                if ((rc = run_layer_prefill(s, L, il, T, max_keys, skinny, false)) != MESH_OK) return rc;
                continue;
            }
        }
        // a mixture-of-experts layer with many tokens: its attention block on the matrix cores, experts below
        bool attn_done = false;
        if (!L.w_gate.present() && T >= std::min(PREFILL_MIN_TOKENS, s->tune.skinny_from()) && s->xn16 && layer_attn_is_kquant(L) &&
            hp.n_embd % 256 == 0 && (hp.n_head * hp.head_dim) % 256 == 0) {
            if ((rc = run_layer_prefill(s, L, il, T, max_keys, T < PREFILL_MIN_TOKENS, true)) != MESH_OK) return rc;
            attn_done = true;
        }
        if (!attn_done) {
        // q, k, v = W{q,k,v} . rms_norm(x)
        GemvArgs qa;
        qa.n_mat = 3;
        qa.mat[0] = mat_of(L.wq, s->q, QD, &L.bq);
        qa.mat[1] = mat_of(L.wk, s->k, KD, &L.bk);
        qa.mat[2] = mat_of(L.wv, s->v, KD, &L.bv);
        qa.x = s->x; qa.ldx = E; qa.K = E; qa.T = T;
        qa.norm_w = static_cast<const float *>(L.attn_norm.data); qa.eps = hp.rms_eps;
        // neighbouring-pair RoPE into an f16 cache without per-head norms: rotation and KV append ride in the
        // projection's epilogue (the same arithmetic as rope_kv_kernel), one launch fewer per layer
        bool rope_fused = false;
        if (s->tune.gemv_rope && hp.rope_mode == ROPE_MODE_NORM && st->k_type == MESH_F16 && st->v_type == MESH_F16 && !L.q_norm.present() && !L.k_norm.present()) {
            qa.rope.pos = s->d_pos; qa.rope.seq = s->d_seq; qa.rope.inv_freq = st->rope_inv_freq;
            qa.rope.kcache = reinterpret_cast<uint16_t *>(s->kcache + il * s->k_layer_bytes);
            qa.rope.vcache = reinterpret_cast<uint16_t *>(s->vcache + il * s->v_layer_bytes);
            qa.rope.head_dim = (int)hp.head_dim; qa.rope.n_rot = (int)hp.n_rot; qa.rope.n_kv = (int)hp.n_head_kv; qa.rope.n_ctx = st->n_ctx;
            qa.kind[0] = GEMV_KIND_Q; qa.kind[1] = GEMV_KIND_K; qa.kind[2] = GEMV_KIND_V;
            rope_fused = gemv_can_fuse_rope(qa);
            if (!rope_fused) qa.rope = GemvRope{};
        }
        { ProfScope ps(s, MESH_PROF_GEMV); rc = gemv(qa, stream); }
        if (rc != MESH_OK) return rc;

        RopeKvArgs ra;
        ra.q = s->q; ra.k = s->k; ra.v = s->v;
        ra.kcache = s->kcache + il * s->k_layer_bytes;
        ra.vcache = s->vcache + il * s->v_layer_bytes;
        ra.k_type = st->k_type; ra.v_type = st->v_type;
        ra.pos = s->d_pos; ra.seq = s->d_seq; ra.inv_freq = st->rope_inv_freq;
        ra.q_norm = L.q_norm.present() ? static_cast<const float *>(L.q_norm.data) : nullptr;
        ra.k_norm = L.k_norm.present() ? static_cast<const float *>(L.k_norm.data) : nullptr;
        ra.eps = hp.rms_eps;
        ra.n_head = (int)hp.n_head; ra.n_kv = (int)hp.n_head_kv; ra.head_dim = (int)hp.head_dim;
        ra.n_rot = (int)hp.n_rot; ra.rope_mode = (int)hp.rope_mode; ra.n_ctx = st->n_ctx;
        if (!rope_fused) {
            ProfScope ps(s, MESH_PROF_ROPE);
            if ((rc = rope_kv(ra, T, stream)) != MESH_OK) return rc;
        }

        AttnArgs aa;
        aa.q = s->q; aa.kcache = ra.kcache; aa.vcache = ra.vcache; aa.k_type = st->k_type; aa.v_type = st->v_type; aa.pos = s->d_pos; aa.seq = s->d_seq;
        aa.part = s->attn_part; aa.ml = s->attn_ml; aa.out = s->attn;
        aa.scale = 1.0f / sqrtf((float)hp.head_dim);
        aa.n_head = (int)hp.n_head; aa.n_kv = (int)hp.n_head_kv; aa.group = (int)(hp.n_head / hp.n_head_kv);
        aa.head_dim = (int)hp.head_dim; aa.n_ctx = st->n_ctx;
        aa.n_splits = attn_splits_for(s->tune, T, (int)hp.n_head_kv, max_keys, st->k_type != MESH_F16);
        {
            ProfScope ps(s, MESH_PROF_ATTN);
            rc = T >= s->tune.attn_mma_min_tokens && attention_mma_supported(aa) ? attention_mma(aa, T, stream) : attention(aa, T, stream);
        }
        if (rc != MESH_OK) return rc;

        // x += Wo . attn
        GemvArgs oa;
        oa.n_mat = 1;
        oa.mat[0] = mat_of(L.wo, s->x, E, nullptr);
        oa.x = s->attn; oa.ldx = QD; oa.K = QD; oa.T = T;
        oa.residual = s->x; oa.ldres = E; oa.epi = EPI_RESIDUAL;
        { ProfScope ps(s, MESH_PROF_GEMV); rc = gemv(oa, stream); }
        if (rc != MESH_OK) return rc;
        }

        if (!L.w_gate.present()) {
            // mixture of experts: router -> top-k -> per-(token, slot) expert FFN -> weighted sum into x
            const int ne = (int)L.gate_inp.M, k = (int)hp.n_expert_used, ffe = (int)hp.n_ff_exp;
            MoeRouteArgs mr;
            mr.logits = s->moe_logits; mr.mask = s->expert_mask_on ? s->expert_mask : nullptr;
            mr.ids = s->moe_ids; mr.weights = s->moe_w; mr.n_expert = ne; mr.top_k = k; mr.norm_w = 1;
            const bool want_groups = s->tune.moe_group && moe_group_supported(T * k, ne) && moe_max_items(T * k, ne) <= 65535;
            // a batch of decode steps over K-quant experts: the expert products on the matrix cores, 16 pairs of an expert per pass
            // (worth it from about four pairs per expert: below that the mat-vec kernel, which only computes the columns an
            // item has, is as fast)
            const bool mfma = want_groups && s->xq && (size_t)T <= s->xq_tokens && T * k >= 4 * ne && E % 256 == 0 && ffe % 256 == 0 &&
                              type_is_tiled(L.gate_exps.type) && L.up_exps.type == L.gate_exps.type && type_is_tiled(L.down_exps.type) &&
                              moe_max_items(T * k, ne, SKINNY_ITEM_PAIRS) <= 65535;
            // a prefill chunk (from MOE_GEMM_MIN_PAIRS_PER_EXPERT pairs per expert on average): the pairs sorted by expert and
            // the expert products as tiles of the large-tile GEMM, up to 128 pairs of an expert per pass over its weights
            const bool big = s->moe_sorted.tiles && s->tune.moe_group && (size_t)T * k >= (size_t)MOE_GEMM_MIN_PAIRS_PER_EXPERT * ne &&
                             s->tune.moe_gemm && E % 256 == 0 && ffe % 256 == 0;
            if (big) {
                if (L.gate_inp.type == MESH_F32 && moe_router_fused_supported(E, ne, k)) {
                    ProfScope ps(s, MESH_PROF_GEMV);
                    if ((rc = moe_router_fused(mr, s->x, E, static_cast<const float *>(L.ffn_norm.data), hp.rms_eps,
                                               static_cast<const float *>(L.gate_inp.data), E, s->moe_logits, T, stream)) != MESH_OK) return rc;
                } else {
                    GemvArgs ra2;
                    ra2.n_mat = 1;
                    ra2.mat[0] = mat_of(L.gate_inp, s->moe_logits, ne, nullptr);
                    ra2.x = s->x; ra2.ldx = E; ra2.K = E; ra2.T = T;
                    ra2.norm_w = static_cast<const float *>(L.ffn_norm.data); ra2.eps = hp.rms_eps;
                    { ProfScope ps(s, MESH_PROF_GEMV); rc = gemv(ra2, stream); }
                    if (rc != MESH_OK) return rc;
                    if ((rc = moe_route(mr, T, stream)) != MESH_OK) return rc;
                }
                const int slots = moe_sort_slots(T * k, ne), max_tiles = moe_sort_max_tiles(T * k, ne);
                {
                    ProfScope ps(s, MESH_PROF_PREP);
                    if ((rc = moe_sort(s->moe_ids, T * k, ne, s->moe_sorted, stream)) != MESH_OK) return rc;
                    if ((rc = rmsnorm_f16_k8_gather(s->x, static_cast<const float *>(L.ffn_norm.data), hp.rms_eps, s->moe_sorted.pair_of_slot, k, slots, E,
                                                    reinterpret_cast<_Float16 *>(s->moe_x16), stream, s->f16_sat)) != MESH_OK) return rc;
                }
                const bool d_big = s->tune.gemm_big, d_narrow = s->tune.gemm_narrow;
                GemmArgs g;
                g.W = L.gate_exps.data; g.Wp = L.exps_gate_up_gemm; g.type = L.gate_exps.type;
                g.M = ffe; g.K = E; g.T = slots;
                g.X = reinterpret_cast<const _Float16 *>(s->moe_x16); g.ldx = E; g.x_k8 = true;
                g.y16_k8 = reinterpret_cast<_Float16 *>(s->moe_ffn16);
                g.sat = s->f16_sat;
                g.big_tile = d_big; g.narrow_tile = d_narrow;
                g.tiles = s->moe_sorted.tiles; g.n_tiles = s->moe_sorted.counts; g.max_tiles = max_tiles; g.expert_stride = L.exps_gate_up_stride;
                { ProfScope ps(s, MESH_PROF_GEMV); rc = gemm_kquant(g, stream); }
                if (rc != MESH_OK) return rc;
                GemmArgs d;
                d.W = L.down_exps.data; d.Wp = L.exps_down_gemm; d.type = L.down_exps.type;
                d.M = E; d.K = ffe; d.T = slots;
                d.X = reinterpret_cast<const _Float16 *>(s->moe_ffn16); d.ldx = ffe; d.x_k8 = true;
                d.Y = s->moe_out_slots; d.ldy = E;
                d.big_tile = d_big; d.narrow_tile = d_narrow;
                d.tiles = s->moe_sorted.tiles; d.n_tiles = s->moe_sorted.counts; d.max_tiles = max_tiles; d.expert_stride = L.exps_down_stride;
                { ProfScope ps(s, MESH_PROF_GEMV); rc = gemm_kquant(d, stream); }
                if (rc != MESH_OK) return rc;
                if ((rc = moe_combine_slots(s->x, s->moe_out_slots, s->moe_w, s->moe_sorted.slot_of_pair, T, E, k, stream)) != MESH_OK) return rc;
                continue;
            }
            const int item_pairs = mfma ? SKINNY_ITEM_PAIRS : MOE_ITEM_PAIRS;
            bool grouped_done = false;
            if (want_groups && L.gate_inp.type == MESH_F32 && moe_router_group_supported(E, ne, k, T)) {
                // a batch of decode steps: logits over many workgroups, then routing and grouping in one launch
                ProfScope ps(s, MESH_PROF_GEMV);
                if ((rc = moe_router_group(mr, s->x, E, static_cast<const float *>(L.ffn_norm.data), hp.rms_eps,
                                           static_cast<const float *>(L.gate_inp.data), E, s->moe_logits, T, s->moe_items, s->moe_n_items,
                                           item_pairs, stream, s->tune.moe_router_tail ? s->moe_arrive : nullptr)) != MESH_OK) return rc;
                grouped_done = true;
            } else if (L.gate_inp.type == MESH_F32 && moe_router_fused_supported(E, ne, k)) {
                // the router matrix is small and f32: logits and routing in one launch
                ProfScope ps(s, MESH_PROF_GEMV);
                if ((rc = moe_router_fused(mr, s->x, E, static_cast<const float *>(L.ffn_norm.data), hp.rms_eps,
                                           static_cast<const float *>(L.gate_inp.data), E, s->moe_logits, T, stream)) != MESH_OK) return rc;
            } else {
                GemvArgs ra2;
                ra2.n_mat = 1;
                ra2.mat[0] = mat_of(L.gate_inp, s->moe_logits, ne, nullptr);
                ra2.x = s->x; ra2.ldx = E; ra2.K = E; ra2.T = T;
                ra2.norm_w = static_cast<const float *>(L.ffn_norm.data); ra2.eps = hp.rms_eps;
                { ProfScope ps(s, MESH_PROF_GEMV); rc = gemv(ra2, stream); }
                if (rc != MESH_OK) return rc;
                if ((rc = moe_route(mr, T, stream)) != MESH_OK) return rc;
            }
            // pairs of one expert share a pass over its weights
            const bool grouped = want_groups;
            if (grouped && !grouped_done && (rc = moe_group(s->moe_ids, T * k, ne, s->moe_items, s->moe_n_items, item_pairs, stream)) != MESH_OK) return rc;
            if (mfma) {
                const int max_items = moe_max_items(T * k, ne, SKINNY_ITEM_PAIRS);
                { ProfScope ps(s, MESH_PROF_PREP); rc = quant16_k8(s->x, static_cast<const float *>(L.ffn_norm.data), hp.rms_eps, T, E, s->xq, stream); }
                if (rc != MESH_OK) return rc;
                SkinnyArgs ga;
                ga.n_mat = 2;
                ga.mat[0] = mat_of(L.gate_exps, s->ffn, ffe, nullptr);
                ga.mat[1] = mat_of(L.up_exps, nullptr, ffe, nullptr);
                ga.xq = s->xq; ga.K = E; ga.T = 1; ga.epi = EPI_SWIGLU;
                ga.items = s->moe_items; ga.n_items = s->moe_n_items; ga.max_items = max_items;
                ga.x_div = k;
                { ProfScope ps(s, MESH_PROF_GEMV); rc = gemm_skinny(ga, stream); }
                if (rc != MESH_OK) return rc;
                { ProfScope ps(s, MESH_PROF_PREP); rc = quant16_k8(s->ffn, nullptr, 0.f, T * k, ffe, s->xq, stream); }
                if (rc != MESH_OK) return rc;
                SkinnyArgs da;
                da.n_mat = 1;
                da.mat[0] = mat_of(L.down_exps, s->moe_out, E, nullptr);
                da.xq = s->xq; da.K = ffe; da.T = 1;
                da.items = s->moe_items; da.n_items = s->moe_n_items; da.max_items = max_items;
                da.x_div = 1;
                { ProfScope ps(s, MESH_PROF_GEMV); rc = gemm_skinny(da, stream); }
                if (rc != MESH_OK) return rc;
                if ((rc = combine(il, k)) != MESH_OK) return rc;
                continue;
            }
            GemvArgs ea;
            ea.n_mat = 2;
            ea.mat[0] = mat_of(L.gate_exps, s->ffn, ffe, nullptr);
            ea.mat[1] = mat_of(L.up_exps, nullptr, ffe, nullptr);
            ea.x = s->x; ea.ldx = E; ea.K = E; ea.T = 1;
            ea.norm_w = static_cast<const float *>(L.ffn_norm.data); ea.eps = hp.rms_eps;
            ea.epi = EPI_SWIGLU;
            ea.expert_ids = s->moe_ids; ea.n_pairs = T * k; ea.x_div = k;
            if (grouped) { ea.grouped_oversub = s->tune.grouped_oversub; ea.items = s->moe_items; ea.n_items = s->moe_n_items; ea.max_items = moe_max_items(T * k, ne); }
            { ProfScope ps(s, MESH_PROF_GEMV); rc = gemv(ea, stream); }
            if (rc != MESH_OK) return rc;
            GemvArgs xa;
            xa.n_mat = 1;
            xa.mat[0] = mat_of(L.down_exps, s->moe_out, E, nullptr);
            xa.x = s->ffn; xa.ldx = ffe; xa.K = ffe; xa.T = 1;
            xa.expert_ids = s->moe_ids; xa.n_pairs = T * k; xa.x_div = 1;
            if (grouped) { xa.grouped_oversub = s->tune.grouped_oversub; xa.items = s->moe_items; xa.n_items = s->moe_n_items; xa.max_items = ea.max_items; }
            { ProfScope ps(s, MESH_PROF_GEMV); rc = gemv(xa, stream); }
            if (rc != MESH_OK) return rc;
            if ((rc = combine(il, k)) != MESH_OK) return rc;
            continue;
        }
        // ffn = silu(Wgate . n) * (Wup . n),  n = rms_norm(x)
        GemvArgs ga;
        ga.n_mat = 2;
        ga.mat[0] = mat_of(L.w_gate, s->ffn, (int)hp.n_ff, nullptr);
        ga.mat[1] = mat_of(L.w_up, nullptr, (int)hp.n_ff, nullptr);
        ga.x = s->x; ga.ldx = E; ga.K = E; ga.T = T;
        ga.norm_w = static_cast<const float *>(L.ffn_norm.data); ga.eps = hp.rms_eps;
        ga.epi = EPI_SWIGLU;
        // x += Wdown . ffn
        GemvArgs da;
        da.n_mat = 1;
        da.mat[0] = mat_of(L.w_down, s->x, E, nullptr);
        da.x = s->ffn; da.ldx = (int)hp.n_ff; da.K = (int)hp.n_ff; da.T = T;
        da.residual = s->x; da.ldres = E; da.epi = EPI_RESIDUAL;
        // a single token: the gate / up launch leaves the FFN vector in the fixed-point form the down projection's
        // workgroups would each derive from it again (the same bits), and the down projection copies that
        if (s->ffn_xq && s->tune.xq_handover && gemv_xq_out_supported(ga) && gemv_xq_in_supported(da)) {
            ga.xq_out = s->ffn_xq;
            da.xq_in = s->ffn_xq;
        }
        { ProfScope ps(s, MESH_PROF_GEMV); rc = gemv(ga, stream); }
        if (rc != MESH_OK) return rc;

        { ProfScope ps(s, MESH_PROF_GEMV); rc = gemv(da, stream); }
        if (rc != MESH_OK) return rc;
    }
    return MESH_OK;
}

static int validate_batch(const mesh_session *s, const mesh_batch *b, int *max_keys) {
    const mesh_stage *st = s->stage;
    if (!b || b->n_tokens <= 0 || !b->pos) return fail(MESH_ERR_INVALID, "mesh_stage_decode: empty batch or null positions");
    if (b->n_tokens > st->n_batch_max) return fail(MESH_ERR_INVALID, "mesh_stage_decode: %d tokens exceed n_batch_max %d", b->n_tokens, st->n_batch_max);
    int mk = 0;
    for (int i = 0; i < b->n_tokens; ++i) {
        const int p = b->pos[i], q = b->seq_id ? b->seq_id[i] : 0;
        if (p < 0 || p >= st->n_ctx) return fail(MESH_ERR_INVALID, "mesh_stage_decode: position %d of token %d outside the context of %d", p, i, st->n_ctx);
        if (q < 0 || q >= st->n_seq_max) return fail(MESH_ERR_INVALID, "mesh_stage_decode: sequence id %d of token %d outside [0,%d)", q, i, st->n_seq_max);
        mk = std::max(mk, p + 1);
    }
    *max_keys = mk;
    return MESH_OK;
}

// run_layers, replayed from a captured graph for decode-sized batches.  The launches depend on T, on the KV split count
// (a function of the deepest position) and on whether an expert mask is set; everything else they read is device
// memory at fixed addresses (hidden state, positions, caches).  The first use of a key runs eagerly (which also
// finishes every lazy initialisation), the second is captured, later ones are replays.
constexpr int GRAPH_MAX_TOKENS = 32;
constexpr size_t GRAPH_MAX_ENTRIES = 96;
static int run_layers_graphed(mesh_session *s, int T, int max_keys) {
    if (!s->tune.graphs || s->graphs_failed || s->profile || T > GRAPH_MAX_TOKENS) return run_layers(s, T, max_keys);
    // A prefill chunk (consecutive positions of one sequence, enough tokens for the large-tile GEMM) runs the chunk
    // attention kernel, whose first position and sequence are launch arguments: a replay would carry the captured
    // chunk's.  Such calls are always launched eagerly.
    if (s->chunk_pos0 >= 0 && T >= PREFILL_MIN_TOKENS) return run_layers(s, T, max_keys);
    const mesh_stage *st = s->stage;
    const int n_splits = attn_splits_for(s->tune, T, (int)st->hp.n_head_kv, max_keys, st->k_type != MESH_F16);
    const uint64_t key = (uint64_t)T | ((uint64_t)n_splits << 8) | ((uint64_t)(s->expert_mask_on ? 1 : 0) << 20);
    auto it = s->graphs.find(key);
    if (it == s->graphs.end()) {
        if (s->graphs.size() >= GRAPH_MAX_ENTRIES) return run_layers(s, T, max_keys);
        it = s->graphs.emplace(key, mesh_session::LayerGraph{}).first;
    }
    mesh_session::LayerGraph &e = it->second;
    if (!e.exec) {
        if (e.uses++ == 0) return run_layers(s, T, max_keys);
        if (hipStreamBeginCapture(s->stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
            (void)hipGetLastError();
            s->graphs_failed = true;
            return run_layers(s, T, max_keys);
        }
        const int rc = run_layers(s, T, max_keys);           // records, does not execute
        hipGraph_t g = nullptr;
        hipError_t err = hipStreamEndCapture(s->stream, &g);
        if (rc == MESH_OK && err == hipSuccess && g) err = hipGraphInstantiate(&e.exec, g, nullptr, nullptr, 0);
        if (g) (void)hipGraphDestroy(g);
        if (rc != MESH_OK || err != hipSuccess || !e.exec) {
            (void)hipGetLastError();
            e.exec = nullptr;
            s->graphs_failed = true;
            return rc != MESH_OK ? rc : run_layers(s, T, max_keys);      // nothing has run yet
        }
    }
    MESH_HIP_TRY(hipGraphLaunch(e.exec, s->stream));
    ++s->graph_replays;
    return MESH_OK;
}

int stage_decode_dev(mesh_session *s, const mesh_batch *b, const void *d_in, int in_fmt, void *d_out, int out_fmt,
                     size_t out_cap, size_t *out_len) {
    if (!s || !d_in || !d_out) return fail(MESH_ERR_INVALID, "mesh_stage_decode: null argument");
    mesh_stage *st = s->stage;
    const HParams &hp = st->hp;
    int max_keys = 0, rc;
    if ((rc = validate_batch(s, b, &max_keys)) != MESH_OK) return rc;
    const int T = b->n_tokens;
    const bool tokens_in = in_fmt == MESH_TOKENS, logits_out = out_fmt == MESH_LOGITS;
    if (tokens_in && (st->layer_begin != 0 || !st->tok_embd.present()))
        return fail(MESH_ERR_INVALID, "mesh_stage_decode: token input needs a stage that starts at layer 0 of a file with token_embd");
    if (!tokens_in && in_fmt != MESH_F32 && in_fmt != MESH_F16 && in_fmt != MESH_Q8_0)
        return fail(MESH_ERR_INVALID, "mesh_stage_decode: input format %d unknown", in_fmt);
    if (logits_out && !st->output.present())
        return fail(MESH_ERR_INVALID, "mesh_stage_decode: logits output needs a stage that ends at the last layer of a file with output weights");
    if (!logits_out && out_fmt != MESH_F32 && out_fmt != MESH_F16 && out_fmt != MESH_Q8_0)
        return fail(MESH_ERR_INVALID, "mesh_stage_decode: output format %d unknown", out_fmt);
    const size_t need = logits_out ? (size_t)T * (size_t)st->output.M * 4 : mesh_act_packed_size(out_fmt, T, hp.n_embd);
    if (need == 0) return fail(MESH_ERR_INVALID, "mesh_stage_decode: n_embd %u is not a whole number of blocks of format %d", hp.n_embd, out_fmt);
    if (out_len) *out_len = need;
    if (out_cap < need) return fail(MESH_ERR_INVALID, "mesh_stage_decode: output needs %zu bytes, capacity is %zu", need, out_cap);
    MESH_HIP_TRY(hipSetDevice(st->device));
    hipStream_t stream = s->stream;

    // a run of consecutive positions of one sequence (a prefill chunk) can use the chunk attention kernel
    s->chunk_pos0 = b->pos[0];
    s->chunk_seq = b->seq_id ? b->seq_id[0] : 0;
    for (int i = 1; i < T && s->chunk_pos0 >= 0; ++i)
        if (b->pos[i] != b->pos[0] + i || (b->seq_id ? b->seq_id[i] : 0) != s->chunk_seq) s->chunk_pos0 = -1;
    // positions / sequence ids -> device, through a ring of pinned slots so calls may be queued back to back
    const size_t B = (size_t)st->n_batch_max;
    if (s->meta_counter && s->meta_counter % META_SLOTS == 0) MESH_HIP_TRY(hipStreamSynchronize(stream));   // ring wraps: older copies are done
    int32_t *slot = s->h_meta + (size_t)(s->meta_counter++ % META_SLOTS) * 3 * B;
    for (int i = 0; i < T; ++i) { slot[i] = b->pos[i]; slot[B + i] = b->seq_id ? b->seq_id[i] : 0; }
    // (one copy for both: the slot and the device buffer have the same layout, positions at 0 and sequence ids at B; a copy is
    // a launch of its own on the stream, and the entries between T and B are never read)
    MESH_HIP_TRY(hipMemcpyAsync(s->d_pos, slot, (B + T) * sizeof(int32_t), hipMemcpyHostToDevice, stream));

    if (tokens_in) {
        // embedding rows: one dequantize per token (ids are read on the host side by the caller's contract)
        return fail(MESH_ERR_UNSUPPORTED, "mesh_stage_decode_dev: token input is only available through the host-pointer entry point");
    }
    { ProfScope ps(s, MESH_PROF_CODEC); rc = act_unpack_dev(in_fmt, d_in, s->x, (int64_t)T * hp.n_embd, stream); }
    if (rc != MESH_OK) return rc;
    if ((rc = run_layers_graphed(s, T, max_keys)) != MESH_OK) return rc;
    if (logits_out) {
        GemvArgs la;
        la.n_mat = 1;
        la.mat[0] = mat_of(st->output, static_cast<float *>(d_out), (int)st->output.M, nullptr);
        la.x = s->x; la.ldx = (int)hp.n_embd; la.K = (int)hp.n_embd; la.T = T;
        la.norm_w = static_cast<const float *>(st->output_norm.data); la.eps = hp.rms_eps;
        ProfScope ps(s, MESH_PROF_GEMV);
        return gemv(la, stream);
    }
    ProfScope ps(s, MESH_PROF_CODEC);
    return act_pack_dev(out_fmt, s->x, d_out, (int64_t)T * hp.n_embd, stream);
}

int stage_decode(mesh_session *s, const mesh_batch *b, const void *in, int in_fmt, void *out, int out_fmt, size_t out_cap,
                 size_t *out_len) {
    if (!s || !in || !out) return fail(MESH_ERR_INVALID, "mesh_stage_decode: null argument");
    mesh_stage *st = s->stage;
    const HParams &hp = st->hp;
    if (!b || b->n_tokens <= 0) return fail(MESH_ERR_INVALID, "mesh_stage_decode: empty batch");
    if (b->n_tokens > st->n_batch_max) return fail(MESH_ERR_INVALID, "mesh_stage_decode: %d tokens exceed n_batch_max %d", b->n_tokens, st->n_batch_max);
    const int T = b->n_tokens;
    if (out_fmt == MESH_LOGITS && T > LOGITS_TOKENS_MAX)
        return fail(MESH_ERR_INVALID, "mesh_stage_decode: logits of %d tokens in one call (at most %d; mesh_stage_decode_dev has no such limit)", T, LOGITS_TOKENS_MAX);
    MESH_HIP_TRY(hipSetDevice(st->device));
    hipStream_t stream = s->stream;
    uint8_t *d_in = static_cast<uint8_t *>(s->io_stage), *d_out = d_in + s->io_stage_bytes;
    int rc;
    int eff_in_fmt = in_fmt;
    if (in_fmt == MESH_TOKENS) {
        if (st->layer_begin != 0 || !st->tok_embd.present())
            return fail(MESH_ERR_INVALID, "mesh_stage_decode: token input needs a stage that starts at layer 0 of a file with token_embd");
        const int32_t *ids = static_cast<const int32_t *>(in);
        const int64_t rb = row_bytes(st->tok_embd.type, hp.n_embd);
        for (int i = 0; i < T; ++i) {
            if (ids[i] < 0 || ids[i] >= st->tok_embd.M) return fail(MESH_ERR_INVALID, "mesh_stage_decode: token id %d outside the vocabulary of %lld", ids[i], (long long)st->tok_embd.M);
            rc = dequantize_dev(st->tok_embd.type, static_cast<const uint8_t *>(st->tok_embd.data) + (size_t)ids[i] * rb,
                                reinterpret_cast<float *>(d_in) + (size_t)i * hp.n_embd, hp.n_embd, stream);
            if (rc != MESH_OK) return rc;
        }
        eff_in_fmt = MESH_F32;
    } else {
        const size_t in_bytes = mesh_act_packed_size(in_fmt, T, hp.n_embd);
        if (in_bytes == 0) return fail(MESH_ERR_INVALID, "mesh_stage_decode: input format %d unknown or n_embd not a whole number of blocks", in_fmt);
        memcpy(s->h_io, in, in_bytes);
        MESH_HIP_TRY(hipMemcpyAsync(d_in, s->h_io, in_bytes, hipMemcpyHostToDevice, stream));
    }
    size_t len = 0;
    if ((rc = stage_decode_dev(s, b, d_in, eff_in_fmt, d_out, out_fmt, std::min(out_cap, s->io_out_bytes), &len)) != MESH_OK) {
        if (out_len) *out_len = len;
        return rc;
    }
    if (out_len) *out_len = len;
    uint8_t *h_out = static_cast<uint8_t *>(s->h_io) + s->io_stage_bytes;
    MESH_HIP_TRY(hipMemcpyAsync(h_out, d_out, len, hipMemcpyDeviceToHost, stream));
    MESH_HIP_TRY(hipStreamSynchronize(stream));
    memcpy(out, h_out, len);
    return MESH_OK;
}

// ---- single graph nodes -------------------------------------------------------------------------
// Decode attention of one layer over the session's KV cache, for callers that bring their own (already rotated) queries.
int session_attention(mesh_session *s, int layer, const float *d_q, const mesh_batch *b, float *d_out, int matrix_cores) {
    const mesh_stage *st = s->stage;
    const HParams &hp = st->hp;
    const int il = layer - st->layer_begin;
    if (il < 0 || il >= (int)st->layers.size()) return fail(MESH_ERR_INVALID, "mesh_session_attn_dev: layer %d is not in this stage", layer);
    const int T = b->n_tokens;
    if (T < 1 || T > st->n_batch_max || !b->pos) return fail(MESH_ERR_INVALID, "mesh_session_attn_dev: bad batch");
    int max_keys = 0;
    std::vector<int32_t> seq((size_t)T, 0);
    for (int i = 0; i < T; ++i) {
        if (b->seq_id) seq[i] = b->seq_id[i];
        if (b->pos[i] < 0 || b->pos[i] >= st->n_ctx || seq[i] < 0 || seq[i] >= st->n_seq_max)
            return fail(MESH_ERR_INVALID, "mesh_session_attn_dev: token %d has position %d / sequence %d outside the cache", i, b->pos[i], seq[i]);
        max_keys = std::max(max_keys, b->pos[i] + 1);
    }
    MESH_HIP_TRY(hipStreamSynchronize(s->stream));
    MESH_HIP_TRY(hipMemcpy(s->d_pos, b->pos, (size_t)T * sizeof(int32_t), hipMemcpyHostToDevice));
    MESH_HIP_TRY(hipMemcpy(s->d_seq, seq.data(), (size_t)T * sizeof(int32_t), hipMemcpyHostToDevice));
    AttnArgs aa;
    aa.q = d_q;
    aa.kcache = s->kcache + il * s->k_layer_bytes;
    aa.vcache = s->vcache + il * s->v_layer_bytes;
    aa.k_type = st->k_type; aa.v_type = st->v_type; aa.pos = s->d_pos; aa.seq = s->d_seq;
    aa.part = s->attn_part; aa.ml = s->attn_ml; aa.out = d_out;
    aa.scale = 1.0f / sqrtf((float)hp.head_dim);
    aa.n_head = (int)hp.n_head; aa.n_kv = (int)hp.n_head_kv; aa.group = (int)(hp.n_head / hp.n_head_kv);
    aa.head_dim = (int)hp.head_dim; aa.n_ctx = st->n_ctx;
    aa.n_splits = T < 64 ? attn_splits_for(s->tune, T, (int)hp.n_head_kv, max_keys, st->k_type != MESH_F16) : 1;
    if (matrix_cores) {
        if (!attention_mma_supported(aa)) return fail(MESH_ERR_UNSUPPORTED, "mesh_session_attn_dev: the matrix-core kernel does not cover this shape");
        return attention_mma(aa, T, s->stream);
    }
    return attention(aa, T, s->stream);
}

}  // namespace mesh

mesh_stage::~mesh_stage() {
    for (void *p : allocations) (void)hipFree(p);
}

mesh_session::~mesh_session() {
    if (stream) (void)hipStreamSynchronize(stream);
    for (hipEvent_t e : prof_events) (void)hipEventDestroy(e);
    for (void *p : allocations) (void)hipFree(p);
    for (auto &kv : graphs)
        if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
    if (h_meta) (void)hipHostFree(h_meta);
    if (h_io) (void)hipHostFree(h_io);
    if (stream) (void)hipStreamDestroy(stream);
}
