// Internal types of the stage executor: hyper-parameters, device-resident weights, session state.
#pragma once

#include <memory>
#include <unordered_map>
#include <string>
#include <vector>

#include "gguf.hpp"
#include "mesh_common.hpp"
#include "moe.hpp"
#include "tuning.hpp"

namespace mesh {

enum RopeMode { ROPE_NORM = 0, ROPE_NEOX = 2 };

struct HParams {
    std::string arch;
    uint32_t n_layer = 0, n_embd = 0, n_head = 0, n_head_kv = 0, head_dim = 0, n_ff = 0, n_vocab = 0;
    uint32_t n_rot = 0, rope_mode = ROPE_NORM;
    uint32_t n_expert = 0, n_expert_used = 0, n_ff_exp = 0;
    float rms_eps = 1e-5f, rope_freq_base = 10000.0f;
};

// Fills `hp` from the GGUF key/value table (keys of the form "<arch>.block_count", ...).
int hparams_from_gguf(const GgufFile &g, HParams &hp);

// A weight matrix resident in HBM.  K-quant matrices are stored in the tiled layout of gemv.hip
// (same byte count as the GGUF tensor); everything else keeps the GGUF row-major layout.
struct DevTensor {
    void *data = nullptr;
    void *gemm = nullptr;   // K-quant projections of stages that can take prefill-sized calls: second copy in the GEMM layout (gemm.hpp)
    int type = -1;
    int64_t K = 0;       // row length (ggml ne[0])
    int64_t M = 0;       // rows (ggml ne[1]); for 1-D tensors M = 1
    int64_t E = 1;       // stacked expert matrices (ggml ne[2])
    size_t bytes = 0;
    bool tiled = false;
    bool present() const { return data != nullptr; }
};

struct LayerWeights {
    DevTensor attn_norm, wq, wk, wv, wo, bq, bk, bv, q_norm, k_norm;
    DevTensor ffn_norm, w_gate, w_up, w_down;
    DevTensor gate_inp, gate_exps, up_exps, down_exps;   // MoE
    // GEMM-layout copies (gemm.hpp) beyond the per-tensor ones: wq / wk (/ wv) of one K-quant type sit back to back in
    // one buffer (qkv_fused = 2 or 3 matrices; their .gemm pointers point into it), and gate / up of one type are
    // packed as a SwiGLU pair.
    int qkv_fused = 0;
    void *gate_up_gemm = nullptr;
    // mixture of experts: every expert's gate / up pair and down projection in the GEMM layout, experts back to back
    void *exps_gate_up_gemm = nullptr, *exps_down_gemm = nullptr;
    size_t exps_gate_up_stride = 0, exps_down_stride = 0;
};

}  // namespace mesh

namespace mesh {
int stage_open(const char *path, int layer_begin, int layer_end, const mesh_stage_opts *opts, mesh_stage **out);
int session_new(mesh_stage *st, mesh_session **out);
int stage_decode(mesh_session *s, const mesh_batch *b, const void *in, int in_fmt, void *out, int out_fmt, size_t out_cap, size_t *out_len);
int profile_collect(mesh_session *s);
int session_attention(mesh_session *s, int layer, const float *d_q, const mesh_batch *b, float *d_out, int matrix_cores);
int stage_decode_dev(mesh_session *s, const mesh_batch *b, const void *d_in, int in_fmt, void *d_out, int out_fmt, size_t out_cap, size_t *out_len);
}  // namespace mesh

struct mesh_stage {
    mesh::HParams hp;
    int device = 0;
    int k_type = MESH_F16, v_type = MESH_F16;          // KV cache row types
    int layer_begin = 0, layer_end = 0;
    int n_ctx = 0, n_seq_max = 1, n_batch_max = 0;
    mesh::Tuning tune;            // process default, then mesh_stage_opts.tuning; fixed from here on
    std::vector<mesh::LayerWeights> layers;
    mesh::DevTensor tok_embd, output_norm, output;
    std::vector<void *> allocations;
    size_t gemm_layout_bytes = 0; // extra HBM held by the GEMM-layout copies
    size_t weight_bytes = 0;      // GGUF bytes of everything resident (the algorithmic weight traffic of one decode step)
    float *rope_inv_freq = nullptr;   // [n_rot/2] f32, theta_scale^i by the f32 recurrence ggml uses
    ~mesh_stage();
};

struct mesh_session {
    mesh_stage *stage = nullptr;
    hipStream_t stream = nullptr;
    mesh::Tuning tune;            // starts as the stage's copy; mesh_session_set_option changes the session-level switches
    bool graphs_failed = false;   // a failed capture turns graph replay off for the rest of the session
    // KV cache: per local layer, K and V as f16 [n_seq_max][n_head_kv][n_ctx][head_dim]
    uint8_t *kcache = nullptr, *vcache = nullptr;       // rows of the stage's k_type / v_type (kv_cache.hpp)
    size_t k_layer_bytes = 0, v_layer_bytes = 0;
    // activations (f32), sized for n_batch_max tokens
    float *x = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr, *ffn = nullptr;
    uint8_t *ffn_xq = nullptr;                          // single-token decode: the FFN vector as its producer quantised it (gemv.hpp: xq layout)
    unsigned *f16_sat = nullptr;                        // device counter: values the f16 producers of the batched paths clamped to +-65504
    uint32_t f16_sat_seen = 0;                          // device counter at its last read
    uint64_t f16_sat_total = 0;                         // running total the ABI reports
    float *attn_part = nullptr, *attn_ml = nullptr;     // split-KV partial outputs and (max, sum) pairs
    size_t attn_part_rows = 0;                          // (token, split) rows they hold
    // prefill path (many tokens per call): f16 copies of the GEMM inputs and a second FFN buffer
    uint16_t *xn16 = nullptr, *ffn16 = nullptr;
    // f16 skinny GEMM with the RMS norms handed over between launches (gemm.hpp: SkinnyF16Args::NormOut): the next norm's
    // input as its producer wrote it, the producer's partial sums of squares, and whose input that is
    uint16_t *norm16 = nullptr;
    float *norm_part = nullptr;
    int norm_parts = 0;              // partial sums per token the last producer wrote
    int norm_layer = -1;             // layer whose attention norm norm16 / norm_part hold (-1: none)
    uint16_t *chunk_kv16 = nullptr;      // quantised KV caches: f16 rows of one sequence and layer for long prefill chunks (attn.hpp)
    size_t xq_tokens = 0;               // tokens the q16 buffer below is sized for
    uint8_t *xq = nullptr;               // 16-bit fixed-point activations of the skinny GEMM (gemm.hpp: q16 layout)
    float *gemm_part = nullptr;          // partial tiles of large-tile GEMM launches that split K (gemm.hpp)
    size_t gemm_part_bytes = 0;
    float *ffn_up = nullptr;
    float *moe_logits = nullptr, *moe_w = nullptr, *moe_out = nullptr, *expert_mask = nullptr;
    bool expert_mask_on = false;
    int32_t *moe_ids = nullptr;
    int32_t *moe_items = nullptr, *moe_n_items = nullptr;      // (token, slot) pairs grouped by expert, see moe_group
    int *moe_arrive = nullptr;                                 // arrival counter of the fused router launch (zero between launches)
    // prefill chunks: the pairs sorted by expert (moe_sort) and their buffers, rows indexed by slot
    mesh::MoeSorted moe_sorted;
    uint16_t *moe_x16 = nullptr, *moe_ffn16 = nullptr;          // k8-major f16: normalised inputs, SwiGLU outputs
    float *moe_out_slots = nullptr;                            // down-projection rows
    int xq_layer = -1;               // layer whose attention-norm activations the previous layer's combine step has left in xq (-1: none)
    int32_t *d_pos = nullptr, *d_seq = nullptr, *d_tok = nullptr;
    int32_t *h_meta = nullptr;      // pinned staging for pos/seq/token ids (ring of slots)
    unsigned meta_counter = 0;
    void *io_stage = nullptr;       // device staging for packed in/out of the host-pointer entry point
    size_t io_stage_bytes = 0;      // input half; the output half (io_out_bytes) follows it
    size_t io_out_bytes = 0;
    void *h_io = nullptr;           // pinned host staging, same split
    int attn_splits_max = 0;
    // set per call: the batch is one run of consecutive positions of one sequence (first position, sequence), else -1
    int chunk_pos0 = -1, chunk_seq = -1;
    std::vector<void *> allocations;
    // optional per-kernel-class timing (HIP events on `stream` around every launch group)
    bool profile = false;
    // Captured launch sequences of run_layers, one per (token count, KV split count, expert mask) seen: a decode step
    // is ~80 dependent launches; replaying them as a graph takes the host out of their submission (about 0.3 ms of CPU
    // per step).  Off by default: on the measured system the stream is GPU-bound and the step time does not change.
    struct LayerGraph { hipGraphExec_t exec = nullptr; int uses = 0; };
    std::unordered_map<uint64_t, LayerGraph> graphs;
    int64_t graph_replays = 0;
    std::vector<hipEvent_t> prof_events;      // pairs (begin, end)
    std::vector<int> prof_kinds;
    size_t prof_used = 0;
    double prof_ms[MESH_PROF_KINDS] = {};
    uint64_t prof_launches[MESH_PROF_KINDS] = {};
    ~mesh_session();
};
