// RoPE + KV append and GQA attention launchers (attn.hip).
#pragma once

#include "kv_cache.hpp"
#include "mesh_common.hpp"

namespace mesh {

constexpr int ROPE_MODE_NORM = 0, ROPE_MODE_NEOX = 2;
constexpr int ATTN_SPLITS_CAP = 64;     // most KV splits per (token, kv head)

struct RopeKvArgs {
    float *q = nullptr;            // [T][n_head][head_dim], rotated in place
    const float *k = nullptr;      // [T][n_kv][head_dim]
    const float *v = nullptr;
    uint8_t *kcache = nullptr;     // this layer's K: [n_seq][n_kv][n_ctx] rows of k_type (kv_cache.hpp)
    uint8_t *vcache = nullptr;
    int k_type = MESH_F16, v_type = MESH_F16;
    const int32_t *pos = nullptr;  // device, [T]
    const int32_t *seq = nullptr;  // device, [T]
    const float *inv_freq = nullptr;   // device, [n_rot/2]
    const float *q_norm = nullptr; // optional per-head RMS norm weights [head_dim]
    const float *k_norm = nullptr;
    float eps = 0.f;
    int n_head = 0, n_kv = 0, head_dim = 0, n_rot = 0, rope_mode = ROPE_MODE_NORM, n_ctx = 0;
};
int rope_kv(const RopeKvArgs &a, int T, hipStream_t stream);

struct AttnArgs {
    const float *q = nullptr;      // [T][n_head][head_dim]
    const uint8_t *kcache = nullptr, *vcache = nullptr;    // rows of k_type / v_type
    int k_type = MESH_F16, v_type = MESH_F16;              // (f16, f16), (q8_0, q4_0) or (q4_0, q4_0)
    const int32_t *pos = nullptr, *seq = nullptr;
    float *part = nullptr;         // [T][n_head][n_splits][head_dim]
    float *ml = nullptr;           // [T][n_head][n_splits][2]
    size_t part_rows = 0;          // attention_chunk only: (token, split) rows part / ml have room for (0: it never splits the keys)
    float *out = nullptr;          // [T][n_head][head_dim]
    // attention_mma only: when set, the result is written as f16 in the k8-major activation layout of the batched GEMM
    // (gemm.hpp; row length n_head * head_dim) INSTEAD of `out`, so the output projection can read it as it is
    _Float16 *out16_k8 = nullptr;
    // or, when set, quantised into the q16 activation layout of the skinny GEMM (gemm.hpp), also instead of `out`
    uint8_t *out_q16 = nullptr;
    // attention_chunk only, optional: scratch of 2 * n_kv * n_ctx * head_dim f16 values; with it a long chunk over a
    // quantised cache decodes the rows it needs once, into the scratch, instead of once per query tile
    _Float16 *chunk_kv16 = nullptr;
    float scale = 1.f;
    int n_head = 0, n_kv = 0, group = 1, head_dim = 0, n_ctx = 0, n_splits = 1;
};
// token t attends to cache positions [0, pos[t]] of sequence seq[t]
int attention(const AttnArgs &a, int T, hipStream_t stream);
// merge of the split partials (a.part, a.ml) into a.out; a no-op contract for n_splits == 1 is the caller's business
int attention_combine(const AttnArgs &a, int T, hipStream_t stream);
// The same attention with the query heads of a KV head as the columns of matrix-core tiles (attn_mma.hip): per-key
// cost independent of the group size; Q and the probabilities rounded to f16.  For batches of decode tokens.
bool attention_mma_supported(const AttnArgs &a);
int attention_mma(const AttnArgs &a, int T, hipStream_t stream);
// The same for a chunk of T consecutive positions pos0 .. pos0 + T - 1 of one sequence, on the matrix cores
// (attn_prefill.hip; head_dim 128).  a.pos / a.seq / a.part / a.ml are not used.
int attention_chunk(const AttnArgs &a, int T, int pos0, int seq, hipStream_t stream);
bool kv_pair_supported(int k_type, int v_type);

// f16 <-> cache rows for mesh_session_kv_write / _read: `half` is a device buffer [n_pos][n_kv][head_dim] of f16
// bits, `cache` one layer's K or V rows; positions pos0 .. pos0 + n_pos - 1 of sequence seq.
int kv_import(int type, uint8_t *cache, const uint16_t *half, int n_kv, int n_ctx, int head_dim, int seq, int pos0, int n_pos, hipStream_t stream);
int kv_export(int type, const uint8_t *cache, uint16_t *half, int n_kv, int n_ctx, int head_dim, int seq, int pos0, int n_pos, hipStream_t stream);

}  // namespace mesh
