/*
 * mesh_oracle.h -- CPU restatement of the arithmetic a mesh-llm pipeline stage runs.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, its C ABI, the
 * Python host mirror) may include, link or call this file; only tests/, the smoke
 * check and the cpu_baseline leg of bench.py do, and only as the checker.
 *
 * Provenance.  mesh-llm holds no inference arithmetic: it launches llama.cpp
 * (third_party/llama.cpp/upstream.txt:1 pins ggml-org/llama.cpp @ 45155597aa23243c5f6d10064bd9bca3eaddee16,
 * fetched at build time by scripts/prepare-llama.sh:26-29, NOT vendored).  The
 * routines below restate ggml's published block formats and reference routines
 * (quantize_row_q8_0_ref, dequantize_row_q8_0/q4_K/q6_K/q5_0, ggml_fp32_to_fp16_row,
 * rms_norm, rope, soft_max/flash_attn_ext, swiglu) as they are reached from the
 * reference's call sites:
 *   third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451  (graph_compute)
 *   third_party/llama.cpp/patches/0002-...:544-622  (boundary tensor push, ggml_nbytes sizing :243)
 *   third_party/llama.cpp/patches/0001-rpc-optimize-local-GGUF-tensor-loading.patch:179-266 (tensor-by-name load)
 *   third_party/llama.cpp/patches/0003-moe-add-expert-analysis-and-split-tools.patch:82-108 (expert mask + top-k)
 *   mesh-llm/src/inference/launch.rs:1350-1353 (-ngl 99 -fa on), :568-591 (KV cache types)
 *
 * PARITY UNPINNED against ggml itself: no ggml source, binary or golden vector is
 * available offline, so every function here is pinned only by what the mathematics
 * fixes (IEEE binary16 via numpy, hand-packed known-answer blocks, closed forms,
 * torch float64 library routines, brute force on tiny inputs) -- see tests/test_oracle_*.py.
 */
#ifndef MESH_ORACLE_H
#define MESH_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids used by a Q4_K_M file, plus Q4_0 (a KV cache type of mesh-llm/src/inference/launch.rs:568-591) */
enum { MO_F32 = 0, MO_F16 = 1, MO_Q4_0 = 2, MO_Q5_0 = 6, MO_Q8_0 = 8, MO_Q4_K = 12, MO_Q6_K = 14 };
/* rope pairings */
enum { MO_ROPE_NORM = 0, MO_ROPE_NEOX = 2 };

/* --- fp16 --- */
uint16_t mo_fp32_to_fp16(float f);
float    mo_fp16_to_fp32(uint16_t h);
void     mo_fp32_to_fp16_row(const float *x, uint16_t *y, int64_t n);
void     mo_fp16_to_fp32_row(const uint16_t *x, float *y, int64_t n);

/* --- block formats --- */
int64_t  mo_block_elems(int type);
int64_t  mo_block_bytes(int type);
int64_t  mo_row_bytes(int type, int64_t k);              /* -1 if k is not a whole number of blocks */
void     mo_quantize_row_q8_0(const float *x, void *y, int64_t k);
void     mo_quantize_row_q4_0(const float *x, void *y, int64_t k);
int      mo_dequantize_row(int type, const void *x, float *y, int64_t k);   /* 0 ok, -1 bad type/size */

/* --- operators --- */
/* y[t*M+m] = sum_k W[m,k] x[t*K+k] (+ bias[m]); W in `type` blocks, row-major, f64 accumulate */
int  mo_mul_mat(int type, const void *W, int64_t M, int64_t K,
                const float *x, int64_t T, const float *bias, float *y);
/* y = x * rsqrt(mean(x^2)+eps) * w, rows of n */
void mo_rms_norm(const float *x, const float *w, float eps, int64_t n, int64_t T, float *y);
/* in-place rotary embedding on x[T][n_head][head_dim], first n_rot dims of each head */
void mo_rope(float *x, int64_t T, int n_head, int head_dim, int n_rot,
             const int32_t *pos, float freq_base, int mode);
/* out[i] = silu(gate[i]) * up[i] */
void mo_swiglu(const float *gate, const float *up, float *out, int64_t n);
/* causal GQA attention of one query token over an f16 KV cache laid out [n_kv][ctx_stride][head_dim];
 * attends to cache positions [0, n_past] inclusive.  q: [n_head][head_dim], out same shape. */
void mo_attn_token(const float *q, const uint16_t *kcache, const uint16_t *vcache,
                   int n_head, int n_kv, int head_dim, int64_t ctx_stride, int64_t n_past,
                   float scale, float *out);
/* the same over caches held as f32 values (what a q8_0 / q4_0 cache dequantises to) */
void mo_attn_token_f32(const float *q, const float *kcache, const float *vcache,
                       int n_head, int n_kv, int head_dim, int64_t ctx_stride, int64_t n_past,
                       float scale, float *out);
/* MoE router: probs = softmax(logits) over n_expert; top-k ids by (probs + mask), mask 0 / -inf (ties: lower id
 * first); weights = unmasked probs of the selected experts, optionally renormalised to sum 1. */
void mo_moe_route(const float *logits, const float *mask, int n_expert, int top_k, int norm_w,
                  int32_t *ids, float *weights);

void mo_set_threads(int n);
int  mo_get_threads(void);

#ifdef __cplusplus
}
#endif
#endif
