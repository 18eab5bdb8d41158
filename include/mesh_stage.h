/*
 * mesh_stage.h -- C ABI of the MI355X pipeline-stage executor (libmeshstage.so).
 *
 * This is the surface a thin Rust `*-ffi` crate binds (plain pointers and sizes, no C++ or
 * framework types).  It stands where mesh-llm reaches llama.cpp for the work one node does when a
 * dense model is split by layers: run a contiguous layer range of a GGUF Q4_K_M model and hand the
 * boundary hidden state to the next stage.  Each entry point cites the reference interface it
 * replaces (paths relative to the mesh-llm tree).
 *
 * Conventions (copied from the reference's FFI layer): every call returns 0 on success or a
 * negative mesh_status; nothing throws across the boundary and no strings are returned by value
 * (mesh-api-ffi/src/lib.rs:12-32, mesh-api-ffi/tests/error_mapping.rs:14-20); the message for the
 * last failure on the calling thread is read with mesh_last_error().  Handles are opaque and are
 * released only by their own close/free call (mesh-api-ffi/src/lib.rs:107-111,269-276).  A
 * mesh_stage is immutable after open; a mesh_session is single-threaded, like the single
 * backend_mutex the reference holds around every backend call
 * (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:324).
 */
#ifndef MESH_STAGE_H
#define MESH_STAGE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mesh_status {
    MESH_OK = 0,
    MESH_ERR_INVALID = -1,     /* bad argument (null pointer, size not a whole number of blocks, ...) */
    MESH_ERR_DEVICE = -2,      /* HIP runtime error or no usable GPU */
    MESH_ERR_NOMEM = -3,
    MESH_ERR_IO = -4,          /* file could not be opened / read */
    MESH_ERR_FORMAT = -5,      /* not a GGUF file, or tensor metadata inconsistent */
    MESH_ERR_UNSUPPORTED = -6  /* tensor type / architecture this build has no kernel for */
} mesh_status;

/* Activation / tensor element formats.  Values are ggml type ids, because the boundary tensor is a ggml
 * tensor in the reference (patches/0002:59-80 rpc_tensor.type; today always F32, patches/0002:238-243). */
typedef enum mesh_dtype {
    MESH_F32 = 0,
    MESH_F16 = 1,
    MESH_Q4_0 = 2,
    MESH_Q5_0 = 6,
    MESH_Q8_0 = 8,
    MESH_Q4_K = 12,
    MESH_Q6_K = 14
} mesh_dtype;

/* Message of the last failing call on this thread ("" if none).  Pointer stays valid until the next
 * failing call on the same thread.  Mirrors the FfiError message (mesh-api-ffi/src/lib.rs:12-32). */
const char *mesh_last_error(void);

/* Number of usable GPUs (0 if none).  Stands in for `rpc-server -d <bogus>` printing "available devices:"
 * (mesh-llm/src/inference/launch.rs:768-782). */
int mesh_device_count(void);

/* Select the GPU for the calling thread.  Accepts "ROCm0", "HIP0" or "0" (either spelling, as
 * mesh-llm/src/inference/launch.rs:812-823 does). */
int mesh_device_select(const char *device);

/* Streaming-read bandwidth of the current GPU: `timed_runs` event-timed passes over a zero-filled buffer of `bytes`
 * (after `warmup_runs` untimed ones), GB/s of each pass into gbps[timed_runs].  The protocol of the reference's GPU
 * fingerprint benchmark (mesh-llm/benchmarks/membench-fingerprint.hip:24-39,151-160: 512 MiB, 3 + 20 runs, p50 / p90
 * taken by the caller; its output feeds mesh-llm/src/system/benchmark.rs:11-29). */
int mesh_hbm_read_probe(size_t bytes, int warmup_runs, int timed_runs, double *gbps);

/* Plain streaming kernel of a given traffic shape, the yardstick for the codec kernels: moves `big_bytes` on the
 * larger side (read if big_is_read, else written) and big_bytes / ratio on the other (ratio 1, 2 or 4), non-temporal
 * 16-byte vectors, queued on `stream` and not waited for; the caller times it like any other launch.  big_bytes must be
 * a multiple of 4096 * ratio.  Same purpose as mesh_hbm_read_probe (mesh-llm/benchmarks/membench-fingerprint.hip:24-39),
 * for kernels that write as well as read. */
int mesh_hbm_mix_probe_dev(const void *d_src, void *d_dst, size_t big_bytes, int ratio, int big_is_read, void *stream);

/* Sustained f16 matrix-core rate of the current GPU: `timed_runs` event-timed launches (after `warmup_runs` untimed
 * ones) of a kernel in which every wave issues `iters` x 4 independent v_mfma_f32_32x32x16_f16 from registers, four
 * waves per SIMD; TFLOP/s of each launch into tflops[timed_runs].  The yardstick for the prefill GEMM beside the
 * nominal 2.5 PFLOP/s: it shows the clock the chip holds with the matrix pipes saturated.  No counterpart in the
 * reference (its fingerprint benchmark, mesh-llm/benchmarks/membench-fingerprint.hip, measures memory only). */
int mesh_mfma_f16_probe(int iters, int warmup_runs, int timed_runs, double *tflops);

/* ---- boundary activation codec -------------------------------------------------------------------
 * The inter-stage hidden state [n_tokens, n_embd] f32, packed for transport.  Replaces the raw-f32
 * ggml_backend_tensor_get -> TCP -> ggml_backend_tensor_set hop of push_tensor_to_peer
 * (patches/0002:544-622,693-705) with the stage wire formats planned in
 * mesh-llm/docs/LLAMA_STAGE_INTEGRATION_PLAN.md:345-362: f16, or q8_0 blocks {fp16 d; int8 qs[32]}
 * produced exactly as ggml's quantize_row_q8_0_ref / ggml_fp32_to_fp16_row would. */

/* Bytes of n_tokens*n_embd elements in `fmt` (ggml_nbytes, patches/0002:243); 0 if fmt is not an
 * activation format or the count is not a whole number of blocks. */
size_t mesh_act_packed_size(int fmt, int64_t n_tokens, int64_t n_embd);

/* Host-pointer forms: n elements, src/dst in host memory (staged through the GPU). */
int mesh_act_pack(int fmt, const float *src, void *dst, int64_t n);
int mesh_act_unpack(int fmt, const void *src, float *dst, int64_t n);

/* mesh_act_pack for callers that cannot allocate GPU memory (a serving loop that packs the boundary activation of
 * every decode step, a harness that forbids hipMalloc): same arguments, same bytes out, but the device staging of
 * the input and the packed output is a fixed array inside the library instead of two allocations per call.  No
 * counterpart in the reference.  Limits: n <= 1 048 576 elements (256 tokens of 4096), MESH_ERR_INVALID beyond
 * that; the array (8 MiB) is held on every GPU the library has run this call on until the process ends; all callers of
 * one GPU share it, so calls are serialised inside the library (and calls from different processes do not interact:
 * each process has its own copy). */
int mesh_act_pack_noalloc(int fmt, const float *src, void *dst, int64_t n);

/* Device-pointer forms: pointers are GPU addresses, work is queued on `stream` (a hipStream_t, NULL =
 * the default stream) and not waited for. */
int mesh_act_pack_dev(int fmt, const float *d_src, void *d_dst, int64_t n, void *stream);
int mesh_act_unpack_dev(int fmt, const void *d_src, float *d_dst, int64_t n, void *stream);

/* Dequantize n elements of a GGUF tensor type (F16, Q8_0, Q5_0, Q4_K, Q6_K) to f32, bit-exact with ggml's
 * dequantize_row_* (what to_float does for a weight tensor).  Device pointers, queued on `stream`. */
int mesh_dequantize_dev(int type, const void *d_src, float *d_dst, int64_t n, void *stream);

/* ---- weights and mul_mat -------------------------------------------------------------------------
 * One weight matrix resident in HBM, as ggml_backend_tensor_set leaves it after SET_TENSOR /
 * SET_TENSOR_GGUF (patches/0001:261), and the mul_mat node of the worker's graph
 * (patches/0002:443-451 -> ggml_backend_graph_compute). */
typedef struct mesh_weight mesh_weight;

/* host_data: n_rows rows of row_len elements in GGUF block layout of `type` (F32, F16, Q8_0, Q5_0, Q4_K, Q6_K). */
int mesh_weight_upload(int type, const void *host_data, int64_t n_rows, int64_t row_len, mesh_weight **out);
void mesh_weight_free(mesh_weight *w);
/* GGUF bytes of the matrix (what one mul_mat must read from HBM). */
size_t mesh_weight_nbytes(const mesh_weight *w);
/* d_y[t][m] = sum_k W[m][k] * d_x[t][k], t < n_tokens; f32 activations on the device, queued on `stream`. */
int mesh_mul_mat_dev(const mesh_weight *w, const float *d_x, int64_t n_tokens, float *d_y, void *stream);
/* Round trip for tests: the matrix back in GGUF block layout (host buffer of mesh_weight_nbytes bytes). */
int mesh_weight_download(const mesh_weight *w, void *host_data);

/* ---- GGUF --------------------------------------------------------------------------------------- */
typedef struct mesh_model_info {
    char arch[32];
    uint32_t n_layer, n_embd, n_head, n_head_kv, head_dim, n_ff, n_vocab;
    uint32_t n_rot, rope_mode;            /* rope_mode: 0 = NORM (llama), 2 = NEOX (qwen2/qwen3) */
    uint32_t n_expert, n_expert_used, n_ff_exp;
    float rms_eps, rope_freq_base;
    uint32_t gguf_version, alignment;
    uint64_t n_tensors, data_offset, file_size;
} mesh_model_info;

typedef struct mesh_tensor_info {
    uint32_t type, n_dims;
    uint64_t ne[4];
    uint64_t file_offset;                 /* data section offset + tensor offset (patches/0001:209) */
    uint64_t nbytes;
} mesh_tensor_info;

/* Header-only scan of a GGUF file: hyper-parameters and container facts, no tensor data touched.
 * The bounded parse of mesh-client/src/models/gguf.rs:318-420 (scan_gguf_compact_meta). */
int mesh_gguf_probe(const char *gguf_path, mesh_model_info *out);
/* Directory entry of one tensor by name -- the lookup rpc_server::set_tensor_gguf does (patches/0001:203-209).
 * MESH_ERR_INVALID if the tensor is absent, MESH_ERR_FORMAT if its bytes would leave the file. */
int mesh_gguf_tensor(const char *gguf_path, const char *name, mesh_tensor_info *out);

/* ---- stage -------------------------------------------------------------------------------------- */
typedef struct mesh_stage mesh_stage;
typedef struct mesh_session mesh_session;

/* Pseudo-formats for the two ends of the pipeline. */
#define MESH_TOKENS 100   /* input: int32 token ids (stage must start at layer 0 and the file hold token_embd) */
#define MESH_LOGITS 101   /* output: f32 [n_tokens][n_vocab] after output_norm and the output projection */
/* Most tokens one mesh_stage_decode call (host pointers) returns logits for: its pinned staging holds that many rows of the
 * vocabulary.  More tokens in one call fail with MESH_ERR_INVALID; mesh_stage_decode_dev writes straight into the caller's
 * device buffer and has no such limit. */
#define MESH_LOGITS_TOKENS_MAX 128

typedef struct mesh_stage_opts {
    const char *device;     /* "ROCm0" / "HIP0" / "0"; NULL = current device               (-d, launch.rs:920-952) */
    int32_t n_ctx;          /* KV positions per sequence; 0 = 4096                          (-c, launch.rs:474-504) */
    int32_t n_seq_max;      /* sequences the KV cache holds; 0 = 1                          (--parallel, launch.rs:1338-1390) */
    int32_t n_batch_max;    /* most tokens one decode call may carry; 0 = 512 */
    int32_t kv_type;        /* K cache rows: 0 or MESH_F16, MESH_Q8_0, MESH_Q4_0            (--cache-type-k, launch.rs:639-644) */
    int32_t kv_type_v;      /* V cache rows: 0 = MESH_F16 when kv_type is f16, else MESH_Q4_0 (--cache-type-v).  The pairs of
                               KvCacheQuant::for_model_size (launch.rs:568-591) are supported: f16/f16, q8_0/q4_0, q4_0/q4_0 */
    const char *tuning;     /* kernel-selection switches as "name=value,name=value"; NULL = the defaults.  See
                               mesh_session_set_option for the names.  No counterpart in the reference. */
} mesh_stage_opts;

typedef struct mesh_batch {
    int32_t n_tokens;
    const int32_t *pos;     /* [n_tokens] cache position of each token */
    const int32_t *seq_id;  /* [n_tokens] sequence of each token; NULL = all 0 */
} mesh_batch;

/* Load layers [layer_begin, layer_end) of the GGUF model at gguf_path into HBM (layer_end < 0 = to the last
 * layer).  What `rpc-server --gguf PATH` plus the SET_TENSOR_GGUF traffic of start-up amount to
 * (mesh-llm/src/inference/launch.rs:887-1030; patches/0001:179-266). */
int mesh_stage_open(const char *gguf_path, int layer_begin, int layer_end, const mesh_stage_opts *opts, mesh_stage **out);
void mesh_stage_close(mesh_stage *stage);
int mesh_stage_info(const mesh_stage *stage, mesh_model_info *out);
/* GGUF bytes of everything this stage keeps resident (the weight traffic of one decode step). */
size_t mesh_stage_weight_bytes(const mesh_stage *stage);

/* A session owns the KV cache of n_seq_max sequences and the activation buffers. */
int mesh_stage_session_new(mesh_stage *stage, mesh_session **out);
void mesh_stage_session_free(mesh_session *session);

/* Run the stage over a batch: `in` holds n_tokens rows of n_embd in in_fmt (MESH_F32 / MESH_F16 / MESH_Q8_0, the
 * boundary tensor of the previous stage) or int32 token ids (MESH_TOKENS); each token's K/V is stored at
 * (seq_id, pos) and it attends to positions [0, pos] of its sequence.  `out` receives the boundary hidden state
 * packed in out_fmt, or logits (MESH_LOGITS).  *out_len = bytes written (set even when out_cap is too small).
 * Host pointers; blocks until done.  The GRAPH_COMPUTE + tensor push of one step (patches/0002:443-451,544-622). */
int mesh_stage_decode(mesh_session *session, const mesh_batch *batch, const void *in, int in_fmt,
                      void *out, int out_fmt, size_t out_cap, size_t *out_len);
/* Same with device pointers for in/out; queued on the session's stream, returns without waiting. */
int mesh_stage_decode_dev(mesh_session *session, const mesh_batch *batch, const void *d_in, int in_fmt,
                          void *d_out, int out_fmt, size_t out_cap, size_t *out_len);
/* The session's hipStream_t (for events), and a wait for everything queued on it. */
void *mesh_session_stream(mesh_session *session);
int mesh_session_synchronize(mesh_session *session);
/* Number of decode steps of this session whose layer launches were replayed from a captured HIP graph (batches of up to
 * 32 tokens, from the third call with the same token count and KV split count on; the switch graphs=1 turns them on:
 * they save the host the submission of ~80 launches per step).  -1 for a null session.  No counterpart in the reference. */
int64_t mesh_session_graph_replays(const mesh_session *session);

/* Per-kernel-class timing of a session: every kernel launched for the session while profiling is on carries its own
 * start / stop event pair (stamped by the dispatch, nothing extra is queued between launches), so ms[] sums pure
 * kernel durations -- the same spans a kernel trace shows -- and launches[] counts kernels.  Off by default.  Kinds
 * index the arrays below. */
#define MESH_PROF_GEMV 0      /* dequant-fused mat-vec launches (q/k/v, o, gate/up, down, output) */
#define MESH_PROF_ROPE 1      /* rope + KV append */
#define MESH_PROF_ATTN 2      /* attention (split + combine) */
#define MESH_PROF_CODEC 3     /* boundary pack / unpack */
#define MESH_PROF_PREP 4      /* activation preparation of the batched paths: RMS norm + quantise / f16 conversion, SwiGLU */
#define MESH_PROF_KINDS 5
typedef struct mesh_profile {
    double ms[MESH_PROF_KINDS];           /* summed kernel time per kind since the last reset */
    uint64_t launches[MESH_PROF_KINDS];   /* kernels per kind */
} mesh_profile;
int mesh_session_profile(mesh_session *session, int enable);          /* also resets the counters */
int mesh_session_profile_read(mesh_session *session, mesh_profile *out);   /* waits for the stream */

/* Mixture-of-experts sessions: restrict routing to a subset of the file's experts.  allowed[e] != 0 keeps expert
 * e; NULL clears the mask.  MESH_ERR_INVALID if n_mask differs from the expert count of the file.  The C API of
 * llama_model_set_expert_mask (patches/0003:46-50: 0 on success, -1 on a count mismatch); the mask is added as
 * 0 / -inf to the selection probabilities before top-k (patches/0003:86-104). */
int mesh_session_set_expert_mask(mesh_session *session, const uint8_t *allowed, int32_t n_mask);
/* Expert ids chosen for the tokens of the last decode call in the LAST mixture-of-experts layer of the stage:
 * ids[n_tokens][n_expert_used].  For tests and for counting distinct experts touched. */
int mesh_session_moe_last_ids(mesh_session *session, int32_t *ids, int32_t n_tokens);

/* Values the session's f16 producers clamped to the f16 range (+-65504) since the session was created.  Calls of 5 or more
 * tokens hand activations to the matrix cores as f16 (normalised hidden state, attention output, SwiGLU product); a value
 * beyond the range is stored as the largest finite f16 instead of infinity and counted here, so a caller can tell a
 * saturated step from an exact one.  Single-token calls use 16-bit fixed point with a scale per 32 values and never
 * count.  Waits for the session's stream.  No counterpart in the reference (ggml's f16 conversions saturate silently to
 * infinity). */
int mesh_session_f16_saturations(mesh_session *session, uint64_t *count);

/* Kernel-selection switches.  Every choice between two kernels for the same arithmetic and every dispatch threshold has
 * a name; the defaults are what the benchmarks run.  A stage takes the defaults, then the environment variable
 * MESH_TUNING ("name=value,...", read once per process, for A/B runs of an unmodified host), then
 * mesh_stage_opts.tuning; a session starts from its stage's values, and mesh_session_set_option changes a
 * session-level switch between decode calls (it waits for the session's stream and drops captured graphs).
 *
 *   stage level (decide what is allocated; mesh_stage_opts.tuning / MESH_TUNING only):
 *     gemm_layout=1        keep a GEMM-layout copy of the projections when n_batch_max reaches gemm_min_tokens
 *     gemm_min_tokens=17   calls of at least this many tokens run the large-tile MFMA GEMM
 *     skinny_min_tokens=0  calls of at least this many (and fewer than the above) run the skinny MFMA GEMM;
 *                          0 = 4 with skinny_f16, 5 without
 *   session level:
 *     gemm_splitk=1        GEMM launches too narrow to fill the chip split K over workgroups
 *     chunk_kv16=1         long prefill chunks over a quantised cache decode a layer's rows once into an f16 copy
 *     gemv_rope=1          RoPE and the KV append in the q/k/v projection's epilogue
 *     xq_handover=1        single-token calls: gate/up leaves the FFN vector quantised for the down projection
 *     skinny_f16=1         the skinny GEMM on the f16 matrix cores (0: integer matrix cores, 16-bit activations)
 *     skinny_norm_fused=1  f16 skinny GEMM: the RMS norms ride in the launches around them
 *     skinny_pair=1        skinny GEMMs: q4_K q/k and a q6_K v projection as one launch (0: one launch per type)
 *     skinny_f16_wide=1    batches of gemm_min_tokens..32 decode steps stay on the f16 skinny GEMM (0: large-tile GEMM)
 *     gemm_fused=1         q/k/v and gate/up of a prefill call as one launch each
 *     gemm_xdirect=1       the prefill GEMM reads k8-major activations directly
 *     gemm_big=1           256-row tiles for wide projections of long calls
 *     gemm_narrow=1        64-token tiles for calls of at most 64 tokens
 *     attn_chunk_ksplit=1  a prefill chunk's key walks split over workgroups when the grid would not fill the chip
 *     attn_mma_min_tokens=1  decode attention on the matrix cores from this many tokens
 *     attn_split_target=0  workgroups a decode attention launch aims at (0 = 256, or 512 for quantised rows)
 *     moe_group=1          (token, slot) pairs grouped by expert
 *     moe_router_tail=1    small decode batches: the router launch's last workgroup routes and groups the pairs
 *     moe_fuse_quant=1     the expert combine step quantises for the next layer
 *     moe_gemm=1, moe_gemm_min_pairs=4   prefill-sized expert products on the large-tile GEMM
 *     grouped_oversub=8    grouped expert mat-vec: workgroups per compute unit and item
 *     graphs=0             decode steps of up to 32 tokens replayed from captured HIP graphs
 *
 * MESH_ERR_INVALID: unknown name, value out of range, or a stage-level switch passed to set_option.  No counterpart in
 * the reference (llama.cpp picks kernels by compile-time flags and GGML_* environment variables). */
int mesh_session_set_option(mesh_session *session, const char *name, int32_t value);
int mesh_session_get_option(const mesh_session *session, const char *name, int32_t *value);

/* KV cache import/export for one sequence and one (absolute) layer: n_pos positions starting at pos0, host
 * buffers of f16 bits laid out [n_pos][n_head_kv][head_dim].  (The reference has no KV hand-over; a restarted
 * stage refills from the prompt -- mesh-llm/src/inference/election.rs:1894-1910.) */
int mesh_session_kv_write(mesh_session *session, int layer, int seq_id, int pos0, int n_pos,
                          const uint16_t *k, const uint16_t *v);
int mesh_session_kv_read(mesh_session *session, int layer, int seq_id, int pos0, int n_pos,
                         uint16_t *k, uint16_t *v);

/* ---- single graph nodes ---------------------------------------------------------------------------
 * The layer's activation producers and its decode attention on their own: the nodes rpc_server::graph_compute
 * (patches/0002:443-451) runs between the mat-muls -- rms_norm + mul, swiglu, flash_attn_ext -- in the forms the
 * batched paths of this library use.  Device pointers; queued on `stream` (the session's stream for attention). */

/* y = quantise(rms_norm(x, eps) * w) for n_tokens rows of n floats (n a multiple of 32; w NULL: quantise(x)) in the
 * "q16" activation layout of the batched decode GEMM: per block of 16 tokens 36 * n bytes = for every 8-element group g
 * and token t a 16-byte record at (g * 16 + t) * 16 holding the high bytes of eight 16-bit fixed-point values, then their
 * low bytes (value = (hi * 256 + lo) * d, lo and hi signed); at 32 * n the f32 scales d[(k / 32) * 16 + t] of the
 * 32-element blocks (d = max|v| / 32512), at 34 * n the f32 block sums.  mesh_op_q16_bytes: bytes of that buffer. */
size_t mesh_op_q16_bytes(int64_t n_tokens, int64_t n);
int mesh_op_rms_norm_q16_dev(const float *d_x, const float *d_w, float eps, int64_t n_tokens, int64_t n, void *d_q16, void *stream);
/* y = f16(rms_norm(x, eps) * w), saturating, in the "k8-major" layout of the prefill GEMM: blocks of 16 tokens, element
 * (t, k) of block t / 16 at ((k / 8) * 16 + t % 16) * 8 + k % 8 within the block's 16 * n halfs; rows beyond n_tokens
 * are zero.  d_y16 holds ceil(n_tokens / 16) * 16 * n halfs. */
int mesh_op_rms_norm_f16k8_dev(const float *d_x, const float *d_w, float eps, int64_t n_tokens, int64_t n, void *d_y16, void *stream);
/* y = f16(silu(gate) * up), saturating, same layout. */
int mesh_op_swiglu_f16k8_dev(const float *d_gate, const float *d_up, int64_t n_tokens, int64_t n, void *d_y16, void *stream);
/* Decode attention of one (absolute) layer over the session's KV cache: token i of the batch attends to positions
 * [0, pos[i]] of its sequence; d_q holds already rotated queries [n_tokens][n_head][head_dim] f32, d_out receives
 * [n_tokens][n_head][head_dim] f32.  matrix_cores != 0 picks the kernel the stage uses (queries and probabilities
 * rounded to f16), 0 the all-f32 one.  Waits for the session's stream before it queues its own work. */
int mesh_session_attn_dev(mesh_session *session, int layer, const float *d_q, const mesh_batch *batch, float *d_out, int matrix_cores);

#ifdef __cplusplus
}
#endif
#endif /* MESH_STAGE_H */
