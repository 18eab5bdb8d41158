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

/* Device-pointer forms: pointers are GPU addresses, work is queued on `stream` (a hipStream_t, NULL =
 * the default stream) and not waited for. */
int mesh_act_pack_dev(int fmt, const float *d_src, void *d_dst, int64_t n, void *stream);
int mesh_act_unpack_dev(int fmt, const void *d_src, float *d_dst, int64_t n, void *stream);

/* Dequantize n elements of a GGUF tensor type (F16, Q8_0, Q5_0, Q4_K, Q6_K) to f32, bit-exact with ggml's
 * dequantize_row_* (what to_float does for a weight tensor).  Device pointers, queued on `stream`. */
int mesh_dequantize_dev(int type, const void *d_src, float *d_dst, int64_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MESH_STAGE_H */
