// extern "C" entry points for single graph nodes of the layer (declared in include/mesh_stage.h): the activation
// producers of the batched paths and decode attention, callable on their own.

#include "gemm.hpp"
#include "stage.hpp"

using namespace mesh;

extern "C" {

size_t mesh_op_q16_bytes(int64_t n_tokens, int64_t n) {
    if (n_tokens < 1 || n < 32 || n % 32) return 0;
    return (size_t)((n_tokens + 15) / 16) * q16_block_bytes((int)n);
}

int mesh_op_rms_norm_q16_dev(const float *d_x, const float *d_w, float eps, int64_t n_tokens, int64_t n, void *d_q16, void *stream) {
    if (!d_x || !d_q16 || n_tokens < 1 || n < 32 || n % 32 || n > (1 << 20)) return fail(MESH_ERR_INVALID, "mesh_op_rms_norm_q16_dev: bad arguments");
    return quant16_k8(d_x, d_w, eps, (int)n_tokens, (int)n, static_cast<uint8_t *>(d_q16), static_cast<hipStream_t>(stream));
}

int mesh_op_rms_norm_f16k8_dev(const float *d_x, const float *d_w, float eps, int64_t n_tokens, int64_t n, void *d_y16, void *stream) {
    if (!d_x || !d_w || !d_y16 || n_tokens < 1 || n < 8 || n % 8) return fail(MESH_ERR_INVALID, "mesh_op_rms_norm_f16k8_dev: bad arguments");
    return rmsnorm_f16_k8(d_x, d_w, eps, (int)n_tokens, (int)n, static_cast<_Float16 *>(d_y16), static_cast<hipStream_t>(stream));
}

int mesh_op_swiglu_f16k8_dev(const float *d_gate, const float *d_up, int64_t n_tokens, int64_t n, void *d_y16, void *stream) {
    if (!d_gate || !d_up || !d_y16 || n_tokens < 1 || n < 8 || n % 8) return fail(MESH_ERR_INVALID, "mesh_op_swiglu_f16k8_dev: bad arguments");
    return swiglu_f16_k8(d_gate, d_up, (int)n_tokens, (int)n, static_cast<_Float16 *>(d_y16), static_cast<hipStream_t>(stream));
}

int mesh_session_attn_dev(mesh_session *session, int layer, const float *d_q, const mesh_batch *batch, float *d_out, int matrix_cores) {
    if (!session || !d_q || !batch || !d_out) return fail(MESH_ERR_INVALID, "mesh_session_attn_dev: null argument");
    return session_attention(session, layer, d_q, batch, d_out, matrix_cores);
}

}  // extern "C"
