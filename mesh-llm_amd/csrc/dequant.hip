// GGUF weight blocks -> f32, bit-exact with ggml's dequantize_row_q4_K / q6_K / q5_0 / q8_0 (the to_float of a
// weight tensor loaded by set_tensor_gguf, third_party/llama.cpp/patches/0001-rpc-optimize-local-GGUF-tensor-loading.patch:179-266).
// One thread per output element; each product and the subtraction are rounded separately (-ffp-contract=off).
// Used for parity checks, token-embedding rows and the LDS-staged prefill path's reference.

#include "mesh_common.hpp"

namespace mesh {

__device__ __forceinline__ uint16_t ld16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

// (scale, min) pair j of the 12 packed bytes of a q4_K super-block
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t *q, int &sc, int &m) {
    if (j < 4) {
        sc = q[j] & 63;
        m = q[j + 4] & 63;
    } else {
        sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
        m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

__global__ __launch_bounds__(256) void dequant_q4_K_kernel(const uint8_t *__restrict__ x, float *__restrict__ y,
                                                           int64_t nsb) {
    const int64_t sb = blockIdx.x;
    if (sb >= nsb) return;
    const int t = threadIdx.x;              // element within the super-block
    const uint8_t *b = x + sb * Q4_K_BYTES;
    const float d = f16_bits_to_f32(ld16(b));
    const float dmin = f16_bits_to_f32(ld16(b + 2));
    int sc, m;
    scale_min_k4(t >> 5, b + 4, sc, m);
    const int c = t >> 6, l = t & 31, hi = (t >> 5) & 1;
    const int q = (b[16 + 32 * c + l] >> (4 * hi)) & 0xF;
    const float d1 = d * (float)sc;
    const float m1 = dmin * (float)m;
    y[sb * QK_K + t] = d1 * (float)q - m1;
}

__global__ __launch_bounds__(256) void dequant_q6_K_kernel(const uint8_t *__restrict__ x, float *__restrict__ y,
                                                           int64_t nsb) {
    const int64_t sb = blockIdx.x;
    if (sb >= nsb) return;
    const int t = threadIdx.x;
    const uint8_t *b = x + sb * Q6_K_BYTES;
    const int n = t >> 7;                    // which half of the super-block
    const int r = t & 127;
    const int grp = r >> 5;                  // 0..3: which of q1..q4
    const int l = r & 31;
    const uint8_t *ql = b + 64 * n;
    const uint8_t *qh = b + 128 + 32 * n;
    const int8_t *sc = reinterpret_cast<const int8_t *>(b + 192) + 8 * n;
    const float d = f16_bits_to_f32(ld16(b + 208));
    const int lo = (grp & 1) ? ql[l + 32] : ql[l];
    const int nib = (grp & 2) ? (lo >> 4) : (lo & 0xF);
    const int q = (nib | (((qh[l] >> (2 * grp)) & 3) << 4)) - 32;
    const int is = l / 16 + 2 * grp;
    y[sb * QK_K + t] = d * (float)sc[is] * (float)q;
}

__global__ __launch_bounds__(256) void dequant_q5_0_kernel(const uint8_t *__restrict__ x, float *__restrict__ y,
                                                           int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint8_t *b = x + (i >> 5) * Q5_0_BYTES;
    const int e = (int)(i & 31);
    const int j = e & 15;
    const float d = f16_bits_to_f32(ld16(b));
    const uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
    int q;
    if (e < 16) q = ((b[6 + j] & 0x0F) | (((qh >> j) << 4) & 0x10)) - 16;
    else        q = ((b[6 + j] >> 4) | ((qh >> (j + 12)) & 0x10)) - 16;
    y[i] = (float)q * d;
}

__global__ __launch_bounds__(256) void dequant_q8_0_kernel(const uint8_t *__restrict__ x, float *__restrict__ y,
                                                           int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint8_t *b = x + (i >> 5) * Q8_0_BYTES;
    y[i] = (float)(int8_t)b[2 + (i & 31)] * f16_bits_to_f32(ld16(b));
}

int act_unpack_dev(int fmt, const void *src, float *dst, int64_t n, hipStream_t stream);

int dequantize_dev(int type, const void *src, float *dst, int64_t n, hipStream_t stream) {
    if (n < 0 || (n > 0 && (!src || !dst))) return fail(MESH_ERR_INVALID, "mesh_dequantize: null pointer or negative count");
    if (row_bytes(type, n) < 0)
        return fail(type == MESH_F32 || block_elems(type) > 0 ? MESH_ERR_INVALID : MESH_ERR_UNSUPPORTED,
                    "mesh_dequantize: type %d with %lld elements is not a whole number of blocks", type, (long long)n);
    if (n == 0) return MESH_OK;
    const uint8_t *x = static_cast<const uint8_t *>(src);
    switch (type) {
        case MESH_F32:
        case MESH_F16:
            return act_unpack_dev(type, src, dst, n, stream);
        case MESH_Q8_0:
            MESH_LAUNCH(dequant_q8_0_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, dst, n);
            break;
        case MESH_Q5_0:
            MESH_LAUNCH(dequant_q5_0_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, dst, n);
            break;
        case MESH_Q4_K:
            MESH_LAUNCH(dequant_q4_K_kernel, dim3((unsigned)(n / QK_K)), dim3(256), 0, stream, x, dst, n / QK_K);
            break;
        case MESH_Q6_K:
            MESH_LAUNCH(dequant_q6_K_kernel, dim3((unsigned)(n / QK_K)), dim3(256), 0, stream, x, dst, n / QK_K);
            break;
        default:
            return fail(MESH_ERR_UNSUPPORTED, "mesh_dequantize: no kernel for ggml type %d", type);
    }
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

}  // namespace mesh
