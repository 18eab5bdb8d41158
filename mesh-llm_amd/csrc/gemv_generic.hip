// GEMV for the GGUF types that are not K-quants (F32, F16, Q8_0, Q5_0), weights in GGUF row-major layout.
// These are the fallback types of a Q4_K_M file whose rows are not a multiple of 256 (hidden size 896) and the
// f32 router of MoE layers; they are a small share of any stage's bytes, so this kernel favours simplicity:
// x is staged in LDS as f32 (with the fused RMS norm), lane (r, g) of each wave walks row r with stride, and the
// same 16-rows-per-workgroup / LDS reduction structure as the K-quant kernel keeps results deterministic.

#include "gemv.hpp"

namespace mesh {

constexpr int GEN_THREADS = 256;
constexpr int GEN_WAVES = GEN_THREADS / 64;
constexpr int KCHUNK = 4096;   // elements of x staged per pass (16 KiB per column)

// element k of a GGUF row
__device__ __forceinline__ float row_elem(int type, const uint8_t *row, int k) {
    switch (type) {
        case MESH_F32: return reinterpret_cast<const float *>(row)[k];
        case MESH_F16: return f16_bits_to_f32(reinterpret_cast<const uint16_t *>(row)[k]);
        case MESH_Q8_0: {
            const uint8_t *b = row + (k >> 5) * Q8_0_BYTES;
            return (float)(int8_t)b[2 + (k & 31)] * f16_bits_to_f32((uint16_t)(b[0] | (b[1] << 8)));
        }
        case MESH_Q5_0: {
            const uint8_t *b = row + (k >> 5) * Q5_0_BYTES;
            const int e = k & 31, j = e & 15;
            const uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
            const int q = e < 16 ? ((b[6 + j] & 0x0F) | (((qh >> j) << 4) & 0x10)) - 16
                                 : ((b[6 + j] >> 4) | ((qh >> (j + 12)) & 0x10)) - 16;
            return (float)q * f16_bits_to_f32((uint16_t)(b[0] | (b[1] << 8)));
        }
        default: return 0.f;
    }
}

struct GenArgs {
    GemvMat mat[3];
    int tile_begin[4];
    int n_mat;
    const float *x;
    int ldx, K;
    const float *norm_w;
    float eps;
    const float *residual;
    int ldres;
    int epi;
};

template <int NB>
__global__ __launch_bounds__(GEN_THREADS) void gemv_generic_kernel(const GenArgs a) {
    extern __shared__ __align__(16) float smem_f[];
    const int kc = a.K < KCHUNK ? a.K : KCHUNK;
    float *xs = smem_f;                    // [NB][kc]
    float *red = xs + NB * kc;             // [2][GEN_WAVES][16][NB]
    __shared__ float scale_s[NB];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int mi = 0;
    if (a.epi != EPI_SWIGLU) {
        while (mi + 1 < a.n_mat && (int)blockIdx.x >= a.tile_begin[mi + 1]) ++mi;
    }
    const int tile_row = blockIdx.x - a.tile_begin[mi];
    const int n_dual = a.epi == EPI_SWIGLU ? 2 : 1;

    if (a.norm_w) {
        float ss[NB];
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            ss[t] = 0.f;
            for (int i = tid; i < a.K; i += GEN_THREADS) {
                const float v = a.x[(size_t)t * a.ldx + i];
                ss[t] += v * v;
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) ss[t] += __shfl_xor(ss[t], o);
        }
        if (lane == 0) {
#pragma unroll
            for (int t = 0; t < NB; ++t) red[wave * NB + t] = ss[t];
        }
        __syncthreads();
        if (tid < NB) {
            float s = 0.f;
            for (int w = 0; w < GEN_WAVES; ++w) s += red[w * NB + tid];
            scale_s[tid] = 1.0f / sqrtf(s / (float)a.K + a.eps);
        }
        __syncthreads();
    }

    float acc[2][NB];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int t = 0; t < NB; ++t) acc[u][t] = 0.f;

    const int r = lane & 15, g = lane >> 4;
    const int row = tile_row * TILE_ROWS + r;
    for (int k0 = 0; k0 < a.K; k0 += kc) {
        const int len = a.K - k0 < kc ? a.K - k0 : kc;
        if (k0) __syncthreads();
        for (int i = tid; i < len; i += GEN_THREADS) {
#pragma unroll
            for (int t = 0; t < NB; ++t) {
                float v = a.x[(size_t)t * a.ldx + k0 + i];
                if (a.norm_w) v = v * scale_s[t] * a.norm_w[k0 + i];
                xs[t * kc + i] = v;
            }
        }
        __syncthreads();
#pragma unroll 1
        for (int u = 0; u < n_dual; ++u) {
            const GemvMat &m = a.mat[mi + u];
            if (row < m.M) {
                const uint8_t *rowp = static_cast<const uint8_t *>(m.W) +
                                      (size_t)row * (size_t)(a.K / block_elems_dev(m.type)) * block_bytes_dev(m.type);
                for (int i = wave * 4 + g; i < len; i += GEN_WAVES * 4) {
                    const float wv = row_elem(m.type, rowp, k0 + i);
#pragma unroll
                    for (int t = 0; t < NB; ++t) acc[u][t] = fmaf(wv, xs[t * kc + i], acc[u][t]);
                }
            }
        }
    }

#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            acc[u][t] += __shfl_xor(acc[u][t], 16);
            acc[u][t] += __shfl_xor(acc[u][t], 32);
        }
    __syncthreads();
    if (lane < 16) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int t = 0; t < NB; ++t) red[((u * GEN_WAVES + wave) * 16 + lane) * NB + t] = acc[u][t];
    }
    __syncthreads();
    if (tid < 16 * NB) {
        const int rr = tid / NB, t = tid % NB;
        const GemvMat &m = a.mat[mi];
        const int orow = tile_row * TILE_ROWS + rr;
        if (orow < m.M) {
            float s0 = 0.f, s1 = 0.f;
            for (int w = 0; w < GEN_WAVES; ++w) {
                s0 += red[((0 * GEN_WAVES + w) * 16 + rr) * NB + t];
                s1 += red[((1 * GEN_WAVES + w) * 16 + rr) * NB + t];
            }
            if (m.bias) s0 += m.bias[orow];
            float out;
            if (a.epi == EPI_SWIGLU) {
                if (a.mat[mi + 1].bias) s1 += a.mat[mi + 1].bias[orow];
                out = (s0 / (1.0f + expf(-s0))) * s1;
            } else if (a.epi == EPI_RESIDUAL) {
                out = a.residual[(size_t)t * a.ldres + orow] + s0;
            } else {
                out = s0;
            }
            m.y[(size_t)t * m.ldy + orow] = out;
        }
    }
}

template <int NB>
static int launch_generic(const GenArgs &ka, int grid, hipStream_t stream) {
    const int kc = ka.K < KCHUNK ? ka.K : KCHUNK;
    const size_t smem = sizeof(float) * ((size_t)NB * kc + 2 * GEN_WAVES * 16 * NB);
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_generic_kernel<NB>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
        attr_set = true;
    }
    MESH_LAUNCH(gemv_generic_kernel<NB>, dim3((unsigned)grid), dim3(GEN_THREADS), smem, stream, ka);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

int gemv_generic(const GemvArgs &a, hipStream_t stream) {
    GenArgs ka{};
    int grid = 0;
    for (int i = 0; i < a.n_mat; ++i) {
        const int ty = a.mat[i].type;
        if (ty != MESH_F32 && ty != MESH_F16 && ty != MESH_Q8_0 && ty != MESH_Q5_0)
            return fail(MESH_ERR_UNSUPPORTED, "gemv: no kernel for ggml type %d", ty);
        ka.mat[i] = a.mat[i];
        ka.tile_begin[i] = grid;
        if (!(a.epi == EPI_SWIGLU && i == 1)) grid += (a.mat[i].M + TILE_ROWS - 1) / TILE_ROWS;
    }
    for (int i = a.n_mat; i < 4; ++i) ka.tile_begin[i] = grid;
    ka.n_mat = a.n_mat;
    ka.ldx = a.ldx;
    ka.K = a.K;
    ka.norm_w = a.norm_w;
    ka.eps = a.eps;
    ka.ldres = a.ldres;
    ka.epi = a.epi;
    int t = 0;
    while (t < a.T) {
        const int left = a.T - t;
        const int nb = left >= 4 ? 4 : left >= 2 ? 2 : 1;
        GenArgs kb = ka;
        kb.x = a.x + (size_t)t * a.ldx;
        kb.residual = a.residual ? a.residual + (size_t)t * a.ldres : nullptr;
        for (int i = 0; i < a.n_mat; ++i)
            if (kb.mat[i].y) kb.mat[i].y = a.mat[i].y + (size_t)t * a.mat[i].ldy;
        int rc;
        if (nb == 4) rc = launch_generic<4>(kb, grid, stream);
        else if (nb == 2) rc = launch_generic<2>(kb, grid, stream);
        else rc = launch_generic<1>(kb, grid, stream);
        if (rc != MESH_OK) return rc;
        t += nb;
    }
    return MESH_OK;
}

}  // namespace mesh
