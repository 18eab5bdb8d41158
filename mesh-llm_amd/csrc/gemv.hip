// Dequant-fused GEMV for decode (batch <= a few tokens): y = W x with W in q4_K / q6_K blocks (tiled layout of
// gemv.hpp) or any other GGUF type on the stage path (row-major, generic loop).  Stands where
// ggml_backend_graph_compute runs mul_mat for a worker's layers
// (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451).
//
// One workgroup (4 waves) owns 16 output rows; its waves take alternate super-blocks along K and their partial
// sums meet in LDS, so results are deterministic (no atomics).  The activation vector is staged once per
// workgroup in LDS as f32 together with sums of 8 (for the q4_K min term and the q6_K -32 offset); the RMS norm
// that precedes every projection is folded into that staging.  Weight bytes cross HBM exactly once per launch.

#include "gemv.hpp"

namespace mesh {

constexpr int GEMV_THREADS = 256;
constexpr int GEMV_WAVES = GEMV_THREADS / 64;
constexpr int KCHUNK = 4096;   // elements of x staged per pass (16 KiB per column)

__device__ __forceinline__ float ub0(uint32_t v) { return (float)(v & 0xFFu); }
__device__ __forceinline__ float ub1(uint32_t v) { return (float)((v >> 8) & 0xFFu); }
__device__ __forceinline__ float ub2(uint32_t v) { return (float)((v >> 16) & 0xFFu); }
__device__ __forceinline__ float ub3(uint32_t v) { return (float)(v >> 24); }

// sum_i byte_i(v0)*xa[i] + byte_i(v1)*xa[4+i]
__device__ __forceinline__ float dot8(uint32_t v0, uint32_t v1, const float4 &xa, const float4 &xb) {
    float s = ub0(v0) * xa.x;
    s = fmaf(ub1(v0), xa.y, s);
    s = fmaf(ub2(v0), xa.z, s);
    s = fmaf(ub3(v0), xa.w, s);
    s = fmaf(ub0(v1), xb.x, s);
    s = fmaf(ub1(v1), xb.y, s);
    s = fmaf(ub2(v1), xb.z, s);
    s = fmaf(ub3(v1), xb.w, s);
    return s;
}

// One q4_K tile (16 rows x 256 k): lane (r, g) adds its share of row r's dot products into acc[t].
// xs: LDS, column t at xs + t*xs_ld, pointing at the super-block's first element; xsum likewise in groups of 8.
template <int NB>
__device__ __forceinline__ void q4k_tile(const uint8_t *__restrict__ tile, int lane, const float *xs, int xs_ld,
                                         const float *xsum, int xsum_ld, float (&acc)[NB]) {
    const int r = lane & 15, g = lane >> 4;
    const uint4 hdr = *reinterpret_cast<const uint4 *>(tile + r * 16);
    const uint4 p0 = *reinterpret_cast<const uint4 *>(tile + 256 + lane * 16);
    const uint4 p1 = *reinterpret_cast<const uint4 *>(tile + 256 + 1024 + lane * 16);
    const float d = f16_bits_to_f32((uint16_t)(hdr.x & 0xFFFFu));
    const float dmin = f16_bits_to_f32((uint16_t)(hdr.x >> 16));
    // 6-bit scales/mins of the 8 sub-blocks, four per dword
    const uint32_t sc_lo = hdr.y & 0x3F3F3F3Fu;
    const uint32_t mn_lo = hdr.z & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    const float dsc[8] = {d * ub0(sc_lo), d * ub1(sc_lo), d * ub2(sc_lo), d * ub3(sc_lo),
                          d * ub0(sc_hi), d * ub1(sc_hi), d * ub2(sc_hi), d * ub3(sc_hi)};
    const float dmn[8] = {dmin * ub0(mn_lo), dmin * ub1(mn_lo), dmin * ub2(mn_lo), dmin * ub3(mn_lo),
                          dmin * ub0(mn_hi), dmin * ub1(mn_hi), dmin * ub2(mn_hi), dmin * ub3(mn_hi)};
    const uint32_t w[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};   // chunk c -> w[2c], w[2c+1]
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int c = s >> 1;
        const uint32_t v0 = (s & 1) ? (w[2 * c] >> 4) & 0x0F0F0F0Fu : w[2 * c] & 0x0F0F0F0Fu;
        const uint32_t v1 = (s & 1) ? (w[2 * c + 1] >> 4) & 0x0F0F0F0Fu : w[2 * c + 1] & 0x0F0F0F0Fu;
        const int k = 32 * s + 8 * g;
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            const float4 xa = *reinterpret_cast<const float4 *>(xs + t * xs_ld + k);
            const float4 xb = *reinterpret_cast<const float4 *>(xs + t * xs_ld + k + 4);
            const float sx = xsum[t * xsum_ld + (k >> 3)];
            acc[t] = fmaf(dsc[s], dot8(v0, v1, xa, xb), acc[t]);
            acc[t] = fmaf(-dmn[s], sx, acc[t]);
        }
    }
}

template <int NB>
__device__ __forceinline__ void q6k_tile(const uint8_t *__restrict__ tile, int lane, const float *xs, int xs_ld,
                                         const float *xsum, int xsum_ld, float (&acc)[NB]) {
    const int r = lane & 15, g = lane >> 4;
    const uint4 l0 = *reinterpret_cast<const uint4 *>(tile + lane * 16);
    const uint4 l1 = *reinterpret_cast<const uint4 *>(tile + 1024 + lane * 16);
    const uint4 h = *reinterpret_cast<const uint4 *>(tile + 2048 + lane * 16);
    const uint4 scv = *reinterpret_cast<const uint4 *>(tile + 3072 + r * 16);
    const float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(tile + 3328 + r * 2));
    const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
    const uint32_t ql[2][4] = {{l0.x, l0.y, l0.z, l0.w}, {l1.x, l1.y, l1.z, l1.w}};   // [n][a0,a1,b0,b1]
    const uint32_t qh[2][2] = {{h.x, h.y}, {h.z, h.w}};
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int n = s >> 2, t4 = s & 3;
        // element 128n + 32*t4 + 8g + i: low/high nibble of ql byte, two bits of qh
        uint32_t v[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t lw = ql[n][(t4 & 1) * 2 + j];
            const uint32_t nib = (t4 & 2) ? (lw >> 4) & 0x0F0F0F0Fu : lw & 0x0F0F0F0Fu;
            const uint32_t hw = qh[n][j];
            const uint32_t hb = t4 == 0 ? (hw << 4) : t4 == 1 ? (hw << 2) : t4 == 2 ? hw : (hw >> 2);
            v[j] = nib | (hb & 0x30303030u);
        }
        const int si = 8 * n + 2 * t4 + (g >> 1);                 // scale index = element / 16
        const int sbyte = (int)(int8_t)((scw[si >> 2] >> (8 * (si & 3))) & 0xFFu);
        const float dsc = d * (float)sbyte;
        const int k = 32 * s + 8 * g;
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            const float4 xa = *reinterpret_cast<const float4 *>(xs + t * xs_ld + k);
            const float4 xb = *reinterpret_cast<const float4 *>(xs + t * xs_ld + k + 4);
            const float sx = xsum[t * xsum_ld + (k >> 3)];
            acc[t] = fmaf(dsc, fmaf(-32.0f, sx, dot8(v[0], v[1], xa, xb)), acc[t]);
        }
    }
}

// element k of a GGUF row in one of the non-tiled types
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

struct GemvKernelArgs {
    GemvMat mat[3];
    int tile_begin[4];     // first tile-row of each matrix in the grid; tile_begin[n_mat] = grid size
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
__global__ __launch_bounds__(GEMV_THREADS) void gemv_kernel(const GemvKernelArgs a) {
    extern __shared__ __align__(16) float smem[];
    const int kc = a.K < KCHUNK ? a.K : KCHUNK;
    float *xs = smem;                      // [NB][kc]
    float *xsum = xs + NB * kc;            // [NB][kc/8]
    float *red = xsum + NB * (kc / 8);     // [2][GEMV_WAVES][16][NB]
    __shared__ float scale_s[NB];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // which matrix / tile-row this workgroup owns
    int mi = 0;
    if (a.epi != EPI_SWIGLU) {
        while (mi + 1 < a.n_mat && (int)blockIdx.x >= a.tile_begin[mi + 1]) ++mi;
    }
    const int tile_row = blockIdx.x - a.tile_begin[mi];
    const int n_dual = a.epi == EPI_SWIGLU ? 2 : 1;

    // fused RMS norm: scale[t] = 1/sqrt(mean(x_t^2) + eps)
    if (a.norm_w) {
        float ss[NB];
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            ss[t] = 0.f;
            for (int i = tid * 4; i < a.K; i += GEMV_THREADS * 4) {
                const float4 v = *reinterpret_cast<const float4 *>(a.x + (size_t)t * a.ldx + i);
                ss[t] += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
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
            for (int w = 0; w < GEMV_WAVES; ++w) s += red[w * NB + tid];
            scale_s[tid] = 1.0f / sqrtf(s / (float)a.K + a.eps);
        }
        __syncthreads();
    }

    float acc[2][NB];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int t = 0; t < NB; ++t) acc[u][t] = 0.f;

    const int nsb_total = a.K / QK_K;
    for (int k0 = 0; k0 < a.K; k0 += kc) {
        const int len = a.K - k0 < kc ? a.K - k0 : kc;
        if (k0) __syncthreads();
        // stage x[k0 .. k0+len) (normalised) and its sums of 8
        for (int j = tid; j < len / 8; j += GEMV_THREADS) {
#pragma unroll
            for (int t = 0; t < NB; ++t) {
                const float *src = a.x + (size_t)t * a.ldx + k0 + j * 8;
                float4 v0 = *reinterpret_cast<const float4 *>(src);
                float4 v1 = *reinterpret_cast<const float4 *>(src + 4);
                if (a.norm_w) {
                    const float sc = scale_s[t];
                    const float4 w0 = *reinterpret_cast<const float4 *>(a.norm_w + k0 + j * 8);
                    const float4 w1 = *reinterpret_cast<const float4 *>(a.norm_w + k0 + j * 8 + 4);
                    v0.x = v0.x * sc * w0.x; v0.y = v0.y * sc * w0.y; v0.z = v0.z * sc * w0.z; v0.w = v0.w * sc * w0.w;
                    v1.x = v1.x * sc * w1.x; v1.y = v1.y * sc * w1.y; v1.z = v1.z * sc * w1.z; v1.w = v1.w * sc * w1.w;
                }
                *reinterpret_cast<float4 *>(xs + t * kc + j * 8) = v0;
                *reinterpret_cast<float4 *>(xs + t * kc + j * 8 + 4) = v1;
                xsum[t * (kc / 8) + j] = ((v0.x + v0.y) + (v0.z + v0.w)) + ((v1.x + v1.y) + (v1.z + v1.w));
            }
        }
        // K not a multiple of 8 only happens for non-tiled types with odd shapes; handle the tail scalar
        for (int i = (len / 8) * 8 + tid; i < len; i += GEMV_THREADS) {
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
            const uint8_t *W = static_cast<const uint8_t *>(m.W);
            if (m.type == MESH_Q4_K) {
                const uint8_t *base = W + (size_t)tile_row * nsb_total * Q4K_TILE_BYTES;
                for (int sb = k0 / QK_K + wave; sb < (k0 + len) / QK_K; sb += GEMV_WAVES)
                    q4k_tile<NB>(base + (size_t)sb * Q4K_TILE_BYTES, lane, xs + (sb * QK_K - k0), kc,
                                 xsum + (sb * QK_K - k0) / 8, kc / 8, acc[u]);
            } else if (m.type == MESH_Q6_K) {
                const uint8_t *base = W + (size_t)tile_row * nsb_total * Q6K_TILE_BYTES;
                for (int sb = k0 / QK_K + wave; sb < (k0 + len) / QK_K; sb += GEMV_WAVES)
                    q6k_tile<NB>(base + (size_t)sb * Q6K_TILE_BYTES, lane, xs + (sb * QK_K - k0), kc,
                                 xsum + (sb * QK_K - k0) / 8, kc / 8, acc[u]);
            } else {
                // generic row-major types: lane (r, g) strides over row r's elements of this chunk
                const int r = lane & 15, g = lane >> 4;
                const int row = tile_row * TILE_ROWS + r;
                if (row < m.M) {
                    const uint8_t *rowp = W + (size_t)row * (size_t)(a.K / block_elems_dev(m.type)) * block_bytes_dev(m.type);
                    for (int i = wave * 4 + g; i < len; i += GEMV_WAVES * 4) {
                        const float wv = row_elem(m.type, rowp, k0 + i);
#pragma unroll
                        for (int t = 0; t < NB; ++t) acc[u][t] = fmaf(wv, xs[t * kc + i], acc[u][t]);
                    }
                }
            }
        }
    }

    // lanes r, r+16, r+32, r+48 hold parts of row r; then the 4 waves meet in LDS
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
            for (int t = 0; t < NB; ++t) red[((u * GEMV_WAVES + wave) * 16 + lane) * NB + t] = acc[u][t];
    }
    __syncthreads();
    if (tid < 16 * NB) {
        const int r = tid / NB, t = tid % NB;
        const GemvMat &m = a.mat[mi];
        const int row = tile_row * TILE_ROWS + r;
        if (row < m.M) {
            float s0 = 0.f, s1 = 0.f;
            for (int w = 0; w < GEMV_WAVES; ++w) {
                s0 += red[((0 * GEMV_WAVES + w) * 16 + r) * NB + t];
                s1 += red[((1 * GEMV_WAVES + w) * 16 + r) * NB + t];
            }
            if (m.bias) s0 += m.bias[row];
            float out;
            if (a.epi == EPI_SWIGLU) {
                if (a.mat[mi + 1].bias) s1 += a.mat[mi + 1].bias[row];
                out = (s0 / (1.0f + expf(-s0))) * s1;
            } else if (a.epi == EPI_RESIDUAL) {
                out = a.residual[(size_t)t * a.ldres + row] + s0;
            } else {
                out = s0;
            }
            m.y[(size_t)t * m.ldy + row] = out;
        }
    }
}

static size_t gemv_smem_bytes(int NB, int K) {
    const int kc = K < KCHUNK ? K : KCHUNK;
    return sizeof(float) * ((size_t)NB * kc + (size_t)NB * (kc / 8) + 2 * GEMV_WAVES * 16 * NB + 16);
}

template <int NB>
static int launch_gemv(const GemvKernelArgs &ka, int grid, hipStream_t stream) {
    const size_t smem = gemv_smem_bytes(NB, ka.K);
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_kernel<NB>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256));
        attr_set = true;
    }
    gemv_kernel<NB><<<dim3((unsigned)grid), dim3(GEMV_THREADS), smem, stream>>>(ka);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

int gemv(const GemvArgs &a, hipStream_t stream) {
    if (a.n_mat < 1 || a.n_mat > 3 || !a.x || a.K <= 0 || a.T < 0)
        return fail(MESH_ERR_INVALID, "gemv: bad arguments (n_mat %d, K %d, T %d)", a.n_mat, a.K, a.T);
    if (a.epi == EPI_SWIGLU && a.n_mat != 2) return fail(MESH_ERR_INVALID, "gemv: swiglu needs exactly gate and up");
    if (a.epi == EPI_SWIGLU && a.mat[0].M != a.mat[1].M) return fail(MESH_ERR_INVALID, "gemv: gate and up differ in rows");
    if (a.epi == EPI_RESIDUAL && !a.residual) return fail(MESH_ERR_INVALID, "gemv: residual epilogue without residual");
    if ((a.ldx % 4) || (reinterpret_cast<uintptr_t>(a.x) & 15)) return fail(MESH_ERR_INVALID, "gemv: x must be 16-byte aligned");
    GemvKernelArgs ka{};
    int grid = 0;
    for (int i = 0; i < a.n_mat; ++i) {
        const GemvMat &m = a.mat[i];
        if (!m.W || m.M <= 0 || (!m.y && !(a.epi == EPI_SWIGLU && i == 1)))
            return fail(MESH_ERR_INVALID, "gemv: matrix %d incomplete", i);
        if (row_bytes(m.type, a.K) < 0)
            return fail(MESH_ERR_INVALID, "gemv: K=%d is not a whole number of type-%d blocks", a.K, m.type);
        if (m.type != MESH_Q4_K && m.type != MESH_Q6_K && m.type != MESH_F32 && m.type != MESH_F16 &&
            m.type != MESH_Q8_0 && m.type != MESH_Q5_0)
            return fail(MESH_ERR_UNSUPPORTED, "gemv: no kernel for ggml type %d", m.type);
        ka.mat[i] = m;
        ka.tile_begin[i] = grid;
        if (!(a.epi == EPI_SWIGLU && i == 1)) grid += (m.M + TILE_ROWS - 1) / TILE_ROWS;
    }
    for (int i = a.n_mat; i < 4; ++i) ka.tile_begin[i] = grid;
    ka.n_mat = a.n_mat;
    ka.ldx = a.ldx;
    ka.K = a.K;
    ka.norm_w = a.norm_w;
    ka.eps = a.eps;
    ka.ldres = a.ldres;
    ka.epi = a.epi;
    // columns in groups of 4, 2, 1
    int t = 0;
    while (t < a.T) {
        const int left = a.T - t;
        const int nb = left >= 4 ? 4 : left >= 2 ? 2 : 1;
        GemvKernelArgs kb = ka;
        kb.x = a.x + (size_t)t * a.ldx;
        kb.residual = a.residual ? a.residual + (size_t)t * a.ldres : nullptr;
        for (int i = 0; i < a.n_mat; ++i)
            if (kb.mat[i].y) kb.mat[i].y = a.mat[i].y + (size_t)t * a.mat[i].ldy;
        int rc;
        if (nb == 4) rc = launch_gemv<4>(kb, grid, stream);
        else if (nb == 2) rc = launch_gemv<2>(kb, grid, stream);
        else rc = launch_gemv<1>(kb, grid, stream);
        if (rc != MESH_OK) return rc;
        t += nb;
    }
    return MESH_OK;
}

}  // namespace mesh
