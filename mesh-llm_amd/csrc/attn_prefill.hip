// Causal GQA attention for a prefill chunk on the matrix cores (head_dim 128; f16 or quantised KV cache rows, which
// are dequantised to f16 on their way into LDS).
//
// The chunk is T consecutive positions pos0 .. pos0 + T - 1 of one sequence whose keys and values are already in
// the cache (rope_kv appended them); token t attends to cache positions [0, pos0 + t].  A workgroup takes 32
// queries of every head of one KV-head group (one wave per head), walks the keys in tiles of 32 and keeps the
// running softmax in registers:
//   S^T = K . Q^T        (32 keys x 32 queries, v_mfma_f32_32x32x16_f16 over the 128 dims)
//   O^T += V^T . P^T     (128 dims x 32 queries, contraction over the 32 keys)
// Both products are arranged transposed so that a lane owns ONE query column: the softmax maximum and sum of a
// query are reductions over the lane's own 16 registers plus one cross-half shuffle, and the rescale of O is a
// per-lane scalar.  K and V tiles are staged once per workgroup in LDS (all heads of the group share them), V
// transposed on the way in because the contraction index (keys) has to be contiguous in an MFMA operand.
// The MFMA k-slots of the second product are the lane's own S^T registers, in the order the hardware leaves them:
// slot (half, j) of the first MFMA is key 4*half + j (j < 4) or 8 + 4*half + j - 4; the V^T operand is read from LDS
// with the same key order, so no data moves between lanes.
//
// Same result as the per-token kernel of attn.hip (ggml's soft_max + mul_mat of the attention block, reached from
// rpc_server::graph_compute, third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451)
// except that Q and the probabilities are rounded to f16 for the matrix cores; sums are f32.

#include "attn.hpp"

namespace mesh {

constexpr int PF_HD = 128;
constexpr int PF_TILE = 32;                 // queries per workgroup and keys per step
constexpr int PF_KPITCH = PF_HD + 8;        // halfs per key row of the K tile in LDS (bank-conflict padding)
constexpr int PF_VPITCH = PF_TILE / 2 + 2;  // dwords (key pairs) per dim row of the transposed V tile

// Column (dword) of key pair kp in dim row `dim` of the transposed V tile.  Rows 32 apart start on the same LDS bank
// (32 * 18 dwords is a multiple of the 64 banks), and the staging writes of a wave touch four such rows at once; the
// XOR moves them onto different banks.  It keeps dwords 2j, 2j + 1 neighbours, which the 8-byte fragment reads need.
__device__ __forceinline__ int pf_vcol(int dim, int kp) { return kp ^ ((dim >> 5) << 2); }
constexpr float PF_RESCALE_STEP = 8.f;      // the softmax reference moves only when the running maximum exceeds it by this (log2)

typedef _Float16 pf_h8 __attribute__((ext_vector_type(8)));
typedef _Float16 pf_h2 __attribute__((ext_vector_type(2)));
typedef float pf_f16v __attribute__((ext_vector_type(16)));
typedef uint32_t pf_u4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t pf_pack(float a, float b) {
    const pf_h2 h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
}

// the 8 values a (key, piece) pair contributes to a tile, as packed f16
template <int TYPE>
__device__ __forceinline__ uint4 pf_row_piece(const uint8_t *row, int piece) {
    const KvRaw<TYPE> r = kv_load<TYPE, PF_HD>(row, piece * 8);
    if constexpr (TYPE == MESH_F16) {
        return r.v;
    } else {
        float u[8];
        const float d = kv_decode<TYPE>(r, u);
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] = (u[e] - KvAffine<TYPE>::off) * d;
        return make_uint4(pf_pack(u[0], u[1]), pf_pack(u[2], u[3]), pf_pack(u[4], u[5]), pf_pack(u[6], u[7]));
    }
}

// NP: (key, 8-dim piece) pairs of a tile one thread carries, at least 512 / (threads of the workgroup).
template <int KT, int VT, int NP>
__global__ __launch_bounds__(512) void attn_chunk_kernel(const AttnArgs a, int T, int pos0, int seq, int hpw) {
    constexpr int KRB = kv_row_bytes(KT, PF_HD), VRB = kv_row_bytes(VT, PF_HD);
    __shared__ __align__(16) _Float16 sK[PF_TILE * PF_KPITCH];
    __shared__ __align__(16) uint32_t sVt[PF_HD * PF_VPITCH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x;
    const int qcol = lane & 31, half = lane >> 5;
    const int qt = blockIdx.x, kvh = blockIdx.y;
    const int h = kvh * a.group + blockIdx.z * hpw + wave;
    const int tq = qt * PF_TILE + qcol;
    const bool q_live = tq < T;
    const int pos_q = pos0 + tq;

    // Q^T fragments of this lane's query, scaled so that the scores are in log2 units
    const float qs = a.scale * 1.44269504088896341f;
    pf_h8 qf[8];
    {
        const float *qp = a.q + ((size_t)(q_live ? tq : 0) * a.n_head + h) * PF_HD + 8 * half;
#pragma unroll
        for (int kc = 0; kc < 8; ++kc) {
            const float4 v0 = *reinterpret_cast<const float4 *>(qp + kc * 16), v1 = *reinterpret_cast<const float4 *>(qp + kc * 16 + 4);
            const float z = q_live ? qs : 0.f;
            const pf_u4 p = {pf_pack(v0.x * z, v0.y * z), pf_pack(v0.z * z, v0.w * z), pf_pack(v1.x * z, v1.y * z), pf_pack(v1.z * z, v1.w * z)};
            qf[kc] = __builtin_bit_cast(pf_h8, p);
        }
    }
    pf_f16v o[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    const size_t base = ((size_t)seq * a.n_kv + kvh) * a.n_ctx;
    const int q_end = qt * PF_TILE + PF_TILE < T ? qt * PF_TILE + PF_TILE : T;      // queries of this tile: [qt*32, q_end)
    const int n_keys = pos0 + q_end;                                                // keys any of them may see
    // The rows of a tile travel through registers: a thread fetches its share of tile k0 + 32 right after it has written
    // that of tile k0 to LDS, so the loads are in flight while the tile is multiplied.  K: (key, 8-dim piece) pairs, 16
    // bytes each.  V: the same 8 dims of two neighbouring keys, so that the transposed tile is written as dwords.
    // Rows past the context end are clamped (masked below).
    constexpr int NPV = (NP + 1) / 2;
    uint4 rk[NP], rv[NPV][2];
    auto fetch_tile = [&](int k0) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int p = tid + i * nthreads;
            if (p < PF_TILE * 16) {
                int kr = k0 + (p >> 4);
                kr = kr < a.n_ctx ? kr : a.n_ctx - 1;
                rk[i] = pf_row_piece<KT>(a.kcache + (base + kr) * KRB, p & 15);
            }
        }
#pragma unroll
        for (int i = 0; i < NPV; ++i) {
            const int p = tid + i * nthreads;
            if (p < PF_TILE * 8) {
                int kr0 = k0 + 2 * (p >> 4), kr1 = kr0 + 1;
                kr0 = kr0 < a.n_ctx ? kr0 : a.n_ctx - 1;
                kr1 = kr1 < a.n_ctx ? kr1 : a.n_ctx - 1;
                rv[i][0] = pf_row_piece<VT>(a.vcache + (base + kr0) * VRB, p & 15);
                rv[i][1] = pf_row_piece<VT>(a.vcache + (base + kr1) * VRB, p & 15);
            }
        }
    };
    fetch_tile(0);
    for (int k0 = 0; k0 < n_keys; k0 += PF_TILE) {
        // the K tile as it is
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int p = tid + i * nthreads;
            if (p < PF_TILE * 16) *reinterpret_cast<uint4 *>(sK + (p >> 4) * PF_KPITCH + (p & 15) * 8) = rk[i];
        }
        // the V tile transposed: 8 dwords, one per dim, each holding the pair of keys
#pragma unroll
        for (int i = 0; i < NPV; ++i) {
            const int p = tid + i * nthreads;
            if (p < PF_TILE * 8) {
                const int kp = p >> 4, piece = p & 15;
                const uint32_t w0[4] = {rv[i][0].x, rv[i][0].y, rv[i][0].z, rv[i][0].w}, w1[4] = {rv[i][1].x, rv[i][1].y, rv[i][1].z, rv[i][1].w};
                uint32_t *dst = sVt + piece * 8 * PF_VPITCH + pf_vcol(piece * 8, kp);
#pragma unroll
                for (int e2 = 0; e2 < 4; ++e2) {
                    dst[(2 * e2) * PF_VPITCH] = (w0[e2] & 0xffffu) | (w1[e2] << 16);
                    dst[(2 * e2 + 1) * PF_VPITCH] = (w0[e2] >> 16) | (w1[e2] & 0xffff0000u);
                }
            }
        }
        __syncthreads();
        if (k0 + PF_TILE < n_keys) fetch_tile(k0 + PF_TILE);

        // S^T = K . Q^T : lane (key row = lane % 32 of the A operand, query column = lane % 32 of the result)
        pf_f16v s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
        for (int kc = 0; kc < 8; ++kc) {
            const pf_h8 kf = *reinterpret_cast<const pf_h8 *>(sK + qcol * PF_KPITCH + kc * 16 + 8 * half);
            s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[kc], s, 0, 0, 0);
        }
        // register i of the result is key k0 + 8 * (i / 4) + 4 * half + i % 4 for query qcol.  Only a tile that reaches
        // past the first query's position has anything to mask (a dead query column has q = 0 and is never stored).
        if (k0 + PF_TILE - 1 > pos0 + qt * PF_TILE) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = k0 + 8 * (i >> 2) + 4 * half + (i & 3);
                s[i] = key <= pos_q ? s[i] : -INFINITY;
            }
        }
        float mx = s[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        // m is the reference the exponentials are taken against.  It follows the running maximum only when that has
        // moved by more than PF_RESCALE_STEP (log2 units), so that most steps skip the rescale of the 64 accumulator
        // registers; in between p <= 2^PF_RESCALE_STEP, which f16 holds comfortably.  (Key 0 is visible to every
        // query, so after the first tile m is finite for every live column.)
        if (__builtin_amdgcn_ballot_w64(mx > m + PF_RESCALE_STEP) != 0ull) {
            const float m_new = mx > m + PF_RESCALE_STEP ? mx : m;
            const float corr = exp2f(m - m_new);                    // exp2(-inf) = 0 while nothing is accumulated; 1 for lanes that stay
            l *= corr;
            m = m_new;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[db][i] *= corr;
        }
        float p[16], ps = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) { p[i] = __builtin_amdgcn_exp2f(s[i] - m); ps += p[i]; }     // s - m <= PF_RESCALE_STEP; far below, 0
        ps += __shfl_xor(ps, 32);
        l += ps;
        // P^T as the B operand: the lane's own registers, 8 per MFMA
        const pf_u4 pu1 = {pf_pack(p[0], p[1]), pf_pack(p[2], p[3]), pf_pack(p[4], p[5]), pf_pack(p[6], p[7])};
        const pf_u4 pu2 = {pf_pack(p[8], p[9]), pf_pack(p[10], p[11]), pf_pack(p[12], p[13]), pf_pack(p[14], p[15])};
        const pf_h8 p1 = __builtin_bit_cast(pf_h8, pu1), p2 = __builtin_bit_cast(pf_h8, pu2);
#pragma unroll
        for (int db = 0; db < 4; ++db) {
            // dim row db * 32 + qcol, this half's keys: key pairs 2 * half + 4 * j (+ 1), j = 0 .. 3
            const uint32_t *vrow = sVt + (db * 32 + qcol) * PF_VPITCH + 2 * half;
            const uint2 a0 = *reinterpret_cast<const uint2 *>(vrow + 4 * (0 ^ db)), a1 = *reinterpret_cast<const uint2 *>(vrow + 4 * (1 ^ db));
            const uint2 a2 = *reinterpret_cast<const uint2 *>(vrow + 4 * (2 ^ db)), a3 = *reinterpret_cast<const uint2 *>(vrow + 4 * (3 ^ db));
            const pf_u4 v1 = {a0.x, a0.y, a1.x, a1.y}, v2 = {a2.x, a2.y, a3.x, a3.y};
            o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_h8, v1), p1, o[db], 0, 0, 0);
            o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_h8, v2), p2, o[db], 0, 0, 0);
        }
        __syncthreads();        // the tiles are overwritten by the next step
    }
    if (a.out16_k8) {
        // f16, in the k8-major layout the output projection's GEMM reads (gemm.hpp); the padding columns of the last
        // block of 16 tokens are written as zeros
        const int t_pad = (T + 15) & ~15;
        if (tq < t_pad) {
            const float inv = q_live ? 1.0f / l : 0.f;
            const size_t KK = (size_t)a.n_head * PF_HD;
            _Float16 *ob = a.out16_k8 + (size_t)(tq >> 4) * 16 * KK + (size_t)(tq & 15) * 8;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    const size_t kk = (size_t)h * PF_HD + db * 32 + 8 * i4 + 4 * half;
                    *reinterpret_cast<uint2 *>(ob + (kk >> 3) * 128 + (kk & 7)) =
                        make_uint2(pf_pack(o[db][4 * i4] * inv, o[db][4 * i4 + 1] * inv), pf_pack(o[db][4 * i4 + 2] * inv, o[db][4 * i4 + 3] * inv));
                }
        }
    } else if (q_live) {
        const float inv = 1.0f / l;
        float *op = a.out + ((size_t)tq * a.n_head + h) * PF_HD;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4)
                *reinterpret_cast<float4 *>(op + db * 32 + 8 * i4 + 4 * half) =
                    make_float4(o[db][4 * i4] * inv, o[db][4 * i4 + 1] * inv, o[db][4 * i4 + 2] * inv, o[db][4 * i4 + 3] * inv);
    }
}

int attention_chunk(const AttnArgs &a, int T, int pos0, int seq, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (a.head_dim != PF_HD) return fail(MESH_ERR_UNSUPPORTED, "attention_chunk: head_dim %d (128 only)", a.head_dim);
    if (a.group < 1 || a.n_head != a.group * a.n_kv || pos0 < 0 || pos0 + T > a.n_ctx || seq < 0)
        return fail(MESH_ERR_INVALID, "attention_chunk: bad head layout or chunk [%d, %d) outside the context of %d", pos0, pos0 + T, a.n_ctx);
    int hpw = a.group;                       // heads (waves) per workgroup: the largest divisor of the group up to 8
    while (hpw > 8 || a.group % hpw) --hpw;
    const dim3 grid((unsigned)((T + PF_TILE - 1) / PF_TILE), (unsigned)a.n_kv, (unsigned)(a.group / hpw));
    const dim3 block((unsigned)(64 * hpw));
#define MESH_CHUNK_LAUNCH(KT, VT)                                                                                         \
    do {                                                                                                                  \
        if (hpw >= 4) MESH_LAUNCH((attn_chunk_kernel<KT, VT, 2>), grid, block, 0, stream, a, T, pos0, seq, hpw);        \
        else if (hpw >= 2) MESH_LAUNCH((attn_chunk_kernel<KT, VT, 4>), grid, block, 0, stream, a, T, pos0, seq, hpw);   \
        else MESH_LAUNCH((attn_chunk_kernel<KT, VT, 8>), grid, block, 0, stream, a, T, pos0, seq, hpw);                  \
    } while (0)
    if (a.k_type == MESH_F16 && a.v_type == MESH_F16) MESH_CHUNK_LAUNCH(MESH_F16, MESH_F16);
    else if (a.k_type == MESH_Q8_0 && a.v_type == MESH_Q4_0) MESH_CHUNK_LAUNCH(MESH_Q8_0, MESH_Q4_0);
    else if (a.k_type == MESH_Q4_0 && a.v_type == MESH_Q4_0) MESH_CHUNK_LAUNCH(MESH_Q4_0, MESH_Q4_0);
    else return fail(MESH_ERR_UNSUPPORTED, "attention_chunk: KV cache types %d/%d", a.k_type, a.v_type);
#undef MESH_CHUNK_LAUNCH
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

}  // namespace mesh
