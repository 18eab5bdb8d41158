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

#include <algorithm>

#include "attn.hpp"

namespace mesh {

constexpr int PF_HD = 128;
constexpr int PF_TILE = 32;                 // queries per workgroup
constexpr int PF_KPITCH = PF_HD + 8;        // halfs per key row of the K tile in LDS (bank-conflict padding)

// Column (dword) of key pair kp in dim row `dim` of the transposed V tile.  Rows 32 apart start on the same LDS bank
// (32 rows of 18 or 34 dwords are a multiple of the 64 banks), and the staging writes of a wave touch four such rows at once; the
// XOR moves them onto different banks.  It keeps dwords 2j, 2j + 1 neighbours, which the 8-byte fragment reads need.
__device__ __forceinline__ int pf_vcol(int dim, int kp) { return kp ^ ((dim >> 5) << 2); }
constexpr int PF_EXPAND_MIN_T = 128;         // chunks from this many tokens decode a quantised cache to f16 once, ahead of the walk
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

// NT: tiles of 32 keys per step (1 or 2; two give the wave two independent score chains and half the barriers per key, at
// ~50 more registers).  NP: (key, 8-dim piece) pairs of a step one thread carries in registers, at least 512 NT /
// (threads of the workgroup); 0 for small workgroups, which load each step's rows where they write them.
template <int KT, int VT, int NP, int NT>
__global__ __launch_bounds__(512) void attn_chunk_kernel(const AttnArgs a, int T, int pos0, int seq, int hpw, int fwd_from, int qtiles, int n_ksplit) {
    constexpr int KRB = kv_row_bytes(KT, PF_HD), VRB = kv_row_bytes(VT, PF_HD);
    constexpr int PF_KEYS = 32 * NT;                // keys per step
    constexpr int PF_VPITCH = PF_KEYS / 2 + 2;      // dwords (key pairs) per dim row of the transposed V tile
    __shared__ __align__(16) _Float16 sK[PF_KEYS * PF_KPITCH];
    __shared__ __align__(16) uint32_t sVt[PF_HD * PF_VPITCH];
    const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x;
    // wave -> (head of the workgroup, one of its `qtiles` consecutive query tiles): groups of fewer than four heads fill the
    // workgroup with several query tiles of the same heads, which share the K / V tiles like heads do
    const int wave = (tid >> 6) % hpw, qtl = (tid >> 6) / hpw;
    const int qcol = lane & 31, half = lane >> 5;
    // the last query tile of a chunk walks the most keys: the launch hands the tiles out from the last one backwards, so
    // that the longest walks start first when the workgroups do not all fit on the chip at once
    // (a launch whose workgroups all fit at once, two per CU, runs its second half forwards: see attention_chunk)
    const int lin = (int)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z));
    const int qg = lin >= fwd_from ? (int)blockIdx.x : (int)(gridDim.x - 1 - blockIdx.x), kvh = blockIdx.y;
    const int qt = qg * qtiles + qtl;           // (past the last tile of the chunk: a wave without queries, q_live false)
    // blockIdx.z = (head group, key split): with n_ksplit > 1 the workgroup walks one n_ksplit-th of the keys and leaves
    // an un-normalised partial for attn_combine_kernel (short chunks on a long history, which have few query tiles)
    const int ks = (int)blockIdx.z % n_ksplit;
    const int h = kvh * a.group + ((int)blockIdx.z / n_ksplit) * hpw + wave;
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
    const int n_keys_own = qt * PF_TILE < T ? pos0 + q_end : 0;                     // keys any of them may see
    const int wg_end = (qg + 1) * qtiles * PF_TILE < T ? (qg + 1) * qtiles * PF_TILE : T;
    const int n_keys_wg = pos0 + wg_end;                                            // keys the workgroup's last tile walks
    const int per_split = (((n_keys_wg + n_ksplit - 1) / n_ksplit) + 63) & ~63;
    const int k_lo = ks * per_split;
    const int n_keys = k_lo + per_split < n_keys_wg ? k_lo + per_split : n_keys_wg;   // end of this workgroup's walk
    const int n_keys_mine = n_keys_own < n_keys ? n_keys_own : n_keys;              // and of this wave's
    // K is staged as it is: (key, 8-dim piece) pairs, 16 bytes each.  V is staged transposed: an item is the same 8 dims
    // of two neighbouring keys, written as 8 dwords, one per dim, each holding the pair of keys.  Rows past the context
    // end are clamped (masked below).
    auto k_row = [&](int k0, int p) {
        int kr = k0 + (p >> 4);
        kr = kr < a.n_ctx ? kr : a.n_ctx - 1;
        return pf_row_piece<KT>(a.kcache + (base + kr) * KRB, p & 15);
    };
    auto v_row = [&](int k0, int p, int second) {
        int kr = k0 + 2 * (p >> 4) + second;
        kr = kr < a.n_ctx ? kr : a.n_ctx - 1;
        return pf_row_piece<VT>(a.vcache + (base + kr) * VRB, p & 15);
    };
    auto k_put = [&](int p, const uint4 &r) { *reinterpret_cast<uint4 *>(sK + (p >> 4) * PF_KPITCH + (p & 15) * 8) = r; };
    auto v_put = [&](int p, const uint4 &r0, const uint4 &r1) {
        const int kp = p >> 4, piece = p & 15;
        const uint32_t w0[4] = {r0.x, r0.y, r0.z, r0.w}, w1[4] = {r1.x, r1.y, r1.z, r1.w};
        uint32_t *dst = sVt + piece * 8 * PF_VPITCH + pf_vcol(piece * 8, kp);
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            dst[(2 * e2) * PF_VPITCH] = (w0[e2] & 0xffffu) | (w1[e2] << 16);
            dst[(2 * e2 + 1) * PF_VPITCH] = (w0[e2] >> 16) | (w1[e2] & 0xffff0000u);
        }
    };
    // With NP > 0 the rows of a step travel through registers: a thread fetches its share of step k0 + 64 right after it
    // has written that of step k0 to LDS, so the loads are in flight while the step is multiplied.
    constexpr int NPK = NP > 0 ? NP : 1, NPV = NP > 0 ? (NP + 1) / 2 : 1;
    uint4 rk[NPK], rv[NPV][2];
    auto fetch_step = [&](int k0) {
#pragma unroll
        for (int i = 0; i < NPK; ++i) {
            const int p = tid + i * nthreads;
            if (p < PF_KEYS * 16) rk[i] = k_row(k0, p);
        }
#pragma unroll
        for (int i = 0; i < NPV; ++i) {
            const int p = tid + i * nthreads;
            if (p < PF_KEYS * 8) { rv[i][0] = v_row(k0, p, 0); rv[i][1] = v_row(k0, p, 1); }
        }
    };
    if constexpr (NP > 0) fetch_step(k_lo);
    for (int k0 = k_lo; k0 < n_keys; k0 += PF_KEYS) {
        if constexpr (NP > 0) {
#pragma unroll
            for (int i = 0; i < NPK; ++i) {
                const int p = tid + i * nthreads;
                if (p < PF_KEYS * 16) k_put(p, rk[i]);
            }
#pragma unroll
            for (int i = 0; i < NPV; ++i) {
                const int p = tid + i * nthreads;
                if (p < PF_KEYS * 8) v_put(p, rv[i][0], rv[i][1]);
            }
        } else {
            for (int p = tid; p < PF_KEYS * 16; p += nthreads) k_put(p, k_row(k0, p));
            for (int p = tid; p < PF_KEYS * 8; p += nthreads) v_put(p, v_row(k0, p, 0), v_row(k0, p, 1));
        }
        __syncthreads();
        if constexpr (NP > 0) {
            if (k0 + PF_KEYS < n_keys) fetch_step(k0 + PF_KEYS);
        }
        if (k0 < n_keys_mine) {     // (an earlier query tile of the workgroup is done before the last one)
        // the second 32 keys of the step lie past every query of the tile at the end of the walk
        const bool two = NT == 2 && k0 + 32 < n_keys_mine;

        // S^T = K . Q^T, two tiles of 32 keys x 32 queries: lane (key row = lane % 32 of the A operand, query column =
        // lane % 32 of the result); two independent accumulation chains
        pf_f16v s[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[t][i] = t == 0 ? 0.f : (two ? 0.f : -INFINITY);
        if (two) {
#pragma unroll
            for (int kc = 0; kc < 8; ++kc)
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const pf_h8 kf = *reinterpret_cast<const pf_h8 *>(sK + (32 * t + qcol) * PF_KPITCH + kc * 16 + 8 * half);
                    s[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[kc], s[t], 0, 0, 0);
                }
        } else {
#pragma unroll
            for (int kc = 0; kc < 8; ++kc) {
                const pf_h8 kf = *reinterpret_cast<const pf_h8 *>(sK + qcol * PF_KPITCH + kc * 16 + 8 * half);
                s[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[kc], s[0], 0, 0, 0);
            }
        }
        // register i of tile t is key k0 + 32 * t + 8 * (i / 4) + 4 * half + i % 4 for query qcol.  Only a step that
        // reaches past the first query's position has anything to mask (a dead query column has q = 0 and is never stored).
        if (k0 + PF_KEYS - 1 > pos0 + qt * PF_TILE) {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = k0 + 32 * t + 8 * (i >> 2) + 4 * half + (i & 3);
                    s[t][i] = key <= pos_q ? s[t][i] : -INFINITY;
                }
        }
        float mxt[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) mxt[t] = s[t][0];
#pragma unroll
        for (int i = 1; i < 16; ++i)
#pragma unroll
            for (int t = 0; t < NT; ++t) mxt[t] = fmaxf(mxt[t], s[t][i]);
        float mx = NT == 2 ? fmaxf(mxt[0], mxt[NT - 1]) : mxt[0];
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        // m is the reference the exponentials are taken against.  It follows the running maximum only when that has
        // moved by more than PF_RESCALE_STEP (log2 units), so that most steps skip the rescale of the 64 accumulator
        // registers; in between p <= 2^PF_RESCALE_STEP, which f16 holds comfortably.  (Key 0 is visible to every
        // query, so after the first step m is finite for every live column.)
        if (__builtin_amdgcn_ballot_w64(mx > m + PF_RESCALE_STEP) != 0ull) {
            const float m_new = mx > m + PF_RESCALE_STEP ? mx : m;
            // 1 for lanes that stay, exp2(-inf) = 0 while nothing is accumulated.  A query that has seen no key yet and
            // sees none in this step either (a key split that begins inside the tile's position range) has m = m_new =
            // -inf: its l and o are still zero, and -inf - -inf must not reach them as NaN.
            const float corr = m_new == -INFINITY ? 1.f : exp2f(m - m_new);
            l *= corr;
            m = m_new;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[db][i] *= corr;
        }
        // (Without key splits key 0 is visible to every query, so m is finite from the first step on.  In a later split a
        // query may see no key at all: all its scores are -inf and so is m; the reference 0 then gives p = 0, not NaN.)
        const float mref = m == -INFINITY ? 0.f : m;
        // P^T as the B operand: the lane's own registers, 8 per MFMA
        pf_h8 pf[NT][2];
        float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            float p[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) p[i] = __builtin_amdgcn_exp2f(s[t][i] - mref);  // s - m <= PF_RESCALE_STEP; far below, 0
#pragma unroll
            for (int i = 0; i < 16; i += 2) { ps0 += p[i]; ps1 += p[i + 1]; }
            const pf_u4 pu1 = {pf_pack(p[0], p[1]), pf_pack(p[2], p[3]), pf_pack(p[4], p[5]), pf_pack(p[6], p[7])};
            const pf_u4 pu2 = {pf_pack(p[8], p[9]), pf_pack(p[10], p[11]), pf_pack(p[12], p[13]), pf_pack(p[14], p[15])};
            pf[t][0] = __builtin_bit_cast(pf_h8, pu1);
            pf[t][1] = __builtin_bit_cast(pf_h8, pu2);
        }
        float ps = ps0 + ps1;
        ps += __shfl_xor(ps, 32);
        l += ps;
#pragma unroll
        for (int db = 0; db < 4; ++db) {
            // dim row db * 32 + qcol, this half's keys of tile t: key pairs 16 * t + 2 * half + 4 * j (+ 1), j = 0 .. 3
            const uint32_t *vrow = sVt + (db * 32 + qcol) * PF_VPITCH + 2 * half;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (t == 1 && !two) break;
                const uint2 a0 = *reinterpret_cast<const uint2 *>(vrow + 16 * t + 4 * (0 ^ db)), a1 = *reinterpret_cast<const uint2 *>(vrow + 16 * t + 4 * (1 ^ db));
                const uint2 a2 = *reinterpret_cast<const uint2 *>(vrow + 16 * t + 4 * (2 ^ db)), a3 = *reinterpret_cast<const uint2 *>(vrow + 16 * t + 4 * (3 ^ db));
                const pf_u4 v1 = {a0.x, a0.y, a1.x, a1.y}, v2 = {a2.x, a2.y, a3.x, a3.y};
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_h8, v1), pf[t][0], o[db], 0, 0, 0);
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_h8, v2), pf[t][1], o[db], 0, 0, 0);
            }
        }
        }
        __syncthreads();        // the tiles are overwritten by the next step
    }
    if (n_ksplit > 1) {
        // un-normalised partial and (maximum, sum) of this key split, in the layout of the split-KV decode kernels
        if (q_live) {
            const size_t prow = ((size_t)tq * a.n_head + h) * n_ksplit + ks;
            float *pp = a.part + prow * PF_HD;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4)
                    *reinterpret_cast<float4 *>(pp + db * 32 + 8 * i4 + 4 * half) =
                        make_float4(o[db][4 * i4], o[db][4 * i4 + 1], o[db][4 * i4 + 2], o[db][4 * i4 + 3]);
            if (half == 0) { a.ml[prow * 2] = m; a.ml[prow * 2 + 1] = l; }
        }
        return;
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

// Rows [0, n_keys) of one sequence's K and V, every KV head, as f16 rows [n_kv][n_ctx][128] (the values the staging
// of attn_chunk_kernel would decode): one thread per (row, 8-dim piece).
template <int KT, int VT>
__global__ __launch_bounds__(256) void kv_expand_kernel(const uint8_t *kcache, const uint8_t *vcache, uint4 *k16, uint4 *v16, int n_keys, int n_ctx,
                                                        int n_kv, int seq) {
    constexpr int KRB = kv_row_bytes(KT, PF_HD), VRB = kv_row_bytes(VT, PF_HD);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int piece = (int)(idx & 15);
    const size_t row = idx >> 4;
    if (row >= (size_t)n_kv * n_keys) return;
    const int kvh = (int)(row / n_keys), key = (int)(row % n_keys);
    const size_t src = ((size_t)seq * n_kv + kvh) * n_ctx + key, dst = (size_t)kvh * n_ctx + key;
    k16[dst * 16 + piece] = pf_row_piece<KT>(kcache + src * KRB, piece);
    v16[dst * 16 + piece] = pf_row_piece<VT>(vcache + src * VRB, piece);
}

static int pf_n_cu() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) n = p.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

int attention_chunk(const AttnArgs &a_in, int T, int pos0, int seq, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    AttnArgs a = a_in;
    if (a.head_dim != PF_HD) return fail(MESH_ERR_UNSUPPORTED, "attention_chunk: head_dim %d (128 only)", a.head_dim);
    if (a.group < 1 || a.n_head != a.group * a.n_kv || pos0 < 0 || pos0 + T > a.n_ctx || seq < 0)
        return fail(MESH_ERR_INVALID, "attention_chunk: bad head layout or chunk [%d, %d) outside the context of %d", pos0, pos0 + T, a.n_ctx);
    if (a.k_type != MESH_F16 && a.chunk_kv16 && T >= PF_EXPAND_MIN_T) {
        // Every query tile's workgroup would decode the quantised rows it walks.  Decode them once instead, into the
        // caller's f16 scratch, and run the f16 kernel on that: the same values reach the matrix cores.
        const int n_keys = pos0 + T;
        uint4 *k16 = reinterpret_cast<uint4 *>(a.chunk_kv16), *v16 = k16 + (size_t)a.n_kv * a.n_ctx * 16;
        const unsigned blocks = (unsigned)(((size_t)a.n_kv * n_keys * 16 + 255) / 256);
        if (a.k_type == MESH_Q8_0 && a.v_type == MESH_Q4_0)
            MESH_LAUNCH((kv_expand_kernel<MESH_Q8_0, MESH_Q4_0>), dim3(blocks), dim3(256), 0, stream, a.kcache, a.vcache, k16, v16, n_keys, a.n_ctx, a.n_kv, seq);
        else if (a.k_type == MESH_Q4_0 && a.v_type == MESH_Q4_0)
            MESH_LAUNCH((kv_expand_kernel<MESH_Q4_0, MESH_Q4_0>), dim3(blocks), dim3(256), 0, stream, a.kcache, a.vcache, k16, v16, n_keys, a.n_ctx, a.n_kv, seq);
        else return fail(MESH_ERR_UNSUPPORTED, "attention_chunk: KV cache types %d/%d", a.k_type, a.v_type);
        MESH_LAUNCH_CHECK();
        a.kcache = reinterpret_cast<const uint8_t *>(k16);
        a.vcache = reinterpret_cast<const uint8_t *>(v16);
        a.k_type = a.v_type = MESH_F16;
        seq = 0;
    }
    int hpw = a.group;                       // heads (waves) per workgroup: the largest divisor of the group up to 8
    while (hpw > 8 || a.group % hpw) --hpw;
    // eight heads per KV head: two workgroups of four waves when one of eight per (query tile, KV head) would leave CUs idle
    if (hpw == 8 && ((T + PF_TILE - 1) / PF_TILE) * a.n_kv < pf_n_cu()) hpw = 4;
    // groups of fewer than four heads: several consecutive query tiles per workgroup (they share the K / V tiles like heads do)
    const int qtiles = hpw >= 4 ? 1 : hpw == 1 ? 4 : 2;
    const int waves = hpw * qtiles, n_tiles = (T + PF_TILE - 1) / PF_TILE;
    dim3 grid((unsigned)((n_tiles + qtiles - 1) / qtiles), (unsigned)a.n_kv, (unsigned)(a.group / hpw));
    const dim3 block((unsigned)(64 * waves));
    // A short chunk on a long history has few query tiles, each with a long walk: split the keys of every walk over
    // several workgroups (partials in the caller's split buffers, merged by attn_combine_kernel) until the launch has a
    // workgroup per CU, at most 8 ways, at least 256 keys each, within the buffers' rows of (token, split).
    int n_ksplit = 1;
    {
        const int wgs = (int)(grid.x * grid.y * grid.z), n_keys = pos0 + T;
        if (a.part && a.ml && a.part_rows > 0 && wgs < pf_n_cu())
            n_ksplit = std::max(1, std::min(std::min(pf_n_cu() / wgs, 8), std::min(n_keys / 256, (int)(a.part_rows / (size_t)T))));
        if (n_ksplit > ATTN_SPLITS_CAP) n_ksplit = ATTN_SPLITS_CAP;
    }
    grid.z *= (unsigned)n_ksplit;
    // When the whole launch is resident at once with two workgroups per CU, the hardware has been seen to give a CU
    // workgroups i and i + (half the launch): handing the second half its query tiles in forward order pairs a long
    // walk with a short one on every CU.  (A guess about placement costs nothing when wrong: the tiles are the same.)
    const int total = (int)(grid.x * grid.y * grid.z);
    // (half the launch has to be whole rows of query tiles: an even number of (KV head, head group) rows)
    const int fwd_from = (n_ksplit == 1 && waves <= 4 && (grid.y * grid.z) % 2 == 0 && total <= 2 * pf_n_cu() && total > pf_n_cu()) ? total / 2 : INT32_MAX;
    // (Two tiles per step everywhere.  With 5 heads per KV head one tile per step keeps the kernel under 170 registers, so
    // that two 5-wave workgroups share a CU instead of one: measured slower, 16.5 against 14.8 ms over 32 layers of 4096 tokens.)
    // NP by the threads of the workgroup: 1024 / threads pairs each, rounded up
#define MESH_CHUNK_LAUNCH(KT, VT)                                                                                         \
    do {                                                                                                                  \
        if (waves == 8) MESH_LAUNCH((attn_chunk_kernel<KT, VT, 2, 2>), grid, block, 0, stream, a, T, pos0, seq, hpw, fwd_from, qtiles, n_ksplit);      \
        else if (waves == 6) MESH_LAUNCH((attn_chunk_kernel<KT, VT, 3, 2>), grid, block, 0, stream, a, T, pos0, seq, hpw, fwd_from, qtiles, n_ksplit); \
        else MESH_LAUNCH((attn_chunk_kernel<KT, VT, 4, 2>), grid, block, 0, stream, a, T, pos0, seq, hpw, fwd_from, qtiles, n_ksplit);                  \
    } while (0)
    if (a.k_type == MESH_F16 && a.v_type == MESH_F16) MESH_CHUNK_LAUNCH(MESH_F16, MESH_F16);
    else if (a.k_type == MESH_Q8_0 && a.v_type == MESH_Q4_0) MESH_CHUNK_LAUNCH(MESH_Q8_0, MESH_Q4_0);
    else if (a.k_type == MESH_Q4_0 && a.v_type == MESH_Q4_0) MESH_CHUNK_LAUNCH(MESH_Q4_0, MESH_Q4_0);
    else return fail(MESH_ERR_UNSUPPORTED, "attention_chunk: KV cache types %d/%d", a.k_type, a.v_type);
#undef MESH_CHUNK_LAUNCH
    MESH_LAUNCH_CHECK();
    if (n_ksplit > 1) {
        a.n_splits = n_ksplit;
        return attention_combine(a, T, stream);
    }
    return MESH_OK;
}

}  // namespace mesh
