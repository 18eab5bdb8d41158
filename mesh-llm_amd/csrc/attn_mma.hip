// GQA decode attention on the matrix cores, for batches of decode tokens over long KV ranges.
//
// Same contract as attn_kernel of attn.hip (token t attends to cache positions [0, pos[t]] of sequence seq[t]; split-KV
// partials merged by attn_combine_kernel), same place in the worker's graph (flash_attn_ext under -fa on,
// mesh-llm/src/inference/launch.rs:1350-1353).  The per-key work of that kernel is vector ALU work that grows with the
// number of query heads per KV head; here the query heads of a KV head are the 16 columns of an MFMA tile, so the
// cost per key does not depend on the group size (up to 16), and the cache rows cross the vector ALUs only to be
// converted (quantised rows) and transposed (V).
//
// A workgroup takes one (split, kv head, token); each of its 4 waves walks its own 16-key blocks of the range and
// keeps its own running softmax, merged at the end:
//   S^T (16 keys x 16 heads)  = K . Q^T      v_mfma_f32_16x16x32_f16 per 32 dims; the K operand is the cache row as it
//                                             lies in memory (lane = key, 8 consecutive dims), loaded straight from HBM
//   O^T (16 dims x 16 heads) += V^T . P^T     v_mfma_f32_16x16x16_f16 per 16 dims; the result registers of S^T (4 keys of
//                                             one head per lane) are the P^T operand as they are; V^T needs the keys
//                                             along a lane, so V rows are transposed through a wave-private LDS tile
// A lane owns one head column throughout: softmax maximum and sum are reductions over its 4 registers and the 4
// lane groups, the rescale of O is a per-lane scalar.
// Q and the probabilities are rounded to f16 for the matrix cores; sums are f32.

#include "attn.hpp"
#include "q16.hpp"

namespace mesh {

constexpr int MMA_THREADS = 256, MMA_WAVES = 4, MMA_KEYS = 16;
constexpr float MMA_RESCALE_STEP = 8.f;  // log2 units
constexpr int MMA_VPITCH = 20;          // halfs per dim row of the transposed V tile (16 keys + padding, 8-byte aligned)

typedef _Float16 mm_h8 __attribute__((ext_vector_type(8)));
typedef _Float16 mm_h4 __attribute__((ext_vector_type(4)));
typedef _Float16 mm_h2 __attribute__((ext_vector_type(2)));
typedef float mm_f4 __attribute__((ext_vector_type(4)));
typedef uint32_t mm_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t mm_u2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t mm_pack(float a, float b) {
    const mm_h2 h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
}

// Bytes / nibbles -> f16 without conversions: 0x6400 | u is the half 1024 + u, so one packed subtraction of
// 1024 + offset leaves the signed quant exactly, and one packed multiply by the block scale (an f16 in the cache)
// gives d * q rounded to f16 -- the same value as the f32 product rounded once.
__device__ __forceinline__ uint32_t mm_scale_pair(uint32_t biased, _Float16 bias, mm_h2 d2) {
    const mm_h2 v = (__builtin_bit_cast(mm_h2, biased) - mm_h2{bias, bias}) * d2;
    return __builtin_bit_cast(uint32_t, v);
}

// the 8 values a lane fetched from a cache row as packed f16 (quantised rows are dequantised in f16, exactly as above)
template <int TYPE>
__device__ __forceinline__ uint4 mm_piece_f16(const KvRaw<TYPE> &r) {
    if constexpr (TYPE == MESH_F16) {
        return r.v;
    } else {
        const _Float16 d = __builtin_bit_cast(_Float16, r.d);
        const mm_h2 d2 = {d, d};
        if constexpr (TYPE == MESH_Q8_0) {
            const uint32_t a = r.v.x ^ 0x80808080u, b = r.v.y ^ 0x80808080u;       // int8 -> biased uint8
            const _Float16 bias = (_Float16)(1024.f + 128.f);
            return make_uint4(mm_scale_pair(__builtin_amdgcn_perm(0x64646464u, a, 0x04010400u), bias, d2),
                              mm_scale_pair(__builtin_amdgcn_perm(0x64646464u, a, 0x04030402u), bias, d2),
                              mm_scale_pair(__builtin_amdgcn_perm(0x64646464u, b, 0x04010400u), bias, d2),
                              mm_scale_pair(__builtin_amdgcn_perm(0x64646464u, b, 0x04030402u), bias, d2));
        } else {
            // byte i of the word holds elements 2i (low nibble) and 2i + 1 (high nibble)
            const uint32_t lo = r.v & 0x0F0F0F0Fu, hi = (r.v >> 4) & 0x0F0F0F0Fu;
            const _Float16 bias = (_Float16)(1024.f + 8.f);
            // pair k = elements (2k, 2k + 1) = (byte k of lo, byte k of hi); selector bytes 0-3 address hi, 4-7 address lo
            return make_uint4(mm_scale_pair(__builtin_amdgcn_perm(lo, hi, 0x0c000c04u) | 0x64006400u, bias, d2),
                              mm_scale_pair(__builtin_amdgcn_perm(lo, hi, 0x0c010c05u) | 0x64006400u, bias, d2),
                              mm_scale_pair(__builtin_amdgcn_perm(lo, hi, 0x0c020c06u) | 0x64006400u, bias, d2),
                              mm_scale_pair(__builtin_amdgcn_perm(lo, hi, 0x0c030c07u) | 0x64006400u, bias, d2));
        }
    }
}

__device__ __forceinline__ void mm_wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// grid (n_splits, n_kv, T), 256 threads.  group <= 16.
// (the arguments on the way to the first K / V loads come first, as scalars, so that they are preloaded into SGPRs:
// see gemv.hip)
template <int HD, int KT, int VT>
__global__ __launch_bounds__(MMA_THREADS) void attn_mma_kernel(const float *p_q, const int32_t *p_pos, const int32_t *p_seq,
                                                               const uint8_t *p_kcache, const uint8_t *p_vcache, int p_n_splits,
                                                               int p_n_ctx, int p_n_kv, int p_group, int p_n_head, float p_scale,
                                                               const AttnArgs a) {
    constexpr int NC = HD / 32;             // 32-dim chunks of the score product
    constexpr int NDB = HD / 16;            // 16-dim blocks of the output
    constexpr int KRB = kv_row_bytes(KT, HD), VRB = kv_row_bytes(VT, HD);
    // the transposed V tiles (one per wave) and, after the key loop, the per-wave results share this memory
    constexpr int STAGE_HALFS = MMA_WAVES * HD * MMA_VPITCH;
    constexpr int MERGE_FLOATS = MMA_WAVES * HD * 16;
    constexpr int SH_BYTES = STAGE_HALFS * 2 > MERGE_FLOATS * 4 ? STAGE_HALFS * 2 : MERGE_FLOATS * 4;
    __shared__ __align__(16) uint8_t s_raw[SH_BYTES];
    __shared__ float s_m[MMA_WAVES][16], s_l[MMA_WAVES][16];

    const int split = blockIdx.x, kvh = blockIdx.y, t = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;         // head column / key row of a tile, lane group
    const int G = p_group;
    const int seq = p_seq[t];
    const int n_keys = p_pos[t] + 1;
    const int per = (n_keys + p_n_splits - 1) / p_n_splits;
    const int j0 = split * per;
    const int j1 = j0 + per < n_keys ? j0 + per : n_keys;

    // Q^T operand: head column c, dims 32*cc + 8*g + j, in log2 units
    mm_h8 qf[NC];
    {
        const float qs = c < G ? p_scale * 1.44269504088896341f : 0.f;
        const float *qp = p_q + ((size_t)t * p_n_head + (size_t)kvh * G + (c < G ? c : 0)) * HD + 8 * g;
#pragma unroll
        for (int cc = 0; cc < NC; ++cc) {
            const float4 v0 = *reinterpret_cast<const float4 *>(qp + 32 * cc), v1 = *reinterpret_cast<const float4 *>(qp + 32 * cc + 4);
            const mm_u4 p = {mm_pack(v0.x * qs, v0.y * qs), mm_pack(v0.z * qs, v0.w * qs), mm_pack(v1.x * qs, v1.y * qs), mm_pack(v1.z * qs, v1.w * qs)};
            qf[cc] = __builtin_bit_cast(mm_h8, p);
        }
    }
    mm_f4 o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[db] = mm_f4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    _Float16 *sV = reinterpret_cast<_Float16 *>(s_raw) + wave * HD * MMA_VPITCH;
    const size_t base = ((size_t)seq * p_n_kv + kvh) * p_n_ctx;
    // what a lane fetches of a 16-key block: its key row c, dims 32*cc + 8*g .. + 8 of K and of V; rows past the range
    // are clamped to its last key (and masked below), so the fetch of the block after the last one is harmless
    // Blocks in flight per wave: quantised rows are 2.5 - 3.5 times smaller than f16 rows, so one block ahead leaves
    // too few bytes in flight to cover the memory latency; they run two ahead (20 more registers).
    constexpr int DEPTH = (KT == MESH_F16 && VT == MESH_F16) ? 1 : 2;
    constexpr int STEP = MMA_WAVES * MMA_KEYS;
    KvRaw<KT> kraw[DEPTH][NC];
    KvRaw<VT> vraw[DEPTH][NC];
    auto fetch = [&](KvRaw<KT> (&kr_)[NC], KvRaw<VT> (&vr_)[NC], int kb) {
        int kr = kb + c;
        kr = kr < j1 ? kr : j1 - 1;
        const uint8_t *krow = p_kcache + (base + kr) * KRB, *vrow = p_vcache + (base + kr) * VRB;
#pragma unroll
        for (int cc = 0; cc < NC; ++cc) kr_[cc] = kv_load<KT, HD>(krow, 32 * cc + 8 * g);
#pragma unroll
        for (int cc = 0; cc < NC; ++cc) vr_[cc] = kv_load<VT, HD>(vrow, 32 * cc + 8 * g);
    };
    const int kb0 = j0 + wave * MMA_KEYS;
    if (kb0 < j1) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) fetch(kraw[d], vraw[d], kb0 + d * STEP);
    }
    for (int kbb = kb0; kbb < j1; kbb += DEPTH * STEP) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int kb = kbb + d * STEP;
        if (kb >= j1) break;
        uint4 kf[NC], vf[NC];
#pragma unroll
        for (int cc = 0; cc < NC; ++cc) kf[cc] = mm_piece_f16<KT>(kraw[d][cc]);
#pragma unroll
        for (int cc = 0; cc < NC; ++cc) vf[cc] = mm_piece_f16<VT>(vraw[d][cc]);
        fetch(kraw[d], vraw[d], kb + DEPTH * STEP);      // rows of a later block travel while this one is worked on

        // S^T = K . Q^T : register i is key kb + 4*g + i for head c
        mm_f4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int cc = 0; cc < NC; ++cc)
            s = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(mm_h8, kf[cc]), qf[cc], s, 0, 0, 0);

        // V rows -> transposed tile: sV[dim][key]
#pragma unroll
        for (int cc = 0; cc < NC; ++cc) {
            const uint32_t w[4] = {vf[cc].x, vf[cc].y, vf[cc].z, vf[cc].w};
#pragma unroll
            for (int e = 0; e < 8; ++e)
                reinterpret_cast<uint16_t *>(sV)[(32 * cc + 8 * g + e) * MMA_VPITCH + c] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
        }

        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            s[i] = kb + 4 * g + i < j1 ? s[i] : -INFINITY;
            mx = fmaxf(mx, s[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        // The reference point m of the exponentials only moves when a score exceeds it by more than 2^RESCALE_STEP
        // (probabilities then stay below that factor, harmless in f16 / f32), and then for the whole wave at once:
        // the rescale of the 32 accumulator registers becomes rare instead of once per block.
        if (__builtin_amdgcn_ballot_w64(mx > m + MMA_RESCALE_STEP) != 0) {      // first block: m = -inf
            const float m_new = fmaxf(m, mx);
            const float corr = __builtin_amdgcn_exp2f(m - m_new);               // exp2(-inf) = 0 on the first block
            l *= corr;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) o[db][i] *= corr;
            m = m_new;
        }
        float p[4], ps = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) { p[i] = __builtin_amdgcn_exp2f(s[i] - m); ps += p[i]; }
        ps += __shfl_xor(ps, 16);
        ps += __shfl_xor(ps, 32);
        l += ps;
        const mm_u2 pu = {mm_pack(p[0], p[1]), mm_pack(p[2], p[3])};
        const mm_h4 pf = __builtin_bit_cast(mm_h4, pu);      // P^T operand: head column c, keys 4*g + j

        mm_wave_lds_sync();
        // O^T += V^T . P^T : the V^T operand is dim row 16*db + c, keys 4*g + j
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
            const mm_u2 vv = *reinterpret_cast<const mm_u2 *>(sV + (16 * db + c) * MMA_VPITCH + 4 * g);
            o[db] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(mm_h4, vv), pf, o[db], 0, 0, 0);
        }
        mm_wave_lds_sync();        // the tile is rewritten by the next block
      }
    }

    // merge the waves: o[db][i] is dim 16*db + 4*g + i of head c
    __syncthreads();               // every wave is done with its V tile: the memory becomes the merge buffer
    float *s_o = reinterpret_cast<float *>(s_raw);          // [wave][dim][16 heads]
    if (g == 0) { s_m[wave][c] = m; s_l[wave][c] = l; }
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_o[(wave * HD + 16 * db + 4 * g + i) * 16 + c] = o[db][i];
    __syncthreads();
    const bool single = p_n_splits == 1;
    for (int idx = tid; idx < G * HD; idx += MMA_THREADS) {
        const int h = idx / HD, dd = idx % HD;
        float mh = -INFINITY;
#pragma unroll
        for (int w = 0; w < MMA_WAVES; ++w) mh = fmaxf(mh, s_m[w][h]);
        float sum = 0.f, ll = 0.f;
#pragma unroll
        for (int w = 0; w < MMA_WAVES; ++w) {
            const float mw = s_m[w][h];
            const float wgt = mw == -INFINITY ? 0.f : exp2f(mw - mh);
            sum = fmaf(s_o[(w * HD + dd) * 16 + h], wgt, sum);
            ll = fmaf(s_l[w][h], wgt, ll);
        }
        const size_t row = (size_t)t * p_n_head + (size_t)kvh * G + h;
        if (single) {
            if (a.out_q16) {
                q16_store_block32(a.out_q16, p_n_head * HD, t, (kvh * G + h) * HD + dd, sum / ll);
            } else if (a.out16_k8) {
                const size_t kk = ((size_t)kvh * G + h) * HD + dd, KK = (size_t)p_n_head * HD;
                a.out16_k8[(size_t)(t / 16) * 16 * KK + ((kk >> 3) * 16 + (t % 16)) * 8 + (kk & 7)] = (_Float16)(sum / ll);
            } else {
                a.out[row * HD + dd] = sum / ll;
            }
        } else {
            a.part[(row * p_n_splits + split) * HD + dd] = sum;
            if (dd == 0) {
                a.ml[(row * p_n_splits + split) * 2 + 0] = mh;
                a.ml[(row * p_n_splits + split) * 2 + 1] = ll;
            }
        }
    }
}

template <int HD>
static int launch_mma(const AttnArgs &a, int T, hipStream_t stream) {
    const dim3 grid((unsigned)a.n_splits, (unsigned)a.n_kv, (unsigned)T), block(MMA_THREADS);
    if (a.k_type == MESH_F16 && a.v_type == MESH_F16) MESH_LAUNCH((attn_mma_kernel<HD, MESH_F16, MESH_F16>), grid, block, 0, stream, a.q, a.pos, a.seq, a.kcache, a.vcache, a.n_splits, a.n_ctx, a.n_kv, a.group, a.n_head, a.scale, a);
    else if (a.k_type == MESH_Q8_0 && a.v_type == MESH_Q4_0) MESH_LAUNCH((attn_mma_kernel<HD, MESH_Q8_0, MESH_Q4_0>), grid, block, 0, stream, a.q, a.pos, a.seq, a.kcache, a.vcache, a.n_splits, a.n_ctx, a.n_kv, a.group, a.n_head, a.scale, a);
    else if (a.k_type == MESH_Q4_0 && a.v_type == MESH_Q4_0) MESH_LAUNCH((attn_mma_kernel<HD, MESH_Q4_0, MESH_Q4_0>), grid, block, 0, stream, a.q, a.pos, a.seq, a.kcache, a.vcache, a.n_splits, a.n_ctx, a.n_kv, a.group, a.n_head, a.scale, a);
    else return fail(MESH_ERR_UNSUPPORTED, "attention_mma: KV cache types %d/%d", a.k_type, a.v_type);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

bool attention_mma_supported(const AttnArgs &a) {
    return (a.head_dim == 64 || a.head_dim == 128) && a.group >= 1 && a.group <= 16 && kv_pair_supported(a.k_type, a.v_type);
}

int attention_mma(const AttnArgs &a, int T, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (a.n_splits < 1 || a.n_splits > ATTN_SPLITS_CAP || a.group < 1 || a.n_head != a.group * a.n_kv)
        return fail(MESH_ERR_INVALID, "attention_mma: bad head layout or split count");
    if (a.n_splits > 1 && (!a.part || !a.ml)) return fail(MESH_ERR_INVALID, "attention_mma: split buffers missing");
    if (!attention_mma_supported(a)) return fail(MESH_ERR_UNSUPPORTED, "attention_mma: head_dim %d / group %d", a.head_dim, a.group);
    int rc = a.head_dim == 128 ? launch_mma<128>(a, T, stream) : launch_mma<64>(a, T, stream);
    if (rc != MESH_OK || a.n_splits == 1) return rc;
    return attention_combine(a, T, stream);
}

}  // namespace mesh
