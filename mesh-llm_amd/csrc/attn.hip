// RoPE + KV append, and GQA attention over the stage-local KV cache (split-KV, online softmax).
// Stands where the worker's graph runs rope -> kv store -> flash_attn_ext (-fa on, mesh-llm/src/inference/launch.rs:1350-1353;
// cache types per KvCacheQuant::for_model_size, launch.rs:568-591: f16/f16, q8_0/q4_0, q4_0/q4_0).
//
// Cache layout per layer: K and V as [n_seq][n_head_kv][n_ctx] rows of head_dim values (kv_cache.hpp); one
// (sequence, kv head) is a contiguous run so a workgroup streams its key range linearly.  The `group` query heads that share a kv head
// are processed together, so each K/V byte is read once per token.

#include "attn.hpp"
#include "q16.hpp"

namespace mesh {

// ------------------------------------------------------------------------------------------------ rope + append
// grid (n_head + 2*n_head_kv, T), one wave per head vector.
constexpr int ROPE_HD_MAX = 256;
// (leading scalar arguments: preloaded into SGPRs, see gemv.hip)
__global__ __launch_bounds__(64) void rope_kv_kernel(const int32_t *p_pos, const int32_t *p_seq, float *p_q, const float *p_k, const float *p_v,
                                                     int p_n_head, int p_n_kv, int p_head_dim, const RopeKvArgs a) {
    __shared__ float s_vec[ROPE_HD_MAX];         // the finished K / V row before it is stored in the cache type
    const int hh = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
    const int hd = p_head_dim;
    const int pos = p_pos[t], seq = p_seq[t];
    float *vec;
    const float *nw = nullptr;
    int kind, head;
    if (hh < p_n_head) { kind = 0; head = hh; vec = p_q + ((size_t)t * p_n_head + head) * hd; nw = a.q_norm; }
    else if (hh < p_n_head + p_n_kv) { kind = 1; head = hh - p_n_head; vec = const_cast<float *>(p_k) + ((size_t)t * p_n_kv + head) * hd; nw = a.k_norm; }
    else { kind = 2; head = hh - p_n_head - p_n_kv; vec = const_cast<float *>(p_v) + ((size_t)t * p_n_kv + head) * hd; }

    const int ctype = kind == 1 ? a.k_type : a.v_type;
    uint8_t *row = nullptr;
    if (kind) row = (kind == 1 ? a.kcache : a.vcache) + (((size_t)seq * p_n_kv + head) * a.n_ctx + pos) * (size_t)kv_row_bytes(ctype, hd);

    if (kind == 2) {
        for (int i = lane; i < hd; i += 64) s_vec[i] = vec[i];
        __syncthreads();
        kv_store_row(ctype, row, s_vec, hd, lane);
        return;
    }
    // optional per-head RMS norm (qwen3: attn_q_norm / attn_k_norm over head_dim)
    float nscale = 1.0f;
    if (nw) {
        float ss = 0.f;
        for (int i = lane; i < hd; i += 64) ss += vec[i] * vec[i];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        nscale = 1.0f / sqrtf(ss / (float)hd + a.eps);
    }
    const int half = a.n_rot / 2;
    for (int i = lane; i < half; i += 64) {
        const int ia = a.rope_mode == ROPE_MODE_NEOX ? i : 2 * i;
        const int ib = a.rope_mode == ROPE_MODE_NEOX ? i + half : 2 * i + 1;
        float x0 = vec[ia], x1 = vec[ib];
        if (nw) { x0 = x0 * nscale * nw[ia]; x1 = x1 * nscale * nw[ib]; }
        float sn, cs;
        sincosf((float)pos * a.inv_freq[i], &sn, &cs);
        const float o0 = x0 * cs - x1 * sn;
        const float o1 = x0 * sn + x1 * cs;
        if (kind == 0) { vec[ia] = o0; vec[ib] = o1; }
        else { s_vec[ia] = o0; s_vec[ib] = o1; }
    }
    // dimensions beyond n_rot are not rotated
    for (int e = a.n_rot + lane; e < hd; e += 64) {
        float x0 = vec[e];
        if (nw) x0 = x0 * nscale * nw[e];
        if (kind == 0) vec[e] = x0;
        else s_vec[e] = x0;
    }
    if (kind == 1) {
        __syncthreads();
        kv_store_row(ctype, row, s_vec, hd, lane);
    }
}

int rope_kv(const RopeKvArgs &a, int T, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (a.head_dim % 2 || a.n_rot % 2 || a.n_rot > a.head_dim || a.head_dim > ROPE_HD_MAX)
        return fail(MESH_ERR_INVALID, "rope: bad head_dim/n_rot %d/%d", a.head_dim, a.n_rot);
    if (!kv_type_supported(a.k_type) || !kv_type_supported(a.v_type) || ((a.k_type != MESH_F16 || a.v_type != MESH_F16) && a.head_dim % 32))
        return fail(MESH_ERR_UNSUPPORTED, "rope: KV cache types %d/%d with head_dim %d", a.k_type, a.v_type, a.head_dim);
    MESH_LAUNCH(rope_kv_kernel, dim3((unsigned)(a.n_head + 2 * a.n_kv), (unsigned)T), dim3(64), 0, stream, a.pos, a.seq, a.q, a.k, a.v, a.n_head, a.n_kv, a.head_dim, a);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// ------------------------------------------------------------------------------------------------ attention
constexpr int ATTN_THREADS = 256;
constexpr int ATTN_WAVES = ATTN_THREADS / 64;
constexpr int KPT = 4;                      // keys per thread per pass: 8 x 16-byte loads in flight per lane

// 2^x by the hardware instruction alone: arguments here are <= 0 (score minus running maximum), and results too small
// for a normal float may flush to zero, which a softmax weight of that size is anyway.
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// Sum over the LPK (8 or 16) consecutive lanes that share a key, result in every one of them: data-parallel-primitive
// moves inside a row of 16 lanes (swap neighbours, swap pairs, mirror the 8, mirror the 16) instead of LDS permutes.
template <int LPK>
__device__ __forceinline__ float slot_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false));    // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false));    // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, false));   // row_half_mirror
    if (LPK == 16) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, false));   // row_mirror
    return v;
}

// grid (n_splits, n_kv * (group/G), T).  HD/8 lanes share one key ("slot"); a thread visits keys
// j0 + slot + SLOTS*i and keeps one online-softmax state (m, l, acc[8]) per query head.  Per pass all KPT keys'
// K and V vectors are requested first, then scored, then folded in with a single rescale.  The slots of a
// workgroup are merged through LDS.  With one split the normalised output is written directly; otherwise each
// workgroup writes an un-normalised partial plus (max, sum) and attn_combine_kernel merges the splits.
// Quantised rows decode to scale * (u - off) with small integers u (kv_cache.hpp): the offset leaves the inner
// loops, as off * sum(q) per score and as one running sum of p * scale per head on the value side.
template <int HD, int G, int KT, int VT>
__global__ __launch_bounds__(ATTN_THREADS) void attn_kernel(AttnArgs a) {
    constexpr int LPK = HD / 8;                 // lanes per key
    constexpr int SLOTS = ATTN_THREADS / LPK;   // keys visited side by side
    __shared__ float s_m[SLOTS][G], s_l[ATTN_WAVES][G], s_mw[G];
    __shared__ float s_acc[ATTN_WAVES][G][HD];  // per-wave sums of the slot states

    const int split = blockIdx.x, t = blockIdx.z;
    const int hgroups = a.group / G;            // G divides group (G == group, or G == 1)
    const int kvh = blockIdx.y / hgroups;
    const int h0 = kvh * a.group + (blockIdx.y % hgroups) * G;   // first query head of this workgroup
    const int tid = threadIdx.x, slot = tid / LPK, ds = (tid % LPK) * 8, wave = tid >> 6;
    const int seq = a.seq[t];
    const int n_keys = a.pos[t] + 1;
    const int per = (n_keys + a.n_splits - 1) / a.n_splits;
    const int j0 = split * per;
    const int j1 = j0 + per < n_keys ? j0 + per : n_keys;

    constexpr int KRB = kv_row_bytes(KT, HD), VRB = kv_row_bytes(VT, HD);
    float q[G][8], acc[G][8], m[G], l[G], qoff[G], voff[G];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        const float4 qa = *reinterpret_cast<const float4 *>(a.q + ((size_t)t * a.n_head + h0 + h) * HD + ds);
        const float4 qb = *reinterpret_cast<const float4 *>(a.q + ((size_t)t * a.n_head + h0 + h) * HD + ds + 4);
        const float qs = a.scale * 1.44269504088896341f;      // scores in log2 units: softmax through exp2
        q[h][0] = qa.x * qs; q[h][1] = qa.y * qs; q[h][2] = qa.z * qs; q[h][3] = qa.w * qs;
        q[h][4] = qb.x * qs; q[h][5] = qb.y * qs; q[h][6] = qb.z * qs; q[h][7] = qb.w * qs;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
        m[h] = -INFINITY;
        l[h] = 0.f;
        voff[h] = 0.f;
        qoff[h] = 0.f;
        if (KT != MESH_F16) {
#pragma unroll
            for (int i = 0; i < 8; ++i) qoff[h] += q[h][i];
            qoff[h] *= -KvAffine<KT>::off;
        }
    }
    const size_t base = ((size_t)seq * a.n_kv + kvh) * a.n_ctx;
    for (int jb = j0; jb < j1; jb += SLOTS * KPT) {
        KvRaw<KT> kr[KPT];
        KvRaw<VT> vr[KPT];
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int j = jb + slot + SLOTS * i;
            kv_zero<KT>(kr[i]);
            kv_zero<VT>(vr[i]);
            if (j < j1) {
                kr[i] = kv_load<KT, HD>(a.kcache + (base + j) * KRB, ds);
                vr[i] = kv_load<VT, HD>(a.vcache + (base + j) * VRB, ds);
            }
        }
        float sc[KPT][G];
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            float kf[8];
            const float kd = kv_decode<KT>(kr[i], kf);
            const bool ok = jb + slot + SLOTS * i < j1;
#pragma unroll
            for (int h = 0; h < G; ++h) {
                float s = qoff[h];
#pragma unroll
                for (int e = 0; e < 8; ++e) s = fmaf(q[h][e], kf[e], s);
                if (KT != MESH_F16) s *= kd;
                s = slot_sum<LPK>(s);
                sc[i][h] = ok ? s : -INFINITY;
            }
        }
        float vf[KPT][8], vd[KPT];
#pragma unroll
        for (int i = 0; i < KPT; ++i) vd[i] = kv_decode<VT>(vr[i], vf[i]);
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float mn = m[h];
#pragma unroll
            for (int i = 0; i < KPT; ++i) mn = fmaxf(mn, sc[i][h]);
            if (mn == -INFINITY) continue;          // this slot had no key in range yet
            const float corr = exp2_fast(m[h] - mn);    // exp2(-inf) = 0 the first time
            float p[KPT], ps = 0.f;
#pragma unroll
            for (int i = 0; i < KPT; ++i) { p[i] = exp2_fast(sc[i][h] - mn); ps += p[i]; }
            l[h] = l[h] * corr + ps;
            if (VT != MESH_F16) {       // from here on p carries the row scale; the offset term is summed apart
                float po = 0.f;
#pragma unroll
                for (int i = 0; i < KPT; ++i) { p[i] *= vd[i]; po += p[i]; }
                voff[h] = voff[h] * corr + po * KvAffine<VT>::off;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float v = acc[h][e] * corr;
#pragma unroll
                for (int i = 0; i < KPT; ++i) v = fmaf(p[i], vf[i][e], v);
                acc[h][e] = v;
            }
            m[h] = mn;
        }
    }
    if (VT != MESH_F16) {
#pragma unroll
        for (int h = 0; h < G; ++h)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[h][e] -= voff[h];
    }
    // merge the slots of this workgroup: every slot state is rescaled to the workgroup's maximum, slots sharing a
    // wave are added with shuffles, the 4 waves meet in LDS
    if ((tid % LPK) == 0) {
#pragma unroll
        for (int h = 0; h < G; ++h) s_m[slot][h] = m[h];
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < G; ++h) {
        float mh = -INFINITY;
#pragma unroll
        for (int s2 = 0; s2 < SLOTS; ++s2) mh = fmaxf(mh, s_m[s2][h]);
        const float w = (m[h] == -INFINITY) ? 0.f : exp2f(m[h] - mh);
        float lw = l[h] * w;
#pragma unroll
        for (int o = LPK; o < 64; o <<= 1) lw += __shfl_xor(lw, o);
        if ((tid & 63) == 0) { s_l[wave][h] = lw; s_mw[h] = mh; }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float v = acc[h][e] * w;
#pragma unroll
            for (int o = LPK; o < 64; o <<= 1) v += __shfl_xor(v, o);   // slots that live in this wave
            if ((tid & 63) < LPK) s_acc[wave][h][ds + e] = v;
        }
    }
    __syncthreads();
    const bool single = a.n_splits == 1;
    for (int o = tid; o < G * HD; o += ATTN_THREADS) {
        const int h = o / HD, dd = o % HD;
        float sum = 0.f, ll = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < ATTN_WAVES; ++w2) { sum += s_acc[w2][h][dd]; ll += s_l[w2][h]; }
        const size_t row = (size_t)t * a.n_head + h0 + h;
        if (single) {
            a.out[row * HD + dd] = sum / ll;
        } else {
            a.part[(row * a.n_splits + split) * HD + dd] = sum;
            if (dd == 0) {
                a.ml[(row * a.n_splits + split) * 2 + 0] = s_mw[h];
                a.ml[(row * a.n_splits + split) * 2 + 1] = ll;
            }
        }
    }
}

// Merge of the KV splits: grid (n_head, T), head_dim threads.  Split statistics go through LDS so every thread
// sees them with broadcast reads and the partial rows are fetched with independent loads.
// (leading scalar arguments: preloaded into SGPRs, see gemv.hip)
__global__ __launch_bounds__(128) void attn_combine_kernel(const float *p_part, const float *p_ml, float *p_out, _Float16 *p_out16_k8,
                                                           uint8_t *p_out_q16, int p_n_splits, int p_n_head, int p_head_dim) {
    __shared__ float s_m[ATTN_SPLITS_CAP], s_l[ATTN_SPLITS_CAP];
    const int h = blockIdx.x, t = blockIdx.y, dd = threadIdx.x;
    const size_t row = (size_t)t * p_n_head + h;
    for (int s2 = dd; s2 < p_n_splits; s2 += blockDim.x) {
        s_m[s2] = p_ml[(row * p_n_splits + s2) * 2 + 0];
        s_l[s2] = p_ml[(row * p_n_splits + s2) * 2 + 1];
    }
    __syncthreads();
    float mh = -INFINITY;
    for (int s2 = 0; s2 < p_n_splits; ++s2) mh = fmaxf(mh, s_m[s2]);
    float num = 0.f, den = 0.f;
    const float *pp = p_part + row * p_n_splits * p_head_dim + dd;
#pragma unroll 8
    for (int s2 = 0; s2 < p_n_splits; ++s2) {
        const float ms = s_m[s2];
        const float w = ms == -INFINITY ? 0.f : exp2f(ms - mh);      // maxima are in log2 units
        // A split that saw no key has weight 0 and must contribute nothing, whatever its partial row holds: the clamp
        // turns NaN and infinities into finite values (fmaxf / fminf return the other operand for NaN) and is the
        // identity otherwise.  (A select on `ms` instead is compiled into a branch around the load, and the 32 loads of
        // a thread then go out one after the other: measured, 9 us per layer at batch 1.)
        const float pv = fminf(fmaxf(pp[(size_t)s2 * p_head_dim], -3.4028234664e38f), 3.4028234664e38f);
        const float lv = fminf(fmaxf(s_l[s2], 0.f), 3.4028234664e38f);
        num = fmaf(pv, w, num);
        den = fmaf(lv, w, den);
    }
    if (p_out_q16) {
        q16_store_block32(p_out_q16, p_n_head * p_head_dim, t, h * p_head_dim + dd, num / den);
    } else if (p_out16_k8) {
        const size_t kk = (size_t)h * p_head_dim + dd, KK = (size_t)p_n_head * p_head_dim;
        p_out16_k8[(size_t)(t / 16) * 16 * KK + ((kk >> 3) * 16 + (t % 16)) * 8 + (kk & 7)] = (_Float16)(num / den);
    } else {
        p_out[row * p_head_dim + dd] = num / den;
    }
}

template <int HD, int KT, int VT>
static int launch_attn(const AttnArgs &a, int T, hipStream_t stream) {
    const dim3 block(ATTN_THREADS);
#define MESH_ATTN_CASE(GG)                                                                          \
    if (a.group == GG) {                                                                            \
        MESH_LAUNCH((attn_kernel<HD, GG, KT, VT>), dim3((unsigned)a.n_splits, (unsigned)a.n_kv, (unsigned)T), block, 0, stream, a); \
        MESH_LAUNCH_CHECK();                                                                        \
        return MESH_OK;                                                                             \
    }
    MESH_ATTN_CASE(1)
    MESH_ATTN_CASE(2)
    MESH_ATTN_CASE(4)
    if (HD == 128) { MESH_ATTN_CASE(5) MESH_ATTN_CASE(8) }
    if (HD == 64) { MESH_ATTN_CASE(7) }
#undef MESH_ATTN_CASE
    // any other group size: one query head per workgroup (K/V re-read per head)
    MESH_LAUNCH((attn_kernel<HD, 1, KT, VT>), dim3((unsigned)a.n_splits, (unsigned)(a.n_kv * a.group), (unsigned)T), block, 0, stream, a);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

template <int HD>
static int launch_attn_typed(const AttnArgs &a, int T, hipStream_t stream) {
    if (a.k_type == MESH_F16 && a.v_type == MESH_F16) return launch_attn<HD, MESH_F16, MESH_F16>(a, T, stream);
    if (a.k_type == MESH_Q8_0 && a.v_type == MESH_Q4_0) return launch_attn<HD, MESH_Q8_0, MESH_Q4_0>(a, T, stream);
    if (a.k_type == MESH_Q4_0 && a.v_type == MESH_Q4_0) return launch_attn<HD, MESH_Q4_0, MESH_Q4_0>(a, T, stream);
    return fail(MESH_ERR_UNSUPPORTED, "attention: KV cache types %d/%d (f16/f16, q8_0/q4_0 and q4_0/q4_0 have kernels)", a.k_type, a.v_type);
}

bool kv_pair_supported(int k_type, int v_type) {
    return (k_type == MESH_F16 && v_type == MESH_F16) || (k_type == MESH_Q8_0 && v_type == MESH_Q4_0) || (k_type == MESH_Q4_0 && v_type == MESH_Q4_0);
}

int attention(const AttnArgs &a, int T, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (a.n_splits < 1 || a.n_splits > ATTN_SPLITS_CAP || a.group < 1 || a.n_head != a.group * a.n_kv)
        return fail(MESH_ERR_INVALID, "attention: bad head layout or split count");
    if (a.n_splits > 1 && (!a.part || !a.ml)) return fail(MESH_ERR_INVALID, "attention: split buffers missing");
    int rc;
    if (a.head_dim == 128) rc = launch_attn_typed<128>(a, T, stream);
    else if (a.head_dim == 64) rc = launch_attn_typed<64>(a, T, stream);
    else return fail(MESH_ERR_UNSUPPORTED, "attention: head_dim %d has no kernel (64 and 128 do)", a.head_dim);
    if (rc != MESH_OK || a.n_splits == 1) return rc;
    return attention_combine(a, T, stream);
}

int attention_combine(const AttnArgs &a, int T, hipStream_t stream) {
    MESH_LAUNCH(attn_combine_kernel, dim3((unsigned)a.n_head, (unsigned)T), dim3((unsigned)a.head_dim), 0, stream, a.part, a.ml, a.out, a.out16_k8, a.out_q16, a.n_splits, a.n_head, a.head_dim);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// ------------------------------------------------------------------------------------------------ f16 <-> cache rows
// grid (n_kv, n_pos), one wave per row
__global__ __launch_bounds__(64) void kv_import_kernel(int type, uint8_t *cache, const uint16_t *half, int n_kv, int n_ctx, int hd, int seq, int pos0) {
    __shared__ float s_vec[ROPE_HD_MAX];
    const int h = blockIdx.x, p = blockIdx.y, lane = threadIdx.x;
    const uint16_t *src = half + ((size_t)p * n_kv + h) * hd;
    for (int i = lane; i < hd; i += 64) s_vec[i] = f16_bits_to_f32(src[i]);
    __syncthreads();
    kv_store_row(type, cache + (((size_t)seq * n_kv + h) * n_ctx + pos0 + p) * (size_t)kv_row_bytes(type, hd), s_vec, hd, lane);
}
__global__ __launch_bounds__(64) void kv_export_kernel(int type, const uint8_t *cache, uint16_t *half, int n_kv, int n_ctx, int hd, int seq, int pos0) {
    const int h = blockIdx.x, p = blockIdx.y, lane = threadIdx.x;
    const uint8_t *row = cache + (((size_t)seq * n_kv + h) * n_ctx + pos0 + p) * (size_t)kv_row_bytes(type, hd);
    uint16_t *dst = half + ((size_t)p * n_kv + h) * hd;
    for (int i = lane; i < hd; i += 64) dst[i] = f32_to_f16_bits(kv_fetch(type, row, hd, i));
}

int kv_import(int type, uint8_t *cache, const uint16_t *half, int n_kv, int n_ctx, int head_dim, int seq, int pos0, int n_pos, hipStream_t stream) {
    if (!kv_type_supported(type) || head_dim > ROPE_HD_MAX || (type != MESH_F16 && head_dim % 32)) return fail(MESH_ERR_UNSUPPORTED, "kv_import: type %d, head_dim %d", type, head_dim);
    MESH_LAUNCH(kv_import_kernel, dim3((unsigned)n_kv, (unsigned)n_pos), dim3(64), 0, stream, type, cache, half, n_kv, n_ctx, head_dim, seq, pos0);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}
int kv_export(int type, const uint8_t *cache, uint16_t *half, int n_kv, int n_ctx, int head_dim, int seq, int pos0, int n_pos, hipStream_t stream) {
    if (!kv_type_supported(type)) return fail(MESH_ERR_UNSUPPORTED, "kv_export: type %d", type);
    MESH_LAUNCH(kv_export_kernel, dim3((unsigned)n_kv, (unsigned)n_pos), dim3(64), 0, stream, type, cache, half, n_kv, n_ctx, head_dim, seq, pos0);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

}  // namespace mesh
