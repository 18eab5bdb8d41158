// Mixture-of-experts routing for decode: softmax gate, expert mask, top-k, and the weighted sum of expert outputs.
// Follows llama.cpp's build_moe_ffn as patched by mesh-llm
// (third_party/llama.cpp/patches/0003-moe-add-expert-analysis-and-split-tools.patch:86-104): probabilities are the
// softmax of the router logits over every expert in the file; a 0 / -inf mask is ADDED to the probabilities used
// for selection only; the weights are the unmasked probabilities of the selected experts, renormalised to sum 1.

#include <algorithm>

#include "moe.hpp"
#include "gemv.hpp"

namespace mesh {

constexpr int ROUTE_MAX_PER_LANE = MOE_EXPERTS_MAX / 64;

// softmax -> (+mask) -> top-k of one token's logits by one wave; NPL = experts per lane (n_expert <= 64 * NPL)
// (ids_copy: optional second destination of the expert ids, e.g. the workgroup's LDS)
template <int NPL>
__device__ __forceinline__ void route_wave(const float *lg, const float *mask, int n_expert, int top_k, int norm_w,
                                           int32_t *ids, float *weights, int lane, int32_t *ids_copy = nullptr) {
    float p[NPL], sel[NPL];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int e = lane + 64 * i;
        p[i] = e < n_expert ? lg[e] : -INFINITY;
        mx = fmaxf(mx, p[i]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    float den = 0.f;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        p[i] = lane + 64 * i < n_expert ? expf(p[i] - mx) : 0.f;
        den += p[i];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) den += __shfl_xor(den, o);
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int e = lane + 64 * i;
        p[i] = p[i] / den;
        sel[i] = e < n_expert ? p[i] + (mask ? mask[e] : 0.f) : -INFINITY;
    }
    float wsum = 0.f, my_w = 0.f;
    int my_id = 0;
    if constexpr (NPL <= 2) {
        // Up to 128 experts: every candidate counts the experts that come before it in the order (value descending, id
        // ascending) -- one broadcast per expert, no dependent cross-lane chain -- and the candidate counting k is the
        // k-th pick.  The same picks in the same order as the loop below (each round of which takes the first expert
        // left in that order).
        int rank[NPL];
#pragma unroll
        for (int i = 0; i < NPL; ++i) rank[i] = lane + 64 * i < n_expert ? 0 : 0x7FFFFFFF;
#pragma unroll
        for (int ii = 0; ii < NPL; ++ii) {
            for (int j = 0; j < 64 && j + 64 * ii < n_expert; ++j) {
                const float ov = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sel[ii]), j));
                const int oe = j + 64 * ii;
#pragma unroll
                for (int i = 0; i < NPL; ++i) {
                    const int e = lane + 64 * i;
                    rank[i] += (ov > sel[i] || (ov == sel[i] && oe < e)) ? 1 : 0;
                }
            }
        }
        for (int k = 0; k < top_k; ++k) {
            int bi = 0;
            float bp = 0.f;
#pragma unroll
            for (int i = 0; i < NPL; ++i) {
                const unsigned long long m = __builtin_amdgcn_ballot_w64(rank[i] == k);
                if (m != 0ull) {
                    const int src = __builtin_ctzll(m);
                    bi = src + 64 * i;
                    bp = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p[i]), src));
                }
            }
            if (lane == k) { my_id = bi; my_w = bp; }
            wsum += bp;
        }
    } else {
    unsigned taken = 0;        // bit i: expert lane + 64*i has been selected
    for (int k = 0; k < top_k; ++k) {
        // best remaining (value, id) of this lane, then of the wave; ties go to the lower id
        float bv = -INFINITY, bp = 0.f;
        int bi = 0x7FFFFFFF;
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
            const int e = lane + 64 * i;
            if (e < n_expert && !((taken >> i) & 1u) && (bi == 0x7FFFFFFF || sel[i] > bv || (sel[i] == bv && e < bi))) { bv = sel[i]; bi = e; bp = p[i]; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o), op = __shfl_xor(bp, o);
            const int oi = __shfl_xor(bi, o);
            if (oi != 0x7FFFFFFF && (bi == 0x7FFFFFFF || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; bp = op; }
        }
        // retire the winner (a masked expert can still win once every allowed one is taken, as in the reference's
        // top-k over probabilities plus mask)
#pragma unroll
        for (int i = 0; i < NPL; ++i)
            if (lane + 64 * i == bi) taken |= 1u << i;
        if (lane == k) { my_id = bi; my_w = bp; }
        wsum += bp;
    }
    }
    if (lane < top_k) {
        ids[lane] = my_id;
        if (ids_copy) ids_copy[lane] = my_id;
        weights[lane] = norm_w && wsum > 0.f ? my_w / wsum : my_w;
    }
}

__device__ __forceinline__ void route_wave_any(const float *lg, const MoeRouteArgs &a, int t, int lane, int32_t *ids_copy = nullptr) {
    int32_t *ids = a.ids + (size_t)t * a.top_k;
    float *w = a.weights + (size_t)t * a.top_k;
    if (ids_copy) ids_copy += (size_t)t * a.top_k;
    if (a.n_expert <= 64) route_wave<1>(lg, a.mask, a.n_expert, a.top_k, a.norm_w, ids, w, lane, ids_copy);
    else if (a.n_expert <= 128) route_wave<2>(lg, a.mask, a.n_expert, a.top_k, a.norm_w, ids, w, lane, ids_copy);
    else route_wave<ROUTE_MAX_PER_LANE>(lg, a.mask, a.n_expert, a.top_k, a.norm_w, ids, w, lane, ids_copy);
}

// one wave per token
__global__ __launch_bounds__(64) void moe_route_kernel(MoeRouteArgs a) {
    const int t = blockIdx.x, lane = threadIdx.x;
    route_wave_any(a.logits + (size_t)t * a.n_expert, a, t, lane);
}

// Router logits and routing in one launch, one workgroup per token: every wave holds the token's normalised hidden
// state in registers (E / 64 values per lane) and takes every fourth expert row of the f32 router matrix; the
// logits meet in LDS and the first wave routes.  logits[t] = W . (x[t] * rsqrt(mean(x^2) + eps) * norm_w).
// With gridDim.y > 1 the experts are split over blockIdx.y and the kernel only writes logits_out (routing follows in
// moe_route_group_kernel): small batches then have enough workgroups to pull the router matrix through quickly.
constexpr int ROUTER_THREADS = 1024, ROUTER_WAVES = ROUTER_THREADS / 64;
// (RT: threads of the workgroup.  A decode batch has few tokens and wants every wave it can get on a token's expert rows;
// a prefill chunk has a workgroup per token anyway, and small workgroups, eight to a CU, hide each other's row loads.)
constexpr int ROUTER_THREADS_WIDE = 256, ROUTER_WIDE_MIN_TOKENS = 512;
// the logits of this workgroup's token and expert slice (blockIdx.y of gridDim.y), into s_logits and logits_out
template <int NV, int RT>      // float4 groups per lane = E / 256
__device__ __forceinline__ void router_logits(const float *__restrict__ x, const float *__restrict__ norm_w, const float *__restrict__ W,
                                              float *__restrict__ logits_out, int ldx, float eps, int p_n_expert, float *s_logits) {
    constexpr int E = NV * 256, ROUTER_WAVES = RT / 64;
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // element index of a lane's values: 4 * (lane + 64 * i) + c
    const float *xt = x + (size_t)t * ldx;
    float4 xr[NV];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        xr[i] = *reinterpret_cast<const float4 *>(xt + 4 * (lane + 64 * i));
        ss += xr[i].x * xr[i].x + xr[i].y * xr[i].y + xr[i].z * xr[i].z + xr[i].w * xr[i].w;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    const float scale = 1.0f / sqrtf(ss / (float)E + eps);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const float4 w = *reinterpret_cast<const float4 *>(norm_w + 4 * (lane + 64 * i));
        xr[i].x = xr[i].x * scale * w.x; xr[i].y = xr[i].y * scale * w.y;
        xr[i].z = xr[i].z * scale * w.z; xr[i].w = xr[i].w * scale * w.w;
    }
    // two expert rows per step, all of their loads in flight together
    const int per = (p_n_expert + (int)gridDim.y - 1) / (int)gridDim.y;
    const int e_lo = (int)blockIdx.y * per, e_hi = e_lo + per < p_n_expert ? e_lo + per : p_n_expert;
    for (int e0 = e_lo + wave; e0 < e_hi; e0 += 2 * ROUTER_WAVES) {
        const int e1 = e0 + ROUTER_WAVES;
        const bool has1 = e1 < e_hi;
        const float *w0 = W + (size_t)e0 * E, *w1 = W + (size_t)(has1 ? e1 : e0) * E;
        float4 r0[NV], r1[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            r0[i] = *reinterpret_cast<const float4 *>(w0 + 4 * (lane + 64 * i));
            r1[i] = *reinterpret_cast<const float4 *>(w1 + 4 * (lane + 64 * i));
        }
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            a0 = fmaf(xr[i].x, r0[i].x, a0); a0 = fmaf(xr[i].y, r0[i].y, a0); a0 = fmaf(xr[i].z, r0[i].z, a0); a0 = fmaf(xr[i].w, r0[i].w, a0);
            a1 = fmaf(xr[i].x, r1[i].x, a1); a1 = fmaf(xr[i].y, r1[i].y, a1); a1 = fmaf(xr[i].z, r1[i].z, a1); a1 = fmaf(xr[i].w, r1[i].w, a1);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { a0 += __shfl_xor(a0, o); a1 += __shfl_xor(a1, o); }
        if (lane == 0) {
            s_logits[e0] = a0;
            if (logits_out) logits_out[(size_t)t * p_n_expert + e0] = a0;
            if (has1) {
                s_logits[e1] = a1;
                if (logits_out) logits_out[(size_t)t * p_n_expert + e1] = a1;
            }
        }
    }
}

template <int NV, int RT = ROUTER_THREADS>
// (scalar arguments first: preloaded into SGPRs, see gemv.hip)
__global__ __launch_bounds__(RT) void moe_router_fused_kernel(const float *__restrict__ x, const float *__restrict__ norm_w,
                                                                          const float *__restrict__ W, float *__restrict__ logits_out,
                                                                          int ldx, float eps, int p_n_expert, const MoeRouteArgs a) {
    __shared__ float s_logits[64 * ROUTE_MAX_PER_LANE];
    router_logits<NV, RT>(x, norm_w, W, logits_out, ldx, eps, p_n_expert, s_logits);
    if (gridDim.y > 1) return;
    __syncthreads();
    if ((threadIdx.x >> 6) == 0) route_wave_any(s_logits, a, blockIdx.x, threadIdx.x & 63);
}

// The same for a prefill chunk, four tokens per workgroup of eight waves: every wave keeps the four normalised hidden
// states in registers and walks every eighth expert row, so a row fetched from L2 serves four tokens (a workgroup per
// token re-reads the whole router matrix per token: 512 MB per launch at 1024 tokens x 64 experts x 2048).  Every
// (token, expert) logit is the sum the kernel above forms, in its order; waves 0 to 3 then route one token each.
constexpr int CHUNK_TOKENS = 4, CHUNK_WAVES = 8, CHUNK_THREADS = 64 * CHUNK_WAVES;
template <int NV>
__global__ __launch_bounds__(CHUNK_THREADS) void moe_router_chunk_kernel(const float *__restrict__ x, const float *__restrict__ norm_w,
                                                                         const float *__restrict__ W, float *__restrict__ logits_out,
                                                                         int ldx, float eps, int T, const MoeRouteArgs a) {
    constexpr int E = NV * 256;
    __shared__ float s_logits[CHUNK_TOKENS][64 * ROUTE_MAX_PER_LANE];
    const int t0 = blockIdx.x * CHUNK_TOKENS, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float4 xr[CHUNK_TOKENS][NV];
#pragma unroll
    for (int k = 0; k < CHUNK_TOKENS; ++k) {
        const int t = t0 + k < T ? t0 + k : T - 1;
        const float *xt = x + (size_t)t * ldx;
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            xr[k][i] = *reinterpret_cast<const float4 *>(xt + 4 * (lane + 64 * i));
            ss += xr[k][i].x * xr[k][i].x + xr[k][i].y * xr[k][i].y + xr[k][i].z * xr[k][i].z + xr[k][i].w * xr[k][i].w;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        const float scale = 1.0f / sqrtf(ss / (float)E + eps);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const float4 w = *reinterpret_cast<const float4 *>(norm_w + 4 * (lane + 64 * i));
            xr[k][i].x = xr[k][i].x * scale * w.x; xr[k][i].y = xr[k][i].y * scale * w.y;
            xr[k][i].z = xr[k][i].z * scale * w.z; xr[k][i].w = xr[k][i].w * scale * w.w;
        }
    }
    for (int e = wave; e < a.n_expert; e += CHUNK_WAVES) {
        const float *wr = W + (size_t)e * E;
        float4 r[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) r[i] = *reinterpret_cast<const float4 *>(wr + 4 * (lane + 64 * i));
        float acc[CHUNK_TOKENS];
#pragma unroll
        for (int k = 0; k < CHUNK_TOKENS; ++k) {
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                v = fmaf(xr[k][i].x, r[i].x, v); v = fmaf(xr[k][i].y, r[i].y, v); v = fmaf(xr[k][i].z, r[i].z, v); v = fmaf(xr[k][i].w, r[i].w, v);
            }
            acc[k] = v;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
#pragma unroll
            for (int k = 0; k < CHUNK_TOKENS; ++k) acc[k] += __shfl_xor(acc[k], o);
        if (lane == 0) {
#pragma unroll
            for (int k = 0; k < CHUNK_TOKENS; ++k) {
                s_logits[k][e] = acc[k];
                if (logits_out && t0 + k < T) logits_out[(size_t)(t0 + k) * a.n_expert + e] = acc[k];
            }
        }
    }
    __syncthreads();
    if (wave < CHUNK_TOKENS && t0 + wave < T) route_wave_any(s_logits[wave], a, t0 + wave, lane);
}

int moe_router_fused(const MoeRouteArgs &a, const float *x, int ldx, const float *norm_w, float eps, const float *W, int E,
                     float *logits_out, int T, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (!moe_router_fused_supported(E, a.n_expert, a.top_k)) return fail(MESH_ERR_UNSUPPORTED, "moe: fused router for hidden size %d / %d experts", E, a.n_expert);
    const dim3 grid((unsigned)T);
    if (T >= ROUTER_WIDE_MIN_TOKENS && E <= 2048) {
        const dim3 cgrid((unsigned)((T + CHUNK_TOKENS - 1) / CHUNK_TOKENS)), cblock(CHUNK_THREADS);
        switch (E / 256) {
            case 2: MESH_LAUNCH(moe_router_chunk_kernel<2>, cgrid, cblock, 0, stream, x, norm_w, W, logits_out, ldx, eps, T, a); break;
            case 4: MESH_LAUNCH(moe_router_chunk_kernel<4>, cgrid, cblock, 0, stream, x, norm_w, W, logits_out, ldx, eps, T, a); break;
            default: MESH_LAUNCH(moe_router_chunk_kernel<8>, cgrid, cblock, 0, stream, x, norm_w, W, logits_out, ldx, eps, T, a); break;
        }
        MESH_LAUNCH_CHECK();
        return MESH_OK;
    }
    if (T >= ROUTER_WIDE_MIN_TOKENS) {
        const dim3 block(ROUTER_THREADS_WIDE);
        switch (E / 256) {
            case 2: MESH_LAUNCH((moe_router_fused_kernel<2, ROUTER_THREADS_WIDE>), grid, block, 0, stream, x, norm_w, W, logits_out, ldx, eps, a.n_expert, a); break;
            case 4: MESH_LAUNCH((moe_router_fused_kernel<4, ROUTER_THREADS_WIDE>), grid, block, 0, stream, x, norm_w, W, logits_out, ldx, eps, a.n_expert, a); break;
            case 8: MESH_LAUNCH((moe_router_fused_kernel<8, ROUTER_THREADS_WIDE>), grid, block, 0, stream, x, norm_w, W, logits_out, ldx, eps, a.n_expert, a); break;
            case 16: MESH_LAUNCH((moe_router_fused_kernel<16, ROUTER_THREADS_WIDE>), grid, block, 0, stream, x, norm_w, W, logits_out, ldx, eps, a.n_expert, a); break;
            default: return fail(MESH_ERR_UNSUPPORTED, "moe: fused router for hidden size %d", E);
        }
        MESH_LAUNCH_CHECK();
        return MESH_OK;
    }
    const dim3 block(ROUTER_THREADS);
    switch (E / 256) {
        case 2: MESH_LAUNCH(moe_router_fused_kernel<2>, grid, block, 0, stream, x, norm_w, W, logits_out, ldx, eps, a.n_expert, a); break;
        case 4: MESH_LAUNCH(moe_router_fused_kernel<4>, grid, block, 0, stream, x, norm_w, W, logits_out, ldx, eps, a.n_expert, a); break;
        case 8: MESH_LAUNCH(moe_router_fused_kernel<8>, grid, block, 0, stream, x, norm_w, W, logits_out, ldx, eps, a.n_expert, a); break;
        case 16: MESH_LAUNCH(moe_router_fused_kernel<16>, grid, block, 0, stream, x, norm_w, W, logits_out, ldx, eps, a.n_expert, a); break;
        default: return fail(MESH_ERR_UNSUPPORTED, "moe: fused router for hidden size %d", E);
    }
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}
bool moe_router_fused_supported(int E, int n_expert, int top_k) {
    return (E == 512 || E == 1024 || E == 2048 || E == 4096) && n_expert >= 1 && n_expert <= 64 * ROUTE_MAX_PER_LANE && top_k >= 1 && top_k <= 64 && top_k <= n_expert;
}

int moe_route(const MoeRouteArgs &a, int T, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (a.n_expert < 1 || a.n_expert > 64 * ROUTE_MAX_PER_LANE || a.top_k < 1 || a.top_k > 64 || a.top_k > a.n_expert)
        return fail(MESH_ERR_UNSUPPORTED, "moe: %d experts / top-%d outside what the router kernel handles", a.n_expert, a.top_k);
    MESH_LAUNCH(moe_route_kernel, dim3((unsigned)T), dim3(64), 0, stream, a);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// Pairs -> per-expert work items, one workgroup.  The pair list sits in LDS; a wave takes every 16th expert and finds
// its pairs with ballots over the list (64 pairs per step), first to count, then -- after a prefix sum over the
// experts' item counts -- to write each pair into its item.
constexpr int GROUP_THREADS = 1024, GROUP_WAVES = GROUP_THREADS / 64;
// (whole workgroup; lds: n_pairs + 2 * n_expert ints)
// ipairs: most pairs per item; an item takes iints = moe_item_ints(ipairs) int32
// ids == nullptr: the pair list is in lds[0 .. n_pairs) already and a barrier has been passed since it was written
__device__ __forceinline__ void group_pairs(const int32_t *__restrict__ ids, int n_pairs, int n_expert, int32_t *__restrict__ items,
                                            int32_t *__restrict__ n_items, int32_t *lds, int ipairs) {
    const int iints = moe_item_ints(ipairs);
    int32_t *s_ids = lds, *s_cnt = lds + n_pairs, *s_base = s_cnt + n_expert;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (ids) {
        for (int p = tid; p < n_pairs; p += GROUP_THREADS) s_ids[p] = ids[p];
        __syncthreads();
    }
    for (int e = wave; e < n_expert; e += GROUP_WAVES) {
        int c = 0;
        for (int p0 = 0; p0 < n_pairs; p0 += 64) {
            const int p = p0 + lane;
            c += __popcll(__ballot(p < n_pairs && s_ids[p] == e));
        }
        if (lane == 0) s_cnt[e] = c;
    }
    __syncthreads();
    if (wave == 0) {
        // exclusive prefix of items per expert: each lane sums a run of experts, the runs are scanned across the wave
        const int per = (n_expert + 63) / 64, e0 = lane * per;
        int mine = 0;
        for (int e = e0; e < e0 + per && e < n_expert; ++e) mine += (s_cnt[e] + ipairs - 1) / ipairs;
        int incl = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(incl, o);
            if (lane >= o) incl += v;
        }
        int run = incl - mine;
        for (int e = e0; e < e0 + per && e < n_expert; ++e) {
            s_base[e] = run;
            run += (s_cnt[e] + ipairs - 1) / ipairs;
        }
        if (lane == 63) n_items[0] = incl;
    }
    __syncthreads();
    for (int e = wave; e < n_expert; e += GROUP_WAVES) {
        const int cnt = s_cnt[e], base = s_base[e];
        int seen = 0;
        for (int p0 = 0; p0 < n_pairs && seen < cnt; p0 += 64) {
            const int p = p0 + lane;
            const bool hit = p < n_pairs && s_ids[p] == e;
            const unsigned long long m = __ballot(hit);
            if (hit) {
                const int r = seen + __popcll(m & ((1ull << lane) - 1ull));
                items[(size_t)(base + r / ipairs) * iints + 2 + r % ipairs] = p;
            }
            seen += __popcll(m);
        }
        const int n_it = (cnt + ipairs - 1) / ipairs;
        for (int i = lane; i < n_it; i += 64) {
            items[(size_t)(base + i) * iints + 0] = e;
            items[(size_t)(base + i) * iints + 1] = i + 1 < n_it ? ipairs : cnt - i * ipairs;
        }
    }
}

__global__ __launch_bounds__(GROUP_THREADS) void moe_group_kernel(const int32_t *__restrict__ ids, int n_pairs, int n_expert,
                                                                  int32_t *__restrict__ items, int32_t *__restrict__ n_items, int ipairs) {
    extern __shared__ int32_t g_lds[];
    group_pairs(ids, n_pairs, n_expert, items, n_items, g_lds, ipairs);
}

// Routing of a small batch and the grouping of its pairs in one single-workgroup launch: wave w routes tokens w,
// w + 16, ... from their logits, then the workgroup groups the pairs it has just written (the barrier in between
// also makes those writes visible to the whole workgroup).
// (the routing arguments as leading scalars: preloaded into SGPRs, see gemv.hip)
__global__ __launch_bounds__(GROUP_THREADS) void moe_route_group_kernel(const float *p_logits, const float *p_mask, int32_t *p_ids, float *p_weights,
                                                                        int T, int p_n_expert, int p_top_k, int p_norm_w,
                                                                        int32_t *__restrict__ items, int32_t *__restrict__ n_items, int ipairs) {
    extern __shared__ int32_t g_lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    MoeRouteArgs a;
    a.logits = p_logits; a.mask = p_mask; a.ids = p_ids; a.weights = p_weights; a.n_expert = p_n_expert; a.top_k = p_top_k; a.norm_w = p_norm_w;
    // (the ids also go to the pair list in LDS: the grouping does not wait for them to come back from memory)
    for (int t = wave; t < T; t += GROUP_WAVES) route_wave_any(p_logits + (size_t)t * p_n_expert, a, t, lane, g_lds);
    __syncthreads();
    group_pairs(nullptr, T * p_top_k, p_n_expert, items, n_items, g_lds, ipairs);
}

// The two launches above as one: every workgroup computes its slice of the logits; the one that arrives last (a device-wide
// counter, release fence before the increment, acquire fence after it) then routes all tokens and groups the pairs, as
// moe_route_group_kernel does.  The counter is back at zero when the launch ends.  No workgroup waits for another.
template <int NV>
__global__ __launch_bounds__(GROUP_THREADS) void moe_router_group_fused_kernel(const float *__restrict__ x, const float *__restrict__ norm_w,
                                                                               const float *__restrict__ W, float *logits, int ldx, float eps,
                                                                               int p_n_expert, const MoeRouteArgs a, int T, int32_t *items, int32_t *n_items,
                                                                               int ipairs, int *arrive) {
    static_assert(GROUP_THREADS == ROUTER_THREADS, "the routing tail runs in a router workgroup");
    extern __shared__ int32_t g_lds[];
    __shared__ float s_logits[64 * ROUTE_MAX_PER_LANE];
    __shared__ int s_last;
    router_logits<NV, ROUTER_THREADS>(x, norm_w, W, logits, ldx, eps, p_n_expert, s_logits);
    // One release per workgroup, by one thread: the barrier orders the other waves' logits stores before it, and a
    // release at device scope covers what the releasing thread has observed.  (A __threadfence() in every wave measured
    // 35 us for this tail: sixteen cache write-backs and invalidations per workgroup.)
    __syncthreads();
    if (threadIdx.x == 0)
        s_last = __hip_atomic_fetch_add(arrive, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == (int)(gridDim.x * gridDim.y) - 1;
    __syncthreads();
    if (!s_last) return;
    if (threadIdx.x == 0) __hip_atomic_store(arrive, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // LDS of the tail: the pair list and the grouping's counters, then a logits row per wave
    const int n_group_ints = T * a.top_k + 2 * p_n_expert;
    for (int t = wave; t < T; t += GROUP_WAVES) {
        // the token's logits through LDS: route_wave reads plain floats
        float *row = reinterpret_cast<float *>(g_lds + n_group_ints) + (size_t)wave * 64 * ROUTE_MAX_PER_LANE;
        // (device-scope loads: written by other workgroups of this launch, possibly on another die)
        for (int e = lane; e < p_n_expert; e += 64) row[e] = __hip_atomic_load(logits + (size_t)t * p_n_expert + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        route_wave_any(row, a, t, lane, g_lds);        // (ids to memory and to the pair list in LDS)
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    group_pairs(nullptr, T * a.top_k, p_n_expert, items, n_items, g_lds, ipairs);
}

int moe_router_group(const MoeRouteArgs &a, const float *x, int ldx, const float *norm_w, float eps, const float *W, int E,
                     float *logits, int T, int32_t *items, int32_t *n_items, int item_pairs, hipStream_t stream, int *arrive) {
    if (T <= 0) return MESH_OK;
    if (!moe_router_group_supported(E, a.n_expert, a.top_k, T) || !logits)
        return fail(MESH_ERR_UNSUPPORTED, "moe: split router for hidden size %d / %d experts / %d tokens", E, a.n_expert, T);
    const int split = (a.n_expert + ROUTER_WAVES - 1) / ROUTER_WAVES;      // one expert row per wave
    const dim3 grid((unsigned)T, (unsigned)split), block(ROUTER_THREADS);
    MoeRouteArgs la = a;
    if (arrive) {
        // one launch: the last workgroup to finish its logits routes and groups
        la.logits = logits;
        // LDS of the tail: the grouping's pair list and counters, then a logits row per wave
        const size_t smem = (size_t)GROUP_WAVES * 64 * ROUTE_MAX_PER_LANE * sizeof(float) + ((size_t)T * a.top_k + 2 * (size_t)a.n_expert) * sizeof(int32_t);
        switch (E / 256) {
            case 2: MESH_LAUNCH(moe_router_group_fused_kernel<2>, grid, block, smem, stream, x, norm_w, W, logits, ldx, eps, la.n_expert, la, T, items, n_items, item_pairs, arrive); break;
            case 4: MESH_LAUNCH(moe_router_group_fused_kernel<4>, grid, block, smem, stream, x, norm_w, W, logits, ldx, eps, la.n_expert, la, T, items, n_items, item_pairs, arrive); break;
            case 8: MESH_LAUNCH(moe_router_group_fused_kernel<8>, grid, block, smem, stream, x, norm_w, W, logits, ldx, eps, la.n_expert, la, T, items, n_items, item_pairs, arrive); break;
            case 16: MESH_LAUNCH(moe_router_group_fused_kernel<16>, grid, block, smem, stream, x, norm_w, W, logits, ldx, eps, la.n_expert, la, T, items, n_items, item_pairs, arrive); break;
            default: return fail(MESH_ERR_UNSUPPORTED, "moe: fused router for hidden size %d", E);
        }
        MESH_LAUNCH_CHECK();
        return MESH_OK;
    }
    switch (E / 256) {
        case 2: MESH_LAUNCH(moe_router_fused_kernel<2>, grid, block, 0, stream, x, norm_w, W, logits, ldx, eps, la.n_expert, la); break;
        case 4: MESH_LAUNCH(moe_router_fused_kernel<4>, grid, block, 0, stream, x, norm_w, W, logits, ldx, eps, la.n_expert, la); break;
        case 8: MESH_LAUNCH(moe_router_fused_kernel<8>, grid, block, 0, stream, x, norm_w, W, logits, ldx, eps, la.n_expert, la); break;
        case 16: MESH_LAUNCH(moe_router_fused_kernel<16>, grid, block, 0, stream, x, norm_w, W, logits, ldx, eps, la.n_expert, la); break;
        default: return fail(MESH_ERR_UNSUPPORTED, "moe: fused router for hidden size %d", E);
    }
    MESH_LAUNCH_CHECK();
    la.logits = logits;
    const size_t smem = ((size_t)T * a.top_k + 2 * (size_t)a.n_expert) * sizeof(int32_t);
    MESH_LAUNCH(moe_route_group_kernel, dim3(1), dim3(GROUP_THREADS), smem, stream, la.logits, la.mask, la.ids, la.weights, T, la.n_expert, la.top_k, la.norm_w,
                                                                           items, n_items, item_pairs);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}
bool moe_router_group_supported(int E, int n_expert, int top_k, int T) {
    return moe_router_fused_supported(E, n_expert, top_k) && n_expert > ROUTER_WAVES && T >= 1 && T <= 64 &&
           ((size_t)T * top_k + 2 * (size_t)n_expert) * sizeof(int32_t) <= 28 * 1024;      // (plus 32 KB of logits rows in the same workgroup)
}

bool moe_group_supported(int n_pairs, int n_expert) {
    return n_pairs >= 1 && n_expert >= 1 && ((size_t)n_pairs + 2 * (size_t)n_expert) * sizeof(int32_t) <= 128 * 1024;
}

int moe_group(const int32_t *ids, int n_pairs, int n_expert, int32_t *items, int32_t *n_items, int item_pairs, hipStream_t stream) {
    if (!moe_group_supported(n_pairs, n_expert)) return fail(MESH_ERR_UNSUPPORTED, "moe: %d pairs over %d experts do not fit the grouping kernel", n_pairs, n_expert);
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(moe_group_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
        attr_set = true;
    }
    const size_t smem = ((size_t)n_pairs + 2 * (size_t)n_expert) * sizeof(int32_t);
    MESH_LAUNCH(moe_group_kernel, dim3(1), dim3(GROUP_THREADS), smem, stream, ids, n_pairs, n_expert, items, n_items, item_pairs);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// x[t][i] += sum_s w[t][s] * y[(t*top_k + s)][i]
__global__ __launch_bounds__(256) void moe_combine_kernel(float *__restrict__ x, const float *__restrict__ y,
                                                          const float *__restrict__ w, int n_embd, int top_k) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_embd) return;
    float acc = x[(size_t)t * n_embd + i];
    for (int s = 0; s < top_k; ++s) acc = fmaf(w[(size_t)t * top_k + s], y[((size_t)t * top_k + s) * n_embd + i], acc);
    x[(size_t)t * n_embd + i] = acc;
}

int moe_combine(float *x, const float *y, const float *w, int T, int n_embd, int top_k, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    MESH_LAUNCH(moe_combine_kernel, dim3((unsigned)((n_embd + 255) / 256), (unsigned)T), dim3(256), 0, stream, x, y, w, n_embd, top_k);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// the same with the rows of y at the slots of moe_sort: x[t][i] += sum_s w[t][s] * y[slot_of_pair[t*top_k + s]][i], four columns a thread
__global__ __launch_bounds__(256) void moe_combine_slots_kernel(float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ w,
                                                                const int32_t *__restrict__ slot_of_pair, int n_embd, int top_k) {
    const int t = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n_embd) return;
    float4 acc = *reinterpret_cast<const float4 *>(x + (size_t)t * n_embd + i);
    for (int s = 0; s < top_k; ++s) {
        const float ws = w[(size_t)t * top_k + s];
        const float4 v = *reinterpret_cast<const float4 *>(y + (size_t)slot_of_pair[(size_t)t * top_k + s] * n_embd + i);
        acc.x = fmaf(ws, v.x, acc.x); acc.y = fmaf(ws, v.y, acc.y); acc.z = fmaf(ws, v.z, acc.z); acc.w = fmaf(ws, v.w, acc.w);
    }
    *reinterpret_cast<float4 *>(x + (size_t)t * n_embd + i) = acc;
}

int moe_combine_slots(float *x, const float *y, const float *w, const int32_t *slot_of_pair, int T, int n_embd, int top_k, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (n_embd % 4) return fail(MESH_ERR_INVALID, "moe_combine_slots: row length %d not a multiple of 4", n_embd);
    MESH_LAUNCH(moe_combine_slots_kernel, dim3((unsigned)((n_embd / 4 + 255) / 256), (unsigned)T), dim3(256), 0, stream, x, y, w, slot_of_pair, n_embd, top_k);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// ---- pairs sorted by expert for the large-tile GEMM ------------------------------------------------------------
// One workgroup: counts per expert (LDS atomics), a scan over the experts for the first slot (a multiple of 16) and the
// first tile of each, then every pair takes the next free slot of its expert.  Which slot of its expert a pair gets
// depends on the order the atomics land in; nothing computed from the slots does (a column of a matrix product depends
// on that column alone, and the combine step finds its rows through slot_of_pair).
constexpr int SORT_THREADS = 1024;
__global__ __launch_bounds__(SORT_THREADS) void moe_sort_kernel(const int32_t *__restrict__ ids, int n_pairs, int n_expert, int cap_slots,
                                                                int32_t *__restrict__ slot_of_pair, int32_t *__restrict__ pair_of_slot,
                                                                int32_t *__restrict__ tiles, int32_t *__restrict__ counts) {
    extern __shared__ int32_t s_lds[];
    int32_t *s_cnt = s_lds, *s_off = s_cnt + n_expert, *s_tile = s_off + n_expert, *s_cur = s_tile + n_expert;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int e = tid; e < n_expert; e += SORT_THREADS) { s_cnt[e] = 0; s_cur[e] = 0; }
    for (int sl = tid; sl < cap_slots; sl += SORT_THREADS) pair_of_slot[sl] = -1;
    __syncthreads();
    for (int p = tid; p < n_pairs; p += SORT_THREADS) atomicAdd(&s_cnt[ids[p]], 1);
    __syncthreads();
    if (wave == 0) {
        // exclusive prefixes of padded slots and of tiles per expert: each lane sums a run of experts, the runs are scanned across the wave
        const int per = (n_expert + 63) / 64, e0 = lane * per;
        int my_s = 0, my_t = 0;
        for (int e = e0; e < e0 + per && e < n_expert; ++e) { my_s += (s_cnt[e] + 15) & ~15; my_t += (s_cnt[e] + 127) >> 7; }
        int in_s = my_s, in_t = my_t;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int vs = __shfl_up(in_s, o), vt = __shfl_up(in_t, o);
            if (lane >= o) { in_s += vs; in_t += vt; }
        }
        int run_s = in_s - my_s, run_t = in_t - my_t;
        for (int e = e0; e < e0 + per && e < n_expert; ++e) {
            s_off[e] = run_s; s_tile[e] = run_t;
            run_s += (s_cnt[e] + 15) & ~15; run_t += (s_cnt[e] + 127) >> 7;
        }
        if (lane == 63) { counts[0] = in_t; counts[1] = in_s; }
    }
    __syncthreads();
    for (int e = tid; e < n_expert; e += SORT_THREADS) {
        const int cnt = s_cnt[e];
        for (int j = 0; j * 128 < cnt; ++j) {
            int32_t *tl = tiles + (size_t)(s_tile[e] + j) * 4;
            tl[0] = e; tl[1] = s_off[e] + 128 * j; tl[2] = cnt - 128 * j < 128 ? cnt - 128 * j : 128; tl[3] = 0;
        }
    }
    for (int p = tid; p < n_pairs; p += SORT_THREADS) {
        const int e = ids[p];
        const int sl = s_off[e] + atomicAdd(&s_cur[e], 1);
        slot_of_pair[p] = sl;
        pair_of_slot[sl] = p;
    }
}

int moe_sort_slots(int n_pairs, int n_expert) { return (n_pairs + 15 * std::min(n_pairs, n_expert) + 15) / 16 * 16; }
int moe_sort_max_tiles(int n_pairs, int n_expert) { return n_pairs / 128 + std::min(n_pairs, n_expert); }

int moe_sort(const int32_t *ids, int n_pairs, int n_expert, const MoeSorted &out, hipStream_t stream) {
    if (n_pairs < 1 || n_expert < 1 || n_expert > 4096 || !ids || !out.slot_of_pair || !out.pair_of_slot || !out.tiles || !out.counts)
        return fail(MESH_ERR_INVALID, "moe_sort: bad arguments (%d pairs, %d experts)", n_pairs, n_expert);
    MESH_LAUNCH(moe_sort_kernel, dim3(1), dim3(SORT_THREADS), 4 * (size_t)n_expert * sizeof(int32_t), stream, ids, n_pairs, n_expert,
                moe_sort_slots(n_pairs, n_expert), out.slot_of_pair, out.pair_of_slot, out.tiles, out.counts);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

}  // namespace mesh
