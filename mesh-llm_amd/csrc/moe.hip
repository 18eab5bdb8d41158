// Mixture-of-experts routing for decode: softmax gate, expert mask, top-k, and the weighted sum of expert outputs.
// Follows llama.cpp's build_moe_ffn as patched by mesh-llm
// (third_party/llama.cpp/patches/0003-moe-add-expert-analysis-and-split-tools.patch:86-104): probabilities are the
// softmax of the router logits over every expert in the file; a 0 / -inf mask is ADDED to the probabilities used
// for selection only; the weights are the unmasked probabilities of the selected experts, renormalised to sum 1.

#include "moe.hpp"

namespace mesh {

constexpr int ROUTE_MAX_PER_LANE = 8;      // up to 512 experts

// softmax -> (+mask) -> top-k of one token's logits by one wave; NPL = experts per lane (n_expert <= 64 * NPL)
template <int NPL>
__device__ __forceinline__ void route_wave(const float *lg, const float *mask, int n_expert, int top_k, int norm_w,
                                           int32_t *ids, float *weights, int lane) {
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
    if (lane < top_k) {
        ids[lane] = my_id;
        weights[lane] = norm_w && wsum > 0.f ? my_w / wsum : my_w;
    }
}

__device__ __forceinline__ void route_wave_any(const float *lg, const MoeRouteArgs &a, int t, int lane) {
    int32_t *ids = a.ids + (size_t)t * a.top_k;
    float *w = a.weights + (size_t)t * a.top_k;
    if (a.n_expert <= 64) route_wave<1>(lg, a.mask, a.n_expert, a.top_k, a.norm_w, ids, w, lane);
    else if (a.n_expert <= 128) route_wave<2>(lg, a.mask, a.n_expert, a.top_k, a.norm_w, ids, w, lane);
    else route_wave<ROUTE_MAX_PER_LANE>(lg, a.mask, a.n_expert, a.top_k, a.norm_w, ids, w, lane);
}

// one wave per token
__global__ __launch_bounds__(64) void moe_route_kernel(MoeRouteArgs a) {
    const int t = blockIdx.x, lane = threadIdx.x;
    route_wave_any(a.logits + (size_t)t * a.n_expert, a, t, lane);
}

// Router logits and routing in one launch, one workgroup per token: every wave holds the token's normalised hidden
// state in registers (E / 64 values per lane) and takes every fourth expert row of the f32 router matrix; the
// logits meet in LDS and the first wave routes.  logits[t] = W . (x[t] * rsqrt(mean(x^2) + eps) * norm_w).
constexpr int ROUTER_THREADS = 1024, ROUTER_WAVES = ROUTER_THREADS / 64, ROUTER_EPL_MAX = 64;     // hidden sizes up to 4096
template <int NV>      // float4 groups per lane = E / 256
__global__ __launch_bounds__(ROUTER_THREADS) void moe_router_fused_kernel(MoeRouteArgs a, const float *__restrict__ x, int ldx,
                                                                          const float *__restrict__ norm_w, float eps,
                                                                          const float *__restrict__ W, float *__restrict__ logits_out) {
    constexpr int E = NV * 256;
    __shared__ float s_logits[64 * ROUTE_MAX_PER_LANE];
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
    for (int e0 = wave; e0 < a.n_expert; e0 += 2 * ROUTER_WAVES) {
        const int e1 = e0 + ROUTER_WAVES;
        const bool has1 = e1 < a.n_expert;
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
            if (logits_out) logits_out[(size_t)t * a.n_expert + e0] = a0;
            if (has1) {
                s_logits[e1] = a1;
                if (logits_out) logits_out[(size_t)t * a.n_expert + e1] = a1;
            }
        }
    }
    __syncthreads();
    if (wave == 0) route_wave_any(s_logits, a, t, lane);
}

int moe_router_fused(const MoeRouteArgs &a, const float *x, int ldx, const float *norm_w, float eps, const float *W, int E,
                     float *logits_out, int T, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (!moe_router_fused_supported(E, a.n_expert, a.top_k)) return fail(MESH_ERR_UNSUPPORTED, "moe: fused router for hidden size %d / %d experts", E, a.n_expert);
    const dim3 grid((unsigned)T), block(ROUTER_THREADS);
    switch (E / 256) {
        case 2: moe_router_fused_kernel<2><<<grid, block, 0, stream>>>(a, x, ldx, norm_w, eps, W, logits_out); break;
        case 4: moe_router_fused_kernel<4><<<grid, block, 0, stream>>>(a, x, ldx, norm_w, eps, W, logits_out); break;
        case 8: moe_router_fused_kernel<8><<<grid, block, 0, stream>>>(a, x, ldx, norm_w, eps, W, logits_out); break;
        case 16: moe_router_fused_kernel<16><<<grid, block, 0, stream>>>(a, x, ldx, norm_w, eps, W, logits_out); break;
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
    moe_route_kernel<<<dim3((unsigned)T), dim3(64), 0, stream>>>(a);
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
    moe_combine_kernel<<<dim3((unsigned)((n_embd + 255) / 256), (unsigned)T), dim3(256), 0, stream>>>(x, y, w, n_embd, top_k);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

}  // namespace mesh
