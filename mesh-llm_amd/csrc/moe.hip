// Mixture-of-experts routing for decode: softmax gate, expert mask, top-k, and the weighted sum of expert outputs.
// Follows llama.cpp's build_moe_ffn as patched by mesh-llm
// (third_party/llama.cpp/patches/0003-moe-add-expert-analysis-and-split-tools.patch:86-104): probabilities are the
// softmax of the router logits over every expert in the file; a 0 / -inf mask is ADDED to the probabilities used
// for selection only; the weights are the unmasked probabilities of the selected experts, renormalised to sum 1.

#include "moe.hpp"

namespace mesh {

constexpr int ROUTE_MAX_PER_LANE = 8;      // up to 512 experts

// one wave per token
__global__ __launch_bounds__(64) void moe_route_kernel(MoeRouteArgs a) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float *lg = a.logits + (size_t)t * a.n_expert;
    float p[ROUTE_MAX_PER_LANE], sel[ROUTE_MAX_PER_LANE];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        p[i] = e < a.n_expert ? lg[e] : -INFINITY;
        mx = fmaxf(mx, p[i]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    float den = 0.f;
#pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
        p[i] = lane + 64 * i < a.n_expert ? expf(p[i] - mx) : 0.f;
        den += p[i];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) den += __shfl_xor(den, o);
#pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        p[i] = p[i] / den;
        sel[i] = e < a.n_expert ? p[i] + (a.mask ? a.mask[e] : 0.f) : -INFINITY;
    }
    float wsum = 0.f, my_w = 0.f;
    int my_id = 0;
    unsigned taken = 0;        // bit i: expert lane + 64*i has been selected
    for (int k = 0; k < a.top_k; ++k) {
        // best remaining (value, id) of this lane, then of the wave; ties go to the lower id
        float bv = -INFINITY, bp = 0.f;
        int bi = 0x7FFFFFFF;
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
            const int e = lane + 64 * i;
            if (e < a.n_expert && !((taken >> i) & 1u) && (bi == 0x7FFFFFFF || sel[i] > bv || (sel[i] == bv && e < bi))) { bv = sel[i]; bi = e; bp = p[i]; }
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
        for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i)
            if (lane + 64 * i == bi) taken |= 1u << i;
        if (lane == k) { my_id = bi; my_w = bp; }
        wsum += bp;
    }
    if (lane < a.top_k) {
        a.ids[(size_t)t * a.top_k + lane] = my_id;
        a.weights[(size_t)t * a.top_k + lane] = a.norm_w && wsum > 0.f ? my_w / wsum : my_w;
    }
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
