// Mixture-of-experts routing launchers (moe.hip).
#pragma once

#include "mesh_common.hpp"

namespace mesh {

// most experts one routing wave can rank (64 lanes x 8 candidates each)
constexpr int MOE_EXPERTS_MAX = 512;

struct MoeRouteArgs {
    const float *logits = nullptr;   // [T][n_expert] router outputs
    const float *mask = nullptr;     // optional [n_expert]: 0 = allowed, -inf = masked out
    int32_t *ids = nullptr;          // [T][top_k]
    float *weights = nullptr;        // [T][top_k]
    int n_expert = 0, top_k = 0, norm_w = 1;
};
int moe_route(const MoeRouteArgs &a, int T, hipStream_t stream);
// Router mat-vec (f32 matrix W [n_expert][E] over the RMS-normalised hidden state) and routing in one launch; a.logits is
// not read, logits_out (optional) receives [T][n_expert].
bool moe_router_fused_supported(int E, int n_expert, int top_k);
int moe_router_fused(const MoeRouteArgs &a, const float *x, int ldx, const float *norm_w, float eps, const float *W, int E,
                     float *logits_out, int T, hipStream_t stream);
// Groups the n_pairs (token, slot) pairs of ids by expert into work items for the expert launches: moe_item_ints(item_pairs)
// int32 per item = {expert, n, pair[0..n)}, n <= item_pairs pairs of that expert, in ascending pair order; experts in
// ascending order (gemv.hpp; item_pairs = MOE_ITEM_PAIRS for the mat-vec kernel, SKINNY_ITEM_PAIRS for the matrix-core
// one).  *n_items receives the count.  The order is a function of ids alone.
bool moe_group_supported(int n_pairs, int n_expert);
int moe_group(const int32_t *ids, int n_pairs, int n_expert, int32_t *items, int32_t *n_items, int item_pairs, hipStream_t stream);
// Small batches (T <= 64): router logits with the experts split over several workgroups per token, then routing and
// grouping in one single-workgroup launch.  Same results as moe_router_fused followed by moe_group; `logits`
// ([T][n_expert]) is required.
bool moe_router_group_supported(int E, int n_expert, int top_k, int T);
// arrive (optional): a device int that is zero between launches; with it the two launches become one, whose last-arriving
// workgroup routes and groups (same results)
int moe_router_group(const MoeRouteArgs &a, const float *x, int ldx, const float *norm_w, float eps, const float *W, int E,
                     float *logits, int T, int32_t *items, int32_t *n_items, int item_pairs, hipStream_t stream, int *arrive = nullptr);
// x[t] += sum_s weights[t][s] * y[t*top_k + s]
int moe_combine(float *x, const float *y, const float *w, int T, int n_embd, int top_k, hipStream_t stream);

// The pairs sorted by expert, for the expert launches of the large-tile GEMM (gemm.hpp): the pairs of an expert take
// consecutive slots from a multiple of 16 on (padding slots in between hold no pair), experts in ascending order, and
// every run of up to 128 slots of one expert is a tile {expert, first slot, pairs, 0}.
struct MoeSorted {
    int32_t *slot_of_pair = nullptr;   // [n_pairs]
    int32_t *pair_of_slot = nullptr;   // [moe_sort_slots()], -1 for a padding slot
    int32_t *tiles = nullptr;          // [moe_sort_max_tiles()][4]
    int32_t *counts = nullptr;         // [2]: tiles, slots in use
};
int moe_sort_slots(int n_pairs, int n_expert);         // slot capacity for any routing
int moe_sort_max_tiles(int n_pairs, int n_expert);
int moe_sort(const int32_t *ids, int n_pairs, int n_expert, const MoeSorted &out, hipStream_t stream);
// x[t] += sum_s weights[t][s] * y[slot_of_pair[t*top_k + s]]
int moe_combine_slots(float *x, const float *y, const float *w, const int32_t *slot_of_pair, int T, int n_embd, int top_k, hipStream_t stream);

}  // namespace mesh
