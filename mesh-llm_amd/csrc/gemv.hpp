// Dequant-fused matrix-vector products over K-quant weights (decode path), and the tiled weight layout they read.
#pragma once

#include "mesh_common.hpp"

namespace mesh {

// ---- tiled K-quant layout -----------------------------------------------------------------------------------
// A K-quant matrix [M rows][K] is stored as tiles of 16 rows x one 256-element super-block, tile (R, sb) at
// byte offset (R * K/256 + sb) * 16 * block_bytes, so the workgroup that owns 16 rows streams one contiguous
// run along K.  Byte count equals the GGUF tensor's (M is padded to 16 with zero blocks).  Inside a tile the
// per-row fields are regrouped so that every access is an aligned 16-byte vector and a wave's loads are dense:
//   q4_K (2304 B): [16 x 16 B headers {d, dmin, scales[12]}] [16 x 128 B qs]
//   q6_K (3360 B): [16 x 128 B ql] [16 x 64 B qh] [16 x 16 B scales] [16 x fp16 d]
// Lane l = 4*r + c of a wave works on row r, quarter c of the super-block:
//   q4_K: qs[32c .. 32c+32)  -> sub-blocks 2c (low nibbles) and 2c+1 (high nibbles)
//   q6_K: half n = c/2, u = c%2: ql[64n+16u..+16), ql[64n+32+16u..+16), qh[32n+16u..+16) -> elements
//         128n + 32t + 16u + i, t = 0..3, i = 0..15 (one 16-element scale group per t)
constexpr int TILE_ROWS = 16;
constexpr int Q4K_TILE_BYTES = TILE_ROWS * Q4_K_BYTES;   // 2304
constexpr int Q6K_TILE_BYTES = TILE_ROWS * Q6_K_BYTES;   // 3360

inline bool type_is_tiled(int type) { return type == MESH_Q4_K || type == MESH_Q6_K; }
inline int64_t padded_rows(int64_t M) { return (M + TILE_ROWS - 1) / TILE_ROWS * TILE_ROWS; }
// bytes of the tiled copy of an [M][K] matrix
inline int64_t tiled_bytes(int type, int64_t M, int64_t K) { return padded_rows(M) * row_bytes(type, K); }

// GGUF row-major blocks (device) -> tiled layout (device).  dst must hold tiled_bytes().
int repack_tiled(int type, const void *src_rowmajor, void *dst_tiled, int64_t M, int64_t K, hipStream_t stream);
// inverse, for tests: tiled -> GGUF row-major
int unpack_tiled(int type, const void *src_tiled, void *dst_rowmajor, int64_t M, int64_t K, hipStream_t stream);

// ---- fused GEMV ---------------------------------------------------------------------------------------------
enum GemvEpilogue {
    EPI_STORE = 0,      // y = W x (+ bias)
    EPI_RESIDUAL = 1,   // y = residual + W x (+ bias)
    EPI_SWIGLU = 2      // y = silu(W0 x) * (W1 x); mat[0] = gate, mat[1] = up
};

struct GemvMat {
    const void *W = nullptr;   // tiled for K-quants, GGUF row-major otherwise
    int type = -1;
    int M = 0;
    float *y = nullptr;        // [T][ldy]
    int ldy = 0;
    const float *bias = nullptr;
};

// RoPE + KV append in the epilogue of a q/k/v launch (NORM pairing: a pair's two rows are neighbours, so they live in
// one 16-row tile): q rows are rotated before they are stored, k rows are rotated and stored as f16 in the K cache
// at the token's position, v rows go to the V cache.  Same arithmetic, hence the same bits, as rope_kv_kernel.
// A work item of a grouped expert launch: MOE_ITEM_INTS int32 = {expert, n, pair[0..n), unused...}, 1 <= n <= MOE_ITEM_PAIRS.
constexpr int MOE_ITEM_PAIRS = 4, MOE_ITEM_INTS = 8;
// int32 per item when an item holds up to item_pairs pairs: expert, n, the pairs, padded to a multiple of 4
__host__ __device__ inline int moe_item_ints(int item_pairs) { return (2 + item_pairs + 3) / 4 * 4; }
// upper bound on the items n_pairs pairs over n_expert experts can form (sum over experts of ceil(count / item_pairs))
inline int moe_max_items(int n_pairs, int n_expert, int item_pairs = MOE_ITEM_PAIRS) {
    const int used = n_pairs < n_expert ? n_pairs : n_expert;
    const int bound = used + n_pairs / item_pairs;
    return bound < n_pairs ? bound : n_pairs;
}

enum { GEMV_KIND_PLAIN = 0, GEMV_KIND_Q = 1, GEMV_KIND_K = 2, GEMV_KIND_V = 3 };
struct GemvRope {
    const int32_t *pos = nullptr, *seq = nullptr;      // device, [T]; pos == nullptr: no fusion
    const float *inv_freq = nullptr;
    uint16_t *kcache = nullptr, *vcache = nullptr;     // this layer's f16 rows [n_seq][n_kv][n_ctx][head_dim]
    int head_dim = 0, n_rot = 0, n_kv = 0, n_ctx = 0;
};

struct GemvArgs {
    GemvMat mat[3];
    int n_mat = 1;             // matrices sharing x (q, k, v); for EPI_SWIGLU exactly 2, written through mat[0].y
    const float *x = nullptr;  // [T][ldx]
    int ldx = 0;
    int K = 0;
    int T = 0;                 // any T; processed a few columns at a time
    const float *norm_w = nullptr;   // if set: x is RMS-normalised (eps) and scaled by norm_w[K] on the fly
    float eps = 0.f;
    const float *residual = nullptr; // EPI_RESIDUAL: [T][ldres]; may alias y
    int ldres = 0;
    int epi = EPI_STORE;
    // Expert indirection (MoE): when expert_ids is set, the launch runs n_pairs independent single-column products;
    // pair p uses expert expert_ids[p] (device array) of every matrix -- W points at expert 0, experts are stacked --
    // reads activation column p / x_div of x and writes row p of y.  T is ignored.
    const int32_t *expert_ids = nullptr;
    int n_pairs = 0;
    int x_div = 1;
    // Pairs grouped by expert (moe_group): when items is set as well, the launch walks the item list instead, so
    // that the pairs of an item (up to MOE_ITEM_PAIRS, all of one expert) share one pass over that expert's weights.
    // items / n_items are device memory, max_items bounds *n_items (the launch's grid is sized by it).
    const int32_t *items = nullptr;
    const int32_t *n_items = nullptr;
    int max_items = 0;
    int grouped_oversub = 8;        // grouped launches: workgroups per compute unit and item
    // Fused RoPE / KV append: kind[i] says what matrix i produces (tiled K-quant matrices, EPI_STORE, no experts only)
    GemvRope rope;
    int kind[3] = {GEMV_KIND_PLAIN, GEMV_KIND_PLAIN, GEMV_KIND_PLAIN};
    // Activations quantised by their producer (T == 1).  xq_out: an EPI_SWIGLU launch also leaves its output vector in
    // the "xq" layout below (the 16-bit fixed-point form every mat-vec workgroup otherwise derives from the f32 vector for
    // itself, the same bits) and skips the f32 store.  xq_in: the launch reads its activations from such a buffer
    // instead of x (no norm).  Callers ask gemv_xq_out_supported / gemv_xq_in_supported first.
    uint8_t *xq_out = nullptr;
    const uint8_t *xq_in = nullptr;
};
// "xq" layout of a vector of K elements (K a multiple of 256): int8 hi[K] | int8 lo[K] | f32 d[K / 32] | f32 s[K / 32] |
// int32 i16[K / 16]: element k ~ d[k / 32] * (256 * hi[k] + lo[k]), s = d * (sum of the block's 32 fixed-point values),
// i16 = sum of 16 of them (what the q6_K kernels need)
inline size_t xq_bytes(int K) { return (size_t)K * 2 + (size_t)(K / 32) * 8 + (size_t)(K / 16) * 4; }
bool gemv_xq_out_supported(const GemvArgs &a);
bool gemv_xq_in_supported(const GemvArgs &a);
// whether gemv() will honour a.rope for this argument set (otherwise the caller runs rope_kv itself)
bool gemv_can_fuse_rope(const GemvArgs &a);

int gemv(const GemvArgs &a, hipStream_t stream);

}  // namespace mesh
