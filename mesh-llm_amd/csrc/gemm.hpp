// Prefill GEMM over tiled K-quant weights with f16 activations (gemm.hip), and its elementwise companions.
#pragma once

#include "gemv.hpp"

namespace mesh {

constexpr int SKINNY_ITEM_PAIRS = 16;      // pairs per work item of an expert launch of the skinny GEMM: one MFMA's columns

struct GemmArgs {
    const void *W = nullptr;         // tiled q4_K / q6_K matrix [M][K]
    const void *Wp = nullptr;        // optional: the same matrix in the GEMM layout (gemm_pack); used instead of W when set
    int type = -1;
    int M = 0, K = 0, T = 0;
    int M_pad = 0;                   // filled in by gemm_kquant
    const _Float16 *X = nullptr;     // [T][ldx] f16 activations; or, with x_k8, the k8-major layout of the skinny GEMM (below)
    int ldx = 0;
    bool x_k8 = false;               // X is k8-major: the matrix-core waves fetch their operand fragments from it directly
    float *Y = nullptr;              // [T][ldy] f32
    int ldy = 0;
    const float *bias = nullptr;     // [M] or null
    const float *residual = nullptr; // [T][ldres] or null; may alias Y
    int ldres = 0;
    // Several matrices sharing X in one launch (GEMM layout only: Wp holds their row blocks back to back, every matrix
    // but the last a whole number of 128-row blocks): matrix i starts at row block seg_begin[i] and has its own output,
    // bias and row count; M is the total.  n_seg == 1: the fields above describe the one matrix.
    int n_seg = 1;
    int seg_begin[3] = {0, 0, 0}, seg_M[3] = {0, 0, 0}, seg_ldy[3] = {0, 0, 0};
    float *seg_Y[3] = {nullptr, nullptr, nullptr};
    const float *seg_bias[3] = {nullptr, nullptr, nullptr};
    // SwiGLU pair: Wp is a gate/up pair packed by gemm_pack_pair (every row block 64 gate rows, then the same 64 up
    // rows), M their common row count; the launch writes f16(silu(gate) * up) in the k8-major layout to y16_k8 (Y unused).
    _Float16 *y16_k8 = nullptr;
    unsigned *sat = nullptr;         // optional device counter of SwiGLU outputs clamped to the f16 range (mesh_common.hpp: note_f16_clamp)
    bool big_tile = true;            // wide projections of long calls may take the 256-row tile
    bool narrow_tile = true;         // calls of at most 64 tokens may take the 64-token tile
    // Optional scratch for launches too narrow to fill the chip (few row blocks x token blocks): K is then split over
    // blockIdx.z, every slice writes its f32 partial tile to `part` ([slice][token][row of the launch]) and a second
    // kernel adds the slices in slice order and applies the epilogue.  Null: never split.  ksplit / k_per_split are
    // filled in by gemm_kquant.
    float *part = nullptr;
    size_t part_bytes = 0;
    int ksplit = 1, k_per_split = 0;
    // Optional, split launches only (ask gemm_split_count first): matrix i is the q / k / v projection of a layer
    // (kind[i], GEMV_KIND_*); the second kernel rotates q and k rows (neighbouring-pair RoPE) and appends k and v to
    // the f16 KV cache instead of storing them to their outputs, like the projection epilogues of the decode kernels.
    GemvRope rope;
    int kind[3] = {GEMV_KIND_PLAIN, GEMV_KIND_PLAIN, GEMV_KIND_PLAIN};
    // Expert launch (mixture of experts; GEMM layout and k8-major activations only, plain store or SwiGLU): X holds the
    // (token, slot) pairs sorted by expert (moe.hpp: moe_sort), T is its capacity in pair slots, and tile i of `tiles` =
    // {expert, first slot, slots, 0} multiplies slots [first, first + slots) (at most 128; first a multiple of 16) by the
    // matrix at Wp + expert * expert_stride.  *n_tiles (device) tiles are live, max_tiles bounds them for the grid.
    // Outputs are indexed by slot.
    const int32_t *tiles = nullptr, *n_tiles = nullptr;
    size_t expert_stride = 0;
    int max_tiles = 0;
};
int gemm_kquant(const GemmArgs &a, hipStream_t stream);
// Number of K slices gemm_kquant will use for this launch (1: not split).
int gemm_split_count(const GemmArgs &a);

// GEMM layout of a K-quant matrix: a second copy for the prefill GEMM, arranged by the workgroup tile that consumes it.
// One chunk per (128-row block, 64-element k-step), chunks of a row block consecutive in k.  A chunk holds, for each of
// the 256 (row, 32-element sub-block) pairs s = 2 * row + half, what the staging thread s needs, at s * stride of
// each section, so that every load of a staging wave covers one contiguous kilobyte:
//   q4_K (6144 B): [256 x 16 B quants: dword j = elements 8j..8j+3 in the low nibbles, 8j+4..8j+7 in the high ones]
//                  [256 x 8 B: f16 sc (the integer block scale), f16 c = 8 d sc - dmin m, f16 d, unused]
//   q6_K (8192 B): [256 x 16 B low nibbles, same order][256 x 8 B upper two bits: byte b of dword j/2 holds, from
//                  bit 4*(j%2), the bits of element 8j+b and, two bits up, of element 8j+4+b]
//                  [256 x 8 B: f16 sc of elements 0..15, f16 sc of elements 16..31, f16 d, unused]
// The kernel forms a weight as ((q - offset) * sc) * d + c: an exact small integer times the super-block's own f16
// scale, rounded once.  The fields are the ones the kernel would otherwise derive from the block headers, so both
// layouts give the same bits.  Rows beyond M are zero.
size_t gemm_packed_bytes(int type, int64_t M, int64_t K);
int gemm_pack(int type, const void *tiled, void *packed, int64_t M, int64_t K, hipStream_t stream);
// gate / up pair for the SwiGLU launch: row block b = gate rows [64b, 64b + 64) followed by up rows [64b, 64b + 64)
size_t gemm_packed_pair_bytes(int type, int64_t M, int64_t K);
int gemm_pack_pair(int type, const void *gate_tiled, const void *up_tiled, void *packed, int64_t M, int64_t K, hipStream_t stream);

// Skinny GEMM for a batch of decode steps (gemm_skinny.hip): up to three tiled K-quant matrices sharing the
// activations, any T (processed 16 columns at a time), epilogues as in the mat-vec kernel, integer dot products on
// the matrix cores.  Activations come in the "q16" layout quant16_k8 produces: per block of 16 tokens
// q16_block_bytes(K) bytes holding 16-bit fixed-point values per 32-element block as two int8 planes, the f32 block
// scales and the f32 block sums (gemm_skinny.hip describes the arrangement); columns beyond T hold zeros.
struct SkinnyArgs {
    GemvMat mat[3];
    int n_mat = 1;                   // for EPI_SWIGLU exactly 2 (gate, up), written through mat[0].y
    const uint8_t *xq = nullptr;     // q16 layout, ceil(T / 16) blocks of q16_block_bytes(K), 16-byte aligned
    int K = 0, T = 0;
    int epi = EPI_STORE;
    const float *residual = nullptr; // EPI_RESIDUAL: [T][ldres]; may alias y
    int ldres = 0;
    // RoPE + KV append in the epilogue of a q/k/v launch, as in the mat-vec kernel (gemv.hpp); EPI_STORE only
    GemvRope rope;
    int kind[3] = {GEMV_KIND_PLAIN, GEMV_KIND_PLAIN, GEMV_KIND_PLAIN};
    bool pair_launch = true;         // q4_K matrices followed by one q6_K matrix (q, k and a q6_K v): one launch for both types
    // Expert launch (mixture of experts): mat[] describe expert 0 of stacked, equally shaped tiled matrices; work
    // item i (blockIdx.y) = {expert, n, pair[0..n)} in the grouping kernel's format with SKINNY_ITEM_PAIRS pairs per item
    // (moe.hpp); slot j of an item reads activation column pair[j] / x_div of xq (any block of 16) and writes output row
    // pair[j].  One matrix or a gate / up pair (EPI_SWIGLU); T is not used.
    const int32_t *items = nullptr, *n_items = nullptr;
    int max_items = 0;
    int x_div = 1;
};
int gemm_skinny(const SkinnyArgs &a, hipStream_t stream);
// Bytes of one 16-token block of the q16 layout for rows of K elements.
size_t q16_block_bytes(int K);
// y (q16 layout) = quantise(rms_norm(x) * w) for T rows of n floats (w == null: quantise(x)); n a multiple of 32
int quant16_k8(const float *x, const float *w, float eps, int T, int n, uint8_t *y, hipStream_t stream);
// Mixture of experts: x[t] += sum_s w[t][s] * y[t * top_k + s] (moe.hpp: moe_combine) and, from the new x, the q16 activations
// quant16_k8(x, norm_w, eps) would produce, in one launch: the same bits as the two launches.  Rows of n <= 8192.
bool moe_combine_quant16_supported(int n);
int moe_combine_quant16(float *x, const float *y, const float *w, int T, int n, int top_k, const float *norm_w, float eps, uint8_t *yq, hipStream_t stream);
// The "k8-major" f16 layout the large-tile GEMM reads: blocks of 16 tokens, element (t, k) of block t / 16 at
// ((k / 8) * 16 + t % 16) * 8 + k % 8 within the block of 16 * K halfs; columns beyond T hold zeros.
// The same launches on the f16 matrix cores (gemm_skinny_f16.hip): activations in the k8-major f16 layout below, weights
// dequantised to f16 with one rounding each.  Faster than the integer kernel, less precise (f16 activations).
struct SkinnyF16Args {
    GemvMat mat[3];
    int n_mat = 1;                   // for EPI_SWIGLU exactly 2 (gate, up), written through mat[0].y and/or y16
    const _Float16 *x = nullptr;     // k8-major, ceil(T / 16) blocks of 16 * K halfs, 16-byte aligned
    int K = 0, T = 0;
    int epi = EPI_STORE;
    const float *residual = nullptr; // EPI_RESIDUAL: [T][ldres]; may alias y
    int ldres = 0;
    _Float16 *y16 = nullptr;         // optional f16 copy of matrix 0's output in the k8-major layout (feeds the next GEMM)
    unsigned *sat = nullptr;         // optional device counter of y16 values clamped to the f16 range
    // RoPE + KV append in the epilogue of a q/k/v launch, as in the mat-vec kernel (gemv.hpp); EPI_STORE only
    GemvRope rope;
    int kind[3] = {GEMV_KIND_PLAIN, GEMV_KIND_PLAIN, GEMV_KIND_PLAIN};
    // q4_K matrices followed by one q6_K matrix (q, k and a q6_K v): one launch for both types instead of two
    bool pair_launch = true;
    // RMS-norm hand-over between two launches (T <= 32: one launch each), in place of a norm kernel of its own between them.  The producer
    // (EPI_RESIDUAL, one matrix) also writes f16(y * norm_w) -- scaled by the next norm's weight but not yet by the
    // token's 1 / rms -- in the k8-major layout to norm_out.x16, and per workgroup the sum of y^2 of its rows for every
    // token to norm_out.part ([workgroups][16], or [workgroups][32] for a call of more than 16 tokens); gemm_skinny_f16_workgroups gives the workgroup count.  The consumer reads
    // those activations as its x, adds the partial sums in workgroup order and multiplies every accumulated product by
    // 1 / sqrt(sum / K + eps) before bias and epilogue: W . (y w / rms) = (W . (y w)) / rms.
    struct NormOut { const float *norm_w = nullptr; _Float16 *x16 = nullptr; float *part = nullptr; } norm_out;
    struct NormIn { const float *part = nullptr; int n_parts = 0; float eps = 0.f; } norm_in;
};
int gemm_skinny_f16(const SkinnyF16Args &a, hipStream_t stream);
// workgroups a producer launch of `a` will have (= partial sums per token it writes); 0 when the launch is not valid
int gemm_skinny_f16_workgroups(const SkinnyF16Args &a);
constexpr int SKINNY_F16_NORM_PARTS_MAX = 256;
constexpr int SKINNY_F16_NORM_TOKENS_MAX = 32;

// y (k8-major) = f16(rms_norm(x) * w) for T rows of n floats; pack_f16_k8: plain conversion
// (sat: optional device counter of values clamped to the f16 range, in all of these)
int rmsnorm_f16_k8(const float *x, const float *w, float eps, int T, int n, _Float16 *y, hipStream_t stream, unsigned *sat = nullptr);
int pack_f16_k8(const float *x, int T, int n, _Float16 *y, hipStream_t stream, unsigned *sat = nullptr);
// the same as rmsnorm_f16_k8 for n_slots (a multiple of 16) gathered rows: slot i holds row row_of_slot[i] / row_div of x, zeros when negative
int rmsnorm_f16_k8_gather(const float *x, const float *w, float eps, const int32_t *row_of_slot, int row_div, int n_slots, int n, _Float16 *y, hipStream_t stream,
                          unsigned *sat = nullptr);
int swiglu_f16_k8(const float *gate, const float *up, int T, int n, _Float16 *y, hipStream_t stream, unsigned *sat = nullptr);

int rmsnorm_f16(const float *x, const float *w, float eps, int T, int n, _Float16 *y, int ldy, hipStream_t stream, unsigned *sat = nullptr);
int swiglu_f16(const float *gate, const float *up, _Float16 *out, int64_t n, hipStream_t stream, unsigned *sat = nullptr);

}  // namespace mesh
