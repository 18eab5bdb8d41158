// Dequant-fused matrix-vector products over K-quant weights (decode path), and the tiled weight layout they read.
#pragma once

#include "mesh_common.hpp"

namespace mesh {

// ---- tiled K-quant layout -----------------------------------------------------------------------------------
// A K-quant matrix [M rows][K] is stored as tiles of 16 rows x one 256-element super-block, tile (R, sb) at
// byte offset (R * K/256 + sb) * 16 * block_bytes: a workgroup streaming 16 rows along K reads one contiguous
// run.  Byte count equals the GGUF tensor's (M is padded to 16 with zero blocks).  Inside a tile, lane
// l = g*16 + r (r = row in tile, g = 0..3) owns the bytes that decode elements 32*s + 8*g + i, s = 0..7, i = 0..7:
//   q4_K (2304 B): [16 x 16 B headers {d, dmin, scales[12]}] [plane0: 64 x 16 B] [plane1: 64 x 16 B];
//                  lane's 16 B of plane p = qs[64p + 8g .. +8] | qs[64p + 32 + 8g .. +8]
//   q6_K (3360 B): [ql plane n=0: 64 x 16 B] [ql plane n=1] [qh: 64 x 16 B] [16 x 16 B scales] [16 x fp16 d];
//                  lane's 16 B of ql plane n = ql[64n + 8g .. +8] | ql[64n + 32 + 8g .. +8],
//                  lane's 16 B of qh = qh[8g .. +8] | qh[32 + 8g .. +8]
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

struct GemvArgs {
    GemvMat mat[3];
    int n_mat = 1;             // matrices sharing x (q, k, v); for EPI_SWIGLU exactly 2, written through mat[0].y
    const float *x = nullptr;  // [T][ldx]
    int ldx = 0;
    int K = 0;
    int T = 0;                 // any T; processed 4 columns at a time
    const float *norm_w = nullptr;   // if set: x is RMS-normalised (eps) and scaled by norm_w[K] on the fly
    float eps = 0.f;
    const float *residual = nullptr; // EPI_RESIDUAL: [T][ldres]; may alias y
    int ldres = 0;
    int epi = EPI_STORE;
};

int gemv(const GemvArgs &a, hipStream_t stream);

}  // namespace mesh
