// GGUF row-major K-quant blocks <-> the tiled layout of gemv.hpp.  A pure permutation of bytes (plus zero
// blocks for rows that pad M to a multiple of 16), run once per tensor at load time.

#include "gemv.hpp"

namespace mesh {

// one wave per tile; lane l = 4*r + c copies a quarter of row r's block
template <bool TO_TILED>
__global__ __launch_bounds__(64) void repack_q4k_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                        int M, int nsb) {
    const int sb = blockIdx.x, R = blockIdx.y, lane = threadIdx.x;
    const int r = lane >> 2, c = lane & 3;
    const int row = R * TILE_ROWS + r;
    uint8_t *rm = const_cast<uint8_t *>(TO_TILED ? src : dst) + ((size_t)row * nsb + sb) * Q4_K_BYTES;
    uint8_t *tl = const_cast<uint8_t *>(TO_TILED ? dst : src) + ((size_t)R * nsb + sb) * Q4K_TILE_BYTES;
    const bool live = row < M;
    uint4 *t_hdr = reinterpret_cast<uint4 *>(tl + r * 16);
    uint4 *t_qs = reinterpret_cast<uint4 *>(tl + 256 + lane * 32);
    if (TO_TILED) {
        const uint4 z = make_uint4(0, 0, 0, 0);
        if (c == 0) *t_hdr = live ? *reinterpret_cast<const uint4 *>(rm) : z;
        t_qs[0] = live ? *reinterpret_cast<const uint4 *>(rm + 16 + 32 * c) : z;
        t_qs[1] = live ? *reinterpret_cast<const uint4 *>(rm + 16 + 32 * c + 16) : z;
    } else if (live) {
        if (c == 0) *reinterpret_cast<uint4 *>(rm) = *t_hdr;
        *reinterpret_cast<uint4 *>(rm + 16 + 32 * c) = t_qs[0];
        *reinterpret_cast<uint4 *>(rm + 16 + 32 * c + 16) = t_qs[1];
    }
}

// q6_K blocks are only 2-byte aligned in GGUF (210 bytes): move them as 16-bit words
template <bool TO_TILED>
__global__ __launch_bounds__(64) void repack_q6k_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                        int M, int nsb) {
    const int sb = blockIdx.x, R = blockIdx.y, lane = threadIdx.x;
    const int r = lane >> 2, c = lane & 3;
    const int row = R * TILE_ROWS + r;
    uint16_t *rm = reinterpret_cast<uint16_t *>(const_cast<uint8_t *>(TO_TILED ? src : dst) + ((size_t)row * nsb + sb) * Q6_K_BYTES);
    uint8_t *tl = const_cast<uint8_t *>(TO_TILED ? dst : src) + ((size_t)R * nsb + sb) * Q6K_TILE_BYTES;
    const bool live = row < M;
    if (!TO_TILED && !live) return;
    uint16_t *t_ql = reinterpret_cast<uint16_t *>(tl + r * 128 + 32 * c);          // 16 words
    uint16_t *t_qh = reinterpret_cast<uint16_t *>(tl + 2048 + r * 64 + 16 * c);    // 8 words
    uint16_t *t_sc = reinterpret_cast<uint16_t *>(tl + 3072 + r * 16);             // 8 words
    uint16_t *t_d = reinterpret_cast<uint16_t *>(tl + 3328 + r * 2);
    uint16_t *r_ql = rm + 16 * c, *r_qh = rm + 64 + 8 * c, *r_sc = rm + 96, *r_d = rm + 104;
    for (int i = 0; i < 16; ++i) {
        if (TO_TILED) t_ql[i] = live ? r_ql[i] : (uint16_t)0; else r_ql[i] = t_ql[i];
    }
    for (int i = 0; i < 8; ++i) {
        if (TO_TILED) t_qh[i] = live ? r_qh[i] : (uint16_t)0; else r_qh[i] = t_qh[i];
    }
    if (c == 0) {
        for (int i = 0; i < 8; ++i) {
            if (TO_TILED) t_sc[i] = live ? r_sc[i] : (uint16_t)0; else r_sc[i] = t_sc[i];
        }
        if (TO_TILED) *t_d = live ? *r_d : (uint16_t)0; else *r_d = *t_d;
    }
}

static int repack_common(bool to_tiled, int type, const void *src, void *dst, int64_t M, int64_t K, hipStream_t stream) {
    if (!type_is_tiled(type)) return fail(MESH_ERR_INVALID, "repack: type %d has no tiled layout", type);
    if (!src || !dst || M <= 0 || K <= 0 || K % QK_K) return fail(MESH_ERR_INVALID, "repack: bad shape M=%lld K=%lld", (long long)M, (long long)K);
    const int nsb = (int)(K / QK_K);
    const int64_t tile_rows = padded_rows(M) / TILE_ROWS;
    if (tile_rows > 65535) return fail(MESH_ERR_INVALID, "repack: %lld rows exceed the launch grid", (long long)M);
    const dim3 grid((unsigned)nsb, (unsigned)tile_rows);
    const uint8_t *s = static_cast<const uint8_t *>(src);
    uint8_t *d = static_cast<uint8_t *>(dst);
    if (type == MESH_Q4_K) {
        if (to_tiled) MESH_LAUNCH(repack_q4k_kernel<true>, grid, dim3(64), 0, stream, s, d, (int)M, nsb);
        else MESH_LAUNCH(repack_q4k_kernel<false>, grid, dim3(64), 0, stream, s, d, (int)M, nsb);
    } else {
        if (to_tiled) MESH_LAUNCH(repack_q6k_kernel<true>, grid, dim3(64), 0, stream, s, d, (int)M, nsb);
        else MESH_LAUNCH(repack_q6k_kernel<false>, grid, dim3(64), 0, stream, s, d, (int)M, nsb);
    }
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

int repack_tiled(int type, const void *src, void *dst, int64_t M, int64_t K, hipStream_t stream) {
    return repack_common(true, type, src, dst, M, K, stream);
}
int unpack_tiled(int type, const void *src, void *dst, int64_t M, int64_t K, hipStream_t stream) {
    return repack_common(false, type, src, dst, M, K, stream);
}

}  // namespace mesh
