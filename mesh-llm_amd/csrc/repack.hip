// GGUF row-major K-quant blocks <-> the tiled layout of gemv.hpp.  A pure permutation of bytes (plus zero
// blocks for rows that pad M to a multiple of 16), run once per tensor at load time.

#include "gemv.hpp"

namespace mesh {

// one wave per tile; lane l = g*16 + r
template <bool TO_TILED>
__global__ __launch_bounds__(64) void repack_q4k_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                        int M, int nsb) {
    const int sb = blockIdx.x, R = blockIdx.y, lane = threadIdx.x;
    const int r = lane & 15, g = lane >> 4;
    const int row = R * TILE_ROWS + r;
    const uint8_t *rm_c = (TO_TILED ? src : dst) + ((size_t)row * nsb + sb) * Q4_K_BYTES;   // row-major block
    uint8_t *tl = const_cast<uint8_t *>(TO_TILED ? dst : src) + ((size_t)R * nsb + sb) * Q4K_TILE_BYTES;
    uint8_t *rm = const_cast<uint8_t *>(rm_c);
    const bool live = row < M;
    if (TO_TILED) {
        if (g == 0) {
            uint4 h = make_uint4(0, 0, 0, 0);
            if (live) h = *reinterpret_cast<const uint4 *>(rm);
            *reinterpret_cast<uint4 *>(tl + r * 16) = h;
        }
        for (int p = 0; p < 2; ++p) {
            uint2 a = make_uint2(0, 0), b = make_uint2(0, 0);
            if (live) {
                a = *reinterpret_cast<const uint2 *>(rm + 16 + 64 * p + 8 * g);
                b = *reinterpret_cast<const uint2 *>(rm + 16 + 64 * p + 32 + 8 * g);
            }
            *reinterpret_cast<uint4 *>(tl + 256 + p * 1024 + lane * 16) = make_uint4(a.x, a.y, b.x, b.y);
        }
    } else if (live) {
        if (g == 0) *reinterpret_cast<uint4 *>(rm) = *reinterpret_cast<const uint4 *>(tl + r * 16);
        for (int p = 0; p < 2; ++p) {
            const uint4 v = *reinterpret_cast<const uint4 *>(tl + 256 + p * 1024 + lane * 16);
            *reinterpret_cast<uint2 *>(rm + 16 + 64 * p + 8 * g) = make_uint2(v.x, v.y);
            *reinterpret_cast<uint2 *>(rm + 16 + 64 * p + 32 + 8 * g) = make_uint2(v.z, v.w);
        }
    }
}

template <bool TO_TILED>
__global__ __launch_bounds__(64) void repack_q6k_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                        int M, int nsb) {
    const int sb = blockIdx.x, R = blockIdx.y, lane = threadIdx.x;
    const int r = lane & 15, g = lane >> 4;
    const int row = R * TILE_ROWS + r;
    uint8_t *rm = const_cast<uint8_t *>(TO_TILED ? src : dst) + ((size_t)row * nsb + sb) * Q6_K_BYTES;   // 2-byte aligned
    uint8_t *tl = const_cast<uint8_t *>(TO_TILED ? dst : src) + ((size_t)R * nsb + sb) * Q6K_TILE_BYTES;
    const bool live = row < M;
    if (!TO_TILED && !live) return;
    for (int n = 0; n < 2; ++n) {
        for (int i = 0; i < 8; ++i) {
            uint8_t *ta = tl + n * 1024 + lane * 16 + i, *tb = ta + 8;
            uint8_t *ra = rm + 64 * n + 8 * g + i, *rb = ra + 32;
            uint8_t *th = tl + 2048 + lane * 16 + 8 * n + i;
            uint8_t *rh = rm + 128 + 32 * n + 8 * g + i;
            if (TO_TILED) {
                *ta = live ? *ra : 0; *tb = live ? *rb : 0; *th = live ? *rh : 0;
            } else {
                *ra = *ta; *rb = *tb; *rh = *th;
            }
        }
    }
    if (g == 0) {
        for (int i = 0; i < 16; ++i) {
            if (TO_TILED) tl[3072 + r * 16 + i] = live ? rm[192 + i] : 0;
            else rm[192 + i] = tl[3072 + r * 16 + i];
        }
        for (int i = 0; i < 2; ++i) {
            if (TO_TILED) tl[3328 + r * 2 + i] = live ? rm[208 + i] : 0;
            else rm[208 + i] = tl[3328 + r * 2 + i];
        }
    }
}

static int repack_common(bool to_tiled, int type, const void *src, void *dst, int64_t M, int64_t K, hipStream_t stream) {
    if (!type_is_tiled(type)) return fail(MESH_ERR_INVALID, "repack: type %d has no tiled layout", type);
    if (!src || !dst || M <= 0 || K <= 0 || K % QK_K) return fail(MESH_ERR_INVALID, "repack: bad shape M=%lld K=%lld", (long long)M, (long long)K);
    const int nsb = (int)(K / QK_K);
    const dim3 grid((unsigned)nsb, (unsigned)(padded_rows(M) / TILE_ROWS));
    if (grid.y > 65535u * 16u) return fail(MESH_ERR_INVALID, "repack: too many rows");
    const uint8_t *s = static_cast<const uint8_t *>(src);
    uint8_t *d = static_cast<uint8_t *>(dst);
    if (type == MESH_Q4_K) {
        if (to_tiled) repack_q4k_kernel<true><<<grid, dim3(64), 0, stream>>>(s, d, (int)M, nsb);
        else repack_q4k_kernel<false><<<grid, dim3(64), 0, stream>>>(s, d, (int)M, nsb);
    } else {
        if (to_tiled) repack_q6k_kernel<true><<<grid, dim3(64), 0, stream>>>(s, d, (int)M, nsb);
        else repack_q6k_kernel<false><<<grid, dim3(64), 0, stream>>>(s, d, (int)M, nsb);
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
