// Boundary activation codec for gfx950: f32 <-> q8_0 blocks and f32 <-> f16.
//
// The packed layouts are ggml's ({fp16 d; int8 qs[32]} = 34 bytes, and IEEE binary16), and the arithmetic is
// that of quantize_row_q8_0_ref / dequantize_row_q8_0 / ggml_fp32_to_fp16_row, so a stage built on this
// library interoperates bit-for-bit with a ggml peer.  It replaces the raw-f32 boundary copy of
// third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:544-622.
//
// All four kernels are HBM-bound (5.0625 B/element for q8_0, 6 B/element for f16).  The q8_0 block is 34 bytes
// and only 2-byte aligned, so packed bytes are staged through LDS and cross HBM as aligned 16-byte vectors.
//
// Must be compiled with -ffp-contract=off: x*id feeds the rounding, and fusing that multiply into the rounding's
// addition would change results.

#include "mesh_common.hpp"

namespace mesh {

constexpr int CODEC_THREADS = 256;

// Streaming accesses: every byte is touched once, so loads and stores carry the non-temporal hint (they do not displace
// what the neighbouring kernels keep in L2 and the memory-side cache; measured +4..8 % on read:write mixes like these).
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float4 nt_load(const float4 *p) {
    const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint4 nt_load(const uint4 *p) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 nt_load(const uint2 *p) {
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p));
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ void nt_store(float4 *p, const float4 &a) {
    const f32x4 v = {a.x, a.y, a.z, a.w};
    __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(p));
}
__device__ __forceinline__ void nt_store(uint4 *p, const uint4 &a) {
    const u32x4 v = {a.x, a.y, a.z, a.w};
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}
constexpr int Q8_WG_BLOCKS = 256;                      // unpack: q8_0 blocks per workgroup, 8704 B packed in, 32 KiB of f32 out
constexpr int Q8_ITERS = Q8_WG_BLOCKS / 32;            // 8 lanes per block, 32 blocks per pass
static_assert((Q8_WG_BLOCKS * Q8_0_BYTES) % 16 == 0, "workgroup input must start 16-byte aligned");
constexpr int Q8_PACK_ITERS = 2;                      // pack: 8 lanes per block, passes of 8 blocks per wave
constexpr int Q8_PACK_WG_BLOCKS = 8 * Q8_PACK_ITERS * (CODEC_THREADS / 64);

template <bool ALIGNED>
__global__ __launch_bounds__(CODEC_THREADS) void unpack_q8_0_kernel(const uint8_t *__restrict__ x,
                                                                    float *__restrict__ y, int64_t nblk) {
    __shared__ __align__(16) uint8_t stage[Q8_WG_BLOCKS * Q8_0_BYTES];
    const int tid = threadIdx.x;
    const int part = tid & 7;
    const int sub = tid >> 3;
    const int64_t blk0 = (int64_t)blockIdx.x * Q8_WG_BLOCKS;
    const int64_t left = nblk - blk0;
    const int nb_here = left < Q8_WG_BLOCKS ? (int)left : Q8_WG_BLOCKS;
    const int nbytes = nb_here * Q8_0_BYTES;
    const uint8_t *in = x + blk0 * Q8_0_BYTES;

    if (ALIGNED) {
        const int n16 = nbytes >> 4;
        const uint4 *i4 = reinterpret_cast<const uint4 *>(in);
        uint4 *s4 = reinterpret_cast<uint4 *>(stage);
        for (int i = tid; i < n16; i += CODEC_THREADS) s4[i] = nt_load(i4 + i);
        const int done = n16 << 4;
        const uint16_t *i2 = reinterpret_cast<const uint16_t *>(in + done);
        uint16_t *s2 = reinterpret_cast<uint16_t *>(stage + done);
        for (int i = tid; i < ((nbytes - done) >> 1); i += CODEC_THREADS) s2[i] = i2[i];
    } else {
        const uint16_t *i2 = reinterpret_cast<const uint16_t *>(in);
        uint16_t *s2 = reinterpret_cast<uint16_t *>(stage);
        for (int i = tid; i < (nbytes >> 1); i += CODEC_THREADS) s2[i] = i2[i];
    }
    __syncthreads();

#pragma unroll
    for (int it = 0; it < Q8_ITERS; ++it) {
        const int b = it * 32 + sub;
        if (b < nb_here) {
            const uint8_t *o = stage + b * Q8_0_BYTES;
            const float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(o));
            const uint16_t *iq = reinterpret_cast<const uint16_t *>(o + 2 + part * 4);
            const uint32_t q = (uint32_t)iq[0] | ((uint32_t)iq[1] << 16);
            float4 r;
            r.x = (float)(int8_t)(q & 0xFF) * d;
            r.y = (float)(int8_t)((q >> 8) & 0xFF) * d;
            r.z = (float)(int8_t)((q >> 16) & 0xFF) * d;
            r.w = (float)(int8_t)(q >> 24) * d;
            float *p = y + (blk0 + b) * QK8_0 + part * 4;
            if (ALIGNED) {
                nt_store(reinterpret_cast<float4 *>(p), r);
            } else {
                p[0] = r.x; p[1] = r.y; p[2] = r.z; p[3] = r.w;
            }
        }
    }
}

// Orders a wave's own LDS writes before its own LDS reads of other lanes' data (no workgroup barrier involved).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// roundf (half away from zero) followed by the float -> int conversion, for |x| < 2^23: adding the largest float
// below one half, with the sign of x, and truncating gives the same integer as roundf for every float (the sum of
// k + 0.5 and the constant is a tie that rounds up to k + 1; every smaller fraction stays below k + 1).
__device__ __forceinline__ int round_half_away_i32(float x) { return (int)(x + copysignf(0.49999997f, x)); }

__device__ __forceinline__ uint32_t pack4_i8_fast(float a, float b, float c, float d) {
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)round_half_away_i32(b), (uint32_t)round_half_away_i32(a), 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)round_half_away_i32(d), (uint32_t)round_half_away_i32(c), 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

template <int CTRL>
__device__ __forceinline__ float quad_swizzle(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}

// f32 -> q8_0.  Eight lanes per block (4 values each), 8 blocks per wave and pass, two passes: every load instruction
// of a wave covers one contiguous kilobyte.  The wave stages its 544 packed bytes (a multiple of 16) in its own LDS
// region and copies them out itself, so no workgroup barrier separates loads and stores.  The kernel is as much VALU-
// as HBM-bound (two IEEE divides, 32 roundings and the byte packing per block), hence the maximum over the eight lanes
// through DPP, the add-and-truncate rounding and v_perm packing.
template <bool ALIGNED>
__global__ __launch_bounds__(CODEC_THREADS) void pack_q8_0_kernel(const float *__restrict__ x,
                                                                       uint8_t *__restrict__ y, int64_t nblk) {
    constexpr int ITERS = Q8_PACK_ITERS, WB = 8 * ITERS, WAVES = CODEC_THREADS / 64;
    static_assert(ITERS % 2 == 0 && (WB * Q8_0_BYTES) % 16 == 0, "passes come in pairs; a wave's output starts 16-byte aligned");
    __shared__ __align__(16) uint8_t stage_all[WAVES][WB * Q8_0_BYTES];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int part = lane & 7, sub = lane >> 3;
    uint8_t *stage = stage_all[wave];
    const int64_t blk0 = ((int64_t)blockIdx.x * WAVES + wave) * WB;
    const int64_t left = nblk - blk0;
    if (left <= 0) return;
    const int nb_here = left < WB ? (int)left : WB;

    float4 va[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int b = it * 8 + sub;
        va[it] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (b < nb_here) {
            const float *p = x + (blk0 + b) * QK8_0 + part * 4;
            if (ALIGNED) va[it] = nt_load(reinterpret_cast<const float4 *>(p));
            else va[it] = make_float4(p[0], p[1], p[2], p[3]);
        }
    }
    // Per pair of passes: the block maxima of both, then one divide sequence for the two (lanes 0..3 of each eight take
    // the first pass's block, lanes 4..7 the second's, and each lane fetches the other pass's values from its mirror lane)
    const bool first = part < 4;
#pragma unroll
    for (int pair = 0; pair < ITERS; pair += 2) {
        float am[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float4 a = va[pair + h];
            float amax = fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w)));
            amax = fmaxf(amax, quad_swizzle<0xB1>(amax));      // lanes 1,0,3,2 of the quad
            amax = fmaxf(amax, quad_swizzle<0x4E>(amax));      // lanes 2,3,0,1
            am[h] = fmaxf(amax, quad_swizzle<0x141>(amax));    // row_half_mirror: the other quad of the eight lanes
        }
        const float d_mine = (first ? am[0] : am[1]) / 127.0f;       // IEEE divide
        const float id_mine = d_mine != 0.0f ? 1.0f / d_mine : 0.0f;  // from the unrounded f32 d
        const float d_other = quad_swizzle<0x141>(d_mine), id_other = quad_swizzle<0x141>(id_mine);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int b = (pair + h) * 8 + sub;
            const float4 a = va[pair + h];
            const bool mine = first == (h == 0);
            const float d = mine ? d_mine : d_other, id = mine ? id_mine : id_other;
            const uint32_t q0 = pack4_i8_fast(a.x * id, a.y * id, a.z * id, a.w * id);
            uint8_t *o = stage + b * Q8_0_BYTES;
            if (part == 0) *reinterpret_cast<uint16_t *>(o) = f32_to_f16_bits(d);
            uint16_t *oq = reinterpret_cast<uint16_t *>(o + 2 + part * 4);      // 2 bytes into a 34-byte block: 16-bit aligned only
            oq[0] = (uint16_t)(q0 & 0xFFFFu);
            oq[1] = (uint16_t)(q0 >> 16);
        }
    }
    wave_lds_sync();

    const int nbytes = nb_here * Q8_0_BYTES;
    uint8_t *out = y + blk0 * Q8_0_BYTES;
    if (ALIGNED) {
        const int n16 = nbytes >> 4;
        const uint4 *s4 = reinterpret_cast<const uint4 *>(stage);
        uint4 *o4 = reinterpret_cast<uint4 *>(out);
        for (int i = lane; i < n16; i += 64) nt_store(o4 + i, s4[i]);
        const int done = n16 << 4;
        const uint16_t *s2 = reinterpret_cast<const uint16_t *>(stage + done);
        uint16_t *o2 = reinterpret_cast<uint16_t *>(out + done);
        for (int i = lane; i < ((nbytes - done) >> 1); i += 64) o2[i] = s2[i];
    } else {
        const uint16_t *s2 = reinterpret_cast<const uint16_t *>(stage);
        uint16_t *o2 = reinterpret_cast<uint16_t *>(out);
        for (int i = lane; i < (nbytes >> 1); i += 64) o2[i] = s2[i];
    }
}

// f16 -> f32, 8 elements per thread as two groups of four, a workgroup's 1024 elements apart: each load instruction of a
// wave covers 512 contiguous bytes and each store instruction one contiguous kilobyte
template <bool ALIGNED>
__global__ __launch_bounds__(CODEC_THREADS) void unpack_f16_kernel(const uint16_t *__restrict__ x,
                                                                   float *__restrict__ y, int64_t n) {
    const int64_t base = (int64_t)blockIdx.x * (CODEC_THREADS * 8);
    if (ALIGNED && base + CODEC_THREADS * 8 <= n) {
        const int64_t i0 = base + threadIdx.x * 4, i1 = i0 + CODEC_THREADS * 4;
        const uint2 v = nt_load(reinterpret_cast<const uint2 *>(x + i0));
        const uint2 w = nt_load(reinterpret_cast<const uint2 *>(x + i1));
        float4 a, b;
        a.x = f16_bits_to_f32((uint16_t)(v.x & 0xFFFF)); a.y = f16_bits_to_f32((uint16_t)(v.x >> 16));
        a.z = f16_bits_to_f32((uint16_t)(v.y & 0xFFFF)); a.w = f16_bits_to_f32((uint16_t)(v.y >> 16));
        b.x = f16_bits_to_f32((uint16_t)(w.x & 0xFFFF)); b.y = f16_bits_to_f32((uint16_t)(w.x >> 16));
        b.z = f16_bits_to_f32((uint16_t)(w.y & 0xFFFF)); b.w = f16_bits_to_f32((uint16_t)(w.y >> 16));
        nt_store(reinterpret_cast<float4 *>(y + i0), a);
        nt_store(reinterpret_cast<float4 *>(y + i1), b);
    } else {
        // last (partial) workgroup, or unaligned pointers
        for (int64_t j = base + threadIdx.x; j < n && j < base + CODEC_THREADS * 8; j += CODEC_THREADS) y[j] = f16_bits_to_f32(x[j]);
    }
}

// f32 -> f16, 8 elements per thread as two groups of four, a workgroup's 1024 elements apart: each load instruction of a
// wave covers one contiguous kilobyte and each store instruction 512 contiguous bytes
template <bool ALIGNED>
__global__ __launch_bounds__(CODEC_THREADS) void pack_f16_kernel(const float *__restrict__ x,
                                                                 uint16_t *__restrict__ y, int64_t n) {
    const int64_t base = (int64_t)blockIdx.x * (CODEC_THREADS * 8);
    if (ALIGNED && base + CODEC_THREADS * 8 <= n) {
        const int64_t i0 = base + threadIdx.x * 4, i1 = i0 + CODEC_THREADS * 4;
        const float4 a = nt_load(reinterpret_cast<const float4 *>(x + i0));
        const float4 b = nt_load(reinterpret_cast<const float4 *>(x + i1));
        const u32x2 oa = {(uint32_t)f32_to_f16_bits(a.x) | ((uint32_t)f32_to_f16_bits(a.y) << 16),
                          (uint32_t)f32_to_f16_bits(a.z) | ((uint32_t)f32_to_f16_bits(a.w) << 16)};
        const u32x2 ob = {(uint32_t)f32_to_f16_bits(b.x) | ((uint32_t)f32_to_f16_bits(b.y) << 16),
                          (uint32_t)f32_to_f16_bits(b.z) | ((uint32_t)f32_to_f16_bits(b.w) << 16)};
        __builtin_nontemporal_store(oa, reinterpret_cast<u32x2 *>(y + i0));
        __builtin_nontemporal_store(ob, reinterpret_cast<u32x2 *>(y + i1));
    } else {
        // last (partial) workgroup, or unaligned pointers
        for (int64_t j = base + threadIdx.x; j < n && j < base + CODEC_THREADS * 8; j += CODEC_THREADS) y[j] = f32_to_f16_bits(x[j]);
    }
}

static inline bool aligned16(const void *a, const void *b) {
    return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
}

int act_pack_dev(int fmt, const float *src, void *dst, int64_t n, hipStream_t stream) {
    if (n < 0 || (n > 0 && (!src || !dst))) return fail(MESH_ERR_INVALID, "mesh_act_pack: null pointer or negative count");
    if (n == 0) return MESH_OK;
    const bool al = aligned16(src, dst);
    switch (fmt) {
        case MESH_F32:
            MESH_HIP_TRY(hipMemcpyAsync(dst, src, (size_t)n * 4, hipMemcpyDeviceToDevice, stream));
            return MESH_OK;
        case MESH_F16: {
            const int64_t grid = (n + CODEC_THREADS * 8 - 1) / (CODEC_THREADS * 8);
            if (al) MESH_LAUNCH(pack_f16_kernel<true>, dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream, src, (uint16_t *)dst, n);
            else MESH_LAUNCH(pack_f16_kernel<false>, dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream, src, (uint16_t *)dst, n);
            MESH_LAUNCH_CHECK();
            return MESH_OK;
        }
        case MESH_Q8_0: {
            if (n % QK8_0) return fail(MESH_ERR_INVALID, "mesh_act_pack: q8_0 needs a multiple of 32 elements, got %lld", (long long)n);
            const int64_t nblk = n / QK8_0;
            const int64_t grid = (nblk + Q8_PACK_WG_BLOCKS - 1) / Q8_PACK_WG_BLOCKS;
            if (al) MESH_LAUNCH(pack_q8_0_kernel<true>, dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream, src, (uint8_t *)dst, nblk);
            else MESH_LAUNCH(pack_q8_0_kernel<false>, dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream, src, (uint8_t *)dst, nblk);
            MESH_LAUNCH_CHECK();
            return MESH_OK;
        }
        default:
            return fail(MESH_ERR_INVALID, "mesh_act_pack: format %d is not an activation format", fmt);
    }
}

int act_unpack_dev(int fmt, const void *src, float *dst, int64_t n, hipStream_t stream) {
    if (n < 0 || (n > 0 && (!src || !dst))) return fail(MESH_ERR_INVALID, "mesh_act_unpack: null pointer or negative count");
    if (n == 0) return MESH_OK;
    const bool al = aligned16(src, dst);
    switch (fmt) {
        case MESH_F32:
            MESH_HIP_TRY(hipMemcpyAsync(dst, src, (size_t)n * 4, hipMemcpyDeviceToDevice, stream));
            return MESH_OK;
        case MESH_F16: {
            const int64_t grid = (n + CODEC_THREADS * 8 - 1) / (CODEC_THREADS * 8);
            if (al) MESH_LAUNCH(unpack_f16_kernel<true>, dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream, (const uint16_t *)src, dst, n);
            else MESH_LAUNCH(unpack_f16_kernel<false>, dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream, (const uint16_t *)src, dst, n);
            MESH_LAUNCH_CHECK();
            return MESH_OK;
        }
        case MESH_Q8_0: {
            if (n % QK8_0) return fail(MESH_ERR_INVALID, "mesh_act_unpack: q8_0 needs a multiple of 32 elements, got %lld", (long long)n);
            const int64_t nblk = n / QK8_0;
            const int64_t grid = (nblk + Q8_WG_BLOCKS - 1) / Q8_WG_BLOCKS;
            if (al) MESH_LAUNCH(unpack_q8_0_kernel<true>, dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream, (const uint8_t *)src, dst, nblk);
            else MESH_LAUNCH(unpack_q8_0_kernel<false>, dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream, (const uint8_t *)src, dst, nblk);
            MESH_LAUNCH_CHECK();
            return MESH_OK;
        }
        default:
            return fail(MESH_ERR_INVALID, "mesh_act_unpack: format %d is not an activation format", fmt);
    }
}

}  // namespace mesh
