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
// Must be compiled with -ffp-contract=off: x*id feeds roundf, and fusing that multiply into roundf's
// internal subtraction would change results.

#include "mesh_common.hpp"

namespace mesh {

constexpr int CODEC_THREADS = 256;
constexpr int Q8_WG_BLOCKS = 256;                      // q8_0 blocks per workgroup: 32 KiB of f32, 8704 B packed
constexpr int Q8_ITERS = Q8_WG_BLOCKS / 32;            // 8 lanes per block, 32 blocks per pass
static_assert((Q8_WG_BLOCKS * Q8_0_BYTES) % 16 == 0, "workgroup output must start 16-byte aligned");

__device__ __forceinline__ uint32_t pack4_i8(float a, float b, float c, float d) {
    const int qa = (int)roundf(a), qb = (int)roundf(b), qc = (int)roundf(c), qd = (int)roundf(d);
    return (uint32_t)(qa & 0xFF) | ((uint32_t)(qb & 0xFF) << 8) | ((uint32_t)(qc & 0xFF) << 16) |
           ((uint32_t)(qd & 0xFF) << 24);
}

template <bool ALIGNED>
__global__ __launch_bounds__(CODEC_THREADS) void pack_q8_0_kernel(const float *__restrict__ x,
                                                                  uint8_t *__restrict__ y, int64_t nblk) {
    __shared__ __align__(16) uint8_t stage[Q8_WG_BLOCKS * Q8_0_BYTES];
    const int tid = threadIdx.x;
    const int part = tid & 7;    // which 4 of the block's 32 values
    const int sub = tid >> 3;    // block within a pass
    const int64_t blk0 = (int64_t)blockIdx.x * Q8_WG_BLOCKS;
    const int64_t left = nblk - blk0;
    const int nb_here = left < Q8_WG_BLOCKS ? (int)left : Q8_WG_BLOCKS;

    float4 v[Q8_ITERS];
#pragma unroll
    for (int it = 0; it < Q8_ITERS; ++it) {
        const int b = it * 32 + sub;
        v[it] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (b < nb_here) {
            const float *p = x + (blk0 + b) * QK8_0 + part * 4;
            if (ALIGNED) {
                v[it] = *reinterpret_cast<const float4 *>(p);
            } else {
                v[it] = make_float4(p[0], p[1], p[2], p[3]);
            }
        }
    }
#pragma unroll
    for (int it = 0; it < Q8_ITERS; ++it) {
        const int b = it * 32 + sub;
        float amax = fmaxf(fmaxf(fabsf(v[it].x), fabsf(v[it].y)), fmaxf(fabsf(v[it].z), fabsf(v[it].w)));
        amax = fmaxf(amax, __shfl_xor(amax, 1));
        amax = fmaxf(amax, __shfl_xor(amax, 2));
        amax = fmaxf(amax, __shfl_xor(amax, 4));
        const float d = amax / 127.0f;                 // IEEE divide
        const float id = d != 0.0f ? 1.0f / d : 0.0f;  // from the unrounded f32 d
        const uint32_t q = pack4_i8(v[it].x * id, v[it].y * id, v[it].z * id, v[it].w * id);
        uint8_t *o = stage + b * Q8_0_BYTES;
        if (part == 0) *reinterpret_cast<uint16_t *>(o) = f32_to_f16_bits(d);
        uint16_t *oq = reinterpret_cast<uint16_t *>(o + 2 + part * 4);
        oq[0] = (uint16_t)(q & 0xFFFFu);
        oq[1] = (uint16_t)(q >> 16);
    }
    __syncthreads();

    const int nbytes = nb_here * Q8_0_BYTES;
    uint8_t *out = y + blk0 * Q8_0_BYTES;
    if (ALIGNED) {
        const int n16 = nbytes >> 4;
        const uint4 *s4 = reinterpret_cast<const uint4 *>(stage);
        uint4 *o4 = reinterpret_cast<uint4 *>(out);
        for (int i = tid; i < n16; i += CODEC_THREADS) o4[i] = s4[i];
        const int done = n16 << 4;
        const uint16_t *s2 = reinterpret_cast<const uint16_t *>(stage + done);
        uint16_t *o2 = reinterpret_cast<uint16_t *>(out + done);
        for (int i = tid; i < ((nbytes - done) >> 1); i += CODEC_THREADS) o2[i] = s2[i];
    } else {
        const uint16_t *s2 = reinterpret_cast<const uint16_t *>(stage);
        uint16_t *o2 = reinterpret_cast<uint16_t *>(out);
        for (int i = tid; i < (nbytes >> 1); i += CODEC_THREADS) o2[i] = s2[i];
    }
}

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
        for (int i = tid; i < n16; i += CODEC_THREADS) s4[i] = i4[i];
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
                *reinterpret_cast<float4 *>(p) = r;
            } else {
                p[0] = r.x; p[1] = r.y; p[2] = r.z; p[3] = r.w;
            }
        }
    }
}

// 8 elements per thread: two 16-byte loads, one 16-byte store
template <bool ALIGNED>
__global__ __launch_bounds__(CODEC_THREADS) void pack_f16_kernel(const float *__restrict__ x,
                                                                 uint16_t *__restrict__ y, int64_t n) {
    const int64_t i = ((int64_t)blockIdx.x * CODEC_THREADS + threadIdx.x) * 8;
    if (i >= n) return;
    if (ALIGNED && i + 8 <= n) {
        const float4 a = *reinterpret_cast<const float4 *>(x + i);
        const float4 b = *reinterpret_cast<const float4 *>(x + i + 4);
        uint4 o;
        o.x = (uint32_t)f32_to_f16_bits(a.x) | ((uint32_t)f32_to_f16_bits(a.y) << 16);
        o.y = (uint32_t)f32_to_f16_bits(a.z) | ((uint32_t)f32_to_f16_bits(a.w) << 16);
        o.z = (uint32_t)f32_to_f16_bits(b.x) | ((uint32_t)f32_to_f16_bits(b.y) << 16);
        o.w = (uint32_t)f32_to_f16_bits(b.z) | ((uint32_t)f32_to_f16_bits(b.w) << 16);
        *reinterpret_cast<uint4 *>(y + i) = o;
    } else {
        const int64_t e = i + 8 < n ? i + 8 : n;
        for (int64_t j = i; j < e; ++j) y[j] = f32_to_f16_bits(x[j]);
    }
}

template <bool ALIGNED>
__global__ __launch_bounds__(CODEC_THREADS) void unpack_f16_kernel(const uint16_t *__restrict__ x,
                                                                   float *__restrict__ y, int64_t n) {
    const int64_t i = ((int64_t)blockIdx.x * CODEC_THREADS + threadIdx.x) * 8;
    if (i >= n) return;
    if (ALIGNED && i + 8 <= n) {
        const uint4 v = *reinterpret_cast<const uint4 *>(x + i);
        float4 a, b;
        a.x = f16_bits_to_f32((uint16_t)(v.x & 0xFFFF)); a.y = f16_bits_to_f32((uint16_t)(v.x >> 16));
        a.z = f16_bits_to_f32((uint16_t)(v.y & 0xFFFF)); a.w = f16_bits_to_f32((uint16_t)(v.y >> 16));
        b.x = f16_bits_to_f32((uint16_t)(v.z & 0xFFFF)); b.y = f16_bits_to_f32((uint16_t)(v.z >> 16));
        b.z = f16_bits_to_f32((uint16_t)(v.w & 0xFFFF)); b.w = f16_bits_to_f32((uint16_t)(v.w >> 16));
        *reinterpret_cast<float4 *>(y + i) = a;
        *reinterpret_cast<float4 *>(y + i + 4) = b;
    } else {
        const int64_t e = i + 8 < n ? i + 8 : n;
        for (int64_t j = i; j < e; ++j) y[j] = f16_bits_to_f32(x[j]);
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
            if (al) pack_f16_kernel<true><<<dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream>>>(src, (uint16_t *)dst, n);
            else pack_f16_kernel<false><<<dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream>>>(src, (uint16_t *)dst, n);
            MESH_LAUNCH_CHECK();
            return MESH_OK;
        }
        case MESH_Q8_0: {
            if (n % QK8_0) return fail(MESH_ERR_INVALID, "mesh_act_pack: q8_0 needs a multiple of 32 elements, got %lld", (long long)n);
            const int64_t nblk = n / QK8_0;
            const int64_t grid = (nblk + Q8_WG_BLOCKS - 1) / Q8_WG_BLOCKS;
            if (al) pack_q8_0_kernel<true><<<dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream>>>(src, (uint8_t *)dst, nblk);
            else pack_q8_0_kernel<false><<<dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream>>>(src, (uint8_t *)dst, nblk);
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
            if (al) unpack_f16_kernel<true><<<dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream>>>((const uint16_t *)src, dst, n);
            else unpack_f16_kernel<false><<<dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream>>>((const uint16_t *)src, dst, n);
            MESH_LAUNCH_CHECK();
            return MESH_OK;
        }
        case MESH_Q8_0: {
            if (n % QK8_0) return fail(MESH_ERR_INVALID, "mesh_act_unpack: q8_0 needs a multiple of 32 elements, got %lld", (long long)n);
            const int64_t nblk = n / QK8_0;
            const int64_t grid = (nblk + Q8_WG_BLOCKS - 1) / Q8_WG_BLOCKS;
            if (al) unpack_q8_0_kernel<true><<<dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream>>>((const uint8_t *)src, dst, nblk);
            else unpack_q8_0_kernel<false><<<dim3((unsigned)grid), dim3(CODEC_THREADS), 0, stream>>>((const uint8_t *)src, dst, nblk);
            MESH_LAUNCH_CHECK();
            return MESH_OK;
        }
        default:
            return fail(MESH_ERR_INVALID, "mesh_act_unpack: format %d is not an activation format", fmt);
    }
}

}  // namespace mesh
