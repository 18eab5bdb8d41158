// KV cache rows in HBM.
//
// A row is the head_dim values of one (sequence, kv head, position).  Three row types, the KV tiers of
// KvCacheQuant::for_model_size (mesh-llm/src/inference/launch.rs:568-591: f16/f16 below 5 GB of model, q8_0 K with
// q4_0 V up to 50 GB, q4_0/q4_0 above):
//   MESH_F16   head_dim halfs
//   MESH_Q8_0  head_dim int8 quants, then head_dim/32 f16 scales          (ggml block_q8_0 values, regrouped)
//   MESH_Q4_0  head_dim/2 bytes of nibbles, then head_dim/32 f16 scales   (ggml block_q4_0 values, regrouped)
// Rows are quantised per 32 consecutive elements exactly as quantize_row_q8_0_ref / quantize_row_q4_0_ref do for
// a cache row; only the arrangement inside the row differs from ggml's array of blocks: quants and scales are
// kept apart so that a lane owning 8 consecutive dimensions fetches its quants with one aligned load, and q4_0
// nibbles are in element order (byte i = elements 2i and 2i+1, low nibble first).  Row sizes are rounded up to 8
// bytes.  The cache is private to the session; mesh_session_kv_read / _write convert to and from f16.
#pragma once

#include "mesh_common.hpp"

namespace mesh {

__host__ __device__ constexpr int kv_quant_bytes(int type, int hd) { return type == MESH_F16 ? hd * 2 : type == MESH_Q8_0 ? hd : hd / 2; }
__host__ __device__ constexpr int kv_row_bytes(int type, int hd) {
    return (kv_quant_bytes(type, hd) + (type == MESH_F16 ? 0 : hd / 32 * 2) + 7) & ~7;
}
inline bool kv_type_supported(int type) { return type == MESH_F16 || type == MESH_Q8_0 || type == MESH_Q4_0; }

#if defined(__HIPCC__)
// ---------------------------------------------------------------------------------------------- lane access
// What a lane holding dimensions [ds, ds + 8) of a row fetches, and its decoding to value = scale * (u - off).
template <int TYPE> struct KvRaw;
template <> struct KvRaw<MESH_F16> { uint4 v; };
template <> struct KvRaw<MESH_Q8_0> { uint2 v; uint16_t d; };
template <> struct KvRaw<MESH_Q4_0> { uint32_t v; uint16_t d; };

template <int TYPE> __device__ __forceinline__ void kv_zero(KvRaw<TYPE> &r);
template <> __device__ __forceinline__ void kv_zero<MESH_F16>(KvRaw<MESH_F16> &r) { r.v = make_uint4(0, 0, 0, 0); }
template <> __device__ __forceinline__ void kv_zero<MESH_Q8_0>(KvRaw<MESH_Q8_0> &r) { r.v = make_uint2(0x80808080u, 0x80808080u); r.d = 0; }
template <> __device__ __forceinline__ void kv_zero<MESH_Q4_0>(KvRaw<MESH_Q4_0> &r) { r.v = 0x88888888u; r.d = 0; }

template <int TYPE, int HD> __device__ __forceinline__ KvRaw<TYPE> kv_load(const uint8_t *row, int ds) {
    KvRaw<TYPE> r;
    if constexpr (TYPE == MESH_F16) {
        r.v = *reinterpret_cast<const uint4 *>(row + ds * 2);
    } else if constexpr (TYPE == MESH_Q8_0) {
        r.v = *reinterpret_cast<const uint2 *>(row + ds);
        r.d = *reinterpret_cast<const uint16_t *>(row + HD + (ds >> 5) * 2);
    } else {
        r.v = *reinterpret_cast<const uint32_t *>(row + (ds >> 1));
        r.d = *reinterpret_cast<const uint16_t *>(row + HD / 2 + (ds >> 5) * 2);
    }
    return r;
}

template <int TYPE> struct KvAffine { static constexpr float off = TYPE == MESH_Q8_0 ? 128.f : TYPE == MESH_Q4_0 ? 8.f : 0.f; };

// u[8] are small non-negative integers (quantised types; the stored quant plus `off`) or the values themselves (f16)
template <int TYPE> __device__ __forceinline__ float kv_decode(const KvRaw<TYPE> &r, float (&u)[8]) {
    if constexpr (TYPE == MESH_F16) {
        u[0] = f16_bits_to_f32((uint16_t)(r.v.x & 0xFFFF)); u[1] = f16_bits_to_f32((uint16_t)(r.v.x >> 16));
        u[2] = f16_bits_to_f32((uint16_t)(r.v.y & 0xFFFF)); u[3] = f16_bits_to_f32((uint16_t)(r.v.y >> 16));
        u[4] = f16_bits_to_f32((uint16_t)(r.v.z & 0xFFFF)); u[5] = f16_bits_to_f32((uint16_t)(r.v.z >> 16));
        u[6] = f16_bits_to_f32((uint16_t)(r.v.w & 0xFFFF)); u[7] = f16_bits_to_f32((uint16_t)(r.v.w >> 16));
        return 1.f;
    } else if constexpr (TYPE == MESH_Q8_0) {
        const uint32_t a = r.v.x ^ 0x80808080u, b = r.v.y ^ 0x80808080u;     // int8 -> biased uint8
        u[0] = (float)(a & 0xFF); u[1] = (float)((a >> 8) & 0xFF); u[2] = (float)((a >> 16) & 0xFF); u[3] = (float)(a >> 24);
        u[4] = (float)(b & 0xFF); u[5] = (float)((b >> 8) & 0xFF); u[6] = (float)((b >> 16) & 0xFF); u[7] = (float)(b >> 24);
        return f16_bits_to_f32(r.d);
    } else {
        const uint32_t lo = r.v & 0x0F0F0F0Fu, hi = (r.v >> 4) & 0x0F0F0F0Fu;  // even / odd elements
        u[0] = (float)(lo & 0xFF); u[1] = (float)(hi & 0xFF); u[2] = (float)((lo >> 8) & 0xFF); u[3] = (float)((hi >> 8) & 0xFF);
        u[4] = (float)((lo >> 16) & 0xFF); u[5] = (float)((hi >> 16) & 0xFF); u[6] = (float)(lo >> 24); u[7] = (float)(hi >> 24);
        return f16_bits_to_f32(r.d);
    }
}

// ---------------------------------------------------------------------------------------------- row store / fetch
// One wave writes the row whose f32 values are in LDS (or any memory the whole wave can read): the block maximum
// is a reduction over the 32 lanes of a block; q4_0 takes the FIRST element of largest magnitude, as the serial
// reference loop does.
__device__ __forceinline__ void kv_store_row(int type, uint8_t *row, const float *vec, int hd, int lane) {
    if (type == MESH_F16) {
        for (int i = lane; i < hd; i += 64) reinterpret_cast<uint16_t *>(row)[i] = f32_to_f16_bits(vec[i]);
        return;
    }
    uint16_t *scales = reinterpret_cast<uint16_t *>(row + kv_quant_bytes(type, hd));
    for (int i0 = 0; i0 < hd; i0 += 64) {
        const int i = i0 + lane;
        const bool live = i < hd;
        const float x = live ? vec[i] : 0.f;
        float am = fabsf(x), mv = x;
        int mi = i;
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) {
            const float a2 = __shfl_xor(am, o), v2 = __shfl_xor(mv, o);
            const int i2 = __shfl_xor(mi, o);
            const bool take = a2 > am || (a2 == am && i2 < mi);
            am = take ? a2 : am; mv = take ? v2 : mv; mi = take ? i2 : mi;
        }
        if (type == MESH_Q8_0) {
            const float d = am / 127.0f;
            const float id = d != 0.0f ? 1.0f / d : 0.0f;
            const int q = (int)roundf(x * id);
            if (live) row[i] = (uint8_t)(q & 0xFF);
            if (live && (lane & 31) == 0) scales[i >> 5] = f32_to_f16_bits(d);
        } else {
            const float d = mv / -8.0f;
            const float id = d != 0.0f ? 1.0f / d : 0.0f;
            int q = (int)(x * id + 8.5f);
            q = q > 15 ? 15 : q;
            const int qn = __shfl_xor(q, 1);
            if (live && !(lane & 1)) row[i >> 1] = (uint8_t)(q | (qn << 4));
            if (live && (lane & 31) == 0) scales[i >> 5] = f32_to_f16_bits(d);
        }
    }
}

// element i of a row as f32 (the value the attention kernels see)
__device__ __forceinline__ float kv_fetch(int type, const uint8_t *row, int hd, int i) {
    if (type == MESH_F16) return f16_bits_to_f32(reinterpret_cast<const uint16_t *>(row)[i]);
    const float d = f16_bits_to_f32(reinterpret_cast<const uint16_t *>(row + kv_quant_bytes(type, hd))[i >> 5]);
    if (type == MESH_Q8_0) return (float)(int8_t)row[i] * d;
    const int b = row[i >> 1];
    return (float)(((i & 1) ? (b >> 4) : (b & 0xF)) - 8) * d;
}
#endif

}  // namespace mesh
