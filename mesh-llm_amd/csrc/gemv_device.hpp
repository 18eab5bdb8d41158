// Device-side building blocks of the dequant-fused GEMV (gemv.hip): the 16-bit fixed-point activation staging in LDS,
// and the per-tile integer dot products for q4_K / q6_K tiles.  See gemv.hip for the design notes.
#pragma once

#include "gemv.hpp"

namespace mesh {

// Loads through a pointer known to be global memory.  A pointer read from a table in memory is "generic" to the
// compiler and costs flat_load instructions, which count on the LDS counter as well and so serialise with the
// LDS traffic of the dot products; the cast restores global_load.  (It goes through an integer: a direct
// pointer-to-pointer address-space cast is folded away again by the optimiser.)
#if defined(__HIP_DEVICE_COMPILE__)
#define MESH_GLOBAL __attribute__((address_space(1)))
#else
#define MESH_GLOBAL          // the host pass only parses device code
#endif
template <typename T>
__device__ __forceinline__ MESH_GLOBAL T *as_global(const void *p) {
    return (MESH_GLOBAL T *)(unsigned long long)p;
}
template <typename T>
__device__ __forceinline__ T ldg(const void *p) {
    return *as_global<const T>(p);
}

constexpr float XQ_LEVELS = 32512.0f;     // 127 * 256: |256*hi + lo| <= 32512 with hi, lo in int8

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

__device__ __forceinline__ uint32_t pack_bytes(int a, int b, int c, int d) {
    return (uint32_t)(a & 0xFF) | ((uint32_t)(b & 0xFF) << 8) | ((uint32_t)(c & 0xFF) << 16) | ((uint32_t)(d & 0xFF) << 24);
}

// LDS view of the quantised activations of NB columns
struct XStage {
    int8_t *xh, *xl;     // [NB][K]
    float *xd, *xs;      // [NB][K/32]: block scale d_b (without the norm scale), block sum of x = d_b * sum of quants
    int *xi16;           // [NB][K/16]: integer sum of quants per 16 elements (q6_K only)
    float *ssq;          // [16 waves][NB] partial sums of x^2 for the norm
    float *red;          // cross-wave partials [KS][rows][NU][16][NB]
};

// ------------------------------------------------------------------------------------------------ prologue
// Eight consecutive elements of each column per thread; 4 neighbouring lanes share a 32-element block.
template <int NB>
struct XRegs {
    float4 a[NB], b[NB];
    float4 w0, w1;           // the norm weights of the same eight elements (ones without a norm)
};

// Issued together with the activation loads, i.e. before the first weight-tile loads: loads return in order, so a
// norm-weight load issued after the tiles would make the prologue wait for the tiles as well.
template <int NB>
__device__ __forceinline__ void norm_fetch(XRegs<NB> &X, const float *__restrict__ norm_w, int g, bool live) {
    X.w0 = make_float4(1.f, 1.f, 1.f, 1.f);
    X.w1 = X.w0;
    if (norm_w && live) {
        X.w0 = ldg<float4>(norm_w + g * 8);
        X.w1 = ldg<float4>(norm_w + g * 8 + 4);
    }
}

template <int NB>
__device__ __forceinline__ void x_fetch(XRegs<NB> &X, const float *__restrict__ x, int ldx, int g, bool live) {
#pragma unroll
    for (int t = 0; t < NB; ++t) {
        X.a[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        X.b[t] = X.a[t];
        if (live) {
            X.a[t] = *reinterpret_cast<const float4 *>(x + (size_t)t * ldx + g * 8);
            X.b[t] = *reinterpret_cast<const float4 *>(x + (size_t)t * ldx + g * 8 + 4);
        }
    }
}

// the same with every column at its own offset (in elements) from x
template <int NB>
__device__ __forceinline__ void x_fetch_at(XRegs<NB> &X, const float *__restrict__ x, const size_t (&off)[NB], int g, bool live) {
#pragma unroll
    for (int t = 0; t < NB; ++t) {
        X.a[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        X.b[t] = X.a[t];
        if (live) {
            X.a[t] = *reinterpret_cast<const float4 *>(x + off[t] + g * 8);
            X.b[t] = *reinterpret_cast<const float4 *>(x + off[t] + g * 8 + 4);
        }
    }
}

template <int NB, bool NEED_I16>
__device__ __forceinline__ void x_quantise(const XRegs<NB> &X, int K, const XStage &S, int g, bool live, float (&ss)[NB]) {
    const int lane = threadIdx.x & 63;
    const float4 w0 = X.w0, w1 = X.w1;
#pragma unroll
    for (int t = 0; t < NB; ++t) {
        const float4 a0 = X.a[t], a1 = X.b[t];
        ss[t] += (a0.x * a0.x + a0.y * a0.y) + (a0.z * a0.z + a0.w * a0.w) + (a1.x * a1.x + a1.y * a1.y) + (a1.z * a1.z + a1.w * a1.w);
        const float v[8] = {a0.x * w0.x, a0.y * w0.y, a0.z * w0.z, a0.w * w0.w, a1.x * w1.x, a1.y * w1.y, a1.z * w1.z, a1.w * w1.w};
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
        amax = fmaxf(amax, __shfl_xor(amax, 1));
        amax = fmaxf(amax, __shfl_xor(amax, 2));
        const float inv = amax > 0.f ? XQ_LEVELS / amax : 0.f;
        int hi[8], lo[8], isum = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int q = __float2int_rn(v[i] * inv);
            lo[i] = ((q + 128) & 0xFF) - 128;
            hi[i] = (q - lo[i]) >> 8;
            isum += q;
        }
        isum += __shfl_xor(isum, 1);                 // sum over 16 elements
        const int isum32 = isum + __shfl_xor(isum, 2);
        if (live) {
            *reinterpret_cast<uint2 *>(S.xh + t * K + g * 8) = make_uint2(pack_bytes(hi[0], hi[1], hi[2], hi[3]), pack_bytes(hi[4], hi[5], hi[6], hi[7]));
            *reinterpret_cast<uint2 *>(S.xl + t * K + g * 8) = make_uint2(pack_bytes(lo[0], lo[1], lo[2], lo[3]), pack_bytes(lo[4], lo[5], lo[6], lo[7]));
            if (NEED_I16 && (lane & 1) == 0) S.xi16[t * (K >> 4) + (g >> 1)] = isum;
            if ((lane & 3) == 0) {
                const float d = amax / XQ_LEVELS;
                S.xd[t * (K >> 5) + (g >> 2)] = d;
                S.xs[t * (K >> 5) + (g >> 2)] = d * (float)isum32;
            }
        }
    }
}

// Producer side of the "xq" layout (gemv.hpp): called by 32 consecutive lanes (an aligned half of a wave, all active) that
// hold elements kk .. kk + 31 of a vector of K elements, one each (kk: this lane's element).  The same arithmetic as
// x_quantise on the same 32 values, hence the same bits.
__device__ __forceinline__ void xq_store_block32(uint8_t *xq, int K, int kk, float v) {
    float amax = fabsf(v);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    const float inv = amax > 0.f ? XQ_LEVELS / amax : 0.f;
    const int q = __float2int_rn(v * inv);
    const int lo = ((q + 128) & 0xFF) - 128, hi = (q - lo) >> 8;
    int isum = q;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) isum += __shfl_xor(isum, o);
    const int isum32 = isum + __shfl_xor(isum, 16);
    xq[kk] = (uint8_t)hi;
    xq[K + kk] = (uint8_t)lo;
    float *xd = reinterpret_cast<float *>(xq + 2 * (size_t)K), *xs = xd + (K >> 5);
    int *xi16 = reinterpret_cast<int *>(xs + (K >> 5));
    if ((kk & 15) == 0) xi16[kk >> 4] = isum;
    if ((kk & 31) == 0) {
        const float d = amax / XQ_LEVELS;
        xd[kk >> 5] = d;
        xs[kk >> 5] = d * (float)isum32;
    }
}

// ------------------------------------------------------------------------------------------------ tiles
template <int TYPE> struct TileRegs;

template <> struct TileRegs<MESH_Q4_K> {
    static constexpr int BYTES = Q4K_TILE_BYTES;
    uint4 hdr, qa, qb;
    __device__ __forceinline__ void load(const uint8_t *__restrict__ tile, int lane) {
        hdr = ldg<uint4>(tile + (lane >> 2) * 16);
        qa = ldg<uint4>(tile + 256 + lane * 32);
        qb = ldg<uint4>(tile + 256 + lane * 32 + 16);
    }
};

template <> struct TileRegs<MESH_Q6_K> {
    static constexpr int BYTES = Q6K_TILE_BYTES;
    uint4 qla, qlb, qh, sc;
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t *__restrict__ tile, int lane) {
        const int r = lane >> 2, c = lane & 3, n = c >> 1, u = c & 1;
        qla = ldg<uint4>(tile + r * 128 + 64 * n + 16 * u);
        qlb = ldg<uint4>(tile + r * 128 + 64 * n + 32 + 16 * u);
        qh = ldg<uint4>(tile + 2048 + r * 64 + 32 * n + 16 * u);
        sc = ldg<uint4>(tile + 3072 + r * 16);
        d = ldg<uint16_t>(tile + 3328 + r * 2);
    }
};

template <int NB>
__device__ __forceinline__ void tile_compute(const TileRegs<MESH_Q4_K> &R, int lane, int sb, const XStage &S, int K, float (&acc)[NB]) {
    const int c = lane & 3;
    const float d = f16_bits_to_f32((uint16_t)(R.hdr.x & 0xFFFFu));
    const float dmin = f16_bits_to_f32((uint16_t)(R.hdr.x >> 16));
    // 6-bit (scale, min) of sub-blocks 2c and 2c+1
    const uint32_t scw = c < 2 ? (R.hdr.y & 0x3F3F3F3Fu) : ((R.hdr.w & 0x0F0F0F0Fu) | ((R.hdr.y >> 2) & 0x30303030u));
    const uint32_t mnw = c < 2 ? (R.hdr.z & 0x3F3F3F3Fu) : (((R.hdr.w >> 4) & 0x0F0F0F0Fu) | ((R.hdr.z >> 2) & 0x30303030u));
    const int sh = (c & 1) * 16;
    const float dsa = d * (float)((scw >> sh) & 0xFFu), dsb = d * (float)((scw >> (sh + 8)) & 0xFFu);
    const float dma = dmin * (float)((mnw >> sh) & 0xFFu), dmb = dmin * (float)((mnw >> (sh + 8)) & 0xFFu);
    const uint32_t w[8] = {R.qa.x, R.qa.y, R.qa.z, R.qa.w, R.qb.x, R.qb.y, R.qb.z, R.qb.w};
    uint32_t lo[8], hi[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        lo[j] = w[j] & 0x0F0F0F0Fu;
        hi[j] = (w[j] >> 4) & 0x0F0F0F0Fu;
    }
    const int k0 = sb * QK_K + c * 64;
    const int b0 = k0 >> 5;
#pragma unroll
    for (int t = 0; t < NB; ++t) {
        const uint4 *ph = reinterpret_cast<const uint4 *>(S.xh + t * K + k0);
        const uint4 *pl = reinterpret_cast<const uint4 *>(S.xl + t * K + k0);
        const uint4 ha0 = ph[0], ha1 = ph[1], hb0 = ph[2], hb1 = ph[3];
        const uint4 la0 = pl[0], la1 = pl[1], lb0 = pl[2], lb1 = pl[3];
        const uint32_t xha[8] = {ha0.x, ha0.y, ha0.z, ha0.w, ha1.x, ha1.y, ha1.z, ha1.w};
        const uint32_t xhb[8] = {hb0.x, hb0.y, hb0.z, hb0.w, hb1.x, hb1.y, hb1.z, hb1.w};
        const uint32_t xla[8] = {la0.x, la0.y, la0.z, la0.w, la1.x, la1.y, la1.z, la1.w};
        const uint32_t xlb[8] = {lb0.x, lb0.y, lb0.z, lb0.w, lb1.x, lb1.y, lb1.z, lb1.w};
        int iha = 0, ila = 0, ihb = 0, ilb = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            iha = sdot4(lo[j], xha[j], iha);
            ila = sdot4(lo[j], xla[j], ila);
            ihb = sdot4(hi[j], xhb[j], ihb);
            ilb = sdot4(hi[j], xlb[j], ilb);
        }
        const float2 dx = *reinterpret_cast<const float2 *>(S.xd + t * (K >> 5) + b0);
        const float2 sx = *reinterpret_cast<const float2 *>(S.xs + t * (K >> 5) + b0);
        float r = acc[t];
        r = fmaf(dsa * dx.x, (float)((iha << 8) + ila), r);
        r = fmaf(dsb * dx.y, (float)((ihb << 8) + ilb), r);
        r = fmaf(-dma, sx.x, r);
        r = fmaf(-dmb, sx.y, r);
        acc[t] = r;
    }
}

template <int NB>
__device__ __forceinline__ void tile_compute(const TileRegs<MESH_Q6_K> &R, int lane, int sb, const XStage &S, int K, float (&acc)[NB]) {
    const int c = lane & 3, n = c >> 1, u = c & 1;
    const float d = f16_bits_to_f32((uint16_t)R.d);
    const uint32_t la[4] = {R.qla.x, R.qla.y, R.qla.z, R.qla.w}, lb[4] = {R.qlb.x, R.qlb.y, R.qlb.z, R.qlb.w};
    const uint32_t qh[4] = {R.qh.x, R.qh.y, R.qh.z, R.qh.w};
    // the 4 scale bytes of this lane: index 8n + 2*t4 + u  ->  word 2n + (t4 >> 1), byte 2*(t4 & 1) + u
    const uint32_t scw0 = n ? R.sc.z : R.sc.x, scw1 = n ? R.sc.w : R.sc.y;
    float dsc[4];
    dsc[0] = d * (float)(int8_t)((scw0 >> (8 * u)) & 0xFFu);
    dsc[1] = d * (float)(int8_t)((scw0 >> (16 + 8 * u)) & 0xFFu);
    dsc[2] = d * (float)(int8_t)((scw1 >> (8 * u)) & 0xFFu);
    dsc[3] = d * (float)(int8_t)((scw1 >> (16 + 8 * u)) & 0xFFu);
    uint32_t v[4][4];      // [t4][j]: 4 six-bit quants (0..63) per dword, elements 128n + 32*t4 + 16u + 4j + i
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        v[0][j] = (la[j] & 0x0F0F0F0Fu) | ((qh[j] << 4) & 0x30303030u);
        v[1][j] = (lb[j] & 0x0F0F0F0Fu) | ((qh[j] << 2) & 0x30303030u);
        v[2][j] = ((la[j] >> 4) & 0x0F0F0F0Fu) | (qh[j] & 0x30303030u);
        v[3][j] = ((lb[j] >> 4) & 0x0F0F0F0Fu) | ((qh[j] >> 2) & 0x30303030u);
    }
    const int k0 = sb * QK_K + 128 * n + 16 * u;
#pragma unroll
    for (int t = 0; t < NB; ++t) {
        float r = acc[t];
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
            const int k = k0 + 32 * t4;
            const uint4 xh = *reinterpret_cast<const uint4 *>(S.xh + t * K + k);
            const uint4 xl = *reinterpret_cast<const uint4 *>(S.xl + t * K + k);
            int ih = sdot4(v[t4][0], xh.x, 0), il = sdot4(v[t4][0], xl.x, 0);
            ih = sdot4(v[t4][1], xh.y, ih); il = sdot4(v[t4][1], xl.y, il);
            ih = sdot4(v[t4][2], xh.z, ih); il = sdot4(v[t4][2], xl.z, il);
            ih = sdot4(v[t4][3], xh.w, ih); il = sdot4(v[t4][3], xl.w, il);
            const int isum = S.xi16[t * (K >> 4) + (k >> 4)];
            const float dx = S.xd[t * (K >> 5) + (k >> 5)];
            r = fmaf(dsc[t4] * dx, (float)((ih << 8) + il - 32 * isum), r);
        }
        acc[t] = r;
    }
}

// Position of a wave in its flat list of tiles: local tile-row j (stride RS), matrix u of a fused pair, index ii
// along K (n_i tiles per segment).
template <int NU>
struct TileCursor {
    int j, u, ii;          // local tile-row, matrix within the pair, index along K
    __device__ __forceinline__ void advance(int n_i, int RS) {
        if (++ii == n_i) {
            ii = 0;
            if (++u == NU) { u = 0; j += RS; }
        }
    }
};

}  // namespace mesh
