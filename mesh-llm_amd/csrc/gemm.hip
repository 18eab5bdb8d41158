// Prefill GEMM: Y[T][M] = X[T][K] . W^T with W in tiled q4_K / q6_K blocks (gemv.hpp) and X in f16.
// The many-token counterpart of the decode GEMV -- what ggml_backend_graph_compute runs for mul_mat when a prompt is
// ingested (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451).
//
// Design (gfx950): a 256-thread workgroup owns a 128 (weight rows) x 128 (tokens) output tile and walks K in
// steps of 64.  Per step the 128 x 64 weight slab is dequantised from its K-quant blocks straight into LDS as
// f16 (each thread: one row, one 32-element sub-block), the 128 x 64 activation slab is copied next to it, and
// the four waves (2 x 2, 64 x 64 each) issue v_mfma_f32_32x32x16_f16 on 16-byte LDS fragments with f32
// accumulation.  Weights cross HBM once per 128 tokens; dequantisation is amortised over 128 columns.  The two
// LDS stages alternate: the raw bytes of step k+1 are fetched into registers before the MFMAs of step k and
// dequantised after them, so global-memory latency and the dequant VALU work overlap the matrix cores (two
// workgroups fit a CU).
//
// MFMA operand layout used below (checked on hardware): A lane l = row l%32, k = 8*(l/32)+j; B lane l = column
// l%32, same k; accumulator register i of lane l = D[8*(i/4) + 4*(l/32) + i%4][l%32].

#include "gemm.hpp"

#include <algorithm>
#include <type_traits>

namespace mesh {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int GM = 128, GN = 128, GK = 64;     // workgroup tile: weight rows x tokens x k-step
constexpr int LDS_LD = GK + 8;                 // f16 elements per LDS row (16-byte pad against bank conflicts)
constexpr int GEMM_THREADS = 512;              // 4 matrix-core waves + 4 staging waves

// f32 pair -> packed f16, saturating: a magnitude beyond the f16 range becomes +-65504 instead of an infinity that the
// next layer's norm would turn into NaN for the whole token.
__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    a = __builtin_amdgcn_fmed3f(a, -65504.f, 65504.f);
    b = __builtin_amdgcn_fmed3f(b, -65504.f, 65504.f);
    return (uint32_t)__half_as_ushort(__float2half_rn(a)) | ((uint32_t)__half_as_ushort(__float2half_rn(b)) << 16);
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// four bytes (values < 64) -> four f16 holding ((value - off) * sc) * d + c, as two packed dwords.  0x6400 | q is the f16
// 1024 + q exactly and the offset comes off exactly; sc is the block's integer scale, so (q - off) * sc is an exact
// small integer (|.| <= 504 for q4_K with off = 1024 + 8; q6_K's reaches 4064, where integers above 2048 round to even);
// d is the super-block's f16 scale as stored in the file.  One packed fma then makes the weight with a single
// rounding: products of ROUNDED per-block scales (f16(d * sc), f16(dmin * m)) carry their rounding error into every
// weight of the block, three times the error of this form on q4_K.
__device__ __forceinline__ void dequant4(uint32_t q, half2v off, half2v sc, half2v d, half2v c, uint32_t &lo, uint32_t &hi) {
    const half2v a = (__builtin_bit_cast(half2v, __builtin_amdgcn_perm(0x64646464u, q, 0x04010400u)) - off) * sc;
    const half2v b = (__builtin_bit_cast(half2v, __builtin_amdgcn_perm(0x64646464u, q, 0x04030402u)) - off) * sc;
    lo = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(a, d, c));
    hi = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(b, d, c));
}
// q4_K: w = d sc (q - 8) + c with c = 8 d sc - dmin m (f32, rounded to f16 once).  {sc, c} of a sub-block:
__device__ __forceinline__ half2v q4k_sc_c(float d, float dmin, uint32_t scb, uint32_t mnb) {
    const float sc = (float)scb;
    return half2v{(_Float16)sc, (_Float16)(8.0f * d * sc - dmin * (float)mnb)};
}
__device__ __forceinline__ half2v h2_splat(float v) {
    const _Float16 h = (_Float16)v;
    return half2v{h, h};
}

// Raw bytes of one (row, 32-element sub-block) of a tile: what a staging thread prefetches one k-step ahead.
template <int TYPE> struct RawSub;

// q4_K: row r of the tile, k-chunk c (64 elements) of the super-block, half h (sub-block 2c + h)
template <> struct RawSub<MESH_Q4_K> {
    uint4 hdr, qa, qb;
    __device__ __forceinline__ void load(const uint8_t *__restrict__ tile, int r, int c, int) {
        hdr = *reinterpret_cast<const uint4 *>(tile + r * 16);
        qa = *reinterpret_cast<const uint4 *>(tile + 256 + r * 128 + c * 32);
        qb = *reinterpret_cast<const uint4 *>(tile + 256 + r * 128 + c * 32 + 16);
    }
    __device__ __forceinline__ void store(int c, int h, _Float16 *dst) const {
        const float d = f16_bits_to_f32((uint16_t)(hdr.x & 0xFFFFu)), dmin = f16_bits_to_f32((uint16_t)(hdr.x >> 16));
        const uint32_t scw = c < 2 ? (hdr.y & 0x3F3F3F3Fu) : ((hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u));
        const uint32_t mnw = c < 2 ? (hdr.z & 0x3F3F3F3Fu) : (((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u));
        const int sh = (c & 1) * 16 + h * 8;
        const half2v sc_c = q4k_sc_c(d, dmin, (scw >> sh) & 0xFFu, (mnw >> sh) & 0xFFu);
        const half2v sc = {sc_c[0], sc_c[0]}, cc = {sc_c[1], sc_c[1]}, dd = h2_splat(d);
        const half2v off = {(_Float16)1032.f, (_Float16)1032.f};
        const uint32_t w[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        uint4 *d4 = reinterpret_cast<uint4 *>(dst);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint4 o;
            dequant4((w[2 * i] >> (4 * h)) & 0x0F0F0F0Fu, off, sc, dd, cc, o.x, o.y);
            dequant4((w[2 * i + 1] >> (4 * h)) & 0x0F0F0F0Fu, off, sc, dd, cc, o.z, o.w);
            d4[i] = o;
        }
    }
    // this thread's part of a GEMM-layout chunk (gemm.hpp); s = 2 * row + h
    __device__ __forceinline__ void pack(int c, int h, uint8_t *chunk, int s) const {
        const float d = f16_bits_to_f32((uint16_t)(hdr.x & 0xFFFFu)), dmin = f16_bits_to_f32((uint16_t)(hdr.x >> 16));
        const uint32_t scw = c < 2 ? (hdr.y & 0x3F3F3F3Fu) : ((hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u));
        const uint32_t mnw = c < 2 ? (hdr.z & 0x3F3F3F3Fu) : (((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u));
        const int sh = (c & 1) * 16 + h * 8;
        const half2v sc_c = q4k_sc_c(d, dmin, (scw >> sh) & 0xFFu, (mnw >> sh) & 0xFFu);
        const uint32_t w[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        uint32_t n[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) n[j] = ((w[2 * j] >> (4 * h)) & 0x0F0F0F0Fu) | (((w[2 * j + 1] >> (4 * h)) & 0x0F0F0F0Fu) << 4);
        *reinterpret_cast<uint4 *>(chunk + s * 16) = make_uint4(n[0], n[1], n[2], n[3]);
        *reinterpret_cast<uint2 *>(chunk + 4096 + s * 8) = make_uint2(__builtin_bit_cast(uint32_t, sc_c), hdr.x & 0xFFFFu);
    }
};

// q6_K: row r, k-chunk c: half n = c/2, elements 128n + 32*t4 + l with t4 = 2*(c%2) + h, l = 0..31
template <> struct RawSub<MESH_Q6_K> {
    uint4 la, lb, ha, hb;
    uint32_t sc, d;
    __device__ __forceinline__ void load(const uint8_t *__restrict__ tile, int r, int c, int h) {
        const int n = c >> 1, t4 = 2 * (c & 1) + h;
        const uint8_t *ql = tile + r * 128 + 64 * n + 32 * (t4 & 1);
        const uint8_t *qh = tile + 2048 + r * 64 + 32 * n;
        la = *reinterpret_cast<const uint4 *>(ql); lb = *reinterpret_cast<const uint4 *>(ql + 16);
        ha = *reinterpret_cast<const uint4 *>(qh); hb = *reinterpret_cast<const uint4 *>(qh + 16);
        sc = *reinterpret_cast<const uint16_t *>(tile + 3072 + r * 16 + 8 * n + 2 * t4);
        d = *reinterpret_cast<const uint16_t *>(tile + 3328 + r * 2);
    }
    __device__ __forceinline__ void store(int c, int h, _Float16 *dst) const {
        const int t4 = 2 * (c & 1) + h;
        const half2v dd = h2_splat(f16_bits_to_f32((uint16_t)d));
        const half2v s0 = h2_splat((float)(int8_t)(sc & 0xFFu)), s1 = h2_splat((float)(int8_t)(sc >> 8));
        const half2v off = {(_Float16)1056.f, (_Float16)1056.f}, zero = {(_Float16)0.f, (_Float16)0.f};
        const uint32_t lw[8] = {la.x, la.y, la.z, la.w, lb.x, lb.y, lb.z, lb.w};
        const uint32_t hw[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
        uint4 *d4 = reinterpret_cast<uint4 *>(dst);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t q[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int j = 2 * i + e;
                const uint32_t nib = (t4 & 2) ? (lw[j] >> 4) & 0x0F0F0F0Fu : lw[j] & 0x0F0F0F0Fu;
                q[e] = nib | (((hw[j] >> (2 * t4)) & 0x03030303u) << 4);
            }
            const half2v s = i < 2 ? s0 : s1;       // one scale per 16 elements
            uint4 o;
            dequant4(q[0], off, s, dd, zero, o.x, o.y);
            dequant4(q[1], off, s, dd, zero, o.z, o.w);
            d4[i] = o;
        }
    }
    __device__ __forceinline__ void pack(int c, int h, uint8_t *chunk, int s) const {
        const int t4 = 2 * (c & 1) + h;
        const half2v s01 = {(_Float16)(float)(int8_t)(sc & 0xFFu), (_Float16)(float)(int8_t)(sc >> 8)};
        const uint32_t lw[8] = {la.x, la.y, la.z, la.w, lb.x, lb.y, lb.z, lb.w};
        const uint32_t hw[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
        uint32_t q[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t nib = (t4 & 2) ? (lw[j] >> 4) & 0x0F0F0F0Fu : lw[j] & 0x0F0F0F0Fu;
            q[j] = nib | (((hw[j] >> (2 * t4)) & 0x03030303u) << 4);
        }
        uint32_t n[4], hb2[2] = {0u, 0u};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            n[j] = (q[2 * j] & 0x0F0F0F0Fu) | ((q[2 * j + 1] & 0x0F0F0F0Fu) << 4);
            hb2[j >> 1] |= (((q[2 * j] >> 4) & 0x03030303u) | (((q[2 * j + 1] >> 4) & 0x03030303u) << 2)) << (4 * (j & 1));
        }
        *reinterpret_cast<uint4 *>(chunk + s * 16) = make_uint4(n[0], n[1], n[2], n[3]);
        *reinterpret_cast<uint2 *>(chunk + 4096 + s * 8) = make_uint2(hb2[0], hb2[1]);
        *reinterpret_cast<uint2 *>(chunk + 6144 + s * 8) = make_uint2(__builtin_bit_cast(uint32_t, s01), d & 0xFFFFu);
    }
};

// The same (row, sub-block) out of the GEMM layout: two or three loads at the thread's own slot of the chunk.
template <int TYPE> struct PackedSub;
template <> struct PackedSub<MESH_Q4_K> {
    static constexpr int CHUNK = 6144;
    uint4 q;
    uint2 sm;          // {f16 sc, f16 c}, {f16 d, -}
    __device__ __forceinline__ void load(const uint8_t *__restrict__ chunk, int s) {
        q = *reinterpret_cast<const uint4 *>(chunk + s * 16);
        sm = *reinterpret_cast<const uint2 *>(chunk + 4096 + s * 8);
    }
    __device__ __forceinline__ void store(_Float16 *dst) const {
        const half2v sc = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(sm.x, sm.x, 0x01000100u));
        const half2v cc = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(sm.x, sm.x, 0x03020302u));
        const half2v dd = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(sm.y, sm.y, 0x01000100u));
        const half2v off = {(_Float16)1032.f, (_Float16)1032.f};
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        uint4 *d4 = reinterpret_cast<uint4 *>(dst);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint4 o;
            dequant4(w[j] & 0x0F0F0F0Fu, off, sc, dd, cc, o.x, o.y);
            dequant4((w[j] >> 4) & 0x0F0F0F0Fu, off, sc, dd, cc, o.z, o.w);
            d4[j] = o;
        }
    }
};
template <> struct PackedSub<MESH_Q6_K> {
    static constexpr int CHUNK = 8192;
    uint4 q;
    uint2 hb;
    uint2 sc;          // {f16 sc of elements 0..15, f16 sc of elements 16..31}, {f16 d, -}
    __device__ __forceinline__ void load(const uint8_t *__restrict__ chunk, int s) {
        q = *reinterpret_cast<const uint4 *>(chunk + s * 16);
        hb = *reinterpret_cast<const uint2 *>(chunk + 4096 + s * 8);
        sc = *reinterpret_cast<const uint2 *>(chunk + 6144 + s * 8);
    }
    __device__ __forceinline__ void store(_Float16 *dst) const {
        const half2v s0 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(sc.x, sc.x, 0x01000100u));
        const half2v s1 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(sc.x, sc.x, 0x03020302u));
        const half2v dd = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(sc.y, sc.y, 0x01000100u));
        const half2v off = {(_Float16)1056.f, (_Float16)1056.f}, zero = {(_Float16)0.f, (_Float16)0.f};
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        uint4 *d4 = reinterpret_cast<uint4 *>(dst);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t hs = (j < 2 ? hb.x : hb.y) >> (4 * (j & 1));
            const half2v s = j < 2 ? s0 : s1;
            uint4 o;
            dequant4((w[j] & 0x0F0F0F0Fu) | ((hs & 0x03030303u) << 4), off, s, dd, zero, o.x, o.y);
            dequant4(((w[j] >> 4) & 0x0F0F0F0Fu) | (((hs >> 2) & 0x03030303u) << 4), off, s, dd, zero, o.z, o.w);
            d4[j] = o;
        }
    }
};

// Role split: waves 0-3 only multiply (each a 64 x 64 corner of the tile out of LDS stage kc & 1), waves 4-7 only
// stage (fetch the raw weight bytes and activations of step kc + 2, dequantise step kc + 1 into the other LDS
// stage).  A SIMD then holds one wave of each kind per workgroup, and the dequantisation (vector ALU) of one runs
// while the MFMAs (matrix core) of the other execute -- in one wave doing both, the ~110 dequant instructions of
// a step only start once its 16 MFMAs have been issued, and the four waves move in lockstep between barriers.
// PACKED: the weights come from the GEMM layout (a.Wp) instead of the mat-vec tiles (a.W).
// XDIRECT: the activations are k8-major (gemm.hpp) and never enter LDS: a matrix-core wave's B fragment of 32 tokens x
// 16 k is four contiguous 256-byte pieces of that layout, so each lane fetches its 16 bytes straight from memory (L2),
// four k16 steps ahead, into a ring of registers.  That halves the LDS reads per MFMA and leaves the staging waves only
// the weights.
// GROUPED: an expert launch (gemm.hpp): the workgroup's token tile and matrix come from a.tiles[blockIdx.y].
template <int TYPE, bool PACKED, bool XDIRECT, bool SPLIT, bool NARROW, bool GROUPED = false>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_kq_kernel(GemmArgs a) {
    static_assert(!GROUPED || (PACKED && XDIRECT && !SPLIT && !NARROW), "expert launches: GEMM layout, k8-major activations, one k range");
    extern __shared__ __align__(16) _Float16 gemm_smem[];
    _Float16 *Ws = gemm_smem;                                  // [2][GM][LDS_LD]
    _Float16 *Xs = gemm_smem + 2 * GM * LDS_LD;                // [2][GN][LDS_LD]
    constexpr int TB = TYPE == MESH_Q4_K ? Q4K_TILE_BYTES : Q6K_TILE_BYTES;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // token tile [t0, t_end) of this workgroup and its matrix
    int t0 = blockIdx.y * GN, t_end = a.T;
    const uint8_t *Wp = static_cast<const uint8_t *>(a.Wp);
    if constexpr (GROUPED) {
        if ((int)blockIdx.y >= *a.n_tiles) return;
        const int4 tl = reinterpret_cast<const int4 *>(a.tiles)[blockIdx.y];
        Wp += (size_t)tl.x * a.expert_stride;
        t0 = tl.y;
        t_end = tl.y + tl.z;
    }
    const int m0 = blockIdx.x * GM;
    const int nsb = a.K / QK_K, n_all = a.K / GK;
    // k-steps [k0, k0 + n_steps) of this workgroup: all of them, or slice blockIdx.z of a split launch
    // (a template parameter: the unsplit kernel must not carry the offsets, they cost it 6%)
    const int k0 = SPLIT ? (int)blockIdx.z * a.k_per_split : 0;
    const int n_steps = SPLIT ? (n_all - k0 < a.k_per_split ? n_all - k0 : a.k_per_split) : n_all;

    if (wave >= 4) {
        // ---- staging waves: thread s (0..255): weights -- row s/2, sub-block half s%2; activations -- token s/2, 32 elements s%2
        const int st = tid - 256;
        const int srow = st >> 1, sh = st & 1;
        const int wrow = m0 + srow;                                  // rows beyond M are zero tiles (M padded to 16)
        const bool wlive = PACKED || wrow < a.M_pad;                 // (the GEMM layout holds its zero rows)
        const uint8_t *wtile_row = PACKED ? Wp + ((size_t)blockIdx.x * n_all + k0) * PackedSub<TYPE>::CHUNK
                                          : static_cast<const uint8_t *>(a.W) + (size_t)((wlive ? wrow : 0) >> 4) * nsb * TB;
        using Sub = typename std::conditional<PACKED, PackedSub<TYPE>, RawSub<TYPE>>::type;
        const int tok = t0 + srow;
        const bool xlive = tok < a.T;
        const _Float16 *xrow = XDIRECT ? a.X : a.X + (size_t)(xlive ? tok : 0) * a.ldx + 32 * sh;
        Sub rw[2];
        uint4 rx[2][4];
        auto fetch = [&](int kc, Sub &w, uint4 (&x)[4]) {
            if constexpr (PACKED) w.load(wtile_row + (size_t)kc * PackedSub<TYPE>::CHUNK, st);
            else w.load(wtile_row + (size_t)((k0 + kc) >> 2) * TB, wrow & 15, (k0 + kc) & 3, sh);
            if constexpr (!XDIRECT) {
                const uint4 *s4 = reinterpret_cast<const uint4 *>(xrow + (size_t)(k0 + kc) * GK);
#pragma unroll
                for (int i = 0; i < 4; ++i) x[i] = s4[i];
            }
        };
        auto stage = [&](int kc, int buf, const Sub &w, const uint4 (&x)[4]) {
            _Float16 *wdst = Ws + (buf * GM + srow) * LDS_LD + 32 * sh;
            if constexpr (PACKED) {
                w.store(wdst);
            } else if (wlive) {
                w.store((k0 + kc) & 3, sh, wdst);
            } else {
                uint4 *d4 = reinterpret_cast<uint4 *>(wdst);
#pragma unroll
                for (int i = 0; i < 4; ++i) d4[i] = make_uint4(0, 0, 0, 0);
            }
            if constexpr (!XDIRECT) {
                uint4 *x4 = reinterpret_cast<uint4 *>(Xs + (buf * GN + srow) * LDS_LD + 32 * sh);
#pragma unroll
                for (int i = 0; i < 4; ++i) x4[i] = xlive ? x[i] : make_uint4(0, 0, 0, 0);
            }
        };
        fetch(0, rw[0], rx[0]);
        fetch(n_steps > 1 ? 1 : 0, rw[1], rx[1]);
        stage(0, 0, rw[0], rx[0]);
        __syncthreads();
        // step kc (its slot parity = kc & 1): the slot of step kc was staged already -> refill it with step kc + 2;
        // then dequantise step kc + 1 (the other slot) into the LDS stage the multiplying waves are not reading
        for (int kc0 = 0; kc0 < n_steps; kc0 += 2) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int kc = kc0 + u;
                if (kc >= n_steps) break;
                fetch(kc + 2 < n_steps ? kc + 2 : n_steps - 1, rw[u], rx[u]);
                if (kc + 1 < n_steps) stage(kc + 1, u ^ 1, rw[u ^ 1], rx[u ^ 1]);
                __syncthreads();
            }
        }
        return;
    }

    // ---- multiplying waves
    // wave's corner of the tile: 64 rows x 64 tokens; NARROW (calls of at most 64 tokens, whose upper token half would
    // be padding): 32 rows x the lower 64 tokens, so all four waves multiply real columns
    static_assert(!NARROW || XDIRECT, "the narrow tile reads its activations from the k8-major layout");
    constexpr int MI = NARROW ? 1 : 2;
    const int wm = NARROW ? wave * 32 : (wave & 1) * 64, wn = NARROW ? 0 : (wave >> 1) * 64;
    float16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    if constexpr (XDIRECT) {
        // lane's slot in the fragments of its two 32-token groups: token (lane & 31), k8 group (lane >> 5) of a k16 step;
        // consecutive k16 steps are 256 halfs apart.  Token blocks past the batch re-read the last one (never stored).
        const int n_blk = (a.T + 15) >> 4, n_g = n_all * (GK / 16), g0 = k0 * (GK / 16);
        const _Float16 *bp[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int tok = t0 + wn + 32 * i + (lane & 31);
            const int blk = (tok >> 4) < n_blk ? (tok >> 4) : n_blk - 1;
            bp[i] = a.X + (size_t)blk * 16 * a.K + ((lane >> 5) * 16 + (tok & 15)) * 8;
        }
        half8 ring[GK / 16][2];
#pragma unroll
        for (int ks = 0; ks < GK / 16; ++ks)
#pragma unroll
            for (int i = 0; i < 2; ++i) ring[ks][i] = *reinterpret_cast<const half8 *>(bp[i] + (size_t)(g0 + ks < n_g ? g0 + ks : n_g - 1) * 256);
        __syncthreads();
        for (int kc = 0; kc < n_steps; ++kc) {
            const _Float16 *Wb = Ws + (kc & 1) * GM * LDS_LD;
#pragma unroll
            for (int ks = 0; ks < GK / 16; ++ks) {
                half8 af[MI];
#pragma unroll
                for (int i = 0; i < MI; ++i)
                    af[i] = *reinterpret_cast<const half8 *>(Wb + (wm + 32 * i + (lane & 31)) * LDS_LD + 16 * ks + 8 * (lane >> 5));
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], ring[ks][j], acc[i][j], 0, 0, 0);
                int gn = g0 + (kc + 1) * (GK / 16) + ks;
                gn = gn < n_g ? gn : n_g - 1;
#pragma unroll
                for (int i = 0; i < 2; ++i) ring[ks][i] = *reinterpret_cast<const half8 *>(bp[i] + (size_t)gn * 256);
                // keep each refill where it is written: left to itself the scheduler sinks all eight loads to the end
                // of the step, where the next step's first MFMA waits for them at full memory latency
                __builtin_amdgcn_sched_barrier(0);
            }
            __syncthreads();
        }
    } else if constexpr (!NARROW) {
    __syncthreads();
    for (int kc = 0; kc < n_steps; ++kc) {
        const int buf = kc & 1;
        const _Float16 *Wb = Ws + buf * GM * LDS_LD, *Xb = Xs + buf * GN * LDS_LD;
#pragma unroll
        for (int ks = 0; ks < GK / 16; ++ks) {
            half8 af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = *reinterpret_cast<const half8 *>(Wb + (wm + 32 * i + (lane & 31)) * LDS_LD + 16 * ks + 8 * (lane >> 5));
                bf[i] = *reinterpret_cast<const half8 *>(Xb + (wn + 32 * i + (lane & 31)) * LDS_LD + 16 * ks + 8 * (lane >> 5));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    }

    // D[m][t]: lane holds column t = lane%32 and rows 8*(e/4) + 4*(lane/32) + e%4 -> four consecutive m per store
    if constexpr (SPLIT) {
        // slice of a split launch: the raw sums go to part[slice][token][row of the launch]
        const size_t ld = (size_t)gridDim.x * GM;
        float *P = a.part + (size_t)blockIdx.z * a.T * ld + m0;
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int t = t0 + wn + 32 * j + (lane & 31);
                if (t >= a.T) continue;
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4)
                    *reinterpret_cast<float4 *>(P + (size_t)t * ld + wm + 32 * i + 8 * e4 + 4 * (lane >> 5)) =
                        make_float4(acc[i][j][4 * e4], acc[i][j][4 * e4 + 1], acc[i][j][4 * e4 + 2], acc[i][j][4 * e4 + 3]);
            }
        return;
    }
    if (a.y16_k8) {
        // SwiGLU pair: the waves of the upper half of the tile hold the up rows of the gate rows in the lower half, at
        // the same (register, lane).  They hand them over through LDS (free by now: the staging waves have left, and
        // the barrier makes sure every matrix-core wave has read its last fragments).
        // (NARROW: waves 2 and 3 hold the up rows of the gate rows of waves 0 and 1)
        float *xch = reinterpret_cast<float *>(gemm_smem);         // [pair of waves][64 registers][64 lanes]
        const bool is_up = NARROW ? wave >= 2 : wm != 0;
        const int pair = NARROW ? (wave & 1) * 2 : (wn >> 6) * 4;  // first 16-register group of this pair of waves
        const int gm = NARROW ? (wave & 1) * 32 : 0;               // gate rows of this wave inside the block's 64
        __syncthreads();
        if (is_up) {
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) xch[((pair + i * 2 + j) * 16 + e) * 64 + lane] = acc[i][j][e];
        }
        __syncthreads();
        if (is_up) return;
        const int t_pad = (t_end + 15) & ~15;
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int t = t0 + wn + 32 * j + (lane & 31);
                if (t >= t_pad) continue;
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    const int m = (int)blockIdx.x * (GM / 2) + gm + 32 * i + 8 * e4 + 4 * (lane >> 5);
                    if (m >= a.M) continue;
                    float o[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float g = acc[i][j][4 * e4 + c], u = xch[((pair + i * 2 + j) * 16 + 4 * e4 + c) * 64 + lane];
                        o[c] = t < t_end ? g / (1.0f + expf(-g)) * u : 0.f;       // padding columns of the last token block hold zeros
                    }
                    note_f16_clamp(a.sat, o[0], o[1], o[2], o[3]);
                    *reinterpret_cast<uint2 *>(a.y16_k8 + (size_t)(t >> 4) * 16 * a.M + ((size_t)(m >> 3) * 16 + (t & 15)) * 8 + (m & 7)) =
                        make_uint2(pack_h2(o[0], o[1]), pack_h2(o[2], o[3]));
                }
            }
        return;
    }
    float *Y = a.Y;
    const float *bias = a.bias;
    int M = a.M, ldy = a.ldy, mb0 = m0;
    if (a.n_seg > 1) {
        // (selected, not indexed: a dynamically indexed kernel-argument array would be spilled to scratch)
        const int bx = blockIdx.x;
        const int sg = (bx >= a.seg_begin[1] ? 1 : 0) + (a.n_seg > 2 && bx >= a.seg_begin[2] ? 1 : 0);
        Y = sg == 0 ? a.seg_Y[0] : sg == 1 ? a.seg_Y[1] : a.seg_Y[2];
        bias = sg == 0 ? a.seg_bias[0] : sg == 1 ? a.seg_bias[1] : a.seg_bias[2];
        M = sg == 0 ? a.seg_M[0] : sg == 1 ? a.seg_M[1] : a.seg_M[2];
        ldy = sg == 0 ? a.seg_ldy[0] : sg == 1 ? a.seg_ldy[1] : a.seg_ldy[2];
        mb0 = (bx - (sg == 0 ? 0 : sg == 1 ? a.seg_begin[1] : a.seg_begin[2])) * GM;
    }
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int t = t0 + wn + 32 * j + (lane & 31);
            if (t >= t_end) continue;
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int m = mb0 + wm + 32 * i + 8 * e4 + 4 * (lane >> 5);
                if (m >= M) continue;      // M is a multiple of 4 for every projection
                float4 o = make_float4(acc[i][j][4 * e4], acc[i][j][4 * e4 + 1], acc[i][j][4 * e4 + 2], acc[i][j][4 * e4 + 3]);
                if (bias) {
                    const float4 b = *reinterpret_cast<const float4 *>(bias + m);
                    o.x += b.x; o.y += b.y; o.z += b.z; o.w += b.w;
                }
                if (a.residual) {
                    const float4 r = *reinterpret_cast<const float4 *>(a.residual + (size_t)t * a.ldres + m);
                    o.x += r.x; o.y += r.y; o.z += r.z; o.w += r.w;
                }
                *reinterpret_cast<float4 *>(Y + (size_t)t * ldy + m) = o;
            }
        }
}

// ---- the same product on a 256 x 128 workgroup tile ----------------------------------------------------------
// What bounds the 128 x 128 kernel above is operand traffic, not the matrix cores: a wave that owns 64 x 64 of the tile
// needs 1 KB of fragments per v_mfma_f32_32x32x16_f16 (2 x 2 register blocking: two weight fragments from LDS and two
// activation fragments from memory per four MFMAs), and four SIMDs at one MFMA per 32 cycles then ask the vector memory
// path for its whole 64 B per cycle and LDS for three quarters of its 128.  Here a matrix-core wave owns 128 weight rows x
// 64 tokens (4 x 2 blocking, 128 accumulator registers): 0.5 KB of weight fragments and 0.25 KB of activation fragments
// per MFMA, half of either path.  The price is one workgroup per CU and one matrix-core wave per SIMD, which therefore
// fetches the weight fragments of the next k16 step before it multiplies the current one; a staging wave shares the
// SIMD and dequantises while the MFMAs execute.
// Production layout only (GEMM-layout weights, k8-major activations), K not split, an even number of 128-row blocks:
// a workgroup takes row blocks 2 * blockIdx.x and + 1, one per pair of matrix-core waves, so everything that depends on
// the row block (matrix of a multi-matrix launch, SwiGLU pairing) is per wave.
constexpr int BGM = 256;
// Workgroup barrier that orders LDS only.  __syncthreads() also waits for every outstanding global load, i.e. at the end
// of each k-step for the activation fragments requested a moment ago for the NEXT step -- with one matrix-core wave per
// SIMD nothing else would run during that wait.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
template <int TYPE>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_big_kernel(GemmArgs a) {
    extern __shared__ __align__(16) _Float16 gemm_smem[];
    _Float16 *Ws = gemm_smem;                                  // [2][BGM][LDS_LD]
    using Sub = PackedSub<TYPE>;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t0 = blockIdx.y * GN;
    const int n_steps = a.K / GK;

    if (wave >= 4) {
        // ---- staging waves: thread s: (row s / 2, sub-block half s % 2) of both row blocks
        const int st = tid - 256;
        const uint8_t *chunk0 = static_cast<const uint8_t *>(a.Wp) + (size_t)(2 * blockIdx.x) * n_steps * Sub::CHUNK;
        const uint8_t *chunk1 = chunk0 + (size_t)n_steps * Sub::CHUNK;
        _Float16 *dst = Ws + (st >> 1) * LDS_LD + 32 * (st & 1);
        Sub rw[2][2];
        auto fetch = [&](int kc, Sub (&w)[2]) {
            w[0].load(chunk0 + (size_t)kc * Sub::CHUNK, st);
            w[1].load(chunk1 + (size_t)kc * Sub::CHUNK, st);
        };
        auto stage = [&](int buf, const Sub (&w)[2]) {
            w[0].store(dst + buf * BGM * LDS_LD);
            w[1].store(dst + (buf * BGM + GM) * LDS_LD);
        };
        fetch(0, rw[0]);
        fetch(n_steps > 1 ? 1 : 0, rw[1]);
        stage(0, rw[0]);
        lds_barrier();
        for (int kc0 = 0; kc0 < n_steps; kc0 += 2) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int kc = kc0 + u;
                if (kc >= n_steps) break;
                fetch(kc + 2 < n_steps ? kc + 2 : n_steps - 1, rw[u]);
                if (kc + 1 < n_steps) stage(u ^ 1, rw[u ^ 1]);
                lds_barrier();
            }
        }
        return;
    }

    // ---- multiplying waves: row block (wave & 1), token half (wave >> 1)
    const int vb = 2 * (int)blockIdx.x + (wave & 1);           // this wave's 128-row block of the launch
    const int wm = (wave & 1) * GM, wn = (wave >> 1) * 64;
    float16v acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    const int n_blk = (a.T + 15) >> 4, n_g = n_steps * (GK / 16);
    const _Float16 *bp[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int tok = t0 + wn + 32 * i + (lane & 31);
        const int blk = (tok >> 4) < n_blk ? (tok >> 4) : n_blk - 1;
        bp[i] = a.X + (size_t)blk * 16 * a.K + ((lane >> 5) * 16 + (tok & 15)) * 8;
    }
    half8 ring[GK / 16][2];
#pragma unroll
    for (int ks = 0; ks < GK / 16; ++ks)
#pragma unroll
        for (int i = 0; i < 2; ++i) ring[ks][i] = *reinterpret_cast<const half8 *>(bp[i] + (size_t)(ks < n_g ? ks : n_g - 1) * 256);
    const int a_off = (wm + (lane & 31)) * LDS_LD + 8 * (lane >> 5);
    lds_barrier();
    for (int kc = 0; kc < n_steps; ++kc) {
        const _Float16 *Wb = Ws + (kc & 1) * BGM * LDS_LD + a_off;
        half8 af[2][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) af[0][i] = *reinterpret_cast<const half8 *>(Wb + 32 * i * LDS_LD);
#pragma unroll
        for (int ks = 0; ks < GK / 16; ++ks) {
            if (ks + 1 < GK / 16) {
#pragma unroll
                for (int i = 0; i < 4; ++i) af[(ks + 1) & 1][i] = *reinterpret_cast<const half8 *>(Wb + 32 * i * LDS_LD + 16 * (ks + 1));
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[ks & 1][i], ring[ks][j], acc[i][j], 0, 0, 0);
            int gn = (kc + 1) * (GK / 16) + ks;
            gn = gn < n_g ? gn : n_g - 1;
#pragma unroll
            for (int i = 0; i < 2; ++i) ring[ks][i] = *reinterpret_cast<const half8 *>(bp[i] + (size_t)gn * 256);
            // Issue order inside the step: the next step's four fragment reads go out between the first MFMAs (an MFMA
            // holds the matrix pipe for 32 cycles, the wave is free to issue meanwhile), the two activation refills after
            // the last.  Left to itself the scheduler puts the reads behind all eight MFMAs, and the next step then
            // starts by waiting out the LDS latency.
            if (ks + 1 < GK / 16) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      // one LDS read
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
            } else {
                __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);              // the two global loads
            __builtin_amdgcn_sched_barrier(0);
        }
        lds_barrier();
    }

    // D[m][t]: lane holds column t = lane % 32 and rows 8 * (e / 4) + 4 * (lane / 32) + e % 4 of each 32 x 32 block
    if (a.y16_k8) {
        // SwiGLU pair: the row block's rows 0..63 are gate rows, 64..127 the up rows of the same outputs: blocks
        // acc[0..1] and acc[2..3] of this very lane
        const int t_pad = (a.T + 15) & ~15;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int t = t0 + wn + 32 * j + (lane & 31);
                if (t >= t_pad) continue;
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    const int m = vb * (GM / 2) + 32 * i + 8 * e4 + 4 * (lane >> 5);
                    if (m >= a.M) continue;
                    float o[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float g = acc[i][j][4 * e4 + c], u = acc[i + 2][j][4 * e4 + c];
                        o[c] = t < a.T ? g / (1.0f + expf(-g)) * u : 0.f;
                    }
                    note_f16_clamp(a.sat, o[0], o[1], o[2], o[3]);
                    *reinterpret_cast<uint2 *>(a.y16_k8 + (size_t)(t >> 4) * 16 * a.M + ((size_t)(m >> 3) * 16 + (t & 15)) * 8 + (m & 7)) =
                        make_uint2(pack_h2(o[0], o[1]), pack_h2(o[2], o[3]));
                }
            }
        return;
    }
    float *Y = a.Y;
    const float *bias = a.bias;
    int M = a.M, ldy = a.ldy, mb0 = vb * GM;
    if (a.n_seg > 1) {
        const int sg = (vb >= a.seg_begin[1] ? 1 : 0) + (a.n_seg > 2 && vb >= a.seg_begin[2] ? 1 : 0);
        Y = sg == 0 ? a.seg_Y[0] : sg == 1 ? a.seg_Y[1] : a.seg_Y[2];
        bias = sg == 0 ? a.seg_bias[0] : sg == 1 ? a.seg_bias[1] : a.seg_bias[2];
        M = sg == 0 ? a.seg_M[0] : sg == 1 ? a.seg_M[1] : a.seg_M[2];
        ldy = sg == 0 ? a.seg_ldy[0] : sg == 1 ? a.seg_ldy[1] : a.seg_ldy[2];
        mb0 = (vb - (sg == 0 ? 0 : sg == 1 ? a.seg_begin[1] : a.seg_begin[2])) * GM;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int t = t0 + wn + 32 * j + (lane & 31);
            if (t >= a.T) continue;
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int m = mb0 + 32 * i + 8 * e4 + 4 * (lane >> 5);
                if (m >= M) continue;
                float4 o = make_float4(acc[i][j][4 * e4], acc[i][j][4 * e4 + 1], acc[i][j][4 * e4 + 2], acc[i][j][4 * e4 + 3]);
                if (bias) {
                    const float4 b = *reinterpret_cast<const float4 *>(bias + m);
                    o.x += b.x; o.y += b.y; o.z += b.z; o.w += b.w;
                }
                if (a.residual) {
                    const float4 r = *reinterpret_cast<const float4 *>(a.residual + (size_t)t * a.ldres + m);
                    o.x += r.x; o.y += r.y; o.z += r.z; o.w += r.w;
                }
                *reinterpret_cast<float4 *>(Y + (size_t)t * ldy + m) = o;
            }
        }
}

template <int TYPE>
static int launch_gemm_big(const GemmArgs &k, int row_blocks, int t_blocks, hipStream_t stream) {
    constexpr size_t smem = sizeof(_Float16) * 2 * BGM * LDS_LD;
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_big_kernel<TYPE>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    MESH_LAUNCH((gemm_big_kernel<TYPE>), dim3((unsigned)(row_blocks / 2), (unsigned)t_blocks), dim3(GEMM_THREADS), smem, stream, k);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// Second kernel of a split launch: adds the slices of part[slice][token][row] in slice order and applies the epilogue
// of the unsplit kernel.  One thread per (token, four consecutive rows); rows run fastest, so partial reads and output
// writes are contiguous.
__global__ __launch_bounds__(256) void gemm_splitk_epilogue_kernel(GemmArgs a, int row_blocks) {
    const size_t ld = (size_t)row_blocks * GM;
    const int t_pad = a.y16_k8 ? (a.T + 15) & ~15 : a.T;
    const int per_block = a.y16_k8 ? GM / 8 : GM / 4;          // threads per row block: 64 gate rows or 128 rows, four each
    const size_t n = (size_t)t_pad * row_blocks * per_block;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < n; idx += (size_t)gridDim.x * 256) {
        const int q = (int)(idx % per_block), bx = (int)((idx / per_block) % row_blocks), t = (int)(idx / ((size_t)per_block * row_blocks));
        auto sum4 = [&](size_t row) {
            // four slices in flight at a time (indices past the end re-read the last slice and are not added)
            float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int z0 = 0; z0 < a.ksplit; z0 += 4) {
                float4 p[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int z = z0 + u < a.ksplit ? z0 + u : a.ksplit - 1;
                    p[u] = *reinterpret_cast<const float4 *>(a.part + ((size_t)z * a.T + t) * ld + row);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (z0 + u < a.ksplit) { o.x += p[u].x; o.y += p[u].y; o.z += p[u].z; o.w += p[u].w; }
            }
            return o;
        };
        if (a.y16_k8) {
            const int m = bx * (GM / 2) + 4 * q;
            if (m >= a.M) continue;
            float o[4] = {0.f, 0.f, 0.f, 0.f};                 // padding columns of the last token block hold zeros
            if (t < a.T) {
                const float4 g = sum4((size_t)bx * GM + 4 * q), u = sum4((size_t)bx * GM + GM / 2 + 4 * q);
                o[0] = g.x / (1.0f + expf(-g.x)) * u.x; o[1] = g.y / (1.0f + expf(-g.y)) * u.y;
                o[2] = g.z / (1.0f + expf(-g.z)) * u.z; o[3] = g.w / (1.0f + expf(-g.w)) * u.w;
            }
            note_f16_clamp(a.sat, o[0], o[1], o[2], o[3]);
            *reinterpret_cast<uint2 *>(a.y16_k8 + (size_t)(t >> 4) * 16 * a.M + ((size_t)(m >> 3) * 16 + (t & 15)) * 8 + (m & 7)) =
                make_uint2(pack_h2(o[0], o[1]), pack_h2(o[2], o[3]));
            continue;
        }
        float *Y = a.Y;
        const float *bias = a.bias;
        int M = a.M, ldy = a.ldy, mb0 = bx * GM, kind = a.kind[0];
        if (a.n_seg > 1) {
            const int sg = (bx >= a.seg_begin[1] ? 1 : 0) + (a.n_seg > 2 && bx >= a.seg_begin[2] ? 1 : 0);
            kind = sg == 0 ? a.kind[0] : sg == 1 ? a.kind[1] : a.kind[2];
            Y = sg == 0 ? a.seg_Y[0] : sg == 1 ? a.seg_Y[1] : a.seg_Y[2];
            bias = sg == 0 ? a.seg_bias[0] : sg == 1 ? a.seg_bias[1] : a.seg_bias[2];
            M = sg == 0 ? a.seg_M[0] : sg == 1 ? a.seg_M[1] : a.seg_M[2];
            ldy = sg == 0 ? a.seg_ldy[0] : sg == 1 ? a.seg_ldy[1] : a.seg_ldy[2];
            mb0 = (bx - (sg == 0 ? 0 : sg == 1 ? a.seg_begin[1] : a.seg_begin[2])) * GM;
        }
        const int m = mb0 + 4 * q;
        if (m >= M) continue;
        float4 o = sum4((size_t)bx * GM + 4 * q);
        if (bias) {
            const float4 b = *reinterpret_cast<const float4 *>(bias + m);
            o.x += b.x; o.y += b.y; o.z += b.z; o.w += b.w;
        }
        if (a.rope.pos && kind != GEMV_KIND_PLAIN) {
            // rows m..m+3 of a q / k / v projection: two neighbouring pairs of one head (head_dim % 4 == 0)
            const int hd = a.rope.head_dim, head = m / hd, dd = m - head * hd, pos = a.rope.pos[t];
            if (kind != GEMV_KIND_V) {
                if (dd < a.rope.n_rot) {
                    float sn, cs;
                    sincosf((float)pos * a.rope.inv_freq[dd >> 1], &sn, &cs);
                    const float x0 = o.x, x1 = o.y;
                    o.x = x0 * cs - x1 * sn; o.y = x0 * sn + x1 * cs;
                }
                if (dd + 2 < a.rope.n_rot) {
                    float sn, cs;
                    sincosf((float)pos * a.rope.inv_freq[(dd >> 1) + 1], &sn, &cs);
                    const float x0 = o.z, x1 = o.w;
                    o.z = x0 * cs - x1 * sn; o.w = x0 * sn + x1 * cs;
                }
            }
            if (kind == GEMV_KIND_Q) {
                *reinterpret_cast<float4 *>(Y + (size_t)t * ldy + m) = o;
            } else {
                uint16_t *cache = kind == GEMV_KIND_K ? a.rope.kcache : a.rope.vcache;
                *reinterpret_cast<uint2 *>(cache + (((size_t)a.rope.seq[t] * a.rope.n_kv + head) * a.rope.n_ctx + pos) * hd + dd) =
                    make_uint2(pack_h2(o.x, o.y), pack_h2(o.z, o.w));
            }
            continue;
        }
        if (a.residual) {
            const float4 r = *reinterpret_cast<const float4 *>(a.residual + (size_t)t * a.ldres + m);
            o.x += r.x; o.y += r.y; o.z += r.z; o.w += r.w;
        }
        *reinterpret_cast<float4 *>(Y + (size_t)t * ldy + m) = o;
    }
}

template <int TYPE, bool PACKED, bool XDIRECT, bool SPLIT, bool NARROW, bool GROUPED = false>
static int launch_gemm_kernel(const GemmArgs &k, dim3 grid, hipStream_t stream) {
    // two stages of the weight slab, and of the activation slab unless the activations bypass LDS: 73 728 / 36 864 B
    constexpr size_t smem = sizeof(_Float16) * 2 * (GM + (XDIRECT ? 0 : GN)) * LDS_LD;
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_kq_kernel<TYPE, PACKED, XDIRECT, SPLIT, NARROW, GROUPED>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    MESH_LAUNCH((gemm_kq_kernel<TYPE, PACKED, XDIRECT, SPLIT, NARROW, GROUPED>), grid, dim3(GEMM_THREADS), smem, stream, k);
    MESH_LAUNCH_CHECK();
    if (SPLIT) {
        const int t_pad = k.y16_k8 ? (k.T + 15) & ~15 : k.T;
        const size_t n = (size_t)t_pad * grid.x * (k.y16_k8 ? GM / 8 : GM / 4);
        const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 4096);
        MESH_LAUNCH(gemm_splitk_epilogue_kernel, dim3(blocks), dim3(256), 0, stream, k, (int)grid.x);
        MESH_LAUNCH_CHECK();
    }
    return MESH_OK;
}

static int gemm_n_cu() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) n = p.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

template <int TYPE, bool PACKED, bool XDIRECT>
static int launch_gemm(const GemmArgs &k, dim3 grid, hipStream_t stream) {
    // calls of at most 64 tokens on the production layout (GEMM-layout weights, k8-major activations): narrow tile
    if constexpr (PACKED && XDIRECT) {
        if (k.T <= GN / 2 && k.narrow_tile)
            return k.ksplit > 1 ? launch_gemm_kernel<TYPE, true, true, true, true>(k, grid, stream) : launch_gemm_kernel<TYPE, true, true, false, true>(k, grid, stream);
    }
    return k.ksplit > 1 ? launch_gemm_kernel<TYPE, PACKED, XDIRECT, true, false>(k, grid, stream) : launch_gemm_kernel<TYPE, PACKED, XDIRECT, false, false>(k, grid, stream);
}

// slices of K for a launch of row_blocks x t_blocks workgroups (1: not split); *k_per_split = k-steps per slice
static int split_plan(const GemmArgs &a, int row_blocks, int t_blocks, int *k_per_split) {
    const int n_all = a.K / GK;
    *k_per_split = n_all;
    if (!a.part) return 1;
    const int wgs = row_blocks * t_blocks, ncu = gemm_n_cu();
    int ks = 1;
    while (ks < 16 && wgs * ks * 2 <= ncu && n_all / (ks * 2) >= 8 &&
           (size_t)(ks * 2) * a.T * row_blocks * GM * sizeof(float) <= a.part_bytes) ks *= 2;
    if (ks <= 1) return 1;
    *k_per_split = (n_all + ks - 1) / ks;
    return (n_all + *k_per_split - 1) / *k_per_split;      // no empty slice
}

int gemm_split_count(const GemmArgs &a) {
    if (a.M <= 0 || a.K <= 0 || a.T <= 0) return 1;
    const int row_blocks = a.y16_k8 ? (a.M + GM / 2 - 1) / (GM / 2) : (a.M + GM - 1) / GM;
    int kps;
    return split_plan(a, row_blocks, (a.T + GN - 1) / GN, &kps);
}

int gemm_kquant(const GemmArgs &a, hipStream_t stream) {
    if (!a.X || a.M <= 0 || a.K <= 0 || a.T <= 0) return fail(MESH_ERR_INVALID, "gemm: null pointer or empty shape");
    if (a.y16_k8 || a.n_seg > 1) {
        if (!a.Wp || (a.y16_k8 && (a.n_seg > 1 || a.bias || a.residual)) || a.n_seg > 3)
            return fail(MESH_ERR_INVALID, "gemm: multi-matrix and SwiGLU launches need the GEMM layout (and no bias / residual for SwiGLU)");
        for (int i = 0; i < a.n_seg && !a.y16_k8; ++i)
            if (!a.seg_Y[i] || a.seg_M[i] <= 0 || a.seg_M[i] % 4 || a.seg_ldy[i] % 4 || (i + 1 < a.n_seg && a.seg_M[i] % GM) || (a.residual))
                return fail(MESH_ERR_INVALID, "gemm: bad matrix %d of a multi-matrix launch", i);
    } else if (!a.W || !a.Y) return fail(MESH_ERR_INVALID, "gemm: null pointer");
    if (a.K % QK_K || a.M % 4 || a.ldx % 8 || a.ldy % 4 || (a.residual && a.ldres % 4))
        return fail(MESH_ERR_INVALID, "gemm: shape M=%d K=%d not supported (K %% 256, M %% 4)", a.M, a.K);
    if ((reinterpret_cast<uintptr_t>(a.X) | reinterpret_cast<uintptr_t>(a.Y)) & 15) return fail(MESH_ERR_INVALID, "gemm: X and Y must be 16-byte aligned");
    GemmArgs k = a;
    k.M_pad = (a.M + TILE_ROWS - 1) / TILE_ROWS * TILE_ROWS;
    const int row_blocks = a.y16_k8 ? (a.M + GM / 2 - 1) / (GM / 2) : (a.M + GM - 1) / GM;
    if (a.tiles) {
        // expert launch: one workgroup row per tile of the list (those past *n_tiles leave at once)
        if (!a.Wp || !a.x_k8 || !a.n_tiles || a.max_tiles <= 0 || a.n_seg > 1 || a.bias || a.residual || a.rope.pos || a.expert_stride % 16)
            return fail(MESH_ERR_INVALID, "gemm: an expert launch needs the GEMM layout, k8-major activations and a plain or SwiGLU epilogue");
        if (a.type != MESH_Q4_K && a.type != MESH_Q6_K) return fail(MESH_ERR_UNSUPPORTED, "gemm: no MFMA kernel for ggml type %d", a.type);
        const dim3 g((unsigned)row_blocks, (unsigned)a.max_tiles);
        k.ksplit = 1;
        k.k_per_split = a.K / GK;
        return a.type == MESH_Q4_K ? launch_gemm_kernel<MESH_Q4_K, true, true, false, false, true>(k, g, stream)
                                   : launch_gemm_kernel<MESH_Q6_K, true, true, false, false, true>(k, g, stream);
    }
    dim3 grid((unsigned)row_blocks, (unsigned)((a.T + GN - 1) / GN));
    // A launch of fewer workgroups than CUs walks all of K in each of them while the rest of the chip idles: split K
    // over blockIdx.z (slices of at least 8 k-steps, at most one workgroup per CU in total, partial tiles within the
    // scratch the caller gave).
    k.k_per_split = a.K / GK;
    k.ksplit = split_plan(a, row_blocks, (int)grid.y, &k.k_per_split);
    grid.z = (unsigned)k.ksplit;
    if (a.rope.pos && k.ksplit <= 1) return fail(MESH_ERR_INVALID, "gemm: RoPE / KV append needs a split launch");
    if (a.rope.pos && (a.y16_k8 || a.residual || a.rope.head_dim % 4 || a.rope.n_rot % 2))
        return fail(MESH_ERR_INVALID, "gemm: RoPE / KV append on a launch it does not fit");
    if (a.type != MESH_Q4_K && a.type != MESH_Q6_K) return fail(MESH_ERR_UNSUPPORTED, "gemm: no MFMA kernel for ggml type %d", a.type);
    const bool q4 = a.type == MESH_Q4_K, packed = a.Wp != nullptr;
    // enough workgroups of the 256 x 128 tile to give every CU one: the big tile (gemm_big_kernel)
    if (a.x_k8 && packed && k.ksplit <= 1 && !a.rope.pos && row_blocks % 2 == 0 && a.big_tile &&
        (row_blocks / 2) * (int)grid.y >= gemm_n_cu())
        return q4 ? launch_gemm_big<MESH_Q4_K>(k, row_blocks, (int)grid.y, stream) : launch_gemm_big<MESH_Q6_K>(k, row_blocks, (int)grid.y, stream);
    if (a.x_k8) {
        if (packed) return q4 ? launch_gemm<MESH_Q4_K, true, true>(k, grid, stream) : launch_gemm<MESH_Q6_K, true, true>(k, grid, stream);
        return q4 ? launch_gemm<MESH_Q4_K, false, true>(k, grid, stream) : launch_gemm<MESH_Q6_K, false, true>(k, grid, stream);
    }
    if (packed) return q4 ? launch_gemm<MESH_Q4_K, true, false>(k, grid, stream) : launch_gemm<MESH_Q6_K, true, false>(k, grid, stream);
    return q4 ? launch_gemm<MESH_Q4_K, false, false>(k, grid, stream) : launch_gemm<MESH_Q6_K, false, false>(k, grid, stream);
}

// ---- GEMM layout ----------------------------------------------------------------------------------------------
// One workgroup writes one chunk: thread s re-reads its (row, sub-block) from the mat-vec tiles the way the staging
// thread of the unpacked kernel does, and writes it in the packed form.
// tiled2 set: a gate / up pair -- the chunk's rows 0..63 are rows [64 mb, 64 mb + 64) of `tiled`, rows 64..127 those of tiled2.
template <int TYPE>
__global__ __launch_bounds__(256) void gemm_pack_kernel(const uint8_t *__restrict__ tiled, const uint8_t *__restrict__ tiled2,
                                                        uint8_t *__restrict__ packed, int M_pad, int nsb) {
    constexpr int TB = TYPE == MESH_Q4_K ? Q4K_TILE_BYTES : Q6K_TILE_BYTES;
    constexpr int CH = PackedSub<TYPE>::CHUNK;
    const int kc = blockIdx.x, mb = blockIdx.y, n_steps = gridDim.x, s = threadIdx.x;
    const int h = s & 1;
    int wrow = mb * GM + (s >> 1);
    if (tiled2) {
        wrow = mb * (GM / 2) + ((s >> 1) & (GM / 2 - 1));
        if ((s >> 1) >= GM / 2) tiled = tiled2;
    }
    uint8_t *chunk = packed + ((size_t)mb * n_steps + kc) * CH;
    if (wrow >= M_pad) {
        *reinterpret_cast<uint4 *>(chunk + s * 16) = make_uint4(0, 0, 0, 0);
        if (TYPE == MESH_Q6_K) *reinterpret_cast<uint2 *>(chunk + 4096 + s * 8) = make_uint2(0, 0);
        *reinterpret_cast<uint2 *>(chunk + (TYPE == MESH_Q6_K ? 6144 : 4096) + s * 8) = make_uint2(0u, 0u);
        return;
    }
    RawSub<TYPE> r;
    r.load(tiled + ((size_t)(wrow >> 4) * nsb + (kc >> 2)) * TB, wrow & 15, kc & 3, h);
    r.pack(kc & 3, h, chunk, s);
}

size_t gemm_packed_bytes(int type, int64_t M, int64_t K) {
    if ((type != MESH_Q4_K && type != MESH_Q6_K) || M <= 0 || K <= 0 || K % QK_K) return 0;
    const size_t chunk = type == MESH_Q4_K ? PackedSub<MESH_Q4_K>::CHUNK : PackedSub<MESH_Q6_K>::CHUNK;
    return (size_t)((M + GM - 1) / GM) * (size_t)(K / GK) * chunk;
}

int gemm_pack(int type, const void *tiled, void *packed, int64_t M, int64_t K, hipStream_t stream) {
    if (!tiled || !packed || gemm_packed_bytes(type, M, K) == 0) return fail(MESH_ERR_INVALID, "gemm_pack: bad arguments (type %d, M %lld, K %lld)", type, (long long)M, (long long)K);
    const dim3 grid((unsigned)(K / GK), (unsigned)((M + GM - 1) / GM));
    const int M_pad = (int)((M + TILE_ROWS - 1) / TILE_ROWS * TILE_ROWS), nsb = (int)(K / QK_K);
    if (grid.y > 65535u) return fail(MESH_ERR_UNSUPPORTED, "gemm_pack: %lld rows are too many", (long long)M);
    if (type == MESH_Q4_K) MESH_LAUNCH(gemm_pack_kernel<MESH_Q4_K>, grid, dim3(256), 0, stream, static_cast<const uint8_t *>(tiled), nullptr, static_cast<uint8_t *>(packed), M_pad, nsb);
    else MESH_LAUNCH(gemm_pack_kernel<MESH_Q6_K>, grid, dim3(256), 0, stream, static_cast<const uint8_t *>(tiled), nullptr, static_cast<uint8_t *>(packed), M_pad, nsb);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

size_t gemm_packed_pair_bytes(int type, int64_t M, int64_t K) {
    if ((type != MESH_Q4_K && type != MESH_Q6_K) || M <= 0 || K <= 0 || K % QK_K) return 0;
    const size_t chunk = type == MESH_Q4_K ? PackedSub<MESH_Q4_K>::CHUNK : PackedSub<MESH_Q6_K>::CHUNK;
    return (size_t)((M + GM / 2 - 1) / (GM / 2)) * (size_t)(K / GK) * chunk;
}

int gemm_pack_pair(int type, const void *gate_tiled, const void *up_tiled, void *packed, int64_t M, int64_t K, hipStream_t stream) {
    if (!gate_tiled || !up_tiled || !packed || gemm_packed_pair_bytes(type, M, K) == 0)
        return fail(MESH_ERR_INVALID, "gemm_pack_pair: bad arguments (type %d, M %lld, K %lld)", type, (long long)M, (long long)K);
    const dim3 grid((unsigned)(K / GK), (unsigned)((M + GM / 2 - 1) / (GM / 2)));
    const int M_pad = (int)((M + TILE_ROWS - 1) / TILE_ROWS * TILE_ROWS), nsb = (int)(K / QK_K);
    if (grid.y > 65535u) return fail(MESH_ERR_UNSUPPORTED, "gemm_pack_pair: %lld rows are too many", (long long)M);
    const uint8_t *g = static_cast<const uint8_t *>(gate_tiled), *u = static_cast<const uint8_t *>(up_tiled);
    if (type == MESH_Q4_K) MESH_LAUNCH(gemm_pack_kernel<MESH_Q4_K>, grid, dim3(256), 0, stream, g, u, static_cast<uint8_t *>(packed), M_pad, nsb);
    else MESH_LAUNCH(gemm_pack_kernel<MESH_Q6_K>, grid, dim3(256), 0, stream, g, u, static_cast<uint8_t *>(packed), M_pad, nsb);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// ---- small elementwise companions of the prefill path ---------------------------------------------------------
// y16[t] = f16( x[t] * rsqrt(mean(x[t]^2) + eps) * w ), one workgroup per token
__global__ __launch_bounds__(256) void rmsnorm_f16_kernel(const float *__restrict__ x, const float *__restrict__ w, float eps,
                                                          int n, _Float16 *__restrict__ y, int ldy, unsigned *sat) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const float *xt = x + (size_t)t * n;
    float ss = 0.f;
    for (int i = tid * 4; i < n; i += 1024) {
        const float4 v = *reinterpret_cast<const float4 *>(xt + i);
        ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    const float scale = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)n + eps);
    for (int i = tid * 4; i < n; i += 1024) {
        const float4 v = *reinterpret_cast<const float4 *>(xt + i);
        const float4 g = *reinterpret_cast<const float4 *>(w + i);
        note_f16_clamp(sat, v.x * scale * g.x, v.y * scale * g.y, v.z * scale * g.z, v.w * scale * g.w);
        *reinterpret_cast<uint2 *>(y + (size_t)t * ldy + i) =
            make_uint2(pack_h2(v.x * scale * g.x, v.y * scale * g.y), pack_h2(v.z * scale * g.z, v.w * scale * g.w));
    }
}

int rmsnorm_f16(const float *x, const float *w, float eps, int T, int n, _Float16 *y, int ldy, hipStream_t stream, unsigned *sat) {
    if (T <= 0) return MESH_OK;
    if (n % 4 || ldy % 4) return fail(MESH_ERR_INVALID, "rmsnorm: row length %d not a multiple of 4", n);
    MESH_LAUNCH(rmsnorm_f16_kernel, dim3((unsigned)T), dim3(256), 0, stream, x, w, eps, n, y, ldy, sat);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// out16 = f16( silu(gate) * up )
__global__ __launch_bounds__(256) void swiglu_f16_kernel(const float *__restrict__ g, const float *__restrict__ u,
                                                         _Float16 *__restrict__ o, int64_t n4, unsigned *sat) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const float4 a = reinterpret_cast<const float4 *>(g)[i], b = reinterpret_cast<const float4 *>(u)[i];
    const float r0 = a.x / (1.0f + expf(-a.x)) * b.x, r1 = a.y / (1.0f + expf(-a.y)) * b.y;
    const float r2 = a.z / (1.0f + expf(-a.z)) * b.z, r3 = a.w / (1.0f + expf(-a.w)) * b.w;
    note_f16_clamp(sat, r0, r1, r2, r3);
    reinterpret_cast<uint2 *>(o)[i] = make_uint2(pack_h2(r0, r1), pack_h2(r2, r3));
}

int swiglu_f16(const float *gate, const float *up, _Float16 *out, int64_t n, hipStream_t stream, unsigned *sat) {
    if (n <= 0) return MESH_OK;
    if (n % 4) return fail(MESH_ERR_INVALID, "swiglu: count not a multiple of 4");
    MESH_LAUNCH(swiglu_f16_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, stream, gate, up, out, n / 4, sat);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

}  // namespace mesh
