// Dequant-fused GEMV for decode (a few tokens per call): y = W x with W in q4_K / q6_K blocks, tiled as described
// in gemv.hpp.  Stands where ggml_backend_graph_compute runs mul_mat for a worker's layers
// (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451).
//
// Design (gfx950, wave64):
//  * One 1024-thread workgroup per CU owns a few consecutive 16-row tile-rows; its 16 waves split K (and, for
//    short rows, the tile-rows) and meet in LDS once, so results are deterministic (no atomics).  Weight bytes
//    cross HBM exactly once per launch, as dense 16-byte vector loads of contiguous tiles; every wave requests the
//    activations and its first tiles before anything else so the two latencies overlap.
//  * The activation vector is converted once per workgroup to 16-bit fixed point per 32-element block
//    (x ~ d_b * (256*hi + lo), hi/lo int8 in LDS).  The RMS norm that precedes every projection is folded in: the
//    norm weight multiplies x before quantisation, and the norm scale -- a scalar -- multiplies the finished dot
//    products in the epilogue, so one pass over x and one barrier suffice.  ggml's own kernels round activations
//    to 8 bits here; 16 bits keeps a 16-layer stage within 2e-4 of the f32-activation oracle where 8 bits would
//    sit at 1.6e-2.
//  * Products are integer: v_dot4_i32_i8 of the raw 4/6-bit quants with hi and lo, combined as (I_hi << 8) + I_lo
//    and scaled once per sub-block.  The q4_K "min" term and the q6_K "-32" offset use per-block sums of x that the
//    prologue leaves in LDS.
//  * Lane l = 4*r + c handles row r, quarter c of a super-block, so it needs only the 2 (q4_K) or 4 (q6_K)
//    sub-scales of its quarter, and the 16 rows of a tile read the same x addresses (LDS broadcast).

#include "gemv.hpp"

#include <algorithm>

namespace mesh {

int gemv_generic(const GemvArgs &a, hipStream_t stream);

constexpr int GEMV_THREADS = 1024;        // one workgroup fills a CU: 16 waves, 4 per SIMD
constexpr int GEMV_WAVES = GEMV_THREADS / 64;
constexpr float XQ_LEVELS = 32512.0f;     // 127 * 256: |256*hi + lo| <= 32512 with hi, lo in int8

struct GemvKernelArgs {
    // matrix i's tiles, biased so that tile-row tr (global index over the launch) starts at wbase[i] + tr * row_stride
    const uint8_t *wbase[3];
    float *y[3];
    const float *bias[3];
    int M[3], ldy[3];
    int tile_begin[4];     // first global tile-row of each matrix; tile_begin[n_mat] = total
    int n_mat;
    const float *x;
    int ldx, K;
    const float *norm_w;
    float eps;
    const float *residual;
    int ldres;
    int epi;
    int ks;                // waves along K (the other 16/ks ways split the workgroup's tile-rows)
    // expert indirection (MoE): blockIdx.y = (token, slot) pair p; it uses expert expert_ids[p]'s copy of every
    // matrix (expert_stride bytes apart), reads activation column p / x_div and writes output row p
    const int32_t *expert_ids;
    size_t expert_stride;
    int x_div;
};

// LDS view of the quantised activations of NB columns
struct XStage {
    int8_t *xh, *xl;     // [NB][K]
    float *xd, *xs;      // [NB][K/32]: block scale d_b (without the norm scale), block sum of x = d_b * sum of quants
    int *xi16;           // [NB][K/16]: integer sum of quants per 16 elements (q6_K only)
    float *ssq;          // [16 waves][NB] partial sums of x^2 for the norm
    float *red;          // cross-wave partials [KS][rows][NU][16][NB]
};

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

__device__ __forceinline__ uint32_t pack_bytes(int a, int b, int c, int d) {
    return (uint32_t)(a & 0xFF) | ((uint32_t)(b & 0xFF) << 8) | ((uint32_t)(c & 0xFF) << 16) | ((uint32_t)(d & 0xFF) << 24);
}

// Phase timestamps for tuning builds (-DMESH_GEMV_TRACE); compiled out of the product.
#ifdef MESH_GEMV_TRACE
__device__ long long *g_gemv_trace = nullptr;
extern "C" int mesh_debug_set_gemv_trace(long long *p) {
    return hipMemcpyToSymbol(HIP_SYMBOL(g_gemv_trace), &p, sizeof p) == hipSuccess ? 0 : -2;
}
#define GEMV_MARK(k)                                                                              \
    do {                                                                                          \
        if (g_gemv_trace && (threadIdx.x & 63) == 0)                                              \
            g_gemv_trace[((size_t)blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6)) * 8 + (k)] = wall_clock64(); \
    } while (0)
#else
#define GEMV_MARK(k) do { } while (0)
#endif

// ------------------------------------------------------------------------------------------------ prologue
// Eight consecutive elements of each column per thread; 4 neighbouring lanes share a 32-element block.
template <int NB>
struct XRegs {
    float4 a[NB], b[NB];
};

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

template <int NB, bool NEED_I16>
__device__ __forceinline__ void x_quantise(const XRegs<NB> &X, const GemvKernelArgs &a, const XStage &S, int g, bool live,
                                           float (&ss)[NB]) {
    const int lane = threadIdx.x & 63, K = a.K;
    float4 w0 = make_float4(1.f, 1.f, 1.f, 1.f), w1 = w0;
    if (a.norm_w && live) {
        w0 = *reinterpret_cast<const float4 *>(a.norm_w + g * 8);
        w1 = *reinterpret_cast<const float4 *>(a.norm_w + g * 8 + 4);
    }
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

// ------------------------------------------------------------------------------------------------ tiles
template <int TYPE> struct TileRegs;

template <> struct TileRegs<MESH_Q4_K> {
    static constexpr int BYTES = Q4K_TILE_BYTES;
    uint4 hdr, qa, qb;
    __device__ __forceinline__ void load(const uint8_t *__restrict__ tile, int lane) {
        hdr = *reinterpret_cast<const uint4 *>(tile + (lane >> 2) * 16);
        qa = *reinterpret_cast<const uint4 *>(tile + 256 + lane * 32);
        qb = *reinterpret_cast<const uint4 *>(tile + 256 + lane * 32 + 16);
    }
};

template <> struct TileRegs<MESH_Q6_K> {
    static constexpr int BYTES = Q6K_TILE_BYTES;
    uint4 qla, qlb, qh, sc;
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t *__restrict__ tile, int lane) {
        const int r = lane >> 2, c = lane & 3, n = c >> 1, u = c & 1;
        qla = *reinterpret_cast<const uint4 *>(tile + r * 128 + 64 * n + 16 * u);
        qlb = *reinterpret_cast<const uint4 *>(tile + r * 128 + 64 * n + 32 + 16 * u);
        qh = *reinterpret_cast<const uint4 *>(tile + 2048 + r * 64 + 32 * n + 16 * u);
        sc = *reinterpret_cast<const uint4 *>(tile + 3072 + r * 16);
        d = *reinterpret_cast<const uint16_t *>(tile + 3328 + r * 2);
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

// ------------------------------------------------------------------------------------------------ kernel
// Work decomposition.  A workgroup owns `rows_here` consecutive tile-rows (16 output rows each) of the launch's
// matrices (all of one K-quant type) and stages the activations once.  Its 16 waves are arranged KS x RS: wave
// (ks, rs) takes super-blocks ks, ks+KS, ... of the local tile-rows rs, rs+RS, ..., for NU matrices each (2 for the
// fused gate/up pair).  A wave walks its tiles as one flat list with the next tile always in flight; at the end of
// each (tile-row, matrix) segment the lanes' sums are reduced over the 4 lanes of a row and parked in LDS, where the
// KS partials of a row meet after one barrier.
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

template <int TYPE, int NB, int NU>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_dot_kernel(const GemvKernelArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int TB = TileRegs<TYPE>::BYTES;
    constexpr bool NEED_I16 = TYPE == MESH_Q6_K;
    const int K = a.K;
    XStage S;
    S.xh = reinterpret_cast<int8_t *>(smem);
    S.xl = S.xh + NB * K;
    S.xd = reinterpret_cast<float *>(S.xl + NB * K);
    S.xs = S.xd + NB * (K >> 5);
    S.xi16 = reinterpret_cast<int *>(S.xs + NB * (K >> 5));
    S.ssq = reinterpret_cast<float *>(S.xi16 + (NEED_I16 ? NB * (K >> 4) : 0));
    S.red = S.ssq + GEMV_WAVES * NB;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    GEMV_MARK(0);
    // activations first: they gate everything
    const int ng = K >> 3;
    const float *xcol = a.x;
    size_t eoff = 0, ycol = 0;
    if (a.expert_ids) {
        const int p = blockIdx.y;
        xcol = a.x + (size_t)(p / a.x_div) * a.ldx;
        eoff = (size_t)a.expert_ids[p] * a.expert_stride;
        ycol = p;
    }
    XRegs<NB> X;
    x_fetch<NB>(X, xcol, a.ldx, tid, tid < ng);

    const int nsb = K / QK_K;
    const int KS = a.ks, RS = GEMV_WAVES / KS;
    const int ks = wave % KS, rs = wave / KS;
    const int total_rows = a.tile_begin[a.n_mat];
    const int tr0 = (int)(((long long)blockIdx.x * total_rows) / gridDim.x);
    const int tr1 = (int)(((long long)(blockIdx.x + 1) * total_rows) / gridDim.x);
    const int rows_here = tr1 - tr0;
    const int n_i = rs < RS ? (nsb - ks + KS - 1) / KS : 0;      // tiles per segment (ks < KS <= nsb)
    const size_t row_stride = (size_t)nsb * TB;

    auto tile_ptr = [&](const TileCursor<NU> &c) -> const uint8_t * {
        const int tr = tr0 + c.j;
        int mi = c.u;
        if (NU == 1) mi = (tr >= a.tile_begin[1] ? 1 : 0) + (tr >= a.tile_begin[2] ? 1 : 0);
        return a.wbase[mi] + eoff + (size_t)tr * row_stride + (size_t)(ks + KS * c.ii) * TB;
    };

    TileCursor<NU> ld{rs, 0, 0}, cp{rs, 0, 0};
    TileRegs<TYPE> t0, t1;
    const bool any = n_i > 0 && rs < rows_here;
    if (any) {
        t0.load(tile_ptr(ld), lane);
        ld.advance(n_i, RS);
        if (ld.j < rows_here) { t1.load(tile_ptr(ld), lane); ld.advance(n_i, RS); }
    }
    GEMV_MARK(1);

    float ss[NB];
#pragma unroll
    for (int t = 0; t < NB; ++t) ss[t] = 0.f;
    x_quantise<NB, NEED_I16>(X, a, S, tid, tid < ng, ss);
    for (int g0 = GEMV_THREADS; g0 < ng; g0 += GEMV_THREADS) {
        x_fetch<NB>(X, xcol, a.ldx, g0 + tid, g0 + tid < ng);
        x_quantise<NB, NEED_I16>(X, a, S, g0 + tid, g0 + tid < ng, ss);
    }
    if (a.norm_w) {
#pragma unroll
        for (int t = 0; t < NB; ++t) {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) ss[t] += __shfl_xor(ss[t], o);
            if (lane == 0) S.ssq[wave * NB + t] = ss[t];
        }
    }
    __syncthreads();
    GEMV_MARK(2);

    float acc[NB];
#pragma unroll
    for (int t = 0; t < NB; ++t) acc[t] = 0.f;
    auto finish_segment = [&](const TileCursor<NU> &c) {
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            float v = acc[t];
            v += __shfl_xor(v, 1);
            v += __shfl_xor(v, 2);
            if ((lane & 3) == 0) S.red[(((ks * rows_here + c.j) * NU + c.u) * 16 + (lane >> 2)) * NB + t] = v;
            acc[t] = 0.f;
        }
    };
    if (any) {
        // two tiles alternate between the register sets; each is reloaded as soon as it has been consumed
        while (true) {
            tile_compute<NB>(t0, lane, ks + KS * cp.ii, S, K, acc);
            if (cp.ii + 1 == n_i) finish_segment(cp);
            cp.advance(n_i, RS);
            if (ld.j < rows_here) { t0.load(tile_ptr(ld), lane); ld.advance(n_i, RS); }
            if (cp.j >= rows_here) break;
            tile_compute<NB>(t1, lane, ks + KS * cp.ii, S, K, acc);
            if (cp.ii + 1 == n_i) finish_segment(cp);
            cp.advance(n_i, RS);
            if (ld.j < rows_here) { t1.load(tile_ptr(ld), lane); ld.advance(n_i, RS); }
            if (cp.j >= rows_here) break;
        }
    }
    GEMV_MARK(3);
    __syncthreads();
    GEMV_MARK(4);

    // outputs of this workgroup: rows_here x 16 rows x NB columns
    for (int o = tid; o < rows_here * 16 * NB; o += GEMV_THREADS) {
        const int t = o % NB, r = (o / NB) % 16, j = o / (NB * 16);
        const int tr = tr0 + j;
        int mi = 0;
        if (NU == 1) mi = (tr >= a.tile_begin[1] ? 1 : 0) + (tr >= a.tile_begin[2] ? 1 : 0);
        const int row = (tr - a.tile_begin[mi]) * TILE_ROWS + r;
        if (row >= a.M[mi]) continue;
        float s0 = 0.f, s1 = 0.f;
        for (int k2 = 0; k2 < KS; ++k2) {
            s0 += S.red[(((k2 * rows_here + j) * NU + 0) * 16 + r) * NB + t];
            if (NU == 2) s1 += S.red[(((k2 * rows_here + j) * NU + 1) * 16 + r) * NB + t];
        }
        if (a.norm_w) {
            float q = 0.f;
#pragma unroll
            for (int w = 0; w < GEMV_WAVES; ++w) q += S.ssq[w * NB + t];
            const float scale = 1.0f / sqrtf(q / (float)K + a.eps);
            s0 *= scale;
            s1 *= scale;
        }
        if (a.bias[mi]) s0 += a.bias[mi][row];
        float out;
        if (NU == 2) {
            if (a.bias[1]) s1 += a.bias[1][row];
            out = (s0 / (1.0f + expf(-s0))) * s1;
        } else if (a.epi == EPI_RESIDUAL) {
            out = a.residual[(size_t)t * a.ldres + row] + s0;
        } else {
            out = s0;
        }
        a.y[mi][((size_t)t + ycol) * a.ldy[mi] + row] = out;
    }
    GEMV_MARK(5);
}

constexpr size_t LDS_LIMIT = 160 * 1024;
constexpr int MAX_ROWS_X_KS = 64;       // bound on (tile-rows per workgroup) x KS, sizes the LDS partial buffer

static size_t dot_smem_bytes(int type, int NB, int K, int rows_here, int KS, int NU) {
    return (size_t)NB * (2 * (size_t)K + (size_t)(K / 32) * 8 + (type == MESH_Q6_K ? (size_t)(K / 16) * 4 : 0)) +
           sizeof(float) * ((size_t)KS * rows_here * NU * 16 * NB + GEMV_WAVES * NB);
}

template <int TYPE, int NB, int NU>
static int launch_dot(const GemvKernelArgs &ka, dim3 grid, size_t smem, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_dot_kernel<TYPE, NB, NU>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT));
        attr_set = true;
    }
    gemv_dot_kernel<TYPE, NB, NU><<<grid, dim3(GEMV_THREADS), smem, stream>>>(ka);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

template <int TYPE, int NU>
static int launch_dot_nb(int nb, const GemvKernelArgs &ka, dim3 grid, size_t smem, hipStream_t stream) {
    if (nb == 4) return launch_dot<TYPE, 4, NU>(ka, grid, smem, stream);
    if (nb == 2) return launch_dot<TYPE, 2, NU>(ka, grid, smem, stream);
    return launch_dot<TYPE, 1, NU>(ka, grid, smem, stream);
}

static int n_compute_units() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) n = p.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

// All matrices of `a` are tiled K-quants of one type.
static int gemv_kquant(const GemvArgs &a, hipStream_t stream) {
    const int type = a.mat[0].type;
    const int nsb = a.K / QK_K, NU = a.epi == EPI_SWIGLU ? 2 : 1;
    const size_t row_stride = (size_t)nsb * (type == MESH_Q4_K ? Q4K_TILE_BYTES : Q6K_TILE_BYTES);
    GemvKernelArgs ka{};
    int total_rows = 0;
    for (int i = 0; i < a.n_mat; ++i) {
        const int begin = (NU == 2 && i == 1) ? 0 : total_rows;     // gate and up share tile-row indices
        ka.tile_begin[i] = begin;
        ka.wbase[i] = static_cast<const uint8_t *>(a.mat[i].W) - (size_t)begin * row_stride;
        ka.y[i] = a.mat[i].y;
        ka.bias[i] = a.mat[i].bias;
        ka.M[i] = a.mat[i].M;
        ka.ldy[i] = a.mat[i].ldy;
        if (!(NU == 2 && i == 1)) total_rows += (a.mat[i].M + TILE_ROWS - 1) / TILE_ROWS;
    }
    const int n_mat_k = NU == 2 ? 1 : a.n_mat;      // boundaries the kernel searches
    for (int i = n_mat_k; i < 4; ++i) ka.tile_begin[i] = total_rows;
    if (NU == 2) ka.tile_begin[1] = total_rows;
    ka.n_mat = n_mat_k;
    // unused boundary slots must compare as "beyond the end"
    for (int i = n_mat_k; i < 3; ++i) { ka.tile_begin[i] = total_rows; }
    ka.ldx = a.ldx;
    ka.K = a.K;
    ka.norm_w = a.norm_w;
    ka.eps = a.eps;
    ka.ldres = a.ldres;
    ka.epi = a.epi;
    const int KS = nsb < GEMV_WAVES ? nsb : GEMV_WAVES;
    ka.ks = KS;
    const int n_pairs = a.expert_ids ? a.n_pairs : 1;
    if (a.expert_ids) {
        if (a.n_pairs <= 0 || a.x_div <= 0 || a.epi == EPI_RESIDUAL) return fail(MESH_ERR_INVALID, "gemv: bad expert-indirection arguments");
        ka.expert_ids = a.expert_ids;
        ka.expert_stride = (size_t)tiled_bytes(type, a.mat[0].M, a.K);
        ka.x_div = a.x_div;
    }
    // tile-rows per workgroup: spread over the CUs, bounded by the LDS partial buffer
    const int ncu = std::max(1, n_compute_units() / n_pairs);
    int rows_per_wg = (total_rows + ncu - 1) / ncu;
    rows_per_wg = std::max(1, std::min(rows_per_wg, MAX_ROWS_X_KS / KS));
    const int grid = (total_rows + rows_per_wg - 1) / rows_per_wg;
    const int rows_max = (total_rows + grid - 1) / grid;
    if (dot_smem_bytes(type, 1, a.K, rows_max, KS, NU) > LDS_LIMIT) return fail(MESH_ERR_UNSUPPORTED, "gemv: row length %d does not fit LDS", a.K);
    if (a.expert_ids) {
        // every pair is its own single-column product
        ka.x = a.x;
        const size_t smem = dot_smem_bytes(type, 1, a.K, rows_max, KS, NU);
        const dim3 g((unsigned)grid, (unsigned)n_pairs);
        if (type == MESH_Q4_K) return NU == 2 ? launch_dot_nb<MESH_Q4_K, 2>(1, ka, g, smem, stream) : launch_dot_nb<MESH_Q4_K, 1>(1, ka, g, smem, stream);
        return NU == 2 ? launch_dot_nb<MESH_Q6_K, 2>(1, ka, g, smem, stream) : launch_dot_nb<MESH_Q6_K, 1>(1, ka, g, smem, stream);
    }
    int t = 0;
    while (t < a.T) {
        const int left = a.T - t;
        int nb = left >= 4 ? 4 : left >= 2 ? 2 : 1;
        while (nb > 1 && dot_smem_bytes(type, nb, a.K, rows_max, KS, NU) > LDS_LIMIT) nb >>= 1;
        GemvKernelArgs kb = ka;
        kb.x = a.x + (size_t)t * a.ldx;
        kb.residual = a.residual ? a.residual + (size_t)t * a.ldres : nullptr;
        for (int i = 0; i < a.n_mat; ++i)
            if (kb.y[i]) kb.y[i] = a.mat[i].y + (size_t)t * a.mat[i].ldy;
        const size_t smem = dot_smem_bytes(type, nb, a.K, rows_max, KS, NU);
        int rc;
        const dim3 g((unsigned)grid);
        if (type == MESH_Q4_K) rc = NU == 2 ? launch_dot_nb<MESH_Q4_K, 2>(nb, kb, g, smem, stream) : launch_dot_nb<MESH_Q4_K, 1>(nb, kb, g, smem, stream);
        else rc = NU == 2 ? launch_dot_nb<MESH_Q6_K, 2>(nb, kb, g, smem, stream) : launch_dot_nb<MESH_Q6_K, 1>(nb, kb, g, smem, stream);
        if (rc != MESH_OK) return rc;
        t += nb;
    }
    return MESH_OK;
}

int gemv(const GemvArgs &a, hipStream_t stream) {
    if (a.n_mat < 1 || a.n_mat > 3 || !a.x || a.K <= 0 || a.T < 0)
        return fail(MESH_ERR_INVALID, "gemv: bad arguments (n_mat %d, K %d, T %d)", a.n_mat, a.K, a.T);
    if (a.epi == EPI_SWIGLU && a.n_mat != 2) return fail(MESH_ERR_INVALID, "gemv: swiglu needs exactly gate and up");
    if (a.epi == EPI_SWIGLU && a.mat[0].M != a.mat[1].M) return fail(MESH_ERR_INVALID, "gemv: gate and up differ in rows");
    if (a.epi == EPI_RESIDUAL && !a.residual) return fail(MESH_ERR_INVALID, "gemv: residual epilogue without residual");
    if ((a.ldx % 4) || (reinterpret_cast<uintptr_t>(a.x) & 15)) return fail(MESH_ERR_INVALID, "gemv: x must be 16-byte aligned");
    bool uniform = true;
    for (int i = 0; i < a.n_mat; ++i) {
        const GemvMat &m = a.mat[i];
        if (!m.W || m.M <= 0 || (!m.y && !(a.epi == EPI_SWIGLU && i == 1)))
            return fail(MESH_ERR_INVALID, "gemv: matrix %d incomplete", i);
        if (row_bytes(m.type, a.K) < 0)
            return fail(MESH_ERR_INVALID, "gemv: K=%d is not a whole number of type-%d blocks", a.K, m.type);
        // one launch handles matrices of one kernel family: q4_K, q6_K, or "everything else"
        const bool same = type_is_tiled(m.type) ? m.type == a.mat[0].type : !type_is_tiled(a.mat[0].type);
        uniform = uniform && same;
    }
    if (a.T == 0) return MESH_OK;
    if (a.expert_ids && !(uniform && type_is_tiled(a.mat[0].type)))
        return fail(MESH_ERR_UNSUPPORTED, "gemv: expert indirection needs K-quant expert matrices of one type");
    if (uniform) return type_is_tiled(a.mat[0].type) ? gemv_kquant(a, stream) : gemv_generic(a, stream);
    if (a.epi == EPI_SWIGLU) return fail(MESH_ERR_UNSUPPORTED, "gemv: gate and up of different types");
    // mixed types side by side (a q/k/v group whose v is q6_K): one launch per run of equal family
    int i = 0;
    while (i < a.n_mat) {
        int j = i + 1;
        auto fam = [](int t) { return type_is_tiled(t) ? t : -1; };
        while (j < a.n_mat && fam(a.mat[j].type) == fam(a.mat[i].type)) ++j;
        GemvArgs b = a;
        b.n_mat = j - i;
        for (int k = i; k < j; ++k) b.mat[k - i] = a.mat[k];
        const int rc = type_is_tiled(b.mat[0].type) ? gemv_kquant(b, stream) : gemv_generic(b, stream);
        if (rc != MESH_OK) return rc;
        i = j;
    }
    return MESH_OK;
}

}  // namespace mesh
