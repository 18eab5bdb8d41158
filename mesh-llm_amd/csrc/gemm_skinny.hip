// Skinny GEMM for batched decode: Y[T][M] = W[M][K] . X[T][K] with 4 <= T <= a few dozen tokens, W a tiled
// q4_K / q6_K matrix, on the integer matrix cores.
//
// Between the mat-vec kernel (gemv.hip: one dot4 chain per activation column, so the weights' integer work is
// repeated per token) and the prefill GEMM (gemm.hip: 128x128 output tiles, far too few workgroups when T is
// small) sits the batch of decode steps.  The weight stream is organised exactly as in the mat-vec kernel -- a
// workgroup owns a few tile-rows (16 rows each), its waves split K and each keeps several weight tiles in flight --
// and so is the arithmetic: activations are 16-bit fixed point per 32-element block (x ~ d_b * (256 hi + lo), hi and lo
// int8), the raw 4- / 6-bit quants are the other integer operand, and the block scales meet the integer sums in f32.
// Only the dot products move from v_dot4 to v_mfma_i32_16x16x32_i8, 16 token columns at a time:
//
//   * A operand = activations (rows = 16 tokens), B operand = weights (columns = the 16 rows of a tile), so lane
//     (m = l % 16, g = l / 16) supplies 8 k-slots of token m and of weight row m, and receives the sums of tokens
//     4g..4g+3 for ITS OWN weight row m: the sub-block scales a lane applies are those of the row whose header it
//     holds, and only the activation scales fan out (one 16-byte load of four tokens' block scales per sub-block).
//   * q4_K: one MFMA pair (hi plane, lo plane) per 32-element sub-block; sum = (I_hi << 8) + I_lo, scaled by
//     d * sc_s * dx_s[token].  The "- dmin * m_s * sum(x)" term of all 8 sub-blocks is itself a small matrix product
//     over s and runs on v_mfma_f32_16x16x4_f32 (two per super-block), straight into the f32 accumulator.
//   * q6_K: scales cover 16 elements, i.e. two lane groups of a 32-element block each, so a block takes two MFMAs per
//     plane, each with the other scale group's weights zeroed; the -32 offset is folded into the quants (int8 q - 32).
//
// A tile arrives with the mat-vec kernel's dense lane mapping (whole cache lines per wave instruction) and passes
// through a wave-private LDS slot to reach the MFMA lanes.
//
// Activation layout ("q16", produced by quant16_k8 below and by the decode attention kernels, q16.hpp) of a block of 16 tokens:
//   planes  [K/8][16 tokens][16 B]: {hi[0..7], lo[0..7]} of elements 8q..8q+7 of the token
//   dx      [K/32][16 tokens] f32: block scale;  sx [K/32][16 tokens] f32: block sum of x (= dx * sum of quants)
// The 16 lanes of a lane group read 256 contiguous bytes of planes; columns beyond T hold whatever they held (an MFMA
// row never mixes tokens, and those rows are not stored).
//
// Same math as ggml's mul_mat for K-quant weights (ggml_vec_dot_q4_K_q8_K / q6_K in third_party/llama.cpp
// ggml-cpu/quants.c, reached from rpc_server::graph_compute, patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451)
// -- an integer dot per sub-block, scales applied in f32 -- with 16-bit instead of 8-bit activations.

#include "gemm.hpp"
#include "gemv_device.hpp"

namespace mesh {

constexpr int SK_THREADS = 512;
constexpr int SK_WAVES = SK_THREADS / 64;
constexpr int SK_DEPTH_Q4 = 4;            // weight tiles a wave keeps in flight (2304 B each)
constexpr int SK_DEPTH_Q6 = 2;            // q6_K tiles are 3360 B
constexpr int SK_NT = 16;                 // activation columns per launch (one MFMA M)
constexpr int SK_SEGS_MAX = 4;            // (tile-row, matrix) segments one wave may own
constexpr size_t SK_LDS_LIMIT = 160 * 1024;
constexpr int SK_ITEM_INTS = (2 + SKINNY_ITEM_PAIRS + 3) / 4 * 4;   // expert, n, pairs, padded to a multiple of 4 (moe_item_ints)

typedef int i4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));

struct SkinnyKernelArgs {
    const uint8_t *wbase[3];      // matrix base minus its first tile-row, so a global tile-row index addresses it
    int tile_begin[4];            // first global tile-row of each matrix; unused slots hold the total
    float *y[3];
    const float *bias[3];
    int M[3];
    int ldy[3];
    int K, T;
    const float *residual;
    int ldres;
    int epi;
    int ks;                       // waves along K
    GemvRope rope;                // rope.pos / rope.seq point at the launch's first column
    int kind[3];
    // expert launches: blockIdx.y = work item {expert, n, pair[0..n)} of SK_ITEM_INTS int32 (n <= 16 pairs of one expert);
    // the matrices are that expert's (expert_stride bytes apart), slot j's activation column is pair[j] / x_div and its
    // output row pair[j]
    const int32_t *items, *n_items;
    size_t expert_stride;
    int x_div;
};

__device__ __forceinline__ long pack64(uint32_t lo, uint32_t hi) { return (long)(((unsigned long long)hi << 32) | lo); }

// Where a lane finds its activations.  Plain launches: token column m = lane % 16 of the launch's block of 16.  Expert
// launches (mixture of experts): the column is whatever (token or pair) the work item lists for slot m, in whichever block
// of 16 it lives, so every lane carries its own base pointers.
struct XSrc {
    const uint4 *pl;        // record (k-group g, own column), super-block 0
    const float *dxa, *dxb; // block-scale entries this lane fetches for the wave's table: block lane / 8, slots 2 (lane % 8) and + 1
    const float *sx;        // block sum (block 0, own column)
    __device__ __forceinline__ static XSrc plain(const uint8_t *xq, int K, int lane) {
        XSrc x;
        x.pl = reinterpret_cast<const uint4 *>(xq) + (lane >> 4) * 16 + (lane & 15);
        x.dxa = reinterpret_cast<const float *>(xq + (size_t)K * 32) + 2 * lane;
        x.dxb = x.dxa + 1;
        x.sx = reinterpret_cast<const float *>(xq + (size_t)K * 34) + (lane & 15);
        return x;
    }
    // col: this lane's column (slot lane % 16 of the item); cola / colb: the columns of slots 2 (lane % 8) and + 1
    __device__ __forceinline__ static XSrc gathered(const uint8_t *xq, int K, int lane, int col, int cola, int colb) {
        const size_t bb = (size_t)K * 36;
        XSrc x;
        const uint8_t *blk = xq + (size_t)(col >> 4) * bb;
        x.pl = reinterpret_cast<const uint4 *>(blk) + (lane >> 4) * 16 + (col & 15);
        x.sx = reinterpret_cast<const float *>(blk + (size_t)K * 34) + (col & 15);
        x.dxa = reinterpret_cast<const float *>(xq + (size_t)(cola >> 4) * bb + (size_t)K * 32) + (lane >> 3) * 16 + (cola & 15);
        x.dxb = reinterpret_cast<const float *>(xq + (size_t)(colb >> 4) * bb + (size_t)K * 32) + (lane >> 3) * 16 + (colb & 15);
        return x;
    }
};

// A operands (activation planes) of one super-block for this lane, the same for both weight types: 32-element block s,
// elements 32s + 8g .. + 7 of the lane's column as {hi8 (x, y), lo8 (z, w)}.  The block scales take a detour through a
// wave-private LDS table ([8 blocks][16 slots] f32, two of them): a lane needs those of four columns for every block -- 32
// registers per super-block if kept in registers -- but the table is only 128 floats, two entries per lane.
struct XFrags {
    uint4 p[8];
    float2 dxpre;      // this lane's two entries of the super-block's scale table
    float sxa, sxb;    // q4_K: block sums of the lane's column, blocks g and g + 4 (operands of the minimum-term MFMAs)
    template <bool SUMS, bool GATHER>
    __device__ __forceinline__ void load(const XSrc &x, int sb, int lane) {
        const uint4 *pl = x.pl + (size_t)sb * 512;
#pragma unroll
        for (int s = 0; s < 8; ++s) p[s] = ldg<uint4>(pl + s * 64);
        if (GATHER) {
            dxpre.x = ldg<float>(x.dxa + (size_t)sb * 128);
            dxpre.y = ldg<float>(x.dxb + (size_t)sb * 128);
        } else {
            dxpre = ldg<float2>(x.dxa + (size_t)sb * 128);
        }
        if (SUMS) {
            const float *sxp = x.sx + (size_t)sb * 128;
            sxa = ldg<float>(sxp + (lane >> 4) * 16);
            sxb = ldg<float>(sxp + ((lane >> 4) + 4) * 16);
        }
    }
};

// The LDS unit executes a wave's accesses in order; the fences only keep the compiler from reordering them.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One tile: dense-mapped registers -> wave-private LDS slot (same arrangement as in memory) -> the view of lane (m, g):
// row m's header and the quants of elements 32s + 8g .. + 7, s = 0..7, of that row.
template <int TYPE> struct TileView;

constexpr int Q4_ROW = 144;                       // LDS stride of a row's 128 quant bytes
constexpr int Q6_ROW_L = 144, Q6_ROW_H = 80;      // of a row's 128 low-nibble bytes and 64 upper-bit bytes
constexpr int Q6_LDS_QH = 16 * Q6_ROW_L, Q6_LDS_SC = Q6_LDS_QH + 16 * Q6_ROW_H, Q6_LDS_D = Q6_LDS_SC + 256;
constexpr int LDS_TILE_Q4 = 256 + 16 * Q4_ROW, LDS_TILE_Q6 = Q6_LDS_D + 32;

template <> struct TileView<MESH_Q4_K> {
    uint4 hdr;
    uint2 v[4];        // chunk c: bytes 8g .. 8g + 7 of qs[32c ..]: low nibbles block 2c, high nibbles block 2c + 1
    __device__ __forceinline__ void stage(const TileRegs<MESH_Q4_K> &R, uint8_t *slot, int lane) {
        const int m = lane & 15, g = lane >> 4;
        wave_lds_sync();                                          // the previous tile's reads are issued before these writes
        // (rows of quants are Q4_ROW bytes apart in LDS, not 128: the 16 rows a read instruction touches then fall into
        // different banks instead of two)
        if ((lane & 3) == 0) *reinterpret_cast<uint4 *>(slot + (lane >> 2) * 16) = R.hdr;
        *reinterpret_cast<uint4 *>(slot + 256 + (lane >> 2) * Q4_ROW + (lane & 3) * 32) = R.qa;
        *reinterpret_cast<uint4 *>(slot + 256 + (lane >> 2) * Q4_ROW + (lane & 3) * 32 + 16) = R.qb;
        wave_lds_sync();
        hdr = *reinterpret_cast<const uint4 *>(slot + m * 16);
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = *reinterpret_cast<const uint2 *>(slot + 256 + m * Q4_ROW + 32 * c + 8 * g);
    }
};

template <> struct TileView<MESH_Q6_K> {
    uint2 la[2], lb[2], qh[2];     // half n: ql[64n + 8g ..], ql[64n + 32 + 8g ..], qh[32n + 8g ..], 8 bytes each
    uint4 sc;
    uint32_t d;
    __device__ __forceinline__ void stage(const TileRegs<MESH_Q6_K> &R, uint8_t *slot, int lane) {
        const int m = lane & 15, g = lane >> 4;
        const int r = lane >> 2, c = lane & 3, n = c >> 1, u = c & 1;
        wave_lds_sync();
        *reinterpret_cast<uint4 *>(slot + r * Q6_ROW_L + 64 * n + 16 * u) = R.qla;
        *reinterpret_cast<uint4 *>(slot + r * Q6_ROW_L + 64 * n + 32 + 16 * u) = R.qlb;
        *reinterpret_cast<uint4 *>(slot + Q6_LDS_QH + r * Q6_ROW_H + 32 * n + 16 * u) = R.qh;
        if (c == 0) {
            *reinterpret_cast<uint4 *>(slot + Q6_LDS_SC + r * 16) = R.sc;
            *reinterpret_cast<uint16_t *>(slot + Q6_LDS_D + r * 2) = (uint16_t)R.d;
        }
        wave_lds_sync();
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            la[h] = *reinterpret_cast<const uint2 *>(slot + m * Q6_ROW_L + 64 * h + 8 * g);
            lb[h] = *reinterpret_cast<const uint2 *>(slot + m * Q6_ROW_L + 64 * h + 32 + 8 * g);
            qh[h] = *reinterpret_cast<const uint2 *>(slot + Q6_LDS_QH + m * Q6_ROW_H + 32 * h + 8 * g);
        }
        sc = *reinterpret_cast<const uint4 *>(slot + Q6_LDS_SC + m * 16);
        d = *reinterpret_cast<const uint16_t *>(slot + Q6_LDS_D + m * 2);
    }
};

// acc[i] += sum over the tile's 256 elements of w[row m][k] * x[token 4g + i][k]
__device__ __forceinline__ void tile_mac(const TileView<MESH_Q4_K> &V, const XFrags &X, const float *dxt, int lane, f4_t &acc) {
    const int g = lane >> 4;
    const float d = f16_bits_to_f32((uint16_t)(V.hdr.x & 0xFFFFu)), dmin = f16_bits_to_f32((uint16_t)(V.hdr.x >> 16));
    // 6-bit scales / minima of the 8 sub-blocks as bytes (get_scale_min_k4 of ggml-quants.c)
    const uint32_t sc_lo = V.hdr.y & 0x3F3F3F3Fu, sc_hi = (V.hdr.w & 0x0F0F0F0Fu) | ((V.hdr.y >> 2) & 0x30303030u);
    const uint32_t mn_lo = V.hdr.z & 0x3F3F3F3Fu, mn_hi = ((V.hdr.w >> 4) & 0x0F0F0F0Fu) | ((V.hdr.z >> 2) & 0x30303030u);
    const i4_t zero = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int c = s >> 1, h = s & 1;
        const long w = pack64((V.v[c].x >> (4 * h)) & 0x0F0F0F0Fu, (V.v[c].y >> (4 * h)) & 0x0F0F0F0Fu);
        const i4_t ih = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(X.p[s].x, X.p[s].y), w, zero, 0, 0, 0);
        const i4_t il = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(X.p[s].z, X.p[s].w), w, zero, 0, 0, 0);
        const float ds = d * (float)(((s < 4 ? sc_lo : sc_hi) >> (8 * (s & 3))) & 0xFFu);
        const f4_t dx = *reinterpret_cast<const f4_t *>(dxt + s * 16 + 4 * g);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf((float)((ih[i] << 8) + il[i]) * dx[i], ds, acc[i]);
    }
    // - dmin * m_s * sum(x_s), s = 0..7: a [16 tokens x 8] . [8 x 16 rows] product in f32
    const float nma = -dmin * (float)((mn_lo >> (8 * g)) & 0xFFu), nmb = -dmin * (float)((mn_hi >> (8 * g)) & 0xFFu);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X.sxa, nma, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X.sxb, nmb, acc, 0, 0, 0);
}

__device__ __forceinline__ uint32_t q6_to_i8(uint32_t v) {       // bytes 0..63 -> int8 bytes v - 32
    return ((v | 0x80808080u) - 0x20202020u) ^ 0x80808080u;
}

// q6_K scales cover 16 elements: of a 32-element block, lane groups 0-1 hold the first scale group and 2-3 the second, so
// the block takes two MFMAs per plane, each with the other group's weights zeroed.
__device__ __forceinline__ void tile_mac(const TileView<MESH_Q6_K> &V, const XFrags &X, const float *dxt, int lane, f4_t &acc) {
    const int g = lane >> 4;
    const float d = f16_bits_to_f32((uint16_t)V.d);
    const uint32_t scs[4] = {V.sc.x, V.sc.y, V.sc.z, V.sc.w};
    const uint32_t first = g < 2 ? 0xFFFFFFFFu : 0u;
    const i4_t zero = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int n = s >> 2, t4 = s & 3;
        const uint2 l = (t4 & 1) ? V.lb[n] : V.la[n], q = V.qh[n];
        uint32_t w0, w1;
        if (t4 == 0) { w0 = (l.x & 0x0F0F0F0Fu) | ((q.x << 4) & 0x30303030u); w1 = (l.y & 0x0F0F0F0Fu) | ((q.y << 4) & 0x30303030u); }
        else if (t4 == 1) { w0 = (l.x & 0x0F0F0F0Fu) | ((q.x << 2) & 0x30303030u); w1 = (l.y & 0x0F0F0F0Fu) | ((q.y << 2) & 0x30303030u); }
        else if (t4 == 2) { w0 = ((l.x >> 4) & 0x0F0F0F0Fu) | (q.x & 0x30303030u); w1 = ((l.y >> 4) & 0x0F0F0F0Fu) | (q.y & 0x30303030u); }
        else { w0 = ((l.x >> 4) & 0x0F0F0F0Fu) | ((q.x >> 2) & 0x30303030u); w1 = ((l.y >> 4) & 0x0F0F0F0Fu) | ((q.y >> 2) & 0x30303030u); }
        w0 = q6_to_i8(w0);
        w1 = q6_to_i8(w1);
        const uint32_t a0 = w0 & first, a1 = w1 & first;
        const long wa = pack64(a0, a1), wb = pack64(w0 ^ a0, w1 ^ a1);
        const long xh = pack64(X.p[s].x, X.p[s].y), xl = pack64(X.p[s].z, X.p[s].w);
        const i4_t ah = __builtin_amdgcn_mfma_i32_16x16x32_i8(xh, wa, zero, 0, 0, 0);
        const i4_t al = __builtin_amdgcn_mfma_i32_16x16x32_i8(xl, wa, zero, 0, 0, 0);
        const i4_t bh = __builtin_amdgcn_mfma_i32_16x16x32_i8(xh, wb, zero, 0, 0, 0);
        const i4_t bl = __builtin_amdgcn_mfma_i32_16x16x32_i8(xl, wb, zero, 0, 0, 0);
        const uint32_t scw = scs[s >> 1] >> (16 * (s & 1));             // scale groups 2s and 2s + 1
        const float dsa = d * (float)(int8_t)(scw & 0xFFu), dsb = d * (float)(int8_t)((scw >> 8) & 0xFFu);
        const f4_t dx = *reinterpret_cast<const f4_t *>(dxt + s * 16 + 4 * g);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float t = fmaf((float)((bh[i] << 8) + bl[i]), dsb, (float)((ah[i] << 8) + al[i]) * dsa);
            acc[i] = fmaf(t, dx[i], acc[i]);
        }
    }
}

// One workgroup's share of a launch.  bx: its index among the workgroups of its launch part (the whole launch, or one side of
// a pair launch); by: its work item (expert launches).
template <int TYPE, int NU, int SEGS, bool GROUPED>
__device__ __forceinline__ void skinny_workgroup(int bx, int by, const uint8_t *p_xq, const uint8_t *p_w0, const uint8_t *p_w1, const uint8_t *p_w2, int p_K,
                                                 int p_ks, unsigned p_begins, unsigned p_split, const SkinnyKernelArgs &a) {
    // (leading scalar arguments: preloaded into SGPRs, see gemv.hip.  p_begins = first tile-row of matrix 1 | of matrix 2
    // << 16; p_split = tile-rows per workgroup | workgroups with one more << 16, computed on the host: no division and
    // no grid-size load stand before the first weight load)
    const int p_begin1 = (int)(p_begins & 0xFFFFu), p_begin2 = (int)(p_begins >> 16);
    // expert launches: this workgroup's item; workgroups past the item count have nothing to do
    int it_n = SK_NT, it_pair = 0;
    if (GROUPED) {
        // item count and item are fetched together (the item buffer holds max_items entries, so the read is in bounds even
        // for a workgroup past the count): one memory round trip before the first weight load instead of two
        const int32_t *it = a.items + (size_t)by * SK_ITEM_INTS;
        const int n_live = ldg<int>(a.n_items);
        const int2 head = ldg<int2>(reinterpret_cast<const int2 *>(it));
        const int slot_l = (int)(threadIdx.x & 15);
        const int p_mine = ldg<int>(it + 2 + slot_l), p_first = ldg<int>(it + 2);
        if (by >= n_live) return;
        const size_t eoff = (size_t)head.x * a.expert_stride;
        p_w0 += eoff; p_w1 += eoff; p_w2 += eoff;
        it_n = head.y;
        it_pair = slot_l < it_n ? p_mine : p_first;              // unused slots repeat slot 0: computed, never stored
    }
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int TB = TileRegs<TYPE>::BYTES;
    constexpr int SLOT = ((TYPE == MESH_Q4_K ? LDS_TILE_Q4 : LDS_TILE_Q6) + 255) / 256 * 256;
    constexpr int SK_DEPTH = TYPE == MESH_Q4_K ? SK_DEPTH_Q4 : SK_DEPTH_Q6;
    constexpr bool SUMS = TYPE == MESH_Q4_K;
    constexpr int WAVE_LDS = SLOT + 2 * 512;                               // tile slot + two scale tables
    float *red = reinterpret_cast<float *>(smem + SK_WAVES * WAVE_LDS);   // [KS][rows_here][NU][16 rows][16 tokens]
    const int K = p_K, nsb = K / QK_K;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // scalar: tile addresses become SGPR base + lane offset
    uint8_t *slot = smem + wave * WAVE_LDS;
    float *dxt = reinterpret_cast<float *>(slot + SLOT);                   // [2][8][16]
    const int m = lane & 15, g = lane >> 4;
    const int KS = p_ks, LK = __builtin_ctz((unsigned)KS), RS = SK_WAVES >> LK;      // KS is a power of two
    const int ks = wave & (KS - 1), rs = wave >> LK;
    const int sq = (int)(p_split & 0xFFFFu), sr = (int)(p_split >> 16);
    const int tr0 = bx * sq + (bx < sr ? bx : sr);
    const int rows_here = sq + (bx < sr ? 1 : 0);
    const int n_i = rs < RS ? (nsb - ks + KS - 1) >> LK : 0;        // super-blocks of this wave (ks < KS <= nsb)
    const size_t row_stride = (size_t)nsb * TB;
    // flat tile index f -> (ii, seg); seg -> (local tile-row j, matrix u)
    auto seg_valid = [&](int seg) { return rs + RS * (seg / NU) < rows_here; };
    auto tile_ptr = [&](int ii, int seg) -> const uint8_t * {
        const int tr = tr0 + rs + RS * (seg / NU);
        int mi = seg % NU;
        if (NU == 1) mi = (tr >= p_begin1 ? 1 : 0) + (tr >= p_begin2 ? 1 : 0);
        // (offsets added under conditions: an indexed kernel-argument array is fetched with a load, and a three-way
        // select of preloaded pointers becomes a table in scratch memory)
        const uint8_t *wb = p_w0 + (mi >= 1 ? p_w1 - p_w0 : (ptrdiff_t)0) + (mi >= 2 ? p_w2 - p_w1 : (ptrdiff_t)0);
        return wb + (size_t)tr * row_stride + (size_t)(ks + KS * ii) * TB;
    };
    // flat tile index f = ii * SEGS + seg, invalid segments included as bubbles; a wave without a valid first
    // segment has nothing at all
    const int total = seg_valid(0) ? n_i * SEGS : 0;

    XSrc xs;
    if (GROUPED) {
        const int col = it_pair / a.x_div;
        xs = XSrc::gathered(p_xq, K, lane, col, __shfl(col, 2 * (lane & 7)), __shfl(col, 2 * (lane & 7) + 1));
    } else {
        xs = XSrc::plain(p_xq, K, lane);
    }
    TileRegs<TYPE> ring[SK_DEPTH];
    XFrags X[2];
    f4_t D[SEGS];
#pragma unroll
    for (int s = 0; s < SEGS; ++s) D[s] = f4_t{0.f, 0.f, 0.f, 0.f};

    // Loads are never under a branch of their own: an index past the end or an invalid segment is clamped to a tile
    // the wave owns (a cache hit).  The compiler then knows exactly how many loads are in flight at every point
    // and waits for one tile without draining the others; a load under a branch makes it assume the worst at the
    // join, which in an unrolled pipeline degenerates to waiting for everything.
    auto load_tile = [&](TileRegs<TYPE> &dst, int f, int seg) {
        const bool ok = f < total && seg_valid(seg);
        dst.load(tile_ptr(ok ? f / SEGS : n_i - 1, ok ? seg : 0), lane);
    };
    // the scale table of super-block ii goes to LDS table ii & 1 before the super-block's first tile
    auto publish = [&](const XFrags &x, int b) {
        wave_lds_sync();
        *reinterpret_cast<float2 *>(dxt + b * 128 + 2 * lane) = x.dxpre;
        wave_lds_sync();
    };
    auto sb_of = [&](int ii) { return ks + KS * (ii < n_i ? ii : n_i - 1); };
    if (total > 0) {
        // Loads return in issue order, so waiting for a load also waits for everything issued before it.  Every wait
        // in the loop below is therefore for something issued at least two super-blocks earlier: activations are
        // fetched two super-blocks ahead, BEFORE the weight tile issued in the same iteration, and a weight tile is
        // consumed SK_DEPTH - 1 iterations after its load was issued.
        X[0].template load<SUMS, GROUPED>(xs, sb_of(0), lane);
        X[1].template load<SUMS, GROUPED>(xs, sb_of(1), lane);
#pragma unroll
        for (int f = 0; f < SK_DEPTH; ++f) load_tile(ring[f], f, f % SEGS);
        constexpr int RB0 = SEGS >= SK_DEPTH ? 1 : SK_DEPTH / SEGS;
        constexpr int RB = RB0 < 2 ? 2 : RB0;              // super-blocks per unrolled block: even, so the activation buffer of a step is static
        constexpr int UB = RB * SEGS;                        // tiles per unrolled block, a multiple of the ring depth
        static_assert(UB % SK_DEPTH == 0 && RB % 2 == 0, "ring slots and activation buffers must be static inside a block");
        // Software pipeline: the LDS round trip of tile f + 1 (its view) is started before tile f is multiplied.
        TileView<TYPE> cur, nxt;
        cur.stage(ring[0], slot, lane);
        load_tile(ring[0], SK_DEPTH, SK_DEPTH % SEGS);
        for (int blk = 0; blk * RB < n_i; ++blk) {
#pragma unroll
            for (int q = 0; q < UB; ++q) {
                const int r = q / SEGS, seg = q % SEGS;
                const int ii = blk * RB + r, f = ii * SEGS + seg;
                nxt.stage(ring[(q + 1) % SK_DEPTH], slot, lane);
                if (seg == 0) publish(X[r % 2], r % 2);
                if (ii < n_i && seg_valid(seg)) tile_mac(cur, X[r % 2], dxt + (r % 2) * 128, lane, D[seg]);
                // last segment of a super-block: its activation buffer is free for the one after next
                if (seg == SEGS - 1) X[r % 2].template load<SUMS, GROUPED>(xs, sb_of(ii + 2), lane);
                load_tile(ring[(q + 1) % SK_DEPTH], f + 1 + SK_DEPTH, (q + 1 + SK_DEPTH) % SEGS);
                cur = nxt;
                __builtin_amdgcn_sched_barrier(0);      // tiles stay in program order: hoisted loads would only cost registers
            }
        }
    }

    // partial sums of this wave: D[seg][i] belongs to weight row m, token 4g + i of segment seg
#pragma unroll
    for (int seg = 0; seg < SEGS; ++seg) {
        if (total > 0 && seg_valid(seg)) {
            const int j = rs + RS * (seg / NU), u = seg % NU;
#pragma unroll
            for (int i = 0; i < 4; ++i) red[((((size_t)ks * rows_here + j) * NU + u) * 16 + m) * 16 + 4 * g + i] = D[seg][i];
        }
    }
    __syncthreads();

    // outputs of this workgroup: rows_here x 16 rows x T columns
    for (int o = tid; o < rows_here * 16 * SK_NT; o += SK_THREADS) {
        const int t = o % SK_NT, r = (o / SK_NT) % 16, j = o / (SK_NT * 16);
        if (t >= (GROUPED ? it_n : a.T)) continue;
        // output row of column t: the token itself, or the pair the item lists for this slot
        const size_t orow = GROUPED ? (size_t)a.items[(size_t)by * SK_ITEM_INTS + 2 + t] : (size_t)t;
        const int tr = tr0 + j;
        int mi = 0;
        if (NU == 1) mi = (tr >= a.tile_begin[1] ? 1 : 0) + (tr >= a.tile_begin[2] ? 1 : 0);
        const int row = (tr - a.tile_begin[mi]) * TILE_ROWS + r;
        if (row >= a.M[mi]) continue;
        float s0 = 0.f, s1 = 0.f;
        for (int k2 = 0; k2 < KS; ++k2) {
            s0 += red[((((size_t)k2 * rows_here + j) * NU + 0) * 16 + r) * 16 + t];
            if (NU == 2) s1 += red[((((size_t)k2 * rows_here + j) * NU + 1) * 16 + r) * 16 + t];
        }
        if (a.bias[mi]) s0 += a.bias[mi][row];
        if (!GROUPED && NU == 1 && a.rope.pos && a.kind[mi] != GEMV_KIND_PLAIN) {
            // q / k / v row of a token (see gemv.hpp): rotate q and k with the neighbouring row, k and v go to the cache
            const int kind = a.kind[mi], hd = a.rope.head_dim;
            const int head = row / hd, dd = row - head * hd;
            const int pos = a.rope.pos[t];
            float val = s0;
            if (kind != GEMV_KIND_V && dd < a.rope.n_rot) {
                float sp = 0.f;
                for (int k2 = 0; k2 < KS; ++k2) sp += red[((((size_t)k2 * rows_here + j) * NU + 0) * 16 + (r ^ 1)) * 16 + t];
                if (a.bias[mi]) sp += a.bias[mi][row ^ 1];
                float sn, cs;
                sincosf((float)pos * a.rope.inv_freq[dd >> 1], &sn, &cs);
                val = (dd & 1) ? sp * sn + s0 * cs : s0 * cs - sp * sn;
            }
            if (kind == GEMV_KIND_Q) {
                a.y[mi][(size_t)t * a.ldy[mi] + row] = val;
            } else {
                uint16_t *cache = kind == GEMV_KIND_K ? a.rope.kcache : a.rope.vcache;
                cache[(((size_t)a.rope.seq[t] * a.rope.n_kv + head) * a.rope.n_ctx + pos) * hd + dd] = f32_to_f16_bits(val);
            }
            continue;
        }
        float out;
        if (NU == 2) {
            if (a.bias[1]) s1 += a.bias[1][row];
            out = (s0 / (1.0f + expf(-s0))) * s1;
        } else if (a.epi == EPI_RESIDUAL) {
            out = a.residual[orow * a.ldres + row] + s0;
        } else {
            out = s0;
        }
        a.y[mi][orow * a.ldy[mi] + row] = out;
    }
}

template <int TYPE, int NU, int SEGS, bool GROUPED>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(const uint8_t *p_xq, const uint8_t *p_w0, const uint8_t *p_w1, const uint8_t *p_w2, int p_K,
                                                                 int p_ks, int p_rows, unsigned p_begins, unsigned p_split,
                                                                 const SkinnyKernelArgs a) {
    (void)p_rows;
    skinny_workgroup<TYPE, NU, SEGS, GROUPED>((int)blockIdx.x, (int)blockIdx.y, p_xq, p_w0, p_w1, p_w2, p_K, p_ks, p_begins, p_split, a);
}

// Two launches over the same activations as one: the first grid_a workgroups run a q4_K launch, the others a q6_K launch (the q
// and k projections of a layer next to a q6_K v projection).  Same arithmetic per workgroup as the separate launches.
template <int SEGS_A, int SEGS_B>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_pair_kernel(const uint8_t *p_xq, const uint8_t *p_w0, const uint8_t *p_w1, int p_K, int p_ks_a,
                                                                      int p_ks_b, int grid_a, unsigned p_begins, unsigned p_split_a, unsigned p_split_b,
                                                                      const uint8_t *p_wb, const SkinnyKernelArgs a, const SkinnyKernelArgs b) {
    const int bx = (int)blockIdx.x;
    if (bx < grid_a) skinny_workgroup<MESH_Q4_K, 1, SEGS_A, false>(bx, 0, p_xq, p_w0, p_w1, p_w1, p_K, p_ks_a, p_begins, p_split_a, a);
    else skinny_workgroup<MESH_Q6_K, 1, SEGS_B, false>(bx - grid_a, 0, p_xq, p_wb, p_wb, p_wb, p_K, p_ks_b, 0xFFFFFFFFu, p_split_b, b);
}

template <int TYPE, int NU, int SEGS, bool GROUPED>
static int launch_skinny(const SkinnyKernelArgs &ka, const uint8_t *xq, int grid, int grid_y, size_t smem, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_skinny_kernel<TYPE, NU, SEGS, GROUPED>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)SK_LDS_LIMIT));
        attr_set = true;
    }
    MESH_LAUNCH((gemm_skinny_kernel<TYPE, NU, SEGS, GROUPED>), dim3((unsigned)grid, (unsigned)grid_y), dim3(SK_THREADS), smem, stream, 
        xq, ka.wbase[0], ka.wbase[1] ? ka.wbase[1] : ka.wbase[0], ka.wbase[2] ? ka.wbase[2] : ka.wbase[0], ka.K, ka.ks, ka.tile_begin[3],
        (unsigned)ka.tile_begin[1] | ((unsigned)ka.tile_begin[2] << 16), (unsigned)(ka.tile_begin[3] / grid) | ((unsigned)(ka.tile_begin[3] % grid) << 16), ka);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

template <int TYPE, int NU>
static int launch_skinny_segs(int segs, const SkinnyKernelArgs &ka, const uint8_t *xq, int grid, int grid_y, size_t smem, hipStream_t stream) {
    if (ka.items) {
        if (segs <= 2) return launch_skinny<TYPE, NU, 2, true>(ka, xq, grid, grid_y, smem, stream);
        return launch_skinny<TYPE, NU, 4, true>(ka, xq, grid, grid_y, smem, stream);
    }
    if (segs <= 1) return launch_skinny<TYPE, NU, NU, false>(ka, xq, grid, 1, smem, stream);       // NU == 2 needs two segments at least
    if (segs <= 2) return launch_skinny<TYPE, NU, 2, false>(ka, xq, grid, 1, smem, stream);
    return launch_skinny<TYPE, NU, 4, false>(ka, xq, grid, 1, smem, stream);
}

static int skinny_n_cu() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) n = p.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

size_t q16_block_bytes(int K) { return (size_t)K * 32 + 2 * (size_t)(K / 32) * 16 * sizeof(float); }

// What a launch over the matrices of `a` (tiled K-quants of one type) needs, before the token block is chosen
struct SkinnyLaunch {
    SkinnyKernelArgs ka;
    int type, NU, KS, grid, segs;
    size_t smem;
};
static int skinny_prepare(const SkinnyArgs &a, SkinnyLaunch &L) {
    const int type = a.mat[0].type;
    const int nsb = a.K / QK_K, NU = a.epi == EPI_SWIGLU ? 2 : 1;
    L.type = type; L.NU = NU;
    const int tile_bytes = type == MESH_Q4_K ? Q4K_TILE_BYTES : Q6K_TILE_BYTES;
    const size_t row_stride = (size_t)nsb * tile_bytes;
    SkinnyKernelArgs &ka = L.ka;
    ka = SkinnyKernelArgs{};
    int total_rows = 0;
    for (int i = 0; i < a.n_mat; ++i) {
        const int begin = (NU == 2 && i == 1) ? 0 : total_rows;     // gate and up share tile-row indices
        ka.tile_begin[i] = begin;
        ka.wbase[i] = static_cast<const uint8_t *>(a.mat[i].W) - (size_t)begin * row_stride;
        ka.y[i] = a.mat[i].y;
        ka.bias[i] = a.mat[i].bias;
        ka.M[i] = a.mat[i].M;
        ka.ldy[i] = a.mat[i].ldy;
        ka.kind[i] = a.kind[i];
        if (!(NU == 2 && i == 1)) total_rows += (a.mat[i].M + TILE_ROWS - 1) / TILE_ROWS;
    }
    const int n_bound = NU == 2 ? 1 : a.n_mat;          // matrix boundaries the kernel searches
    for (int i = n_bound; i < 4; ++i) ka.tile_begin[i] = total_rows;
    ka.K = a.K;
    ka.ldres = a.ldres; ka.epi = a.epi;
    ka.rope = a.rope;
    const bool grouped = a.items != nullptr;
    ka.items = a.items; ka.n_items = a.n_items; ka.expert_stride = (size_t)tiled_bytes(type, a.mat[0].M, a.K); ka.x_div = a.x_div > 0 ? a.x_div : 1;
    // How the 8 waves of a workgroup are arranged (KS along K, a power of two: the kernel splits its waves with shifts; the
    // other 8 / KS along tile-rows) decides how many workgroups the launch has and how long each wave's chain of tiles is.
    // A workgroup costs a fixed start-up / reduction time plus its waves' tiles one after the other, and workgroups beyond one
    // per CU wait for a second round: take the arrangement for which that estimate is smallest (ties: more waves along K).
    // Expert matrices are short in K (a few super-blocks) and their launches have many items, so they get few, long
    // workgroups: at most 2 waves along K and as many tile-rows as a workgroup can hold.
    const int ncu = skinny_n_cu();
    int KS = 1, rows_per_wg = 1;
    {
        double best = 1e30;
        for (int ks = 1; ks <= (grouped ? 2 : SK_WAVES) && ks <= nsb; ks *= 2) {
            const int rs = SK_WAVES / ks;
            const int cap = std::max(1, SK_SEGS_MAX / NU) * rs;
            const int rpw = grouped ? cap : std::max(1, std::min((total_rows + ncu - 1) / ncu, cap));
            const int wgs = (total_rows + rpw - 1) / rpw;
            const int rounds = grouped ? 1 : (wgs + ncu - 1) / ncu;
            const int tiles = ((rpw + rs - 1) / rs) * NU * ((nsb + ks - 1) / ks);
            const double cost = rounds * (5.0 + 0.9 * tiles);
            if (cost <= best) { best = cost; KS = ks; rows_per_wg = rpw; }
        }
    }
    const int RS = SK_WAVES / KS;
    ka.ks = KS;
    L.KS = KS;
    L.grid = (total_rows + rows_per_wg - 1) / rows_per_wg;
    const int rows_max = (total_rows + L.grid - 1) / L.grid;
    L.segs = ((rows_max + RS - 1) / RS) * NU;           // per wave
    if (L.segs > SK_SEGS_MAX) return fail(MESH_ERR_UNSUPPORTED, "gemm_skinny: %d segments per wave", L.segs);
    if (total_rows > 0xFFFF) return fail(MESH_ERR_UNSUPPORTED, "gemm_skinny: %d tile-rows in one launch", total_rows);
    const int lds_tile = ((type == MESH_Q4_K ? LDS_TILE_Q4 : LDS_TILE_Q6) + 255) / 256 * 256;
    L.smem = (size_t)SK_WAVES * (lds_tile + 2 * 512) + sizeof(float) * (size_t)KS * rows_max * NU * 16 * SK_NT;
    if (L.smem > SK_LDS_LIMIT) return fail(MESH_ERR_UNSUPPORTED, "gemm_skinny: %zu bytes of LDS needed", L.smem);
    return MESH_OK;
}
// the kernel arguments for token block t / 16 of the call
static SkinnyKernelArgs skinny_block(const SkinnyArgs &a, const SkinnyLaunch &L, int t) {
    SkinnyKernelArgs kb = L.ka;
    kb.T = std::min(SK_NT, a.T - t);
    if (kb.rope.pos) { kb.rope.pos += t; kb.rope.seq += t; }
    kb.residual = a.residual ? a.residual + (size_t)t * a.ldres : nullptr;
    for (int i = 0; i < a.n_mat; ++i)
        if (kb.y[i]) kb.y[i] = a.mat[i].y + (size_t)t * a.mat[i].ldy;
    return kb;
}

// all matrices of `a` are tiled K-quants of one type
static int skinny_one_type(const SkinnyArgs &a, hipStream_t stream) {
    SkinnyLaunch L;
    int rc = skinny_prepare(a, L);
    if (rc != MESH_OK) return rc;
    const int type = L.type, NU = L.NU, segs = L.segs, grid = L.grid;
    const size_t smem = L.smem;
    if (a.items) {
        SkinnyKernelArgs ka = L.ka;
        ka.T = SK_NT;
        if (type == MESH_Q4_K) return NU == 2 ? launch_skinny_segs<MESH_Q4_K, 2>(segs, ka, a.xq, grid, a.max_items, smem, stream) : launch_skinny_segs<MESH_Q4_K, 1>(segs, ka, a.xq, grid, a.max_items, smem, stream);
        return NU == 2 ? launch_skinny_segs<MESH_Q6_K, 2>(segs, ka, a.xq, grid, a.max_items, smem, stream) : launch_skinny_segs<MESH_Q6_K, 1>(segs, ka, a.xq, grid, a.max_items, smem, stream);
    }
    for (int t = 0; t < a.T; t += SK_NT) {
        const SkinnyKernelArgs kb = skinny_block(a, L, t);
        const uint8_t *xq = a.xq + (size_t)(t / SK_NT) * q16_block_bytes(a.K);
        if (type == MESH_Q4_K) rc = NU == 2 ? launch_skinny_segs<MESH_Q4_K, 2>(segs, kb, xq, grid, 1, smem, stream) : launch_skinny_segs<MESH_Q4_K, 1>(segs, kb, xq, grid, 1, smem, stream);
        else rc = NU == 2 ? launch_skinny_segs<MESH_Q6_K, 2>(segs, kb, xq, grid, 1, smem, stream) : launch_skinny_segs<MESH_Q6_K, 1>(segs, kb, xq, grid, 1, smem, stream);
        if (rc != MESH_OK) return rc;
    }
    return MESH_OK;
}

template <int SEGS_A, int SEGS_B>
static int launch_pair(const SkinnyKernelArgs &ka, const SkinnyKernelArgs &kb, const uint8_t *xq, int grid_a, int grid_b, size_t smem, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_skinny_pair_kernel<SEGS_A, SEGS_B>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)SK_LDS_LIMIT));
        attr_set = true;
    }
    MESH_LAUNCH((gemm_skinny_pair_kernel<SEGS_A, SEGS_B>), dim3((unsigned)(grid_a + grid_b)), dim3(SK_THREADS), smem, stream, xq, ka.wbase[0],
                ka.wbase[1] ? ka.wbase[1] : ka.wbase[0], ka.K, ka.ks, kb.ks, grid_a, (unsigned)ka.tile_begin[1] | ((unsigned)ka.tile_begin[2] << 16),
                (unsigned)(ka.tile_begin[3] / grid_a) | ((unsigned)(ka.tile_begin[3] % grid_a) << 16),
                (unsigned)(kb.tile_begin[3] / grid_b) | ((unsigned)(kb.tile_begin[3] % grid_b) << 16), kb.wbase[0], ka, kb);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// `qa`: one or two q4_K matrices, `qb`: one q6_K matrix, same activations, plain-store epilogues (with or without RoPE): one
// launch whose first workgroups are qa's and whose last are qb's.  MESH_ERR_UNSUPPORTED when the shapes do not fit (the
// caller then launches them one after the other).
static int skinny_pair(const SkinnyArgs &qa, const SkinnyArgs &qb, hipStream_t stream) {
    SkinnyLaunch A, B;
    int rc = skinny_prepare(qa, A);
    if (rc != MESH_OK) return rc;
    if ((rc = skinny_prepare(qb, B)) != MESH_OK) return rc;
    if (B.segs > 2) return MESH_ERR_UNSUPPORTED;
    const size_t smem = std::max(A.smem, B.smem);
    const int sa = A.segs <= 1 ? 1 : A.segs <= 2 ? 2 : 4;
    for (int t = 0; t < qa.T; t += SK_NT) {
        const SkinnyKernelArgs ka = skinny_block(qa, A, t), kb = skinny_block(qb, B, t);
        const uint8_t *xq = qa.xq + (size_t)(t / SK_NT) * q16_block_bytes(qa.K);
        if (B.segs <= 1) rc = sa == 1 ? launch_pair<1, 1>(ka, kb, xq, A.grid, B.grid, smem, stream) : sa == 2 ? launch_pair<2, 1>(ka, kb, xq, A.grid, B.grid, smem, stream)
                                                                                                            : launch_pair<4, 1>(ka, kb, xq, A.grid, B.grid, smem, stream);
        else rc = sa == 1 ? launch_pair<1, 2>(ka, kb, xq, A.grid, B.grid, smem, stream) : sa == 2 ? launch_pair<2, 2>(ka, kb, xq, A.grid, B.grid, smem, stream)
                                                                                                  : launch_pair<4, 2>(ka, kb, xq, A.grid, B.grid, smem, stream);
        if (rc != MESH_OK) return rc;
    }
    return MESH_OK;
}

// ---- producer of the q16 activation layout -------------------------------------------------------------------------
// y = quantise(x[t] * rsqrt(mean(x[t]^2) + eps) * w), or with w == null just quantise(x[t]).  Workgroup (chunk, t)
// quantises elements [1024 chunk, 1024 chunk + 1024) of token t, eight per lane; four neighbouring lanes share a
// 32-element block, as in the mat-vec kernel's prologue (gemv_device.hpp: x_quantise), with the same rounding.  With a
// norm every workgroup of a token sums the whole row's squares itself (the row is a few KB in L2): no second launch.
// Token slots beyond T are not written: an MFMA row never mixes tokens, and the GEMM does not store those rows.
constexpr int Q16_THREADS = 128;
// 8 consecutive values v of token slot t (elements i .. i + 7 of a row of n) into the q16 block at yb; the four lanes of a
// 32-element block (tid % 4) share its scale.  Every lane of the wave calls it (`live` guards the stores).
__device__ __forceinline__ void q16_store8(const float (&v)[8], int i, int t, int n, uint8_t *yb, bool live, int tid) {
    uint4 *planes = reinterpret_cast<uint4 *>(yb);                                  // record (k / 8, t) at planes[(k / 8) * 16 + t]
    float *dxp = reinterpret_cast<float *>(yb + (size_t)n * 32), *sxp = reinterpret_cast<float *>(yb + (size_t)n * 34);
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[e]));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    const float inv = amax > 0.f ? XQ_LEVELS / amax : 0.f;
    int hi[8], lo[8], isum = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int q = __float2int_rn(v[e] * inv);
        lo[e] = ((q + 128) & 0xFF) - 128;
        hi[e] = (q - lo[e]) >> 8;
        isum += q;
    }
    isum += __shfl_xor(isum, 1);
    isum += __shfl_xor(isum, 2);
    if (live) {
        planes[(size_t)(i >> 3) * 16 + t] = make_uint4(pack_bytes(hi[0], hi[1], hi[2], hi[3]), pack_bytes(hi[4], hi[5], hi[6], hi[7]),
                                                       pack_bytes(lo[0], lo[1], lo[2], lo[3]), pack_bytes(lo[4], lo[5], lo[6], lo[7]));
        if ((tid & 3) == 0) {
            const float d = amax / XQ_LEVELS;
            dxp[(i >> 5) * 16 + t] = d;
            sxp[(i >> 5) * 16 + t] = d * (float)isum;
        }
    }
}

__global__ __launch_bounds__(Q16_THREADS) void quant16_kernel(const float *__restrict__ x, const float *__restrict__ w, float eps, int n,
                                                              uint8_t *__restrict__ y) {
    __shared__ float red[Q16_THREADS / 64];
    const int tid = threadIdx.x, tok = blockIdx.y, t = tok & 15;
    uint8_t *yb = y + (size_t)(tok >> 4) * ((size_t)n * 36);
    const float *xt = x + (size_t)tok * n;
    const int i = blockIdx.x * (Q16_THREADS * 8) + tid * 8;
    const bool live = i < n;
    float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0, g0 = make_float4(1.f, 1.f, 1.f, 1.f), g1 = g0;
    if (live) {
        a0 = *reinterpret_cast<const float4 *>(xt + i);
        a1 = *reinterpret_cast<const float4 *>(xt + i + 4);
        if (w) { g0 = *reinterpret_cast<const float4 *>(w + i); g1 = *reinterpret_cast<const float4 *>(w + i + 4); }
    }
    float scale = 1.f;
    if (w) {
        float ss = 0.f;
        for (int k = tid * 4; k < n; k += Q16_THREADS * 4) {
            const float4 v = *reinterpret_cast<const float4 *>(xt + k);
            ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int k = 0; k < Q16_THREADS / 64; ++k) tot += red[k];
        scale = 1.0f / sqrtf(tot / (float)n + eps);
    }
    const float v[8] = {a0.x * scale * g0.x, a0.y * scale * g0.y, a0.z * scale * g0.z, a0.w * scale * g0.w,
                        a1.x * scale * g1.x, a1.y * scale * g1.y, a1.z * scale * g1.z, a1.w * scale * g1.w};
    q16_store8(v, i, t, n, yb, live, tid);
}

int quant16_k8(const float *x, const float *w, float eps, int T, int n, uint8_t *y, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (n % 32) return fail(MESH_ERR_INVALID, "quant16_k8: row length %d not a multiple of 32", n);
    MESH_LAUNCH(quant16_kernel, dim3((unsigned)((n + Q16_THREADS * 8 - 1) / (Q16_THREADS * 8)), (unsigned)T), dim3(Q16_THREADS), 0, stream, x, w, eps, n, y);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// The combine step of a mixture-of-experts layer and the q16 activations of the next layer's first projections in one
// launch, one workgroup per token: x[t] += sum_s w[t][s] * y[t * top_k + s] (the sums of moe_combine_kernel, in its order),
// then y16 = quantise(rms_norm(x[t]) * norm_w) exactly as quant16_kernel forms it: the same partition of the row for the sum
// of squares (its thread j of 128 adds the float4 groups j, j + 128, ... in turn) and the same 8 values per lane for the blocks;
// the row and the groups' squares pass through LDS.  Rows of up to Q16F_MAX_N elements.
constexpr int Q16F_MAX_N = 8192, Q16F_THREADS = 512;
__global__ __launch_bounds__(Q16F_THREADS) void moe_combine_quant16_kernel(float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ wts,
                                                                           int top_k, const float *__restrict__ norm_w, float eps, int n,
                                                                           uint8_t *__restrict__ yq) {
    __shared__ float red[Q16_THREADS / 64];
    __shared__ __align__(16) float row[Q16F_MAX_N];
    __shared__ float psq[Q16F_MAX_N / 4];
    const int tid = threadIdx.x, tok = blockIdx.x, t = tok & 15;
    uint8_t *yb = yq + (size_t)(tok >> 4) * ((size_t)n * 36);
    float *xt = x + (size_t)tok * n;
    // one float4 group per thread and pass: the new hidden state and the group's sum of squares
    for (int g = tid; g < n / 4; g += Q16F_THREADS) {
        float4 acc = *reinterpret_cast<const float4 *>(xt + 4 * g);
        for (int s = 0; s < top_k; ++s) {
            const float ws = wts[(size_t)tok * top_k + s];
            const float4 v = *reinterpret_cast<const float4 *>(y + ((size_t)tok * top_k + s) * n + 4 * g);
            acc.x = fmaf(ws, v.x, acc.x); acc.y = fmaf(ws, v.y, acc.y); acc.z = fmaf(ws, v.z, acc.z); acc.w = fmaf(ws, v.w, acc.w);
        }
        *reinterpret_cast<float4 *>(xt + 4 * g) = acc;
        *reinterpret_cast<float4 *>(row + 4 * g) = acc;
        psq[g] = (acc.x * acc.x + acc.y * acc.y) + (acc.z * acc.z + acc.w * acc.w);
    }
    __syncthreads();
    // the row's sum of squares in quant16_kernel's order: thread j of 128 adds its groups j, j + 128, ... one after the other
    if (tid < Q16_THREADS) {
        float ss = 0.f;
        for (int g = tid; g < n / 4; g += Q16_THREADS) ss += psq[g];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        if ((tid & 63) == 0) red[tid >> 6] = ss;
    }
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int k = 0; k < Q16_THREADS / 64; ++k) tot += red[k];
    const float scale = 1.0f / sqrtf(tot / (float)n + eps);
    for (int i0 = 0; i0 < n; i0 += Q16F_THREADS * 8) {
        const int i = i0 + tid * 8;
        const bool live = i < n;
        float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0, g0 = make_float4(1.f, 1.f, 1.f, 1.f), g1 = g0;
        if (live) {
            a0 = *reinterpret_cast<const float4 *>(row + i);
            a1 = *reinterpret_cast<const float4 *>(row + i + 4);
            g0 = *reinterpret_cast<const float4 *>(norm_w + i);
            g1 = *reinterpret_cast<const float4 *>(norm_w + i + 4);
        }
        const float v[8] = {a0.x * scale * g0.x, a0.y * scale * g0.y, a0.z * scale * g0.z, a0.w * scale * g0.w,
                            a1.x * scale * g1.x, a1.y * scale * g1.y, a1.z * scale * g1.z, a1.w * scale * g1.w};
        q16_store8(v, i, t, n, yb, live, tid);
    }
}

bool moe_combine_quant16_supported(int n) { return n % 32 == 0 && n <= Q16F_MAX_N; }

int moe_combine_quant16(float *x, const float *y, const float *w, int T, int n, int top_k, const float *norm_w, float eps, uint8_t *yq, hipStream_t stream) {
    if (T <= 0) return MESH_OK;
    if (!moe_combine_quant16_supported(n) || !norm_w || !yq) return fail(MESH_ERR_INVALID, "moe_combine_quant16: row length %d", n);
    MESH_LAUNCH(moe_combine_quant16_kernel, dim3((unsigned)T), dim3(Q16F_THREADS), 0, stream, x, y, w, top_k, norm_w, eps, n, yq);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// ---- producers of the k8-major f16 activation layout (read by the large-tile GEMM, gemm.hip) ------------------------
// Tokens are grouped in blocks of 16 columns, and within a block the 8 consecutive k of every column sit together:
// element (t, k) of block b = t / 16 is at ((b * K/8 + k/8) * 16 + t % 16) * 8 + k % 8.
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
// saturating, like gemm.hip's pack_h2; a clamped pair is noted in the caller's counter (mesh_common.hpp), if it has one
__device__ __forceinline__ uint32_t sk_pack_h2(unsigned *sat, float a, float b) {
    note_f16_clamp(sat, a, b);
    const h2_t h = {(_Float16)__builtin_amdgcn_fmed3f(a, -65504.f, 65504.f), (_Float16)__builtin_amdgcn_fmed3f(b, -65504.f, 65504.f)};
    return __builtin_bit_cast(uint32_t, h);
}

// y = f16(x[t] * rsqrt(mean(x[t]^2) + eps) * w), or with w == null just f16(x[t]); one workgroup per token slot of the
// padded batch (slots >= T write zeros).
__global__ __launch_bounds__(256) void to_k8_kernel(const float *__restrict__ x, const float *__restrict__ w, float eps, int T, int n,
                                                    _Float16 *__restrict__ y, unsigned *sat) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    _Float16 *yb = y + (size_t)(t / 16) * 16 * n + (size_t)(t % 16) * 8;        // element (t, k) at yb + (k / 8) * 128 + k % 8
    if (t >= T) {
        for (int i = tid * 8; i < n; i += 2048) *reinterpret_cast<uint4 *>(yb + (size_t)(i >> 3) * 128) = make_uint4(0u, 0u, 0u, 0u);
        return;
    }
    const float *xt = x + (size_t)t * n;
    constexpr int RC = 4;                                   // rows of up to 2048 * RC elements stay in registers: one read
    if (w && n <= 2048 * RC) {
        float4 v[RC][2], g[RC][2];
#pragma unroll
        for (int j = 0; j < RC; ++j) {
            const int i = tid * 8 + j * 2048;
            const bool live = i < n;
            v[j][0] = live ? *reinterpret_cast<const float4 *>(xt + i) : make_float4(0.f, 0.f, 0.f, 0.f);
            v[j][1] = live ? *reinterpret_cast<const float4 *>(xt + i + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int j = 0; j < RC; ++j) {
            const int i = tid * 8 + j * 2048;
            const bool live = i < n;
            g[j][0] = live ? *reinterpret_cast<const float4 *>(w + i) : make_float4(0.f, 0.f, 0.f, 0.f);
            g[j][1] = live ? *reinterpret_cast<const float4 *>(w + i + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < RC; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) ss += (v[j][h].x * v[j][h].x + v[j][h].y * v[j][h].y) + (v[j][h].z * v[j][h].z + v[j][h].w * v[j][h].w);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        const float sc = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)n + eps);
#pragma unroll
        for (int j = 0; j < RC; ++j) {
            const int i = tid * 8 + j * 2048;
            if (i >= n) continue;
            const float4 v0 = v[j][0], v1 = v[j][1], g0 = g[j][0], g1 = g[j][1];
            *reinterpret_cast<uint4 *>(yb + (size_t)(i >> 3) * 128) =
                make_uint4(sk_pack_h2(sat, v0.x * sc * g0.x, v0.y * sc * g0.y), sk_pack_h2(sat, v0.z * sc * g0.z, v0.w * sc * g0.w),
                           sk_pack_h2(sat, v1.x * sc * g1.x, v1.y * sc * g1.y), sk_pack_h2(sat, v1.z * sc * g1.z, v1.w * sc * g1.w));
        }
        return;
    }
    float scale = 1.f;
    if (w) {
        float ss = 0.f;
        for (int i = tid * 4; i < n; i += 1024) {
            const float4 v = *reinterpret_cast<const float4 *>(xt + i);
            ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        scale = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)n + eps);
    }
    for (int i = tid * 8; i < n; i += 2048) {
        const float4 v0 = *reinterpret_cast<const float4 *>(xt + i), v1 = *reinterpret_cast<const float4 *>(xt + i + 4);
        float4 g0 = make_float4(1.f, 1.f, 1.f, 1.f), g1 = g0;
        if (w) { g0 = *reinterpret_cast<const float4 *>(w + i); g1 = *reinterpret_cast<const float4 *>(w + i + 4); }
        *reinterpret_cast<uint4 *>(yb + (size_t)(i >> 3) * 128) =
            make_uint4(sk_pack_h2(sat, v0.x * scale * g0.x, v0.y * scale * g0.y), sk_pack_h2(sat, v0.z * scale * g0.z, v0.w * scale * g0.w),
                       sk_pack_h2(sat, v1.x * scale * g1.x, v1.y * scale * g1.y), sk_pack_h2(sat, v1.z * scale * g1.z, v1.w * scale * g1.w));
    }
}

// The same for prefill-sized calls, one workgroup of 1024 threads per 8 tokens: thread (token = tid % 8, group lane = tid / 8)
// keeps NG groups of 8 consecutive elements of its token's row in registers (one read of the row), the squares are added per
// token over the workgroup, and 8 neighbouring threads write one contiguous 128-byte run of the block -- the per-token
// kernel above writes 16 bytes every 256.  Rows of 1024 * NG elements.  The sum of squares is taken in another order than in
// to_k8_kernel, so the scale can differ from that kernel's in its last bit.
constexpr int K8B_THREADS = 1024, K8B_WAVES = K8B_THREADS / 64, K8B_TOK = 8, K8B_LANES = K8B_THREADS / K8B_TOK;
template <int NG>
__global__ __launch_bounds__(K8B_THREADS) void to_k8_block_kernel(const float *__restrict__ x, const float *__restrict__ w, float eps, int T,
                                                                  _Float16 *__restrict__ y, unsigned *sat) {
    constexpr int n = 8 * K8B_LANES * NG;
    __shared__ float s_ss[K8B_WAVES][K8B_TOK];
    const int tid = threadIdx.x, tl = tid % K8B_TOK, gl = tid / K8B_TOK, lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.x * K8B_TOK + tl;
    const bool live = t < T;
    const float *xt = x + (size_t)(live ? t : 0) * n;
    float4 v[NG][2];
#pragma unroll
    for (int j = 0; j < NG; ++j) {
        const int i = 8 * (gl + K8B_LANES * j);
        v[j][0] = live ? *reinterpret_cast<const float4 *>(xt + i) : make_float4(0.f, 0.f, 0.f, 0.f);
        v[j][1] = live ? *reinterpret_cast<const float4 *>(xt + i + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NG; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h) ss += (v[j][h].x * v[j][h].x + v[j][h].y * v[j][h].y) + (v[j][h].z * v[j][h].z + v[j][h].w * v[j][h].w);
    // the eight lanes of a wave that hold the same token, then the waves in order
    ss += __shfl_xor(ss, 8);
    ss += __shfl_xor(ss, 16);
    ss += __shfl_xor(ss, 32);
    if (lane < K8B_TOK) s_ss[wave][lane] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int k = 0; k < K8B_WAVES; ++k) tot += s_ss[k][tl];
    const float sc = 1.0f / sqrtf(tot / (float)n + eps);
    _Float16 *yb = y + (size_t)(t / 16) * 16 * n + (size_t)(t % 16) * 8;        // element (t, k) at yb + (k / 8) * 128 + k % 8
#pragma unroll
    for (int j = 0; j < NG; ++j) {
        const int i = 8 * (gl + K8B_LANES * j);
        const float4 g0 = *reinterpret_cast<const float4 *>(w + i), g1 = *reinterpret_cast<const float4 *>(w + i + 4);
        const float4 v0 = v[j][0], v1 = v[j][1];
        // (slots past the last token hold zeros: v is zero there)
        *reinterpret_cast<uint4 *>(yb + (size_t)(i >> 3) * 128) =
            make_uint4(sk_pack_h2(sat, v0.x * sc * g0.x, v0.y * sc * g0.y), sk_pack_h2(sat, v0.z * sc * g0.z, v0.w * sc * g0.w),
                       sk_pack_h2(sat, v1.x * sc * g1.x, v1.y * sc * g1.y), sk_pack_h2(sat, v1.z * sc * g1.z, v1.w * sc * g1.w));
    }
}
constexpr int K8B_MIN_TOKENS = 64;       // below: the per-token kernel (decode batches keep its bits)

int rmsnorm_f16_k8(const float *x, const float *w, float eps, int T, int n, _Float16 *y, hipStream_t stream, unsigned *sat) {
    if (T <= 0) return MESH_OK;
    if (n % 8) return fail(MESH_ERR_INVALID, "rmsnorm_f16_k8: row length %d not a multiple of 8", n);
    if (w && T >= K8B_MIN_TOKENS && n % (8 * K8B_LANES) == 0) {
        // (the grid covers the padded batch: slots past the last token of the last block of 16 are written as zeros)
        const dim3 grid((unsigned)((T + 15) / 16 * 16 / K8B_TOK)), block(K8B_THREADS);
        switch (n / (8 * K8B_LANES)) {
            case 2: MESH_LAUNCH(to_k8_block_kernel<2>, grid, block, 0, stream, x, w, eps, T, y, sat); MESH_LAUNCH_CHECK(); return MESH_OK;
            case 4: MESH_LAUNCH(to_k8_block_kernel<4>, grid, block, 0, stream, x, w, eps, T, y, sat); MESH_LAUNCH_CHECK(); return MESH_OK;
            case 5: MESH_LAUNCH(to_k8_block_kernel<5>, grid, block, 0, stream, x, w, eps, T, y, sat); MESH_LAUNCH_CHECK(); return MESH_OK;
            case 8: MESH_LAUNCH(to_k8_block_kernel<8>, grid, block, 0, stream, x, w, eps, T, y, sat); MESH_LAUNCH_CHECK(); return MESH_OK;
            default: break;     // other row lengths: the per-token kernel
        }
    }
    MESH_LAUNCH(to_k8_kernel, dim3((unsigned)((T + 15) / 16 * 16)), dim3(256), 0, stream, x, w, eps, T, n, y, sat);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// The gathered form with one workgroup per block of 16 slots: each wave first sums the squares of four of the block's rows,
// then thread (k8 group, slot) converts 8 values at a time, so that 16 neighbouring threads write one contiguous 256-byte
// run of the block.  The sum of squares is taken in another order than in to_k8_kernel (one wave per row instead of four),
// so the scale can differ from that kernel's in its last bit.
__global__ __launch_bounds__(256) void gather_k8_kernel(const float *__restrict__ x, const float *__restrict__ w, float eps, int n,
                                                        _Float16 *__restrict__ y, const int32_t *__restrict__ row_of_slot, int row_div, unsigned *sat) {
    __shared__ float s_scale[16];
    __shared__ int s_row[16];
    const int blk = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < 16) {
        const int r = row_of_slot[blk * 16 + tid];
        s_row[tid] = r < 0 ? -1 : r / row_div;
    }
    __syncthreads();
    for (int i = 0; i < 4; ++i) {
        const int sl = wave * 4 + i, row = s_row[sl];
        float ss = 0.f;
        if (row >= 0) {
            const float *xt = x + (size_t)row * n;
            for (int k = lane * 8; k < n; k += 512) {
                const float4 a = *reinterpret_cast<const float4 *>(xt + k), b = *reinterpret_cast<const float4 *>(xt + k + 4);
                ss += (a.x * a.x + a.y * a.y) + (a.z * a.z + a.w * a.w);
                ss += (b.x * b.x + b.y * b.y) + (b.z * b.z + b.w * b.w);
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        if (lane == 0) s_scale[sl] = 1.0f / sqrtf(ss / (float)n + eps);
    }
    __syncthreads();
    const int sl = tid & 15, row = s_row[sl];
    const float sc = s_scale[sl];
    _Float16 *yb = y + (size_t)blk * 16 * n + (size_t)sl * 8;
    for (int k8 = tid >> 4; k8 < n / 8; k8 += 16) {
        uint4 o = make_uint4(0u, 0u, 0u, 0u);
        if (row >= 0) {
            const float *xt = x + (size_t)row * n + k8 * 8;
            const float4 v0 = *reinterpret_cast<const float4 *>(xt), v1 = *reinterpret_cast<const float4 *>(xt + 4);
            const float4 g0 = *reinterpret_cast<const float4 *>(w + k8 * 8), g1 = *reinterpret_cast<const float4 *>(w + k8 * 8 + 4);
            o = make_uint4(sk_pack_h2(sat, v0.x * sc * g0.x, v0.y * sc * g0.y), sk_pack_h2(sat, v0.z * sc * g0.z, v0.w * sc * g0.w),
                           sk_pack_h2(sat, v1.x * sc * g1.x, v1.y * sc * g1.y), sk_pack_h2(sat, v1.z * sc * g1.z, v1.w * sc * g1.w));
        }
        *reinterpret_cast<uint4 *>(yb + (size_t)k8 * 128) = o;
    }
}

int rmsnorm_f16_k8_gather(const float *x, const float *w, float eps, const int32_t *row_of_slot, int row_div, int n_slots, int n, _Float16 *y, hipStream_t stream,
                          unsigned *sat) {
    if (n_slots <= 0) return MESH_OK;
    if (n % 8 || n_slots % 16 || !row_of_slot || row_div < 1 || !w) return fail(MESH_ERR_INVALID, "rmsnorm_f16_k8_gather: bad arguments (row length %d, %d slots)", n, n_slots);
    MESH_LAUNCH(gather_k8_kernel, dim3((unsigned)(n_slots / 16)), dim3(256), 0, stream, x, w, eps, n, y, row_of_slot, row_div, sat);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

// out (k8-major) = f16( silu(gate) * up ): one workgroup per token, padding tokens of the last block write zeros
__global__ __launch_bounds__(256) void swiglu_k8_kernel(const float *__restrict__ g, const float *__restrict__ u, int T, int n,
                                                        _Float16 *__restrict__ y, unsigned *sat) {
    const int t = blockIdx.x, tid = threadIdx.x;
    _Float16 *yb = y + (size_t)(t >> 4) * 16 * n + (size_t)(t & 15) * 8;
    if (t >= T) {
        for (int i = tid * 8; i < n; i += 2048) *reinterpret_cast<uint4 *>(yb + (size_t)(i >> 3) * 128) = make_uint4(0, 0, 0, 0);
        return;
    }
    const float *gt = g + (size_t)t * n, *ut = u + (size_t)t * n;
    for (int i = tid * 8; i < n; i += 2048) {
        const float4 a0 = *reinterpret_cast<const float4 *>(gt + i), a1 = *reinterpret_cast<const float4 *>(gt + i + 4);
        const float4 b0 = *reinterpret_cast<const float4 *>(ut + i), b1 = *reinterpret_cast<const float4 *>(ut + i + 4);
        auto f = [](float a, float b) { return a / (1.0f + expf(-a)) * b; };
        uint4 o;
        o.x = sk_pack_h2(sat, f(a0.x, b0.x), f(a0.y, b0.y));
        o.y = sk_pack_h2(sat, f(a0.z, b0.z), f(a0.w, b0.w));
        o.z = sk_pack_h2(sat, f(a1.x, b1.x), f(a1.y, b1.y));
        o.w = sk_pack_h2(sat, f(a1.z, b1.z), f(a1.w, b1.w));
        *reinterpret_cast<uint4 *>(yb + (size_t)(i >> 3) * 128) = o;
    }
}

int swiglu_f16_k8(const float *gate, const float *up, int T, int n, _Float16 *y, hipStream_t stream, unsigned *sat) {
    if (T <= 0) return MESH_OK;
    if (n % 8) return fail(MESH_ERR_INVALID, "swiglu_f16_k8: row length %d not a multiple of 8", n);
    MESH_LAUNCH(swiglu_k8_kernel, dim3((unsigned)((T + 15) / 16 * 16)), dim3(256), 0, stream, gate, up, T, n, y, sat);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

int pack_f16_k8(const float *x, int T, int n, _Float16 *y, hipStream_t stream, unsigned *sat) {
    return rmsnorm_f16_k8(x, nullptr, 0.f, T, n, y, stream, sat);
}

int gemm_skinny(const SkinnyArgs &a, hipStream_t stream) {
    if (a.n_mat < 1 || a.n_mat > 3 || !a.xq || a.T <= 0 || a.K <= 0) return fail(MESH_ERR_INVALID, "gemm_skinny: bad arguments");
    if (a.K % QK_K || (reinterpret_cast<uintptr_t>(a.xq) & 15))
        return fail(MESH_ERR_INVALID, "gemm_skinny: K %d must be a multiple of 256 and the activations 16-byte aligned", a.K);
    if (a.epi == EPI_SWIGLU && (a.n_mat != 2 || a.mat[0].M != a.mat[1].M || a.mat[0].type != a.mat[1].type))
        return fail(MESH_ERR_INVALID, "gemm_skinny: SwiGLU needs a gate and an up matrix of equal shape and type");
    if (a.epi == EPI_RESIDUAL && !a.residual) return fail(MESH_ERR_INVALID, "gemm_skinny: residual epilogue without residual");
    if (a.rope.pos && (a.epi != EPI_STORE || a.rope.head_dim % 2 || a.rope.n_rot % 2)) return fail(MESH_ERR_INVALID, "gemm_skinny: rope epilogue needs a plain store");
    if (a.items) {
        bool ok = a.n_items && a.max_items >= 1 && a.max_items <= 65535 && !a.rope.pos && a.epi != EPI_RESIDUAL && a.n_mat <= 2;
        for (int i = 1; i < a.n_mat; ++i) ok = ok && a.mat[i].type == a.mat[0].type && a.mat[i].M == a.mat[0].M;
        if (!ok) return fail(MESH_ERR_INVALID, "gemm_skinny: an expert launch takes one matrix or a gate / up pair of one type, no rope, no residual");
    }
    for (int i = 0; i < a.n_mat; ++i) {
        if (!a.mat[i].W || a.mat[i].M <= 0 || !type_is_tiled(a.mat[i].type)) return fail(MESH_ERR_INVALID, "gemm_skinny: matrix %d is not a tiled K-quant", i);
        if (!a.mat[i].y && !(i == 1 && a.epi == EPI_SWIGLU)) return fail(MESH_ERR_INVALID, "gemm_skinny: matrix %d has no output", i);
    }
    bool same = true;
    for (int i = 1; i < a.n_mat; ++i) same = same && a.mat[i].type == a.mat[0].type;
    if (same) return skinny_one_type(a, stream);
    // mixed types (q/k in q4_K, v in q6_K): q4_K matrices followed by one q6_K matrix share a launch ...
    if (a.pair_launch && !a.items && a.epi == EPI_STORE && a.mat[a.n_mat - 1].type == MESH_Q6_K) {
        bool lead_q4 = true;
        for (int k2 = 0; k2 + 1 < a.n_mat; ++k2) lead_q4 = lead_q4 && a.mat[k2].type == MESH_Q4_K;
        if (lead_q4) {
            SkinnyArgs qa = a, qb = a;
            qa.n_mat = a.n_mat - 1;
            qb.n_mat = 1;
            qb.mat[0] = a.mat[a.n_mat - 1]; qb.kind[0] = a.kind[a.n_mat - 1];
            const int rc = skinny_pair(qa, qb, stream);
            if (rc != MESH_ERR_UNSUPPORTED) return rc;
        }
    }
    // ... anything else: one launch per run of equal type
    int i = 0;
    while (i < a.n_mat) {
        int j = i + 1;
        while (j < a.n_mat && a.mat[j].type == a.mat[i].type) ++j;
        SkinnyArgs sub = a;
        sub.n_mat = j - i;
        for (int k2 = 0; k2 < sub.n_mat; ++k2) { sub.mat[k2] = a.mat[i + k2]; sub.kind[k2] = a.kind[i + k2]; }
        int rc = skinny_one_type(sub, stream);
        if (rc != MESH_OK) return rc;
        i = j;
    }
    return MESH_OK;
}

}  // namespace mesh
