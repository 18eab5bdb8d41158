// Skinny GEMM for batched decode on the f16 matrix cores: Y[T][M] = W[M][K] . X[T][K] with up to 16 or up to 32 tokens per
// pass, W a tiled q4_K / q6_K matrix, X in f16 (the k8-major layout of gemm.hpp).
//
// The alternative to the integer kernel of gemm_skinny.hip for the same launches: the weight stream is organised as in
// the mat-vec kernel -- a workgroup owns a few tile-rows (16 rows each), its waves split K and each keeps two
// weight tiles in flight -- and a tile is dequantised in registers to f16 and multiplied with 16 activation columns at
// once (v_mfma_f32_16x16x32_f16).  It issues about a third of the integer kernel's vector instructions per tile, so it
// streams weights faster; what it gives up is precision: activations are rounded to f16 (11 significant bits against the
// integer kernel's 16-bit fixed point), and so is every weight, ONCE: a weight is formed as ((q - offset) * sc) * d + c
// with q - offset and the integer sub-block scale sc exact in f16, d the super-block's own f16 scale, and c = 8 d sc -
// dmin m the sub-block's centre (q4_K; 0 for q6_K) -- the formation the prefill GEMM uses (gemm.hip).  The first version
// of this kernel multiplied by the products d * sc and dmin * m rounded to f16, an error shared by all 32 weights of a
// sub-block that does not average out over K and put a 16-layer stage at 1.2e-2 from the oracle; with one rounding per
// weight the same stage measures what the prefill path does (1-2e-3).
//
// Register dequantisation: lane (m = l % 16, g = l / 16) loads what lane 4m + g of the mat-vec kernel loads, i.e.
// quarter g of row m of the super-block (gemv.hpp).  An MFMA's k-slots of lane group g are then 8 consecutive
// elements of that quarter; the B operand (activations) is read with the same element indices, so the k-order of
// the instruction never has to match the order in memory.  Nibbles become f16 through the exponent trick
// (0x6400 | q is 1024 + q exactly).  Weight tiles are loaded with the mat-vec kernel's dense lane mapping and moved to
// the MFMA lanes with ds_bpermute, so that a wave's load touches whole cache lines.
//
// Same place in the worker's graph as the mat-vec kernel: mul_mat for K-quant weights, reached from
// rpc_server::graph_compute (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451).

#include "gemm.hpp"
#include "gemv_device.hpp"

namespace mesh {
namespace f16sk {

constexpr int SK_THREADS = 512;
constexpr int SK_WAVES = SK_THREADS / 64;
constexpr int SK_DEPTH_Q4 = 2;            // weight tiles a wave keeps in flight (2304 B each; three and four measured 8% slower)
constexpr int SK_DEPTH_Q6 = 2;            // q6_K tiles are 3360 B and their fragments need more registers
constexpr int SK_NT = 16;                 // activation columns of one MFMA (a launch takes one or two such blocks)
constexpr int SK_SEGS_MAX = 4;            // (tile-row, matrix) segments one wave may own (8 spills registers)
constexpr size_t SK_LDS_LIMIT = 160 * 1024;

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));

struct SkinnyKernelArgs {
    const uint8_t *wbase[3];      // matrix base minus its first tile-row, so a global tile-row index addresses it
    int tile_begin[4];            // first global tile-row of each matrix; unused slots hold the total
    float *y[3];
    const float *bias[3];
    int M[3];
    int ldy[3];
    const _Float16 *x;            // k8-major block of 16 columns
    int K, T;
    const float *residual;
    int ldres;
    int epi;
    _Float16 *y16;                // optional f16 copy of the output (matrix 0): k8-major block with M16 rows as its k
    unsigned *sat;                // optional counter of y16 values clamped to the f16 range
    int M16;
    int ks;                       // waves along K
    GemvRope rope;                // rope.pos / rope.seq point at the launch's first column
    int kind[3];
    // RMS-norm hand-over (gemm.hpp: SkinnyF16Args::NormOut / NormIn)
    const float *no_w;            // producer: weight of the norm that follows
    _Float16 *no_x16;
    float *no_part;
    const float *ni_part;         // consumer: [ni_parts][16] partial sums of squares
    int ni_parts;
    float ni_eps;
};

// four bytes (values < 64) -> four f16 holding 1024 + value
__device__ __forceinline__ void bytes_to_h1024(uint32_t v, h2_t &lo, h2_t &hi) {
    lo = __builtin_bit_cast(h2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u));
    hi = __builtin_bit_cast(h2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u));
}

// Eight weights as an MFMA A fragment: bytes of v0, v1 hold the quants; w = ((q - off) * sc) * d + c, where (q - off) * sc
// is an exact integer in f16 and the fma rounds once.
__device__ __forceinline__ h8_t dequant8(uint32_t v0, uint32_t v1, h2_t off, h2_t sc, h2_t d, h2_t c) {
    h2_t p[4];
    bytes_to_h1024(v0, p[0], p[1]);
    bytes_to_h1024(v1, p[2], p[3]);
    u4_t a;                                                          // built as four dwords: no half-register moves
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const h2_t q = (p[i] - off) * sc;                            // exact
        a[i] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(q, d, c));
    }
    return __builtin_bit_cast(h8_t, a);
}

__device__ __forceinline__ h2_t h2_of(float v) {
    const _Float16 h = (_Float16)v;
    return h2_t{h, h};
}

// A fragments of one tile, MFMA by MFMA.  frag(t, ...) returns the fragment of MFMA t (0..7) and the element
// offset within the super-block of this lane's 8 k-slots.
template <int TYPE> struct TileFrags;

template <> struct TileFrags<MESH_Q4_K> {
    uint32_t w[8];
    h2_t s_lo, s_hi, c_lo, c_hi, d2;
    int kbase;
    __device__ __forceinline__ void prepare(const TileRegs<MESH_Q4_K> &R, int g) {
        const float d = f16_bits_to_f32((uint16_t)(R.hdr.x & 0xFFFFu));
        const float dmin = f16_bits_to_f32((uint16_t)(R.hdr.x >> 16));
        // 6-bit (scale, min) of sub-blocks 2g and 2g+1 (get_scale_min_k4 of ggml-quants.c)
        const uint32_t scw = g < 2 ? (R.hdr.y & 0x3F3F3F3Fu) : ((R.hdr.w & 0x0F0F0F0Fu) | ((R.hdr.y >> 2) & 0x30303030u));
        const uint32_t mnw = g < 2 ? (R.hdr.z & 0x3F3F3F3Fu) : (((R.hdr.w >> 4) & 0x0F0F0F0Fu) | ((R.hdr.z >> 2) & 0x30303030u));
        const int sh = (g & 1) * 16;
        const float sa = (float)((scw >> sh) & 0xFFu), sb = (float)((scw >> (sh + 8)) & 0xFFu);
        s_lo = h2_of(sa);                                            // integers below 64: exact
        s_hi = h2_of(sb);
        c_lo = h2_of(8.0f * d * sa - dmin * (float)((mnw >> sh) & 0xFFu));
        c_hi = h2_of(8.0f * d * sb - dmin * (float)((mnw >> (sh + 8)) & 0xFFu));
        d2 = h2_of(d);                                               // d is an f16 in the block: exact
        w[0] = R.qa.x; w[1] = R.qa.y; w[2] = R.qa.z; w[3] = R.qa.w;
        w[4] = R.qb.x; w[5] = R.qb.y; w[6] = R.qb.z; w[7] = R.qb.w;
        kbase = 64 * g;
    }
    // MFMA t: t < 4 low nibbles (sub-block 2g), bytes 8t..8t+7; t >= 4 high nibbles (sub-block 2g+1)
    __device__ __forceinline__ h8_t frag(int t) const {
        const int tt = t & 3;
        const bool high = t >= 4;
        const uint32_t v0 = (high ? w[2 * tt] >> 4 : w[2 * tt]) & 0x0F0F0F0Fu;
        const uint32_t v1 = (high ? w[2 * tt + 1] >> 4 : w[2 * tt + 1]) & 0x0F0F0F0Fu;
        const h2_t off = {(_Float16)1032.f, (_Float16)1032.f};       // 1024 + 8: the centred quant q - 8
        return dequant8(v0, v1, off, high ? s_hi : s_lo, d2, high ? c_hi : c_lo);
    }
    __device__ __forceinline__ int koff(int t) const { return kbase + 32 * (t >> 2) + 8 * (t & 3); }
};

template <> struct TileFrags<MESH_Q6_K> {
    uint32_t v[4][4];      // [t4][dword]: six-bit quants in bytes, elements 128n + 32 t4 + 16u + 4 dword + byte
    h2_t s[4], d2;
    int kbase;
    __device__ __forceinline__ void prepare(const TileRegs<MESH_Q6_K> &R, int g) {
        const int n = g >> 1, u = g & 1;
        const float d = f16_bits_to_f32((uint16_t)R.d);
        const uint32_t la[4] = {R.qla.x, R.qla.y, R.qla.z, R.qla.w}, lb[4] = {R.qlb.x, R.qlb.y, R.qlb.z, R.qlb.w};
        const uint32_t qh[4] = {R.qh.x, R.qh.y, R.qh.z, R.qh.w};
        const uint32_t scw0 = n ? R.sc.z : R.sc.x, scw1 = n ? R.sc.w : R.sc.y;
        s[0] = h2_of((float)(int8_t)((scw0 >> (8 * u)) & 0xFFu));     // int8: exact
        s[1] = h2_of((float)(int8_t)((scw0 >> (16 + 8 * u)) & 0xFFu));
        s[2] = h2_of((float)(int8_t)((scw1 >> (8 * u)) & 0xFFu));
        s[3] = h2_of((float)(int8_t)((scw1 >> (16 + 8 * u)) & 0xFFu));
        d2 = h2_of(d);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[0][j] = (la[j] & 0x0F0F0F0Fu) | ((qh[j] << 4) & 0x30303030u);
            v[1][j] = (lb[j] & 0x0F0F0F0Fu) | ((qh[j] << 2) & 0x30303030u);
            v[2][j] = ((la[j] >> 4) & 0x0F0F0F0Fu) | (qh[j] & 0x30303030u);
            v[3][j] = ((lb[j] >> 4) & 0x0F0F0F0Fu) | ((qh[j] >> 2) & 0x30303030u);
        }
        kbase = 128 * n + 16 * u;
    }
    // MFMA t = 2 t4 + h: elements 8h..8h+7 of the 16-element scale group t4
    __device__ __forceinline__ h8_t frag(int t) const {
        const int t4 = t >> 1, h = t & 1;
        const h2_t off = {(_Float16)1056.f, (_Float16)1056.f};       // 1024 + 32: quants are stored with a bias of 32
        const h2_t zero = {(_Float16)0.f, (_Float16)0.f};
        // ((q - 32) * sc reaches 32 * 128 = 4096, one bit more than f16 holds exactly: products above 2048 with an odd value
        // round by 2^-12 of themselves, below the rounding of the multiplication by d that follows)
        return dequant8(v[t4][2 * h], v[t4][2 * h + 1], off, s[t4], d2, zero);
    }
    __device__ __forceinline__ int koff(int t) const { return kbase + 32 * (t >> 1) + 8 * (t & 1); }
};

// B fragments of one super-block for this lane: 8 MFMAs x 8 f16
template <int TYPE>
struct BFrags {
    uint4 b[8];
    // x: the k8-major block (uniform), lane_off: this lane's column and quarter offset in halfs
    __device__ __forceinline__ void load(const _Float16 *x, int lane_off, int sb) {
        const _Float16 *base = x + (size_t)sb * (QK_K * 16);      // uniform
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            int koff;                                      // compile-time part of the element offset
            if (TYPE == MESH_Q4_K) koff = 32 * (t >> 2) + 8 * (t & 3);
            else koff = 32 * (t >> 1) + 8 * (t & 1);
            b[t] = ldg<uint4>(base + lane_off + koff * 16);
        }
    }
};

// Moves a tile loaded with the dense mapping (lane 4r + c holds row r, quarter c) to the MFMA mapping
// (lane m + 16 g holds row m, quarter g).
__device__ __forceinline__ uint32_t lane_gather(uint32_t v, int src_lane4) {
    return (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane4, (int)v);
}
__device__ __forceinline__ uint4 lane_gather(const uint4 &v, int src_lane4) {
    return make_uint4(lane_gather(v.x, src_lane4), lane_gather(v.y, src_lane4), lane_gather(v.z, src_lane4), lane_gather(v.w, src_lane4));
}
__device__ __forceinline__ void to_mfma_lanes(TileRegs<MESH_Q4_K> &R, int src_lane4) {
    R.hdr = lane_gather(R.hdr, src_lane4);
    R.qa = lane_gather(R.qa, src_lane4);
    R.qb = lane_gather(R.qb, src_lane4);
}
__device__ __forceinline__ void to_mfma_lanes(TileRegs<MESH_Q6_K> &R, int src_lane4) {
    R.qla = lane_gather(R.qla, src_lane4);
    R.qlb = lane_gather(R.qlb, src_lane4);
    R.qh = lane_gather(R.qh, src_lane4);
    R.sc = lane_gather(R.sc, src_lane4);
    R.d = lane_gather(R.d, src_lane4);
}

// element (row k, column t) of k8-major f16 activations with K rows per column: block t / 16 of 16 * K halfs
__device__ __forceinline__ size_t k8_at(int K, int k, int t) { return (size_t)(t >> 4) * 16 * K + ((size_t)(k >> 3) * 16 + (t & 15)) * 8 + (k & 7); }

// most tile-rows a workgroup of the launch has (p_split = tile-rows per workgroup | workgroups with one more << 16)
__device__ __forceinline__ int rows_here_max(unsigned p_split) { return (int)(p_split & 0xFFFFu) + ((p_split >> 16) ? 1 : 0); }

// NC: blocks of 16 activation columns one pass over the weights multiplies with (1: up to 16 tokens, 2: up to 32).
// bx: the workgroup's index among those of its launch part (the whole launch, or one side of a pair launch).
template <int TYPE, int NU, int SEGS, int NC>
__device__ __forceinline__ void skinny_workgroup(int bx, const _Float16 *p_x, const uint8_t *p_w0, const uint8_t *p_w1, const uint8_t *p_w2, int p_K,
                                                 int p_ks, unsigned p_begins, unsigned p_split, const SkinnyKernelArgs &a) {
    // (p_begins = first tile-row of matrix 1 | of matrix 2 << 16; p_split = tile-rows per workgroup | workgroups with one
    // more << 16, computed on the host: no division and no grid-size load stand before the first weight load)
    const int p_begin1 = (int)(p_begins & 0xFFFFu), p_begin2 = (int)(p_begins >> 16);
    // (leading scalar arguments: preloaded into SGPRs, see gemv.hip)
    extern __shared__ __align__(16) uint8_t smem[];
    float *red = reinterpret_cast<float *>(smem);         // [KS][rows_here][NU][16 rows][16 NC columns]
    constexpr int TB = TileRegs<TYPE>::BYTES;
    constexpr int SK_DEPTH = TYPE == MESH_Q4_K ? SK_DEPTH_Q4 : SK_DEPTH_Q6;
    const int K = p_K, nsb = K / QK_K;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // scalar: tile addresses become SGPR base + lane offset
    const int m = lane & 15, g = lane >> 4;
    const int src_lane4 = 4 * (4 * m + g);                // byte address, for ds_bpermute, of the lane that loaded row m, quarter g
    const int KS = p_ks, LK = __builtin_ctz((unsigned)KS), RS = SK_WAVES >> LK;      // KS is a power of two
    const int ks = wave & (KS - 1), rs = wave >> LK;
    const int sq = (int)(p_split & 0xFFFFu), sr = (int)(p_split >> 16);
    const int tr0 = bx * sq + (bx < sr ? bx : sr);
    const int rows_here = sq + (bx < sr ? 1 : 0);
    const int n_i = rs < RS ? (nsb - ks + KS - 1) >> LK : 0;        // super-blocks of this wave (ks < KS <= nsb)
    const size_t row_stride = (size_t)nsb * TB;
    // B fragments: lane (n = m, g) supplies column n, quarter g (columns beyond T hold zeros)
    const int lane_off = (TYPE == MESH_Q4_K ? 64 * g : 128 * (g >> 1) + 16 * (g & 1)) * 16 + m * 8;
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

    constexpr int NT = SK_NT * NC;                        // activation columns of this launch
    TileRegs<TYPE> ring[SK_DEPTH];
    f4_t D[SEGS][NC];
#pragma unroll
    for (int s = 0; s < SEGS; ++s)
#pragma unroll
        for (int c = 0; c < NC; ++c) D[s][c] = f4_t{0.f, 0.f, 0.f, 0.f};

    // Loads are never under a branch of their own: an index past the end or an invalid segment is clamped to a tile
    // the wave owns (a cache hit).  The compiler then knows exactly how many loads are in flight at every point
    // and waits for one tile without draining the others; a load under a branch makes it assume the worst at the
    // join, which in an unrolled pipeline degenerates to waiting for everything.
    auto load_tile = [&](TileRegs<TYPE> &dst, int f, int seg) {
        const bool ok = f < total && seg_valid(seg);
        dst.load(tile_ptr(ok ? f / SEGS : n_i - 1, ok ? seg : 0), lane);
    };
    // Activation fragments: 8 KB per super-block, column block and wave.  Only ONE super-block is held (32 registers per
    // column block) and every fragment is fetched again, for the next super-block, right behind the last MFMAs that read
    // it: one tile's time ahead of its use, enough for a hit in L2.  (Two whole super-blocks in registers, fetched a
    // super-block ahead, cost 32 more registers per column block and measured 6% slower at 16 columns.)  A tile that
    // is not computed (past the end, invalid segment) issues the same loads in the same order, so that the compiler's
    // count of loads in flight is the same along both paths.
    BFrags<TYPE> Bw[NC];
    auto frag_koff = [](int t) { return (TYPE == MESH_Q4_K ? 32 * (t >> 2) + 8 * (t & 3) : 32 * (t >> 1) + 8 * (t & 1)) * 16; };
    auto b_base = [&](int sb, int c) { return p_x + (size_t)c * SK_NT * K + (size_t)sb * (QK_K * 16) + lane_off; };
    auto step = [&](const TileRegs<TYPE> &loaded, f4_t (&acc)[NC], bool valid, bool refill, int next_sb) {
        const _Float16 *nb[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) nb[c] = b_base(next_sb, c);
        if (valid) {
            TileRegs<TYPE> tile = loaded;
            to_mfma_lanes(tile, src_lane4);
            TileFrags<TYPE> F;
            F.prepare(tile, g);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const h8_t af = F.frag(t);
#pragma unroll
                for (int c = 0; c < NC; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, __builtin_bit_cast(h8_t, Bw[c].b[t]), acc[c], 0, 0, 0);
                if (refill) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) Bw[c].b[t] = ldg<uint4>(nb[c] + frag_koff(t));
                }
            }
        } else if (refill) {
#pragma unroll
            for (int t = 0; t < 8; ++t)
#pragma unroll
                for (int c = 0; c < NC; ++c) Bw[c].b[t] = ldg<uint4>(nb[c] + frag_koff(t));
        }
    };
    if (total > 0) {
#pragma unroll
        for (int f = 0; f < SK_DEPTH; ++f) load_tile(ring[f], f, f % SEGS);
#pragma unroll
        for (int c = 0; c < NC; ++c) Bw[c].load(p_x + (size_t)c * SK_NT * K, lane_off, ks);
        constexpr int RB = SEGS % SK_DEPTH == 0 ? 1 : SK_DEPTH;      // rounds per unrolled block: ring slots static inside it
        constexpr int UB = RB * SEGS;
        static_assert(UB % SK_DEPTH == 0, "ring slots must be static inside a block");
        for (int blk = 0; blk * RB < n_i; ++blk) {
#pragma unroll
            for (int q = 0; q < UB; ++q) {
                const int r = q / SEGS, seg = q % SEGS, slot = q % SK_DEPTH;
                const int ii = blk * RB + r, f = ii * SEGS + seg;
                step(ring[slot], D[seg], ii < n_i && seg_valid(seg), seg == SEGS - 1, ks + KS * (ii + 1 < n_i ? ii + 1 : n_i - 1));
                load_tile(ring[slot], f + SK_DEPTH, (q + SK_DEPTH) % SEGS);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    // partial sums of this wave: D[seg] holds rows 4g..4g+3, column m of segment seg
#pragma unroll
    for (int seg = 0; seg < SEGS; ++seg) {
        if (total > 0 && seg_valid(seg)) {
            const int j = rs + RS * (seg / NU), u = seg % NU;
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[((((size_t)ks * rows_here + j) * NU + u) * 16 + 4 * g + i) * NT + c * SK_NT + m] = D[seg][c][i];
        }
    }
    // (after the reduction buffer: [NORM_GROUPS][NT] sums of the consumer side, [SK_WAVES][NT] of the producer side)
    constexpr int NORM_GROUPS = SK_THREADS / NT;          // threads sharing a token column in the epilogue
    float *nrm = red + (size_t)KS * rows_here_max(p_split) * NU * 16 * NT;
    if (a.ni_part) {
        // norm hand-over, consumer side: this thread's share of the partial sums of squares of its epilogue column
        // (fetched after the weight stream: before it, the wave would wait for them ahead of its first tile loads)
        float ni_sum = 0.f;
        for (int p = tid / NT; p < a.ni_parts; p += NORM_GROUPS) ni_sum += a.ni_part[(size_t)p * NT + tid % NT];
        nrm[tid] = ni_sum;                             // tid = group * NT + column
    }
    __syncthreads();
    // 1 / rms of this thread's column (every output of a thread is of column tid % NT): groups added in order
    float inv_rms = 1.0f;
    if (a.ni_part) {
        float ss = 0.f;
        for (int q = 0; q < NORM_GROUPS; ++q) ss += nrm[q * NT + tid % NT];
        inv_rms = 1.0f / sqrtf(ss / (float)K + a.ni_eps);
    }
    float no_ss = 0.f;         // producer side: sum of squares of this thread's outputs (one column)
    // outputs of this workgroup: rows_here x 16 rows x T columns; column t is column t % 16 of the f16 layouts' block t / 16
    for (int o = tid; o < rows_here * 16 * NT; o += SK_THREADS) {
        const int t = o % NT, r = (o / NT) % 16, j = o / (NT * 16);
        const int tr = tr0 + j;
        int mi = 0;
        if (NU == 1) mi = (tr >= a.tile_begin[1] ? 1 : 0) + (tr >= a.tile_begin[2] ? 1 : 0);
        const int row = (tr - a.tile_begin[mi]) * TILE_ROWS + r;
        if (row >= a.M[mi]) continue;
        if (t >= a.T) {                                    // unused columns of the f16 output block stay finite
            if (a.y16 && mi == 0) a.y16[k8_at(a.M16, row, t)] = (_Float16)0.f;
            if (a.no_x16) a.no_x16[k8_at(a.M[0], row, t)] = (_Float16)0.f;
            continue;
        }
        float s0 = 0.f, s1 = 0.f;
        for (int k2 = 0; k2 < KS; ++k2) {
            s0 += red[((((size_t)k2 * rows_here + j) * NU + 0) * 16 + r) * NT + t];
            if (NU == 2) s1 += red[((((size_t)k2 * rows_here + j) * NU + 1) * 16 + r) * NT + t];
        }
        s0 *= inv_rms;
        if (NU == 2) s1 *= inv_rms;
        if (a.bias[mi]) s0 += a.bias[mi][row];
        if (NU == 1 && a.rope.pos && a.kind[mi] != GEMV_KIND_PLAIN) {
            // q / k / v row of a token (see gemv.hpp): rotate q and k with the neighbouring row, k and v go to the cache
            const int kind = a.kind[mi], hd = a.rope.head_dim;
            const int head = row / hd, dd = row - head * hd;
            const int pos = a.rope.pos[t];
            float val = s0;
            if (kind != GEMV_KIND_V && dd < a.rope.n_rot) {
                float sp = 0.f;
                for (int k2 = 0; k2 < KS; ++k2) sp += red[((((size_t)k2 * rows_here + j) * NU + 0) * 16 + (r ^ 1)) * NT + t];
                sp *= inv_rms;
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
            out = a.residual[(size_t)t * a.ldres + row] + s0;
        } else {
            out = s0;
        }
        if (a.y[mi]) a.y[mi][(size_t)t * a.ldy[mi] + row] = out;
        // (saturating: a SwiGLU product beyond the f16 range becomes +-65504, not an infinity the next GEMM would spread)
        if (a.y16 && mi == 0) {
            note_f16_clamp(a.sat, out, 0.f);
            a.y16[k8_at(a.M16, row, t)] = (_Float16)__builtin_amdgcn_fmed3f(out, -65504.f, 65504.f);
        }
        if (a.no_x16) {
            const float v = out * a.no_w[row];
            note_f16_clamp(a.sat, v, 0.f);
            a.no_x16[k8_at(a.M[0], row, t)] = (_Float16)__builtin_amdgcn_fmed3f(v, -65504.f, 65504.f);
            no_ss = fmaf(out, out, no_ss);
        }
    }
    if (a.no_part) {
        // this workgroup's sum of squares per column: the lanes of a wave that share a column, then the waves in order
        if (NT == 16) no_ss += __shfl_xor(no_ss, 16);
        no_ss += __shfl_xor(no_ss, 32);
        float *wsum = nrm + NORM_GROUPS * NT;
        if (lane < NT) wsum[wave * NT + lane] = no_ss;
        __syncthreads();
        if (tid < NT) {
            float ss = 0.f;
            for (int w = 0; w < SK_WAVES; ++w) ss += wsum[w * NT + tid];
            a.no_part[(size_t)bx * NT + tid] = ss;
        }
    }
}

template <int TYPE, int NU, int SEGS, int NC>
__global__ __launch_bounds__(SK_THREADS, 2) void gemm_skinny_kernel(const _Float16 *p_x, const uint8_t *p_w0, const uint8_t *p_w1, const uint8_t *p_w2, int p_K,
                                                                 int p_ks, int p_rows, unsigned p_begins, unsigned p_split,
                                                                 const SkinnyKernelArgs a) {
    (void)p_rows;
    skinny_workgroup<TYPE, NU, SEGS, NC>((int)blockIdx.x, p_x, p_w0, p_w1, p_w2, p_K, p_ks, p_begins, p_split, a);
}

// Two launches that read the same activations as one: the first grid_a workgroups run a q4_K launch, the others a q6_K launch
// (the q and k projections of a layer next to a q6_K v projection: 160 + 64 workgroups at Llama-3-8B shape, one wave of
// workgroups instead of two dependent launches).  Same arithmetic per workgroup as the separate launches.
template <int SEGS_A, int SEGS_B, int NC>
__global__ __launch_bounds__(SK_THREADS, 2) void gemm_skinny_pair_kernel(const _Float16 *p_x, const uint8_t *p_w0, const uint8_t *p_w1, int p_K, int p_ks,
                                                                      int grid_a, unsigned p_begins, unsigned p_split_a, unsigned p_split_b,
                                                                      const uint8_t *p_wb, const SkinnyKernelArgs a, const SkinnyKernelArgs b) {
    const int bx = (int)blockIdx.x;
    if (bx < grid_a) skinny_workgroup<MESH_Q4_K, 1, SEGS_A, NC>(bx, p_x, p_w0, p_w1, p_w1, p_K, p_ks, p_begins, p_split_a, a);
    else skinny_workgroup<MESH_Q6_K, 1, SEGS_B, NC>(bx - grid_a, p_x, p_wb, p_wb, p_wb, p_K, p_ks, 0xFFFFFFFFu, p_split_b, b);
}

template <int TYPE, int NU, int SEGS, int NC>
static int launch_skinny(const SkinnyKernelArgs &ka, int grid, size_t smem, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_skinny_kernel<TYPE, NU, SEGS, NC>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)SK_LDS_LIMIT));
        attr_set = true;
    }
    MESH_LAUNCH((gemm_skinny_kernel<TYPE, NU, SEGS, NC>), dim3((unsigned)grid), dim3(SK_THREADS), smem, stream, ka.x, ka.wbase[0], ka.wbase[1] ? ka.wbase[1] : ka.wbase[0],
                ka.wbase[2] ? ka.wbase[2] : ka.wbase[0], ka.K, ka.ks, ka.tile_begin[3], (unsigned)ka.tile_begin[1] | ((unsigned)ka.tile_begin[2] << 16),
                (unsigned)(ka.tile_begin[3] / grid) | ((unsigned)(ka.tile_begin[3] % grid) << 16), ka);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

template <int TYPE, int NU, int NC>
static int launch_skinny_segs(int segs, const SkinnyKernelArgs &ka, int grid, size_t smem, hipStream_t stream) {
    if (segs <= 1) return launch_skinny<TYPE, NU, NU, NC>(ka, grid, smem, stream);   // NU == 2 needs two segments at least
    if (segs <= 2) return launch_skinny<TYPE, NU, 2, NC>(ka, grid, smem, stream);
    return launch_skinny<TYPE, NU, 4, NC>(ka, grid, smem, stream);
}
template <int TYPE, int NU>
static int launch_skinny_cols(int nc, int segs, const SkinnyKernelArgs &ka, int grid, size_t smem, hipStream_t stream) {
    return nc == 2 ? launch_skinny_segs<TYPE, NU, 2>(segs, ka, grid, smem, stream) : launch_skinny_segs<TYPE, NU, 1>(segs, ka, grid, smem, stream);
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

// waves along K: a power of two (the kernel splits its waves with shifts)
static int skinny_ks(int nsb) {
    int KS = 1;
    while (KS * 2 <= nsb && KS * 2 <= SK_WAVES) KS *= 2;
    return KS;
}
// workgroups of a launch over total_rows tile-rows: spread over the CUs, bounded by the segments a wave can hold
static int skinny_grid(int total_rows, int NU, int KS) {
    const int RS = SK_WAVES / KS;
    const int rows_cap = std::max(1, SK_SEGS_MAX / NU) * RS;
    const int ncu = skinny_n_cu();
    int rows_per_wg = std::min((total_rows + ncu - 1) / ncu, rows_cap);
    rows_per_wg = std::max(1, rows_per_wg);
    return (total_rows + rows_per_wg - 1) / rows_per_wg;
}

// What a launch over the matrices of `a` (tiled K-quants of one type) needs, before the token chunk is chosen
struct SkinnyLaunch {
    SkinnyKernelArgs ka;
    int type, NU, KS, total_rows, grid, rows_max, segs;
    size_t smem(int nt) const { return sizeof(float) * ((size_t)KS * rows_max * NU * 16 * nt + (size_t)SK_THREADS + (size_t)SK_WAVES * nt); }
};
static int skinny_prepare(const SkinnyF16Args &a, SkinnyLaunch &L) {
    L.type = a.mat[0].type;
    const int nsb = a.K / QK_K, NU = a.epi == EPI_SWIGLU ? 2 : 1;
    L.NU = NU;
    const size_t row_stride = (size_t)nsb * (L.type == MESH_Q4_K ? Q4K_TILE_BYTES : Q6K_TILE_BYTES);
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
    ka.M16 = a.mat[0].M;
    ka.sat = a.sat;
    ka.no_w = a.norm_out.norm_w; ka.no_x16 = a.norm_out.x16; ka.no_part = a.norm_out.part;
    ka.ni_part = a.norm_in.part; ka.ni_parts = a.norm_in.n_parts; ka.ni_eps = a.norm_in.eps;
    L.KS = skinny_ks(nsb);
    const int RS = SK_WAVES / L.KS;
    ka.ks = L.KS;
    L.total_rows = total_rows;
    if (total_rows > 0xFFFF) return fail(MESH_ERR_UNSUPPORTED, "gemm_skinny_f16: %d tile-rows in one launch", total_rows);
    L.grid = skinny_grid(total_rows, NU, L.KS);
    L.rows_max = (total_rows + L.grid - 1) / L.grid;
    L.segs = ((L.rows_max + RS - 1) / RS) * NU;         // per wave
    if (L.segs > SK_SEGS_MAX) return fail(MESH_ERR_UNSUPPORTED, "gemm_skinny_f16: %d segments per wave", L.segs);
    return MESH_OK;
}
// the kernel arguments of the launch for columns t .. t + nt - 1 of the call
static SkinnyKernelArgs skinny_chunk(const SkinnyF16Args &a, const SkinnyLaunch &L, int t, int nt) {
    SkinnyKernelArgs kb = L.ka;
    kb.T = std::min(nt, a.T - t);
    if (kb.rope.pos) { kb.rope.pos += t; kb.rope.seq += t; }
    kb.x = a.x + (size_t)t * a.K;                  // block t / 16 of the k8-major activations
    kb.residual = a.residual ? a.residual + (size_t)t * a.ldres : nullptr;
    kb.y16 = a.y16 ? a.y16 + (size_t)t * a.mat[0].M : nullptr;
    for (int i = 0; i < a.n_mat; ++i)
        if (kb.y[i]) kb.y[i] = a.mat[i].y + (size_t)t * a.mat[i].ldy;
    return kb;
}

// all matrices of `a` are tiled K-quants of one type
static int skinny_one_type(const SkinnyF16Args &a, hipStream_t stream) {
    SkinnyLaunch L;
    int rc = skinny_prepare(a, L);
    if (rc != MESH_OK) return rc;
    // a pass over the weights takes 32 columns while more than 16 remain, else 16 (a call of up to 32 tokens is one launch)
    for (int t = 0; t < a.T;) {
        const int nc = a.T - t > SK_NT ? 2 : 1, nt = nc * SK_NT;
        const size_t smem = L.smem(nt);
        if (smem > SK_LDS_LIMIT) return fail(MESH_ERR_UNSUPPORTED, "gemm_skinny_f16: reduction buffer of %zu bytes does not fit LDS", smem);
        const SkinnyKernelArgs kb = skinny_chunk(a, L, t, nt);
        if (L.type == MESH_Q4_K) rc = L.NU == 2 ? launch_skinny_cols<MESH_Q4_K, 2>(nc, L.segs, kb, L.grid, smem, stream) : launch_skinny_cols<MESH_Q4_K, 1>(nc, L.segs, kb, L.grid, smem, stream);
        else rc = L.NU == 2 ? launch_skinny_cols<MESH_Q6_K, 2>(nc, L.segs, kb, L.grid, smem, stream) : launch_skinny_cols<MESH_Q6_K, 1>(nc, L.segs, kb, L.grid, smem, stream);
        if (rc != MESH_OK) return rc;
        t += nt;
    }
    return MESH_OK;
}

template <int SEGS_A, int SEGS_B, int NC>
static int launch_pair(const SkinnyKernelArgs &ka, const SkinnyKernelArgs &kb, int grid_a, int grid_b, size_t smem, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_skinny_pair_kernel<SEGS_A, SEGS_B, NC>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)SK_LDS_LIMIT));
        attr_set = true;
    }
    MESH_LAUNCH((gemm_skinny_pair_kernel<SEGS_A, SEGS_B, NC>), dim3((unsigned)(grid_a + grid_b)), dim3(SK_THREADS), smem, stream, ka.x, ka.wbase[0],
                ka.wbase[1] ? ka.wbase[1] : ka.wbase[0], ka.K, ka.ks, grid_a, (unsigned)ka.tile_begin[1] | ((unsigned)ka.tile_begin[2] << 16),
                (unsigned)(ka.tile_begin[3] / grid_a) | ((unsigned)(ka.tile_begin[3] % grid_a) << 16),
                (unsigned)(kb.tile_begin[3] / grid_b) | ((unsigned)(kb.tile_begin[3] % grid_b) << 16), kb.wbase[0], ka, kb);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}
template <int NC>
static int launch_pair_segs(int segs_a, int segs_b, const SkinnyKernelArgs &ka, const SkinnyKernelArgs &kb, int grid_a, int grid_b, size_t smem, hipStream_t stream) {
    const int sa = segs_a <= 1 ? 1 : segs_a <= 2 ? 2 : 4;
    if (segs_b <= 1) {
        if (sa == 1) return launch_pair<1, 1, NC>(ka, kb, grid_a, grid_b, smem, stream);
        if (sa == 2) return launch_pair<2, 1, NC>(ka, kb, grid_a, grid_b, smem, stream);
        return launch_pair<4, 1, NC>(ka, kb, grid_a, grid_b, smem, stream);
    }
    if (sa == 1) return launch_pair<1, 2, NC>(ka, kb, grid_a, grid_b, smem, stream);
    if (sa == 2) return launch_pair<2, 2, NC>(ka, kb, grid_a, grid_b, smem, stream);
    return launch_pair<4, 2, NC>(ka, kb, grid_a, grid_b, smem, stream);
}

// `qa`: one or two q4_K matrices, `qb`: one q6_K matrix, same activations, plain-store epilogues (with or without RoPE):
// one launch whose first workgroups are qa's and whose last are qb's.  MESH_ERR_UNSUPPORTED when the shapes do not fit
// (the caller then launches them one after the other).
static int skinny_pair(const SkinnyF16Args &qa, const SkinnyF16Args &qb, hipStream_t stream) {
    SkinnyLaunch A, B;
    int rc = skinny_prepare(qa, A);
    if (rc != MESH_OK) return rc;
    if ((rc = skinny_prepare(qb, B)) != MESH_OK) return rc;
    if (B.segs > 2 || A.KS != B.KS) return MESH_ERR_UNSUPPORTED;
    for (int t = 0; t < qa.T;) {
        const int nc = qa.T - t > SK_NT ? 2 : 1, nt = nc * SK_NT;
        const size_t smem = std::max(A.smem(nt), B.smem(nt));
        if (smem > SK_LDS_LIMIT) return MESH_ERR_UNSUPPORTED;
        const SkinnyKernelArgs ka = skinny_chunk(qa, A, t, nt), kb = skinny_chunk(qb, B, t, nt);
        rc = nc == 2 ? launch_pair_segs<2>(A.segs, B.segs, ka, kb, A.grid, B.grid, smem, stream) : launch_pair_segs<1>(A.segs, B.segs, ka, kb, A.grid, B.grid, smem, stream);
        if (rc != MESH_OK) return rc;
        t += nt;
    }
    return MESH_OK;
}

}  // namespace f16sk

int gemm_skinny_f16_workgroups(const SkinnyF16Args &a) {
    using namespace f16sk;
    if (a.n_mat != 1 || a.K <= 0 || a.K % QK_K || a.mat[0].M <= 0) return 0;
    return skinny_grid((a.mat[0].M + TILE_ROWS - 1) / TILE_ROWS, 1, skinny_ks(a.K / QK_K));
}

int gemm_skinny_f16(const SkinnyF16Args &a, hipStream_t stream) {
    using namespace f16sk;
    if (a.norm_out.x16 || a.norm_out.part || a.norm_out.norm_w) {
        if (!a.norm_out.x16 || !a.norm_out.part || !a.norm_out.norm_w || a.n_mat != 1 || a.epi != EPI_RESIDUAL || a.T > SKINNY_F16_NORM_TOKENS_MAX || a.mat[0].M % 8 ||
            gemm_skinny_f16_workgroups(a) > SKINNY_F16_NORM_PARTS_MAX)
            return fail(MESH_ERR_INVALID, "gemm_skinny_f16: the norm hand-over needs one matrix with a residual epilogue, at most 32 tokens and a row count that is a multiple of 8");
    }
    if (a.norm_in.part && (a.norm_in.n_parts < 1 || a.norm_in.n_parts > SKINNY_F16_NORM_PARTS_MAX || a.T > SKINNY_F16_NORM_TOKENS_MAX))
        return fail(MESH_ERR_INVALID, "gemm_skinny_f16: bad norm hand-over input (%d partial sums, %d tokens)", a.norm_in.n_parts, a.T);
    if (a.n_mat < 1 || a.n_mat > 3 || !a.x || a.T <= 0 || a.K <= 0) return fail(MESH_ERR_INVALID, "gemm_skinny_f16: bad arguments");
    if (a.K % QK_K || (reinterpret_cast<uintptr_t>(a.x) & 15))
        return fail(MESH_ERR_INVALID, "gemm_skinny_f16: K %d must be a multiple of 256 and the activations 16-byte aligned", a.K);
    if (a.y16 && a.mat[0].M % 8) return fail(MESH_ERR_INVALID, "gemm_skinny_f16: f16 output needs a row count that is a multiple of 8");
    if (a.epi == EPI_SWIGLU && (a.n_mat != 2 || a.mat[0].M != a.mat[1].M || a.mat[0].type != a.mat[1].type))
        return fail(MESH_ERR_INVALID, "gemm_skinny_f16: SwiGLU needs a gate and an up matrix of equal shape and type");
    if (a.epi == EPI_RESIDUAL && !a.residual) return fail(MESH_ERR_INVALID, "gemm_skinny_f16: residual epilogue without residual");
    if (a.rope.pos && (a.epi != EPI_STORE || a.rope.head_dim % 2 || a.rope.n_rot % 2)) return fail(MESH_ERR_INVALID, "gemm_skinny_f16: rope epilogue needs a plain store");
    for (int i = 0; i < a.n_mat; ++i) {
        if (!a.mat[i].W || a.mat[i].M <= 0 || !type_is_tiled(a.mat[i].type)) return fail(MESH_ERR_INVALID, "gemm_skinny_f16: matrix %d is not a tiled K-quant", i);
        if (!a.mat[i].y && !(i == 1 && a.epi == EPI_SWIGLU) && !(i == 0 && a.y16)) return fail(MESH_ERR_INVALID, "gemm_skinny_f16: matrix %d has no output", i);
    }
    bool same = true;
    for (int i = 1; i < a.n_mat; ++i) same = same && a.mat[i].type == a.mat[0].type;
    if (same) return skinny_one_type(a, stream);
    // mixed types (q/k in q4_K, v in q6_K): q4_K matrices followed by one q6_K matrix share a launch ...
    if (a.pair_launch && a.epi == EPI_STORE && !a.y16 && a.mat[a.n_mat - 1].type == MESH_Q6_K) {
        bool lead_q4 = true;
        for (int k2 = 0; k2 + 1 < a.n_mat; ++k2) lead_q4 = lead_q4 && a.mat[k2].type == MESH_Q4_K;
        if (lead_q4) {
            SkinnyF16Args qa = a, qb = a;
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
        SkinnyF16Args sub = a;
        sub.n_mat = j - i;
        for (int k2 = 0; k2 < sub.n_mat; ++k2) { sub.mat[k2] = a.mat[i + k2]; sub.kind[k2] = a.kind[i + k2]; }
        sub.y16 = i == 0 ? a.y16 : nullptr;
        int rc = skinny_one_type(sub, stream);
        if (rc != MESH_OK) return rc;
        i = j;
    }
    return MESH_OK;
}

}  // namespace mesh
