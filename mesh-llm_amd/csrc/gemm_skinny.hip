// Skinny GEMM for batched decode: Y[T][M] = W[M][K] . X[T][K] with 5 <= T <= a few dozen tokens, W a tiled
// q4_K / q6_K matrix, X in f16.
//
// Between the mat-vec kernel (gemv.hip: one dot4 chain per activation column, so the weights' integer work is
// repeated per token) and the prefill GEMM (gemm.hip: 128x128 output tiles, far too few workgroups when T is
// small) sits the batch of decode steps.  Here the weight stream is organised exactly as in the mat-vec kernel --
// a workgroup owns a few tile-rows (16 rows each), its waves split K and each keeps four weight tiles in flight --
// but a tile is dequantised in registers to f16 and multiplied with 16 activation columns at once on the matrix
// cores (v_mfma_f32_16x16x32_f16), so the per-token cost is a fraction of an MFMA instead of a dot4 chain.
//
// Register dequantisation: lane (m = l % 16, g = l / 16) loads what lane 4m + g of the mat-vec kernel loads, i.e.
// quarter g of row m of the super-block (gemv.hpp).  An MFMA's k-slots of lane group g are then 8 consecutive
// elements of that quarter; the B operand (activations) is read with the same element indices, so the k-order of
// the instruction never has to match the order in memory.  Nibbles become f16 through the exponent trick
// (0x6400 | q is 1024 + q exactly), the offset is removed exactly, and the sub-block scale and minimum are applied
// with one packed fma, all in f16 (sums are f32, in the MFMA accumulator).
//
// Same math as ggml's mul_mat for K-quant weights (ggml_vec_dot_q4_K_q8_K / q6_K in
// third_party/llama.cpp ggml-cpu/quants.c, reached from rpc_server::graph_compute,
// patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451) except that activations are rounded to f16
// instead of q8_K.

#include "gemm.hpp"
#include "gemv_device.hpp"

namespace mesh {

constexpr int SK_THREADS = 512;
constexpr int SK_WAVES = SK_THREADS / 64;
constexpr int SK_DEPTH = 4;               // weight tiles a wave keeps in flight
constexpr int SK_NT = 16;                 // activation columns per launch (one MFMA N)
constexpr int SK_SEGS_MAX = 8;            // (tile-row, matrix) segments one wave may own
constexpr size_t SK_LDS_LIMIT = 160 * 1024;

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef float f4_t __attribute__((ext_vector_type(4)));

struct SkinnyKernelArgs {
    const uint8_t *wbase[3];      // matrix base minus its first tile-row, so a global tile-row index addresses it
    int tile_begin[4];            // first global tile-row of each matrix; unused slots hold the total
    float *y[3];
    const float *bias[3];
    int M[3];
    int ldy[3];
    const _Float16 *x;            // [T][ldx]
    int ldx, K, T;
    const float *residual;
    int ldres;
    int epi;
    _Float16 *y16;                // optional f16 copy of the output (matrix 0), [T][ldy16]
    int ldy16;
    int ks;                       // waves along K
};

// four bytes (values < 64) -> four f16 holding 1024 + value
__device__ __forceinline__ void bytes_to_h1024(uint32_t v, h2_t &lo, h2_t &hi) {
    lo = __builtin_bit_cast(h2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u));
    hi = __builtin_bit_cast(h2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u));
}

// Eight weights as an MFMA A fragment: bytes of v0, v1 hold the quants; w = (q - off) * s - mn.
__device__ __forceinline__ h8_t dequant8(uint32_t v0, uint32_t v1, h2_t off, h2_t s, h2_t mn) {
    h2_t p[4];
    bytes_to_h1024(v0, p[0], p[1]);
    bytes_to_h1024(v1, p[2], p[3]);
    h8_t a;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const h2_t q = p[i] - off;                                   // exact
        const h2_t w = __builtin_elementwise_fma(q, s, mn);
        a[2 * i] = w[0];
        a[2 * i + 1] = w[1];
    }
    return a;
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
    h2_t s_lo, s_hi, mn_lo, mn_hi;
    int kbase;
    __device__ __forceinline__ void prepare(const TileRegs<MESH_Q4_K> &R, int g) {
        const float d = f16_bits_to_f32((uint16_t)(R.hdr.x & 0xFFFFu));
        const float dmin = f16_bits_to_f32((uint16_t)(R.hdr.x >> 16));
        // 6-bit (scale, min) of sub-blocks 2g and 2g+1 (get_scale_min_k4 of ggml-quants.c)
        const uint32_t scw = g < 2 ? (R.hdr.y & 0x3F3F3F3Fu) : ((R.hdr.w & 0x0F0F0F0Fu) | ((R.hdr.y >> 2) & 0x30303030u));
        const uint32_t mnw = g < 2 ? (R.hdr.z & 0x3F3F3F3Fu) : (((R.hdr.w >> 4) & 0x0F0F0F0Fu) | ((R.hdr.z >> 2) & 0x30303030u));
        const int sh = (g & 1) * 16;
        s_lo = h2_of(d * (float)((scw >> sh) & 0xFFu));
        s_hi = h2_of(d * (float)((scw >> (sh + 8)) & 0xFFu));
        mn_lo = h2_of(-dmin * (float)((mnw >> sh) & 0xFFu));
        mn_hi = h2_of(-dmin * (float)((mnw >> (sh + 8)) & 0xFFu));
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
        const h2_t off = {(_Float16)1024.f, (_Float16)1024.f};
        return dequant8(v0, v1, off, high ? s_hi : s_lo, high ? mn_hi : mn_lo);
    }
    __device__ __forceinline__ int koff(int t) const { return kbase + 32 * (t >> 2) + 8 * (t & 3); }
};

template <> struct TileFrags<MESH_Q6_K> {
    uint32_t v[4][4];      // [t4][dword]: six-bit quants in bytes, elements 128n + 32 t4 + 16u + 4 dword + byte
    h2_t s[4];
    int kbase;
    __device__ __forceinline__ void prepare(const TileRegs<MESH_Q6_K> &R, int g) {
        const int n = g >> 1, u = g & 1;
        const float d = f16_bits_to_f32((uint16_t)R.d);
        const uint32_t la[4] = {R.qla.x, R.qla.y, R.qla.z, R.qla.w}, lb[4] = {R.qlb.x, R.qlb.y, R.qlb.z, R.qlb.w};
        const uint32_t qh[4] = {R.qh.x, R.qh.y, R.qh.z, R.qh.w};
        const uint32_t scw0 = n ? R.sc.z : R.sc.x, scw1 = n ? R.sc.w : R.sc.y;
        s[0] = h2_of(d * (float)(int8_t)((scw0 >> (8 * u)) & 0xFFu));
        s[1] = h2_of(d * (float)(int8_t)((scw0 >> (16 + 8 * u)) & 0xFFu));
        s[2] = h2_of(d * (float)(int8_t)((scw1 >> (8 * u)) & 0xFFu));
        s[3] = h2_of(d * (float)(int8_t)((scw1 >> (16 + 8 * u)) & 0xFFu));
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
        return dequant8(v[t4][2 * h], v[t4][2 * h + 1], off, s[t4], zero);
    }
    __device__ __forceinline__ int koff(int t) const { return kbase + 32 * (t >> 1) + 8 * (t & 1); }
};

// B fragments of one super-block for this lane: 8 MFMAs x 8 f16
template <int TYPE>
struct BFrags {
    uint4 b[8];
    __device__ __forceinline__ void load(const _Float16 *xcol, bool live, int sb, int g) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            int koff;
            if (TYPE == MESH_Q4_K) koff = 64 * g + 32 * (t >> 2) + 8 * (t & 3);
            else koff = 128 * (g >> 1) + 16 * (g & 1) + 32 * (t >> 1) + 8 * (t & 1);
            b[t] = live ? ldg<uint4>(xcol + sb * QK_K + koff) : make_uint4(0u, 0u, 0u, 0u);
        }
    }
};

template <int TYPE, int NU, int SEGS>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(const SkinnyKernelArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    float *red = reinterpret_cast<float *>(smem);         // [KS][rows_here][NU][16 rows][16 cols]
    constexpr int TB = TileRegs<TYPE>::BYTES;
    constexpr int U = 2 * (SEGS > SK_DEPTH ? SEGS : SK_DEPTH);       // flat tile indices per unrolled round
    const int K = a.K, nsb = K / QK_K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15, g = lane >> 4;
    const int lane_perm = 4 * m + g;                      // the mat-vec kernel's lane that loads row m, quarter g
    const int KS = a.ks, RS = SK_WAVES / KS;
    const int ks = wave % KS, rs = wave / KS;
    const int total_rows = a.tile_begin[3];
    const int tr0 = (int)(((long long)blockIdx.x * total_rows) / gridDim.x);
    const int tr1 = (int)(((long long)(blockIdx.x + 1) * total_rows) / gridDim.x);
    const int rows_here = tr1 - tr0;
    const int n_i = rs < RS ? (nsb - ks + KS - 1) / KS : 0;         // super-blocks of this wave (ks < KS <= nsb)
    const size_t row_stride = (size_t)nsb * TB;
    const bool col_live = m < a.T;                        // B fragments: lane (n = m, g) supplies column n
    const _Float16 *xcol = a.x + (size_t)(col_live ? m : 0) * a.ldx;

    // flat tile index f -> (ii, seg); seg -> (local tile-row j, matrix u)
    auto seg_valid = [&](int seg) { return rs + RS * (seg / NU) < rows_here; };
    auto tile_ptr = [&](int ii, int seg) -> const uint8_t * {
        const int tr = tr0 + rs + RS * (seg / NU);
        int mi = seg % NU;
        if (NU == 1) mi = (tr >= a.tile_begin[1] ? 1 : 0) + (tr >= a.tile_begin[2] ? 1 : 0);
        return a.wbase[mi] + (size_t)tr * row_stride + (size_t)(ks + KS * ii) * TB;
    };
    const int total = n_i * SEGS;                         // flat indices, invalid segments included as bubbles

    TileRegs<TYPE> ring[SK_DEPTH];
    BFrags<TYPE> B[2];
    f4_t D[SEGS];
#pragma unroll
    for (int s = 0; s < SEGS; ++s) D[s] = f4_t{0.f, 0.f, 0.f, 0.f};

    // prologue: the first DEPTH tiles and the activations of the first two super-blocks
#pragma unroll
    for (int f = 0; f < SK_DEPTH; ++f) {
        const int ii = f / SEGS, seg = f % SEGS;
        if (f < total && seg_valid(seg)) ring[f].load(tile_ptr(ii, seg), lane_perm);
    }
    if (n_i > 0) B[0].load(xcol, col_live, ks, g);
    if (n_i > 1) B[1].load(xcol, col_live, ks + KS, g);

    for (int f0 = 0; f0 < total; f0 += U) {
#pragma unroll
        for (int q = 0; q < U; ++q) {
            const int f = f0 + q;
            constexpr int dummy = 0; (void)dummy;
            const int seg = q % SEGS, slot = q % SK_DEPTH, buf = (q / SEGS) % 2;
            const int ii = f / SEGS;
            if (f < total) {
                if (seg_valid(seg)) {
                    TileFrags<TYPE> F;
                    F.prepare(ring[slot], g);
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const h8_t af = F.frag(t);
                        const h8_t bf = __builtin_bit_cast(h8_t, B[buf].b[t]);
                        D[seg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, bf, D[seg], 0, 0, 0);
                    }
                }
                // refill this slot with the tile DEPTH positions ahead
                const int fn = f + SK_DEPTH;
                const int segn = (q + SK_DEPTH) % SEGS;
                if (fn < total && seg_valid(segn)) ring[slot].load(tile_ptr(fn / SEGS, segn), lane_perm);
                // last segment of a super-block: its activation buffer is free for the one after next
                if (seg == SEGS - 1 && ii + 2 < n_i) B[buf].load(xcol, col_live, ks + KS * (ii + 2), g);
            }
        }
    }

    // partial sums of this wave: D[seg] holds rows 4g..4g+3, column m of segment seg
#pragma unroll
    for (int seg = 0; seg < SEGS; ++seg) {
        if (n_i > 0 && seg_valid(seg)) {
            const int j = rs + RS * (seg / NU), u = seg % NU;
#pragma unroll
            for (int i = 0; i < 4; ++i) red[((((size_t)ks * rows_here + j) * NU + u) * 16 + 4 * g + i) * 16 + m] = D[seg][i];
        }
    }
    __syncthreads();

    // outputs of this workgroup: rows_here x 16 rows x T columns
    for (int o = tid; o < rows_here * 16 * SK_NT; o += SK_THREADS) {
        const int t = o % SK_NT, r = (o / SK_NT) % 16, j = o / (SK_NT * 16);
        if (t >= a.T) continue;
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
        if (a.y16 && mi == 0) a.y16[(size_t)t * a.ldy16 + row] = (_Float16)out;
    }
}

template <int TYPE, int NU, int SEGS>
static int launch_skinny(const SkinnyKernelArgs &ka, int grid, size_t smem, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_skinny_kernel<TYPE, NU, SEGS>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)SK_LDS_LIMIT));
        attr_set = true;
    }
    gemm_skinny_kernel<TYPE, NU, SEGS><<<dim3((unsigned)grid), dim3(SK_THREADS), smem, stream>>>(ka);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

template <int TYPE, int NU>
static int launch_skinny_segs(int segs, const SkinnyKernelArgs &ka, int grid, size_t smem, hipStream_t stream) {
    if (segs <= 1) return launch_skinny<TYPE, NU, NU>(ka, grid, smem, stream);       // NU == 2 needs two segments at least
    if (segs <= 2) return launch_skinny<TYPE, NU, 2>(ka, grid, smem, stream);
    if (segs <= 4) return launch_skinny<TYPE, NU, 4>(ka, grid, smem, stream);
    return launch_skinny<TYPE, NU, 8>(ka, grid, smem, stream);
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

// all matrices of `a` are tiled K-quants of one type
static int skinny_one_type(const SkinnyArgs &a, hipStream_t stream) {
    const int type = a.mat[0].type;
    const int nsb = a.K / QK_K, NU = a.epi == EPI_SWIGLU ? 2 : 1;
    const size_t row_stride = (size_t)nsb * (type == MESH_Q4_K ? Q4K_TILE_BYTES : Q6K_TILE_BYTES);
    SkinnyKernelArgs ka{};
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
    const int n_bound = NU == 2 ? 1 : a.n_mat;          // matrix boundaries the kernel searches
    for (int i = n_bound; i < 4; ++i) ka.tile_begin[i] = total_rows;
    ka.ldx = a.ldx; ka.K = a.K;
    ka.ldres = a.ldres; ka.epi = a.epi;
    ka.ldy16 = a.ldy16;
    const int KS = nsb < SK_WAVES ? nsb : SK_WAVES, RS = SK_WAVES / KS;
    ka.ks = KS;
    // tile-rows per workgroup: spread over the CUs, bounded by the segments a wave can hold
    const int rows_cap = std::max(1, SK_SEGS_MAX / NU) * RS;
    const int ncu = skinny_n_cu();
    int rows_per_wg = std::min((total_rows + ncu - 1) / ncu, rows_cap);
    rows_per_wg = std::max(1, rows_per_wg);
    const int grid = (total_rows + rows_per_wg - 1) / rows_per_wg;
    const int rows_max = (total_rows + grid - 1) / grid;
    const int segs = ((rows_max + RS - 1) / RS) * NU;   // per wave
    if (segs > SK_SEGS_MAX) return fail(MESH_ERR_UNSUPPORTED, "gemm_skinny: %d segments per wave", segs);
    const size_t smem = sizeof(float) * (size_t)KS * rows_max * NU * 16 * SK_NT;
    if (smem > SK_LDS_LIMIT) return fail(MESH_ERR_UNSUPPORTED, "gemm_skinny: reduction buffer of %zu bytes does not fit LDS", smem);
    for (int t = 0; t < a.T; t += SK_NT) {
        SkinnyKernelArgs kb = ka;
        kb.T = std::min(SK_NT, a.T - t);
        kb.x = a.x + (size_t)t * a.ldx;
        kb.residual = a.residual ? a.residual + (size_t)t * a.ldres : nullptr;
        kb.y16 = a.y16 ? a.y16 + (size_t)t * a.ldy16 : nullptr;
        for (int i = 0; i < a.n_mat; ++i)
            if (kb.y[i]) kb.y[i] = a.mat[i].y + (size_t)t * a.mat[i].ldy;
        int rc;
        if (type == MESH_Q4_K) rc = NU == 2 ? launch_skinny_segs<MESH_Q4_K, 2>(segs, kb, grid, smem, stream) : launch_skinny_segs<MESH_Q4_K, 1>(segs, kb, grid, smem, stream);
        else rc = NU == 2 ? launch_skinny_segs<MESH_Q6_K, 2>(segs, kb, grid, smem, stream) : launch_skinny_segs<MESH_Q6_K, 1>(segs, kb, grid, smem, stream);
        if (rc != MESH_OK) return rc;
    }
    return MESH_OK;
}

int gemm_skinny(const SkinnyArgs &a, hipStream_t stream) {
    if (a.n_mat < 1 || a.n_mat > 3 || !a.x || a.T <= 0 || a.K <= 0) return fail(MESH_ERR_INVALID, "gemm_skinny: bad arguments");
    if (a.K % QK_K || a.ldx % 8 || (reinterpret_cast<uintptr_t>(a.x) & 15))
        return fail(MESH_ERR_INVALID, "gemm_skinny: K %d must be a multiple of 256 and the activations 16-byte aligned rows (ldx %d)", a.K, a.ldx);
    if (a.epi == EPI_SWIGLU && (a.n_mat != 2 || a.mat[0].M != a.mat[1].M || a.mat[0].type != a.mat[1].type))
        return fail(MESH_ERR_INVALID, "gemm_skinny: SwiGLU needs a gate and an up matrix of equal shape and type");
    if (a.epi == EPI_RESIDUAL && !a.residual) return fail(MESH_ERR_INVALID, "gemm_skinny: residual epilogue without residual");
    for (int i = 0; i < a.n_mat; ++i) {
        if (!a.mat[i].W || a.mat[i].M <= 0 || !type_is_tiled(a.mat[i].type)) return fail(MESH_ERR_INVALID, "gemm_skinny: matrix %d is not a tiled K-quant", i);
        if (!a.mat[i].y && !(i == 1 && a.epi == EPI_SWIGLU) && !(i == 0 && a.y16)) return fail(MESH_ERR_INVALID, "gemm_skinny: matrix %d has no output", i);
    }
    bool same = true;
    for (int i = 1; i < a.n_mat; ++i) same = same && a.mat[i].type == a.mat[0].type;
    if (same) return skinny_one_type(a, stream);
    // mixed types (q/k in q4_K, v in q6_K): one launch per run of equal type
    int i = 0;
    while (i < a.n_mat) {
        int j = i + 1;
        while (j < a.n_mat && a.mat[j].type == a.mat[i].type) ++j;
        SkinnyArgs sub = a;
        sub.n_mat = j - i;
        for (int k2 = 0; k2 < sub.n_mat; ++k2) sub.mat[k2] = a.mat[i + k2];
        sub.y16 = i == 0 ? a.y16 : nullptr;
        int rc = skinny_one_type(sub, stream);
        if (rc != MESH_OK) return rc;
        i = j;
    }
    return MESH_OK;
}

}  // namespace mesh
