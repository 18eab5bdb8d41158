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

#include "gemv_device.hpp"

#include <algorithm>

namespace mesh {

int gemv_generic(const GemvArgs &a, hipStream_t stream);

constexpr int GEMV_THREADS = 1024;        // one workgroup fills a CU: 16 waves, 4 per SIMD
constexpr int GEMV_WAVES = GEMV_THREADS / 64;

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
    // pairs grouped by expert: blockIdx.y = work item (gemv.hpp: MOE_ITEM_INTS int32 each); items past *n_items do nothing
    const int32_t *items, *n_items;
    GemvRope rope;         // rope.pos / rope.seq already point at the launch's first column
    int kind[3];
    uint8_t *xq_out;       // EPI_SWIGLU, one column: the output in the xq layout instead of f32 (gemv.hpp)
};



// rows per workgroup by division (kernels that do not get them from the host)
#define GEMV_HOT_SPLIT const int h_q = (int)((unsigned)h_rows / (unsigned)nblk), h_r = h_rows - h_q * nblk;
// the body's hot fields straight from the argument block
#define GEMV_HOT_FROM_ARGS(a)                                                                                  \
    const float *const h_x = (a).x, *const h_norm_w = (a).norm_w;                                              \
    const int32_t *const h_expert_ids = (a).expert_ids, *const h_items = (a).items;                            \
    const uint8_t *const h_wbase0 = (a).wbase[0], *const h_wbase1 = (a).wbase[1], *const h_wbase2 = (a).wbase[2]; \
    const int h_K = (a).K, h_ldx = (a).ldx, h_ks = (a).ks, h_rows = (a).tile_begin[3], h_begin1 = (a).tile_begin[1], \
              h_begin2 = (a).tile_begin[2], h_x_div = (a).x_div;                                               \
    const size_t h_expert_stride = (a).expert_stride;                                                          \
    GEMV_HOT_SPLIT

// ------------------------------------------------------------------------------------------------ kernel
// Work decomposition.  A workgroup owns `rows_here` consecutive tile-rows (16 output rows each) of the launch's
// matrices (all of one K-quant type) and stages the activations once.  Its 16 waves are arranged KS x RS: wave
// (ks, rs) takes super-blocks ks, ks+KS, ... of the local tile-rows rs, rs+RS, ..., for NU matrices each (2 for the
// fused gate/up pair).  A wave walks its tiles as one flat list with the next tile always in flight; at the end of
// each (tile-row, matrix) segment the lanes' sums are reduced over the 4 lanes of a row and parked in LDS, where the
// KS partials of a row meet after one barrier.
// The arguments every wave needs before it can issue its first loads come first and as scalars: the build asks for
// kernel-argument preloading (-amdgpu-kernarg-preload-count), which delivers the leading scalar arguments in SGPRs at
// wave start instead of through a scalar load that misses every cache (the argument block was just written by the
// host).  The struct carries the same fields; the preloaded copies replace them.
// Fourteen dwords can be preloaded: the small integers travel packed (p_ldx_grid = ldx | gridDim.x << 16, p_rows_q =
// total tile-rows | tile-rows per workgroup << 16, p_begins = first tile-row of matrix 1 | of matrix 2 << 16,
// p_r_nsb_ks = workgroups with one tile-row more | K / 256 << 16 | waves along K << 24), and whether the launch uses the per-pair expert
// indirection is a template parameter, so that the dense kernel does not wait for a pointer only to find it null.
// XQ: p_x points at activations in the xq layout (gemv.hpp) instead of an f32 vector.
template <int TYPE, int NB, int NU, bool EXPERT, bool XQ>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_dot_kernel(const float *p_x, const float *p_norm_w, const uint8_t *p_wbase0,
                                                                const uint8_t *p_wbase1, const uint8_t *p_wbase2, unsigned p_ldx_grid,
                                                                unsigned p_rows_q, unsigned p_begins, unsigned p_r_nsb_ks,
                                                                const GemvKernelArgs a_in) {
    const GemvKernelArgs &a = a_in;
    const float *const h_x = p_x, *const h_norm_w = p_norm_w;
    const int32_t *const h_expert_ids = EXPERT ? a.expert_ids : nullptr, *const h_items = nullptr;
    const uint8_t *const h_wbase0 = p_wbase0, *const h_wbase1 = p_wbase1, *const h_wbase2 = p_wbase2;
    const int h_K = (int)((p_r_nsb_ks >> 16) & 0xFFu) * QK_K, h_ldx = (int)(p_ldx_grid & 0xFFFFu), h_ks = (int)(p_r_nsb_ks >> 24),
              h_rows = (int)(p_rows_q & 0xFFFFu), h_begin1 = (int)(p_begins & 0xFFFFu), h_begin2 = (int)(p_begins >> 16),
              h_q = (int)(p_rows_q >> 16), h_r = (int)(p_r_nsb_ks & 0xFFFFu), h_x_div = EXPERT ? a.x_div : 1;
    const size_t h_expert_stride = EXPERT ? a.expert_stride : 0;
    (void)h_rows;
    const int bid = blockIdx.x;      // (the workgroup count is folded into h_q / h_r: gridDim.x would be one more load from the argument block)
    constexpr bool GROUPED = false, XQ_IN = XQ;
    constexpr int THREADS = GEMV_THREADS, WAVES = GEMV_WAVES;
#include "gemv_body.inc"
}

// Expert matrices over pairs grouped by expert: the workgroup runs the body with as many columns as its item has pairs.
// Workgroups of GROUPED_THREADS: four share a compute unit, so that some stream tiles while others are between their
// dependent start-up loads (work item -> expert -> activations) or in their epilogue.
constexpr int GROUPED_THREADS = 256;
template <int TYPE, int NU>
__global__ __launch_bounds__(GROUPED_THREADS) void gemv_grouped_kernel(const int32_t *p_items, const int32_t *p_n_items, const float *p_x,
                                                                       const float *p_norm_w, const uint8_t *p_wbase0, unsigned p_nsb_ks_rows,
                                                                       unsigned p_ldx_xdiv, unsigned p_expert_stride, int p_w1_delta,
                                                                       const GemvKernelArgs a) {
    // (leading scalar arguments, preloaded into SGPRs, see gemv_dot_kernel: p_nsb_ks_rows = K / 256 | waves along K << 8 |
    // tile-rows << 16, p_ldx_xdiv = ldx | x_div << 16, the expert stride in bytes, and the second matrix's base as a
    // distance from the first in units of 256 bytes)
    const int p_K = (int)(p_nsb_ks_rows & 0xFFu) * QK_K, p_ks = (int)((p_nsb_ks_rows >> 8) & 0xFFu), p_rows = (int)(p_nsb_ks_rows >> 16);
    const int p_ldx = (int)(p_ldx_xdiv & 0xFFFFu);
    if ((int)blockIdx.y >= p_n_items[0]) return;
    const int bid = blockIdx.x, nblk = gridDim.x;
    constexpr bool GROUPED = true, XQ_IN = false;
    constexpr int THREADS = GROUPED_THREADS, WAVES = GROUPED_THREADS / 64;
    const int n = __builtin_amdgcn_readfirstlane(p_items[(size_t)blockIdx.y * MOE_ITEM_INTS + 1]);
    const float *const h_x = p_x, *const h_norm_w = p_norm_w;
    const int32_t *const h_expert_ids = nullptr, *const h_items = p_items;
    const uint8_t *const h_wbase0 = p_wbase0, *const h_wbase1 = p_wbase0 + (ptrdiff_t)p_w1_delta * 256, *const h_wbase2 = h_wbase1;
    const int h_K = p_K, h_ldx = p_ldx, h_ks = p_ks, h_rows = p_rows, h_begin1 = p_rows, h_begin2 = p_rows, h_x_div = (int)(p_ldx_xdiv >> 16);
    const size_t h_expert_stride = p_expert_stride;
    GEMV_HOT_SPLIT
    if (n == 4) {
        constexpr int NB = 4;
#include "gemv_body.inc"
    } else if (n == 3) {
        constexpr int NB = 3;
#include "gemv_body.inc"
    } else if (n == 2) {
        constexpr int NB = 2;
#include "gemv_body.inc"
    } else if (n == 1) {
        constexpr int NB = 1;
#include "gemv_body.inc"
    }
}

// q/k/v groups whose matrices are of both K-quant types (attn_v in q6_K on the "more bits" layers of a Q4_K_M
// file): one launch, the first n4 workgroups run the q4_K matrices, the rest the q6_K ones.
// Preloaded (see gemv_dot_kernel): the activations, both bases of the q4_K part, the first base of the q6_K part and
// the packed integers p_ldx_n4 = ldx | n4 << 16, p_rows = tile-rows of the q4_K part | of the q6_K part << 16,
// p_begin_grid = first tile-row of the q4_K part's second matrix | gridDim.x << 16, p_nsb_ks = K / 256 | waves along K
// << 8.  SIMPLE: the q4_K part has at most two matrices and the q6_K part one (q, k | v, the usual case), so nothing
// else is needed before the first weight load; otherwise the remaining bases and boundaries come from the structs.
template <int NB, bool SIMPLE>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_dual_kernel(const float *p_x, const float *p_norm_w, const uint8_t *p_w4, const uint8_t *p_w4b,
                                                                 const uint8_t *p_w6, unsigned p_ldx_n4, unsigned p_rows, unsigned p_begin_grid,
                                                                 unsigned p_nsb_ks, const GemvKernelArgs a4, const GemvKernelArgs a6) {
    constexpr int NU = 1;
    constexpr bool GROUPED = false, XQ_IN = false;
    constexpr int THREADS = GEMV_THREADS, WAVES = GEMV_WAVES;
    const int n4 = (int)(p_ldx_n4 >> 16);
    const float *const h_x = p_x, *const h_norm_w = p_norm_w;
    const int32_t *const h_expert_ids = nullptr, *const h_items = nullptr;
    const int h_K = (int)(p_nsb_ks & 0xFFu) * QK_K, h_ldx = (int)(p_ldx_n4 & 0xFFFFu), h_ks = (int)(p_nsb_ks >> 8), h_x_div = 1;
    const size_t h_expert_stride = 0;
    if ((int)blockIdx.x < n4) {
        const GemvKernelArgs &a = a4;
        constexpr int TYPE = MESH_Q4_K;
        const int bid = blockIdx.x, nblk = n4;
        const int h_rows = (int)(p_rows & 0xFFFFu), h_begin1 = (int)(p_begin_grid & 0xFFFFu), h_begin2 = SIMPLE ? h_rows : a.tile_begin[2];
        const uint8_t *const h_wbase0 = p_w4, *const h_wbase1 = p_w4b, *const h_wbase2 = SIMPLE ? p_w4b : a.wbase[2];
        GEMV_HOT_SPLIT
#include "gemv_body.inc"
    } else {
        const GemvKernelArgs &a = a6;
        constexpr int TYPE = MESH_Q6_K;
        const int bid = (int)blockIdx.x - n4, nblk = (int)(p_begin_grid >> 16) - n4;
        const int h_rows = (int)(p_rows >> 16), h_begin1 = SIMPLE ? h_rows : a.tile_begin[1], h_begin2 = SIMPLE ? h_rows : a.tile_begin[2];
        const uint8_t *const h_wbase0 = p_w6, *const h_wbase1 = SIMPLE ? p_w6 : a.wbase[1], *const h_wbase2 = SIMPLE ? p_w6 : a.wbase[2];
        GEMV_HOT_SPLIT
#include "gemv_body.inc"
    }
}

constexpr size_t LDS_LIMIT = 160 * 1024;
constexpr int MAX_ROWS_X_KS = 64;       // bound on (tile-rows per workgroup) x KS, sizes the LDS partial buffer

static size_t dot_smem_bytes(int type, int NB, int K, int rows_here, int KS, int NU, int waves = GEMV_WAVES) {
    return (size_t)NB * (2 * (size_t)K + (size_t)(K / 32) * 8 + (type == MESH_Q6_K ? (size_t)(K / 16) * 4 : 0)) +
           sizeof(float) * ((size_t)KS * rows_here * NU * 16 * NB + waves * NB);
}

template <int TYPE, int NB, int NU, bool EXPERT = false, bool XQ = false>
static int launch_dot(const GemvKernelArgs &ka, dim3 grid, size_t smem, hipStream_t stream) {
    if (ka.tile_begin[3] > 0xFFFF || ka.ldx > 0xFFFF || grid.x > 0xFFFFu || ka.K / QK_K > 0xFF)
        return fail(MESH_ERR_UNSUPPORTED, "gemv: %d tile-rows / activation stride %d / %u workgroups / row length %d in one launch",
                    ka.tile_begin[3], ka.ldx, grid.x, ka.K);
    const unsigned rows = (unsigned)ka.tile_begin[3], q = rows / grid.x, r = rows % grid.x;
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_dot_kernel<TYPE, NB, NU, EXPERT, XQ>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT));
        attr_set = true;
    }
    MESH_LAUNCH((gemv_dot_kernel<TYPE, NB, NU, EXPERT, XQ>), grid, dim3(GEMV_THREADS), smem, stream, 
        ka.x, ka.norm_w, ka.wbase[0], ka.wbase[1], ka.wbase[2], (unsigned)ka.ldx | (grid.x << 16), rows | (q << 16),
        (unsigned)ka.tile_begin[1] | ((unsigned)ka.tile_begin[2] << 16), r | ((unsigned)(ka.K / QK_K) << 16) | ((unsigned)ka.ks << 24), ka);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

template <int TYPE, int NU>
static int launch_grouped(const GemvKernelArgs &ka, dim3 grid, size_t smem, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_grouped_kernel<TYPE, NU>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT));
        attr_set = true;
    }
    const ptrdiff_t w1d = ka.wbase[1] ? ka.wbase[1] - ka.wbase[0] : 0;
    if (ka.K / QK_K > 0xFF || ka.tile_begin[3] > 0xFFFF || ka.ldx > 0xFFFF || ka.x_div > 0xFFFF || ka.expert_stride > 0xFFFFFFFFull || (w1d & 255) ||
        w1d / 256 > INT32_MAX || w1d / 256 < INT32_MIN)
        return fail(MESH_ERR_UNSUPPORTED, "gemv: grouped expert launch outside its packed argument ranges");
    MESH_LAUNCH((gemv_grouped_kernel<TYPE, NU>), grid, dim3(GROUPED_THREADS), smem, stream, 
        ka.items, ka.n_items, ka.x, ka.norm_w, ka.wbase[0], (unsigned)(ka.K / QK_K) | ((unsigned)ka.ks << 8) | ((unsigned)ka.tile_begin[3] << 16),
        (unsigned)ka.ldx | ((unsigned)ka.x_div << 16), (unsigned)ka.expert_stride, (int)(w1d / 256), ka);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

template <int TYPE, int NU>
static int launch_dot_nb(int nb, const GemvKernelArgs &ka, dim3 grid, size_t smem, hipStream_t stream) {
    if (nb == 4) return launch_dot<TYPE, 4, NU>(ka, grid, smem, stream);
    if (nb == 3) return launch_dot<TYPE, 3, NU>(ka, grid, smem, stream);
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

// Launch geometry of the K-quant matrices of `a` (all of one type) over `ncu` compute units.
struct KquantPlan {
    GemvKernelArgs ka;
    int type, NU, KS, grid, rows_max;
};
static int plan_kquant(const GemvArgs &a, int ncu, KquantPlan &p, int waves = GEMV_WAVES) {
    const int type = a.mat[0].type;
    const int nsb = a.K / QK_K, NU = a.epi == EPI_SWIGLU ? 2 : 1;
    const size_t row_stride = (size_t)nsb * (type == MESH_Q4_K ? Q4K_TILE_BYTES : Q6K_TILE_BYTES);
    GemvKernelArgs &ka = p.ka;
    ka = GemvKernelArgs{};
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
    const int n_mat_k = NU == 2 ? 1 : a.n_mat;      // boundaries the kernel searches
    for (int i = n_mat_k; i < 4; ++i) ka.tile_begin[i] = total_rows;      // unused slots compare as "beyond the end"
    ka.n_mat = n_mat_k;
    ka.ldx = a.ldx;
    ka.K = a.K;
    ka.norm_w = a.norm_w;
    ka.eps = a.eps;
    ka.ldres = a.ldres;
    ka.epi = a.epi;
    ka.rope = a.rope;
    int KS = 1;
    while (KS * 2 <= nsb && KS * 2 <= waves) KS *= 2;      // a power of two: the kernel splits its waves with shifts
    if (waves != GEMV_WAVES) {
        // half-size workgroups: every wave gets work only if KS divides the waves, evenly only if it divides the row too
        KS = 1;
        for (int d = waves; d > 1; d >>= 1)
            if (d <= nsb && nsb % d == 0) { KS = d; break; }
    }
    ka.ks = KS;
    // tile-rows per workgroup: spread over the CUs, bounded by the LDS partial buffer
    int rows_per_wg = (total_rows + ncu - 1) / ncu;
    rows_per_wg = std::max(1, std::min(rows_per_wg, MAX_ROWS_X_KS / KS));
    p.grid = (total_rows + rows_per_wg - 1) / rows_per_wg;
    p.rows_max = (total_rows + p.grid - 1) / p.grid;
    p.type = type; p.NU = NU; p.KS = KS;
    if (total_rows > 0xFFFF || p.grid > 0xFFFF) return fail(MESH_ERR_UNSUPPORTED, "gemv: %d tile-rows over %d workgroups in one launch", total_rows, p.grid);
    if (dot_smem_bytes(type, 1, a.K, p.rows_max, KS, NU) > LDS_LIMIT) return fail(MESH_ERR_UNSUPPORTED, "gemv: row length %d does not fit LDS", a.K);
    return MESH_OK;
}

// All matrices of `a` are tiled K-quants of one type.
static int gemv_kquant(const GemvArgs &a, hipStream_t stream) {
    const int n_pairs = a.expert_ids ? (a.items ? a.max_items : a.n_pairs) : 1;       // workgroup columns of the grid
    if (a.expert_ids && (a.n_pairs <= 0 || a.x_div <= 0 || a.epi == EPI_RESIDUAL)) return fail(MESH_ERR_INVALID, "gemv: bad expert-indirection arguments");
    if (a.items && (!a.expert_ids || !a.n_items || a.max_items <= 0)) return fail(MESH_ERR_INVALID, "gemv: bad grouped-expert arguments");
    KquantPlan plan;
    // (grouped launches: workgroups of a quarter of the size, several times as many per item)
    const int oversub = std::max(1, a.grouped_oversub);
    int rc0 = a.items ? plan_kquant(a, std::max(1, oversub * n_compute_units() / n_pairs), plan, GROUPED_THREADS / 64)
                      : plan_kquant(a, std::max(1, n_compute_units() / n_pairs), plan);
    if (rc0 != MESH_OK) return rc0;
    GemvKernelArgs &ka = plan.ka;
    const int type = plan.type, NU = plan.NU, KS = plan.KS, grid = plan.grid, rows_max = plan.rows_max;
    if (a.expert_ids) {
        ka.expert_ids = a.expert_ids;
        ka.expert_stride = (size_t)tiled_bytes(type, a.mat[0].M, a.K);
        ka.x_div = a.x_div;
    }
    if (a.items) {
        // pairs of one expert share a pass over its weights, up to MOE_ITEM_PAIRS columns per workgroup
        int nb = MOE_ITEM_PAIRS;
        if (dot_smem_bytes(type, nb, a.K, rows_max, KS, NU, GROUPED_THREADS / 64) > LDS_LIMIT) return fail(MESH_ERR_UNSUPPORTED, "gemv: row length %d does not fit LDS with %d columns", a.K, nb);
        ka.x = a.x;
        ka.items = a.items;
        ka.n_items = a.n_items;
        const size_t smem = dot_smem_bytes(type, nb, a.K, rows_max, KS, NU, GROUPED_THREADS / 64);
        const dim3 g((unsigned)grid, (unsigned)a.max_items);
        if (type == MESH_Q4_K) return NU == 2 ? launch_grouped<MESH_Q4_K, 2>(ka, g, smem, stream) : launch_grouped<MESH_Q4_K, 1>(ka, g, smem, stream);
        return NU == 2 ? launch_grouped<MESH_Q6_K, 2>(ka, g, smem, stream) : launch_grouped<MESH_Q6_K, 1>(ka, g, smem, stream);
    }
    if (a.expert_ids) {
        // every pair is its own single-column product
        ka.x = a.x;
        const size_t smem = dot_smem_bytes(type, 1, a.K, rows_max, KS, NU);
        const dim3 g((unsigned)grid, (unsigned)n_pairs);
        if (type == MESH_Q4_K) return NU == 2 ? launch_dot<MESH_Q4_K, 1, 2, true>(ka, g, smem, stream) : launch_dot<MESH_Q4_K, 1, 1, true>(ka, g, smem, stream);
        return NU == 2 ? launch_dot<MESH_Q6_K, 1, 2, true>(ka, g, smem, stream) : launch_dot<MESH_Q6_K, 1, 1, true>(ka, g, smem, stream);
    }
    if (a.xq_out) {
        if (!gemv_xq_out_supported(a)) return fail(MESH_ERR_INVALID, "gemv: xq output asked of a launch that cannot produce it");
        ka.xq_out = a.xq_out;
    }
    if (a.xq_in) {
        // one column from a quantised vector: the activations argument is that buffer
        if (!gemv_xq_in_supported(a)) return fail(MESH_ERR_INVALID, "gemv: xq input asked of a launch that cannot read it");
        GemvKernelArgs kb = ka;
        kb.x = reinterpret_cast<const float *>(a.xq_in);
        kb.residual = a.residual;
        const size_t smem = dot_smem_bytes(type, 1, a.K, rows_max, KS, NU);
        const dim3 g((unsigned)grid);
        return type == MESH_Q4_K ? launch_dot<MESH_Q4_K, 1, 1, false, true>(kb, g, smem, stream) : launch_dot<MESH_Q6_K, 1, 1, false, true>(kb, g, smem, stream);
    }
    int t = 0;
    while (t < a.T) {
        const int left = a.T - t;
        int nb = left >= 4 ? 4 : left;      // 3 columns have a kernel of their own: no second pass over the weights
        while (nb > 1 && dot_smem_bytes(type, nb, a.K, rows_max, KS, NU) > LDS_LIMIT) --nb;
        GemvKernelArgs kb = ka;
        if (kb.rope.pos) { kb.rope.pos += t; kb.rope.seq += t; }
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

template <int NB, bool SIMPLE>
static int launch_dual2(const GemvKernelArgs &k4, const GemvKernelArgs &k6, int n4, int n6, size_t smem, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_dual_kernel<NB, SIMPLE>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT));
        attr_set = true;
    }
    MESH_LAUNCH((gemv_dual_kernel<NB, SIMPLE>), dim3((unsigned)(n4 + n6)), dim3(GEMV_THREADS), smem, stream, 
        k4.x, k4.norm_w, k4.wbase[0], k4.wbase[1], k6.wbase[0], (unsigned)k4.ldx | ((unsigned)n4 << 16),
        (unsigned)k4.tile_begin[3] | ((unsigned)k6.tile_begin[3] << 16), (unsigned)k4.tile_begin[1] | ((unsigned)(n4 + n6) << 16),
        (unsigned)(k4.K / QK_K) | ((unsigned)k4.ks << 8), k4, k6);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}
template <int NB>
static int launch_dual(const GemvKernelArgs &k4, const GemvKernelArgs &k6, int n4, int n6, size_t smem, hipStream_t stream) {
    if (k4.ldx > 0xFFFF || k4.K / QK_K > 0xFF || k4.ks != k6.ks || n4 + n6 > 0xFFFF || k4.tile_begin[3] > 0xFFFF || k6.tile_begin[3] > 0xFFFF)
        return fail(MESH_ERR_UNSUPPORTED, "gemv: two-type launch outside its packed argument ranges");
    const bool simple = k4.n_mat <= 2 && k6.n_mat == 1;
    return simple ? launch_dual2<NB, true>(k4, k6, n4, n6, smem, stream) : launch_dual2<NB, false>(k4, k6, n4, n6, smem, stream);
}
// a4: the q4_K matrices of a group, a6: its q6_K matrices; same activations, plain store epilogue
static int gemv_dual(const GemvArgs &a4, const GemvArgs &a6, hipStream_t stream) {
    const int ncu = n_compute_units();
    double b4 = 0, b6 = 0;
    for (int i = 0; i < a4.n_mat; ++i) b4 += (double)tiled_bytes(MESH_Q4_K, a4.mat[i].M, a4.K);
    for (int i = 0; i < a6.n_mat; ++i) b6 += (double)tiled_bytes(MESH_Q6_K, a6.mat[i].M, a6.K);
    int c6 = (int)(ncu * b6 / (b4 + b6) + 0.5);              // compute units in proportion to the bytes streamed
    c6 = std::max(1, std::min(ncu - 1, c6));
    KquantPlan p4, p6;
    int rc;
    if ((rc = plan_kquant(a4, ncu - c6, p4)) != MESH_OK || (rc = plan_kquant(a6, c6, p6)) != MESH_OK) return rc;
    int t = 0;
    while (t < a4.T) {
        const int left = a4.T - t;
        int nb = left >= 4 ? 4 : left;
        auto need = [&](int n) { return std::max(dot_smem_bytes(MESH_Q4_K, n, a4.K, p4.rows_max, p4.KS, 1), dot_smem_bytes(MESH_Q6_K, n, a6.K, p6.rows_max, p6.KS, 1)); };
        while (nb > 1 && need(nb) > LDS_LIMIT) --nb;
        GemvKernelArgs k4 = p4.ka, k6 = p6.ka;
        if (k4.rope.pos) { k4.rope.pos += t; k4.rope.seq += t; k6.rope.pos += t; k6.rope.seq += t; }
        k4.x = k6.x = a4.x + (size_t)t * a4.ldx;
        for (int i = 0; i < a4.n_mat; ++i) k4.y[i] = a4.mat[i].y + (size_t)t * a4.mat[i].ldy;
        for (int i = 0; i < a6.n_mat; ++i) k6.y[i] = a6.mat[i].y + (size_t)t * a6.mat[i].ldy;
        if (nb == 4) rc = launch_dual<4>(k4, k6, p4.grid, p6.grid, need(4), stream);
        else if (nb == 3) rc = launch_dual<3>(k4, k6, p4.grid, p6.grid, need(3), stream);
        else if (nb == 2) rc = launch_dual<2>(k4, k6, p4.grid, p6.grid, need(2), stream);
        else rc = launch_dual<1>(k4, k6, p4.grid, p6.grid, need(1), stream);
        if (rc != MESH_OK) return rc;
        t += nb;
    }
    return MESH_OK;
}

static bool all_tiled_one_type(const GemvArgs &a) {
    for (int i = 0; i < a.n_mat; ++i)
        if (!type_is_tiled(a.mat[i].type) || a.mat[i].type != a.mat[0].type) return false;
    return a.n_mat >= 1;
}

// The SwiGLU launch of one column can leave its output quantised when every workgroup owns whole 32-element blocks
// of it: an even number of 16-row tile-rows each, the same for all.
bool gemv_xq_out_supported(const GemvArgs &a) {
    if (a.epi != EPI_SWIGLU || a.n_mat != 2 || a.T != 1 || a.expert_ids || !all_tiled_one_type(a) || a.mat[0].M != a.mat[1].M) return false;
    if (a.mat[0].M % 32 || a.mat[0].M % QK_K || a.K % QK_K) return false;
    KquantPlan p;
    if (plan_kquant(a, n_compute_units(), p) != MESH_OK) return false;
    const int total = a.mat[0].M / TILE_ROWS;
    return total % p.grid == 0 && (total / p.grid) % 2 == 0;
}

bool gemv_xq_in_supported(const GemvArgs &a) {
    return a.T == 1 && a.n_mat == 1 && !a.expert_ids && !a.norm_w && !a.rope.pos && all_tiled_one_type(a) && a.K % QK_K == 0 &&
           (a.epi == EPI_STORE || a.epi == EPI_RESIDUAL);
}

bool gemv_can_fuse_rope(const GemvArgs &a) {
    if (!a.rope.pos || a.epi != EPI_STORE || a.expert_ids || a.rope.head_dim % 2 || a.rope.n_rot % 2) return false;
    for (int i = 0; i < a.n_mat; ++i)
        if (a.mat[i].type != MESH_Q4_K && a.mat[i].type != MESH_Q6_K) return false;
    return true;
}

int gemv(const GemvArgs &a, hipStream_t stream) {
    if (a.rope.pos && !gemv_can_fuse_rope(a)) return fail(MESH_ERR_INVALID, "gemv: rope epilogue asked for a launch that cannot carry it");
    if (a.n_mat < 1 || a.n_mat > 3 || (!a.x && !a.xq_in) || a.K <= 0 || a.T < 0)
        return fail(MESH_ERR_INVALID, "gemv: bad arguments (n_mat %d, K %d, T %d)", a.n_mat, a.K, a.T);
    if (a.epi == EPI_SWIGLU && a.n_mat != 2) return fail(MESH_ERR_INVALID, "gemv: swiglu needs exactly gate and up");
    if (a.epi == EPI_SWIGLU && a.mat[0].M != a.mat[1].M) return fail(MESH_ERR_INVALID, "gemv: gate and up differ in rows");
    if (a.epi == EPI_RESIDUAL && !a.residual) return fail(MESH_ERR_INVALID, "gemv: residual epilogue without residual");
    if (!a.xq_in && ((a.ldx % 4) || (reinterpret_cast<uintptr_t>(a.x) & 15))) return fail(MESH_ERR_INVALID, "gemv: x must be 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(a.xq_in) & 15) || (reinterpret_cast<uintptr_t>(a.xq_out) & 15)) return fail(MESH_ERR_INVALID, "gemv: xq buffers must be 16-byte aligned");
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
    // the common mix -- every matrix q4_K or q6_K, plain store -- runs as one two-type launch
    {
        GemvArgs a4 = a, a6 = a;
        a4.n_mat = a6.n_mat = 0;
        bool kq_only = a.epi == EPI_STORE && !a.expert_ids;
        for (int i = 0; i < a.n_mat && kq_only; ++i) {
            if (a.mat[i].type == MESH_Q4_K) { a4.kind[a4.n_mat] = a.kind[i]; a4.mat[a4.n_mat++] = a.mat[i]; }
            else if (a.mat[i].type == MESH_Q6_K) { a6.kind[a6.n_mat] = a.kind[i]; a6.mat[a6.n_mat++] = a.mat[i]; }
            else kq_only = false;
        }
        if (kq_only && a4.n_mat > 0 && a6.n_mat > 0) return gemv_dual(a4, a6, stream);
    }
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
