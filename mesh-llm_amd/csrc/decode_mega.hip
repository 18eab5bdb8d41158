// Persistent decode kernel: one launch runs every layer of the stage for a small batch of single-token sequences.
//
// Why: a decode step is a chain of ~100 small dependent operators.  Run as separate launches, each one pays its
// own latency chain (launch, activation fetch, first weight tile from HBM, reduction) during which HBM idles; the
// weights -- 98% of the bytes -- do not depend on the activations at all.  Here one 512-thread workgroup per CU
// stays resident for the whole step.  Phases (q/k/v, attention, split merge, o, gate/up, down) are separated by
// a grid barrier, and before a wave arrives at a barrier it issues the loads of its first weight tiles (or KV
// rows) of the NEXT phase, so HBM keeps streaming while the barrier and the activation hand-over run.
//
// Activations move between phases through a small UNCACHED device buffer with device-scope loads and stores, so
// no cache write-back or invalidate is needed between phases.  Vectors that every workgroup reads (x, the
// attention output, the FFN activation) are written to several replicas so that the readers do not all hit the
// same memory channel.
//
// The same per-layer graph as stage.hip's run_layers (rpc_server::graph_compute,
// third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451), restricted to what a
// pure decode batch needs: dense layers, K-quant matrices, head_dim 128, every token in its own sequence.
//
// Safety: the grid barrier spins a bounded number of times; on timeout it raises an abort flag that every later
// barrier and phase observes, so all workgroups drain and the host reports an error instead of hanging.

#include "decode_mega.hpp"

#include "gemv_device.hpp"

namespace mesh {

constexpr int MEGA_THREADS = 512;           // 8 waves per CU: 256 VGPRs each, which is what holds four weight tiles per wave in flight
constexpr int MEGA_WAVES = MEGA_THREADS / 64;
constexpr int HD = 128;                     // head_dim this kernel is built for
constexpr int LPK = HD / 8;                 // lanes per key
constexpr int SLOTS = MEGA_THREADS / LPK;   // keys visited side by side
constexpr int DEPTH = 4;                    // weight tiles a wave keeps in flight
constexpr int KPT = 4;                      // keys per thread and pass in the attention phase

// Phase timestamps for tuning builds (-DMESH_MEGA_TRACE); compiled out of the product.
#ifdef MESH_MEGA_TRACE
__device__ unsigned long long *g_mega_trace = nullptr;      // [phase][workgroup][8]
#define MEGA_MARK(ip, k)                                                                                     \
    do {                                                                                                     \
        if (g_mega_trace && threadIdx.x == 0) g_mega_trace[((size_t)(ip) * gridDim.x + blockIdx.x) * 8 + (k)] = wall_clock64(); \
    } while (0)
#else
#define MEGA_MARK(ip, k) do { } while (0)
#endif
#define MEGA_SUBMARK(k) MEGA_MARK(g.phase, k)

// ------------------------------------------------------------------------------------------------ exchange buffers
// Every access is a device-scope load or store: it misses the CU's vector cache by construction and the L2 does
// not keep uncached lines.  Draining the wave's own stores (vmcnt 0) before it arrives at the grid barrier is all
// the ordering there is.
__device__ __forceinline__ float xld(const float *p) {
    return __hip_atomic_load(as_global<const float>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 xld2(const float *p) {       // 8-byte aligned
    const unsigned long long v = __hip_atomic_load(as_global<const unsigned long long>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(__uint_as_float((unsigned)v), __uint_as_float((unsigned)(v >> 32)));
}
__device__ __forceinline__ void xst(float *p, float v) {
    __hip_atomic_store(as_global<float>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// replica of a broadcast vector this workgroup reads
__device__ __forceinline__ int my_replica() { return (int)(blockIdx.x % MEGA_REPLICAS); }

template <int NB>
__device__ __forceinline__ void x_fetch_exchange(XRegs<NB> &X, const float *x, int ldx, int g, bool live) {
#pragma unroll
    for (int t = 0; t < NB; ++t) {
        X.a[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        X.b[t] = X.a[t];
        if (live) {
            const float *p = x + (size_t)t * ldx + g * 8;
            const float2 v0 = xld2(p), v1 = xld2(p + 2), v2 = xld2(p + 4), v3 = xld2(p + 6);
            X.a[t] = make_float4(v0.x, v0.y, v1.x, v1.y);
            X.b[t] = make_float4(v2.x, v2.y, v3.x, v3.y);
        }
    }
}

// ------------------------------------------------------------------------------------------------ grid barrier
struct GridSync {
    unsigned *counter;
    int *abort_flag;
    unsigned target;       // value the counter reaches when every workgroup has arrived at the next barrier
    unsigned n_wg;
    unsigned spin_limit;
    bool dead;
    int phase;             // index of the running phase (tuning builds label their timestamps with it)
};

// Workgroup barrier that orders LDS only: unlike __syncthreads() it does not wait for outstanding global loads,
// which is what lets prefetches stay in flight across it.
__device__ __forceinline__ void wg_barrier_lds() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Arrival: each wave waits for its own outstanding stores, then issues `prefetch` (loads for the next phase that
// do not depend on what other workgroups are still writing); the workgroup barrier collects the waves, thread 0
// counts the workgroup in and polls until all have arrived.
template <typename PrefetchFn>
__device__ __forceinline__ void grid_barrier(GridSync &g, PrefetchFn prefetch) {
    __builtin_amdgcn_s_waitcnt(0);          // vmcnt(0) expcnt(0) lgkmcnt(0): this wave's exchange stores are done
    prefetch();
    wg_barrier_lds();
    __shared__ int s_dead;
    if (threadIdx.x == 0) {
        int dead = g.dead ? 1 : 0;
        if (!dead) {
            __hip_atomic_fetch_add(g.counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            unsigned spins = 0;
            while ((int)(__hip_atomic_load(g.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - g.target) < 0) {
                ++spins;
                if (spins > g.spin_limit || ((spins & 63u) == 0 && __hip_atomic_load(g.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                    __hip_atomic_store(g.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    dead = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        s_dead = dead;
    }
    wg_barrier_lds();
    g.dead = s_dead != 0;
    g.target += g.n_wg;
}

// ------------------------------------------------------------------------------------------------ GEMV phase
// A weight tile of either K-quant type as raw registers: what a wave carries across a grid barrier.
struct RawTile {
    uint4 a, b, c, d;
    uint32_t e;
};

__device__ __forceinline__ void load_raw(RawTile &r, int type, const uint8_t *tile, int lane) {
    if (type == MESH_Q4_K) {
        TileRegs<MESH_Q4_K> t;
        t.load(tile, lane);
        r.a = t.hdr; r.b = t.qa; r.c = t.qb;
    } else {
        TileRegs<MESH_Q6_K> t;
        t.load(tile, lane);
        r.a = t.qla; r.b = t.qlb; r.c = t.qh; r.d = t.sc; r.e = t.d;
    }
}
__device__ __forceinline__ void from_raw(TileRegs<MESH_Q4_K> &t, const RawTile &r) { t.hdr = r.a; t.qa = r.b; t.qb = r.c; }
__device__ __forceinline__ void from_raw(TileRegs<MESH_Q6_K> &t, const RawTile &r) { t.qla = r.a; t.qlb = r.b; t.qh = r.c; t.sc = r.d; t.d = r.e; }

// The rows of part pi that a workgroup owning tile-rows [g0, g1) of the phase has.
struct PartSpan {
    int tr0, rows, red_row0;
};
__device__ __forceinline__ bool part_span(const MegaPhase &ph, int g0, int g1, int pi, PartSpan &s) {
    const MegaPart &p = ph.part[pi];
    const int p_rows = (p.M + TILE_ROWS - 1) / TILE_ROWS;
    const int lo = g0 > p.begin ? g0 : p.begin;
    const int hi = g1 < p.begin + p_rows ? g1 : p.begin + p_rows;
    s.tr0 = lo - p.begin; s.rows = hi - lo; s.red_row0 = lo - g0;
    return hi > lo;
}

// Loads of the first DEPTH tiles this wave will need in phase `ph` (the first part the workgroup owns rows of).
// run_part() below recomputes the same walk and takes the tiles from r[] instead of loading them.
__device__ __forceinline__ void prefetch_tiles(const MegaPhase &ph, RawTile (&r)[DEPTH]) {
    const int g0 = (int)(((long long)blockIdx.x * ph.total_rows) / gridDim.x);
    const int g1 = (int)(((long long)(blockIdx.x + 1) * ph.total_rows) / gridDim.x);
    if (g1 <= g0) return;
    PartSpan sp;
    int pi = 0;
    while (pi < ph.n_part && !part_span(ph, g0, g1, pi, sp)) ++pi;
    if (pi >= ph.n_part) return;
    const MegaPart &p = ph.part[pi];
    const int nsb = ph.K / QK_K, KS = nsb < MEGA_WAVES ? nsb : MEGA_WAVES, RS = MEGA_WAVES / KS;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ks = wave % KS, rs = wave / KS;
    const int n_i = rs < RS ? (nsb - ks + KS - 1) / KS : 0;
    if (n_i <= 0) return;
    const int TB = p.type == MESH_Q4_K ? Q4K_TILE_BYTES : Q6K_TILE_BYTES, NU = p.W1 ? 2 : 1;
    const size_t row_stride = (size_t)nsb * TB;
    int j = rs, u = 0, ii = 0;
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        if (j < sp.rows) {
            load_raw(r[d], p.type, (u ? p.W1 : p.W0) + (size_t)(sp.tr0 + j) * row_stride + (size_t)(ks + KS * ii) * TB, lane);
            if (++ii == n_i) { ii = 0; if (++u == NU) { u = 0; j += RS; } }
        }
    }
}

// One type-homogeneous part of a phase.  A wave walks its tiles -- (tile-row, matrix, super-block) in one flat
// list -- with DEPTH tiles always in flight in registers.  The first DEPTH come from the prefetch (pre) or are
// loaded here; `stage` (activations into LDS) is run once per phase, by the first part, after those loads.
template <int TYPE, int NB, int NU, typename StageFn>
__device__ __forceinline__ void run_part(const MegaPart &p, const PartSpan &sp, int red_rows, int nsb, int KS, int RS, const XStage &S, int K,
                                         bool pre, const RawTile (&r)[DEPTH], bool stage_now, StageFn stage) {
    constexpr int TB = TileRegs<TYPE>::BYTES;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ks = wave % KS, rs = wave / KS;
    const int n_i = rs < RS ? (nsb - ks + KS - 1) / KS : 0;
    const int rows = n_i > 0 ? sp.rows : 0;      // a wave without tiles sees an empty part
    const size_t row_stride = (size_t)nsb * TB;
    auto tile_ptr = [&](const TileCursor<NU> &c) -> const uint8_t * {
        return (c.u ? p.W1 : p.W0) + (size_t)(sp.tr0 + c.j) * row_stride + (size_t)(ks + KS * c.ii) * TB;
    };
    TileCursor<NU> ld{rs, 0, 0}, cp{rs, 0, 0};
    TileRegs<TYPE> t[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        if (ld.j < rows) {
            if (pre) from_raw(t[d], r[d]); else t[d].load(tile_ptr(ld), lane);
            ld.advance(n_i, RS);
        }
    }
    if (stage_now) {
        stage();
        __syncthreads();
    }
    float acc[NB];
#pragma unroll
    for (int t2 = 0; t2 < NB; ++t2) acc[t2] = 0.f;
    auto finish_segment = [&](const TileCursor<NU> &c) {
#pragma unroll
        for (int t2 = 0; t2 < NB; ++t2) {
            float v = acc[t2];
            v += __shfl_xor(v, 1);
            v += __shfl_xor(v, 2);
            if ((lane & 3) == 0) S.red[(((ks * red_rows + sp.red_row0 + c.j) * 2 + c.u) * 16 + (lane >> 2)) * NB + t2] = v;
            acc[t2] = 0.f;
        }
    };
    bool more = cp.j < rows;
    while (more) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (more) {
                tile_compute<NB>(t[d], lane, ks + KS * cp.ii, S, K, acc);
                if (cp.ii + 1 == n_i) finish_segment(cp);
                cp.advance(n_i, RS);
                if (ld.j < rows) { t[d].load(tile_ptr(ld), lane); ld.advance(n_i, RS); }
                more = cp.j < rows;
            }
        }
    }
}

template <int NB>
__device__ __forceinline__ void gemv_phase(const MegaPhase &ph, float eps, const GridSync &g, const RawTile (&r)[DEPTH]) {
    extern __shared__ __align__(16) uint8_t smem[];      // declared here, not passed in: LDS accesses stay ds_* instructions
    const int K = ph.K, nsb = K / QK_K;
    XStage S;
    S.xh = reinterpret_cast<int8_t *>(smem);
    S.xl = S.xh + NB * K;
    S.xd = reinterpret_cast<float *>(S.xl + NB * K);
    S.xs = S.xd + NB * (K >> 5);
    S.xi16 = reinterpret_cast<int *>(S.xs + NB * (K >> 5));
    S.ssq = reinterpret_cast<float *>(S.xi16 + NB * (K >> 4));
    S.red = S.ssq + MEGA_WAVES * NB;                       // [KS][rows_here][2][16][NB]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    const int g0 = (int)(((long long)blockIdx.x * ph.total_rows) / gridDim.x);
    const int g1 = (int)(((long long)(blockIdx.x + 1) * ph.total_rows) / gridDim.x);
    const int rows_here = g1 - g0;
    if (g.dead || rows_here <= 0) return;       // uniform over the workgroup

    const float *norm_w = ph.norm_w;
    const float *xin = ph.x + (size_t)my_replica() * ph.x_rep_stride;
    auto stage = [&]() {
        const int ng = K >> 3;
        float ss[NB];
#pragma unroll
        for (int t = 0; t < NB; ++t) ss[t] = 0.f;
        for (int gg = tid; gg - tid < ng; gg += MEGA_THREADS) {
            XRegs<NB> X;
            x_fetch_exchange<NB>(X, xin, ph.ldx, gg, gg < ng);
            norm_fetch<NB>(X, norm_w, gg, gg < ng);
            x_quantise<NB, true>(X, K, S, gg, gg < ng, ss);
        }
        if (norm_w) {
#pragma unroll
            for (int t = 0; t < NB; ++t) {
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) ss[t] += __shfl_xor(ss[t], o);
                if (lane == 0) S.ssq[wave * NB + t] = ss[t];
            }
        }
        MEGA_SUBMARK(3);
    };
    const int KS = nsb < MEGA_WAVES ? nsb : MEGA_WAVES, RS = MEGA_WAVES / KS;
    bool first = true;
    for (int pi = 0; pi < ph.n_part; ++pi) {
        PartSpan sp;
        if (!part_span(ph, g0, g1, pi, sp)) continue;
        const MegaPart &p = ph.part[pi];
        if (p.W1) {
            if (p.type == MESH_Q4_K) run_part<MESH_Q4_K, NB, 2>(p, sp, rows_here, nsb, KS, RS, S, K, first, r, first, stage);
            else run_part<MESH_Q6_K, NB, 2>(p, sp, rows_here, nsb, KS, RS, S, K, first, r, first, stage);
        } else {
            if (p.type == MESH_Q4_K) run_part<MESH_Q4_K, NB, 1>(p, sp, rows_here, nsb, KS, RS, S, K, first, r, first, stage);
            else run_part<MESH_Q6_K, NB, 1>(p, sp, rows_here, nsb, KS, RS, S, K, first, r, first, stage);
        }
        first = false;
    }
    MEGA_SUBMARK(5);
    __syncthreads();
    MEGA_SUBMARK(6);
    for (int o = tid; o < rows_here * 16 * NB; o += MEGA_THREADS) {
        const int t = o % NB, r = (o / NB) % 16, j = o / (NB * 16);
        const int gr = g0 + j;
        int pi = 0;
        while (pi + 1 < ph.n_part && gr >= ph.part[pi + 1].begin) ++pi;
        const MegaPart &p = ph.part[pi];
        const int row = (gr - p.begin) * TILE_ROWS + r;
        if (row >= p.M) continue;
        float s0 = 0.f, s1 = 0.f;
        for (int k2 = 0; k2 < KS; ++k2) {
            s0 += S.red[(((k2 * rows_here + j) * 2 + 0) * 16 + r) * NB + t];
            if (p.W1) s1 += S.red[(((k2 * rows_here + j) * 2 + 1) * 16 + r) * NB + t];
        }
        if (norm_w) {
            float q = 0.f;
#pragma unroll
            for (int w = 0; w < MEGA_WAVES; ++w) q += S.ssq[w * NB + t];
            const float scale = 1.0f / sqrtf(q / (float)K + eps);
            s0 *= scale;
            s1 *= scale;
        }
        if (p.bias) s0 += ldg<float>(p.bias + row);
        float out;
        float *yp = p.y + (size_t)t * p.ldy + row;
        if (p.W1) out = (s0 / (1.0f + expf(-s0))) * s1;
        else if (ph.epi == EPI_RESIDUAL) out = xld(yp + (size_t)my_replica() * p.y_rep_stride) + s0;
        else out = s0;
        for (int rep = 0; rep < p.n_rep; ++rep) xst(yp + (size_t)rep * p.y_rep_stride, out);
    }
}

// ------------------------------------------------------------------------------------------------ attention phase
__device__ __forceinline__ void unpack8(const uint4 &v, float (&o)[8]) {
    o[0] = f16_bits_to_f32((uint16_t)(v.x & 0xFFFF)); o[1] = f16_bits_to_f32((uint16_t)(v.x >> 16));
    o[2] = f16_bits_to_f32((uint16_t)(v.y & 0xFFFF)); o[3] = f16_bits_to_f32((uint16_t)(v.y >> 16));
    o[4] = f16_bits_to_f32((uint16_t)(v.z & 0xFFFF)); o[5] = f16_bits_to_f32((uint16_t)(v.z >> 16));
    o[6] = f16_bits_to_f32((uint16_t)(v.w & 0xFFFF)); o[7] = f16_bits_to_f32((uint16_t)(v.w >> 16));
}

// One element of a head vector after RoPE: `vec` is the raw projection output (f32, exchange buffer), dd the
// element, cs/sn the token's table of cos and sin of pos * inv_freq[i].  NORM mode rotates neighbouring pairs, NEOX
// mode pairs dd with dd + n_rot/2; elements at or beyond n_rot pass through.
__device__ __forceinline__ float rope_element(const float *vec, int dd, const float *cs, const float *sn, int n_rot, int mode) {
    float r = xld(vec + dd);
    if (dd < n_rot) {
        const int half = n_rot >> 1;
        int i, partner;
        bool first;
        if (mode == 2) { first = dd < half; i = first ? dd : dd - half; partner = first ? dd + half : dd - half; }
        else { first = (dd & 1) == 0; i = dd >> 1; partner = dd ^ 1; }
        const float other = xld(vec + partner);
        r = first ? r * cs[i] - other * sn[i] : other * sn[i] + r * cs[i];
    }
    return r;
}

// Which (token, KV head, head group, split) an attention work item is, and its key range.
struct AttnItem {
    int t, kvh, h0, split, hsub;
    int pos, j0, jc;            // keys [j0, jc) come from the cache
    bool owns_pos;              // this split covers the token's own position (exactly one does)
    size_t base;                // row index of key 0 of the sequence / KV head in the cache
};
template <int G>
__device__ __forceinline__ AttnItem attn_item(const MegaArgs &a, int item) {
    AttnItem it;
    const int hgroups = a.group / G;
    it.split = item % a.n_splits;
    const int hg = (item / a.n_splits) % (a.n_kv * hgroups);
    it.t = item / (a.n_splits * a.n_kv * hgroups);
    it.kvh = hg / hgroups;
    it.hsub = hg % hgroups;
    it.h0 = it.kvh * a.group + it.hsub * G;
    it.pos = a.pos[it.t];
    const int n_keys = it.pos + 1;
    const int per = (n_keys + a.n_splits - 1) / a.n_splits;
    it.j0 = it.split * per;
    const int j1 = it.j0 + per < n_keys ? it.j0 + per : n_keys;
    it.owns_pos = it.pos >= it.j0 && it.pos < j1;
    it.jc = it.owns_pos ? it.pos : j1;
    it.base = ((size_t)a.seq[it.t] * a.n_kv + it.kvh) * a.n_ctx;
    return it;
}

// KPT keys and values per thread and pass: slot s takes keys jb + s, jb + SLOTS + s, ...
__device__ __forceinline__ void load_kv_pass(const MegaLayer &L, const AttnItem &it, int jb, uint4 (&kr)[KPT], uint4 (&vr)[KPT]) {
    const int slot = threadIdx.x / LPK, ds = (threadIdx.x % LPK) * 8;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        const int j = jb + slot + SLOTS * i;
        const int jr = j < it.jc ? j : it.j0;
        kr[i] = ldg<uint4>(L.kc + (it.base + jr) * HD + ds);
        vr[i] = ldg<uint4>(L.vc + (it.base + jr) * HD + ds);
    }
}

// First pass of the first item of this workgroup, issued before the barrier that precedes the attention phase.
template <int G>
__device__ __forceinline__ void prefetch_kv(const MegaArgs &a, const MegaLayer &L, RawTile (&r)[DEPTH]) {
    static_assert(KPT == 4 && DEPTH >= 2, "the first pass travels in two raw tiles");
    const int n_items = a.B * a.n_kv * (a.group / G) * a.n_splits;
    if ((int)blockIdx.x >= n_items) return;
    const AttnItem it = attn_item<G>(a, blockIdx.x);
    if (it.j0 >= it.jc) return;
    uint4 kr[KPT], vr[KPT];
    load_kv_pass(L, it, it.j0, kr, vr);
    r[0].a = kr[0]; r[0].b = kr[1]; r[0].c = kr[2]; r[0].d = kr[3];
    r[1].a = vr[0]; r[1].b = vr[1]; r[1].c = vr[2]; r[1].d = vr[3];
}

template <int G>
__device__ __forceinline__ void attn_phase(const MegaArgs &a, const MegaLayer &L, const GridSync &g, const RawTile (&r)[DEPTH]) {
    extern __shared__ __align__(16) uint8_t smem[];
    float *s_m = reinterpret_cast<float *>(smem);                 // [MEGA_WAVES][G]
    float *s_l = s_m + MEGA_WAVES * G;                            // [MEGA_WAVES][G]
    float *s_mw = s_l + MEGA_WAVES * G;                           // [G]
    float *s_acc = s_mw + G;                                      // [MEGA_WAVES][G][HD]
    float *s_q = s_acc + MEGA_WAVES * G * HD;                     // [G][HD] roped, scaled queries; then [HD] roped key, [HD] value
    float *s_k = s_q + G * HD;
    float *s_v = s_k + HD;
    const int tid = threadIdx.x, slot = tid / LPK, ds = (tid % LPK) * 8, wave = tid >> 6;
    const int n_items = a.B * a.n_kv * (a.group / G) * a.n_splits;
    if (g.dead) return;
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const AttnItem it = attn_item<G>(a, item);
        const int t = it.t, pos = it.pos, jc = it.jc, j0 = it.j0;
        // first pass of cached keys and values: prefetched for the first item, else loaded here, in flight while
        // the queries are staged
        uint4 kr[KPT], vr[KPT];
        if (item == (int)blockIdx.x) {
            kr[0] = r[0].a; kr[1] = r[0].b; kr[2] = r[0].c; kr[3] = r[0].d;
            vr[0] = r[1].a; vr[1] = r[1].b; vr[2] = r[1].c; vr[3] = r[1].d;
        } else if (j0 < jc) {
            load_kv_pass(L, it, j0, kr, vr);
        }

        // each element of the G query heads, the key and the value is fetched (and rotated) once per workgroup
        for (int el = tid; el < (G + 2) * HD; el += MEGA_THREADS) {
            const int v = el / HD, dd = el % HD;
            const float *cs = a.rope_cs + t * (HD / 2), *sn = a.rope_sn + t * (HD / 2);
            if (v < G) s_q[el] = rope_element(a.q + ((size_t)t * a.n_head + it.h0 + v) * HD, dd, cs, sn, a.n_rot, a.rope_mode) *
                                  (a.attn_scale * 1.44269504088896341f);
            else if (v == G) s_k[dd] = rope_element(a.k + ((size_t)t * a.n_kv + it.kvh) * HD, dd, cs, sn, a.n_rot, a.rope_mode);
            else s_v[dd] = xld(a.v + ((size_t)t * a.n_kv + it.kvh) * HD + dd);
        }
        __syncthreads();

        float q[G][8], acc[G][8], m[G], l[G];
#pragma unroll
        for (int h = 0; h < G; ++h) {
            const float4 qa = *reinterpret_cast<const float4 *>(s_q + h * HD + ds), qb = *reinterpret_cast<const float4 *>(s_q + h * HD + ds + 4);
            q[h][0] = qa.x; q[h][1] = qa.y; q[h][2] = qa.z; q[h][3] = qa.w;
            q[h][4] = qb.x; q[h][5] = qb.y; q[h][6] = qb.z; q[h][7] = qb.w;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[h][e] = 0.f;
            m[h] = -INFINITY;
            l[h] = 0.f;
        }
        MEGA_SUBMARK(3);
        for (int jb = j0; jb < jc; jb += SLOTS * KPT) {
            // one key at a time (few live registers); the last key's loads are replaced by the next pass's
#pragma unroll
            for (int i = 0; i < KPT; ++i) {
                const bool ok = jb + slot + SLOTS * i < jc;
                float kf[8], vf[8], sc[G];
                unpack8(kr[i], kf);
                unpack8(vr[i], vf);
                if (i == KPT - 1 && jb + SLOTS * KPT < jc) load_kv_pass(L, it, jb + SLOTS * KPT, kr, vr);
#pragma unroll
                for (int h = 0; h < G; ++h) {
                    float s = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) s = fmaf(q[h][e], kf[e], s);
#pragma unroll
                    for (int o = LPK / 2; o > 0; o >>= 1) s += __shfl_xor(s, o);
                    sc[h] = s;
                }
                if (ok) {
#pragma unroll
                    for (int h = 0; h < G; ++h) {
                        const float mn = fmaxf(m[h], sc[h]);
                        const float corr = exp2f(m[h] - mn), p0 = exp2f(sc[h] - mn);
                        l[h] = l[h] * corr + p0;
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(p0, vf[e], acc[h][e] * corr);
                        m[h] = mn;
                    }
                }
            }
        }
        MEGA_SUBMARK(4);
        // The token's own key and value come from the projection outputs, rounded to f16 exactly as the cache holds
        // them; the covering split appends them to the cache and slot 0 accounts for them.
        if (it.owns_pos) {
            uint32_t kpk[4], vpk[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                kpk[e] = (uint32_t)f32_to_f16_bits(s_k[ds + 2 * e]) | ((uint32_t)f32_to_f16_bits(s_k[ds + 2 * e + 1]) << 16);
                vpk[e] = (uint32_t)f32_to_f16_bits(s_v[ds + 2 * e]) | ((uint32_t)f32_to_f16_bits(s_v[ds + 2 * e + 1]) << 16);
            }
            const uint4 k16 = make_uint4(kpk[0], kpk[1], kpk[2], kpk[3]), v16 = make_uint4(vpk[0], vpk[1], vpk[2], vpk[3]);
            if (slot == 0 && it.hsub == 0) {
                *as_global<uint4>(L.kc + (it.base + pos) * HD + ds) = k16;
                *as_global<uint4>(L.vc + (it.base + pos) * HD + ds) = v16;
            }
            float kf[8], vf[8];
            unpack8(k16, kf);
            unpack8(v16, vf);
#pragma unroll
            for (int h = 0; h < G; ++h) {
                float s = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) s = fmaf(q[h][e], kf[e], s);
#pragma unroll
                for (int o = LPK / 2; o > 0; o >>= 1) s += __shfl_xor(s, o);
                if (slot == 0) {
                    const float mn = fmaxf(m[h], s);
                    const float corr = exp2f(m[h] - mn), p0 = exp2f(s - mn);
                    l[h] = l[h] * corr + p0;
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(p0, vf[e], acc[h][e] * corr);
                    m[h] = mn;
                }
            }
        }
        MEGA_SUBMARK(5);
        // merge the 64 slots: running maxima first (over the 4 slots of a wave by shuffle, over the waves in LDS)
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float mw = m[h];
#pragma unroll
            for (int o = LPK; o < 64; o <<= 1) mw = fmaxf(mw, __shfl_xor(mw, o));
            if ((tid & 63) == 0) s_m[wave * G + h] = mw;
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float mh = -INFINITY;
#pragma unroll
            for (int w2 = 0; w2 < MEGA_WAVES; ++w2) mh = fmaxf(mh, s_m[w2 * G + h]);
            const float w = (m[h] == -INFINITY) ? 0.f : exp2f(m[h] - mh);
            float lw = l[h] * w;
#pragma unroll
            for (int o = LPK; o < 64; o <<= 1) lw += __shfl_xor(lw, o);
            if ((tid & 63) == 0) { s_l[wave * G + h] = lw; s_mw[h] = mh; }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float v = acc[h][e] * w;
#pragma unroll
                for (int o = LPK; o < 64; o <<= 1) v += __shfl_xor(v, o);
                if ((tid & 63) < LPK) s_acc[(wave * G + h) * HD + ds + e] = v;
            }
        }
        __syncthreads();
        for (int o = tid; o < G * HD; o += MEGA_THREADS) {
            const int h = o / HD, dd = o % HD;
            float sum = 0.f, ll = 0.f;
#pragma unroll
            for (int w2 = 0; w2 < MEGA_WAVES; ++w2) { sum += s_acc[(w2 * G + h) * HD + dd]; ll += s_l[w2 * G + h]; }
            const size_t row = (size_t)t * a.n_head + it.h0 + h;
            xst(a.part + (row * a.n_splits + it.split) * HD + dd, sum);
            if (dd == 0) {
                xst(a.ml + (row * a.n_splits + it.split) * 2 + 0, s_mw[h]);
                xst(a.ml + (row * a.n_splits + it.split) * 2 + 1, ll);
            }
        }
        MEGA_SUBMARK(6);
        __syncthreads();        // LDS is reused by the next item
    }
}

// merge of the KV splits: (token, head, dim) outputs spread over the grid; the n_splits (power of two <= 32)
// partials of one output sit in neighbouring lanes and are combined with shuffles
__device__ __forceinline__ void combine_phase(const MegaArgs &a, const GridSync &g) {
    if (g.dead) return;
    const int ns = a.n_splits;
    const int per_wg = MEGA_THREADS / ns;
    const int n_out = a.B * a.n_head * HD;
    for (int o0 = blockIdx.x * per_wg; o0 < n_out; o0 += gridDim.x * per_wg) {
        const int o = o0 + threadIdx.x / ns, s2 = threadIdx.x % ns;
        const bool live = o < n_out;
        const int row = live ? o / HD : 0, dd = o % HD;
        float ms = -INFINITY, ls = 0.f, pv = 0.f;
        if (live) {
            ms = xld(a.ml + ((size_t)row * ns + s2) * 2 + 0);
            ls = xld(a.ml + ((size_t)row * ns + s2) * 2 + 1);
            pv = xld(a.part + ((size_t)row * ns + s2) * HD + dd);
        }
        float mh = ms;
        for (int w = 1; w < ns; w <<= 1) mh = fmaxf(mh, __shfl_xor(mh, w));
        const float wgt = ms == -INFINITY ? 0.f : exp2f(ms - mh);
        float num = pv * wgt, den = ls * wgt;
        for (int w = 1; w < ns; w <<= 1) { num += __shfl_xor(num, w); den += __shfl_xor(den, w); }
        if (live && s2 == 0) {
            const float out = num / den;
            for (int rep = 0; rep < MEGA_REPLICAS; ++rep) xst(a.attn + (size_t)rep * a.attn_rep_stride + (size_t)row * HD + dd, out);
        }
    }
}

// ------------------------------------------------------------------------------------------------ the kernel
template <int NB, int G>
__global__ __launch_bounds__(MEGA_THREADS) void decode_mega_kernel(const MegaArgs a) {
    GridSync g;
    g.counter = a.bar;
    g.abort_flag = a.abort_flag;
    g.n_wg = gridDim.x;
    g.target = a.bar_base + gridDim.x;
    g.spin_limit = a.spin_limit;
    g.dead = false;
    g.phase = 0;

    // six phases per layer, each closed by a grid barrier; one loop body so that the GEMV code exists once.
    // r[] carries what was prefetched for the coming phase across the barrier.
    RawTile r[DEPTH] = {};
    prefetch_tiles(a.layers[0].ph[0], r);
    const int n_phase = 6 * a.n_layers;
    for (int ip = 0; ip < n_phase; ++ip) {
        const int il = ip / 6, kind = ip - 6 * il;
        const MegaLayer &L = a.layers[il];
        g.phase = ip;
        MEGA_MARK(ip, 0);
        if (kind == 1) attn_phase<G>(a, L, g, r);                              // rope, KV append, split-KV partials
        else if (kind == 2) combine_phase(a, g);                                // merge of the splits (o tiles stay held)
        else gemv_phase<NB>(L.ph[kind == 0 ? 0 : kind - 2], a.eps, g, r);  // q/k/v | o | gate,up | down
        MEGA_MARK(ip, 1);
        grid_barrier(g, [&]() {
            if (kind != 2) {                                                    // nothing older is needed: keeps them out of the phases' live ranges
#pragma unroll
                for (int d = 0; d < DEPTH; ++d) r[d] = RawTile{};
            }
            if (g.dead) return;
            if (kind == 0) prefetch_kv<G>(a, L, r);                            // cached keys and values of the first pass
            else if (kind == 1) prefetch_tiles(L.ph[1], r);                // o, held across the merge phase
            else if (kind == 3) prefetch_tiles(L.ph[2], r);                // gate/up
            else if (kind == 4) prefetch_tiles(L.ph[3], r);                // down
            else if (kind == 5 && il + 1 < a.n_layers) prefetch_tiles(a.layers[il + 1].ph[0], r);
        });
        MEGA_MARK(ip, 2);
    }
}

// Before the persistent kernel: the input hidden state (replica 0) is copied to the other replicas, and the
// cos/sin tables of the batch's positions are computed once for all layers.
__global__ void mega_prologue_kernel(float *x, size_t rep_stride, int n, const int32_t *pos, const float *inv_freq, int half_rot, int B,
                                     float *rope_cs, float *rope_sn) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float v = x[i];
        for (int rep = 1; rep < MEGA_REPLICAS; ++rep) x[(size_t)rep * rep_stride + i] = v;
    }
    if (i < B * (HD / 2)) {
        const int t = i / (HD / 2), k = i % (HD / 2);
        float sn = 0.f, cs = 1.f;
        if (k < half_rot) sincosf((float)pos[t] * inv_freq[k], &sn, &cs);
        rope_cs[i] = cs;
        rope_sn[i] = sn;
    }
}

static int attn_g_of(int group) { return group % 4 == 0 ? 4 : group % 5 == 0 ? 5 : group % 2 == 0 ? 2 : 1; }

size_t mega_smem_bytes(const MegaLayer &layer, int nb, int group, int grid) {
    const int G = attn_g_of(group);
    size_t need = sizeof(float) * ((size_t)MEGA_WAVES * G + (size_t)MEGA_WAVES * G + G + (size_t)MEGA_WAVES * G * HD + (size_t)(G + 2) * HD);
    for (const MegaPhase &ph : layer.ph) {
        const int nsb = ph.K / QK_K, KS = nsb < MEGA_WAVES ? nsb : MEGA_WAVES;
        const int rows = (ph.total_rows + grid - 1) / grid;
        const size_t b = (size_t)nb * (2 * (size_t)ph.K + (size_t)(ph.K / 32) * 8 + (size_t)(ph.K / 16) * 4) +
                         sizeof(float) * ((size_t)MEGA_WAVES * nb + (size_t)KS * rows * 2 * 16 * nb);
        need = b > need ? b : need;
    }
    return need;
}

int mega_barriers_per_launch(int n_layers) { return 6 * n_layers; }

template <int NB, int G>
static int launch_mega(const MegaArgs &a, int grid, size_t smem, hipStream_t stream) {
    static size_t attr_bytes = 0;
    if (smem > attr_bytes) {
        MESH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(decode_mega_kernel<NB, G>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_bytes = smem;
    }
    MegaArgs args = a;
    void *params[] = {&args};
    MESH_HIP_TRY(hipLaunchCooperativeKernel(reinterpret_cast<const void *>(decode_mega_kernel<NB, G>), dim3((unsigned)grid),
                                            dim3(MEGA_THREADS), params, (unsigned)smem, stream));
    return MESH_OK;
}

int decode_mega(const MegaArgs &a, int grid, size_t smem, hipStream_t stream) {
    if (a.B > MEGA_BATCH_MAX || a.B < 1) return fail(MESH_ERR_INVALID, "decode_mega: batch %d outside 1..%d", a.B, MEGA_BATCH_MAX);
    if (a.n_splits < 1 || a.n_splits > MEGA_SPLITS_MAX || (a.n_splits & (a.n_splits - 1)))
        return fail(MESH_ERR_INVALID, "decode_mega: %d KV splits (need a power of two up to %d)", a.n_splits, MEGA_SPLITS_MAX);
    if (a.n_rot > HD || a.n_rot < 0) return fail(MESH_ERR_INVALID, "decode_mega: n_rot %d outside the head", a.n_rot);
    {
        const int n = a.B * a.E, nt = n > a.B * (HD / 2) ? n : a.B * (HD / 2);
        mega_prologue_kernel<<<dim3((unsigned)((nt + 255) / 256)), dim3(256), 0, stream>>>(a.x, a.x_rep_stride, n, a.pos, a.inv_freq,
                                                                                             a.n_rot / 2, a.B, a.rope_cs, a.rope_sn);
        MESH_LAUNCH_CHECK();
    }
    const int NB = a.B <= 1 ? 1 : a.B <= 2 ? 2 : 4, G = attn_g_of(a.group);
#define MESH_MEGA_CASE(NBB, GG)                                                    \
    if (NB == NBB && G == GG) return launch_mega<NBB, GG>(a, grid, smem, stream);
    MESH_MEGA_CASE(1, 1) MESH_MEGA_CASE(2, 1) MESH_MEGA_CASE(4, 1)
    MESH_MEGA_CASE(1, 2) MESH_MEGA_CASE(2, 2) MESH_MEGA_CASE(4, 2)
    MESH_MEGA_CASE(1, 4) MESH_MEGA_CASE(2, 4) MESH_MEGA_CASE(4, 4)
    MESH_MEGA_CASE(1, 5) MESH_MEGA_CASE(2, 5) MESH_MEGA_CASE(4, 5)
#undef MESH_MEGA_CASE
    return fail(MESH_ERR_UNSUPPORTED, "decode_mega: no instantiation for group %d", a.group);
}

bool mega_group_supported(int group) { return group >= 1; }

}  // namespace mesh

#ifdef MESH_MEGA_TRACE
extern "C" int mesh_debug_set_mega_trace(void *p) {
    return hipMemcpyToSymbol(HIP_SYMBOL(mesh::g_mega_trace), &p, sizeof p) == hipSuccess ? 0 : -1;
}
#endif
