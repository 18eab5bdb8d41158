// One-token decode step as ONE launch, sharded over the eight compute dies (XCDs) of the GPU.
//
// The per-layer graph is the one stage.hip runs projection by projection (rpc_server::graph_compute,
// third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451).  Run as ~96 dependent launches a
// step pays each kernel's own start-up and drain (~4.5 us) on top of the time its bytes take to stream.  What makes one
// launch cheaper than six per layer on this part is WHERE the hand-overs happen: a barrier among the 32 workgroups of one
// die, through counters and data that live in that die's L2, costs ~1 us plus ~0.5 us to read 16 KB back; a barrier
// over all 256 workgroups built from those (the last arriver of each die joins an 8-way counter in memory, then
// releases its die) costs ~2 us.  So the work is cut along the dies the way a tensor-parallel layer is cut along GPUs:
//
//   die g (= kv head g, the GPU has 8 dies and the model 8 kv heads)
//     A  q heads 4g..4g+3, k head g, v head g  = rows of Wq / Wk / Wv          -> die barrier
//        rope; the new k / v row goes to the cache
//     B  attention of those 4 heads over kv head g, 32 key ranges              -> die barrier
//        merge of the ranges
//     C  Wo restricted to the columns of heads 4g..4g+3: partial sums of ALL rows -> chip barrier
//        every die adds the 8 partial vectors + residual for itself (32 x 128 rows)   -> die barrier
//     D  rows [1792g, 1792g+1792) of W_gate / W_up                             -> die barrier
//        SwiGLU
//     E  W_down restricted to those 1792 columns: partial sums of all rows      -> chip barrier
//        8 partial vectors + residual                                           -> die barrier
//
// i.e. five die-local and two chip-wide hand-overs per layer.  Weights do not depend on activations, so before a wave
// arrives at a barrier it has already requested its first four weight tiles (or its share of the KV rows) of the NEXT
// phase: HBM keeps streaming while the barrier runs.
//
// Data that crosses workgroups is written with ordinary stores (die-local buffers: the die's L2 is the meeting point) or
// device-scope stores (the two partial-sum buffers all dies read), and always read with device-scope loads, which miss the
// compute unit's vector cache by construction; a wave drains its stores (vmcnt 0) before it arrives.  Every reduction
// has a fixed order, so results do not depend on timing.
//
// Geometry is fixed: 256 workgroups of 512 threads, 32 on each die (the hardware deals a launch's workgroups to the dies in
// turn; a workgroup reads which die it is on and takes a rank there by ticket; a probe launch when the session is created
// and every step check the count).  All waits are bounded:
// a wait that gives up raises a flag that every other wait polls, all workgroups leave, and the host reports an error.
//
// Shape: the Llama-3-8B / Mistral-7B family (hidden 4096, FFN 14336, 32 heads of 128 over 8 kv heads, neighbouring-pair
// RoPE over the whole head, no biases), q4_K / q6_K matrices in the tiled layout, f16 KV cache.  Anything else keeps
// the launch-per-projection path.

#include "decode_die.hpp"

#include "gemv_device.hpp"
#include "kv_cache.hpp"

#include <cstdlib>
#include <mutex>

namespace mesh {

namespace {

constexpr int DD_THREADS = 512, DD_WAVES = DD_THREADS / 64;
constexpr int DEPTH = 4;                          // weight tiles a wave keeps in flight
constexpr int N_DIE = 8, WG_PER_DIE = 32, DD_GRID = N_DIE * WG_PER_DIE;
constexpr int E = 4096, FF = 14336, HD = 128, NKV = 8, G = 4, NH = NKV * G;
constexpr int E_SB = E / QK_K;                    // super-blocks per row of a matrix with 4096 columns
constexpr int QKV_ROWS = (G + 2) * HD;            // q, k, v rows of one die
constexpr int A_K = G * HD;                       // a die's slice of the attention output = its columns of Wo
constexpr int FF_DIE = FF / N_DIE, FF_NSB = FF / QK_K, FF_SB = FF_DIE / QK_K;
constexpr int ROWS_WG = E / WG_PER_DIE;           // rows of the hidden state a workgroup reduces
// weight tiles per wave and phase (a workgroup's tiles, dealt to its 8 waves in runs)
constexpr int CNT_A = 3, CNT_C = 2, CNT_D = 14, CNT_E = 7;
static_assert(QKV_ROWS / 16 * 2 == WG_PER_DIE * 3 && 3 * 8 == DD_WAVES * CNT_A, "phase A: 96 half-rows of tiles over 32 workgroups");
static_assert(E / 16 == WG_PER_DIE * 8 && 8 * (A_K / QK_K) == DD_WAVES * CNT_C, "phase C");
static_assert(FF_DIE / 16 * 2 == WG_PER_DIE * 7 && 7 * 2 * 8 == DD_WAVES * CNT_D, "phase D");
static_assert(8 * FF_SB == DD_WAVES * CNT_E, "phase E");

constexpr int ATT_LPK = HD / 8, ATT_SLOTS = DD_THREADS / ATT_LPK, ATT_KPT = 4;

// counters, 256 bytes apart: [0..8) die barriers, [8..16) chip barrier arrivals per die, [16..24) chip barrier releases per
// die, [24] chip counter, [25] give-up flag, [26..34) rank tickets per die
constexpr int SYNC_STRIDE = 64, SYNC_WORDS = 34 * SYNC_STRIDE;
constexpr int SYNC_CHIP = 24 * SYNC_STRIDE, SYNC_ABORT = 25 * SYNC_STRIDE, SYNC_TICKET = 26 * SYNC_STRIDE;

struct DieLayer {
    const uint8_t *wq, *wk, *wv, *wo, *wg, *wu, *wd;
    const float *attn_norm, *ffn_norm;
    uint8_t *kcache, *vcache;
    unsigned q6;            // bit i: matrix i (order above) is q6_K, else q4_K
};

struct DieArgs {
    const DieLayer *layers;
    int n_layer;
    float *x;                       // [E] in and out
    const int32_t *pos, *seq;
    const float *inv_freq;
    float eps, attn_scale;
    int n_ctx;
    float *qkv_part;                // [die][2 halves of K][768]
    float *att_part;                // [die][32 ranges][G][HD]
    float *att_ml;                  // [die][32 ranges][G][2]
    float *h_loc;                   // [die][E]: every die's own copy of the hidden state
    float *gu_part;                 // [die][gate, up][2 halves of K][1792]
    float *p1, *p2;                 // [die][E] partial sums of the output / down projection
    unsigned *sync;
    unsigned *host_flag;            // pinned host word, set when a wait gives up
    unsigned base_die, base_chip;   // barriers completed before this launch
    unsigned base_ticket;           // rank tickets handed out per die before this launch
    unsigned spin_limit;
};

// ------------------------------------------------------------------------------------------------ small device helpers
__device__ __forceinline__ unsigned xcc_id() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 15u;
}
// a zero the compiler cannot see through: predicates built on it stay per-lane (execution masks) instead of becoming
// branches, so the number of loads in flight is the same on every path
__device__ __forceinline__ int opaque_zero() {
    int z;
    asm volatile("v_mov_b32 %0, 0" : "=v"(z));
    return z;
}
// atomic add that returns the old value; the wait is part of the statement because the result register is written when
// the reply arrives.  SC1: performed in memory (all dies see one counter); otherwise in the issuing die's L2.
template <bool SC1>
__device__ __forceinline__ unsigned atom_add_ret(unsigned *p, unsigned v) {
    unsigned r;
    if constexpr (SC1) asm volatile("global_atomic_add %0, %1, %2, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(r) : "v"(p), "v"(v) : "memory");
    else asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(r) : "v"(p), "v"(v) : "memory");
    return r;
}
// exchange memory: device-scope accesses
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
// Workgroup barrier that orders LDS only: it does not wait for outstanding global loads, so prefetches stay in flight.
__device__ __forceinline__ void wg_barrier_lds() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
__device__ __forceinline__ void drain_stores() { __builtin_amdgcn_s_waitcnt(0); }

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
template <int LPK>
__device__ __forceinline__ float slot_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, false));
    if (LPK == 16) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, false));
    return v;
}

// ------------------------------------------------------------------------------------------------ barriers
struct Sync {
    unsigned *base;
    unsigned *host_flag;
    unsigned n_die, n_chip, spin_limit;
    int die;
};

// thread 0 only.  false: gave up (limit reached, or another workgroup gave up)
template <bool SC1>
__device__ __forceinline__ bool poll_until(const Sync &sy, unsigned *ctr, unsigned want) {
    unsigned spins = 0;
    for (;;) {
        const unsigned seen = atom_add_ret<SC1>(ctr, 0u);
        if ((int)(seen - want) >= 0) return true;
        if (++spins > sy.spin_limit) break;
        if ((spins & 127u) == 0 && atom_add_ret<true>(sy.base + SYNC_ABORT, 0u)) break;
        __builtin_amdgcn_s_sleep(1);
    }
    atom_add_ret<true>(sy.base + SYNC_ABORT, 1u);
    __hip_atomic_store(sy.host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    return false;
}

// The callers have drained their stores and issued their prefetches.  Returns false when the step is being abandoned.
__device__ __forceinline__ bool die_barrier(Sync &sy, int *s_flag) {
    wg_barrier_lds();
    ++sy.n_die;
    if (threadIdx.x == 0) {
        unsigned *c = sy.base + sy.die * SYNC_STRIDE;
        atom_add_ret<false>(c, 1u);
        *s_flag = poll_until<false>(sy, c, sy.n_die * (unsigned)WG_PER_DIE) ? 1 : 0;
    }
    wg_barrier_lds();
    return *s_flag != 0;
}

__device__ __forceinline__ bool chip_barrier(Sync &sy, int *s_flag) {
    wg_barrier_lds();
    ++sy.n_chip;
    if (threadIdx.x == 0) {
        unsigned *arr = sy.base + (8 + sy.die) * SYNC_STRIDE, *rel = sy.base + (16 + sy.die) * SYNC_STRIDE;
        const unsigned mine = atom_add_ret<false>(arr, 1u) + 1u;
        bool ok;
        if (mine == sy.n_chip * (unsigned)WG_PER_DIE) {
            // last of this die: join the other dies, then let the die go
            atom_add_ret<true>(sy.base + SYNC_CHIP, 1u);
            ok = poll_until<true>(sy, sy.base + SYNC_CHIP, sy.n_chip * (unsigned)N_DIE);
            if (ok) atom_add_ret<false>(rel, 1u);
        } else {
            ok = poll_until<false>(sy, rel, sy.n_chip);
        }
        *s_flag = ok ? 1 : 0;
    }
    wg_barrier_lds();
    return *s_flag != 0;
}

// ------------------------------------------------------------------------------------------------ weight tiles
// A tile of either K-quant type as raw registers.  Five loads whatever the type: those a q4_K tile does not have are
// masked off per lane, not branched around.
struct RawTile {
    uint4 a, b, c, d;
    uint32_t e;
};
struct TileDesc {
    const uint8_t *p;
    bool q6;
    int sb;          // super-block index into the staged activations
};

// ALWAYS: the tile exists on every path (a prefetch); otherwise `live` is a per-lane predicate.  Registers a load may skip
// are cleared first, so that no earlier tile stays alive through a skipped load.
template <bool ALWAYS>
__device__ __forceinline__ void load_raw(RawTile &r, const TileDesc &t, int lane, bool live, int vz) {
    const int row = lane >> 2, c = lane & 3, n = c >> 1, u = c & 1;
    const uint8_t *pa = t.q6 ? t.p + row * 128 + 64 * n + 16 * u : t.p + row * 16;
    const uint8_t *pb = t.q6 ? t.p + row * 128 + 64 * n + 32 + 16 * u : t.p + 256 + lane * 32;
    const uint8_t *pc = t.q6 ? t.p + 2048 + row * 64 + 32 * n + 16 * u : t.p + 256 + lane * 32 + 16;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    if constexpr (ALWAYS) {
        r.a = ldg<uint4>(pa);
        r.b = ldg<uint4>(pb);
        r.c = ldg<uint4>(pc);
    } else {
        r.a = zero; r.b = zero; r.c = zero;
        if (live) {
            r.a = ldg<uint4>(pa);
            r.b = ldg<uint4>(pb);
            r.c = ldg<uint4>(pc);
        }
    }
    r.d = zero;
    r.e = 0u;
    if ((ALWAYS || live) && ((int)t.q6 + vz) != 0) {
        r.d = ldg<uint4>(t.p + 3072 + row * 16);
        r.e = ldg<uint16_t>(t.p + 3328 + row * 2);
    }
}

// the tile's 16 rows times the staged activations: lanes 4r hold row r's sum over the tile's super-block
__device__ __forceinline__ float tile_dot(const RawTile &r, const TileDesc &t, int lane, const XStage &S, int K) {
    float acc[1] = {0.f};
    if (t.q6) {
        TileRegs<MESH_Q6_K> q;
        q.qla = r.a; q.qlb = r.b; q.qh = r.c; q.sc = r.d; q.d = r.e;
        tile_compute<1>(q, lane, t.sb, S, K, acc);
    } else {
        TileRegs<MESH_Q4_K> q;
        q.hdr = r.a; q.qa = r.b; q.qb = r.c;
        tile_compute<1>(q, lane, t.sb, S, K, acc);
    }
    float v = acc[0];
    v += __shfl_xor(v, 1);
    v += __shfl_xor(v, 2);
    return v;
}

template <int CNT, typename Desc>
__device__ __forceinline__ void prefetch_tiles(RawTile (&r)[DEPTH], const Desc &desc, int wave, int lane, int vz) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (d < CNT) load_raw<true>(r[d], desc(wave * CNT + d), lane, true, vz);
}

// Tiles wave * CNT + i, i < CNT: the first DEPTH are in r[] already; tile i's partial row sums go to red[tile][16].
template <int CNT, typename Desc>
__device__ __forceinline__ void run_tiles(RawTile (&r)[DEPTH], const Desc &desc, const XStage &S, int K, float *red, int wave, int lane, int vz) {
    constexpr int FULL = CNT > DEPTH ? CNT / DEPTH : 0, REM = CNT - FULL * DEPTH;
    for (int ig = 0; ig < FULL; ++ig) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int i = ig * DEPTH + d;
            const float v = tile_dot(r[d], desc(wave * CNT + i), lane, S, K);
            if ((lane & 3) == 0) red[(wave * CNT + i) * 16 + (lane >> 2)] = v;
            const int in = i + DEPTH;
            load_raw<false>(r[d], desc(wave * CNT + (in < CNT ? in : CNT - 1)), lane, in + vz < CNT, vz);
        }
    }
#pragma unroll
    for (int d = 0; d < REM; ++d) {
        const int i = FULL * DEPTH + d;
        const float v = tile_dot(r[d], desc(wave * CNT + i), lane, S, K);
        if ((lane & 3) == 0) red[(wave * CNT + i) * 16 + (lane >> 2)] = v;
    }
}

__device__ __forceinline__ size_t tile_bytes(bool q6) { return q6 ? (size_t)Q6K_TILE_BYTES : (size_t)Q4K_TILE_BYTES; }

// ------------------------------------------------------------------------------------------------ LDS
struct __align__(16) Lds {
    int8_t xh[E], xl[E];
    float xd[E / 32], xs[E / 32];
    int xi16[E / 16];
    float ssq[DD_WAVES];
    float red[DD_WAVES * CNT_D * 16];
    float sq[G * HD];                       // this step's query heads after rope
    uint16_t sk16[HD], sv16[HD];            // the new cache rows as they are stored
    float att[A_K];                         // merged attention output of the die's heads
    float ml[WG_PER_DIE * G * 2];
    float s_m[ATT_SLOTS][G], s_l[DD_WAVES][G], s_mw[G];
    float s_acc[DD_WAVES][G][HD];
    int flag;
};

// eight values per thread (threads below K / 8) -> 16-bit fixed point in LDS; returns the thread's sum of squares
__device__ __forceinline__ float stage_x(XRegs<1> &X, int K, const XStage &S, int tid) {
    float ss[1] = {0.f};
    x_quantise<1, true>(X, K, S, tid, tid < K / 8, ss);
    return ss[0];
}
__device__ __forceinline__ void x_zero(XRegs<1> &X) {
    X.a[0] = make_float4(0.f, 0.f, 0.f, 0.f);
    X.b[0] = X.a[0];
    X.w0 = make_float4(1.f, 1.f, 1.f, 1.f);
    X.w1 = X.w0;
}
__device__ __forceinline__ void x_from_exchange(XRegs<1> &X, const float *src, int tid) {
    const float2 v0 = xld2(src + tid * 8), v1 = xld2(src + tid * 8 + 2), v2 = xld2(src + tid * 8 + 4), v3 = xld2(src + tid * 8 + 6);
    X.a[0] = make_float4(v0.x, v0.y, v1.x, v1.y);
    X.b[0] = make_float4(v2.x, v2.y, v3.x, v3.y);
}
// 1 / rms over the workgroup (one barrier; also the barrier between staging and the tiles)
__device__ __forceinline__ float wg_norm_scale(float ss, Lds &L, int K, float eps, int wave, int lane) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    if (lane == 0) L.ssq[wave] = ss;
    wg_barrier_lds();
    float q = 0.f;
#pragma unroll
    for (int w = 0; w < DD_WAVES; ++w) q += L.ssq[w];
    return 1.0f / sqrtf(q / (float)K + eps);
}

// ------------------------------------------------------------------------------------------------ attention pieces
struct KvRows {
    KvRaw<MESH_F16> k[ATT_KPT], v[ATT_KPT];
};
// rows j0 + slot + SLOTS * i of the cache, as far as they were written by earlier steps (j < pos)
__device__ __forceinline__ void kv_fetch_pass(KvRows &R, const uint8_t *kb, const uint8_t *vb, int jb, int j1, int pos, int slot, int ds) {
#pragma unroll
    for (int i = 0; i < ATT_KPT; ++i) {
        const int j = jb + slot + ATT_SLOTS * i;
        kv_zero<MESH_F16>(R.k[i]);
        kv_zero<MESH_F16>(R.v[i]);
        if (j < j1 && j < pos) {
            R.k[i] = kv_load<MESH_F16, HD>(kb + (size_t)j * (HD * 2), ds);
            R.v[i] = kv_load<MESH_F16, HD>(vb + (size_t)j * (HD * 2), ds);
        }
    }
}

// ------------------------------------------------------------------------------------------------ the kernel
__global__ __launch_bounds__(DD_THREADS) void decode_die_kernel(const DieArgs a) {
    __shared__ Lds L;
    const int tid_k = threadIdx.x;
    const int wave_k = __builtin_amdgcn_readfirstlane(tid_k >> 6);
    // The die this workgroup runs on, and its rank among the die's workgroups by ticket: the hardware deals the workgroups
    // of a launch to the dies in turn (any 256 consecutive ones are 32 per die), but where a launch starts depends on
    // the launches before it.
    const int g_k = (int)xcc_id();
    if (tid_k == 0) L.flag = (int)(atom_add_ret<false>(a.sync + SYNC_TICKET + (g_k & (N_DIE - 1)) * SYNC_STRIDE, 1u) - a.base_ticket);
    wg_barrier_lds();
    const int w_k = __builtin_amdgcn_readfirstlane(L.flag);
    wg_barrier_lds();

    Sync sy;
    sy.base = a.sync; sy.host_flag = a.host_flag;
    sy.n_die = a.base_die; sy.n_chip = a.base_chip; sy.spin_limit = a.spin_limit;
    sy.die = g_k;
    if (g_k >= N_DIE || (unsigned)w_k >= (unsigned)WG_PER_DIE) {
        // not 32 workgroups on every die: nothing has been written yet, abandon the step
        if (tid_k == 0) {
            atom_add_ret<true>(sy.base + SYNC_ABORT, 1u);
            __hip_atomic_store(sy.host_flag, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        return;
    }

    XStage S;
    S.xh = L.xh; S.xl = L.xl; S.xd = L.xd; S.xs = L.xs; S.xi16 = L.xi16; S.ssq = L.ssq; S.red = L.red;

    const int pos = __builtin_amdgcn_readfirstlane(a.pos[0]), seq = __builtin_amdgcn_readfirstlane(a.seq[0]);
    const int n_keys = pos + 1;
    const int per = (n_keys + WG_PER_DIE - 1) / WG_PER_DIE;
    RawTile r[DEPTH];
    DieLayer cur = a.layers[0];
    XRegs<1> X;
    x_zero(X);

    for (int il = 0; il < a.n_layer; ++il) {
        const bool first = il == 0, last = il + 1 == a.n_layer;
        // As far as the compiler can tell, every layer computes the same addresses; left alone it computes hundreds of
        // them once, ahead of the loop, and keeps them in scratch memory.  What passes through these empty statements is
        // new in every iteration.
        int tid = tid_k, wave = wave_k, g = g_k, w = w_k;
        asm volatile("" : "+v"(tid));
        asm volatile("" : "+s"(wave), "+s"(g), "+s"(w));
        const int lane = tid & 63;
        const int vz = opaque_zero();
        const int j0 = w * per, j1 = j0 + per < n_keys ? j0 + per : n_keys;
        const int slot = tid / ATT_LPK, ds = (tid % ATT_LPK) * 8;

        auto desc_a = [&](int f) -> TileDesc {
            const int ul = f >> 3, sbi = f & 7, u = 3 * w + ul, tr = u >> 1, sb = (u & 1) * 8 + sbi;
            const uint8_t *base = tr < 32 ? cur.wq : tr < 40 ? cur.wk : cur.wv;
            const bool q6 = ((cur.q6 >> (tr < 32 ? 0 : tr < 40 ? 1 : 2)) & 1u) != 0;
            const int trow = tr < 32 ? 32 * g + tr : tr < 40 ? 8 * g + tr - 32 : 8 * g + tr - 40;
            return TileDesc{base + ((size_t)trow * E_SB + sb) * tile_bytes(q6), q6, sb};
        };
        auto desc_c = [&](int f) -> TileDesc {
            const int j = f >> 1, sbi = f & 1;
            const bool q6 = ((cur.q6 >> 3) & 1u) != 0;
            return TileDesc{cur.wo + ((size_t)(8 * w + j) * E_SB + 2 * g + sbi) * tile_bytes(q6), q6, sbi};
        };
        auto desc_d = [&](int f) -> TileDesc {
            const int ul = f >> 4, mat = (f >> 3) & 1, sbi = f & 7, u = 7 * w + ul, trl = u >> 1, sb = (u & 1) * 8 + sbi;
            const bool q6 = ((cur.q6 >> (4 + mat)) & 1u) != 0;
            return TileDesc{(mat ? cur.wu : cur.wg) + ((size_t)(FF_DIE / 16 * g + trl) * E_SB + sb) * tile_bytes(q6), q6, sb};
        };
        auto desc_e = [&](int f) -> TileDesc {
            const int j = f / FF_SB, sbi = f - j * FF_SB;
            const bool q6 = ((cur.q6 >> 6) & 1u) != 0;
            return TileDesc{cur.wd + ((size_t)(8 * w + j) * FF_NSB + FF_SB * g + sbi) * tile_bytes(q6), q6, sbi};
        };

        if (first) {
            // phase A of the first layer: its tiles and norm weights
            prefetch_tiles<CNT_A>(r, desc_a, wave, lane, vz);
            X.w0 = ldg<float4>(cur.attn_norm + tid * 8);
            X.w1 = ldg<float4>(cur.attn_norm + tid * 8 + 4);
        }
        const float *h_src = first ? a.x : a.h_loc + (size_t)g * E;

        // ---- A: q / k / v rows of this die over the normalised hidden state
        x_from_exchange(X, h_src, tid);
        const float scale_a = wg_norm_scale(stage_x(X, E, S, tid), L, E, a.eps, wave, lane);
        run_tiles<CNT_A>(r, desc_a, S, E, L.red, wave, lane, vz);
        wg_barrier_lds();
        if (tid < 48) {
            const int ul = tid >> 4, rr = tid & 15, u = 3 * w + ul;
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) s += L.red[(ul * 8 + i) * 16 + rr];
            a.qkv_part[((size_t)g * 2 + (u & 1)) * QKV_ROWS + (u >> 1) * 16 + rr] = s;
        }
        drain_stores();
        // keys of this workgroup's range that earlier steps wrote
        const uint8_t *kb = cur.kcache + ((size_t)seq * NKV + g) * (size_t)a.n_ctx * (HD * 2);
        const uint8_t *vb = cur.vcache + ((size_t)seq * NKV + g) * (size_t)a.n_ctx * (HD * 2);
        KvRows R;
        kv_fetch_pass(R, kb, vb, j0, j1, pos, slot, ds);
        if (!die_barrier(sy, &L.flag)) return;

        // ---- rope; the new k / v rows
        if (tid < QKV_ROWS / 2) {
            const float *p0 = a.qkv_part + (size_t)g * 2 * QKV_ROWS, *p1 = p0 + QKV_ROWS;
            const int rr0 = 2 * tid;
            const float2 h0 = xld2(p0 + rr0), h1 = xld2(p1 + rr0);
            const float x0 = (h0.x + h1.x) * scale_a, x1 = (h0.y + h1.y) * scale_a;
            if (rr0 < (G + 1) * HD) {
                const int dd = rr0 % HD;
                float sn, cs;
                sincosf((float)pos * a.inv_freq[dd >> 1], &sn, &cs);
                const float o0 = x0 * cs - x1 * sn, o1 = x1 * cs + x0 * sn;
                if (rr0 < G * HD) { L.sq[rr0] = o0; L.sq[rr0 + 1] = o1; }
                else { L.sk16[dd] = f32_to_f16_bits(o0); L.sk16[dd + 1] = f32_to_f16_bits(o1); }
            } else {
                const int dd = rr0 - (G + 1) * HD;
                L.sv16[dd] = f32_to_f16_bits(x0);
                L.sv16[dd + 1] = f32_to_f16_bits(x1);
            }
        }
        wg_barrier_lds();
        if (w == 0 && tid < HD) {
            reinterpret_cast<uint16_t *>(cur.kcache + (((size_t)seq * NKV + g) * (size_t)a.n_ctx + pos) * (HD * 2))[tid] = L.sk16[tid];
            reinterpret_cast<uint16_t *>(cur.vcache + (((size_t)seq * NKV + g) * (size_t)a.n_ctx + pos) * (HD * 2))[tid] = L.sv16[tid];
        }

        // ---- B: the die's 4 query heads over keys [j0, j1) of kv head g
        {
            float q[G][8], acc[G][8], m[G], l[G];
            const float qs = a.attn_scale * 1.44269504088896341f;      // scores in log2 units
#pragma unroll
            for (int h = 0; h < G; ++h) {
#pragma unroll
                for (int i = 0; i < 8; ++i) { q[h][i] = L.sq[h * HD + ds + i] * qs; acc[h][i] = 0.f; }
                m[h] = -INFINITY;
                l[h] = 0.f;
            }
            for (int jb = j0; jb < j1; jb += ATT_SLOTS * ATT_KPT) {
                if (jb != j0) kv_fetch_pass(R, kb, vb, jb, j1, pos, slot, ds);
#pragma unroll
                for (int i = 0; i < ATT_KPT; ++i) {
                    if (jb + slot + ATT_SLOTS * i == pos) {      // the key of this step, from LDS
                        R.k[i].v = *reinterpret_cast<const uint4 *>(L.sk16 + ds);
                        R.v[i].v = *reinterpret_cast<const uint4 *>(L.sv16 + ds);
                    }
                }
                float sc[ATT_KPT][G];
#pragma unroll
                for (int i = 0; i < ATT_KPT; ++i) {
                    float kf[8];
                    kv_decode<MESH_F16>(R.k[i], kf);
                    const bool ok = jb + slot + ATT_SLOTS * i < j1;
#pragma unroll
                    for (int h = 0; h < G; ++h) {
                        float s = 0.f;
#pragma unroll
                        for (int e = 0; e < 8; ++e) s = fmaf(q[h][e], kf[e], s);
                        s = slot_sum<ATT_LPK>(s);
                        sc[i][h] = ok ? s : -INFINITY;
                    }
                }
                float vf[ATT_KPT][8];
#pragma unroll
                for (int i = 0; i < ATT_KPT; ++i) kv_decode<MESH_F16>(R.v[i], vf[i]);
#pragma unroll
                for (int h = 0; h < G; ++h) {
                    float mn = m[h];
#pragma unroll
                    for (int i = 0; i < ATT_KPT; ++i) mn = fmaxf(mn, sc[i][h]);
                    if (mn == -INFINITY) continue;
                    const float corr = exp2_fast(m[h] - mn);
                    float p[ATT_KPT], ps = 0.f;
#pragma unroll
                    for (int i = 0; i < ATT_KPT; ++i) { p[i] = exp2_fast(sc[i][h] - mn); ps += p[i]; }
                    l[h] = l[h] * corr + ps;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        float v = acc[h][e] * corr;
#pragma unroll
                        for (int i = 0; i < ATT_KPT; ++i) v = fmaf(p[i], vf[i][e], v);
                        acc[h][e] = v;
                    }
                    m[h] = mn;
                }
            }
            // merge the slots of this workgroup
            if ((tid % ATT_LPK) == 0) {
#pragma unroll
                for (int h = 0; h < G; ++h) L.s_m[slot][h] = m[h];
            }
            wg_barrier_lds();
#pragma unroll
            for (int h = 0; h < G; ++h) {
                float mh = -INFINITY;
#pragma unroll
                for (int s2 = 0; s2 < ATT_SLOTS; ++s2) mh = fmaxf(mh, L.s_m[s2][h]);
                const float wgt = (m[h] == -INFINITY) ? 0.f : exp2f(m[h] - mh);
                float lw = l[h] * wgt;
#pragma unroll
                for (int o = ATT_LPK; o < 64; o <<= 1) lw += __shfl_xor(lw, o);
                if (lane == 0) { L.s_l[wave][h] = lw; L.s_mw[h] = mh; }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float v = acc[h][e] * wgt;
#pragma unroll
                    for (int o = ATT_LPK; o < 64; o <<= 1) v += __shfl_xor(v, o);
                    if (lane < ATT_LPK) L.s_acc[wave][h][ds + e] = v;
                }
            }
            wg_barrier_lds();
            {
                const int h = tid / HD, dd = tid % HD;            // 512 threads = G x HD outputs
                float sum = 0.f, ll = 0.f;
#pragma unroll
                for (int w2 = 0; w2 < DD_WAVES; ++w2) { sum += L.s_acc[w2][h][dd]; ll += L.s_l[w2][h]; }
                const size_t row = ((size_t)g * WG_PER_DIE + w) * G + h;
                a.att_part[row * HD + dd] = sum;
                if (dd == 0) { a.att_ml[row * 2] = L.s_mw[h]; a.att_ml[row * 2 + 1] = ll; }
            }
        }
        drain_stores();
        prefetch_tiles<CNT_C>(r, desc_c, wave, lane, vz);
        if (!die_barrier(sy, &L.flag)) return;

        // ---- merge of the 32 key ranges, then C: the die's columns of Wo
        if (tid < WG_PER_DIE * G) {
            const float2 v = xld2(a.att_ml + ((size_t)g * WG_PER_DIE * G + tid) * 2);
            L.ml[tid * 2] = v.x;
            L.ml[tid * 2 + 1] = v.y;
        }
        float part[WG_PER_DIE];
        {
            const int h = tid / HD, dd = tid % HD;
#pragma unroll
            for (int s2 = 0; s2 < WG_PER_DIE; ++s2) part[s2] = xld(a.att_part + (((size_t)g * WG_PER_DIE + s2) * G + h) * HD + dd);
            wg_barrier_lds();
            float mh = -INFINITY;
#pragma unroll
            for (int s2 = 0; s2 < WG_PER_DIE; ++s2) mh = fmaxf(mh, L.ml[(s2 * G + h) * 2]);
            float num = 0.f, den = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < WG_PER_DIE; ++s2) {
                const float ms = L.ml[(s2 * G + h) * 2];
                const float wgt = ms == -INFINITY ? 0.f : exp2f(ms - mh);
                num = fmaf(part[s2], wgt, num);
                den = fmaf(L.ml[(s2 * G + h) * 2 + 1], wgt, den);
            }
            L.att[tid] = num / den;
        }
        wg_barrier_lds();
        x_zero(X);
        if (tid < A_K / 8) {
            X.a[0] = *reinterpret_cast<const float4 *>(L.att + tid * 8);
            X.b[0] = *reinterpret_cast<const float4 *>(L.att + tid * 8 + 4);
        }
        (void)stage_x(X, A_K, S, tid);
        wg_barrier_lds();
        run_tiles<CNT_C>(r, desc_c, S, A_K, L.red, wave, lane, vz);
        wg_barrier_lds();
        if (tid < ROWS_WG) {
            const int j = tid >> 4, rr = tid & 15;
            xst(a.p1 + (size_t)g * E + ROWS_WG * w + tid, L.red[(j * 2) * 16 + rr] + L.red[(j * 2 + 1) * 16 + rr]);
        }
        drain_stores();
        prefetch_tiles<CNT_D>(r, desc_d, wave, lane, vz);
        X.w0 = ldg<float4>(cur.ffn_norm + tid * 8);
        X.w1 = ldg<float4>(cur.ffn_norm + tid * 8 + 4);
        if (!chip_barrier(sy, &L.flag)) return;

        // ---- the die's own copy of the hidden state after the attention block
        if (tid < ROWS_WG) {
            const int row = ROWS_WG * w + tid;
            float s = xld(h_src + row);
#pragma unroll
            for (int d = 0; d < N_DIE; ++d) s += xld(a.p1 + (size_t)d * E + row);
            a.h_loc[(size_t)g * E + row] = s;
        }
        drain_stores();
        if (!die_barrier(sy, &L.flag)) return;

        // ---- D: this die's rows of gate and up over the normalised hidden state
        {
            const float4 w0 = X.w0, w1 = X.w1;
            x_from_exchange(X, a.h_loc + (size_t)g * E, tid);
            X.w0 = w0; X.w1 = w1;
        }
        const float scale_f = wg_norm_scale(stage_x(X, E, S, tid), L, E, a.eps, wave, lane);
        run_tiles<CNT_D>(r, desc_d, S, E, L.red, wave, lane, vz);
        wg_barrier_lds();
        if (tid < 7 * 2 * 16) {
            const int ul = tid >> 5, mat = (tid >> 4) & 1, rr = tid & 15, u = 7 * w + ul;
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) s += L.red[((ul * 2 + mat) * 8 + i) * 16 + rr];
            a.gu_part[(((size_t)g * 2 + mat) * 2 + (u & 1)) * FF_DIE + (u >> 1) * 16 + rr] = s;
        }
        drain_stores();
        prefetch_tiles<CNT_E>(r, desc_e, wave, lane, vz);
        if (!die_barrier(sy, &L.flag)) return;

        // ---- SwiGLU over the die's 1792 columns, then E: those columns of W_down
        x_zero(X);
        if (tid < FF_DIE / 8) {
            const float *gp = a.gu_part + (size_t)g * 4 * FF_DIE + tid * 8;
            float act[8];
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const float2 g0 = xld2(gp + i), g1 = xld2(gp + FF_DIE + i), u0 = xld2(gp + 2 * FF_DIE + i), u1 = xld2(gp + 3 * FF_DIE + i);
                const float ga = (g0.x + g1.x) * scale_f, gb = (g0.y + g1.y) * scale_f;
                const float ua = (u0.x + u1.x) * scale_f, ub = (u0.y + u1.y) * scale_f;
                act[i] = (ga / (1.0f + expf(-ga))) * ua;
                act[i + 1] = (gb / (1.0f + expf(-gb))) * ub;
            }
            X.a[0] = make_float4(act[0], act[1], act[2], act[3]);
            X.b[0] = make_float4(act[4], act[5], act[6], act[7]);
        }
        (void)stage_x(X, FF_DIE, S, tid);
        wg_barrier_lds();
        run_tiles<CNT_E>(r, desc_e, S, FF_DIE, L.red, wave, lane, vz);
        wg_barrier_lds();
        if (tid < ROWS_WG) {
            const int j = tid >> 4, rr = tid & 15;
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < FF_SB; ++i) s += L.red[(j * FF_SB + i) * 16 + rr];
            xst(a.p2 + (size_t)g * E + ROWS_WG * w + tid, s);
        }
        drain_stores();
        if (!last) {
            cur = a.layers[il + 1];
            prefetch_tiles<CNT_A>(r, desc_a, wave, lane, vz);
            X.w0 = ldg<float4>(cur.attn_norm + tid * 8);
            X.w1 = ldg<float4>(cur.attn_norm + tid * 8 + 4);
        }
        if (!chip_barrier(sy, &L.flag)) return;

        // ---- hidden state after the layer
        if (tid < ROWS_WG) {
            const int row = ROWS_WG * w + tid;
            float s = xld(a.h_loc + (size_t)g * E + row);
#pragma unroll
            for (int d = 0; d < N_DIE; ++d) s += xld(a.p2 + (size_t)d * E + row);
            if (last) {
                if (g == 0) a.x[row] = s;
            } else {
                a.h_loc[(size_t)g * E + row] = s;
            }
        }
        if (last) break;
        drain_stores();
        if (!die_barrier(sy, &L.flag)) return;
    }
}

// how many workgroups of this launch geometry each die gets
__global__ __launch_bounds__(DD_THREADS) void die_probe_kernel(unsigned *per_die) {
    if (threadIdx.x == 0) atomicAdd(per_die + (xcc_id() & 15u), 1u);
}

// One step at a time on the device, whatever the session: two of these kernels resident together could each hold compute
// units the other is waiting for.  A step of another session first waits for the last launcher's stream.
std::mutex g_chain_mu;
hipEvent_t g_chain_event = nullptr;
DieDecode *g_chain_last = nullptr;

}  // namespace

struct DieDecode {
    DieLayer *d_layers = nullptr;
    float *qkv_part = nullptr, *att_part = nullptr, *att_ml = nullptr, *h_loc = nullptr, *gu_part = nullptr, *p1 = nullptr, *p2 = nullptr;
    unsigned *sync = nullptr;
    unsigned *host_flag = nullptr;         // pinned
    unsigned n_die = 0, n_chip = 0;        // barriers completed so far
    unsigned n_ticket = 0;                 // rank tickets handed out per die so far
    unsigned spin_limit = 1u << 22;
    int n_layer = 0;
    hipStream_t stream = nullptr;
    std::vector<void *> allocations;
};

static bool kq(const DevTensor &t, int64_t M, int64_t K) {
    return t.present() && t.tiled && (t.type == MESH_Q4_K || t.type == MESH_Q6_K) && t.M == M && t.K == K && t.E == 1;
}

bool die_decode_eligible(const mesh_stage *st) {
    const char *env = getenv("MESH_DECODE_DIE");          // MESH_DECODE_DIE=1 when the session is created turns it on
    if (!env || atoi(env) == 0 || !st || st->layers.empty()) return false;
    const HParams &hp = st->hp;
    if (hp.n_embd != E || hp.n_ff != FF || hp.n_head != NH || hp.n_head_kv != NKV || hp.head_dim != HD || hp.n_rot != HD ||
        hp.rope_mode != ROPE_NORM || hp.n_expert != 0 || st->k_type != MESH_F16 || st->v_type != MESH_F16)
        return false;
    for (const LayerWeights &L : st->layers) {
        if (!kq(L.wq, NH * HD, E) || !kq(L.wk, NKV * HD, E) || !kq(L.wv, NKV * HD, E) || !kq(L.wo, E, NH * HD) || !kq(L.w_gate, FF, E) ||
            !kq(L.w_up, FF, E) || !kq(L.w_down, E, FF))
            return false;
        if (L.bq.present() || L.bk.present() || L.bv.present() || L.q_norm.present() || L.k_norm.present() || !L.attn_norm.present() ||
            !L.ffn_norm.present() || L.gate_inp.present())
            return false;
    }
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, st->device) != hipSuccess || p.multiProcessorCount != DD_GRID) return false;
    return true;
}

void die_decode_destroy(DieDecode *d) {
    if (!d) return;
    {
        std::lock_guard<std::mutex> lock(g_chain_mu);
        if (g_chain_last == d) g_chain_last = nullptr;       // (the owner has synchronised its stream)
    }
    for (void *p : d->allocations) (void)hipFree(p);
    if (d->host_flag) (void)hipHostFree(d->host_flag);
    delete d;
}

int die_decode_create(mesh_session *s, DieDecode **out) {
    *out = nullptr;
    const mesh_stage *st = s->stage;
    if (!die_decode_eligible(st)) return MESH_OK;
    std::unique_ptr<DieDecode, void (*)(DieDecode *)> d(new DieDecode, die_decode_destroy);
    auto alloc = [&](auto **p, size_t bytes) -> int {
        void *v = nullptr;
        MESH_HIP_TRY(hipMalloc(&v, bytes));
        d->allocations.push_back(v);
        MESH_HIP_TRY(hipMemset(v, 0, bytes));
        *p = static_cast<std::remove_reference_t<decltype(**p)> *>(v);
        return MESH_OK;
    };
    int rc;
    if ((rc = alloc(&d->qkv_part, sizeof(float) * N_DIE * 2 * QKV_ROWS)) != MESH_OK) return rc;
    if ((rc = alloc(&d->att_part, sizeof(float) * N_DIE * WG_PER_DIE * G * HD)) != MESH_OK) return rc;
    if ((rc = alloc(&d->att_ml, sizeof(float) * N_DIE * WG_PER_DIE * G * 2)) != MESH_OK) return rc;
    if ((rc = alloc(&d->h_loc, sizeof(float) * N_DIE * E)) != MESH_OK) return rc;
    if ((rc = alloc(&d->gu_part, sizeof(float) * N_DIE * 4 * FF_DIE)) != MESH_OK) return rc;
    if ((rc = alloc(&d->p1, sizeof(float) * N_DIE * E)) != MESH_OK) return rc;
    if ((rc = alloc(&d->p2, sizeof(float) * N_DIE * E)) != MESH_OK) return rc;
    if ((rc = alloc(&d->sync, sizeof(unsigned) * SYNC_WORDS)) != MESH_OK) return rc;
    MESH_HIP_TRY(hipHostMalloc(reinterpret_cast<void **>(&d->host_flag), sizeof(unsigned), hipHostMallocDefault));
    *d->host_flag = 0;
    d->n_layer = (int)st->layers.size();
    d->stream = s->stream;
    if (const char *e = getenv("MESH_DECODE_DIE_SPINS")) d->spin_limit = (unsigned)strtoul(e, nullptr, 10);

    std::vector<DieLayer> tab(st->layers.size());
    for (size_t il = 0; il < st->layers.size(); ++il) {
        const LayerWeights &L = st->layers[il];
        DieLayer &t = tab[il];
        const DevTensor *m[7] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.w_gate, &L.w_up, &L.w_down};
        const uint8_t **dst[7] = {&t.wq, &t.wk, &t.wv, &t.wo, &t.wg, &t.wu, &t.wd};
        t.q6 = 0;
        for (int i = 0; i < 7; ++i) {
            *dst[i] = static_cast<const uint8_t *>(m[i]->data);
            if (m[i]->type == MESH_Q6_K) t.q6 |= 1u << i;
        }
        t.attn_norm = static_cast<const float *>(L.attn_norm.data);
        t.ffn_norm = static_cast<const float *>(L.ffn_norm.data);
        t.kcache = s->kcache + il * s->k_layer_bytes;
        t.vcache = s->vcache + il * s->v_layer_bytes;
    }
    if ((rc = alloc(&d->d_layers, sizeof(DieLayer) * tab.size())) != MESH_OK) return rc;
    MESH_HIP_TRY(hipMemcpy(d->d_layers, tab.data(), sizeof(DieLayer) * tab.size(), hipMemcpyHostToDevice));

    // every die must get 32 of the 256 workgroups, also when the launch before it left the dealing order elsewhere
    unsigned *per_die = d->sync + SYNC_ABORT + 16, h_per_die[16];
    for (int offset : {0, 3}) {
        if (offset) {
            MESH_LAUNCH(die_probe_kernel, dim3((unsigned)offset), dim3(64), 0, s->stream, per_die + 16);
            MESH_LAUNCH_CHECK();
        }
        MESH_HIP_TRY(hipMemsetAsync(per_die, 0, sizeof(h_per_die), s->stream));
        MESH_LAUNCH(die_probe_kernel, dim3(DD_GRID), dim3(DD_THREADS), 0, s->stream, per_die);
        MESH_LAUNCH_CHECK();
        MESH_HIP_TRY(hipMemcpyAsync(h_per_die, per_die, sizeof(h_per_die), hipMemcpyDeviceToHost, s->stream));
        MESH_HIP_TRY(hipStreamSynchronize(s->stream));
        for (int i = 0; i < 16; ++i)
            if (h_per_die[i] != (i < N_DIE ? (unsigned)WG_PER_DIE : 0u)) return MESH_OK;      // keep the launch-per-projection path
    }
    MESH_HIP_TRY(hipMemset(d->sync, 0, sizeof(unsigned) * SYNC_WORDS));
    *out = d.release();
    return MESH_OK;
}

int die_decode_check(mesh_session *s, DieDecode *d) {
    if (!d || *static_cast<volatile unsigned *>(d->host_flag) == 0) return MESH_OK;
    const unsigned why = *static_cast<volatile unsigned *>(d->host_flag);
    (void)hipStreamSynchronize(s->stream);
    (void)hipMemset(d->sync, 0, sizeof(unsigned) * SYNC_WORDS);
    d->n_die = d->n_chip = d->n_ticket = 0;
    *d->host_flag = 0;
    return fail(MESH_ERR_DEVICE, why == 2 ? "decode step abandoned: a workgroup ran on a compute die other than the one its index implies"
                                          : "decode step abandoned: a wait between workgroups inside the kernel gave up");
}

int die_decode_step(mesh_session *s, DieDecode *d) {
    int rc;
    if ((rc = die_decode_check(s, d)) != MESH_OK) return rc;
    const mesh_stage *st = s->stage;
    DieArgs a;
    a.layers = d->d_layers; a.n_layer = d->n_layer;
    a.x = s->x; a.pos = s->d_pos; a.seq = s->d_seq; a.inv_freq = st->rope_inv_freq;
    a.eps = st->hp.rms_eps; a.attn_scale = 1.0f / sqrtf((float)HD); a.n_ctx = st->n_ctx;
    a.qkv_part = d->qkv_part; a.att_part = d->att_part; a.att_ml = d->att_ml; a.h_loc = d->h_loc; a.gu_part = d->gu_part;
    a.p1 = d->p1; a.p2 = d->p2; a.sync = d->sync; a.host_flag = d->host_flag;
    a.base_die = d->n_die; a.base_chip = d->n_chip; a.base_ticket = d->n_ticket; a.spin_limit = d->spin_limit;
    std::lock_guard<std::mutex> lock(g_chain_mu);
    if (g_chain_last && g_chain_last != d) {
        if (!g_chain_event) MESH_HIP_TRY(hipEventCreateWithFlags(&g_chain_event, hipEventDisableTiming));
        MESH_HIP_TRY(hipEventRecord(g_chain_event, g_chain_last->stream));
        MESH_HIP_TRY(hipStreamWaitEvent(s->stream, g_chain_event, 0));
    }
    g_chain_last = d;
    MESH_LAUNCH(decode_die_kernel, dim3(DD_GRID), dim3(DD_THREADS), 0, s->stream, a);
    MESH_LAUNCH_CHECK();
    d->n_die += 5u * (unsigned)d->n_layer - 1u;
    d->n_chip += 2u * (unsigned)d->n_layer;
    d->n_ticket += (unsigned)WG_PER_DIE;
    return MESH_OK;
}

}  // namespace mesh
