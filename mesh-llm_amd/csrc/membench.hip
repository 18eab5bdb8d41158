// HBM read-bandwidth probe: what a pure streaming read reaches on this GPU, as the yardstick beside the nominal
// 8 TB/s for every HBM-bound kernel of the library.  Same protocol as the reference's GPU fingerprint benchmark
// (mesh-llm/benchmarks/membench-fingerprint.hip:24-39 buffer and kernel, :151-160 event-timed dispatch, warm-up
// runs then timed runs, percentiles taken by the caller), with a read kernel shaped for gfx950: eight independent
// 16-byte loads per lane in flight, workgroups striding the buffer.

#include <vector>

#include "mesh_common.hpp"

namespace mesh {

constexpr int MB_THREADS = 256, MB_UNROLL = 8;

__global__ __launch_bounds__(MB_THREADS) void memread_kernel(const uint4 *__restrict__ src, uint32_t *sink, size_t n_vec) {
    const size_t per_wg = (size_t)MB_THREADS * MB_UNROLL;
    uint32_t acc = 0;
    for (size_t base = (size_t)blockIdx.x * per_wg; base < n_vec; base += (size_t)gridDim.x * per_wg) {
        uint4 v[MB_UNROLL];
#pragma unroll
        for (int u = 0; u < MB_UNROLL; ++u) {
            const size_t i = base + (size_t)u * MB_THREADS + threadIdx.x;
            v[u] = i < n_vec ? src[i] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < MB_UNROLL; ++u) acc |= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9E3779B9u) atomicAdd(sink, acc);     // never true for a zero-filled buffer; keeps the loads alive
}

// Plain streaming mix: every workgroup pass reads RD and writes WR 16-byte vectors per thread, each instruction of a
// wave covering one contiguous kilobyte, non-temporal both ways, one pass per workgroup.  No arithmetic to speak of:
// what this reaches for a given read : write ratio and size is what the memory system gives a kernel of that traffic
// shape, the yardstick for the codec kernels (q8_0 pack reads 3.8 bytes per byte written, f16 pack 2, the unpacks the
// reverse).
typedef unsigned int mb_u32x4 __attribute__((ext_vector_type(4)));
template <int RD, int WR>
__global__ __launch_bounds__(MB_THREADS) void memmix_kernel(const mb_u32x4 *__restrict__ src, mb_u32x4 *__restrict__ dst) {
    const mb_u32x4 *s = src + (size_t)blockIdx.x * MB_THREADS * RD + threadIdx.x;
    mb_u32x4 *d = dst + (size_t)blockIdx.x * MB_THREADS * WR + threadIdx.x;
    mb_u32x4 v[RD];
#pragma unroll
    for (int r = 0; r < RD; ++r) v[r] = __builtin_nontemporal_load(s + r * MB_THREADS);
    mb_u32x4 a = v[0];
#pragma unroll
    for (int r = 1; r < RD; ++r) a ^= v[r];
#pragma unroll
    for (int w = 0; w < WR; ++w) {
        mb_u32x4 o = a;
        o.x += w;
        __builtin_nontemporal_store(o, d + w * MB_THREADS);
    }
}

// Matrix-core issue probe: every wave keeps four independent v_mfma_f32_32x32x16_f16 accumulation chains going from
// registers alone (no memory traffic at all), four waves per SIMD.  What this sustains is what the matrix pipes deliver
// at the clock the chip holds under that load, the yardstick beside the nominal 2.5 PFLOP/s for the prefill GEMM.
typedef _Float16 mb_half8 __attribute__((ext_vector_type(8)));
typedef float mb_float16 __attribute__((ext_vector_type(16)));
constexpr int MFMA_PROBE_CHAINS = 4;
__global__ __launch_bounds__(MB_THREADS) void mfma_probe_kernel(float *sink, int iters) {
    // operands of mixed sign and magnitude below one, different in every lane, so the accumulators wander instead of running away
    uint32_t h = (uint32_t)(blockIdx.x * MB_THREADS + threadIdx.x) * 2654435761u + 12345u;
    mb_half8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        h = h * 1664525u + 1013904223u;
        a[i] = (_Float16)(((int)(h >> 20) - 2048) * (1.0f / 2048.0f));
        h = h * 1664525u + 1013904223u;
        b[i] = (_Float16)(((int)(h >> 20) - 2048) * (1.0f / 2048.0f));
    }
    mb_float16 c[MFMA_PROBE_CHAINS];
#pragma unroll
    for (int k = 0; k < MFMA_PROBE_CHAINS; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) c[k][i] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < MFMA_PROBE_CHAINS; ++k) c[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c[k], 0, 0, 0);
    }
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < MFMA_PROBE_CHAINS; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) t += c[k][i];
    if (t == 123456.789f) sink[0] = t;       // keeps the chains alive; practically never true
}

}  // namespace mesh

using namespace mesh;

extern "C" int mesh_hbm_read_probe(size_t bytes, int warmup_runs, int timed_runs, double *gbps) {
    if (bytes < (1u << 20) || timed_runs < 1 || warmup_runs < 0 || !gbps) return fail(MESH_ERR_INVALID, "mesh_hbm_read_probe: bad arguments");
    void *src = nullptr;
    uint32_t *sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = MESH_OK;
    auto done = [&](int r) {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        if (src) (void)hipFree(src);
        if (sink) (void)hipFree(sink);
        return r;
    };
#define MB_TRY(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) return done(fail(MESH_ERR_DEVICE, "mesh_hbm_read_probe: %s", hipGetErrorString(e_))); } while (0)
    MB_TRY(hipMalloc(&src, bytes));
    MB_TRY(hipMalloc(reinterpret_cast<void **>(&sink), sizeof(uint32_t)));
    MB_TRY(hipMemset(src, 0, bytes));
    MB_TRY(hipMemset(sink, 0, sizeof(uint32_t)));
    MB_TRY(hipEventCreate(&e0));
    MB_TRY(hipEventCreate(&e1));
    int dev = 0;
    hipDeviceProp_t prop;
    MB_TRY(hipGetDevice(&dev));
    MB_TRY(hipGetDeviceProperties(&prop, dev));
    const size_t n_vec = bytes / 16;
    const size_t per_wg = (size_t)MB_THREADS * MB_UNROLL;
    const size_t want = (n_vec + per_wg - 1) / per_wg;
    const unsigned grid = (unsigned)std::min<size_t>(want, (size_t)prop.multiProcessorCount * 32);
    for (int i = 0; i < warmup_runs + timed_runs; ++i) {
        MB_TRY(hipEventRecord(e0, nullptr));
        memread_kernel<<<dim3(grid), dim3(MB_THREADS), 0, nullptr>>>(static_cast<const uint4 *>(src), sink, n_vec);
        MB_TRY(hipGetLastError());
        MB_TRY(hipEventRecord(e1, nullptr));
        MB_TRY(hipEventSynchronize(e1));
        float ms = 0.f;
        MB_TRY(hipEventElapsedTime(&ms, e0, e1));
        if (i >= warmup_runs) gbps[i - warmup_runs] = (double)(n_vec * 16) / ((double)ms * 1e-3) / 1e9;
    }
#undef MB_TRY
    return done(rc);
}

extern "C" int mesh_hbm_mix_probe_dev(const void *d_src, void *d_dst, size_t big_bytes, int ratio, int big_is_read, void *stream) {
    if (!d_src || !d_dst || (ratio != 1 && ratio != 2 && ratio != 4)) return fail(MESH_ERR_INVALID, "mesh_hbm_mix_probe_dev: bad arguments");
    const size_t per_wg = (size_t)MB_THREADS * 16 * ratio;        // bytes of the larger side one workgroup moves
    if (big_bytes < per_wg || big_bytes % per_wg) return fail(MESH_ERR_INVALID, "mesh_hbm_mix_probe_dev: %zu bytes is not a multiple of %zu", big_bytes, per_wg);
    if ((reinterpret_cast<uintptr_t>(d_src) | reinterpret_cast<uintptr_t>(d_dst)) & 15u) return fail(MESH_ERR_INVALID, "mesh_hbm_mix_probe_dev: pointers must be 16-byte aligned");
    const dim3 grid((unsigned)(big_bytes / per_wg)), block(MB_THREADS);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const mb_u32x4 *s = static_cast<const mb_u32x4 *>(d_src);
    mb_u32x4 *d = static_cast<mb_u32x4 *>(d_dst);
    if (ratio == 1) MESH_LAUNCH((memmix_kernel<1, 1>), grid, block, 0, st, s, d);
    else if (ratio == 2 && big_is_read) MESH_LAUNCH((memmix_kernel<2, 1>), grid, block, 0, st, s, d);
    else if (ratio == 2) MESH_LAUNCH((memmix_kernel<1, 2>), grid, block, 0, st, s, d);
    else if (big_is_read) MESH_LAUNCH((memmix_kernel<4, 1>), grid, block, 0, st, s, d);
    else MESH_LAUNCH((memmix_kernel<1, 4>), grid, block, 0, st, s, d);
    MESH_LAUNCH_CHECK();
    return MESH_OK;
}

extern "C" int mesh_mfma_f16_probe(int iters, int warmup_runs, int timed_runs, double *tflops) {
    if (iters < 1 || timed_runs < 1 || warmup_runs < 0 || !tflops) return fail(MESH_ERR_INVALID, "mesh_mfma_f16_probe: bad arguments");
    float *sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto done = [&](int r) {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        if (sink) (void)hipFree(sink);
        return r;
    };
#define MB_TRY(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) return done(fail(MESH_ERR_DEVICE, "mesh_mfma_f16_probe: %s", hipGetErrorString(e_))); } while (0)
    MB_TRY(hipMalloc(reinterpret_cast<void **>(&sink), sizeof(float)));
    MB_TRY(hipEventCreate(&e0));
    MB_TRY(hipEventCreate(&e1));
    int dev = 0;
    hipDeviceProp_t prop;
    MB_TRY(hipGetDevice(&dev));
    MB_TRY(hipGetDeviceProperties(&prop, dev));
    const unsigned grid = (unsigned)prop.multiProcessorCount * 4;          // four 4-wave workgroups per CU: four waves per SIMD
    const double flop = (double)grid * (MB_THREADS / 64) * (double)iters * MFMA_PROBE_CHAINS * (2.0 * 32 * 32 * 16);
    for (int i = 0; i < warmup_runs + timed_runs; ++i) {
        MB_TRY(hipEventRecord(e0, nullptr));
        mfma_probe_kernel<<<dim3(grid), dim3(MB_THREADS), 0, nullptr>>>(sink, iters);
        MB_TRY(hipGetLastError());
        MB_TRY(hipEventRecord(e1, nullptr));
        MB_TRY(hipEventSynchronize(e1));
        float ms = 0.f;
        MB_TRY(hipEventElapsedTime(&ms, e0, e1));
        if (i >= warmup_runs) tflops[i - warmup_runs] = flop / ((double)ms * 1e-3) / 1e12;
    }
#undef MB_TRY
    return done(MESH_OK);
}
