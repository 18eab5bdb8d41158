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
