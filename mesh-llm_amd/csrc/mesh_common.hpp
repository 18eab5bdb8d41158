// Shared host/device helpers for libmeshstage (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <tuple>
#include <utility>

#include "../../include/mesh_stage.h"

namespace mesh {

// thread-local last-error text behind mesh_last_error()
std::string &last_error_slot();
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define MESH_HIP_TRY(expr)                                                                   \
    do {                                                                                     \
        hipError_t _e = (expr);                                                              \
        if (_e != hipSuccess)                                                                \
            return ::mesh::fail(MESH_ERR_DEVICE, "%s failed: %s (%s:%d)", #expr,             \
                                hipGetErrorString(_e), __FILE__, __LINE__);                  \
    } while (0)

// after a kernel launch
#define MESH_LAUNCH_CHECK()                                                                  \
    do {                                                                                     \
        hipError_t _e = hipGetLastError();                                                   \
        if (_e != hipSuccess)                                                                \
            return ::mesh::fail(MESH_ERR_DEVICE, "kernel launch failed: %s (%s:%d)",         \
                                hipGetErrorString(_e), __FILE__, __LINE__);                  \
    } while (0)

// ---- kernel launches --------------------------------------------------------------------------------------------
// Every kernel goes out through MESH_LAUNCH.  While the calling thread is inside a profiled scope of a session
// (mesh_session_profile), the launch carries a start / stop event pair of its own: the runtime stamps them from the
// dispatch itself, so the measured span is the kernel's and nothing is added to the stream between launches (an event
// recorded around a launch adds a marker packet on either side, which at a few microseconds per kernel is a
// perturbation of the same order as the thing measured).  Otherwise both events are null and this is a plain launch.
struct LaunchTimer {
    hipEvent_t start = nullptr, stop = nullptr;
};
LaunchTimer launch_timer();

template <typename... KArgs, size_t... I>
inline void launch_kernel_impl(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t smem, hipStream_t stream, std::tuple<KArgs...> &formal,
                               std::index_sequence<I...>) {
    void *ptrs[sizeof...(KArgs) ? sizeof...(KArgs) : 1] = {static_cast<void *>(&std::get<I>(formal))...};
    const LaunchTimer t = launch_timer();
    (void)hipExtLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, ptrs, smem, stream, t.start, t.stop, 0);
}
template <typename... KArgs, typename... Args>
inline void launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t smem, hipStream_t stream, Args &&...args) {
    static_assert(sizeof...(KArgs) == sizeof...(Args), "argument count differs from the kernel's parameter list");
    std::tuple<KArgs...> formal(static_cast<KArgs>(args)...);       // the arguments in the kernel's own parameter types
    launch_kernel_impl(kernel, grid, block, smem, stream, formal, std::index_sequence_for<KArgs...>{});
}
#define MESH_LAUNCH(kernel, grid, block, smem, stream, ...) ::mesh::launch_kernel(kernel, grid, block, smem, stream, ##__VA_ARGS__)

// block geometry of the GGUF types on the stage path
constexpr int QK8_0 = 32, Q8_0_BYTES = 34;
constexpr int QK5_0 = 32, Q5_0_BYTES = 22;
constexpr int QK_K = 256, Q4_K_BYTES = 144, Q6_K_BYTES = 210;

// device-side twins (int math)
__host__ __device__ inline int block_elems_dev(int type) {
    return (type == MESH_F32 || type == MESH_F16) ? 1 : (type == MESH_Q5_0 || type == MESH_Q8_0) ? 32 : 256;
}
__host__ __device__ inline int block_bytes_dev(int type) {
    return type == MESH_F32 ? 4 : type == MESH_F16 ? 2 : type == MESH_Q5_0 ? Q5_0_BYTES : type == MESH_Q8_0 ? Q8_0_BYTES
         : type == MESH_Q4_K ? Q4_K_BYTES : Q6_K_BYTES;
}

inline int64_t block_elems(int type) {
    switch (type) {
        case MESH_F32: case MESH_F16: return 1;
        case MESH_Q5_0: case MESH_Q8_0: return 32;
        case MESH_Q4_K: case MESH_Q6_K: return 256;
        default: return -1;
    }
}
inline int64_t block_bytes(int type) {
    switch (type) {
        case MESH_F32: return 4;
        case MESH_F16: return 2;
        case MESH_Q5_0: return Q5_0_BYTES;
        case MESH_Q8_0: return Q8_0_BYTES;
        case MESH_Q4_K: return Q4_K_BYTES;
        case MESH_Q6_K: return Q6_K_BYTES;
        default: return -1;
    }
}
// bytes of a row of k elements, -1 if not a whole number of blocks
inline int64_t row_bytes(int type, int64_t k) {
    const int64_t be = block_elems(type);
    if (be < 0 || k < 0 || k % be) return -1;
    return k / be * block_bytes(type);
}

#ifdef __HIPCC__
// binary16 bits <-> f32.  v_cvt_f16_f32 rounds to nearest even and produces subnormals; NaN is
// canonicalised to sign|0x7E00 (the portable GGML_FP32_TO_FP16 result).
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    const uint16_t h = __half_as_ushort(__float2half_rn(f));
    const uint32_t w = __float_as_uint(f);
    return (w & 0x7FFFFFFFu) > 0x7F800000u ? (uint16_t)(((w >> 16) & 0x8000u) | 0x7E00u) : h;
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return __half2float(__ushort_as_half(h)); }

// The f16 producers of the batched paths clamp what f16 cannot hold to +-65504.  A caller can ask how often that happened
// (mesh_session_f16_saturations): every producer that can meet such a value is handed the session's counter and notes each
// group of values it clamps.  `sat` may be null (no counting).
__device__ __forceinline__ void note_f16_clamp(unsigned *sat, float a, float b, float c = 0.f, float d = 0.f) {
    if (sat && fmaxf(fmaxf(fabsf(a), fabsf(b)), fmaxf(fabsf(c), fabsf(d))) > 65504.f) atomicAdd(sat, 1u);
}
#endif

}  // namespace mesh
