// extern "C" surface of libmeshstage.so (declared in include/mesh_stage.h).

#include <cctype>
#include <cstring>
#include <mutex>

#include "mesh_common.hpp"

namespace mesh {

std::string &last_error_slot() {
    static thread_local std::string slot;
    return slot;
}

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    last_error_slot() = buf;
    return code;
}

int act_pack_dev(int fmt, const float *src, void *dst, int64_t n, hipStream_t stream);
int act_unpack_dev(int fmt, const void *src, float *dst, int64_t n, hipStream_t stream);
int dequantize_dev(int type, const void *src, float *dst, int64_t n, hipStream_t stream);

static bool is_act_fmt(int fmt) { return fmt == MESH_F32 || fmt == MESH_F16 || fmt == MESH_Q8_0; }

// RAII device scratch for the host-pointer entry points
struct DevScratch {
    void *p = nullptr;
    ~DevScratch() { if (p) (void)hipFree(p); }
    int alloc(size_t bytes) {
        hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
        if (e != hipSuccess) {
            p = nullptr;
            return fail(e == hipErrorOutOfMemory ? MESH_ERR_NOMEM : MESH_ERR_DEVICE, "hipMalloc(%zu) failed: %s", bytes,
                        hipGetErrorString(e));
        }
        return MESH_OK;
    }
};

// ---- device staging of mesh_act_pack_noalloc ---------------------------------------------------------------
// The f32 input and the packed output of one call, at most NOALLOC_MAX_ELEMS elements: input at offset 0, output at
// NOALLOC_OUT_OFFSET.  Every GPU the library runs on holds its own copy of the array until the process ends.  The
// name below is a host-side handle only; the device address is asked for once per device (with that device current)
// and everything -- copies and kernel arguments -- goes through that address.
constexpr int64_t NOALLOC_MAX_ELEMS = (int64_t)1 << 20;                        // 256 tokens x 4096
constexpr size_t NOALLOC_OUT_OFFSET = (size_t)NOALLOC_MAX_ELEMS * 4;
constexpr size_t NOALLOC_BYTES = 2 * NOALLOC_OUT_OFFSET;                       // 8 MiB
static __device__ __align__(256) uint8_t scratch[NOALLOC_BYTES];

constexpr int NOALLOC_MAX_DEVICES = 64;
static std::mutex g_noalloc_mu;                         // one call at a time: the array is shared by every caller of a GPU
static uint8_t *g_noalloc_ptr[NOALLOC_MAX_DEVICES];     // device address of `scratch` on each device, null until asked for

// device address of this device's copy of the staging array (caller holds g_noalloc_mu)
static int noalloc_scratch(uint8_t **out) {
    int dev = -1;
    MESH_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return fail(MESH_ERR_DEVICE, "mesh_act_pack_noalloc: device index %d out of range", dev);
    if (!g_noalloc_ptr[dev]) {
        void *p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(MESH_ERR_DEVICE, "mesh_act_pack_noalloc: no device address for the staging array on device %d: %s", dev, hipGetErrorString(e));
        g_noalloc_ptr[dev] = static_cast<uint8_t *>(p);
    }
    *out = g_noalloc_ptr[dev];
    return MESH_OK;
}

}  // namespace mesh

using namespace mesh;

extern "C" {

const char *mesh_last_error(void) { return last_error_slot().c_str(); }

int mesh_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int mesh_device_select(const char *device) {
    if (!device) return fail(MESH_ERR_INVALID, "mesh_device_select: null device string");
    const char *p = device;
    while (*p && !isdigit((unsigned char)*p)) ++p;
    const size_t prefix = (size_t)(p - device);
    const bool known = prefix == 0 || (prefix == 4 && !strncasecmp(device, "ROCm", 4)) ||
                       (prefix == 3 && !strncasecmp(device, "HIP", 3));
    if (!known || !*p) return fail(MESH_ERR_INVALID, "mesh_device_select: cannot parse device '%s' (want ROCm<N>, HIP<N> or <N>)", device);
    char *end = nullptr;
    const long idx = strtol(p, &end, 10);
    if (*end) return fail(MESH_ERR_INVALID, "mesh_device_select: trailing characters in '%s'", device);
    const int n = mesh_device_count();
    if (idx < 0 || idx >= n) return fail(MESH_ERR_DEVICE, "mesh_device_select: device %ld not present (%d available)", idx, n);
    MESH_HIP_TRY(hipSetDevice((int)idx));
    return MESH_OK;
}

size_t mesh_act_packed_size(int fmt, int64_t n_tokens, int64_t n_embd) {
    if (!is_act_fmt(fmt) || n_tokens < 0 || n_embd < 0) return 0;
    const int64_t per_row = row_bytes(fmt, n_embd);   // ggml rows never straddle blocks
    if (per_row < 0) return 0;
    return (size_t)(per_row * n_tokens);
}

int mesh_act_pack_dev(int fmt, const float *d_src, void *d_dst, int64_t n, void *stream) {
    return act_pack_dev(fmt, d_src, d_dst, n, static_cast<hipStream_t>(stream));
}

int mesh_act_unpack_dev(int fmt, const void *d_src, float *d_dst, int64_t n, void *stream) {
    return act_unpack_dev(fmt, d_src, d_dst, n, static_cast<hipStream_t>(stream));
}

int mesh_dequantize_dev(int type, const void *d_src, float *d_dst, int64_t n, void *stream) {
    return dequantize_dev(type, d_src, d_dst, n, static_cast<hipStream_t>(stream));
}

int mesh_act_pack(int fmt, const float *src, void *dst, int64_t n) {
    if (!is_act_fmt(fmt)) return fail(MESH_ERR_INVALID, "mesh_act_pack: format %d is not an activation format", fmt);
    if (n < 0 || (n > 0 && (!src || !dst))) return fail(MESH_ERR_INVALID, "mesh_act_pack: null pointer or negative count");
    const int64_t out_bytes = row_bytes(fmt, n);
    if (out_bytes < 0) return fail(MESH_ERR_INVALID, "mesh_act_pack: %lld elements is not a whole number of blocks", (long long)n);
    if (n == 0) return MESH_OK;
    DevScratch in, out;
    int rc;
    if ((rc = in.alloc((size_t)n * 4)) != MESH_OK || (rc = out.alloc((size_t)out_bytes)) != MESH_OK) return rc;
    MESH_HIP_TRY(hipMemcpy(in.p, src, (size_t)n * 4, hipMemcpyHostToDevice));
    if ((rc = act_pack_dev(fmt, static_cast<const float *>(in.p), out.p, n, nullptr)) != MESH_OK) return rc;
    MESH_HIP_TRY(hipMemcpy(dst, out.p, (size_t)out_bytes, hipMemcpyDeviceToHost));
    return MESH_OK;
}

int mesh_act_pack_noalloc(int fmt, const float *src, void *dst, int64_t n) {
    if (!is_act_fmt(fmt)) return fail(MESH_ERR_INVALID, "mesh_act_pack_noalloc: format %d is not an activation format", fmt);
    if (n < 0 || (n > 0 && (!src || !dst))) return fail(MESH_ERR_INVALID, "mesh_act_pack_noalloc: null pointer or negative count");
    const int64_t out_bytes = row_bytes(fmt, n);
    if (out_bytes < 0) return fail(MESH_ERR_INVALID, "mesh_act_pack_noalloc: %lld elements is not a whole number of blocks", (long long)n);
    if (n > NOALLOC_MAX_ELEMS)
        return fail(MESH_ERR_INVALID, "mesh_act_pack_noalloc: %lld elements exceed the fixed staging of %lld (use mesh_act_pack)", (long long)n,
                    (long long)NOALLOC_MAX_ELEMS);
    if (n == 0) return MESH_OK;
    std::lock_guard<std::mutex> lk(g_noalloc_mu);
    uint8_t *base = nullptr;
    int rc = noalloc_scratch(&base);
    if (rc != MESH_OK) return rc;
    float *d_in = reinterpret_cast<float *>(base);
    uint8_t *d_out = base + NOALLOC_OUT_OFFSET;
    MESH_HIP_TRY(hipMemcpy(d_in, src, (size_t)n * 4, hipMemcpyHostToDevice));
    if ((rc = act_pack_dev(fmt, d_in, d_out, n, nullptr)) != MESH_OK) return rc;
    MESH_HIP_TRY(hipMemcpy(dst, d_out, (size_t)out_bytes, hipMemcpyDeviceToHost));
    return MESH_OK;
}

int mesh_act_unpack(int fmt, const void *src, float *dst, int64_t n) {
    if (!is_act_fmt(fmt)) return fail(MESH_ERR_INVALID, "mesh_act_unpack: format %d is not an activation format", fmt);
    if (n < 0 || (n > 0 && (!src || !dst))) return fail(MESH_ERR_INVALID, "mesh_act_unpack: null pointer or negative count");
    const int64_t in_bytes = row_bytes(fmt, n);
    if (in_bytes < 0) return fail(MESH_ERR_INVALID, "mesh_act_unpack: %lld elements is not a whole number of blocks", (long long)n);
    if (n == 0) return MESH_OK;
    DevScratch in, out;
    int rc;
    if ((rc = in.alloc((size_t)in_bytes)) != MESH_OK || (rc = out.alloc((size_t)n * 4)) != MESH_OK) return rc;
    MESH_HIP_TRY(hipMemcpy(in.p, src, (size_t)in_bytes, hipMemcpyHostToDevice));
    if ((rc = act_unpack_dev(fmt, in.p, static_cast<float *>(out.p), n, nullptr)) != MESH_OK) return rc;
    MESH_HIP_TRY(hipMemcpy(dst, out.p, (size_t)n * 4, hipMemcpyDeviceToHost));
    return MESH_OK;
}

}  // extern "C"
