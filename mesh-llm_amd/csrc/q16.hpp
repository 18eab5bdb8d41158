// Device-side writer of the "q16" activation layout of the skinny GEMM (gemm_skinny.hip): 16-bit fixed point per
// 32-element block as two int8 planes, with f32 block scales and block sums.
#pragma once

#include "gemv_device.hpp"

namespace mesh {

// Called by 32 consecutive lanes (an aligned half of a wave, all active) that hold the 32 elements kk .. kk + 31 of token
// tok's row of K elements, one each (kk: this lane's element): quantises the block exactly as quant16_k8 does and
// stores it.  q16: start of the activation buffer (blocks of 16 tokens, 36 K bytes each).
__device__ __forceinline__ void q16_store_block32(uint8_t *q16, int K, int tok, int kk, float v) {
    float amax = fabsf(v);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    const float inv = amax > 0.f ? XQ_LEVELS / amax : 0.f;
    const int q = __float2int_rn(v * inv);
    const int lo = ((q + 128) & 0xFF) - 128, hi = (q - lo) >> 8;
    int isum = q;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) isum += __shfl_xor(isum, o);
    uint8_t *yb = q16 + (size_t)(tok >> 4) * ((size_t)K * 36);
    const int t = tok & 15;
    uint8_t *rec = yb + ((size_t)(kk >> 3) * 16 + t) * 16 + (kk & 7);
    rec[0] = (uint8_t)hi;
    rec[8] = (uint8_t)lo;
    if ((kk & 31) == 0) {
        const float d = amax / XQ_LEVELS;
        reinterpret_cast<float *>(yb + (size_t)K * 32)[(kk >> 5) * 16 + t] = d;
        reinterpret_cast<float *>(yb + (size_t)K * 34)[(kk >> 5) * 16 + t] = d * (float)isum;
    }
}

}  // namespace mesh
