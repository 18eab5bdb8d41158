/*
 * mesh_oracle.c -- see mesh_oracle.h.  TEST INFRASTRUCTURE ONLY; PARITY UNPINNED against ggml
 * (no ggml source is reachable offline); pinned by tests/test_oracle_*.py.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (oracle/Makefile).  -ffp-contract=off
 * matters: the block formulas below are defined with separately rounded f32 multiplies and adds.
 */
#include "mesh_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 0;
void mo_set_threads(int n) { g_threads = n; }
int mo_get_threads(void) {
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}
#ifdef _OPENMP
#define MO_NT num_threads(mo_get_threads())
#endif

/* ------------------------------------------------------------------ fp16 */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE-754 binary32 -> binary16, round to nearest even; overflow -> inf; NaN -> sign|0x7E00.
 * Restates GGML_FP32_TO_FP16's portable result (ggml_fp32_to_fp16_row is what a boundary
 * f16 pack of patches/0002:544-622's tensor would call). */
uint16_t mo_fp32_to_fp16(float f) {
    const uint32_t w = f2u(f);
    const uint16_t sign = (uint16_t)((w >> 16) & 0x8000u);
    const uint32_t a = w & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);          /* NaN */
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);         /* >= 65520 -> inf */
    if (a < 0x38800000u) {                                           /* < 2^-14: half subnormal */
        if (a < 0x33000000u) return sign;                            /* < 2^-25 -> 0 */
        const uint32_t e = a >> 23;                                  /* 102..112 */
        const uint32_t mant = (a & 0x007FFFFFu) | 0x00800000u;
        const uint32_t shift = 126u - e;                             /* 14..24 */
        uint32_t q = mant >> shift;
        const uint32_t rem = mant & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t h = (((a >> 23) - 112u) << 10) | ((a & 0x007FFFFFu) >> 13);
    const uint32_t rem = a & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

float mo_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0x1Fu) return u2f(sign | 0x7F800000u | (m << 13));      /* inf / NaN */
    if (e == 0) {
        if (m == 0) return u2f(sign);
        int s = 0;                                                   /* normalise the subnormal */
        while (!(m & 0x400u)) { m <<= 1; s++; }
        m &= 0x3FFu;
        return u2f(sign | ((uint32_t)(113 - s) << 23) | (m << 13));
    }
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

void mo_fp32_to_fp16_row(const float *x, uint16_t *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = mo_fp32_to_fp16(x[i]);
}
void mo_fp16_to_fp32_row(const uint16_t *x, float *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = mo_fp16_to_fp32(x[i]);
}

/* ------------------------------------------------------------------ block formats */

#define QK8_0 32
#define QK5_0 32
#define QK4_0 32
#define Q4_0_BYTES 18
#define QK_K 256
#define Q8_0_BYTES 34
#define Q5_0_BYTES 22
#define Q4_K_BYTES 144
#define Q6_K_BYTES 210

int64_t mo_block_elems(int type) {
    switch (type) {
        case MO_F32: case MO_F16: return 1;
        case MO_Q4_0: case MO_Q5_0: case MO_Q8_0: return 32;
        case MO_Q4_K: case MO_Q6_K: return 256;
        default: return -1;
    }
}
int64_t mo_block_bytes(int type) {
    switch (type) {
        case MO_F32: return 4;
        case MO_F16: return 2;
        case MO_Q4_0: return Q4_0_BYTES;
        case MO_Q5_0: return Q5_0_BYTES;
        case MO_Q8_0: return Q8_0_BYTES;
        case MO_Q4_K: return Q4_K_BYTES;
        case MO_Q6_K: return Q6_K_BYTES;
        default: return -1;
    }
}
/* ggml_row_size / ggml_nbytes for a row of k elements (patches/0002:243 sizes transfers with it) */
int64_t mo_row_bytes(int type, int64_t k) {
    const int64_t be = mo_block_elems(type);
    if (be < 0 || k % be) return -1;
    return k / be * mo_block_bytes(type);
}

static inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* quantize_row_q8_0_ref: block = { fp16 d; int8 qs[32] }.  d = amax/127 (f32 divide),
 * id = 1/d computed from the UNROUNDED f32 d, q = roundf(x*id) (half away from zero). */
void mo_quantize_row_q8_0(const float *x, void *vy, int64_t k) {
    uint8_t *y = (uint8_t *)vy;
    const int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; j++) {
            const float v = fabsf(x[i * QK8_0 + j]);
            amax = amax > v ? amax : v;
        }
        const float d = amax / 127.0f;
        const float id = d ? 1.0f / d : 0.0f;
        const uint16_t dh = mo_fp32_to_fp16(d);
        uint8_t *b = y + i * Q8_0_BYTES;
        b[0] = (uint8_t)(dh & 0xFF);
        b[1] = (uint8_t)(dh >> 8);
        for (int j = 0; j < QK8_0; j++) {
            const float x0 = x[i * QK8_0 + j] * id;
            b[2 + j] = (uint8_t)(int8_t)roundf(x0);
        }
    }
}

/* quantize_row_q4_0_ref: block = { fp16 d; uint8 qs[16] }.  max = the element of largest magnitude (the first one on
 * ties), d = max / -8, id = 1/d from the unrounded d; q = min(15, (int8)(x*id + 8.5f)); byte j holds element j in
 * its low nibble and element j + 16 in its high nibble. */
void mo_quantize_row_q4_0(const float *x, void *vy, int64_t k) {
    uint8_t *y = (uint8_t *)vy;
    const int64_t nb = k / QK4_0;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < QK4_0; j++) {
            const float v = x[i * QK4_0 + j];
            if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
        }
        const float d = max / -8.0f;
        const float id = d ? 1.0f / d : 0.0f;
        const uint16_t dh = mo_fp32_to_fp16(d);
        uint8_t *b = y + i * Q4_0_BYTES;
        b[0] = (uint8_t)(dh & 0xFF);
        b[1] = (uint8_t)(dh >> 8);
        for (int j = 0; j < QK4_0 / 2; j++) {
            const float x0 = x[i * QK4_0 + j] * id, x1 = x[i * QK4_0 + QK4_0 / 2 + j] * id;
            int q0 = (int8_t)(x0 + 8.5f), q1 = (int8_t)(x1 + 8.5f);
            if (q0 > 15) q0 = 15;
            if (q1 > 15) q1 = 15;
            b[2 + j] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

/* dequantize_row_q4_0: y[j] = ((qs[j] & 0xF) - 8) * d, y[j + 16] = ((qs[j] >> 4) - 8) * d */
static void dequantize_row_q4_0(const uint8_t *x, float *y, int64_t k) {
    const int64_t nb = k / QK4_0;
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t *b = x + i * Q4_0_BYTES;
        const float d = mo_fp16_to_fp32(rd16(b));
        for (int j = 0; j < QK4_0 / 2; j++) {
            y[i * QK4_0 + j] = (float)((b[2 + j] & 0x0F) - 8) * d;
            y[i * QK4_0 + j + QK4_0 / 2] = (float)((b[2 + j] >> 4) - 8) * d;
        }
    }
}

static void dequantize_row_q8_0(const uint8_t *x, float *y, int64_t k) {
    const int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t *b = x + i * Q8_0_BYTES;
        const float d = mo_fp16_to_fp32(rd16(b));
        for (int j = 0; j < QK8_0; j++) y[i * QK8_0 + j] = (float)(int8_t)b[2 + j] * d;
    }
}

/* q5_0: { fp16 d; u8 qh[4]; u8 qs[16] } -- the fallback type of a Q4_K tensor whose row length is not
 * a multiple of 256 (config with hidden 896) */
static void dequantize_row_q5_0(const uint8_t *x, float *y, int64_t k) {
    const int64_t nb = k / QK5_0;
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t *b = x + i * Q5_0_BYTES;
        const float d = mo_fp16_to_fp32(rd16(b));
        const uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
        const uint8_t *qs = b + 6;
        for (int j = 0; j < 16; j++) {
            const uint8_t xh0 = (uint8_t)(((qh >> (j + 0)) << 4) & 0x10);
            const uint8_t xh1 = (uint8_t)((qh >> (j + 12)) & 0x10);
            const int32_t x0 = ((qs[j] & 0x0F) | xh0) - 16;
            const int32_t x1 = ((qs[j] >> 4) | xh1) - 16;
            y[i * QK5_0 + j] = (float)x0 * d;
            y[i * QK5_0 + j + 16] = (float)x1 * d;
        }
    }
}

/* 6-bit (scale, min) pair j of a q4_K super-block's 12 packed bytes */
static inline void get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* q4_K: { fp16 d; fp16 dmin; u8 scales[12]; u8 qs[128] }, 8 sub-blocks of 32:
 * y = (d*sc)*q - (dmin*m), every product and the subtraction rounded to f32 separately */
static void dequantize_row_q4_K(const uint8_t *x, float *y, int64_t k) {
    const int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t *b = x + i * Q4_K_BYTES;
        const float d = mo_fp16_to_fp32(rd16(b));
        const float dmin = mo_fp16_to_fp32(rd16(b + 2));
        const uint8_t *scales = b + 4;
        const uint8_t *q = b + 16;
        int is = 0;
        for (int c = 0; c < QK_K; c += 64) {
            uint8_t sc, m;
            get_scale_min_k4(is + 0, scales, &sc, &m);
            const float d1 = d * sc, m1 = dmin * m;
            get_scale_min_k4(is + 1, scales, &sc, &m);
            const float d2 = d * sc, m2 = dmin * m;
            for (int l = 0; l < 32; l++) *y++ = d1 * (float)(q[l] & 0xF) - m1;
            for (int l = 0; l < 32; l++) *y++ = d2 * (float)(q[l] >> 4) - m2;
            q += 32;
            is += 2;
        }
    }
}

/* q6_K: { u8 ql[128]; u8 qh[64]; i8 scales[16]; fp16 d }: y = d * sc * q, evaluated as (d*sc)*q */
static void dequantize_row_q6_K(const uint8_t *x, float *y, int64_t k) {
    const int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t *b = x + i * Q6_K_BYTES;
        const uint8_t *ql = b;
        const uint8_t *qh = b + 128;
        const int8_t *sc = (const int8_t *)(b + 192);
        const float d = mo_fp16_to_fp32(rd16(b + 208));
        for (int n = 0; n < QK_K; n += 128) {
            for (int l = 0; l < 32; l++) {
                const int is = l / 16;
                const int8_t q1 = (int8_t)((ql[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                const int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                const int8_t q3 = (int8_t)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                const int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l + 0] = d * sc[is + 0] * q1;
                y[l + 32] = d * sc[is + 2] * q2;
                y[l + 64] = d * sc[is + 4] * q3;
                y[l + 96] = d * sc[is + 6] * q4;
            }
            y += 128;
            ql += 64;
            qh += 32;
            sc += 8;
        }
    }
}

int mo_dequantize_row(int type, const void *vx, float *y, int64_t k) {
    if (mo_row_bytes(type, k) < 0) return -1;
    const uint8_t *x = (const uint8_t *)vx;
    switch (type) {
        case MO_F32: memcpy(y, x, (size_t)k * 4); return 0;
        case MO_F16: mo_fp16_to_fp32_row((const uint16_t *)vx, y, k); return 0;
        case MO_Q8_0: dequantize_row_q8_0(x, y, k); return 0;
        case MO_Q4_0: dequantize_row_q4_0(x, y, k); return 0;
        case MO_Q5_0: dequantize_row_q5_0(x, y, k); return 0;
        case MO_Q4_K: dequantize_row_q4_K(x, y, k); return 0;
        case MO_Q6_K: dequantize_row_q6_K(x, y, k); return 0;
        default: return -1;
    }
}

/* ------------------------------------------------------------------ operators */

/* mul_mat(W, x): the value ggml's kernels approximate -- dequant(W) . x with a float64 accumulator.
 * (ggml's CPU backend additionally rounds x to Q8_K/Q8_0 blocks before an integer dot; that rounding is
 * not restated, so stage-level parity is a tolerance, not bits.) */
int mo_mul_mat(int type, const void *W, int64_t M, int64_t K, const float *x, int64_t T,
               const float *bias, float *y) {
    const int64_t rb = mo_row_bytes(type, K);
    if (rb < 0) return -1;
    const uint8_t *w = (const uint8_t *)W;
#ifdef _OPENMP
#pragma omp parallel MO_NT
#endif
    {
        float *row = (float *)malloc((size_t)K * sizeof(float));
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
        for (int64_t m = 0; m < M; m++) {
            mo_dequantize_row(type, w + m * rb, row, K);
            for (int64_t t = 0; t < T; t++) {
                const float *xt = x + t * K;
                double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
                int64_t k = 0;
                for (; k + 4 <= K; k += 4) {
                    a0 += (double)row[k] * (double)xt[k];
                    a1 += (double)row[k + 1] * (double)xt[k + 1];
                    a2 += (double)row[k + 2] * (double)xt[k + 2];
                    a3 += (double)row[k + 3] * (double)xt[k + 3];
                }
                for (; k < K; k++) a0 += (double)row[k] * (double)xt[k];
                double acc = (a0 + a1) + (a2 + a3);
                if (bias) acc += (double)bias[m];
                y[t * M + m] = (float)acc;
            }
        }
        free(row);
    }
    return 0;
}

/* ggml rms_norm followed by ggml_mul with the norm weight: sum of squares in double,
 * scale = 1/sqrtf(mean+eps) in f32, y = (x*scale)*w */
void mo_rms_norm(const float *x, const float *w, float eps, int64_t n, int64_t T, float *y) {
    for (int64_t t = 0; t < T; t++) {
        const float *xt = x + t * n;
        double sum = 0.0;
        for (int64_t i = 0; i < n; i++) sum += (double)(xt[i] * xt[i]);
        const float mean = (float)(sum / (double)n);
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < n; i++) y[t * n + i] = (xt[i] * scale) * w[i];
    }
}

/* ggml rope, no frequency factors, freq_scale 1, ext_factor 0: theta_i starts at pos and is multiplied by
 * theta_scale = base^(-2/n_rot) per pair (f32 recurrence).  NORM pairs (2i,2i+1) -- llama; NEOX pairs
 * (i, i+n_rot/2) -- qwen2/qwen3. */
void mo_rope(float *x, int64_t T, int n_head, int head_dim, int n_rot, const int32_t *pos,
             float freq_base, int mode) {
    const float theta_scale = powf(freq_base, -2.0f / (float)n_rot);
    for (int64_t t = 0; t < T; t++) {
        for (int h = 0; h < n_head; h++) {
            float *v = x + (t * n_head + h) * head_dim;
            float theta = (float)pos[t];
            for (int i0 = 0; i0 < n_rot; i0 += 2) {
                const float c = cosf(theta), s = sinf(theta);
                theta *= theta_scale;
                const int ia = mode == MO_ROPE_NEOX ? i0 / 2 : i0;
                const int ib = mode == MO_ROPE_NEOX ? i0 / 2 + n_rot / 2 : i0 + 1;
                const float x0 = v[ia], x1 = v[ib];
                v[ia] = x0 * c - x1 * s;
                v[ib] = x0 * s + x1 * c;
            }
        }
    }
}

void mo_swiglu(const float *gate, const float *up, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        const float g = gate[i];
        out[i] = (g / (1.0f + expf(-g))) * up[i];
    }
}

/* softmax(q.K^T * scale) . V for one token, float64 throughout.  K/V are the cache contents as values: f16 bits
 * (kv_f32 = 0) or the f32 values a quantised cache dequantises to (kv_f32 = 1). */
static void attn_token(const float *q, const void *kcache, const void *vcache, int kv_f32, int n_head, int n_kv,
                       int head_dim, int64_t ctx_stride, int64_t n_past, float scale, float *out) {
    const int group = n_head / n_kv;
    const int64_t n = n_past + 1;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) MO_NT
#endif
    for (int h = 0; h < n_head; h++) {
        const int kvh = h / group;
        const int64_t off = (int64_t)kvh * ctx_stride * head_dim;
        const uint16_t *K16 = (const uint16_t *)kcache + off, *V16 = (const uint16_t *)vcache + off;
        const float *K32 = (const float *)kcache + off, *V32 = (const float *)vcache + off;
        const float *qh = q + (int64_t)h * head_dim;
        double *s = (double *)malloc((size_t)n * sizeof(double));
        double *acc = (double *)calloc((size_t)head_dim, sizeof(double));
        double mx = -INFINITY;
        for (int64_t j = 0; j < n; j++) {
            double d = 0.0;
            for (int i = 0; i < head_dim; i++)
                d += (double)qh[i] * (double)(kv_f32 ? K32[j * head_dim + i] : mo_fp16_to_fp32(K16[j * head_dim + i]));
            s[j] = d * (double)scale;
            if (s[j] > mx) mx = s[j];
        }
        double den = 0.0;
        for (int64_t j = 0; j < n; j++) { s[j] = exp(s[j] - mx); den += s[j]; }
        for (int64_t j = 0; j < n; j++) {
            const double p = s[j] / den;
            for (int i = 0; i < head_dim; i++)
                acc[i] += p * (double)(kv_f32 ? V32[j * head_dim + i] : mo_fp16_to_fp32(V16[j * head_dim + i]));
        }
        for (int i = 0; i < head_dim; i++) out[(int64_t)h * head_dim + i] = (float)acc[i];
        free(s);
        free(acc);
    }
}
void mo_attn_token(const float *q, const uint16_t *kcache, const uint16_t *vcache, int n_head, int n_kv,
                   int head_dim, int64_t ctx_stride, int64_t n_past, float scale, float *out) {
    attn_token(q, kcache, vcache, 0, n_head, n_kv, head_dim, ctx_stride, n_past, scale, out);
}
void mo_attn_token_f32(const float *q, const float *kcache, const float *vcache, int n_head, int n_kv,
                       int head_dim, int64_t ctx_stride, int64_t n_past, float scale, float *out) {
    attn_token(q, kcache, vcache, 1, n_head, n_kv, head_dim, ctx_stride, n_past, scale, out);
}

/* MoE gating as llama.cpp's build_moe_ffn runs it for softmax-gated models (qwen3moe), with the expert mask of
 * patches/0003:86-104: probs = softmax(logits) over every expert in the file; the 0 / -inf mask is ADDED to the
 * probabilities used for selection only (selection_probs); the weights are the unmasked probs of the selected
 * experts, divided by their sum when norm_w is set.  Ties go to the lower expert id. */
void mo_moe_route(const float *logits, const float *mask, int n_expert, int top_k, int norm_w,
                  int32_t *ids, float *weights) {
    double *p = (double *)malloc((size_t)n_expert * sizeof(double));
    double mx = -INFINITY;
    for (int e = 0; e < n_expert; e++) if ((double)logits[e] > mx) mx = (double)logits[e];
    double den = 0.0;
    for (int e = 0; e < n_expert; e++) { p[e] = exp((double)logits[e] - mx); den += p[e]; }
    for (int e = 0; e < n_expert; e++) p[e] /= den;
    double wsum = 0.0;
    for (int k = 0; k < top_k; k++) {
        int best = -1;
        double best_sel = 0.0;
        for (int e = 0; e < n_expert; e++) {
            int taken = 0;
            for (int j = 0; j < k; j++) taken |= (ids[j] == e);
            if (taken) continue;
            const double sel = p[e] + (mask ? (double)mask[e] : 0.0);
            if (best < 0 || sel > best_sel) { best = e; best_sel = sel; }
        }
        ids[k] = best;
        weights[k] = (float)p[best];
        wsum += p[best];
    }
    if (norm_w && wsum > 0.0)
        for (int k = 0; k < top_k; k++) weights[k] = (float)((double)weights[k] / wsum);
    free(p);
}
