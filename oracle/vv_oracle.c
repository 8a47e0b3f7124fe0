/*
 * vv_oracle.c — CPU restatement of vibevoice.c's src/cpu layer kernels.
 *
 * TEST INFRASTRUCTURE ONLY (see vv_oracle.h). Build with
 *   gcc -O2 -fopenmp -ffp-contract=off -fPIC -shared vv_oracle.c -lm
 * No -ffast-math, no -march: the reference builds src/cpu/cpu_kernels.c with
 * plain -O3 (CMakeLists.txt:111-128), so products and sums are unfused and in
 * source order, and libm's powf/cosf/sinf/expf/sqrtf are the scalar glibc
 * ones. Keeping that here is what makes the low bits reproducible.
 */
#include "vv_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { VVO_OK = 0, VVO_ERR_INVALID_ARG = -1, VVO_ERR_NULL_PTR = -2 };   /* types.h:19-23 */

/* ── FP16 conversions ─────────────────────────────────────────────────── */

float vvo_half_to_float(uint16_t h) {
    /* types.h:107-129: exact widening. Written here as three value classes:
     * inf/NaN keep the payload, subnormals are an integer times 2^-24, and
     * normals shift the exponent bias from 15 to 127. */
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t mag = h & 0x7FFFu;
    union { uint32_t u; float f; } v;
    if (mag >= 0x7C00u) {
        v.u = sign | 0x7F800000u | ((mag & 0x3FFu) << 13);
    } else if (mag < 0x0400u) {
        v.f = (float)mag * 0x1p-24f;          /* exact: mag < 2^10 */
        v.u |= sign;
    } else {
        v.u = sign | ((mag << 13) + (112u << 23));
    }
    return v.f;
}

uint16_t vvo_float_to_half_rne(float f) {
    /* types.h:171-196: round-to-nearest-even. The subnormal range is rounded
     * by the FPU itself (adding 0.5f leaves round(|f| * 2^24) in the low
     * mantissa bits under the default rounding mode); normals add the
     * classic 0xFFF + lsb bias before dropping 13 bits. */
    union { float f; uint32_t u; } v;
    v.f = f;
    const uint16_t sign = (uint16_t)((v.u >> 16) & 0x8000u);
    uint32_t a = v.u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);       /* NaN */
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);      /* -> inf */
    if (a < 0x38800000u) {                                        /* < 2^-14 */
        union { float f; uint32_t u; } t;
        v.u = a;
        t.f = v.f + 0.5f;
        return (uint16_t)(sign | (t.u - 0x3F000000u));
    }
    a += 0xC8000000u + 0xFFFu + ((a >> 13) & 1u);   /* rebias 127 -> 15 */
    return (uint16_t)(sign | (a >> 13));
}

void vvo_widen_f16(const uint16_t* in, float* out, size_t n) {
    long i;
#pragma omp parallel for schedule(static)
    for (i = 0; i < (long)n; i++) out[i] = vvo_half_to_float(in[i]);
}

void vvo_narrow_f32_rne(const float* in, uint16_t* out, size_t n) {
    long i;
#pragma omp parallel for schedule(static)
    for (i = 0; i < (long)n; i++) out[i] = vvo_float_to_half_rne(in[i]);
}

/* ── the five reference kernels, FP32 activations ─────────────────────── */

int vvo_rmsnorm_f32(const float* input, const uint16_t* weight_f16,
                    float* output, int rows, int n, float eps) {
    /* cpu_kernels.c:1432-1451. Per row: double sum of squares in index
     * order, one float reciprocal square root, then (x * inv) * w. */
    if (!input || !weight_f16 || !output) return VVO_ERR_NULL_PTR;
    int r;
#pragma omp parallel for schedule(static)
    for (r = 0; r < rows; r++) {
        const float* x = input + (size_t)r * n;
        float* y = output + (size_t)r * n;
        double sumsq = 0.0;
        for (int i = 0; i < n; i++) {
            const double xi = (double)x[i];
            sumsq += xi * xi;
        }
        const float mean = (float)(sumsq / n);
        const float inv = 1.0f / sqrtf(mean + eps);
        for (int i = 0; i < n; i++) {
            const float scaled = x[i] * inv;
            y[i] = scaled * vvo_half_to_float(weight_f16[i]);
        }
    }
    return VVO_OK;
}

int vvo_rope_f32(float* x, int rows, int n_heads, int head_dim,
                 int position_offset, float theta) {
    /* cpu_kernels.c:1453-1478. Rotate-half pairing (i, i + head_dim/2); the
     * frequency, angle, cosine and sine are all float, recomputed per head
     * exactly as the reference does (same libm calls, same arguments). */
    if (!x) return VVO_ERR_NULL_PTR;
    const int half = head_dim / 2;
    int r;
#pragma omp parallel for schedule(static)
    for (r = 0; r < rows; r++) {
        const int pos = position_offset + r;
        for (int h = 0; h < n_heads; h++) {
            float* v = x + ((size_t)r * n_heads + h) * head_dim;
            for (int i = 0; i < half; i++) {
                const float expo = -2.0f * (float)i / (float)head_dim;
                const float freq = powf(theta, expo);
                const float ang = (float)pos * freq;
                const float c = cosf(ang);
                const float s = sinf(ang);
                const float a = v[i];
                const float b = v[i + half];
                const float ac = a * c, bs = b * s;
                const float as = a * s, bc = b * c;
                v[i] = ac - bs;
                v[i + half] = as + bc;
            }
        }
    }
    return VVO_OK;
}

int vvo_swiglu_f32(const float* gate, const float* up, float* output, int n) {
    /* cpu_kernels.c:1536-1548: (g / (1 + expf(-g))) * u. Safe for
     * output == gate: element i is read before it is written. */
    if (!gate || !up || !output) return VVO_ERR_NULL_PTR;
    int i;
#pragma omp parallel for schedule(static)
    for (i = 0; i < n; i++) {
        const float g = gate[i];
        const float denom = 1.0f + expf(-g);
        const float silu = g / denom;
        output[i] = silu * up[i];
    }
    return VVO_OK;
}

int vvo_residual_add_f32(float* x, const float* y, int n) {
    /* cpu_kernels.c:1550-1558 */
    if (!x || !y) return VVO_ERR_NULL_PTR;
    int i;
#pragma omp parallel for schedule(static)
    for (i = 0; i < n; i++) x[i] = x[i] + y[i];
    return VVO_OK;
}

int vvo_embedding_f32(const uint16_t* table_f16, const int32_t* ids,
                      float* output, int rows, int hidden) {
    /* cpu_kernels.c:1560-1568: single-threaded row copy, widened to FP32
     * (f16_row, :587-596). Row offsets are size_t; ids are not checked. */
    if (!table_f16 || !ids || !output) return VVO_ERR_NULL_PTR;
    for (int r = 0; r < rows; r++) {
        const uint16_t* src = table_f16 + (size_t)ids[r] * (size_t)hidden;
        float* dst = output + (size_t)r * (size_t)hidden;
        for (int i = 0; i < hidden; i++) dst[i] = vvo_half_to_float(src[i]);
    }
    return VVO_OK;
}

/* ── device-contract forms ─────────────────────────────────────────────── */

static void emit(const float* src, float* out_ref, uint16_t* out_rne, size_t n) {
    if (out_ref && out_ref != src) memcpy(out_ref, src, n * sizeof(float));
    if (out_rne) vvo_narrow_f32_rne(src, out_rne, n);
}

int vvo_rmsnorm_f16(const uint16_t* x, const uint16_t* w, float* out_ref,
                    uint16_t* out_rne, int rows, int n, float eps) {
    if (!x || !w) return VVO_ERR_NULL_PTR;
    const size_t total = (size_t)rows * (size_t)n;
    float* xin = (float*)malloc((total ? total : 1) * sizeof(float));
    float* y = (float*)malloc((total ? total : 1) * sizeof(float));
    if (!xin || !y) { free(xin); free(y); return -3; }
    vvo_widen_f16(x, xin, total);
    const int st = vvo_rmsnorm_f32(xin, w, y, rows, n, eps);
    if (st == VVO_OK) emit(y, out_ref, out_rne, total);
    free(xin); free(y);
    return st;
}

int vvo_residual_add_f16(uint16_t* x, const uint16_t* y, size_t n) {
    if (!x || !y) return VVO_ERR_NULL_PTR;
    long i;
#pragma omp parallel for schedule(static)
    for (i = 0; i < (long)n; i++) {
        float a = vvo_half_to_float(x[i]);
        const float b = vvo_half_to_float(y[i]);
        /* the same FP32 add vvo_residual_add_f32 does, then one RNE round */
        a = a + b;
        x[i] = vvo_float_to_half_rne(a);
    }
    return VVO_OK;
}

int vvo_add_rmsnorm_f16(uint16_t* residual, const uint16_t* x,
                        const uint16_t* w, float* normed_ref,
                        uint16_t* normed_rne, int rows, int n, float eps) {
    if (!residual || !x || !w) return VVO_ERR_NULL_PTR;
    const int st = vvo_residual_add_f16(residual, x, (size_t)rows * (size_t)n);
    if (st != VVO_OK) return st;
    return vvo_rmsnorm_f16(residual, w, normed_ref, normed_rne, rows, n, eps);
}

int vvo_rope_f16(const uint16_t* x, float* out_ref, uint16_t* out_rne,
                 int rows, int n_heads, int head_dim, int position_offset,
                 float theta) {
    if (!x) return VVO_ERR_NULL_PTR;
    const size_t total = (size_t)rows * (size_t)n_heads * (size_t)head_dim;
    float* v = (float*)malloc((total ? total : 1) * sizeof(float));
    if (!v) return -3;
    vvo_widen_f16(x, v, total);
    const int st = vvo_rope_f32(v, rows, n_heads, head_dim, position_offset, theta);
    if (st == VVO_OK) emit(v, out_ref, out_rne, total);
    free(v);
    return st;
}

int vvo_swiglu_f16(const uint16_t* gate, const uint16_t* up, float* out_ref,
                   uint16_t* out_rne, size_t n) {
    if (!gate || !up) return VVO_ERR_NULL_PTR;
    /* chunked so that n beyond INT_MAX never reaches the int-sized kernel */
    const size_t chunk = (size_t)1 << 22;
    float* g = (float*)malloc(chunk * sizeof(float));
    float* u = (float*)malloc(chunk * sizeof(float));
    if (!g || !u) { free(g); free(u); return -3; }
    for (size_t off = 0; off < n; off += chunk) {
        const size_t m = n - off < chunk ? n - off : chunk;
        vvo_widen_f16(gate + off, g, m);
        vvo_widen_f16(up + off, u, m);
        vvo_swiglu_f32(g, u, g, (int)m);        /* in place, as decoder.c:1473 */
        emit(g, out_ref ? out_ref + off : NULL, out_rne ? out_rne + off : NULL, m);
    }
    free(g); free(u);
    return VVO_OK;
}

int vvo_swiglu_fused_f16(const uint16_t* gate_up, float* out_ref,
                         uint16_t* out_rne, int rows, int inter) {
    if (!gate_up) return VVO_ERR_NULL_PTR;
    for (int r = 0; r < rows; r++) {
        const uint16_t* g = gate_up + (size_t)r * 2u * (size_t)inter;
        const size_t o = (size_t)r * (size_t)inter;
        const int st = vvo_swiglu_f16(g, g + inter, out_ref ? out_ref + o : NULL,
                                      out_rne ? out_rne + o : NULL, (size_t)inter);
        if (st != VVO_OK) return st;
    }
    return VVO_OK;
}

int vvo_embedding_f16(const uint16_t* table, const int32_t* ids,
                      uint16_t* out, int rows, int hidden) {
    if (!table || !ids || !out) return VVO_ERR_NULL_PTR;
    for (int r = 0; r < rows; r++)
        memcpy(out + (size_t)r * (size_t)hidden,
               table + (size_t)ids[r] * (size_t)hidden,
               (size_t)hidden * sizeof(uint16_t));
    return VVO_OK;
}

int vvo_bias_add_f16(uint16_t* out, const uint16_t* bias, int M, int N) {
    if (!out || !bias) return VVO_ERR_NULL_PTR;
    int m;
#pragma omp parallel for schedule(static)
    for (m = 0; m < M; m++) {
        uint16_t* row = out + (size_t)m * (size_t)N;
        for (int j = 0; j < N; j++) {
            const float v = vvo_half_to_float(row[j]) + vvo_half_to_float(bias[j]);
            row[j] = vvo_float_to_half_rne(v);
        }
    }
    return VVO_OK;
}

/* ── per-token int8 activation quantiser ──────────────────────────────── */

int vvo_q8_pos(int layout, int j) {
    /* q8.h:56-66. The W4 layouts mirror a 16-byte chunk of packed 4-bit
     * weights: column j lives in 32-bit word (j/2)%4 at nibble slot
     * j/8 + 4*(j%2). */
    const int odd = j & 1, word = (j >> 1) & 3, slot = (j >> 3) + 4 * odd;
    if (layout == 1) return odd ? 16 + (j >> 1) : (j >> 1);
    if (layout == 2) return 8 * word + 4 * (slot & 1) + (slot >> 1);
    if (layout == 3) return 16 * odd + 4 * word + (slot & 3);
    return j;
}

int vvo_quant_act_q8(const float* x, int M, int K, int layout, int8_t* xq,
                     float* sx, int32_t* xsum) {
    /* cpu_int8.c:158-196. All FP32: one division for the scale, one for its
     * reciprocal, one multiply and one round-half-even per element. */
    if (!x || !xq || !sx) return VVO_ERR_NULL_PTR;
    if (M <= 0 || K <= 0 || (K % 32) != 0) return -1;
    if (layout < 0 || layout > 3) return -1;
    int where[32];
    for (int j = 0; j < 32; j++) where[j] = vvo_q8_pos(layout, j);
    int m;
#pragma omp parallel for schedule(static) if (M > 4)
    for (m = 0; m < M; m++) {
        const float* row = x + (size_t)m * K;
        int8_t* out = xq + (size_t)m * K;
        float amax = 0.0f;
        for (int k = 0; k < K; k++) {
            const float a = fabsf(row[k]);
            if (a > amax) amax = a;
        }
        const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
        sx[m] = amax / 127.0f;
        for (int run = 0; run < K / 32; run++) {
            int total = 0;
            for (int j = 0; j < 32; j++) {
                const float scaled = row[run * 32 + j] * inv;
                float r = rintf(scaled);
                if (r > 127.0f) r = 127.0f;
                if (r < -127.0f) r = -127.0f;
                const int q = (int)r;
                total += q;
                out[run * 32 + where[j]] = (int8_t)q;
            }
            if (xsum) xsum[(size_t)m * (K / 32) + run] = total;
        }
    }
    return VVO_OK;
}

/* ── the layer's two contractions ─────────────────────────────────────── */

int vvo_gemm_f16w(const float* x, const uint16_t* w, const uint16_t* bias,
                  float* out, int M, int N, int K) {
    if (!x || !w || !out) return VVO_ERR_NULL_PTR;
    int n;
#pragma omp parallel for schedule(static)
    for (n = 0; n < N; n++) {
        const uint16_t* wr = w + (size_t)n * K;
        const float b = bias ? vvo_half_to_float(bias[n]) : 0.0f;
        for (int m = 0; m < M; m++) {
            const float* xr = x + (size_t)m * K;
            double acc = 0.0;
            for (int k = 0; k < K; k++) acc += (double)xr[k] * (double)vvo_half_to_float(wr[k]);
            out[(size_t)m * N + n] = (float)acc + b;
        }
    }
    return VVO_OK;
}

int vvo_attention_prefill_f32(const float* q, const float* k, const float* v,
                              float* out, int n_q_heads, int n_kv_heads,
                              int head_dim, int rows, int q_offset, int kv_len,
                              int causal) {
    /* cpu_kernels.c:1480-1525. Per (row, head): running maximum m, running
     * denominator l, output rescaled by expf(m_old - m_new) at every key. */
    if (!q || !k || !v || !out) return VVO_ERR_NULL_PTR;
    const int group = n_q_heads / n_kv_heads;
    const size_t q_stride = (size_t)n_q_heads * head_dim;
    const size_t kv_stride = (size_t)n_kv_heads * head_dim;
    const float scale = 1.0f / sqrtf((float)head_dim);
    int r;
#pragma omp parallel for schedule(static)
    for (r = 0; r < rows; r++) {
        for (int h = 0; h < n_q_heads; h++) {
            const int kvh = h / group;
            const int q_abs = q_offset + r;
            int limit = kv_len;
            if (causal && q_abs + 1 < kv_len) limit = q_abs + 1;
            const float* qv = q + (size_t)r * q_stride + (size_t)h * head_dim;
            float* ov = out + (size_t)r * q_stride + (size_t)h * head_dim;
            float m_run = -INFINITY, l_run = 0.0f;
            for (int d = 0; d < head_dim; d++) ov[d] = 0.0f;
            for (int t = 0; t < limit; t++) {
                const float* kt = k + (size_t)t * kv_stride + (size_t)kvh * head_dim;
                const float* vt = v + (size_t)t * kv_stride + (size_t)kvh * head_dim;
                float dot = 0.0f;
                for (int d = 0; d < head_dim; d++) dot += qv[d] * kt[d];
                const float sc = dot * scale;
                const float m_new = sc > m_run ? sc : m_run;
                const float a = (m_run == -INFINITY) ? 0.0f : expf(m_run - m_new);
                const float p = expf(sc - m_new);
                for (int d = 0; d < head_dim; d++) ov[d] = ov[d] * a + p * vt[d];
                l_run = l_run * a + p;
                m_run = m_new;
            }
            const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
            for (int d = 0; d < head_dim; d++) ov[d] *= inv;
        }
    }
    return VVO_OK;
}

int vvo_w8a8_linear(const int8_t* xq, const float* sx, const int8_t* w, const float* sw,
                    const uint16_t* bias16, const uint16_t* res16, float* out_f32,
                    uint16_t* out_f16, int M, int N, int K) {
    if (!xq || !sx || !w || !sw) return VVO_ERR_NULL_PTR;
    int n;
#pragma omp parallel for schedule(static)
    for (n = 0; n < N; n++) {
        const int8_t* wr = w + (size_t)n * K;
        for (int m = 0; m < M; m++) {
            const int8_t* xr = xq + (size_t)m * K;
            int32_t t = 0;
            for (int k = 0; k < K; k++) t += (int32_t)xr[k] * (int32_t)wr[k];
            float v = (float)t * sx[m] * sw[n];
            if (bias16) v += vvo_half_to_float(bias16[n]);
            if (res16) v += vvo_half_to_float(res16[(size_t)m * N + n]);
            if (out_f32) out_f32[(size_t)m * N + n] = v;
            if (out_f16) out_f16[(size_t)m * N + n] = vvo_float_to_half_rne(v);
        }
    }
    return VVO_OK;
}

int vvo_w4a8_linear(const int8_t* xq, const float* sx, const uint8_t* packed,
                    const uint16_t* scales16, const uint8_t* zeros, int G,
                    const uint16_t* bias16, const uint16_t* res16, float* out_f32,
                    uint16_t* out_f16, int M, int N, int K) {
    if (!xq || !sx || !packed || !scales16 || !zeros) return VVO_ERR_NULL_PTR;
    if (G <= 0 || (G % 32) != 0 || (K % G) != 0) return VVO_ERR_INVALID_ARG;
    const int ng = K / G;
    int n;
#pragma omp parallel for schedule(static)
    for (n = 0; n < N; n++) {
        const uint8_t* wr = packed + (size_t)n * (K / 2);
        for (int m = 0; m < M; m++) {
            const int8_t* xr = xq + (size_t)m * K;
            float acc = 0.0f;
            for (int g = 0; g < ng; g++) {
                int32_t dot = 0, xs = 0;
                for (int k = g * G; k < (g + 1) * G; k++) {
                    const uint8_t b = wr[k / 2];
                    const int q = (k & 1) ? (b & 15) : (b >> 4);
                    dot += q * (int32_t)xr[k];
                    xs += xr[k];
                }
                const float s = vvo_half_to_float(scales16[(size_t)n * ng + g]);
                acc += s * (float)(dot - (int32_t)zeros[(size_t)n * ng + g] * xs);
            }
            float v = acc * sx[m];
            if (bias16) v += vvo_half_to_float(bias16[n]);
            if (res16) v += vvo_half_to_float(res16[(size_t)m * N + n]);
            if (out_f32) out_f32[(size_t)m * N + n] = v;
            if (out_f16) out_f16[(size_t)m * N + n] = vvo_float_to_half_rne(v);
        }
    }
    return VVO_OK;
}

int vvo_int4g_dequant_f16(const uint8_t* packed, const uint16_t* scales16, const uint8_t* zeros,
                          int N, int K, int G, uint16_t* out16) {
    if (!packed || !scales16 || !zeros || !out16) return VVO_ERR_NULL_PTR;
    if (N <= 0 || K <= 0 || G <= 0 || (K % G) != 0 || (K % 2) != 0) return VVO_ERR_INVALID_ARG;
    const int ng = K / G;
    for (int n = 0; n < N; n++)
        for (int k = 0; k < K; k++) {
            const uint8_t b = packed[(size_t)n * (K / 2) + k / 2];
            const int q = (k & 1) ? (b & 15) : (b >> 4);
            const size_t g = (size_t)n * ng + k / G;
            /* q - z is an exact small integer, the scale an FP16 value: the FP32 product is exact,
               so this is one rounding of the true product to FP16 */
            const float w = (float)(q - (int)zeros[g]) * vvo_half_to_float(scales16[g]);
            out16[(size_t)n * K + k] = vvo_float_to_half_rne(w);
        }
    return VVO_OK;
}

/* ── the older weight-only formats on FP16 activations ───────────────────── */

/* bitsandbytes' NF4 code book (dequant_nf4.cu:17-22, cpu_kernels.c:61-66). */
static const float kNf4[16] = {
    -1.0f,                 -0.6961928009986877f,  -0.5250730514526367f,  -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f,  0.16093020141124725f,  0.24611230194568634f,  0.33791524171829224f,
    0.44070982933044434f,  0.5626170039176941f,   0.7229568362236023f,   1.0f};

/* dequant_nf4.cu:40-66: element e of the flat weight is code book[nibble] times the
 * FP16 absmax of its block of 64, the high nibble of a byte being the even element. */
int vvo_nf4_dequant(const uint8_t* packed, const uint16_t* scales16, size_t n_elements, uint16_t* out16,
                    float* out32) {
    if (!packed || !scales16) return VVO_ERR_NULL_PTR;
    if ((n_elements & 7) != 0) return VVO_ERR_INVALID_ARG;
    for (size_t e = 0; e < n_elements; e++) {
        const uint8_t b = packed[e / 2];
        const float w = kNf4[(e & 1) ? (b & 15) : (b >> 4)] * vvo_half_to_float(scales16[e >> 6]);
        if (out32) out32[e] = w;
        if (out16) out16[e] = vvo_float_to_half_rne(w);
    }
    return VVO_OK;
}

/* awq_gemv.cu:125-153: w = q * scale + min per group of G along K, one rounding
 * in FP32 (q * scale is exact there), then one to FP16. */
int vvo_awq_dequant(const uint8_t* packed, const uint16_t* scales16, const uint16_t* mins16, int N, int K,
                    int G, uint16_t* out16, float* out32) {
    if (!packed || !scales16 || !mins16) return VVO_ERR_NULL_PTR;
    if (N <= 0 || K <= 0 || G <= 0 || (K % G) != 0 || (K % 8) != 0) return VVO_ERR_INVALID_ARG;
    const int ng = K / G;
    for (int n = 0; n < N; n++)
        for (int k = 0; k < K; k++) {
            const uint8_t b = packed[(size_t)n * (K / 2) + k / 2];
            const float q = (float)((k & 1) ? (b & 15) : (b >> 4));
            const size_t g = (size_t)n * ng + k / G;
            const float w = fmaf(q, vvo_half_to_float(scales16[g]), vvo_half_to_float(mins16[g]));
            if (out32) out32[(size_t)n * K + k] = w;
            if (out16) out16[(size_t)n * K + k] = vvo_float_to_half_rne(w);
        }
    return VVO_OK;
}

/* int8_gemv.cu:139-160: w = q * scale[row], the FP32 product rounded to FP16. */
int vvo_int8_dequant(const int8_t* q, const float* scales, int N, int K, uint16_t* out16, float* out32) {
    if (!q || !scales) return VVO_ERR_NULL_PTR;
    if (N <= 0 || K <= 0) return VVO_ERR_INVALID_ARG;
    for (int n = 0; n < N; n++)
        for (int k = 0; k < K; k++) {
            const float w = (float)q[(size_t)n * K + k] * scales[n];
            if (out32) out32[(size_t)n * K + k] = w;
            if (out16) out16[(size_t)n * K + k] = vvo_float_to_half_rne(w);
        }
    return VVO_OK;
}

int vvo_int4g_to_gpu_layout(uint8_t* packed, const uint16_t* scales16, const uint8_t* zeros,
                            int N, int K, int G, uint16_t* out_sz) {
    if (!packed || !scales16 || !zeros || !out_sz) return VVO_ERR_NULL_PTR;
    if (N <= 0 || K <= 0 || (K % 32) != 0 || G < 32 || (G % 32) != 0 || (K % G) != 0)
        return VVO_ERR_INVALID_ARG;
    const int ng = K / G;
    for (int n = 0; n < N; n++) {
        for (int c = 0; c < K / 32; c++) {
            uint8_t* chunk = packed + (size_t)n * (K / 2) + (size_t)c * 16;
            uint8_t code[32];                       /* code[j]: column 32c + j */
            for (int j = 0; j < 32; j++)
                code[j] = (j & 1) ? (uint8_t)(chunk[j / 2] & 15) : (uint8_t)(chunk[j / 2] >> 4);
            for (int t = 0; t < 4; t++) {
                uint32_t word = 0;
                /* slot s of word t: column 2 (t + 4 (s % 4)) + s / 4 */
                for (int slot = 0; slot < 8; slot++)
                    word |= (uint32_t)code[2 * (t + 4 * (slot & 3)) + (slot >> 2)] << (4 * slot);
                for (int b = 0; b < 4; b++) chunk[4 * t + b] = (uint8_t)(word >> (8 * b));
            }
        }
        for (int g = 0; g < ng; g++) {
            out_sz[((size_t)n * ng + g) * 2] = scales16[(size_t)n * ng + g];
            out_sz[((size_t)n * ng + g) * 2 + 1] =
                vvo_float_to_half_rne((float)zeros[(size_t)n * ng + g]);
        }
    }
    return VVO_OK;
}

/* ── FP8 KV-cache codec (src/cuda/kv_codec.cuh:66-128, emulated in integer arithmetic) ── */

static uint32_t f32_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }
static float bits_f32(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }

/* One value to E4M3 (bias 7, 3 mantissa bits, no infinities, largest finite
 * 448 = 0x7E) or E5M2 (bias 15, 2 mantissa bits, largest finite 57344 = 0x7B):
 * zero and NaN give a signed zero; magnitudes from the half-way point above the
 * largest finite value saturate to it; below the smallest normal the value is
 * a count of subnormal steps rounded half up; else round to nearest even on
 * the FP32 mantissa with the carry going into the exponent. */
static uint8_t fp8_encode_one(float f, int e5m2) {
    const int mant_bits = e5m2 ? 2 : 3, bias = e5m2 ? 15 : 7, drop = 23 - mant_bits;
    const int min_exp = 1 - bias;                       /* exponent of the smallest normal */
    const uint32_t max_code = e5m2 ? 0x7Bu : 0x7Eu;
    const float saturate_from = e5m2 ? 61440.0f : 464.0f;
    const int max_exp = e5m2 ? 15 : 8;
    const uint32_t b = f32_bits(f);
    const uint32_t sign = (b >> 24) & 0x80u;
    const float a = fabsf(f);
    if (!(a > 0.0f)) return (uint8_t)sign;
    if (a >= saturate_from) return (uint8_t)(sign | max_code);
    int e = (int)((b >> 23) & 0xFFu) - 127;
    if (e < min_exp) {
        const float steps = e5m2 ? 65536.0f : 512.0f;   /* 1 / (subnormal step) */
        int q = (int)(a * steps + 0.5f);
        const int top = 1 << mant_bits;                 /* rolls into the smallest normal */
        if (q > top) q = top;
        return (uint8_t)(sign | (uint32_t)q);
    }
    const uint32_t m = b & 0x7FFFFFu;
    uint32_t mm = m >> drop;
    const uint32_t rem = m & ((1u << drop) - 1u), half_way = 1u << (drop - 1);
    if (rem > half_way || (rem == half_way && (mm & 1u))) {
        if (++mm == (1u << mant_bits)) { mm = 0; ++e; }
    }
    if (e > max_exp) return (uint8_t)(sign | max_code);
    return (uint8_t)(sign | ((uint32_t)(e + bias) << mant_bits) | mm);
}

static float fp8_decode_one(uint8_t v, int e5m2) {
    const int mant_bits = e5m2 ? 2 : 3, bias = e5m2 ? 15 : 7;
    const uint32_t e = (v >> mant_bits) & (e5m2 ? 0x1Fu : 0xFu);
    const uint32_t m = v & ((1u << mant_bits) - 1u);
    const float r = e == 0u ? (float)m * (e5m2 ? 1.52587890625e-05f : 0.001953125f)
                            : bits_f32(((e + 127u - (uint32_t)bias) << 23) | (m << (23 - mant_bits)));
    return (v & 0x80u) ? -r : r;
}

int vvo_fp8_encode(const float* x, int n, int e5m2, uint8_t* out) {
    if (!x || !out) return VVO_ERR_NULL_PTR;
    for (int i = 0; i < n; i++) out[i] = fp8_encode_one(x[i], e5m2);
    return VVO_OK;
}

int vvo_fp8_decode(const uint8_t* codes, int n, int e5m2, float* out) {
    if (!codes || !out) return VVO_ERR_NULL_PTR;
    for (int i = 0; i < n; i++) out[i] = fp8_decode_one(codes[i], e5m2);
    return VVO_OK;
}

int vvo_kv_build_ref(const uint16_t* k16, int n_pos, int n_kv_heads, int head_dim, uint16_t* ref16) {
    if (!k16 || !ref16) return VVO_ERR_NULL_PTR;
    if (n_pos <= 0) return VVO_ERR_INVALID_ARG;
    for (int h = 0; h < n_kv_heads; h++)
        for (int d = 0; d < head_dim; d++) {
            float acc = 0.0f;
            for (int p = 0; p < n_pos; p++)
                acc += vvo_half_to_float(k16[((size_t)p * n_kv_heads + h) * head_dim + d]);
            ref16[(size_t)h * head_dim + d] = vvo_float_to_half_rne(acc / (float)n_pos);
        }
    return VVO_OK;
}

int vvo_kv_store_fp8(const uint16_t* src16, const uint16_t* ref16, int n_pos, int n_kv_heads,
                     int head_dim, int e5m2, uint8_t* store) {
    if (!src16 || !store) return VVO_ERR_NULL_PTR;
    for (int p = 0; p < n_pos; p++)
        for (int h = 0; h < n_kv_heads; h++)
            for (int d = 0; d < head_dim; d++) {
                const size_t i = ((size_t)p * n_kv_heads + h) * head_dim + d;
                float v = vvo_half_to_float(src16[i]);
                if (ref16) v -= vvo_half_to_float(ref16[(size_t)h * head_dim + d]);
                store[i] = fp8_encode_one(v, e5m2);
            }
    return VVO_OK;
}

/* ── TurboQuant KV-cache codec (src/cuda/kv_codec.cuh:38-62, 130-165, 180-285; kv_quant.cu:86-119) ── */

/* Lloyd-Max levels of a unit Gaussian (kv_codec.cuh:43-62). */
static const float kLev4[16] = {-2.725112f, -2.065280f, -1.613787f, -1.251845f, -0.938657f, -0.654379f,
                                -0.386970f, -0.127960f, +0.127960f, +0.386970f, +0.654379f, +0.938657f,
                                +1.251845f, +1.613787f, +2.065280f, +2.725112f};
static const float kLev3[8] = {-2.150300f, -1.343258f, -0.755588f, -0.244756f,
                               +0.244756f, +0.755588f, +1.343258f, +2.150300f};
static const float kLev2[4] = {-1.511418f, -0.452456f, +0.452456f, +1.511418f};
static const float kVq15[16] = {-1.500251f, +0.674678f, -1.127883f, -0.787015f, -0.283251f, +0.390133f,
                                -0.103102f, +1.624620f, +0.100120f, -1.618563f, +0.286482f, -0.379555f,
                                +1.134227f, +0.790368f, +1.496572f, -0.666578f};
#define VVO_WHT_NORM 0.0883883476f      /* 1 / sqrt(128) */

enum { VVO_KV_TQ4 = 3, VVO_KV_TQ3 = 4, VVO_KV_TQ2 = 5, VVO_KV_TQ1_5 = 6 };

static int tq_lane_bits(int fmt) { return fmt == VVO_KV_TQ4 ? 16 : fmt == VVO_KV_TQ3 ? 12 : fmt == VVO_KV_TQ2 ? 8 : 6; }
int vvo_kv_bytes_per_vec(int fmt) {      /* head_dim 128 (kv_quant.h:63-76) */
    switch (fmt) {
        case 1: case 2: return 128;
        case VVO_KV_TQ4: return 64;
        case VVO_KV_TQ3: return 48;
        case VVO_KV_TQ2: return 32;
        case VVO_KV_TQ1_5: return 24;
        default: return 256;
    }
}

/* The fixed +-1 pattern of the randomised transform (kv_codec.cuh:132-136). */
static float kv_sign(int d) {
    uint32_t h = (uint32_t)d * 2654435761u + 0x9E3779B9u;
    h ^= h >> 15; h *= 0x85EBCA6Bu; h ^= h >> 13;
    return (h & 1u) ? -1.0f : 1.0f;
}

/* Walsh-Hadamard transform of 128 values in the order the accelerator adds
 * them: value 4 L + i lives in lane L; strides 1 and 2 inside a lane, then
 * lane strides 1 .. 16, the upper partner taking (other - own). */
static void wht128(float v[32][4]) {
    for (int L = 0; L < 32; L++) {
        float* x = v[L];
        float a;
        a = x[0] + x[1]; x[1] = x[0] - x[1]; x[0] = a;
        a = x[2] + x[3]; x[3] = x[2] - x[3]; x[2] = a;
        a = x[0] + x[2]; x[2] = x[0] - x[2]; x[0] = a;
        a = x[1] + x[3]; x[3] = x[1] - x[3]; x[1] = a;
    }
    for (int m = 1; m < 32; m <<= 1) {
        float n[32][4];
        for (int L = 0; L < 32; L++)
            for (int i = 0; i < 4; i++) {
                const float o = v[L ^ m][i];
                n[L][i] = (L & m) ? o - v[L][i] : v[L][i] + o;
            }
        memcpy(v, n, sizeof(n));
    }
}

static void rotate128(float v[32][4], int inverse) {
    if (!inverse) {
        for (int L = 0; L < 32; L++)
            for (int i = 0; i < 4; i++) v[L][i] *= kv_sign(4 * L + i);
        wht128(v);
        for (int L = 0; L < 32; L++)
            for (int i = 0; i < 4; i++) v[L][i] *= VVO_WHT_NORM;
    } else {
        wht128(v);
        for (int L = 0; L < 32; L++)
            for (int i = 0; i < 4; i++) v[L][i] *= VVO_WHT_NORM * kv_sign(4 * L + i);
    }
}

int vvo_kv_rotate(uint16_t* x16, int n_vectors, int inverse) {
    if (!x16) return VVO_ERR_NULL_PTR;
    for (int n = 0; n < n_vectors; n++) {
        float v[32][4];
        for (int d = 0; d < 128; d++) v[d / 4][d % 4] = vvo_half_to_float(x16[(size_t)n * 128 + d]);
        rotate128(v, inverse);
        for (int d = 0; d < 128; d++) x16[(size_t)n * 128 + d] = vvo_float_to_half_rne(v[d / 4][d % 4]);
    }
    return VVO_OK;
}

/* The packed code of a lane's four values (kv_codec.cuh:228-285): per value the
 * number of mid-points between neighbouring levels that it exceeds; for the
 * 1.5-bit form the nearest of eight 2-D code words per pair, first wins ties. */
static uint32_t tq_pack4(int fmt, const float y[4], float inv_sigma) {
    uint32_t bits = 0;
    if (fmt == VVO_KV_TQ1_5) {
        for (int p = 0; p < 2; p++) {
            const float a = y[2 * p] * inv_sigma, b = y[2 * p + 1] * inv_sigma;
            uint32_t best = 0;
            float bd = FLT_MAX;
            for (int c = 0; c < 8; c++) {
                const float da = a - kVq15[2 * c], db = b - kVq15[2 * c + 1];
                const float d = da * da + db * db;
                if (d < bd) { bd = d; best = (uint32_t)c; }
            }
            bits |= best << (3 * p);
        }
        return bits;
    }
    const float* lev = fmt == VVO_KV_TQ4 ? kLev4 : fmt == VVO_KV_TQ3 ? kLev3 : kLev2;
    const int nb = fmt == VVO_KV_TQ4 ? 4 : fmt == VVO_KV_TQ3 ? 3 : 2;
    for (int i = 0; i < 4; i++) {
        const float t = y[i] * inv_sigma;
        uint32_t c = 0;
        for (int j = 0; j + 1 < (1 << nb); j++) c += (t > 0.5f * (lev[j] + lev[j + 1])) ? 1u : 0u;
        bits |= c << (nb * i);
    }
    return bits;
}

static void tq_unpack4(int fmt, uint32_t bits, float sigma, float out[4]) {
    if (fmt == VVO_KV_TQ1_5) {
        for (int p = 0; p < 2; p++) {
            const uint32_t c = (bits >> (3 * p)) & 7u;
            out[2 * p] = sigma * kVq15[2 * c];
            out[2 * p + 1] = sigma * kVq15[2 * c + 1];
        }
        return;
    }
    const float* lev = fmt == VVO_KV_TQ4 ? kLev4 : fmt == VVO_KV_TQ3 ? kLev3 : kLev2;
    const int nb = fmt == VVO_KV_TQ4 ? 4 : fmt == VVO_KV_TQ3 ? 3 : 2;
    for (int i = 0; i < 4; i++) out[i] = sigma * lev[(bits >> (nb * i)) & ((1u << nb) - 1u)];
}

/* One vector: minus the reference, rotated, scaled by its own RMS, coded. The
 * sum of squares is an FMA chain per lane and a butterfly over lane strides
 * 16 .. 1 (kv_codec.cuh:167-171): every lane ends with the same bits. */
static void tq_store_one(int fmt, const uint16_t* src16, const uint16_t* ref16, uint8_t* dst, uint16_t* meta) {
    float v[32][4], ss[32];
    for (int d = 0; d < 128; d++) {
        float x = vvo_half_to_float(src16[d]);
        if (ref16) x -= vvo_half_to_float(ref16[d]);
        v[d / 4][d % 4] = x;
    }
    rotate128(v, 0);
    for (int L = 0; L < 32; L++) {
        float a = 0.0f;
        for (int i = 0; i < 4; i++) a = fmaf(v[L][i], v[L][i], a);
        ss[L] = a;
    }
    for (int o = 16; o > 0; o >>= 1) {
        float n[32];
        for (int L = 0; L < 32; L++) n[L] = ss[L] + ss[L ^ o];
        memcpy(ss, n, sizeof(n));
    }
    const float sigma = sqrtf(fmaxf(ss[0] / 128.0f, 1e-12f));
    const int nb = tq_lane_bits(fmt), bpv = vvo_kv_bytes_per_vec(fmt);
    uint32_t words[16] = {0};
    for (int L = 0; L < 32; L++) {
        const uint32_t bits = tq_pack4(fmt, v[L], 1.0f / sigma);
        const int bit = nb * L;
        words[bit >> 5] |= bits << (bit & 31);
        if ((bit & 31) + nb > 32) words[(bit >> 5) + 1] |= bits >> (32 - (bit & 31));
    }
    memcpy(dst, words, (size_t)bpv);
    *meta = vvo_float_to_half_rne(sigma);
}

int vvo_kv_store_tq(const uint16_t* src16, const uint16_t* ref16, int n_pos, int n_kv_heads, int fmt,
                    uint8_t* store, uint16_t* meta16) {
    if (!src16 || !store || !meta16) return VVO_ERR_NULL_PTR;
    if (fmt < VVO_KV_TQ4 || fmt > VVO_KV_TQ1_5) return VVO_ERR_INVALID_ARG;
    const int bpv = vvo_kv_bytes_per_vec(fmt);
    for (int p = 0; p < n_pos; p++)
        for (int h = 0; h < n_kv_heads; h++) {
            const size_t vec = (size_t)p * n_kv_heads + h;
            tq_store_one(fmt, src16 + vec * 128, ref16 ? ref16 + (size_t)h * 128 : NULL, store + vec * bpv,
                         meta16 + vec);
        }
    return VVO_OK;
}

/* One stored vector as FP32 in the space it was stored in: an FP8 value, or
 * RMS times level for TurboQuant (still rotated). */
static int kv_unpack_one(const uint8_t* src, const uint16_t* meta, int fmt, float val[128]) {
    if (fmt == 1 || fmt == 2) {
        for (int d = 0; d < 128; d++) val[d] = fp8_decode_one(src[d], fmt == 2);
        return VVO_OK;
    }
    if (fmt < VVO_KV_TQ4 || fmt > VVO_KV_TQ1_5) return VVO_ERR_INVALID_ARG;
    if (!meta) return VVO_ERR_NULL_PTR;
    uint32_t words[17] = {0};
    memcpy(words, src, (size_t)vvo_kv_bytes_per_vec(fmt));
    const int nb = tq_lane_bits(fmt);
    const float sigma = vvo_half_to_float(*meta);
    for (int L = 0; L < 32; L++) {
        const int bit = nb * L, sh = bit & 31;
        const uint32_t lo = words[bit >> 5], hi = words[(bit >> 5) + 1];
        const uint32_t bits = (sh ? ((lo >> sh) | (hi << (32 - sh))) : lo) & ((1u << nb) - 1u);
        tq_unpack4(fmt, bits, sigma, val + 4 * L);
    }
    return VVO_OK;
}

/* What attention over a quantised cache multiplies with: the stored vectors as
 * FP16 in the space they were stored in (TurboQuant: rotated, no reference). */
int vvo_kv_unpack(const uint8_t* store, const uint16_t* meta16, int n_vectors, int fmt, uint16_t* out16) {
    if (!store || !out16) return VVO_ERR_NULL_PTR;
    const int bpv = vvo_kv_bytes_per_vec(fmt);
    for (size_t vec = 0; vec < (size_t)n_vectors; vec++) {
        float val[128];
        const int rc = kv_unpack_one(store + vec * bpv, meta16 ? meta16 + vec : NULL, fmt, val);
        if (rc != VVO_OK) return rc;
        for (int d = 0; d < 128; d++) out16[vec * 128 + d] = vvo_float_to_half_rne(val[d]);
    }
    return VVO_OK;
}

/* Stored vectors back to FP16 in the ORIGINAL space (kv_quant.cu:311-338): the
 * unpacked values, for TurboQuant the inverse rotation, plus the reference when
 * given; FP32 throughout, one rounding at the end. */
int vvo_kv_dequant(const uint8_t* store, const uint16_t* meta16, const uint16_t* ref16, int n_pos,
                   int n_kv_heads, int fmt, uint16_t* out16) {
    if (!store || !out16) return VVO_ERR_NULL_PTR;
    const int bpv = vvo_kv_bytes_per_vec(fmt);
    for (int p = 0; p < n_pos; p++)
        for (int h = 0; h < n_kv_heads; h++) {
            const size_t vec = (size_t)p * n_kv_heads + h;
            float flat[128], v[32][4];
            const int rc = kv_unpack_one(store + vec * bpv, meta16 ? meta16 + vec : NULL, fmt, flat);
            if (rc != VVO_OK) return rc;
            memcpy(v, flat, sizeof(flat));
            if (fmt >= VVO_KV_TQ4) rotate128(v, 1);
            for (int d = 0; d < 128; d++) {
                float x = v[d / 4][d % 4];
                if (ref16) x += vvo_half_to_float(ref16[(size_t)h * 128 + d]);
                out16[vec * 128 + d] = vvo_float_to_half_rne(x);
            }
        }
    return VVO_OK;
}

/* ── BitNet: ternary and int8 integer layers (include/vibevoice/bitnet.h) ──── */

/* bitnet.h:13-24, bitnet_cpu.c:222-235: value t in {-1, 0, 1} is stored as code
 * t + 1; byte j of a 32-byte block holds k = j (bits 7:6), j + 32 (5:4),
 * j + 64 (3:2), j + 96 (1:0) of the block's 128 columns. */
int vvo_ternary_pack(const int8_t* t, int64_t N, int64_t K, uint8_t* codes) {
    if (!t || !codes) return VVO_ERR_NULL_PTR;
    if (N <= 0 || K <= 0 || (K % 128) != 0) return VVO_ERR_INVALID_ARG;
    for (int64_t n = 0; n < N; n++)
        for (int64_t b = 0; b < K / 128; b++)
            for (int j = 0; j < 32; j++) {
                uint8_t byte = 0;
                for (int p = 0; p < 4; p++) {
                    const int v = t[n * K + b * 128 + 32 * p + j];
                    if (v < -1 || v > 1) return VVO_ERR_INVALID_ARG;
                    byte |= (uint8_t)((v + 1) << (6 - 2 * p));
                }
                codes[n * (K / 4) + b * 32 + j] = byte;
            }
    return VVO_OK;
}

static int ternary_code(const uint8_t* row, int64_t k) {
    const int64_t b = k / 128, r = k % 128;
    return (row[b * 32 + r % 32] >> (6 - 2 * (int)(r / 32))) & 3;
}

/* bitnet_cpu.c:352-358, 396-441: per row s = (float)(127 / max(amax, 1e-5)) in
 * double; q = the integer that x * s + 1.5 * 2^23, rounded ONCE as a fused
 * multiply-add, carries in its mantissa; clamped to [-128, 127]. */
int vvo_bn_act_quant(const float* x, int M, int K, int8_t* q, float* scale, int32_t* sum) {
    if (!x || !q || !scale) return VVO_ERR_NULL_PTR;
    if (M <= 0 || K <= 0) return VVO_ERR_INVALID_ARG;
    for (int m = 0; m < M; m++) {
        const float* xr = x + (size_t)m * K;
        float amax = 0.0f;
        for (int k = 0; k < K; k++) {
            const float a = fabsf(xr[k]);
            if (a > amax) amax = a;
        }
        const double dmax = amax > 0.00001 ? (double)amax : 0.00001;
        const float s = (float)(127.0 / dmax);
        int32_t acc = 0;
        for (int k = 0; k < K; k++) {
            const float v = fmaf(xr[k], s, 12582912.0f);
            int32_t bits;
            memcpy(&bits, &v, 4);
            int i = (bits & 0x007fffff) - 0x00400000;
            if (i > 127) i = 127;
            if (i < -128) i = -128;
            q[(size_t)m * K + k] = (int8_t)i;
            acc += i;
        }
        scale[m] = s;
        if (sum) sum[m] = acc;
    }
    return VVO_OK;
}

/* bitnet_cpu.c:741-790: acc = sum_k (code - 1) * q, exactly; y = ((float)acc /
 * x_scale[m]) * w_scale (+ bias[n]), each operation rounded on its own. */
int vvo_ternary_linear(const int8_t* q, const float* x_scale, const uint8_t* codes, float w_scale,
                       const float* bias, int M, int N, int K, int32_t* acc_out, float* y) {
    if (!q || !codes) return VVO_ERR_NULL_PTR;
    if (y && !x_scale) return VVO_ERR_NULL_PTR;
    if (M <= 0 || N <= 0 || K <= 0 || (K % 128) != 0) return VVO_ERR_INVALID_ARG;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; n++) {
        const uint8_t* row = codes + (size_t)n * (K / 4);
        for (int m = 0; m < M; m++) {
            int32_t acc = 0;
            for (int k = 0; k < K; k++) acc += (ternary_code(row, k) - 1) * (int32_t)q[(size_t)m * K + k];
            const size_t o = (size_t)m * N + n;
            if (acc_out) acc_out[o] = acc;
            if (y) {
                float v = (float)acc / x_scale[m];
                v = v * w_scale;
                if (bias) v = v + bias[n];
                y[o] = v;
            }
        }
    }
    return VVO_OK;
}

/* bitnet_cpu.c:1048-1131: acc = sum_k w * a; y = (float)acc * (w_scale / a_scale)
 * (+ bias[n]); absmax = max |y|. */
int vvo_i8_linear(const int8_t* a, float a_scale, const int8_t* w, float w_scale, const float* bias,
                  int M, int N, int K, int32_t* acc_out, float* y, float* absmax) {
    if (!a || !w) return VVO_ERR_NULL_PTR;
    if (M <= 0 || N <= 0 || K <= 0) return VVO_ERR_INVALID_ARG;
    const float d = y ? w_scale / a_scale : 0.0f;
    float amax = 0.0f;
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            int32_t acc = 0;
            for (int k = 0; k < K; k++) acc += (int32_t)w[(size_t)n * K + k] * (int32_t)a[(size_t)m * K + k];
            const size_t o = (size_t)m * N + n;
            if (acc_out) acc_out[o] = acc;
            if (y) {
                float v = (float)acc * d;
                if (bias) v = v + bias[n];
                y[o] = v;
                if (fabsf(v) > amax) amax = fabsf(v);
            }
        }
    if (absmax) *absmax = amax;
    return VVO_OK;
}

/* bitnet_cpu.c:1133-1151: inv = 127 / absmax (0 when absmax is 0);
 * q = round_half_even(clamp(y * inv, relu ? 0 : -127, 127)). */
int vvo_i8s_requant(const float* y, int64_t n, float absmax, int relu, int8_t* q, float* out_scale) {
    if (!y || !q) return VVO_ERR_NULL_PTR;
    const float inv = absmax != 0.0f ? 127.0f / absmax : 0.0f;
    const float lo = relu ? 0.0f : -127.0f;
    for (int64_t i = 0; i < n; i++) {
        float v = y[i] * inv;
        v = v < lo ? lo : (v > 127.0f ? 127.0f : v);
        q[i] = (int8_t)nearbyintf(v);
    }
    if (out_scale) *out_scale = inv;
    return VVO_OK;
}

/* bitnet_cpu.c:1153-1213: logit_n = ((float)(w_n . q) * w_scale[n]) / scale; the
 * largest wins, ties to the lowest index. */
int vvo_i8_head_argmax(const int8_t* q, float scale, const int8_t* w, const float* w_scale, int V, int K,
                       int32_t* token, float* value) {
    if (!q || !w || !w_scale || !token) return VVO_ERR_NULL_PTR;
    if (V <= 0 || K <= 0 || !(scale > 0.0f)) return VVO_ERR_INVALID_ARG;
    float bv = -FLT_MAX;
    int32_t bi = 0;
    for (int n = 0; n < V; n++) {
        int32_t acc = 0;
        for (int k = 0; k < K; k++) acc += (int32_t)w[(size_t)n * K + k] * (int32_t)q[k];
        float v = (float)acc * w_scale[n];
        v = v / scale;
        if (n == 0 || v > bv) { bv = v; bi = n; }
    }
    *token = bi;
    if (value) *value = bv;
    return VVO_OK;
}

/* ── Conv-VAE encoder ops (src/cuda/vae_kernels.cu) ───────────────────────── */

/* Column pos of [context ++ input] of an item, channel ic: context from the
 * state (zeros when there is none), then the item's input, then zeros. */
static float vae_item_value(const vvo_vae_conv_desc_t* d, const vvo_vae_conv_item_t* it, const uint16_t* x,
                            int64_t ld_in, int ic, int pos, uint16_t* bits) {
    uint16_t v = 0;
    if (pos >= 0 && pos < it->have + it->in_len) {
        if (pos < it->have) {
            const uint16_t* tl = (const uint16_t*)it->tail_in;
            v = tl ? tl[(size_t)ic * d->cap + pos] : 0;
        } else {
            const uint16_t* xb = it->in_ptr ? (const uint16_t*)it->in_ptr : x + it->in_off;
            v = xb[(size_t)ic * ld_in + (pos - it->have)];
        }
    }
    if (bits) *bits = v;
    return vvo_half_to_float(v);
}

int vvo_vae_conv(const vvo_vae_conv_desc_t* d, const uint16_t* x, int64_t ld_in, const uint16_t* w,
                 const uint16_t* b, uint16_t* y, int64_t ld_out, int in_ch, int out_ch, int k, int stride,
                 int transposed) {
    if (!d || !w) return VVO_ERR_NULL_PTR;
    if (d->n <= 0 || d->n > VVO_VAE_MAX_ITEMS) return VVO_ERR_INVALID_ARG;
    for (int i = 0; i < d->n; i++) {
        const vvo_vae_conv_item_t* it = &d->it[i];
        for (int oc = 0; oc < out_ch; oc++)
            for (int t = 0; t < it->out_len; t++) {
                float sum = 0.0f;
                for (int ic = 0; ic < in_ch; ic++)
                    for (int kk = 0; kk < k; kk++) {
                        const int p = t * stride + kk;
                        if (p < it->have + it->in_len)
                            sum = fmaf(vvo_half_to_float(w[((size_t)oc * in_ch + ic) * k + kk]),
                                       vae_item_value(d, it, x, ld_in, ic, p, NULL), sum);
                    }
                if (b) sum += vvo_half_to_float(b[oc]);
                if (transposed) {
                    if (t >= it->skip)
                        ((uint16_t*)it->out_ptr)[(size_t)(t - it->skip) * it->out_ld + oc] = vvo_float_to_half_rne(sum);
                } else {
                    y[(size_t)oc * ld_out + it->out_off + t] = vvo_float_to_half_rne(sum);
                }
            }
    }
    return VVO_OK;
}

int vvo_vae_tail(const vvo_vae_conv_desc_t* d, const uint16_t* x, int64_t ld_in, int in_ch) {
    if (!d) return VVO_ERR_NULL_PTR;
    for (int i = 0; i < d->n; i++) {
        const vvo_vae_conv_item_t* it = &d->it[i];
        if (!it->tail_out || it->keep <= 0) continue;
        for (int c = 0; c < in_ch; c++)
            for (int j = 0; j < it->keep; j++) {
                uint16_t v;
                vae_item_value(d, it, x, ld_in, c, it->have + it->in_len - it->keep + j, &v);
                ((uint16_t*)it->tail_out)[(size_t)c * d->cap + j] = v;
            }
    }
    return VVO_OK;
}

static const vvo_vae_conv_item_t* vae_item_of(const vvo_vae_conv_desc_t* d, int64_t p) {
    int i = 0;
    while (i + 1 < d->n && p >= d->it[i + 1].out_off) i++;
    return &d->it[i];
}

int vvo_vae_im2col(const vvo_vae_conv_desc_t* d, const uint16_t* x, int64_t ld_in, int in_ch, int k, int stride,
                   int64_t p0, int pc, uint16_t* col, int64_t ldcol) {
    if (!d || !col) return VVO_ERR_NULL_PTR;
    for (int kr = 0; kr < in_ch * k; kr++)
        for (int q = 0; q < pc; q++) {
            const vvo_vae_conv_item_t* it = vae_item_of(d, p0 + q);
            const int t = (int)(p0 + q - it->out_off);
            uint16_t v = 0;
            if (t < it->out_len) vae_item_value(d, it, x, ld_in, kr / k, t * stride + kr % k, &v);
            col[(size_t)kr * ldcol + q] = v;
        }
    return VVO_OK;
}

int vvo_vae_conv_gemm(const uint16_t* w, const uint16_t* col, int64_t ldcol, const uint16_t* b, uint16_t* y,
                      int64_t ld_out, int out_ch, int K, int pc) {
    if (!w || !col || !y) return VVO_ERR_NULL_PTR;
    for (int oc = 0; oc < out_ch; oc++)
        for (int q = 0; q < pc; q++) {
            float sum = 0.0f;
            for (int kr = 0; kr < K; kr++)
                sum = fmaf(vvo_half_to_float(w[(size_t)oc * K + kr]), vvo_half_to_float(col[(size_t)kr * ldcol + q]), sum);
            if (b) sum += vvo_half_to_float(b[oc]);
            y[(size_t)oc * ld_out + q] = vvo_float_to_half_rne(sum);
        }
    return VVO_OK;
}

static float vae_rms_col(const uint16_t* col, int64_t stride, int C, float eps) {
    float ss = 0.0f;
    for (int c = 0; c < C; c++) {
        const float v = vvo_half_to_float(col[(size_t)c * stride]);
        ss = fmaf(v, v, ss);
    }
    return 1.0f / sqrtf(ss / (float)C + eps);
}

int vvo_vae_rms(const uint16_t* x, int64_t ld, int64_t T, int C, float eps, float* rinv,
                const vvo_vae_conv_desc_t* d) {
    if (!x || !rinv) return VVO_ERR_NULL_PTR;
    for (int64_t i = 0; i < T; i++) rinv[i] = vae_rms_col(x + i, ld, C, eps);
    if (d && d->cap > 0)
        for (int item = 0; item < d->n; item++) {
            const vvo_vae_conv_item_t* it = &d->it[item];
            if (!it->tail_in) continue;
            for (int q = 0; q < it->have; q++)
                rinv[T + (int64_t)item * d->cap + q] = vae_rms_col((const uint16_t*)it->tail_in + q, d->cap, C, eps);
        }
    return VVO_OK;
}

int vvo_vae_mixer(const vvo_vae_conv_desc_t* d, const uint16_t* xin, uint16_t* xout, int64_t ld, const float* rinv,
                  int64_t T_total, const uint16_t* nw, const uint16_t* cw, const uint16_t* cb,
                  const uint16_t* gamma, int C, int k) {
    if (!d || !xin || !xout || !rinv || !nw || !cw) return VVO_ERR_NULL_PTR;
    if (k < 1 || k > 16) return VVO_ERR_INVALID_ARG;
    for (int item = 0; item < d->n; item++) {
        const vvo_vae_conv_item_t* it = &d->it[item];
        const uint16_t* tl = (const uint16_t*)it->tail_in;
        for (int c = 0; c < C; c++)
            for (int t = 0; t < it->in_len; t++) {
                float sum = 0.0f;
                for (int kk = 0; kk < k; kk++) {
                    const int p = t - (k - 1) + kk;             /* position in the item's input; negative = context */
                    uint16_t nv = 0;
                    if (p >= 0) {
                        const int64_t col = it->in_off + p;
                        nv = vvo_float_to_half_rne((vvo_half_to_float(xin[(size_t)c * ld + col]) * rinv[col]) *
                                                   vvo_half_to_float(nw[c]));
                    } else {
                        const int tp = it->have + p;
                        if (tl && tp >= 0)
                            nv = vvo_float_to_half_rne((vvo_half_to_float(tl[(size_t)c * d->cap + tp]) *
                                                        rinv[T_total + (int64_t)item * d->cap + tp]) *
                                                       vvo_half_to_float(nw[c]));
                    }
                    sum = fmaf(vvo_half_to_float(cw[c * k + kk]), vvo_half_to_float(nv), sum);
                }
                if (cb) sum += vvo_half_to_float(cb[c]);
                const float yv = vvo_half_to_float(vvo_float_to_half_rne(sum));
                const size_t off = (size_t)c * ld + it->in_off + t;
                const float xv = vvo_half_to_float(xin[off]);
                xout[off] = vvo_float_to_half_rne(gamma ? fmaf(yv, vvo_half_to_float(gamma[c]), xv) : xv + yv);
            }
    }
    return VVO_OK;
}

int vvo_vae_gemm_nn(int epilogue, const uint16_t* A, const uint16_t* B, int64_t ldb, uint16_t* C, int64_t ldc,
                    int M, int K, int P, const uint16_t* bias, const uint16_t* gamma, const float* rinv,
                    const uint16_t* nw) {
    if (!A || !B || !C) return VVO_ERR_NULL_PTR;
    if (epilogue < 0 || epilogue > 2 || ((nw != NULL) != (rinv != NULL))) return VVO_ERR_INVALID_ARG;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < M; r++)
        for (int c = 0; c < P; c++) {
            double acc = 0.0;
            for (int kk = 0; kk < K; kk++) {
                float bv = vvo_half_to_float(B[(size_t)kk * ldb + c]);
                if (nw) bv = vvo_half_to_float(vvo_float_to_half_rne((bv * rinv[c]) * vvo_half_to_float(nw[kk])));
                acc += (double)vvo_half_to_float(A[(size_t)r * K + kk]) * (double)bv;
            }
            const size_t off = (size_t)r * ldc + c;
            if (epilogue == 2) {
                C[off] = vvo_float_to_half_rne((float)acc + (bias ? vvo_half_to_float(bias[r]) : 0.0f));
                continue;
            }
            float v = vvo_half_to_float(vvo_float_to_half_rne((float)acc));
            if (bias) v = vvo_half_to_float(vvo_float_to_half_rne(v + vvo_half_to_float(bias[r])));
            if (epilogue == 0) {
                C[off] = vvo_float_to_half_rne(0.5f * v * (1.0f + erff(v * 0.7071067811865476f)));
            } else {
                const float xv = vvo_half_to_float(C[off]);
                C[off] = vvo_float_to_half_rne(gamma ? fmaf(v, vvo_half_to_float(gamma[r]), xv) : xv + v);
            }
        }
    return VVO_OK;
}

uint16_t vvo_trunc_half(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int e = (int)((u >> 23) & 0xFF) - 127 + 15;
    const uint32_t frac = (u >> 13) & 0x3FFu;
    if (e <= 0) return (uint16_t)sign;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | ((uint32_t)e << 10) | frac);
}

int vvo_vae_gemm_tn(const uint16_t* A, int64_t lda, const uint16_t* B, uint16_t* C, int64_t ldc, int M, int N,
                    int K, const uint16_t* bias, const vvo_vae_rows_t* rows) {
    if (!A || !B) return VVO_ERR_NULL_PTR;
    const int mode = rows ? rows->mode : 0;
    if (mode == 0 && !C) return VVO_ERR_NULL_PTR;
    for (int r = 0; r < M; r++)
        for (int c = 0; c < N; c++) {
            double acc = 0.0;
            for (int kk = 0; kk < K; kk++)
                acc += (double)vvo_half_to_float(A[(size_t)r * lda + kk]) * (double)vvo_half_to_float(B[(size_t)c * K + kk]);
            uint16_t y = vvo_float_to_half_rne((float)acc);
            if (bias) y = vvo_float_to_half_rne(vvo_half_to_float(y) + vvo_half_to_float(bias[c]));
            if (mode == 0) {
                C[(size_t)r * ldc + c] = y;
                continue;
            }
            int s = 0;
            while (s + 1 < rows->n && r >= rows->seg[s + 1].row0) s++;
            uint16_t* dst = (uint16_t*)rows->seg[s].dst + (size_t)(r - rows->seg[s].row0) * rows->seg[s].ld + c;
            if (mode == 1) *dst = y;
            else if (mode == 2) *dst = vvo_trunc_half(vvo_half_to_float(y));
            else *dst = vvo_trunc_half(vvo_half_to_float(*dst) + vvo_half_to_float(y));
        }
    return VVO_OK;
}

int vvo_argmax_first(const float* logits, int n, int32_t* token, float* value) {
    if (!logits || !token) return VVO_ERR_NULL_PTR;
    int best = 0;
    float bv = logits[0];
    for (int i = 1; i < n; i++)
        if (logits[i] > bv) { bv = logits[i]; best = i; }
    *token = best;
    if (value) *value = bv;
    return VVO_OK;
}

/* ── seeded inputs ─────────────────────────────────────────────────────── */

static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* One standard normal per (seed, i): Box-Muller on two counter-based draws. */
static inline double normal_at(uint64_t seed, uint64_t i) {
    const uint64_t base = seed * 0xD1342543DE82EF95ull + 2u * i;
    const uint64_t a = splitmix64(base), b = splitmix64(base + 1u);
    const double u1 = ((double)(a >> 11) + 1.0) * 0x1p-53;   /* (0, 1] */
    const double u2 = (double)(b >> 11) * 0x1p-53;           /* [0, 1) */
    return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
}

void vvo_fill_normal_f32(float* out, size_t n, uint64_t seed,
                         double mean, double std) {
    long i;
#pragma omp parallel for schedule(static)
    for (i = 0; i < (long)n; i++)
        out[i] = (float)(mean + std * normal_at(seed, (uint64_t)i));
}

void vvo_fill_normal_f16(uint16_t* out, size_t n, uint64_t seed,
                         double mean, double std) {
    long i;
#pragma omp parallel for schedule(static)
    for (i = 0; i < (long)n; i++)
        out[i] = vvo_float_to_half_rne(
            (float)(mean + std * normal_at(seed, (uint64_t)i)));
}

void vvo_fill_ids(int32_t* out, size_t n, uint64_t seed, int32_t bound) {
    long i;
#pragma omp parallel for schedule(static)
    for (i = 0; i < (long)n; i++) {
        const uint64_t r = splitmix64(seed * 0xA0761D6478BD642Full + (uint64_t)i);
        /* multiply-shift maps 64 random bits onto [0, bound) */
        out[i] = (int32_t)(((unsigned __int128)r * (uint64_t)bound) >> 64);
    }
}

int vvo_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void vvo_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
