/*
 * mynn_oracle.c -- CPU restatement of the reference engine's quantized-LLM hot path.
 * TEST INFRASTRUCTURE ONLY (see mynn_oracle.h): the checker for the HIP library and the
 * timed CPU baseline; never linked into, or called by, the shipped path.
 *
 * Built with -ffp-contract=off and without fast-math so every f32 operation below rounds
 * exactly where it is written.
 */
#include "mynn_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ settings */
static int g_lanes = 16;
static int g_threads = 0; /* 0 = OpenMP default */

void orc_set_lanes(int lanes) {
    if (lanes < 1) lanes = 1;
    if (lanes > 64) lanes = 64;
    int p = 1;
    while (p * 2 <= lanes) p *= 2;
    g_lanes = p;
}
int orc_get_lanes(void) { return g_lanes; }
void orc_set_threads(int n) { g_threads = n < 0 ? 0 : n; }
int orc_get_threads(void) {
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}
static int nthreads_for(size_t n) {
    /* the reference turns OpenMP on for an outer loop of at least 64 iterations
     * (src/schedule/omp.rs:70-95) */
    if (n < 64) return 1;
    return orc_get_threads();
}

/* ------------------------------------------------------------------ scalar conversions */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ftype.rs:41-50 / quantize.rs:74-81 (NaN -> 0x7FC0 as quantize.rs) */
uint16_t orc_f32_to_bf16(float x) {
    if (x != x) return 0x7FC0;
    uint32_t bits = f2u(x);
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}
float orc_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

/* IEEE binary16, round to nearest even, overflow to inf, subnormals kept */
uint16_t orc_f32_to_f16(float x) {
    uint32_t u = f2u(x);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (a > 0x7F800000u ? 0x200u | ((a >> 13) & 0x3FFu) : 0));
    if (a >= 0x477FF000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (a < 0x33000001u) /* <= 2^-25: rounds to zero (tie at 2^-25 goes to even = 0) */
        return (uint16_t)sign;
    int exp = (int)(a >> 23) - 127;
    uint32_t man = (a & 0x7FFFFFu) | 0x800000u;
    int shift; /* bits dropped from the 24-bit significand */
    uint32_t base;
    if (exp < -14) { shift = 13 + (-14 - exp); base = 0; }          /* subnormal result */
    else { shift = 13; base = (uint32_t)(exp + 15) << 10; man &= 0x7FFFFFu; }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q)); /* a carry out of the mantissa bumps the exponent */
}
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        float v = (float)man * 5.9604644775390625e-08f; /* 2^-24, exact */
        return sign ? -v : v;
    }
    if (exp == 0x1F) return u2f(sign | 0x7F800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline float ld(const void *p, size_t i, int dt) {
    switch (dt) {
    case ORC_BF16: return orc_bf16_to_f32(((const uint16_t *)p)[i]);
    case ORC_F16: return orc_f16_to_f32(((const uint16_t *)p)[i]);
    default: return ((const float *)p)[i];
    }
}
static inline void st(void *p, size_t i, float v, int dt) {
    switch (dt) {
    case ORC_BF16: ((uint16_t *)p)[i] = orc_f32_to_bf16(v); break;
    case ORC_F16: ((uint16_t *)p)[i] = orc_f32_to_f16(v); break;
    default: ((float *)p)[i] = v; break;
    }
}
static inline size_t esize(int dt) { return dt == ORC_F32 ? 4 : 2; }
static inline float rnd(float v, int dt) {
    switch (dt) {
    case ORC_BF16: return orc_bf16_to_f32(orc_f32_to_bf16(v));
    case ORC_F16: return orc_f16_to_f32(orc_f32_to_f16(v));
    default: return v;
    }
}

void orc_convert(void *dst, int dd, const void *src, int sd, size_t n) {
    for (size_t i = 0; i < n; i++) st(dst, i, ld(src, i, sd), dd);
}

static float *widen(const void *p, size_t n, int dt) {
    float *f = (float *)malloc((n ? n : 1) * sizeof(float));
    for (size_t i = 0; i < n; i++) f[i] = ld(p, i, dt);
    return f;
}

/* ------------------------------------------------------------------ fixed-order dot products */
#define MAXL 64
static inline float tree(float *acc, int lanes) {
    for (int s = lanes / 2; s > 0; s >>= 1)
        for (int j = 0; j < s; j++) acc[j] = acc[j] + acc[j + s];
    return acc[0];
}
/* sum_k a[k]*(f32)w[k]: lane k%lanes, then pairwise tree */
static float dot_f32_i8(const float *a, const int8_t *w, size_t K) {
    const int L = g_lanes;
    float acc[MAXL];
    for (int j = 0; j < L; j++) acc[j] = 0.0f;
    size_t k = 0;
    if (L == 16) {
        for (; k + 16 <= K; k += 16)
            for (int j = 0; j < 16; j++) acc[j] = acc[j] + a[k + j] * (float)w[k + j];
    } else if (L == 8) {  /* (constant trip counts: the compiler vectorises these; the sums are those of the generic loop) */
        for (; k + 8 <= K; k += 8)
            for (int j = 0; j < 8; j++) acc[j] = acc[j] + a[k + j] * (float)w[k + j];
    } else if (L == 32) {
        for (; k + 32 <= K; k += 32)
            for (int j = 0; j < 32; j++) acc[j] = acc[j] + a[k + j] * (float)w[k + j];
    } else if (L == 64) {
        for (; k + 64 <= K; k += 64)
            for (int j = 0; j < 64; j++) acc[j] = acc[j] + a[k + j] * (float)w[k + j];
    } else {
        for (; k + (size_t)L <= K; k += (size_t)L)
            for (int j = 0; j < L; j++) acc[j] = acc[j] + a[k + j] * (float)w[k + j];
    }
    for (int j = 0; k < K; k++, j++) acc[j] = acc[j] + a[k] * (float)w[k];
    return tree(acc, L);
}
static float dot_f32_f32(const float *a, const float *b, size_t K) {
    const int L = g_lanes;
    float acc[MAXL];
    for (int j = 0; j < L; j++) acc[j] = 0.0f;
    size_t k = 0;
    if (L == 16) {
        for (; k + 16 <= K; k += 16)
            for (int j = 0; j < 16; j++) acc[j] = acc[j] + a[k + j] * b[k + j];
    } else if (L == 8) {
        for (; k + 8 <= K; k += 8)
            for (int j = 0; j < 8; j++) acc[j] = acc[j] + a[k + j] * b[k + j];
    } else if (L == 32) {
        for (; k + 32 <= K; k += 32)
            for (int j = 0; j < 32; j++) acc[j] = acc[j] + a[k + j] * b[k + j];
    } else if (L == 64) {
        for (; k + 64 <= K; k += 64)
            for (int j = 0; j < 64; j++) acc[j] = acc[j] + a[k + j] * b[k + j];
    } else {
        for (; k + (size_t)L <= K; k += (size_t)L)
            for (int j = 0; j < L; j++) acc[j] = acc[j] + a[k + j] * b[k + j];
    }
    for (int j = 0; k < K; k++, j++) acc[j] = acc[j] + a[k] * b[k];
    return tree(acc, L);
}

/* ------------------------------------------------------------------ A1 */
void orc_dequantize_linear(void *out, const int8_t *x, const void *scale, size_t rows,
                           size_t cols, int dtype) {
    for (size_t r = 0; r < rows; r++) {
        float s = ld(scale, r, dtype);
        for (size_t c = 0; c < cols; c++) st(out, r * cols + c, (float)x[r * cols + c] * s, dtype);
    }
}

/* ------------------------------------------------------------------ A2 */
void orc_dequant_matmul(void *out, const void *act, const int8_t *wq, const void *scale,
                        size_t M, size_t N, size_t K, int act_dtype, int out_dtype, int mode) {
    if (mode < 0) mode = (M == 1) ? 0 : 1;
    float *a = widen(act, M * K, act_dtype);
    if (mode == 0) {
        int nt = nthreads_for(N);
        (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt) if (nt > 1)
        for (long long n = 0; n < (long long)N; n++) {
            float s = ld(scale, (size_t)n, out_dtype);
            for (size_t m = 0; m < M; m++) {
                float acc = dot_f32_i8(a + m * K, wq + (size_t)n * K, K);
                st(out, m * N + (size_t)n, acc * s, out_dtype);
            }
        }
    } else {
        /* dequantise each weight row first (f32 product, optionally rounded to the 16-bit type),
         * then an f32-accumulate GEMM */
        int nt = nthreads_for(N);
        (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt) if (nt > 1)
        for (long long n = 0; n < (long long)N; n++) {
            float *wrow = (float *)malloc((K ? K : 1) * sizeof(float));
            float s = ld(scale, (size_t)n, out_dtype);
            for (size_t k = 0; k < K; k++) {
                float w = (float)wq[(size_t)n * K + k] * s;
                wrow[k] = (mode == 2) ? rnd(w, out_dtype) : w;
            }
            for (size_t m = 0; m < M; m++)
                st(out, m * N + (size_t)n, dot_f32_f32(a + m * K, wrow, K), out_dtype);
            free(wrow);
        }
    }
    free(a);
}

/* ------------------------------------------------------------------ A3 */
void orc_quantized_matmul(void *out, int32_t *acc_out, const int8_t *lhs, const void *lhs_scale,
                          const int8_t *rhs, const void *rhs_scale, size_t M, size_t N, size_t K,
                          int dtype) {
    for (size_t m = 0; m < M; m++) {
        float asc = lhs_scale ? ld(lhs_scale, m, dtype) : 1.0f;
        int nt = nthreads_for(N);
        (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt) if (nt > 1)
        for (long long n = 0; n < (long long)N; n++) {
            const int8_t *a = lhs + m * K, *w = rhs + (size_t)n * K;
            int32_t acc = 0;
            for (size_t k = 0; k < K; k++) acc += (int32_t)w[k] * (int32_t)a[k];
            if (acc_out) acc_out[m * N + (size_t)n] = acc;
            if (out) {
                float wsc = ld(rhs_scale, (size_t)n, dtype);
                st(out, m * N + (size_t)n, (float)acc * asc * wsc, dtype);
            }
        }
    }
}

/* ------------------------------------------------------------------ A4 */
static inline float round_half_away(float v) { return roundf(v); } /* Rust f32::round */

static void dynquant_rows(int8_t *y, void *scale, const void *x, size_t M, size_t K, int dtype) {
    for (size_t m = 0; m < M; m++) {
        float amax = 0.0f;
        for (size_t j = 0; j < K; j++) amax = fmaxf(amax, fabsf(ld(x, m * K + j, dtype)));
        float sc = amax > 0.0f ? amax / 127.0f : 1.0f;
        float inv = 1.0f / sc;
        for (size_t j = 0; j < K; j++) {
            float q = round_half_away(ld(x, m * K + j, dtype) * inv);
            q = q < -127.0f ? -127.0f : (q > 127.0f ? 127.0f : q);
            y[m * K + j] = (int8_t)q;
        }
        st(scale, m, sc, dtype);
    }
}
void orc_dynquant_i8(int8_t *y, void *scale, const void *x, size_t M, size_t K, int dtype) {
    dynquant_rows(y, scale, x, M, K, dtype);
}
void orc_dynquant_i8_per_tensor(int8_t *y, void *scale, const void *x, size_t n, int dtype) {
    dynquant_rows(y, scale, x, 1, n, dtype);
}
void orc_dynquant_u8_asym(uint8_t *y, void *scale, uint8_t *zp, const void *x, size_t M, size_t K,
                          int dtype) {
    for (size_t m = 0; m < M; m++) {
        float mn = INFINITY, mx = -INFINITY;
        for (size_t j = 0; j < K; j++) {
            float v = ld(x, m * K + j, dtype);
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
        }
        mn = fminf(mn, 0.0f);
        mx = fmaxf(mx, 0.0f);
        float sc = (mx - mn) / 255.0f;
        if (sc == 0.0f) sc = 1.0f;
        int z = (int)nearbyintf(-mn / sc);
        z = z < 0 ? 0 : (z > 255 ? 255 : z);
        for (size_t j = 0; j < K; j++) {
            int q = (int)nearbyintf(ld(x, m * K + j, dtype) / sc) + z;
            y[m * K + j] = (uint8_t)(q < 0 ? 0 : (q > 255 ? 255 : q));
        }
        st(scale, m, sc, dtype);
        zp[m] = (uint8_t)z;
    }
}

/* ------------------------------------------------------------------ A5 */
static inline float kv_ld(const void *p, size_t i, int dtype, int kv_int8) {
    return kv_int8 ? (float)((const int8_t *)p)[i] : ld(p, i, dtype);
}
void orc_attention(void *out, const void *q, const void *k, const void *v, const void *k_scale,
                   const void *v_scale, long long active, size_t B, size_t Hq, size_t Hkv,
                   size_t Sq, size_t Sk, size_t D, int is_causal, float scale, int dtype,
                   int kv_int8) {
    long long act = active < 0 ? (long long)Sk : active;
    long long past = act - (long long)Sq;
    size_t group = Hq / Hkv;
    size_t outer = B * Hq * Sq;
    int nt = nthreads_for(outer >= 64 ? outer : 0) ;
    (void)nt;
    /* the reference runs this loop nest on one thread; rows are independent, so the split
     * below changes nothing but the wall time */
#pragma omp parallel for schedule(static) num_threads(nt) if (nt > 1)
    for (long long oi = 0; oi < (long long)outer; oi++) {
        size_t bh = (size_t)oi / Sq, sq = (size_t)oi % Sq;
        size_t b = bh / Hq, h = bh % Hq;
        size_t bhkv = b * Hkv + h / group;
        const size_t qo = (bh * Sq + sq) * D;
        float *o = (float *)malloc(D * sizeof(float));
        for (size_t d = 0; d < D; d++) o[d] = 0.0f;
        long long bound = act;
        if (is_causal) {
            long long cap = past + (long long)sq + 1;
            if (cap < bound) bound = cap;
        }
        if (bound > (long long)Sk) bound = (long long)Sk;
        float m = -INFINITY, s = 0.0f;
        for (long long kk = 0; kk < bound; kk++) {
            size_t ko = (bhkv * Sk + (size_t)kk) * D;
            float sum = 0.0f;
            for (size_t d = 0; d < D; d++) sum = sum + ld(q, qo + d, dtype) * kv_ld(k, ko + d, dtype, kv_int8);
            if (kv_int8) sum = sum * ld(k_scale, bhkv * Sk + (size_t)kk, dtype);
            float qk = sum * scale;
            float m_new = fmaxf(m, qk);
            float factor = expf(m - m_new);
            float e = expf(qk - m_new);
            s = s * factor + e;
            float e_eff = kv_int8 ? e * ld(v_scale, bhkv * Sk + (size_t)kk, dtype) : e;
            for (size_t d = 0; d < D; d++) o[d] = o[d] * factor + e_eff * kv_ld(v, ko + d, dtype, kv_int8);
            m = m_new;
        }
        for (size_t d = 0; d < D; d++) st(out, qo + d, o[d] / s, dtype);
        free(o);
    }
}

void orc_attention_f64(double *out, const void *q, const void *k, const void *v, long long active,
                       size_t B, size_t Hq, size_t Hkv, size_t Sq, size_t Sk, size_t D,
                       int is_causal, double scale, int dtype) {
    long long act = active < 0 ? (long long)Sk : active;
    long long past = act - (long long)Sq;
    size_t group = Hq / Hkv;
    double *p = (double *)malloc((Sk ? Sk : 1) * sizeof(double));
    for (size_t bh = 0; bh < B * Hq; bh++)
        for (size_t sq = 0; sq < Sq; sq++) {
            size_t b = bh / Hq, h = bh % Hq, bhkv = b * Hkv + h / group;
            size_t qo = (bh * Sq + sq) * D;
            long long bound = act;
            if (is_causal && past + (long long)sq + 1 < bound) bound = past + (long long)sq + 1;
            if (bound > (long long)Sk) bound = (long long)Sk;
            double mx = -INFINITY;
            for (long long kk = 0; kk < bound; kk++) {
                double dot = 0;
                for (size_t d = 0; d < D; d++)
                    dot += (double)ld(q, qo + d, dtype) * (double)ld(k, (bhkv * Sk + (size_t)kk) * D + d, dtype);
                p[kk] = dot * scale;
                if (p[kk] > mx) mx = p[kk];
            }
            double den = 0;
            for (long long kk = 0; kk < bound; kk++) { p[kk] = exp(p[kk] - mx); den += p[kk]; }
            for (size_t d = 0; d < D; d++) {
                double acc = 0;
                for (long long kk = 0; kk < bound; kk++)
                    acc += p[kk] * (double)ld(v, (bhkv * Sk + (size_t)kk) * D + d, dtype);
                out[qo + d] = acc / den;
            }
        }
    free(p);
}

/* ------------------------------------------------------------------ A6 / A7 */
void orc_kv_cache_update(void *cache, const void *new_kv, long long offset, size_t BH, size_t S_new,
                         size_t max_seq, size_t D, size_t eb) {
    for (size_t bh = 0; bh < BH; bh++)
        for (size_t t = 0; t < S_new; t++)
            memcpy((char *)cache + ((bh * max_seq + (size_t)offset + t) * D) * eb,
                   (const char *)new_kv + ((bh * S_new + t) * D) * eb, D * eb);
}

void orc_quantizing_kv_cache_update(int8_t *cache, void *scale, const void *new_kv, long long offset,
                                    size_t BH, size_t S_new, size_t max_seq, size_t D, int dtype) {
    for (size_t bh = 0; bh < BH; bh++)
        for (size_t t = 0; t < S_new; t++) {
            size_t src = (bh * S_new + t) * D;
            size_t tok = bh * max_seq + (size_t)offset + t;
            float amax = 0.0f;
            for (size_t d = 0; d < D; d++) {
                float x = ld(new_kv, src + d, dtype);
                /* |x| as max(x, -x) in the reference; for x = +0 the sign of that maximum is
                 * unspecified (maxnum), so the restatement takes fabsf and a zero row has scale +0 */
                amax = fmaxf(amax, fabsf(x));
            }
            float s = amax * (1.0f / 127.0f);
            float inv = amax == 0.0f ? 0.0f : 127.0f / amax;
            st(scale, tok, s, dtype);
            for (size_t d = 0; d < D; d++) {
                float sc = ld(new_kv, src + d, dtype) * inv;
                float biased = sc + (sc >= 0.0f ? 0.5f : -0.5f);
                int32_t qi = (int32_t)biased; /* fptosi: truncates toward zero */
                qi = qi < -128 ? -128 : (qi > 127 ? 127 : qi);
                cache[tok * D + d] = (int8_t)qi;
            }
        }
}

/* ------------------------------------------------------------------ A8 */
void orc_rms_norm(void *out, const void *x, const void *w, size_t rows, size_t dim, double eps,
                  int dtype) {
    const int L = g_lanes;
    for (size_t r = 0; r < rows; r++) {
        float acc[MAXL];
        for (int j = 0; j < L; j++) acc[j] = 0.0f;
        for (size_t i = 0; i < dim; i++) {
            float v = ld(x, r * dim + i, dtype);
            acc[i % (size_t)L] = acc[i % (size_t)L] + v * v;
        }
        float sumsq = tree(acc, L);
        float mean = sumsq / (float)dim;
        float inv = 1.0f / sqrtf(mean + (float)eps);
        for (size_t i = 0; i < dim; i++) {
            float scaled = ld(x, r * dim + i, dtype) * inv;
            st(out, r * dim + i, scaled * ld(w, i, dtype), dtype);
        }
    }
}

/* ------------------------------------------------------------------ A9 */
/* The reference keeps initializer values as f64 and narrows them when the typed buffer is
 * made: f64 -> f32 (RNE), and for bf16 the f32 is then TRUNCATED to its top 16 bits
 * (src/session.rs:160-178, `(x as f32).to_bits() >> 16`).  fp16 has no counterpart there and
 * rounds to nearest even. */
static inline void st_init(void *p, size_t i, double v, int dt) {
    float f = (float)v;
    if (dt == ORC_BF16) ((uint16_t *)p)[i] = (uint16_t)(f2u(f) >> 16);
    else st(p, i, f, dt);
}
void orc_rope_table(void *cos_t, void *sin_t, size_t max_seq, size_t D, float base, int dtype) {
    size_t half = D / 2;
    double *inv = (double *)malloc((half ? half : 1) * sizeof(double));
    for (size_t i = 0; i < half; i++) inv[i] = 1.0 / pow((double)base, 2.0 * (double)i / (double)D);
    for (size_t p = 0; p < max_seq; p++)
        for (size_t j = 0; j < D; j++) {
            double ang = (double)p * inv[j % half];
            st_init(cos_t, p * D + j, cos(ang), dtype);
            st_init(sin_t, p * D + j, sin(ang), dtype);
        }
    free(inv);
}

void orc_rope(void *out, const void *x, const void *cos_t, const void *sin_t, const int64_t *position,
              size_t outer, size_t S, size_t D, int dtype) {
    size_t half = D / 2;
    for (size_t o = 0; o < outer; o++)
        for (size_t s = 0; s < S; s++) {
            size_t row = (o * S + s) * D, tab = (size_t)position[s] * D;
            for (size_t j = 0; j < half; j++) {
                float xl = ld(x, row + j, dtype), xh = ld(x, row + j + half, dtype);
                float cl = ld(cos_t, tab + j, dtype), ch = ld(cos_t, tab + j + half, dtype);
                float sl = ld(sin_t, tab + j, dtype), sh = ld(sin_t, tab + j + half, dtype);
                float lo = xl * cl - xh * sl;
                float hi = xh * ch + xl * sh;
                st(out, row + j, lo, dtype);
                st(out, row + j + half, hi, dtype);
            }
        }
}

/* ------------------------------------------------------------------ A10 / A11 / A13 */
void orc_gather_rows(void *out, const void *data, const int64_t *idx, size_t n_idx, size_t rows,
                     size_t row_bytes) {
    for (size_t i = 0; i < n_idx; i++) {
        int64_t r = idx[i];
        if (r < 0) r += (int64_t)rows;
        memcpy((char *)out + i * row_bytes, (const char *)data + (size_t)r * row_bytes, row_bytes);
    }
}
static inline float swish1(float x) {
    float den = 1.0f + expf(-x);
    float sig = 1.0f / den;
    return x * sig;
}
void orc_swish(void *out, const void *x, size_t n, int dtype) {
    for (size_t i = 0; i < n; i++) st(out, i, swish1(ld(x, i, dtype)), dtype);
}
void orc_swiglu(void *out, const void *gate, const void *up, size_t n, int dtype) {
    for (size_t i = 0; i < n; i++) st(out, i, swish1(ld(gate, i, dtype)) * ld(up, i, dtype), dtype);
}
void orc_add(void *out, const void *a, const void *b, size_t n, int dtype) {
    for (size_t i = 0; i < n; i++) st(out, i, ld(a, i, dtype) + ld(b, i, dtype), dtype);
}
int64_t orc_argmax_last(const void *logits, size_t n, int dtype) {
    /* Iterator::max_by keeps the last of equal maxima */
    int64_t best = 0;
    float bv = ld(logits, 0, dtype);
    for (size_t i = 1; i < n; i++) {
        float v = ld(logits, i, dtype);
        if (v >= bv) { bv = v; best = (int64_t)i; }
    }
    return best;
}

/* ------------------------------------------------------------------ A14 */
void orc_quantize_per_channel(int8_t *q, void *scale, const float *w, size_t rows, size_t cols,
                              int scale_dtype) {
    for (size_t r = 0; r < rows; r++) {
        float amax = 0.0f;
        for (size_t c = 0; c < cols; c++) amax = fmaxf(amax, fabsf(w[r * cols + c]));
        float s = amax == 0.0f ? 1.0f : amax / 127.0f;
        for (size_t c = 0; c < cols; c++) {
            float v = round_half_away(w[r * cols + c] / s);
            v = v < -128.0f ? -128.0f : (v > 127.0f ? 127.0f : v);
            q[r * cols + c] = (int8_t)v;
        }
        st(scale, r, s, scale_dtype);
    }
}

/* ------------------------------------------------------------------ streaming helpers */
int orc_ring_phys_index(int rank, int sink, int window, int start) {
    if (window == 0 || rank < sink) return rank;
    int rel = start + (rank - sink);
    rel %= window;
    return sink + rel;
}
void orc_streaming_kv_position(int64_t *out, size_t sink, size_t window, size_t stream_pos,
                               size_t max_seq) {
    size_t max_active = sink + window;
    size_t ring_start = stream_pos < max_active ? 0 : (stream_pos - sink) % window;
    size_t in_ring = stream_pos > sink ? stream_pos - sink : 0;
    if (in_ring > window) in_ring = window;
    for (size_t slot = 0; slot < max_seq; slot++) {
        if (slot < sink) out[slot] = (int64_t)slot;
        else if (slot < max_active) {
            size_t rel_age = (slot - sink + window - ring_start) % window;
            out[slot] = rel_age < in_ring ? (int64_t)(sink + rel_age) : (int64_t)slot;
        } else out[slot] = (int64_t)slot;
    }
}

/* KVCacheUpdate / QuantizingKVCacheUpdate with the ring inputs (cuda kvcache_update.cuh:12-26,
 * quantizing_kvcache_update.cuh:24-36): row t of new_kv goes to cache row ring_phys_index(offset + t), rows in
 * increasing t, so a later row wins a shared slot.  `offset` is the session's unbounded stream position
 * (session.rs:541, 573), which the map folds into the ring with the session's ring_start -- past sink + window
 * that is slot sink + (ring_start + offset + t - sink) % window, whatever that slot holds.  The quantiser is the
 * one of orc_quantizing_kv_cache_update (the CPU backend's rounding, which the library follows everywhere; the
 * CUDA kernel's roundf(x * (1/s)) differs from it in the last code of some values). */
void orc_kv_cache_update_ring(void *cache, const void *new_kv, long long offset, size_t BH, size_t S_new,
                              size_t max_seq, size_t D, size_t eb, int sink, int window, int start) {
    for (size_t bh = 0; bh < BH; bh++)
        for (size_t t = 0; t < S_new; t++) {
            size_t slot = (size_t)orc_ring_phys_index((int)(offset + (long long)t), sink, window, start);
            memcpy((char *)cache + ((bh * max_seq + slot) * D) * eb,
                   (const char *)new_kv + ((bh * S_new + t) * D) * eb, D * eb);
        }
}
void orc_quantizing_kv_cache_update_ring(int8_t *cache, void *scale, const void *new_kv, long long offset,
                                         size_t BH, size_t S_new, size_t max_seq, size_t D, int dtype,
                                         int sink, int window, int start) {
    size_t eb = esize(dtype);
    int8_t *row = (int8_t *)malloc(D);
    char sc[4];
    for (size_t bh = 0; bh < BH; bh++)
        for (size_t t = 0; t < S_new; t++) {
            size_t slot = (size_t)orc_ring_phys_index((int)(offset + (long long)t), sink, window, start);
            /* one row through the plain quantiser into a one-row cache, then placed */
            orc_quantizing_kv_cache_update(row, sc, (const char *)new_kv + ((bh * S_new + t) * D) * eb, 0, 1, 1, 1, D, dtype);
            memcpy(cache + (bh * max_seq + slot) * D, row, D);
            memcpy((char *)scale + (bh * max_seq + slot) * eb, sc, eb);
        }
    free(row);
}

/* Attention over the sink + ring layout, as the CUDA kernels enumerate it (attention.cuh:495-606 decode,
 * 100-200 / 386-420 tiled): keys by recency rank r = 0 .. bound-1, the key of rank r is cache row
 * ring_phys_index(r); causal rule in ranks, r <= (active - Sq) + query row (cuda.rs:1360-1364).
 * kv_position != NULL: the dequantised key is rotated (half-split) by table row kv_position[r] -- indexed by
 * RANK, as the kernels do (attention.cuh:163, 416, 560), although the session fills the table by slot
 * (session.rs:604-635); everything in f32.  int8 K/V: score = (q . (code * k_scale rotated)) * scale,
 * weight * v_scale before it meets the V codes (attention.cuh:549-598). */
void orc_attention_ring(void *out, const void *q, const void *k, const void *v, const void *k_scale,
                        const void *v_scale, long long active, size_t B, size_t Hq, size_t Hkv, size_t Sq,
                        size_t Sk, size_t D, int is_causal, float scale, int dtype, int kv_int8, int sink,
                        int window, int start, const void *cos_t, const void *sin_t, const int64_t *kv_position) {
    long long past = active - (long long)Sq;
    size_t group = Hq / Hkv, half = D / 2;
    float *o = (float *)malloc(D * sizeof(float)), *kr = (float *)malloc(D * sizeof(float));
    for (size_t bh = 0; bh < B * Hq; bh++)
        for (size_t sq = 0; sq < Sq; sq++) {
            size_t b = bh / Hq, h = bh % Hq, bhkv = b * Hkv + h / group;
            size_t qo = (bh * Sq + sq) * D;
            long long bound = active;
            if (is_causal && past + (long long)sq + 1 < bound) bound = past + (long long)sq + 1;
            for (size_t d = 0; d < D; d++) o[d] = 0.0f;
            float m = -INFINITY, s = 0.0f;
            for (long long r = 0; r < bound; r++) {
                size_t tok = bhkv * Sk + (size_t)orc_ring_phys_index((int)r, sink, window, start);
                float ks = kv_int8 ? ld(k_scale, tok, dtype) : 1.0f;
                for (size_t d = 0; d < D; d++) kr[d] = kv_ld(k, tok * D + d, dtype, kv_int8) * ks;
                float sum = 0.0f;
                if (kv_position) {
                    size_t tab = (size_t)kv_position[r] * D;
                    for (size_t d = 0; d < D; d++) {
                        float kp = d < half ? kr[d + half] : kr[d - half];
                        float sign = d < half ? -1.0f : 1.0f;
                        float rot = kr[d] * ld(cos_t, tab + d, dtype) + (sign * kp) * ld(sin_t, tab + d, dtype);
                        sum = sum + ld(q, qo + d, dtype) * rot;
                    }
                } else {
                    for (size_t d = 0; d < D; d++) sum = sum + ld(q, qo + d, dtype) * kr[d];
                }
                float qk = sum * scale;
                float m_new = fmaxf(m, qk);
                float factor = expf(m - m_new);
                float e = expf(qk - m_new);
                s = s * factor + e;
                float e_eff = kv_int8 ? e * ld(v_scale, tok, dtype) : e;
                for (size_t d = 0; d < D; d++) o[d] = o[d] * factor + e_eff * kv_ld(v, tok * D + d, dtype, kv_int8);
                m = m_new;
            }
            for (size_t d = 0; d < D; d++) st(out, qo + d, o[d] / s, dtype);
        }
    free(o); free(kr);
}

/* ------------------------------------------------------------------ A12 / A13 decoder */
struct orc_layer {
    orc_linear lin[7];
    const void *bias[3]; /* q, k, v projection bias [N] in dtype, or NULL (decoder.rs:167-184, 542-600: qwen2) */
    const void *norm[2];
    void *k_cache, *v_cache; /* [Hkv, max_seq, D] dtype, or int8 with quant_kv_cache */
    void *k_scale, *v_scale; /* quant_kv_cache: [Hkv, max_seq] dtype */
};
struct orc_model {
    orc_model_cfg cfg;
    orc_linear embed, lm_head;
    const void *final_norm;
    struct orc_layer *layers;
    void *cos_t, *sin_t;
    long long past_len;
    int gemm_mode; /* -1: CPU backend's dispatch; 2: CUDA backend's (M >= 16 -> W rounded first) */
    int quant_kv_cache;       /* BuildOptions::quant_kv_cache (decoder.rs:672, 405-470) */
    int quantize_activations; /* Options::quantize_activations (transform/optimize/quantize_activations.rs) */
    int streaming, sink, window; /* BuildOptions::streaming_kv + DecodeKind::LlamaStreaming { sink, window } */
    void *last_hidden;
    size_t last_S;
};

orc_model *orc_model_create(const orc_model_cfg *cfg) {
    orc_model *m = (orc_model *)calloc(1, sizeof(orc_model));
    m->cfg = *cfg;
    m->gemm_mode = -1;
    size_t eb = esize(cfg->dtype);
    m->layers = (struct orc_layer *)calloc((size_t)cfg->n_layers, sizeof(struct orc_layer));
    size_t kvn = (size_t)cfg->n_kv_heads * (size_t)cfg->max_seq * (size_t)cfg->head_dim;
    for (int l = 0; l < cfg->n_layers; l++) {
        /* session state buffers start zeroed (src/session.rs:284-394) */
        m->layers[l].k_cache = calloc(kvn, eb);
        m->layers[l].v_cache = calloc(kvn, eb);
    }
    m->cos_t = malloc((size_t)cfg->max_seq * (size_t)cfg->head_dim * eb);
    m->sin_t = malloc((size_t)cfg->max_seq * (size_t)cfg->head_dim * eb);
    orc_rope_table(m->cos_t, m->sin_t, (size_t)cfg->max_seq, (size_t)cfg->head_dim, cfg->rope_theta,
                   cfg->dtype);
    return m;
}
void orc_model_destroy(orc_model *m) {
    if (!m) return;
    for (int l = 0; l < m->cfg.n_layers; l++) {
        free(m->layers[l].k_cache); free(m->layers[l].v_cache);
        free(m->layers[l].k_scale); free(m->layers[l].v_scale);
    }
    free(m->layers); free(m->cos_t); free(m->sin_t); free(m->last_hidden); free(m);
}
void orc_model_set_embed(orc_model *m, orc_linear w) { m->embed = w; }
void orc_model_set_lm_head(orc_model *m, orc_linear w) { m->lm_head = w; }
void orc_model_set_final_norm(orc_model *m, const void *w) { m->final_norm = w; }
void orc_model_set_linear(orc_model *m, int layer, int which, orc_linear w) { m->layers[layer].lin[which] = w; }
void orc_model_set_norm(orc_model *m, int layer, int which, const void *w) { m->layers[layer].norm[which] = w; }
/* which: 0 q, 1 k, 2 v */
void orc_model_set_bias(orc_model *m, int layer, int which, const void *b) { m->layers[layer].bias[which] = b; }
void orc_model_reset(orc_model *m) { m->past_len = 0; }
void orc_model_set_gemm_mode(orc_model *m, int mode) { m->gemm_mode = mode; }
/* must be called before the first forward: the caches change element type */
void orc_model_set_options(orc_model *m, int quant_kv_cache, int quantize_activations) {
    m->quant_kv_cache = quant_kv_cache;
    m->quantize_activations = quantize_activations;
    size_t rows = (size_t)m->cfg.n_kv_heads * (size_t)m->cfg.max_seq;
    for (int l = 0; l < m->cfg.n_layers && quant_kv_cache; l++) {
        struct orc_layer *L = &m->layers[l];
        free(L->k_cache); free(L->v_cache); free(L->k_scale); free(L->v_scale);
        L->k_cache = calloc(rows * (size_t)m->cfg.head_dim, 1);
        L->v_cache = calloc(rows * (size_t)m->cfg.head_dim, 1);
        L->k_scale = calloc(rows, esize(m->cfg.dtype));
        L->v_scale = calloc(rows, esize(m->cfg.dtype));
    }
}
const void *orc_model_k_scale(const orc_model *m, int layer) { return m->layers[layer].k_scale; }
const void *orc_model_v_scale(const orc_model *m, int layer) { return m->layers[layer].v_scale; }
long long orc_model_past_len(const orc_model *m) { return m->past_len; }
void orc_model_set_past_len(orc_model *m, long long p) { m->past_len = p; }
const void *orc_model_k_cache(const orc_model *m, int layer) { return m->layers[layer].k_cache; }
const void *orc_model_v_cache(const orc_model *m, int layer) { return m->layers[layer].v_cache; }
const void *orc_model_last_hidden(const orc_model *m) { return m->last_hidden; }

/* x [S,K] -> out [S,N]; DequantMatMul for int8 weights (CPU dispatch: M==1 fused decode, else
 * dequantise + sgemm), Gemm(trans_b) for plain weights */
static void linear(const orc_model *m, void *out, const void *x, const orc_linear *w, size_t S,
                   size_t N, size_t K) {
    int dt = m->cfg.dtype;
    if (w->q && m->quantize_activations && K % 32 == 0) {
        /* DequantMatMul -> DynamicQuantizeLinear(axis 0, symmetric) + QuantizedMatMul
         * (quantize_activations.rs:63-84, 121-183); re-quantising a shared activation per
         * consumer gives the same int8 rows as the pass's cached value */
        int8_t *a8 = (int8_t *)malloc(S * K);
        void *as = malloc(S * esize(dt));
        orc_dynquant_i8(a8, as, x, S, K, dt);
        orc_quantized_matmul(out, NULL, a8, as, w->q, w->scale, S, N, K, dt);
        free(a8); free(as);
        return;
    }
    if (w->q) {
        /* kernel choice per backend: CPU (translator.rs:3002-3115) M==1 fused decode else
         * dequantise+sgemm; CUDA (cuda.rs:1518-1652) M>=16 && K%8==0 tensor cores else
         * scale-after-sum */
        int mode = m->gemm_mode == 2 ? ((S >= 16 && K % 8 == 0 && dt != ORC_F32) ? 2 : 0) : -1;
        orc_dequant_matmul(out, x, w->q, w->scale, S, N, K, dt, dt, mode);
    } else {
        float *a = widen(x, S * K, dt);
        int nt = nthreads_for(N);
        (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt) if (nt > 1)
        for (long long n = 0; n < (long long)N; n++) {
            float *wr = widen((const char *)w->w + (size_t)n * K * esize(dt), K, dt);
            for (size_t s = 0; s < S; s++) st(out, s * N + (size_t)n, dot_f32_f32(a + s * K, wr, K), dt);
            free(wr);
        }
        free(a);
    }
}

/* Add(matmul output [S,N], bias [N]) in place: the `{node}_bias` node of decoder.rs:167-184 -- the projection is
 * stored in dtype first (it is the MatMul node's output), then the broadcast Add rounds once more */
static void add_bias(void *y, const void *bias, size_t S, size_t N, int dt) {
    if (!bias) return;
    for (size_t s = 0; s < S; s++)
        for (size_t n = 0; n < N; n++) st(y, s * N + n, ld(y, s * N + n, dt) + ld(bias, n, dt), dt);
}

/* [S, H, D] -> [H, S, D] (reshape + Transpose[0,2,1,3], decoder.rs:253-275) */
static void to_heads(void *dst, const void *src, size_t S, size_t H, size_t D, size_t eb) {
    for (size_t s = 0; s < S; s++)
        for (size_t h = 0; h < H; h++)
            memcpy((char *)dst + ((h * S + s) * D) * eb, (const char *)src + ((s * H + h) * D) * eb, D * eb);
}
static void from_heads(void *dst, const void *src, size_t S, size_t H, size_t D, size_t eb) {
    for (size_t s = 0; s < S; s++)
        for (size_t h = 0; h < H; h++)
            memcpy((char *)dst + ((s * H + h) * D) * eb, (const char *)src + ((h * S + s) * D) * eb, D * eb);
}

/* ring != NULL: the streaming graph (decoder.rs:281-347, 472-487) -- RoPE(q) by `positions`; k and v go
 * UN-ROTATED into the caches through the slot map; 16-bit KV: Rope over the whole K cache by kv_position (one
 * table row per cache SLOT, result rounded to dtype: it is a graph value), then Attention with the ring inputs;
 * int8 KV: Attention rotates the dequantised keys itself, by kv_position[rank]. */
typedef struct { int sink, window, start; const int64_t *kv_position; } orc_ring;
static void forward_impl(orc_model *m, const int64_t *ids, const int64_t *positions, size_t S,
                         long long past_len, long long active, int is_causal, const orc_ring *ring, void *logits) {
    const orc_model_cfg *c = &m->cfg;
    const int dt = c->dtype;
    const size_t eb = esize(dt);
    const size_t H = (size_t)c->hidden, Hq = (size_t)c->n_heads, Hkv = (size_t)c->n_kv_heads;
    const size_t D = (size_t)c->head_dim, F = (size_t)c->ffn, V = (size_t)c->vocab;
    const size_t QD = Hq * D, KD = Hkv * D;
    void *x = malloc(S * H * eb), *n1 = malloc(S * H * eb), *x2 = malloc(S * H * eb);
    void *qb = malloc(S * QD * eb), *kb = malloc(S * KD * eb), *vb = malloc(S * KD * eb);
    void *qh = malloc(S * QD * eb), *kh = malloc(S * KD * eb), *vh = malloc(S * KD * eb);
    void *qr = malloc(S * QD * eb), *kr = malloc(S * KD * eb);
    void *ao = malloc(S * QD * eb), *ab = malloc(S * QD * eb), *ob = malloc(S * H * eb);
    void *g = malloc(S * F * eb), *u = malloc(S * F * eb), *hmid = malloc(S * F * eb);
    void *dn = malloc(S * H * eb);

    /* embed: DequantizeLinear(table) -> Gather(ids) (decoder.rs:824-835) */
    for (size_t s = 0; s < S; s++) {
        int64_t id = ids[s];
        if (id < 0) id += (int64_t)V;
        if (m->embed.q) {
            float sc = ld(m->embed.scale, (size_t)id, dt);
            for (size_t i = 0; i < H; i++) st(x, s * H + i, (float)m->embed.q[(size_t)id * H + i] * sc, dt);
        } else {
            memcpy((char *)x + s * H * eb, (const char *)m->embed.w + (size_t)id * H * eb, H * eb);
        }
    }
    float scale = 1.0f / sqrtf((float)D); /* (head_dim as f32).sqrt().recip(), decoder.rs:303 */
    for (int l = 0; l < c->n_layers; l++) {
        struct orc_layer *L = &m->layers[l];
        orc_rms_norm(n1, x, L->norm[0], S, H, c->eps, dt);
        linear(m, qb, n1, &L->lin[0], S, QD, H);
        linear(m, kb, n1, &L->lin[1], S, KD, H);
        linear(m, vb, n1, &L->lin[2], S, KD, H);
        add_bias(qb, L->bias[0], S, QD, dt);
        add_bias(kb, L->bias[1], S, KD, dt);
        add_bias(vb, L->bias[2], S, KD, dt);
        to_heads(qh, qb, S, Hq, D, eb);
        to_heads(kh, kb, S, Hkv, D, eb);
        to_heads(vh, vb, S, Hkv, D, eb);
        orc_rope(qr, qh, m->cos_t, m->sin_t, positions, Hq, S, D, dt);
        if (ring) {
            const size_t MS = (size_t)c->max_seq;
            if (m->quant_kv_cache) {
                orc_quantizing_kv_cache_update_ring((int8_t *)L->k_cache, L->k_scale, kh, past_len, Hkv, S, MS, D, dt,
                                                    ring->sink, ring->window, ring->start);
                orc_quantizing_kv_cache_update_ring((int8_t *)L->v_cache, L->v_scale, vh, past_len, Hkv, S, MS, D, dt,
                                                    ring->sink, ring->window, ring->start);
                orc_attention_ring(ao, qr, L->k_cache, L->v_cache, L->k_scale, L->v_scale, active, 1, Hq, Hkv, S, MS, D,
                                   is_causal, scale, dt, 1, ring->sink, ring->window, ring->start, m->cos_t, m->sin_t,
                                   ring->kv_position);
            } else {
                orc_kv_cache_update_ring(L->k_cache, kh, past_len, Hkv, S, MS, D, eb, ring->sink, ring->window, ring->start);
                orc_kv_cache_update_ring(L->v_cache, vh, past_len, Hkv, S, MS, D, eb, ring->sink, ring->window, ring->start);
                void *krot = malloc(Hkv * MS * D * eb);
                orc_rope(krot, L->k_cache, m->cos_t, m->sin_t, ring->kv_position, Hkv, MS, D, dt);
                orc_attention_ring(ao, qr, krot, L->v_cache, NULL, NULL, active, 1, Hq, Hkv, S, MS, D, is_causal, scale,
                                   dt, 0, ring->sink, ring->window, ring->start, NULL, NULL, NULL);
                free(krot);
            }
        } else {
        orc_rope(kr, kh, m->cos_t, m->sin_t, positions, Hkv, S, D, dt);
        if (m->quant_kv_cache) {
            orc_quantizing_kv_cache_update((int8_t *)L->k_cache, L->k_scale, kr, past_len, Hkv, S, (size_t)c->max_seq, D, dt);
            orc_quantizing_kv_cache_update((int8_t *)L->v_cache, L->v_scale, vh, past_len, Hkv, S, (size_t)c->max_seq, D, dt);
            orc_attention(ao, qr, L->k_cache, L->v_cache, L->k_scale, L->v_scale, active, 1, Hq, Hkv, S,
                          (size_t)c->max_seq, D, is_causal, scale, dt, 1);
        } else {
            orc_kv_cache_update(L->k_cache, kr, past_len, Hkv, S, (size_t)c->max_seq, D, eb);
            orc_kv_cache_update(L->v_cache, vh, past_len, Hkv, S, (size_t)c->max_seq, D, eb);
            orc_attention(ao, qr, L->k_cache, L->v_cache, NULL, NULL, active, 1, Hq, Hkv, S,
                          (size_t)c->max_seq, D, is_causal, scale, dt, 0);
        }
        }
        from_heads(ab, ao, S, Hq, D, eb);
        linear(m, ob, ab, &L->lin[3], S, H, QD);
        orc_add(x2, x, ob, S * H, dt);                 /* attn residual */
        orc_rms_norm(n1, x2, L->norm[1], S, H, c->eps, dt);
        linear(m, g, n1, &L->lin[4], S, F, H);
        linear(m, u, n1, &L->lin[5], S, F, H);
        orc_swiglu(hmid, g, u, S * F, dt);
        linear(m, dn, hmid, &L->lin[6], S, H, F);
        orc_add(x, x2, dn, S * H, dt);                 /* mlp residual */
    }
    free(m->last_hidden);
    m->last_hidden = malloc(S * H * eb);
    memcpy(m->last_hidden, x, S * H * eb);
    m->last_S = S;
    orc_rms_norm(n1, x, m->final_norm, S, H, c->eps, dt);
    linear(m, logits, n1, &m->lm_head, S, V, H);
    free(x); free(n1); free(x2); free(qb); free(kb); free(vb); free(qh); free(kh); free(vh);
    free(qr); free(kr); free(ao); free(ab); free(ob); free(g); free(u); free(hmid); free(dn);
}

void orc_model_forward(orc_model *m, const int64_t *ids, const int64_t *positions, size_t S,
                       long long past_len, long long active, int is_causal, void *logits) {
    forward_impl(m, ids, positions, S, past_len, active, is_causal, NULL, logits);
}
void orc_model_forward_streaming(orc_model *m, const int64_t *ids, const int64_t *positions, size_t S,
                                 long long past_len, long long active, int is_causal, int sink, int window,
                                 int ring_start, const int64_t *kv_position, void *logits) {
    orc_ring ring = {sink, window, ring_start, kv_position};
    forward_impl(m, ids, positions, S, past_len, active, is_causal, &ring, logits);
}
void orc_model_set_streaming(orc_model *m, int sink, int window) {
    m->streaming = window > 0;
    m->sink = sink;
    m->window = window;
}

/* streaming_decode_inputs (session.rs:571-597) */
static void streaming_decode(orc_model *m, int64_t token, void *logits) {
    long long max_active = m->sink + m->window, sp = m->past_len;
    int64_t qpos = sp < max_active - 1 ? sp : max_active - 1;
    long long active = sp + 1 < max_active ? sp + 1 : max_active;
    int ring_start = sp < max_active ? 0 : (int)((sp - m->sink) % m->window);
    int64_t *kvpos = (int64_t *)malloc((size_t)m->cfg.max_seq * sizeof(int64_t));
    orc_streaming_kv_position(kvpos, (size_t)m->sink, (size_t)m->window, (size_t)sp, (size_t)m->cfg.max_seq);
    orc_model_forward_streaming(m, &token, &qpos, 1, sp, active, 0, m->sink, m->window, ring_start, kvpos, logits);
    free(kvpos);
}

int64_t orc_model_decode_step(orc_model *m, int64_t token) {
    size_t V = (size_t)m->cfg.vocab;
    void *logits = malloc(V * esize(m->cfg.dtype));
    int64_t pos = m->past_len;
    if (m->streaming) streaming_decode(m, token, logits);
    else
    orc_model_forward(m, &token, &pos, 1, m->past_len, m->past_len + 1, 0, logits);
    int64_t next = orc_argmax_last(logits, V, m->cfg.dtype);
    free(logits);
    m->past_len += 1;
    return next;
}

int64_t orc_model_prefill(orc_model *m, const int64_t *ids, size_t n, size_t P) {
    size_t V = (size_t)m->cfg.vocab, eb = esize(m->cfg.dtype);
    void *logits = malloc(P * V * eb);
    int64_t *padded = (int64_t *)malloc(P * sizeof(int64_t)), *pos = (int64_t *)malloc(P * sizeof(int64_t));
    int64_t result = -1;
    while (n > 0) {
        size_t chunk = n < P ? n : P;
        for (size_t i = 0; i < P; i++) { padded[i] = i < chunk ? ids[i] : 0; pos[i] = m->past_len + (int64_t)i; }
        if (m->streaming) {
            /* streaming_prefill_inputs (session.rs:539-569) */
            long long max_active = m->sink + m->window, sp = m->past_len, after = sp + (long long)P;
            for (size_t i = 0; i < P; i++) pos[i] = sp + (long long)i < max_active - 1 ? sp + (long long)i : max_active - 1;
            int ring_start = after <= max_active ? 0 : (int)((after - m->sink) % m->window);
            int64_t *kvpos = (int64_t *)malloc((size_t)m->cfg.max_seq * sizeof(int64_t));
            orc_streaming_kv_position(kvpos, (size_t)m->sink, (size_t)m->window, (size_t)after, (size_t)m->cfg.max_seq);
            orc_model_forward_streaming(m, padded, pos, P, sp, after < max_active ? after : max_active, 1, m->sink,
                                        m->window, ring_start, kvpos, logits);
            free(kvpos);
        } else
        orc_model_forward(m, padded, pos, P, m->past_len, m->past_len + (long long)P, 1, logits);
        m->past_len += (long long)chunk;
        if (chunk == n) result = orc_argmax_last((const char *)logits + (chunk - 1) * V * eb, V, m->cfg.dtype);
        ids += chunk;
        n -= chunk;
    }
    free(logits); free(padded); free(pos);
    return result;
}

long long orc_model_generate(orc_model *m, const int64_t *prompt, size_t n_prompt, size_t max_new,
                             size_t prefill_len, int64_t eos, int64_t *out) {
    if (n_prompt == 0) return 0;
    long long max_seq = m->cfg.max_seq;
    long long needed = prefill_len
        ? m->past_len + (long long)(((n_prompt + prefill_len - 1) / prefill_len) * prefill_len)
        : m->past_len + (long long)n_prompt;
    if (!m->streaming && max_seq < needed) return -1; /* PromptTooLong (not checked in streaming mode, session.rs:357) */
    long long n_new = 0;
    for (size_t i = 0; i < max_new; i++) {
        if (!m->streaming && max_seq < m->past_len + 1) break;
        int64_t tok;
        if (i == 0) {
            if (prefill_len) tok = orc_model_prefill(m, prompt, n_prompt, prefill_len);
            else {
                tok = 0;
                for (size_t j = 0; j < n_prompt; j++) tok = orc_model_decode_step(m, prompt[j]);
            }
        } else tok = orc_model_decode_step(m, out[n_new - 1]);
        out[n_new++] = tok;
        if (tok == eos) break;
    }
    return n_new;
}
