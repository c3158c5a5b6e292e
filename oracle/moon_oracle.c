/*
 * moon_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE (see moon_oracle.h).
 *
 * CPU restatement of moondream-zig's FP16 matmul / attention arithmetic.
 * Build: gcc -O2 -ffp-contract=off -mavx2 -mfma -mf16c -fopenmp -shared -fPIC
 * (-ffp-contract=off keeps every f32 multiply and add a separate IEEE op, so the
 * result does not depend on the compiler's contraction choices).
 */
#include "moon_oracle.h"

#include <immintrin.h>
#include <math.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* ------------------------------------------------------------------ f16 <-> f32 */
/* tensor.zig:258-281: vcvtph2ps / vcvtps2ph with imm 0 = round to nearest even. */
float orc_h2f(orc_f16 h) { return _cvtsh_ss(h); }
orc_f16 orc_f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }

void orc_cast_f16_to_f32(const orc_f16 *src, float *dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_h2f(src[i]);
}
void orc_cast_f32_to_f16(const float *src, orc_f16 *dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_f2h(src[i]);
}

/* ------------------------------------------------------------------ synthetic data */
static inline uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline uint64_t stream_key(uint64_t seed, uint64_t stream) {
    return mix64(mix64(seed + 0x9E3779B97F4A7C15ull) ^ (stream * 0xD1B54A32D192ED03ull + 0x2545F4914F6CDD1Dull));
}
static inline uint64_t counter_word(uint64_t key, uint64_t ctr) {
    return mix64(key + 0x9E3779B97F4A7C15ull * (ctr + 1));
}
static inline int32_t centred_sum8(uint64_t a, uint64_t b) {
    uint32_t s = 0;
    for (int i = 0; i < 4; i++) {
        s += (uint32_t)((a >> (16 * i)) & 0xFFFF);
        s += (uint32_t)((b >> (16 * i)) & 0xFFFF);
    }
    return (int32_t)s - 262140; /* 8 * 32767.5 */
}

void orc_fill_normal_f16(orc_f16 *dst, size_t n, uint64_t seed, uint64_t stream, float std_dev) {
    const uint64_t key = stream_key(seed, stream);
    const float scale = std_dev * (1.0f / 53510.105f); /* sqrt(8*(65536^2-1)/12) */
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        int32_t c = centred_sum8(counter_word(key, 2 * i), counter_word(key, 2 * i + 1));
        dst[i] = orc_f2h((float)c * scale);
    }
}

void orc_fill_uniform_u32(uint32_t *dst, size_t n, uint64_t seed, uint64_t stream, uint32_t modulo) {
    const uint64_t key = stream_key(seed, stream);
    for (size_t i = 0; i < n; i++) dst[i] = (uint32_t)((counter_word(key, i) >> 32) % modulo);
}

/* ------------------------------------------------------------------ GEMM */
/* Sequential-k f32 accumulation for every output element (the reference's own
 * definition of the expected result, matmul_test.zig:83-106).  The j loop is
 * innermost so the compiler can vectorise across outputs without changing the
 * per-element order of additions. */
static void hgemm_nn_rows(const orc_f16 *A, const float *Bf, orc_f16 *C, size_t M, size_t N, size_t K) {
#pragma omp parallel
    {
        float *acc = (float *)malloc(N * sizeof(float));
#pragma omp for schedule(dynamic, 4)
        for (size_t m = 0; m < M; m++) {
            for (size_t j = 0; j < N; j++) acc[j] = 0.0f;
            for (size_t k = 0; k < K; k++) {
                const float a = orc_h2f(A[m * K + k]);
                const float *brow = Bf + k * N;
                for (size_t j = 0; j < N; j++) acc[j] = acc[j] + a * brow[j];
            }
            for (size_t j = 0; j < N; j++) C[m * N + j] = orc_f2h(acc[j]);
        }
        free(acc);
    }
}

void orc_hgemm_nn(const orc_f16 *A, const orc_f16 *B, orc_f16 *C, size_t M, size_t N, size_t K) {
    float *Bf = (float *)malloc(K * N * sizeof(float));
    orc_cast_f16_to_f32(B, Bf, K * N);
    hgemm_nn_rows(A, Bf, C, M, N, K);
    free(Bf);
}

void orc_hgemm_nt(const orc_f16 *A, const orc_f16 *Bt, orc_f16 *C, size_t M, size_t N, size_t K) {
    if (M <= 4) {
        /* GEMV-like: row n of Bt is contiguous (hgemm_trans.zig:59-116). */
        for (size_t m = 0; m < M; m++) {
#pragma omp parallel for schedule(static)
            for (size_t n = 0; n < N; n++) {
                float sum = 0.0f;
                const orc_f16 *row = Bt + n * K;
                for (size_t k = 0; k < K; k++) sum = sum + orc_h2f(A[m * K + k]) * orc_h2f(row[k]);
                C[m * N + n] = orc_f2h(sum);
            }
        }
        return;
    }
    float *Bf = (float *)malloc(K * N * sizeof(float));
#pragma omp parallel for schedule(static)
    for (size_t n = 0; n < N; n++)
        for (size_t k = 0; k < K; k++) Bf[k * N + n] = orc_h2f(Bt[n * K + k]);
    hgemm_nn_rows(A, Bf, C, M, N, K);
    free(Bf);
}

void orc_hgemm_nn_f64(const orc_f16 *A, const orc_f16 *B, orc_f16 *C, size_t M, size_t N, size_t K) {
#pragma omp parallel
    {
        double *acc = (double *)malloc(N * sizeof(double));
#pragma omp for schedule(dynamic, 4)
        for (size_t m = 0; m < M; m++) {
            for (size_t j = 0; j < N; j++) acc[j] = 0.0;
            for (size_t k = 0; k < K; k++) {
                const double a = orc_h2f(A[m * K + k]);
                for (size_t j = 0; j < N; j++) acc[j] += a * (double)orc_h2f(B[k * N + j]);
            }
            for (size_t j = 0; j < N; j++) C[m * N + j] = orc_f2h((float)acc[j]);
        }
        free(acc);
    }
}

void orc_hgemm_nt_f64(const orc_f16 *A, const orc_f16 *Bt, orc_f16 *C, size_t M, size_t N, size_t K) {
#pragma omp parallel for schedule(static) collapse(2)
    for (size_t m = 0; m < M; m++)
        for (size_t n = 0; n < N; n++) {
            double sum = 0.0;
            for (size_t k = 0; k < K; k++) sum += (double)orc_h2f(A[m * K + k]) * (double)orc_h2f(Bt[n * K + k]);
            C[m * N + n] = orc_f2h((float)sum);
        }
}

void orc_sgemm(const float *A, const float *B, float *C, size_t M, size_t N, size_t K) {
    for (size_t m = 0; m < M; m++) {
        float *c = C + m * N;
        for (size_t j = 0; j < N; j++) c[j] = 0.0f;
        for (size_t k = 0; k < K; k++) {
            const float a = A[m * K + k];
            const float *b = B + k * N;
            for (size_t j = 0; j < N; j++) c[j] = c[j] + a * b[j];
        }
    }
}

/* ------------------------------------------------------------------ elementwise */
void orc_bias_add(orc_f16 *a, const orc_f16 *b, size_t rows, size_t cols) {
    for (size_t r = 0; r < rows; r++)
        for (size_t j = 0; j < cols; j++) a[r * cols + j] = orc_f2h(orc_h2f(a[r * cols + j]) + orc_h2f(b[j]));
}

void orc_add(orc_f16 *a, const orc_f16 *b, size_t n) {
    /* f16 + f16 rounded to f16 == f16(f32(a)+f32(b)): the f32 sum of two f16 values is exact. */
    for (size_t i = 0; i < n; i++) a[i] = orc_f2h(orc_h2f(a[i]) + orc_h2f(b[i]));
}

void orc_gelu(orc_f16 *x, size_t n) {
    /* ops.zig:1641-1642: the constants are typed f16, i.e. rounded to f16 before use. */
    const float c = orc_h2f(orc_f2h(0.7978845608028654f)); /* 0.7978515625 */
    const float alpha = orc_h2f(orc_f2h(0.044715f));       /* 0.044708251953125 */
    for (size_t i = 0; i < n; i++) {
        const float v = orc_h2f(x[i]);
        const float cube = v * v * v;
        const float inner = c * (v + alpha * cube);
        const float t = tanhf(inner);
        x[i] = orc_f2h(0.5f * v * (1.0f + t));
    }
}

int orc_layernorm(const orc_f16 *x, const orc_f16 *gamma, const orc_f16 *beta, orc_f16 *y,
                  size_t rows, size_t dim, float eps) {
    if (!(eps > 0.0f)) return -1; /* ops.zig:1174 InvalidEpsilon */
    for (size_t r = 0; r < rows; r++) {
        const orc_f16 *xr = x + r * dim;
        /* mean and biased variance, as the reference's Welford pass delivers them in f32
         * (ops.zig:1209-1283); computed here in f64 and rounded once to f32. */
        double s = 0.0;
        for (size_t i = 0; i < dim; i++) s += orc_h2f(xr[i]);
        const double mean_d = s / (double)dim;
        double m2 = 0.0;
        for (size_t i = 0; i < dim; i++) {
            const double d = (double)orc_h2f(xr[i]) - mean_d;
            m2 += d * d;
        }
        const float mean = (float)mean_d;
        const float variance = (float)(m2 / (double)dim);
        const float std_dev = sqrtf(variance + eps);   /* ops.zig:1292 */
        const float rstd = 1.0f / std_dev;             /* :1300 */
        const float mean_rstd = mean * rstd;           /* :1301 */
        for (size_t i = 0; i < dim; i++) {
            const float n = orc_h2f(xr[i]) * rstd - mean_rstd;              /* :1330 */
            y[r * dim + i] = orc_f2h(n * orc_h2f(gamma[i]) + orc_h2f(beta[i])); /* :1333 */
        }
    }
    return 0;
}

void orc_softmax_rows(float *s, size_t rows, size_t cols) {
    float *tmp = (float *)malloc(cols * sizeof(float));
    for (size_t r = 0; r < rows; r++) {
        float *row = s + r * cols;
        float mx = row[0];
        for (size_t i = 1; i < cols; i++)
            if (row[i] > mx) mx = row[i];
        float sum = 0.0f;
        for (size_t i = 0; i < cols; i++) {
            const float v = row[i] - mx;
            tmp[i] = (v > -88.0f) ? expf(v) : 0.0f; /* ops.zig:1590 */
            sum = sum + tmp[i];
        }
        if (sum > 0.0f) { /* ops.zig:1595 */
            const float inv = 1.0f / sum;
            for (size_t i = 0; i < cols; i++) row[i] = tmp[i] * inv;
        }
    }
    free(tmp);
}

/* ------------------------------------------------------------------ RoPE */
void orc_rope_table(float *table, size_t dim, size_t end, float theta) {
    const size_t half = dim / 2;
    for (size_t p = 0; p < end; p++)
        for (size_t i = 0; i < half; i++) {
            const float power = (float)(2 * i) / (float)dim;   /* rope.zig:51-52 */
            const float inv = 1.0f / powf(theta, power);       /* :59-65 */
            const float ang = (float)p * inv;                  /* :91 */
            table[(p * half + i) * 2 + 0] = cosf(ang);         /* :107 */
            table[(p * half + i) * 2 + 1] = sinf(ang);         /* :108 */
        }
}

void orc_rope_apply(const orc_f16 *x, orc_f16 *out, size_t n_heads, size_t seq_len, size_t head_dim,
                    const float *table, const size_t *position_ids, size_t rot_dim) {
    const size_t half = rot_dim / 2;
    for (size_t h = 0; h < n_heads; h++)
        for (size_t s = 0; s < seq_len; s++) {
            const size_t base = (h * seq_len + s) * head_dim;
            const float *f = table + position_ids[s] * half * 2; /* rope.zig:173 */
            for (size_t i = 0; i < half; i++) {
                const float xr = orc_h2f(x[base + i]);
                const float xi = orc_h2f(x[base + half + i]);
                const float c = f[2 * i], sn = f[2 * i + 1];
                out[base + i] = orc_f2h(xr * c - xi * sn);          /* :223 */
                out[base + half + i] = orc_f2h(xr * sn + xi * c);   /* :224 */
            }
            for (size_t i = rot_dim; i < head_dim; i++) out[base + i] = x[base + i]; /* :256-269 */
        }
}

/* ------------------------------------------------------------------ attention */
void orc_attention_mask(uint8_t *mask, size_t pos, size_t seq_len) {
    const size_t w = pos + seq_len;
    for (size_t i = 0; i < seq_len; i++) {
        for (size_t j = 0; j < pos; j++) mask[i * w + j] = 1;
        for (size_t j = 0; j < seq_len; j++) mask[i * w + pos + j] = (j <= i);
    }
}

void orc_sdpa_multi(const orc_f16 *q, const orc_f16 *k, const orc_f16 *v, const uint8_t *mask,
                    size_t mask_stride, orc_f16 *out, size_t n_heads, size_t q_len, size_t kv_len,
                    size_t head_dim) {
    const float scale = 1.0f / sqrtf((float)head_dim); /* attention.zig:136, :428 */
#pragma omp parallel for schedule(dynamic, 1)
    for (size_t h = 0; h < n_heads; h++) {
        float *qf = (float *)malloc(q_len * head_dim * sizeof(float));
        float *kt = (float *)malloc(head_dim * kv_len * sizeof(float));
        float *vf = (float *)malloc(kv_len * head_dim * sizeof(float));
        float *S = (float *)malloc(q_len * kv_len * sizeof(float));
        float *O = (float *)malloc(q_len * head_dim * sizeof(float));
        orc_cast_f16_to_f32(q + h * q_len * head_dim, qf, q_len * head_dim);
        orc_cast_f16_to_f32(v + h * kv_len * head_dim, vf, kv_len * head_dim);
        for (size_t j = 0; j < kv_len; j++) /* explicit K transpose, attention.zig:443-451 */
            for (size_t d = 0; d < head_dim; d++) kt[d * kv_len + j] = orc_h2f(k[(h * kv_len + j) * head_dim + d]);
        orc_sgemm(qf, kt, S, q_len, kv_len, head_dim);            /* :190 / :485 */
        for (size_t i = 0; i < q_len * kv_len; i++) S[i] = S[i] * scale; /* :192-194 / :487-489 */
        if (mask)
            for (size_t i = 0; i < q_len; i++)
                for (size_t j = 0; j < kv_len; j++)
                    if (!mask[i * mask_stride + j]) S[i * kv_len + j] = -INFINITY; /* :491-499 */
        orc_softmax_rows(S, q_len, kv_len);                       /* :196 / :501 */
        orc_sgemm(S, vf, O, q_len, head_dim, kv_len);             /* :197 / :503 */
        orc_cast_f32_to_f16(O, out + h * q_len * head_dim, q_len * head_dim);
        free(qf); free(kt); free(vf); free(S); free(O);
    }
}

int orc_sdpa_single(const orc_f16 *q, const orc_f16 *k, const orc_f16 *v, const uint8_t *mask,
                    orc_f16 *out, size_t n_heads, size_t kv_len, size_t head_dim) {
    if (kv_len > 2048) return -3; /* attention.zig:769 SequenceTooLong */
    const float scale = 1.0f / sqrtf((float)head_dim); /* :569 */
#pragma omp parallel for schedule(static)
    for (size_t h = 0; h < n_heads; h++) {
        float scores[2048];
        float o[256];
        for (size_t j = 0; j < kv_len; j++) {
            float sum = 0.0f;
            const orc_f16 *kr = k + (h * kv_len + j) * head_dim;
            for (size_t d = 0; d < head_dim; d++) sum = sum + orc_h2f(q[h * head_dim + d]) * orc_h2f(kr[d]);
            scores[j] = sum * scale;                       /* :594 */
            if (mask && !mask[j]) scores[j] = -INFINITY;   /* :595 */
        }
        float mx = scores[0];
        for (size_t j = 1; j < kv_len; j++) mx = fmaxf(mx, scores[j]); /* :601-604 */
        float sum = 0.0f;
        for (size_t j = 0; j < kv_len; j++) {
            scores[j] = expf(scores[j] - mx);              /* :608 (no -88 clamp on this path) */
            sum = sum + scores[j];
        }
        const float inv = 1.0f / sum;                      /* :612 */
        for (size_t j = 0; j < kv_len; j++) scores[j] = scores[j] * inv;
        for (size_t d = 0; d < head_dim; d++) o[d] = 0.0f;
        for (size_t j = 0; j < kv_len; j++) {
            const orc_f16 *vr = v + (h * kv_len + j) * head_dim;
            for (size_t d = 0; d < head_dim; d++) o[d] = o[d] + orc_h2f(vr[d]) * scores[j]; /* :621-632 */
        }
        for (size_t d = 0; d < head_dim; d++) out[h * head_dim + d] = orc_f2h(o[d]);
    }
    return 0;
}

void orc_sdpa_f64(const orc_f16 *q, const orc_f16 *k, const orc_f16 *v, const uint8_t *mask,
                  size_t mask_stride, double *out, size_t n_heads, size_t q_len, size_t kv_len,
                  size_t head_dim) {
    const double scale = 1.0 / sqrt((double)head_dim);
    double *s = (double *)malloc(kv_len * sizeof(double));
    for (size_t h = 0; h < n_heads; h++)
        for (size_t i = 0; i < q_len; i++) {
            double mx = -INFINITY;
            for (size_t j = 0; j < kv_len; j++) {
                double d = 0.0;
                for (size_t e = 0; e < head_dim; e++)
                    d += (double)orc_h2f(q[(h * q_len + i) * head_dim + e]) * (double)orc_h2f(k[(h * kv_len + j) * head_dim + e]);
                s[j] = (mask && !mask[i * mask_stride + j]) ? -INFINITY : d * scale;
                if (s[j] > mx) mx = s[j];
            }
            double sum = 0.0;
            for (size_t j = 0; j < kv_len; j++) { s[j] = exp(s[j] - mx); sum += s[j]; }
            for (size_t e = 0; e < head_dim; e++) {
                double o = 0.0;
                for (size_t j = 0; j < kv_len; j++) o += s[j] * (double)orc_h2f(v[(h * kv_len + j) * head_dim + e]);
                out[(h * q_len + i) * head_dim + e] = o / sum;
            }
        }
    free(s);
}

/* ------------------------------------------------------------------ KV cache, layout */
int orc_kv_update(orc_f16 *cache_k, orc_f16 *cache_v, size_t *current_len, const orc_f16 *k,
                  const orc_f16 *v, size_t n_heads, size_t seq_len, size_t head_dim, size_t max_seq) {
    const size_t new_len = *current_len + seq_len;
    if (new_len > max_seq) return -3; /* text_model.zig:478 SequenceTooLong */
    for (size_t h = 0; h < n_heads; h++)
        for (size_t t = 0; t < seq_len; t++) {
            const size_t src = (h * seq_len + t) * head_dim;
            const size_t dst = (h * max_seq + *current_len + t) * head_dim;
            memcpy(cache_k + dst, k + src, head_dim * sizeof(orc_f16));
            memcpy(cache_v + dst, v + src, head_dim * sizeof(orc_f16));
        }
    *current_len = new_len;
    return 0;
}

void orc_kv_active(const orc_f16 *cache, orc_f16 *out, size_t n_heads, size_t cur_len,
                   size_t head_dim, size_t max_seq) {
    for (size_t h = 0; h < n_heads; h++)
        memcpy(out + h * cur_len * head_dim, cache + h * max_seq * head_dim, cur_len * head_dim * sizeof(orc_f16));
}

void orc_split_heads(const orc_f16 *qkv, size_t row_stride, size_t col_off, orc_f16 *out,
                     size_t seq_len, size_t n_heads, size_t head_dim) {
    for (size_t s = 0; s < seq_len; s++)
        for (size_t h = 0; h < n_heads; h++)
            memcpy(out + (h * seq_len + s) * head_dim, qkv + s * row_stride + col_off + h * head_dim,
                   head_dim * sizeof(orc_f16));
}

void orc_merge_heads(const orc_f16 *x, orc_f16 *out, size_t seq_len, size_t n_heads, size_t head_dim) {
    for (size_t s = 0; s < seq_len; s++)
        for (size_t h = 0; h < n_heads; h++)
            memcpy(out + (s * n_heads + h) * head_dim, x + (h * seq_len + s) * head_dim, head_dim * sizeof(orc_f16));
}

size_t orc_argmax_f16(const orc_f16 *logits, size_t n) {
    size_t idx = 0;
    float best = orc_h2f(logits[0]);
    for (size_t i = 0; i < n; i++) {
        const float v = orc_h2f(logits[i]);
        if (v > best) { best = v; idx = i; } /* strict >: first maximum wins (sampling.zig:265) */
    }
    return idx;
}

/* ------------------------------------------------------------------ sampling (sampling.zig) */
/* exp for the sampling paths.  The reference's @exp(f32) comes from its language runtime's libm port (the classic
 * expf: k = round(x / ln 2), x - k ln2 in two parts, c = x - x^2 (P1 + x^2 P2), 1 + (x c / (2 - c) - lo + hi), scaled
 * by 2^k); which candidate a draw lands on depends on the last bit of every term, so the checker and the device share
 * this one definition, evaluated with separate IEEE f32 operations, instead of each trusting its own library's expf. */
static float orc_expf_sampling(float x) {
    static const float ln2hi = 6.9314575195e-1f, ln2lo = 1.4286067653e-6f, invln2 = 1.4426950216e+0f, P1 = 1.6666625440e-1f,
                       P2 = -2.7667332906e-3f;
    union { float f; uint32_t u; } w;
    w.f = x;
    const int sign = (int)(w.u >> 31);
    const uint32_t hx = w.u & 0x7fffffffu;
    if (hx > 0x7f800000u) return x;                       /* NaN */
    if (hx >= 0x42b17218u && !sign) return x * 0x1p127f;  /* overflow */
    if (sign && hx >= 0x42cff1b5u) return 0.0f;           /* underflow */
    volatile float hi, lo, xr;
    int k;
    if (hx > 0x3eb17218u) {                               /* |x| > 0.5 ln2 */
        if (hx > 0x3f851592u) {                           /* |x| > 1.5 ln2 */
            volatile float kf = invln2 * x;
            kf = kf + (sign ? -0.5f : 0.5f);
            k = (int)kf;
        } else
            k = 1 - sign - sign;
        volatile float t1 = (float)k * ln2hi;
        hi = x - t1;
        lo = (float)k * ln2lo;
        xr = hi - lo;
    } else if (hx > 0x39000000u) {                        /* |x| > 2^-14 */
        k = 0;
        hi = x;
        lo = 0.0f;
        xr = x;
    } else
        return 1.0f + x;
    volatile float xx = xr * xr;
    volatile float p = xx * P2;
    p = P1 + p;
    p = xx * p;
    volatile float c = xr - p;
    volatile float num = xr * c;
    volatile float den = 2.0f - c;
    volatile float q = num / den;
    q = q - lo;
    q = q + hi;
    volatile float y = 1.0f + q;
    if (k == 0) return y;
    return ldexpf(y, k);
}

/* orc_expf_sampling over an array (for the tests that pin it) */
void orc_sampling_expf(const float *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = orc_expf_sampling(x[i]);
}

/* ops.softmax over one f32 row (ops.zig:1574-1601): running maximum, exp with the -88 cut-off, sequential sum,
 * multiply by 1/sum when the sum is positive. */
static void sample_softmax(float *x, size_t n) {
    float max = x[0];
    for (size_t i = 1; i < n; i++)
        if (x[i] > max) max = x[i];
    float sum = 0.f;
    for (size_t i = 0; i < n; i++) {
        const float val = x[i] - max;
        x[i] = val > -88.0f ? orc_expf_sampling(val) : 0.f;
        sum += x[i];
    }
    if (sum > 0.f) {
        const float inv_sum = 1.0f / sum;
        for (size_t i = 0; i < n; i++) x[i] *= inv_sum;
    }
}

/* Merge sort of indices by descending probability; equal probabilities keep their ascending index order, which is
 * what the stable std.mem.sort of sampling.zig:315-319 leaves. */
static void sample_sort_desc(size_t *idx, size_t *tmp, const float *p, size_t n) {
    if (n < 2) return;
    const size_t h = n / 2;
    sample_sort_desc(idx, tmp, p, h);
    sample_sort_desc(idx + h, tmp, p, n - h);
    size_t a = 0, b = h, o = 0;
    while (a < h && b < n) tmp[o++] = p[idx[b]] > p[idx[a]] ? idx[b++] : idx[a++];
    while (a < h) tmp[o++] = idx[a++];
    while (b < n) tmp[o++] = idx[b++];
    memcpy(idx, tmp, n * sizeof(size_t));
}

/* sampling.sample (sampling.zig:353-389) on f32(logits) (moondream.zig:335-337), with the one number the reference
 * draws from its PRNG (rng.float(f32), in [0,1)) passed in as u.  method: 0 greedy, 1 multinomial, 2 top_k, 3 min_p.
 * Returns 0, or 1 InvalidTemperature (sampling.zig:344), 2 a top_k of 0 (the reference indexes [k-1] of an empty
 * slice there), 3 unknown method / empty input. */
int orc_sample_f32(const float *logits, size_t n, int method, float temperature, size_t top_k, float min_p, float u, size_t *index);
int orc_sample_f16(const orc_f16 *logits, size_t n, int method, float temperature, size_t top_k, float min_p, float u, size_t *index) {
    if (!n) return 3;
    float *x = (float *)malloc(n * sizeof(float)); /* moondream.zig:335: logits.castWithSimd(f32) */
    for (size_t i = 0; i < n; i++) x[i] = orc_h2f(logits[i]);
    const int rc = orc_sample_f32(x, n, method, temperature, top_k, min_p, u, index);
    free(x);
    return rc;
}
/* the same on the f32 row sampling.sample takes (sampling.zig:353-358) */
int orc_sample_f32(const float *logits, size_t n, int method, float temperature, size_t top_k, float min_p, float u, size_t *index) {
    if (!n || method < 0 || method > 3) return 3;
    if (method == 0) { /* sampling.zig:370-372: temperature is not applied; argmax: strict >, first maximum wins (:257-273) */
        size_t idx = 0;
        float best = logits[0];
        for (size_t i = 0; i < n; i++)
            if (logits[i] > best) { best = logits[i]; idx = i; }
        *index = idx;
        return 0;
    }
    if (temperature != 1.0f && !(temperature > 0.f)) return 1;
    if (method == 2 && top_k == 0) return 2;
    float *x = (float *)malloc(n * sizeof(float));
    for (size_t i = 0; i < n; i++) x[i] = logits[i];
    if (temperature != 1.0f)
        for (size_t i = 0; i < n; i++) x[i] = x[i] / temperature; /* sampling.zig:347-349 */
    int rc = 0;
    if (method == 1) { /* softmax, then multinomial_sampling (sampling.zig:276-297) */
        sample_softmax(x, n);
        float sum = 0.f;
        for (size_t i = 0; i < n; i++) sum += x[i];
        const float r = u * sum;
        float cumsum = 0.f;
        *index = n - 1;
        for (size_t i = 0; i < n; i++) {
            cumsum += x[i];
            if (r < cumsum) { *index = i; break; }
        }
    } else if (method == 2) { /* softmax, then top_k_sampling (sampling.zig:300-339) */
        sample_softmax(x, n);
        const size_t k = top_k < n ? top_k : n;
        size_t *idx = (size_t *)malloc(2 * n * sizeof(size_t));
        for (size_t i = 0; i < n; i++) idx[i] = i;
        sample_sort_desc(idx, idx + n, x, n);
        float sum = 0.f;
        for (size_t j = 0; j < k; j++) sum += x[idx[j]];
        const float r = u * sum;
        float cumsum = 0.f;
        *index = idx[k - 1];
        for (size_t j = 0; j < k; j++) {
            cumsum += x[idx[j]];
            if (r < cumsum) { *index = idx[j]; break; }
        }
        free(idx);
    } else { /* min_p_sampling (sampling.zig:114-219) */
        float max_logit = -INFINITY;
        for (size_t i = 0; i < n; i++) max_logit = x[i] > max_logit ? x[i] : max_logit;
        float sum = 0.f;
        for (size_t i = 0; i < n; i++) {
            const float d = x[i] - max_logit;
            x[i] = d > -88.0f ? orc_expf_sampling(d) : 0.f;
            sum += x[i];
        }
        const float inv_sum = 1.0f / sum;
        float max_prob = 0.f;
        for (size_t i = 0; i < n; i++) {
            x[i] *= inv_sum;
            max_prob = x[i] > max_prob ? x[i] : max_prob;
        }
        const float threshold = min_p * max_prob;
        size_t first_valid = n, valid_count = 0;
        float valid_sum = 0.f;
        for (size_t i = 0; i < n; i++)
            if (x[i] >= threshold) {
                if (!valid_count++) first_valid = i;
                valid_sum += x[i];
            }
        if (!valid_count) { /* keep the most probable token (sampling.zig:183-197): strict '>' scan */
            size_t max_idx = 0;
            for (size_t i = 0; i < n; i++)
                if (x[i] > x[max_idx]) max_idx = i;
            *index = max_idx;
        } else {
            const float r = u * valid_sum;
            float cumsum = 0.f;
            *index = first_valid;
            for (size_t i = 0; i < n; i++) {
                if (!(x[i] >= threshold)) continue;
                cumsum += x[i];
                if (r < cumsum) { *index = i; break; }
            }
        }
    }
    free(x);
    return rc;
}

double orc_rel_frobenius(const orc_f16 *a, const orc_f16 *b, size_t n) {
    double num = 0.0, den = 0.0;
    for (size_t i = 0; i < n; i++) {
        const double x = orc_h2f(a[i]), y = orc_h2f(b[i]);
        num += (x - y) * (x - y);
        den += y * y;
    }
    return den > 0.0 ? sqrt(num / den) : sqrt(num);
}

/* ------------------------------------------------------------------ reference-style timed kernels */
int orc_host_threads(void) {
    long n = sysconf(_SC_NPROCESSORS_ONLN);
    const char *env = getenv("OMP_NUM_THREADS");
    if (env && atoi(env) > 0 && atoi(env) < n) n = atoi(env);
    return n > 0 ? (int)n : 1;
}

typedef struct {
    const orc_f16 *a, *b;
    orc_f16 *c;
    size_t M, N, K, tiles_n, total;
    int b_transposed;
    atomic_size_t *counter;
} rs_ctx;

static inline __m256 load8h(const orc_f16 *p) { return _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)p)); }

static inline float hsum8(__m256 v) {
    __m128 lo = _mm256_castps256_ps128(v), hi = _mm256_extractf128_ps(v, 1);
    lo = _mm_add_ps(lo, hi);
    lo = _mm_hadd_ps(lo, lo);
    lo = _mm_hadd_ps(lo, lo);
    return _mm_cvtss_f32(lo);
}

/* hgemm_trans.zig:55-118: per output, four 8-lane accumulators over k in steps of 32. */
static void *rs_gemv_worker(void *arg) {
    rs_ctx *x = (rs_ctx *)arg;
    const size_t chunk = 32; /* :431 */
    for (;;) {
        const size_t ci = atomic_fetch_add(x->counter, 1); /* :126 */
        if (ci >= x->total) break;
        const size_t n0 = ci * chunk, n1 = (n0 + chunk < x->N) ? n0 + chunk : x->N;
        for (size_t n = n0; n < n1; n++) {
            const orc_f16 *row = x->b + n * x->K;
            __m256 a0 = _mm256_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
            size_t k = 0;
            const size_t ka = x->K - (x->K % 32);
            for (; k < ka; k += 32) {
                a0 = _mm256_fmadd_ps(load8h(x->a + k), load8h(row + k), a0);
                a1 = _mm256_fmadd_ps(load8h(x->a + k + 8), load8h(row + k + 8), a1);
                a2 = _mm256_fmadd_ps(load8h(x->a + k + 16), load8h(row + k + 16), a2);
                a3 = _mm256_fmadd_ps(load8h(x->a + k + 24), load8h(row + k + 24), a3);
            }
            float tail = 0.0f;
            for (; k < x->K; k++) tail += orc_h2f(x->a[k]) * orc_h2f(row[k]);
            const float sum = hsum8(_mm256_add_ps(_mm256_add_ps(a0, a1), _mm256_add_ps(a2, a3)));
            x->c[n] = orc_f2h(sum + tail);
        }
    }
    return NULL;
}

static void run_threads(void *(*fn)(void *), rs_ctx *ctx, int threads) {
    /* spawn and join one thread per core on every call, as the reference does
     * (hgemm_trans.zig:445-453, hgemm.zig:419-423). */
    if (threads < 1) threads = 1;
    pthread_t *t = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)threads);
    for (int i = 0; i < threads; i++) pthread_create(&t[i], NULL, fn, ctx);
    for (int i = 0; i < threads; i++) pthread_join(t[i], NULL);
    free(t);
}

void orc_refstyle_gemv_nt(const orc_f16 *a, const orc_f16 *Bt, orc_f16 *c, size_t N, size_t K, int threads) {
    atomic_size_t counter = 0;
    rs_ctx ctx = {a, Bt, c, 1, N, K, 0, (N + 31) / 32, 1, &counter};
    run_threads(rs_gemv_worker, &ctx, threads);
}

#define RS_T 168 /* hgemm.zig:34-38, hgemm_trans.zig:20 */

/* hgemm.zig:100-143 + :173-348 / hgemm_trans.zig:257-398: T^3 tiles converted to f32 on the
 * stack, 8x8 broadcast-FMA micro-kernel, scalar edges, f32 tile accumulator, one rounding. */
static void *rs_gemm_worker(void *arg) {
    rs_ctx *x = (rs_ctx *)arg;
    static __thread float Cl[RS_T][RS_T], Al[RS_T][RS_T], Bl[RS_T][RS_T];
    for (;;) {
        const size_t t = atomic_fetch_add(x->counter, 1);
        if (t >= x->total) break;
        const size_t i0 = (t / x->tiles_n) * RS_T, j0 = (t % x->tiles_n) * RS_T;
        const size_t i1 = i0 + RS_T < x->M ? i0 + RS_T : x->M, j1 = j0 + RS_T < x->N ? j0 + RS_T : x->N;
        const size_t is = i1 - i0, js = j1 - j0;
        memset(Cl, 0, sizeof(Cl));
        for (size_t k0 = 0; k0 < x->K; k0 += RS_T) {
            const size_t k1 = k0 + RS_T < x->K ? k0 + RS_T : x->K, ks = k1 - k0;
            for (size_t i = 0; i < is; i++)
                for (size_t k = 0; k < ks; k++) Al[i][k] = orc_h2f(x->a[(i0 + i) * x->K + k0 + k]);
            if (x->b_transposed) {
                for (size_t j = 0; j < js; j++)
                    for (size_t k = 0; k < ks; k++) Bl[k][j] = orc_h2f(x->b[(j0 + j) * x->K + k0 + k]);
            } else {
                for (size_t k = 0; k < ks; k++)
                    for (size_t j = 0; j < js; j++) Bl[k][j] = orc_h2f(x->b[(k0 + k) * x->N + j0 + j]);
            }
            size_t i = 0;
            for (; i + 8 <= is; i += 8) {
                size_t j = 0;
                for (; j + 8 <= js; j += 8) {
                    __m256 acc[8];
                    for (int r = 0; r < 8; r++) acc[r] = _mm256_setzero_ps();
                    for (size_t k = 0; k < ks; k++) {
                        const __m256 b = _mm256_loadu_ps(&Bl[k][j]);
                        for (int r = 0; r < 8; r++) acc[r] = _mm256_fmadd_ps(_mm256_set1_ps(Al[i + r][k]), b, acc[r]);
                    }
                    for (int r = 0; r < 8; r++)
                        _mm256_storeu_ps(&Cl[i + r][j], _mm256_add_ps(_mm256_loadu_ps(&Cl[i + r][j]), acc[r]));
                }
                for (; j < js; j++)
                    for (int r = 0; r < 8; r++) {
                        float s = 0.0f;
                        for (size_t k = 0; k < ks; k++) s = fmaf(Al[i + r][k], Bl[k][j], s);
                        Cl[i + r][j] += s;
                    }
            }
            for (; i < is; i++)
                for (size_t j = 0; j < js; j++) {
                    float s = 0.0f;
                    for (size_t k = 0; k < ks; k++) s = fmaf(Al[i][k], Bl[k][j], s);
                    Cl[i][j] += s;
                }
        }
        for (size_t i = 0; i < is; i++)
            for (size_t j = 0; j < js; j++) x->c[(i0 + i) * x->N + j0 + j] = orc_f2h(Cl[i][j]);
    }
    return NULL;
}

void orc_refstyle_hgemm(const orc_f16 *A, const orc_f16 *B, orc_f16 *C, size_t M, size_t N, size_t K,
                        int b_transposed, int threads) {
    if (b_transposed && M == 1) { /* hgemm_trans.zig:430 fast path */
        orc_refstyle_gemv_nt(A, B, C, N, K, threads);
        return;
    }
    atomic_size_t counter = 0;
    const size_t tm = (M + RS_T - 1) / RS_T, tn = (N + RS_T - 1) / RS_T;
    rs_ctx ctx = {A, B, C, M, N, K, tn, tm * tn, b_transposed, &counter};
    run_threads(rs_gemm_worker, &ctx, threads);
}

typedef struct {
    const orc_f16 *q, *k, *v;
    orc_f16 *out;
    size_t n_heads, kv_len, head_dim;
    atomic_size_t *counter;
} rs_attn;

/* attention.zig:564-642: per head, 8-wide f16->f32 dot products, exp softmax, weighted V sum. */
static void *rs_attn_worker(void *arg) {
    rs_attn *x = (rs_attn *)arg;
    float scores[2048];
    const float scale = 1.0f / sqrtf((float)x->head_dim);
    for (;;) {
        const size_t h = atomic_fetch_add(x->counter, 1);
        if (h >= x->n_heads) break;
        const orc_f16 *qh = x->q + h * x->head_dim;
        for (size_t j = 0; j < x->kv_len; j++) {
            const orc_f16 *kr = x->k + (h * x->kv_len + j) * x->head_dim;
            float s = 0.0f;
            for (size_t d = 0; d + 8 <= x->head_dim; d += 8) s += hsum8(_mm256_mul_ps(load8h(qh + d), load8h(kr + d)));
            scores[j] = s * scale;
        }
        float mx = scores[0];
        for (size_t j = 1; j < x->kv_len; j++) mx = fmaxf(mx, scores[j]);
        float sum = 0.0f;
        for (size_t j = 0; j < x->kv_len; j++) { scores[j] = expf(scores[j] - mx); sum += scores[j]; }
        const float inv = 1.0f / sum;
        __m256 o[32];
        const size_t chunks = x->head_dim / 8;
        for (size_t c = 0; c < chunks; c++) o[c] = _mm256_setzero_ps();
        for (size_t j = 0; j < x->kv_len; j++) {
            const orc_f16 *vr = x->v + (h * x->kv_len + j) * x->head_dim;
            const __m256 w = _mm256_set1_ps(scores[j] * inv);
            for (size_t c = 0; c < chunks; c++) o[c] = _mm256_fmadd_ps(load8h(vr + 8 * c), w, o[c]);
        }
        for (size_t c = 0; c < chunks; c++)
            _mm_storeu_si128((__m128i *)(x->out + h * x->head_dim + 8 * c),
                             _mm256_cvtps_ph(o[c], _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
    }
    return NULL;
}

void orc_refstyle_sdpa_single(const orc_f16 *q, const orc_f16 *k, const orc_f16 *v, orc_f16 *out,
                              size_t n_heads, size_t kv_len, size_t head_dim, int threads) {
    atomic_size_t counter = 0;
    rs_attn ctx = {q, k, v, out, n_heads, kv_len, head_dim, &counter};
    if (threads > (int)n_heads) threads = (int)n_heads;
    if (threads < 1) threads = 1;
    pthread_t *t = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)threads);
    for (int i = 0; i < threads; i++) pthread_create(&t[i], NULL, rs_attn_worker, &ctx);
    for (int i = 0; i < threads; i++) pthread_join(t[i], NULL);
    free(t);
}
