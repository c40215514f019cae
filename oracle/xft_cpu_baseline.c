/*
 * CPU baseline of the decode step: an "xFT-semantics CPU restatement (not the xDNN binary)".
 *
 * TEST / BENCHMARK INFRASTRUCTURE ONLY.  The reference's real CPU path cannot be built offline
 * (its GEMM kernels live in the closed xDNN binary, cmake/xdnn.cmake:28-30), so the number reported
 * beside the GPU result comes from this file: the same data flow as the reference's decoder layer
 * for weight-only quantised models (src/layers/decoder_layer.h:101-170, attention.h:267-496,
 * mlp_llama.h:197-290): fp32 activations end to end, fused QKV GEMV, rotate-half RoPE, FP16 KV
 * cache in [B][H][S][D], attention parallel over (batch, head), concatenated gate/up GEMV with
 * SiLU(gate) * up, down GEMV + residual, final RMSNorm, BF16 lm_head, greedy argmax.
 * Written for speed, not bit-faithfulness (that is xft_oracle.c): loops are laid out so that gcc
 * -O3 -march=native turns them into whatever vector ISA the host has (AVX-512 / AVX2), weights are
 * streamed once per step with OpenMP over output-column blocks.  bench.py compiles it on the machine
 * it runs on and times it on a bounded sample; the product library never links it.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define API __attribute__((visibility("default")))
enum { NB = 64 }; /* output columns per task */

API int cpu_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

#if defined(__F16C__) && defined(__AVX2__) && defined(__FMA__)
#include <immintrin.h>
static inline uint16_t f32_to_fp16(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT); }
static inline float hsum8(__m256 v) {
    __m128 s = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    s = _mm_add_ps(s, _mm_movehl_ps(s, s));
    s = _mm_add_ss(s, _mm_shuffle_ps(s, s, 1));
    return _mm_cvtss_f32(s);
}
/* sum_i q[i] * k[i], k in fp16; D a multiple of 8 */
static inline float dot_fp16(const float *q, const uint16_t *k, int D) {
    __m256 acc = _mm256_setzero_ps();
    for (int i = 0; i < D; i += 8)
        acc = _mm256_fmadd_ps(_mm256_loadu_ps(q + i), _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(k + i))), acc);
    return hsum8(acc);
}
/* o[i] += p * v[i], v in fp16 */
static inline void axpy_fp16(float *o, float p, const uint16_t *v, int D) {
    const __m256 pp = _mm256_set1_ps(p);
    for (int i = 0; i < D; i += 8)
        _mm256_storeu_ps(o + i, _mm256_fmadd_ps(pp, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(v + i))), _mm256_loadu_ps(o + i)));
}
static inline float fp16_to_f32(uint16_t h) { return _cvtsh_ss(h); }
#else
static inline float fp16_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000) << 16, e = (h >> 10) & 31, m = h & 1023, u;
    if (e == 0) {
        if (m == 0) u = s;
        else {
            int sh = 0;
            while (!(m & 1024)) m <<= 1, ++sh;
            u = s | ((uint32_t)(113 - sh) << 23) | ((m & 1023) << 13);
        }
    } else if (e == 31) u = s | 0x7F800000u | (m << 13);
    else u = s | ((e + 112) << 23) | (m << 13);
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t f32_to_fp16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t s = (u >> 16) & 0x8000, a = u & 0x7FFFFFFFu;
    if (a >= 0x47800000u) return (uint16_t)(s | (a > 0x7F800000u ? 0x7E00 : 0x7C00));
    if (a < 0x38800000u) { /* subnormal or zero */
        if (a < 0x33000000u) return (uint16_t)s;
        uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
        int sh = 126 - (int)(a >> 23);
        uint32_t r = m >> sh, rem = m & ((1u << sh) - 1), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (r & 1))) ++r;
        return (uint16_t)(s | r);
    }
    uint32_t r = a - 0x38000000u;
    uint32_t m = r >> 13, rem = r & 0x1FFF;
    if (rem > 0x1000 || (rem == 0x1000 && (m & 1))) ++m;
    return (uint16_t)(s | m);
}
static inline float dot_fp16(const float *q, const uint16_t *k, int D) {
    float d = 0.0f;
    for (int i = 0; i < D; ++i) d += q[i] * fp16_to_f32(k[i]);
    return d;
}
static inline void axpy_fp16(float *o, float p, const uint16_t *v, int D) {
    for (int i = 0; i < D; ++i) o[i] += p * fp16_to_f32(v[i]);
}
#endif

/* y[N] = scale[n] * sum_k a[k] q[k][n] + zero[n] * sum(a)  (+ res), INT8 [K,N] row-major */
static void gemv_int8(int K, int N, const float *a, const int8_t *q, const float *scale, const float *zero, float *y,
        const float *res) {
    float sumA = 0.0f;
    if (zero)
        for (int k = 0; k < K; ++k) sumA += a[k];
#pragma omp parallel for schedule(static)
    for (int n0 = 0; n0 < N; n0 += NB) {
        const int nb = N - n0 < NB ? N - n0 : NB;
        float acc[NB];
        for (int j = 0; j < nb; ++j) acc[j] = 0.0f;
        for (int k = 0; k < K; ++k) {
            const int8_t *row = q + (int64_t)k * N + n0;
            const float ak = a[k];
#pragma omp simd
            for (int j = 0; j < nb; ++j) acc[j] += ak * (float)row[j];
        }
        for (int j = 0; j < nb; ++j) {
            float v = scale[n0 + j] * acc[j] + (zero ? zero[n0 + j] * sumA : 0.0f);
            y[n0 + j] = res ? v + res[n0 + j] : v;
        }
    }
}
/* UINT4 [K,N/2] bytes, even column in the low nibble */
static void gemv_uint4(int K, int N, const float *a, const uint8_t *q, const float *scale, const float *zero, float *y,
        const float *res) {
    float sumA = 0.0f;
    for (int k = 0; k < K; ++k) sumA += a[k];
#pragma omp parallel for schedule(static)
    for (int n0 = 0; n0 < N; n0 += NB) {
        const int nb = N - n0 < NB ? N - n0 : NB;
        float lo[NB / 2], hi[NB / 2];
        for (int j = 0; j < nb / 2; ++j) lo[j] = hi[j] = 0.0f;
        for (int k = 0; k < K; ++k) {
            const uint8_t *row = q + ((int64_t)k * N + n0) / 2;
            const float ak = a[k];
#pragma omp simd
            for (int j = 0; j < nb / 2; ++j) {
                lo[j] += ak * (float)(row[j] & 15);
                hi[j] += ak * (float)(row[j] >> 4);
            }
        }
        for (int j = 0; j < nb; ++j) {
            float v = scale[n0 + j] * ((j & 1) ? hi[j >> 1] : lo[j >> 1]) + (zero ? zero[n0 + j] * sumA : 0.0f);
            y[n0 + j] = res ? v + res[n0 + j] : v;
        }
    }
}
static void gemv(int kind, int K, int N, const float *a, const void *q, const float *scale, const float *zero, float *y,
        const float *res) {
    if (kind == 0) gemv_int8(K, N, a, (const int8_t *)q, scale, zero, y, res);
    else gemv_uint4(K, N, a, (const uint8_t *)q, scale, zero, y, res);
}
/* BF16 [K,N] weights (lm_head) */
static void gemv_bf16(int K, int N, const float *a, const uint16_t *w, float *y) {
#pragma omp parallel for schedule(static)
    for (int n0 = 0; n0 < N; n0 += NB) {
        const int nb = N - n0 < NB ? N - n0 : NB;
        float acc[NB];
        for (int j = 0; j < nb; ++j) acc[j] = 0.0f;
        for (int k = 0; k < K; ++k) {
            const uint16_t *row = w + (int64_t)k * N + n0;
            const float ak = a[k];
#pragma omp simd
            for (int j = 0; j < nb; ++j) {
                uint32_t u = (uint32_t)row[j] << 16;
                float f;
                memcpy(&f, &u, 4);
                acc[j] += ak * f;
            }
        }
        for (int j = 0; j < nb; ++j) y[n0 + j] = acc[j];
    }
}
static void rmsnorm(int n, const float *x, const float *w, float eps, float *y) {
    float s = 0.0f;
    for (int i = 0; i < n; ++i) s += x[i] * x[i];
    const float r = 1.0f / sqrtf(s / (float)n + eps);
    for (int i = 0; i < n; ++i) y[i] = x[i] * r * w[i];
}

typedef struct {
    int kind; /* 0 INT8, 1 UINT4 */
    int layers, hidden, inter, heads, kv_heads, head, vocab, max_seq;
    /* per layer: qkv, o, gateup, down weights in the pre-pack layout + scale/zero, norm weights */
    const void **wq[4];
    const float **ws[4], **wz[4];
    const float *ln1, *ln2, *final_norm; /* shared ones-vectors are fine for timing */
    const uint16_t *embedding_fp16; /* [vocab, hidden] */
    const uint16_t *lm_head_bf16; /* [hidden, vocab] */
    uint16_t *kcache, *vcache; /* [layers][B][kv_heads][max_seq][head] fp16 */
    int batch;
} cpu_model;

/* One greedy decode step for every sequence of the batch at position pos; ids in/out. */
API void cpu_decode_step(const cpu_model *m, int *ids, int pos, float *scratch) {
    const int H = m->hidden, I = m->inter, D = m->head, qh = m->heads, kvh = m->kv_heads;
    const int qkv_cols = (qh + 2 * kvh) * D;
    float *x = scratch, *xn = x + H, *qkv = xn + H, *att = qkv + qkv_cols, *gu = att + qh * D, *h = gu + 2 * I, *logits = h + I;
    const float scale = 1.0f / sqrtf((float)D);
    float rc[128], rs[128]; /* cos / sin of this position (head size up to 256) */
    for (int i = 0; i < D / 2; ++i) {
        const float ang = (float)pos * powf(10000.0f, -2.0f * (float)i / (float)D);
        rc[i] = cosf(ang), rs[i] = sinf(ang);
    }
    for (int b = 0; b < m->batch; ++b) {
        for (int i = 0; i < H; ++i) x[i] = fp16_to_f32(m->embedding_fp16[(int64_t)ids[b] * H + i]);
        for (int l = 0; l < m->layers; ++l) {
            rmsnorm(H, x, m->ln1, 1e-6f, xn);
            gemv(m->kind, H, qkv_cols, xn, m->wq[0][l], m->ws[0][l], m->wz[0] ? m->wz[0][l] : NULL, qkv, NULL);
            /* rotate-half RoPE on q and k heads (rotary_embedding_kernels.cpp:126-199) */
            for (int hh = 0; hh < qh + kvh; ++hh) {
                float *v = qkv + hh * D;
                for (int i = 0; i < D / 2; ++i) {
                    const float c = rc[i], s = rs[i], a = v[i], bb = v[i + D / 2];
                    v[i] = a * c - bb * s;
                    v[i + D / 2] = bb * c + a * s;
                }
            }
            uint16_t *kc = m->kcache + ((int64_t)(l * m->batch + b) * kvh) * m->max_seq * D;
            uint16_t *vc = m->vcache + ((int64_t)(l * m->batch + b) * kvh) * m->max_seq * D;
            for (int hh = 0; hh < kvh; ++hh)
                for (int i = 0; i < D; ++i) {
                    kc[((int64_t)hh * m->max_seq + pos) * D + i] = f32_to_fp16(qkv[(qh + hh) * D + i]);
                    vc[((int64_t)hh * m->max_seq + pos) * D + i] = f32_to_fp16(qkv[(qh + kvh + hh) * D + i]);
                }
            const int n = pos + 1, group = qh / kvh;
#pragma omp parallel for schedule(static)
            for (int hh = 0; hh < qh; ++hh) {
                const float *q = qkv + hh * D;
                const uint16_t *K = kc + (int64_t)(hh / group) * m->max_seq * D, *V = vc + (int64_t)(hh / group) * m->max_seq * D;
                float *sc = (float *)malloc(sizeof(float) * (size_t)n);
                float mx = -1e30f;
                for (int t = 0; t < n; ++t) {
                    sc[t] = dot_fp16(q, K + (int64_t)t * D, D) * scale;
                    mx = sc[t] > mx ? sc[t] : mx;
                }
                float sum = 0.0f;
                for (int t = 0; t < n; ++t) sc[t] = expf(sc[t] - mx), sum += sc[t];
                float o[256];
                for (int i = 0; i < D; ++i) o[i] = 0.0f;
                for (int t = 0; t < n; ++t) axpy_fp16(o, sc[t] / sum, V + (int64_t)t * D, D);
                for (int i = 0; i < D; ++i) att[hh * D + i] = o[i];
                free(sc);
            }
            gemv(m->kind, qh * D, H, att, m->wq[1][l], m->ws[1][l], m->wz[1] ? m->wz[1][l] : NULL, xn, x);
            memcpy(x, xn, sizeof(float) * H);
            rmsnorm(H, x, m->ln2, 1e-6f, xn);
            gemv(m->kind, H, 2 * I, xn, m->wq[2][l], m->ws[2][l], m->wz[2] ? m->wz[2][l] : NULL, gu, NULL);
            for (int i = 0; i < I; ++i) h[i] = gu[i] / (1.0f + expf(-gu[i])) * gu[I + i];
            gemv(m->kind, I, H, h, m->wq[3][l], m->ws[3][l], m->wz[3] ? m->wz[3][l] : NULL, xn, x);
            memcpy(x, xn, sizeof(float) * H);
        }
        rmsnorm(H, x, m->final_norm, 1e-6f, xn);
        gemv_bf16(H, m->vocab, xn, m->lm_head_bf16, logits);
        int best = 0;
        for (int i = 1; i < m->vocab; ++i)
            if (logits[i] > logits[best]) best = i;
        ids[b] = best;
    }
}

/* scratch floats cpu_decode_step needs */
API int64_t cpu_scratch_floats(const cpu_model *m) {
    return (int64_t)2 * m->hidden + (int64_t)(2 * m->heads + 2 * m->kv_heads) * m->head + 3 * (int64_t)m->inter + m->vocab + 64;
}
