/* CPU restatement of the reference's fused kernels (TEST INFRASTRUCTURE ONLY).
 *
 * Only tests, the smoke entry and the benchmark's cpu_baseline leg load this
 * library; no product path links or calls it.
 *
 * Each function follows the algorithm of one reference kernel, in fp32 like the
 * reference (16-bit variants: fp32 math, one final rounding — the rule of
 * Metal/Kernels/FlashAttentionKernel.swift:223-256 and
 * Metal/Kernels/LayerNormKernel.swift:252-349).  tests/test_oracle.py pins every
 * function against the float64 closed forms in oracle.py and the reference's
 * known-answer values.  Rows/heads are split over OpenMP threads; the arithmetic
 * inside one row/head is sequential and therefore independent of thread count.
 *
 * Element type codes: 0 = f32, 1 = bf16 (uint16 storage, RNE on store).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* Runtime/BufferStorage.swift:328-344 */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t bits;
    memcpy(&bits, &f, 4);
    if (f != f) return 0x7FC0;
    uint32_t rounded = bits + 0x7FFFu + ((bits >> 16) & 1u);
    return (uint16_t)(rounded >> 16);
}
static inline float bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
static inline float ld(const void* p, int64_t i, int et) {
    return et == 0 ? ((const float*)p)[i] : bf16_to_f32(((const uint16_t*)p)[i]);
}
static inline void st(void* p, int64_t i, int et, float v) {
    if (et == 0) ((float*)p)[i] = v; else ((uint16_t*)p)[i] = f32_to_bf16(v);
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_f32_to_bf16(const float* x, uint16_t* y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = f32_to_bf16(x[i]);
}

/* Metal/Kernels/SoftmaxKernel.swift:36-100: max pass, exp+sum pass, normalise. */
void orc_softmax(const void* x, void* y, int64_t rows, int64_t cols, int et) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        int64_t o = r * cols;
        float m = -INFINITY;
        for (int64_t c = 0; c < cols; c++) m = fmaxf(m, ld(x, o + c, et));
        float s = 0.f;
        for (int64_t c = 0; c < cols; c++) s += expf(ld(x, o + c, et) - m);
        float inv = 1.f / s;
        for (int64_t c = 0; c < cols; c++) st(y, o + c, et, expf(ld(x, o + c, et) - m) * inv);
    }
}

/* Compiler/CodeGenerator.swift:4645-4686 (two-pass variance);
 * operand order [x, gamma, beta] of Compiler/CustomCallHandlers.swift:285-346. */
void orc_layer_norm(const void* x, const void* g, const void* b, void* y,
                    int64_t rows, int64_t cols, float eps, int et) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        int64_t o = r * cols;
        float sum = 0.f;
        for (int64_t c = 0; c < cols; c++) sum += ld(x, o + c, et);
        float mean = sum / (float)cols;
        float vs = 0.f;
        for (int64_t c = 0; c < cols; c++) { float d = ld(x, o + c, et) - mean; vs += d * d; }
        float inv = 1.f / sqrtf(vs / (float)cols + eps);
        for (int64_t c = 0; c < cols; c++) {
            float v = (ld(x, o + c, et) - mean) * inv;
            if (g) v *= ld(g, c, et);
            if (b) v += ld(b, c, et);
            st(y, o + c, et, v);
        }
    }
}

/* Metal/Kernels/LayerNormKernel.swift:439-520. */
void orc_rms_norm(const void* x, const void* g, void* y,
                  int64_t rows, int64_t cols, float eps, int et) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        int64_t o = r * cols;
        float ss = 0.f;
        for (int64_t c = 0; c < cols; c++) { float v = ld(x, o + c, et); ss += v * v; }
        float inv = 1.f / sqrtf(ss / (float)cols + eps);
        for (int64_t c = 0; c < cols; c++) {
            float v = ld(x, o + c, et) * inv;
            if (g) v *= ld(g, c, et);
            st(y, o + c, et, v);
        }
    }
}

/* Metal/Kernels/GELUKernel.swift:28-44, with the optional per-column bias of
 * Compiler/CodeGenerator.swift:4797-4850 added first. */
void orc_bias_gelu(const void* x, const void* bias, void* y,
                   int64_t rows, int64_t cols, int et) {
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        int64_t o = r * cols;
        for (int64_t c = 0; c < cols; c++) {
            float v = ld(x, o + c, et);
            if (bias) v += ld(bias, c, et);
            float inner = k0 * (v + k1 * v * v * v);
            st(y, o + c, et, 0.5f * v * (1.f + tanhf(inner)));
        }
    }
}

/* C[M,N] = A[M,K] . B[K,N], row-major, fp32 accumulate, one rounding at store
 * (Compiler/CodeGenerator.swift:3544-3549).  i-k-j loop order; per-row fp32
 * accumulator line so the inner loop vectorises. */
void orc_gemm(const void* a, const void* b, void* c,
              int64_t M, int64_t N, int64_t K, int et) {
#pragma omp parallel
    {
        float* acc = (float*)malloc(sizeof(float) * (size_t)N);
        float* brow = (float*)malloc(sizeof(float) * (size_t)N);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < M; i++) {
            for (int64_t j = 0; j < N; j++) acc[j] = 0.f;
            for (int64_t k = 0; k < K; k++) {
                float av = ld(a, i * K + k, et);
                if (et == 0) {
                    const float* bp = (const float*)b + k * N;
                    for (int64_t j = 0; j < N; j++) acc[j] += av * bp[j];
                } else {
                    const uint16_t* bp = (const uint16_t*)b + k * N;
                    for (int64_t j = 0; j < N; j++) brow[j] = bf16_to_f32(bp[j]);
                    for (int64_t j = 0; j < N; j++) acc[j] += av * brow[j];
                }
            }
            for (int64_t j = 0; j < N; j++) st(c, i * N + j, et, acc[j]);
        }
        free(acc);
        free(brow);
    }
}

/* Metal/Kernels/FlashAttentionKernel.swift:489-613: one query row at a time,
 * online softmax over the keys in order (m, l, alpha/beta rescale :589-598),
 * causal rule kv_pos > q_pos stops the scan (:578), l_inv guard (:608).
 * Q [B,H,Sq,D]; K,V [B,H,Skv,D]; O [B,H,Sq,D]. */
void orc_flash_attention(const void* q, const void* k, const void* v, void* o,
                         int64_t B, int64_t H, int64_t Sq, int64_t Skv, int64_t D,
                         float scale, int is_causal, int et) {
    int64_t nrows = B * H * Sq;
#pragma omp parallel
    {
        float* qreg = (float*)malloc(sizeof(float) * (size_t)D);
        float* oacc = (float*)malloc(sizeof(float) * (size_t)D);
#pragma omp for schedule(dynamic, 16)
        for (int64_t row = 0; row < nrows; row++) {
            int64_t bh = row / Sq, qpos = row % Sq;
            int64_t qb = row * D, kvb = bh * Skv * D;
            for (int64_t d = 0; d < D; d++) { qreg[d] = ld(q, qb + d, et); oacc[d] = 0.f; }
            float m_i = -INFINITY, l_i = 0.f;
            for (int64_t j = 0; j < Skv; j++) {
                if (is_causal && j > qpos) break;
                float score = 0.f;
                for (int64_t d = 0; d < D; d++) score += qreg[d] * ld(k, kvb + j * D + d, et);
                score *= scale;
                float m_new = fmaxf(m_i, score);
                float alpha = expf(m_i - m_new);
                float beta = expf(score - m_new);
                for (int64_t d = 0; d < D; d++)
                    oacc[d] = oacc[d] * alpha + beta * ld(v, kvb + j * D + d, et);
                l_i = l_i * alpha + beta;
                m_i = m_new;
            }
            float l_inv = (l_i > 1e-10f) ? (1.f / l_i) : 0.f;
            for (int64_t d = 0; d < D; d++) st(o, qb + d, et, oacc[d] * l_inv);
        }
        free(qreg);
        free(oacc);
    }
}
