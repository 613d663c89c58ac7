/*
 * cf_oracle_gemm.c -- CPU GEMM references and the CPU linear-forward baseline.
 * TEST INFRASTRUCTURE ONLY (see cf_oracle.h).  Build with -ffp-contract=off.
 */
#include "cf_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

void orc_dequant_n(const uint8_t* q, int is_e5m2, float descale, float* out, size_t n) {
    float lut[256];
    for (int b = 0; b < 256; ++b) lut[b] = is_e5m2 ? orc_e5m2_unpack((uint8_t)b) : orc_e4m3_unpack((uint8_t)b);
    for (size_t i = 0; i < n; ++i) out[i] = lut[q[i]] * descale;
}

/* ---- scaled FP8 NT GEMM reference -----------------------------------------
 * What the reference asks of cuBLASLt at src/trainer.cu:4498-4534:
 * C[M,N] = (A[M,K] * a_descale) . (B[N,K] * b_descale)^T with A E4M3 or E5M2
 * and row stride lda.  cuBLASLt is closed, so the answer is defined as the
 * matmul of the dequantised fp32 operands; the sum is carried in double so it
 * is a fixed point for any accumulation order.  Scale groups beyond per-tensor
 * use the same definition with the operand's own group descale. */
typedef struct {
    int M, N, K, lda, ldb, mode, m0, m1;
    const uint8_t *A, *B;
    const float *sa, *sb;
    const float *lut_a, *lut_b;
    double *out, *absdot;
} gemm_job;

static void* gemm_worker(void* arg) {
    gemm_job* j = (gemm_job*)arg;
    const int K = j->K, kb = (K + 127) / 128;
    float* arow = (float*)malloc(sizeof(float) * (size_t)K);
    float* brow = (float*)malloc(sizeof(float) * (size_t)K);
    for (int m = j->m0; m < j->m1; ++m) {
        for (int k = 0; k < K; ++k) {
            const float s = j->mode == 0 ? j->sa[0] : j->mode == 1 ? j->sa[m] : j->sa[(size_t)m * kb + k / 128];
            arow[k] = j->lut_a[j->A[(size_t)m * j->lda + k]] * s;
        }
        for (int n = 0; n < j->N; ++n) {
            for (int k = 0; k < K; ++k) {
                const float s = j->mode == 0 ? j->sb[0] : j->mode == 1 ? j->sb[n] : j->sb[(size_t)(n / 128) * kb + k / 128];
                brow[k] = j->lut_b[j->B[(size_t)n * j->ldb + k]] * s;
            }
            double acc = 0.0, aabs = 0.0;
            for (int k = 0; k < K; ++k) {
                const double p = (double)arow[k] * (double)brow[k];
                acc += p;
                aabs += fabs(p);
            }
            if (j->out) j->out[(size_t)m * j->N + n] = acc;
            if (j->absdot) j->absdot[(size_t)m * j->N + n] = aabs;
        }
    }
    free(arow); free(brow);
    return NULL;
}

void orc_gemm_nt_ref(int M, int N, int K,
                     const uint8_t* A, int lda, int a_is_e5m2, const float* a_descale,
                     const uint8_t* B, int ldb, int b_is_e5m2, const float* b_descale,
                     int scale_mode, double* out_ref, double* abs_dot, int threads) {
    float lut_a[256], lut_b[256];
    for (int b = 0; b < 256; ++b) {
        lut_a[b] = a_is_e5m2 ? orc_e5m2_unpack((uint8_t)b) : orc_e4m3_unpack((uint8_t)b);
        lut_b[b] = b_is_e5m2 ? orc_e5m2_unpack((uint8_t)b) : orc_e4m3_unpack((uint8_t)b);
    }
    if (threads < 1) threads = 1;
    if (threads > 64) threads = 64;
    if (threads > M) threads = M > 0 ? M : 1;
    pthread_t tid[64];
    gemm_job jobs[64];
    for (int t = 0; t < threads; ++t) {
        gemm_job j = { M, N, K, lda, ldb, scale_mode,
                       (int)((long long)M * t / threads), (int)((long long)M * (t + 1) / threads),
                       A, B, a_descale, b_descale, lut_a, lut_b, out_ref, abs_dot };
        jobs[t] = j;
        pthread_create(&tid[t], NULL, gemm_worker, &jobs[t]);
    }
    for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
}

/* ---- CPU linear forward ------------------------------------------------------
 * The reference CPU path computes a linear layer as one scalar dot product
 * per output element, accumulating in fp32 in index order
 * (kernels/cpu_amd_smoke.cpp:39-43,69-74), with the token rows split into
 * contiguous ranges [count*w/workers, count*(w+1)/workers) over worker
 * threads (src/cpu_trainer.cpp:89-108) and the weight stored [out,in]
 * (src/cpu_trainer.cpp:306-324).  Operands are the fp32 dequantised values. */
typedef struct {
    const float *x, *w; const uint16_t* bias; uint16_t* y; int K, N; size_t begin, end;
} linear_job;

static float scalar_dot(const float* left, const float* right, size_t count) {
    float result = 0.0f;
    for (size_t i = 0; i < count; ++i) result += left[i] * right[i];
    return result;
}

static void* linear_worker(void* arg) {
    linear_job* j = (linear_job*)arg;
    for (size_t t = j->begin; t < j->end; ++t)
        for (int n = 0; n < j->N; ++n) {
            float v = scalar_dot(j->x + t * (size_t)j->K, j->w + (size_t)n * j->K, (size_t)j->K);
            if (j->bias) v = orc_bf16_to_f32(orc_bf16_from_f32(v)) + orc_bf16_to_f32(j->bias[n]);
            j->y[t * (size_t)j->N + n] = orc_bf16_from_f32(v);
        }
    return NULL;
}

void orc_linear_forward_f32(const float* xq, const float* wq, const uint16_t* bias,
                            uint16_t* y, int T, int K, int N, int threads) {
    size_t workers = threads < 1 ? 1 : (size_t)threads;
    if (workers > (size_t)T) workers = (size_t)(T > 0 ? T : 1);
    if (workers > 256) workers = 256;
    pthread_t tid[256];
    linear_job jobs[256];
    for (size_t w = 0; w < workers; ++w) {
        linear_job j = { xq, wq, bias, y, K, N, (size_t)T * w / workers, (size_t)T * (w + 1) / workers };
        jobs[w] = j;
        if (workers == 1) { linear_worker(&jobs[0]); return; }
        pthread_create(&tid[w], NULL, linear_worker, &jobs[w]);
    }
    for (size_t w = 0; w < workers; ++w) pthread_join(tid[w], NULL);
}
