/*
 * CPU baseline: what the reference's RUST/RAYON backend executes for attention.
 * TEST/BENCH INFRASTRUCTURE ONLY (timed by bench.py's cpu_baseline leg, checked
 * by tests/); never part of the product path.
 *
 * On CPU the reference has no fused attention (src/models/flash_attention.rs:
 * 405-472 returns None off CUDA/CL/Metal), so `attention_with` runs the general
 * path with the probabilities materialised (src/tensor/mod.rs:2440-2446):
 *   1. S = (Q . K^T) * alpha   packed GEMM, src/runtime/cpu_gemm.rs:213-366
 *   2. P = softmax(S)          exp2((x-max)*(1/ln2)) * (1/sum),
 *                              src/tensor/nn.rs:1402-1410, elementwise.rs:213-225
 *   3. O = P . V               packed GEMM
 * The GEMM is restated with the reference's structure: tiles of MC x NC = 48 x 96
 * distributed over threads (rayon there, OpenMP here), the k extent walked in
 * chunks of KC = 256 that are summed into C, a 6 x 16 AVX2/FMA microkernel for
 * full panels and a scalar microkernel for the fringe (cpu_gemm.rs:27-30,
 * 96-186), batches processed one after the other (cpu_gemm.rs:257), a [n,k]
 * B operand packed to [k,n] once per batch (cpu_gemm.rs:235-248).
 * The scalar factor 1/sqrt(D) is applied as the GEMM's alpha in a final pass
 * over the tile (cpu_gemm.rs:16-18; src/schedule/host_gemm.rs:1034-1069).
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <omp.h>

#define MR 6
#define NR 16
#define MC 48
#define NC 96
#define KC 256

__attribute__((target("avx2,fma")))
static void micro_6x16(int kc, const float *ap, int a_rs, const float *bp, int b_ks,
                       float *c, int ldc, int first)
{
    __m256 acc[12];
    for (int i = 0; i < 12; ++i) acc[i] = _mm256_setzero_ps();
    for (int k = 0; k < kc; ++k) {
        const __m256 b0 = _mm256_loadu_ps(bp + (size_t)k * b_ks);
        const __m256 b1 = _mm256_loadu_ps(bp + (size_t)k * b_ks + 8);
        for (int i = 0; i < MR; ++i) {
            const __m256 a = _mm256_set1_ps(ap[(size_t)i * a_rs + k]);
            acc[2 * i] = _mm256_fmadd_ps(a, b0, acc[2 * i]);
            acc[2 * i + 1] = _mm256_fmadd_ps(a, b1, acc[2 * i + 1]);
        }
    }
    for (int i = 0; i < MR; ++i) {
        float *p = c + (size_t)i * ldc;
        __m256 v0 = acc[2 * i], v1 = acc[2 * i + 1];
        if (!first) {
            v0 = _mm256_add_ps(v0, _mm256_loadu_ps(p));
            v1 = _mm256_add_ps(v1, _mm256_loadu_ps(p + 8));
        }
        _mm256_storeu_ps(p, v0);
        _mm256_storeu_ps(p + 8, v1);
    }
}

static void micro_gen(int mr, int nr, int kc, const float *ap, int a_rs, const float *bp, int b_ks,
                      float *c, int ldc, int first)
{
    float acc[MR][NR];
    memset(acc, 0, sizeof(acc));
    for (int k = 0; k < kc; ++k)
        for (int j = 0; j < nr; ++j) {
            const float b = bp[(size_t)k * b_ks + j];
            for (int i = 0; i < mr; ++i) acc[i][j] += ap[(size_t)i * a_rs + k] * b;
        }
    for (int i = 0; i < mr; ++i)
        for (int j = 0; j < nr; ++j) {
            float *p = c + (size_t)i * ldc + j;
            if (first) *p = acc[i][j]; else *p += acc[i][j];
        }
}

/* C[m,n] = alpha * A[m,k] . B[k,n]; A row-major (k contiguous), B row-major. */
static void gemm_direct(int m, int n, int k, const float *a, const float *b, float *c, float alpha)
{
    const int nb = (n + NC - 1) / NC;
    const int tasks = ((m + MC - 1) / MC) * nb;
#pragma omp parallel for schedule(dynamic, 1)
    for (int task = 0; task < tasks; ++task) {
        const int m0 = (task / nb) * MC, n0 = (task % nb) * NC;
        const int m_cnt = (MC < m - m0) ? MC : m - m0;
        const int n_cnt = (NC < n - n0) ? NC : n - n0;
        const int mpan = (m_cnt + MR - 1) / MR, npan = (n_cnt + NR - 1) / NR;
        int first = 1;
        for (int k0 = 0; k0 < k; k0 += KC) {
            const int kc = (KC < k - k0) ? KC : k - k0;
            for (int ip = 0; ip < mpan; ++ip) {
                const int mr = (MR < m_cnt - ip * MR) ? MR : m_cnt - ip * MR;
                for (int jp = 0; jp < npan; ++jp) {
                    const int nr = (NR < n_cnt - jp * NR) ? NR : n_cnt - jp * NR;
                    float *cb = c + (size_t)(m0 + ip * MR) * n + (n0 + jp * NR);
                    const float *ap = a + (size_t)(m0 + ip * MR) * k + k0;
                    const float *bp = b + (size_t)k0 * n + (n0 + jp * NR);
                    if (mr == MR && nr == NR) micro_6x16(kc, ap, k, bp, n, cb, n, first);
                    else micro_gen(mr, nr, kc, ap, k, bp, n, cb, n, first);
                }
            }
            first = 0;
        }
        if (alpha != 1.0f)
            for (int i = 0; i < m_cnt; ++i)
                for (int j = 0; j < n_cnt; ++j) c[(size_t)(m0 + i) * n + n0 + j] *= alpha;
    }
}

/* softmax over the last axis of s [rows, n], in place. */
static void softmax_rows(float *s, int rows, int n)
{
    const float inv_ln2 = (float)(1.0 / 0.6931471805599453);
#pragma omp parallel for schedule(static)
    for (int i = 0; i < rows; ++i) {
        float *x = s + (size_t)i * n;
        float mx = -INFINITY;
        for (int j = 0; j < n; ++j) mx = x[j] > mx ? x[j] : mx;
        float sum = 0.f;
        for (int j = 0; j < n; ++j) {
            x[j] = exp2f((x[j] - mx) * inv_ln2);
            sum += x[j];
        }
        const float r = 1.0f / sum;
        for (int j = 0; j < n; ++j) x[j] *= r;
    }
}

/* Attention forward for `heads` (batch*head) slices laid out [heads, N, D],
 * no mask; causal != 0 adds the lower-triangular mask before the softmax
 * (src/tensor/mod.rs:2405-2433).  scratch needs N*N + N*D floats.
 * Returns the number of threads OpenMP used. */
int ar_cpu_sdpa(const float *q, const float *k, const float *v, float *o,
                int heads, int N, int D, int causal, float *scratch)
{
    float *s = scratch;
    float *kt = scratch + (size_t)N * N;
    const float alpha = 1.0f / sqrtf((float)D);
    for (int h = 0; h < heads; ++h) {
        const float *qh = q + (size_t)h * N * D, *kh = k + (size_t)h * N * D, *vh = v + (size_t)h * N * D;
        /* pack K [n,k] -> [k,n] (cpu_gemm.rs:235-248) */
#pragma omp parallel for schedule(static)
        for (int d = 0; d < D; ++d)
            for (int j = 0; j < N; ++j) kt[(size_t)d * N + j] = kh[(size_t)j * D + d];
        gemm_direct(N, N, D, qh, kt, s, alpha);
        if (causal) {
#pragma omp parallel for schedule(static)
            for (int i = 0; i < N; ++i)
                for (int j = i + 1; j < N; ++j) s[(size_t)i * N + j] = -INFINITY;
        }
        softmax_rows(s, N, N);
        gemm_direct(N, D, N, s, vh, o + (size_t)h * N * D, 1.0f);
    }
    return omp_get_max_threads();
}
