/*
 * CPU oracle for the fused-attention hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic the reference
 * (apexys/autorust) performs for attention.  It exists so that the HIP kernels
 * can be checked against something that does not share code with them.  Only
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it;
 * the product (autorust_amd/, libarhip.so) never does.
 *
 * Build: `make -C oracle` (gcc -O2 -ffp-contract=off: no FMA contraction, so
 * every fp32 operation below is one IEEE-754 binary32 operation in the order
 * written).
 *
 * All "head" functions work on ONE (batch, head) pair: q [N,D], k [N,D],
 * v [N,D] row-major, optional additive mask [N,N] row-major, and evaluate the
 * query rows listed in rows[0..nrows) (rows == NULL: all N rows, nrows == N),
 * writing out [nrows, D].  kv_len (1..N, or <0 for "N") excludes keys
 * j >= kv_len: that is the key-padding mask of the decoder configuration; the
 * reference expresses it as an additive -inf mask on the general path
 * (src/tensor/mod.rs:2417-2433) and as `gj < N` in the kernels
 * (src/runtime/cuda_flash.rs:104-113).
 *
 * What pins each function (see tests/test_oracle.py):
 *   ar_head_sdpa_f32/f64  the six reference-held vectors of
 *                         tests/attention_golden.rs (tolerance of
 *                         tests/nn_attention.rs:20), torch's CPU SDPA, fp64.
 *   ar_head_lse_f64       scipy.special.logsumexp / torch.logsumexp (library).
 *   ar_head_flash_f32     equals SDPA by the online-softmax identity; special
 *                         cases by brute force (fully masked row -> mean of V).
 *   ar_head_bf16          bf16 RNE against torch.bfloat16 casts; equals
 *                         tests/flash_cuda_masks.rs:41-104 with round=true.
 *   ar_quant_blocks       block size 1 == the reference per-row rule
 *                         (src/runtime/cuda_flash_sage.rs:209-222); max is
 *                         order independent; tiny brute force in Python ints.
 *   ar_logits_i32         exact integer arithmetic; known answer of
 *                         tests/sage_layout_probe.rs:73-84.
 *   ar_head_sage          re-derived with torch tensor operations (integer matmul,
 *                         (sq*sk)*scale, additive mask, causal, key lengths,
 *                         bf16(p) @ bf16(v) / sum p) over causal x mask x kv_len x
 *                         GQA at block sizes (1,1), (128,64), (32,16); closed forms;
 *                         single-line mutations of the masks and rounding points
 *                         each fail a test (tests/test_oracle.py).
 *   ar_k_mean             PARITY UNPINNED by the reference (it has no
 *                         K smoothing, src/runtime/cuda_flash_sage.rs:13-14).
 *                         Pinned by: softmax shift invariance, fp64 mean within
 *                         fp32 rounding, and the fixed summation order below.
 *   per-block scales      PARITY UNPINNED by the reference (it scales per row);
 *                         pinned by reduction to the per-row rule at block 1.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define AR_NEG (-1e30f)

/* ---------------------------------------------------------------- bf16 --- */

/* Round-to-nearest-even f32 -> bf16 -> f32.
 * tests/flash_cuda_bf16.rs:26-30, src/dtype/mod.rs:973-981. NaN kept quiet. */
float ar_bf16_round(float x)
{
    uint32_t bits;
    memcpy(&bits, &x, 4);
    if ((bits & 0x7fffffffu) > 0x7f800000u) { /* NaN: keep it a NaN */
        bits = (bits | 0x00400000u) & 0xffff0000u;
    } else {
        uint32_t lsb = (bits >> 16) & 1u;
        bits = (bits + 0x7fffu + lsb) & 0xffff0000u;
    }
    float r;
    memcpy(&r, &bits, 4);
    return r;
}

uint16_t ar_bf16_bits(float x)
{
    float r = ar_bf16_round(x);
    uint32_t bits;
    memcpy(&bits, &r, 4);
    return (uint16_t)(bits >> 16);
}

void ar_bf16_round_array(const float *x, float *y, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) y[i] = ar_bf16_round(x[i]);
}

void ar_bf16_bits_array(const float *x, uint16_t *y, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) y[i] = ar_bf16_bits(x[i]);
}

static inline int row_of(const int *rows, int r) { return rows ? rows[r] : r; }
static inline int kvn(int kv_len, int N) { return (kv_len < 0 || kv_len > N) ? N : kv_len; }

/* ------------------------------------------------- general SDPA, fp32 --- */

/* The general path: src/tensor/mod.rs:2395-2446 with softmax of
 * src/tensor/nn.rs:1402-1410 and exp(x) = exp2(x * (1/ln 2))
 * (src/tensor/elementwise.rs:213-225).
 *   qk   = (sum_d q*k, sequential fp32) / sqrt(D)
 *   qk  += mask          (causal: tril bool -> 0 / -inf)
 *   e    = exp2((qk - max) * (1/ln2));  p = e * (1 / sum e);  out = sum_j p*v
 * A row whose keys are all masked with -inf yields NaN, as in the reference. */
void ar_head_sdpa_f32(const float *q, const float *k, const float *v, const float *mask,
                      int N, int D, int causal, int kv_len,
                      const int *rows, int nrows, float *out)
{
    const int L = kvn(kv_len, N);
    const float sqrt_d = (float)sqrt((double)D);
    const float inv_ln2 = (float)(1.0 / 0.6931471805599453);
#pragma omp parallel
    {
        float *s = (float *)malloc(sizeof(float) * (size_t)N);
#pragma omp for schedule(dynamic, 4)
        for (int r = 0; r < nrows; ++r) {
            const int i = row_of(rows, r);
            float mx = -INFINITY;
            for (int j = 0; j < N; ++j) {
                float dot = 0.f;
                for (int t = 0; t < D; ++t) dot += q[(size_t)i * D + t] * k[(size_t)j * D + t];
                float x = dot / sqrt_d;
                if (mask) x += mask[(size_t)i * N + j];
                if (causal && j > i) x += -INFINITY;
                if (j >= L) x += -INFINITY;
                s[j] = x;
                if (x > mx) mx = x;
            }
            float sum = 0.f;
            for (int j = 0; j < N; ++j) {
                s[j] = exp2f((s[j] - mx) * inv_ln2);
                sum += s[j];
            }
            const float recip = 1.0f / sum;
            for (int t = 0; t < D; ++t) {
                float acc = 0.f;
                for (int j = 0; j < N; ++j) acc += (s[j] * recip) * v[(size_t)j * D + t];
                out[(size_t)r * D + t] = acc;
            }
        }
        free(s);
    }
}

/* Same function of the inputs evaluated in binary64 throughout and rounded
 * once at the end: the "truth" the fp32 variants are measured against. */
void ar_head_sdpa_f64(const float *q, const float *k, const float *v, const float *mask,
                      int N, int D, int causal, int kv_len, double scale,
                      const int *rows, int nrows, float *out)
{
    const int L = kvn(kv_len, N);
#pragma omp parallel
    {
        double *s = (double *)malloc(sizeof(double) * (size_t)N);
#pragma omp for schedule(dynamic, 4)
        for (int r = 0; r < nrows; ++r) {
            const int i = row_of(rows, r);
            double mx = -INFINITY;
            for (int j = 0; j < N; ++j) {
                double x = -INFINITY;
                if (!(causal && j > i) && j < L) {
                    double dot = 0.0;
                    for (int t = 0; t < D; ++t)
                        dot += (double)q[(size_t)i * D + t] * (double)k[(size_t)j * D + t];
                    x = dot * scale;
                    if (mask) x += (double)mask[(size_t)i * N + j];
                }
                s[j] = x;
                if (x > mx) mx = x;
            }
            double sum = 0.0;
            for (int j = 0; j < N; ++j) {
                s[j] = exp(s[j] - mx);
                sum += s[j];
            }
            for (int t = 0; t < D; ++t) {
                double acc = 0.0;
                for (int j = 0; j < N; ++j) acc += s[j] * (double)v[(size_t)j * D + t];
                out[(size_t)r * D + t] = (float)(acc / sum);
            }
        }
        free(s);
    }
}

/* Log-sum-exp of the masked, scaled logits of every evaluated row, in binary64:
 * lse[r] = log(sum_j exp(s_rj)), the statistic the reference's training forward saves as
 * LSE = m + log(l) (src/runtime/cuda_flash_train.rs:5-11,141).  A row without any visible
 * key gets the finite sentinel -1e30 like there. */
void ar_head_lse_f64(const float *q, const float *k, const float *mask,
                     int N, int D, int causal, int kv_len, double scale,
                     const int *rows, int nrows, float *lse)
{
    const int L = kvn(kv_len, N);
#pragma omp parallel for schedule(dynamic, 4)
    for (int r = 0; r < nrows; ++r) {
        const int i = row_of(rows, r);
        double mx = -INFINITY;
        double *s = (double *)malloc(sizeof(double) * (size_t)N);
        for (int j = 0; j < N; ++j) {
            double x = -INFINITY;
            if (!(causal && j > i) && j < L) {
                double dot = 0.0;
                for (int t = 0; t < D; ++t) dot += (double)q[(size_t)i * D + t] * (double)k[(size_t)j * D + t];
                x = dot * scale;
                if (mask) x += (double)mask[(size_t)i * N + j];
            }
            s[j] = x;
            if (x > mx) mx = x;
        }
        double sum = 0.0;
        for (int j = 0; j < N; ++j) sum += exp(s[j] - mx);
        lse[r] = (mx > -INFINITY) ? (float)(mx + log(sum)) : AR_NEG;
        free(s);
    }
}

/* ------------------------------------------- scalar FA2 kernel, fp32 --- */

/* The fp32 exact-mode kernel, src/runtime/cuda_flash.rs:53-141, restated with
 * its block structure (BQ queries per block, BK keys per step) because the
 * block structure is visible in the results:
 *   - keys are visited up to kend = causal ? min(N, qblk+BQ) : N, rounded up to
 *     whole BK steps; a masked or out-of-range key contributes the finite
 *     sentinel -1e30, not -inf (cuda_flash.rs:105,112);
 *   - a row whose every visited key carries the sentinel gets
 *     p = exp(-1e30 - -1e30) = 1 for each of them, i.e. the mean of the visited
 *     V rows (zero rows past N), where the general path would give NaN;
 *   - normalisation is acc * (l > 0 ? 1/l : 0) (cuda_flash.rs:138-139).
 * Generalised: head_dim D and `scale` are parameters (the reference hard-codes
 * 64 and 0.125), and kv_len bounds the keys like N does. */
void ar_head_flash_f32(const float *q, const float *k, const float *v, const float *mask,
                       int N, int D, int causal, int kv_len, float scale, int BQ, int BK,
                       const int *rows, int nrows, float *out)
{
    const int L = kvn(kv_len, N);
#pragma omp parallel
    {
        float *acc = (float *)malloc(sizeof(float) * (size_t)D);
        float *s = (float *)malloc(sizeof(float) * (size_t)BK);
#pragma omp for schedule(dynamic, 4)
        for (int r = 0; r < nrows; ++r) {
            const int row = row_of(rows, r);
            const int qblk = (row / BQ) * BQ;
            int kend = causal ? (N < qblk + BQ ? N : qblk + BQ) : N;
            if (kend > L) kend = L;
            for (int t = 0; t < D; ++t) acc[t] = 0.f;
            float m = AR_NEG, l = 0.f;
            for (int k0 = 0; k0 < kend; k0 += BK) {
                float mnew = m;
                for (int j = 0; j < BK; ++j) {
                    const int gj = k0 + j;
                    float dot = AR_NEG;
                    if (gj < L) {
                        dot = 0.f;
                        for (int t = 0; t < D; ++t) dot += q[(size_t)row * D + t] * k[(size_t)gj * D + t];
                        dot *= scale;
                        if (mask) dot += mask[(size_t)row * N + gj];
                        if (causal && gj > row) dot = AR_NEG;
                    }
                    s[j] = dot;
                    mnew = fmaxf(mnew, dot);
                }
                const float alpha = expf(m - mnew);
                float sum = 0.f;
                for (int j = 0; j < BK; ++j) {
                    s[j] = expf(s[j] - mnew);
                    sum += s[j];
                }
                l = l * alpha + sum;
                for (int t = 0; t < D; ++t) {
                    float a = acc[t] * alpha;
                    for (int j = 0; j < BK; ++j) {
                        const int gj = k0 + j;
                        const float vv = (gj < L) ? v[(size_t)gj * D + t] : 0.f;
                        a += s[j] * vv;
                    }
                    acc[t] = a;
                }
                m = mnew;
            }
            const float inv = (l > 0.f) ? 1.f / l : 0.f;
            for (int t = 0; t < D; ++t) out[(size_t)r * D + t] = acc[t] * inv;
        }
        free(acc);
        free(s);
    }
}

/* ------------------------------------------------ bf16-emulating ref --- */

/* tests/flash_cuda_masks.rs:41-104 with round = true (and
 * tests/flash_cuda_bf16.rs:33-64, its mask-free special case): operands
 * rounded to bf16, fp32 dot / scale / mask, fp32 exp and sum of the UNROUNDED
 * probabilities, P rounded to bf16 for the P.V product, fp32 accumulate,
 * result acc/sum rounded to bf16.  q/k/v may be given unrounded; they are
 * rounded here.  round_out = 0 keeps acc/sum in fp32 (the Sage kernel's
 * output convention, src/runtime/cuda_flash_sage.rs:401-412). */
void ar_head_bf16(const float *q, const float *k, const float *v, const float *mask,
                  int N, int D, int causal, int kv_len, float scale, int round_out,
                  const int *rows, int nrows, float *out)
{
    const int L = kvn(kv_len, N);
    float *kb = (float *)malloc(sizeof(float) * (size_t)N * D);
    float *vb = (float *)malloc(sizeof(float) * (size_t)N * D);
    ar_bf16_round_array(k, kb, (int64_t)N * D);
    ar_bf16_round_array(v, vb, (int64_t)N * D);
#pragma omp parallel
    {
        float *s = (float *)malloc(sizeof(float) * (size_t)N);
        float *qb = (float *)malloc(sizeof(float) * (size_t)D);
#pragma omp for schedule(dynamic, 4)
        for (int r = 0; r < nrows; ++r) {
            const int i = row_of(rows, r);
            for (int t = 0; t < D; ++t) qb[t] = ar_bf16_round(q[(size_t)i * D + t]);
            float mx = -INFINITY;
            for (int j = 0; j < N; ++j) {
                float x = -INFINITY;
                if (!(causal && j > i) && j < L) {
                    float dot = 0.f;
                    for (int t = 0; t < D; ++t) dot += qb[t] * kb[(size_t)j * D + t];
                    dot *= scale;
                    if (mask) dot += mask[(size_t)i * N + j];
                    x = dot;
                }
                s[j] = x;
                if (x > mx) mx = x;
            }
            float sum = 0.f;
            for (int j = 0; j < N; ++j) {
                s[j] = expf(s[j] - mx);
                sum += s[j];
            }
            for (int t = 0; t < D; ++t) {
                float acc = 0.f;
                for (int j = 0; j < N; ++j) acc += ar_bf16_round(s[j]) * vb[(size_t)j * D + t];
                const float o = acc / sum;
                out[(size_t)r * D + t] = round_out ? ar_bf16_round(o) : o;
            }
        }
        free(s);
        free(qb);
    }
    free(kb);
    free(vb);
}

/* --------------------------------------------------- Sage quantiser --- */

/* Mean of K over the N tokens of one (batch, kv-head): mean[d].
 * NOT IN THE REFERENCE (src/runtime/cuda_flash_sage.rs:13-14: "SmoothK is not
 * implemented yet").  The summation order is part of the definition, because
 * the int8 tensors derived from it must be bit-exact:
 *   part[c][d] = ((k[64c+0][d] + k[64c+1][d]) + ...)   tokens of chunk c in order
 *   tot[d]     = ((part[0][d] + part[1][d]) + ...)     chunks in order
 *   mean[d]    = tot[d] / (float)N
 * all in fp32. */
void ar_k_mean(const float *k, int N, int D, float *mean)
{
    const int CH = 64;
    for (int d = 0; d < D; ++d) {
        float tot = 0.f;
        for (int c0 = 0; c0 < N; c0 += CH) {
            const int c1 = (c0 + CH < N) ? c0 + CH : N;
            float part = 0.f;
            for (int j = c0; j < c1; ++j) part += k[(size_t)j * D + d];
            tot += part;
        }
        mean[d] = tot / (float)N;
    }
}

/* Symmetric int8 quantisation of x [N,D] (one head) in blocks of `blk` tokens,
 * after subtracting sub[d] when sub != NULL.
 *   scale = absmax > 0 ? absmax / 127 : 1          cuda_flash_sage.rs:209-213
 *   inv   = 1 / scale                              cuda_flash_sage.rs:218
 *   q     = clamp(rint(x * inv), -127, 127)        cuda_flash_sage.rs:130,219-221
 * with absmax taken over the whole block of tokens (blk == 1 is the reference's
 * per-row rule).  rint is round-half-to-even (`__float2int_rn`).
 * use_div != 0 switches to q = clamp(round_ties_even(x / scale)), the variant
 * the reference's own CPU emulation uses (tests/sage_int8.rs:26-29,56-57); it
 * can differ from the kernel rule by one step on ties and exists only so that
 * the difference can be measured. */
void ar_quant_blocks(const float *x, int N, int D, int blk, const float *sub, int use_div,
                     int8_t *q, float *scales)
{
    const int nblk = (N + blk - 1) / blk;
    for (int b = 0; b < nblk; ++b) {
        const int r0 = b * blk;
        const int r1 = (r0 + blk < N) ? r0 + blk : N;
        float mx = 0.f;
        for (int i = r0; i < r1; ++i)
            for (int d = 0; d < D; ++d) {
                float xv = x[(size_t)i * D + d];
                if (sub) xv = xv - sub[d];
                mx = fmaxf(mx, fabsf(xv));
            }
        const float scale = (mx > 0.f) ? mx / 127.0f : 1.f;
        const float inv = 1.f / scale;
        scales[b] = scale;
        for (int i = r0; i < r1; ++i)
            for (int d = 0; d < D; ++d) {
                float xv = x[(size_t)i * D + d];
                if (sub) xv = xv - sub[d];
                const float y = use_div ? xv / scale : xv * inv;
                int iv = (int)rintf(y);
                iv = iv < -127 ? -127 : (iv > 127 ? 127 : iv);
                q[(size_t)i * D + d] = (int8_t)iv;
            }
    }
}

/* int32 logits acc[i][j] = sum_d q8[i][d] * k8[j][d] for rows [i0,i1) and
 * keys [j0,j1): src/runtime/cuda_flash_sage.rs:294-304 (exact in integers). */
void ar_logits_i32(const int8_t *q8, const int8_t *k8, int D, int i0, int i1, int j0, int j1,
                   int32_t *out)
{
    const int W = j1 - j0;
    for (int i = i0; i < i1; ++i)
        for (int j = j0; j < j1; ++j) {
            int32_t acc = 0;
            for (int d = 0; d < D; ++d) acc += (int32_t)q8[(size_t)i * D + d] * (int32_t)k8[(size_t)j * D + d];
            out[(size_t)(i - i0) * W + (j - j0)] = acc;
        }
}

/* Attention from already-quantised Q/K with block scales, emulating the
 * quantised kernel (src/runtime/cuda_flash_sage.rs:280-412, and its CPU
 * emulation tests/sage_int8.rs:33-76):
 *   s   = (float)acc_i32 * ((sq * sk) * scale)     cuda_flash_sage.rs:315-322
 *   p   = exp(s - max);  sum over unrounded p
 *   out = (sum_j bf16(p_j) * bf16(v_j)) / sum      fp32, or bf16 if round_out
 * sq is indexed by i / bq, sk by j / bk. */
void ar_head_sage(const int8_t *q8, const int8_t *k8, const float *sq, const float *sk,
                  const float *v, const float *mask, int N, int D, int bq, int bk,
                  int causal, int kv_len, float scale, int round_out,
                  const int *rows, int nrows, float *out)
{
    const int L = kvn(kv_len, N);
    float *vb = (float *)malloc(sizeof(float) * (size_t)N * D);
    ar_bf16_round_array(v, vb, (int64_t)N * D);
#pragma omp parallel
    {
        float *s = (float *)malloc(sizeof(float) * (size_t)N);
#pragma omp for schedule(dynamic, 4)
        for (int r = 0; r < nrows; ++r) {
            const int i = row_of(rows, r);
            float mx = -INFINITY;
            for (int j = 0; j < N; ++j) {
                float x = -INFINITY;
                if (!(causal && j > i) && j < L) {
                    int32_t acc = 0;
                    for (int t = 0; t < D; ++t)
                        acc += (int32_t)q8[(size_t)i * D + t] * (int32_t)k8[(size_t)j * D + t];
                    const float a = (sq[i / bq] * sk[j / bk]) * scale;
                    x = (float)acc * a;
                    if (mask) x += mask[(size_t)i * N + j];
                }
                s[j] = x;
                if (x > mx) mx = x;
            }
            float sum = 0.f;
            for (int j = 0; j < N; ++j) {
                s[j] = expf(s[j] - mx);
                sum += s[j];
            }
            for (int t = 0; t < D; ++t) {
                float acc = 0.f;
                for (int j = 0; j < N; ++j) acc += ar_bf16_round(s[j]) * vb[(size_t)j * D + t];
                const float o = acc / sum;
                out[(size_t)r * D + t] = round_out ? ar_bf16_round(o) : o;
            }
        }
        free(s);
    }
    free(vb);
}
