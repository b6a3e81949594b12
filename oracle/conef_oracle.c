/*
 * conef_oracle.c -- CPU restatement of the ConEF compress + error-feedback
 * arithmetic.  TEST INFRASTRUCTURE ONLY: it exists to check the HIP kernels
 * and to be timed as a CPU baseline.  Nothing in the shipped package may call it.
 *
 * Every function cites the reference lines it restates (paths relative to the
 * reference checkout).  Where the reference leaves the floating-point
 * accumulation order open (float atomicAdd), this file fixes one order:
 * ascending column index, sequential fp32 adds onto the sketch cell.
 *
 * Plain C99, scalar, single threaded.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------- hash ---- */

/* communication/compressors/CountSketch.py:7-18.
 * `h` is a signed int there: the three `>>` are arithmetic shifts, the two
 * multiplications by 0x85ebca6b / 0xc2b2ae35 happen in unsigned arithmetic and
 * wrap, and the final arithmetic `h ^= h >> 16` always clears the sign bit, so
 * the C `%` sees a non-negative left operand. */
static uint32_t mix32(int32_t value, int32_t a, int32_t b)
{
    uint32_t h = (uint32_t)a * (uint32_t)value + (uint32_t)b;
    h ^= (uint32_t)((int32_t)h >> 16);
    h *= 0x85ebca6bu;
    h ^= (uint32_t)((int32_t)h >> 13);
    h *= 0xc2b2ae35u;
    h ^= (uint32_t)((int32_t)h >> 16);
    return h;
}

int32_t conef_oracle_mix(int32_t value, int32_t a, int32_t b)
{
    return (int32_t)mix32(value, a, b);
}

int32_t conef_oracle_hash(int32_t value, int32_t range, int32_t a, int32_t b)
{
    int32_t h = (int32_t)mix32(value, a, b);
    return h % range;
}

/* Bucket and sign of every column of a row, CountSketch.py:60-62:
 * bucket = hash(i, W, a, b); sign bit = hash(i, W, a+2, b+3) & 1 (the parity is
 * taken AFTER the modulo, so it depends on W); sign = bit ? +1 : -1. */
void conef_oracle_hash_table(int32_t *bucket, int32_t *sign, int64_t d, int32_t w,
                             int32_t a, int32_t b, int32_t sa, int32_t sb)
{
    for (int64_t i = 0; i < d; ++i) {
        bucket[i] = conef_oracle_hash((int32_t)i, w, a, b);
        sign[i] = (conef_oracle_hash((int32_t)i, w, sa, sb) & 1) ? 1 : -1;
    }
}

/* CountSketch.py:20-25 */
static float median3(float a, float b, float c)
{
    return fmaxf(fminf(a, b), fminf(fmaxf(a, b), c));
}

float conef_oracle_median3(float a, float b, float c) { return median3(a, b, c); }

/* ------------------------------------------------- one-hash count sketch ---- */

/* dense_cs_query, CountSketch.py:70-98:  x[r,i] += (sign_i * cs[r,h_i]) * alpha,
 * all in fp32, left to right. */
void conef_oracle_cs_query(float *x, const float *cs, int64_t n, int64_t d, int32_t w,
                           float alpha, int32_t a, int32_t b)
{
    for (int64_t r = 0; r < n; ++r) {
        const float *row = cs + r * (int64_t)w;
        float *xr = x + r * d;
        for (int64_t i = 0; i < d; ++i) {
            int32_t j = conef_oracle_hash((int32_t)i, w, a, b);
            float sign = (conef_oracle_hash((int32_t)i, w, a + 2, b + 3) & 1) ? 1.0f : -1.0f;
            float update = sign * row[j] * alpha;
            xr[i] = xr[i] + update;
        }
    }
}

/* dense_cs_update, CountSketch.py:27-67.  `aux` is the snapshot of the row
 * taken before any add (:47-52).  The term is evaluated in double because of
 * the literal `1.` (:63) and rounded to float on assignment; the adds onto the
 * sketch cell are fp32.  Order fixed here: ascending i. */
void conef_oracle_cs_update(const float *vec, float *cs, int64_t n, int64_t d, int32_t w,
                            float beta, int32_t a, int32_t b)
{
    float *aux = (float *)malloc(sizeof(float) * (size_t)w);
    for (int64_t r = 0; r < n; ++r) {
        float *row = cs + r * (int64_t)w;
        const float *vr = vec + r * d;
        memcpy(aux, row, sizeof(float) * (size_t)w);
        for (int64_t i = 0; i < d; ++i) {
            float value = vr[i];
            int32_t j = conef_oracle_hash((int32_t)i, w, a, b);
            float sign = (conef_oracle_hash((int32_t)i, w, a + 2, b + 3) & 1) ? 1.0f : -1.0f;
            float update = (float)((double)sign *
                                   ((double)value - (1. - (double)beta) * (double)sign * (double)aux[j]));
            row[j] = row[j] + update;
        }
    }
    free(aux);
}

/* ----------------------------------------------- three-hash count sketch ---- */

static const int32_t H3A[3] = {994443, 4113759, 9171025};  /* CountSketchHash3.py:40 */
static const int32_t H3B[3] = {609478, 2949676, 2171464};  /* CountSketchHash3.py:41 */
/* sign seeds: (a0+2,b0+3) :68, (a1+4,b1+5) :77, (a2+8,b2+4) in update :85 but
 * (a2+8,b2+7) in query :137 -- the reference disagrees with itself and the
 * restatement keeps both. */
static const int32_t H3SA[3] = {2, 4, 8};
static const int32_t H3SB_UPDATE[3] = {3, 5, 4};
static const int32_t H3SB_QUERY[3] = {3, 5, 7};

/* 3-hash dense_cs_query, CountSketchHash3.py:101-147 */
void conef_oracle_cs3_query(float *x, const float *cs0, const float *cs1, const float *cs2,
                            int64_t n, int64_t d, int32_t w, float alpha)
{
    const float *mem[3] = {cs0, cs1, cs2};
    for (int64_t r = 0; r < n; ++r) {
        float *xr = x + r * d;
        for (int64_t i = 0; i < d; ++i) {
            float u[3];
            for (int k = 0; k < 3; ++k) {
                int32_t j = conef_oracle_hash((int32_t)i, w, H3A[k], H3B[k]);
                float sign = (conef_oracle_hash((int32_t)i, w, H3A[k] + H3SA[k], H3B[k] + H3SB_QUERY[k]) & 1)
                                 ? 1.0f : -1.0f;
                u[k] = sign * mem[k][r * (int64_t)w + j] * alpha;
            }
            xr[i] = xr[i] + median3(u[0], u[1], u[2]);
        }
    }
}

/* 3-hash dense_cs_update, CountSketchHash3.py:27-98.
 *   u0 = sign0 * aux0[h0] * (beta - 1.0)        float*float, then *double  (:70)
 *   u1 = -(1. - beta) * sign1 * aux1[h1]        double chain              (:79)
 *   u2 = -(1. - beta) * sign2 * aux2[h2]                                   (:87)
 * each rounded to float; m = median(u0,u1,u2); mem_k[h_k] += sign_k*(m + v) in fp32. */
void conef_oracle_cs3_update(const float *vec, float *cs0, float *cs1, float *cs2,
                             int64_t n, int64_t d, int32_t w, float beta)
{
    float *mem[3] = {cs0, cs1, cs2};
    float *aux = (float *)malloc(sizeof(float) * 3 * (size_t)w);
    for (int64_t r = 0; r < n; ++r) {
        for (int k = 0; k < 3; ++k)
            memcpy(aux + (size_t)k * w, mem[k] + r * (int64_t)w, sizeof(float) * (size_t)w);
        const float *vr = vec + r * d;
        for (int64_t i = 0; i < d; ++i) {
            float value = vr[i];
            int32_t j[3];
            float sign[3], u[3];
            for (int k = 0; k < 3; ++k) {
                j[k] = conef_oracle_hash((int32_t)i, w, H3A[k], H3B[k]);
                sign[k] = (conef_oracle_hash((int32_t)i, w, H3A[k] + H3SA[k], H3B[k] + H3SB_UPDATE[k]) & 1)
                              ? 1.0f : -1.0f;
            }
            u[0] = (float)((double)(sign[0] * aux[j[0]]) * ((double)beta - 1.0));
            u[1] = (float)(-(1. - (double)beta) * (double)sign[1] * (double)aux[(size_t)w + j[1]]);
            u[2] = (float)(-(1. - (double)beta) * (double)sign[2] * (double)aux[2 * (size_t)w + j[2]]);
            float m = median3(u[0], u[1], u[2]);
            for (int k = 0; k < 3; ++k) {
                float *cell = mem[k] + r * (int64_t)w + j[k];
                *cell = *cell + sign[k] * (m + value);
            }
        }
    }
    free(aux);
}

/* --------------------------------------------------------- Gram-Schmidt ---- */

/* _orthogonalize, communication/powerSGD_hook.py:12-44 (copy at
 * hPowerSGD_hook.py:13-45).  Column by column: col /= ||col||_2 (+ eps when
 * eps != 0), then every later column loses its projection on col:
 * rest -= sum(col * rest, dim=0) * col.  Norms and dot products are reduced in
 * double and rounded to fp32 once (torch's own fp32 reduction order is not
 * specified); everything elementwise is fp32 as in the reference.
 * `a` is row-major [rows, cols] with leading dimension `ld`. */
void conef_oracle_gram_schmidt(float *a, int64_t rows, int64_t cols, int64_t ld, float eps)
{
    for (int64_t i = 0; i < cols; ++i) {
        double ss = 0.0;
        for (int64_t k = 0; k < rows; ++k) {
            double v = a[k * ld + i];
            ss += v * v;
        }
        float nrm = (float)sqrt(ss);
        float den = (eps == 0.0f) ? nrm : nrm + eps;
        for (int64_t k = 0; k < rows; ++k)
            a[k * ld + i] = a[k * ld + i] / den;
        for (int64_t j = i + 1; j < cols; ++j) {
            double dot = 0.0;
            for (int64_t k = 0; k < rows; ++k) {
                float prod = a[k * ld + i] * a[k * ld + j];   /* col * rest is an fp32 tensor */
                dot += (double)prod;
            }
            float dotf = (float)dot;
            for (int64_t k = 0; k < rows; ++k)
                a[k * ld + j] = a[k * ld + j] - dotf * a[k * ld + i];
        }
    }
}

/* ------------------------------------------------ skinny PowerSGD products ---- */

/* P = M Q, powerSGD_hook.py:498.  M [n,m], Q [m,r], P [n,r], row-major.
 * Accumulated in double, rounded once. */
void conef_oracle_mq(const float *mat, const float *q, float *p, int64_t n, int64_t m, int64_t r)
{
    for (int64_t i = 0; i < n; ++i)
        for (int64_t c = 0; c < r; ++c) {
            double acc = 0.0;
            for (int64_t k = 0; k < m; ++k)
                acc += (double)mat[i * m + k] * (double)q[k * r + c];
            p[i * r + c] = (float)acc;
        }
}

/* Q = M^T P, powerSGD_hook.py:532 */
void conef_oracle_mtp(const float *mat, const float *p, float *q, int64_t n, int64_t m, int64_t r)
{
    double *acc = (double *)calloc((size_t)(m * r), sizeof(double));
    for (int64_t i = 0; i < n; ++i)
        for (int64_t k = 0; k < m; ++k) {
            double v = mat[i * m + k];
            for (int64_t c = 0; c < r; ++c)
                acc[k * r + c] += v * (double)p[i * r + c];
        }
    for (int64_t t = 0; t < m * r; ++t)
        q[t] = (float)acc[t];
    free(acc);
}

/* M = P Q^T, powerSGD_hook.py:551 */
void conef_oracle_pqt(const float *p, const float *q, float *mat, int64_t n, int64_t m, int64_t r)
{
    for (int64_t i = 0; i < n; ++i)
        for (int64_t k = 0; k < m; ++k) {
            double acc = 0.0;
            for (int64_t c = 0; c < r; ++c)
                acc += (double)p[i * r + c] * (double)q[k * r + c];
            mat[i * m + k] = (float)acc;
        }
}

/* ------------------------------------------ fused steps, for CPU timing ---- */

/* One RandomBlock + ConEF step on one [n,m] tensor, RandomBlock_hook.py:190,
 * 216-243, 272-280 at world size 1: query, take the wrap-around block
 * [start,start+block) of the flat tensor as payload, sketch the rest, and
 * leave zeros + block in the tensor.  Calls the restatements above, in the
 * reference's order of operations (clone included). */
void conef_oracle_randblock_conef_step(float *x, float *cs, float *payload, int64_t n, int64_t m,
                                       int32_t w, int64_t start, int64_t block,
                                       float alpha, float beta, int32_t a, int32_t b)
{
    int64_t numel = n * m;
    int64_t end = start + block < numel ? start + block : numel;
    int64_t rest = block - (end - start);
    conef_oracle_cs_query(x, cs, n, m, w, alpha, a, b);
    memcpy(payload, x + start, sizeof(float) * (size_t)(end - start));
    float *cp = (float *)malloc(sizeof(float) * (size_t)numel);
    memcpy(cp, x, sizeof(float) * (size_t)numel);
    memset(cp + start, 0, sizeof(float) * (size_t)(end - start));
    if (rest > 0) {
        memcpy(payload + (end - start), x, sizeof(float) * (size_t)rest);
        memset(cp, 0, sizeof(float) * (size_t)rest);
    }
    conef_oracle_cs_update(cp, cs, n, m, w, beta, a, b);
    free(cp);
    memset(x, 0, sizeof(float) * (size_t)numel);
    memcpy(x + start, payload, sizeof(float) * (size_t)(end - start));
    if (rest > 0)
        memcpy(x, payload + (end - start), sizeof(float) * (size_t)rest);
}
