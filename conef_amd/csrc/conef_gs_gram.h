// Gram-Schmidt through the Gram matrix: ONE exchange between workgroups instead of one per column.
//
// The reference's routine (powerSGD_hook.py:21-43) is a chain of r column steps
//     col_i /= ||col_i|| + eps;   col_j -= (col_i . col_j) col_i   for every j > i,
// and a kernel that follows it literally needs r reductions over all rows, one after the other: at
// rank 32 on a [4096, 32] factor that is 32 trips between workgroups, 2.5 us each.  But every
// quantity those steps need is a function of the Gram matrix G = A^T A of the ORIGINAL columns:
// step i replaces col_j by col_j - b_ij col_i with b_ij = G_ij / d_i^2, d_i = sqrt(G_ii) + eps, and
// the Gram matrix of the new columns follows from the old one,
//     G_jk <- G_jk - b_ij G_ik - b_ik G_ij + b_ij b_ik G_ii          (j, k > i).
// So the kernel
//   1. forms its rows' share of G on the matrix cores in double precision
//      (v_mfma_f64_16x16x4_f64; a product of two floats is exact in a double),
//   2. exchanges the r (r + 1) / 2 partial sums between the matrix's workgroups ONCE and adds
//      them in workgroup order,
//   3. runs the r steps on the r x r matrix in LDS (double), which yields all b_ij and d_i,
//   4. applies the steps to its own rows, row by row, in registers: x_j -= b_ij x_i, x_i /= d_i,
//      the reference's column operations (fp32, as there) with the coefficients already known.
// In exact arithmetic this is the reference's algorithm.  In floating point the coefficients here
// are accurate to double precision (the cancellation in step 3 costs eps_double * cond(A)^2),
// whereas the fp32 chain of the reference carries eps_float * cond(A) from column to column: the
// two agree to the reference's own rounding noise, 1e-6 or better on the well-conditioned factors
// PowerSGD produces.  A zero column gives d = 0 and NaN from there on, as in the reference.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "conef_gs_lanes.h"      // gs_count_give_up

constexpr int kGsgThreads = 256;
constexpr int kGsgMaxItems = 24;            // matrices per launch
constexpr int kGsgMaxWgs = 128;             // workgroups per launch
constexpr int kGsgMaxWgsPerItem = 48;       // every workgroup of a matrix reads all the others' sums
constexpr int kGsgMaxEntries = 32 * 33 / 2; // upper triangle at rank 32
constexpr unsigned kGsgSpinLimit = 1u << 22;

// slot[g][2 e], slot[g][2 e + 1]: high and low word of workgroup g's partial sum for entry e, each
// with the launch's tag in the upper half: one relaxed load tells a reader whether the word is this
// launch's, and nothing has to be cleared between launches.
struct GsgWs {
    unsigned gave_up;
    unsigned pad[63];
    unsigned long long slot[kGsgMaxWgs][2 * kGsgMaxEntries];
};

// Matrix k of a launch: [rows[k], RP] row-major at a[k], workgroups first[k] .. first[k + 1] - 1,
// slab[k] rows each.
struct GsgBatch {
    float* a[kGsgMaxItems];
    int rows[kGsgMaxItems];
    int slab[kGsgMaxItems];
    int first[kGsgMaxItems + 1];
};

typedef double gsg_v4d __attribute__((ext_vector_type(4)));

// Phase timestamps of workgroup 0 (100 MHz counter) into the workspace's padding: only in builds
// that define GSG_TRACE, for measuring where a launch spends its time.
#ifdef GSG_TRACE
#define GSG_STAMP(k)                                                                                         \
    do {                                                                                                     \
        if (blockIdx.x == 0 && threadIdx.x == 0)                                                             \
            reinterpret_cast<unsigned long long*>(&ws->pad[1])[k] = (unsigned long long)wall_clock64();      \
    } while (0)
#else
#define GSG_STAMP(k) do { } while (0)
#endif

// Rows a workgroup takes at least (32 KB of fp32) and the workgroups a matrix gets.
inline int gsg_min_slab(int rp) { return rp >= 32 ? 256 : rp >= 16 ? 512 : 1024; }

inline void gsg_split(int64_t rows, int rp, int* slab, int* wgs)
{
    int64_t s = gsg_min_slab(rp);
    int64_t w = (rows + s - 1) / s;
    if (w > kGsgMaxWgsPerItem) {
        w = kGsgMaxWgsPerItem;
        s = ((rows + w - 1) / w + 15) / 16 * 16;
        w = (rows + s - 1) / s;
    }
    *slab = (int)s;
    *wgs = (int)w;
}

// entry e of the row-major upper triangle of an rp x rp matrix -> (i, j), i <= j
__device__ __forceinline__ void gsg_entry(int e, int rp, int* pi, int* pj)
{
    const int t = 2 * rp + 1;
    int i = (int)(((float)t - sqrtf((float)(t * t - 8 * e))) * 0.5f);
    if (i < 0) i = 0;
    if (i > rp - 1) i = rp - 1;
    while (i > 0 && i * rp - (i * (i - 1)) / 2 > e) --i;               // rows before i hold i rp - i (i - 1) / 2 entries
    while (i + 1 < rp && (i + 1) * rp - ((i + 1) * i) / 2 <= e) ++i;
    *pi = i;
    *pj = i + (e - (i * rp - (i * (i - 1)) / 2));
}

// A workgroup's share of G = A^T A over rows [r0, r1) of the row-major [*, RP] matrix a, on the matrix
// cores in double: per-wave partial tiles into `tiles` ([waves][NT][256], [i][j] row-major inside a
// 16 x 16 tile; tiles in the order (0,0), (0,1), (1,1)).  All kGsgThreads threads call this; a
// barrier must follow before the tiles are read (gsg_tiles_entry).
template <int RP>
__device__ __forceinline__ void
gsg_gram_tiles(const float* __restrict__ a, int r0, int r1, double (*tiles)[(RP >= 16 ? (RP / 16) * (RP / 16 + 1) / 2 : 1)][256])
{
    constexpr int NW = kGsgThreads / 64;
    constexpr int NC = RP >= 16 ? RP / 16 : 1;
    constexpr int NT = NC * (NC + 1) / 2;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // a wave takes blocks of four rows, lane = (row l / 16,
    // column l % 16 of each column group); D[i][j] += sum_k A[k][i] A[k][j] over the block's rows.
    // At rank 8 lanes 8..15 of a row group take the same columns of the NEXT four rows: the two
    // diagonal 8 x 8 blocks of the product are then two partial sums of G (the off-diagonal blocks
    // mix the row blocks and are dropped).  Sixteen blocks' loads are in flight per wave: the
    // phase is a few trips to memory, not arithmetic.
    constexpr int U = 16;
    constexpr int RPB = RP == 8 ? 8 : 4;                    // rows a block covers
    gsg_v4d acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = (gsg_v4d){0., 0., 0., 0.};
    const int lr = lane >> 4, lc = lane & 15;
    const int nblk = (r1 - r0 + RPB - 1) / RPB;
    for (int b0 = wave; b0 < nblk; b0 += U * NW) {
        float x[U][NC];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int blk = b0 + u * NW;
            const int row = r0 + blk * RPB + (RP == 8 ? (lc >> 3) * 4 : 0) + lr;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const int col = RP == 8 ? (lc & 7) : c * 16 + lc;
                const bool in = blk < nblk && row < r1;
                x[u][c] = in ? a[(int64_t)row * RP + col] : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            double d[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c) d[c] = (double)x[u][c];
            int t = 0;
#pragma unroll
            for (int ci = 0; ci < NC; ++ci) {
#pragma unroll
                for (int cj = ci; cj < NC; ++cj) {
                    acc[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(d[ci], d[cj], acc[t], 0, 0, 0);
                    ++t;
                }
            }
        }
    }
    // result register v of lane l is element (4 v + l / 16, l % 16) of the tile
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int v = 0; v < 4; ++v) tiles[wave][t][(4 * v + lr) * 16 + lc] = acc[t][v];
    }
}

// entry (i, j), i <= j, of the share: the waves' partial tiles added in wave order
template <int RP>
__device__ __forceinline__ double
gsg_tiles_entry(const double (*tiles)[(RP >= 16 ? (RP / 16) * (RP / 16 + 1) / 2 : 1)][256], int i, int j)
{
    constexpr int NW = kGsgThreads / 64;
    constexpr int NC = RP >= 16 ? RP / 16 : 1;
    const int ci = i >> 4, cj = j >> 4;
    const int t = NC == 1 ? 0 : (ci == 0 ? cj : 2);
    const int at = (i & 15) * 16 + (j & 15);
    double s = 0.;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        s += tiles[w][t][at];
        if (RP == 8) s += tiles[w][t][at + 8 * 16 + 8];   // the second row block's partial sum
    }
    return s;
}

// The r column steps on the upper triangle of the r x r Gram matrix in LDS (all T threads of the
// workgroup call this; `gram` must be complete and visible).  Leaves b_ij in coef[i][j] (i < j) and
// 1 / d_i in dinvf[i]; `dinv` and `diag0` (RP doubles each) are scratch.
//
// Columns that depend on earlier ones.  The squared norm a column has left when its turn comes is
// G_ii minus what the earlier steps took away, and for a column that lies in the span of the earlier
// ones that difference is rounding noise around zero, of either sign.  The reference
// (powerSGD_hook.py:21-43) meets the same case in fp32: what its subtractions leave of such a column
// is their own rounding residue, about 2^-23 of the column's original norm, which it then scales to
// unit length - finite numbers that mean nothing.  A pivot below that residue, (2^-23)^2 of the
// column's original G_ii, is therefore raised to it: the column comes out finite, as in the
// reference, and no result above the reference's own noise changes.  A column that was zero to begin
// with keeps its pivot of zero and gives NaN (eps = 0) or zeros (eps != 0), as in the reference.
template <int RP, int T>
__device__ __forceinline__ void gsg_recurrence(double (*gram)[RP + 1], float (*coef)[RP], double* dinv, float* dinvf,
                                               double* diag0, float eps, int tid)
{
    constexpr int NG = RP * (RP + 1) / 2;
    if (tid < RP) diag0[tid] = gram[tid][tid] * 0x1p-46;
    __syncthreads();
    // Thread (j, part) owns
    // entries (j, k), k = j + part, j + part + parts, ...  Step i reads row i (final since the
    // barrier of step i - 1) and rewrites the rows below it; its coefficients go to `coef`, which
    // nobody reads before the last barrier.  One barrier per step.
    // A thread owns the same few entries (j, k), j <= k, throughout.  The r steps run in panels of
    // four pivots: a panel's pivot rows at the thread's columns and the panel's own 4 x 4 block are
    // read once, the four steps then run in registers (every thread repeats the small block's
    // arithmetic, so nobody waits for anybody inside a panel), and one barrier ends the panel:
    // r / 4 trips through LDS and the barrier instead of r.
    constexpr int EPT = (NG + T - 1) / T;                   // entries per thread: 1, 1, 3 at ranks 8, 16, 32
    constexpr int B = RP < 4 ? RP : 4;
    int ej[EPT], ek[EPT];
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
        const int e = tid + u * T;
        int i, j2;
        gsg_entry(e < NG ? e : 0, RP, &i, &j2);
        ej[u] = e < NG ? i : -1;                            // -1: no entry, never active
        ek[u] = j2;
    }
#pragma unroll 1
    for (int i0 = 0; i0 < RP; i0 += B) {
        double P[B][B];                                     // the panel's block, upper triangle
#pragma unroll
        for (int a2 = 0; a2 < B; ++a2) {
#pragma unroll
            for (int b2 = a2; b2 < B; ++b2) P[a2][b2] = gram[i0 + a2][i0 + b2];
        }
        double g[EPT], Rj[EPT][B], Rk[EPT][B];
        int na[EPT];                                        // steps of this panel that reach the entry
#pragma unroll
        for (int u = 0; u < EPT; ++u) {
            const int dj = ej[u] - i0;
            na[u] = dj <= 0 ? 0 : (dj < B ? dj : B);
            const bool on = dj >= 0;                        // rows of the panel itself are read for their coefficients
            g[u] = gram[on ? ej[u] : i0][on ? ek[u] : i0];
#pragma unroll
            for (int a2 = 0; a2 < B; ++a2) {
                const bool use = a2 < na[u];
                Rj[u][a2] = gram[i0 + a2][use ? ej[u] : i0 + a2];
                Rk[u][a2] = gram[i0 + a2][use ? ek[u] : i0 + a2];
            }
        }
        double inv2[B];
#pragma unroll
        for (int a2 = 0; a2 < B; ++a2) {
            // 1 / d^2: hardware estimate and two Newton steps (exact to the last bits of a double)
            // instead of a division.  With eps = 0, d^2 is the pivot itself and the square root
            // for 1 / d waits until after the loop.
            const double least = diag0[i0 + a2];
            const double piv = P[a2][a2] < least ? least : P[a2][a2];
            double dd = piv;
            if (eps != 0.f) {
                double y = __builtin_amdgcn_rsq(piv);
                y = y * (1.5 - 0.5 * piv * y * y);
                y = y * (1.5 - 0.5 * piv * y * y);
                const double d = (piv == 0. ? 0. : piv * y) + (double)eps;
                dd = d * d;
            }
            double r = __builtin_amdgcn_rcp(dd);
            r = fma(fma(-dd, r, 1.), r, r);
            r = fma(fma(-dd, r, 1.), r, r);
            inv2[a2] = r;
            if (tid == 0) dinv[i0 + a2] = piv;
            // G_jk - b_j G_ik - b_k G_ij + b_j b_k G_ii  =  G_jk - (G_ij G_ik) (2 - G_ii / d^2) / d^2
            const double scale = r * fma(-piv, r, 2.);
#pragma unroll
            for (int b2 = a2 + 1; b2 < B; ++b2) {
                const double pb = P[a2][b2] * scale;
#pragma unroll
                for (int c2 = b2; c2 < B; ++c2) P[b2][c2] = fma(-pb, P[a2][c2], P[b2][c2]);
            }
#pragma unroll
            for (int u = 0; u < EPT; ++u) {
                if (a2 < na[u]) {
                    g[u] = fma(-(Rj[u][a2] * Rk[u][a2]), scale, g[u]);
#pragma unroll
                    for (int b2 = a2 + 1; b2 < B; ++b2) {
                        const double pb = P[a2][b2] * scale;
                        Rj[u][b2] = fma(-pb, Rj[u][a2], Rj[u][b2]);
                        Rk[u][b2] = fma(-pb, Rk[u][a2], Rk[u][b2]);
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < EPT; ++u) {
            if (na[u] > 0) gram[ej[u]][ek[u]] = g[u];
            const int dj = ej[u] - i0;
            if (dj >= 0 && dj < B && ek[u] > ej[u]) {       // an entry of pivot row j is final after dj steps
                double r = inv2[0];
#pragma unroll
                for (int a2 = 1; a2 < B; ++a2) r = dj == a2 ? inv2[a2] : r;
                coef[ej[u]][ek[u]] = (float)(g[u] * r);
            }
        }
        __syncthreads();
    }
    if (tid < RP) dinvf[tid] = (float)(1. / (sqrt(dinv[tid]) + (double)eps));
    __syncthreads();

}

template <int RP>
__global__ void __launch_bounds__(kGsgThreads)
gsg_kernel(GsgBatch batch, int count, float eps, GsgWs* ws, unsigned tag)
{
    constexpr int T = kGsgThreads, NW = T / 64;
    constexpr int NC = RP >= 16 ? RP / 16 : 1;             // column groups of 16
    constexpr int NT = NC * (NC + 1) / 2;                  // tiles of the upper triangle: 1 or 3
    constexpr int NG = RP * (RP + 1) / 2;
    __shared__ double tiles[NW][NT][256];                   // per-wave partial tiles, [i][j] row-major inside a tile
    __shared__ double gram[RP][RP + 1];                     // upper triangle of the current Gram matrix
    __shared__ __attribute__((aligned(16))) float coef[RP][RP];       // b_ij for i < j, rounded once for step 4
    __shared__ double dinv[RP];                             // the pivots G_ii, then 1 / d_i
    __shared__ double diag0[RP];                            // the least pivot each column may end up with
    __shared__ float dinvf[RP];
    __shared__ int failed;

    int it = 0;
    while (it + 1 < count && (int)blockIdx.x >= batch.first[it + 1]) ++it;
    const int wg0 = batch.first[it];
    const int nwg = batch.first[it + 1] - wg0;
    const int local = (int)blockIdx.x - wg0;
    const int rows = batch.rows[it], slab = batch.slab[it];
    const int r0 = local * slab;
    const int r1 = r0 + slab < rows ? r0 + slab : rows;
    float* __restrict__ a = batch.a[it];

    const int tid = threadIdx.x;
    if (tid == 0) failed = 0;
    GSG_STAMP(0);

    // ---- 1. this workgroup's share of G on the matrix cores
    gsg_gram_tiles<RP>(a, r0, r1, tiles);
    __syncthreads();
    GSG_STAMP(1);

    // ---- 2. upper-triangle entries: sum over the waves, publish, collect every workgroup's share
    for (int e = tid; e < NG; e += T) {
        int i, j;
        gsg_entry(e, RP, &i, &j);
        const double s = gsg_tiles_entry<RP>(tiles, i, j);
        if (nwg > 1) {
            const unsigned long long bits = (unsigned long long)__double_as_longlong(s);
            const unsigned long long hi = ((unsigned long long)tag << 32) | (bits >> 32);
            const unsigned long long lo = ((unsigned long long)tag << 32) | (bits & 0xffffffffull);
            __hip_atomic_store(&ws->slot[blockIdx.x][2 * e], hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&ws->slot[blockIdx.x][2 * e + 1], lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            gram[i][j] = s;
        }
    }
    if (nwg > 1) {
        constexpr int CH = 16;                              // workgroups whose records are requested together
        for (int e = tid; e < NG; e += T) {
            int i, j;
            gsg_entry(e, RP, &i, &j);
            double s = 0.;
            for (int g0 = 0; g0 < nwg; g0 += CH) {
                const int ng = nwg - g0 < CH ? nwg - g0 : CH;
                unsigned long long rec[2 * CH];
#pragma unroll
                for (int u = 0; u < 2 * CH; ++u) {          // 2 CH loads in flight; past the end: a valid slot, unused
                    const int g = g0 + ((u >> 1) < ng ? (u >> 1) : 0);
                    rec[u] = __hip_atomic_load(&ws->slot[wg0 + g][2 * e + (u & 1)], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int u = 0; u < 2 * CH; ++u) {
                    if ((u >> 1) >= ng) continue;
                    unsigned spins = 0;
                    while ((unsigned)(rec[u] >> 32) != tag) {          // not there yet: ask again
                        ++spins;
                        if (spins > kGsgSpinLimit ||
                            ((spins & 255u) == 0 && __hip_atomic_load(&ws->gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == tag)) {
                            __hip_atomic_store(&ws->gave_up, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            failed = 1;
                            rec[u] = (unsigned long long)tag << 32;
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                        rec[u] = __hip_atomic_load(&ws->slot[wg0 + g0 + (u >> 1)][2 * e + (u & 1)], __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
#pragma unroll
                for (int u = 0; u < CH; ++u) {              // the same order in every workgroup
                    if (u < ng)
                        s += __longlong_as_double((long long)(((rec[2 * u] & 0xffffffffull) << 32) | (rec[2 * u + 1] & 0xffffffffull)));
                }
            }
            gram[i][j] = s;
        }
    }
    __syncthreads();
    GSG_STAMP(2);
    if (failed) {
        if (tid == 0) gs_count_give_up();
        // a half-orthogonalised matrix would pass for a result: leave one that cannot
        for (int e = tid; e < (r1 - r0) * RP; e += T) a[(int64_t)r0 * RP + e] = __builtin_nanf("");
        return;
    }

    // ---- 3. the r column steps on the r x r matrix
    gsg_recurrence<RP, T>(gram, coef, dinv, dinvf, diag0, eps, tid);
    GSG_STAMP(4);

    // ---- 4. the same steps on this workgroup's rows, a row per thread: the reference's column
    // operations in its own precision (fp32, one fused multiply-add per element and step), with
    // coefficients that were computed in double and rounded once
    for (int row = r0 + tid; row < r1; row += T) {
        float* p = a + (int64_t)row * RP;
        float x[RP];
#pragma unroll
        for (int c = 0; c < RP; c += 4) {
            const float4 v = *reinterpret_cast<const float4*>(p + c);
            x[c] = v.x;
            x[c + 1] = v.y;
            x[c + 2] = v.z;
            x[c + 3] = v.w;
        }
        // One row of coefficients at a time, the next row requested before this row's multiply-adds
        // (without the fences the compiler requests all r (r - 1) / 2 up front and runs out of
        // registers at rank 32).
        float cur[RP], nxt[RP];
#pragma unroll
        for (int k = 0; k < RP; ++k) cur[k] = coef[0][k];
#pragma unroll
        for (int i = 0; i < RP; ++i) {
            asm volatile("" ::: "memory");
            if (i + 1 < RP) {
#pragma unroll
                for (int k = (i + 2) & ~3; k < RP; ++k) nxt[k] = coef[i + 1][k];      // whole 16-byte groups
            }
            asm volatile("" ::: "memory");
#pragma unroll
            for (int k = i + 1; k < RP; ++k) x[k] = fmaf(-cur[k], x[i], x[k]);
            x[i] = __fmul_rn(x[i], dinvf[i]);
#pragma unroll
            for (int k = (i + 2) & ~3; k < RP; ++k) cur[k] = nxt[k];
        }
#pragma unroll
        for (int c = 0; c < RP; c += 4) *reinterpret_cast<float4*>(p + c) = make_float4(x[c], x[c + 1], x[c + 2], x[c + 3]);
    }
    GSG_STAMP(5);
}
