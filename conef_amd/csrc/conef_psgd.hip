// PowerSGD inner-loop kernels (gfx950) and their C entry points.
//
// Reference semantics: communication/powerSGD_hook.py:12-44 (_orthogonalize), :498 (P = M Q),
// :532 (Q = M^T P), :551 (M = P Q^T), :361/:558 (dense error feedback), :409/:563-564 (count-sketched
// error feedback).  All matrices are row-major fp32: M [n,m], Q [m,r], P [n,r], r <= 32.
//
// At the ranks gradient compression uses (1..8) these products move 4 bytes of M per 2r flops, far
// below the fp32 ridge of the machine, so they are written as streaming kernels: M is read exactly
// once per product with 16-byte accesses, the rank dimension lives in registers, and the
// error-feedback add (before the first product) and the residual (after the last) are fused into
// the passes that touch M anyway.  Sums that cross workgroups meet through a caller-provided
// workspace in a fixed order: no atomics, results do not change from run to run.
#include <cstdlib>
#include <type_traits>
#include <algorithm>
#include <atomic>
#include <vector>

#include "conef_device.h"
#include "conef_sketch_core.h"
#include "conef_plan.h"
#include "conef_psgd_mfma.h"
#include "conef_gs_lanes.h"
#include "conef_gs_gram.h"
#include "conef_psgd_stream.h"
#include "conef_psgd_small.h"
#include "conef_hip.h"      // ConefPsgdItem, and a check of this file's definitions against the public header

extern "C" int conef_cs_query_f32(float* x, const float* cs, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                                  int32_t b, void* stream);

namespace {

constexpr int kMaxRank = 32;

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

__device__ __forceinline__ void ld4(const float* p, float* v)
{
    float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void st4(float* p, const float* v)
{
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

// All kernels come in a FAST form (r equals the compile-time rank bound RP, m % 4 == 0, every
// pointer 16-byte aligned: 16-byte accesses, Q rows of a column quad are one contiguous run) and a
// general form (any r <= RP, any alignment, 4-byte accesses).

// ------------------------------------------------------------ batched launches ----
// A gradient bucket holds several matrices whose products are independent of each other, and most
// of them are too small to fill 256 CUs on their own.  Every product kernel therefore exists in
// two forms: one matrix per launch, and up to kPsgdBatchMax matrices per launch with the
// per-matrix arguments in a table passed by value; a workgroup finds its matrix from the table's
// running workgroup count and then does exactly what it would do in a launch of its own.
constexpr int kPsgdBatchMax = 24;

template <typename Item>
struct PsgdBatch {
    Item item[kPsgdBatchMax];
    int first[kPsgdBatchMax + 1];   // first workgroup of item i; first[count] = workgroups in all
    int count;
};

template <typename Item>
__device__ __forceinline__ int psgd_batch_locate(const PsgdBatch<Item>& b, int* local)
{
    int i = 0;
    while (i + 1 < b.count && (int)blockIdx.x >= b.first[i + 1]) ++i;
    *local = (int)blockIdx.x - b.first[i];
    return i;
}

// ---------------------------------------------------------------- P = X Q ----
// MODE 0: X = M as stored.  MODE 1: X = M + E (dense error), written back into M.
// MODE 2: X = M + alpha * unsketch(cs), written back into M (DenseCS.query fused); the sketch rows
// of the workgroup's matrix rows are parked in LDS first.
// A workgroup owns RB consecutive rows and all columns; a thread owns column quads tid, tid+256, ...
// and keeps RB x RP partial sums, reduced over the workgroup at the end in a fixed order.
template <int RB, int RP, int MODE, bool FAST>
__device__ __forceinline__ void
psgd_mq_body(float* __restrict__ x, const float* __restrict__ err, const float* __restrict__ cs,
             const uint32_t* __restrict__ pktab, const float* __restrict__ q, float* __restrict__ p, int64_t n,
             int m, int r, ConefMod mod, float alpha, ConefSeeds hs, int bx)
{
    extern __shared__ float mq_lds[];
    float* red = mq_lds;                    // [4][RB*RP]
    float* cells = mq_lds + 4 * RB * RP;    // [RB][w], MODE 2 only
    const int64_t row0 = (int64_t)bx * RB;
    const int w = (int)mod.w;
    int64_t rowc[RB];                       // rows past the end are clamped for loads, their stores are skipped
#pragma unroll
    for (int a = 0; a < RB; ++a) rowc[a] = row0 + a < n ? row0 + a : n - 1;
    if (MODE == 2) {
#pragma unroll
        for (int a = 0; a < RB; ++a)
            for (int j = threadIdx.x; j < w; j += 256) cells[a * w + j] = cs[rowc[a] * w + j];
        __syncthreads();
    }
    float acc[RB][RP];
#pragma unroll
    for (int a = 0; a < RB; ++a)
#pragma unroll
        for (int c = 0; c < RP; ++c) acc[a][c] = 0.f;

    if (FAST) {
        const int m4 = m >> 2;
        // column quads in flight per thread, at most: registers for more of them cost more in
        // resident waves than the extra loads in flight bring
        constexpr int UMAX = (RB * RP <= 16) ? 2 : 1;
        // narrow matrices do not have that many quads per thread: fewer in flight rather than
        // clamped duplicates of the last quad
        auto sweep = [&](auto u_tag) {
        constexpr int U = decltype(u_tag)::value;
        for (int j0 = threadIdx.x; j0 < m4; j0 += U * 256) {
            float xv[U][RB][4];
            float qf[U][4 * RP];                        // Q rows 4j..4j+3: 4*RP consecutive floats
            float ev[U][RB][4];
            uint32_t pk[U][4];
#pragma unroll
            for (int u = 0; u < U; ++u) {               // past the last quad: a valid address, result unused
                const int j = j0 + u * 256 < m4 ? j0 + u * 256 : m4 - 1;
#pragma unroll
                for (int a = 0; a < RB; ++a) ld4(x + rowc[a] * m + 4 * j, xv[u][a]);
#pragma unroll
                for (int t = 0; t < RP; ++t) ld4(q + (int64_t)j * 4 * RP + 4 * t, qf[u] + 4 * t);
                if (MODE == 1) {
#pragma unroll
                    for (int a = 0; a < RB; ++a) ld4(err + rowc[a] * m + 4 * j, ev[u][a]);
                }
                if (MODE == 2) {
                    if (pktab) {
                        uint4 t = reinterpret_cast<const uint4*>(pktab)[j];
                        pk[u][0] = t.x; pk[u][1] = t.y; pk[u][2] = t.z; pk[u][3] = t.w;
                    } else {
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            pk[u][k] = conef_bucket_sign(4 * j + k, mod, hs.a, hs.b, hs.sa, hs.sb);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = j0 + u * 256;
                if (j >= m4) break;
                if (MODE == 1) {
#pragma unroll
                    for (int a = 0; a < RB; ++a) {
#pragma unroll
                        for (int k = 0; k < 4; ++k) xv[u][a][k] = __fadd_rn(xv[u][a][k], ev[u][a][k]);
                        if (row0 + a < n) st4(x + rowc[a] * m + 4 * j, xv[u][a]);
                    }
                } else if (MODE == 2) {
#pragma unroll
                    for (int a = 0; a < RB; ++a) {
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            xv[u][a][k] = __fadd_rn(xv[u][a][k], conef_query_term(cells[a * w + (pk[u][k] & 0x7fffffffu)],
                                                                                   pk[u][k], alpha));
                        if (row0 + a < n) st4(x + rowc[a] * m + 4 * j, xv[u][a]);
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; ++k)
#pragma unroll
                    for (int a = 0; a < RB; ++a)
#pragma unroll
                        for (int c = 0; c < RP; ++c) acc[a][c] = fmaf(xv[u][a][k], qf[u][k * RP + c], acc[a][c]);
            }
        }
        };
        if (m4 <= 256 || UMAX == 1) sweep(std::integral_constant<int, 1>());
        else sweep(std::integral_constant<int, UMAX>());
    } else {
        for (int k = threadIdx.x; k < m; k += 256) {
            float qk[RP];
#pragma unroll
            for (int c = 0; c < RP; ++c) qk[c] = c < r ? q[(int64_t)k * r + c] : 0.f;
            uint32_t pk = 0;
            if (MODE == 2) pk = pktab ? pktab[k] : conef_bucket_sign(k, mod, hs.a, hs.b, hs.sa, hs.sb);
#pragma unroll
            for (int a = 0; a < RB; ++a) {
                float v = x[rowc[a] * m + k];
                if (MODE == 1) v = __fadd_rn(v, err[rowc[a] * m + k]);
                if (MODE == 2) v = __fadd_rn(v, conef_query_term(cells[a * w + (pk & 0x7fffffffu)], pk, alpha));
                if (MODE != 0 && row0 + a < n) x[rowc[a] * m + k] = v;
#pragma unroll
                for (int c = 0; c < RP; ++c) acc[a][c] = fmaf(v, qk[c], acc[a][c]);
            }
        }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int a = 0; a < RB; ++a)
#pragma unroll
        for (int c = 0; c < RP; ++c) {
            float s = conef_wave_sum(acc[a][c]);
            if (lane == 0) red[wave * RB * RP + a * RP + c] = s;
        }
    __syncthreads();
    if (threadIdx.x < RB * RP) {
        int a = threadIdx.x / RP, c = threadIdx.x % RP;
        int t = threadIdx.x;
        if (row0 + a < n && c < r)
            p[(row0 + a) * r + c] = (red[t] + red[RB * RP + t]) + (red[2 * RB * RP + t] + red[3 * RB * RP + t]);
    }
}

template <int RB, int RP, int MODE, bool FAST>
__global__ void __launch_bounds__(256)
psgd_mq_kernel(float* __restrict__ x, const float* __restrict__ err, const float* __restrict__ cs,
               const uint32_t* __restrict__ pktab, const float* __restrict__ q, float* __restrict__ p, int64_t n,
               int m, int r, ConefMod mod, float alpha, ConefSeeds hs)
{
    psgd_mq_body<RB, RP, MODE, FAST>(x, err, cs, pktab, q, p, n, m, r, mod, alpha, hs, (int)blockIdx.x);
}

struct MqItem {
    float* x;
    const float* err;
    const float* cs;
    const uint32_t* pktab;
    const float* q;
    float* p;
    int64_t n;
    int m, r;
    ConefMod mod;
};

template <int RB, int RP, int MODE, bool FAST>
__global__ void __launch_bounds__(256)
psgd_mq_batch_kernel(PsgdBatch<MqItem> b, float alpha, ConefSeeds hs)
{
    int local;
    const MqItem& it = b.item[psgd_batch_locate(b, &local)];
    psgd_mq_body<RB, RP, MODE, FAST>(it.x, it.err, it.cs, it.pktab, it.q, it.p, it.n, it.m, it.r, it.mod, alpha, hs, local);
}

// streaming form (conef_psgd_stream.h): the kernel of every matrix whose shape allows 16-byte accesses
template <int RP, int MODE, int T>
__global__ void __launch_bounds__(T)
psgd_mqs_batch_kernel(PsgdBatch<MqsItem> b, float alpha, ConefSeeds hs)
{
    int local;
    const MqsItem& it = b.item[psgd_batch_locate(b, &local)];
    psgd_mqs_body<RP, MODE, T>(it, alpha, hs, local);
}

// -------------------------------------------------------------- Q = X^T P ----
// A workgroup of 8 waves owns 256 columns and a slab of rows.  A lane owns a column quad, wave v
// takes rows v, v+8, ... of the slab (one contiguous kilobyte per row), the 8 waves meet in LDS.
// With one slab the result is stored, with several each slab writes a partial [m,r] and a second
// small kernel adds the partials in slab order: deterministic, no atomics.
constexpr int kMtpWaves = 8;
constexpr int kMtpThreads = 64 * kMtpWaves;

template <int RP, bool FAST>
__device__ __forceinline__ void
psgd_mtp_body(const float* __restrict__ x, const float* __restrict__ p, float* __restrict__ out, int64_t n, int m,
              int r, int rows_per_slab, int bx, int by)
{
    constexpr int CH = RP < 4 ? RP : 4;            // ranks reduced per LDS round
    __shared__ float red[kMtpWaves][CH][256];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int c0 = bx * 256 + lane * 4;            // first column of my quad
    const int64_t i0 = (int64_t)by * rows_per_slab;
    const int64_t i1 = i0 + rows_per_slab < n ? i0 + rows_per_slab : n;
    float acc[4][RP];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int c = 0; c < RP; ++c) acc[k][c] = 0.f;
    if (FAST) {
        const int cc = c0 < m ? c0 : m - 4;         // clamped: lanes past the edge load a valid quad, results unused
        int64_t i = i0 + wave;
        for (; i + 3 * kMtpWaves < i1; i += 4 * kMtpWaves) {      // four rows in flight
            float xv[4][4];
#pragma unroll
            for (int u = 0; u < 4; ++u) ld4(x + (i + u * kMtpWaves) * m + cc, xv[u]);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float* pi = p + (i + u * kMtpWaves) * RP;
#pragma unroll
                for (int c = 0; c < RP; ++c) {
                    float pc = pi[c];
#pragma unroll
                    for (int k = 0; k < 4; ++k) acc[k][c] = fmaf(xv[u][k], pc, acc[k][c]);
                }
            }
        }
        for (; i < i1; i += kMtpWaves) {
            float xv[4];
            ld4(x + i * m + cc, xv);
            const float* pi = p + i * RP;
#pragma unroll
            for (int c = 0; c < RP; ++c) {
                float pc = pi[c];
#pragma unroll
                for (int k = 0; k < 4; ++k) acc[k][c] = fmaf(xv[k], pc, acc[k][c]);
            }
        }
    } else {
        for (int64_t i = i0 + wave; i < i1; i += kMtpWaves) {
            float xv[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) xv[k] = x[i * m + (c0 + k < m ? c0 + k : m - 1)];
            const float* pi = p + i * r;
#pragma unroll
            for (int c = 0; c < RP; ++c) {
                float pc = c < r ? pi[c] : 0.f;
#pragma unroll
                for (int k = 0; k < 4; ++k) acc[k][c] = fmaf(xv[k], pc, acc[k][c]);
            }
        }
    }
    float* dst = out + (int64_t)by * m * r;           // partial of this slab (or Q itself with one slab)
#pragma unroll
    for (int cb = 0; cb < RP; cb += CH) {
        if (cb) __syncthreads();
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int k = 0; k < 4; ++k) red[wave][c][lane * 4 + k] = acc[k][cb + c];
        __syncthreads();
        if (threadIdx.x < 256) {
            const int col = bx * 256 + threadIdx.x;
            float s[CH];
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                float t = 0.f;
#pragma unroll
                for (int v = 0; v < kMtpWaves; ++v) t += red[v][c][threadIdx.x];
                s[c] = t;
            }
            if (col < m) {
                if (FAST && CH == 4) {
                    st4(dst + (int64_t)col * RP + cb, s);
                } else {
#pragma unroll
                    for (int c = 0; c < CH; ++c)
                        if (cb + c < r) dst[(int64_t)col * r + cb + c] = s[c];
                }
            }
        }
    }
}

template <int RP, bool FAST>
__global__ void __launch_bounds__(kMtpThreads)
psgd_mtp_kernel(const float* __restrict__ x, const float* __restrict__ p, float* __restrict__ out, int64_t n, int m,
                int r, int rows_per_slab)
{
    psgd_mtp_body<RP, FAST>(x, p, out, n, m, r, rows_per_slab, (int)blockIdx.x, (int)blockIdx.y);
}

struct MtpItem {
    const float* x;
    const float* p;
    float* out;
    int64_t n;
    int m, r, rows_per_slab, col_tiles;
};

template <int RP, bool FAST>
__global__ void __launch_bounds__(kMtpThreads)
psgd_mtp_batch_kernel(PsgdBatch<MtpItem> b)
{
    int local;
    const MtpItem& it = b.item[psgd_batch_locate(b, &local)];
    psgd_mtp_body<RP, FAST>(it.x, it.p, it.out, it.n, it.m, it.r, it.rows_per_slab, local % it.col_tiles,
                            local / it.col_tiles);
}

// out[i] = sum over slabs of partial[s][i], slabs in ascending order
__device__ __forceinline__ void
psgd_sum_partials_body(const float* __restrict__ partial, float* __restrict__ out, int64_t count, int slabs, int bx)
{
    int64_t i = bx * (int64_t)256 + threadIdx.x;
    if (i >= count) return;
    float s = 0.f;
    int k = 0;
    for (; k + 8 <= slabs; k += 8) {        // eight loads in flight, added in slab order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = partial[(int64_t)(k + u) * count + i];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; k < slabs; ++k) s += partial[(int64_t)k * count + i];
    out[i] = s;
}

__global__ void __launch_bounds__(256)
psgd_sum_partials_kernel(const float* __restrict__ partial, float* __restrict__ out, int64_t count, int slabs)
{
    psgd_sum_partials_body(partial, out, count, slabs, (int)blockIdx.x);
}

struct SumItem {
    const float* partial;
    float* out;
    int64_t count;
    int slabs;
};

__global__ void __launch_bounds__(256)
psgd_sum_partials_batch_kernel(PsgdBatch<SumItem> b)
{
    int local;
    const SumItem& it = b.item[psgd_batch_locate(b, &local)];
    psgd_sum_partials_body(it.partial, it.out, it.count, it.slabs, local);
}

// --------------------------------------- orthogonalisation of P, deferred ----
// The reference orthogonalises P between the two products (powerSGD_hook.py:516-531): a chain of
// r column steps over a tall thin matrix, all latency, with the machine idle around it.  Both
// things it feeds are linear in P: with P' = P T (T the upper triangular matrix of the column
// steps), Q = M^T P' = (M^T P) T.  So the round computes Q from the raw P at once, and gets T from
// the Gram matrix P^T P alone (conef_gs_gram.h): the first product leaves each workgroup's share of
// it, a workgroup per matrix riding in the second product's launch adds the shares and runs the r
// steps on the r x r matrix, and one short launch then applies T to the rows of P and of the raw Q
// (adding up Q's row-slab partials on the way, which was a launch of its own before).
struct GramTask {
    const double* parts[kPsgdBatchMax];   // [nparts][RP (RP + 1) / 2]
    int nparts[kPsgdBatchMax];
    float* tmat[kPsgdBatchMax];           // out: b_ij row-major [RP][RP] (zero unless i < j), then 1 / d_i [RP]
    int count;
    float eps;
};

// adds the shares, runs the r steps, leaves b_ij [RP][RP] and 1 / d_i [RP] in t_l (LDS, RP RP + RP
// floats), visible to every thread on return; all T threads of the workgroup call this
template <int RP, int T>
__device__ __forceinline__ void
gram_solve_lds(const double* __restrict__ parts, int nparts, float eps, float* t_l)
{
    constexpr int NG = RP * (RP + 1) / 2;
    constexpr bool kSideBySide = 2 * NG <= T;      // ranks up to 8: groups of NG threads add shares side by side
    constexpr int G = kSideBySide ? T / NG : 1;
    __shared__ double psum[G][kSideBySide ? NG : 1];
    __shared__ double gram[RP][RP + 1];
    __shared__ __attribute__((aligned(16))) float coef[RP][RP];
    __shared__ double dinv[RP];
    __shared__ double diag0[RP];
    __shared__ float dinvf[RP];
    const int tid = threadIdx.x;
    for (int i = tid; i < RP * RP; i += T) (&coef[0][0])[i] = 0.f;
    if constexpr (kSideBySide) {
        const int grp = tid / NG, e = tid - grp * NG;
        if (grp < G) {
            double s = 0.;
#pragma unroll 8
            for (int p = grp; p < nparts; p += G) s += parts[(size_t)p * NG + e];
            psum[grp][e] = s;
        }
        __syncthreads();
        if (tid < NG) {
            double s = 0.;
            for (int g = 0; g < G; ++g) s += psum[g][tid];       // the same order on every run
            int i, j;
            gsg_entry(tid, RP, &i, &j);
            gram[i][j] = s;
        }
    } else {
        // more entries than threads to share them out: a thread adds all shares of its entries, in
        // order, eight shares of each entry requested at a time (a share a trip otherwise: the sums
        // of a 16-share rank-32 matrix were most of what this workgroup spent)
        constexpr int EPT = (NG + T - 1) / T, kAhead = 8;
        double s[EPT];
#pragma unroll
        for (int u = 0; u < EPT; ++u) s[u] = 0.;
        for (int p0 = 0; p0 < nparts; p0 += kAhead) {
            double v[EPT][kAhead];
#pragma unroll
            for (int u = 0; u < EPT; ++u) {
                const int e = tid + u * T < NG ? tid + u * T : NG - 1;
#pragma unroll
                for (int q = 0; q < kAhead; ++q)
                    v[u][q] = parts[(size_t)(p0 + q < nparts ? p0 + q : nparts - 1) * NG + e];
            }
#pragma unroll
            for (int u = 0; u < EPT; ++u)
#pragma unroll
                for (int q = 0; q < kAhead; ++q)
                    if (p0 + q < nparts) s[u] += v[u][q];
        }
#pragma unroll
        for (int u = 0; u < EPT; ++u) {
            const int e = tid + u * T;
            if (e < NG) {
                int i, j;
                gsg_entry(e, RP, &i, &j);
                gram[i][j] = s[u];
            }
        }
    }
    __syncthreads();
    gsg_recurrence<RP, T>(gram, coef, dinv, dinvf, diag0, eps, tid);
    for (int i = tid; i < RP * RP; i += T) t_l[i] = (&coef[0][0])[i];
    if (tid < RP) t_l[RP * RP + tid] = dinvf[tid];
    __syncthreads();
}

// x_k -= b_ik x_i (k > i), x_i *= 1 / d_i for i = 0 .. r - 1: the reference's column steps
// (powerSGD_hook.py:21-43) on one row, coefficients from t_l as gram_solve_lds leaves them
template <int RP>
__device__ __forceinline__ void gram_apply_row(float* x, const float* t_l)
{
#pragma unroll
    for (int i = 0; i < RP; ++i) {
#pragma unroll
        for (int k = i + 1; k < RP; ++k) x[k] = fmaf(-t_l[i * RP + k], x[i], x[k]);
        x[i] = __fmul_rn(x[i], t_l[RP * RP + i]);
    }
}

// tmat receives the steps themselves (b_ij, 1 / d_i) or, EXPLICIT, their product: the upper
// triangular matrix T with orth(A) = A T, row-major [RP][RP] (row i is what the steps make of the
// unit vector e_i).  A row times T is RP independent multiply-adds a column where the steps are a
// chain of RP dependent exchanges, which is what the wide fix launch needs.
template <int RP, int T, bool EXPLICIT = false>
__device__ __forceinline__ void
gram_solve_body(const double* __restrict__ parts, int nparts, float* __restrict__ tmat, float eps)
{
    __shared__ float t_l[RP * RP + RP];
    gram_solve_lds<RP, T>(parts, nparts, eps, t_l);
    if (!EXPLICIT) {
        for (int i = threadIdx.x; i < RP * RP + RP; i += T) tmat[i] = t_l[i];
        return;
    }
    if constexpr (RP % 8 == 0 && RP * 8 <= T) {
        // eight lanes a row of T, lane c holding columns c, c + 8, ...: step j takes x_j from the lane
        // that holds it, the same multiply-adds in the same order as gram_apply_row on e_i
        constexpr int M = RP / 8;
        const int i = threadIdx.x >> 3, c = threadIdx.x & 7, lane = threadIdx.x & 63;
        if (i < RP) {
            float x[M];
#pragma unroll
            for (int m = 0; m < M; ++m) x[m] = c + 8 * m == i ? 1.f : 0.f;
#pragma unroll
            for (int j = 0; j < RP; ++j) {
                const float xj = __shfl(x[j >> 3], (lane & ~7) | (j & 7), 64);
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const int k = c + 8 * m;
                    if (k > j) x[m] = fmaf(-t_l[j * RP + k], xj, x[m]);
                    else if (k == j) x[m] = __fmul_rn(x[m], t_l[RP * RP + j]);
                }
            }
#pragma unroll
            for (int m = 0; m < M; ++m) tmat[i * RP + c + 8 * m] = x[m];
        }
    } else if ((int)threadIdx.x < RP) {
        float x[RP];
#pragma unroll
        for (int k = 0; k < RP; ++k) x[k] = k == (int)threadIdx.x ? 1.f : 0.f;
        gram_apply_row<RP>(x, t_l);
#pragma unroll
        for (int k = 0; k < RP; ++k) tmat[threadIdx.x * RP + k] = x[k];
    }
}

template <int RP>
__device__ __forceinline__ void load_row(const float* p, float* x)
{
    if (RP >= 4) {
#pragma unroll
        for (int c = 0; c < RP; c += 4) ld4(p + c, x + c);
    } else {
#pragma unroll
        for (int c = 0; c < RP; ++c) x[c] = p[c];
    }
}

template <int RP>
__device__ __forceinline__ void store_row(float* p, const float* x)
{
    if (RP >= 4) {
#pragma unroll
        for (int c = 0; c < RP; c += 4) st4(p + c, x + c);
    } else {
#pragma unroll
        for (int c = 0; c < RP; ++c) p[c] = x[c];
    }
}

// A whole matrix orthogonalised out of place by one workgroup of T threads from the shares of its
// Gram matrix: solve, then the column steps row by row (four rows a thread in flight).
template <int RP, int T>
__device__ __forceinline__ void
gram_orthogonalise_body(const float* __restrict__ src, float* __restrict__ dst, int rows, const double* parts, int nparts,
                        float eps)
{
    __shared__ float t_l[RP * RP + RP];
    gram_solve_lds<RP, T>(parts, nparts, eps, t_l);
    for (int r0 = threadIdx.x; r0 < rows; r0 += 4 * T) {
        float x[4][RP];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int row = r0 + u * T;
            load_row<RP>(src + (int64_t)(row < rows ? row : rows - 1) * RP, x[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int row = r0 + u * T;
            gram_apply_row<RP>(x[u], t_l);
            if (row < rows) store_row<RP>(dst + (int64_t)row * RP, x[u]);
        }
    }
}

template <int RP, bool FAST>
__global__ void __launch_bounds__(kMtpThreads)
psgd_mtp_gram_batch_kernel(PsgdBatch<MtpItem> b, GramTask g)
{
    if ((int)blockIdx.x < g.count) {
        gram_solve_body<RP, kMtpThreads>(g.parts[blockIdx.x], g.nparts[blockIdx.x], g.tmat[blockIdx.x], g.eps);
        return;
    }
    const int bx = (int)blockIdx.x - g.count;
    int i = 0;
    while (i + 1 < b.count && bx >= b.first[i + 1]) ++i;
    const MtpItem& it = b.item[i];
    const int local = bx - b.first[i];
    psgd_mtp_body<RP, FAST>(it.x, it.p, it.out, it.n, it.m, it.r, it.rows_per_slab, local % it.col_tiles,
                            local / it.col_tiles);
}

// rows of P and of the raw Q times T, a row a thread: x_k -= b_ik x_i (k > i), x_i *= 1 / d_i for
// i = 0 .. r - 1, the reference's column steps (powerSGD_hook.py:21-43) with the coefficients known
struct DeferFixItem {
    float* p;
    const float* qsrc;       // [slabs][m][RP] partials of Q = M^T P, or q itself with one slab
    float* q;
    const float* tmat;
    double* qgram;           // not null: the workgroups of Q also leave their rows' share of Q^T Q, [m / 256][RP (RP + 1) / 2]
    int64_t n, m;
    int slabs;
    int pblocks;             // workgroups that take rows of P; the others take rows of Q
};

template <int RP>
__global__ void __launch_bounds__(256)
psgd_defer_fix_batch_kernel(PsgdBatch<DeferFixItem> b)
{
    constexpr int NG = RP * (RP + 1) / 2;
    __shared__ float t_l[RP * RP + RP];
    __shared__ float rows_l[256][RP + 1];
    __shared__ double part_l[4][NG];
    int local;
    const DeferFixItem& it = b.item[psgd_batch_locate(b, &local)];
    const bool is_p = local < it.pblocks;
    const int64_t rows = is_p ? it.n : it.m;
    const int64_t row = (int64_t)(is_p ? local : local - it.pblocks) * 256 + threadIdx.x;
    const int64_t rc = row < rows ? row : rows - 1;
    const float* src = is_p ? it.p : it.qsrc;
    const int slabs = is_p ? 1 : it.slabs;
    const int64_t stride = it.m * RP;
    if (threadIdx.x < RP * RP + RP) t_l[threadIdx.x] = it.tmat[threadIdx.x];      // requested first: it travels with the rows
    float x[RP];
#pragma unroll
    for (int c = 0; c < RP; ++c) x[c] = 0.f;
    int sl = 0;
    for (; sl + 4 <= slabs; sl += 4) {                      // slabs in ascending order, four requested together
        float v[4][RP];
#pragma unroll
        for (int u = 0; u < 4; ++u) load_row<RP>(src + (int64_t)(sl + u) * stride + rc * RP, v[u]);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int c = 0; c < RP; ++c) x[c] += v[u][c];
    }
    for (; sl < slabs; ++sl) {
        float v[RP];
        load_row<RP>(src + (int64_t)sl * stride + rc * RP, v);
#pragma unroll
        for (int c = 0; c < RP; ++c) x[c] += v[c];
    }
    __syncthreads();
    gram_apply_row<RP>(x, t_l);
    if (row < rows) store_row<RP>((is_p ? it.p : it.q) + row * RP, x);
    if (!is_p && it.qgram) {                                // uniform over the workgroup
#pragma unroll
        for (int c = 0; c < RP; ++c) rows_l[threadIdx.x][c] = row < rows ? x[c] : 0.f;
        __syncthreads();
        const int e = threadIdx.x >> 2, quarter = threadIdx.x & 3;      // four threads an entry, 64 rows each
        if (e < NG) {
            int i, j;
            gsg_entry(e, RP, &i, &j);
            double s = 0.;
            for (int t = quarter * 64; t < quarter * 64 + 64; ++t) s = fma((double)rows_l[t][i], (double)rows_l[t][j], s);
            part_l[quarter][e] = s;
        }
        __syncthreads();
        if (threadIdx.x < NG)
            it.qgram[(size_t)(local - it.pblocks) * NG + threadIdx.x] =
                (part_l[0][threadIdx.x] + part_l[1][threadIdx.x]) + (part_l[2][threadIdx.x] + part_l[3][threadIdx.x]);
    }
}

// ---- ranks 16 and 32 ----
// The shares of P^T P of a finished P (the matrix-core product leaves P in column splits that a
// second kernel adds, so they cannot come out of the product itself): a workgroup per 256 rows,
// on the matrix cores in double (the first phase of gsg_kernel).
struct GramShareItem {
    const float* a;
    int64_t rows;
    double* parts;           // [ceil(rows / 256)][RP (RP + 1) / 2]
};

template <int RP>
__global__ void __launch_bounds__(kGsgThreads)
psgd_gram_shares_batch_kernel(PsgdBatch<GramShareItem> b)
{
    constexpr int NC = RP / 16, NT = NC * (NC + 1) / 2, NG = RP * (RP + 1) / 2;
    __shared__ double tiles[kGsgThreads / 64][NT][256];
    int local;
    const GramShareItem& it = b.item[psgd_batch_locate(b, &local)];
    const int r0 = local * 256;
    const int r1 = (int64_t)r0 + 256 < it.rows ? r0 + 256 : (int)it.rows;
    gsg_gram_tiles<RP>(it.a, r0, r1, tiles);
    __syncthreads();
    for (int e = threadIdx.x; e < NG; e += kGsgThreads) {
        int i, j;
        gsg_entry(e, RP, &i, &j);
        it.parts[(size_t)local * NG + e] = gsg_tiles_entry<RP>(tiles, i, j);
    }
}

// P <- P T and Q <- (sum of the slab partials of the raw Q) T at ranks 16 and 32.  A workgroup
// takes 32 rows; a thread adds the slabs of one 16-byte piece of a row (eight slabs requested
// together: a matrix-core Q has up to 32 of them), the rows meet in LDS, and a wave then forms
// row times T for a few rows at a time, a lane per column.
template <int RP>
__global__ void __launch_bounds__(256)
psgd_defer_fix_wide_batch_kernel(PsgdBatch<DeferFixItem> b)
{
    constexpr int QPR = RP / 4;                 // 16-byte pieces of a row
    constexpr int ROWS = 256 / QPR;             // rows a workgroup takes: 64 at rank 16, 32 at rank 32
    __shared__ float t_l[RP * RP + RP];
    __shared__ float rows_l[ROWS][RP + 1];
    int local;
    const DeferFixItem& it = b.item[psgd_batch_locate(b, &local)];
    const bool is_p = local < it.pblocks;
    const int64_t rows = is_p ? it.n : it.m;
    const int lrow = threadIdx.x / QPR, piece = threadIdx.x - lrow * QPR;
    const int64_t row = (int64_t)(is_p ? local : local - it.pblocks) * ROWS + lrow;
    const int64_t rc = row < rows ? row : rows - 1;
    const float* src = (is_p ? it.p : it.qsrc) + rc * RP + 4 * piece;
    const int slabs = is_p ? 1 : it.slabs;
    const int64_t stride = it.m * RP;
    for (int i = threadIdx.x; i < RP * RP; i += 256) t_l[i] = it.tmat[i];      // T itself here (gram_solve_body, EXPLICIT)
    float x[4] = {0.f, 0.f, 0.f, 0.f};
    int sl = 0;
    for (; sl + 8 <= slabs; sl += 8) {          // slabs in ascending order
        float v[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u) ld4(src + (int64_t)(sl + u) * stride, v[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int c = 0; c < 4; ++c) x[c] += v[u][c];
    }
    for (; sl < slabs; ++sl) {
        float v[4];
        ld4(src + (int64_t)sl * stride, v);
#pragma unroll
        for (int c = 0; c < 4; ++c) x[c] += v[c];
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) rows_l[lrow][4 * piece + c] = x[c];
    __syncthreads();
    // row times T: a wave takes 64 / RP rows at a time, a lane per column, RP independent multiply-adds
    // in ascending order of the row's entries
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int RPW = 64 / RP;                // rows a wave holds at once: 4 or 2
    const int col = lane % RP, sub = lane / RP;
    float out[ROWS / (4 * RPW)];
#pragma unroll
    for (int u = 0; u < ROWS / (4 * RPW); ++u) {
        const int lr = wave * RPW + u * 4 * RPW + sub;
        float acc = 0.f;
#pragma unroll 8
        for (int i = 0; i < RP; ++i) acc = fmaf(rows_l[lr][i], t_l[i * RP + col], acc);      // T is zero below the diagonal
        out[u] = acc;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < ROWS / (4 * RPW); ++u) rows_l[wave * RPW + u * 4 * RPW + sub][col] = out[u];
    __syncthreads();
    if (row < rows) {
        float o[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) o[c] = rows_l[lrow][4 * piece + c];
        st4((is_p ? it.p : it.q) + row * RP + 4 * piece, o);
    }
}

// ------------------------------------------- matrix-core products, batched ----
// The MFMA kernels of conef_psgd_mfma.h over the matrices of a bucket: workgroup `local` of an
// item is workgroup (local % its first grid dimension, local / it) of the single-matrix launch.
struct MfmaMqItem {
    float* x;
    const float* err;
    const float* q;
    float* out;
    int64_t n;
    int m, r, cols_per_split, row_tiles;
    ConefMod mod;       // of width 1: the batched kernel never unsketches
};

template <int MODE>
__global__ void __launch_bounds__(kMfmaThreads)
psgd_mfma_mq_batch_kernel(PsgdBatch<MfmaMqItem> b)
{
    static_assert(MODE == 0 || MODE == 1, "the sketch query of a batch runs as a launch of its own");
    int local;
    const MfmaMqItem& it = b.item[psgd_batch_locate(b, &local)];
    const ConefSeeds hs = {0, 0, 0, 0};
    psgd_mfma_mq_body<MODE>(it.x, it.err, nullptr, nullptr, it.q, it.out, it.n, it.m, it.r, it.cols_per_split, it.mod, 0.f,
                            hs, local % it.row_tiles, local / it.row_tiles);
}

struct MfmaMtpItem {
    const float* x;
    const float* p;
    float* out;
    int64_t n;
    int m, r, rows_per_slab, col_tiles;
    int v;              // floats a lane loads at a time (4, 2, 1): read by the launch that takes every width
};

template <int V>
__global__ void __launch_bounds__(kMfmaThreads)
psgd_mfma_mtp_batch_kernel(PsgdBatch<MfmaMtpItem> b)
{
    int local;
    const MfmaMtpItem& it = b.item[psgd_batch_locate(b, &local)];
    psgd_mfma_mtp_body<V>(it.x, it.p, it.out, it.n, it.m, it.r, it.rows_per_slab, local % it.col_tiles, local / it.col_tiles);
}

// the same with the workgroups in front that solve the matrices' Gram systems (deferred
// orthogonalisation of P at ranks 16 and 32), and one launch for the matrices of every vector
// width: the solving workgroups outlast the products of one width, and a launch per width would
// each wait for its slowest workgroup
template <int RP>
__global__ void __launch_bounds__(kMfmaThreads)
psgd_mfma_mtp_gram_batch_kernel(PsgdBatch<MfmaMtpItem> b, GramTask g)
{
    if ((int)blockIdx.x < g.count) {
        gram_solve_body<RP, kMfmaThreads, true>(g.parts[blockIdx.x], g.nparts[blockIdx.x], g.tmat[blockIdx.x], g.eps);
        return;
    }
    const int bx = (int)blockIdx.x - g.count;
    int i = 0;
    while (i + 1 < b.count && bx >= b.first[i + 1]) ++i;
    const MfmaMtpItem& it = b.item[i];
    const int local = bx - b.first[i];
    const int ct = local % it.col_tiles, slab = local / it.col_tiles;
    if (it.v == 4) psgd_mfma_mtp_body<4>(it.x, it.p, it.out, it.n, it.m, it.r, it.rows_per_slab, ct, slab);
    else if (it.v == 2) psgd_mfma_mtp_body<2>(it.x, it.p, it.out, it.n, it.m, it.r, it.rows_per_slab, ct, slab);
    else psgd_mfma_mtp_body<1>(it.x, it.p, it.out, it.n, it.m, it.r, it.rows_per_slab, ct, slab);
}

struct MfmaPqtItem {
    float* x;
    float* err;
    const float* p;
    const float* q;
    int64_t n;
    int m, rows_per_slab, col_wgs;
};

template <int R, int MODE>
__global__ void __launch_bounds__(kMfmaThreads)
psgd_mfma_pqt_batch_kernel(PsgdBatch<MfmaPqtItem> b)
{
    int local;
    const MfmaPqtItem& it = b.item[psgd_batch_locate(b, &local)];
    psgd_mfma_pqt_body<R, MODE>(it.x, it.err, it.p, it.q, it.n, it.m, it.rows_per_slab, local % it.col_wgs,
                                local / it.col_wgs);
}

// X += alpha * unsketch(cs) over the matrices of a bucket (DenseCS.query, CountSketch.py:51-66):
// a thread owns a column quad of a group of rows, its (bucket, sign) words from the plan's table
// or hashed, once for the group.  VEC: m % 4 == 0 and 16-byte aligned x (and table).
struct QueryItem {
    float* x;
    const float* cs;
    const uint32_t* pktab;
    int64_t n;
    int m, rows_per_block, col_blocks;
    ConefMod mod;
};

template <bool VEC>
__global__ void __launch_bounds__(256)
psgd_cs_query_batch_kernel(PsgdBatch<QueryItem> b, float alpha, ConefSeeds hs)
{
    int local;
    const QueryItem& it = b.item[psgd_batch_locate(b, &local)];
    const int bx = local % it.col_blocks, by = local / it.col_blocks;
    const int c0 = (bx * 256 + (int)threadIdx.x) * 4;
    if (c0 >= it.m) return;
    uint32_t pk[4];
    if (VEC && it.pktab) {
        const uint4 t = *reinterpret_cast<const uint4*>(it.pktab + c0);
        pk[0] = t.x; pk[1] = t.y; pk[2] = t.z; pk[3] = t.w;
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
            pk[k] = c0 + k < it.m ? (it.pktab ? it.pktab[c0 + k] : conef_bucket_sign(c0 + k, it.mod, hs.a, hs.b, hs.sa, hs.sb))
                                  : 0u;
    }
    const int64_t r0 = (int64_t)by * it.rows_per_block;
    const int64_t r1 = r0 + it.rows_per_block < it.n ? r0 + it.rows_per_block : it.n;
    const int w = (int)it.mod.w;
    for (int64_t r = r0; r < r1; ++r) {
        const float* row = it.cs + r * w;
        float* xr = it.x + r * it.m + c0;
        if (VEC) {
            float4 v = *reinterpret_cast<const float4*>(xr);
            v.x = __fadd_rn(v.x, conef_query_term(row[pk[0] & 0x7fffffffu], pk[0], alpha));
            v.y = __fadd_rn(v.y, conef_query_term(row[pk[1] & 0x7fffffffu], pk[1], alpha));
            v.z = __fadd_rn(v.z, conef_query_term(row[pk[2] & 0x7fffffffu], pk[2], alpha));
            v.w = __fadd_rn(v.w, conef_query_term(row[pk[3] & 0x7fffffffu], pk[3], alpha));
            *reinterpret_cast<float4*>(xr) = v;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (c0 + k < it.m) xr[k] = __fadd_rn(xr[k], conef_query_term(row[pk[k] & 0x7fffffffu], pk[k], alpha));
        }
    }
}

// DenseCS.update(vec, beta) (CountSketch.py:27-48) of the sketches of a bucket's matrices on
// row-list plans, vec = the item's dense residual.
struct RowlistVecItem {
    ConefListVec front;
    ConefRowlistView plan;
    const float* cs_in;
    float* cs_out;
    int64_t n;
    int d, w, rb;
};

__global__ void __launch_bounds__(kConefRowlistThreads)
psgd_rowlist_vec_batch_kernel(PsgdBatch<RowlistVecItem> b, double one_minus_beta)
{
    int local;
    const RowlistVecItem& it = b.item[psgd_batch_locate(b, &local)];
    conef_rowlist_body<float, ConefListVec>(it.front, it.plan, it.cs_in, it.cs_out, it.n, it.d, it.w, it.rb, one_minus_beta,
                                            local);
}

// ------------------------------------------------------------ M = P Q^T ----
// MODE 0: write M.  MODE 1: also write the dense residual E = X - M (X = what M held on entry).
// A thread owns a column quad (its 4 x r slice of Q stays in registers), the workgroup walks a slab
// of rows; the row of P is uniform over the workgroup.
template <int RP, int MODE, bool FAST>
__device__ __forceinline__ void
psgd_pqt_body(float* __restrict__ x, float* __restrict__ err, const float* __restrict__ p,
              const float* __restrict__ q, int64_t n, int m, int r, int rows_per_slab, int bx, int by)
{
    const int c0 = (bx * 256 + threadIdx.x) * 4;
    if (c0 >= m) return;
    const int64_t i0 = (int64_t)by * rows_per_slab;
    const int64_t i1 = i0 + rows_per_slab < n ? i0 + rows_per_slab : n;
    float qf[4][RP];
    if (FAST) {
        float flat[4 * RP];
#pragma unroll
        for (int t = 0; t < RP; ++t) ld4(q + (int64_t)c0 * RP + 4 * t, flat + 4 * t);
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int c = 0; c < RP; ++c) qf[k][c] = flat[k * RP + c];
        for (int64_t ib = i0; ib < i1; ib += 4) {          // four rows in flight
            float xv[4][4];
            if (MODE == 1) {
#pragma unroll
                for (int u = 0; u < 4; ++u) ld4(x + (ib + u < i1 ? ib + u : i1 - 1) * m + c0, xv[u]);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int64_t i = ib + u;
                if (i >= i1) break;
                const float* pi = p + i * RP;
                float mh[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < RP; ++c) {
                    float pc = pi[c];
#pragma unroll
                    for (int k = 0; k < 4; ++k) mh[k] = fmaf(pc, qf[k][c], mh[k]);
                }
                if (MODE == 1) {
                    float ev[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) ev[k] = __fsub_rn(xv[u][k], mh[k]);
                    st4(err + i * m + c0, ev);
                }
                st4(x + i * m + c0, mh);
            }
        }
    } else {
        const int valid = m - c0 < 4 ? m - c0 : 4;
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int c = 0; c < RP; ++c) qf[k][c] = (k < valid && c < r) ? q[(int64_t)(c0 + k) * r + c] : 0.f;
        for (int64_t i = i0; i < i1; ++i) {
            const float* pi = p + i * r;
            float mh[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < RP; ++c) {
                float pc = c < r ? pi[c] : 0.f;
#pragma unroll
                for (int k = 0; k < 4; ++k) mh[k] = fmaf(pc, qf[k][c], mh[k]);
            }
            for (int k = 0; k < valid; ++k) {
                int64_t f = i * m + c0 + k;
                if (MODE == 1) err[f] = __fsub_rn(x[f], mh[k]);
                x[f] = mh[k];
            }
        }
    }
}

template <int RP, int MODE, bool FAST>
__global__ void __launch_bounds__(256)
psgd_pqt_kernel(float* __restrict__ x, float* __restrict__ err, const float* __restrict__ p,
                const float* __restrict__ q, int64_t n, int m, int r, int rows_per_slab)
{
    psgd_pqt_body<RP, MODE, FAST>(x, err, p, q, n, m, r, rows_per_slab, (int)blockIdx.x, (int)blockIdx.y);
}

struct PqtItem {
    float* x;
    float* err;
    const float* p;
    const float* q;
    int64_t n;
    int m, r, rows_per_slab, col_tiles;
};

template <int RP, int MODE, bool FAST>
__global__ void __launch_bounds__(256)
psgd_pqt_batch_kernel(PsgdBatch<PqtItem> b)
{
    int local;
    const PqtItem& it = b.item[psgd_batch_locate(b, &local)];
    psgd_pqt_body<RP, MODE, FAST>(it.x, it.err, it.p, it.q, it.n, it.m, it.r, it.rows_per_slab, local % it.col_tiles,
                                  local / it.col_tiles);
}

// Front of the row-list sketch kernel: the value to sketch is the residual X - P Q^T, and M is
// overwritten with P Q^T on the way (powerSGD_hook.py:551,563-564).
template <int RP, bool FAST>
struct ListPsgdResidual {
    float* x;
    const float* p;
    const float* q;
    int r;
    static constexpr bool kNeedsCells = false;
    struct Regs {};
    __device__ __forceinline__ void stage(int64_t row0, int rows, int d, int, float* vals, const float*,
                                          const uint32_t*) const
    {
        float* base = x + row0 * d;
        if (FAST) {
            // A thread owns column quads c4 = t, t + 256, ... and takes the tile's rows two at a time
            // with the quad's slice of Q (4 x RP floats) in registers: Q is read once per quad and
            // tile, not once per element.  Narrow matrices (fewer quads than threads) split the rows
            // over thread groups instead.  The tile's rows of P wait in LDS; the next two rows of the
            // quad - or the next quad's slice of Q and its first two rows - are requested before the
            // current two are used, so that a thread has one round trip per tile, not one per step.
            __shared__ float ptile[16 * RP];              // at most 16 rows a tile
            for (int i = threadIdx.x; i < rows * RP; i += kConefRowlistThreads) ptile[i] = p[row0 * RP + i];
            const int d4 = d >> 2;
            const int lanes = d4 < kConefRowlistThreads ? d4 : kConefRowlistThreads;
            const int groups = kConefRowlistThreads / lanes, grp = threadIdx.x / lanes;
            const int step = 2 * groups;
            int c4 = threadIdx.x - grp * lanes, rw = 2 * grp;
            bool have = grp < groups && c4 < d4 && rw < rows;
            float flat[4 * RP], flatn[4 * RP], x0n[4], x1n[4];
            auto request_rows = [&](int quad, int row) {
                const int r1 = row + 1 < rows ? row + 1 : row;
                ld4(base + (int64_t)row * d + 4 * quad, x0n);
                ld4(base + (int64_t)r1 * d + 4 * quad, x1n);
            };
            if (have) {
#pragma unroll
                for (int v = 0; v < RP; ++v) ld4(q + (int64_t)c4 * 4 * RP + 4 * v, flat + 4 * v);
                request_rows(c4, rw);
            }
            __syncthreads();
            while (have) {
                const int cur_c4 = c4, cur_rw = rw;
                const int r1 = cur_rw + 1 < rows ? cur_rw + 1 : cur_rw;
                float x0[4], x1[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    x0[k] = x0n[k];
                    x1[k] = x1n[k];
                }
                rw += step;
                bool new_quad = false;
                if (rw >= rows) {
                    rw = 2 * grp;
                    c4 += lanes;
                    new_quad = true;
                }
                have = c4 < d4;
                if (have) {
                    if (new_quad) {
#pragma unroll
                        for (int v = 0; v < RP; ++v) ld4(q + (int64_t)c4 * 4 * RP + 4 * v, flatn + 4 * v);
                    }
                    request_rows(c4, rw);
                }
                const float* pa = ptile + cur_rw * RP;
                const float* pb = ptile + r1 * RP;
                float m0[4] = {0.f, 0.f, 0.f, 0.f}, m1[4] = {0.f, 0.f, 0.f, 0.f}, v0[4], v1[4];
#pragma unroll
                for (int c = 0; c < RP; ++c) {
                    const float p0 = pa[c], p1 = pb[c];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        m0[k] = fmaf(p0, flat[k * RP + c], m0[k]);
                        m1[k] = fmaf(p1, flat[k * RP + c], m1[k]);
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v0[k] = __fsub_rn(x0[k], m0[k]);
                    v1[k] = __fsub_rn(x1[k], m1[k]);
                }
                st4(base + (int64_t)cur_rw * d + 4 * cur_c4, m0);
                st4(vals + cur_rw * d + 4 * cur_c4, v0);
                if (cur_rw + 1 < rows) {
                    st4(base + (int64_t)r1 * d + 4 * cur_c4, m1);
                    st4(vals + r1 * d + 4 * cur_c4, v1);
                }
                if (new_quad && have) {
#pragma unroll
                    for (int t = 0; t < 4 * RP; ++t) flat[t] = flatn[t];
                }
            }
        } else {
            const int total = rows * d;
            int row = threadIdx.x / d, col = threadIdx.x - row * d;
            const int srow = kConefRowlistThreads / d, sc = kConefRowlistThreads - srow * d;
            for (int e = threadIdx.x; e < total; e += kConefRowlistThreads) {
                const float* pi = p + (row0 + row) * r;
                const float* qk = q + (int64_t)col * r;
                float mh = 0.f;
#pragma unroll
                for (int c = 0; c < RP; ++c)
                    if (c < r) mh = fmaf(pi[c], qk[c], mh);
                vals[e] = __fsub_rn(base[e], mh);
                base[e] = mh;
                row += srow;
                col += sc;
                if (col >= d) {
                    col -= d;
                    ++row;
                }
            }
        }
    }
};

// Same residual as a front of the atomics-based sketch kernels (no plan given).
struct FrontPsgdResidual {
    float* x;
    const float* p;
    const float* q;
    int64_t d;
    int r;
    __device__ __forceinline__ float lowrank(int64_t row, int64_t col) const
    {
        const float* pi = p + row * r;
        const float* qk = q + col * r;
        float mh = 0.f;
        for (int c = 0; c < r; ++c) mh = fmaf(pi[c], qk[c], mh);
        return mh;
    }
    __device__ __forceinline__ float one(int64_t row, int64_t i, float, uint32_t) const
    {
        float mh = lowrank(row, i);
        float v = __fsub_rn(x[row * d + i], mh);
        x[row * d + i] = mh;
        return v;
    }
    template <bool VEC>
    __device__ __forceinline__ void four(int64_t row, int64_t c0, int valid, const float*, const uint32_t*,
                                         float* v) const
    {
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = k < valid ? one(row, c0 + k, 0.f, 0u) : 0.f;
    }
};

// ------------------------------------------------------------ Gram-Schmidt ----
// In place on a row-major [rows, r] matrix.  Column by column: col /= ||col|| (+eps when eps != 0),
// then every later column loses its projection on col (powerSGD_hook.py:21-43).  Each thread keeps
// to its own rows, so the only exchange per column is one reduction of (||col||^2, col . later
// columns); the projection coefficients of the normalised column are those dot products divided
// by the norm.
//
// Small matrices: one workgroup, the matrix lives in LDS (row stride r+1: no bank conflicts) for
// the whole factorisation.
constexpr size_t kGsLdsLimit = 144 * 1024;

template <int RP>
__global__ void __launch_bounds__(1024)
gram_schmidt_lds_kernel(float* __restrict__ a, int rows, int r, float eps)
{
    extern __shared__ float gs_lds[];
    float* red = gs_lds;                 // [16][RP]
    float* tot = red + 16 * RP;          // [RP]
    float* al = tot + RP;                // [rows][r+1]
    const int ld = r + 1;
    const int nthreads = blockDim.x, nwaves = nthreads >> 6;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int e = threadIdx.x; e < rows * r; e += nthreads) {
        int k = e / r;
        al[k * ld + (e - k * r)] = a[e];
    }
    __syncthreads();
    for (int i = 0; i < r; ++i) {
        float acc[RP];
#pragma unroll
        for (int c = 0; c < RP; ++c) acc[c] = 0.f;
        for (int k = threadIdx.x; k < rows; k += nthreads) {
            const float* row = al + k * ld;
            float ci = row[i];
#pragma unroll
            for (int c = 0; c < RP; ++c)
                if (i + c < r) acc[c] = fmaf(ci, row[i + c], acc[c]);
        }
#pragma unroll
        for (int c = 0; c < RP; ++c) {
            if (i + c < r) {
                float s = conef_wave_sum(acc[c]);
                if (lane == 0) red[wave * RP + c] = s;
            }
        }
        __syncthreads();
        if (threadIdx.x < RP) {
            float s = 0.f;
            for (int wv = 0; wv < nwaves; ++wv) s += red[wv * RP + threadIdx.x];
            tot[threadIdx.x] = s;
        }
        __syncthreads();
        float nrm = sqrtf(tot[0]);
        float den = eps == 0.f ? nrm : nrm + eps;
        float coef[RP];
#pragma unroll
        for (int c = 1; c < RP; ++c) coef[c] = (i + c < r) ? tot[c] / den : 0.f;
        for (int k = threadIdx.x; k < rows; k += nthreads) {
            float* row = al + k * ld;
            float ci = row[i] / den;
            row[i] = ci;
#pragma unroll
            for (int c = 1; c < RP; ++c)
                if (i + c < r) row[i + c] = __fsub_rn(row[i + c], __fmul_rn(coef[c], ci));
        }
        // the next column's sums read only the thread's own rows; red/tot are rewritten after the
        // next pair of barriers has been passed by everyone who read them
    }
    __syncthreads();
    for (int e = threadIdx.x; e < rows * r; e += nthreads) {
        int k = e / r;
        a[e] = al[k * ld + (e - k * r)];
    }
}

// Matrices of up to 32768 elements: one workgroup of four waves keeps the whole matrix in
// registers (thread t owns rows t, t+256, ...: 128 / RP of them at most), so a column step is the
// thread's own multiply-adds, one DPP reduction per remaining column, one barrier, and four LDS
// reads per remaining column (the waves' sums, added in wave order by every thread alike).
constexpr int kGsRegThreads = 256;
constexpr int kGsRegFloats = 128;      // matrix elements a thread may hold

// one column step; I is a template argument so that every register index is a constant
template <int RP, int RPT, int I>
__device__ __forceinline__ void gs_reg_step(float (&v)[RPT][RP], float (&red)[2][4][RP], int nrt, float eps, int wave,
                                            int lane)
{
    float acc[RP];
#pragma unroll
    for (int c = I; c < RP; ++c) acc[c] = 0.f;
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        if (t < nrt) {
#pragma unroll
            for (int c = I; c < RP; ++c) acc[c] = fmaf(v[t][I], v[t][c], acc[c]);
        }
    }
#pragma unroll
    for (int c = I; c < RP; ++c) {
        float s = conef_wave_sum_to_last(acc[c]);
        if (lane == 63) red[I & 1][wave][c] = s;
    }
    __syncthreads();
    float tot[RP];
#pragma unroll
    for (int c = I; c < RP; ++c) tot[c] = (red[I & 1][0][c] + red[I & 1][1][c]) + (red[I & 1][2][c] + red[I & 1][3][c]);
    const float nrm = sqrtf(tot[I]);
    const float inv = 1.f / (eps == 0.f ? nrm : nrm + eps);     // one division per column, products after
    float coef[RP];
#pragma unroll
    for (int c = I + 1; c < RP; ++c) coef[c] = __fmul_rn(tot[c], inv);
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        if (t < nrt) {
            const float ci = __fmul_rn(v[t][I], inv);
            v[t][I] = ci;
#pragma unroll
            for (int c = I + 1; c < RP; ++c) v[t][c] = fmaf(-coef[c], ci, v[t][c]);
        }
    }
}

template <int RP, int RPT, int I>
__device__ __forceinline__ void gs_reg_steps(float (&v)[RPT][RP], float (&red)[2][4][RP], int r, int nrt, float eps,
                                             int wave, int lane)
{
    if constexpr (I < RP) {
        if (I < r) {                    // uniform: columns past r hold zeros and are not stored
            gs_reg_step<RP, RPT, I>(v, red, nrt, eps, wave, lane);
            gs_reg_steps<RP, RPT, I + 1>(v, red, r, nrt, eps, wave, lane);
        }
    }
}

// One launch orthogonalises up to kGsBatchMax matrices of the same rank, one workgroup each: the P
// (or Q) factors of all tensors of a gradient bucket are independent of each other.
constexpr int kGsBatchMax = 48;
struct GsBatch {
    float* a[kGsBatchMax];
    int rows[kGsBatchMax];
};

template <int RP, int RPT>
__device__ __forceinline__ void gs_reg_body(float* a, int rows, float (&red)[2][4][RP], int r, float eps,
                                            const float* src = nullptr)
{
    if (!src) src = a;          // in place unless the matrix is to be read from elsewhere
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nrt = (rows + kGsRegThreads - 1) / kGsRegThreads;      // row slots in use (uniform)
    float v[RPT][RP];
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int k = threadIdx.x + t * kGsRegThreads;
#pragma unroll
        for (int c = 0; c < RP; ++c) v[t][c] = 0.f;
        if (t < nrt && k < rows) {
            const float* row = src + (int64_t)k * r;
            if (RP >= 4 && r == RP) {
#pragma unroll
                for (int c = 0; c < RP; c += 4) ld4(row + c, &v[t][c]);
            } else {
#pragma unroll
                for (int c = 0; c < RP; ++c)
                    if (c < r) v[t][c] = row[c];
            }
        }
    }
    gs_reg_steps<RP, RPT, 0>(v, red, r, nrt, eps, wave, lane);
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int k = threadIdx.x + t * kGsRegThreads;
        if (t < nrt && k < rows) {
            float* row = a + (int64_t)k * r;
            if (RP >= 4 && r == RP) {
#pragma unroll
                for (int c = 0; c < RP; c += 4) st4(row + c, &v[t][c]);
            } else {
#pragma unroll
                for (int c = 0; c < RP; ++c)
                    if (c < r) row[c] = v[t][c];
            }
        }
    }
}

template <int RP, int RPT>
__global__ void __launch_bounds__(kGsRegThreads)
gram_schmidt_reg_kernel(GsBatch batch, int r, float eps)
{
    __shared__ float red[2][4][RP];
    gs_reg_body<RP, RPT>(batch.a[blockIdx.x], batch.rows[blockIdx.x], red, r, eps);
}

// The same, for a launch whose matrices differ in height: every workgroup takes the body sized
// for its own matrix (1, 4, 16 or all row slots a thread), so the short factors of a bucket are
// not a launch of their own in front of the tall ones.  A workgroup runs exactly the code the
// one-size kernel would run on its matrix.
template <int RP>
__device__ __forceinline__ void gs_reg_any_height(float* a, int rows, float (&red)[2][4][RP], int r, float eps,
                                                  const float* src = nullptr)
{
    constexpr int kAll = kGsRegFloats / RP;
    const int nrt = (rows + kGsRegThreads - 1) / kGsRegThreads;
    if (nrt <= 1) gs_reg_body<RP, 1>(a, rows, red, r, eps, src);
    else if (nrt <= 4 && kAll >= 4) gs_reg_body<RP, (kAll >= 4 ? 4 : kAll)>(a, rows, red, r, eps, src);
    else if (nrt <= 16 && kAll >= 16) gs_reg_body<RP, (kAll >= 16 ? 16 : kAll)>(a, rows, red, r, eps, src);
    else gs_reg_body<RP, kAll>(a, rows, red, r, eps, src);
}

template <int RP>
__global__ void __launch_bounds__(kGsRegThreads)
gram_schmidt_reg_mixed_kernel(GsBatch batch, int r, float eps)
{
    __shared__ float red[2][4][RP];
    gs_reg_any_height<RP>(batch.a[blockIdx.x], batch.rows[blockIdx.x], red, r, eps);
}

// Matrices to orthogonalise out of place by workgroups that ride along in another kernel's launch.
constexpr int kGsAheadRowSlots = 4;      // rows a thread of such a workgroup holds at most
struct GsAhead {
    const float* src[kPsgdBatchMax];
    float* dst[kPsgdBatchMax];
    int rows[kPsgdBatchMax];
    int count, r;
    float eps;
    // not null: the shares of src^T src are known (nparts of them); the matrix is then
    // orthogonalised from its Gram matrix, whatever its height (gram_orthogonalise_body)
    const double* parts[kPsgdBatchMax];
    int nparts[kPsgdBatchMax];
};

template <int RP>
__device__ __forceinline__ void gs_ahead_body(const GsAhead& g, int k)
{
    if (g.parts[k]) {
        gram_orthogonalise_body<RP, kGsRegThreads>(g.src[k], g.dst[k], g.rows[k], g.parts[k], g.nparts[k], g.eps);
        return;
    }
    // at most kGsAheadRowSlots rows a thread: the taller bodies hold over a hundred values in
    // registers, and the host kernel's allocation is what every workgroup of its launch gets
    __shared__ float red[2][4][RP];
    if (g.rows[k] <= kGsRegThreads) gs_reg_body<RP, 1>(g.dst[k], g.rows[k], red, g.r, g.eps, g.src[k]);
    else gs_reg_body<RP, kGsAheadRowSlots>(g.dst[k], g.rows[k], red, g.r, g.eps, g.src[k]);
}

// Matrices beyond one workgroup's registers: the same register-resident scheme over up to 128
// workgroups launched cooperatively (all resident at once).  A column step ends with every
// workgroup leaving its partial sums in the workspace and meeting the others at a counter; after
// that every workgroup adds all partials in the same order.  The wait is bounded: a workgroup that
// does not see the others arrive within about a second gives up and the kernel ends (the matrix
// is then garbage; with a cooperative launch this cannot happen unless the device is lost).
constexpr int kGsGridMaxWgs = 128;
constexpr unsigned kGsSpinLimit = 1u << 22;

struct GsGridWs {
    unsigned arrived;      // workgroups that have reached a barrier, over all steps so far
    unsigned gave_up;
    unsigned pad[62];
    float sums[2][kGsGridMaxWgs][32];
};

__global__ void gs_grid_reset_kernel(GsGridWs* ws)
{
    ws->arrived = 0;
    ws->gave_up = 0;
}

template <int RP, int RPT, int I>
__device__ __forceinline__ bool gs_grid_step(float (&v)[RPT][RP], float (&red)[4][RP], float* part, float* tot_l,
                                             GsGridWs* ws, int nrt, float eps, int wave, int lane)
{
    float acc[RP];
#pragma unroll
    for (int c = I; c < RP; ++c) acc[c] = 0.f;
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        if (t < nrt) {
#pragma unroll
            for (int c = I; c < RP; ++c) acc[c] = fmaf(v[t][I], v[t][c], acc[c]);
        }
    }
#pragma unroll
    for (int c = I; c < RP; ++c) {
        float s = conef_wave_sum_to_last(acc[c]);
        if (lane == 63) red[wave][c] = s;
    }
    __syncthreads();
    const int nwg = (int)gridDim.x;
    float* mine = ws->sums[I & 1][blockIdx.x];
    if ((int)threadIdx.x >= I && (int)threadIdx.x < RP)
        mine[threadIdx.x] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
    __syncthreads();      // the partials are out before thread 0 announces the workgroup (release below)
    if (threadIdx.x == 0) {
        const unsigned target = (unsigned)(I + 1) * (unsigned)nwg;
        __hip_atomic_fetch_add(&ws->arrived, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        unsigned spins = 0;
        bool ok = true;
        while (__hip_atomic_load(&ws->arrived, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < target) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > kGsSpinLimit || __hip_atomic_load(&ws->gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                ok = false;
                __hip_atomic_store(&ws->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                gs_count_give_up();
                break;
            }
        }
        tot_l[RP] = ok ? 1.f : 0.f;
    }
    __syncthreads();
    if (tot_l[RP] == 0.f) return false;      // thread 0's acquire, handed on by the barrier, covers the reads below
    // all partials of this step: thread (g, c) reads one, one thread per column adds them in order
    for (int e = threadIdx.x; e < nwg * RP; e += kGsRegThreads) {
        const int g = e / RP, c = e - g * RP;
        part[e] = c >= I ? ws->sums[I & 1][g][c] : 0.f;
    }
    __syncthreads();
    if ((int)threadIdx.x >= I && (int)threadIdx.x < RP) {
        float s = 0.f;
        for (int g = 0; g < nwg; ++g) s += part[g * RP + threadIdx.x];
        tot_l[threadIdx.x] = s;
    }
    __syncthreads();
    const float nrm = sqrtf(tot_l[I]);
    const float inv = 1.f / (eps == 0.f ? nrm : nrm + eps);
    float coef[RP];
#pragma unroll
    for (int c = I + 1; c < RP; ++c) coef[c] = __fmul_rn(tot_l[c], inv);
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        if (t < nrt) {
            const float ci = __fmul_rn(v[t][I], inv);
            v[t][I] = ci;
#pragma unroll
            for (int c = I + 1; c < RP; ++c) v[t][c] = fmaf(-coef[c], ci, v[t][c]);
        }
    }
    return true;
}

template <int RP, int RPT, int I>
__device__ __forceinline__ void gs_grid_steps(float (&v)[RPT][RP], float (&red)[4][RP], float* part, float* tot_l,
                                              GsGridWs* ws, int r, int nrt, float eps, int wave, int lane)
{
    if constexpr (I < RP) {
        if (I < r) {
            if (gs_grid_step<RP, RPT, I>(v, red, part, tot_l, ws, nrt, eps, wave, lane))
                gs_grid_steps<RP, RPT, I + 1>(v, red, part, tot_l, ws, r, nrt, eps, wave, lane);
        }
    }
}

// workgroup b owns rows [b * rows_per_wg, +rows_per_wg); thread t its rows t, t+256, ...
template <int RP, int RPT>
__global__ void __launch_bounds__(kGsRegThreads)
gram_schmidt_grid_kernel(float* __restrict__ a, int64_t rows, int r, float eps, int rows_per_wg, GsGridWs* ws)
{
    __shared__ float red[4][RP];
    __shared__ float part[kGsGridMaxWgs * RP];
    __shared__ float tot_l[RP + 1];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t k0 = (int64_t)blockIdx.x * rows_per_wg;
    const int mine = (int)(rows - k0 < rows_per_wg ? rows - k0 : rows_per_wg);
    const int nrt = (mine + kGsRegThreads - 1) / kGsRegThreads;
    float v[RPT][RP];
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int k = threadIdx.x + t * kGsRegThreads;
#pragma unroll
        for (int c = 0; c < RP; ++c) v[t][c] = 0.f;
        if (t < nrt && k < mine) {
            const float* row = a + (k0 + k) * r;
            if (RP >= 4 && r == RP) {
#pragma unroll
                for (int c = 0; c < RP; c += 4) ld4(row + c, &v[t][c]);
            } else {
#pragma unroll
                for (int c = 0; c < RP; ++c)
                    if (c < r) v[t][c] = row[c];
            }
        }
    }
    gs_grid_steps<RP, RPT, 0>(v, red, part, tot_l, ws, r, nrt, eps, wave, lane);
    if (tot_l[RP] == 0.f) {
        // a wait ran out: a half-orthogonalised matrix would pass for a result, NaN cannot
#pragma unroll
        for (int t = 0; t < RPT; ++t)
#pragma unroll
            for (int c = 0; c < RP; ++c) v[t][c] = __builtin_nanf("");
    }
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int k = threadIdx.x + t * kGsRegThreads;
        if (t < nrt && k < mine) {
            float* row = a + (k0 + k) * r;
            if (RP >= 4 && r == RP) {
#pragma unroll
                for (int c = 0; c < RP; c += 4) st4(row + c, &v[t][c]);
            } else {
#pragma unroll
                for (int c = 0; c < RP; ++c)
                    if (c < r) row[c] = v[t][c];
            }
        }
    }
}

// Large matrices: r+1 launches over all CUs.  Launch i first finishes column i-1 on its own rows
// (normalise it, take its projection off the later columns) from the sums launch i-1 left, then
// sums column i against the later columns over its rows and leaves one partial per workgroup.
// Every workgroup adds the partials in the same order, so all of them see the same sums.
template <int RP>
__global__ void __launch_bounds__(256)
gram_schmidt_step_kernel(float* __restrict__ a, int64_t rows, int r, float eps, int i, const float* __restrict__ sums_in,
                         float* __restrict__ sums_out, int rows_per_wg)
{
    __shared__ float red[4][RP];
    __shared__ float tot[RP];
    __shared__ float part[256];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float coef[RP];
    float den = 1.f;
    if (i > 0) {
        // the workgroups' partial sums of the previous launch: 256 / RP threads per column take
        // every (256 / RP)-th workgroup, then one thread per column adds their sums in order
        {
            constexpr int G = 256 / RP;
            const int c = threadIdx.x % RP, g0 = threadIdx.x / RP;
            float s = 0.f;
            int g = g0;
            for (; g + 3 * G < (int)gridDim.x; g += 4 * G) {
                float v0 = sums_in[g * RP + c], v1 = sums_in[(g + G) * RP + c];
                float v2 = sums_in[(g + 2 * G) * RP + c], v3 = sums_in[(g + 3 * G) * RP + c];
                s += v0; s += v1; s += v2; s += v3;
            }
            for (; g < (int)gridDim.x; g += G) s += sums_in[g * RP + c];
            part[threadIdx.x] = s;
        }
        __syncthreads();
        if (threadIdx.x < RP) {
            constexpr int G = 256 / RP;
            float s = 0.f;
            for (int g = 0; g < G; ++g) s += part[g * RP + threadIdx.x];
            tot[threadIdx.x] = s;
        }
        __syncthreads();
        float nrm = sqrtf(tot[0]);
        den = eps == 0.f ? nrm : nrm + eps;
#pragma unroll
        for (int c = 1; c < RP; ++c) coef[c] = (i - 1 + c < r) ? tot[c] / den : 0.f;
    }
    float acc[RP];
#pragma unroll
    for (int c = 0; c < RP; ++c) acc[c] = 0.f;
    const int64_t k0 = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t k1 = k0 + rows_per_wg < rows ? k0 + rows_per_wg : rows;
    for (int64_t k = k0 + threadIdx.x; k < k1; k += 256) {
        float* row = a + k * r;
        float cur[RP];                  // columns i.. of this row after column i-1 has been dealt with
#pragma unroll
        for (int c = 0; c < RP; ++c) cur[c] = 0.f;
        if (i > 0) {
            float ci = row[i - 1] / den;
            row[i - 1] = ci;
#pragma unroll
            for (int c = 1; c < RP; ++c)
                if (i - 1 + c < r) {
                    float v = __fsub_rn(row[i - 1 + c], __fmul_rn(coef[c], ci));
                    row[i - 1 + c] = v;
                    cur[c - 1] = v;
                }
        } else {
#pragma unroll
            for (int c = 0; c < RP; ++c)
                if (c < r) cur[c] = row[c];
        }
        if (i < r) {
#pragma unroll
            for (int c = 0; c < RP; ++c)
                if (i + c < r) acc[c] = fmaf(cur[0], cur[c], acc[c]);
        }
    }
    if (i >= r) return;
#pragma unroll
    for (int c = 0; c < RP; ++c) {
        float s = conef_wave_sum(acc[c]);
        if (lane == 0) red[wave][c] = s;
    }
    __syncthreads();
    if (threadIdx.x < RP)
        sums_out[blockIdx.x * RP + threadIdx.x] =
            (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

constexpr int kGsMaxWorkgroups = 256;

// ---------------------------------------------------------------- dispatch ----
inline int rank_bound(int r) { return r <= 1 ? 1 : r <= 2 ? 2 : r <= 4 ? 4 : r <= 8 ? 8 : r <= 16 ? 16 : 32; }

#define CONEF_RANK_SWITCH(r, CALL)      \
    switch (rank_bound(r)) {            \
        case 1: CALL(1); break;         \
        case 2: CALL(2); break;         \
        case 4: CALL(4); break;         \
        case 8: CALL(8); break;         \
        case 16: CALL(16); break;       \
        default: CALL(32); break;       \
    }

// Column splits of the MFMA P = X Q kernel: enough workgroups for the machine, each at least 128
// columns wide; the partial tiles of a row tile are added in split order by a second kernel.
struct MfmaMqShape {
    int row_tiles, splits, cols_per_split;
};

inline MfmaMqShape mfma_mq_shape(int64_t n, int64_t m)
{
    MfmaMqShape g;
    g.row_tiles = (int)((n + 31) / 32);
    int64_t want = (512 + g.row_tiles - 1) / g.row_tiles;
    int64_t most = (m + 127) / 128;
    int64_t splits = want < most ? want : most;
    if (splits > 64) splits = 64;
    if (splits < 1) splits = 1;
    int64_t cps = ((m + splits - 1) / splits + 127) / 128 * 128;
    g.cols_per_split = (int)cps;
    g.splits = (int)((m + cps - 1) / cps);
    return g;
}

constexpr size_t kMfmaMqLdsLimit = 144 * 1024;

// Launches of the streaming P = X Q kernel over `table` (ranks below 16, shapes that allow 16-byte
// accesses), kPsgdBatchMax matrices a launch.  kMqsNoFit, with nothing launched: a sketch row too
// wide for LDS, or too little work for this kernel; the caller then takes the row-block kernel.
constexpr int kMqsNoFit = -100;

template <int MODE>
int mqs_run(const std::vector<MqsItem>& table, int rp, float alpha, ConefSeeds hs, hipStream_t s, bool gram = false)
{
    struct Chunk { size_t k; int nb, T, S; size_t lds; };
    std::vector<Chunk> chunks;
    for (size_t k = 0; k < table.size();) {
        Chunk c;
        c.k = k;
        c.nb = (int)std::min(table.size() - k, (size_t)kPsgdBatchMax);
        if (!mqs_plan_launch(&table[k], c.nb, rp, MODE == 2, &c.T, &c.S, &c.lds, gram)) return kMqsNoFit;
        chunks.push_back(c);
        k += (size_t)c.nb;
    }
    for (const Chunk& c : chunks) {
        PsgdBatch<MqsItem> b;
        int total = 0;
        for (int i = 0; i < c.nb; ++i) {
            MqsItem it = table[c.k + (size_t)i];
            it.gw = mqs_group_width(it.m, c.T);
            it.S = c.S;
            b.item[i] = it;
            b.first[i] = total;
            total += (int)mqs_workgroups(it.n, it.gw, c.S, c.T);
        }
        b.first[c.nb] = total;
        b.count = c.nb;
#define CONEF_MQS(RP)                                                                                               \
    do {                                                                                                            \
        if (RP >= 16) break;                                                                                        \
        if (c.T == 256)                                                                                             \
            hipLaunchKernelGGL((psgd_mqs_batch_kernel<(RP < 16 ? RP : 8), MODE, 256>), dim3((unsigned)total), dim3(256),  \
                               c.lds, s, b, alpha, hs);                                                             \
        else                                                                                                        \
            hipLaunchKernelGGL((psgd_mqs_batch_kernel<(RP < 16 ? RP : 8), MODE, 1024>), dim3((unsigned)total), dim3(1024), \
                               c.lds, s, b, alpha, hs);                                                             \
    } while (0)
        CONEF_RANK_SWITCH(rp, CONEF_MQS)
#undef CONEF_MQS
    }
    return (int)hipGetLastError();
}

template <int MODE>
int launch_mq(float* x, const float* err, const float* cs, const uint32_t* pktab, const float* q, float* p, int64_t n,
              int64_t m, int r, int32_t w, float alpha, ConefSeeds hs, void* workspace, int64_t workspace_bytes,
              hipStream_t s)
{
    ConefMod mod = conef_make_mod(w > 0 ? w : 1);
    if (rank_bound(r) >= 16 && m % 4 == 0 && aligned16(x) && (MODE != 1 || aligned16(err)) &&
        (!pktab || aligned16(pktab))) {
        size_t lds = (size_t)kMfmaWaves * 16 * 64 * 4 + (MODE == 2 ? (size_t)32 * w * 4 : 0);
        if (MODE == 2 && (mfma_mq_shape(n, m).splits > 1 || lds > kMfmaMqLdsLimit)) {
            // Parking 32 sketch rows per workgroup costs more than the tile's share of M once the
            // matrix is split over columns: unsketch in a launch of its own, then the plain product.
            int rc = conef_cs_query_f32(x, cs, n, m, w, alpha, hs.a, hs.b, (void*)s);
            if (rc != CONEF_OK) return rc;
            return launch_mq<0>(x, nullptr, nullptr, nullptr, q, p, n, m, r, 1, 0.f, hs, workspace, workspace_bytes, s);
        }
        if (lds <= kMfmaMqLdsLimit) {
            MfmaMqShape g = mfma_mq_shape(n, m);
            if (g.splits > 1 && (!workspace || workspace_bytes < (int64_t)g.splits * n * r * 4)) {
                g.splits = 1;
                g.cols_per_split = (int)((m + 127) / 128 * 128);
            }
            float* out = g.splits > 1 ? (float*)workspace : p;
            auto k = psgd_mfma_mq_kernel<MODE>;
            if (hipError_t e = conef_allow_lds((const void*)k, lds); e != hipSuccess) return (int)e;
            hipLaunchKernelGGL(k, dim3((unsigned)g.row_tiles, (unsigned)g.splits), dim3(kMfmaThreads), lds, s, x, err, cs,
                               pktab, q, out, n, (int)m, r, g.cols_per_split, mod, alpha, hs);
            if (g.splits > 1) {
                int64_t count = n * r;
                hipLaunchKernelGGL(psgd_sum_partials_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, out,
                                   p, count, g.splits);
            }
            return (int)hipGetLastError();
        }
    }
    const bool fast = r == rank_bound(r) && m % 4 == 0 && aligned16(x) && aligned16(q) && (MODE != 1 || aligned16(err)) &&
                      (!pktab || aligned16(pktab));
    const int rp = rank_bound(r);
    if (fast && rp < 16) {
        std::vector<MqsItem> one(1);
        one[0] = MqsItem{x, err, cs, pktab, q, p, n, (int)m, (int)(MODE == 2 ? w : 1), 0, 0, mod};
        const int rc = mqs_run<MODE>(one, rp, alpha, hs, s);
        if (rc != kMqsNoFit) return rc;
    }
    // rows per workgroup: 4 amortises the Q traffic, but small matrices need the workgroups
    int rb = rp >= 32 ? 2 : 4;
    if (n / rb < 256) rb = rp >= 32 ? 2 : 1;
    size_t lds = (size_t)4 * rb * rp * 4 + (MODE == 2 ? (size_t)rb * w * 4 : 0);
    if (lds > 64 * 1024) return CONEF_ERR_INVALID;   // sketch rows wider than 16K cells per matrix row group
    dim3 grid((unsigned)((n + rb - 1) / rb));
#define CONEF_MQ_GO(RB, RP, F)                                                                                    \
    hipLaunchKernelGGL((psgd_mq_kernel<RB, RP, MODE, F>), grid, dim3(256), lds, s, x, err, cs, pktab, q, p, n, (int)m, \
                       r, mod, alpha, hs)
#define CONEF_MQ(RP)                                     \
    do {                                                 \
        if (RP >= 32) {                                  \
            if (fast) CONEF_MQ_GO(2, RP, true);          \
            else CONEF_MQ_GO(2, RP, false);              \
        } else if (rb == 4) {                            \
            if (fast) CONEF_MQ_GO(4, RP, true);          \
            else CONEF_MQ_GO(4, RP, false);              \
        } else {                                         \
            if (fast) CONEF_MQ_GO(1, RP, true);          \
            else CONEF_MQ_GO(1, RP, false);              \
        }                                                \
    } while (0)
    CONEF_RANK_SWITCH(r, CONEF_MQ)
#undef CONEF_MQ
#undef CONEF_MQ_GO
    return (int)hipGetLastError();
}

struct MtpShape {
    int col_tiles, slabs, rows_per_slab;
};

// enough slabs for about 256 workgroups of 8 waves, each wave at least eight rows
inline MtpShape mtp_shape(int64_t n, int64_t m)
{
    MtpShape g;
    g.col_tiles = (int)((m + 255) / 256);
    int64_t slabs = (256 + g.col_tiles - 1) / g.col_tiles;
    int64_t rps = (n + slabs - 1) / slabs;
    rps = (rps + 8 * kMtpWaves - 1) / (8 * kMtpWaves) * (8 * kMtpWaves);
    g.rows_per_slab = (int)rps;
    g.slabs = (int)((n + rps - 1) / rps);
    return g;
}

// MFMA Q = X^T P: V floats per lane (column tile 32 V), row slabs whose partials cost at most a
// quarter of the matrix's own bytes.
struct MfmaMtpShape {
    int v, col_tiles, slabs, rows_per_slab;
};

// want_wgs: workgroups the matrix should bring (512 alone; its share of them inside a batch, where
// wider lanes then win: fewer, fuller workgroups per matrix)
inline MfmaMtpShape mfma_mtp_shape(int64_t n, int64_t m, int r, int vmax, int64_t want_wgs = 512)
{
    MfmaMtpShape g = {1, 0, 1, 0};
    int64_t slabs_most = n / (4 * (int64_t)r);
    if (slabs_most < 1) slabs_most = 1;
    if (slabs_most > (n + 7) / 8) slabs_most = (n + 7) / 8;
    for (int v = vmax; v >= 1; v >>= 1) {
        int64_t tiles = (m + 32 * v - 1) / (32 * v);
        int64_t want = (want_wgs + tiles - 1) / tiles;
        int64_t slabs = want < slabs_most ? want : slabs_most;
        g.v = v;
        g.col_tiles = (int)tiles;
        g.slabs = (int)slabs;
        if (tiles * slabs >= want_wgs || v == 1) break;
    }
    int64_t rps = ((n + g.slabs - 1) / g.slabs + 7) / 8 * 8;
    g.rows_per_slab = (int)rps;
    g.slabs = (int)((n + rps - 1) / rps);
    return g;
}

inline int64_t gs_sums_floats(int64_t rows, int r)
{
    int64_t steps = 2 * (int64_t)kGsMaxWorkgroups * rank_bound(r);
    int64_t grid = (int64_t)(sizeof(GsGridWs) + 3) / 4;
    int64_t lanes = (int64_t)(sizeof(GslWs) + 3) / 4;
    if (lanes > grid) grid = lanes;
    int64_t gramws = (int64_t)(sizeof(GsgWs) + 3) / 4;
    if (gramws > grid) grid = gramws;
    return steps > grid ? steps : grid;
}

inline bool gs_fits_lds(int64_t rows, int r)
{
    return (size_t)(rows * (r + 1) + 17 * rank_bound(r)) * 4 <= kGsLdsLimit;
}

// Row slots per thread the register kernel needs for a matrix: the smallest of 1, 4, 16, all that
// holds it (the unrolled code grows with the slots, and a small kernel is mostly instruction
// fetch); -1 when the matrix does not fit one workgroup's registers or its rows are not 16-byte
// aligned for the vector accesses.
inline int gs_reg_class(const float* a, int64_t rows, int r)
{
    const int rp = rank_bound(r);
    const int all = kGsRegFloats / rp;
    if (rows > (int64_t)kGsRegThreads * all) return -1;
    if (!(rp < 4 || r != rp || aligned16(a))) return -1;
    const int nrt = (int)((rows + kGsRegThreads - 1) / kGsRegThreads);
    if (nrt <= 1) return 1;
    if (nrt <= 4 && all >= 4) return 4;
    if (nrt <= 16 && all >= 16) return 16;
    return all;
}

// slots: the one class all matrices of the batch share, or 0 for a batch of mixed classes
inline int gs_launch_reg_batch(const GsBatch& batch, int count, int r, int slots, float eps, hipStream_t s)
{
    if (slots == 0) {
#define CONEF_GSM(RP) \
    hipLaunchKernelGGL((gram_schmidt_reg_mixed_kernel<RP>), dim3((unsigned)count), dim3(kGsRegThreads), 0, s, batch, r, eps)
        switch (rank_bound(r)) {
            case 1: CONEF_GSM(1); break;
            case 2: CONEF_GSM(2); break;
            case 4: CONEF_GSM(4); break;
            case 8: CONEF_GSM(8); break;
            default: return CONEF_ERR_INVALID;
        }
#undef CONEF_GSM
        return (int)hipGetLastError();
    }
#define CONEF_GSR_GO(RP, RPT) \
    hipLaunchKernelGGL((gram_schmidt_reg_kernel<RP, (RPT)>), dim3((unsigned)count), dim3(kGsRegThreads), 0, s, batch, r, eps)
#define CONEF_GSR(RP)                                                       \
    do {                                                                    \
        constexpr int kAll = kGsRegFloats / RP;                             \
        if (slots == 1) CONEF_GSR_GO(RP, 1);                                \
        else if (slots == 4 && kAll >= 4) CONEF_GSR_GO(RP, (kAll >= 4 ? 4 : kAll));      \
        else if (slots == 16 && kAll >= 16) CONEF_GSR_GO(RP, (kAll >= 16 ? 16 : kAll));  \
        else CONEF_GSR_GO(RP, kAll);                                        \
    } while (0)
    CONEF_RANK_SWITCH(r, CONEF_GSR)
#undef CONEF_GSR
#undef CONEF_GSR_GO
    return (int)hipGetLastError();
}

// Kernels of conef_gs_lanes.h: which one a matrix takes.  kind 0: none (rank not 8, 16 or 32, the
// matrix narrower than its rank bound, or larger than 128 workgroups hold); kind 1: one workgroup,
// a wave per two columns (rank 32 up to 2048 rows) or per column (rank 16 up to 1024 rows), rpt
// rows a lane; kind 2: wgs workgroups of the column-per-lane kernel, rpt rows a thread, launched
// cooperatively.  Other matrices that fit one workgroup's registers (32768 elements) stay with
// the row-per-thread kernel, which is faster there.
struct GslChoice {
    int kind, rpt, wgs;
};

inline GslChoice gsl_choose(int64_t rows, int r)
{
    GslChoice ch = {0, 0, 0};
    if (r != rank_bound(r) || r < 8) return ch;
    if ((r == 32 && rows <= 2048) || (r == 16 && rows <= 1024)) {
        ch.kind = 1;
        ch.rpt = rows <= 256 ? 4 : rows <= 512 ? 8 : rows <= 1024 ? 16 : 32;
        ch.wgs = 1;
        return ch;
    }
    const int64_t elements = rows * r;
    if (elements <= (int64_t)kGsRegThreads * kGsRegFloats) return ch;      // the row-per-thread kernel, one workgroup
    static const int kRpt[4] = {4, 8, 16, 64};
    for (int k = 0; k < (r == 8 ? 3 : 4); ++k) {
        const int64_t per = (int64_t)kGslThreads * kRpt[k];
        const int64_t wgs = (elements + per - 1) / per;
        if (wgs <= kGslMaxWgs) {
            ch.kind = 2;
            ch.rpt = kRpt[k];
            ch.wgs = (int)wgs;
            return ch;
        }
    }
    return ch;
}

template <int RP, int RPT, int CW>
inline hipError_t gsw_go(const GswBatch& batch, int count, float eps, hipStream_t s)
{
    constexpr int kLds = gsw_lds_floats<RP, RPT>() * 4;
    static const hipError_t attr =
        kLds > 48 * 1024 ? hipFuncSetAttribute((const void*)gsw_kernel<RP, RPT, CW>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLds)
                         : hipSuccess;
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL((gsw_kernel<RP, RPT, CW>), dim3((unsigned)count), dim3(64 * RP / CW), kLds, s, batch, eps);
    return hipGetLastError();
}

// kind 1: `count` matrices of rank r, all of class rpt, one workgroup each
inline int gsw_launch(const GswBatch& batch, int count, int r, int rpt, float eps, hipStream_t s)
{
    hipError_t e = hipErrorInvalidValue;
    if (r == 32) {
        e = rpt == 4 ? gsw_go<32, 4, 2>(batch, count, eps, s) : rpt == 8 ? gsw_go<32, 8, 2>(batch, count, eps, s)
          : rpt == 16 ? gsw_go<32, 16, 2>(batch, count, eps, s) : gsw_go<32, 32, 2>(batch, count, eps, s);
    } else if (r == 16) {
        e = rpt == 4 ? gsw_go<16, 4, 1>(batch, count, eps, s) : rpt == 8 ? gsw_go<16, 8, 1>(batch, count, eps, s)
                                                                          : gsw_go<16, 16, 1>(batch, count, eps, s);
    }
    if (e != hipSuccess) (void)hipGetLastError();
    return (int)e;
}

// kind 2: one batch of matrices of rank r and class rpt over wgs workgroups in all.  A cooperative
// launch the runtime refuses comes back as an error for the caller to take the other kernels.
inline int gsl_launch(const GslBatch& batch, int count, int r, int rpt, int wgs, float eps, void* workspace, hipStream_t s)
{
    GslWs* ws = (GslWs*)workspace;
    const void* fn = nullptr;
#define CONEF_GSL(RP)                                                                                     \
    fn = rpt == 4 ? (const void*)gsl_kernel<RP, 4> : rpt == 8 ? (const void*)gsl_kernel<RP, 8>            \
       : rpt == 16 ? (const void*)gsl_kernel<RP, 16> : (const void*)gsl_kernel<RP, 64>
    if (r == 32) CONEF_GSL(32);
    else if (r == 16) CONEF_GSL(16);
    else if (r == 8 && rpt <= 16) fn = rpt == 4 ? (const void*)gsl_kernel<8, 4> : rpt == 8 ? (const void*)gsl_kernel<8, 8>
                                                                                            : (const void*)gsl_kernel<8, 16>;
#undef CONEF_GSL
    if (!fn) return CONEF_ERR_INVALID;
    hipLaunchKernelGGL(gsl_reset_kernel, dim3(8), dim3(1024), 0, s, ws, wgs);
    void* args[] = {(void*)&batch, (void*)&count, (void*)&eps, (void*)&ws};
    hipError_t e = hipLaunchCooperativeKernel(fn, dim3((unsigned)wgs), dim3(kGslThreads), args, 0, s);
    if (e != hipSuccess) (void)hipGetLastError();
    return (int)e;
}

// Kernel of conef_gs_gram.h (one exchange between workgroups instead of one per column).  It can
// take any matrix that is exactly 8, 16 or 32 wide and 16-byte aligned (gsg_can); it is the better
// kernel (gsg_wants) at ranks 16 and 32 above 1024 rows and at rank 8 above the 4096 rows one
// workgroup's registers hold: a launch lasts 20 to 30 us whatever it holds, where the
// column-by-column kernels pay per step and per workgroup involved.  Shorter factors of rank 16 or
// 32 join a launch that a taller one of their bucket needs anyway (each on its own workgroups);
// short rank-8 factors stay with the row-per-thread kernel, which also orthogonalises them inside
// the last launch of a round.
inline bool gsg_can(const float* a, int64_t rows, int r)
{
    return (r == 8 || r == 16 || r == 32) && aligned16(a) && rows <= 0x7fffffffLL;
}

inline bool gsg_wants(const float* a, int64_t rows, int r)
{
    if (!gsg_can(a, rows, r)) return false;
    return r >= 16 ? rows > 1024 : rows * r > (int64_t)kGsRegThreads * kGsRegFloats;
}

std::atomic<unsigned> g_gsg_launches{0};
std::atomic<unsigned> g_small_launches{0};

// One launch over `count` matrices of rank r (workgroup ranges in batch.first).  A normal launch:
// at most 128 workgroups of 256 threads, which a GPU that is running anything else still holds
// side by side; the waits inside are bounded either way.
inline int gsg_launch(const GsgBatch& batch, int count, int r, int wgs, float eps, void* workspace, hipStream_t s)
{
    unsigned tag = (g_gsg_launches.fetch_add(1u) + 1u) * 0x9E3779B9u;
    if (tag == 0u) tag = 1u;
    GsgWs* ws = (GsgWs*)workspace;
    if (r == 32) hipLaunchKernelGGL(gsg_kernel<32>, dim3((unsigned)wgs), dim3(kGsgThreads), 0, s, batch, count, eps, ws, tag);
    else if (r == 16) hipLaunchKernelGGL(gsg_kernel<16>, dim3((unsigned)wgs), dim3(kGsgThreads), 0, s, batch, count, eps, ws, tag);
    else if (r == 8) hipLaunchKernelGGL(gsg_kernel<8>, dim3((unsigned)wgs), dim3(kGsgThreads), 0, s, batch, count, eps, ws, tag);
    else return CONEF_ERR_INVALID;
    return (int)hipGetLastError();
}

inline bool gsg_workspace_ok(const void* workspace, int64_t workspace_bytes)
{
    return workspace && workspace_bytes >= (int64_t)sizeof(GsgWs) && (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0;
}

inline bool psgd_args_ok(int64_t n, int64_t m, int32_t r)
{
    return n >= 1 && m >= 1 && r >= 1 && r <= kMaxRank && m <= 0x7fffffffLL && n <= 0x7fffffffLL;
}

}  // namespace

extern "C" {

int conef_psgd_mq_f32(float* x, const float* q, float* p, int64_t n, int64_t m, int32_t r, void* workspace,
                      int64_t workspace_bytes, void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !q || !p) return CONEF_ERR_INVALID;
    ConefSeeds hs = {0, 0, 0, 0};
    return launch_mq<0>(x, nullptr, nullptr, nullptr, q, p, n, m, r, 1, 0.f, hs, workspace, workspace_bytes,
                        (hipStream_t)stream);
}

int conef_psgd_mq_ef_f32(float* x, const float* err, const float* q, float* p, int64_t n, int64_t m, int32_t r,
                         void* workspace, int64_t workspace_bytes, void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !err || !q || !p) return CONEF_ERR_INVALID;
    ConefSeeds hs = {0, 0, 0, 0};
    return launch_mq<1>(x, err, nullptr, nullptr, q, p, n, m, r, 1, 0.f, hs, workspace, workspace_bytes,
                        (hipStream_t)stream);
}

int conef_psgd_mq_conef_f32(float* x, const float* cs, const float* q, float* p, int64_t n, int64_t m, int32_t r,
                            int32_t w, float alpha, int32_t a, int32_t b, void* workspace, int64_t workspace_bytes,
                            void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !cs || !q || !p || w < 1 || w > (1 << 30)) return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    return launch_mq<2>(x, nullptr, cs, nullptr, q, p, n, m, r, w, alpha, hs, workspace, workspace_bytes,
                        (hipStream_t)stream);
}

// The same with the (bucket, sign) of every column read from a plan's table instead of hashed.
int conef_psgd_mq_conef_planned_f32(float* x, const float* cs, const float* q, float* p, const void* plan_host,
                                    const void* plan_dev, int64_t n, int64_t m, int32_t r, int32_t w, float alpha,
                                    int32_t a, int32_t b, void* workspace, int64_t workspace_bytes, void* stream)
{
    const ConefPlanHeader* hp = (const ConefPlanHeader*)plan_host;
    if (!psgd_args_ok(n, m, r) || !x || !cs || !q || !p || !plan_dev || !conef_plan_matches(hp, n, m, w, a, b))
        return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    const uint32_t* pk = (const uint32_t*)((const char*)plan_dev + hp->off_pk);
    return launch_mq<2>(x, nullptr, cs, pk, q, p, n, m, r, w, alpha, hs, workspace, workspace_bytes, (hipStream_t)stream);
}

// Bytes of device workspace conef_psgd_mtp_f32 and conef_gram_schmidt_f32 may need for an [n,m]
// matrix at rank r (partial sums that meet across workgroups).
int64_t conef_psgd_workspace_bytes(int64_t n, int64_t m, int32_t r)
{
    if (!psgd_args_ok(n, m, r)) return -1;
    MtpShape g = mtp_shape(n, m);
    int64_t need = g.slabs > 1 ? (int64_t)g.slabs * m * r : 0;
    int64_t rows = n > m ? n : m;
    int64_t gs = gs_sums_floats(rows, r);
    if (gs > need) need = gs;
    if (rank_bound(r) >= 16) {
        for (int v = 4; v >= 1; v >>= 1) {      // which one runs depends on the alignment of the call's pointers
            MfmaMtpShape t = mfma_mtp_shape(n, m, r, v);
            int64_t b = t.slabs > 1 ? (int64_t)t.slabs * m * r : 0;
            if (b > need) need = b;
        }
        MfmaMqShape q = mfma_mq_shape(n, m);
        int64_t b = q.splits > 1 ? (int64_t)q.splits * n * r : 0;
        if (b > need) need = b;
    }
    return conef_align256(4 * need);
}

int conef_psgd_mtp_f32(const float* x, const float* p, float* q, int64_t n, int64_t m, int32_t r, void* workspace,
                       int64_t workspace_bytes, void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !q || !p) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    if (rank_bound(r) >= 16) {
        const uintptr_t xa = reinterpret_cast<uintptr_t>(x);
        int vmax = (m % 4 == 0 && (xa & 15u) == 0) ? 4 : (m % 2 == 0 && (xa & 7u) == 0) ? 2 : 1;
        MfmaMtpShape t = mfma_mtp_shape(n, m, r, vmax);
        float* dst = q;
        if (t.slabs > 1) {
            if (!workspace || workspace_bytes < (int64_t)t.slabs * m * r * 4) return CONEF_ERR_INVALID;
            dst = (float*)workspace;
        }
        dim3 grid((unsigned)t.col_tiles, (unsigned)t.slabs);
        if (t.v == 4) hipLaunchKernelGGL(psgd_mfma_mtp_kernel<4>, grid, dim3(kMfmaThreads), 0, s, x, p, dst, n, (int)m, r, t.rows_per_slab);
        else if (t.v == 2) hipLaunchKernelGGL(psgd_mfma_mtp_kernel<2>, grid, dim3(kMfmaThreads), 0, s, x, p, dst, n, (int)m, r, t.rows_per_slab);
        else hipLaunchKernelGGL(psgd_mfma_mtp_kernel<1>, grid, dim3(kMfmaThreads), 0, s, x, p, dst, n, (int)m, r, t.rows_per_slab);
        if (t.slabs > 1) {
            int64_t count = m * r;
            hipLaunchKernelGGL(psgd_sum_partials_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, dst, q,
                               count, t.slabs);
        }
        return (int)hipGetLastError();
    }
    MtpShape g = mtp_shape(n, m);
    float* out = q;
    if (g.slabs > 1) {
        if (!workspace || workspace_bytes < (int64_t)g.slabs * m * r * 4) return CONEF_ERR_INVALID;
        out = (float*)workspace;
    }
    const bool fast = r == rank_bound(r) && m % 4 == 0 && aligned16(x) && aligned16(p) && aligned16(out);
    dim3 grid((unsigned)g.col_tiles, (unsigned)g.slabs);
#define CONEF_MTP(RP)                                                                                            \
    do {                                                                                                         \
        if (fast) hipLaunchKernelGGL((psgd_mtp_kernel<RP, true>), grid, dim3(kMtpThreads), 0, s, x, p, out, n, (int)m, r, \
                                     g.rows_per_slab);                                                           \
        else hipLaunchKernelGGL((psgd_mtp_kernel<RP, false>), grid, dim3(kMtpThreads), 0, s, x, p, out, n, (int)m, r,     \
                                g.rows_per_slab);                                                                \
    } while (0)
    CONEF_RANK_SWITCH(r, CONEF_MTP)
#undef CONEF_MTP
    if (g.slabs > 1) {
        int64_t count = m * r;
        hipLaunchKernelGGL(psgd_sum_partials_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, out, q,
                           count, g.slabs);
    }
    return (int)hipGetLastError();
}

static int launch_pqt(float* x, float* err, const float* p, const float* q, int64_t n, int64_t m, int32_t r,
                      hipStream_t s)
{
    if ((r == 16 || r == 32) && aligned16(p) && aligned16(q)) {
        int64_t col_wgs = (m + 32 * kMfmaWaves - 1) / (32 * kMfmaWaves);
        int64_t slabs = (1024 + col_wgs - 1) / col_wgs;
        int64_t rps = ((n + slabs - 1) / slabs + 31) / 32 * 32;
        slabs = (n + rps - 1) / rps;
        if (slabs > 65535) {
            rps = ((n + 65534) / 65535 + 31) / 32 * 32;
            slabs = (n + rps - 1) / rps;
        }
        dim3 grid((unsigned)col_wgs, (unsigned)slabs);
        if (r == 32) {
            if (err) hipLaunchKernelGGL((psgd_mfma_pqt_kernel<32, 1>), grid, dim3(kMfmaThreads), 0, s, x, err, p, q, n, (int)m, (int)rps);
            else hipLaunchKernelGGL((psgd_mfma_pqt_kernel<32, 0>), grid, dim3(kMfmaThreads), 0, s, x, err, p, q, n, (int)m, (int)rps);
        } else {
            if (err) hipLaunchKernelGGL((psgd_mfma_pqt_kernel<16, 1>), grid, dim3(kMfmaThreads), 0, s, x, err, p, q, n, (int)m, (int)rps);
            else hipLaunchKernelGGL((psgd_mfma_pqt_kernel<16, 0>), grid, dim3(kMfmaThreads), 0, s, x, err, p, q, n, (int)m, (int)rps);
        }
        return (int)hipGetLastError();
    }
    const bool fast = r == rank_bound(r) && m % 4 == 0 && aligned16(x) && aligned16(q) && (!err || aligned16(err));
    int64_t col_tiles = (m + 1023) / 1024;
    int64_t slabs = (1024 + col_tiles - 1) / col_tiles;       // about a thousand workgroups ...
    int64_t rps = (n + slabs - 1) / slabs;
    if (rps < 4) rps = 4;                                     // ... of at least four rows
    slabs = (n + rps - 1) / rps;
    if (slabs > 65535) {
        rps = (n + 65534) / 65535;
        slabs = (n + rps - 1) / rps;
    }
    dim3 grid((unsigned)col_tiles, (unsigned)slabs);
#define CONEF_PQT_GO(RP, MODE, F) \
    hipLaunchKernelGGL((psgd_pqt_kernel<RP, MODE, F>), grid, dim3(256), 0, s, x, err, p, q, n, (int)m, r, (int)rps)
#define CONEF_PQT(RP)                                 \
    do {                                              \
        if (err) {                                    \
            if (fast) CONEF_PQT_GO(RP, 1, true);      \
            else CONEF_PQT_GO(RP, 1, false);          \
        } else {                                      \
            if (fast) CONEF_PQT_GO(RP, 0, true);      \
            else CONEF_PQT_GO(RP, 0, false);          \
        }                                             \
    } while (0)
    CONEF_RANK_SWITCH(r, CONEF_PQT)
#undef CONEF_PQT
#undef CONEF_PQT_GO
    return (int)hipGetLastError();
}

int conef_psgd_pqt_f32(float* x, const float* p, const float* q, int64_t n, int64_t m, int32_t r, void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !q || !p) return CONEF_ERR_INVALID;
    return launch_pqt(x, nullptr, p, q, n, m, r, (hipStream_t)stream);
}

int conef_psgd_pqt_ef_f32(float* x, float* err, const float* p, const float* q, int64_t n, int64_t m, int32_t r,
                          void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !err || !q || !p) return CONEF_ERR_INVALID;
    return launch_pqt(x, err, p, q, n, m, r, (hipStream_t)stream);
}

int conef_psgd_pqt_conef_f32(float* x, const float* p, const float* q, const float* cs_in, float* cs_out, int64_t n,
                             int64_t m, int32_t r, int32_t w, float beta, int32_t a, int32_t b, void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !q || !p || !cs_in || !cs_out || w < 1 || w > (1 << 30))
        return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    FrontPsgdResidual front = {x, p, q, m, r};
    return conef_launch_sketch_step<float>(front, cs_in, cs_out, n, m, w, beta, hs, (hipStream_t)stream, false);
}

// The same on a row-list plan: no atomics, bit-exact accumulation order, cs_out may be cs_in.
int conef_psgd_pqt_conef_planned_f32(float* x, const float* p, const float* q, const float* cs_in, float* cs_out,
                                     const void* plan_host, const void* plan_dev, int64_t n, int64_t m, int32_t r,
                                     int32_t w, float beta, int32_t a, int32_t b, void* stream)
{
    const ConefPlanHeader* hp = (const ConefPlanHeader*)plan_host;
    if (!psgd_args_ok(n, m, r) || !x || !q || !p || !cs_in || !cs_out || !plan_dev ||
        !conef_plan_matches(hp, n, m, w, a, b) || hp->kind != kConefPlanRowlist)
        return CONEF_ERR_INVALID;
    const bool fast = r == rank_bound(r) && m % 4 == 0 && aligned16(x) && aligned16(q) && aligned16(p);
    ConefRowlistView view = conef_rowlist_view(hp, plan_dev);
    hipStream_t s = (hipStream_t)stream;
    int rc = CONEF_ERR_INVALID;
#define CONEF_RES(RP)                                                                          \
    do {                                                                                       \
        if (fast) {                                                                            \
            ListPsgdResidual<RP, true> front = {x, p, q, r};                                   \
            rc = conef_launch_rowlist(front, view, cs_in, cs_out, n, m, w, beta, s);           \
        } else {                                                                               \
            ListPsgdResidual<RP, false> front = {x, p, q, r};                                  \
            rc = conef_launch_rowlist(front, view, cs_in, cs_out, n, m, w, beta, s);           \
        }                                                                                      \
    } while (0)
    CONEF_RANK_SWITCH(r, CONEF_RES)
#undef CONEF_RES
    return rc;
}

int conef_gram_schmidt_f32(float* a, int64_t rows, int32_t r, float eps, void* workspace, int64_t workspace_bytes,
                           void* stream)
{
    if (rows < 1 || rows > 0x7fffffffLL || r < 1 || r > kMaxRank || !a) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    const int rp = rank_bound(r);
    if (gsg_wants(a, rows, r)) {
        GsgBatch one;
        int slab, wgs;
        gsg_split(rows, r, &slab, &wgs);
        if (wgs == 1 || gsg_workspace_ok(workspace, workspace_bytes)) {
            one.a[0] = a;
            one.rows[0] = (int)rows;
            one.slab[0] = slab;
            one.first[0] = 0;
            one.first[1] = wgs;
            return gsg_launch(one, 1, r, wgs, eps, workspace, s);
        }
    }
    {
        const GslChoice ch = gsl_choose(rows, r);
        if (ch.kind == 1) {
            GswBatch one;
            one.a[0] = a;
            one.rows[0] = (int)rows;
            if (gsw_launch(one, 1, r, ch.rpt, eps, s) == CONEF_OK) return CONEF_OK;
        } else if (ch.kind == 2 && workspace && workspace_bytes >= (int64_t)sizeof(GslWs) &&
                   (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0) {
            GslBatch one;
            one.a[0] = a;
            one.elements[0] = rows * r;
            one.first[0] = 0;
            one.first[1] = ch.wgs;
            if (gsl_launch(one, 1, r, ch.rpt, ch.wgs, eps, workspace, s) == CONEF_OK) return CONEF_OK;
        }
    }
    if (gs_reg_class(a, rows, r) >= 0) {
        GsBatch one;
        one.a[0] = a;
        one.rows[0] = (int)rows;
        return gs_launch_reg_batch(one, 1, r, gs_reg_class(a, rows, r), eps, s);
    }
    if (gs_fits_lds(rows, r)) {
        size_t lds = (size_t)(rows * (r + 1) + 17 * rp) * 4;
        int threads = (int)((rows + 63) / 64 * 64);
        if (threads > 1024) threads = 1024;
#define CONEF_GS(RP)                                                                                              \
    do {                                                                                                          \
        auto k = gram_schmidt_lds_kernel<RP>;                                                                     \
        if (hipError_t e = conef_allow_lds((const void*)k, lds); e != hipSuccess) return (int)e; \
        hipLaunchKernelGGL(k, dim3(1), dim3(threads), lds, s, a, (int)rows, r, eps);                              \
    } while (0)
        CONEF_RANK_SWITCH(r, CONEF_GS)
#undef CONEF_GS
        return (int)hipGetLastError();
    }
    if (!workspace || workspace_bytes < gs_sums_floats(rows, r) * 4) return CONEF_ERR_INVALID;
    {
        // cooperative register-resident kernel.  A step costs a trip through the barrier whatever
        // the arithmetic, and the barrier grows with the workgroups: as many row slots per thread
        // as the registers hold (4 at rank 32, 16 below rank 16), hence few workgroups
        const int slots = rp >= 32 ? 4 : rp >= 16 ? 4 : 16;
        const bool vec_ok = rp < 4 || r != rp || aligned16(a);
        if (vec_ok && rows <= (int64_t)kGsGridMaxWgs * kGsRegThreads * slots &&
            (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0) {
            int64_t per = (int64_t)kGsRegThreads * slots;
            int64_t wgs = (rows + per - 1) / per;
            // fewer, fuller workgroups do not help: the step is bound by the barrier, not by arithmetic
            int rows_per_wg = (int)((rows + wgs - 1) / wgs);
            GsGridWs* gws = (GsGridWs*)workspace;
            hipLaunchKernelGGL(gs_grid_reset_kernel, dim3(1), dim3(1), 0, s, gws);
            void* args[] = {(void*)&a, (void*)&rows, (void*)&r, (void*)&eps, (void*)&rows_per_wg, (void*)&gws};
            hipError_t e = hipErrorInvalidValue;
#define CONEF_GSG(RP)                                                                                                 \
    do {                                                                                                              \
        constexpr int kSlots = RP >= 16 ? 4 : 16;                                                                     \
        e = hipLaunchCooperativeKernel((const void*)gram_schmidt_grid_kernel<RP, kSlots>, dim3((unsigned)wgs),        \
                                       dim3(kGsRegThreads), args, 0, s);                                              \
    } while (0)
            CONEF_RANK_SWITCH(r, CONEF_GSG)
#undef CONEF_GSG
            if (e == hipSuccess) return (int)hipGetLastError();
            (void)hipGetLastError();       // cooperative launch refused: fall through to the multi-launch path
        }
    }
    // a thread walks whole rows (r strided floats), so the launch is bound by the number of CUs
    // it reaches rather than by threads: 64 rows per workgroup until the workgroup cap
    int64_t wgs = (rows + 63) / 64;
    if (wgs > kGsMaxWorkgroups) wgs = kGsMaxWorkgroups;
    int rows_per_wg = (int)((rows + wgs - 1) / wgs);
    wgs = (rows + rows_per_wg - 1) / rows_per_wg;
    float* sums = (float*)workspace;
    for (int i = 0; i <= r; ++i) {
        const float* in = sums + ((i + 1) & 1) * (int64_t)kGsMaxWorkgroups * rp;
        float* out = sums + (i & 1) * (int64_t)kGsMaxWorkgroups * rp;
#define CONEF_GSS(RP) \
    hipLaunchKernelGGL(gram_schmidt_step_kernel<RP>, dim3((unsigned)wgs), dim3(256), 0, s, a, rows, r, eps, i, in, out, rows_per_wg)
        CONEF_RANK_SWITCH(r, CONEF_GSS)
#undef CONEF_GSS
    }
    return (int)hipGetLastError();
}

// Diagnostic: how many Gram-Schmidt workgroups on the current device have run out their bounded wait
// for another workgroup (and left NaN in their rows) since the library was loaded.  Waits for the
// device, then reads the library's per-GPU counter.
int conef_gram_schmidt_give_ups(int64_t* count)
{
    if (!count) return CONEF_ERR_INVALID;
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    unsigned long long v = 0;
    e = hipMemcpyFromSymbol(&v, HIP_SYMBOL(g_gs_give_ups), sizeof(v), 0, hipMemcpyDeviceToHost);
    if (e != hipSuccess) return (int)e;
    *count = (int64_t)v;
    return CONEF_OK;
}

// Gram-Schmidt of `count` independent matrices (matrix k: mats[k], [rows[k], ranks[k]] row-major,
// in place).  Matrices of equal rank that fit one workgroup's registers share launches, one
// workgroup each; the others go through conef_gram_schmidt_f32 one by one.  mats / rows / ranks
// are host arrays, read before the call returns.
int conef_gram_schmidt_batch_f32(float* const* mats, const int64_t* rows, const int32_t* ranks, int32_t count, float eps,
                                 void* workspace, int64_t workspace_bytes, void* stream)
{
    if (count < 0 || (count > 0 && (!mats || !rows || !ranks))) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    std::vector<char> done((size_t)count, 0);
    for (int k = 0; k < count; ++k) {
        if (rows[k] < 1 || rows[k] > 0x7fffffffLL || ranks[k] < 1 || ranks[k] > kMaxRank || !mats[k]) return CONEF_ERR_INVALID;
    }
    // kernel of conef_gs_gram.h: matrices of one rank share launches, each on its own workgroups
    const bool gram_ws_ok = gsg_workspace_ok(workspace, workspace_bytes);
    for (int k = 0; k < count; ++k) {
        if (done[(size_t)k] || !gsg_wants(mats[k], rows[k], ranks[k])) continue;
        GsgBatch batch;
        std::vector<int> members;
        int nb = 0, wgs = 0;
        // the matrices that want this kernel first, then (ranks 16 and 32) the bucket's shorter ones as guests
        for (int pass = 0; pass < 2; ++pass) {
            for (int j = 0; j < count && nb < kGsgMaxItems; ++j) {
                if (done[(size_t)j] || ranks[j] != ranks[k] || !gsg_can(mats[j], rows[j], ranks[j])) continue;
                const bool wants = gsg_wants(mats[j], rows[j], ranks[j]);
                if (pass == 0 ? !wants : (wants || ranks[j] < 16)) continue;
                if (std::find(members.begin(), members.end(), j) != members.end()) continue;
                int slab, w;
                gsg_split(rows[j], ranks[j], &slab, &w);
                if (w > 1 && !gram_ws_ok) continue;
                if (wgs + w > kGsgMaxWgs) continue;
                batch.a[nb] = mats[j];
                batch.rows[nb] = (int)rows[j];
                batch.slab[nb] = slab;
                batch.first[nb] = wgs;
                wgs += w;
                ++nb;
                members.push_back(j);
            }
        }
        if (nb == 0) continue;
        batch.first[nb] = wgs;
        const int rc = gsg_launch(batch, nb, ranks[k], wgs, eps, workspace, s);
        if (rc != CONEF_OK) return rc;
        for (int j : members) done[(size_t)j] = 1;
    }
    // kernels of conef_gs_lanes.h: matrices of one rank and class share launches (up to 48 matrices
    // of the one-workgroup kernel; up to 24 matrices and 128 workgroups of the other)
    const bool ws_ok = workspace && workspace_bytes >= (int64_t)sizeof(GslWs) && (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0;
    // Two rounds: first the launches of the several-workgroup kernel, then what is left for the
    // one-workgroup kernel.  A launch of the former lasts about r exchanges whatever it holds, so
    // it also takes the bucket's shorter factors of the same rank while it has workgroups to
    // spare, each on its own group of workgroups: they are then no launch of their own.
    for (int round = 2; round >= 1; --round) {
        for (int k = 0; k < count; ++k) {
            if (done[(size_t)k]) continue;
            const GslChoice ck = gsl_choose(rows[k], ranks[k]);
            if (ck.kind != round || (ck.kind == 2 && !ws_ok)) continue;
            GslBatch grid;
            GswBatch single;
            std::vector<int> members;
            int nb = 0, wgs = 0;
            const int cap = ck.kind == 1 ? kGswBatchMax : kGslMaxItems;
            for (int j = ck.kind == 2 ? 0 : k; j < count && nb < cap; ++j) {      // guests may come before the lead
                if (done[(size_t)j] || ranks[j] != ranks[k]) continue;
                GslChoice cj = gsl_choose(rows[j], ranks[j]);
                if (ck.kind == 2 && cj.kind == 1) {       // a shorter factor as a guest of this launch
                    const int64_t per = (int64_t)kGslThreads * ck.rpt;
                    cj.kind = 2;
                    cj.rpt = ck.rpt;
                    cj.wgs = (int)((rows[j] * ranks[j] + per - 1) / per);
                }
                if (cj.kind != ck.kind || cj.rpt != ck.rpt) continue;
                if (ck.kind == 2 && wgs + cj.wgs > kGslMaxWgs) continue;
                if (ck.kind == 1) {
                    single.a[nb] = mats[j];
                    single.rows[nb] = (int)rows[j];
                } else {
                    grid.a[nb] = mats[j];
                    grid.elements[nb] = rows[j] * ranks[j];
                    grid.first[nb] = wgs;
                }
                wgs += cj.wgs;
                ++nb;
                members.push_back(j);
            }
            if (ck.kind == 2) grid.first[nb] = wgs;
            const int rc = ck.kind == 1 ? gsw_launch(single, nb, ranks[k], ck.rpt, eps, s)
                                        : gsl_launch(grid, nb, ranks[k], ck.rpt, wgs, eps, workspace, s);
            if (rc != CONEF_OK) break;      // the other kernels below take what is left
            for (int j : members) done[(size_t)j] = 1;
        }
    }
    for (int k = 0; k < count; ++k) {
        if (done[(size_t)k]) continue;
        const int cls = gs_reg_class(mats[k], rows[k], ranks[k]);
        if (cls < 0) {
            int rc = conef_gram_schmidt_f32(mats[k], rows[k], ranks[k], eps, workspace, workspace_bytes, stream);
            if (rc != CONEF_OK) return rc;
            done[(size_t)k] = 1;
            continue;
        }
        // all matrices of this rank that fit one workgroup's registers, whatever their height
        GsBatch batch;
        int nb = 0;
        bool mixed = false;
        const bool mix_ok = rank_bound(ranks[k]) <= 8;     // above that the unrolled bodies are too large to pair up
        for (int j = k; j < count && nb < kGsBatchMax; ++j) {
            if (done[(size_t)j] || ranks[j] != ranks[k]) continue;
            const int cj = gs_reg_class(mats[j], rows[j], ranks[j]);
            if (cj < 0 || (cj != cls && !mix_ok)) continue;
            mixed = mixed || cj != cls;
            batch.a[nb] = mats[j];
            batch.rows[nb] = (int)rows[j];
            ++nb;
            done[(size_t)j] = 1;
        }
        int rc = gs_launch_reg_batch(batch, nb, ranks[k], mixed ? 0 : cls, eps, s);
        if (rc != CONEF_OK) return rc;
    }
    return CONEF_OK;
}

}  // extern "C"

// ------------------------------------------------------------ batch dispatch ----
namespace {

// Launches `table` (workgroup counts in `blocks`) in runs of kPsgdBatchMax with `go(batch, grid)`.
template <typename Item, typename Go>
int run_batches(const std::vector<Item>& table, const std::vector<int>& blocks, Go go)
{
    size_t k = 0;
    while (k < table.size()) {
        PsgdBatch<Item> b;
        int nb = 0, total = 0;
        while (k < table.size() && nb < kPsgdBatchMax) {
            b.item[nb] = table[k];
            b.first[nb] = total;
            total += blocks[k];
            ++nb;
            ++k;
        }
        b.first[nb] = total;
        b.count = nb;
        if (total > 0) go(b, total);
    }
    return (int)hipGetLastError();
}

inline bool item_ok(const ConefPsgdItem& it)
{
    return psgd_args_ok(it.n, it.m, it.r) && it.x && it.p && it.q;
}

inline const uint32_t* item_pktab(const ConefPsgdItem& it)
{
    const ConefPlanHeader* hp = (const ConefPlanHeader*)it.plan_host;
    return (hp && it.plan_dev) ? (const uint32_t*)((const char*)it.plan_dev + hp->off_pk) : nullptr;
}

// Matrix-core items of a batch run side by side, so each needs its own region for the partial
// tiles of its column splits (P = X Q) and row slabs (Q = X^T P); the two are never alive at once.
// offs[k]: where item k's region starts, in floats, -1 for ranks below 16.
inline int64_t mfma_batch_layout(const ConefPsgdItem* items, int count, std::vector<int64_t>* offs)
{
    int64_t off = 0;
    for (int k = 0; k < count; ++k) {
        int64_t at = -1;
        if (rank_bound(items[k].r) >= 16) {
            const int64_t n = items[k].n, m = items[k].m;
            const int r = items[k].r;
            MfmaMqShape q = mfma_mq_shape(n, m);
            int64_t need = q.splits > 1 ? (int64_t)q.splits * n * r : 0;
            // The slabs of Q = X^T P depend on how many workgroups the matrix is asked to bring, which
            // depends on what else is in the launch (a wider lane with more slabs can win there): room
            // for the most the shape function ever takes.
            int64_t slabs_most = n / (4 * (int64_t)r);
            if (slabs_most < 1) slabs_most = 1;
            if (slabs_most > (n + 7) / 8) slabs_most = (n + 7) / 8;
            if (slabs_most > 1 && slabs_most * m * r > need) need = slabs_most * m * r;
            at = off;
            off += (need + 63) / 64 * 64;
        }
        if (offs) offs->push_back(at);
    }
    return off;
}

// bytes at the front of a batch workspace that matrix-core items launched one by one share
inline int64_t batch_single_bytes(const ConefPsgdItem* items, int count)
{
    int64_t single = 0;
    for (int k = 0; k < count; ++k)
        if (rank_bound(items[k].r) >= 16) {
            int64_t b = conef_psgd_workspace_bytes(items[k].n, items[k].m, items[k].r);
            if (b > single) single = b;
        }
    return single;
}

struct MtpPlan;
inline int64_t mtp_batch_layout(const ConefPsgdItem* items, int count, std::vector<MtpPlan>* plans);

// where the matrix-core partial regions start inside a batch workspace; nullptr when it is too small
inline float* mfma_partial_base(const ConefPsgdItem* items, int count, void* workspace, int64_t workspace_bytes,
                                std::vector<int64_t>* offs)
{
    const int64_t floats = mfma_batch_layout(items, count, offs);
    const int64_t front = batch_single_bytes(items, count) + conef_align256(4 * mtp_batch_layout(items, count, nullptr));
    if (floats > 0 && (!workspace || workspace_bytes < front + 4 * floats)) return nullptr;
    return (float*)((char*)workspace + front);
}

inline int rows_per_query_block(int64_t n, int64_t col_blocks)
{
    int64_t rpb = (n * col_blocks + 1023) / 1024;       // about a thousand workgroups a matrix, eight rows at least
    if (rpb < 8) rpb = 8;
    if (rpb > n) rpb = n;
    return (int)(rpb < 1 ? 1 : rpb);
}

// rows per workgroup of the streaming P = X Q kernel inside a batch: four amortise the Q traffic
// once the batch as a whole has workgroups to spare
inline int mq_rows_per_wg(int64_t total_rows) { return total_rows / 4 >= 256 ? 4 : 1; }

template <int MODE>
int mq_batch(const ConefPsgdItem* items, int count, float alpha, int32_t a, int32_t b, void* workspace,
             int64_t workspace_bytes, hipStream_t s)
{
    ConefSeeds hs = {a, b, a + 2, b + 3};
    std::vector<char> done((size_t)count, 0);
    for (int k = 0; k < count; ++k) {
        if (done[(size_t)k]) continue;
        const ConefPsgdItem& lead = items[k];
        const int rp = rank_bound(lead.r);
        auto fast_of = [&](const ConefPsgdItem& it) {
            return it.r == rank_bound(it.r) && it.m % 4 == 0 && aligned16(it.x) && aligned16(it.q) &&
                   (MODE != 1 || aligned16(it.err)) && (MODE != 2 || !item_pktab(it) || aligned16(item_pktab(it)));
        };
        const bool fast = fast_of(lead);
        // ranks on the matrix cores, and sketch rows too wide for LDS, go one by one
        auto alone = [&](const ConefPsgdItem& it) {
            return rank_bound(it.r) >= 16 || (MODE == 2 && (size_t)4 * it.w * 4 + 4 * 4 * 8 * 4 > 64 * 1024);
        };
        // ranks on the matrix cores whose shapes allow the 16-byte paths share launches: the sketch
        // query first when there is one, then the plain (or error-adding) product, then the sums
        // of the column splits
        auto mfma_ok = [&](const ConefPsgdItem& it) {
            return rank_bound(it.r) >= 16 && it.m % 4 == 0 && aligned16(it.x) && (MODE != 1 || aligned16(it.err)) &&
                   (MODE != 2 || !item_pktab(it) || aligned16(item_pktab(it)));
        };
        if (mfma_ok(lead)) {
            std::vector<int64_t> offs;
            float* partials = mfma_partial_base(items, count, workspace, workspace_bytes, &offs);
            std::vector<QueryItem> queries;
            std::vector<MfmaMqItem> table;
            std::vector<SumItem> sums;
            std::vector<int> qblocks, blocks, sum_blocks;
            for (int j = k; j < count; ++j) {
                if (done[(size_t)j] || !mfma_ok(items[j])) continue;
                const ConefPsgdItem& it = items[j];
                MfmaMqShape g = mfma_mq_shape(it.n, it.m);
                if (g.splits > 1 && !partials) {
                    g.splits = 1;
                    g.cols_per_split = (int)((it.m + 127) / 128 * 128);
                }
                float* out = g.splits > 1 ? partials + offs[(size_t)j] : it.p;
                if (MODE == 2) {
                    const int64_t col_blocks = (it.m + 1023) / 1024;
                    const int rpb = rows_per_query_block(it.n, col_blocks);
                    QueryItem qi = {it.x, it.cs, item_pktab(it), it.n, (int)it.m, rpb, (int)col_blocks, conef_make_mod(it.w)};
                    queries.push_back(qi);
                    qblocks.push_back((int)(col_blocks * ((it.n + rpb - 1) / rpb)));
                }
                MfmaMqItem t = {it.x, MODE == 1 ? it.err : nullptr, it.q, out, it.n, (int)it.m, it.r, g.cols_per_split,
                                g.row_tiles, conef_make_mod(1)};
                table.push_back(t);
                blocks.push_back(g.row_tiles * g.splits);
                if (g.splits > 1) {
                    const int64_t cnt = it.n * it.r;
                    SumItem si = {out, it.p, cnt, g.splits};
                    sums.push_back(si);
                    sum_blocks.push_back((int)((cnt + 255) / 256));
                }
                done[(size_t)j] = 1;
            }
            int rc = CONEF_OK;
            if (MODE == 2)
                rc = run_batches(queries, qblocks, [&](const PsgdBatch<QueryItem>& bt, int grid) {
                    hipLaunchKernelGGL(psgd_cs_query_batch_kernel<true>, dim3((unsigned)grid), dim3(256), 0, s, bt, alpha, hs);
                });
            if (rc != CONEF_OK) return rc;
            const size_t lds = (size_t)kMfmaWaves * 16 * 64 * 4;
            rc = run_batches(table, blocks, [&](const PsgdBatch<MfmaMqItem>& bt, int grid) {
                hipLaunchKernelGGL((psgd_mfma_mq_batch_kernel<(MODE == 1 ? 1 : 0)>), dim3((unsigned)grid), dim3(kMfmaThreads),
                                   lds, s, bt);
            });
            if (rc != CONEF_OK) return rc;
            if (!sums.empty()) {
                rc = run_batches(sums, sum_blocks, [&](const PsgdBatch<SumItem>& bt, int grid) {
                    hipLaunchKernelGGL(psgd_sum_partials_batch_kernel, dim3((unsigned)grid), dim3(256), 0, s, bt);
                });
                if (rc != CONEF_OK) return rc;
            }
            continue;
        }
        if (alone(lead)) {
            int rc = launch_mq<MODE>(lead.x, lead.err, lead.cs, item_pktab(lead), lead.q, lead.p, lead.n, lead.m, lead.r,
                                     MODE == 2 ? lead.w : 1, alpha, hs, workspace, workspace_bytes, s);
            if (rc != CONEF_OK) return rc;
            done[(size_t)k] = 1;
            continue;
        }
        std::vector<int> members;
        int64_t rows = 0;
        for (int j = k; j < count; ++j) {
            if (done[(size_t)j] || alone(items[j]) || rank_bound(items[j].r) != rp || fast_of(items[j]) != fast) continue;
            members.push_back(j);
            rows += items[j].n;
            done[(size_t)j] = 1;
        }
        if (fast) {
            std::vector<MqsItem> stream_table;
            for (int j : members) {
                const ConefPsgdItem& it = items[j];
                stream_table.push_back(MqsItem{it.x, it.err, it.cs, item_pktab(it), it.q, it.p, it.n, (int)it.m,
                                               (int)(MODE == 2 ? it.w : 1), 0, 0, conef_make_mod(MODE == 2 ? it.w : 1)});
            }
            const int rc = mqs_run<MODE>(stream_table, rp, alpha, hs, s);
            if (rc != kMqsNoFit) {
                if (rc != CONEF_OK) return rc;
                continue;
            }
        }
        const int rb = mq_rows_per_wg(rows);
        std::vector<MqItem> table;
        std::vector<int> blocks;
        size_t lds = 0;
        for (int j : members) {
            const ConefPsgdItem& it = items[j];
            MqItem t = {it.x, it.err, it.cs, item_pktab(it), it.q, it.p, it.n, (int)it.m, it.r,
                        conef_make_mod(MODE == 2 ? it.w : 1)};
            table.push_back(t);
            blocks.push_back((int)((it.n + rb - 1) / rb));
            size_t need = (size_t)4 * rb * rp * 4 + (MODE == 2 ? (size_t)rb * it.w * 4 : 0);
            if (need > lds) lds = need;
        }
#define CONEF_MQB_GO(RB, RP, F)                                                                                    \
    run_batches(table, blocks, [&](const PsgdBatch<MqItem>& bt, int grid) {                                        \
        hipLaunchKernelGGL((psgd_mq_batch_kernel<RB, RP, MODE, F>), dim3((unsigned)grid), dim3(256), lds, s, bt, alpha, hs); \
    })
#define CONEF_MQB(RP)                                                  \
    do {                                                               \
        if (RP >= 16) break;                                           \
        if (rb == 4) {                                                 \
            if (fast) rc = CONEF_MQB_GO(4, (RP < 16 ? RP : 8), true);  \
            else rc = CONEF_MQB_GO(4, (RP < 16 ? RP : 8), false);      \
        } else {                                                       \
            if (fast) rc = CONEF_MQB_GO(1, (RP < 16 ? RP : 8), true);  \
            else rc = CONEF_MQB_GO(1, (RP < 16 ? RP : 8), false);      \
        }                                                              \
    } while (0)
        int rc = CONEF_OK;
        CONEF_RANK_SWITCH(lead.r, CONEF_MQB)
#undef CONEF_MQB
#undef CONEF_MQB_GO
        if (rc != CONEF_OK) return rc;
    }
    return CONEF_OK;
}

// per item: slabs of the streaming Q = X^T P kernel and where its partials start in the workspace
struct MtpPlan {
    MtpShape g;
    int64_t partial_off;    // floats; -1: one slab, the result goes straight to q
};

inline int64_t mtp_batch_layout(const ConefPsgdItem* items, int count, std::vector<MtpPlan>* plans)
{
    int64_t off = 0;
    for (int k = 0; k < count; ++k) {
        MtpPlan pl;
        pl.g = mtp_shape(items[k].n, items[k].m);
        pl.partial_off = -1;
        if (rank_bound(items[k].r) < 16 && pl.g.slabs > 1) {
            pl.partial_off = off;
            off += ((int64_t)pl.g.slabs * items[k].m * items[k].r + 63) / 64 * 64;     // 256-byte aligned regions
        }
        if (plans) plans->push_back(pl);
    }
    return off;
}

// `gram` (deferred orthogonalisation of P): count workgroups in front of the launch solve the
// matrices' Gram systems, and the row-slab partials are left for the caller's fix launch instead
// of being added here; outs[k] then says where item k's raw Q is ([slabs][m][r]).  Only for a batch
// that is one launch of this kernel (one rank below 16, all items 16-byte shaped or none).
struct MtpRaw {
    const float* src;
    int slabs;
};

int mtp_batch(const ConefPsgdItem* items, int count, void* workspace, int64_t workspace_bytes, hipStream_t s,
              const GramTask* gram = nullptr, std::vector<MtpRaw>* outs = nullptr)
{
    std::vector<MtpPlan> plans;
    const int64_t floats = mtp_batch_layout(items, count, &plans);
    // matrix-core items that have to run one by one share the front of the workspace
    const int64_t single = batch_single_bytes(items, count);
    if ((floats > 0 || single > 0) && (!workspace || workspace_bytes < floats * 4 + single)) return CONEF_ERR_INVALID;
    float* partial_base = (float*)((char*)workspace + single);
    std::vector<int64_t> mfma_offs;
    float* mfma_partials = mfma_partial_base(items, count, workspace, workspace_bytes, &mfma_offs);
    std::vector<char> done((size_t)count, 0);
    std::vector<SumItem> sums;
    std::vector<int> sum_blocks;
    bool riders_done = false;
    // matrix-core items: one launch per vector width (4, 2 or 1 floats a lane, by the alignment of x
    // and by how many workgroups the matrix has to bring to a launch it shares)
    int mfma_items = 0;
    for (int k = 0; k < count; ++k) mfma_items += rank_bound(items[k].r) >= 16;
    const int64_t want_wgs = mfma_items > 0 && 768 / mfma_items > 96 ? 768 / mfma_items : 96;
    // with riders: every width in the one launch they ride in (v = 0 below stands for "any")
    for (int pass = 0; pass < (gram ? 1 : 3) && mfma_partials; ++pass) {
        const int v = gram ? 0 : 4 >> pass;
        std::vector<MfmaMtpItem> table;
        std::vector<int> blocks;
        for (int k = 0; k < count; ++k) {
            const ConefPsgdItem& it = items[k];
            if (done[(size_t)k] || rank_bound(it.r) < 16) continue;
            const uintptr_t xa = reinterpret_cast<uintptr_t>(it.x);
            const int vmax = (it.m % 4 == 0 && (xa & 15u) == 0) ? 4 : (it.m % 2 == 0 && (xa & 7u) == 0) ? 2 : 1;
            MfmaMtpShape t = mfma_mtp_shape(it.n, it.m, it.r, vmax, want_wgs < 512 ? want_wgs : 512);
            if (v != 0 && t.v != v) continue;
            float* out = t.slabs > 1 ? mfma_partials + mfma_offs[(size_t)k] : it.q;
            MfmaMtpItem mi = {it.x, it.p, out, it.n, (int)it.m, it.r, t.rows_per_slab, t.col_tiles, t.v};
            table.push_back(mi);
            blocks.push_back(t.col_tiles * t.slabs);
            if (outs) (*outs)[(size_t)k] = MtpRaw{out, t.slabs > 1 ? t.slabs : 1};
            if (t.slabs > 1 && !gram) {
                const int64_t cnt = it.m * it.r;
                SumItem si = {out, it.q, cnt, t.slabs};
                sums.push_back(si);
                sum_blocks.push_back((int)((cnt + 255) / 256));
            }
            done[(size_t)k] = 1;
        }
        if (table.empty()) continue;
        if (gram) {
            // the Gram systems ride in this launch (the caller has checked that the batch is one launch)
            if (riders_done) return CONEF_ERR_INVALID;
            riders_done = true;
            const int rp = rank_bound(items[0].r);
            int rc = run_batches(table, blocks, [&](const PsgdBatch<MfmaMtpItem>& bt, int grid) {
                const dim3 g3((unsigned)(grid + gram->count)), b3(kMfmaThreads);
                if (rp == 32) hipLaunchKernelGGL(psgd_mfma_mtp_gram_batch_kernel<32>, g3, b3, 0, s, bt, *gram);
                else hipLaunchKernelGGL(psgd_mfma_mtp_gram_batch_kernel<16>, g3, b3, 0, s, bt, *gram);
            });
            if (rc != CONEF_OK) return rc;
            continue;
        }
        int rc = run_batches(table, blocks, [&](const PsgdBatch<MfmaMtpItem>& bt, int grid) {
            if (v == 4) hipLaunchKernelGGL(psgd_mfma_mtp_batch_kernel<4>, dim3((unsigned)grid), dim3(kMfmaThreads), 0, s, bt);
            else if (v == 2) hipLaunchKernelGGL(psgd_mfma_mtp_batch_kernel<2>, dim3((unsigned)grid), dim3(kMfmaThreads), 0, s, bt);
            else hipLaunchKernelGGL(psgd_mfma_mtp_batch_kernel<1>, dim3((unsigned)grid), dim3(kMfmaThreads), 0, s, bt);
        });
        if (rc != CONEF_OK) return rc;
    }
    for (int k = 0; k < count; ++k) {
        if (done[(size_t)k]) continue;
        const ConefPsgdItem& lead = items[k];
        const int rp = rank_bound(lead.r);
        if (rp >= 16) {
            int rc = conef_psgd_mtp_f32(lead.x, lead.p, lead.q, lead.n, lead.m, lead.r, workspace, single, (void*)s);
            if (rc != CONEF_OK) return rc;
            done[(size_t)k] = 1;
            continue;
        }
        auto fast_of = [&](int j) {
            const ConefPsgdItem& it = items[j];
            const float* out = plans[(size_t)j].partial_off >= 0 ? partial_base + plans[(size_t)j].partial_off : it.q;
            return it.r == rank_bound(it.r) && it.m % 4 == 0 && aligned16(it.x) && aligned16(it.p) && aligned16(out);
        };
        const bool fast = fast_of(k);
        std::vector<MtpItem> table;
        std::vector<int> blocks;
        for (int j = k; j < count; ++j) {
            if (done[(size_t)j] || rank_bound(items[j].r) != rp || fast_of(j) != fast) continue;
            const ConefPsgdItem& it = items[j];
            const MtpPlan& pl = plans[(size_t)j];
            float* out = pl.partial_off >= 0 ? partial_base + pl.partial_off : it.q;
            MtpItem t = {it.x, it.p, out, it.n, (int)it.m, it.r, pl.g.rows_per_slab, pl.g.col_tiles};
            table.push_back(t);
            blocks.push_back(pl.g.col_tiles * pl.g.slabs);
            if (outs) (*outs)[(size_t)j] = MtpRaw{out, pl.partial_off >= 0 ? pl.g.slabs : 1};
            if (pl.partial_off >= 0 && !gram) {
                int64_t cnt = it.m * it.r;
                SumItem si = {out, it.q, cnt, pl.g.slabs};
                sums.push_back(si);
                sum_blocks.push_back((int)((cnt + 255) / 256));
            }
            done[(size_t)j] = 1;
        }
        int rc = CONEF_OK;
#define CONEF_MTPB(RP)                                                                                              \
    do {                                                                                                            \
        if (RP >= 16) break;                                                                                        \
        if (gram) rc = run_batches(table, blocks, [&](const PsgdBatch<MtpItem>& bt, int grid) {                     \
            if (fast) hipLaunchKernelGGL((psgd_mtp_gram_batch_kernel<(RP < 16 ? RP : 8), true>), dim3((unsigned)(grid + gram->count)), dim3(kMtpThreads), 0, s, bt, *gram); \
            else hipLaunchKernelGGL((psgd_mtp_gram_batch_kernel<(RP < 16 ? RP : 8), false>), dim3((unsigned)(grid + gram->count)), dim3(kMtpThreads), 0, s, bt, *gram); \
        });                                                                                                         \
        else if (fast) rc = run_batches(table, blocks, [&](const PsgdBatch<MtpItem>& bt, int grid) {                \
            hipLaunchKernelGGL((psgd_mtp_batch_kernel<(RP < 16 ? RP : 8), true>), dim3((unsigned)grid), dim3(kMtpThreads), 0, s, bt); \
        });                                                                                                         \
        else rc = run_batches(table, blocks, [&](const PsgdBatch<MtpItem>& bt, int grid) {                          \
            hipLaunchKernelGGL((psgd_mtp_batch_kernel<(RP < 16 ? RP : 8), false>), dim3((unsigned)grid), dim3(kMtpThreads), 0, s, bt); \
        });                                                                                                         \
    } while (0)
        CONEF_RANK_SWITCH(lead.r, CONEF_MTPB)
#undef CONEF_MTPB
        if (rc != CONEF_OK) return rc;
    }
    if (!sums.empty()) {
        int rc = run_batches(sums, sum_blocks, [&](const PsgdBatch<SumItem>& bt, int grid) {
            hipLaunchKernelGGL(psgd_sum_partials_batch_kernel, dim3((unsigned)grid), dim3(256), 0, s, bt);
        });
        if (rc != CONEF_OK) return rc;
    }
    return CONEF_OK;
}

// ---- deferred orthogonalisation of P: host side ----
// The end of a batch workspace holds, per matrix, the shares of P^T P (ranks up to 8: one per
// workgroup of the first product, at most one per four rows; ranks 16 and 32: one per 256 rows),
// the solved system (b_ij and 1 / d_i) and, at ranks up to 8, the shares of Q^T Q (one per 256
// rows of Q).
inline int64_t defer_tmat_bytes(int rp) { return conef_align256((int64_t)(rp * rp + rp) * 4); }

inline int64_t defer_gram_doubles(const ConefPsgdItem& it)
{
    const int rp = rank_bound(it.r);
    return (rp <= 8 ? (it.n + 3) / 4 : (it.n + 255) / 256) * (int64_t)(rp * (rp + 1) / 2);
}

// shares of Q^T Q, one per 256 rows of Q (the fix launch leaves them for the workgroups that
// orthogonalise Q for the bucket's next round)
inline int64_t defer_qgram_doubles(const ConefPsgdItem& it)
{
    const int rp = rank_bound(it.r);
    return rp <= 8 ? ((it.m + 255) / 256) * (int64_t)(rp * (rp + 1) / 2) : 0;
}

inline int64_t defer_region_bytes(const ConefPsgdItem* items, int count)
{
    int64_t bytes = 0;
    for (int k = 0; k < count; ++k)
        bytes += conef_align256(8 * defer_gram_doubles(items[k])) + defer_tmat_bytes(rank_bound(items[k].r)) +
                 conef_align256(8 * defer_qgram_doubles(items[k]));
    return bytes;
}

inline int64_t defer_region_offset(const ConefPsgdItem* items, int count)
{
    int64_t single = 256;
    for (int k = 0; k < count; ++k) {
        int64_t b = conef_psgd_workspace_bytes(items[k].n, items[k].m, items[k].r);
        if (b > single) single = b;
    }
    return conef_align256(single) + conef_align256(4 * mtp_batch_layout(items, count, nullptr)) +
           conef_align256(4 * mfma_batch_layout(items, count, nullptr));
}

// P = X Q (raw) with the Gram shares, Q = X^T P (raw) with the systems solved on the side, then T
// applied to both.  `mq_items` differ from `items` in q only: the Q the first product reads.
// q_shares (optional): the fix launch also leaves the shares of Q^T Q of the new Q factors; their
// places are recorded in q_shares->parts / nparts.
// kMqsNoFit with nothing launched: the batch is not one this path takes (ranks
// above 8 or mixed, shapes without 16-byte accesses, a workspace without the region above).
template <int MODE>
int round_products_deferred(const ConefPsgdItem* items, const ConefPsgdItem* mq_items, int count, float alpha, float eps,
                            int32_t a, int32_t b, void* workspace, int64_t workspace_bytes, hipStream_t s,
                            GsAhead* q_shares)
{
    if (count < 1 || count > kPsgdBatchMax || !workspace) return kMqsNoFit;
    const int rp = rank_bound(items[0].r);
    if (rp > 8) return kMqsNoFit;
    const int ng = rp * (rp + 1) / 2;
    const int64_t region = defer_region_offset(items, count);
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0 || workspace_bytes < region + defer_region_bytes(items, count))
        return kMqsNoFit;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    std::vector<MqsItem> table;
    std::vector<float*> tmats;
    std::vector<double*> qgrams;
    char* at = (char*)workspace + region;
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = items[k];
        const uint32_t* pk = MODE == 2 ? item_pktab(it) : nullptr;
        const float* q_in = mq_items[k].q;       // the first product's Q (last round's, orthogonalised); it.q receives the new one
        if (it.r != rp || it.m % 4 != 0 || it.n > 0x7fffffffLL || !aligned16(it.x) || !aligned16(it.q) || !aligned16(it.p) ||
            !aligned16(q_in) || (MODE == 1 && !aligned16(it.err)) || (pk && !aligned16(pk)))
            return kMqsNoFit;
        MqsItem t = {it.x, it.err, it.cs, pk, q_in, it.p, it.n, (int)it.m, (int)(MODE == 2 ? it.w : 1), 0, 0,
                     conef_make_mod(MODE == 2 ? it.w : 1), (double*)at};
        table.push_back(t);
        at += conef_align256(8 * defer_gram_doubles(it));
        tmats.push_back((float*)at);
        at += defer_tmat_bytes(rp);
        qgrams.push_back((double*)at);
        at += conef_align256(8 * defer_qgram_doubles(it));
    }
    int T, S;
    size_t lds;
    if (!mqs_plan_launch(table.data(), count, rp, MODE == 2, &T, &S, &lds, true)) return kMqsNoFit;
    // the second product must be the 16-byte form of one launch, its partials inside the workspace
    std::vector<MtpPlan> plans;
    const int64_t mtp_floats = mtp_batch_layout(items, count, &plans);
    if (workspace_bytes < 4 * mtp_floats) return kMqsNoFit;
    for (int k = 0; k < count; ++k) {
        const float* out = plans[(size_t)k].partial_off >= 0 ? (const float*)workspace + plans[(size_t)k].partial_off : items[k].q;
        if (!aligned16(out)) return kMqsNoFit;
    }

    int rc = mqs_run<MODE>(table, rp, alpha, hs, s, true);
    if (rc != CONEF_OK) return rc;         // mqs_plan_launch above is the same decision: not kMqsNoFit here
    GramTask gram;
    gram.count = count;
    gram.eps = eps;
    for (int k = 0; k < count; ++k) {
        const int gw = mqs_group_width(items[k].m, T);
        gram.parts[k] = table[(size_t)k].gram;
        gram.nparts[k] = (int)mqs_workgroups(items[k].n, gw, S, T);
        gram.tmat[k] = tmats[(size_t)k];
    }
    std::vector<MtpRaw> raw((size_t)count);
    rc = mtp_batch(items, count, workspace, workspace_bytes, s, &gram, &raw);
    if (rc != CONEF_OK) return rc;
    std::vector<DeferFixItem> fix;
    std::vector<int> blocks;
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = items[k];
        const int pb = (int)((it.n + 255) / 256), qb = (int)((it.m + 255) / 256);
        fix.push_back(DeferFixItem{it.p, raw[(size_t)k].src, it.q, tmats[(size_t)k], q_shares ? qgrams[(size_t)k] : nullptr,
                                   it.n, it.m, raw[(size_t)k].slabs, pb});
        blocks.push_back(pb + qb);
        if (q_shares) {
            q_shares->parts[k] = qgrams[(size_t)k];
            q_shares->nparts[k] = qb;
        }
    }
    (void)ng;
#define CONEF_DFX(RP)                                                                                               \
    do {                                                                                                            \
        if (RP >= 16) break;                                                                                        \
        rc = run_batches(fix, blocks, [&](const PsgdBatch<DeferFixItem>& bt, int grid) {                            \
            hipLaunchKernelGGL((psgd_defer_fix_batch_kernel<(RP < 16 ? RP : 8)>), dim3((unsigned)grid), dim3(256), 0, s, bt); \
        });                                                                                                         \
    } while (0)
    CONEF_RANK_SWITCH(rp, CONEF_DFX)
#undef CONEF_DFX
    return rc;
}

// The same for ranks 16 and 32, whose products run on the matrix cores: the shares of P^T P come
// from a short launch of their own over the finished P, the systems ride in the second product's
// first launch, and the fix launch is the wide form.  `mq_mode` as in conef_psgd_mq_batch_f32.
int round_products_deferred_mfma(const ConefPsgdItem* items, const ConefPsgdItem* mq_items, int count, int mq_mode,
                                 float alpha, float eps, int32_t a, int32_t b, void* workspace, int64_t workspace_bytes,
                                 hipStream_t s)
{
    if (count < 1 || count > kPsgdBatchMax || !workspace) return kMqsNoFit;
    const int rp = items[0].r;
    if (rp != 16 && rp != 32) return kMqsNoFit;
    const int64_t region = defer_region_offset(items, count);
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0 || workspace_bytes < region + defer_region_bytes(items, count))
        return kMqsNoFit;
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = items[k];
        if (it.r != rp || it.m % 4 != 0 || it.n > 0x7fffffffLL || !aligned16(it.x) || !aligned16(it.q) || !aligned16(it.p) ||
            !aligned16(mq_items[k].q) || (mq_mode == 1 && !aligned16(it.err)))
            return kMqsNoFit;
    }
    // the second product must run as matrix-core launches (the systems ride in the first of them)
    // with their slabs inside the workspace
    std::vector<int64_t> offs;
    if (!mfma_partial_base(items, count, workspace, workspace_bytes, &offs)) return kMqsNoFit;
    int rc = conef_psgd_mq_batch_f32(mq_items, count, mq_mode, alpha, a, b, workspace, workspace_bytes, (void*)s);
    if (rc != CONEF_OK) return rc;
    std::vector<GramShareItem> shares;
    std::vector<int> share_blocks;
    std::vector<float*> tmats;
    GramTask gram;
    gram.count = count;
    gram.eps = eps;
    char* at = (char*)workspace + region;
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = items[k];
        const int nb = (int)((it.n + 255) / 256);
        shares.push_back(GramShareItem{it.p, it.n, (double*)at});
        share_blocks.push_back(nb);
        gram.parts[k] = (const double*)at;
        gram.nparts[k] = nb;
        at += conef_align256(8 * defer_gram_doubles(it));
        tmats.push_back((float*)at);
        gram.tmat[k] = (float*)at;
        at += defer_tmat_bytes(rp) + conef_align256(8 * defer_qgram_doubles(it));
    }
    rc = run_batches(shares, share_blocks, [&](const PsgdBatch<GramShareItem>& bt, int grid) {
        if (rp == 32) hipLaunchKernelGGL(psgd_gram_shares_batch_kernel<32>, dim3((unsigned)grid), dim3(kGsgThreads), 0, s, bt);
        else hipLaunchKernelGGL(psgd_gram_shares_batch_kernel<16>, dim3((unsigned)grid), dim3(kGsgThreads), 0, s, bt);
    });
    if (rc != CONEF_OK) return rc;
    std::vector<MtpRaw> raw((size_t)count);
    rc = mtp_batch(items, count, workspace, workspace_bytes, s, &gram, &raw);
    if (rc != CONEF_OK) return rc;
    std::vector<DeferFixItem> fix;
    std::vector<int> blocks;
    const int rows_per_wg = 256 / (rp / 4);
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = items[k];
        const int pb = (int)((it.n + rows_per_wg - 1) / rows_per_wg), qb = (int)((it.m + rows_per_wg - 1) / rows_per_wg);
        fix.push_back(DeferFixItem{it.p, raw[(size_t)k].src, it.q, tmats[(size_t)k], nullptr, it.n, it.m, raw[(size_t)k].slabs, pb});
        blocks.push_back(pb + qb);
    }
    return run_batches(fix, blocks, [&](const PsgdBatch<DeferFixItem>& bt, int grid) {
        if (rp == 32) hipLaunchKernelGGL(psgd_defer_fix_wide_batch_kernel<32>, dim3((unsigned)grid), dim3(256), 0, s, bt);
        else hipLaunchKernelGGL(psgd_defer_fix_wide_batch_kernel<16>, dim3((unsigned)grid), dim3(256), 0, s, bt);
    });
}

template <int RP, bool FAST>
struct RowlistResidualItem {
    ListPsgdResidual<RP, FAST> front;
    ConefRowlistView plan;
    const float* cs_in;
    float* cs_out;
    int64_t n;
    int d, w, rb;
};

template <int RP, bool FAST>
__global__ void __launch_bounds__(kConefRowlistThreads)
psgd_residual_rowlist_batch_kernel(PsgdBatch<RowlistResidualItem<RP, FAST>> b, double one_minus_beta)
{
    int local;
    const RowlistResidualItem<RP, FAST>& it = b.item[psgd_batch_locate(b, &local)];
    conef_rowlist_body<float, ListPsgdResidual<RP, FAST>>(it.front, it.plan, it.cs_in, it.cs_out, it.n, it.d, it.w, it.rb,
                                                          one_minus_beta, local);
}

// The same launch with a few more workgroups in front that orthogonalise the bucket's new Q factors
// into a second buffer (Q itself is still being read by the other workgroups): the reference does
// that at the start of the bucket's next round (powerSGD_hook.py:496-497), where it is a launch of
// half a dozen workgroups with the machine idle around it; here it costs nothing.
template <int RP, bool FAST>
__global__ void __launch_bounds__(kConefRowlistThreads)
psgd_residual_rowlist_gs_batch_kernel(PsgdBatch<RowlistResidualItem<RP, FAST>> b, double one_minus_beta, GsAhead g)
{
    static_assert(kConefRowlistThreads == kGsRegThreads, "one block size for both kinds of workgroup");
    if ((int)blockIdx.x < g.count) {
        gs_ahead_body<RP>(g, (int)blockIdx.x);
        return;
    }
    const int bx = (int)blockIdx.x - g.count;
    int i = 0;
    while (i + 1 < b.count && bx >= b.first[i + 1]) ++i;
    const RowlistResidualItem<RP, FAST>& it = b.item[i];
    conef_rowlist_body<float, ListPsgdResidual<RP, FAST>>(it.front, it.plan, it.cs_in, it.cs_out, it.n, it.d, it.w, it.rb,
                                                          one_minus_beta, bx - b.first[i]);
}

// The dense M = P Q^T kernel (with or without the residual written out) with the same riders.
template <int RP, int MODE, bool FAST>
__global__ void __launch_bounds__(256)
psgd_pqt_gs_batch_kernel(PsgdBatch<PqtItem> b, GsAhead g)
{
    static_assert(kGsRegThreads == 256, "one block size for both kinds of workgroup");
    if ((int)blockIdx.x < g.count) {
        gs_ahead_body<RP>(g, (int)blockIdx.x);
        return;
    }
    const int bx = (int)blockIdx.x - g.count;
    int i = 0;
    while (i + 1 < b.count && bx >= b.first[i + 1]) ++i;
    const PqtItem& it = b.item[i];
    const int local = bx - b.first[i];
    psgd_pqt_body<RP, MODE, FAST>(it.x, it.err, it.p, it.q, it.n, it.m, it.r, it.rows_per_slab, local % it.col_tiles,
                                  local / it.col_tiles);
}

template <int RP, bool FAST>
int pqt_sketch_group(const ConefPsgdItem* items, const std::vector<int>& members, float beta, hipStream_t s,
                     const GsAhead* ahead = nullptr)
{
    std::vector<RowlistResidualItem<RP, FAST>> table;
    std::vector<int> blocks;
    size_t lds = 0;
    // Full-height tiles when the bucket has 600 of them that way (over two a CU); shorter ones otherwise.
    // (Resident workgroups are bounded by LDS, so fewer, fuller tiles mean fewer rounds of them.)
    int64_t full_tiles = 0;
    for (int j : members) {
        ConefRowlistShape shape;
        if (!conef_rowlist_shape(items[j].n, items[j].m, items[j].w, false, &shape, 0)) return CONEF_ERR_INVALID;
        full_tiles += shape.tiles;
    }
    const int companions = full_tiles >= 600 ? 0 : (int)members.size();
    for (int j : members) {
        const ConefPsgdItem& it = items[j];
        ConefRowlistShape shape;
        if (!conef_rowlist_shape(it.n, it.m, it.w, false, &shape, companions)) return CONEF_ERR_INVALID;
        RowlistResidualItem<RP, FAST> t = {{it.x, it.p, it.q, it.r},
                                           conef_rowlist_view((const ConefPlanHeader*)it.plan_host, it.plan_dev),
                                           it.cs, it.cs, it.n, (int)it.m, it.w, shape.rb};
        table.push_back(t);
        blocks.push_back((int)shape.tiles);
        if (shape.lds > lds) lds = shape.lds;
    }
    auto kern = psgd_residual_rowlist_batch_kernel<RP, FAST>;
    if (hipError_t e = conef_allow_lds((const void*)kern, lds); e != hipSuccess) return (int)e;
    const double omb = 1. - (double)beta;
    if (ahead && ahead->count > 0 && table.size() <= (size_t)kPsgdBatchMax) {
        auto fused = psgd_residual_rowlist_gs_batch_kernel<RP, FAST>;
        if (hipError_t e = conef_allow_lds((const void*)fused, lds); e != hipSuccess) return (int)e;
        const GsAhead g = *ahead;
        return run_batches(table, blocks, [&](const PsgdBatch<RowlistResidualItem<RP, FAST>>& bt, int grid) {
            hipLaunchKernelGGL(fused, dim3((unsigned)(grid + g.count)), dim3(kConefRowlistThreads), lds, s, bt, omb, g);
        });
    }
    return run_batches(table, blocks, [&](const PsgdBatch<RowlistResidualItem<RP, FAST>>& bt, int grid) {
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kConefRowlistThreads), lds, s, bt, omb);
    });
}

// ahead: the Q factors to orthogonalise alongside (mode 2, one rank class over the whole bucket
// only); *ahead_used says whether that was done.
int pqt_batch(const ConefPsgdItem* items, int count, int mode, float beta, int32_t a, int32_t b, hipStream_t s,
              const GsAhead* ahead = nullptr, bool* ahead_used = nullptr)
{
    if (ahead_used) *ahead_used = false;
    std::vector<char> done((size_t)count, 0);
    for (int k = 0; k < count; ++k) {
        if (done[(size_t)k]) continue;
        const ConefPsgdItem& lead = items[k];
        const int rp = rank_bound(lead.r);
        if (mode != 2 && (lead.r == 16 || lead.r == 32) && aligned16(lead.p) && aligned16(lead.q)) {
            // matrix-core items of one rank share a launch
            std::vector<MfmaPqtItem> table;
            std::vector<int> blocks;
            for (int j = k; j < count; ++j) {
                const ConefPsgdItem& it = items[j];
                if (done[(size_t)j] || it.r != lead.r || !aligned16(it.p) || !aligned16(it.q)) continue;
                int64_t col_wgs = (it.m + 32 * kMfmaWaves - 1) / (32 * kMfmaWaves);
                int64_t slabs = (1024 + col_wgs - 1) / col_wgs;
                int64_t rps = ((it.n + slabs - 1) / slabs + 31) / 32 * 32;
                slabs = (it.n + rps - 1) / rps;
                MfmaPqtItem t = {it.x, mode == 1 ? it.err : nullptr, it.p, it.q, it.n, (int)it.m, (int)rps, (int)col_wgs};
                table.push_back(t);
                blocks.push_back((int)(col_wgs * slabs));
                done[(size_t)j] = 1;
            }
            int rc = run_batches(table, blocks, [&](const PsgdBatch<MfmaPqtItem>& bt, int grid) {
                if (lead.r == 32) {
                    if (mode == 1) hipLaunchKernelGGL((psgd_mfma_pqt_batch_kernel<32, 1>), dim3((unsigned)grid), dim3(kMfmaThreads), 0, s, bt);
                    else hipLaunchKernelGGL((psgd_mfma_pqt_batch_kernel<32, 0>), dim3((unsigned)grid), dim3(kMfmaThreads), 0, s, bt);
                } else {
                    if (mode == 1) hipLaunchKernelGGL((psgd_mfma_pqt_batch_kernel<16, 1>), dim3((unsigned)grid), dim3(kMfmaThreads), 0, s, bt);
                    else hipLaunchKernelGGL((psgd_mfma_pqt_batch_kernel<16, 0>), dim3((unsigned)grid), dim3(kMfmaThreads), 0, s, bt);
                }
            });
            if (rc != CONEF_OK) return rc;
            continue;
        }
        if (rp >= 16 || mode == 2) {
            if (mode == 2 && rp < 16) {
                // residual sketch on row-list plans: items of one rank class share launches
                auto fast_of = [&](const ConefPsgdItem& it) {
                    return it.r == rank_bound(it.r) && it.m % 4 == 0 && aligned16(it.x) && aligned16(it.q) && aligned16(it.p);
                };
                const bool fast = fast_of(lead);
                std::vector<int> members;
                for (int j = k; j < count; ++j) {
                    if (done[(size_t)j] || rank_bound(items[j].r) != rp || fast_of(items[j]) != fast) continue;
                    const ConefPlanHeader* hp = (const ConefPlanHeader*)items[j].plan_host;
                    if (!conef_plan_matches(hp, items[j].n, items[j].m, items[j].w, a, b) || hp->kind != kConefPlanRowlist ||
                        !items[j].plan_dev || !items[j].cs)
                        return CONEF_ERR_INVALID;
                    members.push_back(j);
                    done[(size_t)j] = 1;
                }
                int rc = CONEF_ERR_INVALID;
                const GsAhead* ride = (ahead && ahead->count > 0 && members.size() == (size_t)count &&
                                       count <= kPsgdBatchMax && rank_bound(ahead->r) == rp) ? ahead : nullptr;
#define CONEF_PQS(RP)                                                                  \
    do {                                                                               \
        if (RP >= 16) break;                                                           \
        if (fast) rc = pqt_sketch_group<(RP < 16 ? RP : 8), true>(items, members, beta, s, ride);  \
        else rc = pqt_sketch_group<(RP < 16 ? RP : 8), false>(items, members, beta, s, ride);      \
    } while (0)
                CONEF_RANK_SWITCH(lead.r, CONEF_PQS)
#undef CONEF_PQS
                if (rc != CONEF_OK) return rc;
                if (ride && ahead_used) *ahead_used = true;
                continue;
            }
            int rc;
            if (mode == 2)
                rc = conef_psgd_pqt_conef_planned_f32(lead.x, lead.p, lead.q, lead.cs, lead.cs, lead.plan_host, lead.plan_dev,
                                                      lead.n, lead.m, lead.r, lead.w, beta, a, b, (void*)s);
            else
                rc = launch_pqt(lead.x, mode == 1 ? lead.err : nullptr, lead.p, lead.q, lead.n, lead.m, lead.r, s);
            if (rc != CONEF_OK) return rc;
            done[(size_t)k] = 1;
            continue;
        }
        auto fast_of = [&](const ConefPsgdItem& it) {
            return it.r == rank_bound(it.r) && it.m % 4 == 0 && aligned16(it.x) && aligned16(it.q) &&
                   (mode != 1 || aligned16(it.err));
        };
        const bool fast = fast_of(lead);
        std::vector<PqtItem> table;
        std::vector<int> blocks;
        for (int j = k; j < count; ++j) {
            if (done[(size_t)j] || rank_bound(items[j].r) != rp || fast_of(items[j]) != fast) continue;
            const ConefPsgdItem& it = items[j];
            // about a thousand workgroups for the batch as a whole, slabs of at least four rows
            int64_t col_tiles = (it.m + 1023) / 1024;
            int64_t slabs = (256 + col_tiles - 1) / col_tiles;
            int64_t rps = (it.n + slabs - 1) / slabs;
            if (rps < 4) rps = 4;
            slabs = (it.n + rps - 1) / rps;
            PqtItem t = {it.x, mode == 1 ? it.err : nullptr, it.p, it.q, it.n, (int)it.m, it.r, (int)rps, (int)col_tiles};
            table.push_back(t);
            blocks.push_back((int)(col_tiles * slabs));
            done[(size_t)j] = 1;
        }
        int rc = CONEF_OK;
        const GsAhead* ride = (ahead && ahead->count > 0 && table.size() == (size_t)count && count <= kPsgdBatchMax &&
                               rank_bound(ahead->r) == rp) ? ahead : nullptr;
        GsAhead g;
        g.count = 0;
        if (ride) g = *ride;
#define CONEF_PQB_GO(RP, MODE, F)                                                                                  \
    run_batches(table, blocks, [&](const PsgdBatch<PqtItem>& bt, int grid) {                                       \
        if (ride)                                                                                                  \
            hipLaunchKernelGGL((psgd_pqt_gs_batch_kernel<RP, MODE, F>), dim3((unsigned)(grid + g.count)), dim3(256), 0, s, \
                               bt, g);                                                                             \
        else                                                                                                       \
            hipLaunchKernelGGL((psgd_pqt_batch_kernel<RP, MODE, F>), dim3((unsigned)grid), dim3(256), 0, s, bt);   \
    })
#define CONEF_PQB(RP)                                                          \
    do {                                                                       \
        if (RP >= 16) break;                                                   \
        if (mode == 1) {                                                       \
            if (fast) rc = CONEF_PQB_GO((RP < 16 ? RP : 8), 1, true);          \
            else rc = CONEF_PQB_GO((RP < 16 ? RP : 8), 1, false);              \
        } else {                                                               \
            if (fast) rc = CONEF_PQB_GO((RP < 16 ? RP : 8), 0, true);          \
            else rc = CONEF_PQB_GO((RP < 16 ? RP : 8), 0, false);              \
        }                                                                      \
    } while (0)
        CONEF_RANK_SWITCH(lead.r, CONEF_PQB)
#undef CONEF_PQB
#undef CONEF_PQB_GO
        if (rc != CONEF_OK) return rc;
        if (ride && ahead_used) *ahead_used = true;
    }
    return CONEF_OK;
}

}  // namespace

extern "C" {

int64_t conef_psgd_batch_workspace_bytes(const ConefPsgdItem* items, int32_t count)
{
    if (count < 0 || (count > 0 && !items)) return -1;
    int64_t single = 256;
    for (int k = 0; k < count; ++k) {
        if (!psgd_args_ok(items[k].n, items[k].m, items[k].r)) return -1;
        int64_t b = conef_psgd_workspace_bytes(items[k].n, items[k].m, items[k].r);
        if (b > single) single = b;
    }
    const int64_t launches = conef_align256(single) + conef_align256(4 * mtp_batch_layout(items, count, nullptr)) +
                             conef_align256(4 * mfma_batch_layout(items, count, nullptr)) + defer_region_bytes(items, count);
    const int64_t small = conef_psgd_round_small_workspace_bytes(items, count);      // the one-launch round's records
    return small > launches ? small : launches;
}

int conef_psgd_mq_batch_f32(const ConefPsgdItem* items, int32_t count, int32_t mode, float alpha, int32_t a, int32_t b,
                            void* workspace, int64_t workspace_bytes, void* stream)
{
    if (count < 0 || (count > 0 && !items) || mode < 0 || mode > 2) return CONEF_ERR_INVALID;
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = items[k];
        if (!item_ok(it) || (mode == 1 && !it.err) || (mode == 2 && (!it.cs || it.w < 1 || it.w > (1 << 30))))
            return CONEF_ERR_INVALID;
        if (mode == 2 && it.plan_host && !conef_plan_matches((const ConefPlanHeader*)it.plan_host, it.n, it.m, it.w, a, b))
            return CONEF_ERR_INVALID;
    }
    hipStream_t s = (hipStream_t)stream;
    if (mode == 0) return mq_batch<0>(items, count, 0.f, a, b, workspace, workspace_bytes, s);
    if (mode == 1) return mq_batch<1>(items, count, 0.f, a, b, workspace, workspace_bytes, s);
    return mq_batch<2>(items, count, alpha, a, b, workspace, workspace_bytes, s);
}

int conef_psgd_mtp_batch_f32(const ConefPsgdItem* items, int32_t count, void* workspace, int64_t workspace_bytes,
                             void* stream)
{
    if (count < 0 || (count > 0 && !items)) return CONEF_ERR_INVALID;
    for (int k = 0; k < count; ++k)
        if (!item_ok(items[k])) return CONEF_ERR_INVALID;
    return mtp_batch(items, count, workspace, workspace_bytes, (hipStream_t)stream);
}

int conef_psgd_pqt_batch_f32(const ConefPsgdItem* items, int32_t count, int32_t mode, float beta, int32_t a, int32_t b,
                             void* stream)
{
    if (count < 0 || (count > 0 && !items) || mode < 0 || mode > 2) return CONEF_ERR_INVALID;
    for (int k = 0; k < count; ++k)
        if (!item_ok(items[k]) || (mode == 1 && !items[k].err)) return CONEF_ERR_INVALID;
    return pqt_batch(items, count, mode, beta, a, b, (hipStream_t)stream);
}

// cs = update(cs, err, beta) in place for every item (DenseCS.update, CountSketch.py:27-48, with
// vec = the item's dense [n,m] residual at err): the sketches of a bucket in one launch.  Every
// item needs a row-list plan built for (n, m, w, a, b).
int conef_psgd_sketch_update_batch_f32(const ConefPsgdItem* items, int32_t count, float beta, int32_t a, int32_t b,
                                       void* stream)
{
    if (count < 0 || (count > 0 && !items)) return CONEF_ERR_INVALID;
    std::vector<RowlistVecItem> table;
    std::vector<int> blocks;
    size_t lds = 0;
    int64_t full_tiles = 0;     // as in pqt_sketch_group: full-height tiles when there are 600 of them
    for (int k = 0; k < count; ++k) {
        ConefRowlistShape shape;
        if (conef_rowlist_shape(items[k].n, items[k].m, items[k].w, ConefListVec::kNeedsCells, &shape, 0))
            full_tiles += shape.tiles;
    }
    const int companions = full_tiles >= 600 ? 0 : count;
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = items[k];
        const ConefPlanHeader* hp = (const ConefPlanHeader*)it.plan_host;
        if (!psgd_args_ok(it.n, it.m, it.r) || !it.err || !it.cs || !it.plan_dev ||
            !conef_plan_matches(hp, it.n, it.m, it.w, a, b) || hp->kind != kConefPlanRowlist)
            return CONEF_ERR_INVALID;
        ConefRowlistShape shape;
        if (!conef_rowlist_shape(it.n, it.m, it.w, ConefListVec::kNeedsCells, &shape, companions)) return CONEF_ERR_INVALID;
        RowlistVecItem t = {{it.err, aligned16(it.err) && it.m % 4 == 0}, conef_rowlist_view(hp, it.plan_dev), it.cs, it.cs,
                            it.n, (int)it.m, it.w, shape.rb};
        table.push_back(t);
        blocks.push_back((int)shape.tiles);
        if (shape.lds > lds) lds = shape.lds;
    }
    if (hipError_t e = conef_allow_lds((const void*)psgd_rowlist_vec_batch_kernel, lds); e != hipSuccess) return (int)e;
    const double omb = 1. - (double)beta;
    hipStream_t s = (hipStream_t)stream;
    return run_batches(table, blocks, [&](const PsgdBatch<RowlistVecItem>& bt, int grid) {
        hipLaunchKernelGGL(psgd_rowlist_vec_batch_kernel, dim3((unsigned)grid), dim3(kConefRowlistThreads), lds, s, bt, omb);
    });
}

// One PowerSGD round over the matrices of a bucket in a single call (powerSGD_hook.py:473-564 at
// world size 1): orthogonalise every Q, P = X Q with the error added first (mq_mode as in
// conef_psgd_mq_batch_f32), orthogonalise every P, Q = X^T P, X = P Q^T with the new error
// (pqt_mode 0, 1, 2 as in conef_psgd_pqt_batch_f32; 3 = mode 1 followed by
// conef_psgd_sketch_update_batch_f32 on the residuals).  The same launches as the separate calls,
// in the same order; what it saves is the caller's trips through its foreign-function interface.
int conef_psgd_round_ahead_f32(const ConefPsgdItem* items, int32_t count, int32_t mq_mode, int32_t pqt_mode, float alpha,
                               float beta, float eps, int32_t a, int32_t b, float* const* q_next, int32_t flags,
                               int32_t* made, void* workspace, int64_t workspace_bytes, void* stream)
{
    if (made) *made = 0;
    if (count < 0 || (count > 0 && !items) || pqt_mode < 0 || pqt_mode > 3) return CONEF_ERR_INVALID;
    if ((flags & (CONEF_ROUND_Q_READY | CONEF_ROUND_MAKE_NEXT)) && (!q_next || !made)) return CONEF_ERR_INVALID;
    if (count == 0) return CONEF_OK;
    std::vector<float*> mats((size_t)count);
    std::vector<int64_t> rows((size_t)count);
    std::vector<int32_t> ranks((size_t)count);
    for (int k = 0; k < count; ++k) {
        if (!item_ok(items[k])) return CONEF_ERR_INVALID;
        mats[(size_t)k] = items[k].q;
        rows[(size_t)k] = items[k].m;
        ranks[(size_t)k] = items[k].r;
    }
    // P = X Q, P orthogonalised, Q = X^T P: with the orthogonalisation deferred where the batch
    // allows (round_products_deferred; CONEF_ROUND_DEFER=0 keeps the reference's order of steps,
    // for comparisons), else as three steps
    const char* defer_env = getenv("CONEF_ROUND_DEFER");      // read on every call: a test switches it
    const bool defer_on = !(defer_env && defer_env[0] == '0');
    GsAhead ahead;
    ahead.count = 0;
    for (int k = 0; k < kPsgdBatchMax; ++k) {
        ahead.parts[k] = nullptr;
        ahead.nparts[k] = 0;
    }
    // the next round's Q factors are wanted in q_next, by workgroups of this round's last launch
    bool want_next = (flags & CONEF_ROUND_MAKE_NEXT) && pqt_mode <= 2 && count <= kPsgdBatchMax && rank_bound(items[0].r) <= 8;
    for (int k = 0; k < count && want_next; ++k)
        want_next = q_next[k] && items[k].r == items[0].r && aligned16(q_next[k]) && aligned16(items[k].q) &&
                    items[k].m <= 0x7fffffffLL;
    bool q_shares_made = false;
    auto products = [&](const ConefPsgdItem* its) -> int {      // its: the items with the Q the first product reads
        if (mq_mode < 0 || mq_mode > 2) return CONEF_ERR_INVALID;
        for (int k = 0; k < count; ++k) {
            const ConefPsgdItem& it = its[k];
            if ((mq_mode == 1 && !it.err) || (mq_mode == 2 && (!it.cs || it.w < 1 || it.w > (1 << 30)))) return CONEF_ERR_INVALID;
            if (mq_mode == 2 && it.plan_host && !conef_plan_matches((const ConefPlanHeader*)it.plan_host, it.n, it.m, it.w, a, b))
                return CONEF_ERR_INVALID;
        }
        if (defer_on) {
            hipStream_t hs = (hipStream_t)stream;
            GsAhead* qs = want_next ? &ahead : nullptr;
            const int rd = mq_mode == 0   ? round_products_deferred<0>(items, its, count, 0.f, eps, a, b, workspace, workspace_bytes, hs, qs)
                           : mq_mode == 1 ? round_products_deferred<1>(items, its, count, 0.f, eps, a, b, workspace, workspace_bytes, hs, qs)
                                          : round_products_deferred<2>(items, its, count, alpha, eps, a, b, workspace, workspace_bytes, hs, qs);
            if (rd == CONEF_OK) q_shares_made = want_next;
            if (rd != kMqsNoFit) return rd;
            const int rm = round_products_deferred_mfma(items, its, count, mq_mode, alpha, eps, a, b, workspace, workspace_bytes, hs);
            if (rm != kMqsNoFit) return rm;
        }
        int rp = conef_psgd_mq_batch_f32(its, count, mq_mode, alpha, a, b, workspace, workspace_bytes, stream);
        if (rp != CONEF_OK) return rp;
        for (int k = 0; k < count; ++k) {
            mats[(size_t)k] = items[k].p;
            rows[(size_t)k] = items[k].n;
        }
        rp = conef_gram_schmidt_batch_f32(mats.data(), rows.data(), ranks.data(), count, eps, workspace, workspace_bytes, stream);
        if (rp != CONEF_OK) return rp;
        return conef_psgd_mtp_batch_f32(items, count, workspace, workspace_bytes, stream);
    };
    int rc = CONEF_OK;
    if (flags & CONEF_ROUND_Q_READY) {
        // q_next holds this round's Q factors, orthogonalised at the end of the bucket's last round
        std::vector<ConefPsgdItem> with_q(items, items + count);
        for (int k = 0; k < count; ++k) {
            if (!q_next[k]) return CONEF_ERR_INVALID;
            with_q[(size_t)k].q = q_next[k];
        }
        rc = products(with_q.data());
    } else {
        rc = conef_gram_schmidt_batch_f32(mats.data(), rows.data(), ranks.data(), count, eps, workspace, workspace_bytes, stream);
        if (rc != CONEF_OK) return rc;
        rc = products(items);
    }
    if (rc != CONEF_OK) return rc;
    // The new Q factors orthogonalised into q_next by workgroups of the last launch, where that
    // launch covers the whole bucket (one rank, at most 8): from the shares of Q^T Q when the
    // products above left them, else by the column steps themselves, which takes a short Q factor.
    if (want_next) {
        bool ok = true;
        for (int k = 0; k < count && ok && !q_shares_made; ++k)
            ok = gs_reg_class(items[k].q, items[k].m, items[k].r) >= 0 &&
                 items[k].m <= (int64_t)kGsAheadRowSlots * kGsRegThreads;
        if (ok) {
            for (int k = 0; k < count; ++k) {
                ahead.src[k] = items[k].q;
                ahead.dst[k] = q_next[k];
                ahead.rows[k] = (int)items[k].m;
                if (!q_shares_made) ahead.parts[k] = nullptr;
            }
            ahead.count = count;
            ahead.r = items[0].r;
            ahead.eps = eps;
        }
    }
    bool used = false;
    for (int k = 0; k < count; ++k)
        if ((pqt_mode == 1 || pqt_mode == 3) && !items[k].err) return CONEF_ERR_INVALID;
    rc = pqt_batch(items, count, pqt_mode == 3 ? 1 : pqt_mode, pqt_mode == 2 ? beta : 0.f, a, b, (hipStream_t)stream,
                   ahead.count ? &ahead : nullptr, &used);
    if (rc != CONEF_OK) return rc;
    if (made) *made = used ? 1 : 0;
    if (pqt_mode == 3) rc = conef_psgd_sketch_update_batch_f32(items, count, beta, a, b, stream);
    return rc;
}

// Whether conef_psgd_round_small_f32 takes this bucket: at most 24 matrices of at most 73728 elements
// each (a matrix goes whole to one workgroup up to 10240 elements, over up to 16 otherwise), 128
// workgroups in all, every workgroup's rows fit its LDS with the factors and the sketch's bucket
// lists, ranks up to 8, and (modes 2) a row-list plan per sketch.
int conef_psgd_round_small_fits(const ConefPsgdItem* items, int32_t count, int32_t mq_mode, int32_t pqt_mode, int32_t a,
                                int32_t b)
{
    if (count < 1 || count > kSmallMaxItems || !items || mq_mode < 0 || mq_mode > 2 || pqt_mode < 0 || pqt_mode > 2) return 0;
    if ((mq_mode == 2) != (pqt_mode == 2)) return 0;
    int rp = 1, wgs = 0;
    for (int k = 0; k < count; ++k)
        if (item_ok(items[k]) && rank_bound(items[k].r) > rp) rp = rank_bound(items[k].r);      // a launch is sized for its largest rank
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = items[k];
        if (!item_ok(it) || it.r > 8 || it.n * it.m > kSmallMaxSlices * kSmallSliceElements) return 0;
        if ((mq_mode == 1 || pqt_mode == 1) && !it.err) return 0;
        int w = 0;
        if (mq_mode == 2) {
            const ConefPlanHeader* hp = (const ConefPlanHeader*)it.plan_host;
            if (!it.cs || !it.plan_dev || !conef_plan_matches(hp, it.n, it.m, it.w, a, b) || hp->kind != kConefPlanRowlist)
                return 0;
            w = it.w;
        }
        int rows_per;
        wgs += small_slices(it.n, it.m, &rows_per);
        if (small_lds_bytes(rows_per, (int)it.n, (int)it.m, rp, w) > kSmallLdsLimit) return 0;
    }
    return wgs <= kSmallMaxWgs ? 1 : 0;
}

// Bytes of workspace conef_psgd_round_small_f32 needs for this bucket (the records its sliced
// matrices exchange; 0 when every matrix goes to one workgroup).
int64_t conef_psgd_round_small_workspace_bytes(const ConefPsgdItem* items, int32_t count)
{
    if (count < 0 || (count > 0 && !items)) return -1;
    int64_t recs = 0;
    for (int k = 0; k < count; ++k) {
        if (!item_ok(items[k])) return -1;
        int rows_per;
        const int sl = small_slices(items[k].n, items[k].m, &rows_per);
        recs += (small_record_count(items[k].n, items[k].m, items[k].r, sl) + 31) / 32 * 32;
    }
    return recs * 8;
}

// The round of conef_psgd_round_f32 for a bucket of small matrices, in ONE launch: a workgroup per
// matrix, the matrix in LDS, workgroup barriers between the stages (conef_psgd_small.h).
int conef_psgd_round_small_f32(const ConefPsgdItem* items, int32_t count, int32_t mq_mode, int32_t pqt_mode, float alpha,
                               float beta, float eps, int32_t a, int32_t b, void* workspace, int64_t workspace_bytes,
                               void* stream)
{
    if (!conef_psgd_round_small_fits(items, count, mq_mode, pqt_mode, a, b)) return CONEF_ERR_INVALID;
    const int64_t ws_need = conef_psgd_round_small_workspace_bytes(items, count);
    if (ws_need > 0 && (!workspace || workspace_bytes < ws_need || ((uintptr_t)workspace & 7))) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    const double omb = 1. - (double)beta;
    unsigned tag = (g_small_launches.fetch_add(1u) + 1u) * 0x9E3779B9u;      // never the tag of the records' last use
    if (tag == 0u) tag = 1u;
    {
        const int k0 = 0, nb = count;
        SmallBatch batch;
        batch.count = nb;
        int rp = 1, wgs = 0;
        size_t lds = 0;
        unsigned long long* recs = (unsigned long long*)workspace;
        for (int k = 0; k < nb; ++k) {
            const ConefPsgdItem& it = items[k0 + k];
            SmallItem& t = batch.item[k];
            t.x = it.x;
            t.err = it.err;
            t.cs = it.cs;
            t.csr = nullptr;
            t.ent = nullptr;
            t.pk = nullptr;
            t.w = 0;
            if (mq_mode == 2) {
                const ConefRowlistView v = conef_rowlist_view((const ConefPlanHeader*)it.plan_host, it.plan_dev);
                t.csr = v.csr;
                t.ent = v.ent;
                t.pk = v.pk;
                t.w = it.w;
            }
            t.p = it.p;
            t.q = it.q;
            t.n = (int)it.n;
            t.m = (int)it.m;
            t.r = it.r;
            t.fast = it.m % 4 == 0 && aligned16(it.x) && ((mq_mode != 1 && pqt_mode != 1) || aligned16(it.err));
            t.slices = small_slices(it.n, it.m, &t.rows_per);
            wgs += t.slices;
            t.recs = t.slices > 1 ? recs : nullptr;
            recs += (small_record_count(it.n, it.m, it.r, t.slices) + 31) / 32 * 32;
            if (rank_bound(it.r) > rp) rp = rank_bound(it.r);
        }
        for (int k = 0; k < nb; ++k) {
            const size_t need = small_lds_bytes(batch.item[k].rows_per, batch.item[k].n, batch.item[k].m, rp, batch.item[k].w);
            if (need > lds) lds = need;
        }
        if (lds > kSmallLdsLimit || wgs > kSmallMaxWgs) return CONEF_ERR_INVALID;
        // which workgroup does what: slices on the workgroups of XCDs 0..3 (b % 8 < 4), whole matrices on
        // those of XCDs 4..7 first; with nothing sliced, in plain order
        std::vector<unsigned short> sliced, whole;
        for (int k = 0; k < nb; ++k) {
            if (batch.item[k].slices > 1)
                for (int sl = 0; sl < batch.item[k].slices; ++sl) sliced.push_back((unsigned short)(k | (sl << 8)));
            else
                whole.push_back((unsigned short)k);
        }
        for (int b2 = 0; b2 < kSmallMaxGrid; ++b2) batch.where[b2] = kSmallIdle;
        int grid = wgs;
        if (sliced.empty()) {
            for (int b2 = 0; b2 < wgs; ++b2) batch.where[b2] = whole[(size_t)b2];
        } else {
            int groups = (wgs + 7) / 8;
            if ((int)sliced.size() > 4 * groups) groups = ((int)sliced.size() + 3) / 4;
            auto early = [](int e) { return (e / 4) * 8 + e % 4; };
            auto late = [](int l) { return (l / 4) * 8 + 4 + l % 4; };
            int e = 0, l = 0;
            grid = 0;
            for (unsigned short w2 : sliced) {
                const int b2 = early(e++);
                batch.where[b2] = w2;
                if (b2 + 1 > grid) grid = b2 + 1;
            }
            for (unsigned short w2 : whole) {
                const int b2 = l < 4 * groups ? late(l++) : early(e++);
                batch.where[b2] = w2;
                if (b2 + 1 > grid) grid = b2 + 1;
            }
        }
#define CONEF_SMALL(RP)                                                                                         \
    do {                                                                                                        \
        auto kern = psgd_small_round_kernel<RP>;                                                                \
        if (hipError_t e = conef_allow_lds((const void*)kern, lds); e != hipSuccess) return (int)e;             \
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kSmallThreads), lds, s, batch, tag, mq_mode, pqt_mode, alpha, omb, eps); \
    } while (0)
        switch (rp) {
            case 1: CONEF_SMALL(1); break;
            case 2: CONEF_SMALL(2); break;
            case 4: CONEF_SMALL(4); break;
            default: CONEF_SMALL(8); break;
        }
#undef CONEF_SMALL
        const int rc = (int)hipGetLastError();
        if (rc != CONEF_OK) return rc;
    }
    return CONEF_OK;
}

int conef_psgd_round_f32(const ConefPsgdItem* items, int32_t count, int32_t mq_mode, int32_t pqt_mode, float alpha,
                         float beta, float eps, int32_t a, int32_t b, void* workspace, int64_t workspace_bytes,
                         void* stream)
{
    return conef_psgd_round_ahead_f32(items, count, mq_mode, pqt_mode, alpha, beta, eps, a, b, nullptr, 0, nullptr,
                                      workspace, workspace_bytes, stream);
}

// The middle of a round as a call of its own, for a caller that splits the round (the hooks at
// ranks above 8 do, to run the Gram-Schmidt of the new Q on a side stream): P = X Q with the Q of
// `first` (items whose q may point elsewhere, or null for items' own), P orthogonalised,
// Q = X^T P into items[k].q - deferred where the batch allows, as in conef_psgd_round_f32.
int conef_psgd_products_f32(const ConefPsgdItem* items, const ConefPsgdItem* first, int32_t count, int32_t mq_mode,
                            float alpha, float eps, int32_t a, int32_t b, void* workspace, int64_t workspace_bytes,
                            void* stream)
{
    if (count < 0 || (count > 0 && !items) || mq_mode < 0 || mq_mode > 2) return CONEF_ERR_INVALID;
    if (count == 0) return CONEF_OK;
    const ConefPsgdItem* its = first ? first : items;
    for (int k = 0; k < count; ++k) {
        const ConefPsgdItem& it = its[k];
        if (!item_ok(items[k]) || !item_ok(it) || it.n != items[k].n || it.m != items[k].m || it.r != items[k].r ||
            it.x != items[k].x || it.p != items[k].p)
            return CONEF_ERR_INVALID;
        if ((mq_mode == 1 && !it.err) || (mq_mode == 2 && (!it.cs || it.w < 1 || it.w > (1 << 30)))) return CONEF_ERR_INVALID;
        if (mq_mode == 2 && it.plan_host && !conef_plan_matches((const ConefPlanHeader*)it.plan_host, it.n, it.m, it.w, a, b))
            return CONEF_ERR_INVALID;
    }
    const char* defer_env = getenv("CONEF_ROUND_DEFER");
    if (!(defer_env && defer_env[0] == '0')) {
        hipStream_t hs = (hipStream_t)stream;
        const int rd = mq_mode == 0   ? round_products_deferred<0>(items, its, count, 0.f, eps, a, b, workspace, workspace_bytes, hs, nullptr)
                       : mq_mode == 1 ? round_products_deferred<1>(items, its, count, 0.f, eps, a, b, workspace, workspace_bytes, hs, nullptr)
                                      : round_products_deferred<2>(items, its, count, alpha, eps, a, b, workspace, workspace_bytes, hs, nullptr);
        if (rd != kMqsNoFit) return rd;
        const int rm = round_products_deferred_mfma(items, its, count, mq_mode, alpha, eps, a, b, workspace, workspace_bytes, hs);
        if (rm != kMqsNoFit) return rm;
    }
    int rc = conef_psgd_mq_batch_f32(its, count, mq_mode, alpha, a, b, workspace, workspace_bytes, stream);
    if (rc != CONEF_OK) return rc;
    std::vector<float*> mats((size_t)count);
    std::vector<int64_t> rows((size_t)count);
    std::vector<int32_t> ranks((size_t)count);
    for (int k = 0; k < count; ++k) {
        mats[(size_t)k] = items[k].p;
        rows[(size_t)k] = items[k].n;
        ranks[(size_t)k] = items[k].r;
    }
    rc = conef_gram_schmidt_batch_f32(mats.data(), rows.data(), ranks.data(), count, eps, workspace, workspace_bytes, stream);
    if (rc != CONEF_OK) return rc;
    return conef_psgd_mtp_batch_f32(items, count, workspace, workspace_bytes, stream);
}

// dense error feedback on the parts of a bucket that are not compressed: x += e; e = 0
// (powerSGD_hook.py:361 and :558, where copy - result is exactly zero for untouched tensors)
int conef_ef_passthrough_f32(float* x, float* err, int64_t count, void* stream);

}  // extern "C"

namespace {
__global__ void ef_passthrough_kernel(float* __restrict__ x, float* __restrict__ err, int64_t count)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        x[i] = __fadd_rn(x[i], err[i]);
        err[i] = 0.f;
    }
}
}  // namespace

extern "C" int conef_ef_passthrough_f32(float* x, float* err, int64_t count, void* stream)
{
    if (count < 0 || (count > 0 && (!x || !err))) return CONEF_ERR_INVALID;
    if (count == 0) return CONEF_OK;
    int64_t g = (count + 255) / 256;
    if (g > 4096) g = 4096;
    hipLaunchKernelGGL(ef_passthrough_kernel, dim3((unsigned)g), dim3(256), 0, (hipStream_t)stream, x, err, count);
    return (int)hipGetLastError();
}
