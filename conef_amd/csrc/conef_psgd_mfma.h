// PowerSGD products at rank 16..32 on the matrix cores (v_mfma_f32_32x32x2f32: true fp32 inputs and
// accumulation, so the 1e-5 parity bar of the rank 1..8 streaming kernels holds here too).
//
// At these ranks a thread-per-column-quad kernel re-reads 4*r floats of Q (or P) for every 16 bytes
// of M it streams: the L2 -> CU traffic is 8..16 times the HBM traffic and the kernels fall to a
// twentieth of the HBM rate.  An MFMA tile shares one operand over 32 rows (or columns) of M
// instead, and the products are HBM-bound again: 2*r flops per 4 bytes of M is 16 flop/byte at
// r = 32, just below the fp32 ridge of the machine (157 TFLOP/s over 8 TB/s).
//
// Operand layout of v_mfma_f32_32x32x2f32 (D[32x32] += A[32x2] * B[2x32], one float per lane):
//   A: lane l holds A[l % 32][l / 32]          B: lane l holds B[l / 32][l % 32]
//   D: lane l, register v holds D[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32]
// The two k of a step only have to agree between A and B, not to be adjacent in memory, so a lane
// may feed consecutive steps from one 16-byte load: the kernels below pick k per lane half that way.
#pragma once
#include "conef_device.h"
#include "conef_sketch_core.h"

typedef float conef_f16v __attribute__((ext_vector_type(16)));

__device__ __forceinline__ conef_f16v conef_mfma32(float a, float b, conef_f16v c)
{
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ int conef_mfma_row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }

constexpr int kMfmaWaves = 4;
constexpr int kMfmaThreads = 64 * kMfmaWaves;

// ------------------------------------------------------------------ P = X Q ----
// MODE 0: X = M.  MODE 1: X = M + E, written back.  MODE 2: X = M + alpha * unsketch(cs), written
// back (the sketch rows of the tile's 32 matrix rows are parked in LDS).
// A workgroup owns 32 rows and the column range [blockIdx.y * cols_per_split, +cols_per_split); its
// four waves take 32-column blocks of that range in turn.  Lane (row = l % 32, half = l / 32) loads
// X[row][c .. c+3] with c = block + 8u + 4 * half for u = 0..3 and feeds step (u, j) with component j;
// the matching B operand is Q[c + j][l % 32].  The waves' tiles meet in LDS in a fixed order; with
// more than one column split the tile goes to a partial buffer [split][n][r] that a second kernel
// adds up in split order.  Requires m % 4 == 0 and 16-byte aligned x (err, pktab).
template <int MODE>
__device__ __forceinline__ void
psgd_mfma_mq_body(float* __restrict__ x, const float* __restrict__ err, const float* __restrict__ cs,
                  const uint32_t* __restrict__ pktab, const float* __restrict__ q, float* __restrict__ out, int64_t n,
                  int m, int r, int cols_per_split, ConefMod mod, float alpha, ConefSeeds hs, int bx, int by)
{
    extern __shared__ float mfma_lds[];
    float* red = mfma_lds;                              // [kMfmaWaves][16][64]
    float* cells = mfma_lds + kMfmaWaves * 16 * 64;     // [32][w], MODE 2 only
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int lrow = lane & 31, half = lane >> 5;
    const int64_t row0 = (int64_t)bx * 32;
    const int64_t row = row0 + lrow < n ? row0 + lrow : n - 1;     // clamped for loads, stores are guarded
    const bool row_ok = row0 + lrow < n;
    const int w = (int)mod.w;
    if (MODE == 2) {
        for (int e = threadIdx.x; e < 32 * w; e += kMfmaThreads) {
            int a = e / w;
            int64_t rr = row0 + a < n ? row0 + a : n - 1;
            cells[e] = cs[rr * w + (e - a * w)];
        }
        __syncthreads();
    }
    const int c_begin = by * cols_per_split;
    const int c_end = c_begin + cols_per_split < m ? c_begin + cols_per_split : m;
    const bool rank_ok = lrow < r;
    conef_f16v acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float* xrow = x + row * m;
    const float* erow = MODE == 1 ? err + row * m : nullptr;
    // One stage = one 32-column block: every load of a stage is issued before the previous stage's
    // products, so a wave always has a block's worth of loads in flight while it multiplies.
    struct Stage {
        float xv[4][4], ev[4][4], qv[4][4];
        uint32_t pk[4][4];
    };
    auto load = [&](Stage& st, int cb) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = cb + 8 * u + 4 * half;
            const int cc = c < c_end ? c : c_begin;     // a valid quad, its products are zeroed
            float4 t = *reinterpret_cast<const float4*>(xrow + cc);
            st.xv[u][0] = t.x; st.xv[u][1] = t.y; st.xv[u][2] = t.z; st.xv[u][3] = t.w;
            if (MODE == 1) {
                float4 e = *reinterpret_cast<const float4*>(erow + cc);
                st.ev[u][0] = e.x; st.ev[u][1] = e.y; st.ev[u][2] = e.z; st.ev[u][3] = e.w;
            }
            if (MODE == 2) {
                if (pktab) {
                    uint4 p4 = *reinterpret_cast<const uint4*>(pktab + cc);
                    st.pk[u][0] = p4.x; st.pk[u][1] = p4.y; st.pk[u][2] = p4.z; st.pk[u][3] = p4.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) st.pk[u][j] = conef_bucket_sign(cc + j, mod, hs.a, hs.b, hs.sa, hs.sb);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) st.qv[u][j] = q[(int64_t)(cc + j) * r + (rank_ok ? lrow : 0)];
        }
    };
    auto compute = [&](Stage& st, int cb) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool ok = cb + 8 * u + 4 * half < c_end;
            if (MODE == 1) {
#pragma unroll
                for (int j = 0; j < 4; ++j) st.xv[u][j] = __fadd_rn(st.xv[u][j], st.ev[u][j]);
            }
            if (MODE == 2) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    st.xv[u][j] = __fadd_rn(st.xv[u][j], conef_query_term(cells[lrow * w + (st.pk[u][j] & 0x7fffffffu)],
                                                                          st.pk[u][j], alpha));
            }
            if (MODE != 0 && ok && row_ok)
                *reinterpret_cast<float4*>(xrow + cb + 8 * u + 4 * half) =
                    make_float4(st.xv[u][0], st.xv[u][1], st.xv[u][2], st.xv[u][3]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float a = ok ? st.xv[u][j] : 0.f;
                float b = (ok && rank_ok) ? st.qv[u][j] : 0.f;
                acc = conef_mfma32(a, b, acc);
            }
        }
    };
    constexpr int kStep = kMfmaWaves * 32;
    int cb = c_begin + wave * 32;
    if (cb < c_end) {
        Stage s0, s1;
        load(s0, cb);
        while (true) {
            int nb = cb + kStep;
            load(s1, nb < c_end ? nb : cb);             // past the end: a block already in cache, unused
            compute(s0, cb);
            if (nb >= c_end) break;
            cb = nb;
            nb = cb + kStep;
            load(s0, nb < c_end ? nb : cb);
            compute(s1, cb);
            if (nb >= c_end) break;
            cb = nb;
        }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) red[(wave * 16 + v) * 64 + lane] = acc[v];
    __syncthreads();
    float* dst = out + (int64_t)by * n * r;
    for (int e = threadIdx.x; e < 16 * 64; e += kMfmaThreads) {
        const int v = e >> 6, l = e & 63;
        float s = (red[e] + red[16 * 64 + e]) + (red[2 * 16 * 64 + e] + red[3 * 16 * 64 + e]);
        const int64_t i = row0 + conef_mfma_row(v, l);
        const int j = l & 31;
        if (i < n && j < r) dst[i * r + j] = s;
    }
}

template <int MODE>
__global__ void __launch_bounds__(kMfmaThreads)
psgd_mfma_mq_kernel(float* __restrict__ x, const float* __restrict__ err, const float* __restrict__ cs,
                    const uint32_t* __restrict__ pktab, const float* __restrict__ q, float* __restrict__ out, int64_t n,
                    int m, int r, int cols_per_split, ConefMod mod, float alpha, ConefSeeds hs)
{
    psgd_mfma_mq_body<MODE>(x, err, cs, pktab, q, out, n, m, r, cols_per_split, mod, alpha, hs, (int)blockIdx.x,
                            (int)blockIdx.y);
}

// -------------------------------------------------------------- Q = X^T P ----
// D[c][j] = sum_i X[i][c] P[i][j]: A[c][k] = X[i0 + k][c] is a row of X read along its columns, so
// the loads are contiguous as they come.  A wave owns 32 * V columns (V floats per lane: lane
// (q = l % 32, half) reads X[i][c0 + V*q .. + V) of row i = pair + half) and keeps V tiles, tile t
// for the columns c0 + V*q + t; a step consumes two rows.  The four waves of a workgroup split the
// rows of the slab, meet in LDS, and the slab's tile is stored (one slab) or left as a partial.
// Requires m % V == 0 and V*4-byte aligned x.
template <int V>
__device__ __forceinline__ void
psgd_mfma_mtp_body(const float* __restrict__ x, const float* __restrict__ p, float* __restrict__ out, int64_t n, int m,
                   int r, int rows_per_slab, int bx, int by)
{
    __shared__ float red[kMfmaWaves][16][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int lq = lane & 31, half = lane >> 5;
    const int c0 = bx * 32 * V;
    const int c = c0 + V * lq;
    const bool col_ok = c < m;
    const int cc = col_ok ? c : 0;
    const int64_t i0 = (int64_t)by * rows_per_slab;
    const int64_t i1 = i0 + rows_per_slab < n ? i0 + rows_per_slab : n;
    const bool rank_ok = lq < r;
    conef_f16v acc[V];
#pragma unroll
    for (int t = 0; t < V; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
    constexpr int U = V == 4 ? 4 : 8;                  // row pairs per stage
    struct Stage {
        float xv[U][V], pv[U];
    };
    auto load = [&](Stage& st, int64_t ib) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t i = ib + 2 * u + half;
            const int64_t ii = i < i1 ? i : i0;         // past the slab: a valid row, its products are zeroed
            const float* src = x + ii * m + cc;
            if constexpr (V == 4) {
                float4 t = *reinterpret_cast<const float4*>(src);
                st.xv[u][0] = t.x; st.xv[u][1] = t.y; st.xv[u][2] = t.z; st.xv[u][3] = t.w;
            } else if constexpr (V == 2) {
                float2 t = *reinterpret_cast<const float2*>(src);
                st.xv[u][0] = t.x; st.xv[u][1] = t.y;
            } else {
                st.xv[u][0] = *src;
            }
            st.pv[u] = p[ii * r + (rank_ok ? lq : 0)];
        }
    };
    auto compute = [&](Stage& st, int64_t ib) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool ok = ib + 2 * u + half < i1;
            const float b = (ok && rank_ok) ? st.pv[u] : 0.f;
#pragma unroll
            for (int t = 0; t < V; ++t) acc[t] = conef_mfma32((ok && col_ok) ? st.xv[u][t] : 0.f, b, acc[t]);
        }
    };
    constexpr int kStep = 2 * kMfmaWaves * U;
    int64_t ib = i0 + 2 * wave * U;
    if (ib < i1) {
        Stage s0, s1;
        load(s0, ib);
        while (true) {
            int64_t nb = ib + kStep;
            load(s1, nb < i1 ? nb : ib);
            compute(s0, ib);
            if (nb >= i1) break;
            ib = nb;
            nb = ib + kStep;
            load(s0, nb < i1 ? nb : ib);
            compute(s1, ib);
            if (nb >= i1) break;
            ib = nb;
        }
    }
    float* dst = out + (int64_t)by * m * r;
#pragma unroll
    for (int t = 0; t < V; ++t) {
        if (t) __syncthreads();
#pragma unroll
        for (int v = 0; v < 16; ++v) red[wave][v][lane] = acc[t][v];
        __syncthreads();
        for (int e = threadIdx.x; e < 16 * 64; e += kMfmaThreads) {
            const int v = e >> 6, l = e & 63;
            const float* rr = &red[0][0][0];
            float s = (rr[e] + rr[16 * 64 + e]) + (rr[2 * 16 * 64 + e] + rr[3 * 16 * 64 + e]);
            const int col = c0 + V * conef_mfma_row(v, l) + t;
            const int j = l & 31;
            if (col < m && j < r) dst[(int64_t)col * r + j] = s;
        }
    }
}

template <int V>
__global__ void __launch_bounds__(kMfmaThreads)
psgd_mfma_mtp_kernel(const float* __restrict__ x, const float* __restrict__ p, float* __restrict__ out, int64_t n, int m,
                     int r, int rows_per_slab)
{
    psgd_mfma_mtp_body<V>(x, p, out, n, m, r, rows_per_slab, (int)blockIdx.x, (int)blockIdx.y);
}

// ------------------------------------------------------------ M = P Q^T ----
// D[i][c] = sum_k P[i][k] Q[c][k] with K = R (16 or 32): R/2 steps per 32x32 tile.  Lane
// (t = l % 32, half) supplies k = half * R/2 + s at step s for both operands, so its slice of a
// row of P (and of Q) is R/2 consecutive floats: 16-byte loads.  A wave keeps the Q operand of its
// 32 columns in registers and walks the row tiles of its slab; a half-wave stores 128 contiguous
// bytes of a row of M.  MODE 1 also writes the residual E = X - M (X = what M held on entry).
template <int R, int MODE>
__device__ __forceinline__ void
psgd_mfma_pqt_body(float* __restrict__ x, float* __restrict__ err, const float* __restrict__ p,
                   const float* __restrict__ q, int64_t n, int m, int rows_per_slab, int bx, int by)
{
    constexpr int KS = R / 2;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int lt = lane & 31, half = lane >> 5;
    const int c = (bx * kMfmaWaves + wave) * 32 + lt;
    if ((bx * kMfmaWaves + wave) * 32 >= m) return;        // whole wave past the edge (no barriers below)
    const bool col_ok = c < m;
    float qb[KS];
    {
        const float* src = q + (int64_t)(col_ok ? c : m - 1) * R + half * KS;
#pragma unroll
        for (int s = 0; s < KS; s += 4) {
            float4 t = *reinterpret_cast<const float4*>(src + s);
            qb[s] = t.x; qb[s + 1] = t.y; qb[s + 2] = t.z; qb[s + 3] = t.w;
        }
    }
    const int64_t i0 = (int64_t)by * rows_per_slab;
    const int64_t i1 = i0 + rows_per_slab < n ? i0 + rows_per_slab : n;
    for (int64_t ib = i0; ib < i1; ib += 32) {
        float pa[KS], xv[16];
        {
            const int64_t i = ib + lt < n ? ib + lt : n - 1;
            const float* src = p + i * R + half * KS;
#pragma unroll
            for (int s = 0; s < KS; s += 4) {
                float4 t = *reinterpret_cast<const float4*>(src + s);
                pa[s] = t.x; pa[s + 1] = t.y; pa[s + 2] = t.z; pa[s + 3] = t.w;
            }
        }
        if (MODE == 1) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int64_t i = ib + conef_mfma_row(v, lane);
                xv[v] = x[(i < i1 ? i : i1 - 1) * m + (col_ok ? c : m - 1)];
            }
        }
        conef_f16v acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s) acc = conef_mfma32(pa[s], qb[s], acc);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t i = ib + conef_mfma_row(v, lane);
            if (i < i1 && col_ok) {
                if (MODE == 1) __builtin_nontemporal_store(__fsub_rn(xv[v], acc[v]), err + i * m + c);
                __builtin_nontemporal_store(acc[v], x + i * m + c);
            }
        }
    }
}

template <int R, int MODE>
__global__ void __launch_bounds__(kMfmaThreads)
psgd_mfma_pqt_kernel(float* __restrict__ x, float* __restrict__ err, const float* __restrict__ p,
                     const float* __restrict__ q, int64_t n, int m, int rows_per_slab)
{
    psgd_mfma_pqt_body<R, MODE>(x, err, p, q, n, m, rows_per_slab, (int)blockIdx.x, (int)blockIdx.y);
}
