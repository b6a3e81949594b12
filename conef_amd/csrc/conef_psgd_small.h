// A whole PowerSGD round of a bucket of SMALL matrices in one launch.
//
// The matrices of a bucket are independent (powerSGD_hook.py:473-564 loops over them), and a bucket
// of matrices of a few thousand elements each is, as separate launches
// per stage (P = M Q, orthogonalise, Q = M^T P, M = P Q^T with the residual), nothing
// but launch latency.  Here one workgroup takes one matrix through the whole round, with the
// matrix, both factors and the bucket lists of its sketch resident in LDS and workgroup barriers
// between the stages, in the reference's order:
//
//   1. Q <- orthogonalise(Q)                              (:475-477; a fresh Q is orthogonalised too, :494)
//   2. X = M + e, the remembered error: nothing, the dense error tensor, or alpha * unsketch(cs)
//                                                          (:361 / hPowerSGD_hook.py:399 / :409)
//   3. P = X Q                                             (:498)
//   4. P <- orthogonalise(P)                               (:527-528)
//   5. Q = X^T P                                           (:532)
//   6. M = P Q^T; the residual X - M goes to the dense error or into the sketch, a bucket's terms
//      in ascending column order                           (:551, :558 / :563-564)
//
// Global memory is touched once per operand: the gradient is read and the low-rank product written,
// the sketch cells are gathered and rewritten, P and Q are read and written.
#pragma once
#include "conef_device.h"
#include "conef_sketch_core.h"

constexpr int kSmallThreads = 1024;
constexpr int kSmallWaves = kSmallThreads / 64;
constexpr int kSmallMaxItems = 24;
constexpr size_t kSmallLdsLimit = 160 * 1024;     // all of a CU's LDS: one workgroup a CU
// One workgroup does all of a matrix's work on one CU - its gathers of sketch cells, its list walks -
// where the separate launches spread a matrix over many.  Up to about this many elements the
// launches saved outweigh that ([32,288]: 16 us for the round against 24 us of four launches;
// [64,576], 36864 elements: 32 us); a bucket with a larger matrix takes the separate launches.
constexpr int64_t kSmallMaxElements = 16384;

struct SmallItem {
    float* x;               // [n,m] gradient in, P Q^T out
    float* err;             // dense error [n,m] (read when mq_mode is 1, written when pqt_mode is 1)
    float* cs;              // sketch [n,w], updated in place (modes 2)
    const uint32_t* csr;    // row-list plan of the sketch: first list entry of bucket j, [w+1]
    const uint16_t* ent;    //   column | sign bit << 15, buckets ascending, columns ascending, [m]
    const uint32_t* pk;     //   bucket | sign bit << 31 of every column, [m]
    float* p;               // [n,r]
    float* q;               // [m,r]
    int n, m, r, w;
    int fast;               // m % 4 == 0 and x (and err, where used) 16-byte aligned: the element-wise phases go by column quads
};

struct SmallBatch {
    SmallItem item[kSmallMaxItems];
};

__device__ __forceinline__ void ld4s(const float* p, float* v)
{
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void st4s(float* p, const float* v)
{
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

__host__ __device__ inline int small_row_stride(int rp) { return rp > 1 ? rp + 1 : 1; }   // odd: lanes over rows hit distinct banks

// floats of LDS before the (16-bit) bucket lists: matrix, Q, P, two sets of per-wave partial sums, and
// with a sketch (w > 0) its list offsets and column table
__host__ __device__ inline size_t small_lds_floats(int n, int m, int rp, int w)
{
    const size_t rs = (size_t)small_row_stride(rp);
    return (((size_t)n * m + 3) & ~(size_t)3) + (size_t)m * rs + (size_t)n * rs + 2 * (size_t)kSmallWaves * rp + (size_t)w + 1 + 3 +
           (w > 0 ? (((size_t)m + 3) & ~(size_t)3) : 0);
}

inline size_t small_lds_bytes(int n, int m, int rp, int w) { return small_lds_floats(n, m, rp, w) * 4 + (((size_t)m + 7) & ~(size_t)7) * 2; }

// In-place Gram-Schmidt (powerSGD_hook.py:21-43) of a [rows, r] matrix in LDS (row stride RS), all
// threads of the workgroup.  A thread keeps to its own rows, so a column step is one reduction of
// (||col||^2, col . later columns) over the workgroup; the projection coefficients of the
// normalised column are those dot products times 1 / norm.  A zero column at eps = 0 turns to NaN
// and takes the later columns with it, as 0 / 0 does in the reference.
template <int RP>
__device__ __forceinline__ void small_gram_schmidt(float* a, int rows, int r, float eps, float* red)
{
    constexpr int RS = RP > 1 ? RP + 1 : 1;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i < RP; ++i) {
        if (i < r) {
            float d[RP];
#pragma unroll
            for (int c = 0; c < RP; ++c) d[c] = 0.f;
            for (int row = threadIdx.x; row < rows; row += kSmallThreads) {
                const float ai = a[row * RS + i];
#pragma unroll
                for (int c = i; c < RP; ++c) d[c] = fmaf(ai, a[row * RS + c], d[c]);
            }
            float* mine = red + (i & 1) * kSmallWaves * RP;
#pragma unroll
            for (int c = i; c < RP; ++c) {
                const float s = conef_wave_sum(d[c]);
                if (lane == 0) mine[wave * RP + c] = s;
            }
            __syncthreads();
            float tot[RP];
#pragma unroll
            for (int c = i; c < RP; ++c) {
                float s = 0.f;
#pragma unroll
                for (int v = 0; v < kSmallWaves; ++v) s += mine[v * RP + c];       // the same order in every thread
                tot[c] = s;
            }
            const float nrm = sqrtf(tot[i]);
            const float inv = 1.f / (eps == 0.f ? nrm : nrm + eps);
            for (int row = threadIdx.x; row < rows; row += kSmallThreads) {
                const float ci = __fmul_rn(a[row * RS + i], inv);
                a[row * RS + i] = ci;
#pragma unroll
                for (int c = i + 1; c < RP; ++c)
                    if (c < r) a[row * RS + c] = fmaf(-__fmul_rn(tot[c], inv), ci, a[row * RS + c]);
            }
        }
    }
    __syncthreads();
}

// (row, column) of the flat element index a thread starts at and the step that takes it to its
// next one, kSmallThreads further on: one division a thread and phase instead of one per element.
struct SmallWalk {
    int row, col, drow, dcol;
    __device__ __forceinline__ SmallWalk(int first, int width)
    {
        row = first / width;
        col = first - row * width;
        drow = kSmallThreads / width;
        dcol = kSmallThreads - drow * width;
    }
    __device__ __forceinline__ void next(int width)
    {
        row += drow;
        col += dcol;
        if (col >= width) {
            col -= width;
            ++row;
        }
    }
};

// mq_mode: 0 no error, 1 dense error, 2 count sketch.  pqt_mode: 0 nothing kept, 1 dense residual to
// `err`, 2 residual into the sketch.  FAST: the item's `fast`.
template <int RP, bool FAST>
__device__ __forceinline__ void
psgd_small_round_body(const SmallItem& it, int mq_mode, int pqt_mode, float alpha, double one_minus_beta, float eps)
{
    constexpr int RS = RP > 1 ? RP + 1 : 1;
    constexpr int W = FAST ? 4 : 1;                        // elements a thread takes at a time
    extern __shared__ float small_lds[];
    const int n = it.n, m = it.m, r = it.r, w = it.w;
    const int total = n * m;
    float* X = small_lds;
    float* Qs = X + ((total + 3) & ~3);
    float* Ps = Qs + m * RS;
    float* red = Ps + n * RS;
    uint32_t* csr_l = reinterpret_cast<uint32_t*>(red + 2 * kSmallWaves * RP);
    uint32_t* pk_l = csr_l + ((w + 1 + 3) & ~3);
    uint16_t* ent_l = reinterpret_cast<uint16_t*>(pk_l + (mq_mode == 2 ? ((m + 3) & ~3) : 0));
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;

    // ---- 1. Q into LDS (padding columns zero); the sketch's tables ride along
    {
        constexpr int U = 4;
        const int count = m * r;
        for (int e0 = tid; e0 < count; e0 += U * kSmallThreads) {
            float t[U];
#pragma unroll
            for (int u = 0; u < U; ++u) t[u] = it.q[e0 + u * kSmallThreads < count ? e0 + u * kSmallThreads : count - 1];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int e = e0 + u * kSmallThreads;
                if (e < count) {
                    const int row = e / r;
                    Qs[row * RS + (e - row * r)] = t[u];
                }
            }
        }
        if (r < RP)
            for (int e = tid; e < m * (RP - r); e += kSmallThreads) {
                const int row = e / (RP - r);
                Qs[row * RS + r + (e - row * (RP - r))] = 0.f;
            }
    }
    if (mq_mode == 2) {
        for (int j = tid; j <= w; j += kSmallThreads) csr_l[j] = it.csr[j];
        for (int e = tid; e < m; e += kSmallThreads) {
            ent_l[e] = it.ent[e];
            pk_l[e] = it.pk[e];
        }
    }
    __syncthreads();
    // ---- 2. X = M + remembered error, into LDS.  With 16-byte accesses every load of the matrix
    // (and of the dense error, or every gather of a sketch cell) is requested before the first is
    // used, and Q is orthogonalised while they travel: the matrix is one trip to memory.
    if (FAST) {
        // a matrix has at most 40960 elements, ten quads a thread: five are requested, Q is orthogonalised
        // while they travel, then the other five (all ten at once would not fit the registers)
        constexpr int QH = 5;
        const int groups = total >> 2, width = m >> 2;
        SmallWalk issue(tid, width), finish(tid, width);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float4 gq[QH];
            float ev[QH][4];
#pragma unroll
            for (int u = 0; u < QH; ++u) {
                const bool in = tid + (half * QH + u) * kSmallThreads < groups;
                const int row = in ? issue.row : 0, col = in ? issue.col : 0;
                const int e = (row * width + col) * 4;
                gq[u] = *reinterpret_cast<const float4*>(it.x + e);
                if (mq_mode == 1) ld4s(it.err + e, ev[u]);
                if (mq_mode == 2) {
                    const uint4 pw = *reinterpret_cast<const uint4*>(pk_l + col * 4);
                    const float* cells = it.cs + row * w;
                    ev[u][0] = cells[pw.x & 0x7fffffffu];
                    ev[u][1] = cells[pw.y & 0x7fffffffu];
                    ev[u][2] = cells[pw.z & 0x7fffffffu];
                    ev[u][3] = cells[pw.w & 0x7fffffffu];
                }
                issue.next(width);
            }
            if (half == 0) {
                small_gram_schmidt<RP>(Qs, m, r, eps, red);
            }
#pragma unroll
            for (int u = 0; u < QH; ++u) {
                if (tid + (half * QH + u) * kSmallThreads < groups) {
                    float xv[4] = {gq[u].x, gq[u].y, gq[u].z, gq[u].w};
                    if (mq_mode == 1) {
#pragma unroll
                        for (int k = 0; k < 4; ++k) xv[k] = __fadd_rn(xv[k], ev[u][k]);
                    }
                    if (mq_mode == 2) {
                        const uint4 pw = *reinterpret_cast<const uint4*>(pk_l + finish.col * 4);
                        xv[0] = __fadd_rn(xv[0], conef_query_term(ev[u][0], pw.x, alpha));
                        xv[1] = __fadd_rn(xv[1], conef_query_term(ev[u][1], pw.y, alpha));
                        xv[2] = __fadd_rn(xv[2], conef_query_term(ev[u][2], pw.z, alpha));
                        xv[3] = __fadd_rn(xv[3], conef_query_term(ev[u][3], pw.w, alpha));
                    }
                    st4s(X + (finish.row * width + finish.col) * 4, xv);
                }
                finish.next(width);
            }
        }
    } else {
        constexpr int kAhead = 8;
        SmallWalk at(tid, m);
        for (int g0 = tid; g0 < total; g0 += kAhead * kSmallThreads) {
            float gv[kAhead], ev[kAhead];
            uint32_t pw[kAhead];
            int where[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const bool in = g0 + u * kSmallThreads < total;
                const int row = in ? at.row : 0, col = in ? at.col : 0;
                where[u] = in ? row * m + col : -1;
                const int e = in ? where[u] : 0;
                gv[u] = it.x[e];
                if (mq_mode == 1) ev[u] = it.err[e];
                if (mq_mode == 2) {
                    pw[u] = pk_l[col];
                    ev[u] = it.cs[row * w + (int)(pw[u] & 0x7fffffffu)];
                }
                at.next(m);
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                if (where[u] < 0) continue;
                float xv = gv[u];
                if (mq_mode == 1) xv = __fadd_rn(xv, ev[u]);
                if (mq_mode == 2) xv = __fadd_rn(xv, conef_query_term(ev[u], pw[u], alpha));
                X[where[u]] = xv;
            }
        }
        small_gram_schmidt<RP>(Qs, m, r, eps, red);
    }
    __syncthreads();

    // ---- 3. P = X Q: a wave takes rows, its lanes the columns
    for (int row = wave; row < n; row += kSmallWaves) {
        float acc[RP];
#pragma unroll
        for (int c = 0; c < RP; ++c) acc[c] = 0.f;
        const float* xr = X + row * m;
        for (int col = lane; col < m; col += 64) {
            const float xv = xr[col];
#pragma unroll
            for (int c = 0; c < RP; ++c) acc[c] = fmaf(xv, Qs[col * RS + c], acc[c]);
        }
#pragma unroll
        for (int c = 0; c < RP; ++c) {
            const float s = conef_wave_sum(acc[c]);
            if (lane == 0) Ps[row * RS + c] = s;
        }
    }
    __syncthreads();
    // ---- 4.
    small_gram_schmidt<RP>(Ps, n, r, eps, red);

    // ---- 5. Q = X^T P, left in LDS column by column (QT[c][col]: the last step reads quads of it) in
    // the place of the old Q, which nobody needs any more.  The columns go over the lanes; a matrix
    // narrower than the workgroup splits its rows over groups of threads, whose sums are folded in
    // group order.
    float* QT = Qs;
    {
        const int groups = m >= kSmallThreads ? 1 : (kSmallThreads / m < 8 ? kSmallThreads / m : 8);
        float acc[RP];
        if (groups > 1) {
            const int grp = tid / m, col = tid - grp * m;
#pragma unroll
            for (int c = 0; c < RP; ++c) acc[c] = 0.f;
            if (grp < groups) {
                for (int row = grp; row < n; row += groups) {
                    const float xv = X[row * m + col];
#pragma unroll
                    for (int c = 0; c < RP; ++c) acc[c] = fmaf(xv, Ps[row * RS + c], acc[c]);
                }
            }
            for (int g = 0; g < groups; ++g) {
                if (grp == g) {
#pragma unroll
                    for (int c = 0; c < RP; ++c) QT[c * m + col] = g == 0 ? acc[c] : __fadd_rn(QT[c * m + col], acc[c]);
                }
                __syncthreads();
            }
        } else {
            // (the old Q is read by nobody after step 3, and every thread writes only its own columns)
            for (int c0 = tid; c0 < m; c0 += kSmallThreads) {
#pragma unroll
                for (int c = 0; c < RP; ++c) acc[c] = 0.f;
                for (int row = 0; row < n; ++row) {
                    const float xv = X[row * m + c0];
#pragma unroll
                    for (int c = 0; c < RP; ++c) acc[c] = fmaf(xv, Ps[row * RS + c], acc[c]);
                }
#pragma unroll
                for (int c = 0; c < RP; ++c) QT[c * m + c0] = acc[c];
            }
            __syncthreads();
        }
        for (int e = tid; e < m * r; e += kSmallThreads) {
            const int col = e / r, c = e - col * r;
            it.q[e] = QT[c * m + col];
        }
    }
    for (int e = tid; e < n * r; e += kSmallThreads) {
        const int row = e / r;
        it.p[e] = Ps[row * RS + (e - row * r)];
    }

    // the old cells the residual will be added onto are requested now and travel during step 6
    constexpr int kCells = 20;
    const int pairs = pqt_mode == 2 ? n * w : 0;
    float aux[kCells];
#pragma unroll
    for (int u = 0; u < kCells; ++u)
        aux[u] = pairs > 0 ? it.cs[tid + u * kSmallThreads < pairs ? tid + u * kSmallThreads : pairs - 1] : 0.f;

    // ---- 6. M = P Q^T, residual kept in LDS (and, dense error feedback, written out)
    {
        const int groups = FAST ? total >> 2 : total, width = FAST ? m >> 2 : m;
        SmallWalk at(tid, width);
        for (int g0 = tid; g0 < groups; g0 += kSmallThreads) {
            const int e = (at.row * width + at.col) * W;
            float pr[RP];
#pragma unroll
            for (int c = 0; c < RP; ++c) pr[c] = Ps[at.row * RS + c];
            float xv[W], mh[W], res[W];
            if (FAST) ld4s(X + e, xv);
            else xv[0] = X[e];
#pragma unroll
            for (int k = 0; k < W; ++k) mh[k] = 0.f;
#pragma unroll
            for (int c = 0; c < RP; ++c) {
                if (c < r) {
                    float qv[W];
                    if (FAST) ld4s(QT + c * m + at.col * 4, qv);
                    else qv[0] = QT[c * m + at.col];
#pragma unroll
                    for (int k = 0; k < W; ++k) mh[k] = fmaf(pr[c], qv[k], mh[k]);
                }
            }
#pragma unroll
            for (int k = 0; k < W; ++k) res[k] = __fsub_rn(xv[k], mh[k]);
            if (FAST) {
                st4s(it.x + e, mh);
                st4s(X + e, res);
                if (pqt_mode == 1) st4s(it.err + e, res);
            } else {
                it.x[e] = mh[0];
                X[e] = res[0];
                if (pqt_mode == 1) it.err[e] = res[0];
            }
            at.next(width);
        }
    }
    if (pqt_mode != 2) return;
    __syncthreads();
    // the residual into the sketch: one thread per (row, bucket), the bucket's columns ascending
    // (DenseCS.update, CountSketch.py:27-67: every term's decay reads the cell as it was before)
    {
        SmallWalk at(tid, w);
        auto one = [&](int idx, float old) {
            const int j = at.col;
            const double decay = __dmul_rn(one_minus_beta, (double)old);
            const float* xr = X + at.row * m;
            float acc = old;
            for (uint32_t e = csr_l[j]; e < csr_l[j + 1]; ++e) {
                const uint32_t en = ent_l[e];
                const uint32_t flip = ((~en) & 0x8000u) << 16;         // sign bit clear (-1): flip the float's sign
                const double sv = (double)__uint_as_float(__float_as_uint(xr[en & 0x7fffu]) ^ flip);
                acc = __fadd_rn(acc, (float)__dsub_rn(sv, decay));
            }
            it.cs[idx] = acc;
            at.next(w);
        };
#pragma unroll
        for (int u = 0; u < kCells; ++u) {
            const int idx = tid + u * kSmallThreads;
            if (idx < pairs) one(idx, aux[u]);
        }
        for (int idx = tid + kCells * kSmallThreads; idx < pairs; idx += kSmallThreads) one(idx, it.cs[idx]);
    }
}

template <int RP>
__global__ void __launch_bounds__(kSmallThreads)
psgd_small_round_kernel(SmallBatch batch, int mq_mode, int pqt_mode, float alpha, double one_minus_beta, float eps)
{
    const SmallItem& it = batch.item[blockIdx.x];
    if (it.fast) psgd_small_round_body<RP, true>(it, mq_mode, pqt_mode, alpha, one_minus_beta, eps);
    else psgd_small_round_body<RP, false>(it, mq_mode, pqt_mode, alpha, one_minus_beta, eps);
}
