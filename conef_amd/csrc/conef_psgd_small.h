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
//
// A matrix of more than kSmallWholeElements elements is dealt out by rows over several workgroups
// (`slices`), because everything a workgroup does for its rows - loading them, the products, the
// gathers of sketch cells, the list walks - runs on one CU.  Rows are independent in steps 2, 3 and 6;
// the slices meet twice: after step 3 every slice publishes its rows of the raw P and collects the
// others' (step 4 then runs on the whole P in every slice, the same arithmetic on the same values),
// and in step 5 every slice publishes its rows' share of X^T P and all add the shares up in slice
// order.  Published values are 8-byte records {launch tag, float}: one relaxed agent-scope load
// tells a reader whether the record is this launch's, so nothing is cleared between launches and no
// fence is needed.  The waits are bounded: a slice whose peers never show up (they were never
// resident) counts a give-up, leaves NaN in its rows of the result and ends.
#pragma once
#include "conef_device.h"
#include "conef_gs_lanes.h"      // gs_count_give_up
#include "conef_sketch_core.h"

constexpr int kSmallThreads = 1024;
constexpr int kSmallWaves = kSmallThreads / 64;
constexpr int kSmallMaxItems = 24;
constexpr size_t kSmallLdsLimit = 160 * 1024;     // all of a CU's LDS: one workgroup a CU
// One workgroup does all the work for its rows on one CU - their gathers of sketch cells, their list
// walks - where the separate launches spread a matrix over many: [32,288] takes 14 us in the kernel
// and [64,576] on one workgroup 33 us, against 24-30 us for a round of four launches.
// Matrices above kSmallWholeElements go over slices of about kSmallSliceElements ([64,576] over
// eight workgroups: 15 us against 33 us on one), at most kSmallMaxSlices of them; a launch holds at
// most kSmallMaxWgs workgroups, far fewer than the machine has CUs, so the slices of a matrix (which
// the launch's table keeps side by side) are resident together.
constexpr int64_t kSmallWholeElements = 10240;
constexpr int64_t kSmallSliceElements = 4608;
constexpr int kSmallMaxSlices = 16;
constexpr int kSmallMaxWgs = 128;
constexpr unsigned kSmallSpinLimit = 1u << 20;

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
    int slices;             // workgroups the rows are dealt over
    int rows_per;           // rows a slice (the last one may hold fewer)
    unsigned long long* recs;   // slices > 1: n*r records of the raw P, then slices * r*m records of the shares of X^T P
};

// Workgroup b of the grid runs on XCD b % 8 (the hardware deals workgroups out round robin), and
// on this part the workgroups of XCDs 4..7 start about 2 us after those of XCDs 0..3 (measured
// with timestamps: 0-3.2 us against 2.3-6.2 us for a grid of 58).  The slices of a matrix wait for
// each other twice, so a late slice holds up its whole matrix: the launch's table puts the slices
// on the early XCDs' workgroups and the matrices that go whole (and are done long before the
// sliced ones) on the late ones; slots that are left over end at once.
constexpr int kSmallMaxGrid = 2 * kSmallMaxWgs;
constexpr unsigned short kSmallIdle = 0xffffu;

struct SmallBatch {
    SmallItem item[kSmallMaxItems];
    unsigned short where[kSmallMaxGrid];     // item | slice << 8 of every workgroup of the grid, or kSmallIdle
    int count;
};

// Slices a matrix goes over, and rows a slice.
inline int small_slices(int64_t n, int64_t m, int* rows_per)
{
    int64_t s = n * m <= kSmallWholeElements ? 1 : (n * m + kSmallSliceElements - 1) / kSmallSliceElements;
    if (s > kSmallMaxSlices) s = kSmallMaxSlices;
    if (s > n) s = n;
    const int64_t rp = (n + s - 1) / s;
    *rows_per = (int)rp;
    return (int)((n + rp - 1) / rp);
}

inline int64_t small_record_count(int64_t n, int64_t m, int r, int slices) { return slices > 1 ? n * r + (int64_t)slices * r * m : 0; }

// A published float of this launch: waits (bounded) until the record carries the tag.
__device__ __forceinline__ float small_await(const unsigned long long* rec, unsigned long long first, unsigned tag, int* failed)
{
    unsigned long long v = first;
    unsigned spins = 0;
    while ((unsigned)(v >> 32) != tag) {
        ++spins;
        if (spins > kSmallSpinLimit || ((spins & 255u) == 0 && *(volatile int*)failed)) {
            *(volatile int*)failed = 1;
            return 0.f;
        }
        __builtin_amdgcn_s_sleep(1);
        v = __hip_atomic_load(rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return __uint_as_float((unsigned)v);
}

__device__ __forceinline__ void small_publish(unsigned long long* rec, float v, unsigned tag)
{
    __hip_atomic_store(rec, ((unsigned long long)tag << 32) | __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

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
// (nl: the rows a workgroup holds, n: the rows of the matrix, whose whole P every slice keeps)
__host__ __device__ inline size_t small_lds_floats(int nl, int n, int m, int rp, int w)
{
    const size_t rs = (size_t)small_row_stride(rp);
    return (((size_t)nl * m + 3) & ~(size_t)3) + (size_t)m * rs + (size_t)n * rs + 2 * (size_t)kSmallWaves * rp + 3 + 4 + (size_t)w + 1 + 3 +
           (w > 0 ? (((size_t)m + 3) & ~(size_t)3) : 0);
}

inline size_t small_lds_bytes(int nl, int n, int m, int rp, int w)
{
    return small_lds_floats(nl, n, m, rp, w) * 4 + (((size_t)m + 7) & ~(size_t)7) * 2;
}

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
psgd_small_round_body(const SmallItem& it, int slice, unsigned tag, int mq_mode, int pqt_mode, float alpha,
                      double one_minus_beta, float eps)
{
    constexpr int RS = RP > 1 ? RP + 1 : 1;
    constexpr int W = FAST ? 4 : 1;                        // elements a thread takes at a time
    extern __shared__ float small_lds[];
    const int rows = it.n, m = it.m, r = it.r, w = it.w;   // rows: of the whole matrix
    const int slices = it.slices;
    const int row0 = slice * it.rows_per;
    const int n = rows - row0 < it.rows_per ? rows - row0 : it.rows_per;       // this workgroup's rows
    const int total = n * m;
    float* const gx = it.x + (size_t)row0 * m;
    float* const gerr = it.err ? it.err + (size_t)row0 * m : nullptr;
    float* const gcs = it.cs ? it.cs + (size_t)row0 * w : nullptr;
    float* X = small_lds;
    float* Qs = X + ((total + 3) & ~3);
    float* Pall = Qs + m * RS;                             // the whole P
    float* Ps = Pall + row0 * RS;                          // this workgroup's rows of it
    float* red = Pall + rows * RS;
    int* failed = reinterpret_cast<int*>(small_lds + (((int)(red + 2 * kSmallWaves * RP - small_lds) + 3) & ~3));
    uint32_t* csr_l = reinterpret_cast<uint32_t*>(failed + 4);
    uint32_t* pk_l = csr_l + ((w + 1 + 3) & ~3);
    uint16_t* ent_l = reinterpret_cast<uint16_t*>(pk_l + (mq_mode == 2 ? ((m + 3) & ~3) : 0));
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (tid == 0) *failed = 0;

    // The first quads of the matrix (and of the dense error) are asked for before anything else:
    // they depend on nothing, and travel while Q and the tables arrive.
    constexpr int QH = 5;
    float4 gq_first[QH];
    float ev_first[QH][4];
    if (FAST) {
        const int groups = total >> 2, width = m >> 2;
        SmallWalk pre(tid, width);
#pragma unroll
        for (int u = 0; u < QH; ++u) {
            // (a slot past the end asks for nothing: a request is a request, whatever its address)
            if (tid + u * kSmallThreads < groups) {
                const int e = (pre.row * width + pre.col) * 4;
                gq_first[u] = *reinterpret_cast<const float4*>(gx + e);
                if (mq_mode == 1) ld4s(gerr + e, ev_first[u]);
            }
            pre.next(width);
        }
    }

    // ---- 1. Q into LDS (padding columns zero); the sketch's tables ride along
    {
        constexpr int U = 4;
        const int count = m * r;
        for (int e0 = tid; e0 < count; e0 += U * kSmallThreads) {
            float t[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                t[u] = 0.f;
                if (e0 + u * kSmallThreads < count) t[u] = it.q[e0 + u * kSmallThreads];
            }
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
        // a matrix has at most 40960 elements, ten quads a thread: five are requested (the matrix's own
        // values at the kernel's start, the sketch cells now that the table is there), Q is orthogonalised
        // while they travel, then the other five (all ten at once would not fit the registers)
        const int groups = total >> 2, width = m >> 2;
        SmallWalk issue(tid, width), finish(tid, width);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float4 gq[QH];
            float ev[QH][4];
#pragma unroll
            for (int u = 0; u < QH; ++u) {
                const bool in = tid + (half * QH + u) * kSmallThreads < groups;
                const int row = issue.row, col = issue.col;
                const int e = (row * width + col) * 4;
                if (half == 0) {
                    gq[u] = gq_first[u];
                    if (mq_mode == 1) {
#pragma unroll
                        for (int k = 0; k < 4; ++k) ev[u][k] = ev_first[u][k];
                    }
                } else if (in) {
                    gq[u] = *reinterpret_cast<const float4*>(gx + e);
                    if (mq_mode == 1) ld4s(gerr + e, ev[u]);
                }
                if (mq_mode == 2 && in) {
                    const uint4 pw = *reinterpret_cast<const uint4*>(pk_l + col * 4);
                    const float* cells = gcs + row * w;
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
                const int row = at.row, col = at.col;
                where[u] = in ? row * m + col : -1;
                if (in) {
                    gv[u] = gx[where[u]];
                    if (mq_mode == 1) ev[u] = gerr[where[u]];
                    if (mq_mode == 2) {
                        pw[u] = pk_l[col];
                        ev[u] = gcs[row * w + (int)(pw[u] & 0x7fffffffu)];
                    }
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
            if (lane == 0) {
                Ps[row * RS + c] = s;
                if (slices > 1 && c < r) small_publish(it.recs + (size_t)(row0 + row) * r + c, s, tag);
            }
        }
    }
    if (slices > 1) {
        // the other slices' rows of the raw P
        for (int e = tid; e < rows * r; e += kSmallThreads) {
            const int row = e / r, c = e - row * r;
            if (row >= row0 && row < row0 + n) continue;
            const unsigned long long* rec = it.recs + e;
            Pall[row * RS + c] = small_await(rec, __hip_atomic_load(rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), tag, failed);
        }
        if (r < RP)
            for (int e = tid; e < rows * (RP - r); e += kSmallThreads) {
                const int row = e / (RP - r);
                if (row < row0 || row >= row0 + n) Pall[row * RS + r + (e - row * (RP - r))] = 0.f;
            }
    }
    __syncthreads();
    // ---- 4. (on the whole P, in every slice alike)
    small_gram_schmidt<RP>(Pall, rows, r, eps, red);

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
        if (slices > 1) {
            // this slice's share of X^T P out, then all shares added up in slice order: the same sum in
            // every slice.  A thread publishes and collects the same entries, so no barrier in between.
            unsigned long long* shares = it.recs + (size_t)rows * r;
            const int count = r * m;
            for (int e = tid; e < count; e += kSmallThreads) small_publish(shares + (size_t)slice * count + e, QT[e], tag);
            // (a thread takes two entries at a time and four slices' shares of each: eight requests in flight)
            for (int e0 = tid; e0 < count; e0 += 2 * kSmallThreads) {
                const int e1 = e0 + kSmallThreads;
                const bool two = e1 < count;
                float sum0 = 0.f, sum1 = 0.f;
                for (int g0 = 0; g0 < slices; g0 += 4) {
                    unsigned long long f0[4], f1[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int g = g0 + u;
                        const bool ask = g < slices && g != slice;
                        const unsigned long long* at = shares + (size_t)(ask ? g : slice) * count;
                        f0[u] = ask ? __hip_atomic_load(at + e0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
                        f1[u] = ask && two ? __hip_atomic_load(at + e1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int g = g0 + u;
                        if (g < slices) {
                            const unsigned long long* at = shares + (size_t)g * count;
                            const float v0 = g == slice ? QT[e0] : small_await(at + e0, f0[u], tag, failed);
                            sum0 = g == 0 ? v0 : __fadd_rn(sum0, v0);
                            if (two) {
                                const float v1 = g == slice ? QT[e1] : small_await(at + e1, f1[u], tag, failed);
                                sum1 = g == 0 ? v1 : __fadd_rn(sum1, v1);
                            }
                        }
                    }
                }
                QT[e0] = sum0;
                if (two) QT[e1] = sum1;
            }
            __syncthreads();
        }
        if (slice == 0)
            for (int e = tid; e < m * r; e += kSmallThreads) {
                const int col = e / r, c = e - col * r;
                it.q[e] = QT[c * m + col];
            }
    }
    for (int e = tid; e < n * r; e += kSmallThreads) {
        const int row = e / r;
        it.p[(size_t)row0 * r + e] = Ps[row * RS + (e - row * r)];
    }

    // the old cells the residual will be added onto are requested now and travel during step 6
    constexpr int kCells = 20;
    const int pairs = pqt_mode == 2 ? n * w : 0;
    float aux[kCells];
#pragma unroll
    for (int u = 0; u < kCells; ++u) {
        aux[u] = 0.f;
        if (tid + u * kSmallThreads < pairs) aux[u] = gcs[tid + u * kSmallThreads];
    }

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
                st4s(gx + e, mh);
                st4s(X + e, res);
                if (pqt_mode == 1) st4s(gerr + e, res);
            } else {
                gx[e] = mh[0];
                X[e] = res[0];
                if (pqt_mode == 1) gerr[e] = res[0];
            }
            at.next(width);
        }
    }
    __syncthreads();
    if (*failed) {
        // a peer never published: what this slice computed is not the round's result, and must not pass for it
        if (tid == 0) gs_count_give_up();
        for (int e = tid; e < total; e += kSmallThreads) gx[e] = __builtin_nanf("");
        return;
    }
    if (pqt_mode != 2) return;
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
            gcs[idx] = acc;
            at.next(w);
        };
#pragma unroll
        for (int u = 0; u < kCells; ++u) {
            const int idx = tid + u * kSmallThreads;
            if (idx < pairs) one(idx, aux[u]);
        }
        for (int idx = tid + kCells * kSmallThreads; idx < pairs; idx += kSmallThreads) one(idx, gcs[idx]);
    }
}

template <int RP>
__global__ void __launch_bounds__(kSmallThreads)
psgd_small_round_kernel(SmallBatch batch, unsigned tag, int mq_mode, int pqt_mode, float alpha, double one_minus_beta, float eps)
{
    const unsigned where = batch.where[blockIdx.x];
    if (where == kSmallIdle) return;
    const SmallItem& it = batch.item[where & 0xffu];
    const int slice = (int)(where >> 8);
    if (it.fast) psgd_small_round_body<RP, true>(it, slice, tag, mq_mode, pqt_mode, alpha, one_minus_beta, eps);
    else psgd_small_round_body<RP, false>(it, slice, tag, mq_mode, pqt_mode, alpha, one_minus_beta, eps);
}
