// PowerSGD inner-loop kernels (gfx950) and their C entry points.
//
// Reference semantics: communication/powerSGD_hook.py:12-44 (_orthogonalize), :498 (P = M Q),
// :532 (Q = M^T P), :551 (M = P Q^T), :361/:558 (dense error feedback), :409/:563-564 (count-sketched
// error feedback).  All matrices are row-major fp32: M [n,m], Q [m,r], P [n,r], r <= 32.
//
// At the ranks gradient compression uses (1..8) these products move 4 bytes of M per 2r flops, far
// below the fp32 ridge of the machine, so they are written as streaming kernels: M is read exactly
// once per product, the rank dimension lives in registers, and the error-feedback add (before the
// first product) and the residual (after the last) are fused into the passes that touch M anyway.
#include "conef_device.h"
#include "conef_sketch_core.h"

namespace {

constexpr int kMaxRank = 32;

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- P = X Q ----
// MODE 0: X = M as stored.  MODE 1: X = M + E (dense error), written back into M.
// MODE 2: X = M + alpha * unsketch(cs), written back into M (DenseCS.query fused).
// A workgroup owns RB consecutive rows and all columns; a thread owns columns tid, tid+256, ...
// and keeps RB x RP partial sums, reduced over the workgroup at the end in a fixed order.
template <int RB, int RP, int MODE>
__global__ void __launch_bounds__(256)
psgd_mq_kernel(float* __restrict__ x, const float* __restrict__ err, const float* __restrict__ cs,
               const float* __restrict__ q, float* __restrict__ p, int64_t n, int64_t m, int r, ConefMod mod,
               float alpha, ConefSeeds hs)
{
    __shared__ float red[4][RB * RP];
    const int64_t row0 = (int64_t)blockIdx.x * RB;
    float acc[RB][RP];
#pragma unroll
    for (int a = 0; a < RB; ++a)
#pragma unroll
        for (int c = 0; c < RP; ++c) acc[a][c] = 0.f;

    for (int64_t k = threadIdx.x; k < m; k += 256) {
        float qk[RP];
#pragma unroll
        for (int c = 0; c < RP; ++c) qk[c] = c < r ? q[k * r + c] : 0.f;
        uint32_t pk = 0;
        if (MODE == 2) pk = conef_bucket_sign((int32_t)k, mod, hs.a, hs.b, hs.sa, hs.sb);
#pragma unroll
        for (int a = 0; a < RB; ++a) {
            int64_t row = row0 + a;
            if (row < n) {
                float v = x[row * m + k];
                if (MODE == 1) {
                    v = __fadd_rn(v, err[row * m + k]);
                    x[row * m + k] = v;
                } else if (MODE == 2) {
                    float cell = cs[row * (int64_t)mod.w + (pk & 0x7fffffffu)];
                    v = __fadd_rn(v, conef_query_term(cell, pk, alpha));
                    x[row * m + k] = v;
                }
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
            if (lane == 0) red[wave][a * RP + c] = s;
        }
    __syncthreads();
    if (threadIdx.x < RB * RP) {
        int a = threadIdx.x / RP, c = threadIdx.x % RP;
        int64_t row = row0 + a;
        if (row < n && c < r)
            p[row * r + c] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
    }
}

// -------------------------------------------------------------- Q = X^T P ----
// A thread owns one column of X; the workgroup walks a slab of rows.  With one slab the result is
// stored, with several the slabs meet through float atomics on a zeroed Q.
template <int RP>
__global__ void __launch_bounds__(256)
psgd_mtp_kernel(const float* __restrict__ x, const float* __restrict__ p, float* q, int64_t n, int64_t m, int r,
                int64_t rows_per_slab, int use_atomics)
{
    int64_t k = blockIdx.x * (int64_t)256 + threadIdx.x;
    if (k >= m) return;
    int64_t i0 = (int64_t)blockIdx.y * rows_per_slab;
    int64_t i1 = i0 + rows_per_slab < n ? i0 + rows_per_slab : n;
    float acc[RP];
#pragma unroll
    for (int c = 0; c < RP; ++c) acc[c] = 0.f;
    for (int64_t i = i0; i < i1; ++i) {
        float v = x[i * m + k];
        const float* pi = p + i * r;
#pragma unroll
        for (int c = 0; c < RP; ++c)
            if (c < r) acc[c] = fmaf(v, pi[c], acc[c]);
    }
#pragma unroll
    for (int c = 0; c < RP; ++c)
        if (c < r) {
            if (use_atomics) unsafeAtomicAdd(q + k * r + c, acc[c]);
            else q[k * r + c] = acc[c];
        }
}

__global__ void zero_kernel(float* x, int64_t count)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) x[i] = 0.f;
}

// ------------------------------------------------------------ M = P Q^T ----
// MODE 0: write M.  MODE 1: also write the dense residual E = X - M (X = what M held on entry).
template <int RP, int MODE>
__global__ void __launch_bounds__(256)
psgd_pqt_kernel(float* __restrict__ x, float* __restrict__ err, const float* __restrict__ p,
                const float* __restrict__ q, int64_t n, int64_t m, int r, int64_t rows_per_slab)
{
    int64_t k = blockIdx.x * (int64_t)256 + threadIdx.x;
    if (k >= m) return;
    float qk[RP];
#pragma unroll
    for (int c = 0; c < RP; ++c) qk[c] = c < r ? q[k * r + c] : 0.f;
    int64_t i0 = (int64_t)blockIdx.y * rows_per_slab;
    int64_t i1 = i0 + rows_per_slab < n ? i0 + rows_per_slab : n;
    for (int64_t i = i0; i < i1; ++i) {
        const float* pi = p + i * r;
        float mh = 0.f;
#pragma unroll
        for (int c = 0; c < RP; ++c)
            if (c < r) mh = fmaf(pi[c], qk[c], mh);
        if (MODE == 1) err[i * m + k] = __fsub_rn(x[i * m + k], mh);
        x[i * m + k] = mh;
    }
}

// Front for the sketch back end: the value to sketch is the residual X - P Q^T, and M is
// overwritten with P Q^T on the way (powerSGD_hook.py:551,563-564).
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
// In place on a row-major [rows, r] matrix; one workgroup per matrix.  Column by column:
// col /= ||col|| (+eps when eps != 0), then every later column loses its projection on col
// (powerSGD_hook.py:21-43).  Each thread keeps to its own rows, so the only exchange per column
// is one workgroup reduction of (||col||^2, col . later columns); the projection coefficients of
// the normalised column are those dot products divided by the norm.
template <int RP>
__global__ void __launch_bounds__(1024)
gram_schmidt_kernel(float* __restrict__ a, int64_t rows, int r, float eps)
{
    __shared__ float red[16][RP];
    __shared__ float tot[RP];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int i = 0; i < r; ++i) {
        float acc[RP];
#pragma unroll
        for (int c = 0; c < RP; ++c) acc[c] = 0.f;
        for (int64_t k = threadIdx.x; k < rows; k += 1024) {
            const float* row = a + k * r;
            float ci = row[i];
#pragma unroll
            for (int c = 0; c < RP; ++c)
                if (i + c < r) acc[c] = fmaf(ci, row[i + c], acc[c]);
        }
#pragma unroll
        for (int c = 0; c < RP; ++c) {
            float s = conef_wave_sum(acc[c]);
            if (lane == 0) red[wave][c] = s;
        }
        __syncthreads();
        if (threadIdx.x < RP) {
            float s = 0.f;
#pragma unroll
            for (int wv = 0; wv < 16; ++wv) s += red[wv][threadIdx.x];
            tot[threadIdx.x] = s;
        }
        __syncthreads();
        float nrm = sqrtf(tot[0]);
        float den = eps == 0.f ? nrm : nrm + eps;
        float coef[RP];
#pragma unroll
        for (int c = 1; c < RP; ++c) coef[c] = (i + c < r) ? tot[c] / den : 0.f;
        for (int64_t k = threadIdx.x; k < rows; k += 1024) {
            float* row = a + k * r;
            float ci = row[i] / den;
            row[i] = ci;
#pragma unroll
            for (int c = 1; c < RP; ++c)
                if (i + c < r) row[i + c] = __fsub_rn(row[i + c], __fmul_rn(coef[c], ci));
        }
        __syncthreads();   // red/tot are reused by the next column
    }
}

// ---------------------------------------------------------------- dispatch ----
template <int MODE>
int launch_mq(float* x, const float* err, const float* cs, const float* q, float* p, int64_t n, int64_t m, int r,
              int32_t w, float alpha, ConefSeeds hs, hipStream_t s)
{
    ConefMod mod = conef_make_mod(w > 0 ? w : 1);
#define CONEF_MQ(RB, RP)                                                                                          \
    hipLaunchKernelGGL((psgd_mq_kernel<RB, RP, MODE>), dim3((unsigned)((n + RB - 1) / RB)), dim3(256), 0, s, x, err, \
                       cs, q, p, n, m, r, mod, alpha, hs)
    if (r <= 1) CONEF_MQ(8, 1);
    else if (r <= 2) CONEF_MQ(8, 2);
    else if (r <= 4) CONEF_MQ(8, 4);
    else if (r <= 8) CONEF_MQ(4, 8);
    else if (r <= 16) CONEF_MQ(2, 16);
    else CONEF_MQ(1, 32);
#undef CONEF_MQ
    return (int)hipGetLastError();
}

inline int64_t slab_rows(int64_t n, int64_t col_tiles)
{
    int64_t slabs = (1024 + col_tiles - 1) / col_tiles;
    if (slabs > (n + 7) / 8) slabs = (n + 7) / 8;
    if (slabs < 1) slabs = 1;
    if (slabs > 65535) slabs = 65535;
    return (n + slabs - 1) / slabs;
}

inline bool psgd_args_ok(int64_t n, int64_t m, int32_t r)
{
    return n >= 1 && m >= 1 && r >= 1 && r <= kMaxRank && n * m > 0;
}

}  // namespace

extern "C" {

int conef_psgd_mq_f32(float* x, const float* q, float* p, int64_t n, int64_t m, int32_t r, void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !q || !p) return CONEF_ERR_INVALID;
    ConefSeeds hs = {0, 0, 0, 0};
    return launch_mq<0>(x, nullptr, nullptr, q, p, n, m, r, 1, 0.f, hs, (hipStream_t)stream);
}

int conef_psgd_mq_ef_f32(float* x, const float* err, const float* q, float* p, int64_t n, int64_t m, int32_t r,
                         void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !err || !q || !p) return CONEF_ERR_INVALID;
    ConefSeeds hs = {0, 0, 0, 0};
    return launch_mq<1>(x, err, nullptr, q, p, n, m, r, 1, 0.f, hs, (hipStream_t)stream);
}

int conef_psgd_mq_conef_f32(float* x, const float* cs, const float* q, float* p, int64_t n, int64_t m, int32_t r,
                            int32_t w, float alpha, int32_t a, int32_t b, void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !cs || !q || !p || w < 1 || w > (1 << 30) || m > 0x7fffffffLL)
        return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    return launch_mq<2>(x, nullptr, cs, q, p, n, m, r, w, alpha, hs, (hipStream_t)stream);
}

int conef_psgd_mtp_f32(const float* x, const float* p, float* q, int64_t n, int64_t m, int32_t r, void* stream)
{
    if (!psgd_args_ok(n, m, r) || !x || !q || !p) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    int64_t col_tiles = (m + 255) / 256;
    int64_t rps = slab_rows(n, col_tiles);
    int64_t slabs = (n + rps - 1) / rps;
    int atom = slabs > 1;
    if (atom) {
        int64_t cnt = m * r;
        int64_t g = (cnt + 255) / 256;
        if (g > 4096) g = 4096;
        hipLaunchKernelGGL(zero_kernel, dim3((unsigned)g), dim3(256), 0, s, q, cnt);
    }
    dim3 grid((unsigned)col_tiles, (unsigned)slabs);
#define CONEF_MTP(RP) hipLaunchKernelGGL(psgd_mtp_kernel<RP>, grid, dim3(256), 0, s, x, p, q, n, m, r, rps, atom)
    if (r <= 1) CONEF_MTP(1);
    else if (r <= 2) CONEF_MTP(2);
    else if (r <= 4) CONEF_MTP(4);
    else if (r <= 8) CONEF_MTP(8);
    else if (r <= 16) CONEF_MTP(16);
    else CONEF_MTP(32);
#undef CONEF_MTP
    return (int)hipGetLastError();
}

static int launch_pqt(float* x, float* err, const float* p, const float* q, int64_t n, int64_t m, int32_t r,
                      hipStream_t s)
{
    int64_t col_tiles = (m + 255) / 256;
    int64_t rps = slab_rows(n, col_tiles);
    dim3 grid((unsigned)col_tiles, (unsigned)((n + rps - 1) / rps));
#define CONEF_PQT(RP)                                                                                        \
    do {                                                                                                     \
        if (err) hipLaunchKernelGGL((psgd_pqt_kernel<RP, 1>), grid, dim3(256), 0, s, x, err, p, q, n, m, r, rps); \
        else hipLaunchKernelGGL((psgd_pqt_kernel<RP, 0>), grid, dim3(256), 0, s, x, err, p, q, n, m, r, rps);     \
    } while (0)
    if (r <= 1) CONEF_PQT(1);
    else if (r <= 2) CONEF_PQT(2);
    else if (r <= 4) CONEF_PQT(4);
    else if (r <= 8) CONEF_PQT(8);
    else if (r <= 16) CONEF_PQT(16);
    else CONEF_PQT(32);
#undef CONEF_PQT
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
    if (!psgd_args_ok(n, m, r) || !x || !q || !p || !cs_in || !cs_out || w < 1 || w > (1 << 30) ||
        m > 0x7fffffffLL)
        return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    FrontPsgdResidual front = {x, p, q, m, r};
    return conef_launch_sketch_step<float>(front, cs_in, cs_out, n, m, w, beta, hs, (hipStream_t)stream, false);
}

int conef_gram_schmidt_f32(float* a, int64_t rows, int32_t r, float eps, void* stream)
{
    if (rows < 1 || r < 1 || r > kMaxRank || !a) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
#define CONEF_GS(RP) hipLaunchKernelGGL(gram_schmidt_kernel<RP>, dim3(1), dim3(1024), 0, s, a, rows, r, eps)
    if (r <= 1) CONEF_GS(1);
    else if (r <= 2) CONEF_GS(2);
    else if (r <= 4) CONEF_GS(4);
    else if (r <= 8) CONEF_GS(8);
    else if (r <= 16) CONEF_GS(16);
    else CONEF_GS(32);
#undef CONEF_GS
    return (int)hipGetLastError();
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
