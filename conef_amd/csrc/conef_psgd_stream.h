// P = X Q for ranks up to 8, streaming form (gfx950).
//
// X is the matrix M as stored (MODE 0), M + E with a dense error (MODE 1) or M + alpha * unsketch(cs)
// (MODE 2: DenseCS.query fused, CountSketch.py:40-47); in modes 1 and 2 X is written back into M.
// Reference semantics: powerSGD_hook.py:596-640 (error added, P = M Q by bmm).
//
// A workgroup of T threads is split into groups of `gw` threads (a multiple of 64, at least a
// quarter of the matrix's columns).  A group owns S consecutive rows; a thread owns the column
// quads slab * gw + t and keeps their 4 x RP block of Q, and their buckets and signs, in registers
// for all rows of a slab.  Rows go four at a time, the next four requested before the current four
// are used.  The 4 x RP sums of a thread are reduced over the wave by a butterfly that halves the
// number of values with every exchange (4 RP exchanges instead of 6 for each of the 4 RP values),
// the waves' results are parked in LDS and added in a fixed order at the end: no atomics, the same
// result on every run.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "conef_device.h"

__device__ __forceinline__ void mqs_ld4(const float* p, float* v)
{
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void mqs_st4(float* p, const float* v)
{
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

struct MqsItem {
    float* x;
    const float* err;
    const float* cs;
    const uint32_t* pktab;   // bucket | sign << 31 per column, or null: hashed
    const float* q;
    float* p;
    int64_t n;
    int m, w;
    int gw, S;               // threads of a group, rows of a group (multiple of 4)
    ConefMod mod;
    // not null: workgroup g of the matrix also leaves the upper triangle of (its rows of P)^T (its
    // rows of P), RP (RP + 1) / 2 doubles, at gram[g * RP (RP + 1) / 2]: the shares of P^T P
    double* gram;
};

// threads of a group for a matrix of m columns in a workgroup of T threads
inline int mqs_group_width(int64_t m, int T)
{
    const int64_t m4 = m >> 2;
    const int64_t nslab = (m4 + T - 1) / T;
    int64_t gw = ((m4 + nslab - 1) / nslab + 63) / 64 * 64;
    if (gw < 64) gw = 64;
    // a group width that does not divide T leaves threads idle: take the next one that does when that is cheaper
    if (T % gw != 0) {
        int64_t up = gw;
        while (T % up != 0) up += 64;
        if (up - gw < T % gw) gw = up;
    }
    return (int)gw;
}

inline int64_t mqs_workgroups(int64_t n, int gw, int S, int T)
{
    const int64_t rows = (int64_t)(T / gw) * S;
    return (n + rows - 1) / rows;
}

inline size_t mqs_lds_bytes(int64_t m, int w, int gw, int S, int T, int rp, bool sketch, bool gram = false)
{
    const int64_t m4 = m >> 2;
    const int64_t niter = (m4 + gw - 1) / gw * (S >> 2);
    return (size_t)niter * (T / 64) * 4 * rp * 4 + (sketch ? (size_t)(T / gw) * S * w * 4 : 0) +
           (gram ? (size_t)(T / gw) * S * rp * 4 : 0);
}

// Workgroup size and rows per group for one launch over `count` matrices.  Wide matrices need the
// threads of a large workgroup side by side; rows per group are as many as still leave the launch
// enough workgroups, and as the parked sketch rows leave room for in LDS.  False: no geometry fits,
// or the matrices are too small for this kernel to pay.
inline bool mqs_plan_launch(const MqsItem* items, int count, int rp, bool sketch, int* T_out, int* S_out, size_t* lds_out,
                            bool gram = false)
{
    int T = 256;
    for (int k = 0; k < count; ++k)
        if ((items[k].m >> 2) > 512) T = 1024;
    const int want = T == 256 ? 384 : 160;
    for (int S = T == 256 ? 16 : 8; S >= 4; S >>= 1) {
        int64_t wgs = 0;
        size_t lds = 0;
        for (int k = 0; k < count; ++k) {
            const int gw = mqs_group_width(items[k].m, T);
            wgs += mqs_workgroups(items[k].n, gw, S, T);
            const size_t need = mqs_lds_bytes(items[k].m, items[k].w, gw, S, T, rp, sketch, gram);
            if (need > lds) lds = need;
        }
        if (lds > 64 * 1024) continue;
        // a launch that cannot give every CU a workgroup's worth of threads is better served by the
        // row-block kernel, whose workgroups are a row or four each
        if (S == 4 && wgs * T < 256 * 256) return false;
        if (wgs >= want || S == 4) {
            *T_out = T;
            *S_out = S;
            *lds_out = lds;
            return true;
        }
    }
    return false;
}

template <int N>
__device__ __forceinline__ void mqs_halve(float* v, int lane, int mask)
{
    const bool hi = (lane & mask) != 0;
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
        const float keep = hi ? v[N / 2 + i] : v[i];
        const float send = hi ? v[i] : v[N / 2 + i];
        v[i] = keep + __shfl_xor(send, mask, 64);
    }
}

// Sums NV values over the 64 lanes.  Afterwards lane l holds in v[0] the sum of value
// l >> (6 - log2 NV); every lane of that run holds the same number.
template <int NV>
__device__ __forceinline__ void mqs_wave_reduce(float* v, int lane)
{
    if (NV >= 32) mqs_halve<(NV >= 32 ? 32 : 2)>(v, lane, 32);
    if (NV >= 16) mqs_halve<(NV >= 16 ? 16 : 2)>(v, lane, NV >= 32 ? 16 : 32);
    if (NV >= 8) mqs_halve<(NV >= 8 ? 8 : 2)>(v, lane, NV >= 32 ? 8 : NV >= 16 ? 16 : 32);
    if (NV >= 4) mqs_halve<4>(v, lane, NV >= 32 ? 4 : NV >= 16 ? 8 : NV >= 8 ? 16 : 32);
    mqs_halve<2>(v, lane, NV >= 32 ? 2 : NV >= 16 ? 4 : NV >= 8 ? 8 : NV >= 4 ? 16 : 32);
    constexpr int kLeft = NV >= 32 ? 1 : NV >= 16 ? 2 : NV >= 8 ? 4 : NV >= 4 ? 8 : 16;   // lanes that still differ
#pragma unroll
    for (int mask = kLeft; mask >= 1; mask >>= 1) v[0] += __shfl_xor(v[0], mask, 64);
}

template <int RP, int MODE, int T>
__device__ __forceinline__ void
psgd_mqs_body(const MqsItem& it, float alpha, ConefSeeds hs, int bx)
{
    constexpr int NV = 4 * RP;
    constexpr int WAVES = T / 64;
    constexpr int kShift = NV >= 32 ? 1 : NV >= 16 ? 2 : NV >= 8 ? 3 : NV >= 4 ? 4 : 5;   // 6 - log2 NV
    extern __shared__ float mqs_lds[];
    const int m = it.m, m4 = m >> 2, w = it.w, gw = it.gw, S = it.S;
    const int64_t n = it.n;
    const int groups = T / gw;
    const int nslab = (m4 + gw - 1) / gw;
    const int nblk = S >> 2;
    const int niter = nslab * nblk;
    float* red = mqs_lds;                                  // [niter][WAVES][NV]
    float* cells = mqs_lds + (size_t)niter * WAVES * NV;   // [groups * S][w], MODE 2 only
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    int g = tid / gw;
    const int gt = tid - g * gw;
    const bool idle = g >= groups;                         // threads past the last whole group
    if (idle) g = groups - 1;
    const int64_t wg_row0 = (int64_t)bx * groups * S;
    const int rows_here = n - wg_row0 < (int64_t)groups * S ? (int)(n - wg_row0) : groups * S;   // >= 1
    // local row of (block b, row a of the block), clamped to the last row this workgroup has
    auto local_row = [&](int b, int a) {
        const int lr = g * S + 4 * b + a;
        return lr < rows_here ? lr : rows_here - 1;
    };
    auto quad_of = [&](int slab) {
        const int j = slab * gw + gt;
        return j < m4 ? j : m4 - 1;
    };
    float xn[4][4], en[4][4];
    auto request = [&](int iter) {
        const int slab = iter / nblk, b = iter - slab * nblk;
        const int j = quad_of(slab);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t off = (wg_row0 + local_row(b, a)) * m + 4 * j;
            mqs_ld4(it.x + off, xn[a]);
            if (MODE == 1) mqs_ld4(it.err + off, en[a]);
        }
    };
    request(0);
    if (MODE == 2) {
        const float* src = it.cs + wg_row0 * w;
        for (int i = tid; i < rows_here * w; i += T) cells[i] = src[i];
        __syncthreads();
    }
    float qreg[4 * RP];
    uint32_t pk[4] = {0u, 0u, 0u, 0u};
    bool valid = false;
    int j = 0;
    for (int iter = 0; iter < niter; ++iter) {
        const int slab = iter / nblk, b = iter - slab * nblk;
        if (b == 0) {
            j = quad_of(slab);
            valid = !idle && slab * gw + gt < m4;
#pragma unroll
            for (int t = 0; t < RP; ++t) mqs_ld4(it.q + (int64_t)j * 4 * RP + 4 * t, qreg + 4 * t);
            if (!valid) {                                  // a duplicate of the last quad: it adds nothing
#pragma unroll
                for (int t = 0; t < 4 * RP; ++t) qreg[t] = 0.f;
            }
            if (MODE == 2) {
                if (it.pktab) {
                    const uint4 t = reinterpret_cast<const uint4*>(it.pktab)[j];
                    pk[0] = t.x; pk[1] = t.y; pk[2] = t.z; pk[3] = t.w;
                } else {
#pragma unroll
                    for (int k = 0; k < 4; ++k) pk[k] = conef_bucket_sign(4 * j + k, it.mod, hs.a, hs.b, hs.sa, hs.sb);
                }
            }
        }
        float xv[4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                xv[a][k] = xn[a][k];
                if (MODE == 1) xv[a][k] = __fadd_rn(xv[a][k], en[a][k]);
            }
        if (iter + 1 < niter) request(iter + 1);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int lr = g * S + 4 * b + a;
            if (MODE == 2) {
                const float* crow = cells + (size_t)(lr < rows_here ? lr : rows_here - 1) * w;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    xv[a][k] = __fadd_rn(xv[a][k], conef_query_term(crow[pk[k] & 0x7fffffffu], pk[k], alpha));
            }
            if (MODE != 0 && valid && lr < rows_here) mqs_st4(it.x + (wg_row0 + lr) * m + 4 * j, xv[a]);
        }
        float acc[NV];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int c = 0; c < RP; ++c) {
                float s = 0.f;
#pragma unroll
                for (int k = 0; k < 4; ++k) s = fmaf(xv[a][k], qreg[k * RP + c], s);
                acc[a * RP + c] = s;
            }
        mqs_wave_reduce<NV>(acc, lane);
        if ((lane & ((1 << kShift) - 1)) == 0) red[((size_t)iter * WAVES + wave) * NV + (lane >> kShift)] = acc[0];
    }
    __syncthreads();
    const int wpg = gw >> 6;                               // waves of a group
    float* prow = cells + (MODE == 2 ? (size_t)groups * S * w : 0);   // [groups * S][RP], only with it.gram
    for (int o = tid; o < rows_here * RP; o += T) {
        const int lr = o / RP, c = o - lr * RP;
        const int gg = lr / S, rr = lr - gg * S;
        const int b = rr >> 2, idx = (rr & 3) * RP + c;
        float s = 0.f;
        for (int slab = 0; slab < nslab; ++slab) {
            const float* base = red + ((size_t)(slab * nblk + b) * WAVES + gg * wpg) * NV + idx;
            for (int v = 0; v < wpg; ++v) s += base[(size_t)v * NV];
        }
        it.p[(wg_row0 + lr) * RP + c] = s;
        if (it.gram) prow[o] = s;
    }
    if (it.gram) {
        constexpr int NG = RP * (RP + 1) / 2;
        __syncthreads();
        if (tid < NG) {
            int i = 0, e0 = 0;                             // entry tid of the row-major upper triangle is (i, j)
            while (tid >= e0 + RP - i) {
                e0 += RP - i;
                ++i;
            }
            const int j = i + (tid - e0);
            double s = 0.;
            for (int lr = 0; lr < rows_here; ++lr) s = fma((double)prow[lr * RP + i], (double)prow[lr * RP + j], s);
            it.gram[(size_t)bx * NG + tid] = s;
        }
    }
}
