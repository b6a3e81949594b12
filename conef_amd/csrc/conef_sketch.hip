// Count-sketch error compressor kernels for gfx950 and their C entry points.
//
// Two launch shapes cover the sketch shapes that occur:
//   * "row" shape  - short rows, many of them (low-rank compressors: W <= a few thousand).
//     One wavefront owns one row at a time; the row of the sketch lives in LDS (snapshot +
//     accumulator), the per-column (bucket, sign) table is computed once per workgroup and kept in
//     LDS for every row the workgroup handles.  In place is fine (a row is read before it is written).
//   * "tile" shape - few very long rows (a flat 25 MB bucket viewed [5, 1.3M], W = 130k).  A sketch
//     row does not fit LDS, so a thread owns a few columns for ALL rows (the hash is the same for
//     every row and is computed once), gathers the snapshot from L2 and accumulates with float
//     atomics into a second buffer that starts as a copy of the snapshot.
//
// Reference semantics: communication/compressors/CountSketch.py:27-98 (one hash),
// CountSketchHash3.py:27-147 (three hashes + median), halfCountSketch.py (fp16 storage).
#include "conef_device.h"
#include "conef_sketch_core.h"

namespace {

// ------------------------------------------------------------ hash table ----
__global__ void hash_table_kernel(int32_t* bucket, int32_t* sign, int64_t d, ConefMod mod, ConefSeeds hs)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i < d) {
        uint32_t p = conef_bucket_sign((int32_t)i, mod, hs.a, hs.b, hs.sa, hs.sb);
        bucket[i] = (int32_t)(p & 0x7fffffffu);
        sign[i] = (p >> 31) ? 1 : -1;
    }
}

// ----------------------------------------------------------------- query ----
// x[r,i] += (sign_i * cs[r,h_i]) * alpha.  Thread = 4 consecutive columns, loop over a group of
// rows so the two hashes per column are paid once per row group.  The rows are taken RB at a time
// with every load of the batch (values and gathered cells) issued before the first is used: a
// thread's stores and later loads retire through one in-order counter, so row-at-a-time code pays
// a full memory round trip per row.
template <typename CsT, int VW, int RB>
__global__ void __launch_bounds__(256)
cs_query_kernel(float* __restrict__ x, const CsT* __restrict__ cs, int64_t n, int64_t d, ConefMod mod,
                float alpha, ConefSeeds hs, int rows_per_block, const uint32_t* __restrict__ pktab)
{
    int64_t c0 = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * 4;
    if (c0 >= d) return;
    // bucket | sign << 31 of the thread's four columns: from a plan's table when the caller has one
    // (16 bytes a thread instead of eight hashes and modulos), else computed
    uint32_t pk[4];
    if (pktab && c0 + 4 <= d) {
        const uint4 t = *reinterpret_cast<const uint4*>(pktab + c0);      // tables are 256-byte aligned, c0 a multiple of 4
        pk[0] = t.x; pk[1] = t.y; pk[2] = t.z; pk[3] = t.w;
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
            pk[k] = (c0 + k < d) ? (pktab ? pktab[c0 + k] : conef_bucket_sign((int32_t)(c0 + k), mod, hs.a, hs.b, hs.sa, hs.sb))
                                 : 0u;
    }
    int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    // VW = 4: rows are 16-byte aligned, one float4 per row; VW = 2: 8-byte aligned, two float2
    if (VW > 1 && c0 + 4 <= d) {
        for (int64_t r = r0; r < r1; r += RB) {
            float4 v[RB];
            float cell[RB][4];
#pragma unroll
            for (int u = 0; u < RB; ++u) {
                const int64_t rr = r + u < r1 ? r + u : r1 - 1;     // clamped: the loads are unconditional
                const CsT* row = cs + rr * (int64_t)mod.w;
                const float* xr = x + rr * d + c0;
                if (VW == 4) {
                    v[u] = *reinterpret_cast<const float4*>(xr);
                } else {
                    const float2 lo = *reinterpret_cast<const float2*>(xr), hi = *reinterpret_cast<const float2*>(xr + 2);
                    v[u] = make_float4(lo.x, lo.y, hi.x, hi.y);
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) cell[u][k] = conef_ld(row + (pk[k] & 0x7fffffffu));
            }
#pragma unroll
            for (int u = 0; u < RB; ++u) {
                if (r + u < r1) {
                    float4 o;
                    o.x = __fadd_rn(v[u].x, conef_query_term(cell[u][0], pk[0], alpha));
                    o.y = __fadd_rn(v[u].y, conef_query_term(cell[u][1], pk[1], alpha));
                    o.z = __fadd_rn(v[u].z, conef_query_term(cell[u][2], pk[2], alpha));
                    o.w = __fadd_rn(v[u].w, conef_query_term(cell[u][3], pk[3], alpha));
                    float* xo = x + (r + u) * d + c0;
                    if (VW == 4) {
                        *reinterpret_cast<float4*>(xo) = o;
                    } else {
                        *reinterpret_cast<float2*>(xo) = make_float2(o.x, o.y);
                        *reinterpret_cast<float2*>(xo + 2) = make_float2(o.z, o.w);
                    }
                }
            }
        }
    } else {
        for (int64_t r = r0; r < r1; ++r) {
            const CsT* row = cs + r * (int64_t)mod.w;
            float* xr = x + r * d + c0;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (c0 + k < d)
                    xr[k] = __fadd_rn(xr[k], conef_query_term(conef_ld(row + (pk[k] & 0x7fffffffu)), pk[k], alpha));
        }
    }
}

// three sketches, median of the three estimates (CountSketchHash3.py:101-147)
__global__ void __launch_bounds__(256)
cs3_query_kernel(float* __restrict__ x, const float* __restrict__ cs0, const float* __restrict__ cs1,
                 const float* __restrict__ cs2, int64_t n, int64_t d, ConefMod mod, float alpha, int rows_per_block)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i >= d) return;
    uint32_t pk[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        ConefSeeds s = conef_hash3_seeds(k, /*for_query=*/true);
        pk[k] = conef_bucket_sign((int32_t)i, mod, s.a, s.b, s.sa, s.sb);
    }
    int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    for (int64_t r = r0; r < r1; ++r) {
        int64_t base = r * (int64_t)mod.w;
        float u0 = conef_query_term(cs0[base + (pk[0] & 0x7fffffffu)], pk[0], alpha);
        float u1 = conef_query_term(cs1[base + (pk[1] & 0x7fffffffu)], pk[1], alpha);
        float u2 = conef_query_term(cs2[base + (pk[2] & 0x7fffffffu)], pk[2], alpha);
        x[r * d + i] = __fadd_rn(x[r * d + i], conef_median3(u0, u1, u2));
    }
}

// The same with a thread on 4 consecutive columns of 16-byte aligned rows, RB rows at a time, every
// load of a batch (the values and 12 gathered cells a row) requested before the first is used; the
// six hashes of a column are paid once per row group.  Same arithmetic per element as above.
template <int RB>
__global__ void __launch_bounds__(256)
cs3_query_vec_kernel(float* __restrict__ x, const float* __restrict__ cs0, const float* __restrict__ cs1,
                     const float* __restrict__ cs2, int64_t n, int64_t d, ConefMod mod, float alpha, int rows_per_block)
{
    const int64_t c0 = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * 4;
    if (c0 >= d) return;                      // d is a multiple of 4 here
    uint32_t pk[3][4];
#pragma unroll
    for (int h = 0; h < 3; ++h) {
        ConefSeeds s = conef_hash3_seeds(h, /*for_query=*/true);
#pragma unroll
        for (int k = 0; k < 4; ++k) pk[h][k] = conef_bucket_sign((int32_t)(c0 + k), mod, s.a, s.b, s.sa, s.sb);
    }
    const float* cs[3] = {cs0, cs1, cs2};
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    for (int64_t r = r0; r < r1; r += RB) {
        float4 v[RB];
        float cell[RB][3][4];
#pragma unroll
        for (int u = 0; u < RB; ++u) {
            const int64_t rr = r + u < r1 ? r + u : r1 - 1;     // clamped: the loads are unconditional
            v[u] = *reinterpret_cast<const float4*>(x + rr * d + c0);
#pragma unroll
            for (int h = 0; h < 3; ++h)
#pragma unroll
                for (int k = 0; k < 4; ++k) cell[u][h][k] = cs[h][rr * (int64_t)mod.w + (pk[h][k] & 0x7fffffffu)];
        }
#pragma unroll
        for (int u = 0; u < RB; ++u) {
            if (r + u < r1) {
                float in[4] = {v[u].x, v[u].y, v[u].z, v[u].w}, o[4];
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    o[k] = __fadd_rn(in[k], conef_median3(conef_query_term(cell[u][0][k], pk[0][k], alpha),
                                                          conef_query_term(cell[u][1][k], pk[1][k], alpha),
                                                          conef_query_term(cell[u][2][k], pk[2][k], alpha)));
                *reinterpret_cast<float4*>(x + (r + u) * d + c0) = make_float4(o[0], o[1], o[2], o[3]);
            }
        }
    }
}

// three-sketch update (CountSketchHash3.py:27-98); out buffers start as copies of the snapshots
__global__ void __launch_bounds__(256)
cs3_update_kernel(const float* __restrict__ vec, const float* __restrict__ in0, const float* __restrict__ in1,
                  const float* __restrict__ in2, float* out0, float* out1, float* out2, int64_t n, int64_t d,
                  ConefMod mod, float beta, int rows_per_block)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i >= d) return;
    uint32_t pk[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        ConefSeeds s = conef_hash3_seeds(k, /*for_query=*/false);
        pk[k] = conef_bucket_sign((int32_t)i, mod, s.a, s.b, s.sa, s.sb);
    }
    const double bm1 = (double)beta - 1.0;          // :70  (beta - 1.0)
    const double neg_omb = -(1. - (double)beta);    // :79,:87  -(1. - beta)
    int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    for (int64_t r = r0; r < r1; ++r) {
        int64_t base = r * (int64_t)mod.w;
        float value = vec[r * d + i];
        uint32_t j0 = pk[0] & 0x7fffffffu, j1 = pk[1] & 0x7fffffffu, j2 = pk[2] & 0x7fffffffu;
        float u0 = (float)__dmul_rn((double)conef_apply_sign(in0[base + j0], pk[0]), bm1);
        float u1 = (float)__dmul_rn(neg_omb, (double)conef_apply_sign(in1[base + j1], pk[1]));
        float u2 = (float)__dmul_rn(neg_omb, (double)conef_apply_sign(in2[base + j2], pk[2]));
        float t = __fadd_rn(conef_median3(u0, u1, u2), value);
        unsafeAtomicAdd(out0 + base + j0, conef_apply_sign(t, pk[0]));
        unsafeAtomicAdd(out1 + base + j1, conef_apply_sign(t, pk[1]));
        unsafeAtomicAdd(out2 + base + j2, conef_apply_sign(t, pk[2]));
    }
}

// The value all three sketches accumulate for an element (CountSketchHash3.py:70-93):
// t = median(u0, u1, u2) + v with u_k = -(1 - beta) * s_k * cs_k[h_k] taken from the snapshots.
// With t in hand, each sketch's update is the one-hash update of t with beta = 1 (no decay of its
// own), which the planned kernels do without atomics and in the serial definition's order.
__global__ void __launch_bounds__(256)
cs3_value_kernel(const float* __restrict__ vec, const float* __restrict__ in0, const float* __restrict__ in1,
                 const float* __restrict__ in2, float* __restrict__ out_t, int64_t n, int64_t d, ConefMod mod, float beta,
                 int rows_per_block)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i >= d) return;
    uint32_t pk[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        ConefSeeds s = conef_hash3_seeds(k, /*for_query=*/false);
        pk[k] = conef_bucket_sign((int32_t)i, mod, s.a, s.b, s.sa, s.sb);
    }
    const double bm1 = (double)beta - 1.0;
    const double neg_omb = -(1. - (double)beta);
    const uint32_t j0 = pk[0] & 0x7fffffffu, j1 = pk[1] & 0x7fffffffu, j2 = pk[2] & 0x7fffffffu;
    int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    for (int64_t r = r0; r < r1; ++r) {
        int64_t base = r * (int64_t)mod.w;
        float value = vec[r * d + i];
        float u0 = (float)__dmul_rn((double)conef_apply_sign(in0[base + j0], pk[0]), bm1);
        float u1 = (float)__dmul_rn(neg_omb, (double)conef_apply_sign(in1[base + j1], pk[1]));
        float u2 = (float)__dmul_rn(neg_omb, (double)conef_apply_sign(in2[base + j2], pk[2]));
        out_t[r * d + i] = __fadd_rn(conef_median3(u0, u1, u2), value);
    }
}

// The same with a thread on 4 consecutive columns of 16-byte aligned rows, RB rows at a time, every
// load of a batch requested before the first is used.  Same arithmetic per element as above.
template <int RB>
__global__ void __launch_bounds__(256)
cs3_value_vec_kernel(const float* __restrict__ vec, const float* __restrict__ in0, const float* __restrict__ in1,
                     const float* __restrict__ in2, float* __restrict__ out_t, int64_t n, int64_t d, ConefMod mod,
                     float beta, int rows_per_block)
{
    const int64_t c0 = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * 4;
    if (c0 >= d) return;                      // d is a multiple of 4 here
    uint32_t pk[3][4];
#pragma unroll
    for (int h = 0; h < 3; ++h) {
        ConefSeeds s = conef_hash3_seeds(h, /*for_query=*/false);
#pragma unroll
        for (int k = 0; k < 4; ++k) pk[h][k] = conef_bucket_sign((int32_t)(c0 + k), mod, s.a, s.b, s.sa, s.sb);
    }
    const float* in[3] = {in0, in1, in2};
    const double bm1 = (double)beta - 1.0;
    const double neg_omb = -(1. - (double)beta);
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    for (int64_t r = r0; r < r1; r += RB) {
        float4 v[RB];
        float cell[RB][3][4];
#pragma unroll
        for (int u = 0; u < RB; ++u) {
            const int64_t rr = r + u < r1 ? r + u : r1 - 1;     // clamped: the loads are unconditional
            v[u] = *reinterpret_cast<const float4*>(vec + rr * d + c0);
#pragma unroll
            for (int h = 0; h < 3; ++h)
#pragma unroll
                for (int k = 0; k < 4; ++k) cell[u][h][k] = in[h][rr * (int64_t)mod.w + (pk[h][k] & 0x7fffffffu)];
        }
#pragma unroll
        for (int u = 0; u < RB; ++u) {
            if (r + u < r1) {
                float val[4] = {v[u].x, v[u].y, v[u].z, v[u].w}, o[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float u0 = (float)__dmul_rn((double)conef_apply_sign(cell[u][0][k], pk[0][k]), bm1);
                    float u1 = (float)__dmul_rn(neg_omb, (double)conef_apply_sign(cell[u][1][k], pk[1][k]));
                    float u2 = (float)__dmul_rn(neg_omb, (double)conef_apply_sign(cell[u][2][k], pk[2][k]));
                    o[k] = __fadd_rn(conef_median3(u0, u1, u2), val[k]);
                }
                *reinterpret_cast<float4*>(out_t + (r + u) * d + c0) = make_float4(o[0], o[1], o[2], o[3]);
            }
        }
    }
}

// -------------------------------------------------------------- utilities ----
template <typename T>
__global__ void scale_kernel(T* x, int64_t count, float alpha)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) conef_st(x + i, __fmul_rn(conef_ld(x + i), alpha));
}

template <typename D, typename S>
__global__ void convert_kernel(D* __restrict__ dst, const S* __restrict__ src, int64_t count)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) conef_st(dst + i, conef_ld(src + i));
}

inline int grid_for(int64_t count, int threads, int64_t cap = 8192)
{
    int64_t g = (count + threads - 1) / threads;
    if (g < 1) g = 1;
    if (g > cap) g = cap;
    return (int)g;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int rows_per_block_for(int64_t n, int64_t col_blocks)
{
    // enough workgroups to fill 256 CUs several times over, but at least 8 rows per workgroup
    // (when there are that many) so the per-column hashes are amortised
    int64_t want_blocks = 4096;
    int64_t rpb = (n * col_blocks + want_blocks - 1) / want_blocks;
    if (rpb < 8) rpb = 8;
    if (rpb > n) rpb = n;
    if (rpb < 1) rpb = 1;
    // gridDim.y limit
    while ((n + rpb - 1) / rpb > 65535) rpb *= 2;
    return (int)rpb;
}

template <typename CsT>
int launch_query(float* x, const CsT* cs, int64_t n, int64_t d, int32_t w, float alpha, int32_t a, int32_t b,
                 hipStream_t stream, const uint32_t* pktab = nullptr)
{
    if (n < 0 || d < 0 || w < 1 || w > (1 << 30) || d > 0x7fffffffLL) return CONEF_ERR_INVALID;
    if (n == 0 || d == 0) return CONEF_OK;
    if (!x || !cs) return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    int64_t col_blocks = (d + 1023) / 1024;
    int rpb = rows_per_block_for(n, col_blocks);
    dim3 grid((unsigned)col_blocks, (unsigned)((n + rpb - 1) / rpb));
    const int vw = (d % 4 == 0 && aligned16(x)) ? 4 : (d % 2 == 0 && (reinterpret_cast<uintptr_t>(x) & 7u) == 0) ? 2 : 1;
    ConefMod mod = conef_make_mod(w);
    if (vw == 1) {
        hipLaunchKernelGGL((cs_query_kernel<CsT, 1, 1>), grid, dim3(256), 0, stream, x, cs, n, d, mod, alpha, hs, rpb, pktab);
        return (int)hipGetLastError();
    }
    // Rows in flight per thread: the whole row group when it is small; four at a time when the
    // launch has too few workgroups to hide a round trip per row behind other waves; one otherwise
    // (more costs registers, and with them resident waves, on the shapes that have rows to spare).
    const int64_t wgs = (int64_t)grid.x * grid.y;
    switch (rpb <= 5 ? rpb : wgs <= 256 ? 4 : 1) {
#define CONEF_QUERY_CASE(RB)                                                                                          \
    case RB:                                                                                                          \
        if (vw == 4)                                                                                                  \
            hipLaunchKernelGGL((cs_query_kernel<CsT, 4, RB>), grid, dim3(256), 0, stream, x, cs, n, d, mod, alpha, hs, \
                               rpb, pktab);                                                                           \
        else                                                                                                          \
            hipLaunchKernelGGL((cs_query_kernel<CsT, 2, RB>), grid, dim3(256), 0, stream, x, cs, n, d, mod, alpha, hs, \
                               rpb, pktab);                                                                           \
        break
        CONEF_QUERY_CASE(1);
        CONEF_QUERY_CASE(2);
        CONEF_QUERY_CASE(3);
        CONEF_QUERY_CASE(4);
        CONEF_QUERY_CASE(5);
#undef CONEF_QUERY_CASE
    }
    return (int)hipGetLastError();
}

template <typename CsT>
int launch_update(const float* vec, const CsT* cs_in, CsT* cs_out, int64_t n, int64_t d, int32_t w, float beta,
                  int32_t a, int32_t b, hipStream_t stream)
{
    if (n < 0 || d < 0 || w < 1 || w > (1 << 30) || d > 0x7fffffffLL) return CONEF_ERR_INVALID;
    if (n == 0) return CONEF_OK;
    if (!cs_in || !cs_out || (!vec && d > 0)) return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    ConefFrontVec front = {vec, d};
    return conef_launch_sketch_step<CsT>(front, cs_in, cs_out, n, d, w, beta, hs, stream, aligned16(vec));
}

}  // namespace

// ---- the query for a few long rows (at most 8 rows, a sketch row far beyond LDS) ----
// Every row of the tensor uses the same bucket for a column, so with the sketch transposed to
// [w][8] (32 bytes a bucket, rows past n zero) a column's cells of ALL rows are one 32-byte gather
// instead of one 4-byte gather per row, each of which drags a cache line from L2: five times fewer
// lines for the flat 25 MB bucket, whose query was bound by exactly that.
namespace {

__global__ void __launch_bounds__(256)
cs_interleave8_kernel(const float* __restrict__ cs, float* __restrict__ inter, int n, int w)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= w) return;
    float v[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = r < n ? cs[(int64_t)r * w + j] : 0.f;
    float4* dst = reinterpret_cast<float4*>(inter + (int64_t)j * 8);
    dst[0] = make_float4(v[0], v[1], v[2], v[3]);
    dst[1] = make_float4(v[4], v[5], v[6], v[7]);
}

// a thread owns a column quad of all rows; d % 4 == 0, x and the table 16-byte aligned
template <int NR>
__global__ void __launch_bounds__(256)
cs_query_rows8_kernel(float* __restrict__ x, const float* __restrict__ inter, int64_t d, float alpha,
                      const uint32_t* __restrict__ pktab)
{
    const int64_t c0 = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * 4;
    if (c0 >= d) return;
    const uint4 t = *reinterpret_cast<const uint4*>(pktab + c0);
    const uint32_t pk[4] = {t.x, t.y, t.z, t.w};
    float4 v[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) v[r] = *reinterpret_cast<const float4*>(x + (int64_t)r * d + c0);
    float cell[4][8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float4* src = reinterpret_cast<const float4*>(inter + (int64_t)(pk[k] & 0x7fffffffu) * 8);
        const float4 lo = src[0];
        cell[k][0] = lo.x; cell[k][1] = lo.y; cell[k][2] = lo.z; cell[k][3] = lo.w;
        if (NR > 4) {
            const float4 hi = src[1];
            cell[k][4] = hi.x; cell[k][5] = hi.y; cell[k][6] = hi.z; cell[k][7] = hi.w;
        }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        float4 o;
        o.x = __fadd_rn(v[r].x, conef_query_term(cell[0][r], pk[0], alpha));
        o.y = __fadd_rn(v[r].y, conef_query_term(cell[1][r], pk[1], alpha));
        o.z = __fadd_rn(v[r].z, conef_query_term(cell[2][r], pk[2], alpha));
        o.w = __fadd_rn(v[r].w, conef_query_term(cell[3][r], pk[3], alpha));
        *reinterpret_cast<float4*>(x + (int64_t)r * d + c0) = o;
    }
}

}  // namespace

// scratch: at least 32 w bytes, 16-byte aligned.  Returns CONEF_ERR_INVALID for shapes this form
// does not take (more than 8 rows, d % 4 != 0, unaligned x or table); the caller then takes the
// general query.
int conef_launch_query_rows8_f32(float* x, const float* cs, int64_t n, int64_t d, int32_t w, float alpha,
                                 const uint32_t* pktab, float* scratch, hipStream_t stream)
{
    if (n < 1 || n > 8 || d < 4 || d % 4 != 0 || !aligned16(x) || !aligned16(pktab) || !aligned16(scratch)) return CONEF_ERR_INVALID;
    hipLaunchKernelGGL(cs_interleave8_kernel, dim3((unsigned)((w + 255) / 256)), dim3(256), 0, stream, cs, scratch, (int)n, (int)w);
    const dim3 grid((unsigned)((d / 4 + 255) / 256));
    switch ((int)n) {
#define CONEF_ROWS8(NR) \
    case NR: hipLaunchKernelGGL(cs_query_rows8_kernel<NR>, grid, dim3(256), 0, stream, x, scratch, d, alpha, pktab); break
        CONEF_ROWS8(1); CONEF_ROWS8(2); CONEF_ROWS8(3); CONEF_ROWS8(4);
        CONEF_ROWS8(5); CONEF_ROWS8(6); CONEF_ROWS8(7); CONEF_ROWS8(8);
#undef CONEF_ROWS8
    }
    return (int)hipGetLastError();
}

// The query with buckets and signs read from a table (uint32[d]: bucket | sign bit << 31, the `pk`
// table of a plan); called by conef_cs_query_planned_f32 / _f16 in conef_plan.hip.
int conef_launch_query_table_f32(float* x, const float* cs, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                                 int32_t b, const uint32_t* pktab, hipStream_t stream)
{
    return launch_query<float>(x, cs, n, d, w, alpha, a, b, stream, pktab);
}

int conef_launch_query_table_f16(float* x, const void* cs_half, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                                 int32_t b, const uint32_t* pktab, hipStream_t stream)
{
    return launch_query<__half>(x, (const __half*)cs_half, n, d, w, alpha, a, b, stream, pktab);
}

// ============================================================ C entry points ====
extern "C" {

int conef_version(void) { return 1; }

int conef_hash_table_i32(int32_t* bucket, int32_t* sign, int64_t d, int32_t w, int32_t a, int32_t b, int32_t sa,
                         int32_t sb, void* stream)
{
    if (d < 0 || w < 1 || w > (1 << 30) || d > 0x7fffffffLL) return CONEF_ERR_INVALID;
    if (d == 0) return CONEF_OK;
    if (!bucket || !sign) return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, sa, sb};
    hipLaunchKernelGGL(hash_table_kernel, dim3((unsigned)((d + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       bucket, sign, d, conef_make_mod(w), hs);
    return (int)hipGetLastError();
}

// Same table computed by the host compilation of the very same hash code; lets a machine
// without a GPU check the shipped hash (fast modulo included) bit for bit.
int conef_hash_table_host_i32(int32_t* bucket, int32_t* sign, int64_t d, int32_t w, int32_t a, int32_t b,
                              int32_t sa, int32_t sb)
{
    if (d < 0 || w < 1 || w > (1 << 30) || d > 0x7fffffffLL || (d > 0 && (!bucket || !sign)))
        return CONEF_ERR_INVALID;
    ConefMod mod = conef_make_mod(w);
    for (int64_t i = 0; i < d; ++i) {
        uint32_t p = conef_bucket_sign((int32_t)i, mod, a, b, sa, sb);
        bucket[i] = (int32_t)(p & 0x7fffffffu);
        sign[i] = (p >> 31) ? 1 : -1;
    }
    return CONEF_OK;
}

int conef_cs_query_f32(float* x, const float* cs, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                       int32_t b, void* stream)
{
    return launch_query<float>(x, cs, n, d, w, alpha, a, b, (hipStream_t)stream);
}

int conef_cs_query_f16(float* x, const void* cs_half, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                       int32_t b, void* stream)
{
    return launch_query<__half>(x, (const __half*)cs_half, n, d, w, alpha, a, b, (hipStream_t)stream);
}

int conef_cs_update_inplace_ok(int64_t n, int64_t d, int32_t w)
{
    (void)n;
    return conef_row_shape_fits(d, w, sizeof(float)) ? 1 : 0;
}

int conef_cs_update_f32(const float* vec, const float* cs_in, float* cs_out, int64_t n, int64_t d, int32_t w,
                        float beta, int32_t a, int32_t b, void* stream)
{
    return launch_update<float>(vec, cs_in, cs_out, n, d, w, beta, a, b, (hipStream_t)stream);
}

int conef_cs_update_f16(const float* vec, const void* cs_in_half, void* cs_out_half, int64_t n, int64_t d,
                        int32_t w, float beta, int32_t a, int32_t b, void* stream)
{
    // fp16 storage accumulates in fp32 and rounds once per call, which only the row shape can do
    // without an fp32 staging buffer; larger sketches go through conef_convert_* + the f32 entry.
    if (!conef_row_shape_fits(d, w, sizeof(float))) return CONEF_ERR_INVALID;
    return launch_update<__half>(vec, (const __half*)cs_in_half, (__half*)cs_out_half, n, d, w, beta, a, b,
                                 (hipStream_t)stream);
}

int conef_cs3_query_f32(float* x, const float* cs0, const float* cs1, const float* cs2, int64_t n, int64_t d,
                        int32_t w, float alpha, void* stream)
{
    if (n < 0 || d < 0 || w < 1 || w > (1 << 30) || d > 0x7fffffffLL) return CONEF_ERR_INVALID;
    if (n == 0 || d == 0) return CONEF_OK;
    if (!x || !cs0 || !cs1 || !cs2) return CONEF_ERR_INVALID;
    if (d % 4 == 0 && aligned16(x)) {
        const int64_t cb = (d + 1023) / 1024;
        const int rows = rows_per_block_for(n, cb);
        dim3 g4((unsigned)cb, (unsigned)((n + rows - 1) / rows));
        if (rows == 1)
            hipLaunchKernelGGL(cs3_query_vec_kernel<1>, g4, dim3(256), 0, (hipStream_t)stream, x, cs0, cs1, cs2, n, d,
                               conef_make_mod(w), alpha, rows);
        else
            hipLaunchKernelGGL(cs3_query_vec_kernel<4>, g4, dim3(256), 0, (hipStream_t)stream, x, cs0, cs1, cs2, n, d,
                               conef_make_mod(w), alpha, rows);
        return (int)hipGetLastError();
    }
    int64_t col_blocks = (d + 255) / 256;
    int rpb = rows_per_block_for(n, col_blocks);
    dim3 grid((unsigned)col_blocks, (unsigned)((n + rpb - 1) / rpb));
    hipLaunchKernelGGL(cs3_query_kernel, grid, dim3(256), 0, (hipStream_t)stream, x, cs0, cs1, cs2, n, d,
                       conef_make_mod(w), alpha, rpb);
    return (int)hipGetLastError();
}

int conef_cs3_update_f32(const float* vec, const float* in0, const float* in1, const float* in2, float* out0,
                         float* out1, float* out2, int64_t n, int64_t d, int32_t w, float beta, void* stream)
{
    if (n < 0 || d < 0 || w < 1 || w > (1 << 30) || d > 0x7fffffffLL) return CONEF_ERR_INVALID;
    if (n == 0) return CONEF_OK;
    if (!in0 || !in1 || !in2 || !out0 || !out1 || !out2 || (!vec && d > 0)) return CONEF_ERR_INVALID;
    if (in0 == out0 || in1 == out1 || in2 == out2) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    int64_t cells = n * (int64_t)w;
    int g = grid_for(cells, 256);
    hipLaunchKernelGGL(conef_copy_f32_kernel, dim3(g), dim3(256), 0, s, out0, in0, cells);
    hipLaunchKernelGGL(conef_copy_f32_kernel, dim3(g), dim3(256), 0, s, out1, in1, cells);
    hipLaunchKernelGGL(conef_copy_f32_kernel, dim3(g), dim3(256), 0, s, out2, in2, cells);
    if (d == 0) return (int)hipGetLastError();
    int64_t col_blocks = (d + 255) / 256;
    int rpb = rows_per_block_for(n, col_blocks);
    dim3 grid((unsigned)col_blocks, (unsigned)((n + rpb - 1) / rpb));
    hipLaunchKernelGGL(cs3_update_kernel, grid, dim3(256), 0, s, vec, in0, in1, in2, out0, out1, out2, n, d,
                       conef_make_mod(w), beta, rpb);
    return (int)hipGetLastError();
}

int conef_cs3_value_f32(const float* vec, const float* in0, const float* in1, const float* in2, float* out_t,
                        int64_t n, int64_t d, int32_t w, float beta, void* stream)
{
    if (n < 0 || d < 0 || w < 1 || w > (1 << 30) || d > 0x7fffffffLL) return CONEF_ERR_INVALID;
    if (n == 0 || d == 0) return CONEF_OK;
    if (!vec || !in0 || !in1 || !in2 || !out_t) return CONEF_ERR_INVALID;
    if (d % 4 == 0 && aligned16(vec) && aligned16(out_t)) {
        const int64_t cb = (d + 1023) / 1024;
        const int rows = rows_per_block_for(n, cb);
        dim3 g4((unsigned)cb, (unsigned)((n + rows - 1) / rows));
        if (rows == 1)
            hipLaunchKernelGGL(cs3_value_vec_kernel<1>, g4, dim3(256), 0, (hipStream_t)stream, vec, in0, in1, in2, out_t,
                               n, d, conef_make_mod(w), beta, rows);
        else
            hipLaunchKernelGGL(cs3_value_vec_kernel<4>, g4, dim3(256), 0, (hipStream_t)stream, vec, in0, in1, in2, out_t,
                               n, d, conef_make_mod(w), beta, rows);
        return (int)hipGetLastError();
    }
    int64_t col_blocks = (d + 255) / 256;
    int rpb = rows_per_block_for(n, col_blocks);
    dim3 grid((unsigned)col_blocks, (unsigned)((n + rpb - 1) / rpb));
    hipLaunchKernelGGL(cs3_value_kernel, grid, dim3(256), 0, (hipStream_t)stream, vec, in0, in1, in2, out_t, n, d,
                       conef_make_mod(w), beta, rpb);
    return (int)hipGetLastError();
}

int conef_scale_f32(float* x, int64_t count, float alpha, void* stream)
{
    if (count < 0 || (count > 0 && !x)) return CONEF_ERR_INVALID;
    if (count == 0) return CONEF_OK;
    hipLaunchKernelGGL(scale_kernel<float>, dim3(grid_for(count, 256)), dim3(256), 0, (hipStream_t)stream, x, count,
                       alpha);
    return (int)hipGetLastError();
}

int conef_scale_f16(void* x_half, int64_t count, float alpha, void* stream)
{
    if (count < 0 || (count > 0 && !x_half)) return CONEF_ERR_INVALID;
    if (count == 0) return CONEF_OK;
    hipLaunchKernelGGL(scale_kernel<__half>, dim3(grid_for(count, 256)), dim3(256), 0, (hipStream_t)stream,
                       (__half*)x_half, count, alpha);
    return (int)hipGetLastError();
}

int conef_convert_f16_to_f32(float* dst, const void* src_half, int64_t count, void* stream)
{
    if (count < 0 || (count > 0 && (!dst || !src_half))) return CONEF_ERR_INVALID;
    if (count == 0) return CONEF_OK;
    hipLaunchKernelGGL((convert_kernel<float, __half>), dim3(grid_for(count, 256)), dim3(256), 0,
                       (hipStream_t)stream, dst, (const __half*)src_half, count);
    return (int)hipGetLastError();
}

int conef_convert_f32_to_f16(void* dst_half, const float* src, int64_t count, void* stream)
{
    if (count < 0 || (count > 0 && (!dst_half || !src))) return CONEF_ERR_INVALID;
    if (count == 0) return CONEF_OK;
    hipLaunchKernelGGL((convert_kernel<__half, float>), dim3(grid_for(count, 256)), dim3(256), 0,
                       (hipStream_t)stream, (__half*)dst_half, src, count);
    return (int)hipGetLastError();
}

}  // extern "C"
