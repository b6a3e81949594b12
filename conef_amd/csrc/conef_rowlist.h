// Row-list sketch accumulation: the count-sketch update without atomics for rows that fit LDS.
//
// The bucket and sign of a column depend on the column alone, so every row of an [n,d] tensor
// scatters the same way.  A plan built once per sketch lists, per bucket, the columns that fall
// into it (ascending).  A workgroup then takes a tile of `rb` consecutive rows:
//
//   (the bucket lists and their offsets, d + w small integers, are requested first and parked in
//   LDS once the tile is staged)
//   stage   the values to be sketched are produced in column order with 16-byte accesses and
//           parked in LDS; whatever the fused step has to do in column order (payload, writing
//           the decompressed gradient, the low-rank product) happens here;
//   gather  one thread per (row, bucket) walks the bucket's list, picks its values out of LDS
//           and adds the terms in ascending column order; the new cell leaves with a coalesced
//           store.
//
// No atomics, one read of the tensor, deterministic, and the order of the adds is the CPU
// oracle's, so the sketch comes out bit for bit.  cs_out may be cs_in: a tile reads its rows'
// old cells before it writes them and no other tile touches those rows.
#pragma once
#include "conef_device.h"
#include "conef_sketch_core.h"

constexpr int kConefRowlistThreads = 256;
constexpr int64_t kConefRowlistMaxCols = 24576;       // 4 B value + 2 B list entry per column in LDS
constexpr size_t kConefRowlistLdsLimit = 160 * 1024;   // LDS of a gfx950 CU

struct ConefRowlistView {
    const uint32_t* csr;   // [w+1] first list entry of bucket j
    const uint16_t* ent;   // [d] column | sign bit << 15, buckets ascending, columns ascending
    const uint32_t* pk;    // [d] bucket | sign bit << 31 of every column
};

struct ConefRowlistShape {
    int rb;          // rows per tile
    size_t lds;      // bytes of dynamic LDS
    int64_t tiles;
};

inline size_t conef_rowlist_lds(int rb, int64_t d, int32_t w, bool cells)
{
    size_t vals = (((size_t)rb * d + 3) & ~(size_t)3) * 4;
    size_t ent = (((size_t)d + 7) & ~(size_t)7) * 2;
    size_t csr = (((size_t)w + 1 + 3) & ~(size_t)3) * 4;
    (void)cells;      // every front parks the tile's old sketch rows in LDS
    return vals + ent + csr + (size_t)rb * w * 4;
}

// Rows per tile: about 32 KB of values (several tiles per CU), but no more than leaves a
// thousand tiles for the 256 CUs.
// `companions`: matrices of about this size that share the launch (a batch leaves enough tiles
// for the machine with taller tiles per matrix); 0: full-height tiles whatever the count (for a
// batch whose caller has checked that it has tiles enough that way).
inline bool conef_rowlist_shape(int64_t n, int64_t d, int32_t w, bool cells, ConefRowlistShape* s, int companions = 1)
{
    if (d < 1 || d > kConefRowlistMaxCols || n < 1 || w < 1) return false;
    int64_t rb = 8192 / d;
    // tiles to spare: half-height ones, twice as many resident per CU (a quarter was slower again)
    if (rb >= 2 && n / rb >= 2048) rb = (rb + 1) / 2;
    if (companions > 0 && rb > n * companions / 1024) rb = n * companions / 1024;
    if (rb > 16) rb = 16;
    if (rb < 1) rb = 1;
    while (rb > 1 && conef_rowlist_lds((int)rb, d, w, cells) > 64 * 1024) --rb;
    // rows that are not a whole number of 16-byte quads: tiles of 2 (4) rows start on a quad again,
    // and the fronts then read a tile as one flat run of quads
    if (d % 4 == 2 && rb > 1) rb &= ~(int64_t)1;
    else if (d % 2 == 1 && rb >= 4) rb &= ~(int64_t)3;
    size_t lds = conef_rowlist_lds((int)rb, d, w, cells);
    if (lds > kConefRowlistLdsLimit) return false;
    s->rb = (int)rb;
    s->lds = lds;
    s->tiles = (n + rb - 1) / rb;
    return s->tiles <= 0x7fffffff;
}

// ------------------------------------------------------------------ fronts ----
// A front fills vals[row_in_tile * d + col] for the tile's rows.  `cells` (only when
// kNeedsCells) holds the tile's old sketch rows, [rows][w].

// DenseCS.update: the value is the dense tensor itself.
struct ConefListVec {
    const float* vec;
    bool vec_ok;           // base 16-byte aligned and d % 4 == 0 (the tile copy works either way)
    static constexpr bool kNeedsCells = false;
    __device__ __forceinline__ void stage(int64_t row0, int rows, int d, int, float* vals, const float*,
                                          const uint32_t*) const
    {
        const float* base = vec + row0 * d;
        const int total = rows * d;
        // A tile is one contiguous run: up to three leading elements bring it to a 16-byte
        // boundary, 16-byte loads from there (eight in flight per thread; indices past the end are
        // clamped, not branched around), the last few elements one by one.
        int lead = (int)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(base) & 15u)) & 15u) >> 2);
        if (lead > total) lead = total;
        const int total4 = (total - lead) >> 2;
        const float4* src4 = reinterpret_cast<const float4*>(base + lead);
        for (int q0 = threadIdx.x; q0 < total4; q0 += 8 * kConefRowlistThreads) {
            float4 t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                int q = q0 + u * kConefRowlistThreads;
                t[u] = src4[q < total4 ? q : total4 - 1];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                int q = q0 + u * kConefRowlistThreads;
                if (q < total4) {
                    if (lead == 0) {
                        reinterpret_cast<float4*>(vals)[q] = t[u];
                    } else {
                        float* o = vals + lead + (q << 2);
                        o[0] = t[u].x; o[1] = t[u].y; o[2] = t[u].z; o[3] = t[u].w;
                    }
                }
            }
        }
        const int rest = total - (total4 << 2);          // leading and trailing elements, at most 6
        if ((int)threadIdx.x < rest) {
            const int e = (int)threadIdx.x < lead ? (int)threadIdx.x : (int)threadIdx.x + (total4 << 2);
            vals[e] = base[e];
        }
    }
};

// RandomBlock + ConEF (reference: communication/RandomBlock_hook.py:190,216-243,272-280 at world
// size 1): xq = x + alpha * unsketch(old cells); inside the wrap-around block xq goes to the
// payload and stays in x and a zero is sketched, outside x becomes zero and xq is sketched.
struct ConefListRandBlock {
    float* x;
    float* payload;
    ConefBlock blk;
    float alpha;
    bool vec_ok;
    static constexpr bool kNeedsCells = true;

    __device__ __forceinline__ float finish(int64_t f, float g, float cell, uint32_t pk, float* out) const
    {
        float xq = __fadd_rn(g, conef_query_term(cell, pk, alpha));
        int64_t pos = conef_payload_pos(f, blk);
        if (pos >= 0) {
            payload[pos] = xq;
            *out = xq;
            return 0.f;
        }
        *out = 0.f;
        return xq;
    }

    __device__ __forceinline__ void stage(int64_t row0, int rows, int d, int w, float* vals, const float* cells,
                                          const uint32_t* pk) const
    {
        const int64_t f0 = row0 * d;
        float* base = x + f0;
        if (vec_ok) {
            const int d4 = d >> 2, total4 = rows * d4;
            int row = threadIdx.x / d4, c4 = threadIdx.x - row * d4;
            const int srow = kConefRowlistThreads / d4, sc = kConefRowlistThreads - srow * d4;
            for (int q0 = threadIdx.x; q0 < total4; q0 += 4 * kConefRowlistThreads) {
                float4 g[4];
                uint4 p[4];
                int rw[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {      // four quads in flight; past the end: a valid address, result unused
                    int q = q0 + u * kConefRowlistThreads;
                    bool in = q < total4;
                    g[u] = reinterpret_cast<const float4*>(base)[in ? q : total4 - 1];
                    p[u] = reinterpret_cast<const uint4*>(pk)[in ? c4 : 0];
                    rw[u] = in ? row : 0;
                    row += srow;
                    c4 += sc;
                    if (c4 >= d4) {
                        c4 -= d4;
                        ++row;
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    int q = q0 + u * kConefRowlistThreads;
                    if (q >= total4) break;
                    const float* cr = cells + rw[u] * w;
                    float c0 = cr[p[u].x & 0x7fffffffu], c1 = cr[p[u].y & 0x7fffffffu];
                    float c2 = cr[p[u].z & 0x7fffffffu], c3 = cr[p[u].w & 0x7fffffffu];
                    int64_t f = f0 + ((int64_t)q << 2);
                    float4 o, v;
                    if ((f < blk.end && f + 4 > blk.start) || f < blk.rest) {
                        v.x = finish(f, g[u].x, c0, p[u].x, &o.x);
                        v.y = finish(f + 1, g[u].y, c1, p[u].y, &o.y);
                        v.z = finish(f + 2, g[u].z, c2, p[u].z, &o.z);
                        v.w = finish(f + 3, g[u].w, c3, p[u].w, &o.w);
                    } else {      // the block is one wrap-around range: most quads are entirely outside it
                        o = make_float4(0.f, 0.f, 0.f, 0.f);
                        v.x = __fadd_rn(g[u].x, conef_query_term(c0, p[u].x, alpha));
                        v.y = __fadd_rn(g[u].y, conef_query_term(c1, p[u].y, alpha));
                        v.z = __fadd_rn(g[u].z, conef_query_term(c2, p[u].z, alpha));
                        v.w = __fadd_rn(g[u].w, conef_query_term(c3, p[u].w, alpha));
                    }
                    reinterpret_cast<float4*>(base)[q] = o;
                    reinterpret_cast<float4*>(vals)[q] = v;
                }
            }
        } else {
            // Rows that are not whole aligned quads: the tile as one flat run.  Up to three leading
            // elements bring it to a 16-byte boundary; from there quads, whose four elements may
            // sit in two rows; the last few elements one by one.
            const int total = rows * d;
            int lead = (int)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(base) & 15u)) & 15u) >> 2);
            if (lead > total) lead = total;
            const int total4 = (total - lead) >> 2;
            float4* base4 = reinterpret_cast<float4*>(base + lead);
            for (int q0 = threadIdx.x; q0 < total4; q0 += 4 * kConefRowlistThreads) {
                float4 g[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    int q = q0 + u * kConefRowlistThreads;
                    g[u] = base4[q < total4 ? q : total4 - 1];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    int q = q0 + u * kConefRowlistThreads;
                    if (q >= total4) break;
                    const int e = lead + (q << 2);
                    int row = e / d, col = e - row * d;
                    const float gv[4] = {g[u].x, g[u].y, g[u].z, g[u].w};
                    uint32_t p[4];
                    float c[4], o[4], v[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        p[k] = pk[col];
                        c[k] = cells[row * w + (p[k] & 0x7fffffffu)];
                        if (++col == d) {
                            col = 0;
                            ++row;
                        }
                    }
                    const int64_t f = f0 + e;
                    if ((f < blk.end && f + 4 > blk.start) || f < blk.rest) {
#pragma unroll
                        for (int k = 0; k < 4; ++k) v[k] = finish(f + k, gv[k], c[k], p[k], &o[k]);
                    } else {
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            o[k] = 0.f;
                            v[k] = __fadd_rn(gv[k], conef_query_term(c[k], p[k], alpha));
                        }
                    }
                    base4[q] = make_float4(o[0], o[1], o[2], o[3]);
                    if (lead == 0) {
                        reinterpret_cast<float4*>(vals)[q] = make_float4(v[0], v[1], v[2], v[3]);
                    } else {
#pragma unroll
                        for (int k = 0; k < 4; ++k) vals[e + k] = v[k];
                    }
                }
            }
            const int rest = total - (total4 << 2);      // leading and trailing elements, at most 6
            if ((int)threadIdx.x < rest) {
                const int e = (int)threadIdx.x < lead ? (int)threadIdx.x : (int)threadIdx.x + (total4 << 2);
                const int row = e / d, col = e - row * d;
                const uint32_t p = pk[col];
                float o;
                vals[e] = finish(f0 + e, base[e], cells[row * w + (p & 0x7fffffffu)], p, &o);
                base[e] = o;
            }
        }
    }
};

// ------------------------------------------------------------------ kernel ----
// count >= 1 words from global memory to LDS, eight loads in flight per thread
__device__ __forceinline__ void conef_copy_words_to_lds(uint32_t* dst, const uint32_t* __restrict__ src, int count)
{
    for (int i0 = threadIdx.x; i0 < count; i0 += 8 * kConefRowlistThreads) {
        uint32_t t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            int i = i0 + u * kConefRowlistThreads;
            t[u] = src[i < count ? i : count - 1];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            int i = i0 + u * kConefRowlistThreads;
            if (i < count) dst[i] = t[u];
        }
    }
}

template <typename CsT, typename Front>
__device__ __forceinline__ void
conef_rowlist_body(const Front& front, ConefRowlistView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int d, int w,
                   int rb, double one_minus_beta, int bx)
{
    extern __shared__ float conef_rl[];
    float* vals = conef_rl;
    uint16_t* ent_l = reinterpret_cast<uint16_t*>(vals + ((rb * d + 3) & ~3));
    uint32_t* csr_l = reinterpret_cast<uint32_t*>(ent_l + ((d + 7) & ~7));
    float* cells = reinterpret_cast<float*>(csr_l + ((w + 1 + 3) & ~3));
    const int64_t row0 = (int64_t)bx * rb;
    const int rows = n - row0 < rb ? (int)(n - row0) : rb;

    // The bucket lists (two entries per load; the table is padded to a multiple of 256 bytes) and
    // their offsets are only needed by the walk: the first words of both are requested now and
    // parked after the tile has been staged, so that they travel while the tile does.
    constexpr int kPreE = 8, kPreC = 2;
    const int ent_words = (d + 1) >> 1, csr_words = w + 1;
    const uint32_t* ent_src = reinterpret_cast<const uint32_t*>(plan.ent);
    uint32_t ent_pre[kPreE], csr_pre[kPreC];
#pragma unroll
    for (int u = 0; u < kPreE; ++u) {
        const int i = threadIdx.x + u * kConefRowlistThreads;
        ent_pre[u] = ent_src[i < ent_words ? i : ent_words - 1];
    }
#pragma unroll
    for (int u = 0; u < kPreC; ++u) {
        const int i = threadIdx.x + u * kConefRowlistThreads;
        csr_pre[u] = plan.csr[i < csr_words ? i : csr_words - 1];
    }
    if (Front::kNeedsCells) {
        const CsT* src = cs_in + row0 * w;
        const int count = rows * w;
        for (int i0 = threadIdx.x; i0 < count; i0 += 4 * kConefRowlistThreads) {
            float t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int i = i0 + u * kConefRowlistThreads;
                t[u] = conef_ld(src + (i < count ? i : count - 1));
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int i = i0 + u * kConefRowlistThreads;
                if (i < count) cells[i] = t[u];
            }
        }
        __syncthreads();
    }
    // The tile's cells are rows * w consecutive values; thread t owns cells t, t + 256, ...  Fronts
    // that do not need the old rows for staging request their cells now, so that the values arrive
    // while the tile is staged, and park them in LDS before the barrier.
    const int total = rows * w;
    constexpr int kPre = 8;
    float aux_pre[kPre];
    if (!Front::kNeedsCells) {
#pragma unroll
        for (int u = 0; u < kPre; ++u) {
            const int p = threadIdx.x + u * kConefRowlistThreads;
            aux_pre[u] = conef_ld(cs_in + row0 * w + (p < total ? p : total - 1));
        }
    }
    front.stage(row0, rows, d, w, vals, cells, plan.pk);
    {
        uint32_t* ent_w = reinterpret_cast<uint32_t*>(ent_l);
#pragma unroll
        for (int u = 0; u < kPreE; ++u) {
            const int i = threadIdx.x + u * kConefRowlistThreads;
            if (i < ent_words) ent_w[i] = ent_pre[u];
        }
#pragma unroll
        for (int u = 0; u < kPreC; ++u) {
            const int i = threadIdx.x + u * kConefRowlistThreads;
            if (i < csr_words) csr_l[i] = csr_pre[u];
        }
        if (ent_words > kPreE * kConefRowlistThreads)
            conef_copy_words_to_lds(ent_w + kPreE * kConefRowlistThreads, ent_src + kPreE * kConefRowlistThreads,
                                    ent_words - kPreE * kConefRowlistThreads);
        if (csr_words > kPreC * kConefRowlistThreads)
            conef_copy_words_to_lds(csr_l + kPreC * kConefRowlistThreads, plan.csr + kPreC * kConefRowlistThreads,
                                    csr_words - kPreC * kConefRowlistThreads);
    }
    if (!Front::kNeedsCells) {
#pragma unroll
        for (int u = 0; u < kPre; ++u) {
            const int p = threadIdx.x + u * kConefRowlistThreads;
            if (p < total) cells[p] = aux_pre[u];
        }
        for (int p = threadIdx.x + kPre * kConefRowlistThreads; p < total; p += kConefRowlistThreads)
            cells[p] = conef_ld(cs_in + row0 * w + p);
    }
    __syncthreads();

    int row = threadIdx.x / w, j = threadIdx.x - row * w;
    const int srow = kConefRowlistThreads / w, sj = kConefRowlistThreads - srow * w;
    for (int p = threadIdx.x; p < total; p += kConefRowlistThreads) {
        const uint32_t e0 = csr_l[j], e1 = csr_l[j + 1];
        const float aux = cells[p];
        const double decay = __dmul_rn(one_minus_beta, (double)aux);
        const float* vr = vals + row * d;
        float acc = aux;
        for (uint32_t e = e0; e < e1; ++e) {
            uint32_t en = ent_l[e];
            uint32_t flip = ((~en) & 0x8000u) << 16;      // sign bit clear (-1): flip the float's sign
            double sv = (double)__uint_as_float(__float_as_uint(vr[en & 0x7fffu]) ^ flip);
            acc = __fadd_rn(acc, (float)__dsub_rn(sv, decay));
        }
        conef_st(cs_out + row0 * w + p, acc);
        row += srow;
        j += sj;
        if (j >= w) {
            j -= w;
            ++row;
        }
    }
}

template <typename CsT, typename Front>
__global__ void __launch_bounds__(kConefRowlistThreads)
conef_rowlist_kernel(Front front, ConefRowlistView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int d, int w,
                     int rb, double one_minus_beta)
{
    conef_rowlist_body<CsT, Front>(front, plan, cs_in, cs_out, n, d, w, rb, one_minus_beta, (int)blockIdx.x);
}

template <typename CsT, typename Front>
int conef_launch_rowlist(Front front, ConefRowlistView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int64_t d,
                         int32_t w, float beta, hipStream_t s)
{
    ConefRowlistShape shape;
    if (!conef_rowlist_shape(n, d, w, Front::kNeedsCells, &shape)) return CONEF_ERR_INVALID;
    auto k = conef_rowlist_kernel<CsT, Front>;
    if (shape.lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shape.lds);
        if (e != hipSuccess) return (int)e;
    }
    const double omb = 1. - (double)beta;   // (1. - beta) with beta an fp32 value, CountSketch.py:38,63
    hipLaunchKernelGGL(k, dim3((unsigned)shape.tiles), dim3(kConefRowlistThreads), shape.lds, s, front, plan, cs_in,
                       cs_out, n, (int)d, (int)w, shape.rb, omb);
    return (int)hipGetLastError();
}
