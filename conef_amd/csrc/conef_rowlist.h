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
//           and adds the terms in ascending column order, several entries a trip; buckets are
//           handed out in the order of falling list length (a table of the plan), so that the
//           lanes of a wave have lists of about the same length to walk.
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
    const uint16_t* order; // [w] the buckets by falling list length
};

struct ConefRowlistShape {
    int rb;          // rows per tile
    size_t lds;      // bytes of dynamic LDS
    int64_t tiles;
    bool pk_lds;     // the column table (bucket and sign per column) has room in LDS behind the cells
};

// Fronts that read the old cells while they stage look up every column's bucket there too.
inline size_t conef_rowlist_pk_bytes(int64_t d) { return (((size_t)d + 3) & ~(size_t)3) * 4; }

inline size_t conef_rowlist_lds(int rb, int64_t d, int32_t w, bool cells)
{
    size_t vals = (((size_t)rb * d + 3) & ~(size_t)3) * 4;
    size_t ent = (((size_t)d + 7) & ~(size_t)7) * 2;
    size_t csr = (((size_t)w + 1 + 3) & ~(size_t)3) * 4;
    size_t ord = (((size_t)w + 7) & ~(size_t)7) * 2;
    (void)cells;      // every front parks the tile's old sketch rows in LDS
    return vals + ent + csr + ord + (size_t)rb * w * 4;
}

// Rows per tile: about 32 KB of values (several tiles per CU), but no more than leaves a
// thousand tiles for the 256 CUs.
// `companions`: matrices of about this size that share the launch (a batch leaves enough tiles
// for the machine with taller tiles per matrix); 0: full-height tiles whatever the count (for a
// batch whose caller has checked that it has tiles enough that way).
inline bool conef_rowlist_shape(int64_t n, int64_t d, int32_t w, bool cells, ConefRowlistShape* s, int companions = 1)
{
    if (d < 1 || d > kConefRowlistMaxCols || n < 1 || w < 1 || w > 0xffff) return false;
    int64_t rb = 8192 / d;
    // tiles to spare: half-height ones, twice as many resident per CU (a quarter was slower again)
    if (rb >= 2 && n / rb >= 2048) rb = (rb + 1) / 2;
    if (companions > 0 && rb > n * companions / 1024) rb = n * companions / 1024;
    if (rb > 16) rb = 16;
    if (rb < 1) rb = 1;
    // the column table goes to LDS where a tile has at least two rows to use it for (a launch takes
    // the LDS of its largest tile for every tile, and a one-row tile would double that for nothing)
    const size_t pk = cells && rb >= 2 ? conef_rowlist_pk_bytes(d) : 0;
    while (rb > 1 && conef_rowlist_lds((int)rb, d, w, cells) + pk > 64 * 1024) --rb;
    // rows that are not a whole number of 16-byte quads: tiles of 2 (4) rows start on a quad again,
    // and the fronts then read a tile as one flat run of quads
    if (d % 4 == 2 && rb > 1) rb &= ~(int64_t)1;
    else if (d % 2 == 1 && rb >= 4) rb &= ~(int64_t)3;
    size_t lds = conef_rowlist_lds((int)rb, d, w, cells);
    if (lds > kConefRowlistLdsLimit) return false;
    s->pk_lds = pk > 0 && rb >= 2 && lds + pk <= kConefRowlistLdsLimit;
    if (s->pk_lds) lds += pk;
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
    struct Regs {};
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
//
// The tile is one flat run of quads (up to three leading elements bring it to a 16-byte boundary,
// the last few go one by one).  The first kQuads quads of a thread are requested before the old
// cells and the column table are parked in LDS (`request`), so that the tile travels with them;
// `stage` then works from LDS: row and column of a quad advance with it (no division per quad),
// the block is a pair of tile-relative ranges, and a tile that does not touch the block at all -
// most of them - runs without any of that.
struct ConefListRandBlock {
    float* x;
    float* payload;
    ConefBlock blk;
    float alpha;
    static constexpr bool kNeedsCells = true;
    static constexpr int kQuads = 4;
    struct Regs {          // a thread's first kQuads quads, by name: no array for the compiler to keep in memory
        float4 g0, g1, g2, g3;
    };

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

    static __device__ __forceinline__ int lead_of(const float* base, int total)
    {
        int lead = (int)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(base) & 15u)) & 15u) >> 2);
        return lead > total ? total : lead;
    }

    __device__ __forceinline__ Regs request(int64_t row0, int rows, int d) const
    {
        const float* base = x + row0 * d;
        const int total = rows * d, lead = lead_of(base, total), total4 = (total - lead) >> 2;
        const float4* base4 = reinterpret_cast<const float4*>(base + lead);
        Regs r;
        r.g0 = r.g1 = r.g2 = r.g3 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (total4 > 0) {
            const int q = threadIdx.x, last = total4 - 1;      // past the end: a valid address, result unused
            r.g0 = base4[q < last ? q : last];
            r.g1 = base4[q + kConefRowlistThreads < last ? q + kConefRowlistThreads : last];
            r.g2 = base4[q + 2 * kConefRowlistThreads < last ? q + 2 * kConefRowlistThreads : last];
            r.g3 = base4[q + 3 * kConefRowlistThreads < last ? q + 3 * kConefRowlistThreads : last];
        }
        return r;
    }

    // One quad: element e of the tile onwards, which sits in column `col` of the row whose cells
    // start at `roff`.  pk_l: the column table, in LDS or (rows too long for that) in global memory.
    template <bool BLOCK>
    __device__ __forceinline__ void quad(float4 g, int q, int e, int col, int roff, float4* base4, int64_t f0,
                                         int lead, int d, int w, float* vals, const float* cells,
                                         const uint32_t* pk_l, int lo, int hi, int rest) const
    {
        const float gv[4] = {g.x, g.y, g.z, g.w};
        float o[4], v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            int c = col + k, ro = roff;
            if (c >= d) {
                c -= d;
                ro += w;
                if (d < 4)                     // a quad may then cross several rows
                    while (c >= d) {
                        c -= d;
                        ro += w;
                    }
            }
            const uint32_t p = pk_l[c];
            const float xq = __fadd_rn(gv[k], conef_query_term(cells[ro + (p & 0x7fffffffu)], p, alpha));
            const int ek = e + k;
            if (BLOCK && ((ek >= lo && ek < hi) || ek < rest)) {
                payload[conef_payload_pos(f0 + ek, blk)] = xq;
                o[k] = xq;
                v[k] = 0.f;
            } else {
                o[k] = 0.f;
                v[k] = xq;
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

    template <bool BLOCK>
    __device__ __forceinline__ void quads(Regs r, float* base, int64_t f0, int lead, int total4, int d, int w,
                                          float* vals, const float* cells, const uint32_t* pk_l, int lo, int hi,
                                          int rest) const
    {
        float4* base4 = reinterpret_cast<float4*>(base + lead);
        constexpr int kStep = 4 * kConefRowlistThreads;          // elements between a thread's quads
        const int drow = kStep / d, dcol = kStep - drow * d;
        int q = threadIdx.x;
        int e = lead + (q << 2);
        int col = e % d;
        int roff = (e / d) * w;
        auto one = [&](float4 g) {
            if (q < total4) quad<BLOCK>(g, q, e, col, roff, base4, f0, lead, d, w, vals, cells, pk_l, lo, hi, rest);
            q += kConefRowlistThreads;
            e += kStep;
            col += dcol;
            roff += drow * w;
            if (col >= d) {
                col -= d;
                roff += w;
            }
        };
        one(r.g0);
        one(r.g1);
        one(r.g2);
        one(r.g3);
        while (q < total4) {                 // taller tiles: four more quads a trip
            const int last = total4 - 1;
            const float4 g0 = base4[q];
            const float4 g1 = base4[q + kConefRowlistThreads < last ? q + kConefRowlistThreads : last];
            const float4 g2 = base4[q + 2 * kConefRowlistThreads < last ? q + 2 * kConefRowlistThreads : last];
            const float4 g3 = base4[q + 3 * kConefRowlistThreads < last ? q + 3 * kConefRowlistThreads : last];
            one(g0);
            one(g1);
            one(g2);
            one(g3);
        }
    }

    __device__ __forceinline__ void stage(Regs r, int64_t row0, int rows, int d, int w, float* vals,
                                          const float* cells, const uint32_t* pk_l) const
    {
        const int64_t f0 = row0 * d;
        float* base = x + f0;
        const int total = rows * d, lead = lead_of(base, total), total4 = (total - lead) >> 2;
        // the block's two ranges, [start,end) and [0,rest), relative to the tile
        const int64_t a0 = blk.start - f0, a1 = blk.end - f0, a2 = blk.rest - f0;
        const int lo = a0 < 0 ? 0 : a0 > total ? total : (int)a0;
        const int hi = a1 < 0 ? 0 : a1 > total ? total : (int)a1;
        const int rest = a2 < 0 ? 0 : a2 > total ? total : (int)a2;
        if (hi > lo || rest > 0) quads<true>(r, base, f0, lead, total4, d, w, vals, cells, pk_l, lo, hi, rest);
        else quads<false>(r, base, f0, lead, total4, d, w, vals, cells, pk_l, 0, 0, 0);
        const int tail = total - (total4 << 2);      // leading and trailing elements, at most 6
        if ((int)threadIdx.x < tail) {
            const int e = (int)threadIdx.x < lead ? (int)threadIdx.x : (int)threadIdx.x + (total4 << 2);
            const int row = e / d, col = e - row * d;
            const uint32_t p = pk_l[col];
            float o;
            vals[e] = finish(f0 + e, base[e], cells[row * w + (p & 0x7fffffffu)], p, &o);
            base[e] = o;
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
                   int rb, double one_minus_beta, int bx, bool pk_lds = false)
{
    extern __shared__ float conef_rl[];
    float* vals = conef_rl;
    uint16_t* ent_l = reinterpret_cast<uint16_t*>(vals + ((rb * d + 3) & ~3));
    uint32_t* csr_l = reinterpret_cast<uint32_t*>(ent_l + ((d + 7) & ~7));
    uint16_t* ord_l = reinterpret_cast<uint16_t*>(csr_l + ((w + 1 + 3) & ~3));
    float* cells = reinterpret_cast<float*>(ord_l + ((w + 7) & ~7));
    const int64_t row0 = (int64_t)bx * rb;
    const int rows = n - row0 < rb ? (int)(n - row0) : rb;

    // The bucket lists (two entries per load; the table is padded to a multiple of 256 bytes) and
    // their offsets are only needed by the walk: the first words of both are requested now and
    // parked after the tile has been staged, so that they travel while the tile does.
    constexpr int kPreE = 8, kPreC = 2;
    const int ent_words = (d + 1) >> 1, csr_words = w + 1, ord_words = (w + 1) >> 1;
    const uint32_t* ent_src = reinterpret_cast<const uint32_t*>(plan.ent);
    const uint32_t* ord_src = reinterpret_cast<const uint32_t*>(plan.order);
    uint32_t ent_pre[kPreE], csr_pre[kPreC];
    const uint32_t ord_pre = ord_src[(int)threadIdx.x < ord_words ? (int)threadIdx.x : ord_words - 1];
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
    typename Front::Regs regs;
    uint32_t* pk_l = reinterpret_cast<uint32_t*>(cells + rb * w);
    if constexpr (Front::kNeedsCells) {
        // The tile's first quads, its rows' old cells and the column table are requested together;
        // cells and table are parked in LDS, the quads wait in registers.
        regs = front.request(row0, rows, d);
        const CsT* src = cs_in + row0 * w;
        const int count = rows * w;
        constexpr int kPark = 4;
        float ct[kPark];
        uint32_t pt[kPark];
#pragma unroll
        for (int u = 0; u < kPark; ++u) {
            const int i = threadIdx.x + u * kConefRowlistThreads;
            ct[u] = conef_ld(src + (i < count ? i : count - 1));
            pt[u] = plan.pk[i < d ? i : d - 1];
        }
#pragma unroll
        for (int u = 0; u < kPark; ++u) {
            const int i = threadIdx.x + u * kConefRowlistThreads;
            if (i < count) cells[i] = ct[u];
            if (pk_lds && i < d) pk_l[i] = pt[u];
        }
        for (int i = threadIdx.x + kPark * kConefRowlistThreads; i < count; i += kConefRowlistThreads)
            cells[i] = conef_ld(src + i);
        if (pk_lds)
            for (int i = threadIdx.x + kPark * kConefRowlistThreads; i < d; i += kConefRowlistThreads)
                pk_l[i] = plan.pk[i];
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
    if constexpr (Front::kNeedsCells) {
        if (pk_lds) front.stage(regs, row0, rows, d, w, vals, cells, pk_l);
        else front.stage(regs, row0, rows, d, w, vals, cells, plan.pk);
    }
    else front.stage(row0, rows, d, w, vals, cells, plan.pk);
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
        uint32_t* ord_w = reinterpret_cast<uint32_t*>(ord_l);
        if ((int)threadIdx.x < ord_words) ord_w[threadIdx.x] = ord_pre;
        if (ord_words > kConefRowlistThreads)
            conef_copy_words_to_lds(ord_w + kConefRowlistThreads, ord_src + kConefRowlistThreads,
                                    ord_words - kConefRowlistThreads);
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

    // One thread per (bucket, row), buckets in the order of falling list length and the rows of a
    // bucket on neighbouring lanes: the lanes of a wave walk lists of about the same length (a wave
    // takes as many trips as its longest list).
    constexpr int kWalk = 4;
    int jj = threadIdx.x / rows, row = threadIdx.x - jj * rows;
    const int sjj = kConefRowlistThreads / rows, srow = kConefRowlistThreads - sjj * rows;
    for (int p = threadIdx.x; p < total; p += kConefRowlistThreads) {
        const int j = ord_l[jj];
        const int cell = row * w + j;
        const uint32_t e0 = csr_l[j], e1 = csr_l[j + 1];
        const float aux = cells[cell];
        const double decay = __dmul_rn(one_minus_beta, (double)aux);
        const float* vr = vals + row * d;
        float acc = aux;
        // kWalk entries a trip: their list words and values are requested together and the terms
        // formed side by side; only the adds onto the cell are a chain.  Slots past the end of the
        // list read its last entry and are not added.
        for (uint32_t e = e0; e < e1; e += kWalk) {
            uint32_t en[kWalk];
            float term[kWalk];
#pragma unroll
            for (int u = 0; u < kWalk; ++u) en[u] = ent_l[e + u < e1 ? e + u : e1 - 1];
#pragma unroll
            for (int u = 0; u < kWalk; ++u) {
                uint32_t flip = ((~en[u]) & 0x8000u) << 16;      // sign bit clear (-1): flip the float's sign
                double sv = (double)__uint_as_float(__float_as_uint(vr[en[u] & 0x7fffu]) ^ flip);
                term[u] = (float)__dsub_rn(sv, decay);
            }
#pragma unroll
            for (int u = 0; u < kWalk; ++u)
                if (e + u < e1) acc = __fadd_rn(acc, term[u]);
        }
        conef_st(cs_out + row0 * w + cell, acc);
        jj += sjj;
        row += srow;
        if (row >= rows) {
            row -= rows;
            ++jj;
        }
    }
}

template <typename CsT, typename Front>
__global__ void __launch_bounds__(kConefRowlistThreads)
conef_rowlist_kernel(Front front, ConefRowlistView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int d, int w,
                     int rb, double one_minus_beta, bool pk_lds)
{
    conef_rowlist_body<CsT, Front>(front, plan, cs_in, cs_out, n, d, w, rb, one_minus_beta, (int)blockIdx.x, pk_lds);
}

template <typename CsT, typename Front>
int conef_launch_rowlist(Front front, ConefRowlistView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int64_t d,
                         int32_t w, float beta, hipStream_t s)
{
    ConefRowlistShape shape;
    if (!conef_rowlist_shape(n, d, w, Front::kNeedsCells, &shape)) return CONEF_ERR_INVALID;
    auto k = conef_rowlist_kernel<CsT, Front>;
    hipError_t e = conef_allow_lds((const void*)k, shape.lds);
    if (e != hipSuccess) return (int)e;
    const double omb = 1. - (double)beta;   // (1. - beta) with beta an fp32 value, CountSketch.py:38,63
    hipLaunchKernelGGL(k, dim3((unsigned)shape.tiles), dim3(kConefRowlistThreads), shape.lds, s, front, plan, cs_in,
                       cs_out, n, (int)d, (int)w, shape.rb, omb, shape.pk_lds);
    return (int)hipGetLastError();
}
