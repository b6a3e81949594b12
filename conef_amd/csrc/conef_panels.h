// Row lists in column panels: the count-sketch update without atomics for rows that are too long
// for conef_rowlist.h (a row's values, its bucket lists and its cells together exceed LDS), on
// matrices with rows enough to fill the machine - e.g. a [4096, 25088] fully connected layer.
//
// A workgroup takes a tile of `rb` rows and keeps that tile's sketch cells in LDS for the whole
// kernel: the old values (every term's decay reads the cell as it was before the call,
// CountSketch.py:47-52,63) and the running sums.  The columns go by in panels of `pc`:
//
//   park    the panel's values are read in column order with 16-byte accesses, with whatever the
//           fused step has to do in column order (the `front`), and the term each adds to its cell
//           is parked in LDS at the place the plan names for its column (`epos`: which entry of
//           the panel the column is | sign << 15; `colb`: its bucket): the panel's columns grouped
//           by bucket, ascending inside a group;
//   walk    `entg` (by entry: its bucket | the length of the group it opens << 16, zero for the
//           other entries of a group) says where a group starts and ends.  The thread that meets
//           a group's first entry adds the group's terms, which now sit side by side, onto the
//           cell in that order; the other threads of the group have nothing to do.
//
// Panels are taken in ascending order, so a cell receives its terms in ascending column order:
// the CPU oracle's order, bit for bit, no atomics, one read of the tensor.  cs_out may be cs_in.
#pragma once
#include "conef_device.h"
#include "conef_sketch_core.h"

constexpr int kConefPanelThreads = 1024;    // a walk is chains of LDS trips: many waves a CU hide them
constexpr size_t kConefPanelLdsLimit = 156 * 1024;

struct ConefPanelView {
    const uint32_t* entg;   // [d] by panel, grouped by bucket (columns ascending inside a group): the entry's
                            // bucket | (entries in the group, if this is its first, else 0) << 16
    const uint16_t* epos;   // [d] by column: which entry of its panel the column is | sign bit << 15
    const uint16_t* colb;   // [d] by column: the column's bucket
    int pc;                 // columns per panel (a multiple of 8, at most 4096)
};

struct ConefPanelShape {
    int rb;          // rows per tile
    int pc;          // columns per panel
    size_t lds;
    int64_t tiles;
};

__host__ __device__ inline size_t conef_panel_cells(int rb, int32_t w) { return (((size_t)rb * w + 3) & ~(size_t)3); }

inline size_t conef_panel_lds(int rb, int pc, int32_t w)
{
    return (size_t)rb * pc * 4 + (size_t)pc * 4 + 16 + 2 * conef_panel_cells(rb, w) * 4;
}

// Tile height and panel width are functions of (d, w) alone, so that one plan serves every matrix of
// that row length and sketch width.  Two workgroups a CU where the cells leave room for it (their
// barriers then overlap), one otherwise.
inline bool conef_panel_shape(int64_t n, int64_t d, int32_t w, ConefPanelShape* s)
{
    if (d < 1 || d > 0x7fffffffLL || n < 1 || w < 1 || w > 0xffff) return false;
    static const size_t limits[2] = {78 * 1024, kConefPanelLdsLimit};
    for (size_t limit : limits) {
        for (int rb = 4; rb >= 1; rb >>= 1) {
            for (int elems = 8192; elems >= 2048; elems >>= 1) {
                int pc = elems / rb;
                if (pc > 4096) continue;             // an entry index has 12 bits; a thread parks two quads of values
                if ((int64_t)pc > ((d + 7) & ~(int64_t)7)) pc = (int)((d + 7) & ~(int64_t)7);
                size_t lds = conef_panel_lds(rb, pc, w);
                if (lds > limit) continue;
                s->rb = rb;
                s->pc = pc;
                s->lds = lds;
                s->tiles = (n + rb - 1) / rb;
                return s->tiles <= 0x7fffffff;
            }
        }
    }
    return false;
}

// ------------------------------------------------------------------ fronts ----
// A front supplies the value to be sketched for element (row, col) from the element's raw value g,
// the old sketch cell it maps to and its (bucket | sign << 31) word, with the side effects of the
// fused step; `raw` names the tensor the raw values are read from.

// DenseCS.update: the value is the dense tensor itself.
struct ConefPanelVec {
    const float* vec;
    bool vec_ok;           // base 16-byte aligned and d % 4 == 0
    __device__ __forceinline__ const float* raw() const { return vec; }
    __device__ __forceinline__ float4 value4(int64_t, float4 g, const float*, const uint32_t*) const { return g; }
    __device__ __forceinline__ float value(int64_t, float g, float, uint32_t) const { return g; }
};

// RandomBlock + ConEF (reference: communication/RandomBlock_hook.py:190,216-243,272-280 at world
// size 1): xq = x + alpha * unsketch(old cells); inside the wrap-around block xq goes to the
// payload and stays in x and a zero is sketched, outside x becomes zero and xq is sketched.
struct ConefPanelRandBlock {
    float* x;
    float* payload;
    ConefBlock blk;
    float alpha;
    bool vec_ok;
    __device__ __forceinline__ const float* raw() const { return x; }
    __device__ __forceinline__ float one(int64_t f, float g, float cell, uint32_t p, float* out) const
    {
        const float xq = __fadd_rn(g, conef_query_term(cell, p, alpha));
        const int64_t pos = conef_payload_pos(f, blk);
        if (pos >= 0) {
            payload[pos] = xq;
            *out = xq;
            return 0.f;
        }
        *out = 0.f;
        return xq;
    }
    __device__ __forceinline__ float4 value4(int64_t f, float4 g, const float* cell, const uint32_t* p) const
    {
        float4 o, v;
        v.x = one(f, g.x, cell[0], p[0], &o.x);
        v.y = one(f + 1, g.y, cell[1], p[1], &o.y);
        v.z = one(f + 2, g.z, cell[2], p[2], &o.z);
        v.w = one(f + 3, g.w, cell[3], p[3], &o.w);
        *reinterpret_cast<float4*>(x + f) = o;
        return v;
    }
    __device__ __forceinline__ float value(int64_t f, float g, float cell, uint32_t p) const
    {
        float o;
        const float v = one(f, g, cell, p, &o);
        x[f] = o;
        return v;
    }
};

// ------------------------------------------------------------------ kernel ----
// What a thread has in flight for the next panel while the current one is walked: two quads of
// values with their columns' entry positions and buckets, and four entries of the panel's group table.
struct ConefPanelRegs {      // by name: arrays here end up in scratch memory
    float4 g0, g1;
    uint2 ep0, ep1, cb0, cb1;
    uint4 eg;
};

// quad i of a panel of q_row quads a row -> (row, quad of the row).  Panels are a power of two wide
// except a matrix's last one, so the division is a shift nearly always.
__device__ __forceinline__ void conef_panel_quad_at(int i, int q_row, int* row, int* q)
{
    if ((q_row & (q_row - 1)) == 0) {
        const int sh = 31 - __clz(q_row);
        *row = i >> sh;
        *q = i & (q_row - 1);
    } else {
        *row = i / q_row;
        *q = i - *row * q_row;
    }
}

template <typename Front>
__device__ __forceinline__ void
conef_panel_request(const Front& front, const ConefPanelView& plan, ConefPanelRegs& r, int64_t row0, int rows, int c0, int d)
{
    const int cols = d - c0 < plan.pc ? d - c0 : plan.pc;
    // the panel's group table, four entries a thread (c0 is a multiple of 8; the tables are padded)
    const uint4* gs = reinterpret_cast<const uint4*>(plan.entg + c0);
    const int fours = (cols + 3) >> 2;
    const int i0 = threadIdx.x, i1 = threadIdx.x + kConefPanelThreads;
    r.eg = gs[i0 < fours ? i0 : fours - 1];
    if (!front.vec_ok) return;
    const int q_row = (cols + 3) >> 2;           // d % 4 == 0 and pc % 8 == 0: a panel is whole quads
    const int total = rows * q_row;
    const float* raw = front.raw();
    {
        const int i = i0 < total ? i0 : total - 1;
        int row, q;
        conef_panel_quad_at(i, q_row, &row, &q);
        r.g0 = *reinterpret_cast<const float4*>(raw + (row0 + row) * d + c0 + 4 * q);
        r.ep0 = *reinterpret_cast<const uint2*>(plan.epos + c0 + 4 * q);
        r.cb0 = *reinterpret_cast<const uint2*>(plan.colb + c0 + 4 * q);
    }
    {
        const int i = i1 < total ? i1 : total - 1;
        int row, q;
        conef_panel_quad_at(i, q_row, &row, &q);
        r.g1 = *reinterpret_cast<const float4*>(raw + (row0 + row) * d + c0 + 4 * q);
        r.ep1 = *reinterpret_cast<const uint2*>(plan.epos + c0 + 4 * q);
        r.cb1 = *reinterpret_cast<const uint2*>(plan.colb + c0 + 4 * q);
    }
}

// The term element (row, col) adds to its cell (CountSketch.py:63) goes to terms[entry * rows + row]:
// the walk then finds a group's terms side by side, in the order they are to be added.
template <typename Front>
__device__ __forceinline__ void
conef_panel_park_quad(const Front& front, float4 g, uint2 ep, uint2 cb, int i, int q_row, int64_t row0, int rows, int c0,
                      int d, int w, float* terms, const float* aux, double one_minus_beta)
{
    int row, q;
    conef_panel_quad_at(i, q_row, &row, &q);
    const int64_t f = (row0 + row) * d + c0 + 4 * q;
    const uint32_t e[4] = {ep.x & 0xffffu, ep.x >> 16, ep.y & 0xffffu, ep.y >> 16};
    const uint32_t j[4] = {cb.x & 0xffffu, cb.x >> 16, cb.y & 0xffffu, cb.y >> 16};
    float cell[4];
    uint32_t p[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        cell[k] = aux[row * w + (int)j[k]];
        p[k] = j[k] | ((e[k] >> 15) << 31);
    }
    const float4 v4 = front.value4(f, g, cell, p);
    const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
    for (int k = 0; k < 4; ++k)
        terms[(int)(e[k] & 0x7fffu) * rows + row] = conef_update_term(v[k], cell[k], p[k], one_minus_beta);
}

template <typename CsT, typename Front>
__device__ __forceinline__ void
conef_panel_body(const Front& front, ConefPanelView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int d, int w, int rb,
                 double one_minus_beta, int bx)
{
    extern __shared__ float conef_pl[];
    const int pc = plan.pc;
    float* terms = conef_pl;                                   // [entry][row]
    uint32_t* entg_l = reinterpret_cast<uint32_t*>(terms + rb * pc);
    float* aux = reinterpret_cast<float*>(entg_l + pc + 4);
    float* acc = aux + conef_panel_cells(rb, w);
    const int64_t row0 = (int64_t)bx * rb;
    const int rows = n - row0 < rb ? (int)(n - row0) : rb;
    const int total = rows * w;

    ConefPanelRegs regs;
    conef_panel_request(front, plan, regs, row0, rows, 0, d);
    for (int p = threadIdx.x; p < total; p += kConefPanelThreads) {
        const float c = conef_ld(cs_in + row0 * w + p);
        aux[p] = c;
        acc[p] = c;
    }
    __syncthreads();       // parking reads the old cells
    for (int c0 = 0; c0 < d; c0 += pc) {
        const int cols = d - c0 < pc ? d - c0 : pc;
        if ((int)threadIdx.x < ((cols + 3) >> 2)) reinterpret_cast<uint4*>(entg_l)[threadIdx.x] = regs.eg;
        if (front.vec_ok) {
            const int q_row = (cols + 3) >> 2;
            const int quads = rows * q_row;
            const int i0 = threadIdx.x, i1 = threadIdx.x + kConefPanelThreads;
            if (i0 < quads)
                conef_panel_park_quad(front, regs.g0, regs.ep0, regs.cb0, i0, q_row, row0, rows, c0, d, w, terms, aux, one_minus_beta);
            if (i1 < quads)
                conef_panel_park_quad(front, regs.g1, regs.ep1, regs.cb1, i1, q_row, row0, rows, c0, d, w, terms, aux, one_minus_beta);
        } else {
            const float* raw = front.raw();
            for (int i = threadIdx.x; i < rows * cols; i += kConefPanelThreads) {
                const int row = i / cols, c = i - row * cols;
                const int64_t f = (row0 + row) * d + c0 + c;
                const uint32_t ep = plan.epos[c0 + c], j = plan.colb[c0 + c];
                const uint32_t p = j | ((ep >> 15) << 31);
                const float cell = aux[row * w + (int)j];
                const float v = front.value(f, raw[f], cell, p);
                terms[(int)(ep & 0x7fffu) * rows + row] = conef_update_term(v, cell, p, one_minus_beta);
            }
        }
        __syncthreads();
        if (c0 + pc < d) conef_panel_request(front, plan, regs, row0, rows, c0 + pc, d);   // travels during the walk
        // One thread per (entry, row); the thread of a group's first entry adds the group's terms onto
        // the cell in order.  Its first four terms are read together: groups are short (a panel holds
        // pc / w columns of a bucket on average), so most of them are one trip to LDS.
        const int pairs = cols * rows;
        for (int idx = threadIdx.x; idx < pairs; idx += kConefPanelThreads) {
            const int e = rows == 1 ? idx : rows == 2 ? idx >> 1 : rows == 4 ? idx >> 2 : idx / rows;
            const int row = idx - e * rows;
            const uint32_t g = entg_l[e];
            const int len = (int)(g >> 16);
            if (len == 0) continue;                              // the group's first entry does the group
            const int cell = row * w + (int)(g & 0xffffu);
            const float* t = terms + e * rows + row;
            const float t0 = t[0], t1 = t[len > 1 ? rows : 0], t2 = t[len > 2 ? 2 * rows : 0], t3 = t[len > 3 ? 3 * rows : 0];
            float sum = __fadd_rn(acc[cell], t0);
            if (len > 1) sum = __fadd_rn(sum, t1);
            if (len > 2) sum = __fadd_rn(sum, t2);
            if (len > 3) sum = __fadd_rn(sum, t3);
            for (int k = 4; k < len; ++k) sum = __fadd_rn(sum, t[k * rows]);
            acc[cell] = sum;
        }
        __syncthreads();
    }
    for (int p = threadIdx.x; p < total; p += kConefPanelThreads) conef_st(cs_out + row0 * w + p, acc[p]);
}

// (two 1024-thread workgroups a CU: 64 registers a thread)
template <typename CsT, typename Front>
__global__ void __launch_bounds__(kConefPanelThreads, 8)
conef_panel_kernel(Front front, ConefPanelView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int d, int w, int rb,
                   double one_minus_beta)
{
    conef_panel_body<CsT, Front>(front, plan, cs_in, cs_out, n, d, w, rb, one_minus_beta, (int)blockIdx.x);
}

template <typename CsT, typename Front>
int conef_launch_panels(Front front, ConefPanelView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int64_t d, int32_t w,
                        float beta, hipStream_t s)
{
    ConefPanelShape shape;
    if (!conef_panel_shape(n, d, w, &shape) || shape.pc != plan.pc) return CONEF_ERR_INVALID;
    auto k = conef_panel_kernel<CsT, Front>;
    hipError_t e = conef_allow_lds((const void*)k, shape.lds);
    if (e != hipSuccess) return (int)e;
    const double omb = 1. - (double)beta;   // (1. - beta) with beta an fp32 value, CountSketch.py:38,63
    hipLaunchKernelGGL(k, dim3((unsigned)shape.tiles), dim3(kConefPanelThreads), shape.lds, s, front, plan, cs_in, cs_out,
                       n, (int)d, (int)w, shape.rb, omb);
    return (int)hipGetLastError();
}
