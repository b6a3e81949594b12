// Row lists in column panels: the count-sketch update without atomics for rows that are too long
// for conef_rowlist.h (a row's values, its bucket lists and its cells together exceed LDS), on
// matrices with rows enough to fill the machine - e.g. a [4096, 25088] fully connected layer.
//
// A workgroup takes a tile of `rb` rows and keeps that tile's sketch cells in LDS for the whole
// kernel: the old values (every term's decay reads the cell as it was before the call,
// CountSketch.py:47-52,63) and the running sums.  The columns go by in panels of `pc`:
//
//   stage   the panel's values are produced in column order with 16-byte accesses and parked in
//           LDS, with whatever the fused step has to do in column order (the `front`);
//   walk    the plan lists the panel's columns grouped by bucket, ascending inside a bucket
//           (`ent`: column inside the panel | sign << 15; `entb`: the bucket).  The thread that
//           meets the first entry of a bucket's group adds the group's terms onto the cell, in
//           that order; the other threads of the group have nothing to do.
//
// Panels are taken in ascending order, so a cell receives its terms in ascending column order:
// the CPU oracle's order, bit for bit, no atomics, one read of the tensor.  cs_out may be cs_in.
#pragma once
#include "conef_device.h"
#include "conef_sketch_core.h"

constexpr int kConefPanelThreads = 256;
constexpr size_t kConefPanelLdsLimit = 156 * 1024;

struct ConefPanelView {
    const uint16_t* ent;    // [d] by panel: column inside the panel | sign bit << 15, grouped by bucket, columns ascending
    const uint16_t* entb;   // [d] the bucket of the same entry
    const uint32_t* pk;     // [d] bucket | sign bit << 31 of every column, in column order
    int pc;                 // columns per panel (a multiple of 8)
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
    return (size_t)rb * pc * 4 + (size_t)pc * 4 + 2 * conef_panel_cells(rb, w) * 4;
}

// Tile height and panel width are functions of (d, w) alone, so that one plan serves every matrix of
// that row length and sketch width.  Two workgroups a CU where the cells leave room for it (their
// phases - stage, walk - overlap only between workgroups), one otherwise.
inline bool conef_panel_shape(int64_t n, int64_t d, int32_t w, ConefPanelShape* s)
{
    if (d < 1 || d > 0x7fffffffLL || n < 1 || w < 1 || w > 0xffff) return false;
    static const size_t limits[2] = {78 * 1024, kConefPanelLdsLimit};
    for (size_t limit : limits) {
        for (int rb = 4; rb >= 1; rb >>= 1) {
            for (int elems = 8192; elems >= 2048; elems >>= 1) {
                int pc = elems / rb;
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
// A front fills vals[row * pc + c] for the tile's rows and the panel's columns [c0, c0 + cols).
// `aux` holds the tile's old sketch rows, [rows][w].

// DenseCS.update: the value is the dense tensor itself.
struct ConefPanelVec {
    const float* vec;
    bool vec_ok;           // base 16-byte aligned and d % 4 == 0
    __device__ __forceinline__ void stage(int64_t row0, int rows, int c0, int cols, int d, int, float* vals, int pc,
                                          const float*, const uint32_t*) const
    {
        if (vec_ok) {
            const int q_row = (cols + 3) >> 2;       // d % 4 == 0 and pc % 4 == 0: a panel is whole quads
            const int total = rows * q_row;
            for (int i0 = threadIdx.x; i0 < total; i0 += 4 * kConefPanelThreads) {
                float4 t[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    int i = i0 + u * kConefPanelThreads;
                    i = i < total ? i : total - 1;
                    const int row = i / q_row, q = i - row * q_row;
                    t[u] = *reinterpret_cast<const float4*>(vec + (row0 + row) * d + c0 + 4 * q);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int i = i0 + u * kConefPanelThreads;
                    if (i < total) {
                        const int row = i / q_row, q = i - row * q_row;
                        *reinterpret_cast<float4*>(vals + row * pc + 4 * q) = t[u];
                    }
                }
            }
        } else {
            const int total = rows * cols;
            for (int i = threadIdx.x; i < total; i += kConefPanelThreads) {
                const int row = i / cols, c = i - row * cols;
                vals[row * pc + c] = vec[(row0 + row) * d + c0 + c];
            }
        }
    }
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
    __device__ __forceinline__ void stage(int64_t row0, int rows, int c0, int cols, int d, int w, float* vals, int pc,
                                          const float* aux, const uint32_t* pk) const
    {
        if (vec_ok) {
            const int q_row = (cols + 3) >> 2;
            const int total = rows * q_row;
            for (int i0 = threadIdx.x; i0 < total; i0 += 2 * kConefPanelThreads) {
                float4 t[2];
                uint4 pp[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    int i = i0 + u * kConefPanelThreads;
                    i = i < total ? i : total - 1;
                    const int row = i / q_row, q = i - row * q_row;
                    t[u] = *reinterpret_cast<const float4*>(x + (row0 + row) * d + c0 + 4 * q);
                    pp[u] = *reinterpret_cast<const uint4*>(pk + c0 + 4 * q);
                }
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int i = i0 + u * kConefPanelThreads;
                    if (i < total) {
                        const int row = i / q_row, q = i - row * q_row;
                        const int64_t f = (row0 + row) * d + c0 + 4 * q;
                        const float* cells = aux + row * w;
                        const float g[4] = {t[u].x, t[u].y, t[u].z, t[u].w};
                        const uint32_t p[4] = {pp[u].x, pp[u].y, pp[u].z, pp[u].w};
                        float o[4], v[4];
#pragma unroll
                        for (int k = 0; k < 4; ++k) v[k] = one(f + k, g[k], cells[p[k] & 0x7fffffffu], p[k], &o[k]);
                        *reinterpret_cast<float4*>(x + f) = make_float4(o[0], o[1], o[2], o[3]);
                        *reinterpret_cast<float4*>(vals + row * pc + 4 * q) = make_float4(v[0], v[1], v[2], v[3]);
                    }
                }
            }
        } else {
            const int total = rows * cols;
            for (int i = threadIdx.x; i < total; i += kConefPanelThreads) {
                const int row = i / cols, c = i - row * cols;
                const int64_t f = (row0 + row) * d + c0 + c;
                const uint32_t p = pk[c0 + c];
                float o;
                vals[row * pc + c] = one(f, x[f], aux[row * w + (p & 0x7fffffffu)], p, &o);
                x[f] = o;
            }
        }
    }
};

// ------------------------------------------------------------------ kernel ----
template <typename CsT, typename Front>
__device__ __forceinline__ void
conef_panel_body(const Front& front, ConefPanelView plan, const CsT* cs_in, CsT* cs_out, int64_t n, int d, int w, int rb,
                 double one_minus_beta, int bx)
{
    extern __shared__ float conef_pl[];
    const int pc = plan.pc;
    float* vals = conef_pl;
    uint16_t* ent_l = reinterpret_cast<uint16_t*>(vals + rb * pc);
    uint16_t* entb_l = ent_l + pc;
    float* aux = reinterpret_cast<float*>(entb_l + pc);
    float* acc = aux + conef_panel_cells(rb, w);
    const int64_t row0 = (int64_t)bx * rb;
    const int rows = n - row0 < rb ? (int)(n - row0) : rb;
    const int total = rows * w;
    for (int p = threadIdx.x; p < total; p += kConefPanelThreads) {
        const float c = conef_ld(cs_in + row0 * w + p);
        aux[p] = c;
        acc[p] = c;
    }
    __syncthreads();
    for (int c0 = 0; c0 < d; c0 += pc) {
        const int cols = d - c0 < pc ? d - c0 : pc;
        // the panel's lists: two entries a word (c0 is a multiple of 8; the tables are padded to whole words)
        {
            const uint32_t* es = reinterpret_cast<const uint32_t*>(plan.ent + c0);
            const uint32_t* bs = reinterpret_cast<const uint32_t*>(plan.entb + c0);
            uint32_t* ed = reinterpret_cast<uint32_t*>(ent_l);
            uint32_t* bd = reinterpret_cast<uint32_t*>(entb_l);
            const int words = (cols + 1) >> 1;
            for (int i0 = threadIdx.x; i0 < words; i0 += 4 * kConefPanelThreads) {
                uint32_t te[4], tb[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    int i = i0 + u * kConefPanelThreads;
                    i = i < words ? i : words - 1;
                    te[u] = es[i];
                    tb[u] = bs[i];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int i = i0 + u * kConefPanelThreads;
                    if (i < words) {
                        ed[i] = te[u];
                        bd[i] = tb[u];
                    }
                }
            }
        }
        front.stage(row0, rows, c0, cols, d, w, vals, pc, aux, plan.pk);
        __syncthreads();
        const int pairs = cols * rows;
        for (int idx = threadIdx.x; idx < pairs; idx += kConefPanelThreads) {
            const int e = rows == 1 ? idx : idx / rows;
            const int row = idx - e * rows;
            const uint32_t j = entb_l[e];
            if (e > 0 && entb_l[e - 1] == j) continue;          // the group's first entry does the group
            const int cell = row * w + (int)j;
            const double decay = __dmul_rn(one_minus_beta, (double)aux[cell]);
            const float* vr = vals + row * pc;
            float a = acc[cell];
            int ee = e;
            do {
                const uint32_t en = ent_l[ee];
                const uint32_t flip = ((~en) & 0x8000u) << 16;   // sign bit clear (-1): flip the float's sign
                const double sv = (double)__uint_as_float(__float_as_uint(vr[en & 0x7fffu]) ^ flip);
                a = __fadd_rn(a, (float)__dsub_rn(sv, decay));
                ++ee;
            } while (ee < cols && entb_l[ee] == j);
            acc[cell] = a;
        }
        __syncthreads();
    }
    for (int p = threadIdx.x; p < total; p += kConefPanelThreads) conef_st(cs_out + row0 * w + p, acc[p]);
}

template <typename CsT, typename Front>
__global__ void __launch_bounds__(kConefPanelThreads)
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
    if (shape.lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shape.lds);
        if (e != hipSuccess) return (int)e;
    }
    const double omb = 1. - (double)beta;   // (1. - beta) with beta an fp32 value, CountSketch.py:38,63
    hipLaunchKernelGGL(k, dim3((unsigned)shape.tiles), dim3(kConefPanelThreads), shape.lds, s, front, plan, cs_in, cs_out,
                       n, (int)d, (int)w, shape.rb, omb);
    return (int)hipGetLastError();
}
