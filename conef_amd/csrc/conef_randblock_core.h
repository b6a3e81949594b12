// Device bodies of the dense random-block steps, shared by the single-tensor kernels
// (conef_randblock.hip) and the one-launch-per-bucket kernels (conef_randblock_batch.hip).
// A body covers the workgroups [0, gx) of one tensor; `bx` is the workgroup's index among them.
#pragma once
#include "conef_device.h"

// x = g + e;  selected: payload = x, out = x, e' = 0;  not selected: out = 0, e' = x.
// (RandomBlock_hook.py:182-184,222,228,237,240,276-280)
template <bool VEC>
__device__ __forceinline__ void
conef_randblock_ef_body(float* __restrict__ x, float* __restrict__ err, float* __restrict__ payload, int64_t numel,
                        ConefBlock blk, int bx, int gx)
{
    int64_t quads = (numel + 3) / 4;
    int64_t stride = (int64_t)gx * blockDim.x;
    for (int64_t q = bx * (int64_t)blockDim.x + threadIdx.x; q < quads; q += stride) {
        int64_t f = q * 4;
        int valid = numel - f < 4 ? (int)(numel - f) : 4;
        float g[4], e[4], o[4], ne[4];
        if (VEC && valid == 4) {
            float4 tg = *reinterpret_cast<const float4*>(x + f);
            float4 te = *reinterpret_cast<const float4*>(err + f);
            g[0] = tg.x; g[1] = tg.y; g[2] = tg.z; g[3] = tg.w;
            e[0] = te.x; e[1] = te.y; e[2] = te.z; e[3] = te.w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                g[k] = k < valid ? x[f + k] : 0.f;
                e[k] = k < valid ? err[f + k] : 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float xq = __fadd_rn(g[k], e[k]);
            int64_t pos = k < valid ? conef_payload_pos(f + k, blk) : -1;
            if (pos >= 0) {
                payload[pos] = xq;
                o[k] = xq;
                ne[k] = 0.f;
            } else {
                o[k] = 0.f;
                ne[k] = xq;
            }
        }
        if (VEC && valid == 4) {
            *reinterpret_cast<float4*>(x + f) = make_float4(o[0], o[1], o[2], o[3]);
            *reinterpret_cast<float4*>(err + f) = make_float4(ne[0], ne[1], ne[2], ne[3]);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (k < valid) {
                    x[f + k] = o[k];
                    err[f + k] = ne[k];
                }
        }
    }
}

// selected: payload = x / prob, out = payload;  not selected: out = 0
// (UnbiasedRandomBlock_hook.py:155,161-167,200-204)
template <bool VEC>
__device__ __forceinline__ void
conef_randblock_unbiased_body(float* __restrict__ x, float* __restrict__ payload, int64_t numel, ConefBlock blk,
                              float prob, int bx, int gx)
{
    int64_t quads = (numel + 3) / 4;
    int64_t stride = (int64_t)gx * blockDim.x;
    for (int64_t q = bx * (int64_t)blockDim.x + threadIdx.x; q < quads; q += stride) {
        int64_t f = q * 4;
        int valid = numel - f < 4 ? (int)(numel - f) : 4;
        // a quad with no selected element is only written, never read
        bool any = false;
#pragma unroll
        for (int k = 0; k < 4; ++k) any |= (k < valid) && conef_payload_pos(f + k, blk) >= 0;
        float o[4] = {0.f, 0.f, 0.f, 0.f};
        if (any) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                int64_t pos = k < valid ? conef_payload_pos(f + k, blk) : -1;
                if (pos >= 0) {
                    float s = __fdiv_rn(x[f + k], prob);
                    payload[pos] = s;
                    o[k] = s;
                }
            }
        }
        if (VEC && valid == 4) {
            *reinterpret_cast<float4*>(x + f) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (k < valid) x[f + k] = o[k];
        }
    }
}

// workgroups of 256 threads for `work_items` items, capped
inline int conef_grid_for(int64_t work_items, int threads, int64_t cap = 16384)
{
    int64_t g = (work_items + threads - 1) / threads;
    if (g < 1) g = 1;
    if (g > cap) g = cap;
    return (int)g;
}
