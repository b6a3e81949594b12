// Random contiguous-block compressor kernels (gfx950) and their C entry points.
//
// Reference semantics: communication/RandomBlock_hook.py:138-295 (biased block + error feedback,
// dense or count-sketched) and communication/UnbiasedRandomBlock_hook.py:98-219 (block scaled by
// numel/block, no error state).  The block is one wrap-around range [start, start+block) of the flat
// tensor.  At world size 1 the all-reduce of the payload is the identity, so the fused "step"
// entry points leave the decompressed tensor (zeros + block) in place in one pass; the gather /
// scatter pair is what a multi-rank caller puts either side of its all-reduce.
#include "conef_device.h"
#include "conef_randblock_core.h"
#include "conef_sketch_core.h"

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int grid_for(int64_t work_items, int threads, int64_t cap = 16384)
{
    int64_t g = (work_items + threads - 1) / threads;
    if (g < 1) g = 1;
    if (g > cap) g = cap;
    return (int)g;
}

template <bool VEC>
__global__ void __launch_bounds__(256)
randblock_ef_kernel(float* __restrict__ x, float* __restrict__ err, float* __restrict__ payload, int64_t numel,
                    ConefBlock blk)
{
    conef_randblock_ef_body<VEC>(x, err, payload, numel, blk, (int)blockIdx.x, (int)gridDim.x);
}

template <bool VEC>
__global__ void __launch_bounds__(256)
randblock_unbiased_kernel(float* __restrict__ x, float* __restrict__ payload, int64_t numel, ConefBlock blk,
                          float prob)
{
    conef_randblock_unbiased_body<VEC>(x, payload, numel, blk, prob, (int)blockIdx.x, (int)gridDim.x);
}

// payload[p] = x[(start + p) mod numel] / scale   (scale = 1 for the biased compressor)
__global__ void __launch_bounds__(256)
randblock_gather_kernel(const float* __restrict__ x, float* __restrict__ payload, int64_t numel, int64_t start,
                        int64_t block, float scale)
{
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < block; p += stride) {
        int64_t f = start + p;
        if (f >= numel) f -= numel;
        float v = x[f];
        payload[p] = scale == 1.0f ? v : __fdiv_rn(v, scale);
    }
}

// x = 0 everywhere except the block, which receives the payload
template <bool VEC>
__global__ void __launch_bounds__(256)
randblock_scatter_kernel(float* __restrict__ x, const float* __restrict__ payload, int64_t numel, ConefBlock blk)
{
    int64_t quads = (numel + 3) / 4;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t q = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; q < quads; q += stride) {
        int64_t f = q * 4;
        int valid = numel - f < 4 ? (int)(numel - f) : 4;
        float o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            int64_t pos = k < valid ? conef_payload_pos(f + k, blk) : -1;
            o[k] = pos >= 0 ? payload[pos] : 0.f;
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

inline bool block_args_ok(int64_t numel, int64_t start, int64_t block)
{
    return numel >= 1 && start >= 0 && start < numel && block >= 1 && block <= numel;
}

}  // namespace

extern "C" {

int conef_randblock_conef_step_f32(float* x, const float* cs_in, float* cs_out, float* payload, int64_t n, int64_t m,
                                   int32_t w, int64_t start, int64_t block, float alpha, float beta, int32_t a,
                                   int32_t b, void* stream)
{
    if (n < 1 || m < 1 || m > 0x7fffffffLL || w < 1 || w > (1 << 30)) return CONEF_ERR_INVALID;
    if (!block_args_ok(n * m, start, block) || !x || !cs_in || !cs_out || !payload) return CONEF_ERR_INVALID;
    ConefSeeds hs = {a, b, a + 2, b + 3};
    ConefFrontRandBlock front = {x, payload, m, conef_make_block(n * m, start, block), alpha};
    return conef_launch_sketch_step<float>(front, cs_in, cs_out, n, m, w, beta, hs, (hipStream_t)stream,
                                           aligned16(x));
}

int conef_randblock_ef_step_f32(float* x, float* err, float* payload, int64_t numel, int64_t start, int64_t block,
                                void* stream)
{
    if (!block_args_ok(numel, start, block) || !x || !err || !payload) return CONEF_ERR_INVALID;
    ConefBlock blk = conef_make_block(numel, start, block);
    int g = grid_for((numel + 3) / 4, 256);
    if (aligned16(x) && aligned16(err))
        hipLaunchKernelGGL(randblock_ef_kernel<true>, dim3(g), dim3(256), 0, (hipStream_t)stream, x, err, payload,
                           numel, blk);
    else
        hipLaunchKernelGGL(randblock_ef_kernel<false>, dim3(g), dim3(256), 0, (hipStream_t)stream, x, err, payload,
                           numel, blk);
    return (int)hipGetLastError();
}

int conef_randblock_unbiased_step_f32(float* x, float* payload, int64_t numel, int64_t start, int64_t block,
                                      float prob, void* stream)
{
    if (!block_args_ok(numel, start, block) || !x || !payload || !(prob > 0.f)) return CONEF_ERR_INVALID;
    ConefBlock blk = conef_make_block(numel, start, block);
    int g = grid_for((numel + 3) / 4, 256);
    if (aligned16(x))
        hipLaunchKernelGGL(randblock_unbiased_kernel<true>, dim3(g), dim3(256), 0, (hipStream_t)stream, x, payload,
                           numel, blk, prob);
    else
        hipLaunchKernelGGL(randblock_unbiased_kernel<false>, dim3(g), dim3(256), 0, (hipStream_t)stream, x, payload,
                           numel, blk, prob);
    return (int)hipGetLastError();
}

int conef_randblock_gather_f32(const float* x, float* payload, int64_t numel, int64_t start, int64_t block,
                               float scale, void* stream)
{
    if (!block_args_ok(numel, start, block) || !x || !payload || !(scale > 0.f)) return CONEF_ERR_INVALID;
    hipLaunchKernelGGL(randblock_gather_kernel, dim3(grid_for(block, 256)), dim3(256), 0, (hipStream_t)stream, x,
                       payload, numel, start, block, scale);
    return (int)hipGetLastError();
}

int conef_randblock_scatter_f32(float* x, const float* payload, int64_t numel, int64_t start, int64_t block,
                                void* stream)
{
    if (!block_args_ok(numel, start, block) || !x || !payload) return CONEF_ERR_INVALID;
    ConefBlock blk = conef_make_block(numel, start, block);
    int g = grid_for((numel + 3) / 4, 256);
    if (aligned16(x))
        hipLaunchKernelGGL(randblock_scatter_kernel<true>, dim3(g), dim3(256), 0, (hipStream_t)stream, x, payload,
                           numel, blk);
    else
        hipLaunchKernelGGL(randblock_scatter_kernel<false>, dim3(g), dim3(256), 0, (hipStream_t)stream, x, payload,
                           numel, blk);
    return (int)hipGetLastError();
}

}  // extern "C"
