// Device-side building blocks shared by the ConEF kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <utility>

#define CONEF_OK 0
#define CONEF_ERR_INVALID (-1)

// ------------------------------------------------------------- launch helper ----
// A kernel that wants more than 48 KB of dynamic LDS has to be allowed to, per device.  The runtime
// call costs the host a few microseconds, a hook issues a handful of such launches per bucket: the
// largest size granted per (kernel, device) is remembered and the runtime is only asked again for
// a larger one.  (The one piece of bookkeeping the library keeps between calls; guarded by a mutex.)
inline hipError_t conef_allow_lds(const void* kernel, size_t bytes)
{
    if (bytes <= 48 * 1024) return hipSuccess;
    static std::mutex lock;
    static std::map<std::pair<const void*, int>, size_t> granted;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> hold(lock);
    size_t& have = granted[std::make_pair(kernel, dev)];
    if (have >= bytes) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) have = bytes;
    return e;
}

// ------------------------------------------------------------------ hash ----
// Integer mixer of the count sketch (reference: communication/compressors/CountSketch.py:7-18).
// The reference's `h` is a signed int, so all three shifts are arithmetic; the last one always
// clears the sign bit and the `% range` that follows sees a non-negative value.
__host__ __device__ __forceinline__ uint32_t conef_mix32(int32_t value, int32_t a, int32_t b)
{
    uint32_t h = (uint32_t)a * (uint32_t)value + (uint32_t)b;
    h ^= (uint32_t)((int32_t)h >> 16);
    h *= 0x85ebca6bu;
    h ^= (uint32_t)((int32_t)h >> 13);
    h *= 0xc2b2ae35u;
    h ^= (uint32_t)((int32_t)h >> 16);
    return h;
}

// Division by the sketch width, which is uniform over a launch: one fp64 multiply gives the
// quotient to within one, and two compares repair it.  Exact for h < 2^31 and 0 < w <= 2^30.
struct ConefMod {
    uint32_t w;
    double inv;
};

static inline ConefMod conef_make_mod(int32_t w)
{
    ConefMod m;
    m.w = (uint32_t)w;
    m.inv = 1.0 / (double)w;
    return m;
}

__host__ __device__ __forceinline__ uint32_t conef_umod(uint32_t h, ConefMod m)
{
    uint32_t q = (uint32_t)((double)h * m.inv);
    int32_t r = (int32_t)(h - q * m.w);
    if (r < 0) r += (int32_t)m.w;
    else if (r >= (int32_t)m.w) r -= (int32_t)m.w;
    return (uint32_t)r;
}

// Bucket in the low 31 bits, sign bit (1 = +1, 0 = -1) in bit 31.
// Sign = parity of the second hash AFTER the modulo (CountSketch.py:61-62).
__host__ __device__ __forceinline__ uint32_t conef_bucket_sign(int32_t col, ConefMod m, int32_t a, int32_t b,
                                                                int32_t sa, int32_t sb)
{
    uint32_t j = conef_umod(conef_mix32(col, a, b), m);
    uint32_t s = conef_umod(conef_mix32(col, sa, sb), m) & 1u;
    return j | (s << 31);
}

__device__ __forceinline__ float conef_apply_sign(float v, uint32_t packed)
{
    // sign bit set in `packed` means +1: flip the float's sign when it is clear
    return __uint_as_float(__float_as_uint(v) ^ ((~packed) & 0x80000000u));
}

// ------------------------------------------------------- sketch arithmetic ----
// Query term (CountSketch.py:93): (sign * cell) * alpha, two fp32 roundings, no contraction.
__device__ __forceinline__ float conef_query_term(float cell, uint32_t packed, float alpha)
{
    return __fmul_rn(conef_apply_sign(cell, packed), alpha);
}

// Update term (CountSketch.py:63): sign * (value - (1. - beta) * sign * aux), evaluated in double
// and rounded to float once.  With sign = +-1 this equals fl32(fl64(sign*value - fl64(c*aux))),
// c = 1. - beta held in double.
__device__ __forceinline__ float conef_update_term(float value, float aux, uint32_t packed, double one_minus_beta)
{
    double sv = (double)conef_apply_sign(value, packed);
    double decay = __dmul_rn(one_minus_beta, (double)aux);
    return (float)__dsub_rn(sv, decay);
}

__device__ __forceinline__ float conef_median3(float a, float b, float c)
{
    return fmaxf(fminf(a, b), fminf(fmaxf(a, b), c));   // CountSketch.py:20-25
}

// --------------------------------------------------------------- block test ----
// Wrap-around block [start, start+block) of a flat tensor of `numel` elements
// (reference: communication/RandomBlock_hook.py:216-223,236-237).
struct ConefBlock {
    int64_t start, end, rest;   // selected ranges are [start,end) and [0,rest)
};

static inline ConefBlock conef_make_block(int64_t numel, int64_t start, int64_t block)
{
    ConefBlock b;
    b.start = start;
    b.end = start + block < numel ? start + block : numel;
    b.rest = block - (b.end - b.start);
    return b;
}

// position inside the payload, or -1 when the element is not selected
__device__ __forceinline__ int64_t conef_payload_pos(int64_t flat, ConefBlock b)
{
    if (flat >= b.start) return flat < b.end ? flat - b.start : -1;
    return flat < b.rest ? (b.end - b.start) + flat : -1;
}

// ------------------------------------------------------------ wave helpers ----
// Butterfly sum over the 64 lanes; every lane ends with the total.  The four steps inside a row
// of 16 lanes are DPP operands of the adds (vector ALU), only the last two cross rows and go
// through the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float conef_dpp(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

__device__ __forceinline__ float conef_wave_sum(float v)
{
    v += conef_dpp<0xB1>(v);    // quad_perm [1,0,3,2]: lane ^ 1
    v += conef_dpp<0x4E>(v);    // quad_perm [2,3,0,1]: lane ^ 2
    v += conef_dpp<0x141>(v);   // row_half_mirror: the other quad of the 8
    v += conef_dpp<0x140>(v);   // row_mirror: the other half of the 16
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// Sum over the 64 lanes that ends in lane 63 only, all six steps on the vector ALU: four butterfly
// steps inside each row of 16 lanes, then lane 15 of rows 0 and 2 is added into rows 1 and 3
// (row_bcast15) and lane 31 into rows 2 and 3 (row_bcast31).
__device__ __forceinline__ float conef_wave_sum_to_last(float v)
{
    v += conef_dpp<0xB1>(v);
    v += conef_dpp<0x4E>(v);
    v += conef_dpp<0x141>(v);
    v += conef_dpp<0x140>(v);
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xa, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xc, 0xf, false));
    return v;
}
