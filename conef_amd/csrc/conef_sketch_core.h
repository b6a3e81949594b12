// The sketch-accumulation back end shared by every kernel that ends in a count-sketch update:
// the plain DenseCS.update, the fused RandomBlock + ConEF step and the fused PowerSGD
// decompress + residual step differ only in where the value to be sketched comes from (the
// "front"), so the two launch shapes are templates over a front functor.
//
// A front provides
//   float one(r, i, aux, packed)                         - value of element (r,i) for the sketch,
//                                                          with whatever side effects the fusion needs
//   template<bool VEC> void four(r, c0, valid, aux[4], packed[4], v[4])
//                                                        - same for 4 consecutive columns
// where aux is the snapshot cell cs_in[r, bucket(i)] the element maps to.
#pragma once
#include "conef_device.h"

struct ConefSeeds {
    int32_t a, b;     // bucket hash
    int32_t sa, sb;   // sign hash
};

// (a,b) and sign seeds of the three-hash variant (CountSketchHash3.py:40-41,68,77,85,137).
// The reference uses b2+4 for the third sign in update and b2+7 in query; kept as is.
__host__ __device__ __forceinline__ ConefSeeds conef_hash3_seeds(int k, bool for_query)
{
    const int32_t A[3] = {994443, 4113759, 9171025};
    const int32_t B[3] = {609478, 2949676, 2171464};
    const int32_t DA[3] = {2, 4, 8};
    const int32_t DBU[3] = {3, 5, 4};
    const int32_t DBQ[3] = {3, 5, 7};
    ConefSeeds s = {A[k], B[k], A[k] + DA[k], B[k] + (for_query ? DBQ[k] : DBU[k])};
    return s;
}

__device__ __forceinline__ float conef_ld(const float* p) { return *p; }
__device__ __forceinline__ float conef_ld(const __half* p) { return __half2float(*p); }
__device__ __forceinline__ void conef_st(float* p, float v) { *p = v; }
__device__ __forceinline__ void conef_st(__half* p, float v) { *p = __float2half_rn(v); }

// Orders one wavefront's LDS traffic: LDS serves a wave's requests in issue order, so all that is
// needed is that the compiler neither reorders nor caches across this point.
__device__ __forceinline__ void conef_wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int kConefRowThreads = 256;
constexpr int kConefRowWaves = kConefRowThreads / 64;
constexpr size_t kConefRowLdsBudget = 64 * 1024;

// LDS the row shape needs: packed (bucket,sign) per column + per wave a snapshot and an accumulator row
__host__ __device__ inline size_t conef_row_shape_lds(int64_t d, int32_t w)
{
    return (size_t)d * 4 + (size_t)kConefRowWaves * 2 * (size_t)w * 4;
}

inline bool conef_row_shape_fits(int64_t d, int32_t w, size_t /*cell_bytes*/)
{
    return d <= (1 << 20) && conef_row_shape_lds(d, w) <= kConefRowLdsBudget;
}

// ------------------------------------------------------------------ fronts ----
// DenseCS.update: the value is read from a dense [n,d] tensor.
struct ConefFrontVec {
    const float* vec;
    int64_t d;
    __device__ __forceinline__ float one(int64_t r, int64_t i, float, uint32_t) const { return vec[r * d + i]; }
    template <bool VEC>
    __device__ __forceinline__ void four(int64_t r, int64_t c0, int valid, const float*, const uint32_t*, float* v) const
    {
        const float* p = vec + r * d + c0;
        if (VEC) {
            float4 t = *reinterpret_cast<const float4*>(p);
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = k < valid ? p[k] : 0.f;
        }
    }
};

// RandomBlock + ConEF (reference: communication/RandomBlock_hook.py:190,216-243,272-280 at world
// size 1).  x holds the gradient on entry.  xq = x + unsketch*alpha is the error-corrected
// gradient; elements inside the wrap-around block go to the payload and stay in x, the rest are
// zeroed in x and become the residual that is sketched.
struct ConefFrontRandBlock {
    float* x;
    float* payload;
    int64_t d;
    ConefBlock blk;
    float alpha;
    __device__ __forceinline__ float one(int64_t r, int64_t i, float aux, uint32_t pk) const
    {
        int64_t f = r * d + i;
        float xq = __fadd_rn(x[f], conef_query_term(aux, pk, alpha));
        int64_t pos = conef_payload_pos(f, blk);
        if (pos >= 0) {
            payload[pos] = xq;
            x[f] = xq;
            return 0.f;
        }
        x[f] = 0.f;
        return xq;
    }
    template <bool VEC>
    __device__ __forceinline__ void four(int64_t r, int64_t c0, int valid, const float* aux, const uint32_t* pk,
                                         float* v) const
    {
        int64_t f = r * d + c0;
        float* p = x + f;
        float g[4];
        if (VEC) {
            float4 t = *reinterpret_cast<const float4*>(p);
            g[0] = t.x; g[1] = t.y; g[2] = t.z; g[3] = t.w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) g[k] = k < valid ? p[k] : 0.f;
        }
        float o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float xq = __fadd_rn(g[k], conef_query_term(aux[k], pk[k], alpha));
            int64_t pos = k < valid ? conef_payload_pos(f + k, blk) : -1;
            if (pos >= 0) {
                payload[pos] = xq;
                o[k] = xq;
                v[k] = 0.f;
            } else {
                o[k] = 0.f;
                v[k] = xq;
            }
        }
        if (VEC) {
            *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (k < valid) p[k] = o[k];
        }
    }
};

// ------------------------------------------------------------- row shape ----
template <typename CsT, typename Front>
__global__ void __launch_bounds__(kConefRowThreads)
conef_sketch_row_kernel(Front front, const CsT* cs_in, CsT* cs_out, int64_t n, int64_t d, ConefMod mod,
                        double one_minus_beta, ConefSeeds hs)
{
    extern __shared__ uint32_t conef_lds[];
    uint32_t* table = conef_lds;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t w = mod.w;
    float* aux = reinterpret_cast<float*>(conef_lds + d) + (size_t)wave * 2 * w;
    float* acc = aux + w;

    for (int64_t i = threadIdx.x; i < d; i += kConefRowThreads)
        table[i] = conef_bucket_sign((int32_t)i, mod, hs.a, hs.b, hs.sa, hs.sb);
    __syncthreads();

    for (int64_t r = (int64_t)blockIdx.x * kConefRowWaves + wave; r < n; r += (int64_t)gridDim.x * kConefRowWaves) {
        const CsT* in_row = cs_in + r * (int64_t)w;
        for (uint32_t j = lane; j < w; j += 64) {
            float c = conef_ld(in_row + j);
            aux[j] = c;
            acc[j] = c;
        }
        conef_wave_sync();
        for (int64_t i = lane; i < d; i += 64) {
            uint32_t pk = table[i];
            uint32_t j = pk & 0x7fffffffu;
            float a = aux[j];
            float v = front.one(r, i, a, pk);
            atomicAdd(&acc[j], conef_update_term(v, a, pk, one_minus_beta));
        }
        conef_wave_sync();
        CsT* out_row = cs_out + r * (int64_t)w;
        for (uint32_t j = lane; j < w; j += 64) conef_st(out_row + j, acc[j]);
        conef_wave_sync();
    }
}

// ------------------------------------------------------------ tile shape ----
template <typename Front, bool VEC>
__global__ void __launch_bounds__(256)
conef_sketch_tile_kernel(Front front, const float* __restrict__ cs_in, float* cs_out, int64_t n, int64_t d,
                         ConefMod mod, double one_minus_beta, ConefSeeds hs, int rows_per_block)
{
    int64_t c0 = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * 4;
    if (c0 >= d) return;
    int valid = d - c0 < 4 ? (int)(d - c0) : 4;
    uint32_t pk[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
        pk[k] = k < valid ? conef_bucket_sign((int32_t)(c0 + k), mod, hs.a, hs.b, hs.sa, hs.sb) : 0u;
    int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    for (int64_t r = r0; r < r1; ++r) {
        int64_t base = r * (int64_t)mod.w;
        float aux[4], v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) aux[k] = cs_in[base + (pk[k] & 0x7fffffffu)];
        front.template four<VEC>(r, c0, valid, aux, pk, v);
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (k < valid)
                unsafeAtomicAdd(cs_out + base + (pk[k] & 0x7fffffffu),
                                conef_update_term(v[k], aux[k], pk[k], one_minus_beta));
    }
}

static __global__ void conef_copy_f32_kernel(float* __restrict__ dst, const float* __restrict__ src, int64_t count)
{
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) dst[i] = src[i];
}

// ---------------------------------------------------------------- launcher ----
// cs_out may alias cs_in only when the row shape is used (conef_row_shape_fits).
// `vec_ok` tells whether 4-wide accesses of the front's dense tensor are aligned.
template <typename CsT, typename Front>
int conef_launch_sketch_step(Front front, const CsT* cs_in, CsT* cs_out, int64_t n, int64_t d, int32_t w, float beta,
                             ConefSeeds hs, hipStream_t stream, bool vec_ok = false)
{
    const double omb = 1. - (double)beta;   // (1. - beta) with beta an fp32 value, CountSketch.py:38,63
    ConefMod mod = conef_make_mod(w);
    if (conef_row_shape_fits(d, w, sizeof(CsT))) {
        int64_t blocks = (n + kConefRowWaves - 1) / kConefRowWaves;
        if (blocks > 4096) blocks = 4096;
        size_t lds = conef_row_shape_lds(d, w);
        hipLaunchKernelGGL((conef_sketch_row_kernel<CsT, Front>), dim3((unsigned)blocks), dim3(kConefRowThreads), lds,
                           stream, front, cs_in, cs_out, n, d, mod, omb, hs);
        return (int)hipGetLastError();
    }
    if (sizeof(CsT) != sizeof(float)) return CONEF_ERR_INVALID;
    if ((const void*)cs_in == (const void*)cs_out) return CONEF_ERR_INVALID;
    const float* in = reinterpret_cast<const float*>(cs_in);
    float* out = reinterpret_cast<float*>(cs_out);
    int64_t cells = n * (int64_t)w;
    int64_t cg = (cells + 1023) / 1024;
    if (cg > 2048) cg = 2048;
    hipLaunchKernelGGL(conef_copy_f32_kernel, dim3((unsigned)cg), dim3(256), 0, stream, out, in, cells);
    if (d == 0) return (int)hipGetLastError();
    int64_t col_blocks = (d + 1023) / 1024;
    int64_t rpb = (n * col_blocks + 4095) / 4096;
    if (rpb < 8) rpb = 8;
    if (rpb > n) rpb = n;
    while ((n + rpb - 1) / rpb > 65535) rpb *= 2;
    dim3 grid((unsigned)col_blocks, (unsigned)((n + rpb - 1) / rpb));
    if (vec_ok && d % 4 == 0)
        hipLaunchKernelGGL((conef_sketch_tile_kernel<Front, true>), grid, dim3(256), 0, stream, front, in, out, n, d,
                           mod, omb, hs, (int)rpb);
    else
        hipLaunchKernelGGL((conef_sketch_tile_kernel<Front, false>), grid, dim3(256), 0, stream, front, in, out, n,
                           d, mod, omb, hs, (int)rpb);
    return (int)hipGetLastError();
}
