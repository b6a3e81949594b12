// Gram-Schmidt kernels for the wider ranks (8, 16, 32 with the matrix exactly r wide), where
// kernels that unroll the column steps over register-indexed columns spend most of their time
// fetching instructions.  Both kernels here keep the step loop a real loop (the column index only
// selects lanes or waves), so the code stays a few KB whatever the rank.
//
// Same arithmetic as powerSGD_hook.py:21-43 of the reference: col /= ||col|| (+eps when eps != 0),
// rest -= (col . rest) col, with the sums taken in a fixed order of each kernel's own.
//
// ------------------------------------------ several workgroups, one matrix column per lane ----
// A workgroup of 1024 threads reads its share of the row-major matrix as a flat array: element
// e = tid + 1024 t sits in column tid % r for every t, so a thread holds RPT rows of ONE column in
// registers and every global access is a plain coalesced row of dwords.  Column step i:
//   1. the threads of column i lay their values out in LDS (the pivot column, not yet scaled);
//   2. every thread multiplies the pivot rows into its own column and the products are added over
//      the wave's lanes of equal column (shuffles), over the waves (LDS) and over the workgroups
//      (one 8-byte {sum, step} record per workgroup and column in device memory: the step number
//      travels with the value, so a single relaxed load tells a waiting thread whether the value
//      is there, and nothing has to be cleared between steps);
//   3. later columns lose their projection on column i / (norm + eps); column i itself keeps its
//      raw values and its 1 / (norm + eps), and is scaled when it is stored at the end.
// One exchange across workgroups per step (about 2 us) is what bounds this kernel, so the matrix
// is spread thin: few rows a thread, many workgroups.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

constexpr int kGslThreads = 1024;
constexpr int kGslMaxItems = 24;          // matrices per launch
constexpr int kGslMaxWgs = 128;           // workgroups per launch
constexpr unsigned kGslSpinLimit = 1u << 22;

// Workgroups of the Gram-Schmidt kernels that exchange sums between workgroups inside one launch
// (this file, conef_gs_gram.h, gram_schmidt_grid_kernel) wait for each other with a bounded spin.
// One that runs out its wait leaves NaN in its rows and counts itself here, per GPU, since the
// library was loaded: the host reads the count with conef_gram_schmidt_give_ups.  A diagnostic
// only: nothing in the kernels reads it.
static __device__ unsigned long long g_gs_give_ups;

__device__ __forceinline__ void gs_count_give_up()
{
    __hip_atomic_fetch_add(&g_gs_give_ups, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Workspace of the kernel.  slot[i & 1][g][c]: workgroup g's sum for column c at step i, low word
// the float, high word i + 1.
struct GslWs {
    unsigned gave_up;
    unsigned pad[63];
    unsigned long long slot[2][kGslMaxWgs][32];
};

// Matrix k of a launch: elements[k] floats at a[k], workgroups first[k] .. first[k + 1] - 1.
struct GslBatch {
    float* a[kGslMaxItems];
    int64_t elements[kGslMaxItems];
    int first[kGslMaxItems + 1];
};

__global__ void gsl_reset_kernel(GslWs* ws, int wgs)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) ws->gave_up = 0;
    unsigned long long* s = &ws->slot[0][0][0];
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < 2 * kGslMaxWgs * 32; e += gridDim.x * blockDim.x) {
        const int g = (e >> 5) % kGslMaxWgs;
        if (g < wgs) s[e] = 0ull;
    }
}

// sum over the wave's lanes of equal (lane % RP); every lane of a column ends with the same bits
template <int RP>
__device__ __forceinline__ float gsl_column_sum(float x)
{
#pragma unroll
    for (int off = RP; off < 64; off <<= 1) x += __shfl_xor(x, off, 64);
    return x;
}

// Workgroup b of a matrix owns elements [1024 RPT b, 1024 RPT (b + 1)).  The launch must be
// cooperative (all workgroups resident) and ws reset for its workgroups.  A workgroup that waits
// about a second for another one's record gives up, tells the others, and every workgroup that
// hears of it fills its share of the matrix with NaN before it ends.
template <int RP, int RPT>
__global__ void __launch_bounds__(kGslThreads)
gsl_kernel(GslBatch batch, int count, float eps, GslWs* ws)
{
    constexpr int T = kGslThreads, NW = T / 64, G = T / RP, PS = RPT + 4;
    static_assert(64 % RP == 0 && RPT % 4 == 0, "column-lane layout");
    __shared__ __attribute__((aligned(16))) float piv[2][G * PS];
    __shared__ __attribute__((aligned(16))) float red[RP][NW];
    __shared__ float tot[RP];
    __shared__ float part[RP * kGslMaxWgs];
    __shared__ int failed;

    int it = 0;
    while (it + 1 < count && (int)blockIdx.x >= batch.first[it + 1]) ++it;
    const int wg0 = batch.first[it];
    const int nwg = batch.first[it + 1] - wg0;
    const int64_t base = (int64_t)((int)blockIdx.x - wg0) * T * RPT;
    float* __restrict__ a = batch.a[it] + base;
    const int64_t left = batch.elements[it] - base;
    const int mine = (int)(left < (int64_t)T * RPT ? left : (int64_t)T * RPT);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = tid % RP, g = tid / RP;
    float v[RPT];
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int e = tid + T * t;
        v[t] = e < mine ? a[e] : 0.f;
    }
    if (tid == 0) failed = 0;
    float myinv = 1.f;      // 1 / (norm + eps) of this thread's column, known after step c

#pragma unroll 1
    for (int i = 0; i < RP; ++i) {
        float* pv = piv[i & 1] + g * PS;
        if (c == i) {
#pragma unroll
            for (int t = 0; t < RPT; t += 4) *reinterpret_cast<float4*>(pv + t) = make_float4(v[t], v[t + 1], v[t + 2], v[t + 3]);
        }
        __syncthreads();
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < RPT; t += 4) {
            const float4 p = *reinterpret_cast<const float4*>(pv + t);
            acc[0] = fmaf(p.x, v[t], acc[0]);
            acc[1] = fmaf(p.y, v[t + 1], acc[1]);
            acc[2] = fmaf(p.z, v[t + 2], acc[2]);
            acc[3] = fmaf(p.w, v[t + 3], acc[3]);
        }
        const float mysum = gsl_column_sum<RP>((acc[0] + acc[1]) + (acc[2] + acc[3]));
        if (lane < RP) red[lane][wave] = mysum;      // lane == c for these lanes: 64 and 1024 are multiples of RP
        __syncthreads();
        const unsigned tag = (unsigned)(i + 1);
        if (tid < RP) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w += 4) {
                const float4 x = *reinterpret_cast<const float4*>(&red[tid][w]);
                s += (x.x + x.y) + (x.z + x.w);
            }
            const unsigned long long rec = ((unsigned long long)tag << 32) | (unsigned long long)__float_as_uint(s);
            __hip_atomic_store(&ws->slot[i & 1][blockIdx.x][tid], rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        for (int e = tid; e < nwg * RP; e += T) {
            const int g2 = e / RP, c2 = e - g2 * RP;
            unsigned long long* src = &ws->slot[i & 1][wg0 + g2][c2];
            unsigned long long rec;
            unsigned spins = 0;
            while ((unsigned)((rec = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >> 32) != tag) {
                ++spins;
                if (spins > kGslSpinLimit ||
                    ((spins & 255u) == 0 && __hip_atomic_load(&ws->gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                    __hip_atomic_store(&ws->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    failed = 1;
                    rec = 0;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
            part[c2 * kGslMaxWgs + g2] = __uint_as_float((unsigned)rec);
        }
        __syncthreads();
        if (failed) {
            if (tid == 0) gs_count_give_up();
            // a half-orthogonalised matrix would pass for a result: leave one that cannot
#pragma unroll
            for (int t = 0; t < RPT; ++t) {
                const int e = tid + T * t;
                if (e < mine) a[e] = __builtin_nanf("");
            }
            return;
        }
        if (tid < RP) {
            float s = 0.f;
            for (int g2 = 0; g2 < nwg; ++g2) s += part[tid * kGslMaxWgs + g2];      // same order in every workgroup
            tot[tid] = s;
        }
        __syncthreads();
        const float nrm = sqrtf(tot[i]);
        const float inv = 1.f / (eps == 0.f ? nrm : nrm + eps);      // one division per column, products after
        if (c == i) myinv = inv;
        if (c > i) {
            const float coef = -__fmul_rn(tot[c], inv);
#pragma unroll
            for (int t = 0; t < RPT; t += 4) {
                const float4 p = *reinterpret_cast<const float4*>(pv + t);
                v[t] = fmaf(coef, __fmul_rn(p.x, inv), v[t]);
                v[t + 1] = fmaf(coef, __fmul_rn(p.y, inv), v[t + 1]);
                v[t + 2] = fmaf(coef, __fmul_rn(p.z, inv), v[t + 2]);
                v[t + 3] = fmaf(coef, __fmul_rn(p.w, inv), v[t + 3]);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int e = tid + T * t;
        if (e < mine) a[e] = __fmul_rn(v[t], myinv);
    }
}

// ------------------------------------------------------- one workgroup, a wave owns columns ----
// For a matrix that fits one workgroup's registers the cheaper arrangement gives every wave CW
// whole columns: lane l of the wave holds rows l, l + 64, ... of each of them.  Then every sum of
// a column step stays inside a wave (DPP adds, the total read from lane 63: no LDS, no second
// barrier), and the step follows the reference's order of operations exactly
//     col /= ||col|| + eps;  rest -= (col . rest) col        (powerSGD_hook.py:21-43)
// with the owner of column i normalising it and publishing it in LDS, one barrier, and everyone
// else taking dot product and update from the published column: two multiply-adds per element and
// step.  Waves whose columns are all finished skip the work of a step and only meet the barrier,
// so the arithmetic shrinks with the columns left.  The row-major matrix goes through an LDS tile
// (row stride r + 1) on the way in and out, so global accesses stay coalesced rows.
constexpr int kGswBatchMax = 48;
constexpr int kGswTileRows = 1024;

struct GswBatch {
    float* a[kGswBatchMax];
    int rows[kGswBatchMax];
};

// Sum over the 64 lanes, returned to all of them (the total ends in lane 63 and is read from there).
__device__ __forceinline__ float gsw_wave_total(float v)
{
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false));      // lane ^ 1
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false));      // lane ^ 2
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false));     // other quad of 8
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, false));     // other half of 16
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xa, 0xf, false));     // lanes 15, 47 into rows 1, 3
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xc, 0xf, false));     // lane 31 into rows 2, 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// LDS floats the kernel needs
template <int RP, int RPT>
constexpr int gsw_lds_floats()
{
    constexpr int CAP = 64 * RPT, TR = CAP < kGswTileRows ? CAP : kGswTileRows;
    return 2 * 64 * (RPT + 4) + TR * (RP + 1);
}

// col /= ||col|| + eps over the wave (a lane holds RPT elements), the result also written to pb
template <int RPT>
__device__ __forceinline__ void gsw_publish_column(float (&col)[RPT], float* pb, float eps)
{
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < RPT; t += 4) {
        acc[0] = fmaf(col[t], col[t], acc[0]);
        acc[1] = fmaf(col[t + 1], col[t + 1], acc[1]);
        acc[2] = fmaf(col[t + 2], col[t + 2], acc[2]);
        acc[3] = fmaf(col[t + 3], col[t + 3], acc[3]);
    }
    const float nrm = sqrtf(gsw_wave_total((acc[0] + acc[1]) + (acc[2] + acc[3])));
    const float inv = 1.f / (eps == 0.f ? nrm : nrm + eps);
#pragma unroll
    for (int t = 0; t < RPT; t += 4) {
        col[t] = __fmul_rn(col[t], inv);
        col[t + 1] = __fmul_rn(col[t + 1], inv);
        col[t + 2] = __fmul_rn(col[t + 2], inv);
        col[t + 3] = __fmul_rn(col[t + 3], inv);
        *reinterpret_cast<float4*>(pb + t) = make_float4(col[t], col[t + 1], col[t + 2], col[t + 3]);
    }
}

// The workgroup's rows of a row-major [rows, RP] matrix into registers and back: v[cc][t] is row
// lane + 64 t of column col0 + cc.  Coalesced dwords to an LDS tile (row stride RP + 1), columns
// out of the tile; rows past the end read as zero.  All threads of the workgroup call these.
template <int RP, int RPT, int CW>
__device__ __forceinline__ void gsw_load_columns(const float* __restrict__ a, int rows, float* tile, float (&v)[CW][RPT],
                                                 int tid, int lane, int col0)
{
    constexpr int T = 64 * RP / CW, LD = RP + 1;
    constexpr int CAP = 64 * RPT, TR = CAP < kGswTileRows ? CAP : kGswTileRows, NCH = CAP / TR, SPC = TR / 64;
    constexpr int JN = TR * RP / T, JU = JN % 16 == 0 ? 16 : JN % 8 == 0 ? 8 : 4;      // tile elements per thread, loads in flight
    static_assert(RPT % 4 == 0 && CAP % TR == 0 && RP % CW == 0 && JN % JU == 0, "wave-owns-columns layout");
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int r0 = k * TR;
        if (r0 < rows) {
            const int n = (rows - r0 < TR ? rows - r0 : TR) * RP;
            const float* src = a + (int64_t)r0 * RP;
#pragma unroll
            for (int j0 = 0; j0 < JN; j0 += JU) {
                float x[JU];
#pragma unroll
                for (int u = 0; u < JU; ++u) {
                    const int e = tid + T * (j0 + u);
                    x[u] = e < n ? src[e] : 0.f;
                }
#pragma unroll
                for (int u = 0; u < JU; ++u) {
                    const int e = tid + T * (j0 + u);
                    const int row = e / RP, c = e - row * RP;
                    tile[row * LD + c] = x[u];
                }
            }
            __syncthreads();
#pragma unroll
            for (int t = 0; t < SPC; ++t) {
#pragma unroll
                for (int cc = 0; cc < CW; ++cc) v[cc][k * SPC + t] = tile[(lane + 64 * t) * LD + col0 + cc];
            }
            __syncthreads();
        } else {
#pragma unroll
            for (int t = 0; t < SPC; ++t) {
#pragma unroll
                for (int cc = 0; cc < CW; ++cc) v[cc][k * SPC + t] = 0.f;
            }
        }
    }
}

template <int RP, int RPT, int CW>
__device__ __forceinline__ void gsw_store_columns(float* __restrict__ a, int rows, float* tile, const float (&v)[CW][RPT],
                                                  int tid, int lane, int col0)
{
    constexpr int T = 64 * RP / CW, LD = RP + 1;
    constexpr int CAP = 64 * RPT, TR = CAP < kGswTileRows ? CAP : kGswTileRows, NCH = CAP / TR, SPC = TR / 64;
    constexpr int JN = TR * RP / T;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int r0 = k * TR;
        if (r0 < rows) {
            if (k > 0) __syncthreads();
#pragma unroll
            for (int t = 0; t < SPC; ++t) {
#pragma unroll
                for (int cc = 0; cc < CW; ++cc) tile[(lane + 64 * t) * LD + col0 + cc] = v[cc][k * SPC + t];
            }
            __syncthreads();
            const int n = (rows - r0 < TR ? rows - r0 : TR) * RP;
            float* dst = a + (int64_t)r0 * RP;
#pragma unroll 8
            for (int j = 0; j < JN; ++j) {
                const int e = tid + T * j;
                const int row = e / RP, c = e - row * RP;
                if (e < n) dst[e] = tile[row * LD + c];
            }
        }
    }
}

// Matrix batch.a[blockIdx.x]: [rows, RP] row-major, rows <= 64 RPT, in place.
template <int RP, int RPT, int CW>
__global__ void __launch_bounds__(64 * RP / CW)
gsw_kernel(GswBatch batch, float eps)
{
    constexpr int PS = RPT + 4;      // a lane's slice of the pivot column: 16-byte accesses of 16 lanes then cover all banks once
    extern __shared__ __attribute__((aligned(16))) float gsw_lds[];
    float* piv = gsw_lds;                       // [2][64][PS]: the normalised pivot column, lane-major
    float* tile = gsw_lds + 2 * 64 * PS;        // [TR][RP + 1]
    float* __restrict__ a = batch.a[blockIdx.x];
    const int rows = batch.rows[blockIdx.x];
    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col0 = w * CW;

    float v[CW][RPT];
    gsw_load_columns<RP, RPT, CW>(a, rows, tile, v, tid, lane, col0);

    // Normalises this wave's column i and publishes it: a lane's slice of the column is RPT words,
    // written and read 16 bytes at a time.
    auto publish = [&](int i) __attribute__((always_inline)) {
        float* pb = piv + (i & 1) * (64 * PS) + lane * PS;
        if constexpr (CW == 1) {
            gsw_publish_column<RPT>(v[0], pb, eps);
        } else {
            static_assert(CW == 2, "columns per wave");
            if (i % 2 == 0) gsw_publish_column<RPT>(v[0], pb, eps);
            else gsw_publish_column<RPT>(v[1], pb, eps);
        }
    };

    if (w == 0) publish(0);
    __syncthreads();
    // Step i: everyone with a column right of i takes its projection on column i off; the owner of
    // column i + 1 then normalises and publishes it before the barrier that ends the step.  That
    // wave is the critical path of the step (the others only have to reach the barrier), so it
    // runs at raised priority.
#pragma unroll 1
    for (int i = 0; i < RP; ++i) {
        const bool next_owner = i + 1 < RP && w == (i + 1) / CW;
        if (next_owner) __builtin_amdgcn_s_setprio(3);
        if (col0 + CW - 1 > i) {      // some column of this wave is still to the right of i
            const float* pb = piv + (i & 1) * (64 * PS) + lane * PS;
            float q[RPT];
#pragma unroll
            for (int t = 0; t < RPT; t += 4) {
                const float4 x = *reinterpret_cast<const float4*>(pb + t);
                q[t] = x.x;
                q[t + 1] = x.y;
                q[t + 2] = x.z;
                q[t + 3] = x.w;
            }
            float dot[CW];
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) {
                float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < RPT; t += 4) {
                    acc[0] = fmaf(q[t], v[cc][t], acc[0]);
                    acc[1] = fmaf(q[t + 1], v[cc][t + 1], acc[1]);
                    acc[2] = fmaf(q[t + 2], v[cc][t + 2], acc[2]);
                    acc[3] = fmaf(q[t + 3], v[cc][t + 3], acc[3]);
                }
                dot[cc] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
            }
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) dot[cc] = gsw_wave_total(dot[cc]);
#pragma unroll
            for (int cc = 0; cc < CW; ++cc) {
                if (col0 + cc > i) {
                    const float coef = -dot[cc];
#pragma unroll
                    for (int t = 0; t < RPT; ++t) v[cc][t] = fmaf(coef, q[t], v[cc][t]);
                }
            }
        }
        if (next_owner) {
            publish(i + 1);
            __builtin_amdgcn_s_setprio(0);
        }
        __syncthreads();
    }
    gsw_store_columns<RP, RPT, CW>(a, rows, tile, v, tid, lane, col0);
}
