// Magnitude top-k sparsifier (gfx950) for the dense error kept by the hPowerSGD hook.
//
// Reference semantics: communication/hPowerSGD_hook.py:90-97 - keep the k entries of largest
// magnitude, zero everything else, in place.  The reference asks torch.topk for unsorted
// positions and so leaves ties open; here ties on the threshold magnitude keep the lowest flat
// indices, which makes the result a function of the input alone.
//
// Selection is a most-significant-digit radix select on the magnitude bits (a non-negative
// float orders like its bit pattern): four 8-bit histogram passes narrow the k-th largest key,
// then one counting pass and one filtering pass resolve ties in index order.  Nothing returns to
// the host between passes; the running (prefix, remaining) pair lives in the workspace.
#include "conef_device.h"

namespace {

constexpr int kBins = 256;
constexpr int kFilterChunk = 1024;   // elements per workgroup iteration in the ordered passes

struct TopkState {
    uint32_t prefix;      // selected high digits so far
    uint32_t remaining;   // how many keys to take among those matching the prefix
    uint32_t hist[4][kBins];
};

__device__ __forceinline__ uint32_t mag_key(float v) { return __float_as_uint(v) & 0x7fffffffu; }

__global__ void topk_init_kernel(TopkState* st, uint32_t k)
{
    for (int i = threadIdx.x; i < 4 * kBins; i += blockDim.x) (&st->hist[0][0])[i] = 0u;
    if (threadIdx.x == 0) {
        st->prefix = 0u;
        st->remaining = k;
    }
}

__global__ void __launch_bounds__(256)
topk_hist_kernel(const float* __restrict__ x, int64_t numel, TopkState* st, int pass)
{
    __shared__ uint32_t bins[kBins];
    bins[threadIdx.x] = 0u;
    __syncthreads();
    const int shift = 24 - 8 * pass;
    const uint32_t prefix = st->prefix;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < numel; i += stride) {
        uint32_t key = mag_key(x[i]);
        bool match = pass == 0 || (key >> (shift + 8)) == prefix;
        if (match) atomicAdd(&bins[(key >> shift) & 0xffu], 1u);
    }
    __syncthreads();
    uint32_t c = bins[threadIdx.x];
    if (c) atomicAdd(&st->hist[pass][threadIdx.x], c);
}

// one workgroup: pick the digit that holds the k-th largest key among those matching the prefix
__global__ void __launch_bounds__(256)
topk_select_kernel(TopkState* st, int pass)
{
    __shared__ uint32_t cnt[kBins];
    cnt[threadIdx.x] = st->hist[pass][threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t remaining = st->remaining;
        uint32_t above = 0;
        int d = kBins - 1;
        for (; d > 0; --d) {
            if (above + cnt[d] >= remaining) break;
            above += cnt[d];
        }
        st->prefix = (st->prefix << 8) | (uint32_t)d;
        st->remaining = remaining - above;
    }
}

// per-chunk count of keys equal to the threshold
__global__ void __launch_bounds__(256)
topk_count_ties_kernel(const float* __restrict__ x, int64_t numel, const TopkState* st, uint32_t* chunk_ties,
                       int64_t chunks)
{
    __shared__ uint32_t total;
    const uint32_t thr = st->prefix;
    for (int64_t c = blockIdx.x; c < chunks; c += gridDim.x) {
        if (threadIdx.x == 0) total = 0u;
        __syncthreads();
        uint32_t mine = 0;
        int64_t base = c * kFilterChunk + (int64_t)threadIdx.x * 4;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (base + k < numel && mag_key(x[base + k]) == thr) ++mine;
        if (mine) atomicAdd(&total, mine);
        __syncthreads();
        if (threadIdx.x == 0) chunk_ties[c] = total;
        __syncthreads();
    }
}

// one workgroup: exclusive prefix sum of the per-chunk tie counts, in place
__global__ void __launch_bounds__(1024)
topk_scan_kernel(uint32_t* chunk_ties, int64_t chunks)
{
    __shared__ uint32_t part[1024];
    int64_t per = (chunks + 1023) / 1024;
    int64_t lo = (int64_t)threadIdx.x * per;
    int64_t hi = lo + per < chunks ? lo + per : chunks;
    uint32_t s = 0;
    for (int64_t i = lo; i < hi; ++i) s += chunk_ties[i];
    part[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (int t = 0; t < 1024; ++t) {
            uint32_t v = part[t];
            part[t] = run;
            run += v;
        }
    }
    __syncthreads();
    uint32_t run = part[threadIdx.x];
    for (int64_t i = lo; i < hi; ++i) {
        uint32_t v = chunk_ties[i];
        chunk_ties[i] = run;
        run += v;
    }
}

// keep key > threshold, keep the first `remaining` keys == threshold in index order, zero the rest
__global__ void __launch_bounds__(256)
topk_filter_kernel(float* __restrict__ x, int64_t numel, const TopkState* st, const uint32_t* chunk_ties,
                   int64_t chunks)
{
    __shared__ uint32_t wave_ties[4];
    const uint32_t thr = st->prefix;
    const uint32_t keep_ties = st->remaining;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int64_t c = blockIdx.x; c < chunks; c += gridDim.x) {
        int64_t base = c * kFilterChunk + (int64_t)threadIdx.x * 4;
        float v[4];
        uint32_t mine = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            v[k] = base + k < numel ? x[base + k] : 0.f;
            if (base + k < numel && mag_key(v[k]) == thr) ++mine;
        }
        // exclusive rank of this thread's first tie inside the chunk: scan over lanes, then waves
        uint32_t incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            uint32_t t = __shfl_up(incl, off, 64);
            if (lane >= off) incl += t;
        }
        if (lane == 63) wave_ties[wave] = incl;
        __syncthreads();
        uint32_t rank = chunk_ties[c] + incl - mine;
        for (int wv = 0; wv < wave; ++wv) rank += wave_ties[wv];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if (base + k < numel) {
                uint32_t key = mag_key(v[k]);
                bool keep = key > thr;
                if (key == thr) {
                    keep = rank < keep_ties;
                    ++rank;
                }
                if (!keep) x[base + k] = 0.f;
            }
        }
        __syncthreads();
    }
}

inline int64_t topk_chunks(int64_t numel) { return (numel + kFilterChunk - 1) / kFilterChunk; }

}  // namespace

extern "C" {

int64_t conef_topk_workspace_bytes(int64_t numel)
{
    if (numel < 0) return -1;
    return (int64_t)sizeof(TopkState) + (int64_t)sizeof(uint32_t) * (topk_chunks(numel) + 1);
}

int conef_topk_sparsify_f32(float* x, int64_t numel, int64_t k, void* workspace, int64_t workspace_bytes,
                            void* stream)
{
    if (numel < 1 || k < 1 || !x || numel > 0xffffffffLL) return CONEF_ERR_INVALID;
    if (k >= numel) return CONEF_OK;
    if (!workspace || workspace_bytes < conef_topk_workspace_bytes(numel)) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    TopkState* st = (TopkState*)workspace;
    uint32_t* chunk_ties = (uint32_t*)((char*)workspace + sizeof(TopkState));
    int64_t g = (numel + 255) / 256 / 8;
    if (g < 1) g = 1;
    if (g > 2048) g = 2048;
    hipLaunchKernelGGL(topk_init_kernel, dim3(1), dim3(256), 0, s, st, (uint32_t)k);
    for (int pass = 0; pass < 4; ++pass) {
        hipLaunchKernelGGL(topk_hist_kernel, dim3((unsigned)g), dim3(256), 0, s, x, numel, st, pass);
        hipLaunchKernelGGL(topk_select_kernel, dim3(1), dim3(256), 0, s, st, pass);
    }
    int64_t chunks = topk_chunks(numel);
    int64_t cg = chunks < 4096 ? chunks : 4096;
    hipLaunchKernelGGL(topk_count_ties_kernel, dim3((unsigned)cg), dim3(256), 0, s, x, numel, st, chunk_ties, chunks);
    hipLaunchKernelGGL(topk_scan_kernel, dim3(1), dim3(1024), 0, s, chunk_ties, chunks);
    hipLaunchKernelGGL(topk_filter_kernel, dim3((unsigned)cg), dim3(256), 0, s, x, numel, st, chunk_ties, chunks);
    return (int)hipGetLastError();
}

}  // extern "C"
