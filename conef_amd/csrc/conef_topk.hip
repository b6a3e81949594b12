// Magnitude top-k sparsifier (gfx950) for the dense error kept by the hPowerSGD hook.
//
// Reference semantics: communication/hPowerSGD_hook.py:90-97 - keep the k entries of largest
// magnitude, zero everything else, in place.  The reference asks torch.topk for unsorted
// positions and so leaves ties open; here ties on the threshold magnitude keep the lowest flat
// indices, which makes the result a function of the input alone.
//
// Selection is a most-significant-digit radix select on the 31 magnitude bits (a non-negative
// float orders like its bit pattern) in three histogram passes of 11, 11 and 9 bits.  Choosing the
// digit that holds the k-th largest key is not a launch of its own: every workgroup of the next
// pass does it from the finished histogram before it starts (2048 counters, one suffix scan).
// The filter keeps every key at or above the threshold.  If more keys equal the threshold than may
// be kept (two equal magnitudes at the threshold turn up in a few percent of million-element
// gradients; at a zero threshold it makes no difference which zeros stay), the filter's workgroups
// also note where those keys sit, and the workgroup that finishes last ranks the noted indices
// and clears the ties past the first `remaining` of them.  More than 1024 such ties (a tensor of
// repeated values) are settled by one workgroup walking the tensor in index order instead: exact,
// slow, and of no practical concern.  Nothing returns to the host between passes.
#include <mutex>

#include "conef_device.h"
#include "conef_hip.h"

namespace {

constexpr int kPasses = 3;
constexpr int kDigitBits[kPasses] = {11, 11, 9};
constexpr int kDigitShift[kPasses] = {20, 9, 0};
constexpr int kBins = 2048;          // bins of the widest digit
constexpr int kFilterChunk = 1024;   // elements per workgroup iteration in the ordered walk
constexpr int kTieMax = 1024;        // surplus ties up to this many are ranked from a list, more by a walk

struct TopkState {
    uint32_t k;
    uint32_t prefix[kPasses];       // prefix[p]: selected digits of passes 0..p, written by pass p + 1
    uint32_t remaining[kPasses];    // how many keys to take among those matching prefix[p]
    uint32_t ties[kPasses];         // keys that match prefix[p] exactly in their high digits
    uint32_t done;                  // workgroups of the filter that have finished (surplus ties only)
    uint32_t tie_count;             // indices recorded in tie_idx so far
    uint32_t pad[4];
    uint32_t hist[kPasses][kBins];
    uint32_t tie_idx[kTieMax];      // where the keys equal to the threshold sit, in no order
};

__device__ __forceinline__ uint32_t mag_key(float v) { return __float_as_uint(v) & 0x7fffffffu; }

// Several tensors per launch (the dense errors of a bucket's matrices, each with its own k and its
// own state): the table travels by value, a workgroup finds its tensor from the running workgroup
// count (`first`, the same for every pass) and then
// does what it would do in a launch of its own.
constexpr int kTopkBatchMax = 24;

struct TopkItem {
    float* x;
    int64_t numel;
    TopkState* st;
    uint32_t k;
};

struct TopkBatch {
    TopkItem item[kTopkBatchMax];
    int first[kTopkBatchMax + 1];
    int count;
};

__device__ __forceinline__ int topk_locate(const int* first, int count, int* local, int* width)
{
    int i = 0;
    while (i + 1 < count && (int)blockIdx.x >= first[i + 1]) ++i;
    *local = (int)blockIdx.x - first[i];
    *width = first[i + 1] - first[i];
    return i;
}

__device__ __forceinline__ void topk_init_body(TopkState* st, uint32_t k)
{
    for (int i = threadIdx.x; i < kPasses * kBins; i += blockDim.x) (&st->hist[0][0])[i] = 0u;
    if (threadIdx.x == 0) {
        st->k = k;
        st->done = 0u;
        st->tie_count = 0u;
    }
}

__global__ void topk_init_kernel(TopkState* st, uint32_t k) { topk_init_body(st, k); }

__global__ void topk_init_batch_kernel(TopkBatch b) { topk_init_body(b.item[blockIdx.x].st, b.item[blockIdx.x].k); }

// What pass `p` selected, from its finished histogram: the digit holding the k-th largest key
// among those matching the earlier digits.  Every thread of a 256-thread workgroup returns the
// same (prefix, remaining, ties); workgroup 0 (bx) of the tensor also leaves them in the state for
// the next kernel.
__device__ __forceinline__ void topk_resolve(TopkState* st, int p, uint32_t* prefix, uint32_t* remaining, uint32_t* ties,
                                             int bx)
{
    __shared__ uint32_t wave_sum[4];
    __shared__ uint32_t picked[3];
    const uint32_t before_prefix = p == 0 ? 0u : st->prefix[p - 1];
    const uint32_t before_remaining = p == 0 ? st->k : st->remaining[p - 1];
    const int bins = 1 << kDigitBits[p], per = bins / 256;          // 8, 8, 2 bins per thread
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    uint32_t cnt[8];
    uint32_t mine = 0;
    for (int b = 0; b < per; ++b) {
        cnt[b] = st->hist[p][threadIdx.x * per + b];
        mine += cnt[b];
    }
    // suffix sums over threads: keys in digits above mine
    uint32_t incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        uint32_t t = __shfl_down(incl, off, 64);
        if (lane + off < 64) incl += t;
    }
    if (lane == 0) wave_sum[wave] = incl;
    __syncthreads();
    uint32_t above = incl - mine;
    for (int wv = wave + 1; wv < 4; ++wv) above += wave_sum[wv];
    // exactly one (thread, bin) satisfies above < remaining <= above + count
    for (int b = per - 1; b >= 0; --b) {
        if (above < before_remaining && before_remaining <= above + cnt[b]) {
            picked[0] = (before_prefix << kDigitBits[p]) | (uint32_t)(threadIdx.x * per + b);
            picked[1] = before_remaining - above;
            picked[2] = cnt[b];
        }
        above += cnt[b];
    }
    __syncthreads();
    *prefix = picked[0];
    *remaining = picked[1];
    *ties = picked[2];
    if (bx == 0 && threadIdx.x == 0) {
        st->prefix[p] = picked[0];
        st->remaining[p] = picked[1];
        st->ties[p] = picked[2];
    }
    __syncthreads();
}

// REP copies of every bin, copy = lane % REP, laid out [bin][copy]: the keys of a gradient crowd
// into a few dozen bins of the first digit (one exponent and three mantissa bits), and lanes of a
// wave that meet in a bin then add to different LDS banks instead of queueing on one address.
// `kept` (a state that stays with its tensor from call to call, zero-filled before the first): no
// launch clears the state; the first workgroup of pass 0 clears what the later passes count into,
// and the filter's clears what pass 0 of the next call counts into (topk_filter_body).
template <int REP>
__device__ __forceinline__ void
topk_hist_body(const float* __restrict__ x, int64_t numel, TopkState* st, int pass, int bx, int gx, bool kept = false,
               uint32_t k = 0)
{
    __shared__ uint32_t bins[kBins * REP];
    uint32_t prefix = 0, remaining = 0, ties = 0;
    if (pass > 0) topk_resolve(st, pass - 1, &prefix, &remaining, &ties, bx);
    if (kept && pass == 0 && bx == 0) {
        for (int i = threadIdx.x; i < (kPasses - 1) * kBins; i += 256) (&st->hist[1][0])[i] = 0u;
        if (threadIdx.x == 0) {
            st->k = k;
            st->done = 0u;
            st->tie_count = 0u;
        }
    }
    const int nb = 1 << kDigitBits[pass];
    for (int i = threadIdx.x; i < nb * REP; i += 256) bins[i] = 0u;
    __syncthreads();
    const int shift = kDigitShift[pass], hi = shift + kDigitBits[pass];
    const uint32_t mask = (uint32_t)nb - 1u;
    const int copy = (int)(threadIdx.x & (REP - 1));
    const int64_t quads = numel >> 2;
    const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    const int64_t stride = (int64_t)gx * blockDim.x;
    if (vec) {
        // eight 16-byte loads in flight per thread: a thread's share is sixteen quads or so, and every
        // round of loads is a trip to memory
        constexpr int U = 8;
        for (int64_t q0 = bx * (int64_t)blockDim.x + threadIdx.x; q0 < quads; q0 += U * stride) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t q = q0 + u * stride;
                v[u] = reinterpret_cast<const float4*>(x)[q < quads ? q : q0];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (q0 + u * stride >= quads) break;
                const uint32_t key[4] = {mag_key(v[u].x), mag_key(v[u].y), mag_key(v[u].z), mag_key(v[u].w)};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (pass == 0 || (key[e] >> hi) == prefix) atomicAdd(&bins[((key[e] >> shift) & mask) * REP + copy], 1u);
            }
        }
    }
    for (int64_t i = (vec ? quads * 4 : 0) + bx * (int64_t)blockDim.x + threadIdx.x; i < numel; i += stride) {
        uint32_t key = mag_key(x[i]);
        if (pass == 0 || (key >> hi) == prefix) atomicAdd(&bins[((key >> shift) & mask) * REP + copy], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nb; i += 256) {
        uint32_t c = 0;
#pragma unroll
        for (int k = 0; k < REP; ++k) c += bins[i * REP + k];
        if (c) atomicAdd(&st->hist[pass][i], c);
    }
}

// pass 0 counts every key (replicated bins), the later passes only the few that match the prefix
__global__ void __launch_bounds__(256)
topk_hist_kernel(const float* __restrict__ x, int64_t numel, TopkState* st, int pass)
{
    if (pass == 0) topk_hist_body<4>(x, numel, st, 0, (int)blockIdx.x, (int)gridDim.x);
    else topk_hist_body<1>(x, numel, st, pass, (int)blockIdx.x, (int)gridDim.x);
}

__global__ void __launch_bounds__(256)
topk_hist_batch_kernel(TopkBatch b, int pass, bool kept)
{
    int local, width;
    const TopkItem& it = b.item[topk_locate(b.first, b.count, &local, &width)];
    if (pass == 0) topk_hist_body<4>(it.x, it.numel, it.st, 0, local, width, kept, it.k);
    else topk_hist_body<1>(it.x, it.numel, it.st, pass, local, width);
}

// keys equal to the threshold, in index order: the first `keep_ties` stay, the rest are cleared.
// One workgroup of 256 threads, 1024 elements a round; once the quota is used up the rounds need
// no scan any more.
__device__ __forceinline__ void topk_order_ties(float* __restrict__ x, int64_t numel, uint32_t thr, uint32_t keep_ties)
{
    __shared__ uint32_t wave_ties[4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    uint32_t running = 0;                       // ties seen in earlier rounds: the same in every thread
    for (int64_t base0 = 0; base0 < numel; base0 += kFilterChunk) {
        const int64_t base = base0 + (int64_t)threadIdx.x * 4;
        bool tie[4];
        uint32_t mine = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            tie[k] = base + k < numel && mag_key(x[base + k]) == thr;
            mine += tie[k];
        }
        if (running >= keep_ties) {             // uniform: nothing more may stay
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (tie[k]) x[base + k] = 0.f;
            continue;
        }
        uint32_t incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            uint32_t t = __shfl_up(incl, off, 64);
            if (lane >= off) incl += t;
        }
        if (lane == 63) wave_ties[wave] = incl;
        __syncthreads();
        uint32_t rank = running + incl - mine;
        for (int wv = 0; wv < wave; ++wv) rank += wave_ties[wv];
        const uint32_t total = (wave_ties[0] + wave_ties[1]) + (wave_ties[2] + wave_ties[3]);
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (tie[k]) {
                if (rank >= keep_ties) x[base + k] = 0.f;
                ++rank;
            }
        running += total;
        __syncthreads();
    }
}

// keep key >= threshold, zero the rest, settle surplus ties on the threshold by index
__device__ __forceinline__ void
topk_filter_body(float* __restrict__ x, int64_t numel, TopkState* st, int bx, int gx, bool kept = false)
{
    __shared__ uint32_t ticket;
    __shared__ uint32_t idx_l[kTieMax];
    uint32_t thr, keep_ties, ties;
    topk_resolve(st, kPasses - 1, &thr, &keep_ties, &ties, bx);
    if (kept && bx == 0)       // nobody reads the first digit's counters any more: ready for the next call
        for (int i = threadIdx.x; i < kBins; i += 256) st->hist[0][i] = 0u;
    const bool surplus = ties != keep_ties && thr != 0u;      // a zero threshold has only zeros for ties
    const bool listed = surplus && ties <= (uint32_t)kTieMax;
    auto note = [&](int64_t i) {
        const uint32_t slot = atomicAdd(&st->tie_count, 1u);
        if (slot < (uint32_t)kTieMax) st->tie_idx[slot] = (uint32_t)i;
    };
    const int64_t quads = numel >> 2;
    const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    const int64_t stride = (int64_t)gx * blockDim.x;
    if (vec) {
        // eight quads requested before the first is used (a load behind a store to the same array is
        // not moved up by the compiler: one quad a trip otherwise)
        constexpr int U = 8;
        for (int64_t q0 = bx * (int64_t)blockDim.x + threadIdx.x; q0 < quads; q0 += U * stride) {
            float4 vv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t q = q0 + u * stride;
                vv[u] = reinterpret_cast<const float4*>(x)[q < quads ? q : q0];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t q = q0 + u * stride;
                if (q >= quads) break;
                const float4 v = vv[u];
                const uint32_t key[4] = {mag_key(v.x), mag_key(v.y), mag_key(v.z), mag_key(v.w)};
                bool k0 = key[0] >= thr, k1 = key[1] >= thr, k2 = key[2] >= thr, k3 = key[3] >= thr;
                if (!(k0 && k1 && k2 && k3))
                    reinterpret_cast<float4*>(x)[q] = make_float4(k0 ? v.x : 0.f, k1 ? v.y : 0.f, k2 ? v.z : 0.f, k3 ? v.w : 0.f);
                if (listed) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (key[e] == thr) note(4 * q + e);
                }
            }
        }
    }
    for (int64_t i = (vec ? quads * 4 : 0) + bx * (int64_t)blockDim.x + threadIdx.x; i < numel; i += stride) {
        const uint32_t key = mag_key(x[i]);
        if (key < thr) x[i] = 0.f;
        else if (listed && key == thr) note(i);
    }
    if (!surplus) return;
    // The workgroup that finishes last sees every noted index, and nobody else's 16-byte stores
    // (which rewrite a tie with its own value when a neighbour in the quad goes) can land after
    // the zeros it writes.
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) ticket = atomicAdd(&st->done, 1u);
    __syncthreads();
    if (ticket != (uint32_t)gx - 1u) return;
    __threadfence();
    if (!listed) {
        topk_order_ties(x, numel, thr, keep_ties);
        return;
    }
    const int n = (int)ties;
    for (int j = threadIdx.x; j < n; j += blockDim.x)
        idx_l[j] = __hip_atomic_load(&st->tie_idx[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    for (int j = threadIdx.x; j < n; j += blockDim.x) {
        const uint32_t mine = idx_l[j];
        uint32_t rank = 0;
        for (int t = 0; t < n; ++t) rank += idx_l[t] < mine;
        if (rank >= keep_ties) x[mine] = 0.f;
    }
}

__global__ void __launch_bounds__(256)
topk_filter_kernel(float* __restrict__ x, int64_t numel, TopkState* st)
{
    topk_filter_body(x, numel, st, (int)blockIdx.x, (int)gridDim.x);
}

__global__ void __launch_bounds__(256)
topk_filter_batch_kernel(TopkBatch b, bool kept)
{
    int local, width;
    const TopkItem& it = b.item[topk_locate(b.first, b.count, &local, &width)];
    topk_filter_body(it.x, it.numel, it.st, local, width, kept);
}


// Workgroups of a pass over a tensor.  A histogram workgroup ends with one global atomic per bin
// it touched, all workgroups on the same few dozen counters, and a filter workgroup that has to
// settle ties ends with one on a single counter: fewer workgroups with longer loops (16 quads a
// thread) beat many short ones.
inline int64_t topk_hist_groups(int64_t numel)
{
    int64_t g = (numel + 255) / 256 / 64;
    return g < 1 ? 1 : g > 512 ? 512 : g;
}


// ---- selection state of the entry point that allocates nothing ------------------------------
// One TopkState per GPU, inside the code object: every GPU the library runs on holds its own
// copy at its own address until the process ends.  `scratch` is only a host-side handle of the
// symbol; kernels (topk_init_kernel clears the state at the start of every call) need the address
// hipGetSymbolAddress returns for the device that is current, looked up once per device and kept.
constexpr size_t kScratchBytes = (sizeof(TopkState) + 255) / 256 * 256;      // 29 184 bytes
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kScratchMaxDevices = 64;
std::mutex g_scratch_lock;
void* g_scratch_ptr[kScratchMaxDevices] = {};

// Address of the current device's copy of `scratch`, or null with *err set.
inline void* topk_scratch_of_current_device(int* err)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        *err = (int)e;
        return nullptr;
    }
    if (dev < 0 || dev >= kScratchMaxDevices) {
        *err = CONEF_ERR_INVALID;
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            *err = e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *err = CONEF_OK;
    return g_scratch_ptr[dev];
}

}  // namespace

extern "C" {

int64_t conef_topk_workspace_bytes(int64_t numel)
{
    if (numel < 0) return -1;
    return ((int64_t)sizeof(TopkState) + 255) / 256 * 256;      // the selection state; nothing grows with numel
}

int conef_topk_sparsify_f32(float* x, int64_t numel, int64_t k, void* workspace, int64_t workspace_bytes,
                            void* stream)
{
    if (numel < 1 || k < 1 || !x || numel > 0xffffffffLL) return CONEF_ERR_INVALID;
    if (k >= numel) return CONEF_OK;
    if (!workspace || workspace_bytes < conef_topk_workspace_bytes(numel)) return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    TopkState* st = (TopkState*)workspace;
    const int64_t g = topk_hist_groups(numel);
    hipLaunchKernelGGL(topk_init_kernel, dim3(1), dim3(256), 0, s, st, (uint32_t)k);
    for (int pass = 0; pass < kPasses; ++pass)
        hipLaunchKernelGGL(topk_hist_kernel, dim3((unsigned)g), dim3(256), 0, s, x, numel, st, pass);
    hipLaunchKernelGGL(topk_filter_kernel, dim3((unsigned)g), dim3(256), 0, s, x, numel, st);
    return (int)hipGetLastError();
}

// The same for `count` tensors, every pass one launch over all of them (in runs of 24): tensor i
// is xs[i] with numels[i] elements and keeps ks[i]; tensors with ks[i] >= numels[i] are left as
// they are.  xs / numels / ks are host arrays, read before the call returns.
int64_t conef_topk_batch_workspace_bytes(const int64_t* numels, int32_t count)
{
    if (count < 0 || (count > 0 && !numels)) return -1;
    int64_t total = 0;
    for (int i = 0; i < count; ++i) {
        if (numels[i] < 0) return -1;
        total += (conef_topk_workspace_bytes(numels[i]) + 255) / 256 * 256;
    }
    return total > 256 ? total : 256;
}

namespace {
int topk_sparsify_batch(float* const* xs, const int64_t* numels, const int64_t* ks, int32_t count, void* workspace,
                        int64_t workspace_bytes, void* stream, bool kept)
{
    if (count < 0 || (count > 0 && (!xs || !numels || !ks))) return CONEF_ERR_INVALID;
    for (int i = 0; i < count; ++i)
        if (numels[i] < 1 || ks[i] < 1 || !xs[i] || numels[i] > 0xffffffffLL) return CONEF_ERR_INVALID;
    if (count > 0 && (!workspace || workspace_bytes < conef_topk_batch_workspace_bytes(numels, count) ||
                      (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0))
        return CONEF_ERR_INVALID;
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    int i = 0;
    while (i < count) {
        TopkBatch b;
        int nb = 0, wgs = 0;
        for (; i < count && nb < kTopkBatchMax; ++i) {
            char* mine = ws;
            ws += (conef_topk_workspace_bytes(numels[i]) + 255) / 256 * 256;
            if (ks[i] >= numels[i]) continue;
            TopkItem& it = b.item[nb];
            it.x = xs[i];
            it.numel = numels[i];
            it.st = (TopkState*)mine;
            it.k = (uint32_t)ks[i];
            b.first[nb] = wgs;
            wgs += (int)topk_hist_groups(numels[i]);
            ++nb;
        }
        if (nb == 0) continue;
        b.first[nb] = wgs;
        b.count = nb;
        if (!kept) hipLaunchKernelGGL(topk_init_batch_kernel, dim3((unsigned)nb), dim3(256), 0, s, b);
        for (int pass = 0; pass < kPasses; ++pass)
            hipLaunchKernelGGL(topk_hist_batch_kernel, dim3((unsigned)wgs), dim3(256), 0, s, b, pass, kept);
        hipLaunchKernelGGL(topk_filter_batch_kernel, dim3((unsigned)wgs), dim3(256), 0, s, b, kept);
    }
    return (int)hipGetLastError();
}
}  // namespace

int conef_topk_sparsify_batch_f32(float* const* xs, const int64_t* numels, const int64_t* ks, int32_t count,
                                  void* workspace, int64_t workspace_bytes, void* stream)
{
    return topk_sparsify_batch(xs, numels, ks, count, workspace, workspace_bytes, stream, false);
}

// The same for a workspace that stays with its tensors: zero-filled by the caller before its first
// use and passed to nothing but this entry point, with the same xs / numels / count, afterwards.
// No launch clears the selection state then (the passes clear behind themselves): four launches a
// call instead of five.
int conef_topk_sparsify_batch_kept_f32(float* const* xs, const int64_t* numels, const int64_t* ks, int32_t count,
                                       void* workspace, int64_t workspace_bytes, void* stream)
{
    return topk_sparsify_batch(xs, numels, ks, count, workspace, workspace_bytes, stream, true);
}


// conef_topk_sparsify_f32 for callers that may not allocate (HIP graph capture, serving loops):
// the selection state lives in the library's own per-GPU scratch (29 184 bytes), so no workspace
// is passed.  The device the stream belongs to must be current.  Calls on one GPU share that
// scratch: calls that may overlap there (different streams, different threads) race; calls on
// one stream are safe back to back because the first kernel of a call resets the state.
int conef_topk_sparsify_noalloc_f32(float* x, int64_t numel, int64_t k, void* stream)
{
    if (numel < 1 || k < 1 || !x) return CONEF_ERR_INVALID;
    if (numel > CONEF_TOPK_NOALLOC_MAX_NUMEL) return CONEF_ERR_TOO_LARGE;
    if (k >= numel) return CONEF_OK;
    int err = CONEF_OK;
    void* ptr = topk_scratch_of_current_device(&err);
    if (!ptr) return err;
    hipStream_t s = (hipStream_t)stream;
    TopkState* st = (TopkState*)ptr;
    const int64_t g = topk_hist_groups(numel);
    hipLaunchKernelGGL(topk_init_kernel, dim3(1), dim3(256), 0, s, st, (uint32_t)k);      // clears what the last call left
    for (int pass = 0; pass < kPasses; ++pass)
        hipLaunchKernelGGL(topk_hist_kernel, dim3((unsigned)g), dim3(256), 0, s, x, numel, st, pass);
    hipLaunchKernelGGL(topk_filter_kernel, dim3((unsigned)g), dim3(256), 0, s, x, numel, st);
    return (int)hipGetLastError();
}

}  // extern "C"
