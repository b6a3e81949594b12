// One foreign call per bucket for the random-block hooks: every >= 2-D tensor of a bucket goes
// through its fused step from a table of items, instead of one call per tensor from the hook's
// Python loop (reference loops: RandomBlock_hook.py:215-245, UnbiasedRandomBlock_hook.py:150-170).
//
// The dense steps (unbiased block, dense error feedback) of all tensors share one launch: the table
// travels by value, a workgroup finds its tensor from the running workgroup count and then does
// what it would do in a launch of its own.  Sketched steps on row-list plans share one launch the
// same way; a sketched step on a binned plan (a few long rows) or without a plan is issued by its
// single-tensor launcher from inside this call.  Same kernels' arithmetic on the same values: the
// results are bit-identical to the single-tensor entry points.
#include <vector>

#include "conef_plan.h"
#include "conef_randblock_core.h"
#include "conef_hip.h"

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kRbBatchMax = 16;

template <typename Item>
struct RbBatch {
    Item item[kRbBatchMax];
    int first[kRbBatchMax + 1];   // first workgroup of item i; first[count] = workgroups in all
    int count;
};

template <typename Item>
__device__ __forceinline__ int rb_locate(const RbBatch<Item>& b, int* local, int* width)
{
    int i = 0;
    while (i + 1 < b.count && (int)blockIdx.x >= b.first[i + 1]) ++i;
    *local = (int)blockIdx.x - b.first[i];
    *width = b.first[i + 1] - b.first[i];
    return i;
}

struct DenseItem {
    float* x;
    float* err;        // dense error (mode 1), unused otherwise
    float* payload;
    int64_t numel;
    ConefBlock blk;
    float prob;        // mode 0
    int vec;
};

__global__ void __launch_bounds__(256) randblock_unbiased_batch_kernel(RbBatch<DenseItem> b)
{
    int local, width;
    const DenseItem& it = b.item[rb_locate(b, &local, &width)];
    if (it.vec) conef_randblock_unbiased_body<true>(it.x, it.payload, it.numel, it.blk, it.prob, local, width);
    else conef_randblock_unbiased_body<false>(it.x, it.payload, it.numel, it.blk, it.prob, local, width);
}

__global__ void __launch_bounds__(256) randblock_ef_batch_kernel(RbBatch<DenseItem> b)
{
    int local, width;
    const DenseItem& it = b.item[rb_locate(b, &local, &width)];
    if (it.vec) conef_randblock_ef_body<true>(it.x, it.err, it.payload, it.numel, it.blk, local, width);
    else conef_randblock_ef_body<false>(it.x, it.err, it.payload, it.numel, it.blk, local, width);
}

struct ListItem {
    ConefListRandBlock front;
    ConefRowlistView plan;
    const float* cs_in;
    float* cs_out;
    int64_t n;
    int d, w, rb;
    bool pk_lds;
};

__global__ void __launch_bounds__(kConefRowlistThreads)
randblock_rowlist_batch_kernel(RbBatch<ListItem> b, double one_minus_beta)
{
    int local, width;
    const ListItem& it = b.item[rb_locate(b, &local, &width)];
    conef_rowlist_body<float, ConefListRandBlock>(it.front, it.plan, it.cs_in, it.cs_out, it.n, it.d, it.w, it.rb,
                                                  one_minus_beta, local, it.pk_lds);
}

template <typename Item, typename Go>
int rb_run(const std::vector<Item>& table, const std::vector<int>& blocks, Go go)
{
    size_t k = 0;
    while (k < table.size()) {
        RbBatch<Item> b;
        int nb = 0, total = 0;
        while (k < table.size() && nb < kRbBatchMax) {
            b.item[nb] = table[k];
            b.first[nb] = total;
            total += blocks[k];
            ++nb;
            ++k;
        }
        b.first[nb] = total;
        b.count = nb;
        if (total > 0) go(b, total);
    }
    return (int)hipGetLastError();
}

}  // namespace

extern "C" {

int conef_randblock_step_batch_f32(const ConefRandBlockItem* items, int32_t count, int32_t mode, float alpha,
                                   float beta, int32_t a, int32_t b, void* stream)
{
    if (count < 0 || (count > 0 && !items) || mode < 0 || mode > 2) return CONEF_ERR_INVALID;
    if (count == 0) return CONEF_OK;
    // everything is checked before anything is enqueued
    for (int k = 0; k < count; ++k) {
        const ConefRandBlockItem& it = items[k];
        if (it.n < 1 || it.m < 1 || (mode == 2 && it.m > 0x7fffffffLL) || !it.x || !it.payload) return CONEF_ERR_INVALID;
        const int64_t numel = it.n * it.m;
        if (!(it.start >= 0 && it.start < numel && it.block >= 1 && it.block <= numel)) return CONEF_ERR_INVALID;
        if (mode == 1 && !it.err) return CONEF_ERR_INVALID;
        if (mode == 2) {
            if (!it.cs_in || !it.cs_out || it.w < 1 || it.w > (1 << 30)) return CONEF_ERR_INVALID;
            if (it.plan_host) {
                const ConefPlanHeader* hp = (const ConefPlanHeader*)it.plan_host;
                if (!conef_plan_matches(hp, it.n, it.m, it.w, a, b) || !it.plan_dev) return CONEF_ERR_INVALID;
                if (hp->kind == kConefPlanBinned && (!it.staging || it.cs_in == it.cs_out)) return CONEF_ERR_INVALID;
            }
        }
    }
    hipStream_t s = (hipStream_t)stream;
    if (mode == 0 || mode == 1) {
        std::vector<DenseItem> table;
        std::vector<int> blocks;
        for (int k = 0; k < count; ++k) {
            const ConefRandBlockItem& it = items[k];
            const int64_t numel = it.n * it.m;
            DenseItem d;
            d.x = it.x;
            d.err = it.err;
            d.payload = it.payload;
            d.numel = numel;
            d.blk = conef_make_block(numel, it.start, it.block);
            // the reference divides by the Python double block / numel, which reaches the tensor as fp32
            d.prob = (float)((double)it.block / (double)numel);
            d.vec = aligned16(it.x) && (mode == 0 || aligned16(it.err));
            table.push_back(d);
            blocks.push_back(conef_grid_for((numel + 3) / 4, 256));
        }
        if (mode == 0)
            return rb_run(table, blocks, [&](const RbBatch<DenseItem>& bt, int grid) {
                hipLaunchKernelGGL(randblock_unbiased_batch_kernel, dim3((unsigned)grid), dim3(256), 0, s, bt);
            });
        return rb_run(table, blocks, [&](const RbBatch<DenseItem>& bt, int grid) {
            hipLaunchKernelGGL(randblock_ef_batch_kernel, dim3((unsigned)grid), dim3(256), 0, s, bt);
        });
    }
    // sketched error: row-list plans share launches, the rest go one by one
    std::vector<ListItem> table;
    std::vector<int> blocks;
    size_t lds = 0;
    for (int k = 0; k < count; ++k) {
        const ConefRandBlockItem& it = items[k];
        const ConefPlanHeader* hp = (const ConefPlanHeader*)it.plan_host;
        if (!hp || hp->kind != kConefPlanRowlist) continue;
        ConefRowlistShape shape;
        if (!conef_rowlist_shape(it.n, it.m, it.w, ConefListRandBlock::kNeedsCells, &shape)) return CONEF_ERR_INVALID;
        ListItem t = {{it.x, it.payload, conef_make_block(it.n * it.m, it.start, it.block), alpha},
                      conef_rowlist_view(hp, it.plan_dev), it.cs_in, it.cs_out, it.n, (int)it.m, it.w, shape.rb, shape.pk_lds};
        table.push_back(t);
        blocks.push_back((int)shape.tiles);
        if (shape.lds > lds) lds = shape.lds;
    }
    if (!table.empty()) {
        hipError_t e = conef_allow_lds((const void*)randblock_rowlist_batch_kernel, lds);
        if (e != hipSuccess) return (int)e;
        const double omb = 1. - (double)beta;
        int rc = rb_run(table, blocks, [&](const RbBatch<ListItem>& bt, int grid) {
            hipLaunchKernelGGL(randblock_rowlist_batch_kernel, dim3((unsigned)grid), dim3(kConefRowlistThreads), lds, s,
                               bt, omb);
        });
        if (rc != CONEF_OK) return rc;
    }
    for (int k = 0; k < count; ++k) {
        const ConefRandBlockItem& it = items[k];
        const ConefPlanHeader* hp = (const ConefPlanHeader*)it.plan_host;
        if (hp && hp->kind == kConefPlanRowlist) continue;
        int rc;
        if (hp)
            rc = conef_randblock_conef_step_planned_f32(it.x, it.cs_in, it.cs_out, it.payload, it.plan_host, it.plan_dev,
                                                        it.staging, it.n, it.m, it.w, it.start, it.block, alpha, beta, a,
                                                        b, stream);
        else
            rc = conef_randblock_conef_step_f32(it.x, it.cs_in, it.cs_out, it.payload, it.n, it.m, it.w, it.start,
                                                it.block, alpha, beta, a, b, stream);
        if (rc != CONEF_OK) return rc;
    }
    return CONEF_OK;
}

}  // extern "C"
