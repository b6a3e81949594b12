// Entry points of the planned (atomic-free, deterministic) sketch accumulation: row lists when a
// row fits LDS (conef_rowlist.h), two binned passes for a few long rows (conef_plan.h).
#include "conef_plan.h"

namespace {
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// the sign-hash seeds a plan's tables were built with
inline bool plan_has_default_sign_seeds(const ConefPlanHeader* hp, int32_t a, int32_t b)
{
    return hp->seeds == (((int64_t)(uint32_t)(a + 2) << 32) | (uint32_t)(b + 3));
}
}  // namespace

// conef_sketch.hip
int conef_launch_query_rows8_f32(float* x, const float* cs, int64_t n, int64_t d, int32_t w, float alpha,
                                 const uint32_t* pktab, float* scratch, hipStream_t stream);
int conef_launch_query_table_f32(float* x, const float* cs, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                                 int32_t b, const uint32_t* pktab, hipStream_t stream);
int conef_launch_query_table_f16(float* x, const void* cs_half, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                                 int32_t b, const uint32_t* pktab, hipStream_t stream);

extern "C" {

// Bytes of a plan for an [n,d] tensor sketched at width w; 0 when no planned path applies (more
// than half a million long rows), -1 on invalid arguments.  chunk_cols / bin_buckets: 0 picks the
// kind and its defaults, a positive value asks for a binned plan with that tiling.
int64_t conef_plan_bytes(int64_t n, int64_t d, int32_t w, int32_t chunk_cols, int32_t bin_buckets)
{
    if (n < 1 || d < 1 || w < 1 || w > (1 << 30) || d > 0x7fffffffLL) return -1;
    ConefPlanHeader h;
    if (!conef_plan_shape(n, d, w, chunk_cols, bin_buckets, &h)) return 0;
    return h.total_bytes;
}

// Builds the plan into HOST memory.  The caller copies the same bytes to the device and passes
// both copies to the *_planned entry points (the host copy is read for launch geometry only).
// The same for a sketch whose sign hash uses the seeds (sa, sb) instead of (a + 2, b + 3): the
// second and third sketch of the three-hash compressor (CountSketchHash3.py:77,85).
int conef_plan_build_host_seeded(void* plan_host, int64_t plan_bytes, int64_t n, int64_t d, int32_t w, int32_t a,
                                 int32_t b, int32_t sa, int32_t sb, int32_t chunk_cols, int32_t bin_buckets)
{
    ConefPlanHeader h;
    if (!plan_host || !conef_plan_shape(n, d, w, chunk_cols, bin_buckets, &h)) return CONEF_ERR_INVALID;
    if (plan_bytes < h.total_bytes) return CONEF_ERR_INVALID;
    if (!conef_plan_fill(plan_host, h, a, b, sa, sb)) return CONEF_ERR_INVALID;
    const ConefPlanHeader* built = (const ConefPlanHeader*)plan_host;
    if (built->kind == kConefPlanBinned &&
        conef_binned_lds_b(built, (int)(n < kConefPlanMaxRows ? n : kConefPlanMaxRows)) > 160 * 1024)
        return CONEF_ERR_INVALID;
    return CONEF_OK;
}

int conef_plan_build_host(void* plan_host, int64_t plan_bytes, int64_t n, int64_t d, int32_t w, int32_t a, int32_t b,
                          int32_t chunk_cols, int32_t bin_buckets)
{
    return conef_plan_build_host_seeded(plan_host, plan_bytes, n, d, w, a, b, a + 2, b + 3, chunk_cols, bin_buckets);
}

int64_t conef_plan_workspace_bytes(const void* plan_host)
{
    const ConefPlanHeader* h = (const ConefPlanHeader*)plan_host;
    if (!h || h->magic != kConefPlanMagic) return -1;
    return h->workspace_bytes;
}

int conef_cs_update_planned_f32(const float* vec, const float* cs_in, float* cs_out, const void* plan_host,
                                const void* plan_dev, void* workspace, int64_t n, int64_t d, int32_t w, float beta,
                                int32_t a, int32_t b, void* stream)
{
    const ConefPlanHeader* hp = (const ConefPlanHeader*)plan_host;
    if (!conef_plan_matches(hp, n, d, w, a, b) || !plan_dev || !vec || !cs_in || !cs_out) return CONEF_ERR_INVALID;
    if (hp->kind == kConefPlanRowlist) {
        ConefListVec front = {vec, aligned16(vec) && d % 4 == 0};
        return conef_launch_rowlist(front, conef_rowlist_view(hp, plan_dev), cs_in, cs_out, n, d, w, beta,
                                    (hipStream_t)stream);
    }
    if (hp->kind == kConefPlanPanels) {
        ConefPanelVec front = {vec, aligned16(vec) && d % 4 == 0};
        return conef_launch_panels(front, conef_panel_view(hp, plan_dev), cs_in, cs_out, n, d, w, beta, (hipStream_t)stream);
    }
    if (!workspace) return CONEF_ERR_INVALID;
    ConefStageVec stage = {vec, d};
    ConefBlockWork none = {};
    return conef_launch_binned(stage, hp, plan_dev, (float*)workspace, cs_in, cs_out, 0.f, beta, aligned16(vec), none,
                               (hipStream_t)stream);
}

// fp16-storage sketch on a row-list plan (cells read as fp16, arithmetic as in the f32 update,
// one rounding to nearest-even when a cell is written); binned plans are f32 only.
int conef_cs_update_planned_f16(const float* vec, const void* cs_in_half, void* cs_out_half, const void* plan_host,
                                const void* plan_dev, int64_t n, int64_t d, int32_t w, float beta, int32_t a,
                                int32_t b, void* stream)
{
    const ConefPlanHeader* hp = (const ConefPlanHeader*)plan_host;
    if (!conef_plan_matches(hp, n, d, w, a, b) || !plan_dev || !vec || !cs_in_half || !cs_out_half)
        return CONEF_ERR_INVALID;
    if (hp->kind == kConefPlanPanels) {
        ConefPanelVec front = {vec, aligned16(vec) && d % 4 == 0};
        return conef_launch_panels(front, conef_panel_view(hp, plan_dev), (const __half*)cs_in_half, (__half*)cs_out_half, n,
                                   d, w, beta, (hipStream_t)stream);
    }
    if (hp->kind != kConefPlanRowlist) return CONEF_ERR_INVALID;
    ConefListVec front = {vec, aligned16(vec) && d % 4 == 0};
    return conef_launch_rowlist(front, conef_rowlist_view(hp, plan_dev), (const __half*)cs_in_half,
                                (__half*)cs_out_half, n, d, w, beta, (hipStream_t)stream);
}

// DenseCS.query with the buckets and signs of a plan's table instead of hashing (either kind of
// plan, built for (n, d, w, a, b) with the default sign seeds): same values, bit for bit.
int conef_cs_query_planned_f32(float* x, const float* cs, const void* plan_host, const void* plan_dev, void* workspace,
                               int64_t n, int64_t d, int32_t w, float alpha, int32_t a, int32_t b, void* stream)
{
    const ConefPlanHeader* hp = (const ConefPlanHeader*)plan_host;
    if (!conef_plan_matches(hp, n, d, w, a, b) || !plan_dev || !plan_has_default_sign_seeds(hp, a, b)) return CONEF_ERR_INVALID;
    const uint32_t* pk = (const uint32_t*)((const char*)plan_dev + hp->off_pk);
    // A few long rows (the binned plans' shapes) with the plan's workspace at hand: the sketch is
    // interleaved into it first and a column's cells of all rows come with one gather.
    if (workspace && hp->kind == kConefPlanBinned && n <= 8 && x && cs && hp->workspace_bytes >= 32 * (int64_t)w) {
        const int rc = conef_launch_query_rows8_f32(x, cs, n, d, w, alpha, pk, (float*)workspace, (hipStream_t)stream);
        if (rc != CONEF_ERR_INVALID) return rc;
    }
    return conef_launch_query_table_f32(x, cs, n, d, w, alpha, a, b, pk, (hipStream_t)stream);
}

int conef_cs_query_planned_f16(float* x, const void* cs_half, const void* plan_host, const void* plan_dev, int64_t n,
                               int64_t d, int32_t w, float alpha, int32_t a, int32_t b, void* stream)
{
    const ConefPlanHeader* hp = (const ConefPlanHeader*)plan_host;
    if (!conef_plan_matches(hp, n, d, w, a, b) || !plan_dev || !plan_has_default_sign_seeds(hp, a, b)) return CONEF_ERR_INVALID;
    const uint32_t* pk = (const uint32_t*)((const char*)plan_dev + hp->off_pk);
    return conef_launch_query_table_f16(x, cs_half, n, d, w, alpha, a, b, pk, (hipStream_t)stream);
}

// 0 = binned (needs the workspace, fused step needs cs_out != cs_in), 1 = row lists, 2 = row lists in
// column panels (both: no workspace, in place allowed), -1 = not a plan.
int conef_plan_kind(const void* plan_host)
{
    const ConefPlanHeader* h = (const ConefPlanHeader*)plan_host;
    if (!h || h->magic != kConefPlanMagic) return -1;
    return (int)h->kind;
}

int conef_randblock_conef_step_planned_f32(float* x, const float* cs_in, float* cs_out, float* payload,
                                           const void* plan_host, const void* plan_dev, void* workspace, int64_t n,
                                           int64_t m, int32_t w, int64_t start, int64_t block, float alpha,
                                           float beta, int32_t a, int32_t b, void* stream)
{
    const ConefPlanHeader* hp = (const ConefPlanHeader*)plan_host;
    if (!conef_plan_matches(hp, n, m, w, a, b) || !plan_dev || !x || !cs_in || !cs_out || !payload)
        return CONEF_ERR_INVALID;
    int64_t numel = n * m;
    if (!(start >= 0 && start < numel && block >= 1 && block <= numel)) return CONEF_ERR_INVALID;
    ConefBlock blk = conef_make_block(numel, start, block);
    if (hp->kind == kConefPlanRowlist) {
        ConefListRandBlock front = {x, payload, blk, alpha};
        return conef_launch_rowlist(front, conef_rowlist_view(hp, plan_dev), cs_in, cs_out, n, m, w, beta,
                                    (hipStream_t)stream);
    }
    if (hp->kind == kConefPlanPanels) {
        ConefPanelRandBlock front = {x, payload, blk, alpha, aligned16(x) && m % 4 == 0};
        return conef_launch_panels(front, conef_panel_view(hp, plan_dev), cs_in, cs_out, n, m, w, beta, (hipStream_t)stream);
    }
    if (!workspace) return CONEF_ERR_INVALID;
    if (cs_in == cs_out) return CONEF_ERR_INVALID;   // the block is finished while buckets are being rewritten
    ConefSeeds hs = {a, b, a + 2, b + 3};
    ConefStageRandBlock stage = {x, m, blk};
    ConefBlockWork bw = {x, payload, numel, m, block, blk, conef_make_mod(w), hs, alpha};
    return conef_launch_binned(stage, hp, plan_dev, (float*)workspace, cs_in, cs_out, alpha, beta, aligned16(x), bw,
                               (hipStream_t)stream);
}

#ifdef CONEF_TRACE
// copies the phase timestamps of the last binned launch pair to host memory (2 * 1024 * 8 uint64)
int conef_trace_read(void* host_dst)
{
    return (int)hipMemcpyFromSymbol(host_dst, HIP_SYMBOL(conef_trace_buf), sizeof(conef_trace_buf));
}
#endif

}  // extern "C"
