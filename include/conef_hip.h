/*
 * conef_hip.h - C ABI of libconef_hip.so, the MI355X (gfx950) kernels behind the ConEF
 * gradient-compression hooks.
 *
 * This is the boundary the reference crosses in communication/compressors/cupy_kernel.py:36-45
 * (`func(grid, block, args, smem, stream=...)` with raw `tensor.data_ptr()` integers), widened to
 * the torch-op sequences of the hooks that are fused into single kernels here.  Conventions:
 *
 *   - every pointer is a DEVICE pointer into memory the caller owns and keeps alive until the
 *     stream has run the call (the one exception, conef_hash_table_host_i32, takes host memory);
 *   - `stream` is a hipStream_t (NULL = the default stream); every call is asynchronous on it,
 *     never synchronises the host, never allocates or frees device memory, keeps no global or
 *     thread-local state and may be called from any thread (the one exception is
 *     conef_topk_sparsify_noalloc_f32, which works in a per-GPU scratch array of the library);
 *   - scalars (alpha, beta, hash seeds) travel by value - the reference passes them as pointers
 *     to 1-element device tensors it allocates per call (CountSketch.py:144,167);
 *   - matrices are dense row-major fp32; a sketch is [n, w] row-major, fp32 unless the name says f16;
 *   - return value: 0 = enqueued, -1 = invalid argument, -2 = input larger than the entry point's
 *     stated maximum (nothing enqueued either way), > 0 = hipError_t.
 *   - empty inputs (n == 0 or d == 0) are accepted and do nothing.
 *
 * Floating point: multiplications and additions are done in the order the reference's kernels
 * write them, without contraction; only the order in which a sketch cell accumulates its terms is
 * not fixed (the reference uses float atomicAdd and does not fix it either).
 */
#ifndef CONEF_HIP_H
#define CONEF_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CONEF_OK 0
#define CONEF_ERR_INVALID (-1)
#define CONEF_ERR_TOO_LARGE (-2) /* an input exceeds the stated maximum of the entry point */

/* Library ABI version (1). */
int conef_version(void);

/* ---------------------------------------------------------------- hashing ---------------- */

/* bucket[i] = hash(i, w, a, b), sign[i] = (hash(i, w, sa, sb) & 1) ? +1 : -1 for i in [0, d).
 * Replaces: the `hash` device function and its two call sites, CountSketch.py:7-18,60-62.
 * Exists so that buckets and signs can be checked bit for bit against the reference arithmetic. */
int conef_hash_table_i32(int32_t* bucket, int32_t* sign, int64_t d, int32_t w, int32_t a, int32_t b,
                         int32_t sa, int32_t sb, void* stream);

/* Same table computed on the HOST by the host compilation of the same source (host pointers, no
 * stream): lets a machine without a GPU check the shipped hash, fast modulo included. */
int conef_hash_table_host_i32(int32_t* bucket, int32_t* sign, int64_t d, int32_t w, int32_t a, int32_t b,
                              int32_t sa, int32_t sb);

/* ------------------------------------------------------- one-hash count sketch ---------- */

/* x[r,i] += (sign_i * cs[r, bucket_i]) * alpha, x is [n,d], cs is [n,w].
 * Replaces: kernel dense_cs_query, CountSketch.py:70-98, launched from DenseCS.query :165-179. */
int conef_cs_query_f32(float* x, const float* cs, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                       int32_t b, void* stream);

/* cs_out[r,j] = cs_in[r,j] + sum_{i: bucket_i = j} fl32( sign_i*(vec[r,i] - (1.-beta)*sign_i*cs_in[r,j]) ),
 * the inner expression in double as in the reference.
 * Replaces: kernel dense_cs_update, CountSketch.py:27-67, launched from DenseCS.update :143-158.
 * cs_out may be the same buffer as cs_in only if conef_cs_update_inplace_ok(n,d,w) is 1 (a sketch
 * row then fits LDS and is snapshotted there, as the reference does in shared memory :47-52);
 * otherwise the snapshot is cs_in itself and cs_out must be a different buffer (-1 if not). */
int conef_cs_update_f32(const float* vec, const float* cs_in, float* cs_out, int64_t n, int64_t d, int32_t w,
                        float beta, int32_t a, int32_t b, void* stream);

/* 1 if an update (or fused step) of this shape may run in place, else 0.  Pure host function. */
int conef_cs_update_inplace_ok(int64_t n, int64_t d, int32_t w);

/* fp16-storage variants: cells are read as fp16, all arithmetic is fp32, cells are rounded to
 * nearest-even once when written.  Replaces: halfCountSketch.py:151-194, which casts the whole
 * sketch to fp32 before and back to fp16 after each kernel.  The update requires
 * conef_cs_update_inplace_ok(n,d,w) == 1 (larger sketches: convert, f32 update, convert back). */
int conef_cs_query_f16(float* x, const void* cs_half, int64_t n, int64_t d, int32_t w, float alpha, int32_t a,
                       int32_t b, void* stream);
int conef_cs_update_f16(const float* vec, const void* cs_in_half, void* cs_out_half, int64_t n, int64_t d,
                        int32_t w, float beta, int32_t a, int32_t b, void* stream);
int conef_convert_f16_to_f32(float* dst, const void* src_half, int64_t count, void* stream);
int conef_convert_f32_to_f16(void* dst_half, const float* src, int64_t count, void* stream);

/* x *= alpha.  Replaces: DenseCS.clean, CountSketch.py:181-182 / halfCountSketch.py:196-197. */
int conef_scale_f32(float* x, int64_t count, float alpha, void* stream);
int conef_scale_f16(void* x_half, int64_t count, float alpha, void* stream);

/* ----------------------------------------------------- three-hash count sketch ---------- */

/* x[r,i] += median_k( sign_k,i * cs_k[r, bucket_k,i] * alpha ), k = 0..2, fixed hash constants.
 * Replaces: CountSketchHash3.py:101-147 (query uses sign seed (a2+8, b2+7) for the third hash). */
int conef_cs3_query_f32(float* x, const float* cs0, const float* cs1, const float* cs2, int64_t n, int64_t d,
                        int32_t w, float alpha, void* stream);

/* Median-coupled update of the three sketches.  Replaces: CountSketchHash3.py:27-98 (update uses
 * sign seed (a2+8, b2+4) for the third hash).  out_k must differ from in_k. */
int conef_cs3_update_f32(const float* vec, const float* in0, const float* in1, const float* in2, float* out0,
                         float* out1, float* out2, int64_t n, int64_t d, int32_t w, float beta, void* stream);
/* First half of the same update without atomics: out_t[r,i] = median_k(-(1 - beta) * sign_k,i *
 * in_k[r, bucket_k,i]) + vec[r,i], the value all three sketches accumulate for element (r,i)
 * (CountSketchHash3.py:70-93).  The second half is conef_cs_update_planned_f32(out_t, cs_k, ...,
 * beta = 1) once per sketch, on plans built with that sketch's hash seeds
 * (conef_plan_build_host_seeded): same terms, same order as the serial definition. */
int conef_cs3_value_f32(const float* vec, const float* in0, const float* in1, const float* in2, float* out_t,
                        int64_t n, int64_t d, int32_t w, float beta, void* stream);

/* ------------------------------------------------ planned accumulation (no atomics) ---- */
/* The hash is a fixed function of (column, w, a, b), so where every column of an [n,d] tensor
 * goes is known before the first step.  A plan built once per sketch turns the update into
 * streaming passes without atomics that add every bucket's terms in ascending column order -
 * deterministic, and bit for bit the order of the reference's serial definition.  Three kinds
 * cover every shape the reference's kernel takes (any N, D: CountSketch.py:27-67,143-158):
 *   row lists  a row fits LDS (d <= 24576), any number of rows: one pass, per-bucket column
 *              lists, no workspace, cs_out may be cs_in;
 *   panels     longer rows of a matrix tall enough to fill the machine with row tiles (and
 *              w <= 65535): the same lists cut into column panels, the tile's cells resident in
 *              LDS while the panels go by; one pass, no workspace, cs_out may be cs_in;
 *   binned     long rows otherwise (a flat bucket viewed as a few long rows): two passes through
 *              a staging workspace of n*d floats, over groups of 8 rows.
 * No counterpart in the reference (its update is one atomicAdd per element, CountSketch.py:63). */

/* Bytes of a plan; 0 when no kind applies (more than 8 * 65535 long rows), -1 on invalid arguments.
 * chunk_cols / bin_buckets: 0 picks kind and tiling, a positive value asks for a binned plan with
 * that tiling (columns per staging workgroup, buckets per accumulating workgroup). */
int64_t conef_plan_bytes(int64_t n, int64_t d, int32_t w, int32_t chunk_cols, int32_t bin_buckets);
/* Builds the plan into HOST memory (plan_bytes >= conef_plan_bytes(...)).  The caller copies the
 * same bytes to the device and hands both copies to the *_planned entry points; the host copy
 * is only read for the launch geometry.  Host function, O(d). */
int conef_plan_build_host(void* plan_host, int64_t plan_bytes, int64_t n, int64_t d, int32_t w, int32_t a,
                          int32_t b, int32_t chunk_cols, int32_t bin_buckets);
/* The same for a sketch whose sign hash is seeded (sa, sb) rather than (a + 2, b + 3): the second
 * and third sketch of the three-hash compressor (CountSketchHash3.py:77,85). */
int conef_plan_build_host_seeded(void* plan_host, int64_t plan_bytes, int64_t n, int64_t d, int32_t w, int32_t a,
                                 int32_t b, int32_t sa, int32_t sb, int32_t chunk_cols, int32_t bin_buckets);
/* Bytes of device staging memory the planned entry points need (binned: n*d floats, rounded up;
 * row lists and panels: 0, the workspace argument may then be null). */
int64_t conef_plan_workspace_bytes(const void* plan_host);
/* 0 = binned, 1 = row lists, 2 = row lists in column panels, -1 = not a plan. */
int conef_plan_kind(const void* plan_host);

/* conef_cs_update_f32 on a plan.  cs_out may be the same buffer as cs_in.  Calls that share a
 * workspace must be ordered on one stream.  The f16 form (fp16-storage sketch, replaces
 * halfCountSketch.py:151-172) takes row-list plans, whole or in panels. */
int conef_cs_update_planned_f16(const float* vec, const void* cs_in_half, void* cs_out_half, const void* plan_host,
                                const void* plan_dev, int64_t n, int64_t d, int32_t w, float beta, int32_t a,
                                int32_t b, void* stream);
int conef_cs_update_planned_f32(const float* vec, const float* cs_in, float* cs_out, const void* plan_host,
                                const void* plan_dev, void* workspace, int64_t n, int64_t d, int32_t w, float beta,
                                int32_t a, int32_t b, void* stream);

/* ------------------------------------------------------------ random block ------------- */
/* The block is the wrap-around range [start, start+block) of the flat tensor: [start, end) with
 * end = min(start+block, numel), then [0, block-(end-start)).  0 <= start < numel, 1 <= block <= numel. */

/* One fused RandomBlock + count-sketch error-feedback step on one [n,m] gradient, in place:
 *   xq = x + alpha*unsketch(cs_in);  payload = xq[block];  x = xq on the block, 0 elsewhere;
 *   cs_out = update(cs_in, xq off the block / 0 on it, beta).
 * Replaces, for one tensor: DenseCS.query, clone, slice copies, zero_ calls, DenseCS.update,
 * tensor.zero_ and copies back of RandomBlock_hook.py:190,216-243,272-280 (world size 1).
 * Aliasing of cs_out/cs_in as for conef_cs_update_f32. */
int conef_randblock_conef_step_f32(float* x, const float* cs_in, float* cs_out, float* payload, int64_t n,
                                   int64_t m, int32_t w, int64_t start, int64_t block, float alpha, float beta,
                                   int32_t a, int32_t b, void* stream);

/* conef_cs_query_f32 / _f16 with every column's bucket and sign read from the plan's table instead of
 * hashed (a plan of either kind built for (n, d, w, a, b) with the default sign seeds): same values,
 * bit for bit.  workspace (f32 only): the plan's workspace (conef_plan_workspace_bytes) or null; with
 * it, a tensor of at most 8 long rows on a binned plan has its sketch interleaved into the workspace
 * first, so that a column's cells of all rows are one gather (the flat 25 MB bucket: 40 -> 17 us). */
int conef_cs_query_planned_f32(float* x, const float* cs, const void* plan_host, const void* plan_dev, void* workspace,
                               int64_t n, int64_t d, int32_t w, float alpha, int32_t a, int32_t b, void* stream);
int conef_cs_query_planned_f16(float* x, const void* cs_half, const void* plan_host, const void* plan_dev, int64_t n,
                               int64_t d, int32_t w, float alpha, int32_t a, int32_t b, void* stream);

/* conef_randblock_conef_step_f32 on a plan (see above).  With a binned plan cs_out must NOT be
 * cs_in (-1): the selected block is finished from the old sketch while the new one is being
 * written.  With a row-list plan it may. */
int conef_randblock_conef_step_planned_f32(float* x, const float* cs_in, float* cs_out, float* payload,
                                           const void* plan_host, const void* plan_dev, void* workspace, int64_t n,
                                           int64_t m, int32_t w, int64_t start, int64_t block, float alpha,
                                           float beta, int32_t a, int32_t b, void* stream);

/* Same step with a dense error tensor: xq = x + err; payload = xq[block]; x = xq on the block,
 * 0 elsewhere; err = 0 on the block, xq elsewhere.
 * Replaces: RandomBlock_hook.py:182-184,222,228,237,240,276-280. */
int conef_randblock_ef_step_f32(float* x, float* err, float* payload, int64_t numel, int64_t start,
                                int64_t block, void* stream);

/* Unbiased variant: payload = x[block] / prob; x = payload on the block, 0 elsewhere.
 * Replaces: UnbiasedRandomBlock_hook.py:155,161-167,200-204. */
int conef_randblock_unbiased_step_f32(float* x, float* payload, int64_t numel, int64_t start, int64_t block,
                                      float prob, void* stream);

/* The two halves a multi-rank caller puts around its all-reduce of the payload:
 * gather: payload[p] = x[(start+p) mod numel] / scale;  scatter: x = 0 except the block = payload.
 * Replace: RandomBlock_hook.py:222,237 and :276-280. */
int conef_randblock_gather_f32(const float* x, float* payload, int64_t numel, int64_t start, int64_t block,
                               float scale, void* stream);
int conef_randblock_scatter_f32(float* x, const float* payload, int64_t numel, int64_t start, int64_t block,
                                void* stream);

/* One tensor of a bucket for conef_randblock_step_batch_f32 (a HOST array of these is read before
 * the call returns; the pointers inside are device pointers unless the name says host). */
typedef struct ConefRandBlockItem {
    float* x;              /* [n,m] gradient, in place */
    float* err;            /* mode 1: dense error, n*m floats */
    const float* cs_in;    /* mode 2: sketch [n,w] read ... */
    float* cs_out;         /* ... and written (may equal cs_in except on a binned plan) */
    float* payload;        /* `block` floats */
    const void* plan_host; /* mode 2: the sketch's plan (host copy) or NULL for the unplanned kernels */
    const void* plan_dev;  /*         the same bytes on the device */
    void* staging;         /*         binned plans: conef_plan_workspace_bytes(plan_host) bytes */
    int64_t n, m;
    int64_t start, block;  /* the wrap-around block [start, start+block) of the flat tensor */
    int32_t w;             /* mode 2: sketch width */
    int32_t reserved;
} ConefRandBlockItem;

/* The fused step of every >= 2-D tensor of a bucket in one call.  mode 0: unbiased block
 * (conef_randblock_unbiased_step_f32 with prob = fl32(block / numel)); mode 1: dense error feedback
 * (conef_randblock_ef_step_f32); mode 2: count-sketched error (conef_randblock_conef_step[_planned]_f32).
 * Dense steps of all items share one launch, and so do sketched steps on row-list plans; results are
 * bit-identical to the single-tensor entry points.
 * Replaces the per-tensor loops RandomBlock_hook.py:215-245 and UnbiasedRandomBlock_hook.py:150-170
 * (and the query loop RandomBlock_hook.py:171-193) for a whole bucket. */
int conef_randblock_step_batch_f32(const ConefRandBlockItem* items, int32_t count, int32_t mode, float alpha,
                                   float beta, int32_t a, int32_t b, void* stream);

/* ------------------------------------------------------------------ PowerSGD ---------- */
/* M is [n,m], Q is [m,r], P is [n,r], 1 <= r <= 32. */

/* In-place Gram-Schmidt of a row-major [rows, r] matrix: column by column, col /= ||col|| (+ eps
 * if eps != 0), then every later column loses its projection on col.
 * Replaces: _orthogonalize, powerSGD_hook.py:12-44 (about 4r torch kernels per matrix).
 * Matrices spread over several workgroups exchange their sums through device memory inside one
 * cooperative launch; should a workgroup ever wait about a second for another, the kernel ends
 * and leaves NaN in the matrix instead of a half-orthogonalised one. */
int conef_gram_schmidt_f32(float* a, int64_t rows, int32_t r, float eps, void* workspace, int64_t workspace_bytes,
                           void* stream);

/* The same for `count` independent matrices in as few launches as their shapes allow (matrix k:
 * mats[k], [rows[k], ranks[k]]; host arrays, read before the call returns): the factors of all
 * tensors of a bucket are orthogonalised side by side, one workgroup each, instead of one after
 * the other.  Replaces: the `for p in ps: _orthogonalize(p)` loops, powerSGD_hook.py:475-477,527-528. */
int conef_gram_schmidt_batch_f32(float* const* mats, const int64_t* rows, const int32_t* ranks, int32_t count,
                                 float eps, void* workspace, int64_t workspace_bytes, void* stream);

/* Diagnostic, with no counterpart in the reference: *count = the number of Gram-Schmidt workgroups
 * on the current device that ran out their bounded wait for a neighbouring workgroup of the same
 * launch (about a second; they leave NaN in their rows) since the library was loaded.  The kernels
 * that spread one matrix over several workgroups assume those workgroups are resident together (at
 * most 128 of 256 threads); a count above zero says that assumption failed.  Unlike every other
 * entry point this one waits for the device (HOST pointer, no stream). */
int conef_gram_schmidt_give_ups(int64_t* count);

/* Bytes of device workspace conef_gram_schmidt_f32 (matrices too large for LDS), conef_psgd_mtp_f32
 * (sums across row slabs) and the conef_psgd_mq_* family (sums across column splits at rank >= 16)
 * may need for an [n,m] matrix at rank r.  The sums meet in a fixed order: no atomics, results do
 * not change from run to run.  The mq entry points also run without a workspace (null, 0): they
 * then keep every row tile's sum inside one workgroup. */
int64_t conef_psgd_workspace_bytes(int64_t n, int64_t m, int32_t r);

/* P = M Q.  Replaces: torch.matmul(tensor, q, out=p), powerSGD_hook.py:498. */
int conef_psgd_mq_f32(float* x, const float* q, float* p, int64_t n, int64_t m, int32_t r, void* workspace,
                      int64_t workspace_bytes, void* stream);
/* M += E (kept in M), then P = M Q.  Replaces: input_tensor.add_(error) :361 + :498 for one matrix
 * (also hPowerSGD_hook.py:399). */
int conef_psgd_mq_ef_f32(float* x, const float* err, const float* q, float* p, int64_t n, int64_t m, int32_t r,
                         void* workspace, int64_t workspace_bytes, void* stream);
/* M += alpha*unsketch(cs) (kept in M), then P = M Q.  Replaces: DenseCS.query :409 + :498. */
int conef_psgd_mq_conef_f32(float* x, const float* cs, const float* q, float* p, int64_t n, int64_t m,
                            int32_t r, int32_t w, float alpha, int32_t a, int32_t b, void* workspace,
                            int64_t workspace_bytes, void* stream);
/* The same with bucket and sign of every column read from a plan's table instead of hashed. */
int conef_psgd_mq_conef_planned_f32(float* x, const float* cs, const float* q, float* p, const void* plan_host,
                                    const void* plan_dev, int64_t n, int64_t m, int32_t r, int32_t w, float alpha,
                                    int32_t a, int32_t b, void* workspace, int64_t workspace_bytes, void* stream);

/* Q = M^T P.  Replaces: torch.matmul(tensor.t(), p, out=q), powerSGD_hook.py:532. */
int conef_psgd_mtp_f32(const float* x, const float* p, float* q, int64_t n, int64_t m, int32_t r, void* workspace,
                       int64_t workspace_bytes, void* stream);

/* M = P Q^T.  Replaces: torch.matmul(p, q.t(), out=tensor), powerSGD_hook.py:551. */
int conef_psgd_pqt_f32(float* x, const float* p, const float* q, int64_t n, int64_t m, int32_t r, void* stream);
/* E = M - P Q^T, then M = P Q^T.  Replaces: clone :375 + :551 + `input_tensor_cp - input_tensor` :558
 * for one matrix (also hPowerSGD_hook.py:553). */
int conef_psgd_pqt_ef_f32(float* x, float* err, const float* p, const float* q, int64_t n, int64_t m, int32_t r,
                          void* stream);
/* cs_out = update(cs_in, M - P Q^T, beta), then M = P Q^T.  Replaces: clone :410 + :551 +
 * cp_tensor.add_(-1, tensor) :563 + DenseCS.update :564.  Aliasing as for conef_cs_update_f32. */
int conef_psgd_pqt_conef_f32(float* x, const float* p, const float* q, const float* cs_in, float* cs_out,
                             int64_t n, int64_t m, int32_t r, int32_t w, float beta, int32_t a, int32_t b,
                             void* stream);
/* The same on a row-list plan: no atomics, the oracle's accumulation order, cs_out may be cs_in. */
int conef_psgd_pqt_conef_planned_f32(float* x, const float* p, const float* q, const float* cs_in, float* cs_out,
                                     const void* plan_host, const void* plan_dev, int64_t n, int64_t m, int32_t r,
                                     int32_t w, float beta, int32_t a, int32_t b, void* stream);

/* ---- all matrices of a bucket per launch -------------------------------------------------- */
/* The tensors of a gradient bucket are independent of each other and most are too small to fill
 * the GPU alone, so the three products also come as batch calls: one table entry per matrix
 * (host array, read before the call returns), matrices of one kernel class share launches of up
 * to 24, a workgroup finds its matrix from the table.  Results are those of the per-matrix calls.
 * Replaces: the `for tensor, q, p in zip(...)` loops, powerSGD_hook.py:497-498,530-532,550-551,
 * 561-564. */
typedef struct ConefPsgdItem {
    float* x;               /* the matrix [n,m], inside the bucket */
    float* err;             /* dense error / residual [n,m], or NULL */
    float* cs;              /* sketch [n,w] (updated in place by pqt mode 2), or NULL */
    const void* plan_host;  /* row-list plan of the sketch (host and device copy), or NULL */
    const void* plan_dev;
    float* p;               /* [n,r] */
    float* q;               /* [m,r] */
    int64_t n, m;
    int32_t r, w;
} ConefPsgdItem;

/* Bytes of workspace conef_psgd_mtp_batch_f32 needs for these items (sums across row slabs). */
int64_t conef_psgd_batch_workspace_bytes(const ConefPsgdItem* items, int32_t count);
/* mode 0: P = M Q.  mode 1: M += err first.  mode 2: M += alpha*unsketch(cs) first (bucket and
 * sign from the plan's table when a plan is given).  Per item as conef_psgd_mq_f32 / _ef_ / _conef_. */
int conef_psgd_mq_batch_f32(const ConefPsgdItem* items, int32_t count, int32_t mode, float alpha, int32_t a, int32_t b,
                            void* workspace, int64_t workspace_bytes, void* stream);
/* Q = M^T P for every item. */
int conef_psgd_mtp_batch_f32(const ConefPsgdItem* items, int32_t count, void* workspace, int64_t workspace_bytes,
                             void* stream);
/* mode 0: M = P Q^T.  mode 1: err = M - P Q^T as well.  mode 2: cs = update(cs, M - P Q^T, beta) in
 * place on the item's row-list plan (every item needs one) as well. */
int conef_psgd_pqt_batch_f32(const ConefPsgdItem* items, int32_t count, int32_t mode, float beta, int32_t a, int32_t b,
                             void* stream);

/* cs = update(cs, err, beta) in place for every item, err the item's dense [n,m] residual
 * (DenseCS.update, compressors/CountSketch.py:27-48, once per matrix in the reference's hook,
 * powerSGD_hook.py:564): the sketches of a bucket in one launch.  Every item needs a row-list
 * plan for (n, m, w, a, b). */
int conef_psgd_sketch_update_batch_f32(const ConefPsgdItem* items, int32_t count, float beta, int32_t a, int32_t b,
                                       void* stream);

/* One PowerSGD round over the matrices of a bucket in a single call: Gram-Schmidt of every Q,
 * conef_psgd_mq_batch_f32 (mq_mode), Gram-Schmidt of every P, conef_psgd_mtp_batch_f32,
 * conef_psgd_pqt_batch_f32 (pqt_mode 0..2; 3 = mode 1, then conef_psgd_sketch_update_batch_f32 on the
 * residuals it wrote to err).  Replaces powerSGD_hook.py:473-564 at world size 1 (the all-reduces in
 * between are the identity there).  Same launches as the separate calls, in the same order. */
int conef_psgd_round_f32(const ConefPsgdItem* items, int32_t count, int32_t mq_mode, int32_t pqt_mode, float alpha,
                         float beta, float eps, int32_t a, int32_t b, void* workspace, int64_t workspace_bytes,
                         void* stream);

/* The same round in ONE launch for a bucket of small matrices (a few thousand elements each, where a
 * round of separate launches is nothing but launch latency): a workgroup
 * per matrix keeps the matrix, both factors and the sketch's bucket lists in LDS and takes it through
 * the reference's steps in the reference's order - orthogonalise Q, X = M + error, P = X Q,
 * orthogonalise P, Q = X^T P, M = P Q^T, residual to the dense error or into the sketch (a bucket's
 * terms in ascending column order).  Replaces powerSGD_hook.py:473-564 at world size 1.
 * A matrix of more than 10240 elements is dealt out by rows over up to 16 workgroups, which meet
 * twice (the rows of the raw P, the shares of X^T P added in a fixed order) through 8-byte records
 * {launch tag, value} in `workspace` (conef_psgd_round_small_workspace_bytes of it, 8-byte aligned;
 * nothing to clear, contents are scratch): one workgroup does all the work for its rows on one CU,
 * and beyond that size more CUs are worth two exchanges.  The waits are bounded; a workgroup whose
 * peers never publish leaves NaN in its rows of M and counts in conef_gram_schmidt_give_ups.
 * mq_mode / pqt_mode as above (0, 1, or both 2).  conef_psgd_round_small_fits says (1 / 0) whether
 * a bucket qualifies: at most 24 matrices of at most 73728 elements each, 128 workgroups in all,
 * every workgroup's rows fit LDS with the factors and the sketch's bucket lists, ranks up to 8, a
 * row-list plan per sketch in mode 2; the round returns CONEF_ERR_INVALID for a bucket that does
 * not.  conef_psgd_batch_workspace_bytes covers what this round needs. */
int conef_psgd_round_small_fits(const ConefPsgdItem* items, int32_t count, int32_t mq_mode, int32_t pqt_mode, int32_t a,
                                int32_t b);
int64_t conef_psgd_round_small_workspace_bytes(const ConefPsgdItem* items, int32_t count);
int conef_psgd_round_small_f32(const ConefPsgdItem* items, int32_t count, int32_t mq_mode, int32_t pqt_mode, float alpha,
                               float beta, float eps, int32_t a, int32_t b, void* workspace, int64_t workspace_bytes,
                               void* stream);

/* The middle of that round as a call of its own, for a caller that splits the round (the hooks above
 * rank 8 do, to orthogonalise the new Q on a side stream meanwhile): P = X Q with the Q factors of
 * `first` (a copy of `items` whose q may point elsewhere; null: items' own), P orthogonalised
 * (powerSGD_hook.py:516-531), Q = X^T P into items[k].q.  Deferred orthogonalisation of P where the
 * batch allows, as in conef_psgd_round_f32 (ranks 1, 2, 4, 8, 16, 32 of 16-byte shaped matrices). */
int conef_psgd_products_f32(const ConefPsgdItem* items, const ConefPsgdItem* first, int32_t count, int32_t mq_mode,
                            float alpha, float eps, int32_t a, int32_t b, void* workspace, int64_t workspace_bytes,
                            void* stream);

/* The same round for callers that keep a second buffer per Q factor (q_next[k], [m,r] like items[k].q).
 * The reference orthogonalises a bucket's Q factors at the start of the bucket's next round
 * (powerSGD_hook.py:496-497), a launch of a few workgroups with the machine idle around it.  Here
 * flags & CONEF_ROUND_MAKE_NEXT asks for that to be done at the end of this round instead, out of
 * place into q_next, by workgroups that ride along in the round's last launch; *made tells whether it
 * was (only for pqt_mode 0..2 over a bucket of at most 24 matrices of one rank <= 8 whose Q factors have
 * at most 1024 rows).  items[k].q keeps what the reference keeps there.  In the next round
 * flags & CONEF_ROUND_Q_READY says q_next holds the orthogonal Q factors: the first step is left out
 * and P = M Q reads them.  Same arithmetic on the same values either way.  No counterpart in the
 * reference's interface. */
#define CONEF_ROUND_Q_READY 1
#define CONEF_ROUND_MAKE_NEXT 2
int conef_psgd_round_ahead_f32(const ConefPsgdItem* items, int32_t count, int32_t mq_mode, int32_t pqt_mode, float alpha,
                               float beta, float eps, int32_t a, int32_t b, float* const* q_next, int32_t flags,
                               int32_t* made, void* workspace, int64_t workspace_bytes, void* stream);

/* Dense error feedback on a stretch of the bucket that is not compressed: x += err; err = 0
 * (the copy-minus-result of powerSGD_hook.py:558 is exactly zero there). */
int conef_ef_passthrough_f32(float* x, float* err, int64_t count, void* stream);

/* ------------------------------------------------------------- magnitude top-k ---------- */

/* Bytes of device workspace conef_topk_sparsify_f32 needs for `numel` elements (host function). */
int64_t conef_topk_workspace_bytes(int64_t numel);

/* Keeps the k entries of largest magnitude of x[0..numel) and zeroes the rest, in place; ties on
 * the threshold magnitude keep the lowest indices.  k >= numel keeps everything.
 * Replaces: _topk, hPowerSGD_hook.py:90-97 (torch.topk on |x|, zero_, scatter back). */
int conef_topk_sparsify_f32(float* x, int64_t numel, int64_t k, void* workspace, int64_t workspace_bytes,
                            void* stream);

/* The same for `count` tensors with every pass one launch over all of them: tensor i is xs[i] with
 * numels[i] elements and keeps ks[i].  Replaces the `_topk(...)` call inside the per-tensor loop of
 * hpowerSGD_hook (hPowerSGD_hook.py:554) for all matrices of a bucket at once.  xs / numels / ks
 * are host arrays, read before the call returns; the workspace (16-byte aligned) holds
 * conef_topk_batch_workspace_bytes(numels, count) bytes. */
int64_t conef_topk_batch_workspace_bytes(const int64_t* numels, int32_t count);
int conef_topk_sparsify_batch_f32(float* const* xs, const int64_t* numels, const int64_t* ks, int32_t count,
                                  void* workspace, int64_t workspace_bytes, void* stream);
/* The same call (hPowerSGD_hook.py:554, every matrix of a bucket) for a workspace that stays with
 * its tensors from step to step: the caller zero-fills it once, before its first use, and passes
 * it to nothing but this entry point, with the same xs / numels / count, afterwards.  The passes
 * then clear the selection state behind themselves and the launch that clears it is left out (four
 * launches a call instead of five).  Same results, bit for bit. */
int conef_topk_sparsify_batch_kept_f32(float* const* xs, const int64_t* numels, const int64_t* ks, int32_t count,
                                       void* workspace, int64_t workspace_bytes, void* stream);

/* conef_topk_sparsify_f32 without a workspace argument and without any allocation.  No counterpart
 * in the reference: it is for callers that cannot allocate device memory - code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The selection state (29 184
 * bytes) lives in a per-GPU scratch array inside the library, which every GPU the library runs on
 * holds until the process ends.  The device `stream` belongs to must be the current device.
 * numel > CONEF_TOPK_NOALLOC_MAX_NUMEL returns CONEF_ERR_TOO_LARGE (nothing enqueued).  All calls on
 * one GPU share the scratch: back-to-back calls on one stream are safe (a call first resets it),
 * calls that can overlap on one GPU (other streams, other threads) race. */
#define CONEF_TOPK_NOALLOC_MAX_NUMEL 0xffffffffLL
int conef_topk_sparsify_noalloc_f32(float* x, int64_t numel, int64_t k, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CONEF_HIP_H */
