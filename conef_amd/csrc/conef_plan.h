// Binned ("planned") sketch accumulation for long rows: a count-sketch update without atomics.
//
// When a sketch row does not fit LDS (a flat 25 MB bucket viewed [5, 1.3M] has W = 130k), the
// scatter-add cs[r, bucket(i)] += term(r, i) has no locality: consecutive columns hash to
// unrelated buckets.  Float atomics on global memory run at about 2e10 per second on this part,
// thirty times too slow.  But the hash is a fixed function of (column, W, seeds), so where every
// column goes is known before the first step.  A plan, built once per sketch, turns the scatter
// into two streaming passes:
//
//   pass A (column order)  a workgroup takes a chunk of C consecutive columns (all n rows),
//          permutes the n-float records inside LDS so that records of the same bin (a range of
//          T buckets) are adjacent, and writes the chunk image out linearly.  Whatever has to
//          happen in column order (payload extraction, writing the decompressed gradient) is
//          fused here.
//   pass B (bucket order)  a workgroup owns one bin; it collects the bin's segment from every
//          chunk image into LDS (in chunk order, which is ascending column order) and one
//          thread per bucket adds that bucket's terms in ascending column order, for all rows.
//
// The result is deterministic and reproduces the CPU oracle's accumulation order bit for bit.
// Cost: one extra write and one extra read of the tensor (the staging buffer), all coalesced.
#pragma once
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "conef_device.h"
#include "conef_sketch_core.h"
#include "conef_rowlist.h"
#include "conef_panels.h"

constexpr uint32_t kConefPlanMagic = 0x50464E43u;   // "CNFP"
constexpr int kConefPlanMaxRows = 8;
// Three kinds of plan share the header.  Row lists (conef_rowlist.h): a row fits LDS, any number of
// rows, tables csr / ent (column | sign << 15) / pk only, no staging buffer.  Row lists in column
// panels (conef_panels.h): rows too long for that on a matrix with rows enough to fill the machine,
// tables epos / entg / colb / pk, no staging buffer.  Binned (this file): a few long rows, in groups of up to 8.
constexpr int64_t kConefPlanBinned = 0;
constexpr int64_t kConefPlanRowlist = 1;
constexpr int64_t kConefPlanPanels = 2;
// Tall matrices go to the panels (one pass over the tensor); with fewer row tiles than this the
// binned passes, which split the columns over the machine, are the better fit.
constexpr int64_t kConefPanelMinTiles = 256;

struct ConefPlanHeader {
    uint32_t magic;
    uint32_t version;
    int64_t n, d;
    int32_t w, a, b;
    int32_t chunk_cols;        // C: columns per pass-A workgroup
    int32_t nchunks;
    int32_t bin_buckets;       // T: buckets per pass-B workgroup
    int32_t nbins;
    int32_t max_bin_records;   // largest number of columns that map into one bin
    int64_t off_pos;           // uint16[d]: record position of column i inside its chunk image
                               // (panels: `entg`; their `epos` sits at off_ent, their `colb` at off_csr)
    int64_t off_seg;           // uint32[nbins][nchunks+1]: (start inside chunk image) | (offset inside bin image << 16);
                               // entry [nchunks] holds the bin's record count in the high half
    int64_t off_csr;           // uint32[w+1]: first entry of bucket j
    int64_t off_ent;           // uint16[d]: (slot inside bin image) | (sign bit << 15), buckets ascending, columns ascending
    int64_t off_pk;            // uint32[d]: bucket | (sign bit << 31) of every column, for the column-order work
    int64_t total_bytes;
    int64_t workspace_bytes;   // staging buffer: n * d floats, rounded up (binned plans only)
    int64_t kind;              // kConefPlanBinned, kConefPlanRowlist or kConefPlanPanels
    int64_t seeds;             // sign-hash seeds the tables were built with, sa << 32 | sb
    int64_t off_order;         // row lists: uint16[w], the buckets by falling list length (ties: by index)
};

inline int64_t conef_align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

// Shape decisions that do not depend on the hash values.  Tile hints ask for a binned plan.
inline bool conef_plan_shape(int64_t n, int64_t d, int32_t w, int32_t hint_chunk, int32_t hint_bin,
                             ConefPlanHeader* h)
{
    if (n < 1 || d < 1 || d > 0x7fffffffLL || w < 1 || w > (1 << 30)) return false;
    ConefRowlistShape rl;
    if (hint_chunk <= 0 && hint_bin <= 0 && conef_rowlist_shape(n, d, w, true, &rl)) {
        memset(h, 0, sizeof(*h));
        h->magic = kConefPlanMagic;
        h->version = 1;
        h->kind = kConefPlanRowlist;
        h->n = n;
        h->d = d;
        h->w = w;
        int64_t off = conef_align256(sizeof(ConefPlanHeader));
        h->off_csr = off;
        off += conef_align256(4 * ((int64_t)w + 1));
        h->off_ent = off;
        off += conef_align256(2 * d);
        h->off_pk = off;
        off += conef_align256(4 * d);
        h->off_order = off;
        off += conef_align256(2 * (int64_t)w);
        h->total_bytes = off;
        h->workspace_bytes = 0;
        return true;
    }
    ConefPanelShape pl;
    const bool panels_fit = hint_chunk <= 0 && hint_bin <= 0 && conef_panel_shape(n, d, w, &pl);
    if (panels_fit && pl.tiles >= kConefPanelMinTiles) {
        memset(h, 0, sizeof(*h));
        h->magic = kConefPlanMagic;
        h->version = 1;
        h->kind = kConefPlanPanels;
        h->n = n;
        h->d = d;
        h->w = w;
        h->chunk_cols = pl.pc;
        h->nchunks = (int32_t)((d + pl.pc - 1) / pl.pc);
        int64_t off = conef_align256(sizeof(ConefPlanHeader));
        h->off_ent = off;                       // epos: uint16[d] by column, entry of its panel | sign << 15
        off += conef_align256(2 * d + 16);
        h->off_pos = off;                       // entg: uint32[d] by panel and entry, bucket | group length << 16
        off += conef_align256(4 * d + 16);
        h->off_csr = off;                       // colb: uint16[d] by column, the column's bucket
        off += conef_align256(2 * d + 16);
        h->off_pk = off;
        off += conef_align256(4 * d + 16);
        h->total_bytes = off;
        h->workspace_bytes = 0;
        return true;
    }
    if (n / kConefPlanMaxRows > 65535) return false;     // the row groups are a grid dimension
    memset(h, 0, sizeof(*h));
    // long rows in groups of up to 8: the tiles are those of a full group
    const int64_t ng = n < kConefPlanMaxRows ? n : kConefPlanMaxRows;
    int64_t c = hint_chunk > 0 ? hint_chunk : (100 * 1024) / (4 * ng);   // a 100 KB chunk image: one workgroup per CU
    if (c > 16384) c = 16384;
    c = c / 1024 * 1024;
    if (c < 1024) c = 1024;
    int64_t t;
    if (hint_bin > 0) {
        t = hint_bin;
    } else {
        // aim at a bin image of about 52 KB (two workgroups per CU): records = 52K / (4n),
        // buckets = records * w / d
        double records = 52.0 * 1024 / (4.0 * ng);
        t = (int64_t)(records * (double)w / (double)d);
        if (t >= 64) t = t / 64 * 64;      // narrow sketches: fewer buckets than lanes per bin rather than an image that overflows LDS
    }
    if (t < 1) t = 1;
    if (t > 768) t = 768;      // leaves room in a 1024-thread workgroup for the waves that do column work
    h->magic = kConefPlanMagic;
    h->version = 1;
    h->kind = kConefPlanBinned;
    h->n = n;
    h->d = d;
    h->w = w;
    h->chunk_cols = (int32_t)c;
    h->nchunks = (int32_t)((d + c - 1) / c);
    h->bin_buckets = (int32_t)t;
    h->nbins = (int32_t)((w + t - 1) / t);
    int64_t off = conef_align256(sizeof(ConefPlanHeader));
    h->off_pos = off;
    off += conef_align256(2 * d);
    h->off_seg = off;
    off += conef_align256(4 * (int64_t)h->nbins * (h->nchunks + 1));
    h->off_csr = off;
    off += conef_align256(4 * ((int64_t)w + 1));
    h->off_ent = off;
    off += conef_align256(2 * d);
    h->off_pk = off;
    off += conef_align256(4 * d);
    h->total_bytes = off;
    h->workspace_bytes = conef_align256(4 * n * d);
    return true;
}

// Fills a host buffer of header.total_bytes with the plan.  Returns false when a bin would hold
// more records than a slot index can name.
inline bool conef_plan_fill(void* buf, const ConefPlanHeader& shape, int32_t a, int32_t b, int32_t sa, int32_t sb)
{
    ConefPlanHeader h = shape;
    h.a = a;
    h.b = b;
    h.seeds = ((int64_t)(uint32_t)sa << 32) | (uint32_t)sb;
    const int64_t d = h.d;
    if (h.kind == kConefPlanRowlist) {
        char* rbase = (char*)buf;
        uint32_t* rcsr = (uint32_t*)(rbase + h.off_csr);
        uint16_t* rent = (uint16_t*)(rbase + h.off_ent);
        uint32_t* rpk = (uint32_t*)(rbase + h.off_pk);
        ConefMod rmod = conef_make_mod(h.w);
        std::vector<uint32_t> count((size_t)h.w + 1, 0);
        for (int64_t i = 0; i < d; ++i) {
            rpk[i] = conef_bucket_sign((int32_t)i, rmod, a, b, sa, sb);
            count[(rpk[i] & 0x7fffffffu) + 1]++;
        }
        rcsr[0] = 0;
        for (int32_t j = 0; j < h.w; ++j) rcsr[j + 1] = rcsr[j] + count[(size_t)j + 1];
        std::vector<uint32_t> cur(rcsr, rcsr + h.w);
        for (int64_t i = 0; i < d; ++i)       // ascending columns inside every bucket
            rent[cur[rpk[i] & 0x7fffffffu]++] = (uint16_t)((uint32_t)i | ((rpk[i] >> 31) << 15));
        // The walk gives neighbouring lanes neighbouring entries of this order, so that the lanes of
        // a wave walk lists of about the same length.
        uint16_t* rord = (uint16_t*)(rbase + h.off_order);
        std::vector<uint32_t> by_len((size_t)h.w);
        for (int32_t j = 0; j < h.w; ++j) by_len[(size_t)j] = (uint32_t)j;
        std::stable_sort(by_len.begin(), by_len.end(), [&](uint32_t x, uint32_t y) {
            return rcsr[x + 1] - rcsr[x] > rcsr[y + 1] - rcsr[y];
        });
        for (int32_t j = 0; j < h.w; ++j) rord[j] = (uint16_t)by_len[(size_t)j];
        memcpy(rbase, &h, sizeof(h));
        return true;
    }
    if (h.kind == kConefPlanPanels) {
        char* pbase = (char*)buf;
        memset(pbase, 0, (size_t)h.total_bytes);
        uint16_t* pepos = (uint16_t*)(pbase + h.off_ent);
        uint32_t* pentg = (uint32_t*)(pbase + h.off_pos);
        uint16_t* pcolb = (uint16_t*)(pbase + h.off_csr);
        uint32_t* ppk = (uint32_t*)(pbase + h.off_pk);
        ConefMod pmod = conef_make_mod(h.w);
        for (int64_t i = 0; i < d; ++i) ppk[i] = conef_bucket_sign((int32_t)i, pmod, a, b, sa, sb);
        const int64_t pc = h.chunk_cols;
        std::vector<uint32_t> first((size_t)h.w + 1);
        for (int64_t c0 = 0; c0 < d; c0 += pc) {
            const int64_t c1 = c0 + pc < d ? c0 + pc : d;
            std::fill(first.begin(), first.end(), 0u);
            for (int64_t i = c0; i < c1; ++i) first[(ppk[i] & 0x7fffffffu) + 1]++;
            for (int32_t j = 0; j < h.w; ++j) first[(size_t)j + 1] += first[(size_t)j];
            for (int64_t i = c0; i < c1; ++i) {        // ascending columns inside every bucket
                const uint32_t j = ppk[i] & 0x7fffffffu;
                const uint32_t k = first[j]++;
                pepos[i] = (uint16_t)(k | ((ppk[i] >> 31) << 15));
                pcolb[i] = (uint16_t)j;
                pentg[c0 + k] = j;
            }
            for (int64_t k = c1 - c0 - 1, run = 0; k >= 0; --k) {        // the first entry of a group carries its length
                ++run;
                if (k == 0 || pentg[c0 + k - 1] != pentg[c0 + k]) {
                    pentg[c0 + k] |= (uint32_t)run << 16;
                    run = 0;
                }
            }
        }
        memcpy(pbase, &h, sizeof(h));
        return true;
    }
    const int32_t w = h.w, C = h.chunk_cols, T = h.bin_buckets, nbins = h.nbins, nchunks = h.nchunks;
    char* base = (char*)buf;
    uint16_t* pos = (uint16_t*)(base + h.off_pos);
    uint32_t* seg = (uint32_t*)(base + h.off_seg);
    uint32_t* csr = (uint32_t*)(base + h.off_csr);
    uint16_t* ent = (uint16_t*)(base + h.off_ent);
    ConefMod mod = conef_make_mod(w);
    uint32_t* packed = (uint32_t*)(base + h.off_pk);
    for (int64_t i = 0; i < d; ++i) packed[(size_t)i] = conef_bucket_sign((int32_t)i, mod, a, b, sa, sb);

    // pass-A side: inside every chunk, records grouped by bin (stable in column order)
    std::vector<uint32_t> bin_fill((size_t)nbins, 0);          // records of each bin so far (earlier chunks)
    std::vector<uint32_t> cnt((size_t)nbins), start((size_t)nbins);
    std::vector<uint32_t> slot((size_t)d);                     // slot of column i inside its bin image
    for (int32_t c = 0; c < nchunks; ++c) {
        int64_t c0 = (int64_t)c * C, c1 = c0 + C < d ? c0 + C : d;
        std::fill(cnt.begin(), cnt.end(), 0u);
        for (int64_t i = c0; i < c1; ++i) cnt[(packed[(size_t)i] & 0x7fffffffu) / (uint32_t)T]++;
        uint32_t run = 0;
        for (int32_t bn = 0; bn < nbins; ++bn) {
            start[(size_t)bn] = run;
            if (bin_fill[(size_t)bn] > 0x7fff) return false;    // a slot index has 15 bits
            seg[(size_t)bn * (nchunks + 1) + c] = run | (bin_fill[(size_t)bn] << 16);
            run += cnt[(size_t)bn];
        }
        std::fill(cnt.begin(), cnt.end(), 0u);
        for (int64_t i = c0; i < c1; ++i) {
            uint32_t bn = (packed[(size_t)i] & 0x7fffffffu) / (uint32_t)T;
            uint32_t k = cnt[bn]++;
            pos[i] = (uint16_t)(start[bn] + k);
            slot[(size_t)i] = bin_fill[bn] + k;
        }
        for (int32_t bn = 0; bn < nbins; ++bn) bin_fill[(size_t)bn] += cnt[(size_t)bn];
    }
    uint32_t max_rec = 0;
    for (int32_t bn = 0; bn < nbins; ++bn) {
        if (bin_fill[(size_t)bn] > 0x7fff) return false;
        seg[(size_t)bn * (nchunks + 1) + nchunks] = bin_fill[(size_t)bn] << 16;
        if (bin_fill[(size_t)bn] > max_rec) max_rec = bin_fill[(size_t)bn];
    }
    h.max_bin_records = (int32_t)max_rec;

    // pass-B side: per bucket, its columns in ascending order
    std::vector<uint32_t> bcount((size_t)w + 1, 0);
    for (int64_t i = 0; i < d; ++i) bcount[(packed[(size_t)i] & 0x7fffffffu) + 1]++;
    csr[0] = 0;
    for (int32_t j = 0; j < w; ++j) csr[j + 1] = csr[j] + bcount[(size_t)j + 1];
    std::vector<uint32_t> cursor(csr, csr + w);
    for (int64_t i = 0; i < d; ++i) {
        uint32_t p = packed[(size_t)i];
        uint32_t j = p & 0x7fffffffu;
        ent[cursor[j]++] = (uint16_t)(slot[(size_t)i] | ((p >> 31) << 15));
    }
    memcpy(base, &h, sizeof(h));
    return true;
}

// Device-side view handed to the kernels.
struct ConefPlanView {
    const uint16_t* pos;
    const uint32_t* seg;
    const uint32_t* csr;
    const uint16_t* ent;
    const uint32_t* pk;
    int32_t chunk_cols, nchunks, bin_buckets, nbins;
    int32_t flags;   // bit 0: XCD-major work mapping, bit 1: streaming (nontemporal) stores
};

// XCD-major work mapping and streaming stores for the zero fill: both measured faster on the
// 25 MB bucket; streaming stores for the staging image (bit 2) measured slower.
inline int32_t conef_plan_flags() { return 3; }

inline ConefRowlistView conef_rowlist_view(const ConefPlanHeader* host, const void* dev)
{
    const char* b = (const char*)dev;
    ConefRowlistView v = {(const uint32_t*)(b + host->off_csr), (const uint16_t*)(b + host->off_ent),
                          (const uint32_t*)(b + host->off_pk), (const uint16_t*)(b + host->off_order)};
    return v;
}

inline ConefPanelView conef_panel_view(const ConefPlanHeader* host, const void* dev)
{
    const char* b = (const char*)dev;
    ConefPanelView v = {(const uint32_t*)(b + host->off_pos), (const uint16_t*)(b + host->off_ent),
                        (const uint16_t*)(b + host->off_csr), host->chunk_cols};
    return v;
}

inline ConefPlanView conef_plan_view(const ConefPlanHeader* host, const void* dev)
{
    const char* b = (const char*)dev;
    ConefPlanView v;
    v.pos = (const uint16_t*)(b + host->off_pos);
    v.seg = (const uint32_t*)(b + host->off_seg);
    v.csr = (const uint32_t*)(b + host->off_csr);
    v.ent = (const uint16_t*)(b + host->off_ent);
    v.pk = (const uint32_t*)(b + host->off_pk);
    v.chunk_cols = host->chunk_cols;
    v.nchunks = host->nchunks;
    v.bin_buckets = host->bin_buckets;
    v.nbins = host->nbins;
    v.flags = conef_plan_flags();
    return v;
}

// Workgroups are handed to the 8 XCDs round robin.  Mapping workgroup -> work item so that an XCD
// gets a contiguous run of items keeps neighbouring chunk images / bin segments in one L2.
__device__ __forceinline__ int conef_xcd_major(int bid, int nblocks_padded, int flags = 1)
{
    if (!(flags & 1)) return bid;
    int per = nblocks_padded >> 3;
    return (bid & 7) * per + (bid >> 3);
}

typedef float conef_v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void conef_store4(float* p, float a, float b, float c, float d, bool streaming)
{
    conef_v4f v = {a, b, c, d};
    if (streaming) __builtin_nontemporal_store(v, reinterpret_cast<conef_v4f*>(p));
    else *reinterpret_cast<conef_v4f*>(p) = v;
}

// -------------------------------------------------------------- stage fronts ----
// A stage front supplies the values pass B will accumulate and does the column-order side effects
// of the fused step.  The kernels are written so that every global load of a thread is issued
// before the first value is used: no load sits inside a data-dependent branch (addresses are
// clamped instead), because a conditional load makes the compiler wait for it on the spot.

// plain update: the values are the dense tensor itself
struct ConefStageVec {
    const float* vec;
    int64_t d;
    static constexpr bool kFusedQuery = false;
    __device__ __forceinline__ void load4(int r, int64_t c0, float* s) const
    {
        float4 t = *reinterpret_cast<const float4*>(vec + (int64_t)r * d + c0);
        s[0] = t.x; s[1] = t.y; s[2] = t.z; s[3] = t.w;
    }
    __device__ __forceinline__ float element(int r, int64_t col) const { return vec[(int64_t)r * d + col]; }
};

// A staged value with this bit pattern (a NaN no arithmetic produces) tells pass B "this element
// was selected for the payload: sketch a zero for it".
constexpr uint32_t kConefSelectedBits = 0xffffffffu;

// RandomBlock + ConEF.  The staging pass only moves data: elements outside the block are staged
// raw (pass B adds the unsketched error itself, it has the sketch cell in a register), elements
// inside the block are staged as the marker above.  x is not written at all here: pass B, which
// otherwise writes next to nothing, zeroes the elements outside the block and finishes the ones
// inside it (gather the cell, xq = x + term, payload and x receive xq).
struct ConefStageRandBlock {
    const float* x;
    int64_t d;
    ConefBlock blk;
    static constexpr bool kFusedQuery = true;
    __device__ __forceinline__ void load4(int r, int64_t c0, float* s) const
    {
        float4 t = *reinterpret_cast<const float4*>(x + (int64_t)r * d + c0);
        int64_t f = (int64_t)r * d + c0;
        s[0] = t.x; s[1] = t.y; s[2] = t.z; s[3] = t.w;
        // the block is one wrap-around range: most quads are entirely outside it
        if ((f < blk.end && f + 4 > blk.start) || f < blk.rest) {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (conef_payload_pos(f + k, blk) >= 0) s[k] = __uint_as_float(kConefSelectedBits);
        }
    }
    __device__ __forceinline__ float element(int r, int64_t col) const
    {
        int64_t f = (int64_t)r * d + col;
        return conef_payload_pos(f, blk) >= 0 ? __uint_as_float(kConefSelectedBits) : x[f];
    }
};

// Phase timestamps (100 MHz counter) of every workgroup of the two passes: only in builds that define
// CONEF_TRACE, read back with conef_trace_read (conef_plan.hip).
#ifdef CONEF_TRACE
static __device__ unsigned long long conef_trace_buf[2][1024][8];
#define CONEF_STAMP(pass, who, slot)                                                                   \
    do {                                                                                               \
        if ((int)threadIdx.x == (who) && blockIdx.x < 1024)                                            \
            conef_trace_buf[pass][blockIdx.x][slot] = (unsigned long long)wall_clock64();              \
    } while (0)
#else
#define CONEF_STAMP(pass, who, slot) do { } while (0)
#endif

// ------------------------------------------------------------------ pass A ----
// One workgroup per chunk: loads, permutes the records into the LDS image, and after the barrier
// the image leaves LDS with linear 16-byte stores.
template <int NROWS, typename Stage, bool VEC>
__global__ void __launch_bounds__(1024)
conef_binned_stage_kernel(Stage stage, ConefPlanView plan, float* __restrict__ staging, int64_t d, int nblocks_padded,
                          int row_first)
{
    extern __shared__ float conef_img[];   // [chunk_cols][NROWS]
    // blockIdx.y: the group of NROWS rows, each with its own region of the staging buffer
    const int rg = row_first + (int)blockIdx.y * NROWS;
    staging += (int64_t)rg * d;
    const int chunk = conef_xcd_major(blockIdx.x, nblocks_padded, plan.flags);
    CONEF_STAMP(0, 0, 0);
    if (chunk >= plan.nchunks) return;
    const int64_t c_begin = (int64_t)chunk * plan.chunk_cols;
    const int cols = d - c_begin < plan.chunk_cols ? (int)(d - c_begin) : plan.chunk_cols;
    const int quads = (cols + 3) >> 2;
    for (int q = threadIdx.x; q < quads; q += blockDim.x) {
        const int64_t c0 = c_begin + (int64_t)q * 4;
        const int valid = cols - q * 4 < 4 ? cols - q * 4 : 4;
        if (VEC && valid == 4) {
            float g[NROWS][4];
#pragma unroll
            for (int r = 0; r < NROWS; ++r) stage.load4(rg + r, c0, g[r]);
            const uint2 pp = *reinterpret_cast<const uint2*>(plan.pos + c0);   // chunk starts are multiples of 4
            const uint32_t p0 = (pp.x & 0xffffu) * NROWS, p1 = (pp.x >> 16) * NROWS;
            const uint32_t p2 = (pp.y & 0xffffu) * NROWS, p3 = (pp.y >> 16) * NROWS;
#pragma unroll
            for (int r = 0; r < NROWS; ++r) {
                conef_img[p0 + r] = g[r][0];
                conef_img[p1 + r] = g[r][1];
                conef_img[p2 + r] = g[r][2];
                conef_img[p3 + r] = g[r][3];
            }
        } else {
            for (int k = 0; k < valid; ++k) {
                uint32_t pk = plan.pos[c0 + k] * NROWS;
                for (int r = 0; r < NROWS; ++r) conef_img[pk + r] = stage.element(rg + r, c0 + k);
            }
        }
    }
    CONEF_STAMP(0, 0, 1);
    __syncthreads();
    CONEF_STAMP(0, 0, 2);
    float* out = staging + c_begin * NROWS;        // 16-byte aligned: c_begin is a multiple of 4
    const int total = cols * NROWS;
    const int total4 = total >> 2;
    for (int e = threadIdx.x; e < total4; e += blockDim.x) {
        float4 v = reinterpret_cast<const float4*>(conef_img)[e];
        conef_store4(out + 4 * e, v.x, v.y, v.z, v.w, (plan.flags & 4) != 0);
    }
    for (int e = (total4 << 2) + threadIdx.x; e < total; e += blockDim.x) out[e] = conef_img[e];
    CONEF_STAMP(0, 0, 3);
}

// Column-order work of the fused RandomBlock step that pass B carries (x == null: none).
struct ConefBlockWork {
    float* x;
    float* payload;
    int64_t numel, m, block;
    ConefBlock blk;
    ConefMod mod;
    ConefSeeds hs;
    float alpha;
};

// ------------------------------------------------------------------ pass B ----
// One workgroup per bin.  LDS holds the bin image [records][NROWS] (ascending column order) and
// the bin's bucket lists.  A group of 2^glog lanes collects the bin's segment of one chunk image,
// four chunks per group in flight, all segment descriptors fetched before the first record.
// Then `bin_buckets` threads times `nsub` row groups walk the bucket lists.
//
// This pass reads a lot and writes next to nothing, the staging pass is the other way round.  So
// the column-order work of the fused RandomBlock step is done here, by the last `col_threads`
// threads of every workgroup, which take no part in the bin's own work: (1) the selected block -
// gather the sketch cell, xq = x + term, payload and x receive xq; (2) zeros over everything
// else.  Separate waves, because on this architecture a wave's loads and stores retire through
// one in-order counter: a wave that has stores in flight cannot wait for a younger load alone.
// Both jobs read only cs_in and x, which is why cs_out must not be cs_in in that mode.
// (at most 64 SGPRs: with about 80 or more, a second 1024-thread workgroup no longer fits on a CU)
template <int NROWS, bool FUSED_QUERY>
__attribute__((amdgpu_num_sgpr(72))) __global__ void __launch_bounds__(1024, 8)
conef_binned_accumulate_kernel(const float* __restrict__ staging, ConefPlanView plan, const float* cs_in, float* cs_out,
                               int32_t w, float alpha, double one_minus_beta, int nblocks_padded, int max_bin_records,
                               int glog, int col_threads, ConefBlockWork bw, int row_first, int64_t d)
{
    extern __shared__ float conef_img[];
    const int gthreads = blockDim.x - col_threads;      // threads that work on the bin
    const float* cs_all = cs_in;                        // the column-order work looks up cells of any row
    {
        // blockIdx.y: the group of NROWS rows this workgroup's bin work is for
        const int64_t rg = row_first + (int64_t)blockIdx.y * NROWS;
        staging += rg * d;
        cs_in += rg * w;
        cs_out += rg * w;
    }
    if ((int)threadIdx.x >= gthreads) {
        // ---- column-order work of the fused step.  These waves owe the bin's threads nothing:
        // they pass the workgroup's one barrier first and then work on their own.
        __syncthreads();
        CONEF_STAMP(1, gthreads, 5);
        const int64_t me = ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * col_threads + (threadIdx.x - gthreads);
        const int64_t nworkers = (int64_t)gridDim.x * gridDim.y * col_threads;
        const int64_t bquads = (bw.block + 3) >> 2;
        for (int64_t q = me; q < bquads; q += nworkers) {
            int64_t p0 = q << 2;
            int n = bw.block - p0 < 4 ? (int)(bw.block - p0) : 4;
            int64_t f = bw.blk.start + p0;
            if (f >= bw.numel) f -= bw.numel;
            int64_t r = f / bw.m, col = f - r * bw.m;
            float* px[4];
            float g[4], cell[4];
            uint32_t pk[4];
            int64_t rr[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                px[k] = bw.x + r * bw.m + col;
                rr[k] = r;
                pk[k] = plan.pk[col];
                g[k] = *px[k];
                if (k + 1 < n) {      // next element of the wrap-around block (else stay on a valid address)
                    ++col;
                    if (col == bw.m) {
                        col = 0;
                        r = (r + 1) * bw.m < bw.numel ? r + 1 : 0;
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) cell[k] = cs_all[rr[k] * (int64_t)w + (pk[k] & 0x7fffffffu)];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if (k < n) {
                    float xq = __fadd_rn(g[k], conef_query_term(cell[k], pk[k], bw.alpha));
                    bw.payload[p0 + k] = xq;
                    *px[k] = xq;
                }
            }
        }
        CONEF_STAMP(1, gthreads, 6);
        const bool vec_ok = (reinterpret_cast<uintptr_t>(bw.x) & 15u) == 0;
        const int64_t nquads = (bw.numel + 3) >> 2;
        for (int64_t q = me; q < nquads; q += nworkers) {
            int64_t f = q << 2;
            int valid = bw.numel - f < 4 ? (int)(bw.numel - f) : 4;
            bool any_sel = (f < bw.blk.end && f + valid > bw.blk.start) || f < bw.blk.rest;
            if (!any_sel && vec_ok && valid == 4) {
                conef_store4(bw.x + f, 0.f, 0.f, 0.f, 0.f, (plan.flags & 2) != 0);
            } else {
                for (int k = 0; k < valid; ++k)
                    if (!any_sel || conef_payload_pos(f + k, bw.blk) < 0) bw.x[f + k] = 0.f;
            }
        }
        CONEF_STAMP(1, gthreads, 7);
        return;
    }
    CONEF_STAMP(1, 0, 0);

    const int bin_raw = conef_xcd_major(blockIdx.x, nblocks_padded, plan.flags);
    const bool has_bin = bin_raw < plan.nbins;          // padding workgroups only share the column work
    const int bin = has_bin ? bin_raw : 0;
    uint16_t* ent_l = reinterpret_cast<uint16_t*>(conef_img + (size_t)max_bin_records * NROWS);

    // who am I in the accumulate phase; every index is clamped so the loads below are unconditional
    const int tpad = (plan.bin_buckets + 63) & ~63;
    const int nsub = gthreads / tpad;                   // row groups working on the same bucket
    const int jl = threadIdx.x % tpad, sub = threadIdx.x / tpad;
    const int64_t j_first = (int64_t)bin * plan.bin_buckets;
    const int64_t j_last = j_first + plan.bin_buckets < w ? j_first + plan.bin_buckets : w;
    const bool active = has_bin && sub < nsub && j_first + jl < j_last;
    const int64_t j = active ? j_first + jl : j_first;

    // ---- level 1: everything addressable from the bin number alone
    const int gsize = 1 << glog;
    const int group = threadIdx.x >> glog, gl = threadIdx.x & (gsize - 1), ngroups = gthreads >> glog;
    const uint32_t* seg = plan.seg + (int64_t)bin * (plan.nchunks + 1);
    const int last_c = plan.nchunks - 1;
    uint32_t sg0[4], sg1[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        int c = group + u * ngroups;
        int cc = c < plan.nchunks ? c : last_c;
        sg0[u] = seg[cc];
        sg1[u] = seg[cc + 1];
    }
    const uint32_t e_first = plan.csr[j_first], e_last = plan.csr[j_last];
    const uint32_t e0g = plan.csr[j], e1g = plan.csr[j + 1];
    float aux[NROWS];
#pragma unroll
    for (int k = 0; k < NROWS; ++k) {
        int r = sub + k * nsub;
        aux[k] = cs_in[(int64_t)(r < NROWS ? r : NROWS - 1) * w + j];
    }

    // ---- level 2: the first record of each of my four segments (lane gl of the group)
    float v[4][NROWS];
    int dst[4], len[4];
    const float* srcp[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        int c = group + u * ngroups;
        int off = (int)(sg0[u] >> 16);
        len[u] = (c < plan.nchunks && has_bin) ? (int)(sg1[u] >> 16) - off : 0;
        int cc = c < plan.nchunks ? c : last_c;
        srcp[u] = staging + ((int64_t)cc * plan.chunk_cols + (sg0[u] & 0xffffu)) * NROWS;
        dst[u] = off * NROWS;
        int k = gl < len[u] ? gl : 0;                   // clamped: the load is unconditional
#pragma unroll
        for (int r = 0; r < NROWS; ++r) v[u][r] = srcp[u][k * NROWS + r];
    }
    CONEF_STAMP(1, 0, 1);       // the first records of my segments have arrived
    if (has_bin)
        for (uint32_t t = threadIdx.x; t < e_last - e_first; t += gthreads) ent_l[t] = plan.ent[e_first + t];

    // records into the image; segments longer than a lane group, and chunks beyond the first
    // four per group, take the slow lane-strided loop
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        if (gl < len[u]) {
#pragma unroll
            for (int r = 0; r < NROWS; ++r) conef_img[dst[u] + gl * NROWS + r] = v[u][r];
        }
        for (int k = gl + gsize; k < len[u]; k += gsize) {
#pragma unroll
            for (int r = 0; r < NROWS; ++r) conef_img[dst[u] + k * NROWS + r] = srcp[u][k * NROWS + r];
        }
    }
    if (has_bin) {
        for (int c = group + 4 * ngroups; c < plan.nchunks; c += ngroups) {
            uint32_t s0 = seg[c], s1 = seg[c + 1];
            int off = (int)(s0 >> 16), ln = (int)(s1 >> 16) - off;
            const float* sp = staging + ((int64_t)c * plan.chunk_cols + (s0 & 0xffffu)) * NROWS;
            for (int k = gl; k < ln; k += gsize) {
#pragma unroll
                for (int r = 0; r < NROWS; ++r) conef_img[(off + k) * NROWS + r] = sp[k * NROWS + r];
            }
        }
    }
    CONEF_STAMP(1, 0, 2);
    __syncthreads();
    CONEF_STAMP(1, 0, 3);

    if (!active) return;
    // per row: the decay c*aux (double) and the query term for sign +1 do not change along the
    // bucket list; for sign -1 the query term is the exact negation (multiplication is symmetric)
    double decay[NROWS];
    float qterm[NROWS], acc[NROWS];
#pragma unroll
    for (int k = 0; k < NROWS; ++k) {
        decay[k] = __dmul_rn(one_minus_beta, (double)aux[k]);
        qterm[k] = __fmul_rn(aux[k], alpha);
        acc[k] = aux[k];
    }
    for (uint32_t e = e0g - e_first; e < e1g - e_first; ++e) {
        uint32_t en = ent_l[e];
        const float* rec = conef_img + (en & 0x7fffu) * NROWS;
        uint32_t flip = ((~en) & 0x8000u) << 16;       // sign bit clear (-1): flip the float's sign
#pragma unroll
        for (int k = 0; k < NROWS; ++k) {
            int r = sub + k * nsub;
            if (r < NROWS) {
                float val = rec[r];
                if (FUSED_QUERY) {
                    bool selected = __float_as_uint(val) == kConefSelectedBits;
                    val = __fadd_rn(val, __uint_as_float(__float_as_uint(qterm[k]) ^ flip));
                    val = selected ? 0.f : val;
                }
                double sv = (double)__uint_as_float(__float_as_uint(val) ^ flip);
                acc[k] = __fadd_rn(acc[k], (float)__dsub_rn(sv, decay[k]));
            }
        }
    }
#pragma unroll
    for (int k = 0; k < NROWS; ++k) {
        int r = sub + k * nsub;
        if (r < NROWS) cs_out[(int64_t)r * w + j] = acc[k];
    }
    CONEF_STAMP(1, 0, 4);
}

// ---------------------------------------------------------------- launcher ----
inline size_t conef_binned_lds_b(const ConefPlanHeader* hp, int nrows)
{
    size_t b = (size_t)hp->max_bin_records * nrows * 4 + (size_t)hp->max_bin_records * 2 + 16;
    return (b + 15) & ~(size_t)15;
}


// Pass A over `groups` groups of NROWS rows, the first of them starting at row `row_first`.
template <int NROWS, typename Stage>
int conef_launch_stage_rows(Stage stage, const ConefPlanHeader* hp, const void* plan_dev, float* staging, bool vec_ok,
                            int row_first, int groups, hipStream_t s)
{
    ConefPlanView view = conef_plan_view(hp, plan_dev);
    size_t lds_a = (size_t)hp->chunk_cols * NROWS * 4;
    if (lds_a > 160 * 1024) return CONEF_ERR_INVALID;
    int ga = (hp->nchunks + 7) & ~7;
    int threads_a = (hp->chunk_cols / 4 + 63) & ~63;
    if (threads_a > 1024) threads_a = 1024;
    hipError_t e;
    if (vec_ok && hp->d % 4 == 0) {
        auto ka = conef_binned_stage_kernel<NROWS, Stage, true>;
        e = conef_allow_lds((const void*)ka, lds_a);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(ka, dim3(ga, groups), dim3(threads_a), lds_a, s, stage, view, staging, hp->d, ga, row_first);
    } else {
        auto ka = conef_binned_stage_kernel<NROWS, Stage, false>;
        e = conef_allow_lds((const void*)ka, lds_a);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(ka, dim3(ga, groups), dim3(threads_a), lds_a, s, stage, view, staging, hp->d, ga, row_first);
    }
    return (int)hipGetLastError();
}

// Pass B over the same groups; `bw` (the fused step's column-order work over the whole tensor) rides in it.
template <int NROWS, bool FUSED_QUERY>
int conef_launch_accumulate_rows(const ConefPlanHeader* hp, const void* plan_dev, const float* staging, const float* cs_in,
                                 float* cs_out, float alpha, float beta, ConefBlockWork bw, int row_first, int groups,
                                 hipStream_t s)
{
    ConefPlanView view = conef_plan_view(hp, plan_dev);
    const double omb = 1. - (double)beta;
    size_t lds_b = conef_binned_lds_b(hp, NROWS);
    if (lds_b > 160 * 1024) return CONEF_ERR_INVALID;
    int gb = (hp->nbins + 7) & ~7;
    int tpad = (hp->bin_buckets + 63) & ~63;
    int col_threads = bw.x ? 256 : 0;                   // waves of pass B that do the fused step's column work
    if (tpad + col_threads > 1024) col_threads = 1024 - tpad;
    if (bw.x && col_threads < 64) return CONEF_ERR_INVALID;
    int threads_b = (1024 - col_threads) / tpad * tpad + col_threads;
    auto kb = conef_binned_accumulate_kernel<NROWS, FUSED_QUERY>;
    {
        hipError_t e = conef_allow_lds((const void*)kb, lds_b);
        if (e != hipSuccess) return (int)e;
    }
    // lanes per segment: the power of two above 1.3 x the mean segment length, 8..64
    double mean_seg = (double)hp->chunk_cols * hp->bin_buckets / (double)hp->w * 1.3;
    int glog = 3;
    while (glog < 6 && (1 << glog) < mean_seg) ++glog;
    hipLaunchKernelGGL(kb, dim3(gb, groups), dim3(threads_b), lds_b, s, staging, view, cs_in, cs_out, hp->w, alpha, omb, gb,
                       hp->max_bin_records, glog, col_threads, bw, row_first, hp->d);
    return (int)hipGetLastError();
}

// The two passes over all rows of the plan's tensor: whole groups of 8 rows in one launch of each
// pass (the group is the second grid dimension), the remaining 1 to 7 rows in a launch of their
// own.  Every pass A runs before the first pass B, because the column-order work that rides in
// pass B rewrites the tensor pass A reads.
template <typename Stage>
int conef_launch_binned(Stage stage, const ConefPlanHeader* hp, const void* plan_dev, float* staging,
                        const float* cs_in, float* cs_out, float alpha, float beta, bool vec_ok, ConefBlockWork bw,
                        hipStream_t s)
{
    const int full = (int)(hp->n / kConefPlanMaxRows), rem = (int)(hp->n % kConefPlanMaxRows);
    if (full > 65535) return CONEF_ERR_INVALID;
    int rc = CONEF_OK;
    if (full > 0) rc = conef_launch_stage_rows<kConefPlanMaxRows, Stage>(stage, hp, plan_dev, staging, vec_ok, 0, full, s);
    if (rc != CONEF_OK) return rc;
    const int rf = full * kConefPlanMaxRows;
    switch (rem) {
#define CONEF_CASE(NR) \
    case NR: rc = conef_launch_stage_rows<NR, Stage>(stage, hp, plan_dev, staging, vec_ok, rf, 1, s); break
        CONEF_CASE(1);
        CONEF_CASE(2);
        CONEF_CASE(3);
        CONEF_CASE(4);
        CONEF_CASE(5);
        CONEF_CASE(6);
        CONEF_CASE(7);
#undef CONEF_CASE
    }
    if (rc != CONEF_OK) return rc;
    ConefBlockWork none = {};
    if (full > 0)
        rc = conef_launch_accumulate_rows<kConefPlanMaxRows, Stage::kFusedQuery>(hp, plan_dev, staging, cs_in, cs_out, alpha,
                                                                                 beta, bw, 0, full, s);
    if (rc != CONEF_OK) return rc;
    const ConefBlockWork& rest = full > 0 ? none : bw;
    switch (rem) {
#define CONEF_CASE(NR)                                                                                              \
    case NR:                                                                                                        \
        rc = conef_launch_accumulate_rows<NR, Stage::kFusedQuery>(hp, plan_dev, staging, cs_in, cs_out, alpha, beta, rest, \
                                                                  rf, 1, s);                                        \
        break
        CONEF_CASE(1);
        CONEF_CASE(2);
        CONEF_CASE(3);
        CONEF_CASE(4);
        CONEF_CASE(5);
        CONEF_CASE(6);
        CONEF_CASE(7);
#undef CONEF_CASE
    }
    return rc;
}

// validates a host-side plan header against the call's shape
inline bool conef_plan_matches(const ConefPlanHeader* hp, int64_t n, int64_t d, int32_t w, int32_t a, int32_t b)
{
    return hp && hp->magic == kConefPlanMagic && hp->version == 1 &&
           (hp->kind == kConefPlanBinned || hp->kind == kConefPlanRowlist || hp->kind == kConefPlanPanels) && hp->n == n && hp->d == d && hp->w == w &&
           hp->a == a && hp->b == b;
}
