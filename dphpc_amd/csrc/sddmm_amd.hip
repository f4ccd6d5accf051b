// C ABI of the gfx950 SDDMM engine: context, operand upload, plan, launch.
// See include/sddmm_amd.h for the contract of every entry point.
#include "../../include/sddmm_amd.h"

#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <climits>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "kernels_fused.h"
#include "kernels_gather.h"
#include "kernels_plan.h"
#include "kernels_tile.h"

using namespace sddmm;

// ---------------------------------------------------------------------------
struct sddmm_ctx {
    int device = 0;
    hipStream_t stream = nullptr;      // where work is enqueued: own_stream unless the caller lent one
    hipStream_t own_stream = nullptr;
    bool lent_stream = false;
    bool oversize = false;             // a launch was skipped because its grid does not fit one dispatch
    hipEvent_t ev0 = nullptr, ev1 = nullptr;

    char err[512] = {0};

    // dense operands
    int M = 0, N = 0, K = 0, dtype = SDDMM_F32;
    bool have_dense = false;
    void *dA = nullptr, *dB = nullptr;
    bool own_dense = false;

    // sparse operand
    bool have_sparse = false, have_rowptr = false, own_sparse = false, from_coo = false;
    int sM = 0, sN = 0;
    int64_t nnz = 0;
    int32_t *d_rowptr = nullptr, *d_col = nullptr, *d_rowidx = nullptr;
    float *d_sval = nullptr, *dP = nullptr;
    bool own_rowptr = false, own_rowidx = false;

    // plan
    bool planned = false;
    int strategy = SDDMM_AUTO;       // resolved
    int requested = SDDMM_AUTO;
    DevCounters *d_pc = nullptr;     // device counters
    DevCounters raw{};               // host copy of the device block
    DevCounters *h_pc = nullptr;     // pinned landing place of the read-back (no staging copy)
    PlanCounters pc{};               // its summary
    sddmm_stats stats{};
    // AUTO: rows shorter than ts go to the many-rows-per-wave kernel, the others
    // become wave-per-segment items of at most seg entries
    int ts = 0, seg = 0, rpw = 64;
    RowItem *d_items = nullptr;
    int64_t n_items = 0, items_cap = 0;
    unsigned int *d_block_sums = nullptr;
    int64_t block_sums_cap = 0;
    int64_t rows_short = 0;
    int launches = 0;
    // dense-tile (MFMA) path
    unsigned int *d_strip_ntiles = nullptr, *d_strip_off = nullptr;
    int64_t strips_cap = 0;
    TileDesc *d_tiles = nullptr;
    int64_t n_tiles = 0, tiles_cap = 0, nnz_tiles = 0;
    int tile_steps = 0;
    bool tiles_active = false;       // d_tiles describes the current pattern
    int32_t *d_win_order = nullptr;  // order in which the launch takes the windows (null: storage order)
    unsigned int *d_win_bins = nullptr;
    int64_t win_order_cap = 0;
    bool use_win_order = false;
    TileWindow *d_windows = nullptr; // one record per TILE_WINDOW consecutive descriptors
    int64_t n_windows = 0, windows_cap = 0;
    bool use_windows = false;        // tile kernels take windows as batches (else they walk them tile by tile)
    int64_t n_tiles_natural = 0;     // descriptors: 16-row strips first, then union strips, then gathered strips
    int64_t n_tiles_lead = 0;        // empty descriptors that fill the last window before the gathered strips
    int64_t n_win_single = 0;        // windows taken one per wavefront; the rest (gathered pairs) two per wavefront
    int64_t n_tile_units = 0;        // wavefronts of a tile launch
    int64_t n_tiles_union = 0, nnz_tiles_union = 0;
    unsigned int *d_ustrip_ntiles = nullptr, *d_ustrip_off = nullptr;
    int64_t ustrips_cap = 0;
    int32_t *d_tile_cols = nullptr;  // 16 B rows per descriptor
    bool union_counted = false;
    // gathered strips: candidate rows, sorted by first column, 16 per strip
    unsigned long long *d_cand_keys = nullptr, *d_sorted_keys = nullptr;   // (first column << 32) | row
    int32_t *d_vrows = nullptr;
    void *d_sort_tmp = nullptr;
    size_t sort_tmp_bytes = 0;
    int64_t cand_cap = 0, vstrips_cap = 0, n_cand = 0, n_vstrips = 0;
    unsigned int *d_vstrip_ntiles = nullptr, *d_vstrip_off = nullptr;
    // row ownership (one byte per row: 0 row kernels, 1 dense tiles, 2 row panels, 3 gathered strips, 4 union strips)
    unsigned char *d_owner = nullptr;
    int64_t owner_cap = 0;
    // every work array of the plan whose size follows from the number of rows lives in one
    // allocation (a first plan then pays for one hipMalloc instead of a dozen)
    char *d_arena = nullptr;
    int64_t arena_rows = -1;
    bool owner_active = false;
    // row-panel path
    unsigned int *d_panel_counts = nullptr, *d_panel_off = nullptr;
    int64_t panels_cap = 0;
    int2 *d_short_list = nullptr;    // {position, row} of the entries of the short rows nobody owns
    int64_t n_short_list = 0, short_list_cap = 0;
    ScanJobs scan_jobs{};            // short scans waiting for the next read-back of the counters
    int n_scan_jobs = 0;
    bool use_short_list = false;
    unsigned int *d_short_sums = nullptr;   // arena view: entries of short rows per block of the row scan
    RowItem *d_panel_items = nullptr;
    int64_t n_panel_items = 0, panel_items_cap = 0, n_panels = 0, nnz_panels = 0;
    bool panel_mfma = false;         // panels run on k_panel_mfma (else on k_panel)
    bool panels_flagged = false;     // the panel detector ran in this plan
    // fused SDDMM + SpMM: items covering every non-empty row, output M x K
    RowItem *d_fused_items = nullptr;
    int64_t n_fused_items = 0, fused_items_cap = 0;
    bool fused_items_valid = false;
    bool fused_items_panels = false; // the fused items leave out the rows that the panel kernel owns
    double fused_short_avg = 0.0;    // entries per non-empty row of at most FUSED_ROW_MAX entries (panel rows apart)
    float *dO = nullptr;
    size_t o_cap = 0;
    bool have_fused = false;
};

namespace {

int fail(sddmm_ctx *c, int code, const char *fmt, ...) {
    if (c) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(c->err, sizeof(c->err), fmt, ap);
        va_end(ap);
    }
    return code;
}

#define HIP_TRY(c, call)                                                                         \
    do {                                                                                         \
        hipError_t e_ = (call);                                                                  \
        if (e_ != hipSuccess)                                                                    \
            return fail((c), SDDMM_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                        __FILE__, __LINE__);                                                     \
    } while (0)

#define ALLOC_TRY(c, ptr, bytes)                                                                 \
    do {                                                                                         \
        hipError_t e_ = hipMalloc((void **)&(ptr), (bytes) ? (bytes) : 16);                      \
        if (e_ != hipSuccess) {                                                                  \
            (ptr) = nullptr;                                                                     \
            return fail((c), SDDMM_ERR_ALLOC, "hipMalloc(%zu bytes) failed: %s", (size_t)(bytes), \
                        hipGetErrorString(e_));                                                  \
        }                                                                                        \
    } while (0)

// A dispatch packet counts the work-items of a grid dimension in 32 bits: a launch of 2^32
// threads or more would run only part of its grid, without any error.  Such a launch is not
// made; launch_status() turns the skipped launch into an error of the entry point.
#define SDDMM_LAUNCH(c, kernel, grid, block, ...)                                                        \
    do {                                                                                                 \
        const int64_t g_ = (int64_t)(grid);                                                              \
        const int b_ = (int)(block);                                                                     \
        if (g_ * b_ >= ((int64_t)1 << 32)) (c)->oversize = true;                                         \
        else hipLaunchKernelGGL(kernel, dim3((unsigned)g_), dim3((unsigned)b_), 0, (c)->stream, __VA_ARGS__); \
    } while (0)

int launch_status(sddmm_ctx *c) {
    if (!c->oversize) return SDDMM_OK;
    c->oversize = false;
    return fail(c, SDDMM_ERR_UNSUPPORTED,
                "a kernel of this strategy needs 2^32 threads or more in one launch for this matrix "
                "(one wavefront per row or per work item): use SDDMM_AUTO or SDDMM_FLAT");
}

// after a group of launches: a failed launch, or one that was not made
#define LAUNCH_CHECK(c)                                \
    do {                                               \
        HIP_TRY(c, hipGetLastError());                 \
        const int ls_ = launch_status(c);              \
        if (ls_) return ls_;                           \
    } while (0)

template <class T>
void dfree(T *&p) {
    if (p) (void)hipFree((void *)p);
    p = nullptr;
}

// Views into the plan arena: nothing here is freed on its own.
void release_arena(sddmm_ctx *c) {
    dfree(c->d_arena);
    c->arena_rows = -1;
    c->d_owner = nullptr;
    c->d_strip_ntiles = c->d_strip_off = c->d_ustrip_ntiles = c->d_ustrip_off = nullptr;
    c->d_panel_counts = c->d_panel_off = c->d_vstrip_ntiles = c->d_vstrip_off = nullptr;
    c->d_cand_keys = c->d_sorted_keys = nullptr;
    c->d_vrows = nullptr;
    c->d_block_sums = c->d_short_sums = nullptr;
    c->owner_cap = c->strips_cap = c->ustrips_cap = c->panels_cap = c->cand_cap = c->vstrips_cap = 0;
    c->block_sums_cap = 0;
}

int ensure_arena(sddmm_ctx *c) {
    const int64_t M = c->sM;
    if (c->d_arena && c->arena_rows == M) return SDDMM_OK;
    release_arena(c);
    const int64_t n_strips = (M + 15) / 16, n_panels = M / 8 + 1, n_sums = M / 1024 + 2;
    size_t at = 0;
    auto take = [&](size_t bytes) {
        const size_t here = at;
        at += (bytes + 255) & ~(size_t)255;
        return here;
    };
    const size_t o_owner = take((size_t)M + 64);
    const size_t o_strip_n = take((size_t)n_strips * 4), o_strip_o = take((size_t)n_strips * 4);
    const size_t o_ustrip_n = take((size_t)n_strips * 4), o_ustrip_o = take((size_t)n_strips * 4);
    // (gathered strips come in pairs: up to two more than M / 16)
    const size_t o_vstrip_n = take((size_t)(n_strips + 2) * 4), o_vstrip_o = take((size_t)(n_strips + 2) * 4);
    const size_t o_vrows = take((size_t)(n_strips + 2) * 16 * 4);
    const size_t o_panel_n = take((size_t)n_panels * 4), o_panel_o = take((size_t)n_panels * 4);
    const size_t o_keys = take((size_t)(M + 1) * 8), o_sorted = take((size_t)(M + 1) * 8);
    const size_t o_sums = take((size_t)n_sums * 4), o_short_sums = take((size_t)n_sums * 4);
    ALLOC_TRY(c, c->d_arena, at);
    char *b = c->d_arena;
    c->d_owner = (unsigned char *)(b + o_owner);
    c->d_strip_ntiles = (unsigned int *)(b + o_strip_n); c->d_strip_off = (unsigned int *)(b + o_strip_o);
    c->d_ustrip_ntiles = (unsigned int *)(b + o_ustrip_n); c->d_ustrip_off = (unsigned int *)(b + o_ustrip_o);
    c->d_vstrip_ntiles = (unsigned int *)(b + o_vstrip_n); c->d_vstrip_off = (unsigned int *)(b + o_vstrip_o);
    c->d_vrows = (int32_t *)(b + o_vrows);
    c->d_panel_counts = (unsigned int *)(b + o_panel_n); c->d_panel_off = (unsigned int *)(b + o_panel_o);
    c->d_cand_keys = (unsigned long long *)(b + o_keys); c->d_sorted_keys = (unsigned long long *)(b + o_sorted);
    c->d_block_sums = (unsigned int *)(b + o_sums);
    c->d_short_sums = (unsigned int *)(b + o_short_sums);
    c->owner_cap = M + 64;
    c->strips_cap = c->ustrips_cap = n_strips;
    c->vstrips_cap = n_strips + 2;
    c->panels_cap = n_panels;
    c->cand_cap = M + 1;
    c->block_sums_cap = n_sums;
    c->arena_rows = M;
    return SDDMM_OK;
}

// an arena view turned out too small: the sizes above are upper bounds, so this is a bug
#define ARENA_HOLDS(c, need, cap, what)                                                             \
    do {                                                                                            \
        if ((int64_t)(need) > (int64_t)(cap))                                                       \
            return fail((c), SDDMM_ERR_HIP, "internal: plan arena too small for %s (%lld > %lld)", what, \
                        (long long)(need), (long long)(cap));                                       \
    } while (0)

void release_dense(sddmm_ctx *c) {
    if (c->own_dense) { dfree(c->dA); dfree(c->dB); }
    c->dA = c->dB = nullptr;
    c->have_fused = false;
    c->own_dense = false;
    c->have_dense = false;
    c->planned = false;
}

void release_sparse(sddmm_ctx *c) {
    if (c->own_sparse) { dfree(c->d_col); dfree(c->d_sval); }
    if (c->own_rowptr) dfree(c->d_rowptr);
    if (c->own_rowidx) dfree(c->d_rowidx);
    dfree(c->dP);
    dfree(c->d_items);
    dfree(c->d_tiles);
    dfree(c->d_tile_cols);
    dfree(c->d_windows);
    dfree(c->d_win_order);
    dfree(c->d_win_bins);
    c->win_order_cap = 0;
    c->use_win_order = false;
    c->n_windows = c->windows_cap = 0;
    c->ustrips_cap = 0;
    dfree(c->d_sort_tmp);
    release_arena(c);
    c->sort_tmp_bytes = 0;
    c->cand_cap = c->vstrips_cap = c->n_cand = c->n_vstrips = 0;
    dfree(c->d_panel_items);
    dfree(c->d_short_list);
    c->short_list_cap = c->n_short_list = 0;
    c->use_short_list = false;
    dfree(c->d_fused_items);
    c->n_fused_items = c->fused_items_cap = 0;
    c->fused_items_valid = c->have_fused = false;
    c->owner_cap = c->panels_cap = c->panel_items_cap = 0;
    c->n_panel_items = c->n_panels = c->nnz_panels = 0;
    c->owner_active = false;
    c->items_cap = c->block_sums_cap = c->n_items = 0;
    c->strips_cap = c->tiles_cap = c->n_tiles = c->nnz_tiles = 0;
    c->tiles_active = false;
    c->d_col = nullptr; c->d_sval = nullptr; c->d_rowptr = nullptr; c->d_rowidx = nullptr;
    c->own_sparse = c->own_rowptr = c->own_rowidx = false;
    c->have_sparse = c->have_rowptr = false;
    c->from_coo = false;
    c->planned = false;
    c->nnz = 0;
}

size_t elem_size(int dtype) { return dtype == SDDMM_F32 ? 4 : 2; }

int grid_for(int64_t n, int block) { return (int)std::max<int64_t>(1, (n + block - 1) / block); }
int grid_capped(int64_t n, int block, int cap = 16384) {
    return (int)std::min<int64_t>(cap, std::max<int64_t>(1, (n + block - 1) / block));
}

// The short scans of a plan (tiles per strip, items per panel, block sums of the row classes ...) feed
// nothing before the next read-back of the counters, so they are collected and run as ONE launch
// there instead of one launch each behind its producer.
int flush_scans(sddmm_ctx *c) {
    if (c->n_scan_jobs == 0) return SDDMM_OK;
    SDDMM_LAUNCH(c, k_scan_jobs, c->n_scan_jobs, SCAN_BLOCK, c->scan_jobs);
    c->n_scan_jobs = 0;
    LAUNCH_CHECK(c);
    return SDDMM_OK;
}
int queue_scan(sddmm_ctx *c, const unsigned int *in, unsigned int *out, int64_t n, unsigned long long *d_total) {
    if (c->n_scan_jobs == SCAN_JOBS_MAX) {
        const int rc = flush_scans(c);
        if (rc) return rc;
    }
    c->scan_jobs.job[c->n_scan_jobs++] = ScanJob{in, out, d_total, (int)n, 0};
    return SDDMM_OK;
}

int fetch_counters(sddmm_ctx *c) {
    {
        const int rc = flush_scans(c);
        if (rc) return rc;
    }
    HIP_TRY(c, hipMemcpyAsync(c->h_pc, c->d_pc, sizeof(DevCounters), hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    c->raw = *c->h_pc;
    c->pc = summarize(c->raw);
    return SDDMM_OK;
}

// ---- kernel dispatch over the (unit type, lanes per entry, units per lane) layouts ----
struct Shape {
    int unit;    // 0: fp32 x4, 1: fp32 x1, 2: bf16 x8, 3: fp16 x8
    int KU;      // units per row
    int LPN;     // lanes per entry (0: row too long for the register layout)
    int UPL;     // units per lane
    bool fullk;  // KU == LPN*UPL
    bool wide;   // operands of 4 GiB or more: 64-bit byte offsets
};

int pow2ceil(int x) {
    int l = 1;
    while (l < x) l <<= 1;
    return l;
}

Shape shape_of(const sddmm_ctx *c) {
    Shape s{};
    size_t unit_bytes;
    if (c->dtype == SDDMM_BF16 || c->dtype == SDDMM_F16) { s.unit = c->dtype == SDDMM_BF16 ? 2 : 3; s.KU = c->K / 8; unit_bytes = 16; }
    else if (c->K % 4 == 0) { s.unit = 0; s.KU = c->K / 4; unit_bytes = 16; }
    else { s.unit = 1; s.KU = c->K; unit_bytes = 4; }
    if (s.unit == 1) {
        // 4-byte units: 16 lanes cover 64 contiguous bytes
        if (s.KU <= 4) { s.LPN = 4; s.UPL = 1; }
        else if (s.KU <= 16) { s.LPN = 16; s.UPL = 1; }
        else if (s.KU <= 64) { s.LPN = 16; s.UPL = 4; }
        else if (s.KU <= 128) { s.LPN = 16; s.UPL = 8; }
        else { s.LPN = 0; s.UPL = 0; }
    } else {
        // 16-byte units: 8 lanes cover one whole 128-byte cache line per load
        // instruction (measured faster than 4 lanes x 64 bytes: half the lines per
        // instruction for the same bytes)
        if (s.KU <= 8) { s.LPN = pow2ceil(s.KU); s.UPL = 1; }
        else if (s.KU <= 64) { s.LPN = 8; s.UPL = pow2ceil((s.KU + 7) / 8); }
        else if (s.KU <= 128) { s.LPN = 16; s.UPL = 8; }
        else { s.LPN = 0; s.UPL = 0; }
    }
    s.fullk = s.LPN > 0 && s.KU == s.LPN * s.UPL;
    const size_t rows = (size_t)std::max(c->M, c->N);
    s.wide = rows * (size_t)s.KU * unit_bytes >= ((size_t)1 << 32);
    return s;
}

// Calls f(Layout<...>{}) for the layout matching s.
template <class U, int LPN, int UPL, class F>
void with_mask_width(const Shape &s, F &&f) {
    if (s.wide) f(Layout<U, LPN, UPL, false, true>{});
    else if (s.fullk && U::ELEMS > 1) f(Layout<U, LPN, UPL, true, false>{});
    else f(Layout<U, LPN, UPL, false, false>{});
}

template <class U, class F>
void with_layout16(const Shape &s, F &&f) {
    if (s.LPN == 0) { f(Layout<U, 0, 1, false, true>{}); return; }
    if (s.LPN == 1) with_mask_width<U, 1, 1>(s, f);
    else if (s.LPN == 2) with_mask_width<U, 2, 1>(s, f);
    else if (s.LPN == 4) with_mask_width<U, 4, 1>(s, f);
    else if (s.LPN == 16) with_mask_width<U, 16, 8>(s, f);
    else if (s.UPL == 1) with_mask_width<U, 8, 1>(s, f);
    else if (s.UPL == 2) with_mask_width<U, 8, 2>(s, f);
    else if (s.UPL == 4) with_mask_width<U, 8, 4>(s, f);
    else with_mask_width<U, 8, 8>(s, f);
}

template <class F>
void with_layout(const Shape &s, F &&f) {
    if (s.unit == 0) with_layout16<UnitF32x4>(s, f);
    else if (s.unit == 2) with_layout16<UnitBF16x8>(s, f);
    else if (s.unit == 3) with_layout16<UnitF16x8>(s, f);
    else if (s.LPN == 0) f(Layout<UnitF32x1, 0, 1, false, true>{});
    else if (s.LPN == 4) with_mask_width<UnitF32x1, 4, 1>(s, f);
    else if (s.UPL == 1) with_mask_width<UnitF32x1, 16, 1>(s, f);
    else if (s.UPL == 4) with_mask_width<UnitF32x1, 16, 4>(s, f);
    else with_mask_width<UnitF32x1, 16, 8>(s, f);
}

void launch_flat(sddmm_ctx *c) {
    const Shape s = shape_of(c);
    const int64_t chunks = (c->nnz + WAVE - 1) / WAVE;
    const int cpw = (int)std::min<int64_t>(8, std::max<int64_t>(1, chunks / (WAVES_PER_BLOCK * 4096)));
    const int64_t waves = (chunks + cpw - 1) / cpw;
    const int64_t nblocks = (waves + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    with_layout(s, [&](auto L) {
        using LT = decltype(L);
        SDDMM_LAUNCH(c, (k_flat<LT>), xcd_grid(nblocks), BLOCK,
                           (const void *)c->dA, (const void *)c->dB, s.KU, c->d_rowidx, c->d_col, c->d_sval, c->dP,
                           c->nnz, cpw, nblocks);
    });
}

void launch_row_wave(sddmm_ctx *c, const RowItem *items, int64_t n_items) {
    const Shape s = shape_of(c);
    const int64_t nblocks = (n_items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    with_layout(s, [&](auto L) {
        using LT = decltype(L);
        SDDMM_LAUNCH(c, (k_row_wave<LT>), xcd_grid(nblocks), BLOCK,
                           (const void *)c->dA, (const void *)c->dB, s.KU, c->d_rowptr, c->d_col, c->d_sval, c->dP,
                           items, n_items, nblocks);
    });
}

// rows per wavefront of the many-rows body: about 256 short entries per wave, so
// that small matrices still produce enough waves to fill the chip
int rows_per_wave(double avg_short_len) {
    int rpw = 64;
    while (rpw > 8 && rpw * std::max(avg_short_len, 1.0) > 384.0) rpw >>= 1;
    return rpw;
}

void launch_short_rows(sddmm_ctx *c, int ts, int rpw) {
    const Shape s = shape_of(c);
    const int64_t waves = ((int64_t)c->sM + rpw - 1) / rpw;
    const int64_t nblocks = (waves + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    with_layout(s, [&](auto L) {
        using LT = decltype(L);
        SDDMM_LAUNCH(c, (k_short_rows<LT>), xcd_grid(nblocks), BLOCK,
                           (const void *)c->dA, (const void *)c->dB, s.KU, c->d_rowptr, c->d_col, c->d_sval, c->dP,
                           c->sM, ts, rpw, nblocks);
    });
}

int env_int(const char *name, int fallback) {
    const char *e = getenv(name);
    return e && *e ? atoi(e) : fallback;
}

// wavefronts of the short-row part of the AUTO launches: 64 entries of the entry list each, or
// rpw consecutive rows each
int64_t short_row_waves(const sddmm_ctx *c) {
    if (c->rows_short <= 0) return 0;
    if (c->use_short_list) return (c->n_short_list + WAVE - 1) / WAVE;
    return ((int64_t)c->sM + c->rpw - 1) / c->rpw;
}

// Tiles and rows in one launch (k_auto_tiles); measured faster than two launches at
// every row size the tile path takes (mixed-density shape: 23 -> 20 us at 128-byte
// rows, 107 -> 92 us at 1 KiB rows).  Returns false when the layout has no fused
// kernel; the caller then launches the two kernels in turn.
bool launch_auto_with_tiles(sddmm_ctx *c) {
    const Shape s = shape_of(c);
    if (c->tile_steps < 1 || c->tile_steps > env_int("SDDMM_FUSE_STEPS", 16) || !s.fullk || s.wide || s.unit == 1 || s.KU != 4 * c->tile_steps)
        return false;
    const int64_t waves = short_row_waves(c);
    const int64_t short_blocks = (waves + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    const int64_t item_blocks = (c->n_items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    const int64_t tile_blocks = (c->n_tile_units + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    const int64_t nblocks = short_blocks + item_blocks + tile_blocks;
    // Order of the blocks on every XCD.  Rows of up to 256 bytes: the tile windows (the wavefronts that
    // live longest) start first, then the items, then the chunks of the entry list -- measured
    // 14.7 -> 13.5 us on the mixed-density shape at 128 bytes, 21.3 -> 21.1 us (cold 29.7 -> 27.8) at
    // 256; at 1 KiB, where the gathers of the short rows are the longer half, the even deal is 3 % faster.
    const int longest_first = env_int("SDDMM_LONGEST_FIRST", c->tile_steps <= 4 ? 1 : 0);
    auto eighth = [](int64_t n) { return (n + NUM_XCD - 1) / NUM_XCD; };
    const int64_t grid = longest_first ? NUM_XCD * (eighth(short_blocks) + eighth(item_blocks) + eighth(tile_blocks))
                                       : xcd_grid(nblocks);
    bool launched = false;
    with_layout(s, [&](auto L) {
        using LT = decltype(L);
        constexpr int KU_ = LT::LPN * LT::UPL;
        if constexpr (!LT::LONG && LT::FULLK && !LT::WIDE && LT::U::ELEMS > 1 && (KU_ == 4 || KU_ == 8 || KU_ == 16 || KU_ == 32 || KU_ == 64)) {
            SDDMM_LAUNCH(c, (k_auto_tiles<LT, KU_ / 4>), grid, BLOCK,
                               (const void *)c->dA, (const void *)c->dB, s.KU, c->d_rowptr,
                               (const unsigned char *)(c->owner_active ? c->d_owner : nullptr), c->d_col, c->d_sval,
                               c->dP, c->sM, c->N, c->ts, c->rpw, short_blocks, c->d_items, c->n_items,
                               (const int32_t *)c->d_vrows, (const int32_t *)c->d_tile_cols,
                               (const TileDesc *)c->d_tiles, c->n_tiles,
                               (const TileWindow *)(c->use_windows ? c->d_windows : nullptr), c->n_windows, c->nnz,
                               tile_blocks, nblocks, (const int2 *)(c->use_short_list ? c->d_short_list : nullptr),
                               c->n_short_list, longest_first,
                               (const int32_t *)(c->use_win_order ? c->d_win_order : nullptr), c->n_win_single);
            launched = true;
        }
    });
    return launched;
}

void launch_auto(sddmm_ctx *c) {
    const Shape s = shape_of(c);
    const int64_t waves = short_row_waves(c);
    const int64_t short_blocks = (waves + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    const int64_t item_blocks = (c->n_items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    const int64_t nblocks = short_blocks + item_blocks;
    with_layout(s, [&](auto L) {
        using LT = decltype(L);
        SDDMM_LAUNCH(c, (k_auto<LT>), xcd_grid(nblocks), BLOCK,
                           (const void *)c->dA, (const void *)c->dB, s.KU, c->d_rowptr,
                           (const unsigned char *)(c->owner_active ? c->d_owner : nullptr), c->d_col, c->d_sval,
                           c->dP, c->sM, c->ts, c->rpw, short_blocks, c->d_items, c->n_items, nblocks,
                           (const int2 *)(c->use_short_list ? c->d_short_list : nullptr), c->n_short_list);
    });
}

// Row classifier: statistics, then the item list of the wave-per-segment kernel.
// Row classes and work items of the rows nobody owns, in two halves around a read-back of the
// counters: the count (launch only; it may be launched again after more rows found an owner) ...
int classify_rows_count(sddmm_ctx *c, bool again = false) {
    const int64_t nb = ((int64_t)c->sM + SCAN_TILE - 1) / SCAN_TILE;
    ARENA_HOLDS(c, nb, c->block_sums_cap, "block sums");
    // the first count of a plan finds its counters cleared (begin_ownership); a second one keeps what
    // validation and the ownership classifiers measured and clears the row classes
    if (again) {
        SDDMM_LAUNCH(c, k_plan_reset, 1, 256, c->d_owner, (int64_t)0, c->d_pc, 1);
        LAUNCH_CHECK(c);
    }
    if (nb > 0) {
        const unsigned char *owner = c->owner_active ? c->d_owner : nullptr;
        SDDMM_LAUNCH(c, k_classify_count, nb, SCAN_BLOCK, c->d_rowptr, owner,
                           c->sM, c->ts, c->seg, c->d_block_sums, c->d_pc, 0, c->d_short_sums);
        LAUNCH_CHECK(c);
        if (nb <= SCAN_SMALL_MAX) {
            int rc = queue_scan(c, c->d_block_sums, c->d_block_sums, nb, &c->d_pc->n_items);
            if (rc) return rc;
            rc = queue_scan(c, c->d_short_sums, c->d_short_sums, nb, &c->d_pc->short_scanned);
            if (rc) return rc;
        } else {
            SDDMM_LAUNCH(c, k_scan_block_sums, 1, SCAN_BLOCK, c->d_block_sums, (int)nb,
                               &c->d_pc->n_items);
            SDDMM_LAUNCH(c, k_scan_block_sums, 1, SCAN_BLOCK, c->d_short_sums, (int)nb,
                               &c->d_pc->short_scanned);
            LAUNCH_CHECK(c);
        }
    }
    return SDDMM_OK;
}
// ... and the items, once the counters are on the host (nothing may use the block sums in between)
int classify_rows_items(sddmm_ctx *c, bool with_short_list = true) {
    const int64_t nb = ((int64_t)c->sM + SCAN_TILE - 1) / SCAN_TILE;
    c->n_items = (int64_t)c->pc.n_items;
    c->rows_short = (int64_t)c->pc.rows_short;
    c->rpw = env_int("SDDMM_RPW", rows_per_wave(c->rows_short ? (double)c->pc.nnz_short / (double)c->rows_short : 0.0));
    c->rpw = std::min(64, std::max(1, c->rpw));
    if (c->n_items > c->items_cap) {
        dfree(c->d_items);
        ALLOC_TRY(c, c->d_items, (size_t)c->n_items * sizeof(RowItem));
        c->items_cap = c->n_items;
    }
    if (c->n_items > 0) {
        SDDMM_LAUNCH(c, k_classify_write, nb, SCAN_BLOCK, c->d_rowptr,
                           (const unsigned char *)(c->owner_active ? c->d_owner : nullptr), c->sM, c->ts, c->seg,
                           c->d_block_sums, c->d_items, 0);
        LAUNCH_CHECK(c);
    }
    // the entries of the short rows as a list, taken 64 at a time (entry_list_body)
    c->n_short_list = 0;
    c->use_short_list = with_short_list && env_int("SDDMM_SHORT_LIST", 1) != 0 && c->rows_short > 0;
    if (c->use_short_list) {
        c->n_short_list = (int64_t)c->pc.nnz_short;
        if ((int64_t)c->raw.short_scanned != c->n_short_list)
            return fail(c, SDDMM_ERR_HIP, "internal: scan of the short rows disagrees with their entry count");
        // The list is a convenience of 8 bytes per entry of a short row.  Above a cap
        // (SDDMM_SHORT_LIST_MAX entries, default 2^27 = 1 GiB), or when the device cannot
        // hold it, the launch walks the short rows themselves (short_rows_body) instead.
        const int64_t cap = (int64_t)env_int("SDDMM_SHORT_LIST_MAX", 1 << 27);
        if (c->n_short_list > cap) c->use_short_list = false;
        if (c->use_short_list && c->n_short_list > c->short_list_cap) {
            dfree(c->d_short_list);
            c->short_list_cap = 0;
            void *p = nullptr;
            if (hipMalloc(&p, (size_t)c->n_short_list * sizeof(int2)) == hipSuccess && p) {
                c->d_short_list = static_cast<decltype(c->d_short_list)>(p);
                c->short_list_cap = c->n_short_list;
            } else {
                (void)hipGetLastError();                       // the failed allocation is not an error of the plan
                c->use_short_list = false;
            }
        }
        if (!c->use_short_list) c->n_short_list = 0;
    }
    if (c->use_short_list) {
        SDDMM_LAUNCH(c, k_short_list_write, nb, SCAN_BLOCK, c->d_rowptr,
                           (const unsigned char *)(c->owner_active ? c->d_owner : nullptr), c->sM, c->ts,
                           (const unsigned int *)c->d_short_sums, c->d_short_list);
        LAUNCH_CHECK(c);
    }
    return SDDMM_OK;
}

// Exclusive scan of n unsigned ints on the device (in != out), total to *d_total.
int device_scan(sddmm_ctx *c, const unsigned int *in, unsigned int *out, int64_t n, unsigned long long *d_total) {
    if (n <= SCAN_SMALL_MAX) return queue_scan(c, in, out, n, d_total);
    {
        const int rc = flush_scans(c);             // (the long scan borrows the block sums)
        if (rc) return rc;
    }
    const int64_t nb = (n + SCAN_TILE - 1) / SCAN_TILE;
    ARENA_HOLDS(c, nb, c->block_sums_cap, "block sums");
    SDDMM_LAUNCH(c, k_scan_sums, nb, SCAN_BLOCK, in, n, c->d_block_sums);
    SDDMM_LAUNCH(c, k_scan_block_sums, 1, SCAN_BLOCK, c->d_block_sums, (int)nb, d_total);
    SDDMM_LAUNCH(c, k_scan_apply, nb, SCAN_BLOCK, in, n,
                       (const unsigned int *)c->d_block_sums, out);
    LAUNCH_CHECK(c);
    return SDDMM_OK;
}

// Clears the row-ownership bytes and the tile / panel counters before the classifiers run.
int begin_ownership(sddmm_ctx *c) {
    const int64_t bytes = (int64_t)c->sM + 64;
    const int arc = ensure_arena(c);
    if (arc) return arc;
    ARENA_HOLDS(c, bytes, c->owner_cap, "row owners");
    // one launch clears the owners and every counter of the classifiers, the row classes included
    SDDMM_LAUNCH(c, k_plan_reset, grid_for((bytes + 15) / 16, 256), 256, c->d_owner, bytes, c->d_pc, 0);
    LAUNCH_CHECK(c);
    c->owner_active = true;
    c->tiles_active = false;
    c->n_tiles = c->nnz_tiles = c->n_tiles_natural = c->n_tiles_union = c->nnz_tiles_union = 0;
    c->n_tiles_lead = c->n_win_single = c->n_tile_units = 0;
    c->n_cand = c->n_vstrips = 0;
    c->union_counted = false;
    c->n_panel_items = c->n_panels = c->nnz_panels = 0;
    return SDDMM_OK;
}

// Dense-tile classifier, in three steps so that the row panels can be looked for in
// between: (1) 16-row strips, (2) strips of rows gathered by column window among the
// rows nobody owns yet, (3) descriptors of both.  min_fill = average stored entries
// per 16x16 tile a strip needs to be taken.  tile_steps stays 0 when the path does not
// apply (row size not a multiple of 64 bytes).
bool tile_path_applies(sddmm_ctx *c) {
    c->tile_steps = 0;
    if (c->nnz == 0) return false;
    const size_t row_bytes = (size_t)c->K * elem_size(c->dtype);
    if (row_bytes % 64) return false;
    const int steps = (int)(row_bytes / 64);
    if (steps != 1 && steps != 2 && steps != 4 && steps != 8 && steps != 16) return false;
    c->tile_steps = steps;
    return true;
}

int plan_tiles_count(sddmm_ctx *c, int min_fill) {
    if (!tile_path_applies(c)) return SDDMM_OK;
    const int64_t n_strips = ((int64_t)c->sM + 15) / 16;
    ARENA_HOLDS(c, n_strips, c->strips_cap, "strips");
    const unsigned strip_grid = (unsigned)((n_strips + STRIPS_PER_BLOCK - 1) / STRIPS_PER_BLOCK);
    SDDMM_LAUNCH(c, k_strip_count, strip_grid, WAVE * STRIPS_PER_BLOCK, c->d_rowptr,
                       c->d_col, c->sM, n_strips, min_fill, c->d_strip_ntiles, c->d_owner, c->d_pc);
    LAUNCH_CHECK(c);
    return device_scan(c, c->d_strip_ntiles, c->d_strip_off, n_strips, &c->d_pc->tiles_scanned);
}

// after a fetch_counters that follows plan_tiles_count (and precedes the gathered strips)
int take_tile_counts(sddmm_ctx *c) {
    c->n_tiles = c->n_tiles_natural = (int64_t)c->pc.n_tiles;
    c->nnz_tiles = (int64_t)c->pc.nnz_tiles;
    if (c->tile_steps != 0 && (int64_t)c->pc.tiles_scanned != c->n_tiles)
        return fail(c, SDDMM_ERR_HIP, "internal: tile scan disagrees with tile count");
    c->n_tiles_union = c->union_counted ? (int64_t)c->pc.n_utiles : 0;
    c->nnz_tiles_union = c->union_counted ? (int64_t)c->pc.nnz_utiles : 0;
    if (c->union_counted && (int64_t)c->pc.utiles_scanned != c->n_tiles_union)
        return fail(c, SDDMM_ERR_HIP, "internal: union tile scan disagrees with tile count");
    c->n_tiles += c->n_tiles_union;
    c->nnz_tiles += c->nnz_tiles_union;
    return SDDMM_OK;
}

// Union strips among the 16-row strips nobody owns yet (launch only; after the panel
// detector, before the candidates of the gathered strips).
int plan_union_count(sddmm_ctx *c, int min_fill) {
    if (c->tile_steps == 0) return SDDMM_OK;
    const int64_t n_strips = ((int64_t)c->sM + 15) / 16;
    ARENA_HOLDS(c, n_strips, c->ustrips_cap, "union strips");
    const unsigned strip_grid = (unsigned)((n_strips + STRIPS_PER_BLOCK - 1) / STRIPS_PER_BLOCK);
    SDDMM_LAUNCH(c, k_union_count, strip_grid, WAVE * STRIPS_PER_BLOCK, c->d_rowptr,
                       c->d_col, c->sM, n_strips, min_fill, c->d_owner, c->d_ustrip_ntiles, c->d_pc);
    LAUNCH_CHECK(c);
    c->union_counted = true;
    return device_scan(c, c->d_ustrip_ntiles, c->d_ustrip_off, n_strips, &c->d_pc->utiles_scanned);
}

// Candidates of the gathered strips (launch only; the count arrives with the next
// fetch_counters).
int plan_gathered_candidates(sddmm_ctx *c, int min_len) {
    if (c->tile_steps == 0 || c->sM < 2) return SDDMM_OK;
    const int64_t M = c->sM;
    ARENA_HOLDS(c, M, c->cand_cap, "candidate rows");
    SDDMM_LAUNCH(c, k_gather_candidates, ((M + 255) / 256), 256, c->d_rowptr,
                       c->d_col, c->sM, (const unsigned char *)c->d_owner, min_len, c->d_cand_keys,
                       &c->d_pc->n_candidates);
    LAUNCH_CHECK(c);
    return SDDMM_OK;
}

// after the fetch_counters that follows plan_gathered_candidates
int plan_gathered_count(sddmm_ctx *c, int min_fill, bool *launched) {
    *launched = false;
    if (c->tile_steps == 0 || c->sM < 2) return SDDMM_OK;
    c->n_cand = (int64_t)c->raw.n_candidates;
    if (c->n_cand < 2) { c->n_cand = 0; return SDDMM_OK; }
    int rc;
    // candidates ordered by (first column, row): a few thousand by their ranks in one launch (4 us against 23 us
    // for the radix sort on 3 000 keys), more by the library's radix sort
    if (c->n_cand <= RANK_SORT_MAX && env_int("SDDMM_RANK_SORT", 1) != 0) {
        constexpr int per_block = RANK_SORT_BLOCK / RANK_SORT_SPLIT;
        SDDMM_LAUNCH(c, k_rank_sort, (unsigned)((c->n_cand + per_block - 1) / per_block), RANK_SORT_BLOCK,
                           (const unsigned long long *)c->d_cand_keys, (unsigned long long *)c->d_sorted_keys, (int)c->n_cand);
        LAUNCH_CHECK(c);
    } else {
        size_t need = 0;
        HIP_TRY(c, rocprim::radix_sort_keys(nullptr, need, c->d_cand_keys, c->d_sorted_keys, (size_t)c->n_cand, 0, 64,
                                            c->stream));
        if (need > c->sort_tmp_bytes) {
            dfree(c->d_sort_tmp);
            ALLOC_TRY(c, c->d_sort_tmp, need);
            c->sort_tmp_bytes = need;
        }
        HIP_TRY(c, rocprim::radix_sort_keys(c->d_sort_tmp, need, c->d_cand_keys, c->d_sorted_keys, (size_t)c->n_cand, 0, 64,
                                            c->stream));
    }
    // pairs of strips: 32 consecutive candidates share one list of tile columns
    const int64_t n_vpairs = (c->n_cand + 31) / 32;
    c->n_vstrips = 2 * n_vpairs;
    ARENA_HOLDS(c, c->n_vstrips, c->vstrips_cap, "gathered strips");
    SDDMM_LAUNCH(c, k_gathered_count, n_vpairs, GATHERED_BLOCK, c->d_rowptr, c->d_col,
                       (const unsigned long long *)c->d_sorted_keys, c->n_cand, n_vpairs, min_fill, c->d_vstrip_ntiles,
                       c->d_vrows, c->d_owner, c->d_pc);
    LAUNCH_CHECK(c);
    rc = device_scan(c, c->d_vstrip_ntiles, c->d_vstrip_off, c->n_vstrips, &c->d_pc->tiles_scanned);
    if (rc) return rc;
    *launched = true;
    return SDDMM_OK;
}
// after the counters came back
int plan_gathered_take(sddmm_ctx *c) {
    const int64_t gathered = (int64_t)c->pc.n_tiles - c->n_tiles_natural;
    if ((int64_t)c->pc.tiles_scanned != gathered)
        return fail(c, SDDMM_ERR_HIP, "internal: gathered tile scan disagrees with tile count");
    // the gathered descriptors start a window of their own: the strips before them are padded
    // to a multiple of TILE_WINDOW with descriptors that stand for nothing
    const int64_t before = c->n_tiles_natural + c->n_tiles_union;
    c->n_tiles_lead = gathered > 0 ? (TILE_WINDOW - before % TILE_WINDOW) % TILE_WINDOW : 0;
    c->n_tiles = before + c->n_tiles_lead + gathered;
    c->nnz_tiles = (int64_t)c->pc.nnz_tiles + c->nnz_tiles_union;
    return SDDMM_OK;
}

// When the storage order of the windows (strip by strip) makes every XCD touch more of A and B
// than its L2 holds, the launch takes them block by block of a RB x CB grid over (strips, tile
// columns), one block per XCD (k_window_histogram and following).
int plan_window_order(sddmm_ctx *c) {
    c->use_win_order = false;
    const int mode = env_int("SDDMM_WINDOW_ORDER", -1);          // -1: decide here, 0: never, 1: always
    const double row_bytes = (double)c->K * (double)elem_size(c->dtype);
    const double a_bytes = (double)c->sM * row_bytes, b_bytes = (double)c->N * row_bytes;
    const double l2 = 4.0 * 1024 * 1024;
    // storage order: an XCD has an eighth of the strips and, over the launch, all of B
    if (mode == 0 || c->n_windows < 8 * NUM_XCD) return SDDMM_OK;
    // (gathered strips come sorted by column window already: reordering them measured 12 % slower)
    if (mode < 0 && c->n_tiles != c->n_tiles_natural) return SDDMM_OK;
    if (mode < 0 && a_bytes / NUM_XCD + b_bytes <= 0.75 * l2) return SDDMM_OK;
    // resident part of A per XCD within half an L2, then the least traffic A * CB + B * RB
    int RB = NUM_XCD, CB = 1;
    double best = -1.0;
    for (int rb = 1; rb <= NUM_XCD; rb *= 2) {
        const int cb = NUM_XCD / rb;
        const double traffic = a_bytes * cb + b_bytes * rb;
        const bool fits = a_bytes / rb <= 0.6 * l2;
        if (!fits && rb != NUM_XCD) continue;
        if (best < 0 || traffic < best) { best = traffic; RB = rb; CB = cb; }
    }
    if (c->n_windows > c->win_order_cap) {
        dfree(c->d_win_order);
        c->win_order_cap = 0;
        ALLOC_TRY(c, c->d_win_order, (size_t)c->n_windows * sizeof(int32_t));
        c->win_order_cap = c->n_windows;
    }
    if (!c->d_win_bins) ALLOC_TRY(c, c->d_win_bins, (size_t)WINDOW_BINS * sizeof(unsigned int));
    HIP_TRY(c, hipMemsetAsync(c->d_win_bins, 0, (size_t)WINDOW_BINS * sizeof(unsigned int), c->stream));
    const int64_t strip_span = std::max<int64_t>(1, std::max(((int64_t)c->sM + 15) / 16, c->n_vstrips));
    const int64_t tile_col_span = std::max<int64_t>(1, ((int64_t)c->N + 15) / 16);
    const unsigned grid = (unsigned)((c->n_windows + 255) / 256);
    SDDMM_LAUNCH(c, k_window_histogram, grid, 256, (const TileDesc *)c->d_tiles, c->n_windows, strip_span, tile_col_span,
                       RB, CB, c->d_win_bins);
    SDDMM_LAUNCH(c, k_window_offsets, 1, WINDOW_BINS, c->d_win_bins);
    SDDMM_LAUNCH(c, k_window_scatter, grid, 256, (const TileDesc *)c->d_tiles, c->n_windows, strip_span, tile_col_span,
                       RB, CB, c->d_win_bins, c->d_win_order);
    LAUNCH_CHECK(c);
    c->use_win_order = true;
    return SDDMM_OK;
}

int plan_tiles_fill(sddmm_ctx *c) {
    if (c->n_tiles == 0) return SDDMM_OK;
    if (c->n_tiles > c->tiles_cap) {
        dfree(c->d_tiles);
        dfree(c->d_tile_cols);
        c->tiles_cap = 0;
        ALLOC_TRY(c, c->d_tiles, (size_t)c->n_tiles * sizeof(TileDesc));
        ALLOC_TRY(c, c->d_tile_cols, (size_t)c->n_tiles * 16 * sizeof(int32_t));
        c->tiles_cap = c->n_tiles;
    }
    if (c->n_tiles_natural > 0) {
        const int64_t n_strips = ((int64_t)c->sM + 15) / 16;
        const unsigned strip_grid = (unsigned)((n_strips + STRIPS_PER_BLOCK - 1) / STRIPS_PER_BLOCK);
        SDDMM_LAUNCH(c, k_strip_tiles, strip_grid, WAVE * STRIPS_PER_BLOCK, c->d_rowptr,
                           c->d_col, c->sM, n_strips, c->d_strip_ntiles, c->d_strip_off, c->d_tiles, c->d_tile_cols);
        LAUNCH_CHECK(c);
    }
    if (c->n_tiles_union > 0) {
        const int64_t n_strips = ((int64_t)c->sM + 15) / 16;
        const unsigned strip_grid = (unsigned)((n_strips + STRIPS_PER_BLOCK - 1) / STRIPS_PER_BLOCK);
        SDDMM_LAUNCH(c, k_union_tiles, strip_grid, WAVE * STRIPS_PER_BLOCK, c->d_rowptr,
                           c->d_col, c->sM, n_strips, c->d_ustrip_ntiles, c->d_ustrip_off,
                           c->d_tiles + c->n_tiles_natural, c->d_tile_cols + c->n_tiles_natural * 16);
        LAUNCH_CHECK(c);
    }
    const int64_t gathered_lo = c->n_tiles_natural + c->n_tiles_union + c->n_tiles_lead;
    if (c->n_tiles > gathered_lo) {
        SDDMM_LAUNCH(c, k_gathered_tiles, c->n_vstrips / 2, GATHERED_BLOCK, c->d_rowptr,
                           c->d_col, (const unsigned long long *)c->d_sorted_keys, c->n_cand, c->n_vstrips / 2,
                           c->d_vstrip_ntiles, c->d_vstrip_off, c->d_tiles + gathered_lo,
                           c->d_tile_cols + gathered_lo * 16, (int)c->n_tiles_lead);
        LAUNCH_CHECK(c);
    }
    SDDMM_LAUNCH(c, k_tile_rows, ((c->n_tiles * 16 + 255) / 256), 256,
                       c->d_rowptr, c->d_col, c->sM, (const int32_t *)c->d_vrows, (const int32_t *)c->d_tile_cols,
                       c->d_tiles, c->n_tiles);
    LAUNCH_CHECK(c);
    // windows of TILE_WINDOW descriptors: what a wavefront of the tile kernels takes.  As a batch
    // (one access per run of a row's entries, which costs reading the column indices) where the
    // tiles are sparsely filled; tile by tile from the descriptors' masks where they are nearly
    // full (measured: 92 entries per tile 12.8 -> 11.3 us as batches, 256 per tile 8.5 -> 9.4 us)
    c->n_windows = (c->n_tiles + TILE_WINDOW - 1) / TILE_WINDOW;
    {
        const int rc = plan_window_order(c);
        if (rc) return rc;
    }
    c->use_windows = c->nnz_tiles < (int64_t)env_int("SDDMM_WINDOW_FILL", 176) * c->n_tiles;
    // wavefronts of a tile launch: one per window, and one per two windows of a pair of gathered strips
    // (their descriptors come last and fill whole windows, an even number of them)
    c->n_win_single = c->n_windows;
    // (rows of up to 256 bytes: beyond that the second A panel and the kept products do not fit the registers)
    if (c->use_windows && c->n_tiles > gathered_lo && c->tile_steps <= PAIR_MAX_STEPS && env_int("SDDMM_PAIRS", 1) != 0)
        c->n_win_single = gathered_lo / TILE_WINDOW;
    c->n_tile_units = c->n_win_single + (c->n_windows - c->n_win_single + 1) / 2;
    if (!c->use_windows) {
        c->tiles_active = true;
        return SDDMM_OK;
    }
    if (c->n_windows > c->windows_cap) {
        dfree(c->d_windows);
        c->windows_cap = 0;
        ALLOC_TRY(c, c->d_windows, (size_t)c->n_windows * sizeof(TileWindow));
        c->windows_cap = c->n_windows;
    }
    SDDMM_LAUNCH(c, k_tile_windows, ((c->n_windows * 16 + 255) / 256), 256, (const int32_t *)c->d_vrows, c->sM,
                       c->nnz, (const TileDesc *)c->d_tiles, c->n_tiles, c->n_tiles_natural,
                       c->n_tiles_natural + c->n_tiles_union, c->n_tiles > gathered_lo ? gathered_lo : c->n_tiles,
                       c->d_windows, c->n_windows);
    LAUNCH_CHECK(c);
    c->tiles_active = true;
    return SDDMM_OK;
}

// Row-panel detector (8 consecutive rows, 8-aligned, same column list).  Two
// kernels can run the panels: the MFMA one (row size a multiple of 64 bytes, up to
// 1 KiB) and the VALU one (8-lanes-per-entry layouts whose 8 A rows fit in
// registers: fp32 K = 32 or 64, bf16 / fp16 K = 64, 32-bit offsets); the VALU kernel has
// the per-entry arithmetic of the gather kernels, the MFMA kernel is faster.
int panel_mfma_steps(const sddmm_ctx *c) {
    const size_t row_bytes = (size_t)c->K * elem_size(c->dtype);
    if (row_bytes % 64) return 0;
    const int steps = (int)(row_bytes / 64);
    return (steps == 1 || steps == 2 || steps == 4 || steps == 8 || steps == 16) ? steps : 0;
}
bool panel_valu_applicable(const sddmm_ctx *c) {
    const Shape s = shape_of(c);
    if (s.unit == 1 || s.LPN != 8 || !s.fullk || s.wide) return false;
    return s.unit == 0 ? s.UPL <= 2 : s.UPL == 1;
}

// panel detector (launch only) / panel items (after the next fetch_counters)
int plan_panels_flags(sddmm_ctx *c, int min_len, int pseg) {
    c->panels_flagged = false;
    if (c->nnz == 0) return SDDMM_OK;
    c->panel_mfma = panel_mfma_steps(c) != 0 && env_int("SDDMM_PANEL_MFMA", 1) != 0;
    if (!c->panel_mfma && !panel_valu_applicable(c)) return SDDMM_OK;
    if (c->panel_mfma) min_len = std::max(min_len, 4);   // 16-byte S/P accesses stay inside a row
    const int64_t n_panels = (int64_t)c->sM / 8;
    if (n_panels == 0) return SDDMM_OK;
    ARENA_HOLDS(c, n_panels, c->panels_cap, "panels");
    SDDMM_LAUNCH(c, k_panel_flags, ((n_panels * WAVE + 255) / 256), 256,
                       c->d_rowptr, c->d_col, c->sM, n_panels, min_len, pseg, c->d_owner, c->d_panel_counts, c->d_pc);
    LAUNCH_CHECK(c);
    c->panels_flagged = true;
    return device_scan(c, c->d_panel_counts, c->d_panel_off, n_panels, &c->d_pc->panel_items);
}

int plan_panels_items(sddmm_ctx *c, int pseg) {
    if (!c->panels_flagged) return SDDMM_OK;
    const int64_t n_panels = (int64_t)c->sM / 8;
    c->n_panels = (int64_t)c->pc.n_panels;
    c->nnz_panels = (int64_t)c->pc.nnz_panels;
    c->n_panel_items = (int64_t)c->pc.panel_items;
    if (c->n_panel_items == 0) return SDDMM_OK;
    if (c->n_panel_items > c->panel_items_cap) {
        dfree(c->d_panel_items);
        ALLOC_TRY(c, c->d_panel_items, (size_t)c->n_panel_items * sizeof(RowItem));
        c->panel_items_cap = c->n_panel_items;
    }
    SDDMM_LAUNCH(c, k_panel_items, ((n_panels + 255) / 256), 256, c->d_rowptr,
                       n_panels, pseg, (const unsigned int *)c->d_panel_counts, (const unsigned int *)c->d_panel_off,
                       c->d_panel_items);
    LAUNCH_CHECK(c);
    return SDDMM_OK;
}

template <class U, int UPL>
void launch_panel_t(sddmm_ctx *c, int KU) {
    using LT = Layout<U, 8, UPL, true, false>;
    const int64_t nblocks = (c->n_panel_items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    SDDMM_LAUNCH(c, (k_panel<LT>), xcd_grid(nblocks), BLOCK,
                       (const void *)c->dA, (const void *)c->dB, KU, c->d_rowptr, c->d_col, c->d_sval, c->dP,
                       (const RowItem *)c->d_panel_items, c->n_panel_items, nblocks);
}
template <class U>
void launch_panel_u(sddmm_ctx *c, const Shape &s) {
    if (s.UPL == 1) launch_panel_t<U, 1>(c, s.KU);
    else launch_panel_t<U, 2>(c, s.KU);
}
template <int DT, int STEPS>
void launch_panel_mfma_t(sddmm_ctx *c) {
    constexpr int PW = panel_mfma_waves(STEPS);
    const int64_t nblocks = (c->n_panel_items + PW - 1) / PW;
    SDDMM_LAUNCH(c, (k_panel_mfma<DT, STEPS>), xcd_grid(nblocks), PW * WAVE,
                       (const void *)c->dA, (const void *)c->dB, c->d_rowptr, c->d_col, (const float *)c->d_sval,
                       c->dP, (const RowItem *)c->d_panel_items, c->n_panel_items, nblocks, (float *)nullptr);
}
// the panels of the fused SDDMM+SpMM: P and the panels' part of O
template <int DT, int STEPS>
void launch_panel_fused_t(sddmm_ctx *c) {
    constexpr int PW = panel_mfma_waves(STEPS);
    const int64_t nblocks = (c->n_panel_items + PW - 1) / PW;
    SDDMM_LAUNCH(c, (k_panel_mfma<DT, STEPS, true>), xcd_grid(nblocks), PW * WAVE,
                       (const void *)c->dA, (const void *)c->dB, c->d_rowptr, c->d_col, (const float *)c->d_sval,
                       c->dP, (const RowItem *)c->d_panel_items, c->n_panel_items, nblocks, c->dO);
}
template <int DT>
void launch_panel_mfma_steps(sddmm_ctx *c) {
    switch (panel_mfma_steps(c)) {
        case 1: launch_panel_mfma_t<DT, 1>(c); break;
        case 2: launch_panel_mfma_t<DT, 2>(c); break;
        case 4: launch_panel_mfma_t<DT, 4>(c); break;
        case 8: launch_panel_mfma_t<DT, 8>(c); break;
        default: launch_panel_mfma_t<DT, 16>(c); break;
    }
}

void launch_panels(sddmm_ctx *c) {
    if (c->panel_mfma) {
        if (c->dtype == SDDMM_BF16) launch_panel_mfma_steps<DT_BF16>(c);
        else if (c->dtype == SDDMM_F16) launch_panel_mfma_steps<DT_F16>(c);
        else launch_panel_mfma_steps<DT_F32>(c);
        return;
    }
    const Shape s = shape_of(c);
    if (s.unit == 0) launch_panel_u<UnitF32x4>(c, s);
    else if (s.unit == 2) launch_panel_t<UnitBF16x8, 1>(c, s.KU);
    else launch_panel_t<UnitF16x8, 1>(c, s.KU);
}

template <int DT, int STEPS>
void launch_tile_t(sddmm_ctx *c) {
    // Well-filled tiles (walked from the descriptors' masks) of rows of 256 bytes and more, fewer
    // windows than keep the chip busy on their own: one workgroup per window, K in four parts.
    if constexpr (STEPS % KSPLIT == 0) {
        if (!c->use_windows && c->n_windows <= (int64_t)env_int("SDDMM_KSPLIT_MAX", 32768) && env_int("SDDMM_KSPLIT", 1) != 0) {
            const int64_t nb = c->n_windows;
            SDDMM_LAUNCH(c, (k_tile_ksplit<DT, STEPS>), xcd_grid(nb), BLOCK,
                               (const void *)c->dA, (const void *)c->dB, c->M, c->N, (const int32_t *)c->d_vrows,
                               (const int32_t *)c->d_tile_cols, (const TileDesc *)c->d_tiles, c->n_tiles,
                               (const float *)c->d_sval, c->dP, nb,
                               (const int32_t *)(c->use_win_order ? c->d_win_order : nullptr));
            return;
        }
    }
    const int64_t nblocks = (c->n_tile_units + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
    SDDMM_LAUNCH(c, (k_tile<DT, STEPS>), xcd_grid(nblocks), BLOCK,
                       (const void *)c->dA, (const void *)c->dB, c->M, c->N, (const int32_t *)c->d_vrows,
                       (const int32_t *)c->d_tile_cols, (const TileDesc *)c->d_tiles, c->n_tiles,
                       (const TileWindow *)(c->use_windows ? c->d_windows : nullptr), c->n_windows,
                       (const int32_t *)c->d_col, (const float *)c->d_sval, c->dP, c->nnz, nblocks,
                       (const int32_t *)(c->use_win_order ? c->d_win_order : nullptr), c->n_win_single);
}
template <int DT>
void launch_tile_steps(sddmm_ctx *c) {
    switch (c->tile_steps) {
        case 1: launch_tile_t<DT, 1>(c); break;
        case 2: launch_tile_t<DT, 2>(c); break;
        case 4: launch_tile_t<DT, 4>(c); break;
        case 8: launch_tile_t<DT, 8>(c); break;
        default: launch_tile_t<DT, 16>(c); break;
    }
}
void launch_tiles(sddmm_ctx *c) {
    if (c->dtype == SDDMM_BF16) launch_tile_steps<DT_BF16>(c);
    else if (c->dtype == SDDMM_F16) launch_tile_steps<DT_F16>(c);
    else launch_tile_steps<DT_F32>(c);
}

int ensure_rowidx(sddmm_ctx *c) {
    if (c->d_rowidx) return SDDMM_OK;
    ALLOC_TRY(c, c->d_rowidx, (size_t)c->nnz * sizeof(int32_t));
    c->own_rowidx = true;
    if (c->sM > 0 && c->nnz > 0)
        SDDMM_LAUNCH(c, k_expand_rows, grid_for(c->sM, 256), 256, c->d_rowptr, c->sM,
                           c->d_rowidx, c->nnz);
    LAUNCH_CHECK(c);
    return SDDMM_OK;
}

// Validate the device-resident CSR and gather row statistics.
int validate_csr(sddmm_ctx *c) {
    HIP_TRY(c, hipMemsetAsync(c->d_pc, 0, sizeof(DevCounters), c->stream));
    if (c->sM > 0)
        SDDMM_LAUNCH(c, k_check_rowptr, grid_for(c->sM, 256), 256, c->d_rowptr, c->sM,
                           c->nnz, c->d_pc);
    LAUNCH_CHECK(c);
    int rc = fetch_counters(c);
    if (rc) return rc;
    if (c->pc.bad_pattern) return fail(c, SDDMM_ERR_PATTERN, "rowptr is not a valid CSR row pointer array");
    // only now is it safe to walk col[0..nnz)
    if (c->nnz > 0) {
        SDDMM_LAUNCH(c, k_check_index, grid_capped(c->nnz, 256), 256, c->d_col, c->nnz,
                           c->sN, c->d_pc);
        LAUNCH_CHECK(c);
        rc = fetch_counters(c);
        if (rc) return rc;
        if (c->pc.bad_pattern) return fail(c, SDDMM_ERR_PATTERN, "column index outside [0,N)");
    }
    return SDDMM_OK;
}

int check_dims(sddmm_ctx *c, int M, int N, int64_t nnz) {
    if (M < 0 || N < 0 || nnz < 0) return fail(c, SDDMM_ERR_INVALID, "negative dimension");
    if (nnz > 0 && (M == 0 || N == 0)) return fail(c, SDDMM_ERR_INVALID, "entries in an empty matrix");
    // positions are 32-bit like the reference's row pointers; the kernels look up to a few chunks
    // past a position before clamping, so the last 64 Ki values stay unused
    if (nnz > (int64_t)INT32_MAX - 65536) return fail(c, SDDMM_ERR_INVALID, "nnz exceeds 32-bit row pointers");
    return SDDMM_OK;
}

int enqueue_run(sddmm_ctx *c) {
    c->launches = 0;
    if (c->nnz == 0) return SDDMM_OK;
    c->launches = 1;
    switch (c->strategy) {
        case SDDMM_AUTO:
        case SDDMM_MFMA_TILE:
        case SDDMM_LDS_TILED: {
            // (a second stream for the first of these independent kernels was measured:
            // the fork/join events cost more than the overlap returns, 33 us against 23 us
            // on the mixed-density shape)
            c->launches = 0;
            const bool tiles = c->tiles_active && c->n_tiles > 0, rows = c->rows_short > 0 || c->n_items > 0;
            bool fused = false;
            if (tiles && rows && env_int("SDDMM_FUSE", 1) != 0) fused = launch_auto_with_tiles(c);
            if (fused) ++c->launches;
            if (tiles && !fused) { launch_tiles(c); ++c->launches; }
            if (c->n_panel_items > 0) { launch_panels(c); ++c->launches; }
            if (rows && !fused) { launch_auto(c); ++c->launches; }
            break;
        }
        case SDDMM_FLAT: launch_flat(c); break;
        case SDDMM_ROW_WAVE: launch_row_wave(c, nullptr, c->sM); break;
        case SDDMM_SHORT_ROWS:
            launch_short_rows(c, INT32_MAX, rows_per_wave(c->sM ? (double)c->nnz / c->sM : 0.0));
            break;
        case SDDMM_EXACT:
            if (c->dtype == SDDMM_BF16)
                SDDMM_LAUNCH(c, k_exact<DT_BF16>, grid_for(c->nnz, BLOCK), BLOCK, c->dA,
                                   c->dB, c->K, c->d_rowidx, c->d_col, c->d_sval, c->dP, c->nnz);
            else if (c->dtype == SDDMM_F16)
                SDDMM_LAUNCH(c, k_exact<DT_F16>, grid_for(c->nnz, BLOCK), BLOCK, c->dA,
                                   c->dB, c->K, c->d_rowidx, c->d_col, c->d_sval, c->dP, c->nnz);
            else
                SDDMM_LAUNCH(c, k_exact<DT_F32>, grid_for(c->nnz, BLOCK), BLOCK, c->dA,
                                   c->dB, c->K, c->d_rowidx, c->d_col, c->d_sval, c->dP, c->nnz);
            break;
        default: return fail(c, SDDMM_ERR_STATE, "no kernel for strategy %d", c->strategy);
    }
    LAUNCH_CHECK(c);
    c->stats.kernels_launched = c->launches;
    return SDDMM_OK;
}

int do_plan(sddmm_ctx *c, int strategy) {
    // the plan state is rewritten in place: a plan that fails half way must not leave the
    // previous one looking valid (its items exclude rows that tiles and panels owned)
    c->planned = false;
    c->n_scan_jobs = 0;
    c->fused_items_valid = false;    // they leave out the rows of this plan's panels
    int resolved = strategy;
    const bool csr_ok = c->have_rowptr;
    // without a row pointer (unsorted COO) only the flat kernels apply
    if (strategy == SDDMM_AUTO && !csr_ok) resolved = SDDMM_FLAT;
    switch (resolved) {
        case SDDMM_AUTO:
        case SDDMM_MFMA_TILE:
        case SDDMM_LDS_TILED: {
            // Row ownership in this order: well-filled 16-row strips go to the MFMA tile
            // path, then 8-row panels with a common column list to the panel kernel, the
            // rest is split by length.  MFMA_TILE takes every sorted strip and no panel,
            // LDS_TILED every panel and no strip; AUTO applies the thresholds.
            if (!csr_ok) return fail(c, SDDMM_ERR_UNSUPPORTED, "strategy %d needs row-sorted entries", resolved);
            int rc = begin_ownership(c);
            if (rc) return rc;
            // entries per 16x16 tile from which the tile kernel beats the gather kernels,
            // measured on banded matrices of varying fill: 74 at 128-byte rows, 50 at 256
            // and 512 bytes; 64-byte rows keep the older, conservative figure
            const size_t row_bytes = (size_t)c->K * elem_size(c->dtype);
            const int tile_fill = std::max(1, env_int("SDDMM_TILE_FILL", row_bytes <= 64 ? 96 : row_bytes <= 128 ? 80 : 56));
            const int pseg = std::max(WAVE, env_int("SDDMM_PANEL_SEG", 512));
            const bool gathered = resolved == SDDMM_AUTO && env_int("SDDMM_GATHERED", 1) != 0;
            c->tile_steps = 0;
            // the classifiers are launched back to back; their totals come back together
            if (resolved != SDDMM_LDS_TILED) {
                // 16-row strips are looked at before the row panels and must not take what the
                // panel kernel does better (8x8-block rows reach ~80 entries per tile); the
                // strips gathered after the panels use the measured break-even
                rc = plan_tiles_count(c, resolved == SDDMM_MFMA_TILE ? 1 : std::max(96, tile_fill));
                if (rc) return rc;
            }
            if (resolved != SDDMM_MFMA_TILE) {
                rc = plan_panels_flags(c, resolved == SDDMM_LDS_TILED ? 1 : std::max(1, env_int("SDDMM_PANEL_MIN", 16)), pseg);
                if (rc) return rc;
            } else {
                c->panels_flagged = false;
            }
            if (resolved == SDDMM_AUTO && env_int("SDDMM_UNION", 1) != 0) {
                rc = plan_union_count(c, std::max(1, env_int("SDDMM_UNION_FILL", tile_fill)));
                if (rc) return rc;
            }
            if (gathered) {
                rc = plan_gathered_candidates(c, std::max(16, env_int("SDDMM_GATHERED_MIN", 64)));
                if (rc) return rc;
            }
            // the rows nobody owns so far are classified in the same batch: most matrices have
            // no gathered strips, and their plan then waits for the device once
            c->ts = std::max(1, env_int("SDDMM_TS", 24));
            // segment items of 256 entries: a wavefront walks its item chunk by chunk, one dependent
            // round trip each, so a few long items set the duration of a short launch (eight rows of
            // 554 entries as single items: 17.5 us on the mixed-density shape, 14.6 us in pieces of
            // 256); on a matrix of 36 M entries pieces of 128..2048 differ by 3 %
            c->seg = std::max(WAVE, env_int("SDDMM_SEG", 256));
            rc = classify_rows_count(c);
            if (rc) return rc;
            rc = fetch_counters(c);
            if (rc) return rc;
            rc = take_tile_counts(c);
            if (rc) return rc;
            rc = plan_panels_items(c, pseg);
            if (rc) return rc;
            if (gathered) {
                bool launched = false;
                // (gathered strips come in pairs that share every B tile they load: a tile pays for
                // itself at three quarters of the entries a tile of a lone strip needs)
                rc = plan_gathered_count(c, std::max(1, env_int("SDDMM_GATHERED_FILL", tile_fill * 3 / 4)), &launched);
                if (rc) return rc;
                if (launched) {
                    // gathered strips may have taken rows: classify again, one more read-back
                    rc = classify_rows_count(c, true);
                    if (rc) return rc;
                    rc = fetch_counters(c);
                    if (rc) return rc;
                    rc = plan_gathered_take(c);
                    if (rc) return rc;
                }
            }
            if (resolved != SDDMM_LDS_TILED) {
                rc = plan_tiles_fill(c);
                if (rc) return rc;
            }
            // A matrix whose rows are short on average (fewer than 32 entries per non-empty
            // row), with no strip or panel taken, is a flat stream of entries: the flat
            // kernel (row index per entry, perfectly balanced) measured 6 % faster there than
            // the row split (power-law shape, K=32: 634 us against 672 us).
            const double avg_len = c->pc.rows_nonempty ? (double)c->nnz / (double)c->pc.rows_nonempty : 0.0;
            const bool flat = resolved == SDDMM_AUTO && c->n_tiles == 0 && c->n_panel_items == 0 &&
                              avg_len < (double)env_int("SDDMM_FLAT_AVG", 32);
            rc = classify_rows_items(c, !flat);      // (the flat kernel has no use for the entry list of the short rows)
            if (rc) return rc;
            if (flat) {
                rc = ensure_rowidx(c);
                if (rc) return rc;
                resolved = SDDMM_FLAT;
            }
            break;
        }
        case SDDMM_FLAT:
        case SDDMM_EXACT: {
            int rc = ensure_rowidx(c);
            if (rc) return rc;
            break;
        }
        case SDDMM_ROW_WAVE:
        case SDDMM_SHORT_ROWS:
            if (!csr_ok) return fail(c, SDDMM_ERR_UNSUPPORTED, "strategy %d needs row-sorted entries", resolved);
            break;
        default: return fail(c, SDDMM_ERR_INVALID, "unknown strategy %d", strategy);
    }
    c->requested = strategy;
    c->strategy = resolved;
    c->planned = true;
    return SDDMM_OK;
}

void fill_model(sddmm_ctx *c) {
    sddmm_stats &s = c->stats;
    s.strategy_used = c->strategy;
    s.nnz = c->nnz;
    s.rows_nonempty = (int64_t)c->pc.rows_nonempty;
    if (c->strategy == SDDMM_AUTO || c->strategy == SDDMM_MFMA_TILE || c->strategy == SDDMM_LDS_TILED) {
        s.mfma_tiles = c->tiles_active ? c->n_tiles : 0;
        s.nnz_mfma = c->tiles_active ? c->nnz_tiles : 0;
        s.panels = c->n_panels;
        s.nnz_panel = c->nnz_panels;
        s.rows_short = (int64_t)c->pc.rows_short; s.rows_medium = (int64_t)c->pc.rows_medium;
        s.rows_long = (int64_t)c->pc.rows_long;
        s.nnz_short = (int64_t)c->pc.nnz_short; s.nnz_medium = (int64_t)c->pc.nnz_medium;
        s.nnz_long = (int64_t)c->pc.nnz_long;
    }
    const double e = (double)elem_size(c->dtype);
    s.flops = 2.0 * (double)c->nnz * (double)c->K;
    s.bytes_gathered = 4.0 * ((double)c->sM + 1.0) + 12.0 * (double)c->nnz +
                       e * (double)c->K * (double)s.rows_nonempty + e * (double)c->K * (double)c->nnz;
}

}  // namespace

// ===========================================================================
extern "C" {

const char *sddmm_version(void) { return "sddmm_amd 0.1 (gfx950, wave64)"; }

const char *sddmm_strerror(int code) {
    switch (code) {
        case SDDMM_OK: return "ok";
        case SDDMM_ERR_INVALID: return "invalid argument";
        case SDDMM_ERR_NULL: return "null pointer";
        case SDDMM_ERR_STATE: return "operands or plan missing";
        case SDDMM_ERR_ALLOC: return "allocation failed";
        case SDDMM_ERR_HIP: return "HIP runtime error";
        case SDDMM_ERR_UNSUPPORTED: return "strategy not applicable";
        case SDDMM_ERR_NO_DEVICE: return "no usable HIP device";
        case SDDMM_ERR_PATTERN: return "malformed sparse structure";
        case SDDMM_ERR_TOO_LARGE:
            return "more stored entries than the static scratch buffer of sddmm_launch_noalloc holds "
                   "(SDDMM_NOALLOC_MAX_NNZ)";
        default: return "unknown error";
    }
}

const char *sddmm_last_error(const sddmm_ctx *ctx) { return ctx ? ctx->err : ""; }

int sddmm_create(sddmm_ctx **out, int device) {
    if (!out) return SDDMM_ERR_NULL;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) return SDDMM_ERR_NO_DEVICE;
    if (device < 0 || device >= count) return SDDMM_ERR_INVALID;
    if (hipSetDevice(device) != hipSuccess) return SDDMM_ERR_NO_DEVICE;
    sddmm_ctx *c = new (std::nothrow) sddmm_ctx();
    if (!c) return SDDMM_ERR_ALLOC;
    c->device = device;
    if (hipStreamCreate(&c->own_stream) != hipSuccess || hipEventCreate(&c->ev0) != hipSuccess ||
        hipEventCreate(&c->ev1) != hipSuccess || hipMalloc((void **)&c->d_pc, sizeof(DevCounters)) != hipSuccess ||
        hipHostMalloc((void **)&c->h_pc, sizeof(DevCounters), hipHostMallocDefault) != hipSuccess) {
        sddmm_destroy(c);
        return SDDMM_ERR_HIP;
    }
    c->stream = c->own_stream;
    *out = c;
    return SDDMM_OK;
}

int sddmm_set_stream(sddmm_ctx *c, void *stream, int lent) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    // nothing of this context may still be in flight on the stream it leaves
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    c->lent_stream = lent != 0;
    c->stream = c->lent_stream ? (hipStream_t)stream : c->own_stream;
    return SDDMM_OK;
}

int sddmm_get_stream(const sddmm_ctx *c, void **stream) {
    if (!c || !stream) return SDDMM_ERR_NULL;
    *stream = (void *)c->stream;
    return SDDMM_OK;
}

void sddmm_destroy(sddmm_ctx *c) {
    if (!c) return;
    (void)hipSetDevice(c->device);
    if (c->own_stream) (void)hipStreamSynchronize(c->stream);
    release_dense(c);
    release_sparse(c);
    dfree(c->dO);
    dfree(c->d_pc);
    if (c->h_pc) (void)hipHostFree(c->h_pc);
    if (c->ev0) (void)hipEventDestroy(c->ev0);
    if (c->ev1) (void)hipEventDestroy(c->ev1);
    if (c->own_stream) (void)hipStreamDestroy(c->own_stream);
    delete c;
}

static int set_dense_common(sddmm_ctx *c, int M, int N, int K, const void *A, const void *B, int dtype,
                            bool on_device) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    if (M < 0 || N < 0 || K < 1) return fail(c, SDDMM_ERR_INVALID, "need M,N >= 0 and K >= 1 (got %d,%d,%d)", M, N, K);
    if (dtype != SDDMM_F32 && dtype != SDDMM_BF16 && dtype != SDDMM_F16)
        return fail(c, SDDMM_ERR_INVALID, "unknown dtype %d", dtype);
    if (dtype != SDDMM_F32 && K % 8) return fail(c, SDDMM_ERR_INVALID, "16-bit operands need K %% 8 == 0 (got %d)", K);
    if ((M > 0 && !A) || (N > 0 && !B)) return fail(c, SDDMM_ERR_NULL, "A or B is NULL");
    // a plan depends on the pattern and on the shape and type of the dense operands, not on their
    // values: new A and B of the same shape (the next iteration of a solver) keep it
    const bool keep_plan = c->planned && c->have_dense && c->M == M && c->N == N && c->K == K && c->dtype == dtype;
    release_dense(c);
    const size_t es = elem_size(dtype);
    const size_t a_bytes = (size_t)M * K * es, b_bytes = (size_t)N * K * es;
    if (on_device) {
        if (((uintptr_t)A | (uintptr_t)B) & 15) return fail(c, SDDMM_ERR_INVALID, "device A/B must be 16-byte aligned");
        c->dA = const_cast<void *>(A);
        c->dB = const_cast<void *>(B);
        c->own_dense = false;
    } else {
        c->own_dense = true;
        ALLOC_TRY(c, c->dA, a_bytes);
        ALLOC_TRY(c, c->dB, b_bytes);
        if (a_bytes) HIP_TRY(c, hipMemcpyAsync(c->dA, A, a_bytes, hipMemcpyHostToDevice, c->stream));
        if (b_bytes) HIP_TRY(c, hipMemcpyAsync(c->dB, B, b_bytes, hipMemcpyHostToDevice, c->stream));
        HIP_TRY(c, hipStreamSynchronize(c->stream));
    }
    c->M = M; c->N = N; c->K = K; c->dtype = dtype;
    c->have_dense = true;
    c->planned = keep_plan;
    return SDDMM_OK;
}

int sddmm_set_dense(sddmm_ctx *c, int M, int N, int K, const void *A, const void *B, int dtype) {
    return set_dense_common(c, M, N, K, A, B, dtype, false);
}
int sddmm_set_dense_device(sddmm_ctx *c, int M, int N, int K, const void *dA, const void *dB, int dtype) {
    return set_dense_common(c, M, N, K, dA, dB, dtype, true);
}

int sddmm_set_csr(sddmm_ctx *c, int M, int N, int64_t nnz, const int32_t *rowptr, const int32_t *col,
                  const float *sval) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_dims(c, M, N, nnz);
    if (rc) return rc;
    if (!rowptr || (nnz > 0 && (!col || !sval))) return fail(c, SDDMM_ERR_NULL, "rowptr, col or values is NULL");
    release_sparse(c);
    c->own_sparse = c->own_rowptr = true;
    ALLOC_TRY(c, c->d_rowptr, (size_t)(M + 1) * sizeof(int32_t));
    ALLOC_TRY(c, c->d_col, (size_t)nnz * sizeof(int32_t));
    ALLOC_TRY(c, c->d_sval, (size_t)nnz * sizeof(float));
    ALLOC_TRY(c, c->dP, (size_t)nnz * sizeof(float));
    HIP_TRY(c, hipMemcpyAsync(c->d_rowptr, rowptr, (size_t)(M + 1) * sizeof(int32_t), hipMemcpyHostToDevice, c->stream));
    if (nnz) {
        HIP_TRY(c, hipMemcpyAsync(c->d_col, col, (size_t)nnz * sizeof(int32_t), hipMemcpyHostToDevice, c->stream));
        HIP_TRY(c, hipMemcpyAsync(c->d_sval, sval, (size_t)nnz * sizeof(float), hipMemcpyHostToDevice, c->stream));
        HIP_TRY(c, hipMemsetAsync(c->dP, 0, (size_t)nnz * sizeof(float), c->stream));
    }
    c->sM = M; c->sN = N; c->nnz = nnz;
    rc = validate_csr(c);
    if (rc) { release_sparse(c); return rc; }
    c->have_sparse = c->have_rowptr = true;
    return SDDMM_OK;
}

int sddmm_set_csr_device(sddmm_ctx *c, int M, int N, int64_t nnz, const int32_t *d_rowptr, const int32_t *d_col,
                         const float *d_sval) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_dims(c, M, N, nnz);
    if (rc) return rc;
    if (!d_rowptr || (nnz > 0 && (!d_col || !d_sval))) return fail(c, SDDMM_ERR_NULL, "rowptr, col or values is NULL");
    release_sparse(c);
    c->own_sparse = c->own_rowptr = false;
    c->d_rowptr = const_cast<int32_t *>(d_rowptr);
    c->d_col = const_cast<int32_t *>(d_col);
    c->d_sval = const_cast<float *>(d_sval);
    ALLOC_TRY(c, c->dP, (size_t)nnz * sizeof(float));
    if (nnz) HIP_TRY(c, hipMemsetAsync(c->dP, 0, (size_t)nnz * sizeof(float), c->stream));
    c->sM = M; c->sN = N; c->nnz = nnz;
    rc = validate_csr(c);
    if (rc) { release_sparse(c); return rc; }
    c->have_sparse = c->have_rowptr = true;
    return SDDMM_OK;
}

static int set_coo_common(sddmm_ctx *c, int M, int N, int64_t nnz, const int32_t *row, const int32_t *col,
                          const float *sval, bool on_device) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_dims(c, M, N, nnz);
    if (rc) return rc;
    if (nnz > 0 && (!row || !col || !sval)) return fail(c, SDDMM_ERR_NULL, "row, col or values is NULL");
    release_sparse(c);
    c->own_sparse = c->own_rowidx = !on_device;
    c->own_rowptr = true;                 // the row pointer is always built here
    c->from_coo = true;
    if (on_device) {
        c->d_rowidx = const_cast<int32_t *>(row);
        c->d_col = const_cast<int32_t *>(col);
        c->d_sval = const_cast<float *>(sval);
    } else {
        ALLOC_TRY(c, c->d_rowidx, (size_t)nnz * sizeof(int32_t));
        ALLOC_TRY(c, c->d_col, (size_t)nnz * sizeof(int32_t));
        ALLOC_TRY(c, c->d_sval, (size_t)nnz * sizeof(float));
    }
    ALLOC_TRY(c, c->dP, (size_t)nnz * sizeof(float));
    ALLOC_TRY(c, c->d_rowptr, (size_t)(M + 1) * sizeof(int32_t));
    c->sM = M; c->sN = N; c->nnz = nnz;
    HIP_TRY(c, hipMemsetAsync(c->d_pc, 0, sizeof(DevCounters), c->stream));
    if (nnz) {
        if (!on_device) {
            HIP_TRY(c, hipMemcpyAsync(c->d_rowidx, row, (size_t)nnz * sizeof(int32_t), hipMemcpyHostToDevice, c->stream));
            HIP_TRY(c, hipMemcpyAsync(c->d_col, col, (size_t)nnz * sizeof(int32_t), hipMemcpyHostToDevice, c->stream));
            HIP_TRY(c, hipMemcpyAsync(c->d_sval, sval, (size_t)nnz * sizeof(float), hipMemcpyHostToDevice, c->stream));
        }
        HIP_TRY(c, hipMemsetAsync(c->dP, 0, (size_t)nnz * sizeof(float), c->stream));
        const int g = grid_capped(nnz, 256);
        SDDMM_LAUNCH(c, k_check_index, g, 256, c->d_rowidx, nnz, M, c->d_pc);
        SDDMM_LAUNCH(c, k_check_index, g, 256, c->d_col, nnz, N, c->d_pc);
        SDDMM_LAUNCH(c, k_check_coo_sorted, g, 256, c->d_rowidx, nnz, c->d_pc);
        LAUNCH_CHECK(c);
    }
    rc = fetch_counters(c);
    if (rc) { release_sparse(c); return rc; }
    if (c->pc.bad_pattern) {
        release_sparse(c);
        return fail(c, SDDMM_ERR_PATTERN, "COO row or column index out of range");
    }
    const bool sorted = c->pc.coo_unsorted == 0;
    if (sorted) {
        SDDMM_LAUNCH(c, k_rowptr_from_sorted_coo, grid_for(nnz + 1, 256), 256,
                           c->d_rowidx, nnz, M, c->d_rowptr);
        LAUNCH_CHECK(c);
        HIP_TRY(c, hipMemsetAsync(c->d_pc, 0, sizeof(DevCounters), c->stream));
        if (M > 0)
            SDDMM_LAUNCH(c, k_check_rowptr, grid_for(M, 256), 256, c->d_rowptr, M, nnz,
                               c->d_pc);
        LAUNCH_CHECK(c);
        rc = fetch_counters(c);
        if (rc) { release_sparse(c); return rc; }
        if (c->pc.bad_pattern) {
            release_sparse(c);
            return fail(c, SDDMM_ERR_HIP, "internal: row pointer built from COO is inconsistent");
        }
        c->have_rowptr = true;
    } else {
        // row statistics are not available without a row pointer; count distinct rows as unknown
        c->have_rowptr = false;
        c->pc.rows_nonempty = 0;
    }
    c->have_sparse = true;
    return SDDMM_OK;
}

int sddmm_set_coo(sddmm_ctx *c, int M, int N, int64_t nnz, const int32_t *row, const int32_t *col,
                  const float *sval) {
    return set_coo_common(c, M, N, nnz, row, col, sval, false);
}
int sddmm_set_coo_device(sddmm_ctx *c, int M, int N, int64_t nnz, const int32_t *d_row, const int32_t *d_col,
                         const float *d_sval) {
    return set_coo_common(c, M, N, nnz, d_row, d_col, d_sval, true);
}

int sddmm_update_values(sddmm_ctx *c, const float *sval) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    if (!c->have_sparse) return fail(c, SDDMM_ERR_STATE, "no sparse operand set");
    if (!c->own_sparse) return fail(c, SDDMM_ERR_STATE, "values are caller-owned device memory");
    if (c->nnz > 0 && !sval) return fail(c, SDDMM_ERR_NULL, "values is NULL");
    if (c->nnz) HIP_TRY(c, hipMemcpyAsync(c->d_sval, sval, (size_t)c->nnz * sizeof(float), hipMemcpyHostToDevice, c->stream));
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    return SDDMM_OK;
}

static int check_ready(sddmm_ctx *c) {
    if (!c->have_dense || !c->have_sparse) return fail(c, SDDMM_ERR_STATE, "set dense and sparse operands first");
    if (c->sM > c->M || c->sN > c->N)
        return fail(c, SDDMM_ERR_INVALID, "S is %dx%d but A has %d rows and B has %d rows", c->sM, c->sN, c->M, c->N);
    return SDDMM_OK;
}

int sddmm_plan(sddmm_ctx *c, int strategy) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_ready(c);
    if (rc) return rc;
    HIP_TRY(c, hipEventRecord(c->ev0, c->stream));
    rc = do_plan(c, strategy);
    if (rc) return rc;
    HIP_TRY(c, hipEventRecord(c->ev1, c->stream));
    HIP_TRY(c, hipEventSynchronize(c->ev1));
    float ms = 0.f;
    HIP_TRY(c, hipEventElapsedTime(&ms, c->ev0, c->ev1));
    c->stats = sddmm_stats{};
    c->stats.plan_ms = ms;
    fill_model(c);
    return SDDMM_OK;
}

int sddmm_launch(sddmm_ctx *c) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_ready(c);
    if (rc) return rc;
    if (!c->planned) {
        // operands were replaced since the last plan: plan again as last asked (AUTO on a new context)
        rc = sddmm_plan(c, c->requested);
        if (rc) return rc;
    }
    return enqueue_run(c);
}

int sddmm_synchronize(sddmm_ctx *c) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    return SDDMM_OK;
}

int sddmm_run(sddmm_ctx *c) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_ready(c);
    if (rc) return rc;
    if (!c->planned) {
        // operands were replaced since the last plan: plan again as last asked (AUTO on a new context)
        rc = sddmm_plan(c, c->requested);
        if (rc) return rc;
    }
    HIP_TRY(c, hipEventRecord(c->ev0, c->stream));
    rc = enqueue_run(c);
    if (rc) return rc;
    HIP_TRY(c, hipEventRecord(c->ev1, c->stream));
    HIP_TRY(c, hipEventSynchronize(c->ev1));
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    float ms = 0.f;
    HIP_TRY(c, hipEventElapsedTime(&ms, c->ev0, c->ev1));
    c->stats.run_ms = ms;
    c->stats.kernels_launched = c->launches;
    return SDDMM_OK;
}

// items of the fused kernel: the rows of more than FUSED_ROW_MAX entries, cut into segments of
// SDDMM_FUSED_SEG entries (default 2048, shortened below when there are few items; a knob of its own,
// apart from SDDMM_SEG of the plain SDDMM, because the pieces of a row add to O atomically: the segment
// length decides which rows are summed in an order that may differ from run to run)
static int plan_fused_items(sddmm_ctx *c, const unsigned char *panel_owner) {
    if (c->fused_items_valid && c->fused_items_panels == (panel_owner != nullptr)) return SDDMM_OK;
    int seg = std::max(WAVE, env_int("SDDMM_FUSED_SEG", 2048));
    const int64_t nb = ((int64_t)c->sM + SCAN_TILE - 1) / SCAN_TILE;
    const int arc = ensure_arena(c);
    if (arc) return arc;
    ARENA_HOLDS(c, nb, c->block_sums_cap, "block sums");
    c->n_fused_items = 0;
    if (nb > 0) {
        DevCounters tmp;
        auto count = [&]() -> int {
            HIP_TRY(c, hipMemsetAsync(&c->d_pc->k[K_ROWS_SHORT][0], 0,
                                      sizeof(unsigned long long) * SPREAD * (K_NNZ_LONG - K_ROWS_SHORT + 1), c->stream));
            HIP_TRY(c, hipMemsetAsync(&c->d_pc->n_items, 0, sizeof(unsigned long long), c->stream));
            SDDMM_LAUNCH(c, k_classify_count, nb, SCAN_BLOCK, c->d_rowptr,
                               panel_owner, c->sM, FUSED_ROW_MAX + 1, seg, c->d_block_sums, c->d_pc, 2,
                               (unsigned int *)nullptr);
            SDDMM_LAUNCH(c, k_scan_block_sums, 1, SCAN_BLOCK, c->d_block_sums, (int)nb,
                               &c->d_pc->n_items);
            LAUNCH_CHECK(c);
            HIP_TRY(c, hipMemcpyAsync(&tmp, c->d_pc, sizeof(DevCounters), hipMemcpyDeviceToHost, c->stream));
            HIP_TRY(c, hipStreamSynchronize(c->stream));
            return SDDMM_OK;
        };
        int rc = count();
        if (rc) return rc;
        // Few long rows: one wavefront per row walks its chunks one after the other and the launch
        // waits for them (3 000 rows of 554 entries: 50 us as single items, 42 us in pieces of 256,
        // the pieces of a row adding to O atomically).  With enough items to fill the chip several
        // times the long segments stay: there the atomic adds cost more than they return.
        const PlanCounters first = summarize(tmp);
        const int64_t item_entries = (int64_t)(first.nnz_medium + first.nnz_long);
        c->fused_short_avg = first.rows_short ? (double)first.nnz_short / (double)first.rows_short : 0.0;
        // (rows of up to 128 bytes; at 256 bytes it changes nothing, at 1 KiB the adds of 256 floats per piece lose 4 %)
        if ((int64_t)tmp.n_items > 0 && (int64_t)tmp.n_items < 4096 && !getenv("SDDMM_FUSED_SEG") &&
            (size_t)c->K * elem_size(c->dtype) <= 128) {
            int shorter = (int)std::min<int64_t>(seg, ((item_entries / 8192 + WAVE - 1) / WAVE) * WAVE);
            shorter = std::max(shorter, 256);
            if (shorter < seg) {
                seg = shorter;
                rc = count();
                if (rc) return rc;
            }
        }
        c->n_fused_items = (int64_t)tmp.n_items;
        if (c->n_fused_items > c->fused_items_cap) {
            dfree(c->d_fused_items);
            ALLOC_TRY(c, c->d_fused_items, (size_t)c->n_fused_items * sizeof(RowItem));
            c->fused_items_cap = c->n_fused_items;
        }
        if (c->n_fused_items > 0) {
            SDDMM_LAUNCH(c, k_classify_write, nb, SCAN_BLOCK, c->d_rowptr,
                               panel_owner, c->sM, FUSED_ROW_MAX + 1, seg, c->d_block_sums, c->d_fused_items, 2);
            LAUNCH_CHECK(c);
        }
    }
    c->fused_items_valid = true;
    c->fused_items_panels = panel_owner != nullptr;
    return SDDMM_OK;
}

int sddmm_run_fused(sddmm_ctx *c) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_ready(c);
    if (rc) return rc;
    const Shape s = shape_of(c);
    // 16-byte units, at most 8 lanes per entry and 32 fp32 accumulators of the output row per lane
    if (s.unit == 1 || s.LPN == 0 || s.LPN > 8 || c->K > 256)
        return fail(c, SDDMM_ERR_UNSUPPORTED,
                    "the fused SDDMM+SpMM needs K <= 256, a multiple of 4 (fp32) or 8 (bf16, fp16)");
    if (!c->have_rowptr) return fail(c, SDDMM_ERR_UNSUPPORTED, "the fused SDDMM+SpMM needs row-sorted entries");
    // rows of 32, 64 or 128 components: the 8-row panels of the current plan (AUTO if there is none
    // yet) take the matrix-core kernel, which shares every gathered B row between 8 rows and both
    // products; the other rows take the gather kernels
    bool panels = (c->K == 32 || c->K == 64 || c->K == 128) && env_int("SDDMM_FUSED_PANELS", 1) != 0;
    if (panels && !c->planned) {
        rc = sddmm_plan(c, c->requested);
        if (rc) return rc;
    }
    panels = panels && c->planned && c->panel_mfma && c->n_panel_items > 0 && c->owner_active &&
             (c->strategy == SDDMM_AUTO || c->strategy == SDDMM_LDS_TILED || c->strategy == SDDMM_MFMA_TILE);
    const unsigned char *panel_owner = panels ? (const unsigned char *)c->d_owner : nullptr;
    rc = plan_fused_items(c, panel_owner);
    if (rc) return rc;
    const size_t o_bytes = (size_t)c->M * (size_t)c->K * sizeof(float);
    if (o_bytes > c->o_cap) {
        dfree(c->dO);
        c->o_cap = 0;
        ALLOC_TRY(c, c->dO, o_bytes);
        c->o_cap = o_bytes;
    }
    HIP_TRY(c, hipEventRecord(c->ev0, c->stream));
    // (when the panels own every row that has entries, O is complete after a memset and the panel kernel;
    // otherwise the kernel of the short rows, first in the stream, writes every row of O below sM, zeros
    // for the rows that the kernels after it add to, and only the rows of A beyond S are cleared here)
    const bool others = c->sM > 0 && c->nnz > 0 && (!panels || c->n_tiles > 0 || c->rows_short > 0 || c->n_items > 0);
    if (o_bytes) {
        const size_t written = others ? (size_t)c->sM * (size_t)c->K * sizeof(float) : 0;
        if (written < o_bytes) HIP_TRY(c, hipMemsetAsync((char *)c->dO + written, 0, o_bytes - written, c->stream));
    }
    int launches = 0;
    bool rows_written = false;
    // Short rows of fewer entries, on average, than half of what a lane group takes per step (a power-law
    // graph: 3.5 against 8 lanes per entry at 128-byte rows): one row per lane group would idle most of its
    // steps (20 % of them useful there), so the wavefronts deal whole rows out to their groups by entry
    // count instead (576 -> 369 us for those rows).  With longer rows, or 4 lanes per entry, the extra
    // gathers of the A rows and the longer walks cost more than the idle steps (mixed-density shape, 12.5
    // entries per short row: 33 -> 65 us; power-law with 64-byte rows: 396 -> 432 us).
    const int balanced_env = env_int("SDDMM_FUSED_BALANCED", -1);
    const bool balanced = balanced_env >= 0 ? balanced_env != 0
                                            : (c->fused_short_avg > 0.0 && 2.0 * c->fused_short_avg < (double)s.LPN);
    if (c->sM > 0 && c->nnz > 0) {
        with_layout(s, [&](auto L) {
            using LT = decltype(L);
            if (!others) return;
            if constexpr (!LT::LONG && LT::LPN <= 8 && LT::U::ELEMS > 1 && LT::UPL * LT::U::ELEMS <= 32) {
                const int64_t rows_per_wave = WAVE / LT::LPN;
                const int64_t waves = ((int64_t)c->sM + rows_per_wave - 1) / rows_per_wave;
                const int64_t rblocks = (waves + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
                if (balanced) {
                    const int64_t bwaves = ((int64_t)c->sM + WAVE - 1) / WAVE;
                    const int64_t bblocks = (bwaves + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
                    SDDMM_LAUNCH(c, (k_fusedmm_rows_balanced<LT>), xcd_grid(bblocks), BLOCK,
                                       (const void *)c->dA, (const void *)c->dB, s.KU, c->d_rowptr, c->d_col, c->d_sval,
                                       c->dP, c->dO, c->sM, FUSED_ROW_MAX, bblocks, panel_owner);
                } else {
                    SDDMM_LAUNCH(c, (k_fusedmm_rows<LT>), xcd_grid(rblocks), BLOCK,
                                       (const void *)c->dA, (const void *)c->dB, s.KU, c->d_rowptr, c->d_col, c->d_sval,
                                       c->dP, c->dO, c->sM, FUSED_ROW_MAX, rblocks, panel_owner);
                }
                ++launches;
                rows_written = true;
                if (c->n_fused_items > 0) {
                    const int64_t nblocks = (c->n_fused_items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
                    SDDMM_LAUNCH(c, (k_fusedmm<LT>), xcd_grid(nblocks), BLOCK,
                                       (const void *)c->dA, (const void *)c->dB, s.KU, c->d_rowptr, c->d_col,
                                       c->d_sval, c->dP, c->dO, (const RowItem *)c->d_fused_items, c->n_fused_items,
                                       nblocks);
                    ++launches;
                }
            }
        });
        if (others && !rows_written) return fail(c, SDDMM_ERR_UNSUPPORTED, "internal: no fused kernel for this row layout");
        if (panels) {
            if (c->dtype == SDDMM_F32) {
                if (c->K == 32) launch_panel_fused_t<DT_F32, 2>(c);
                else if (c->K == 64) launch_panel_fused_t<DT_F32, 4>(c);
                else launch_panel_fused_t<DT_F32, 8>(c);
            } else if (c->dtype == SDDMM_BF16) {
                if (c->K == 32) launch_panel_fused_t<DT_BF16, 1>(c);
                else if (c->K == 64) launch_panel_fused_t<DT_BF16, 2>(c);
                else launch_panel_fused_t<DT_BF16, 4>(c);
            } else {
                if (c->K == 32) launch_panel_fused_t<DT_F16, 1>(c);
                else if (c->K == 64) launch_panel_fused_t<DT_F16, 2>(c);
                else launch_panel_fused_t<DT_F16, 4>(c);
            }
            ++launches;
        }
        LAUNCH_CHECK(c);
    }
    HIP_TRY(c, hipEventRecord(c->ev1, c->stream));
    HIP_TRY(c, hipEventSynchronize(c->ev1));
    float ms = 0.f;
    HIP_TRY(c, hipEventElapsedTime(&ms, c->ev0, c->ev1));
    c->stats.run_ms = ms;
    c->stats.kernels_launched = launches;
    c->have_fused = true;
    return SDDMM_OK;
}

int sddmm_get_fused(sddmm_ctx *c, float *O) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    if (!c->have_fused) return fail(c, SDDMM_ERR_STATE, "no fused result: call sddmm_run_fused first");
    const size_t o_bytes = (size_t)c->M * (size_t)c->K * sizeof(float);
    if (o_bytes > 0 && !O) return fail(c, SDDMM_ERR_NULL, "O is NULL");
    if (o_bytes) HIP_TRY(c, hipMemcpyAsync(O, c->dO, o_bytes, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    return SDDMM_OK;
}

int sddmm_get_fused_device(sddmm_ctx *c, const float **dO) {
    if (!c || !dO) return SDDMM_ERR_NULL;
    if (!c->have_fused) return fail(c, SDDMM_ERR_STATE, "no fused result: call sddmm_run_fused first");
    *dO = c->dO;
    return SDDMM_OK;
}

int sddmm_time_runs(sddmm_ctx *c, int warmup, int reps, int include_plan, float *ms_each) {
    if (!c) return SDDMM_ERR_NULL;
    if (reps < 0 || warmup < 0) return fail(c, SDDMM_ERR_INVALID, "negative repetition count");
    if (reps > 0 && !ms_each) return fail(c, SDDMM_ERR_NULL, "ms_each is NULL");
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_ready(c);
    if (rc) return rc;
    if (!c->planned) {
        // operands were replaced since the last plan: plan again as last asked (AUTO on a new context)
        rc = sddmm_plan(c, c->requested);
        if (rc) return rc;
    }
    const int requested = c->requested;
    for (int i = 0; i < warmup + reps; ++i) {
        HIP_TRY(c, hipEventRecord(c->ev0, c->stream));
        if (include_plan) {
            rc = do_plan(c, requested);
            if (rc) return rc;
        }
        rc = enqueue_run(c);
        if (rc) return rc;
        HIP_TRY(c, hipEventRecord(c->ev1, c->stream));
        HIP_TRY(c, hipEventSynchronize(c->ev1));
        if (i >= warmup) HIP_TRY(c, hipEventElapsedTime(&ms_each[i - warmup], c->ev0, c->ev1));
    }
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    return SDDMM_OK;
}

int sddmm_time_region(sddmm_ctx *c, int reps, int include_plan, float *total_ms) {
    if (!c) return SDDMM_ERR_NULL;
    if (reps < 1) return fail(c, SDDMM_ERR_INVALID, "repetition count must be positive");
    if (!total_ms) return fail(c, SDDMM_ERR_NULL, "total_ms is NULL");
    HIP_TRY(c, hipSetDevice(c->device));
    int rc = check_ready(c);
    if (rc) return rc;
    if (!c->planned) {
        // operands were replaced since the last plan: plan again as last asked (AUTO on a new context)
        rc = sddmm_plan(c, c->requested);
        if (rc) return rc;
    }
    const int requested = c->requested;
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    HIP_TRY(c, hipEventRecord(c->ev0, c->stream));
    for (int i = 0; i < reps; ++i) {
        if (include_plan) {
            rc = do_plan(c, requested);
            if (rc) return rc;
        }
        rc = enqueue_run(c);
        if (rc) return rc;
    }
    HIP_TRY(c, hipEventRecord(c->ev1, c->stream));
    HIP_TRY(c, hipEventSynchronize(c->ev1));
    HIP_TRY(c, hipEventElapsedTime(total_ms, c->ev0, c->ev1));
    return SDDMM_OK;
}

int sddmm_get_values(sddmm_ctx *c, float *P_values) {
    if (!c) return SDDMM_ERR_NULL;
    HIP_TRY(c, hipSetDevice(c->device));
    if (!c->have_sparse) return fail(c, SDDMM_ERR_STATE, "no sparse operand set");
    if (c->nnz > 0 && !P_values) return fail(c, SDDMM_ERR_NULL, "P_values is NULL");
    if (c->nnz) HIP_TRY(c, hipMemcpyAsync(P_values, c->dP, (size_t)c->nnz * sizeof(float), hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    return SDDMM_OK;
}

int sddmm_get_values_device(sddmm_ctx *c, const float **dP) {
    if (!c || !dP) return SDDMM_ERR_NULL;
    if (!c->have_sparse) return fail(c, SDDMM_ERR_STATE, "no sparse operand set");
    *dP = c->dP;
    return SDDMM_OK;
}

int sddmm_last_stats(const sddmm_ctx *c, sddmm_stats *out) {
    if (!c || !out) return SDDMM_ERR_NULL;
    *out = c->stats;
    return SDDMM_OK;
}

// ---- the entry point that allocates nothing ---------------------------------------
// The row index per stored entry that the flat kernel reads (k_expand_rows writes it,
// k_flat reads it) lives in a static device array instead of a hipMalloc'ed buffer.
// Every device the library runs on holds its own copy of the array at its own address
// until the process ends; in host code the array's name is only a handle for
// hipGetSymbolAddress, never an address to hand to a kernel.
}  // extern "C"

static __device__ __align__(256) int32_t scratch[SDDMM_NOALLOC_MAX_NNZ];

namespace {
constexpr int NOALLOC_MAX_DEVICES = 64;
int32_t *g_scratch_ptr[NOALLOC_MAX_DEVICES] = {nullptr};   // device address of `scratch`, per device
std::mutex g_scratch_mu;

// Device address of the current device's copy of `scratch` (looked up once per device).
int scratch_of_current_device(int *device, int32_t **ptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) return SDDMM_ERR_NO_DEVICE;
    if (dev >= NOALLOC_MAX_DEVICES) return SDDMM_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> guard(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return SDDMM_ERR_HIP;
        g_scratch_ptr[dev] = static_cast<int32_t *>(p);
    }
    *device = dev;
    *ptr = g_scratch_ptr[dev];
    return SDDMM_OK;
}
}  // namespace

extern "C" {

int sddmm_launch_noalloc(int M, int N, int K, int64_t nnz, const float *dA, const float *dB,
                         const int32_t *d_rowptr, const int32_t *d_col, const float *d_sval, float *dP,
                         void *stream) {
    if (M < 0 || N < 0 || K < 1 || nnz < 0) return SDDMM_ERR_INVALID;
    if (nnz > 0 && (M == 0 || N == 0)) return SDDMM_ERR_INVALID;
    if (nnz > (int64_t)SDDMM_NOALLOC_MAX_NNZ) return SDDMM_ERR_TOO_LARGE;
    if (!d_rowptr || (nnz > 0 && (!dA || !dB || !d_col || !d_sval || !dP))) return SDDMM_ERR_NULL;
    if (((uintptr_t)dA | (uintptr_t)dB) & 15) return SDDMM_ERR_INVALID;
    int device = -1;
    int32_t *rowidx = nullptr;
    const int rc = scratch_of_current_device(&device, &rowidx);
    if (rc) return rc;
    if (nnz == 0) return SDDMM_OK;
    // a context on the stack: nothing is allocated for it, it only carries the launch arguments
    sddmm_ctx c;
    c.device = device;
    c.stream = static_cast<hipStream_t>(stream);
    c.M = M; c.N = N; c.K = K; c.dtype = SDDMM_F32;
    c.dA = const_cast<float *>(dA);
    c.dB = const_cast<float *>(dB);
    c.sM = M; c.sN = N; c.nnz = nnz;
    c.d_rowptr = const_cast<int32_t *>(d_rowptr);
    c.d_col = const_cast<int32_t *>(d_col);
    c.d_sval = const_cast<float *>(d_sval);
    c.dP = dP;
    c.d_rowidx = rowidx;                       // every position below nnz is rewritten: nothing to clear
    // (bounded by nnz: a row pointer that runs past it cannot make the kernel leave the array)
    SDDMM_LAUNCH(&c, k_expand_rows, grid_for(M, 256), 256, c.d_rowptr, M, rowidx, nnz);
    launch_flat(&c);
    if (hipGetLastError() != hipSuccess) return SDDMM_ERR_HIP;
    if (c.oversize) return SDDMM_ERR_UNSUPPORTED;
    return SDDMM_OK;
}

// Smallest feasible maximum load by bisection, then a greedy left-to-right fill
// with that load: the contract of CSR<T>::_dispatch (src/matrices/CSR.hpp:196-264).
int sddmm_partition_rows(int M, const int32_t *rowptr, int parts, int stride, int32_t *start_idx) {
    if (!rowptr || !start_idx) return SDDMM_ERR_NULL;
    if (M <= 0 || parts <= 0 || stride <= 0 || M % stride) return SDDMM_ERR_INVALID;
    const int64_t groups = M / stride;
    auto load = [&](int64_t g) { return (int64_t)rowptr[(g + 1) * stride] - (int64_t)rowptr[g * stride]; };
    int64_t heaviest = 0;
    for (int64_t g = 0; g < groups; ++g) heaviest = std::max(heaviest, load(g));
    auto parts_needed = [&](int64_t cap) {
        int64_t used = 1, acc = 0;
        for (int64_t g = 0; g < groups; ++g) {
            acc += load(g);
            if (acc > cap) { ++used; acc = load(g); }
        }
        return used;
    };
    int64_t lo = std::max<int64_t>(1, heaviest), hi = std::max<int64_t>(lo, rowptr[M]);
    int64_t cap = 0;                       // stays 0 when even cap == nnz needs too many parts
    if (parts_needed(hi) <= parts) {
        while (lo < hi) {
            const int64_t mid = lo + (hi - lo) / 2;
            if (parts_needed(mid) <= parts) hi = mid; else lo = mid + 1;
        }
        cap = lo;
    }
    int w = 0;
    int64_t acc = 0;
    start_idx[w++] = 0;
    for (int64_t g = 0; g < groups; ++g) {
        acc += load(g);
        if (acc > cap) {
            if (w > parts) return SDDMM_ERR_INVALID;
            start_idx[w++] = (int32_t)(g * stride);
            acc = load(g);
        }
    }
    while (w <= parts) start_idx[w++] = M;
    return SDDMM_OK;
}

}  // extern "C"
