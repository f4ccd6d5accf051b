/*
 * sddmm_amd.h -- C ABI of the MI355X (gfx950) SDDMM engine.
 *
 *     P[i,j] = S[i,j] * sum_k A[i,k] * B[j,k]      for every stored (i,j) of S
 *
 * A is M x K row-major, B is N x K row-major (already "transposed"), S is a
 * sparse M x N sampling matrix in CSR or COO with 32-bit indices, and P keeps
 * S's pattern and entry order verbatim.
 *
 * The entry points are what a binding of the reference's competitor interface
 * (src/benchmark/competitor.hpp:12-60) needs for this one path:
 *
 *   reference phase                          entry points
 *   init_csr / init_coo    (:27-28)          sddmm_create, sddmm_set_dense,
 *                                            sddmm_set_csr | sddmm_set_coo, sddmm_plan
 *   run_csr / run_coo      (:30-31)          sddmm_run   (complete on return)
 *   cleanup_csr/cleanup_coo(:33-34)          sddmm_get_values, sddmm_destroy
 *
 * Conventions
 *   - every function returns 0 (SDDMM_OK) or a negative sddmm_status; nothing throws;
 *   - host pointers are borrowed for the duration of the call only;
 *   - all device memory belongs to the context, except buffers handed in through
 *     the *_device variants, which stay owned by the caller and must outlive the ctx;
 *   - a context is not thread-safe; distinct contexts may be used from distinct threads;
 *   - there is no CPU fallback: without a HIP device sddmm_create fails.
 */
#ifndef SDDMM_AMD_H
#define SDDMM_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct sddmm_ctx sddmm_ctx;

enum sddmm_status {
    SDDMM_OK = 0,
    SDDMM_ERR_INVALID = -1,     /* bad size / enum / inconsistent arguments          */
    SDDMM_ERR_NULL = -2,        /* required pointer is NULL                          */
    SDDMM_ERR_STATE = -3,       /* call order: dense + sparse operands must be set   */
    SDDMM_ERR_ALLOC = -4,       /* device or host allocation failed                  */
    SDDMM_ERR_HIP = -5,         /* a HIP runtime call or kernel launch failed        */
    SDDMM_ERR_UNSUPPORTED = -6, /* strategy not applicable to these operands         */
    SDDMM_ERR_NO_DEVICE = -7,   /* no usable gfx950 device                           */
    SDDMM_ERR_PATTERN = -8,     /* CSR/COO structure is malformed (see sddmm_set_*)  */
    SDDMM_ERR_TOO_LARGE = -9    /* sddmm_launch_noalloc: nnz > SDDMM_NOALLOC_MAX_NNZ */
};

enum sddmm_dtype {
    SDDMM_F32 = 0,  /* A,B fp32; fp32 accumulate                                     */
    SDDMM_BF16 = 1, /* A,B bfloat16 (uint16 storage); fp32 accumulate and output     */
    SDDMM_F16 = 2   /* A,B IEEE half (uint16 storage); fp32 accumulate and output --
                       the input type of the reference's tensor-core sketch,
                       src/competitors/gpu/gpu_tensor.cu:27-99                       */
};

/* Kernel selection.  The reference picks between two kernels from one global
 * density number (src/competitors/gpu/gpu_dynamic.hpp:27-55); AUTO here classifies
 * per row / per 16x16 tile on the device.  The fixed strategies exist as
 * comparators and for tests. */
enum sddmm_strategy {
    SDDMM_AUTO = 0,
    SDDMM_FLAT = 1,       /* one lane group per stored entry over a flat entry range
                             (the role of src/competitors/gpu/gpu_convert.cu:8-50)    */
    SDDMM_ROW_WAVE = 2,   /* one wavefront per row segment, A row held in registers   */
    SDDMM_SHORT_ROWS = 3, /* many short rows per wavefront                            */
    SDDMM_LDS_TILED = 4,  /* ROW PANELS (also spelled SDDMM_ROW_PANEL): 8 rows with a common
                             column list share every gathered B row, which is held in
                             registers -- nothing is staged in LDS, the name is the slot of
                             the reference's LDS-tiled row-panel kernels that this strategy
                             fills (src/competitors/gpu/gpu_shared.cu:18-88,
                             gpu_preprocessing.cu:18-96: B reused across a row panel);
                             other rows run on AUTO's gather kernels                       */
    SDDMM_MFMA_TILE = 5,  /* near-dense 16x16 tiles on MFMA, remainder on AUTO's
                             gather kernels (the role of gpu_tensor.cu:27-99).  AUTO
                             also cuts tiles from the union of the columns of 16
                             similar rows (the active-column lists of
                             gpu_preprocessing.hpp:57-141) and from near-dense rows
                             gathered by column window                                */
    SDDMM_ROW_PANEL = SDDMM_LDS_TILED,
    SDDMM_EXACT = 6       /* one lane per entry, k ascending, separate fp32 multiply
                             and add: bit-identical to cpu_basic.hpp:18-51            */
};

/* Filled by sddmm_last_stats.  Times are device times from HIP events recorded on
 * the context's stream around the most recent sddmm_plan / sddmm_run. */
typedef struct sddmm_stats {
    float plan_ms;            /* classifier + auxiliary structure build               */
    float run_ms;             /* all kernels of the last sddmm_run                    */
    int32_t strategy_used;    /* SDDMM_AUTO = per-strip/panel/row dispatch; a fixed
                                 strategy otherwise -- also when AUTO resolved to one
                                 (FLAT for unsorted COO and for matrices whose rows
                                 are short on average)                                */
    int32_t kernels_launched; /* launches per sddmm_run                               */
    int64_t nnz;
    int64_t rows_nonempty;
    int64_t rows_short;       /* rows sent to the many-rows-per-wave kernel           */
    int64_t rows_medium;      /* rows sent to the wave-per-row kernel                 */
    int64_t rows_long;        /* rows split into several wave segments                */
    int64_t nnz_short, nnz_medium, nnz_long;
    int64_t mfma_tiles;       /* 16x16 tiles on the MFMA path                         */
    int64_t nnz_mfma;         /* stored entries covered by those tiles                */
    int64_t cols_touched;     /* distinct B rows referenced (0 when not computed)     */
    /* byte / flop model of one run: 2*nnz*K flops;
       gathered = 4(M+1) + 12 nnz + e K rows_nonempty + e K nnz  (e = 4 or 2)         */
    double flops;
    double bytes_gathered;
    int64_t panels;           /* 8-row panels with a common column list (panel kernel) */
    int64_t nnz_panel;        /* stored entries covered by those panels               */
} sddmm_stats;

/* ---- life cycle --------------------------------------------------------- */
int sddmm_create(sddmm_ctx **out, int device);
void sddmm_destroy(sddmm_ctx *ctx);
const char *sddmm_strerror(int code);
/* Text of the last failure on this context ("" if none); owned by the context. */
const char *sddmm_last_error(const sddmm_ctx *ctx);

/* Every context enqueues its copies and kernels on a stream of its own (the
 * reference's competitors launch on the null stream, e.g.
 * src/competitors/gpu/gpu_basic.cu:83,95).
 * lent != 0: from now on enqueue on `stream` instead, a hipStream_t of this
 * context's device that the caller keeps alive (NULL is the device's null stream);
 * producers of borrowed device operands and consumers of sddmm_get_values_device
 * ordered on that stream then need no host synchronisation around sddmm_launch.
 * lent == 0: back to the context's own stream (`stream` is ignored).  The call
 * waits for the work of this context that is still in flight. */
int sddmm_set_stream(sddmm_ctx *ctx, void *stream, int lent);
/* The hipStream_t in use. */
int sddmm_get_stream(const sddmm_ctx *ctx, void **stream);

/* ---- operands (init phase) ---------------------------------------------- */
/* A: M*K elements, B: N*K elements, row-major, leading dimension K
 * (src/matrices/Dense.hpp:43-50).  K >= 1; any K is accepted for SDDMM_F32
 * (the reference's kernels need K%8 or K%32, gpu_basic.cu:77-80, gpu_shared.cu:98-101);
 * SDDMM_BF16 and SDDMM_F16 need K % 8 == 0. */
int sddmm_set_dense(sddmm_ctx *ctx, int M, int N, int K, const void *A, const void *B, int dtype);
/* Same, A and B already in device memory of this ctx's device (borrowed, 16-byte aligned). */
int sddmm_set_dense_device(sddmm_ctx *ctx, int M, int N, int K, const void *dA, const void *dB, int dtype);

/* CSR as in src/matrices/CSR.hpp:162-167: rowptr[M+1] non-decreasing with rowptr[0]==0
 * and rowptr[M]==nnz, col[nnz] in [0,N); nnz <= 2^31 - 2^16 (32-bit positions like the
 * reference's, with room for the kernels' look-ahead).  Columns need not be sorted; duplicates are
 * computed independently.  Violations return SDDMM_ERR_PATTERN. */
int sddmm_set_csr(sddmm_ctx *ctx, int M, int N, int64_t nnz,
                  const int32_t *rowptr, const int32_t *col, const float *sval);
/* COO as in src/matrices/COO.hpp:171-175: row[nnz], col[nnz], val[nnz].  Any entry
 * order is accepted; when rows are non-decreasing (the reference always stores them
 * sorted, COO.hpp:39-40) every strategy is available, otherwise only FLAT and EXACT. */
int sddmm_set_coo(sddmm_ctx *ctx, int M, int N, int64_t nnz,
                  const int32_t *row, const int32_t *col, const float *sval);
/* Device-resident CSR (borrowed).  The structure is validated on the device. */
int sddmm_set_csr_device(sddmm_ctx *ctx, int M, int N, int64_t nnz,
                         const int32_t *d_rowptr, const int32_t *d_col, const float *d_sval);
/* Device-resident COO (borrowed), same rules as sddmm_set_coo; the row pointer of
 * row-sorted input is built by the context. */
int sddmm_set_coo_device(sddmm_ctx *ctx, int M, int N, int64_t nnz,
                         const int32_t *d_row, const int32_t *d_col, const float *d_sval);
/* Replace the S values only (same pattern), e.g. between iterations of a solver. */
int sddmm_update_values(sddmm_ctx *ctx, const float *sval);

/* ---- plan (init phase) + run -------------------------------------------- */
/* Classify rows / tiles and build whatever the chosen strategy needs.  All of it
 * runs on the device; nothing is read back except a few counters.  Replacing the
 * sparse operand, or the dense ones by operands of another shape or type, drops the
 * plan; the next run then plans again by itself with the strategy asked for last
 * (SDDMM_AUTO on a context that was never planned).  New A and B of the same shape and
 * type keep the plan: it depends on the pattern only. */
int sddmm_plan(sddmm_ctx *ctx, int strategy);
/* Launch and wait.  P is complete on return (every reference run_csr ends in a
 * device synchronise, e.g. src/competitors/gpu/gpu_basic.hpp:72). */
int sddmm_run(sddmm_ctx *ctx);
/* Enqueue on the context's stream without waiting / wait for it.  On a planned
 * context sddmm_launch only enqueues kernels (no allocation, copy, fill or wait), so
 * it may be recorded into a HIP graph on a lent stream under capture. */
int sddmm_launch(sddmm_ctx *ctx);
int sddmm_synchronize(sddmm_ctx *ctx);
/* warmup untimed launches, then reps launches each bracketed by HIP events on the
 * context's stream; ms_each[reps] receives device milliseconds per launch.
 * include_plan != 0 re-runs the classifier inside every timed region. */
int sddmm_time_runs(sddmm_ctx *ctx, int warmup, int reps, int include_plan, float *ms_each);
/* reps launches back to back between ONE pair of HIP events on the context's stream:
 * *total_ms / reps is the average duration of a launch inside a stream of launches
 * (what a kernel trace of the same loop reports), without the idle gap that the
 * per-launch synchronisation of sddmm_time_runs puts in front of every launch. */
int sddmm_time_region(sddmm_ctx *ctx, int reps, int include_plan, float *total_ms);

/* ---- one launch that allocates nothing ----------------------------------------- */
/* No counterpart in the reference.  For callers that cannot call hipMalloc: code under
 * HIP graph capture, tight serving loops, harnesses that forbid allocation.  One complete
 * fp32 SDDMM on caller-owned device buffers, enqueued on `stream` (a hipStream_t of the
 * current device, NULL = the null stream) without waiting, like sddmm_launch on a context
 * planned with SDDMM_FLAT over sddmm_set_dense_device / sddmm_set_csr_device operands --
 * same kernels, bit-identical values -- except that the row index per stored entry which
 * the flat kernel reads is written into a static device array of the library
 * (SDDMM_NOALLOC_MAX_NNZ int32 = 64 MiB per device, held until the process ends) instead
 * of an allocated buffer.  It calls no hipMalloc, hipFree or other allocating routine and
 * waits for nothing.  The first call on a device looks up that device's copy of the
 * array (hipGetSymbolAddress): make it outside a graph capture (nnz = 0 will do).
 *   - dA [M x K], dB [N x K] row-major fp32, 16-byte aligned; d_rowptr[M+1], d_col[nnz],
 *     d_sval[nnz], dP[nnz]; P is complete when `stream` has executed the call;
 *   - the structure is NOT validated here (that needs a read-back): pass arrays that
 *     sddmm_set_csr_device would accept; row pointer values beyond nnz are clamped when
 *     the row indices are written, so a bad row pointer cannot write outside the array;
 *   - every process that loads the library reserves the array on each device it uses,
 *     whether or not this entry point is called; a deployment that never calls it can
 *     build the library with a smaller -DSDDMM_NOALLOC_MAX_NNZ=<n>;
 *   - nnz > SDDMM_NOALLOC_MAX_NNZ returns SDDMM_ERR_TOO_LARGE and launches nothing;
 *   - all calls on one device share the array: calls that may overlap on one GPU
 *     (different streams, different threads) race; order them on one stream. */
#ifndef SDDMM_NOALLOC_MAX_NNZ
#define SDDMM_NOALLOC_MAX_NNZ (1 << 24)
#endif
int sddmm_launch_noalloc(int M, int N, int K, int64_t nnz, const float *dA, const float *dB,
                         const int32_t *d_rowptr, const int32_t *d_col, const float *d_sval, float *dP,
                         void *stream);

/* ---- SDDMM followed by SpMM over the same pattern ("FusedMM") -------------- */
/* O[i,:] = sum over the stored (i,j) of P[i,j] * B[j,:], with P as sddmm_run computes
 * it (and written like it): the step that consumes an SDDMM result in the applications
 * the reference names.  No counterpart in the reference's code, which stops at P
 * (src/competitors/cpu/cpu_basic.hpp:18-51).  O is M x K fp32 row-major, owned by the
 * context.  Needs K <= 256, a multiple of 4 (fp32 operands) or 8 (bf16, fp16), and
 * row-sorted entries (CSR, or COO with non-decreasing rows); SDDMM_ERR_UNSUPPORTED otherwise.
 * Rows cut into several work items (longer than 2048 entries; longer than 256 where a
 * matrix of rows of up to 128 bytes has only a few thousand such rows) are accumulated
 * with atomic adds, so their last bits may differ from run to run.
 * K = 32, 64 or 128 (fp32, bf16 or fp16 operands): the rows that the current plan (SDDMM_AUTO
 * is planned if there is none) runs as 8-row panels take a matrix-core kernel that shares
 * every gathered B row between the 8 rows and between both products; the output rows of a
 * panel are accumulated with atomic adds as above.  The other rows take the gather kernels.
 * In either kernel a B row is read only for entries that are stored: a non-finite value in B
 * reaches the output rows that have an entry in its column and no others. */
int sddmm_run_fused(sddmm_ctx *ctx);
int sddmm_get_fused(sddmm_ctx *ctx, float *O);                    /* M*K floats to the host */
int sddmm_get_fused_device(sddmm_ctx *ctx, const float **dO);     /* valid until the next set_* / destroy */

/* ---- results (cleanup phase) -------------------------------------------- */
/* nnz floats in the entry order of the input (pattern is never permuted). */
int sddmm_get_values(sddmm_ctx *ctx, float *P_values);
/* Device address of P (nnz floats), valid until the next sddmm_set_* / destroy. */
int sddmm_get_values_device(sddmm_ctx *ctx, const float **dP);
int sddmm_last_stats(const sddmm_ctx *ctx, sddmm_stats *out);

/* ---- host helpers -------------------------------------------------------- */
/* nnz-balanced contiguous row partition into `parts` ranges of whole `stride`-row
 * groups: the smallest feasible maximum load, then greedy fill -- the contract of
 * CSR<T>::_dispatch (src/matrices/CSR.hpp:196-264).  start_idx[parts+1]; unused
 * trailing parts start at M.  Host only; this is how row panels are cut per device. */
int sddmm_partition_rows(int M, const int32_t *rowptr, int parts, int stride, int32_t *start_idx);

/* Library / device description for logs: "sddmm_amd <ver> gfx950 ..." */
const char *sddmm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SDDMM_AMD_H */
