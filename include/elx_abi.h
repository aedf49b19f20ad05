/*
 * C ABI of libelx_hip.so -- the optimizer-step kernels for gfx950 (MI355X).
 *
 * The library implements, over chunk-packed parameters, the device work of the reference's
 * ElixirOptimizer.step (elixir/wrapper/optimizer.py:192-220):
 *
 *   stats     overflow flag and sum of squares of the (still loss-scaled) gradients that sit in
 *             each low-precision chunk shard;
 *   update    unscale + Adam/AdamW on the fp32 master, exp_avg and exp_avg_sq held in flat
 *             per-chunk storage + low-precision writeback, in one pass;
 *   writeback the low-precision refresh alone (the skip-step branch and state loading).
 *
 * Conventions
 *   - plain C, no C++ or torch types; every pointer in a table is a DEVICE pointer;
 *   - the caller owns all memory (chunk buffers, tables, workspaces); the library allocates
 *     nothing and keeps no mutable global state; all entry points are reentrant (the one exception,
 *     elx_grad_stats_mt_static, says so in its own comment);
 *   - all device work is enqueued on the hipStream_t passed as `stream` (NULL = default
 *     stream) and is asynchronous with respect to the host; borrowed pointers must stay valid
 *     until that work has completed;
 *   - every function returns an int: 0 = success, > 0 = a hipError_t raised by a launch,
 *     < 0 = an ELX_E_* argument error.  An overflow in the gradients is data
 *     (ElxStats.overflow), never an error.
 */
#ifndef ELX_ABI_H
#define ELX_ABI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ELX_ABI_VERSION 3

/* element types of gradient / low-precision buffers */
enum { ELX_F32 = 0, ELX_F16 = 1, ELX_BF16 = 2, ELX_NONE = -1 };

/* argument errors */
enum {
    ELX_E_NULL = -1,     /* a required pointer is NULL */
    ELX_E_DTYPE = -2,    /* unknown or unsupported dtype combination */
    ELX_E_ALIGN = -3,    /* a chunk base pointer is not aligned to its element size */
    ELX_E_RANGE = -4,    /* begin >= end, end > n_valid, n_valid > n_alloc, bad segment range or hyper index */
    ELX_E_ORDER = -5,    /* segments of a chunk are not sorted by begin or overlap */
    ELX_E_TILES = -6,    /* tile_begin / total_tiles disagree with the chunk sizes */
    ELX_E_SIZE = -7,     /* a count is zero, out of its allowed range, or exceeds what a launch can address */
    ELX_E_STATE = -8     /* elx_grad_stats_mt_static: `stream` belongs to another GPU than the current one, or the
                            first call on a device was made while `stream` is capturing */
};

/* flags of the update, writeback and stats launches */
enum {
    ELX_FLAG_SCALAR_ONLY = 1u,   /* take the element-by-element path for every tile (set by the host when
                                    elx_check_tables reports base pointers that are not 16-byte aligned) */
    ELX_FLAG_KEEP_CACHED = 2u,   /* stats and landing launches: touch the gradients with ordinary loads / stores
                                    instead of non-temporal ones, so that they stay in the memory-side cache
                                    (256 MiB) for the update launch that reads them next.  Pays when all
                                    gradients of the launch fit that cache (2-5 % of the step at 64-256 MiB);
                                    a larger set streams faster without it (the stats pass of a 2.6 GB set is
                                    16 % slower with it).
                                    Update launches: the low-precision copy is written with stores that the
                                    memory-side cache takes in (over the gradients it replaces, when they are
                                    still there) and writes back later, instead of streaming stores.  Pays up
                                    to about 2 GB of low-precision shards (3 % of the step at 0.25-0.5 GB, 1 %
                                    at 1-2 GB); larger sets lose up to 1 % with it.
                                    Results never depend on it */
    ELX_FLAG_KEEP_STATE_CACHED = 4u  /* update launches: everything the launch touches (gradients, master, m, v,
                                    low-precision copy) fits the memory-side cache: ordinary loads, and every
                                    store as ELX_FLAG_KEEP_CACHED stores the low-precision copy, so that the
                                    next step finds the state there.  7 % of the step for 16 Mi fp32 elements
                                    with fp32 gradients (256 MiB in all); a set twice that size loses 14 %
                                    with it.  Implies ELX_FLAG_KEEP_CACHED.  Results never depend on it */
};

/*
 * One flat chunk: the paired low-precision / fp32 shards of the reference's Chunk
 * (elixir/chunk/core/chunk.py:59-139) plus the flat exp_avg / exp_avg_sq this build keeps beside
 * the master shard.  `grad` and `lowp_out` may be the same buffer: in the reference the
 * low-precision parameter shard holds the reduced gradients at step time (chunk.py:313) and is
 * overwritten with the refreshed parameters afterwards (chunk.py:414).
 */
typedef struct ElxChunk {
    const void *grad;    /* n_alloc elements of the gradient dtype; NULL = gradient is zero */
    void *lowp_out;      /* n_alloc elements of the low-precision dtype; NULL = no writeback */
    float *master;       /* n_alloc fp32 master weights */
    float *m;            /* n_alloc fp32 exp_avg */
    float *v;            /* n_alloc fp32 exp_avg_sq */
    uint64_t n_alloc;    /* shard_size: elements allocated, padding included */
    uint64_t n_valid;    /* elements of the head of the shard that hold tensors (valid_end clipped to n_alloc) */
    uint64_t tile_begin; /* launch-wide index of this chunk's first tile: sum over earlier chunks of
                            ceil(n_alloc / elx_tile_elems()); checked by elx_check_tables, not read by kernels */
    uint32_t seg_begin;  /* this chunk's segments are segs[seg_begin, seg_end) */
    uint32_t seg_end;
} ElxChunk;

/*
 * One tensor's slice [begin, end) of a chunk -- the (begin, end) pair of
 * elixir/wrapper/optimizer.py:240-244 -- and the index of the hyper-parameter record it uses.
 * Elements of a chunk that no segment covers (padding, tensors the optimizer does not own) are
 * not updated; they still take part in the writeback, as in chunk.py:414.
 */
typedef struct ElxSeg {
    uint64_t begin;
    uint64_t end;
    uint32_t hyper;
    uint32_t reserved;
} ElxSeg;

/* flags of ElxHyper */
enum {
    ELX_HYPER_L2 = 1u,          /* L2 mode: g += l2_wd * p before the moments */
    ELX_HYPER_LERP_FROM_G = 2u  /* 1-beta1 >= 0.5: m = g + lerp_w*(g-m) with lerp_w = (1-beta1)-1 */
};

/*
 * Hyper-parameters of one (param group, step count) pair, narrowed to fp32 on the host from the
 * float64 values a torch optimizer holds (torch/optim/adam.py:528-545):
 *   bc1 = 1 - beta1^step, bc2 = 1 - beta2^step (both 1 when bias correction is off)
 */
typedef struct ElxHyper {
    float decay_mul; /* AdamW: (float)(1 - lr*wd); 1.0f when there is no decoupled decay */
    float l2_wd;     /* L2 mode: (float)wd */
    float lerp_w;    /* (float)(1-beta1), or that minus 1 when ELX_HYPER_LERP_FROM_G */
    float beta2;     /* (float)beta2 */
    float omb2;      /* (float)(1-beta2) */
    float bc2_sqrt;  /* (float)sqrt(bc2) */
    float eps;       /* (float)eps */
    float neg_step;  /* (float)(-(lr/bc1)) */
    uint32_t flags;
    /* the gate: read only by elx_adam_step_gated_mt, written by elx_decide (whatever the caller puts
       here is overwritten) */
    float gate_div_scale; /* the step's div_scale, -1 when no unscale is needed */
    float gate_inv_scale; /* 1 / div_scale when that is exact */
    uint32_t gate;        /* unscale mode (0 none, 1 multiply by the reciprocal, 2 divide) | skip << 8 */
} ElxHyper;

/* Result of the stats pass for one chunk; also the element type of its partials workspace. */
typedef struct ElxStats {
    double sumsq;      /* sum over the valid elements of (double)(float)g * (float)g */
    uint32_t overflow; /* 1 if any valid element is +inf, -inf or NaN */
    uint32_t reserved;
} ElxStats;

/*
 * The decisions of one step as elx_decide leaves them in device memory for elx_adam_step_gated_mt, and
 * for the host to read back: elixir/wrapper/optimizer.py:137-183.
 */
typedef struct ElxDecision {
    float div_scale;       /* (float)combined_scale, -1 when no unscale is needed */
    float inv_scale;       /* 1 / div_scale when that is exact (div_scale a power of two), else 1 */
    uint32_t mode;         /* 0 no unscale, 1 multiply by inv_scale, 2 divide by div_scale */
    uint32_t skip;         /* 1: some chunk overflowed, the step must not update anything */
    double total_norm;     /* global L2 norm of the scaled gradients (0 when clipping is off) */
    double combined_scale; /* loss scale x clip coefficient as a float64, -1 when it equals 1 */
} ElxDecision;

/*
 * Control block of one step for elx_finish_decide: what changes from step to step, kept in memory so
 * that the launches of a step take the same arguments every time (and can be replayed from a recorded
 * HIP graph).  The host rewrites it before every step; it may live in device memory or in pinned host
 * memory (the kernel reads it with system-scope loads).  n_hypers ElxHyper records follow it directly.
 */
typedef struct ElxStepCtl {
    double loss_scale;  /* > 0 */
    double max_norm;    /* > 0 when clipping */
    uint32_t clipping;  /* 0 / 1 */
    uint32_t n_hypers;  /* records that follow; at most elx_max_ctl_hypers() and the max_hypers of the call */
    uint64_t seq;       /* any number the host chooses; echoed in ElxStepReport.seq */
} ElxStepCtl;

/*
 * What elx_finish_decide reports back: the decision, then one ElxStats record per chunk directly behind
 * this header.  Written with system-scope stores, `seq` last (release): a host that polls `seq` in pinned
 * host memory and finds the number it put into the control block may read the rest.
 */
typedef struct ElxStepReport {
    ElxDecision decision;
    uint64_t seq;
    uint32_t n_chunks;
    int32_t status;     /* 0, or ELX_E_RANGE when the control block was unusable (then decision.skip = 1) */
} ElxStepReport;

/* ABI version of the loaded library (ELX_ABI_VERSION). */
int elx_version(void);

/*
 * The first 16 hex digits of the SHA-256 over the sources the library was built from (its .hip / .cpp / .h
 * files and this header, in sorted order of their names), as the build passed it in; "" for a build that
 * did not.  A binding compares it with the same digest of the sources beside it and refuses a library
 * that was built from other sources.
 */
const char *elx_source_sha(void);

/* Text for a return code of this library (argument errors and hipError_t values). */
const char *elx_strerror(int code);

/* Elements per tile of the update / writeback launch; ElxChunk.tile_begin is counted in these. */
uint32_t elx_tile_elems(void);

/* sizeof() of the table records as compiled, for bindings to verify their mirrors. */
uint32_t elx_sizeof_chunk(void);
uint32_t elx_sizeof_seg(void);
uint32_t elx_sizeof_hyper(void);
uint32_t elx_sizeof_stats(void);
uint32_t elx_sizeof_decision(void);
uint32_t elx_sizeof_step_ctl(void);
uint32_t elx_sizeof_step_report(void);

/*
 * Host-side validation of HOST copies of the tables, to be called once before they are uploaded:
 * NULL / dtype / range / ordering / tile checks as listed under the ELX_E_* codes.  On success
 * writes
 *   *total_tiles          the tile count over all chunks (one workgroup per tile, < 2^31),
 *   *max_tiles_per_chunk  the largest tile count of any chunk (the x extent of the 2-D grid),
 *   *all_aligned16        whether every non-NULL base pointer is 16-byte aligned (if not, pass
 *                         ELX_FLAG_SCALAR_ONLY to the launches).
 * lowp_dtype may be ELX_NONE when no chunk has a lowp_out buffer.
 * Replaces the per-tensor asserts and range bookkeeping of optimizer.py:238-265 at the boundary.
 */
int elx_check_tables(const ElxChunk *h_chunks, uint32_t n_chunks, const ElxSeg *h_segs, uint32_t n_segs,
                     uint32_t n_hypers, int grad_dtype, int lowp_dtype, uint64_t *total_tiles,
                     uint32_t *max_tiles_per_chunk, int *all_aligned16);

/*
 * Stats pass over grad[0, n_valid) of every chunk: replaces Chunk.set_overflow_flag and
 * Chunk.set_l2_norm (elixir/chunk/core/chunk.py:214-221) for a whole chunk list in two launches.
 *   d_partials  workspace of n_chunks * blocks_per_chunk ElxStats records (contents ignored)
 *   d_stats     n_chunks results; the reduction order is fixed, so results are reproducible
 *   blocks_per_chunk  1..1024
 *   flags       0, ELX_FLAG_SCALAR_ONLY (gradient bases not 16-byte aligned), ELX_FLAG_KEEP_CACHED, or both;
 *               any other bit: ELX_E_RANGE
 */
int elx_grad_stats_mt(const ElxChunk *d_chunks, uint32_t n_chunks, int grad_dtype, uint32_t blocks_per_chunk,
                      ElxStats *d_partials, ElxStats *d_stats, int flags, void *stream);

/*
 * The first launch of elx_grad_stats_mt alone: n_chunks * blocks_per_chunk partials, chunk by chunk, left
 * for elx_finish_decide (or any fold of the caller's) to reduce.
 */
int elx_grad_partials_mt(const ElxChunk *d_chunks, uint32_t n_chunks, int grad_dtype, uint32_t blocks_per_chunk,
                         ElxStats *d_partials, int flags, void *stream);

/*
 * The fold of the partials and elx_decide in one launch whose arguments do not change from step to step:
 * loss scale, clipping threshold and the hyper records of the step come from *ctl.  Per chunk the
 * blocks_per_chunk partials at d_partials are folded exactly as elx_grad_stats_mt folds them into
 * d_stats (with blocks_per_chunk = 1 the "partials" are finished records, e.g. those a landing launch
 * left: 1..elx_land_max_blocks()); then the decisions of optimizer.py:137-183 are taken as by elx_decide,
 * the ctl->n_hypers records behind *ctl are copied to d_hypers with their gate words filled in (the table
 * elx_adam_step_gated_mt reads next on the same stream), *d_decision is written and, when `report` is not
 * NULL, so is the report (see ElxStepReport; room for n_chunks ElxStats records behind the header).
 *   max_hypers  capacity of d_hypers in records, at most elx_max_ctl_hypers(); *ctl must be readable for
 *               sizeof(ElxStepCtl) + max_hypers * sizeof(ElxHyper) bytes (the kernel fetches the first
 *               records together with the header, before it knows n_hypers)
 *   d_counter   one uint32 of device memory, zero before the first call; the launch leaves it zero
 * An unusable control block (loss_scale <= 0, n_hypers > max_hypers ...) cannot be refused by the host
 * (it may be device memory): the kernel then sets the skip gate in all max_hypers records, so that the
 * update launch changes nothing, and reports status ELX_E_RANGE.
 */
int elx_finish_decide(const ElxStats *d_partials, uint32_t n_chunks, uint32_t blocks_per_chunk, ElxStats *d_stats,
                      const ElxStepCtl *ctl, ElxHyper *d_hypers, uint32_t max_hypers, ElxDecision *d_decision,
                      ElxStepReport *report, uint32_t *d_counter, void *stream);

uint32_t elx_max_ctl_hypers(void);

/*
 * elx_finish_decide that also arms the row table of the gated update launch: a skipped step
 * (optimizer.py:196-203) then costs what its refresh costs.  d_gated_rows is a second device copy of the n_rows
 * ElxChunk records at d_rows, and the table handed to elx_adam_step_gated_mt next on the same stream.  When the
 * step is skipped the deciding workgroup zeroes the n_valid column of d_gated_rows; at the first step that
 * happens after that it writes the counts of d_rows (which nobody writes) back.  A record without valid elements
 * only has its low-precision copy refreshed, and the update launch knows that from the record it fetches first of
 * all, before it has issued a load: a skipped step moves 4 B + 2 B per element instead of 14 B + 2 B, and an
 * ordinary step pays nothing (reading the skip flag itself at the top of the update kernel cost every step
 * 3.6 %).
 *   d_armed  one uint32 of device memory that belongs to d_gated_rows: 0 while the table holds the counts of
 *            d_rows (as a fresh copy does), 1 while it holds zeros; read and kept by the launch, so that an
 *            ordinary step after an ordinary step writes nothing
 * d_gated_rows NULL: exactly elx_finish_decide.  d_rows == d_gated_rows: ELX_E_RANGE.
 */
int elx_finish_decide_rows(const ElxStats *d_partials, uint32_t n_chunks, uint32_t blocks_per_chunk, ElxStats *d_stats,
                           const ElxStepCtl *ctl, ElxHyper *d_hypers, uint32_t max_hypers, ElxDecision *d_decision,
                           ElxStepReport *report, uint32_t *d_counter, const ElxChunk *d_rows, ElxChunk *d_gated_rows,
                           uint32_t n_rows, uint32_t *d_armed, void *stream);

/*
 * elx_grad_stats_mt without a workspace argument, for callers that cannot allocate one (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  The partials go into a fixed array of elx_static_partials() ElxStats records (1 MiB)
 * that the library holds in the memory of every GPU it runs on until the process ends; the call
 * allocates and frees nothing.  Same kernels, same reduction order, same results as
 * elx_grad_stats_mt.
 *   - n_chunks * blocks_per_chunk must not exceed elx_static_partials(): ELX_E_SIZE otherwise;
 *   - the device that owns `stream` must be the current device of the calling thread: ELX_E_STATE
 *     otherwise.  The array's address is looked up once per device, on the first call there: make that
 *     first call outside stream capture (under capture it is refused with ELX_E_STATE and nothing is
 *     launched), later ones may be captured;
 *   - all calls on one GPU share the array: two calls whose work overlaps on that GPU (different
 *     streams, or different threads) race.  Calls on one stream are ordered and safe; the array keeps
 *     the last call's partials, and every record a call reads it has written first.
 */
int elx_grad_stats_mt_static(const ElxChunk *d_chunks, uint32_t n_chunks, int grad_dtype, uint32_t blocks_per_chunk,
                             ElxStats *d_stats, int flags, void *stream);

/* Capacity, in ElxStats records, of the fixed partials array of elx_grad_stats_mt_static. */
uint32_t elx_static_partials(void);

/*
 * Fused update over every chunk: for each element inside a segment
 *   g = (float)grad; if (div_scale > 0) g /= div_scale;            -- the div_scale of optimizer.py:216
 *   Adam / AdamW on master, m, v with the segment's ElxHyper;
 * and for every element of the chunk (padding included), when lowp_out is set,
 *   lowp_out = round-to-nearest-even(master)                       -- chunk.py:414
 * Replaces the inner optimizer's step over the fake parameters plus Chunk.optim_update.
 *
 * A "chunk" of this table need not be a whole shard: callers get the best throughput by listing
 * equal-sized blocks of the shards that contain tensors as separate records and leaving runs of
 * pure padding to elx_writeback_mt (whose workgroups move four times as much per tile and read
 * no tables).
 *   total_tiles            as returned by elx_check_tables for these tables
 *   grid_tiles_per_chunk   x extent of the 2-D launch grid (grid_tiles_per_chunk, n_chunks): record y,
 *                          tile x, nothing is looked up.  At least the max_tiles_per_chunk that
 *                          elx_check_tables reported; 0, or a grid that cannot hold total_tiles, is
 *                          ELX_E_TILES.  n_chunks <= 65535: list a long shard as several records
 *   flags          0, ELX_FLAG_SCALAR_ONLY (elx_check_tables found a base pointer that is not 16-byte
 *                  aligned), ELX_FLAG_KEEP_CACHED / ELX_FLAG_KEEP_STATE_CACHED (cache policy, above), or a sum;
 *                  any other bit is ELX_E_RANGE
 *   blocks_per_cu  cap on resident workgroups per compute unit, 3..32; 0 = the library default (13 for
 *                  16-bit gradients, 12 for fp32 gradients).
 *                  The update streams best with a shallow, orderly queue of memory requests.
 */
int elx_adam_step_mt(const ElxChunk *d_chunks, uint32_t n_chunks, const ElxSeg *d_segs, uint32_t n_segs,
                     const ElxHyper *d_hypers, uint32_t n_hypers, uint64_t total_tiles,
                     uint32_t grid_tiles_per_chunk, float div_scale, int grad_dtype, int lowp_dtype,
                     uint32_t flags, uint32_t blocks_per_cu, void *stream);

/*
 * Writes n_hypers records from HOST memory into the device table d_hypers, ordered on `stream`: the
 * records travel in the arguments of a one-wavefront launch (32 per launch), so there is no staging
 * buffer to keep alive and no host-to-device copy; h_hypers may be reused as soon as the call returns.
 * This is how a host-decided or standalone step gets its per-step scalars (bias corrections, learning
 * rate) to the device: the `lr`, `betas`, `step` ... arguments of the reference's
 * fused_optim.multi_tensor_adam call (optimizer.py:216 -> HybridAdam.step).
 */
int elx_put_hypers(const ElxHyper *h_hypers, uint32_t n_hypers, ElxHyper *d_hypers, void *stream);

/*
 * The whole of `self.optim.step(div_scale=...)` (optimizer.py:216) for a host-decided or standalone step,
 * in one call: the hyper records come from HOST memory (h_hypers, reusable as soon as the call returns).
 * Up to 32 records travel in the arguments of the update launch itself, which reads them there: one
 * launch, and d_hypers is NOT written.  More than 32: elx_put_hypers into d_hypers followed by
 * elx_adam_step_mt on that table, the launches going out back to back.  The other arguments are those
 * of elx_adam_step_mt; nothing is launched when the update would be refused.
 */
int elx_adam_step_put_mt(const ElxChunk *d_chunks, uint32_t n_chunks, const ElxSeg *d_segs, uint32_t n_segs,
                         const ElxHyper *h_hypers, ElxHyper *d_hypers, uint32_t n_hypers, uint64_t total_tiles,
                         uint32_t grid_tiles_per_chunk, float div_scale, int grad_dtype, int lowp_dtype, uint32_t flags,
                         uint32_t blocks_per_cu, void *stream);

/*
 * The host decisions of optimizer.py:137-183 taken on the device, so that the update can be enqueued
 * without waiting for the flags to reach the host: one thread reads the n_chunks records of a stats or
 * landing launch (in the order given), ORs the overflow flags and, with `clipping`, forms the global
 * norm and the clip coefficient in the float64 arithmetic the reference's Python uses
 *   l2_i = (double)(float)sqrt(sumsq_i) squared;  norm = sqrt((double)(float)sum_i l2_i);
 *   clip = ((norm / loss_scale) + 1e-6) / max_norm;  combined = clip > 1 ? clip * loss_scale : loss_scale
 * and writes *d_decision and the gate words of the n_hypers records at d_hypers (the table of the
 * update launch that follows).  loss_scale > 0; max_norm > 0 when clipping.
 */
int elx_decide(const ElxStats *d_stats, uint32_t n_chunks, double loss_scale, double max_norm, int clipping,
               ElxHyper *d_hypers, uint32_t n_hypers, ElxDecision *d_decision, void *stream);

/*
 * elx_adam_step_mt with the unscale parameters and the skip flag read from the gate words of the hyper
 * records when the kernel runs (elx_decide on the same d_hypers must precede it on the same stream);
 * they arrive with the record a tile loads anyway.  With skip set nothing is updated and every element
 * of every record only has its low-precision copy refreshed -- what the skip branch of
 * optimizer.py:196-203 does through Chunk.optim_update.
 */
int elx_adam_step_gated_mt(const ElxChunk *d_chunks, uint32_t n_chunks, const ElxSeg *d_segs, uint32_t n_segs,
                           const ElxHyper *d_hypers, uint32_t n_hypers, uint64_t total_tiles,
                           uint32_t grid_tiles_per_chunk, int grad_dtype, int lowp_dtype, uint32_t flags,
                           uint32_t blocks_per_cu, void *stream);

/*
 * Low-precision refresh alone: lowp_out[0, n_alloc) = round-to-nearest-even(master) for every
 * record (only lowp_out, master and n_alloc are read).  The skip-step branch
 * (optimizer.py:196-203 -> chunk.py:403-414), state loading (elixir/wrapper/module.py:343) and the
 * padding runs left out of an update launch use it.
 *   blocks_per_chunk  workgroups per record, 1..2^20; best: ceil(max n_alloc / elx_refresh_piece_elems()),
 *                     one piece per workgroup, with records of about equal size (with fewer, a
 *                     workgroup takes several pieces)
 */
int elx_writeback_mt(const ElxChunk *d_chunks, uint32_t n_chunks, int lowp_dtype, uint32_t blocks_per_chunk,
                     uint32_t flags, void *stream);

/* Elements of one piece of the refresh launch (one wavefront, four 128-bit loads per lane). */
uint32_t elx_refresh_piece_elems(void);

/*
 * The same two passes for ONE buffer described in the arguments: no table in device memory.
 *   elx_writeback   lowp[0, n) = round-to-nearest-even(master[0, n)): Chunk.optim_update for one chunk
 *                   (chunk.py:403-414) and the source copy of a gather whose refresh was deferred
 *                   (chunk.py:264-270, 475-482); `master` may be pinned host memory
 *   elx_grad_stats  flags of grad[0, n): Chunk.set_overflow_flag / set_l2_norm for one chunk
 *                   (chunk.py:214-221); blocks = 1..1024 workgroups, d_partials holds `blocks`
 *                   records, *d_stats receives the result
 */
int elx_writeback(const float *master, void *lowp, int lowp_dtype, uint64_t n, void *stream);
int elx_grad_stats(const void *grad, int grad_dtype, uint64_t n, uint32_t blocks, ElxStats *d_partials,
                   ElxStats *d_stats, void *stream);

/*
 * Gradient landing with the stats riding the copy: for every row
 *   lowp_out[i] = cast_dst(grad[i])                          for i in [0, n_alloc)
 * and d_stats[row] = overflow flag and sum of squares of lowp_out[0, n_valid) as stored.  Replaces the
 * tail of Chunk.reduce, `__update_shard(reduce_buffer, self.shard)` (elixir/chunk/core/chunk.py:309-315,
 * 484-489), fused with Chunk.update_extra_reduce_info (chunk.py:345-356): the flags are known when
 * the gradients have landed, and the optimizer step needs no pass of its own over them.
 * A row reads `grad` (the source: n_alloc elements of src_dtype; NULL = all zeros), `lowp_out` (the
 * destination: n_alloc elements of dst_dtype), n_alloc and n_valid; nothing else.  A row can be a whole
 * shard with the payload slice that belongs to it, or any piece of one: listing every tensor's
 * gradient as rows (cut into equal blocks) with the gaps and the padding as zero rows lands a chunk
 * straight from the per-parameter gradients, which also replaces the copies of
 * Chunk.copy_tensor_to_chunk_slice (chunk.py:386-393) and the intermediate payload.
 *   d_slot_offsets / n_slots  NULL: one result record per row (n_slots is ignored).  Otherwise
 *              n_slots + 1 ascending row indices: the rows [offsets[s], offsets[s+1]) feed d_stats[s]
 *              (the rows of one chunk are consecutive), offsets[0] = 0, offsets[n_slots] = n_rows
 *   src_dtype / dst_dtype  equal, or fp32 -> fp16 / bf16 (a payload reduced in fp32, chunk.py:291-296)
 *   mul        1.0f: plain copy / cast.  Otherwise each element is multiplied in fp32, rounded to
 *              src_dtype and then cast, as the in-place `reduce_buffer /= pg_size` of chunk.py:299
 *              does on the device for mul = 1.0f / pg_size.  Must be finite and > 0.
 *   blocks_per_row  workgroups per row, 1..elx_land_max_blocks().  One workgroup lands one tile of
 *              elx_land_tile_elems(src_dtype) elements at a time; the launch streams best with one
 *              tile per workgroup, blocks_per_row = ceil(max n_alloc / tile); with fewer, a workgroup
 *              takes several tiles
 *   d_partials workspace of n_rows * blocks_per_row + n_slots * elx_land_fold_blocks() ElxStats
 *              records (contents ignored)
 *   d_stats    n_slots results; fixed reduction order
 *   flags      ELX_FLAG_SCALAR_ONLY forces the element-by-element path (rows whose ends are not both
 *              16-byte aligned take it by themselves); ELX_FLAG_KEEP_CACHED writes the destination with
 *              ordinary instead of non-temporal stores, so that a destination of at most 256 MiB is still
 *              in the memory-side cache when the optimizer step reads it (a loss on larger ones);
 *              bits 8..15: cap on resident workgroups per
 *              compute unit, 3..32 (0 = the library default: 10, or 13 when an fp32 payload lands in a
 *              16-bit shard)
 */
int elx_land_grads_mt(const ElxChunk *d_rows, uint32_t n_rows, const uint32_t *d_slot_offsets, uint32_t n_slots,
                      int src_dtype, int dst_dtype, float mul, uint32_t blocks_per_row, ElxStats *d_partials,
                      ElxStats *d_stats, uint32_t flags, void *stream);

/*
 * Host-side validation of HOST copies of a landing table before it is uploaded (the launch itself
 * sees device pointers only): NULL destination, element alignment, n_valid <= n_alloc, slot offsets
 * that start at 0, end at n_rows and never decrease (h_slot_offsets may be NULL: one slot per row).
 * On success *blocks_per_row is the one-tile-per-workgroup grid width, ceil(max n_alloc / tile), or
 * elx_land_max_blocks() when the longest row has more tiles than that (its workgroups take several).
 */
int elx_check_land_rows(const ElxChunk *h_rows, uint32_t n_rows, const uint32_t *h_slot_offsets, uint32_t n_slots,
                        int src_dtype, int dst_dtype, uint32_t *blocks_per_row);

uint32_t elx_land_max_blocks(void);
uint32_t elx_land_tile_elems(int src_dtype);
uint32_t elx_land_fold_blocks(void);

/*
 * Two host-side queries (no GPU work) about what a launch would do with an argument:
 *   elx_unscale_mode         how an update launch divides the gradients by div_scale (the div_scale of
 *                            optimizer.py:216): returns 0 not at all (div_scale <= 0), 1 by an exact multiply
 *                            with *inv_scale = 1 / div_scale (div_scale a power of two whose reciprocal is a
 *                            normal fp32 number: same bits as the division), 2 by an IEEE division;
 *                            inv_scale may be NULL
 *   elx_occupancy_lds_bytes  the dynamic LDS reservation by which an update launch holds `blocks_per_cu`
 *                            workgroups per compute unit (0 = the default for fp32 gradients); ELX_E_SIZE
 *                            outside 3..32
 */
int elx_unscale_mode(float div_scale, float *inv_scale);
int elx_occupancy_lds_bytes(uint32_t blocks_per_cu, uint32_t *lds_bytes);

#ifdef __cplusplus
}
#endif
#endif /* ELX_ABI_H */
