/*
 * galvatron_dp_hip.h -- C ABI of libgalvatron_dp_hip.so
 *
 * MI355X (gfx950) implementation of the Galvatron search engine's layer-wise
 * dynamic program.  Every entry point below replaces, for one or many DP
 * instances, the single reference callable
 *
 *     galvatron_dp_core.dynamic_programming_core(layer_num, max_mem, strategy_num,
 *         v_data, _mark, _f, inter_cost, intra_cost,
 *         other_mem_cost, other_time_cost, res_list)          csrc/dp_core.cpp:24-35,122-124
 *
 * as it is called from DPAlg.fit
 * (galvatron/core/search_engine/dynamic_programming.py:77-91).
 *
 * Plain C: pointers and sizes only.  All input and output pointers are HOST
 * memory owned by the caller and borrowed for the duration of the call (or, for
 * a plan, until gdp_plan_create returns: inputs are copied to the device
 * there).  The library is re-entrant: no call shares mutable state with another
 * call, so it may be used from many threads at once (ctypes releases the GIL).
 * There is no CPU fallback: without a usable HIP device every compute entry
 * point fails with GDP_E_HIP.
 */
#ifndef GALVATRON_DP_HIP_H
#define GALVATRON_DP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GDP_VERSION 102 /* major*10000 + minor*100 + patch */

/* return codes */
#define GDP_OK 0
#define GDP_E_BADARG (-1)      /* null pointer, non-positive size, S / V / L above GDP_MAX_*, negative mem or other_mem, ... */
#define GDP_E_UNSUPPORTED (-2) /* kept for callers built against earlier headers; no input is answered with it any more */
#define GDP_E_NONFINITE (-3)   /* NaN or -inf in a cost array (the reference's result is then order-dependent) */
#define GDP_E_NOMEM (-4)       /* device or host allocation failed */
#define GDP_E_HIP (-5)         /* any other HIP runtime error; text in gdp_last_error() */

#define GDP_MAX_S 1024      /* strategies per layer */
#define GDP_MAX_V (1 << 30) /* budget bins */
#define GDP_MAX_L 65535     /* layers */
#define GDP_MAX_S_MARKS 256 /* ... when the argmin table is kept (GDP_KEEP_MARKS, GDP_EXPORT_MARK): its entries are bytes */

/* gdp_problem.flags */
#define GDP_EXPORT_F 1u    /* write result.f_out    (final f, reference layout [V][S])       */
#define GDP_EXPORT_MARK 2u /* write result.mark_out (argmin table, reference layout [L][V][S]) */
#define GDP_LAUNCH_FUSED 4u     /* lay the plan out for, and use, ONE launch over all layers          */
#define GDP_LAUNCH_PER_LAYER 8u /* one launch per layer; default: chosen by size                          */
#define GDP_COMPUTE_ALL 16u     /* carry out every one of the L*V*S*S relaxations (see gdp_timing.executed) */
#define GDP_KEEP_MARKS 32u      /* store the argmin of every cell while relaxing, as the reference does
                                   (csrc/dp_core.cpp:70-72).  Default: the relaxation computes costs only, the
                                   cost buffers of all layers stay in device memory, and the backtrack recomputes
                                   the argmin of the L cells on its path -- same results, two fifths fewer
                                   instructions.  Implied by GDP_EXPORT_MARK; chosen by the library when the
                                   per-layer cost buffers do not fit in device memory (GDP_E_NOMEM instead if S
                                   is above GDP_MAX_S_MARKS). */

/* One DP instance == one reference call.  Field <- reference argument (csrc/dp_core.cpp:24-35):
 *   L <- layer_num, V <- max_mem (number of budget bins, valid v in [0,V)),
 *   S <- strategy_num, mem <- v_data, intra <- intra_cost, inter <- inter_cost,
 *   other_mem/other_time <- other_mem_cost/other_time_cost values, in the caller's key order
 *   (the dictionary keys themselves are never used by the arithmetic),
 *   f0 <- the contents of _f on entry: the reference relaxes in place, starting from whatever the
 *   caller's array holds (csrc/dp_core.cpp:46-47,67; DPAlg hands in zeros, dynamic_programming.py:16). */
typedef struct gdp_problem {
    int32_t L, V, S;
    const int32_t *mem;         /* [L][S]  memory cost in bins, >= 0.  An entry of 0 is computed with the reference's
                                            in-place semantics (such a cell reads its own row, where lower strategies
                                            already hold the layer's values: csrc/dp_core.cpp:58-73); a plan with such
                                            entries runs one launch per layer.  The reference's walk back does not
                                            know of those same-layer candidates and can then arrive at a negative
                                            row, with which it indexes its argmin table (csrc/dp_core.cpp:105-113:
                                            undefined behaviour); the library stops there and reports the key as
                                            infeasible (total +inf, remaining -1)                              */
    const double *intra;        /* [L][S]                                                          */
    const double *inter;        /* [n_inter][S][S], row = source strategy, column = target        */
    const int32_t *inter_index; /* [L] layer -> matrix in `inter`; NULL means n_inter == L, identity */
    int32_t n_inter;
    int32_t n_key;              /* number of (other_mem, other_time) pairs to finish for           */
    const int64_t *other_mem;   /* [n_key]  every entry must be >= 0 (start row V-1-other_mem inside the table;
                                            an entry above V-1 is an infeasible key: total +inf, remaining -1) */
    const double *other_time;   /* [n_key]                                                         */
    uint32_t flags;
    const double *f0;           /* [V][S] initial costs, or NULL for all zeros.  Entries may be finite or +inf;
                                            NaN and -inf are refused like in the cost arrays (GDP_E_NONFINITE), and
                                            so is -0.0 (GDP_E_BADARG): the reference keeps the first of two equal
                                            candidates, so with a negative zero among them the sign of a zero cost
                                            would depend on the order of evaluation.  An array of zeros is treated
                                            as NULL.                                                          */
} gdp_problem;

/* Outputs of one instance <- reference return values / written arguments (csrc/dp_core.cpp:78-119):
 *   total[k]     <- total_cost[key k]     (+inf when infeasible)
 *   remaining[k] <- remaining_mem[key k]  (-1 when infeasible)
 *   res[k][0..L) <- res_list[key k]; rows of infeasible keys are left untouched, as the
 *                   reference leaves the caller's -1 fill                          */
typedef struct gdp_result {
    double *total;      /* [n_key]                                   */
    int32_t *remaining; /* [n_key]                                   */
    int32_t *res;       /* [n_key][L]                                */
    double *f_out;      /* [V][S]    or NULL (needs GDP_EXPORT_F)    */
    int32_t *mark_out;  /* [L][V][S] or NULL (needs GDP_EXPORT_MARK) */
} gdp_result;

/* Device-side timings of one gdp_plan_run, taken with HIP events on the plan's stream. */
typedef struct gdp_timing {
    float total_ms;        /* first kernel to last kernel (relaxation layers + epilogue)      */
    float relax_ms;        /* sum of the per-launch durations of the relaxation kernel         */
    int32_t relax_launches;
    int32_t fused;         /* 1: all layers in one launch, 0: one launch per layer             */
    double relaxations;    /* sum over instances of L*V*S*S                                    */
    double executed;       /* relaxations actually carried out: cells whose sources are all +inf, and cells
                              that no requested start row can reach back to, are not computed           */
    double relax_bytes;    /* algorithmic HBM bytes of the relaxation kernels (f read+write, argmin write if kept) */
    /* how the plan was laid out (of its first group of instances with one S) */
    int32_t tile_ts;       /* target strategies per register tile                               */
    int32_t tile_r;        /* budget rows per lane                                              */
    int32_t keep_marks;    /* 1: the argmin table is stored while relaxing                      */
    int32_t chunk;         /* instances taken through a fused launch together; 0: all, layer by layer */
    int32_t latency_variant; /* > 0: per-layer launches use the kernel variant for launches with few waves,
                                with the source strategies of a task on this many waves (1, 2 or 4) */
    int32_t flow;          /* 1: all layers in one launch whose tasks wait on the cost cells themselves (small plans) */
    int32_t fused_split;   /* fused launches: waves that share the source strategies of a wave task (1 or 2)         */
} gdp_timing;

typedef struct gdp_plan gdp_plan;

/* Solve one instance: validate, upload, run, download.  Replaces one
 * dynamic_programming_core call (csrc/dp_core.cpp:24-120). */
int gdp_solve(const gdp_problem *p, gdp_result *r);

/* Solve n independent instances (e.g. every pipeline stage of every pp_deg, or a whole
 * bsz x chunk sweep: the DPAlg.fit calls issued from dynamic_programming.py:446-488 and
 * search_engine.py:477-498) with one launch grid per layer index.  A batch whose cost buffers would
 * exceed GALVATRON_DP_ARENA_MB (default 8192) of device memory is solved in consecutive parts that
 * reuse one allocation. */
int gdp_solve_batch(int32_t n, const gdp_problem *const *p, gdp_result *const *r);

/* gdp_solve for callers that cannot allocate.  No counterpart in the reference: it exists for callers that
 * may not obtain memory while they run -- serving loops that must stay off the allocator, harnesses that
 * forbid hipMalloc.  (Not for use while a stream is being captured in hipStreamCaptureModeGlobal: the call
 * makes synchronous copies and launches on the null stream, both prohibited then.)  Same arguments (host
 * pointers, borrowed for the call) and the same results, bit for bit, as gdp_solve, but the call
 * obtains no device memory, no page-locked memory, no stream and no event, and uses no host allocator:
 * its cost buffers, argmin table, tables and results live in one static device array of
 * GDP_STATIC_SCRATCH_BYTES that every device the library runs on holds until the process ends, the
 * inputs' device layout is built in a fixed host array, and the work runs on the null stream with
 * synchronous copies.  It keeps two cost buffers and the one-byte argmin table (the layout of
 * GDP_KEEP_MARKS), one launch per layer, every cell computed.
 *   - An instance that needs more than the array (roughly 17*(V + max mem)*(S+1) + L*S*V bytes, or
 *     tables above 8 MiB) is refused with GDP_E_NOMEM and a message that gives both sizes; so are
 *     S > GDP_MAX_S_MARKS and the export flags (GDP_E_BADARG).  Other flags are ignored.
 *   - All calls of a process share the array of their device, which keeps what the last call left; a
 *     call rewrites everything it reads, and calls take a process-wide lock, so they run one after the
 *     other.  Work that other code queues on the null stream is ordered with it as usual. */
#ifndef GDP_STATIC_SCRATCH_BYTES
#define GDP_STATIC_SCRATCH_BYTES (64 << 20) /* held on every device the library runs on, by every process that loads it */
#endif
int gdp_solve_static(const gdp_problem *p, gdp_result *r);

/* The same in three steps, so that a caller (or a benchmark) can keep inputs resident in
 * device memory and run the device part repeatedly:
 *   create  -- validate + allocate + copy inputs to the device
 *   run     -- layer kernels + on-device backtrack; timing may be NULL.
 *              timing_mode 0: none, 1: total_ms only, 2: also per-launch relaxation events
 *   fetch   -- copy results of the last run to the caller's arrays
 *   destroy -- release everything                                              */
int gdp_plan_create(int32_t n, const gdp_problem *const *p, gdp_plan **out);
int gdp_plan_run(gdp_plan *plan, int32_t timing_mode, gdp_timing *timing);
int gdp_plan_fetch(gdp_plan *plan, gdp_result *const *r);
void gdp_plan_destroy(gdp_plan *plan);

/* Tuning / test knobs of a plan (no counterpart in the reference).
 *   GDP_OPT_FUSED      1: all layers run in ONE launch (grid.y = layer), a workgroup waits on the
 *                      completion counters of the tiles it reads; 0: one launch per layer.  Results
 *                      are identical; the default is chosen by problem size.  A plan that keeps only
 *                      two cost buffers (GDP_KEEP_MARKS together with GDP_LAUNCH_PER_LAYER, or per-layer
 *                      buffers that did not fit in device memory) cannot be switched to 1.
 *   GDP_OPT_SPIN_LIMIT polls a waiting wavefront makes before it gives up; when that happens the
 *                      launch drains normally, the plan switches itself to one launch per layer
 *                      and the run is repeated that way (GDP_E_HIP with GDP_OPT_NO_FALLBACK).  Default: a
 *                      time, not a count -- 50 times what the plan's relaxations take at 5e12 per second,
 *                      between 5 ms and 1 s -- turned into polls per launch scheme.  A plan that gave up
 *                      is armed again with its launch scheme once GALVATRON_DP_SHARED_BACKOFF_MS (default
 *                      30000) have passed. */
#define GDP_OPT_FUSED 1
#define GDP_OPT_SPIN_LIMIT 2
#define GDP_OPT_POISON 3 /* test aid: NaN-fill every not-yet-written cost buffer before each run */
#define GDP_OPT_NO_FALLBACK 4 /* test aid: an abandoned fused launch is an error, not a switch to per-layer */
#define GDP_OPT_FLOW 5 /* 1: all layers in one launch whose tasks wait on the cost cells themselves: before a run
                          every cell it writes holds NaN, a task reads its cost rows at agent scope and asks again
                          for rows that are not whole yet.  Chosen by the library for plans too small for
                          GDP_OPT_FUSED to pay (unless a launch scheme was asked for); only a plan laid out for it
                          can be switched to 1.  0: one launch per layer.  Waits are bounded like GDP_OPT_FUSED's. */
#define GDP_OPT_DEBUG_STALL 6 /* test aid: in launches whose workgroups wait (GDP_OPT_FUSED, GDP_OPT_FLOW) the tasks of
                                 the first layer leave out the signal the next layer waits for, so that every such wait
                                 runs into its bound: the launch drains, every kernel ends normally, and the solve is
                                 repeated with one launch per layer */
int gdp_plan_set_option(gdp_plan *plan, int32_t option, int64_t value);

/* Frees the device allocations that finished plans left behind for reuse (no counterpart in the
 * reference).  The library keeps them, up to GALVATRON_DP_CACHE_MB in total (default 20480 or an eighth of the device memory, whichever is less; 0 keeps
 * nothing), because obtaining device memory costs far more than a solve.  Finished plans also leave
 * their stream, two events and page-locked result buffer for the next plan (at most 64 sets; creating
 * and destroying a stream takes a third as long as a small solve); this call releases those too. */
void gdp_cache_trim(void);

/* Test aid (no counterpart in the reference): validates the problems, lays a plan out exactly as
 * gdp_plan_create would for a device with num_cu compute units and lds_per_cu bytes of LDS per unit --
 * once in the default layout and once in the one that keeps the argmin table -- and checks every
 * address the kernels would form from the resulting tables against the sub-allocation it must stay
 * in.  Needs no device: nothing is allocated, uploaded or launched.  GDP_OK, a validation error, or
 * GDP_E_HIP with the violated bound in gdp_last_error().  The plan options that can be preset from the
 * environment (GALVATRON_DP_FUSED, _SKIP, _TILE_TS, _TILE_R, _CHUNK, _LATENCY_VARIANT ...) apply. */
int gdp_debug_check_layout(int32_t n, const gdp_problem *const *p, int32_t num_cu, int64_t lds_per_cu);

/* Test aid (no counterpart in the reference).  After a launch whose workgroups wait (GDP_OPT_FUSED,
 * GDP_OPT_FLOW) has been given up with the default spin limit, the library takes the device to be shared
 * with another process and, for the next 30 seconds (GALVATRON_DP_SHARED_BACKOFF_MS), chooses one launch per layer wherever the choice is
 * its own (explicit requests -- flags, options, environment -- still count).  This call puts the library
 * into that state (1) or ends it (0) without a launch having to time out. */
void gdp_debug_shared_device(int32_t seems_shared);

/* Benchmark aid (no counterpart in the reference): what the gdp_solve_batch calls of the whole process did
 * between gdp_batch_stats_begin() and gdp_batch_stats_end().  While it is on, every part of a batch is
 * bracketed by two HIP events on its stream; device_ms is the sum of those intervals (first kernel of the
 * part to its last one: relaxation launches and backtrack), so the host's share of a sweep's wall time is
 * what is left of the wall clock. */
typedef struct gdp_batch_stats {
    double relaxations;   /* sum over the solved instances of L*V*S*S                      */
    double executed;      /* of those, carried out (see gdp_timing.executed)               */
    double device_ms;     /* sum over the parts of first kernel -> last kernel              */
    int64_t instances;
    int64_t parts;        /* plans (a batch above GALVATRON_DP_ARENA_MB is solved in parts) */
    int64_t flow_parts, fused_parts, per_layer_parts; /* by launch scheme of the run        */
} gdp_batch_stats;
void gdp_batch_stats_begin(void);
int gdp_batch_stats_end(gdp_batch_stats *out);

/* Text of the calling thread's last error ("" if none). */
const char *gdp_last_error(void);
/* GDP_VERSION of the built library. */
int gdp_version(void);
/* Writes "name;arch;CUs;HBM bytes" of the current device into buf; GDP_E_HIP without a device. */
int gdp_device_info(char *buf, size_t len);

#ifdef __cplusplus
}
#endif
#endif /* GALVATRON_DP_HIP_H */
