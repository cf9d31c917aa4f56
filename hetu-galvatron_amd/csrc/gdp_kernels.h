// Device-side data layout and kernel launchers of the layer-wise DP (gfx950).
//
// Layout of one instance in HBM (all per instance, one sub-allocation each):
//
//   H      nbuf cost buffers of (S+1) rows of `ld` doubles each, row = strategy; layer l reads
//          buffer l % nbuf and writes buffer (l+1) % nbuf.  nbuf is L+1 when all layers run in one
//          launch (no address is ever rewritten inside that launch, so a cache line read by some
//          XCD can never be a stale copy) and 2 when every layer is its own launch.
//          Row s, element P+u holds
//          h[u][s] = min over source strategies of ((f_prev[u][s'] + inter[s'][s]) + intra[s])
//          for SOURCE row u, i.e. the value the reference stores at f[u + mem[l][s]][s]
//          (csrc/dp_core.cpp:67-73).  The first P elements of every row are +inf for good, so
//          that reading f[v][s] = H[s][P + v - mem[l][s]] yields +inf for v < mem[l][s]
//          (csrc/dp_core.cpp:60-64) without a branch.  Row S is +inf everywhere and stands in
//          for strategies whose mem reaches V and for the padding source strategies.
//   M      argmin table, L*S rows of `ldm` entries (one byte each), indexed by the SOURCE row u
//          like H: mark[l][v][s] of the reference is M[l][s][v - mem[l][s]].  Only present when the
//          plan keeps marks; otherwise nbuf is L+1 and the backtrack recomputes the argmin of the
//          cells on its path from H.
//   roff   (L+1) rows of SU+GDP_SRC_PAD int64: element offset, from the base of a cost buffer,
//          at which "f of the previous layer, strategy s', row 0" is found (SU = S rounded up to
//          the source unroll; the entries from S on point at the +inf row: padding sources and the
//          targets of the last prefetches).
//   inter  n_inter matrices, each SU+GDP_SRC_PAD rows (rows >= S zero) of SP doubles (columns
//          padded with zeros up to SP = a multiple of the target tile).
//   intra  L rows of SP doubles (zero padded).
//   mem    L rows of S int32, as given.
//
// The relaxation kernels do not read the instance record at all: everything one (instance, layer)
// step needs is precomputed into one 256-byte GdpDevLayer record (one scalar load away from the
// kernel arguments), in a table of n_inst x max_L records per group of instances.
//   dep    ceil(max mem[l] / tile rows): a reader of layer l's output at tile t touches tiles
//          [t-dep, t].
//   lo/hi  the band of tiles of layer l that has to be computed.  Source rows below
//          sum_{k<l} min_s mem[k][s] hold only +inf, so tiles entirely below are filled with
//          +inf / argmin 0 without arithmetic (bit-identical to computing them).  Source rows above
//          max start row - sum_{k>=l} min_s mem[k][s] cannot lie on any path that ends at a
//          requested start row; they are skipped unless the caller asked for the full f / mark arrays.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef GDP_WAVES_PER_BLOCK
#define GDP_WAVES_PER_BLOCK 4
#endif
#define GDP_SRC_UNROLL 4  // source strategies are consumed up to four per trip (padded with +inf sources)
#define GDP_SRC_PAD 16    // dummy source rows after SU in roff / inter: targets of the last prefetches
#define GDP_SRC_UNROLL_LAT 8  // sources per trip of the latency variant (its groups pad S to this)

struct GdpDevInst {
    double *H;        // buffer b starts at H + b * hstride
    int64_t hstride;  // (S+1) * ld
    uint8_t *M;
    const double *inter;
    const double *intra;
    const int32_t *inter_index;
    const int64_t *roff;
    const int32_t *mem;
    const int32_t *zcols;   // null, or L rows of S+1 int32: {n, the n strategies of the layer whose memory cost is 0, ascending}
    int64_t ld;          // elements per row of H
    int64_t ldm;         // entries per row of M
    int32_t L, V, S, SP;
    int32_t SU;     // S rounded up to GDP_SRC_UNROLL (GDP_SRC_UNROLL_LAT where the latency variant runs)
    int32_t P;      // +inf elements in front of every H row
    int32_t ntile;  // row tiles covering [0, V)
    int32_t nbuf;
};

// One relaxation step of one instance, ready to use.
struct GdpDevLayer {
    const double *src;  // cost buffer this layer reads; roff offsets are relative to it
    double *dst;        // row 0, source row 0 (element P) of the cost buffer this layer writes
    const int64_t *ro;  // this layer's row of roff
    const double *it;   // this layer's transition matrix
    const double *ia;   // this layer's row of intra
    uint8_t *m;         // this layer's S rows of the argmin table (null when marks are not kept)
    int64_t ld, ldm;    // elements per row of H / entries per row of M
    int32_t S, SU, SP, ntile;
    int32_t dep, lo, hi;  // see above; an entry of an instance without this layer has lo = 0, hi = -1
    uint32_t gate;        // flow launches: per part of a task (byte p for part p), the source strategy -- counted
                          // within the part -- whose cost row lies highest (smallest memory cost in the layer before)
    int32_t fill_from;    // first row of this layer's output below its band that anything reads (rows fill_from ..
                          // lo * tile rows - 1 are filled with +inf once per plan; the rows below are never touched)
    int32_t pad_[7];
    int64_t ro_head[16];  // copy of ro[0..16): a task that starts from them needs no second round trip
};
static_assert(sizeof(GdpDevLayer) == 256, "one record = four 64-byte scalar loads");

// Bookkeeping of one fused (all layers) launch over a group of instances.  Passed to the kernel by
// value: its fields arrive with the kernel arguments, one dependent load fewer at the start of every
// workgroup.
struct GdpSched {
    const GdpDevLayer *lay;   // [n_inst][max_L]
    int32_t *cnt;             // [n_inst][max_L][max_ntile] finished wave tasks    (zeroed per run)
    int32_t *abort_flag;      // set when a bounded wait ran out                   (zeroed per run)
    const int32_t *n_active;  // [max_L] instances that still have layer l (a prefix of the table)
    int32_t max_L, max_ntile, ntb;
    const int32_t *rows;      // per grid row (blockIdx.y) of a chunked launch: {first instance, instances, layer};
                              // null: grid row y is layer layer0+y of the first n_active[layer] instances
    int32_t group;            // consecutive block tasks that go to one XCD (whole tiles)
    int32_t slots;            // workgroups per XCD, instance and layer: ceil(ceil(block tasks / group) / 8) * group
    int64_t spin_limit;       // polls before a waiting wave gives up
    int32_t debug_stall;      // test aid: tasks of layer 0 do not signal their completion, so that every wait for
                              // them runs into its bound (the launch drains, the host repeats the solve)
};

struct GdpDevKey {
    int64_t other_mem;
    double other_time;
    int32_t inst;     // index into the instance table
    int32_t res_off;  // offset (elements) of this key's strategy list in the result array
};

struct GdpDevOut {
    double total;
    int32_t remaining;
    int32_t feasible;
};

// Register tile of the relaxation kernel: TS target strategies x (64 lanes x R rows) per wavefront.
// Variants of one width are listed tallest first.  The host picks the width that covers S with the
// fewest target blocks: every block of a row tile reads all of the tile's source rows again, and a
// wave task's time is set by that stream of loads rather than by its arithmetic (measured on batches
// of 96-256 instances, ms per solve by width: S = 44: 8 -> 30.4, 11 -> 24.5, 15 -> 20.3; S = 40:
// 8 -> 27.8, 15 -> 18.9; S = 88: 11 -> 20.6, 15 -> 17.4; S = 56: 8 -> 22.0, 14 -> 15.6), then the one
// that pads S least.  Widths 12 to 16 exist for the costs-only relaxation alone: with the argmin
// tracked as well they would not fit the registers (the transition costs of a step alone take
// 4*TS scalar registers, double-buffered).
struct GdpVariant {
    int ts, r;
    bool marks;  // also built with the argmin table
};
static const GdpVariant GDP_VARIANTS[] = {
    {16, 3, false}, {16, 2, false}, {16, 1, false}, {15, 3, false}, {15, 2, false}, {15, 1, false},
    {14, 3, false}, {14, 2, false}, {14, 1, false}, {13, 3, false}, {13, 2, false}, {13, 1, false},
    {12, 3, false}, {12, 2, false}, {12, 1, false}, {11, 3, true},  {11, 2, true},  {11, 1, true},
    {8, 4, true},   {8, 2, true},   {8, 1, true}};
#define GDP_NUM_VARIANTS 21

// One relaxation step (layer `layer`) for the first n_inst instances of the table.
// marks: track and store the argmin table (otherwise costs only).  lay: the group's table of
// n_inst x max_L records.
// latency: 0, or K = 1, 2, 4: the variant for launches too small to hide memory latency behind other
// waves (costs only, tile GDP_LAT_TS x GDP_LAT_R), the source strategies of a task split over K
// waves; SU is a multiple of K * GDP_SRC_UNROLL_LAT then.  See relax_task_lat.
hipError_t gdp_launch_relax(int variant, bool marks, int latency, const GdpDevLayer *lay, int max_L, int n_inst,
                            int max_ntile, int SP, int layer, hipStream_t stream);
#define GDP_LAT_TS 8
#define GDP_LAT_R 1
// Layers layer0 .. layer0+layers-1 of a group in one launch (grid = block tasks of a layer x
// layers): a block waits on per-tile completion counters instead of on a kernel boundary.
// lds_bytes: dynamic LDS per workgroup, unused by the kernel; it limits how many workgroups a CU holds.
// With sched->rows set, layer0 is the first entry of that table and `layers` the number of entries.
// split: 1, or 2 -- the source strategies of a wave task on two waves of a workgroup (costs only, register
// tiles of 64 rows, GDP_SPLIT_R == 1; the layers' SU is then a multiple of 2 * GDP_SRC_UNROLL, sched.ntb counts
// both parts of every task, and every workgroup also takes GDP_SPLIT_LDS_BYTES(ts) of static LDS).
#define GDP_SPLIT_R 1
#define GDP_SPLIT_LDS_BYTES(ts) (GDP_WAVES_PER_BLOCK * GDP_SPLIT_R * (ts) * 64 * 8)
hipError_t gdp_launch_relax_fused(int variant, bool marks, int split, const GdpSched &sched, int grid_blocks, int layer0,
                                  int layers, unsigned lds_bytes, hipStream_t stream);
// (sources per wave, waves per task) of the flow kernels that are built
#define GDP_FOR_EACH_FLOW(X) \
    X(8, 1) X(12, 1) X(16, 1) X(20, 1) X(24, 1) X(28, 1) X(32, 1) X(8, 2) X(12, 2) X(16, 2) X(20, 2) X(24, 2) X(28, 2) X(32, 2) \
    X(8, 4) X(12, 4) X(16, 4) X(20, 4) X(24, 4) X(28, 4) X(32, 4)
static const int GDP_FLOW_NSRC[] = {8, 12, 16, 20, 24, 28, 32};
#define GDP_FLOW_MAX_S (4 * 32)   // most sources per wave x most waves per task
// Layers layer0 .. layer0+layers-1 of the first n_inst instances of a group in one launch whose tasks
// wait on the cost cells themselves (gdp_relax_flow_kernel; costs only, the tile of the latency variant,
// `latency` = waves that share the sources of a task, nsrc = sources per wave: one of GDP_FLOW_NSRC, the
// layers' SU being nsrc * latency).  grid_blocks: workgroups of the widest band.
// The cells the launch writes must hold NaN beforehand and the abort flag zero: gdp_launch_flow_reset
// (bands of all layers of n_inst instances).
// debug_stall: test aid -- the tasks of layer 0 leave their stores out, so that every wait for them runs into
// its bound.
hipError_t gdp_launch_relax_flow(int nsrc, int latency, const GdpDevLayer *lay, int max_L, int n_inst, int grid_blocks, int SP,
                                 int layer0, int layers, int32_t *abort_flag, int64_t spin_limit, bool debug_stall,
                                 hipStream_t stream);
hipError_t gdp_launch_flow_reset(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, const GdpDevLayer *lay,
                                 int max_L, int tile_rows, int32_t *abort_flag, hipStream_t stream);
// Sets up H.  what = GDP_INIT_PADS: +inf pads and +inf row of every buffer (once per plan);
// GDP_INIT_ZERO: zeros in the data region of buffer 0 (the caller's initial f); GDP_INIT_POISON: NaN
// in the data region of every other buffer (test aid: a read of a not-yet-written cell shows up);
// GDP_INIT_FILL (one cost buffer per layer only): +inf in the rows of layer l's output below its
// first tile with arithmetic, lay[i * max_L + l].lo (every source cell of those rows is +inf, so the
// cells are +inf whatever the costs: written once per plan, the costs-only kernels leave them alone).
// GDP_INIT_PADS | GDP_INIT_ZERO | GDP_INIT_FILL of a costs-only plan (one cost buffer per layer) in one
// launch, and, with nan_bands, what gdp_launch_flow_reset does as well.
hipError_t gdp_launch_prepare(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, const GdpDevLayer *lay,
                              int max_L, int tile_rows, bool nan_bands, int32_t *abort_flag, hipStream_t stream);
// The same from the kernel's own arguments, for a few small instances (no table of the plan has to be on
// the device yet): per instance where its cost buffers lie, per layer -- `first_layer` of an instance on --
// the band and the first filled row of its output.
#define GDP_PREP_MAX_INST 16
#define GDP_PREP_MAX_LAYERS 224
struct GdpPrepArgs {
    struct Inst {
        double *H;
        int64_t hstride, ld, P;
        int32_t S, L, tile_rows, first_layer;
    } inst[GDP_PREP_MAX_INST];
    int32_t lo[GDP_PREP_MAX_LAYERS], hi[GDP_PREP_MAX_LAYERS], fill_from[GDP_PREP_MAX_LAYERS];
    int32_t *abort_flag;
    int32_t n_inst, nan_bands;
};
static_assert(sizeof(GdpPrepArgs) <= 3584, "passed by value with the kernel arguments");
hipError_t gdp_launch_prepare_args(const GdpPrepArgs &A, hipStream_t stream);
#define GDP_INIT_PADS 1
#define GDP_INIT_ZERO 2
#define GDP_INIT_POISON 4
#define GDP_INIT_FILL 8
hipError_t gdp_launch_init(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, const GdpDevLayer *lay,
                           int max_L, int tile_rows, int what, hipStream_t stream);
// Fills n int32 with zero (queue counters; a kernel rather than a memset so that it can be captured).
hipError_t gdp_launch_zero(int32_t *p, int64_t n, hipStream_t stream);
// Strategies whose memory cost is 0 in layer `layer`, for the first n_inst instances (those that have
// such a layer and such strategies; the others are skipped).  The reference updates f in place, bin v
// downwards and strategy s upwards (csrc/dp_core.cpp:58-73): a cell with mem == 0 reads its OWN row,
// where the entries of lower strategies already hold this layer's values.  After the layer's ordinary
// launch (which has given every strategy with mem > 0 its final value, from the previous layer's
// buffer alone) this pass recomputes the mem == 0 columns, one lane per bin, in ascending strategy
// order: candidates from lower strategies come from the buffer the layer writes, the others from the
// buffer it reads.  One launch per layer only (plans with such strategies never fuse layers).
// lay: the table of n_inst x max_L layer records that belongs to `insts` (the pass keeps to each layer's band
// of tile_rows-row tiles).
hipError_t gdp_launch_zero_pass(bool marks, const GdpDevInst *insts, const GdpDevLayer *lay, int max_L, int tile_rows,
                                int n_inst, int max_V, int layer, hipStream_t stream);
// argmin over the last layer's row + backtrack, one wavefront per key (marks: through the stored
// argmin table; otherwise recomputed from the cost buffers of all layers).
hipError_t gdp_launch_epilogue(bool marks, const GdpDevInst *insts, const GdpDevKey *keys, int n_key, GdpDevOut *out,
                               int32_t *res, hipStream_t stream);
// Debug exports in the reference's layouts.
hipError_t gdp_launch_export_f(const GdpDevInst *inst, double *f_out, int V, int S, hipStream_t stream);
hipError_t gdp_launch_export_mark(const GdpDevInst *inst, int layer, int32_t *mark_out, int V, int S,
                                  hipStream_t stream);
