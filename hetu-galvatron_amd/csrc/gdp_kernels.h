// Device-side data layout and kernel launchers of the layer-wise DP (gfx950).
//
// Layout of one instance in HBM (all per instance, one sub-allocation each):
//
//   H[2]   two cost buffers, each (S+1) rows of `ld` doubles, row = strategy.
//          Row s, element P+u holds h[u][s] = min over source strategies of
//          ((f_prev[u][s'] + inter[s'][s]) + intra[s]) for SOURCE row u, i.e. the value
//          the reference stores at f[u + mem[l][s]][s] (csrc/dp_core.cpp:67-73).  The
//          first P elements of every row are +inf for good, so that reading
//          f[v][s] = H[s][P + v - mem[l][s]] yields +inf for v < mem[l][s]
//          (csrc/dp_core.cpp:60-64) without a branch.  Row S is +inf everywhere and
//          stands in for strategies whose mem reaches V.
//   M      argmin table, L*S rows of `ldm` entries (one byte each), indexed by the
//          SOURCE row u like H: mark[l][v][s] of the reference is M[l][s][v - mem[l][s]].
//   roff   (L+1) rows of S+1 int64: element offset, from the base of a cost buffer, at
//          which "f of the previous layer, strategy s', row 0" is found.
//   inter  n_inter matrices, each S+1 rows (last row zero) of SP doubles (columns
//          padded with zeros up to SP = a multiple of the target tile).
//   intra  L rows of SP doubles (zero padded).
//   mem    L rows of S int32, as given.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

struct GdpDevInst {
    double *H[2];
    uint8_t *M;
    const double *inter;
    const double *intra;
    const int32_t *inter_index;
    const int64_t *roff;
    const int32_t *mem;
    int64_t ld;   // elements per row of H
    int64_t ldm;  // entries per row of M
    int32_t L, V, S, SP;
    int32_t P;      // +inf elements in front of every H row
    int32_t ntile;  // row tiles of GDP_TILE_ROWS rows covering [0, V)
    int32_t pad0, pad1;
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

// rows of the budget axis handled by one wavefront (64 lanes x GDP_R rows per lane)
#define GDP_TS 8
#define GDP_R 4
#define GDP_TILE_ROWS (64 * GDP_R)
#define GDP_WAVES_PER_BLOCK 4

// One relaxation step (layer `layer`) for the first n_inst instances of the table.
hipError_t gdp_launch_relax(const GdpDevInst *insts, int n_inst, int max_ntile, int SP, int layer,
                            hipStream_t stream);
// Sets up H: +inf pads and +inf row in both buffers, zeros in the data region of buffer 0.
hipError_t gdp_launch_init(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, hipStream_t stream);
// argmin over the last layer's row + backtrack, one wavefront per key.
hipError_t gdp_launch_epilogue(const GdpDevInst *insts, const GdpDevKey *keys, int n_key, GdpDevOut *out,
                               int32_t *res, hipStream_t stream);
// Debug exports in the reference's layouts.
hipError_t gdp_launch_export_f(const GdpDevInst *inst, double *f_out, int V, int S, hipStream_t stream);
hipError_t gdp_launch_export_mark(const GdpDevInst *inst, int layer, int32_t *mark_out, int V, int S,
                                  hipStream_t stream);
