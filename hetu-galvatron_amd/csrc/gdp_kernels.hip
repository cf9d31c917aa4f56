// Hand-written gfx950 kernels of the layer-wise DP (see gdp_kernels.h for the HBM layout).
//
// The recurrence of csrc/dp_core.cpp:57-76 is evaluated per SOURCE row u instead of per
// destination row v:  h[u][s] = min_{s'} ((f_prev[u][s'] + inter[s'][s]) + intra[s]) is what the
// reference stores at f[u + mem[l][s]][s], so one lane owns a few rows u, reads the S values
// f_prev[u][.] with lanes running along u (coalesced, no per-target shift), and keeps a tile of
// running minima in registers.  Scanning s' upward and replacing only on strict '<' is the
// comparison sequence of std::min_element (csrc/dp_core.cpp:12-16,70), so ties go to the lowest
// index with no cross-lane traffic.  Both additions are done per candidate, in the reference's
// order, before the comparison; nothing is pre-added or reassociated.
#include "gdp_kernels.h"

#include <math.h>

namespace {

// Uniform (wave-invariant) data is read through the constant address space so that it lands in
// SGPRs (scalar loads only; nothing is ever written through the scalar cache).
template <typename T>
__device__ __forceinline__ T uload(const T *p)
{
    return *reinterpret_cast<const __attribute__((address_space(4))) T *>(reinterpret_cast<uintptr_t>(p));
}

// min of two non-NaN doubles.  Written as the bare instruction: the compiler's fmin adds a
// canonicalising v_max_f64 per operand, which is pure overhead here because every operand is the
// result of an addition (already canonical) and NaN inputs are rejected on the host.
__device__ __forceinline__ double min_f64(double a, double b)
{
    double r;
    asm("v_min_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

__device__ __forceinline__ unsigned xcd_swizzle(unsigned x, unsigned nblk)
{
    // Workgroups are handed to the 8 XCDs round-robin by linear id; nblk is a multiple of 8.  Give
    // every XCD one contiguous range of logical blocks (neighbouring budget rows share an L2).
    return (x & 7u) * (nblk >> 3) + (x >> 3);
}

// One wave task: targets [tb*TS, tb*TS+TS) of rows [tile*64*R, (tile+1)*64*R) of layer `layer`.
// PUBLISH: the cost stores are write-through at agent scope, so that a wave on another XCD that
// waits for this task's completion counter finds them in memory.
template <int TS, int R, bool PUBLISH>
__device__ __forceinline__ void relax_task(const GdpDevInst *I, int layer, unsigned tile, unsigned tb,
                                           unsigned lane)
{
    const int S = uload(&I->S);
    const int SU = uload(&I->SU);
    const int SP = uload(&I->SP);
    const int P = uload(&I->P);
    const int64_t ld = uload(&I->ld);
    const int64_t ldm = uload(&I->ldm);
    const int nbuf = uload(&I->nbuf);
    const int64_t hstride = uload(&I->hstride);
    double *const hbase = uload(&I->H);
    const double *src = hbase + (int64_t)(layer % nbuf) * hstride;
    double *dst = hbase + (int64_t)((layer + 1) % nbuf) * hstride;
    uint8_t *M = uload(&I->M);
    const int64_t *ro = uload(&I->roff) + (int64_t)layer * (SU + GDP_SRC_UNROLL);
    const int s0 = tb * TS;
    const int mat = uload(uload(&I->inter_index) + layer);
    const double *it = uload(&I->inter) + (int64_t)mat * (SU + GDP_SRC_UNROLL) * SP + s0;
    const double *ia = uload(&I->intra) + (int64_t)layer * SP + s0;
    const int64_t u0 = (int64_t)tile * (64 * R);

    double add[TS];
#pragma unroll
    for (int j = 0; j < TS; ++j) add[j] = uload(ia + j);

    double best[R][TS];
    int arg[R][TS];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < TS; ++j) {
            best[r][j] = INFINITY;
            arg[r][j] = 0;
        }

    // Two register sets (A: even source strategies, B: odd) so that the loads for strategy sp+2 are
    // in flight while strategy sp+1 is being consumed.  Entries SU, SU+1 of roff / inter are valid
    // dummies, and source strategies in [S, SU) read the +inf row: +inf never wins a strict '<'.
    double fpA[R], fpB[R], scA[TS], scB[TS];
    {
        const double *pa = src + uload(ro) + u0;
        const double *pb = src + uload(ro + 1) + u0;
#pragma unroll
        for (int r = 0; r < R; ++r) fpA[r] = pa[lane + 64u * r];
#pragma unroll
        for (int r = 0; r < R; ++r) fpB[r] = pb[lane + 64u * r];
#pragma unroll
        for (int j = 0; j < TS; ++j) scA[j] = uload(it + j);
#pragma unroll
        for (int j = 0; j < TS; ++j) scB[j] = uload(it + SP + j);
    }

    const int S2 = (S + 1) & ~1;
    for (int sp = 0; sp < S2; sp += 2) {
#pragma unroll
        for (int j = 0; j < TS; ++j)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const double c = (fpA[r] + scA[j]) + add[j];
                const bool lt = c < best[r][j];
                best[r][j] = min_f64(best[r][j], c);
                arg[r][j] = lt ? sp : arg[r][j];
            }
        {
            const double *pn = src + uload(ro + sp + 2) + u0;
#pragma unroll
            for (int r = 0; r < R; ++r) fpA[r] = pn[lane + 64u * r];
#pragma unroll
            for (int j = 0; j < TS; ++j) scA[j] = uload(it + (int64_t)(sp + 2) * SP + j);
        }
#pragma unroll
        for (int j = 0; j < TS; ++j)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const double c = (fpB[r] + scB[j]) + add[j];
                const bool lt = c < best[r][j];
                best[r][j] = min_f64(best[r][j], c);
                arg[r][j] = lt ? (sp + 1) : arg[r][j];
            }
        {
            const double *pn = src + uload(ro + sp + 3) + u0;
#pragma unroll
            for (int r = 0; r < R; ++r) fpB[r] = pn[lane + 64u * r];
#pragma unroll
            for (int j = 0; j < TS; ++j) scB[j] = uload(it + (int64_t)(sp + 3) * SP + j);
        }
    }

#pragma unroll
    for (int j = 0; j < TS; ++j) {
        const int s = s0 + j;
        if (s < S) {
            double *drow = dst + (int64_t)s * ld + P + u0;
            uint8_t *mrow = M + ((int64_t)layer * S + s) * ldm + u0;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (PUBLISH)
                    __hip_atomic_store(drow + (lane + 64u * r), best[r][j], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                else
                    drow[lane + 64u * r] = best[r][j];
                mrow[lane + 64u * r] = (uint8_t)arg[r][j];
            }
        }
    }
}

// A tile whose source rows all lie below the first row that can hold a finite cost: every
// candidate is +inf, so the cell is +inf and its argmin 0 (all-equal candidates go to index 0,
// csrc/dp_core.cpp:12-16,70).  Same stores as relax_task, no arithmetic.
template <int TS, int R, bool PUBLISH>
__device__ __forceinline__ void fill_task(const GdpDevInst *I, int layer, unsigned tile, unsigned tb, unsigned lane)
{
    const int S = uload(&I->S);
    const int P = uload(&I->P);
    const int64_t ld = uload(&I->ld);
    const int64_t ldm = uload(&I->ldm);
    const int nbuf = uload(&I->nbuf);
    double *dst = uload(&I->H) + (int64_t)((layer + 1) % nbuf) * uload(&I->hstride);
    uint8_t *M = uload(&I->M);
    const int s0 = tb * TS;
    const int64_t u0 = (int64_t)tile * (64 * R);
#pragma unroll
    for (int j = 0; j < TS; ++j) {
        const int s = s0 + j;
        if (s < S) {
            double *drow = dst + (int64_t)s * ld + P + u0;
            uint8_t *mrow = M + ((int64_t)layer * S + s) * ldm + u0;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (PUBLISH)
                    __hip_atomic_store(drow + (lane + 64u * r), (double)INFINITY, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                else
                    drow[lane + 64u * r] = INFINITY;
                mrow[lane + 64u * r] = 0;
            }
        }
    }
}

// Rows of a layer that have to be computed (band[3*l+1] .. band[3*l+2], in tiles): below the band
// every source cell is +inf (fill_task); above it no cell can lie on a path that ends at one of
// the requested start rows, so nothing is read from there later and nothing is written.
template <int TS, int R, bool PUBLISH>
__device__ __forceinline__ void tile_task(const GdpDevInst *I, int layer, unsigned tile, unsigned tb, unsigned lane)
{
    const int32_t *band = uload(&I->dep) + 3 * layer;
    const unsigned lo = (unsigned)uload(band + 1), hi = (unsigned)uload(band + 2);
    if (tile > hi) return;
    if (tile < lo)
        fill_task<TS, R, PUBLISH>(I, layer, tile, tb, lane);
    else
        relax_task<TS, R, PUBLISH>(I, layer, tile, tb, lane);
}

// ---- one launch per layer ------------------------------------------------------------------------
// __launch_bounds__(256, 4): register allocation is held to 4 resident blocks per CU (4 waves per
// SIMD, at most 128 VGPRs).
template <int TS, int R>
__global__ __launch_bounds__(64 * GDP_WAVES_PER_BLOCK, 4) void gdp_relax_kernel(
    const GdpDevInst *__restrict__ insts, int layer, unsigned ntb, unsigned nblk_x)
{
    const GdpDevInst *I = insts + blockIdx.y;
    if (layer >= uload(&I->L)) return;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned lane = threadIdx.x & 63u;
    // Only the tiles lo..hi of this layer carry arithmetic.  The first blocks of the grid share them
    // out, every XCD getting one contiguous range of them (equal work per XCD, neighbouring budget
    // rows in one L2); the blocks after those fill the tiles below lo; tiles above hi are left alone.
    const int32_t *band = uload(&I->dep) + 3 * layer;
    const int lo = uload(band + 1), hi = uload(band + 2);
    const unsigned live_tasks = hi >= lo ? (unsigned)(hi - lo + 1) * ntb : 0u;
    const unsigned live_blocks = ((live_tasks + GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK + 7u) & ~7u;
    (void)nblk_x;
    if (blockIdx.x < live_blocks) {
        const unsigned task = xcd_swizzle(blockIdx.x, live_blocks) * GDP_WAVES_PER_BLOCK + wave;
        if (task >= live_tasks) return;
        const unsigned t = task / ntb;
        relax_task<TS, R, false>(I, layer, (unsigned)lo + t, task - t * ntb, lane);
    } else {
        const unsigned task = (blockIdx.x - live_blocks) * GDP_WAVES_PER_BLOCK + wave;
        const unsigned t = task / ntb;
        const int top = lo - 1 < hi ? lo - 1 : hi;  // fill tiles 0 .. min(lo-1, hi)
        if ((int)t > top) return;
        fill_task<TS, R, false>(I, layer, t, task - t * ntb, lane);
    }
}

// ---- all layers in one launch --------------------------------------------------------------------
// Agent-scope (all XCDs) relaxed load / add of a queue word.
__device__ __forceinline__ int ld_agent(const int32_t *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Waits until cnt[lo..hi] have all reached `full`.  The first poll comes at once; after a miss the
// wave sleeps, longer each time (all waiting waves of a layer look at the same few cache lines, and
// polling them back to back would queue the very counter updates they are waiting for behind the
// polls).  Every wait is bounded: after `limit` polls, or as soon as another wave has given up, the
// wave gives up too (returns false) and the launch drains.
__device__ __forceinline__ bool wait_tiles(const int32_t *cnt, int lo, int hi, int full, unsigned lane,
                                           int32_t *abort_flag, int64_t limit)
{
    int64_t polls = 0;
    for (int base = lo; base <= hi; base += 64) {
        const int t = base + (int)lane;
        for (;;) {
            const int v = (t <= hi) ? ld_agent(cnt + t) : full;
            if (__builtin_amdgcn_ballot_w64(v < full) == 0) break;  // wave-uniform
            ++polls;
            const int stop = (polls & 15) ? 0 : __builtin_amdgcn_readfirstlane(ld_agent(abort_flag));
            if (polls > limit || stop != 0) {
                if (lane == 0) __hip_atomic_store(abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return false;
            }
            if (polls < 4) __builtin_amdgcn_s_sleep(32);        // ~1 us
            else __builtin_amdgcn_s_sleep(127);                  // ~3.5 us
        }
    }
    return true;
}

// One launch for a run of layers (all of them, unless instances of different depth share the
// batch: then one launch per run of layers with the same set of active instances, so that no
// launch carries empty workgroups): grid.y = layer - layer0, grid.x = block task (four consecutive
// (tile, target block) wave tasks of one instance).  Workgroups are dispatched in order of their linear id, x
// fastest, so every block of layer l is dispatched before any block of layer l+1; a block only
// ever waits for blocks of the layer before its own, which therefore run or have finished, and the
// oldest unfinished block never waits: the launch cannot deadlock.  (Each XCD takes every eighth
// workgroup and dispatches its share in order, which is all the argument needs.)  Older workgroups
// also win the issue arbitration of their SIMD, so the work that others wait for runs first.
//
// Instead of a kernel boundary between layers, a task waits only for the tiles it reads: layer l,
// tile t reads rows of layer l-1's output in tiles [t-dep[l-1], t].  Every layer has its own cost
// buffer inside a fused launch, so nothing is overwritten and read-after-write is the only
// dependence.  Waits are bounded; if one runs out the launch drains and the host repeats the solve
// with one launch per layer.
//
// Visibility across the 8 XCDs, whose L2s are not coherent with each other:
//  - a cost cell is written once per launch with a write-through (agent scope) store, the writer
//    waits for its stores to be acknowledged and only then bumps its tile's counter;
//  - a reader polls the counter with agent-scope loads and only afterwards touches the tile.  Its
//    L2 cannot hold an older copy of those lines: tiles are whole cache lines, nobody reads a tile
//    before its counter is full, and the caches are invalidated when the launch begins.
template <int TS, int R>
__global__ __launch_bounds__(64 * GDP_WAVES_PER_BLOCK, 4) void gdp_relax_fused_kernel(
    const GdpDevInst *__restrict__ insts, const GdpSched *__restrict__ Q, int layer0)
{
    __shared__ int sh_ok;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned lane = threadIdx.x & 63u;
    const int layer = layer0 + (int)blockIdx.y;
    const int max_L = uload(&Q->max_L);
    const int max_ntile = uload(&Q->max_ntile);
    const int ntb = uload(&Q->ntb);
    const int nbt = uload(&Q->nbt);
    const int nat = uload(uload(&Q->n_active) + layer);
    // The grid is as wide as the fullest layer.  Inside a layer the first `total8` workgroups share
    // out its block tasks, every XCD getting one contiguous range of them; the rest have nothing to do.
    const unsigned total = (unsigned)(nat * nbt);
    const unsigned total8 = (total + 7u) & ~7u;
    if (blockIdx.x >= total8) return;
    const unsigned x = xcd_swizzle(blockIdx.x, total8);
    if (x >= total) return;
    int32_t *cnt_all = uload(&Q->cnt);
    int32_t *abort_flag = uload(&Q->abort_flag);
    const int bt = (int)(x / (unsigned)nat);  // block task within the instance: tiles ascend with x
    const int ii = (int)x - bt * nat;         // instance (a prefix of the table is active)
    const GdpDevInst *I = insts + ii;
    const int ntile = uload(&I->ntile);
    const unsigned q0 = (unsigned)bt * GDP_WAVES_PER_BLOCK;
    if (layer >= 1) {
        // the block's first wave waits for everything its four wave tasks read
        if (wave == 0) {
            const int t_lo = (int)(q0 / (unsigned)ntb);
            int t_hi = (int)((q0 + GDP_WAVES_PER_BLOCK - 1) / (unsigned)ntb);
            if (t_hi >= ntile) t_hi = ntile - 1;
            bool ok = true;
            if (t_lo < ntile) {
                const int d = uload(uload(&I->dep) + 3 * (layer - 1));
                const int lo = t_lo - d < 0 ? 0 : t_lo - d;
                ok = wait_tiles(cnt_all + ((int64_t)ii * max_L + (layer - 1)) * max_ntile, lo, t_hi, ntb, lane,
                                abort_flag, uload(&Q->spin_limit));
            }
            if (lane == 0) sh_ok = ok ? 1 : 0;
        }
        __syncthreads();
        if (__builtin_amdgcn_readfirstlane(sh_ok) == 0) return;  // the launch is being abandoned
    }
    const unsigned q = q0 + wave;
    const unsigned tile = q / (unsigned)ntb;
    const unsigned tb = q - tile * (unsigned)ntb;
    if (tile >= (unsigned)ntile) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // keeps the tile's loads after the wait
    tile_task<TS, R, true>(I, layer, tile, tb, lane);        // tiles outside the band still count as done
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // every write-through store acknowledged
    if (lane == 0)
        __hip_atomic_fetch_add(cnt_all + ((int64_t)ii * max_L + layer) * max_ntile + tile, 1, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(256) void gdp_zero_kernel(int32_t *p, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        p[i] = 0;
}

// Fills of the cost buffers (see GDP_INIT_* in gdp_kernels.h).  grid = (x chunks, rows 0..S, instances).
__global__ __launch_bounds__(256) void gdp_init_kernel(const GdpDevInst *__restrict__ insts, int what)
{
    const GdpDevInst *I = insts + blockIdx.z;
    const int S = uload(&I->S);
    const int row = blockIdx.y;
    if (row > S) return;
    const int64_t ld = uload(&I->ld);
    const int P = uload(&I->P);
    const int nbuf = uload(&I->nbuf);
    const int64_t hstride = uload(&I->hstride);
    double *h = uload(&I->H) + (int64_t)row * ld;
    const double inf = INFINITY;
    const double nan = __builtin_nan("");
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < ld; i += (int64_t)gridDim.x * blockDim.x) {
        const bool pad = (row == S) || (i < P);
        if (pad) {
            if (what & GDP_INIT_PADS)
                for (int b = 0; b < nbuf; ++b) h[(int64_t)b * hstride + i] = inf;
        } else {
            if (what & GDP_INIT_ZERO) h[i] = 0.0;
            if (what & GDP_INIT_POISON)
                for (int b = 1; b < nbuf; ++b) h[(int64_t)b * hstride + i] = nan;
        }
    }
}

// ---- wavefront (value, index) reduction: lower value wins, equal values -> lower index ----------
__device__ __forceinline__ double swz_f64(double x, int pattern_sel)
{
    int lo = __double2loint(x), hi = __double2hiint(x);
    switch (pattern_sel) {  // ds_swizzle bit-mode: and=0x1f, or=0, xor=1<<k, within groups of 32 lanes
        case 0: lo = __builtin_amdgcn_ds_swizzle(lo, 0x041f); hi = __builtin_amdgcn_ds_swizzle(hi, 0x041f); break;
        case 1: lo = __builtin_amdgcn_ds_swizzle(lo, 0x081f); hi = __builtin_amdgcn_ds_swizzle(hi, 0x081f); break;
        case 2: lo = __builtin_amdgcn_ds_swizzle(lo, 0x101f); hi = __builtin_amdgcn_ds_swizzle(hi, 0x101f); break;
        case 3: lo = __builtin_amdgcn_ds_swizzle(lo, 0x201f); hi = __builtin_amdgcn_ds_swizzle(hi, 0x201f); break;
        default: lo = __builtin_amdgcn_ds_swizzle(lo, 0x401f); hi = __builtin_amdgcn_ds_swizzle(hi, 0x401f); break;
    }
    return __hiloint2double(hi, lo);
}
__device__ __forceinline__ int swz_i32(int x, int pattern_sel)
{
    switch (pattern_sel) {
        case 0: return __builtin_amdgcn_ds_swizzle(x, 0x041f);
        case 1: return __builtin_amdgcn_ds_swizzle(x, 0x081f);
        case 2: return __builtin_amdgcn_ds_swizzle(x, 0x101f);
        case 3: return __builtin_amdgcn_ds_swizzle(x, 0x201f);
        default: return __builtin_amdgcn_ds_swizzle(x, 0x401f);
    }
}

__device__ __forceinline__ void wave_argmin(double &val, int &idx)
{
#pragma unroll
    for (int k = 0; k < 5; ++k) {
        const double ov = swz_f64(val, k);
        const int oi = swz_i32(idx, k);
        if (ov < val || (ov == val && oi < idx)) { val = ov; idx = oi; }
    }
    // halves of the wavefront: lanes l and l^32 (ds_swizzle works within 32 lanes)
    const int partner = (int)((threadIdx.x & 63u) ^ 32u) << 2;
    const int olo = __builtin_amdgcn_ds_bpermute(partner, __double2loint(val));
    const int ohi = __builtin_amdgcn_ds_bpermute(partner, __double2hiint(val));
    const int oi = __builtin_amdgcn_ds_bpermute(partner, idx);
    const double ov = __hiloint2double(ohi, olo);
    if (ov < val || (ov == val && oi < idx)) { val = ov; idx = oi; }
}

// Epilogue of csrc/dp_core.cpp:78-117 for one key per wavefront: first argmin of the start row,
// then the dependent walk through the argmin table.
__global__ __launch_bounds__(64) void gdp_epilogue_kernel(const GdpDevInst *__restrict__ insts,
                                                          const GdpDevKey *__restrict__ keys,
                                                          GdpDevOut *__restrict__ out,
                                                          int32_t *__restrict__ res)
{
    const GdpDevKey *K = keys + blockIdx.x;
    const GdpDevInst *I = insts + uload(&K->inst);
    const int lane = threadIdx.x;
    const int L = uload(&I->L), V = uload(&I->V), S = uload(&I->S);
    const int64_t v0 = (int64_t)V - 1 - uload(&K->other_mem);
    GdpDevOut o;
    o.total = INFINITY;
    o.remaining = -1;
    o.feasible = 0;
    if (v0 < 0) {  // csrc/dp_core.cpp:82-86
        if (lane == 0) out[blockIdx.x] = o;
        return;
    }
    const double *fin = uload(&I->H) + (int64_t)(L % uload(&I->nbuf)) * uload(&I->hstride);  // last written
    const int64_t *ro = uload(&I->roff) + (int64_t)L * (uload(&I->SU) + GDP_SRC_UNROLL);
    double val = INFINITY;
    int idx = 0x7fffffff;
    for (int s = lane; s < S; s += 64) {  // ascending within the lane: strict '<' keeps the first
        const double x = fin[ro[s] + v0];
        if (x < val || idx == 0x7fffffff) { val = x; idx = s; }
    }
    wave_argmin(val, idx);
    if (lane != 0) return;
    if (!(val < INFINITY)) {  // csrc/dp_core.cpp:93-97
        out[blockIdx.x] = o;
        return;
    }
    o.total = val + uload(&K->other_time);  // csrc/dp_core.cpp:99
    const int32_t *mem = uload(&I->mem);
    const uint8_t *M = uload(&I->M);
    const int64_t ldm = uload(&I->ldm);
    int32_t *path = res + uload(&K->res_off);
    int64_t v = v0;
    path[L - 1] = idx;
    for (int i = L - 1; i > 0; --i) {  // csrc/dp_core.cpp:105-113, with mark[i][v][s] = M[i][s][v - mem[i][s]]
        const int cur = idx;
        v -= mem[(int64_t)i * S + cur];
        if (v < 0) break;  // cannot happen on a finite path; keeps a damaged table from being indexed
        idx = M[((int64_t)i * S + cur) * ldm + v];
        if (idx >= S) { v = -1; break; }
        path[i - 1] = idx;
    }
    if (v < 0) {
        o.total = INFINITY;
        out[blockIdx.x] = o;
        return;
    }
    o.remaining = (int32_t)(v - mem[idx]);  // csrc/dp_core.cpp:115
    o.feasible = 1;
    out[blockIdx.x] = o;
}

// f of the last layer in the reference's [V][S] layout.
__global__ __launch_bounds__(256) void gdp_export_f_kernel(const GdpDevInst *__restrict__ I, double *__restrict__ f)
{
    const int L = I->L, V = I->V, S = I->S;
    const double *fin = I->H + (int64_t)(L % I->nbuf) * I->hstride;
    const int64_t *ro = I->roff + (int64_t)L * (I->SU + GDP_SRC_UNROLL);
    const int64_t n = (int64_t)V * S;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t v = i / S;
        const int s = (int)(i - v * S);
        f[i] = fin[ro[s] + v];
    }
}

// One layer of the argmin table in the reference's [V][S] int32 layout (-1 where v < mem).
__global__ __launch_bounds__(256) void gdp_export_mark_kernel(const GdpDevInst *__restrict__ I, int layer,
                                                              int32_t *__restrict__ mark)
{
    const int V = I->V, S = I->S;
    const int32_t *mem = I->mem + (int64_t)layer * S;
    const uint8_t *M = I->M + (int64_t)layer * S * I->ldm;
    const int64_t n = (int64_t)V * S;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t v = i / S;
        const int s = (int)(i - v * S);
        const int64_t u = v - mem[s];
        mark[i] = (u < 0) ? -1 : (int32_t)M[(int64_t)s * I->ldm + u];
    }
}

}  // namespace

template <int TS, int R>
static hipError_t launch_relax_t(const GdpDevInst *insts, int n_inst, int max_ntile_rows, int SP, int layer,
                                 hipStream_t stream)
{
    const unsigned ntb = (unsigned)(SP / TS);
    const unsigned tasks = (unsigned)max_ntile_rows * ntb;
    unsigned nblk = (tasks + GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK;
    nblk = ((nblk + 7u) & ~7u) + 8u;  // live blocks are rounded up to 8, the fill blocks come after them
    dim3 grid(nblk, (unsigned)n_inst, 1), block(64 * GDP_WAVES_PER_BLOCK, 1, 1);
    hipLaunchKernelGGL((gdp_relax_kernel<TS, R>), grid, block, 0, stream, insts, layer, ntb, nblk);
    return hipGetLastError();
}

// one entry per element of GDP_VARIANTS, in the same order
#define GDP_FOR_EACH_VARIANT(X) X(0, 8, 4) X(1, 8, 2) X(2, 8, 1) X(3, 11, 3) X(4, 11, 2) X(5, 11, 1)

hipError_t gdp_launch_relax(int variant, const GdpDevInst *insts, int n_inst, int max_ntile, int SP, int layer,
                            hipStream_t stream)
{
#define X(id, ts, r) \
    case id: return launch_relax_t<ts, r>(insts, n_inst, max_ntile, SP, layer, stream);
    switch (variant) {
        GDP_FOR_EACH_VARIANT(X)
        default: return hipErrorInvalidValue;
    }
#undef X
}

hipError_t gdp_launch_relax_fused(int variant, const GdpDevInst *insts, const GdpSched *sched, int grid_blocks,
                                  int layer0, int layers, hipStream_t stream)
{
    dim3 grid((unsigned)grid_blocks, (unsigned)layers), block(64 * GDP_WAVES_PER_BLOCK);
#define X(id, ts, r)                                                                                       \
    case id:                                                                                               \
        hipLaunchKernelGGL((gdp_relax_fused_kernel<ts, r>), grid, block, 0, stream, insts, sched, layer0); \
        break;
    switch (variant) {
        GDP_FOR_EACH_VARIANT(X)
        default: return hipErrorInvalidValue;
    }
#undef X
    return hipGetLastError();
}

hipError_t gdp_launch_zero(int32_t *p, int64_t n, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    unsigned nb = (unsigned)((n + 1023) / 1024);
    if (nb > 4096u) nb = 4096u;
    hipLaunchKernelGGL(gdp_zero_kernel, dim3(nb), dim3(256), 0, stream, p, n);
    return hipGetLastError();
}

hipError_t gdp_launch_init(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, int max_nbuf, int what,
                           hipStream_t stream)
{
    (void)max_nbuf;
    unsigned bx = (unsigned)((max_ld + 256 * 8 - 1) / (256 * 8));
    if (bx == 0) bx = 1;
    dim3 grid(bx, (unsigned)(max_S + 1), (unsigned)n_inst), block(256, 1, 1);
    hipLaunchKernelGGL(gdp_init_kernel, grid, block, 0, stream, insts, what);
    return hipGetLastError();
}

hipError_t gdp_launch_epilogue(const GdpDevInst *insts, const GdpDevKey *keys, int n_key, GdpDevOut *out,
                               int32_t *res, hipStream_t stream)
{
    if (n_key <= 0) return hipSuccess;
    hipLaunchKernelGGL(gdp_epilogue_kernel, dim3((unsigned)n_key), dim3(64), 0, stream, insts, keys, out, res);
    return hipGetLastError();
}

hipError_t gdp_launch_export_f(const GdpDevInst *inst, double *f_out, int V, int S, hipStream_t stream)
{
    const int64_t n = (int64_t)V * S;
    unsigned nb = (unsigned)((n + 1023) / 1024);
    if (nb > 65535u * 16u) nb = 65535u * 16u;
    hipLaunchKernelGGL(gdp_export_f_kernel, dim3(nb), dim3(256), 0, stream, inst, f_out);
    return hipGetLastError();
}

hipError_t gdp_launch_export_mark(const GdpDevInst *inst, int layer, int32_t *mark_out, int V, int S,
                                  hipStream_t stream)
{
    const int64_t n = (int64_t)V * S;
    unsigned nb = (unsigned)((n + 1023) / 1024);
    if (nb > 65535u * 16u) nb = 65535u * 16u;
    hipLaunchKernelGGL(gdp_export_mark_kernel, dim3(nb), dim3(256), 0, stream, inst, layer, mark_out);
    return hipGetLastError();
}
