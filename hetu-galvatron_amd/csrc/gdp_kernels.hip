// Hand-written gfx950 kernels of the layer-wise DP (see gdp_kernels.h for the HBM layout).
//
// The recurrence of csrc/dp_core.cpp:57-76 is evaluated per SOURCE row u instead of per
// destination row v:  h[u][s] = min_{s'} ((f_prev[u][s'] + inter[s'][s]) + intra[s]) is what the
// reference stores at f[u + mem[l][s]][s], so one lane owns a few rows u, reads the S values
// f_prev[u][.] with lanes running along u (coalesced, no per-target shift), and keeps a tile of
// running minima in registers.  Scanning s' upward and replacing only on strict '<' is the
// comparison sequence of std::min_element (csrc/dp_core.cpp:12-16,70), so ties go to the lowest
// index with no cross-lane traffic.
//
// Where the argmin is tracked, both additions are done per candidate, in the reference's order,
// before the comparison.  Where only the cost is wanted, intra[s] is added once, after the minimum:
//   min_{s'} fl(fl(f + inter) + intra)  ==  fl(min_{s'} fl(f + inter) + intra)
// holds exactly, because rounding x -> fl(x + c) is monotone (x <= y implies fl(x+c) <= fl(y+c)), so
// the smallest pre-sum yields the smallest candidate; +inf behaves the same on both sides and NaN
// and -inf are rejected on the host.  (Which s' attains the minimum can differ between the two
// sides when two candidates round to the same value; the argmin is therefore never taken from the
// hoisted form.)
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

// Element lane + 64 r of a wave-uniform row: uniform 64-bit base plus a 32-bit per-lane byte offset,
// the form that needs no per-lane address arithmetic (scalar base register + vector offset).  The
// callers pass the base through an empty asm, and the offset once per basic block (GDP_PIN_LANE), or
// the compiler folds the per-lane part into a 64-bit vector base outside the loop and spends one
// vector instruction per load on adding the row offset to it.
__device__ __forceinline__ double lane_load(const double *row, unsigned lane_bytes, int r)
{
    typedef const __attribute__((address_space(1))) char *gbytes;     // global memory, not "flat"
    typedef const __attribute__((address_space(1))) double *gdouble;
    return *reinterpret_cast<gdouble>(reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(row)) + lane_bytes +
                                      512u * (unsigned)r);
}

#define GDP_PIN_LANE(x) asm volatile("" : "+v"(x))

// Nothing is moved across this point by the instruction scheduler.
#define GDP_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// Relaxations of target columns [J0, J1) of the register tile against one source strategy.
// ARG: candidate = (f_prev + inter) + intra in that association (csrc/dp_core.cpp:68), strict '<' for
// the argmin (csrc/dp_core.cpp:12-16).  Otherwise: the running minimum of f_prev + inter; the caller
// adds intra at the end.
template <int TS, int R, bool ARG, int J0, int J1>
__device__ __forceinline__ void relax_cols(double (&best)[R][TS], int (&arg)[ARG ? R : 1][ARG ? TS : 1],
                                           const double (&fp)[R], const double (&sc)[TS], const double (&add)[TS],
                                           int sp)
{
#pragma unroll
    for (int j = J0; j < J1; ++j)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const double c = ARG ? (fp[r] + sc[j]) + add[j] : fp[r] + sc[j];
            if constexpr (ARG) {
                // compare into vcc and select at once: left to the compiler, the compare results of a
                // whole step end up in as many scalar register pairs, which then spill
                asm("v_cmp_lt_f64 vcc, %1, %2\n\tv_cndmask_b32 %0, %0, %3, vcc"
                    : "+v"(arg[r][j])
                    : "v"(c), "v"(best[r][j]), "v"(sp)
                    : "vcc");
            }
            best[r][j] = min_f64(best[r][j], c);
        }
}

// relax_task for launches with too few waves to hide memory latency (costs only, per-layer launches).
// In relax_task every step waits for a scalar load issued one step earlier (the next row of transition
// costs; scalar loads return out of order, so there is no waiting for "all but the latest"), about
// 0.2 us when it misses the scalar cache -- nothing when other waves fill the gap, the whole run time
// of a layer when there are one or two waves per SIMD.  Here nothing inside a trip waits for a
// scalar load:
//   - the row of transition costs travels as a vector load (lane j of every row of 16 lanes holds
//     column j), NS steps ahead like the cost rows -- vector loads return in order, so a wait can
//     leave the younger ones in flight -- and is spread over the lanes with one 64-bit DPP move per
//     column (v_mov_b64 row_newbcast: lane j of a row to the whole row; TS more vector instructions
//     per step -- instruction issue is not what such a launch is short of);
//   - the row offsets of a whole trip are fetched with the previous trip's.
// Same arithmetic in the same order as relax_task, hence the same bits.
//
// K > 1: the source strategies of a task are split over K waves of the workgroup (vtb = target block
// * K + part; part p takes sources [p * SU / K, (p + 1) * SU / K)), which shortens the chain of
// dependent steps K times where there are wave slots to spare.  The partial minima meet in LDS; the
// minimum of the parts is the minimum over all sources exactly (min is associative and commutative),
// and the wave of part j % K adds intra to column j and stores it.
// What a task of the latency variant needs from its layer record, fetched by the caller in one round
// of scalar loads (with the band the caller itself needs) and kept in scalar registers.
struct LatHead {
    const double *src, *it, *ia;
    double *dst;
    const int64_t *ro;
    int64_t ld;
    int S, SU, SP, lo, hi;
    int64_t head[2 * 8];   // ro[0..16)
};

__device__ __forceinline__ LatHead load_lat_head(const GdpDevLayer *Y)
{
    LatHead h;
    h.src = uload(&Y->src); h.dst = uload(&Y->dst); h.ro = uload(&Y->ro); h.it = uload(&Y->it);
    h.ia = uload(&Y->ia); h.ld = uload(&Y->ld);
    h.S = uload(&Y->S); h.SU = uload(&Y->SU); h.SP = uload(&Y->SP); h.lo = uload(&Y->lo); h.hi = uload(&Y->hi);
#pragma unroll
    for (int u = 0; u < 16; ++u) h.head[u] = uload(&Y->ro_head[u]);
    // all of it has arrived before the first branch: left alone, the compiler fetches the fields where
    // they are first used, one dependent round trip after the other
#pragma unroll
    for (int u = 0; u < 16; ++u) asm volatile("" : "+s"(h.head[u]));
    asm volatile("" : "+s"(h.src), "+s"(h.dst), "+s"(h.ro), "+s"(h.it), "+s"(h.ia), "+s"(h.ld));
    asm volatile("" : "+s"(h.S), "+s"(h.SU), "+s"(h.SP), "+s"(h.lo), "+s"(h.hi));
    return h;
}

template <int TS, int R, bool PUBLISH, int K>
__device__ __forceinline__ void relax_task_lat(const LatHead &H, unsigned tile, unsigned vtb, unsigned lane)
{
    constexpr int NS = 8;
    static_assert(GDP_SRC_UNROLL_LAT % NS == 0 && GDP_SRC_PAD >= 2 * NS, "padding of roff / inter");
    static_assert(K == 1 || (R == 1 && GDP_WAVES_PER_BLOCK % K == 0), "parts of one task share a workgroup");
    const unsigned tb = vtb / K, part = vtb % K;
    const int SU = H.SU / K;   // a multiple of NS in the groups this variant runs for
    const int SP = H.SP;
    const double *src = H.src;
    const int64_t *ro = H.ro + part * SU;
    const int s0 = tb * TS;
    const double *it = H.it + s0 + (int64_t)part * SU * SP;
    const int64_t u0 = (int64_t)tile * (64 * R);
    const unsigned lane_bytes = lane * 8u;
    static_assert(TS <= 16, "a row of 16 lanes holds the transition costs of a step");
    const unsigned col_bytes = ((lane & 15u) < (unsigned)TS ? (lane & 15u) : (unsigned)(TS - 1)) * 8u;

    double best[R][TS];
    int arg_unused[1][1];
    double add_unused[TS];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < TS; ++j) best[r][j] = INFINITY;
#pragma unroll
    for (int j = 0; j < TS; ++j) add_unused[j] = 0.0;

    double fp[NS][R], scv[NS], iav;
    int64_t ocur[NS], onext[NS];
    const double *itp = it;   // row of the transition matrix that the next request fetches
    {
        int64_t o0[NS];
        if constexpr (K == 1) {
#pragma unroll
            for (int u = 0; u < NS; ++u) o0[u] = H.head[u];
#pragma unroll
            for (int u = 0; u < NS; ++u) ocur[u] = H.head[NS + u];
        } else {
#pragma unroll
            for (int u = 0; u < NS; ++u) o0[u] = uload(ro + u);
#pragma unroll
            for (int u = 0; u < NS; ++u) ocur[u] = uload(ro + NS + u);
        }
        GDP_SCHED_FENCE();
        unsigned lb = lane_bytes, cb = col_bytes;
        GDP_PIN_LANE(lb);
        GDP_PIN_LANE(cb);
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            const double *p = src + o0[u] + u0;
            asm volatile("" : "+s"(p));
#pragma unroll
            for (int r = 0; r < R; ++r) fp[u][r] = lane_load(p, lb, r);
            const double *q = itp;
            asm volatile("" : "+s"(q));
            scv[u] = lane_load(q, cb, 0);
            itp += SP;
            GDP_SCHED_FENCE();
        }
        // the intra costs of the target columns travel like a row of transition costs (lane j of
        // every row of 16 lanes holds column j) and are long there when the loop ends
        const double *qa = H.ia + s0;
        asm volatile("" : "+s"(qa));
        iav = lane_load(qa, cb, 0);
        GDP_SCHED_FENCE();
    }
    const int64_t *rop = ro + 2 * NS;
    for (int sp = 0; sp < SU; sp += NS) {
        unsigned lb = lane_bytes, cb = col_bytes;
        GDP_PIN_LANE(lb);
        GDP_PIN_LANE(cb);
        // row offsets for the requests of the next trip: a whole trip ahead of their use
        {
            typedef long long trip_t __attribute__((ext_vector_type(NS)));   // one wide scalar load
            typedef trip_t trip_a8 __attribute__((aligned(8)));
            const trip_t t =
                *reinterpret_cast<const __attribute__((address_space(4))) trip_a8 *>(reinterpret_cast<uintptr_t>(rop));
#pragma unroll
            for (int u = 0; u < NS; ++u) onext[u] = t[u];
        }
        GDP_SCHED_FENCE();
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            double sc[TS];
#pragma unroll
            for (int j = 0; j < TS; ++j)   // lane j of every row of 16 lanes holds column j: one move spreads it
                asm("v_mov_b64_dpp %0, %1 row_newbcast:%2 row_mask:0xf bank_mask:0xf" : "=v"(sc[j]) : "v"(scv[u]), "n"(j));
            relax_cols<TS, R, false, 0, TS>(best, arg_unused, fp[u], sc, add_unused, sp + u);
            GDP_SCHED_FENCE();
            {
                const double *pn = src + ocur[u] + u0;
                asm volatile("" : "+s"(pn));
#pragma unroll
                for (int r = 0; r < R; ++r) fp[u][r] = lane_load(pn, lb, r);
                const double *q = itp;
                asm volatile("" : "+s"(q));
                scv[u] = lane_load(q, cb, 0);
                itp += SP;
            }
            GDP_SCHED_FENCE();
        }
#pragma unroll
        for (int u = 0; u < NS; ++u) ocur[u] = onext[u];
        rop += NS;
    }

    bool mine[TS];
#pragma unroll
    for (int j = 0; j < TS; ++j) mine[j] = true;
    if constexpr (K > 1) {
        __shared__ double xch[GDP_WAVES_PER_BLOCK][TS][64];
        const unsigned wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
        for (int j = 0; j < TS; ++j) xch[wv][j][lane] = best[0][j];
        __syncthreads();   // waves of the workgroup that had no task have ended and are not waited for
        const unsigned w0 = wv - part;   // the task's first wave
#pragma unroll
        for (int j = 0; j < TS; ++j) {
            mine[j] = (unsigned)(j % K) == part;
            if (mine[j]) {
#pragma unroll
                for (int pp = 0; pp < K; ++pp) best[0][j] = min_f64(best[0][j], xch[w0 + pp][j][lane]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < TS; ++j) {
        double a;
        asm("v_mov_b64_dpp %0, %1 row_newbcast:%2 row_mask:0xf bank_mask:0xf" : "=v"(a) : "v"(iav), "n"(j));
#pragma unroll
        for (int r = 0; r < R; ++r) best[r][j] += a;
    }
    const int64_t ld = H.ld;
    const int nvalid = H.S - s0;
    double *drow = H.dst + (int64_t)s0 * ld + u0;
#pragma unroll
    for (int j = 0; j < TS; ++j) {
        if (j < nvalid) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (!mine[j]) continue;
                if (PUBLISH)
                    __hip_atomic_store(drow + (lane + 64u * r), best[r][j], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                else
                    drow[lane + 64u * r] = best[r][j];
            }
            drow += ld;
        }
    }
}

// ---- tasks of a flow launch (gdp_relax_flow_kernel): waiting on the cost cells themselves --------------
// lane_load at agent scope: the value comes from memory, never from a line that this XCD's L2 holds
// from before another XCD wrote it.
__device__ __forceinline__ double lane_load_agent(const double *row, unsigned lane_bytes)
{
    typedef const __attribute__((address_space(1))) char *gbytes;
    typedef const __attribute__((address_space(1))) double *gdouble;
    return __hip_atomic_load(
        reinterpret_cast<gdouble>(reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(row)) + lane_bytes),
        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The abort flag of the launch, the number of polls after which a wave gives up, and what this wave
// has used of it.  Every wait is bounded: a wave that has polled `limit` times, or finds the flag
// raised, raises it and stops waiting (it finishes with whatever it reads; the host discards the run).
struct FlowWait {
    int32_t *abort_flag;
    int64_t limit;
    int64_t polls;
    bool gave_up;
};

// One more poll: false when the wave has to stop waiting.  Sleeps a little first (waiting waves look
// at single cells, one request per poll, so polling this often does not crowd the memory system).
__device__ __forceinline__ bool flow_poll(FlowWait &w, unsigned lane)
{
    ++w.polls;
    const int stop = (w.polls & 15) ? 0
                                    : __builtin_amdgcn_readfirstlane(__hip_atomic_load(
                                          w.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    if (w.polls > w.limit || stop != 0) {
        if (lane == 0) __hip_atomic_store(w.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        w.gave_up = true;
        return false;
    }
    if (w.polls < 4) __builtin_amdgcn_s_sleep(1);
    else __builtin_amdgcn_s_sleep(4);   // ~0.12 us
    return true;
}

struct FlowHead {
    const double *src, *it, *ia;
    double *dst;
    const int64_t *ro;
    int64_t ld;
    int S, SP, lo, hi;
    unsigned gate;   // per part of a task (one byte each): the source, within the part, whose row lies highest
};

__device__ __forceinline__ FlowHead load_flow_head(const GdpDevLayer *Y)
{
    FlowHead h;
    h.src = uload(&Y->src); h.dst = uload(&Y->dst); h.ro = uload(&Y->ro); h.it = uload(&Y->it);
    h.ia = uload(&Y->ia); h.ld = uload(&Y->ld);
    h.S = uload(&Y->S); h.SP = uload(&Y->SP); h.lo = uload(&Y->lo); h.hi = uload(&Y->hi);
    h.gate = (unsigned)uload(&Y->gate);
    // one round of scalar loads, all of it there before the first branch
    asm volatile("" : "+s"(h.src), "+s"(h.dst), "+s"(h.ro), "+s"(h.it), "+s"(h.ia), "+s"(h.ld));
    asm volatile("" : "+s"(h.S), "+s"(h.SP), "+s"(h.lo), "+s"(h.hi), "+s"(h.gate));
    return h;
}

// One wave task of a flow launch: targets [tb*TS, tb*TS+TS) of the 64 rows of `tile`, against the NSRC
// source strategies [part*NSRC, (part+1)*NSRC) (K parts per task, on K waves of the workgroup, as in
// relax_task_lat; the layer's SU is NSRC*K).  Same arithmetic in the same order as relax_task, hence the
// same bits.
//   - What does not depend on the previous layer -- row offsets, the NSRC rows of transition costs (lane
//     j of every row of 16 lanes holds column j), the intra costs -- is fetched first.
//   - Then the task waits at a gate.  Before a run every cell that the run writes holds NaN, and no
//     cost is ever NaN.  First one cell is asked for again and again (one request per poll) until it
//     holds a cost: the highest cell the task reads (last row of the tile, source with the smallest
//     memory cost), whose writer is the last to have been dispatched.  Then the first and the last cell
//     of every one of the NSRC rows (one gathered load, lane u and lane NSRC + u for row u; the two
//     can come from two tasks of the layer before), until all of them hold costs.
//   - Then all NSRC cost rows are asked for at once and consumed in order -- with ordinary loads, so that
//     the tasks that share a tile's rows (its target blocks) share them in the L2: a line can only have
//     got into an L2 after a gate saw both ends of its row written, and should it hold a cell from before
//     that cell was written, the cell reads as NaN.  A row in which a lane still sees NaN (a task's stores
//     need not show up together) is asked for again, at agent scope, until it is whole.  (All rows at
//     agent scope: S=44 V=32768 L=32 0.44 instead of 0.38 ms, S=40 V=29493 L=28 0.22 instead of 0.19.)
template <int TS, int NSRC, int K>
__device__ __forceinline__ void relax_task_flow(const FlowHead &H, unsigned tile, unsigned vtb, unsigned lane,
                                                FlowWait &w, bool stall)
{
    static_assert(K == 1 || GDP_WAVES_PER_BLOCK % K == 0, "parts of one task share a workgroup");
    static_assert(TS <= 16, "a row of 16 lanes holds the transition costs of a step");
    const unsigned tb = vtb / K, part = vtb % K;
    const int SP = H.SP;
    const double *src = H.src;
    const int64_t *ro = H.ro + part * NSRC;
    const int s0 = tb * TS;
    const double *it = H.it + s0 + (int64_t)part * NSRC * SP;
    const int64_t u0 = (int64_t)tile * 64;
    unsigned lb = lane * 8u;
    unsigned cb = ((lane & 15u) < (unsigned)TS ? (lane & 15u) : (unsigned)(TS - 1)) * 8u;
    GDP_PIN_LANE(lb);
    GDP_PIN_LANE(cb);

    double best[1][TS];
    int arg_unused[1][1];
    double add_unused[TS];
#pragma unroll
    for (int j = 0; j < TS; ++j) { best[0][j] = INFINITY; add_unused[j] = 0.0; }

    int64_t off[NSRC];
#pragma unroll
    for (int u = 0; u < NSRC; ++u) off[u] = uload(ro + u);
    // The task's NSRC x TS transition costs wait in LDS, not in registers (registers decide how many
    // tasks are resident, and the tasks of the next layer should be): each wave has a corner of its own,
    // source-major, so that lane j of every row of 16 lanes reads column j of a step's row.
    __shared__ double costs[GDP_WAVES_PER_BLOCK][NSRC * TS];
    double *my_costs = costs[__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)];
    double iav;
    {
        static_assert(TS == 8, "eight lanes fetch a row of transition costs");
#pragma unroll
        for (int i0 = 0; i0 < NSRC * TS; i0 += 64) {
            const unsigned i = (unsigned)i0 + lane;
            if ((NSRC * TS) % 64 == 0 || i < (unsigned)(NSRC * TS)) {
                const double *q = it;
                asm volatile("" : "+s"(q));
                my_costs[i] = lane_load(q, ((i >> 3) * (unsigned)SP + (i & 7u)) * 8u, 0);
            }
        }
        const double *qa = H.ia + s0;
        asm volatile("" : "+s"(qa));
        iav = lane_load(qa, cb, 0);
    }
    // the gate
    {
        static_assert(2 * NSRC <= 64, "one lane per end of a row");
        const unsigned gu = lane < (unsigned)NSRC ? lane : lane < 2u * NSRC ? lane - NSRC : 0u;
        const int64_t goff = ro[gu] + u0 + (lane >= (unsigned)NSRC ? 63 : 0);   // (a vector load of the row offsets)
        const unsigned g1 = (H.gate >> (8u * part)) & 0xffu;
        const double *cell1 = src + uload(ro + g1) + u0 + 63;
        asm volatile("" : "+s"(cell1));
        for (;;) {
            const double y = lane_load_agent(cell1, 0u);
            if (__builtin_amdgcn_ballot_w64(y != y) == 0) break;
            if (!flow_poll(w, lane)) break;
        }
        // (asking for the rows right behind this load, without waiting for its answer, was slower:
        // S=22 V=16384 L=24 0.099 -> 0.110 ms)
        const double *cells = src + goff;
        for (;;) {
            double y = 0.0;
            if (lane < 2u * NSRC) y = lane_load_agent(cells, 0u);
            if (__builtin_amdgcn_ballot_w64(y != y) == 0) break;
            if (w.gave_up || !flow_poll(w, lane)) break;
        }
    }
    GDP_SCHED_FENCE();
    double fp[NSRC][1];
#pragma unroll
    for (int u = 0; u < NSRC; ++u) {
        const double *pr = src + off[u] + u0;
        asm volatile("" : "+s"(pr));
        fp[u][0] = lane_load(pr, lb, 0);
        GDP_SCHED_FENCE();
    }
#pragma unroll
    for (int u = 0; u < NSRC; ++u) {
        if (__builtin_amdgcn_ballot_w64(fp[u][0] != fp[u][0]) != 0) {
            const double *row = src + uload(ro + u) + u0;   // (fetched again: the offsets are not kept in registers)
            while (!w.gave_up && flow_poll(w, lane)) {
                fp[u][0] = lane_load_agent(row, lb);
                if (__builtin_amdgcn_ballot_w64(fp[u][0] != fp[u][0]) == 0) break;
            }
        }
        double sc[TS];
        const double scv = my_costs[u * TS + (cb >> 3)];
#pragma unroll
        for (int j = 0; j < TS; ++j)   // lane j of every row of 16 lanes holds column j: one move spreads it
            asm("v_mov_b64_dpp %0, %1 row_newbcast:%2 row_mask:0xf bank_mask:0xf" : "=v"(sc[j]) : "v"(scv), "n"(j));
        relax_cols<TS, 1, false, 0, TS>(best, arg_unused, fp[u], sc, add_unused, u);
    }

    bool mine[TS];
#pragma unroll
    for (int j = 0; j < TS; ++j) mine[j] = true;
    if constexpr (K > 1) {
        __shared__ double xch[GDP_WAVES_PER_BLOCK][TS][64];
        const unsigned wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
        for (int j = 0; j < TS; ++j) xch[wv][j][lane] = best[0][j];
        __syncthreads();   // waves of the workgroup that had no task have ended and are not waited for
        const unsigned w0 = wv - part;   // the task's first wave
#pragma unroll
        for (int j = 0; j < TS; ++j) {
            mine[j] = (unsigned)(j % K) == part;
            if (mine[j]) {
#pragma unroll
                for (int pp = 0; pp < K; ++pp) best[0][j] = min_f64(best[0][j], xch[w0 + pp][j][lane]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < TS; ++j) {
        double a;
        asm("v_mov_b64_dpp %0, %1 row_newbcast:%2 row_mask:0xf bank_mask:0xf" : "=v"(a) : "v"(iav), "n"(j));
        best[0][j] += a;
    }
    const int64_t ld = H.ld;
    const int nvalid = H.S - s0;
    double *drow = H.dst + (int64_t)s0 * ld + u0;
#pragma unroll
    for (int j = 0; j < TS; ++j) {
        if (j < nvalid) {
            if (mine[j] && !stall)
                __hip_atomic_store(drow + lane, best[0][j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            drow += ld;
        }
    }
}

// One wave task: targets [tb*TS, tb*TS+TS) of rows [tile*64*R, (tile+1)*64*R) of the layer described
// by Y.
// PUBLISH: the cost stores are write-through at agent scope, so that a wave on another XCD that
// waits for this task's completion counter finds them in memory.
// ARG: also track and store the argmin (the reference's mark table, csrc/dp_core.cpp:70-72).  Without
// it a relaxation is one addition and one minimum (intra is added once per cell, see the top of this
// file); the backtrack then recomputes the argmin of the few cells on its path from the cost
// buffers, all of which are kept in that mode.
// K > 1 (costs only): the source strategies of a task are split over K waves of the workgroup (vtb =
// target block * K + part; part p takes sources [p * SU / K, (p + 1) * SU / K), SU being a multiple of K times
// the sources per trip) -- for launches whose layers hold too few wave tasks to keep the device's wave slots
// filled: twice the waves, each half as long.  The partial minima meet in LDS; the minimum of the parts is
// the minimum over all sources exactly (min is associative and commutative), and the wave of part j % K adds
// intra to column j and stores it.  Every part counts as a finished wave task of its tile.
template <int TS, int R, bool PUBLISH, bool ARG, int K = 1>
__device__ __forceinline__ void relax_task(const GdpDevLayer *Y, unsigned tile, unsigned vtb, unsigned lane)
{
    static_assert(K == 1 || (!ARG && GDP_WAVES_PER_BLOCK % K == 0), "parts of one task share a workgroup; costs only");
    const unsigned tb = vtb / K, part = vtb % K;
    const int SU = uload(&Y->SU) / K;
    const int SP = uload(&Y->SP);
    const double *src = uload(&Y->src);
    const int64_t *ro = uload(&Y->ro) + part * SU;
    const int s0 = tb * TS;
    const double *it = uload(&Y->it) + s0 + (int64_t)part * SU * SP;
    const double *ia = uload(&Y->ia) + s0;
    const int64_t u0 = (int64_t)tile * (64 * R);

    const unsigned lane_bytes = lane * 8u;

    double add[TS];
#pragma unroll
    for (int j = 0; j < TS; ++j) add[j] = ARG ? uload(ia + j) : 0.0;  // without ARG: fetched after the loop

    double best[R][TS];
    int arg[ARG ? R : 1][ARG ? TS : 1];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < TS; ++j) {
            best[r][j] = INFINITY;
            if constexpr (ARG) arg[r][j] = 0;
        }

    // Software pipeline over the source strategies, NS per trip, with the order of issue pinned by
    // scheduling fences, because a load has to be in flight long before its first use:
    //   - there are NS register sets of cost rows; the rows of strategy sp+NS are requested as soon
    //     as those of sp have been consumed, i.e. NS-1 steps (of TS*R cells each) before they are
    //     needed -- a request that misses the L2 takes several such steps to come back;
    //   - the transition costs of the next strategy and the row offset for the next request are
    //     fetched right after the first column of a step.  Scalar loads return out of order, so
    //     waiting for one means waiting for all: after that first column nothing else is pending.
    // Entries S.. of roff / inter are valid dummies (+inf row, zeros); +inf never wins.
    constexpr int NS = ARG ? 2 : 4;
    static_assert(GDP_SRC_UNROLL % NS == 0 && NS % 2 == 0 && GDP_SRC_PAD > NS, "padding of roff / inter");
    double fp[NS][R], sc[2][TS];
    const double *itp = it;      // row sp of the transition matrix
    const int64_t *rop = ro;     // roff[sp]
    int64_t off = uload(ro + NS);
    {
        // same order of issue as inside the loop, so that the waits at the loop head count alike
        // on both ways into it
        int64_t o0[NS];
#pragma unroll
        for (int u = 0; u < NS; ++u) o0[u] = uload(ro + u);
        GDP_SCHED_FENCE();
        unsigned lb = lane_bytes;
        GDP_PIN_LANE(lb);
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            const double *p = src + o0[u] + u0;
            asm volatile("" : "+s"(p));   // stays a scalar base (see lane_load)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                fp[u][r] = lane_load(p, lb, r);
                GDP_SCHED_FENCE();
            }
        }
#pragma unroll
        for (int j = 0; j < TS; ++j) sc[0][j] = uload(itp + j);
        GDP_SCHED_FENCE();
    }
    for (int sp = 0; sp < SU; sp += NS) {
        unsigned lb = lane_bytes;
        GDP_PIN_LANE(lb);
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            relax_cols<TS, R, ARG, 0, 1>(best, arg, fp[u], sc[u & 1], add, sp + u);
            GDP_SCHED_FENCE();
            itp += SP;
#pragma unroll
            for (int j = 0; j < TS; ++j) sc[(u + 1) & 1][j] = uload(itp + j);
            const int64_t off_next = uload(rop + NS + u + 1);
            GDP_SCHED_FENCE();
            relax_cols<TS, R, ARG, 1, TS>(best, arg, fp[u], sc[u & 1], add, sp + u);
            GDP_SCHED_FENCE();
            {
                const double *pn = src + off + u0;
                asm volatile("" : "+s"(pn));
#pragma unroll
                for (int r = 0; r < R; ++r) fp[u][r] = lane_load(pn, lb, r);
            }
            GDP_SCHED_FENCE();
            off = off_next;
        }
        rop += NS;
    }

    // What the stores need is fetched only now: held in scalar registers across the loop it would
    // crowd out the loop's own operands.  (The opaque copy keeps the compiler from reusing loads
    // made before the loop.)
    const GdpDevLayer *Z = Y;
    asm volatile("" : "+s"(Z));
    bool mine[TS];
#pragma unroll
    for (int j = 0; j < TS; ++j) mine[j] = true;
    if constexpr (K > 1) {
        __shared__ double xch[GDP_WAVES_PER_BLOCK][R][TS][64];
        const unsigned wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < TS; ++j) xch[wv][r][j][lane] = best[r][j];
        __syncthreads();   // waves of the workgroup that had no task have ended and are not waited for
        const unsigned w0 = wv - part;   // the task's first wave
#pragma unroll
        for (int j = 0; j < TS; ++j) {
            mine[j] = (unsigned)(j % K) == part;
            if (mine[j]) {
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int pp = 0; pp < K; ++pp) best[r][j] = min_f64(best[r][j], xch[w0 + pp][r][j][lane]);
            }
        }
    }
    if constexpr (!ARG) {
        const double *iz = uload(&Z->ia) + s0;
#pragma unroll
        for (int j = 0; j < TS; ++j) {
            const double a = uload(iz + j);
#pragma unroll
            for (int r = 0; r < R; ++r) best[r][j] += a;
        }
    }
    const int64_t ld = uload(&Z->ld);
    const int nvalid = uload(&Z->S) - s0;  // target strategies of this block that exist (>= 1)
    double *drow = uload(&Z->dst) + (int64_t)s0 * ld + u0;
    [[maybe_unused]] uint8_t *mrow = nullptr;
    [[maybe_unused]] int64_t ldm = 0;
    if constexpr (ARG) {
        ldm = uload(&Z->ldm);
        mrow = uload(&Z->m) + (int64_t)s0 * ldm + u0;
    }
#pragma unroll
    for (int j = 0; j < TS; ++j) {
        if (j < nvalid) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (!mine[j]) continue;
                if (PUBLISH)
                    __hip_atomic_store(drow + (lane + 64u * r), best[r][j], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                else
                    drow[lane + 64u * r] = best[r][j];
            }
            if constexpr (ARG) {
#pragma unroll
                for (int r = 0; r < R; ++r) mrow[lane + 64u * r] = (uint8_t)arg[r][j];
                mrow += ldm;
            }
            drow += ld;
        }
    }
}

// A tile whose source rows all lie below the first row that can hold a finite cost: every
// candidate is +inf, so the cell is +inf and its argmin 0 (all-equal candidates go to index 0,
// csrc/dp_core.cpp:12-16,70).  Same stores as relax_task, no arithmetic.
template <int TS, int R, bool PUBLISH, bool ARG>
__device__ __forceinline__ void fill_task(const GdpDevLayer *Y, unsigned tile, unsigned tb, unsigned lane)
{
    const int s0 = tb * TS;
    const int64_t u0 = (int64_t)tile * (64 * R);
    const int64_t ld = uload(&Y->ld);
    const int nvalid = uload(&Y->S) - s0;
    double *drow = uload(&Y->dst) + (int64_t)s0 * ld + u0;
    [[maybe_unused]] uint8_t *mrow = nullptr;
    [[maybe_unused]] int64_t ldm = 0;
    if constexpr (ARG) {
        ldm = uload(&Y->ldm);
        mrow = uload(&Y->m) + (int64_t)s0 * ldm + u0;
    }
#pragma unroll
    for (int j = 0; j < TS; ++j) {
        if (j < nvalid) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (PUBLISH)
                    __hip_atomic_store(drow + (lane + 64u * r), (double)INFINITY, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                else
                    drow[lane + 64u * r] = INFINITY;
            }
            if constexpr (ARG) {
#pragma unroll
                for (int r = 0; r < R; ++r) mrow[lane + 64u * r] = 0;
                mrow += ldm;
            }
            drow += ld;
        }
    }
}

// Rows of a layer that have to be computed (tiles lo .. hi): below the band every source cell is
// +inf (fill_task); above it no cell can lie on a path that ends at one of the requested start
// rows, so nothing is read from there later and nothing is written.
template <int TS, int R, bool PUBLISH, bool ARG, int K = 1>
__device__ __forceinline__ void tile_task(const GdpDevLayer *Y, int lo, int hi, unsigned tile, unsigned tb,
                                          unsigned lane)
{
    if ((int)tile > hi) return;
    if ((int)tile < lo) {
        // costs only: every layer has a buffer of its own, and these rows were filled when the plan was made
        if constexpr (ARG) fill_task<TS, R, PUBLISH, ARG>(Y, tile, tb, lane);
    } else {
        relax_task<TS, R, PUBLISH, ARG, K>(Y, tile, tb, lane);   // (K > 1: tb counts the parts of the split tasks too)
    }
}

// ---- one launch per layer ------------------------------------------------------------------------
// __launch_bounds__: register allocation is held to 16 resident waves per CU (4 per SIMD, at most
// 128 VGPRs).
// LAT: 0 = the ordinary task; K >= 1: the latency variant with the sources split over K waves.
template <int TS, int R, bool ARG, int LAT = 0>
__global__ __launch_bounds__(64 * GDP_WAVES_PER_BLOCK, 16 / GDP_WAVES_PER_BLOCK) void gdp_relax_kernel(
    const GdpDevLayer *__restrict__ lay, int max_L, int layer, unsigned ntb)
{
    const GdpDevLayer *Y = lay + ((int64_t)blockIdx.y * max_L + layer);
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned lane = threadIdx.x & 63u;
    // Only the tiles lo..hi of this layer carry arithmetic.  The first blocks of the grid share them
    // out, every XCD getting one contiguous range of them (equal work per XCD, neighbouring budget
    // rows in one L2); the blocks after those fill the tiles below lo; tiles above hi are left alone.
    // (A table entry of an instance that has no such layer has hi = -1 and lo = 0.)
    if constexpr (LAT > 0) {
        const LatHead H = load_lat_head(Y);
        const unsigned live_tasks = H.hi >= H.lo ? (unsigned)(H.hi - H.lo + 1) * ntb : 0u;
        const unsigned live_blocks = ((live_tasks + GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK + 7u) & ~7u;
        if (blockIdx.x >= live_blocks) return;   // (costs only: the rows below the band were filled when the plan was made)
        const unsigned task = xcd_swizzle(blockIdx.x, live_blocks) * GDP_WAVES_PER_BLOCK + wave;
        if (task >= live_tasks) return;
        const unsigned t = task / ntb;
        relax_task_lat<TS, R, false, LAT>(H, (unsigned)H.lo + t, task - t * ntb, lane);
    } else {
        const int lo = uload(&Y->lo), hi = uload(&Y->hi);
        const unsigned live_tasks = hi >= lo ? (unsigned)(hi - lo + 1) * ntb : 0u;
        const unsigned live_blocks = ((live_tasks + GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK + 7u) & ~7u;
        if (blockIdx.x < live_blocks) {
            const unsigned task = xcd_swizzle(blockIdx.x, live_blocks) * GDP_WAVES_PER_BLOCK + wave;
            if (task >= live_tasks) return;
            const unsigned t = task / ntb;
            relax_task<TS, R, false, ARG>(Y, (unsigned)lo + t, task - t * ntb, lane);
        } else if constexpr (ARG) {  // (costs only: those rows were filled when the plan was made)
            const unsigned task = (blockIdx.x - live_blocks) * GDP_WAVES_PER_BLOCK + wave;
            const unsigned t = task / ntb;
            const int top = lo - 1 < hi ? lo - 1 : hi;  // fill tiles 0 .. min(lo-1, hi)
            if ((int)t > top) return;
            fill_task<TS, R, false, ARG>(Y, t, task - t * ntb, lane);
        }
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
    // First a look at up to four lanes-wide chunks at once (one round trip instead of four when
    // everything is ready, as it mostly is); the chunks that are not are polled one after the other.
    int first_unready = lo;
    {
        int v[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int t = lo + 64 * c + (int)lane;
            v[c] = (t <= hi) ? ld_agent(cnt + t) : full;
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (__builtin_amdgcn_ballot_w64(v[c] < full) != 0) break;
            first_unready = lo + 64 * (c + 1);
        }
    }
    for (int base = first_unready; base <= hi; base += 64) {
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
// (tile, target block) wave tasks of one instance).  Workgroups are dispatched in order of their
// linear id, x fastest, so every block of layer l is dispatched before any block of layer l+1; a
// block only ever waits for blocks of the layer before its own, which therefore run or have
// finished, and the oldest unfinished block never waits: the launch cannot deadlock.  (Each XCD
// takes every eighth workgroup and dispatches its share in order, which is all the argument needs.)
// Older workgroups also win the issue arbitration of their SIMD, so the work that others wait for
// runs first.
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
//
// Share of an XCD: of every instance, every eighth group of block tasks (see below).
// K > 1: the sources of a task are split over K waves (see relax_task); Q.ntb then counts the parts, so that
// a tile is finished when ntb wave tasks have counted themselves.
template <int TS, int R, bool ARG, int K = 1>
__global__ __launch_bounds__(64 * GDP_WAVES_PER_BLOCK, 16 / GDP_WAVES_PER_BLOCK) void gdp_relax_fused_kernel(
    const GdpSched Q, int layer0)
{
    __shared__ int sh_ok;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned lane = threadIdx.x & 63u;
    // What this grid row is: layer layer0+y of all instances that have it, or -- chunked launch -- one
    // layer of a few consecutive instances.  Grid rows are dispatched in order, so a chunked launch
    // takes a few instances through ALL their layers before it turns to the next few: what a layer
    // wrote is then still in the memory-side cache when the next layer reads it.
    const int32_t *rows = Q.rows;
    int layer = layer0 + (int)blockIdx.y;
    unsigned first_inst = 0, n_inst = ~0u;
    if (rows) {
        const int32_t *row = rows + 3 * (int64_t)(layer0 + (int)blockIdx.y);
        first_inst = (unsigned)uload(row);
        n_inst = (unsigned)uload(row + 1);
        layer = uload(row + 2);
    }
    const int max_L = Q.max_L;
    const int max_ntile = Q.max_ntile;
    const unsigned ntb = (unsigned)Q.ntb;
    const unsigned nat = (unsigned)uload(Q.n_active + layer);
    const unsigned xcd = blockIdx.x & 7u;   // workgroups go to the XCDs round-robin by linear id;
    const unsigned pos = blockIdx.x >> 3;   // gridDim.x is a multiple of 8
    // Instance-major: the workgroups that an XCD runs at the same time work on a few instances only.
    const unsigned slots = (unsigned)Q.slots;
    const unsigned k = pos / slots;         // instance within the grid row
    const unsigned ii = first_inst + k;     // instance (a prefix of the table has this layer)
    const unsigned w = pos - k * slots;     // slot within the XCD's share of that instance
    if (k >= n_inst || ii >= nat) return;
    const GdpDevLayer *Y = Q.lay + ((int64_t)ii * max_L + layer);
    const int ntile = uload(&Y->ntile);
    const unsigned nbt = ((unsigned)ntile * ntb + GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK;
    const int lo = uload(&Y->lo), hi = uload(&Y->hi);
    // Block tasks run over (tile, target block) in that order; groups of `group` consecutive ones
    // (whole tiles) are dealt to the XCDs in turn, and every XCD takes its groups in ascending order.
    // So all XCDs move up the budget rows of a layer side by side: whatever the band of the layer is,
    // each carries an eighth of it, and what a block waits for -- tiles at and below its own in the
    // layer before -- was handed out a whole layer earlier on every XCD.
    const unsigned G = (unsigned)Q.group;
    const unsigned grp = w / G;
    unsigned bt = (grp * 8u + xcd) * G + (w - grp * G);
    bool live = false;
    if constexpr (ARG) {
        if (bt >= nbt) return;
        if (hi >= lo) {
            const unsigned bt_lo = ((unsigned)lo * ntb) / GDP_WAVES_PER_BLOCK;
            const unsigned bt_hi = (((unsigned)hi + 1u) * ntb - 1u) / GDP_WAVES_PER_BLOCK;
            live = bt >= bt_lo && bt <= bt_hi;   // carries arithmetic; the others only fill or count as done
        }
    } else {
        // Costs only: the rows below the band were filled when the plan was made and the rows above
        // it are never read, so only the band's block tasks exist: the slots count from the band's
        // first group of whole tiles, and a reader waits for tiles of the previous band only.
        if (hi < lo) return;
        const unsigned bt_lo = ((unsigned)lo * ntb) / GDP_WAVES_PER_BLOCK;
        const unsigned bt_hi = (((unsigned)hi + 1u) * ntb - 1u) / GDP_WAVES_PER_BLOCK;
        bt += bt_lo / G * G;
        if (bt < bt_lo || bt > bt_hi || bt >= nbt) return;
        live = true;
    }
    int32_t *cnt_all = Q.cnt;
    // touch what the task reads first (row offsets, first transition costs), so that it sits in the
    // scalar cache by the time the wait is over
    int64_t pf_o = 0;
    double pf_a = 0, pf_b = 0;
    if (live) {
        const unsigned qq = bt * GDP_WAVES_PER_BLOCK + wave;
        const unsigned tl = qq / ntb, tbb = qq - tl * ntb;
        const int64_t *ro_ = uload(&Y->ro);
        const double *it_ = uload(&Y->it) + (tbb / K) * TS;
        pf_o = uload(ro_);
        pf_a = uload(it_);
        pf_b = uload(it_ + (TS - 1));
    }
    const unsigned q0 = bt * GDP_WAVES_PER_BLOCK;
    if (live && layer >= 1) {
        // the block's first wave waits for everything its four wave tasks read
        if (wave == 0) {
            const int t_lo = (int)(q0 / ntb);
            int t_hi = (int)((q0 + GDP_WAVES_PER_BLOCK - 1) / ntb);
            if (t_hi >= ntile) t_hi = ntile - 1;
            const int d = uload(&Y[-1].dep);
            int first = t_lo - d < 0 ? 0 : t_lo - d;
            if constexpr (!ARG) {  // tiles outside the previous band have no counter to wait for
                const int plo = uload(&Y[-1].lo), phi = uload(&Y[-1].hi);
                if (first < plo) first = plo;
                if (t_hi > phi) t_hi = phi;
            }
            const bool ok = wait_tiles(cnt_all + ((int64_t)ii * max_L + (layer - 1)) * max_ntile, first, t_hi, (int)ntb,
                                       lane, Q.abort_flag, Q.spin_limit);
            if (lane == 0) sh_ok = ok ? 1 : 0;
        }
        __syncthreads();
        if (__builtin_amdgcn_readfirstlane(sh_ok) == 0) return;  // the launch is being abandoned
    }
    asm volatile("" ::"s"(pf_o), "s"(pf_a), "s"(pf_b));
    const unsigned q = q0 + wave;
    const unsigned tile = q / ntb;
    const unsigned tb = q - tile * ntb;
    if (tile >= (unsigned)ntile) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");    // keeps the tile's loads after the wait
    tile_task<TS, R, true, ARG, K>(Y, lo, hi, tile, tb, lane);   // with the argmin table: tiles outside the band
                                                              // are filled or skipped there and count as done
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // every write-through store acknowledged
    if (lane == 0 && !(Q.debug_stall && layer == 0))
        __hip_atomic_fetch_add(cnt_all + ((int64_t)ii * max_L + layer) * max_ntile + tile, 1, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
}

// ---- all layers in one launch, waiting on the cost cells themselves (small problems) ---------------
// A problem whose layers are over in a few microseconds each spends its time between the layers: a
// launch gap, the start of the workgroups, the first dependent loads; completion counters cost more
// than they save at that size (a counter needs the stores acknowledged before it is bumped and a
// round trip to be seen, before the first cost row can even be asked for).  Here the cost cells are
// their own flags: before a run every cell that the run writes holds NaN (gdp_flow_reset_kernel) -- no
// cost is ever NaN: NaN and -inf inputs are rejected on the host and +inf - inf cannot arise -- and a
// task looks at them at agent scope before it reads its cost rows, and asks again for any row in which
// a lane still sees NaN (relax_task_flow).  A cell is one aligned 8-byte store, so a reader sees the pattern or the
// cost, nothing in between; the stores are write-through at agent scope and nobody waits for them.
// What a layer's task needs apart from the cost rows (its record, row offsets, transition and intra
// costs) is fetched while the previous layer is still at work.
// grid = (block tasks of the widest band, layers, instances): workgroups are dispatched in order of
// their linear id, so every task a task waits for was dispatched before it (the argument of
// gdp_relax_fused_kernel); waits are bounded, a wave that gives up raises the abort flag, the launch
// drains and the host repeats the solve with one launch per layer.
// The bands must be closed under reading: every row that a task of layer l's band reads from layer
// l-1's output lies in that layer's band, below it (filled once per plan) or in the pads.
template <int NSRC, int K>
__global__ __launch_bounds__(64 * GDP_WAVES_PER_BLOCK, 8 / GDP_WAVES_PER_BLOCK) void gdp_relax_flow_kernel(
    const GdpDevLayer *__restrict__ lay, int max_L, int layer0, unsigned ntb, int32_t *abort_flag, int64_t spin_limit,
    int debug_stall)
{
    const GdpDevLayer *Y = lay + ((int64_t)blockIdx.z * max_L + layer0 + (int)blockIdx.y);
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned lane = threadIdx.x & 63u;
    const FlowHead H = load_flow_head(Y);
    const unsigned live_tasks = H.hi >= H.lo ? (unsigned)(H.hi - H.lo + 1) * ntb : 0u;
    const unsigned task = blockIdx.x * GDP_WAVES_PER_BLOCK + wave;   // ascending: what others wait for comes first
    if (task >= live_tasks) return;
    const unsigned t = task / ntb;
    FlowWait fw = {abort_flag, spin_limit, 0, false};
    relax_task_flow<GDP_LAT_TS, NSRC, K>(H, (unsigned)H.lo + t, task - t * ntb, lane, fw,
                                         debug_stall != 0 && layer0 + (int)blockIdx.y == 0);
}

// NaN into every cell that a flow launch writes (the bands of all layers), and zero into its abort flag.
// grid = (x chunks, rows 0..S-1, instances x layers); buffer l + 1 holds the output of layer l.
__global__ __launch_bounds__(256) void gdp_flow_reset_kernel(const GdpDevInst *__restrict__ insts,
                                                             const GdpDevLayer *__restrict__ lay, int max_L,
                                                             int tile_rows, int32_t *abort_flag)
{
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0) *abort_flag = 0;
    const int inst = blockIdx.z / max_L, l = blockIdx.z - inst * max_L;
    const GdpDevInst *I = insts + inst;
    if (l >= uload(&I->L) || (int)blockIdx.y >= uload(&I->S)) return;
    const GdpDevLayer *Y = lay + ((int64_t)inst * max_L + l);
    const int lo = uload(&Y->lo), hi = uload(&Y->hi);
    if (hi < lo) return;
    const int64_t first = (int64_t)lo * tile_rows, n = (int64_t)(hi - lo + 1) * tile_rows;
    double *h = uload(&I->H) + (int64_t)(l + 1) * uload(&I->hstride) + (int64_t)blockIdx.y * uload(&I->ld) + uload(&I->P) + first;
    const double nan = __builtin_nan("");
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        h[i] = nan;
}

__global__ __launch_bounds__(256) void gdp_zero_kernel(int32_t *p, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        p[i] = 0;
}

// Fills of the cost buffers (see GDP_INIT_* in gdp_kernels.h).  grid = (x chunks, rows 0..S, instances).
// GDP_INIT_FILL: grid = (x chunks, rows 0..S-1, instances x layers); buffer l + 1 holds the output of layer l.
__global__ __launch_bounds__(256) void gdp_fill_kernel(const GdpDevInst *__restrict__ insts,
                                                       const GdpDevLayer *__restrict__ lay, int max_L, int tile_rows)
{
    const int inst = blockIdx.z / max_L, l = blockIdx.z - inst * max_L;
    const GdpDevInst *I = insts + inst;
    if (l >= uload(&I->L) || (int)blockIdx.y >= uload(&I->S)) return;
    int64_t n = (int64_t)uload(&lay[(int64_t)inst * max_L + l].lo) * tile_rows;
    const int64_t from = uload(&lay[(int64_t)inst * max_L + l].fill_from);
    const int64_t ldm = uload(&I->ldm);
    if (n > ldm) n = ldm;
    double *h = uload(&I->H) + (int64_t)(l + 1) * uload(&I->hstride) + (int64_t)blockIdx.y * uload(&I->ld) + uload(&I->P);
    for (int64_t i = from + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        h[i] = INFINITY;
}

// Everything a costs-only plan needs in its cost buffers before its first run, in one launch: +inf in
// the pads in front of every row and in the +inf row of every buffer, zeros in buffer 0 (the caller's
// initial f), +inf in the rows below the band of every layer's output that something reads, and -- with
// `nan_bands`, for a plan that will run as a flow launch -- NaN in the bands.
// grid = (x chunks, rows 0..S, instances x (max_L + 1) buffers).
// Row `row` of one cost buffer (h: its first element, pad included): the output of a layer whose band is
// [lo, hi] tiles and whose rows from fill_from up to the band are read by something -- or, `whole`, buffer 0
// (zeros behind the pad) or the +inf row of any buffer.
__device__ __forceinline__ void prepare_row(double *h, bool whole, bool inf_row, int64_t ld, int64_t P, int lo, int hi,
                                            int64_t fill_from, int tile_rows, int nan_bands)
{
    const double inf = INFINITY;
    const double nan = __builtin_nan("");
    if (whole) {
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < ld; i += (int64_t)gridDim.x * blockDim.x)
            h[i] = (inf_row || i < P) ? inf : 0.0;
        return;
    }
    int64_t band_from = (int64_t)lo * tile_rows;
    int64_t band_to = hi >= lo ? (int64_t)(hi + 1) * tile_rows : band_from;
    if (band_from > ld - P) band_from = ld - P;
    if (band_to > ld - P) band_to = ld - P;
    // the pad, then rows fill_from .. end of what is written (nothing in between is touched)
    const int64_t end = nan_bands ? band_to : band_from;
    const int64_t n = P + (end > fill_from ? end - fill_from : 0);
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += (int64_t)gridDim.x * blockDim.x) {
        const int64_t u = j < P ? j - P : j - P + fill_from;
        h[P + u] = (u < band_from) ? inf : nan;
    }
}

__global__ __launch_bounds__(256) void gdp_prepare_kernel(const GdpDevInst *__restrict__ insts,
                                                          const GdpDevLayer *__restrict__ lay, int max_L, int tile_rows,
                                                          int nan_bands, int32_t *abort_flag)
{
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0) *abort_flag = 0;
    const int inst = blockIdx.z / (max_L + 1), b = blockIdx.z - inst * (max_L + 1);
    const GdpDevInst *I = insts + inst;
    const int S = uload(&I->S), L = uload(&I->L);
    const int row = blockIdx.y;
    if (b > L || row > S) return;
    const int64_t ld = uload(&I->ld);
    const int64_t P = uload(&I->P);
    double *h = uload(&I->H) + (int64_t)b * uload(&I->hstride) + (int64_t)row * ld;
    int lo = 0, hi = -1;
    int64_t fill_from = 0;   // rows of this buffer (layer b - 1's output)
    if (b >= 1) {
        const GdpDevLayer *Y = lay + ((int64_t)inst * max_L + (b - 1));
        lo = uload(&Y->lo);
        hi = uload(&Y->hi);
        fill_from = uload(&Y->fill_from);
    }
    prepare_row(h, row == S || b == 0, row == S, ld, P, lo, hi, fill_from, tile_rows, nan_bands);
}

// The same for a few small instances, everything it needs in its arguments: it can then run before the
// plan's tables have been uploaded, beside their upload (and beside the host's work on them).
// grid = (x chunks, rows 0..max S, buffers of all instances).
__global__ __launch_bounds__(256) void gdp_prepare_args_kernel(const GdpPrepArgs A)
{
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0) *A.abort_flag = 0;
    int inst = 0, b = (int)blockIdx.z;     // buffer b of instance inst
    while (inst + 1 < A.n_inst && b > A.inst[inst].L) {
        b -= A.inst[inst].L + 1;
        ++inst;
    }
    const int S = A.inst[inst].S, L = A.inst[inst].L;
    const int row = blockIdx.y;
    if (b > L || row > S) return;
    const int64_t ld = A.inst[inst].ld;
    const int64_t P = A.inst[inst].P;
    double *h = A.inst[inst].H + (int64_t)b * A.inst[inst].hstride + (int64_t)row * ld;
    int lo = 0, hi = -1;
    int64_t fill_from = 0;
    if (b >= 1) {
        const int e = A.inst[inst].first_layer + (b - 1);
        lo = A.lo[e];
        hi = A.hi[e];
        fill_from = A.fill_from[e];
    }
    prepare_row(h, row == S || b == 0, row == S, ld, P, lo, hi, fill_from, A.inst[inst].tile_rows, A.nan_bands);
}

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

// ---- strategies with a memory cost of 0 -------------------------------------------------------------
// See gdp_launch_zero_pass.  grid = (blocks of 256 bins, instances).  Only the bins of the layer's band are
// redone: below it every candidate is +inf (the cells hold +inf, argmin 0, from the fills), above it nothing
// was written by the layer's launch and nothing is read later.  A lane owns bin v and walks the
// layer's mem == 0 strategies in ascending order; what it stores for one of them is what it (and only
// it) reads back as a candidate of the next ones.  Candidates, association and tie-break are the
// reference's: (f + inter) + intra, ascending source strategies, replaced on strict '<'
// (csrc/dp_core.cpp:65-72).
template <bool MARKS>
__global__ __launch_bounds__(256) void gdp_zero_pass_kernel(const GdpDevInst *insts, const GdpDevLayer *lay, int max_L,
                                                            int tile_rows, int layer)
{
    const GdpDevInst *I = insts + blockIdx.y;
    const int32_t *zc = uload(&I->zcols);
    if (!zc || layer >= uload(&I->L)) return;
    const int S = uload(&I->S), V = uload(&I->V);
    const int32_t *z = zc + (int64_t)layer * (S + 1);
    const int nz = uload(z);
    const int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (nz == 0 || v >= V) return;
    const GdpDevLayer *Y = lay + ((int64_t)blockIdx.y * max_L + layer);
    const int lo = uload(&Y->lo), hi = uload(&Y->hi);
    if (hi < lo || v < (int64_t)lo * tile_rows || v >= (int64_t)(hi + 1) * tile_rows) return;
    const int rows = uload(&I->SU) + GDP_SRC_PAD, SP = uload(&I->SP), nbuf = uload(&I->nbuf);
    const int64_t hstride = uload(&I->hstride);
    double *H = uload(&I->H);
    const double *old_costs = H + (int64_t)(layer % nbuf) * hstride;      // what the layer reads
    double *new_costs = H + (int64_t)((layer + 1) % nbuf) * hstride;      // what it writes
    const int64_t *ro_old = uload(&I->roff) + (int64_t)layer * rows;
    const int64_t *ro_new = ro_old + rows;
    const double *it = uload(&I->inter) + (int64_t)uload(uload(&I->inter_index) + layer) * rows * SP;
    const double *ia = uload(&I->intra) + (int64_t)layer * SP;
    [[maybe_unused]] uint8_t *M = nullptr;
    [[maybe_unused]] int64_t ldm = 0;
    if constexpr (MARKS) {
        ldm = uload(&I->ldm);
        M = uload(&I->M) + (int64_t)layer * S * ldm;
    }
    for (int k = 0; k < nz; ++k) {
        const int s = uload(z + 1 + k);
        const double a = uload(ia + s);
        double best = 0;
        int arg = 0;
        for (int sp = 0; sp < S; ++sp) {
            const double x = sp < s ? new_costs[uload(ro_new + sp) + v] : old_costs[uload(ro_old + sp) + v];
            const double c = (x + uload(it + (int64_t)sp * SP + s)) + a;
            if (sp == 0 || c < best) {
                best = c;
                arg = sp;
            }
        }
        new_costs[uload(ro_new + s) + v] = best;     // mem == 0: the cell's own bin
        if constexpr (MARKS) M[(int64_t)s * ldm + v] = (uint8_t)arg;
    }
}

// ---- wavefront (value, index) reduction: lower value wins, equal values -> lower index ----------
// One combining step through the data-parallel-primitive path of the vector ALU (no LDS round trip):
// every enabled lane looks at the pair of the lane that CTRL names and keeps the better of the two;
// lanes that CTRL gives no source, and rows outside ROW_MASK, see their own pair again and keep it.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void argmin_step(double &val, int &idx)
{
    const int lo = __double2loint(val), hi = __double2hiint(val);
    const int olo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xf, false);
    const int ohi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xf, false);
    const int oi = __builtin_amdgcn_update_dpp(idx, idx, CTRL, ROW_MASK, 0xf, false);
    const double ov = __hiloint2double(ohi, olo);
    if (ov < val || (ov == val && oi < idx)) { val = ov; idx = oi; }
}

// On return every lane holds the wavefront's best pair.  Within each row of 16 lanes the pairs are
// folded towards lane 15 (shifts by 1, 2, 4, 8), lane 15 of rows 0 and 2 is then broadcast into rows 1
// and 3, lane 31 into rows 2 and 3; lane 63 ends up with the result, which is read out of it.
__device__ __forceinline__ void wave_argmin(double &val, int &idx)
{
    argmin_step<0x111, 0xf>(val, idx);   // row_shr:1
    argmin_step<0x112, 0xf>(val, idx);   // row_shr:2
    argmin_step<0x114, 0xf>(val, idx);   // row_shr:4
    argmin_step<0x118, 0xf>(val, idx);   // row_shr:8
    argmin_step<0x142, 0xa>(val, idx);   // row_bcast:15 into rows 1 and 3
    argmin_step<0x143, 0xc>(val, idx);   // row_bcast:31 into rows 2 and 3
    idx = __builtin_amdgcn_readlane(idx, 63);
    val = __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(val), 63),
                           __builtin_amdgcn_readlane(__double2loint(val), 63));
}

// The wavefront's lowest value, in every lane; same folding as wave_argmin.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void min_step(double &val)
{
    const int lo = __double2loint(val), hi = __double2hiint(val);
    const int olo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xf, false);
    const int ohi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xf, false);
    val = min_f64(val, __hiloint2double(ohi, olo));
}

__device__ __forceinline__ double wave_min(double val)
{
    min_step<0x111, 0xf>(val);
    min_step<0x112, 0xf>(val);
    min_step<0x114, 0xf>(val);
    min_step<0x118, 0xf>(val);
    min_step<0x142, 0xa>(val);
    min_step<0x143, 0xc>(val);
    return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(val), 63),
                            __builtin_amdgcn_readlane(__double2loint(val), 63));
}

// Lane s holds candidate s (+inf in lanes that hold none): the lowest index among the lowest candidates
// -- the lowest lane whose value equals the wavefront's minimum; lane 0 when all are +inf.  A third of
// the instructions of the reduction over (value, index) pairs.
__device__ __forceinline__ int wave_argmin_by_lane(double val)
{
    const double lowest = wave_min(val);
    const unsigned long long eq = __builtin_amdgcn_ballot_w64(val == lowest);
    return eq ? (int)__builtin_ctzll(eq) : 64;   // (no lane equals the minimum only if the values are NaN)
}

// Epilogue of csrc/dp_core.cpp:78-117 for one key per wavefront: first argmin of the start row,
// then the dependent walk back through the layers.  MARKS: the walk reads the stored argmin table.
// Otherwise every cost buffer of the run is still there, and the wavefront recomputes the argmin of
// the one cell per layer that lies on its path, with the arithmetic and the tie-break of the
// relaxation (csrc/dp_core.cpp:67-73: ascending source strategies, strict '<', so the lowest index
// among equal candidates, and index 0 when all are +inf).
template <bool MARKS>
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
    const int nbuf = uload(&I->nbuf);
    const int64_t hstride = uload(&I->hstride);
    const double *H = uload(&I->H);
    const int rows = uload(&I->SU) + GDP_SRC_PAD;
    const int64_t *roff = uload(&I->roff);
    const double *fin = H + (int64_t)(L % nbuf) * hstride;  // last written
    const int64_t *ro = roff + (int64_t)L * rows;
    double val = INFINITY;
    int idx = 0x7fffffff;
    for (int s = lane; s < S; s += 64) {  // ascending within the lane: strict '<' keeps the first
        const double x = fin[ro[s] + v0];
        if (x < val || idx == 0x7fffffff) { val = x; idx = s; }
    }
    wave_argmin(val, idx);  // every lane holds the result
    idx = __builtin_amdgcn_readfirstlane(idx);
    if (!(val < INFINITY)) {  // csrc/dp_core.cpp:93-97
        if (lane == 0) out[blockIdx.x] = o;
        return;
    }
    o.total = val + uload(&K->other_time);  // csrc/dp_core.cpp:99
    const int32_t *mem = uload(&I->mem);
    int32_t *path = res + uload(&K->res_off);
    int64_t v = v0;
    if (lane == 0) path[L - 1] = idx;
    if constexpr (MARKS) {
        const uint8_t *M = uload(&I->M);
        const int64_t ldm = uload(&I->ldm);
        for (int i = L - 1; i > 0; --i) {  // csrc/dp_core.cpp:105-113, with mark[i][v][s] = M[i][s][v - mem[i][s]]
            const int cur = idx;
            v -= uload(mem + (int64_t)i * S + cur);
            if (v < 0) break;  // cannot happen on a finite path; keeps a damaged table from being indexed
            idx = __builtin_amdgcn_readfirstlane((int)M[((int64_t)i * S + cur) * ldm + v]);
            if (idx >= S) { v = -1; break; }
            if (lane == 0) path[i - 1] = idx;
        }
    } else {
        const int SP = uload(&I->SP);
        const double *inter = uload(&I->inter);
        const double *intra = uload(&I->intra);
        const int32_t *inter_index = uload(&I->inter_index);
        int i = L - 1;
        if (S <= 64) {
            // Up to 64 strategies: lane s keeps what layer i holds for strategy s -- memory cost, row
            // offset, intra cost -- fetched one layer ahead, so that the step from a cell to its
            // predecessor is a lane read, one round of gathered loads (cost row and transition column
            // together) and the reduction, instead of a dependent scalar load before the gather.
            // The one wavefront is bound by its own chain of instructions as much as by the round trip, so the
            // step is kept short: the addresses move by a stride per layer instead of being multiplied out, and
            // the reduction is over values only (wave_argmin_by_lane).
            const int sl = lane < S ? lane : S - 1;
            const int32_t *mem_p = mem + (int64_t)i * S + sl;          // layer i, this lane's strategy
            const int64_t *roff_p = roff + (int64_t)i * rows + sl;
            const double *intra_p = intra + (int64_t)i * SP + sl;
            const int32_t *index_p = inter_index + i;
            const double *inter_lane = inter + (int64_t)sl * SP;      // row `lane` of matrix 0
            const int64_t mat_stride = (int64_t)rows * SP;
            int b = i % nbuf;                                         // the cost buffer that holds the costs before layer i
            const double *src = H + (int64_t)b * hstride;
            int m_next = *mem_p;
            int64_t r_next = *roff_p;
            double a_next = *intra_p;
            int64_t t_next = uload(index_p) * mat_stride;
            for (; i > 0; --i) {
                const int cur = idx;
                const int m_cur = m_next;
                const int64_t r_cur = r_next;
                const double a_cur = a_next;
                const int64_t t_cur = t_next;
                if (i > 1) {
                    mem_p -= S;
                    roff_p -= rows;
                    intra_p -= SP;
                    index_p -= 1;
                    m_next = *mem_p;
                    r_next = *roff_p;
                    a_next = *intra_p;
                    t_next = uload(index_p) * mat_stride;
                }
                const int m_here = __builtin_amdgcn_readlane(m_cur, cur);
                v -= m_here;  // the source row of cell (i, v, cur)
                if (v < 0) break;
                const double a = __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(a_cur), cur),
                                                  __builtin_amdgcn_readlane(__double2loint(a_cur), cur));
                double bv = INFINITY;
                if (lane < S) {
                    double x = src[r_cur + v];
                    // a cell with mem == 0 took its lower strategies from its own layer (gdp_launch_zero_pass)
                    if (m_here == 0 && lane < cur)
                        x = H[(int64_t)((i + 1) % nbuf) * hstride + roff[(int64_t)(i + 1) * rows + lane] + v];
                    bv = (x + inter_lane[t_cur + cur]) + a;
                }
                idx = wave_argmin_by_lane(bv);
                if (idx >= S) { v = -1; break; }
                if (lane == 0) path[i - 1] = idx;
                if (--b < 0) {
                    b = nbuf - 1;
                    src = H + (int64_t)b * hstride;
                } else {
                    src -= hstride;
                }
            }
            i = 0;
        }
        for (; i > 0; --i) {
            const int cur = idx;
            const int m_here = uload(mem + (int64_t)i * S + cur);
            v -= m_here;  // the source row of cell (i, v, cur)
            if (v < 0) break;
            const double *src = H + (int64_t)(i % nbuf) * hstride;  // costs before layer i
            const double *own = H + (int64_t)((i + 1) % nbuf) * hstride;  // costs after it
            const int64_t *rl = roff + (int64_t)i * rows;
            const double *it = inter + (int64_t)uload(inter_index + i) * rows * SP + cur;
            const double a = uload(intra + (int64_t)i * SP + cur);
            double bv = INFINITY;
            int bi = 0x7fffffff;
            for (int s = lane; s < S; s += 64) {
                const double x = (m_here == 0 && s < cur) ? own[rl[rows + s] + v] : src[rl[s] + v];
                const double c = (x + it[(int64_t)s * SP]) + a;
                if (c < bv || bi == 0x7fffffff) { bv = c; bi = s; }
            }
            wave_argmin(bv, bi);
            idx = __builtin_amdgcn_readfirstlane(bi);
            if (idx >= S) { v = -1; break; }
            if (lane == 0) path[i - 1] = idx;
        }
    }
    if (lane != 0) return;
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
    const int64_t *ro = I->roff + (int64_t)L * (I->SU + GDP_SRC_PAD);
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

template <int TS, int R, bool ARG, int LAT = 0>
static hipError_t launch_relax_t(const GdpDevLayer *lay, int max_L, int n_inst, int max_ntile_rows, int SP, int layer,
                                 hipStream_t stream)
{
    const unsigned ntb = (unsigned)(SP / TS) * (LAT > 1 ? (unsigned)LAT : 1u);  // with the parts of a split task
    const unsigned tasks = (unsigned)max_ntile_rows * ntb;
    unsigned nblk = (tasks + GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK;
    nblk = ((nblk + 7u) & ~7u) + 8u;  // live blocks are rounded up to 8, the fill blocks come after them
    dim3 grid(nblk, (unsigned)n_inst, 1), block(64 * GDP_WAVES_PER_BLOCK, 1, 1);
    hipLaunchKernelGGL((gdp_relax_kernel<TS, R, ARG, LAT>), grid, block, 0, stream, lay, max_L, layer, ntb);
    return hipGetLastError();
}

// one entry per element of GDP_VARIANTS, in the same order: (index, TS, R, built with the argmin table)
#define GDP_FOR_EACH_VARIANT(X)                                                                       \
    X(0, 16, 3, false) X(1, 16, 2, false) X(2, 16, 1, false) X(3, 15, 3, false) X(4, 15, 2, false)        \
    X(5, 15, 1, false) X(6, 14, 3, false) X(7, 14, 2, false) X(8, 14, 1, false) X(9, 13, 3, false)        \
    X(10, 13, 2, false) X(11, 13, 1, false) X(12, 12, 3, false) X(13, 12, 2, false) X(14, 12, 1, false)   \
    X(15, 11, 3, true) X(16, 11, 2, true) X(17, 11, 1, true) X(18, 8, 4, true) X(19, 8, 2, true)          \
    X(20, 8, 1, true)

template <int TS, int R, bool MARKS_BUILT>
static hipError_t launch_relax_v(bool marks, const GdpDevLayer *lay, int max_L, int n_inst, int max_ntile, int SP, int layer,
                          hipStream_t stream)
{
    if constexpr (MARKS_BUILT) {
        if (marks) return launch_relax_t<TS, R, true>(lay, max_L, n_inst, max_ntile, SP, layer, stream);
    } else if (marks) {
        return hipErrorInvalidValue;
    }
    return launch_relax_t<TS, R, false>(lay, max_L, n_inst, max_ntile, SP, layer, stream);
}

template <int TS, int R, bool MARKS_BUILT>
static hipError_t launch_fused_v(bool marks, int split, dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream,
                          const GdpSched &sched, int layer0)
{
    if (split != 1) {
        if constexpr (R == GDP_SPLIT_R) {
            if (split == 2 && !marks) {
                hipLaunchKernelGGL((gdp_relax_fused_kernel<TS, R, false, 2>), grid, block, lds_bytes, stream, sched, layer0);
                return hipGetLastError();
            }
        }
        return hipErrorInvalidValue;
    }
    if constexpr (MARKS_BUILT) {
        if (marks) {
            hipLaunchKernelGGL((gdp_relax_fused_kernel<TS, R, true>), grid, block, lds_bytes, stream, sched, layer0);
            return hipGetLastError();
        }
    } else if (marks) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL((gdp_relax_fused_kernel<TS, R, false>), grid, block, lds_bytes, stream, sched, layer0);
    return hipGetLastError();
}

hipError_t gdp_launch_relax(int variant, bool marks, int latency, const GdpDevLayer *lay, int max_L, int n_inst,
                            int max_ntile, int SP, int layer, hipStream_t stream)
{
    if (latency) {
        if (marks || variant < 0 || variant >= GDP_NUM_VARIANTS || GDP_VARIANTS[variant].ts != GDP_LAT_TS ||
            GDP_VARIANTS[variant].r != GDP_LAT_R)
            return hipErrorInvalidValue;
        switch (latency) {
            case 1: return launch_relax_t<GDP_LAT_TS, GDP_LAT_R, false, 1>(lay, max_L, n_inst, max_ntile, SP, layer, stream);
            case 2: return launch_relax_t<GDP_LAT_TS, GDP_LAT_R, false, 2>(lay, max_L, n_inst, max_ntile, SP, layer, stream);
            case 4: return launch_relax_t<GDP_LAT_TS, GDP_LAT_R, false, 4>(lay, max_L, n_inst, max_ntile, SP, layer, stream);
            default: return hipErrorInvalidValue;
        }
    }
#define X(id, ts, r, m) \
    case id: return launch_relax_v<ts, r, m>(marks, lay, max_L, n_inst, max_ntile, SP, layer, stream);
    switch (variant) {
        GDP_FOR_EACH_VARIANT(X)
        default: return hipErrorInvalidValue;
    }
#undef X
}

hipError_t gdp_launch_relax_fused(int variant, bool marks, int split, const GdpSched &sched, int grid_blocks, int layer0,
                                  int layers, unsigned lds_bytes, hipStream_t stream)
{
    dim3 grid((unsigned)grid_blocks, (unsigned)layers), block(64 * GDP_WAVES_PER_BLOCK);
#define X(id, ts, r, m) \
    case id: return launch_fused_v<ts, r, m>(marks, split, grid, block, lds_bytes, stream, sched, layer0);
    switch (variant) {
        GDP_FOR_EACH_VARIANT(X)
        default: return hipErrorInvalidValue;
    }
#undef X
}

hipError_t gdp_launch_relax_flow(int nsrc, int latency, const GdpDevLayer *lay, int max_L, int n_inst, int grid_blocks, int SP,
                                 int layer0, int layers, int32_t *abort_flag, int64_t spin_limit, bool debug_stall,
                                 hipStream_t stream)
{
    if (n_inst < 1 || n_inst > 65535 || layers < 1 || layers > 65535 || grid_blocks < 1) return hipErrorInvalidValue;
    const unsigned ntb = (unsigned)(SP / GDP_LAT_TS) * (unsigned)latency;  // with the parts of a split task
    dim3 grid((unsigned)grid_blocks, (unsigned)layers, (unsigned)n_inst), block(64 * GDP_WAVES_PER_BLOCK);
#define X(NSRC, K)                                                                                                   \
    if (nsrc == NSRC && latency == K) {                                                                              \
        hipLaunchKernelGGL((gdp_relax_flow_kernel<NSRC, K>), grid, block, 0, stream, lay, max_L, layer0, ntb, \
                           abort_flag, spin_limit, debug_stall ? 1 : 0);                                             \
        return hipGetLastError();                                                                                    \
    }
    GDP_FOR_EACH_FLOW(X)
#undef X
    return hipErrorInvalidValue;
}

hipError_t gdp_launch_flow_reset(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, const GdpDevLayer *lay,
                                 int max_L, int tile_rows, int32_t *abort_flag, hipStream_t stream)
{
    if (max_L < 1 || max_L > 65535 || n_inst < 1) return hipErrorInvalidValue;
    unsigned bx = (unsigned)((max_ld + 256 * 8 - 1) / (256 * 8));
    if (bx == 0) bx = 1;
    if (bx > 64u) bx = 64u;
    const int per = 65535 / max_L;  // instances per launch: grid.z holds at most 65535 (instance, layer) pairs
    for (int i0 = 0; i0 < n_inst; i0 += per) {
        const int n = n_inst - i0 < per ? n_inst - i0 : per;
        hipLaunchKernelGGL(gdp_flow_reset_kernel, dim3(bx, (unsigned)max_S, (unsigned)(n * max_L)), dim3(256), 0, stream,
                           insts + i0, lay + (int64_t)i0 * max_L, max_L, tile_rows, abort_flag);
    }
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

hipError_t gdp_launch_prepare(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, const GdpDevLayer *lay,
                              int max_L, int tile_rows, bool nan_bands, int32_t *abort_flag, hipStream_t stream)
{
    if (max_L < 1 || max_L > 65534 || n_inst < 1) return hipErrorInvalidValue;
    unsigned bx = (unsigned)((max_ld + 256 * 4 - 1) / (256 * 4));
    if (bx == 0) bx = 1;
    if (bx > 64u) bx = 64u;
    const int per = 65535 / (max_L + 1);  // instances per launch: grid.z holds at most 65535 (instance, buffer) pairs
    for (int i0 = 0; i0 < n_inst; i0 += per) {
        const int n = n_inst - i0 < per ? n_inst - i0 : per;
        hipLaunchKernelGGL(gdp_prepare_kernel, dim3(bx, (unsigned)(max_S + 1), (unsigned)(n * (max_L + 1))), dim3(256), 0,
                           stream, insts + i0, lay + (int64_t)i0 * max_L, max_L, tile_rows, nan_bands ? 1 : 0, abort_flag);
    }
    return hipGetLastError();
}

hipError_t gdp_launch_prepare_args(const GdpPrepArgs &A, hipStream_t stream)
{
    if (A.n_inst < 1 || A.n_inst > GDP_PREP_MAX_INST) return hipErrorInvalidValue;
    int64_t max_ld = 0;
    int max_S = 0, buffers = 0, layers = 0;
    for (int i = 0; i < A.n_inst; ++i) {
        if (A.inst[i].L < 1 || A.inst[i].first_layer != layers) return hipErrorInvalidValue;
        max_ld = A.inst[i].ld > max_ld ? A.inst[i].ld : max_ld;
        max_S = A.inst[i].S > max_S ? A.inst[i].S : max_S;
        buffers += A.inst[i].L + 1;
        layers += A.inst[i].L;
    }
    if (layers > GDP_PREP_MAX_LAYERS) return hipErrorInvalidValue;
    unsigned bx = (unsigned)((max_ld + 256 * 4 - 1) / (256 * 4));
    if (bx == 0) bx = 1;
    if (bx > 64u) bx = 64u;
    hipLaunchKernelGGL(gdp_prepare_args_kernel, dim3(bx, (unsigned)(max_S + 1), (unsigned)buffers), dim3(256), 0, stream, A);
    return hipGetLastError();
}

hipError_t gdp_launch_init(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, const GdpDevLayer *lay,
                           int max_L, int tile_rows, int what, hipStream_t stream)
{
    unsigned bx = (unsigned)((max_ld + 256 * 8 - 1) / (256 * 8));
    if (bx == 0) bx = 1;
    dim3 grid(bx, (unsigned)(max_S + 1), (unsigned)n_inst), block(256, 1, 1);
    if (what & ~GDP_INIT_FILL) hipLaunchKernelGGL(gdp_init_kernel, grid, block, 0, stream, insts, what & ~GDP_INIT_FILL);
    if (what & GDP_INIT_FILL) {  // after the poison, if both are asked for
        if (max_L < 1 || max_L > 65535) return hipErrorInvalidValue;
        if (bx > 64u) bx = 64u;
        const int per = 65535 / max_L;  // instances per launch: grid.z holds at most 65535 (instance, layer) pairs
        for (int i0 = 0; i0 < n_inst; i0 += per) {
            const int n = n_inst - i0 < per ? n_inst - i0 : per;
            hipLaunchKernelGGL(gdp_fill_kernel, dim3(bx, (unsigned)max_S, (unsigned)(n * max_L)), block, 0, stream,
                               insts + i0, lay + (int64_t)i0 * max_L, max_L, tile_rows);
        }
    }
    return hipGetLastError();
}

hipError_t gdp_launch_zero_pass(bool marks, const GdpDevInst *insts, const GdpDevLayer *lay, int max_L, int tile_rows,
                                int n_inst, int max_V, int layer, hipStream_t stream)
{
    if (n_inst <= 0 || max_V <= 0) return hipSuccess;
    dim3 grid((unsigned)((max_V + 255) / 256), (unsigned)n_inst), block(256);
    if (marks)
        hipLaunchKernelGGL(gdp_zero_pass_kernel<true>, grid, block, 0, stream, insts, lay, max_L, tile_rows, layer);
    else
        hipLaunchKernelGGL(gdp_zero_pass_kernel<false>, grid, block, 0, stream, insts, lay, max_L, tile_rows, layer);
    return hipGetLastError();
}

hipError_t gdp_launch_epilogue(bool marks, const GdpDevInst *insts, const GdpDevKey *keys, int n_key, GdpDevOut *out,
                               int32_t *res, hipStream_t stream)
{
    if (n_key <= 0) return hipSuccess;
    if (marks)
        hipLaunchKernelGGL(gdp_epilogue_kernel<true>, dim3((unsigned)n_key), dim3(64), 0, stream, insts, keys, out, res);
    else
        hipLaunchKernelGGL(gdp_epilogue_kernel<false>, dim3((unsigned)n_key), dim3(64), 0, stream, insts, keys, out, res);
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
