/*
 * dp_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Plain-C, single-threaded CPU restatement of the reference's layer-wise
 * dynamic program, csrc/dp_core.cpp:24-120 (`dynamic_programming_core`).
 * It exists only as the checker for the HIP path (tests, the smoke check and
 * the bench's cpu_baseline leg).  The shipped library never links, loads or
 * calls anything in this file, and has no CPU fallback.
 *
 * Parity status of each function (what pins it):
 *   dp_oracle_relax     (csrc/dp_core.cpp:57-76)  pinned: hand-derived known
 *       answer, brute-force path enumeration on tiny inputs, closed forms
 *       (S=1, budget too small), and bit-for-bit comparison of f, mark and
 *       results against the reference's own translation unit compiled into
 *       oracle/_ref/ (tests/test_oracle_*.py).
 *   dp_oracle_epilogue  (csrc/dp_core.cpp:78-117) pinned: same tests, plus
 *       the memory/cost identities along the returned path.
 *   dp_oracle_coarse    (galvatron/core/search_engine/dynamic_programming.py:62-75)
 *       pinned: on every coarse instance of the two coarse-mode scenarios whose
 *       results were recorded from the reference's own DpOnModel
 *       (tests/golden/dp_on_model_golden.json) it must give what the host
 *       class gives, and the run as a whole the recorded tuples
 *       (tests/test_oracle_pins.py::test_coarse_branch_against_the_reference_scenarios).
 *
 * Semantics restated (all from csrc/dp_core.cpp unless noted):
 *   - one f[V][S] buffer updated in place, v descending, s ascending (:57-59);
 *   - cell with v < mem[l][s]: f = +inf, mark = -1 (:60-64);
 *   - candidate si: (f[v-mem][si] + inter[l][si][s]) + intra[l][s], evaluated
 *     left to right in binary64 (:67);
 *   - argmin = first minimum under strict '<' (std::min_element, :12-16,70);
 *   - epilogue per key, ascending key order (std::map iteration, :78-117).
 * The reference allocates a candidates vector per cell and scans it twice;
 * here the running minimum is kept in the same scan.  The comparison sequence
 * (ascending si, replace only on strict <) is unchanged, so results are
 * bit-identical.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#define DP_ORACLE_ABI 1

int dp_oracle_abi(void) { return DP_ORACLE_ABI; }

/* Layer loop, csrc/dp_core.cpp:57-76.
 * mem   int32 [L][S]        (v_data)
 * intra f64   [L][S]
 * inter f64   [L][S][S]     row = source strategy si, column = target s
 * f     f64   [V][S]        in: initial values (callers pass zeros), out: last layer
 * mark  int32 [L][V][S]     may be NULL (not recorded); mark8 likewise as int8
 */
void dp_oracle_relax(int L, int V, int S, const int32_t *mem,
                     const double *intra, const double *inter, double *f,
                     int32_t *mark, int8_t *mark8)
{
    for (int i = 0; i < L; ++i) {
        const int32_t *mem_i = mem + (size_t)i * S;
        const double *intra_i = intra + (size_t)i * S;
        const double *inter_i = inter + (size_t)i * S * S;
        for (int v = V - 1; v >= 0; --v) {
            for (int s = 0; s < S; ++s) {
                size_t cell = ((size_t)i * V + v) * S + s;
                if (v < mem_i[s]) {
                    if (mark) mark[cell] = -1;
                    if (mark8) mark8[cell] = -1;
                    f[(size_t)v * S + s] = INFINITY;
                    continue;
                }
                const double *src = f + (size_t)(v - mem_i[s]) * S;
                double add = intra_i[s];
                double best = (src[0] + inter_i[s]) + add;
                int arg = 0;
                for (int si = 1; si < S; ++si) {
                    double c = (src[si] + inter_i[(size_t)si * S + s]) + add;
                    if (c < best) { best = c; arg = si; }
                }
                if (mark) mark[cell] = arg;
                if (mark8) mark8[cell] = (int8_t)arg;
                f[(size_t)v * S + s] = best;
            }
        }
    }
}

/* Epilogue for ONE key, csrc/dp_core.cpp:80-116.  Callers iterate keys in
 * ascending order.  res[L] is written only when the key is feasible (the
 * reference leaves the caller's -1 fill in place otherwise).
 * Exactly one of mark / mark8 must be non-NULL when L > 1.
 *
 * With memory costs of 0 the reference's walk can leave the table: such a
 * cell took candidates from its OWN layer (the update is in place), the walk
 * back does not know that, follows the argmin as if it pointed into the layer
 * before, and can arrive at a negative row, which the reference then uses in
 * its flat index `mark[i*V*S + v*S + cur]` (:110) -- an element of an earlier
 * layer's rows, or memory in front of the array: undefined behaviour.  This
 * restatement forms the same flat index while it stays inside the array (so
 * that it gives what the reference's build gives there) and stops where it
 * would not; dp_oracle_walk_leaves_table() says whether a key is such a case. */
void dp_oracle_epilogue(int L, int V, int S, const int32_t *mem,
                        const double *f, const int32_t *mark,
                        const int8_t *mark8, int64_t other_mem,
                        double other_time, double *total, int32_t *remaining,
                        int32_t *res)
{
    int64_t v0 = (int64_t)V - 1 - other_mem;
    if (v0 < 0) { *total = INFINITY; *remaining = -1; return; }
    const double *row = f + (size_t)v0 * S;
    int idx = 0;
    for (int s = 1; s < S; ++s) if (row[s] < row[idx]) idx = s;
    double t = row[idx];
    if (!(t < INFINITY)) { *total = INFINITY; *remaining = -1; return; }
    *total = t + other_time;
    int v = (int)v0;
    res[L - 1] = idx;
    for (int i = L - 1; i > 0; --i) {
        int cur = idx;
        int64_t row = (int64_t)i * V + v;           /* v may be negative here: see above */
        if (row < 0) { *remaining = INT32_MIN; return; }
        size_t cell = (size_t)row * S + idx;
        idx = mark ? mark[cell] : (int)mark8[cell];
        if (idx < 0 || idx >= S) { *remaining = INT32_MIN; return; }   /* a -1 read from an earlier layer's rows */
        v -= mem[(size_t)i * S + cur];
        res[i - 1] = idx;
    }
    *remaining = v - mem[idx];
}

/* 1 when the reference's walk back for this key indexes mark with a negative
 * row (undefined behaviour in the reference, see above), else 0. */
int dp_oracle_walk_leaves_table(int L, int V, int S, const int32_t *mem,
                                const double *f, const int32_t *mark,
                                const int8_t *mark8, int64_t other_mem)
{
    int64_t v0 = (int64_t)V - 1 - other_mem;
    if (v0 < 0) return 0;
    const double *row = f + (size_t)v0 * S;
    int idx = 0;
    for (int s = 1; s < S; ++s) if (row[s] < row[idx]) idx = s;
    if (!(row[idx] < INFINITY)) return 0;
    int64_t v = v0;
    for (int i = L - 1; i > 0; --i) {
        if (v < 0) return 1;
        int cur = idx;
        size_t cell = ((size_t)i * V + (size_t)v) * S + idx;
        idx = mark ? mark[cell] : (int)mark8[cell];
        if (idx < 0 || idx >= S) return 1;
        v -= mem[(size_t)i * S + cur];
    }
    return 0;
}

/* Whole call: layer loop + epilogue for n_key keys (already ascending). */
void dp_oracle_solve(int L, int V, int S, const int32_t *mem,
                     const double *intra, const double *inter, double *f,
                     int32_t *mark, int8_t *mark8, int n_key,
                     const int64_t *other_mem, const double *other_time,
                     double *total, int32_t *remaining, int32_t *res)
{
    dp_oracle_relax(L, V, S, mem, intra, inter, f, mark, mark8);
    for (int k = 0; k < n_key; ++k)
        dp_oracle_epilogue(L, V, S, mem, f, mark, mark8, other_mem[k],
                           other_time[k], total + k, remaining + k,
                           res + (size_t)k * L);
}

/* Coarse branch, dynamic_programming.py:62-75: one strategy for every layer.
 * strategy_tp[i] is strategy_set[i][1]; key_id is the key being filled.
 * Python's sum() adds left to right starting from int 0, which is exact for
 * the first term, so a 0.0 start is the same value. */
void dp_oracle_coarse(int L, int V, int S, const int32_t *mem,
                      const double *intra, const double *inter,
                      const int32_t *strategy_tp, int key_id,
                      int64_t other_mem, double other_time, double *total,
                      int32_t *remaining, int32_t *res)
{
    *total = INFINITY;
    *remaining = -1;
    for (int i = 0; i < S; ++i) {
        if (strategy_tp[i] != key_id) continue;
        double a = 0.0, b = 0.0;
        int64_t m = 0;
        for (int l = 0; l < L; ++l) a += intra[(size_t)l * S + i];
        for (int l = 0; l < L; ++l) b += inter[((size_t)l * S + i) * S + i];
        for (int l = 0; l < L; ++l) m += mem[(size_t)l * S + i];
        double t = (a + b) + other_time;
        m += other_mem;
        if ((int64_t)V - 1 - m >= 0 && *total > t) {
            *remaining = (int32_t)((int64_t)V - 1 - m);
            *total = t;
            for (int l = 0; l < L; ++l) res[l] = i;
        }
    }
}
