/*
 * The C restatement of the reference's dynamic program (oracle/dp_oracle.c) under AddressSanitizer and
 * UndefinedBehaviorSanitizer: seeded problems of many shapes, the corner cases of the recurrence
 * included (one bin, one strategy, memory costs of 0 and of V and more, all-infinite columns, keys
 * whose start row lies below the table).  The sanitizers abort on any out-of-bounds access or
 * undefined arithmetic; beyond that the program checks the identities that hold along every returned
 * path.  Built and run by tests/test_sanitizers.py:
 *   gcc -O1 -g -fsanitize=address,undefined -fno-sanitize-recover=all -static-libasan oracle_check.c -lm
 */
#include <stdio.h>
#include <stdlib.h>

#include "../../oracle/dp_oracle.c"

static unsigned long long rng_state = 88172645463325252ULL;
static unsigned long long rnd(void)
{
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return rng_state;
}
static int rnd_int(int lo, int hi) { return lo + (int)(rnd() % (unsigned long long)(hi - lo + 1)); }
static double rnd_unit(void) { return (double)(rnd() >> 11) / 9007199254740992.0; }

static int one_case(int L, int S, int V, int mem_lo, int mem_hi, double inf_frac, int integer_costs)
{
    int32_t *mem = malloc(sizeof *mem * (size_t)L * S);
    double *intra = malloc(sizeof *intra * (size_t)L * S);
    double *inter = malloc(sizeof *inter * (size_t)L * S * S);
    double *f = calloc((size_t)V * S, sizeof *f);
    int32_t *mark = malloc(sizeof *mark * (size_t)L * V * S);
    enum { NK = 5 };
    int64_t other_mem[NK] = {0, V / 7, V / 2, V - 1, (int64_t)V + 3};
    double other_time[NK] = {0.0, 1.5, 0.25, 3.0, 1.0}, total[NK];
    int32_t remaining[NK], *res = malloc(sizeof *res * (size_t)NK * L);
    if (!mem || !intra || !inter || !f || !mark || !res) return 2;
    for (size_t k = 0; k < (size_t)L * S; ++k) {
        mem[k] = rnd_int(mem_lo, mem_hi);
        intra[k] = rnd_unit() < inf_frac ? INFINITY : (integer_costs ? rnd_int(1, 6) : 1.0 + 19.0 * rnd_unit());
    }
    for (size_t k = 0; k < (size_t)L * S * S; ++k) inter[k] = integer_costs ? rnd_int(0, 3) : 5.0 * rnd_unit();
    for (size_t k = 0; k < (size_t)NK * L; ++k) res[k] = -1;
    dp_oracle_solve(L, V, S, mem, intra, inter, f, mark, NULL, NK, other_mem, other_time, total, remaining, res);
    int bad = 0;
    for (int k = 0; k < NK; ++k) {
        const int32_t *path = res + (size_t)k * L;
        if (remaining[k] == -1) {                       /* infeasible: nothing written */
            bad |= !(total[k] == INFINITY);
            for (int l = 0; l < L; ++l) bad |= path[l] != -1;
            continue;
        }
        /* sum of the memory along the path + what is left = start row; the path's cost, summed in the
           recurrence's order, + other_time = the reported total (csrc/dp_core.cpp:99-115) */
        int64_t used = 0;
        double cost = 0.0;
        for (int l = 0; l < L; ++l) {
            bad |= path[l] < 0 || path[l] >= S;
            if (bad) break;
            used += mem[(size_t)l * S + path[l]];
            const int from = l ? path[l - 1] : 0;
            /* layer 0 starts from f = 0 whatever the source strategy; its best source is its argmin */
            if (l == 0) {
                double best = INFINITY;
                for (int si = 0; si < S; ++si) {
                    const double c = (0.0 + inter[(size_t)si * S + path[0]]) + intra[path[0]];
                    if (c < best) best = c;
                }
                cost = best;
            } else {
                cost = (cost + inter[((size_t)l * S + from) * S + path[l]]) + intra[(size_t)l * S + path[l]];
            }
        }
        bad |= used + remaining[k] != (int64_t)V - 1 - other_mem[k];
        bad |= remaining[k] < 0;
        if (mem_lo >= 1) bad |= !(cost + other_time[k] == total[k]);   /* (with mem == 0 a cell may take a same-layer source) */
    }
    free(mem); free(intra); free(inter); free(f); free(mark); free(res);
    return bad;
}

int main(void)
{
    int cases = 0;
    static const int shapes[][3] = {{1, 1, 1}, {1, 1, 2}, {2, 1, 5}, {3, 2, 1}, {4, 3, 17}, {5, 7, 64}, {6, 22, 300},
                                    {3, 44, 129}, {2, 64, 65}, {2, 65, 40}, {7, 5, 1000}, {12, 4, 257}};
    for (size_t i = 0; i < sizeof shapes / sizeof shapes[0]; ++i)
        for (int rep = 0; rep < 6; ++rep) {
            const int L = shapes[i][0], S = shapes[i][1], V = shapes[i][2];
            const int hi = rep == 0 ? 1 : rep == 1 ? V + 2 : rep == 2 ? V / 2 + 1 : V / (L + 1) + 1;
            const int lo = rep == 5 ? 0 : 1;            /* memory costs of 0: the in-place update reads its own row */
            if (one_case(L, S, V, lo, hi, rep == 3 ? 0.3 : 0.05, rep & 1)) {
                fprintf(stderr, "oracle_check: identity violated for L=%d S=%d V=%d rep=%d\n", L, S, V, rep);
                return 1;
            }
            ++cases;
        }
    /* coarse branch */
    {
        enum { L = 4, S = 3, V = 50 };
        int32_t mem[L * S], tp[S] = {1, 2, 1}, res[L], remaining;
        double intra[L * S], inter[L * S * S], total;
        for (int k = 0; k < L * S; ++k) { mem[k] = 1 + k % 5; intra[k] = 1.0 + k; }
        for (int k = 0; k < L * S * S; ++k) inter[k] = 0.5 * (k % 7);
        for (int key = 1; key <= 4; ++key) {
            for (int l = 0; l < L; ++l) res[l] = -1;
            dp_oracle_coarse(L, V, S, mem, intra, inter, tp, key, 3, 0.5, &total, &remaining, res);
            ++cases;
        }
    }
    printf("oracle_check: %d cases clean\n", cases);
    return 0;
}
