// Host side of libgalvatron_dp_hip.so under AddressSanitizer and UndefinedBehaviorSanitizer, without a
// GPU: this program is linked with the library's own sources (host code instrumented, device code as
// usual) and drives the parts that run before anything touches the device --
//   * argument validation (every rejection of include/galvatron_dp_hip.h),
//   * the complete plan layout of gdp_plan_create, through gdp_debug_check_layout, which lays the plan
//     out for a described device and then bounds every address the kernels would form, for seeded
//     problems of many shapes, single and batched, under every layout preset of the environment,
//   * the size check of gdp_solve_static.
// The sanitizers abort on any out-of-bounds write into the host copy of the tables or undefined
// arithmetic in the offset computations.  Built and run by tests/test_sanitizers.py.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/galvatron_dp_hip.h"

namespace {

unsigned long long rng_state = 0x9E3779B97F4A7C15ULL;
unsigned long long rnd()
{
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return rng_state;
}
int rnd_int(int lo, int hi) { return lo + (int)(rnd() % (unsigned long long)(hi - lo + 1)); }
double rnd_unit() { return (double)(rnd() >> 11) / 9007199254740992.0; }

struct Case {
    std::vector<int32_t> mem, index;
    std::vector<double> intra, inter, other_time;
    std::vector<int64_t> other_mem;
    gdp_problem p;
};

// mem_hi above V gives strategies that never fit; shared: T matrices and a layer index instead of L matrices
void make(Case &c, int L, int S, int V, int mem_hi, bool shared, unsigned flags)
{
    const int T = shared ? rnd_int(1, 3) : L;
    c.mem.resize((size_t)L * S);
    c.intra.resize((size_t)L * S);
    c.inter.resize((size_t)T * S * S);
    c.index.resize((size_t)L);
    const int mem_lo = rnd_int(0, 9) == 0 ? 0 : 1;    // now and then strategies with a memory cost of 0
    for (auto &m : c.mem) m = rnd_int(mem_lo, mem_hi);
    for (auto &x : c.intra) x = rnd_unit() < 0.05 ? INFINITY : 1.0 + 19.0 * rnd_unit();
    for (auto &x : c.inter) x = 5.0 * rnd_unit();
    for (auto &x : c.index) x = rnd_int(0, T - 1);
    if (!shared && rnd_int(0, 1))   // a dense array as the reference's callers pass it: mostly copies of a few matrices
        for (int l = 1; l < L; ++l) {
            const int r = rnd_int(0, 9);
            const int from = r < 6 ? l - 1 : r < 8 ? rnd_int(0, l - 1) : l;
            if (from != l)
                memcpy(c.inter.data() + (size_t)l * S * S, c.inter.data() + (size_t)from * S * S, sizeof(double) * S * S);
        }
    c.other_mem = {0, V / 64, V / 4, (int64_t)V + 5};
    c.other_time = {0.0, 1.0, 2.0, 3.0};
    c.p = gdp_problem{L, V, S, c.mem.data(), c.intra.data(), c.inter.data(), shared ? c.index.data() : nullptr,
                      T, (int32_t)c.other_mem.size(), c.other_mem.data(), c.other_time.data(), flags};
}

int failures = 0;
void expect(int got, int want, const char *what)
{
    if (got != want) {
        fprintf(stderr, "host_check: %s: got %d (%s), expected %d\n", what, got, gdp_last_error(), want);
        ++failures;
    }
}

int layouts = 0;
void check(const std::vector<Case *> &cases, const char *what)
{
    std::vector<const gdp_problem *> ps;
    for (Case *c : cases) ps.push_back(&c->p);
    // an MI355X (256 CUs, 160 KB of LDS each) and a small part, which changes the launch choices
    expect(gdp_debug_check_layout((int32_t)ps.size(), ps.data(), 256, 160 * 1024), GDP_OK, what);
    expect(gdp_debug_check_layout((int32_t)ps.size(), ps.data(), 16, 64 * 1024), GDP_OK, what);
    layouts += 2;
}

}  // namespace

int main()
{
    static const int S_values[] = {1, 2, 7, 8, 9, 11, 15, 16, 17, 22, 31, 32, 33, 44, 63, 64, 65, 88, 127, 128, 255, 256, 257, 1024};
    static const char *presets[][2] = {
        {nullptr, nullptr},
        {"GALVATRON_DP_FUSED", "0"}, {"GALVATRON_DP_FUSED", "1"}, {"GALVATRON_DP_SKIP", "0"},
        {"GALVATRON_DP_KEEP_MARKS", "1"}, {"GALVATRON_DP_CHUNK", "2"}, {"GALVATRON_DP_TILE_R", "2"},
        {"GALVATRON_DP_TILE_TS", "8"}, {"GALVATRON_DP_TILE_TS", "11"}, {"GALVATRON_DP_TILE_TS", "16"},
        {"GALVATRON_DP_LATENCY_VARIANT", "1"}, {"GALVATRON_DP_LATENCY_VARIANT", "2"}, {"GALVATRON_DP_LATENCY_VARIANT", "4"},
        {"GALVATRON_DP_MAX_GRID_ROWS", "3"}, {"GALVATRON_DP_OCCUPANCY_CAP", "0"}};
    for (const auto &preset : presets) {
        if (preset[0]) setenv(preset[0], preset[1], 1);
        const bool marks_forced = preset[0] && !strcmp(preset[0], "GALVATRON_DP_KEEP_MARKS");
        const bool lat = preset[0] && !strcmp(preset[0], "GALVATRON_DP_LATENCY_VARIANT");
        if (lat) setenv("GALVATRON_DP_FUSED", "0", 1);
        // single instances of every strategy count, small and large tables
        for (int S : S_values) {
            if (marks_forced && S > GDP_MAX_S_MARKS) continue;
            for (int rep = 0; rep < 3; ++rep) {
                Case c;
                const int L = rnd_int(1, rep == 2 ? 40 : 6);
                const int V = rep == 0 ? rnd_int(1, 70) : rep == 1 ? rnd_int(64, 5000) : rnd_int(5000, S > 256 ? 20000 : 300000);
                make(c, L, S, V, rep == 0 ? V + 2 : V / (L + 1) + 1, rep == 1, 0);
                check({&c}, "single instance");
            }
        }
        // batches: mixed depths, widths and budgets
        for (int rep = 0; rep < 4; ++rep) {
            std::vector<Case> cs((size_t)rnd_int(2, 40));
            std::vector<Case *> ptrs;
            for (Case &c : cs) {
                static const int widths[] = {22, 44, 44, 64, 40, 88};
                const int V = rnd_int(50, rep == 3 ? 70000 : 6000);
                make(c, rnd_int(1, 32), widths[rnd_int(0, 5)], V, V / 8 + 1, rnd_int(0, 1), 0);
                ptrs.push_back(&c);
            }
            check(ptrs, "batch");
        }
        // the debug exports and the explicit launch requests
        for (unsigned flags : {GDP_EXPORT_F, GDP_EXPORT_MARK, GDP_EXPORT_F | GDP_EXPORT_MARK, GDP_LAUNCH_FUSED,
                               GDP_LAUNCH_PER_LAYER, GDP_COMPUTE_ALL, GDP_KEEP_MARKS, GDP_KEEP_MARKS | GDP_LAUNCH_PER_LAYER}) {
            Case c;
            make(c, 5, 44, 3000, 300, false, flags);
            check({&c}, "flags");
        }
        // instances that point at the same transition matrices (they read one device copy), among others that do not
        for (int shared = 0; shared < 2; ++shared) {
            std::vector<Case> cs(7);
            std::vector<Case *> ptrs;
            for (size_t k = 0; k < cs.size(); ++k) {
                make(cs[k], 6, k == 5 ? 22 : 44, 2500, 300, shared != 0, 0);
                if (k >= 1 && k <= 4 && k != 3) {
                    cs[k].p.inter = cs[0].p.inter;
                    cs[k].p.inter_index = cs[0].p.inter_index;
                    cs[k].p.n_inter = cs[0].p.n_inter;
                }
                ptrs.push_back(&cs[k]);
            }
            check(ptrs, "batch with shared matrices");
        }
        if (preset[0]) unsetenv(preset[0]);
        if (lat) unsetenv("GALVATRON_DP_FUSED");
    }

    // ---- rejections ---------------------------------------------------------------------------------
    {
        Case c;
        make(c, 3, 5, 100, 20, false, 0);
        const gdp_problem *pp[1] = {&c.p};
        gdp_plan *plan = nullptr;
        auto create = [&]() { return gdp_plan_create(1, pp, &plan); };
        c.mem[4] = -2;                 expect(create(), GDP_E_BADARG, "mem < 0");
        c.mem[4] = 3;
        c.other_mem[1] = -1;           expect(create(), GDP_E_BADARG, "other_mem < 0");
        c.other_mem[1] = 1;
        c.intra[2] = NAN;              expect(create(), GDP_E_NONFINITE, "NaN intra");
        c.intra[2] = 1.0;
        c.inter[7] = -INFINITY;        expect(create(), GDP_E_NONFINITE, "-inf inter");
        c.inter[7] = 1.0;
        c.other_time[0] = NAN;         expect(create(), GDP_E_NONFINITE, "NaN other_time");
        c.other_time[0] = 0.0;
        for (auto &x : c.intra) x = 1e300;
        expect(create(), GDP_E_NONFINITE, "overflowing costs");
        for (auto &x : c.intra) x = 1.0;
        c.p.V = GDP_MAX_V + 1;         expect(create(), GDP_E_BADARG, "V too large");
        c.p.V = 0;                     expect(create(), GDP_E_BADARG, "V == 0");
        c.p.V = 100;
        c.p.S = GDP_MAX_S + 1;         expect(create(), GDP_E_BADARG, "S too large");
        c.p.S = 5;
        c.p.mem = nullptr;             expect(create(), GDP_E_BADARG, "null mem");
        c.p.mem = c.mem.data();
        c.index = {0, 7, 0};
        c.p.inter_index = c.index.data();
        c.p.n_inter = 3;               expect(create(), GDP_E_BADARG, "inter_index out of range");
        c.p.inter_index = nullptr;
        expect(gdp_plan_create(0, pp, &plan), GDP_E_BADARG, "n == 0");
        expect(gdp_plan_create(1, nullptr, &plan), GDP_E_BADARG, "null problems");
        expect(gdp_plan_run(nullptr, 0, nullptr), GDP_E_BADARG, "null plan");
        expect(gdp_debug_check_layout(1, pp, 0, 0), GDP_E_BADARG, "no CUs");
        // the entry point without allocation: an instance beyond its fixed working memory, then bad arguments
        Case big;
        make(big, 32, 44, 65536, 4000, true, 0);
        gdp_result r = {};
        std::vector<double> total(4);
        std::vector<int32_t> remaining(4), res((size_t)4 * 32);
        r.total = total.data(); r.remaining = remaining.data(); r.res = res.data();
        expect(gdp_solve_static(&big.p, &r), GDP_E_NOMEM, "gdp_solve_static beyond its working memory");
        expect(gdp_solve_static(nullptr, &r), GDP_E_BADARG, "gdp_solve_static null problem");
        big.p.flags = GDP_EXPORT_F;
        expect(gdp_solve_static(&big.p, &r), GDP_E_BADARG, "gdp_solve_static with an export flag");
    }
    if (failures) {
        fprintf(stderr, "host_check: %d failures\n", failures);
        return 1;
    }
    printf("host_check: %d layouts audited, rejections as documented\n", layouts);
    return 0;
}
