// gdp_solve_static: one DP instance solved without obtaining any memory.
//
// Every other compute entry point of the library gets device memory for its cost buffers, argmin
// table, layer records and results (hipMalloc, or an allocation kept from an earlier plan), a stream,
// events and page-locked host memory.  Some callers may do none of that: tight serving loops that must
// not touch the allocator, harnesses that forbid it.  (It is no call for a process in which a stream is
// being captured in the global capture mode: synchronous copies and null-stream launches are prohibited
// then.)  For them this entry point keeps all of its device-side working
// memory in ONE file-scope device array of GDP_STATIC_SCRATCH_BYTES, builds the device layout of the
// inputs in a fixed host array, runs on the null stream with synchronous copies, and calls no
// hipMalloc / hipFree / hipHostMalloc / stream or event creation and no host allocator.
//
// It uses the kernels of the other entry points in the layout that needs the least memory: two cost
// buffers used in turn plus the one-byte argmin table (what GDP_KEEP_MARKS selects), one launch per
// layer, every cell computed.  Results are the same bits as gdp_solve's.
//
// The array is per process and per device (every device the library's code object is loaded on holds
// its own copy at its own address) and keeps the contents of the last call; a call rewrites everything
// it reads (pads, zeros of the initial costs, tables), so nothing of an earlier call is ever read.  Calls
// take a process-wide lock for their whole duration: two of them never work in the array at once.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "gdp_host.h"
#include "gdp_kernels.h"

// Device working memory of gdp_solve_static.  In host code this name is only a handle for
// hipGetSymbolAddress; the address the kernels get is the one that call returns (scratch_of_device).
static __device__ __align__(256) unsigned char scratch[GDP_STATIC_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex g_mu;                       // one call at a time: the arrays below and `scratch` are shared
unsigned char *g_scratch_ptr[MAX_DEVICES];  // device address of `scratch` on device d, once asked for

// Host side: the device layout of the inputs is built here and uploaded in one copy; the results are
// copied back into it.
constexpr size_t STAGE_BYTES = (size_t)8 << 20;
alignas(256) unsigned char g_stage[STAGE_BYTES];

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// The address of `scratch` on the current device; asked for once per device, with that device current.
int scratch_of_device(unsigned char **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return gdp_fail_hip(e, "hipGetDevice");
    if (dev < 0 || dev >= MAX_DEVICES) return gdp_fail(GDP_E_HIP, "gdp_solve_static: device index above 63");
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return gdp_fail_hip(e, "hipGetSymbolAddress(scratch)");
        if (!p) return gdp_fail(GDP_E_HIP, "hipGetSymbolAddress(scratch) returned a null address");
        g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
    }
    *out = g_scratch_ptr[dev];
    return GDP_OK;
}

struct Layout {
    int L, V, S, T, n_key, ts, variant, SP, SU, rows, P, ntile;
    int64_t ld, ldm;
    size_t off_inst, off_keys, off_lay, off_inter, off_intra, off_index, off_roff, off_mem, off_zcols, small_bytes;
    bool has_zero;
    size_t off_out, off_res, back_bytes, off_H, off_M, total_bytes;
};

// Shapes and offsets (bytes from the start of `scratch`); the same rules as a plan laid out with
// GDP_KEEP_MARKS and one launch per layer.
void lay_out(const gdp_problem *p, Layout *y)
{
    y->L = p->L; y->V = p->V; y->S = p->S;
    y->T = p->inter_index ? p->n_inter : p->L;
    y->n_key = p->n_key;
    // register tile among those built with the argmin table (11 or 8 wide, 64 rows): least padding of S,
    // then the wider one
    const size_t sp11 = align_up((size_t)p->S, 11), sp8 = align_up((size_t)p->S, 8);
    y->ts = sp11 <= sp8 ? 11 : 8;
    y->variant = gdp_find_variant(y->ts, 1);
    y->SP = (int)(y->ts == 11 ? sp11 : sp8);
    y->SU = (int)align_up((size_t)p->S, GDP_SRC_UNROLL);
    y->rows = y->SU + GDP_SRC_PAD;
    int maxm = 1;
    y->has_zero = false;
    for (size_t k = 0; k < (size_t)p->L * p->S; ++k) {
        if (p->mem[k] < p->V) maxm = std::max(maxm, p->mem[k]);
        if (p->mem[k] == 0) y->has_zero = true;
    }
    y->P = (int)align_up((size_t)maxm, 64);
    y->ntile = (p->V + 63) / 64;
    y->ldm = (int64_t)align_up((size_t)y->ntile * 64, 256);
    y->ld = y->P + y->ldm;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t o = off;
        off = align_up(off + bytes, 256);
        return o;
    };
    y->off_inst = take(sizeof(GdpDevInst));
    y->off_keys = take(sizeof(GdpDevKey) * (size_t)std::max(y->n_key, 1));
    y->off_lay = take(sizeof(GdpDevLayer) * (size_t)y->L);
    y->off_inter = take(sizeof(double) * (size_t)y->T * y->rows * y->SP);
    y->off_intra = take(sizeof(double) * (size_t)y->L * y->SP);
    y->off_index = take(sizeof(int32_t) * (size_t)y->L);
    y->off_roff = take(sizeof(int64_t) * (size_t)(y->L + 1) * y->rows);
    y->off_mem = take(sizeof(int32_t) * (size_t)y->L * y->S);
    y->off_zcols = y->has_zero ? take(sizeof(int32_t) * (size_t)y->L * (size_t)(y->S + 1)) : 0;
    y->small_bytes = off;
    y->off_out = take(sizeof(GdpDevOut) * (size_t)std::max(y->n_key, 1));
    y->off_res = take(sizeof(int32_t) * std::max<size_t>((size_t)y->n_key * y->L, 1));
    y->back_bytes = off - y->off_out;
    y->off_H = take(sizeof(double) * 2 * (size_t)(y->S + 1) * (size_t)y->ld);
    y->off_M = take((size_t)y->L * y->S * (size_t)y->ldm);
    y->total_bytes = off;
}

// The device layout of the inputs, written into g_stage; `base` is the device address of `scratch`.
void build(const gdp_problem *p, const Layout &y, unsigned char *base)
{
    memset(g_stage, 0, y.small_bytes);
    GdpDevInst &d = *reinterpret_cast<GdpDevInst *>(g_stage + y.off_inst);
    d.H = reinterpret_cast<double *>(base + y.off_H);
    d.hstride = (int64_t)(y.S + 1) * y.ld;
    d.M = base + y.off_M;
    d.inter = reinterpret_cast<const double *>(base + y.off_inter);
    d.intra = reinterpret_cast<const double *>(base + y.off_intra);
    d.inter_index = reinterpret_cast<const int32_t *>(base + y.off_index);
    d.roff = reinterpret_cast<const int64_t *>(base + y.off_roff);
    d.mem = reinterpret_cast<const int32_t *>(base + y.off_mem);
    d.ld = y.ld; d.ldm = y.ldm;
    d.L = y.L; d.V = y.V; d.S = y.S; d.SP = y.SP; d.SU = y.SU; d.P = y.P; d.ntile = y.ntile;
    d.nbuf = 2;
    // transition matrices [T][rows][SP] and intra [L][SP], zero padded
    double *it = reinterpret_cast<double *>(g_stage + y.off_inter);
    for (int t = 0; t < y.T; ++t)
        for (int a = 0; a < y.S; ++a)
            memcpy(it + ((size_t)t * y.rows + a) * y.SP, p->inter + ((size_t)t * y.S + a) * y.S,
                   sizeof(double) * (size_t)y.S);
    double *ia = reinterpret_cast<double *>(g_stage + y.off_intra);
    for (int l = 0; l < y.L; ++l) memcpy(ia + (size_t)l * y.SP, p->intra + (size_t)l * y.S, sizeof(double) * (size_t)y.S);
    int32_t *ix = reinterpret_cast<int32_t *>(g_stage + y.off_index);
    for (int l = 0; l < y.L; ++l) ix[l] = p->inter_index ? p->inter_index[l] : l;
    memcpy(g_stage + y.off_mem, p->mem, sizeof(int32_t) * (size_t)y.L * y.S);
    d.zcols = nullptr;
    if (y.has_zero) {   // per layer: {n, the n strategies whose memory cost is 0} (see gdp_launch_zero_pass)
        d.zcols = reinterpret_cast<const int32_t *>(base + y.off_zcols);
        int32_t *z = reinterpret_cast<int32_t *>(g_stage + y.off_zcols);
        for (int l = 0; l < y.L; ++l) {
            int32_t *row = z + (size_t)l * (y.S + 1);
            row[0] = 0;
            for (int s = 0; s < y.S; ++s)
                if (p->mem[(size_t)l * y.S + s] == 0) row[++row[0]] = s;
        }
    }
    // roff[l][s']: element offset, from the base of a cost buffer, of "f after layer l-1, strategy s', row 0";
    // a strategy whose memory cost reaches V, and every padding source, reads the +inf row
    int64_t *ro = reinterpret_cast<int64_t *>(g_stage + y.off_roff);
    const int64_t inf_row = (int64_t)y.S * y.ld + y.P;
    for (int l = 0; l <= y.L; ++l) {
        int64_t *row = ro + (size_t)l * y.rows;
        for (int s = 0; s < y.S; ++s) {
            if (l == 0) {
                row[s] = (int64_t)s * y.ld + y.P;
            } else {
                const int m = p->mem[(size_t)(l - 1) * y.S + s];
                row[s] = (m >= y.V) ? inf_row : (int64_t)s * y.ld + y.P - m;
            }
        }
        for (int s = y.S; s < y.rows; ++s) row[s] = inf_row;
    }
    GdpDevLayer *lay = reinterpret_cast<GdpDevLayer *>(g_stage + y.off_lay);
    for (int l = 0; l < y.L; ++l) {
        GdpDevLayer &r = lay[l];
        int maxm = 0;
        for (int s = 0; s < y.S; ++s) {
            const int m = p->mem[(size_t)l * y.S + s];
            if (m < y.V) maxm = std::max(maxm, m);
        }
        const int mat = p->inter_index ? p->inter_index[l] : l;
        r.src = d.H + (int64_t)(l % 2) * d.hstride;
        r.dst = d.H + (int64_t)((l + 1) % 2) * d.hstride + y.P;
        r.ro = d.roff + (int64_t)l * y.rows;
        memcpy(r.ro_head, ro + (size_t)l * y.rows, sizeof(r.ro_head));
        r.it = d.inter + (int64_t)mat * y.rows * y.SP;
        r.ia = d.intra + (int64_t)l * y.SP;
        r.m = d.M + (int64_t)l * y.S * y.ldm;
        r.ld = y.ld; r.ldm = y.ldm;
        r.S = y.S; r.SU = y.SU; r.SP = y.SP; r.ntile = y.ntile;
        r.dep = (maxm + 63) / 64;
        r.lo = 0;               // every tile is computed
        r.hi = y.ntile - 1;
    }
    GdpDevKey *keys = reinterpret_cast<GdpDevKey *>(g_stage + y.off_keys);
    for (int k = 0; k < y.n_key; ++k) {
        keys[k].other_mem = p->other_mem[k];
        keys[k].other_time = p->other_time[k];
        keys[k].inst = 0;
        keys[k].res_off = k * y.L;
    }
}

}  // namespace

extern "C" int gdp_solve_static(const gdp_problem *p, gdp_result *r)
{
    gdp_clear_error();
    if (!p || !r) return gdp_fail(GDP_E_BADARG, "null problem or result");
    bool f0_live = false;
    int rc = gdp_validate(p, 0);
    if (rc == GDP_OK) rc = gdp_validate_f0(p, 0, &f0_live);
    if (rc != GDP_OK) return rc;
    if (p->flags & (GDP_EXPORT_F | GDP_EXPORT_MARK))
        return gdp_fail(GDP_E_BADARG, "gdp_solve_static does not export f / mark");
    if (p->S > GDP_MAX_S_MARKS) return gdp_fail(GDP_E_BADARG, "gdp_solve_static: S exceeds GDP_MAX_S_MARKS");
    if (p->n_key > 0 && (!r->total || !r->remaining || !r->res)) return gdp_fail(GDP_E_BADARG, "null result array");
    Layout y;
    lay_out(p, &y);
    if (y.variant < 0) return gdp_fail(GDP_E_HIP, "gdp_solve_static: register tile not built");
    if (y.total_bytes > (size_t)GDP_STATIC_SCRATCH_BYTES || y.small_bytes > STAGE_BYTES || y.back_bytes > STAGE_BYTES) {
        char buf[256];
        snprintf(buf, sizeof buf,
                 "gdp_solve_static: this instance needs %zu bytes of device working memory (tables %zu, results %zu); "
                 "the static array holds %zu (tables and results up to %zu each): use gdp_solve",
                 y.total_bytes, y.small_bytes, y.back_bytes, (size_t)GDP_STATIC_SCRATCH_BYTES, STAGE_BYTES);
        return gdp_fail(GDP_E_NOMEM, buf);
    }
    std::lock_guard<std::mutex> lk(g_mu);
    unsigned char *base = nullptr;
    const int rs = scratch_of_device(&base);
    if (rs != GDP_OK) return rs;
    build(p, y, base);
    hipStream_t stream = nullptr;  // the null stream: nothing is created
    hipError_t e = hipMemcpy(base, g_stage, y.small_bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) return gdp_fail_hip(e, "gdp_solve_static: upload");
    const GdpDevInst *d_inst = reinterpret_cast<const GdpDevInst *>(base + y.off_inst);
    const GdpDevLayer *d_lay = reinterpret_cast<const GdpDevLayer *>(base + y.off_lay);
    // +inf pads and +inf row of both cost buffers, zeros in the first one (the caller's initial f): whatever
    // the last call left there is overwritten before anything reads it
    e = gdp_launch_init(d_inst, 1, y.ld, y.S, d_lay, y.L, 64, GDP_INIT_PADS | GDP_INIT_ZERO, stream);
    if (e == hipSuccess && f0_live) {
        // The caller's initial costs [V][S] into buffer 0, one row per strategy: turned round in the host
        // array a slice of budget rows at a time (the tables it held are on the device by now; the copies
        // are synchronous and follow the launch above in stream order).
        double *stage = reinterpret_cast<double *>(g_stage);
        double *h0 = reinterpret_cast<double *>(base + y.off_H) + y.P;
        const int slice = (int)std::max<size_t>(1, STAGE_BYTES / (sizeof(double) * (size_t)y.S));
        for (int v0 = 0; v0 < y.V && e == hipSuccess; v0 += slice) {
            const int nv = std::min(slice, y.V - v0);
            for (int v = 0; v < nv; ++v)
                for (int s = 0; s < y.S; ++s) stage[(size_t)s * nv + v] = p->f0[(size_t)(v0 + v) * y.S + s];
            e = hipMemcpy2D(h0 + v0, sizeof(double) * (size_t)y.ld, stage, sizeof(double) * (size_t)nv,
                            sizeof(double) * (size_t)nv, (size_t)y.S, hipMemcpyHostToDevice);
        }
    }
    for (int l = 0; l < y.L && e == hipSuccess; ++l) {
        e = gdp_launch_relax(y.variant, true, 0, d_lay, y.L, 1, y.ntile, y.SP, l, stream);
        if (e == hipSuccess && y.has_zero) e = gdp_launch_zero_pass(true, d_inst, d_lay, y.L, 64, 1, y.V, l, stream);
    }
    if (e == hipSuccess)
        e = gdp_launch_epilogue(true, d_inst, reinterpret_cast<const GdpDevKey *>(base + y.off_keys), y.n_key,
                                reinterpret_cast<GdpDevOut *>(base + y.off_out),
                                reinterpret_cast<int32_t *>(base + y.off_res), stream);
    if (e != hipSuccess) {
        (void)hipDeviceSynchronize();
        return gdp_fail_hip(e, "gdp_solve_static: kernel launch");
    }
    e = hipMemcpy(g_stage, base + y.off_out, y.back_bytes, hipMemcpyDeviceToHost);  // after the kernels, in stream order
    if (e != hipSuccess) return gdp_fail_hip(e, "gdp_solve_static: download");
    const GdpDevOut *out = reinterpret_cast<const GdpDevOut *>(g_stage);
    const int32_t *res = reinterpret_cast<const int32_t *>(g_stage + (y.off_res - y.off_out));
    for (int k = 0; k < y.n_key; ++k) {
        r->total[k] = out[k].total;
        r->remaining[k] = out[k].remaining;
        if (out[k].feasible) memcpy(r->res + (size_t)k * y.L, res + (size_t)k * y.L, sizeof(int32_t) * (size_t)y.L);
    }
    return GDP_OK;
}
