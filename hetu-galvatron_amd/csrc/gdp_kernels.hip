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

template <int TS, int R>
__global__ __launch_bounds__(64 * GDP_WAVES_PER_BLOCK) void gdp_relax_kernel(
    const GdpDevInst *__restrict__ insts, int layer, unsigned ntb, unsigned nblk_x)
{
    const GdpDevInst *I = insts + blockIdx.y;
    const int L = uload(&I->L);
    if (layer >= L) return;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned lane = threadIdx.x & 63u;
    const unsigned task = xcd_swizzle(blockIdx.x, nblk_x) * GDP_WAVES_PER_BLOCK + wave;
    const unsigned tile = task / ntb;
    const unsigned tb = task - tile * ntb;
    if (tile >= (unsigned)uload(&I->ntile)) return;

    const int S = uload(&I->S);
    const int SP = uload(&I->SP);
    const int P = uload(&I->P);
    const int64_t ld = uload(&I->ld);
    const int64_t ldm = uload(&I->ldm);
    const double *src = uload(&I->H[layer & 1]);
    double *dst = uload(&I->H[(layer + 1) & 1]);
    uint8_t *M = uload(&I->M);
    const int64_t *ro = uload(&I->roff) + (int64_t)layer * (S + 1);
    const int s0 = tb * TS;
    const int mat = uload(uload(&I->inter_index) + layer);
    const double *it = uload(&I->inter) + (int64_t)mat * (S + 1) * SP + s0;
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

    double fp[R], sc[TS];
    {
        const double *p = src + uload(ro) + u0;
#pragma unroll
        for (int r = 0; r < R; ++r) fp[r] = p[lane + 64u * r];
#pragma unroll
        for (int j = 0; j < TS; ++j) sc[j] = uload(it + j);
    }

    for (int sp = 0; sp < S; ++sp) {
        // prefetch the next source strategy (row S of roff / inter is a valid dummy)
        double fpn[R], scn[TS];
        const double *pn = src + uload(ro + sp + 1) + u0;
#pragma unroll
        for (int r = 0; r < R; ++r) fpn[r] = pn[lane + 64u * r];
#pragma unroll
        for (int j = 0; j < TS; ++j) scn[j] = uload(it + (int64_t)(sp + 1) * SP + j);

#pragma unroll
        for (int j = 0; j < TS; ++j)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const double c = (fp[r] + sc[j]) + add[j];
                const bool lt = c < best[r][j];
                best[r][j] = min_f64(best[r][j], c);
                arg[r][j] = lt ? sp : arg[r][j];
            }
#pragma unroll
        for (int r = 0; r < R; ++r) fp[r] = fpn[r];
#pragma unroll
        for (int j = 0; j < TS; ++j) sc[j] = scn[j];
    }

#pragma unroll
    for (int j = 0; j < TS; ++j) {
        const int s = s0 + j;
        if (s < S) {
            double *drow = dst + (int64_t)s * ld + P + u0;
            uint8_t *mrow = M + ((int64_t)layer * S + s) * ldm + u0;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                drow[lane + 64u * r] = best[r][j];
                mrow[lane + 64u * r] = (uint8_t)arg[r][j];
            }
        }
    }
}

// +inf pads / +inf row in both buffers, zeros in the data region of buffer 0
// (the caller's f is all zeros on entry: dynamic_programming.py:16).
__global__ __launch_bounds__(256) void gdp_init_kernel(const GdpDevInst *__restrict__ insts)
{
    const GdpDevInst *I = insts + blockIdx.z;
    const int S = uload(&I->S);
    const int row = blockIdx.y;
    if (row > S) return;
    const int64_t ld = uload(&I->ld);
    const int P = uload(&I->P);
    double *h0 = uload(&I->H[0]) + (int64_t)row * ld;
    double *h1 = uload(&I->H[1]) + (int64_t)row * ld;
    const double inf = INFINITY;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < ld; i += (int64_t)gridDim.x * blockDim.x) {
        const bool pad = (row == S) || (i < P);
        h0[i] = pad ? inf : 0.0;
        if (pad) h1[i] = inf;
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
    const double *fin = uload(&I->H[L & 1]);  // layer l writes buffer (l+1)&1
    const int64_t *ro = uload(&I->roff) + (int64_t)L * (S + 1);
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
        idx = M[((int64_t)i * S + cur) * ldm + v];
        path[i - 1] = idx;
    }
    o.remaining = (int32_t)(v - mem[idx]);  // csrc/dp_core.cpp:115
    o.feasible = 1;
    out[blockIdx.x] = o;
}

// f of the last layer in the reference's [V][S] layout.
__global__ __launch_bounds__(256) void gdp_export_f_kernel(const GdpDevInst *__restrict__ I, double *__restrict__ f)
{
    const int L = I->L, V = I->V, S = I->S;
    const double *fin = I->H[L & 1];
    const int64_t *ro = I->roff + (int64_t)L * (S + 1);
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

hipError_t gdp_launch_relax(const GdpDevInst *insts, int n_inst, int max_ntile, int SP, int layer,
                            hipStream_t stream)
{
    const unsigned ntb = (unsigned)(SP / GDP_TS);
    const unsigned tasks = (unsigned)max_ntile * ntb;
    unsigned nblk = (tasks + GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK;
    nblk = (nblk + 7u) & ~7u;
    dim3 grid(nblk, (unsigned)n_inst, 1), block(64 * GDP_WAVES_PER_BLOCK, 1, 1);
    hipLaunchKernelGGL((gdp_relax_kernel<GDP_TS, GDP_R>), grid, block, 0, stream, insts, layer, ntb, nblk);
    return hipGetLastError();
}

hipError_t gdp_launch_init(const GdpDevInst *insts, int n_inst, int64_t max_ld, int max_S, hipStream_t stream)
{
    unsigned bx = (unsigned)((max_ld + 256 * 8 - 1) / (256 * 8));
    if (bx == 0) bx = 1;
    dim3 grid(bx, (unsigned)(max_S + 1), (unsigned)n_inst), block(256, 1, 1);
    hipLaunchKernelGGL(gdp_init_kernel, grid, block, 0, stream, insts);
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
