// gfx950 (CDNA4, wave64) kernels of the reuse-aware neighbour aggregation and their launchers.
//
// One kernel template does all the summing.  A *task* gathers a list of rows and writes their
// weighted sum to one output row:
//     out[task_out[t], :] = scale[t] * sum_i w[i] * row(col[i])        i in task_ptr[t] .. task_ptr[t+1]
// where row(c) is x[c, :] for c < nsplit and the partial-sum row part[c - nsplit, :] otherwise
// (the first task_nref[t] entries of a task are of the second kind).  Up to three launches in stream
// order: reuse groups that several destinations share -> partial-sum rows; segments of very long rows
// (which may read group rows) -> partial-sum rows; every destination row -> out.  There are no
// atomics: each output row has one writer.
//
// Mapping to the machine:
//   * the feature dimension runs across lanes, VEC consecutive elements per lane (one 16-byte
//     load), LPR lanes per row, so a wavefront gathers G = 64/LPR rows per load instruction and a
//     row is read as one contiguous 16*LPR-byte burst;
//   * long tasks get a whole wavefront: its G lane groups take every G-th entry and are combined
//     at the end by a cross-lane butterfly (__shfl_xor -> DPP / ds_swizzle class instructions);
//   * short tasks are packed G to a wavefront, one lane group each; they are pre-sorted by length
//     so the groups of one wavefront finish together;
//   * column ids and weights are fetched coalesced, one per lane, and handed to the lane groups
//     with ds_bpermute, so the only per-entry memory instruction is the row gather itself;
//   * workgroups are renumbered so that each XCD (own L2) works on runs of consecutive tasks.
// MFMA is not used: there is no dense contraction here, only gather + add, bounded by HBM.
//
// Reference semantics: ROF/reuse_conv/reuse_conv_kernel.cu:205-286 (GNNA), 396-601 (v1),
// 836-954 (v2 fused), 123-196 (SAG).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <new>

#include "rof.h"
#include "rof_internal.h"

namespace {

thread_local char g_dev_err[256] = "";

// process-wide launch tuning (rof_set_xcd_run, rof_set_lds_pad)
int g_xcd_run_a = 1, g_xcd_run_b = 16;
int g_lds_pad = 0;   // bytes of unused LDS requested per workgroup: caps the workgroups resident per CU

#define HIP_TRY(expr)                                                                  \
    do {                                                                               \
        hipError_t e_ = (expr);                                                        \
        if (e_ != hipSuccess) {                                                        \
            rof_set_device_error(#expr, hipGetErrorString(e_));                        \
            return ROF_ERR_DEVICE;                                                     \
        }                                                                              \
    } while (0)

struct AggArgs {
    const void *x;         // feature rows
    int64_t ldx;
    const float *part;     // partial-sum rows (ids >= nsplit)
    int64_t ldp;
    int32_t nsplit;
    const int32_t *task_ptr, *task_nref, *task_out;
    const float *task_scale;   // null: no scaling
    const int32_t *col;
    const float *w;            // null: unweighted
    float *out;
    int64_t ldo;
    int32_t feat;
    int32_t n_wave, n_tasks;
    int32_t n_blocks;          // logical workgroups
    int32_t xcd_run;           // consecutive logical workgroups kept on one XCD
    int32_t vec_store;         // output rows allow aligned 16-byte stores
};

// Row gathers a lane group keeps in flight.  Measured on MI355X with all eight wave slots per SIMD
// occupied: 2 beats 4 by ~10 % on the miss-dominated workloads (more outstanding gathers per CU slow the
// L1/L2 miss path down) and loses ~2 % where gathers hit in L2; 8 loses everywhere.
#ifndef ROF_UNROLL
#define ROF_UNROLL 2
#endif
#ifndef ROF_MIN_BLOCKS
#define ROF_MIN_BLOCKS 1
#endif
constexpr int kWavesPerBlock = 4;
constexpr int kXcds = 8;

template <typename XT, int VEC>
struct RowLoad;

#ifdef ROF_NT_LOADS
#define ROF_LD16(T, p) __builtin_nontemporal_load(reinterpret_cast<const T *>(p))
#else
#define ROF_LD16(T, p) (*reinterpret_cast<const T *>(p))
#endif
// 16-byte vectors that only promise 4-byte alignment: gfx950 executes global_load_dwordx4 at any dword
// address, so packed rows (e.g. 47 floats = 188 bytes) are gathered with the same instruction as padded ones
typedef float rof_f4 __attribute__((ext_vector_type(4), aligned(4)));
typedef unsigned int rof_u4 __attribute__((ext_vector_type(4), aligned(4)));

template <>
struct RowLoad<float, 4> {
    static __device__ __forceinline__ void load(const float *p, float (&v)[4]) {
        rof_f4 t = ROF_LD16(rof_f4, p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
};
template <>
struct RowLoad<float, 8> {
    static __device__ __forceinline__ void load(const float *p, float (&v)[8]) {
        rof_f4 t = ROF_LD16(rof_f4, p);
        rof_f4 u = ROF_LD16(rof_f4, p + 4);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        v[4] = u.x; v[5] = u.y; v[6] = u.z; v[7] = u.w;
    }
};
template <>
struct RowLoad<float, 1> {
    static __device__ __forceinline__ void load(const float *p, float (&v)[1]) { v[0] = *p; }
};
// bf16 is the upper half of an fp32
template <>
struct RowLoad<uint16_t, 8> {
    static __device__ __forceinline__ void load(const uint16_t *p, float (&v)[8]) {
        rof_u4 t = ROF_LD16(rof_u4, p);
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
        v[4] = __uint_as_float(t.z << 16); v[5] = __uint_as_float(t.z & 0xffff0000u);
        v[6] = __uint_as_float(t.w << 16); v[7] = __uint_as_float(t.w & 0xffff0000u);
    }
};
template <>
struct RowLoad<uint16_t, 1> {
    static __device__ __forceinline__ void load(const uint16_t *p, float (&v)[1]) {
        v[0] = __uint_as_float(((uint32_t)*p) << 16);
    }
};

// Address of this lane's slice of gathered row `c`.  xb / pb already include the lane's column
// offset; ld in bytes.  With DUAL ids >= nsplit name partial-sum rows (pb), chosen by selects, not
// branches.  OFF32: all byte offsets fit 32 bits and row ids fit 24 (checked on the host), so one
// 24-bit multiply and a 32-bit add replace the 64-bit multiply.
template <bool DUAL, bool OFF32>
__device__ __forceinline__ const char *row_ptr(int32_t c, const char *xb, uint32_t xld, const char *pb, uint32_t pld,
                                               int32_t nsplit, int32_t bias) {
    uint32_t r = (uint32_t)(c - bias), l = xld;
    const char *b = xb;
    if (DUAL) {
        const bool p = c >= nsplit;
        r = p ? (uint32_t)(c - nsplit) : r;
        l = p ? pld : xld;
        b = p ? pb : xb;
    }
    if (OFF32) return b + __umul24(r, l);
    return b + (uint64_t)r * l;
}

// Sum the entries [beg, end) of one task into acc.  WAVE: all lane groups of the wavefront share
// the task (beg/end wave-uniform) and take every G-th entry; otherwise each lane group owns its
// task.  ST is the element type of the source rows.  Blocks of U entries that are complete for every
// lane group run without any per-entry predicate; ragged ends are predicated entry by entry.
template <typename ST, int VEC, int LPR, bool WAVE, bool DUAL, bool OFF32>
__device__ __forceinline__ void gather_sum(const char *xb, uint32_t xld, const char *pb, uint32_t pld, int32_t nsplit,
                                           int32_t bias, const int32_t *__restrict__ col,
                                           const float *__restrict__ w, int32_t beg, int32_t end, int lane, int sub,
                                           int li, bool act, float (&acc)[VEC]) {
    constexpr int G = 64 / LPR;
    constexpr int U = LPR >= ROF_UNROLL ? ROF_UNROLL : LPR;   // row gathers in flight per lane group
    constexpr int CH = WAVE ? 64 : LPR;     // entries fetched per step by the wave / by the lane group
    for (int32_t base = beg; __any(base < end); base += CH) {
        const int32_t mine = base + (WAVE ? lane : li);
        int32_t mycol = bias;               // past the end: row 0 of the source, weight 0
        float myw = 0.0f;
        if (mine < end) {
            mycol = col[mine];
            myw = w ? w[mine] : 1.0f;
        }
#pragma unroll
        for (int j0 = 0; j0 < LPR; j0 += U) {
            const int first = WAVE ? j0 * G + sub : j0;
            if (!__any(base + first < end)) break;
            int32_t c[U];
            float wt[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int slot = WAVE ? (j0 + u) * G + sub : (j0 + u);          // entry of the chunk
                const int from = WAVE ? slot : sub * LPR + slot;                // lane that fetched it
                c[u] = __shfl(mycol, from);
                wt[u] = __shfl(myw, from);
            }
            const int last = WAVE ? (j0 + U - 1) * G + sub : (j0 + U - 1);
            const bool full = __all(base + last < end);
            if (act) {
                float v[U][VEC];
                if (full) {
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        RowLoad<ST, VEC>::load(
                            reinterpret_cast<const ST *>(row_ptr<DUAL, OFF32>(c[u], xb, xld, pb, pld, nsplit, bias)),
                            v[u]);
#pragma unroll
                    for (int u = 0; u < U; ++u)
#pragma unroll
                        for (int k = 0; k < VEC; ++k) acc[k] = fmaf(wt[u], v[u][k], acc[k]);
                } else {
                    // ragged end of a task: gather only the entries that exist (a dummy gather of one
                    // fixed row from every lane group would pile onto a single L2 channel)
                    bool ok[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int slot = WAVE ? (j0 + u) * G + sub : (j0 + u);
                        ok[u] = base + slot < end;
                        if (ok[u])
                            RowLoad<ST, VEC>::load(reinterpret_cast<const ST *>(
                                                       row_ptr<DUAL, OFF32>(c[u], xb, xld, pb, pld, nsplit, bias)),
                                                   v[u]);
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (ok[u]) {
#pragma unroll
                            for (int k = 0; k < VEC; ++k) acc[k] = fmaf(wt[u], v[u][k], acc[k]);
                        }
                }
            }
        }
    }
}

// PHASE 0: the partial-sum launches (no scaling); PHASE 1: the destination-row launch.  Same code; the
// parameter only gives them distinct kernel names in profiles.
template <typename XT, int VEC, int LPR, int PHASE, bool OFF32>
__global__ __launch_bounds__(256, ROF_MIN_BLOCKS) void rof_rows_kernel(AggArgs a) {
    constexpr int G = 64 / LPR;
    // XCD-aware renumbering: the hardware deals workgroup ids round-robin to the 8 XCDs; give each
    // XCD runs of `xcd_run` consecutive logical workgroups instead of every 8th one.
    const int hw = blockIdx.x;
    const int xcd = hw % kXcds, nth = hw / kXcds;
    const int run = a.xcd_run;
    const int logical = ((nth / run) * kXcds + xcd) * run + (nth % run);
    if (logical >= a.n_blocks) return;

    const int lane = threadIdx.x & 63;
    const int sub = lane / LPR, li = lane % LPR;
    const int gw = logical * kWavesPerBlock + (threadIdx.x >> 6);

    int32_t t, beg = 0, end = 0, mid = 0;
    bool valid;
    const bool wave_mode = gw < a.n_wave;
    if (wave_mode) {
        t = gw;
        valid = true;
    } else {
        t = a.n_wave + (gw - a.n_wave) * G + sub;
        valid = t < a.n_tasks;
    }
    if (valid) {
        beg = a.task_ptr[t];
        end = a.task_ptr[t + 1];
        mid = beg + a.task_nref[t];
    }
    const uint32_t xld = (uint32_t)(a.ldx * (int64_t)sizeof(XT)), pld = (uint32_t)(a.ldp * 4);

    for (int c0 = 0; c0 < a.feat; c0 += LPR * VEC) {
        const int cbase = c0 + li * VEC;
        const bool act = cbase < a.feat;
        // The lane that would run past the end of the row starts VEC elements before the end instead
        // (its first `skip` elements repeat its neighbour's and are not stored), so no load ever leaves
        // the row and rows need no padding.  The host guarantees feat >= VEC.
        const int cstart = (VEC > 1 && cbase + VEC > a.feat) ? a.feat - VEC : cbase;
        const int skip = cbase - cstart;
        const char *xb = reinterpret_cast<const char *>(a.x) + (size_t)cstart * sizeof(XT);
        const char *pb = reinterpret_cast<const char *>(a.part) + (size_t)cstart * 4;
        float acc[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;

        constexpr bool kF32 = sizeof(XT) == 4;   // fp32 features: partial rows have the same element type
        if (wave_mode) {
            if (kF32) {
                gather_sum<XT, VEC, LPR, true, true, OFF32>(xb, xld, pb, pld, a.nsplit, 0, a.col, a.w, beg, end, lane,
                                                            sub, li, act, acc);
            } else {
                if (mid > beg)
                    gather_sum<float, VEC, LPR, true, false, OFF32>(pb, pld, nullptr, 0, 0, a.nsplit, a.col, a.w, beg,
                                                                    mid, lane, sub, li, act, acc);
                gather_sum<XT, VEC, LPR, true, false, OFF32>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, mid, end, lane, sub,
                                                             li, act, acc);
            }
#pragma unroll
            for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] += __shfl_xor(acc[k], off);
            }
        } else {
            if (kF32) {
                gather_sum<XT, VEC, LPR, false, true, OFF32>(xb, xld, pb, pld, a.nsplit, 0, a.col, a.w, beg, end, lane,
                                                             sub, li, act, acc);
            } else {
                if (__any(mid > beg))
                    gather_sum<float, VEC, LPR, false, false, OFF32>(pb, pld, nullptr, 0, 0, a.nsplit, a.col, a.w, beg,
                                                                     mid, lane, sub, li, act, acc);
                gather_sum<XT, VEC, LPR, false, false, OFF32>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, mid, end, lane, sub,
                                                              li, act, acc);
            }
        }

        const bool writer = valid && act && (!wave_mode || sub == 0);
        if (writer) {
            // an empty task writes zeros whatever its scale is (a node without in-edges keeps the
            // zero-initialised output upstream: reuse_conv_kernel.cu:303)
            float s = 1.0f;
            if (a.task_scale && end > beg) s = a.task_scale[t];
            float *o = a.out + (int64_t)a.task_out[t] * a.ldo + cstart;
            if (VEC >= 4 && a.vec_store && skip == 0) {
#pragma unroll
                for (int k = 0; k < VEC; k += 4)
                    *reinterpret_cast<float4 *>(o + k) =
                        make_float4(acc[k] * s, acc[k + 1] * s, acc[k + 2] * s, acc[k + 3] * s);
            } else {
#pragma unroll
                for (int k = 0; k < VEC; ++k)
                    if (k >= skip && cstart + k < a.feat) o[k] = acc[k] * s;
            }
        }
    }
}

// rsqrt of the in-degree, correctly rounded like __frsqrt_rn (reuse_conv_kernel.cu:254,276)
__device__ __forceinline__ float rsqrt_rn(float d) { return (float)(1.0 / sqrt((double)d)); }

__global__ void rof_entry_weights_kernel(const int32_t *__restrict__ col, int64_t m, const float *__restrict__ deg,
                                         int32_t nsplit, float *__restrict__ w) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < m) {
        int32_t c = col[i];
        w[i] = c < nsplit ? rsqrt_rn(deg[c]) : 1.0f;
    }
}

__global__ void rof_task_scale_kernel(const int32_t *__restrict__ task_out, int32_t T, const float *__restrict__ deg,
                                      float *__restrict__ scale) {
    int32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < T) scale[i] = rsqrt_rn(deg[task_out[i]]);
}

// plain streaming copy, used only to calibrate profiler byte counters against a known size
__global__ void rof_copy_kernel(const float4 *__restrict__ src, float4 *__restrict__ dst, int64_t n16) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

template <typename XT, int VEC, int PHASE, bool OFF32>
int launch_lpr(const AggArgs &a0, int lpr, hipStream_t st) {
    AggArgs a = a0;
    const int g = 64 / lpr;
    const int64_t shorts = (int64_t)a.n_tasks - a.n_wave;
    const int64_t waves = a.n_wave + (shorts + g - 1) / g;
    if (waves == 0) return ROF_OK;
    a.n_blocks = (int32_t)((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    const int64_t span = (int64_t)kXcds * a.xcd_run;
    const int64_t grid = (a.n_blocks + span - 1) / span * span;
    dim3 gr((unsigned)grid), bl(64 * kWavesPerBlock);
    switch (lpr) {
        case 4: hipLaunchKernelGGL((rof_rows_kernel<XT, VEC, 4, PHASE, OFF32>), gr, bl, g_lds_pad, st, a); break;
        case 8: hipLaunchKernelGGL((rof_rows_kernel<XT, VEC, 8, PHASE, OFF32>), gr, bl, g_lds_pad, st, a); break;
        case 16: hipLaunchKernelGGL((rof_rows_kernel<XT, VEC, 16, PHASE, OFF32>), gr, bl, g_lds_pad, st, a); break;
        case 32: hipLaunchKernelGGL((rof_rows_kernel<XT, VEC, 32, PHASE, OFF32>), gr, bl, g_lds_pad, st, a); break;
        default: hipLaunchKernelGGL((rof_rows_kernel<XT, VEC, 64, PHASE, OFF32>), gr, bl, g_lds_pad, st, a); break;
    }
    HIP_TRY(hipGetLastError());
    return ROF_OK;
}

// off32: every byte offset into the feature matrix and into the partial-sum workspace fits 32 bits and
// every row id fits 24 bits, so the kernels may use the short address arithmetic.
template <int PHASE>
int launch_phase(const AggArgs &a, int dtype, int vec, bool off32, hipStream_t st) {
    int need = (a.feat + vec - 1) / vec, lpr = 4;
    while (lpr < need && lpr < 64) lpr <<= 1;
    if (dtype == ROF_F32) {
        if (vec == 4)
            return off32 ? launch_lpr<float, 4, PHASE, true>(a, lpr, st) : launch_lpr<float, 4, PHASE, false>(a, lpr, st);
        return launch_lpr<float, 1, PHASE, false>(a, lpr, st);
    }
    if (vec == 8)
        return off32 ? launch_lpr<uint16_t, 8, PHASE, true>(a, lpr, st)
                     : launch_lpr<uint16_t, 8, PHASE, false>(a, lpr, st);
    return launch_lpr<uint16_t, 1, PHASE, false>(a, lpr, st);
}

int upload_phase(const rof_phase_host &h, rof_phase_dev &d, bool with_scale, hipStream_t st, int64_t *bytes) {
    d.n_wave = h.n_wave;
    d.n_tasks = h.n_tasks;
    d.n_entries = (int64_t)h.col.size();
    auto put = [&](int32_t **dst, const std::vector<int32_t> &src) -> int {
        size_t nb = (src.size() ? src.size() : 1) * sizeof(int32_t);
        HIP_TRY(hipMalloc((void **)dst, nb));
        *bytes += (int64_t)nb;
        if (!src.empty()) HIP_TRY(hipMemcpyAsync(*dst, src.data(), src.size() * sizeof(int32_t), hipMemcpyHostToDevice, st));
        return ROF_OK;
    };
    int rc;
    if ((rc = put(&d.task_ptr, h.task_ptr))) return rc;
    if ((rc = put(&d.task_nref, h.task_nref))) return rc;
    if ((rc = put(&d.task_out, h.task_out))) return rc;
    if ((rc = put(&d.col, h.col))) return rc;
    size_t wb = (h.col.size() ? h.col.size() : 1) * sizeof(float);
    HIP_TRY(hipMalloc((void **)&d.w, wb));
    *bytes += (int64_t)wb;
    if (with_scale) {
        size_t sb = (size_t)(h.n_tasks ? h.n_tasks : 1) * sizeof(float);
        HIP_TRY(hipMalloc((void **)&d.scale, sb));
        *bytes += (int64_t)sb;
    }
    return ROF_OK;
}

void free_phase(rof_phase_dev &d) {
    if (d.task_ptr) (void)hipFree(d.task_ptr);
    if (d.task_nref) (void)hipFree(d.task_nref);
    if (d.task_out) (void)hipFree(d.task_out);
    if (d.col) (void)hipFree(d.col);
    if (d.w) (void)hipFree(d.w);
    if (d.scale) (void)hipFree(d.scale);
    d = rof_phase_dev();
}

inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }



}  // namespace

void rof_set_device_error(const char *what, const char *text) {
    snprintf(g_dev_err, sizeof(g_dev_err), "%s: %s", what, text);
}

extern "C" {

const char *rof_last_device_error(void) { return g_dev_err; }

const char *rof_strerror(int status) {
    switch (status) {
        case ROF_OK: return "ok";
        case ROF_ERR_ARG: return "invalid argument";
        case ROF_ERR_RANGE: return "index out of range";
        case ROF_ERR_ALLOC: return "allocation failed";
        case ROF_ERR_DEVICE: return "HIP call failed";
        case ROF_ERR_STATE: return "layout is not in the required state";
        case ROF_ERR_UNSUPPORTED: return "unsupported size or type";
        case ROF_ERR_WORKSPACE: return "workspace too small";
        default: return "unknown status";
    }
}

int rof_version(void) { return 1; }

// Tuning knob used by the benchmark sweeps: consecutive workgroups per XCD for launch 1 / launch 2.
int rof_set_lds_pad(int bytes) {
    if (bytes < 0 || bytes > 64 * 1024) return ROF_ERR_ARG;
    g_lds_pad = bytes;
    return ROF_OK;
}

int rof_set_xcd_run(int run_a, int run_b) {
    if (run_a < 1 || run_b < 1 || run_a > 4096 || run_b > 4096) return ROF_ERR_ARG;
    g_xcd_run_a = run_a;
    g_xcd_run_b = run_b;
    return ROF_OK;
}

int rof_device_copy(void *dst, const void *src, size_t nbytes, void *stream) {
    if (!dst || !src || (nbytes & 15) || (((uintptr_t)dst | (uintptr_t)src) & 15)) return ROF_ERR_ARG;
    if (nbytes == 0) return ROF_OK;
    hipLaunchKernelGGL(rof_copy_kernel, dim3(256 * 32), dim3(256), 0, (hipStream_t)stream, (const float4 *)src,
                       (float4 *)dst, (int64_t)(nbytes / 16));
    HIP_TRY(hipGetLastError());
    return ROF_OK;
}

int rof_layout_upload(rof_layout *L, void *stream) {
    if (!L) return ROF_ERR_ARG;
    if (L->uploaded) return ROF_OK;
    hipStream_t st = (hipStream_t)stream;
    HIP_TRY(hipGetDevice(&L->device));
    int rc;
    if ((rc = upload_phase(L->g, L->dg, false, st, &L->device_bytes))) return rc;
    if ((rc = upload_phase(L->s, L->ds, false, st, &L->device_bytes))) return rc;
    if ((rc = upload_phase(L->b, L->db, true, st, &L->device_bytes))) return rc;
    HIP_TRY(hipStreamSynchronize(st));   // the host vectors may be released after this call
    L->uploaded = true;
    return ROF_OK;
}

int rof_layout_set_degrees(rof_layout *L, const float *deg, void *stream) {
    if (!L || !deg) return ROF_ERR_ARG;
    if (!L->uploaded) return ROF_ERR_STATE;
    hipStream_t st = (hipStream_t)stream;
    const int tb = 256;
    for (rof_phase_dev *d : {&L->dg, &L->ds})
        if (d->n_entries)
            hipLaunchKernelGGL(rof_entry_weights_kernel, dim3((unsigned)((d->n_entries + tb - 1) / tb)), dim3(tb), 0,
                               st, d->col, d->n_entries, deg, L->n, d->w);
    if (L->db.n_entries)
        hipLaunchKernelGGL(rof_entry_weights_kernel, dim3((unsigned)((L->db.n_entries + tb - 1) / tb)), dim3(tb), 0, st,
                           L->db.col, L->db.n_entries, deg, L->n, L->db.w);
    if (L->db.n_tasks)
        hipLaunchKernelGGL(rof_task_scale_kernel, dim3((unsigned)((L->db.n_tasks + tb - 1) / tb)), dim3(tb), 0, st,
                           L->db.task_out, L->db.n_tasks, deg, L->db.scale);
    HIP_TRY(hipGetLastError());
    L->weights_set = true;
    return ROF_OK;
}

size_t rof_layout_workspace_bytes(const rof_layout *L, int feat_dim) {
    if (!L || feat_dim < 1) return 0;
    return (size_t)L->n_slots * (size_t)round_up(feat_dim, 8) * sizeof(float);
}

void rof_layout_free(rof_layout *L) {
    if (!L) return;
    if (L->uploaded) {
        free_phase(L->dg);
        free_phase(L->ds);
        free_phase(L->db);
    }
    delete L;
}

static int aggregate_impl(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, float *out, int64_t ldo,
                          int feat, int normalized, void *workspace, size_t workspace_bytes, void *stream,
                          int launches) {
    if (!L || !x || !out || feat < 1 || ldx < feat || ldo < feat) return ROF_ERR_ARG;
    if (x_dtype != ROF_F32 && x_dtype != ROF_BF16) return ROF_ERR_UNSUPPORTED;
    if (!L->uploaded || (normalized && !L->weights_set)) return ROF_ERR_STATE;
    if ((int64_t)L->n * ldx >= ((int64_t)1 << 40) || (int64_t)L->n * ldo >= ((int64_t)1 << 40)) return ROF_ERR_UNSUPPORTED;
    const size_t need = rof_layout_workspace_bytes(L, feat);
    if (need && (!workspace || workspace_bytes < need)) return ROF_ERR_WORKSPACE;
    if (need && ((uintptr_t)workspace & 15)) return ROF_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;

    const int esz = x_dtype == ROF_F32 ? 4 : 2;
    const int wide = x_dtype == ROF_F32 ? 4 : 8;
    // 16-byte gathers need rows that start on a 4-byte boundary and hold at least one full vector
    const bool dword_rows = (((uintptr_t)x) % 4 == 0) && ((ldx * esz) % 4 == 0);
    const int vec = (dword_rows && feat >= wide) ? wide : 1;
    const int64_t ldp = round_up(feat, 8);
    const int64_t rows_x = L->n, rows_p = L->n_slots;
    const bool off32 = rows_x < (1 << 24) && rows_p < (1 << 24) && ldx * esz < (1 << 24) && ldp * 4 < (1 << 24) &&
                       (rows_x + 1) * ldx * esz < ((int64_t)1 << 32) && (rows_p + 1) * ldp * 4 < ((int64_t)1 << 32);

    AggArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x;
    a.ldx = ldx;
    a.part = (const float *)workspace;
    a.ldp = ldp;
    a.nsplit = L->n;
    a.feat = feat;
    int rc;
    // launches 1 and 2: partial-sum rows (shared groups, then segments of long rows)
    const rof_phase_dev *partial[2] = {&L->dg, &L->ds};
    for (int i = 0; i < 2 && (launches & 1); ++i) {
        const rof_phase_dev &d = *partial[i];
        if (!d.n_tasks) continue;
        a.task_ptr = d.task_ptr;
        a.task_nref = d.task_nref;
        a.task_out = d.task_out;
        a.task_scale = nullptr;
        a.col = d.col;
        a.w = normalized ? d.w : nullptr;
        a.out = (float *)workspace;
        a.ldo = ldp;
        a.n_wave = d.n_wave;
        a.n_tasks = d.n_tasks;
        a.xcd_run = g_xcd_run_a;
        a.vec_store = 1;
        if ((rc = launch_phase<0>(a, x_dtype, vec, off32, st))) return rc;
    }
    if (L->db.n_tasks && (launches & 2)) {   // last launch: destination rows
        a.task_ptr = L->db.task_ptr;
        a.task_nref = L->db.task_nref;
        a.task_out = L->db.task_out;
        a.task_scale = normalized ? L->db.scale : nullptr;
        a.col = L->db.col;
        a.w = normalized ? L->db.w : nullptr;
        a.out = out;
        a.ldo = ldo;
        a.n_wave = L->db.n_wave;
        a.n_tasks = L->db.n_tasks;
        a.xcd_run = g_xcd_run_b;
        a.vec_store = (ldo % 4 == 0) && (((uintptr_t)out) % 16 == 0);
        if ((rc = launch_phase<1>(a, x_dtype, vec, off32, st))) return rc;
    }
    return ROF_OK;
}

int rof_aggregate(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, float *out, int64_t ldo, int feat,
                  int normalized, void *workspace, size_t workspace_bytes, void *stream) {
    return aggregate_impl(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, stream, 3);
}

int rof_aggregate_timed(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, float *out, int64_t ldo,
                        int feat, int normalized, void *workspace, size_t workspace_bytes, void *stream, int iters,
                        float *ms_per_call) {
    if (!ms_per_call || iters < 1) return ROF_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0, e1;
    HIP_TRY(hipEventCreate(&e0));
    HIP_TRY(hipEventCreate(&e1));
    int rc = ROF_OK;
    HIP_TRY(hipEventRecord(e0, st));
    for (int i = 0; i < iters && rc == ROF_OK; ++i)
        rc = rof_aggregate(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, st);
    HIP_TRY(hipEventRecord(e1, st));
    HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *ms_per_call = ms / iters;
    return rc;
}

int rof_aggregate_launch_times(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, float *out, int64_t ldo,
                               int feat, int normalized, void *workspace, size_t workspace_bytes, void *stream,
                               int iters, float ms_launch[2]) {
    if (!ms_launch || iters < 1 || !L) return ROF_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    // each iteration times [launch 1 + launch 2] and then [launch 2 alone]; launch 2 alone is a
    // complete run because launch 1's rows are still in the workspace
    hipEvent_t e0, e1, e2;
    HIP_TRY(hipEventCreate(&e0));
    HIP_TRY(hipEventCreate(&e1));
    HIP_TRY(hipEventCreate(&e2));
    double both = 0.0, second = 0.0;
    int rc = rof_aggregate(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, st);
    for (int i = 0; i < iters && rc == ROF_OK; ++i) {
        HIP_TRY(hipEventRecord(e0, st));
        rc = rof_aggregate(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, st);
        HIP_TRY(hipEventRecord(e1, st));
        if (rc == ROF_OK)
            rc = aggregate_impl(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, st, 2);
        HIP_TRY(hipEventRecord(e2, st));
        HIP_TRY(hipEventSynchronize(e2));
        float a = 0.f, b = 0.f;
        HIP_TRY(hipEventElapsedTime(&a, e0, e1));
        HIP_TRY(hipEventElapsedTime(&b, e1, e2));
        both += a;
        second += b;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipEventDestroy(e2);
    ms_launch[1] = (float)(second / iters);
    ms_launch[0] = (float)((both - second) / iters);
    return rc;
}

}  // extern "C"
