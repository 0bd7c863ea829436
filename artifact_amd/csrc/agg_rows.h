// Row-gather kernels of the reuse-aware aggregation and their launcher template, shared by the
// translation units that instantiate them (by feature type and by launch, compiled separately so that the
// build can run them in parallel).  See agg_kernels.hip for the description of the scheme.
#ifndef ROF_AGG_ROWS_H_
#define ROF_AGG_ROWS_H_

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "rof.h"
#include "rof_internal.h"

#define HIP_TRY(expr)                                                                  \
    do {                                                                               \
        hipError_t e_ = (expr);                                                        \
        if (e_ != hipSuccess) {                                                        \
            rof_set_device_error(#expr, hipGetErrorString(e_));                        \
            return ROF_ERR_DEVICE;                                                     \
        }                                                                              \
    } while (0)

namespace rofk {

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
    void *out;                 // float rows, or bf16 rows when out_bf16 (destination-row launch only)
    int64_t ldo;
    int32_t feat;
    int32_t n_wave, n_tasks;
    int32_t n_blocks;          // logical workgroups
    int32_t xcd_run;           // consecutive logical workgroups kept on one XCD
    int32_t wave_cap;          // host side only: at most this many wavefronts per SIMD (0: as many as fit)
    int32_t lds_pad;           // host side only: bytes of unused LDS requested per workgroup (benchmark tuning)
    int32_t lds_per_cu;        // host side only: LDS bytes of one CU on the layout's device (queried at upload)
    int32_t vec_store;         // output rows start on 4-byte boundaries: whole-vector stores
    const float *bias;         // destination-row launch only: added to every output row (null: none)
    int32_t relu;              // destination-row launch only: clamp the output at zero
    int32_t out_bf16;          // destination-row launch only: store bf16 (round to nearest even)
    float self_weight;         // destination-row launch only: + self_weight * x[out row] (0: none)
    // cluster launch only (CLUSTER instantiations): workgroup i has its own list of short tasks lg_task_first[i] ..
    // lg_task_first[i+1] and its local groups lg_ptr[i] .. lg_ptr[i+1] (local group j gathers
    // lg_col[lg_task_ptr[j] .. lg_task_ptr[j+1])), which it sums into LDS before its tasks run
    const int32_t *lg_ptr, *lg_task_ptr, *lg_col, *lg_task_first;
    const float *lg_w;         // null: unweighted
};

// fp32 -> bf16, round to nearest even, NaN -> quiet NaN (the conversion PyTorch's .to(bfloat16) performs)
__device__ __forceinline__ uint32_t rof_bf16_bits(float f) {
    const uint32_t u = __float_as_uint(f);
    if (f != f) return 0x7fc0u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// Row gathers a lane group keeps in flight.  Measured on MI355X with all eight wave slots per SIMD
// occupied: 2 beats 4 by ~10 % on the miss-dominated workloads (more outstanding gathers per CU slow the
// L1/L2 miss path down) and loses ~2 % where gathers hit in L2; 8 loses everywhere.
constexpr int kGathersInFlight = 2;
constexpr int kWavesPerBlock = 4;
constexpr int kXcds = 8;
constexpr int64_t kLdsPerCu = 160 * 1024;   // gfx950; the launch path uses what the device reports at upload

template <typename XT, int VEC>
struct RowLoad;

#define ROF_LD16(T, p) (*reinterpret_cast<const T *>(p))
// 16-byte vectors that only promise 4-byte alignment: gfx950 executes global_load_dwordx4 at any dword
// address, so packed rows (e.g. 47 floats = 188 bytes) are gathered with the same instruction as padded ones
typedef float rof_f4 __attribute__((ext_vector_type(4), aligned(4)));
typedef unsigned int rof_u4 __attribute__((ext_vector_type(4), aligned(4)));
typedef unsigned int rof_u2s __attribute__((ext_vector_type(2), aligned(4)));

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
    // HIP declares __umul24 as returning int: without the cast a byte offset of 2^31 or more would be
    // sign-extended into a negative one
    if (OFF32) return b + (uint32_t)__umul24(r, l);
    return b + (uint64_t)r * l;
}

// Byte address of a lane for ds_bpermute: a per-lane base plus a compile-time constant, added where it is used.
// Left to the compiler, the 2 * LPR lane numbers of the hand-offs below are loop invariants that it keeps in as
// many registers (an occupancy step at 10, 12 and 20 lanes per row); the volatile statement pins the addition to
// its place, one instruction and one short-lived register per hand-off.
__device__ __forceinline__ int lane_addr(int base, int offset) {
    int r;
    asm volatile("v_add_u32 %0, %2, %1" : "=v"(r) : "v"(base), "i"(offset));
    return r;
}

// Sum the entries [beg, end) of one task into acc.  WAVE: all lane groups of the wavefront share
// the task (beg/end wave-uniform) and take every G-th entry; otherwise each lane group owns its
// task.  ST is the element type of the source rows.  Blocks of U entries that are complete for every
// lane group run without any per-entry predicate; ragged ends are predicated entry by entry.
template <typename ST, int VEC, int LPR, bool WAVE, bool DUAL, bool OFF32, bool STREAM_IDS, int INFLIGHT = kGathersInFlight>
__device__ __forceinline__ void gather_sum(const char *xb, uint32_t xld, const char *pb, uint32_t pld, int32_t nsplit,
                                           int32_t bias, const int32_t *__restrict__ col,
                                           const float *__restrict__ w, int32_t beg, int32_t end, int lane, int sub,
                                           int li, bool act, float (&acc)[VEC]) {
    constexpr int G = 64 / LPR;             // lane groups per wavefront; lanes >= G*LPR stay idle
    constexpr int U = LPR >= INFLIGHT ? INFLIGHT : LPR;   // row gathers in flight per lane group
    constexpr int CH = WAVE ? G * LPR : LPR;   // entries fetched per step by the wave / by the lane group
    static_assert(LPR % U == 0, "the unroll factor must divide the lanes per row");
    const bool idle = (G * LPR < 64) && lane >= G * LPR;
    for (int32_t base = beg; __any(!idle && base < end); base += CH) {
        const int32_t mine = base + (WAVE ? lane : li);
        int32_t mycol = bias;               // past the end: row 0 of the source, weight 0
        float myw = 0.0f;
        if (!idle && mine < end) {
            if constexpr (STREAM_IDS) {
                // read once per launch, and the launch is a large one (see PHASE 2): streaming loads, so that they
                // do not push feature rows out of the caches.  Small graphs keep their index arrays cached from one
                // layer to the next and are better off with ordinary loads.
                mycol = __builtin_nontemporal_load(col + mine);
                myw = w ? __builtin_nontemporal_load(w + mine) : 1.0f;
            } else {
                mycol = col[mine];
                myw = w ? w[mine] : 1.0f;
            }
        }
#pragma unroll
        for (int j0 = 0; j0 < LPR; j0 += U) {
            const int first = WAVE ? j0 * G + sub : j0;
            if (!__any(!idle && base + first < end)) break;
            int32_t c[U];
            float wt[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                // entry (j0 + u) * G + sub of the wave's chunk (WAVE), entry j0 + u of the lane group's chunk
                // otherwise: fetched by the lane of that number / by lane sub * LPR + j0 + u
                constexpr int kStep = WAVE ? G * 4 : 4;
                const int addr = lane_addr(WAVE ? sub * 4 : sub * LPR * 4, (j0 + u) * kStep);
                c[u] = __builtin_amdgcn_ds_bpermute(addr, mycol);
                wt[u] = __int_as_float(__builtin_amdgcn_ds_bpermute(addr, __float_as_int(myw)));
            }
            const int last = WAVE ? (j0 + U - 1) * G + sub : (j0 + U - 1);
            const bool full = __all(idle || base + last < end);
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

// Scale the finished sum of task t, apply the layer's epilogue (PHASE 1, 2 and 4) and store this lane's piece of the
// output row.  `acc` holds the columns cstart .. cstart + VEC - 1; `skip` of them repeat the neighbouring lane's.
template <typename XT, int VEC, int PHASE>
__device__ __forceinline__ void finish_row(const AggArgs &a, int32_t out_row, float scale, bool nonempty, const float (&acc)[VEC],
                                           const char *xb, uint32_t xld, int cstart, int skip) {
    // an empty task writes zeros whatever its scale is (a node without in-edges keeps the
    // zero-initialised output upstream: reuse_conv_kernel.cu:303)
    const float s = nonempty ? scale : 1.0f;
    const int64_t at = (int64_t)out_row * a.ldo + cstart;
    float r[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) r[k] = acc[k] * s;
    constexpr bool kDst = PHASE == 1 || PHASE == 2 || PHASE == 4;   // a destination-row launch
    if (kDst) {   // epilogue of the layer: + own row, + bias, then ReLU (columns cstart .. cstart+VEC-1 exist)
        if (a.self_weight != 0.0f) {
            float own[VEC];
            RowLoad<XT, VEC>::load(reinterpret_cast<const XT *>(xb + (int64_t)out_row * xld), own);
#pragma unroll
            for (int k = 0; k < VEC; ++k) r[k] = fmaf(a.self_weight, own[k], r[k]);
        }
        if (a.bias) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) r[k] = __fadd_rn(r[k], a.bias[cstart + k]);   // never fused into the scaling: same bits as a separate pass
        }
        if (a.relu) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) r[k] = fmaxf(r[k], 0.0f);
        }
    }
    // A large output is not read again before the caches have turned over, so its rows are written as
    // streaming stores (`nt`): they then do not push feature rows out of L2 and the Infinity Cache.
    // Every lane stores whole 16-byte pieces (8-byte for bf16 output) wherever the piece starts on a 4-byte
    // boundary -- gfx950 executes global_store_dwordx4 at any dword address, like the loads -- so packed rows
    // (47 floats = 188 bytes) are written as one contiguous burst per row.  The lane that was shifted back
    // to stay inside the row rewrites `skip` elements of its neighbour's piece with the same bits (both
    // lanes sum the same entries in the same order).
    constexpr bool stream = PHASE == 2 || PHASE == 3;
    if (kDst && a.out_bf16) {
        uint16_t *o = reinterpret_cast<uint16_t *>(a.out) + at;
        if (VEC == 8 && a.vec_store && (at & 1) == 0) {   // the lane's 8 columns are one 16-byte piece
            const rof_u4 t = {rof_bf16_bits(r[0]) | (rof_bf16_bits(r[1 % VEC]) << 16),   // (% VEC: well-formed in the
                              rof_bf16_bits(r[2 % VEC]) | (rof_bf16_bits(r[3 % VEC]) << 16),   //  narrower instantiations)
                              rof_bf16_bits(r[4 % VEC]) | (rof_bf16_bits(r[5 % VEC]) << 16),
                              rof_bf16_bits(r[6 % VEC]) | (rof_bf16_bits(r[7 % VEC]) << 16)};
            if (stream) __builtin_nontemporal_store(t, reinterpret_cast<rof_u4 *>(o));
            else *reinterpret_cast<rof_u4 *>(o) = t;
        } else if (VEC >= 4 && a.vec_store && (at & 1) == 0) {
#pragma unroll
            for (int k = 0; k < VEC; k += 4) {
                const rof_u2s t = {rof_bf16_bits(r[k]) | (rof_bf16_bits(r[k + 1]) << 16),
                                   rof_bf16_bits(r[k + 2]) | (rof_bf16_bits(r[k + 3]) << 16)};
                if (stream) __builtin_nontemporal_store(t, reinterpret_cast<rof_u2s *>(o + k));
                else *reinterpret_cast<rof_u2s *>(o + k) = t;
            }
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k)
                if (k >= skip && cstart + k < a.feat) o[k] = (uint16_t)rof_bf16_bits(r[k]);
        }
    } else {
        float *o = reinterpret_cast<float *>(a.out) + at;
        if (VEC == 8 && stream && a.vec_store && (a.feat & 15) == 0) {
            // A lane holds 8 columns = 32 bytes, so each of its two 16-byte stores would leave a 16-byte hole
            // between lanes, and streaming stores are not merged in L2: such rows reached memory as partial
            // lines (WRITE_SIZE 9-13 % above the bytes stored).  Neighbouring lanes swap halves instead -- the even
            // lane of a pair hands over its upper four columns for the odd lane's lower four -- and both store
            // instructions then write one gap-free run of 16 bytes per lane.  (feat % 16 == 0: every lane has its
            // partner, in the same row, and no lane is shifted.)
            const bool odd = (cstart >> 3) & 1;
            float got[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) got[k] = __shfl_xor(odd ? r[k % VEC] : r[(4 + k) % VEC], 1);
            const rof_f4 lo = {odd ? got[0] : r[0], odd ? got[1] : r[1 % VEC], odd ? got[2] : r[2 % VEC],
                               odd ? got[3] : r[3 % VEC]};
            const rof_f4 hi = {odd ? r[4 % VEC] : got[0], odd ? r[5 % VEC] : got[1], odd ? r[6 % VEC] : got[2],
                               odd ? r[7 % VEC] : got[3]};
            float *p = o - (odd ? 4 : 0);   // even: columns B .. B+3 and B+8 .. B+11; odd: B+4 .. B+7 and B+12 .. B+15
            __builtin_nontemporal_store(lo, reinterpret_cast<rof_f4 *>(p));
            __builtin_nontemporal_store(hi, reinterpret_cast<rof_f4 *>(p + 8));
        } else if (VEC >= 4 && a.vec_store) {
#pragma unroll
            for (int k = 0; k < VEC; k += 4) {
                const rof_f4 t = {r[k], r[k + 1], r[k + 2], r[k + 3]};
                if (stream) __builtin_nontemporal_store(t, reinterpret_cast<rof_f4 *>(o + k));
                else *reinterpret_cast<rof_f4 *>(o + k) = t;
            }
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k)
                if (k >= skip && cstart + k < a.feat) o[k] = r[k];
        }
    }
}

// PHASE 0: the partial-sum launches (no scaling, no epilogue); PHASE 3: the same with the partial rows written as
// streaming stores (a workspace too large to stay in the caches until the destination rows read it); PHASE 1: the
// destination-row launch; PHASE 2: the same with the output rows written as streaming stores and the index arrays
// read as streaming loads (large outputs, hence large graphs).  (A run-time switch between the two kinds of store does
// not survive the optimiser, which merges the two stores into an ordinary one.)  PHASE 5 and 4: PHASE 0 and 1 with
// more row gathers in flight, for feature matrices that the caches serve (fp32 rows only).
template <typename XT, int VEC, int LPR, int PHASE, bool OFF32>
__global__ __launch_bounds__(256) void rof_rows_kernel(AggArgs a) {
    constexpr int G = 64 / LPR;
    // The partial-sum launches sweep the feature matrix and mostly hit in L2; with rows of 16 lanes or more (4 rows
    // per wavefront or fewer) two gathers in flight leave them short of requests and four run faster wherever the
    // caches serve the sweep (2^18 nodes x 256 floats: 133 -> 124 us, x 128 floats: 70 -> 59 us; 2.4 M nodes x 160
    // floats: 2.27 -> 2.13 ms, x 64 / 100 / 128 / 256 floats unchanged).  bf16 rows (8 values to widen per piece)
    // measured 2 % slower with four, and the destination rows of the same widths +8 %, -4 % and +2 %: both keep two.
    // A matrix that the caches serve answers quickly, and two gathers per lane group leave every launch short of
    // requests: four (five at 10 lanes per row) measured -18 % on the 2^14-node workload (32 floats), -8.5 % at
    // 2^18 nodes x 32 floats, -15 % at 2^14 x 256; 0 on the block model and +2 ... +8 % on matrices of 0.27-2.5 GB.
    constexpr bool kDeep = PHASE == 4 || PHASE == 5;
    constexpr int kU = kDeep ? (LPR % 4 == 0 ? 4 : LPR % 5 == 0 ? 5 : kGathersInFlight)
                             : ((PHASE == 0 || PHASE == 3) && LPR >= 16 && sizeof(XT) == 4) ? 4 : kGathersInFlight;
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
    const bool idle = (G * LPR < 64) && lane >= G * LPR;   // lanes left over when LPR does not divide 64
    if (wave_mode) {
        t = gw;
        valid = true;
    } else {
        t = a.n_wave + (gw - a.n_wave) * G + sub;
        valid = !idle && t < a.n_tasks;
    }
    // The output row and its scale are needed last.  The launches that run with more gathers in flight serve small
    // matrices and are bound by the latency of their longest chain of dependent loads, so they fetch both up front,
    // with the task's range; everywhere else the two registers would cost an occupancy step, and the loads wait
    // until the sum is finished.
    int32_t out_row = 0;
    float out_scale = 1.0f;
    if (valid) {
        beg = a.task_ptr[t];
        end = a.task_ptr[t + 1];
        mid = beg + a.task_nref[t];
        if constexpr (kDeep) {
            out_row = a.task_out[t];
            if (a.task_scale) out_scale = a.task_scale[t];
        }
    }
    const uint32_t xld = (uint32_t)(a.ldx * (int64_t)sizeof(XT)), pld = (uint32_t)(a.ldp * 4);

    for (int c0 = 0; c0 < a.feat; c0 += LPR * VEC) {
        const int cbase = c0 + li * VEC;
        const bool act = !idle && cbase < a.feat;
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
                // only tasks that reference partial rows pay for the select between the two matrices
                if (mid > beg)
                    gather_sum<XT, VEC, LPR, true, true, OFF32, PHASE == 2, kU>(xb, xld, pb, pld, a.nsplit, 0, a.col, a.w, beg, end,
                                                                lane, sub, li, act, acc);
                else
                    gather_sum<XT, VEC, LPR, true, false, OFF32, PHASE == 2, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, beg, end, lane,
                                                                 sub, li, act, acc);
            } else {
                if (mid > beg)
                    gather_sum<float, VEC, LPR, true, false, OFF32, PHASE == 2, kU>(pb, pld, nullptr, 0, 0, a.nsplit, a.col, a.w, beg,
                                                                    mid, lane, sub, li, act, acc);
                gather_sum<XT, VEC, LPR, true, false, OFF32, PHASE == 2, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, mid, end, lane, sub,
                                                             li, act, acc);
            }
            if ((G & (G - 1)) == 0) {   // power-of-two group count: butterfly
#pragma unroll
                for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) acc[k] += __shfl_xor(acc[k], off);
                }
            } else {                    // otherwise group 0 collects the others one by one
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    float tot = acc[k];
#pragma unroll
                    for (int g = 1; g < G; ++g)   // from lane li + g * LPR (< 64)
                        tot += __int_as_float(__builtin_amdgcn_ds_bpermute(lane_addr(li * 4, g * LPR * 4), __float_as_int(acc[k])));
                    acc[k] = tot;
                }
            }
        } else {
            if (kF32) {
                if (__any(mid > beg))
                    gather_sum<XT, VEC, LPR, false, true, OFF32, PHASE == 2, kU>(xb, xld, pb, pld, a.nsplit, 0, a.col, a.w, beg, end,
                                                                 lane, sub, li, act, acc);
                else
                    gather_sum<XT, VEC, LPR, false, false, OFF32, PHASE == 2, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, beg, end, lane,
                                                                  sub, li, act, acc);
            } else {
                if (__any(mid > beg))
                    gather_sum<float, VEC, LPR, false, false, OFF32, PHASE == 2, kU>(pb, pld, nullptr, 0, 0, a.nsplit, a.col, a.w, beg,
                                                                     mid, lane, sub, li, act, acc);
                gather_sum<XT, VEC, LPR, false, false, OFF32, PHASE == 2, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, mid, end, lane, sub,
                                                              li, act, acc);
            }
        }

        if (valid && act && (!wave_mode || sub == 0)) {
            if constexpr (!kDeep) {
                if (c0 == 0) {
                    out_row = a.task_out[t];
                    if (a.task_scale && end > beg) out_scale = a.task_scale[t];
                }
            }
            finish_row<XT, VEC, PHASE>(a, out_row, out_scale, end > beg, acc, xb, xld, cstart, skip);
        }
    }
}

// Add the LDS rows of one clustered task (their numbers are the first `nlds` entries of its list) into acc.  The
// numbers are fetched LPR at a time, one by each lane of the lane group, and handed round: one memory latency per LPR
// rows instead of one per row.  EARLY: `mine0` holds the first LPR numbers, requested by the caller beforehand.
template <int VEC, int LPR, bool EARLY>
__device__ __forceinline__ void add_lds_rows(const float *lds_rows, const int32_t *__restrict__ col, int32_t first, int32_t nlds,
                                             int32_t mine0, int sub, int li, float (&acc)[VEC]) {
    constexpr int kLdsRow = LPR * VEC + 4;
    if constexpr (!EARLY && LPR < 10) {   // (bf16 at 16 and 8 rows per wavefront: the hand-off would cost a wavefront)
        for (int j = 0; j < nlds; ++j) {
            const float *row = lds_rows + col[first + j] * kLdsRow + li * VEC;
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[k] += row[k];
        }
        return;
    }
#pragma unroll 1
    for (int j0 = 0; __any(j0 < nlds); j0 += LPR) {
        const int32_t mine = (EARLY && j0 == 0) ? mine0 : (j0 + li < nlds) ? col[first + j0 + li] : 0;
#pragma unroll
        for (int j = 0; j < LPR; ++j) {
            if (!__any(j0 + j < nlds)) break;
            const int32_t r = __builtin_amdgcn_ds_bpermute(lane_addr(sub * LPR * 4, j * 4), mine);
            if (j0 + j < nlds) {
                const float *row = lds_rows + r * kLdsRow + li * VEC;
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] += row[k];
            }
        }
    }
}

// The launch of the clustered destinations (PHASE >= 1 only).  Workgroup i holds cluster i: destinations that share
// reuse groups.  It first sums its local groups lg_ptr[i] .. lg_ptr[i+1] into LDS rows, one lane group per group,
// then works through its own list of short tasks (lg_task_first[i] .. lg_task_first[i+1], in rounds of 4 * G), and
// those tasks add LDS rows instead of gathering the groups' sources.  An LDS row holds the LPR * VEC columns of the
// current feature chunk, laid out by lane, so a lane reads back exactly the columns it accumulates.  (A kernel of
// its own rather than a branch of rof_rows_kernel: there the extra live values cost an occupancy step, 6-8 % of
// the launch.)
template <typename XT, int VEC, int LPR, int PHASE, bool OFF32>
__global__ __launch_bounds__(256) void rof_cluster_kernel(AggArgs a) {
    static_assert(PHASE == 1 || PHASE == 2, "clusters belong to the destination-row launch");
    constexpr int G = 64 / LPR;
    constexpr int kLdsRow = LPR * VEC + 4;
    HIP_DYNAMIC_SHARED(float, lds_rows)
    const int hw = blockIdx.x;
    const int xcd = hw % kXcds, nth = hw / kXcds;
    const int run = a.xcd_run;
    const int cb = ((nth / run) * kXcds + xcd) * run + (nth % run);
    if (cb >= a.n_blocks) return;

    const int lane = threadIdx.x & 63;
    const int sub = lane / LPR, li = lane % LPR;
    const int wid = threadIdx.x >> 6;
    const bool idle = (G * LPR < 64) && lane >= G * LPR;   // lanes left over when LPR does not divide 64
    const int32_t ct0 = a.lg_task_first[cb], ct1 = a.lg_task_first[cb + 1];
    const int32_t lg0 = a.lg_ptr[cb], lg1 = a.lg_ptr[cb + 1];
    const uint32_t xld = (uint32_t)(a.ldx * (int64_t)sizeof(XT)), pld = (uint32_t)(a.ldp * 4);
    constexpr bool kF32 = sizeof(XT) == 4;

    for (int c0 = 0; c0 < a.feat; c0 += LPR * VEC) {
        const int cbase = c0 + li * VEC;
        const bool act = !idle && cbase < a.feat;
        const int cstart = (VEC > 1 && cbase + VEC > a.feat) ? a.feat - VEC : cbase;   // see rof_rows_kernel
        const int skip = cbase - cstart;
        const char *xb = reinterpret_cast<const char *>(a.x) + (size_t)cstart * sizeof(XT);
        const char *pb = reinterpret_cast<const char *>(a.part) + (size_t)cstart * 4;

        if (c0 > 0) __syncthreads();   // the previous chunk's rows have been read by every task
        for (int g0 = lg0 + wid * G; g0 < lg1; g0 += kWavesPerBlock * G) {
            const int g = g0 + sub;
            int32_t gb = 0, ge = 0;
            if (!idle && g < lg1) {
                gb = a.lg_task_ptr[g];
                ge = a.lg_task_ptr[g + 1];
            }
            float part[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) part[k] = 0.0f;
            gather_sum<XT, VEC, LPR, false, false, OFF32, false>(xb, xld, nullptr, 0, 0, 0, a.lg_col, a.lg_w, gb, ge, lane,
                                                                 sub, li, act, part);
            if (!idle && g < lg1) {
                float *row = lds_rows + (g - lg0) * kLdsRow + li * VEC;
#pragma unroll
                for (int k = 0; k < VEC; ++k) row[k] = part[k];
            }
        }
        __syncthreads();

        for (int32_t t0 = ct0 + wid * G; t0 < ct1; t0 += kWavesPerBlock * G) {   // one lane group per task
            const int32_t t = t0 + sub;
            const bool valid = !idle && t < ct1;
            int32_t first = 0, beg = 0, mid = 0, end = 0, nlds = 0, out_row = 0;
            float out_scale = 1.0f;
            if (valid) {
                first = a.task_ptr[t];
                end = a.task_ptr[t + 1];
                if constexpr (kF32) {   // with the task's range, not after its sum: one latency less before the store
                    out_row = a.task_out[t];   // (the bf16 instantiations would pay for the two registers with a wavefront)
                    if (a.task_scale) out_scale = a.task_scale[t];
                }
                const uint32_t packed = (uint32_t)a.task_nref[t];   // references in the low 24 bits, LDS rows above
                nlds = (int32_t)(packed >> 24);
                beg = first + nlds;
                mid = beg + (int32_t)(packed & 0xffffffu);
            }
            float acc[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
            // fp32: the numbers of the first LPR LDS rows are requested before the row gathers what it does not share,
            // and the rows added after it, by when the numbers have long arrived (the bf16 instantiations would pay for
            // that order with a wavefront per SIMD and add their LDS rows first)
            const int32_t mine0 = (kF32 && li < nlds) ? a.col[first + li] : 0;
            if constexpr (!kF32) add_lds_rows<VEC, LPR, false>(lds_rows, a.col, first, nlds, mine0, sub, li, acc);
            if (kF32) {
                if (__any(mid > beg))
                    gather_sum<XT, VEC, LPR, false, true, OFF32, PHASE == 2>(xb, xld, pb, pld, a.nsplit, 0, a.col, a.w, beg, end,
                                                                            lane, sub, li, act, acc);
                else
                    gather_sum<XT, VEC, LPR, false, false, OFF32, PHASE == 2>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, beg, end,
                                                                             lane, sub, li, act, acc);
            } else {
                if (__any(mid > beg))
                    gather_sum<float, VEC, LPR, false, false, OFF32, PHASE == 2>(pb, pld, nullptr, 0, 0, a.nsplit, a.col, a.w,
                                                                                beg, mid, lane, sub, li, act, acc);
                gather_sum<XT, VEC, LPR, false, false, OFF32, PHASE == 2>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, mid, end, lane,
                                                                         sub, li, act, acc);
            }
            if constexpr (kF32) add_lds_rows<VEC, LPR, true>(lds_rows, a.col, first, nlds, mine0, sub, li, acc);
            if constexpr (!kF32) {
                if (valid && act) {
                    out_row = a.task_out[t];
                    if (a.task_scale && end > first) out_scale = a.task_scale[t];
                }
            }
            if (valid && act) finish_row<XT, VEC, PHASE>(a, out_row, out_scale, end > first, acc, xb, xld, cstart, skip);
        }
    }
}

// The destination-row launch of a small graph (fp32 rows, short offsets).  A launch that cannot fill the machine lasts
// as long as its longest chain of dependent gathers, and cutting long rows into segments shortens that chain only at
// the price of a second, dependent launch (a quarter to a half of the whole on graphs of 2^14 ... 2^16 nodes).  Here
// the workgroups are 16 wavefronts wide and the first of them take the long rows (the layout puts the longest tasks
// first): the n16 longest get a workgroup each, the next n8 share one between two (8 wavefronts a row), the next n4
// between four.  Every wavefront sums its share of the row's entries, the sums meet in LDS, and the row's first
// wavefront adds them up and stores the row -- the chain of a segment, no partial row through memory and no second
// launch.  The other workgroups run the remaining tasks exactly like rof_rows_kernel, sixteen wavefronts each.
// DEEP: four row gathers in flight per lane group (five at 10 lanes per row) instead of two (fp32 rows).
constexpr int kCoopWaves = 16;
struct CoopSplit {
    int32_t n16, n8, n4;   // leading tasks that get 16, 8 and 4 wavefronts each
    __host__ __device__ int32_t tasks() const { return n16 + n8 + n4; }
    __host__ __device__ int32_t blocks() const { return n16 + (n8 + 1) / 2 + (n4 + 3) / 4; }
};

template <typename XT, int VEC, int LPR, bool DEEP>
__global__ __launch_bounds__(64 * kCoopWaves) void rof_coop_kernel(AggArgs a, CoopSplit cs) {
    constexpr int G = 64 / LPR;
    constexpr bool kF32 = sizeof(XT) == 4;   // fp32 features: partial rows have the same element type
    constexpr int kU = DEEP ? (LPR % 4 == 0 ? 4 : LPR % 5 == 0 ? 5 : kGathersInFlight) : kGathersInFlight;
    constexpr int PHASE = 1;
    __shared__ float red[kCoopWaves][LPR * VEC];
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int sub = lane / LPR, li = lane % LPR;
    const bool idle = (G * LPR < 64) && lane >= G * LPR;   // lanes left over when LPR does not divide 64
    const uint32_t xld = (uint32_t)(a.ldx * (int64_t)sizeof(XT)), pld = (uint32_t)(a.ldp * 4);
    const int hw = blockIdx.x;

    const int32_t n_coop = cs.tasks(), coop_blocks = cs.blocks();
    if (hw < coop_blocks) {   // long rows, summed by 16, 8 or 4 wavefronts each (no thread leaves before the last barrier)
        int per, first, limit;   // wavefronts per row, the workgroup's first task, end of its class of tasks
        if (hw < cs.n16) {
            per = 16, first = hw, limit = cs.n16;
        } else if (hw < cs.n16 + (cs.n8 + 1) / 2) {
            per = 8, first = cs.n16 + (hw - cs.n16) * 2, limit = cs.n16 + cs.n8;
        } else {
            per = 4, first = cs.n16 + cs.n8 + (hw - cs.n16 - (cs.n8 + 1) / 2) * 4, limit = n_coop;
        }
        const int32_t t = first + wid / per;   // this wavefront's row
        const int wsh = wid % per;             // and its share of it
        const bool have = t < limit;
        int32_t beg = 0, end = 0, mid = 0, out_row = 0;
        float out_scale = 1.0f;
        if (have) {
            beg = a.task_ptr[t];
            end = a.task_ptr[t + 1];
            mid = beg + a.task_nref[t];
            out_row = a.task_out[t];
            if (a.task_scale) out_scale = a.task_scale[t];
        }
        const int32_t share = (end - beg + per - 1) / per;
        const int32_t wb = min(end, beg + wsh * share), we = min(end, wb + share);
        for (int c0 = 0; c0 < a.feat; c0 += LPR * VEC) {
            const int cbase = c0 + li * VEC;
            const bool act = !idle && cbase < a.feat;
            const int cstart = (VEC > 1 && cbase + VEC > a.feat) ? a.feat - VEC : cbase;   // see rof_rows_kernel
            const int skip = cbase - cstart;
            const char *xb = reinterpret_cast<const char *>(a.x) + (size_t)cstart * sizeof(XT);
            const char *pb = reinterpret_cast<const char *>(a.part) + (size_t)cstart * 4;
            float acc[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
            if (kF32) {
                if (mid > beg)   // the row references partial rows of shared groups
                    gather_sum<XT, VEC, LPR, true, true, true, false, kU>(xb, xld, pb, pld, a.nsplit, 0, a.col, a.w, wb, we, lane,
                                                                         sub, li, act, acc);
                else
                    gather_sum<XT, VEC, LPR, true, false, true, false, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, wb, we, lane,
                                                                          sub, li, act, acc);
            } else {   // bf16 features: the references (fp32 partial rows) come first in the row's list
                if (mid > wb)
                    gather_sum<float, VEC, LPR, true, false, true, false, kU>(pb, pld, nullptr, 0, 0, a.nsplit, a.col, a.w, wb,
                                                                             min(we, mid), lane, sub, li, act, acc);
                gather_sum<XT, VEC, LPR, true, false, true, false, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, max(wb, mid), we, lane,
                                                                      sub, li, act, acc);
            }
            if ((G & (G - 1)) == 0) {
#pragma unroll
                for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) acc[k] += __shfl_xor(acc[k], off);
                }
            } else {
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    float tot = acc[k];
#pragma unroll
                    for (int g = 1; g < G; ++g)
                        tot += __int_as_float(__builtin_amdgcn_ds_bpermute(lane_addr(li * 4, g * LPR * 4), __float_as_int(acc[k])));
                    acc[k] = tot;
                }
            }
            if (c0 > 0) __syncthreads();   // the previous chunk's sums have been read
            if (act && sub == 0) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) red[wid][li * VEC + k] = acc[k];
            }
            __syncthreads();
            if (wsh == 0 && have && act && sub == 0) {
                float tot[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) tot[k] = red[wid][li * VEC + k];
                for (int w = 1; w < per; ++w) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) tot[k] += red[wid + w][li * VEC + k];
                }
                finish_row<XT, VEC, PHASE>(a, out_row, out_scale, end > beg, tot, xb, xld, cstart, skip);
            }
        }
        return;
    }

    // the remaining tasks: a wavefront each while they are long, a lane group each after that
    const int hb = hw - coop_blocks;
    const int xcd = hb % kXcds, nth = hb / kXcds;
    const int run = a.xcd_run;
    const int logical = ((nth / run) * kXcds + xcd) * run + (nth % run);
    if (logical >= a.n_blocks) return;
    const int gw = n_coop + logical * kCoopWaves + wid;
    int32_t t, beg = 0, end = 0, mid = 0, out_row = 0;
    float out_scale = 1.0f;
    bool valid;
    const bool wave_mode = gw < a.n_wave;
    if (wave_mode) {
        t = gw;
        valid = true;
    } else {
        t = a.n_wave + (gw - a.n_wave) * G + sub;
        valid = !idle && t < a.n_tasks;
    }
    if (valid) {
        beg = a.task_ptr[t];
        end = a.task_ptr[t + 1];
        mid = beg + a.task_nref[t];
        out_row = a.task_out[t];
        if (a.task_scale) out_scale = a.task_scale[t];
    }
    for (int c0 = 0; c0 < a.feat; c0 += LPR * VEC) {
        const int cbase = c0 + li * VEC;
        const bool act = !idle && cbase < a.feat;
        const int cstart = (VEC > 1 && cbase + VEC > a.feat) ? a.feat - VEC : cbase;
        const int skip = cbase - cstart;
        const char *xb = reinterpret_cast<const char *>(a.x) + (size_t)cstart * sizeof(XT);
        const char *pb = reinterpret_cast<const char *>(a.part) + (size_t)cstart * 4;
        float acc[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
        if (wave_mode) {
            if (kF32) {
                if (mid > beg)
                    gather_sum<XT, VEC, LPR, true, true, true, false, kU>(xb, xld, pb, pld, a.nsplit, 0, a.col, a.w, beg, end, lane,
                                                                         sub, li, act, acc);
                else
                    gather_sum<XT, VEC, LPR, true, false, true, false, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, beg, end, lane,
                                                                          sub, li, act, acc);
            } else {
                if (mid > beg)
                    gather_sum<float, VEC, LPR, true, false, true, false, kU>(pb, pld, nullptr, 0, 0, a.nsplit, a.col, a.w, beg,
                                                                             mid, lane, sub, li, act, acc);
                gather_sum<XT, VEC, LPR, true, false, true, false, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, mid, end, lane, sub,
                                                                      li, act, acc);
            }
            if ((G & (G - 1)) == 0) {
#pragma unroll
                for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) acc[k] += __shfl_xor(acc[k], off);
                }
            } else {
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    float tot = acc[k];
#pragma unroll
                    for (int g = 1; g < G; ++g)
                        tot += __int_as_float(__builtin_amdgcn_ds_bpermute(lane_addr(li * 4, g * LPR * 4), __float_as_int(acc[k])));
                    acc[k] = tot;
                }
            }
        } else if (kF32) {
            if (__any(mid > beg))
                gather_sum<XT, VEC, LPR, false, true, true, false, kU>(xb, xld, pb, pld, a.nsplit, 0, a.col, a.w, beg, end, lane, sub,
                                                                      li, act, acc);
            else
                gather_sum<XT, VEC, LPR, false, false, true, false, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, beg, end, lane, sub,
                                                                       li, act, acc);
        } else {
            if (__any(mid > beg))
                gather_sum<float, VEC, LPR, false, false, true, false, kU>(pb, pld, nullptr, 0, 0, a.nsplit, a.col, a.w, beg, mid,
                                                                          lane, sub, li, act, acc);
            gather_sum<XT, VEC, LPR, false, false, true, false, kU>(xb, xld, nullptr, 0, 0, 0, a.col, a.w, mid, end, lane, sub, li,
                                                                   act, acc);
        }
        if (valid && act && (!wave_mode || sub == 0))
            finish_row<XT, VEC, PHASE>(a, out_row, out_scale, end > beg, acc, xb, xld, cstart, skip);
    }
}

// Lanes one gathered row occupies: the smallest supported count that covers ceil(feat / vec).  Counts
// that do not divide 64 (10, 12, 20) leave 4 lanes idle but fit 6, 5 or 3 rows into one load instruction
// where the next power of two would fit 4, 4 or 2.
inline int rof_lanes_per_row(int feat, int vec) {
    static const int kChoices[] = {4, 8, 10, 12, 16, 20, 32, 64};
    const int need = (feat + vec - 1) / vec;
    for (int c : kChoices)
        if (c >= need && (vec > 1 || (c & (c - 1)) == 0)) return c;   // the scalar fallback is built for powers of two
    return 64;
}

// Dynamic LDS one workgroup of a launch asks for: the rows of the workgroup-local groups of a cluster launch
// (`lds_rows` rows of lpr * vec columns plus 4 floats of padding; none: 0 bytes) on top of the benchmark interface's
// padding.  A cap on the wavefronts per SIMD (= workgroups of 4 wavefronts per CU) of an ordinary launch is put into
// effect by asking for so much unused LDS that no more workgroups fit into the CU's 160 KB.
constexpr int64_t kMaxLdsRequest = 64 * 1024;
inline int64_t lds_request(bool cluster, int lpr, int vec, int lds_rows, int wave_cap, int lds_pad, int64_t lds_per_cu) {
    int64_t lds = (int64_t)lds_pad + (cluster ? (int64_t)lds_rows * (lpr * vec + 4) * 4 : 0);
    // more than 1 / (cap + 1) of the CU's LDS per workgroup: cap + 1 workgroups no longer fit, cap still do
    // (a device whose CU had so little LDS that the request would exceed a workgroup's 64 KB runs uncapped)
    if (!cluster && wave_cap >= 2 && wave_cap < 8) {
        const int64_t want = ((lds_per_cu > 0 ? lds_per_cu : kLdsPerCu) / (wave_cap + 1) + 2048) / 2048 * 2048;
        if (want <= kMaxLdsRequest) lds = std::max<int64_t>(lds, want);
    }
    return lds;
}

// CLUSTER: a.n_blocks clusters (one workgroup each) that need `lds_rows` LDS rows; otherwise the tasks [0, n_tasks)
// of `a`, the first n_wave of them long.
template <typename XT, int VEC, int PHASE, bool OFF32, bool CLUSTER>
int launch_lpr(const AggArgs &a0, int lpr, int lds_rows, hipStream_t st) {
    AggArgs a = a0;
    const int g = 64 / lpr;
    if (!CLUSTER) {
        const int64_t shorts = (int64_t)a.n_tasks - a.n_wave;
        const int64_t waves = a.n_wave + (shorts + g - 1) / g;
        a.n_blocks = (int32_t)((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    }
    if (a.n_blocks == 0) return ROF_OK;
    const int64_t lds = lds_request(CLUSTER, lpr, VEC, lds_rows, a.wave_cap, a.lds_pad, a.lds_per_cu);
    if (lds > kMaxLdsRequest) return ROF_ERR_UNSUPPORTED;   // (aggregate_impl checks every launch before the first one)
    const int64_t span = (int64_t)kXcds * a.xcd_run;
    const int64_t grid = (a.n_blocks + span - 1) / span * span;
    dim3 gr((unsigned)grid), bl(64 * kWavesPerBlock);
#define ROF_LAUNCH(LPR)                                                                                              \
    do {                                                                                                             \
        if constexpr (CLUSTER)                                                                                       \
            hipLaunchKernelGGL((rof_cluster_kernel<XT, VEC, LPR, (PHASE == 2 ? 2 : 1), OFF32>), gr, bl, (unsigned)lds, st, a); \
        else                                                                                                         \
            hipLaunchKernelGGL((rof_rows_kernel<XT, VEC, LPR, PHASE, OFF32>), gr, bl, (unsigned)lds, st, a);         \
    } while (0)
    switch (lpr) {
        case 4: ROF_LAUNCH(4); break;
        case 8: ROF_LAUNCH(8); break;
        case 10:
            if constexpr (VEC > 1) ROF_LAUNCH(10);
            break;
        case 12:
            if constexpr (VEC > 1) ROF_LAUNCH(12);
            break;
        case 20:
            if constexpr (VEC > 1) ROF_LAUNCH(20);
            break;
        case 16: ROF_LAUNCH(16); break;
        case 32: ROF_LAUNCH(32); break;
        default: ROF_LAUNCH(64); break;
    }
#undef ROF_LAUNCH
    HIP_TRY(hipGetLastError());
    return ROF_OK;
}

template <typename XT, int VEC, bool DEEP>
int launch_coop(const AggArgs &a0, int lpr, const CoopSplit &cs, hipStream_t st) {
    AggArgs a = a0;
    const int g = 64 / lpr;
    const int32_t n_coop = cs.tasks();
    if (cs.n16 < 0 || cs.n8 < 0 || cs.n4 < 0 || n_coop > a.n_wave || a.n_wave > a.n_tasks) return ROF_ERR_ARG;
    const int64_t waves = (int64_t)(a.n_wave - n_coop) + ((int64_t)a.n_tasks - a.n_wave + g - 1) / g;
    a.n_blocks = (int32_t)((waves + kCoopWaves - 1) / kCoopWaves);
    a.xcd_run = std::max(1, a.xcd_run / (kCoopWaves / kWavesPerBlock));   // runs counted in workgroups four times as wide
    const int64_t span = (int64_t)kXcds * a.xcd_run;
    const int64_t grid = cs.blocks() + (a.n_blocks + span - 1) / span * span;
    if (grid == 0) return ROF_OK;
    dim3 gr((unsigned)grid), bl(64 * kCoopWaves);
#define ROF_LAUNCH(LPR) hipLaunchKernelGGL((rof_coop_kernel<XT, VEC, LPR, DEEP>), gr, bl, 0, st, a, cs)
    switch (lpr) {
        case 4: ROF_LAUNCH(4); break;
        case 8: ROF_LAUNCH(8); break;
        case 10: ROF_LAUNCH(10); break;
        case 12: ROF_LAUNCH(12); break;
        case 16: ROF_LAUNCH(16); break;
        case 20: ROF_LAUNCH(20); break;
        case 32: ROF_LAUNCH(32); break;
        default: ROF_LAUNCH(64); break;
    }
#undef ROF_LAUNCH
    HIP_TRY(hipGetLastError());
    return ROF_OK;
}

// Instantiated in agg_rows_{f32,bf16}_partial.hip (partial-sum launches; phase 0, 3 or 5 / stream: phase 3), agg_rows_{f32,bf16}_dst.hip (destination
// rows; phase 1, or 2 = streaming stores), agg_cluster_{f32,bf16}.hip (the clustered destination rows: a.n_blocks
// clusters whose workgroups need lds_rows LDS rows) and agg_coop_{f32,bf16}.hip (the destination rows of a small graph), one
// translation unit each so that the build runs them side by side.
// off32: every byte offset into the feature matrix and into the partial-sum workspace fits 32 bits and
// every row id fits 24 bits, so the kernels may use the short address arithmetic.
int launch_rows_f32_partial(const AggArgs &a, int phase, int vec, bool off32, hipStream_t st);
int launch_rows_f32_dst(const AggArgs &a, int phase, int vec, bool off32, hipStream_t st);
int launch_rows_f32_cluster(const AggArgs &a, int phase, int vec, bool off32, int lds_rows, hipStream_t st);
// agg_coop_{f32,bf16}.hip: the destination-row launch of a small graph whose first cs.tasks() tasks are summed by 16, 8
// or 4 wavefronts each (rof_coop_kernel; rows gathered as 16-byte vectors with short offsets); a.n_tasks: the tasks
// of this launch
int launch_rows_f32_coop(const AggArgs &a, bool deep, const CoopSplit &cs, hipStream_t st);
int launch_rows_bf16_coop(const AggArgs &a, const CoopSplit &cs, hipStream_t st);
int launch_rows_bf16_partial(const AggArgs &a, bool stream, int vec, bool off32, hipStream_t st);
int launch_rows_bf16_dst(const AggArgs &a, int phase, int vec, bool off32, hipStream_t st);
int launch_rows_bf16_cluster(const AggArgs &a, int phase, int vec, bool off32, int lds_rows, hipStream_t st);

// phase 0: partial-sum launches, 3: the same with streaming stores, 5: with more gathers in flight; 1: destination
// rows, 2: with streaming stores, 4: with more gathers in flight (5 and 4 exist for fp32 vector rows with short
// offsets and run as 0 and 1 otherwise); lds_rows > 0: the cluster launch of the destination rows
inline int launch_rows(bool bf16, const AggArgs &a, int phase, int vec, bool off32, int lds_rows, hipStream_t st) {
    if (phase == 0 || phase == 3 || phase == 5)
        return bf16 ? launch_rows_bf16_partial(a, phase == 3, vec, off32, st) : launch_rows_f32_partial(a, phase, vec, off32, st);
    if (lds_rows > 0)
        return bf16 ? launch_rows_bf16_cluster(a, phase == 2 ? 2 : 1, vec, off32, lds_rows, st)
                    : launch_rows_f32_cluster(a, phase == 2 ? 2 : 1, vec, off32, lds_rows, st);
    return bf16 ? launch_rows_bf16_dst(a, phase == 2 ? 2 : 1, vec, off32, st) : launch_rows_f32_dst(a, phase, vec, off32, st);
}

}  // namespace rofk

#endif
