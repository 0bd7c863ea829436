// gfx950 (CDNA4, wave64) kernels of the reuse-aware neighbour aggregation: C ABI, launch logic and the
// small helper kernels.  The row-gather kernels themselves are in agg_rows.h (instantiated in
// agg_rows_*_partial.hip, agg_rows_*_dst.hip and agg_cluster_*.hip).
//
// One kernel template does all the summing.  A *task* gathers a list of rows and writes their
// weighted sum to one output row:
//     out[task_out[t], :] = scale[t] * sum_i w[i] * row(col[i])        i in task_ptr[t] .. task_ptr[t+1]
// where row(c) is x[c, :] for c < nsplit and the partial-sum row part[c - nsplit, :] otherwise
// (the first task_nref[t] entries of a task are of the second kind).  Up to four launches in stream
// order: reuse groups that several destinations share -> partial-sum rows; segments of very long rows
// (which may read group rows) -> partial-sum rows; every destination row -> out; and, for destinations that the
// schedule has clustered around groups they share, one workgroup per cluster that sums those groups once into LDS
// before it gathers the cluster's rows (rof_cluster_kernel).  There are no atomics: each output row has one writer.
// On a small graph the layout keeps long rows whole instead of cutting them into segments, and the destination-row
// launch is rof_coop_kernel: workgroups of sixteen wavefronts, the first of which sum one, two or four long rows
// each (the sums of a row's wavefronts meet in LDS),
// the others running the remaining tasks as below -- one launch where segments would need two.
//
// Mapping to the machine:
//   * the feature dimension runs across lanes, VEC consecutive elements per lane (one 16-byte
//     load), LPR lanes per row (4, 8, 10, 12, 16, 20, 32 or 64), so a wavefront gathers G = 64/LPR rows
//     per load instruction and a row is read as one contiguous burst; rows may be packed: the loads
//     only need 4-byte alignment and the last lane of a row is shifted back instead of reading past it;
//   * long tasks get a whole wavefront: its G lane groups take every G-th entry and are combined
//     at the end by a cross-lane butterfly (__shfl_xor -> DPP / ds_swizzle class instructions);
//   * short tasks are packed G to a wavefront, one lane group each; they are pre-sorted by length
//     so the groups of one wavefront finish together;
//   * column ids and weights are fetched coalesced, one per lane, and handed to the lane groups
//     with ds_bpermute, so the only per-entry memory instruction is the row gather itself;
//   * workgroups are renumbered so that each XCD (own L2) works on runs of consecutive tasks;
//   * the store of a destination row can apply the rest of the layer -- the node's own row times a factor,
//     a bias, ReLU, rounding to bf16 (rof_aggregate_epilogue) -- instead of separate passes over the output.
// MFMA is not used: there is no dense contraction here, only gather + add, bounded by HBM.
//
// Reference semantics: ROF/reuse_conv/reuse_conv_kernel.cu:205-286 (GNNA), 396-601 (v1),
// 836-954 (v2 fused), 123-196 (SAG).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <atomic>
#include <mutex>
#include <new>
#include <vector>

#include "agg_rows.h"
#include "rof.h"
#include "rof_bench.h"
#include "rof_internal.h"

using rofk::AggArgs;

namespace {

thread_local char g_dev_err[256] = "";

// An output of this size or more is written with streaming stores: it would not survive in the 256 MB Infinity
// Cache until its consumer runs anyway, and written normally it evicts the feature rows the gathers re-read.
// Measured on MI355X (outputs of 268 MB): block-structured graph -9 %, R-MAT 2^18 x 256 floats -2.5 %; packed
// 47-float rows (2.4 M of them, stored as 16-byte pieces at dword alignment) -1.8 %.  Rows whose pieces cannot be
// stored whole (scalar instantiation, bf16 rows of odd stride) keep ordinary stores: streamed element by element
// they were 17 % slower.
constexpr int64_t kStreamOutBytes = 128 << 20;
// Partial rows of one launch beyond this many bytes are written as streaming stores: the destination rows read them
// only after the launch has ended, by which time rows of a workspace this large have left the caches anyway, and
// until then they would take the place of feature rows there.  (Below it the partial rows are still in L2 when
// they are read: streaming them costs time.)
constexpr int64_t kStreamPartialBytes = 64 << 20;

// Wavefronts per SIMD of the destination-row launch.  On a heavy-tailed graph whose feature matrix is far larger
// than the L2s, the launch mixes gathers of hub rows, which hit, with gathers that miss, and the miss path of a CU
// slows down when too many lines are asked for at once: with two row gathers in flight per lane group, rows of up
// to 64 bytes (16 rows per wavefront) run best at 6 wavefronts per SIMD, rows of two 128-byte lines (129-256 bytes)
// at 7 (6 when their stride lets them straddle a third line), all others with every slot taken.  Measured on the 2.4 M-node R-MAT graph (destination-row launch at 8 / 7 /
// 6 wavefronts): 16 floats 570 / 558 / 549 us, 32 floats 570 / 581 / 600, 47 floats 972 / 922 / 934, 64 floats
// 982 / 931 / 938, 100 floats 1052 / 1086 / 1144.  Every other case loses 2-10 % per slot given up: matrices that
// the caches serve (2^18 nodes x 40 floats; the block model, whose rows gather from their own neighbourhood), the
// partial-sum launches, and graphs without hub rows (uniform degrees, 2^20 nodes x 64 floats: 689 / 700 us).  The
// layout knows the latter by having no segmented rows.
constexpr int64_t kServedMatrixBytes = 96 << 20;
constexpr int64_t kLatencyBoundGatherBytes = (int64_t)8 << 30;
constexpr int64_t kColdMatrixBytes = 128 << 20;   // 4x the L2 of the eight XCDs; the 42 MB matrix above is served, the 154 MB one (16 floats) is not
int dst_wave_cap(const rof_layout *L, int64_t matrix_bytes, int64_t row_bytes, int64_t stride_bytes) {
    if (L->local_sources || L->n_segments == 0 || matrix_bytes < kColdMatrixBytes) return 0;
    if (row_bytes <= 64) return 6;
    // packed rows (47 floats 188 bytes apart) straddle a third line in 44 % of the cases: 1488 / 1448 / 1494 us per
    // layer at 7 / 6 / 5 wavefronts, against 1257 / 1288 / 1371 for the same rows 192 bytes apart
    if (row_bytes > 128 && row_bytes <= 256) return stride_bytes % 64 == 0 ? 7 : 6;
    return 0;
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

// plain streaming read (every 16-byte piece once, grid-stride); the sums go to `sink` only so that the loads cannot be
// dropped.  Gives the read rate the memory side sustains, against which gather traffic is put.  (Measured shapes on
// MI355X: 2048 workgroups of 256 lanes with one load per lane and trip reach 6.5 TB/s from HBM and 6.8-6.9 TB/s from
// the Infinity Cache; unrolling to 2 ... 8 loads in flight per lane or 8192 / 32768 workgroups: 5.4-5.9 and 6.4-6.7.)
__global__ __launch_bounds__(256) void rof_read_kernel(const float4 *__restrict__ src, int64_t n16, int repeat,
                                                       float *__restrict__ sink) {
    const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    float a = 0.f;
    for (int r = 0; r < repeat; ++r) {   // repeat > 1: the same buffer again (a buffer small enough stays in L2)
#pragma unroll 1
        for (int64_t i = first; i < n16; i += stride) {
            const float4 p = src[i];
            a += p.x + p.y + p.z + p.w;
        }
    }
    if (a == 1.2345e-30f) sink[0] = a;   // practically never true; keeps the loads alive
}

// nothing but row gathers: every lane group of LPR lanes fetches pseudo-random rows of LPR * 16 bytes from a table of
// rows_mask + 1 rows, two in flight, and adds them up.  The rate it reaches from a table that the L2s hold, that the
// Infinity Cache holds, or that only HBM holds is the yardstick for the aggregation launches, whose gathers are of
// exactly this shape (plus indices, weights and stores).
template <int LPR>
__global__ __launch_bounds__(256) void rof_gather_kernel(const char *__restrict__ table, uint32_t rows_mask, int iters,
                                                         float *__restrict__ sink) {
    const int lane = threadIdx.x & 63, sub = lane / LPR, li = lane % LPR;
    if (lane >= (64 / LPR) * LPR) return;   // lanes left over when LPR does not divide 64
    uint32_t s = (blockIdx.x * 256u + (threadIdx.x & ~63u)) * 2654435761u + sub * 40503u + 12345u;
    float a = 0.f;
    for (int it = 0; it < iters; ++it) {
        s = s * 1664525u + 1013904223u;
        const uint32_t r0 = (s >> 8) & rows_mask;
        s = s * 1664525u + 1013904223u;
        const uint32_t r1 = (s >> 8) & rows_mask;
        const rofk::rof_f4 p = *reinterpret_cast<const rofk::rof_f4 *>(table + (size_t)r0 * (LPR * 16) + li * 16);
        const rofk::rof_f4 q = *reinterpret_cast<const rofk::rof_f4 *>(table + (size_t)r1 * (LPR * 16) + li * 16);
        a += (p.x + p.y + p.z + p.w) + (q.x + q.y + q.z + q.w);
    }
    if (a == 1.2345e-30f) sink[0] = a;   // practically never true; keeps the loads alive
}

// Column sums of a row-major [n, f] matrix (the bias gradient of a layer), in two launches with a fixed
// order of summation.  A workgroup owns a run of rows; its four wavefronts take every fourth row of the run,
// 64 lanes across 64 consecutive columns, so each load instruction reads one contiguous piece of a row.
constexpr int kColsumBlocks = 2048;

template <typename XT>
__device__ __forceinline__ float colsum_load(const XT *p);
template <>
__device__ __forceinline__ float colsum_load<float>(const float *p) { return *p; }
template <>
__device__ __forceinline__ float colsum_load<uint16_t>(const uint16_t *p) { return __uint_as_float(((uint32_t)*p) << 16); }

template <typename XT>
__global__ __launch_bounds__(256) void rof_colsum_partial_kernel(const XT *__restrict__ x, int64_t ldx, int64_t n, int f,
                                                                  int64_t rows_per_block, float *__restrict__ partial) {
    __shared__ float red[4][64];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    for (int c0 = 0; c0 < f; c0 += 64) {
        const int c = c0 + tx;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        if (c < f) {
            const XT *p = x + c;
            int64_t r = r0 + ty;
            for (; r + 12 < r1; r += 16) {   // four independent loads in flight per lane
                a0 += colsum_load<XT>(p + r * ldx);
                a1 += colsum_load<XT>(p + (r + 4) * ldx);
                a2 += colsum_load<XT>(p + (r + 8) * ldx);
                a3 += colsum_load<XT>(p + (r + 12) * ldx);
            }
            for (; r < r1; r += 4) a0 += colsum_load<XT>(p + r * ldx);
        }
        red[ty][tx] = (a0 + a1) + (a2 + a3);
        __syncthreads();
        if (ty == 0 && c < f) partial[(int64_t)blockIdx.x * f + c] = (red[0][tx] + red[1][tx]) + (red[2][tx] + red[3][tx]);
        __syncthreads();
    }
}

__global__ __launch_bounds__(1024) void rof_colsum_final_kernel(const float *__restrict__ partial, int blocks, int f,
                                                                 float *__restrict__ out) {
    __shared__ float red[16][64];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;   // 64 columns x 16 slices of the partial rows
    const int c = blockIdx.x * 64 + tx;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (c < f) {
        int b = ty;
        for (; b + 48 < blocks; b += 64) {
            a0 += partial[(int64_t)b * f + c];
            a1 += partial[(int64_t)(b + 16) * f + c];
            a2 += partial[(int64_t)(b + 32) * f + c];
            a3 += partial[(int64_t)(b + 48) * f + c];
        }
        for (; b < blocks; b += 16) a0 += partial[(int64_t)b * f + c];
    }
    red[ty][tx] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (ty == 0 && c < f) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc += red[i][tx];
        out[c] = acc;
    }
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
    if (h.task_nlds.empty()) {
        if ((rc = put(&d.task_nref, h.task_nref))) return rc;
    } else {
        // the kernel reads one word per task: references in the low 24 bits, LDS rows above
        std::vector<int32_t> packed(h.task_nref.size());
        for (size_t i = 0; i < packed.size(); ++i) {
            if (h.task_nref[i] >= (1 << 24) || h.task_nlds[i] >= 128) return ROF_ERR_UNSUPPORTED;
            packed[i] = (int32_t)((uint32_t)h.task_nref[i] | ((uint32_t)h.task_nlds[i] << 24));
        }
        if ((rc = put(&d.task_nref, packed))) return rc;
        HIP_TRY(hipStreamSynchronize(st));   // `packed` goes out of scope
    }
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
    d.n_regular = h.lg_blocks > 0 ? h.n_regular : h.n_tasks;
    d.lg_blocks = h.lg_blocks;
    d.lg_max_rows = h.lg_max_rows;
    d.lg_entries = (int64_t)h.lg_col.size();
    if (h.lg_blocks > 0) {
        if ((rc = put(&d.lg_task_first, h.lg_task_first))) return rc;
        if ((rc = put(&d.lg_ptr, h.lg_ptr))) return rc;
        if ((rc = put(&d.lg_task_ptr, h.lg_task_ptr))) return rc;
        if ((rc = put(&d.lg_col, h.lg_col))) return rc;
        size_t lb = (h.lg_col.size() ? h.lg_col.size() : 1) * sizeof(float);
        HIP_TRY(hipMalloc((void **)&d.lg_w, lb));
        *bytes += (int64_t)lb;
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
    if (d.lg_ptr) (void)hipFree(d.lg_ptr);
    if (d.lg_task_first) (void)hipFree(d.lg_task_first);
    if (d.lg_task_ptr) (void)hipFree(d.lg_task_ptr);
    if (d.lg_col) (void)hipFree(d.lg_col);
    if (d.lg_w) (void)hipFree(d.lg_w);
    d = rof_phase_dev();
}

inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

// Partial-sum rows of rof_aggregate_noalloc: device memory that belongs to the library's code object, so a
// caller that may not allocate (HIP graph capture, a serving loop) does not have to bring a workspace.  Each
// GPU the library runs on holds its own copy, at its own address, until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; the address it returns for the current device is what
// kernels and copies are given.
constexpr size_t kScratchBytes = ROF_NOALLOC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mu;

// Address of `scratch` on the current device, looked up once per device.
int scratch_of_current_device(void **out) {
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return ROF_ERR_UNSUPPORTED;
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(g_scratch_mu);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            if (!p) return ROF_ERR_DEVICE;
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return ROF_OK;
}

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

int rof_version(void) { return ROF_ABI_VERSION; }

// Launch tuning of one layout, used by the benchmark sweeps.
int rof_layout_set_tuning(rof_layout *L, const rof_launch_tuning *t) {
    if (!L || !t) return ROF_ERR_ARG;
    if (t->xcd_run_partial < 0 || t->xcd_run_dst < 0 || t->xcd_run_partial > 4096 || t->xcd_run_dst > 4096) return ROF_ERR_ARG;
    if (t->wave_cap < -1 || t->wave_cap == 1 || t->wave_cap > 7) return ROF_ERR_ARG;
    if (t->lds_pad < 0 || t->lds_pad > 64 * 1024) return ROF_ERR_ARG;
    if (t->deep < -1 || t->deep > 1) return ROF_ERR_ARG;
    L->tune_xcd_run_partial = t->xcd_run_partial;
    L->tune_xcd_run_dst = t->xcd_run_dst;
    L->tune_wave_cap = t->wave_cap;
    L->tune_lds_pad = t->lds_pad;
    L->tune_deep = t->deep;
    return ROF_OK;
}

int rof_layout_get_tuning(const rof_layout *L, rof_launch_tuning *t) {
    if (!L || !t) return ROF_ERR_ARG;
    memset(t, 0, sizeof(*t));
    t->xcd_run_partial = L->tune_xcd_run_partial;
    t->xcd_run_dst = L->tune_xcd_run_dst;
    t->wave_cap = L->tune_wave_cap;
    t->lds_pad = L->tune_lds_pad;
    t->deep = L->tune_deep;
    return ROF_OK;
}

size_t rof_column_sums_workspace_bytes(int64_t n, int f) {
    if (n <= 0 || f <= 0) return 0;
    return (size_t)kColsumBlocks * (size_t)f * sizeof(float);
}

int rof_column_sums(const void *x, int x_dtype, int64_t ldx, int64_t n, int f, float *out, void *workspace,
                    size_t workspace_bytes, void *stream) {
    if (!out || n < 0 || f < 1 || ldx < f || (n && !x)) return ROF_ERR_ARG;
    if (x_dtype != ROF_F32 && x_dtype != ROF_BF16) return ROF_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < rof_column_sums_workspace_bytes(n > 0 ? n : 1, f)) return ROF_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    const int64_t want = (n + 63) / 64;   // at least 64 rows per workgroup
    const int blocks = (int)(want < 1 ? 1 : (want > kColsumBlocks ? kColsumBlocks : want));
    const int64_t rows_per_block = n ? (n + blocks - 1) / blocks : 0;
    float *partial = (float *)workspace;
    if (x_dtype == ROF_F32)
        hipLaunchKernelGGL(rof_colsum_partial_kernel<float>, dim3(blocks), dim3(256), 0, st, (const float *)x, ldx, n, f,
                           rows_per_block, partial);
    else
        hipLaunchKernelGGL(rof_colsum_partial_kernel<uint16_t>, dim3(blocks), dim3(256), 0, st, (const uint16_t *)x, ldx,
                           n, f, rows_per_block, partial);
    HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(rof_colsum_final_kernel, dim3((f + 63) / 64), dim3(1024), 0, st, partial, blocks, f, out);
    HIP_TRY(hipGetLastError());
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

int rof_device_read(const void *src, size_t nbytes, int repeat, float *sink, void *stream) {
    if (!src || !sink || repeat < 1 || (nbytes & 15) || ((uintptr_t)src & 15)) return ROF_ERR_ARG;
    if (nbytes == 0) return ROF_OK;
    hipLaunchKernelGGL(rof_read_kernel, dim3(2048), dim3(256), 0, (hipStream_t)stream, (const float4 *)src,
                       (int64_t)(nbytes / 16), repeat, sink);
    HIP_TRY(hipGetLastError());
    return ROF_OK;
}

int rof_device_gather(const void *table, uint32_t rows, int lanes_per_row, int iters, float *sink, void *stream,
                      uint64_t *gathered_rows) {
    if (!table || !sink || iters < 1 || rows == 0 || (rows & (rows - 1)) || ((uintptr_t)table & 15)) return ROF_ERR_ARG;
    const dim3 grid(256 * 32), block(256);
    hipStream_t st = (hipStream_t)stream;
    switch (lanes_per_row) {
        case 4: hipLaunchKernelGGL(rof_gather_kernel<4>, grid, block, 0, st, (const char *)table, rows - 1, iters, sink); break;
        case 8: hipLaunchKernelGGL(rof_gather_kernel<8>, grid, block, 0, st, (const char *)table, rows - 1, iters, sink); break;
        case 10: hipLaunchKernelGGL(rof_gather_kernel<10>, grid, block, 0, st, (const char *)table, rows - 1, iters, sink); break;
        case 12: hipLaunchKernelGGL(rof_gather_kernel<12>, grid, block, 0, st, (const char *)table, rows - 1, iters, sink); break;
        case 16: hipLaunchKernelGGL(rof_gather_kernel<16>, grid, block, 0, st, (const char *)table, rows - 1, iters, sink); break;
        case 20: hipLaunchKernelGGL(rof_gather_kernel<20>, grid, block, 0, st, (const char *)table, rows - 1, iters, sink); break;
        case 32: hipLaunchKernelGGL(rof_gather_kernel<32>, grid, block, 0, st, (const char *)table, rows - 1, iters, sink); break;
        case 64: hipLaunchKernelGGL(rof_gather_kernel<64>, grid, block, 0, st, (const char *)table, rows - 1, iters, sink); break;
        default: return ROF_ERR_UNSUPPORTED;
    }
    HIP_TRY(hipGetLastError());
    if (gathered_rows) *gathered_rows = (uint64_t)grid.x * 4 * (64 / lanes_per_row) * 2 * (uint64_t)iters;
    return ROF_OK;
}

int rof_layout_upload(rof_layout *L, void *stream) {
    if (!L) return ROF_ERR_ARG;
    if (L->uploaded) return ROF_OK;
    hipStream_t st = (hipStream_t)stream;
    HIP_TRY(hipGetDevice(&L->device));
    int lds_per_cu = 0;   // what an occupancy cap by LDS request has to be measured against
    if (hipDeviceGetAttribute(&lds_per_cu, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, L->device) == hipSuccess)
        L->lds_per_cu = lds_per_cu;
    int rc;
    if ((rc = upload_phase(L->g, L->dg, false, st, &L->device_bytes)) ||
        (rc = upload_phase(L->s, L->ds, false, st, &L->device_bytes)) ||
        (rc = upload_phase(L->b, L->db, true, st, &L->device_bytes))) {
        free_phase(L->dg);   // nothing half-uploaded is kept
        free_phase(L->ds);
        free_phase(L->db);
        L->device_bytes = 0;
        return rc;
    }
    HIP_TRY(hipStreamSynchronize(st));   // the host vectors may be released after this call
    L->uploaded = true;
    // set-up is also where this device's copy of the static scratch gets its address; best effort here, because a
    // caller who never uses rof_aggregate_noalloc must not see its failures (that entry point reports them itself)
    void *unused = nullptr;
    (void)scratch_of_current_device(&unused);
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
    if (L->db.lg_entries)
        hipLaunchKernelGGL(rof_entry_weights_kernel, dim3((unsigned)((L->db.lg_entries + tb - 1) / tb)), dim3(tb), 0, st,
                           L->db.lg_col, L->db.lg_entries, deg, L->n, L->db.lg_w);
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

static int aggregate_impl(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                          int feat, int normalized, void *workspace, size_t workspace_bytes, void *stream,
                          int launches, const float *bias = nullptr, int relu = 0, int out_dtype = ROF_F32,
                          float self_weight = 0.0f, int pad_columns = 0) {
    if (!L || !x || !out || feat < 1 || ldx < feat || ldo < feat) return ROF_ERR_ARG;
    if (x_dtype != ROF_F32 && x_dtype != ROF_BF16) return ROF_ERR_UNSUPPORTED;
    if (out_dtype != ROF_F32 && out_dtype != ROF_BF16) return ROF_ERR_UNSUPPORTED;
    if (((uintptr_t)out) % (out_dtype == ROF_F32 ? 4 : 2)) return ROF_ERR_ARG;
    if (((uintptr_t)x) % (x_dtype == ROF_F32 ? 4 : 2) || ((uintptr_t)bias) % 4) return ROF_ERR_ARG;   // whole elements
    if (!L->uploaded || (normalized && !L->weights_set)) return ROF_ERR_STATE;
    if ((int64_t)L->n * ldx >= ((int64_t)1 << 40) || (int64_t)L->n * ldo >= ((int64_t)1 << 40)) return ROF_ERR_UNSUPPORTED;
    if (ldx >= ((int64_t)1 << 28) || feat >= (1 << 24)) return ROF_ERR_UNSUPPORTED;   // the kernel keeps row bytes in 32 bits
    int device = -1;
    HIP_TRY(hipGetDevice(&device));
    if (device != L->device) return ROF_ERR_STATE;   // the schedule lives on the device it was uploaded to
    const size_t need = rof_layout_workspace_bytes(L, feat);
    if (need && (!workspace || workspace_bytes < need)) return ROF_ERR_WORKSPACE;
    if (need && ((uintptr_t)workspace & 15)) return ROF_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;

    const int esz = x_dtype == ROF_F32 ? 4 : 2;
    const int wide = x_dtype == ROF_F32 ? 4 : 8;
    // 16-byte gathers need rows that start on a 4-byte boundary and hold at least one full vector
    const bool dword_rows = (((uintptr_t)x) % 4 == 0) && ((ldx * esz) % 4 == 0);
    const int vec = (dword_rows && feat >= wide) ? wide : 1;
    if (pad_columns && vec > 1 && feat % wide) {   // the caller lets the rows be taken as whole vectors
        const int padded = (int)round_up(feat, wide);
        if (ldx < padded || ldo < padded) return ROF_ERR_ARG;
        feat = padded;   // the workspace rows are round_up(feat, 8) floats wide either way
    }
    const int64_t ldp = round_up(feat, 8);
    const int64_t rows_x = L->n, rows_p = L->n_slots;
    const bool off32 = rows_x < (1 << 24) && rows_p < (1 << 24) && ldx * esz < (1 << 24) && ldp * 4 < (1 << 24) &&
                       (rows_x + 1) * ldx * esz < ((int64_t)1 << 32) && (rows_p + 1) * ldp * 4 < ((int64_t)1 << 32);

    // every launch of the call is checked before the first one is enqueued, so that a refusal leaves `out` untouched
    {
        const int lpr = rofk::rof_lanes_per_row(feat, vec);
        const int cap = L->tune_wave_cap >= 0 ? L->tune_wave_cap
                                              : dst_wave_cap(L, (int64_t)L->n * ldx * esz, (int64_t)feat * esz, ldx * esz);
        const int64_t plain_lds = rofk::lds_request(false, lpr, vec, 0, cap, L->tune_lds_pad, L->lds_per_cu);
        const int64_t cluster_lds = L->db.lg_blocks > 0
                                        ? rofk::lds_request(true, lpr, vec, L->db.lg_max_rows, 0, L->tune_lds_pad, L->lds_per_cu) : 0;
        if (plain_lds > rofk::kMaxLdsRequest || cluster_lds > rofk::kMaxLdsRequest) {
            rof_set_device_error("rof_aggregate", "the LDS rows of the layout's clusters do not fit a workgroup's 64 KB at this "
                                                  "feature width; build the layout for this width (lanes_per_row, elem_bytes)");
            return ROF_ERR_UNSUPPORTED;
        }
    }
    AggArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x;
    a.ldx = ldx;
    a.part = (const float *)workspace;
    a.ldp = ldp;
    a.nsplit = L->n;
    a.feat = feat;
    a.lds_pad = L->tune_lds_pad;
    a.lds_per_cu = L->lds_per_cu;
    int rc;
    // a feature matrix that the caches serve: more row gathers in flight in every launch (fp32 rows).  2^18-node
    // R-MAT graph against two in flight: 42 MB -8 %, 67 MB -7 %, 84 MB -2.8 %, 105 MB 0, 126 MB +1.9 %.
    // That is a gain of launches bound by latency; a dense graph on a small matrix keeps the caches busy instead, and
    // two in flight are as good or better from 8 GB gathered per launch (R-MAT, 233 000 nodes x 72 floats, average
    // degree 435, 29 GB: 2.02 ms with four, 1.85 with two; 2^16 nodes x 160 floats, degree 341, 14 GB: 0.712 / 0.689;
    // uniform degrees of 600: equal; below 8 GB four win by 1-20 %).
    const bool deep = x_dtype == ROF_F32 &&
                      (L->tune_deep >= 0 ? L->tune_deep == 1
                                         : (int64_t)L->n * ldx * esz < kServedMatrixBytes &&
                                               L->gathered_rows * (int64_t)feat * esz < kLatencyBoundGatherBytes);
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
        a.xcd_run = L->tune_xcd_run_partial > 0 ? L->tune_xcd_run_partial : 1;
        a.vec_store = 1;
        const int phase = (int64_t)d.n_tasks * feat * 4 >= kStreamPartialBytes && vec > 1 ? 3 : deep ? 5 : 0;
        if ((rc = rofk::launch_rows(x_dtype != ROF_F32, a, phase, vec, off32, 0, st))) return rc;
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
        a.xcd_run = L->tune_xcd_run_dst > 0 ? L->tune_xcd_run_dst : L->xcd_run;
        a.out_bf16 = out_dtype == ROF_BF16;
        a.vec_store = ((uintptr_t)out) % 4 == 0;   // pieces of a row are stored whole wherever they start on a dword
        a.bias = bias;
        a.relu = relu ? 1 : 0;
        a.self_weight = self_weight;
        a.lg_task_first = L->db.lg_task_first;
        a.lg_ptr = L->db.lg_ptr;
        a.lg_task_ptr = L->db.lg_task_ptr;
        a.lg_col = L->db.lg_col;
        a.lg_w = normalized ? L->db.lg_w : nullptr;
        const int phase = ((int64_t)L->n * feat * (a.out_bf16 ? 2 : 4) >= kStreamOutBytes && a.vec_store && vec > 1 &&
                           (!a.out_bf16 || ldo % 2 == 0)) ? 2 : deep ? 4 : 1;
        a.n_tasks = L->db.n_regular;   // the clustered destinations at the end of the list have a launch of their own
        a.wave_cap = L->tune_wave_cap >= 0 ? L->tune_wave_cap
                                           : dst_wave_cap(L, (int64_t)L->n * ldx * esz, (int64_t)feat * esz, ldx * esz);
        // a small graph whose layout keeps long rows whole: one launch in which a workgroup of 16 wavefronts sums each
        // of them (the kernel exists for rows gathered as 16-byte vectors with short offsets; any other call runs the
        // ordinary kernel, which sums such a row with one wavefront)
        if (L->coop_tasks > 0 && vec == wide && off32 && phase != 2) {
            const rofk::CoopSplit cs = {L->coop16, L->coop8, L->coop_tasks - L->coop16 - L->coop8};
            rc = x_dtype == ROF_F32 ? rofk::launch_rows_f32_coop(a, phase == 4, cs, st) : rofk::launch_rows_bf16_coop(a, cs, st);
        } else
        {
            rc = rofk::launch_rows(x_dtype != ROF_F32, a, phase, vec, off32, 0, st);
        }
        if (rc) return rc;
        a.wave_cap = 0;
        if (L->db.lg_blocks > 0) {
            a.n_tasks = L->db.n_tasks;
            a.n_blocks = L->db.lg_blocks;
            a.xcd_run = 1;
            if ((rc = rofk::launch_rows(x_dtype != ROF_F32, a, phase, vec, off32, L->db.lg_max_rows, st))) return rc;
        }
    }
    return ROF_OK;
}

int rof_aggregate(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, float *out, int64_t ldo, int feat,
                  int normalized, void *workspace, size_t workspace_bytes, void *stream) {
    return aggregate_impl(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, stream, 3);
}

int rof_aggregate_epilogue(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                           int feat, int normalized, const rof_epilogue *ep, void *workspace, size_t workspace_bytes,
                           void *stream) {
    if (!ep) return aggregate_impl(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, stream, 3);
    if (!(ep->self_weight == ep->self_weight)) return ROF_ERR_ARG;   // NaN
    return aggregate_impl(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, stream, 3,
                          ep->bias, ep->relu, ep->out_dtype, ep->self_weight, ep->pad_columns);
}

int rof_aggregate_noalloc(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                          int feat, int normalized, const rof_epilogue *ep, void *stream) {
    if (!L || feat < 1) return ROF_ERR_ARG;
    const size_t need = rof_layout_workspace_bytes(L, feat);
    if (need > kScratchBytes) {
        rof_set_device_error("rof_aggregate_noalloc",
                             "the layout's partial-sum rows exceed ROF_NOALLOC_WORKSPACE_BYTES; use rof_aggregate "
                             "with a caller-allocated workspace");
        return ROF_ERR_WORKSPACE;
    }
    void *ws = nullptr;
    int rc = scratch_of_current_device(&ws);
    if (rc) return rc;
    // every partial row a launch reads was written earlier in the same call, so nothing has to be cleared
    return rof_aggregate_epilogue(L, x, x_dtype, ldx, out, ldo, feat, normalized, ep, ws, kScratchBytes, stream);
}

static int aggregate_with(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo, int feat,
                          int normalized, const rof_epilogue *ep, void *workspace, size_t workspace_bytes, void *stream,
                          int launches) {
    if (!ep) return aggregate_impl(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, stream, launches);
    if (!(ep->self_weight == ep->self_weight)) return ROF_ERR_ARG;   // NaN
    return aggregate_impl(L, x, x_dtype, ldx, out, ldo, feat, normalized, workspace, workspace_bytes, stream, launches,
                          ep->bias, ep->relu, ep->out_dtype, ep->self_weight, ep->pad_columns);
}

namespace {
// HIP events that are destroyed on every exit path
struct EventSet {
    hipEvent_t ev[3] = {nullptr, nullptr, nullptr};
    int n = 0;
    int create(int count) {
        for (; n < count; ++n) HIP_TRY(hipEventCreate(&ev[n]));
        return ROF_OK;
    }
    ~EventSet() {
        for (int i = 0; i < n; ++i) (void)hipEventDestroy(ev[i]);
    }
};
}  // namespace

int rof_aggregate_timed(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                        int feat, int normalized, const rof_epilogue *ep, void *workspace, size_t workspace_bytes,
                        void *stream, int iters, float *ms_per_call) {
    if (!ms_per_call || iters < 1) return ROF_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    EventSet e;
    int rc = e.create(2);
    if (rc) return rc;
    HIP_TRY(hipEventRecord(e.ev[0], st));
    for (int i = 0; i < iters && rc == ROF_OK; ++i)
        rc = aggregate_with(L, x, x_dtype, ldx, out, ldo, feat, normalized, ep, workspace, workspace_bytes, st, 3);
    HIP_TRY(hipEventRecord(e.ev[1], st));
    HIP_TRY(hipEventSynchronize(e.ev[1]));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, e.ev[0], e.ev[1]));
    *ms_per_call = ms / iters;
    return rc;
}

int rof_layout_calibrate(rof_layout *L, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo, int feat,
                         int normalized, const rof_epilogue *ep, void *workspace, size_t workspace_bytes, void *stream,
                         int rounds, int iters, rof_launch_tuning *chosen) {
    if (!L || rounds < 1 || iters < 1) return ROF_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    EventSet e;
    int rc = e.create(2);
    if (rc) return rc;
    // one timing of the whole call under the layout's current settings; < 0: failed
    auto timed = [&](float *ms) -> int {
        float best = -1.f;
        for (int r = 0; r < rounds; ++r) {
            HIP_TRY(hipEventRecord(e.ev[0], st));
            int status = ROF_OK;
            for (int i = 0; i < iters && status == ROF_OK; ++i)
                status = aggregate_with(L, x, x_dtype, ldx, out, ldo, feat, normalized, ep, workspace, workspace_bytes, st, 3);
            HIP_TRY(hipEventRecord(e.ev[1], st));
            HIP_TRY(hipEventSynchronize(e.ev[1]));
            if (status != ROF_OK) return status;
            float t = 0.f;
            HIP_TRY(hipEventElapsedTime(&t, e.ev[0], e.ev[1]));
            if (best < 0.f || t < best) best = t;
        }
        *ms = best / iters;
        return ROF_OK;
    };
    const rof_launch_tuning before = {L->tune_xcd_run_partial, L->tune_xcd_run_dst, L->tune_wave_cap, L->tune_lds_pad,
                                      L->tune_deep, {0, 0, 0}};
    float t = 0.f;
    if ((rc = aggregate_with(L, x, x_dtype, ldx, out, ldo, feat, normalized, ep, workspace, workspace_bytes, st, 3)) ||
        (rc = timed(&t))) {   // warm-up, then the settings the size rules give
        return rc;
    }
    float best = t;
    // one setting after the other; a candidate replaces the incumbent only if it is measurably faster (1 %)
    auto sweep = [&](int32_t *field, const int32_t *values, int count) -> int {
        int32_t keep = *field;
        for (int i = 0; i < count; ++i) {
            if (values[i] == keep) continue;
            *field = values[i];
            float ms = 0.f;
            int status = timed(&ms);
            if (status == ROF_ERR_UNSUPPORTED) continue;   // e.g. a cap whose LDS request does not fit beside the padding
            if (status != ROF_OK) {
                *field = keep;
                return status;
            }
            if (ms < best * 0.99f) {
                best = ms;
                keep = values[i];
            }
        }
        *field = keep;
        return ROF_OK;
    };
    const int32_t caps[] = {0, 7, 6}, deeps[] = {0, 1}, runs[] = {4, 16, 256, L->xcd_run};
    if ((rc = sweep(&L->tune_wave_cap, caps, 3)) || (x_dtype == ROF_F32 && (rc = sweep(&L->tune_deep, deeps, 2))) ||
        (rc = sweep(&L->tune_xcd_run_dst, runs, 4))) {
        L->tune_wave_cap = before.wave_cap;
        L->tune_deep = before.deep;
        L->tune_xcd_run_dst = before.xcd_run_dst;
        return rc;
    }
    if (chosen) rof_layout_get_tuning(L, chosen);
    return ROF_OK;
}

int rof_aggregate_launch_times(const rof_layout *L, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                               int feat, int normalized, const rof_epilogue *ep, void *workspace,
                               size_t workspace_bytes, void *stream, int iters, float ms_launch[2]) {
    if (!ms_launch || iters < 1 || !L) return ROF_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    // each iteration times [launch 1 + launch 2] and then [launch 2 alone]; launch 2 alone is a
    // complete run because launch 1's rows are still in the workspace
    EventSet e;
    int rc = e.create(3);
    if (rc) return rc;
    double both = 0.0, second = 0.0;
    rc = aggregate_with(L, x, x_dtype, ldx, out, ldo, feat, normalized, ep, workspace, workspace_bytes, st, 3);
    for (int i = 0; i < iters && rc == ROF_OK; ++i) {
        HIP_TRY(hipEventRecord(e.ev[0], st));
        rc = aggregate_with(L, x, x_dtype, ldx, out, ldo, feat, normalized, ep, workspace, workspace_bytes, st, 3);
        HIP_TRY(hipEventRecord(e.ev[1], st));
        if (rc == ROF_OK)
            rc = aggregate_with(L, x, x_dtype, ldx, out, ldo, feat, normalized, ep, workspace, workspace_bytes, st, 2);
        HIP_TRY(hipEventRecord(e.ev[2], st));
        HIP_TRY(hipEventSynchronize(e.ev[2]));
        float a = 0.f, b = 0.f;
        HIP_TRY(hipEventElapsedTime(&a, e.ev[0], e.ev[1]));
        HIP_TRY(hipEventElapsedTime(&b, e.ev[1], e.ev[2]));
        both += a;
        second += b;
    }
    ms_launch[1] = (float)(second / iters);
    ms_launch[0] = (float)((both - second) / iters);
    return rc;
}

}  // extern "C"
