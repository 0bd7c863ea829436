/* TEST INFRASTRUCTURE -- not part of the shipped library.
 *
 * CPU oracle for the aggregation kernels: a sequential fp32 restatement of what each upstream
 * CUDA kernel computes (ROF/reuse_conv/reuse_conv_kernel.cu), one "warp" at a time, in part
 * order.  Upstream flushes with a float atomic (cu:16-21), so its own summation order is not
 * fixed; any order agrees to fp32 re-association, which is why the parity bar for sums is
 * rel 1e-5 / abs 1e-6 rather than bit equality.
 *
 * The upstream kernels cannot be built or run here (CUDA only), so this file is pinned by
 * mathematics instead (tests/test_oracle_agg.py): the float64 closed form
 * D^-1/2 A D^-1/2 X computed with scipy, a brute-force per-edge loop on a toy graph, and the
 * identity that v1/v2 plans are re-bracketings of the same sum.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this library.
 * Build with -ffp-contract=off so that multiply and add stay separate roundings (cu:270 uses
 * __fmul_rn followed by +=).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* __frsqrt_rn (cu:254,276): correctly rounded 1/sqrt(x).  The double result is exact to
 * 53 bits, far beyond the 24+2 needed for a correctly rounded float except on exact ties,
 * which 1/sqrt of a float cannot produce. */
static inline float rsqrt_rn(float x) { return (float)(1.0 / sqrt((double)x)); }

float orc_rsqrt_rn(float x) { return rsqrt_rn(x); }

/* One warp's inner loop (cu:250-274 = cu:449-473 = cu:910-935): partial[d] += rs(deg[u]) * in[u][d]. */
static void part_sum(const float *in, int64_t ld, const float *deg, const int32_t *col, int beg, int end,
                     int dim, int normalized, float *partial) {
    for (int d = 0; d < dim; ++d) partial[d] = 0.0f;
    for (int k = beg; k < end; ++k) {
        int32_t u = col[k];
        const float *row = in + (int64_t)u * ld;
        if (normalized) {
            float w = rsqrt_rn(deg[u]);
            for (int d = 0; d < dim; ++d) { float t = w * row[d]; partial[d] += t; }
        } else {
            for (int d = 0; d < dim; ++d) partial[d] += row[d];
        }
    }
}

/* spmm_forward_cuda_kernel_GNNA (cu:205-286) when normalized=1;
 * SAG_cuda_kernel (cu:123-196) when normalized=0.  `out` must be zeroed by the caller (cu:303, cu:58). */
void orc_agg_parts(const float *in, int64_t ld, const float *deg, const int32_t *col, const int32_t *part_ptr,
                   const int32_t *part2node, int num_parts, int dim, int normalized, float *out, int64_t ldo) {
    float *partial = (float *)malloc(sizeof(float) * (size_t)(dim > 0 ? dim : 1));
    for (int p = 0; p < num_parts; ++p) {
        part_sum(in, ld, deg, col, part_ptr[p], part_ptr[p + 1], dim, normalized, partial);
        int32_t v = part2node[p];
        float s = normalized ? rsqrt_rn(deg[v]) : 1.0f;
        float *o = out + (int64_t)v * ldo;
        for (int d = 0; d < dim; ++d) { float t = partial[d] * s; o[d] += t; }
    }
    free(partial);
}

/* v1: spmm_forward_cuda_kernel_caching (cu:396-487) then _reusing (cu:489-601).
 * cache is [cache_num, dim+1]; column dim receives the ready flag 1.0 (cu:485). */
void orc_agg_v1(const float *in, int64_t ld, const float *deg, const int32_t *col, const int32_t *part_ptr,
                const int32_t *part2node, int num_parts, int dim, float *cache, const int32_t *flag,
                const int32_t *cache_ptr, const int32_t *cache_col, int cache_num, float *out, int64_t ldo) {
    float *partial = (float *)malloc(sizeof(float) * (size_t)(dim > 0 ? dim : 1));
    for (int c = 0; c < cache_num; ++c) {
        part_sum(in, ld, deg, cache_col, cache_ptr[c], cache_ptr[c + 1], dim, 1, partial);
        memcpy(cache + (int64_t)c * (dim + 1), partial, sizeof(float) * (size_t)dim);
        cache[(int64_t)c * (dim + 1) + dim] = 1.0f;
    }
    for (int p = 0; p < num_parts; ++p) {
        int32_t v = part2node[p];
        float s = rsqrt_rn(deg[v]);
        float *o = out + (int64_t)v * ldo;
        int f = flag[p];
        if (f > 0 && cache[(int64_t)(f - 1) * (dim + 1) + dim] != 0.0f) {        /* cu:525-529, 587-598 */
            const float *c = cache + (int64_t)(f - 1) * (dim + 1);
            for (int d = 0; d < dim; ++d) { float t = c[d] * s; o[d] += t; }
        } else {                                                                   /* cu:534-585 */
            part_sum(in, ld, deg, col, part_ptr[p], part_ptr[p + 1], dim, 1, partial);
            for (int d = 0; d < dim; ++d) { float t = partial[d] * s; o[d] += t; }
        }
    }
    free(partial);
}

/* v2: spmm_forward_cuda_kernel_fuse (cu:836-954): one partial per unique part, fanned out to
 * every destination in part2Node_col[part2Node_ptr[w] : part2Node_ptr[w+1]]. */
void orc_agg_v2(const float *in, int64_t ld, const float *deg, const int32_t *ucol, const int32_t *uptr,
                const int32_t *dptr, const int32_t *dcol, int num_uniq, int dim, int normalized, float *out,
                int64_t ldo) {
    float *partial = (float *)malloc(sizeof(float) * (size_t)(dim > 0 ? dim : 1));
    for (int w = 0; w < num_uniq; ++w) {
        part_sum(in, ld, deg, ucol, uptr[w], uptr[w + 1], dim, normalized, partial);
        for (int j = dptr[w]; j < dptr[w + 1]; ++j) {
            int32_t v = dcol[j];
            float s = normalized ? rsqrt_rn(deg[v]) : 1.0f;
            float *o = out + (int64_t)v * ldo;
            for (int d = 0; d < dim; ++d) { float t = partial[d] * s; o[d] += t; }
        }
    }
    free(partial);
}

/* CPU baseline leg: the same sum, destination-parallel over host cores (one row per task, no
 * atomics), i.e. the GNNA kernel with whole rows as parts.  deg_rs = rsqrt_rn(deg) precomputed. */
void orc_spmm_rows(const float *in, int64_t ld, const float *deg_rs, const int32_t *indptr, const int32_t *indices,
                   int n, int dim, int normalized, float *out, int64_t ldo) {
#pragma omp parallel for schedule(dynamic, 256)
    for (int v = 0; v < n; ++v) {
        float *o = out + (int64_t)v * ldo;
        for (int d = 0; d < dim; ++d) o[d] = 0.0f;
        for (int k = indptr[v]; k < indptr[v + 1]; ++k) {
            int32_t u = indices[k];
            const float *row = in + (int64_t)u * ld;
            if (normalized) {
                float w = deg_rs[u];
                for (int d = 0; d < dim; ++d) o[d] += w * row[d];
            } else {
                for (int d = 0; d < dim; ++d) o[d] += row[d];
            }
        }
        if (normalized) {
            float s = deg_rs[v];
            for (int d = 0; d < dim; ++d) o[d] *= s;
        }
    }
}
