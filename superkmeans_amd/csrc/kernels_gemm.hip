// MFMA kernels built on gemm_core.h: dense store (rotation, partial distances) and
// fused distance + per-granule argmin (exact nearest-centroid search).
#include "gemm_core.h"
#include "skm_internal.h"

#include <float.h>

namespace skm {

// The double-buffered operand stages need 72 KiB of LDS, above the 64 KiB a kernel may use without
// opting in; gfx950 has 160 KiB per CU, so two workgroups still fit on one CU.
template <class Kernel>
static int allow_large_lds(Kernel kernel, size_t bytes) {
    return check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int) bytes),
                     "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
}

#define SKM_LAUNCH_GEMM(kernel, grid, block, lds_bytes, stream, ...)                               \
    do {                                                                                           \
        static bool configured = false;                                                            \
        if (!configured) {                                                                         \
            SKM_TRY(allow_large_lds(kernel, lds_bytes));                                           \
            configured = true;                                                                     \
        }                                                                                          \
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, __VA_ARGS__);                   \
    } while (0)

// ---------------------------------------------------------------------------------------------
// Dense store: out[m][n] = D[m][n]                        (rotation, reference adsampling.h:191-215)
//           or out[m][n] = -2 D[m][n] + rn[m] + cn[n]     (batch_computers.h:361-366)
// Rows of D are the M operand (points), so that the 32 lanes of an accumulator column group write
// 128 contiguous bytes of one output row.
// ---------------------------------------------------------------------------------------------
template <bool VEC, bool DIST>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_store_kernel(
    GemmOperands g, float* __restrict__ out, int64_t ldo, const float* __restrict__ rn,
    const float* __restrict__ cn
) {
    extern __shared__ float lds[];
    int tm, tn;
    tile_of_block(g, blockIdx.x, tm, tn);
    WaveAcc acc;
    gemm_tile<VEC>(g, tm, tn, lds, acc);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int m0 = tm * GEMM_TM + (wave >> 1) * 64;
    const int n0 = tn * GEMM_TN + (wave & 1) * 64;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int n = n0 + acc_col(nb, lane);
        if (n >= g.N) continue;
        float cnv = 0.0f;
        if (DIST) cnv = cn[n];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + acc_row(mb, r, lane);
                if (m < g.M) {
                    float v = acc.v[mb][nb][r];
                    if (DIST) v = fmaf(-2.0f, v, rn[m]) + cnv;
                    out[(int64_t) m * ldo + n] = v;
                }
            }
        }
    }
}

int launch_gemm_store(skm_ctx* ctx, const float* A, int M, int64_t lda, const float* B, int N,
                      int64_t ldb, int K, float* out, int64_t ldo, const float* row_norm,
                      const float* col_norm) {
    if (M <= 0 || N <= 0 || K <= 0) return SKM_OK;
    GemmOperands g;
    g.A = A; g.B = B; g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb;
    g.tiles_m = (M + GEMM_TM - 1) / GEMM_TM;
    g.tiles_n = (N + GEMM_TN - 1) / GEMM_TN;
    const long long total = (long long) g.tiles_m * g.tiles_n;
    if (total > 0x7fffffffLL) return set_error(SKM_ERR_INVALID, "gemm grid too large");
    const bool vec = gemm_operands_vectorizable(g);
    const bool dist = row_norm != nullptr && col_norm != nullptr;
    const size_t lds_bytes = GEMM_LDS_FLOATS * sizeof(float);
    dim3 grid((unsigned) total), block(GEMM_THREADS);
    if (vec && dist)
        SKM_LAUNCH_GEMM((gemm_store_kernel<true, true>), grid, block, lds_bytes, ctx->stream, g, out, ldo, row_norm, col_norm);
    else if (vec)
        SKM_LAUNCH_GEMM((gemm_store_kernel<true, false>), grid, block, lds_bytes, ctx->stream, g, out, ldo, row_norm, col_norm);
    else if (dist)
        SKM_LAUNCH_GEMM((gemm_store_kernel<false, true>), grid, block, lds_bytes, ctx->stream, g, out, ldo, row_norm, col_norm);
    else
        SKM_LAUNCH_GEMM((gemm_store_kernel<false, false>), grid, block, lds_bytes, ctx->stream, g, out, ldo, row_norm, col_norm);
    return check_hip(hipGetLastError(), "gemm_store_kernel launch");
}

// ---------------------------------------------------------------------------------------------
// Distance + argmin: the M operand is the centroid tile, the N operand the point tile, so every
// lane owns one point column and scans 2 x 16 centroid rows in ascending index order in registers.
// The two half-wavefronts (rows 0-3 | 4-7 of every group of 8) are merged with one cross-lane
// exchange; the result of the 64-centroid granule is stored, never reduced with atomics.
// ---------------------------------------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_argmin_kernel(
    GemmOperands g, const float* __restrict__ xnorm, const float* __restrict__ cnorm,
    uint2* __restrict__ granule_min
) {
    extern __shared__ float lds[];
    int tm, tn;
    tile_of_block(g, blockIdx.x, tm, tn);
    WaveAcc acc;
    gemm_tile<VEC>(g, tm, tn, lds, acc);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = tm * GEMM_TM + wm * 64;
    const int n0 = tn * GEMM_TN + wn * 64;
    const int granule = tm * 2 + wm;
    if (m0 >= g.M) return;  // granule entirely past the last centroid: never read by the merge

    // ||c||^2 of the 32 rows this lane touches.
    float cn[2][16];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = m0 + acc_row(mb, r, lane);
            cn[mb][r] = (m < g.M) ? cnorm[m] : 0.0f;
        }

#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int n = n0 + acc_col(nb, lane);
        const float xn = (n < g.N) ? xnorm[n] : 0.0f;
        float best = FLT_MAX;
        uint32_t best_idx = (uint32_t) m0;
        bool have = false;
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + acc_row(mb, r, lane);
                const float v = fmaf(-2.0f, acc.v[mb][nb][r], xn) + cn[mb][r];
                if (m < g.M && (!have || v < best)) {
                    best = v;
                    best_idx = (uint32_t) m;
                    have = true;
                }
            }
        }
        // Merge with the other half-wavefront (same point, interleaved rows).
        const float o_best = __shfl_xor(best, 32);
        const uint32_t o_idx = (uint32_t) __shfl_xor((int) best_idx, 32);
        const int o_have = __shfl_xor((int) have, 32);
        if (o_have && (!have || o_best < best || (o_best == best && o_idx < best_idx))) {
            best = o_best;
            best_idx = o_idx;
        }
        if (lane < 32 && n < g.N) {
            granule_min[(int64_t) granule * g.N + n] = make_uint2(__float_as_uint(best), best_idx);
        }
    }
}

int launch_gemm_argmin(skm_ctx* ctx, const float* C, int k, const float* X, int n, int d,
                       int64_t ldc, int64_t ldx, const float* xnorm, const float* cnorm,
                       uint2* granule_min) {
    if (k <= 0 || n <= 0 || d <= 0) return SKM_OK;
    GemmOperands g;
    g.A = C; g.B = X; g.M = k; g.N = n; g.K = d; g.lda = ldc; g.ldb = ldx;
    g.tiles_m = (k + GEMM_TM - 1) / GEMM_TM;
    g.tiles_n = (n + GEMM_TN - 1) / GEMM_TN;
    const long long total = (long long) g.tiles_m * g.tiles_n;
    if (total > 0x7fffffffLL) return set_error(SKM_ERR_INVALID, "gemm grid too large");
    const size_t lds_bytes = GEMM_LDS_FLOATS * sizeof(float);
    dim3 grid((unsigned) total), block(GEMM_THREADS);
    if (gemm_operands_vectorizable(g))
        SKM_LAUNCH_GEMM((gemm_argmin_kernel<true>), grid, block, lds_bytes, ctx->stream, g, xnorm, cnorm, granule_min);
    else
        SKM_LAUNCH_GEMM((gemm_argmin_kernel<false>), grid, block, lds_bytes, ctx->stream, g, xnorm, cnorm, granule_min);
    return check_hip(hipGetLastError(), "gemm_argmin_kernel launch");
}

// ---------------------------------------------------------------------------------------------
// Partial distances with the first pruning test fused into the epilogue.  Same operand roles as the
// argmin kernel (one point per lane).  A (point, centroid) pair is emitted only when its partial
// distance is below thr0[point] = seed distance * ratios[d'], the loosest threshold that point can
// ever see (its best distance only shrinks from batch to batch, batch_computers.h:372-380), so the
// emitted set is a superset of the reference's survivors of every batch; the pruning kernel re-applies
// the exact per-batch threshold.  Pairs go to a per-point list of `cap` slots; the per-point counter
// keeps counting past `cap` so that overflowing points can be detected and redone densely.
// ---------------------------------------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_candidates_kernel(
    GemmOperands g, const float* __restrict__ xnorm, const float* __restrict__ cnorm,
    const float* __restrict__ thr0, uint32_t* __restrict__ cand_count, uint2* __restrict__ cand, uint32_t cap
) {
    extern __shared__ float lds[];
    int tm, tn;
    tile_of_block(g, blockIdx.x, tm, tn);
    WaveAcc acc;
    gemm_tile<VEC>(g, tm, tn, lds, acc);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int m0 = tm * GEMM_TM + (wave >> 1) * 64;
    const int n0 = tn * GEMM_TN + (wave & 1) * 64;
    if (m0 >= g.M) return;
    float cn[2][16];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = m0 + acc_row(mb, r, lane);
            cn[mb][r] = (m < g.M) ? cnorm[m] : 0.0f;
        }
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int n = n0 + acc_col(nb, lane);
        if (n >= g.N) continue;
        const float xn = xnorm[n];
        const float thr = thr0[n];
        uint32_t pass = 0;  // bit (mb * 16 + r)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + acc_row(mb, r, lane);
                const float v = fmaf(-2.0f, acc.v[mb][nb][r], xn) + cn[mb][r];
                acc.v[mb][nb][r] = v;
                if (m < g.M && v < thr) pass |= 1u << (mb * 16 + r);
            }
        if (pass) {
            const uint32_t cnt = (uint32_t) __popc(pass);
            uint32_t slot = atomicAdd(&cand_count[n], cnt);
            uint2* list = cand + (int64_t) n * cap;
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if (pass & (1u << (mb * 16 + r))) {
                        if (slot < cap)
                            list[slot] = make_uint2((uint32_t) (m0 + acc_row(mb, r, lane)), __float_as_uint(acc.v[mb][nb][r]));
                        ++slot;
                    }
                }
        }
    }
}

int launch_gemm_candidates(skm_ctx* ctx, const float* C, int k, const float* X, int n, int partial_d, int64_t ld,
                           const float* xnorm_p, const float* cnorm_p, const float* thr0, uint32_t* cand_count,
                           uint2* cand, uint32_t cap) {
    if (k <= 0 || n <= 0 || partial_d <= 0) return SKM_OK;
    GemmOperands g;
    g.A = C; g.B = X; g.M = k; g.N = n; g.K = partial_d; g.lda = ld; g.ldb = ld;
    g.tiles_m = (k + GEMM_TM - 1) / GEMM_TM;
    g.tiles_n = (n + GEMM_TN - 1) / GEMM_TN;
    const long long total = (long long) g.tiles_m * g.tiles_n;
    if (total > 0x7fffffffLL) return set_error(SKM_ERR_INVALID, "gemm grid too large");
    const size_t lds_bytes = GEMM_LDS_FLOATS * sizeof(float);
    dim3 grid((unsigned) total), block(GEMM_THREADS);
    if (gemm_operands_vectorizable(g))
        SKM_LAUNCH_GEMM((gemm_candidates_kernel<true>), grid, block, lds_bytes, ctx->stream, g, xnorm_p, cnorm_p, thr0, cand_count, cand, cap);
    else
        SKM_LAUNCH_GEMM((gemm_candidates_kernel<false>), grid, block, lds_bytes, ctx->stream, g, xnorm_p, cnorm_p, thr0, cand_count, cand, cap);
    return check_hip(hipGetLastError(), "gemm_candidates_kernel launch");
}

// ---------------------------------------------------------------------------------------------
// Sequential merge of granule minima, reproducing batch_computers.h:118,162-167:
//   out = FLT_MAX; for each batch of 1024 centroids in order:
//       m = first minimum of the batch;  if (m < out) { out = max(0, m); idx = argmin; }
// ---------------------------------------------------------------------------------------------
__global__ void merge_granules_kernel(
    const uint2* __restrict__ granule_min, int n, int k, uint32_t* __restrict__ out_idx,
    float* __restrict__ out_dist
) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int n_granules = (k + 63) / 64;
    const int per_batch = SKM_Y_BATCH_SIZE / 64;
    float out = FLT_MAX;
    uint32_t idx = 0;
    for (int g0 = 0; g0 < n_granules; g0 += per_batch) {
        float bm = 0.0f;
        uint32_t bi = 0;
        const int g1 = (g0 + per_batch < n_granules) ? g0 + per_batch : n_granules;
        for (int g = g0; g < g1; ++g) {
            const uint2 e = granule_min[(int64_t) g * n + i];
            const float v = __uint_as_float(e.x);
            if (g == g0 || v < bm) {
                bm = v;
                bi = e.y;
            }
        }
        if (bm < out) {
            out = fmaxf(0.0f, bm);
            idx = bi;
        }
    }
    out_idx[i] = idx;
    out_dist[i] = out;
}

int launch_merge_granules(skm_ctx* ctx, const uint2* granule_min, int n, int k, uint32_t* out_idx,
                          float* out_dist) {
    if (n <= 0) return SKM_OK;
    dim3 grid((n + 255) / 256), block(256);
    hipLaunchKernelGGL(merge_granules_kernel, grid, block, 0, ctx->stream, granule_min, n, k, out_idx, out_dist);
    return check_hip(hipGetLastError(), "merge_granules_kernel launch");
}

} // namespace skm
