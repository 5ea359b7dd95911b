// Dense stages: norms, rotation, transposition, exact nearest-centroid search.
#include "skm_internal.h"

#include <algorithm>
#include <mutex>

// Scratch of skm_assign_full_noalloc: per-(granule, point) minima of one chunk of points.  One copy per device
// that loads the library, held until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress; kernels and copies get the resolved device address.
static __device__ __align__(256) unsigned char scratch[SKM_NOALLOC_SCRATCH_BYTES];

namespace skm {

int resolve_noalloc_scratch(int device, void** out) {
    constexpr int MAX_DEVICES = 64;
    static std::mutex lock;
    static void* resolved[MAX_DEVICES] = {};
    if (device < 0 || device >= MAX_DEVICES) return set_error(SKM_ERR_INVALID, "device index out of range");
    std::lock_guard<std::mutex> guard(lock);
    if (!resolved[device]) {
        void* ptr = nullptr;
        SKM_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return set_error(SKM_ERR_HIP, "hipGetSymbolAddress returned a null address");
        resolved[device] = ptr;
    }
    *out = resolved[device];
    return SKM_OK;
}

// One wavefront per row; lane-strided accumulation then a fixed butterfly, so the result does not
// depend on launch geometry.
__global__ __launch_bounds__(256) void row_sqnorm_kernel(
    const float* __restrict__ m, size_t rows, size_t d, size_t cols, float* __restrict__ out
) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t) blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* p = m + row * d;
    float acc = 0.0f;
    if ((d % 4 == 0) && (reinterpret_cast<uintptr_t>(m) % 16 == 0)) {
        const size_t c4 = cols / 4;
        const float4* p4 = reinterpret_cast<const float4*>(p);
        for (size_t j = lane; j < c4; j += 64) {
            const float4 v = p4[j];
            acc += v.x * v.x;
            acc += v.y * v.y;
            acc += v.z * v.z;
            acc += v.w * v.w;
        }
        for (size_t j = c4 * 4 + lane; j < cols; j += 64) acc += p[j] * p[j];
    } else {
        for (size_t j = lane; j < cols; j += 64) acc += p[j] * p[j];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (lane == 0) out[row] = acc;
}

// 32 x 32 tiles through LDS (+1 padding): coalesced reads along the input rows and coalesced writes
// along the output rows.
__global__ __launch_bounds__(256) void transpose_kernel(
    const float* __restrict__ in, size_t rows, size_t cols, float* __restrict__ out
) {
    __shared__ float tile[32][33];
    const size_t c0 = (size_t) blockIdx.x * 32, r0 = (size_t) blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int i = ty; i < 32; i += 8) {
        const size_t r = r0 + i, c = c0 + tx;
        if (r < rows && c < cols) tile[i][tx] = in[r * cols + c];
    }
    __syncthreads();
    for (int i = ty; i < 32; i += 8) {
        const size_t c = c0 + i, r = r0 + tx;
        if (r < rows && c < cols) out[c * rows + r] = tile[tx][i];
    }
}

} // namespace skm

using namespace skm;

extern "C" {

int skm_norms(skm_ctx* ctx, const float* d_m, size_t rows, size_t d, size_t cols, float* d_out) {
    SKM_REQUIRE(ctx, "null context");
    if (rows == 0) return SKM_OK;
    SKM_REQUIRE(d_m && d_out, "null pointer");
    SKM_REQUIRE(d > 0 && cols <= d, "cols must be <= d");
    SKM_REQUIRE(rows <= 0x7fffffffULL * 4, "too many rows");
    ScopedStage st(ctx, "norms_calc");
    const unsigned blocks = (unsigned) ((rows + 3) / 4);
    hipLaunchKernelGGL(row_sqnorm_kernel, dim3(blocks), dim3(256), 0, ctx->stream, d_m, rows, d, cols, d_out);
    return check_hip(hipGetLastError(), "row_sqnorm_kernel launch");
}

int skm_transpose(skm_ctx* ctx, const float* d_in, size_t rows, size_t cols, float* d_out) {
    SKM_REQUIRE(ctx, "null context");
    if (rows == 0 || cols == 0) return SKM_OK;
    SKM_REQUIRE(d_in && d_out, "null pointer");
    SKM_REQUIRE(rows <= 65535u * 32u, "too many rows");
    dim3 grid((unsigned) ((cols + 31) / 32), (unsigned) ((rows + 31) / 32));
    hipLaunchKernelGGL(transpose_kernel, grid, dim3(256), 0, ctx->stream, d_in, rows, cols, d_out);
    return check_hip(hipGetLastError(), "transpose_kernel launch");
}

static int rotate_like(skm_ctx* ctx, const float* d_x, size_t n, size_t d, const float* d_mat, float* d_out,
                       const char* scope) {
    SKM_REQUIRE(ctx, "null context");
    if (n == 0) return SKM_OK;
    SKM_REQUIRE(d_x && d_mat && d_out, "null pointer");
    SKM_REQUIRE(d > 0 && d <= (1u << 20), "dimensionality out of range");
    SKM_REQUIRE(d_x != d_out, "rotation cannot run in place");
    ScopedStage st(ctx, scope);
    // Rows are processed in slabs so that the tile grid stays below 2^31.
    const size_t slab = size_t(1) << 24;
    for (size_t r0 = 0; r0 < n; r0 += slab) {
        const size_t m = std::min(slab, n - r0);
        SKM_TRY(launch_gemm_store(ctx, d_x + r0 * d, (int) m, (int64_t) d, d_mat, (int) d, (int64_t) d, (int) d,
                                  d_out + r0 * d, (int64_t) d, nullptr, nullptr));
    }
    return SKM_OK;
}

int skm_rotate(skm_ctx* ctx, const float* d_x, size_t n, size_t d, const float* d_q, float* d_out) {
    // out[i][j] = sum_k X[i][k] Q[j][k]
    return rotate_like(ctx, d_x, n, d, d_q, d_out, "rotator");
}

int skm_unrotate(skm_ctx* ctx, const float* d_r, size_t n, size_t d, const float* d_qt, float* d_out) {
    // out[i][j] = sum_k R[i][k] Q[k][j] = sum_k R[i][k] Qt[j][k]
    return rotate_like(ctx, d_r, n, d, d_qt, d_out, "unrotator");
}

int skm_assign_full(skm_ctx* ctx, const float* d_x, size_t n, const float* d_c, size_t k, size_t d,
                    const float* d_xnorm, const float* d_cnorm, uint32_t* d_out_idx, float* d_out_dist) {
    SKM_REQUIRE(ctx, "null context");
    if (n == 0) return SKM_OK;
    SKM_REQUIRE(d_x && d_c && d_xnorm && d_cnorm && d_out_idx && d_out_dist, "null pointer");
    SKM_REQUIRE(k > 0 && d > 0, "k and d must be positive");
    SKM_REQUIRE(k <= 0x7fffffffULL && d <= (1u << 20), "k or d out of range");
    ScopedStage outer(ctx, "search");
    const size_t n_granules = (k + 63) / 64;  // the smallest granule: an upper bound for every chunk
    // Points per chunk so that the granule scratch respects the workspace limit.
    size_t chunk = ctx->workspace_limit / (n_granules * sizeof(uint2));
    chunk = std::max<size_t>(128, (chunk / 128) * 128);
    chunk = std::min<size_t>(chunk, size_t(1) << 23);
    chunk = std::min(chunk, ((n + 127) / 128) * 128);
    void* scratch = nullptr;
    SKM_TRY(workspace(ctx, 0, n_granules * std::min(chunk, n) * sizeof(uint2), &scratch));
    for (size_t i0 = 0; i0 < n; i0 += chunk) {
        const size_t m = std::min(chunk, n - i0);
        const int granule = gemm_argmin_granule((int) k, (int) m);
        {
            ScopedStage st(ctx, "search/1st_blas");
            SKM_TRY(launch_gemm_argmin(ctx, d_c, (int) k, d_x + i0 * d, (int) m, (int) d, (int64_t) d, (int64_t) d,
                                       d_xnorm + i0, d_cnorm, (uint2*) scratch, granule));
        }
        {
            ScopedStage st(ctx, "search/merge");
            SKM_TRY(launch_merge_granules(ctx, (const uint2*) scratch, (int) m, (int) k, granule, d_out_idx + i0,
                                          d_out_dist + i0));
        }
    }
    return SKM_OK;
}

int skm_assign_full_noalloc(skm_ctx* ctx, const float* d_x, size_t n, const float* d_c, size_t k, size_t d,
                            const float* d_xnorm, const float* d_cnorm, uint32_t* d_out_idx, float* d_out_dist) {
    SKM_REQUIRE(ctx, "null context");
    if (n == 0) return SKM_OK;
    SKM_REQUIRE(d_x && d_c && d_xnorm && d_cnorm && d_out_idx && d_out_dist, "null pointer");
    SKM_REQUIRE(k > 0 && d > 0, "k and d must be positive");
    SKM_REQUIRE(d <= (1u << 20), "d out of range");
    if (k > SKM_NOALLOC_MAX_CENTROIDS)
        return set_error(SKM_ERR_INVALID, "skm_assign_full_noalloc: k = %zu exceeds the limit of %d centroids that the "
                         "static scratch of %d MiB allows; use skm_assign_full", k, SKM_NOALLOC_MAX_CENTROIDS,
                         (int) (SKM_NOALLOC_SCRATCH_BYTES >> 20));
    SKM_REQUIRE(ctx->noalloc_scratch, "static scratch was not resolved for this context");
    // Same two kernels as skm_assign_full; the granule minima of a chunk of points live in the static array.
    // No device timers here: they take events from a pool that may have to create them.
    const size_t n_granules = (k + 63) / 64;  // the smallest granule: an upper bound for every chunk
    size_t chunk = SKM_NOALLOC_SCRATCH_BYTES / (n_granules * sizeof(uint2));
    chunk = (chunk / 128) * 128;  // >= 128 by the limit on k
    uint2* granule_min = (uint2*) ctx->noalloc_scratch;
    for (size_t i0 = 0; i0 < n; i0 += chunk) {
        const size_t m = std::min(chunk, n - i0);
        const int granule = gemm_argmin_granule((int) k, (int) m);
        SKM_TRY(launch_gemm_argmin(ctx, d_c, (int) k, d_x + i0 * d, (int) m, (int) d, (int64_t) d, (int64_t) d,
                                   d_xnorm + i0, d_cnorm, granule_min, granule));
        SKM_TRY(launch_merge_granules(ctx, granule_min, (int) m, (int) k, granule, d_out_idx + i0, d_out_dist + i0));
    }
    return SKM_OK;
}

} // extern "C"
