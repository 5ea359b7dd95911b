// Layout kernels: PDX relayout of the centroids, row gather / assignment scatter for the
// hierarchical driver.
#include "skm_internal.h"

namespace skm {

// Vertical part of PDXLayout::PDXify<false> (reference pdx/layout.h:176-183,205-213): inside each
// chunk of up to 1024 centroids the first vertical_d columns become dimension-major.  32 x 32 tiles
// are staged through LDS so that both the row-major reads and the dimension-major writes are
// coalesced.
__device__ __forceinline__ void pdx_vertical_tile(
    const float* __restrict__ in, size_t k, size_t d, size_t V, float* __restrict__ out, size_t tile_x, size_t tile_y,
    size_t chunk
) {
    __shared__ float tile[32][33];
    const size_t base_row = chunk * SKM_Y_BATCH_SIZE;
    const size_t m = (k - base_row) < SKM_Y_BATCH_SIZE ? (k - base_row) : SKM_Y_BATCH_SIZE;
    const size_t r0 = tile_y * 32, c0 = tile_x * 32;
    if (r0 >= m) return;
    const float* src = in + base_row * d;
    float* dst = out + base_row * d;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int i = ty; i < 32; i += 8) {
        const size_t r = r0 + i, c = c0 + tx;
        if (r < m && c < V) tile[i][tx] = src[r * d + c];
    }
    __syncthreads();
    for (int i = ty; i < 32; i += 8) {
        const size_t c = c0 + i, r = r0 + tx;
        if (r < m && c < V) dst[c * m + r] = tile[tx][i];
    }
}

// Horizontal part (pdx/layout.h:186-192,216-222): 64-wide row-major blocks, one after the other.
// Also emits the dense copy of the first V columns (superkmeans.h:1206-1212) when aux != nullptr.
__device__ __forceinline__ void pdx_horizontal_row(
    const float* __restrict__ in, size_t k, size_t d, size_t V, float* __restrict__ out, float* __restrict__ aux, size_t row
) {
    const size_t chunk = row / SKM_Y_BATCH_SIZE;
    const size_t base_row = chunk * SKM_Y_BATCH_SIZE;
    const size_t m = (k - base_row) < SKM_Y_BATCH_SIZE ? (k - base_row) : SKM_Y_BATCH_SIZE;
    const size_t r = row - base_row;
    const float* src = in + row * d;
    float* dst = out + base_row * d + V * m;
    for (size_t j = V + threadIdx.x; j < d; j += blockDim.x) {
        const size_t h = j - V;
        dst[(h / SKM_H_DIM_SIZE) * m * SKM_H_DIM_SIZE + r * SKM_H_DIM_SIZE + (h % SKM_H_DIM_SIZE)] = src[j];
    }
    if (aux) {
        float* a = aux + row * V;
        for (size_t j = threadIdx.x; j < V; j += blockDim.x) a[j] = src[j];
    }
}

// Both parts in one launch: the first vertical_tiles workgroups (tile column fastest, then tile row, then chunk) transpose
// tiles of the vertical part, the next horizontal_rows take one centroid each.
__global__ __launch_bounds__(256) void pdxify_kernel(
    const float* __restrict__ in, size_t k, size_t d, size_t V, float* __restrict__ out, float* __restrict__ aux,
    uint32_t tiles_x, uint32_t vertical_tiles
) {
    if (blockIdx.x < vertical_tiles) {
        constexpr uint32_t TILES_Y = SKM_Y_BATCH_SIZE / 32;
        const uint32_t b = blockIdx.x;
        pdx_vertical_tile(in, k, d, V, out, b % tiles_x, (b / tiles_x) % TILES_Y, b / (tiles_x * TILES_Y));
    } else {
        pdx_horizontal_row(in, k, d, V, out, aux, blockIdx.x - vertical_tiles);
    }
}

__global__ __launch_bounds__(256) void gather_rows_kernel(
    const float* __restrict__ x, size_t d, const uint64_t* __restrict__ index, size_t m,
    float* __restrict__ out, const float* __restrict__ norms_in, float* __restrict__ norms_out, int vec
) {
    const size_t j = blockIdx.x;
    const size_t i = index[j];
    const float* src = x + i * d;
    float* dst = out + j * d;
    if (vec) {
        const size_t d4 = d / 4;
        for (size_t t = threadIdx.x; t < d4; t += blockDim.x)
            reinterpret_cast<float4*>(dst)[t] = reinterpret_cast<const float4*>(src)[t];
    } else {
        for (size_t t = threadIdx.x; t < d; t += blockDim.x) dst[t] = src[t];
    }
    if (norms_in && norms_out && threadIdx.x == 0) norms_out[j] = norms_in[i];
}

__global__ __launch_bounds__(256) void scatter_assignments_kernel(
    const uint64_t* __restrict__ index, const uint32_t* __restrict__ local, size_t m, uint32_t offset,
    uint32_t* __restrict__ out
) {
    const size_t j = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (j < m) out[index[j]] = local[j] + offset;
}

__global__ __launch_bounds__(256) void seeds_from_groups_kernel(
    uint32_t* __restrict__ seeds, const uint32_t* __restrict__ group, const uint32_t* __restrict__ representative,
    uint32_t n_groups, size_t n
) {
    const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && seeds[i] == 0xffffffffu) {
        const uint32_t g = group[i];
        seeds[i] = representative[g < n_groups ? g : n_groups - 1];  // a group out of range reads no stray memory
    }
}

} // namespace skm

using namespace skm;

extern "C" {

int skm_pdxify(skm_ctx* ctx, const float* d_c, size_t k, size_t d, size_t vertical_d, float* d_pdx, float* d_aux) {
    SKM_REQUIRE(ctx, "null context");
    if (k == 0) return SKM_OK;
    SKM_REQUIRE(d_c && d_pdx, "null pointer");
    SKM_REQUIRE(d > 0 && vertical_d > 0 && vertical_d <= d, "vertical_d must be in (0, d]");
    SKM_REQUIRE((d - vertical_d) % SKM_H_DIM_SIZE == 0, "d - vertical_d must be a multiple of 64");
    SKM_REQUIRE(d_c != d_pdx, "relayout cannot run in place");
    ScopedStage st(ctx, "consolidate/pdxify");
    const size_t n_chunks = (k + SKM_Y_BATCH_SIZE - 1) / SKM_Y_BATCH_SIZE;
    SKM_REQUIRE(n_chunks <= 65535, "too many centroids");
    const uint32_t tiles_x = (uint32_t) ((vertical_d + 31) / 32);
    const size_t vertical_tiles = (size_t) tiles_x * (SKM_Y_BATCH_SIZE / 32) * n_chunks;
    const size_t horizontal_rows = (d > vertical_d || d_aux) ? k : 0;
    SKM_REQUIRE(vertical_tiles + horizontal_rows <= 0x7fffffffULL, "too many centroids for one launch");
    hipLaunchKernelGGL(pdxify_kernel, dim3((unsigned) (vertical_tiles + horizontal_rows)), dim3(256), 0, ctx->stream, d_c, k, d,
                       vertical_d, d_pdx, d_aux, tiles_x, (uint32_t) vertical_tiles);
    return check_hip(hipGetLastError(), "pdxify_kernel launch");
}

int skm_gather_rows(skm_ctx* ctx, const float* d_x, size_t d, const uint64_t* d_index, size_t m, float* d_out,
                    const float* d_norms_in, float* d_norms_out) {
    SKM_REQUIRE(ctx, "null context");
    if (m == 0) return SKM_OK;
    SKM_REQUIRE(d_x && d_index && d_out, "null pointer");
    SKM_REQUIRE(m <= 0x7fffffffULL, "too many rows");
    ScopedStage st(ctx, "compact_mesocluster");
    const int vec = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(d_x) % 16 == 0) &&
                    (reinterpret_cast<uintptr_t>(d_out) % 16 == 0);
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned) m), dim3(256), 0, ctx->stream, d_x, d, d_index, m, d_out,
                       d_norms_in, d_norms_out, vec);
    return check_hip(hipGetLastError(), "gather_rows_kernel launch");
}

int skm_scatter_assignments(skm_ctx* ctx, const uint64_t* d_index, const uint32_t* d_local, size_t m, uint32_t offset,
                            uint32_t* d_out) {
    SKM_REQUIRE(ctx, "null context");
    if (m == 0) return SKM_OK;
    SKM_REQUIRE(d_index && d_local && d_out, "null pointer");
    ScopedStage st(ctx, "get_indirection_assignments");
    hipLaunchKernelGGL(scatter_assignments_kernel, dim3((unsigned) ((m + 255) / 256)), dim3(256), 0, ctx->stream, d_index,
                       d_local, m, offset, d_out);
    return check_hip(hipGetLastError(), "scatter_assignments_kernel launch");
}

int skm_seeds_from_groups(skm_ctx* ctx, uint32_t* d_seeds, const uint32_t* d_group, const uint32_t* d_representative,
                          size_t n_groups, size_t n) {
    SKM_REQUIRE(ctx, "null context");
    if (n == 0) return SKM_OK;
    SKM_REQUIRE(d_seeds && d_group && d_representative, "null pointer");
    SKM_REQUIRE(n_groups > 0 && n_groups <= 0xffffffffULL, "the number of groups must be in [1, 2^32)");
    SKM_REQUIRE((n + 255) / 256 <= 0x7fffffffULL, "too many points");
    hipLaunchKernelGGL(seeds_from_groups_kernel, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, ctx->stream, d_seeds,
                       d_group, d_representative, (uint32_t) n_groups, n);
    return check_hip(hipGetLastError(), "seeds_from_groups_kernel launch");
}

} // extern "C"
