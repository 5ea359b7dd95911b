// skm_assign_pruned: partial-distance GEMM on the leading d' dimensions followed by the per-point
// pruned search (reference distance_computers/batch_computers.h:297-409).
#include "skm_internal.h"

#include <algorithm>
#include <vector>

namespace skm {
int reduce_u32_sum_to_host(skm_ctx* ctx, const uint32_t* a, size_t n, double* h_out);
}

using namespace skm;

extern "C" int skm_assign_pruned(skm_ctx* ctx, const float* d_x, size_t n, const float* d_c, const float* d_pdx,
                                 const float* d_aux, size_t k, size_t d, size_t vertical_d, uint32_t partial_d,
                                 const float* d_ratios, const float* d_xnorm_p, const float* d_cnorm_p,
                                 uint32_t* d_inout_idx, float* d_out_dist, uint64_t* h_out_not_pruned,
                                 uint64_t* h_out_stage_pairs) {
    SKM_REQUIRE(ctx, "null context");
    if (h_out_not_pruned) *h_out_not_pruned = 0;
    const size_t n_hblocks = (d > vertical_d) ? (d - vertical_d) / SKM_H_DIM_SIZE : 0;
    if (h_out_stage_pairs)
        for (size_t s = 0; s < n_hblocks + 2; ++s) h_out_stage_pairs[s] = 0;
    if (n == 0) return SKM_OK;
    SKM_REQUIRE(d_x && d_c && d_pdx && d_aux && d_ratios && d_xnorm_p && d_cnorm_p && d_inout_idx && d_out_dist,
                "null pointer");
    SKM_REQUIRE(k > 0 && k <= 0x7fffffffULL, "k out of range");
    SKM_REQUIRE(d > 0 && d <= (1u << 20), "d out of range");
    SKM_REQUIRE(vertical_d > 0 && vertical_d <= d && (d - vertical_d) % SKM_H_DIM_SIZE == 0,
                "vertical_d must be in (0, d] with d - vertical_d a multiple of 64");
    SKM_REQUIRE(partial_d > 0 && partial_d <= vertical_d, "partial_d must be in (0, vertical_d]");
    ScopedStage outer(ctx, "search");

    const size_t ld = ((k + 63) / 64) * 64;
    size_t chunk = ctx->workspace_limit / (ld * sizeof(float));
    chunk = std::max<size_t>(128, (chunk / 128) * 128);
    chunk = std::min<size_t>(chunk, size_t(1) << 22);
    chunk = std::min(chunk, ((n + 127) / 128) * 128);
    void* ws_partial = nullptr;
    SKM_TRY(workspace(ctx, 0, std::min(chunk, n) * ld * sizeof(float), &ws_partial));
    void* ws_counts = nullptr;
    SKM_TRY(workspace(ctx, 1, n * sizeof(uint32_t) + (n_hblocks + 2) * sizeof(unsigned long long) + 64, &ws_counts));
    unsigned long long* d_stage = (unsigned long long*) ws_counts;
    uint32_t* d_counts = (uint32_t*) (d_stage + n_hblocks + 2);
    if (h_out_stage_pairs) SKM_TRY(skm_fill_u32(ctx, d_stage, 0u, 2 * (n_hblocks + 2)));

    for (size_t i0 = 0; i0 < n; i0 += chunk) {
        const size_t m = std::min(chunk, n - i0);
        {
            ScopedStage st(ctx, "search/blas");
            SKM_TRY(launch_gemm_store(ctx, d_x + i0 * d, (int) m, (int64_t) d, d_c, (int) k, (int64_t) d, (int) partial_d,
                                      (float*) ws_partial, (int64_t) ld, d_xnorm_p + i0, d_cnorm_p));
        }
        {
            ScopedStage st(ctx, "search/pdx");
            SKM_TRY(launch_prune(ctx, (const float*) ws_partial, (int64_t) ld, d_x + i0 * d, (int) m, d_c, d_pdx, d_aux,
                                 (int) k, (int) d, (int) vertical_d, (int) partial_d, d_ratios, d_inout_idx + i0,
                                 d_out_dist + i0, d_counts + i0, h_out_stage_pairs ? d_stage : nullptr));
        }
    }
    if (h_out_not_pruned) {
        double total = 0.0;
        SKM_TRY(reduce_u32_sum_to_host(ctx, d_counts, n, &total));
        *h_out_not_pruned = (uint64_t) total;
    }
    if (h_out_stage_pairs) {
        std::vector<unsigned long long> tmp(n_hblocks + 2);
        SKM_HIP_TRY(hipMemcpyAsync(tmp.data(), d_stage, tmp.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost,
                                   ctx->stream));
        SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
        for (size_t s = 0; s < tmp.size(); ++s) h_out_stage_pairs[s] = tmp[s];
    }
    return SKM_OK;
}
