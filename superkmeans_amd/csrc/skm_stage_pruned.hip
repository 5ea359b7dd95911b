// skm_assign_pruned: partial-distance GEMM on the leading d' dimensions followed by the per-point
// pruned search (reference distance_computers/batch_computers.h:297-409).
//
// Per chunk of points:
//   1. seed_distance_kernel     full distance to the previous assignment -> best0, thr0 = best0 * ratios[d']
//   2. gemm_candidates_kernel or gemm_candidates_stationary_kernel (d' up to 160 and enough points to fill the
//                               chip with 256-point workgroups): MFMA partial distances; the epilogue emits only
//                               pairs below thr0 into per-point lists (nothing dense is written)
//   3. prune_pool_kernel (rows 16-byte aligned) or prune_list_kernel: exact per-batch thresholds, block-wise
//                               pruning, best candidate
// After the last chunk, the points whose list overflowed (loose seeds, points with no centroid nearby)
// are gathered and searched again through dense rows of partial distances (gemm_store_kernel with the distance
// epilogue + the walk whose first test scans the row): same results, more traffic, and only for those points.
#include "skm_internal.h"

#include <algorithm>
#include <vector>

namespace skm {
int reduce_u32_sum_to_host(skm_ctx* ctx, const uint32_t* a, size_t n, double* h_out);
int reduce_u32_sum_enqueue(skm_ctx* ctx, const uint32_t* a, size_t n, double** h_slot, const uint32_t* d_word,
                           uint32_t* h_word);
int overflow_count_slot(skm_ctx* ctx, uint32_t** h_slot);
}

using namespace skm;

namespace {

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct SearchOperands {
    const float *d_c, *d_pdx, *d_aux, *d_ratios, *d_cnorm_p;
    size_t k, d, vertical_d;
    uint32_t partial_d;
};

// Seed, candidate lists and list walk of one chunk of m points whose lists have `cap` slots each.  Points whose list
// overflows are left untouched and appended to d_over_ids (as id_offset + row).
int search_chunk(skm_ctx* ctx, const SearchOperands& o, const float* xc, size_t m, const float* d_xnorm_p, uint32_t cap,
                 uint2* d_cand, float* d_best0, float* d_thr0, uint32_t* d_cand_count, uint32_t* d_inout_idx, float* d_out_dist,
                 uint32_t* d_counts, unsigned long long* stage_arg, const uint32_t* order, uint64_t* d_over_ids,
                 uint32_t* d_n_over, uint64_t id_offset, bool zero_n_over, uint32_t* d_cursor) {
    {
        ScopedStage st(ctx, "search/seed");
        SKM_TRY(launch_seed_distance(ctx, xc, o.d_c, d_inout_idx, (int) m, (int) o.d, o.d_ratios, (int) o.partial_d, d_best0,
                                     d_thr0, order, zero_n_over ? d_n_over : (uint32_t*) nullptr));
    }
    {
        ScopedStage st(ctx, "search/blas");
        // the register-stationary kernel addresses the 64 lists of a wavefront with 32-bit byte offsets
        const bool lists_fit = (uint64_t) cap * 64 * sizeof(uint2) < (uint64_t(1) << 32);
        if (ctx->candidate_kernel != 1 && ctx->candidate_kernel != 3 && lists_fit &&
            gemm_candidates_stationary_serves(o.d_c, (int) o.k, xc, (int) m, (int) o.partial_d, (int64_t) o.d,
                                              ctx->candidate_kernel == 2))
            SKM_TRY(launch_gemm_candidates_stationary(ctx, o.d_c, (int) o.k, xc, (int) m, (int) o.partial_d, (int64_t) o.d,
                                                      d_xnorm_p, o.d_cnorm_p, d_thr0, d_cand_count, d_cand, cap));
        else
            SKM_TRY(launch_gemm_candidates(ctx, o.d_c, (int) o.k, xc, (int) m, (int) o.partial_d, (int64_t) o.d, d_xnorm_p,
                                           o.d_cnorm_p, d_thr0, d_cand_count, d_cand, cap));
    }
    {
        ScopedStage st(ctx, "search/pdx");
        // Several points per wavefront pay when the points are many: with few points an eighth as many wavefronts
        // do not fill the chip.
        const bool pooled = ctx->walk_kernel != 1 && prune_pool_serves(xc, o.d_pdx, (int) o.d) &&
                            (ctx->walk_kernel >= 2 || m >= 32768);
        const int points_per_wavefront = ctx->walk_kernel == 2 ? 4 : (ctx->walk_kernel == 3 ? 8 : 0);
        if (pooled) {
            const int n_batches = (int) ((o.k + SKM_Y_BATCH_SIZE - 1) / SKM_Y_BATCH_SIZE);
            const int phases = std::max(1, std::min(ctx->walk_launches, n_batches));
            for (int ph = 0; ph < phases; ++ph) {
                const int lo = (int) ((int64_t) n_batches * ph / phases), hi = (int) ((int64_t) n_batches * (ph + 1) / phases);
                SKM_TRY(launch_prune_pool(ctx, d_cand, d_cand_count, cap, d_best0, xc, (int) m, o.d_pdx, o.d_aux, (int) o.k,
                                          (int) o.d, (int) o.vertical_d, (int) o.partial_d, o.d_ratios, d_inout_idx, d_out_dist,
                                          d_counts, stage_arg, order, d_over_ids, d_n_over, id_offset, lo, hi, d_cursor,
                                          points_per_wavefront));
            }
        } else
            SKM_TRY(launch_prune_list(ctx, d_cand, d_cand_count, cap, d_best0, xc, (int) m, o.d_pdx, o.d_aux, (int) o.k,
                                      (int) o.d, (int) o.vertical_d, (int) o.partial_d, o.d_ratios, d_inout_idx, d_out_dist,
                                      d_counts, stage_arg, order, d_over_ids, d_n_over, id_offset, nullptr, 0));
    }
    return SKM_OK;
}

// The points `d_ids`, whose lists overflowed, searched again from the same seeds through rows of partial distances to
// all centroids: rows, norms and seeds are gathered into a compact block; per chunk that fits the workspace the seed
// distances, the dense partial distances (the GEMM core with the distance epilogue: the same values as the candidate
// kernels compute) and the walk whose first test scans the dense row; results are scattered back.  For a point that a
// quarter of the centroids pass, a dense row costs less than appending and walking that many list entries (measured
// against a second pass of the candidate kernel with lists that hold every centroid: 137 against 154 ms for the
// 685,000 overflowing points of an AssignTrainingPoints with the reference's defaults at n = 1M, k = 10,000; 12.3
// against 14.5 ms for the 86,000 of the second iteration of a Train), and for a handful of points the GEMM spreads
// over centroid tiles where a candidate kernel sweeps them with one workgroup (0.7 ms per iteration).
int redo_with_dense_rows(skm_ctx* ctx, const SearchOperands& o, const float* d_x, const uint64_t* d_ids, size_t mo,
                         const float* d_xnorm_p, uint32_t* d_inout_idx, float* d_out_dist, uint32_t* d_counts,
                         unsigned long long* stage_arg) {
    const size_t ld = align_up(o.k, 64);
    size_t chunk = ctx->workspace_limit / (ld * sizeof(float));
    chunk = std::max<size_t>(128, (chunk / 128) * 128);
    chunk = std::min<size_t>(chunk, size_t(1) << 22);
    chunk = std::min(chunk, align_up(mo, 128));
    const size_t mo_pad = align_up(mo, 64);
    void* ws_o = nullptr;
    SKM_TRY(workspace(ctx, 3, mo * o.d * sizeof(float) + 6 * mo_pad * sizeof(uint32_t), &ws_o));
    float* xo = (float*) ws_o;
    float* xnorm_o = xo + mo * o.d;
    uint32_t* idx_o = (uint32_t*) (xnorm_o + mo_pad);
    float* dist_o = (float*) (idx_o + mo_pad);
    uint32_t* cnt_o = (uint32_t*) (dist_o + mo_pad);
    float* best0_o = (float*) (cnt_o + mo_pad);
    float* thr0_o = best0_o + mo_pad;
    SKM_TRY(skm_gather_rows(ctx, d_x, o.d, d_ids, mo, xo, d_xnorm_p, xnorm_o));
    SKM_TRY(launch_gather_u32(ctx, d_inout_idx, d_ids, (int) mo, idx_o));
    void* ws_partial = nullptr;
    SKM_TRY(workspace(ctx, 0, std::min(chunk, mo) * ld * sizeof(float), &ws_partial));
    for (size_t i0 = 0; i0 < mo; i0 += chunk) {
        const size_t m = std::min(chunk, mo - i0);
        {
            ScopedStage st(ctx, "search/overflow/seed");
            SKM_TRY(launch_seed_distance(ctx, xo + i0 * o.d, o.d_c, idx_o + i0, (int) m, (int) o.d, o.d_ratios,
                                         (int) o.partial_d, best0_o + i0, thr0_o + i0, nullptr, nullptr));
        }
        {
            ScopedStage st(ctx, "search/overflow/blas");
            SKM_TRY(launch_gemm_store(ctx, xo + i0 * o.d, (int) m, (int64_t) o.d, o.d_c, (int) o.k, (int64_t) o.d,
                                      (int) o.partial_d, (float*) ws_partial, (int64_t) ld, xnorm_o + i0, o.d_cnorm_p));
        }
        {
            ScopedStage st(ctx, "search/overflow/pdx");
            SKM_TRY(launch_prune_list(ctx, nullptr, nullptr, 0, best0_o + i0, xo + i0 * o.d, (int) m, o.d_pdx, o.d_aux,
                                      (int) o.k, (int) o.d, (int) o.vertical_d, (int) o.partial_d, o.d_ratios, idx_o + i0,
                                      dist_o + i0, cnt_o + i0, stage_arg, nullptr, nullptr, nullptr, 0,
                                      (const float*) ws_partial, (int64_t) ld));
        }
    }
    SKM_TRY(launch_scatter_u32(ctx, idx_o, d_ids, (int) mo, d_inout_idx));
    SKM_TRY(launch_scatter_u32(ctx, (const uint32_t*) dist_o, d_ids, (int) mo, (uint32_t*) d_out_dist));
    SKM_TRY(launch_scatter_u32(ctx, cnt_o, d_ids, (int) mo, d_counts));
    return SKM_OK;
}

} // namespace

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

    // Candidate slots per point: a quarter of the centroids (every centroid when there is one batch).
    const uint32_t cap = (k <= SKM_Y_BATCH_SIZE) ? (uint32_t) align_up(k, 64)
                                                 : (uint32_t) std::min<size_t>(8192, std::max<size_t>(1024, align_up(k / 4, 64)));
    size_t chunk = ctx->workspace_limit / (size_t(cap) * sizeof(uint2));
    chunk = std::max<size_t>(128, (chunk / 128) * 128);
    chunk = std::min<size_t>(chunk, size_t(1) << 22);
    chunk = std::min(chunk, align_up(n, 128));
    const size_t cn = std::min(chunk, n);

    void* ws_counts = nullptr;
    SKM_TRY(workspace(ctx, 1, 2 * n * sizeof(uint32_t) + SKM_ACCT_COPIES * (n_hblocks + 2) * sizeof(unsigned long long) + 64, &ws_counts));
    unsigned long long* d_stage = (unsigned long long*) ws_counts;
    uint32_t* d_counts = (uint32_t*) (d_stage + SKM_ACCT_COPIES * (n_hblocks + 2));
    uint32_t* d_cursor = d_counts + n;  // place of every point in its list, for a walk split over several launches
    if (h_out_stage_pairs) SKM_TRY(skm_fill_u32(ctx, d_stage, 0u, 2 * SKM_ACCT_COPIES * (n_hblocks + 2)));
    unsigned long long* stage_arg = h_out_stage_pairs ? d_stage : nullptr;

    // Overflow ids of the whole call, then per-chunk scalars: best0, thr0, candidate counts.
    void* ws_chunk = nullptr;
    SKM_TRY(workspace(ctx, 2, n * sizeof(uint64_t) + cn * 3 * sizeof(uint32_t) + 256, &ws_chunk));
    uint64_t* d_over_ids = (uint64_t*) ws_chunk;
    float* d_best0 = (float*) (d_over_ids + n);
    float* d_thr0 = d_best0 + cn;
    uint32_t* d_cand_count = (uint32_t*) (d_thr0 + cn);
    uint32_t* d_n_over = d_cand_count + cn;

    // The order the last centroid update left, when it covers exactly these points and they are one chunk.
    const uint32_t* order = (chunk >= n && ctx->cluster_order_n == n) ? ctx->cluster_order : nullptr;
    const SearchOperands o{d_c, d_pdx, d_aux, d_ratios, d_cnorm_p, k, d, vertical_d, partial_d};
    for (size_t i0 = 0; i0 < n; i0 += chunk) {
        const size_t m = std::min(chunk, n - i0);
        void* ws_cand = nullptr;
        SKM_TRY(workspace(ctx, 0, m * size_t(cap) * sizeof(uint2), &ws_cand));
        SKM_TRY(search_chunk(ctx, o, d_x + i0 * d, m, d_xnorm_p + i0, cap, (uint2*) ws_cand, d_best0, d_thr0, d_cand_count,
                             d_inout_idx + i0, d_out_dist + i0, d_counts + i0, stage_arg, order, d_over_ids, d_n_over,
                             (uint64_t) i0, i0 == 0, d_cursor + i0));
    }
    // Points whose list overflowed (loose seeds, or points with no centroid nearby) are searched again through dense
    // rows of partial distances.  The sum of the
    // per-point counts is queued before the number of overflowing points is known and both arrive with one wait;
    // it is taken again only if a redo changed some counts.
    double* h_not_pruned = nullptr;
    uint32_t* h_n_over = nullptr;
    SKM_TRY(overflow_count_slot(ctx, &h_n_over));
    if (h_out_not_pruned) {
        // the reduction's last block also leaves the number of overflowing points in its host slot
        SKM_TRY(reduce_u32_sum_enqueue(ctx, d_counts, n, &h_not_pruned, d_n_over, h_n_over));
    } else {
        SKM_HIP_TRY(hipMemcpyAsync(h_n_over, d_n_over, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    }
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    const size_t mo = *(volatile uint32_t*) h_n_over;
    ctx->last_overflow_points = mo;
    if (mo > 0) {
        ScopedStage st(ctx, "search/overflow");
        SKM_TRY(redo_with_dense_rows(ctx, o, d_x, d_over_ids, mo, d_xnorm_p, d_inout_idx, d_out_dist, d_counts, stage_arg));
    }
    if (h_out_not_pruned) {
        double total = *(volatile double*) h_not_pruned;
        if (mo > 0) SKM_TRY(reduce_u32_sum_to_host(ctx, d_counts, n, &total));
        *h_out_not_pruned = (uint64_t) total;
    }
    if (h_out_stage_pairs) {
        std::vector<unsigned long long> tmp(SKM_ACCT_COPIES * (n_hblocks + 2));
        SKM_HIP_TRY(hipMemcpyAsync(tmp.data(), d_stage, tmp.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost,
                                   ctx->stream));
        SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
        for (size_t s = 0; s < tmp.size(); ++s) h_out_stage_pairs[s % (n_hblocks + 2)] += tmp[s];
    }
    return SKM_OK;
}
