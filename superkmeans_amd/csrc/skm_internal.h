// Internal glue shared by the translation units of libskm_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <map>
#include <string>
#include <vector>

#include "skm_hip.h"

struct skm_scope_timer {
    double ms = 0.0;
    uint64_t calls = 0;
};

struct skm_pending_interval {
    std::string scope;
    hipEvent_t start, stop;
};

struct skm_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    // Transfer stream of skm_upload_overlapped (created on first use) and the events that order it before `stream`.
    hipStream_t copy_stream = nullptr;
    hipEvent_t copy_done[8] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    unsigned copy_seq = 0;
    size_t workspace_limit = size_t(24) << 30;
    int candidate_kernel = 0;  // skm_ctx_set_candidate_kernel
    int walk_kernel = 0;       // skm_ctx_set_walk_kernel
    int walk_launches = 1;     // skm_ctx_set_walk_launches
    uint64_t last_overflow_points = 0;  // skm_ctx_get_last_overflow
    // Grow-only scratch buffers, one per role, so that stages never free inside a hot loop.
    static constexpr int WS_SLOTS = 6;
    void* ws[WS_SLOTS] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    size_t ws_bytes[WS_SLOTS] = {0, 0, 0, 0, 0, 0};
    // Point ids grouped by assignment, as the last centroid update sorted them (workspace slot 4, valid for
    // cluster_order_n points).  The pruned search visits the points in this order: neighbours in it share their
    // centroid row and most of their candidate blocks, which then come from the cache of the compute die that
    // fetched them first.  Any permutation of the points gives the same results.
    const uint32_t* cluster_order = nullptr;
    size_t cluster_order_n = 0;
    // "Blocks done" counter of the single-launch reductions (device memory, zero between launches).
    uint32_t* d_reduction_counter = nullptr;
    // One pinned host block: result slots of the reductions, a copy of the cluster sizes written by the kernel that
    // scales the sums, and a ring that kernels read small host-made tables from (row edits); h_ring_used is the
    // ring's fill.
    size_t h_ring_used = 0;
    void* h_pinned = nullptr;
    size_t h_pinned_bytes = 0;
    // Lanes of a large download (skm_download of DOWNLOAD_LANES_MIN_BYTES or more into pageable memory): a stream
    // and a pinned staging block each, made on first use.
    static constexpr int DOWNLOAD_LANES = 4;
    hipStream_t download_stream[DOWNLOAD_LANES] = {nullptr, nullptr, nullptr, nullptr};
    void* download_staging = nullptr;  // DOWNLOAD_LANES blocks of DOWNLOAD_CHUNK bytes
    // Address, on this context's device, of the library's static scratch array (skm_assign_full_noalloc).
    void* noalloc_scratch = nullptr;
    bool prof = false;
    std::map<std::string, skm_scope_timer> timers;
    std::vector<skm_pending_interval> pending;
    std::vector<hipEvent_t> event_pool;
};

namespace skm {

int set_error(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);

#define SKM_HIP_TRY(expr)                                                                          \
    do {                                                                                           \
        int _rc = ::skm::check_hip((expr), #expr);                                                 \
        if (_rc != SKM_OK) return _rc;                                                             \
    } while (0)

#define SKM_TRY(expr)                                                                              \
    do {                                                                                           \
        int _rc = (expr);                                                                          \
        if (_rc != SKM_OK) return _rc;                                                             \
    } while (0)

#define SKM_REQUIRE(cond, msg)                                                                     \
    do {                                                                                           \
        if (!(cond)) return ::skm::set_error(SKM_ERR_INVALID, "%s: %s", __func__, msg);           \
    } while (0)

// Device blocks through the per-device cache of released blocks (skm_context.hip).
int device_alloc(int device, size_t bytes, void** out);
int device_release(int device, void* ptr);

// Returns a scratch buffer of at least `bytes` for slot `slot` (grow-only).
int workspace(skm_ctx* ctx, int slot, size_t bytes, void** out);
int pinned(skm_ctx* ctx, size_t bytes, void** out);
int reduction_counter(skm_ctx* ctx, uint32_t** out);
int host_ring(skm_ctx* ctx, void** out, size_t* out_bytes);
int pinned_sizes(skm_ctx* ctx, uint32_t** out, size_t* out_entries);

// RAII device timer for one profiler scope; no-op unless profiling is enabled.
class ScopedStage {
  public:
    ScopedStage(skm_ctx* ctx, const char* scope);
    ~ScopedStage();

  private:
    skm_ctx* ctx_;
    bool active_ = false;
    skm_pending_interval iv_;
};

int resolve_pending(skm_ctx* ctx);

// Device address of the static scratch array of skm_assign_full_noalloc on `device` (which must be the current
// device); resolved once per device and kept.
int resolve_noalloc_scratch(int device, void** out);

// ---- launchers implemented in the kernel translation units ----

// D = A . B^T stored row-major (ldo), optionally turned into squared distances
// out[m][n] = -2 * D[m][n] + row_norm[m] + col_norm[n] when both norm pointers are non-null.
int launch_gemm_store(skm_ctx* ctx, const float* A, int M, int64_t lda, const float* B, int N,
                      int64_t ldb, int K, float* out, int64_t ldo, const float* row_norm,
                      const float* col_norm);

// Per (granule of consecutive centroids, point) minimum of -2 x.c + |x|^2 + |c|^2 and its lowest index,
// written as uint2 {float bits, index} to granule_min[granule * n + point].  The granule size (64 or 128,
// a divisor of the 1024-centroid batch) follows from the tile shape picked for the problem size.
int gemm_argmin_granule(int k, int n);
int launch_gemm_argmin(skm_ctx* ctx, const float* C, int k, const float* X, int n, int d,
                       int64_t ldc, int64_t ldx, const float* xnorm, const float* cnorm,
                       uint2* granule_min, int granule);

int launch_merge_granules(skm_ctx* ctx, const uint2* granule_min, int n, int k, int granule, uint32_t* out_idx,
                          float* out_dist);

// Number of striped copies of the per-stage accounting counters (each n_hblocks + 2 entries long).
constexpr int SKM_ACCT_COPIES = 64;

int launch_gemm_candidates(skm_ctx* ctx, const float* C, int k, const float* X, int n, int partial_d, int64_t ld,
                           const float* xnorm_p, const float* cnorm_p, const float* thr0, uint32_t* cand_count,
                           uint2* cand, uint32_t cap);
// The same for short d' (the points stay in registers); `serves` says whether a call qualifies.
bool gemm_candidates_stationary_serves(const float* C, int k, const float* X, int n, int partial_d, int64_t ld,
                                       bool whatever_n);
int launch_gemm_candidates_stationary(skm_ctx* ctx, const float* C, int k, const float* X, int n, int partial_d, int64_t ld,
                                      const float* xnorm_p, const float* cnorm_p, const float* thr0,
                                      uint32_t* cand_count, uint2* cand, uint32_t cap);
// `order`: null, or a permutation of the n points giving the sequence in which wavefronts take them.
// launch_prune_list with dense_partial non-null: the points have rows of partial distances to all centroids
// (n_chunk x ld_partial) instead of lists (cand, cand_count, over_ids and n_over are then unused).
int launch_seed_distance(skm_ctx* ctx, const float* x, const float* c, const uint32_t* idx, int n, int d,
                         const float* ratios, int partial_d, float* best0, float* thr0, const uint32_t* order,
                         uint32_t* zero_this);
int launch_prune_list(skm_ctx* ctx, const uint2* cand, const uint32_t* cand_count, uint32_t cap, const float* best0,
                      const float* x, int n_chunk, const float* pdx, const float* aux, int k, int d, int vertical_d,
                      int partial_d, const float* ratios, uint32_t* inout_idx, float* out_dist, uint32_t* out_not_pruned,
                      unsigned long long* d_stage_pairs, const uint32_t* order, uint64_t* over_ids, uint32_t* n_over,
                      uint64_t id_offset, const float* dense_partial, int64_t ld_partial);
// The same walk with several points per wavefront (rows 16-byte aligned, d a multiple of 4); `serves` says whether a
// call qualifies.  Same results bit for bit.  One launch walks the batches [jb_lo, jb_hi) of 1024 centroids; a walk
// split over several launches (ascending ranges) keeps its place in `cursor` (n_chunk words).  points_per_wavefront: 4, 8,
// or 0 for the choice by the number of points.
bool prune_pool_serves(const float* x, const float* pdx, int d);
int launch_prune_pool(skm_ctx* ctx, const uint2* cand, const uint32_t* cand_count, uint32_t cap, const float* best0,
                      const float* x, int n_chunk, const float* pdx, const float* aux, int k, int d, int vertical_d,
                      int partial_d, const float* ratios, uint32_t* inout_idx, float* out_dist, uint32_t* out_not_pruned,
                      unsigned long long* d_stage_pairs, const uint32_t* order, uint64_t* over_ids, uint32_t* n_over,
                      uint64_t id_offset, int jb_lo, int jb_hi, uint32_t* cursor, int points_per_wavefront);
int launch_gather_u32(skm_ctx* ctx, const uint32_t* in, const uint64_t* ids, int m, uint32_t* out);
int launch_scatter_u32(skm_ctx* ctx, const uint32_t* in, const uint64_t* ids, int m, uint32_t* out);

} // namespace skm
