/* C ABI of libskm_hip.so: the MI355X (gfx950) device side of the Super K-Means
 * assign/update hot path.
 *
 * The reference library is header-only C++ whose per-point work is done by
 * BLAS sgemm_, OpenMP loops and AVX/NEON kernels.  Each entry point below
 * replaces one of those CPU routines with hand-written HIP kernels; the cited
 * file:line is the reference routine it stands in for (paths relative to the
 * reference's include/superkmeans/).  Host C++ (the headers under include/superkmeans) and
 * the language bindings call only this header; no HIP type crosses it.
 *
 * Conventions
 *   - every function returns 0 on success and a negative code on failure;
 *     skm_last_error() returns the message of the calling thread's last failure;
 *   - pointers named d_* are device pointers obtained from skm_malloc (or any
 *     other HIP allocation on the context's device); h_* are host pointers;
 *   - matrices are row-major fp32, indices are uint32_t, counts are uint32_t
 *     unless stated;
 *   - work is enqueued on the context's stream; functions that return a value
 *     through a host pointer synchronise that stream before returning, all
 *     others are asynchronous with respect to the host;
 *   - a context is not thread-safe (the reference objects are not either,
 *     superkmeans.h:132-133).
 */
#ifndef SKM_HIP_H
#define SKM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SKM_OK 0
#define SKM_ERR_INVALID (-1) /* bad argument (null pointer, zero size, size over a limit) */
#define SKM_ERR_HIP (-2)     /* a HIP runtime call failed                                  */
#define SKM_ERR_NO_DEVICE (-3)
#define SKM_ERR_OOM (-4)

/* Tuning constants of the reference (common.h:89-115) that shape device work. */
#define SKM_H_DIM_SIZE 64
#define SKM_Y_BATCH_SIZE 1024
#define SKM_X_BATCH_SIZE 4096

typedef struct skm_ctx skm_ctx;

const char* skm_last_error(void);
int skm_device_count(int* out_count);

/* One context = one device + one HIP stream + reusable workspace. */
int skm_ctx_create(int device, skm_ctx** out_ctx);
int skm_ctx_destroy(skm_ctx* ctx);
int skm_sync(skm_ctx* ctx);
/* Upper bound, in bytes, of the scratch a single stage call may allocate (default 24 GiB of the
 * 288 GB of HBM: large enough that the headline shapes run as one launch per stage). */
int skm_ctx_set_workspace_limit(skm_ctx* ctx, size_t bytes);

/* Which kernel computes the partial distances of skm_assign_pruned (tuning and test knob; results do not depend on
 * it): 0 = automatic (default: the register-stationary kernel for partial_d <= 160 and at least 49,152 points per
 * call, the kernel with 256 x 256 tiles for partial_d > 160 and at least 49,152 points, the tiled 128 x 128 kernel
 * otherwise), 1 = always the 128 x 128 kernel, 2 = the register-stationary kernel whenever partial_d <= 160 and the rows
 * are 16-byte aligned, whatever the number of points, 3 = always the 256 x 256 kernel. */
int skm_ctx_set_candidate_kernel(skm_ctx* ctx, int which);

/* Which kernel walks the candidate lists of skm_assign_pruned (tuning and test knob; results do not depend on it):
 * 0 = automatic (default: several points pooled per wavefront for calls of at least 32,768 points whose rows are
 * 16-byte aligned with d a multiple of 4, eight points from 500,000 points on and four below; one point per wavefront
 * otherwise), 1 = always one point per wavefront, 2 / 3 = pooled with four / eight points per wavefront wherever the
 * rows allow it.  The second pass over points whose list overflowed always takes one point per wavefront. */
int skm_ctx_set_walk_kernel(skm_ctx* ctx, int which);
/* Into how many launches the pooled walk of a call is split, each over a contiguous range of the batches of 1024
 * centroids, all points walking one range before any walks the next (default 1; capped at the number of batches;
 * results do not depend on it).  With one launch per batch the compute dies gather from one batch's blocks at a time
 * and less than half as many gathers miss their L2, but the launches' tails and the reloaded per-point state cost
 * more time than the misses did, which the memory-side cache serves: a knob for measuring that trade. */
int skm_ctx_set_walk_launches(skm_ctx* ctx, int launches);
/* How many points of the last skm_assign_pruned call on this context collected more candidates than their list holds
 * and went through the second pass over dense rows of partial distances (a measure of how loose the seeds were). */
int skm_ctx_get_last_overflow(skm_ctx* ctx, uint64_t* out_points);

/* Device memory and transfers (stand in for the reference's std::unique_ptr<float[]> buffers,
 * superkmeans.h:191-201). */
int skm_malloc(skm_ctx* ctx, size_t bytes, void** out_d_ptr);
/* Waits for this context's streams, then hands the block to the per-device cache below, from which the next allocation
 * of about its size, by any context of the process, may take it at once.  No other context and no other stream may
 * still have work queued that uses the block when it is freed. */
int skm_free(skm_ctx* ctx, void* d_ptr);
/* Blocks released through skm_free, by a context's workspace or by skm_ctx_destroy are kept per device and handed
 * out again by later allocations of about the same size (allocating and releasing the multi-gigabyte buffers of a
 * Train costs milliseconds each time, and a release waits for the whole device).  The cache holds at most 48 GiB
 * (or the number of bytes in SKM_DEVICE_CACHE_BYTES when the process first uses the device; 0 keeps nothing) and
 * 2,048 blocks, and empties itself when an allocation of this process fails.  Other processes on the same GPU do not
 * see these blocks as free: lower the limit, or trim, where the GPU is shared. */
int skm_device_cache_set_limit(int device, size_t bytes); /* blocks beyond the new limit go back to the driver */
int skm_device_cache_trim(int device);                    /* returns every idle block to the driver */
int skm_upload(skm_ctx* ctx, void* d_dst, const void* h_src, size_t bytes);
int skm_download(skm_ctx* ctx, void* h_dst, const void* d_src, size_t bytes);
/* Upload on the context's transfer stream: work queued on the context before the call keeps running during the
 * copy, work queued after it starts when the copy is complete.  Lets Train/Assign on host pointers (reference
 * superkmeans.h:162,346 take host pointers only) compute on one slab of rows while the next one is on its way.
 * d_dst must not be in use by work queued earlier.  A pageable h_src has been read when the call returns (the
 * runtime stages it); pinned memory must stay unchanged until the context is synchronised (skm_sync,
 * skm_download or skm_upload). */
int skm_upload_overlapped(skm_ctx* ctx, void* d_dst, const void* h_src, size_t bytes);
/* Upload on the context's transfer stream that returns when the bytes are in device memory and leaves the context's
 * own stream alone: meant for a second host thread that feeds slabs of rows while the first one queues the work on
 * the slabs that have arrived (AssignTrainingPoints, reference superkmeans.h:397, takes host pointers only).  One
 * transfer per context at a time (this call or skm_upload_overlapped).  The first call on a context makes its transfer
 * stream: make that call (zero bytes will do) on the thread that owns the context before a feeder thread starts.
 * d_dst must not be in use by queued work. */
int skm_upload_detached(skm_ctx* ctx, void* d_dst, const void* h_src, size_t bytes);
int skm_copy(skm_ctx* ctx, void* d_dst, const void* d_src, size_t bytes);
int skm_fill_u32(skm_ctx* ctx, void* d_dst, uint32_t value, size_t count);

/* Per-stage device timers, named like the reference's profiler scopes (profiler.h:296-312;
 * "search/1st_blas", "search/blas", "search/pdx", "rotator", "update_centroids", ...).
 * While enabled every stage brackets its kernels with events on the context's stream. */
int skm_prof_enable(skm_ctx* ctx, int enabled);
int skm_prof_reset(skm_ctx* ctx);
/* Sum of device milliseconds and number of recorded intervals of one scope (synchronises). */
int skm_prof_get(skm_ctx* ctx, const char* scope, double* out_ms, uint64_t* out_calls);
/* Writes "name=ms/calls;" pairs for every scope seen; returns needed length incl. NUL. */
int skm_prof_dump(skm_ctx* ctx, char* h_buf, size_t buf_len, size_t* out_needed);

/* Row-wise squared L2 norms over the first `cols` columns of an rows x d matrix.
 * cols == d : GetL2NormsRowMajor (superkmeans.h:1162-1171)
 * cols <  d : GetPartialL2NormsRowMajor (superkmeans.h:1147-1157) */
int skm_norms(skm_ctx* ctx, const float* d_m, size_t rows, size_t d, size_t cols, float* d_out);

/* out(n x d) = X(n x d) . Q^T with Q row-major d x d: ADSamplingPruner::Rotate,
 * pdx/adsampling.h:156-216 (sgemm_('T','N') with the pruner's matrix). MFMA GEMM. */
int skm_rotate(skm_ctx* ctx, const float* d_x, size_t n, size_t d, const float* d_q, float* d_out);
/* out(n x d) = R(n x d) . Q, given Q^T (row-major transpose of Q): ADSamplingPruner::Unrotate,
 * pdx/adsampling.h:223-299. */
int skm_unrotate(skm_ctx* ctx, const float* d_r, size_t n, size_t d, const float* d_qt, float* d_out);
/* out(cols x rows) = in(rows x cols)^T (used once to keep Q^T next to Q). */
int skm_transpose(skm_ctx* ctx, const float* d_in, size_t rows, size_t cols, float* d_out);

/* PDXLayout::PDXify<false> (pdx/layout.h:155-232) plus CentroidsToAuxiliaryHorizontal
 * (superkmeans.h:1206-1212): per chunk of 1024 centroids the first vertical_d dimensions are
 * written dimension-major, the remaining ones as 64-wide row-major blocks; d_aux (k x vertical_d)
 * receives a dense copy of the first vertical_d columns (may be NULL).
 * vertical_d must equal GetDimensionSplit(d).vertical_d (pdx/layout.h:115-140). */
int skm_pdxify(skm_ctx* ctx, const float* d_c, size_t k, size_t d, size_t vertical_d, float* d_pdx,
               float* d_aux);

/* BatchComputer::FindNearestNeighbor (distance_computers/batch_computers.h:104-171): exact top-1 of
 * every row of X among the k rows of C using ||x||^2 + ||c||^2 - 2 x.c, evaluated per batch of 1024
 * centroids in ascending order with the reference's update rule (strict <, clamp at 0, lowest
 * index on ties).  d_xnorm / d_cnorm are full squared norms. */
int skm_assign_full(skm_ctx* ctx, const float* d_x, size_t n, const float* d_c, size_t k, size_t d,
                    const float* d_xnorm, const float* d_cnorm, uint32_t* d_out_idx, float* d_out_dist);

/* skm_assign_full for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and
 * bit-identical results; the per-(granule of centroids, point) minima that skm_assign_full keeps in the context's
 * workspace live in a static device array of SKM_NOALLOC_SCRATCH_BYTES that every GPU running the library holds
 * until the process ends.  The call allocates and releases nothing (its address was resolved by skm_ctx_create)
 * and records no device timers.  Points are processed in chunks that fit the array, so n is not limited;
 * k > SKM_NOALLOC_MAX_CENTROIDS is rejected with SKM_ERR_INVALID.  All calls on one GPU share the array: calls
 * that overlap in time on the same GPU (two contexts, two threads) race; nothing in it has to be cleared
 * between calls (every entry a merge reads was written by the launch before it). */
#define SKM_NOALLOC_SCRATCH_BYTES (32u << 20)
#define SKM_NOALLOC_MAX_CENTROIDS 2097152 /* 128 points x ceil(k / 64) granules x 8 bytes fill the array */
int skm_assign_full_noalloc(skm_ctx* ctx, const float* d_x, size_t n, const float* d_c, size_t k, size_t d,
                            const float* d_xnorm, const float* d_cnorm, uint32_t* d_out_idx, float* d_out_dist);

/* BatchComputer::FindNearestNeighborWithPruning (batch_computers.h:297-409) with
 * PDXearch::Top1PartialSearchWithThresholdAndPartialDistances / Prune / SetBestCandidate
 * (pdx/pdxearch.h:118-238,266-327).
 *   d_c        row-major centroids (GEMM operand and seed distance, batch_computers.h:372-377)
 *   d_pdx      the same centroids in PDX layout, d_aux their first vertical_d columns
 *   d_ratios   d + 1 floats, ADSamplingPruner::ratios (pdx/adsampling.h:93-99)
 *   d_xnorm_p / d_cnorm_p  squared norms over the first partial_d columns
 *   d_inout_idx in: previous assignment (seed; every entry below k, the search reads that centroid's row); out:
 *               new assignment
 *   d_out_dist  out: squared distance to the new assignment (unclamped, as the reference)
 *   h_out_not_pruned  sum over points of the per-point not-pruned counts (input of TunePartialD,
 *                     superkmeans.h:1230-1241); synchronises.
 *   h_out_stage_pairs optional array of (d - vertical_d) / 64 + 2 counters: live (point, centroid)
 *                     pairs entering each pruning step (algorithmic-bytes accounting); may be NULL. */
int skm_assign_pruned(skm_ctx* ctx, const float* d_x, size_t n, const float* d_c, const float* d_pdx,
                      const float* d_aux, size_t k, size_t d, size_t vertical_d, uint32_t partial_d,
                      const float* d_ratios, const float* d_xnorm_p, const float* d_cnorm_p,
                      uint32_t* d_inout_idx, float* d_out_dist, uint64_t* h_out_not_pruned,
                      uint64_t* h_out_stage_pairs);

/* SuperKMeans::UpdateCentroids (superkmeans.h:729-765): sums[c] = sum of rows assigned to c, taken
 * in ascending point order per centroid exactly like the reference's per-thread scan, and
 * sizes[c] = number of such rows.  No floating-point atomics: point ids are stably sorted by
 * assignment and each centroid's segment is reduced by one workgroup. */
int skm_update(skm_ctx* ctx, const float* d_x, size_t n, size_t d, const uint32_t* d_idx, size_t k,
               float* d_out_sums, uint32_t* d_out_sizes);
/* First loop of SuperKMeans::ConsolidateCentroids (superkmeans.h:940-951): c *= float(1.0 / size)
 * for every non-empty cluster. */
int skm_scale_by_size(skm_ctx* ctx, float* d_sums, const uint32_t* d_sizes, size_t k, size_t d);
/* The same, and the sizes arrive in h_sizes (k entries) with the one wait on the stream the call ends with: the next
 * step of ConsolidateCentroids, SplitClusters, decides on the host from the sizes. */
int skm_scale_by_size_fetch(skm_ctx* ctx, float* d_sums, const uint32_t* d_sizes, size_t k, size_t d, uint32_t* h_sizes);
/* SuperKMeans::PostprocessCentroids (superkmeans.h:1357-1371): c /= ||c||. */
int skm_normalize_rows(skm_ctx* ctx, float* d_c, size_t k, size_t d);
/* Row edits of SplitClusters (superkmeans.h:905-920; hierarchical_superkmeans.h:606-625,665-673),
 * applied in list order.  op[4*i] = kind (0: copy row src->dst then perturb dst by (1 +/- eps) and
 * src by (1 -/+ eps) alternating per column; 1: dst = (w * dst + src) / (w + 1)), op[4*i+1] = dst,
 * op[4*i+2] = src, op[4*i+3] = bit pattern of float w. */
int skm_edit_rows(skm_ctx* ctx, float* d_c, size_t d, const uint32_t* h_ops, size_t n_ops);
/* SuperKMeans::ComputeCost (superkmeans.h:973-981): sum of n distances, accumulated in fp64 with a
 * fixed reduction tree. */
int skm_wcss(skm_ctx* ctx, const float* d_dist, size_t n, double* h_out_cost);
/* The same in two steps, for callers that have other work to queue in between: skm_wcss_begin queues the reduction
 * (d_dist must stay unchanged until it has run), skm_wcss_end waits for the stream and returns the sum of the last
 * skm_wcss_begin on this context.  Same reduction tree, same result as skm_wcss. */
int skm_wcss_begin(skm_ctx* ctx, const float* d_dist, size_t n);
int skm_wcss_end(skm_ctx* ctx, double* h_out_cost);
/* SuperKMeans::ComputeShift (superkmeans.h:988-998): sum_c ||new_c - prev_c||^2. */
int skm_shift(skm_ctx* ctx, const float* d_new, const float* d_prev, size_t k, size_t d,
              double* h_out_shift);
/* HierarchicalSuperKMeans::CompactMesoclusterToBuffer (hierarchical_superkmeans.h:685-704):
 * out[j] = X[index[j]], norms_out[j] = norms_in[index[j]] (norm pointers may be NULL). */
int skm_gather_rows(skm_ctx* ctx, const float* d_x, size_t d, const uint64_t* d_index, size_t m,
                    float* d_out, const float* d_norms_in, float* d_norms_out);
/* The partitioned index HierarchicalSuperKMeans::Train builds between its mesoclustering and its fine clustering
 * (hierarchical_superkmeans.h:270-286): d_out_ids lists the n points grouped by assignment, ascending inside each
 * group, as 64-bit row ids for skm_gather_rows, and d_out_sizes[c] is the number of points assigned to c.  Runs the
 * stable sort of skm_update on the device instead of a counting sort over a host copy of the assignments. */
int skm_group_by_assignment(skm_ctx* ctx, const uint32_t* d_idx, size_t n, size_t k, uint64_t* d_out_ids,
                            uint32_t* d_out_sizes);
/* GetTrueAssignmentsFromIndirectionBuffer (hierarchical_superkmeans.h:763-779):
 * out[index[j]] = local[j] + offset. */
int skm_scatter_assignments(skm_ctx* ctx, const uint64_t* d_index, const uint32_t* d_local, size_t m,
                            uint32_t offset, uint32_t* d_out);
/* The seeding of the unsampled points in AssignTrainingPoints (superkmeans.h:553-560): every entry of d_seeds that
 * holds 0xffffffff becomes d_representative[d_group[i]] (the point's nearest meso-centroid, and one centroid of that
 * meso-cluster; d_representative has n_groups entries and a group at or past n_groups counts as the last one); the
 * other entries, the training assignments of the sampled points, stay. */
int skm_seeds_from_groups(skm_ctx* ctx, uint32_t* d_seeds, const uint32_t* d_group, const uint32_t* d_representative,
                          size_t n_groups, size_t n);
/* BatchComputer::FindKNearestNeighbors (batch_computers.h:191-274): for every row of x the k rows of
 * y with the smallest -2 x.y + ||x||^2 + ||y||^2, ordered by (distance, index), y taken in batches of
 * 1024 rows: entries kept from earlier batches compete with their distance clamped at 0, the result
 * is clamped at 0; slots beyond n_y hold {FLT_MAX, 0xffffffff}.  k <= 1024.
 * d_out_idx / d_out_dist: n_x * k. */
int skm_knn(skm_ctx* ctx, const float* d_x, size_t n_x, const float* d_y, size_t n_y, size_t d,
            const float* d_xnorm, const float* d_ynorm, size_t k, uint32_t* d_out_idx, float* d_out_dist);
/* Inner loops of SuperKMeans::ComputeRecall (superkmeans.h:1064-1082): h_out_hits[q] = how many of
 * query q's objective_k ground-truth neighbours (row ids into the training sample) are assigned to one
 * of the query's `explore` promising centroids.  explore <= 1024.  The caller forms
 * sum_q (float) hits[q] / objective_k in query order, then divides by n_queries. */
int skm_recall_hits(skm_ctx* ctx, const uint32_t* d_gt, const uint32_t* d_promising,
                    const uint32_t* d_assignments, size_t n_assignments, size_t n_queries,
                    size_t objective_k, size_t explore, uint32_t* h_out_hits);

/* Orthogonal factor Q = H_0 H_1 ... H_{d-1} of the Householder QR of the d x d matrix h_a (row-major, double), as
 * float, into h_out_q.  The reference obtains its rotation matrix this way on the CPU (pdx/adsampling.h:76-85,
 * Eigen::HouseholderQR of a Gaussian matrix).  Evaluated on the device in double with the operations and the
 * summation order of skmeans::detail::OrthogonalFactor (superkmeans/pdx/adsampling.h), whose result it equals
 * bit for bit; d <= SKM_HOUSEHOLDER_Q_MAX_D (a workgroup keeps all rows of eight columns in LDS). */
#define SKM_HOUSEHOLDER_Q_MAX_D 2272
int skm_householder_q(skm_ctx* ctx, const double* h_a, size_t d, float* h_out_q);

/* Benchmark / test utility: seeded Gaussian-mixture rows generated in device memory.  Row i (logical
 * index row_offset + local row) is  s_j * (center_sigma * g(center_seed, u_i, j) + noise_sigma *
 * g(point_seed, i, j)),  s_j = (j + 1)^(-decay_exponent),  u_i = hash(i) mod n_centers (n_centers == 0:
 * pure noise), optionally L2-normalised.  Every value depends only on (seeds, i, j), so any slice can
 * be regenerated.  The reference's generator for its tests is MakeBlobs (pdx/utils.h:74-123), which
 * fills host memory from std::mt19937; there is no device counterpart in the reference. */
int skm_synth_gaussian_mixture(skm_ctx* ctx, float* d_out, size_t n, size_t d, size_t row_offset,
                               uint32_t n_centers, uint32_t center_seed, uint32_t point_seed,
                               float center_sigma, float noise_sigma, float decay_exponent, int normalize);

/* Same kind of utility for the other benchmark shapes: a two-level mixture (n_coarse coarse centres,
 * n_fine fine centres split evenly among them: x = coarse + fine_sigma * fine + noise_sigma * noise)
 * and low-intrinsic-dimension rows with heavy tails (x = A z + noise_scale * Student-t(3), z ~ N(0, I_rank),
 * A a fixed d x rank Gaussian map); rows are L2-normalised. */
int skm_synth_two_level_mixture(skm_ctx* ctx, float* d_out, size_t n, size_t d, size_t row_offset,
                                uint32_t n_coarse, uint32_t n_fine, uint32_t seed, float fine_sigma,
                                float noise_sigma);
int skm_synth_low_rank(skm_ctx* ctx, float* d_out, size_t n, size_t d, size_t row_offset, uint32_t rank,
                       uint32_t seed, float noise_scale);

#ifdef __cplusplus
}
#endif
#endif /* SKM_HIP_H */
