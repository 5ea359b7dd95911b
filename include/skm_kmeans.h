/* C ABI over the skmeans::SuperKMeans / skmeans::HierarchicalSuperKMeans objects of the HIP backend.
 *
 * This is the boundary a foreign-function binding attaches to: it carries exactly the calls the
 * reference exposes through its pybind11 module (python/bindings/bindings.cpp:158-378,433-670:
 * constructor with config, train, assign, assign_training_points, get_n_clusters, is_trained,
 * iteration_stats) with plain pointers and sizes.  Two entry points have no counterpart in the
 * reference and exist for callers whose data already lives in HBM: skm_kmeans_train_device and
 * skm_kmeans_assign_device.
 *
 * Errors: 0 on success; SKM_ERR_INVALID for what the reference reports as std::invalid_argument,
 * SKM_ERR_RUNTIME for std::runtime_error (superkmeans.h:125-131,168-190,404-406); text through
 * skm_last_error().
 */
#ifndef SKM_KMEANS_H
#define SKM_KMEANS_H

#include "skm_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define SKM_ERR_RUNTIME (-5)

/* SuperKMeansConfig (superkmeans.h:23-55) followed by the three fields of
 * HierarchicalSuperKMeansConfig (hierarchical_superkmeans.h:11-17); booleans are int32. */
typedef struct skm_kmeans_config {
    uint32_t iters;
    float sampling_fraction;
    uint32_t max_points_per_cluster;
    uint32_t n_threads;
    uint32_t seed;
    int32_t use_blas_only;
    float tol;
    float recall_tol;
    int32_t early_termination;
    int32_t sample_queries;
    uint64_t objective_k;
    float ann_explore_fraction;
    float min_not_pruned_pct;
    float max_not_pruned_pct;
    float adjustment_factor_for_partial_d;
    int32_t unrotate_centroids;
    int32_t verbose;
    int32_t angular;
    int32_t suppress_warnings;
    int32_t data_already_rotated;
    uint32_t iters_mesoclustering;
    uint32_t iters_fineclustering;
    uint32_t iters_refinement;
    /* Rotation variant; a build option of the reference (pdx/adsampling.h:52-74), a field here:
     * 0 dense Gaussian matrix, 1 sign flip + DCT-II when d >= 512 and d is a power of two, 2 DCT
     * whenever d >= 512. */
    int32_t dct_rotation;
} skm_kmeans_config;

/* SuperKMeansIterationStats (superkmeans.h:60-72). */
typedef struct skm_kmeans_iteration_stats {
    uint64_t iteration;
    float objective;
    float shift;
    uint64_t split;
    float recall;
    float not_pruned_pct;
    uint32_t partial_d;
    int32_t is_gemm_only;
} skm_kmeans_iteration_stats;

typedef struct skm_kmeans skm_kmeans;

/* Defaults of the reference structs; hierarchical != 0 sets sampling_fraction = 1. */
void skm_kmeans_default_config(skm_kmeans_config* out, int hierarchical);

int skm_kmeans_create(size_t n_clusters, size_t dimensionality, const skm_kmeans_config* config, int hierarchical,
                      skm_kmeans** out);
int skm_kmeans_destroy(skm_kmeans* km);

/* Train (superkmeans.h:162 / hierarchical_superkmeans.h:84): h_data is n x d row-major on the host;
 * h_out_centroids receives k x d floats. */
int skm_kmeans_train(skm_kmeans* km, const float* h_data, size_t n, const float* h_queries, size_t n_queries,
                     float* h_out_centroids);
/* Same with d_data (and d_queries, when n_queries > 0 and queries are not sampled) already in device
 * memory (no counterpart in the reference). */
int skm_kmeans_train_device(skm_kmeans* km, const float* d_data, size_t n, const float* d_queries,
                            size_t n_queries, float* h_out_centroids);

/* Assign (superkmeans.h:346): exact nearest centroid of each of the n vectors. */
int skm_kmeans_assign(skm_kmeans* km, const float* h_vectors, const float* h_centroids, size_t n_vectors,
                      size_t n_centroids, uint32_t* h_out_assignments);
/* Same on device-resident inputs and output; synchronises before returning (no counterpart in the reference). */
int skm_kmeans_assign_device(skm_kmeans* km, const float* d_vectors, const float* d_centroids, size_t n_vectors,
                             size_t n_centroids, uint32_t* d_out_assignments);
/* AssignTrainingPoints (superkmeans.h:397). */
int skm_kmeans_assign_training_points(skm_kmeans* km, const float* h_vectors, const float* h_centroids,
                                      size_t n_vectors, size_t n_centroids, uint32_t* h_out_assignments);

/* The centroid each of the vectors of the last skm_kmeans_assign_training_points started its pruned search from: the
 * training assignment, a size-weighted draw or the representative of the nearest meso-centroid, by the branch of
 * superkmeans.h:454-563 (the reference builds them in place in its result array; kept here so that a binding's tests
 * can compare them).  count must equal that call's n_vectors; SKM_ERR_RUNTIME when there was no such call or it fell
 * back to Assign. */
int skm_kmeans_get_training_seeds(skm_kmeans* km, uint32_t* h_out, size_t count);
/* How many vectors of that call left more candidates than a candidate list holds and went through the second pass of
 * the pruned search (no counterpart in the reference, whose search keeps no lists; 0 before the first call). */
int skm_kmeans_get_training_overflow(skm_kmeans* km, uint64_t* out_points);

/* Test hook, no counterpart in the reference: SplitClusters of the object's class (flat: superkmeans.h:890-928;
 * hierarchical: hierarchical_superkmeans.h:579-678) on a given state.  h_centroids (k x d) and h_sizes (k) are replaced
 * by the edited rows and sizes, out_n_split receives the number of splits.  Untrained objects only. */
int skm_kmeans_split_clusters_on_state(skm_kmeans* km, float* h_centroids, uint32_t* h_sizes, size_t k, size_t n_samples,
                                       uint64_t* out_n_split);

int skm_kmeans_get_n_clusters(skm_kmeans* km, size_t* out);
int skm_kmeans_is_trained(skm_kmeans* km, int* out);
/* which: 0 iteration_stats (flat), 1 mesoclustering, 2 fineclustering, 3 refinement. */
int skm_kmeans_n_stats(skm_kmeans* km, int which, size_t* out);
int skm_kmeans_get_stats(skm_kmeans* km, int which, skm_kmeans_iteration_stats* out, size_t capacity);
/* Public member `assignments` (superkmeans.h:1491): assignments of the training samples. */
int skm_kmeans_get_assignments(skm_kmeans* km, uint32_t* h_out, size_t count);
/* The device context of the object: use it for skm_malloc / skm_upload of device-resident inputs
 * and for the per-stage device timers. */
int skm_kmeans_context(skm_kmeans* km, skm_ctx** out);
/* Pruning accounting (no counterpart in the reference): when enabled before Train, every pruned
 * iteration records the number of (point, centroid) pairs entering each pruning step.
 * skm_kmeans_get_prune_accounting copies row `iteration` (0-based over pruned iterations) into
 * h_out (capacity entries) and writes the row length to out_len; out_rows receives the row count. */
int skm_kmeans_set_prune_accounting(skm_kmeans* km, int enabled);
int skm_kmeans_get_prune_accounting(skm_kmeans* km, size_t iteration, uint64_t* h_out, size_t capacity,
                                    size_t* out_len, size_t* out_rows);
/* PDXLayout::GetDimensionSplit (pdx/layout.h:115-140) as used by the host code. */
void skm_dimension_split(size_t d, size_t* out_horizontal_d, size_t* out_vertical_d);
/* ADSamplingPruner matrix and ratios as built by the host code for (d, epsilon0, seed) and the
 * rotation variant `rotation_kind` (the values of skm_kmeans_config.dct_rotation): fills
 * h_out_matrix (d*d, may be NULL) and h_out_ratios (d+1, may be NULL). Needs a device. */
int skm_pruner_tables(size_t d, float epsilon0, uint32_t seed, int rotation_kind, float* h_out_matrix,
                      float* h_out_ratios);

#ifdef __cplusplus
}
#endif
#endif /* SKM_KMEANS_H */
