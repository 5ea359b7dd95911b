// extern "C" surface over the host classes in include/superkmeans/*.h (see include/skm_kmeans.h).
#include "skm_kmeans.h"

#include <cstring>
#include <memory>

#include "skm_internal.h"
#include "superkmeans/hierarchical_superkmeans.h"
#include "superkmeans/superkmeans.h"

namespace {

// Gives the C layer access to what the reference keeps public or returns by value.
class FlatModel : public skmeans::SuperKMeans<> {
  public:
    using skmeans::SuperKMeans<>::SuperKMeans;
};
class HierModel : public skmeans::HierarchicalSuperKMeans<> {
  public:
    using skmeans::HierarchicalSuperKMeans<>::HierarchicalSuperKMeans;
};

void fill_base(skmeans::SuperKMeansConfig& c, const skm_kmeans_config& in) {
    c.iters = in.iters;
    c.sampling_fraction = in.sampling_fraction;
    c.max_points_per_cluster = in.max_points_per_cluster;
    c.n_threads = in.n_threads;
    c.seed = in.seed;
    c.use_blas_only = in.use_blas_only != 0;
    c.tol = in.tol;
    c.recall_tol = in.recall_tol;
    c.early_termination = in.early_termination != 0;
    c.sample_queries = in.sample_queries != 0;
    c.objective_k = in.objective_k;
    c.ann_explore_fraction = in.ann_explore_fraction;
    c.min_not_pruned_pct = in.min_not_pruned_pct;
    c.max_not_pruned_pct = in.max_not_pruned_pct;
    c.adjustment_factor_for_partial_d = in.adjustment_factor_for_partial_d;
    c.unrotate_centroids = in.unrotate_centroids != 0;
    c.verbose = in.verbose != 0;
    c.angular = in.angular != 0;
    c.suppress_warnings = in.suppress_warnings != 0;
    c.data_already_rotated = in.data_already_rotated != 0;
    c.dct_rotation = in.dct_rotation;
}

} // namespace

struct skm_kmeans {
    std::unique_ptr<FlatModel> flat;
    std::unique_ptr<HierModel> hier;
    size_t k = 0, d = 0;
    size_t n_trained = 0;
    skmeans::SuperKMeans<>* base() { return hier ? static_cast<skmeans::SuperKMeans<>*>(hier.get()) : flat.get(); }
};

// Points the model's centroid download at the caller's buffer for the duration of one Train call.
struct SinkScope {
    skmeans::SuperKMeans<>* model;
    SinkScope(skmeans::SuperKMeans<>* m, float* sink) : model(m) { model->output_sink = sink; }
    ~SinkScope() { model->output_sink = nullptr; }
};

#define SKM_API_GUARD(body)                                                                        \
    try {                                                                                          \
        body;                                                                                      \
        return SKM_OK;                                                                             \
    } catch (const std::invalid_argument& e) {                                                     \
        return skm::set_error(SKM_ERR_INVALID, "%s", e.what());                                    \
    } catch (const std::bad_alloc& e) {                                                            \
        return skm::set_error(SKM_ERR_OOM, "host allocation failed: %s", e.what());                \
    } catch (const std::exception& e) {                                                            \
        return skm::set_error(SKM_ERR_RUNTIME, "%s", e.what());                                    \
    }

extern "C" {

void skm_kmeans_default_config(skm_kmeans_config* out, int hierarchical) {
    if (!out) return;
    skmeans::HierarchicalSuperKMeansConfig h;
    skmeans::SuperKMeansConfig f;
    const skmeans::SuperKMeansConfig& c = hierarchical ? static_cast<const skmeans::SuperKMeansConfig&>(h) : f;
    out->iters = c.iters;
    out->sampling_fraction = c.sampling_fraction;
    out->max_points_per_cluster = c.max_points_per_cluster;
    out->n_threads = c.n_threads;
    out->seed = c.seed;
    out->use_blas_only = c.use_blas_only;
    out->tol = c.tol;
    out->recall_tol = c.recall_tol;
    out->early_termination = c.early_termination;
    out->sample_queries = c.sample_queries;
    out->objective_k = c.objective_k;
    out->ann_explore_fraction = c.ann_explore_fraction;
    out->min_not_pruned_pct = c.min_not_pruned_pct;
    out->max_not_pruned_pct = c.max_not_pruned_pct;
    out->adjustment_factor_for_partial_d = c.adjustment_factor_for_partial_d;
    out->unrotate_centroids = c.unrotate_centroids;
    out->verbose = c.verbose;
    out->angular = c.angular;
    out->suppress_warnings = c.suppress_warnings;
    out->data_already_rotated = c.data_already_rotated;
    out->iters_mesoclustering = h.iters_mesoclustering;
    out->iters_fineclustering = h.iters_fineclustering;
    out->iters_refinement = h.iters_refinement;
    out->dct_rotation = c.dct_rotation;
}

int skm_kmeans_create(size_t n_clusters, size_t dimensionality, const skm_kmeans_config* config, int hierarchical,
                      skm_kmeans** out) {
    if (!out || !config) return skm::set_error(SKM_ERR_INVALID, "skm_kmeans_create: null argument");
    *out = nullptr;
    SKM_API_GUARD({
        auto km = std::make_unique<skm_kmeans>();
        km->k = n_clusters;
        km->d = dimensionality;
        if (hierarchical) {
            skmeans::HierarchicalSuperKMeansConfig c;
            fill_base(c, *config);
            c.iters_mesoclustering = config->iters_mesoclustering;
            c.iters_fineclustering = config->iters_fineclustering;
            c.iters_refinement = config->iters_refinement;
            km->hier = std::make_unique<HierModel>(n_clusters, dimensionality, c);
        } else {
            skmeans::SuperKMeansConfig c;
            fill_base(c, *config);
            km->flat = std::make_unique<FlatModel>(n_clusters, dimensionality, c);
        }
        *out = km.release();
    });
}

int skm_kmeans_destroy(skm_kmeans* km) {
    delete km;
    return SKM_OK;
}

int skm_kmeans_train(skm_kmeans* km, const float* h_data, size_t n, const float* h_queries, size_t n_queries,
                     float* h_out_centroids) {
    if (!km || !h_data || !h_out_centroids) return skm::set_error(SKM_ERR_INVALID, "skm_kmeans_train: null argument");
    SKM_API_GUARD({
        SinkScope sink(km->base(), h_out_centroids);  // centroids are downloaded straight into the caller's buffer
        if (km->hier) km->hier->Train(h_data, n, h_queries, n_queries); else km->flat->Train(h_data, n, h_queries, n_queries);
        km->n_trained = n;
    });
}

int skm_kmeans_train_device(skm_kmeans* km, const float* d_data, size_t n, const float* d_queries, size_t n_queries,
                            float* h_out_centroids) {
    if (!km || !d_data || !h_out_centroids)
        return skm::set_error(SKM_ERR_INVALID, "skm_kmeans_train_device: null argument");
    SKM_API_GUARD({
        SinkScope sink(km->base(), h_out_centroids);
        if (km->hier) km->hier->TrainDevice(d_data, n, d_queries, n_queries);
        else km->flat->TrainDevice(d_data, n, d_queries, n_queries);
        km->n_trained = n;
    });
}

int skm_kmeans_assign(skm_kmeans* km, const float* h_vectors, const float* h_centroids, size_t n_vectors,
                      size_t n_centroids, uint32_t* h_out_assignments) {
    if (!km || !h_vectors || !h_centroids || !h_out_assignments)
        return skm::set_error(SKM_ERR_INVALID, "skm_kmeans_assign: null argument");
    SKM_API_GUARD({
        auto a = km->base()->Assign(h_vectors, h_centroids, n_vectors, n_centroids);
        std::memcpy(h_out_assignments, a.data(), a.size() * sizeof(uint32_t));
    });
}

int skm_kmeans_assign_device(skm_kmeans* km, const float* d_vectors, const float* d_centroids, size_t n_vectors,
                             size_t n_centroids, uint32_t* d_out_assignments) {
    if (!km || !d_vectors || !d_centroids || !d_out_assignments)
        return skm::set_error(SKM_ERR_INVALID, "skm_kmeans_assign_device: null argument");
    SKM_API_GUARD({
        km->base()->AssignDevice(d_vectors, d_centroids, n_vectors, n_centroids, d_out_assignments);
        skmeans::hip::Check(skm_sync(km->base()->GetContext()));
    });
}

int skm_kmeans_assign_training_points(skm_kmeans* km, const float* h_vectors, const float* h_centroids,
                                      size_t n_vectors, size_t n_centroids, uint32_t* h_out_assignments) {
    if (!km || !h_vectors || !h_centroids || !h_out_assignments)
        return skm::set_error(SKM_ERR_INVALID, "skm_kmeans_assign_training_points: null argument");
    SKM_API_GUARD({
        auto a = km->base()->AssignTrainingPoints(h_vectors, h_centroids, n_vectors, n_centroids);
        std::memcpy(h_out_assignments, a.data(), a.size() * sizeof(uint32_t));
    });
}

int skm_kmeans_split_clusters_on_state(skm_kmeans* km, float* h_centroids, uint32_t* h_sizes, size_t k, size_t n_samples,
                                       uint64_t* out_n_split) {
    if (!km || !h_centroids || !h_sizes || !out_n_split)
        return skm::set_error(SKM_ERR_INVALID, "skm_kmeans_split_clusters_on_state: null argument");
    if (n_samples <= k) return skm::set_error(SKM_ERR_INVALID, "skm_kmeans_split_clusters_on_state: n_samples must exceed k");
    SKM_API_GUARD({ *out_n_split = km->base()->SplitClustersOnState(h_centroids, h_sizes, k, n_samples); });
}

int skm_kmeans_get_n_clusters(skm_kmeans* km, size_t* out) {
    if (!km || !out) return skm::set_error(SKM_ERR_INVALID, "null argument");
    *out = km->base()->GetNClusters();
    return SKM_OK;
}

int skm_kmeans_is_trained(skm_kmeans* km, int* out) {
    if (!km || !out) return skm::set_error(SKM_ERR_INVALID, "null argument");
    *out = km->base()->IsTrained() ? 1 : 0;
    return SKM_OK;
}

static const std::vector<skmeans::SuperKMeansIterationStats>* stats_of(skm_kmeans* km, int which) {
    if (which == 0) return &km->base()->iteration_stats;
    if (!km->hier) return nullptr;
    auto& h = km->hier->hierarchical_iteration_stats;
    if (which == 1) return &h.mesoclustering_iteration_stats;
    if (which == 2) return &h.fineclustering_iteration_stats;
    if (which == 3) return &h.refinement_iteration_stats;
    return nullptr;
}

int skm_kmeans_n_stats(skm_kmeans* km, int which, size_t* out) {
    if (!km || !out) return skm::set_error(SKM_ERR_INVALID, "null argument");
    auto* v = stats_of(km, which);
    *out = v ? v->size() : 0;
    return SKM_OK;
}

int skm_kmeans_get_stats(skm_kmeans* km, int which, skm_kmeans_iteration_stats* out, size_t capacity) {
    if (!km || !out) return skm::set_error(SKM_ERR_INVALID, "null argument");
    auto* v = stats_of(km, which);
    if (!v) return SKM_OK;
    for (size_t i = 0; i < v->size() && i < capacity; ++i) {
        const auto& s = (*v)[i];
        out[i].iteration = s.iteration;
        out[i].objective = s.objective;
        out[i].shift = s.shift;
        out[i].split = s.split;
        out[i].recall = s.recall;
        out[i].not_pruned_pct = s.not_pruned_pct;
        out[i].partial_d = s.partial_d;
        out[i].is_gemm_only = s.is_gemm_only ? 1 : 0;
    }
    return SKM_OK;
}

int skm_kmeans_get_assignments(skm_kmeans* km, uint32_t* h_out, size_t count) {
    if (!km || !h_out) return skm::set_error(SKM_ERR_INVALID, "null argument");
    if (!km->base()->IsTrained()) return skm::set_error(SKM_ERR_RUNTIME, "the model has not been trained");
    if (count > km->n_trained) return skm::set_error(SKM_ERR_INVALID, "count exceeds the number of training points");
    std::memcpy(h_out, km->base()->assignments.get(), count * sizeof(uint32_t));
    return SKM_OK;
}

int skm_kmeans_get_training_seeds(skm_kmeans* km, uint32_t* h_out, size_t count) {
    if (!km || !h_out) return skm::set_error(SKM_ERR_INVALID, "null argument");
    const std::vector<uint32_t>& seeds = km->base()->GetTrainingSeeds();
    if (seeds.empty()) return skm::set_error(SKM_ERR_RUNTIME, "no pruned AssignTrainingPoints has run on this object");
    if (count != seeds.size()) return skm::set_error(SKM_ERR_INVALID, "count differs from the number of vectors of that call");
    std::memcpy(h_out, seeds.data(), count * sizeof(uint32_t));
    return SKM_OK;
}

int skm_kmeans_get_training_overflow(skm_kmeans* km, uint64_t* out_points) {
    if (!km || !out_points) return skm::set_error(SKM_ERR_INVALID, "null argument");
    *out_points = km->base()->GetTrainingOverflow();
    return SKM_OK;
}

int skm_kmeans_context(skm_kmeans* km, skm_ctx** out) {
    if (!km || !out) return skm::set_error(SKM_ERR_INVALID, "null argument");
    *out = km->base()->GetContext();
    return SKM_OK;
}

int skm_kmeans_set_prune_accounting(skm_kmeans* km, int enabled) {
    if (!km) return skm::set_error(SKM_ERR_INVALID, "null argument");
    km->base()->SetCollectPruneAccounting(enabled != 0);
    return SKM_OK;
}

int skm_kmeans_get_prune_accounting(skm_kmeans* km, size_t iteration, uint64_t* h_out, size_t capacity,
                                    size_t* out_len, size_t* out_rows) {
    if (!km) return skm::set_error(SKM_ERR_INVALID, "null argument");
    const auto& table = km->base()->GetPruneAccounting();
    if (out_rows) *out_rows = table.size();
    if (out_len) *out_len = 0;
    if (iteration >= table.size()) return SKM_OK;
    const auto& row = table[iteration];
    if (out_len) *out_len = row.size();
    if (h_out)
        for (size_t i = 0; i < row.size() && i < capacity; ++i) h_out[i] = row[i];
    return SKM_OK;
}

void skm_dimension_split(size_t d, size_t* out_horizontal_d, size_t* out_vertical_d) {
    const auto s = skmeans::PDXLayout<>::GetDimensionSplit(d);
    if (out_horizontal_d) *out_horizontal_d = s.horizontal_d;
    if (out_vertical_d) *out_vertical_d = s.vertical_d;
}

int skm_pruner_tables(size_t d, float epsilon0, uint32_t seed, int rotation_kind, float* h_out_matrix,
                      float* h_out_ratios) {
    if (d == 0) return skm::set_error(SKM_ERR_INVALID, "skm_pruner_tables: d must be positive");
    SKM_API_GUARD({
        skmeans::hip::Context c(0);
        skmeans::ADSamplingPruner<> p(c.get(), (uint32_t) d, epsilon0, seed, rotation_kind);
        if (h_out_matrix) std::memcpy(h_out_matrix, p.HostMatrix().data(), d * d * sizeof(float));
        if (h_out_ratios) std::memcpy(h_out_ratios, p.ratios.data(), (d + 1) * sizeof(float));
    });
}

} // extern "C"
