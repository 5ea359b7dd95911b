// skmeans::SuperKMeans, HIP backend for MI355X.
//
// Same public interface as the reference's include/superkmeans/superkmeans.h (config and stats
// structs :23-98, constructor :123-149, Train :162, Assign :346, AssignTrainingPoints :397,
// accessors :567-628, public members :1491-1492).  What differs is where the work happens: every
// per-point step (rotation, norms, distance GEMM, pruned search, centroid update, relayout, cost,
// shift) is a call into libskm_hip.so on device-resident buffers; this header only keeps the
// iteration control flow, the RNG-dependent host decisions (initial centroids, sampling, cluster
// splitting, d' tuning, early stopping) and the transfers at the API boundary.
//
// Additions over the reference interface (they do not change existing calls):
//   TrainDevice / AssignDevice   same as Train / Assign for inputs that already live in HBM.
//   GetContext                   the skm_ctx used by this object (device timers, workspace limit).
#pragma once

#include <algorithm>
#include <cmath>
#include <cstring>
#include <functional>
#include <iostream>
#include <memory>
#include <numeric>
#include <random>
#include <sstream>
#include <thread>
#include <vector>

#include "superkmeans/common.h"
#include "superkmeans/pdx/adsampling.h"
#include "superkmeans/pdx/layout.h"

namespace skmeans {

struct SuperKMeansConfig {
    // Training parameters
    uint32_t iters = 10;
    float sampling_fraction = 0.3f;
    uint32_t max_points_per_cluster = 256;
    uint32_t n_threads = 0;  // accepted for compatibility; device work does not use host threads
    uint32_t seed = 42;
    bool use_blas_only = false;  // GEMM-only iterations (no pruning)

    // Convergence parameters
    float tol = 1e-4f;
    float recall_tol = 0.005f;
    bool early_termination = true;
    bool sample_queries = false;
    size_t objective_k = 100;
    float ann_explore_fraction = 0.01f;

    // Sweet range for d' tuning
    float min_not_pruned_pct = 0.03f;
    float max_not_pruned_pct = 0.05f;
    float adjustment_factor_for_partial_d = 0.20f;

    // Output parameters
    bool unrotate_centroids = true;
    bool verbose = false;
    bool angular = false;
    bool suppress_warnings = false;

    bool data_already_rotated = false;

    // Not in the reference's struct, where it is a build option (FFTW present or not): which rotation the
    // pruner uses.  0 = dense Gaussian (builds without FFTW), 1 = sign flip + DCT-II when d >= 512 and d
    // is a power of two (FFTW builds on AVX2 machines), 2 = DCT whenever d >= 512 (other FFTW builds).
    int dct_rotation = 0;
};

struct SuperKMeansIterationStats {
    size_t iteration = 0;
    float objective = 0.0f;
    float shift = 0.0f;
    size_t split = 0;
    float recall = 0.0f;
    float not_pruned_pct = -1.0f;
    uint32_t partial_d = 0;
    bool is_gemm_only = false;
};

struct ClusterBalanceStats {
    float mean = 0.0f;
    float geometric_mean = 0.0f;
    float stdev = 0.0f;
    float cv = 0.0f;
    size_t min = 0;
    size_t max = 0;

    std::string to_json() const {
        std::ostringstream oss;
        oss << "{\"mean\":" << mean << ",\"geometric_mean\":" << geometric_mean << ",\"stdev\":" << stdev
            << ",\"cv\":" << cv << ",\"min\":" << min << ",\"max\":" << max << "}";
        return oss.str();
    }

    void print() const {
        std::cout << "Cluster size stats: mean=" << mean << ", gmean=" << geometric_mean << ", std=" << stdev
                  << ", CV=" << cv << ", min=" << min << ", max=" << max << std::endl;
    }
};

template <Quantization q = Quantization::f32, DistanceFunction alpha = DistanceFunction::l2>
class SuperKMeans {
    static_assert(q == Quantization::f32 && alpha == DistanceFunction::l2,
                  "only <f32, l2> is instantiated, as in the reference");

  public:
    virtual ~SuperKMeans() { FinishHostOutputs(); }

  protected:
    using centroid_value_t = skmeans_centroid_value_t<q>;
    using vector_value_t = skmeans_value_t<q>;
    using distance_t = skmeans_distance_t<q>;
    using pruner_t = ADSamplingPruner<q>;
    using layout_t = PDXLayout<q, alpha>;
    template <class T>
    using dbuf = hip::Buffer<T>;

  public:
    SuperKMeans(size_t n_clusters, size_t dimensionality, const SuperKMeansConfig& config)
        : d(dimensionality), n_clusters(n_clusters), config(config) {
        SKMEANS_ENSURE_POSITIVE(n_clusters);
        SKMEANS_ENSURE_POSITIVE(dimensionality);
        SKMEANS_ENSURE_POSITIVE(config.iters);
        SKMEANS_ENSURE_POSITIVE(config.sampling_fraction);
        if (config.sampling_fraction > 1.0) {
            throw std::invalid_argument("sampling_fraction must be <= 1.0");
        }
        n_threads = (config.n_threads == 0) ? 1 : config.n_threads;
        g_n_threads = n_threads;
        context = std::make_shared<hip::Context>(0);
        ctx = context->get();
        pruner = std::make_shared<pruner_t>(ctx, dimensionality, PRUNER_INITIAL_THRESHOLD, config.seed,
                                            config.dct_rotation);
        if (this->config.data_already_rotated) {
            this->config.unrotate_centroids = false;
        }
    }

  protected:
    // A helper object for concurrent sub-problems of another object: its own device context (stream,
    // scratch), the owner's pruner tables (building the rotation matrix again would cost O(d^3) on the host).
    SuperKMeans(size_t n_clusters, size_t dimensionality, const SuperKMeansConfig& config,
                std::shared_ptr<pruner_t> shared_pruner)
        : d(dimensionality), n_clusters(n_clusters), config(config) {
        n_threads = 1;
        context = std::make_shared<hip::Context>(0);
        ctx = context->get();
        pruner = std::move(shared_pruner);
        // same rule as the public constructor (reference superkmeans.h:137-139): centroids of data that was
        // never rotated here must not be "un-rotated"
        if (this->config.data_already_rotated) {
            this->config.unrotate_centroids = false;
        }
    }

  public:

    SuperKMeans(size_t n_clusters, size_t dimensionality)
        : SuperKMeans(n_clusters, dimensionality, SuperKMeansConfig{}) {}

    /** Runs k-means on host-resident row-major data (n x d) and returns the k x d centroids. */
    std::vector<centroid_value_t> Train(const vector_value_t* data, const size_t n,
                                        const vector_value_t* queries = nullptr, const size_t n_queries = 0) {
        return TrainImpl(data, n, queries, n_queries, /*on_device=*/false);
    }

    /** Train for data that already lives in device memory of this object's context. */
    std::vector<centroid_value_t> TrainDevice(const vector_value_t* d_data, const size_t n,
                                              const vector_value_t* d_queries = nullptr,
                                              const size_t n_queries = 0) {
        return TrainImpl(d_data, n, d_queries, n_queries, /*on_device=*/true);
    }

    /**
     * Exact nearest-centroid assignment; vectors and centroids must be in the same space.  The vectors go to the
     * device in slabs of rows and every slab is searched while the next one is on its way.
     */
    [[nodiscard]] std::vector<uint32_t> Assign(const vector_value_t* vectors, const vector_value_t* centroids,
                                               const size_t n_vectors, const size_t n_centroids) {
        dbuf<float> d_v(ctx, n_vectors * d), d_c(ctx, n_centroids * d);
        d_c.Upload(centroids, n_centroids * d);
        dbuf<uint32_t> d_out(ctx, n_vectors);
        dbuf<float> v_norms(ctx, n_vectors), c_norms(ctx, n_centroids), dist(ctx, n_vectors);
        hip::Check(skm_norms(ctx, d_c.get(), n_centroids, d, d, c_norms.get()));
        const size_t slab = UploadSlabRows();
        for (size_t r0 = 0; r0 < n_vectors; r0 += slab) {
            const size_t m = std::min(slab, n_vectors - r0);
            d_v.UploadOverlapped(vectors + r0 * d, m * d, r0 * d);
            hip::Check(skm_norms(ctx, d_v.get() + r0 * d, m, d, d, v_norms.get() + r0));
            hip::Check(skm_assign_full(ctx, d_v.get() + r0 * d, m, d_c.get(), n_centroids, d, v_norms.get() + r0,
                                       c_norms.get(), d_out.get() + r0, dist.get() + r0));
        }
        std::vector<uint32_t> result(n_vectors);
        d_out.Download(result.data(), n_vectors);
        return result;
    }

    // Row offsets, from 0 to n_rows, of the slabs that AssignTrainingPoints searches one by one: UploadSlabRows() rows,
    // but at least 65,536 (the kernels of the pruned search that are made for many points need 49,152 of them).
    // Measured on 1 M rows of 1024 dimensions (reference defaults): slabs of 64 MiB (16,384 rows) 420 ms, 256 MiB 229 ms,
    // 512 MiB 225 ms but 320 ms for the first call (the scratch memory of a slab's search grows with it); a smaller
    // first slab changed nothing.
    std::vector<size_t> UploadSlabEdges(const size_t n_rows) const {
        std::vector<size_t> edges{0};
        const size_t rows = std::max<size_t>(UploadSlabRows(), 65536);
        while (edges.back() < n_rows) edges.push_back(std::min(n_rows, edges.back() + rows));
        return edges;
    }
    // Rows per slab of a host-to-device transfer that overlaps with compute: 256 MiB of rows, a multiple of 256.
    size_t UploadSlabRows() const {
        const size_t rows = (size_t(256) << 20) / (d * sizeof(float));
        return std::max<size_t>(256, rows / 256 * 256);
    }

    /** Assign on device-resident inputs; writes n_vectors indices to d_out_assignments.  Queued on the object's
     *  context, not waited for: read the output after skm_sync (or through a download on the same context). */
    void AssignDevice(const vector_value_t* d_vectors, const vector_value_t* d_centroids, const size_t n_vectors,
                      const size_t n_centroids, uint32_t* d_out_assignments) {
        // norms and distances live in buffers that the object keeps between calls (allocating and releasing
        // them costs a third of a millisecond per call, and a release waits for the device)
        if (assign_v_norms.size() < n_vectors) assign_v_norms.Reset(ctx, n_vectors);
        if (assign_dist.size() < n_vectors) assign_dist.Reset(ctx, n_vectors);
        if (assign_c_norms.size() < n_centroids) assign_c_norms.Reset(ctx, n_centroids);
        hip::Check(skm_norms(ctx, d_vectors, n_vectors, d, d, assign_v_norms.get()));
        hip::Check(skm_norms(ctx, d_centroids, n_centroids, d, d, assign_c_norms.get()));
        hip::Check(skm_assign_full(ctx, d_vectors, n_vectors, d_centroids, n_centroids, d, assign_v_norms.get(),
                                   assign_c_norms.get(), d_out_assignments, assign_dist.get()));
    }

    /** Pruned assignment of the training points, seeded with the assignments found by Train. */
    [[nodiscard]] std::vector<uint32_t> AssignTrainingPoints(const vector_value_t* vectors,
                                                             const vector_value_t* centroids,
                                                             const size_t n_vectors, const size_t n_centroids) {
        if (!trained) {
            throw std::runtime_error("AssignTrainingPoints requires SuperKMeans to be trained first");
        }
        training_seeds.clear();
        if (config.use_blas_only || d < DIMENSION_THRESHOLD_FOR_PRUNING ||
            n_clusters <= N_CLUSTERS_THRESHOLD_FOR_PRUNING) {
            if (!config.suppress_warnings) {
                std::cout << "WARNING: AssignTrainingPoints cannot use pruning, falling back to "
                             "brute force Assign"
                          << std::endl;
            }
            return Assign(vectors, centroids, n_vectors, n_centroids);
        }
        partial_d = std::max<uint32_t>(MIN_PARTIAL_D, vertical_d / 2);

        // The caller's vectors go to the device in slabs, from a thread of their own; below, every slab is rotated
        // and searched while the later ones are still on their way (already rotated vectors are used as they arrive).
        dbuf<float> d_rot(ctx, n_vectors * d), d_raw;
        if (!config.data_already_rotated) d_raw.Reset(ctx, n_vectors * d);
        dbuf<float>& landing = config.data_already_rotated ? d_rot : d_raw;
        hip::RowFeeder feed(ctx, landing.get(), vectors, d, UploadSlabEdges(n_vectors));
        // Final centroids: horizontal_centroids / centroids (PDX) / partial_horizontal_centroids were
        // all refreshed by the last ConsolidateCentroids.
        hip::Check(skm_norms(ctx, horizontal_centroids.get(), n_centroids, d, partial_d, centroid_norms.get()));
        EnsurePdxLayout(horizontal_centroids.get(), n_centroids);

        // Seeds that do not depend on the vectors are made here; an entry of NO_SEED is resolved on the device, slab
        // by slab, from the nearest meso-centroid of the vector.
        constexpr uint32_t NO_SEED = 0xffffffffu;
        std::vector<uint32_t> seeds(n_vectors);
        dbuf<float> d_meso;
        dbuf<uint32_t> d_meso_to_original, d_meso_assignments;
        size_t n_meso = 0;
        if (config.sampling_fraction == 1.0f) {
            std::memcpy(seeds.data(), assignments.get(), n_vectors * sizeof(uint32_t));
        } else if (config.sampling_fraction > 0.8f) {
            // Sampled points keep their training assignment, the rest draw a cluster with
            // probability proportional to its size.
            size_t cur = 0;
            for (; cur < n_samples; ++cur) seeds[sampled_indices[cur]] = assignments[cur];
            std::mt19937 rng(config.seed + 1);
            std::discrete_distribution<uint32_t> cluster_dist(cluster_sizes.get(), cluster_sizes.get() + n_clusters);
            for (; cur < n_vectors; ++cur) seeds[sampled_indices[cur]] = cluster_dist(rng);
        } else {
            // Few samples: cluster the centroids into sqrt(k) meso-centroids and seed every
            // unsampled point with a representative of its nearest meso-centroid.
            SuperKMeansConfig tmp_config;
            tmp_config.iters = 10;
            tmp_config.sampling_fraction = 1.0f;
            tmp_config.use_blas_only = false;
            tmp_config.verbose = config.verbose;
            tmp_config.suppress_warnings = config.suppress_warnings;
            tmp_config.seed = config.seed;
            tmp_config.angular = config.angular;
            tmp_config.data_already_rotated = config.data_already_rotated;
            tmp_config.dct_rotation = config.dct_rotation;
            n_meso = static_cast<size_t>(std::sqrt(n_centroids));
            // Same dimensionality and seed as this object: the rotation matrix and ratios would come out the same,
            // so the tables are shared instead of being factorised again on the host (the hierarchical variant
            // holds tables with another epsilon and builds fresh ones, as the reference does).
            std::unique_ptr<SuperKMeans> tmp_owner(
                pruner->Epsilon0() == PRUNER_INITIAL_THRESHOLD
                    ? new SuperKMeans(n_meso, d, tmp_config, pruner)
                    : new SuperKMeans(n_meso, d, tmp_config));
            SuperKMeans& tmp_kmeans = *tmp_owner;
            auto meso_centroids = tmp_kmeans.Train(centroids, n_centroids);
            auto centroids_to_meso = tmp_kmeans.Assign(centroids, meso_centroids.data(), n_centroids, n_meso);
            g_n_threads = n_threads;
            std::vector<uint32_t> meso_to_original(n_meso, 0);
            for (size_t c = 0; c < n_centroids; ++c) meso_to_original[centroids_to_meso[c]] = static_cast<uint32_t>(c);
            d_meso.Reset(ctx, n_meso * d);
            d_meso.Upload(meso_centroids.data(), n_meso * d);
            d_meso_to_original.Reset(ctx, n_meso);
            d_meso_to_original.Upload(meso_to_original.data(), n_meso);
            d_meso_assignments.Reset(ctx, n_vectors);
            std::fill(seeds.begin(), seeds.end(), NO_SEED);
            for (size_t cur = 0; cur < n_samples; ++cur) seeds[sampled_indices[cur]] = assignments[cur];
        }
        dbuf<uint32_t> d_seed(ctx, n_vectors), d_first_seed;
        d_seed.Upload(seeds.data(), n_vectors);
        if (n_meso > 0) d_first_seed.Reset(ctx, n_vectors);
        dbuf<float> d_norms_p(ctx, n_vectors), d_dist(ctx, n_vectors);
        training_overflow_points = 0;
        for (size_t s = 0; s < feed.NumSlabs(); ++s) {
            const size_t r0 = feed.FirstRow(s), m = feed.Rows(s);
            feed.WaitFor(s);
            if (!config.data_already_rotated) pruner->Rotate(ctx, d_raw.get() + r0 * d, d_rot.get() + r0 * d, m);
            if (n_meso > 0) {
                // nearest meso-centroid in the space the caller's centroids are in, then the seeds still open
                AssignDevice(landing.get() + r0 * d, d_meso.get(), m, n_meso, d_meso_assignments.get() + r0);
                hip::Check(skm_seeds_from_groups(ctx, d_seed.get() + r0, d_meso_assignments.get() + r0,
                                                 d_meso_to_original.get(), n_meso, m));
                hip::Check(skm_copy(ctx, d_first_seed.get() + r0, d_seed.get() + r0, m * sizeof(uint32_t)));
            }
            hip::Check(skm_norms(ctx, d_rot.get() + r0 * d, m, d, partial_d, d_norms_p.get() + r0));
            hip::Check(skm_assign_pruned(ctx, d_rot.get() + r0 * d, m, horizontal_centroids.get(), this->centroids.get(),
                                         partial_horizontal_centroids.get(), n_clusters, d, vertical_d, partial_d,
                                         pruner->DeviceRatios(), d_norms_p.get() + r0, centroid_norms.get(),
                                         d_seed.get() + r0, d_dist.get() + r0, nullptr, nullptr));
            uint64_t overflowed = 0;
            hip::Check(skm_ctx_get_last_overflow(ctx, &overflowed));
            training_overflow_points += overflowed;
        }
        if (n_meso > 0) d_first_seed.Download(seeds.data(), n_vectors);
        training_seeds = std::move(seeds);
        std::vector<uint32_t> result(n_vectors);
        d_seed.Download(result.data(), n_vectors);
        if (config.sampling_fraction == 1.0f) {
            // The reference updates the object's assignments/distances in this branch (:454-469).
            std::memcpy(assignments.get(), result.data(), n_vectors * sizeof(uint32_t));
            host_distances.resize(n_vectors);
            d_dist.Download(host_distances.data(), n_vectors);
        }
        return result;
    }

    [[nodiscard]] size_t GetNClusters() const noexcept { return n_clusters; }
    [[nodiscard]] bool IsTrained() const noexcept { return trained; }
    /**
     * Test hook, no counterpart in the reference: SplitClusters of this object's class (the flat rule here,
     * superkmeans.h:890-928; the balancing rule in HierarchicalSuperKMeans, hierarchical_superkmeans.h:579-678) applied
     * to a given state, so that its decisions and row arithmetic can be compared with another implementation's on
     * hand-made states.  h_centroids (k x d) and h_sizes (k) are replaced by the edited rows and sizes; returns the
     * number of splits.  Untrained objects only (it overwrites the object's centroid buffers).
     */
    size_t SplitClustersOnState(centroid_value_t* h_centroids, uint32_t* h_sizes, const size_t k, const size_t n_samples_) {
        if (trained) throw std::runtime_error("SplitClustersOnState needs an untrained object");
        SKMEANS_ENSURE_POSITIVE(k);
        horizontal_centroids.Reset(ctx, k * d);
        horizontal_centroids.Upload(h_centroids, k * d);
        cluster_sizes.reset(new uint32_t[k]);
        std::memcpy(cluster_sizes.get(), h_sizes, k * sizeof(uint32_t));
        SplitClusters(n_samples_, k);
        horizontal_centroids.Download(h_centroids, k * d);
        std::memcpy(h_sizes, cluster_sizes.get(), k * sizeof(uint32_t));
        return n_split;
    }

    /** The centroid every vector of the last AssignTrainingPoints started its pruned search from (the reference
     *  builds them in place in its result array, superkmeans.h:454-563); empty before the first call and after a
     *  call that fell back to Assign. */
    [[nodiscard]] const std::vector<uint32_t>& GetTrainingSeeds() const noexcept { return training_seeds; }
    /** How many vectors of the last pruned AssignTrainingPoints left more candidates than their list holds and took
     *  the second pass of the search (no counterpart in the reference, whose search keeps no lists). */
    [[nodiscard]] uint64_t GetTrainingOverflow() const noexcept { return training_overflow_points; }
    [[nodiscard]] float GetSamplingFraction() const noexcept { return config.sampling_fraction; }
    /** Host copy of the per-point squared distances of the last training iteration. */
    [[nodiscard]] distance_t* GetDistancesPointer() { return host_distances.data(); }
    [[nodiscard]] skm_ctx* GetContext() const noexcept { return ctx; }
    /**
     * When enabled, every pruned iteration also records how many (point, centroid) pairs entered
     * each pruning step (first test, each 64-dimension block, the [d', vertical_d) step); one row per
     * pruned iteration is appended to the returned table.  Used to state the algorithmic bytes of the
     * pruning stage; off by default because it adds atomics to the kernel.
     */
    void SetCollectPruneAccounting(bool on) noexcept { collect_prune_accounting = on; }
    [[nodiscard]] const std::vector<std::vector<uint64_t>>& GetPruneAccounting() const noexcept {
        return prune_accounting;
    }

    [[nodiscard]] static ClusterBalanceStats GetClustersBalanceStats(const uint32_t* assignments_in, size_t n_samples_in,
                                                                     size_t n_clusters_in) {
        ClusterBalanceStats stats;
        std::vector<size_t> sizes(n_clusters_in, 0);
        for (size_t i = 0; i < n_samples_in; ++i) sizes[assignments_in[i]]++;
        const auto sum = std::accumulate(sizes.begin(), sizes.end(), size_t{0});
        stats.mean = static_cast<float>(sum) / static_cast<float>(sizes.size());
        float log_sum = 0.0f;
        size_t non_zero = 0;
        size_t sq_sum = 0;
        for (size_t s : sizes) {
            if (s > 0) {
                log_sum += std::log(static_cast<float>(s));
                non_zero++;
            }
            sq_sum += s * s;
        }
        stats.geometric_mean = non_zero > 0 ? std::exp(log_sum / static_cast<float>(non_zero)) : 0.0f;
        stats.stdev = std::sqrt(static_cast<float>(sq_sum) / static_cast<float>(sizes.size()) - stats.mean * stats.mean);
        stats.cv = stats.stdev / stats.mean;
        const auto mm = std::minmax_element(sizes.begin(), sizes.end());
        stats.min = *mm.first;
        stats.max = *mm.second;
        return stats;
    }

  protected:
    // ------------------------------------------------------------------------------------------
    // Train, flat variant (reference superkmeans.h:162-332)
    // ------------------------------------------------------------------------------------------
    std::vector<centroid_value_t> TrainImpl(const vector_value_t* data, const size_t n, const vector_value_t* queries,
                                            const size_t n_queries, const bool on_device) {
        SKMEANS_ENSURE_POSITIVE(n);
        if (trained) {
            throw std::runtime_error("The clustering has already been trained");
        }
        iteration_stats.clear();
        if (n < n_clusters) {
            throw std::runtime_error("The number of points should be at least as large as the number of clusters");
        }
        if (n_queries > 0 && queries == nullptr && !config.sample_queries) {
            throw std::invalid_argument("Queries must be provided if n_queries > 0 and sample_queries is false");
        }
        n_samples = GetNVectorsToSample(n, n_clusters);
        if (n_samples < n_clusters) {
            throw std::runtime_error(
                "Not enough samples to train. Try increasing the sampling_fraction or max_points_per_cluster");
        }
        AllocateState(n, n_clusters);
        PrepareHostOutputs(n_samples);
        partial_d = std::max<uint32_t>(MIN_PARTIAL_D, vertical_d / 2);
        if (partial_d > vertical_d) partial_d = vertical_d;
        if (config.verbose) {
            std::cout << "Front dimensions (d') = " << partial_d << std::endl;
            std::cout << "Trailing dimensions (d'') = " << d - vertical_d << std::endl;
        }

        const bool rotate = !config.data_already_rotated;
        const float* data_to_cluster = nullptr;
        first_search_done = false;
        if (!on_device && config.iters > 0) {
            // Host rows (all of them, or the sampled ones): they reach the device in slabs, and every slab is rotated and searched
            // against the initial centroids (the first iteration is always exact) while the next one is on its
            // way.  The initial centroids come first for that; they are rows of the host matrix.
            GenerateCentroids(data, n_samples, n_clusters, rotate, on_device);
            RotateOrCopy(horizontal_centroids.get(), prev_centroids.get(), n_clusters, rotate);
            hip::Check(skm_norms(ctx, prev_centroids.get(), n_clusters, d, d, centroid_norms.get()));
            data_to_cluster = SampleAndRotateVectors(
                data, n, n_samples, rotate, on_device, [&](const float* d_rows, const size_t r0, const size_t m) {
                    hip::Check(skm_norms(ctx, d_rows, m, d, d, data_norms.get() + r0));
                    hip::Check(skm_assign_full(ctx, d_rows, m, prev_centroids.get(), n_clusters, d,
                                               data_norms.get() + r0, centroid_norms.get(),
                                               d_assignments.get() + r0, distances.get() + r0));
                });
            first_search_done = true;
        } else {
            // The rotation of the training matrix is queued first so that it runs on the device while the host
            // draws the initial centroids; the two steps share no state (each seeds its own mt19937).
            data_to_cluster = SampleAndRotateVectors(data, n, n_samples, rotate, on_device);
            GenerateCentroids(data, n_samples, n_clusters, rotate, on_device);
            // prev_centroids <- rotated initial centroids; horizontal_centroids still holds the raw rows.
            RotateOrCopy(horizontal_centroids.get(), prev_centroids.get(), n_clusters, rotate);
            hip::Check(skm_norms(ctx, data_to_cluster, n_samples, d, d, data_norms.get()));
        }
        n_tracked_queries = 0;
        if (n_queries) PrepareQueries(data_to_cluster, queries, n_queries, on_device);

        const bool always_gemm_only = d < DIMENSION_THRESHOLD_FOR_PRUNING || config.use_blas_only ||
                                      n_clusters <= N_CLUSTERS_THRESHOLD_FOR_PRUNING;
        bool partial_norms_computed = false;
        float best_recall = 0.0f;
        size_t iters_without_improvement = 0;
        for (size_t iter_idx = 0; iter_idx < config.iters; ++iter_idx) {
            const bool use_gemm_only = (iter_idx == 0) || always_gemm_only;
            if (!use_gemm_only && !partial_norms_computed) {
                hip::Check(skm_norms(ctx, data_to_cluster, n_samples, d, partial_d, data_norms.get()));
                partial_norms_computed = true;
            }
            RunIteration(use_gemm_only, data_to_cluster, n_samples, n_clusters, iter_idx,
                         use_gemm_only && iter_idx == 0, iteration_stats);
            if (config.early_termination &&
                ShouldStopEarly(n_queries > 0, best_recall, iters_without_improvement, iter_idx)) {
                break;
            }
        }
        trained = true;
        PublishAssignments(n_samples);
        return GetOutputCentroids(config.unrotate_centroids);
    }

    // Device and host state sized like the reference's buffers (superkmeans.h:191-209).
    void AllocateState(const size_t n, const size_t k) {
        FinishHostOutputs();  // a helper thread of an earlier, failed Train may still be touching the host buffers
        vertical_d = static_cast<uint32_t>(layout_t::GetDimensionSplit(d).vertical_d);
        centroids.Reset(ctx, k * d);
        horizontal_centroids.Reset(ctx, k * d);
        prev_centroids.Reset(ctx, k * d);
        partial_horizontal_centroids.Reset(ctx, k * vertical_d);
        d_cluster_sizes.Reset(ctx, k);
        d_assignments.Reset(ctx, n);
        distances.Reset(ctx, n);
        data_norms.Reset(ctx, n_samples);
        centroid_norms.Reset(ctx, k);
        cluster_sizes.reset(new uint32_t[k]);
        assignments.reset(new uint32_t[n]);
    }

    // One k-means iteration (reference RunIteration<GEMM_ONLY>, superkmeans.h:786-879).
    void RunIteration(const bool gemm_only, const float* data_to_cluster, const size_t n_samples_, const size_t k,
                      const size_t iter_idx, const bool is_first_iter,
                      std::vector<SuperKMeansIterationStats>& target_stats) {
        if (!is_first_iter) horizontal_centroids.swap(prev_centroids);
        uint64_t not_pruned_total = 0;
        if (gemm_only && is_first_iter && first_search_done) {
            first_search_done = false;  // Train searched slab by slab while the rows were uploaded
        } else if (gemm_only) {
            hip::Check(skm_norms(ctx, prev_centroids.get(), k, d, d, centroid_norms.get()));
            hip::Check(skm_assign_full(ctx, data_to_cluster, n_samples_, prev_centroids.get(), k, d, data_norms.get(),
                                       centroid_norms.get(), d_assignments.get(), distances.get()));
        } else {
            hip::Check(skm_norms(ctx, prev_centroids.get(), k, d, partial_d, centroid_norms.get()));
            EnsurePdxLayout(prev_centroids.get(), k);
            std::vector<uint64_t> stage_pairs;
            if (collect_prune_accounting) stage_pairs.assign((d - vertical_d) / H_DIM_SIZE + 2, 0);
            hip::Check(skm_assign_pruned(ctx, data_to_cluster, n_samples_, prev_centroids.get(), centroids.get(),
                                         partial_horizontal_centroids.get(), k, d, vertical_d, partial_d,
                                         pruner->DeviceRatios(), data_norms.get(), centroid_norms.get(),
                                         d_assignments.get(), distances.get(), &not_pruned_total,
                                         collect_prune_accounting ? stage_pairs.data() : nullptr));
            if (collect_prune_accounting) prune_accounting.push_back(std::move(stage_pairs));
        }
        // The sum of the distances is queued here and collected in ComputeCost: by then the stream has been waited for
        // anyway (cluster sizes), so the cost takes no wait of its own.
        hip::Check(skm_wcss_begin(ctx, distances.get(), n_samples_));
        // Sums and counts (zero-filled by the kernel itself for empty clusters).
        hip::Check(skm_update(ctx, data_to_cluster, n_samples_, d, d_assignments.get(), k, horizontal_centroids.get(),
                              d_cluster_sizes.get()));

        float avg_not_pruned_pct = -1.0f;
        const uint32_t old_partial_d = partial_d;
        if (!gemm_only) {
            bool partial_d_changed = false;
            avg_not_pruned_pct = TunePartialD(not_pruned_total, n_samples_, k, partial_d_changed);
            if (partial_d_changed) {
                hip::Check(skm_norms(ctx, data_to_cluster, n_samples_, d, partial_d, data_norms.get()));
            }
        }
        ConsolidateCentroids(n_samples_, k);
        ComputeCost(n_samples_);
        ComputeShift(k);
        if (n_tracked_queries) {
            hip::Check(skm_norms(ctx, horizontal_centroids.get(), k, d, d, centroid_norms.get()));
            recall = ComputeRecall(n_samples_, k);
        }

        SuperKMeansIterationStats stats;
        stats.iteration = iter_idx + 1;
        stats.objective = cost;
        stats.shift = shift;
        stats.split = n_split;
        stats.recall = recall;
        stats.is_gemm_only = gemm_only;
        if (!gemm_only) {
            stats.not_pruned_pct = avg_not_pruned_pct;
            stats.partial_d = old_partial_d;
        }
        target_stats.push_back(stats);
        if (config.verbose) {
            std::cout << "Iteration " << iter_idx + 1 << "/" << config.iters << " | Objective: " << cost
                      << " | Objective improvement: " << (iter_idx > 0 ? 1 - (cost / prev_cost) : 0.0f)
                      << " | Shift: " << shift << " | Split: " << n_split << " | Recall: " << recall;
            if (gemm_only) {
                std::cout << " [GEMM-only]";
            } else {
                std::cout << " | Not Pruned %: " << avg_not_pruned_pct * 100.0f << " | d': " << old_partial_d << " -> "
                          << partial_d;
            }
            std::cout << std::endl << std::endl;
        }
    }

    // A pending row edit for skm_edit_rows.
    struct RowEdit {
        uint32_t kind, dst, src;
        float weight;
    };
    void ApplyRowEdits(const std::vector<RowEdit>& edits) {
        if (edits.empty()) return;
        std::vector<uint32_t> ops(edits.size() * 4);
        for (size_t i = 0; i < edits.size(); ++i) {
            ops[4 * i] = edits[i].kind;
            ops[4 * i + 1] = edits[i].dst;
            ops[4 * i + 2] = edits[i].src;
            std::memcpy(&ops[4 * i + 3], &edits[i].weight, sizeof(float));
        }
        hip::Check(skm_edit_rows(ctx, horizontal_centroids.get(), d, ops.data(), edits.size()));
    }

    /**
     * Empty clusters are re-seeded from a large one (FAISS rule; reference superkmeans.h:890-928):
     * walk the clusters cyclically and accept cj with probability (size_cj - 1) / (n - k), one
     * uniform draw from mt19937(seed) per visit; the donor row is copied and both copies perturbed by
     * (1 +/- 1/1024) alternating per column; the donor's size is split in two.  Decisions need only
     * the sizes, so they are taken on the host and the row arithmetic is queued for the device.
     */
    virtual void SplitClusters(const size_t n_samples_, const size_t k) {
        n_split = 0;
        std::mt19937 rng(config.seed);
        std::vector<RowEdit> edits;
        // Acceptance probabilities of the walk, tabulated (an empty cluster takes thousands of visits) and
        // refreshed for the two clusters a split changes; same arithmetic as the reference's expression.
        const auto accept_probability = [&](const size_t c) -> float {
            return (cluster_sizes[c] - 1.0) / (float) (n_samples_ - k);
        };
        // With the direct form of the draws the test `draw < p` is decided on the engine's raw 32-bit output
        // against an integer bound per cluster (same decisions, no float conversion in the walk), and the
        // outputs come in blocks so that the walk scans arrays.  A bound of 2^32 (p >= 1, which sizes of a
        // real clustering do not produce) does not fit the table: then every draw goes through the engine.
        std::vector<float> prob;
        std::vector<uint32_t> bound;
        UnitUniformDraws draw(rng);
        Mt19937Blocks blocks(static_cast<uint32_t>(config.seed));
        bool on_raw = draw.direct();
        const auto set_bound = [&](const size_t c) -> bool {
            const uint64_t b = UnitUniformDraws::AcceptBelow(prob[c]);
            bound[c] = static_cast<uint32_t>(b);
            return b <= 0xffffffffu;
        };
        for (size_t ci = 0; ci < k; ci++) {
            if (cluster_sizes[ci] != 0) continue;
            if (prob.empty()) {
                prob.resize(k);
                for (size_t c = 0; c < k; ++c) prob[c] = accept_probability(c);
                if (on_raw) {
                    bound.resize(k);
                    bool any = false;
                    for (size_t c = 0; c < k; ++c) {
                        on_raw = set_bound(c) && on_raw;
                        any = any || bound[c] != 0;
                    }
                    on_raw = on_raw && any;  // with no acceptable cluster the walk below never ends, as in the reference
                }
            }
            size_t cj;
            if (on_raw) {
                cj = blocks.WalkToFirstAccepted(bound.data(), k);
            } else {
                for (cj = 0; true; cj = (cj + 1 == k) ? 0 : cj + 1) {
                    if (draw() < prob[cj]) break;
                }
            }
            edits.push_back({0u, static_cast<uint32_t>(ci), static_cast<uint32_t>(cj), 0.0f});
            cluster_sizes[ci] = cluster_sizes[cj] / 2;
            cluster_sizes[cj] -= cluster_sizes[ci];
            prob[ci] = accept_probability(ci);
            prob[cj] = accept_probability(cj);
            if (on_raw) {
                // probabilities only shrink (a split halves the donor), so the bounds keep fitting
                set_bound(ci);
                set_bound(cj);
            }
            n_split++;
        }
        ApplyRowEdits(edits);
    }

    // Means, empty-cluster handling, optional normalisation, PDX relayout (superkmeans.h:936-968).
    void ConsolidateCentroids(const size_t n_samples_, const size_t k) {
        hip::Check(skm_scale_by_size_fetch(ctx, horizontal_centroids.get(), d_cluster_sizes.get(), k, d, cluster_sizes.get()));
        SplitClusters(n_samples_, k);
        if (config.angular) {
            hip::Check(skm_normalize_rows(ctx, horizontal_centroids.get(), k, d));
        }
        // The PDX copies are read by pruned searches only: they are brought up to date when one is about to run
        // (EnsurePdxLayout), so exact-only clusterings never pay for the relayout.
        pdx_layout_stale = true;
    }

    // PDX copy and dense leading columns of `rows` (the current centroids, wherever the last swap left them), if
    // the last ConsolidateCentroids has not been followed by a relayout yet (reference superkmeans.h:962-967).
    void EnsurePdxLayout(const float* rows, const size_t k) {
        if (!pdx_layout_stale) return;
        hip::Check(skm_pdxify(ctx, rows, k, d, vertical_d, centroids.get(), partial_horizontal_centroids.get()));
        pdx_layout_stale = false;
    }

    // WCSS of this iteration's assignments; accumulated in fp64 on the device (superkmeans.h:973-981
    // sums the same values in fp32).
    void ComputeCost(const size_t n_samples_) {
        prev_cost = cost;
        double c = 0.0;
        (void) n_samples_;
        hip::Check(skm_wcss_end(ctx, &c));
        cost_f64 = c;
        cost = static_cast<float>(c);
    }

    void ComputeShift(const size_t k) {
        double s = 0.0;
        hip::Check(skm_shift(ctx, horizontal_centroids.get(), prev_centroids.get(), k, d, &s));
        shift = static_cast<float>(s);
    }

    /**
     * Query set-up of Train (reference superkmeans.h:243-274): the rotated queries (given, or drawn from the
     * training sample with the first n_queries entries of a mt19937(seed) shuffle of [0, n_samples)), their
     * norms, and for every query its objective_k nearest training rows (GetGTAssignmentsAndDistances,
     * superkmeans.h:1010-1031).  data_norms must hold full-dimension norms, as they do at this point of Train.
     * The reference's draw reuses the member that maps sampled rows back to the input, which breaks a later
     * AssignTrainingPoints on sampled data; here that map is left alone.
     */
    void PrepareQueries(const float* data_to_cluster, const vector_value_t* queries, const size_t n_queries,
                        const bool on_device) {
        centroids_to_explore = std::max<size_t>(static_cast<size_t>(n_clusters * config.ann_explore_fraction), 1);
        if (config.verbose) {
            std::cout << "Centroids to explore: " << centroids_to_explore << " ("
                      << config.ann_explore_fraction * 100.0f << "% of " << n_clusters << ")" << std::endl;
        }
        if (config.objective_k == 0 || config.objective_k > 1024 || centroids_to_explore > 1024) {
            throw std::invalid_argument(
                "recall tracking supports objective_k and n_clusters * ann_explore_fraction up to 1024");
        }
        rotated_queries.Reset(ctx, n_queries * d);
        if (config.sample_queries) {
            if (n_queries > n_samples) {
                throw std::invalid_argument("cannot sample more queries than there are training samples");
            }
            if (n_queries < n_samples) {
                std::mt19937 rng(config.seed);
                std::vector<size_t> order(n_samples);
                std::iota(order.begin(), order.end(), size_t{0});
                std::shuffle(order.begin(), order.end(), rng);
                std::vector<uint64_t> rows(order.begin(), order.begin() + n_queries);
                dbuf<uint64_t> d_rows(ctx, n_queries);
                d_rows.Upload(rows.data(), n_queries);
                hip::Check(skm_gather_rows(ctx, data_to_cluster, d, d_rows.get(), n_queries, rotated_queries.get(),
                                           nullptr, nullptr));
                hip::Check(skm_sync(ctx));
            } else {
                hip::Check(skm_copy(ctx, rotated_queries.get(), data_to_cluster, sizeof(float) * n_queries * d));
            }
        } else if (on_device) {
            RotateOrCopy(queries, rotated_queries.get(), n_queries, !config.data_already_rotated);
        } else {
            dbuf<float> raw(ctx, n_queries * d);
            raw.Upload(queries, n_queries * d);
            RotateOrCopy(raw.get(), rotated_queries.get(), n_queries, !config.data_already_rotated);
            hip::Check(skm_sync(ctx));  // `raw` is released on return
        }
        query_norms.Reset(ctx, n_queries);
        gt_assignments.Reset(ctx, n_queries * config.objective_k);
        gt_distances.Reset(ctx, n_queries * config.objective_k);
        promising_centroids.Reset(ctx, n_queries * centroids_to_explore);
        recall_distances.Reset(ctx, n_queries * centroids_to_explore);
        hip::Check(skm_norms(ctx, rotated_queries.get(), n_queries, d, d, query_norms.get()));
        hip::Check(skm_knn(ctx, rotated_queries.get(), n_queries, data_to_cluster, n_samples, d, query_norms.get(),
                           data_norms.get(), config.objective_k, gt_assignments.get(), gt_distances.get()));
        n_tracked_queries = n_queries;
    }

    /**
     * recall@objective_k of the current centroids (reference superkmeans.h:1044-1087): the share of a query's
     * ground-truth neighbours whose cluster is among the query's centroids_to_explore nearest centroids,
     * averaged over the queries with the reference's fp32 accumulation order.  centroid_norms must hold the
     * full norms of horizontal_centroids.
     */
    float ComputeRecall(const size_t n_samples_, const size_t k) {
        const size_t nq = n_tracked_queries;
        hip::Check(skm_knn(ctx, rotated_queries.get(), nq, horizontal_centroids.get(), k, d, query_norms.get(),
                           centroid_norms.get(), centroids_to_explore, promising_centroids.get(),
                           recall_distances.get()));
        std::vector<uint32_t> hits(nq);
        hip::Check(skm_recall_hits(ctx, gt_assignments.get(), promising_centroids.get(), d_assignments.get(),
                                   n_samples_, nq, config.objective_k, centroids_to_explore, hits.data()));
        float sum_recall = 0.0f;
        for (size_t i = 0; i < nq; ++i) {
            sum_recall += static_cast<float>(hits[i]) / static_cast<float>(config.objective_k);
        }
        return sum_recall / static_cast<float>(nq);
    }

    /**
     * Forgy initialisation (reference superkmeans.h:1100-1142): shuffle [0, n_points) with
     * mt19937(seed) and take the first k rows of `data`; the rows land in horizontal_centroids
     * (raw) and, when no iteration will replace it, their rotated, PDX-laid-out copy in `centroids`.
     */
    void GenerateCentroids(const vector_value_t* data, const size_t n_points, const size_t k, const bool rotate,
                           const bool on_device) {
        if (k > n_points) {
            throw std::runtime_error("cannot draw more initial centroids than there are points");
        }
        std::mt19937 rng(config.seed);
        const std::vector<size_t> indices = ShuffledPrefix::Draw(n_points, k, rng);
        if (on_device) {
            std::vector<uint64_t> rows(indices.begin(), indices.begin() + k);
            dbuf<uint64_t> d_rows(ctx, k);
            d_rows.Upload(rows.data(), k);
            hip::Check(skm_gather_rows(ctx, data, d, d_rows.get(), k, horizontal_centroids.get(), nullptr, nullptr));
            hip::Check(skm_sync(ctx));
        } else {
            std::vector<float> staged(k * d);
            GatherHostRows(staged.data(), data, indices.data(), k);
            horizontal_centroids.Upload(staged.data(), k * d);
        }
        // The PDX copy of the initial centroids is read only if no iteration follows: the first iteration is always
        // exact and ConsolidateCentroids replaces the copy before any pruned search.
        pdx_layout_stale = false;
        if (config.iters == 0) {
            dbuf<float> rotated(ctx, k * d);
            RotateOrCopy(horizontal_centroids.get(), rotated.get(), k, rotate);
            hip::Check(skm_pdxify(ctx, rotated.get(), k, d, vertical_d, centroids.get(), nullptr));
            hip::Check(skm_sync(ctx));
        }
    }

    void RotateOrCopy(const float* d_in, float* d_out, const size_t n_vectors, const bool rotate) {
        if (rotate) {
            pruner->Rotate(ctx, d_in, d_out, n_vectors);
        } else {
            hip::Check(skm_copy(ctx, d_out, d_in, sizeof(float) * n_vectors * d));
        }
    }

    /**
     * d' tuning (reference superkmeans.h:1230-1258): p = not-pruned pairs / (n * k); above
     * max_not_pruned_pct grow d' by 2 * adjustment (at least 1) up to vertical_d, below
     * min_not_pruned_pct shrink it by adjustment (at least 1) down to MIN_PARTIAL_D.  The pair count
     * is summed exactly on the device.
     */
    float TunePartialD(const uint64_t not_pruned_total, size_t n_samples_, size_t n_y, bool& partial_d_changed) {
        float avg_not_pruned_pct = static_cast<float>(static_cast<double>(not_pruned_total));
        avg_not_pruned_pct /= static_cast<float>(n_samples_ * n_y);
        const uint32_t old_partial_d = partial_d;
        if (avg_not_pruned_pct > config.max_not_pruned_pct) {
            auto increase = static_cast<uint32_t>(partial_d * config.adjustment_factor_for_partial_d * 2);
            partial_d = std::min(partial_d + std::max(increase, 1u), vertical_d);
        } else if (avg_not_pruned_pct < config.min_not_pruned_pct) {
            auto decrease = static_cast<uint32_t>(partial_d * config.adjustment_factor_for_partial_d);
            partial_d = std::max(partial_d - std::max(decrease, 1u), MIN_PARTIAL_D);
        }
        partial_d_changed = (old_partial_d != partial_d);
        return avg_not_pruned_pct;
    }

    [[nodiscard]] virtual size_t GetNVectorsToSample(const size_t n, size_t k) const {
        if (config.sampling_fraction == 1.0) return n;
        auto samples_by_clusters = k * config.max_points_per_cluster;
        auto samples_by_n = static_cast<size_t>(std::floor(static_cast<float>(n) * config.sampling_fraction));
        return std::min<size_t>(samples_by_n, samples_by_clusters);
    }

    bool ShouldStopEarly(const bool tracking_recall, float& best_recall, size_t& iters_without_improvement,
                         const size_t iter_idx) {
        if (shift < config.tol) {
            if (config.verbose)
                std::cout << "Converged at iteration " << iter_idx + 1 << " (shift " << shift << " < tol "
                          << config.tol << ")" << std::endl;
            return true;
        }
        if (iter_idx > 0) {
            auto cost_delta = cost / prev_cost;
            if (cost_delta > 1 - config.tol) {
                if (config.verbose)
                    std::cout << "Converged at iteration " << iter_idx + 1 << " (cost improved by only "
                              << 1 - cost_delta << ")" << std::endl;
                return true;
            }
        }
        if (tracking_recall) {
            float improvement = recall - best_recall;
            if (improvement > config.recall_tol) {
                best_recall = recall;
                iters_without_improvement = 0;
            } else {
                iters_without_improvement++;
                if (iters_without_improvement >= RECALL_CONVERGENCE_PATIENCE) return true;
            }
        }
        return false;
    }

    std::vector<centroid_value_t> GetOutputCentroids(bool should_unrotate) {
        // With a sink set the centroids go straight to the caller's buffer and the returned vector is empty.
        std::vector<centroid_value_t> out;
        dbuf<float> unrotated;
        if (should_unrotate) {
            unrotated.Reset(ctx, n_clusters * d);
            pruner->Unrotate(ctx, horizontal_centroids.get(), unrotated.get(), n_clusters);
        }
        FinishHostOutputs();
        centroid_value_t* dst = output_sink;
        if (dst == nullptr) {
            if (prepared_centroids.size() == n_clusters * d) {
                out = std::move(prepared_centroids);
                prepared_centroids = std::vector<centroid_value_t>();
            } else {
                out.resize(n_clusters * d);
            }
            dst = out.data();
        }
        if (should_unrotate) {
            unrotated.Download(dst, n_clusters * d);
        } else {
            horizontal_centroids.Download(dst, n_clusters * d);
        }
        return out;
    }

    /**
     * Produces the (sampled, rotated) training matrix on the device and returns its address
     * (reference superkmeans.h:1385-1443).  Sampling shuffles [0, n) with mt19937(seed) and takes the
     * first n_samples indices.  Without rotation and without sampling a device-resident input is
     * used in place.
     */
    const float* SampleAndRotateVectors(const vector_value_t* data, const size_t n, const size_t n_samples_,
                                        const bool rotate, const bool on_device,
                                        const std::function<void(const float*, size_t, size_t)>& after_slab = {}) {
        const bool sample = n_samples_ < n;
        if (sample) {
            std::mt19937 rng(config.seed);
            sampled_indices.reset(new size_t[n]);
            for (size_t i = 0; i < n; ++i) sampled_indices[i] = i;
            std::shuffle(sampled_indices.get(), sampled_indices.get() + n, rng);
        }
        if (on_device && !sample && !rotate) return data;
        if (!on_device) {
            // Host rows: slab after slab on the transfer stream, each one rotated (and handed to after_slab:
            // training rows on the device, first row, count) while the next is copied.  All rows in order are
            // copied from where they lie; sampled rows are gathered into one of two staging buffers, the next
            // slab by a helper thread during the copy of the current one (a copy from pageable memory returns
            // once the source has been read).
            training_data.Reset(ctx, n_samples_ * d);
            dbuf<float> raw;
            if (rotate) raw.Reset(ctx, n_samples_ * d);
            dbuf<float>& landing = rotate ? raw : training_data;
            const size_t slab = sample ? std::max<size_t>(1, (size_t(64) << 20) / (d * sizeof(float))) : UploadSlabRows();
            std::vector<float> host[2];
            const auto gather = [&](const size_t which, const size_t i0) {
                const size_t m = std::min(slab, n_samples_ - i0);
                host[which].resize(m * d);
                GatherHostRows(host[which].data(), data, sampled_indices.get() + i0, m);
            };
            if (sample) gather(0, 0);
            size_t which = 0;
            for (size_t r0 = 0; r0 < n_samples_; r0 += slab, which ^= 1) {
                const size_t m = std::min(slab, n_samples_ - r0);
                std::thread ahead;
                if (sample && r0 + slab < n_samples_) ahead = std::thread(gather, which ^ 1, r0 + slab);
                try {
                    landing.UploadOverlapped(sample ? host[which].data() : data + r0 * d, m * d, r0 * d);
                    if (rotate) pruner->Rotate(ctx, raw.get() + r0 * d, training_data.get() + r0 * d, m);
                    if (after_slab) after_slab(training_data.get() + r0 * d, r0, m);
                } catch (...) {
                    if (ahead.joinable()) ahead.join();
                    throw;
                }
                if (ahead.joinable()) ahead.join();
            }
            if (rotate) hip::Check(skm_sync(ctx));  // `raw` is released on return
            return training_data.get();
        }
        dbuf<float> staged;  // raw rows on the device, in training order
        const float* d_raw = nullptr;
        if (!sample) {
            d_raw = data;
        } else {
            std::vector<uint64_t> rows(sampled_indices.get(), sampled_indices.get() + n_samples_);
            dbuf<uint64_t> d_rows(ctx, n_samples_);
            d_rows.Upload(rows.data(), n_samples_);
            staged.Reset(ctx, n_samples_ * d);
            hip::Check(skm_gather_rows(ctx, data, d, d_rows.get(), n_samples_, staged.get(), nullptr, nullptr));
            hip::Check(skm_sync(ctx));
            d_raw = staged.get();
        }
        if (!rotate) {
            training_data = std::move(staged);
            return training_data.get();
        }
        training_data.Reset(ctx, n_samples_ * d);
        pruner->Rotate(ctx, d_raw, training_data.get(), n_samples_);
        if (staged.get() != nullptr) hip::Check(skm_sync(ctx));  // `staged` is released on return
        return training_data.get();
    }

    // dst[i] = data[rows[i]] for i < count.  The rows are scattered over a matrix of gigabytes, so the copy is
    // bound by memory latency: a few host threads split the range.
    void GatherHostRows(float* dst, const vector_value_t* data, const size_t* rows, const size_t count) const {
        const size_t row_bytes = sizeof(float) * d;
        size_t workers = std::min<size_t>(std::max(1u, std::thread::hardware_concurrency()), 8);
        workers = std::min(workers, std::max<size_t>(1, count * row_bytes >> 22));  // at least 4 MiB per thread
        const auto copy_range = [&](const size_t begin, const size_t end) {
            for (size_t i = begin; i < end; ++i) std::memcpy(dst + i * d, data + rows[i] * d, row_bytes);
        };
        if (workers <= 1) {
            copy_range(0, count);
            return;
        }
        std::vector<std::thread> pool;
        for (size_t w = 1; w < workers; ++w) pool.emplace_back(copy_range, count * w / workers, count * (w + 1) / workers);
        copy_range(0, count / workers);
        for (auto& t : pool) t.join();
    }

    // Copies the device assignments / distances of the training points to the public host members.
    void PublishAssignments(const size_t count) {
        FinishHostOutputs();
        d_assignments.Download(assignments.get(), count);
        host_distances.resize(count);
        distances.Download(host_distances.data(), count);
    }

    // The host memory the end of Train fills: the assignments, the distances and the returned centroids.  Every
    // fresh page costs a fault and a zeroing (20 ms for the 268 MB of 65,536 centroids of 1,024 dimensions), so a
    // helper thread touches them while the device trains.  FinishHostOutputs comes before anything else reads or
    // writes these buffers.
    void PrepareHostOutputs(const size_t count) {
        FinishHostOutputs();
        const bool want_centroids = output_sink == nullptr;
        const size_t bytes = count * (sizeof(uint32_t) + sizeof(float)) +
                             (want_centroids ? n_clusters * d * sizeof(centroid_value_t) : 0);
        if (bytes < HOST_OUTPUTS_AHEAD_BYTES) return;
        host_outputs_thread = std::thread([this, count, want_centroids] {
            try {
                std::memset(assignments.get(), 0, count * sizeof(uint32_t));
                host_distances.assign(count, 0.0f);
                if (want_centroids) prepared_centroids.assign(n_clusters * d, centroid_value_t(0));
            } catch (...) {
                prepared_centroids.clear();  // the buffers are then made where they are filled
            }
        });
    }
    void FinishHostOutputs() {
        if (host_outputs_thread.joinable()) host_outputs_thread.join();
    }
    static constexpr size_t HOST_OUTPUTS_AHEAD_BYTES = size_t(16) << 20;

    const size_t d;
    const size_t n_clusters;
    SuperKMeansConfig config;

    uint32_t n_threads;
    size_t n_samples = 0;
    uint32_t partial_d = 0;

    bool trained = false;
    bool first_search_done = false;  // Train's first exact search ran during the upload of the rows
    bool pdx_layout_stale = false;   // ConsolidateCentroids ran since the PDX copies were last written
    size_t n_split = 0;
    uint32_t vertical_d = 0;
    float prev_cost = 0.0f;
    float cost = 0.0f;
    double cost_f64 = 0.0;
    float shift = 0.0f;
    float recall = 0.0f;

    std::shared_ptr<hip::Context> context;
    skm_ctx* ctx = nullptr;
    std::shared_ptr<pruner_t> pruner;

    // Device state (names follow the reference's members, superkmeans.h:1470-1480).  Declared after `context`:
    // members are destroyed in reverse order and a buffer releases its memory through the context.
    dbuf<float> centroids;                     // PDX layout
    dbuf<float> horizontal_centroids;          // row-major: raw init rows -> sums -> means
    dbuf<float> prev_centroids;                // centroids the current iteration searches against
    dbuf<float> partial_horizontal_centroids;  // first vertical_d columns, dense
    dbuf<float> distances;
    dbuf<uint32_t> d_cluster_sizes;
    dbuf<uint32_t> d_assignments;
    dbuf<float> data_norms;
    dbuf<float> centroid_norms;
    dbuf<float> training_data;  // rotated samples (unused when the caller's device buffer is used in place)
    dbuf<float> assign_v_norms, assign_c_norms, assign_dist;  // scratch of AssignDevice, kept between calls

    // Host state
    std::unique_ptr<uint32_t[]> cluster_sizes;
    std::unique_ptr<size_t[]> sampled_indices;

    // Recall tracking (training with queries): device-resident lists.
    size_t n_tracked_queries = 0;
    size_t centroids_to_explore = 0;
    dbuf<float> rotated_queries, query_norms, gt_distances, recall_distances;
    dbuf<uint32_t> gt_assignments, promising_centroids;
    std::vector<float> host_distances;
    std::vector<uint32_t> training_seeds;  // GetTrainingSeeds
    uint64_t training_overflow_points = 0;  // GetTrainingOverflow
    std::vector<centroid_value_t> prepared_centroids;  // PrepareHostOutputs
    std::thread host_outputs_thread;
    bool collect_prune_accounting = false;
    std::vector<std::vector<uint64_t>> prune_accounting;

  public:
    std::unique_ptr<uint32_t[]> assignments;
    std::vector<SuperKMeansIterationStats> iteration_stats;
    // Not in the reference.  When set, Train() writes the n_clusters * d centroids here and returns an empty
    // vector: the C ABI passes the caller's buffer in, which saves a zero-filled temporary and a copy (41 MB
    // each at k=10,000, d=1024).
    centroid_value_t* output_sink = nullptr;
};

} // namespace skmeans
