// skmeans::HierarchicalSuperKMeans, HIP backend for MI355X.
//
// Same public interface as the reference's include/superkmeans/hierarchical_superkmeans.h
// (config :11-17, stats :22-26, constructors :43-72, Train :84, GetNMesoclusters :549, public
// members :817-825).  Three phases, all built from SuperKMeans::RunIteration on device buffers:
//   1. mesoclustering: round(sqrt(k)) clusters over every sample;
//   2. fine clustering: every mesocluster is gathered into a contiguous device buffer
//      (skm_gather_rows) and clustered on its own; local ids are scattered back with the running
//      cluster offset (skm_scatter_assignments);
//   3. refinement: optional pruned iterations over all k clusters.
#pragma once

#include <atomic>
#include <exception>
#include <thread>

#include "superkmeans/superkmeans.h"

namespace skmeans {

struct HierarchicalSuperKMeansConfig : SuperKMeansConfig {
    uint32_t iters_mesoclustering = 3;
    uint32_t iters_fineclustering = 5;
    uint32_t iters_refinement = 0;

    HierarchicalSuperKMeansConfig() { sampling_fraction = 1.0f; }
};

struct HierarchicalSuperKMeansIterationStats {
    std::vector<SuperKMeansIterationStats> mesoclustering_iteration_stats;
    std::vector<SuperKMeansIterationStats> refinement_iteration_stats;
    std::vector<SuperKMeansIterationStats> fineclustering_iteration_stats;
};

template <Quantization q = Quantization::f32, DistanceFunction alpha = DistanceFunction::l2>
class HierarchicalSuperKMeans : public SuperKMeans<q, alpha> {
    using base = SuperKMeans<q, alpha>;
    using typename base::centroid_value_t;
    using typename base::vector_value_t;
    using typename base::pruner_t;
    using typename base::RowEdit;
    template <class T>
    using dbuf = hip::Buffer<T>;

  public:
    HierarchicalSuperKMeans(size_t n_clusters, size_t dimensionality, const HierarchicalSuperKMeansConfig& config)
        : base(n_clusters, dimensionality, config), hierarchical_config(config) {
        // Looser ADSampling epsilon for the hierarchical driver (common.h of the reference, :115): same
        // rotation matrix (same seed), other threshold ratios.
        this->pruner->SetEpsilon0(HIERARCHICAL_PRUNER_INITIAL_THRESHOLD);
        SKMEANS_ENSURE_POSITIVE(config.iters_mesoclustering);
        SKMEANS_ENSURE_POSITIVE(config.iters_fineclustering);
        static_cast<SuperKMeansConfig&>(hierarchical_config) = this->config;
        hierarchical_config.sampling_fraction = config.sampling_fraction;
        if (n_clusters <= 128 && !this->hierarchical_config.suppress_warnings) {
            std::cout << "WARNING: n_clusters <= 128 is not recommended for HierarchicalSuperKMeans. "
                         "Consider using at least 128 clusters."
                      << std::endl;
        }
    }

    HierarchicalSuperKMeans(size_t n_clusters, size_t dimensionality)
        : HierarchicalSuperKMeans(n_clusters, dimensionality, HierarchicalSuperKMeansConfig{}) {}

  protected:
    // Fine-phase helper of `owner`: own device context, the owner's pruner tables and configuration.
    struct FineHelperTag {};
    HierarchicalSuperKMeans(const HierarchicalSuperKMeans& owner, FineHelperTag)
        : base(owner.n_clusters, owner.d, owner.config, owner.pruner), hierarchical_config(owner.hierarchical_config) {}

  public:

    /** Hierarchical training on host-resident data; queries are ignored (as in the reference). */
    std::vector<centroid_value_t> Train(const vector_value_t* data, const size_t n,
                                        const vector_value_t* queries = nullptr, const size_t n_queries = 0) {
        (void) queries;
        return TrainHierarchical(data, n, n_queries, /*on_device=*/false);
    }

    std::vector<centroid_value_t> TrainDevice(const vector_value_t* d_data, const size_t n,
                                              const vector_value_t* d_queries = nullptr,
                                              const size_t n_queries = 0) {
        (void) d_queries;
        return TrainHierarchical(d_data, n, n_queries, /*on_device=*/true);
    }

    static size_t GetNMesoclusters(const size_t n_clusters) {
        return static_cast<size_t>(std::round(std::sqrt(n_clusters)));
    }

  protected:
    std::vector<centroid_value_t> TrainHierarchical(const vector_value_t* data, const size_t n, const size_t n_queries,
                                                    const bool on_device) {
        SKMEANS_ENSURE_POSITIVE(n);
        if (this->trained) {
            throw std::runtime_error("The clustering has already been trained");
        }
        if (n_queries > 0 && !hierarchical_config.suppress_warnings) {
            std::cout << "WARNING: Early Termination by Recall is not supported in HierarchicalSuperKMeans"
                      << std::endl;
        }
        const size_t k = this->n_clusters;
        const size_t d = this->d;
        skm_ctx* ctx = this->ctx;
        n_mesoclusters = GetNMesoclusters(k);
        hierarchical_iteration_stats = HierarchicalSuperKMeansIterationStats{};
        if (n < k) {
            throw std::runtime_error("The number of points should be at least as large as the number of clusters");
        }
        this->n_samples = this->GetNVectorsToSample(n, k);
        if (this->n_samples < k) {
            throw std::runtime_error(
                "Not enough samples to train. Try increasing the sampling_fraction or max_points_per_cluster");
        }
        const size_t total_samples = this->n_samples;
        this->AllocateState(n, k);
        this->PrepareHostOutputs(total_samples);
        final_assignments.Reset(ctx, total_samples);
        final_centroids.Reset(ctx, k * d);
        this->partial_d = std::max<uint32_t>(MIN_PARTIAL_D, this->vertical_d / 2);
        if (this->partial_d > this->vertical_d) this->partial_d = this->vertical_d;
        const uint32_t initial_partial_d = this->partial_d;
        const bool rotate = !hierarchical_config.data_already_rotated;

        // ---- phase 1: mesoclustering over all samples ----
        if (hierarchical_config.verbose)
            std::cout << "\n=== PHASE 1: MESOCLUSTERING (k=" << n_mesoclusters << " clusters) ===" << std::endl;
        // The fine phase's helper objects (a device context each: a stream, pinned result slots) are made first, while
        // the device is idle: their number depends on nothing the mesoclustering computes, and creating streams and
        // pinned memory while a kernel runs slows that kernel down (the rotation of 10 M points took 170 instead of
        // 150 ms with the eight helpers made beside it).
        const size_t wanted = this->config.n_threads == 0 ? FINE_HELPERS_DEFAULT : this->config.n_threads;
        const size_t n_helpers = std::max<size_t>(1, std::min<size_t>({wanted, FINE_HELPERS_MAX, n_mesoclusters}));
        std::vector<std::unique_ptr<HierarchicalSuperKMeans>> helpers;
        for (size_t h = 0; n_helpers > 1 && h < n_helpers; ++h)
            helpers.emplace_back(new HierarchicalSuperKMeans(*this, FineHelperTag{}));
        // Rotation next: it runs on the device while the host draws the initial mesocluster centroids.
        const float* data_to_cluster = this->SampleAndRotateVectors(data, n, total_samples, rotate, on_device);
        this->GenerateCentroids(data, total_samples, n_mesoclusters, rotate, on_device);
        this->RotateOrCopy(this->horizontal_centroids.get(), this->prev_centroids.get(), n_mesoclusters, rotate);
        hip::Check(skm_norms(ctx, data_to_cluster, total_samples, d, d, this->data_norms.get()));
        // Full norms of every sample, kept for the fine phase whose first iteration is always exact.
        immutable_data_norms.Reset(ctx, total_samples);
        hip::Check(skm_copy(ctx, immutable_data_norms.get(), this->data_norms.get(), sizeof(float) * total_samples));

        RunPhase(hierarchical_config.iters_mesoclustering, data_to_cluster, total_samples, n_mesoclusters,
                 hierarchical_config.use_blas_only, /*first_iteration_exact=*/true,
                 hierarchical_iteration_stats.mesoclustering_iteration_stats, hierarchical_config.early_termination);

        // The number of points the last search gives every mesocluster, and the point ids grouped by mesocluster,
        // ascending inside each group (hierarchical_superkmeans.h:262-286).  The reference takes the sizes from
        // cluster_sizes, which SplitClusters has already edited when a mesocluster was empty in the last iteration;
        // its partition of the points is then inconsistent with the assignments.  Here the sizes are recounted from
        // the assignments, which is identical whenever no such split happened; an empty mesocluster simply receives
        // no fine clusters.  Both come from one stable sort on the device: only the sizes travel to the host, and
        // the assignments of the mesoclustering stay on the device (mesoclusters_assignments is left empty).
        dbuf<uint64_t> d_indices(ctx, total_samples);
        {
            dbuf<uint32_t> d_meso_sizes(ctx, n_mesoclusters);
            hip::Check(skm_group_by_assignment(ctx, this->d_assignments.get(), total_samples, n_mesoclusters, d_indices.get(),
                                               d_meso_sizes.get()));
            mesoclusters_sizes.assign(n_mesoclusters, 0u);
            d_meso_sizes.Download(mesoclusters_sizes.data(), n_mesoclusters);
        }
        mesoclusters_assignments.clear();
        std::vector<size_t> offsets(n_mesoclusters + 1, 0);
        for (size_t m = 0; m < n_mesoclusters; ++m) offsets[m + 1] = offsets[m] + mesoclusters_sizes[m];

        // ---- phase 2: fine clustering, one mesocluster after the other ----
        if (hierarchical_config.verbose)
            std::cout << "\n=== PHASE 2: FINE-CLUSTERING (subdividing " << n_mesoclusters << " mesoclusters into total "
                      << k << " clusters) ===" << std::endl;
        const auto fine_clusters_nums = ArrangeFineClusters(k, n_mesoclusters, total_samples, mesoclusters_sizes);
        const size_t max_mesocluster_size = *std::max_element(mesoclusters_sizes.begin(), mesoclusters_sizes.end());
        const size_t max_fineclusters = *std::max_element(fine_clusters_nums.begin(), fine_clusters_nums.end());
        std::vector<size_t> fine_offsets(n_mesoclusters + 1, 0);
        for (size_t m = 0; m < n_mesoclusters; ++m) fine_offsets[m + 1] = fine_offsets[m] + fine_clusters_nums[m];
        FineInputs in;
        in.data_to_cluster = data_to_cluster;
        in.full_norms = immutable_data_norms.get();
        in.member_ids = d_indices.get();
        in.member_offsets = offsets.data();
        in.sizes = mesoclusters_sizes.data();
        in.fine_counts = fine_clusters_nums.data();
        in.fine_offsets = fine_offsets.data();
        in.initial_partial_d = initial_partial_d;
        in.out_assignments = final_assignments.get();
        in.out_centroids = final_centroids.get();
        dbuf<float> fine_norms(ctx, total_samples);
        in.out_norms = fine_norms.get();
        // The mesoclusters are independent problems of a few thousand points each, far too small to fill the
        // device one at a time: several helpers, each with its own stream and scratch, take them from a common
        // counter.  Every problem is computed exactly as it would be alone; the statistics are put back in
        // mesocluster order afterwards.
        std::vector<std::vector<SuperKMeansIterationStats>> fine_stats(n_mesoclusters);
        hip::Check(skm_sync(ctx));  // everything the helpers read is complete
        if (n_helpers == 1) {
            dbuf<float> mesocluster_buffer(ctx, std::max<size_t>(1, max_mesocluster_size) * d);
            for (size_t m = 0; m < n_mesoclusters; ++m) FineClusterOne(in, m, mesocluster_buffer.get(), fine_stats[m]);
        } else {
            for (size_t h = 0; h < n_helpers; ++h) {
                helpers[h]->n_samples = std::max<size_t>(1, max_mesocluster_size);  // sizes the per-point buffers
                helpers[h]->AllocateState(std::max<size_t>(1, max_mesocluster_size), std::max<size_t>(1, max_fineclusters));
            }
            std::atomic<size_t> next{0};
            std::vector<std::exception_ptr> failures(n_helpers);
            std::vector<std::thread> threads;
            for (size_t h = 0; h < n_helpers; ++h) {
                threads.emplace_back([&, h] {
                    try {
                        HierarchicalSuperKMeans& helper = *helpers[h];
                        dbuf<float> buffer(helper.ctx, std::max<size_t>(1, max_mesocluster_size) * d);
                        for (size_t m = next.fetch_add(1); m < n_mesoclusters; m = next.fetch_add(1)) {
                            helper.FineClusterOne(in, m, buffer.get(), fine_stats[m]);
                        }
                        hip::Check(skm_sync(helper.ctx));
                    } catch (...) {
                        failures[h] = std::current_exception();
                        next.store(n_mesoclusters);  // the others stop taking work
                    }
                });
            }
            for (auto& t : threads) t.join();
            for (auto& f : failures)
                if (f) std::rethrow_exception(f);
        }
        for (size_t m = 0; m < n_mesoclusters; ++m) {
            auto& all = hierarchical_iteration_stats.fineclustering_iteration_stats;
            all.insert(all.end(), fine_stats[m].begin(), fine_stats[m].end());
        }

        // ---- phase 3: refinement over all k clusters ----
        if (hierarchical_config.verbose)
            std::cout << "\n=== PHASE 3: REFINEMENT (fine-tuning all " << k << " clusters) ===" << std::endl;
        this->n_samples = total_samples;
        this->partial_d = std::max<uint32_t>(MIN_PARTIAL_D, this->vertical_d / 3);
        // SetupCentroids: the concatenated fine centroids become the current centroids in all three
        // layouts; prev_centroids gets a copy because the next iteration starts with a swap.
        hip::Check(skm_copy(ctx, this->horizontal_centroids.get(), final_centroids.get(), sizeof(float) * k * d));
        hip::Check(skm_pdxify(ctx, this->horizontal_centroids.get(), k, d, this->vertical_d, this->centroids.get(),
                              this->partial_horizontal_centroids.get()));
        this->pdx_layout_stale = false;
        hip::Check(skm_copy(ctx, this->prev_centroids.get(), final_centroids.get(), sizeof(float) * k * d));
        hip::Check(skm_copy(ctx, this->d_assignments.get(), final_assignments.get(), sizeof(uint32_t) * total_samples));
        const bool refinement_exact = d < DIMENSION_THRESHOLD_FOR_PRUNING || k <= N_CLUSTERS_THRESHOLD_FOR_PRUNING;
        // The reference runs the fine clusterings one after the other on its own norm buffer: mesocluster m leaves
        // the norms of its members (compacted order; over d' columns if it went on to prune) in the first size(m)
        // entries, the rest keeps what the mesoclustering left.  A pruned refinement recomputes the norms
        // (hierarchical_superkmeans.h:474-483); an exact one does not and searches with that buffer as it is
        // (:484-499).  A point's norm is the same addend for all its distances, so assignments and centroids do
        // not depend on it, but the distances and therefore the refinement objectives the reference reports (and
        // its tests pin, tests/test_hierarchical_superkmeans.cpp:636-670) do.  The buffer is rebuilt here in the
        // reference's order, whichever helper clustered which mesocluster, when an exact refinement follows (nothing
        // else reads it).
        for (size_t m = 0; refinement_exact && hierarchical_config.iters_refinement > 0 && m < n_mesoclusters; ++m) {
            if (fine_clusters_nums[m] == 0 || mesoclusters_sizes[m] == 0) continue;
            hip::Check(skm_copy(ctx, this->data_norms.get(), fine_norms.get() + offsets[m],
                                sizeof(float) * mesoclusters_sizes[m]));
        }
        bool refinement_norms_ready = refinement_exact;
        for (size_t it = 0; it < hierarchical_config.iters_refinement; ++it) {
            if (!refinement_norms_ready) {
                hip::Check(skm_norms(ctx, data_to_cluster, total_samples, d, this->partial_d, this->data_norms.get()));
                refinement_norms_ready = true;
            }
            this->RunIteration(refinement_exact, data_to_cluster, total_samples, k, it, /*is_first_iter=*/false,
                               hierarchical_iteration_stats.refinement_iteration_stats);
        }
        this->trained = true;
        this->PublishAssignments(total_samples);
        return this->GetOutputCentroids(hierarchical_config.unrotate_centroids);
    }

    static constexpr size_t FINE_HELPERS_DEFAULT = 8;  // concurrent fine-phase problems when n_threads is 0
    // Every helper thread waits for its stream by polling; sixteen of them on a sixteen-core share of the host were
    // throttled and took four times as long as twelve.
    static constexpr size_t FINE_HELPERS_MAX = 12;

    // What every fine-phase problem reads (device pointers of the owner, host tables) and where it writes.
    struct FineInputs {
        const float* data_to_cluster = nullptr;   // rotated samples
        const float* full_norms = nullptr;         // their norms over all d
        const uint64_t* member_ids = nullptr;      // sample ids grouped by mesocluster
        const size_t* member_offsets = nullptr;    // start of every group in member_ids
        const uint32_t* sizes = nullptr;           // points per mesocluster
        const size_t* fine_counts = nullptr;       // fine clusters per mesocluster
        const size_t* fine_offsets = nullptr;      // first global cluster id of every mesocluster
        uint32_t initial_partial_d = 0;
        uint32_t* out_assignments = nullptr;       // global cluster id of every sample
        float* out_centroids = nullptr;            // k x d
        float* out_norms = nullptr;                // per mesocluster (at its member offset): the norms it ended with
    };

    // Fine clustering of mesocluster m on this object's context (reference hierarchical_superkmeans.h:300-440):
    // members gathered into `buffer`, Forgy seeding inside the mesocluster, iters_fineclustering iterations,
    // local ids scattered back with the mesocluster's cluster offset.
    void FineClusterOne(const FineInputs& in, const size_t m, float* buffer,
                        std::vector<SuperKMeansIterationStats>& stats) {
        const size_t n_fineclusters = in.fine_counts[m];
        if (n_fineclusters == 0) return;
        const size_t dd = this->d;
        this->partial_d = in.initial_partial_d;
        const size_t mesocluster_size = in.sizes[m];
        this->n_samples = mesocluster_size;
        const uint64_t* d_member_ids = in.member_ids + in.member_offsets[m];
        // Rows and full norms of the members, contiguous (CompactMesoclusterToBuffer).
        hip::Check(skm_gather_rows(this->ctx, in.data_to_cluster, dd, d_member_ids, mesocluster_size, buffer,
                                   in.full_norms, this->data_norms.get()));
        this->GenerateCentroids(buffer, mesocluster_size, n_fineclusters, /*rotate=*/false, /*on_device=*/true);
        hip::Check(skm_copy(this->ctx, this->prev_centroids.get(), this->horizontal_centroids.get(),
                            sizeof(float) * n_fineclusters * dd));
        RunPhase(hierarchical_config.iters_fineclustering, buffer, mesocluster_size, n_fineclusters,
                 hierarchical_config.use_blas_only, /*first_iteration_exact=*/true, stats,
                 hierarchical_config.early_termination);
        hip::Check(skm_scatter_assignments(this->ctx, d_member_ids, this->d_assignments.get(), mesocluster_size,
                                           static_cast<uint32_t>(in.fine_offsets[m]), in.out_assignments));
        hip::Check(skm_copy(this->ctx, in.out_centroids + in.fine_offsets[m] * dd, this->horizontal_centroids.get(),
                            sizeof(float) * n_fineclusters * dd));
        hip::Check(skm_copy(this->ctx, in.out_norms + in.member_offsets[m], this->data_norms.get(),
                            sizeof(float) * mesocluster_size));
    }

    // Iterations of one phase: the first is always exact (GEMM only); the others are pruned unless the
    // problem is below the pruning thresholds or use_blas_only is set.
    void RunPhase(const uint32_t iters, const float* d_points, const size_t n_points, const size_t k_phase,
                  const bool blas_only, const bool first_iteration_exact, std::vector<SuperKMeansIterationStats>& stats,
                  const bool early_termination) {
        const bool always_exact = this->d < DIMENSION_THRESHOLD_FOR_PRUNING || blas_only ||
                                  k_phase <= N_CLUSTERS_THRESHOLD_FOR_PRUNING;
        bool partial_norms_computed = false;
        float best_recall = 0.0f;
        size_t iters_without_improvement = 0;
        for (size_t it = 0; it < iters; ++it) {
            const bool exact = (first_iteration_exact && it == 0) || always_exact;
            if (!exact && !partial_norms_computed) {
                hip::Check(skm_norms(this->ctx, d_points, n_points, this->d, this->partial_d, this->data_norms.get()));
                partial_norms_computed = true;
            }
            this->RunIteration(exact, d_points, n_points, k_phase, it, exact && it == 0, stats);
            if (early_termination && this->ShouldStopEarly(false, best_recall, iters_without_improvement, it)) break;
        }
    }

    [[nodiscard]] size_t GetNVectorsToSample(const size_t n, size_t /*n_clusters*/) const override {
        if (hierarchical_config.sampling_fraction == 1.0) return n;
        return static_cast<size_t>(std::floor(static_cast<double>(n) * hierarchical_config.sampling_fraction));
    }

    /**
     * Empty clusters are re-seeded as in the flat variant; then every cluster smaller than a quarter
     * of the average size is pulled towards a large cluster chosen with probability proportional to
     * its excess over the average: c <- (w c + c_large) / (w + 1), w = min(size, 7)
     * (reference hierarchical_superkmeans.h:579-678).
     */
    void SplitClusters(const size_t n_samples_, const size_t k) override {
        constexpr float CENTER_ADJUSTMENT_WEIGHT = 7.0f;
        constexpr float BALANCING_THRESHOLD = 0.25f;
        this->n_split = 0;
        std::mt19937 rng(this->config.seed);
        std::vector<RowEdit> edits;
        auto& sizes = this->cluster_sizes;
        const size_t average_size = n_samples_ / k;
        const size_t threshold_size = static_cast<size_t>(static_cast<float>(average_size) * BALANCING_THRESHOLD);
        // Acceptance probabilities of the walk, tabulated and refreshed for the two clusters a split changes.
        const auto accept_probability = [&](const size_t c) -> float {
            return (sizes[c] - 1.0f) / static_cast<float>(n_samples_ - k);
        };
        std::vector<float> prob;
        UnitUniformDraws draw(rng);
        for (size_t ci = 0; ci < k; ci++) {
            if (sizes[ci] != 0) continue;
            if (prob.empty()) {
                prob.resize(k);
                for (size_t c = 0; c < k; ++c) prob[c] = accept_probability(c);
            }
            size_t cj;
            for (cj = 0; true; cj = (cj + 1 == k) ? 0 : cj + 1) {
                if (draw() < prob[cj]) break;
            }
            edits.push_back({0u, static_cast<uint32_t>(ci), static_cast<uint32_t>(cj), 0.0f});
            sizes[ci] = sizes[cj] / 2;
            sizes[cj] -= sizes[ci];
            prob[ci] = accept_probability(ci);
            prob[cj] = accept_probability(cj);
            this->n_split++;
        }
        for (size_t ci = 0; ci < k; ci++) {
            const size_t csize = sizes[ci];
            if (csize == 0 || csize > threshold_size) continue;
            size_t large;
            for (large = 0; true; large = (large + 1) % k) {
                const size_t large_size = sizes[large];
                if (large_size < average_size) continue;
                float p = static_cast<float>(large_size - average_size + 1) /
                          static_cast<float>(n_samples_ - average_size * k + k);
                if (draw() < p) break;
            }
            const float wc = std::min(static_cast<float>(csize), CENTER_ADJUSTMENT_WEIGHT);
            edits.push_back({1u, static_cast<uint32_t>(ci), static_cast<uint32_t>(large), wc});
            this->n_split++;
        }
        this->ApplyRowEdits(edits);
    }

    /**
     * Fine clusters per mesocluster, proportional to size: lround(remaining_clusters * size /
     * remaining_samples), at least 1 for a non-empty mesocluster, never so many that a later
     * non-empty one would get none; the last mesocluster takes what is left
     * (reference hierarchical_superkmeans.h:718-761).
     */
    static std::vector<size_t> ArrangeFineClusters(size_t n_clusters, size_t n_meso, size_t n_samples_,
                                                   const std::vector<uint32_t>& sizes) {
        std::vector<size_t> out(n_meso, 0);
        size_t clusters_left = n_clusters, samples_left = n_samples_;
        size_t nonempty_left = 0;
        for (size_t i = 0; i < n_meso; ++i) nonempty_left += sizes[i] > 0 ? 1 : 0;
        for (size_t i = 0; i < n_meso; ++i) {
            if (i + 1 == n_meso) {
                out[i] = clusters_left;
            } else if (sizes[i] > 0) {
                nonempty_left--;
                const double proportion =
                    static_cast<double>(clusters_left * sizes[i]) / static_cast<double>(samples_left);
                size_t allocated = static_cast<size_t>(std::lround(proportion));
                allocated = std::min(allocated, clusters_left - nonempty_left);
                out[i] = std::max(allocated, size_t{1});
            }
            clusters_left -= out[i];
            samples_left -= sizes[i];
        }
        return out;
    }

    size_t n_mesoclusters = 0;
    std::vector<uint32_t> mesoclusters_assignments;
    std::vector<uint32_t> mesoclusters_sizes;
    dbuf<uint32_t> final_assignments;
    dbuf<float> immutable_data_norms;
    dbuf<float> final_centroids;

  public:
    HierarchicalSuperKMeansConfig hierarchical_config;
    HierarchicalSuperKMeansIterationStats hierarchical_iteration_stats;
};

} // namespace skmeans
