// Host-side helpers that callers of the reference include next to the clustering classes: a stopwatch, integer
// rounding helpers, seeded data generators and brute-force checkers.  Same names, arguments and results as the
// reference's include/superkmeans/pdx/utils.h (TicToc :17-38, rounding helpers :40-50, MakeBlobs :74-123,
// GenerateRandomVectors :138-152, brute-force checkers and generators for tests :162-356); nothing here touches the device.
#pragma once

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <limits>
#include <random>
#include <utility>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace skmeans {

/** Accumulating stopwatch: Tic() starts an interval, Toc() adds it, GetMilliseconds() reads the sum. */
class TicToc {
  public:
    size_t accum_time = 0;  // nanoseconds
    std::chrono::high_resolution_clock::time_point start = std::chrono::high_resolution_clock::now();

    void Reset() {
        accum_time = 0;
        Tic();
    }
    void Tic() { start = std::chrono::high_resolution_clock::now(); }
    void Toc() {
        const auto now = std::chrono::high_resolution_clock::now();
        accum_time += static_cast<size_t>(std::chrono::duration_cast<std::chrono::nanoseconds>(now - start).count());
    }
    double GetMilliseconds() const { return static_cast<double>(accum_time) * 1e-6; }
};

inline uint32_t CeilXToMultipleOfM(uint32_t x, uint32_t m) { return m == 0 ? x : (x + m - 1) / m * m; }
inline uint32_t FloorXToMultipleOfM(uint32_t x, uint32_t m) { return m == 0 ? x : x / m * m; }
inline bool IsPowerOf2(const uint32_t x) { return x != 0 && (x & (x - 1)) == 0; }

/**
 * Clusterable rows in the style of scikit-learn's make_blobs: n_centers centres ~ N(0, center_spread^2) drawn from
 * mt19937(random_state); row i takes a uniformly drawn centre and adds N(0, cluster_std^2) noise, both from the
 * engine of the OpenMP thread that owns the row, seeded random_state + thread number (so the rows depend on the
 * number of threads, as in the reference; one thread reproduces the matrices its tests were generated from).
 */
inline std::vector<float> MakeBlobs(size_t n_samples, size_t n_features, size_t n_centers, bool normalize = false,
                                    float cluster_std = 1.0f, float center_spread = 10.0f, uint32_t random_state = 42) {
    std::vector<float> centers(n_centers * n_features);
    {
        std::mt19937 engine(random_state);
        std::normal_distribution<float> spread(0.0f, center_spread);
        for (float& c : centers) c = spread(engine);
    }
    std::vector<float> rows(n_samples * n_features);
#pragma omp parallel
    {
        int thread = 0;
#ifdef _OPENMP
        thread = omp_get_thread_num();
#endif
        std::mt19937 engine(random_state + static_cast<uint32_t>(thread));
        std::uniform_int_distribution<size_t> pick(0, n_centers - 1);
        std::normal_distribution<float> noise(0.0f, cluster_std);
#pragma omp for
        for (size_t i = 0; i < n_samples; ++i) {
            const float* center = centers.data() + pick(engine) * n_features;
            float* row = rows.data() + i * n_features;
            for (size_t j = 0; j < n_features; ++j) row[j] = center[j] + noise(engine);
        }
    }
    if (normalize) {
#pragma omp parallel for
        for (size_t i = 0; i < n_samples; ++i) {
            float* row = rows.data() + i * n_features;
            float sq = 0.0f;
            for (size_t j = 0; j < n_features; ++j) sq += row[j] * row[j];
            const float inv = 1.0f / std::sqrt(sq);
            for (size_t j = 0; j < n_features; ++j) row[j] *= inv;
        }
    }
    return rows;
}

/** n x d values uniform in [min_val, max_val) from mt19937(seed), row-major. */
inline std::vector<float> GenerateRandomVectors(size_t n, size_t d, float min_val = -1.0f, float max_val = 1.0f,
                                                uint32_t seed = 42) {
    std::vector<float> out(n * d);
    std::mt19937 engine(seed);
    std::uniform_real_distribution<float> uniform(min_val, max_val);
    for (float& v : out) v = uniform(engine);
    return out;
}

// ---- brute-force checkers (the reference uses them in its tests only) ----

inline float ComputeL2DistanceSquared(const float* a, const float* b, size_t d) {
    float sum = 0.0f;
    for (size_t j = 0; j < d; ++j) {
        const float t = a[j] - b[j];
        sum += t * t;
    }
    return sum;
}

inline std::vector<float> ComputeNorms(const float* data, size_t n, size_t d) {
    std::vector<float> norms(n);
#pragma omp parallel for
    for (size_t i = 0; i < n; ++i) {
        float sq = 0.0f;
        for (size_t j = 0; j < d; ++j) sq += data[i * d + j] * data[i * d + j];
        norms[i] = sq;
    }
    return norms;
}

/** Index of the row of `centroids` nearest to `point` (first one on ties). */
inline uint32_t FindNearestCentroidBruteForce(const float* point, const float* centroids, size_t n_clusters, size_t d) {
    uint32_t best = 0;
    float best_distance = std::numeric_limits<float>::max();
    for (size_t c = 0; c < n_clusters; ++c) {
        const float distance = ComputeL2DistanceSquared(point, centroids + c * d, d);
        if (distance < best_distance) {
            best_distance = distance;
            best = static_cast<uint32_t>(c);
        }
    }
    return best;
}

inline void FindNearestNeighborBruteForce(const float* x, const float* y, size_t n_x, size_t n_y, size_t d,
                                          uint32_t* out_knn, float* out_distances) {
    for (size_t i = 0; i < n_x; ++i) {
        const uint32_t best = FindNearestCentroidBruteForce(x + i * d, y, n_y, d);
        out_knn[i] = best;
        out_distances[i] = n_y ? ComputeL2DistanceSquared(x + i * d, y + best * d, d) : std::numeric_limits<float>::max();
    }
}

/** The k rows of y nearest to every row of x, ascending by (distance, index); slots past n_y stay untouched. */
inline void FindKNearestNeighborsBruteForce(const float* x, const float* y, size_t n_x, size_t n_y, size_t d, size_t k,
                                            uint32_t* out_knn, float* out_distances) {
    std::vector<std::pair<float, uint32_t>> all(n_y);
    const size_t keep = std::min(k, n_y);
    for (size_t i = 0; i < n_x; ++i) {
#pragma omp parallel for
        for (size_t j = 0; j < n_y; ++j)
            all[j] = {ComputeL2DistanceSquared(x + i * d, y + j * d, d), static_cast<uint32_t>(j)};
        std::partial_sort(all.begin(), all.begin() + keep, all.end());
        for (size_t r = 0; r < keep; ++r) {
            out_knn[i * k + r] = all[r].second;
            out_distances[i * k + r] = all[r].first;
        }
    }
}

/** Values uniform in [-100, 100) and, per value, a mask that is 0x80000000 with probability flip_probability. */
inline void GenerateRandomDataWithMasks(float* data, uint32_t* masks, size_t n, float flip_probability = 0.5f,
                                        uint32_t seed = 42) {
    std::mt19937 engine(seed);
    std::uniform_real_distribution<float> value(-100.0f, 100.0f);
    std::uniform_real_distribution<float> flip(0.0f, 1.0f);
    for (size_t i = 0; i < n; ++i) {
        data[i] = value(engine);
        masks[i] = flip(engine) < flip_probability ? 0x80000000u : 0u;
    }
}

/** n distances of which floor(n * selectivity) lie below `threshold` and the rest above it, in shuffled order. */
inline void GenerateRandomDistances(float* pruning_distances, size_t n, float threshold, float selectivity = 0.03f,
                                    uint32_t seed = 42) {
    std::mt19937 engine(seed);
    const size_t below = static_cast<size_t>(static_cast<float>(n) * selectivity);
    std::uniform_real_distribution<float> low(0.0f, threshold * 0.99f);
    std::uniform_real_distribution<float> high(threshold * 1.01f, threshold * 10.0f);
    for (size_t i = 0; i < n; ++i) pruning_distances[i] = i < below ? low(engine) : high(engine);
    std::shuffle(pruning_distances, pruning_distances + n, engine);
}

} // namespace skmeans
