// CPU ORACLE -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A plain C++17 + OpenMP restatement of the Super K-Means assign/update path of the reference
// (cwida/SuperKMeans, include/superkmeans/...).  It exists to check the HIP path and to serve as
// the CPU baseline that is timed next to it.  Only tests/, __graft_entry__.smoke() and the
// cpu_baseline leg of bench.py may load it; nothing under superkmeans_amd/ or include/ does.
//
// The reference itself cannot be compiled here (every hot-path header includes <Eigen/Dense>, and
// the Eigen submodule directory of the checkout is empty), so each function below restates the
// reference routine it cites.  What pins each function (tests/test_oracle_*.py):
//   dimension_split      closed form + hand-derived table + properties of tests/test_pdx_layout.cpp:61-108
//   pdxify               closed-form element map of tests/test_pdx_layout.cpp:30-52 (independent formula)
//   ratios               closed form, spot values
//   rotation matrix      orthogonality / norm / inner-product / round-trip invariants of tests/test_rotation.cpp
//   find_nn              fp64 brute force, tolerance rule of tests/test_distance_computers.cpp:83-152
//   find_nn_pruned       equals brute force when every ratio is 1; invariants; >= 98 % agreement rule
//   update/consolidate   fp64 means, exact counts
//   split_clusters       hand-placed empty clusters, size conservation, perturbation factors
//   cost/shift/tune_d'   closed forms, table-driven
//   train                WCSS monotonicity, is_gemm_only rule, stats bookkeeping, exceptions
// PARITY UNPINNED (no reference test or fixture fixes them, and the reference cannot be built):
//   the numeric entries of the rotation matrix for a given seed (the reference takes them from
//   Eigen::HouseholderQR, pdx/adsampling.h:76-85) and therefore exact rotated coordinates, exact
//   not_pruned_pct / partial_d trajectories; the low-order bits of every sgemm_/Eigen reduction.
//
// Build: make -C oracle   (g++ -O3 -march=native -fopenmp; sgemm_ resolved at run time).
#include <dlfcn.h>
#include <omp.h>

#include <algorithm>
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <memory>
#include <numeric>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

namespace oracle {

// ---- constants: common.h:89-115 ----
static constexpr float PROPORTION_HORIZONTAL_DIM = 0.75;
static constexpr size_t H_DIM_SIZE = 64;
static constexpr uint32_t MIN_PARTIAL_D = 16;
static constexpr size_t DIMENSION_THRESHOLD_FOR_PRUNING = 128;
static constexpr size_t N_CLUSTERS_THRESHOLD_FOR_PRUNING = 256;
static constexpr size_t X_BATCH_SIZE = 4096;
static constexpr size_t Y_BATCH_SIZE = 1024;
static constexpr size_t VECTOR_CHUNK_SIZE = Y_BATCH_SIZE;
static constexpr size_t RECALL_CONVERGENCE_PATIENCE = 2;
static constexpr float CENTROID_PERTURBATION_EPS = 1.0f / 1024.0f;
static constexpr float PRUNER_INITIAL_THRESHOLD = 1.5f;
static constexpr float HIERARCHICAL_PRUNER_INITIAL_THRESHOLD = 1.1f;

static uint32_t g_n_threads = 1;  // common.h:120

// ---- BLAS: the reference links sgemm_ (common.h:7-23); here it is looked up at run time ----
typedef int (*sgemm_fn)(const char*, const char*, int*, int*, int*, const float*, const float*, int*,
                        const float*, int*, float*, float*, int*);
static sgemm_fn g_sgemm = nullptr;
static std::string g_blas_name = "internal";

static void internal_sgemm_tn_or_nn(char ta, int m, int n, int k, const float* a, int lda, const float* b,
                                    int ldb, float* c, int ldc) {
    // Column-major C(m x n) = op(A) * B with op = T or N; B is never transposed on this path.
    // For 'T': C[i + j*ldc] = sum_p A[p + i*lda] * B[p + j*ldb]  (dot of two contiguous vectors).
    if (ta == 'T') {
#pragma omp parallel for num_threads(g_n_threads) schedule(static)
        for (int j = 0; j < n; ++j) {
            const float* bj = b + (size_t) j * ldb;
            for (int i = 0; i < m; ++i) {
                const float* ai = a + (size_t) i * lda;
                float s0 = 0, s1 = 0, s2 = 0, s3 = 0;
                int p = 0;
                for (; p + 3 < k; p += 4) {
                    s0 += ai[p] * bj[p];
                    s1 += ai[p + 1] * bj[p + 1];
                    s2 += ai[p + 2] * bj[p + 2];
                    s3 += ai[p + 3] * bj[p + 3];
                }
                for (; p < k; ++p) s0 += ai[p] * bj[p];
                c[i + (size_t) j * ldc] = (s0 + s1) + (s2 + s3);
            }
        }
    } else {
#pragma omp parallel for num_threads(g_n_threads) schedule(static)
        for (int j = 0; j < n; ++j) {
            float* cj = c + (size_t) j * ldc;
            for (int i = 0; i < m; ++i) cj[i] = 0.0f;
            for (int p = 0; p < k; ++p) {
                const float bpj = b[p + (size_t) j * ldb];
                const float* ap = a + (size_t) p * lda;
                for (int i = 0; i < m; ++i) cj[i] += ap[i] * bpj;
            }
        }
    }
}

static void sgemm(char ta, char tb, int m, int n, int k, const float* a, int lda, const float* b, int ldb,
                  float* c, int ldc) {
    if (g_sgemm) {
        float alpha = 1.0f, beta = 0.0f;
        g_sgemm(&ta, &tb, &m, &n, &k, &alpha, a, &lda, b, &ldb, &beta, c, &ldc);
    } else {
        internal_sgemm_tn_or_nn(ta, m, n, k, a, lda, b, ldb, c, ldc);
    }
}

// ---- pdx/layout.h:115-140 ----
struct DimSplit {
    size_t horizontal_d, vertical_d;
};
static DimSplit GetDimensionSplit(const size_t d) {
    auto local_proportion_horizontal_dim = PROPORTION_HORIZONTAL_DIM;
    if (d <= 256) local_proportion_horizontal_dim = 0.25;
    size_t horizontal_d = static_cast<size_t>(static_cast<double>(d) * local_proportion_horizontal_dim);
    size_t vertical_d = d - horizontal_d;
    if (horizontal_d % H_DIM_SIZE > 0) {
        horizontal_d = static_cast<size_t>(std::lround(
                           static_cast<double>(horizontal_d) / static_cast<double>(H_DIM_SIZE))) *
                       H_DIM_SIZE;
        vertical_d = d - horizontal_d;
    }
    if (!vertical_d) {
        horizontal_d = H_DIM_SIZE;
        vertical_d = d - horizontal_d;
    }
    if (d <= H_DIM_SIZE) {
        horizontal_d = 0;
        vertical_d = d;
    }
    return {horizontal_d, vertical_d};
}

// ---- pdx/layout.h:155-232 (PDXify<false>): transposes written as explicit loops ----
static void PDXify(const float* in, float* out, const size_t n, const size_t d) {
    auto [horizontal_d, vertical_d] = GetDimensionSplit(d);
    const size_t full_chunks = n / VECTOR_CHUNK_SIZE;
    const size_t n_remaining = n % VECTOR_CHUNK_SIZE;
    const size_t n_chunks = full_chunks + (n_remaining ? 1 : 0);
    for (size_t i = 0; i < n_chunks; ++i) {
        const size_t rows = (i < full_chunks) ? VECTOR_CHUNK_SIZE : n_remaining;
        const size_t chunk_offset = (i * VECTOR_CHUNK_SIZE) * d;
        const float* chunk_p = in + chunk_offset;
        float* out_chunk_p = out + chunk_offset;
        // vertical block: out(vertical_d x rows) = in.leftCols(vertical_d)^T
        for (size_t dim = 0; dim < vertical_d; ++dim)
            for (size_t r = 0; r < rows; ++r) out_chunk_p[dim * rows + r] = chunk_p[r * d + dim];
        out_chunk_p += rows * vertical_d;
        // horizontal blocks: rows x 64 row-major copies
        for (size_t j = 0; j < horizontal_d; j += H_DIM_SIZE) {
            for (size_t r = 0; r < rows; ++r)
                std::memcpy(out_chunk_p + r * H_DIM_SIZE, chunk_p + r * d + vertical_d + j,
                            H_DIM_SIZE * sizeof(float));
            out_chunk_p += rows * H_DIM_SIZE;
        }
    }
}

// ---- scalar_computers.h:20-32 ----
static inline float Horizontal(const float* v1, const float* v2, size_t num_dimensions) {
    float distance = 0.0;
    // SKM_VECTORIZE_LOOP in the reference; its x86/ARM builds use the SIMD variants of this loop
    // (avx2_computers.h:35-80, avx512_computers.h:80-111), so the reduction is vectorised here too.
#pragma omp simd reduction(+ : distance)
    for (size_t i = 0; i < num_dimensions; ++i) {
        float to_multiply = v1[i] - v2[i];
        distance += to_multiply * to_multiply;
    }
    return distance;
}

// ---- pdx/adsampling.h: pruner.  Dense-matrix variant and, on request, the FFTW/DCT variant ----
// FFTW is not available, so the DCT branch (adsampling.h:60-71,162-189,229-271) is restated from the
// definitions of the transforms FFTW documents: REDFT10 Y_k = 2 sum_j X_j cos(pi (j + 1/2) k / n) and
// REDFT01 Y_k = X_0 + 2 sum_{j>=1} X_j cos(pi j (k + 1/2) / n), evaluated directly in double (O(d^2) per
// vector), with the reference's sign flip and scale factors around them.  PARITY UNPINNED at the level of
// FFTW's fp32 butterflies; pinned against scipy.fft.dct(norm="ortho") in the tests.
// The rotation matrix is the Q factor of a Householder QR of a d x d matrix of N(0,1) draws
// (adsampling.h:76-85).  Eigen is unavailable, so the factorisation is a textbook Householder QR in
// double precision; the value sequence of the draws (std::mt19937 + std::normal_distribution<float>,
// row by row) is the reference's.
// Implemented in rotation_matrix.cpp, which is compiled with -ffp-contract=off so that the draws and
// the factorisation give the same bits under every compiler.
void MakeRotationMatrix(uint32_t d, uint32_t seed, std::vector<float>& out);

class ADSamplingPruner {
  public:
    uint32_t num_dimensions;
    std::vector<float> ratios;
    std::vector<float> matrix;  // d x d row-major

    bool use_dct = false;
    std::vector<float> flip;      // +1 / -1 per dimension (adsampling.h:60-70)
    std::vector<double> cos_tab;  // cos(pi (j + 1/2) k / d) at [k * d + j]

    // rotation_kind: 0 dense, 1 DCT when d >= 512 and a power of two (HAS_FFTW && __AVX2__), 2 DCT when
    // d >= 512 (HAS_FFTW otherwise); adsampling.h:52-59.
    ADSamplingPruner(uint32_t num_dimensions_, float epsilon0_, uint32_t seed = 42, int rotation_kind = 0)
        : num_dimensions(num_dimensions_), epsilon0(epsilon0_) {
        InitializeRatios();
        const size_t d = num_dimensions;
        const bool pow2 = (d & (d - 1)) == 0;
        use_dct = rotation_kind != 0 && d >= 512 && (rotation_kind == 2 || pow2);
        if (!use_dct) {
            MakeRotationMatrix(num_dimensions, seed, matrix);
            return;
        }
        std::mt19937 gen(seed);
        std::uniform_int_distribution<int> dist(0, 1);
        flip.resize(d);
        for (size_t i = 0; i < d; ++i) flip[i] = dist(gen) ? 1.0f : -1.0f;
        cos_tab.resize(d * d);
        const double pi = 3.14159265358979323846;
        for (size_t k = 0; k < d; ++k)
            for (size_t j = 0; j < d; ++j)
                cos_tab[k * d + j] = std::cos(pi * (static_cast<double>(j) + 0.5) * static_cast<double>(k) /
                                              static_cast<double>(d));
        // The explicit matrix, for callers that ask for it: row k = image of nothing, column j = R e_j.
        matrix.resize(d * d);
        std::vector<float> e(d, 0.0f), col(d);
        for (size_t j = 0; j < d; ++j) {
            e[j] = 1.0f;
            RotateDct(e.data(), col.data(), 1);
            e[j] = 0.0f;
            for (size_t k = 0; k < d; ++k) matrix[k * d + j] = col[k];
        }
    }

    // adsampling.h:162-189: FlipSign, REDFT10 in place, column 0 scaled by sqrt(1/(4d)), the rest by sqrt(1/(2d)).
    void RotateDct(const float* vectors, float* out_buffer, const uint32_t n) const {
        const size_t d = num_dimensions;
        const float s0 = std::sqrt(1.0f / (4.0f * num_dimensions));
        const float s = std::sqrt(1.0f / (2.0f * num_dimensions));
#pragma omp parallel for num_threads(g_n_threads)
        for (size_t i = 0; i < (size_t) n; ++i) {
            std::vector<float> x(d);
            for (size_t j = 0; j < d; ++j) x[j] = vectors[i * d + j] * flip[j];
            for (size_t k = 0; k < d; ++k) {
                double acc = 0.0;
                const double* c = &cos_tab[k * d];
                for (size_t j = 0; j < d; ++j) acc += static_cast<double>(x[j]) * c[j];
                const float y = static_cast<float>(2.0 * acc);
                out_buffer[i * d + k] = y * (k == 0 ? s0 : s);
            }
        }
    }

    // adsampling.h:229-271: undo the scaling, REDFT01, times 1/(2d), FlipSign.
    void UnrotateDct(const float* rotated, float* out_buffer, const uint32_t n) const {
        const size_t d = num_dimensions;
        const float inv_s0 = std::sqrt(4.0f * num_dimensions);
        const float inv_s = std::sqrt(2.0f * num_dimensions);
        const float norm = 1.0f / (2.0f * num_dimensions);
#pragma omp parallel for num_threads(g_n_threads)
        for (size_t i = 0; i < (size_t) n; ++i) {
            std::vector<float> x(d);
            for (size_t j = 0; j < d; ++j) x[j] = rotated[i * d + j] * (j == 0 ? inv_s0 : inv_s);
            for (size_t k = 0; k < d; ++k) {
                double acc = 0.0;
                // cos(pi j (k + 1/2) / d) is the transposed entry of the forward table
                for (size_t j = 1; j < d; ++j) acc += static_cast<double>(x[j]) * cos_tab[j * d + k];
                const float y = static_cast<float>(static_cast<double>(x[0]) + 2.0 * acc);
                out_buffer[i * d + k] = (y * norm) * flip[k];
            }
        }
    }

    // adsampling.h:93-99
    void InitializeRatios() {
        ratios.resize(num_dimensions + 1);
        for (size_t i = 0; i < num_dimensions + 1; ++i) ratios[i] = GetRatio(i);
    }

    // adsampling.h:156-216 (dense branch): out = vectors * matrix^T
    void Rotate(const float* vectors, float* out_buffer, const uint32_t n) const {
        if (use_dct) return RotateDct(vectors, out_buffer, n);
        sgemm('T', 'N', (int) num_dimensions, (int) n, (int) num_dimensions, matrix.data(), (int) num_dimensions,
              vectors, (int) num_dimensions, out_buffer, (int) num_dimensions);
    }
    // adsampling.h:223-299 (dense branch): out = rotated * matrix
    void Unrotate(const float* rotated, float* out_buffer, const uint32_t n) const {
        if (use_dct) return UnrotateDct(rotated, out_buffer, n);
        sgemm('N', 'N', (int) num_dimensions, (int) n, (int) num_dimensions, matrix.data(), (int) num_dimensions,
              rotated, (int) num_dimensions, out_buffer, (int) num_dimensions);
    }

    // adsampling.h:315-327
    float GetRatio(const size_t visited_dimensions) const {
        if (visited_dimensions == 0) return 1.0;
        if (visited_dimensions == num_dimensions) return 1.0;
        return static_cast<float>(
            static_cast<double>(visited_dimensions) / static_cast<double>(num_dimensions) *
            (1.0 + epsilon0 / std::sqrt(static_cast<double>(visited_dimensions))) *
            (1.0 + epsilon0 / std::sqrt(static_cast<double>(visited_dimensions))));
    }

  private:
    float epsilon0;
};

// ---- pdx_ivf.h:16-26, common.h:187-195, layout.h:67-106 ----
struct Cluster {
    uint32_t num_embeddings = 0;
    uint32_t first_index = 0;  // indices are an iota (layout.h:80-81), so only the start is kept
    const float* data = nullptr;
    const float* aux_vertical_dimensions_in_horizontal_layout = nullptr;
};

struct PDXIndex {
    uint32_t num_dimensions = 0, num_horizontal_dimensions = 0, num_vertical_dimensions = 0;
    std::vector<Cluster> clusters;
    const float* ratios = nullptr;

    void FromBuffer(const float* pdx_data, size_t n_points, size_t d, const float* hor_data, const float* ratios_) {
        auto [horizontal_d, vertical_d] = GetDimensionSplit(d);
        const size_t full_clusters = n_points / VECTOR_CHUNK_SIZE;
        const size_t n_remaining = n_points % VECTOR_CHUNK_SIZE;
        num_dimensions = d;
        num_horizontal_dimensions = horizontal_d;
        num_vertical_dimensions = vertical_d;
        ratios = ratios_;
        clusters.assign(full_clusters + (n_remaining ? 1 : 0), Cluster{});
        const float* pdx_p = pdx_data;
        const float* hor_p = hor_data;
        size_t ci = 0;
        for (; ci < full_clusters; ++ci) {
            clusters[ci].num_embeddings = VECTOR_CHUNK_SIZE;
            clusters[ci].data = pdx_p;
            clusters[ci].first_index = ci * VECTOR_CHUNK_SIZE;
            clusters[ci].aux_vertical_dimensions_in_horizontal_layout = hor_p;
            hor_p += VECTOR_CHUNK_SIZE * vertical_d;
            pdx_p += VECTOR_CHUNK_SIZE * d;
        }
        if (n_remaining) {
            clusters[ci].num_embeddings = n_remaining;
            clusters[ci].data = pdx_p;
            clusters[ci].first_index = ci * VECTOR_CHUNK_SIZE;
            clusters[ci].aux_vertical_dimensions_in_horizontal_layout = hor_p;
        }
    }
};

struct KNNCandidate {
    uint32_t index;
    float distance;
};

// Optional accounting of the pairs entering each pruning step (not in the reference; used to state
// the algorithmic bytes of the pruning stage).  stage 0 = survivors of the first test, stage s>=1 =
// pairs entering the s-th horizontal block, last = pairs entering the [d', V) step.
struct PruneAccounting {
    std::vector<uint64_t> pairs;
};

// ---- pdx/pdxearch.h:118-217 ----
static void Prune(const PDXIndex& pdx, const float* query, const float* data, const size_t n_vectors,
                  uint32_t* pruning_positions, float* pruning_distances, float& pruning_threshold,
                  const KNNCandidate& best_candidate, size_t& n_vectors_not_pruned, uint32_t& current_dimension_idx,
                  const uint32_t first_index, const uint32_t prev_top_1, const float* aux, size_t& initial_not_pruned_out,
                  uint64_t* acct) {
    pruning_threshold = best_candidate.distance * pdx.ratios[current_dimension_idx];
    // scalar_computers.h:87-98 InitPositionsArray
    n_vectors_not_pruned = 0;
    for (size_t v = 0; v < n_vectors; ++v) {
        pruning_positions[n_vectors_not_pruned] = v;
        n_vectors_not_pruned += pruning_distances[v] < pruning_threshold;
    }
    initial_not_pruned_out = n_vectors_not_pruned;
    if (acct) acct[0] += n_vectors_not_pruned;
    if (n_vectors_not_pruned == 1 && first_index + pruning_positions[0] == prev_top_1) {
        n_vectors_not_pruned = 0;
        return;
    }
    size_t cur_n_vectors_not_pruned = 0;
    size_t current_vertical_dimension = current_dimension_idx;
    size_t current_horizontal_dimension = 0;
    size_t stage = 1;
    while (pdx.num_horizontal_dimensions && n_vectors_not_pruned &&
           current_horizontal_dimension < pdx.num_horizontal_dimensions) {
        cur_n_vectors_not_pruned = n_vectors_not_pruned;
        if (acct) acct[stage] += n_vectors_not_pruned;
        ++stage;
        size_t offset_data = (pdx.num_vertical_dimensions * n_vectors) + (current_horizontal_dimension * n_vectors);
        size_t offset_query = pdx.num_vertical_dimensions + current_horizontal_dimension;
        for (size_t vector_idx = 0; vector_idx < n_vectors_not_pruned; vector_idx++) {
            size_t v_idx = pruning_positions[vector_idx];
            size_t data_pos = offset_data + (v_idx * H_DIM_SIZE);
            pruning_distances[v_idx] += Horizontal(query + offset_query, data + data_pos, H_DIM_SIZE);
        }
        current_horizontal_dimension += H_DIM_SIZE;
        current_dimension_idx += H_DIM_SIZE;
        pruning_threshold = best_candidate.distance * pdx.ratios[current_dimension_idx];
        // pdxearch.h:67-80 EvaluatePruningPredicateOnPositionsArray
        n_vectors_not_pruned = 0;
        for (size_t vector_idx = 0; vector_idx < cur_n_vectors_not_pruned; ++vector_idx) {
            pruning_positions[n_vectors_not_pruned] = pruning_positions[vector_idx];
            n_vectors_not_pruned += pruning_distances[pruning_positions[vector_idx]] < pruning_threshold;
        }
    }
    if (n_vectors_not_pruned && current_vertical_dimension < pdx.num_vertical_dimensions) {
        cur_n_vectors_not_pruned = n_vectors_not_pruned;
        if (acct) acct[pdx.num_horizontal_dimensions / H_DIM_SIZE + 1] += n_vectors_not_pruned;
        size_t dimensions_left = pdx.num_vertical_dimensions - current_vertical_dimension;
        size_t offset_query = current_vertical_dimension;
        for (size_t vector_idx = 0; vector_idx < n_vectors_not_pruned; vector_idx++) {
            size_t v_idx = pruning_positions[vector_idx];
            auto data_pos = aux + (v_idx * pdx.num_vertical_dimensions) + current_vertical_dimension;
            pruning_distances[v_idx] += Horizontal(query + offset_query, data_pos, dimensions_left);
        }
        current_dimension_idx = pdx.num_dimensions;
        pruning_threshold = best_candidate.distance * pdx.ratios[current_dimension_idx];
        n_vectors_not_pruned = 0;
        for (size_t vector_idx = 0; vector_idx < cur_n_vectors_not_pruned; ++vector_idx) {
            pruning_positions[n_vectors_not_pruned] = pruning_positions[vector_idx];
            n_vectors_not_pruned += pruning_distances[pruning_positions[vector_idx]] < pruning_threshold;
        }
    }
}

// ---- pdx/pdxearch.h:266-327 (+ SetBestCandidate :223-238) ----
static KNNCandidate Top1PartialSearchWithThresholdAndPartialDistances(
    const PDXIndex& pdx, const float* query, const float prev_pruning_threshold, const uint32_t prev_top_1,
    float* partial_pruning_distances, const uint32_t computed_distance_until, const size_t start_cluster,
    const size_t end_cluster, size_t& initial_not_pruned_accum, uint64_t* acct) {
    alignas(64) thread_local uint32_t pruning_positions[VECTOR_CHUNK_SIZE];
    float pruning_threshold = prev_pruning_threshold;
    size_t n_vectors_not_pruned = 0;
    KNNCandidate top_embedding{prev_top_1, prev_pruning_threshold};
    size_t data_offset = 0;
    for (size_t cluster_idx = start_cluster; cluster_idx < end_cluster; ++cluster_idx) {
        uint32_t current_dimension_idx = computed_distance_until;
        float* pruning_distances = partial_pruning_distances + data_offset;
        const Cluster& cluster = pdx.clusters[cluster_idx];
        data_offset += cluster.num_embeddings;
        size_t initial_not_pruned = 0;
        Prune(pdx, query, cluster.data, cluster.num_embeddings, pruning_positions, pruning_distances,
              pruning_threshold, top_embedding, n_vectors_not_pruned, current_dimension_idx, cluster.first_index,
              prev_top_1, cluster.aux_vertical_dimensions_in_horizontal_layout, initial_not_pruned, acct);
        initial_not_pruned_accum += initial_not_pruned;
        if (n_vectors_not_pruned) {
            for (size_t position_idx = 0; position_idx < n_vectors_not_pruned; ++position_idx) {
                size_t index = pruning_positions[position_idx];
                float current_distance = pruning_distances[index];
                if (current_distance < top_embedding.distance) {
                    top_embedding.distance = current_distance;
                    top_embedding.index = cluster.first_index + index;
                }
            }
        }
    }
    return top_embedding;
}

// ---- batch_computers.h:47-83 ----
static void BlasMatrixMultiplication(const float* batch_x_p, const float* batch_y_p, const size_t batch_n_x,
                                     const size_t batch_n_y, const size_t d, const size_t partial_d,
                                     float* tmp_distances_buf) {
    int k = static_cast<int>(partial_d > 0 && partial_d < d ? partial_d : d);
    sgemm('T', 'N', (int) batch_n_y, (int) batch_n_x, k, batch_y_p, (int) d, batch_x_p, (int) d, tmp_distances_buf,
          (int) batch_n_y);
}

// ---- batch_computers.h:104-171 ----
static void FindNearestNeighbor(const float* x, const float* y, const size_t n_x, const size_t n_y, const size_t d,
                                const float* norms_x, const float* norms_y, uint32_t* out_knn, float* out_distances,
                                float* tmp_distances_buf) {
    std::fill_n(out_distances, n_x, std::numeric_limits<float>::max());
    for (size_t i = 0; i < n_x; i += X_BATCH_SIZE) {
        auto batch_n_x = X_BATCH_SIZE;
        auto batch_x_p = x + (i * d);
        if (i + X_BATCH_SIZE > n_x) batch_n_x = n_x - i;
        for (size_t j = 0; j < n_y; j += Y_BATCH_SIZE) {
            auto batch_n_y = Y_BATCH_SIZE;
            auto batch_y_p = y + (j * d);
            if (j + Y_BATCH_SIZE > n_y) batch_n_y = n_y - j;
            BlasMatrixMultiplication(batch_x_p, batch_y_p, batch_n_x, batch_n_y, d, 0, tmp_distances_buf);
#pragma omp parallel for num_threads(g_n_threads)
            for (size_t r = 0; r < batch_n_x; ++r) {
                const auto i_idx = i + r;
                const float norm_x_i = norms_x[i_idx];
                float* row_p = tmp_distances_buf + r * batch_n_y;
                for (size_t c = 0; c < batch_n_y; ++c) row_p[c] = -2.0f * row_p[c] + norm_x_i + norms_y[j + c];
                // Eigen minCoeff(&idx): first minimum
                uint32_t knn_idx = 0;
                float batch_top_1 = row_p[0];
                for (size_t c = 1; c < batch_n_y; ++c) {
                    if (row_p[c] < batch_top_1) {
                        batch_top_1 = row_p[c];
                        knn_idx = c;
                    }
                }
                if (batch_top_1 < out_distances[i_idx]) {
                    out_distances[i_idx] = std::max(0.0f, batch_top_1);
                    out_knn[i_idx] = j + knn_idx;
                }
            }
        }
    }
}

// ---- batch_computers.h:191-274 ----
static void FindKNearestNeighbors(const float* x, const float* y, const size_t n_x, const size_t n_y, const size_t d,
                                  const float* norms_x, const float* norms_y, const size_t k, uint32_t* out_knn,
                                  float* out_distances, float* tmp_distances_buf) {
    std::fill_n(out_distances, n_x * k, std::numeric_limits<float>::max());
    std::fill_n(out_knn, n_x * k, static_cast<uint32_t>(-1));
    const size_t max_candidates = k + Y_BATCH_SIZE;
    std::vector<std::vector<std::pair<float, uint32_t>>> thread_candidates(g_n_threads);
    for (auto& tc : thread_candidates) tc.reserve(max_candidates);
    for (size_t i = 0; i < n_x; i += X_BATCH_SIZE) {
        auto batch_n_x = X_BATCH_SIZE;
        auto batch_x_p = x + (i * d);
        if (i + X_BATCH_SIZE > n_x) batch_n_x = n_x - i;
        for (size_t j = 0; j < n_y; j += Y_BATCH_SIZE) {
            auto batch_n_y = Y_BATCH_SIZE;
            auto batch_y_p = y + (j * d);
            if (j + Y_BATCH_SIZE > n_y) batch_n_y = n_y - j;
            BlasMatrixMultiplication(batch_x_p, batch_y_p, batch_n_x, batch_n_y, d, 0, tmp_distances_buf);
#pragma omp parallel for num_threads(g_n_threads)
            for (size_t r = 0; r < batch_n_x; ++r) {
                const auto i_idx = i + r;
                const float norm_x_i = norms_x[i_idx];
                float* row_p = tmp_distances_buf + r * batch_n_y;
                for (size_t c = 0; c < batch_n_y; ++c) row_p[c] = -2.0f * row_p[c] + norm_x_i + norms_y[j + c];
                auto& candidates = thread_candidates[omp_get_thread_num()];
                candidates.clear();
                for (size_t ki = 0; ki < k; ++ki)
                    if (out_distances[i_idx * k + ki] < std::numeric_limits<float>::max())
                        candidates.emplace_back(out_distances[i_idx * k + ki], out_knn[i_idx * k + ki]);
                for (size_t c = 0; c < batch_n_y; ++c) candidates.emplace_back(row_p[c], static_cast<uint32_t>(j + c));
                size_t actual_k = std::min(k, candidates.size());
                std::partial_sort(candidates.begin(), candidates.begin() + actual_k, candidates.end());
                for (size_t ki = 0; ki < actual_k; ++ki) {
                    out_distances[i_idx * k + ki] = std::max(0.0f, candidates[ki].first);
                    out_knn[i_idx * k + ki] = candidates[ki].second;
                }
                for (size_t ki = actual_k; ki < k; ++ki) {
                    out_distances[i_idx * k + ki] = std::numeric_limits<float>::max();
                    out_knn[i_idx * k + ki] = static_cast<uint32_t>(-1);
                }
            }
        }
    }
}

// ---- superkmeans.h:1059-1086: recall@objective_k from the ground-truth and promising-centroid lists ----
static float RecallFromLists(const uint32_t* gt_assignments, const uint32_t* promising_centroids,
                             const uint32_t* assignments, const size_t n_queries, const size_t objective_k,
                             const size_t centroids_to_explore) {
    float sum_recall = 0.0f;
    for (size_t i = 0; i < n_queries; ++i) {
        size_t found_in_query = 0;
        for (size_t j = 0; j < objective_k; ++j) {
            uint32_t gt = gt_assignments[i * objective_k + j];
            bool found = false;
            for (size_t t = 0; t < centroids_to_explore; ++t) {
                if (promising_centroids[i * centroids_to_explore + t] == assignments[gt]) {
                    found = true;
                    break;
                }
            }
            if (found) ++found_in_query;
        }
        sum_recall += static_cast<float>(found_in_query) / static_cast<float>(objective_k);
    }
    return sum_recall / static_cast<float>(n_queries);
}

// ---- batch_computers.h:297-409 ----
static void FindNearestNeighborWithPruning(const float* x, const float* y, const size_t n_x, const size_t n_y,
                                           const size_t d, const float* norms_x, const float* norms_y,
                                           uint32_t* out_knn, float* out_distances, float* tmp_distances_buf,
                                           const PDXIndex& pdx_centroids, uint32_t partial_d,
                                           size_t* out_not_pruned_counts, PruneAccounting* acct) {
    const size_t n_stages = pdx_centroids.num_horizontal_dimensions / H_DIM_SIZE + 2;
    std::vector<std::vector<uint64_t>> tacct;
    if (acct) {
        acct->pairs.assign(n_stages, 0);
        tacct.assign(g_n_threads, std::vector<uint64_t>(n_stages, 0));
    }
    for (size_t i = 0; i < n_x; i += X_BATCH_SIZE) {
        auto batch_n_x = X_BATCH_SIZE;
        auto batch_x_p = x + (i * d);
        if (i + X_BATCH_SIZE > n_x) batch_n_x = n_x - i;
        for (size_t j = 0; j < n_y; j += Y_BATCH_SIZE) {
            auto batch_n_y = Y_BATCH_SIZE;
            auto batch_y_p = y + (j * d);
            if (j + Y_BATCH_SIZE > n_y) batch_n_y = n_y - j;
            BlasMatrixMultiplication(batch_x_p, batch_y_p, batch_n_x, batch_n_y, d, partial_d, tmp_distances_buf);
#pragma omp parallel for num_threads(g_n_threads) schedule(dynamic, 8)
            for (size_t r = 0; r < batch_n_x; ++r) {
                const auto i_idx = i + r;
                const float norm_x_i = norms_x[i_idx];
                float* row_p = tmp_distances_buf + r * batch_n_y;
                for (size_t c = 0; c < batch_n_y; ++c) row_p[c] = -2.0f * row_p[c] + norm_x_i + norms_y[j + c];
                auto data_p = x + (i_idx * d);
                const auto prev_assignment = out_knn[i_idx];
                float dist_to_prev_centroid;
                if (j == 0) {
                    dist_to_prev_centroid = Horizontal(y + (prev_assignment * d), data_p, d);
                } else {
                    dist_to_prev_centroid = out_distances[i_idx];
                }
                size_t local_not_pruned = 0;
                KNNCandidate assignment = Top1PartialSearchWithThresholdAndPartialDistances(
                    pdx_centroids, data_p, dist_to_prev_centroid, prev_assignment, row_p, partial_d,
                    j / VECTOR_CHUNK_SIZE, (j + Y_BATCH_SIZE) / VECTOR_CHUNK_SIZE, local_not_pruned,
                    acct ? tacct[omp_get_thread_num()].data() : nullptr);
                out_not_pruned_counts[i_idx] += local_not_pruned;
                out_knn[i_idx] = assignment.index;
                out_distances[i_idx] = assignment.distance;
            }
        }
    }
    if (acct)
        for (auto& t : tacct)
            for (size_t s = 0; s < n_stages; ++s) acct->pairs[s] += t[s];
}

// ---- pdx/utils.h:198-224, in fp64 so that it is an exact arbiter ----
static void BruteForce(const float* x, const float* y, size_t n_x, size_t n_y, size_t d, uint32_t* out_knn,
                       double* out_distances, double* out_second) {
#pragma omp parallel for num_threads(g_n_threads)
    for (size_t i = 0; i < n_x; ++i) {
        double best = std::numeric_limits<double>::max(), second = std::numeric_limits<double>::max();
        uint32_t best_idx = 0;
        for (size_t j = 0; j < n_y; ++j) {
            double dist = 0.0;
            for (size_t k = 0; k < d; ++k) {
                double diff = (double) x[i * d + k] - (double) y[j * d + k];
                dist += diff * diff;
            }
            if (dist < best) {
                second = best;
                best = dist;
                best_idx = j;
            } else if (dist < second) {
                second = dist;
            }
        }
        out_knn[i] = best_idx;
        if (out_distances) out_distances[i] = best;
        if (out_second) out_second[i] = second;
    }
}

// =================================================================================================
// superkmeans.h / hierarchical_superkmeans.h
// =================================================================================================
struct Config {  // superkmeans.h:23-55 + hierarchical_superkmeans.h:11-17, C layout shared with Python
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
    int32_t dct_rotation;  // 0: build without FFTW; 1: HAS_FFTW && __AVX2__; 2: HAS_FFTW (adsampling.h:52-59)
};

struct IterationStats {  // superkmeans.h:60-72
    uint64_t iteration;
    float objective;
    float shift;
    uint64_t split;
    float recall;
    float not_pruned_pct;
    uint32_t partial_d;
    int32_t is_gemm_only;
    double objective_f64;  // oracle extra: the same WCSS accumulated in fp64
};

#define ENSURE_POSITIVE(x)                                                                         \
    if ((x) <= 0) {                                                                                \
        throw std::invalid_argument("Value must be positive: " #x);                                \
    }

class KMeans {
  public:
    KMeans(size_t n_clusters_, size_t dimensionality, const Config& config_, bool hierarchical_)
        : d(dimensionality), n_clusters(n_clusters_), config(config_), hierarchical(hierarchical_) {
        // superkmeans.h:123-140
        ENSURE_POSITIVE(n_clusters);
        ENSURE_POSITIVE(dimensionality);
        ENSURE_POSITIVE(config.iters);
        ENSURE_POSITIVE(config.sampling_fraction);
        if (config.sampling_fraction > 1.0) throw std::invalid_argument("sampling_fraction must be <= 1.0");
        n_threads = (config.n_threads == 0) ? omp_get_max_threads() : config.n_threads;
        g_n_threads = n_threads;
        if (hierarchical) {
            // hierarchical_superkmeans.h:48-65
            pruner = std::make_unique<ADSamplingPruner>(dimensionality, HIERARCHICAL_PRUNER_INITIAL_THRESHOLD, config.seed,
                                                        config.dct_rotation);
            ENSURE_POSITIVE(config.iters_mesoclustering);
            ENSURE_POSITIVE(config.iters_fineclustering);
            if (n_clusters <= 128 && !config.suppress_warnings)
                printf("WARNING: n_clusters <= 128 is not recommended for HierarchicalSuperKMeans. Consider using at least 128 clusters.\n");
        } else {
            pruner = std::make_unique<ADSamplingPruner>(dimensionality, PRUNER_INITIAL_THRESHOLD, config.seed,
                                                        config.dct_rotation);
        }
        if (config.data_already_rotated) config.unrotate_centroids = false;
    }

    std::vector<float> Train(const float* data, const size_t n, const float* queries, const size_t n_queries) {
        return hierarchical ? TrainHierarchical(data, n, queries, n_queries) : TrainFlat(data, n, queries, n_queries);
    }

    // superkmeans.h:162-332
    std::vector<float> TrainFlat(const float* data, const size_t n, const float* queries, const size_t n_queries) {
        ENSURE_POSITIVE(n);
        if (trained) throw std::runtime_error("The clustering has already been trained");
        iteration_stats.clear();
        if (n < n_clusters)
            throw std::runtime_error("The number of points should be at least as large as the number of clusters");
        if (n_queries > 0 && queries == nullptr && !config.sample_queries)
            throw std::invalid_argument("Queries must be provided if n_queries > 0 and sample_queries is false");
        const float* data_p = data;
        n_samples = GetNVectorsToSample(n, n_clusters);
        if (n_samples < n_clusters)
            throw std::runtime_error(
                "Not enough samples to train. Try increasing the sampling_fraction or max_points_per_cluster");
        centroids.reset(new float[n_clusters * d]);
        horizontal_centroids.reset(new float[n_clusters * d]);
        prev_centroids.reset(new float[n_clusters * d]);
        cluster_sizes.reset(new uint32_t[n_clusters]);
        assignments.reset(new uint32_t[n]);
        distances.reset(new float[n]);
        data_norms.reset(new float[n_samples]);
        centroid_norms.reset(new float[n_clusters]);
        std::vector<float> centroids_partial_norms(n_clusters);
        std::vector<size_t> not_pruned_counts(n_samples);
        std::vector<float> tmp_distances_buf(X_BATCH_SIZE * Y_BATCH_SIZE);
        vertical_d = GetDimensionSplit(d).vertical_d;
        partial_horizontal_centroids.reset(new float[n_clusters * vertical_d]);
        partial_d = std::max<uint32_t>(MIN_PARTIAL_D, vertical_d / 2);
        if (partial_d > vertical_d) partial_d = vertical_d;

        PDXIndex centroids_pdx_wrapper = GenerateCentroids(data_p, n_samples, n_clusters, !config.data_already_rotated);
        std::vector<float> data_samples_buffer;
        const float* data_to_cluster =
            SampleAndRotateVectors(data_p, data_samples_buffer, n, n_samples, !config.data_already_rotated);
        RotateOrCopy(horizontal_centroids.get(), prev_centroids.get(), n_clusters, !config.data_already_rotated);
        GetL2NormsRowMajor(data_to_cluster, n_samples, data_norms.get());
        GetL2NormsRowMajor(prev_centroids.get(), n_clusters, centroid_norms.get());

        std::vector<float> rotated_queries;
        if (n_queries) {
            centroids_to_explore = std::max<size_t>(static_cast<size_t>(n_clusters * config.ann_explore_fraction), 1);
            gt_assignments.reset(new uint32_t[n_queries * config.objective_k]);
            gt_distances.reset(new float[n_queries * config.objective_k]);
            tmp_distances_buffer.reset(new float[X_BATCH_SIZE * Y_BATCH_SIZE]);
            promising_centroids.reset(new uint32_t[n_queries * centroids_to_explore]);
            recall_distances.reset(new float[n_queries * centroids_to_explore]);
            query_norms.reset(new float[n_queries]);
            rotated_queries.resize(n_queries * d);
            if (config.sample_queries) {
                std::vector<float> tmp;
                const float* q = SampleAndRotateVectors(data_to_cluster, tmp, n_samples, n_queries, false);
                std::memcpy(rotated_queries.data(), q, sizeof(float) * n_queries * d);
            } else {
                RotateOrCopy(queries, rotated_queries.data(), n_queries, !config.data_already_rotated);
            }
            GetL2NormsRowMajor(rotated_queries.data(), n_queries, query_norms.get());
            GetGTAssignmentsAndDistances(data_to_cluster, rotated_queries.data(), n_queries);
        }

        bool always_gemm_only = d < DIMENSION_THRESHOLD_FOR_PRUNING || config.use_blas_only ||
                                n_clusters <= N_CLUSTERS_THRESHOLD_FOR_PRUNING;
        bool partial_norms_computed = false;
        float best_recall = 0.0f;
        size_t iters_without_improvement = 0;
        for (size_t iter_idx = 0; iter_idx < config.iters; ++iter_idx) {
            bool use_gemm_only = (iter_idx == 0) || always_gemm_only;
            if (!use_gemm_only && !partial_norms_computed) {
                GetPartialL2NormsRowMajor(data_to_cluster, n_samples, data_norms.get(), partial_d);
                partial_norms_computed = true;
            }
            RunIteration(use_gemm_only, data_to_cluster, tmp_distances_buf.data(), centroids_pdx_wrapper,
                         centroids_partial_norms, not_pruned_counts, rotated_queries.data(), n_queries, n_samples,
                         n_clusters, iter_idx, use_gemm_only ? (iter_idx == 0) : false, iteration_stats);
            if (config.early_termination &&
                ShouldStopEarly(n_queries > 0, best_recall, iters_without_improvement, iter_idx))
                break;
        }
        trained = true;
        return GetOutputCentroids(config.unrotate_centroids);
    }

    // superkmeans.h:346-382
    std::vector<uint32_t> Assign(const float* vectors, const float* centroids_in, const size_t n_vectors,
                                 const size_t n_centroids) {
        std::vector<uint32_t> result_assignments(n_vectors);
        std::unique_ptr<float[]> tmp_distances_buf(new float[X_BATCH_SIZE * Y_BATCH_SIZE]);
        std::vector<float> vector_norms(n_vectors);
        std::vector<float> centroid_norms_local(n_centroids);
        std::vector<float> result_distances(n_vectors);
        GetL2NormsRowMajor(vectors, n_vectors, vector_norms.data());
        GetL2NormsRowMajor(centroids_in, n_centroids, centroid_norms_local.data());
        FindNearestNeighbor(vectors, centroids_in, n_vectors, n_centroids, d, vector_norms.data(),
                            centroid_norms_local.data(), result_assignments.data(), result_distances.data(),
                            tmp_distances_buf.get());
        return result_assignments;
    }

    // superkmeans.h:397-564
    std::vector<uint32_t> AssignTrainingPoints(const float* vectors, const float* centroids_in, const size_t n_vectors,
                                               const size_t n_centroids) {
        if (!trained) throw std::runtime_error("AssignTrainingPoints requires SuperKMeans to be trained first");
        if (config.use_blas_only || d < DIMENSION_THRESHOLD_FOR_PRUNING ||
            n_clusters <= N_CLUSTERS_THRESHOLD_FOR_PRUNING) {
            if (!config.suppress_warnings)
                printf("WARNING: AssignTrainingPoints cannot use pruning, falling back to brute force Assign\n");
            return Assign(vectors, centroids_in, n_vectors, n_centroids);
        }
        std::vector<uint32_t> result_assignments(n_vectors);
        std::vector<float> tmp_distances_buf(X_BATCH_SIZE * Y_BATCH_SIZE);
        partial_d = std::max<uint32_t>(MIN_PARTIAL_D, vertical_d / 2);
        std::vector<size_t> not_pruned_counts(n_vectors, 0);
        std::vector<float> data_buffer;
        const float* data_p;
        if (config.data_already_rotated) {
            data_p = vectors;
        } else {
            data_buffer.resize(n_vectors * d);
            RotateOrCopy(vectors, data_buffer.data(), n_vectors, true);
            data_p = data_buffer.data();
        }
        GetPartialL2NormsRowMajor(horizontal_centroids.get(), n_centroids, centroid_norms.get(), partial_d);
        PDXIndex pdx_centroids;
        pdx_centroids.FromBuffer(centroids.get(), n_clusters, d, partial_horizontal_centroids.get(), pruner->ratios.data());
        if (config.sampling_fraction == 1.0f) {
            last_seeds.assign(assignments.get(), assignments.get() + n_vectors);
            GetPartialL2NormsRowMajor(data_p, n_vectors, data_norms.get(), partial_d);
            FindNearestNeighborWithPruning(data_p, horizontal_centroids.get(), n_vectors, n_clusters, d,
                                           data_norms.get(), centroid_norms.get(), assignments.get(), distances.get(),
                                           tmp_distances_buf.data(), pdx_centroids, partial_d,
                                           not_pruned_counts.data(), nullptr);
            std::memcpy(result_assignments.data(), assignments.get(), n_vectors * sizeof(uint32_t));
            return result_assignments;
        } else if (config.sampling_fraction > 0.8f) {
            size_t cur_vector_idx = 0;
            for (; cur_vector_idx < n_samples; ++cur_vector_idx)
                result_assignments[sampled_indices[cur_vector_idx]] = assignments[cur_vector_idx];
            std::mt19937 rng(config.seed + 1);
            std::discrete_distribution<uint32_t> cluster_dist(cluster_sizes.get(), cluster_sizes.get() + n_clusters);
            for (; cur_vector_idx < n_vectors; ++cur_vector_idx)
                result_assignments[sampled_indices[cur_vector_idx]] = cluster_dist(rng);
            last_seeds = result_assignments;
            data_norms.reset(new float[n_vectors]);
            GetPartialL2NormsRowMajor(data_p, n_vectors, data_norms.get(), partial_d);
            FindNearestNeighborWithPruning(data_p, horizontal_centroids.get(), n_vectors, n_clusters, d,
                                           data_norms.get(), centroid_norms.get(), result_assignments.data(),
                                           distances.get(), tmp_distances_buf.data(), pdx_centroids, partial_d,
                                           not_pruned_counts.data(), nullptr);
            return result_assignments;
        } else {
            Config tmp_config = DefaultConfig();
            tmp_config.iters = 10;
            tmp_config.sampling_fraction = 1.0f;
            tmp_config.use_blas_only = false;
            tmp_config.verbose = config.verbose;
            tmp_config.suppress_warnings = config.suppress_warnings;
            tmp_config.seed = config.seed;
            tmp_config.angular = config.angular;
            tmp_config.data_already_rotated = config.data_already_rotated;
            auto new_n_centroids = static_cast<size_t>(std::sqrt(n_centroids));
            KMeans tmp_kmeans(new_n_centroids, d, tmp_config, false);
            auto meso_centroids = tmp_kmeans.Train(centroids_in, n_centroids, nullptr, 0);
            auto meso_assignments = tmp_kmeans.Assign(vectors, meso_centroids.data(), n_vectors, new_n_centroids);
            auto centroids_to_meso = tmp_kmeans.Assign(centroids_in, meso_centroids.data(), n_centroids, new_n_centroids);
            g_n_threads = n_threads;  // the temporary object's constructor overwrote the global (superkmeans.h:132-133)
            std::vector<uint32_t> meso_to_original(new_n_centroids, 0);
            for (size_t c = 0; c < n_centroids; ++c) meso_to_original[centroids_to_meso[c]] = static_cast<uint32_t>(c);
            size_t cur_vector_idx = 0;
            for (; cur_vector_idx < n_samples; ++cur_vector_idx)
                result_assignments[sampled_indices[cur_vector_idx]] = assignments[cur_vector_idx];
            for (; cur_vector_idx < n_vectors; ++cur_vector_idx) {
                size_t orig_idx = sampled_indices[cur_vector_idx];
                result_assignments[orig_idx] = meso_to_original[meso_assignments[orig_idx]];
            }
            last_seeds = result_assignments;
            data_norms.reset(new float[n_vectors]);
            GetPartialL2NormsRowMajor(data_p, n_vectors, data_norms.get(), partial_d);
            FindNearestNeighborWithPruning(data_p, horizontal_centroids.get(), n_vectors, n_clusters, d,
                                           data_norms.get(), centroid_norms.get(), result_assignments.data(),
                                           distances.get(), tmp_distances_buf.data(), pdx_centroids, partial_d,
                                           not_pruned_counts.data(), nullptr);
            return result_assignments;
        }
    }

    static Config DefaultConfig() {
        Config c;
        c.iters = 10;
        c.sampling_fraction = 0.3f;
        c.max_points_per_cluster = 256;
        c.n_threads = 0;
        c.seed = 42;
        c.use_blas_only = 0;
        c.tol = 1e-4f;
        c.recall_tol = 0.005f;
        c.early_termination = 1;
        c.sample_queries = 0;
        c.objective_k = 100;
        c.ann_explore_fraction = 0.01f;
        c.min_not_pruned_pct = 0.03f;
        c.max_not_pruned_pct = 0.05f;
        c.adjustment_factor_for_partial_d = 0.20f;
        c.unrotate_centroids = 1;
        c.verbose = 0;
        c.angular = 0;
        c.suppress_warnings = 0;
        c.data_already_rotated = 0;
        c.iters_mesoclustering = 3;
        c.iters_fineclustering = 5;
        c.iters_refinement = 0;
        c.dct_rotation = 0;
        return c;
    }

    // Test hook, no counterpart in the reference: the seeds of the last AssignTrainingPoints, which the reference
    // builds in place in its result array before the pruned search overwrites them.
    std::vector<uint32_t> last_seeds;

    // ---- members mirrored from superkmeans.h:1445-1492 ----
    const size_t d;
    const size_t n_clusters;
    Config config;
    bool hierarchical;
    uint32_t n_threads;
    size_t n_samples = 0;
    uint32_t partial_d = 0;
    bool trained = false;
    size_t n_split = 0;
    size_t centroids_to_explore = 0;
    uint32_t vertical_d = 0;
    float prev_cost = 0.0f, cost = 0.0f, shift = 0.0f, recall = 0.0f;
    double cost_f64 = 0.0;
    std::unique_ptr<ADSamplingPruner> pruner;
    std::unique_ptr<float[]> centroids, horizontal_centroids, prev_centroids, partial_horizontal_centroids;
    std::unique_ptr<float[]> distances;
    std::unique_ptr<uint32_t[]> cluster_sizes;
    std::unique_ptr<float[]> data_norms, centroid_norms;
    std::unique_ptr<size_t[]> sampled_indices;
    std::unique_ptr<uint32_t[]> gt_assignments;
    std::unique_ptr<float[]> gt_distances, query_norms, tmp_distances_buffer;
    std::unique_ptr<uint32_t[]> promising_centroids;
    std::unique_ptr<float[]> recall_distances;
    std::unique_ptr<uint32_t[]> assignments;
    std::vector<IterationStats> iteration_stats;
    // hierarchical_superkmeans.h:817-825
    size_t n_mesoclusters = 0;
    std::vector<uint32_t> mesoclusters_assignments, mesoclusters_sizes;
    std::unique_ptr<uint32_t[]> final_assignments;
    std::unique_ptr<float[]> immutable_data_norms, final_centroids;
    std::vector<IterationStats> meso_stats, fine_stats, refinement_stats;
    // pruning accounting of the last pruned iteration (oracle extra)
    PruneAccounting last_accounting;
    bool collect_accounting = false;

    // superkmeans.h:729-765. The per-thread centroid ranges make the summation order ascending in i
    // for every centroid whatever the thread count.
    void UpdateCentroids(const float* data, const size_t n_samples_, const size_t n_clusters_) {
#pragma omp parallel if (n_threads > 1) num_threads(n_threads)
        {
            // The reference uses n_threads here; the team size is read back instead so that a smaller
            // team than requested still covers every centroid range.
            uint32_t nt = omp_get_num_threads();
            uint32_t rank = omp_get_thread_num();
            size_t c0 = (n_clusters_ * rank) / nt;
            size_t c1 = (n_clusters_ * (rank + 1)) / nt;
            for (size_t i = 0; i < n_samples_; i++) {
                uint32_t ci = assignments[i];
                if (ci >= c0 && ci < c1) {
                    auto vector_p = data + i * d;
                    cluster_sizes[ci] += 1;
                    float* acc = horizontal_centroids.get() + (size_t) ci * d;
                    for (size_t t = 0; t < d; ++t) acc[t] += vector_p[t];
                }
            }
        }
    }

    // superkmeans.h:786-879
    void RunIteration(bool GEMM_ONLY, const float* data_to_cluster, float* tmp_distances_buf,
                      PDXIndex& centroids_pdx_wrapper, std::vector<float>& centroids_partial_norms,
                      std::vector<size_t>& not_pruned_counts, const float* rotated_queries, const size_t n_queries,
                      const size_t n_samples_, const size_t n_clusters_, size_t iter_idx, const bool is_first_iter,
                      std::vector<IterationStats>& target_stats) {
        if (!is_first_iter) std::swap(horizontal_centroids, prev_centroids);
        if (GEMM_ONLY) {
            GetL2NormsRowMajor(prev_centroids.get(), n_clusters_, centroid_norms.get());
            // FirstAssignAndUpdateCentroids, superkmeans.h:644-670
            FindNearestNeighbor(data_to_cluster, prev_centroids.get(), n_samples_, n_clusters_, d, data_norms.get(),
                                centroid_norms.get(), assignments.get(), distances.get(), tmp_distances_buf);
        } else {
            if (centroids_partial_norms.size() < n_clusters_) centroids_partial_norms.resize(n_clusters_);
            if (not_pruned_counts.size() < n_samples_) not_pruned_counts.resize(n_samples_);
            GetPartialL2NormsRowMajor(prev_centroids.get(), n_clusters_, centroids_partial_norms.data(), partial_d);
            std::fill(not_pruned_counts.data(), not_pruned_counts.data() + n_samples_, 0);
            // The wrapper built once in the reference holds pointers into `centroids` /
            // `partial_horizontal_centroids`; its chunk table depends only on (n_clusters, d).
            centroids_pdx_wrapper.FromBuffer(centroids.get(), n_clusters_, d, partial_horizontal_centroids.get(),
                                             pruner->ratios.data());
            // AssignAndUpdateCentroids, superkmeans.h:685-717
            FindNearestNeighborWithPruning(data_to_cluster, prev_centroids.get(), n_samples_, n_clusters_, d,
                                           data_norms.get(), centroids_partial_norms.data(), assignments.get(),
                                           distances.get(), tmp_distances_buf, centroids_pdx_wrapper, partial_d,
                                           not_pruned_counts.data(), collect_accounting ? &last_accounting : nullptr);
        }
        std::fill(horizontal_centroids.get(), horizontal_centroids.get() + (n_clusters_ * d), 0.0f);
        std::fill(cluster_sizes.get(), cluster_sizes.get() + n_clusters_, 0);
        UpdateCentroids(data_to_cluster, n_samples_, n_clusters_);

        float avg_not_pruned_pct = -1.0f;
        uint32_t old_partial_d = partial_d;
        if (!GEMM_ONLY) {
            bool partial_d_changed = false;
            avg_not_pruned_pct = TunePartialD(not_pruned_counts.data(), n_samples_, n_clusters_, partial_d_changed);
            if (partial_d_changed) GetPartialL2NormsRowMajor(data_to_cluster, n_samples_, data_norms.get(), partial_d);
        }
        ConsolidateCentroids(n_samples_, n_clusters_);
        ComputeCost(n_samples_);
        ComputeShift(n_clusters_);
        if (n_queries) {
            GetL2NormsRowMajor(horizontal_centroids.get(), n_clusters_, centroid_norms.get());
            recall = ComputeRecall(rotated_queries, n_queries);
        }
        IterationStats stats{};
        stats.iteration = iter_idx + 1;
        stats.objective = cost;
        stats.objective_f64 = cost_f64;
        stats.shift = shift;
        stats.split = n_split;
        stats.recall = recall;
        stats.is_gemm_only = GEMM_ONLY;
        stats.not_pruned_pct = -1.0f;
        stats.partial_d = 0;
        if (!GEMM_ONLY) {
            stats.not_pruned_pct = avg_not_pruned_pct;
            stats.partial_d = old_partial_d;
        }
        target_stats.push_back(stats);
        if (config.verbose) {
            printf("Iteration %zu | Objective: %g | Shift: %g | Split: %zu | Recall: %g", iter_idx + 1, cost, shift,
                   n_split, recall);
            if (GEMM_ONLY)
                printf(" [BLAS-only]\n");
            else
                printf(" | Not Pruned %%: %g | d': %u -> %u\n", avg_not_pruned_pct * 100.0f, old_partial_d, partial_d);
        }
    }

    // superkmeans.h:890-928 and hierarchical_superkmeans.h:579-678
    void SplitClusters(const size_t n_samples_, const size_t n_clusters_) {
        n_split = 0;
        std::mt19937 rng(config.seed);
        auto horizontal_centroids_p = horizontal_centroids.get();
        if (!hierarchical) {
            for (size_t ci = 0; ci < n_clusters_; ci++) {
                if (cluster_sizes[ci] == 0) {
                    size_t cj;
                    for (cj = 0; true; cj = (cj + 1) % n_clusters_) {
                        float p = (cluster_sizes[cj] - 1.0) / (float) (n_samples_ - n_clusters_);
                        float r = std::uniform_real_distribution<float>(0, 1)(rng);
                        if (r < p) break;
                    }
                    std::memcpy(horizontal_centroids_p + ci * d, horizontal_centroids_p + cj * d, sizeof(float) * d);
                    for (size_t j = 0; j < d; j++) {
                        if (j % 2 == 0) {
                            horizontal_centroids_p[ci * d + j] *= 1 + CENTROID_PERTURBATION_EPS;
                            horizontal_centroids_p[cj * d + j] *= 1 - CENTROID_PERTURBATION_EPS;
                        } else {
                            horizontal_centroids_p[ci * d + j] *= 1 - CENTROID_PERTURBATION_EPS;
                            horizontal_centroids_p[cj * d + j] *= 1 + CENTROID_PERTURBATION_EPS;
                        }
                    }
                    cluster_sizes[ci] = cluster_sizes[cj] / 2;
                    cluster_sizes[cj] -= cluster_sizes[ci];
                    n_split++;
                }
            }
            return;
        }
        constexpr float CENTER_ADJUSTMENT_WEIGHT = 7.0f;
        constexpr float BALANCING_THRESHOLD = 0.25f;
        size_t average_size = n_samples_ / n_clusters_;
        size_t threshold_size = static_cast<size_t>(static_cast<float>(average_size) * BALANCING_THRESHOLD);
        for (size_t ci = 0; ci < n_clusters_; ci++) {
            if (cluster_sizes[ci] == 0) {
                size_t cj;
                for (cj = 0; true; cj = (cj + 1) % n_clusters_) {
                    float p = (cluster_sizes[cj] - 1.0f) / static_cast<float>(n_samples_ - n_clusters_);
                    float r = std::uniform_real_distribution<float>(0, 1)(rng);
                    if (r < p) break;
                }
                std::memcpy(horizontal_centroids_p + ci * d, horizontal_centroids_p + cj * d, sizeof(float) * d);
                for (size_t j = 0; j < d; j++) {
                    if (j % 2 == 0) {
                        horizontal_centroids_p[ci * d + j] *= 1.0f + CENTROID_PERTURBATION_EPS;
                        horizontal_centroids_p[cj * d + j] *= 1.0f - CENTROID_PERTURBATION_EPS;
                    } else {
                        horizontal_centroids_p[ci * d + j] *= 1.0f - CENTROID_PERTURBATION_EPS;
                        horizontal_centroids_p[cj * d + j] *= 1.0f + CENTROID_PERTURBATION_EPS;
                    }
                }
                cluster_sizes[ci] = cluster_sizes[cj] / 2;
                cluster_sizes[cj] -= cluster_sizes[ci];
                n_split++;
            }
        }
        for (size_t ci = 0; ci < n_clusters_; ci++) {
            size_t csize = cluster_sizes[ci];
            if (csize == 0 || csize > threshold_size) continue;
            size_t large_cluster_idx;
            for (large_cluster_idx = 0; true; large_cluster_idx = (large_cluster_idx + 1) % n_clusters_) {
                size_t large_size = cluster_sizes[large_cluster_idx];
                if (large_size < average_size) continue;
                float p = static_cast<float>(large_size - average_size + 1) /
                          static_cast<float>(n_samples_ - average_size * n_clusters_ + n_clusters_);
                float r = std::uniform_real_distribution<float>(0, 1)(rng);
                if (r < p) break;
            }
            float wc = std::min(static_cast<float>(csize), CENTER_ADJUSTMENT_WEIGHT);
            float wd = 1.0f;
            for (size_t j = 0; j < d; j++) {
                float val = 0.0f;
                val += wc * horizontal_centroids_p[ci * d + j];
                val += wd * horizontal_centroids_p[large_cluster_idx * d + j];
                val /= (wc + wd);
                horizontal_centroids_p[ci * d + j] = val;
            }
            n_split++;
        }
    }

    // superkmeans.h:936-968
    void ConsolidateCentroids(const size_t n_samples_, const size_t n_clusters_) {
#pragma omp parallel for if (n_threads > 1) num_threads(n_threads)
        for (size_t i = 0; i < n_clusters_; ++i) {
            auto p = horizontal_centroids.get() + i * d;
            if (cluster_sizes[i] == 0) continue;
            float mult_factor = 1.0 / cluster_sizes[i];
            for (size_t j = 0; j < d; ++j) p[j] *= mult_factor;
        }
        SplitClusters(n_samples_, n_clusters_);
        if (config.angular) PostprocessCentroids(n_clusters_);
        PDXify(horizontal_centroids.get(), centroids.get(), n_clusters_, d);
        CentroidsToAuxiliaryHorizontal(n_clusters_);
    }

    // superkmeans.h:973-981 (fp32, sequential) plus the same sum in fp64
    void ComputeCost(const size_t n_samples_) {
        prev_cost = cost;
        cost = 0.0f;
        cost_f64 = 0.0;
        for (size_t i = 0; i < n_samples_; ++i) {
            cost += distances[i];
            cost_f64 += (double) distances[i];
        }
    }

    // superkmeans.h:988-998
    void ComputeShift(const size_t n_clusters_) {
        float total_shift = 0.0f;
#pragma omp parallel for reduction(+ : total_shift) if (n_threads > 1) num_threads(n_threads)
        for (size_t i = 0; i < n_clusters_; ++i) {
            const float* a = horizontal_centroids.get() + i * d;
            const float* b = prev_centroids.get() + i * d;
            float s = 0.0f;
            for (size_t j = 0; j < d; ++j) {
                float t = a[j] - b[j];
                s += t * t;
            }
            total_shift += s;
        }
        shift = total_shift;
    }

    // superkmeans.h:1010-1031
    void GetGTAssignmentsAndDistances(const float* data, const float* queries, const size_t n_queries) {
        std::vector<float> gt_query_norms(n_queries);
        GetL2NormsRowMajor(queries, n_queries, gt_query_norms.data());
        FindKNearestNeighbors(queries, data, n_queries, n_samples, d, gt_query_norms.data(), data_norms.get(),
                              config.objective_k, gt_assignments.get(), gt_distances.get(), tmp_distances_buffer.get());
    }

    // superkmeans.h:1044-1087
    float ComputeRecall(const float* queries, const size_t n_queries) {
        FindKNearestNeighbors(queries, horizontal_centroids.get(), n_queries, n_clusters, d, query_norms.get(),
                              centroid_norms.get(), centroids_to_explore, promising_centroids.get(),
                              recall_distances.get(), tmp_distances_buffer.get());
        return RecallFromLists(gt_assignments.get(), promising_centroids.get(), assignments.get(), n_queries,
                               config.objective_k, centroids_to_explore);
    }

    // superkmeans.h:1100-1142
    PDXIndex GenerateCentroids(const float* data, const size_t n_points, const size_t n_clusters_, const bool rotate) {
        auto tmp_centroids_p = horizontal_centroids.get();
        std::mt19937 rng(config.seed);
        std::vector<size_t> indices(n_points);
        for (size_t i = 0; i < n_points; ++i) indices[i] = i;
        std::shuffle(indices.begin(), indices.end(), rng);
        for (size_t i = 0; i < n_clusters_; i += 1) {
            std::memcpy(tmp_centroids_p, data + (indices[i] * d), sizeof(float) * d);
            tmp_centroids_p += d;
        }
        std::vector<float> rotated_centroids(n_clusters_ * d);
        RotateOrCopy(horizontal_centroids.get(), rotated_centroids.data(), n_clusters_, rotate);
        PDXify(rotated_centroids.data(), centroids.get(), n_clusters_, d);
        PDXIndex idx;
        idx.FromBuffer(centroids.get(), n_clusters_, d, partial_horizontal_centroids.get(), pruner->ratios.data());
        return idx;
    }

    // superkmeans.h:1147-1171 (Eigen rowwise().squaredNorm() written as a plain loop)
    void GetPartialL2NormsRowMajor(const float* data, const size_t n, float* out_norm, const size_t partial_d_) {
#pragma omp parallel for num_threads(n_threads)
        for (size_t i = 0; i < n; ++i) {
            const float* p = data + i * d;
            float s = 0.0f;
            for (size_t j = 0; j < partial_d_; ++j) s += p[j] * p[j];
            out_norm[i] = s;
        }
    }
    void GetL2NormsRowMajor(const float* data, const size_t n, float* out_norm) {
        GetPartialL2NormsRowMajor(data, n, out_norm, d);
    }

    // superkmeans.h:1183-1199
    void RotateOrCopy(const float* in, float* out, const size_t n_vectors, const bool rotate) {
        if (rotate)
            pruner->Rotate(in, out, n_vectors);
        else
            std::memcpy(out, in, sizeof(float) * n_vectors * d);
    }

    // superkmeans.h:1206-1212
    void CentroidsToAuxiliaryHorizontal(const size_t n_clusters_) {
        for (size_t i = 0; i < n_clusters_; ++i)
            std::memcpy(partial_horizontal_centroids.get() + i * vertical_d, horizontal_centroids.get() + i * d,
                        sizeof(float) * vertical_d);
    }

    // superkmeans.h:1230-1258
    float TunePartialD(const size_t* not_pruned_counts, size_t n_samples_, size_t n_y, bool& partial_d_changed) {
        float avg_not_pruned_pct = 0.0f;
        for (size_t i = 0; i < n_samples_; ++i) avg_not_pruned_pct += static_cast<float>(not_pruned_counts[i]);
        avg_not_pruned_pct /= static_cast<float>(n_samples_ * n_y);
        uint32_t old_partial_d = partial_d;
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

    // superkmeans.h:1269-1277 and hierarchical_superkmeans.h:559-567
    size_t GetNVectorsToSample(const size_t n, size_t n_clusters_) const {
        if (config.sampling_fraction == 1.0) return n;
        if (hierarchical)
            return static_cast<size_t>(std::floor(static_cast<double>(n) * config.sampling_fraction));
        auto samples_byn_clusters = n_clusters_ * config.max_points_per_cluster;
        auto samples_by_n = static_cast<size_t>(std::floor(static_cast<float>(n) * config.sampling_fraction));
        return std::min<size_t>(samples_by_n, samples_byn_clusters);
    }

    // superkmeans.h:1294-1333
    bool ShouldStopEarly(const bool tracking_recall, float& best_recall, size_t& iters_without_improvement,
                         const size_t iter_idx) {
        if (shift < config.tol) return true;
        if (iter_idx > 0) {
            auto cost_delta = cost / prev_cost;
            if (cost_delta > 1 - config.tol) return true;
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

    // superkmeans.h:1341-1351
    std::vector<float> GetOutputCentroids(bool should_unrotate) {
        if (should_unrotate) {
            std::vector<float> unrotated(n_clusters * d);
            pruner->Unrotate(horizontal_centroids.get(), unrotated.data(), n_clusters);
            return unrotated;
        }
        return std::vector<float>(horizontal_centroids.get(), horizontal_centroids.get() + n_clusters * d);
    }

    // superkmeans.h:1357-1371
    void PostprocessCentroids(const size_t n_clusters_) {
        auto p = horizontal_centroids.get();
#pragma omp parallel for if (n_threads > 1) num_threads(n_threads)
        for (size_t i = 0; i < n_clusters_; ++i) {
            auto pi = p + i * d;
            float sum = 0.0f;
            for (size_t j = 0; j < d; ++j) sum += pi[j] * pi[j];
            float norm = 1.0f / std::sqrt(sum);
            for (size_t j = 0; j < d; ++j) pi[j] *= norm;
        }
    }

    // superkmeans.h:1385-1443
    const float* SampleAndRotateVectors(const float* data, std::vector<float>& out, const size_t n,
                                        const size_t n_samples_, const bool rotate) {
        std::vector<float> samples_tmp;
        const float* src_data = data;
        if (n_samples_ < n) {
            std::mt19937 rng(config.seed);
            sampled_indices.reset(new size_t[n]);
            for (size_t i = 0; i < n; ++i) sampled_indices[i] = i;
            std::shuffle(sampled_indices.get(), sampled_indices.get() + n, rng);
            if (rotate) {
                samples_tmp.resize(n_samples_ * d);
                for (size_t i = 0; i < n_samples_; ++i)
                    std::memcpy(samples_tmp.data() + i * d, data + sampled_indices[i] * d, sizeof(float) * d);
                src_data = samples_tmp.data();
            } else {
                out.resize(n_samples_ * d);
                for (size_t i = 0; i < n_samples_; ++i)
                    std::memcpy(out.data() + i * d, data + sampled_indices[i] * d, sizeof(float) * d);
                return out.data();
            }
        }
        if (!rotate) return data;
        out.resize(n_samples_ * d);
        RotateOrCopy(src_data, out.data(), n_samples_, rotate);
        return out.data();
    }

    // ---- hierarchical_superkmeans.h:84-541 ----
    std::vector<float> TrainHierarchical(const float* data, const size_t n, const float* /*queries*/,
                                         const size_t n_queries) {
        ENSURE_POSITIVE(n);
        if (trained) throw std::runtime_error("The clustering has already been trained");
        if (n_queries > 0 && !config.suppress_warnings)
            printf("WARNING: Early Termination by Recall is not supported in HierarchicalSuperKMeans\n");
        n_mesoclusters = GetNMesoclusters(n_clusters);
        fine_stats.clear();
        meso_stats.clear();
        refinement_stats.clear();
        if (n < n_clusters)
            throw std::runtime_error("The number of points should be at least as large as the number of clusters");
        const float* data_p = data;
        n_samples = GetNVectorsToSample(n, n_clusters);
        if (n_samples < n_clusters)
            throw std::runtime_error(
                "Not enough samples to train. Try increasing the sampling_fraction or max_points_per_cluster");
        final_assignments.reset(new uint32_t[n_samples]);
        final_centroids.reset(new float[n_clusters * d]);
        centroids.reset(new float[n_clusters * d]);
        horizontal_centroids.reset(new float[n_clusters * d]);
        prev_centroids.reset(new float[n_clusters * d]);
        cluster_sizes.reset(new uint32_t[n_clusters]);
        assignments.reset(new uint32_t[n]);
        distances.reset(new float[n]);
        data_norms.reset(new float[n_samples]);
        centroid_norms.reset(new float[n_clusters]);
        std::vector<float> tmp_distances_buf(X_BATCH_SIZE * Y_BATCH_SIZE);
        vertical_d = GetDimensionSplit(d).vertical_d;
        partial_horizontal_centroids.reset(new float[n_clusters * vertical_d]);
        partial_d = std::max<uint32_t>(MIN_PARTIAL_D, vertical_d / 2);
        if (partial_d > vertical_d) partial_d = vertical_d;
        auto initial_partial_d = partial_d;

        // PHASE 1
        PDXIndex centroids_pdx_wrapper = GenerateCentroids(data_p, n_samples, n_mesoclusters, !config.data_already_rotated);
        std::vector<float> data_samples_buffer;
        const float* data_to_cluster =
            SampleAndRotateVectors(data_p, data_samples_buffer, n, n_samples, !config.data_already_rotated);
        auto initialn_samples = n_samples;
        RotateOrCopy(horizontal_centroids.get(), prev_centroids.get(), n_mesoclusters, !config.data_already_rotated);
        GetL2NormsRowMajor(data_to_cluster, n_samples, data_norms.get());
        GetL2NormsRowMajor(prev_centroids.get(), n_mesoclusters, centroid_norms.get());
        std::vector<float> centroids_partial_norms(n_clusters);
        std::vector<size_t> not_pruned_counts(n_samples);
        immutable_data_norms.reset(new float[n_samples]);
        std::memcpy(immutable_data_norms.get(), data_norms.get(), sizeof(float) * n_samples);

        bool always_gemm_only = d < DIMENSION_THRESHOLD_FOR_PRUNING || config.use_blas_only ||
                                n_mesoclusters <= N_CLUSTERS_THRESHOLD_FOR_PRUNING;
        bool partial_norms_computed = false;
        float best_recall = 0.0f;
        size_t iters_without_improvement = 0;
        for (size_t iter_idx = 0; iter_idx < config.iters_mesoclustering; ++iter_idx) {
            bool use_gemm_only = (iter_idx == 0) || always_gemm_only;
            if (!use_gemm_only && !partial_norms_computed) {
                GetPartialL2NormsRowMajor(data_to_cluster, n_samples, data_norms.get(), partial_d);
                partial_norms_computed = true;
            }
            RunIteration(use_gemm_only, data_to_cluster, tmp_distances_buf.data(), centroids_pdx_wrapper,
                         centroids_partial_norms, not_pruned_counts, nullptr, 0, n_samples, n_mesoclusters, iter_idx,
                         use_gemm_only ? (iter_idx == 0) : false, meso_stats);
            if (config.early_termination && ShouldStopEarly(false, best_recall, iters_without_improvement, iter_idx))
                break;
        }
        mesoclusters_sizes.assign(cluster_sizes.get(), cluster_sizes.get() + n_mesoclusters);
        mesoclusters_assignments.assign(assignments.get(), assignments.get() + n_samples);
        std::vector<size_t> mesocluster_indices_flat(n_samples);
        std::vector<size_t> mesocluster_offsets(n_mesoclusters + 1);
        mesocluster_offsets[0] = 0;
        for (size_t k = 0; k < n_mesoclusters; ++k) mesocluster_offsets[k + 1] = mesocluster_offsets[k] + mesoclusters_sizes[k];
        {
            std::vector<size_t> next_to_write_index = mesocluster_offsets;
            for (size_t i = 0; i < n_samples; ++i) {
                size_t cluster_id = mesoclusters_assignments[i];
                mesocluster_indices_flat[next_to_write_index[cluster_id]++] = i;
            }
        }

        // PHASE 2
        auto fine_clusters_nums = ArrangeFineClusters(n_clusters, n_mesoclusters, n_samples, mesoclusters_sizes);
        size_t max_mesocluster_size = *std::max_element(cluster_sizes.get(), cluster_sizes.get() + n_mesoclusters);
        std::vector<float> mesocluster_buffer(max_mesocluster_size * d);
        std::vector<uint32_t> assignments_indirection_buffer(max_mesocluster_size);
        size_t fineclusters_offset = 0;
        for (size_t k = 0; k < n_mesoclusters; ++k) {
            size_t n_fineclusters = fine_clusters_nums[k];
            if (n_fineclusters == 0) continue;
            partial_d = initial_partial_d;
            auto mesocluster_size = mesoclusters_sizes[k];
            n_samples = mesocluster_size;
            // CompactMesoclusterToBuffer, hierarchical_superkmeans.h:685-704
            {
                const size_t* mesocluster_indices = mesocluster_indices_flat.data() + mesocluster_offsets[k];
#pragma omp parallel for if (n_threads > 1) num_threads(n_threads)
                for (size_t j = 0; j < mesocluster_size; ++j) {
                    size_t i = mesocluster_indices[j];
                    data_norms[j] = immutable_data_norms[i];
                    assignments_indirection_buffer[j] = i;
                    std::memcpy(mesocluster_buffer.data() + j * d, data_to_cluster + i * d, sizeof(float) * d);
                }
            }
            auto mesocluster_data_to_cluster = mesocluster_buffer.data();
            PDXIndex meso_wrapper = GenerateCentroids(mesocluster_data_to_cluster, mesocluster_size, n_fineclusters, false);
            std::memcpy(prev_centroids.get(), horizontal_centroids.get(), sizeof(float) * n_fineclusters * d);
            GetL2NormsRowMajor(prev_centroids.get(), n_fineclusters, centroid_norms.get());
            bool fine_always_gemm_only = d < DIMENSION_THRESHOLD_FOR_PRUNING || config.use_blas_only ||
                                         n_fineclusters <= N_CLUSTERS_THRESHOLD_FOR_PRUNING;
            bool fine_partial_norms_computed = false;
            float fine_best_recall = 0.0f;
            iters_without_improvement = 0;
            for (size_t fine_iter_idx = 0; fine_iter_idx < config.iters_fineclustering; ++fine_iter_idx) {
                bool use_gemm_only = (fine_iter_idx == 0) || fine_always_gemm_only;
                if (!use_gemm_only && !fine_partial_norms_computed) {
                    GetPartialL2NormsRowMajor(mesocluster_data_to_cluster, n_samples, data_norms.get(), partial_d);
                    fine_partial_norms_computed = true;
                }
                RunIteration(use_gemm_only, mesocluster_data_to_cluster, tmp_distances_buf.data(), meso_wrapper,
                             centroids_partial_norms, not_pruned_counts, nullptr, 0, n_samples, n_fineclusters,
                             fine_iter_idx, use_gemm_only ? (fine_iter_idx == 0) : false, fine_stats);
                if (config.early_termination &&
                    ShouldStopEarly(false, fine_best_recall, iters_without_improvement, fine_iter_idx))
                    break;
            }
            // GetTrueAssignmentsFromIndirectionBuffer, hierarchical_superkmeans.h:763-779
            for (size_t i = 0; i < mesocluster_size; ++i) {
                size_t original_idx = assignments_indirection_buffer[i];
                final_assignments[original_idx] = assignments[i] + fineclusters_offset;
            }
            std::memcpy(final_centroids.get() + fineclusters_offset * d, horizontal_centroids.get(),
                        sizeof(float) * n_fineclusters * d);
            fineclusters_offset += n_fineclusters;
        }

        // PHASE 3
        n_samples = initialn_samples;
        partial_d = std::max<uint32_t>(MIN_PARTIAL_D, vertical_d / 3);
        // SetupCentroids, hierarchical_superkmeans.h:788-815
        std::memcpy(horizontal_centroids.get(), final_centroids.get(), sizeof(float) * n_clusters * d);
        PDXify(horizontal_centroids.get(), centroids.get(), n_clusters, d);
        PDXIndex final_refinement_pdx_wrapper;
        final_refinement_pdx_wrapper.FromBuffer(centroids.get(), n_clusters, d, partial_horizontal_centroids.get(),
                                                pruner->ratios.data());
        CentroidsToAuxiliaryHorizontal(n_clusters);
        std::memcpy(prev_centroids.get(), final_centroids.get(), sizeof(float) * n_clusters * d);
        std::memcpy(assignments.get(), final_assignments.get(), sizeof(uint32_t) * n_samples);
        GetL2NormsRowMajor(prev_centroids.get(), n_clusters, centroid_norms.get());
        bool refinement_always_gemm_only =
            d < DIMENSION_THRESHOLD_FOR_PRUNING || n_clusters <= N_CLUSTERS_THRESHOLD_FOR_PRUNING;
        bool refinement_partial_norms_computed = false;
        for (size_t refinement_iter_idx = 0; refinement_iter_idx < config.iters_refinement; ++refinement_iter_idx) {
            if (!refinement_always_gemm_only && !refinement_partial_norms_computed) {
                GetPartialL2NormsRowMajor(data_to_cluster, n_samples, data_norms.get(), partial_d);
                refinement_partial_norms_computed = true;
            }
            if (refinement_always_gemm_only) {
                // The fine phase left per-mesocluster norms in data_norms (hierarchical_superkmeans.h:475-478
                // notes the same for the pruned branch); the GEMM-only branch reads them as they are.
            }
            RunIteration(refinement_always_gemm_only, data_to_cluster, tmp_distances_buf.data(),
                         final_refinement_pdx_wrapper, centroids_partial_norms, not_pruned_counts, nullptr, 0,
                         n_samples, n_clusters, refinement_iter_idx, false, refinement_stats);
        }
        trained = true;
        return GetOutputCentroids(config.unrotate_centroids);
    }

    // hierarchical_superkmeans.h:549-551
    static size_t GetNMesoclusters(const size_t n_clusters_) {
        return static_cast<size_t>(std::round(std::sqrt(n_clusters_)));
    }

    // hierarchical_superkmeans.h:718-761
    static std::vector<size_t> ArrangeFineClusters(size_t n_clusters_, size_t n_mesoclusters_, size_t n_samples_,
                                                   const std::vector<uint32_t>& mesocluster_sizes) {
        std::vector<size_t> fine_clusters_nums(n_mesoclusters_);
        size_t n_clusters_remaining = n_clusters_;
        size_t n_nonempty_mesoclusters_remaining = 0;
        for (size_t i = 0; i < n_mesoclusters_; ++i)
            if (mesocluster_sizes[i] > 0) n_nonempty_mesoclusters_remaining++;
        size_t n_samples_remaining = n_samples_;
        for (size_t i = 0; i < n_mesoclusters_; ++i) {
            if (i < n_mesoclusters_ - 1) {
                if (mesocluster_sizes[i] == 0) {
                    fine_clusters_nums[i] = 0;
                } else {
                    n_nonempty_mesoclusters_remaining--;
                    double proportion = static_cast<double>(n_clusters_remaining * mesocluster_sizes[i]) /
                                        static_cast<double>(n_samples_remaining);
                    size_t allocated = static_cast<size_t>(std::lround(proportion));
                    allocated = std::min(allocated, n_clusters_remaining - n_nonempty_mesoclusters_remaining);
                    fine_clusters_nums[i] = std::max(allocated, size_t{1});
                }
            } else {
                fine_clusters_nums[i] = n_clusters_remaining;
            }
            n_clusters_remaining -= fine_clusters_nums[i];
            n_samples_remaining -= mesocluster_sizes[i];
        }
        return fine_clusters_nums;
    }
};

} // namespace oracle

// =================================================================================================
// C entry points for the tests and the CPU baseline
// =================================================================================================
using namespace oracle;

static thread_local std::string g_err;
static thread_local int g_err_kind = 0;  // 1 invalid_argument, 2 runtime_error, 3 other

#define ORACLE_GUARD(body)                                                                         \
    try {                                                                                          \
        g_err_kind = 0;                                                                            \
        body;                                                                                      \
        return 0;                                                                                  \
    } catch (const std::invalid_argument& e) {                                                     \
        g_err = e.what();                                                                          \
        g_err_kind = 1;                                                                            \
        return -1;                                                                                 \
    } catch (const std::runtime_error& e) {                                                        \
        g_err = e.what();                                                                          \
        g_err_kind = 2;                                                                            \
        return -2;                                                                                 \
    } catch (const std::exception& e) {                                                            \
        g_err = e.what();                                                                          \
        g_err_kind = 3;                                                                            \
        return -3;                                                                                 \
    }

extern "C" {

const char* oracle_last_error() { return g_err.c_str(); }

// Tries the given shared libraries in order for a Fortran-ABI sgemm_; returns 1 when one was bound.
int oracle_bind_blas(const char* const* paths, int n_paths) {
    for (int i = 0; i < n_paths; ++i) {
        void* h = dlopen(paths[i], RTLD_NOW | RTLD_LOCAL);
        if (!h) continue;
        void* sym = dlsym(h, "sgemm_");
        if (sym) {
            g_sgemm = reinterpret_cast<sgemm_fn>(sym);
            g_blas_name = paths[i];
            return 1;
        }
    }
    return 0;
}
const char* oracle_blas_name() { return g_blas_name.c_str(); }
void oracle_set_threads(uint32_t n) { g_n_threads = n == 0 ? (uint32_t) omp_get_max_threads() : n; }
uint32_t oracle_get_threads() { return g_n_threads; }
int oracle_max_threads() { return omp_get_max_threads(); }

void oracle_dimension_split(size_t d, size_t* horizontal_d, size_t* vertical_d) {
    auto s = GetDimensionSplit(d);
    *horizontal_d = s.horizontal_d;
    *vertical_d = s.vertical_d;
}
void oracle_pdxify(const float* in, float* out, size_t n, size_t d) { PDXify(in, out, n, d); }
void oracle_ratios(uint32_t d, float epsilon0, float* out) {
    // Same closed form as ADSamplingPruner::GetRatio without building a rotation matrix.
    for (size_t v = 0; v <= d; ++v) {
        if (v == 0 || v == d) {
            out[v] = 1.0f;
        } else {
            out[v] = static_cast<float>(static_cast<double>(v) / static_cast<double>(d) *
                                        (1.0 + epsilon0 / std::sqrt(static_cast<double>(v))) *
                                        (1.0 + epsilon0 / std::sqrt(static_cast<double>(v))));
        }
    }
}
void oracle_rotation_matrix(uint32_t d, uint32_t seed, float* out) {
    ADSamplingPruner p(d, PRUNER_INITIAL_THRESHOLD, seed);
    std::memcpy(out, p.matrix.data(), sizeof(float) * (size_t) d * d);
}
// Rotation of the DCT variant (rotation_kind 1 or 2); forward != 0: Rotate, else Unrotate.  out_matrix (d*d, may
// be NULL) receives the equivalent explicit matrix.  Returns 1 when the variant applies to this d, else 0
// (then the dense rotation is used, as in the reference).
int oracle_rotate_kind(uint32_t d, uint32_t seed, int rotation_kind, int forward, const float* x, uint32_t n,
                       float* out, float* out_matrix) {
    ADSamplingPruner p(d, 1.5f, seed, rotation_kind);
    if (x && out) {
        if (forward) p.Rotate(x, out, n); else p.Unrotate(x, out, n);
    }
    if (out_matrix) std::memcpy(out_matrix, p.matrix.data(), sizeof(float) * d * d);
    return p.use_dct ? 1 : 0;
}
void oracle_rotate(const float* q, uint32_t d, const float* x, uint32_t n, float* out) {
    sgemm('T', 'N', (int) d, (int) n, (int) d, q, (int) d, x, (int) d, out, (int) d);
}
void oracle_unrotate(const float* q, uint32_t d, const float* x, uint32_t n, float* out) {
    sgemm('N', 'N', (int) d, (int) n, (int) d, q, (int) d, x, (int) d, out, (int) d);
}
void oracle_norms(const float* x, size_t n, size_t d, size_t cols, float* out) {
#pragma omp parallel for num_threads(g_n_threads)
    for (size_t i = 0; i < n; ++i) {
        float s = 0.0f;
        for (size_t j = 0; j < cols; ++j) s += x[i * d + j] * x[i * d + j];
        out[i] = s;
    }
}
float oracle_horizontal(const float* a, const float* b, size_t n) { return Horizontal(a, b, n); }

void oracle_find_nn(const float* x, const float* y, size_t n_x, size_t n_y, size_t d, const float* norms_x,
                    const float* norms_y, uint32_t* out_knn, float* out_distances) {
    std::vector<float> tmp(X_BATCH_SIZE * Y_BATCH_SIZE);
    FindNearestNeighbor(x, y, n_x, n_y, d, norms_x, norms_y, out_knn, out_distances, tmp.data());
}

// pdx / aux: PDX copy and first-vertical_d-columns copy of y (as produced by oracle_pdxify and a column slice).
// stage_pairs (optional): d_horizontal / 64 + 2 counters.
void oracle_find_nn_pruned(const float* x, const float* y, size_t n_x, size_t n_y, size_t d, const float* norms_x_p,
                           const float* norms_y_p, uint32_t* inout_knn, float* out_distances, const float* pdx,
                           const float* aux, uint32_t partial_d, const float* ratios, uint64_t* not_pruned_counts,
                           uint64_t* stage_pairs) {
    std::vector<float> tmp(X_BATCH_SIZE * Y_BATCH_SIZE);
    PDXIndex idx;
    idx.FromBuffer(pdx, n_y, d, aux, ratios);
    std::vector<size_t> counts(n_x, 0);
    PruneAccounting acct;
    FindNearestNeighborWithPruning(x, y, n_x, n_y, d, norms_x_p, norms_y_p, inout_knn, out_distances, tmp.data(), idx,
                                   partial_d, counts.data(), stage_pairs ? &acct : nullptr);
    if (not_pruned_counts)
        for (size_t i = 0; i < n_x; ++i) not_pruned_counts[i] = counts[i];
    if (stage_pairs)
        for (size_t s = 0; s < acct.pairs.size(); ++s) stage_pairs[s] = acct.pairs[s];
}

void oracle_find_knn(const float* x, const float* y, size_t n_x, size_t n_y, size_t d, const float* norms_x,
                     const float* norms_y, size_t k, uint32_t* out_knn, float* out_distances) {
    std::vector<float> tmp(X_BATCH_SIZE * Y_BATCH_SIZE);
    FindKNearestNeighbors(x, y, n_x, n_y, d, norms_x, norms_y, k, out_knn, out_distances, tmp.data());
}
float oracle_recall_from_lists(const uint32_t* gt, const uint32_t* promising, const uint32_t* assignments,
                               size_t n_queries, size_t objective_k, size_t explore) {
    return RecallFromLists(gt, promising, assignments, n_queries, objective_k, explore);
}
void oracle_brute_force(const float* x, const float* y, size_t n_x, size_t n_y, size_t d, uint32_t* out_knn,
                        double* out_distances, double* out_second) {
    BruteForce(x, y, n_x, n_y, d, out_knn, out_distances, out_second);
}

void oracle_default_config(Config* out, int hierarchical) {
    *out = KMeans::DefaultConfig();
    if (hierarchical) out->sampling_fraction = 1.0f;  // hierarchical_superkmeans.h:16
}

int oracle_kmeans_create(size_t n_clusters, size_t d, const Config* config, int hierarchical, void** out) {
    ORACLE_GUARD(*out = new KMeans(n_clusters, d, *config, hierarchical != 0));
}
void oracle_kmeans_destroy(void* h) { delete static_cast<KMeans*>(h); }
int oracle_error_kind() { return g_err_kind; }

int oracle_kmeans_train(void* h, const float* data, size_t n, const float* queries, size_t n_queries,
                        float* out_centroids) {
    ORACLE_GUARD({
        auto* km = static_cast<KMeans*>(h);
        auto c = km->Train(data, n, queries, n_queries);
        std::memcpy(out_centroids, c.data(), sizeof(float) * c.size());
    });
}
int oracle_kmeans_assign(void* h, const float* vectors, const float* centroids, size_t n_vectors, size_t n_centroids,
                         uint32_t* out) {
    ORACLE_GUARD({
        auto a = static_cast<KMeans*>(h)->Assign(vectors, centroids, n_vectors, n_centroids);
        std::memcpy(out, a.data(), sizeof(uint32_t) * a.size());
    });
}
int oracle_kmeans_assign_training_points(void* h, const float* vectors, const float* centroids, size_t n_vectors,
                                         size_t n_centroids, uint32_t* out) {
    ORACLE_GUARD({
        auto a = static_cast<KMeans*>(h)->AssignTrainingPoints(vectors, centroids, n_vectors, n_centroids);
        std::memcpy(out, a.data(), sizeof(uint32_t) * a.size());
    });
}
// which: 0 flat iteration_stats, 1 meso, 2 fine, 3 refinement
size_t oracle_kmeans_n_stats(void* h, int which) {
    auto* km = static_cast<KMeans*>(h);
    const std::vector<IterationStats>* v[4] = {&km->iteration_stats, &km->meso_stats, &km->fine_stats, &km->refinement_stats};
    return v[which]->size();
}
void oracle_kmeans_get_stats(void* h, int which, IterationStats* out) {
    auto* km = static_cast<KMeans*>(h);
    const std::vector<IterationStats>* v[4] = {&km->iteration_stats, &km->meso_stats, &km->fine_stats, &km->refinement_stats};
    std::memcpy(out, v[which]->data(), sizeof(IterationStats) * v[which]->size());
}
int oracle_kmeans_is_trained(void* h) { return static_cast<KMeans*>(h)->trained ? 1 : 0; }
// Training-time state, for single-iteration parity checks: row-major rotated centroids of the last
// iteration, assignments and distances of the sampled points.
void oracle_kmeans_state(void* h, float* out_rotated_centroids, uint32_t* out_assignments, float* out_distances,
                         uint32_t* out_cluster_sizes) {
    auto* km = static_cast<KMeans*>(h);
    if (out_rotated_centroids)
        std::memcpy(out_rotated_centroids, km->horizontal_centroids.get(), sizeof(float) * km->n_clusters * km->d);
    if (out_assignments) std::memcpy(out_assignments, km->assignments.get(), sizeof(uint32_t) * km->n_samples);
    if (out_distances) std::memcpy(out_distances, km->distances.get(), sizeof(float) * km->n_samples);
    if (out_cluster_sizes) std::memcpy(out_cluster_sizes, km->cluster_sizes.get(), sizeof(uint32_t) * km->n_clusters);
}
size_t oracle_kmeans_last_seeds(void* h, uint32_t* out, size_t cap) {
    const auto& s = static_cast<KMeans*>(h)->last_seeds;
    if (out && cap >= s.size()) std::memcpy(out, s.data(), s.size() * sizeof(uint32_t));
    return s.size();
}
size_t oracle_kmeans_n_samples(void* h) { return static_cast<KMeans*>(h)->n_samples; }
void oracle_kmeans_collect_accounting(void* h, int on) { static_cast<KMeans*>(h)->collect_accounting = on != 0; }
size_t oracle_kmeans_accounting(void* h, uint64_t* out, size_t cap) {
    auto& p = static_cast<KMeans*>(h)->last_accounting.pairs;
    for (size_t i = 0; i < p.size() && i < cap; ++i) out[i] = p[i];
    return p.size();
}

// ---- single-step helpers (each is the cited member run on caller-provided state) ----

// UpdateCentroids + the scaling loop of ConsolidateCentroids: sums (k x d), sizes (k), then means in place when scale != 0.
void oracle_update_centroids(const float* data, size_t n, size_t d, const uint32_t* assign, size_t k, float* out_sums,
                             uint32_t* out_sizes, int scale, uint32_t n_threads) {
    std::fill(out_sums, out_sums + k * d, 0.0f);
    std::fill(out_sizes, out_sizes + k, 0u);
    uint32_t nt_req = n_threads == 0 ? omp_get_max_threads() : n_threads;
#pragma omp parallel num_threads(nt_req)
    {
        uint32_t nt = omp_get_num_threads();
        uint32_t rank = omp_get_thread_num();
        size_t c0 = (k * rank) / nt;
        size_t c1 = (k * (rank + 1)) / nt;
        for (size_t i = 0; i < n; i++) {
            uint32_t ci = assign[i];
            if (ci >= c0 && ci < c1) {
                out_sizes[ci] += 1;
                float* acc = out_sums + (size_t) ci * d;
                const float* v = data + i * d;
                for (size_t t = 0; t < d; ++t) acc[t] += v[t];
            }
        }
    }
    if (scale) {
        for (size_t i = 0; i < k; ++i) {
            if (out_sizes[i] == 0) continue;
            float mult_factor = 1.0 / out_sizes[i];
            for (size_t j = 0; j < d; ++j) out_sums[i * d + j] *= mult_factor;
        }
    }
}

// SplitClusters on caller state; returns n_split.
size_t oracle_split_clusters(float* centroids_rm, uint32_t* sizes, size_t k, size_t d, size_t n_samples, uint32_t seed,
                             int hierarchical) {
    // SplitClusters reads only the centroid rows, the sizes and the seed; the object is built just
    // to carry them (its constructor factorises a d x d matrix, so tests keep d small).
    Config c = KMeans::DefaultConfig();
    c.seed = seed;
    c.suppress_warnings = 1;
    if (hierarchical) c.sampling_fraction = 1.0f;
    KMeans real(k, d, c, hierarchical != 0);
    real.horizontal_centroids.reset(new float[k * d]);
    real.cluster_sizes.reset(new uint32_t[k]);
    std::memcpy(real.horizontal_centroids.get(), centroids_rm, sizeof(float) * k * d);
    std::memcpy(real.cluster_sizes.get(), sizes, sizeof(uint32_t) * k);
    real.SplitClusters(n_samples, k);
    std::memcpy(centroids_rm, real.horizontal_centroids.get(), sizeof(float) * k * d);
    std::memcpy(sizes, real.cluster_sizes.get(), sizeof(uint32_t) * k);
    return real.n_split;
}

// TunePartialD on caller state; returns avg_not_pruned_pct, writes the new partial_d.
float oracle_tune_partial_d(const uint64_t* counts, size_t n, size_t k, uint32_t partial_d, uint32_t vertical_d,
                            float min_pct, float max_pct, float adj, uint32_t* out_partial_d) {
    float avg = 0.0f;
    for (size_t i = 0; i < n; ++i) avg += static_cast<float>(counts[i]);
    avg /= static_cast<float>(n * k);
    uint32_t pd = partial_d;
    if (avg > max_pct) {
        auto increase = static_cast<uint32_t>(pd * adj * 2);
        pd = std::min(pd + std::max(increase, 1u), vertical_d);
    } else if (avg < min_pct) {
        auto decrease = static_cast<uint32_t>(pd * adj);
        pd = std::max(pd - std::max(decrease, 1u), MIN_PARTIAL_D);
    }
    *out_partial_d = pd;
    return avg;
}

// MakeBlobs of the reference's test utilities (pdx/utils.h:74-123) as it behaves with one OpenMP
// thread (its golden data was generated that way, tests/generate_wcss_ground_truth.cpp:26): centres
// from mt19937(seed) + normal(0, center_spread); points from a second mt19937(seed + 0) that draws,
// per row, the centre index with uniform_int_distribution<size_t> and then one normal(0, cluster_std)
// per feature.
void oracle_make_blobs(size_t n_samples, size_t n_features, size_t n_centers, int normalize, float cluster_std,
                       float center_spread, uint32_t random_state, float* out) {
    std::mt19937 gen(random_state);
    std::normal_distribution<float> center_dist(0.0f, center_spread);
    std::vector<float> centers(n_centers * n_features);
    for (size_t i = 0; i < n_centers * n_features; ++i) centers[i] = center_dist(gen);
    std::uniform_int_distribution<size_t> cluster_dist(0, n_centers - 1);
    std::normal_distribution<float> point_dist(0.0f, cluster_std);
    std::mt19937 thread_gen(random_state + 0u);
    for (size_t i = 0; i < n_samples; ++i) {
        size_t center_idx = cluster_dist(thread_gen) * n_features;
        float* row = &out[i * n_features];
        const float* center = &centers[center_idx];
        for (size_t j = 0; j < n_features; ++j) row[j] = center[j] + point_dist(thread_gen);
    }
    if (normalize) {
        for (size_t i = 0; i < n_samples; ++i) {
            float* row = &out[i * n_features];
            float norm_sq = 0.0f;
            for (size_t j = 0; j < n_features; ++j) norm_sq += row[j] * row[j];
            float inv_norm = 1.0f / std::sqrt(norm_sq);
            for (size_t j = 0; j < n_features; ++j) row[j] *= inv_norm;
        }
    }
}

void oracle_arrange_fine_clusters(size_t n_clusters, size_t n_meso, size_t n_samples, const uint32_t* sizes,
                                  uint64_t* out) {
    std::vector<uint32_t> s(sizes, sizes + n_meso);
    auto r = KMeans::ArrangeFineClusters(n_clusters, n_meso, n_samples, s);
    for (size_t i = 0; i < n_meso; ++i) out[i] = r[i];
}
size_t oracle_n_mesoclusters(size_t n_clusters) { return KMeans::GetNMesoclusters(n_clusters); }

} // extern "C"
