// ADSampling pruner, HIP backend: threshold ratios and the random orthogonal rotation.
//
// Mirrors the interface of the reference's ADSamplingPruner (pdx/adsampling.h:29-328): the ratios
// table, Rotate and Unrotate.  The d x d matrix is built on the host and kept on the device (Q and
// Q^T); Rotate/Unrotate are MFMA GEMMs (skm_rotate / skm_unrotate).  Both rotations of the reference
// are orthonormal matrices, so both run through the same GEMM: the dense Gaussian one (default build
// of the reference) and the sign flip + DCT-II one (reference builds with FFTW, d >= 512).
#pragma once

#include <cmath>
#include <random>
#include <vector>

#include "superkmeans/common.h"

namespace skmeans {

namespace detail {

// Q factor of the Householder QR of `a` (d x d, row-major, double), i.e. H_0 H_1 ... H_{d-1}.
// Evaluated in double.  Translation units that must reproduce the matrix bit for bit across
// compilers (the library's own) are built with -ffp-contract=off; otherwise fused multiply-adds may
// change the last bits of the draws and of the factor, which is harmless for clustering.
inline std::vector<float> OrthogonalFactor(std::vector<double> a, const size_t d) {
    std::vector<double> reflectors(d * d, 0.0);  // column j holds reflector j in rows j..d-1
    std::vector<double> scale(d, 0.0);
    std::vector<double> w(d);
    for (size_t j = 0; j < d; ++j) {
        double norm2 = 0.0;
        for (size_t r = j; r < d; ++r) {
            const double v = a[r * d + j];
            reflectors[r * d + j] = v;
            norm2 += v * v;
        }
        const double norm = std::sqrt(norm2);
        if (norm == 0.0) continue;
        const double head = reflectors[j * d + j];
        const double alpha = (head >= 0.0) ? -norm : norm;
        reflectors[j * d + j] = head - alpha;
        double vtv = 0.0;
        for (size_t r = j; r < d; ++r) vtv += reflectors[r * d + j] * reflectors[r * d + j];
        if (vtv == 0.0) continue;
        scale[j] = 2.0 / vtv;
        for (size_t c = j; c < d; ++c) w[c] = 0.0;
        for (size_t r = j; r < d; ++r) {
            const double vr = reflectors[r * d + j];
            const double* row = &a[r * d];
            for (size_t c = j; c < d; ++c) w[c] += vr * row[c];
        }
        for (size_t r = j; r < d; ++r) {
            const double f = scale[j] * reflectors[r * d + j];
            double* row = &a[r * d];
            for (size_t c = j; c < d; ++c) row[c] -= f * w[c];
        }
    }
    std::vector<double> q(d * d, 0.0);
    for (size_t i = 0; i < d; ++i) q[i * d + i] = 1.0;
    for (size_t j = d; j-- > 0;) {
        if (scale[j] == 0.0) continue;
        for (size_t c = 0; c < d; ++c) w[c] = 0.0;
        for (size_t r = j; r < d; ++r) {
            const double vr = reflectors[r * d + j];
            const double* row = &q[r * d];
            for (size_t c = 0; c < d; ++c) w[c] += vr * row[c];
        }
        for (size_t r = j; r < d; ++r) {
            const double f = scale[j] * reflectors[r * d + j];
            double* row = &q[r * d];
            for (size_t c = 0; c < d; ++c) row[c] -= f * w[c];
        }
    }
    std::vector<float> out(d * d);
    for (size_t i = 0; i < d * d; ++i) out[i] = static_cast<float>(q[i]);
    return out;
}

// Which rotation the pruner builds (reference pdx/adsampling.h:52-85).
enum RotationKind : int {
    kRotationDense = 0,        // Q of a Gaussian matrix: reference builds without FFTW
    kRotationDctPow2Only = 1,  // DCT when d >= 512 and d is a power of two: FFTW builds with AVX2
    kRotationDct = 2           // DCT when d >= 512: FFTW builds without AVX2
};

inline bool UsesDctRotation(const int kind, const size_t d) {
    if (kind == kRotationDense || d < D_THRESHOLD_FOR_DCT_ROTATION) return false;
    if (kind == kRotationDctPow2Only) return (d & (d - 1)) == 0;
    return true;
}

// Sign flip followed by the orthonormal DCT-II, as one matrix (pdx/adsampling.h:60-71,162-189):
// Q[k][j] = sign_j * c_k * cos(pi * (j + 1/2) * k / d), c_0 = sqrt(1/d), c_k = sqrt(2/d);
// sign_j = +1 where std::uniform_int_distribution<int>(0, 1) over std::mt19937(seed) draws 1.
// FFTW's REDFT10 returns 2 * sum_j x_j cos(...); the reference scales bin 0 by sqrt(1/(4d)) and the
// others by sqrt(1/(2d)), which gives the c_k above.
inline std::vector<float> DctRotationMatrix(const size_t d, const uint32_t seed) {
    std::mt19937 gen(seed);
    std::uniform_int_distribution<int> dist(0, 1);
    std::vector<double> sign(d);
    for (size_t j = 0; j < d; ++j) sign[j] = dist(gen) ? 1.0 : -1.0;
    const double pi = 3.14159265358979323846;
    const double c0 = std::sqrt(1.0 / static_cast<double>(d)), c = std::sqrt(2.0 / static_cast<double>(d));
    std::vector<float> out(d * d);
    for (size_t k = 0; k < d; ++k) {
        for (size_t j = 0; j < d; ++j) {
            // (2j + 1) * k reduced modulo 4d keeps the cosine argument small and exact for large d
            const size_t m = ((2 * j + 1) * k) % (4 * d);
            const double v = std::cos(pi * static_cast<double>(m) / (2.0 * static_cast<double>(d)));
            out[k * d + j] = static_cast<float>(sign[j] * (k == 0 ? c0 : c) * v);
        }
    }
    return out;
}

} // namespace detail

template <Quantization q = Quantization::f32>
class ADSamplingPruner {
  public:
    uint32_t num_dimensions;
    std::vector<float> ratios;  // ratios[v]: factor applied to the best distance after v dimensions
    // Below this the factorisation is a few milliseconds on the host and the device's launches cost as much.
    static constexpr size_t DEVICE_FACTORISATION_MIN_D = 384;

    // Draws d*d N(0,1) values row by row from std::mt19937(seed) through
    // std::normal_distribution<float> (the reference's sequence, pdx/adsampling.h:76-82) and keeps
    // the orthogonal factor of their QR decomposition.
    // With a DCT rotation kind that applies to this d, the matrix is the sign flip + DCT-II instead.
    ADSamplingPruner(skm_ctx* ctx, uint32_t num_dimensions_, float epsilon0_, uint32_t seed = 42,
                     int rotation_kind = detail::kRotationDense)
        : num_dimensions(num_dimensions_), ctx_(ctx), epsilon0(epsilon0_) {
        InitializeRatios();
        const size_t d = num_dimensions;
        if (detail::UsesDctRotation(rotation_kind, d)) {
            matrix_ = detail::DctRotationMatrix(d, seed);
        } else {
            std::mt19937 gen(seed);
            std::normal_distribution<float> dist(0.0f, 1.0f);
            std::vector<double> a(d * d);
            for (size_t i = 0; i < d * d; ++i) a[i] = dist(gen);
            if (d >= DEVICE_FACTORISATION_MIN_D && d <= SKM_HOUSEHOLDER_Q_MAX_D) {
                // same operations in the same order on the device: the matrix is the host routine's, bit for bit,
                // in a fraction of the time at d = 1024
                matrix_.resize(d * d);
                hip::Check(skm_householder_q(ctx_, a.data(), d, matrix_.data()));
            } else {
                matrix_ = detail::OrthogonalFactor(std::move(a), d);
            }
        }
        d_q_.Reset(ctx_, d * d);
        d_qt_.Reset(ctx_, d * d);
        d_q_.Upload(matrix_.data(), d * d);
        hip::Check(skm_transpose(ctx_, d_q_.get(), d, d, d_qt_.get()));
    }

    void InitializeRatios() {
        ratios.resize(num_dimensions + 1);
        for (size_t v = 0; v <= num_dimensions; ++v) ratios[v] = GetRatio(v);
        d_ratios_.Reset(ctx_, ratios.size());
        d_ratios_.Upload(ratios.data(), ratios.size());
    }

    void SetEpsilon0(float eps0) {
        epsilon0 = eps0;
        InitializeRatios();
    }

    // out = vectors . Q^T, both device-resident (n x d), queued on `on` (objects that share these tables each
    // rotate on their own context).
    void Rotate(skm_ctx* on, const float* d_vectors, float* d_out, const size_t n) const {
        hip::Check(skm_rotate(on, d_vectors, n, num_dimensions, d_q_.get(), d_out));
    }
    // out = rotated . Q, both device-resident.
    void Unrotate(skm_ctx* on, const float* d_rotated, float* d_out, const size_t n) const {
        hip::Check(skm_unrotate(on, d_rotated, n, num_dimensions, d_qt_.get(), d_out));
    }
    float Epsilon0() const { return epsilon0; }

    const float* DeviceRatios() const { return d_ratios_.get(); }
    const std::vector<float>& HostMatrix() const { return matrix_; }

    // (v / d) * (1 + eps0 / sqrt(v))^2 in double, 1 at v = 0 and v = d (pdx/adsampling.h:315-327).
    float GetRatio(const size_t visited_dimensions) const {
        if (visited_dimensions == 0 || visited_dimensions == num_dimensions) return 1.0f;
        const double v = static_cast<double>(visited_dimensions);
        const double slack = 1.0 + epsilon0 / std::sqrt(v);
        return static_cast<float>(v / static_cast<double>(num_dimensions) * slack * slack);
    }

  private:
    skm_ctx* ctx_;
    float epsilon0;
    std::vector<float> matrix_;
    hip::Buffer<float> d_q_, d_qt_, d_ratios_;
};

} // namespace skmeans
