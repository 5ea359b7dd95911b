// CPU ORACLE -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// Rotation matrix of the ADSampling pruner (reference pdx/adsampling.h:76-85): d*d draws from
// std::normal_distribution<float>(0,1) over std::mt19937(seed), row by row, then the orthogonal factor
// of their Householder QR.  The reference takes that factor from Eigen::HouseholderQR, which is not
// available; this is a textbook Householder QR in double precision (PARITY UNPINNED: no reference test
// fixes the entries of Q, only its orthogonality).
//
// This file is compiled with -ffp-contract=off: the draws (x*x + y*y inside the polar method of
// libstdc++) and the factorisation must not depend on whether a compiler fuses multiply-adds, because
// the HIP backend builds the same matrix with another compiler and the two must agree bit for bit.
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <random>
#include <vector>

namespace oracle {

static void HouseholderQ(std::vector<double>& a, size_t d, std::vector<float>& q_out) {
    // a: d x d row-major, overwritten. vs[j] holds the j-th reflector (length d - j), betas[j] its factor.
    std::vector<std::vector<double>> vs(d);
    std::vector<double> betas(d, 0.0);
    std::vector<double> w(d);
    for (size_t j = 0; j < d; ++j) {
        const size_t len = d - j;
        std::vector<double>& v = vs[j];
        v.resize(len);
        double norm2 = 0.0;
        for (size_t r = 0; r < len; ++r) {
            v[r] = a[(j + r) * d + j];
            norm2 += v[r] * v[r];
        }
        const double norm = std::sqrt(norm2);
        if (norm == 0.0) {
            betas[j] = 0.0;
            continue;
        }
        const double alpha = (v[0] >= 0.0) ? -norm : norm;
        v[0] -= alpha;
        double vtv = 0.0;
        for (size_t r = 0; r < len; ++r) vtv += v[r] * v[r];
        if (vtv == 0.0) {
            betas[j] = 0.0;
            continue;
        }
        const double beta = 2.0 / vtv;
        betas[j] = beta;
        // A[j:, j:] -= beta * v * (v^T A[j:, j:])
        for (size_t c = j; c < d; ++c) w[c] = 0.0;
        for (size_t r = 0; r < len; ++r) {
            const double vr = v[r];
            const double* row = &a[(j + r) * d];
            for (size_t c = j; c < d; ++c) w[c] += vr * row[c];
        }
        for (size_t r = 0; r < len; ++r) {
            const double f = beta * v[r];
            double* row = &a[(j + r) * d];
            for (size_t c = j; c < d; ++c) row[c] -= f * w[c];
        }
    }
    // Q = H_0 H_1 ... H_{d-1} * I
    std::vector<double> q(d * d, 0.0);
    for (size_t i = 0; i < d; ++i) q[i * d + i] = 1.0;
    for (size_t jj = d; jj-- > 0;) {
        if (betas[jj] == 0.0) continue;
        const std::vector<double>& v = vs[jj];
        const size_t len = d - jj;
        for (size_t c = 0; c < d; ++c) w[c] = 0.0;
        for (size_t r = 0; r < len; ++r) {
            const double vr = v[r];
            const double* row = &q[(jj + r) * d];
            for (size_t c = 0; c < d; ++c) w[c] += vr * row[c];
        }
        for (size_t r = 0; r < len; ++r) {
            const double f = betas[jj] * v[r];
            double* row = &q[(jj + r) * d];
            for (size_t c = 0; c < d; ++c) row[c] -= f * w[c];
        }
    }
    q_out.resize(d * d);
    for (size_t i = 0; i < d * d; ++i) q_out[i] = static_cast<float>(q[i]);
}

void MakeRotationMatrix(uint32_t d, uint32_t seed, std::vector<float>& out) {
    std::mt19937 gen(seed);
    std::vector<double> a((size_t) d * d);
    std::normal_distribution<float> dist(0.0f, 1.0f);
    for (uint32_t i = 0; i < d; ++i)
        for (uint32_t j = 0; j < d; ++j) a[(size_t) i * d + j] = dist(gen);
    HouseholderQ(a, d, out);
}

} // namespace oracle
