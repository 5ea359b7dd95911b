// Orthogonal factor of a Householder QR in double precision on the device.
//
// The ADSampling rotation is the Q of the QR factorisation of a d x d Gaussian matrix (reference
// pdx/adsampling.h:76-85, Eigen's HouseholderQR).  On one host core the factorisation takes 0.3 s at d = 1024 and
// 0.9 s at d = 1536, as long as a whole Train on the device.  The kernels below perform exactly the operations of
// skmeans::detail::OrthogonalFactor (include/superkmeans/pdx/adsampling.h), every sum in the same order and
// without fused multiply-adds (this file is compiled with -ffp-contract=off), so the float matrix that comes out
// is the one the host routine returns: which of the two ran is not observable.
//
// Per reflector j: one workgroup builds the reflector from column j (sums over the column are taken by a single
// thread, in row order); then every group of 16 (or 8) columns is updated by one workgroup that holds rows j..d-1
// of its columns in LDS: one read of the block with every thread's loads in flight together, the dot product of
// each column with the reflector accumulated by one thread in row order, the rank-one update element-wise, one
// write.  The launches are short (a few microseconds); the chain of 3 d of them is what the factorisation costs.
#include "skm_internal.h"

#include <algorithm>

namespace skm {

constexpr int QR_THREADS = 256;
constexpr size_t QR_LDS_BYTES = 160 * 1024;

// reflectors[j * d + r], r >= j: reflector j (contiguous); scale[j] = 2 / (v . v), 0 when the column is already zero.
__global__ __launch_bounds__(QR_THREADS) void qr_reflector_kernel(const double* __restrict__ a, size_t d, size_t j,
                                                                   double* __restrict__ reflectors, double* __restrict__ scale) {
    extern __shared__ double col[];  // 2 d doubles: the column and its squares
    for (size_t r = j + threadIdx.x; r < d; r += QR_THREADS) col[r] = a[r * d + j];
    __syncthreads();
    // squares by all threads, their sum by one thread in row order (reads unrolled so that only the additions
    // form a chain)
    double* square = col + d;
    for (size_t r = j + threadIdx.x; r < d; r += QR_THREADS) square[r] = col[r] * col[r];
    __syncthreads();
    const auto ordered_sum = [&]() {
        double sum = 0.0;
        size_t r = j;
        for (; r + 16 <= d; r += 16) {
            double p[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) p[u] = square[r + u];
#pragma unroll
            for (int u = 0; u < 16; ++u) sum += p[u];
        }
        for (; r < d; ++r) sum += square[r];
        return sum;
    };
    if (threadIdx.x == 0) {
        const double norm2 = ordered_sum();
        const double norm = sqrt(norm2);
        double s = 0.0;
        if (norm != 0.0) {
            const double head = col[j];
            const double alpha = (head >= 0.0) ? -norm : norm;
            col[j] = head - alpha;
            square[j] = col[j] * col[j];
            const double vtv = ordered_sum();
            if (vtv != 0.0) s = 2.0 / vtv;
        }
        scale[j] = s;
    }
    __syncthreads();
    for (size_t r = j + threadIdx.x; r < d; r += QR_THREADS) reflectors[j * d + r] = col[r];
}

// m[r][c] -= (scale_j v_r) * (sum_r v_r m[r][c]) for rows j..d-1 and the columns [first_col, d) of this workgroup's
// group of COLS columns.
template <int COLS>
__global__ __launch_bounds__(QR_THREADS) void qr_apply_kernel(double* __restrict__ m, size_t d, size_t j, size_t first_col,
                                                               const double* __restrict__ reflectors,
                                                               const double* __restrict__ scale) {
    const double s = scale[j];
    if (s == 0.0) return;  // uniform over the grid
    extern __shared__ double lds[];
    const size_t rows = d - j;
    double* v = lds;                 // rows
    double* block = lds + rows;      // rows x COLS
    double* w = block + rows * COLS; // COLS
    const size_t c_base = (first_col / COLS + blockIdx.x) * COLS;
    for (size_t r = threadIdx.x; r < rows; r += QR_THREADS) v[r] = reflectors[j * d + j + r];
    // the block, 16 loads in flight per thread; columns outside [first_col, d) read a valid neighbour and are never
    // written back
    const size_t elements = rows * COLS;
    constexpr int BATCH = 16;
    for (size_t e0 = threadIdx.x; e0 < elements; e0 += (size_t) QR_THREADS * BATCH) {
        double tmp[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            size_t e = e0 + (size_t) u * QR_THREADS;
            e = e < elements ? e : elements - 1;
            size_t c = c_base + e % COLS;
            c = c < d ? c : d - 1;
            tmp[u] = m[(j + e / COLS) * d + c];
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const size_t e = e0 + (size_t) u * QR_THREADS;
            if (e < elements) block[e] = tmp[u];
        }
    }
    __syncthreads();
    if (threadIdx.x < COLS) {
        double acc = 0.0;
        size_t r = 0;
        for (; r + 16 <= rows; r += 16) {
            double p[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) p[u] = v[r + u] * block[(r + u) * COLS + threadIdx.x];
#pragma unroll
            for (int u = 0; u < 16; ++u) acc += p[u];
        }
        for (; r < rows; ++r) {
            const double p = v[r] * block[r * COLS + threadIdx.x];
            acc += p;
        }
        w[threadIdx.x] = acc;
    }
    __syncthreads();
    for (size_t e = threadIdx.x; e < elements; e += QR_THREADS) {
        const size_t r = e / COLS, c = c_base + e % COLS;
        if (c >= d || c < first_col) continue;
        const double f = s * v[r];
        const double p = f * w[e % COLS];
        m[(j + r) * d + c] = block[e] - p;
    }
}

__global__ __launch_bounds__(256) void qr_identity_kernel(double* __restrict__ q, size_t d) {
    const size_t i = (size_t) blockIdx.x * 256 + threadIdx.x;
    if (i < d * d) q[i] = (i / d == i % d) ? 1.0 : 0.0;
}

__global__ __launch_bounds__(256) void qr_narrow_kernel(const double* __restrict__ q, size_t count, float* __restrict__ out) {
    const size_t i = (size_t) blockIdx.x * 256 + threadIdx.x;
    if (i < count) out[i] = (float) q[i];
}

} // namespace skm

using namespace skm;

extern "C" int skm_householder_q(skm_ctx* ctx, const double* h_a, size_t d, float* h_out_q) {
    SKM_REQUIRE(ctx && h_a && h_out_q, "null argument");
    SKM_REQUIRE(d > 0 && d <= SKM_HOUSEHOLDER_Q_MAX_D, "d out of range for the device factorisation");
    SKM_HIP_TRY(hipSetDevice(ctx->device));
    const size_t dd = d * d;
    // a, reflectors, q (double), scale, narrowed output
    void* ws = nullptr;
    SKM_TRY(workspace(ctx, 0, (3 * dd + d) * sizeof(double) + dd * sizeof(float) + 256, &ws));
    double* a = (double*) ws;
    double* reflectors = a + dd;
    double* q = reflectors + dd;
    double* scale = q + dd;
    float* narrowed = (float*) (scale + d);
    SKM_HIP_TRY(hipMemcpyAsync(a, h_a, dd * sizeof(double), hipMemcpyHostToDevice, ctx->stream));
    const unsigned flat_blocks = (unsigned) ((dd + 255) / 256);
    hipLaunchKernelGGL(qr_identity_kernel, dim3(flat_blocks), dim3(256), 0, ctx->stream, q, d);
    SKM_HIP_TRY(hipGetLastError());
    const size_t lds_reflector = 2 * d * sizeof(double);
    // columns per workgroup: the widest group whose rows fit the 160 KB of LDS
    const int cols = (d * (16 + 1) + 16) * sizeof(double) <= QR_LDS_BYTES ? 16 : 8;
    const auto lds_apply = [&](const size_t j) { return ((d - j) * (size_t) (cols + 1) + cols) * sizeof(double); };
    SKM_REQUIRE(lds_apply(0) <= QR_LDS_BYTES, "d too large for the device factorisation");
    SKM_HIP_TRY(hipFuncSetAttribute((const void*) qr_apply_kernel<16>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) QR_LDS_BYTES));
    SKM_HIP_TRY(hipFuncSetAttribute((const void*) qr_apply_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) QR_LDS_BYTES));
    const auto apply = [&](double* m, const size_t j, const size_t first_col) {
        const unsigned blocks = (unsigned) ((d + cols - 1) / cols - first_col / cols);
        if (cols == 16)
            hipLaunchKernelGGL(qr_apply_kernel<16>, dim3(blocks), dim3(QR_THREADS), lds_apply(j), ctx->stream, m, d, j, first_col, reflectors, scale);
        else
            hipLaunchKernelGGL(qr_apply_kernel<8>, dim3(blocks), dim3(QR_THREADS), lds_apply(j), ctx->stream, m, d, j, first_col, reflectors, scale);
        return check_hip(hipGetLastError(), "qr_apply_kernel launch");
    };
    for (size_t j = 0; j < d; ++j) {
        hipLaunchKernelGGL(qr_reflector_kernel, dim3(1), dim3(QR_THREADS), lds_reflector, ctx->stream, a, d, j, reflectors, scale);
        SKM_HIP_TRY(hipGetLastError());
        SKM_TRY(apply(a, j, j));
    }
    for (size_t j = d; j-- > 0;) SKM_TRY(apply(q, j, 0));
    hipLaunchKernelGGL(qr_narrow_kernel, dim3(flat_blocks), dim3(256), 0, ctx->stream, q, dd, narrowed);
    SKM_HIP_TRY(hipGetLastError());
    SKM_HIP_TRY(hipMemcpyAsync(h_out_q, narrowed, dd * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SKM_OK;
}
