// Synthetic Gaussian-mixture embeddings generated directly in device memory, for benchmarks and
// large-shape tests (the reference's generator for its own tests is MakeBlobs, pdx/utils.h:74-123,
// which fills host memory with std::mt19937 draws).  A counter-based generator is used instead so
// that any element can be produced independently: value(i, j) depends only on (seed, i, j).
#include "skm_internal.h"

namespace skm {

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

__device__ __forceinline__ uint32_t hash3(uint32_t seed, uint32_t a, uint32_t b) {
    return mix32(mix32(mix32(seed ^ 0x9e3779b9u) + a) * 0x85ebca6bu + b);
}

// Standard normal from two hashed uniforms (Box-Muller).
__device__ __forceinline__ float gauss(uint32_t seed, uint32_t a, uint32_t b) {
    const uint32_t h1 = hash3(seed, a, b), h2 = hash3(seed ^ 0x68bc21ebu, b, a);
    const float u1 = ((float) (h1 >> 8) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
    const float u2 = (float) (h2 >> 8) * (1.0f / 16777216.0f);           // [0, 1)
    return sqrtf(-2.0f * __logf(u1)) * __cosf(6.28318530718f * u2);
}

struct SynthArgs {
    float* out;
    size_t n, d;
    uint32_t n_centers, center_seed, point_seed;
    float center_sigma, noise_sigma, decay_exponent;
    int normalize;
    size_t row_offset;  // logical index of out's first row (rows are a pure function of their index)
};

// One wavefront per row: x[j] = s_j * (center_sigma * g_c(u, j) + noise_sigma * g_p(i, j)),
// s_j = (j + 1)^(-decay_exponent), u = hash(i) mod n_centers; optionally scaled to unit L2 norm.
__global__ __launch_bounds__(256) void synth_mixture_kernel(SynthArgs a) {
    const int lane = threadIdx.x & 63;
    const size_t r = (size_t) blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= a.n) return;
    const size_t i = a.row_offset + r;
    const uint32_t ilo = (uint32_t) i, ihi = (uint32_t) (i >> 32);
    const uint32_t u = a.n_centers ? hash3(a.point_seed ^ 0x51ed270bu, ilo, ihi) % a.n_centers : 0u;
    float* row = a.out + r * a.d;
    float ss = 0.0f;
    for (size_t j = lane; j < a.d; j += 64) {
        const float s = a.decay_exponent == 0.0f ? 1.0f : __powf((float) (j + 1), -a.decay_exponent);
        float v = a.noise_sigma * gauss(a.point_seed + ihi * 0x27d4eb2fu, ilo, (uint32_t) j);
        if (a.n_centers) v += a.center_sigma * gauss(a.center_seed, u, (uint32_t) j);
        v *= s;
        row[j] = v;
        ss += v * v;
    }
    if (a.normalize) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
        const float inv = ss > 0.0f ? 1.0f / sqrtf(ss) : 0.0f;
        for (size_t j = lane; j < a.d; j += 64) row[j] *= inv;
    }
}

// Two-level mixture: fine centre u belongs to coarse centre u / (n_fine / n_coarse);
// x[j] = g_coarse(u / group, j) + fine_sigma * g_fine(u, j) + noise_sigma * g_point(i, j), normalised.
struct SynthTwoLevelArgs {
    float* out;
    size_t n, d, row_offset;
    uint32_t n_coarse, n_fine, seed;
    float fine_sigma, noise_sigma;
};

__global__ __launch_bounds__(256) void synth_two_level_kernel(SynthTwoLevelArgs a) {
    const int lane = threadIdx.x & 63;
    const size_t r = (size_t) blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= a.n) return;
    const size_t i = a.row_offset + r;
    const uint32_t ilo = (uint32_t) i, ihi = (uint32_t) (i >> 32);
    const uint32_t u = hash3(a.seed ^ 0x51ed270bu, ilo, ihi) % a.n_fine;
    const uint32_t group = a.n_fine / a.n_coarse;
    const uint32_t cu = u / (group ? group : 1u);
    float* row = a.out + r * a.d;
    float ss = 0.0f;
    for (size_t j = lane; j < a.d; j += 64) {
        const float v = gauss(a.seed + 1u, cu, (uint32_t) j) + a.fine_sigma * gauss(a.seed + 2u, u, (uint32_t) j) +
                        a.noise_sigma * gauss(a.seed + 3u + ihi * 0x27d4eb2fu, ilo, (uint32_t) j);
        row[j] = v;
        ss += v * v;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
    const float inv = ss > 0.0f ? 1.0f / sqrtf(ss) : 0.0f;
    for (size_t j = lane; j < a.d; j += 64) row[j] *= inv;
}

// Low intrinsic dimension with heavy tails: x = A z + noise_scale * t3, z ~ N(0, I_rank), A a fixed
// d x rank Gaussian map (a pure function of the seed), t3 Student-t with 3 degrees of freedom
// (normal / sqrt(chi2_3 / 3)); rows normalised.  One workgroup per row; z is staged in LDS.
struct SynthLowRankArgs {
    float* out;
    size_t n, d, row_offset;
    uint32_t rank, seed;
    float noise_scale;
};

__global__ __launch_bounds__(256) void synth_low_rank_kernel(SynthLowRankArgs a) {
    __shared__ float z[256];
    __shared__ float red[4];
    const size_t r = blockIdx.x;
    const size_t i = a.row_offset + r;
    const uint32_t ilo = (uint32_t) i, ihi = (uint32_t) (i >> 32);
    if (threadIdx.x < a.rank) z[threadIdx.x] = gauss(a.seed + 11u + ihi * 0x27d4eb2fu, ilo, threadIdx.x);
    __syncthreads();
    float* row = a.out + r * a.d;
    float ss = 0.0f;
    for (size_t j = threadIdx.x; j < a.d; j += 256) {
        float v = 0.0f;
        for (uint32_t q = 0; q < a.rank; ++q) v += gauss(a.seed + 12u, (uint32_t) j, q) * z[q];
        const uint32_t ps = a.seed + 13u + ihi * 0x27d4eb2fu;
        const float g0 = gauss(ps, ilo, (uint32_t) (4 * j)), g1 = gauss(ps, ilo, (uint32_t) (4 * j + 1));
        const float g2 = gauss(ps, ilo, (uint32_t) (4 * j + 2)), g3 = gauss(ps, ilo, (uint32_t) (4 * j + 3));
        const float chi = (g1 * g1 + g2 * g2 + g3 * g3) * (1.0f / 3.0f);
        v += a.noise_scale * g0 / sqrtf(fmaxf(chi, 1e-12f));
        row[j] = v;
        ss += v * v;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float tot = red[0] + red[1] + red[2] + red[3];
    const float inv = tot > 0.0f ? 1.0f / sqrtf(tot) : 0.0f;
    for (size_t j = threadIdx.x; j < a.d; j += 256) row[j] *= inv;
}

} // namespace skm

using namespace skm;

extern "C" int skm_synth_two_level_mixture(skm_ctx* ctx, float* d_out, size_t n, size_t d, size_t row_offset,
                                           uint32_t n_coarse, uint32_t n_fine, uint32_t seed, float fine_sigma,
                                           float noise_sigma) {
    SKM_REQUIRE(ctx, "null context");
    if (n == 0) return SKM_OK;
    SKM_REQUIRE(d_out && d > 0, "null output or zero d");
    SKM_REQUIRE(n_coarse > 0 && n_fine >= n_coarse, "need 0 < n_coarse <= n_fine");
    SKM_REQUIRE(n <= 0x7fffffffULL * 4, "too many rows");
    SynthTwoLevelArgs a;
    a.out = d_out; a.n = n; a.d = d; a.row_offset = row_offset; a.n_coarse = n_coarse; a.n_fine = n_fine; a.seed = seed;
    a.fine_sigma = fine_sigma; a.noise_sigma = noise_sigma;
    hipLaunchKernelGGL(synth_two_level_kernel, dim3((unsigned) ((n + 3) / 4)), dim3(256), 0, ctx->stream, a);
    return check_hip(hipGetLastError(), "synth_two_level_kernel launch");
}

extern "C" int skm_synth_low_rank(skm_ctx* ctx, float* d_out, size_t n, size_t d, size_t row_offset, uint32_t rank,
                                  uint32_t seed, float noise_scale) {
    SKM_REQUIRE(ctx, "null context");
    if (n == 0) return SKM_OK;
    SKM_REQUIRE(d_out && d > 0, "null output or zero d");
    SKM_REQUIRE(rank > 0 && rank <= 256, "rank must be in [1, 256]");
    SKM_REQUIRE(n <= 0x7fffffffULL, "too many rows");
    SynthLowRankArgs a;
    a.out = d_out; a.n = n; a.d = d; a.row_offset = row_offset; a.rank = rank; a.seed = seed; a.noise_scale = noise_scale;
    hipLaunchKernelGGL(synth_low_rank_kernel, dim3((unsigned) n), dim3(256), 0, ctx->stream, a);
    return check_hip(hipGetLastError(), "synth_low_rank_kernel launch");
}

extern "C" int skm_synth_gaussian_mixture(skm_ctx* ctx, float* d_out, size_t n, size_t d, size_t row_offset,
                                          uint32_t n_centers, uint32_t center_seed, uint32_t point_seed,
                                          float center_sigma, float noise_sigma, float decay_exponent, int normalize) {
    SKM_REQUIRE(ctx, "null context");
    if (n == 0) return SKM_OK;
    SKM_REQUIRE(d_out && d > 0, "null output or zero d");
    SKM_REQUIRE(n <= 0x7fffffffULL * 4, "too many rows");
    SynthArgs a;
    a.out = d_out; a.n = n; a.d = d; a.n_centers = n_centers; a.center_seed = center_seed; a.point_seed = point_seed;
    a.center_sigma = center_sigma; a.noise_sigma = noise_sigma; a.decay_exponent = decay_exponent;
    a.normalize = normalize; a.row_offset = row_offset;
    hipLaunchKernelGGL(synth_mixture_kernel, dim3((unsigned) ((n + 3) / 4)), dim3(256), 0, ctx->stream, a);
    return check_hip(hipGetLastError(), "synth_mixture_kernel launch");
}
