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

} // namespace skm

using namespace skm;

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
