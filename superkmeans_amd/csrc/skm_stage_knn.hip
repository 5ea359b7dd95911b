// k nearest rows of y for every row of x, and the recall count built on it: the two routines behind
// training with queries (reference: batch_computers.h:191-274, superkmeans.h:1044-1087).
#include <algorithm>
#include <vector>

#include "skm_internal.h"

namespace skm {

namespace {

constexpr int KNN_THREADS = 256;
constexpr int KNN_MAX_K = 1024;            // list entries kept in LDS next to one batch of 1024 candidates
constexpr int KNN_LDS_KEYS = 2 * 1024;

// (distance, index) pairs ordered like std::pair<float, uint32_t>: the float is mapped to an unsigned
// integer with the same order, the index breaks ties.  -0.0f cannot occur (see the clamp below).
__device__ __forceinline__ unsigned long long knn_key(float dist, uint32_t idx) {
    const uint32_t b = __float_as_uint(dist);
    const uint32_t o = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return ((unsigned long long) o << 32) | idx;
}
__device__ __forceinline__ float knn_key_dist(unsigned long long key) {
    const uint32_t o = (uint32_t) (key >> 32);
    const uint32_t b = (o & 0x80000000u) ? (o & 0x7fffffffu) : ~o;
    return __uint_as_float(b);
}
__device__ __forceinline__ bool knn_key_negative(unsigned long long key) { return (key >> 63) == 0ull; }

// Ascending bitonic sort of keys[0, P), P a power of two, by the whole workgroup.
__device__ void knn_sort(unsigned long long* keys, int P) {
    for (int size = 2; size <= P; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int t = threadIdx.x; t < (P >> 1); t += KNN_THREADS) {
                const int i = 2 * t - (t & (stride - 1));
                const int j = i + stride;
                const bool up = (i & size) == 0;
                const unsigned long long a = keys[i], b = keys[j];
                if ((a > b) == up) {
                    keys[i] = b;
                    keys[j] = a;
                }
            }
            __syncthreads();
        }
    }
}

__device__ __forceinline__ int knn_pow2_at_least(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

// One workgroup per row of x.  `dist` holds that row's distances to `n_cols` consecutive rows of y whose
// first global index is `col0` (a multiple of 1024).  The row's current list (k entries, unfilled ones
// are {FLT_MAX, 0xffffffff}) is merged with one batch of 1024 columns after the other, which is the order
// the reference processes them in: previous entries take part with their clamped distance, the batch
// with raw distances, the k smallest (distance, index) pairs survive and are clamped at zero afterwards.
// A batch none of whose columns beats the current k-th entry leaves the list as a re-sort would.
__global__ __launch_bounds__(KNN_THREADS) void knn_merge_kernel(
    const float* __restrict__ dist, int64_t ld, int n_cols, uint32_t col0, int k, uint32_t* __restrict__ out_idx,
    float* __restrict__ out_dist
) {
    __shared__ unsigned long long keys[KNN_LDS_KEYS];
    __shared__ int s_count;
    __shared__ int s_dirty;
    const int q = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const float* row = dist + (int64_t) q * ld;
    for (int t = tid; t < k; t += KNN_THREADS) keys[t] = knn_key(out_dist[(int64_t) q * k + t], out_idx[(int64_t) q * k + t]);
    if (tid == 0) {
        s_dirty = 1;  // the stored list may hold clamped entries that are out of order
        s_count = 0;
    }
    __syncthreads();
    const int Pk = knn_pow2_at_least(k);

    for (int b0 = 0; b0 < n_cols; b0 += 1024) {
        const int nb = min(1024, n_cols - b0);
        if (s_dirty) {  // uniform: written before the last barrier
            __syncthreads();
            for (int t = k + tid; t < Pk; t += KNN_THREADS) keys[t] = ~0ull;
            if (tid == 0) s_dirty = 0;
            __syncthreads();
            knn_sort(keys, Pk);
        }
        const unsigned long long tau = keys[k - 1];
        __syncthreads();  // everyone holds tau before the tail of the array is overwritten
        // Columns of this batch that beat the current k-th entry, appended in any order.
        for (int c = tid; c < 1024; c += KNN_THREADS) {
            const bool in = c < nb;
            const unsigned long long key = in ? knn_key(row[b0 + c], col0 + (uint32_t) (b0 + c)) : ~0ull;
            const bool pass = in && key < tau;
            const unsigned long long mask = __ballot(pass);
            int base = 0;
            if (lane == 0 && mask) base = atomicAdd(&s_count, (int) __popcll(mask));
            base = __shfl(base, 0);
            if (pass) keys[k + base + (int) __popcll(mask & ((1ull << lane) - 1ull))] = key;
        }
        __syncthreads();
        const int m = s_count;
        __syncthreads();
        if (tid == 0) s_count = 0;
        if (m == 0) continue;
        const int P = knn_pow2_at_least(k + m);
        for (int t = k + m + tid; t < P; t += KNN_THREADS) keys[t] = ~0ull;
        __syncthreads();
        knn_sort(keys, P);
        // Clamp at zero (batch_computers.h:262): order is kept as sorted, the next batch sorts again.
        bool clamped = false;
        for (int t = tid; t < k; t += KNN_THREADS) {
            const unsigned long long key = keys[t];
            if (knn_key_negative(key)) {
                keys[t] = knn_key(0.0f, (uint32_t) key);
                clamped = true;
            }
        }
        if (clamped) s_dirty = 1;
        __syncthreads();
    }
    for (int t = tid; t < k; t += KNN_THREADS) {
        const unsigned long long key = keys[t];
        out_dist[(int64_t) q * k + t] = knn_key_dist(key);
        out_idx[(int64_t) q * k + t] = (uint32_t) key;
    }
}

// hits[q] = number of the row's ground-truth neighbours whose cluster is among the row's promising
// centroids (superkmeans.h:1064-1082).  Unfilled ground-truth slots (0xffffffff) count as misses.
__global__ __launch_bounds__(KNN_THREADS) void recall_hits_kernel(
    const uint32_t* __restrict__ gt, const uint32_t* __restrict__ promising, const uint32_t* __restrict__ assignments,
    uint32_t n_assignments, int objective_k, int explore, uint32_t* __restrict__ hits
) {
    extern __shared__ uint32_t s_list[];
    __shared__ uint32_t s_hits;
    const int q = blockIdx.x;
    for (int t = threadIdx.x; t < explore; t += KNN_THREADS) s_list[t] = promising[(int64_t) q * explore + t];
    if (threadIdx.x == 0) s_hits = 0;
    __syncthreads();
    uint32_t mine = 0;
    for (int j = threadIdx.x; j < objective_k; j += KNN_THREADS) {
        const uint32_t g = gt[(int64_t) q * objective_k + j];
        if (g >= n_assignments) continue;
        const uint32_t a = assignments[g];
        bool found = false;
        for (int t = 0; t < explore && !found; ++t) found = s_list[t] == a;
        mine += found ? 1u : 0u;
    }
    if (mine) atomicAdd(&s_hits, mine);
    __syncthreads();
    if (threadIdx.x == 0) hits[q] = s_hits;
}

} // namespace

} // namespace skm

using namespace skm;

extern "C" {

int skm_knn(skm_ctx* ctx, const float* d_x, size_t n_x, const float* d_y, size_t n_y, size_t d, const float* d_xnorm,
            const float* d_ynorm, size_t k, uint32_t* d_out_idx, float* d_out_dist) {
    SKM_REQUIRE(ctx, "null context");
    SKM_REQUIRE(k > 0 && k <= (size_t) KNN_MAX_K, "k must be in [1, 1024]");
    if (n_x == 0) return SKM_OK;
    SKM_REQUIRE(d_out_idx && d_out_dist, "null pointer");
    SKM_REQUIRE(n_x <= 0x7fffffffULL && n_y <= 0xfffffffeULL, "n_x or n_y out of range");
    SKM_REQUIRE(d > 0 && d <= (1u << 20), "d out of range");
    ScopedStage outer(ctx, "knn");
    // Lists start unfilled: {FLT_MAX, 0xffffffff} (batch_computers.h:204-205).
    SKM_TRY(skm_fill_u32(ctx, d_out_dist, 0x7f7fffffu, n_x * k));
    SKM_TRY(skm_fill_u32(ctx, d_out_idx, 0xffffffffu, n_x * k));
    if (n_y == 0) return SKM_OK;
    SKM_REQUIRE(d_x && d_y && d_xnorm && d_ynorm, "null pointer");
    // Columns per chunk: whole batches of 1024, as many as the workspace allows.
    size_t chunk = ctx->workspace_limit / (n_x * sizeof(float));
    chunk = std::max<size_t>(1024, (chunk / 1024) * 1024);
    chunk = std::min<size_t>(chunk, size_t(1) << 30);
    chunk = std::min(chunk, ((n_y + 1023) / 1024) * 1024);
    void* scratch = nullptr;
    SKM_TRY(workspace(ctx, 0, n_x * chunk * sizeof(float), &scratch));
    float* d_dist = (float*) scratch;
    for (size_t j0 = 0; j0 < n_y; j0 += chunk) {
        const size_t m = std::min(chunk, n_y - j0);
        {
            ScopedStage st(ctx, "knn/blas");
            SKM_TRY(launch_gemm_store(ctx, d_x, (int) n_x, (int64_t) d, d_y + j0 * d, (int) m, (int64_t) d, (int) d,
                                      d_dist, (int64_t) chunk, d_xnorm, d_ynorm + j0));
        }
        {
            ScopedStage st(ctx, "knn/select");
            hipLaunchKernelGGL(knn_merge_kernel, dim3((unsigned) n_x), dim3(KNN_THREADS), 0, ctx->stream, d_dist,
                               (int64_t) chunk, (int) m, (uint32_t) j0, (int) k, d_out_idx, d_out_dist);
            SKM_HIP_TRY(hipGetLastError());
        }
    }
    return SKM_OK;
}

int skm_recall_hits(skm_ctx* ctx, const uint32_t* d_gt, const uint32_t* d_promising, const uint32_t* d_assignments,
                    size_t n_assignments, size_t n_queries, size_t objective_k, size_t explore, uint32_t* h_out_hits) {
    SKM_REQUIRE(ctx, "null context");
    if (n_queries == 0) return SKM_OK;
    SKM_REQUIRE(d_gt && d_promising && d_assignments && h_out_hits, "null pointer");
    SKM_REQUIRE(objective_k > 0 && objective_k <= 0x7fffffffULL, "objective_k out of range");
    SKM_REQUIRE(explore > 0 && explore <= (size_t) KNN_MAX_K, "explore must be in [1, 1024]");
    SKM_REQUIRE(n_queries <= 0x7fffffffULL && n_assignments <= 0xffffffffULL, "sizes out of range");
    ScopedStage st(ctx, "recall");
    void* scratch = nullptr;
    SKM_TRY(workspace(ctx, 1, n_queries * sizeof(uint32_t), &scratch));
    uint32_t* d_hits = (uint32_t*) scratch;
    hipLaunchKernelGGL(recall_hits_kernel, dim3((unsigned) n_queries), dim3(KNN_THREADS), explore * sizeof(uint32_t),
                       ctx->stream, d_gt, d_promising, d_assignments, (uint32_t) n_assignments, (int) objective_k,
                       (int) explore, d_hits);
    SKM_HIP_TRY(hipGetLastError());
    SKM_HIP_TRY(hipMemcpyAsync(h_out_hits, d_hits, n_queries * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SKM_OK;
}

} // extern "C"
