// Centroid update without floating-point atomics.
//
// SuperKMeans::UpdateCentroids (reference superkmeans.h:729-765) lets every OpenMP thread scan all
// assignments and accumulate the rows of the centroids it owns, so each centroid's sum is taken in
// ascending point order.  Here the point ids are first sorted by assignment with a stable LSD radix
// sort (integer work only), then one workgroup per centroid walks its segment in that same
// ascending order and accumulates in registers.  The result is run-to-run deterministic and has the
// reference's summation order.
#include "skm_internal.h"

#include <algorithm>
#include <cstring>
#include <unordered_map>
#include <vector>

namespace skm {

constexpr int SORT_THREADS = 256;
// Elements per workgroup and pass.  Smaller tiles give more workgroups (a workgroup is four wavefronts whose rounds are
// separated by barriers, so a compute unit needs several to hide their latencies) but shorter runs of equal digits per
// tile and a longer table of per-tile digit counts.  Measured with a million 14-bit keys (7 + 7 bits), both passes
// together: 4,096 keys per tile 64 us, 2,048 58 us, 1,024 65 us (there the scans of the 977-entry rows take 10 us each).
// A sort of a few ten thousand keys (a fine clustering) is a matter of latency: there the smallest tile is the fastest.
constexpr int SORT_TILE = 2048, SORT_TILE_FEW_KEYS = 1024;  // multiples of the scatter's round of 1,024 elements
constexpr size_t SORT_FEW_KEYS = size_t(1) << 18;
constexpr int RADIX = 256;

// Second step of a radix pass.  The histograms are stored digit-major, so the global base of a (digit, tile) pair is
// (sum of all smaller digits) + (sum of the same digit over the earlier tiles).  One wavefront per digit scans its own
// row of tile counts and leaves the digit's total; the scatter kernel adds the 256 totals up by itself.  The 256 rows
// are scanned side by side instead of one scan over 256 * n_tiles counters by a single workgroup.  A lane owns a
// contiguous piece of the row: it adds the piece up (independent loads), one scan over the 64 lane sums gives the
// piece's base, and a second walk of the piece writes the running bases: one shuffle scan per row, whatever its length.
__global__ __launch_bounds__(64) void digit_rows_scan_kernel(
    const uint32_t* __restrict__ hist, uint32_t n_tiles, uint32_t* __restrict__ bases, uint32_t* __restrict__ totals
) {
    const int lane = threadIdx.x;
    const uint32_t* row = hist + (size_t) blockIdx.x * n_tiles;
    uint32_t* out = bases + (size_t) blockIdx.x * n_tiles;
    const uint32_t piece = (n_tiles + 63) / 64;
    const uint32_t from = min((uint32_t) lane * piece, n_tiles), to = min(from + piece, n_tiles);
    uint32_t sum = 0;
#pragma unroll 8
    for (uint32_t i = from; i < to; ++i) sum += row[i];
    uint32_t incl = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t t = __shfl_up(incl, off);
        if (lane >= off) incl += t;
    }
    uint32_t running = incl - sum;
#pragma unroll 8
    for (uint32_t i = from; i < to; ++i) {
        out[i] = running;
        running += row[i];
    }
    if (lane == 63) totals[blockIdx.x] = incl;
}

// Segment boundaries of the sorted assignment keys: offsets[c] = first position whose key is >= c
// (offsets[k] = number of keys below k), written by the thread that sees the key change.
__global__ __launch_bounds__(256) void segment_bounds_kernel(
    const uint32_t* __restrict__ sorted_keys, size_t n, uint32_t k, uint32_t* __restrict__ offsets
) {
    const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i > n) return;
    // Position n closes the last segment: it behaves like a key equal to k.
    uint32_t key = i < n ? sorted_keys[i] : k;
    key = key < k ? key : k;
    uint32_t first = 0;
    if (i > 0) {
        const uint32_t prev = sorted_keys[i - 1];
        first = (prev < k ? prev : k) + 1;
    }
    for (uint32_t c = first; c <= key; ++c) offsets[c] = (uint32_t) i;
}

// First step of a radix pass: digit histogram of one tile, stored digit-major ([digit][tile]) so that every digit's
// counts over the tiles are one contiguous row for digit_rows_scan_kernel.
__global__ __launch_bounds__(SORT_THREADS) void radix_hist_kernel(
    const uint32_t* __restrict__ keys, size_t n, int shift, uint32_t mask, uint32_t n_tiles, int tile, uint32_t* __restrict__ hist
) {
    __shared__ uint32_t s_hist[RADIX];
    s_hist[threadIdx.x] = 0;
    __syncthreads();
    const size_t t0 = (size_t) blockIdx.x * tile;
    for (int r = 0; r < tile / SORT_THREADS; ++r) {
        const size_t i = t0 + (size_t) r * SORT_THREADS + threadIdx.x;
        if (i < n) atomicAdd(&s_hist[(keys[i] >> shift) & mask], 1u);
    }
    __syncthreads();
    hist[(size_t) threadIdx.x * n_tiles + blockIdx.x] = s_hist[threadIdx.x];
}

// Third step: stable scatter.  The tile is consumed in sub-rounds of 256 consecutive elements; inside a
// sub-round the rank of an element among equal digits is (equal digits in earlier wavefronts) +
// (equal digits in lower lanes of its wavefront), the latter from eight ballots.
__global__ __launch_bounds__(SORT_THREADS) void radix_scatter_kernel(
    const uint32_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, size_t n, int shift, uint32_t mask,
    uint32_t n_tiles, int tile, const uint32_t* __restrict__ bases, const uint32_t* __restrict__ totals,
    uint32_t* __restrict__ keys_out, uint32_t* __restrict__ vals_out, int vals_are_iota,
    uint32_t* __restrict__ offsets_out, uint32_t k
) {
    static_assert(SORT_THREADS == RADIX, "thread t owns digit t");
    __shared__ uint32_t s_base[RADIX];
    __shared__ uint32_t s_wave_cnt[SORT_THREADS / 64][RADIX];
    __shared__ uint32_t s_wave_total[SORT_THREADS / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    {
        // exclusive prefix of the digit totals: 64 digits per wavefront with shuffles, the four partial totals through LDS
        const uint32_t total = totals[tid];
        uint32_t incl = total;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        if (lane == 63) s_wave_total[wave] = incl;
        __syncthreads();
        uint32_t below = incl - total;
        for (int w = 0; w < wave; ++w) below += s_wave_total[w];
        s_base[tid] = below + bases[(size_t) tid * n_tiles + blockIdx.x];
        // A sort of one pass (k <= 256): the digit is the key, so the number of keys below digit c is where the
        // segment of centroid c starts; offsets_out[k] is the number of keys below k.
        if (offsets_out && blockIdx.x == 0) {
            if ((uint32_t) tid <= k) offsets_out[tid] = below;
            if (k == RADIX && tid == 0) offsets_out[RADIX] = (uint32_t) n;
        }
    }
    // Rounds of 4 x 256 consecutive elements: the four sub-rounds of a round share its barriers.  s_wave_cnt[w][digit]
    // holds four byte counters, one per sub-round (a wavefront has at most 64 equal digits in a sub-round).
    constexpr int SUB = 4;
    const size_t t0 = (size_t) blockIdx.x * tile;
    for (int r = 0; r < tile / (SORT_THREADS * SUB); ++r) {
#pragma unroll
        for (int w = 0; w < SORT_THREADS / 64; ++w) s_wave_cnt[w][tid] = 0;
        __syncthreads();
        uint32_t key[SUB], val[SUB], digit[SUB], rank_in_wave[SUB];
        bool in[SUB];
#pragma unroll
        for (int j = 0; j < SUB; ++j) {
            const size_t i = t0 + ((size_t) r * SUB + j) * SORT_THREADS + tid;
            in[j] = i < n;
            key[j] = val[j] = digit[j] = 0;
            if (in[j]) {
                key[j] = keys_in[i];
                val[j] = vals_are_iota ? (uint32_t) i : vals_in[i];
                digit[j] = (key[j] >> shift) & mask;
            }
        }
#pragma unroll
        for (int j = 0; j < SUB; ++j) {
            // Lanes holding the same digit (inactive lanes never match an active one).
            unsigned long long match = __ballot(in[j]);
#pragma unroll
            for (int b = 0; b < 8; ++b) {
                const unsigned long long vote = __ballot(in[j] && ((digit[j] >> b) & 1u));
                match &= ((digit[j] >> b) & 1u) ? vote : ~vote;
            }
            rank_in_wave[j] = (uint32_t) __popcll(match & ((1ull << lane) - 1ull));
            if (in[j] && rank_in_wave[j] == 0) atomicAdd(&s_wave_cnt[wave][digit[j]], (uint32_t) __popcll(match) << (8 * j));
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < SUB; ++j) {
            if (in[j]) {
                // equal digits of the earlier sub-rounds in every wavefront, and of this sub-round in the wavefronts below
                uint32_t before = 0;
#pragma unroll
                for (int w = 0; w < SORT_THREADS / 64; ++w) {
                    const uint32_t c = s_wave_cnt[w][digit[j]];
                    before += __builtin_amdgcn_sad_u8(c & ((1u << (8 * j)) - 1u), 0u, 0u);
                    if (w < wave) before += (c >> (8 * j)) & 0xffu;
                }
                const uint32_t dst = s_base[digit[j]] + before + rank_in_wave[j];
                keys_out[dst] = key[j];
                vals_out[dst] = val[j];
            }
        }
        __syncthreads();
        uint32_t add = 0;
#pragma unroll
        for (int w = 0; w < SORT_THREADS / 64; ++w) add += __builtin_amdgcn_sad_u8(s_wave_cnt[w][tid], 0u, 0u);
        s_base[tid] += add;
        __syncthreads();
    }
}

// Fallback for rows that cannot be read as aligned float4 (d not a multiple of 4, or an unaligned base): one
// workgroup per centroid, one column per thread, rows in ascending point id.
__global__ __launch_bounds__(256) void segment_sum_columns_kernel(
    const float* __restrict__ x, size_t d, const uint32_t* __restrict__ sorted_ids,
    const uint32_t* __restrict__ offsets, float* __restrict__ sums, uint32_t* __restrict__ sizes
) {
    const uint32_t c = blockIdx.x;
    const uint32_t j0 = offsets[c], j1 = offsets[c + 1];
    if (threadIdx.x == 0) sizes[c] = j1 - j0;
    float* out = sums + (size_t) c * d;
    for (size_t t = threadIdx.x; t < d; t += blockDim.x) {
        float acc = 0.0f;
        for (uint32_t j = j0; j < j1; ++j) acc += x[(size_t) sorted_ids[j] * d + t];
        out[t] = acc;
    }
}

// Stores a result that nothing on this compute die reads again at device scope ("sc1"): it is written through the
// die's cache instead of staying there as a dirty line that the stream of point rows evicts later.  The k * d sums
// are 1 % of an update's traffic, but written among the reads they cost 11 % of its time as ordinary stores and
// 8 % written through (690, 665 and, with the stores left out, 615 us for a million rows of 4 KiB).
__device__ __forceinline__ void store_through(float __attribute__((ext_vector_type(4)))* dst,
                                              const float __attribute__((ext_vector_type(4))) v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
}
__device__ __forceinline__ void store_through(float __attribute__((ext_vector_type(2)))* dst,
                                              const float __attribute__((ext_vector_type(2))) v) {
    asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
}
__device__ __forceinline__ void store_through(float __attribute__((ext_vector_type(1)))* dst,
                                              const float __attribute__((ext_vector_type(1))) v) {
    const float first = v[0];
    asm volatile("global_store_dword %0, %1, off sc1" ::"v"(dst), "v"(first) : "memory");
}

// Sums of the rows of every centroid's segment, in ascending point id (the reference's order of additions), so the
// additions of one column are a chain and the time of a launch is the walk of the longest segment: hundreds of rows
// with many centroids, tens of thousands in a mesoclustering.  One wavefront owns 64 * W consecutive columns of
// one centroid (W = 4, 2 or 1 floats per lane: the widest that still gives every SIMD a couple of wavefronts),
// keeps a ring of ROWS row loads in flight (a slot is requested again as soon as its row has been added) and keeps
// the per-row work on the chain to two lane reads, the load and the add.  Requests past the end of the segment are
// clamped to its last row so that no load sits under a condition.
template <int W, int ROWS>
__global__ __launch_bounds__(64) void segment_sum_deep_kernel(
    const float* __restrict__ x, size_t d, const uint32_t* __restrict__ sorted_ids,
    const uint32_t* __restrict__ offsets, float* __restrict__ sums, uint32_t* __restrict__ sizes, uint32_t groups
) {
    static_assert(ROWS <= 64, "lane u prepares the address of row u of a batch");
    typedef float vec_t __attribute__((ext_vector_type(W)));
    const uint32_t c = blockIdx.x / groups, g = blockIdx.x % groups;
    const uint32_t j0 = offsets[c], j1 = offsets[c + 1];
    if (g == 0 && threadIdx.x == 0) sizes[c] = j1 - j0;  // the cluster's size is the length of its segment
    const size_t t = (size_t) g * 64 + threadIdx.x;  // column group of this lane
    const size_t n_groups = d / W;
    const size_t t_load = t < n_groups ? t : n_groups - 1;  // lanes past the last column load it again and store nothing
    vec_t acc = 0.0f;
    if (j1 > j0) {
        const size_t last = j1 - 1;
        // Row addresses of a batch are prepared by the lanes in parallel (lane u: one coalesced id load and one
        // 64-bit multiply-add for row u) and read from that lane's registers when the row is requested, which
        // leaves two lane reads, the load and the add per row on the chain.
        const auto batch_ids = [&](const size_t from) {
            const size_t pos = from + threadIdx.x;
            return sorted_ids[pos <= last ? pos : last];
        };
        const auto address_of = [&](const uint32_t id) { return reinterpret_cast<uint64_t>(x + (size_t) id * d); };
        const auto row = [&](const uint64_t addresses, const int u) {
            const uint32_t lo = __builtin_amdgcn_readlane((uint32_t) addresses, u);
            const uint32_t hi = __builtin_amdgcn_readlane((uint32_t) (addresses >> 32), u);
            // an address built from integers is "flat" unless it says that it is global memory; flat loads would
            // make every wait a wait for all loads
            typedef const vec_t __attribute__((address_space(1))) * global_row_t;
            // every row is read once per update: a non-temporal load keeps it from displacing what the caches hold
            return __builtin_nontemporal_load(reinterpret_cast<global_row_t>(((uint64_t) hi << 32) | lo) + t_load);
        };
        vec_t ring[ROWS];
        uint64_t addresses = address_of(batch_ids(j0));
#pragma unroll
        for (int u = 0; u < ROWS; ++u) ring[u] = row(addresses, u);
        addresses = address_of(batch_ids((size_t) j0 + ROWS));
        size_t j = j0;
        for (; j + ROWS <= j1; j += ROWS) {
            const uint32_t ids_after = batch_ids(j + 2 * ROWS);
            __builtin_amdgcn_sched_barrier(0);
            // every slot is added and at once requested again for the row ROWS further on: ROWS - 1 loads stay in flight
#pragma unroll
            for (int u = 0; u < ROWS; ++u) {
                acc += ring[u];
                ring[u] = row(addresses, u);
                __builtin_amdgcn_sched_barrier(0);  // keeps the request next to the add instead of after all adds
            }
            addresses = address_of(ids_after);
            // The addresses are finished here, at the end of the pass that requested their ids (the ids are
            // ROWS requests old by now).  Left to itself the compiler carries the ids into the next pass and
            // computes there, where it must wait for every load in flight.
            asm volatile("" : "+v"(addresses));
        }
#pragma unroll
        for (int u = 0; u < ROWS; ++u)
            if (j + u < j1) acc += ring[u];
    }
    if (t < n_groups) store_through(reinterpret_cast<vec_t*>(sums + (size_t) c * d) + t, acc);
}

__global__ __launch_bounds__(256) void scale_by_size_kernel(
    float* __restrict__ sums, const uint32_t* __restrict__ sizes, size_t k, size_t d, uint32_t* __restrict__ sizes_copy
) {
    const size_t c = blockIdx.x;
    const uint32_t s = sizes[c];
    if (sizes_copy && threadIdx.x == 0) sizes_copy[c] = s;  // pinned host memory: the host reads the sizes after its wait
    if (s == 0) return;
    const float mult = (float) (1.0 / (double) s);  // float mult_factor = 1.0 / cluster_sizes[i]
    float* row = sums + c * d;
    for (size_t t = threadIdx.x; t < d; t += blockDim.x) row[t] *= mult;
}

__global__ __launch_bounds__(256) void normalize_rows_kernel(float* __restrict__ c, size_t k, size_t d) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t) blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= k) return;
    float* p = c + row * d;
    float s = 0.0f;
    for (size_t t = lane; t < d; t += 64) s += p[t] * p[t];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
    const float inv = 1.0f / sqrtf(s);
    for (size_t t = lane; t < d; t += 64) p[t] *= inv;
}

// Applies row edits of SplitClusters, one workgroup per edit.  The edits of one launch touch disjoint rows (or only
// read a common one); the host orders edits that depend on each other into successive launches.
__global__ __launch_bounds__(256) void edit_rows_kernel(float* __restrict__ c, size_t d, const uint32_t* __restrict__ ops) {
    const float eps = 1.0f / 1024.0f;
    const size_t o = blockIdx.x;
    const uint32_t kind = ops[4 * o], dst = ops[4 * o + 1], src = ops[4 * o + 2];
    const float w = __uint_as_float(ops[4 * o + 3]);
    float* pd = c + (size_t) dst * d;
    float* ps = c + (size_t) src * d;
    if (kind == 0) {
        for (size_t j = threadIdx.x; j < d; j += blockDim.x) {
            const float v = ps[j];
            if (j % 2 == 0) {
                pd[j] = v * (1 + eps);
                ps[j] = v * (1 - eps);
            } else {
                pd[j] = v * (1 - eps);
                ps[j] = v * (1 + eps);
            }
        }
    } else {
        for (size_t j = threadIdx.x; j < d; j += blockDim.x) {
            float val = 0.0f;
            val += w * pd[j];
            val += 1.0f * ps[j];
            val /= (w + 1.0f);
            pd[j] = val;
        }
    }
}

// Workgroups of a reduction: one per 2,048 elements, at most 512.  A short input (the distances of a fine-phase
// problem, the centroids of a small one) would otherwise pay for 512 workgroups that hold one element per thread
// or none, and above all for their 512 additions to one counter, which the memory system performs one after the other.
constexpr int REDUCE_BLOCKS = 512;
constexpr size_t REDUCE_ELEMENTS_PER_BLOCK = 2048;
static inline unsigned reduce_blocks(const size_t n) {
    const size_t wanted = (n + REDUCE_ELEMENTS_PER_BLOCK - 1) / REDUCE_ELEMENTS_PER_BLOCK;
    return (unsigned) std::min<size_t>(REDUCE_BLOCKS, std::max<size_t>(1, wanted));
}

// Fixed-shape two-stage reductions in fp64 in one launch: block b of B sums elements b*256+tid, +B*256, ... and the
// block that finishes last (a counter tells it) adds the B <= 512 block sums in a fixed tree, so the association
// depends only on the element count, never on which block came last.  The counter is left at zero for the next launch.
// Sum of one double per thread of a 256-thread workgroup in the tree s[t] += s[t + off], off = 128, 64, ..., 1
// (thread 0 holds the result).  The levels off = 128 and 64 pair values of different wavefronts and go through LDS;
// from off = 32 down both operands sit in wavefront 0, where lane t takes lane t + off's value with a shuffle: the
// same additions in the same order with three barriers instead of nine.
__device__ __forceinline__ double block_tree_sum(const double mine, double* s) {
    s[threadIdx.x] = mine;
    __syncthreads();
    if (threadIdx.x < 128) s[threadIdx.x] += s[threadIdx.x + 128];
    __syncthreads();
    double v = 0.0;
    if (threadIdx.x < 64) {
        v = s[threadIdx.x] + s[threadIdx.x + 64];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off);  // lanes at or above off compute values nobody reads
    }
    __syncthreads();  // s may be written again by the caller
    return v;
}

template <int MODE>  // 0: sum a[i]; 1: sum (a[i]-b[i])^2; 2: sum of uint32 a[i] (as exact integers)
__global__ __launch_bounds__(256) void reduce_kernel(
    const float* __restrict__ a, const float* __restrict__ b, size_t n, double* __restrict__ partial,
    uint32_t* __restrict__ counter, double* __restrict__ out, const uint32_t* __restrict__ word_in,
    uint32_t* __restrict__ word_out
) {
    __shared__ double s[256];
    __shared__ uint32_t s_done;
    double acc = 0.0;
    const auto term = [&](const size_t i) -> double {
        if (MODE == 0) return (double) a[i];
        if (MODE == 1) {
            const float t = a[i] - b[i];
            return (double) (t * t);
        }
        return (double) reinterpret_cast<const uint32_t*>(a)[i];
    };
    // the elements of a thread, in ascending order; four at a time are requested before any is added
    const size_t stride = (size_t) gridDim.x * 256;
    size_t i = (size_t) blockIdx.x * 256 + threadIdx.x;
    for (; i + 3 * stride < n; i += 4 * stride) {
        const double t0 = term(i), t1 = term(i + stride), t2 = term(i + 2 * stride), t3 = term(i + 3 * stride);
        acc += t0;
        acc += t1;
        acc += t2;
        acc += t3;
    }
    for (; i < n; i += stride) acc += term(i);
    const double block_sum = block_tree_sum(acc, s);
    if (threadIdx.x == 0) {
        partial[blockIdx.x] = block_sum;
        __threadfence();  // the block sum is visible device-wide before the counter says so
        s_done = atomicAdd(counter, 1u);
    }
    __syncthreads();
    if (s_done != gridDim.x - 1) return;
    __threadfence();
    const volatile double* all = partial;  // written by other compute units: read past this one's cache
    // sums of blocks that do not exist count as zero: with 512 blocks this is the sum it always was
    const double low = threadIdx.x < gridDim.x ? all[threadIdx.x] : 0.0;
    const double high = threadIdx.x + 256 < gridDim.x ? all[threadIdx.x + 256] : 0.0;
    const double total = block_tree_sum(low + high, s);
    if (threadIdx.x == 0) {
        out[0] = total;
        *counter = 0u;
        if (word_in) *word_out = *word_in;  // a device word the host wants with the same wait (earlier kernels wrote it)
    }
}

// Result slots in the context's pinned host buffer (8 bytes each).  The reduction writes its result
// straight into the slot, which the device reaches through the buffer's host address: no copy operation, the host reads
// the slot after its next wait on the stream.
enum { SLOT_SCALAR = 0, SLOT_OVERFLOW = 1, SLOT_NOT_PRUNED = 2, SLOT_WCSS = 3, N_RESULT_SLOTS = 8 };

static int result_slot(skm_ctx* ctx, int slot, double** out) {
    void* hp = nullptr;
    SKM_TRY(pinned(ctx, N_RESULT_SLOTS * sizeof(double), &hp));
    *out = (double*) hp + slot;
    return SKM_OK;
}

// Queues the reduction; the result is in *h_slot once the stream has been waited for.
static int reduce_enqueue(skm_ctx* ctx, int mode, const float* a, const float* b, size_t n, double* h_slot,
                          const uint32_t* d_word = nullptr, uint32_t* h_word = nullptr) {
    void* ws = nullptr;
    SKM_TRY(workspace(ctx, 3, (REDUCE_BLOCKS + 8) * sizeof(double), &ws));
    double* partial = (double*) ws;
    uint32_t* counter = nullptr;
    SKM_TRY(reduction_counter(ctx, &counter));
    if (mode == 0)
        hipLaunchKernelGGL(reduce_kernel<0>, dim3(reduce_blocks(n)), dim3(256), 0, ctx->stream, a, b, n, partial, counter, h_slot, d_word, h_word);
    else if (mode == 1)
        hipLaunchKernelGGL(reduce_kernel<1>, dim3(reduce_blocks(n)), dim3(256), 0, ctx->stream, a, b, n, partial, counter, h_slot, d_word, h_word);
    else
        hipLaunchKernelGGL(reduce_kernel<2>, dim3(reduce_blocks(n)), dim3(256), 0, ctx->stream, a, b, n, partial, counter, h_slot, d_word, h_word);
    return check_hip(hipGetLastError(), "reduce_kernel launch");
}

static int reduce_to_host(skm_ctx* ctx, int mode, const float* a, const float* b, size_t n, double* h_out) {
    double* slot = nullptr;
    SKM_TRY(result_slot(ctx, SLOT_SCALAR, &slot));
    SKM_TRY(reduce_enqueue(ctx, mode, a, b, n, slot));
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    *h_out = *(volatile double*) slot;
    return SKM_OK;
}

int reduce_u32_sum_to_host(skm_ctx* ctx, const uint32_t* a, size_t n, double* h_out) {
    return reduce_to_host(ctx, 2, reinterpret_cast<const float*>(a), nullptr, n, h_out);
}

int reduce_u32_sum_enqueue(skm_ctx* ctx, const uint32_t* a, size_t n, double** h_slot, const uint32_t* d_word,
                           uint32_t* h_word) {
    SKM_TRY(result_slot(ctx, SLOT_NOT_PRUNED, h_slot));
    return reduce_enqueue(ctx, 2, reinterpret_cast<const float*>(a), nullptr, n, *h_slot, d_word, h_word);
}

int overflow_count_slot(skm_ctx* ctx, uint32_t** h_slot) {
    double* slot = nullptr;
    SKM_TRY(result_slot(ctx, SLOT_OVERFLOW, &slot));
    *h_slot = reinterpret_cast<uint32_t*>(slot);
    return SKM_OK;
}

// Stable sort of the point ids by assignment (one radix pass per 7 or 8 key bits): *out_sorted_ids lists the n points
// grouped by cluster, ascending inside each group, and (*out_offsets)[c] is the first position of cluster c
// ((*out_offsets)[k] = n).  Both live in the context's workspace until its slots 1 and 4 are used again; the ids are
// also kept as the context's visiting order of these n points.
static int sort_by_assignment(skm_ctx* ctx, const uint32_t* d_idx, size_t n, size_t k, const uint32_t** out_sorted_ids,
                              uint32_t** out_offsets) {
    // Scratch: keys/vals double buffers (4n u32), offsets (k+1), per-tile histograms.
    const int tile = n <= SORT_FEW_KEYS ? SORT_TILE_FEW_KEYS : SORT_TILE;
    const uint32_t n_tiles = (uint32_t) ((n + tile - 1) / tile);
    const size_t hist_len = (size_t) RADIX * std::max<uint32_t>(n_tiles, 1);
    const size_t words = 4 * n + (k + 1) + 2 * hist_len + RADIX + 64;
    void* ws = nullptr;
    SKM_TRY(workspace(ctx, 1, words * sizeof(uint32_t), &ws));
    uint32_t* keys_a = (uint32_t*) ws;
    uint32_t* keys_b = keys_a + n;
    uint32_t* vals_a = keys_b + n;
    uint32_t* vals_b = vals_a + n;
    uint32_t* offsets = vals_b + n;
    uint32_t* hist = offsets + (k + 1);
    uint32_t* bases = hist + hist_len;
    uint32_t* totals = bases + hist_len;

    const uint32_t* sorted_ids = nullptr;
    if (n > 0) {
        int bits = 0;
        while (bits < 32 && ((k - 1) >> bits) != 0) ++bits;
        const int passes = std::max(1, (bits + 7) / 8);
        const int digit_bits = passes == 1 ? 8 : (bits + passes - 1) / passes;
        const uint32_t mask = (1u << digit_bits) - 1u;
        const uint32_t* kin = d_idx;
        const uint32_t* vin = nullptr;
        uint32_t* kout = keys_a;
        // the last pass writes the ids into the context's own buffer: the pruned search of the next iteration visits
        // the points in this order
        void* ws_order = nullptr;
        SKM_TRY(workspace(ctx, 4, n * sizeof(uint32_t), &ws_order));
        ctx->cluster_order = nullptr;
        ctx->cluster_order_n = 0;
        uint32_t* vout = passes == 1 ? (uint32_t*) ws_order : vals_a;
        for (int p = 0; p < passes; ++p) {
            // the key bits are spread evenly over the passes (14 bits: 7 + 7, not 8 + 6): fewer distinct digits in a pass
            // mean longer runs of equal digits per tile, which the scatter writes as longer contiguous pieces
            const int shift = digit_bits * p;
            hipLaunchKernelGGL(radix_hist_kernel, dim3(n_tiles), dim3(SORT_THREADS), 0, ctx->stream, kin, n, shift, mask, n_tiles, tile, hist);
            SKM_HIP_TRY(hipGetLastError());
            hipLaunchKernelGGL(digit_rows_scan_kernel, dim3(RADIX), dim3(64), 0, ctx->stream, hist, n_tiles, bases, totals);
            SKM_HIP_TRY(hipGetLastError());
            hipLaunchKernelGGL(radix_scatter_kernel, dim3(n_tiles), dim3(SORT_THREADS), 0, ctx->stream, kin, vin, n, shift, mask,
                               n_tiles, tile, bases, totals, kout, vout, p == 0 ? 1 : 0,
                               passes == 1 ? offsets : (uint32_t*) nullptr, (uint32_t) k);
            SKM_HIP_TRY(hipGetLastError());
            kin = kout;
            vin = vout;
            kout = (kout == keys_a) ? keys_b : keys_a;
            vout = (p + 2 == passes) ? (uint32_t*) ws_order : ((vout == vals_a) ? vals_b : vals_a);
        }
        ctx->cluster_order = (const uint32_t*) ws_order;
        ctx->cluster_order_n = n;
        sorted_ids = vin;
        // Sizes and segment offsets come from the sorted keys: no counting pass over the assignments.  The scatter of
        // a one-pass sort has written them already.
        if (passes > 1) {
            hipLaunchKernelGGL(segment_bounds_kernel, dim3((unsigned) ((n + 1 + 255) / 256)), dim3(256), 0, ctx->stream, kin, n,
                               (uint32_t) k, offsets);
            SKM_HIP_TRY(hipGetLastError());
        }
    } else {
        sorted_ids = vals_a;
        ctx->cluster_order = nullptr;
        ctx->cluster_order_n = 0;
        SKM_TRY(skm_fill_u32(ctx, offsets, 0u, k + 1));
    }
    *out_sorted_ids = sorted_ids;
    *out_offsets = offsets;
    return SKM_OK;
}

// Ids widened to the 64-bit row ids the gathers take, and the group sizes from the offsets.
__global__ __launch_bounds__(256) void groups_out_kernel(
    const uint32_t* __restrict__ sorted_ids, const uint32_t* __restrict__ offsets, size_t n, size_t k,
    uint64_t* __restrict__ out_ids, uint32_t* __restrict__ out_sizes
) {
    const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out_ids[i] = sorted_ids[i];
    if (i < k) out_sizes[i] = offsets[i + 1] - offsets[i];
}

} // namespace skm

using namespace skm;

extern "C" {

int skm_update(skm_ctx* ctx, const float* d_x, size_t n, size_t d, const uint32_t* d_idx, size_t k,
               float* d_out_sums, uint32_t* d_out_sizes) {
    SKM_REQUIRE(ctx, "null context");
    SKM_REQUIRE(d_out_sums && d_out_sizes, "null output");
    SKM_REQUIRE(k > 0 && d > 0, "k and d must be positive");
    SKM_REQUIRE(k < 0xffffffffULL && n < 0xffffffffULL, "n and k must fit in 32 bits");
    SKM_REQUIRE(n == 0 || (d_x && d_idx), "null input");
    ScopedStage st(ctx, "update_centroids");
    const uint32_t* sorted_ids = nullptr;
    uint32_t* offsets = nullptr;
    SKM_TRY(sort_by_assignment(ctx, d_idx, n, k, &sorted_ids, &offsets));
    const bool vec = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(d_x) % 16 == 0) &&
                     (reinterpret_cast<uintptr_t>(d_out_sums) % 16 == 0);
    if (vec) {
        // widest lanes that still give about 2,048 wavefronts
        int w = 4;
        while (w > 1 && k * ((d / w + 63) / 64) < 2048) w /= 2;
        const size_t groups = (d / w + 63) / 64;
        SKM_REQUIRE(k * groups <= 0x7fffffffULL, "k * d too large for one launch");
        dim3 grid((unsigned) (k * groups));
        if (w == 4)
            hipLaunchKernelGGL((segment_sum_deep_kernel<4, 32>), grid, dim3(64), 0, ctx->stream, d_x, d, sorted_ids, offsets, d_out_sums, d_out_sizes, (uint32_t) groups);
        else if (w == 2)
            hipLaunchKernelGGL((segment_sum_deep_kernel<2, 32>), grid, dim3(64), 0, ctx->stream, d_x, d, sorted_ids, offsets, d_out_sums, d_out_sizes, (uint32_t) groups);
        else
            hipLaunchKernelGGL((segment_sum_deep_kernel<1, 32>), grid, dim3(64), 0, ctx->stream, d_x, d, sorted_ids, offsets, d_out_sums, d_out_sizes, (uint32_t) groups);
    } else {
        hipLaunchKernelGGL(segment_sum_columns_kernel, dim3((unsigned) k), dim3(256), 0, ctx->stream, d_x, d, sorted_ids, offsets, d_out_sums, d_out_sizes);
    }
    return check_hip(hipGetLastError(), "segment sum launch");
}

int skm_group_by_assignment(skm_ctx* ctx, const uint32_t* d_idx, size_t n, size_t k, uint64_t* d_out_ids,
                            uint32_t* d_out_sizes) {
    SKM_REQUIRE(ctx, "null context");
    SKM_REQUIRE(d_out_sizes, "null output");
    SKM_REQUIRE(k > 0, "k must be positive");
    SKM_REQUIRE(k < 0xffffffffULL && n < 0xffffffffULL, "n and k must fit in 32 bits");
    SKM_REQUIRE(n == 0 || (d_idx && d_out_ids), "null argument");
    const uint32_t* sorted_ids = nullptr;
    uint32_t* offsets = nullptr;
    SKM_TRY(sort_by_assignment(ctx, d_idx, n, k, &sorted_ids, &offsets));
    const size_t threads = std::max(n, k);
    hipLaunchKernelGGL(groups_out_kernel, dim3((unsigned) ((threads + 255) / 256)), dim3(256), 0, ctx->stream, sorted_ids,
                       offsets, n, k, d_out_ids, d_out_sizes);
    return check_hip(hipGetLastError(), "groups_out_kernel launch");
}

int skm_scale_by_size(skm_ctx* ctx, float* d_sums, const uint32_t* d_sizes, size_t k, size_t d) {
    SKM_REQUIRE(ctx && d_sums && d_sizes, "null argument");
    if (k == 0) return SKM_OK;
    ScopedStage st(ctx, "consolidate/splitting");
    hipLaunchKernelGGL(scale_by_size_kernel, dim3((unsigned) k), dim3(256), 0, ctx->stream, d_sums, d_sizes, k, d,
                       (uint32_t*) nullptr);
    return check_hip(hipGetLastError(), "scale_by_size_kernel launch");
}

int skm_scale_by_size_fetch(skm_ctx* ctx, float* d_sums, const uint32_t* d_sizes, size_t k, size_t d, uint32_t* h_sizes) {
    SKM_REQUIRE(ctx && d_sums && d_sizes && h_sizes, "null argument");
    if (k == 0) return SKM_OK;
    // Up to a few thousand clusters the kernel leaves a copy of the sizes in pinned host memory on its way (one
    // 4-byte write per cluster); beyond that one copy operation moves them.
    uint32_t* mirror = nullptr;
    size_t mirror_entries = 0;
    SKM_TRY(pinned_sizes(ctx, &mirror, &mirror_entries));
    if (k > mirror_entries) mirror = nullptr;
    {
        ScopedStage st(ctx, "consolidate/splitting");
        hipLaunchKernelGGL(scale_by_size_kernel, dim3((unsigned) k), dim3(256), 0, ctx->stream, d_sums, d_sizes, k, d, mirror);
        SKM_TRY(check_hip(hipGetLastError(), "scale_by_size_kernel launch"));
    }
    if (mirror) {
        SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
        std::memcpy(h_sizes, mirror, k * sizeof(uint32_t));
        return SKM_OK;
    }
    SKM_HIP_TRY(hipMemcpyAsync(h_sizes, d_sizes, k * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SKM_OK;
}

int skm_normalize_rows(skm_ctx* ctx, float* d_c, size_t k, size_t d) {
    SKM_REQUIRE(ctx && d_c, "null argument");
    if (k == 0) return SKM_OK;
    ScopedStage st(ctx, "consolidate/normalize");
    hipLaunchKernelGGL(normalize_rows_kernel, dim3((unsigned) ((k + 3) / 4)), dim3(256), 0, ctx->stream, d_c, k, d);
    return check_hip(hipGetLastError(), "normalize_rows_kernel launch");
}

int skm_edit_rows(skm_ctx* ctx, float* d_c, size_t d, const uint32_t* h_ops, size_t n_ops) {
    SKM_REQUIRE(ctx && d_c, "null argument");
    if (n_ops == 0) return SKM_OK;
    SKM_REQUIRE(h_ops, "null ops");
    SKM_REQUIRE(n_ops <= 0x7fffffffu, "too many edits");
    // Later edits see earlier ones.  Edits that touch disjoint rows commute, so every edit gets the earliest
    // round in which all edits it depends on are done (an earlier edit wrote a row it reads or writes, or read a
    // row it writes), and the rounds run one launch after the other with one workgroup per edit.
    std::unordered_map<uint32_t, int> last_write, last_read;
    std::vector<int> round(n_ops);
    int n_rounds = 0;
    const auto seen = [](const std::unordered_map<uint32_t, int>& m, const uint32_t row) {
        const auto it = m.find(row);
        return it == m.end() ? -1 : it->second;
    };
    for (size_t o = 0; o < n_ops; ++o) {
        const uint32_t kind = h_ops[4 * o], dst = h_ops[4 * o + 1], src = h_ops[4 * o + 2];
        SKM_REQUIRE(kind <= 1, "unknown edit kind");
        // kind 0 writes both rows, kind 1 writes dst and reads both
        int r = std::max({seen(last_write, dst), seen(last_write, src), seen(last_read, dst)});
        if (kind == 0) r = std::max(r, seen(last_read, src));
        r += 1;
        round[o] = r;
        n_rounds = std::max(n_rounds, r + 1);
        last_write[dst] = r;
        if (kind == 0) {
            last_write[src] = r;
        } else {
            last_read[src] = std::max(seen(last_read, src), r);
        }
    }
    std::vector<uint32_t> ordered(n_ops * 4);
    std::vector<size_t> first(n_rounds + 1, 0);
    for (size_t o = 0; o < n_ops; ++o) first[round[o] + 1]++;
    for (int r = 0; r < n_rounds; ++r) first[r + 1] += first[r];
    {
        std::vector<size_t> cursor(first.begin(), first.end() - 1);
        for (size_t o = 0; o < n_ops; ++o) std::memcpy(&ordered[4 * cursor[round[o]]++], h_ops + 4 * o, 4 * sizeof(uint32_t));
    }
    // The kernels read the edits from pinned host memory, a ring the context owns: no copy operation and no wait.  A
    // call that does not fit behind the previous ones starts over at the front after a wait for the stream; a call
    // larger than the ring goes through device memory.
    const void* ws = nullptr;
    const size_t bytes = n_ops * 4 * sizeof(uint32_t);
    void* ring = nullptr;
    size_t ring_bytes = 0;
    SKM_TRY(host_ring(ctx, &ring, &ring_bytes));
    if (bytes <= ring_bytes) {
        if (ctx->h_ring_used + bytes > ring_bytes) {
            SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
            ctx->h_ring_used = 0;
        }
        void* at = (char*) ring + ctx->h_ring_used;
        std::memcpy(at, ordered.data(), bytes);
        ctx->h_ring_used += (bytes + 63) / 64 * 64;
        ws = at;
    } else {
        void* dev = nullptr;
        SKM_TRY(workspace(ctx, 2, bytes, &dev));
        SKM_HIP_TRY(hipMemcpyAsync(dev, ordered.data(), bytes, hipMemcpyHostToDevice, ctx->stream));
        SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));  // `ordered` is released on return
        ws = dev;
    }
    for (int r = 0; r < n_rounds; ++r) {
        const size_t count = first[r + 1] - first[r];
        hipLaunchKernelGGL(edit_rows_kernel, dim3((unsigned) count), dim3(256), 0, ctx->stream, d_c, d,
                           (const uint32_t*) ws + 4 * first[r]);
        SKM_TRY(check_hip(hipGetLastError(), "edit_rows_kernel launch"));
    }
    return SKM_OK;
}

int skm_wcss(skm_ctx* ctx, const float* d_dist, size_t n, double* h_out_cost) {
    SKM_REQUIRE(ctx && h_out_cost, "null argument");
    SKM_REQUIRE(n == 0 || d_dist, "null input");
    ScopedStage st(ctx, "compute_cost");
    return reduce_to_host(ctx, 0, d_dist, nullptr, n, h_out_cost);
}

int skm_wcss_begin(skm_ctx* ctx, const float* d_dist, size_t n) {
    SKM_REQUIRE(ctx, "null argument");
    SKM_REQUIRE(n == 0 || d_dist, "null input");
    ScopedStage st(ctx, "compute_cost");
    double* slot = nullptr;
    SKM_TRY(result_slot(ctx, SLOT_WCSS, &slot));
    return reduce_enqueue(ctx, 0, d_dist, nullptr, n, slot);
}

int skm_wcss_end(skm_ctx* ctx, double* h_out_cost) {
    SKM_REQUIRE(ctx && h_out_cost, "null argument");
    double* slot = nullptr;
    SKM_TRY(result_slot(ctx, SLOT_WCSS, &slot));
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    *h_out_cost = *(volatile double*) slot;
    return SKM_OK;
}

int skm_shift(skm_ctx* ctx, const float* d_new, const float* d_prev, size_t k, size_t d, double* h_out_shift) {
    SKM_REQUIRE(ctx && h_out_shift, "null argument");
    SKM_REQUIRE(k * d == 0 || (d_new && d_prev), "null input");
    ScopedStage st(ctx, "shift");
    return reduce_to_host(ctx, 1, d_new, d_prev, k * d, h_out_shift);
}

} // extern "C"
