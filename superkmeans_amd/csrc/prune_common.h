// Device helpers shared by the pruning walks (kernels_prune.hip, kernels_prune_pool.hip).
#pragma once

#include "skm_internal.h"

#include <float.h>

namespace skm {

constexpr int PRUNE_WAVES = 4;
constexpr int PRUNE_CAP = SKM_Y_BATCH_SIZE;
constexpr int LIST_PAD = 32;  // survivors per pass of the list walk

// Sum over each group of 16 consecutive lanes, returned in all of them.  Rotations inside a row of 16 lanes are
// data-parallel primitives of the vector unit (no trip through the LDS crossbar); the pairing is that of a
// butterfly over lane distances 8, 4, 2, 1, so every lane adds the same pairs in the same order.
template <int N>
__device__ __forceinline__ float row_ror(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xf, 0xf, true));
}
__device__ __forceinline__ float group16_sum(float v) {
    v += row_ror<8>(v);
    v += row_ror<4>(v);
    v += row_ror<2>(v);
    v += row_ror<1>(v);
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// Which point a wavefront takes.  Workgroups go to the eight compute dies in turn (workgroup b runs on die b % 8, each
// with its own L2), so the grid is read as eight contiguous ranges of slots, one per die: consecutive slots, which
// under a cluster order hold points that gather the same centroid rows and blocks, stay on one die.  The launch has
// 8 * ceil(workgroups / 8) workgroups; a slot past the end returns -1.
__device__ __forceinline__ int point_of_wave(const uint32_t* __restrict__ order, int n, int waves_per_group) {
    const int per_die = (int) (gridDim.x / 8);
    const int group = (int) (blockIdx.x % 8) * per_die + (int) (blockIdx.x / 8);
    const int slot = group * waves_per_group + (int) (threadIdx.x >> 6);
    if (slot >= n) return -1;
    return order ? (int) order[slot] : slot;
}
inline unsigned die_striped_groups(int n, int waves_per_group) {
    const unsigned groups = (unsigned) ((n + waves_per_group - 1) / waves_per_group);
    return (groups + 7) / 8 * 8;
}

// The same pointer, said to be equal in all lanes (it is: it derives from the batch and block indices) and to point to
// global memory (an address built from integers is otherwise taken for a flat one, whose loads are waited for all at
// once): the compiler then keeps it in scalar registers and a gather needs only its 32-bit lane offset in a vector
// register.
typedef const char __attribute__((address_space(1)))* global_bytes_t;
typedef float gather4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ global_bytes_t uniform_pointer(const void* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t) v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t) (v >> 32));
    return reinterpret_cast<global_bytes_t>(((uint64_t) hi << 32) | lo);
}
// Four floats at byte offset `off` of a block (16-byte load when VEC).
template <bool VEC>
__device__ __forceinline__ float4 gather4(global_bytes_t base, uint32_t off) {
    if (VEC) {
        const gather4_t g = *reinterpret_cast<const gather4_t __attribute__((address_space(1)))*>(base + off);
        return make_float4(g.x, g.y, g.z, g.w);
    }
    const float __attribute__((address_space(1)))* f = reinterpret_cast<const float __attribute__((address_space(1)))*>(base + off);
    return make_float4(f[0], f[1], f[2], f[3]);
}

// Four consecutive floats of a point row (16-byte load when rows are aligned).
template <bool VEC>
__device__ __forceinline__ float4 load_x4(const float* p) {
    if (VEC) return *reinterpret_cast<const float4*>(p);
    return make_float4(p[0], p[1], p[2], p[3]);
}

// The same for data that is read once per launch: a non-temporal load, which leaves the caches to the centroids.
__device__ __forceinline__ float4 load_once4(const float* p) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    const v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}

// Arguments of the walks over per-point candidate lists (prune_list_kernel, prune_pool_kernel).
struct PruneListArgs {
    const uint2* cand;            // n_chunk x cap {centroid index, partial distance bits}
    const uint32_t* cand_count;   // n_chunk
    uint32_t cap;
    const float* best0;           // seed distances
    const float* x;
    const float* pdx;
    const float* aux;
    const float* ratios;
    uint32_t* idx;
    float* dist;
    uint32_t* not_pruned;
    unsigned long long* stage_pairs;
    const uint32_t* order;        // null, or the sequence in which the wavefronts take the points
    uint64_t* over_ids;           // ids (id_offset + point) of the points whose list overflowed, appended here
    uint32_t* n_over;             // their count
    uint64_t id_offset;
    int n, k, d, vertical_d, partial_d;
    // prune_pool_kernel only: the launch walks the batches [jb_lo, jb_hi); with jb_lo > 0 it resumes from idx, dist,
    // not_pruned and cursor as the launch over the batches before left them.  cursor: per point, entries consumed.
    int jb_lo, jb_hi;
    uint32_t* cursor;
    // prune_list_kernel<.., DENSE> only: n x ld_partial partial distances to all centroids instead of the lists
    const float* partial;
    int64_t ld_partial;
};

} // namespace skm
