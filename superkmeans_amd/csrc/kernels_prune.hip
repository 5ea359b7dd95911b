// Pruned top-1 search over per-point candidate lists, one wavefront per point: walks the batches of 1024 centroids
// in order and reproduces PDXearch::Top1PartialSearchWithThresholdAndPartialDistances / Prune / SetBestCandidate
// (reference pdx/pdxearch.h:118-238,266-327) and the per-row body of
// BatchComputer::FindNearestNeighborWithPruning (distance_computers/batch_computers.h:357-405).  Also the seed
// distances of the search.  This walk serves rows that are not 16-byte aligned; kernels_prune_pool.hip holds the walk
// with several points per wavefront that serves all others.
//
// Wavefront mapping
//   * first test against best * ratios[d']: the candidates of the batch, 64 per step, survivors compacted with a
//     ballot + prefix popcount into an LDS list (InitPositionsArray, scalar_computers.h:87-98);
//   * every 64-dimension horizontal block: 32 survivors per pass, 16 lanes x float4 each, reduced with four
//     cross-lane exchanges, followed by the same ballot compaction
//     (EvaluatePruningPredicateOnPositionsArray, pdxearch.h:67-80);
//   * the [d', vertical_d) dimensions are read last from the dense auxiliary copy;
//   * survivors of the final test (ratio 1) update the best candidate, lowest position first.
// The threshold of a batch is fixed while the batch is processed and only tightens between
// batches, exactly as on the CPU, so the order in which survivors are visited cannot change results.
#include "prune_common.h"

namespace skm {

// Keeps the survivors whose accumulated distance is below thr, preserving order. In-place: slot s
// is rewritten only by elements read from slots >= s, and each step reads before it writes.
__device__ __forceinline__ int compact_survivors(uint16_t* pos, float* acc, int cnt, float thr, int lane) {
    int out = 0;
    for (int s0 = 0; s0 < cnt; s0 += 64) {
        const int s = s0 + lane;
        const bool in = s < cnt;
        const uint16_t p = in ? pos[s] : 0;
        const float a = in ? acc[s] : 0.0f;
        const bool keep = in && (a < thr);
        const unsigned long long mask = __ballot(keep);
        if (keep) {
            const int slot = out + __popcll(mask & ((1ull << lane) - 1ull));
            pos[slot] = p;
            acc[slot] = a;
        }
        out += __popcll(mask);
    }
    return out;
}

// ---------------------------------------------------------------------------------------------
// Seed of the pruned search: squared distance of every point to its previous assignment over all d
// dimensions (batch_computers.h:372-377) and the loosest first-test threshold derived from it.
// ---------------------------------------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(PRUNE_WAVES * 64) void seed_distance_kernel(
    const float* __restrict__ x, const float* __restrict__ c, const uint32_t* __restrict__ idx, int n, int d,
    const float* __restrict__ ratios, int partial_d, float* __restrict__ best0, float* __restrict__ thr0,
    const uint32_t* __restrict__ order, uint32_t* __restrict__ zero_this
) {
    const int lane = threadIdx.x & 63;
    // the first launch of a search also clears the count of overflowing points that later kernels add to
    if (zero_this && blockIdx.x == 0 && threadIdx.x == 0) *zero_this = 0u;
    const int p = point_of_wave(order, n, PRUNE_WAVES);
    if (p < 0) return;
    const float* xq = x + (int64_t) p * d;
    const float* cp = c + (int64_t) idx[p] * d;
    float s = 0.0f;
    if (VEC) {
        // four strides of 256 columns are requested together (eight loads in flight), then added in column order
        int t = lane * 4;
        for (; t + 768 < d; t += 1024) {
            float4 xv[4], cv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                xv[u] = load_once4(xq + t + 256 * u);
                cv[u] = *reinterpret_cast<const float4*>(cp + t + 256 * u);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                float e;
                e = cv[u].x - xv[u].x; s += e * e;
                e = cv[u].y - xv[u].y; s += e * e;
                e = cv[u].z - xv[u].z; s += e * e;
                e = cv[u].w - xv[u].w; s += e * e;
            }
        }
        for (; t < d; t += 256) {
            const float4 xv = load_once4(xq + t);
            const float4 cv = *reinterpret_cast<const float4*>(cp + t);
            float e;
            e = cv.x - xv.x; s += e * e;
            e = cv.y - xv.y; s += e * e;
            e = cv.z - xv.z; s += e * e;
            e = cv.w - xv.w; s += e * e;
        }
    } else {
        for (int t = lane; t < d; t += 64) {
            const float e = cp[t] - xq[t];
            s += e * e;
        }
    }
    s = wave_sum(s);
    if (lane == 0) {
        best0[p] = s;
        thr0[p] = s * ratios[partial_d];
    }
}

// ---------------------------------------------------------------------------------------------
// Pruned search over per-point candidate lists (see gemm_candidates_kernel).  The first test of a batch
// filters the point's candidates that belong to the batch with the exact threshold best * ratios[d'].
// Candidates arrive in no particular order inside a batch; every later step is order
// independent (thresholds are fixed inside a batch, the final minimum breaks ties by position).
// Batches that hold no candidate are skipped: they would prune everything (count 0) anyway.
// Points whose list overflowed (count > cap) are left untouched and reported to the caller.
// ---------------------------------------------------------------------------------------------

// DENSE: instead of a candidate list the point has a row of partial distances to all k centroids (a.partial), and the
// first test of a batch scans the batch's 1024 entries of that row (InitPositionsArray, scalar_computers.h:87-98).
// This serves the points whose list overflowed: for a point that a quarter of the centroids pass, writing and reading
// the dense row is cheaper than appending and walking that many list entries.
template <bool VEC, bool ACCT, bool DENSE>  // ACCT: per-step pair counts requested (adds atomics and keeps lone incumbents walking)
__global__ __launch_bounds__(PRUNE_WAVES * 64, 5) void prune_list_kernel(PruneListArgs a) {
    // LIST_PAD slots past the live survivors: a pass of 32 gathers reads positions and adds partial sums without
    // asking whether a slot is live; the pad positions are kept at 0 (a valid centroid of any batch), what is added to
    // the pad sums is never read.
    __shared__ uint16_t s_pos[PRUNE_WAVES][PRUNE_CAP + LIST_PAD];
    __shared__ float s_acc[PRUNE_WAVES][PRUNE_CAP + LIST_PAD];
    __shared__ float s_parts[PRUNE_WAVES][16 * 8];  // [block of the group][survivor]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int p = point_of_wave(a.order, a.n, PRUNE_WAVES);
    if (p < 0) return;
    float* parts = s_parts[wave];
    const uint32_t n_cand = DENSE ? 0u : a.cand_count[p];
    if (!DENSE && n_cand > a.cap) {  // handled by the caller, who finds the point in the list of overflowing ones
        if (lane == 0) a.over_ids[atomicAdd(a.n_over, 1u)] = a.id_offset + (uint64_t) p;
        return;
    }
    uint16_t* pos = s_pos[wave];
    float* acc = s_acc[wave];
    const int d = a.d, V = a.vertical_d, dp = a.partial_d;
    const int n_hblocks = (d - V) / SKM_H_DIM_SIZE;
    // Accounting counters come in SKM_ACCT_COPIES striped copies (summed by the host) so that the
    // atomics of concurrently running workgroups spread over many addresses.
    unsigned long long* acct = ACCT ? a.stage_pairs + (size_t) (blockIdx.x % SKM_ACCT_COPIES) * (n_hblocks + 2) : nullptr;
    const float* xq = a.x + (int64_t) p * d;
    const uint2* list = a.cand + (int64_t) p * a.cap;
    const float* prow = DENSE ? a.partial + (int64_t) p * a.ld_partial : nullptr;
    const int n_batches = (a.k + SKM_Y_BATCH_SIZE - 1) / SKM_Y_BATCH_SIZE;
    const int sub = lane & 15, grp = lane >> 4;

    uint32_t best_idx = a.idx[p];
    float best = a.best0[p];
    uint32_t not_pruned_total = 0;

    // The list is ordered by batch (the producer appends tile after tile and a batch is eight consecutive
    // tiles), so one forward walk serves every batch: 64 entries are held in registers at a time, `cur` is
    // the first entry not yet consumed.
    uint32_t chunk0 = 0, cur = 0;
    uint2 entry = make_uint2(0xffffffffu, 0u);
    if (!DENSE && lane < n_cand) entry = list[lane];

    for (uint32_t jb_dense = 0; DENSE ? jb_dense < (uint32_t) n_batches : cur < n_cand; ++jb_dense) {
        // the same value in every lane: saying so keeps the batch's base pointers in scalar registers
        const uint32_t jb = DENSE ? jb_dense
                                  : (uint32_t) __builtin_amdgcn_readfirstlane(__shfl((int) entry.x, (int) (cur - chunk0))) / SKM_Y_BATCH_SIZE;
        const int base = (int) jb * SKM_Y_BATCH_SIZE;
        const int m = (a.k - base) < SKM_Y_BATCH_SIZE ? (a.k - base) : SKM_Y_BATCH_SIZE;
        const uint32_t prev_top_1 = best_idx;
        float thr = best * a.ratios[dp];
        int cnt = 0;
        for (int c0 = 0; DENSE && c0 < m; c0 += 64) {
            const int c = c0 + lane;
            const bool in = c < m;
            const float v = in ? prow[base + c] : 0.0f;
            const bool keep = in && (v < thr);
            const unsigned long long mask = __ballot(keep);
            if (keep) {
                const int slot = cnt + __popcll(mask & ((1ull << lane) - 1ull));
                pos[slot] = (uint16_t) c;
                acc[slot] = v;
            }
            cnt += __popcll(mask);
        }
        for (; !DENSE;) {
            const uint32_t s = chunk0 + lane;
            const bool mine = s >= cur && s < n_cand && entry.x / SKM_Y_BATCH_SIZE == jb;
            const bool keep = mine && __uint_as_float(entry.y) < thr;
            const unsigned long long mask = __ballot(keep);
            if (keep) {
                const int slot = cnt + __popcll(mask & ((1ull << lane) - 1ull));
                pos[slot] = (uint16_t) (entry.x - (uint32_t) base);
                acc[slot] = __uint_as_float(entry.y);
            }
            cnt += __popcll(mask);
            cur += (uint32_t) __popcll(__ballot(mine));  // the entries of the batch are consecutive
            if (cur < chunk0 + 64 || cur >= n_cand) break;  // the batch ended inside this chunk, or the list did
            chunk0 += 64;
            entry = make_uint2(0xffffffffu, 0u);
            if (chunk0 + lane < n_cand) entry = list[chunk0 + lane];
        }
        not_pruned_total += (uint32_t) cnt;
        if (ACCT && lane == 0 && cnt) atomicAdd(&acct[0], (unsigned long long) cnt);
        if (cnt == 1 && (uint32_t) (base + pos[0]) == prev_top_1) continue;
        if (cnt == 0) continue;

        const float* chunk = a.pdx + (int64_t) base * d;
        int dims_seen = dp;
        for (int hb = 0; hb < n_hblocks && cnt > 0;) {
            const float* blk = chunk + (int64_t) V * m + (int64_t) hb * m * SKM_H_DIM_SIZE;
            if (cnt <= 8) {
                // Few survivors: a block per round trip would leave the wavefront waiting on one dependent gather
                // after the other.  The 16 gather slots of a pass take G consecutive blocks of every survivor
                // instead (G = 16 / cnt rounded to a power of two); the blocks are then applied in order by the
                // lane that owns the survivor: add, test against the threshold of that depth, stop when pruned.
                // Same additions in the same order as block by block; gathers past a survivor's end are wasted.
                const int cp = cnt <= 1 ? 1 : (cnt <= 2 ? 2 : (cnt <= 4 ? 4 : 8));
                const int shift = cnt <= 1 ? 0 : (cnt <= 2 ? 1 : (cnt <= 4 ? 2 : 3));
                int G = 16 / cp;
                if (G > n_hblocks - hb) G = n_hblocks - hb;
                float4 cv[4], xs[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int slot = 4 * u + grp;
                    const int sv = slot & (cp - 1), g = slot >> shift;
                    const bool valid = sv < cnt && g < G;
                    const int cpos = valid ? pos[sv] : pos[0];
                    const int gg = valid ? g : 0;
                    const float* cb = blk + (int64_t) gg * m * SKM_H_DIM_SIZE + (int64_t) cpos * SKM_H_DIM_SIZE + sub * 4;
                    if (VEC) {
                        cv[u] = *reinterpret_cast<const float4*>(cb);
                    } else {
                        cv[u] = make_float4(cb[0], cb[1], cb[2], cb[3]);
                    }
                    xs[u] = load_x4<VEC>(xq + V + (hb + gg) * SKM_H_DIM_SIZE + sub * 4);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int slot = 4 * u + grp;
                    const int sv = slot & (cp - 1), g = slot >> shift;
                    float e, part = 0.0f;
                    e = xs[u].x - cv[u].x; part += e * e;
                    e = xs[u].y - cv[u].y; part += e * e;
                    e = xs[u].z - cv[u].z; part += e * e;
                    e = xs[u].w - cv[u].w; part += e * e;
                    part = group16_sum(part);
                    if (sv < cnt && g < G && sub == 0) parts[g * 8 + sv] = part;
                }
                const bool owner = lane < cnt;
                const uint16_t my_pos = owner ? pos[lane] : (uint16_t) 0;
                float my_acc = owner ? acc[lane] : 0.0f;
                bool alive = owner;
                int done = 0;
                for (; done < G; ++done) {
                    const int entering = __popcll(__ballot(alive));
                    if (entering == 0) break;
                    if (ACCT && lane == 0) atomicAdd(&acct[1 + hb + done], (unsigned long long) entering);
                    if (alive) my_acc += parts[done * 8 + lane];
                    alive = alive && my_acc < best * a.ratios[dims_seen + (done + 1) * SKM_H_DIM_SIZE];
                }
                const unsigned long long mask = __ballot(alive);
                if (alive) {
                    const int slot = __popcll(mask & ((1ull << lane) - 1ull));
                    pos[slot] = my_pos;
                    acc[slot] = my_acc;
                }
                cnt = __popcll(mask);
                hb += G;
                dims_seen += G * SKM_H_DIM_SIZE;
            } else {
                if (ACCT && lane == 0) atomicAdd(&acct[1 + hb], (unsigned long long) cnt);
                const float4 xv = load_x4<VEC>(xq + V + hb * SKM_H_DIM_SIZE + sub * 4);
                // 32 survivors per pass: the eight gathers of a lane are issued before any of them is used.  Slots past
                // the last survivor read the pad (position 0) and their sums land in the pad.
                if (lane < LIST_PAD) pos[cnt + lane] = 0;
                const global_bytes_t blk_bytes = uniform_pointer(blk);
                const uint32_t lane_bytes = (uint32_t) sub * 16u;
                for (int s0 = 0; s0 < cnt; s0 += 32) {
                    float4 cv[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const uint32_t cpos = pos[s0 + 4 * u + grp];
                        cv[u] = gather4<VEC>(blk_bytes, (cpos << 8) | lane_bytes);
                    }
                    // all 16 lanes of a group hold the sum of each of its eight survivors: lane u of the group keeps
                    // the u-th and the first eight lanes add theirs in one go
                    float mine = 0.0f;
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        float e, part = 0.0f;
                        e = xv.x - cv[u].x; part += e * e;
                        e = xv.y - cv[u].y; part += e * e;
                        e = xv.z - cv[u].z; part += e * e;
                        e = xv.w - cv[u].w; part += e * e;
                        part = group16_sum(part);
                        mine = sub == u ? part : mine;
                    }
                    if (sub < 8) acc[s0 + 4 * sub + grp] += mine;
                }
                hb += 1;
                dims_seen += SKM_H_DIM_SIZE;
                cnt = compact_survivors(pos, acc, cnt, best * a.ratios[dims_seen], lane);
            }
            thr = best * a.ratios[dims_seen];
            // Only the incumbent is left: whatever the remaining steps do to it, the best candidate stays what
            // it is (the rule of pdxearch.h:140-143, applied after a step as well as before the first one).  It
            // would otherwise walk all remaining blocks alone, one dependent gather after the other.  With
            // per-step accounting requested it keeps walking, so that the counts are those of the reference.
            if (cnt == 1 && !ACCT && (uint32_t) (base + pos[0]) == prev_top_1) cnt = 0;
        }
        if (cnt > 0 && dp < V) {
            if (ACCT && lane == 0) atomicAdd(&acct[1 + n_hblocks], (unsigned long long) cnt);
            const int left = V - dp;
            for (int s0 = 0; s0 < cnt; s0 += 4) {
                const int s = s0 + grp;
                const bool in = s < cnt;
                const int cpos = in ? pos[s] : pos[0];
                const float* cb = a.aux + (int64_t) (base + cpos) * V + dp;
                // Four independent loads per operand in flight; the sum keeps the order t = sub, sub + 16, ...
                float part = 0.0f;
                for (int t = sub; t < left; t += 64) {
                    float xe[4], ce[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int tt = t + 16 * u;
                        xe[u] = tt < left ? xq[dp + tt] : 0.0f;
                        ce[u] = tt < left ? cb[tt] : 0.0f;
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const float e = xe[u] - ce[u];
                        part += e * e;
                    }
                }
                part = group16_sum(part);
                if (in && sub == 0) acc[s] += part;
            }
            thr = best * a.ratios[d];
            cnt = compact_survivors(pos, acc, cnt, thr, lane);
        }
        if (cnt > 0) {
            float bv = FLT_MAX;
            int bp = 0x7fffffff;
            for (int s = lane; s < cnt; s += 64) {
                const float v = acc[s];
                const int q = pos[s];
                if (v < bv || (v == bv && q < bp)) {
                    bv = v;
                    bp = q;
                }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float ov = __shfl_xor(bv, off);
                const int op = __shfl_xor(bp, off);
                if (ov < bv || (ov == bv && op < bp)) {
                    bv = ov;
                    bp = op;
                }
            }
            if (bp != 0x7fffffff && bv < best) {
                best = bv;
                best_idx = (uint32_t) (base + bp);
            }
        }
    }
    if (lane == 0) {
        a.idx[p] = best_idx;
        a.dist[p] = best;
        a.not_pruned[p] = not_pruned_total;
    }
}

__global__ __launch_bounds__(256) void gather_u32_kernel(const uint32_t* __restrict__ in, const uint64_t* __restrict__ ids, int m, uint32_t* __restrict__ out) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j < m) out[j] = in[ids[j]];
}

__global__ __launch_bounds__(256) void scatter_u32_kernel(const uint32_t* __restrict__ in, const uint64_t* __restrict__ ids, int m, uint32_t* __restrict__ out) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j < m) out[ids[j]] = in[j];
}

int launch_seed_distance(skm_ctx* ctx, const float* x, const float* c, const uint32_t* idx, int n, int d,
                         const float* ratios, int partial_d, float* best0, float* thr0, const uint32_t* order,
                         uint32_t* zero_this) {
    if (n <= 0) return SKM_OK;
    const bool vec = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(c) % 16 == 0);
    dim3 grid(die_striped_groups(n, PRUNE_WAVES)), block(PRUNE_WAVES * 64);
    if (vec)
        hipLaunchKernelGGL(seed_distance_kernel<true>, grid, block, 0, ctx->stream, x, c, idx, n, d, ratios, partial_d, best0, thr0, order, zero_this);
    else
        hipLaunchKernelGGL(seed_distance_kernel<false>, grid, block, 0, ctx->stream, x, c, idx, n, d, ratios, partial_d, best0, thr0, order, zero_this);
    return check_hip(hipGetLastError(), "seed_distance_kernel launch");
}

int launch_prune_list(skm_ctx* ctx, const uint2* cand, const uint32_t* cand_count, uint32_t cap, const float* best0,
                      const float* x, int n_chunk, const float* pdx, const float* aux, int k, int d, int vertical_d,
                      int partial_d, const float* ratios, uint32_t* inout_idx, float* out_dist, uint32_t* out_not_pruned,
                      unsigned long long* d_stage_pairs, const uint32_t* order, uint64_t* over_ids, uint32_t* n_over,
                      uint64_t id_offset, const float* dense_partial, int64_t ld_partial) {
    if (n_chunk <= 0) return SKM_OK;
    PruneListArgs a;
    a.order = order;
    a.over_ids = over_ids; a.n_over = n_over; a.id_offset = id_offset;
    a.cand = cand; a.cand_count = cand_count; a.cap = cap; a.best0 = best0; a.x = x; a.pdx = pdx; a.aux = aux;
    a.ratios = ratios; a.idx = inout_idx; a.dist = out_dist; a.not_pruned = out_not_pruned; a.stage_pairs = d_stage_pairs;
    a.n = n_chunk; a.k = k; a.d = d; a.vertical_d = vertical_d; a.partial_d = partial_d;
    a.jb_lo = 0; a.jb_hi = 0x7fffffff; a.cursor = nullptr;  // one launch walks every batch
    a.partial = dense_partial; a.ld_partial = ld_partial;
    const bool vec = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(pdx) % 16 == 0);
    dim3 grid(die_striped_groups(n_chunk, PRUNE_WAVES)), block(PRUNE_WAVES * 64);
#define SKM_LAUNCH_WALK(V, A, D) hipLaunchKernelGGL((prune_list_kernel<V, A, D>), grid, block, 0, ctx->stream, a)
    const bool acct = d_stage_pairs != nullptr;
    if (dense_partial) {
        if (vec && acct) SKM_LAUNCH_WALK(true, true, true);
        else if (vec) SKM_LAUNCH_WALK(true, false, true);
        else if (acct) SKM_LAUNCH_WALK(false, true, true);
        else SKM_LAUNCH_WALK(false, false, true);
    } else {
        if (vec && acct) SKM_LAUNCH_WALK(true, true, false);
        else if (vec) SKM_LAUNCH_WALK(true, false, false);
        else if (acct) SKM_LAUNCH_WALK(false, true, false);
        else SKM_LAUNCH_WALK(false, false, false);
    }
#undef SKM_LAUNCH_WALK
    return check_hip(hipGetLastError(), "prune_list_kernel launch");
}

int launch_gather_u32(skm_ctx* ctx, const uint32_t* in, const uint64_t* ids, int m, uint32_t* out) {
    if (m <= 0) return SKM_OK;
    hipLaunchKernelGGL(gather_u32_kernel, dim3((m + 255) / 256), dim3(256), 0, ctx->stream, in, ids, m, out);
    return check_hip(hipGetLastError(), "gather_u32_kernel launch");
}

int launch_scatter_u32(skm_ctx* ctx, const uint32_t* in, const uint64_t* ids, int m, uint32_t* out) {
    if (m <= 0) return SKM_OK;
    hipLaunchKernelGGL(scatter_u32_kernel, dim3((m + 255) / 256), dim3(256), 0, ctx->stream, in, ids, m, out);
    return check_hip(hipGetLastError(), "scatter_u32_kernel launch");
}

} // namespace skm
