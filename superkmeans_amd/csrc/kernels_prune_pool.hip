// Pruned search over per-point candidate lists, several points (POOL_PTS: 4 or 8) per wavefront.
//
// Same contract and same arithmetic as prune_list_kernel (kernels_prune.hip): for every point the batches of 1024
// centroids are taken in ascending order, the candidates of a batch meet the threshold best * ratios[d'] and then
// PDXearch's steps (pdx/pdxearch.h:118-238,266-327).  What differs is how the work is laid out.  The walk of one
// point is a chain of short dependent steps: a batch of a point enters a 64-dimension block with a handful of
// survivors, and a wavefront that serves one point spends most of its instructions on empty gather slots and most
// of its time waiting for one round trip after the other.  Inside a batch the threshold of a point is fixed, so the
// (point, candidate) pairs of a batch are independent of each other.  A wavefront therefore takes POOL_PTS
// consecutive points of the visiting order (neighbours in a cluster order: they share most of their candidate
// blocks) and walks the batches for all of them together:
//   * the survivors of the first test of all its points go into ONE list (the pool), each entry tagged with the
//     slot of its point; a block step gathers for the whole pool, 32 entries per pass, so the passes are as full
//     as the pool is, and the chain of dependent steps of a batch is paid once for POOL_PTS points;
//   * the slices of the points' rows that a block needs are staged in LDS (POOL_PTS x 64 floats), an entry reads
//     its point's slice from there; thresholds and the incumbents are looked up per entry by the point slot;
//   * the pool holds at most 1024 entries, the most one point can contribute per batch: when the next point does
//     not fit, the batch is walked in rounds, each round over whole points;
//   * the best candidate of a point is the minimum over its final survivors of (distance, position), taken with
//     an LDS atomic minimum on a 64-bit key: the same result as the ordered scan, whatever the order.
// The rules that depend on a point's own survivor count (a lone incumbent leaves the walk: pdxearch.h:140-143,
// applied after every step as in prune_list_kernel) are evaluated on the pool through the tags: compaction keeps
// the entries in order, so a point's survivors stay contiguous.  Results equal prune_list_kernel's bit for bit.
#include "prune_common.h"

namespace skm {

// Points per wavefront: 8 where the call has points enough to fill the chip many times over, 4 below (the chain of
// dependent steps of a batch is shorter and there are twice as many wavefronts; measured on the walks of a whole
// Train: 2,000,000 points 216 ms with 8 and 233 ms with 4, 1,000,000 points 15.5 and 16.0 ms, 100,000 points 5.3 and
// 4.0 ms; 16 points per wavefront lose everywhere).
constexpr int POOL_PTS_MANY = 8, POOL_PTS_FEW = 4;
constexpr int POOL_MANY_POINTS = 500000;
constexpr int POOL_CAP = SKM_Y_BATCH_SIZE;    // pool entries: one whole batch of one point always fits
constexpr int POOL_NONE = 0x7fffffff;
constexpr int POOL_Q_SHIFT = 10;              // entry key = point slot << 10 | position in the batch
constexpr uint32_t POOL_POS_MASK = SKM_Y_BATCH_SIZE - 1;
static_assert(SKM_Y_BATCH_SIZE == 1024 && SKM_H_DIM_SIZE == 64, "key layout and block addressing assume 1024 x 64");

template <int POOL_PTS>
struct __attribute__((aligned(16))) PoolLds {  // per wavefront
    float xs[POOL_PTS * SKM_H_DIM_SIZE];   // slices of the points' rows for the current block
    float acc[POOL_CAP + LIST_PAD];
    float parts[16 * 8];                   // few-survivor path: [block of the group][survivor]
    unsigned long long bestkey[POOL_PTS];  // minimum over a batch's final survivors of (ordered distance, position)
    float best[POOL_PTS];
    float thr[POOL_PTS];
    int pid[POOL_PTS];
    uint16_t key[POOL_CAP + LIST_PAD];
    uint16_t incpos[POOL_PTS];             // position of the incumbent in the current batch, 0xffff if elsewhere
};

// Order-preserving map of a float onto an unsigned integer (and back).
__device__ __forceinline__ uint32_t float_order(float f) {
    const uint32_t b = __float_as_uint(f);
    return b ^ ((uint32_t) ((int32_t) b >> 31) | 0x80000000u);
}
__device__ __forceinline__ float float_unorder(uint32_t u) {
    return __uint_as_float(u ^ ((u >> 31) ? 0x80000000u : 0xffffffffu));
}

__device__ __forceinline__ float readlane_f(float v, int l) {
    return __uint_as_float((uint32_t) __builtin_amdgcn_readlane((int) __float_as_uint(v), l));
}

// Keeps the entries below their point's threshold (L.thr), preserving order; in place (see compact_survivors).
template <class Lds>
__device__ __forceinline__ int pool_compact(Lds& L, int cnt, int lane) {
    int out = 0;
    for (int s0 = 0; s0 < cnt; s0 += 64) {
        const int s = s0 + lane;
        const bool in = s < cnt;
        const uint16_t key = in ? L.key[s] : (uint16_t) 0;
        const float a = in ? L.acc[s] : 0.0f;
        const bool keep = in && (a < L.thr[key >> POOL_Q_SHIFT]);
        const unsigned long long mask = __ballot(keep);
        if (keep) {
            const int slot = out + __popcll(mask & ((1ull << lane) - 1ull));
            L.key[slot] = key;
            L.acc[slot] = a;
        }
        out += __popcll(mask);
    }
    return out;
}

// Drops every entry that is its point's only one and is that point's incumbent: whatever the remaining steps do to
// it, the point's best candidate stays what it is.  A point's entries are contiguous, so "only one" is read off the
// neighbours' tags.  In place: slot s0 - 1, which the first lane of a later round of the loop reads, is rewritten by
// the round before only with the entry it already holds.
template <class Lds>
__device__ __forceinline__ int pool_drop_lone_incumbents(Lds& L, int cnt, int lane) {
    int out = 0;
    for (int s0 = 0; s0 < cnt; s0 += 64) {
        const int s = s0 + lane;
        const bool in = s < cnt;
        const uint32_t key = in ? L.key[s] : 0u;
        const float a = in ? L.acc[s] : 0.0f;
        const uint32_t prev = (in && s > 0) ? L.key[s - 1] : 0xffffu;
        const uint32_t next = (s + 1 < cnt) ? L.key[s + 1] : 0xffffu;
        const uint32_t q = key >> POOL_Q_SHIFT;
        const bool lone = (prev >> POOL_Q_SHIFT) != q && (next >> POOL_Q_SHIFT) != q;
        const bool keep = in && !(lone && (key & POOL_POS_MASK) == (uint32_t) L.incpos[q]);
        const unsigned long long mask = __ballot(keep);
        if (keep) {
            const int slot = out + __popcll(mask & ((1ull << lane) - 1ull));
            L.key[slot] = (uint16_t) key;
            L.acc[slot] = a;
        }
        out += __popcll(mask);
    }
    return out;
}

// ACCT: per-step pair counts requested (adds atomics and keeps lone incumbents walking).  POOL_PTS: points per
// wavefront, 4 or 8.
template <bool ACCT, int POOL_PTS>
__global__ __launch_bounds__(PRUNE_WAVES * 64, 4) void prune_pool_kernel(PruneListArgs a) {
    constexpr int POOL_XL = POOL_PTS / 4;  // slices a lane stages per block
    __shared__ PoolLds<POOL_PTS> s_all[PRUNE_WAVES];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    PoolLds<POOL_PTS>& L = s_all[wave];
    const int sub = lane & 15, grp = lane >> 4;
    // consecutive slots of the visiting order stay on one compute die (see point_of_wave)
    const int per_die = (int) (gridDim.x / 8);
    const int group = (int) (blockIdx.x % 8) * per_die + (int) (blockIdx.x / 8);
    const int slot0 = (group * PRUNE_WAVES + wave) * POOL_PTS;
    if (slot0 >= a.n) return;

    const int d = a.d, V = a.vertical_d, dp = a.partial_d;
    const int n_hblocks = (d - V) / SKM_H_DIM_SIZE;
    unsigned long long* acct = ACCT ? a.stage_pairs + (size_t) (blockIdx.x % SKM_ACCT_COPIES) * (n_hblocks + 2) : nullptr;

    // ---- the state of point slot q lives in lane q ----
    int pid = -1;
    uint32_t ncand = 0, cursor = 0, np = 0, bidx = 0;
    float best = 0.0f;
    if (lane < POOL_PTS && slot0 + lane < a.n) {
        pid = a.order ? (int) a.order[slot0 + lane] : slot0 + lane;
        ncand = a.cand_count[pid];
        if (ncand > a.cap) {  // handled by the caller, who finds the point in the list of overflowing ones
            if (a.jb_lo == 0) a.over_ids[atomicAdd(a.n_over, 1u)] = a.id_offset + (uint64_t) pid;
            pid = -1;
            ncand = 0;
        } else if (a.jb_lo > 0) {  // the walk continues where an earlier launch left it
            bidx = a.idx[pid];
            best = a.dist[pid];
            np = a.not_pruned[pid];
            cursor = a.cursor[pid];
        } else {
            bidx = a.idx[pid];
            best = a.best0[pid];
        }
    }
    const unsigned long long live = __ballot(pid >= 0);
    if (live == 0ull) return;
    {
        const int any = __shfl(pid, __ffsll((long long) live) - 1);
        if (lane < POOL_PTS) L.pid[lane] = pid >= 0 ? pid : any;  // slots without a point read a valid row, unused
    }
    // 64 entries of every point's list from its cursor on, held in registers: requested when the cursor moves,
    // used a batch later
    uint2 ent[POOL_PTS];
#pragma unroll
    for (int q = 0; q < POOL_PTS; ++q) {
        const int pq = __builtin_amdgcn_readlane(pid, q);
        const uint32_t nq = (uint32_t) __builtin_amdgcn_readlane((int) ncand, q);
        const uint32_t cq = (uint32_t) __builtin_amdgcn_readlane((int) cursor, q);
        ent[q] = make_uint2(0xffffffffu, 0u);
        if (cq + (uint32_t) lane < nq) ent[q] = (a.cand + (int64_t) pq * a.cap)[cq + lane];
    }
    const float ratio_dp = a.ratios[dp];
    const float ratio_d = a.ratios[d];

    for (;;) {
        // ---- next batch: the lowest batch any point has an entry in ----
        int nextb = POOL_NONE;
#pragma unroll
        for (int q = 0; q < POOL_PTS; ++q) {
            const uint32_t first = (uint32_t) __builtin_amdgcn_readfirstlane((int) ent[q].x);
            nextb = (lane == q && cursor < ncand) ? (int) (first / SKM_Y_BATCH_SIZE) : nextb;
        }
        int jb = nextb;
#pragma unroll
        for (int off = 1; off < POOL_PTS; off <<= 1) jb = min(jb, __shfl_xor(jb, off));
        jb = __builtin_amdgcn_readfirstlane(jb);
        if (jb >= a.jb_hi) break;  // POOL_NONE: no entry left
        const int base = jb * SKM_Y_BATCH_SIZE;
        const int m = (a.k - base) < SKM_Y_BATCH_SIZE ? (a.k - base) : SKM_Y_BATCH_SIZE;
        const float thr_dp = best * ratio_dp;
        const uint32_t inc = (bidx - (uint32_t) base) < (uint32_t) m ? bidx - (uint32_t) base : 0xffffu;
        if (lane < POOL_PTS) {
            L.best[lane] = best;
            L.incpos[lane] = (uint16_t) inc;
            L.bestkey[lane] = ~0ull;
        }
        const bool any_incumbent = __ballot(lane < POOL_PTS && nextb == jb && inc != 0xffffu) != 0ull;
        const float* chunk = a.pdx + (int64_t) base * d;

        int q_start = 0;
        while (q_start < POOL_PTS) {
            // ---- first test of the batch for as many points as the pool holds ----
            int cnt = 0;
            int q_stop = POOL_PTS;
            uint32_t contrib = 0;
#pragma unroll
            for (int q = 0; q < POOL_PTS; ++q) {
                if (q < q_start || q >= q_stop || __builtin_amdgcn_readlane(nextb, q) != jb) continue;
                const int pq = __builtin_amdgcn_readlane(pid, q);
                const uint32_t nq = (uint32_t) __builtin_amdgcn_readlane((int) ncand, q);
                uint32_t cur = (uint32_t) __builtin_amdgcn_readlane((int) cursor, q);
                const float thrq = readlane_f(thr_dp, q);
                const uint32_t incq = (uint32_t) __builtin_amdgcn_readlane((int) inc, q);
                const uint2* list = a.cand + (int64_t) pq * a.cap;
                const int cnt0 = cnt;
                bool deferred = false, keep_more = true;
                uint2 e = ent[q];
                for (;;) {
                    const bool mine = cur + (uint32_t) lane < nq && e.x / SKM_Y_BATCH_SIZE == (uint32_t) jb;
                    const bool keep = keep_more && mine && __uint_as_float(e.y) < thrq;
                    const unsigned long long mask = __ballot(keep);
                    const int nk = __popcll(mask);
                    if (cnt + nk > POOL_CAP) {
                        // the point waits for the next round.  The first point of a round always fits (a batch holds
                        // 1024 distinct centroids); a list that says otherwise is malformed, and its batch is cut short
                        // rather than waited for forever
                        deferred = cnt0 > 0;
                        if (deferred) break;
                        keep_more = false;
                    }
                    if (keep && keep_more) {
                        const int slot = cnt + __popcll(mask & ((1ull << lane) - 1ull));
                        L.key[slot] = (uint16_t) ((q << POOL_Q_SHIFT) | (e.x - (uint32_t) base));
                        L.acc[slot] = __uint_as_float(e.y);
                    }
                    cnt += keep_more ? nk : 0;
                    const int run = __popcll(__ballot(mine));  // the entries of the batch are consecutive
                    cur += (uint32_t) run;
                    if (run < 64 || cur >= nq) break;
                    e = make_uint2(0xffffffffu, 0u);
                    if (cur + (uint32_t) lane < nq) e = list[cur + lane];
                }
                if (deferred) {
                    cnt = cnt0;
                    q_stop = q;
                    continue;
                }
                const int got = cnt - cnt0;
                np += (lane == q) ? (uint32_t) got : 0u;
                if (ACCT && lane == 0 && got) atomicAdd(&acct[0], (unsigned long long) got);
                if (got == 1) {
                    // only survivor is the incumbent: nothing to do (pdxearch.h:140-143)
                    const uint32_t only = (uint32_t) __builtin_amdgcn_readfirstlane((int) L.key[cnt0]);
                    if ((only & POOL_POS_MASK) == incq) cnt = cnt0;
                }
                if (cnt > cnt0) contrib |= 1u << q;
                cursor = (lane == q) ? cur : cursor;
                ent[q] = make_uint2(0xffffffffu, 0u);
                if (cur + (uint32_t) lane < nq) ent[q] = list[cur + lane];
            }
            q_start = q_stop;
            if (cnt == 0) continue;

            // rows whose slices are staged: lanes of group g serve point slots g, g + 4, ...; a slot that contributed
            // nothing to this round reads the row of one that did
            const int q_any = __builtin_ctz(contrib);
            const float* xrow[POOL_XL];
            float4 xnext[POOL_XL];
#pragma unroll
            for (int j = 0; j < POOL_XL; ++j) {
                const int qj = ((contrib >> (grp + 4 * j)) & 1u) ? grp + 4 * j : q_any;
                xrow[j] = a.x + (int64_t) L.pid[qj] * d + V + sub * 4;
                xnext[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
            bool staged = false;

            // ---- horizontal blocks of 64 dimensions, PDX layout (pdxearch.h:149-180) ----
            int dims_seen = dp;
            for (int hb = 0; hb < n_hblocks && cnt > 0;) {
                const float* blk = chunk + (int64_t) V * m + (int64_t) hb * m * SKM_H_DIM_SIZE;
                if (cnt <= 8) {
                    // Few entries: the 16 gather slots of a pass take G consecutive blocks of every entry (G = 16 / cnt
                    // rounded to a power of two); the blocks are then applied in order by the lane that owns the
                    // entry: add, test against the threshold of that depth, stop when pruned.
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
                        const uint32_t key = valid ? L.key[sv] : L.key[0];
                        const int gg = valid ? g : 0;
                        const float* cb = blk + (int64_t) gg * m * SKM_H_DIM_SIZE + (int64_t) (key & POOL_POS_MASK) * SKM_H_DIM_SIZE + sub * 4;
                        cv[u] = *reinterpret_cast<const float4*>(cb);
                        xs[u] = *reinterpret_cast<const float4*>(a.x + (int64_t) L.pid[key >> POOL_Q_SHIFT] * d + V +
                                                                 (hb + gg) * SKM_H_DIM_SIZE + sub * 4);
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
                        if (sv < cnt && g < G && sub == 0) L.parts[g * 8 + sv] = part;
                    }
                    const bool owner = lane < cnt;
                    const uint16_t my_key = owner ? L.key[lane] : (uint16_t) 0;
                    float my_acc = owner ? L.acc[lane] : 0.0f;
                    const float my_best = L.best[my_key >> POOL_Q_SHIFT];
                    bool alive = owner;
                    for (int done = 0; done < G; ++done) {
                        const int entering = __popcll(__ballot(alive));
                        if (entering == 0) break;
                        if (ACCT && lane == 0) atomicAdd(&acct[1 + hb + done], (unsigned long long) entering);
                        if (alive) my_acc += L.parts[done * 8 + lane];
                        alive = alive && my_acc < my_best * a.ratios[dims_seen + (done + 1) * SKM_H_DIM_SIZE];
                    }
                    const unsigned long long mask = __ballot(alive);
                    if (alive) {
                        const int slot = __popcll(mask & ((1ull << lane) - 1ull));
                        L.key[slot] = my_key;
                        L.acc[slot] = my_acc;
                    }
                    cnt = __popcll(mask);
                    hb += G;
                    dims_seen += G * SKM_H_DIM_SIZE;
                } else {
                    if (ACCT && lane == 0) atomicAdd(&acct[1 + hb], (unsigned long long) cnt);
                    // this block's slices were requested one block ago; the next ones are requested now
                    if (!staged) {
#pragma unroll
                        for (int j = 0; j < POOL_XL; ++j) xnext[j] = *reinterpret_cast<const float4*>(xrow[j] + hb * SKM_H_DIM_SIZE);
                        staged = true;
                    }
#pragma unroll
                    for (int j = 0; j < POOL_XL; ++j)
                        *reinterpret_cast<float4*>(&L.xs[(grp + 4 * j) * SKM_H_DIM_SIZE + sub * 4]) = xnext[j];
                    if (hb + 1 < n_hblocks) {
#pragma unroll
                        for (int j = 0; j < POOL_XL; ++j)
                            xnext[j] = *reinterpret_cast<const float4*>(xrow[j] + (hb + 1) * SKM_H_DIM_SIZE);
                    }
                    // 32 entries per pass: the eight gathers of a lane are issued before any of them is used.  Slots
                    // past the last entry read the pad (key 0) and their sums land in the pad.
                    if (lane < LIST_PAD) L.key[cnt + lane] = 0;
                    const global_bytes_t blk_bytes = uniform_pointer(blk);
                    const uint32_t lane_bytes = (uint32_t) sub * 16u;
                    for (int s0 = 0; s0 < cnt; s0 += 32) {
                        float4 cv[8];
                        uint32_t xoff[8];
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            const uint32_t key = L.key[s0 + 4 * u + grp];
                            cv[u] = gather4<true>(blk_bytes, ((key & POOL_POS_MASK) << 8) | lane_bytes);
                            xoff[u] = ((key >> POOL_Q_SHIFT) << 8) | lane_bytes;
                        }
                        float mine = 0.0f;
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            const float4 xv = *reinterpret_cast<const float4*>(reinterpret_cast<const char*>(L.xs) + xoff[u]);
                            float e, part = 0.0f;
                            e = xv.x - cv[u].x; part += e * e;
                            e = xv.y - cv[u].y; part += e * e;
                            e = xv.z - cv[u].z; part += e * e;
                            e = xv.w - cv[u].w; part += e * e;
                            part = group16_sum(part);
                            mine = sub == u ? part : mine;
                        }
                        if (sub < 8) L.acc[s0 + 4 * sub + grp] += mine;
                    }
                    hb += 1;
                    dims_seen += SKM_H_DIM_SIZE;
                    if (lane < POOL_PTS) L.thr[lane] = best * a.ratios[dims_seen];
                    cnt = pool_compact(L, cnt, lane);
                }
                // A point whose only entry left is its incumbent is done with this batch (the rule of
                // pdxearch.h:140-143 applied after a step).  With per-step accounting requested it keeps walking, so
                // that the counts are those of the reference.
                if (!ACCT && any_incumbent && cnt > 0) cnt = pool_drop_lone_incumbents(L, cnt, lane);
            }

            // ---- remaining vertical dimensions [d', V) from the dense auxiliary copy (pdxearch.h:183-216) ----
            if (cnt > 0 && dp < V) {
                if (ACCT && lane == 0) atomicAdd(&acct[1 + n_hblocks], (unsigned long long) cnt);
                const int left = V - dp;
                for (int s0 = 0; s0 < cnt; s0 += 4) {
                    const int s = s0 + grp;
                    const bool in = s < cnt;
                    const uint32_t key = in ? L.key[s] : L.key[0];
                    const float* cb = a.aux + (int64_t) (base + (int) (key & POOL_POS_MASK)) * V + dp;
                    const float* xq = a.x + (int64_t) L.pid[key >> POOL_Q_SHIFT] * d + dp;
                    // Four independent loads per operand in flight; the sum keeps the order t = sub, sub + 16, ...
                    float part = 0.0f;
                    for (int t = sub; t < left; t += 64) {
                        float xe[4], ce[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int tt = t + 16 * u;
                            xe[u] = tt < left ? xq[tt] : 0.0f;
                            ce[u] = tt < left ? cb[tt] : 0.0f;
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const float e = xe[u] - ce[u];
                            part += e * e;
                        }
                    }
                    part = group16_sum(part);
                    if (in && sub == 0) L.acc[s] += part;
                }
                if (lane < POOL_PTS) L.thr[lane] = best * ratio_d;
                cnt = pool_compact(L, cnt, lane);
            }

            // ---- SetBestCandidate (pdxearch.h:223-238): lowest distance, lowest position on ties ----
            for (int s = lane; s < cnt; s += 64) {
                const uint32_t key = L.key[s];
                const float v = L.acc[s] + 0.0f;  // -0 and +0 are one value
                atomicMin(&L.bestkey[key >> POOL_Q_SHIFT],
                          ((unsigned long long) float_order(v) << 32) | (unsigned long long) (key & POOL_POS_MASK));
            }
            __builtin_amdgcn_wave_barrier();
        }
        // strict <: a batch replaces the best candidate only with a closer one
        if (lane < POOL_PTS) {
            const unsigned long long kk = L.bestkey[lane];
            if (kk != ~0ull) {
                const float bv = float_unorder((uint32_t) (kk >> 32));
                if (bv < best) {
                    best = bv;
                    bidx = (uint32_t) base + (uint32_t) (kk & 0xffffffffull);
                }
            }
        }
    }
    if (pid >= 0) {
        a.idx[pid] = bidx;
        a.dist[pid] = best;
        a.not_pruned[pid] = np;
        if (a.cursor) a.cursor[pid] = cursor;
    }
}

bool prune_pool_serves(const float* x, const float* pdx, int d) {
    return d % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(pdx) % 16 == 0;
}

int launch_prune_pool(skm_ctx* ctx, const uint2* cand, const uint32_t* cand_count, uint32_t cap, const float* best0,
                      const float* x, int n_chunk, const float* pdx, const float* aux, int k, int d, int vertical_d,
                      int partial_d, const float* ratios, uint32_t* inout_idx, float* out_dist, uint32_t* out_not_pruned,
                      unsigned long long* d_stage_pairs, const uint32_t* order, uint64_t* over_ids, uint32_t* n_over,
                      uint64_t id_offset, int jb_lo, int jb_hi, uint32_t* cursor, int points_per_wavefront) {
    if (n_chunk <= 0) return SKM_OK;
    if (points_per_wavefront != 0 && points_per_wavefront != POOL_PTS_FEW && points_per_wavefront != POOL_PTS_MANY)
        return set_error(SKM_ERR_INVALID, "pooled list walk: 4 or 8 points per wavefront");
    if (jb_lo < 0 || jb_hi <= jb_lo || ((jb_lo > 0 || jb_hi < (k + SKM_Y_BATCH_SIZE - 1) / SKM_Y_BATCH_SIZE) && !cursor))
        return set_error(SKM_ERR_INVALID, "pooled list walk: a range of batches needs the cursor array");
    if (!prune_pool_serves(x, pdx, d))
        return set_error(SKM_ERR_INVALID, "pooled list walk: rows must be 16-byte aligned with d a multiple of 4");
    PruneListArgs a;
    a.order = order;
    a.over_ids = over_ids; a.n_over = n_over; a.id_offset = id_offset;
    a.cand = cand; a.cand_count = cand_count; a.cap = cap; a.best0 = best0; a.x = x; a.pdx = pdx; a.aux = aux;
    a.ratios = ratios; a.idx = inout_idx; a.dist = out_dist; a.not_pruned = out_not_pruned; a.stage_pairs = d_stage_pairs;
    a.n = n_chunk; a.k = k; a.d = d; a.vertical_d = vertical_d; a.partial_d = partial_d;
    a.jb_lo = jb_lo; a.jb_hi = jb_hi; a.cursor = cursor;
    a.partial = nullptr; a.ld_partial = 0;
    const int pts = points_per_wavefront ? points_per_wavefront
                                         : (n_chunk >= POOL_MANY_POINTS ? POOL_PTS_MANY : POOL_PTS_FEW);
    const int wavefronts = (n_chunk + pts - 1) / pts;
    dim3 grid(die_striped_groups(wavefronts, PRUNE_WAVES)), block(PRUNE_WAVES * 64);
    if (d_stage_pairs && pts == POOL_PTS_MANY)
        hipLaunchKernelGGL((prune_pool_kernel<true, POOL_PTS_MANY>), grid, block, 0, ctx->stream, a);
    else if (d_stage_pairs)
        hipLaunchKernelGGL((prune_pool_kernel<true, POOL_PTS_FEW>), grid, block, 0, ctx->stream, a);
    else if (pts == POOL_PTS_MANY)
        hipLaunchKernelGGL((prune_pool_kernel<false, POOL_PTS_MANY>), grid, block, 0, ctx->stream, a);
    else
        hipLaunchKernelGGL((prune_pool_kernel<false, POOL_PTS_FEW>), grid, block, 0, ctx->stream, a);
    return check_hip(hipGetLastError(), "prune_pool_kernel launch");
}

} // namespace skm
