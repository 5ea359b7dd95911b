// MFMA kernels built on gemm_core.h: dense store (rotation, partial distances) and
// fused distance + per-granule argmin (exact nearest-centroid search).
#include "gemm_core.h"
#include "skm_internal.h"

#include <float.h>

namespace skm {

// The double-buffered operand stages need 72 KiB (small shape) or 144 KiB (large shape) of LDS, above the
// 64 KiB a kernel may use without opting in; gfx950 has 160 KiB per CU.
template <class Kernel>
static int allow_large_lds(Kernel kernel, size_t bytes) {
    return check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int) bytes),
                     "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
}

#define SKM_LAUNCH_GEMM(kernel, grid, block, lds_bytes, stream, ...)                               \
    do {                                                                                           \
        /* once per kernel and process; the initialisation of a local static is thread safe */    \
        static const int lds_rc = allow_large_lds(kernel, lds_bytes);                              \
        SKM_TRY(lds_rc);                                                                           \
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, __VA_ARGS__);                   \
    } while (0)

// The large shape pays off once its tiles fill the chip a few times over; below that (hierarchical fine
// clusterings, tests) the small shape keeps more workgroups in flight.  Its loop is about 4.5 % faster per
// flop, so it is also passed over when padding M and N to multiples of 256 instead of 128 adds more work
// than that (k = 300 would be computed as 512 rows instead of 384).
static bool use_big_tiles(int M, int N) {
    if (M < 192 || N < 192) return false;
    auto padded = [](int v, int t) { return (double) ((v + t - 1) / t) * t; };
    const long long tiles = (long long) ((M + GemmBig::TM - 1) / GemmBig::TM) * ((N + GemmBig::TN - 1) / GemmBig::TN);
    const double work_big = padded(M, GemmBig::TM) * padded(N, GemmBig::TN);
    const double work_small = padded(M, GemmSmall::TM) * padded(N, GemmSmall::TN);
    return tiles >= 1024 && work_big <= 1.045 * work_small;
}

// Small problems (a fine clustering of the hierarchical variant: 39,000 points x 256 centroids is 610 tiles of
// 128 x 128 on 512 workgroup slots) finish in a few rounds of workgroups, the last one nearly empty.  Tiles of half
// the width cost about 0.58 of a whole one and fill the rounds better; the shape is taken when that model promises
// 8 % or more (39,000 x 256: 214 -> 196 us; 80,000 x 256, where the model is at par, is 3 % slower with them).
static bool use_half_tiles(int M, int N) {
    const long long slots = 512;  // 256 CUs x 2 workgroups
    const long long whole = (long long) ((M + GemmSmall::TM - 1) / GemmSmall::TM) * ((N + GemmSmall::TN - 1) / GemmSmall::TN);
    const long long half = (long long) ((M + GemmHalf::TM - 1) / GemmHalf::TM) * ((N + GemmHalf::TN - 1) / GemmHalf::TN);
    if (whole > 8 * slots) return false;
    const double t_whole = (double) ((whole + slots - 1) / slots);
    const double t_half = 0.58 * (double) ((half + slots - 1) / slots);
    return t_half < 0.92 * t_whole;
}

template <class S>
static int fill_operands(GemmOperands& g, const float* A, int M, int64_t lda, const float* B, int N, int64_t ldb, int K) {
    g.A = A; g.B = B; g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.m_base = 0;
    g.tiles_m = (M + S::TM - 1) / S::TM;
    g.tiles_n = (N + S::TN - 1) / S::TN;
    if ((long long) g.tiles_m * g.tiles_n > 0x7fffffffLL) return set_error(SKM_ERR_INVALID, "gemm grid too large");
    // Operand rows are addressed with 32-bit byte offsets from the tile's first row (at most 256 rows).
    if (lda > (int64_t(1) << 20) || ldb > (int64_t(1) << 20)) return set_error(SKM_ERR_INVALID, "gemm row stride above 2^20");
    return SKM_OK;
}

// ---------------------------------------------------------------------------------------------
// Dense store: out[m][n] = D[m][n]                        (rotation, reference adsampling.h:191-215)
//           or out[m][n] = -2 D[m][n] + rn[m] + cn[n]     (batch_computers.h:361-366)
// Rows of D are the M operand (points), so that the 32 lanes of an accumulator column group write
// 128 contiguous bytes of one output row.
// ---------------------------------------------------------------------------------------------
template <bool VEC, bool DIST, class S>
__global__ __launch_bounds__(S::THREADS, S::WG_PER_CU) void gemm_store_kernel(
    GemmOperands g, float* __restrict__ out, int64_t ldo, const float* __restrict__ rn,
    const float* __restrict__ cn, int wide_out
) {
    extern __shared__ float lds[];
    int tm, tn;
    tile_of_block<S::BAND>(g, blockIdx.x, tm, tn);
    WaveAccT<S::FM, S::FN> acc;
    gemm_tile<VEC, S>(g, tm, tn, lds, acc);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / S::WN, wn = wave % S::WN;
    const int m0 = tm * S::TM + wm * S::WAVE_M;
    const int n0 = tn * S::TN + wn * S::WAVE_N;
    if (wide_out) {
        // Output rows are 16-byte aligned: the tile goes out through LDS, one block of 32 rows per wavefront row
        // at a time, so that every store instruction writes whole 16-byte pieces of contiguous row segments
        // (1 KiB per wavefront with the large shape) instead of 128-byte fragments of two rows.  Past the last
        // barrier of the tile loop no wavefront reads the operand stages any more.
        constexpr int PASS_ROWS = S::WM * 32;
        constexpr int LDW = S::TN + 8;  // rows 4 apart land 32 banks apart: the 64 lanes of a store hit 64 banks
        constexpr int LANES_PER_ROW = S::TN / 4;
        constexpr int ROWS_PER_ITER = S::THREADS / LANES_PER_ROW;
        static_assert(PASS_ROWS * LDW <= S::LDS_FLOATS, "staging block must fit the operand stages");
        float cnv[S::FN];
#pragma unroll
        for (int nb = 0; nb < S::FN; ++nb) {
            const int n = n0 + acc_col(nb, lane);
            cnv[nb] = (DIST && n < g.N) ? cn[n] : 0.0f;
        }
#pragma unroll
        for (int mb = 0; mb < S::FM; ++mb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = acc_row(0, r, lane);  // within the 32-row block
                float rnv = 0.0f;
                if (DIST) {
                    const int m = m0 + mb * 32 + row;
                    rnv = rn[m < g.M ? m : g.M - 1];
                }
#pragma unroll
                for (int nb = 0; nb < S::FN; ++nb) {
                    float v = acc.v[mb][nb][r];
                    if (DIST) v = fmaf(-2.0f, v, rnv) + cnv[nb];
                    lds[(wm * 32 + row) * LDW + wn * S::WAVE_N + acc_col(nb, lane)] = v;
                }
            }
            __syncthreads();
#pragma unroll
            for (int it = 0; it < PASS_ROWS / ROWS_PER_ITER; ++it) {
                const int rl = it * ROWS_PER_ITER + tid / LANES_PER_ROW;
                const int c4 = (tid % LANES_PER_ROW) * 4;
                const int m = tm * S::TM + (rl / 32) * S::WAVE_M + mb * 32 + (rl % 32);
                const int n = tn * S::TN + c4;
                if (m < g.M && n < g.N) {
                    const floatx4 v4 = *reinterpret_cast<const floatx4*>(&lds[rl * LDW + c4]);
                    float* dst = out + (int64_t) m * ldo + n;
                    if (n + 3 < g.N) {
                        *reinterpret_cast<floatx4*>(dst) = v4;
                    } else {
                        dst[0] = v4.x;
                        if (n + 1 < g.N) dst[1] = v4.y;
                        if (n + 2 < g.N) dst[2] = v4.z;
                    }
                }
            }
            __syncthreads();
        }
        return;
    }
#pragma unroll
    for (int nb = 0; nb < S::FN; ++nb) {
        const int n = n0 + acc_col(nb, lane);
        if (n >= g.N) continue;
        float cnv = 0.0f;
        if (DIST) cnv = cn[n];
#pragma unroll
        for (int mb = 0; mb < S::FM; ++mb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + acc_row(mb, r, lane);
                if (m < g.M) {
                    float v = acc.v[mb][nb][r];
                    if (DIST) v = fmaf(-2.0f, v, rn[m]) + cnv;
                    out[(int64_t) m * ldo + n] = v;
                }
            }
        }
    }
}

template <class S>
static int launch_gemm_store_shape(skm_ctx* ctx, const float* A, int M, int64_t lda, const float* B, int N,
                                   int64_t ldb, int K, float* out, int64_t ldo, const float* row_norm,
                                   const float* col_norm) {
    GemmOperands g;
    SKM_TRY(fill_operands<S>(g, A, M, lda, B, N, ldb, K));
    const bool vec = gemm_operands_vectorizable(g);
    const bool dist = row_norm != nullptr && col_norm != nullptr;
    const size_t lds_bytes = S::LDS_FLOATS * sizeof(float);
    dim3 grid((unsigned) (g.tiles_m * g.tiles_n)), block(S::THREADS);
    const int wide_out = (reinterpret_cast<uintptr_t>(out) % 16 == 0 && ldo % 4 == 0) ? 1 : 0;
    if (vec && dist)
        SKM_LAUNCH_GEMM((gemm_store_kernel<true, true, S>), grid, block, lds_bytes, ctx->stream, g, out, ldo, row_norm, col_norm, wide_out);
    else if (vec)
        SKM_LAUNCH_GEMM((gemm_store_kernel<true, false, S>), grid, block, lds_bytes, ctx->stream, g, out, ldo, row_norm, col_norm, wide_out);
    else if (dist)
        SKM_LAUNCH_GEMM((gemm_store_kernel<false, true, S>), grid, block, lds_bytes, ctx->stream, g, out, ldo, row_norm, col_norm, wide_out);
    else
        SKM_LAUNCH_GEMM((gemm_store_kernel<false, false, S>), grid, block, lds_bytes, ctx->stream, g, out, ldo, row_norm, col_norm, wide_out);
    return check_hip(hipGetLastError(), "gemm_store_kernel launch");
}

int launch_gemm_store(skm_ctx* ctx, const float* A, int M, int64_t lda, const float* B, int N,
                      int64_t ldb, int K, float* out, int64_t ldo, const float* row_norm,
                      const float* col_norm) {
    if (M <= 0 || N <= 0 || K <= 0) return SKM_OK;
    if (use_big_tiles(M, N))
        return launch_gemm_store_shape<GemmBig>(ctx, A, M, lda, B, N, ldb, K, out, ldo, row_norm, col_norm);
    return launch_gemm_store_shape<GemmSmall>(ctx, A, M, lda, B, N, ldb, K, out, ldo, row_norm, col_norm);
}

// ---------------------------------------------------------------------------------------------
// Distance + argmin: the M operand is the centroid tile, the N operand the point tile, so every
// lane owns one point column per accumulator block and scans its FM x 16 centroid rows in ascending
// index order in registers.  The two half-wavefronts (rows 0-3 | 4-7 of every group of 8) are merged
// with one cross-lane exchange; the result of the wavefront's granule (64 or 128 centroids, by shape)
// is stored, never reduced with atomics.  The centroid norms of the tile go through LDS once the
// operand stages are no longer read.
// ---------------------------------------------------------------------------------------------
template <bool VEC, class S>
__global__ __launch_bounds__(S::THREADS, S::WG_PER_CU) void gemm_argmin_kernel(
    GemmOperands g, const float* __restrict__ xnorm, const float* __restrict__ cnorm,
    uint2* __restrict__ granule_min
) {
    extern __shared__ float lds[];
    int tm, tn;
    tile_of_block<S::BAND>(g, blockIdx.x, tm, tn);
    float cn_mine = 0.0f;
    if (threadIdx.x < S::TM) {
        const int m = tm * S::TM + (int) threadIdx.x;
        cn_mine = (m < g.M) ? cnorm[m] : 0.0f;
    }
    WaveAccT<S::FM, S::FN> acc;
    gemm_tile<VEC, S>(g, tm, tn, lds, acc);
    // Past the last barrier of the tile loop no wavefront reads the operand stages any more.
    if (threadIdx.x < S::TM) lds[threadIdx.x] = cn_mine;
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / S::WN, wn = wave % S::WN;
    const int m0 = tm * S::TM + wm * S::WAVE_M;
    const int n0 = tn * S::TN + wn * S::WAVE_N;
    const int granule = tm * S::WM + wm;
    if (m0 >= g.M) return;  // granule entirely past the last centroid: never read by the merge
    const float* cns = lds + wm * S::WAVE_M;
    const bool whole = m0 + S::WAVE_M <= g.M;  // every row of the granule is a centroid

#pragma unroll
    for (int nb = 0; nb < S::FN; ++nb) {
        const int n = n0 + acc_col(nb, lane);
        const float xn = (n < g.N) ? xnorm[n] : 0.0f;
        // Row m0 + 4 * (lane / 32) may lie past M in the last granule; `have` says whether `best` is a centroid yet.
        float best = FLT_MAX;
        uint32_t best_idx = (uint32_t) (m0 + g.m_base);
        bool have = false;
#pragma unroll
        for (int mb = 0; mb < S::FM; ++mb) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const floatx4 c4 = *reinterpret_cast<const floatx4*>(&cns[acc_row(mb, r4 * 4, lane)]);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int r = r4 * 4 + j;
                    const int m = m0 + acc_row(mb, r, lane);
                    const float v = fmaf(-2.0f, acc.v[mb][nb][r], xn) + c4[j];
                    if ((whole || m < g.M) && (!have || v < best)) {
                        best = v;
                        best_idx = (uint32_t) (m + g.m_base);
                        have = true;
                    }
                }
            }
        }
        // Merge with the other half-wavefront (same point, interleaved rows).
        const float o_best = __shfl_xor(best, 32);
        const uint32_t o_idx = (uint32_t) __shfl_xor((int) best_idx, 32);
        const int o_have = __shfl_xor((int) have, 32);
        if (o_have && (!have || o_best < best || (o_best == best && o_idx < best_idx))) {
            best = o_best;
            best_idx = o_idx;
        }
        if (lane < 32 && n < g.N) {
            granule_min[(int64_t) granule * g.N + n] = make_uint2(__float_as_uint(best), best_idx);
        }
    }
}

template <class S>
static int launch_gemm_argmin_shape(skm_ctx* ctx, const float* C, int k, const float* X, int n, int d,
                                    int64_t ldc, int64_t ldx, const float* xnorm, const float* cnorm,
                                    uint2* granule_min, int first_centroid = 0) {
    GemmOperands g;
    SKM_TRY(fill_operands<S>(g, C, k, ldc, X, n, ldx, d));
    g.m_base = first_centroid;
    const size_t lds_bytes = S::LDS_FLOATS * sizeof(float);
    dim3 grid((unsigned) (g.tiles_m * g.tiles_n)), block(S::THREADS);
    if (gemm_operands_vectorizable(g))
        SKM_LAUNCH_GEMM((gemm_argmin_kernel<true, S>), grid, block, lds_bytes, ctx->stream, g, xnorm, cnorm, granule_min);
    else
        SKM_LAUNCH_GEMM((gemm_argmin_kernel<false, S>), grid, block, lds_bytes, ctx->stream, g, xnorm, cnorm, granule_min);
    return check_hip(hipGetLastError(), "gemm_argmin_kernel launch");
}

// Centroids that the large shape would compute as a nearly empty tile row (k = 10,000 is 39 rows of 256 and 16
// centroids: 2.4 % of the launch for 0.16 % of the work) are searched by a second, thin launch instead, which costs
// one more read of the points.  Returns how many leading centroids go to the main launch; the rest (at most 128, one
// granule slot of the large shape) go to the thin one.
int gemm_argmin_main_rows(int k, int n) {
    const int rest = k % GemmBig::TM;
    if (rest == 0 || rest > GEMM_THIN_MAX_ROWS || k - rest < GemmBig::TM) return k;
    return use_big_tiles(k - rest, n) ? k - rest : k;
}

int gemm_argmin_granule(int k, int n) {
    return use_big_tiles(gemm_argmin_main_rows(k, n), n) ? GemmBig::WAVE_M : GemmSmall::WAVE_M;
}

int launch_gemm_argmin(skm_ctx* ctx, const float* C, int k, const float* X, int n, int d,
                       int64_t ldc, int64_t ldx, const float* xnorm, const float* cnorm,
                       uint2* granule_min, int granule) {
    if (k <= 0 || n <= 0 || d <= 0) return SKM_OK;
    if (granule == GemmBig::WAVE_M) {
        const int k_main = gemm_argmin_main_rows(k, n);
        SKM_TRY(launch_gemm_argmin_shape<GemmBig>(ctx, C, k_main, X, n, d, ldc, ldx, xnorm, cnorm, granule_min));
        if (k_main == k) return SKM_OK;
        // the leftover centroids (at most 128) fill the granule slot that follows the main launch's (k_main is a
        // multiple of 256); the thin shape is as tall as they need, in steps of 32 rows
        const float* c_rest = C + (int64_t) k_main * ldc;
        uint2* slot = granule_min + (int64_t) (k_main / granule) * n;
        const int rest = k - k_main;
        if (rest <= 32)
            return launch_gemm_argmin_shape<GemmThin<1>>(ctx, c_rest, rest, X, n, d, ldc, ldx, xnorm, cnorm + k_main, slot, k_main);
        if (rest <= 64)
            return launch_gemm_argmin_shape<GemmThin<2>>(ctx, c_rest, rest, X, n, d, ldc, ldx, xnorm, cnorm + k_main, slot, k_main);
        if (rest <= 96)
            return launch_gemm_argmin_shape<GemmThin<3>>(ctx, c_rest, rest, X, n, d, ldc, ldx, xnorm, cnorm + k_main, slot, k_main);
        return launch_gemm_argmin_shape<GemmThin<4>>(ctx, c_rest, rest, X, n, d, ldc, ldx, xnorm, cnorm + k_main, slot, k_main);
    }
    if (granule == GemmSmall::WAVE_M) {
        static_assert(GemmHalf::WAVE_M == GemmSmall::WAVE_M, "both shapes fill the same granule slots");
        if (use_half_tiles(k, n))
            return launch_gemm_argmin_shape<GemmHalf>(ctx, C, k, X, n, d, ldc, ldx, xnorm, cnorm, granule_min);
        return launch_gemm_argmin_shape<GemmSmall>(ctx, C, k, X, n, d, ldc, ldx, xnorm, cnorm, granule_min);
    }
    return set_error(SKM_ERR_INVALID, "unsupported argmin granule");
}

// ---------------------------------------------------------------------------------------------
// Partial distances with the first pruning test fused into the epilogue.  Same operand roles as the
// argmin kernel (one point per lane).  A (point, centroid) pair is emitted only when its partial
// distance is below thr0[point] = seed distance * ratios[d'], the loosest threshold that point can
// ever see (its best distance only shrinks from batch to batch, batch_computers.h:372-380), so the
// emitted set is a superset of the reference's survivors of every batch; the pruning kernel re-applies
// the exact per-batch threshold.  Pairs go to a per-point list of `cap` slots; the per-point counter
// keeps counting past `cap` so that overflowing points can be detected and redone densely.
// ---------------------------------------------------------------------------------------------
// One workgroup owns a tile of 128 points and sweeps every 128-centroid tile in ascending order, so
//   * a point's candidates are appended batch after batch (a batch of 1024 centroids = 8 consecutive
//     tiles), which lets the pruning kernel walk its list once;
//   * ||x||^2 and the thresholds of the workgroup's points stay in registers for the whole sweep, the
//     128 centroid norms of a tile are staged through LDS: the epilogue issues no global load.
// d' is short (16 to a few hundred columns), so a tile is only one to a few operand slices long and a
// per-tile prologue would cost as much as the tile.  The slices of all tiles therefore form ONE software
// pipeline: while slice s is multiplied, slice s + 1 sits in the other LDS buffer and slice s + 2 is on
// its way into registers, across tile boundaries; a tile's epilogue runs after the last group of its
// last slice with the loads of the next tiles in flight.  Step s (LDS buffer s & 1):
//   registers (slice s + 1) -> other buffer; request slice s + 2; groups of 8 columns with the next
//   group's fragments fetched ahead; workgroup barrier before the last group; first fragments of slice
//   s + 1; last group; epilogue if the tile ends here.
// FAST: rows are 16-byte aligned and hold at least round_up(d', 32) columns, so every slice is fetched
// without guards; columns at or past d' in the last group are zeroed in the fragments of both operands.
// Otherwise slices are fetched with guards (zeros past d').
// Workgroups of one XCD sweep the centroid tiles roughly in step and share them through that XCD's L2.
template <bool FAST>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_candidates_kernel(
    GemmOperands g, const float* __restrict__ xnorm, const float* __restrict__ cnorm,
    const float* __restrict__ thr0, uint32_t* __restrict__ cand_count, uint2* __restrict__ cand, uint32_t cap
) {
    extern __shared__ float lds[];
    float* As = lds;
    float* Bs = lds + 2 * GEMM_TM * GEMM_LDS_STRIDE;
    float* cn_s = lds + GEMM_LDS_FLOATS;  // [3][GEMM_TM]: tile t uses slot t % 3 (written two tiles ahead of its readers' successors)
    // The workgroup is the only writer of its points' lists, so the slot counters live in LDS.
    uint32_t* cnt_s = reinterpret_cast<uint32_t*>(cn_s + 3 * GEMM_TM);  // [GEMM_TN]
    const int tn = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int ld_row = tid >> 3;
    const int ld_k = (tid & 7) * 4;

    // Rows of the four point rows this thread stages (clamped: padding points never pass).
    const float* b_rows[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        int rb = tn * GEMM_TN + ld_row + 32 * p;
        rb = rb < g.N ? rb : g.N - 1;
        b_rows[p] = g.B + (int64_t) rb * g.ldb + ld_k;
    }
    // The two points of this lane.
    int pt[2];
    float xn[2], thr[2];
    uint2* list[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        pt[nb] = tn * GEMM_TN + wn * 64 + acc_col(nb, lane);
        const bool valid = pt[nb] < g.N;
        xn[nb] = valid ? xnorm[pt[nb]] : 0.0f;
        thr[nb] = valid ? thr0[pt[nb]] : -3.0e38f;  // nothing passes for padding columns
        list[nb] = cand + (int64_t) (valid ? pt[nb] : 0) * cap;
    }

    const int nk = (g.K + GEMM_BK - 1) / GEMM_BK;              // slices per tile
    const int last_groups = (g.K - (nk - 1) * GEMM_BK + 7) / 8;  // groups of 8 columns in a tile's last slice
    const int total = g.tiles_m * nk;                           // slices of the whole sweep
    // FAST: columns of the last group at or past d' (this lane supplies columns 4 * (lane / 32) + i of a group).
    const int last_col0 = (nk - 1) * GEMM_BK + (last_groups - 1) * 8 + (lane >> 5) * 4;
    floatx4 ra[4], rb[4];
    float cn_next = 0.0f;

    // Slice (tm, kt) -> registers, together with one centroid norm of that tile per thread.  Every load is
    // unconditional (a load under a condition would have to be waited for right where it is issued).
    auto request = [&](int tm, int kt) {
        const int k0 = kt * GEMM_BK;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            int r = tm * GEMM_TM + ld_row + 32 * p;
            r = r < g.M ? r : g.M - 1;
            const float* a_row = g.A + (int64_t) r * g.lda;
            if (FAST) {
                ra[p] = load_k4<true, false>(a_row + ld_k, k0, g.K);
                rb[p] = load_k4<true, false>(b_rows[p], k0, g.K);
            } else {
                ra[p] = load_k4<false, true>(a_row, k0 + ld_k, g.K);
                rb[p] = load_k4<false, true>(b_rows[p] - ld_k, k0 + ld_k, g.K);
            }
        }
        const int m = tm * GEMM_TM + (tid & (GEMM_TM - 1));
        cn_next = cnorm[m < g.M ? m : g.M - 1];
    };
    const int st_off = ld_row * GEMM_LDS_STRIDE + ld_k;
    // Registers -> LDS buffer `buf`; `first_of` >= 0: the slice opens tile `first_of`, whose norms go along
    // (rows past M get a norm nothing passes with).
    auto publish = [&](int buf, int first_of) {
        float* as = As + buf * GEMM_TM * GEMM_LDS_STRIDE + st_off;
        float* bs = Bs + buf * GEMM_TN * GEMM_LDS_STRIDE + st_off;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            *reinterpret_cast<floatx4*>(&as[32 * p * GEMM_LDS_STRIDE]) = ra[p];
            *reinterpret_cast<floatx4*>(&bs[32 * p * GEMM_LDS_STRIDE]) = rb[p];
        }
        if (first_of >= 0 && tid < GEMM_TM)
            cn_s[(first_of % 3) * GEMM_TM + tid] = (first_of * GEMM_TM + tid < g.M) ? cn_next : 3.0e38f;
    };
    const int frag_off = (lane & 31) * GEMM_LDS_STRIDE + (lane >> 5) * 4;
    const int a_frag = (wm * 64) * GEMM_LDS_STRIDE + frag_off;
    const int b_frag = (wn * 64) * GEMM_LDS_STRIDE + frag_off;
    auto fetch = [&](int buf, int kg, floatx4& f0, floatx4& f1, floatx4& g0, floatx4& g1) {
        const float* as = As + buf * GEMM_TM * GEMM_LDS_STRIDE + a_frag + kg * 8;
        const float* bs = Bs + buf * GEMM_TN * GEMM_LDS_STRIDE + b_frag + kg * 8;
        f0 = *reinterpret_cast<const floatx4*>(as);
        f1 = *reinterpret_cast<const floatx4*>(as + 32 * GEMM_LDS_STRIDE);
        g0 = *reinterpret_cast<const floatx4*>(bs);
        g1 = *reinterpret_cast<const floatx4*>(bs + 32 * GEMM_LDS_STRIDE);
    };

    WaveAcc acc;
    auto clear = [&]() {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc.v[mb][nb][r] = 0.0f;
    };

    // First pruning test of tile tm and the appends to the per-point lists.  Passing pairs are rare (a fraction
    // of a percent).  The outcome of the 32 tests of one point is collected in a per-lane bit mask (the sign of
    // v - thr is shifted in, so a test costs four vector instructions and no scalar dependency); lanes with an
    // empty mask skip the append.
    auto epilogue = [&](int tm) {
        const float* cns = cn_s + (tm % 3) * GEMM_TM + wm * 64;
        const int m0 = tm * GEMM_TM + wm * 64;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            uint32_t pass = 0;  // element (mb, r) lands in bit 31 - (mb * 16 + r)
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const floatx4 c4 = *reinterpret_cast<const floatx4*>(&cns[acc_row(mb, r4 * 4, lane)]);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int r = r4 * 4 + j;
                        const float v = fmaf(-2.0f, acc.v[mb][nb][r], xn[nb]) + c4[j];
                        acc.v[mb][nb][r] = v;
                        // v < thr  <=>  the IEEE difference v - thr carries a set sign bit.
                        pass = __builtin_amdgcn_alignbit(pass, __float_as_uint(v - thr[nb]), 31);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // bounds how many norms are held at once
            }
            if (pass) {
                uint32_t slot = atomicAdd(&cnt_s[wn * 64 + acc_col(nb, lane)], (uint32_t) __popc(pass));
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        if (pass & (0x80000000u >> (mb * 16 + r))) {
                            if (slot < cap)
                                list[nb][slot] = make_uint2((uint32_t) (m0 + acc_row(mb, r, lane)), __float_as_uint(acc.v[mb][nb][r]));
                            ++slot;
                        }
                    }
            }
        }
    };

    // Prologue: slice 0 in buffer 0, slice 1 in registers, first fragments of slice 0 fetched.  The request
    // cursor stops at the last slice: requests past the end fetch that slice again and are never published.
    int req_tm = 0, req_kt = 0;
    auto advance_cursor = [&]() {
        if (req_kt + 1 < nk) {
            ++req_kt;
        } else if (req_tm + 1 < g.tiles_m) {
            req_kt = 0;
            ++req_tm;
        }
    };
    if (tid < GEMM_TN) cnt_s[tid] = 0u;
    request(0, 0);
    advance_cursor();
    publish(0, 0);
    int pub_tm = req_tm, pub_kt = req_kt;  // slice held in the registers (next to publish)
    request(req_tm, req_kt);
    advance_cursor();
    __syncthreads();
    floatx4 a0, a1, b0, b1;
    fetch(0, 0, a0, a1, b0, b1);
    clear();

    int s = 0;
    for (int tm = 0; tm < g.tiles_m; ++tm) {
        for (int kt = 0; kt < nk; ++kt, ++s) {
            const int cur = s & 1;
            const bool last = kt + 1 == nk;
            if (s + 1 < total) publish(cur ^ 1, pub_kt == 0 ? pub_tm : -1);
            pub_tm = req_tm;
            pub_kt = req_kt;
            request(req_tm, req_kt);
            advance_cursor();
            __builtin_amdgcn_sched_barrier(0);
            // The accumulators flow through one straight line of code: a branch around MFMAs would make the
            // register allocator keep two copies of them.
            floatx4 na0, na1, nb0, nb1;
            const int n_ahead = (last ? last_groups : GEMM_BK / 8) - 1;
            for (int kg = 0; kg < n_ahead; ++kg) {
                fetch(cur, kg + 1, na0, na1, nb0, nb1);
                mfma_group(a0, a1, b0, b1, acc);
                a0 = na0; a1 = na1; b0 = nb0; b1 = nb1;
            }
            if (FAST) {
                // zero the columns at or past d' in the last group of the tile's last slice (both operands, so that
                // whatever lies there, even a non-finite value, contributes an exact zero)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool live = !last || last_col0 + i < g.K;
                    a0[i] = live ? a0[i] : 0.0f;
                    a1[i] = live ? a1[i] : 0.0f;
                    b0[i] = live ? b0[i] : 0.0f;
                    b1[i] = live ? b1[i] : 0.0f;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();  // every read of buffer `cur` has returned, slice s + 1 is complete in the other one
            fetch(cur ^ 1, 0, na0, na1, nb0, nb1);  // past the last slice: stale data, never used
            __builtin_amdgcn_sched_barrier(0);
            mfma_group(a0, a1, b0, b1, acc);
            a0 = na0; a1 = na1; b0 = nb0; b1 = nb1;
            if (last) {
                epilogue(tm);
                clear();
            }
        }
    }
    __syncthreads();
    if (tid < GEMM_TN && tn * GEMM_TN + tid < g.N) cand_count[tn * GEMM_TN + tid] = cnt_s[tid];
}

// ---------------------------------------------------------------------------------------------
// The same contract for long d' (from about 160 leading dimensions on): a tile is then many operand slices long, the
// per-tile prologue is a few per cent of the tile, and what counts is the main loop.  A workgroup of the large shape
// (8 wavefronts of 128 x 64, one per CU) owns 256 points and sweeps the 256-centroid tiles in ascending order (a batch
// of 1024 centroids is four consecutive tiles, so a point's candidates are still appended batch after batch) with the
// tile loop of the GEMM core: per MFMA half the global loads, LDS stores and barriers of the 128 x 128 shape.  The
// epilogue is gemm_candidates_kernel's on 4 x 2 accumulator blocks: the norms of the tile's centroids come from LDS
// (two slots: tile t + 1 writes the slot tile t - 1 read, and every wavefront has passed a barrier of tile t's loop in
// between), the 64 tests of a point are shifted into two bit masks, lanes with a bit append.  Products are accumulated
// in the order of every other shape, so the emitted pairs carry the same bits.
// ---------------------------------------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(GemmBig::THREADS, 1) void gemm_candidates_big_kernel(
    GemmOperands g, const float* __restrict__ xnorm, const float* __restrict__ cnorm,
    const float* __restrict__ thr0, uint32_t* __restrict__ cand_count, uint2* __restrict__ cand, uint32_t cap
) {
    using S = GemmBig;
    extern __shared__ float lds[];
    float* cn_s = lds + S::LDS_FLOATS;                                      // [2][TM]
    uint32_t* cnt_s = reinterpret_cast<uint32_t*>(cn_s + 2 * S::TM);        // [TN]
    const int tn = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / S::WN, wn = wave % S::WN;

    // |x|^2 and the threshold of the workgroup's points wait in LDS for the epilogues: held in registers across the
    // tile loop they would not fit next to its 128 accumulators
    float2* pt_s = reinterpret_cast<float2*>(cnt_s + S::TN);  // [TN] {|x|^2, threshold}
    if (tid < S::TN) {
        const int p = tn * S::TN + tid;
        const bool valid = p < g.N;
        pt_s[tid] = make_float2(valid ? xnorm[p] : 0.0f, valid ? thr0[p] : -3.0e38f);  // nothing passes for padding columns
        cnt_s[tid] = 0u;
    }

    for (int tm = 0; tm < g.tiles_m; ++tm) {
        if (tid < S::TM) {
            const int m = tm * S::TM + tid;
            cn_s[(tm & 1) * S::TM + tid] = m < g.M ? cnorm[m] : 3.0e38f;  // rows past M never pass
        }
        WaveAccT<S::FM, S::FN> acc;
        gemm_tile<VEC, S>(g, tm, tn, lds, acc);  // its barriers order the norms (and cnt_s) before the epilogue

        const float* cns = cn_s + (tm & 1) * S::TM + wm * S::WAVE_M;
        const int m0 = tm * S::TM + wm * S::WAVE_M;
#pragma unroll
        for (int nb = 0; nb < S::FN; ++nb) {
            const int col = wn * S::WAVE_N + acc_col(nb, lane);
            const float2 xt = pt_s[col];
            const float xn = xt.x, thr = xt.y;
            uint32_t pass[S::FM / 2];  // element (mb, r) lands in bit 31 - ((mb % 2) * 16 + r) of pass[mb / 2]
#pragma unroll
            for (int h = 0; h < S::FM / 2; ++h) pass[h] = 0u;
#pragma unroll
            for (int mb = 0; mb < S::FM; ++mb) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const floatx4 c4 = *reinterpret_cast<const floatx4*>(&cns[acc_row(mb, r4 * 4, lane)]);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int r = r4 * 4 + j;
                        const float v = fmaf(-2.0f, acc.v[mb][nb][r], xn) + c4[j];
                        acc.v[mb][nb][r] = v;
                        // v < thr  <=>  the IEEE difference v - thr carries a set sign bit.
                        pass[mb / 2] = __builtin_amdgcn_alignbit(pass[mb / 2], __float_as_uint(v - thr), 31);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // bounds how many norms are held at once
            }
            uint32_t any = 0u, total = 0u;
#pragma unroll
            for (int h = 0; h < S::FM / 2; ++h) {
                any |= pass[h];
                total += (uint32_t) __popc(pass[h]);
            }
            if (any) {
                uint32_t slot = atomicAdd(&cnt_s[col], total);
                const int p = tn * S::TN + col;  // a padding column has no bit set
                uint2* const list = cand + (int64_t) p * cap;
#pragma unroll
                for (int mb = 0; mb < S::FM; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        if (pass[mb / 2] & (0x80000000u >> ((mb % 2) * 16 + r))) {
                            if (slot < cap)
                                list[slot] = make_uint2((uint32_t) (m0 + acc_row(mb, r, lane)), __float_as_uint(acc.v[mb][nb][r]));
                            ++slot;
                        }
                    }
            }
        }
    }
    __syncthreads();
    if (tid < S::TN && tn * S::TN + tid < g.N) cand_count[tn * S::TN + tid] = cnt_s[tid];
}

// The large shape serves long d' on enough points to fill the chip with 256-point workgroups.
constexpr int CANDIDATES_BIG_MIN_D = 161;
constexpr int CANDIDATES_BIG_MIN_POINTS = 192 * GemmBig::TN;

int launch_gemm_candidates(skm_ctx* ctx, const float* C, int k, const float* X, int n, int partial_d, int64_t ld,
                           const float* xnorm_p, const float* cnorm_p, const float* thr0, uint32_t* cand_count,
                           uint2* cand, uint32_t cap) {
    if (k <= 0 || n <= 0 || partial_d <= 0) return SKM_OK;
    GemmOperands g;
    if (ctx->candidate_kernel == 3 ||
        (partial_d >= CANDIDATES_BIG_MIN_D && n >= CANDIDATES_BIG_MIN_POINTS && ctx->candidate_kernel != 1)) {
        SKM_TRY(fill_operands<GemmBig>(g, C, k, ld, X, n, ld, partial_d));
        const size_t lds_bytes = (GemmBig::LDS_FLOATS + 2 * GemmBig::TM + 3 * GemmBig::TN) * sizeof(float);
        dim3 grid((unsigned) g.tiles_n), block(GemmBig::THREADS);
        if (gemm_operands_vectorizable(g))
            SKM_LAUNCH_GEMM((gemm_candidates_big_kernel<true>), grid, block, lds_bytes, ctx->stream, g, xnorm_p, cnorm_p, thr0, cand_count, cand, cap);
        else
            SKM_LAUNCH_GEMM((gemm_candidates_big_kernel<false>), grid, block, lds_bytes, ctx->stream, g, xnorm_p, cnorm_p, thr0, cand_count, cand, cap);
        return check_hip(hipGetLastError(), "gemm_candidates_big_kernel launch");
    }
    SKM_TRY(fill_operands<GemmSmall>(g, C, k, ld, X, n, ld, partial_d));
    const size_t lds_bytes = (GEMM_LDS_FLOATS + 3 * GEMM_TM + GEMM_TN) * sizeof(float);
    dim3 grid((unsigned) g.tiles_n), block(GEMM_THREADS);
    const int64_t padded_k = ((int64_t) partial_d + GEMM_BK - 1) / GEMM_BK * GEMM_BK;
    if (gemm_operands_vectorizable(g) && padded_k <= ld)
        SKM_LAUNCH_GEMM((gemm_candidates_kernel<true>), grid, block, lds_bytes, ctx->stream, g, xnorm_p, cnorm_p, thr0, cand_count, cand, cap);
    else
        SKM_LAUNCH_GEMM((gemm_candidates_kernel<false>), grid, block, lds_bytes, ctx->stream, g, xnorm_p, cnorm_p, thr0, cand_count, cand, cap);
    return check_hip(hipGetLastError(), "gemm_candidates_kernel launch");
}

// ---------------------------------------------------------------------------------------------
// Sequential merge of granule minima, reproducing batch_computers.h:118,162-167:
//   out = FLT_MAX; for each batch of 1024 centroids in order:
//       m = first minimum of the batch;  if (m < out) { out = max(0, m); idx = argmin; }
// ---------------------------------------------------------------------------------------------
__global__ void merge_granules_kernel(
    const uint2* __restrict__ granule_min, int n, int k, int granule, uint32_t* __restrict__ out_idx,
    float* __restrict__ out_dist
) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int n_granules = (k + granule - 1) / granule;
    const int per_batch = SKM_Y_BATCH_SIZE / granule;
    float out = FLT_MAX;
    uint32_t idx = 0;
    for (int g0 = 0; g0 < n_granules; g0 += per_batch) {
        float bm = 0.0f;
        uint32_t bi = 0;
        const int g1 = (g0 + per_batch < n_granules) ? g0 + per_batch : n_granules;
        for (int g = g0; g < g1; ++g) {
            const uint2 e = granule_min[(int64_t) g * n + i];
            const float v = __uint_as_float(e.x);
            if (g == g0 || v < bm) {
                bm = v;
                bi = e.y;
            }
        }
        if (bm < out) {
            out = fmaxf(0.0f, bm);
            idx = bi;
        }
    }
    out_idx[i] = idx;
    out_dist[i] = out;
}

int launch_merge_granules(skm_ctx* ctx, const uint2* granule_min, int n, int k, int granule, uint32_t* out_idx,
                          float* out_dist) {
    if (n <= 0) return SKM_OK;
    dim3 grid((n + 255) / 256), block(256);
    hipLaunchKernelGGL(merge_granules_kernel, grid, block, 0, ctx->stream, granule_min, n, k, granule, out_idx, out_dist);
    return check_hip(hipGetLastError(), "merge_granules_kernel launch");
}

} // namespace skm
