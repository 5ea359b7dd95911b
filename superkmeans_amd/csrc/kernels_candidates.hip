// Partial distances with the first pruning test fused in, for short d' (at most 8 * CS_MAX_GROUPS leading
// dimensions): the point operand never leaves the registers.
//
// Same contract as gemm_candidates_kernel (kernels_gemm.hip): for every point the pairs (centroid, partial
// distance over the first d' rotated dimensions, batch_computers.h:344-366) whose distance is below
// thr0[point] are appended to the point's list, batch after batch.  The arithmetic of a distance is the same
// instruction sequence (v_mfma_f32_32x32x2_f32 over ascending groups of 8 columns, then
// fma(-2, dot, |x|^2) + |c|^2), so both kernels emit the same pairs with the same bits.
//
// On this hardware fp32 MFMAs and ordinary vector instructions do not run side by side on a SIMD, whichever
// wavefront they come from (a wavefront of back-to-back MFMAs next to a wavefront of vector instructions takes the
// sum of their times): every vector instruction of the epilogue is paid in MFMA time.  At d' = 24 a tile of
// 64 x 64 distances is 48 MFMAs = 3,072 cycles, so the test has to cost well under one vector instruction per
// distance.  Shape of the work:
//   * a workgroup is 4 wavefronts and owns 256 points; a wavefront owns 64 of them and holds their first d'
//     columns as MFMA row-operand fragments in registers for the whole sweep (8 registers per group of 8 columns).
//     Only centroid tiles (64 centroids x d' columns) stream through LDS: per flop a quarter of the global loads
//     and LDS stores and half the LDS reads of the 128 x 128 kernel, and half as many sweeps of the centroids;
//   * a whole tile is one pipeline step: tile t + 1 sits in the other LDS buffer while tile t is multiplied and
//     tile t + 2 is on its way into registers; one workgroup barrier per tile;
//   * sign test: one more MFMA per 32 x 32 block adds (thr0 - |x|^2) / 2 (row operand) and -|c|^2 / 2 (column
//     operand) to a copy of the accumulators, which turns "distance < thr0" into "value >= 0".  Both addends carry
//     a relative slack of 2^-17, far above the rounding of either formula, so the sign can only flag too many
//     pairs, never too few.  The 16 sign bits of a block are shifted into one register per lane (one instruction
//     per accumulator register);
//   * the two half-wavefronts, which hold rows 0-3 and 4-7 (mod 8) of a column, exchange their sign registers
//     (v_permlane32_swap), after which every lane owns ONE CENTROID of the tile and a bit per point.  Lanes then
//     walk their own bits.  Candidates pile up on few points (a point with a loose threshold passes hundreds of
//     centroids) but spread evenly over centroids, so walking per centroid keeps the 64 lanes about equally busy;
//     walking per point took three times as many rounds;
//   * a round of the walk: the accumulator named by the bit comes from the wavefront's LDS copy of the block row,
//     the point's |x|^2, threshold and list address from an LDS table in bit order, and the list slot from an LDS
//     atomic on the point's counter, all requested together (one LDS round trip per candidate); then the exact
//     distance and the exact test.  The slot is taken before the exact test is known: where the exact test fails
//     (two in ten thousand flagged pairs) the slot receives the centroid with distance +inf, which no threshold
//     of the pruning kernel lets through.
#include "gemm_core.h"
#include "skm_internal.h"

namespace skm {

constexpr int CS_POINTS = 256;  // per workgroup: 4 wavefronts of 64 points (d' <= 88) or 8 wavefronts of 32 points
constexpr int CS_TN = 64;       // centroids per tile
constexpr float CS_SLACK = 1.0f / 131072.0f;
constexpr float CS_NEVER = -1.5e38f;  // addend of rows and columns that must not pass

// Per point of a wavefront, in the order of the sign bits (see emit): what a lane needs to append to that point's list.
struct __attribute__((aligned(16))) CsPoint {
    float xn;          // |x|^2 over the first d' dimensions
    float thr;         // first-test threshold
    uint32_t list_off; // byte offset of the point's list from the wavefront's first list
    uint32_t count;    // candidates so far (keeps counting past the capacity)
};

// Row of a 32-row accumulator block row that sign bit `bit` stands for: bits 0-15 are the registers of the lanes
// 0-31 (rows 8 (r / 4) + r % 4), bits 16-31 those of the lanes 32-63 (4 rows further down).
__device__ __forceinline__ int cs_row_of_bit(int bit) {
    return 8 * ((bit & 15) >> 2) + 4 * (bit >> 4) + (bit & 3);
}

// NG: groups of 8 columns, ceil(d' / 8).  FM: 32-point accumulator block rows per wavefront (2 or 1); the wavefronts of
// a workgroup are 8 / FM, so that it always owns 256 points and streams a centroid tile once for all of them.
template <int NG, int FM>
__global__ __launch_bounds__(512 / FM, FM) void gemm_candidates_stationary_kernel(
    const float* __restrict__ C, int M, const float* __restrict__ X, int N, int K, int64_t ld,
    const float* __restrict__ xnorm, const float* __restrict__ cnorm, const float* __restrict__ thr0,
    uint32_t* __restrict__ cand_count, uint2* __restrict__ cand, uint32_t cap
) {
    constexpr int WAVES = 8 / FM, CS_THREADS = 64 * WAVES;
    constexpr int S = NG * 8 + 4;           // LDS row stride in floats: 16-byte fragment reads of 32 rows hit all banks
    constexpr int CHUNKS = CS_TN * NG * 2;  // 16-byte pieces of a tile
    constexpr int NL = (CHUNKS + CS_THREADS - 1) / CS_THREADS;
    constexpr bool RAGGED = CHUNKS % CS_THREADS != 0;  // NG odd: the last load of half the threads has no piece
    extern __shared__ __attribute__((aligned(16))) float cs_lds[];
    float (*Bs)[CS_TN * S] = reinterpret_cast<float (*)[CS_TN * S]>(cs_lds);  // [2]: centroid tiles
    float* const dump_all = cs_lds + 2 * CS_TN * S;                                     // [WAVES][32 bits][64 centroids]
    CsPoint* const table_all = reinterpret_cast<CsPoint*>(dump_all + WAVES * 32 * 64);  // [WAVES][FM block rows][32 bits]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;  // which 4 of every 8 accumulator rows / which 4 of every 8 columns this lane feeds
    const int wave_pt0 = blockIdx.x * CS_POINTS + wave * (32 * FM);
    float* const dump = dump_all + wave * (32 * 64);
    CsPoint* const table = table_all + wave * (32 * FM);

    // ---- per point: table entry (lane j fills entry j = 32 mb + bit) and row addend of the sign test ----
    if (lane < 32 * FM) {
        const int local = (lane & 32) + cs_row_of_bit(lane & 31);
        const int pt = wave_pt0 + local;
        CsPoint e;
        e.xn = pt < N ? xnorm[pt] : 0.0f;
        e.thr = pt < N ? thr0[pt] : -3.0e38f;
        e.list_off = (uint32_t) local * cap * (uint32_t) sizeof(uint2);
        e.count = 0u;
        table[lane] = e;
    }
    // MFMA row operand of the extra step: k = 0 (lanes 0-31) supplies (thr - |x|^2) / 2 plus slack for point
    // mb * 32 + lane, k = 1 (lanes 32-63) multiplies the column addend by 1
    float a_aug[FM];
#pragma unroll
    for (int mb = 0; mb < FM; ++mb) {
        const int pt = wave_pt0 + mb * 32 + (lane & 31);
        const float xn = pt < N ? xnorm[pt] : 0.0f;
        const float thr = pt < N ? thr0[pt] : -3.0e38f;
        a_aug[mb] = half ? 1.0f : 0.5f * (thr - xn) + CS_SLACK * (xn + fabsf(thr));
    }
    // first list of the wavefront; a point's list starts list_off bytes further
    char* const wave_lists = reinterpret_cast<char*>(cand + (int64_t) wave_pt0 * cap);

    // ---- point fragments: a[kg][mb] = columns kg * 8 + half * 4 .. + 3 of point mb * 32 + lane % 32 ----
    floatx4 a[NG][FM];
#pragma unroll
    for (int mb = 0; mb < FM; ++mb) {
        int q = wave_pt0 + mb * 32 + (lane & 31);
        q = q < N ? q : N - 1;
        const float* row = X + (int64_t) q * ld + half * 4;
#pragma unroll
        for (int kg = 0; kg < NG; ++kg) a[kg][mb] = *reinterpret_cast<const floatx4*>(row + kg * 8);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if ((NG - 1) * 8 + half * 4 + i >= K) a[NG - 1][mb][i] = 0.0f;
    }

    // ---- centroid tiles: global -> registers -> LDS ----
    // Piece c = tid + 256 p of a tile is 16 bytes of row c / (2 NG) at column 4 (c % (2 NG)).  Rows at or past M
    // (the last tile, and the tiles the pipeline requests past the end) lie outside the buffer descriptor and
    // read as zeros.
    const __amdgpu_buffer_rsrc_t c_desc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(C), 0, (int) ((uint32_t) M * (uint32_t) ld * 4u), 0x00020000);
    uint32_t voff[NL];
    int lds_off[NL];
#pragma unroll
    for (int p = 0; p < NL; ++p) {
        int c = tid + CS_THREADS * p;
        if (RAGGED && c >= CHUNKS) c = CHUNKS - 1;  // loaded again, not stored
        const int r = c / (2 * NG), c4 = c % (2 * NG);
        voff[p] = ((uint32_t) r * (uint32_t) ld + (uint32_t) c4 * 4u) * 4u;
        lds_off[p] = r * S + c4 * 4;
    }
    const uint32_t tile_bytes = (uint32_t) CS_TN * (uint32_t) ld * 4u;
    floatx4 rb[NL];
    auto request = [&](int tile) {
        const uint32_t base = (uint32_t) tile * tile_bytes;
#pragma unroll
        for (int p = 0; p < NL; ++p)
            rb[p] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(c_desc, (int) (voff[p] + base), 0, 0));
    };
    auto publish = [&](int buf) {
#pragma unroll
        for (int p = 0; p < NL; ++p)
            if (!RAGGED || p + 1 < NL || tid + CS_THREADS * p < CHUNKS)
                *reinterpret_cast<floatx4*>(&Bs[buf][lds_off[p]]) = rb[p];
    };
    // squared norms of the tile's centroids: of the lane's own centroid (tile column `lane`) and of column lane % 32
    float cn_own = 0.0f, cn_low = 0.0f;
    bool own_live = false, low_live = false;  // the column is a centroid (false before the first tile)
    auto request_norms = [&](int tile) {
        const int m_own = tile * CS_TN + lane, m_low = tile * CS_TN + (lane & 31);
        own_live = m_own < M;
        low_live = m_low < M;
        cn_own = cnorm[own_live ? m_own : M - 1];
        cn_low = cnorm[low_live ? m_low : M - 1];
    };

    const int frag_off = (lane & 31) * S + half * 4;
    floatx4 fb0, fb1;
    auto fetch = [&](int buf, int kg, floatx4& f0, floatx4& f1) {
        const float* bs = &Bs[buf][frag_off + kg * 8];
        f0 = *reinterpret_cast<const floatx4*>(bs);
        f1 = *reinterpret_cast<const floatx4*>(bs + 32 * S);
    };

    // acc.v[mb][nb][r] of lane l: point mb * 32 + 8 (r / 4) + 4 (l / 32) + r % 4, centroid nb * 32 + l % 32
    WaveAccT<FM, 2> acc;
#pragma unroll
    for (int mb = 0; mb < FM; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc.v[mb][nb][r] = 0.0f;

    // Products of tile `buf`; the fragments of its first group are already in fb0 / fb1.
    auto multiply = [&](int buf) {
#pragma unroll
        for (int kg = 0; kg < NG; ++kg) {
            floatx4 nb0, nb1;
            if (kg + 1 < NG) fetch(buf, kg + 1, nb0, nb1);
            if (kg == NG - 1) {
                // columns at or past d' contribute exact zeros whatever lies there (both operands are cleared)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool live = (NG - 1) * 8 + half * 4 + i < K;
                    fb0[i] = live ? fb0[i] : 0.0f;
                    fb1[i] = live ? fb1[i] : 0.0f;
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int mb = 0; mb < FM; ++mb) {
                    if (kg == 0 && i == 0) {
                        const floatx16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                        acc.v[mb][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kg][mb][i], fb0[i], zero, 0, 0, 0);
                        acc.v[mb][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kg][mb][i], fb1[i], zero, 0, 0, 0);
                    } else {
                        acc.v[mb][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kg][mb][i], fb0[i], acc.v[mb][0], 0, 0, 0);
                        acc.v[mb][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kg][mb][i], fb1[i], acc.v[mb][1], 0, 0, 0);
                    }
                }
            }
            if (kg + 1 < NG) {
                fb0 = nb0;
                fb1 = nb1;
            }
        }
    };

    // First test of the tile whose products are in `acc` and whose norms are in cn_own / cn_low, and the appends.
    auto emit = [&](int tile) {
        // column operand of the extra step: k = 0 (lanes 0-31) multiplies the row addend by 1, k = 1 (lanes 32-63)
        // supplies -|c|^2 / 2 with slack for centroid nb * 32 + lane % 32 (for nb = 1 that is the lane's own column)
        float b_aug[2];
        b_aug[0] = half ? (low_live ? -0.5f * (1.0f - CS_SLACK) * cn_low : CS_NEVER) : 1.0f;
        b_aug[1] = half ? (own_live ? -0.5f * (1.0f - CS_SLACK) * cn_own : CS_NEVER) : 1.0f;
        const uint32_t centroid = (uint32_t) (tile * CS_TN + lane);
#pragma unroll
        for (int mb = 0; mb < FM; ++mb) {
            // dump[bit][centroid] = product of the point of that bit with that centroid.  Written for every block
            // row, candidates or not: LDS traffic runs beside the MFMAs, vector instructions do not, and with the
            // products safe in LDS the sign test may overwrite the accumulators (a copy would cost 32 moves).
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 16; ++r) dump[(half * 16 + r) * 64 + nb * 32 + (lane & 31)] = acc.v[mb][nb][r];
            uint32_t negative[2];
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                acc.v[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_aug[mb], b_aug[nb], acc.v[mb][nb], 0, 0, 0);
                uint32_t bits = 0;
#pragma unroll
                for (int r = 15; r >= 0; --r) bits = __builtin_amdgcn_alignbit(bits, __float_as_uint(acc.v[mb][nb][r]), 31);
                negative[nb] = bits;  // bit r: the value carries a set sign bit (no candidate)
            }
            // lanes 0-31 keep their low-row bits of column block 0 and receive its high-row bits from lanes 32-63;
            // lanes 32-63 receive the low-row bits of column block 1 from lanes 0-31 and keep their high-row bits:
            // lane l then holds the 32 bits of centroid l of the tile
            const auto sw = __builtin_amdgcn_permlane32_swap(negative[0], negative[1], false, false);
            uint32_t mask = ~((sw[0] & 0xffffu) | (sw[1] << 16));
            if (__builtin_amdgcn_ballot_w64(mask != 0u) == 0ull) continue;
            __builtin_amdgcn_wave_barrier();  // LDS serves a wavefront's requests in order: the reads below see the writes
            CsPoint* const points = table + mb * 32;
            for (;;) {
                const bool active = mask != 0u;
                if (__builtin_amdgcn_ballot_w64(active) == 0ull) break;
                // lanes without a bit left read along (bit 31) and append nothing
                const int bit = __builtin_ctz(mask | 0x80000000u);
                mask &= mask - 1u;
                float dot = dump[bit * 64 + lane];
                float xn = points[bit].xn;
                float thr = points[bit].thr;
                uint32_t list_off = points[bit].list_off;
                uint32_t slot = 0xffffffffu;
                if (active) slot = atomicAdd(&points[bit].count, 1u);
                // all four LDS requests are on their way before the first result is used (one round trip)
                asm volatile("" : "+v"(dot), "+v"(xn), "+v"(thr), "+v"(list_off), "+v"(slot));
                float v = fmaf(-2.0f, dot, xn) + cn_own;
                v = v < thr ? v : __builtin_inff();
                if (slot < cap)
                    *reinterpret_cast<uint2*>(wave_lists + list_off + slot * (uint32_t) sizeof(uint2)) =
                        make_uint2(centroid, __float_as_uint(v));
            }
            __builtin_amdgcn_wave_barrier();
        }
    };

    // ---- sweep: step t publishes tile t + 1, tests tile t - 1, requests tile t + 2 and multiplies tile t ----
    // The appends of a step are issued before its loads, so waiting for those loads a step later never waits
    // for stores.  Step 0 tests nothing; the last step multiplies a tile past the end (zeros).
    const int tiles = (M + CS_TN - 1) / CS_TN;
    request(0);
    publish(0);
    request(1);
    __syncthreads();  // also: the point tables are complete
    fetch(0, 0, fb0, fb1);
    for (int t = 0; t <= tiles; ++t) {
        publish((t + 1) & 1);
        if (t > 0) emit(t - 1);
        request(t + 2);
        request_norms(t);
        __builtin_amdgcn_sched_barrier(0);
        multiply(t & 1);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();  // every read of buffer t & 1 has returned, tile t + 1 is complete in the other one
        fetch((t + 1) & 1, 0, fb0, fb1);
    }
    if (lane < 32 * FM) {
        const int pt = wave_pt0 + (lane & 32) + cs_row_of_bit(lane & 31);
        if (pt < N) cand_count[pt] = table[lane].count;
    }
}

// Up to 11 groups of 8 columns a wavefront holds the fragments of 64 points next to its 64 x 64 accumulators
// (256 registers) and up to 10 groups two such workgroups of 4 wavefronts share a CU (79,872 bytes of LDS each; at 11
// groups 83,968 bytes, so one workgroup has the CU to itself: measured at d' = 83 and 88 that is as fast as, or 2 %
// faster than, the 8-wavefront shape); from 12 to 20 groups a wavefront holds 32 points and one workgroup of 8
// wavefronts has the CU's LDS to itself.
constexpr int CS_MAX_GROUPS_WIDE = 11;
constexpr int CS_MAX_GROUPS = 20;

template <int NG>
static int launch_stationary(skm_ctx* ctx, dim3 grid, const float* C, int k, const float* X, int n, int partial_d, int64_t ld,
                             const float* xnorm_p, const float* cnorm_p, const float* thr0, uint32_t* cand_count,
                             uint2* cand, uint32_t cap) {
    constexpr int FM = NG <= CS_MAX_GROUPS_WIDE ? 2 : 1;
    constexpr int WAVES = 8 / FM;
    const size_t lds_bytes = (2 * CS_TN * (NG * 8 + 4) + WAVES * 32 * 64) * sizeof(float) + WAVES * 32 * FM * sizeof(CsPoint);
    // above 64 KiB a kernel has to opt in; once per instantiation and process
    static const int lds_rc = check_hip(
        hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_candidates_stationary_kernel<NG, FM>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds_bytes),
        "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    SKM_TRY(lds_rc);
    hipLaunchKernelGGL((gemm_candidates_stationary_kernel<NG, FM>), grid, dim3(64 * WAVES), lds_bytes, ctx->stream, C, k, X, n,
                       partial_d, ld, xnorm_p, cnorm_p, thr0, cand_count, cand, cap);
    return SKM_OK;
}

// Whether the register-stationary kernel serves this call; otherwise gemm_candidates_kernel does.
bool gemm_candidates_stationary_serves(const float* C, int k, const float* X, int n, int partial_d, int64_t ld,
                                       bool whatever_n) {
    const int groups = (partial_d + 7) / 8;
    if (groups > CS_MAX_GROUPS) return false;
    // 16-byte loads of whole groups of 8 columns, rows at least that long
    if (reinterpret_cast<uintptr_t>(C) % 16 != 0 || reinterpret_cast<uintptr_t>(X) % 16 != 0 || ld % 4 != 0) return false;
    if ((int64_t) groups * 8 > ld) return false;
    // centroid rows are addressed with 32-bit byte offsets, the tiles requested past the end included
    if (((int64_t) k + 4 * CS_TN) * ld * 4 >= (int64_t(1) << 32)) return false;
    // a workgroup owns 256 points: with fewer workgroups than about three quarters of the compute units the 128-point
    // kernel fills the chip better (measured at k = 1,000: 20 % faster than that kernel at 100,000 points, 8 % at 50,000)
    return whatever_n || n >= 192 * CS_POINTS;
}

int launch_gemm_candidates_stationary(skm_ctx* ctx, const float* C, int k, const float* X, int n, int partial_d, int64_t ld,
                                      const float* xnorm_p, const float* cnorm_p, const float* thr0,
                                      uint32_t* cand_count, uint2* cand, uint32_t cap) {
    if (k <= 0 || n <= 0 || partial_d <= 0) return SKM_OK;
    if (!gemm_candidates_stationary_serves(C, k, X, n, partial_d, ld, true))
        return set_error(SKM_ERR_INVALID, "register-stationary candidate kernel: unsupported shape");
    // list offsets inside a wavefront's 64 lists are 32-bit
    if ((uint64_t) cap * 64 * sizeof(uint2) >= (uint64_t(1) << 32))
        return set_error(SKM_ERR_INVALID, "register-stationary candidate kernel: candidate lists too long");
    dim3 grid((unsigned) ((n + CS_POINTS - 1) / CS_POINTS));
#define SKM_CS_CASE(G)                                                                                              \
    case G:                                                                                                         \
        SKM_TRY(launch_stationary<G>(ctx, grid, C, k, X, n, partial_d, ld, xnorm_p, cnorm_p, thr0, cand_count, cand, cap)); \
        break;
    switch ((partial_d + 7) / 8) {
        SKM_CS_CASE(1) SKM_CS_CASE(2) SKM_CS_CASE(3) SKM_CS_CASE(4) SKM_CS_CASE(5) SKM_CS_CASE(6)
        SKM_CS_CASE(7) SKM_CS_CASE(8) SKM_CS_CASE(9) SKM_CS_CASE(10) SKM_CS_CASE(11) SKM_CS_CASE(12)
        SKM_CS_CASE(13) SKM_CS_CASE(14) SKM_CS_CASE(15) SKM_CS_CASE(16) SKM_CS_CASE(17) SKM_CS_CASE(18)
        SKM_CS_CASE(19) SKM_CS_CASE(20)
    }
#undef SKM_CS_CASE
    return check_hip(hipGetLastError(), "gemm_candidates_stationary_kernel launch");
}

} // namespace skm
