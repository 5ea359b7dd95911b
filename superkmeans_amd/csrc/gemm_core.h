// fp32 MFMA GEMM core for gfx950 (CDNA4): D[m][n] = sum_k A[m][k] * B[n][k].
//
// Both operands are row-major with the reduction dimension contiguous, which is
// exactly the shape of every dense product on the Super K-Means hot path:
//   * distances  x . c     (reference: batch_computers.h:47-83, sgemm_('T','N'))
//   * rotation   X . Q^T   (reference: pdx/adsampling.h:191-215)
// A workgroup owns one tile of D and each of its wavefronts a block of FM x FN accumulators of the
// v_mfma_f32_32x32x2_f32 instruction.  Two shapes are built:
//   * 128 x 128, 4 wavefronts of 64 x 64, two workgroups per CU   (small problems, fused candidate kernel)
//   * 256 x 256, 8 wavefronts of 128 x 64, one workgroup per CU   (large problems: per MFMA half the global
//     loads, LDS stores and barriers and three quarters of the fragment reads of the small shape)
// Operand slices of BK = 32 columns are staged through LDS (double buffered, row stride 36 floats so
// that both the 16-byte stores and the 16-byte fragment reads are bank-conflict free).
//
// The k index inside a group of 8 columns is permuted so that one ds_read_b128
// per operand fragment feeds four consecutive MFMAs: lane l supplies columns
// (l / 32) * 4 + i to the i-th MFMA for both A and B, which is a valid GEMM
// because A and B use the same permutation.  The order in which the products of one output element are
// accumulated does not depend on the tile shape, so both shapes give bit-identical results.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace skm {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int GEMM_BK = 32;
constexpr int GEMM_LDS_STRIDE = GEMM_BK + 4;
constexpr int GEMM_XCDS = 8;

// WM x WN wavefronts, each FM x FN accumulator blocks of 32 x 32.
template <int WM_, int WN_, int FM_, int FN_, int WG_PER_CU_>
struct GemmShape {
    static constexpr int WM = WM_, WN = WN_, FM = FM_, FN = FN_, WG_PER_CU = WG_PER_CU_;
    static constexpr int THREADS = WM * WN * 64;
    static constexpr int TM = WM * FM * 32;
    static constexpr int TN = WN * FN * 32;
    static constexpr int WAVE_M = FM * 32;            // rows of D per wavefront
    static constexpr int WAVE_N = FN * 32;
    static constexpr int ROWS_PER_LOAD = THREADS / 8;  // operand rows covered by one 16-byte load per thread
    static constexpr int NLA = TM / ROWS_PER_LOAD;     // loads per thread and slice, A operand
    static constexpr int NLB = TN / ROWS_PER_LOAD;
    static constexpr int LDS_FLOATS = 2 * (TM + TN) * GEMM_LDS_STRIDE;
    static constexpr int BAND = WG_PER_CU == 1 ? 4 : 8;  // M-tiles per band of the workgroup-to-tile map
    static_assert(TM % ROWS_PER_LOAD == 0 && TN % ROWS_PER_LOAD == 0, "tile rows must split evenly over the loads");
};
using GemmSmall = GemmShape<2, 2, 2, 2, 2>;
using GemmBig = GemmShape<2, 4, 4, 2, 1>;
// 128 x 64: for problems of a few hundred 128 x 128 tiles, where whole tiles leave part of the chip idle in the last round.
using GemmHalf = GemmShape<2, 2, 2, 1, 2>;
// (32 FM) x 128: a few M rows against all N rows, bound by the loads of the N operand.  Used for the centroids left
// over when k is up to 128 rows more than a multiple of the large shape's 256.
template <int FM>
using GemmThin = GemmShape<1, 4, FM, 1, 2>;
constexpr int GEMM_THIN_MAX_ROWS = 128;

constexpr int GEMM_TM = GemmSmall::TM;
constexpr int GEMM_TN = GemmSmall::TN;
constexpr int GEMM_THREADS = GemmSmall::THREADS;

struct GemmOperands {
    const float* A;  // M x K, row stride lda
    const float* B;  // N x K, row stride ldb
    int M, N, K;
    int64_t lda, ldb;
    int tiles_m, tiles_n;
    int m_base;  // added to the row indices the argmin kernel reports (a launch over rows m_base.. of a larger matrix)
};

// Accumulators of one wavefront: acc.v[mb][nb] is a 32 x 32 block.  Element r of
// acc[mb][nb] held by lane l is D[m][n] with
//   m = wave_m0 + mb * 32 + 8 * (r / 4) + 4 * (l / 32) + (r % 4)
//   n = wave_n0 + nb * 32 + (l % 32)
template <int FM, int FN>
struct WaveAccT {
    floatx16 v[FM][FN];
};
using WaveAcc = WaveAccT<2, 2>;

__device__ __forceinline__ int acc_row(int mb, int r, int lane) {
    return mb * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}
__device__ __forceinline__ int acc_col(int nb, int lane) {
    return nb * 32 + (lane & 31);
}

// Maps the hardware workgroup id to a tile so that the workgroups resident on
// one XCD (ids congruent mod 8 are dispatched to the same XCD) cover a compact
// block of BAND M-tiles x several N-tiles and share operand panels in that XCD's L2
// (64 resident workgroups of the small shape: 8 x 8; 32 of the large one: 4 x 8).
template <int BAND>
__device__ __forceinline__ void tile_of_block(const GemmOperands& g, int bid, int& tm, int& tn) {
    const int total = g.tiles_m * g.tiles_n;
    const int q = total / GEMM_XCDS, r = total % GEMM_XCDS;
    const int x = bid % GEMM_XCDS, within = bid / GEMM_XCDS;
    const int L = x * q + (x < r ? x : r) + within;
    const int band_tiles = BAND * g.tiles_n;
    const int band = L / band_tiles;
    const int in_band = L - band * band_tiles;
    const int rows_in_band = (g.tiles_m - band * BAND) < BAND ? (g.tiles_m - band * BAND) : BAND;
    tn = in_band / rows_in_band;
    tm = band * BAND + in_band % rows_in_band;
}

// Four consecutive operand columns starting at k.  GUARD: columns at or past K read as zero (last,
// partial BK step, and every step of the scalar path).
template <bool VEC, bool GUARD>
__device__ __forceinline__ floatx4 load_k4(const float* row, int k, int K) {
    floatx4 v;
    if (VEC && !GUARD) {
        v = *reinterpret_cast<const floatx4*>(row + k);
    } else if (VEC) {
        if (k + 3 < K) {
            v = *reinterpret_cast<const floatx4*>(row + k);
        } else {
            v.x = (k + 0 < K) ? row[k + 0] : 0.0f;
            v.y = (k + 1 < K) ? row[k + 1] : 0.0f;
            v.z = (k + 2 < K) ? row[k + 2] : 0.0f;
            v.w = 0.0f;
        }
    } else {
        v.x = (k + 0 < K) ? row[k + 0] : 0.0f;
        v.y = (k + 1 < K) ? row[k + 1] : 0.0f;
        v.z = (k + 2 < K) ? row[k + 2] : 0.0f;
        v.w = (k + 3 < K) ? row[k + 3] : 0.0f;
    }
    return v;
}

// 16 bytes through a buffer descriptor: address = descriptor base + voffset (per lane, bytes) + soffset
// (wavefront-uniform, bytes).  One 32-bit register per lane addresses a row whatever the step, where a
// pointer per load would take two.
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t operand_rows(const float* base) {
    // raw buffer, no stride, no bounds clamp needed (rows are clamped by the caller); dword 3 = 32-bit data format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ floatx4 load_rows_x4(__amdgpu_buffer_rsrc_t rows, uint32_t voffset, uint32_t soffset) {
    return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rows, (int) voffset, (int) soffset, 0));
}

// The 16 MFMAs of one group of 8 columns (fragments a0, a1, b0, b1 hold 4 columns each per lane).
__device__ __forceinline__ void mfma_group(const floatx4& a0, const floatx4& a1, const floatx4& b0, const floatx4& b1,
                                           WaveAcc& acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc.v[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[i], b0[i], acc.v[0][0], 0, 0, 0);
        acc.v[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[i], b1[i], acc.v[0][1], 0, 0, 0);
        acc.v[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[i], b0[i], acc.v[1][0], 0, 0, 0);
        acc.v[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[i], b1[i], acc.v[1][1], 0, 0, 0);
    }
}

// Computes the tile (tm, tn) of shape S.  VEC: row starts and strides are 16-byte aligned so operand
// slices can be fetched with dwordx4 loads; then every full BK step is fetched without any guard (the
// loads of a thread are issued back to back) and only a trailing partial step is guarded.
//
// Schedule of one full step kt (LDS buffer kt & 1 holds slice kt, registers hold slice kt + 1):
//   1. slice kt + 1 goes from registers to the other LDS buffer (its last readers passed the barrier of
//      step kt - 1), then the loads of slice kt + 2 are issued into the same registers;
//   2. groups 0..2 of the slice: FM * FN * 4 MFMAs each, the fragments of the next group requested before them;
//   3. the workgroup barrier sits before the last group, when every LDS read of the step has returned
//      and the stores of 1. have long completed; right after it the first fragments of slice kt + 1
//      are requested, so that they arrive under the MFMAs of group 3.
// No phase of the step is without MFMAs in flight: a wavefront never waits for memory and then for
// the barrier and then for LDS with the matrix pipe idle.
template <bool VEC, class S>
__device__ __forceinline__ void gemm_tile(
    const GemmOperands& g, int tm, int tn, float* lds, WaveAccT<S::FM, S::FN>& acc
) {
    constexpr int FM = S::FM, FN = S::FN;
    float* As = lds;                                  // [2][TM * STRIDE]
    float* Bs = lds + 2 * S::TM * GEMM_LDS_STRIDE;    // [2][TN * STRIDE]
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / S::WN, wn = wave % S::WN;

    // Global -> register staging: thread covers rows (tid / 8) + ROWS_PER_LOAD * p, 4 floats at column 4 * (tid % 8).
    // Rows past the end are clamped to the last row: duplicates are masked by the epilogue.  Unguarded slices
    // are fetched through one buffer descriptor per operand (tile base, wavefront-uniform) plus a 32-bit byte
    // offset per row; the slice's column offset is a scalar.
    const int ld_row = tid >> 3;
    const int ld_k = (tid & 7) * 4;
    const float* a_base = g.A + (int64_t) (tm * S::TM) * g.lda;
    const float* b_base = g.B + (int64_t) (tn * S::TN) * g.ldb;
    const __amdgpu_buffer_rsrc_t a_desc = operand_rows(a_base);
    const __amdgpu_buffer_rsrc_t b_desc = operand_rows(b_base);
    uint32_t a_off[S::NLA], b_off[S::NLB];  // bytes from the tile base to this thread's 4 columns of slice 0
    const int a_last = g.M - 1 - tm * S::TM, b_last = g.N - 1 - tn * S::TN;
#pragma unroll
    for (int p = 0; p < S::NLA; ++p) {
        const int r = ld_row + S::ROWS_PER_LOAD * p;
        a_off[p] = ((uint32_t) (r < a_last ? r : a_last) * (uint32_t) g.lda + (uint32_t) ld_k) * 4u;
    }
#pragma unroll
    for (int p = 0; p < S::NLB; ++p) {
        const int r = ld_row + S::ROWS_PER_LOAD * p;
        b_off[p] = ((uint32_t) (r < b_last ? r : b_last) * (uint32_t) g.ldb + (uint32_t) ld_k) * 4u;
    }
    floatx4 ra[S::NLA], rb[S::NLB];

#pragma unroll
    for (int mb = 0; mb < FM; ++mb)
#pragma unroll
        for (int nb = 0; nb < FN; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc.v[mb][nb][r] = 0.0f;

    const int nk = (g.K + GEMM_BK - 1) / GEMM_BK;
    const int nk_full = VEC ? g.K / GEMM_BK : 0;  // slices that need no guard
    const int n_full_steps = g.K / GEMM_BK;       // slices whose 32 columns all hold data

    auto request = [&](int kt) {  // slice kt -> registers
        const int k0 = kt * GEMM_BK;
        if (kt < nk_full) {
#pragma unroll
            for (int p = 0; p < S::NLA; ++p) ra[p] = load_rows_x4(a_desc, a_off[p], (uint32_t) k0 * 4u);
#pragma unroll
            for (int p = 0; p < S::NLB; ++p) rb[p] = load_rows_x4(b_desc, b_off[p], (uint32_t) k0 * 4u);
        } else {
#pragma unroll
            for (int p = 0; p < S::NLA; ++p) ra[p] = load_k4<VEC, true>(a_base + (a_off[p] / 4u - ld_k), k0 + ld_k, g.K);
#pragma unroll
            for (int p = 0; p < S::NLB; ++p) rb[p] = load_k4<VEC, true>(b_base + (b_off[p] / 4u - ld_k), k0 + ld_k, g.K);
        }
    };
    const int st_off = ld_row * GEMM_LDS_STRIDE + ld_k;
    auto publish = [&](int buf) {  // registers -> LDS buffer
        float* as = As + buf * S::TM * GEMM_LDS_STRIDE + st_off;
        float* bs = Bs + buf * S::TN * GEMM_LDS_STRIDE + st_off;
#pragma unroll
        for (int p = 0; p < S::NLA; ++p) *reinterpret_cast<floatx4*>(&as[S::ROWS_PER_LOAD * p * GEMM_LDS_STRIDE]) = ra[p];
#pragma unroll
        for (int p = 0; p < S::NLB; ++p) *reinterpret_cast<floatx4*>(&bs[S::ROWS_PER_LOAD * p * GEMM_LDS_STRIDE]) = rb[p];
    };

    const int frag_off = (lane & 31) * GEMM_LDS_STRIDE + (lane >> 5) * 4;
    const int a_frag = (wm * S::WAVE_M) * GEMM_LDS_STRIDE + frag_off;
    const int b_frag = (wn * S::WAVE_N) * GEMM_LDS_STRIDE + frag_off;
    floatx4 fa[FM], fb[FN];
    auto fetch = [&](int buf, int kg, floatx4* xa, floatx4* xb) {
        const float* as = As + buf * S::TM * GEMM_LDS_STRIDE + a_frag + kg * 8;
        const float* bs = Bs + buf * S::TN * GEMM_LDS_STRIDE + b_frag + kg * 8;
#pragma unroll
        for (int i = 0; i < FM; ++i) xa[i] = *reinterpret_cast<const floatx4*>(as + i * 32 * GEMM_LDS_STRIDE);
#pragma unroll
        for (int j = 0; j < FN; ++j) xb[j] = *reinterpret_cast<const floatx4*>(bs + j * 32 * GEMM_LDS_STRIDE);
    };
    // The FM * FN * 4 MFMAs of one group of 8 columns; consecutive MFMAs never share an accumulator.
    auto group = [&]() {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc.v[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][q], fb[j][q], acc.v[i][j], 0, 0, 0);
    };
    auto advance = [&](const floatx4* na, const floatx4* nb) {
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[i] = na[i];
#pragma unroll
        for (int j = 0; j < FN; ++j) fb[j] = nb[j];
    };

    // Prologue: slice 0 in LDS buffer 0, slice 1 (if any) on its way into the registers.
    request(0);
    publish(0);
    if (nk > 1) request(1);
    __syncthreads();
    if (n_full_steps > 0) fetch(0, 0, fa, fb);

    // One full step.  HOT: slices kt + 1 and kt + 2 exist and need no guard (no condition in the step).
    auto step = [&](const int kt, auto hot) {
        constexpr bool HOT = decltype(hot)::value;
        const int cur = kt & 1;
        if (HOT) {
            publish(cur ^ 1);
            const int k0 = (kt + 2) * GEMM_BK;
#pragma unroll
            for (int p = 0; p < S::NLA; ++p) ra[p] = load_rows_x4(a_desc, a_off[p], (uint32_t) k0 * 4u);
#pragma unroll
            for (int p = 0; p < S::NLB; ++p) rb[p] = load_rows_x4(b_desc, b_off[p], (uint32_t) k0 * 4u);
        } else {
            if (kt + 1 < nk) publish(cur ^ 1);
            if (kt + 2 < nk) request(kt + 2);
        }
        __builtin_amdgcn_sched_barrier(0);
        floatx4 na[FM], nb[FN];
#pragma unroll
        for (int kg = 0; kg < GEMM_BK / 8 - 1; ++kg) {
            fetch(cur, kg + 1, na, nb);
            group();
            advance(na, nb);
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();  // every read of buffer `cur` has returned, slice kt + 1 is complete in the other one
        if (HOT || kt + 1 < n_full_steps) fetch(cur ^ 1, 0, na, nb);
        __builtin_amdgcn_sched_barrier(0);
        group();
        advance(na, nb);
    };
    auto sweep = [&]() {
        int kt = 0;
        for (; kt + 2 < nk_full; ++kt) step(kt, std::true_type{});
        for (; kt < n_full_steps; ++kt) step(kt, std::false_type{});
        if (n_full_steps < nk) {
            // Trailing partial slice: only the groups of 8 columns that hold data (the rest is zero).
            const int cur = n_full_steps & 1;
            const int kg_live = (g.K - n_full_steps * GEMM_BK + 7) / 8;
            for (int kg = 0; kg < kg_live; ++kg) {
                fetch(cur, kg, fa, fb);
                group();
            }
            __syncthreads();
        }
    };
    sweep();
}

constexpr int GEMM_LDS_FLOATS = GemmSmall::LDS_FLOATS;

inline bool gemm_operands_vectorizable(const GemmOperands& g) {
    return (reinterpret_cast<uintptr_t>(g.A) % 16 == 0) && (reinterpret_cast<uintptr_t>(g.B) % 16 == 0) &&
           (g.lda % 4 == 0) && (g.ldb % 4 == 0);
}

} // namespace skm
