// Constants and enums of the Super K-Means public interface, HIP backend.
// Values follow the reference's include/superkmeans/common.h:89-129; they are part of the
// algorithm (batch shapes decide tie-breaking and threshold schedules), not tuning knobs.
#pragma once

#include <algorithm>
#include <cmath>
#include <condition_variable>
#include <cstddef>
#include <cstdint>
#include <exception>
#include <mutex>
#include <random>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "skm_hip.h"

#define SKMEANS_ENSURE_POSITIVE(x)                                                                 \
    if ((x) <= 0) {                                                                                \
        throw std::invalid_argument("Value must be positive: " #x);                                \
    }

namespace skmeans {

static inline constexpr float PROPORTION_HORIZONTAL_DIM = 0.75;
static inline constexpr size_t D_THRESHOLD_FOR_DCT_ROTATION = 512;
static inline constexpr size_t H_DIM_SIZE = SKM_H_DIM_SIZE;
static inline constexpr uint32_t MIN_PARTIAL_D = 16;
static inline constexpr size_t DIMENSION_THRESHOLD_FOR_PRUNING = 128;
static inline constexpr size_t N_CLUSTERS_THRESHOLD_FOR_PRUNING = 256;
static inline constexpr size_t X_BATCH_SIZE = SKM_X_BATCH_SIZE;
static inline constexpr size_t Y_BATCH_SIZE = SKM_Y_BATCH_SIZE;
static inline constexpr size_t VECTOR_CHUNK_SIZE = Y_BATCH_SIZE;
static inline constexpr size_t RECALL_CONVERGENCE_PATIENCE = 2;
static inline constexpr float CENTROID_PERTURBATION_EPS = 1.0f / 1024.0f;
static inline constexpr float PRUNER_INITIAL_THRESHOLD = 1.5f;
static inline constexpr float HIERARCHICAL_PRUNER_INITIAL_THRESHOLD = 1.1f;

// Kept for source compatibility: host-side loops of this backend are single threaded, the
// per-point work runs on the device.
inline uint32_t g_n_threads = 1;

// The value sequence of std::uniform_real_distribution<float>(0, 1)(rng) over a std::mt19937, drawn by the
// cluster-splitting walk millions of times per call.  With libstdc++ that is one 32-bit draw scaled by 2^-32
// and kept below 1; the direct form is several times faster than going through generate_canonical.  Whether
// the two agree is checked once per process on a fixed stream; if they do not (another standard library), every
// draw goes through the standard distribution, which is what the reference calls.
class UnitUniformDraws {
  public:
    explicit UnitUniformDraws(std::mt19937& rng) : rng_(rng), direct_(DirectFormMatches()) {}
    float operator()() {
        if (!direct_) return std::uniform_real_distribution<float>(0, 1)(rng_);
        return FromRaw(rng_());
    }
    // True when a draw is FromRaw(one 32-bit output of the engine); then `draw() < p` can be decided on the raw
    // integer: FromRaw is monotone, so the accepted outputs are exactly those below AcceptBelow(p).
    bool direct() const { return direct_; }
    uint32_t raw() { return static_cast<uint32_t>(rng_()); }
    static float FromRaw(const uint32_t r) {
        const float u = static_cast<float>(r) * 0x1p-32f;
        return u < 1.0f ? u : std::nextafter(1.0f, 0.0f);
    }
    // Number of 32-bit outputs r with FromRaw(r) < p (0 ... 2^32), found by bisection on the monotone predicate.
    static uint64_t AcceptBelow(const float p) {
        uint64_t lo = 0, hi = uint64_t(1) << 32;  // FromRaw(r) < p for r < lo, not for r >= hi
        if (!(FromRaw(0) < p)) return 0;
        if (FromRaw(0xffffffffu) < p) return hi;
        lo = 1;
        hi = 0xffffffffu;
        while (lo < hi) {
            const uint64_t mid = lo + (hi - lo) / 2;
            if (FromRaw(static_cast<uint32_t>(mid)) < p) lo = mid + 1; else hi = mid;
        }
        return lo;
    }

  private:
    static bool DirectFormMatches() {
        static const bool ok = [] {
            std::mt19937 a(20240229u), b(20240229u);
            for (int i = 0; i < 1 << 16; ++i) {
                const float ref = std::uniform_real_distribution<float>(0, 1)(a);
                float r = static_cast<float>(b()) * 0x1p-32f;
                if (!(r < 1.0f)) r = std::nextafter(1.0f, 0.0f);
                if (r != ref) return false;
            }
            // the largest draws round up to 2^32 as floats: the clamp must give what the library gives
            struct Top {
                using result_type = std::mt19937::result_type;
                static constexpr result_type min() { return std::mt19937::min(); }
                static constexpr result_type max() { return std::mt19937::max(); }
                result_type operator()() { return max(); }
            } top;
            return std::uniform_real_distribution<float>(0, 1)(top) == std::nextafter(1.0f, 0.0f);
        }();
        return ok;
    }
    std::mt19937& rng_;
    const bool direct_;
};

// The output stream of std::mt19937 (the 32-bit Mersenne Twister of Matsumoto and Nishimura with the standard's
// seeding recurrence), produced 624 outputs at a time into an array.  The cluster-splitting walk tests millions
// of consecutive draws against a table; on an array that test is a vector compare instead of one engine call
// per draw.  Outputs, in order, are exactly those of std::mt19937(seed).
class Mt19937Blocks {
  public:
    static constexpr size_t BLOCK = 624;
    explicit Mt19937Blocks(const uint32_t seed) {
        state_[0] = seed;
        for (uint32_t i = 1; i < BLOCK; ++i) state_[i] = 1812433253u * (state_[i - 1] ^ (state_[i - 1] >> 30)) + i;
    }
    // Unconsumed outputs of the current block (refilled when none is left) and their count.
    const uint32_t* Peek() {
        if (pos_ == BLOCK) Refill();
        return out_ + pos_;
    }
    size_t Remaining() const { return BLOCK - pos_; }
    void Consume(const size_t count) { pos_ += count; }

    /**
     * The walk of SplitClusters for one empty cluster: starting at cluster 0 and cycling over [0, k), one draw
     * per visited cluster, returns the first cluster whose draw is below its bound.  bound[c] is the number of
     * 32-bit outputs accepted for cluster c and must be below 2^32 for every c and positive for at least one.
     */
    size_t WalkToFirstAccepted(const uint32_t* bound, const size_t k) {
        size_t c = 0;
        for (;;) {
            const uint32_t* r = Peek();
            const size_t len = std::min(Remaining(), k - c);
            const uint32_t* b = bound + c;
            size_t i = 0;
            for (; i + 16 <= len; i += 16) {
                uint32_t any = 0;
                for (size_t j = 0; j < 16; ++j) any |= static_cast<uint32_t>(r[i + j] < b[i + j]);
                if (any) break;
            }
            for (; i < len; ++i) {
                if (r[i] < b[i]) {
                    Consume(i + 1);
                    return c + i;
                }
            }
            Consume(len);
            c += len;
            if (c == k) c = 0;
        }
    }

  private:
    static uint32_t Twist(const uint32_t upper, const uint32_t lower, const uint32_t far) {
        const uint32_t y = (upper & 0x80000000u) | (lower & 0x7fffffffu);
        return far ^ (y >> 1) ^ ((lower & 1u) ? 0x9908b0dfu : 0u);
    }
    void Refill() {
        constexpr size_t M = 397;
        for (size_t i = 0; i < BLOCK - M; ++i) state_[i] = Twist(state_[i], state_[i + 1], state_[i + M]);
        for (size_t i = BLOCK - M; i < BLOCK - 1; ++i) state_[i] = Twist(state_[i], state_[i + 1], state_[i + M - BLOCK]);
        state_[BLOCK - 1] = Twist(state_[BLOCK - 1], state_[0], state_[M - 1]);
        for (size_t i = 0; i < BLOCK; ++i) {
            uint32_t y = state_[i];
            y ^= y >> 11;
            y ^= (y << 7) & 0x9d2c5680u;
            y ^= (y << 15) & 0xefc60000u;
            y ^= y >> 18;
            out_[i] = y;
        }
        pos_ = 0;
    }
    uint32_t state_[BLOCK];
    uint32_t out_[BLOCK];
    size_t pos_ = BLOCK;
};

enum class DistanceFunction : uint8_t { l2, dp };
enum class Quantization : uint8_t { f32, u8, f16, bf16 };

template <Quantization q>
struct DistanceType {
    using type = uint32_t;
};
template <>
struct DistanceType<Quantization::f32> {
    using type = float;
};
template <Quantization q>
using skmeans_distance_t = typename DistanceType<q>::type;

template <Quantization q>
struct DataType {
    using type = uint8_t;
};
template <>
struct DataType<Quantization::f32> {
    using type = float;
};
template <Quantization q>
using skmeans_value_t = typename DataType<q>::type;

template <Quantization q>
struct CentroidDataType {
    using type = float;
};
template <Quantization q>
using skmeans_centroid_value_t = typename CentroidDataType<q>::type;

namespace hip {

// Turns a C-ABI status into the exception type the reference's callers expect.
inline void Check(int rc) {
    if (rc == SKM_OK) return;
    const char* msg = skm_last_error();
    std::string text = std::string("libskm_hip: ") + (msg ? msg : "unknown error");
    if (rc == SKM_ERR_INVALID) throw std::invalid_argument(text);
    throw std::runtime_error(text);
}

// Owns one skm_ctx (device + stream + workspace).
class Context {
  public:
    explicit Context(int device = 0) { Check(skm_ctx_create(device, &ctx_)); }
    ~Context() {
        if (ctx_) skm_ctx_destroy(ctx_);
    }
    Context(const Context&) = delete;
    Context& operator=(const Context&) = delete;
    skm_ctx* get() const { return ctx_; }

  private:
    skm_ctx* ctx_ = nullptr;
};

// A typed device allocation; replaces the std::unique_ptr<T[]> members of the reference.
template <class T>
class Buffer {
  public:
    Buffer() = default;
    Buffer(skm_ctx* ctx, size_t count) { Reset(ctx, count); }
    ~Buffer() { Release(); }
    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
    Buffer(Buffer&& o) noexcept { MoveFrom(o); }
    Buffer& operator=(Buffer&& o) noexcept {
        if (this != &o) {
            Release();
            MoveFrom(o);
        }
        return *this;
    }
    void Reset(skm_ctx* ctx, size_t count) {
        Release();
        ctx_ = ctx;
        count_ = count;
        void* p = nullptr;
        Check(skm_malloc(ctx, count * sizeof(T), &p));
        ptr_ = static_cast<T*>(p);
    }
    void Release() {
        if (ptr_) skm_free(ctx_, ptr_);
        ptr_ = nullptr;
        count_ = 0;
    }
    T* get() const { return ptr_; }
    size_t size() const { return count_; }
    void Upload(const T* host, size_t count, size_t dst_offset = 0) {
        Check(skm_upload(ctx_, ptr_ + dst_offset, host, count * sizeof(T)));
    }
    // Copy on the transfer stream: queued work keeps running, later work waits (skm_upload_overlapped).
    void UploadOverlapped(const T* host, size_t count, size_t dst_offset = 0) {
        Check(skm_upload_overlapped(ctx_, ptr_ + dst_offset, host, count * sizeof(T)));
    }
    void Download(T* host, size_t count, size_t src_offset = 0) const {
        Check(skm_download(ctx_, host, ptr_ + src_offset, count * sizeof(T)));
    }
    void swap(Buffer& o) noexcept {
        std::swap(ctx_, o.ctx_);
        std::swap(ptr_, o.ptr_);
        std::swap(count_, o.count_);
    }

  private:
    void MoveFrom(Buffer& o) {
        ctx_ = o.ctx_;
        ptr_ = o.ptr_;
        count_ = o.count_;
        o.ptr_ = nullptr;
        o.count_ = 0;
    }
    skm_ctx* ctx_ = nullptr;
    T* ptr_ = nullptr;
    size_t count_ = 0;
};

// Sends host rows to the device in slabs from a thread of its own (skm_upload_detached), so that the caller's thread
// can queue the work on every slab as soon as it has arrived, whatever that work waits for in between.  Slab s holds
// the rows [edges[s], edges[s + 1]).  WaitFor(s) returns when slab s is in device memory and rethrows what the
// transfer thread failed with.
class RowFeeder {
  public:
    RowFeeder(skm_ctx* ctx, float* d_dst, const float* h_src, size_t row_floats, std::vector<size_t> edges)
        : edges_(std::move(edges)) {
        Check(skm_upload_detached(ctx, d_dst, h_src, 0));  // the context's transfer stream exists before the thread does
        worker_ = std::thread([this, ctx, d_dst, h_src, row_floats] {
            try {
                for (size_t s = 0; s + 1 < edges_.size(); ++s) {
                    {
                        std::lock_guard<std::mutex> lock(mutex_);
                        if (stop_) return;
                    }
                    const size_t r0 = edges_[s], m = edges_[s + 1] - r0;
                    Check(skm_upload_detached(ctx, d_dst + r0 * row_floats, h_src + r0 * row_floats,
                                              m * row_floats * sizeof(float)));
                    {
                        std::lock_guard<std::mutex> lock(mutex_);
                        landed_ = s + 1;
                    }
                    arrived_.notify_all();
                }
            } catch (...) {
                {
                    std::lock_guard<std::mutex> lock(mutex_);
                    error_ = std::current_exception();
                }
                arrived_.notify_all();
            }
        });
    }
    ~RowFeeder() {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            stop_ = true;
        }
        if (worker_.joinable()) worker_.join();
    }
    RowFeeder(const RowFeeder&) = delete;
    RowFeeder& operator=(const RowFeeder&) = delete;
    size_t NumSlabs() const { return edges_.size() - 1; }
    size_t FirstRow(size_t slab) const { return edges_[slab]; }
    size_t Rows(size_t slab) const { return edges_[slab + 1] - edges_[slab]; }
    void WaitFor(size_t slab) {
        std::unique_lock<std::mutex> lock(mutex_);
        arrived_.wait(lock, [&] { return landed_ > slab || error_; });
        if (landed_ <= slab) std::rethrow_exception(error_);
    }

  private:
    const std::vector<size_t> edges_;  // ascending row offsets, the first 0, the last the number of rows
    std::thread worker_;
    std::mutex mutex_;
    std::condition_variable arrived_;
    size_t landed_ = 0;
    bool stop_ = false;
    std::exception_ptr error_;
};

} // namespace hip
// The first k entries of {0, 1, ..., n - 1} after std::shuffle(first, last, rng), which is how the reference draws
// its initial centroids (superkmeans.h:1100-1120: shuffle all n indices, keep k).  libstdc++'s shuffle for a
// generator range below n * n is the forward walk "for i = 1 .. n-1: swap(a[i], a[uniform(0, i)])", each position
// through one call of uniform_int_distribution<size_t> with the bounds as parameters.  Position i still holds i
// when the walk reaches it and is never visited again afterwards, so what the first k positions end up with follows
// from the draws alone: no n-entry array, no cache miss per swap (ten million indices take a third of the time).
// Whether the library's shuffle is this walk is checked once per process on a fixed case; if it is not (another
// standard library, or the two-positions-per-draw form libstdc++ uses for small n), the array is shuffled as before.
class ShuffledPrefix {
  public:
    static std::vector<size_t> Draw(const size_t n, const size_t k, std::mt19937& rng) {
        if (n >= MIN_N_FOR_WALK && k <= n && WalkMatches()) return ByWalk(n, k, rng);
        return ByArray(n, k, rng);
    }
    static std::vector<size_t> ByArray(const size_t n, const size_t k, std::mt19937& rng) {
        std::vector<size_t> all(n);
        for (size_t i = 0; i < n; ++i) all[i] = i;
        std::shuffle(all.begin(), all.end(), rng);
        all.resize(std::min(k, n));
        return all;
    }
    static std::vector<size_t> ByWalk(const size_t n, const size_t k, std::mt19937& rng) {
        using distribution_t = std::uniform_int_distribution<size_t>;
        using bounds_t = distribution_t::param_type;
        distribution_t uniform;
        const size_t head_n = std::min(k, n);
        std::vector<size_t> head(head_n);
        for (size_t i = 0; i < head_n; ++i) head[i] = i;
        for (size_t i = 1; i < head_n; ++i) std::swap(head[i], head[uniform(rng, bounds_t(0, i))]);
        for (size_t i = std::max<size_t>(head_n, 1); i < n; ++i) {
            const size_t j = uniform(rng, bounds_t(0, i));
            if (j < head_n) head[j] = i;  // position i held i; what it receives is never read again
        }
        return head;
    }
    // Below this many indices the array is cheap, and libstdc++ takes two positions from one draw while n * n fits
    // the generator's range (n < 65,536).
    static constexpr size_t MIN_N_FOR_WALK = size_t(1) << 17;
    static bool WalkMatches() {
        static const bool ok = [] {
            const size_t n = MIN_N_FOR_WALK + 3;
            std::mt19937 a(20240301u), b(20240301u);
            if (ByArray(n, n, a) != ByWalk(n, n, b)) return false;
            return a() == b();  // the same number of draws
        }();
        return ok;
    }
};

} // namespace skmeans
