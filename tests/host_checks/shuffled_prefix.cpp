// ShuffledPrefix (superkmeans/common.h) against std::shuffle of the whole index array, on both sides of its size
// switch and for k = 1, a few and all.
#include <chrono>
#include <cstdio>
#include <random>
#include <vector>

#include "superkmeans/common.h"

int main() {
    size_t mismatches = 0, cases = 0;
    const size_t sizes[] = {1, 2, 7, 1000, 65535, 65536, 65537, 131071, 131072, 131075, 300001, 1000000};
    for (const size_t n : sizes) {
        for (const size_t k : {size_t(1), size_t(5), n / 3 + 1, n}) {
            if (k > n) continue;
            for (const uint32_t seed : {42u, 7u}) {
                std::mt19937 a(seed), b(seed);
                std::vector<size_t> all(n);
                for (size_t i = 0; i < n; ++i) all[i] = i;
                std::shuffle(all.begin(), all.end(), a);
                all.resize(k);
                const std::vector<size_t> got = skmeans::ShuffledPrefix::Draw(n, k, b);
                ++cases;
                if (got != all || a() != b()) ++mismatches;
            }
        }
    }
    std::printf("walk_used %d\n", skmeans::ShuffledPrefix::WalkMatches() ? 1 : 0);
    std::printf("cases %zu mismatches %zu\n", cases, mismatches);
    // timing of the two forms at ten million indices (informative)
    {
        std::mt19937 a(1), b(1);
        const auto t0 = std::chrono::steady_clock::now();
        const auto x = skmeans::ShuffledPrefix::ByArray(10000000, 256, a);
        const auto t1 = std::chrono::steady_clock::now();
        const auto y = skmeans::ShuffledPrefix::ByWalk(10000000, 256, b);
        const auto t2 = std::chrono::steady_clock::now();
        std::printf("ten_million array_ms %.1f walk_ms %.1f equal %d\n", std::chrono::duration<double, std::milli>(t1 - t0).count(),
                    std::chrono::duration<double, std::milli>(t2 - t1).count(), x == y ? 1 : 0);
    }
    return mismatches == 0 ? 0 : 1;
}
