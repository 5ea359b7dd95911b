// CPU check of skmeans::UnitUniformDraws (include/superkmeans/common.h): the integer bound used by the cluster
// splitting walk must make the same decision as the float test `draw < p` for every raw engine output, and a
// stream of draws must equal std::uniform_real_distribution<float>(0, 1) over the same engine.  Mt19937Blocks
// must give the outputs of std::mt19937 and its walk must stop where a draw-by-draw walk over std::mt19937 stops,
// consuming the same number of outputs.
#include "superkmeans/common.h"

#include <cmath>
#include <cstdio>
#include <random>
#include <vector>

int main() {
    using U = skmeans::UnitUniformDraws;
    long bad = 0;
    const float edge[] = {0.0f, -1.0f, 1e-9f, 1.0001e-4f, 9.9e-5f, 0.5f, 0.123456f, 0.99999994f, 1.0f, 2.0f,
                          5.9604645e-8f, 2.3283064e-10f};
    for (float p : edge) {
        const uint64_t b = U::AcceptBelow(p);
        for (long d = -300; d <= 300; ++d) {
            const long long r = (long long) b + d;
            if (r < 0 || r > 0xffffffffLL) continue;
            if ((U::FromRaw((uint32_t) r) < p) != ((uint64_t) r < b)) ++bad;
        }
    }
    std::mt19937 g(7);
    for (int i = 0; i < 300000; ++i) {
        const float p = std::ldexp((float) (g() >> 8), -24 - (int) (g() % 20));
        const uint64_t b = U::AcceptBelow(p);
        const uint32_t probes[4] = {(uint32_t) g(), (uint32_t) g(), (uint32_t) b, (uint32_t) (b - 1)};
        for (uint32_t r : probes)
            if ((U::FromRaw(r) < p) != ((uint64_t) r < b)) ++bad;
    }
    std::mt19937 a(123), c(123);
    U draws(a);
    for (int i = 0; i < 200000; ++i)
        if (draws() != std::uniform_real_distribution<float>(0, 1)(c)) ++bad;
    for (uint32_t seed : {0u, 1u, 42u, 5489u, 0xffffffffu}) {
        std::mt19937 ref(seed);
        skmeans::Mt19937Blocks blocks(seed);
        for (int i = 0; i < 5000;) {
            const uint32_t* r = blocks.Peek();
            const size_t take = 1 + (size_t) i % 7 < blocks.Remaining() ? 1 + (size_t) i % 7 : blocks.Remaining();
            for (size_t j = 0; j < take; ++j, ++i)
                if (r[j] != (uint32_t) ref()) ++bad;
            blocks.Consume(take);
        }
    }
    std::mt19937 shape(99);
    for (size_t k : {1u, 2u, 15u, 16u, 17u, 100u, 623u, 624u, 625u, 1000u, 5000u}) {
        for (int density = 0; density < 3; ++density) {
            std::vector<uint32_t> bound(k);
            // from "nearly every draw accepted" to "one in a few thousand", with clusters that never accept
            for (size_t c = 0; c < k; ++c)
                bound[c] = (shape() % 3 == 0) ? 0u : (uint32_t) (shape() >> (density * 6));
            bound[shape() % k] = 0x00200000u >> density;
            std::mt19937 ref(1234 + (uint32_t) k);
            skmeans::Mt19937Blocks blocks(1234 + (uint32_t) k);
            for (int walk = 0; walk < 300; ++walk) {
                size_t c;
                for (c = 0; true; c = (c + 1 == k) ? 0 : c + 1)
                    if ((uint32_t) ref() < bound[c]) break;
                if (blocks.WalkToFirstAccepted(bound.data(), k) != c) ++bad;
            }
            // both streams stand at the same output afterwards
            if (*blocks.Peek() != (uint32_t) ref()) ++bad;
        }
    }
    std::printf("mismatches %ld direct %d\n", bad, (int) draws.direct());
    return bad != 0;
}
