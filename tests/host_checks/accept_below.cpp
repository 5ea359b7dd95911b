// CPU check of skmeans::UnitUniformDraws (include/superkmeans/common.h): the integer bound used by the cluster
// splitting walk must make the same decision as the float test `draw < p` for every raw engine output, and a
// stream of draws must equal std::uniform_real_distribution<float>(0, 1) over the same engine.
#include "superkmeans/common.h"

#include <cmath>
#include <cstdio>
#include <random>

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
    std::printf("mismatches %ld direct %d\n", bad, (int) draws.direct());
    return bad != 0;
}
