// Exercises superkmeans/pdx/utils.h on the CPU: prints values that tests/test_host_headers.py compares with the
// oracle's restatement of the same reference routines and with closed forms.
#include <cstdio>
#include <vector>

#include "superkmeans/pdx/utils.h"

int main() {
    using namespace skmeans;
    const auto blobs = MakeBlobs(50, 7, 5, false, 0.25f, 5.0f, 42);
    std::printf("blobs");
    for (float v : blobs) std::printf(" %.9g", v);
    std::printf("\n");
    const auto unit = MakeBlobs(20, 6, 3, true);
    const auto norms = ComputeNorms(unit.data(), 20, 6);
    float worst = 0.0f;
    for (float v : norms) worst = std::max(worst, std::fabs(v - 1.0f));
    std::printf("unit_norm_error %.3g\n", worst);
    const auto uniform = GenerateRandomVectors(100, 4, -2.0f, 3.0f, 7);
    float lo = uniform[0], hi = uniform[0];
    for (float v : uniform) lo = std::min(lo, v), hi = std::max(hi, v);
    std::printf("uniform_range %.3f %.3f\n", lo, hi);
    // three points on a line: nearest neighbours are known
    const float y[] = {0.f, 0.f, 1.f, 0.f, 5.f, 0.f};
    const float x[] = {0.9f, 0.f, 4.f, 0.f};
    uint32_t nn[2], knn[4];
    float nd[2], kd[4];
    FindNearestNeighborBruteForce(x, y, 2, 3, 2, nn, nd);
    FindKNearestNeighborsBruteForce(x, y, 2, 3, 2, 2, knn, kd);
    std::printf("nn %u %u %.4f %.4f\n", nn[0], nn[1], nd[0], nd[1]);
    std::printf("knn %u %u %u %u\n", knn[0], knn[1], knn[2], knn[3]);
    std::printf("nearest_centroid %u\n", FindNearestCentroidBruteForce(x + 2, y, 3, 2));
    std::printf("rounding %u %u %d %d\n", CeilXToMultipleOfM(65, 64), FloorXToMultipleOfM(127, 64), (int) IsPowerOf2(64),
                (int) IsPowerOf2(96));
    std::vector<float> dist(1000);
    GenerateRandomDistances(dist.data(), dist.size(), 2.0f, 0.03f, 1);
    int below = 0;
    for (float v : dist) below += v < 2.0f;
    std::printf("below %d\n", below);
    TicToc t;
    t.Tic();
    t.Toc();
    std::printf("timer_ok %d\n", (int) (t.GetMilliseconds() >= 0.0));
    return 0;
}
