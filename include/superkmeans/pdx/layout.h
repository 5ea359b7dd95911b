// PDX dimension split used by the centroid relayout (device kernel: skm_pdxify).
#pragma once

#include <cmath>

#include "superkmeans/common.h"

namespace skmeans {

struct PDXDimensionSplit {
    size_t horizontal_d{0};
    size_t vertical_d{0};
};

template <Quantization q = Quantization::f32, DistanceFunction alpha = DistanceFunction::l2>
class PDXLayout {
  public:
    // Same rule as the reference's PDXLayout::GetDimensionSplit (pdx/layout.h:115-140):
    // 75 % of the dimensions (25 % when d <= 256) go to 64-wide horizontal blocks, rounded to the
    // nearest multiple of 64; never zero vertical dimensions; everything vertical when d <= 64.
    static PDXDimensionSplit GetDimensionSplit(const size_t d) {
        if (d <= H_DIM_SIZE) return {0, d};
        const double proportion = (d <= 256) ? 0.25 : static_cast<double>(PROPORTION_HORIZONTAL_DIM);
        size_t horizontal = static_cast<size_t>(static_cast<double>(d) * proportion);
        if (horizontal % H_DIM_SIZE != 0) {
            horizontal = static_cast<size_t>(std::lround(static_cast<double>(horizontal) /
                                                         static_cast<double>(H_DIM_SIZE))) *
                         H_DIM_SIZE;
        }
        if (horizontal == d) horizontal = H_DIM_SIZE;
        return {horizontal, d - horizontal};
    }
};

} // namespace skmeans
