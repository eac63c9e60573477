#pragma once
// Lloyd-Max codebooks.  Same types and functions as the reference's
// include/turboquant/codebook.h:1-55, with turboquant::Array in place of mlx::core::array.
// Element work (bin search, centroid gather, the Lloyd-Max assignment pass) runs on the GPU.

#include "array.h"
#include <cstdint>
#include <vector>

namespace turboquant {

/// Where a codebook's centroids came from: analytical codebooks are symmetric by
/// construction, empirical ones need not be (reference codebook.h:15-18).
enum class CodebookOrigin : uint8_t {
    Analytical,
    Empirical,
};

struct Codebook {
    std::vector<float> centroids;   ///< sorted, 2^bits entries
    std::vector<float> boundaries;  ///< midpoints between neighbouring centroids
    uint8_t bits = 0;               ///< 1..5
    CodebookOrigin origin = CodebookOrigin::Analytical;
};

/// Precomputed N(0,1) Lloyd-Max codebook.  Throws std::invalid_argument outside 1..5 bits
/// (reference src/codebook.cpp:72-85).
Codebook generate_codebook(uint8_t bits);

/// Data-adaptive Lloyd-Max fit (reference src/codebook.cpp:99-143 and :269-282): analytic
/// initialisation, lower_bound bins, double sums, early exit below a 1e-6 shift.  Empty data
/// returns the analytic codebook.
Codebook generate_codebook_from_data(const std::vector<float>& data, uint8_t bits, int iterations = 100);

/// fp32 values -> uint8 bin indices, flat [n] (reference src/codebook.cpp:284-302).
Array quantize(const Array& values, const Codebook& codebook);

/// uint8 indices -> fp32 centroid values, flat [n] (reference src/codebook.cpp:304-321).
Array dequantize(const Array& indices, const Codebook& codebook);

/// Sorted centroids, midpoint boundaries, exact symmetry for analytical codebooks
/// (reference src/codebook.cpp:323-353).
bool validate_codebook(const Codebook& codebook);

}  // namespace turboquant
