#pragma once
// Umbrella header (reference include/turboquant/turboquant.h) for the quantized-linear path.

#include "array.h"
#include "codebook.h"
#include "quantizer.h"
#include "dequantizer.h"
#include "linear.h"
#include "serialization.h"

namespace turboquant {

/// Library version string, "0.1.0" as the reference reports (src/turboquant_c.cpp:11-15).
const char* version();

}  // namespace turboquant
