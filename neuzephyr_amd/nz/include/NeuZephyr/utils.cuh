// Small macros kept for source compatibility (reference: include/NeuZephyr/utils.cuh:9-19).
// MMA / CEIL described the reference's pad-to-16 scheme; nothing is padded here, they remain
// only so that user code naming them still compiles.
#ifndef NZ_UTILS_CUH
#define NZ_UTILS_CUH
#include <iostream>

#define TILE_SIZE 32
#define MMA 16
#define CEIL(X) (((X) + 15) & ~15)

#define WARN(message) \
    (std::cerr << "Warning: " << message << " (File: " << __FILE__ << ", Line: " << __LINE__ << std::endl)
#endif
