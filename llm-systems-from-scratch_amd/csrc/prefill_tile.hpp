// LDS tile layout shared by the prefill forward and backward kernels: row-major tiles of D bf16
// per row, unpadded (direct-to-LDS loads write 1 KiB of consecutive LDS per wavefront), with an
// XOR swizzle of the 16-byte chunk index instead of padding.
#pragma once
#include "common.hpp"

namespace mi355 {

// XOR pattern applied to the 16-byte chunk index of LDS row `row` (rows hold D bf16).
// Chosen so that (a) 16 lanes reading one logical chunk of 16 consecutive rows and
// (b) a transposed read touching 4 consecutive rows x 32 bytes both spread over
// distinct banks (LDS banks repeat every 256 bytes).
template <int D>
__device__ __forceinline__ int swz(int row) {
    if constexpr (D == 128) return ((row & 3) << 2) | ((row >> 2) & 3);
    else if constexpr (D == 64) return (((row >> 1) & 3) << 1) | ((row >> 3) & 1);
    else return (row >> 2) & 3;
}

}  // namespace mi355
