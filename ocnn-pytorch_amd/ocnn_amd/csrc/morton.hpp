// Bit arithmetic of the Morton keys, shared by the key and neighbour kernels.
#pragma once
#include <stdint.h>

#include <hip/hip_runtime.h>

namespace ocnn {

// spreads the low 16 bits of v so that bit i lands on bit 3i
__host__ __device__ __forceinline__ uint64_t spread3(uint64_t v) {
  v &= 0xffffull;
  v = (v | (v << 32)) & 0x001f00000000ffffull;
  v = (v | (v << 16)) & 0x001f0000ff0000ffull;
  v = (v | (v << 8)) & 0x100f00f00f00f00full;
  v = (v | (v << 4)) & 0x10c30c30c30c30c3ull;
  v = (v | (v << 2)) & 0x1249249249249249ull;
  return v;
}

// inverse of spread3: collects every third bit
__host__ __device__ __forceinline__ uint64_t compact3(uint64_t v) {
  v &= 0x1249249249249249ull;
  v = (v | (v >> 2)) & 0x10c30c30c30c30c3ull;
  v = (v | (v >> 4)) & 0x100f00f00f00f00full;
  v = (v | (v >> 8)) & 0x001f0000ff0000ffull;
  v = (v | (v >> 16)) & 0x001f00000000ffffull;
  v = (v | (v >> 32)) & 0xffffull;
  return v;
}

// The reference masks each coordinate to 8 bits (depth bits when depth <= 8)
// and, for depth > 8, adds bits 8..depth-1: together the low `depth` bits.
__host__ __device__ __forceinline__ int64_t encode(int64_t x, int64_t y, int64_t z, int depth) {
  uint64_t m = (1ull << depth) - 1;
  return (int64_t)((spread3((uint64_t)x & m) << 2) | (spread3((uint64_t)y & m) << 1) |
                   spread3((uint64_t)z & m));
}

}  // namespace ocnn
