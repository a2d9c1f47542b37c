// Second pass of every two-pass reduction in the library.
#pragma once
#include "common.hpp"

namespace ocnn {

// fixed-order reduction over the splits; writes (K, ca, cb) or (K, cb, ca)
template <typename T>
__global__ void wgrad_reduce_kernel(const float* __restrict__ partial, int splits, int K, int ca,
                                    int cb, int out_transposed, T* __restrict__ out) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t per = (int64_t)K * ca * cb;
  if (e >= per) return;
  float acc = 0.f;
  for (int s = 0; s < splits; ++s) acc += partial[(int64_t)s * per + e];
  int64_t o = e;
  if (out_transposed) {
    int b = (int)(e % cb);
    int a = (int)((e / cb) % ca);
    int64_t k = e / ((int64_t)ca * cb);
    o = (k * cb + b) * ca + a;
  }
  out[o] = from_f32<T>(acc);
}

}  // namespace ocnn
