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

// The same for cb % 4 == 0: 16 bytes per thread and eight loads
// in flight; the additions stay in split order, so the result has the same bits.
// With ca > 0 the output is (K, cb, ca): the four sums of a thread (consecutive b) go to
// four rows of the transposed block.
template <typename T>
__global__ void wgrad_reduce4_kernel(const float* __restrict__ partial, int splits, int64_t per,
                                     T* __restrict__ out, int ca, int cb) {
  typedef __attribute__((ext_vector_type(4))) float v4;
  int64_t e = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (e >= per) return;
  v4 acc = v4{0.f, 0.f, 0.f, 0.f};
  int s = 0;
  for (; s + 8 <= splits; s += 8) {
    v4 v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = *(const v4*)(partial + (int64_t)(s + i) * per + e);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc += v[i];
  }
  for (; s < splits; ++s) acc += *(const v4*)(partial + (int64_t)s * per + e);
  if (ca > 0) {
    const int b = (int)(e % cb);
    const int a = (int)((e / cb) % ca);
    const int64_t k = e / ((int64_t)ca * cb);
#pragma unroll
    for (int i = 0; i < 4; ++i) out[(k * cb + b + i) * ca + a] = from_f32<T>(acc[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) out[e + i] = from_f32<T>(acc[i]);
  }
}

// fp32 values as two bf16 pieces: x = hi + lo (+ 2^-17 |x|); a product of two such values is
// hi_a hi_b + hi_a lo_b + lo_a hi_b to about 1e-5 relative
static __global__ void split2_kernel(const float* __restrict__ x, int64_t n, bf16* __restrict__ hi,
                              bf16* __restrict__ lo) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  float v = x[e];
  bf16 h = (bf16)v;
  hi[e] = h;
  lo[e] = (bf16)(v - (float)h);
}

// launches the reduction that fits
template <typename T>
inline void launch_wgrad_reduce(const float* partial, int splits, int K, int ca, int cb,
                                int out_transposed, T* out, hipStream_t st) {
  const int64_t per = (int64_t)K * ca * cb;
  if (cb % 4 == 0 && ((uintptr_t)partial % 16) == 0) {
    hipLaunchKernelGGL(wgrad_reduce4_kernel<T>, dim3((unsigned)cdiv(per / 4, 64)), dim3(64), 0, st, partial,
                       splits, per, out, out_transposed ? ca : 0, cb);
  } else {
    hipLaunchKernelGGL(wgrad_reduce_kernel<T>, dim3((unsigned)cdiv(per, 256)), dim3(256), 0, st, partial,
                       splits, K, ca, cb, out_transposed, out);
  }
}

}  // namespace ocnn
