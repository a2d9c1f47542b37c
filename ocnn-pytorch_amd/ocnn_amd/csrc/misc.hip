// Depth-wise convolution (gather form), its weight gradient, pad / depad of
// feature rows, and the column sum used for the bias gradient.
#include <algorithm>

#include "common.hpp"
#include "reduce.hpp"

namespace ocnn {

template <typename T, int VEC> struct alignas(sizeof(T) * VEC) Vec { T v[VEC]; };

template <typename T, int VEC>
__global__ __launch_bounds__(256) void dw_gather_kernel(
    const T* __restrict__ in, int64_t rows_in, const int32_t* __restrict__ table,
    int64_t rows_out, int K, const T* __restrict__ w, int C, int reverse,
    const T* __restrict__ bias, T* __restrict__ out) {
  typedef Vec<T, VEC> V;
  const int lpr = C / VEC;
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows_out * lpr) return;
  int64_t row = t / lpr;
  int c0 = (int)(t % lpr) * VEC;
  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
  for (int k = 0; k < K; ++k) {
    int32_t idx = table[row * K + k];
    if (idx < 0 || idx >= rows_in) continue;
    int kk = reverse ? K - 1 - k : k;
    V x = *(const V*)(in + (int64_t)idx * C + c0);
    V ww = *(const V*)(w + (int64_t)kk * C + c0);
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] += to_f32(x.v[v]) * to_f32(ww.v[v]);
  }
  V o;
#pragma unroll
  for (int v = 0; v < VEC; ++v) o.v[v] = from_f32<T>(acc[v] + (bias ? to_f32(bias[c0 + v]) : 0.f));
  *(V*)(out + row * C + c0) = o;
}

// partial[s][k][c] = sum over rows of split s; 4 row lanes x 64 channel lanes
template <typename T>
__global__ __launch_bounds__(256) void dw_wgrad_kernel(
    const T* __restrict__ x, int64_t rows_x, const T* __restrict__ g,
    const int32_t* __restrict__ table, int64_t rows, int K, int C, int64_t rows_per_split,
    float* __restrict__ partial) {
  __shared__ float s_acc[4][64];
  const int split = blockIdx.x, k = blockIdx.y;
  const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
  const int64_t r_begin = (int64_t)split * rows_per_split;
  const int64_t r_end = min(rows, r_begin + rows_per_split);
  for (int c0 = 0; c0 < C; c0 += 64) {
    int c = c0 + cl;
    float acc = 0.f;
    if (c < C) {
      for (int64_t i = r_begin + rl; i < r_end; i += 4) {
        int32_t idx = table[i * K + k];
        if (idx < 0 || idx >= rows_x) continue;
        acc += to_f32(x[(int64_t)idx * C + c]) * to_f32(g[i * C + c]);
      }
    }
    __syncthreads();
    s_acc[rl][cl] = acc;
    __syncthreads();
    if (rl == 0 && c < C)
      partial[((int64_t)split * K + k) * C + c] =
          ((s_acc[0][cl] + s_acc[1][cl]) + s_acc[2][cl]) + s_acc[3][cl];
  }
}

template <typename T>
__global__ void pad_kernel(const T* __restrict__ data, const int32_t* __restrict__ children,
                           int64_t n, int C, float val, T* __restrict__ out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * C) return;
  int64_t q = t / C;
  int c = (int)(t % C);
  int32_t ch = children[q];
  out[t] = ch >= 0 ? data[(int64_t)ch * C + c] : from_f32<T>(val);
}

template <typename T>
__global__ void depad_kernel(const T* __restrict__ data, const int32_t* __restrict__ children,
                             int64_t n, int C, T* __restrict__ out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * C) return;
  int64_t q = t / C;
  int c = (int)(t % C);
  int32_t ch = children[q];
  if (ch >= 0) out[(int64_t)ch * C + c] = data[t];
}

// partial[s][c] = sum of rows [s*rps, (s+1)*rps); 4 row lanes x 64 channel lanes
template <typename T>
__global__ __launch_bounds__(256) void colsum_kernel(const T* __restrict__ g, int64_t rows, int C,
                                                     int64_t rows_per_split,
                                                     float* __restrict__ partial) {
  __shared__ float s_acc[4][64];
  const int split = blockIdx.x;
  const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
  const int64_t r_begin = (int64_t)split * rows_per_split;
  const int64_t r_end = min(rows, r_begin + rows_per_split);
  for (int c0 = 0; c0 < C; c0 += 64) {
    int c = c0 + cl;
    float acc = 0.f;
    if (c < C)
      for (int64_t i = r_begin + rl; i < r_end; i += 4) acc += to_f32(g[i * C + c]);
    __syncthreads();
    s_acc[rl][cl] = acc;
    __syncthreads();
    if (rl == 0 && c < C)
      partial[(int64_t)split * C + c] =
          ((s_acc[0][cl] + s_acc[1][cl]) + s_acc[2][cl]) + s_acc[3][cl];
  }
}

static void split_rows(int64_t rows, int64_t cols, int64_t* splits, int64_t* rps) {
  int64_t s = std::max<int64_t>(1, std::min<int64_t>(cdiv(2048, std::max<int64_t>(1, cols)),
                                                     cdiv(rows, 256)));
  s = std::min<int64_t>(s, 512);
  *rps = cdiv(rows, s);
  *splits = cdiv(rows, *rps);
}

}  // namespace ocnn

using namespace ocnn;

#define OCNN_DISPATCH_DTYPE(dtype, ...)                      \
  do {                                                       \
    if (dtype == OCNN_F32) { typedef float T; __VA_ARGS__; } \
    else if (dtype == OCNN_F16) { typedef f16 T; __VA_ARGS__; } \
    else { typedef bf16 T; __VA_ARGS__; }                    \
  } while (0)

extern "C" int ocnn_dwconv_gather(int dtype, const void* in, int64_t rows_in,
                                  const int32_t* table, int64_t rows_out, int K, const void* w,
                                  int channels, int reverse_slots, const void* bias, void* out,
                                  void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2, "dwconv_gather: dtype %d", dtype);
  OCNN_REQUIRE(K >= 1 && K <= 27 && channels >= 1, "dwconv_gather: K=%d channels=%d", K, channels);
  if (rows_out <= 0) return OCNN_OK;
  hipStream_t st = (hipStream_t)stream;
  const int C = channels;
  OCNN_DISPATCH_DTYPE(dtype, {
    constexpr int VEC = 16 / sizeof(T);
    if (C % VEC == 0) {
      int64_t n = rows_out * (C / VEC);
      hipLaunchKernelGGL((dw_gather_kernel<T, VEC>), dim3(cdiv(n, 256)), dim3(256), 0, st,
                         (const T*)in, rows_in, table, rows_out, K, (const T*)w, C, reverse_slots,
                         (const T*)bias, (T*)out);
    } else {
      int64_t n = rows_out * C;
      hipLaunchKernelGGL((dw_gather_kernel<T, 1>), dim3(cdiv(n, 256)), dim3(256), 0, st,
                         (const T*)in, rows_in, table, rows_out, K, (const T*)w, C, reverse_slots,
                         (const T*)bias, (T*)out);
    }
  });
  return check_launch("dwconv_gather");
}

extern "C" int64_t ocnn_dwconv_wgrad_workspace_bytes(int64_t rows, int K, int channels) {
  return align_up((int64_t)512 * K * channels * 4, 256);
}

extern "C" int ocnn_dwconv_wgrad(int dtype, const void* x, int64_t rows_x, const void* g,
                                 const int32_t* table, int64_t rows, int K, int channels, void* gw,
                                 void* workspace, int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2, "dwconv_wgrad: dtype %d", dtype);
  OCNN_REQUIRE(K >= 1 && K <= 27 && channels >= 1, "dwconv_wgrad: K=%d channels=%d", K, channels);
  hipStream_t st = (hipStream_t)stream;
  int64_t splits = 0, rps = 0;
  if (rows > 0) split_rows(rows, K, &splits, &rps);
  if (workspace_bytes < splits * K * channels * 4) {
    set_error("dwconv_wgrad: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  float* partial = (float*)workspace;
  OCNN_DISPATCH_DTYPE(dtype, {
    if (rows > 0)
      hipLaunchKernelGGL(dw_wgrad_kernel<T>, dim3((unsigned)splits, K), dim3(256), 0, st,
                         (const T*)x, rows_x, (const T*)g, table, rows, K, channels, rps, partial);
    hipLaunchKernelGGL(wgrad_reduce_kernel<T>, dim3(cdiv((int64_t)K * channels, 256)), dim3(256), 0,
                       st, partial, (int)splits, K, 1, channels, 0, (T*)gw);
  });
  return check_launch("dwconv_wgrad");
}

extern "C" int ocnn_pad(int dtype, const void* data, const int32_t* children, int64_t n,
                        int channels, float val, void* out, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1, "pad: bad arguments");
  if (n <= 0) return OCNN_OK;
  hipStream_t st = (hipStream_t)stream;
  OCNN_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL(pad_kernel<T>, dim3(cdiv(n * channels, 256)), dim3(256), 0, st,
                       (const T*)data, children, n, channels, val, (T*)out);
  });
  return check_launch("pad");
}

extern "C" int ocnn_depad(int dtype, const void* data, const int32_t* children, int64_t n,
                          int channels, void* out, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1, "depad: bad arguments");
  if (n <= 0) return OCNN_OK;
  hipStream_t st = (hipStream_t)stream;
  OCNN_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL(depad_kernel<T>, dim3(cdiv(n * channels, 256)), dim3(256), 0, st,
                       (const T*)data, children, n, channels, (T*)out);
  });
  return check_launch("depad");
}

extern "C" int64_t ocnn_colsum_workspace_bytes(int64_t rows, int channels) {
  return align_up((int64_t)512 * channels * 4, 256);
}

extern "C" int ocnn_colsum(int dtype, const void* g, int64_t rows, int channels, void* out,
                           void* workspace, int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1, "colsum: bad arguments");
  hipStream_t st = (hipStream_t)stream;
  int64_t splits = 0, rps = 0;
  if (rows > 0) split_rows(rows, 1, &splits, &rps);
  if (workspace_bytes < splits * channels * 4) {
    set_error("colsum: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  float* partial = (float*)workspace;
  OCNN_DISPATCH_DTYPE(dtype, {
    if (rows > 0)
      hipLaunchKernelGGL(colsum_kernel<T>, dim3((unsigned)splits), dim3(256), 0, st, (const T*)g,
                         rows, channels, rps, partial);
    hipLaunchKernelGGL(wgrad_reduce_kernel<T>, dim3(cdiv((int64_t)channels, 256)), dim3(256), 0, st,
                       partial, (int)splits, 1, 1, channels, 0, (T*)out);
  });
  return check_launch("colsum");
}
