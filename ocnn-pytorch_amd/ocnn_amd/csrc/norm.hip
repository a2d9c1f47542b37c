// Batch normalisation over the rows of a (rows, C) feature matrix with the ReLU that follows
// it in every conv-bn-relu block fused in: training statistics, the normalise (+ ReLU) pass,
// and the gradient.  Everything here is HBM-bound; the point of the fusion is the number of
// passes over the tensor (forward 2 reads + 1 write, backward 4 reads + 1 write, the ReLU
// costs none) and 16-byte accesses on channels-last rows.  Reductions are two-level with a
// fixed order (per-workgroup partial sums, then one thread per channel in fp64): no atomics,
// bit-reproducible.
#include <algorithm>
#include <mutex>
#include <utility>
#include <vector>

#include "common.hpp"

namespace ocnn {

constexpr int kBnMaxBlocks = 512;     // workgroups of a reduction (their partial sums are added by one more kernel)
constexpr int kBnApplyBlocks = 2048;  // workgroups of an elementwise pass, at most (fewer where the device holds fewer at once)

template <typename T, int VEC> struct alignas(sizeof(T) * VEC) BnVec { T v[VEC]; };

// element c of a per-channel parameter held as f32 / f16 / bf16 (p == nullptr: dflt)
__device__ __forceinline__ float bn_param(const void* p, int dtype, int c, float dflt) {
  if (!p) return dflt;
  if (dtype == OCNN_F32) return ((const float*)p)[c];
  if (dtype == OCNN_F16) return to_f32(((const f16*)p)[c]);
  return to_f32(((const bf16*)p)[c]);
}

// gamma and beta of the channels c0 .. c0 + VEC - 1 (1 and 0 where the pointer is null).  The raw
// values of both are requested before either is converted, so that a workgroup waits for one
// round trip to memory and not for one per channel.
template <int VEC>
__device__ __forceinline__ void bn_params(const void* __restrict__ gamma, const void* __restrict__ beta, int dtype,
                                          int c0, float (&ga)[VEC], float (&be)[VEC]) {
  if (dtype == OCNN_F32) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      ga[v] = gamma ? ((const float*)gamma)[c0 + v] : 1.f;
      be[v] = beta ? ((const float*)beta)[c0 + v] : 0.f;
    }
    return;
  }
  // f16: 1.0 = 0x3c00; bf16: 1.0 = 0x3f80
  unsigned short rg[VEC], rb[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    rg[v] = gamma ? ((const unsigned short*)gamma)[c0 + v] : (unsigned short)(dtype == OCNN_F16 ? 0x3c00 : 0x3f80);
    rb[v] = beta ? ((const unsigned short*)beta)[c0 + v] : (unsigned short)0;
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    if (dtype == OCNN_F16) {
      ga[v] = to_f32(__builtin_bit_cast(f16, rg[v]));
      be[v] = to_f32(__builtin_bit_cast(f16, rb[v]));
    } else {
      ga[v] = __uint_as_float((uint32_t)rg[v] << 16);
      be[v] = __uint_as_float((uint32_t)rb[v] << 16);
    }
  }
}

__device__ __forceinline__ void bn_store(void* p, int dtype, int c, float v) {
  if (dtype == OCNN_F32) ((float*)p)[c] = v;
  else if (dtype == OCNN_F16) ((f16*)p)[c] = from_f32<f16>(v);
  else ((bf16*)p)[c] = from_f32<bf16>(v);
}

// partial[blk][0][c] = sum_r (x[r][c] - x[0][c]),  partial[blk][1][c] = sum_r (x[r][c] - x[0][c])^2
// over the rows of the workgroup (shifting by the first row keeps the variance free of
// cancellation when the mean is large against the spread).  Thread: VEC channels of every
// rpp-th row.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void bn_stats_kernel(const T* __restrict__ x, int64_t rows, int C,
                                                       int64_t rows_per_blk, float* __restrict__ partial) {
  typedef BnVec<T, VEC> V;
  __shared__ float s_a[256 * VEC], s_b[256 * VEC];
  const int lpr = C / VEC, rpp = 256 / lpr;
  const int tid = threadIdx.x, rl = tid / lpr, cl = tid - rl * lpr;
  float s1[VEC], s2[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) s1[v] = s2[v] = 0.f;
  if (rl < rpp) {
    const V k = *(const V*)(x + cl * VEC);
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_blk;
    const int64_t r1 = min(rows, r0 + rows_per_blk);
    // four rows in flight per thread (rows past the end repeat row 0, whose shifted value is 0)
    for (int64_t r = r0 + rl; r < r1; r += 4 * rpp) {
      V a[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t ru = r + (int64_t)u * rpp;
        a[u] = *(const V*)(x + (ru < r1 ? ru * C : 0) + cl * VEC);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          const float d = to_f32(a[u].v[v]) - to_f32(k.v[v]);
          s1[v] += d;
          s2[v] += d * d;
        }
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    s_a[tid * VEC + v] = s1[v];
    s_b[tid * VEC + v] = s2[v];
  }
  __syncthreads();
  if (tid < lpr) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float a = 0.f, b = 0.f;
      for (int g = 0; g < rpp; ++g) {
        a += s_a[(g * lpr + tid) * VEC + v];
        b += s_b[(g * lpr + tid) * VEC + v];
      }
      partial[((int64_t)blockIdx.x * 2 + 0) * C + tid * VEC + v] = a;
      partial[((int64_t)blockIdx.x * 2 + 1) * C + tid * VEC + v] = b;
    }
  }
}

// Sum of the per-workgroup partial sums of a channel, in a fixed order: 256 threads = 64
// lanes x 4 channels, lane l adds the partials l, l + 64, .. (fp64), then lane 0 adds the
// 64 lane sums.  Returns the channel for the threads that hold a result, -1 for the others.
__device__ __forceinline__ int bn_sum_partials(const float* __restrict__ partial, int nblk, int C, double& a,
                                               double& b) {
  __shared__ double s_pa[256], s_pb[256];
  const int tid = threadIdx.x, l = tid >> 2;
  const int c = blockIdx.x * 4 + (tid & 3);
  double sa = 0.0, sb = 0.0;
  if (c < C) {
    for (int i = l; i < nblk; i += 256) {                    // four loads of each kind in flight
      float va[4], vb[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int iu = i + 64 * u;
        va[u] = iu < nblk ? partial[((int64_t)iu * 2 + 0) * C + c] : 0.f;
        vb[u] = iu < nblk ? partial[((int64_t)iu * 2 + 1) * C + c] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        sa += (double)va[u];
        sb += (double)vb[u];
      }
    }
  }
  s_pa[tid] = sa;
  s_pb[tid] = sb;
  __syncthreads();
  if (l != 0 || c >= C) return -1;
  a = 0.0;
  b = 0.0;
  for (int k = 0; k < 64; ++k) {
    a += s_pa[4 * k + tid];
    b += s_pb[4 * k + tid];
  }
  return c;
}

// mean, biased variance and 1 / sqrt(var + eps) per channel from the partial sums
// running_mean / running_var (dtype rdtype), when given, move towards the batch statistics by
// `factor` (the running variance towards the unbiased one), as torch.nn.functional.batch_norm.
template <typename T>
__global__ void bn_stats_finish_kernel(const float* __restrict__ partial, int nblk, const T* __restrict__ x,
                                       int64_t rows, int C, float eps, float* __restrict__ mean,
                                       float* __restrict__ var, float* __restrict__ invstd,
                                       void* running_mean, void* running_var, int rdtype, float factor,
                                       long long* batches_tracked) {
  // (the module's count of training batches, kept here to spare a launch of its own)
  if (batches_tracked != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *batches_tracked += 1;
  double a, b;
  const int c = bn_sum_partials(partial, nblk, C, a, b);
  if (c < 0) return;
  const double m = a / (double)rows;
  const double v = fmax(b / (double)rows - m * m, 0.0);
  mean[c] = (float)((double)to_f32(x[c]) + m);
  var[c] = (float)v;
  invstd[c] = (float)(1.0 / sqrt(v + (double)eps));
  if (running_mean) {
    const float unbiased = (float)(v * ((double)rows / (double)max(rows - 1, (int64_t)1)));
    bn_store(running_mean, rdtype, c, (1.f - factor) * bn_param(running_mean, rdtype, c, 0.f) + factor * mean[c]);
    bn_store(running_var, rdtype, c, (1.f - factor) * bn_param(running_var, rdtype, c, 0.f) + factor * unbiased);
  }
}

// y = (x - mean) * (invstd * gamma) + beta (+ res), then max(., 0) when relu.  A thread keeps the
// constants of its VEC channels in registers and walks every rpp-th row of the workgroup's
// range, four rows in flight.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void bn_apply_kernel(const T* __restrict__ x, int64_t rows, int C,
                                                       int64_t rows_per_blk,
                                                       const float* __restrict__ mean,
                                                       const float* __restrict__ invstd,
                                                       const void* __restrict__ gamma,
                                                       const void* __restrict__ beta, int pdtype, int relu,
                                                       const T* __restrict__ res, T* __restrict__ y) {
  typedef BnVec<T, VEC> V;
  const int lpr = C / VEC, rpp = 256 / lpr;
  const int tid = threadIdx.x, rl = tid / lpr, cl = tid - rl * lpr;
  if (rl >= rpp) return;
  float m[VEC], sc[VEC], be[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    m[v] = mean[cl * VEC + v];
    sc[v] = invstd[cl * VEC + v];
  }
  {
    float ga[VEC];
    bn_params<VEC>(gamma, beta, pdtype, cl * VEC, ga, be);
#pragma unroll
    for (int v = 0; v < VEC; ++v) sc[v] *= ga[v];
  }
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_blk;
  const int64_t r1 = min(rows, r0 + rows_per_blk);
  for (int64_t r = r0 + rl; r < r1; r += 4 * rpp) {
    V a[4], b[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t ru = r + (int64_t)u * rpp;
      if (ru < r1) {
        a[u] = *(const V*)(x + ru * C + cl * VEC);
        if (res) b[u] = *(const V*)(res + ru * C + cl * VEC);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t ru = r + (int64_t)u * rpp;
      if (ru >= r1) continue;
      V o;
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        float t = (to_f32(a[u].v[v]) - m[v]) * sc[v] + be[v];
        if (res) t = to_f32(from_f32<T>(t)) + to_f32(b[u].v[v]);      // (rounded as the separate passes would)
        if (relu) t = fmaxf(t, 0.f);
        o.v[v] = from_f32<T>(t);
      }
      *(V*)(y + ru * C + cl * VEC) = o;
    }
  }
}

// partial[blk][0][c] = sum_r dy'[r][c],  partial[blk][1][c] = sum_r dy'[r][c] * xhat[r][c], with
// xhat = (x - mean) * invstd and dy' = dy where the forward output was positive (relu) or dy.
// ymask: the forward output, when it is not a function of x alone (a residual was added).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void bn_bwd_stats_kernel(const T* __restrict__ x, const T* __restrict__ dy,
                                                           int64_t rows, int C, int64_t rows_per_blk,
                                                           const float* __restrict__ mean,
                                                           const float* __restrict__ invstd,
                                                           const void* __restrict__ gamma,
                                                           const void* __restrict__ beta, int pdtype, int relu,
                                                           const T* __restrict__ ymask,
                                                           float* __restrict__ partial) {
  typedef BnVec<T, VEC> V;
  __shared__ float s_a[256 * VEC], s_b[256 * VEC];
  const int lpr = C / VEC, rpp = 256 / lpr;
  const int tid = threadIdx.x, rl = tid / lpr, cl = tid - rl * lpr;
  float s1[VEC], s2[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) s1[v] = s2[v] = 0.f;
  if (rl < rpp) {
    float m[VEC], is[VEC], ga[VEC], be[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      m[v] = mean[cl * VEC + v];
      is[v] = invstd[cl * VEC + v];
    }
    bn_params<VEC>(gamma, beta, pdtype, cl * VEC, ga, be);
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_blk;
    const int64_t r1 = min(rows, r0 + rows_per_blk);
    for (int64_t r = r0 + rl; r < r1; r += 4 * rpp) {          // four rows of both tensors in flight
      V a[4], g[4], ym[4];
      bool ok[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t ru = r + (int64_t)u * rpp;
        ok[u] = ru < r1;
        a[u] = *(const V*)(x + (ok[u] ? ru * C : 0) + cl * VEC);
        g[u] = *(const V*)(dy + (ok[u] ? ru * C : 0) + cl * VEC);
        if (ymask) ym[u] = *(const V*)(ymask + (ok[u] ? ru * C : 0) + cl * VEC);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          const float xc = to_f32(a[u].v[v]) - m[v];
          const float xh = xc * is[v];
          float d = ok[u] ? to_f32(g[u].v[v]) : 0.f;
          if (relu && !(ymask ? to_f32(ym[u].v[v]) > 0.f
                              : xc * (is[v] * ga[v]) + be[v] > 0.f)) d = 0.f;       // the forward pass's expression
          s1[v] += d;
          s2[v] += d * xh;
        }
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    s_a[tid * VEC + v] = s1[v];
    s_b[tid * VEC + v] = s2[v];
  }
  __syncthreads();
  if (tid < lpr) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float a = 0.f, b = 0.f;
      for (int g = 0; g < rpp; ++g) {
        a += s_a[(g * lpr + tid) * VEC + v];
        b += s_b[(g * lpr + tid) * VEC + v];
      }
      partial[((int64_t)blockIdx.x * 2 + 0) * C + tid * VEC + v] = a;
      partial[((int64_t)blockIdx.x * 2 + 1) * C + tid * VEC + v] = b;
    }
  }
}

// (gw / gb: the same sums in the parameters' dtype, when given)
__global__ void bn_bwd_finish_kernel(const float* __restrict__ partial, int nblk, int C,
                                     float* __restrict__ dbeta, float* __restrict__ dgamma, void* gw, void* gb,
                                     int pdtype) {
  double a, b;
  const int c = bn_sum_partials(partial, nblk, C, a, b);
  if (c < 0) return;
  dbeta[c] = (float)a;
  dgamma[c] = (float)b;
  if (gw) bn_store(gw, pdtype, c, (float)b);
  if (gb) bn_store(gb, pdtype, c, (float)a);
}

// training: dx = gamma * invstd * (dy' - dbeta / N - xhat * dgamma / N); with fixed statistics
// (evaluation mode): dx = gamma * invstd * dy'.  Thread layout as in bn_apply_kernel.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void bn_bwd_apply_kernel(const T* __restrict__ x, const T* __restrict__ dy,
                                                           int64_t rows, int C, int64_t rows_per_blk,
                                                           const float* __restrict__ mean,
                                                           const float* __restrict__ invstd,
                                                           const void* __restrict__ gamma,
                                                           const void* __restrict__ beta, int pdtype, int relu,
                                                           const float* __restrict__ dbeta,
                                                           const float* __restrict__ dgamma, int training,
                                                           const T* __restrict__ ymask, T* __restrict__ dres,
                                                           T* __restrict__ dx) {
  typedef BnVec<T, VEC> V;
  const int lpr = C / VEC, rpp = 256 / lpr;
  const int tid = threadIdx.x, rl = tid / lpr, cl = tid - rl * lpr;
  if (rl >= rpp) return;
  const float inv_n = 1.0f / (float)rows;
  float m[VEC], is[VEC], sc[VEC], be[VEC], db[VEC], dg[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    const int c = cl * VEC + v;
    m[v] = mean[c];
    is[v] = invstd[c];
    db[v] = training ? dbeta[c] * inv_n : 0.f;
    dg[v] = training ? dgamma[c] * inv_n : 0.f;
  }
  bn_params<VEC>(gamma, beta, pdtype, cl * VEC, sc, be);
#pragma unroll
  for (int v = 0; v < VEC; ++v) sc[v] *= is[v];
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_blk;
  const int64_t r1 = min(rows, r0 + rows_per_blk);
  for (int64_t r = r0 + rl; r < r1; r += 2 * rpp) {     // (four rows in flight cost more in occupancy than they gain)
    V a[2], g[2], ym[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int64_t ru = r + (int64_t)u * rpp;
      if (ru < r1) {
        a[u] = *(const V*)(x + ru * C + cl * VEC);
        g[u] = *(const V*)(dy + ru * C + cl * VEC);
        if (ymask) ym[u] = *(const V*)(ymask + ru * C + cl * VEC);
      }
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int64_t ru = r + (int64_t)u * rpp;
      if (ru >= r1) continue;
      V o, gr;
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float xc = to_f32(a[u].v[v]) - m[v];
        float d = to_f32(g[u].v[v]);
        if (relu && !(ymask ? to_f32(ym[u].v[v]) > 0.f : xc * sc[v] + be[v] > 0.f)) d = 0.f;
        gr.v[v] = from_f32<T>(d);                                      // the gradient of the residual
        if (training) d = d - db[v] - (xc * is[v]) * dg[v];
        o.v[v] = from_f32<T>(d * sc[v]);
      }
      *(V*)(dx + ru * C + cl * VEC) = o;
      if (dres) *(V*)(dres + ru * C + cl * VEC) = gr;
    }
  }
}

}  // namespace ocnn

using namespace ocnn;

#define OCNN_DISPATCH_DTYPE(dtype, ...)                      \
  do {                                                       \
    if (dtype == OCNN_F32) { typedef float T; __VA_ARGS__; } \
    else if (dtype == OCNN_F16) { typedef f16 T; __VA_ARGS__; } \
    else { typedef bf16 T; __VA_ARGS__; }                    \
  } while (0)

static int bn_vec(int dtype) { return dtype == OCNN_F32 ? 4 : 8; }

extern "C" int ocnn_batch_norm_supported(int dtype, int64_t rows, int channels) {
  if (dtype < 0 || dtype > 2) return 0;
  const int vec = bn_vec(dtype);
  if (channels < vec || channels % vec != 0 || channels / vec > 256) return 0;
  return rows >= 1;
}

// rows of a workgroup (a multiple of the rows its threads cover per pass) and their number
static void bn_blocks(int dtype, int64_t rows, int channels, int max_blocks, int64_t* per, int* nblk) {
  const int rpp = 256 / (channels / bn_vec(dtype));
  *per = align_up(std::max<int64_t>(cdiv(rows, max_blocks), 4 * rpp), rpp);
  *nblk = (int)cdiv(rows, *per);
}

// Workgroups of 256 threads of `kernel` that the device holds at once, kBnApplyBlocks at most:
// an elementwise pass launched with more runs them in rounds, and the last round leaves CUs idle.
static int bn_resident_blocks(const void* kernel) {
  static std::mutex mu;
  static std::vector<std::pair<const void*, int>> known;
  std::lock_guard<std::mutex> lock(mu);
  for (const auto& k : known)
    if (k.first == kernel) return k.second;
  int per_cu = 0, dev = 0, n_cu = 256;
  (void)hipGetDevice(&dev);
  (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess || per_cu < 1) {
    (void)hipGetLastError();
    per_cu = 2;
  }
  const int cap = std::min(kBnApplyBlocks, std::max(1, per_cu * n_cu));
  known.emplace_back(kernel, cap);
  return cap;
}

extern "C" int64_t ocnn_batch_norm_workspace_bytes(int channels) {
  return align_up((int64_t)kBnMaxBlocks * 2 * channels * 4, 256);
}

extern "C" int ocnn_batch_norm_stats(int dtype, const void* x, int64_t rows, int channels, float eps,
                                     float* mean, float* var, float* invstd, void* running_mean,
                                     void* running_var, int running_dtype, float factor,
                                     int64_t* batches_tracked, void* workspace, int64_t workspace_bytes,
                                     void* stream) {
  OCNN_REQUIRE(ocnn_batch_norm_supported(dtype, rows, channels), "batch_norm_stats: shape not supported");
  OCNN_REQUIRE_PTRS("batch_norm_stats", x, mean, var, invstd, workspace);
  OCNN_REQUIRE(workspace_bytes >= ocnn_batch_norm_workspace_bytes(channels), "batch_norm_stats: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  int64_t per;
  int nblk;
  bn_blocks(dtype, rows, channels, kBnMaxBlocks, &per, &nblk);
  float* partial = (float*)workspace;
  OCNN_DISPATCH_DTYPE(dtype, {
    constexpr int VEC = 16 / sizeof(T);
    hipLaunchKernelGGL((bn_stats_kernel<T, VEC>), dim3(nblk), dim3(256), 0, st, (const T*)x, rows, channels, per,
                       partial);
    hipLaunchKernelGGL(bn_stats_finish_kernel<T>, dim3((unsigned)cdiv(channels, 4)), dim3(256), 0, st, partial, nblk,
                       (const T*)x, rows, channels, eps, mean, var, invstd, running_mean, running_var, running_dtype,
                       factor, (long long*)batches_tracked);
  });
  return check_launch("batch_norm_stats");
}

extern "C" int ocnn_batch_norm_apply(int dtype, const void* x, int64_t rows, int channels, const float* mean,
                                     const float* invstd, const void* gamma, const void* beta, int param_dtype,
                                     int relu, const void* residual, void* y, void* stream) {
  OCNN_REQUIRE(ocnn_batch_norm_supported(dtype, rows, channels), "batch_norm_apply: shape not supported");
  OCNN_REQUIRE_PTRS("batch_norm_apply", x, mean, invstd, y);
  hipStream_t st = (hipStream_t)stream;
  int64_t per;
  int nblk;
  OCNN_DISPATCH_DTYPE(dtype, {
    constexpr int VEC = 16 / sizeof(T);
    bn_blocks(dtype, rows, channels, bn_resident_blocks((const void*)bn_apply_kernel<T, VEC>), &per, &nblk);
    hipLaunchKernelGGL((bn_apply_kernel<T, VEC>), dim3(nblk), dim3(256), 0, st, (const T*)x, rows, channels, per,
                       mean, invstd, gamma, beta, param_dtype, relu, (const T*)residual, (T*)y);
  });
  return check_launch("batch_norm_apply");
}

extern "C" int ocnn_batch_norm_backward(int dtype, const void* x, const void* dy, int64_t rows, int channels,
                                        const float* mean, const float* invstd, const void* gamma,
                                        const void* beta, int param_dtype, int relu, int training,
                                        const void* y, void* dx, void* d_residual, float* dgamma, float* dbeta,
                                        void* grad_gamma, void* grad_beta, void* workspace,
                                        int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(!d_residual || dx, "batch_norm_backward: d_residual needs dx");
  OCNN_REQUIRE(ocnn_batch_norm_supported(dtype, rows, channels), "batch_norm_backward: shape not supported");
  OCNN_REQUIRE_PTRS("batch_norm_backward", x, dy, mean, invstd, dgamma, dbeta, workspace);
  OCNN_REQUIRE(workspace_bytes >= ocnn_batch_norm_workspace_bytes(channels),
               "batch_norm_backward: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  int64_t per;
  int nblk;
  int64_t per_a;
  int nblk_a;
  bn_blocks(dtype, rows, channels, kBnMaxBlocks, &per, &nblk);
  float* partial = (float*)workspace;
  OCNN_DISPATCH_DTYPE(dtype, {
    constexpr int VEC = 16 / sizeof(T);
    bn_blocks(dtype, rows, channels, bn_resident_blocks((const void*)bn_bwd_apply_kernel<T, VEC>), &per_a, &nblk_a);
    hipLaunchKernelGGL((bn_bwd_stats_kernel<T, VEC>), dim3(nblk), dim3(256), 0, st, (const T*)x, (const T*)dy, rows,
                       channels, per, mean, invstd, gamma, beta, param_dtype, relu, (const T*)y, partial);
    hipLaunchKernelGGL(bn_bwd_finish_kernel, dim3((unsigned)cdiv(channels, 4)), dim3(256), 0, st, partial, nblk,
                       channels, dbeta, dgamma, grad_gamma, grad_beta, param_dtype);
    if (dx)
      hipLaunchKernelGGL((bn_bwd_apply_kernel<T, VEC>), dim3(nblk_a), dim3(256), 0, st, (const T*)x, (const T*)dy, rows,
                         channels, per_a, mean, invstd, gamma, beta, param_dtype, relu, dbeta, dgamma, training,
                         (const T*)y, (T*)d_residual, (T*)dx);
  });
  return check_launch("batch_norm_backward");
}
