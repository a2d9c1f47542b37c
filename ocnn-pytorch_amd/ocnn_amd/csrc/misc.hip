// Depth-wise convolution (gather form), its weight gradient, pad / depad of
// feature rows, and the column sum used for the bias gradient.
#include <algorithm>

#include "common.hpp"
#include "mma.hpp"
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

// ---- depth-wise kernels with all KK slots per thread -------------------------------
// A thread owns 4 consecutive channels; C / 4 lanes cover a row and 256 / (C / 4) rows
// are in flight per workgroup.  The table rows of 64 rows are brought into LDS with
// coalesced loads; the feature rows are read with raw buffer loads whose offset is
// out of range for an empty entry (reads zero, no branch).  KK is a template parameter
// so that the slot loop has no branches at all.
constexpr int kDwChunk = 64;

template <typename T> struct DwVec;     // 4 channels
template <> struct DwVec<float> {
  static __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, uint32_t off, float (&v)[4]) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    const f32x4 f = __builtin_bit_cast(f32x4, t);     // (a bit cast of one element t[i] reads element 0)
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = f[i];
  }
};
template <> struct DwVec<f16> {
  static __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, uint32_t off, float (&v)[4]) {
    u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    typedef __attribute__((ext_vector_type(4))) _Float16 h4;
    h4 h = __builtin_bit_cast(h4, t);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (float)h[i];
  }
};
template <> struct DwVec<bf16> {
  static __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, uint32_t off, float (&v)[4]) {
    u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    v[0] = __builtin_bit_cast(float, t[0] << 16);
    v[1] = __builtin_bit_cast(float, t[0] & 0xffff0000u);
    v[2] = __builtin_bit_cast(float, t[1] << 16);
    v[3] = __builtin_bit_cast(float, t[1] & 0xffff0000u);
  }
};

template <typename T, int KK>
__global__ __launch_bounds__(256) void dw_gather_rows_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const int32_t* __restrict__ table, int64_t rows_out,
    const T* __restrict__ w, int C, int reverse, const T* __restrict__ bias, T* __restrict__ out,
    uint32_t out_bytes, int64_t rows_per_wg) {
  __shared__ int32_t s_tab[kDwChunk * KK];
  const int tid = threadIdx.x;
  const int lpr = C >> 2, rp = 256 / lpr;
  const int cl = tid % lpr, rl = tid / lpr;
  const uint32_t coff = (uint32_t)cl * 4u * (uint32_t)sizeof(T);
  const uint32_t row_bytes = (uint32_t)C * (uint32_t)sizeof(T);
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(w, (uint32_t)(KK * C) * (uint32_t)sizeof(T));
  float wr[KK][4], b4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < KK; ++k) DwVec<T>::load(rs_w, (uint32_t)(reverse ? KK - 1 - k : k) * row_bytes + coff, wr[k]);
  if (bias) {
    const __amdgpu_buffer_rsrc_t rs_b = make_rsrc(bias, row_bytes);
    DwVec<T>::load(rs_b, coff, b4);
  }
  const int64_t r_begin = (int64_t)blockIdx.x * rows_per_wg;
  const int64_t r_end = min(rows_out, r_begin + rows_per_wg);
  for (int64_t r0 = r_begin; r0 < r_end; r0 += kDwChunk) {
    const int nrows = (int)min<int64_t>(kDwChunk, r_end - r0);
    __syncthreads();
    for (int e = tid; e < nrows * KK; e += 256) s_tab[e] = table[r0 * KK + e];
    __syncthreads();
    for (int rr = rl; rr < nrows; rr += rp) {
      float acc[4] = {b4[0], b4[1], b4[2], b4[3]};
      float xv[KK][4];
#pragma unroll
      for (int k = 0; k < KK; ++k) {
        const int32_t idx = s_tab[rr * KK + k];
        DwVec<T>::load(rs_in, idx < 0 ? 0xffffff00u : (uint32_t)idx * row_bytes + coff, xv[k]);
      }
#pragma unroll
      for (int k = 0; k < KK; ++k)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[v] += xv[k][v] * wr[k][v];
      T* dst = out + (r0 + rr) * C + cl * 4;
      if constexpr (sizeof(T) == 4) {
        *(f32x4*)dst = f32x4{acc[0], acc[1], acc[2], acc[3]};
      } else {
        *(u32x2*)dst = u32x2{pack2<T>(acc[0], acc[1]), pack2<T>(acc[2], acc[3])};
      }
    }
  }
}

// partial[wg][k][c] = sum over the rows of workgroup wg
template <typename T, int KK>
__global__ __launch_bounds__(256) void dw_wgrad_rows_kernel(
    const T* __restrict__ x, uint32_t x_bytes, const T* __restrict__ g, uint32_t g_bytes,
    const int32_t* __restrict__ table, int64_t rows, int C, int64_t rows_per_wg,
    float* __restrict__ partial) {
  __shared__ int32_t s_tab[kDwChunk * KK];
  __shared__ float s_red[256 * 4];
  const int tid = threadIdx.x;
  const int lpr = C >> 2, rp = 256 / lpr;
  const int cl = tid % lpr, rl = tid / lpr;
  const uint32_t coff = (uint32_t)cl * 4u * (uint32_t)sizeof(T);
  const uint32_t row_bytes = (uint32_t)C * (uint32_t)sizeof(T);
  const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, x_bytes);
  const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(g, g_bytes);
  float acc[KK][4];
#pragma unroll
  for (int k = 0; k < KK; ++k)
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[k][v] = 0.f;
  const int64_t r_begin = (int64_t)blockIdx.x * rows_per_wg;
  const int64_t r_end = min(rows, r_begin + rows_per_wg);
  for (int64_t r0 = r_begin; r0 < r_end; r0 += kDwChunk) {
    const int nrows = (int)min<int64_t>(kDwChunk, r_end - r0);
    __syncthreads();
    for (int e = tid; e < nrows * KK; e += 256) s_tab[e] = table[r0 * KK + e];
    __syncthreads();
    for (int rr = rl; rr < nrows; rr += rp) {
      float gv[4], xv[KK][4];
      DwVec<T>::load(rs_g, (uint32_t)(r0 + rr) * row_bytes + coff, gv);
#pragma unroll
      for (int k = 0; k < KK; ++k) {
        const int32_t idx = s_tab[rr * KK + k];
        DwVec<T>::load(rs_x, idx < 0 ? 0xffffff00u : (uint32_t)idx * row_bytes + coff, xv[k]);
      }
#pragma unroll
      for (int k = 0; k < KK; ++k)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[k][v] += xv[k][v] * gv[v];
    }
  }
  // the row lanes of the workgroup, added in lane order
  float* dst = partial + (int64_t)blockIdx.x * KK * C;
#pragma unroll
  for (int k = 0; k < KK; ++k) {
    __syncthreads();
#pragma unroll
    for (int v = 0; v < 4; ++v) s_red[(rl * lpr + cl) * 4 + v] = acc[k][v];
    __syncthreads();
    for (int c = tid; c < C; c += 256) {                     // (more channels than threads from 512 on)
      float sum = 0.f;
      for (int r = 0; r < rp; ++r) sum += s_red[(r * lpr + (c >> 2)) * 4 + (c & 3)];
      dst[k * C + c] = sum;
    }
  }
}

// shapes the all-slots kernels take: C / 4 lanes per row must tile a 256-thread workgroup
static bool dw_rows_ok(int K, int C, int64_t rows_in, int es) {
  if (K != 27 && K != 9 && K != 8 && K != 3) return false;
  if (C < 4 || C > 1024 || (C & (C - 1)) != 0) return false;
  return (int64_t)rows_in * C * es < 0xfff00000ll;
}

// 16 bytes per thread: `chunks` 16-byte pieces per row
__global__ void pad16_kernel(const u32x4* __restrict__ data, const int32_t* __restrict__ children,
                             int64_t n, int chunks, u32x4 fill, u32x4* __restrict__ out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * chunks) return;
  int64_t q = t / chunks;
  int c = (int)(t % chunks);
  int32_t ch = children[q];
  if (data == nullptr) {                                   // only the rows of the empty nodes
    if (ch < 0) out[t] = fill;
    return;
  }
  out[t] = ch >= 0 ? data[(int64_t)ch * chunks + c] : fill;
}

__global__ void depad16_kernel(const u32x4* __restrict__ data, const int32_t* __restrict__ children,
                               int64_t n, int chunks, u32x4* __restrict__ out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * chunks) return;
  int64_t q = t / chunks;
  int c = (int)(t % chunks);
  int32_t ch = children[q];
  if (ch >= 0) out[(int64_t)ch * chunks + c] = data[t];
}

template <typename T>
__global__ void pad_kernel(const T* __restrict__ data, const int32_t* __restrict__ children,
                           int64_t n, int C, float val, T* __restrict__ out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * C) return;
  int64_t q = t / C;
  int c = (int)(t % C);
  int32_t ch = children[q];
  if (data == nullptr) {                                   // only the rows of the empty nodes
    if (ch < 0) out[t] = from_f32<T>(val);
    return;
  }
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

// The same with 16-byte pieces: a thread keeps one piece of the row (8 or 4 channels) and walks
// every (256 / pieces)-th row of the split, four loads in flight; the row lanes meet in LDS and
// are added in lane order.  C % (16 / sizeof(T)) == 0.
template <typename T>
__global__ __launch_bounds__(256) void colsum_rows_kernel(const T* __restrict__ g, int64_t rows, int C,
                                                          int64_t rows_per_split, float* __restrict__ partial) {
  constexpr int VEC = 16 / sizeof(T);
  struct alignas(16) Piece { T v[VEC]; };
  __shared__ float s_acc[256][VEC + 1];
  const int cpr = C / VEC;
  const int lanes_c = cpr < 256 ? cpr : 256, rpi = 256 / lanes_c;
  const int pc = threadIdx.x % lanes_c, rl = threadIdx.x / lanes_c;
  const int64_t r_begin = (int64_t)blockIdx.x * rows_per_split;
  const int64_t r_end = min(rows, r_begin + rows_per_split);
  for (int p0 = 0; p0 < cpr; p0 += lanes_c) {
    const int piece = p0 + pc;
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    if (rl < rpi && piece < cpr) {
      const Piece* src = reinterpret_cast<const Piece*>(g) + piece;
      int64_t i = r_begin + rl;
      for (; i + 3 * rpi < r_end; i += 4 * rpi) {
        Piece q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) q[u] = src[(i + u * rpi) * cpr];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int v = 0; v < VEC; ++v) acc[v] += to_f32(q[u].v[v]);
      }
      for (; i < r_end; i += rpi) {
        const Piece q = src[i * cpr];
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += to_f32(q.v[v]);
      }
    }
    __syncthreads();
#pragma unroll
    for (int v = 0; v < VEC; ++v) s_acc[threadIdx.x][v] = acc[v];
    __syncthreads();
    if (rl == 0 && piece < cpr) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        float sum = 0.f;
        for (int r = 0; r < rpi; ++r) sum += s_acc[r * lanes_c + pc][v];
        partial[(int64_t)blockIdx.x * C + piece * VEC + v] = sum;
      }
    }
  }
}

// Few channels that do not fill 16-byte pieces (C <= 256): the split's elements as one flat run,
// (256 / C) C threads walk it with that stride, so that a thread stays on one channel and a wave
// reads consecutive elements; eight loads in flight; threads of a channel meet in LDS, in thread order.
template <typename T>
__global__ __launch_bounds__(256) void colsum_flat_kernel(const T* __restrict__ g, int64_t rows, int C,
                                                          int64_t rows_per_split, float* __restrict__ partial) {
  __shared__ float s_acc[256];
  const int active = (256 / C) * C;
  const int64_t r_begin = (int64_t)blockIdx.x * rows_per_split;
  const int64_t r_end = min(rows, r_begin + rows_per_split);
  const int64_t f_end = r_end * C;
  float acc = 0.f;
  if ((int)threadIdx.x < active) {
    int64_t f = r_begin * C + threadIdx.x;
    for (; f + 7 * (int64_t)active < f_end; f += 8 * (int64_t)active) {
      T q[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) q[u] = g[f + u * (int64_t)active];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += to_f32(q[u]);
    }
    for (; f < f_end; f += active) acc += to_f32(g[f]);
  }
  s_acc[threadIdx.x] = acc;
  __syncthreads();
  if ((int)threadIdx.x < C) {
    float sum = 0.f;
    for (int t = threadIdx.x; t < active; t += C) sum += s_acc[t];
    partial[(int64_t)blockIdx.x * C + threadIdx.x] = sum;
  }
}

// out[c] = sum over the splits, 16 split lanes a channel, each adding every 16th split in order,
// the lanes then in lane order
template <typename T>
__global__ __launch_bounds__(1024) void colsum_finish_kernel(const float* __restrict__ partial, int splits, int C,
                                                             T* __restrict__ out) {
  __shared__ float s_acc[16][64];
  const int cl = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + cl;
  float acc = 0.f;
  if (c < C) {
#pragma unroll 4
    for (int s = sl; s < splits; s += 16) acc += partial[(int64_t)s * C + c];
  }
  s_acc[sl][cl] = acc;
  __syncthreads();
  if (sl == 0 && c < C) {
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) sum += s_acc[r][cl];
    out[c] = from_f32<T>(sum);
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
  OCNN_REQUIRE(rows_out >= 0 && rows_in >= 0, "dwconv_gather: negative row count");
  if (rows_out == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("dwconv_gather", in, table, w, out);
  hipStream_t st = (hipStream_t)stream;
  const int C = channels;
  if (dw_rows_ok(K, C, std::max(rows_in, rows_out), dtype_size(dtype))) {
    const int64_t wgs = std::min<int64_t>(cdiv(rows_out, kDwChunk), 2048);
    const int64_t per = align_up(cdiv(rows_out, wgs), kDwChunk);
    const unsigned grid = (unsigned)cdiv(rows_out, per);
#define OCNN_DW_GATHER(KK_)                                                                          \
  OCNN_DISPATCH_DTYPE(dtype, {                                                                       \
    hipLaunchKernelGGL((dw_gather_rows_kernel<T, KK_>), dim3(grid), dim3(256), 0, st, (const T*)in,  \
                       (uint32_t)(rows_in * C * sizeof(T)), table, rows_out, (const T*)w, C,         \
                       reverse_slots, (const T*)bias, (T*)out, (uint32_t)(rows_out * C * sizeof(T)), per); \
  })
    if (K == 27) OCNN_DW_GATHER(27);
    else if (K == 9) OCNN_DW_GATHER(9);
    else if (K == 8) OCNN_DW_GATHER(8);
    else OCNN_DW_GATHER(3);
#undef OCNN_DW_GATHER
    return check_launch("dwconv_gather");
  }
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
  OCNN_REQUIRE(rows >= 0 && rows_x >= 0, "dwconv_wgrad: negative row count");
  OCNN_REQUIRE_PTRS("dwconv_wgrad", gw, workspace);
  OCNN_REQUIRE(rows == 0 || (x && g && table), "dwconv_wgrad: a required pointer is NULL (of x, g, table)");
  hipStream_t st = (hipStream_t)stream;
  int64_t splits = 0, rps = 0;
  if (rows > 0) split_rows(rows, K, &splits, &rps);
  if (workspace_bytes < splits * K * channels * 4) {
    set_error("dwconv_wgrad: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  if (rows > 0 && dw_rows_ok(K, channels, std::max(rows_x, rows), dtype_size(dtype))) {
    const int C = channels;
    const int64_t wgs = std::min<int64_t>(cdiv(rows, kDwChunk), 512);
    const int64_t per = align_up(cdiv(rows, wgs), kDwChunk);
    const int used = (int)cdiv(rows, per);
    float* part = (float*)workspace;
#define OCNN_DW_WGRAD(KK_)                                                                         \
  OCNN_DISPATCH_DTYPE(dtype, {                                                                     \
    hipLaunchKernelGGL((dw_wgrad_rows_kernel<T, KK_>), dim3(used), dim3(256), 0, st, (const T*)x,  \
                       (uint32_t)(rows_x * C * sizeof(T)), (const T*)g,                            \
                       (uint32_t)(rows * C * sizeof(T)), table, rows, C, per, part);               \
    hipLaunchKernelGGL(wgrad_reduce_kernel<T>, dim3(cdiv((int64_t)K * C, 256)), dim3(256), 0, st,  \
                       part, used, K, 1, C, 0, (T*)gw);                                            \
  })
    if (K == 27) OCNN_DW_WGRAD(27);
    else if (K == 9) OCNN_DW_WGRAD(9);
    else if (K == 8) OCNN_DW_WGRAD(8);
    else OCNN_DW_WGRAD(3);
#undef OCNN_DW_WGRAD
    return check_launch("dwconv_wgrad");
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
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1 && n >= 0, "pad: bad arguments");
  if (n == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("pad", children, out);      // (data may be NULL: only the empty nodes' rows are written)
  hipStream_t st = (hipStream_t)stream;
  const int64_t row_bytes = (int64_t)channels * dtype_size(dtype);
  if (row_bytes % 16 == 0 && ((uintptr_t)data % 16 == 0) && ((uintptr_t)out % 16 == 0)) {
    const int chunks = (int)(row_bytes / 16);
    u32x4 fill;
    if (dtype == OCNN_F32) {
      const unsigned b = __builtin_bit_cast(unsigned, val);
      fill = u32x4{b, b, b, b};
    } else {
      unsigned short h;
      if (dtype == OCNN_F16) { f16 v = (f16)val; h = __builtin_bit_cast(unsigned short, v); }
      else { bf16 v = (bf16)val; h = __builtin_bit_cast(unsigned short, v); }
      const unsigned b = (unsigned)h | ((unsigned)h << 16);
      fill = u32x4{b, b, b, b};
    }
    hipLaunchKernelGGL(pad16_kernel, dim3(cdiv(n * chunks, 256)), dim3(256), 0, st, (const u32x4*)data,
                       children, n, chunks, fill, (u32x4*)out);
    return check_launch("pad");
  }
  OCNN_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL(pad_kernel<T>, dim3(cdiv(n * channels, 256)), dim3(256), 0, st,
                       (const T*)data, children, n, channels, val, (T*)out);
  });
  return check_launch("pad");
}

extern "C" int ocnn_depad(int dtype, const void* data, const int32_t* children, int64_t n,
                          int channels, void* out, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1 && n >= 0, "depad: bad arguments");
  if (n == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("depad", data, children, out);
  hipStream_t st = (hipStream_t)stream;
  const int64_t row_bytes = (int64_t)channels * dtype_size(dtype);
  if (row_bytes % 16 == 0 && ((uintptr_t)data % 16 == 0) && ((uintptr_t)out % 16 == 0)) {
    const int chunks = (int)(row_bytes / 16);
    hipLaunchKernelGGL(depad16_kernel, dim3(cdiv(n * chunks, 256)), dim3(256), 0, st, (const u32x4*)data,
                       children, n, chunks, (u32x4*)out);
    return check_launch("depad");
  }
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
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1 && rows >= 0, "colsum: bad arguments");
  OCNN_REQUIRE_PTRS("colsum", out, workspace);
  OCNN_REQUIRE(rows == 0 || g, "colsum: g is NULL");
  hipStream_t st = (hipStream_t)stream;
  int64_t splits = 0, rps = 0;
  if (rows > 0) split_rows(rows, 1, &splits, &rps);
  if (workspace_bytes < splits * channels * 4) {
    set_error("colsum: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  float* partial = (float*)workspace;
  OCNN_DISPATCH_DTYPE(dtype, {
    constexpr int VEC = 16 / sizeof(T);
    if (rows > 0) {
      if (channels % VEC == 0 && ((uintptr_t)g % 16) == 0)
        hipLaunchKernelGGL(colsum_rows_kernel<T>, dim3((unsigned)splits), dim3(256), 0, st, (const T*)g, rows,
                           channels, rps, partial);
      else if (channels <= 256)
        hipLaunchKernelGGL(colsum_flat_kernel<T>, dim3((unsigned)splits), dim3(256), 0, st, (const T*)g, rows,
                           channels, rps, partial);
      else
        hipLaunchKernelGGL(colsum_kernel<T>, dim3((unsigned)splits), dim3(256), 0, st, (const T*)g,
                           rows, channels, rps, partial);
    }
    hipLaunchKernelGGL(colsum_finish_kernel<T>, dim3((unsigned)cdiv((int64_t)channels, 64)), dim3(1024), 0, st,
                       partial, (int)splits, channels, (T*)out);
  });
  return check_launch("colsum");
}
