// Depth-wise convolution and its weight gradient on the tile plan of the neighbour table.
//
//   out[i][c]  = sum_k x[T[i][k]][c] * w[k][c]
//   gw[k][c]   = sum_i x[T[i][k]][c] * g[i][c]
//
// Reading the 27 neighbour rows of every row from L2 makes the plan-free kernels L2-bound
// (27 x the algorithmic bytes).  Here a workgroup stages the distinct rows of a 128-row
// tile, 64 channels of them, ONCE in LDS (asynchronous global->LDS loads) and every
// neighbour read is a 16-byte LDS read.  Two workgroups share a CU: one computes while the
// other one's rows are in flight.  fp32 accumulation; the weight gradient keeps the sums of
// KG slots in registers over a range of tiles, adds the threads of a workgroup in a fixed
// order and leaves per-range sums to the split reduction (no atomics).
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "mma.hpp"
#include "reduce.hpp"

namespace ocnn {

constexpr int kDpRows = 128;   // rows per tile (the plan's tile size)
constexpr int kDpCap = 416;    // staged rows; plans with a larger tile use another kernel
constexpr int kDpRowsAlloc = (kDpCap + 8) / 8 * 8;

// (Not in the kernel templates: the arguments of the global->LDS load builtin must not be
// type-dependent expressions.)
static __device__ __forceinline__ void dp_dma16(__amdgpu_buffer_rsrc_t rs, char* dst, uint32_t off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)dst, 16, off, 0, 0, 0);
}

template <typename T> struct Dp8 { typedef T V __attribute__((ext_vector_type(8))); };

template <typename T>
static __device__ __forceinline__ void dp_unpack(u32x4 v, float (&f)[8]) {
  typename Dp8<T>::V t = __builtin_bit_cast(typename Dp8<T>::V, v);
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (float)t[e];
}

// acc += a.lo * b.lo + a.hi * b.hi in fp32 (v_dot2c_f32_{f16,bf16}), a and b pairs of 16-bit
// values.  With one half of b zero this is a multiply-add of ONE channel of the pair straight
// out of the packed register: no unpacking of the 16-bit operand, one instruction per product.
template <typename T> static __device__ __forceinline__ float dp_dot2(unsigned a, unsigned b, float acc);
template <> __device__ __forceinline__ float dp_dot2<bf16>(unsigned a, unsigned b, float acc) {
  typedef __attribute__((ext_vector_type(2))) __bf16 v2;
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), acc, false);
}
template <> __device__ __forceinline__ float dp_dot2<f16>(unsigned a, unsigned b, float acc) {
  typedef __attribute__((ext_vector_type(2))) _Float16 v2;
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), acc, false);
}

// 8 channels of one operand as (value, 0) and (0, value) pairs: lo[e] multiplies channel 2 e of a
// packed register, hi[e] channel 2 e + 1.
static __device__ __forceinline__ void dp_split(u32x4 v, unsigned (&lo)[4], unsigned (&hi)[4]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    lo[e] = v[e] & 0x0000ffffu;
    hi[e] = v[e] & 0xffff0000u;
  }
}

// Table positions (16 bits each, two per dword, at most 511) -> byte offsets of the LDS rows with
// the swizzle bits in place: (p << 7) | (((p >> 1) & 7) << 4); a thread's 16-byte chunk c of that
// row is then at offset ^ (c << 4).  Position 0 (empty entry) stays 0: the zero row.
static __device__ __forceinline__ u32x4 dp_loc_offsets(u32x4 v) {
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = (v[e] << 7) | ((v[e] & 0x000e000eu) << 3);
  return v;
}

// Stages the 64-channel chunk `chunk` of the rows in the list s_u (LDS row p = list entry
// p - 1, row 0 and everything past the list = zeros) into s_rows.  A lane's 16-byte chunk c
// of LDS row p lands at chunk c ^ ((p >> 1) & 7) (bank swizzle).
static __device__ __forceinline__ void dp_stage_rows(__amdgpu_buffer_rsrc_t rs, char* s_rows, const int32_t* s_u,
                                                     int groups, uint32_t pitch, uint32_t coff, int wave, int lane) {
  const uint32_t st_c = (uint32_t)(((lane & 7) ^ (((lane >> 4) + 4 * wave) & 7)) * 16);
  const int st_p = 8 * wave + (lane >> 3);
  constexpr int kRowPieces = (kDpCap + 1 + 31) / 32;
#pragma unroll
  for (int i = 0; i < kRowPieces; ++i) {
    const int g = wave + 4 * i;
    if (g < groups) {
      const int32_t id = s_u[st_p + 32 * i];                 // -1: out of range, loads zeros
      dp_dma16(rs, s_rows + g * 1024, (uint32_t)id * pitch + (coff + st_c));
    }
  }
}

// One workgroup: 128 rows x 64 channels.  Thread t: 16-byte chunk t % 8 of the rows
// t / 8 + 32 j, j = 0..3.
template <typename T>
__global__ __launch_bounds__(256, 2) void dw_gather_planned_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const uint16_t* __restrict__ loc,
    const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows, const T* __restrict__ w,
    const T* __restrict__ bias, T* __restrict__ out, int64_t rows_out, int K, int C, int reverse,
    int64_t tiles, int64_t tiles_per_xcd, int nchunk) {
  __shared__ __attribute__((aligned(16))) T s_rows[kDpRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc[27 * kDpRows];
  __shared__ __attribute__((aligned(16))) T s_w[27 * 64];
  __shared__ int32_t s_u[kDpRowsAlloc];

  // the chunks of a tile run on the same XCD (they read the same rows and positions)
  const int bid = blockIdx.x;
  const int64_t idx = bid >> 3;
  const int chunk = (int)(idx % nchunk);
  const int64_t tile = (bid & 7) * tiles_per_xcd + idx / nchunk;
  if (tile >= tiles) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = tid & 7, r0 = tid >> 3;

  const int32_t p0 = uptr[tile];
  const int U = uptr[tile + 1] - p0;
  for (int i = tid; i < kDpRowsAlloc; i += 256) s_u[i] = (i >= 1 && i <= U) ? urows[p0 + i - 1] : -1;
  {
    const u32x4* src = (const u32x4*)(loc + tile * (int64_t)(kDpRows * K));
    for (int i = tid; i < K * 16; i += 256) ((u32x4*)s_loc)[i] = dp_loc_offsets(src[i]);
    if (tid < K * 8) {
      const int k = tid >> 3, kk = reverse ? K - 1 - k : k;
      ((u32x4*)s_w)[tid] = *(const u32x4*)(w + (int64_t)kk * C + 64 * chunk + 8 * (tid & 7));
    }
  }
  __syncthreads();
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  dp_stage_rows(rs_in, (char*)s_rows, s_u, (U + 8) >> 3, (uint32_t)C * 2u, (uint32_t)chunk * 128u, wave, lane);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  float acc[4][8];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[j][e] = 0.f;
  const char* rows_c = (const char*)s_rows;
  const uint16_t* lcw = s_loc + r0;
  const uint32_t cx = (uint32_t)c << 4;
#pragma unroll 3
  for (int k = 0; k < K; ++k) {
    unsigned wlo[4], whi[4];
    dp_split(((const u32x4*)s_w)[k * 8 + c], wlo, whi);
    uint32_t p[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) p[j] = lcw[k * kDpRows + 32 * j];
    u32x4 xv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) xv[j] = *(const u32x4*)(rows_c + (p[j] ^ cx));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[j][2 * e] = dp_dot2<T>(xv[j][e], wlo[e], acc[j][2 * e]);
        acc[j][2 * e + 1] = dp_dot2<T>(xv[j][e], whi[e], acc[j][2 * e + 1]);
      }
    }
  }
  float bv[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) bv[e] = bias ? to_f32(bias[64 * chunk + 8 * c + e]) : 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t row = tile * kDpRows + r0 + 32 * j;
    if (row >= rows_out) continue;
    unsigned pk[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) pk[e] = pack2<T>(acc[j][2 * e] + bv[2 * e], acc[j][2 * e + 1] + bv[2 * e + 1]);
    *(u32x4*)(out + row * C + 64 * chunk + 8 * c) = u32x4{pk[0], pk[1], pk[2], pk[3]};
  }
}

// Weight gradient: a persistent workgroup owns a range of tiles, a 64-channel chunk and KG
// slots; thread mapping as above, sums of its KG x 8 (slot, channel) pairs in registers.
template <typename T, int KG>
__global__ __launch_bounds__(256, 2) void dw_wgrad_planned_kernel(
    const T* __restrict__ x, uint32_t x_bytes, const T* __restrict__ g, const uint16_t* __restrict__ loc,
    const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows, int64_t rows, int K, int C,
    int64_t tiles, int64_t tiles_per_split, int nsplit, int nchunk, float* __restrict__ partial) {
  __shared__ __attribute__((aligned(16))) T s_rows[kDpRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc[KG * kDpRows];
  __shared__ int32_t s_u[2][kDpRowsAlloc];

  const int bid = blockIdx.x;
  const int ngrp = K / KG;
  const int idx = bid >> 3;
  const int sub = idx % (nchunk * ngrp);
  const int chunk = sub % nchunk, k0 = (sub / nchunk) * KG;
  const int split = (bid & 7) * (nsplit >> 3) + idx / (nchunk * ngrp);
  const int64_t t_begin = (int64_t)split * tiles_per_split;
  const int64_t t_end = min(tiles, t_begin + tiles_per_split);
  if (t_begin >= t_end) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = tid & 7, r0 = tid >> 3;

  float acc[KG][8];
#pragma unroll
  for (int k = 0; k < KG; ++k)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[k][e] = 0.f;

  const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, x_bytes);
  const char* rows_c = (const char*)s_rows;
  const uint16_t* lcw = s_loc + r0;
  auto load_list = [&](int64_t tile, int32_t* su) -> int {
    const int32_t p0 = uptr[tile];
    const int U = uptr[tile + 1] - p0;
    for (int i = tid; i < kDpRowsAlloc; i += 256) su[i] = (i >= 1 && i <= U) ? urows[p0 + i - 1] : -1;
    return U;
  };
  int U = load_list(t_begin, s_u[0]);
  int b = 0;
  for (int64_t tile = t_begin; tile < t_end; ++tile, b ^= 1) {
    // every wave is done with the tile before; this tile's list is complete
    __syncthreads();
    dp_stage_rows(rs_x, (char*)s_rows, s_u[b], (U + 8) >> 3, (uint32_t)C * 2u, (uint32_t)chunk * 128u, wave, lane);
    {
      const u32x4* src = (const u32x4*)(loc + (tile * K + k0) * (int64_t)kDpRows);
      for (int i = tid; i < KG * 16; i += 256) ((u32x4*)s_loc)[i] = dp_loc_offsets(src[i]);
    }
    u32x4 gv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t row = tile * kDpRows + r0 + 32 * j;
      gv[j] = row < rows ? *(const u32x4*)(g + row * C + 64 * chunk + 8 * c) : u32x4{0u, 0u, 0u, 0u};
    }
    if (tile + 1 < t_end) U = load_list(tile + 1, s_u[b ^ 1]);       // the next list, under this tile's loads
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    unsigned glo[4][4], ghi[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) dp_split(gv[j], glo[j], ghi[j]);
    const uint32_t cx = (uint32_t)c << 4;
#pragma unroll
    for (int k = 0; k < KG; ++k) {
      uint32_t p[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) p[j] = lcw[k * kDpRows + 32 * j];
      u32x4 xv[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) xv[j] = *(const u32x4*)(rows_c + (p[j] ^ cx));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc[k][2 * e] = dp_dot2<T>(xv[j][e], glo[j][e], acc[k][2 * e]);
          acc[k][2 * e + 1] = dp_dot2<T>(xv[j][e], ghi[j][e], acc[k][2 * e + 1]);
        }
      }
    }
  }

  // ---- the 32 threads of a chunk column, added in thread order ----
  __syncthreads();
  float* s_red = (float*)s_rows;                             // [32 row threads][64 channels]
#pragma unroll
  for (int k = 0; k < KG; ++k) {
#pragma unroll
    for (int e = 0; e < 8; ++e) s_red[r0 * 64 + 8 * c + e] = acc[k][e];
    __syncthreads();
    if (tid < 64) {
      float s = 0.f;
      for (int r = 0; r < 32; ++r) s += s_red[r * 64 + tid];
      partial[((int64_t)split * K + k0 + k) * C + 64 * chunk + tid] = s;
    }
    __syncthreads();
  }
}

}  // namespace ocnn

using namespace ocnn;

static int dp_cu_count() {
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
    n_cu = prop.multiProcessorCount;
  }
  return n_cu;
}

static int dp_kg(int K) { return K == 27 || K == 9 ? 9 : K == 8 ? 8 : K == 3 ? 3 : 0; }

static int dp_splits(int K, int C, int n_cu) {
  const int per = (C / 64) * (K / dp_kg(K));                 // workgroups per tile range
  return std::min(1024, std::max(8, 2 * n_cu / per / 8 * 8));  // a multiple of 8: ranges are dealt to the XCDs
}

extern "C" int ocnn_dwconv_gather_planned_supported(int dtype, int64_t rows_in, int K, int channels,
                                                    int plan_max_distinct) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (channels < 64 || channels % 64 != 0 || channels > 4096) return 0;
  if (K < 1 || K > 27) return 0;
  if (plan_max_distinct > kDpCap) return 0;
  if ((int64_t)rows_in * channels * 2 > 0xfff00000ll) return 0;
  return 1;
}

extern "C" int ocnn_dwconv_gather_planned(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                                          const int32_t* uptr, const int32_t* urows, int plan_max_distinct,
                                          int64_t plan_total, int64_t rows_out, int K, const void* w,
                                          int channels, int reverse_slots, const void* bias, void* out,
                                          void* stream) {
  OCNN_REQUIRE(ocnn_dwconv_gather_planned_supported(dtype, rows_in, K, channels, plan_max_distinct),
               "dwconv_gather_planned: shape not supported");
  OCNN_REQUIRE(rows_out >= 0 && rows_out < (1ll << 31) && plan_total >= 0 && plan_total < (1ll << 29),
               "dwconv_gather_planned: rows out of range");
  if (rows_out == 0) return OCNN_OK;
  hipStream_t st = (hipStream_t)stream;
  const int C = channels, nchunk = C / 64;
  const int64_t tiles = cdiv(rows_out, kDpRows);
  const int64_t per_xcd = cdiv(tiles, 8);
  const dim3 grid((unsigned)(per_xcd * 8 * nchunk));
  const uint32_t in_bytes = (uint32_t)(rows_in * C * 2);
  if (dtype == OCNN_F16)
    hipLaunchKernelGGL(dw_gather_planned_kernel<f16>, grid, dim3(256), 0, st, (const f16*)in, in_bytes, loc, uptr,
                       urows, (const f16*)w, (const f16*)bias, (f16*)out, rows_out, K, C, reverse_slots, tiles,
                       per_xcd, nchunk);
  else
    hipLaunchKernelGGL(dw_gather_planned_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)in, in_bytes, loc,
                       uptr, urows, (const bf16*)w, (const bf16*)bias, (bf16*)out, rows_out, K, C, reverse_slots,
                       tiles, per_xcd, nchunk);
  return check_launch("dwconv_gather_planned");
}

extern "C" int ocnn_dwconv_wgrad_planned_supported(int dtype, int64_t rows_x, int64_t rows, int K,
                                                   int channels, int plan_max_distinct) {
  if (!ocnn_dwconv_gather_planned_supported(dtype, rows_x, K, channels, plan_max_distinct)) return 0;
  if (dp_kg(K) == 0) return 0;
  if ((int64_t)rows * channels * 2 > 0xfff00000ll) return 0;
  return 1;
}

extern "C" int64_t ocnn_dwconv_wgrad_planned_workspace_bytes(int K, int channels) {
  const int n_cu = dp_cu_count();
  if (dp_kg(K) == 0 || channels < 64) return 0;
  const int64_t splits = n_cu > 0 ? dp_splits(K, channels, n_cu) : 1024;
  return align_up(splits * K * channels * 4, 256);
}

template <typename T>
static int run_dp_wgrad(const void* x, int64_t rows_x, const void* g, const uint16_t* loc, const int32_t* uptr,
                        const int32_t* urows, int64_t rows, int K, int C, void* gw, void* ws, int64_t ws_bytes,
                        hipStream_t st) {
  const int n_cu = dp_cu_count();
  if (n_cu <= 0) {
    set_error("dwconv_wgrad_planned: cannot query the device");
    return OCNN_ERR_HIP;
  }
  const int nsplit = dp_splits(K, C, n_cu);
  const int64_t tiles = cdiv(rows, kDpRows);
  const int64_t per = std::max<int64_t>(1, cdiv(tiles, nsplit));
  const int used = (int)cdiv(tiles, per);
  if (ws_bytes < (int64_t)used * K * C * 4) {
    set_error("dwconv_wgrad_planned: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  float* partial = (float*)ws;
  if (rows > 0) {
    const int nchunk = C / 64, kg = dp_kg(K);
    const dim3 grid((unsigned)(nsplit * nchunk * (K / kg)));
    const uint32_t xb = (uint32_t)(rows_x * C * 2);
#define OCNN_DP_WGRAD(KG_)                                                                              \
  hipLaunchKernelGGL((dw_wgrad_planned_kernel<T, KG_>), grid, dim3(256), 0, st, (const T*)x, xb, (const T*)g, \
                     loc, uptr, urows, rows, K, C, tiles, per, nsplit, nchunk, partial)
    if (kg == 9) OCNN_DP_WGRAD(9);
    else if (kg == 8) OCNN_DP_WGRAD(8);
    else OCNN_DP_WGRAD(3);
#undef OCNN_DP_WGRAD
  }
  launch_wgrad_reduce<T>(partial, rows > 0 ? used : 0, K, 1, C, 0, (T*)gw, st);
  return check_launch("dwconv_wgrad_planned");
}

extern "C" int ocnn_dwconv_wgrad_planned(int dtype, const void* x, int64_t rows_x, const void* g,
                                         const uint16_t* loc, const int32_t* uptr, const int32_t* urows,
                                         int plan_max_distinct, int64_t plan_total, int64_t rows, int K,
                                         int channels, void* gw, void* workspace, int64_t workspace_bytes,
                                         void* stream) {
  OCNN_REQUIRE(ocnn_dwconv_wgrad_planned_supported(dtype, rows_x, rows, K, channels, plan_max_distinct),
               "dwconv_wgrad_planned: shape not supported");
  OCNN_REQUIRE(rows >= 0 && rows < (1ll << 31) && plan_total >= 0 && plan_total < (1ll << 29),
               "dwconv_wgrad_planned: rows out of range");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16)
    return run_dp_wgrad<f16>(x, rows_x, g, loc, uptr, urows, rows, K, channels, gw, workspace, workspace_bytes, st);
  return run_dp_wgrad<bf16>(x, rows_x, g, loc, uptr, urows, rows, K, channels, gw, workspace, workspace_bytes, st);
}
