// Gather-GEMM for 64 -> 64 channels with the weights resident in registers.
//
// The weights of a 3x3x3 layer (27 x 64 x 64 x 2 B = 216 KiB) are 7.5 times larger
// than the distinct input rows a 128-row tile touches, so streaming them per
// tile makes the kernel L2-bound.  Here one persistent workgroup per CU (4 waves,
// one per SIMD) loads them ONCE: wave w keeps the A-operand fragments of the
// (slot, input-channel half) units u*4 + w, u = 0..UPW-1 in VGPRs (14 units =
// 224 VGPRs for K = 27).  Per tile the distinct rows are staged in LDS through
// the tile plan (asynchronous global->LDS loads, issued while the previous tile
// is being reduced), every wave multiplies ALL 128 rows of the tile with its own
// units (v_mfma_f32_32x32x16, M = 64 output channels, N = 128 rows), and the four
// partial sums are added through LDS in wave order (deterministic).
#include <algorithm>

#include "common.hpp"
#include "mma.hpp"

namespace ocnn {

constexpr int kRwRows = 128;   // rows per tile (the plan's tile size)
constexpr int kRwCap = 512;    // staged rows; plans with a larger tile use another kernel

// Packed weights: [gid = 2 * slot + half][k-step s][M tile tM][lane][8].
// v_mfma_f32_32x32x16 A operand: lane l holds A[l % 32][8 * (l / 32) + j];
// D: lane l, register r holds D[8 * (r / 4) + 4 * (l / 32) + r % 4][l % 32].
//   input channel  = 32 half + 16 s + 8 (lane / 32) + j
//   output channel = 32 tM + perm(lane % 32), perm(8a + 4q + b) = 16 q + 4 a + b,
// so that a lane ends with 16 consecutive output channels per M tile.
template <typename T>
__global__ void pack_weights_rw_kernel(const T* __restrict__ w, T* __restrict__ out, int K,
                                       int transposed, int reverse) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)K * 4096) return;
  int j = (int)(e & 7);
  int lane = (int)((e >> 3) & 63);
  int tM = (int)((e >> 9) & 1);
  int s = (int)((e >> 10) & 1);
  int gid = (int)(e >> 11);
  int k = gid >> 1, half = gid & 1;
  int q = lane >> 5, m = lane & 31;
  int chan = 32 * half + 16 * s + 8 * q + j;
  int co = 32 * tM + 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3);
  int kk = reverse ? K - 1 - k : k;
  out[e] = transposed ? w[((int64_t)kk * 64 + co) * 64 + chan] : w[((int64_t)kk * 64 + chan) * 64 + co];
}

template <typename T, int UPW>
__global__ __launch_bounds__(256, 1) void conv_gather_rw_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const uint16_t* __restrict__ loc,
    uint32_t loc_bytes, const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows,
    uint32_t urows_bytes, const T* __restrict__ wpk, const T* __restrict__ bias,
    T* __restrict__ out, int64_t rows_out, int K, int64_t tiles, int64_t tiles_per_wg,
    long long* dbg) {
  __shared__ __attribute__((aligned(16))) T s_rows[(kRwCap + 1) * 64];
  // table positions, double buffered; filled 1 KiB per wave instruction, hence the rounding
  __shared__ __attribute__((aligned(16))) uint16_t s_loc[2][(kRwRows * 27 * 2 + 1023) / 1024 * 512];
  __shared__ f32x4 s_red[4 * 3 * 4 * 64];                                  // 48 KiB
  __shared__ __attribute__((aligned(16))) int32_t s_u[2][kRwCap + 64];     // row lists, 2 tiles ahead

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // wave-uniform: lives in an SGPR
  const int q = lane >> 5, r32 = lane & 31;
  const int64_t t_begin = (int64_t)blockIdx.x * tiles_per_wg;
  const int64_t t_end = min(tiles, t_begin + tiles_per_wg);
  if (t_begin >= t_end) return;

  // ---- this wave's weights -> registers, once ----
  u32x4 wreg[UPW][2][2];
#pragma unroll
  for (int u = 0; u < UPW; ++u) {
    int gid = u * 4 + wave;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int tM = 0; tM < 2; ++tM) {
        u32x4 v = u32x4{0u, 0u, 0u, 0u};
        if (gid < 2 * K) v = *(const u32x4*)(wpk + ((int64_t)((gid * 2 + s) * 2 + tM) * 64 + lane) * 8);
        wreg[u][s][tM] = v;
      }
  }

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t rs_loc = make_rsrc(loc, loc_bytes);
  const __amdgpu_buffer_rsrc_t rs_u = make_rsrc(urows, urows_bytes);

  // asynchronous load of a tile's list of distinct rows (first entry `first`) -> s_u[buf]
  auto stage_list = [&](int32_t first, int buf) {
    if (wave < 2)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_u, (lds_ptr_t)(&s_u[buf][wave * 256]), 16,
                                               (uint32_t)first * 4u + (uint32_t)wave * 1024u + lane * 16u,
                                               0, 0, 0);
  };
  // asynchronous staging of one tile: its U distinct rows (ids in s_u[ubuf]) -> s_rows, its
  // table positions -> s_loc[buf]
  auto stage = [&](int64_t tile, int U, int ubuf, int buf) {
    // LDS row p (p >= 1) holds the (p - 1)-th distinct row; row 0 is the zero row that the
    // empty table entries (position 0) read: its lanes load from an out-of-range offset
    const int ngrp = (U + 8) >> 3;
    // four groups of 8 rows per round: the four row ids are read first, then the loads go out
    for (int g0 = wave; g0 < ngrp; g0 += 16) {
      int32_t g[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int u = (g0 + 4 * i) * 8 + (lane >> 3);
        g[i] = (u >= 1 && u <= U) ? s_u[ubuf][u - 1] : -1;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int grp = g0 + 4 * i;
        if (grp < ngrp) {
          int u = grp * 8 + (lane >> 3);
          uint32_t chunk = (uint32_t)((lane & 7) ^ ((u >> 1) & 7));      // bank swizzle
          uint32_t off = g[i] < 0 ? 0xffffff00u : (uint32_t)g[i] * 128u + chunk * 16u;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_in, (lds_ptr_t)(&s_rows[grp * 8 * 64]), 16, off, 0,
                                                   0, 0);
        }
      }
    }
    // kRwRows * K positions (2 B each, [slot][row]), 1 KiB per wave instruction
    const uint32_t lbase = (uint32_t)(tile * kRwRows * K * 2);
    const int nchunk = (kRwRows * K * 2 + 1023) >> 10;
    for (int c = wave; c < nchunk; c += 4)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_loc, (lds_ptr_t)(&s_loc[buf][c * 512]), 16,
                                               lbase + (uint32_t)c * 1024u + lane * 16u, 0, 0, 0);
  };

  // prologue: list of the first tile, then its rows and the list of the second tile
  int32_t p_nxt = uptr[t_begin + 1];
  int32_t p_nx2 = uptr[min(t_begin + 2, tiles)];
  {
    int32_t p_cur = uptr[t_begin];
    stage_list(p_cur, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    stage(t_begin, p_nxt - p_cur, 0, 0);
    stage_list(p_nxt, 1);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
  }

#ifdef OCNN_RW_TIMING
  const bool timing = dbg != nullptr;
#else
  constexpr bool timing = false;
#endif
  long long t_main = 0, t_epi = 0, t_wait = 0, t_mark = 0, t_e0 = 0, t_e1 = 0, t_e2 = 0, t_e3 = 0;
  for (int64_t tile = t_begin; tile < t_end; ++tile) {
    const int cur = (int)(tile - t_begin) & 1;
    const uint16_t* lc = s_loc[cur];
    // list boundary three tiles ahead (scalar load, used after the main loop)
    const int32_t p_nx3 = uptr[min(tile + 3, tiles)];

    // the tile is processed as two halves of 64 rows, so that the accumulators take 64
    // registers and the weights have room next to them
    for (int half_t = 0; half_t < 2; ++half_t) {
      if (timing) t_mark = clock64();
      f32x16 acc[2][2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int tM = 0; tM < 2; ++tM)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[nt][tM][r] = 0.f;

      // The main loop is a flat sequence of steps (unit u, row tile nt).  The B operand of
      // a step (lane: row r32 of the row tile, k group q -> 2 x 16 B of its neighbour row)
      // is fetched from LDS three steps ahead of its four MFMAs; the table positions of a
      // unit are read three units ahead.  Units past 2K have zero weights.
      const int rbase = 64 * half_t + r32;
      auto read_loc = [&](int u, uint32_t (&l)[2]) {
        int gid = min(u * 4 + wave, 2 * K - 1);
        int k = gid >> 1;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) l[nt] = lc[k * kRwRows + rbase + 32 * nt];
      };
      // LDS addresses of the two 16-byte pieces a lane reads of its neighbour row
      auto addr = [&](int u, uint32_t lv, const T*& p0, const T*& p1) {
        int gid = min(u * 4 + wave, 2 * K - 1);
        int half = gid & 1;
        const uint32_t l = lv;                                            // 0 = empty = the zero row
        uint32_t swz = (l >> 1) & 7;
        p0 = &s_rows[l * 64 + (((uint32_t)(4 * half + q) ^ swz) * 8)];
        p1 = &s_rows[l * 64 + (((uint32_t)(4 * half + 2 + q) ^ swz) * 8)];
      };

      constexpr int STEPS = UPW * 2;
      uint32_t lcur[2], lnxt[2], lnx2[2] = {0u, 0u};
      u32x4 ring[4][2];
      const T *pa, *pb;
      read_loc(0, lcur);
      if (UPW > 1) read_loc(1, lnxt);
      if (UPW > 2) read_loc(2, lnx2);
      addr(0, lcur[0], pa, pb);
      ring[0][0] = *(const u32x4*)pa;
      ring[0][1] = *(const u32x4*)pb;
      addr(0, lcur[1], pa, pb);
      ring[1][0] = *(const u32x4*)pa;
      ring[1][1] = *(const u32x4*)pb;
      if (UPW > 1) {
        addr(1, lnxt[0], pa, pb);
        ring[2][0] = *(const u32x4*)pa;
        ring[2][1] = *(const u32x4*)pb;
      }
      __builtin_amdgcn_sched_barrier(0);
      // Every step issues its four MFMAs with the LDS traffic of step j + 3 placed between
      // them, so that the address arithmetic and the reads issue while an MFMA executes.
#pragma unroll
      for (int j = 0; j < STEPS; ++j) {
        const int u = j >> 1, nt = j & 1;
        const bool pre = j + 3 < STEPS;
        const int u3 = (j + 3) >> 1, nt3 = (j + 3) & 1;
        acc[nt][0] = Mma32<T>::run(wreg[u][0][0], ring[j & 3][0], acc[nt][0]);
        if (pre) addr(u3, u3 == u + 1 ? lnxt[nt3] : lnx2[nt3], pa, pb);
        acc[nt][1] = Mma32<T>::run(wreg[u][0][1], ring[j & 3][0], acc[nt][1]);
        if (pre) ring[(j + 3) & 3][0] = *(const u32x4*)pa;
        acc[nt][0] = Mma32<T>::run(wreg[u][1][0], ring[j & 3][1], acc[nt][0]);
        if (pre) ring[(j + 3) & 3][1] = *(const u32x4*)pb;
        if (nt == 1) {
          // the next unit becomes current; read the positions of the one three units on
          lcur[0] = lnxt[0];
          lcur[1] = lnxt[1];
          lnxt[0] = lnx2[0];
          lnxt[1] = lnx2[1];
          if (u + 3 < UPW) read_loc(u + 3, lnx2);
        }
        acc[nt][1] = Mma32<T>::run(wreg[u][1][1], ring[j & 3][1], acc[nt][1]);
        // 1 MFMA, then some VALU / LDS work in its shadow, four times
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (timing) { long long t = clock64(); t_main += t - t_mark; t_mark = t; }

      // ---- cross-wave sum: wave w finishes (row tile w / 2, M tile w % 2) of this half ----
      __syncthreads();           // s_red is free; after the second half also s_rows / s_loc[cur]
      long long tq = 0;
      if (timing) { tq = clock64(); t_e0 += tq - t_mark; }
      if (half_t == 1) {
        if (tile + 1 < t_end) {
          stage(tile + 1, p_nx2 - p_nxt, cur ^ 1, cur ^ 1);      // ids came in one tile ago
          if (tile + 2 < t_end) stage_list(p_nx2, cur);          // s_u[cur] was consumed a tile ago
        }
        p_nxt = p_nx2;
        p_nx2 = p_nx3;
      }
      if (timing) { long long t = clock64(); t_e1 += t - tq; tq = t; }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int tM = 0; tM < 2; ++tM) {
          const int owner = nt * 2 + tM;
          if (owner != wave) {
            const int d3 = owner < wave ? owner : owner - 1;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4)
              s_red[((wave * 3 + d3) * 4 + r4) * 64 + lane] =
                  f32x4{acc[nt][tM][4 * r4], acc[nt][tM][4 * r4 + 1], acc[nt][tM][4 * r4 + 2],
                        acc[nt][tM][4 * r4 + 3]};
          }
        }
      if (timing) { long long t = clock64(); t_e2 += t - tq; tq = t; }
      __syncthreads();
      if (timing) { long long t = clock64(); t_e3 += t - tq; tq = t; }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int tM = 0; tM < 2; ++tM) {
          const int owner = nt * 2 + tM;
          if (owner == wave) {
            const int64_t row = tile * kRwRows + 64 * half_t + 32 * nt + r32;
            const int co0 = 32 * tM + 16 * q;
            unsigned pk[8];
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
              f32x4 sum = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
              for (int src = 0; src < 4; ++src) {          // wave order: deterministic
                f32x4 v;
                if (src == owner) {
                  v = f32x4{acc[nt][tM][4 * r4], acc[nt][tM][4 * r4 + 1], acc[nt][tM][4 * r4 + 2],
                            acc[nt][tM][4 * r4 + 3]};
                } else {
                  const int d3 = owner < src ? owner : owner - 1;
                  v = s_red[((src * 3 + d3) * 4 + r4) * 64 + lane];
                }
                sum = src == 0 ? v : sum + v;
              }
              float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
              if (bias) {
                b0 = to_f32(bias[co0 + 4 * r4]);
                b1 = to_f32(bias[co0 + 4 * r4 + 1]);
                b2 = to_f32(bias[co0 + 4 * r4 + 2]);
                b3 = to_f32(bias[co0 + 4 * r4 + 3]);
              }
              pk[2 * r4] = pack2<T>(sum[0] + b0, sum[1] + b1);
              pk[2 * r4 + 1] = pack2<T>(sum[2] + b2, sum[3] + b3);
            }
            if (row < rows_out) {
              T* dst = out + row * 64 + co0;
              *(u32x4*)(dst) = u32x4{pk[0], pk[1], pk[2], pk[3]};
              *(u32x4*)(dst + 8) = u32x4{pk[4], pk[5], pk[6], pk[7]};
            }
          }
        }
      if (timing) { long long t = clock64(); t_epi += t - t_mark; t_mark = t; }
    }
    __builtin_amdgcn_s_waitcnt(0);            // the next tile has landed (own loads)
    __syncthreads();                          // ... everyone's
    if (timing) { long long t = clock64(); t_wait += t - t_mark; t_mark = t; }
  }
  if (timing && lane == 0) {
    long long* d = dbg + ((int64_t)blockIdx.x * 4 + wave) * 8;
    d[0] = t_main; d[1] = t_epi; d[2] = t_wait; d[3] = t_end - t_begin;
    d[4] = t_e0; d[5] = t_e1; d[6] = t_e2; d[7] = t_e3;
  }
}

}  // namespace ocnn

using namespace ocnn;

static long long* g_rw_dbg = nullptr;

#ifdef OCNN_RW_TIMING
// per-wave cycle counters of the kernel phases (development aid)
extern "C" void ocnn_debug_set_rw_timing(long long* p) { g_rw_dbg = p; }
#endif

extern "C" int ocnn_conv_gather_rw_supported(int dtype, int64_t rows_in, int K, int cin, int cout,
                                             int plan_max_distinct) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (cin != 64 || cout != 64) return 0;
  if (K != 27 && K != 9 && K != 8 && K != 3) return 0;
  if (plan_max_distinct > kRwCap) return 0;
  if ((int64_t)rows_in * 128 > 0xfff00000ll) return 0;
  return 1;
}

template <typename T, int UPW>
static void launch_rw(const void* in, int64_t rows_in, const uint16_t* loc, const int32_t* uptr,
                      const int32_t* urows, uint32_t urows_bytes, int64_t rows_out, int K, const void* ws,
                      const void* bias, void* out, int n_cu, hipStream_t st) {
  int64_t tiles = cdiv(rows_out, kRwRows);
  int64_t wgs = std::min<int64_t>(tiles, n_cu);
  int64_t per = cdiv(tiles, wgs);
  wgs = cdiv(tiles, per);
  hipLaunchKernelGGL((conv_gather_rw_kernel<T, UPW>), dim3((unsigned)wgs), dim3(256), 0, st,
                     (const T*)in, (uint32_t)(rows_in * 128), loc, (uint32_t)(tiles * kRwRows * K * 2), uptr,
                     urows, urows_bytes, (const T*)ws, (const T*)bias, (T*)out, rows_out, K, tiles, per, g_rw_dbg);
}

template <typename T>
static int run_rw(const void* in, int64_t rows_in, const uint16_t* loc, const int32_t* uptr,
                  const int32_t* urows, int64_t plan_total, int64_t rows_out, int K, const void* w, int w_transposed,
                  int reverse, const void* bias, void* out, void* ws, hipStream_t st) {
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
      set_error("conv_gather_rw: cannot query the device");
      return OCNN_ERR_HIP;
    }
    n_cu = prop.multiProcessorCount;
  }
  const uint32_t ub = (uint32_t)(plan_total * 4);
  hipLaunchKernelGGL(pack_weights_rw_kernel<T>, dim3(cdiv((int64_t)K * 4096, 256)), dim3(256), 0, st,
                     (const T*)w, (T*)ws, K, w_transposed, reverse);
  if (K == 27) launch_rw<T, 14>(in, rows_in, loc, uptr, urows, ub, rows_out, K, ws, bias, out, n_cu, st);
  else if (K == 9) launch_rw<T, 5>(in, rows_in, loc, uptr, urows, ub, rows_out, K, ws, bias, out, n_cu, st);
  else if (K == 8) launch_rw<T, 4>(in, rows_in, loc, uptr, urows, ub, rows_out, K, ws, bias, out, n_cu, st);
  else launch_rw<T, 2>(in, rows_in, loc, uptr, urows, ub, rows_out, K, ws, bias, out, n_cu, st);
  return check_launch("conv_gather_rw");
}

extern "C" int ocnn_conv_gather_rw(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                                   const int32_t* uptr, const int32_t* urows,
                                   int plan_max_distinct, int64_t plan_total, int64_t rows_out, int K, const void* w,
                                   int cin, int cout, int w_transposed, int reverse_slots,
                                   const void* bias, void* out, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(ocnn_conv_gather_rw_supported(dtype, rows_in, K, cin, cout, plan_max_distinct),
               "conv_gather_rw: shape not supported");
  OCNN_REQUIRE(rows_out >= 0 && rows_out < (1ll << 31) && (int64_t)rows_out * K * 2 < 0xfff00000ll &&
                   plan_total >= 0 && plan_total < (1ll << 29),
               "conv_gather_rw: rows out of range");
  if (rows_out == 0) return OCNN_OK;
  if (workspace_bytes < (int64_t)K * 8192) {
    set_error("conv_gather_rw: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16)
    return run_rw<f16>(in, rows_in, loc, uptr, urows, plan_total, rows_out, K, w, w_transposed, reverse_slots,
                       bias, out, workspace, st);
  return run_rw<bf16>(in, rows_in, loc, uptr, urows, plan_total, rows_out, K, w, w_transposed, reverse_slots, bias,
                      out, workspace, st);
}
