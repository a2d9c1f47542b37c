// Gather-GEMM over a tile plan: every distinct input row a 128-row tile needs is
// brought into LDS exactly once (asynchronous global->LDS loads, full 128-byte
// rows), and all 27 slots then take their operand from LDS.  Rows are in Morton
// order, so a tile re-reads each staged row ~8-10 times: the L2->CU traffic drops
// by that factor compared with gathering per (row, slot).
//
// Workgroup = 4 waves over one tile of 128 output rows x 64 output channels:
// wave (rh, h) owns rows [64 rh, 64 rh + 64) and the input-channel half h of the
// current 64-channel block (split-K inside the workgroup); the two halves are
// summed through LDS at the end.  MFMA M = output channels, N = rows.
#include "common.hpp"
#include "mma.hpp"

#define OCNN_MMA_4X4(a, b)                                                        \
  _Pragma("unroll") for (int n_ = 0; n_ < 4; ++n_)                               \
  _Pragma("unroll") for (int t_ = 0; t_ < 4; ++t_)                               \
      acc[t_][n_] = Mma<T>::run(a[t_], b[n_], acc[t_][n_])

namespace ocnn {

constexpr int kRT = 128;       // rows per tile (must equal the plan's tile size)
constexpr int kUCAP = 320;     // staged rows per pass; tiles needing more take several passes
constexpr int kGroupsPerWave = kUCAP / 8 / 4;

// packed weights: [cout tile of 64][unit = k * (cin/64) + cb][half s][M tile t][lane][8]
// lane (i = lane % 16, g = lane / 16), element j:
//   input channel  = cb*64 + 32 s + 8 g + j
//   output channel = ct*64 + 16 (i / 4) + 4 t + (i % 4)
template <typename T>
__global__ void pack_weights_staged_kernel(const T* __restrict__ w, T* __restrict__ out, int K,
                                           int cin, int cout, int transposed, int reverse) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)K * cin * cout;
  if (e >= total) return;
  const int ncb = cin / 64;
  int j = (int)(e & 7);
  int lane = (int)((e >> 3) & 63);
  int t = (int)((e >> 9) & 3);
  int s = (int)((e >> 11) & 1);
  int64_t r = e >> 12;
  int64_t units = (int64_t)K * ncb;
  int64_t u = r % units;
  int ct = (int)(r / units);
  int k = (int)(u / ncb), cb = (int)(u % ncb);
  int g = lane >> 4, i = lane & 15;
  int chan = cb * 64 + 32 * s + 8 * g + j;
  int co = ct * 64 + (i >> 2) * 16 + 4 * t + (i & 3);
  int kk = reverse ? K - 1 - k : k;
  out[e] = transposed ? w[((int64_t)kk * cout + co) * cin + chan]
                      : w[((int64_t)kk * cin + chan) * cout + co];
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <typename T>
__global__ __launch_bounds__(256) void conv_gather_staged_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const uint16_t* __restrict__ loc,
    const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows,
    const T* __restrict__ wpk, uint32_t wpk_bytes, const T* __restrict__ bias,
    T* __restrict__ out, int64_t rows_out, int K, int cin, int cout, int64_t tiles,
    int64_t tiles_per_xcd) {
  __shared__ __attribute__((aligned(16))) T s_rows[(kUCAP + 1) * 64];
  __shared__ __attribute__((aligned(16))) T s_w[3][4096];
  __shared__ uint16_t s_loc[kRT * 27];

  const int64_t tile = xcd_tile(blockIdx.x, tiles_per_xcd);
  if (tile >= tiles) return;
  const int ct = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rh = wave & 1, h = wave >> 1;
  const int g = lane >> 4, r16 = lane & 15;
  const int64_t row0 = tile * kRT;
  const int ncb = cin >> 6;
  const uint32_t row_bytes = (uint32_t)cin * 2u;

  // table positions of the tile ([slot][row], padded to whole tiles by the plan) -> LDS
  {
    const int64_t base = row0 * K;
    for (int e = tid; e < kRT * K; e += 256) s_loc[e] = loc[base + e];
  }
  if (tid < 8) *(u32x4*)(&s_rows[kUCAP * 64 + tid * 8]) = u32x4{0u, 0u, 0u, 0u};   // the zero row

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(wpk, wpk_bytes);
  const int32_t ub = uptr[tile];
  const int U = uptr[tile + 1] - ub;
  const uint32_t wtile_off = (uint32_t)ct * (uint32_t)K * ncb * 8192u;

  f32x4 acc[4][4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int n = 0; n < 4; ++n) acc[t][n] = f32x4{0.f, 0.f, 0.f, 0.f};

  // each wave moves 2 KiB of the 8 KiB weight unit
  auto load_weights = [&](int unit, int buf) {
    uint32_t src = wtile_off + (uint32_t)unit * 8192u + (uint32_t)(wave * 2) * 1024u + lane * 16u;
    T* dst = &s_w[buf][wave * 1024];
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr_t)dst, 16, src, 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr_t)(dst + 512), 16, src + 1024u, 0, 0, 0);
  };

  const int passes = U > 0 ? (U + kUCAP - 1) / kUCAP : 1;
  for (int pass = 0; pass < passes; ++pass) {
    const int p0 = pass * kUCAP;
    const int nrows = min(kUCAP, U - p0);
    const int ngrp = (nrows + 7) >> 3;
    for (int cb = 0; cb < ncb; ++cb) {
      __syncthreads();                       // everyone is done with the previous staging
      // ---- stage the distinct rows of this pass: 8 rows (1 KiB) per wave instruction ----
      int32_t gr[kGroupsPerWave];
#pragma unroll
      for (int i = 0; i < kGroupsPerWave; ++i) {
        int grp = wave + 4 * i;
        int gu = p0 + grp * 8 + (lane >> 3);
        gr[i] = (grp < ngrp && gu < U) ? urows[ub + gu] : -1;
      }
#pragma unroll
      for (int i = 0; i < kGroupsPerWave; ++i) {
        int grp = wave + 4 * i;
        if (grp < ngrp) {
          int u = grp * 8 + (lane >> 3);
          uint32_t chunk = (uint32_t)((lane & 7) ^ ((u >> 1) & 7));     // bank swizzle
          uint32_t off = gr[i] < 0 ? 0xffffff00u
                                   : (uint32_t)gr[i] * row_bytes + (uint32_t)cb * 128u + chunk * 16u;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_in, (lds_ptr_t)(&s_rows[grp * 8 * 64]), 16, off,
                                                   0, 0, 0);
        }
      }
      load_weights(0 * ncb + cb, 0);
      if (K > 1) load_weights(1 * ncb + cb, 1);
      __builtin_amdgcn_s_waitcnt(0);          // own loads landed
      __syncthreads();                        // everyone's loads landed

      // ---- slots: operands of slot k+1 are fetched from LDS while slot k multiplies ----
      auto fetch = [&](int k, u32x4 (&a)[4], u32x4 (&b)[4]) {
        const T* wsrc = &s_w[k % 3][(h * 4) * 512 + lane * 8];
#pragma unroll
        for (int t = 0; t < 4; ++t) a[t] = *(const u32x4*)(wsrc + t * 512);
#pragma unroll
        for (int n = 0; n < 4; ++n) {
          uint32_t local = (uint32_t)s_loc[k * kRT + 64 * rh + 16 * n + r16] - 1u - (uint32_t)p0;   // 0 = empty
          if (local >= (uint32_t)kUCAP) local = kUCAP;                  // empty or other pass: zero row
          uint32_t pos = (uint32_t)(4 * h + g) ^ ((local >> 1) & 7);
          b[n] = *(const u32x4*)(&s_rows[local * 64 + pos * 8]);
        }
      };
      u32x4 a0[4], b0[4], a1[4], b1[4];
      fetch(0, a0, b0);
      for (int k = 0; k < K; k += 2) {
        if (k + 1 < K) fetch(k + 1, a1, b1);
        if (k + 2 < K) load_weights((k + 2) * ncb + cb, (k + 2) % 3);
        OCNN_MMA_4X4(a0, b0);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (k + 1 < K) {
          if (k + 2 < K) fetch(k + 2, a0, b0);
          if (k + 3 < K) load_weights((k + 3) * ncb + cb, (k + 3) % 3);
          OCNN_MMA_4X4(a1, b1);
          __builtin_amdgcn_s_waitcnt(0);
          __syncthreads();
        }
      }
    }
  }

  // ---- sum the two input-channel halves through LDS; each wave finishes 2 of its 4 row tiles ----
  __syncthreads();
  f32x4* scratch = (f32x4*)s_rows;            // [wave][2][4][64] f32x4 = 32 KiB
  {
    // row tiles handed to the partner wave: 2,3 from half 0; 0,1 from half 1
    // (static register indices: a runtime index would push acc to scratch memory)
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        scratch[((wave * 2 + n2) * 4 + t) * 64 + lane] = h == 0 ? acc[t][2 + n2] : acc[t][n2];
  }
  __syncthreads();
  const int keep = h == 0 ? 0 : 2;
  const int partner = wave ^ 2;
  const int co0 = ct * 64 + g * 16;
  float bv[16];
#pragma unroll
  for (int c = 0; c < 16; ++c) bv[c] = bias ? to_f32(bias[co0 + c]) : 0.f;
#pragma unroll
  for (int n2 = 0; n2 < 2; ++n2) {
    const int n = keep + n2;
    int64_t row = row0 + 64 * rh + 16 * n + r16;
    unsigned pk[8];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      f32x4 o = scratch[((partner * 2 + n2) * 4 + t) * 64 + lane];
      f32x4 v = h == 0 ? acc[t][n2] : acc[t][2 + n2];
      pk[2 * t + 0] = pack2<T>(v[0] + o[0] + bv[4 * t + 0], v[1] + o[1] + bv[4 * t + 1]);
      pk[2 * t + 1] = pack2<T>(v[2] + o[2] + bv[4 * t + 2], v[3] + o[3] + bv[4 * t + 3]);
    }
    if (row < rows_out) {
      T* dst = out + row * cout + co0;
      *(u32x4*)(dst) = u32x4{pk[0], pk[1], pk[2], pk[3]};
      *(u32x4*)(dst + 8) = u32x4{pk[4], pk[5], pk[6], pk[7]};
    }
  }
}

}  // namespace ocnn

using namespace ocnn;

extern "C" int ocnn_conv_gather_planned_supported(int dtype, int64_t rows_in, int cin, int cout) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (cin <= 0 || cout <= 0 || cin % 64 != 0 || cout % 64 != 0) return 0;
  if (rows_in < 0 || (int64_t)rows_in * cin * 2 > 0xfff00000ll) return 0;       // 32-bit buffer offsets
  return 1;
}

template <typename T>
static int run_planned(const void* in, int64_t rows_in, const uint16_t* loc, const int32_t* uptr,
                       const int32_t* urows, int64_t rows_out, int K, const void* w, int cin,
                       int cout, int w_transposed, int reverse, const void* bias, void* out,
                       void* ws, hipStream_t st) {
  int64_t total = (int64_t)K * cin * cout;
  hipLaunchKernelGGL(pack_weights_staged_kernel<T>, dim3(cdiv(total, 256)), dim3(256), 0, st,
                     (const T*)w, (T*)ws, K, cin, cout, w_transposed, reverse);
  int64_t tiles = cdiv(rows_out, kRT);
  int64_t per_xcd = cdiv(tiles, 8);
  dim3 grid((unsigned)(per_xcd * 8), (unsigned)(cout / 64));
  hipLaunchKernelGGL(conv_gather_staged_kernel<T>, grid, dim3(256), 0, st, (const T*)in,
                     (uint32_t)(rows_in * cin * 2), loc, uptr, urows, (const T*)ws,
                     (uint32_t)(total * 2), (const T*)bias, (T*)out, rows_out, K, cin, cout, tiles,
                     per_xcd);
  return check_launch("conv_gather_planned");
}

extern "C" int ocnn_conv_gather_planned(int dtype, const void* in, int64_t rows_in,
                                        const uint16_t* loc, const int32_t* uptr,
                                        const int32_t* urows, int64_t rows_out, int K,
                                        const void* w, int cin, int cout, int w_transposed,
                                        int reverse_slots, const void* bias, void* out,
                                        void* workspace, int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(ocnn_conv_gather_planned_supported(dtype, rows_in, cin, cout),
               "conv_gather_planned: dtype %d cin %d cout %d rows_in %lld not supported", dtype,
               cin, cout, (long long)rows_in);
  OCNN_REQUIRE(K >= 1 && K <= 27 && rows_out >= 0 && rows_out < (1ll << 31),
               "conv_gather_planned: bad shape");
  if (rows_out == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("conv_gather_planned", loc, uptr, urows, w, out, workspace);
  OCNN_REQUIRE(rows_in == 0 || in, "conv_gather_planned: in is NULL");
  if (workspace_bytes < (int64_t)K * cin * cout * 2) {
    set_error("conv_gather_planned: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16)
    return run_planned<f16>(in, rows_in, loc, uptr, urows, rows_out, K, w, cin, cout,
                            w_transposed, reverse_slots, bias, out, workspace, st);
  return run_planned<bf16>(in, rows_in, loc, uptr, urows, rows_out, K, w, cin, cout, w_transposed,
                           reverse_slots, bias, out, workspace, st);
}
