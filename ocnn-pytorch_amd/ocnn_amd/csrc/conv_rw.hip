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
#include <type_traits>

#include "common.hpp"
#include "mma.hpp"

#ifndef OCNN_RW_EXP
#define OCNN_RW_EXP 0   // timing experiments: bit 0 no partial-sum writes, 1 no barriers, 2 no reads/adds, 3 no stores
#endif

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
  __shared__ f32x4 s_red[4 * 4 * 4 * 64];                                  // 64 KiB: [writer][combination][quarter][lane]
  __shared__ __attribute__((aligned(16))) float s_bias[64];
  __shared__ __attribute__((aligned(16))) int32_t s_u[2][kRwCap + 64];     // row lists, 2 tiles ahead

  constexpr int KK = UPW == 14 ? 27 : UPW == 5 ? 9 : UPW == 4 ? 8 : 3;   // slots (= K)
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
  long long t_main = 0, t_stage = 0, t_wait = 0, t_mark = 0;

  // bias as fp32 in LDS (zeros without one); a lane finishes the 16 output channels
  // 32 (wave % 2) + 16 q .. of a row
  if (tid < 64) s_bias[tid] = bias ? to_f32(bias[tid]) : 0.f;
  const f32x4* bias4 = (const f32x4*)(&s_bias[32 * (wave & 1) + 16 * q]);

  // Two accumulator sets: while a 64-row half is being multiplied into one, the partial sums
  // of the half before it (the other set) are exchanged through LDS and stored, a piece per
  // step of the main loop, in the shadow of the MFMAs.
  f32x16 acc[2][2][2];

  // ---- the cross-wave sum of one half, cut into pieces for the steps of a main loop ----
  // Wave w finishes (row tile w / 2, M tile w % 2).  Pieces 0..15 write all four
  // combinations to s_red (also the own one: the code is then the same for every wave and
  // free of branches, which cost a wave far more than an LDS round trip), piece 19 is
  // the barrier after them, 20..23 read the four partial sums of the own combination,
  // 21..24 add them in wave order, 23 and 25 store.
  f32x4 red[4], rb;        // partial sums and bias of a quarter (read at piece j, used at j + 1)
  unsigned pk[4];
  auto exch_piece = [&](auto SETC, int j, int64_t row0, bool drain) {     // row0: first row of that half
    constexpr int S = decltype(SETC)::value;
    if (j < 16) {
      const int c = j >> 2, r4 = j & 3;                       // combination c = 2 nt + tM
      if (!(OCNN_RW_EXP & 1))
        s_red[((wave * 4 + c) * 4 + r4) * 64 + lane] =
            f32x4{acc[S][c >> 1][c & 1][4 * r4], acc[S][c >> 1][c & 1][4 * r4 + 1],
                  acc[S][c >> 1][c & 1][4 * r4 + 2], acc[S][c >> 1][c & 1][4 * r4 + 3]};
    } else if (j == 19) {
      // With 28 steps a wave has by now consumed LDS reads that it issued after its last
      // write, so the writes are done (LDS operations of a wave complete in order); in the
      // shorter loops, and without a main loop around, it waits for them.
      if (OCNN_RW_EXP & 2) {}
      else if (drain) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else asm volatile("s_barrier" ::: "memory");
    } else if (j >= 20 && j <= 25) {
      if (j == 23 || j == 25) {                               // channels 0-7 after quarter 1, 8-15 after 3
        const int64_t row = row0 + 32 * (wave >> 1) + r32;
        if (row < rows_out && !(OCNN_RW_EXP & 8))
          *(u32x4*)(out + row * 64 + 32 * (wave & 1) + 16 * q + (j == 23 ? 0 : 8)) =
              u32x4{pk[0], pk[1], pk[2], pk[3]};
      }
      if (j >= 21 && j <= 24 && !(OCNN_RW_EXP & 4)) {         // add quarter j - 21 in wave order, pack
        const int r4 = j - 21;
        const f32x4 sum = ((red[0] + red[1]) + red[2]) + red[3];
        pk[2 * (r4 & 1)] = pack2<T>(sum[0] + rb[0], sum[1] + rb[1]);
        pk[2 * (r4 & 1) + 1] = pack2<T>(sum[2] + rb[2], sum[3] + rb[3]);
      }
      if (j <= 23 && !(OCNN_RW_EXP & 4)) {                    // read the partial sums of quarter j - 20
        const int r4 = j - 20;
#pragma unroll
        for (int src = 0; src < 4; ++src) red[src] = s_red[((src * 4 + wave) * 4 + r4) * 64 + lane];
        rb = bias4[r4];
      }
    }
  };

  // ---- one 64-row half: main loop into acc[S], exchange of the previous half (acc[1 - S]) ----
  // (prev_row0 past the last row: nothing is stored, as for the first half of a range)
  auto half_body = [&](auto SETC, const uint16_t* lc, int64_t prev_row0) {
    constexpr int S = decltype(SETC)::value;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int tM = 0; tM < 2; ++tM)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[S][nt][tM][r] = 0.f;

    // The main loop is a flat sequence of steps (unit u, row tile nt).  The B operand of
    // a step (lane: row r32 of the row tile, k group q -> 2 x 16 B of its neighbour row)
    // is fetched from LDS three steps ahead of its four MFMAs; the table positions of a
    // unit are read three units ahead.  Units past 2K have zero weights.
    // unit u of wave w is (slot 2u + w / 2, input-channel half w % 2): one base address per
    // half, immediate offsets per unit
    const uint16_t* lcw = lc + (wave >> 1) * kRwRows + 64 * S + r32;
    auto read_loc = [&](int u, uint32_t (&l)[2]) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        uint32_t v = lcw[2 * u * kRwRows + 32 * nt];
        if (4 * u + 3 >= 2 * KK) v = (4 * u + wave < 2 * KK) ? v : 0u;   // a unit past the last slot: zero row
        l[nt] = v;
      }
    };
    // LDS addresses of the two 16-byte pieces a lane reads of its neighbour row
    const uint32_t c0 = (uint32_t)(4 * (wave & 1) + q);
    auto addr = [&](int u, uint32_t l, const T*& p0, const T*& p1) {   // l = 0: empty = the zero row
      (void)u;
      if (OCNN_RW_EXP & 64) {            // timing experiment: one VALU per look-up
        p0 = &s_rows[(l << 3) + c0 * 8];
        p1 = p0 + 16;
        return;
      }
      const uint32_t swz = (l >> 1) & 7;
      p0 = &s_rows[l * 64 + ((c0 ^ swz) * 8)];
      p1 = &s_rows[l * 64 + (((c0 + 2) ^ swz) * 8)];
    };

    constexpr int STEPS = UPW * 2;
    uint32_t lcur[2], lnxt[2] = {0u, 0u};
    u32x4 ring[3][2];
    const T *pa, *pb;
    read_loc(0, lcur);
    if (UPW > 1) read_loc(1, lnxt);
    addr(0, lcur[0], pa, pb);
    ring[0][0] = *(const u32x4*)pa;
    ring[0][1] = *(const u32x4*)pb;
    addr(0, lcur[1], pa, pb);
    ring[1][0] = *(const u32x4*)pa;
    ring[1][1] = *(const u32x4*)pb;
    __builtin_amdgcn_sched_barrier(0);
    // Every step issues its four MFMAs with the LDS traffic of step j + 2 placed between
    // them, so that the address arithmetic and the reads issue while an MFMA executes.
    // The exchange pieces are spread over the steps whatever their number.
    constexpr int EPS = (26 + STEPS - 1) / STEPS;           // exchange pieces per step
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
      const int u = j >> 1, nt = j & 1;
      const bool pre = j + 2 < STEPS;
      const int nt2 = nt;                                    // step j + 2: unit u + 1, same row tile
      acc[S][nt][0] = Mma32<T>::run(wreg[u][0][0], ring[j % 3][0], acc[S][nt][0]);
      if (pre) addr(u + 1, lnxt[nt2], pa, pb);
      acc[S][nt][1] = Mma32<T>::run(wreg[u][0][1], ring[j % 3][0], acc[S][nt][1]);
      if (pre) ring[(j + 2) % 3][0] = *(const u32x4*)pa;
      acc[S][nt][0] = Mma32<T>::run(wreg[u][1][0], ring[j % 3][1], acc[S][nt][0]);
      if (pre) ring[(j + 2) % 3][1] = *(const u32x4*)pb;
      if (nt == 1) {
        // the next unit becomes current; read the positions of the one two units on
        lcur[0] = lnxt[0];
        lcur[1] = lnxt[1];
        if (u + 2 < UPW) read_loc(u + 2, lnxt);
      }
      acc[S][nt][1] = Mma32<T>::run(wreg[u][1][1], ring[j % 3][1], acc[S][nt][1]);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int e = j * EPS; e < (j + 1) * EPS && e < 26; ++e)
        exch_piece(std::integral_constant<int, 1 - S>{}, e, prev_row0, UPW != 14);
      __builtin_amdgcn_sched_barrier(0);
    }
    // s_red may be written again (next half) once every owner has used what it read
    if (!(OCNN_RW_EXP & 2)) asm volatile("s_barrier" ::: "memory");
  };

  for (int64_t tile = t_begin; tile < t_end; ++tile) {
    const int cur = (int)(tile - t_begin) & 1;
    const uint16_t* lc = s_loc[cur];
    // list boundary three tiles ahead (scalar load, used after the main loop)
    const int32_t p_nx3 = uptr[min(tile + 3, tiles)];
    if (timing) t_mark = clock64();
    half_body(std::integral_constant<int, 0>{}, lc, tile > t_begin ? (tile - 1) * kRwRows + 64 : rows_out);
    half_body(std::integral_constant<int, 1>{}, lc, tile * kRwRows);
    if (timing) { long long t = clock64(); t_main += t - t_mark; t_mark = t; }
    // every wave is past its last read of s_rows / s_loc[cur] (the barrier closing the half)
    if (tile + 1 < t_end) {
      stage(tile + 1, p_nx2 - p_nxt, cur ^ 1, cur ^ 1);      // ids came in one tile ago
      if (tile + 2 < t_end) stage_list(p_nx2, cur);          // s_u[cur] was consumed a tile ago
    }
    p_nxt = p_nx2;
    p_nx2 = p_nx3;
    if (timing) { long long t = clock64(); t_stage += t - t_mark; t_mark = t; }
    __builtin_amdgcn_s_waitcnt(0);            // the next tile has landed (own loads)
    __syncthreads();                          // ... everyone's
    if (timing) { long long t = clock64(); t_wait += t - t_mark; t_mark = t; }
  }
  // the last half of the range: its exchange has no main loop to hide under
#pragma unroll
  for (int e = 0; e < 26; ++e) {
    exch_piece(std::integral_constant<int, 1>{}, e, (t_end - 1) * kRwRows + 64, true);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (timing && lane == 0) {
    long long* d = dbg + ((int64_t)blockIdx.x * 4 + wave) * 8;
    d[0] = t_main; d[1] = t_stage; d[2] = t_wait; d[3] = t_end - t_begin;
    d[4] = 0; d[5] = 0; d[6] = 0; d[7] = 0;
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
