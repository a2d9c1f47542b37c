// Gather-GEMM for wide layers (input channels a multiple of 64, output channels a
// multiple of 128) on the tile plan of the neighbour table.
//
// The weights of such a layer (27 x 256 x 256 x 2 B = 3.4 MiB) fit neither registers
// nor LDS, so they stream from L2 straight into registers, already in the layout of
// the MFMA A operand (no LDS round trip, no sharing between waves: the four waves of
// a workgroup split the output channels).  The distinct input rows of a 128-row tile
// are staged in LDS 64 input channels at a time (asynchronous global->LDS loads); every
// wave multiplies ALL 128 rows with its own output channels (v_mfma_f32_32x32x16, M =
// output channels, N = rows), so one 16-byte LDS read per lane feeds 2 MB MFMAs.  Two
// workgroups share a CU: while one waits for its next 64 channels the other computes.
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "mma.hpp"

namespace ocnn {

constexpr int kWdRows = 128;   // rows per tile (the plan's tile size)
constexpr int kWdCap = 416;    // staged rows; plans with a larger tile use another kernel
constexpr int kWdRowsAlloc = (kWdCap + 8) / 8 * 8;   // LDS rows 0..kWdCap in whole 8-row groups
// share of a table's entries that are set up to which the kernel tests for empty (32-row block,
// slot) units: at 32 - 38 % (the non-empty nodes of depths 7 and 6 of a depth-9 octree) a quarter
// to a half of the units are empty and the launches are 3 - 14 % faster, at 41 - 50 % 0 - 7 % slower
constexpr double kWdSkipMaxOccupancy = 0.40;

// (Not in the kernel template: the arguments of the global->LDS load builtin must not be
// type-dependent expressions.)
static __device__ __forceinline__ void wd_dma16(__amdgpu_buffer_rsrc_t rs, char* dst, uint32_t off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)dst, 16, off, 0, 0, 0);
}

// Packed weights: [input-channel chunk cc][slot k][32 output channels cg][k-step s][lane][8].
// v_mfma_f32_32x32x16 A operand: lane l holds A[l % 32][8 * (l / 32) + j];
// D: lane l, register r holds D[8 * (r / 4) + 4 * (l / 32) + r % 4][l % 32].
//   input channel  = 64 cc + 16 s + 8 (lane / 32) + j
//   output channel = 32 cg + perm(lane % 32), perm(8a + 4q + b) = 16 q + 4 a + b,
// so that a lane ends with 16 consecutive output channels per M tile.
// Input channels are padded to whole chunks of 64 with zero weights.
template <typename T>
__global__ void pack_weights_wide_kernel(const T* __restrict__ w, T* __restrict__ out, int K, int cin,
                                         int cout, int transposed, int reverse) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)K * ((cin + 63) & ~63) * cout) return;
  int j = (int)(e & 7);
  int lane = (int)((e >> 3) & 63);
  int s = (int)((e >> 9) & 3);
  int64_t rest = e >> 11;
  const int ncg = cout >> 5;
  int cg = (int)(rest % ncg);
  rest /= ncg;
  int k = (int)(rest % K);
  int cc = (int)(rest / K);
  int q = lane >> 5, m = lane & 31;
  int chan = 64 * cc + 16 * s + 8 * q + j;
  int co = 32 * cg + 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3);
  int kk = reverse ? K - 1 - k : k;
  if (chan >= cin) out[e] = (T)0.f;
  else out[e] = transposed ? w[((int64_t)kk * cout + co) * cin + chan] : w[((int64_t)kk * cin + chan) * cout + co];
}

// One workgroup: one tile of 128 rows x 128 MB output channels (blockIdx.y); wave w owns
// the output channels 32 MB w .. of that block.  Channel counts are multiples of 32: the
// last 64-channel chunk of the input may be half a chunk (its other half is staged as zeros
// and meets zero weights), and waves whose output channels lie past the end idle.
//
// SKIP: per slot and 32-row block of the tile a wave asks whether any row has an entry there (a
// ballot over the positions it reads anyway) and leaves the block's MFMAs out otherwise.  The
// kernel is bound by the power its MFMAs draw (also those on zero rows), and the branches cost
// 2 - 7 % where nothing is empty: it pays from about a quarter of the (block, slot) units empty -
// the non-empty nodes of coarse levels -, which the launch decides from the table's occupancy.
template <typename T, int MB, bool SKIP>
__global__ __launch_bounds__(256, 2) void conv_gather_wide_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const uint16_t* __restrict__ loc,
    const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows, const T* __restrict__ wpk,
    const T* __restrict__ bias, T* __restrict__ out, int64_t rows_out, int K, int cin, int cout,
    int64_t tiles, int64_t tiles_per_xcd) {
  __shared__ __attribute__((aligned(16))) T s_rows[kWdRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc[27 * kWdRows];
  __shared__ int32_t s_u[kWdRowsAlloc];

  const int64_t tile = xcd_tile(blockIdx.x, tiles_per_xcd);
  if (tile >= tiles) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 5, r32 = lane & 31;
  const int ncc = (cin + 63) >> 6;
  const int ncg = cout >> 5;
  const int cg0 = ((int)blockIdx.y * 4 + wave) * MB;        // first 32-channel group of this wave
  const uint32_t pitch = (uint32_t)cin * 2u;

  // ---- the tile's list of distinct rows and its table positions -> LDS ----
  const int32_t p0 = uptr[tile];
  const int U = uptr[tile + 1] - p0;
  for (int i = tid; i < kWdRowsAlloc; i += 256)
    s_u[i] = (i >= 1 && i <= U) ? urows[p0 + i - 1] : -1;  // LDS row p holds list entry p - 1; row 0 = zeros
  {
    const u32x4* src = (const u32x4*)(loc + tile * (int64_t)(kWdRows * K));
    for (int i = tid; i < K * 16; i += 256) ((u32x4*)s_loc)[i] = src[i];
  }
  const int groups = (U + 8) >> 3;                          // 8-row groups of LDS rows 0..U

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  // a lane's 16-byte chunk c of LDS row p lands at chunk c ^ ((p >> 1) & 7) (bank swizzle)
  const uint32_t st_c = (uint32_t)(((lane & 7) ^ (((lane >> 4) + 4 * wave) & 7)) * 16);
  const int st_p = 8 * wave + (lane >> 3);                  // LDS row of piece 0; piece i: + 32 i
  const bool half_oob = (cin & 63) != 0 && st_c >= 64;      // this lane's piece of a half chunk at the end
  constexpr int kRowPieces = (kWdCap + 1 + 31) / 32;

  f32x16 acc[4][MB];
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][mb][r] = 0.f;

  // ---- operands ----
  // A: weights of (chunk, slot) kk = cc K + k, k-step s; one 16-byte load per lane and M tile
  const int64_t kstride = (int64_t)ncg * 2048;               // elements between consecutive kk
  const T* wbase = wpk + lane * 8;
  const int kk_last = ncc * K - 1;
  const bool active = cg0 < ncg;                             // (wave-uniform)
  u32x4 A[4][MB];                                            // ring over the k-steps
  auto load_a = [&](int kk, int s, u32x4 (&a)[MB]) {
    const T* p = wbase + (int64_t)min(kk, kk_last) * kstride + s * 512;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) a[mb] = *(const u32x4*)(p + (int64_t)min(cg0 + mb, ncg - 1) * 2048);
  };
  // B: a lane reads 16 bytes (8 input channels) of the neighbour row of row 32 rb + r32.
  // pv = byte address of the row in s_rows with the swizzle of k-step 0 folded in.
  const char* rows_c = (const char*)s_rows;
  const uint16_t* lcw = s_loc + r32;
  uint32_t pvc[4], pvn[4];
  u32x4 Bb[2][4];
  // (SKIP) which 32-row blocks of the tile have an entry in the slot at all, wave-uniform
  bool nzc[4] = {true, true, true, true}, nzn[4] = {true, true, true, true};
  auto load_pos = [&](int k, uint32_t (&pv)[4], bool (&nz)[4]) {
    const uint16_t* p = lcw + k * kWdRows;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const uint32_t l = p[32 * rb];                         // 0 = empty = the zero row
      pv[rb] = (l << 7) | (((l << 3) & 0x70u) ^ ((uint32_t)q << 4));
      if constexpr (SKIP) nz[rb] = __builtin_amdgcn_ballot_w64(l != 0u) != 0ull;
    }
  };
  auto read_b = [&](const uint32_t (&pv)[4], int s, u32x4 (&b)[4]) {
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) b[rb] = *(const u32x4*)(rows_c + (pv[rb] ^ ((uint32_t)s << 5)));
  };

  // the distinct rows' channels 64 cc .. of the tile -> LDS
  // the list entries of this lane's pieces, read once for all chunks (one LDS wait, not one per piece)
  __syncthreads();
  int32_t ids[kRowPieces];
#pragma unroll
  for (int i = 0; i < kRowPieces; ++i) ids[i] = s_u[min(st_p + 32 * i, kWdRowsAlloc - 1)];   // -1: out of range, loads zeros
  auto stage_chunk = [&](int cc) {
    // every wave is done with the chunk before
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kRowPieces; ++i) {
      const int g = wave + 4 * i;
      if (g < groups) {
        const int32_t id = ids[i];
        uint32_t off = (uint32_t)id * pitch + ((uint32_t)cc * 128u + st_c);
        if (cc == ncc - 1 && half_oob) off = 0xffffff00u;    // past the row's channels: zeros, not the next row
        wd_dma16(rs_in, (char*)s_rows + g * 1024, off);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  const int nfull = cin >> 6;                                // whole 64-channel chunks
  load_a(0, 0, A[0]);
  load_a(0, 1, A[1]);
  for (int cc = 0; cc < nfull; ++cc) {
    stage_chunk(cc);
    load_pos(0, pvc, nzc);
    read_b(pvc, 0, Bb[0]);
    for (int k = 0; k < K; ++k) {
      const int kk = cc * K + k;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        // fetches: positions of the next slot, weights two k-steps ahead, rows one k-step ahead
        if (s == 0) load_pos(k + 1 < K ? k + 1 : 0, pvn, nzn);
        load_a(kk + (s >= 2 ? 1 : 0), (s + 2) & 3, A[(s + 2) & 3]);
        if (s < 3) read_b(pvc, s + 1, Bb[(s + 1) & 1]);
        else read_b(pvn, 0, Bb[0]);                          // (past the last slot: unused)
        if (active) {
#pragma unroll
          for (int rb = 0; rb < 4; ++rb)
            if (!SKIP || nzc[rb]) {
#pragma unroll
              for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = Mma32<T>::run(A[s][mb], Bb[s & 1][rb], acc[rb][mb]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int rb = 0; rb < 4; ++rb) {
        pvc[rb] = pvn[rb];
        if constexpr (SKIP) nzc[rb] = nzn[rb];
      }
    }
  }
  if (nfull < ncc) {
    // Half a chunk at the end (cin % 64 == 32): two k-steps per slot instead of four.  The
    // weights of a slot sit in one pair of the ring while the next slot's go into the other,
    // so the slots are taken two at a time (the chunk before left the first pair filled).
    const int cc = nfull;
    stage_chunk(cc);
    load_pos(0, pvc, nzc);
    read_b(pvc, 0, Bb[0]);
    auto half_slot = [&](int k, auto ring) {
      constexpr int r = decltype(ring)::value;               // this slot's pair of the ring: 0 or 2
      const int kk = cc * K + k;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        if (s == 0) load_pos(k + 1 < K ? k + 1 : 0, pvn, nzn);
        load_a(kk + 1, s, A[(r ^ 2) + s]);
        if (s == 0) read_b(pvc, 1, Bb[1]);
        else read_b(pvn, 0, Bb[0]);                          // (past the last slot: unused)
        if (active) {
#pragma unroll
          for (int rb = 0; rb < 4; ++rb)
            if (!SKIP || nzc[rb]) {
#pragma unroll
              for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = Mma32<T>::run(A[r + s][mb], Bb[s][rb], acc[rb][mb]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int rb = 0; rb < 4; ++rb) {
        pvc[rb] = pvn[rb];
        if constexpr (SKIP) nzc[rb] = nzn[rb];
      }
    };
    for (int k = 0; k < K; k += 2) {
      half_slot(k, std::integral_constant<int, 0>{});
      if (k + 1 < K) half_slot(k + 1, std::integral_constant<int, 2>{});
    }
  }

  // ---- epilogue: a lane holds 16 consecutive output channels of a row per M tile ----
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    if (cg0 + mb >= ncg) continue;
    const int co = 32 * (cg0 + mb) + 16 * q;
    float bv[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) bv[r] = bias ? to_f32(bias[co + r]) : 0.f;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int64_t row = tile * kWdRows + 32 * rb + r32;
      if (row >= rows_out) continue;
      unsigned pk[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) pk[r] = pack2<T>(acc[rb][mb][2 * r] + bv[2 * r], acc[rb][mb][2 * r + 1] + bv[2 * r + 1]);
      T* dst = out + row * cout + co;
      *(u32x4*)(dst) = u32x4{pk[0], pk[1], pk[2], pk[3]};
      *(u32x4*)(dst + 8) = u32x4{pk[4], pk[5], pk[6], pk[7]};
    }
  }
}

// ---------------------------------------------------------------------------------------
// Dense rows (one slot, row i reads row i): out = in W (+ bias), the form a 2x2x2 stride-2
// layer over all nodes takes on the (parents, 8 C) view of its children.  HBM-bound: a
// workgroup brings its 32 RB rows in whole (all input channels, one burst of global->LDS
// loads), then multiplies as above; two workgroups per CU overlap one's loads with the
// other's MFMAs.  Weights: the packed layout above with K = 1.
// ---------------------------------------------------------------------------------------
template <typename T, int RB, int MB>
__global__ __launch_bounds__(256, 2) void conv_dense_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const T* __restrict__ wpk, const T* __restrict__ bias,
    T* __restrict__ out, int64_t rows, int cin, int cout) {
  constexpr int RT = 32 * RB;
  extern __shared__ __attribute__((aligned(16))) char s_dyn[];     // [chunk][RT rows][128 B]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 5, r32 = lane & 31;
  const int ncc = cin >> 6;
  const int cg0 = ((int)blockIdx.y * 4 + wave) * MB;
  const int64_t row0 = (int64_t)blockIdx.x * RT;
  const uint32_t pitch = (uint32_t)cin * 2u;

  // ---- all rows of the tile -> LDS; rows past the end read zeros (out of range) ----
  {
    const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
    const int rl = lane >> 3;                                       // row within a piece of 8
    const int pieces = ncc * (RT / 8);
    for (int i = wave; i < pieces; i += 4) {
      const int cc = i / (RT / 8), g = i - cc * (RT / 8);
      const uint32_t swz = (uint32_t)((4 * g + (lane >> 4)) & 7);
      const uint32_t src = (uint32_t)(row0 + 8 * g + rl) * pitch + (uint32_t)cc * 128u +
                           (((uint32_t)(lane & 7) ^ swz) << 4);
      wd_dma16(rs_in, s_dyn + (cc * RT + 8 * g) * 128, src);
    }
  }

  f32x16 acc[RB][MB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][mb][r] = 0.f;

  // A: weights of k-step t = 4 cc + s, fetched D = R - 1 k-steps ahead into a ring of R (64
  // registers whatever MB): a k-step is only RB MB MFMAs long, an L2 round trip is many of them
  constexpr int R = 16 / MB, D = R - 1;
  const int nsub = 4 * ncc;
  const T* wbase = wpk + (int64_t)cg0 * 2048 + lane * 8;
  const int64_t kstride = (int64_t)(cout >> 5) * 2048;       // elements between consecutive chunks
  u32x4 A[R][MB];
  auto load_a = [&](int t, u32x4 (&a)[MB]) {
    const int tc = min(t, nsub - 1);
    const T* p = wbase + (int64_t)(tc >> 2) * kstride + (tc & 3) * 512;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) a[mb] = *(const u32x4*)(p + mb * 2048);
  };
  uint32_t pvb[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const uint32_t l = (uint32_t)(32 * rb + r32);
    pvb[rb] = (l << 7) | (((l << 3) & 0x70u) ^ ((uint32_t)q << 4));
  }
  u32x4 Bb[2][RB];
  auto read_b = [&](int t, u32x4 (&b)[RB]) {
    const int tc = min(t, nsub - 1);
    const char* base = s_dyn + (tc >> 2) * (RT * 128);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) b[rb] = *(const u32x4*)(base + (pvb[rb] ^ ((uint32_t)(tc & 3) << 5)));
  };

#pragma unroll
  for (int t = 0; t < D; ++t) load_a(t, A[t]);               // (the rows are still in flight)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  read_b(0, Bb[0]);
  for (int t0 = 0; t0 < nsub; t0 += R) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int t = t0 + j;
      if (t < nsub) {
        load_a(t + D, A[(j + D) % R]);
        read_b(t + 1, Bb[(j + 1) & 1]);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = Mma32<T>::run(A[j][mb], Bb[j & 1][rb], acc[rb][mb]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int co = 32 * (cg0 + mb) + 16 * q;
    float bv[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) bv[r] = bias ? to_f32(bias[co + r]) : 0.f;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int64_t row = row0 + 32 * rb + r32;
      if (row >= rows) continue;
      unsigned pk[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) pk[r] = pack2<T>(acc[rb][mb][2 * r] + bv[2 * r], acc[rb][mb][2 * r + 1] + bv[2 * r + 1]);
      T* dst = out + row * cout + co;
      *(u32x4*)(dst) = u32x4{pk[0], pk[1], pk[2], pk[3]};
      *(u32x4*)(dst + 8) = u32x4{pk[4], pk[5], pk[6], pk[7]};
    }
  }
}

}  // namespace ocnn

using namespace ocnn;

extern "C" int ocnn_conv_gather_wide_supported(int dtype, int64_t rows_in, int K, int cin, int cout,
                                               int plan_max_distinct) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (cin < 64 || cin % 32 != 0 || cout < 96 || cout % 32 != 0 || cin > 2048 || cout > 2048) return 0;
  if (K < 1 || K > 27) return 0;
  if (plan_max_distinct < 0 || plan_max_distinct > kWdCap) return 0;
  if (rows_in < 0 || (int64_t)rows_in * cin * 2 > 0xfff00000ll) return 0;
  return 1;
}

template <typename T>
static int run_wide(const void* in, int64_t rows_in, const uint16_t* loc, const int32_t* uptr,
                    const int32_t* urows, int64_t rows_out, int K, int cin, int cout, const void* w,
                    int w_transposed, int reverse, const void* bias, void* out, void* ws, bool skip,
                    hipStream_t st) {
  const int64_t total = (int64_t)K * align_up(cin, 64) * cout;
  hipLaunchKernelGGL(pack_weights_wide_kernel<T>, dim3((unsigned)cdiv(total, 256)), dim3(256), 0, st,
                     (const T*)w, (T*)ws, K, cin, cout, w_transposed, reverse);
  const int64_t tiles = cdiv(rows_out, kWdRows);
  const int64_t per_xcd = cdiv(tiles, 8);
  const uint32_t in_bytes = (uint32_t)(rows_in * cin * 2);
  // 256 output channels per workgroup halve the LDS reads per MFMA; a launch with a handful of tiles
  // (a quarter of the CUs or fewer) is faster with 128 per workgroup on twice as many CUs
  const bool mb2 = cout % 256 == 0 && tiles * (cout / 256) > 64;
  const dim3 grid((unsigned)(per_xcd * 8), (unsigned)(mb2 ? cout / 256 : cdiv(cout, 128)));
#define OCNN_WIDE_LAUNCH(MB_, SKIP_)                                                                          \
  hipLaunchKernelGGL((conv_gather_wide_kernel<T, MB_, SKIP_>), grid, dim3(256), 0, st, (const T*)in, in_bytes, \
                     loc, uptr, urows, (const T*)ws, (const T*)bias, (T*)out, rows_out, K, cin, cout, tiles,   \
                     per_xcd)
  if (mb2) {
    if (skip) OCNN_WIDE_LAUNCH(2, true);
    else OCNN_WIDE_LAUNCH(2, false);
  } else {
    if (skip) OCNN_WIDE_LAUNCH(1, true);
    else OCNN_WIDE_LAUNCH(1, false);
  }
#undef OCNN_WIDE_LAUNCH
  return check_launch("conv_gather_wide");
}

extern "C" int ocnn_conv_gather_wide(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                                     const int32_t* uptr, const int32_t* urows, int plan_max_distinct,
                                     int64_t plan_total, double plan_occupancy, int64_t rows_out, int K,
                                     const void* w, int cin, int cout, int w_transposed, int reverse_slots,
                                     const void* bias, void* out, void* workspace, int64_t workspace_bytes,
                                     void* stream) {
  OCNN_REQUIRE(ocnn_conv_gather_wide_supported(dtype, rows_in, K, cin, cout, plan_max_distinct),
               "conv_gather_wide: shape not supported");
  OCNN_REQUIRE(rows_out >= 0 && rows_out < (1ll << 31) && plan_total >= 0 && plan_total < (1ll << 29),
               "conv_gather_wide: rows out of range");
  if (rows_out == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("conv_gather_wide", loc, uptr, urows, w, out, workspace);
  OCNN_REQUIRE(rows_in == 0 || in, "conv_gather_wide: in is NULL");
  if (workspace_bytes < (int64_t)K * align_up(cin, 64) * cout * 2) {
    set_error("conv_gather_wide: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  // (a 2x2x2 table has an entry in every slot of every 32 rows, whatever its occupancy)
  const bool skip = K != 8 && plan_occupancy >= 0.0 && plan_occupancy <= kWdSkipMaxOccupancy;
  if (dtype == OCNN_F16)
    return run_wide<f16>(in, rows_in, loc, uptr, urows, rows_out, K, cin, cout, w, w_transposed, reverse_slots,
                         bias, out, workspace, skip, st);
  return run_wide<bf16>(in, rows_in, loc, uptr, urows, rows_out, K, cin, cout, w, w_transposed, reverse_slots,
                        bias, out, workspace, skip, st);
}

// ---- dense rows ----
struct DensePlan { int rb, mb; };
static DensePlan dense_plan(int cin, int cout) {
  DensePlan p;
  const int cap = std::max(1, 32768 / cin / 32);             // 32-row blocks whose rows fit 64 KiB of LDS
  if (cout % 512 == 0) { p.mb = 4; p.rb = std::min(2, cap); }
  else if (cout % 256 == 0) { p.mb = 2; p.rb = std::min(4, cap); }
  else { p.mb = 1; p.rb = std::min(4, cap); }
  if (p.rb == 3) p.rb = 2;
  return p;
}

extern "C" int ocnn_conv_dense_supported(int dtype, int64_t rows, int cin, int cout) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (cin < 64 || cin % 64 != 0 || cin > 1024 || cout < 128 || cout % 128 != 0 || cout > 4096) return 0;
  if (rows < 0 || ((int64_t)rows + 128) * cin * 2 > 0xfff00000ll) return 0;
  return 1;
}

template <typename T, int RB, int MB>
static void launch_dense(const void* in, int64_t rows, int cin, int cout, const void* ws, const void* bias,
                         void* out, hipStream_t st) {
  const size_t lds = (size_t)32 * RB * cin * 2;
  static bool attr_set = false;
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)conv_dense_kernel<T, RB, MB>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    attr_set = true;
  }
  hipLaunchKernelGGL((conv_dense_kernel<T, RB, MB>), dim3((unsigned)cdiv(rows, 32 * RB), (unsigned)(cout / (128 * MB))),
                     dim3(256), lds, st, (const T*)in, (uint32_t)(rows * cin * 2), (const T*)ws, (const T*)bias,
                     (T*)out, rows, cin, cout);
}

template <typename T>
static int run_dense(const void* in, int64_t rows, const void* w, int cin, int cout, int w_transposed,
                     const void* bias, void* out, void* ws, hipStream_t st) {
  const int64_t total = (int64_t)cin * cout;
  hipLaunchKernelGGL(pack_weights_wide_kernel<T>, dim3((unsigned)cdiv(total, 256)), dim3(256), 0, st,
                     (const T*)w, (T*)ws, 1, cin, cout, w_transposed, 0);
  const DensePlan p = dense_plan(cin, cout);
#define OCNN_DENSE_CASE(RB_, MB_) \
  if (p.rb == RB_ && p.mb == MB_) { launch_dense<T, RB_, MB_>(in, rows, cin, cout, ws, bias, out, st); return check_launch("conv_dense"); }
  OCNN_DENSE_CASE(4, 1) OCNN_DENSE_CASE(2, 1) OCNN_DENSE_CASE(1, 1)
  OCNN_DENSE_CASE(4, 2) OCNN_DENSE_CASE(2, 2) OCNN_DENSE_CASE(1, 2)
  OCNN_DENSE_CASE(2, 4) OCNN_DENSE_CASE(1, 4)
#undef OCNN_DENSE_CASE
  set_error("conv_dense: no kernel for rb=%d mb=%d", p.rb, p.mb);
  return OCNN_ERR_ARG;
}

extern "C" int ocnn_conv_dense(int dtype, const void* in, int64_t rows, const void* w, int cin, int cout,
                               int w_transposed, const void* bias, void* out, void* workspace,
                               int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(ocnn_conv_dense_supported(dtype, rows, cin, cout), "conv_dense: shape not supported");
  if (rows == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("conv_dense", in, w, out, workspace);
  if (workspace_bytes < (int64_t)cin * cout * 2) {
    set_error("conv_dense: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16) return run_dense<f16>(in, rows, w, cin, cout, w_transposed, bias, out, workspace, st);
  return run_dense<bf16>(in, rows, w, cin, cout, w_transposed, bias, out, workspace, st);
}
