// Depth-wise convolution and its weight gradient on the tile plan of the neighbour table.
//
//   out[i][c]  = sum_k x[T[i][k]][c] * w[k][c]
//   gw[k][c]   = sum_i x[T[i][k]][c] * g[i][c]
//
// Reading the 27 neighbour rows of every row from L2 makes the plan-free kernels L2-bound
// (27 x the algorithmic bytes).  Here a workgroup stages the distinct rows of a 128-row
// tile, 64 channels of them, ONCE in LDS (asynchronous global->LDS loads) and every
// neighbour read is an LDS read.  The products run on the 4x4x4 matrix instruction (a
// depth-wise product is a 4x4 block with a diagonal operand), four times the vector unit's
// rate, which leaves the kernels bound by LDS reads and by how many bytes a CU keeps in flight.
// One workgroup of eight waves per CU walks a range of tiles: the rows of the next tile are in
// flight while a tile is multiplied (a third row buffer, which would keep two tiles in flight
// and is what the measured time per tile asks for, does not fit the 160 KB of LDS at 416 staged
// rows).  fp32 accumulation; the weight gradient keeps the sums of all slots in registers over
// its range of tiles, adds lanes and waves in a fixed order and leaves per-range sums to the
// split reduction (no atomics).  Slot counts 27, 9, 8 and 3 (the kernel shapes the layers use).
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "mma.hpp"
#include "reduce.hpp"

namespace ocnn {

constexpr int kDpRows = 128;   // rows per tile (the plan's tile size)
constexpr int kDpCap = 416;    // staged rows; plans with a larger tile use another kernel
constexpr int kDpRowsAlloc = (kDpCap + 8) / 8 * 8;
constexpr int kDpThreads = 512;   // eight waves a workgroup, two a SIMD: one computes while the other waits
constexpr int kDpWaves = kDpThreads / 64;
constexpr int kDpListAlloc = 448;   // entries of a list array in LDS (read in whole pieces of 8 rows a wave)

// (Not in the kernel templates: the arguments of the global->LDS load builtin must not be
// type-dependent expressions.)
static __device__ __forceinline__ void dp_dma16(__amdgpu_buffer_rsrc_t rs, char* dst, uint32_t off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)dst, 16, off, 0, 0, 0);
}

// v_mfma_f32_4x4x4_16b_{f16,bf16}: 16 independent 4x4 products D_b = A_b B_b + C_b.  Lane l = 4 b + i
// holds A_b[i][0..3] and B_b[0..3][i] in its two operand registers (four 16-bit values each) and
// D_b[0..3][i] in its four result registers.  8 cycles an instruction: a depth-wise product costs
// 1/32 of a cycle here against 1/8 on the vector unit (v_dot2c_f32 issues every 8 cycles), with
// three quarters of the multipliers fed zeros.
template <typename T> struct Mma4;
template <> struct Mma4<bf16> {
  static __device__ __forceinline__ f32x4 run(u32x2 a, u32x2 b, f32x4 c) {
    typedef __attribute__((ext_vector_type(4))) short s4;
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s4, a), __builtin_bit_cast(s4, b), c, 0, 0, 0);
  }
};
template <> struct Mma4<f16> {
  static __device__ __forceinline__ f32x4 run(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
};

// Bank swizzle of the staged rows: the 16-byte chunk c of LDS row p sits at chunk c ^ s(p),
// s(p) = (bit 1, bit 2, bit 3 of p) as its bits 2, 1, 0.  The neighbours of 4 (8) consecutive rows
// of a tile mostly sit at 4 (8) consecutive positions; with the row's parity, which picks the half
// of the 64 banks, bits 1 and 2 of p then give every row of such a group banks of its own, for the
// gather's 16-byte reads (16 lanes: 4 rows x 4 chunks) and for the weight gradient's 8-byte
// transposing reads (32 lanes: 8 rows x 32 bytes) alike (1.2 - 1.35 instead of 1.9 - 2.9 LDS
// cycles per access measured against the plain (p >> 1) % 8).
// Table positions (16 bits each, two per dword, at most 511) -> byte offsets of the LDS rows with
// the swizzle bits in place; a thread's chunk c of that row is then at offset ^ (c << 4).
// Position 0 (empty entry) stays 0: the zero row.
static __device__ __forceinline__ u32x4 dp_loc_offsets(u32x4 v) {
#pragma unroll
  for (int e = 0; e < 4; ++e)
    v[e] = (v[e] << 7) | ((v[e] & 0x00020002u) << 5) | ((v[e] & 0x00040004u) << 3) | ((v[e] & 0x00080008u) << 1);
  return v;
}

// Stages the 64-channel chunk `chunk` of the rows in the list s_u (LDS row p = list entry
// p - 1, row 0 and everything past the list = zeros) into s_rows, chunks swizzled as above.
static __device__ __forceinline__ void dp_stage_rows(__amdgpu_buffer_rsrc_t rs, char* s_rows, const int32_t* s_u,
                                                     int groups, uint32_t pitch, uint32_t coff, int wave, int lane) {
  // LDS row p = 8 (wave + 8 i) + lane / 8: bits 1, 2 of p are those of lane / 8, bit 3 that of the wave
  const int st_r = lane >> 3;
  const uint32_t st_c = (uint32_t)(((lane & 7) ^ (((st_r & 2) << 1) | ((st_r & 4) >> 1) | (wave & 1))) * 16);
  const int st_p = 8 * wave + st_r;
  constexpr int kRowPieces = (kDpCap + 1 + 8 * kDpWaves - 1) / (8 * kDpWaves);
  static_assert(8 * kDpWaves * kRowPieces <= kDpListAlloc, "the list array covers every piece");
  int32_t id[kRowPieces];                                    // all list entries first: one LDS wait
#pragma unroll
  for (int i = 0; i < kRowPieces; ++i) id[i] = s_u[st_p + 8 * kDpWaves * i];   // -1: out of range, loads zeros
#pragma unroll
  for (int i = 0; i < kRowPieces; ++i) {
    const int g = wave + kDpWaves * i;
    if (g < groups) dp_dma16(rs, s_rows + g * 1024, (uint32_t)id[i] * pitch + (coff + st_c));
  }
}

// s_waitcnt immediates (vmcnt in bits 3:0 and 15:14, no wait on the export and LDS counters).  As an
// instruction of its own, not inline assembly: the compiler's own wait insertion then knows that
// the loads have landed and adds no waits of its own for their registers further down.
constexpr int kDpWaitVm0 = 0x0f70, kDpWaitVm2 = 0x0f72;

static __device__ __forceinline__ void dp_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// What a thread carries from global memory to LDS for the tile after next: its entries of the
// list of distinct rows and its 16-byte pieces of the table positions (as LDS byte offsets).
template <int KT>
struct DpAhead {
  static constexpr int kLoc = (KT * 16 + kDpThreads - 1) / kDpThreads;
  static constexpr int kIds = (kDpRowsAlloc + kDpThreads - 1) / kDpThreads;
  int32_t id[kIds];
  u32x4 lc[kLoc];
};

template <int KT>
static __device__ __forceinline__ void dp_ahead_load(DpAhead<KT>& a, const uint16_t* loc, const int32_t* urows,
                                                     int64_t tile, int32_t p0, int U, int tid) {
#pragma unroll
  for (int r = 0; r < DpAhead<KT>::kIds; ++r) {
    const int i = tid + kDpThreads * r;
    a.id[r] = (i >= 1 && i <= U) ? urows[p0 + i - 1] : -1;
  }
  const u32x4* src = (const u32x4*)(loc + tile * (int64_t)(kDpRows * KT));
#pragma unroll
  for (int r = 0; r < DpAhead<KT>::kLoc; ++r) {
    const int i = tid + kDpThreads * r;
    a.lc[r] = src[min(i, KT * 16 - 1)];
  }
}

// Positions go to LDS as 16-bit byte offsets in the order the kernel reads them: element
// PERM::index(row in tile) of the slot's 128, so that what a lane needs of a slot is one read.
struct DpGatherOrder {      // lane R of 64, its rows 8 (R / 4) + 4 j + R % 4, j = 0, 1, side by side
  static __device__ __forceinline__ int piece(int i16) { return 8 * i16; }
  static constexpr int element(int e) { return 2 * (e & 3) + (e >> 2); }
};
struct DpWgradOrder {       // row 64 b + 8 t + e at 64 b + 8 e + t: a lane's rows 8 apart side by side
  static __device__ __forceinline__ int piece(int i16) { return 64 * (i16 >> 3) + (i16 & 7); }
  static constexpr int element(int e) { return 8 * e; }
};

template <int KT, typename ORDER>
static __device__ __forceinline__ void dp_ahead_store(const DpAhead<KT>& a, int32_t* s_u, uint16_t* s_loc, int tid) {
#pragma unroll
  for (int r = 0; r < DpAhead<KT>::kIds; ++r) {
    const int i = tid + kDpThreads * r;
    if (i < kDpRowsAlloc) s_u[i] = a.id[r];
  }
#pragma unroll
  for (int r = 0; r < DpAhead<KT>::kLoc; ++r) {
    const int i = tid + kDpThreads * r;                      // piece i: rows 8 (i % 16) .. + 7 of slot i / 16
    if (i < KT * 16) {
      const u32x4 off = dp_loc_offsets(a.lc[r]);
      uint16_t* dst = s_loc + (i >> 4) * kDpRows + ORDER::piece(i & 15);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        dst[ORDER::element(e)] = (uint16_t)((e & 1) ? off[e >> 1] >> 16 : off[e >> 1] & 0xffffu);
    }
  }
}

// First tile and tile count of workgroup `range` of `ranges` (whole tiles, sizes differ by one).
static __device__ __forceinline__ void dp_tile_range(int64_t tiles, int range, int ranges, int64_t& first, int& n) {
  const int64_t q = tiles / ranges, r = tiles % ranges;
  first = range * q + min<int64_t>(range, r);
  n = (int)(q + (range < r ? 1 : 0));
}

// Gather on the 4x4x4 matrix instruction.  A workgroup owns a 64-channel chunk and a range of
// 128-row tiles and stays on its CU: while it multiplies tile i, the rows of tile i + 1 are in
// flight into the other half of s_rows and list and positions of tile i + 2 into registers.
// Lane l of wave v: 16-byte chunk c = (l / 4) % 8 of the rows 8 (R / 4) + 4 j + R % 4, j = 0, 1,
// R = l % 4 + 4 (l / 32) + 8 v (16 lanes read 4 consecutive rows x 4 chunks: the swizzle above).
// The four lanes of a block share the chunk; the weights are
// operand A as diag(w[k][4 channels]) and stay in registers, the lane's half chunk (4 channels
// of the gathered row) is operand B: D_b[i][n] = w[i] x_n[i], so a lane's four result registers
// are the 4 channels of its own row.  (0 x a non-finite channel is NaN: a non-finite input
// value reaches the other three channels of its group of four.)
template <typename T, int KT>
__global__ __launch_bounds__(kDpThreads, 1) void dw_gather_planned_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const uint16_t* __restrict__ loc,
    const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows, const T* __restrict__ w,
    const T* __restrict__ bias, T* __restrict__ out, uint32_t out_bytes, int64_t rows_out, int C,
    int reverse, int64_t tiles, int ranges, int nchunk) {
  // two arrays, not one of two halves: the compiler then knows that the reads of one cannot meet
  // the loads in flight into the other and does not wait for them
  __shared__ __attribute__((aligned(16))) T s_rows0[kDpRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) T s_rows1[kDpRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc[3][KT * kDpRows];
  __shared__ int32_t s_u[2][kDpListAlloc];

  const int chunk = blockIdx.x % nchunk;
  int64_t t_begin;
  int n;
  dp_tile_range(tiles, blockIdx.x / nchunk, ranges, t_begin, n);
  if (n <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = (lane >> 2) & 7;
  const int R = (lane & 3) + 4 * (lane >> 5) + 8 * wave;

  // operand A of slot k: the lane's channel 8 c + l % 4 of the chunk at element l % 4 of the
  // first operand, channel + 4 at the same element of the second
  u32x2 wd[KT][2];
  {
    const int q = lane & 3;
    const uint32_t sh = 16u * (q & 1);
    const bool first = (q & 2) == 0;
#pragma unroll
    for (int k = 0; k < KT; ++k) {
      const T* wp = w + (int64_t)(reverse ? KT - 1 - k : k) * C + 64 * chunk + 8 * c + q;
      const uint32_t lo = (uint32_t)__builtin_bit_cast(uint16_t, wp[0]) << sh;
      const uint32_t hi = (uint32_t)__builtin_bit_cast(uint16_t, wp[4]) << sh;
      wd[k][0] = u32x2{first ? lo : 0u, first ? 0u : lo};
      wd[k][1] = u32x2{first ? hi : 0u, first ? 0u : hi};
    }
  }
  float bv[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) bv[e] = bias ? to_f32(bias[64 * chunk + 8 * c + e]) : 0.f;

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t rs_out = make_rsrc(out, out_bytes);
  const uint32_t pitch = (uint32_t)C * 2u, coff = (uint32_t)chunk * 128u;
  const uint32_t cxx = ((uint32_t)c << 4) * 0x00010001u;
  const uint32_t out_lane = coff + (uint32_t)c * 16u;

  // ---- prologue: tile 0 staged, tile 1 on its way to registers, the list range of tile 2 ----
  DpAhead<KT> ahead;
  int32_t pa = uptr[t_begin], pb = uptr[t_begin + 1];        // list range of the tile `ahead` is for
  dp_ahead_load<KT>(ahead, loc, urows, t_begin, pa, pb - pa, tid);
  dp_ahead_store<KT, DpGatherOrder>(ahead, s_u[0], s_loc[0], tid);
  int U_next = pb - pa;                                      // distinct rows of the tile staged next
  dp_barrier();
  dp_stage_rows(rs_in, (char*)s_rows0, s_u[0], (U_next + 8) >> 3, pitch, coff, wave, lane);
  if (n > 1) {
    pa = pb;
    pb = uptr[t_begin + 2];
    dp_ahead_load<KT>(ahead, loc, urows, t_begin + 1, pa, pb - pa, tid);
    U_next = pb - pa;
  }
  // end of the list of the tile after that: a vector load, whose wait does not hold up LDS reads
  const __amdgpu_buffer_rsrc_t rs_uptr = make_rsrc(uptr, (uint32_t)(tiles + 1) * 4u);
  int32_t pc_v = n > 2 ? uptr[t_begin + 3] : 0;
  __builtin_amdgcn_s_waitcnt(kDpWaitVm0);

  int b3 = 0;
  auto tile_step = [&](auto BUF, int i) {
    constexpr int b = decltype(BUF)::value;
    T* rows_cur = b ? s_rows1 : s_rows0;
    T* rows_nxt = b ? s_rows0 : s_rows1;
    const int b3n = b3 == 2 ? 0 : b3 + 1;
    // rows of tile i and the registers for tile i + 1 have arrived (memory operations complete
    // in issue order; the two stores of the tile before may still be on their way)
    __builtin_amdgcn_s_waitcnt(kDpWaitVm2);
    if (i + 1 < n) dp_ahead_store<KT, DpGatherOrder>(ahead, s_u[b ^ 1], s_loc[b3n], tid);
    dp_barrier();
    if (i + 1 < n) dp_stage_rows(rs_in, (char*)rows_nxt, s_u[b ^ 1], (U_next + 8) >> 3, pitch, coff, wave, lane);
    if (i + 2 < n) {
      pa = pb;
      pb = __builtin_amdgcn_readfirstlane(pc_v);
      dp_ahead_load<KT>(ahead, loc, urows, t_begin + i + 2, pa, pb - pa, tid);
      U_next = pb - pa;
      if (i + 3 < n) pc_v = __builtin_amdgcn_raw_buffer_load_b32(rs_uptr, (uint32_t)(t_begin + i + 4) * 4u, 0, 0);
    }
    asm volatile("" ::: "memory");

    f32x4 acc[2][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[j][0] = acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    const char* rows_c = (const char*)rows_cur;
    const char* loc_c = (const char*)s_loc[b3] + 4 * R;
    // all positions of the lane's two rows first (one wait), then the rows of two slots in
    // flight under the instructions of a slot
    uint32_t pp[KT];
#pragma unroll
    for (int k = 0; k < KT; ++k) pp[k] = *(const uint32_t*)(loc_c + k * (2 * kDpRows));
    constexpr int AHEAD = 4;                                 // slots whose rows are in flight
    u32x4 xv[AHEAD + 1][2];
    auto read_rows = [&](u32x4 (&v)[2], uint32_t p) {
      p ^= cxx;
      v[0] = *(const u32x4*)(rows_c + (p & 0xffffu));
      v[1] = *(const u32x4*)(rows_c + (p >> 16));
    };
#pragma unroll
    for (int k = 0; k < AHEAD; ++k)
      if (k < KT) read_rows(xv[k], pp[k]);
#pragma unroll
    for (int k = 0; k < KT; ++k) {
      if (k + AHEAD < KT) read_rows(xv[(k + AHEAD) % (AHEAD + 1)], pp[k + AHEAD]);
      __builtin_amdgcn_sched_barrier(0);
      constexpr int M = AHEAD + 1;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        acc[j][0] = Mma4<T>::run(wd[k][0], u32x2{xv[k % M][j][0], xv[k % M][j][1]}, acc[j][0]);
        acc[j][1] = Mma4<T>::run(wd[k][1], u32x2{xv[k % M][j][2], xv[k % M][j][3]}, acc[j][1]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    const int64_t row0 = (t_begin + i) * kDpRows + 8 * (R >> 2) + (R & 3);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      unsigned pk[4];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int e = 0; e < 2; ++e)
          pk[2 * h + e] = pack2<T>(acc[j][h][2 * e] + bv[4 * h + 2 * e], acc[j][h][2 * e + 1] + bv[4 * h + 2 * e + 1]);
      // every lane issues its two stores (the wait at the top counts on it); rows past the end are dropped
      const uint32_t off = row0 + 4 * j < rows_out ? (uint32_t)(row0 + 4 * j) * pitch + out_lane : 0xfffffff0u;
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{pk[0], pk[1], pk[2], pk[3]}, rs_out, off, 0, 0);
    }
    asm volatile("" ::: "memory");
    b3 = b3n;
  };
  for (int i = 0; i < n; i += 2) {
    tile_step(std::integral_constant<int, 0>{}, i);
    if (i + 1 < n) tile_step(std::integral_constant<int, 1>{}, i + 1);
  }
}

// Weight gradient, organised like the gather kernel (a workgroup per CU, rows of the next tile in
// flight, list and positions of the one after in registers).  The sum over rows is the
// contraction of the 4x4x4 instruction: both operands are read with the transposing LDS load
// (a lane receives ONE channel of four rows), operand A from the staged rows at the table's
// positions, operand B from the tile of g, which is staged once, read into registers and held
// there over the slots.  Lane l of wave v: channel 16 (v % 4) + l % 16; the four lanes l / 4 % 4 = j
// that share their channels address the rows 64 (l / 32) + 8 t + 4 (l / 16 % 2) + j, contracted
// over j, t = 4 (v / 4) .. + 3 one instruction each; of D_b = A_b B_b the diagonal is the wanted
// sum (element l % 4 of the lane), the rest is dropped.
template <typename T, int KT>
__global__ __launch_bounds__(kDpThreads, 1) void dw_wgrad_planned_kernel(
    const T* __restrict__ x, uint32_t x_bytes, const T* __restrict__ g, uint32_t g_bytes,
    const uint16_t* __restrict__ loc, const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows,
    int64_t rows, int C, int64_t tiles, int nsplit, int nchunk, float* __restrict__ partial) {
  __shared__ __attribute__((aligned(16))) T s_rows0[kDpRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) T s_rows1[kDpRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) T s_g[kDpRows * 64];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc[3][KT * kDpRows];
  __shared__ int32_t s_u[2][kDpListAlloc];

  const int chunk = blockIdx.x % nchunk, split = blockIdx.x / nchunk;
  int64_t t_begin;
  int n;
  dp_tile_range(tiles, split, nsplit, t_begin, n);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int G = lane >> 4, jj = (lane >> 2) & 3, q = lane & 3;
  const int cidx = 2 * (wave & 3) + (q >> 1);                 // the 16-byte chunk the lane addresses
  const int t0 = 4 * (wave >> 2);                             // its four rows of eight

  f32x4 acc[KT];
#pragma unroll
  for (int k = 0; k < KT; ++k) acc[k] = f32x4{0.f, 0.f, 0.f, 0.f};

  const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, x_bytes);
  const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(g, g_bytes);
  const uint32_t pitch = (uint32_t)C * 2u, coff = (uint32_t)chunk * 128u;
  // the lane's rows: 64 (G / 2) + 8 t + e, e = 4 (G % 2) + jj, t = 0..7; the 32 lanes of half a wave
  // read 8 consecutive rows x 32 bytes.  s_g is row-major with chunk cc of row r at chunk
  // cc ^ 2 ((r / 2) % 4), which gives the 8 rows banks of their own
  const int e_row = 4 * (G & 1) + jj;
  const char* g_c = (const char*)s_g + (64 * (G >> 1) + 8 * t0 + e_row) * 128 + ((cidx ^ (((e_row >> 1) & 3) << 1)) << 4) + ((q & 1) << 3);
  const uint32_t loc_lane = 2u * (32 * G + 8 * jj + t0);
  const uint32_t lanec = (((uint32_t)cidx << 4) | ((uint32_t)(q & 1) << 3)) * 0x00010001u;
  auto stage_g = [&](int64_t tile) {
#pragma unroll
    for (int i = 0; i < 16 / kDpWaves; ++i) {
      const int u = wave + kDpWaves * i;
      const int r8 = lane >> 3, cc = (lane & 7) ^ (((r8 >> 1) & 3) << 1);
      const int64_t row = tile * kDpRows + 8 * u + r8;
      const uint32_t off = row < rows ? (uint32_t)row * pitch + (coff + (uint32_t)cc * 16u) : 0xfffffff0u;
      dp_dma16(rs_g, (char*)s_g + u * 1024, off);
    }
  };

  if (n > 0) {
    DpAhead<KT> ahead;
    int32_t pa = uptr[t_begin], pb = uptr[t_begin + 1];
    dp_ahead_load<KT>(ahead, loc, urows, t_begin, pa, pb - pa, tid);
    dp_ahead_store<KT, DpWgradOrder>(ahead, s_u[0], s_loc[0], tid);
    int U_next = pb - pa;
    dp_barrier();
    dp_stage_rows(rs_x, (char*)s_rows0, s_u[0], (U_next + 8) >> 3, pitch, coff, wave, lane);
    stage_g(t_begin);
    if (n > 1) {
      pa = pb;
      pb = uptr[t_begin + 2];
      dp_ahead_load<KT>(ahead, loc, urows, t_begin + 1, pa, pb - pa, tid);
      U_next = pb - pa;
    }
    const __amdgpu_buffer_rsrc_t rs_uptr = make_rsrc(uptr, (uint32_t)(tiles + 1) * 4u);
    int32_t pc_v = n > 2 ? uptr[t_begin + 3] : 0;

    int b3 = 0;
    auto tile_step = [&](auto BUF, int i) {
      constexpr int b = decltype(BUF)::value;
      T* rows_cur = b ? s_rows1 : s_rows0;
      T* rows_nxt = b ? s_rows0 : s_rows1;
      const int b3n = b3 == 2 ? 0 : b3 + 1;
      __builtin_amdgcn_s_waitcnt(kDpWaitVm0);
      if (i + 1 < n) dp_ahead_store<KT, DpWgradOrder>(ahead, s_u[b ^ 1], s_loc[b3n], tid);
      dp_barrier();
      u32x2 gf[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) gf[t] = Mma<T>::read_tr((const T*)(g_c + t * 1024));
      dp_barrier();                                           // s_g is free for the next tile
      if (i + 1 < n) {
        dp_stage_rows(rs_x, (char*)rows_nxt, s_u[b ^ 1], (U_next + 8) >> 3, pitch, coff, wave, lane);
        stage_g(t_begin + i + 1);
      }
      if (i + 2 < n) {
        pa = pb;
        pb = __builtin_amdgcn_readfirstlane(pc_v);
        dp_ahead_load<KT>(ahead, loc, urows, t_begin + i + 2, pa, pb - pa, tid);
        U_next = pb - pa;
        if (i + 3 < n) pc_v = __builtin_amdgcn_raw_buffer_load_b32(rs_uptr, (uint32_t)(t_begin + i + 4) * 4u, 0, 0);
      }
      asm volatile("" ::: "memory");

      const char* rows_c = (const char*)rows_cur;
      const char* loc_c = (const char*)s_loc[b3] + loc_lane;
      // Two slots a step, their instructions alternating (an instruction that adds to the result
      // of the one before it waits for it).  Under a step the rows of the next two slots are in
      // flight; positions are read two steps ahead of the row reads that use them.
      u32x2 d[KT];
      u32x2 xf[4][4];
      auto read_pos = [&](int k) { d[k] = *(const u32x2*)(loc_c + k * (2 * kDpRows)); };
      auto read_rows = [&](u32x2 (&v)[4], u32x2 dk) {
        dk ^= u32x2{lanec, lanec};
#pragma unroll
        for (int t = 0; t < 4; ++t)
          v[t] = Mma<T>::read_tr((const T*)(rows_c + ((t & 1) ? dk[t >> 1] >> 16 : dk[t >> 1] & 0xffffu)));
      };
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (k < KT) read_pos(k);
      read_rows(xf[0], d[0]);
      if (KT > 1) read_rows(xf[1], d[1]);
#pragma unroll
      for (int k = 0; k < KT; k += 2) {
        if (k + 2 < KT) read_rows(xf[(k + 2) & 3], d[k + 2]);
        if (k + 3 < KT) read_rows(xf[(k + 3) & 3], d[k + 3]);
        if (k + 4 < KT) read_pos(k + 4);
        if (k + 5 < KT) read_pos(k + 5);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          acc[k] = Mma4<T>::run(xf[k & 3][t], gf[t], acc[k]);
          if (k + 1 < KT) acc[k + 1] = Mma4<T>::run(xf[(k + 1) & 3][t], gf[t], acc[k + 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      b3 = b3n;
    };
    for (int i = 0; i < n; i += 2) {
      tile_step(std::integral_constant<int, 0>{}, i);
      if (i + 1 < n) tile_step(std::integral_constant<int, 1>{}, i + 1);
    }
  }

  // ---- the diagonal elements of the eight row groups of a channel, added in a fixed order ----
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  float* s_red = (float*)s_rows0;                            // [KT][2 halves of the rows][64 channels]
#pragma unroll
  for (int k = 0; k < KT; ++k) {
    float v = q == 0 ? acc[k][0] : q == 1 ? acc[k][1] : q == 2 ? acc[k][2] : acc[k][3];
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    if (lane < 16) s_red[(k * 2 + (wave >> 2)) * 64 + 16 * (wave & 3) + lane] = v;
  }
  __syncthreads();
  for (int i = tid; i < KT * 64; i += kDpThreads) {
    const int k = i >> 6, ch = i & 63;
    partial[((int64_t)split * KT + k) * C + 64 * chunk + ch] = s_red[k * 128 + ch] + s_red[k * 128 + 64 + ch];
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

static bool dp_slots_ok(int K) { return K == 27 || K == 9 || K == 8 || K == 3; }

// Tile ranges of the weight gradient: one workgroup per CU over the chunks of the channels.
static int dp_splits(int C, int n_cu) { return std::min(1024, std::max(1, n_cu / (C / 64))); }

extern "C" int ocnn_dwconv_gather_planned_supported(int dtype, int64_t rows_in, int K, int channels,
                                                    int plan_max_distinct) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (channels < 64 || channels % 64 != 0 || channels > 4096) return 0;
  if (!dp_slots_ok(K)) return 0;
  if (plan_max_distinct < 0 || plan_max_distinct > kDpCap) return 0;
  if (rows_in < 0 || (int64_t)rows_in * channels * 2 > 0xfff00000ll) return 0;
  return 1;
}

template <typename T>
static int run_dp_gather(const void* in, int64_t rows_in, const uint16_t* loc, const int32_t* uptr,
                         const int32_t* urows, int64_t rows_out, int K, const void* w, int C, int reverse,
                         const void* bias, void* out, hipStream_t st) {
  const int n_cu = dp_cu_count();
  if (n_cu <= 0) {
    set_error("dwconv_gather_planned: cannot query the device");
    return OCNN_ERR_HIP;
  }
  const int nchunk = C / 64;
  const int64_t tiles = cdiv(rows_out, kDpRows);
  const int ranges = (int)std::min<int64_t>(tiles, std::max(1, n_cu / nchunk));
  const dim3 grid((unsigned)(ranges * nchunk));
  const uint32_t in_bytes = (uint32_t)(rows_in * C * 2), out_bytes = (uint32_t)(rows_out * C * 2);
#define OCNN_DP_GATHER(KT_)                                                                                  \
  hipLaunchKernelGGL((dw_gather_planned_kernel<T, KT_>), grid, dim3(kDpThreads), 0, st, (const T*)in, in_bytes, loc, \
                     uptr, urows, (const T*)w, (const T*)bias, (T*)out, out_bytes, rows_out, C, reverse,      \
                     tiles, ranges, nchunk)
  if (K == 27) OCNN_DP_GATHER(27);
  else if (K == 9) OCNN_DP_GATHER(9);
  else if (K == 8) OCNN_DP_GATHER(8);
  else OCNN_DP_GATHER(3);
#undef OCNN_DP_GATHER
  return check_launch("dwconv_gather_planned");
}

extern "C" int ocnn_dwconv_gather_planned(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                                          const int32_t* uptr, const int32_t* urows, int plan_max_distinct,
                                          int64_t plan_total, int64_t rows_out, int K, const void* w,
                                          int channels, int reverse_slots, const void* bias, void* out,
                                          void* stream) {
  OCNN_REQUIRE(ocnn_dwconv_gather_planned_supported(dtype, rows_in, K, channels, plan_max_distinct),
               "dwconv_gather_planned: shape not supported");
  OCNN_REQUIRE(rows_out >= 0 && rows_out < (1ll << 31) && plan_total >= 0 && plan_total < (1ll << 29) &&
                   (int64_t)rows_out * channels * 2 <= 0xfff00000ll,
               "dwconv_gather_planned: rows out of range");
  if (rows_out == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("dwconv_gather_planned", loc, uptr, urows, w, out);
  OCNN_REQUIRE(rows_in == 0 || in, "dwconv_gather_planned: in is NULL");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16)
    return run_dp_gather<f16>(in, rows_in, loc, uptr, urows, rows_out, K, w, channels, reverse_slots, bias, out, st);
  return run_dp_gather<bf16>(in, rows_in, loc, uptr, urows, rows_out, K, w, channels, reverse_slots, bias, out, st);
}

extern "C" int ocnn_dwconv_wgrad_planned_supported(int dtype, int64_t rows_x, int64_t rows, int K,
                                                   int channels, int plan_max_distinct) {
  if (!ocnn_dwconv_gather_planned_supported(dtype, rows_x, K, channels, plan_max_distinct)) return 0;
  if (rows < 0 || (int64_t)rows * channels * 2 > 0xfff00000ll) return 0;
  return 1;
}

extern "C" int64_t ocnn_dwconv_wgrad_planned_workspace_bytes(int K, int channels) {
  const int n_cu = dp_cu_count();
  if (!dp_slots_ok(K) || channels < 64) return 0;
  const int64_t splits = n_cu > 0 ? dp_splits(channels, n_cu) : 1024;
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
  const int64_t tiles = cdiv(rows, kDpRows);
  const int nsplit = (int)std::min<int64_t>(std::max<int64_t>(tiles, 1), dp_splits(C, n_cu));
  if (ws_bytes < (int64_t)nsplit * K * C * 4) {
    set_error("dwconv_wgrad_planned: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  float* partial = (float*)ws;
  if (rows > 0) {
    const int nchunk = C / 64;
    const dim3 grid((unsigned)(nsplit * nchunk));
    const uint32_t xb = (uint32_t)(rows_x * C * 2), gb = (uint32_t)(rows * C * 2);
#define OCNN_DP_WGRAD(KT_)                                                                              \
  hipLaunchKernelGGL((dw_wgrad_planned_kernel<T, KT_>), grid, dim3(kDpThreads), 0, st, (const T*)x, xb, (const T*)g, \
                     gb, loc, uptr, urows, rows, C, tiles, nsplit, nchunk, partial)
    if (K == 27) OCNN_DP_WGRAD(27);
    else if (K == 9) OCNN_DP_WGRAD(9);
    else if (K == 8) OCNN_DP_WGRAD(8);
    else OCNN_DP_WGRAD(3);
#undef OCNN_DP_WGRAD
  }
  launch_wgrad_reduce<T>(partial, rows > 0 ? nsplit : 0, K, 1, C, 0, (T*)gw, st);
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
  OCNN_REQUIRE_PTRS("dwconv_wgrad_planned", gw, workspace);
  OCNN_REQUIRE(rows == 0 || (g && loc && uptr && urows && (rows_x == 0 || x)),
               "dwconv_wgrad_planned: a required pointer is NULL (of x, g, loc, uptr, urows)");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16)
    return run_dp_wgrad<f16>(x, rows_x, g, loc, uptr, urows, rows, K, channels, gw, workspace, workspace_bytes, st);
  return run_dp_wgrad<bf16>(x, rows_x, g, loc, uptr, urows, rows, K, channels, gw, workspace, workspace_bytes, st);
}
