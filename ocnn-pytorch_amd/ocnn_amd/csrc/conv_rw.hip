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
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "mma.hpp"

namespace ocnn {

constexpr int kRwRows = 128;   // rows per tile (the plan's tile size)
constexpr int kRwCap = 416;    // staged rows; plans with a larger tile use another kernel

// Packed weights: [gid = 2 * slot + half][k-step s][M tile tM][lane][8].
// v_mfma_f32_32x32x16 A operand: lane l holds A[l % 32][8 * (l / 32) + j];
// D: lane l, register r holds D[8 * (r / 4) + 4 * (l / 32) + r % 4][l % 32].
//   input channel  = 32 half + 16 s + 8 (lane / 32) + j
//   output channel = 32 tM + perm(lane % 32), perm(8a + 4q + b) = 16 (a / 2) + 8 q + 4 (a % 2) + b,
// so that registers 8 R .. 8 R + 7 of a lane are the 8 consecutive output channels
// 16 R + 8 q ..: a 16-byte store per lane, and the two lanes (q = 0, 1) of a row write 32
// contiguous bytes.
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
  int co = 32 * tM + 16 * (m >> 4) + 8 * ((m >> 2) & 1) + 4 * ((m >> 3) & 1) + (m & 3);
  int kk = reverse ? K - 1 - k : k;
  out[e] = transposed ? w[((int64_t)kk * 64 + co) * 64 + chan] : w[((int64_t)kk * 64 + chan) * 64 + co];
}

// What the staging pieces of a tile need (plain types: the arguments of the global->LDS
// load builtin must not be type-dependent expressions).
struct RwStage {
  uint32_t loc_off;     // byte offset of the tile's table positions
  uint32_t list_off;    // per lane: byte offset of its part of the list of the tile after, or out of range
  int groups;           // 8-row groups of LDS rows the tile fills (row 0 = zero row included)
  const int32_t* su;    // list of the tile's distinct rows (LDS), entry -1 readable and -1
  int32_t* su_out;      // where the next list goes (LDS)
  char* rows;           // destination buffers (LDS)
  char* locs;
};

template <typename T, int UPW>
__global__ __launch_bounds__(256, 1) void conv_gather_rw_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const uint16_t* __restrict__ loc,
    uint32_t loc_bytes, const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows,
    uint32_t urows_bytes, const T* __restrict__ wpk, const T* __restrict__ bias,
    T* __restrict__ out, int64_t rows_out, int K, int64_t tiles, int64_t tiles_per_wg) {
  constexpr int kLocElems = (kRwRows * 27 * 2 + 1023) / 1024 * 512;   // whole KiB: filled 1 KiB per instruction
  // Everything a tile needs is double buffered, one array per buffer so that the compiler
  // can tell the buffer being filled from the one being read.
  constexpr int kRowsAlloc = (kRwCap + 8) / 8 * 8;               // rows 0..kRwCap, whole 8-row groups
  __shared__ __attribute__((aligned(16))) T s_rows0[kRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) T s_rows1[kRowsAlloc * 64];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc0[kLocElems];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc1[kLocElems];
  // lists of distinct rows from entry 4 on; entry 3 stays -1 ("the row before the first")
  __shared__ __attribute__((aligned(16))) int32_t s_u0[4 + 512];
  __shared__ __attribute__((aligned(16))) int32_t s_u1[4 + 512];
  __shared__ f32x4 s_red[4 * 4 * 2 * 64];      // 32 KiB: [writer][combination][quarter of a round][lane]
  __shared__ __attribute__((aligned(16))) float s_bias[64];

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
  // bias as fp32 in LDS (zeros without one); a lane finishes the output channels
  // 32 (wave % 2) + 16 round + 8 q .. + 7 of a row
  if (tid < 64) s_bias[tid] = bias ? to_f32(bias[tid]) : 0.f;
  if (tid == 0) s_u0[3] = s_u1[3] = -1;
  const f32x4* bias4 = (const f32x4*)(&s_bias[32 * (wave & 1) + 8 * q]);

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t rs_loc = make_rsrc(loc, loc_bytes);
  const __amdgpu_buffer_rsrc_t rs_u = make_rsrc(urows, urows_bytes);
  const __amdgpu_buffer_rsrc_t rs_p = make_rsrc(uptr, (uint32_t)(tiles + 1) * 4u);
  const __amdgpu_buffer_rsrc_t rs_out = make_rsrc(out, (uint32_t)(rows_out * 128));

  // ---- staging of one tile, cut into per-wave pieces (one 1 KiB load instruction each) ----
  //   piece 0, 1      table positions (chunks wave, wave + 4)
  //   piece 2         the list of distinct rows of the tile after (waves 0 and 1)
  //   piece 3 + i     LDS rows 8 (wave + 4 i) .. + 7: row p >= 1 holds the (p - 1)-th distinct
  //                   row, row 0 is the zero row that empty table entries (position 0) read;
  //                   it comes from an out-of-range offset (list entry -1 = -1)
  // A lane's 16-byte chunk c of row p lands at chunk c ^ ((p >> 1) & 7) (bank swizzle); with
  // p = 8 (wave + 4 i) + lane / 8 that is a per-lane constant.
  constexpr int kRowPieces = (kRwCap + 1 + 31) / 32;            // per wave
  constexpr int kPieces = 3 + kRowPieces;
  const uint32_t st_c = (uint32_t)(((lane & 7) ^ (((lane >> 4) + 4 * wave) & 7)) * 16);
  const int st_p = 8 * wave + (lane >> 3);                      // LDS row of row piece 0; piece i: + 32 i
  auto make_stage = [&](int64_t tile, int U, int32_t list_first, int32_t list_len, const int32_t* su,
                        int32_t* su_out, T* rows, uint16_t* locs) {
    RwStage st;
    const int64_t tc = min(tile, tiles - 1);                    // past the range: any valid tile
    st.loc_off = (uint32_t)(tc * kRwRows * KK * 2);
    const int e = wave * 256 + lane * 4;                        // the four list entries this lane brings in
    st.list_off = e < list_len ? (uint32_t)(list_first + e) * 4u : 0xffffff00u;
    st.groups = (U + 8) >> 3;
    st.su = su; st.su_out = su_out; st.rows = (char*)rows; st.locs = (char*)locs;
    return st;
  };
  auto stage_id = [&](int t, const RwStage& st) -> int32_t {    // the list entry a lane needs for piece t
    return t >= 3 ? st.su[st_p + 32 * (t - 3) - 1] : 0;
  };
  auto stage_piece = [&](int t, const RwStage& st, int32_t id) {
    if (t < 2) {
      constexpr int nchunk = (kRwRows * KK * 2 + 1023) >> 10;
      if (4 * t < nchunk) {
        const int c = min(wave + 4 * t, nchunk - 1);            // a spare wave repeats the last chunk
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_loc, (lds_ptr_t)(st.locs + c * 1024), 16,
                                                 st.loc_off + (uint32_t)c * 1024u + lane * 16u, 0, 0, 0);
      }
    } else if (t == 2) {
      if (wave < 2)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_u, (lds_ptr_t)(st.su_out + wave * 256), 16, st.list_off,
                                                 0, 0, 0);
    } else {
      if (wave + 4 * (t - 3) < st.groups)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_in, (lds_ptr_t)(st.rows + (wave + 4 * (t - 3)) * 1024), 16,
                                                 ((uint32_t)id << 7) | st_c, 0, 0, 0);
    }
  };


  // Two accumulator sets: while a 64-row half is being multiplied into one, the partial sums
  // of the half before it (the other set) are exchanged through LDS and stored, a piece per
  // step of the main loop, in the shadow of the MFMAs.
  f32x16 acc[2][2][2];

  // ---- the cross-wave sum of one half, cut into pieces for the steps of a main loop ----
  // Wave w finishes (row tile w / 2, M tile w % 2).  Two rounds of two register quarters:
  // every wave writes all four combinations to s_red (also its own: the code is then the
  // same for every wave and free of branches, which cost a wave far more than an LDS round
  // trip), barrier, the owner reads the four partial sums, adds them in wave order, stores.
  f32x4 red[4], rb;        // partial sums and bias of a quarter (read at one piece, used at the next)
  unsigned pk[4];
  auto exch_piece = [&](auto SETC, int e, int64_t row0, bool drain) {     // row0: first row of that half
    constexpr int S = decltype(SETC)::value;
    const int rnd = e >= 13 ? 1 : 0, f = e - 13 * rnd;       // round, piece of the round
    auto barrier = [&]() {
      // With 28 steps a wave has consumed, before a barrier piece, LDS reads that it issued
      // after its last write or read of s_red (LDS operations of a wave complete in order);
      // in the shorter loops, and without a main loop around, it waits.
      if (drain) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else asm volatile("s_barrier" ::: "memory");
    };
    if (e >= 26) return;
    if (f < 4) {                                              // two writes: combination f, both quarters
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int r4 = 2 * rnd + h;
        s_red[((wave * 4 + f) * 2 + h) * 64 + lane] =
            f32x4{acc[S][f >> 1][f & 1][4 * r4], acc[S][f >> 1][f & 1][4 * r4 + 1],
                  acc[S][f >> 1][f & 1][4 * r4 + 2], acc[S][f >> 1][f & 1][4 * r4 + 3]};
      }
    } else if (f == 7) {
      barrier();                                              // the partial sums are in place
    } else if (f >= 8 && f <= 11) {
      if (f == 9 || f == 10) {                                // add the quarter read one piece ago
        const int h = f - 9;
        const f32x4 sum = ((red[0] + red[1]) + red[2]) + red[3];
        pk[2 * h] = pack2<T>(sum[0] + rb[0], sum[1] + rb[1]);
        pk[2 * h + 1] = pack2<T>(sum[2] + rb[2], sum[3] + rb[3]);
      }
      if (f == 8 || f == 9) {                                 // read quarter f - 8 of the round
        const int h = f - 8;
#pragma unroll
        for (int src = 0; src < 4; ++src) red[src] = s_red[((src * 4 + wave) * 2 + h) * 64 + lane];
        rb = bias4[4 * rnd + h];
      }
      if (f == 11) {                                          // 8 channels = 16 bytes per lane
        // a buffer store: rows past the end are out of its range and dropped, so every wave
        // issues this instruction whatever the tile (the wait at the end of a tile counts on it)
        const int64_t row = row0 + 32 * (wave >> 1) + r32;
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{pk[0], pk[1], pk[2], pk[3]}, rs_out,
                                               (uint32_t)(row * 128 + 64 * (wave & 1) + 32 * rnd + 16 * q), 0, 0);
      }
    } else if (f == 12) {
      barrier();                                              // the round has been read: s_red is free again
    }
  };

  // ---- one 64-row half out of the buffers (rows, lc): main loop into acc[S], exchange of the
  // half before it (acc[1 - S]; prev_row0 past the last row: nothing is stored), staging
  // pieces t0, t0 + 1, .. of the next tile every other step (t0 < 0: none)
  auto half_body = [&](auto SETC, const T* rows, const uint16_t* lc, int64_t prev_row0, int t0, int tn,
                       const RwStage& st) {
    constexpr int S = decltype(SETC)::value;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int tM = 0; tM < 2; ++tM)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[S][nt][tM][r] = 0.f;

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
    auto addr = [&](uint32_t l, const T*& p0, const T*& p1) {   // l = 0: empty = the zero row
      const uint32_t swz = (l >> 1) & 7;
      p0 = &rows[l * 64 + ((c0 ^ swz) * 8)];
      p1 = &rows[l * 64 + (((c0 + 2) ^ swz) * 8)];
    };

    // The main loop is a flat sequence of steps (unit u, row tile nt).  The B operand of
    // a step (lane: row r32 of the row tile, k group q -> 2 x 16 B of its neighbour row)
    // is fetched from LDS three steps ahead of its four MFMAs; the table positions of a
    // unit are read three units ahead.  Units past 2K have zero weights.
    constexpr int STEPS = UPW * 2;
    uint32_t lcur[2], lnxt[2] = {0u, 0u}, lnx2[2] = {0u, 0u};
    u32x4 ring[4][2];
    const T *pa, *pb;
    read_loc(0, lcur);
    if (UPW > 1) read_loc(1, lnxt);
    if (UPW > 2) read_loc(2, lnx2);
    addr(lcur[0], pa, pb);
    ring[0][0] = *(const u32x4*)pa;
    ring[0][1] = *(const u32x4*)pb;
    addr(lcur[1], pa, pb);
    ring[1][0] = *(const u32x4*)pa;
    ring[1][1] = *(const u32x4*)pb;
    if (UPW > 1) {
      addr(lnxt[0], pa, pb);
      ring[2][0] = *(const u32x4*)pa;
      ring[2][1] = *(const u32x4*)pb;
    }
    __builtin_amdgcn_sched_barrier(0);
    constexpr int EPS = (26 + STEPS - 1) / STEPS;           // exchange pieces per step
    constexpr int SPS = STEPS >= 28 ? 1 : (kPieces + STEPS - 1) / STEPS + 1;   // staging pieces per step slot
    int32_t id_next = 0;
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
      const int u = j >> 1, nt = j & 1;
      const bool pre = j + 3 < STEPS;
      const int u3 = (j + 3) >> 1, nt3 = (j + 3) & 1;
      acc[S][nt][0] = Mma32<T>::run(wreg[u][0][0], ring[j & 3][0], acc[S][nt][0]);
      if (pre) addr(u3 == u + 1 ? lnxt[nt3] : lnx2[nt3], pa, pb);      // step j + 3
      acc[S][nt][1] = Mma32<T>::run(wreg[u][0][1], ring[j & 3][0], acc[S][nt][1]);
      if (pre) ring[(j + 3) & 3][0] = *(const u32x4*)pa;
      acc[S][nt][0] = Mma32<T>::run(wreg[u][1][0], ring[j & 3][1], acc[S][nt][0]);
      if (pre) ring[(j + 3) & 3][1] = *(const u32x4*)pb;
      if (nt == 1) {
        // the next unit becomes current; read the positions of the one three units on
        lcur[0] = lnxt[0];
        lcur[1] = lnxt[1];
        lnxt[0] = lnx2[0];
        lnxt[1] = lnx2[1];
        if (u + 3 < UPW) read_loc(u + 3, lnx2);
      }
      acc[S][nt][1] = Mma32<T>::run(wreg[u][1][1], ring[j & 3][1], acc[S][nt][1]);
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
      // staging: the list entry is read on an even step, its load goes out on the odd one after
      if (t0 >= 0) {
        if (STEPS >= 28) {
          const int t = t0 + (j >> 1);
          if (t < tn) {
            if ((j & 1) == 0) id_next = stage_id(t, st);
            else stage_piece(t, st, id_next);
          }
        } else {
#pragma unroll
          for (int i = 0; i < SPS; ++i) {
            const int t = t0 + j * SPS + i;
            if (t < tn) stage_piece(t, st, stage_id(t, st));
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- prologue: first list, first tile, second list ----
  int32_t p_nxt = uptr[t_begin + 1];
  int32_t p_nx2 = uptr[min(t_begin + 2, tiles)];
  int32_t p_nx3 = uptr[min(t_begin + 3, tiles)];
  {
    const int32_t p_cur = uptr[t_begin];
    RwStage st = make_stage(t_begin, 0, p_cur, p_nxt - p_cur, s_u0 + 4, s_u0 + 4, s_rows0, s_loc0);
    stage_piece(2, st, 0);                                   // list of the first tile -> s_u0
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    st = make_stage(t_begin, p_nxt - p_cur, p_nxt, p_nx2 - p_nxt, s_u0 + 4, s_u1 + 4, s_rows0, s_loc0);
#pragma unroll
    for (int t = 0; t < kPieces; ++t) stage_piece(t, st, stage_id(t, st));     // also: list of the second tile
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
  }

  // one tile out of buffer B; the next tile is staged into buffer 1 - B meanwhile
  constexpr int kHalfSteps = UPW;                            // staging slots in a half (one per two steps)
  auto tile_body = [&](auto BC, int64_t tile) {
    constexpr int B = decltype(BC)::value;
    const T* rows = B ? s_rows1 : s_rows0;
    const uint16_t* lc = B ? s_loc1 : s_loc0;
    // next tile -> the other buffers (its list is in the other s_u); list of the tile after
    // it -> this tile's s_u, which has been used up
    const RwStage st = make_stage(tile + 1, p_nx2 - p_nxt, p_nx2, p_nx3 - p_nx2, B ? s_u0 + 4 : s_u1 + 4,
                                  B ? s_u1 + 4 : s_u0 + 4, B ? s_rows0 : s_rows1, B ? s_loc0 : s_loc1);
    // list boundary four tiles ahead, as a vector load: a scalar load would share its counter
    // with the LDS reads and force them to drain where it is used
    const uint32_t p_raw = __builtin_amdgcn_raw_buffer_load_b32(rs_p, (uint32_t)min(tile + 4, tiles) * 4u, 0, 0);
    p_nxt = p_nx2;
    p_nx2 = p_nx3;
    half_body(std::integral_constant<int, 0>{}, rows, lc, tile > t_begin ? (tile - 1) * kRwRows + 64 : rows_out,
              0, kPieces, st);
    half_body(std::integral_constant<int, 1>{}, rows, lc, tile * kRwRows, (UPW >= 14 ? kHalfSteps : kPieces), kPieces, st);
    // The next tile has landed (own loads, then everyone's); every wave is past its last read
    // of this tile's buffers and of s_red.  Vector memory operations complete in issue order,
    // and with 28 steps the last two of this tile are the output stores of the exchange (steps
    // 11 and 24 of the second half; its staging loads end at step 5): they need not be waited
    // for, and waiting for their acknowledgement cost a tenth of the kernel's time.
    if (UPW == 14) asm volatile("s_waitcnt vmcnt(2)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    p_nx3 = __builtin_amdgcn_readfirstlane((int32_t)p_raw);
  };
  for (int64_t tile = t_begin; tile < t_end; tile += 2) {
    tile_body(std::integral_constant<int, 0>{}, tile);
    if (tile + 1 < t_end) tile_body(std::integral_constant<int, 1>{}, tile + 1);
  }
  // the last half of the range: its exchange has no main loop to hide under
#pragma unroll
  for (int e = 0; e < 26; ++e) {
    exch_piece(std::integral_constant<int, 1>{}, e, (t_end - 1) * kRwRows + 64, true);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// ---------------------------------------------------------------------------------------
// 32 -> 32 channels: the weights of all K slots (27 x 32 x 32 x 2 B = 54 KiB) fit the registers
// of ONE wave, so every wave keeps all of them and finishes its own 32 rows of a tile alone:
// no split over the slots, no cross-wave sum.  A row is 64 bytes; per slot a lane reads two
// 16-byte pieces of its neighbour row (the two k steps of 16 input channels) and issues two
// v_mfma_f32_32x32x16.  LDS reads and MFMAs take the same number of clocks at their peaks
// (64 flop per input byte at 32 output channels), so this shape is LDS-bound by nature.
// ---------------------------------------------------------------------------------------

// packed weights: [slot][k step s][lane][8]; input channel = 16 s + 8 (lane / 32) + j,
// output channel = perm(lane % 32) as above (a lane ends with 16 consecutive output channels)
template <typename T>
__global__ void pack_weights_rw32_kernel(const T* __restrict__ w, T* __restrict__ out, int K,
                                         int transposed, int reverse) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)K * 1024) return;
  int j = (int)(e & 7);
  int lane = (int)((e >> 3) & 63);
  int s = (int)((e >> 9) & 1);
  int k = (int)(e >> 10);
  int q = lane >> 5, m = lane & 31;
  int chan = 16 * s + 8 * q + j;
  int co = 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3);
  int kk = reverse ? K - 1 - k : k;
  out[e] = transposed ? w[((int64_t)kk * 32 + co) * 32 + chan] : w[((int64_t)kk * 32 + chan) * 32 + co];
}

// 32 -> 32 channels: per tile half the bytes of the 64-channel kernel and a quarter of its
// matrix work, so what bounds this kernel is how much a CU has in flight.  A ring of THREE
// tiles in LDS: while tile i is multiplied, the rows and positions of tiles i + 1 and i + 2
// are in flight.  Vector memory operations complete in issue order, so "tile i + 1 has landed"
// is a count: every wave issues exactly kOps operations per tile (pieces that a tile does not
// need go to a dump area out of range, rows past the end are stored out of range), the first
// of them the list boundary six tiles ahead, and the wait at the end of a tile leaves the
// kOps - 1 after that one in flight.  What an operation of tile i loads may therefore be used
// from tile i + 2 on: list boundary (six tiles ahead) -> the lane's entries of the list of
// distinct rows (four ahead, straight into registers, no list in LDS) -> rows and positions
// (two ahead) -> products.
template <typename T, int KK>
__global__ __launch_bounds__(256, 1) void conv_gather_rw32_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const uint16_t* __restrict__ loc,
    uint32_t loc_bytes, const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows,
    uint32_t urows_bytes, const T* __restrict__ wpk, const T* __restrict__ bias,
    T* __restrict__ out, uint32_t out_bytes, int64_t rows_out, int64_t tiles, int64_t tiles_per_wg) {
  constexpr int kLocElems = (kRwRows * 27 * 2 + 1023) / 1024 * 512;
  constexpr int kRowsAlloc = (kRwCap + 16) / 16 * 16;            // rows 0..kRwCap, whole 16-row groups
  // one array per buffer of the ring: the compiler then knows that the reads of one cannot meet
  // the loads in flight into the others and does not wait for them
  __shared__ __attribute__((aligned(16))) T s_rows0[kRowsAlloc * 32];
  __shared__ __attribute__((aligned(16))) T s_rows1[kRowsAlloc * 32];
  __shared__ __attribute__((aligned(16))) T s_rows2[kRowsAlloc * 32];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc0[kLocElems];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc1[kLocElems];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc2[kLocElems];
  __shared__ __attribute__((aligned(16))) char s_dump[1024];     // where the pieces a tile does not need go

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 5, r32 = lane & 31;
  const int64_t t_begin = (int64_t)blockIdx.x * tiles_per_wg;
  const int64_t t_end = min(tiles, t_begin + tiles_per_wg);
  if (t_begin >= t_end) return;

  u32x4 wreg[KK][2];
#pragma unroll
  for (int k = 0; k < KK; ++k)
#pragma unroll
    for (int s = 0; s < 2; ++s) wreg[k][s] = *(const u32x4*)(wpk + ((int64_t)(k * 2 + s) * 64 + lane) * 8);
  float bq[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) bq[i] = bias ? to_f32(bias[16 * q + i]) : 0.f;

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t rs_loc = make_rsrc(loc, loc_bytes);
  const __amdgpu_buffer_rsrc_t rs_u = make_rsrc(urows, urows_bytes);
  const __amdgpu_buffer_rsrc_t rs_p = make_rsrc(uptr, (uint32_t)(tiles + 1) * 4u);
  const __amdgpu_buffer_rsrc_t rs_out = make_rsrc(out, out_bytes);

  // Staging pieces of a tile per wave: kLocPieces of table positions, then kRowPieces of LDS rows
  // 16 (wave + 4 i) .. + 15 (row p >= 1 = distinct row p - 1, row 0 = zero row).  The 16-byte
  // chunk c of row p lands at chunk c ^ ((p >> 2) & 3), a per-lane constant here.
  constexpr int kRowPieces = (kRwCap + 1 + 63) / 64;
  constexpr int kLocChunks = (kRwRows * KK * 2 + 1023) >> 10;
  constexpr int kLocPieces = (kLocChunks + 3) / 4;
  constexpr int kPieces = kLocPieces + kRowPieces;
  constexpr int kOps = 1 + kRowPieces + kPieces + 2;             // boundary, list entries, pieces, stores
  static_assert(kOps - 1 <= 63, "vmcnt is a 6-bit counter");
  const uint32_t st_c = (uint32_t)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
  const int st_p = 16 * wave + (lane >> 2);                       // LDS row of row piece 0; piece i: + 64 i
  // the lane's entry of the list that starts at `first` for row piece i (position 0: the zero row)
  auto load_id = [&](int i, int32_t first) -> int32_t {
    return (int32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_u, (uint32_t)(first + st_p + 64 * i - 1) * 4u, 0, 0);
  };
  auto stage_piece = [&](int t, int64_t tile, int groups, const int32_t (&ids)[kRowPieces], char* rows, char* locs) {
    if (t < kLocPieces) {
      const int c = min(wave + 4 * t, kLocChunks - 1);            // a spare wave repeats the last chunk
      const uint32_t loc_off = (uint32_t)(min(tile, tiles - 1) * kRwRows * KK * 2);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_loc, (lds_ptr_t)(locs + c * 1024), 16,
                                               loc_off + (uint32_t)c * 1024u + lane * 16u, 0, 0, 0);
    } else {
      const int i = t - kLocPieces;
      const int g = wave + 4 * i;
      const bool need = g < groups;
      const int32_t id = (st_p + 64 * i == 0) ? -1 : ids[i];     // -1: out of range, zeros
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_in, (lds_ptr_t)(need ? rows + g * 1024 : s_dump), 16,
                                               need ? (((uint32_t)id << 6) | st_c) : 0xffffff00u, 0, 0, 0);
    }
  };

  // ---- prologue: tiles 0 and 1 staged, list entries of tiles 2 and 3 in registers ----
  // p_a .. p_d: list boundaries of the tiles i + 2 .. i + 5 while tile i is multiplied
  int32_t ids[3][kRowPieces];
  int32_t p_a, p_b, p_c, p_d;
  {
    const int32_t p0 = uptr[t_begin], p1 = uptr[min(t_begin + 1, tiles)];
    p_a = uptr[min(t_begin + 2, tiles)];
    p_b = uptr[min(t_begin + 3, tiles)];
    p_c = uptr[min(t_begin + 4, tiles)];
    p_d = uptr[min(t_begin + 5, tiles)];
#pragma unroll
    for (int i = 0; i < kRowPieces; ++i) {
      ids[0][i] = load_id(i, p0);
      ids[1][i] = load_id(i, p1);
    }
#pragma unroll
    for (int t = 0; t < kPieces; ++t) stage_piece(t, t_begin, (p1 - p0 + 16) >> 4, ids[0], (char*)s_rows0, (char*)s_loc0);
#pragma unroll
    for (int t = 0; t < kPieces; ++t) stage_piece(t, t_begin + 1, (p_a - p1 + 16) >> 4, ids[1], (char*)s_rows1, (char*)s_loc1);
#pragma unroll
    for (int i = 0; i < kRowPieces; ++i) {
      ids[2][i] = load_id(i, p_a);
      ids[0][i] = load_id(i, p_b);
    }
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("s_barrier" ::: "memory");
  }

  constexpr int PD = 8;      // table positions are read PD slots ahead of their MFMAs ...
  constexpr int BD = 4;      // ... and the neighbour rows BD slots ahead
  auto tile_body = [&](auto BC, int64_t tile) {
    constexpr int B = decltype(BC)::value;                       // this tile's buffer of the ring
    constexpr int B1 = (B + 1) % 3, B2 = (B + 2) % 3;
    const T* rows = B == 0 ? s_rows0 : B == 1 ? s_rows1 : s_rows2;
    const uint16_t* lc = B == 0 ? s_loc0 : B == 1 ? s_loc1 : s_loc2;
    char* rows_st = (char*)(B2 == 0 ? s_rows0 : B2 == 1 ? s_rows1 : s_rows2);
    char* locs_st = (char*)(B2 == 0 ? s_loc0 : B2 == 1 ? s_loc1 : s_loc2);
    const int groups_st = (p_b - p_a + 16) >> 4;                 // tile + 2 fills this many 16-row groups
    // the first operation of the tile: list boundary six tiles ahead
    const uint32_t p_raw = __builtin_amdgcn_raw_buffer_load_b32(rs_p, (uint32_t)min(tile + 6, tiles) * 4u, 0, 0);

    const uint16_t* lcw = lc + 32 * wave + r32;                 // this lane's row, slot k at + 128 k
    uint32_t pos[PD];
    u32x4 ring[PD][2];
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    auto issue_b = [&](int k) {                                  // the two 16-byte pieces of slot k
      const uint32_t l = pos[k % PD];
      const uint32_t swz = (l >> 2) & 3;
      ring[k % PD][0] = *(const u32x4*)(&rows[l * 32 + (((uint32_t)q ^ swz) * 8)]);
      ring[k % PD][1] = *(const u32x4*)(&rows[l * 32 + (((uint32_t)(2 + q) ^ swz) * 8)]);
    };
#pragma unroll
    for (int k = 0; k < PD && k < KK; ++k) pos[k] = lcw[kRwRows * k];
#pragma unroll
    for (int k = 0; k < BD && k < KK; ++k) issue_b(k);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < KK; ++k) {
      acc = Mma32<T>::run(wreg[k][0], ring[k % PD][0], acc);
      if (k + BD < KK) issue_b(k + BD);
      acc = Mma32<T>::run(wreg[k][1], ring[k % PD][1], acc);
      if (k + PD < KK) pos[k % PD] = lcw[kRwRows * (k + PD)];
      __builtin_amdgcn_sched_barrier(0);
      // staging: the list entries of tile + 4 on the even slots, the pieces of tile + 2 on the odd ones
      {
        const int t = k >> 1;
        if ((k & 1) == 0) {
          if (t < kRowPieces) ids[B1][t] = load_id(t, p_c);
        } else {
          if (t < kPieces) stage_piece(t, tile + 2, groups_st, ids[B2], rows_st, locs_st);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // few slots: the rest of the staging
#pragma unroll
    for (int t = (KK + 1) / 2; t < kRowPieces; ++t) ids[B1][t] = load_id(t, p_c);
#pragma unroll
    for (int t = KK / 2; t < kPieces; ++t) stage_piece(t, tile + 2, groups_st, ids[B2], rows_st, locs_st);
    // bias, pack, two 16-byte stores: 16 consecutive output channels of one row per lane
    // (every lane issues both: the wait below counts on it; rows past the end are dropped)
    {
      const int64_t row = tile * kRwRows + 32 * wave + r32;
      unsigned pk[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) pk[i] = pack2<T>(acc[2 * i] + bq[2 * i], acc[2 * i + 1] + bq[2 * i + 1]);
      const uint32_t off = row < rows_out ? (uint32_t)row * 64u + 32u * q : 0xffffff00u;
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{pk[0], pk[1], pk[2], pk[3]}, rs_out, off, 0, 0);
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{pk[4], pk[5], pk[6], pk[7]}, rs_out, off + 16u, 0, 0);
    }
    // tile + 1 has landed (everything up to this tile's first operation has); every wave is past
    // its last read of this tile's buffers.  vmcnt in bits 3:0 and 15:14, LDS counter (bits 11:8) 0.
    __builtin_amdgcn_s_waitcnt(0x0070 | ((kOps - 1) & 15) | (((kOps - 1) >> 4) << 14));
    asm volatile("s_barrier" ::: "memory");
    p_a = p_b;
    p_b = p_c;
    p_c = p_d;
    p_d = __builtin_amdgcn_readfirstlane((int32_t)p_raw);
  };
  // whole rounds of the ring in the loop, the last one or two tiles after it: no path skips a
  // tile, so the compiler's own wait insertion sees the real order of loads and uses
  int64_t tile = t_begin;
  for (; tile + 3 <= t_end; tile += 3) {
    tile_body(std::integral_constant<int, 0>{}, tile);
    tile_body(std::integral_constant<int, 1>{}, tile + 1);
    tile_body(std::integral_constant<int, 2>{}, tile + 2);
  }
  if (tile < t_end) {
    tile_body(std::integral_constant<int, 0>{}, tile);
    if (tile + 1 < t_end) tile_body(std::integral_constant<int, 1>{}, tile + 1);
  }
  // The waits above COUNT operations, so every tile must issue all kOps of them - also the last
  // tiles of the range, whose list entries and list boundaries nobody reads any more: without a
  // reader the compiler drops those loads, the count of the tile comes out short and the wait
  // at its end no longer covers the rows of the tile after it.  These empty statements are
  // that reader.
#pragma unroll
  for (int b = 0; b < 3; ++b)
#pragma unroll
    for (int i = 0; i < kRowPieces; ++i) asm volatile("" ::"v"(ids[b][i]));
  asm volatile("" ::"s"(p_a), "s"(p_b), "s"(p_c), "s"(p_d));
  __builtin_amdgcn_s_waitcnt(0x0070);                            // loads past the range still write LDS
}

}  // namespace ocnn

using namespace ocnn;


extern "C" int ocnn_conv_gather_rw_supported(int dtype, int64_t rows_in, int K, int cin, int cout,
                                             int plan_max_distinct) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (!((cin == 64 && cout == 64) || (cin == 32 && cout == 32))) return 0;
  if (K != 27 && K != 9 && K != 8 && K != 3) return 0;
  if (plan_max_distinct < 0 || plan_max_distinct > kRwCap) return 0;
  if (rows_in < 0 || (int64_t)rows_in * cin * 2 > 0xfff00000ll) return 0;
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
                     urows, urows_bytes, (const T*)ws, (const T*)bias, (T*)out, rows_out, K, tiles, per);
}

template <typename T, int KK>
static void launch_rw32(const void* in, int64_t rows_in, const uint16_t* loc, const int32_t* uptr,
                        const int32_t* urows, uint32_t urows_bytes, int64_t rows_out, const void* ws,
                        const void* bias, void* out, int n_cu, hipStream_t st) {
  int64_t tiles = cdiv(rows_out, kRwRows);
  int64_t wgs = std::min<int64_t>(tiles, n_cu);
  int64_t per = cdiv(tiles, wgs);
  wgs = cdiv(tiles, per);
  hipLaunchKernelGGL((conv_gather_rw32_kernel<T, KK>), dim3((unsigned)wgs), dim3(256), 0, st, (const T*)in,
                     (uint32_t)(rows_in * 64), loc, (uint32_t)(tiles * kRwRows * KK * 2), uptr, urows,
                     urows_bytes, (const T*)ws, (const T*)bias, (T*)out, (uint32_t)(rows_out * 64), rows_out, tiles,
                     per);
}

template <typename T>
static int run_rw(const void* in, int64_t rows_in, const uint16_t* loc, const int32_t* uptr,
                  const int32_t* urows, int64_t plan_total, int64_t rows_out, int K, int cin, const void* w,
                  int w_transposed, int reverse, const void* bias, void* out, void* ws, hipStream_t st) {
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
  if (cin == 32) {
    hipLaunchKernelGGL(pack_weights_rw32_kernel<T>, dim3(cdiv((int64_t)K * 1024, 256)), dim3(256), 0, st,
                       (const T*)w, (T*)ws, K, w_transposed, reverse);
    if (K == 27) launch_rw32<T, 27>(in, rows_in, loc, uptr, urows, ub, rows_out, ws, bias, out, n_cu, st);
    else if (K == 9) launch_rw32<T, 9>(in, rows_in, loc, uptr, urows, ub, rows_out, ws, bias, out, n_cu, st);
    else if (K == 8) launch_rw32<T, 8>(in, rows_in, loc, uptr, urows, ub, rows_out, ws, bias, out, n_cu, st);
    else launch_rw32<T, 3>(in, rows_in, loc, uptr, urows, ub, rows_out, ws, bias, out, n_cu, st);
    return check_launch("conv_gather_rw32");
  }
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
                   ((int64_t)rows_out + 128) * cout * 2 < 0xfff00000ll &&
                   plan_total >= 0 && plan_total < (1ll << 29),
               "conv_gather_rw: rows out of range");
  if (rows_out == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("conv_gather_rw", loc, uptr, urows, w, out, workspace);
  OCNN_REQUIRE(rows_in == 0 || in, "conv_gather_rw: in is NULL");
  if (workspace_bytes < (int64_t)K * cin * cout * 2) {
    set_error("conv_gather_rw: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16)
    return run_rw<f16>(in, rows_in, loc, uptr, urows, plan_total, rows_out, K, cin, w, w_transposed, reverse_slots,
                       bias, out, workspace, st);
  return run_rw<bf16>(in, rows_in, loc, uptr, urows, plan_total, rows_out, K, cin, w, w_transposed, reverse_slots, bias,
                      out, workspace, st);
}

// ---------------------------------------------------------------------------------------
// Entry point that allocates nothing and takes no workspace.  The packed weights (what the
// workspace of ocnn_conv_gather_rw holds) go to a file-scope device array instead.  Its
// address on the current device is looked up once per device; host code never uses the
// array's name for anything else.  Every call on a GPU shares that GPU's array: calls that
// overlap on one GPU (two streams, two threads) race.  The pre-pass rewrites all K * cin *
// cout elements that the kernel reads, so nothing needs clearing between calls.
// ---------------------------------------------------------------------------------------
constexpr int64_t kRwScratchBytes = 27 * 64 * 64 * 2;          // the largest shape: 216 KiB
static __device__ __align__(256) unsigned char scratch[kRwScratchBytes];

constexpr int kRwMaxDevices = 64;
static void* g_rw_scratch_ptr[kRwMaxDevices];
static std::mutex g_rw_scratch_mutex;

static int rw_scratch_of_current_device(void** ptr) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kRwMaxDevices) {
    set_error("conv_gather_rw_static: cannot tell the current device");
    return OCNN_ERR_HIP;
  }
  std::lock_guard<std::mutex> lock(g_rw_scratch_mutex);
  if (g_rw_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("conv_gather_rw_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
      return OCNN_ERR_HIP;
    }
    g_rw_scratch_ptr[dev] = p;
  }
  *ptr = g_rw_scratch_ptr[dev];
  return OCNN_OK;
}

extern "C" int64_t ocnn_conv_gather_rw_static_max_weight_bytes(void) { return kRwScratchBytes; }

extern "C" int ocnn_conv_gather_rw_static(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                                          const int32_t* uptr, const int32_t* urows, int plan_max_distinct,
                                          int64_t plan_total, int64_t rows_out, int K, const void* w, int cin,
                                          int cout, int w_transposed, int reverse_slots, const void* bias,
                                          void* out, void* stream) {
  OCNN_REQUIRE(ocnn_conv_gather_rw_supported(dtype, rows_in, K, cin, cout, plan_max_distinct),
               "conv_gather_rw_static: shape not supported");
  OCNN_REQUIRE((int64_t)K * cin * cout * 2 <= kRwScratchBytes,
               "conv_gather_rw_static: %lld bytes of weights exceed the built-in buffer of %lld bytes",
               (long long)K * cin * cout * 2, (long long)kRwScratchBytes);
  OCNN_REQUIRE(rows_out >= 0 && plan_total >= 0, "conv_gather_rw_static: negative row count");
  if (rows_out == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("conv_gather_rw_static", loc, uptr, urows, w, out);
  OCNN_REQUIRE(rows_in == 0 || in, "conv_gather_rw_static: in is NULL");
  void* ws = nullptr;
  int rc = rw_scratch_of_current_device(&ws);
  if (rc != OCNN_OK) return rc;
  return ocnn_conv_gather_rw(dtype, in, rows_in, loc, uptr, urows, plan_max_distinct, plan_total, rows_out, K, w,
                             cin, cout, w_transposed, reverse_slots, bias, out, ws, kRwScratchBytes, stream);
}
