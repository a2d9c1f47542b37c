// Weight gradient for 32 x 32 channels and for multiples of 64 channels (in 64 x 64 blocks)
// on the tile plan of the neighbour table.
//
//   dW[k][a][b] = sum over table rows r of  x[table[r][k]][a] * g[r][b]
//
// Per 128-row tile the distinct x rows (through the plan), the g rows and the
// table positions are staged ONCE in LDS with asynchronous global->LDS loads,
// double buffered, so the loads of tile i + 1 run under the MFMAs of tile i.  A
// persistent workgroup (4 waves, one per SIMD) owns a range of tiles and a group
// of kernel slots; each wave keeps the 64 x 64 (or 32 x 64) fp32 sums of its slots
// in accumulator registers for the whole range (v_mfma_f32_32x32x16, M = x
// channels, N = g channels, reduction over 16 rows per instruction).  Both
// operands are read with the transposing LDS load, whose per-lane address does
// the gather of the x rows for free.  Per-range sums go to `partial` and are
// added in range order by a second kernel: no atomics, fixed summation order.
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "mma.hpp"
#include "reduce.hpp"

namespace ocnn {

constexpr int kWpRows = 128;   // rows per tile (the plan's tile size)
constexpr int kWpCap = 415;    // staged distinct rows per tile: with the zero row, 26 groups of 16
constexpr int kWpLoc = (kWpRows * 27 * 2 + 1023) / 1024 * 512;   // u16 per buffer, whole KiB
constexpr int kWpXHalf = (kWpCap + 1) * 32;   // elements of one channel half of the x rows (+ zero row)
constexpr int kWpGHalf = kWpRows * 32;

struct WpOps {
  u32x2 a[7][2];    // [unit][rows 0-3 / 4-7 of the lane's 8]
  u32x2 b[2][2];    // [g-channel half][rows]
};

// What the staging pieces of a tile need.  (Not a local class of the kernel template: the
// arguments of the global->LDS load builtin must not be type-dependent expressions.)
struct WpStage {
  uint32_t g_off;       // byte offset of the tile's first g row
  uint32_t loc_off;     // byte offset of the tile's table positions
  uint32_t list_off;    // byte offset of the list of the tile after it, per lane (or out of range)
  int groups;           // number of 16-row groups of distinct x rows of the tile
  const int32_t* su;    // list of this tile's distinct rows (LDS)
  int32_t* su_out;      // where the next list goes (LDS)
  char* sx;             // destination buffers (LDS)
  char* sg;
  char* sl;
};

// A workgroup sums a C x C block (C = 64 or 32) of the channel pairs; blockIdx.y picks
// the block when the layer has more channels (BLK; C = 64).  NFULL slots per wave with all
// C x channels, NHALF (0/1, C = 64 only) slot shared by two waves (one x-channel half each);
// GROUPS workgroups split the K slots.
//
// LDS layout: the two 32-channel halves of the staged rows live in separate arrays
// of 64-byte rows.  A transposing read of a 16-lane group touches 4 rows x 32 B, a
// half wave 4 rows x 64 B; at a 64-byte pitch four consecutive positions cover all
// 64 banks, and the second half is the first plus a constant.
template <typename T, int C, int KK, int NFULL, int NHALF, int GROUPS, bool BLK>
__global__ __launch_bounds__(256, 1) void conv_wgrad_planned_kernel(
    const T* __restrict__ x, uint32_t x_bytes, const T* __restrict__ g, uint32_t g_bytes,
    const uint16_t* __restrict__ loc, uint32_t loc_bytes, const int32_t* __restrict__ uptr,
    const int32_t* __restrict__ urows, uint32_t urows_bytes, int64_t tiles,
    int64_t tiles_per_split, int nsplit, int ca, int cb, float* __restrict__ partial) {
  constexpr int H = C / 32;                   // 32-channel halves of a row
  constexpr int NU = H * NFULL + NHALF;       // 32 x C accumulator units per wave
  constexpr int NS = NFULL + NHALF;           // distinct slots per wave
  constexpr int SPG = 4 * NFULL + 2 * NHALF;  // slots per group
  constexpr int NL = 2 * NS;                  // table look-ups per lane and step
  constexpr int NM = H * NU;                  // MFMAs per step
  constexpr int XH = kWpXHalf * 2, GH = kWpGHalf * 2;   // byte offsets of the second halves
  // C = 64: MFMAs between the position reads and their use
  constexpr int PF0 = H == 1 ? 1 : ((NM - NL) < 4 ? (NM - NL) : 4);
  constexpr int IP = (NL + 4 + PF0 - 1) / PF0;
  // C = 32: positions and g with the first MFMA, the x reads XP per MFMA from MFMA XS on
  constexpr int XS = NM > 2 ? 2 : NM - 1;
  constexpr int XP = (NL + (NM - XS) - 1) / (NM - XS);
  static_assert((H == 1 || H == 2) && NU <= 7 && PF0 >= 1 && (H == 2 || NHALF == 0), "unit layout");

  // one array per buffer, so that the compiler can tell the buffer being filled
  // from the one being read
  __shared__ __attribute__((aligned(16))) T s_x0[H * kWpXHalf];
  __shared__ __attribute__((aligned(16))) T s_x1[H * kWpXHalf];
  __shared__ __attribute__((aligned(16))) T s_g0[H * kWpGHalf];
  __shared__ __attribute__((aligned(16))) T s_g1[H * kWpGHalf];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc0[kWpLoc];
  __shared__ __attribute__((aligned(16))) uint16_t s_loc1[kWpLoc];
  // lists of distinct rows, from entry 4 on; entry 3 stays -1 ("the row before the first")
  __shared__ __attribute__((aligned(16))) int32_t s_u0[4 + 512];
  __shared__ __attribute__((aligned(16))) int32_t s_u1[4 + 512];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // workgroups of one tile range sit on the same XCD (they stage the same rows)
  const int bid = blockIdx.x;
  const int xcd = bid & 7, idx = bid >> 3;
  const int grp = idx % GROUPS;
  const int split = xcd * (nsplit >> 3) + idx / GROUPS;
  const int64_t t_begin = (int64_t)split * tiles_per_split;
  const int64_t t_end = min(tiles, t_begin + tiles_per_split);
  if (t_begin >= t_end) return;

  const int k0 = grp * SPG;
  const int slotF = k0 + NFULL * wave;                    // first full slot of this wave
  const int slotH = k0 + 4 * NFULL + (wave >> 1);         // the shared slot
  const int slotF_rd = min(slotF, KK - (NFULL > 0 ? NFULL : 1));   // padded slots read a valid column
  const int slotH_rd = min(slotH, KK - 1);
  const uint32_t ahH = (uint32_t)(wave & 1) * (uint32_t)XH;        // this wave's half of the shared slot

  // lane (i16, gq): rows 8 q + 4 h + i16 / 4 of a 16-row step, channels 16 (gq & 1) + 4 (i16 & 3) ..
  const int i16 = lane & 15, gq = lane >> 4, q = lane >> 5;
  const int rs = i16 >> 2;
  const uint32_t byte0 = 32u * (gq & 1) + 8u * (i16 & 3);
  const uint32_t lbF = (uint32_t)(slotF_rd * kWpRows + 8 * q + rs) * 2u;   // [slot][row] positions, 2 B each
  const uint32_t lbH = (uint32_t)(slotH_rd * kWpRows + 8 * q + rs) * 2u;
  // C = 32: a wave's slots can end inside its group of NFULL (K = 27: slots 21..27), so
  // every slot clamps on its own
  uint32_t lbS[H == 1 ? NFULL : 1];
  if constexpr (H == 1) {
#pragma unroll
    for (int sl = 0; sl < NFULL; ++sl)
      lbS[sl] = (uint32_t)(min(slotF + sl, KK - 1) * kWpRows + 8 * q + rs) * 2u;
  }
  uint32_t gad[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) gad[h] = (uint32_t)(8 * q + 4 * h + rs) * 64u + byte0;

  if (tid == 0) s_u0[3] = s_u1[3] = -1;     // position 0 is the zero row: it is staged from out of range

  const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, x_bytes);
  const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(g, g_bytes);
  const __amdgpu_buffer_rsrc_t rs_loc = make_rsrc(loc, loc_bytes);
  const __amdgpu_buffer_rsrc_t rs_u = make_rsrc(urows, urows_bytes);
  const __amdgpu_buffer_rsrc_t rs_p = make_rsrc(uptr, (uint32_t)(tiles + 1) * 4u);

  // ---- staging of one tile, cut into per-wave pieces `t` (one load instruction each, 1 KiB):
  //   NG pieces  g rows: 16 rows of one channel half
  //   2 pieces   table positions
  //   NX pieces  x rows: 16 distinct rows (ids in su) of one channel half
  //   1 piece    the list of distinct rows of the tile after (waves 0 and 1)
  // (C = 64: 4 + 2 + 13 + 1, a wave takes one half of every second 16-row group;
  //  C = 32: 2 + 2 + 7 + 1, a wave takes every fourth group.)
  // The pieces are branch-free: whatever lies past the end of a list, of the table or of
  // the tile range is an out-of-range offset (loads zeros) or row 0.  A wave has one
  // instruction stream for the MFMAs and everything else, so each instruction saved here
  // is MFMA issue time won.
  constexpr int NG = 2 * H, GST = 4 / H;                   // g pieces; 16-row groups between a wave's pieces
  constexpr int NX = ((kWpCap + 16) / 16 + GST - 1) / GST;
  constexpr int tL = NG, tX = NG + 2, tU = NG + 2 + NX, kPieces = tU + 1;
  static_assert(kPieces <= 20 && (kWpCap + 1) % 16 == 0, "five steps of four pieces stage a tile");
  constexpr int RSH = 5 + H;                               // log2 of the bytes of a C-channel row
  // a block of a wider layer: rows of ca (cb) channels, this block's 64 start at xb (gb)
  const int nbb = BLK ? (cb + C - 1) / C : 1;             // (channel counts are multiples of 32: the last block may be half)
  const int blk_a = BLK ? (int)blockIdx.y / nbb : 0, blk_b = BLK ? (int)blockIdx.y % nbb : 0;
  const uint32_t x_pitch = BLK ? (uint32_t)ca * 2u : (1u << RSH), g_pitch = BLK ? (uint32_t)cb * 2u : (1u << RSH);
  const uint32_t xb = (uint32_t)blk_a << RSH, gb = (uint32_t)blk_b << RSH;
  const int st_half = H == 2 ? (wave & 1) : 0, st_g16 = H == 2 ? (wave >> 1) : wave;
  const uint32_t st_xc = (uint32_t)st_half * 64u + (uint32_t)(lane & 3) * 16u;   // byte within a row
  const int st_pos = st_g16 * 16 + (lane >> 2);            // position / row of piece 0; piece j: + 16 GST j
  const uint32_t st_gc = (BLK ? (uint32_t)st_pos * g_pitch + gb : ((uint32_t)st_pos << RSH)) + st_xc;
  const uint32_t st_gstep = BLK ? 16u * GST * g_pitch : 4096u;   // 16 GST rows further
  auto make_stage = [&](int64_t tile, int U, int32_t list_first, int32_t list_len, const int32_t* su,
                        int32_t* su_out, T* sx, T* sg, uint16_t* sl) {
    WpStage st;
    const int64_t tc = min(tile, tiles - 1);              // past the range: any valid tile
    st.g_off = BLK ? (uint32_t)(tc * kWpRows) * g_pitch : (uint32_t)(tc * kWpRows) << RSH;
    st.loc_off = (uint32_t)(tc * kWpRows * KK * 2);
    const int e = wave * 256 + lane * 4;                   // the four list entries this lane brings in
    st.list_off = e < list_len ? (uint32_t)(list_first + e) * 4u : 0xffffff00u;
    st.groups = (U + 16) >> 4;                             // positions 0..U
    st.su = su; st.su_out = su_out; st.sx = (char*)sx; st.sg = (char*)sg; st.sl = (char*)sl;
    return st;
  };
  auto stage_id = [&](int t, const WpStage& st) -> int32_t {     // row id a lane needs for piece t
    return (t >= tX && t < tU) ? st.su[st_pos + 16 * GST * (t - tX) - 1] : 0;   // position p holds list entry p - 1
  };
  auto stage_piece = [&](int t, const WpStage& st, int32_t id) {
    if (t < NG) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs_g, (lds_ptr_t)(st.sg + (st_half * kWpGHalf + (st_g16 + GST * t) * 512) * 2), 16,
          st.g_off + st_gc + (uint32_t)t * st_gstep, 0, 0, 0);
    } else if (t < tX) {
      constexpr int nchunk = (kWpRows * KK * 2 + 1023) >> 10;
      if (4 * (t - tL) < nchunk) {
        const int c = min(wave + 4 * (t - tL), nchunk - 1);     // a spare wave repeats the last chunk
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_loc, (lds_ptr_t)(st.sl + c * 1024), 16,
                                                 st.loc_off + (uint32_t)c * 1024u + lane * 16u, 0, 0, 0);
      }
    } else if (t < tU) {
      if ((st_g16 + GST * (t - tX)) < st.groups)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs_x, (lds_ptr_t)(st.sx + (st_half * kWpXHalf + (st_g16 + GST * (t - tX)) * 512) * 2), 16,
          BLK ? (uint32_t)id * x_pitch + (xb + st_xc) : (((uint32_t)id << RSH) | st_xc), 0, 0, 0);
    } else if (wave < 2) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_u, (lds_ptr_t)(st.su_out + wave * 256), 16, st.list_off, 0,
                                               0, 0);
    }
  };

  f32x16 acc[NU][H];
#pragma unroll
  for (int u = 0; u < NU; ++u)
#pragma unroll
    for (int bh = 0; bh < H; ++bh)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[u][bh][r] = 0.f;

  WpOps ops[2];
  uint32_t pv[NL];       // positions (0 = empty) of the lane's two rows, per slot

  // ---- the pieces of one step's operand fetch ----
  auto pf_loc = [&](int j, const char* lcs, int sn) {       // j = 2 * slot + h
    const int sl = j >> 1, h = j & 1;
    uint32_t off;
    if constexpr (H == 1) off = lbS[sl] + (uint32_t)(sn * 32 + h * 8);
    else off = (sl < NFULL ? lbF + (uint32_t)(sl * kWpRows * 2) : lbH) + (uint32_t)(sn * 32 + h * 8);
    pv[j] = *(const uint16_t*)(lcs + off);
  };
  auto pf_g = [&](int j, const char* gs, int sn, WpOps& on) {   // j = 2 * bh + h
    const int h = j & 1, bh = j >> 1;
    on.b[bh][h] = Mma<T>::read_tr((const T*)(gs + gad[h] + (uint32_t)(bh * GH + sn * 1024)));
  };
  auto pf_x = [&](int j, const char* xs, WpOps& on) {            // j = 2 * slot + h
    const int sl = j >> 1, h = j & 1;
    const uint32_t ad = (pv[j] << 6) + byte0;                 // position 0 is the zero row
    if (sl < NFULL) {
      on.a[H * sl][h] = Mma<T>::read_tr((const T*)(xs + ad));
      if constexpr (H == 2) on.a[2 * sl + 1][h] = Mma<T>::read_tr((const T*)(xs + ad + (uint32_t)XH));
    } else {
      on.a[H * NFULL][h] = Mma<T>::read_tr((const T*)(xs + ad + ahH));
    }
  };
  auto mm = [&](int m, const WpOps& oc) {
    const int u = m / H, bh = m % H;
    const u32x4 av = u32x4{oc.a[u][0][0], oc.a[u][0][1], oc.a[u][1][0], oc.a[u][1][1]};
    const u32x4 bv = u32x4{oc.b[bh][0][0], oc.b[bh][0][1], oc.b[bh][1][0], oc.b[bh][1][1]};
    acc[u][bh] = Mma32<T>::run(av, bv, acc[u][bh]);
  };

  // One step: the MFMAs of 16 rows on `oc`; between them the operand fetch of the
  // following step (rows 16 sn.. of the buffers xs/gs/lcs) into `on`, and four staging
  // pieces t0..t0+3 of the next tile (t0 < 0: none).
  auto step = [&](const WpOps& oc, WpOps& on, const char* xs, const char* gs, const char* lcs, int sn,
                  int t0, const WpStage& sg) {
    int32_t ids[4] = {0, 0, 0, 0};
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      mm(m, oc);
      // operand fetch of the next step: table positions and g first, then the x reads
      // that depend on the positions, PF0 MFMAs later
      if constexpr (H == 2) {
        if (m < PF0) {
#pragma unroll
          for (int t = m * IP; t < (m + 1) * IP && t < NL + 4; ++t) {
            if (t < NL) pf_loc(t, lcs, sn);
            else pf_g(t - NL, gs, sn, on);
          }
        } else if (m - PF0 < NL) {
          pf_x(m - PF0, xs, on);
        }
      } else {
        if (m == 0) {
#pragma unroll
          for (int t = 0; t < NL; ++t) pf_loc(t, lcs, sn);
#pragma unroll
          for (int t = 0; t < 2; ++t) pf_g(t, gs, sn, on);
        }
        if (m >= XS) {
#pragma unroll
          for (int t = (m - XS) * XP; t < (m - XS + 1) * XP && t < NL; ++t) pf_x(t, xs, on);
        }
      }
      if (t0 >= 0) {
        if (m == 0) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (t0 + j < kPieces) ids[j] = stage_id(t0 + j, sg);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int mj = (j * NM) / 4 + 1 < NM ? (j * NM) / 4 + 1 : NM - 1;
          if (m == mj && t0 + j < kPieces) {
            stage_piece(t0 + j, sg, ids[j]);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // operand fetch of a tile's first step when there is no previous step to hide it under
  auto first_fetch = [&](const char* xs, const char* gs, const char* lcs, WpOps& on) {
#pragma unroll
    for (int t = 0; t < NL; ++t) pf_loc(t, lcs, 0);
#pragma unroll
    for (int t = 0; t < 2 * H; ++t) pf_g(t, gs, 0, on);
#pragma unroll
    for (int t = 0; t < NL; ++t) pf_x(t, xs, on);
  };

  // ---- prologue: first list, first tile, second list ----
  int32_t p_nxt = uptr[t_begin + 1];
  int32_t p_nx2 = uptr[min(t_begin + 2, tiles)];
  int32_t p_nx3 = uptr[min(t_begin + 3, tiles)];
  {
    const int32_t p_cur = uptr[t_begin];
    WpStage st = make_stage(t_begin, 0, p_cur, p_nxt - p_cur, s_u0 + 4, s_u0 + 4, s_x0, s_g0, s_loc0);
    stage_piece(tU, st, 0);                                // list of the first tile -> s_u0
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    st = make_stage(t_begin, p_nxt - p_cur, p_nxt, p_nx2 - p_nxt, s_u0 + 4, s_u1 + 4, s_x0, s_g0, s_loc0);
#pragma unroll
    for (int t = 0; t < kPieces; ++t) stage_piece(t, st, stage_id(t, st));     // also: list of the second tile
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    first_fetch((const char*)s_x0, (const char*)s_g0, (const char*)s_loc0, ops[0]);
  }

  // one tile out of buffer B; stages the next tile into buffer 1 - B meanwhile
  auto tile_body = [&](auto BC, int64_t tile) {
    constexpr int B = decltype(BC)::value;
    const char* xs = B ? (const char*)s_x1 : (const char*)s_x0;
    const char* gs = B ? (const char*)s_g1 : (const char*)s_g0;
    const char* lcs = B ? (const char*)s_loc1 : (const char*)s_loc0;
    // next tile -> the other buffers (its list is in the other s_u); list of the tile after
    // it -> this tile's s_u, which has been used up
    const WpStage sg = make_stage(tile + 1, p_nx2 - p_nxt, p_nx2, p_nx3 - p_nx2, B ? s_u0 + 4 : s_u1 + 4,
                                  B ? s_u1 + 4 : s_u0 + 4, B ? s_x0 : s_x1, B ? s_g0 : s_g1,
                                  B ? s_loc0 : s_loc1);
    // list boundary four tiles ahead, as a vector load: a scalar load would share its counter
    // with the LDS reads and force them to drain where it is used
    const uint32_t p_raw = __builtin_amdgcn_raw_buffer_load_b32(
        rs_p, (uint32_t)min(tile + 4, tiles) * 4u, 0, 0);
    p_nxt = p_nx2;
    p_nx2 = p_nx3;
#pragma unroll
    for (int s = 0; s < 7; ++s)
      step(ops[s & 1], ops[(s + 1) & 1], xs, gs, lcs, s + 1, s < 5 ? 4 * s : -1, sg);
    // The next tile has landed: own loads, then everyone's.  The LDS reads in flight belong
    // to this tile's buffers and need not drain, so neither barrier is a __syncthreads().
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    p_nx3 = __builtin_amdgcn_readfirstlane((int32_t)p_raw);
    // last step, with the first operands of the next tile fetched from the other buffer
    step(ops[1], ops[0], sg.sx, sg.sg, sg.sl, 0, -1, sg);
    asm volatile("s_barrier" ::: "memory");  // buffer B may be overwritten now: its last reads fed this step
  };

  for (int64_t tile = t_begin; tile < t_end; tile += 2) {
    tile_body(std::integral_constant<int, 0>{}, tile);
    if (tile + 1 < t_end) tile_body(std::integral_constant<int, 1>{}, tile + 1);
  }

  // ---- per-range sums -> partial[split][slot][a][b] ----
  const int b32 = lane & 31;
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int slot = u < H * NFULL ? slotF + u / H : slotH;
    const int ah = u < H * NFULL ? u % H : (wave & 1);
    if (slot >= KK) continue;
    const int ldb = BLK ? cb : C;
    float* dst = BLK ? partial + (((int64_t)split * KK + slot) * ca + blk_a * C) * cb + blk_b * C
                     : partial + ((int64_t)split * KK + slot) * (C * C);
    // a half block at the end of the channels: what the staging loads brought in beyond a
    // row only reached sums that are not written
    if (BLK && blk_a * C + 32 * ah >= ca) continue;
#pragma unroll
    for (int bh = 0; bh < H; ++bh) {
      if (BLK && blk_b * C + 32 * bh >= cb) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int a = 32 * ah + 8 * (r >> 2) + 4 * q + (r & 3);
        dst[a * ldb + 32 * bh + b32] = acc[u][bh][r];
      }
    }
  }
}

}  // namespace ocnn

using namespace ocnn;


static int wp_splits(int K, int ca, int cb, int n_cu) {
  const int groups = (K == 27 && ca >= 64) ? 2 : 1;
  const int blocks = ca >= 64 ? ((ca + 63) / 64) * ((cb + 63) / 64) : 1;
  int s = std::max(8, n_cu / (groups * blocks) / 8 * 8);      // a multiple of 8: ranges are dealt to the XCDs
  return std::min(s, 256);
}

static int wp_cu_count() {
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
    n_cu = prop.multiProcessorCount;
  }
  return n_cu;
}

extern "C" int ocnn_conv_wgrad_planned_supported(int dtype, int64_t rows_x, int64_t rows, int K, int ca,
                                                 int cb, int plan_max_distinct) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16 && dtype != OCNN_F32) return 0;   // (fp32: as bf16 pieces)
  if (!(ca == 32 && cb == 32) && !(ca >= 64 && cb >= 64 && ca % 32 == 0 && cb % 32 == 0 && ca <= 1024 && cb <= 1024))
    return 0;
  if (K != 27 && K != 9 && K != 8 && K != 3) return 0;
  if (plan_max_distinct < 0 || plan_max_distinct > kWpCap) return 0;
  if (rows_x < 0 || rows < 0) return 0;
  if ((int64_t)rows_x * ca * 2 > 0xfff00000ll || ((int64_t)rows + kWpRows) * cb * 2 > 0xfff00000ll) return 0;
  return 1;
}

extern "C" int64_t ocnn_conv_wgrad_planned_workspace_bytes(int K, int ca, int cb) {
  const int n_cu = wp_cu_count();
  const int64_t splits = n_cu > 0 ? wp_splits(K, ca, cb, n_cu) : 256;
  return align_up(splits * K * ca * cb * 4, 256);
}

// fp32: three sets of per-range sums (hi_x hi_g, hi_x lo_g, lo_x hi_g) after the bf16 pieces
// of both tensors
extern "C" int64_t ocnn_conv_wgrad_planned_workspace_bytes_for(int dtype, int64_t rows_x, int64_t rows, int K,
                                                               int ca, int cb) {
  const int64_t sums = ocnn_conv_wgrad_planned_workspace_bytes(K, ca, cb);
  if (dtype != OCNN_F32 || rows_x < 0 || rows < 0) return sums;
  return 2 * align_up(rows_x * ca * 2, 256) + 2 * align_up(rows * cb * 2, 256) + 3 * sums;
}

template <typename T, int C, int KK, int NFULL, int NHALF, int GROUPS>
static void launch_wp(const void* x, int64_t rows_x, const void* g, const uint16_t* loc, const int32_t* uptr,
                      const int32_t* urows, int64_t plan_total, int64_t rows, int ca, int cb, int nsplit,
                      int64_t per, float* partial, hipStream_t st) {
  const int64_t tiles = cdiv(rows, kWpRows);
  const uint32_t xb = (uint32_t)(rows_x * ca * 2), gb = (uint32_t)(rows * cb * 2);
  const uint32_t lb = (uint32_t)(tiles * kWpRows * KK * 2), ub = (uint32_t)(plan_total * 4);
  if (ca == C && cb == C)
    hipLaunchKernelGGL((conv_wgrad_planned_kernel<T, C, KK, NFULL, NHALF, GROUPS, false>), dim3(nsplit * GROUPS),
                       dim3(256), 0, st, (const T*)x, xb, (const T*)g, gb, loc, lb, uptr, urows, ub, tiles, per,
                       nsplit, ca, cb, partial);
  else if constexpr (C == 64)
    hipLaunchKernelGGL((conv_wgrad_planned_kernel<T, C, KK, NFULL, NHALF, GROUPS, true>),
                       dim3(nsplit * GROUPS, ((ca + C - 1) / C) * ((cb + C - 1) / C)), dim3(256), 0, st, (const T*)x, xb, (const T*)g,
                       gb, loc, lb, uptr, urows, ub, tiles, per, nsplit, ca, cb, partial);
}

// the launches of one pass over the plan: per-range sums of x^T g into `partial`
template <typename T>
static void launch_wp_pass(const void* x, int64_t rows_x, const void* g, const uint16_t* loc, const int32_t* uptr,
                           const int32_t* urows, int64_t plan_total, int64_t rows, int K, int ca, int cb,
                           int nsplit, int64_t per, float* partial, hipStream_t st) {
#define OCNN_WP_LAUNCH(CC, KK, NF, NH, GR) \
  launch_wp<T, CC, KK, NF, NH, GR>(x, rows_x, g, loc, uptr, urows, plan_total, rows, ca, cb, nsplit, per, partial, st)
  if (ca >= 64) {
    if (K == 27) OCNN_WP_LAUNCH(64, 27, 3, 1, 2);
    else if (K == 9) OCNN_WP_LAUNCH(64, 9, 2, 1, 1);
    else if (K == 8) OCNN_WP_LAUNCH(64, 8, 2, 0, 1);
    else OCNN_WP_LAUNCH(64, 3, 1, 0, 1);
  } else {
    if (K == 27) OCNN_WP_LAUNCH(32, 27, 7, 0, 1);
    else if (K == 9) OCNN_WP_LAUNCH(32, 9, 3, 0, 1);
    else if (K == 8) OCNN_WP_LAUNCH(32, 8, 2, 0, 1);
    else OCNN_WP_LAUNCH(32, 3, 1, 0, 1);
  }
#undef OCNN_WP_LAUNCH
}

// T: the type of x, g and gw (float: x and g go through the kernels as two bf16 pieces each,
// three passes into three sets of sums, one reduction over all of them)
template <typename T>
static int run_wp(const void* x, int64_t rows_x, const void* g, const uint16_t* loc, const int32_t* uptr,
                  const int32_t* urows, int64_t plan_total, int64_t rows, int K, int ca, int cb,
                  int out_transposed, void* gw, void* ws, int64_t ws_bytes, hipStream_t st) {
  constexpr bool kPieces = std::is_same<T, float>::value;
  const int n_cu = wp_cu_count();
  if (n_cu <= 0) {
    set_error("conv_wgrad_planned: cannot query the device");
    return OCNN_ERR_HIP;
  }
  const int nsplit = wp_splits(K, ca, cb, n_cu);
  const int64_t tiles = cdiv(rows, kWpRows);
  const int64_t per = std::max<int64_t>(1, cdiv(tiles, nsplit));
  const int used = (int)cdiv(tiles, per);                 // ranges that hold tiles
  const int64_t set = (int64_t)used * K * ca * cb;         // floats of one set of sums
  const int64_t xb = kPieces ? align_up(rows_x * ca * 2, 256) : 0, gb = kPieces ? align_up(rows * cb * 2, 256) : 0;
  if (ws_bytes < 2 * xb + 2 * gb + (kPieces ? 3 : 1) * set * 4) {
    set_error("conv_wgrad_planned: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  float* partial = (float*)((char*)ws + 2 * xb + 2 * gb);
  if constexpr (kPieces) {
    if (rows > 0) {
      bf16* xh = (bf16*)ws;
      bf16* xl = (bf16*)((char*)ws + xb);
      bf16* gh = (bf16*)((char*)ws + 2 * xb);
      bf16* gl = (bf16*)((char*)ws + 2 * xb + gb);
      if (rows_x > 0)
        hipLaunchKernelGGL(split2_kernel, dim3((unsigned)cdiv(rows_x * ca, 256)), dim3(256), 0, st, (const float*)x,
                           rows_x * ca, xh, xl);
      hipLaunchKernelGGL(split2_kernel, dim3((unsigned)cdiv(rows * cb, 256)), dim3(256), 0, st, (const float*)g,
                         rows * cb, gh, gl);
      const bf16* xs[3] = {xh, xh, xl};
      const bf16* gs[3] = {gh, gl, gh};
      for (int i = 0; i < 3; ++i)
        launch_wp_pass<bf16>(xs[i], rows_x, gs[i], loc, uptr, urows, plan_total, rows, K, ca, cb, nsplit, per,
                             partial + i * set, st);
    }
    launch_wgrad_reduce<float>(partial, rows > 0 ? 3 * used : 0, K, ca, cb, out_transposed, (float*)gw, st);
  } else {
    if (rows > 0)
      launch_wp_pass<T>(x, rows_x, g, loc, uptr, urows, plan_total, rows, K, ca, cb, nsplit, per, partial, st);
    launch_wgrad_reduce<T>(partial, rows > 0 ? used : 0, K, ca, cb, out_transposed, (T*)gw, st);
  }
  return check_launch("conv_wgrad_planned");
}

extern "C" int ocnn_conv_wgrad_planned(int dtype, const void* x, int64_t rows_x, const void* g,
                                       const uint16_t* loc, const int32_t* uptr, const int32_t* urows,
                                       int plan_max_distinct, int64_t plan_total, int64_t rows, int K,
                                       int ca, int cb, int out_transposed, void* gw, void* workspace,
                                       int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(ocnn_conv_wgrad_planned_supported(dtype, rows_x, rows, K, ca, cb, plan_max_distinct),
               "conv_wgrad_planned: shape not supported");
  OCNN_REQUIRE(rows >= 0 && (int64_t)rows * K * 2 < 0xfff00000ll && plan_total >= 0 &&
                   plan_total < (1ll << 29),
               "conv_wgrad_planned: rows out of range");
  OCNN_REQUIRE_PTRS("conv_wgrad_planned", gw, workspace);
  OCNN_REQUIRE(rows == 0 || (g && loc && uptr && urows && (rows_x == 0 || x)),
               "conv_wgrad_planned: a required pointer is NULL (of x, g, loc, uptr, urows)");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F32)
    return run_wp<float>(x, rows_x, g, loc, uptr, urows, plan_total, rows, K, ca, cb, out_transposed, gw, workspace,
                         workspace_bytes, st);
  if (dtype == OCNN_F16)
    return run_wp<f16>(x, rows_x, g, loc, uptr, urows, plan_total, rows, K, ca, cb, out_transposed, gw, workspace,
                       workspace_bytes, st);
  return run_wp<bf16>(x, rows_x, g, loc, uptr, urows, plan_total, rows, K, ca, cb, out_transposed, gw, workspace,
                      workspace_bytes, st);
}
