// Dense rows (one-slot identity table) with everything that is reused kept in registers:
// the form a 2x2x2 stride-2 layer over all nodes takes on the (parents, 8 C) view of its
// children.  These GEMMs are HBM-bound (about 100 flop per byte), so each tensor must cross
// L2 -> CU once:
//   * out = in W (+ bias): persistent workgroups keep their slice of W in VGPRs (wave w: all
//     input channels x its 32 MB output channels) and stream 64-row tiles through a ring of
//     two to four buffers in LDS;
//   * dW = in^T g: persistent workgroups keep a 512 x 128 (or 256 x 256, 128 x 512) block of
//     fp32 sums in accumulator registers (256 per lane; smaller layers fill a part of one
//     block, the rest is staged as zeros: the pass is bound by HBM) and stream 32-row tiles of both
//     operands through a ring of three LDS buffers; per-range sums go to the split reduction
//     (fixed order, no atomics).
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "mma.hpp"
#include "reduce.hpp"

namespace ocnn {

// (Not in the kernel templates: the arguments of the global->LDS load builtin must not be
// type-dependent expressions.)
static __device__ __forceinline__ void dr_dma16(__amdgpu_buffer_rsrc_t rs, char* dst, uint32_t off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)dst, 16, off, 0, 0, 0);
}

// ---------------------------------------------------------------------------------------
// out = in W.  Packed weights: [64-channel chunk cc][32 output channels cg][k-step s][lane][8]
// (the output channels of a block permuted so that the two lanes of a row hold adjacent
// 16-byte pieces).  LDS: [chunk][row][128 B],
// 16-byte chunk c of row r at c ^ ((r >> 1) & 7).
// ---------------------------------------------------------------------------------------
template <typename T, int NKS, int MB>
__global__ __launch_bounds__(256, 1) void conv_dense_rw_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const int32_t* __restrict__ row_index, const T* __restrict__ wpk,
    const T* __restrict__ bias, T* __restrict__ out, uint32_t out_bytes, const int32_t* __restrict__ out_index,
    int64_t rows, int cout, int64_t tiles, int64_t tiles_per_wg) {
  constexpr int RB = 2, RT = 32 * RB, NCC = NKS / 4, CIN = 16 * NKS;
  constexpr int BUF = NCC * RT * 128;
  constexpr int NBUF = NCC >= 8 ? 2 : 4;                           // tiles resident in LDS
  extern __shared__ __attribute__((aligned(16))) char s_dyn[];     // NBUF buffers
  __shared__ __attribute__((aligned(16))) float s_bias[128 * MB];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 5, r32 = lane & 31;
  const int64_t t_begin = (int64_t)blockIdx.x * tiles_per_wg;
  const int64_t t_end = min(tiles, t_begin + tiles_per_wg);
  if (t_begin >= t_end) return;
  const int ncg = cout >> 5;
  const int cg0 = ((int)blockIdx.y * 4 + wave) * MB;

  // ---- this wave's weights -> registers, once ----
  u32x4 wreg[NKS][MB];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      wreg[ks][mb] = *(const u32x4*)(wpk + ((int64_t)(((ks >> 2) * ncg + cg0 + mb) * 4 + (ks & 3)) * 64 + lane) * 8);

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t rs_out = make_rsrc(out, out_bytes);
  const int rl = lane >> 3;
  // Output row r goes to row out_index[r] of `out` when an index is given (the compact rows of the
  // non-empty nodes written straight into a tensor over all nodes): one entry per row block and
  // lane, loaded NBUF - 1 tiles before its tile is stored, in registers taken in turn.
  const bool scattered = out_index != nullptr;
  const __amdgpu_buffer_rsrc_t rs_oidx = make_rsrc(out_index, scattered ? (uint32_t)(rows * 4) : 0u);
  struct Odx { int32_t r[RB]; };
  auto load_out_index = [&](int64_t tile) {
    Odx x;
    const uint32_t row0 = (uint32_t)min(tile, tiles) * RT;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
      x.r[rb] = (int32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_oidx, (row0 + 32 * rb + r32) * 4u, 0, 0);
    return x;
  };
  // Row r of the operand is row row_index[r] of `in` when an index is given (the compact rows of
  // the non-empty nodes read straight from the tensor over all nodes).  A lane stages the rows
  // 8 wave + rl and 8 (wave + 4) + rl of a tile: two index entries per tile, loaded IDXD tiles
  // before the tile is staged (without an index the loads point out of range and cost nothing;
  // they are issued all the same, the waits below count operations).
  const bool indexed = row_index != nullptr;
  const __amdgpu_buffer_rsrc_t rs_idx = make_rsrc(row_index, indexed ? (uint32_t)(rows * 4) : 0u);
  struct Idx { int32_t r[2]; };
  auto load_index = [&](int64_t tile) {
    Idx x;
    const uint32_t row0 = (uint32_t)min(tile, tiles) * RT;
#pragma unroll
    for (int h = 0; h < 2; ++h)
      x.r[h] = (int32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_idx, (row0 + 8 * (wave + 4 * h) + rl) * 4u, 0, 0);
    return x;
  };
  auto stage = [&](int64_t tile, char* buf, const Idx& x) {
    const uint32_t row0 = (uint32_t)min(tile, tiles) * RT;        // past the table: out of range, zeros
#pragma unroll
    for (int j = 0; j < NCC * 2; ++j) {                           // NCC * 8 pieces of 1 KiB, 4 waves
      const int i = wave + 4 * j;
      const int cc = i >> 3, g = i & 7;
      const uint32_t swz = (uint32_t)((4 * g + (lane >> 4)) & 7);
      // (with an index, rows past the end read entry 0 = some row: their results are dropped)
      const uint32_t src = indexed ? (uint32_t)x.r[j & 1] : row0 + 8 * g + rl;
      dr_dma16(rs_in, buf + (cc * RT + 8 * g) * 128,
               src * (uint32_t)(CIN * 2) + (uint32_t)cc * 128u + (((uint32_t)(lane & 7) ^ swz) << 4));
    }
  };
  // B operand of k-step ks, row block rb: 16 bytes of row 32 rb + r32
  uint32_t pvs[RB][4];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint32_t l = (uint32_t)(32 * rb + r32);
      pvs[rb][s] = (l << 7) | ((((l << 3) & 0x70u) ^ ((uint32_t)q << 4)) ^ ((uint32_t)s << 5));
    }

  // ---- ring of NBUF tiles: tile i is multiplied while i + 1 .. i + NBUF - 1 are in flight ----
  // Vector memory operations complete in issue order, so "tile i + 1 has landed" is a count of
  // the operations issued after its loads: per tile P loads and NST stores, always exactly
  // (tiles past the range load zeros or rows of another range; rows past the end are stored
  // out of range and dropped).  NST dropped stores per prologue tile make the count right from
  // the first tile on.
  constexpr int P = NCC * 2 + 2 + RB, NST = RB * MB * 2;            // a tile's loads: its pieces, two + RB index entries
  // (vmcnt is a 6-bit counter; a smaller count only waits for more)
  constexpr int kWait = (NBUF - 2) * P + (NBUF - 1) * NST < 63 ? (NBUF - 2) * P + (NBUF - 1) * NST : 63;
  // s_waitcnt vmcnt(kWait) lgkmcnt(0) as an instruction of its own (vmcnt in bits 3:0 and 15:14,
  // lgkmcnt in bits 11:8), which the compiler's wait insertion takes into account
  constexpr int kWaitImm = 0x0070 | (kWait & 15) | ((kWait >> 4) << 14);
  // Index entries loaded with the operations of tile i have landed when tile i + NBUF - 2 ends:
  // they are loaded IDXD = 2 NBUF - 2 tiles ahead of their tile and used NBUF - 1 tiles later
  constexpr int IDXD = 2 * NBUF - 2;
  Idx iq[NBUF - 1];                                                // iq[0]: of the tile staged next
#pragma unroll
  for (int v = 0; v < NBUF - 1; ++v) {
    const Idx x = load_index(t_begin + v);
    stage(t_begin + v, s_dyn + v * BUF, x);
#pragma unroll
    for (int j = 0; j < NST; ++j)
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{0u, 0u, 0u, 0u}, rs_out, 0xfffffff0u, 0, 0);
  }
#pragma unroll
  for (int v = 0; v < NBUF - 1; ++v) iq[v] = load_index(t_begin + NBUF - 1 + v);
  Odx oq[NBUF - 1];                                                // oq[0]: of the tile stored next
#pragma unroll
  for (int v = 0; v < NBUF - 1; ++v) oq[v] = load_out_index(t_begin + v);
  for (int i = tid; i < 128 * MB; i += 256)
    s_bias[i] = bias ? to_f32(bias[(int)blockIdx.y * 128 * MB + i]) : 0.f;
  __builtin_amdgcn_s_waitcnt(0x0070);
  __syncthreads();

  int slot = 0;
  // one tile; U: which of the NBUF - 1 index registers it consumes and refills (the registers are
  // taken in turn and never copied: a copy would wait for the load of the tile before)
  auto tile_step = [&](auto UC, int64_t tile) {
    constexpr int U = decltype(UC)::value;
    const char* cur = s_dyn + slot * BUF;
    {
      const int sn = slot == 0 ? NBUF - 1 : slot - 1;              // the buffer of the tile before
      stage(tile + NBUF - 1, s_dyn + sn * BUF, iq[U]);
      iq[U] = load_index(tile + IDXD);
    }
    f32x16 acc[RB][MB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rb][mb][r] = 0.f;
    constexpr int PD = 3;                                         // k-steps a read runs ahead
    u32x4 Bb[4][RB];
    auto read_b = [&](int ks, u32x4 (&b)[RB]) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) b[rb] = *(const u32x4*)(cur + (ks >> 2) * (RT * 128) + pvs[rb][ks & 3]);
    };
#pragma unroll
    for (int ks = 0; ks < PD && ks < NKS; ++ks) read_b(ks, Bb[ks & 3]);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (ks + PD < NKS) read_b(ks + PD, Bb[(ks + PD) & 3]);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = Mma32<T>::run(wreg[ks][mb], Bb[ks & 3][rb], acc[rb][mb]);
      __builtin_amdgcn_sched_barrier(0);
    }
    // a lane holds the output channels 8 q .. 8 q + 7 and 16 + 8 q .. of a row per M tile: the
    // two lanes of a row write 32 contiguous bytes per store
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int cl = 32 * (wave * MB + mb) + 8 * q;               // channel within the workgroup's block
      const f32x4* b4 = (const f32x4*)(&s_bias[cl]);
      const f32x4 bv[4] = {b4[0], b4[1], b4[4], b4[5]};
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int64_t row = tile * RT + 32 * rb + r32;
        // (with an index, rows past the end have no entry: out of range, dropped like the others)
        const uint32_t orow = scattered ? (uint32_t)oq[U].r[rb] : (uint32_t)row;
        const uint32_t off = scattered && row >= rows
                                 ? 0xffffff00u                     // (+ 32 for the second store stays out of range)
                                 : (orow * (uint32_t)cout + (uint32_t)((int)blockIdx.y * 128 * MB + cl)) * 2u;
        unsigned pk[8];
#pragma unroll
        for (int r = 0; r < 8; ++r)
          pk[r] = pack2<T>(acc[rb][mb][2 * r] + bv[r >> 1][(2 * r) & 3], acc[rb][mb][2 * r + 1] + bv[r >> 1][(2 * r + 1) & 3]);
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{pk[0], pk[1], pk[2], pk[3]}, rs_out, off, 0, 0);
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{pk[4], pk[5], pk[6], pk[7]}, rs_out, off + 32u, 0, 0);
      }
    }
    oq[U] = load_out_index(tile + NBUF - 1);
    // the next tile has landed; every wave is done with this one
    __builtin_amdgcn_sched_barrier(0);
    // (a bare barrier: __syncthreads() would wait for every load in flight, the ring's included)
    __builtin_amdgcn_s_waitcnt(kWaitImm);
    asm volatile("s_barrier" ::: "memory");
    slot = slot == NBUF - 1 ? 0 : slot + 1;
  };
  // whole rounds of the index registers in the loop, the rest after it (no path skips a tile, so
  // the compiler's wait insertion sees the real order of loads and uses)
  int64_t tile = t_begin;
  if constexpr (NBUF == 4) {
    for (; tile + 3 <= t_end; tile += 3) {
      tile_step(std::integral_constant<int, 0>{}, tile);
      tile_step(std::integral_constant<int, 1>{}, tile + 1);
      tile_step(std::integral_constant<int, 2>{}, tile + 2);
    }
    if (tile < t_end) {
      tile_step(std::integral_constant<int, 0>{}, tile);
      if (tile + 1 < t_end) tile_step(std::integral_constant<int, 1>{}, tile + 1);
    }
  } else {
    static_assert(NBUF == 2 || NBUF == 4, "index registers are taken in turn");
    for (; tile < t_end; ++tile) tile_step(std::integral_constant<int, 0>{}, tile);
  }
  // The waits count operations: the index entries loaded by the last tiles of the range have no
  // reader, and without one the compiler drops those loads and a tile's count comes out short.
  // These empty statements are that reader.
#pragma unroll
  for (int v = 0; v < NBUF - 1; ++v) {
    asm volatile("" ::"v"(iq[v].r[0]), "v"(iq[v].r[1]));
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) asm volatile("" ::"v"(oq[v].r[rb]));
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                 // loads past the range still write LDS
}

// ---------------------------------------------------------------------------------------
// dW = x^T g.  A workgroup sums a block of 128 WA x 512 / WA channel pairs (WA = 4, 2, 1
// waves along the x channels); a wave 128 x 128 of it (4 x 4 accumulators of 32 x 32).
// LDS per 32-row tile: [64-channel group][row][128 B], x groups first; the 64-byte halves
// of the rows 2, 3 (mod 4) are swapped, so that the four rows of a transposing read fall
// on different banks.  Both operands are read with ds_read_b64_tr_b16.
// ---------------------------------------------------------------------------------------
// (Blocks at the edges multiply the zeros staged past the channels like everything else:
// skipping those 32 x 32 pieces with wave-uniform branches made the kernel slower.)
template <typename T, int WA>
__global__ __launch_bounds__(256, 1) void conv_dense_wgrad_rw_kernel(
    const T* __restrict__ x, uint32_t x_bytes, const int32_t* __restrict__ x_index, const T* __restrict__ g,
    uint32_t g_bytes, const int32_t* __restrict__ g_index, int64_t rows, int ca, int cb, int64_t tiles,
    int64_t tiles_per_split, float* __restrict__ partial) {
  constexpr int WB = 4 / WA;
  constexpr int GA = 2 * WA, GB = 2 * WB, NG = GA + GB;            // 64-channel groups of a tile
  constexpr int RT = 32, TILE = NG * RT * 128;                     // 40 KiB (32 KiB at WA = 2)
  constexpr int PW = NG * (RT / 8) / 4;                            // staging pieces per wave and tile
  // ring of three tiles: three arrays, not thirds of one, so that the compiler knows that the
  // reads of a tile cannot meet the loads in flight into the other two and does not wait for them
  __shared__ __attribute__((aligned(16))) char s_t0[TILE];
  __shared__ __attribute__((aligned(16))) char s_t1[TILE];
  __shared__ __attribute__((aligned(16))) char s_t2[TILE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wa = wave / WB, wb = wave % WB;
  const int nbb = (cb + 128 * WB - 1) / (128 * WB);   // blocks at the edges may hold fewer channels
  const int blk_a = (int)blockIdx.y / nbb, blk_b = (int)blockIdx.y % nbb;
  const int64_t t_begin = (int64_t)blockIdx.x * tiles_per_split;
  const int64_t t_end = min(tiles, t_begin + tiles_per_split);
  if (t_begin >= t_end) return;

  const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, x_bytes);
  const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(g, g_bytes);
  const uint32_t xp = (uint32_t)ca * 2u, gp = (uint32_t)cb * 2u;
  const int rl = lane >> 3;
  // source chunk of the lane: its LDS chunk, with the halves swapped for rows 2, 3 (mod 4)
  const uint32_t sc = (((uint32_t)(lane & 7) ^ (uint32_t)(4 * ((rl >> 1) & 1))) << 4);
  // Row r of an operand is row index[r] of its tensor when an index is given (the compact rows
  // of the non-empty nodes read straight from a tensor over all nodes).  A lane stages row
  // 8 wave + rl of a tile for every channel group: one index entry per operand and tile, loaded
  // four tiles ahead (without an index the loads point out of range and cost nothing; they are
  // issued all the same, the waits count operations).
  const bool x_indexed = x_index != nullptr, g_indexed = g_index != nullptr;
  const __amdgpu_buffer_rsrc_t rs_xi = make_rsrc(x_index, x_indexed ? (uint32_t)(rows * 4) : 0u);
  const __amdgpu_buffer_rsrc_t rs_gi = make_rsrc(g_index, g_indexed ? (uint32_t)(rows * 4) : 0u);
  struct Idx { int32_t x, g; };
  auto load_index = [&](int64_t tile) {
    const uint32_t row = (uint32_t)min(tile, tiles) * RT + 8 * wave + rl;
    Idx r;
    r.x = (int32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_xi, row * 4u, 0, 0);
    r.g = (int32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_gi, row * 4u, 0, 0);
    return r;
  };
  auto stage = [&](int64_t tile, char* buf, const Idx& ix) {       // every wave issues exactly PW loads
    const uint32_t row0 = (uint32_t)min(tile, tiles) * RT;        // past the range: past the rows, zeros
    const uint32_t row = row0 + 8 * wave + rl;                    // (piece i = wave + 4 j: row group i % 4 = wave)
    const bool live = (int64_t)row < rows;                        // an indexed row past the end must read zeros too
    const uint32_t xrow = x_indexed ? (uint32_t)ix.x : row, grow = g_indexed ? (uint32_t)ix.g : row;
#pragma unroll
    for (int j = 0; j < PW; ++j) {
      const int i = wave + 4 * j;
      const int grp = i >> 2, rg = i & 3;
      char* dst = buf + (grp * RT + 8 * rg) * 128;
      // channels past the end of a row: an offset past the buffer, which reads as zeros
      if (grp < GA) {
        const uint32_t cbyte = (uint32_t)((blk_a * GA + grp) * 128) + sc;
        dr_dma16(rs_x, dst, cbyte < xp && live ? xrow * xp + cbyte : 0xffffff00u);
      } else {
        const uint32_t cbyte = (uint32_t)((blk_b * GB + grp - GA) * 128) + sc;
        dr_dma16(rs_g, dst, cbyte < gp && live ? grow * gp + cbyte : 0xffffff00u);
      }
    }
  };

  f32x16 acc[4][4];
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.f;

  // lane (i16, gq): rows 8 q + 4 h + i16 / 4 of a 16-row step, channels 16 (gq & 1) + 4 (i16 & 3) ..
  const int i16 = lane & 15, gq = lane >> 4, q = lane >> 5, rs = i16 >> 2;
  const uint32_t byte0 = 32u * (gq & 1) + 8u * (i16 & 3);
  const uint32_t rowb = (uint32_t)(8 * q + rs) * 128u + byte0;
  const uint32_t hsw = 64u * ((rs >> 1) & 1);                      // where the first half of this row lives
  const uint32_t xe = rowb + hsw + (uint32_t)(2 * wa) * (RT * 128), xo = rowb + (64u - hsw) + (uint32_t)(2 * wa) * (RT * 128);
  const uint32_t ge = rowb + hsw + (uint32_t)(GA + 2 * wb) * (RT * 128), go = rowb + (64u - hsw) + (uint32_t)(GA + 2 * wb) * (RT * 128);

  const int a_base = blk_a * 128 * WA + 128 * wa, b_base = blk_b * 128 * WB + 128 * wb;

  struct Ops { u32x2 a[4][2], b[4][2]; };
  auto fetch = [&](const char* buf, int sn, Ops& o) {
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t off = (uint32_t)((m >> 1) * (RT * 128) + sn * 2048 + h * 512);
        o.a[m][h] = Mma<T>::read_tr((const T*)(buf + ((m & 1) ? xo : xe) + off));
        o.b[m][h] = Mma<T>::read_tr((const T*)(buf + ((m & 1) ? go : ge) + off));
      }
  };
  auto mma = [&](const Ops& o) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const u32x4 av = u32x4{o.a[m][0][0], o.a[m][0][1], o.a[m][1][0], o.a[m][1][1]};
#pragma unroll
      for (int n = 0; n < 4; ++n) {
        const u32x4 bv = u32x4{o.b[n][0][0], o.b[n][0][1], o.b[n][1][0], o.b[n][1][1]};
        acc[m][n] = Mma32<T>::run(av, bv, acc[m][n]);
      }
    }
  };

  // ---- ring of three: tile i is multiplied while i + 1 and i + 2 are in flight ----
  Idx iq[3];                                                     // iq[t % 3]: index entries of tile t_begin + t
  stage(t_begin, s_t0, load_index(t_begin));
  stage(t_begin + 1, s_t1, load_index(t_begin + 1));
  iq[2] = load_index(t_begin + 2);
  iq[0] = load_index(t_begin + 3);
  auto step = [&](auto SLOT, int64_t tile) {
    constexpr int slot = decltype(SLOT)::value;
    // own pieces of this tile have landed (those of the next one and its two index entries may be
    // in flight), then everyone's; every wave is also done with the tile before, whose buffer is
    // filled next
    // (a bare barrier: __syncthreads() would wait for the next tile's loads too; the wait as an
    // instruction of its own, which the compiler's wait insertion takes into account:
    // s_waitcnt vmcnt(PW + 2) lgkmcnt(0), vmcnt in bits 3:0, lgkmcnt in bits 11:8)
    __builtin_amdgcn_s_waitcnt(0x0070 | (PW + 2));
    asm volatile("s_barrier" ::: "memory");
    stage(tile + 2, slot == 0 ? s_t2 : slot == 1 ? s_t0 : s_t1, iq[(slot + 2) % 3]);
    iq[(slot + 1) % 3] = load_index(tile + 4);
    const char* buf = slot == 0 ? s_t0 : slot == 1 ? s_t1 : s_t2;
    Ops o0, o1;
    fetch(buf, 0, o0);
    fetch(buf, 1, o1);
    mma(o0);
    __builtin_amdgcn_sched_barrier(0);
    mma(o1);
    __builtin_amdgcn_sched_barrier(0);
  };
  // whole rounds of the ring in the loop, the last one or two tiles after it: no path skips a
  // step, so the compiler's wait insertion sees the real order of loads and reads
  int64_t tile = t_begin;
  for (; tile + 3 <= t_end; tile += 3) {
    step(std::integral_constant<int, 0>{}, tile);
    step(std::integral_constant<int, 1>{}, tile + 1);
    step(std::integral_constant<int, 2>{}, tile + 2);
  }
  if (tile < t_end) {
    step(std::integral_constant<int, 0>{}, tile);
    if (tile + 1 < t_end) step(std::integral_constant<int, 1>{}, tile + 1);
  }
  // (a reader for the index entries that the last steps load: the waits count operations, and the
  // compiler drops a load whose result nobody reads)
#pragma unroll
  for (int v = 0; v < 3; ++v) asm volatile("" ::"v"(iq[v].x), "v"(iq[v].g));
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                 // loads past the range still write LDS

  // ---- per-range sums -> partial[split][a][b] ----
  float* dst = partial + (int64_t)blockIdx.x * ca * cb;
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int a = a_base + 32 * m + 8 * (r >> 2) + 4 * q + (r & 3);
        const int b = b_base + 32 * n + (lane & 31);
        if (a < ca && b < cb) dst[(int64_t)a * cb + b] = acc[m][n][r];
      }
}

}  // namespace ocnn

using namespace ocnn;

static int dr_cu_count() {
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
    n_cu = prop.multiProcessorCount;
  }
  return n_cu;
}

// 32-channel output blocks per wave: as many as registers allow (weights cin / 16 * MB * 4
// registers, sums 2 * MB * 16) among those that divide the output channels
static int dr_mb(int cin, int cout) {
  if (cin != 64 && cin != 128 && cin != 256 && cin != 512) return 0;
  if (cout % 128 != 0) return 0;
  for (int mb = 4; mb >= 1; mb >>= 1)
    if (cin * mb <= 512 && cout % (128 * mb) == 0) return mb;
  return 0;
}

extern "C" int ocnn_conv_dense_rw_supported(int dtype, int64_t rows, int cin, int cout) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (cin <= 0 || cout <= 0 || dr_mb(cin, cout) == 0 || cout > 4096) return 0;
  if (rows < 0 || ((int64_t)rows + 128) * std::max(cin, cout) * 2 > 0xfff00000ll) return 0;
  return 1;
}

template <typename T, int NKS, int MB>
static void launch_dense_rw(const void* in, int64_t rows_in, const int32_t* row_index, int64_t rows, int cout,
                            const void* ws, const void* bias, void* out, int64_t rows_out, const int32_t* out_index,
                            int n_cu, hipStream_t st) {
  const int lds = ((NKS / 4) >= 8 ? 2 : 4) * (NKS / 4) * 64 * 128;
  static bool attr_set = false;
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)conv_dense_rw_kernel<T, NKS, MB>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    attr_set = true;
  }
  const int ny = cout / (128 * MB);
  const int64_t tiles = cdiv(rows, 64);
  int64_t wgs = std::min<int64_t>(tiles, std::max(1, n_cu / ny));
  const int64_t per = cdiv(tiles, wgs);
  wgs = cdiv(tiles, per);
  hipLaunchKernelGGL((conv_dense_rw_kernel<T, NKS, MB>), dim3((unsigned)wgs, (unsigned)ny), dim3(256), lds, st,
                     (const T*)in, (uint32_t)(rows_in * NKS * 32), row_index, (const T*)ws, (const T*)bias, (T*)out,
                     (uint32_t)(rows_out * cout * 2), out_index, rows, cout, tiles, per);
}

template <typename T>
__global__ void pack_weights_dense_kernel(const T* __restrict__ w, T* __restrict__ out, int cin, int cout,
                                          int transposed) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)cin * cout) return;
  int j = (int)(e & 7);
  int lane = (int)((e >> 3) & 63);
  int s = (int)((e >> 9) & 3);
  int64_t rest = e >> 11;
  const int ncg = cout >> 5;
  int cg = (int)(rest % ncg);
  int cc = (int)(rest / ncg);
  int q = lane >> 5, m = lane & 31;
  int chan = 64 * cc + 16 * s + 8 * q + j;
  // M index m = 8 a + 4 q + b is register 4 a + b of the lanes with lane / 32 = q
  int a = m >> 3;
  int co = 32 * cg + 16 * (a >> 1) + 8 * ((m >> 2) & 1) + 4 * (a & 1) + (m & 3);
  out[e] = transposed ? w[(int64_t)co * cin + chan] : w[(int64_t)chan * cout + co];
}

template <typename T>
static int run_dense_rw(const void* in, int64_t rows_in, const int32_t* row_index, int64_t rows, const void* w,
                        int cin, int cout, int w_transposed, const void* bias, void* out, int64_t rows_out,
                        const int32_t* out_index, void* ws, hipStream_t st) {
  const int n_cu = dr_cu_count();
  if (n_cu <= 0) {
    set_error("conv_dense_rw: cannot query the device");
    return OCNN_ERR_HIP;
  }
  hipLaunchKernelGGL(pack_weights_dense_kernel<T>, dim3((unsigned)cdiv((int64_t)cin * cout, 256)), dim3(256), 0, st,
                     (const T*)w, (T*)ws, cin, cout, w_transposed);
  const int mb = dr_mb(cin, cout);
#define OCNN_DRW(CIN_, MB_) \
  if (cin == CIN_ && mb == MB_) { launch_dense_rw<T, CIN_ / 16, MB_>(in, rows_in, row_index, rows, cout, ws, bias, out, rows_out, out_index, n_cu, st); return check_launch("conv_dense_rw"); }
  OCNN_DRW(512, 1) OCNN_DRW(256, 1) OCNN_DRW(256, 2) OCNN_DRW(128, 1) OCNN_DRW(128, 2) OCNN_DRW(128, 4)
  OCNN_DRW(64, 1) OCNN_DRW(64, 2) OCNN_DRW(64, 4)
#undef OCNN_DRW
  set_error("conv_dense_rw: no kernel for cin=%d mb=%d", cin, mb);
  return OCNN_ERR_ARG;
}

extern "C" int ocnn_conv_dense_rw_indexed(int dtype, const void* in, int64_t rows_in, const int32_t* row_index,
                                          int64_t rows, const void* w, int cin, int cout, int w_transposed,
                                          const void* bias, void* out, int64_t rows_out, const int32_t* out_index,
                                          void* workspace, int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(ocnn_conv_dense_rw_supported(dtype, rows, cin, cout), "conv_dense_rw: shape not supported");
  OCNN_REQUIRE(row_index != nullptr || rows_in == rows, "conv_dense_rw: without an index the operand has `rows` rows");
  OCNN_REQUIRE(out_index != nullptr || rows_out == rows, "conv_dense_rw: without an index the result has `rows` rows");
  OCNN_REQUIRE(rows_in >= 0 && ((int64_t)rows_in + 128) * cin * 2 <= 0xfff00000ll, "conv_dense_rw: operand too large");
  OCNN_REQUIRE(rows_out >= 0 && ((int64_t)rows_out + 128) * cout * 2 <= 0xfff00000ll, "conv_dense_rw: result too large");
  if (rows == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("conv_dense_rw", in, w, out, workspace);
  if (workspace_bytes < (int64_t)cin * cout * 2) {
    set_error("conv_dense_rw: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16)
    return run_dense_rw<f16>(in, rows_in, row_index, rows, w, cin, cout, w_transposed, bias, out, rows_out, out_index,
                             workspace, st);
  return run_dense_rw<bf16>(in, rows_in, row_index, rows, w, cin, cout, w_transposed, bias, out, rows_out, out_index,
                            workspace, st);
}

extern "C" int ocnn_conv_dense_rw(int dtype, const void* in, int64_t rows, const void* w, int cin, int cout,
                                  int w_transposed, const void* bias, void* out, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
  return ocnn_conv_dense_rw_indexed(dtype, in, rows, nullptr, rows, w, cin, cout, w_transposed, bias, out, rows, nullptr,
                                    workspace, workspace_bytes, stream);
}

// ---- weight gradient ----
// waves along the x channels of a workgroup's block, or 0 if the shape is not taken
// blocks of 128 WA x 512 / WA channel pairs that cover ca x cb
static int dr_wgrad_blocks(int ca, int cb, int wa) {
  return (int)(cdiv(ca, 128 * wa) * cdiv(cb, 512 / wa));
}

// the block shape with the fewest blocks (ties: the squarer one stages less per tile)
static int dr_wa(int ca, int cb) {
  if (ca < 8 || cb < 8 || ca % 8 != 0 || cb % 8 != 0) return 0;
  int best = 2;
  if (dr_wgrad_blocks(ca, cb, 4) < dr_wgrad_blocks(ca, cb, best)) best = 4;
  if (dr_wgrad_blocks(ca, cb, 1) < dr_wgrad_blocks(ca, cb, best)) best = 1;
  return best;
}

// row ranges per block of channel pairs at most: a workgroup on every CU
static int dr_wgrad_splits(int ca, int cb, int n_cu) {
  return std::max(1, n_cu / dr_wgrad_blocks(ca, cb, dr_wa(ca, cb)));
}

// Every range costs a set of fp32 sums written and read back.  Where those sets weigh against the
// operands (512 x 128 sums on 236 k rows: 128 MB against 301 MB), workgroups on three quarters of
// the CUs do better (2x2x2 stride-2 64 -> 128 on 1.9 M rows: 0.300 -> 0.290 ms for the layer; twice
// the ranges 0.33 ms); where they do not (96 x 96 sums on 925 k rows) every CU is needed to stream
// the rows (70 us on all, 81 us on three quarters).
static int dr_wgrad_ranges(int ca, int cb, int64_t rows, int n_cu) {
  const int all = dr_wgrad_splits(ca, cb, n_cu);
  const int64_t sums = (int64_t)all * ca * cb * 8, operands = rows * (int64_t)(ca + cb) * 2;
  return 10 * sums >= 3 * operands ? std::max(1, all * 3 / 4) : all;
}

extern "C" int ocnn_conv_dense_wgrad_rw_supported(int dtype, int64_t rows, int ca, int cb) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (dr_wa(ca, cb) == 0 || ca > 4096 || cb > 4096) return 0;
  if (rows < 0 || ((int64_t)rows + 128) * std::max(ca, cb) * 2 > 0xfff00000ll) return 0;
  return 1;
}

extern "C" int64_t ocnn_conv_dense_wgrad_rw_workspace_bytes(int ca, int cb) {
  const int n_cu = dr_cu_count();
  if (dr_wa(ca, cb) == 0) return 0;
  return align_up((int64_t)dr_wgrad_splits(ca, cb, n_cu > 0 ? n_cu : 1024) * ca * cb * 4, 256);
}

struct DrOperand {            // a (rows x channels) operand, its rows taken through an index if there is one
  const void* data;
  int64_t rows_total;         // rows of the tensor `data` points to (= rows without an index)
  const int32_t* index;
};

template <typename T, int WA>
static void launch_dense_wgrad(const DrOperand& x, const DrOperand& g, int64_t rows, int ca, int cb, int nsplit,
                               int64_t per, int64_t tiles, float* partial, hipStream_t st) {
  hipLaunchKernelGGL((conv_dense_wgrad_rw_kernel<T, WA>), dim3((unsigned)nsplit, (unsigned)dr_wgrad_blocks(ca, cb, WA)),
                     dim3(256), 0, st, (const T*)x.data, (uint32_t)(x.rows_total * ca * 2), x.index, (const T*)g.data,
                     (uint32_t)(g.rows_total * cb * 2), g.index, rows, ca, cb, tiles, per, partial);
}

template <typename T>
static int run_dense_wgrad(const DrOperand& x, const DrOperand& g, int64_t rows, int ca, int cb, int out_transposed,
                           void* gw, void* ws, int64_t ws_bytes, hipStream_t st) {
  const int n_cu = dr_cu_count();
  if (n_cu <= 0) {
    set_error("conv_dense_wgrad_rw: cannot query the device");
    return OCNN_ERR_HIP;
  }
  const int64_t tiles = cdiv(rows, 32);
  const int nsplit = dr_wgrad_ranges(ca, cb, rows, n_cu);
  const int64_t per = std::max<int64_t>(1, cdiv(tiles, nsplit));
  const int used = (int)cdiv(tiles, per);
  if (ws_bytes < (int64_t)used * ca * cb * 4) {
    set_error("conv_dense_wgrad_rw: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  float* partial = (float*)ws;
  if (rows > 0) {
    const int wa = dr_wa(ca, cb);
    if (wa == 4) launch_dense_wgrad<T, 4>(x, g, rows, ca, cb, used, per, tiles, partial, st);
    else if (wa == 2) launch_dense_wgrad<T, 2>(x, g, rows, ca, cb, used, per, tiles, partial, st);
    else launch_dense_wgrad<T, 1>(x, g, rows, ca, cb, used, per, tiles, partial, st);
  }
  launch_wgrad_reduce<T>(partial, rows > 0 ? used : 0, 1, ca, cb, out_transposed, (T*)gw, st);
  return check_launch("conv_dense_wgrad_rw");
}

extern "C" int ocnn_conv_dense_wgrad_rw_indexed(int dtype, const void* x, int64_t rows_x, const int32_t* x_index,
                                                const void* g, int64_t rows_g, const int32_t* g_index, int64_t rows,
                                                int ca, int cb, int out_transposed, void* gw, void* workspace,
                                                int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(ocnn_conv_dense_wgrad_rw_supported(dtype, rows, ca, cb), "conv_dense_wgrad_rw: shape not supported");
  OCNN_REQUIRE((x_index != nullptr || rows_x == rows) && (g_index != nullptr || rows_g == rows),
               "conv_dense_wgrad_rw: without an index an operand has `rows` rows");
  OCNN_REQUIRE(rows_x >= 0 && rows_g >= 0 && ((int64_t)rows_x + 128) * ca * 2 <= 0xfff00000ll &&
                   ((int64_t)rows_g + 128) * cb * 2 <= 0xfff00000ll,
               "conv_dense_wgrad_rw: operand too large");
  OCNN_REQUIRE_PTRS("conv_dense_wgrad_rw", gw, workspace);
  OCNN_REQUIRE(rows == 0 || (x && g), "conv_dense_wgrad_rw: a required pointer is NULL (of x, g)");
  hipStream_t st = (hipStream_t)stream;
  const DrOperand xo{x, rows_x, x_index}, go{g, rows_g, g_index};
  if (dtype == OCNN_F16)
    return run_dense_wgrad<f16>(xo, go, rows, ca, cb, out_transposed, gw, workspace, workspace_bytes, st);
  return run_dense_wgrad<bf16>(xo, go, rows, ca, cb, out_transposed, gw, workspace, workspace_bytes, st);
}

extern "C" int ocnn_conv_dense_wgrad_rw(int dtype, const void* x, const void* g, int64_t rows, int ca, int cb,
                                        int out_transposed, void* gw, void* workspace, int64_t workspace_bytes,
                                        void* stream) {
  return ocnn_conv_dense_wgrad_rw_indexed(dtype, x, rows, nullptr, g, rows, nullptr, rows, ca, cb, out_transposed, gw,
                                          workspace, workspace_bytes, stream);
}
