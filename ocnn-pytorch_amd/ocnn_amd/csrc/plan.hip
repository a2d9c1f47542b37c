// Tile plan of a neighbour table: for every tile of kPlanRows consecutive table
// rows, the sorted list of distinct rows the tile reads (so a kernel can stage
// each of them once in LDS) and, per table entry, its position in that list.
#include <algorithm>
#include <vector>

#include "common.hpp"
#include "mma.hpp"

namespace ocnn {

constexpr int kPlanRows = 128;          // table rows per tile
constexpr int kPlanMaxEntries = 4096;   // >= kPlanRows * 27, power of two
constexpr int kPlanHash = 4096;         // open-addressing slots that hold any tile (at most 84 % full)
constexpr int kPlanHashQuick = 1024;    // slots of the one-pass build: an octree table fills a tenth of them, and
                                        // with 20 KiB of LDS instead of 72 four tiles share a CU instead of two
constexpr int kPlanRankMax = 1024;      // up to here the distinct rows are ordered by counting
constexpr int kPlanThreads = 512;       // threads a tile: the kernel waits on LDS round trips, more waves hide them
constexpr int kPlanOverflow = 1 << 20;  // count of a tile whose blocks did not fit the quick build's slots
constexpr int kPlanPosWords = (27 * (kPlanRows + 8) + 1) / 2;   // the staged positions, in 32-bit words

template <int HASH>
__device__ __forceinline__ int plan_hash(int32_t v) {
  static_assert(HASH == 4096 || HASH == 1024, "12 or 10 bits");
  return (int)(((uint32_t)v * 2654435761u) >> (HASH == 4096 ? 20 : 22));
}

// mode 0: ucount[tile] = number of distinct valid entries, tile_nnz[tile] = valid entries
// mode 1: urows[uptr[tile] + u] = u-th distinct row; loc[tile][k][row in tile] = u + 1, or
//         0 for an empty entry (also for the rows of the last tile that lie past the table)
// mode 2: both in one pass over the table: counts as mode 0, positions as mode 1, and the
//         list at the fixed place urows[tile * pad + u] (only when it has at most `pad`
//         rows); tile_plan_compact_kernel moves the lists to their offsets afterwards
//
// The distinct rows of a tile (a few hundred among its 3456 entries in an octree table) come
// in runs of consecutive row numbers, so the set is kept by BLOCKS of 32 row numbers: a hash
// set of block numbers in LDS, each with a 32-bit mask of the rows present.  Ordering the rows
// then means ordering the blocks (a tenth as many: by counting, no barriers; tables without
// locality: by a bitonic sort) and counting bits: the position of a row is the number of rows
// in smaller blocks plus the bits below its own in its block's mask.
//
// HASH = kPlanHashQuick (mode 2 only): a tile whose blocks do not fit gives up, ucount[tile] =
// kPlanOverflow; the caller then plans the table in two passes with HASH = kPlanHash.
template <int HASH>
__global__ __launch_bounds__(kPlanThreads) void tile_plan_kernel(
    const int32_t* __restrict__ table, int64_t rows, int K, int mode,
    int32_t* __restrict__ ucount, const int32_t* __restrict__ uptr, int32_t* __restrict__ urows,
    uint16_t* __restrict__ loc, int32_t* __restrict__ tile_nnz, int pad) {
  constexpr int kList = HASH == kPlanHash ? kPlanMaxEntries : (HASH + 16 > kPlanPosWords ? HASH + 16 : kPlanPosWords);
  __shared__ int32_t s_key[HASH];                         // block number, -1 = free
  __shared__ uint32_t s_mask[HASH];                       // its rows
  __shared__ uint16_t s_base[HASH];                       // rows in smaller blocks
  __shared__ __attribute__((aligned(16))) int32_t s_uq[(kList + 15) & ~15];   // the blocks; later: the positions, [slot][row]
  __shared__ __attribute__((aligned(16))) int32_t s_w[HASH == kPlanHash ? kPlanMaxEntries : HASH + 16];   // rows of each of them
  __shared__ int32_t s_scan[2][kPlanThreads / 64];
  __shared__ int32_t s_nnz, s_over;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t tile = blockIdx.x;
  const int64_t e0 = tile * kPlanRows * K;
  const int64_t lim = rows * (int64_t)K;
  const int n = kPlanRows * K;
  // the tile's entries: all loads in flight at once; a thread keeps its entries and the hash
  // slots of their blocks
  constexpr int kPer = (kPlanRows * 27 + kPlanThreads - 1) / kPlanThreads;      // entries per thread, at most
  int32_t ent[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int e = tid + kPlanThreads * i;
    ent[i] = (e < n && e0 + e < lim) ? table[e0 + e] : -1;
  }
  for (int i = tid; i < HASH; i += kPlanThreads) {
    s_key[i] = -1;
    s_mask[i] = 0u;
  }
  if (tid == 0) {
    s_nnz = 0;
    s_over = 0;
  }
  __syncthreads();
  if (mode != 1 && tile_nnz != nullptr) {
    int set = 0;
#pragma unroll
    for (int i = 0; i < kPer; ++i) set += ent[i] >= 0 ? 1 : 0;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) set += __shfl_xor(set, o);
    if (lane == 0) atomicAdd(&s_nnz, set);
  }
  int slot[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int32_t v = ent[i];
    slot[i] = -1;
    if (v >= 0) {
      // a block is met by dozens of entries of the tile: look before the atomics, most find
      // block and bit in place
      const int32_t blk = v >> 5;
      const uint32_t bit = 1u << (v & 31);
      int h = plan_hash<HASH>(blk);
      bool found = true;
      for (int probes = 0;; ++probes) {
        int32_t old = ((volatile int32_t*)s_key)[h];
        if (old == -1) old = atomicCAS(&s_key[h], -1, blk);
        if (old == -1 || old == blk) break;
        if (HASH != kPlanHash && probes >= HASH - 1) {     // every slot holds another block
          found = false;
          s_over = 1;
          break;
        }
        h = (h + 1) & (HASH - 1);
      }
      if (found) {
        if ((((volatile uint32_t*)s_mask)[h] & bit) == 0u) atomicOr(&s_mask[h], bit);
        slot[i] = h;
      }
    }
  }
  __syncthreads();
  if (HASH != kPlanHash && s_over != 0) {
    if (tid == 0) {
      ucount[tile] = kPlanOverflow;
      if (tile_nnz != nullptr) tile_nnz[tile] = s_nnz;
    }
    return;
  }
  // occupied slots: per-thread counts of blocks and rows (slots tid, tid + kPlanThreads, ..: the
  // order of the blocks does not matter before they are ranked), scanned within a wave by lane
  // exchanges, across the waves through LDS
  constexpr int per = HASH / kPlanThreads;
  int32_t held[per];
  uint32_t hmask[per];
  int cnt = 0, nrows = 0;
#pragma unroll
  for (int i = 0; i < per; ++i) {
    held[i] = s_key[tid + kPlanThreads * i];
    hmask[i] = s_mask[tid + kPlanThreads * i];
    cnt += held[i] >= 0 ? 1 : 0;
    nrows += __popc(hmask[i]);
  }
  int incl = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(incl, o);
    if (lane >= o) incl += v;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) nrows += __shfl_xor(nrows, o);
  if (lane == 63) s_scan[0][wave] = incl;
  if (lane == 0) s_scan[1][wave] = nrows;
  __syncthreads();
  int before = 0, nblk = 0, total = 0;                    // blocks in the waves before, blocks, distinct rows
#pragma unroll
  for (int w = 0; w < kPlanThreads / 64; ++w) {
    const int v = s_scan[0][w];
    if (w < wave) before += v;
    nblk += v;
    total += s_scan[1][w];
  }
  if (mode != 1) {
    if (tid == 0) {
      ucount[tile] = total;
      if (tile_nnz != nullptr) tile_nnz[tile] = s_nnz;
    }
    if (mode == 0) return;
  }
  const bool keep_list = mode == 1 || total <= pad;
  int pos = before + incl - cnt;
#pragma unroll
  for (int i = 0; i < per; ++i)
    if (held[i] >= 0) {
      s_uq[pos] = held[i];
      s_w[pos] = __popc(hmask[i]);
      ++pos;
    }
  __syncthreads();
  const int64_t ub = mode == 1 ? (int64_t)uptr[tile] : tile * (int64_t)pad;
  auto slot_of = [&](int32_t blk) {
    int h = plan_hash<HASH>(blk);
    while (s_key[h] != blk) h = (h + 1) & (HASH - 1);
    return h;
  };
  // a block's rows go to the list from `base` on, in the order of their bits
  auto put_block = [&](int32_t blk, int h, int base) {
    s_base[h] = (uint16_t)base;
    if (keep_list) {
      uint32_t m = s_mask[h];
      int32_t* dst = urows + ub + base;
      while (m != 0u) {
        *dst++ = blk * 32 + (__ffs(m) - 1);
        m &= m - 1u;
      }
    }
  };
  if (HASH <= kPlanRankMax || nblk <= kPlanRankMax) {
    // rows before a block = rows of the smaller blocks
    const int tpad = (nblk + 15) & ~15;                   // whole groups of 16; the padding ranks last and weighs nothing
    for (int e = nblk + tid; e < tpad; e += kPlanThreads) {
      s_uq[e] = 0x7fffffff;
      s_w[e] = 0;
    }
    __syncthreads();
    typedef __attribute__((ext_vector_type(4))) int i32x4;
    for (int j = tid; j < nblk; j += kPlanThreads) {
      const int32_t v = s_uq[j];
      int r = 0;
      for (int i = 0; i < tpad; i += 16) {                // 8 x 16-byte broadcast reads in flight
        i32x4 q[4], w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          q[u] = *(const i32x4*)(&s_uq[i + 4 * u]);
          w[u] = *(const i32x4*)(&s_w[i + 4 * u]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          r += (q[u][0] < v ? w[u][0] : 0) + (q[u][1] < v ? w[u][1] : 0) + (q[u][2] < v ? w[u][2] : 0) +
               (q[u][3] < v ? w[u][3] : 0);
      }
      put_block(v, slot_of(v), r);
    }
  } else if constexpr (HASH > kPlanRankMax) {
    int npad = kPlanRankMax * 2;
    while (npad < nblk) npad <<= 1;
    for (int e = nblk + tid; e < npad; e += kPlanThreads) s_uq[e] = 0x7fffffff;
    __syncthreads();
    for (int k = 2; k <= npad; k <<= 1) {          // bitonic sort, ascending
      for (int j = k >> 1; j > 0; j >>= 1) {
        for (int t = tid; t < (npad >> 1); t += kPlanThreads) {
          int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
          int p = i | j;
          int32_t a = s_uq[i], b = s_uq[p];
          bool up = (i & k) == 0;
          if ((a > b) == up) { s_uq[i] = b; s_uq[p] = a; }
        }
        __syncthreads();
      }
    }
    // rows before each block of the sorted list: a thread takes 8 consecutive blocks, their row
    // counts are scanned like the block counts above
    constexpr int kSeq = kPlanMaxEntries / kPlanThreads;
    int hs[kSeq], ws[kSeq], sum = 0;
#pragma unroll
    for (int i = 0; i < kSeq; ++i) {
      const int j = tid * kSeq + i;
      hs[i] = j < nblk ? slot_of(s_uq[j]) : -1;
      ws[i] = hs[i] >= 0 ? __popc(s_mask[hs[i]]) : 0;
      sum += ws[i];
    }
    int inc2 = sum;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int v = __shfl_up(inc2, o);
      if (lane >= o) inc2 += v;
    }
    __syncthreads();                                      // (s_scan is read above by every thread)
    if (lane == 63) s_scan[0][wave] = inc2;
    __syncthreads();
    int base = inc2 - sum;
#pragma unroll
    for (int w = 0; w < kPlanThreads / 64; ++w)
      if (w < wave) base += s_scan[0][w];
#pragma unroll
    for (int i = 0; i < kSeq; ++i) {
      if (hs[i] >= 0) put_block(s_uq[tid * kSeq + i], hs[i], base);
      base += ws[i];
    }
  }
  __syncthreads();
  // positions: every entry knows the slot of its block; through LDS into the order they are
  // stored in ([slot][row]), then out in 16-byte pieces
  uint16_t* s_pos = (uint16_t*)s_uq;                      // (the list of blocks is done with)
  uint16_t pp[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    pp[i] = 0;
    if (slot[i] >= 0) {
      const uint32_t below = (1u << (ent[i] & 31)) - 1u;
      pp[i] = (uint16_t)(s_base[slot[i]] + __popc(s_mask[slot[i]] & below) + 1);
    }
  }
  __syncthreads();
  // (e / K by a multiplication: exact for e < 4096 and K <= 27; a slot's positions 136 apart in
  // LDS, so that the entries of a row, which neighbouring lanes hold, fall on different banks)
  constexpr int kPitch = kPlanRows + 8;
  const uint32_t inv_k = ((1u << 20) + (uint32_t)K - 1u) / (uint32_t)K;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int e = tid + kPlanThreads * i;
    if (e < n) {
      const int row = (int)(((uint32_t)e * inv_k) >> 20), k = e - row * K;
      s_pos[k * kPitch + row] = pp[i];
    }
  }
  __syncthreads();
  u32x4* dst = (u32x4*)(loc + e0);
  for (int i = tid; i < K * (kPlanRows / 8); i += kPlanThreads)
    dst[i] = *(const u32x4*)(s_pos + (i >> 4) * kPitch + (i & 15) * 8);
}

// Pair plan of a table, on top of its tile plan: per tile and LIST the rows that have a
// neighbour, in blocks of 16 entries (position of the neighbour in the tile's list of rows
// | row of the tile << 16).  A list is a slot, or
// the rows r0 .. r1 - 1 of the tiles of a slot that holds many pairs (list = slot |
// r0 << 8 | (r1 - 1) << 16).  One wave per (tile, list); mode 0 counts the blocks, mode 1
// writes the entries and fills the last block up.
__global__ void pair_plan_kernel(const uint16_t* __restrict__ loc, int64_t tiles, int K,
                                 const int32_t* __restrict__ lists, int nl, int mode, int32_t* __restrict__ nblk,
                                 const int32_t* __restrict__ cptr, uint32_t* __restrict__ ent) {
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);   // tile * nl + j
  if (item >= tiles * nl) return;
  const int64_t tile = item / nl;
  const int32_t list = lists[(int)(item - tile * nl)];
  const int k = list & 255, r0 = (list >> 8) & 255, r1 = ((list >> 16) & 255) + 1;
  const uint16_t* p = loc + (tile * K + k) * kPlanRows;
  const uint32_t l0 = (lane >= r0 && lane < r1) ? p[lane] : 0u;
  const uint32_t l1 = (lane + 64 >= r0 && lane + 64 < r1) ? p[lane + 64] : 0u;
  const unsigned long long m0 = __ballot(l0 != 0), m1 = __ballot(l1 != 0);
  const int n0 = __popcll(m0), n = n0 + __popcll(m1);
  if (mode == 0) {
    if (lane == 0) nblk[item] = (n + 15) >> 4;
    return;
  }
  uint32_t* e = ent + (int64_t)cptr[item] * 16;
  const unsigned long long below = (1ull << lane) - 1ull;
  auto entry = [](uint32_t pos, int r) { return pos | ((uint32_t)r << 16); };
  if (l0 != 0) e[__popcll(m0 & below)] = entry(l0, lane);
  if (l1 != 0) e[n0 + __popcll(m1 & below)] = entry(l1, lane + 64);
  const int padded = (n + 15) & ~15;
  if (n + lane < padded) e[n + lane] = entry(0u, kPlanRows);                 // the zero row, to a spare row
}

// What the host needs to know of the counts, and the offsets of the row lists, in one
// workgroup (a table has tens of thousands of tiles at most).  Tiles with more than `cap`
// distinct rows are dropped (counted as empty) when they are few: at most a tenth of the
// tiles.  stats: [tiles over cap, dropped (0 | 1), total, largest count, entries set, tiles the
// quick one-pass build gave up on (then nothing else here means anything)], the third to fifth
// without the dropped tiles.
__global__ __launch_bounds__(1024) void tile_plan_offsets_kernel(
    const int32_t* __restrict__ ucount, const int32_t* __restrict__ tile_nnz, int64_t tiles, int cap,
    int32_t* __restrict__ uptr, int64_t* __restrict__ stats) {
  // the tiles in rounds of 4096, thread t on the four tiles from 4096 r + 4 t (consecutive
  // 16-byte loads, two rounds in flight); a round's counts fit 32 bits, the running offset is
  // carried from round to round by every thread
  __shared__ int s_wsum[2][16];
  __shared__ long long s_wnnz[16];
  __shared__ int s_wbig[16], s_wover[16], s_wmax[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t rounds = (tiles + 4095) / 4096;
  auto wave_sum = [&](long long v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
  };
  struct Four { int v[4]; };
  auto load4 = [&](const int32_t* p, int64_t t) {
    Four q;
#pragma unroll
    for (int i = 0; i < 4; ++i) q.v[i] = t + i < tiles ? p[t + i] : 0;
    return q;
  };
  int big = 0, over = 0;
  for (int64_t r = 0; r < rounds; r += 4) {               // four rounds in flight
    Four c4[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) c4[u] = load4(ucount, (r + u) * 4096 + 4 * tid);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        big += c4[u].v[i] > cap && c4[u].v[i] < kPlanOverflow ? 1 : 0;
        over += c4[u].v[i] >= kPlanOverflow ? 1 : 0;
      }
  }
  big = (int)wave_sum(big);
  over = (int)wave_sum(over);
  if (lane == 0) {
    s_wbig[wave] = big;
    s_wover[wave] = over;
  }
  __syncthreads();
  int n_big = 0, n_over = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    n_big += s_wbig[w];
    n_over += s_wover[w];
  }
  const bool drop = n_big > 0 && n_big <= max((int64_t)1, tiles / 10);
  long long base = 0, nnz = 0;
  int mx = 0;
  Four cn = load4(ucount, 4 * tid), zn = load4(tile_nnz, 4 * tid);
  for (int64_t r = 0; r < rounds; ++r) {
    const int64_t t = r * 4096 + 4 * tid;
    Four c = cn;
    const Four z = zn;
    cn = load4(ucount, t + 4096);                         // the next round's, under this round's scan
    zn = load4(tile_nnz, t + 4096);
    int own = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool skip = (drop && c.v[i] > cap) || c.v[i] >= kPlanOverflow;
      if (skip) c.v[i] = 0;
      if (!skip) {
        mx = max(mx, c.v[i]);
        nnz += z.v[i];
      }
      own += c.v[i];
    }
    int incl = own;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int v = __shfl_up(incl, o);
      if (lane >= o) incl += v;
    }
    if (lane == 63) s_wsum[r & 1][wave] = incl;
    __syncthreads();                                      // (the other set of slots is the one read a round ago)
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int v = s_wsum[r & 1][w];
      if (w < wave) before += v;
      total += v;
    }
    long long at = base + before + incl - own;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (t + i < tiles) uptr[t + i] = (int32_t)at;
      at += c.v[i];
    }
    base += total;
  }
  const long long wnnz = wave_sum(nnz);
  int wmx = mx;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) wmx = max(wmx, __shfl_xor(wmx, o));
  if (lane == 0) {
    s_wnnz[wave] = wnnz;
    s_wmax[wave] = wmx;
  }
  __syncthreads();
  if (tid == 0) {
    long long nnz_all = 0;
    int max_all = 0;
    for (int w = 0; w < 16; ++w) {
      nnz_all += s_wnnz[w];
      max_all = max(max_all, s_wmax[w]);
    }
    uptr[tiles] = (int32_t)base;
    stats[0] = n_big;
    stats[1] = drop ? 1 : 0;
    stats[2] = base;
    stats[3] = max_all;
    stats[4] = nnz_all;
    stats[5] = n_over;
  }
}

// After a one-pass build (mode 2 above): a wave per tile moves the tile's list from its fixed
// place to its offset; a tile that the offsets dropped (more than `cap` distinct rows, few such
// tiles) becomes empty: its positions are cleared.
__global__ __launch_bounds__(256) void tile_plan_compact_kernel(
    const int32_t* __restrict__ ucount, const int32_t* __restrict__ uptr, const int64_t* __restrict__ stats,
    int cap, int pad, const int32_t* __restrict__ ulist, int32_t* __restrict__ urows, uint16_t* __restrict__ loc,
    int K, int64_t tiles) {
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= tiles) return;
  const int U = ucount[tile];
  if (stats[1] != 0 && U > cap) {
    u32x4* p = (u32x4*)(loc + tile * (int64_t)(K * kPlanRows));
    for (int i = lane; i < K * (kPlanRows / 8); i += 64) p[i] = u32x4{0u, 0u, 0u, 0u};
    return;
  }
  if (U > pad) return;                                    // (the caller fills such a plan in two passes)
  const int32_t* src = ulist + tile * (int64_t)pad;
  int32_t* dst = urows + uptr[tile];
  for (int i = lane; i < U; i += 64) dst[i] = src[i];
}

__global__ void pair_plan_zero_kernel(unsigned long long* __restrict__ slot_count, int K) {
  if ((int)threadIdx.x < K) slot_count[threadIdx.x] = 0;
}

__global__ void pair_plan_slot_count_kernel(const uint16_t* __restrict__ loc, int64_t tiles, int K,
                                            unsigned long long* __restrict__ slot_count) {
  // workgroup (k, y): slot k over the tiles y, y + gridDim.y, ..; integer sums, so the order
  // in which the workgroups add theirs does not show in the result
  __shared__ unsigned long long s_part[256];
  const int k = blockIdx.x;
  unsigned long long acc = 0;
  const int64_t chunks = tiles * (kPlanRows / 8);
  for (int64_t t = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; t < chunks; t += (int64_t)gridDim.y * blockDim.x) {
    const int64_t tile = t / (kPlanRows / 8);
    const int c = (int)(t - tile * (kPlanRows / 8));
    const u32x4 v = *(const u32x4*)(loc + (tile * K + k) * kPlanRows + 8 * c);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc += ((v[i] & 0xffffu) != 0) + ((v[i] >> 16) != 0);
  }
  s_part[threadIdx.x] = acc;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) s_part[threadIdx.x] += s_part[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0 && s_part[0] != 0) atomicAdd(&slot_count[k], s_part[0]);
}

}  // namespace ocnn

using namespace ocnn;

extern "C" int ocnn_tile_plan_rows(void) { return kPlanRows; }

static int plan_launch(const int32_t* table, int64_t rows, int K, int mode, int32_t* ucount,
                       const int32_t* uptr, int32_t* urows, uint16_t* loc, int32_t* tile_nnz, int pad,
                       void* stream) {
  OCNN_REQUIRE(K >= 1 && K <= 27 && rows >= 0 && rows < (1ll << 31), "tile_plan: bad shape");
  if (rows == 0) return OCNN_OK;
  // count: the table and the counts; fill: the offsets, the lists and the positions; build: all but the offsets
  OCNN_REQUIRE(table && (mode == 1 ? (uptr && urows && loc) : ucount != nullptr) && (mode != 2 || (urows && loc)),
               "tile_plan: a required pointer is NULL");
  int64_t tiles = cdiv(rows, kPlanRows);
  if (mode == 2)
    hipLaunchKernelGGL(tile_plan_kernel<kPlanHashQuick>, dim3((unsigned)tiles), dim3(kPlanThreads), 0,
                       (hipStream_t)stream, table, rows, K, mode, ucount, uptr, urows, loc, tile_nnz, pad);
  else
    hipLaunchKernelGGL(tile_plan_kernel<kPlanHash>, dim3((unsigned)tiles), dim3(kPlanThreads), 0,
                       (hipStream_t)stream, table, rows, K, mode, ucount, uptr, urows, loc, tile_nnz, pad);
  return check_launch("tile_plan");
}

extern "C" int ocnn_tile_plan_build(const int32_t* table, int64_t rows, int K, int pad, int32_t* ucount,
                                    int32_t* tile_nnz, int32_t* ulist, uint16_t* loc, void* stream) {
  OCNN_REQUIRE(pad >= 1 && pad <= 4096, "tile_plan_build: bad list size");
  return plan_launch(table, rows, K, 2, ucount, nullptr, ulist, loc, tile_nnz, pad, stream);
}

extern "C" int ocnn_tile_plan_compact(const int32_t* ucount, const int32_t* uptr, const int64_t* stats, int cap,
                                      int pad, const int32_t* ulist, int32_t* urows, uint16_t* loc, int K,
                                      int64_t tiles, void* stream) {
  OCNN_REQUIRE(K >= 1 && K <= 27 && tiles >= 0 && tiles < (1ll << 31) && cap >= 0 && cap <= pad,
               "tile_plan_compact: bad shape");
  if (tiles == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("tile_plan_compact", ucount, uptr, stats, ulist, urows, loc);
  hipLaunchKernelGGL(tile_plan_compact_kernel, dim3((unsigned)cdiv(tiles, 4)), dim3(256), 0, (hipStream_t)stream,
                     ucount, uptr, stats, cap, pad, ulist, urows, loc, K, tiles);
  return check_launch("tile_plan_compact");
}

extern "C" int ocnn_tile_plan_count(const int32_t* table, int64_t rows, int K, int32_t* ucount,
                                    int32_t* tile_nnz, void* stream) {
  return plan_launch(table, rows, K, 0, ucount, nullptr, nullptr, nullptr, tile_nnz, 0, stream);
}

extern "C" int ocnn_tile_plan_offsets(const int32_t* ucount, const int32_t* tile_nnz, int64_t tiles, int cap,
                                      int32_t* uptr, int64_t* stats, void* stream) {
  OCNN_REQUIRE(tiles >= 0 && tiles < (1ll << 31) && cap >= 0, "tile_plan_offsets: bad shape");
  OCNN_REQUIRE_PTRS("tile_plan_offsets", uptr, stats);
  OCNN_REQUIRE(tiles == 0 || (ucount && tile_nnz), "tile_plan_offsets: a required pointer is NULL (of ucount, tile_nnz)");
  hipLaunchKernelGGL(tile_plan_offsets_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, ucount, tile_nnz,
                     tiles, cap, uptr, stats);
  return check_launch("tile_plan_offsets");
}

extern "C" int ocnn_tile_plan_fill(const int32_t* table, int64_t rows, int K, const int32_t* uptr,
                                   int32_t* urows, uint16_t* loc, void* stream) {
  return plan_launch(table, rows, K, 1, nullptr, uptr, urows, loc, nullptr, 0, stream);
}

extern "C" int ocnn_pair_plan_slot_counts(const uint16_t* loc, int64_t tiles, int K, int64_t* slot_count,
                                          void* stream) {
  OCNN_REQUIRE(K >= 1 && K <= 27 && tiles >= 0 && tiles < (1ll << 24), "pair_plan: bad shape");
  OCNN_REQUIRE(slot_count && (tiles == 0 || loc), "pair_plan_slot_counts: a required pointer is NULL");
  hipLaunchKernelGGL(pair_plan_zero_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream,
                     (unsigned long long*)slot_count, K);
  const unsigned gy = (unsigned)std::max<int64_t>(1, std::min<int64_t>(64, cdiv(tiles, 16)));
  hipLaunchKernelGGL(pair_plan_slot_count_kernel, dim3((unsigned)K, gy), dim3(256), 0, (hipStream_t)stream, loc,
                     tiles, K, (unsigned long long*)slot_count);
  return check_launch("pair_plan_slot_counts");
}

extern "C" int ocnn_pair_plan_lists(int K, const int64_t* slot_count, int32_t* lists, int64_t* list_count,
                                    int32_t* group_bounds, int* n_lists) {
  OCNN_REQUIRE(K >= 1 && K <= 27, "pair_plan_lists: bad slot count");
  OCNN_REQUIRE_PTRS("pair_plan_lists", slot_count, lists, list_count, group_bounds, n_lists);
  struct List { int k, r0, r1; int64_t load; };
  std::vector<List> all;
  int64_t total = 0;
  for (int k = 0; k < K; ++k) {
    all.push_back({k, 0, kPlanRows, slot_count[k]});
    total += slot_count[k];
  }
  // heavy slots (the centre of a 3x3x3 table holds a third of all pairs) are cut by rows,
  // down to 32 rows, until no list holds more than 1/24 of the pairs or 32 lists are made
  while ((int)all.size() < 32) {
    int best = -1;
    for (int i = 0; i < (int)all.size(); ++i)
      if (all[i].r1 - all[i].r0 >= 64 && (best < 0 || all[i].load > all[best].load)) best = i;
    if (best < 0 || all[best].load * 24 <= total) break;
    List lo = all[best], hi = all[best];
    lo.r1 = hi.r0 = (lo.r0 + lo.r1) / 2;
    lo.load = all[best].load / 2;
    hi.load = all[best].load - lo.load;
    all[best] = lo;
    all.push_back(hi);
  }
  // four groups of at most 8 lists: largest first, each to the lightest group with room
  std::stable_sort(all.begin(), all.end(), [](const List& x, const List& y) { return x.load > y.load; });
  std::vector<List> grp[4];
  int64_t load[4] = {0, 0, 0, 0};
  for (const List& l : all) {
    int g = -1;
    for (int c = 0; c < 4; ++c)
      if (grp[c].size() < 8 && (g < 0 || load[c] < load[g])) g = c;
    grp[g].push_back(l);
    load[g] += l.load;
  }
  int n = 0;
  for (int g = 0; g < 4; ++g) {
    group_bounds[g] = n;
    for (const List& l : grp[g]) {
      lists[n] = l.k | (l.r0 << 8) | ((l.r1 - 1) << 16);
      list_count[n] = l.load;
      ++n;
    }
  }
  group_bounds[4] = n;
  *n_lists = n;
  return OCNN_OK;
}

static int pair_plan_launch(const uint16_t* loc, int64_t tiles, int K, const int32_t* lists, int nl, int mode,
                            int32_t* nblk, const int32_t* cptr, uint32_t* ent, void* stream) {
  OCNN_REQUIRE(K >= 1 && K <= 27 && nl >= 1 && nl <= 32 && tiles >= 0 && tiles < (1ll << 24),
               "pair_plan: bad shape");
  if (tiles == 0) return OCNN_OK;
  OCNN_REQUIRE(loc && lists && (mode == 0 ? nblk != nullptr : (cptr && ent)), "pair_plan: a required pointer is NULL");
  hipLaunchKernelGGL(pair_plan_kernel, dim3((unsigned)cdiv(tiles * nl, 4)), dim3(256), 0, (hipStream_t)stream, loc,
                     tiles, K, lists, nl, mode, nblk, cptr, ent);
  return check_launch("pair_plan");
}

extern "C" int ocnn_pair_plan_count(const uint16_t* loc, int64_t tiles, int K, const int32_t* lists, int n_lists,
                                    int32_t* nblk, void* stream) {
  return pair_plan_launch(loc, tiles, K, lists, n_lists, 0, nblk, nullptr, nullptr, stream);
}

extern "C" int ocnn_pair_plan_fill(const uint16_t* loc, int64_t tiles, int K, const int32_t* lists, int n_lists,
                                   const int32_t* cptr, uint32_t* ent, void* stream) {
  return pair_plan_launch(loc, tiles, K, lists, n_lists, 1, nullptr, cptr, ent, stream);
}
