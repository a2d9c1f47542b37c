// Weight gradient over the pair plan of a sparse table:
//
//   D[k][a][b] = sum over the pairs (row r of a tile, position p) of slot k of  A[list[p]][a] * B[r][b]
//
// A = the rows that the table points at (reached through the tile's list of distinct rows),
// B = the rows of the table.  The work follows the pairs: per (tile, slot) the pair plan holds
// blocks of 16 pairs, and a block is one v_mfma_f32_32x32x16 per 32 x 32 channels (M = A
// channels, N = B channels, reduction over the 16 pairs).  Both operands come from LDS with
// the transposing load, whose per-lane address does the gather.
//
// A workgroup owns 32 A channels (blockIdx.y), all B channels (<= 96) and a range of tiles,
// and keeps the sums of ALL lists of the pair plan (a list: a slot, or a range of the tiles'
// rows of a heavy slot) in accumulator registers for the whole range: its eight waves (two
// per SIMD: one computes while the other waits for LDS) share the lists; the units left
// over go to the heaviest lists, which are cut into S units that take every S-th block
// (units are dealt to the waves by load on the host).
// Per tile it stages its 64-byte half of the distinct A rows, the B rows and the tile's
// blocks with asynchronous global->LDS loads into the second set of buffers while the
// blocks of the tile before are multiplied.  Per-range sums go to `partial`; a second
// kernel adds them in a fixed order (no atomics).
#include <algorithm>
#include <type_traits>
#include <vector>

#include "common.hpp"
#include "mma.hpp"

namespace ocnn {

constexpr int kWsRows = 128;              // rows per tile (the plan's tile size)
constexpr int kWsCap = 511;               // distinct rows per tile (+ the zero row = 512 LDS rows)
constexpr int kWsEnt = 14 * 256;          // entries per tile: 27 x 8 blocks of 16 at most, in whole KiB

struct WsUnits {                          // (a kernel argument)
  int32_t unit[32];                       // per wave and unit: list j | S << 8 | s << 16, or -1
  int32_t slot[32];                       // the table slot of the unit, or -1
};

static __device__ __forceinline__ void ws_dma16(__amdgpu_buffer_rsrc_t rs, char* dst, uint32_t off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)dst, 16, off, 0, 0, 0);
}

struct WsTile {          // what the loads of a tile need (wave-uniform)
  int32_t U, nb;
  uint32_t cb, b_off;
};

// The global->LDS loads of a tile: pieces of 1 KiB (16 rows of 64 bytes, or 16 blocks of
// entries), dealt to the eight waves.  u: row numbers of the tile's list (LDS; entry p is
// the row of position p, entry 0 = -1: the zero row comes from out of range).
template <int HB>
static __device__ __forceinline__ void ws_stage(char* __restrict__ sa, char* __restrict__ sb,
                                                char* __restrict__ se, const int32_t* __restrict__ u,
                                                const WsTile& t, __amdgpu_buffer_rsrc_t rs_a,
                                                __amdgpu_buffer_rsrc_t rs_b, __amdgpu_buffer_rsrc_t rs_e,
                                                uint32_t a_pitch, uint32_t a_col, uint32_t b_pitch, int wave,
                                                int lane) {
  const int row = lane >> 2;
  const uint32_t chunk = (uint32_t)(lane & 3) * 16u;
  const int na = (t.U + 16) >> 4;                                         // positions 0 .. U
  // four pieces at a time: their list entries first (one LDS wait for the four), then the loads
  for (int p0 = wave; p0 < na; p0 += 32) {
    int32_t id[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) id[e] = u[min(p0 + 8 * e, na - 1) * 16 + row];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int p = p0 + 8 * e;
      if (p < na) ws_dma16(rs_a, sa + p * 1024, id[e] >= 0 ? (uint32_t)id[e] * a_pitch + a_col + chunk : 0xffffff00u);
    }
  }
#pragma unroll
  for (int half = 0; half < HB; ++half)                                   // 8 HB pieces, HB per wave
    ws_dma16(rs_b, sb + half * (kWsRows * 64) + wave * 1024,
             t.b_off + (uint32_t)(wave * 16 + row) * b_pitch + (uint32_t)half * 64u + chunk);
  for (int p = wave; p * 16 < t.nb; p += 8)
    ws_dma16(rs_e, se + p * 1024, t.cb * 64u + (uint32_t)(p * 1024 + lane * 16));
}

// The blocks of one tile.  unit[i] = list j | S << 8 | s << 16 (blocks s, s + S, .. of list
// j), or -1.  cp: block offsets of the tile's lists.
template <typename T, int HB, int NU>
static __device__ __forceinline__ void ws_tile(const char* __restrict__ sa, const char* __restrict__ sb,
                                               const uint32_t* __restrict__ se, const int32_t* __restrict__ cp,
                                               const int (&unit)[NU], f32x16 (&acc)[NU][HB], int lane) {
  const int i16 = lane & 15, q = lane >> 5;
  const uint32_t byte0 = 32u * ((lane >> 4) & 1) + 8u * (i16 & 3);
  const int erow = 8 * q + (i16 >> 2);                                   // the lane's pairs: erow, erow + 4
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    if (unit[i] < 0) continue;
    const int j = unit[i] & 255, S = (unit[i] >> 8) & 255, s = unit[i] >> 16;
    const int b1 = __builtin_amdgcn_readfirstlane(cp[j + 1]);
    for (int b = __builtin_amdgcn_readfirstlane(cp[j]) + s; b < b1; b += S) {
      u32x2 av[2], bv[HB][2];
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const uint32_t e = se[b * 16 + erow + 4 * hh];
        const uint32_t pos = e & 0xffffu, r = min(e >> 16, (uint32_t)(kWsRows - 1));   // filling: zero row x any row
        av[hh] = Mma<T>::read_tr((const T*)(sa + (pos << 6) + byte0));
#pragma unroll
        for (int bh = 0; bh < HB; ++bh)
          bv[bh][hh] = Mma<T>::read_tr((const T*)(sb + bh * (kWsRows * 64) + (r << 6) + byte0));
      }
      const u32x4 a4 = u32x4{av[0][0], av[0][1], av[1][0], av[1][1]};
#pragma unroll
      for (int bh = 0; bh < HB; ++bh)
        acc[i][bh] = Mma32<T>::run(a4, u32x4{bv[bh][0][0], bv[bh][0][1], bv[bh][1][0], bv[bh][1][1]}, acc[i][bh]);
    }
  }
}

// grid: (nsplit, A channels / 32).  units: 8 NU entries (wave-major).  partial:
// [split][A block][wave NU + i][32][32 HB] floats.
template <typename T, int HB, int NU>
__global__ __launch_bounds__(512, 1) void conv_wgrad_sparse_kernel(
    const T* __restrict__ a, uint32_t a_bytes, uint32_t a_pitch, const T* __restrict__ bt, uint32_t b_bytes,
    const int32_t* __restrict__ uptr, const int32_t* __restrict__ urows, uint32_t u_bytes,
    const int32_t* __restrict__ cptr, const uint32_t* __restrict__ ent, uint32_t ent_bytes,
    WsUnits units, int64_t tiles, int64_t tiles_per_split, int nl, float* __restrict__ partial) {
  // one array per buffer, so that the compiler can tell the buffers being filled from the
  // ones being read
  __shared__ __attribute__((aligned(16))) char s_a0[(kWsCap + 1) * 64];
  __shared__ __attribute__((aligned(16))) char s_a1[(kWsCap + 1) * 64];
  __shared__ __attribute__((aligned(16))) char s_b0[HB * kWsRows * 64];
  __shared__ __attribute__((aligned(16))) char s_b1[HB * kWsRows * 64];
  __shared__ __attribute__((aligned(16))) uint32_t s_e0[kWsEnt];
  __shared__ __attribute__((aligned(16))) uint32_t s_e1[kWsEnt];
  __shared__ int32_t s_u0[512];
  __shared__ int32_t s_u1[512];
  __shared__ int32_t s_cp[4][40];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int split = blockIdx.x, ablk = blockIdx.y;
  const int64_t t_begin = (int64_t)split * tiles_per_split;
  const int64_t t_end = min(tiles, t_begin + tiles_per_split);
  constexpr uint32_t b_pitch = HB * 64;

  int unit[NU];
#pragma unroll
  for (int i = 0; i < NU; ++i) unit[i] = __builtin_amdgcn_readfirstlane(units.unit[wave * NU + i]);
  f32x16 acc[NU][HB];
#pragma unroll
  for (int i = 0; i < NU; ++i)
#pragma unroll
    for (int bh = 0; bh < HB; ++bh)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][bh][r] = 0.f;

  const __amdgpu_buffer_rsrc_t rs_a = make_rsrc(a, a_bytes);
  const __amdgpu_buffer_rsrc_t rs_b = make_rsrc(bt, b_bytes);
  const __amdgpu_buffer_rsrc_t rs_e = make_rsrc(ent, ent_bytes);
  const __amdgpu_buffer_rsrc_t rs_u = make_rsrc(urows, u_bytes);
  const __amdgpu_buffer_rsrc_t rs_cp = make_rsrc(cptr, (uint32_t)((tiles * nl + 1) * 4));
  const uint32_t a_col = (uint32_t)ablk * 64u;

  struct Meta { int32_t p0, U, cb, nb; int64_t t; };
  auto meta = [&](int64_t t) {                                           // (wave-uniform loads)
    Meta m;
    const int64_t tc = min(t, tiles - 1);
    const bool in = t < t_end;
    m.t = tc;
    m.p0 = uptr[tc];
    m.U = in ? uptr[tc + 1] - m.p0 : -16;                                // past the range: nothing to load
    m.cb = cptr[tc * nl];
    m.nb = in ? cptr[tc * nl + nl] - m.cb : 0;
    return m;
  };
  auto tile_of = [&](const Meta& m) {
    WsTile t;
    t.U = m.U;
    t.nb = m.nb;
    t.cb = (uint32_t)m.cb;
    t.b_off = m.U >= 0 ? (uint32_t)(m.t * kWsRows) * b_pitch : 0xfff00000u;   // (past the range: zeros)
    return t;
  };
  // row numbers and block offsets of a tile: unconditional buffer loads now, looked at later
  struct Ids { int32_t u, cp, U, cb; };
  auto load_ids = [&](const Meta& m) {
    Ids r;
    r.u = __builtin_amdgcn_raw_buffer_load_b32(rs_u, (uint32_t)(m.p0 + tid - 1) * 4u, 0, 0);
    r.cp = __builtin_amdgcn_raw_buffer_load_b32(rs_cp, (uint32_t)((int)m.t * nl + min(tid, nl)) * 4u, 0, 0);
    r.U = m.U;
    r.cb = m.cb;
    return r;
  };
  auto put_ids = [&](int32_t* su, int seq, const Ids& r) {
    su[tid] = (tid >= 1 && tid <= r.U) ? r.u : -1;
    if (tid < 40) s_cp[seq & 3][tid] = r.cp - r.cb;
  };

  if (t_begin >= t_end) return;

  // ---- prologue: tile 0 lands in the buffers 0, the row numbers of tile 1 in s_u1 ----
  Meta m0 = meta(t_begin), m1 = meta(t_begin + 1), m2 = meta(t_begin + 2);
  put_ids(s_u0, 0, load_ids(m0));
  put_ids(s_u1, 1, load_ids(m1));
  __syncthreads();
  ws_stage<HB>(s_a0, s_b0, (char*)s_e0, s_u0, tile_of(m0), rs_a, rs_b, rs_e, a_pitch, a_col, b_pitch, wave, lane);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // Iteration `seq` (tile t_begin + seq, buffers seq & 1): the loads of the next tile go out,
  // the row numbers of the one after are fetched, the blocks of this tile are multiplied.
  auto iteration = [&](int seq, const char* sa, const char* sb, const uint32_t* se, char* sa_n, char* sb_n,
                       char* se_n, const int32_t* su_n, int32_t* su_c) {
    ws_stage<HB>(sa_n, sb_n, se_n, su_n, tile_of(m1), rs_a, rs_b, rs_e, a_pitch, a_col, b_pitch, wave, lane);
    const Ids ids = load_ids(m2);
    const Meta m3 = meta(t_begin + seq + 3);
    ws_tile<T, HB, NU>(sa, sb, se, s_cp[seq & 3], unit, acc, lane);
    put_ids(su_c, seq + 2, ids);          // (this tile's row numbers were read when its loads went out)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    m1 = m2;
    m2 = m3;
  };
  const int64_t n = t_end - t_begin;
  for (int64_t seq = 0; seq < n; seq += 2) {
    iteration((int)seq, s_a0, s_b0, s_e0, s_a1, s_b1, (char*)s_e1, s_u1, s_u0);
    if (seq + 1 < n) iteration((int)seq + 1, s_a1, s_b1, s_e1, s_a0, s_b0, (char*)s_e0, s_u0, s_u1);
  }

  // ---- the sums of this range ----
  constexpr int CB = 32 * HB;
  float* pw = partial + (((int64_t)split * gridDim.y + ablk) * (8 * NU) + wave * NU) * (32 * CB);
  const int col = lane & 31, rq = lane >> 5;
#pragma unroll
  for (int i = 0; i < NU; ++i)
#pragma unroll
    for (int bh = 0; bh < HB; ++bh)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        pw[i * (32 * CB) + (8 * (r >> 2) + 4 * rq + (r & 3)) * CB + bh * 32 + col] = acc[i][bh][r];
}

// out[k][a][b] (a_major) or out[k][b][a] = sum over the ranges and over the units of slot k,
// in that order.
template <typename T>
__global__ void wgrad_sparse_reduce_kernel(const float* __restrict__ partial, int nsplit, int nunits,
                                           WsUnits units, int K, int ca, int cb, int a_major,
                                           T* __restrict__ out) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)K * ca * cb) return;
  const int b = (int)(e % cb);
  const int a = (int)((e / cb) % ca);
  const int k = (int)(e / ((int64_t)ca * cb));
  const int ablk = a >> 5, al = a & 31, nablk = ca >> 5;
  // (the unit table is a kernel argument: constant indices keep it in scalar registers)
  const int64_t stride = (int64_t)nablk * nunits * 32 * cb;              // floats from range to range
  float sum = 0.f;
#pragma unroll
  for (int u = 0; u < 32; ++u) {
    if (u >= nunits || units.slot[u] != k) continue;
    const float* p = partial + (((int64_t)ablk * nunits + u) * 32 + al) * cb + b;
#pragma unroll 8
    for (int s = 0; s < nsplit; ++s) sum += p[s * stride];
  }
  const int64_t o = a_major ? ((int64_t)k * ca + a) * cb + b : ((int64_t)k * cb + b) * ca + a;
  out[o] = from_f32<T>(sum);
}

}  // namespace ocnn

using namespace ocnn;

constexpr int kWsUnitsPerWave = 4;        // 32 units >= the lists of any plan

extern "C" int ocnn_conv_wgrad_sparse_supported(int dtype, int64_t rows_a, int64_t rows_b, int K, int ca, int cb,
                                                int plan_max_distinct) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (ca < 32 || ca % 32 != 0 || ca > 1024 || cb < 32 || cb % 32 != 0 || cb > 96) return 0;
  if (K < 1 || K > 27 || plan_max_distinct < 0 || plan_max_distinct > kWsCap) return 0;
  if (rows_a < 0 || rows_b < 0) return 0;
  if ((int64_t)rows_a * ca * 2 > 0xfff00000ll || ((int64_t)rows_b + 128) * cb * 2 > 0xfff00000ll) return 0;
  return 1;
}

static int ws_splits(int64_t tiles, int ca) {
  int dev = 0, n_cu = 256;
  (void)hipGetDevice(&dev);
  (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
  return (int)std::max<int64_t>(1, std::min<int64_t>(tiles, std::max(1, n_cu / (ca / 32))));
}

extern "C" int64_t ocnn_conv_wgrad_sparse_workspace_bytes(int64_t rows_b, int ca, int cb) {
  const int64_t tiles = cdiv(std::max<int64_t>(rows_b, 1), kWsRows);
  const int nu = 8 * kWsUnitsPerWave;
  return (int64_t)ws_splits(tiles, ca) * (ca / 32) * nu * 32 * cb * 4;
}

// The units of a launch: every list once, the spare units to the heaviest lists (cut into S
// units that take every S-th block), dealt to the eight waves largest first.
static void ws_make_units(int nl, const int32_t* lists, const int64_t* list_count, int nu, int32_t* units,
                          int32_t* unit_slot) {
  int S[32];
  for (int j = 0; j < nl; ++j) S[j] = 1;
  for (int spare = 8 * nu - nl; spare > 0; --spare) {
    int best = 0;
    for (int j = 1; j < nl; ++j)
      if (list_count[j] * S[best] > list_count[best] * S[j]) best = j;
    ++S[best];
  }
  struct U { int j, s, S; int64_t load; };
  std::vector<U> all;
  for (int j = 0; j < nl; ++j)
    for (int s = 0; s < S[j]; ++s) all.push_back({j, s, S[j], list_count[j] / S[j]});
  std::stable_sort(all.begin(), all.end(), [](const U& x, const U& y) { return x.load > y.load; });
  int cnt[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int64_t load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int i = 0; i < 8 * nu; ++i) units[i] = unit_slot[i] = -1;
  for (const U& u : all) {
    int w = -1;
    for (int c = 0; c < 8; ++c)
      if (cnt[c] < nu && (w < 0 || load[c] < load[w])) w = c;
    units[w * nu + cnt[w]] = u.j | (u.S << 8) | (u.s << 16);
    unit_slot[w * nu + cnt[w]] = lists[u.j] & 255;
    ++cnt[w];
    load[w] += u.load;
  }
}

template <typename T, int HB, int NU>
static void launch_ws(const void* a, int64_t rows_a, int ca, const void* b, int64_t rows_b, const int32_t* uptr,
                      const int32_t* urows, int64_t plan_total, const int32_t* cptr, const uint32_t* ent,
                      int64_t n_blocks, const WsUnits& units, int64_t tiles, int nsplit, int nl, float* partial,
                      hipStream_t st) {
  hipLaunchKernelGGL((conv_wgrad_sparse_kernel<T, HB, NU>), dim3((unsigned)nsplit, (unsigned)(ca / 32)), dim3(512), 0,
                     st, (const T*)a, (uint32_t)(rows_a * ca * 2), (uint32_t)(ca * 2), (const T*)b,
                     (uint32_t)(rows_b * HB * 64), uptr, urows, (uint32_t)(plan_total * 4), cptr, ent,
                     (uint32_t)(n_blocks * 64), units, tiles, cdiv(tiles, nsplit), nl, partial);
}

template <typename T>
static int run_ws(const void* a, int64_t rows_a, int ca, const void* b, int64_t rows_b, int cb, const int32_t* uptr,
                  const int32_t* urows, int64_t plan_total, const int32_t* cptr, const uint32_t* ent,
                  int64_t n_blocks, const int32_t* lists, const int64_t* list_count, int nl, int K, int a_major,
                  void* out, void* ws, hipStream_t st) {
  const int nuw = kWsUnitsPerWave, nu = 8 * nuw;
  const int64_t tiles = cdiv(rows_b, kWsRows);
  const int64_t per_split = cdiv(tiles, ws_splits(tiles, ca));
  const int nsplit = (int)cdiv(tiles, per_split);          // every range holds at least one tile
  WsUnits units;
  for (int i = 0; i < 32; ++i) units.unit[i] = units.slot[i] = -1;
  ws_make_units(nl, lists, list_count, nuw, units.unit, units.slot);
  float* partial = (float*)ws;
  const int hb = cb / 32;
#define OCNN_WS_CASE(HB_)                                                                                    \
  if (hb == HB_) {                                                                                           \
    launch_ws<T, HB_, kWsUnitsPerWave>(a, rows_a, ca, b, rows_b, uptr, urows, plan_total, cptr, ent, n_blocks, \
                                       units, tiles, nsplit, nl, partial, st);                               \
  }
  OCNN_WS_CASE(1) OCNN_WS_CASE(2) OCNN_WS_CASE(3)
#undef OCNN_WS_CASE
  if (check_launch("conv_wgrad_sparse") != OCNN_OK) return OCNN_ERR_HIP;
  const int64_t total = (int64_t)K * ca * cb;
  hipLaunchKernelGGL(wgrad_sparse_reduce_kernel<T>, dim3((unsigned)cdiv(total, 256)), dim3(256), 0, st, partial,
                     nsplit, nu, units, K, ca, cb, a_major, (T*)out);
  return check_launch("wgrad_sparse_reduce");
}

extern "C" int ocnn_conv_wgrad_sparse(int dtype, const void* a, int64_t rows_a, int ca, const void* b,
                                      int64_t rows_b, int cb, const int32_t* uptr, const int32_t* urows,
                                      int plan_max_distinct, int64_t plan_total, const int32_t* cptr,
                                      const uint32_t* ent, int64_t n_blocks, const int32_t* lists,
                                      const int64_t* list_count, int n_lists, int K, int a_major, void* out,
                                      void* workspace, int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(ocnn_conv_wgrad_sparse_supported(dtype, rows_a, rows_b, K, ca, cb, plan_max_distinct),
               "conv_wgrad_sparse: shape not supported");
  OCNN_REQUIRE(rows_b >= 0 && rows_b < (1ll << 31) && plan_total >= 0 && plan_total < (1ll << 29) &&
                   n_blocks >= 0 && n_blocks < (1ll << 25) && n_lists >= 1 && n_lists <= 32,
               "conv_wgrad_sparse: rows or lists out of range");
  OCNN_REQUIRE_PTRS("conv_wgrad_sparse", out);
  OCNN_REQUIRE(rows_b == 0 || (b && uptr && urows && cptr && ent && lists && list_count && workspace && (rows_a == 0 || a)),
               "conv_wgrad_sparse: a required pointer is NULL");
  hipStream_t st = (hipStream_t)stream;
  if (rows_b == 0) {                                   // nothing to add up: zeros
    WsUnits none;
    for (int i = 0; i < 32; ++i) none.unit[i] = none.slot[i] = -1;
    const int64_t total = (int64_t)K * ca * cb;
    if (dtype == OCNN_F16)
      hipLaunchKernelGGL(wgrad_sparse_reduce_kernel<f16>, dim3((unsigned)cdiv(total, 256)), dim3(256), 0, st,
                         (const float*)nullptr, 0, 0, none, K, ca, cb, a_major, (f16*)out);
    else
      hipLaunchKernelGGL(wgrad_sparse_reduce_kernel<bf16>, dim3((unsigned)cdiv(total, 256)), dim3(256), 0, st,
                         (const float*)nullptr, 0, 0, none, K, ca, cb, a_major, (bf16*)out);
    return check_launch("wgrad_sparse_reduce");
  }
  if (workspace_bytes < ocnn_conv_wgrad_sparse_workspace_bytes(rows_b, ca, cb)) {
    set_error("conv_wgrad_sparse: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  if (dtype == OCNN_F16)
    return run_ws<f16>(a, rows_a, ca, b, rows_b, cb, uptr, urows, plan_total, cptr, ent, n_blocks, lists,
                       list_count, n_lists, K, a_major, out, workspace, st);
  return run_ws<bf16>(a, rows_a, ca, b, rows_b, cb, uptr, urows, plan_total, cptr, ent, n_blocks, lists,
                      list_count, n_lists, K, a_major, out, workspace, st);
}
