// Tile plan of a neighbour table: for every tile of kPlanRows consecutive table
// rows, the sorted list of distinct rows the tile reads (so a kernel can stage
// each of them once in LDS) and, per table entry, its position in that list.
#include "common.hpp"

namespace ocnn {

constexpr int kPlanRows = 128;          // table rows per tile
constexpr int kPlanMaxEntries = 4096;   // >= kPlanRows * 27, power of two

// mode 0: ucount[tile] = number of distinct valid entries
// mode 1: urows[uptr[tile] + u] = u-th distinct row; loc[tile][k][row in tile] = u + 1, or
//         0 for an empty entry (also for the rows of the last tile that lie past the table)
__global__ __launch_bounds__(256) void tile_plan_kernel(
    const int32_t* __restrict__ table, int64_t rows, int K, int npad, int mode,
    int32_t* __restrict__ ucount, const int32_t* __restrict__ uptr, int32_t* __restrict__ urows,
    uint16_t* __restrict__ loc) {
  __shared__ int32_t s_key[kPlanMaxEntries];
  __shared__ int32_t s_uq[kPlanMaxEntries];
  __shared__ int32_t s_scan[256];
  const int tid = threadIdx.x;
  const int64_t tile = blockIdx.x;
  const int64_t e0 = tile * kPlanRows * K;
  const int64_t lim = rows * (int64_t)K;
  const int n = kPlanRows * K;
  for (int e = tid; e < npad; e += 256) {
    int32_t v = (e < n && e0 + e < lim) ? table[e0 + e] : -1;
    s_key[e] = v < 0 ? 0x7fffffff : v;
  }
  __syncthreads();
  // bitonic sort, ascending
  for (int k = 2; k <= npad; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = tid; t < (npad >> 1); t += 256) {
        int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
        int p = i | j;
        int32_t a = s_key[i], b = s_key[p];
        bool up = (i & k) == 0;
        if ((a > b) == up) { s_key[i] = b; s_key[p] = a; }
      }
      __syncthreads();
    }
  }
  // distinct values: head flags, block scan over per-thread counts
  const int per = npad / 256;           // npad is a multiple of 256
  const int b0 = tid * per;
  int cnt = 0;
  for (int e = b0; e < b0 + per; ++e) {
    int32_t v = s_key[e];
    cnt += (v != 0x7fffffff && (e == 0 || s_key[e - 1] != v)) ? 1 : 0;
  }
  s_scan[tid] = cnt;
  __syncthreads();
  for (int off = 1; off < 256; off <<= 1) {
    int v = tid >= off ? s_scan[tid - off] : 0;
    __syncthreads();
    s_scan[tid] += v;
    __syncthreads();
  }
  const int total = s_scan[255];
  if (mode == 0) {
    if (tid == 0) ucount[tile] = total;
    return;
  }
  int pos = s_scan[tid] - cnt;
  for (int e = b0; e < b0 + per; ++e) {
    int32_t v = s_key[e];
    if (v != 0x7fffffff && (e == 0 || s_key[e - 1] != v)) s_uq[pos++] = v;
  }
  __syncthreads();
  const int32_t ub = uptr[tile];
  for (int u = tid; u < total; u += 256) urows[ub + u] = s_uq[u];
  for (int e = tid; e < n; e += 256) {
    int32_t v = e0 + e < lim ? table[e0 + e] : -1;
    uint16_t r = 0;
    if (v >= 0) {
      int lo = 0, hi = total - 1;
      while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (s_uq[mid] < v) lo = mid + 1; else hi = mid;
      }
      r = (uint16_t)(lo + 1);
    }
    loc[e0 + (int64_t)(e % K) * kPlanRows + e / K] = r;
  }
}

}  // namespace ocnn

using namespace ocnn;

extern "C" int ocnn_tile_plan_rows(void) { return kPlanRows; }

static int plan_launch(const int32_t* table, int64_t rows, int K, int mode, int32_t* ucount,
                       const int32_t* uptr, int32_t* urows, uint16_t* loc, void* stream) {
  OCNN_REQUIRE(K >= 1 && K <= 27 && rows >= 0 && rows < (1ll << 31), "tile_plan: bad shape");
  if (rows == 0) return OCNN_OK;
  int npad = 256;
  while (npad < kPlanRows * K) npad <<= 1;
  int64_t tiles = cdiv(rows, kPlanRows);
  hipLaunchKernelGGL(tile_plan_kernel, dim3((unsigned)tiles), dim3(256), 0, (hipStream_t)stream,
                     table, rows, K, npad, mode, ucount, uptr, urows, loc);
  return check_launch("tile_plan");
}

extern "C" int ocnn_tile_plan_count(const int32_t* table, int64_t rows, int K, int32_t* ucount,
                                    void* stream) {
  return plan_launch(table, rows, K, 0, ucount, nullptr, nullptr, nullptr, stream);
}

extern "C" int ocnn_tile_plan_fill(const int32_t* table, int64_t rows, int K, const int32_t* uptr,
                                   int32_t* urows, uint16_t* loc, void* stream) {
  return plan_launch(table, rows, K, 1, nullptr, uptr, urows, loc, stream);
}
