// Neighbour search: 27-neighbour tables of full layers and of sparse layers
// (from the parent level's table), non-empty index lists, the table variants
// get_neigh hands out, and the inverse table used by the gather-form backward.
#include "common.hpp"
#include "morton.hpp"

namespace ocnn {

__global__ void neigh_full_kernel(int depth, int64_t total, int64_t* out64, int32_t* out32) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total * 27) return;
  int64_t node = t / 27;
  int k = (int)(t % 27);
  int64_t per = 1ll << (3 * depth);
  int64_t b = node >> (3 * depth);
  uint64_t local = (uint64_t)(node & (per - 1));
  int64_t x = (int64_t)compact3(local >> 2) + (k / 9 - 1);
  int64_t y = (int64_t)compact3(local >> 1) + ((k / 3) % 3 - 1);
  int64_t z = (int64_t)compact3(local) + (k % 3 - 1);
  int64_t bound = 1ll << depth;
  int64_t v = -1;
  if (x >= 0 && y >= 0 && z >= 0 && x < bound && y < bound && z < bound)
    v = encode(x, y, z, depth) + b * per;
  if (out64) out64[t] = v;
  if (out32) out32[t] = (int32_t)v;
}

// For child j of a node and slot k of the 3x3x3 window: which of the parent's
// 27 neighbours holds the cell (lp) and which child of that node it is (lc).
__host__ __device__ __forceinline__ void child_slot_lut(int j, int k, int* lp, int* lc) {
  int gx = 1 + (j >> 2) + k / 9;          // 2 + child bit + displacement(-1..1)
  int gy = 1 + ((j >> 1) & 1) + (k / 3) % 3;
  int gz = 1 + (j & 1) + k % 3;
  *lp = (gx >> 1) * 9 + (gy >> 1) * 3 + (gz >> 1);
  *lc = (gx & 1) * 4 + (gy & 1) * 2 + (gz & 1);
}

constexpr int kParentsPerBlock = 32;

// The 8 x 27 entries below one parent repeat the same (parent slot, child number) pattern, so
// the pattern sits in LDS once a workgroup, and a thread writes four entries at a time: they
// never straddle two parents (216 = 4 * 54).
__global__ __launch_bounds__(256) void neigh_from_parent_kernel(
    const int32_t* __restrict__ child_p, const int32_t* __restrict__ neigh_p,
    const int32_t* __restrict__ nempty_p, int64_t n_ne, int64_t* __restrict__ out64,
    int32_t* __restrict__ out32) {
  __shared__ int32_t cp[kParentsPerBlock * 27];
  __shared__ uint16_t lut[216];
  const int64_t c0 = (int64_t)blockIdx.x * kParentsPerBlock;
  if (threadIdx.x < 216) {
    int lp, lc;
    child_slot_lut(threadIdx.x / 27, threadIdx.x % 27, &lp, &lc);
    lut[threadIdx.x] = (uint16_t)(lp | (lc << 8));
  }
  for (int e = threadIdx.x; e < kParentsPerBlock * 27; e += 256) {
    int p = e / 27, s = e % 27;
    int32_t v = -1;
    if (c0 + p < n_ne) {
      int32_t q = nempty_p[c0 + p];
      int32_t np = neigh_p[(int64_t)q * 27 + s];
      if (np >= 0) v = child_p[np];        // test before dereferencing
    }
    cp[e] = v;
  }
  __syncthreads();
  const int64_t base = c0 * 216;
  const int parents = (int)(n_ne - c0 < kParentsPerBlock ? n_ne - c0 : kParentsPerBlock);
  for (int c = threadIdx.x; c < parents * 54; c += 256) {
    const int p = c / 54, w = (c - p * 54) * 4;
    int32_t r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int l = lut[w + e];
      const int32_t v = cp[p * 27 + (l & 255)];
      r[e] = v < 0 ? -1 : v * 8 + (l >> 8);
    }
    const int64_t o = base + 4 * (int64_t)c;
    if (out32) *reinterpret_cast<int4*>(out32 + o) = make_int4(r[0], r[1], r[2], r[3]);
    if (out64) {
      *reinterpret_cast<longlong2*>(out64 + o) = make_longlong2((int64_t)r[0], (int64_t)r[1]);
      *reinterpret_cast<longlong2*>(out64 + o + 2) = make_longlong2((int64_t)r[2], (int64_t)r[3]);
    }
  }
}

__global__ void nempty_index_kernel(const int32_t* children, int64_t n, int32_t* i32,
                                    int64_t* i64) {
  int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= n) return;
  int32_t c = children[q];
  if (c < 0) return;
  if (i32) i32[c] = (int32_t)q;
  if (i64) i64[c] = q;
}

struct Cols { int c[27]; };

__global__ void neigh_select_kernel(const int32_t* __restrict__ neigh,
                                    const int32_t* __restrict__ row_index, int row_stride,
                                    const int32_t* __restrict__ children, Cols cols, int K,
                                    int64_t rows, int64_t* out64, int32_t* out32) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows * K) return;
  int64_t i = t / K;
  int c = (int)(t % K);
  int64_t r = row_index ? (int64_t)row_index[i] : i * row_stride;
  int32_t v = neigh[r * 27 + cols.c[c]];
  if (v >= 0 && children) v = children[v];
  if (out64) out64[t] = (int64_t)v;
  if (out32) out32[t] = v;
}

__global__ void widen_kernel(const int32_t* in, int64_t n, int64_t* out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) out[t] = (int64_t)in[t];
}

__global__ void narrow_kernel(const int64_t* in, int64_t n, int32_t* out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) out[t] = (int32_t)in[t];
}

__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) p[t] = v;
}

__global__ void table_transpose_kernel(const int32_t* table, int64_t rows, int K,
                                       int64_t rows_in, int32_t* out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows * K) return;
  int32_t j = table[t];
  if (j < 0 || j >= rows_in) return;
  out[(int64_t)j * K + (t % K)] = (int32_t)(t / K);
}

}  // namespace ocnn

using namespace ocnn;

extern "C" void ocnn_host_child_slot_lut(int j, int k, int* lut_parent, int* lut_child) {
  child_slot_lut(j, k, lut_parent, lut_child);
}

extern "C" int ocnn_neigh_full(int depth, int batch, int64_t* out64, int32_t* out32,
                               void* stream) {
  OCNN_REQUIRE(depth >= 0 && depth <= 7 && batch >= 1, "neigh_full: depth=%d batch=%d", depth, batch);
  int64_t total = (int64_t)batch << (3 * depth);
  OCNN_REQUIRE(total * 27 < (1ll << 31), "neigh_full: table too large for a full layer");
  OCNN_REQUIRE(out64 || out32, "neigh_full: both outputs are NULL");
  hipLaunchKernelGGL(neigh_full_kernel, dim3(cdiv(total * 27, 256)), dim3(256), 0,
                     (hipStream_t)stream, depth, total, out64, out32);
  return check_launch("neigh_full");
}

extern "C" int ocnn_neigh_from_parent(const int32_t* child_p, const int32_t* neigh_p,
                                      const int32_t* nempty_p, int64_t n_ne, int64_t* out64,
                                      int32_t* out32, void* stream) {
  OCNN_REQUIRE(n_ne > 0 && n_ne * 8 < (1ll << 31), "neigh_from_parent: n_ne=%lld", (long long)n_ne);
  OCNN_REQUIRE(child_p && neigh_p && nempty_p && (out64 || out32), "neigh_from_parent: a null array");
  hipLaunchKernelGGL(neigh_from_parent_kernel, dim3(cdiv(n_ne, kParentsPerBlock)), dim3(256), 0,
                     (hipStream_t)stream, child_p, neigh_p, nempty_p, n_ne, out64, out32);
  return check_launch("neigh_from_parent");
}

// All tables of an octree with one call: the launches of the shallow layers, a few microseconds
// each, then follow each other without the host between them.
extern "C" int ocnn_neigh_all(int depth, int full_depth, int batch, const int64_t* h_nnum,
                              const int64_t* h_nnum_nempty, const int32_t* const* h_children,
                              int32_t* const* h_nempty_index, int32_t* const* h_neigh, void* stream) {
  // (the table of a layer below the full ones is made from its parents' table, and layer 0 has
  // none: as in the reference, whose construct_neigh(1) fails on an octree with full_depth = 0)
  OCNN_REQUIRE(depth >= 1 && depth <= 16 && full_depth >= 1 && full_depth <= depth && full_depth <= 7 && batch >= 1,
               "neigh_all: depth=%d full_depth=%d batch=%d (1 <= full_depth <= min(depth, 7): layer 1 must be "
               "full, and the table of a full layer has batch x 8^depth x 27 < 2^31 entries)",
               depth, full_depth, batch);
  OCNN_REQUIRE_PTRS("neigh_all", h_nnum, h_nnum_nempty, h_children, h_nempty_index, h_neigh);
  hipStream_t st = (hipStream_t)stream;
  for (int d = 1; d <= depth; ++d) {
    OCNN_REQUIRE(h_neigh[d] != nullptr && h_nnum[d] > 0 && h_nnum[d] * 27 < (1ll << 31),
                 "neigh_all: layer %d: no table, or no nodes, or 2^31 table entries and more", d);
    if (d <= full_depth) {
      const int64_t total = (int64_t)batch << (3 * d);
      OCNN_REQUIRE(h_nnum[d] == total, "neigh_all: layer %d is not full", d);
      hipLaunchKernelGGL(neigh_full_kernel, dim3((unsigned)cdiv(total * 27, 256)), dim3(256), 0, st, d, total,
                         (int64_t*)nullptr, h_neigh[d]);
      continue;
    }
    const int64_t n_ne = h_nnum_nempty[d - 1];
    OCNN_REQUIRE(n_ne > 0 && 8 * n_ne == h_nnum[d] && h_children[d - 1] && h_nempty_index[d - 1] && h_neigh[d - 1],
                 "neigh_all: layers %d and %d are inconsistent", d - 1, d);
    hipLaunchKernelGGL(nempty_index_kernel, dim3((unsigned)cdiv(h_nnum[d - 1], 256)), dim3(256), 0, st,
                       h_children[d - 1], h_nnum[d - 1], h_nempty_index[d - 1], (int64_t*)nullptr);
    hipLaunchKernelGGL(neigh_from_parent_kernel, dim3((unsigned)cdiv(n_ne, kParentsPerBlock)), dim3(256), 0, st,
                       h_children[d - 1], h_neigh[d - 1], h_nempty_index[d - 1], n_ne, (int64_t*)nullptr, h_neigh[d]);
  }
  return check_launch("neigh_all");
}

extern "C" int ocnn_nempty_index(const int32_t* children, int64_t n, int32_t* index32,
                                 int64_t* index64, void* stream) {
  OCNN_REQUIRE(n >= 0, "nempty_index: negative count");
  if (n == 0) return OCNN_OK;
  OCNN_REQUIRE(children && (index32 || index64), "nempty_index: a required pointer is NULL");
  hipLaunchKernelGGL(nempty_index_kernel, dim3(cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream,
                     children, n, index32, index64);
  return check_launch("nempty_index");
}

extern "C" int ocnn_neigh_select(const int32_t* neigh, const int32_t* row_index, int row_stride,
                                 const int32_t* children, const int* h_cols, int K, int64_t rows,
                                 int64_t* out64, int32_t* out32, void* stream) {
  OCNN_REQUIRE(K >= 1 && K <= 27, "neigh_select: K=%d", K);
  OCNN_REQUIRE(rows >= 0, "neigh_select: negative row count");
  if (rows == 0) return OCNN_OK;
  OCNN_REQUIRE(neigh && (out64 || out32), "neigh_select: a required pointer is NULL");
  Cols cols;
  for (int c = 0; c < 27; ++c) cols.c[c] = c;
  if (h_cols)
    for (int c = 0; c < K; ++c) {
      OCNN_REQUIRE(h_cols[c] >= 0 && h_cols[c] < 27, "neigh_select: column %d", h_cols[c]);
      cols.c[c] = h_cols[c];
    }
  hipLaunchKernelGGL(neigh_select_kernel, dim3(cdiv(rows * K, 256)), dim3(256), 0,
                     (hipStream_t)stream, neigh, row_index, row_stride, children, cols, K, rows,
                     out64, out32);
  return check_launch("neigh_select");
}

extern "C" int ocnn_table_to_i64(const int32_t* in, int64_t n, int64_t* out, void* stream) {
  OCNN_REQUIRE(n >= 0, "table_to_i64: negative count");
  if (n == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("table_to_i64", in, out);
  hipLaunchKernelGGL(widen_kernel, dim3(cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream, in, n, out);
  return check_launch("table_to_i64");
}

extern "C" int ocnn_table_to_i32(const int64_t* in, int64_t n, int32_t* out, void* stream) {
  OCNN_REQUIRE(n >= 0, "table_to_i32: negative count");
  if (n == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("table_to_i32", in, out);
  hipLaunchKernelGGL(narrow_kernel, dim3(cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream, in, n, out);
  return check_launch("table_to_i32");
}

extern "C" int ocnn_table_transpose(const int32_t* table, int64_t rows, int K, int64_t rows_in,
                                    int32_t* out, void* stream) {
  OCNN_REQUIRE(K >= 1 && K <= 27 && rows >= 0 && rows_in >= 0, "table_transpose: bad shape");
  OCNN_REQUIRE((rows_in == 0 || out) && (rows == 0 || (table && out)), "table_transpose: a required pointer is NULL");
  hipStream_t st = (hipStream_t)stream;
  if (rows_in > 0)
    hipLaunchKernelGGL(fill_i32_kernel, dim3(cdiv(rows_in * K, 256)), dim3(256), 0, st, out,
                       rows_in * K, -1);
  if (rows > 0)
    hipLaunchKernelGGL(table_transpose_kernel, dim3(cdiv(rows * K, 256)), dim3(256), 0, st, table,
                       rows, K, rows_in, out);
  return check_launch("table_transpose");
}
