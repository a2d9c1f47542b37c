// Key search, point interpolation (nearest / trilinear) and 2x2x2 max pooling on octrees.
//
// All of it is index arithmetic plus row gathers: HBM / L2-latency bound.  Every output
// element is produced by exactly one thread from a fixed list of inputs (gather form), so
// nothing here needs atomics and every result is reproducible bit for bit.
#include <algorithm>
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "common.hpp"
#include "morton.hpp"

namespace ocnn {

// first position whose key is >= q (keys ascending)
__device__ __forceinline__ int64_t lower_bound_key(const int64_t* __restrict__ keys, int64_t n, int64_t q) {
  int64_t lo = 0, len = n;
  while (len > 0) {
    const int64_t half = len >> 1;
    const bool less = keys[lo + half] < q;
    lo = less ? lo + half + 1 : lo;
    len = less ? len - half - 1 : half;
  }
  return lo;
}

__device__ __forceinline__ int64_t find_key(const int64_t* __restrict__ keys, int64_t n, int64_t q) {
  const int64_t i = lower_bound_key(keys, n, q);
  return (i < n && keys[i] == q) ? i : -1;
}

__global__ void search_key_kernel(const int64_t* __restrict__ keys, int64_t n,
                                  const int64_t* __restrict__ query, int64_t m, int64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < m) out[i] = find_key(keys, n, query[i]);
}

// key of a float (x, y, z, b): truncation toward zero like Tensor.long(), then the masks of
// every key (a coordinate outside the volume wraps; bound_check is what rejects it)
__device__ __forceinline__ int64_t key_of(float x, float y, float z, float b, int depth) {
  return encode((int64_t)x, (int64_t)y, (int64_t)z, depth) | ((int64_t)b << 48);
}

__global__ void search_points_kernel(const float* __restrict__ pts, int64_t m, int depth,
                                     const int64_t* __restrict__ keys, int64_t n, int bound_check,
                                     int32_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= m) return;
  const float x = pts[4 * i], y = pts[4 * i + 1], z = pts[4 * i + 2], b = pts[4 * i + 3];
  int64_t r = find_key(keys, n, key_of(x, y, z, b, depth));
  const float hi = (float)(1 << depth);
  if (bound_check && !(x >= 0.f && x < hi && y >= 0.f && y < hi && z >= 0.f && z < hi)) r = -1;
  out[i] = (int32_t)r;
}

// ---- the same searches down the tree -------------------------------------------------------
// A node's place in its layer follows from its parent's: the children of the c-th non-empty node
// of a layer are the nodes 8 c .. 8 c + 7 of the next one.  Walking down from the deepest full
// layer finds a key in depth - full_depth dependent loads, most of them in small, cache-resident
// arrays, where the binary search over the layer's keys takes log2(nodes): the same answer, a
// node or -1.
constexpr int kLocateMaxDepth = 16;
struct LocateTree {
  const int32_t* children[kLocateMaxDepth + 1];
  int depth, full_depth, batch_size, nempty;
};

__device__ __forceinline__ int32_t locate_key(const LocateTree& t, int64_t key) {
  const int64_t b = key >> 48;
  if (b < 0 || b >= t.batch_size) return -1;
  const int64_t m = key & ((1ll << 48) - 1);
  if ((m >> (3 * t.depth)) != 0) return -1;               // beyond the layer's keys
  const int top = t.depth < t.full_depth ? t.depth : t.full_depth;
  int64_t pos = (b << (3 * top)) | (m >> (3 * (t.depth - top)));
  for (int l = top; l < t.depth; ++l) {
    const int32_t c = t.children[l][pos];
    if (c < 0) return -1;
    pos = ((int64_t)c << 3) | ((m >> (3 * (t.depth - 1 - l))) & 7);
  }
  return t.nempty ? t.children[t.depth][pos] : (int32_t)pos;
}

__global__ void locate_points_kernel(const float* __restrict__ pts, int64_t m, LocateTree t, int bound_check,
                                     int32_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= m) return;
  const float x = pts[4 * i], y = pts[4 * i + 1], z = pts[4 * i + 2], b = pts[4 * i + 3];
  int32_t r = locate_key(t, key_of(x, y, z, b, t.depth));
  const float hi = (float)(1 << t.depth);
  if (bound_check && !(x >= 0.f && x < hi && y >= 0.f && y < hi && z >= 0.f && z < hi)) r = -1;
  out[i] = r;
}

// Trilinear weights: values sit at voxel centres, so f = p - 0.5, corner = floor(f), and the
// neighbour j = (gx, gy, gz) weighs |((1 - gx) - frac_x) ((1 - gy) - frac_y) ((1 - gz) - frac_z)|.
// One thread per (point, neighbour); the 8 threads of a point add their weights in neighbour
// order for the normalisation.
template <bool LOCATE>
__global__ void interp_linear_prepare_kernel(const float* __restrict__ pts, int64_t m, int depth,
                                             const int64_t* __restrict__ keys, int64_t n, LocateTree tree,
                                             int bound_check, int32_t* __restrict__ idx, float* __restrict__ w,
                                             float* __restrict__ norm) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t i = t >> 3;
  const int j = (int)(t & 7);
  float wj = 0.f;
  int32_t r = -1;
  if (i < m) {
    const float gx = (float)(j >> 2), gy = (float)((j >> 1) & 1), gz = (float)(j & 1);
    const float fx = pts[4 * i] - 0.5f, fy = pts[4 * i + 1] - 0.5f, fz = pts[4 * i + 2] - 0.5f;
    const float ix = floorf(fx), iy = floorf(fy), iz = floorf(fz);
    const float nx = ix + gx, ny = iy + gy, nz = iz + gz;
    const int64_t key = key_of(nx, ny, nz, pts[4 * i + 3], depth);
    int64_t f = LOCATE ? (int64_t)locate_key(tree, key) : find_key(keys, n, key);
    const float hi = (float)(1 << depth);
    if (bound_check && !(nx >= 0.f && nx < hi && ny >= 0.f && ny < hi && nz >= 0.f && nz < hi)) f = -1;
    if (f >= 0) {
      const float tx = (1.0f - gx) - (fx - ix), ty = (1.0f - gy) - (fy - iy), tz = (1.0f - gz) - (fz - iz);
      wj = fabsf((tx * ty) * tz);
      r = (int32_t)f;
    }
    idx[t] = r;
    w[t] = wj;
  }
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) s += __shfl(wj, (threadIdx.x & ~7) + k, 64);
  if (i < m && j == 0) norm[i] = s;
}

// out[r][c] = (sum_e val[e] * data[col[e]][c]) / (rowdiv[r] + 1e-12), e over the entries of
// row r: rowptr[r] .. rowptr[r + 1] - 1, or kfixed entries per row.  col < 0 = no entry.
// fp32 sums in entry order.
template <typename T, int VEC> struct alignas(sizeof(T) * VEC) PoolVec { T v[VEC]; };

template <typename T, int VEC>
__global__ void csr_rows_kernel(const int32_t* __restrict__ rowptr, int kfixed, const int32_t* __restrict__ col,
                                const float* __restrict__ val, const T* __restrict__ data, int C,
                                const float* __restrict__ rowdiv, T* __restrict__ out, int64_t rows) {
  typedef PoolVec<T, VEC> V;
  const int lpr = C / VEC;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows * lpr) return;
  const int64_t r = t / lpr;
  const int c0 = (int)(t - r * lpr) * VEC;
  const int64_t e0 = rowptr ? rowptr[r] : r * kfixed;
  const int64_t e1 = rowptr ? rowptr[r + 1] : e0 + kfixed;
  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
  int64_t e = e0;
  for (; e + 4 <= e1; e += 4) {                // four rows in flight, added in entry order
    int32_t cidx[4];
    float we[4];
    V q[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      cidx[u] = col[e + u];
      we[u] = val ? val[e + u] : 1.0f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (cidx[u] >= 0) q[u] = *(const V*)(data + (int64_t)cidx[u] * C + c0);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (cidx[u] >= 0) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += we[u] * to_f32(q[u].v[v]);
      }
  }
  for (; e < e1; ++e) {
    const int32_t cidx = col[e];
    if (cidx < 0) continue;
    const float we = val ? val[e] : 1.0f;
    const V q = *(const V*)(data + (int64_t)cidx * C + c0);
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] += we * to_f32(q.v[v]);
  }
  const float div = rowdiv ? rowdiv[r] + 1e-12f : 1.0f;
  V o;
#pragma unroll
  for (int v = 0; v < VEC; ++v) o.v[v] = from_f32<T>(rowdiv ? acc[v] / div : acc[v]);
  *(V*)(out + r * C + c0) = o;
}

// ---- row form of the transposed matrix ------------------------------------------------------
// Entry e = (point e / k, slot e % k) of idx names data row idx[e] (< 0: none).  Sorted by data
// row (stable: the points of a row ascend), the entries of row r are rowptr[r] .. rowptr[r + 1].
struct RowKey {
  const int32_t* idx;
  uint32_t rows;
  __host__ __device__ uint32_t operator()(int64_t e) const {
    const int32_t v = idx[e];
    return v < 0 ? rows : (uint32_t)v;
  }
};

__global__ void csr_transpose_finish_kernel(const uint32_t* __restrict__ sorted, const int32_t* __restrict__ order,
                                            int64_t n, int k, uint32_t rows, const float* __restrict__ w,
                                            const float* __restrict__ norm, int32_t* __restrict__ col,
                                            float* __restrict__ val) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n || sorted[i] >= rows) return;
  const int32_t e = order[i];
  const int32_t p = e / k;
  col[i] = p;
  if (val) {
    const float we = w ? w[e] : 1.0f;
    val[i] = norm ? we / (norm[p] + 1e-12f) : we;
  }
}

__global__ void csr_transpose_rowptr_kernel(const uint32_t* __restrict__ sorted, int64_t n, uint32_t rows,
                                            int32_t* __restrict__ rowptr) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r > rows) return;
  int64_t lo = 0, hi = n;                       // first entry whose row is at least r
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (sorted[mid] < (uint32_t)r) lo = mid + 1; else hi = mid;
  }
  rowptr[r] = (int32_t)lo;
}



// Max over the 8 children of a node (first one on ties) and which child it was.
//   out row r: node r of the coarse level when `coarse_child` is given (rows of empty
//   nodes are zeros), else the r-th non-empty node;
//   child q = 8 p + j of the p-th non-empty node: data row fine_child[q] (< 0: -inf) when
//   `fine_child` is given, else row q.
// A thread owns VEC consecutive channels of an output row.
template <typename T, int VEC>
__global__ void max_pool_kernel(const T* __restrict__ data, const int32_t* __restrict__ fine_child,
                                const int32_t* __restrict__ coarse_child, int64_t out_rows, int C,
                                T* __restrict__ out, int64_t* __restrict__ indices) {
  typedef PoolVec<T, VEC> V;
  const int lpr = C / VEC;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= out_rows * lpr) return;
  const int64_t r = t / lpr;
  const int c = (int)(t - r * lpr) * VEC;
  const int64_t p = coarse_child ? coarse_child[r] : r;
  V o;
  if (p < 0) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) o.v[v] = from_f32<T>(0.f);
    *(V*)(out + r * C + c) = o;
    return;
  }
  V x[8];
  int64_t row[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int64_t q = 8 * p + j;
    row[j] = fine_child ? fine_child[q] : q;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (row[j] >= 0) x[j] = *(const V*)(data + row[j] * C + c);
  float best[VEC];
  int bj[VEC];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float val = row[j] >= 0 ? to_f32(x[j].v[v]) : -INFINITY;
      if (j == 0 || val > best[v]) {
        best[v] = val;
        bj[v] = j;
      }
    }
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    o.v[v] = from_f32<T>(best[v]);
    indices[p * C + c + v] = bj[v];
  }
  *(V*)(out + r * C + c) = o;
}

// out row r is child j = q % 8 of parent p = q / 8 (q = out_node[r], or r): it takes
// src[src_row[p] or p][c] if indices[p][c] == j, else zero.  (Unpooling, and the gradient
// of pooling.)
template <typename T, int VEC>
__global__ void max_unpool_kernel(const T* __restrict__ src, const int64_t* __restrict__ indices,
                                  const int32_t* __restrict__ out_node, const int32_t* __restrict__ src_row,
                                  int64_t out_rows, int C, T* __restrict__ out) {
  typedef PoolVec<T, VEC> V;
  const int lpr = C / VEC;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= out_rows * lpr) return;
  const int64_t r = t / lpr;
  const int c = (int)(t - r * lpr) * VEC;
  const int64_t q = out_node ? out_node[r] : r;
  const int64_t p = q >> 3;
  const int j = (int)(q & 7);
  const int64_t s = src_row ? src_row[p] : p;
  const V x = *(const V*)(src + s * C + c);
  V o;
#pragma unroll
  for (int v = 0; v < VEC; ++v) o.v[v] = indices[p * C + c + v] == j ? x.v[v] : from_f32<T>(0.f);
  *(V*)(out + r * C + c) = o;
}

// out[p][c] = src[row of child 8 p + indices[p][c]][c] (row = fine_child[q], < 0: zero, or q).
// (The gradient of unpooling.)
template <typename T>
__global__ void max_gather_kernel(const T* __restrict__ src, const int64_t* __restrict__ indices,
                                  const int32_t* __restrict__ fine_child, int64_t parents, int C,
                                  T* __restrict__ out) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= parents * C) return;
  const int64_t p = t / C;
  const int c = (int)(t - p * C);
  const int64_t q = 8 * p + indices[t];
  const int64_t row = fine_child ? fine_child[q] : q;
  out[t] = row >= 0 ? src[row * C + c] : from_f32<T>(0.f);
}

}  // namespace ocnn

using namespace ocnn;

#define OCNN_DISPATCH_DTYPE(dtype, ...)                      \
  do {                                                       \
    if (dtype == OCNN_F32) { typedef float T; __VA_ARGS__; } \
    else if (dtype == OCNN_F16) { typedef f16 T; __VA_ARGS__; } \
    else { typedef bf16 T; __VA_ARGS__; }                    \
  } while (0)

extern "C" int ocnn_search_key(const int64_t* keys, int64_t n, const int64_t* query, int64_t m, int64_t* out,
                               void* stream) {
  OCNN_REQUIRE(n >= 0 && m >= 0, "search_key: bad sizes");
  if (m == 0) return OCNN_OK;
  OCNN_REQUIRE(query && out && (n == 0 || keys), "search_key: a required pointer is NULL");
  hipLaunchKernelGGL(search_key_kernel, dim3((unsigned)cdiv(m, 256)), dim3(256), 0, (hipStream_t)stream, keys, n,
                     query, m, out);
  return check_launch("search_key");
}

extern "C" int ocnn_search_points(const float* pts, int64_t m, int depth, const int64_t* keys, int64_t n,
                                  int bound_check, int32_t* out, void* stream) {
  OCNN_REQUIRE(n >= 0 && n < (1ll << 31) && m >= 0 && depth >= 0 && depth <= 16, "search_points: bad arguments");
  if (m == 0) return OCNN_OK;
  OCNN_REQUIRE(pts && out && (n == 0 || keys), "search_points: a required pointer is NULL");
  hipLaunchKernelGGL(search_points_kernel, dim3((unsigned)cdiv(m, 256)), dim3(256), 0, (hipStream_t)stream, pts, m,
                     depth, keys, n, bound_check, out);
  return check_launch("search_points");
}

extern "C" int ocnn_interp_linear_prepare(const float* pts, int64_t m, int depth, const int64_t* keys, int64_t n,
                                          int bound_check, int32_t* idx, float* w, float* norm, void* stream) {
  OCNN_REQUIRE(n >= 0 && n < (1ll << 31) && m >= 0 && m < (1ll << 28) && depth >= 0 && depth <= 16,
               "interp_linear_prepare: bad arguments");
  if (m == 0) return OCNN_OK;
  OCNN_REQUIRE(pts && idx && w && norm && (n == 0 || keys), "interp_linear_prepare: a required pointer is NULL");
  hipLaunchKernelGGL(interp_linear_prepare_kernel<false>, dim3((unsigned)cdiv(m * 8, 256)), dim3(256), 0,
                     (hipStream_t)stream, pts, m, depth, keys, n, LocateTree{}, bound_check, idx, w, norm);
  return check_launch("interp_linear_prepare");
}

static int locate_tree(const int32_t* const* h_children, int depth, int full_depth, int batch_size, int nempty,
                       LocateTree* t) {
  OCNN_REQUIRE(depth >= 0 && depth <= kLocateMaxDepth && full_depth >= 0 && full_depth <= 8 && batch_size >= 1 &&
                   ((int64_t)batch_size << (3 * (depth < full_depth ? depth : full_depth))) < (1ll << 31),
               "locate: depth=%d full_depth=%d batch_size=%d out of range", depth, full_depth, batch_size);
  OCNN_REQUIRE_PTRS("locate", h_children);
  for (int l = 0; l <= kLocateMaxDepth; ++l) t->children[l] = nullptr;
  for (int l = depth < full_depth ? depth : full_depth; l <= depth; ++l) {
    OCNN_REQUIRE(h_children[l] != nullptr || (l == depth && !nempty), "locate: no children array of layer %d", l);
    t->children[l] = h_children[l];
  }
  t->depth = depth;
  t->full_depth = full_depth;
  t->batch_size = batch_size;
  t->nempty = nempty;
  return OCNN_OK;
}

extern "C" int ocnn_locate_points(const float* pts, int64_t m, const int32_t* const* h_children, int depth,
                                  int full_depth, int batch_size, int nempty, int bound_check, int32_t* out,
                                  void* stream) {
  OCNN_REQUIRE(m >= 0, "locate_points: bad size");
  LocateTree t;
  if (int rc = locate_tree(h_children, depth, full_depth, batch_size, nempty, &t)) return rc;
  if (m == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("locate_points", pts, out);
  hipLaunchKernelGGL(locate_points_kernel, dim3((unsigned)cdiv(m, 256)), dim3(256), 0, (hipStream_t)stream, pts, m, t,
                     bound_check, out);
  return check_launch("locate_points");
}

extern "C" int ocnn_interp_linear_locate(const float* pts, int64_t m, const int32_t* const* h_children, int depth,
                                         int full_depth, int batch_size, int nempty, int bound_check, int32_t* idx,
                                         float* w, float* norm, void* stream) {
  OCNN_REQUIRE(m >= 0 && m < (1ll << 28), "interp_linear_locate: bad size");
  LocateTree t;
  if (int rc = locate_tree(h_children, depth, full_depth, batch_size, nempty, &t)) return rc;
  if (m == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("interp_linear_locate", pts, idx, w, norm);
  hipLaunchKernelGGL(interp_linear_prepare_kernel<true>, dim3((unsigned)cdiv(m * 8, 256)), dim3(256), 0,
                     (hipStream_t)stream, pts, m, depth, (const int64_t*)nullptr, (int64_t)0, t, bound_check, idx, w,
                     norm);
  return check_launch("interp_linear_locate");
}

extern "C" int ocnn_csr_rows(int dtype, const int32_t* rowptr, int kfixed, const int32_t* col, const float* val,
                             const void* data, int channels, const float* rowdiv, void* out, int64_t rows,
                             void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1 && rows >= 0 && (rowptr || kfixed >= 1),
               "csr_rows: bad arguments");
  if (rows == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("csr_rows", col, data, out);
  hipStream_t st = (hipStream_t)stream;
  OCNN_DISPATCH_DTYPE(dtype, {
    constexpr int VEC = 16 / sizeof(T);
    if (channels % VEC == 0 && ((uintptr_t)data % 16) == 0 && ((uintptr_t)out % 16) == 0)
      hipLaunchKernelGGL((csr_rows_kernel<T, VEC>), dim3((unsigned)cdiv(rows * (channels / VEC), 256)), dim3(256), 0,
                         st, rowptr, kfixed, col, val, (const T*)data, channels, rowdiv, (T*)out, rows);
    else
      hipLaunchKernelGGL((csr_rows_kernel<T, 1>), dim3((unsigned)cdiv(rows * channels, 256)), dim3(256), 0, st,
                         rowptr, kfixed, col, val, (const T*)data, channels, rowdiv, (T*)out, rows);
  });
  return check_launch("csr_rows");
}

struct TransposeLayout {
  int64_t sorted, order, temp, temp_bytes, total;
};

static int transpose_layout(int64_t n, TransposeLayout* L) {
  size_t sort_bytes = 0;
  auto kin = rocprim::make_transform_iterator(rocprim::make_counting_iterator<int64_t>(0), RowKey{nullptr, 0u});
  auto vin = rocprim::make_counting_iterator<int32_t>(0);
  if (rocprim::radix_sort_pairs(nullptr, sort_bytes, kin, (uint32_t*)nullptr, vin, (int32_t*)nullptr, (size_t)n, 0,
                                32) != hipSuccess)
    return OCNN_ERR_HIP;
  int64_t off = 0;
  L->sorted = off; off += align_up(n * 4, 256);
  L->order = off;  off += align_up(n * 4, 256);
  L->temp = off;
  L->temp_bytes = align_up((int64_t)sort_bytes + 256, 256);
  L->total = off + L->temp_bytes;
  return OCNN_OK;
}

extern "C" int64_t ocnn_csr_transpose_workspace_bytes(int64_t entries) {
  if (entries <= 0) return 256;
  TransposeLayout L;
  return transpose_layout(entries, &L) == OCNN_OK ? L.total : (int64_t)-1;
}

extern "C" int ocnn_csr_transpose(const int32_t* idx, const float* w, const float* norm, int64_t points, int k,
                                  int64_t rows, void* workspace, int64_t workspace_bytes, int32_t* rowptr,
                                  int32_t* col, float* val, void* stream) {
  const int64_t n = points * k;
  OCNN_REQUIRE(points >= 0 && k >= 1 && rows >= 0 && rows < (1ll << 31) - 1 && n < (1ll << 31),
               "csr_transpose: points=%lld k=%d rows=%lld out of range", (long long)points, k, (long long)rows);
  OCNN_REQUIRE((w != nullptr || norm != nullptr) == (val != nullptr),
               "csr_transpose: values are written exactly when weights or a norm are given");
  OCNN_REQUIRE_PTRS("csr_transpose", workspace, rowptr);
  OCNN_REQUIRE(n == 0 || (idx && col), "csr_transpose: a required pointer is NULL (of idx, col)");
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  TransposeLayout L;
  L.sorted = L.order = 0;
  if (n > 0) {
    if (transpose_layout(n, &L) != OCNN_OK) { set_error("csr_transpose: rocprim size query failed"); return OCNN_ERR_HIP; }
    if (workspace_bytes < L.total) { set_error("csr_transpose: workspace %lld < %lld", (long long)workspace_bytes, (long long)L.total); return OCNN_ERR_WORKSPACE; }
    uint32_t* sorted = (uint32_t*)(ws + L.sorted);
    int32_t* order = (int32_t*)(ws + L.order);
    int bits = 1;
    while ((1ll << bits) <= rows) ++bits;                  // the key `rows` of an empty entry included
    size_t tb = (size_t)L.temp_bytes;
    auto kin = rocprim::make_transform_iterator(rocprim::make_counting_iterator<int64_t>(0), RowKey{idx, (uint32_t)rows});
    auto vin = rocprim::make_counting_iterator<int32_t>(0);
    hipError_t e = rocprim::radix_sort_pairs(ws + L.temp, tb, kin, sorted, vin, order, (size_t)n, 0u, (unsigned)bits, st);
    if (e != hipSuccess) { set_error("csr_transpose: radix sort: %s", hipGetErrorString(e)); return OCNN_ERR_HIP; }
    hipLaunchKernelGGL(csr_transpose_finish_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, st, sorted, order, n, k,
                       (uint32_t)rows, w, norm, col, val);
  }
  hipLaunchKernelGGL(csr_transpose_rowptr_kernel, dim3((unsigned)cdiv(rows + 1, 256)), dim3(256), 0, st,
                     (const uint32_t*)(ws + L.sorted), n, (uint32_t)rows, rowptr);
  return check_launch("csr_transpose");
}

extern "C" int ocnn_max_pool(int dtype, const void* data, const int32_t* fine_child, const int32_t* coarse_child,
                             int64_t out_rows, int channels, void* out, int64_t* indices, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1 && out_rows >= 0, "max_pool: bad arguments");
  if (out_rows == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("max_pool", data, out, indices);
  hipStream_t st = (hipStream_t)stream;
  OCNN_DISPATCH_DTYPE(dtype, {
    constexpr int VEC = 16 / sizeof(T);
    if (channels % VEC == 0)
      hipLaunchKernelGGL((max_pool_kernel<T, VEC>), dim3((unsigned)cdiv(out_rows * (channels / VEC), 256)), dim3(256),
                         0, st, (const T*)data, fine_child, coarse_child, out_rows, channels, (T*)out, indices);
    else
      hipLaunchKernelGGL((max_pool_kernel<T, 1>), dim3((unsigned)cdiv(out_rows * channels, 256)), dim3(256), 0, st,
                         (const T*)data, fine_child, coarse_child, out_rows, channels, (T*)out, indices);
  });
  return check_launch("max_pool");
}

extern "C" int ocnn_max_unpool(int dtype, const void* src, const int64_t* indices, const int32_t* out_node,
                               const int32_t* src_row, int64_t out_rows, int channels, void* out, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1 && out_rows >= 0, "max_unpool: bad arguments");
  if (out_rows == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("max_unpool", src, indices, out);
  hipStream_t st = (hipStream_t)stream;
  OCNN_DISPATCH_DTYPE(dtype, {
    constexpr int VEC = 16 / sizeof(T);
    if (channels % VEC == 0)
      hipLaunchKernelGGL((max_unpool_kernel<T, VEC>), dim3((unsigned)cdiv(out_rows * (channels / VEC), 256)),
                         dim3(256), 0, st, (const T*)src, indices, out_node, src_row, out_rows, channels, (T*)out);
    else
      hipLaunchKernelGGL((max_unpool_kernel<T, 1>), dim3((unsigned)cdiv(out_rows * channels, 256)), dim3(256), 0, st,
                         (const T*)src, indices, out_node, src_row, out_rows, channels, (T*)out);
  });
  return check_launch("max_unpool");
}

extern "C" int ocnn_max_gather(int dtype, const void* src, const int64_t* indices, const int32_t* fine_child,
                               int64_t parents, int channels, void* out, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2 && channels >= 1 && parents >= 0, "max_gather: bad arguments");
  if (parents == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("max_gather", src, indices, out);
  hipStream_t st = (hipStream_t)stream;
  OCNN_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL(max_gather_kernel<T>, dim3((unsigned)cdiv(parents * channels, 256)), dim3(256), 0, st,
                       (const T*)src, indices, fine_child, parents, channels, (T*)out);
  });
  return check_launch("max_gather");
}
