// Octree construction: sorted-unique of the point keys, the per-level parent
// pass, and the per-leaf signal averages.
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "common.hpp"

namespace ocnn {

__global__ void sort_prep_kernel(const int64_t* key, int64_t n, int key_bits, uint64_t* ckey,
                                 int32_t* iota) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  uint64_t k = (uint64_t)key[i];
  // pack the batch id right above the Morton bits: fewer radix passes
  ckey[i] = ((k >> 48) << key_bits) | (k & ((1ull << key_bits) - 1));
  iota[i] = (int32_t)i;
}

template <typename K>
__global__ void head_flag_kernel(const K* sorted, int64_t n, int shift, int32_t* flag) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  flag[i] = (i == 0 || (sorted[i] >> shift) != (sorted[i - 1] >> shift)) ? 1 : 0;
}

__global__ void unique_finish_kernel(const uint64_t* ckey, const int32_t* uid,
                                     const int32_t* perm, int64_t n, int key_bits,
                                     int64_t* node_key, int64_t* inverse, int32_t* seg_start,
                                     int64_t* n_unique) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int32_t u = uid[i] - 1;
  inverse[perm[i]] = u;
  if (i == 0 || uid[i - 1] != uid[i]) {
    uint64_t c = ckey[i];
    node_key[u] = (int64_t)(((c >> key_bits) << 48) | (c & ((1ull << key_bits) - 1)));
    seg_start[u] = (int32_t)i;
  }
  if (i == n - 1) {
    seg_start[u + 1] = (int32_t)n;
    *n_unique = (int64_t)u + 1;
  }
}

__global__ void counts_kernel(const int32_t* seg_start, const int64_t* n_unique, int64_t n,
                              int64_t* counts) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n || i >= *n_unique) return;
  counts[i] = (int64_t)(seg_start[i + 1] - seg_start[i]);
}

__global__ void level_count_finish_kernel(const int32_t* uid, int64_t n, int32_t* pidx,
                                          int64_t* n_parent) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int32_t u = uid[i];
  pidx[i] = u - 1;
  if (i == n - 1) *n_parent = (int64_t)u;
}

__global__ void level_fill_parent_kernel(const int64_t* node_key, const int32_t* pidx, int64_t n,
                                         int batched, int64_t* keys, int32_t* children,
                                         int64_t* next_key) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int32_t p = pidx[i];
  if (i != 0 && pidx[i - 1] == p) return;   // only the first child of a parent writes
  int64_t pk = node_key[i] >> 3;
  for (int j = 0; j < 8; ++j) {
    keys[8 * (int64_t)p + j] = (pk << 3) + j;
    children[8 * (int64_t)p + j] = -1;
  }
  next_key[p] = batched ? (((pk >> 45) << 48) | (pk & ((1ll << 45) - 1))) : pk;
}

__global__ void level_fill_child_kernel(const int64_t* node_key, const int32_t* pidx, int64_t n,
                                        int32_t* children) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  children[((int64_t)pidx[i] << 3) | (node_key[i] & 7)] = (int32_t)i;
}

__global__ void leaf_mean_kernel(const float* src, int C, const int32_t* perm,
                                 const int32_t* seg_start, int64_t n_leaf, float* out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n_leaf * C) return;
  int64_t leaf = t / C;
  int c = (int)(t % C);
  int32_t s = seg_start[leaf], e = seg_start[leaf + 1];
  float acc = 0.f;
  for (int32_t q = s; q < e; ++q) acc += src[(int64_t)perm[q] * C + c];   // point order
  out[t] = acc / (float)(e - s);
}

__global__ void leaf_normal_kernel(const float* src, const int32_t* perm,
                                   const int32_t* seg_start, int64_t n_leaf, float* out) {
  int64_t leaf = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (leaf >= n_leaf) return;
  int32_t s = seg_start[leaf], e = seg_start[leaf + 1];
  float ax = 0.f, ay = 0.f, az = 0.f;
  for (int32_t q = s; q < e; ++q) {
    const float* p = src + (int64_t)perm[q] * 3;
    ax += p[0];
    ay += p[1];
    az += p[2];
  }
  float nrm = sqrtf(ax * ax + ay * ay + az * az);
  float d = fmaxf(nrm, 1e-12f);
  out[3 * leaf + 0] = ax / d;
  out[3 * leaf + 1] = ay / d;
  out[3 * leaf + 2] = az / d;
}

// ---- regrowing an octree from split decisions (generative decoders) ----------------------
__global__ void split_flag_kernel(const int32_t* split, int64_t n, int32_t* flag) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) flag[i] = split[i] != 0;
}

// rank = inclusive count of the split nodes up to i.  A layer in which nothing is split keeps
// node 0 as its one non-empty node (the reference does, so that the next layer is never empty).
__global__ void split_children_kernel(const int32_t* flag, const int32_t* rank, int64_t n,
                                      int32_t* children, int64_t* count) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int32_t total = rank[n - 1];
  int32_t c = flag[i] ? rank[i] - 1 : -1;
  if (total == 0 && i == 0) c = 0;
  children[i] = c;
  if (i == 0) *count = total == 0 ? 1 : total;
}

// Node 8 p + j of the new layer is child j of the p-th non-empty node of the layer above:
// its key is that node's key with j appended below the batch bits; it is numbered as itself.
__global__ void grow_layer_kernel(const int64_t* key_above, const int32_t* nempty_index, int64_t n_out,
                                  int64_t* keys, int32_t* children) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_out) return;
  const int64_t k = key_above[nempty_index[i >> 3]];
  const int64_t low = k & ((1ll << 48) - 1);
  keys[i] = (k - low) | (low << 3) | (i & 7);
  children[i] = (int32_t)i;
}

struct SortLayout {
  int64_t ckey, csorted, iota, flag, uid, temp, temp_bytes, total;
};

static int sort_layout(int64_t n, SortLayout* L) {
  size_t sort_bytes = 0, scan_bytes = 0;
  hipError_t e = rocprim::radix_sort_pairs(nullptr, sort_bytes, (uint64_t*)nullptr,
                                           (uint64_t*)nullptr, (int32_t*)nullptr,
                                           (int32_t*)nullptr, (size_t)n, 0, 64);
  if (e != hipSuccess) return OCNN_ERR_HIP;
  e = rocprim::inclusive_scan(nullptr, scan_bytes, (int32_t*)nullptr, (int32_t*)nullptr,
                              (size_t)n, rocprim::plus<int32_t>());
  if (e != hipSuccess) return OCNN_ERR_HIP;
  int64_t off = 0;
  L->ckey = off;    off += align_up(n * 8, 256);
  L->csorted = off; off += align_up(n * 8, 256);
  L->iota = off;    off += align_up(n * 4, 256);
  L->flag = off;    off += align_up(n * 4, 256);
  L->uid = off;     off += align_up(n * 4, 256);
  L->temp = off;
  L->temp_bytes = (int64_t)align_up((int64_t)(sort_bytes > scan_bytes ? sort_bytes : scan_bytes) + 256, 256);
  L->total = off + L->temp_bytes;
  return OCNN_OK;
}

struct LevelLayout {
  int64_t flag, uid, temp, temp_bytes, total;
};

static int level_layout(int64_t n, LevelLayout* L) {
  size_t scan_bytes = 0;
  hipError_t e = rocprim::inclusive_scan(nullptr, scan_bytes, (int32_t*)nullptr,
                                         (int32_t*)nullptr, (size_t)n, rocprim::plus<int32_t>());
  if (e != hipSuccess) return OCNN_ERR_HIP;
  int64_t off = 0;
  L->flag = off; off += align_up(n * 4, 256);
  L->uid = off;  off += align_up(n * 4, 256);
  L->temp = off;
  L->temp_bytes = align_up((int64_t)scan_bytes + 256, 256);
  L->total = off + L->temp_bytes;
  return OCNN_OK;
}

}  // namespace ocnn

using namespace ocnn;

extern "C" int64_t ocnn_sort_unique_workspace_bytes(int64_t n) {
  if (n <= 0) return 256;
  SortLayout L;
  if (sort_layout(n, &L) != OCNN_OK) return -1;
  return L.total;
}

extern "C" int ocnn_sort_unique(const int64_t* key, int64_t n, int key_bits, int batch_bits,
                                void* workspace, int64_t workspace_bytes, int64_t* node_key,
                                int64_t* inverse, int64_t* counts, int32_t* seg_start,
                                int32_t* perm, int64_t* n_unique, void* stream) {
  OCNN_REQUIRE(n > 0 && n < (1ll << 31), "sort_unique: n=%lld out of range", (long long)n);
  OCNN_REQUIRE(key_bits >= 3 && key_bits <= 48 && batch_bits >= 0 && batch_bits <= 15,
               "sort_unique: key_bits=%d batch_bits=%d", key_bits, batch_bits);
  SortLayout L;
  if (sort_layout(n, &L) != OCNN_OK) { set_error("sort_unique: rocprim size query failed"); return OCNN_ERR_HIP; }
  if (workspace_bytes < L.total) { set_error("sort_unique: workspace %lld < %lld", (long long)workspace_bytes, (long long)L.total); return OCNN_ERR_WORKSPACE; }
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  uint64_t* ckey = (uint64_t*)(ws + L.ckey);
  uint64_t* csorted = (uint64_t*)(ws + L.csorted);
  int32_t* iota = (int32_t*)(ws + L.iota);
  int32_t* flag = (int32_t*)(ws + L.flag);
  int32_t* uid = (int32_t*)(ws + L.uid);
  dim3 grid(cdiv(n, 256)), block(256);
  hipLaunchKernelGGL(sort_prep_kernel, grid, block, 0, st, key, n, key_bits, ckey, iota);
  size_t tb = (size_t)L.temp_bytes;
  hipError_t e = rocprim::radix_sort_pairs(ws + L.temp, tb, ckey, csorted, iota, perm, (size_t)n,
                                           0u, (unsigned)(key_bits + batch_bits), st);
  if (e != hipSuccess) { set_error("sort_unique: radix sort: %s", hipGetErrorString(e)); return OCNN_ERR_HIP; }
  hipLaunchKernelGGL(head_flag_kernel<uint64_t>, grid, block, 0, st, csorted, n, 0, flag);
  tb = (size_t)L.temp_bytes;
  e = rocprim::inclusive_scan(ws + L.temp, tb, flag, uid, (size_t)n, rocprim::plus<int32_t>(), st);
  if (e != hipSuccess) { set_error("sort_unique: scan: %s", hipGetErrorString(e)); return OCNN_ERR_HIP; }
  hipLaunchKernelGGL(unique_finish_kernel, grid, block, 0, st, csorted, uid, perm, n, key_bits,
                     node_key, inverse, seg_start, n_unique);
  hipLaunchKernelGGL(counts_kernel, grid, block, 0, st, seg_start, n_unique, n, counts);
  return check_launch("sort_unique");
}

extern "C" int64_t ocnn_build_level_workspace_bytes(int64_t n) {
  if (n <= 0) return 256;
  LevelLayout L;
  if (level_layout(n, &L) != OCNN_OK) return -1;
  return L.total;
}

extern "C" int ocnn_build_level_count(const int64_t* node_key, int64_t n, void* workspace,
                                      int64_t workspace_bytes, int32_t* pidx, int64_t* n_parent,
                                      void* stream) {
  OCNN_REQUIRE(n > 0 && n < (1ll << 28), "build_level_count: n=%lld out of range", (long long)n);
  LevelLayout L;
  if (level_layout(n, &L) != OCNN_OK) { set_error("build_level: rocprim size query failed"); return OCNN_ERR_HIP; }
  if (workspace_bytes < L.total) { set_error("build_level: workspace %lld < %lld", (long long)workspace_bytes, (long long)L.total); return OCNN_ERR_WORKSPACE; }
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  int32_t* flag = (int32_t*)(ws + L.flag);
  int32_t* uid = (int32_t*)(ws + L.uid);
  dim3 grid(cdiv(n, 256)), block(256);
  hipLaunchKernelGGL(head_flag_kernel<int64_t>, grid, block, 0, st, node_key, n, 3, flag);
  size_t tb = (size_t)L.temp_bytes;
  hipError_t e = rocprim::inclusive_scan(ws + L.temp, tb, flag, uid, (size_t)n,
                                         rocprim::plus<int32_t>(), st);
  if (e != hipSuccess) { set_error("build_level: scan: %s", hipGetErrorString(e)); return OCNN_ERR_HIP; }
  hipLaunchKernelGGL(level_count_finish_kernel, grid, block, 0, st, uid, n, pidx, n_parent);
  return check_launch("build_level_count");
}

extern "C" int ocnn_build_level_fill(const int64_t* node_key, const int32_t* pidx, int64_t n,
                                     int64_t n_parent, int batched, int64_t* keys,
                                     int32_t* children, int64_t* next_key, void* stream) {
  OCNN_REQUIRE(n > 0 && n_parent > 0 && n_parent <= n, "build_level_fill: n=%lld n_parent=%lld",
               (long long)n, (long long)n_parent);
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(cdiv(n, 256)), block(256);
  hipLaunchKernelGGL(level_fill_parent_kernel, grid, block, 0, st, node_key, pidx, n, batched, keys,
                     children, next_key);
  hipLaunchKernelGGL(level_fill_child_kernel, grid, block, 0, st, node_key, pidx, n, children);
  return check_launch("build_level_fill");
}

extern "C" int ocnn_split_children(const int32_t* split, int64_t n, void* workspace, int64_t workspace_bytes,
                                   int32_t* children, int64_t* count, void* stream) {
  OCNN_REQUIRE(n > 0 && n < (1ll << 28), "split_children: n=%lld out of range", (long long)n);
  LevelLayout L;
  if (level_layout(n, &L) != OCNN_OK) { set_error("split_children: rocprim size query failed"); return OCNN_ERR_HIP; }
  if (workspace_bytes < L.total) { set_error("split_children: workspace %lld < %lld", (long long)workspace_bytes, (long long)L.total); return OCNN_ERR_WORKSPACE; }
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  int32_t* flag = (int32_t*)(ws + L.flag);
  int32_t* rank = (int32_t*)(ws + L.uid);
  dim3 grid(cdiv(n, 256)), block(256);
  hipLaunchKernelGGL(split_flag_kernel, grid, block, 0, st, split, n, flag);
  size_t tb = (size_t)L.temp_bytes;
  hipError_t e = rocprim::inclusive_scan(ws + L.temp, tb, flag, rank, (size_t)n, rocprim::plus<int32_t>(), st);
  if (e != hipSuccess) { set_error("split_children: scan: %s", hipGetErrorString(e)); return OCNN_ERR_HIP; }
  hipLaunchKernelGGL(split_children_kernel, grid, block, 0, st, flag, rank, n, children, count);
  return check_launch("split_children");
}

extern "C" int ocnn_grow_layer(const int64_t* key_above, const int32_t* nempty_index, int64_t n_nempty,
                               int64_t* keys, int32_t* children, void* stream) {
  OCNN_REQUIRE(n_nempty > 0 && n_nempty < (1ll << 28), "grow_layer: n_nempty=%lld out of range",
               (long long)n_nempty);
  hipLaunchKernelGGL(grow_layer_kernel, dim3(cdiv(8 * n_nempty, 256)), dim3(256), 0, (hipStream_t)stream,
                     key_above, nempty_index, 8 * n_nempty, keys, children);
  return check_launch("grow_layer");
}

extern "C" int ocnn_leaf_average(const float* src, int channels, const int32_t* perm,
                                 const int32_t* seg_start, int64_t n_leaf, int mode, float* out,
                                 void* stream) {
  OCNN_REQUIRE(channels > 0 && n_leaf > 0, "leaf_average: channels=%d n_leaf=%lld", channels,
               (long long)n_leaf);
  hipStream_t st = (hipStream_t)stream;
  if (mode == 1) {
    OCNN_REQUIRE(channels == 3, "leaf_average: normalise mode needs 3 channels, got %d", channels);
    hipLaunchKernelGGL(leaf_normal_kernel, dim3(cdiv(n_leaf, 256)), dim3(256), 0, st, src, perm,
                       seg_start, n_leaf, out);
  } else {
    hipLaunchKernelGGL(leaf_mean_kernel, dim3(cdiv(n_leaf * channels, 256)), dim3(256), 0, st, src,
                       channels, perm, seg_start, n_leaf, out);
  }
  return check_launch("leaf_average");
}
