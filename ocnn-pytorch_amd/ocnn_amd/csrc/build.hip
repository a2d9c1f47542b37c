// Octree construction: the sort of the point keys, the numbering of every layer's nodes in one
// pass over the sorted points, keys and children of all layers, the per-leaf signal averages, and
// the regrowing of an octree from split decisions.
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "common.hpp"

namespace ocnn {

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

// both of them for a cloud with normals: a leaf's points are walked once
__global__ void leaf_points_normals_kernel(const float* __restrict__ pts, const float* __restrict__ nrm,
                                           const int32_t* __restrict__ perm, const int32_t* __restrict__ seg_start,
                                           int64_t n_leaf, float* __restrict__ out_pts, float* __restrict__ out_nrm) {
  int64_t leaf = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (leaf >= n_leaf) return;
  const int32_t s = seg_start[leaf], e = seg_start[leaf + 1];
  float px = 0.f, py = 0.f, pz = 0.f, ax = 0.f, ay = 0.f, az = 0.f;
  for (int32_t q = s; q < e; ++q) {
    const int64_t at = (int64_t)perm[q] * 3;
    const float* p = pts + at;
    const float* v = nrm + at;
    px += p[0];
    py += p[1];
    pz += p[2];
    ax += v[0];
    ay += v[1];
    az += v[2];
  }
  const float cnt = (float)(e - s);
  out_pts[3 * leaf + 0] = px / cnt;
  out_pts[3 * leaf + 1] = py / cnt;
  out_pts[3 * leaf + 2] = pz / cnt;
  const float d = fmaxf(sqrtf(ax * ax + ay * ay + az * az), 1e-12f);
  out_nrm[3 * leaf + 0] = ax / d;
  out_nrm[3 * leaf + 1] = ay / d;
  out_nrm[3 * leaf + 2] = az / d;
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

// ---- the whole tree above the sorted point keys in one scan and one scatter ---------------
// A sorted point starts a new node l layers above the leaves (l = 0: a new leaf) iff its key
// differs from its predecessor's in a bit at or above 3 l, or in the batch id.  Counting those
// starts for all layers together numbers the nodes of every layer in one scan over the points.
constexpr int kBuildMaxDepth = 16;

constexpr int kBuildSpan = 1024;     // sorted points per workgroup of the counting and the scatter kernel
constexpr int kBuildThreads = 256;   // four waves, each on a run of 256 consecutive points

// number of layers at which sorted point i starts a node, minus one (-1: same leaf as i - 1)
template <typename K>
__device__ inline int start_level(const K* __restrict__ sorted, int64_t i, int key_bits, int levels) {
  if (i == 0) return levels;
  const K x = sorted[i] ^ sorted[i - 1];
  if (x == 0) return -1;
  const int hb = 63 - __builtin_clzll((unsigned long long)x);
  if (hb >= key_bits) return levels;
  const int l = hb / 3;
  return l < levels ? l : levels;
}

__device__ inline uint32_t lanes_below(unsigned long long mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// starts of nodes, by layer, among the points of each workgroup's span: sums[span][N]
template <typename K, int N>
__global__ __launch_bounds__(kBuildThreads) void build_count_kernel(const K* __restrict__ sorted, int64_t n,
                                                                    int key_bits, int levels,
                                                                    uint32_t* __restrict__ sums) {
  __shared__ uint32_t s_cnt[kBuildThreads / 64][N];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t base = (int64_t)blockIdx.x * kBuildSpan + wave * (kBuildSpan / 4);
  uint32_t cnt[N];
#pragma unroll
  for (int l = 0; l < N; ++l) cnt[l] = 0u;
#pragma unroll
  for (int it = 0; it < kBuildSpan / kBuildThreads; ++it) {
    const int64_t q = base + it * 64 + lane;
    const int lv = q < n ? start_level(sorted, q, key_bits, levels) : -1;
#pragma unroll
    for (int l = 0; l < N; ++l) cnt[l] += (uint32_t)__popcll(__ballot(lv >= l));
  }
  if (lane == 0) {
#pragma unroll
    for (int l = 0; l < N; ++l) s_cnt[wave][l] = cnt[l];
  }
  __syncthreads();
  if (threadIdx.x < N) {
    uint32_t c = 0u;
    for (int w = 0; w < kBuildThreads / 64; ++w) c += s_cnt[w][threadIdx.x];
    sums[(int64_t)blockIdx.x * N + threadIdx.x] = c;
  }
}

// offs[span][l] = starts at layer l before the span; sizes[l] = their total.  One workgroup: thread
// (chunk, l) walks a chunk of spans twice, the chunks' totals meet in LDS in between.
template <int N>
__global__ __launch_bounds__(1024) void build_offsets_kernel(const uint32_t* __restrict__ sums, int64_t spans,
                                                             int levels, uint32_t* __restrict__ offs,
                                                             int64_t* __restrict__ sizes) {
  constexpr int kChunks = 1024 / N;
  __shared__ uint32_t s_tot[kChunks][N];
  const int l = threadIdx.x % N, c = threadIdx.x / N;
  const int64_t per = (spans + kChunks - 1) / kChunks;
  const int64_t lo = c * per < spans ? c * per : spans, hi = lo + per < spans ? lo + per : spans;
  uint32_t tot = 0u;
  for (int64_t b = lo; b < hi; ++b) tot += sums[b * N + l];
  s_tot[c][l] = tot;
  __syncthreads();
  uint32_t run = 0u;
  for (int cc = 0; cc < c; ++cc) run += s_tot[cc][l];
  if (c == kChunks - 1 && l <= levels) sizes[l] = (int64_t)(run + tot);
  for (int64_t b = lo; b < hi; ++b) {
    offs[b * N + l] = run;
    run += sums[b * N + l];
  }
}

struct BuildTree {
  int64_t* keys[kBuildMaxDepth + 1];
  int32_t* children[kBuildMaxDepth + 1];
  int64_t begin[kBuildMaxDepth + 2];   // running total of the node counts, by depth
};

// full layers, and -1 in the children of every other layer
__global__ void build_init_kernel(BuildTree t, int depth, int full_depth) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= t.begin[depth + 1]) return;
  int d = 0;
  while (i >= t.begin[d + 1]) ++d;
  const int64_t j = i - t.begin[d];
  if (d <= full_depth) {
    t.keys[d][j] = (j & ((1ll << (3 * d)) - 1)) | ((j >> (3 * d)) << 48);
    t.children[d][j] = d < full_depth ? (int32_t)j : -1;
  } else {
    t.children[d][j] = -1;
  }
}

// Numbers every point's nodes (its span's offsets + the starts before it inside the span, counted
// with wave ballots) and writes what the point starts: a leaf's entry in its parent's children, a
// parent's eight keys, and so on up to the deepest full layer.
template <typename K, int N>
__global__ __launch_bounds__(kBuildThreads) void build_scatter_kernel(
    const K* __restrict__ sorted, const uint32_t* __restrict__ offs, const int32_t* __restrict__ perm, int64_t n,
    int key_bits, int depth, int full_depth, BuildTree t, int64_t* __restrict__ inverse,
    int32_t* __restrict__ seg_start) {
  __shared__ uint32_t s_cnt[kBuildThreads / 64][N];
  constexpr int kIt = kBuildSpan / kBuildThreads;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t base = (int64_t)blockIdx.x * kBuildSpan + wave * (kBuildSpan / 4);
  const int levels = depth - full_depth;
  int lv[kIt];
  uint32_t run[N];
#pragma unroll
  for (int l = 0; l < N; ++l) run[l] = 0u;
#pragma unroll
  for (int it = 0; it < kIt; ++it) {
    const int64_t q = base + it * 64 + lane;
    lv[it] = q < n ? start_level(sorted, q, key_bits, levels) : -1;
#pragma unroll
    for (int l = 0; l < N; ++l) run[l] += (uint32_t)__popcll(__ballot(lv[it] >= l));
  }
  if (lane == 0) {
#pragma unroll
    for (int l = 0; l < N; ++l) s_cnt[wave][l] = run[l];
  }
  __syncthreads();
#pragma unroll
  for (int l = 0; l < N; ++l) {
    uint32_t r = offs[(int64_t)blockIdx.x * N + l];
    for (int w = 0; w < wave; ++w) r += s_cnt[w][l];
    run[l] = r;
  }
#pragma unroll
  for (int it = 0; it < kIt; ++it) {
    const int64_t q = base + it * 64 + lane;
    uint32_t s[N];                      // inclusive: nodes of layer l started up to and with this point
#pragma unroll
    for (int l = 0; l < N; ++l) {
      const unsigned long long mask = __ballot(lv[it] >= l);
      s[l] = run[l] + lanes_below(mask) + (lv[it] >= l ? 1u : 0u);
      run[l] += (uint32_t)__popcll(mask);
    }
    if (q >= n) continue;
    const int32_t leaf = (int32_t)s[0] - 1;
    inverse[perm[q]] = leaf;
    if (q == n - 1) seg_start[leaf + 1] = (int32_t)n;
    if (lv[it] < 0) continue;
    seg_start[leaf] = (int32_t)q;
    const uint64_t c = (uint64_t)sorted[q];
    const int64_t b = (int64_t)(c >> key_bits);
    const int64_t m = (int64_t)(c & ((1ull << key_bits) - 1));
    uint32_t top = 0u;
#pragma unroll
    for (int l = 0; l < N; ++l) {
      if (l == levels) top = s[l];
      if (l < N - 1 && l < levels && l <= lv[it]) {
        const int d = depth - l;
        const int64_t kl = m >> (3 * l);
        const int64_t p = (int64_t)s[l + 1 < N ? l + 1 : l] - 1;
        t.children[d][(p << 3) | (kl & 7)] = (int32_t)s[l] - 1;
        if (l + 1 <= lv[it]) {
          const int64_t first = (b << 48) | ((kl >> 3) << 3);
          int64_t* dst = t.keys[d] + (p << 3);
#pragma unroll
          for (int j = 0; j < 8; ++j) dst[j] = first + j;
        }
      }
    }
    if (lv[it] >= levels) {
      const int64_t at = (b << (3 * full_depth)) | (m >> (3 * levels));
      if (at < t.begin[full_depth + 1] - t.begin[full_depth])      // a batch id beyond batch_size has no node
        t.children[full_depth][at] = (int32_t)top - 1;
    }
  }
}

using ForceOnesweep = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                                 rocprim::default_config, 0>;

struct BuildLayout {
  int64_t csorted, sums, offs, temp, temp_bytes, total, spans;
};

// batch id packed right above the Morton bits, read straight from the 64-bit keys by the sort
template <typename K>
struct PackKey {
  int key_bits;
  __host__ __device__ K operator()(int64_t key) const {
    const uint64_t k = (uint64_t)key;
    return (K)(((k >> 48) << key_bits) | (k & ((1ull << key_bits) - 1)));
  }
};

template <typename K, int N>
static int build_layout_t(int64_t n, BuildLayout* L) {
  size_t sort_bytes = 0;
  auto kin = rocprim::make_transform_iterator((const int64_t*)nullptr, PackKey<K>{0});
  auto vin = rocprim::make_counting_iterator<int32_t>(0);
  hipError_t e = rocprim::radix_sort_pairs<ForceOnesweep>(nullptr, sort_bytes, kin, (K*)nullptr, vin,
                                                          (int32_t*)nullptr, (size_t)n, 0, 8 * sizeof(K));
  if (e != hipSuccess) return OCNN_ERR_HIP;
  L->spans = cdiv(n, kBuildSpan);
  int64_t off = 0;
  L->csorted = off; off += align_up(n * (int64_t)sizeof(K), 256);
  L->sums = off;    off += align_up(L->spans * N * 4, 256);
  L->offs = off;    off += align_up(L->spans * N * 4, 256);
  L->temp = off;
  L->temp_bytes = align_up((int64_t)sort_bytes + 256, 256);
  L->total = off + L->temp_bytes;
  return OCNN_OK;
}

template <typename K, int N>
static int build_scan_t(const int64_t* key, int64_t n, int key_bits, int batch_bits, int levels, char* ws,
                        int64_t ws_bytes, int32_t* perm, int64_t* sizes, hipStream_t st) {
  BuildLayout L;
  if (build_layout_t<K, N>(n, &L) != OCNN_OK) { set_error("octree_build_scan: rocprim size query failed"); return OCNN_ERR_HIP; }
  if (ws_bytes < L.total) { set_error("octree_build_scan: workspace %lld < %lld", (long long)ws_bytes, (long long)L.total); return OCNN_ERR_WORKSPACE; }
  K* csorted = (K*)(ws + L.csorted);
  uint32_t* sums = (uint32_t*)(ws + L.sums);
  uint32_t* offs = (uint32_t*)(ws + L.offs);
  size_t tb = (size_t)L.temp_bytes;
  auto kin = rocprim::make_transform_iterator(key, PackKey<K>{key_bits});
  auto vin = rocprim::make_counting_iterator<int32_t>(0);
  hipError_t e = rocprim::radix_sort_pairs<ForceOnesweep>(ws + L.temp, tb, kin, csorted, vin, perm, (size_t)n, 0u,
                                                          (unsigned)(key_bits + batch_bits), st);
  if (e != hipSuccess) { set_error("octree_build_scan: radix sort: %s", hipGetErrorString(e)); return OCNN_ERR_HIP; }
  hipLaunchKernelGGL((build_count_kernel<K, N>), dim3((unsigned)L.spans), dim3(kBuildThreads), 0, st, csorted, n,
                     key_bits, levels, sums);
  hipLaunchKernelGGL(build_offsets_kernel<N>, dim3(1), dim3(1024), 0, st, sums, L.spans, levels, offs, sizes);
  return check_launch("octree_build_scan");
}

template <typename K, int N>
static int build_fill_t(const char* ws, int64_t n, int key_bits, int depth, int full_depth, const BuildTree& t,
                        const int32_t* perm, int64_t* inverse, int32_t* seg_start, hipStream_t st) {
  BuildLayout L;
  if (build_layout_t<K, N>(n, &L) != OCNN_OK) { set_error("octree_build_fill: rocprim size query failed"); return OCNN_ERR_HIP; }
  const K* csorted = (const K*)(ws + L.csorted);
  const uint32_t* offs = (const uint32_t*)(ws + L.offs);
  hipLaunchKernelGGL(build_init_kernel, dim3((unsigned)cdiv(t.begin[depth + 1], 256)), dim3(256), 0, st, t, depth,
                     full_depth);
  hipLaunchKernelGGL((build_scatter_kernel<K, N>), dim3((unsigned)L.spans), dim3(kBuildThreads), 0, st, csorted, offs,
                     perm, n, key_bits, depth, full_depth, t, inverse, seg_start);
  return check_launch("octree_build_fill");
}

// key type and counter count of a build: 32-bit sort keys when batch id and Morton bits fit
#define OCNN_BUILD_DISPATCH(CALL)                                   \
  do {                                                               \
    const bool narrow = key_bits + batch_bits <= 32;                 \
    if (levels + 1 <= 8) {                                           \
      if (narrow) return CALL(uint32_t, 8); else return CALL(uint64_t, 8);   \
    } else {                                                         \
      if (narrow) return CALL(uint32_t, 16); else return CALL(uint64_t, 16); \
    }                                                                \
  } while (0)

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

extern "C" int64_t ocnn_build_level_workspace_bytes(int64_t n) {
  if (n <= 0) return 256;
  LevelLayout L;
  if (level_layout(n, &L) != OCNN_OK) return -1;
  return L.total;
}

// A full layer: every node of every octree of the batch exists, in key order.
__global__ void full_layer_kernel(int depth, int64_t total, int32_t child_fill, int64_t* __restrict__ keys,
                                  int32_t* __restrict__ children) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t b = i >> (3 * depth);
  keys[i] = (i & ((1ll << (3 * depth)) - 1)) | (b << 48);
  children[i] = child_fill < 0 ? child_fill : (int32_t)i;
}

extern "C" int ocnn_build_full_layer(int depth, int batch_size, int with_children, int64_t* keys,
                                     int32_t* children, void* stream) {
  OCNN_REQUIRE(depth >= 0 && depth <= 8 && batch_size >= 1 && ((int64_t)batch_size << (3 * depth)) < (1ll << 31),
               "build_full_layer: depth=%d batch_size=%d out of range", depth, batch_size);
  OCNN_REQUIRE_PTRS("build_full_layer", keys, children);
  const int64_t total = (int64_t)batch_size << (3 * depth);
  hipLaunchKernelGGL(full_layer_kernel, dim3((unsigned)cdiv(total, 256)), dim3(256), 0, (hipStream_t)stream, depth,
                     total, with_children ? 0 : -1, keys, children);
  return check_launch("build_full_layer");
}

extern "C" int ocnn_split_children(const int32_t* split, int64_t n, void* workspace, int64_t workspace_bytes,
                                   int32_t* children, int64_t* count, void* stream) {
  OCNN_REQUIRE(n > 0 && n < (1ll << 28), "split_children: n=%lld out of range", (long long)n);
  OCNN_REQUIRE_PTRS("split_children", split, workspace, children, count);
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
  OCNN_REQUIRE_PTRS("grow_layer", key_above, nempty_index, keys, children);
  hipLaunchKernelGGL(grow_layer_kernel, dim3(cdiv(8 * n_nempty, 256)), dim3(256), 0, (hipStream_t)stream,
                     key_above, nempty_index, 8 * n_nempty, keys, children);
  return check_launch("grow_layer");
}

extern "C" int ocnn_leaf_average(const float* src, int channels, const int32_t* perm,
                                 const int32_t* seg_start, int64_t n_leaf, int mode, float* out,
                                 void* stream) {
  OCNN_REQUIRE(channels > 0 && n_leaf > 0, "leaf_average: channels=%d n_leaf=%lld", channels,
               (long long)n_leaf);
  OCNN_REQUIRE_PTRS("leaf_average", src, perm, seg_start, out);
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

extern "C" int ocnn_leaf_points_normals(const float* pts, const float* normals, const int32_t* perm,
                                        const int32_t* seg_start, int64_t n_leaf, float* out_pts, float* out_normals,
                                        void* stream) {
  OCNN_REQUIRE(n_leaf > 0, "leaf_points_normals: n_leaf=%lld", (long long)n_leaf);
  OCNN_REQUIRE_PTRS("leaf_points_normals", pts, normals, perm, seg_start, out_pts, out_normals);
  hipLaunchKernelGGL(leaf_points_normals_kernel, dim3((unsigned)cdiv(n_leaf, 256)), dim3(256), 0, (hipStream_t)stream,
                     pts, normals, perm, seg_start, n_leaf, out_pts, out_normals);
  return check_launch("leaf_points_normals");
}

// ---- fused build ---------------------------------------------------------------------------
static int build_args_ok(int64_t n, int depth, int full_depth, int batch_bits) {
  OCNN_REQUIRE(n > 0 && n < (1ll << 31), "octree_build: n=%lld out of range", (long long)n);
  OCNN_REQUIRE(depth >= 1 && depth <= kBuildMaxDepth && full_depth >= 0 && full_depth <= depth && full_depth <= 8,
               "octree_build: depth=%d full_depth=%d out of range", depth, full_depth);
  OCNN_REQUIRE(batch_bits >= 0 && batch_bits <= 15, "octree_build: batch_bits=%d out of range", batch_bits);
  // (a point counts its node starts in depth - full_depth + 1 layers, sixteen counters at most)
  OCNN_REQUIRE(depth - full_depth + 1 <= 16, "octree_build: %d layers below the full ones, at most 15",
               depth - full_depth);
  return OCNN_OK;
}

extern "C" int64_t ocnn_octree_build_workspace_bytes(int64_t n, int depth, int full_depth, int batch_bits) {
  if (n <= 0 || depth < 1 || depth > kBuildMaxDepth || full_depth < 0 || full_depth > depth ||
      depth - full_depth + 1 > 16)
    return -1;
  const int key_bits = 3 * depth, levels = depth - full_depth;
  BuildLayout L;
#define OCNN_BUILD_BYTES(K, N) (build_layout_t<K, N>(n, &L) == OCNN_OK ? L.total : (int64_t)-1)
  OCNN_BUILD_DISPATCH(OCNN_BUILD_BYTES);
#undef OCNN_BUILD_BYTES
}

extern "C" int ocnn_octree_build_scan(const int64_t* key, int64_t n, int depth, int full_depth, int batch_bits,
                                      void* workspace, int64_t workspace_bytes, int32_t* perm, int64_t* sizes,
                                      void* stream) {
  if (int rc = build_args_ok(n, depth, full_depth, batch_bits)) return rc;
  OCNN_REQUIRE_PTRS("octree_build_scan", key, workspace, perm, sizes);
  const int key_bits = 3 * depth, levels = depth - full_depth;
#define OCNN_BUILD_SCAN(K, N) \
  build_scan_t<K, N>(key, n, key_bits, batch_bits, levels, (char*)workspace, workspace_bytes, perm, sizes, (hipStream_t)stream)
  OCNN_BUILD_DISPATCH(OCNN_BUILD_SCAN);
#undef OCNN_BUILD_SCAN
}

extern "C" int ocnn_octree_build_fill(const void* workspace, int64_t n, int depth, int full_depth, int batch_size,
                                      int batch_bits, const int64_t* h_sizes, const int32_t* perm,
                                      int64_t* const* h_keys, int32_t* const* h_children, int64_t* inverse,
                                      int32_t* seg_start, void* stream) {
  if (int rc = build_args_ok(n, depth, full_depth, batch_bits)) return rc;
  OCNN_REQUIRE(batch_size >= 1 && batch_size <= (1 << batch_bits) && ((int64_t)batch_size << (3 * full_depth)) < (1ll << 31),
               "octree_build_fill: batch_size=%d does not fit batch_bits=%d / full_depth=%d", batch_size, batch_bits,
               full_depth);
  OCNN_REQUIRE_PTRS("octree_build_fill", workspace, h_sizes, perm, h_keys, h_children, inverse, seg_start);
  const int key_bits = 3 * depth, levels = depth - full_depth;
  BuildTree t;
  t.begin[0] = 0;
  for (int d = 0; d <= depth; ++d) {
    const int64_t nnum = d <= full_depth ? ((int64_t)batch_size << (3 * d)) : 8 * h_sizes[depth - d + 1];
    OCNN_REQUIRE(nnum > 0 && nnum < (1ll << 31) && h_keys[d] && h_children[d],
                 "octree_build_fill: depth %d: %lld nodes or a missing array", d, (long long)nnum);
    t.keys[d] = h_keys[d];
    t.children[d] = h_children[d];
    t.begin[d + 1] = t.begin[d] + nnum;
  }
  OCNN_REQUIRE(h_sizes[levels] <= ((int64_t)batch_size << (3 * full_depth)),
               "octree_build_fill: %lld nodes at the deepest full layer of %d octrees", (long long)h_sizes[levels],
               batch_size);
#define OCNN_BUILD_FILL(K, N) \
  build_fill_t<K, N>((const char*)workspace, n, key_bits, depth, full_depth, t, perm, inverse, seg_start, (hipStream_t)stream)
  OCNN_BUILD_DISPATCH(OCNN_BUILD_FILL);
#undef OCNN_BUILD_FILL
}
