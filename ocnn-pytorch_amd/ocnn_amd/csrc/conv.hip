// Convolution engine: gather-GEMM (forward / data gradient in gather form) and
// the split-K weight gradient, as MFMA kernels for f16/bf16 with channel counts
// that are multiples of 32, and as plain kernels for everything else.
//
// MFMA operand layout used throughout (v_mfma_f32_16x16x32_{f16,bf16}):
//   A (16 x 32): lane l holds A[l % 16][8 * (l / 16) + j], j = 0..7
//   B (32 x 16): lane l holds B[8 * (l / 16) + j][l % 16], j = 0..7
//   D (16 x 16): lane l holds D[4 * (l / 16) + r][l % 16], r = 0..3
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "reduce.hpp"
#include "mma.hpp"

namespace ocnn {

// --------------------------------------------------------------------------
// weight packing: (K, cin, cout) [or (K, cout, cin)] -> A-operand fragments
// --------------------------------------------------------------------------
// layout: [cout_tile][unit = k * (cin / CB) + cb][s][t][lane][8]
template <typename T>
__global__ void pack_weights_kernel(const T* __restrict__ w, T* __restrict__ out, int K, int cin,
                                    int cout, int CB, int MT, int transposed, int reverse) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)K * cin * cout;
  if (e >= total) return;
  const int KS = CB / 32;
  const int ncb = cin / CB;
  int j = (int)(e & 7);
  int lane = (int)((e >> 3) & 63);
  int64_t r = e >> 9;
  int t = (int)(r % MT); r /= MT;
  int s = (int)(r % KS); r /= KS;
  int64_t units = (int64_t)K * ncb;
  int64_t u = r % units;
  int ct = (int)(r / units);
  int k = (int)(u / ncb), cb = (int)(u % ncb);
  int g = lane >> 4, i = lane & 15;
  int chan = cb * CB + (CB == 64 ? 16 * g + 8 * s + j : 8 * g + j);
  int co = ct * 16 * MT + (i >> 2) * (4 * MT) + 4 * t + (i & 3);
  int kk = reverse ? K - 1 - k : k;
  out[e] = transposed ? w[((int64_t)kk * cout + co) * cin + chan]
                      : w[((int64_t)kk * cin + chan) * cout + co];
}

// --------------------------------------------------------------------------
// gather-GEMM, MFMA
// --------------------------------------------------------------------------
// One workgroup (4 waves) owns 4*NT*16 output rows and 16*MT output channels.
// Output rows are the N dimension of the MFMA, output channels the M dimension,
// so that a lane ends up with 4*MT consecutive channels of one row.
// O is the output (and bias) type: T, or float when the operands are bf16 pieces of fp32 data.
template <typename T, typename O, int CB, int MT, int NT>
__global__ __launch_bounds__(256) void conv_gather_mfma_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const int32_t* __restrict__ table,
    const T* __restrict__ wpk, const O* __restrict__ bias, O* __restrict__ out,
    int64_t rows_out, int K, int cin, int cout, int64_t tiles, int64_t tiles_per_xcd) {
  constexpr int KS = CB / 32;
  constexpr int ROWS = 4 * NT * 16;
  constexpr int UNIT = KS * MT * 512;                 // elements per weight unit
  constexpr int WL = (KS * MT * 64 + 255) / 256;      // 16-byte chunks per thread
  __shared__ int32_t s_idx[ROWS * 27];
  __shared__ __attribute__((aligned(16))) T s_w[2][UNIT];

  const int64_t tile = xcd_tile(blockIdx.x, tiles_per_xcd);
  if (tile >= tiles) return;
  const int ct = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, r16 = lane & 15;
  const int64_t row0 = tile * ROWS;
  const int ncb = cin / CB;
  const int units = K * ncb;

  // neighbour indices of the tile -> LDS (coalesced), -1 past the end
  {
    const int64_t base = row0 * K;
    const int64_t lim = rows_out * (int64_t)K;
    for (int e = tid; e < ROWS * K; e += 256)
      s_idx[e] = (base + e < lim) ? table[base + e] : -1;
  }
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const T* wbase = wpk + (int64_t)ct * units * UNIT;
  const uint32_t row_bytes = (uint32_t)cin * (uint32_t)sizeof(T);
  const uint32_t lane_off = (uint32_t)g * (CB / 4) * (uint32_t)sizeof(T);

  u32x4 wreg[WL];
#pragma unroll
  for (int c = 0; c < WL; ++c) {
    int ch = tid + c * 256;
    if (ch < KS * MT * 64) wreg[c] = *(const u32x4*)(wbase + (int64_t)ch * 8);
  }
#pragma unroll
  for (int c = 0; c < WL; ++c) {
    int ch = tid + c * 256;
    if (ch < KS * MT * 64) *(u32x4*)(&s_w[0][ch * 8]) = wreg[c];
  }
  __syncthreads();

  f32x4 acc[MT][NT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[t][n] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 bcur[NT][KS], bnext[NT][KS];
  const int lrow = wave * NT * 16 + r16;
  auto gather = [&](int u, u32x4 (&b)[NT][KS]) {
    int k = u / ncb, cb = u - k * ncb;
    uint32_t coff = (uint32_t)cb * CB * (uint32_t)sizeof(T) + lane_off;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      int32_t idx = s_idx[(lrow + n * 16) * K + k];
      uint32_t off = (uint32_t)idx * row_bytes + coff;
#pragma unroll
      for (int s = 0; s < KS; ++s)
        b[n][s] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, off + 16 * s, 0, 0);
    }
  };
  gather(0, bcur);

  int cur = 0;
  for (int u = 0; u < units; ++u) {
    const bool more = u + 1 < units;
    if (more) {
      const T* wsrc = wbase + (int64_t)(u + 1) * UNIT;
#pragma unroll
      for (int c = 0; c < WL; ++c) {
        int ch = tid + c * 256;
        if (ch < KS * MT * 64) wreg[c] = *(const u32x4*)(wsrc + (int64_t)ch * 8);
      }
      gather(u + 1, bnext);
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      u32x4 a[MT];
#pragma unroll
      for (int t = 0; t < MT; ++t) a[t] = *(const u32x4*)(&s_w[cur][((s * MT + t) * 64 + lane) * 8]);
#pragma unroll
      for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t][n] = Mma<T>::run(a[t], bcur[n][s], acc[t][n]);
    }
    if (more) {
#pragma unroll
      for (int c = 0; c < WL; ++c) {
        int ch = tid + c * 256;
        if (ch < KS * MT * 64) *(u32x4*)(&s_w[cur ^ 1][ch * 8]) = wreg[c];
      }
    }
    __syncthreads();
    if (more) {
#pragma unroll
      for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int s = 0; s < KS; ++s) bcur[n][s] = bnext[n][s];
    }
    cur ^= 1;
  }

  // epilogue: lane holds channels ct*16*MT + g*4*MT + [0, 4*MT) of row lrow + n*16
  const int co0 = ct * 16 * MT + g * 4 * MT;
  float bv[4 * MT];
#pragma unroll
  for (int c = 0; c < 4 * MT; ++c) bv[c] = bias ? to_f32(bias[co0 + c]) : 0.f;
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    int64_t row = row0 + lrow + n * 16;
    if (row >= rows_out) continue;
    O* dst = out + row * cout + co0;
    if constexpr (std::is_same<O, float>::value) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
        *(f32x4*)(dst + 4 * t) = f32x4{acc[t][n][0] + bv[4 * t + 0], acc[t][n][1] + bv[4 * t + 1],
                                       acc[t][n][2] + bv[4 * t + 2], acc[t][n][3] + bv[4 * t + 3]};
    } else {
      unsigned pk[2 * MT];
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        pk[2 * t + 0] = pack2<T>(acc[t][n][0] + bv[4 * t + 0], acc[t][n][1] + bv[4 * t + 1]);
        pk[2 * t + 1] = pack2<T>(acc[t][n][2] + bv[4 * t + 2], acc[t][n][3] + bv[4 * t + 3]);
      }
      if constexpr (MT >= 2) {
#pragma unroll
        for (int c = 0; c < 2 * MT; c += 4)
          *(u32x4*)(dst + 2 * c) = u32x4{pk[c], pk[c + 1], pk[c + 2], pk[c + 3]};
      } else {
        *(u32x2*)(dst) = u32x2{pk[0], pk[1]};
      }
    }
  }
}

// fp32 data as three bf16 pieces: x = hi + lo (+ 2^-17 |x|), and
// x * w = hi_x hi_w + hi_x lo_w + lo_x hi_w (+ 3 * 2^-18 |x w|), so a bf16 MFMA over the
// input channels [hi | hi | lo] against the weights [hi; lo; hi] accumulates, in fp32,
// the fp32 product to about 1e-5 relative.
__global__ void split3_rows_kernel(const float* __restrict__ x, int64_t n, int cin,
                                   bf16* __restrict__ out) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n * cin) return;
  int64_t r = e / cin;
  int c = (int)(e % cin);
  float v = x[e];
  bf16 hi = (bf16)v;
  bf16 lo = (bf16)(v - (float)hi);
  bf16* o = out + r * 3 * cin;
  o[c] = hi;
  o[cin + c] = hi;
  o[2 * cin + c] = lo;
}

// (K, cin, cout) -> (K, 3 cin, cout) rows [hi; lo; hi]; stored transposed (K, cout, cin) ->
// (K, cout, 3 cin) columns [hi | lo | hi]
__global__ void split3_weights_kernel(const float* __restrict__ w, int K, int cin, int cout,
                                      int transposed, bf16* __restrict__ out) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)K * cin * cout) return;
  float v = w[e];
  bf16 hi = (bf16)v;
  bf16 lo = (bf16)(v - (float)hi);
  if (transposed) {
    int ci = (int)(e % cin);
    int64_t kc = e / cin;                        // k * cout + co
    bf16* o = out + kc * 3 * cin;
    o[ci] = hi;
    o[cin + ci] = lo;
    o[2 * cin + ci] = hi;
  } else {
    int co = (int)(e % cout);
    int ci = (int)((e / cout) % cin);
    int64_t k = e / ((int64_t)cin * cout);
    bf16* o = out + k * 3 * cin * cout + co;
    o[(int64_t)ci * cout] = hi;
    o[(int64_t)(cin + ci) * cout] = lo;
    o[(int64_t)(2 * cin + ci) * cout] = hi;
  }
}


// --------------------------------------------------------------------------
// gather-GEMM, plain (any dtype, any channel count)
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void conv_gather_plain_kernel(
    const T* __restrict__ in, int64_t rows_in, const int32_t* __restrict__ table,
    const T* __restrict__ w, const T* __restrict__ bias, T* __restrict__ out, int64_t rows_out,
    int K, int cin, int cout, int transposed, int reverse) {
  constexpr int RB = 16, CCH = 128;       // rows per block, input-channel chunk
  __shared__ float s_x[RB][CCH];
  __shared__ int32_t s_i[RB];
  const int tid = threadIdx.x;
  const int r = tid >> 4, cg = tid & 15;
  const int64_t row = (int64_t)blockIdx.x * RB + r;
  for (int co_blk = 0; co_blk < cout; co_blk += 128) {
    float acc[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) acc[m] = 0.f;
    for (int k = 0; k < K; ++k) {
      const int kk = reverse ? K - 1 - k : k;
      __syncthreads();
      if (tid < RB) {
        int64_t rr = (int64_t)blockIdx.x * RB + tid;
        int32_t v = rr < rows_out ? table[rr * K + k] : -1;
        s_i[tid] = (v >= 0 && v < rows_in) ? v : -1;
      }
      for (int c0 = 0; c0 < cin; c0 += CCH) {
        __syncthreads();
        for (int e = tid; e < RB * CCH; e += 256) {
          int rr = e / CCH, cc = e % CCH;
          int32_t idx = s_i[rr];
          s_x[rr][cc] = (idx >= 0 && c0 + cc < cin) ? to_f32(in[(int64_t)idx * cin + c0 + cc]) : 0.f;
        }
        __syncthreads();
        if (s_i[r] < 0) continue;
        int cend = min(CCH, cin - c0);
        for (int cc = 0; cc < cend; ++cc) {
          float xv = s_x[r][cc];
          int ci = c0 + cc;
#pragma unroll
          for (int m = 0; m < 8; ++m) {
            int co = co_blk + cg + 16 * m;
            if (co < cout) {
              float wv = to_f32(transposed ? w[((int64_t)kk * cout + co) * cin + ci]
                                           : w[((int64_t)kk * cin + ci) * cout + co]);
              acc[m] += xv * wv;
            }
          }
        }
      }
    }
    if (row < rows_out) {
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        int co = co_blk + cg + 16 * m;
        if (co < cout) out[row * cout + co] = from_f32<T>(acc[m] + (bias ? to_f32(bias[co]) : 0.f));
      }
    }
  }
}

// --------------------------------------------------------------------------
// weight gradient, MFMA: partial[s][k][a][b] = sum over the rows of split s
// --------------------------------------------------------------------------
// M = x channels (a), N = g channels (b), reduction = rows, 32 rows per MFMA.
// Both operands are needed "transposed" (a lane wants 8 consecutive rows of one
// channel): tiles are staged row-major in LDS and read with the transposing
// LDS load.
template <typename T>
__device__ __forceinline__ u32x4 read_frag_t(const T* tile, int pitch, int c0, int lane) {
  const int g = lane >> 4, i = lane & 15;
  // lane i of a 16-lane group addresses 4 consecutive channels of row i/4 and
  // receives channel c0+i of rows 0..3 of the group's block
  const T* p = tile + (8 * g + (i >> 2)) * pitch + c0 + 4 * (i & 3);
  u32x2 lo = Mma<T>::read_tr(p);
  u32x2 hi = Mma<T>::read_tr(p + 4 * pitch);
  return u32x4{lo[0], lo[1], hi[0], hi[1]};
}

// TILE = 64: wave w owns x-channel tile w and all 4 g-channel tiles.
// TILE = 32: wave w owns x-channel tile w/2 and g-channel tile w%2.
template <typename T, int TILE, int KG>
__global__ __launch_bounds__(256) void conv_wgrad_mfma_kernel(
    const T* __restrict__ x, uint32_t x_bytes, const T* __restrict__ gmat, uint32_t g_bytes,
    const int32_t* __restrict__ table, int64_t rows, int K, int ca, int cb,
    int64_t rows_per_split, float* __restrict__ partial) {
  constexpr int PITCH = TILE + 8;
  constexpr int CH16 = TILE / 8;                   // 16-byte chunks per tile row
  constexpr int LOADS = (32 * CH16) / 256 ? (32 * CH16) / 256 : 1;  // per thread per tile
  constexpr int NB = TILE == 64 ? 4 : 1;           // g tiles per wave
  __shared__ __attribute__((aligned(16))) T s_g[32 * PITCH];
  __shared__ __attribute__((aligned(16))) T s_x[KG][32 * PITCH];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int split = blockIdx.x;
  const int kgroups = (K + KG - 1) / KG;
  const int kg = blockIdx.y % kgroups;
  const int atile = blockIdx.y / kgroups;          // x-channel block
  const int btile = blockIdx.z;                    // g-channel block
  const int k0 = kg * KG;
  const int64_t r_begin = (int64_t)split * rows_per_split;
  const int64_t r_end = min(rows, r_begin + rows_per_split);

  const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, x_bytes);
  const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(gmat, g_bytes);
  const bool loader = tid < 32 * CH16;             // TILE=32: only 128 threads load
  const int lrow = tid / CH16, lchunk = tid % CH16;
  const uint32_t a_off = ((uint32_t)atile * TILE + lchunk * 8) * (uint32_t)sizeof(T);
  const uint32_t b_off = ((uint32_t)btile * TILE + lchunk * 8) * (uint32_t)sizeof(T);
  const uint32_t xrow_bytes = (uint32_t)ca * (uint32_t)sizeof(T);
  const uint32_t grow_bytes = (uint32_t)cb * (uint32_t)sizeof(T);

  const int a_t = TILE == 64 ? wave : (wave >> 1);
  const int b_t0 = TILE == 64 ? 0 : (wave & 1);

  f32x4 acc[KG][NB];
#pragma unroll
  for (int q = 0; q < KG; ++q)
#pragma unroll
    for (int n = 0; n < NB; ++n) acc[q][n] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 greg, xreg[KG];
  int32_t idxn[KG];
  // table entries are fetched one step ahead of the rows they address, so the
  // row loads of the next step never wait on an index load
  auto load_idx = [&](int64_t r0) {
    int64_t row = r0 + lrow;
    bool ok = loader && row < r_end;
#pragma unroll
    for (int q = 0; q < KG; ++q) idxn[q] = (ok && k0 + q < K) ? table[row * K + k0 + q] : -1;
  };
  auto issue = [&](int64_t r0) {
    int64_t row = r0 + lrow;
    bool ok = loader && row < r_end;
    // rows past the end read as zero through an out-of-range offset
    uint32_t goff = ok ? (uint32_t)row * grow_bytes + b_off : 0xffffffffu - 64u;
    greg = __builtin_amdgcn_raw_buffer_load_b128(rs_g, goff, 0, 0);
#pragma unroll
    for (int q = 0; q < KG; ++q) {
      int32_t idx = idxn[q];
      uint32_t off = idx >= 0 ? (uint32_t)idx * xrow_bytes + a_off : 0xffffffffu - 64u;
      xreg[q] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, off, 0, 0);
    }
  };

  if (r_begin < r_end) {
    load_idx(r_begin);
    issue(r_begin);
    load_idx(r_begin + 32);
  }
  for (int64_t r0 = r_begin; r0 < r_end; r0 += 32) {
    if (loader) {
      *(u32x4*)(&s_g[lrow * PITCH + lchunk * 8]) = greg;
#pragma unroll
      for (int q = 0; q < KG; ++q) *(u32x4*)(&s_x[q][lrow * PITCH + lchunk * 8]) = xreg[q];
    }
    __syncthreads();
    if (r0 + 32 < r_end) {
      issue(r0 + 32);
      load_idx(r0 + 64);
    }
    u32x4 bf[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) bf[n] = read_frag_t<T>(s_g, PITCH, (b_t0 + n) * 16, lane);
#pragma unroll
    for (int q = 0; q < KG; ++q) {
      if (k0 + q < K) {
        u32x4 af = read_frag_t<T>(s_x[q], PITCH, a_t * 16, lane);
#pragma unroll
        for (int n = 0; n < NB; ++n) acc[q][n] = Mma<T>::run(af, bf[n], acc[q][n]);
      }
    }
    __syncthreads();
  }

  // D[4*(l/16)+r][l%16]: x channel = a_t*16 + 4g + r, g channel = (b_t0+n)*16 + l%16
  const int g4 = lane >> 4, c16 = lane & 15;
#pragma unroll
  for (int q = 0; q < KG; ++q) {
    if (k0 + q >= K) continue;
    float* dst = partial + ((int64_t)split * K + (k0 + q)) * ca * cb;
#pragma unroll
    for (int n = 0; n < NB; ++n)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int a = atile * TILE + a_t * 16 + 4 * g4 + r;
        int b = btile * TILE + (b_t0 + n) * 16 + c16;
        dst[(int64_t)a * cb + b] = acc[q][n][r];
      }
  }
}

// plain weight gradient: one thread per (a, b) pair, block = 256 pairs
template <typename T>
__global__ __launch_bounds__(256) void conv_wgrad_plain_kernel(
    const T* __restrict__ x, int64_t rows_x, const T* __restrict__ gmat,
    const int32_t* __restrict__ table, int64_t rows, int K, int ca, int cb,
    int64_t rows_per_split, float* __restrict__ partial) {
  const int split = blockIdx.x, k = blockIdx.y;
  const int64_t pair = (int64_t)blockIdx.z * 256 + threadIdx.x;
  const bool ok = pair < (int64_t)ca * cb;
  const int a = ok ? (int)(pair / cb) : 0, b = ok ? (int)(pair % cb) : 0;
  const int64_t r_begin = (int64_t)split * rows_per_split;
  const int64_t r_end = min(rows, r_begin + rows_per_split);
  float acc = 0.f;
  for (int64_t i = r_begin; i < r_end; ++i) {
    int32_t idx = table[i * K + k];
    if (idx < 0 || idx >= rows_x) continue;
    acc += to_f32(x[(int64_t)idx * ca + a]) * to_f32(gmat[i * cb + b]);
  }
  if (ok) partial[(((int64_t)split * K + k) * ca + a) * cb + b] = acc;
}

// --------------------------------------------------------------------------
// host side
// --------------------------------------------------------------------------
struct GatherPlan {
  bool mfma;
  int CB, MT, NT;
};

static GatherPlan plan_gather(int dtype, int64_t rows_in, int64_t rows_out, int cin, int cout) {
  GatherPlan p{false, 0, 0, 0};
  if (dtype == OCNN_F32) return p;
  if (cin % 32 != 0 || cout % 16 != 0) return p;
  if ((int64_t)rows_in * cin * 2 > 0xfffff000ll - (int64_t)cin * 2) return p;  // 32-bit offsets
  p.mfma = true;
  p.CB = cin % 64 == 0 ? 64 : 32;
  p.MT = cout % 64 == 0 ? 4 : (cout % 32 == 0 ? 2 : 1);
  // fewer rows per workgroup when there are few rows, to fill the 256 CUs
  int64_t ct = cout / (16 * p.MT);
  p.NT = 4;
  while (p.NT > 1 && cdiv(rows_out, 64 * p.NT) * ct < 1024) p.NT >>= 1;
  return p;
}

template <typename T, typename O, int CB, int MT, int NT>
static void launch_gather(const GatherPlan&, const void* in, int64_t rows_in, const int32_t* table,
                          int64_t rows_out, int K, int cin, int cout, const void* wpk,
                          const void* bias, void* out, hipStream_t st) {
  constexpr int ROWS = 64 * NT;
  int64_t tiles = cdiv(rows_out, ROWS);
  int64_t per_xcd = cdiv(tiles, 8);
  dim3 grid((unsigned)(per_xcd * 8), (unsigned)(cout / (16 * MT)));
  hipLaunchKernelGGL((conv_gather_mfma_kernel<T, O, CB, MT, NT>), grid, dim3(256), 0, st,
                     (const T*)in, (uint32_t)(rows_in * cin * sizeof(T)), table, (const T*)wpk,
                     (const O*)bias, (O*)out, rows_out, K, cin, cout, tiles, per_xcd);
}

template <typename T, typename O = T>
static int run_gather_mfma(const GatherPlan& p, const void* in, int64_t rows_in,
                           const int32_t* table, int64_t rows_out, int K, const void* w, int cin,
                           int cout, int w_transposed, int reverse, const void* bias, void* out,
                           void* ws, hipStream_t st) {
  int64_t total = (int64_t)K * cin * cout;
  hipLaunchKernelGGL(pack_weights_kernel<T>, dim3(cdiv(total, 256)), dim3(256), 0, st,
                     (const T*)w, (T*)ws, K, cin, cout, p.CB, p.MT, w_transposed, reverse);
#define OCNN_GATHER_CASE(cb_, mt_, nt_)                                                        \
  if (p.CB == cb_ && p.MT == mt_ && p.NT == nt_) {                                             \
    launch_gather<T, O, cb_, mt_, nt_>(p, in, rows_in, table, rows_out, K, cin, cout, ws, bias,   \
                                    out, st);                                                  \
    return check_launch("conv_gather_mfma");                                                   \
  }
  OCNN_GATHER_CASE(64, 4, 4) OCNN_GATHER_CASE(64, 4, 2) OCNN_GATHER_CASE(64, 4, 1)
  OCNN_GATHER_CASE(64, 2, 4) OCNN_GATHER_CASE(64, 2, 2) OCNN_GATHER_CASE(64, 2, 1)
  OCNN_GATHER_CASE(64, 1, 4) OCNN_GATHER_CASE(64, 1, 2) OCNN_GATHER_CASE(64, 1, 1)
  OCNN_GATHER_CASE(32, 4, 4) OCNN_GATHER_CASE(32, 4, 2) OCNN_GATHER_CASE(32, 4, 1)
  OCNN_GATHER_CASE(32, 2, 4) OCNN_GATHER_CASE(32, 2, 2) OCNN_GATHER_CASE(32, 2, 1)
  OCNN_GATHER_CASE(32, 1, 4) OCNN_GATHER_CASE(32, 1, 2) OCNN_GATHER_CASE(32, 1, 1)
#undef OCNN_GATHER_CASE
  set_error("conv_gather: no kernel for plan CB=%d MT=%d NT=%d", p.CB, p.MT, p.NT);
  return OCNN_ERR_ARG;
}

template <typename T>
static int run_gather_plain(const void* in, int64_t rows_in, const int32_t* table,
                            int64_t rows_out, int K, const void* w, int cin, int cout,
                            int w_transposed, int reverse, const void* bias, void* out,
                            hipStream_t st) {
  hipLaunchKernelGGL(conv_gather_plain_kernel<T>, dim3((unsigned)cdiv(rows_out, 16)), dim3(256), 0,
                     st, (const T*)in, rows_in, table, (const T*)w, (const T*)bias, (T*)out,
                     rows_out, K, cin, cout, w_transposed, reverse);
  return check_launch("conv_gather_plain");
}

constexpr int kWgradSlots = 3;   // kernel slots accumulated by one workgroup

struct WgradPlan {
  bool mfma;
  int TILE;
  int splits;
  int64_t rows_per_split;
};

static WgradPlan plan_wgrad(int dtype, int64_t rows_x, int64_t rows, int K, int ca, int cb) {
  WgradPlan p{false, 0, 1, rows};
  bool fits = (int64_t)rows_x * ca * 2 < 0xffff0000ll && (int64_t)rows * cb * 2 < 0xffff0000ll;
  if (dtype != OCNN_F32 && ca % 32 == 0 && cb % 32 == 0 && fits) {
    p.mfma = true;
    p.TILE = (ca % 64 == 0 && cb % 64 == 0) ? 64 : 32;
  }
  int64_t cols;   // workgroups per split
  if (p.mfma) cols = (int64_t)cdiv(K, kWgradSlots) * (ca / p.TILE) * (cb / p.TILE);
  else cols = (int64_t)K * cdiv((int64_t)ca * cb, 256);
  int64_t want = cdiv(2048, cols);
  int64_t min_rows = p.mfma ? 512 : 64;
  int64_t s = std::min<int64_t>(want, cdiv(rows, min_rows));
  int64_t cap = std::max<int64_t>(1, (48ll << 20) / ((int64_t)K * ca * cb * 4));   // <= 48 MiB of partials
  s = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(s, cap), 256));
  p.rows_per_split = std::max<int64_t>(32, align_up(cdiv(rows, s), 32));   // (rows may be 0)
  p.splits = (int)cdiv(rows, p.rows_per_split);
  return p;
}

}  // namespace ocnn

using namespace ocnn;

extern "C" int64_t ocnn_conv_workspace_bytes(int K, int cin, int cout) {
  return align_up((int64_t)K * cin * cout * 4, 256);
}

// room for the bf16 pieces of an fp32 layer: packed weights, split weights, split rows;
// 0 when the shape cannot take that path
static int64_t f32_gather_workspace(int64_t rows_in, int K, int cin, int cout) {
  if (cin % 32 != 0 || cout % 16 != 0) return 0;
  if ((int64_t)rows_in * 3 * cin * 2 > 0xfffff000ll - (int64_t)3 * cin * 2) return 0;
  return 2 * align_up((int64_t)K * 3 * cin * cout * 2, 256) + align_up(rows_in * 3 * cin * 2, 256);
}

extern "C" int64_t ocnn_conv_gather_workspace_bytes(int dtype, int64_t rows_in, int K, int cin,
                                                    int cout) {
  int64_t base = ocnn_conv_workspace_bytes(K, cin, cout);
  if (dtype == OCNN_F32) base = std::max(base, f32_gather_workspace(rows_in, K, cin, cout));
  return base;
}

extern "C" int ocnn_conv_gather(int dtype, const void* in, int64_t rows_in, const int32_t* table,
                                int64_t rows_out, int K, const void* w, int cin, int cout,
                                int w_transposed, int reverse_slots, const void* bias, void* out,
                                void* workspace, int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2, "conv_gather: dtype %d", dtype);
  OCNN_REQUIRE(K >= 1 && K <= 27 && cin >= 1 && cout >= 1, "conv_gather: K=%d cin=%d cout=%d", K,
               cin, cout);
  OCNN_REQUIRE(rows_in >= 0 && rows_out >= 0 && rows_out < (1ll << 31) && rows_in < (1ll << 31),
               "conv_gather: rows out of range");
  if (rows_out == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("conv_gather", table, w, out, workspace);
  OCNN_REQUIRE(rows_in == 0 || in, "conv_gather: in is NULL");
  hipStream_t st = (hipStream_t)stream;
  GatherPlan p = plan_gather(dtype, rows_in, rows_out, cin, cout);
  if (p.mfma) {
    if (workspace_bytes < (int64_t)K * cin * cout * 2) {
      set_error("conv_gather: workspace %lld too small", (long long)workspace_bytes);
      return OCNN_ERR_WORKSPACE;
    }
    if (dtype == OCNN_F16)
      return run_gather_mfma<f16>(p, in, rows_in, table, rows_out, K, w, cin, cout, w_transposed,
                                  reverse_slots, bias, out, workspace, st);
    return run_gather_mfma<bf16>(p, in, rows_in, table, rows_out, K, w, cin, cout, w_transposed,
                                 reverse_slots, bias, out, workspace, st);
  }
  if (dtype == OCNN_F32) {
    // bf16 pieces on the MFMA kernel when the shape allows and the caller brought the room
    // (ocnn_conv_gather_workspace_bytes); else the plain kernel
    const int64_t need = f32_gather_workspace(rows_in, K, cin, cout);
    GatherPlan p3 = plan_gather(OCNN_BF16, rows_in, rows_out, 3 * cin, cout);
    if (p3.mfma && need > 0 && workspace_bytes >= need && rows_in > 0) {
      const int64_t wbytes = align_up((int64_t)K * 3 * cin * cout * 2, 256);
      bf16* wpk = (bf16*)workspace;
      bf16* wsp = (bf16*)((char*)workspace + wbytes);
      bf16* xs = (bf16*)((char*)workspace + 2 * wbytes);
      hipLaunchKernelGGL(split3_rows_kernel, dim3((unsigned)cdiv(rows_in * cin, 256)), dim3(256), 0, st,
                         (const float*)in, rows_in, cin, xs);
      hipLaunchKernelGGL(split3_weights_kernel, dim3((unsigned)cdiv((int64_t)K * cin * cout, 256)),
                         dim3(256), 0, st, (const float*)w, K, cin, cout, w_transposed, wsp);
      return run_gather_mfma<bf16, float>(p3, xs, rows_in, table, rows_out, K, wsp, 3 * cin, cout,
                                          w_transposed, reverse_slots, bias, out, wpk, st);
    }
    return run_gather_plain<float>(in, rows_in, table, rows_out, K, w, cin, cout, w_transposed,
                                   reverse_slots, bias, out, st);
  }
  if (dtype == OCNN_F16)
    return run_gather_plain<f16>(in, rows_in, table, rows_out, K, w, cin, cout, w_transposed,
                                 reverse_slots, bias, out, st);
  return run_gather_plain<bf16>(in, rows_in, table, rows_out, K, w, cin, cout, w_transposed,
                                reverse_slots, bias, out, st);
}

extern "C" int64_t ocnn_conv_wgrad_workspace_bytes(int64_t rows, int K, int ca, int cb) {
  // upper bound over both plans: at most 256 splits
  int64_t per = (int64_t)K * ca * cb * 4;
  int64_t s = std::min<int64_t>(256, std::max<int64_t>(1, cdiv(rows, 64)));
  return align_up(per * s, 256);
}

template <typename T>
static int run_wgrad(int dtype, const void* x, int64_t rows_x, const void* g, const int32_t* table,
                     int64_t rows, int K, int ca, int cb, int out_transposed, void* gw, void* ws,
                     int64_t ws_bytes, hipStream_t st) {
  WgradPlan p = plan_wgrad(dtype, rows_x, rows, K, ca, cb);
  if (rows == 0) p.splits = 0;    // the reduction then writes zeros
  int64_t need = (int64_t)p.splits * K * ca * cb * 4;
  if (ws_bytes < need) {
    set_error("conv_wgrad: workspace %lld < %lld", (long long)ws_bytes, (long long)need);
    return OCNN_ERR_WORKSPACE;
  }
  float* partial = (float*)ws;
  if constexpr (!std::is_same<T, float>::value) {
    if (p.mfma && rows > 0) {
      constexpr int KG = kWgradSlots;
      dim3 grid(p.splits, (unsigned)(cdiv(K, KG) * (ca / p.TILE)), (unsigned)(cb / p.TILE));
      uint32_t xb = (uint32_t)(rows_x * ca * sizeof(T)), gb = (uint32_t)(rows * cb * sizeof(T));
#define OCNN_WGRAD_CASE(tile_)                                                                  \
  hipLaunchKernelGGL((conv_wgrad_mfma_kernel<T, tile_, KG>), grid, dim3(256), 0, st,            \
                     (const T*)x, xb, (const T*)g, gb, table, rows, K, ca, cb, p.rows_per_split, \
                     partial)
      if (p.TILE == 64) OCNN_WGRAD_CASE(64);
      else OCNN_WGRAD_CASE(32);
#undef OCNN_WGRAD_CASE
    }
  }
  if (!p.mfma && rows > 0) {
    dim3 grid(p.splits, K, (unsigned)cdiv((int64_t)ca * cb, 256));
    hipLaunchKernelGGL(conv_wgrad_plain_kernel<T>, grid, dim3(256), 0, st, (const T*)x, rows_x,
                       (const T*)g, table, rows, K, ca, cb, p.rows_per_split, partial);
  }
  int64_t per = (int64_t)K * ca * cb;
  (void)per;
  launch_wgrad_reduce<T>(partial, p.splits, K, ca, cb, out_transposed, (T*)gw, st);
  return check_launch("conv_wgrad");
}

// fp32 weight gradient through bf16 pieces: three passes of the MFMA kernel
// (hi_x hi_g, hi_x lo_g, lo_x hi_g) into three sets of partial sums, one reduction
static int64_t f32_wgrad_workspace(int64_t rows_x, int64_t rows, int K, int ca, int cb) {
  if (ca % 32 != 0 || cb % 32 != 0) return 0;
  if ((int64_t)rows_x * ca * 2 >= 0xffff0000ll || (int64_t)rows * cb * 2 >= 0xffff0000ll) return 0;
  WgradPlan p = plan_wgrad(OCNN_BF16, rows_x, rows, K, ca, cb);
  return 2 * align_up(rows_x * ca * 2, 256) + 2 * align_up(rows * cb * 2, 256) +
         align_up((int64_t)3 * p.splits * K * ca * cb * 4, 256);
}

static int run_wgrad_f32_split(const void* x, int64_t rows_x, const void* g, const int32_t* table,
                               int64_t rows, int K, int ca, int cb, int out_transposed, void* gw,
                               void* ws, hipStream_t st) {
  WgradPlan p = plan_wgrad(OCNN_BF16, rows_x, rows, K, ca, cb);
  const int64_t xb = align_up(rows_x * ca * 2, 256), gb = align_up(rows * cb * 2, 256);
  bf16* xh = (bf16*)ws;
  bf16* xl = (bf16*)((char*)ws + xb);
  bf16* gh = (bf16*)((char*)ws + 2 * xb);
  bf16* gl = (bf16*)((char*)ws + 2 * xb + gb);
  float* partial = (float*)((char*)ws + 2 * xb + 2 * gb);
  hipLaunchKernelGGL(split2_kernel, dim3((unsigned)cdiv(rows_x * ca, 256)), dim3(256), 0, st,
                     (const float*)x, rows_x * ca, xh, xl);
  hipLaunchKernelGGL(split2_kernel, dim3((unsigned)cdiv(rows * cb, 256)), dim3(256), 0, st,
                     (const float*)g, rows * cb, gh, gl);
  constexpr int KG = kWgradSlots;
  dim3 grid(p.splits, (unsigned)(cdiv(K, KG) * (ca / p.TILE)), (unsigned)(cb / p.TILE));
  const uint32_t xbytes = (uint32_t)(rows_x * ca * 2), gbytes = (uint32_t)(rows * cb * 2);
  const int64_t pstride = (int64_t)p.splits * K * ca * cb;
  const bf16* xs[3] = {xh, xh, xl};
  const bf16* gs[3] = {gh, gl, gh};
  for (int i = 0; i < 3; ++i) {
    if (p.TILE == 64)
      hipLaunchKernelGGL((conv_wgrad_mfma_kernel<bf16, 64, KG>), grid, dim3(256), 0, st, xs[i], xbytes,
                         gs[i], gbytes, table, rows, K, ca, cb, p.rows_per_split, partial + i * pstride);
    else
      hipLaunchKernelGGL((conv_wgrad_mfma_kernel<bf16, 32, KG>), grid, dim3(256), 0, st, xs[i], xbytes,
                         gs[i], gbytes, table, rows, K, ca, cb, p.rows_per_split, partial + i * pstride);
  }
  int64_t per = (int64_t)K * ca * cb;
  (void)per;
  launch_wgrad_reduce<float>(partial, 3 * p.splits, K, ca, cb, out_transposed, (float*)gw, st);
  return check_launch("conv_wgrad (bf16 pieces)");
}

extern "C" int64_t ocnn_conv_wgrad_workspace_bytes_for(int dtype, int64_t rows_x, int64_t rows, int K,
                                                       int ca, int cb) {
  int64_t base = ocnn_conv_wgrad_workspace_bytes(rows, K, ca, cb);
  if (dtype == OCNN_F32) base = std::max(base, f32_wgrad_workspace(rows_x, rows, K, ca, cb));
  return base;
}

extern "C" int ocnn_conv_wgrad(int dtype, const void* x, int64_t rows_x, const void* g,
                               const int32_t* table, int64_t rows, int K, int ca, int cb,
                               int out_transposed, void* gw, void* workspace,
                               int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(dtype >= 0 && dtype <= 2, "conv_wgrad: dtype %d", dtype);
  OCNN_REQUIRE(K >= 1 && K <= 27 && ca >= 1 && cb >= 1, "conv_wgrad: K=%d ca=%d cb=%d", K, ca, cb);
  OCNN_REQUIRE(rows >= 0 && rows < (1ll << 31) && rows_x >= 0 && rows_x < (1ll << 31),
               "conv_wgrad: rows out of range");
  OCNN_REQUIRE_PTRS("conv_wgrad", gw, workspace);
  OCNN_REQUIRE(rows == 0 || (g && table && (rows_x == 0 || x)), "conv_wgrad: a required pointer is NULL (of x, g, table)");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F32) {
    const int64_t need = f32_wgrad_workspace(rows_x, rows, K, ca, cb);
    if (need > 0 && workspace_bytes >= need && rows > 0 && rows_x > 0)
      return run_wgrad_f32_split(x, rows_x, g, table, rows, K, ca, cb, out_transposed, gw, workspace, st);
    return run_wgrad<float>(dtype, x, rows_x, g, table, rows, K, ca, cb, out_transposed, gw,
                            workspace, workspace_bytes, st);
  }
  if (dtype == OCNN_F16)
    return run_wgrad<f16>(dtype, x, rows_x, g, table, rows, K, ca, cb, out_transposed, gw,
                          workspace, workspace_bytes, st);
  return run_wgrad<bf16>(dtype, x, rows_x, g, table, rows, K, ca, cb, out_transposed, gw, workspace,
                         workspace_bytes, st);
}
