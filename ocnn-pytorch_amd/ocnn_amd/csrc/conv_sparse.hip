// Gather-GEMM for sparse tables: the work follows the (output row, input row) pairs of the
// table, not rows x slots.
//
// On the non-empty nodes of a deep level only 10 - 25 % of the 27 slots of a row hold a
// neighbour; a kernel that multiplies whole slots spends most of its MFMAs on zero rows and,
// worse, streams the weights of every slot once per 128-row tile.  Here
//   * the weights stay in registers: a workgroup serves 32 output channels (blockIdx.y) and
//     walks over many tiles; its waves are NG groups of lists x 2 halves of the 32 channels
//     (NG = 4, two waves per SIMD, where LDS has room for four sets of sums, else 2); wave
//     (g, h) keeps the weights of the lists of group g for its 16 channels in the layout of
//     the MFMA A operand (<= 16 lists x cin / 32 k-steps x 4 registers).  A list of the pair
//     plan is a slot, or a range of a tile's rows of a slot that holds many pairs (the
//     centre of a 3x3x3 table holds a third of them), so that the groups carry equal loads;
//   * per tile and list the pair plan names the rows that have a neighbour, in blocks of 16
//     pairs (entry = position p of the input row among the tile's staged rows, 0 = the zero
//     row, | row r of the tile << 16; a block is filled up with entries for (0, 128): zeros
//     added to a spare row);
//   * the distinct input rows of the tile are staged in LDS once (global->LDS loads, row
//     pitch cin * 2 + 16 bytes so that 16 rows spread over the banks);
//   * a block is one v_mfma_f32_16x16x32 chain (M = 16 pairs, N = 16 channels, K = cin) whose
//     result (a lane: 4 consecutive channels of one pair) is added to fp32 accumulators of
//     the tile's 128 rows in LDS with a plain read - add - write: each slot group has its own
//     copy and a wave owns its columns, so no two waves touch the same word and the order of
//     the additions is the program order of one wave (results are reproducible; LDS float
//     atomics turned out an order of magnitude slower);
//   * at the end of a tile the two copies are added, the bias goes on, and the rows leave.
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "mma.hpp"

namespace ocnn {

constexpr int kSpRows = 128;              // rows per tile (the plan's tile size)
constexpr int kSpAccPitch = 36;           // floats per accumulator row: 144 bytes, so that the same 16-byte
                                          // piece of 16 rows falls on 16 different groups of four banks when
                                          // the rows differ mod 16 (9 r mod 16 is one to one)
constexpr int kSpAccRows = kSpRows + 1;   // + a spare row that the filling entries of a block go to
constexpr int kSpAccCopy = kSpAccRows * kSpAccPitch * 4;   // bytes of the sums of one group
constexpr int kSpLists = 32;              // lists of a plan at most
constexpr int kSpCp = 40;                 // block offsets per tile kept in LDS (>= kSpLists + 1)

struct SpGroups {                         // (a kernel argument) the four groups of a plan: lists gb[g] .. gb[g + 1] - 1
  int32_t gb[5];
};
constexpr int kSpLdsLimit = 160 * 1024;

static __device__ __forceinline__ void sp_dma16(__amdgpu_buffer_rsrc_t rs, char* dst, uint32_t off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)dst, 16, off, 0, 0, 0);
}

__host__ __device__ constexpr int sp_ent_bytes(int max_blocks) { return (max_blocks * 64 + 1023) / 1024 * 1024; }
__host__ __device__ constexpr int sp_rows_bytes(int cin, int umax) {
  return ((umax + 1) * (cin * 2 + 16) + 1023) / 1024 * 1024;
}

// Packed weights: [32-channel class][list j][half h][k-step s][lane][8] (slot of the list):
// the B operand of v_mfma_f32_16x16x32 (lane l holds B[8 (l / 16) + i][l % 16]) with
//   input channel = 32 s + 8 (lane / 16) + i,  output channel = 32 class + 16 h + lane % 16.
template <typename T>
__global__ void pack_weights_sparse_kernel(const T* __restrict__ w, T* __restrict__ out,
                                           const int32_t* __restrict__ lists, int nl, int K, int cin, int cout,
                                           int transposed, int reverse) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)nl * cin * cout) return;
  const int nks = cin >> 5;
  int i = (int)(e & 7);
  int lane = (int)((e >> 3) & 63);
  int64_t rest = e >> 9;
  int s = (int)(rest % nks);
  rest /= nks;
  int h = (int)(rest & 1);
  rest >>= 1;
  int j = (int)(rest % nl);
  int cls = (int)(rest / nl);
  int k = lists[j] & 255;
  if (reverse) k = K - 1 - k;
  int chan = 32 * s + 8 * (lane >> 4) + i;
  int co = 32 * cls + 16 * h + (lane & 15);
  out[e] = transposed ? w[((int64_t)k * cout + co) * cin + chan] : w[((int64_t)k * cin + chan) * cout + co];
}

// One workgroup: 32 output channels (blockIdx.y), tiles blockIdx.x, blockIdx.x + gridDim.x, ...
// cptr: (tiles * nl + 1) block offsets (nl lists per tile); ent: 16 entries per block.
//
// Per tile: [blocks of the tile] barrier [global->LDS loads of the next tile's rows and entries
// | the two accumulator copies are added and leave | wait for the loads] barrier.  What the
// loads need (list bounds, row numbers, block offsets) is fetched one and two tiles ahead, so
// that the only memory latency between two tiles is that of the global->LDS loads themselves.
template <typename T, int NKS, int NG, int WPC>
__global__ __launch_bounds__(128 * NG, WPC) void conv_gather_sparse_kernel(
    const T* __restrict__ in, uint32_t in_bytes, const int32_t* __restrict__ uptr,
    const int32_t* __restrict__ urows, const int32_t* __restrict__ cptr, const uint32_t* __restrict__ ent,
    uint32_t ent_bytes, const T* __restrict__ wpk, const T* __restrict__ bias, T* __restrict__ out,
    uint32_t out_bytes, uint32_t u_bytes, int64_t rows_out, int nl, SpGroups groups, int cout, int64_t tiles,
    int rows_bytes, int ent_bytes_lds, int su) {
  constexpr int NT = 128 * NG;                     // threads
  constexpr int NSL = 32 / NG;                     // lists per group at most
  constexpr int kSpAccBytes = NG * kSpAccCopy;
  constexpr int CPR = 4 * NKS + 1;                 // 16-byte chunks per staged row (one of padding)
  constexpr int PITCH = CPR * 16;
  extern __shared__ __attribute__((aligned(16))) char s_dyn[];
  // (the regions filled by global->LDS loads are whole KiB: a load always writes 1 KiB)
  char* s_rows = s_dyn;                                                  // (max distinct + 1) x PITCH
  float* s_acc = (float*)(s_dyn + rows_bytes);                           // [NG][129][32]
  uint32_t* s_ent = (uint32_t*)((char*)s_acc + kSpAccBytes);             // blocks of 16 entries
  int32_t* s_u = (int32_t*)((char*)s_ent + ent_bytes_lds);               // [2][su] row numbers (su: 256 | 512)
  int32_t* s_cp = s_u + 2 * su;                                          // [2][kSpCp] block offsets

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = wave >> 1, h = wave & 1;
  const int cls = blockIdx.y;
  const int jbase = groups.gb[g * (4 / NG)];
  const int ns = groups.gb[(g + 1) * (4 / NG)] - jbase;                  // lists of this wave
  const uint32_t pitch_g = (uint32_t)(NKS * 64);                         // bytes of an input row
  const int64_t step = gridDim.x;

  // ---- weights of this wave's slots -> registers ----
  u32x4 W[NSL][NKS];
#pragma unroll
  for (int i = 0; i < NSL; ++i) {
    const int j = min(jbase + min(i, max(ns - 1, 0)), nl - 1);
    const T* p = wpk + ((((int64_t)cls * nl + j) * 2 + h) * NKS) * 512 + lane * 8;
#pragma unroll
    for (int s = 0; s < NKS; ++s) W[i][s] = *(const u32x4*)(p + s * 512);
  }
  // bias of the 16 channels this thread writes at the end of a tile
  // (at the end of a tile a thread adds up, for one row, CH of the 32 channels)
  constexpr int CH = 32 * kSpRows / NT;
  const int wr = tid / (32 / CH), wh = tid % (32 / CH);
  float bv[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) bv[c] = bias ? to_f32(bias[32 * cls + CH * wh + c]) : 0.f;

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t rs_ent = make_rsrc(ent, ent_bytes);
  const __amdgpu_buffer_rsrc_t rs_out = make_rsrc(out, out_bytes);
  const __amdgpu_buffer_rsrc_t rs_u = make_rsrc(urows, u_bytes);
  const __amdgpu_buffer_rsrc_t rs_cp = make_rsrc(cptr, (uint32_t)((tiles * nl + 1) * 4));

  struct Meta { int32_t p0, U, cb, nb; int64_t t; };
  auto meta = [&](int64_t t) {                                           // (wave-uniform loads)
    Meta m;
    const int64_t tc = min(t, tiles - 1);
    m.t = tc;
    m.p0 = uptr[tc];
    m.U = t < tiles ? uptr[tc + 1] - m.p0 : -1;
    m.cb = cptr[tc * nl];
    m.nb = t < tiles ? cptr[tc * nl + nl] - m.cb : 0;
    return m;
  };
  // (unconditional buffer loads, out of range reads zero; what they return is only looked at
  // in put_ids, a tile later: no wait between these loads and the global->LDS loads)
  struct Ids { int32_t u0, u1, cp, U, cb; };
  auto load_ids = [&](const Meta& m) {
    Ids r;
    r.u0 = __builtin_amdgcn_raw_buffer_load_b32(rs_u, (uint32_t)(m.p0 + tid - 1) * 4u, 0, 0);
    r.u1 = __builtin_amdgcn_raw_buffer_load_b32(rs_u, (uint32_t)(m.p0 + tid + NT - 1) * 4u, 0, 0);
    r.cp = __builtin_amdgcn_raw_buffer_load_b32(rs_cp, (uint32_t)((int)m.t * nl + min(tid, nl)) * 4u, 0, 0);
    r.U = m.U;
    r.cb = m.cb;
    return r;
  };
  auto put_ids = [&](int buf, const Ids& r) {
    if (tid < su) s_u[buf * su + tid] = (tid >= 1 && tid <= r.U) ? r.u0 : -1;   // LDS row 0 = zeros
    if (su > NT) s_u[buf * su + NT + tid] = (tid + NT <= r.U) ? r.u1 : -1;
    if (tid < kSpCp) s_cp[buf * kSpCp + tid] = r.cp - r.cb;
  };
  // global->LDS loads of a tile's rows and entries (asynchronous)
  auto dma = [&](const Meta& m, int buf) {
    const int chunks = (m.U + 1) * CPR;
    // four pieces at a time: their list entries first (one LDS wait for the four), then the loads
    for (int piece0 = wave; piece0 * 64 < chunks; piece0 += 8 * NG) {
      int32_t id[4];
      uint32_t cb16[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int L = (piece0 + 2 * NG * e) * 64 + lane;
        const int p = L / CPR, c = L - p * CPR;
        id[e] = s_u[buf * su + min(p, su - 1)];
        cb16[e] = c < CPR - 1 ? (uint32_t)c * 16u : 0xffffffffu;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int piece = piece0 + 2 * NG * e;
        if (piece * 64 < chunks) {
          const uint32_t off = (id[e] >= 0 && cb16[e] != 0xffffffffu) ? (uint32_t)id[e] * pitch_g + cb16[e] : 0xffffff00u;
          sp_dma16(rs_in, s_rows + piece * 1024, off);
        }
      }
    }
    for (int piece = wave; piece * 16 < m.nb; piece += 2 * NG)           // 16 blocks (1 KiB) per load
      sp_dma16(rs_ent, (char*)s_ent + piece * 1024, (uint32_t)m.cb * 64u + (uint32_t)(piece * 1024 + lane * 16));
  };

  // ---- accumulators start at zero; so do the entries (a wave without blocks reads one) ----
  for (int i = tid; i < (kSpAccBytes + ent_bytes_lds) / 16; i += NT) ((u32x4*)s_acc)[i] = u32x4{0u, 0u, 0u, 0u};

  int64_t tile = blockIdx.x;
  Meta m_nxt = meta(tile);
  put_ids(0, load_ids(m_nxt));
  __syncthreads();
  dma(m_nxt, 0);
  m_nxt = meta(tile + step);
  Ids ids = load_ids(m_nxt);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // this lane's accumulators: piece 4 h + lane / 16 of a row (before the row's swizzle)
  char* acc_w = (char*)s_acc + g * kSpAccCopy;
  const uint32_t acc_c = (uint32_t)(4 * h + (lane >> 4)) << 4;
  const char* a_base = s_rows + 16 * (lane >> 4);
  const int em = lane & 15;
  int buf = 0;

  for (; tile < tiles; tile += step) {
    put_ids(buf ^ 1, ids);                                                // of the next tile
    const Meta m_nn = meta(tile + 2 * step);
    // ---- the blocks of this wave's slots ----
    const int32_t* cp = s_cp + buf * kSpCp;
    int b = __builtin_amdgcn_readfirstlane(cp[jbase]);
    const int bend = __builtin_amdgcn_readfirstlane(cp[jbase + ns]);
    const int blast = max(bend - 1, 0);
    u32x4 Ac[NKS], An[NKS];
    f32x4 dp = {0.f, 0.f, 0.f, 0.f};                                      // result of the block before
    char* ap = acc_w + (kSpRows * kSpAccPitch * 4 + acc_c);               // and where it goes (spare row)
    uint32_t ec, en;
    {
      ec = s_ent[min(b, blast) * 16 + em];
      const char* a = a_base + (ec & 0xffffu) * PITCH;
#pragma unroll
      for (int s = 0; s < NKS; ++s) Ac[s] = *(const u32x4*)(a + s * 64);
      en = s_ent[min(b + 1, blast) * 16 + em];
    }
#pragma unroll
    for (int i = 0; i < NSL; ++i) {
      if (i < ns) {
        const int be = __builtin_amdgcn_readfirstlane(cp[jbase + i + 1]);
        while (b < be) {
          // rows of the next block, entry of the one after, accumulators of the one before
          // (LDS reads come back in the order of their issue: the sums first, so that their
          // read - add - write does not wait for the gathered rows)
          f32x4 av = *(const f32x4*)ap;
          const uint32_t e2 = s_ent[min(b + 2, blast) * 16 + em];
          const char* a = a_base + (en & 0xffffu) * PITCH;
#pragma unroll
          for (int s = 0; s < NKS; ++s) An[s] = *(const u32x4*)(a + s * 64);
          __builtin_amdgcn_sched_barrier(0);
          f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < NKS; ++s) d = Mma<T>::run(W[i][s], Ac[s], d);
          av += dp;
          *(f32x4*)ap = av;
          dp = d;
          ap = acc_w + ((ec >> 16) * (uint32_t)(kSpAccPitch * 4) + acc_c);
          ec = en;
          en = e2;
#pragma unroll
          for (int s = 0; s < NKS; ++s) Ac[s] = An[s];
          ++b;
        }
      }
    }
    {
      f32x4 av = *(const f32x4*)ap;
      av += dp;
      *(f32x4*)ap = av;
    }
    __syncthreads();

    // ---- the next tile comes in while this one leaves ----
    ids = load_ids(m_nn);
    __builtin_amdgcn_sched_barrier(0);
    dma(m_nxt, buf ^ 1);
    __builtin_amdgcn_sched_barrier(0);
    {
      float* a0 = s_acc + wr * kSpAccPitch;
      float v[CH];
#pragma unroll
      for (int q4 = 0; q4 < CH / 4; ++q4) {
        const int pc = 4 * ((CH / 4) * wh + q4);
        f32x4 x = *(const f32x4*)(a0 + pc);
        *(f32x4*)(a0 + pc) = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int gg = 1; gg < NG; ++gg) {                                   // the groups' sums, in their order
          x += *(const f32x4*)(a0 + gg * (kSpAccCopy / 4) + pc);
          *(f32x4*)(a0 + gg * (kSpAccCopy / 4) + pc) = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) v[4 * q4 + c] = x[c] + bv[4 * q4 + c];
      }
      const int64_t row = tile * kSpRows + wr;
      unsigned pk[CH / 2];
#pragma unroll
      for (int c = 0; c < CH / 2; ++c) pk[c] = pack2<T>(v[2 * c], v[2 * c + 1]);
      // (rows past the end: out of range, dropped; every wave issues all its stores)
      const uint32_t off = row < rows_out ? (uint32_t)((row * cout + 32 * cls + CH * wh) * 2) : 0xffffff00u;
#pragma unroll
      for (int c = 0; c < CH / 8; ++c)
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{pk[4 * c], pk[4 * c + 1], pk[4 * c + 2], pk[4 * c + 3]}, rs_out,
                                               off + 16u * c, 0, 0);
    }
    // everything but the stores has landed (memory operations complete in issue order)
    if constexpr (CH == 16) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    __syncthreads();
    m_nxt = m_nn;
    buf ^= 1;
  }
}

}  // namespace ocnn

using namespace ocnn;

static int sp_su(int umax) { return umax + 1 <= 256 ? 256 : 512; }
static int sp_lds_bytes(int max_blocks, int cin, int umax, int ng) {
  return sp_rows_bytes(cin, umax) + ng * kSpAccCopy + sp_ent_bytes(max_blocks) + 2 * sp_su(umax) * 4 + 2 * kSpCp * 4;
}

extern "C" int ocnn_conv_gather_sparse_supported(int dtype, int64_t rows_in, int K, int cin, int cout,
                                                 int plan_max_distinct) {
  if (dtype != OCNN_F16 && dtype != OCNN_BF16) return 0;
  if (cin < 32 || cin > 128 || cin % 32 != 0 || cout < 32 || cout % 32 != 0 || cout > 4096) return 0;
  if (K < 1 || K > 27) return 0;
  if (plan_max_distinct < 0 || plan_max_distinct > 511 ||
      sp_lds_bytes(8 * kSpLists, cin, plan_max_distinct, 2) > kSpLdsLimit)
    return 0;
  if (rows_in < 0 || (int64_t)rows_in * cin * 2 > 0xfff00000ll) return 0;
  return 1;
}

extern "C" int64_t ocnn_conv_gather_sparse_workspace_bytes(int cin, int cout) {
  return (int64_t)kSpLists * cin * cout * 2;
}

template <typename T, int NKS, int NG, int WPC>
static void launch_sparse(const void* in, int64_t rows_in, const int32_t* uptr, const int32_t* urows, int umax,
                          int64_t plan_total, const int32_t* cptr, const uint32_t* ent, int64_t n_blocks,
                          int max_blocks, int nl, const SpGroups& groups, int64_t rows_out, int cin, int cout,
                          const void* ws, const void* bias, void* out, hipStream_t st) {
  const int lds = sp_lds_bytes(max_blocks, cin, umax, NG);
  static bool attr_set = false;
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)conv_gather_sparse_kernel<T, NKS, NG, WPC>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, kSpLdsLimit / WPC);
    attr_set = true;
  }
  const int64_t tiles = cdiv(rows_out, kSpRows);
  const int ncls = cout / 32;
  int dev = 0, n_cu = 256;
  (void)hipGetDevice(&dev);
  (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
  const int64_t gx = std::max<int64_t>(1, std::min<int64_t>(tiles, std::max(1, WPC * n_cu / ncls)));
  hipLaunchKernelGGL((conv_gather_sparse_kernel<T, NKS, NG, WPC>), dim3((unsigned)gx, (unsigned)ncls),
                     dim3(128 * NG), (size_t)lds, st, (const T*)in, (uint32_t)(rows_in * cin * 2), uptr, urows, cptr,
                     ent, (uint32_t)std::min<int64_t>(n_blocks * 64, 0xfffffff0ll), (const T*)ws, (const T*)bias,
                     (T*)out, (uint32_t)(rows_out * cout * 2), (uint32_t)(plan_total * 4), rows_out, nl, groups, cout,
                     tiles, sp_rows_bytes(cin, umax), sp_ent_bytes(max_blocks), sp_su(umax));
}

template <typename T>
static int run_sparse(const void* in, int64_t rows_in, const int32_t* uptr, const int32_t* urows, int umax,
                      int64_t plan_total, const int32_t* cptr, const uint32_t* ent, int64_t n_blocks,
                      int max_blocks, const int32_t* lists, int nl, const SpGroups& groups, int64_t rows_out, int K,
                      const void* w, int cin, int cout, int w_transposed, int reverse, const void* bias, void* out,
                      void* ws, hipStream_t st) {
  const int64_t total = (int64_t)nl * cin * cout;
  hipLaunchKernelGGL(pack_weights_sparse_kernel<T>, dim3((unsigned)cdiv(total, 256)), dim3(256), 0, st,
                     (const T*)w, (T*)ws, lists, nl, K, cin, cout, w_transposed, reverse);
  const int nks = cin / 32;
  // two waves per SIMD (one's LDS waits are the other's issue slots): two workgroups of 4 waves
  // (2 groups) per CU where they fit, else one of 8 waves (4 groups) where LDS holds four sets
  // of sums, else one workgroup of 4 waves
  const int wpc = (nks <= 3 && sp_lds_bytes(max_blocks, cin, umax, 2) <= kSpLdsLimit / 2) ? 2 : 1;
  const int ng = (wpc == 1 && sp_lds_bytes(max_blocks, cin, umax, 4) <= kSpLdsLimit) ? 4 : 2;
#define OCNN_SP_CASE(NKS_, NG_, WPC_)                                                                        \
  if (nks == NKS_ && ng == NG_ && wpc == WPC_) {                                                             \
    launch_sparse<T, NKS_, NG_, WPC_>(in, rows_in, uptr, urows, umax, plan_total, cptr, ent, n_blocks,      \
                                      max_blocks, nl, groups, rows_out, cin, cout, ws, bias, out, st);       \
    return check_launch("conv_gather_sparse");                                                               \
  }
  OCNN_SP_CASE(1, 4, 1) OCNN_SP_CASE(2, 4, 1) OCNN_SP_CASE(3, 4, 1) OCNN_SP_CASE(4, 4, 1)
  OCNN_SP_CASE(1, 2, 1) OCNN_SP_CASE(2, 2, 1) OCNN_SP_CASE(3, 2, 1) OCNN_SP_CASE(4, 2, 1)
  OCNN_SP_CASE(1, 2, 2) OCNN_SP_CASE(2, 2, 2) OCNN_SP_CASE(3, 2, 2)
#undef OCNN_SP_CASE
  set_error("conv_gather_sparse: no kernel for cin=%d", cin);
  return OCNN_ERR_ARG;
}

extern "C" int ocnn_conv_gather_sparse(int dtype, const void* in, int64_t rows_in, const int32_t* uptr,
                                       const int32_t* urows, int plan_max_distinct, int64_t plan_total,
                                       const int32_t* cptr, const uint32_t* ent, int64_t n_blocks,
                                       int max_blocks, const int32_t* lists, int n_lists,
                                       const int32_t* group_bounds, int64_t rows_out, int K, const void* w,
                                       int cin, int cout, int w_transposed, int reverse_slots, const void* bias,
                                       void* out, void* workspace, int64_t workspace_bytes, void* stream) {
  OCNN_REQUIRE(ocnn_conv_gather_sparse_supported(dtype, rows_in, K, cin, cout, plan_max_distinct),
               "conv_gather_sparse: shape not supported");
  OCNN_REQUIRE(rows_out >= 0 && rows_out < (1ll << 31) && rows_out * cout * 2 <= 0xfff00000ll &&
                   plan_total >= 0 && plan_total < (1ll << 29) && n_blocks >= 0 && n_blocks < (1ll << 25) &&
                   max_blocks >= 0 && max_blocks <= 8 * kSpLists && n_lists >= 1 && n_lists <= kSpLists,
               "conv_gather_sparse: rows or lists out of range");
  OCNN_REQUIRE_PTRS("conv_gather_sparse", group_bounds);
  SpGroups groups;
  for (int g = 0; g < 5; ++g) groups.gb[g] = group_bounds[g];
  bool ok = groups.gb[0] == 0 && groups.gb[4] == n_lists;
  for (int g = 0; g < 4; ++g) ok = ok && groups.gb[g + 1] >= groups.gb[g] && groups.gb[g + 1] - groups.gb[g] <= 8;
  OCNN_REQUIRE(ok, "conv_gather_sparse: the four groups must split the lists into ranges of at most 8");
  if (rows_out == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("conv_gather_sparse", uptr, urows, cptr, ent, lists, w, out, workspace);
  OCNN_REQUIRE(rows_in == 0 || in, "conv_gather_sparse: in is NULL");
  if (workspace_bytes < (int64_t)n_lists * cin * cout * 2) {
    set_error("conv_gather_sparse: workspace too small");
    return OCNN_ERR_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OCNN_F16)
    return run_sparse<f16>(in, rows_in, uptr, urows, plan_max_distinct, plan_total, cptr, ent, n_blocks, max_blocks,
                           lists, n_lists, groups, rows_out, K, w, cin, cout, w_transposed, reverse_slots, bias,
                           out, workspace, st);
  return run_sparse<bf16>(in, rows_in, uptr, urows, plan_max_distinct, plan_total, cptr, ent, n_blocks, max_blocks,
                          lists, n_lists, groups, rows_out, K, w, cin, cout, w_transposed, reverse_slots, bias, out,
                          workspace, st);
}
