// Measurement probes of the part itself, built into a library of their own
// (libocnn_probe.so; the product library does not contain them).  bench.py reports what they
// measure next to the kernels' figures: the MFMA rate the GPU sustains with the operand
// statistics of the benchmark (clocks fall under matrix load, so the published peak is not
// what any kernel can reach), and what the LDS delivers to the waves of one workgroup.
//
// Every probe launches one workgroup of 256 or 512 threads per CU, times the launch with
// events on the given stream and returns milliseconds; nothing is allocated by the caller
// except the small operand / address arrays it passes in.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

namespace {

// 14 independent accumulators per wave (the register-resident kernels keep as many), two B
// operands, seven A operands: `iters` x 14 v_mfma_f32_32x32x16 back to back.
template <bool BF16>
__global__ __launch_bounds__(256, 1) void mfma_rate_kernel(const u32x4* __restrict__ src, float* __restrict__ out,
                                                           int iters, long long* __restrict__ ticks) {
  u32x4 a[7], b[2];
#pragma unroll
  for (int i = 0; i < 7; ++i) a[i] = src[i * 256 + threadIdx.x];
  b[0] = src[7 * 256 + threadIdx.x];
  b[1] = src[8 * 256 + threadIdx.x];
  f32x16 c[14];
#pragma unroll
  for (int i = 0; i < 14; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) c[i][j] = 0.f;
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 14; ++i) {
      if constexpr (BF16)
        c[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[i % 7]),
                                                       __builtin_bit_cast(bf16x8, b[i & 1]), c[i], 0, 0, 0);
      else
        c[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[i % 7]),
                                                      __builtin_bit_cast(f16x8, b[i & 1]), c[i], 0, 0, 0);
    }
  }
  const long long t1 = clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 14; ++i) s += c[i][0] + c[i][9];
  out[blockIdx.x * 256 + threadIdx.x] = s;
  if (threadIdx.x == 0) ticks[blockIdx.x] = t1 - t0;
}

// The MFMA loop again, now with what a wave of the register-resident gather-GEMM kernel issues
// around its MFMAs, in that kernel's proportions per 8 MFMAs: NV independent VALU operations
// per MFMA, NR 16-byte LDS reads, NW 16-byte LDS writes, NU 2-byte LDS reads (results awaited
// half an iteration later).  STRIDE: bytes between the 16-byte chunks of consecutive lanes (16:
// conflict-free, 32: two lanes per bank group).  NB > 0: an s_barrier every NB iterations.  Two
// accumulator chains, as in that kernel.
template <int NV, int NR, int NW, int NU, int STRIDE = 16, int NB = 0>
__global__ __launch_bounds__(256, 1) void mfma_mix_kernel(const u32x4* __restrict__ src, float* __restrict__ out,
                                                          int iters, long long* __restrict__ ticks) {
  __shared__ __attribute__((aligned(16))) char lds[65536];
  for (int i = threadIdx.x * 16; i < 65536; i += 256 * 16) *(u32x4*)(lds + i) = u32x4{1u, 2u, 3u, 4u};
  __syncthreads();
  u32x4 a[4], b[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = src[i * 256 + threadIdx.x];
  b[0] = src[7 * 256 + threadIdx.x];
  b[1] = src[8 * 256 + threadIdx.x];
  f32x16 c[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) c[i][j] = 0.f;
  unsigned v[8] = {1, 2, 3, 4, 5, 6, 7, 8}, u[4] = {0, 0, 0, 0};
  u32x4 r[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = u32x4{0u, 0u, 0u, 0u};
  const unsigned wave = threadIdx.x >> 6;
  const unsigned off = ((threadIdx.x & 63) * STRIDE + wave * 8192) & 0x7ff0, offw = off + 32768;
  constexpr int kWait = (NR + NW + NU) / 2 > 15 ? 15 : (NR + NW + NU) / 2;
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      c[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[i & 3]),
                                                         __builtin_bit_cast(bf16x8, b[(i >> 1) & 1]), c[i & 1], 0, 0, 0);
#pragma unroll
      for (int k = 0; k < NV; ++k)
        asm volatile("v_xor_b32 %0, %0, %1" : "+v"(v[(i + k) & 7]) : "v"(v[(i + k + 3) & 7]));
#pragma unroll
      for (int k = (i * NR) / 8; k < ((i + 1) * NR) / 8; ++k)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r[k & 7]) : "v"(off), "n"(1024 * (k & 7)) : "memory");
#pragma unroll
      for (int k = (i * NW) / 8; k < ((i + 1) * NW) / 8; ++k)
        asm volatile("ds_write_b128 %0, %1 offset:%2" :: "v"(offw), "v"(r[0]), "n"(1024 * (k & 7)) : "memory");
#pragma unroll
      for (int k = (i * NU) / 8; k < ((i + 1) * NU) / 8; ++k)
        asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(u[k & 3]) : "v"(off), "n"(64 * (k & 7)) : "memory");
      if (i == 3 || i == 7) asm volatile("s_waitcnt lgkmcnt(%0)" :: "n"(kWait) : "memory");
      if (NB > 0 && i == 7 && (it % (NB > 0 ? NB : 1)) == 0) asm volatile("s_barrier" ::: "memory");
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  const long long t1 = clock64();
  float s = c[0][0] + c[0][9] + c[1][0] + c[1][9];
#pragma unroll
  for (int i = 0; i < 8; ++i) s += (float)(v[i] ^ r[i][0]);
#pragma unroll
  for (int i = 0; i < 4; ++i) s += (float)u[i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
  if (threadIdx.x == 0) ticks[blockIdx.x] = t1 - t0;
}

// Every lane reads (WRITE: writes) 16 bytes at its 8 byte offsets `addr[j * threads + tid]`,
// `iters` times.  The caller chooses the offsets, i.e. the bank pattern: consecutive lanes on
// consecutive 16-byte chunks, rows gathered through a swizzle, a deliberate conflict ...
template <bool WRITE>
__global__ __launch_bounds__(512, 1) void lds_rate_kernel(const uint32_t* __restrict__ addr, float* __restrict__ out,
                                                          int iters, long long* __restrict__ ticks) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x, nt = blockDim.x;
  for (int i = tid * 16; i < 64 * 1024; i += nt * 16) *(u32x4*)(lds + i) = u32x4{(unsigned)i, 1u, 2u, 3u};
  uint32_t off[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) off[j] = addr[j * nt + tid] & 0xfff0u;
  __syncthreads();
  u32x4 acc = u32x4{0u, 0u, 0u, 0u};
  u32x4 va[8], vb[8];
  // The accesses are asm statements (the compiler would hoist loop-invariant reads), two
  // batches of eight in flight: while one batch is consumed the other one is on its way.
  auto issue = [&](u32x4 (&v)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (WRITE) asm volatile("ds_write_b128 %0, %1" :: "v"(off[j]), "v"(acc) : "memory");
      else asm volatile("ds_read_b128 %0, %1" : "=v"(v[j]) : "v"(off[j]) : "memory");
    }
  };
  auto consume = [&](u32x4 (&v)[8]) {
    if constexpr (!WRITE) {
#pragma unroll
      for (int j = 0; j < 8; ++j) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(acc[j & 3]) : "v"(v[j][j & 3]));
    }
  };
  const long long t0 = clock64();
  issue(va);
  for (int it = 0; it < iters; it += 2) {
    issue(vb);
    asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
    consume(va);
    issue(va);
    asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
    consume(vb);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  consume(va);
  const long long t1 = clock64();
  if constexpr (WRITE) {
    __syncthreads();
    acc = *(const u32x4*)(lds + tid * 16);
  }
  out[blockIdx.x * nt + tid] = (float)(acc[0] ^ acc[1] ^ acc[2] ^ acc[3]);
  if (tid == 0) ticks[blockIdx.x] = t1 - t0;
}

int cu_count() {
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return -1;
  return prop.multiProcessorCount;
}

template <typename F>
int timed(hipStream_t st, F launch, double* ms) {
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1;
  launch();                                   // warm-up (code load, clocks)
  (void)hipEventRecord(e0, st);
  launch();
  (void)hipEventRecord(e1, st);
  int rc = hipEventSynchronize(e1) == hipSuccess && hipGetLastError() == hipSuccess ? 0 : -1;
  float t = 0.f;
  if (rc == 0) (void)hipEventElapsedTime(&t, e0, e1);
  *ms = t;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return rc;
}

}  // namespace

// operands: 9 x 256 x 16 bytes (device) of f16 / bf16 values; out: CUs x 256 floats; ticks: CUs
// int64 (s_memtime ticks of wave 0 of each workgroup around its loop).  flops = CUs x 4 waves
// x iters x 14 x 32768.
extern "C" int ocnn_probe_mfma_rate(int bf16, const void* operands, void* out, void* ticks, int iters,
                                    void* stream, double* ms, double* flops) {
  const int n_cu = cu_count();
  if (n_cu <= 0 || iters <= 0 || iters > (1 << 22)) return -1;
  hipStream_t st = (hipStream_t)stream;
  *flops = (double)n_cu * 4.0 * iters * 14.0 * 32768.0;
  return timed(st, [&]() {
    if (bf16)
      hipLaunchKernelGGL(mfma_rate_kernel<true>, dim3(n_cu), dim3(256), 0, st, (const u32x4*)operands, (float*)out,
                         iters, (long long*)ticks);
    else
      hipLaunchKernelGGL(mfma_rate_kernel<false>, dim3(n_cu), dim3(256), 0, st, (const u32x4*)operands, (float*)out,
                         iters, (long long*)ticks);
  }, ms);
}

// addr: 8 x threads uint32 byte offsets (device) into 64 KiB of LDS, multiples of 16; threads
// = 256 or 512 (4 or 8 waves on the CU); iters even; bytes = CUs x threads x (iters + 1) x 8 x 16.
extern "C" int ocnn_probe_lds_rate(int write, int threads, const void* addr, void* out, void* ticks, int iters,
                                   void* stream, double* ms, double* bytes) {
  const int n_cu = cu_count();
  if (n_cu <= 0 || iters <= 0 || iters > (1 << 22) || (iters & 1) || (threads != 256 && threads != 512)) return -1;
  hipStream_t st = (hipStream_t)stream;
  *bytes = (double)n_cu * threads * (double)(iters + 1) * 8.0 * 16.0;
  return timed(st, [&]() {
    if (write)
      hipLaunchKernelGGL(lds_rate_kernel<true>, dim3(n_cu), dim3(threads), 64 * 1024, st, (const uint32_t*)addr,
                         (float*)out, iters, (long long*)ticks);
    else
      hipLaunchKernelGGL(lds_rate_kernel<false>, dim3(n_cu), dim3(threads), 64 * 1024, st, (const uint32_t*)addr,
                         (float*)out, iters, (long long*)ticks);
  }, ms);
}

// An iteration is 8 bf16 MFMAs of one wave (ocnn_probe_mfma_rate: 14) with side work chosen by
// `mix` (per 8 MFMAs; V = VALU operations, R = 16-byte LDS reads, W = 16-byte LDS writes, U =
// 2-byte LDS reads):
//   0 none                     1 the gather-GEMM kernel's: 16 V, 6 R, 1 W, 2 U
//   2 16 V      3 32 V         4 4 R     5 6 R     6 8 R     7 8 R, two lanes per bank group
//   8 1 W       9 2 W          10 2 U
//   11 as 1, two lanes per bank group    12 as 1 without the write
//   13 16 V, 8 R, 2 U (a wave that owns its outputs: one operand read per MFMA, no exchange)
//   14 as 1 with an s_barrier every 32 MFMAs
// flops = CUs x 4 waves x iters x 8 x 32768.
extern "C" int ocnn_probe_mfma_mix(int mix, const void* operands, void* out, void* ticks, int iters, void* stream,
                                   double* ms, double* flops) {
  const int n_cu = cu_count();
  if (n_cu <= 0 || iters <= 0 || iters > (1 << 22) || mix < 0 || mix > 14) return -1;
  hipStream_t st = (hipStream_t)stream;
  *flops = (double)n_cu * 4.0 * iters * 8.0 * 32768.0;
#define OCNN_MIX_CASE(id, ...)                                                                                  \
  case id:                                                                                                      \
    hipLaunchKernelGGL((mfma_mix_kernel<__VA_ARGS__>), dim3(n_cu), dim3(256), 0, st, (const u32x4*)operands,    \
                       (float*)out, iters, (long long*)ticks);                                                  \
    break;
  return timed(st, [&]() {
    switch (mix) {
      OCNN_MIX_CASE(0, 0, 0, 0, 0)
      OCNN_MIX_CASE(1, 2, 6, 1, 2)
      OCNN_MIX_CASE(2, 2, 0, 0, 0)
      OCNN_MIX_CASE(3, 4, 0, 0, 0)
      OCNN_MIX_CASE(4, 0, 4, 0, 0)
      OCNN_MIX_CASE(5, 0, 6, 0, 0)
      OCNN_MIX_CASE(6, 0, 8, 0, 0)
      OCNN_MIX_CASE(7, 0, 8, 0, 0, 32)
      OCNN_MIX_CASE(8, 0, 0, 1, 0)
      OCNN_MIX_CASE(9, 0, 0, 2, 0)
      OCNN_MIX_CASE(10, 0, 0, 0, 2)
      OCNN_MIX_CASE(11, 2, 6, 1, 2, 32)
      OCNN_MIX_CASE(12, 2, 6, 0, 2)
      OCNN_MIX_CASE(13, 2, 8, 0, 2)
      OCNN_MIX_CASE(14, 2, 6, 1, 2, 16, 4)
    }
  }, ms);
#undef OCNN_MIX_CASE
}
