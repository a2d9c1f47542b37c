// Morton ("shuffled") keys: x bit i -> key bit 3i+2, y -> 3i+1, z -> 3i,
// batch id at bit 48.  Pure ALU bit spreading, no lookup tables.
#include <stdarg.h>

#include "common.hpp"
#include "morton.hpp"

namespace ocnn {

static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

__global__ void xyz2key_kernel(const int64_t* x, const int64_t* y, const int64_t* z,
                               const int64_t* b, int64_t n, int depth, int64_t* key) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int64_t k = encode(x[i], y[i], z[i], depth);
  if (b) k |= b[i] << 48;
  key[i] = k;
}

__global__ void key2xyz_kernel(const int64_t* key, int64_t n, int nbits, int64_t* x,
                               int64_t* y, int64_t* z, int64_t* b) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int64_t k = key[i];
  b[i] = k >> 48;
  uint64_t low = (uint64_t)k & ((1ull << 48) - 1);
  if (nbits < 48) low &= (1ull << nbits) - 1;   // only ceil(depth/3) groups of 9 bits
  x[i] = (int64_t)compact3(low >> 2);
  y[i] = (int64_t)compact3(low >> 1);
  z[i] = (int64_t)compact3(low);
}

__global__ void points2key_kernel(const float* pts, int64_t n, float bx, float by, float bz,
                                  float factor, const void* batch, int batch_is_float,
                                  int depth, float* pts_out, int64_t* key) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  // (p - bbmin) * factor: a subtraction then a multiplication, each rounded
  float px = (pts[3 * i + 0] - bx) * factor;
  float py = (pts[3 * i + 1] - by) * factor;
  float pz = (pts[3 * i + 2] - bz) * factor;
  pts_out[3 * i + 0] = px;
  pts_out[3 * i + 1] = py;
  pts_out[3 * i + 2] = pz;
  int64_t k = encode((int64_t)px, (int64_t)py, (int64_t)pz, depth);  // trunc toward 0
  if (batch) {
    int64_t bb = batch_is_float ? (int64_t)((const float*)batch)[i] : ((const int64_t*)batch)[i];
    k |= bb << 48;
  }
  key[i] = k;
}

}  // namespace ocnn

using namespace ocnn;

extern "C" const char* ocnn_last_error(void) { return g_err; }
extern "C" int ocnn_abi_version(void) { return 1; }

// Host evaluation of the same bit arithmetic the kernels use (for CPU checks).
extern "C" int64_t ocnn_host_encode_key(int64_t x, int64_t y, int64_t z, int64_t b, int depth) {
  return encode(x, y, z, depth) | (b << 48);
}
extern "C" void ocnn_host_decode_key(int64_t key, int depth, int64_t* xyzb) {
  int nbits = 9 * ((depth + 2) / 3);
  uint64_t low = (uint64_t)key & ((1ull << 48) - 1);
  if (nbits < 48) low &= (1ull << nbits) - 1;
  xyzb[0] = (int64_t)compact3(low >> 2);
  xyzb[1] = (int64_t)compact3(low >> 1);
  xyzb[2] = (int64_t)compact3(low);
  xyzb[3] = key >> 48;
}

extern "C" int ocnn_xyz2key(const int64_t* x, const int64_t* y, const int64_t* z,
                            const int64_t* b, int64_t n, int depth, int64_t* key,
                            void* stream) {
  OCNN_REQUIRE(depth >= 0 && depth <= 16, "xyz2key: depth %d not in [0,16]", depth);
  OCNN_REQUIRE(n >= 0, "xyz2key: negative count");
  if (n == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("xyz2key", x, y, z, key);
  hipLaunchKernelGGL(xyz2key_kernel, dim3(cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream, x, y,
                     z, b, n, depth, key);
  return check_launch("xyz2key");
}

extern "C" int ocnn_key2xyz(const int64_t* key, int64_t n, int depth, int64_t* x, int64_t* y,
                            int64_t* z, int64_t* b, void* stream) {
  OCNN_REQUIRE(depth >= 0 && depth <= 16, "key2xyz: depth %d not in [0,16]", depth);
  OCNN_REQUIRE(n >= 0, "key2xyz: negative count");
  if (n == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("key2xyz", key, x, y, z, b);
  int nbits = 9 * ((depth + 2) / 3);
  hipLaunchKernelGGL(key2xyz_kernel, dim3(cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream, key,
                     n, nbits, x, y, z, b);
  return check_launch("key2xyz");
}

extern "C" int ocnn_points2key(const float* pts, int64_t n, const float* h_bbmin, float factor,
                               const void* batch, int batch_is_float, int depth,
                               float* pts_out, int64_t* key, void* stream) {
  OCNN_REQUIRE(depth >= 1 && depth <= 16, "points2key: depth %d not in [1,16]", depth);
  OCNN_REQUIRE(n >= 0, "points2key: negative count");
  if (n == 0) return OCNN_OK;
  OCNN_REQUIRE_PTRS("points2key", pts, h_bbmin, pts_out, key);
  hipLaunchKernelGGL(points2key_kernel, dim3(cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream,
                     pts, n, h_bbmin[0], h_bbmin[1], h_bbmin[2], factor, batch, batch_is_float,
                     depth, pts_out, key);
  return check_launch("points2key");
}
