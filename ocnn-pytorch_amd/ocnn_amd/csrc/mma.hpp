// MFMA wrappers and small device helpers shared by the convolution kernels.
//
// Operand layout of v_mfma_f32_16x16x32_{f16,bf16}:
//   A (16 x 32): lane l holds A[l % 16][8 * (l / 16) + j], j = 0..7
//   B (32 x 16): lane l holds B[8 * (l / 16) + j][l % 16], j = 0..7
//   D (16 x 16): lane l holds D[4 * (l / 16) + r][l % 16], r = 0..3
#pragma once
#include "common.hpp"

namespace ocnn {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;

template <typename T> struct Mma;
template <> struct Mma<bf16> {
  typedef bf16x8 V;
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ u32x2 read_tr(const bf16* p) {
    bf16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (bf16x4 __attribute__((address_space(3)))*)(p));
    return __builtin_bit_cast(u32x2, v);
  }
};
template <> struct Mma<f16> {
  typedef f16x8 V;
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ u32x2 read_tr(const f16* p) {
    typedef __attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16 h4;
    h4 v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((h4 __attribute__((address_space(3)))*)(p));
    return __builtin_bit_cast(u32x2, v);
  }
};

// v_mfma_f32_32x32x16_{f16,bf16}: A (32 x 16): lane l holds A[l % 32][8 * (l / 32) + j];
// B (16 x 32): lane l holds B[8 * (l / 32) + j][l % 32];
// D (32 x 32): lane l, register r holds D[8 * (r / 4) + 4 * (l / 32) + r % 4][l % 32].
typedef __attribute__((ext_vector_type(16))) float f32x16;
template <typename T> struct Mma32;
template <> struct Mma32<bf16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma32<f16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <typename T> __device__ __forceinline__ unsigned pack2(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) T v2;
  v2 v = {(T)a, (T)b};
  return __builtin_bit_cast(unsigned, v);
}

// Raw buffer descriptor: loads whose byte offset is >= `bytes` return zero, so a
// table entry of -1 (offset 2^32 - row_bytes + ...) needs no branch.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// Maps a linear workgroup id to a tile so that consecutive tiles run on the same
// XCD (workgroups are dealt to the 8 XCDs round-robin; each XCD has its own L2
// and neighbouring row tiles gather overlapping rows).
__device__ __forceinline__ int64_t xcd_tile(int64_t bid, int64_t per_xcd) {
  return (bid & 7) * per_xcd + (bid >> 3);
}

}  // namespace ocnn
