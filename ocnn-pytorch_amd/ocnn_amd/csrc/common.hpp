// Shared helpers of the HIP library: error reporting, launch checks, dtypes.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "ocnn_hip.h"

namespace ocnn {

void set_error(const char* fmt, ...);

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return OCNN_ERR_HIP;
  }
  return OCNN_OK;
}

#define OCNN_REQUIRE(cond, ...)        \
  do {                                 \
    if (!(cond)) {                     \
      ::ocnn::set_error(__VA_ARGS__);  \
      return OCNN_ERR_ARG;             \
    }                                  \
  } while (0)

// Pointers that an entry point dereferences (or hands to a kernel) must not be null: a null
// goes straight to a launch otherwise, and a kernel that reads through it takes the GPU down.
template <typename... P>
inline bool all_set(const P*... p) {
  return (... && (p != nullptr));
}
#define OCNN_REQUIRE_PTRS(what, ...) \
  OCNN_REQUIRE(::ocnn::all_set(__VA_ARGS__), what ": a required pointer is NULL (of " #__VA_ARGS__ ")")

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t align_up(int64_t a, int64_t b) { return cdiv(a, b) * b; }

typedef _Float16 f16;
typedef __bf16 bf16;

template <typename T> __device__ inline float to_f32(T v) { return (float)v; }
template <typename T> __device__ inline T from_f32(float v) { return (T)v; }

inline int dtype_size(int dtype) { return dtype == OCNN_F32 ? 4 : 2; }

}  // namespace ocnn
