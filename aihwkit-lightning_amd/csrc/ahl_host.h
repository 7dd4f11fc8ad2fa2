// Host-side helpers of the C ABI launchers: argument checks, tiling validation, error capture.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <stdio.h>
#include "../../include/analog_hip.h"
#include "ahl_device.h"

namespace ahl {

// Records the text of a failed HIP call for ahl_last_hip_error(); returns AHL_ERR_LAUNCH.
int record_hip_error(hipError_t e, const char* where);

// Converts the reference's cumulative tile ends into the closed-form split. Returns false if
// the ends do not follow the reference rule (nn/modules/linear.py:155-170) or do not end at K.
inline bool make_tiling(const int32_t* ends, int32_t n_tiles, int64_t K, Tiling* out) {
  if (ends == nullptr || n_tiles <= 0 || K <= 0 || K > 0x7fffffff) return false;
  if ((int64_t)ends[n_tiles - 1] != K) return false;
  const int32_t base = (int32_t)(K / n_tiles), extra = (int32_t)(K % n_tiles);
  if (base <= 0) return false;
  int32_t prev = 0;
  for (int32_t t = 0; t < n_tiles; ++t) {
    const int32_t want = base + (t < extra ? 1 : 0);
    if (ends[t] - prev != want) return false;
    prev = ends[t];
  }
  out->n_tiles = n_tiles;
  out->base = base;
  out->extra = extra;
  return true;
}

// Columns of the widest tile of a split (host side; Tiling's own accessors are device code).
inline int32_t widest_tile(const Tiling& tl) { return tl.base + (tl.extra > 0 ? 1 : 0); }

// Round-to-nearest-even of a float to bfloat16 precision, on the host.
inline float host_round_bf16(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  if ((u & 0x7f800000u) == 0x7f800000u) return x;
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  memcpy(&x, &u, 4);
  return x;
}

// Round-to-nearest-even of a float to float16 precision, on the host (normal range; what the
// launchers round are small constants such as half a number of quantiser states).
inline float host_round_f16(float x) { return (float)(_Float16)x; }

// a host constant as the tensor dtype holds it
inline float host_round_dtype(int32_t dtype, float x) {
  return dtype == AHL_BF16 ? host_round_bf16(x) : dtype == AHL_F16 ? host_round_f16(x) : x;
}

inline bool dtype_known(int32_t dtype) { return dtype == AHL_F32 || dtype == AHL_BF16 || dtype == AHL_F16; }
inline int64_t dtype_bytes(int32_t dtype) { return dtype == AHL_F32 ? 4 : 2; }

inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline int check_launch(const char* where) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return record_hip_error(e, where);
  return AHL_OK;
}

}  // namespace ahl

#define AHL_DISPATCH_DTYPE(dtype, ...)                 \
  do {                                                 \
    if ((dtype) == AHL_F32) {                          \
      typedef ahl::F32 D;                              \
      __VA_ARGS__                                      \
    } else if ((dtype) == AHL_BF16) {                  \
      typedef ahl::BF16 D;                             \
      __VA_ARGS__                                      \
    } else if ((dtype) == AHL_F16) {                   \
      typedef ahl::F16 D;                              \
      __VA_ARGS__                                      \
    } else {                                           \
      return AHL_ERR_ARG;                              \
    }                                                  \
  } while (0)
