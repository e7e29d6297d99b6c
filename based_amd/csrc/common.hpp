// Shared device/host helpers for the gfx950 kernels of libbased_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "based_hip.h"

namespace based {

constexpr int kFeat = BASED_FEATURE_DIM;      // 16
constexpr int kExp = BASED_EXPANDED_DIM;      // 273
constexpr int kWave = 64;

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __builtin_bit_cast(float, bits16 << 16);
}
__device__ __forceinline__ float to_f32(__bf16 x) { return (float)x; }
__device__ __forceinline__ float to_f32(float x) { return x; }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ __bf16 from_f32<__bf16>(float x) { return (__bf16)x; }

// Packs two floats into one dword of two bf16 (round-to-nearest-even), low half = a.
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  f32x2 p = {a, b};
  bf16x2 h = __builtin_convertvector(p, bf16x2);
  return __builtin_bit_cast(uint32_t, h);
}

// Sum over the 64 lanes of a wavefront; every lane receives the total.
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
  return x;
}

// Error reporting shared by the C entry points (thread-local last-error string).
void set_error(const char* fmt, ...);

#define BASED_REQUIRE(cond, code, ...)   \
  do {                                   \
    if (!(cond)) {                       \
      ::based::set_error(__VA_ARGS__);   \
      return (code);                     \
    }                                    \
  } while (0)

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return BASED_ERR_LAUNCH;
  }
  return BASED_OK;
}

}  // namespace based
