// Shared helpers for the gfx950 kernels and their C-ABI launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <math.h>
#include "../../include/jetfire_amd.h"

namespace jf {

constexpr int D = 128;        // head_dim
constexpr int BS = 16;        // paged block size
constexpr int WAVE = 64;

void set_error(const char* fmt, ...);

#define JF_CHECK_ARG(cond, ...)                                   \
  do {                                                            \
    if (!(cond)) {                                                \
      jf::set_error(__VA_ARGS__);                                 \
      return JF_ERR_ARG;                                          \
    }                                                             \
  } while (0)

#define JF_CHECK_HIP(expr)                                                            \
  do {                                                                                \
    hipError_t _e = (expr);                                                           \
    if (_e != hipSuccess) {                                                           \
      jf::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
      return JF_ERR_HIP;                                                              \
    }                                                                                 \
  } while (0)

#define JF_CHECK_LAUNCH() JF_CHECK_HIP(hipGetLastError())

__device__ __host__ inline float bf16_to_f32(uint16_t b) {
  union { uint32_t u; float f; } v;
  v.u = (uint32_t)b << 16;
  return v.f;
}

// IEEE round-to-nearest-even, NaN kept quiet.
__device__ __host__ inline uint16_t f32_to_bf16(float f) {
  union { uint32_t u; float f; } v;
  v.f = f;
  if ((v.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((v.u >> 16) | 0x0040u);
  v.u += 0x7fffu + ((v.u >> 16) & 1u);
  return (uint16_t)(v.u >> 16);
}

// Order-preserving key of an fp32 score: larger score <=> larger key.
__device__ __host__ inline uint32_t score_key(float f) {
  union { uint32_t u; float f; } v;
  v.f = f;
  return (v.u & 0x80000000u) ? ~v.u : (v.u | 0x80000000u);
}

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}
__device__ inline int wave_sum_i(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

inline bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

}  // namespace jf
