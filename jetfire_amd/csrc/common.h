// Shared helpers for the gfx950 kernels and their C-ABI launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <math.h>
#include "../../include/jetfire_amd.h"
#ifdef JF_DEBUG_HOOKS
#include "../../include/jetfire_amd_debug.h"
#endif

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
  return v.u ^ ((uint32_t)((int32_t)v.u >> 31) | 0x80000000u);  // negative: all bits flipped; else: sign bit set
}

// Wavefront-wide reductions and scans on the DPP network (row shifts inside 16-lane rows, then the two
// row broadcasts), no LDS traffic.  After the sequence lane 63 holds the reduction over all 64 lanes.
template <int CTRL, int ROW_MASK>
__device__ inline int dpp_mov(int old, int v) {
  return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, 0xf, false);
}
#define JF_DPP_REDUCE(v, OP, T, IDENT)                                                               \
  do {                                                                                               \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x111, 0xf>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x112, 0xf>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x114, 0xf>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x118, 0xf>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x142, 0xa>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x143, 0xc>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
  } while (0)

// reduction inside each 16-lane row only: lane 15 of a row holds the row's result
#define JF_DPP_ROW_REDUCE(v, OP, T, IDENT)                                                           \
  do {                                                                                               \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x111, 0xf>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x112, 0xf>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x114, 0xf>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
    v = OP(v, __builtin_bit_cast(T, dpp_mov<0x118, 0xf>(__builtin_bit_cast(int, (T)(IDENT)), __builtin_bit_cast(int, v)))); \
  } while (0)

__device__ inline float op_fmax(float a, float b) { return fmaxf(a, b); }
__device__ inline float op_fadd(float a, float b) { return a + b; }
__device__ inline int op_iadd(int a, int b) { return a + b; }
__device__ inline uint32_t op_umax(uint32_t a, uint32_t b) { return a > b ? a : b; }
__device__ inline uint32_t op_umin(uint32_t a, uint32_t b) { return a < b ? a : b; }

// result broadcast to every lane
__device__ inline float wave_max(float v) {
  JF_DPP_REDUCE(v, op_fmax, float, -INFINITY);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ inline float wave_sum(float v) {
  JF_DPP_REDUCE(v, op_fadd, float, 0.0f);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ inline int wave_sum_i(int v) {
  JF_DPP_REDUCE(v, op_iadd, int, 0);
  return __builtin_amdgcn_readlane(v, 63);
}
__device__ inline uint32_t wave_max_u(uint32_t v) {
  JF_DPP_REDUCE(v, op_umax, uint32_t, 0u);
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
__device__ inline uint32_t wave_min_u(uint32_t v) {
  JF_DPP_REDUCE(v, op_umin, uint32_t, 0xffffffffu);
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
// inclusive prefix sum over lanes 0..l
__device__ inline int wave_incl_scan_i(int v) {
  JF_DPP_REDUCE(v, op_iadd, int, 0);
  return v;
}

inline bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

// Pre-correction terms of INT4 values (one scale per row) over given winners with given softmax statistics, on the
// merge kernel of the fused step (fused_stage_b.hip); top_k <= 2048, num_slots <= 2^26.
int precorr_int4_given_stats(const float* scores, const float* softmax_m, const float* softmax_inv_z,
                             const uint8_t* v_data, const uint16_t* v_scales, const int64_t* block_table,
                             const int32_t* seq_lens, const int64_t* topk_idx, int B, int H_q, int H_kv, int max_S,
                             int max_blocks, int64_t num_slots, int top_k, float* o_old_unnorm, float* W, void* stream);

}  // namespace jf
