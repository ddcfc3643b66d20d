// Stage A in its split form: scores (B, H_q, max_S) fp32 written to HBM, one thread per key position.
// These are the drop-in forms of the reference's int3_qk_scores / int8tc_qk_scores; the fused scan
// (fused_scan.hip) is the fast path that never materialises the score tensor.
//
//   INT3 keys (bf16 model, jetfire_vllm/csrc/int3_qk_scores.cu:90-99,268-311):
//       score = (sum_d f32(q_d) * f32(bf16(code_d - 4) * scale_g))) * attn_scale       fp32 accumulate
//   INT4 keys (int8-Q model, jetfire_vllm/csrc/int8tc_qk_scores.cu:250-290,435-488):
//       qs = max(amax_32(|q|)/127, 1e-12); qi = clamp(rint(q * (1/qs)), -128, 127)
//       acc_kk = sum_{32 ch} qi * (nibble - 8)                                          int32, exact
//       s = fma(acc3,qs3, fma(acc2,qs2, fma(acc1,qs1, acc0*qs0))); score = (s * ks) * attn_scale
#include "common.h"

namespace jf {
namespace {

constexpr int QK_THREADS = 256;

template <int G, int NG>
__global__ __launch_bounds__(QK_THREADS) void int3_qk_scores_kernel(
    const uint16_t* __restrict__ q, const uint8_t* __restrict__ k_data, const uint16_t* __restrict__ k_scales,
    const int64_t* __restrict__ block_table, const int32_t* __restrict__ seq_lens, float* __restrict__ scores,
    int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots, int bs, float attn_scale, int ga) {
  __shared__ float qs[G][D];
  const int b = blockIdx.z, hkv = blockIdx.y, tid = threadIdx.x;
  for (int i = tid; i < G * D; i += QK_THREADS)  // (rows past ga: zero query rows whose scores are never stored)
    qs[i / D][i % D] = (i < ga * D) ? bf16_to_f32(q[((size_t)b * H_q + (size_t)hkv * ga + i / D) * D + i % D]) : 0.f;
  __syncthreads();
  const int s = blockIdx.x * QK_THREADS + tid;
  if (s >= max_S) return;
  float* out = scores + ((size_t)b * H_q + (size_t)hkv * ga) * max_S + s;
  const int S = seq_lens[b];
  if (s >= S) {
#pragma unroll
    for (int g = 0; g < G; ++g)
      if (g < ga) out[(size_t)g * max_S] = -INFINITY;
    return;
  }
  const int64_t slot = block_table[(size_t)b * max_blocks + s / bs] * bs + s % bs;
  const uint32_t* row = reinterpret_cast<const uint32_t*>(k_data + ((size_t)hkv * num_slots + slot) * 48);
  uint32_t p[12];
#pragma unroll
  for (int i = 0; i < 12; ++i) p[i] = row[i];
  float sc[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) sc[g] = bf16_to_f32(k_scales[((size_t)hkv * num_slots + slot) * NG + g]);
  float acc[G];
#pragma unroll
  for (int g = 0; g < G; ++g) acc[g] = 0.0f;
#pragma unroll
  for (int gi = 0; gi < 16; ++gi) {
    const int sh8 = 8 * (gi & 3);
    const uint32_t w = (((p[gi >> 2] >> sh8) & 255u) << 16) | (((p[4 + (gi >> 2)] >> sh8) & 255u) << 8) |
                       ((p[8 + (gi >> 2)] >> sh8) & 255u);
    const float scale = sc[(gi * 8 * NG) / D];
    float kv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int code = (int)((w >> (21 - 3 * j)) & 7u) - 4;
      kv[j] = bf16_to_f32(f32_to_bf16((float)code * scale));
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[g] = __builtin_fmaf(qs[g][gi * 8 + j], kv[j], acc[g]);
  }
#pragma unroll
  for (int g = 0; g < G; ++g)
    if (g < ga) out[(size_t)g * max_S] = acc[g] * attn_scale;
}

// INT2 / INT4 keys with the same bf16 model (jetfire_vllm/csrc/int2_qk_scores.cu:66-79, int4_qk_scores.cu:68-80):
//     score = (sum_d f32(q_d) * f32(bf16((code_d - 2^(bits-1)) * scale_g))) * attn_scale       fp32 accumulate
// INT2 rows: 32 bytes, four codes per byte MSB first; INT4 rows: 64 bytes, (even << 4) | odd.
template <int KBITS, int G, int NG>
__global__ __launch_bounds__(QK_THREADS) void intn_qk_scores_kernel(
    const uint16_t* __restrict__ q, const uint8_t* __restrict__ k_data, const uint16_t* __restrict__ k_scales,
    const uint16_t* __restrict__ k_zp, const int64_t* __restrict__ block_table, const int32_t* __restrict__ seq_lens, float* __restrict__ scores,
    int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots, int bs, float attn_scale, int ga) {
  static_assert(KBITS == 2 || KBITS == 4, "planar INT3 rows have their own kernel");
  constexpr int P = D * KBITS / 8, NDW = P / 4, OFF = 1 << (KBITS - 1);
  __shared__ float qs[G][D];
  const int b = blockIdx.z, hkv = blockIdx.y, tid = threadIdx.x;
  for (int i = tid; i < G * D; i += QK_THREADS)  // (rows past ga: zero query rows whose scores are never stored)
    qs[i / D][i % D] = (i < ga * D) ? bf16_to_f32(q[((size_t)b * H_q + (size_t)hkv * ga + i / D) * D + i % D]) : 0.f;
  __syncthreads();
  const int s = blockIdx.x * QK_THREADS + tid;
  if (s >= max_S) return;
  float* out = scores + ((size_t)b * H_q + (size_t)hkv * ga) * max_S + s;
  const int S = seq_lens[b];
  if (s >= S) {
#pragma unroll
    for (int g = 0; g < G; ++g)
      if (g < ga) out[(size_t)g * max_S] = -INFINITY;
    return;
  }
  const int64_t slot = block_table[(size_t)b * max_blocks + s / bs] * bs + s % bs;
  const uint32_t* row = reinterpret_cast<const uint32_t*>(k_data + ((size_t)hkv * num_slots + slot) * P);
  uint32_t p[NDW];
#pragma unroll
  for (int i = 0; i < NDW; ++i) p[i] = row[i];
  // asymmetric keys add a zero-point per group: bf16(fma(code - off, scale, zp)) (int2_qk_scores.cu:66-79)
  float sc[NG], zp[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    sc[g] = bf16_to_f32(k_scales[((size_t)hkv * num_slots + slot) * NG + g]);
    zp[g] = k_zp ? bf16_to_f32(k_zp[((size_t)hkv * num_slots + slot) * NG + g]) : 0.0f;
  }
  float acc[G];
#pragma unroll
  for (int g = 0; g < G; ++g) acc[g] = 0.0f;
#pragma unroll
  for (int gi = 0; gi < 16; ++gi) {  // eight channels at a time
    const float scale = sc[(gi * 8 * NG) / D], zero = zp[(gi * 8 * NG) / D];
    float kv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      int code;
      if (KBITS == 4) code = (int)((p[gi] >> (8 * (j >> 1) + ((j & 1) ? 0 : 4))) & 15u);
      else code = (int)((p[gi >> 1] >> (16 * (gi & 1) + 8 * (j >> 2) + (6 - 2 * (j & 3)))) & 3u);
      kv[j] = bf16_to_f32(f32_to_bf16(__builtin_fmaf((float)(code - OFF), scale, zero)));
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[g] = __builtin_fmaf(qs[g][gi * 8 + j], kv[j], acc[g]);
  }
#pragma unroll
  for (int g = 0; g < G; ++g)
    if (g < ga) out[(size_t)g * max_S] = acc[g] * attn_scale;
}

// q quantisation shared by the INT4 kernels: qi packed so that dword j of `qe` holds channels
// 8j+{0,2,4,6} (the high nibbles of key dword j) and `qo` holds 8j+{1,3,5,7} (the low nibbles).
template <int G>
struct QInt8 {
  int qe[G][16];
  int qo[G][16];
  float qs[G][4];
  int sum8[G][4];  // 8 * sum of qi over the 32-channel group
};

template <int G>
__device__ inline void quantize_query_int8(const uint16_t* __restrict__ qrow0, QInt8<G>& sh, float* scratch, int tid,
                                           int nthreads, int ga) {
  // scratch: G*4 floats.  Rows past ga (the group padded to the kernel's G) are zero rows: nothing is read for them.
  for (int i = tid; i < G * 4; i += nthreads) {
    const int g = i >> 2, kk = i & 3;
    float amax = 0.0f;
    for (int d = 0; d < 32 && g < ga; ++d) amax = fmaxf(amax, fabsf(bf16_to_f32(qrow0[(size_t)g * D + kk * 32 + d])));
    const float s = fmaxf(amax / 127.0f, 1e-12f);
    sh.qs[g][kk] = s;
    scratch[i] = 1.0f / s;
  }
  __syncthreads();
  for (int i = tid; i < G * 16; i += nthreads) {
    const int g = i >> 4, j = i & 15, kk = j >> 2;
    const float inv = scratch[g * 4 + kk];
    int v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float f = (g < ga) ? bf16_to_f32(qrow0[(size_t)g * D + 8 * j + e]) : 0.f;
      v[e] = max(-128, min(127, (int)rintf(f * inv)));
    }
    sh.qe[g][j] = (v[0] & 255) | ((v[2] & 255) << 8) | ((v[4] & 255) << 16) | ((v[6] & 255) << 24);
    sh.qo[g][j] = (v[1] & 255) | ((v[3] & 255) << 8) | ((v[5] & 255) << 16) | ((v[7] & 255) << 24);
  }
  __syncthreads();
  for (int i = tid; i < G * 4; i += nthreads) {
    const int g = i >> 2, kk = i & 3;
    int sum = 0;
    for (int j = 4 * kk; j < 4 * kk + 4; ++j) {
      const int e = sh.qe[g][j], o = sh.qo[g][j];
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) sum += (int)(int8_t)((e >> (8 * bb)) & 255) + (int)(int8_t)((o >> (8 * bb)) & 255);
    }
    sh.sum8[g][kk] = 8 * sum;
  }
  __syncthreads();
}

template <int G>
__global__ __launch_bounds__(QK_THREADS) void int8tc_qk_scores_kernel(
    const uint16_t* __restrict__ q, const uint8_t* __restrict__ k_data, const uint16_t* __restrict__ k_scales,
    const int64_t* __restrict__ block_table, const int32_t* __restrict__ seq_lens, float* __restrict__ scores,
    int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots, int bs, float attn_scale, int ga) {
  __shared__ QInt8<G> sh;
  __shared__ float scratch[G * 4];
  const int b = blockIdx.z, hkv = blockIdx.y, tid = threadIdx.x;
  quantize_query_int8<G>(q + ((size_t)b * H_q + (size_t)hkv * ga) * D, sh, scratch, tid, QK_THREADS, ga);
  const int s = blockIdx.x * QK_THREADS + tid;
  if (s >= max_S) return;
  float* out = scores + ((size_t)b * H_q + (size_t)hkv * ga) * max_S + s;
  const int S = seq_lens[b];
  if (s >= S) {
#pragma unroll
    for (int g = 0; g < G; ++g)
      if (g < ga) out[(size_t)g * max_S] = -INFINITY;
    return;
  }
  const int64_t slot = block_table[(size_t)b * max_blocks + s / bs] * bs + s % bs;
  const uint4* row = reinterpret_cast<const uint4*>(k_data + ((size_t)hkv * num_slots + slot) * 64);
  uint32_t p[16];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint4 v = row[i];
    p[4 * i] = v.x; p[4 * i + 1] = v.y; p[4 * i + 2] = v.z; p[4 * i + 3] = v.w;
  }
  const float ks = bf16_to_f32(k_scales[(size_t)hkv * num_slots + slot]);
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float sacc = 0.0f;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      int acc = 0;
#pragma unroll
      for (int j = 4 * kk; j < 4 * kk + 4; ++j) {
        const int hi = (int)((p[j] >> 4) & 0x0f0f0f0fu), lo = (int)(p[j] & 0x0f0f0f0fu);
        acc = __builtin_amdgcn_sdot4(hi, sh.qe[g][j], acc, false);
        acc = __builtin_amdgcn_sdot4(lo, sh.qo[g][j], acc, false);
      }
      acc -= sh.sum8[g][kk];
      sacc = (kk == 0) ? ((float)acc * sh.qs[g][0]) : __builtin_fmaf((float)acc, sh.qs[g][kk], sacc);
    }
    if (g < ga) out[(size_t)g * max_S] = __fmul_rn(__fmul_rn(sacc, ks), attn_scale);
  }
}

int check_stage_a(const char* name, const void* q, const void* kd, const void* ks, const void* bt, const void* sl,
                  const void* scores, int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots, int bs) {
  JF_CHECK_ARG(B >= 0 && H_q > 0 && H_kv > 0 && max_S >= 0, "%s: bad shape", name);
  JF_CHECK_ARG(H_q % H_kv == 0, "%s: H_q must be divisible by H_kv", name);
  const int G = H_q / H_kv;
  JF_CHECK_ARG(G >= 1 && G <= 16, "%s: GQA group %d not in 1..16", name, G);
  JF_CHECK_ARG(bs > 0 && (int64_t)max_blocks * bs >= max_S, "%s: block_table (%d blocks of %d) does not cover max_S=%d",
               name, max_blocks, bs, max_S);
  JF_CHECK_ARG(num_slots > 0, "%s: num_slots must be positive", name);
  if (B == 0 || max_S == 0) return JF_OK;
  JF_CHECK_ARG(q && kd && ks && bt && sl && scores, "%s: null pointer", name);
  JF_CHECK_ARG(((uintptr_t)kd & 15) == 0, "%s: k_data must be 16-byte aligned", name);
  return JF_OK;
}

}  // namespace
}  // namespace jf

using namespace jf;

// The kernels come for 1, 2, 4, 8 and 16 query heads per kv-head; other group sizes run the next larger one with
// the actual size as an argument (zero query rows past it, nothing stored for them).
#define JF_DISPATCH_G(G, ...)                      \
  switch ((G) <= 2 ? (G) : ((G) <= 4 ? 4 : ((G) <= 8 ? 8 : 16))) {  \
    case 1: { constexpr int GG = 1; __VA_ARGS__; } break;  \
    case 2: { constexpr int GG = 2; __VA_ARGS__; } break;  \
    case 4: { constexpr int GG = 4; __VA_ARGS__; } break;  \
    case 8: { constexpr int GG = 8; __VA_ARGS__; } break;  \
    default: { constexpr int GG = 16; __VA_ARGS__; } break; \
  }

extern "C" int jf_int3_qk_scores(const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                                 const int64_t* block_table, const int32_t* seq_lens, int B, int H_q, int H_kv,
                                 int max_S, int max_blocks, int64_t num_slots, int n_scale_groups, int block_size,
                                 float attn_scale, float* scores, void* stream) {
  int rc = check_stage_a("int3_qk_scores", q, k_data, k_scales, block_table, seq_lens, scores, B, H_q, H_kv, max_S,
                         max_blocks, num_slots, block_size);
  if (rc != JF_OK) return rc;
  JF_CHECK_ARG(n_scale_groups == 1 || n_scale_groups == 2,
               "int3_qk_scores currently supports K quant groups 1 or 2, got %d", n_scale_groups);
  if (B == 0 || max_S == 0) return JF_OK;
  dim3 grid((unsigned)((max_S + QK_THREADS - 1) / QK_THREADS), (unsigned)H_kv, (unsigned)B), block(QK_THREADS);
  hipStream_t st = (hipStream_t)stream;
  const int G = H_q / H_kv;
  JF_DISPATCH_G(G, {
    if (n_scale_groups == 1)
      hipLaunchKernelGGL((int3_qk_scores_kernel<GG, 1>), grid, block, 0, st, q, k_data, k_scales, block_table, seq_lens,
                         scores, H_q, H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, G);
    else
      hipLaunchKernelGGL((int3_qk_scores_kernel<GG, 2>), grid, block, 0, st, q, k_data, k_scales, block_table, seq_lens,
                         scores, H_q, H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, G);
  });
  JF_CHECK_LAUNCH();
  return JF_OK;
}

extern "C" int jf_intn_qk_scores(int k_nbits, const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                                 const uint16_t* k_zp, const int64_t* block_table, const int32_t* seq_lens, int B, int H_q, int H_kv,
                                 int max_S, int max_blocks, int64_t num_slots, int n_scale_groups, int block_size,
                                 float attn_scale, float* scores, void* stream) {
  JF_CHECK_ARG(k_zp == nullptr || k_nbits == 2, "intn_qk_scores: zero-points are only defined for INT2 keys");
  if (k_nbits == 3)
    return jf_int3_qk_scores(q, k_data, k_scales, block_table, seq_lens, B, H_q, H_kv, max_S, max_blocks, num_slots,
                             n_scale_groups, block_size, attn_scale, scores, stream);
  JF_CHECK_ARG(k_nbits == 2 || k_nbits == 4, "intn_qk_scores: k_nbits must be 2, 3 or 4 (got %d)", k_nbits);
  int rc = check_stage_a("intn_qk_scores", q, k_data, k_scales, block_table, seq_lens, scores, B, H_q, H_kv, max_S,
                         max_blocks, num_slots, block_size);
  if (rc != JF_OK) return rc;
  JF_CHECK_ARG(n_scale_groups == 1 || n_scale_groups == 2, "intn_qk_scores supports K quant groups 1 or 2, got %d",
               n_scale_groups);
  if (B == 0 || max_S == 0) return JF_OK;
  dim3 grid((unsigned)((max_S + QK_THREADS - 1) / QK_THREADS), (unsigned)H_kv, (unsigned)B), block(QK_THREADS);
  hipStream_t st = (hipStream_t)stream;
  const int G = H_q / H_kv;
#define JF_INTN_LAUNCH(KB, NGV)                                                                                        \
  hipLaunchKernelGGL((intn_qk_scores_kernel<KB, GG, NGV>), grid, block, 0, st, q, k_data, k_scales, k_zp, block_table, \
                     seq_lens, scores, H_q, H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, G)
  JF_DISPATCH_G(G, {
    if (k_nbits == 2) {
      if (n_scale_groups == 1) JF_INTN_LAUNCH(2, 1); else JF_INTN_LAUNCH(2, 2);
    } else {
      if (n_scale_groups == 1) JF_INTN_LAUNCH(4, 1); else JF_INTN_LAUNCH(4, 2);
    }
  });
#undef JF_INTN_LAUNCH
  JF_CHECK_LAUNCH();
  return JF_OK;
}

extern "C" int jf_int8tc_qk_scores(const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                                   const int64_t* block_table, const int32_t* seq_lens, int B, int H_q, int H_kv,
                                   int max_S, int max_blocks, int64_t num_slots, int block_size, float attn_scale,
                                   float* scores, void* stream) {
  int rc = check_stage_a("int8tc_qk_scores", q, k_data, k_scales, block_table, seq_lens, scores, B, H_q, H_kv, max_S,
                         max_blocks, num_slots, block_size);
  if (rc != JF_OK) return rc;
  if (B == 0 || max_S == 0) return JF_OK;
  dim3 grid((unsigned)((max_S + QK_THREADS - 1) / QK_THREADS), (unsigned)H_kv, (unsigned)B), block(QK_THREADS);
  hipStream_t st = (hipStream_t)stream;
  const int G = H_q / H_kv;
  JF_DISPATCH_G(G, {
    hipLaunchKernelGGL((int8tc_qk_scores_kernel<GG>), grid, block, 0, st, q, k_data, k_scales, block_table, seq_lens,
                       scores, H_q, H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, G);
  });
  JF_CHECK_LAUNCH();
  return JF_OK;
}
