// Stage B in its split form: consumes an fp32 score tensor and produces o_hat, o_old_unnorm, W.
//
//   w_s   = exp(score_s - m) * inv_z                (jetfire_vllm/csrc/int4_softmax_v.cu:162-176)
//   ws    = w_s * f32(v_scale[s, group(d)])         (jetfire_vllm/csrc/int2_softmax_v.cu:681-694)
//   o_hat[d] = sum_s fma(ws, code[s, d] - offset)   (:696-706), positions in ascending order
//   o_old_unnorm / W: the same sums over the top-k positions only (:738-788)
//
// Three launches: row statistics (only when the caller has none), a split-S weighted-V pass in which
// one workgroup owns a (sequence, kv-head, S-range) and serves all G query heads from one read of V,
// and a combine pass that adds the split partials in ascending order (deterministic, no atomics) and
// does the top-k pre-correction.
#include "common.h"

namespace jf {
namespace {

constexpr int SV_THREADS = 128;

__device__ inline float block_max_128(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(red[0], red[1]);
}
__device__ inline float block_sum_128(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return red[0] + red[1];
}

__global__ __launch_bounds__(SV_THREADS) void softmax_stats_kernel(const float* __restrict__ scores,
                                                                   const int32_t* __restrict__ seq_lens,
                                                                   float* __restrict__ m_out, float* __restrict__ iz_out,
                                                                   int max_S, int H_q) {
  __shared__ float red[2];
  const int b = blockIdx.x, hq = blockIdx.y, tid = threadIdx.x;
  const size_t bh = (size_t)b * H_q + hq;
  const int n = max(0, min(max_S, seq_lens[b]));
  const float* row = scores + bh * (size_t)max_S;
  float lm = -INFINITY;
  for (int i = tid; i < n; i += SV_THREADS) lm = fmaxf(lm, row[i]);
  float m = block_max_128(lm, red);
  if (!isfinite(m)) m = 0.0f;
  float ls = 0.0f;
  for (int i = tid; i < n; i += SV_THREADS) ls += __expf(row[i] - m);
  const float z = block_sum_128(ls, red);
  if (tid == 0) {
    m_out[bh] = m;
    iz_out[bh] = (z > 0.0f) ? (1.0f / z) : 0.0f;
  }
}

template <int NBITS>
__device__ inline int v_code(const uint8_t* row, int d) {
  if (NBITS == 2) return (int)((row[d >> 2] >> ((3 - (d & 3)) * 2)) & 3) - 2;
  if (NBITS == 3) {  // planar: codes 8w .. 8w+7 are the 24-bit word whose bytes sit at w, 16 + w, 32 + w (MSB first)
    const int w = d >> 3;
    const uint32_t word = ((uint32_t)row[w] << 16) | ((uint32_t)row[16 + w] << 8) | (uint32_t)row[32 + w];
    return (int)((word >> (21 - 3 * (d & 7))) & 7u) - 4;
  }
  return (int)((row[d >> 1] >> ((1 - (d & 1)) * 4)) & 15) - 8;
}

// grid (n_splits, H_kv, B); thread = output channel d; acc[g] for the G query heads of this kv-head.
template <int NBITS, int G, int NG>
__global__ __launch_bounds__(SV_THREADS) void weighted_v_split_kernel(
    const float* __restrict__ scores, const float* __restrict__ softmax_m, const float* __restrict__ softmax_inv_z,
    const uint8_t* __restrict__ v_data, const uint16_t* __restrict__ v_scales, const int64_t* __restrict__ block_table,
    const int32_t* __restrict__ seq_lens, float* __restrict__ partial, int H_q, int H_kv, int max_S, int max_blocks,
    int64_t num_slots, int chunk, int n_splits, int ga) {
  // ga: the query heads that belong to a kv-head; G is ga rounded up to a kernel size, the heads past ga carry no weight
  constexpr int P = D * NBITS / 8;
  __shared__ __align__(16) uint8_t vbuf[BS * P];
  __shared__ float wsbuf[G][BS][NG];
  const int split = blockIdx.x, hkv = blockIdx.y, b = blockIdx.z, tid = threadIdx.x;
  const int S = max(0, min(max_S, seq_lens[b]));
  const int s0 = split * chunk, s1 = min(s0 + chunk, S);
  float acc[G];
#pragma unroll
  for (int g = 0; g < G; ++g) acc[g] = 0.0f;
  const int grp = (NG == 1) ? 0 : (tid / (D / NG));
  const uint8_t* vbase = v_data + (size_t)hkv * num_slots * P;
  const uint16_t* sbase = v_scales + (size_t)hkv * num_slots * NG;
  const int64_t* bt = block_table + (size_t)b * max_blocks;
  for (int p0 = s0; p0 < s1; p0 += BS) {  // chunk is a multiple of BS, so pages are aligned
    const int64_t base_slot = bt[p0 / BS] * BS;
    __syncthreads();
    {
      constexpr int NDW = BS * P / 4;  // dwords of a page (128, 192 or 256)
      const uint32_t* src = reinterpret_cast<const uint32_t*>(vbase + base_slot * P);
#pragma unroll
      for (int i = 0; i < (NDW + SV_THREADS - 1) / SV_THREADS; ++i)
        if (NDW % SV_THREADS == 0 || tid + i * SV_THREADS < NDW)
          reinterpret_cast<uint32_t*>(vbuf)[tid + i * SV_THREADS] = src[tid + i * SV_THREADS];
    }
    for (int i = tid; i < G * BS; i += SV_THREADS) {
      const int g = i / BS, j = i % BS;
      const int p = p0 + j;
      const size_t bh = (size_t)b * H_q + (size_t)hkv * ga + g;
      const bool live = p < s1 && g < ga;
      float w = 0.0f;
      if (live) w = __expf(scores[bh * (size_t)max_S + p] - softmax_m[bh]) * softmax_inv_z[bh];
#pragma unroll
      for (int k = 0; k < NG; ++k)
        wsbuf[g][j][k] = live ? w * bf16_to_f32(sbase[(size_t)(base_slot + j) * NG + k]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < BS; ++j) {
      const float c = (float)v_code<NBITS>(vbuf + j * P, tid);
#pragma unroll
      for (int g = 0; g < G; ++g) acc[g] = __builtin_fmaf(wsbuf[g][j][grp], c, acc[g]);
    }
  }
#pragma unroll
  for (int g = 0; g < G; ++g)
    if (g < ga) partial[(((size_t)b * H_q + (size_t)hkv * ga + g) * n_splits + split) * D + tid] = acc[g];
}

// INT4 values with int8-quantised weights, the arithmetic of the reference's register-MMA Stage B
// (jetfire_vllm/csrc/int8tc_softmax_v_fused.cu:1049-1052 split geometry, :1178 tile origin, :1203-1236 weight
// quantisation, :1298-1311 accumulation): the sequence is cut into TQ_SPLITS ranges of ceil(max_S / TQ_SPLITS)
// positions; a range is walked in tiles of two pages that start at the page holding its first position; per tile
// and query head
//     pv_t = exp(score_t - m) * inv_z * f32(v_scale_t)   (0 outside the range)
//     rs   = max_t |pv_t| / 127,  pq_t = clamp(rint(pv_t * (1 / rs)), -127, 127)   (rs == 0: pq = 0)
//     o_hat[d] += f32(sum_t pq_t * (nibble_t,d - 8)) * rs
// with an exact int32 sum per tile and an fp32 running sum over the tiles in ascending order.
// grid (TQ_SPLITS * sub_count, H_kv, B); thread = output channel d; the 32-lane quarters of the workgroup take the heads
// in turn.  A range's tiles are dealt out in runs to `sub_count` workgroups (the tiles themselves, and with them every
// quantisation step, stay those of the reference's eight ranges; only the association of the fp32 sum over tiles
// changes, at the 1e-7 level), so that a long context fills the chip.
constexpr int TQ_SPLITS = 8;
constexpr int TQ_TILE = 2 * BS;
template <int G>
__global__ __launch_bounds__(SV_THREADS) void tile_quantised_v_split_kernel(
    const float* __restrict__ scores, const float* __restrict__ softmax_m, const float* __restrict__ softmax_inv_z,
    const uint8_t* __restrict__ v_data, const uint16_t* __restrict__ v_scales, const int64_t* __restrict__ block_table,
    const int32_t* __restrict__ seq_lens, float* __restrict__ partial, int H_q, int H_kv, int max_S, int max_blocks,
    int64_t num_slots, int sub_count, int ga) {
  constexpr int P = D / 2;
  __shared__ __align__(16) uint8_t vbuf[TQ_TILE * P];
  __shared__ int pq[G][TQ_TILE];
  __shared__ float rs_sh[G];
  const int split = blockIdx.x / sub_count, sub = blockIdx.x % sub_count;
  const int hkv = blockIdx.y, b = blockIdx.z, tid = threadIdx.x;
  const int S = max(0, min(max_S, seq_lens[b]));
  const int chunk = (max_S + TQ_SPLITS - 1) / TQ_SPLITS;
  const int s_start = split * chunk, s_end = min(s_start + chunk, S);
  float acc[G];
#pragma unroll
  for (int g = 0; g < G; ++g) acc[g] = 0.0f;
  const uint8_t* vbase = v_data + (size_t)hkv * num_slots * P;
  const uint16_t* sbase = v_scales + (size_t)hkv * num_slots;
  const int64_t* bt = block_table + (size_t)b * max_blocks;
  const int q32 = tid >> 5, l32 = tid & 31;
  const int t_first = (s_start / BS) * BS;
  const int n_tiles = (s_end > t_first) ? (s_end - t_first + TQ_TILE - 1) / TQ_TILE : 0;
  const int per_sub = (n_tiles + sub_count - 1) / sub_count;
  const int tile_end = min(n_tiles, (sub + 1) * per_sub);
  for (int tile = sub * per_sub; tile < tile_end; ++tile) {
    const int t0 = t_first + tile * TQ_TILE;
    __syncthreads();
    // the two pages of the tile (a page past the table or the sequence contributes zero weights; its codes are not read)
    int64_t base_slot[2];
#pragma unroll
    for (int pg = 0; pg < 2; ++pg) {
      const int blk = t0 / BS + pg;
      const int64_t e = (blk < max_blocks && blk * BS < s_end) ? bt[blk] : -1;
      base_slot[pg] = (e >= 0 && (e + 1) * BS <= num_slots) ? e * BS : -1;
    }
    {
      constexpr int NDW = BS * P / 4;  // 256 dwords per page
#pragma unroll
      for (int pg = 0; pg < 2; ++pg) {
        const uint32_t* src = reinterpret_cast<const uint32_t*>(vbase + (base_slot[pg] < 0 ? 0 : base_slot[pg]) * P);
#pragma unroll
        for (int i = 0; i < NDW / SV_THREADS; ++i)
          reinterpret_cast<uint32_t*>(vbuf)[pg * NDW + tid + i * SV_THREADS] = base_slot[pg] < 0 ? 0x88888888u : src[tid + i * SV_THREADS];
      }
    }
    for (int g = q32; g < G; g += SV_THREADS / 32) {
      const size_t bh = (size_t)b * H_q + (size_t)hkv * ga + g;
      const int pos = t0 + l32;
      const int64_t bs = base_slot[l32 / BS];
      float pv = 0.0f;
      if (pos >= s_start && pos < s_end && bs >= 0 && g < ga) {
        const float pr = __expf(scores[bh * (size_t)max_S + pos] - softmax_m[bh]) * softmax_inv_z[bh];
        pv = pr * bf16_to_f32(sbase[bs + (l32 % BS)]);
      }
      float a = fabsf(pv);
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) a = fmaxf(a, __shfl_xor(a, o, 32));
      const float row_scale = a / 127.0f;
      const float inv_scale = (row_scale > 0.0f) ? (1.0f / row_scale) : 0.0f;
      int qv = (int)rintf(pv * inv_scale);
      qv = max(-127, min(127, qv));
      pq[g][l32] = qv;
      if (l32 == 0) rs_sh[g] = row_scale;
    }
    __syncthreads();
    int dot[G];
#pragma unroll
    for (int g = 0; g < G; ++g) dot[g] = 0;
#pragma unroll 8
    for (int j = 0; j < TQ_TILE; ++j) {
      const int c = v_code<4>(vbuf + j * P, tid);
#pragma unroll
      for (int g = 0; g < G; ++g) dot[g] += pq[g][j] * c;
    }
#pragma unroll
    for (int g = 0; g < G; ++g) acc[g] += (float)dot[g] * rs_sh[g];
  }
#pragma unroll
  for (int g = 0; g < G; ++g)
    if (g < ga)
      partial[(((size_t)b * H_q + (size_t)hkv * ga + g) * (TQ_SPLITS * sub_count) + blockIdx.x) * D + tid] = acc[g];
}

// grid (B, H_q); adds split partials in order, then the top-k pre-correction.
template <int NBITS, int NG>
__global__ __launch_bounds__(SV_THREADS) void combine_precorr_kernel(
    const float* __restrict__ partial, const float* __restrict__ scores, const float* __restrict__ softmax_m,
    const float* __restrict__ softmax_inv_z, const uint8_t* __restrict__ v_data, const uint16_t* __restrict__ v_scales,
    const int64_t* __restrict__ block_table, const int32_t* __restrict__ seq_lens, const int64_t* __restrict__ topk_idx,
    float* __restrict__ o_hat, float* __restrict__ o_old, float* __restrict__ W_out, int H_q, int H_kv, int max_S,
    int max_blocks, int64_t num_slots, int n_splits, int K) {
  constexpr int P = D * NBITS / 8;
  constexpr int STEP = 128;
  __shared__ int64_t slot_buf[STEP];
  __shared__ float ws_buf[STEP][NG];
  __shared__ float w_buf[STEP];
  const int b = blockIdx.x, hq = blockIdx.y, tid = threadIdx.x;
  const size_t bh = (size_t)b * H_q + hq;
  const int hkv = hq / (H_q / H_kv);
  float acc = 0.0f;
  for (int s0 = 0; s0 < n_splits; s0 += 8) {  // eight loads in flight, the sum keeps its order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = (s0 + u < n_splits) ? partial[(bh * n_splits + s0 + u) * D + tid] : 0.0f;
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  o_hat[bh * D + tid] = acc;
  if (topk_idx == nullptr) return;
  const int S = max(0, min(max_S, seq_lens[b]));
  const int grp = (NG == 1) ? 0 : (tid / (D / NG));
  const uint8_t* vbase = v_data + (size_t)hkv * num_slots * P;
  const uint16_t* sbase = v_scales + (size_t)hkv * num_slots * NG;
  const int64_t* bt = block_table + (size_t)b * max_blocks;
  const float m = softmax_m[bh], iz = softmax_inv_z[bh];
  float acc_old = 0.0f, acc_w = 0.0f;
  for (int k0 = 0; k0 < K; k0 += STEP) {
    __syncthreads();
    {
      const int kk = k0 + tid;
      int64_t slot = -1;
      float w = 0.0f;
      if (kk < K) {
        const int64_t pos = topk_idx[bh * (size_t)K + kk];
        if (pos >= 0 && pos < S) {
          const int64_t blk = bt[pos / BS];
          if (blk >= 0) {
            slot = blk * BS + pos % BS;
            w = __expf(scores[bh * (size_t)max_S + pos] - m) * iz;
          }
        }
      }
      slot_buf[tid] = slot;
      w_buf[tid] = w;
#pragma unroll
      for (int g = 0; g < NG; ++g) ws_buf[tid][g] = (slot >= 0) ? w * bf16_to_f32(sbase[(size_t)slot * NG + g]) : 0.0f;
    }
    __syncthreads();
    const int kend = min(STEP, K - k0);
    for (int j = 0; j < kend; ++j) {
      const int64_t slot = slot_buf[j];
      if (slot < 0) continue;
      const float c = (float)v_code<NBITS>(vbase + slot * P, tid);
      acc_old = __builtin_fmaf(ws_buf[j][grp], c, acc_old);
      acc_w += w_buf[j];
    }
  }
  o_old[bh * D + tid] = acc_old;
  if (tid == 0) W_out[bh] = acc_w;
}

inline int sv_splits(int B, int H_kv, int max_S) {
  const int units = B * H_kv;
  int want = (2048 + units - 1) / units;
  const int max_by_len = (max_S + 63) / 64;
  want = want < 1 ? 1 : want;
  want = want > max_by_len ? max_by_len : want;
  return want < 1 ? 1 : want;
}

}  // namespace
}  // namespace jf

using namespace jf;

extern "C" size_t jf_softmax_v_workspace_bytes(int B, int H_q, int max_S) {
  if (B <= 0 || H_q <= 0) return 256;
  // partials for the largest split count any H_kv can produce, plus the two statistics rows
  size_t max_splits = (size_t)((max_S + 63) / 64 < 2048 ? (max_S + 63) / 64 : 2048);
  if (max_splits < (size_t)TQ_SPLITS) max_splits = TQ_SPLITS;  // the tile-quantised form always uses TQ_SPLITS ranges
  return ((size_t)B * H_q * max_splits * D + 2 * (size_t)B * H_q) * sizeof(float) + 256;
}

extern "C" int jf_softmax_v_pre_corr(const float* scores, const float* softmax_m, const float* softmax_inv_z,
                                     const uint8_t* v_data, const uint16_t* v_scales, const int64_t* block_table,
                                     const int32_t* seq_lens, const int64_t* topk_idx, int B, int H_q, int H_kv,
                                     int max_S, int max_blocks, int64_t num_slots, int block_size, int top_k,
                                     int v_nbits, int n_scale_groups, float* o_hat, float* o_old_unnorm, float* W,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  JF_CHECK_ARG(B >= 0 && H_q > 0 && H_kv > 0 && max_S >= 0 && H_q % H_kv == 0, "softmax_v: bad shape");
  const int G = H_q / H_kv;
  JF_CHECK_ARG(G >= 1 && G <= 16, "softmax_v: GQA group %d not in 1..16", G);
  JF_CHECK_ARG(block_size == 16, "wvs2 only supports block_size=16");
  JF_CHECK_ARG(v_nbits == 2 || v_nbits == 3 || v_nbits == 4, "softmax_v: v_nbits must be 2, 3 or 4 (got %d)", v_nbits);
  JF_CHECK_ARG(n_scale_groups == 1 || n_scale_groups == 2, "wvs2 requires num_groups=1 or 2 (got %d)", n_scale_groups);
  JF_CHECK_ARG((int64_t)max_blocks * block_size >= max_S, "softmax_v: block_table does not cover max_S");
  JF_CHECK_ARG((softmax_m == nullptr) == (softmax_inv_z == nullptr), "softmax_v: softmax_m and softmax_inv_z go together");
  JF_CHECK_ARG(topk_idx == nullptr || top_k > 0, "softmax_v: top_k must be positive");
  if (B == 0) return JF_OK;
  JF_CHECK_ARG(scores && v_data && v_scales && block_table && seq_lens && o_hat, "softmax_v: null pointer");
  JF_CHECK_ARG(topk_idx == nullptr || (o_old_unnorm && W), "softmax_v: o_old_unnorm / W required with topk_idx");
  JF_CHECK_ARG(workspace && workspace_bytes >= jf_softmax_v_workspace_bytes(B, H_q, max_S),
               "softmax_v: workspace too small (%zu < %zu)", workspace_bytes, jf_softmax_v_workspace_bytes(B, H_q, max_S));
  hipStream_t st = (hipStream_t)stream;
  const int n_splits = sv_splits(B, H_kv, max_S);
  int chunk = (max_S + n_splits - 1) / n_splits;
  chunk = (chunk + BS - 1) / BS * BS;
  if (chunk < BS) chunk = BS;
  float* partial = reinterpret_cast<float*>(workspace);
  float* m_ws = partial + (size_t)B * H_q * n_splits * D;
  float* iz_ws = m_ws + (size_t)B * H_q;
  if (softmax_m == nullptr) {
    hipLaunchKernelGGL(softmax_stats_kernel, dim3(B, H_q), dim3(SV_THREADS), 0, st, scores, seq_lens, m_ws, iz_ws, max_S, H_q);
    JF_CHECK_LAUNCH();
    softmax_m = m_ws;
    softmax_inv_z = iz_ws;
  }
  dim3 grid(n_splits, H_kv, B), block(SV_THREADS);
#define JF_SV_LAUNCH(NB, NGC)                                                                                           \
  JF_DISPATCH_G2(G, {                                                                                                    \
    hipLaunchKernelGGL((weighted_v_split_kernel<NB, GG, NGC>), grid, block, 0, st, scores, softmax_m, softmax_inv_z,     \
                       v_data, v_scales, block_table, seq_lens, partial, H_q, H_kv, max_S, max_blocks, num_slots, chunk, \
                       n_splits, G);                                                                                     \
  });                                                                                                                    \
  JF_CHECK_LAUNCH();                                                                                                     \
  hipLaunchKernelGGL((combine_precorr_kernel<NB, NGC>), dim3(B, H_q), block, 0, st, partial, scores, softmax_m,          \
                     softmax_inv_z, v_data, v_scales, block_table, seq_lens, topk_idx, o_hat, o_old_unnorm, W, H_q, H_kv, \
                     max_S, max_blocks, num_slots, n_splits, top_k);                                                     \
  JF_CHECK_LAUNCH();
#define JF_DISPATCH_G2(G, ...)                               \
  switch ((G) <= 2 ? (G) : ((G) <= 4 ? 4 : ((G) <= 8 ? 8 : 16))) {  /* the next kernel size; the kernels take G itself too */ \
    case 1: { constexpr int GG = 1; __VA_ARGS__; } break;    \
    case 2: { constexpr int GG = 2; __VA_ARGS__; } break;    \
    case 4: { constexpr int GG = 4; __VA_ARGS__; } break;    \
    case 8: { constexpr int GG = 8; __VA_ARGS__; } break;    \
    default: { constexpr int GG = 16; __VA_ARGS__; } break;  \
  }
  if (v_nbits == 2 && n_scale_groups == 1) { JF_SV_LAUNCH(2, 1) }
  else if (v_nbits == 2) { JF_SV_LAUNCH(2, 2) }
  else if (v_nbits == 3 && n_scale_groups == 1) { JF_SV_LAUNCH(3, 1) }
  else if (v_nbits == 3) { JF_SV_LAUNCH(3, 2) }
  else if (n_scale_groups == 1) { JF_SV_LAUNCH(4, 1) }
  else { JF_SV_LAUNCH(4, 2) }
  return JF_OK;
}

extern "C" int jf_softmax_v_int8_tiles(const float* scores, const float* softmax_m, const float* softmax_inv_z,
                                       const uint8_t* v_data, const uint16_t* v_scales, const int64_t* block_table,
                                       const int32_t* seq_lens, const int64_t* topk_idx, int B, int H_q, int H_kv,
                                       int max_S, int max_blocks, int64_t num_slots, int block_size, int top_k,
                                       float* o_hat, float* o_old_unnorm, float* W, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  JF_CHECK_ARG(B >= 0 && H_q > 0 && H_kv > 0 && max_S >= 0 && H_q % H_kv == 0, "int8tc_softmax_v: bad shape");
  const int G = H_q / H_kv;
  JF_CHECK_ARG(G >= 1 && G <= 16, "int8tc_softmax_v requires H_q/H_kv in 1..16 (got %d)", G);
  JF_CHECK_ARG(block_size == 16, "int8tc_softmax_v only supports block_size=16");
  JF_CHECK_ARG((int64_t)max_blocks * block_size >= max_S, "int8tc_softmax_v: block_table does not cover max_S");
  JF_CHECK_ARG(topk_idx == nullptr || top_k > 0, "int8tc_softmax_v: top_k must be positive");
  if (B == 0) return JF_OK;
  JF_CHECK_ARG(scores && softmax_m && softmax_inv_z && v_data && v_scales && block_table && seq_lens && o_hat,
               "int8tc_softmax_v: null pointer (the Stage-A statistics are required)");
  JF_CHECK_ARG(topk_idx == nullptr || (o_old_unnorm && W), "int8tc_softmax_v: o_old_unnorm / W required with topk_idx");
  JF_CHECK_ARG(workspace && workspace_bytes >= jf_softmax_v_workspace_bytes(B, H_q, max_S) &&
                   workspace_bytes >= (size_t)B * H_q * TQ_SPLITS * D * sizeof(float),
               "int8tc_softmax_v: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  float* partial = reinterpret_cast<float*>(workspace);
  // runs of at least four tiles per workgroup, at most sixteen workgroups per range (8 * sub_count <= max_S / 128
  // partial rows: inside the workspace, which holds max(8, max_S / 64))
  const int tiles_per_range = ((max_S + TQ_SPLITS - 1) / TQ_SPLITS + TQ_TILE - 1) / TQ_TILE + 1;
  int sub_count = tiles_per_range / 4;
  sub_count = sub_count < 1 ? 1 : (sub_count > 16 ? 16 : sub_count);
  while (sub_count > 1 && (size_t)TQ_SPLITS * sub_count > (size_t)(max_S + 63) / 64) --sub_count;
  dim3 grid(TQ_SPLITS * sub_count, H_kv, B), block(SV_THREADS);
  JF_DISPATCH_G2(G, {
    hipLaunchKernelGGL((tile_quantised_v_split_kernel<GG>), grid, block, 0, st, scores, softmax_m, softmax_inv_z, v_data,
                       v_scales, block_table, seq_lens, partial, H_q, H_kv, max_S, max_blocks, num_slots, sub_count, G);
  });
  JF_CHECK_LAUNCH();
  // the pre-correction terms run on the merge kernel of the fused step where its limits allow (the same
  // formula, p_j = exp(score_j - m) * inv_z with the caller's statistics), else in the combine kernel
  const bool fast_precorr = topk_idx != nullptr && top_k <= 2048 && num_slots <= (1ll << 26) && ((uintptr_t)v_data & 3) == 0;
  hipLaunchKernelGGL((combine_precorr_kernel<4, 1>), dim3(B, H_q), block, 0, st, partial, scores, softmax_m, softmax_inv_z,
                     v_data, v_scales, block_table, seq_lens, fast_precorr ? nullptr : topk_idx, o_hat, o_old_unnorm, W, H_q,
                     H_kv, max_S, max_blocks, num_slots, TQ_SPLITS * sub_count, top_k);
  JF_CHECK_LAUNCH();
  if (fast_precorr)
    return precorr_int4_given_stats(scores, softmax_m, softmax_inv_z, v_data, v_scales, block_table, seq_lens, topk_idx, B,
                                    H_q, H_kv, max_S, max_blocks, num_slots, top_k, o_old_unnorm, W, stream);
  return JF_OK;
}
