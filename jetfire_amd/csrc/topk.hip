// Exact top-k over a row of fp32 scores by wavefront radix select (no sort).
//
// One 512-thread workgroup per (sequence, query head) row.  Four 8-bit levels over the
// order-preserving key of the score find the K-th largest key tau and the number of keys above it;
// every level builds one 256-bin histogram per wavefront in LDS (no cross-wave contention) and the
// cut bin is found with a wavefront suffix scan.  Winners are all keys > tau plus the lowest-position
// keys == tau that fill the quota, emitted in ascending position with a ballot/popcount ordered
// compaction, so the output is deterministic.  (The reference's topk_slots_kernel_v5,
// jetfire_vllm/csrc/int3_qk_scores.cu:426-554, selects the same value multiset but in atomic order.)
#include "common.h"

namespace jf {
namespace {

constexpr int TK_THREADS = 512;
constexpr int TK_WAVES = TK_THREADS / 64;

struct TopkShared {
  int hist[TK_WAVES][256];
  int suffix_wave[4];
  int cut_bin;
  int above_in_level;
  int wave_above[TK_WAVES];
  int wave_tie[TK_WAVES];
  float red[TK_WAVES];
};

__device__ inline float block_reduce_max(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int i = 1; i < TK_WAVES; ++i) r = fmaxf(r, red[i]);
  return r;
}
__device__ inline float block_reduce_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int i = 1; i < TK_WAVES; ++i) r += red[i];
  return r;
}

__global__ __launch_bounds__(TK_THREADS) void topk_slots_kernel(
    const float* __restrict__ scores, const int32_t* __restrict__ seq_lens,
    const int64_t* __restrict__ block_table, int max_S, int max_blocks, int H_q, int bs, int K,
    int64_t* __restrict__ topk_idx, int64_t* __restrict__ topk_slots, float* __restrict__ softmax_m,
    float* __restrict__ softmax_inv_z) {
  __shared__ TopkShared sh;
  const int b = blockIdx.x, hq = blockIdx.y, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const size_t bh = (size_t)b * H_q + hq;
  const int n = max(0, min(max_S, seq_lens[b]));
  const float* row = scores + bh * (size_t)max_S;
  int64_t* out_idx = topk_idx + bh * (size_t)K;
  int64_t* out_slot = topk_slots + bh * (size_t)K;
  const int64_t* bt = block_table + (size_t)b * max_blocks;

  if (softmax_m != nullptr) {
    float lm = -INFINITY;
    for (int i = tid; i < n; i += TK_THREADS) lm = fmaxf(lm, row[i]);
    float m = block_reduce_max(lm, sh.red);
    if (!isfinite(m)) m = 0.0f;
    float ls = 0.0f;
    for (int i = tid; i < n; i += TK_THREADS) ls += __expf(row[i] - m);
    const float z = block_reduce_sum(ls, sh.red);
    if (tid == 0) {
      softmax_m[bh] = m;
      softmax_inv_z[bh] = (z > 0.0f) ? (1.0f / z) : 0.0f;
    }
    __syncthreads();
  }

  uint32_t tau = 0;
  int quota = 0;  // number of keys == tau to take
  bool take_all = (n <= K);
  if (!take_all) {
    uint32_t prefix = 0;
    int k_rem = K;
    for (int level = 0; level < 4; ++level) {
      for (int i = tid; i < TK_WAVES * 256; i += TK_THREADS) (&sh.hist[0][0])[i] = 0;
      __syncthreads();
      const int shift = 24 - 8 * level;
      for (int i = tid; i < n; i += TK_THREADS) {
        const uint32_t key = score_key(row[i]);
        const bool in_prefix = (level == 0) || ((key >> (shift + 8)) == prefix);
        if (in_prefix) atomicAdd(&sh.hist[wave][(key >> shift) & 255u], 1);
      }
      __syncthreads();
      // bins -> threads 0..255; suffix sums (count of keys in bins strictly above)
      int cnt = 0, incl = 0;
      if (tid < 256) {
#pragma unroll
        for (int w = 0; w < TK_WAVES; ++w) cnt += sh.hist[w][tid];
        incl = cnt;  // inclusive suffix within the wave: sum over lanes >= lane
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const int o = __shfl_down(incl, off);
          if (lane + off < 64) incl += o;
        }
        if (lane == 0) sh.suffix_wave[wave] = incl;
      }
      __syncthreads();
      if (tid < 256) {
        int higher = 0;
        for (int w = wave + 1; w < 4; ++w) higher += sh.suffix_wave[w];
        const int s_incl = incl + higher;
        const int s_excl = s_incl - cnt;
        if (s_excl < k_rem && k_rem <= s_incl) {
          sh.cut_bin = tid;
          sh.above_in_level = s_excl;
        }
      }
      __syncthreads();
      prefix = (prefix << 8) | (uint32_t)sh.cut_bin;
      k_rem -= sh.above_in_level;
      __syncthreads();
    }
    tau = prefix;
    quota = k_rem;
  }

  // ordered emission
  int base_above = 0, base_tie = 0;
  const int n_round = (n + TK_THREADS - 1) / TK_THREADS * TK_THREADS;
  for (int i0 = 0; i0 < n_round; i0 += TK_THREADS) {
    const int i = i0 + tid;
    bool above = false, tie = false;
    if (i < n) {
      if (take_all) {
        above = true;
      } else {
        const uint32_t key = score_key(row[i]);
        above = key > tau;
        tie = key == tau;
      }
    }
    const unsigned long long ma = __ballot(above), mt = __ballot(tie);
    const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    if (lane == 0) {
      sh.wave_above[wave] = __popcll(ma);
      sh.wave_tie[wave] = __popcll(mt);
    }
    __syncthreads();
    int pa = base_above + __popcll(ma & lt), pt = base_tie + __popcll(mt & lt);
    int tot_a = 0, tot_t = 0;
#pragma unroll
    for (int w = 0; w < TK_WAVES; ++w) {
      const int a = sh.wave_above[w], t = sh.wave_tie[w];
      if (w < wave) { pa += a; pt += t; }
      tot_a += a; tot_t += t;
    }
    if (above || (tie && pt < quota)) {
      const int pos = pa + min(pt, quota);
      if (pos < K) {
        out_idx[pos] = i;
        const int blk = i / bs;
        out_slot[pos] = (blk < max_blocks) ? bt[blk] * (int64_t)bs + (i % bs) : -1;
      }
    }
    base_above += tot_a;
    base_tie += tot_t;
    __syncthreads();
  }
  const int n_out = min(K, base_above + min(base_tie, quota));
  for (int r = n_out + tid; r < K; r += TK_THREADS) {
    out_idx[r] = -1;
    out_slot[r] = -1;
  }
}

}  // namespace
}  // namespace jf

using namespace jf;

extern "C" int jf_topk_slots(const float* scores, const int32_t* seq_lens, const int64_t* block_table,
                             int B, int H_q, int max_S, int max_blocks, int block_size, int top_k,
                             int64_t* topk_idx, int64_t* topk_slots, float* softmax_m, float* softmax_inv_z,
                             void* stream) {
  JF_CHECK_ARG(B >= 0 && H_q > 0 && max_S >= 0 && max_blocks >= 0, "topk_slots: bad shape");
  JF_CHECK_ARG(is_pow2(top_k) && top_k >= 32 && top_k <= 8192,
               "topk_slots: unsupported radix-select top_k=%d (supported: 32,64,128,256,512,1024,2048,4096,8192)", top_k);
  JF_CHECK_ARG(max_S <= 262144, "topk_slots: max_S=%d exceeds supported limit (262144)", max_S);
  JF_CHECK_ARG(block_size > 0, "topk_slots: bad block_size=%d", block_size);
  JF_CHECK_ARG((softmax_m == nullptr) == (softmax_inv_z == nullptr), "topk_slots: softmax_m and softmax_inv_z go together");
  if (B == 0) return JF_OK;
  JF_CHECK_ARG(scores && seq_lens && block_table && topk_idx && topk_slots, "topk_slots: null pointer");
  dim3 grid((unsigned)B, (unsigned)H_q), block(TK_THREADS);
  hipLaunchKernelGGL(topk_slots_kernel, grid, block, 0, (hipStream_t)stream, scores, seq_lens, block_table, max_S,
                     max_blocks, H_q, block_size, top_k, topk_idx, topk_slots, softmax_m, softmax_inv_z);
  JF_CHECK_LAUNCH();
  return JF_OK;
}
