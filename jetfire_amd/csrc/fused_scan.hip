// Fused decode scan + top-k for gfx950: one pass over the packed K and V of every (sequence, kv-head),
// no (B, H_q, S) score tensor in HBM.
//
// Launch 1, fused_scan_kernel, grid (n_splits, H_kv, B), 256 threads.  A workgroup owns L consecutive
// positions of one (sequence, kv-head) and all G query heads of that kv-head:
//   phase A  Q.K^T            scores[G][L] -> LDS (fp32), running max per head
//            INT3 keys: K-hat = bf16((code-4)*scale) built in registers, v_mfma_f32_16x16x32_bf16 with the
//                       tokens on the N side; the four 16-token tiles of a wavefront land one per
//                       16-lane group, so lane l ends up holding the G scores of token l.
//            INT4 keys: int8-quantised Q, exact nibble codes, v_dot4_i32_i8, fp32 rescale (every step
//                       is exactly reproducible, so it is bit-equal to the split-form kernel).
//   phase B  P.V on v_mfma_i32_16x16x64_i8.  p = exp(s - m_split) is known exactly because phase A is
//            complete, so w = p * v_scale is converted to 22-bit fixed point once (fma with 2^23), its
//            three bytes are the A-operand rows (limb, head), and the int32 accumulators live for the whole
//            split: every product is exact.  V codes are staged packed in LDS and transposed by
//            ds_read_b64_tr_b4 (16 tokens of one channel per lane), then nibble-spread to bytes.
//            sum_t w_t*(code - off) = sum_t w_t*code - off * sum_t w_t; a constant-ones row gives sum_t code.
//   phase C  per-head radix select over the LDS scores: the split's top-min(K, n) candidates
//            (key, position), ascending position.
// Launch 2, fused_merge_kernel, grid (B, H_q): selects the global top-k among the candidates (ties to
// the lower position, ascending output), merges the split partials
//   M = max m_i, l = sum l_i e^{m_i-M}, o_hat = sum o_i e^{m_i-M} / l
// (the split-KV combine of jetfire_vllm/csrc/fused_decode_wmma.cu:1226-1253), and computes the
// pre-correction terms o_old_unnorm, W over the winners (jetfire_vllm/csrc/int2_softmax_v.cu:738-788).
#include "common.h"

#include <vector>

namespace jf {
namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

constexpr int FS_THREADS = 256;
constexpr int FS_WAVES = 4;

struct FusedParams {
  const uint16_t* q;
  const uint8_t* k_data;
  const uint16_t* k_scales;
  const uint8_t* v_data;
  const uint16_t* v_scales;
  const int64_t* block_table;
  const int32_t* seq_lens;
  int B, H_q, H_kv, max_S, max_blocks;
  int64_t num_slots;
  float attn_scale;
  int top_k;
  int L, n_splits, Kc;
  float* scores;  // optional (B, H_q, max_S)
  float* part_m;  // (B, H_q, NS)
  float* part_l;  // (B, H_q, NS)
  float* part_o;  // (B, H_q, NS, D)
  uint32_t* cand_key;  // (B, H_q, NS, Kc)
  int32_t* cand_idx;   // (B, H_q, NS, Kc)
  int32_t* cand_cnt;   // (B, H_q, NS)
  // merge outputs
  int64_t* topk_idx;
  int64_t* topk_slots;
  float* o_hat;
  float* o_old;
  float* W;
  float* softmax_m;
  float* softmax_inv_z;
};

__device__ inline uint32_t pack_bf16x2(float a, float b) {
  v2f f = {a, b};
  v2bf h = __builtin_convertvector(f, v2bf);  // v_cvt_pk_bf16_f32, round-to-nearest-even
  return __builtin_bit_cast(uint32_t, h);
}

__device__ inline float key_to_score(uint32_t key) {
  const uint32_t u = (key & 0x80000000u) ? (key & 0x7fffffffu) : ~key;
  return __builtin_bit_cast(float, u);
}

// position of token r (0..15) of a 16-token block inside the 16-byte MFMA K-run: the nibble spread of a
// transposed V dword yields tokens 0,2,4,6 | 1,3,5,7 | 8,10,12,14 | 9,11,13,15.
__device__ inline int token_byte_pos(int r) { return (r & 8) | ((r & 1) << 2) | ((r >> 1) & 3); }

template <int G>
struct QInt8F {
  int qe[G][16];
  int qo[G][16];
  float qs[G][4];
  int sum8[G][4];
};

// ---------------------------------------------------------------------------------------------------
template <int SCHEME, int G, int NG>
__global__ __launch_bounds__(FS_THREADS) void fused_scan_kernel(FusedParams p) {
  constexpr bool K3 = (SCHEME == JF_SCHEME_K3V2);
  constexpr int NSET = (G + 3) / 4;
  constexpr int KP = K3 ? 48 : 64;
  constexpr int VP = K3 ? 32 : 64;
  constexpr int VROW = VP + 8;          // LDS row stride: 16 consecutive rows hit 16 distinct bank pairs
  constexpr int VOFF = K3 ? 2 : 8;      // code offset of the V format
  constexpr int NTILE = 8;              // 8 MFMA column tiles of 16 channels
  constexpr int WL_WAVE = NG * NSET * 16 * 64;  // bytes of limb rows per wavefront

  extern __shared__ __align__(16) uint8_t smem[];
  const int L = p.L;
  float* sc = reinterpret_cast<float*>(smem);                 // [G][L]
  uint8_t* stage = smem + (size_t)G * L * sizeof(float);      // staging, reused between phases
  __shared__ float red_f[FS_WAVES][16];
  __shared__ float m_sh[16];
  __shared__ float vmax_sh[FS_WAVES][2];
  __shared__ int e_sh[2];
  __shared__ unsigned long long wsum_sh[16][2];

  const int split = blockIdx.x, hkv = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int S = max(0, min(p.max_S, p.seq_lens[b]));
  const int s0 = split * L;
  const int s1 = min(s0 + L, S);
  const int n = max(0, s1 - s0);
  const int s_cover = min(s0 + L, p.max_S);
  const int64_t* bt = p.block_table + (size_t)b * p.max_blocks;
  const size_t head0 = (size_t)b * p.H_q + (size_t)hkv * G;
  const uint8_t* kbase = p.k_data + (size_t)hkv * p.num_slots * KP;

  float mx[G];
#pragma unroll
  for (int h = 0; h < G; ++h) mx[h] = -INFINITY;

  // ------------------------------------------------------------------ phase A
  if (K3) {
    const int r = lane & 15, kb = lane >> 4;
    v8bf qA[NSET][4];
#pragma unroll
    for (int set = 0; set < NSET; ++set) {
      const int h = set * 4 + (r & 3);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (h < G) v = *reinterpret_cast<const uint4*>(p.q + (head0 + h) * D + 32 * kb + 8 * i);
        qA[set][i] = __builtin_bit_cast(v8bf, v);
      }
    }
    const uint16_t* ksbase = p.k_scales + (size_t)hkv * p.num_slots * NG;
    const int kgrp = (NG == 1) ? 0 : (kb >> 1);
    const int cover_end = s0 + ((max(s_cover - s0, 0) + 63) & ~63);
    for (int c0 = s0 + wave * 64; c0 < cover_end; c0 += FS_THREADS) {
      v4f Dt[NSET][4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int set = 0; set < NSET; ++set) Dt[set][j] = (v4f){0.f, 0.f, 0.f, 0.f};
        const int t0 = c0 + 16 * j;
        uint32_t P0 = 0, P1 = 0, P2 = 0;
        float s = 0.f;
        if (t0 + r < s1) {
          const int64_t slot = bt[t0 >> 4] * BS + r;
          const uint32_t* row = reinterpret_cast<const uint32_t*>(kbase + slot * KP);
          P0 = row[kb];
          P1 = row[4 + kb];
          P2 = row[8 + kb];
          s = bf16_to_f32(ksbase[slot * NG + kgrp]);
        }
        if (t0 < s1) {  // wavefront-uniform: skip tiles with no valid token
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t w = (((P0 >> (8 * i)) & 255u) << 16) | (((P1 >> (8 * i)) & 255u) << 8) | ((P2 >> (8 * i)) & 255u);
            uint4 kv;
            uint32_t* kvp = reinterpret_cast<uint32_t*>(&kv);
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
              const int ca = (int)((w >> (21 - 6 * jj)) & 7u) - 4;
              const int cb = (int)((w >> (18 - 6 * jj)) & 7u) - 4;
              kvp[jj] = pack_bf16x2((float)ca * s, (float)cb * s);
            }
            const v8bf kB = __builtin_bit_cast(v8bf, kv);
#pragma unroll
            for (int set = 0; set < NSET; ++set)
              Dt[set][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qA[set][i], kB, Dt[set][j], 0, 0, 0);
          }
        }
      }
      // lane group g keeps tile g: lane l <-> token c0 + l, register <-> head
      const int pos = c0 + lane;
      const bool valid = pos < s1;
#pragma unroll
      for (int set = 0; set < NSET; ++set) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int h = set * 4 + rr;
          if (h < G) {
            const float a = (kb == 0) ? Dt[set][0][rr] : (kb == 1) ? Dt[set][1][rr] : (kb == 2) ? Dt[set][2][rr] : Dt[set][3][rr];
            const float sv = valid ? a * p.attn_scale : -INFINITY;
            if (pos < s_cover) {
              sc[h * L + (pos - s0)] = sv;
              if (p.scores) p.scores[(head0 + h) * (size_t)p.max_S + pos] = sv;
            }
            mx[h] = fmaxf(mx[h], sv);
          }
        }
      }
    }
  } else {
    // INT4 keys, int8-Q model: lane = token
    QInt8F<G>* qsh = reinterpret_cast<QInt8F<G>*>(stage);
    float* scratch = reinterpret_cast<float*>(stage + sizeof(QInt8F<G>));
    const uint16_t* qrow0 = p.q + head0 * D;
    for (int i = tid; i < G * 4; i += FS_THREADS) {
      const int g = i >> 2, kk = i & 3;
      float amax = 0.0f;
      for (int d = 0; d < 32; ++d) amax = fmaxf(amax, fabsf(bf16_to_f32(qrow0[(size_t)g * D + kk * 32 + d])));
      const float s = fmaxf(amax / 127.0f, 1e-12f);
      qsh->qs[g][kk] = s;
      scratch[i] = 1.0f / s;
    }
    __syncthreads();
    for (int i = tid; i < G * 16; i += FS_THREADS) {
      const int g = i >> 4, j = i & 15, kk = j >> 2;
      const float inv = scratch[g * 4 + kk];
      int v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = max(-128, min(127, (int)rintf(bf16_to_f32(qrow0[(size_t)g * D + 8 * j + e]) * inv)));
      qsh->qe[g][j] = (v[0] & 255) | ((v[2] & 255) << 8) | ((v[4] & 255) << 16) | ((v[6] & 255) << 24);
      qsh->qo[g][j] = (v[1] & 255) | ((v[3] & 255) << 8) | ((v[5] & 255) << 16) | ((v[7] & 255) << 24);
    }
    __syncthreads();
    for (int i = tid; i < G * 4; i += FS_THREADS) {
      const int g = i >> 2, kk = i & 3;
      int sum = 0;
      for (int j = 4 * kk; j < 4 * kk + 4; ++j) {
        const int e = qsh->qe[g][j], o = qsh->qo[g][j];
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) sum += (int)(int8_t)((e >> (8 * bb)) & 255) + (int)(int8_t)((o >> (8 * bb)) & 255);
      }
      qsh->sum8[g][kk] = 8 * sum;
    }
    __syncthreads();
    const uint16_t* ksbase = p.k_scales + (size_t)hkv * p.num_slots;
    for (int pos = s0 + tid; pos < s_cover; pos += FS_THREADS) {
      const bool valid = pos < s1;
      uint32_t pk[16];
      float ks = 0.f;
      if (valid) {
        const int64_t slot = bt[pos >> 4] * BS + (pos & 15);
        const uint4* row = reinterpret_cast<const uint4*>(kbase + slot * KP);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint4 v = row[i];
          pk[4 * i] = v.x; pk[4 * i + 1] = v.y; pk[4 * i + 2] = v.z; pk[4 * i + 3] = v.w;
        }
        ks = bf16_to_f32(ksbase[slot]);
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) pk[i] = 0;
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float sacc = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          int acc = 0;
#pragma unroll
          for (int j = 4 * kk; j < 4 * kk + 4; ++j) {
            acc = __builtin_amdgcn_sdot4((int)((pk[j] >> 4) & 0x0f0f0f0fu), qsh->qe[g][j], acc, false);
            acc = __builtin_amdgcn_sdot4((int)(pk[j] & 0x0f0f0f0fu), qsh->qo[g][j], acc, false);
          }
          acc -= qsh->sum8[g][kk];
          sacc = (kk == 0) ? ((float)acc * qsh->qs[g][0]) : __builtin_fmaf((float)acc, qsh->qs[g][kk], sacc);
        }
        const float sv = valid ? __fmul_rn(__fmul_rn(sacc, ks), p.attn_scale) : -INFINITY;
        sc[g * L + (pos - s0)] = sv;
        if (p.scores) p.scores[(head0 + g) * (size_t)p.max_S + pos] = sv;
        mx[g] = fmaxf(mx[g], sv);
      }
    }
  }

  // split max per head
#pragma unroll
  for (int h = 0; h < G; ++h) {
    const float v = wave_max(mx[h]);
    if (lane == 0) red_f[wave][h] = v;
  }
  __syncthreads();
  if (tid < G) m_sh[tid] = fmaxf(fmaxf(red_f[0][tid], red_f[1][tid]), fmaxf(red_f[2][tid], red_f[3][tid]));
  if (tid < 16 * 2) wsum_sh[tid >> 1][tid & 1] = 0ull;
  __syncthreads();

  const size_t part_base = head0 * p.n_splits + split;  // + h * n_splits
  if (n == 0) {
    for (int i = tid; i < G * D; i += FS_THREADS) p.part_o[(part_base + (size_t)(i / D) * p.n_splits) * D + (i % D)] = 0.f;
    if (tid < G) {
      p.part_m[part_base + (size_t)tid * p.n_splits] = -INFINITY;
      p.part_l[part_base + (size_t)tid * p.n_splits] = 0.f;
      p.cand_cnt[part_base + (size_t)tid * p.n_splits] = 0;
    }
    return;
  }

  // ------------------------------------------------------------------ phase B
  const uint8_t* vbase = p.v_data + (size_t)hkv * p.num_slots * VP;
  const uint16_t* vsbase = p.v_scales + (size_t)hkv * p.num_slots * NG;
  {
    float vm[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) vm[g] = 0.f;
    for (int pos = s0 + tid; pos < s1; pos += FS_THREADS) {
      const int64_t slot = bt[pos >> 4] * BS + (pos & 15);
#pragma unroll
      for (int g = 0; g < NG; ++g) vm[g] = fmaxf(vm[g], fabsf(bf16_to_f32(vsbase[slot * NG + g])));
    }
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const float v = wave_max(vm[g]);
      if (lane == 0) vmax_sh[wave][g] = v;
    }
    __syncthreads();
    if (tid < NG) {
      float v = fmaxf(fmaxf(vmax_sh[0][tid], vmax_sh[1][tid]), fmaxf(vmax_sh[2][tid], vmax_sh[3][tid]));
      int e = 0;
      if (v > 0.f && isfinite(v)) (void)frexpf(v, &e);  // v = f * 2^e, f in [0.5, 1)
      e_sh[tid] = 22 - e;                               // v * 2^E in [2^21, 2^22)
    }
    __syncthreads();
  }
  int E[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) E[g] = e_sh[g];

  uint8_t* vst = stage;                                   // [256][VROW]
  uint8_t* wl = stage + FS_THREADS * VROW;                // [4 waves][NG][NSET][16][64]
  v4i acc[NSET][NTILE];
#pragma unroll
  for (int set = 0; set < NSET; ++set)
#pragma unroll
    for (int t = 0; t < NTILE; ++t) acc[set][t] = (v4i){0, 0, 0, 0};
  float lsum[G];
  uint32_t wsum[G][NG];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    lsum[h] = 0.f;
#pragma unroll
    for (int g = 0; g < NG; ++g) wsum[h][g] = 0u;
  }
  float mh[G];
#pragma unroll
  for (int h = 0; h < G; ++h) mh[h] = m_sh[h];
  const int r16 = lane & 15, kb4 = lane >> 4;
  const int bytepos = (kb4 << 4) | token_byte_pos(r16);
  uint8_t* wl_w = wl + wave * WL_WAVE;

  for (int base = s0; base < s1; base += FS_THREADS) {
    __syncthreads();
    const int pos = base + tid;
    const bool valid = pos < s1;
    float vsf[NG];
    {
      uint2* dst = reinterpret_cast<uint2*>(vst + tid * VROW);
      if (valid) {
        const int64_t slot = bt[pos >> 4] * BS + (pos & 15);
        const uint4* src = reinterpret_cast<const uint4*>(vbase + slot * VP);
#pragma unroll
        for (int i = 0; i < VP / 16; ++i) {
          const uint4 v = src[i];
          dst[2 * i] = make_uint2(v.x, v.y);
          dst[2 * i + 1] = make_uint2(v.z, v.w);
        }
#pragma unroll
        for (int g = 0; g < NG; ++g) vsf[g] = ldexpf(bf16_to_f32(vsbase[slot * NG + g]), E[g]);
      } else {
#pragma unroll
        for (int i = 0; i < VP / 8; ++i) dst[i] = make_uint2(0u, 0u);
#pragma unroll
        for (int g = 0; g < NG; ++g) vsf[g] = 0.f;
      }
    }
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const float pw = valid ? __expf(sc[h * L + (pos - s0)] - mh[h]) : 0.f;
      lsum[h] += pw;
      const int set = h >> 2, hh = h & 3;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const uint32_t bits = __builtin_bit_cast(uint32_t, __builtin_fmaf(pw, vsf[g], 8388608.0f));
        wsum[h][g] += bits & 0x7fffffu;
        const uint32_t lim = bits ^ 0x00008080u;
        uint8_t* rowp = wl_w + ((g * NSET + set) * 16) * 64 + bytepos;
        rowp[(0 * 4 + hh) * 64] = (uint8_t)(lim & 255u);
        rowp[(1 * 4 + hh) * 64] = (uint8_t)((lim >> 8) & 255u);
        rowp[(2 * 4 + hh) * 64] = (uint8_t)((lim >> 16) & 255u);
      }
    }
    __syncthreads();
    if (base + wave * 64 < s1) {  // this wavefront's 64-token chunk holds at least one valid token
      v4i A[NG][NSET];
#pragma unroll
      for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int set = 0; set < NSET; ++set) {
          if (r16 < 12) {
            A[g][set] = *reinterpret_cast<const v4i*>(wl_w + ((g * NSET + set) * 16 + r16) * 64 + kb4 * 16);
          } else if (r16 == 12) {
            A[g][set] = (v4i){0x01010101, 0x01010101, 0x01010101, 0x01010101};
          } else {
            A[g][set] = (v4i){0, 0, 0, 0};
          }
        }
      const uint8_t* vrow = vst + (wave * 64 + lane) * VROW;
      if (K3) {
#pragma unroll
        for (int qc = 0; qc < 4; ++qc) {
          const v2i x = __builtin_amdgcn_ds_read_tr4_b64_v2i32(
              (__attribute__((address_space(3))) v2i*)(vrow + 8 * qc));
          const uint32_t x0 = (uint32_t)x[0], x1 = (uint32_t)x[1];
          const v4i Ba = {(int)((x0 >> 2) & 0x03030303u), (int)((x0 >> 6) & 0x03030303u),
                          (int)((x1 >> 2) & 0x03030303u), (int)((x1 >> 6) & 0x03030303u)};
          const v4i Bb = {(int)(x0 & 0x03030303u), (int)((x0 >> 4) & 0x03030303u),
                          (int)(x1 & 0x03030303u), (int)((x1 >> 4) & 0x03030303u)};
          const int g = (NG == 1) ? 0 : (qc >> 1);
#pragma unroll
          for (int set = 0; set < NSET; ++set) {
            acc[set][2 * qc] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[g][set], Ba, acc[set][2 * qc], 0, 0, 0);
            acc[set][2 * qc + 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[g][set], Bb, acc[set][2 * qc + 1], 0, 0, 0);
          }
        }
      } else {
#pragma unroll
        for (int qc = 0; qc < 8; ++qc) {
          const v2i x = __builtin_amdgcn_ds_read_tr4_b64_v2i32(
              (__attribute__((address_space(3))) v2i*)(vrow + 8 * qc));
          const uint32_t x0 = (uint32_t)x[0], x1 = (uint32_t)x[1];
          const v4i Bv = {(int)(x0 & 0x0f0f0f0fu), (int)((x0 >> 4) & 0x0f0f0f0fu),
                          (int)(x1 & 0x0f0f0f0fu), (int)((x1 >> 4) & 0x0f0f0f0fu)};
          const int g = (NG == 1) ? 0 : (qc >> 2);
#pragma unroll
          for (int set = 0; set < NSET; ++set)
            acc[set][qc] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[g][set], Bv, acc[set][qc], 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();

  // reduce the four wavefronts' integer accumulators in LDS: red_i[set][tile][row][col]
  int* red_i = reinterpret_cast<int*>(stage);
  for (int i = tid; i < NSET * NTILE * 256; i += FS_THREADS) red_i[i] = 0;
  __syncthreads();
#pragma unroll
  for (int set = 0; set < NSET; ++set)
#pragma unroll
    for (int t = 0; t < NTILE; ++t)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int row = 4 * kb4 + rr;
        if (row <= 12) atomicAdd(&red_i[((set * NTILE + t) * 16 + row) * 16 + r16], acc[set][t][rr]);
      }
#pragma unroll
  for (int h = 0; h < G; ++h) {
    const float ls = wave_sum(lsum[h]);
    if (lane == 0) red_f[wave][h] = ls;  // summed in wavefront order below: run-to-run deterministic
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      unsigned long long wv = wsum[h][g];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) wv += __shfl_xor(wv, off);
      if (lane == 0) atomicAdd(&wsum_sh[h][g], wv);
    }
  }
  __syncthreads();
  for (int i = tid; i < G * D; i += FS_THREADS) {
    const int h = i / D, d = i % D;
    const int set = h >> 2, hh = h & 3;
    int tile, col;
    if (K3) {
      const int qc = d >> 5, rem = d & 31, kbyte = rem >> 2, e = rem & 3;
      col = 2 * kbyte + ((e < 2) ? 1 : 0);
      tile = 2 * qc + (e & 1);
    } else {
      const int qc = d >> 4, rem = d & 15, kbyte = rem >> 1;
      col = 2 * kbyte + ((rem & 1) ? 0 : 1);
      tile = qc;
    }
    const int g = (NG == 1) ? 0 : (d / (D / NG));
    const int* tb = red_i + (set * NTILE + tile) * 256;
    const long long i0 = tb[(0 * 4 + hh) * 16 + col], i1 = tb[(1 * 4 + hh) * 16 + col], i2 = tb[(2 * 4 + hh) * 16 + col];
    const long long cs = tb[12 * 16 + col];
    const long long tot = i2 * 65536ll + i1 * 256ll + i0 + 32896ll * cs - (long long)VOFF * (long long)wsum_sh[h][g];
    p.part_o[(part_base + (size_t)h * p.n_splits) * D + d] = (float)ldexp((double)tot, -E[g]);
  }
  if (tid < G) {
    p.part_m[part_base + (size_t)tid * p.n_splits] = m_sh[tid];
    p.part_l[part_base + (size_t)tid * p.n_splits] = ((red_f[0][tid] + red_f[1][tid]) + red_f[2][tid]) + red_f[3][tid];
  }
  __syncthreads();

  // ------------------------------------------------------------------ phase C: per-head radix select
  int* hist = reinterpret_cast<int*>(stage) + wave * 256;
  const int Kc = p.Kc;
  for (int h = wave; h < G; h += FS_WAVES) {
    const float* row = sc + h * L;
    uint32_t* ck = p.cand_key + (part_base + (size_t)h * p.n_splits) * Kc;
    int32_t* ci = p.cand_idx + (part_base + (size_t)h * p.n_splits) * Kc;
    uint32_t tau = 0;
    int quota = 0;
    const bool take_all = (n <= Kc);
    if (!take_all) {
      uint32_t prefix = 0;
      int k_rem = Kc;
      for (int level = 0; level < 4; ++level) {
        for (int i = lane; i < 256; i += 64) hist[i] = 0;
        const int shift = 24 - 8 * level;
        for (int i = lane; i < n; i += 64) {
          const uint32_t key = score_key(row[i]);
          if (level == 0 || (key >> (shift + 8)) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1);
        }
        // suffix scan over 256 bins, 4 bins per lane (lane owns bins 4*lane .. 4*lane+3)
        const int c0 = hist[4 * lane], c1 = hist[4 * lane + 1], c2 = hist[4 * lane + 2], c3 = hist[4 * lane + 3];
        const int mine = c0 + c1 + c2 + c3;
        int incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const int o = __shfl_down(incl, off);
          if (lane + off < 64) incl += o;
        }
        const int above_lane = incl - mine;  // keys in bins of higher lanes
        int cut = -1, above = 0;
        const int s3 = above_lane, s2 = s3 + c3, s1x = s2 + c2, s0x = s1x + c1;
        if (s3 < k_rem && k_rem <= s3 + c3) { cut = 4 * lane + 3; above = s3; }
        else if (s2 < k_rem && k_rem <= s2 + c2) { cut = 4 * lane + 2; above = s2; }
        else if (s1x < k_rem && k_rem <= s1x + c1) { cut = 4 * lane + 1; above = s1x; }
        else if (s0x < k_rem && k_rem <= s0x + c0) { cut = 4 * lane; above = s0x; }
        const unsigned long long who = __ballot(cut >= 0);
        const int src = __ffsll((long long)who) - 1;
        cut = __shfl(cut, src);
        above = __shfl(above, src);
        prefix = (prefix << 8) | (uint32_t)cut;
        k_rem -= above;
      }
      tau = prefix;
      quota = k_rem;
    }
    int base_above = 0, base_tie = 0;
    for (int i0 = 0; i0 < n; i0 += 64) {
      const int i = i0 + lane;
      bool above = false, tie = false;
      uint32_t key = 0;
      if (i < n) {
        key = score_key(row[i]);
        if (take_all) above = true;
        else { above = key > tau; tie = key == tau; }
      }
      const unsigned long long ma = __ballot(above), mt = __ballot(tie);
      const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
      const int pa = base_above + __popcll(ma & lt), pt = base_tie + __popcll(mt & lt);
      if (above || (tie && pt < quota)) {
        const int pos = pa + min(pt, quota);
        if (pos < Kc) {
          ck[pos] = key;
          ci[pos] = s0 + i;
        }
      }
      base_above += __popcll(ma);
      base_tie += __popcll(mt);
    }
    if (lane == 0) p.cand_cnt[part_base + (size_t)h * p.n_splits] = min(Kc, base_above + min(base_tie, quota));
  }
}

// ---------------------------------------------------------------------------------------------------
constexpr int MG_THREADS = 256;
constexpr int MG_WAVES = MG_THREADS / 64;

template <int VBITS, int NG>
__global__ __launch_bounds__(MG_THREADS) void fused_merge_kernel(FusedParams p) {
  constexpr int VP = D * VBITS / 8;
  constexpr int VOFF = 1 << (VBITS - 1);
  __shared__ int hist[MG_WAVES][256];
  __shared__ int suffix_wave[4];
  __shared__ int cut_bin_sh, above_sh;
  __shared__ int wave_above[MG_WAVES], wave_tie[MG_WAVES];
  __shared__ float coef_sh[1024];
  __shared__ float stat_sh[2];
  __shared__ int64_t slot_buf[128];
  __shared__ float ws_buf[128][NG];
  __shared__ float w_buf[128];

  const int b = blockIdx.x, hq = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t bh = (size_t)b * p.H_q + hq;
  const int NS = p.n_splits, Kc = p.Kc, K = p.top_k;
  const int hkv = hq / (p.H_q / p.H_kv);
  const uint32_t* ck = p.cand_key + bh * NS * Kc;
  const int32_t* ci = p.cand_idx + bh * NS * Kc;
  const int32_t* cc = p.cand_cnt + bh * NS;
  const int64_t* bt = p.block_table + (size_t)b * p.max_blocks;
  int64_t* out_idx = p.topk_idx + bh * (size_t)K;
  int64_t* out_slot = p.topk_slots + bh * (size_t)K;

  // ---- split statistics: M, l, coefficients
  float mloc = -INFINITY;
  for (int s = tid; s < NS; s += MG_THREADS) mloc = fmaxf(mloc, p.part_m[bh * NS + s]);
  mloc = wave_max(mloc);
  if (lane == 0) coef_sh[wave] = mloc;
  __syncthreads();
  float M = fmaxf(fmaxf(coef_sh[0], coef_sh[1]), fmaxf(coef_sh[2], coef_sh[3]));
  if (!isfinite(M)) M = 0.f;
  __syncthreads();
  if (tid == 0) {
    float l = 0.f;
    for (int s = 0; s < NS; ++s) {  // fixed order: deterministic
      const float ms = p.part_m[bh * NS + s];
      const float c = (ms == -INFINITY) ? 0.f : __expf(ms - M);
      if (s < 1024) coef_sh[s] = c;
      l += p.part_l[bh * NS + s] * c;
    }
    stat_sh[0] = l;
    stat_sh[1] = (l > 0.f) ? 1.0f / l : 0.f;
  }
  __syncthreads();
  const float inv_z = stat_sh[1];
  if (tid < D) {
    float o = 0.f;
    for (int s = 0; s < NS; ++s) o = __builtin_fmaf(p.part_o[(bh * NS + s) * D + tid], coef_sh[s], o);
    p.o_hat[bh * D + tid] = o * inv_z;
  }
  if (tid == 0 && p.softmax_m) {
    p.softmax_m[bh] = M;
    p.softmax_inv_z[bh] = inv_z;
  }

  // ---- global top-k among the candidates
  int total = 0;
  for (int s = 0; s < NS; ++s) total += cc[s];  // uniform scalar loop (NS <= 1024)
  const int flat = NS * Kc;
  uint32_t tau = 0;
  int quota = 0;
  const bool take_all = (total <= K);
  if (!take_all) {
    uint32_t prefix = 0;
    int k_rem = K;
    for (int level = 0; level < 4; ++level) {
      for (int i = tid; i < MG_WAVES * 256; i += MG_THREADS) (&hist[0][0])[i] = 0;
      __syncthreads();
      const int shift = 24 - 8 * level;
      for (int f = tid; f < flat; f += MG_THREADS) {
        if ((f % Kc) < cc[f / Kc]) {
          const uint32_t key = ck[f];
          if (level == 0 || (key >> (shift + 8)) == prefix) atomicAdd(&hist[wave][(key >> shift) & 255u], 1);
        }
      }
      __syncthreads();
      int cnt = hist[0][tid] + hist[1][tid] + hist[2][tid] + hist[3][tid];  // MG_THREADS == 256 bins
      int incl = cnt;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int o = __shfl_down(incl, off);
        if (lane + off < 64) incl += o;
      }
      if (lane == 0) suffix_wave[wave] = incl;
      __syncthreads();
      int higher = 0;
      for (int w = wave + 1; w < 4; ++w) higher += suffix_wave[w];
      const int s_incl = incl + higher, s_excl = s_incl - cnt;
      if (s_excl < k_rem && k_rem <= s_incl) {
        cut_bin_sh = tid;
        above_sh = s_excl;
      }
      __syncthreads();
      prefix = (prefix << 8) | (uint32_t)cut_bin_sh;
      k_rem -= above_sh;
      __syncthreads();
    }
    tau = prefix;
    quota = k_rem;
  }
  int base_above = 0, base_tie = 0;
  const int flat_round = (flat + MG_THREADS - 1) / MG_THREADS * MG_THREADS;
  for (int f0 = 0; f0 < flat_round; f0 += MG_THREADS) {
    const int f = f0 + tid;
    bool above = false, tie = false;
    if (f < flat && (f % Kc) < cc[f / Kc]) {
      if (take_all) above = true;
      else {
        const uint32_t key = ck[f];
        above = key > tau;
        tie = key == tau;
      }
    }
    const unsigned long long ma = __ballot(above), mt = __ballot(tie);
    const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    if (lane == 0) {
      wave_above[wave] = __popcll(ma);
      wave_tie[wave] = __popcll(mt);
    }
    __syncthreads();
    int pa = base_above + __popcll(ma & lt), pt = base_tie + __popcll(mt & lt);
    int tot_a = 0, tot_t = 0;
#pragma unroll
    for (int w = 0; w < MG_WAVES; ++w) {
      if (w < wave) { pa += wave_above[w]; pt += wave_tie[w]; }
      tot_a += wave_above[w];
      tot_t += wave_tie[w];
    }
    if (above || (tie && pt < quota)) {
      const int pos = pa + min(pt, quota);
      if (pos < K) out_idx[pos] = ((int64_t)f << 32) | (uint32_t)ci[f];  // provisional: candidate id + position
    }
    base_above += tot_a;
    base_tie += tot_t;
    __syncthreads();
  }
  const int n_out = min(K, base_above + min(base_tie, quota));
  __syncthreads();

  // ---- winners: finalise indices/slots and the pre-correction terms
  const int grp = (NG == 1) ? 0 : ((tid & (D - 1)) / (D / NG));
  const uint8_t* vbase = p.v_data + (size_t)hkv * p.num_slots * VP;
  const uint16_t* vsbase = p.v_scales + (size_t)hkv * p.num_slots * NG;
  const int dch = tid & (D - 1), half = tid >> 7;  // two halves of the 256 threads split the winners
  float acc_old = 0.f, acc_w = 0.f;
  for (int k0 = 0; k0 < K; k0 += 128) {
    __syncthreads();
    if (tid < 128) {
      const int kk = k0 + tid;
      int64_t slot = -1;
      float w = 0.f;
      if (kk < K) {
        if (kk < n_out) {
          const int64_t packed = out_idx[kk];
          const int f = (int)(packed >> 32);
          const int pos = (int)(packed & 0xffffffffll);
          const int blk = pos / BS;
          slot = (blk < p.max_blocks) ? bt[blk] * BS + (pos % BS) : -1;
          out_idx[kk] = pos;
          out_slot[kk] = slot;
          if (slot >= 0) w = __expf(key_to_score(ck[f]) - M) * inv_z;
        } else {
          out_idx[kk] = -1;
          out_slot[kk] = -1;
        }
      }
      slot_buf[tid] = slot;
      w_buf[tid] = w;
#pragma unroll
      for (int g = 0; g < NG; ++g) ws_buf[tid][g] = (slot >= 0) ? w * bf16_to_f32(vsbase[slot * NG + g]) : 0.f;
    }
    __syncthreads();
    const int kend = min(128, K - k0);
    for (int j = half; j < kend; j += 2) {
      const int64_t slot = slot_buf[j];
      if (slot < 0) continue;
      const uint8_t* vr = vbase + slot * VP;
      int c;
      if (VBITS == 2) c = (int)((vr[dch >> 2] >> ((3 - (dch & 3)) * 2)) & 3) - VOFF;
      else c = (int)((vr[dch >> 1] >> ((1 - (dch & 1)) * 4)) & 15) - VOFF;
      acc_old = __builtin_fmaf(ws_buf[j][grp], (float)c, acc_old);
      acc_w += w_buf[j];
    }
  }
  // combine the two halves (fixed order)
  __syncthreads();
  float* comb = coef_sh;  // reuse: [2][D] + [2]
  comb[half * D + dch] = acc_old;
  if (dch == 0) comb[2 * D + half] = acc_w;
  __syncthreads();
  if (tid < D) p.o_old[bh * D + tid] = comb[tid] + comb[D + tid];
  if (tid == 0) p.W[bh] = comb[2 * D] + comb[2 * D + 1];
}

// Optional measurement hook: when armed, every fused_scan_kernel launch is bracketed by a pair of HIP
// events on its own stream, so a benchmark can read the kernel's device time without a profiler.
struct ScanProfile {
  std::vector<hipEvent_t> ev;
  int used = 0;
  bool armed = false;
};
ScanProfile g_prof;

inline int lmax_for_group(int G) { return G <= 4 ? 2048 : (G <= 8 ? 1024 : 512); }

inline void fused_plan(int B, int H_q, int H_kv, int max_S, int top_k, int* L_out, int* ns_out, int* kc_out) {
  const int G = H_q / H_kv;
  const int units = B * H_kv > 0 ? B * H_kv : 1;
  int target = 512 / units;
  if (target < 1) target = 1;
  int L = (max_S + target - 1) / target;
  L = (L + 255) / 256 * 256;
  const int lmax = lmax_for_group(G);
  if (L > lmax) L = lmax;
  if (L < 256) L = 256;
  int ns = (max_S + L - 1) / L;
  if (ns < 1) ns = 1;
  *L_out = L;
  *ns_out = ns;
  *kc_out = top_k < L ? top_k : L;
}

struct WsLayout {
  size_t off_m, off_l, off_o, off_key, off_idx, off_cnt, total;
};
inline WsLayout ws_layout(int B, int H_q, int ns, int kc) {
  WsLayout w;
  const size_t rows = (size_t)B * H_q;
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t r = o; o += (bytes + 255) / 256 * 256; return r; };
  w.off_m = take(rows * ns * 4);
  w.off_l = take(rows * ns * 4);
  w.off_o = take(rows * ns * D * 4);
  w.off_key = take(rows * ns * kc * 4);
  w.off_idx = take(rows * ns * kc * 4);
  w.off_cnt = take(rows * ns * 4);
  w.total = o + 256;
  return w;
}

template <int SCHEME, int G, int NG>
int launch_scan(const FusedParams& p, hipStream_t st) {
  constexpr bool K3 = (SCHEME == JF_SCHEME_K3V2);
  constexpr int NSET = (G + 3) / 4;
  constexpr int VROW = (K3 ? 32 : 64) + 8;
  size_t stage = (size_t)FS_THREADS * VROW + (size_t)FS_WAVES * NG * NSET * 16 * 64;
  const size_t red = (size_t)NSET * 8 * 256 * 4;
  if (red > stage) stage = red;
  const size_t qsz = sizeof(QInt8F<G>) + G * 4 * sizeof(float);
  if (!K3 && qsz > stage) stage = qsz;
  const size_t smem = (size_t)G * p.L * sizeof(float) + stage;
  auto kern = fused_scan_kernel<SCHEME, G, NG>;
  static size_t attr_smem = 0;  // per instantiation: raise the dynamic-LDS limit only when it grows
  if (smem > attr_smem) {
    JF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    attr_smem = smem;
  }
  const bool prof = g_prof.armed && g_prof.used + 2 <= (int)g_prof.ev.size();
  if (prof) JF_CHECK_HIP(hipEventRecord(g_prof.ev[g_prof.used], st));
  hipLaunchKernelGGL(kern, dim3(p.n_splits, p.H_kv, p.B), dim3(FS_THREADS), smem, st, p);
  JF_CHECK_LAUNCH();
  if (prof) {
    JF_CHECK_HIP(hipEventRecord(g_prof.ev[g_prof.used + 1], st));
    g_prof.used += 2;
  }
  return JF_OK;
}

}  // namespace
}  // namespace jf

using namespace jf;

extern "C" size_t jf_fused_workspace_bytes(int scheme, int B, int H_q, int H_kv, int max_S, int top_k) {
  (void)scheme;
  if (B <= 0 || H_q <= 0 || H_kv <= 0 || H_q % H_kv != 0 || max_S < 0 || top_k <= 0) return 256;
  int L, ns, kc;
  fused_plan(B, H_q, H_kv, max_S, top_k, &L, &ns, &kc);
  return ws_layout(B, H_q, ns, kc).total;
}

extern "C" int jf_fused_scan_topk(int scheme, int group_size, const uint16_t* q, const uint8_t* k_data,
                                  const uint16_t* k_scales, const uint8_t* v_data, const uint16_t* v_scales,
                                  const int64_t* block_table, const int32_t* seq_lens, int B, int H_q, int H_kv,
                                  int max_S, int max_blocks, int64_t num_slots, int block_size, float attn_scale,
                                  int top_k, int64_t* topk_idx, int64_t* topk_slots, float* o_hat,
                                  float* o_old_unnorm, float* W, float* softmax_m, float* softmax_inv_z, float* scores,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  JF_CHECK_ARG(scheme == JF_SCHEME_K3V2 || scheme == JF_SCHEME_K4V4, "fused_scan: unknown scheme %d", scheme);
  JF_CHECK_ARG(B >= 0 && H_q > 0 && H_kv > 0 && max_S >= 0 && H_q % H_kv == 0, "fused_scan: bad shape");
  const int G = H_q / H_kv;
  JF_CHECK_ARG(G == 1 || G == 2 || G == 4 || G == 8 || G == 16, "fused_scan: GQA group %d not in {1,2,4,8,16}", G);
  JF_CHECK_ARG(block_size == 16, "fused_scan only supports block_size=16");
  JF_CHECK_ARG(group_size == 64 || group_size == 128, "fused_scan: group_size must be 64 or 128 (got %d)", group_size);
  JF_CHECK_ARG(scheme != JF_SCHEME_K4V4 || group_size == 128, "fused_scan: the INT4 int8-Q path needs group_size 128");
  JF_CHECK_ARG(is_pow2(top_k) && top_k >= 32 && top_k <= 8192, "fused_scan: unsupported top_k=%d", top_k);
  JF_CHECK_ARG(max_S <= 262144, "fused_scan: max_S=%d exceeds supported limit (262144)", max_S);
  JF_CHECK_ARG((int64_t)max_blocks * block_size >= max_S, "fused_scan: block_table does not cover max_S");
  JF_CHECK_ARG((softmax_m == nullptr) == (softmax_inv_z == nullptr), "fused_scan: softmax_m and softmax_inv_z go together");
  if (B == 0) return JF_OK;
  JF_CHECK_ARG(q && k_data && k_scales && v_data && v_scales && block_table && seq_lens, "fused_scan: null input");
  JF_CHECK_ARG(topk_idx && topk_slots && o_hat && o_old_unnorm && W, "fused_scan: null output");
  JF_CHECK_ARG(((uintptr_t)k_data & 15) == 0 && ((uintptr_t)v_data & 15) == 0 && ((uintptr_t)q & 15) == 0,
               "fused_scan: q, k_data and v_data must be 16-byte aligned");
  FusedParams p;
  p.q = q; p.k_data = k_data; p.k_scales = k_scales; p.v_data = v_data; p.v_scales = v_scales;
  p.block_table = block_table; p.seq_lens = seq_lens;
  p.B = B; p.H_q = H_q; p.H_kv = H_kv; p.max_S = max_S; p.max_blocks = max_blocks; p.num_slots = num_slots;
  p.attn_scale = attn_scale; p.top_k = top_k;
  fused_plan(B, H_q, H_kv, max_S, top_k, &p.L, &p.n_splits, &p.Kc);
  JF_CHECK_ARG(p.n_splits <= 1024, "fused_scan: too many splits (%d)", p.n_splits);
  const WsLayout wl = ws_layout(B, H_q, p.n_splits, p.Kc);
  JF_CHECK_ARG(workspace && workspace_bytes >= wl.total, "fused_scan: workspace too small (%zu < %zu)", workspace_bytes, wl.total);
  JF_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fused_scan: workspace must be 256-byte aligned");
  uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
  p.scores = scores;
  p.part_m = reinterpret_cast<float*>(ws + wl.off_m);
  p.part_l = reinterpret_cast<float*>(ws + wl.off_l);
  p.part_o = reinterpret_cast<float*>(ws + wl.off_o);
  p.cand_key = reinterpret_cast<uint32_t*>(ws + wl.off_key);
  p.cand_idx = reinterpret_cast<int32_t*>(ws + wl.off_idx);
  p.cand_cnt = reinterpret_cast<int32_t*>(ws + wl.off_cnt);
  p.topk_idx = topk_idx; p.topk_slots = topk_slots; p.o_hat = o_hat; p.o_old = o_old_unnorm; p.W = W;
  p.softmax_m = softmax_m; p.softmax_inv_z = softmax_inv_z;
  hipStream_t st = (hipStream_t)stream;
  const int NGv = D / group_size;
  int rc = JF_OK;
#define JF_FUSED_CASE(SCH, GG, NGG) rc = launch_scan<SCH, GG, NGG>(p, st)
  if (scheme == JF_SCHEME_K3V2) {
    if (NGv == 2) {
      switch (G) {
        case 1: JF_FUSED_CASE(JF_SCHEME_K3V2, 1, 2); break;
        case 2: JF_FUSED_CASE(JF_SCHEME_K3V2, 2, 2); break;
        case 4: JF_FUSED_CASE(JF_SCHEME_K3V2, 4, 2); break;
        case 8: JF_FUSED_CASE(JF_SCHEME_K3V2, 8, 2); break;
        default: JF_FUSED_CASE(JF_SCHEME_K3V2, 16, 2); break;
      }
    } else {
      switch (G) {
        case 1: JF_FUSED_CASE(JF_SCHEME_K3V2, 1, 1); break;
        case 2: JF_FUSED_CASE(JF_SCHEME_K3V2, 2, 1); break;
        case 4: JF_FUSED_CASE(JF_SCHEME_K3V2, 4, 1); break;
        case 8: JF_FUSED_CASE(JF_SCHEME_K3V2, 8, 1); break;
        default: JF_FUSED_CASE(JF_SCHEME_K3V2, 16, 1); break;
      }
    }
  } else {
    switch (G) {
      case 1: JF_FUSED_CASE(JF_SCHEME_K4V4, 1, 1); break;
      case 2: JF_FUSED_CASE(JF_SCHEME_K4V4, 2, 1); break;
      case 4: JF_FUSED_CASE(JF_SCHEME_K4V4, 4, 1); break;
      case 8: JF_FUSED_CASE(JF_SCHEME_K4V4, 8, 1); break;
      default: JF_FUSED_CASE(JF_SCHEME_K4V4, 16, 1); break;
    }
  }
  if (rc != JF_OK) return rc;
  dim3 mgrid(B, H_q), mblock(MG_THREADS);
  if (scheme == JF_SCHEME_K3V2) {
    if (NGv == 2) hipLaunchKernelGGL((fused_merge_kernel<2, 2>), mgrid, mblock, 0, st, p);
    else hipLaunchKernelGGL((fused_merge_kernel<2, 1>), mgrid, mblock, 0, st, p);
  } else {
    hipLaunchKernelGGL((fused_merge_kernel<4, 1>), mgrid, mblock, 0, st, p);
  }
  JF_CHECK_LAUNCH();
  return JF_OK;
}

extern "C" int jf_profile_scan_begin(int max_launches) {
  JF_CHECK_ARG(max_launches > 0 && max_launches <= (1 << 20), "profile_scan_begin: bad max_launches=%d", max_launches);
  for (hipEvent_t e : g_prof.ev) (void)hipEventDestroy(e);
  g_prof.ev.assign((size_t)max_launches * 2, nullptr);
  for (auto& e : g_prof.ev) JF_CHECK_HIP(hipEventCreate(&e));
  g_prof.used = 0;
  g_prof.armed = true;
  return JF_OK;
}

extern "C" int jf_profile_scan_end(double* total_ms, int* launches) {
  JF_CHECK_ARG(total_ms && launches, "profile_scan_end: null output");
  g_prof.armed = false;
  double tot = 0.0;
  for (int i = 0; i + 1 < g_prof.used; i += 2) {
    JF_CHECK_HIP(hipEventSynchronize(g_prof.ev[i + 1]));
    float ms = 0.f;
    JF_CHECK_HIP(hipEventElapsedTime(&ms, g_prof.ev[i], g_prof.ev[i + 1]));
    tot += ms;
  }
  *total_ms = tot;
  *launches = g_prof.used / 2;
  for (hipEvent_t e : g_prof.ev) (void)hipEventDestroy(e);
  g_prof.ev.clear();
  g_prof.used = 0;
  return JF_OK;
}
