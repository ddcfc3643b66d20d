// Fused decode scan + top-k for gfx950: one pass over the packed K and V of every (sequence, kv-head),
// no (B, H_q, S) score tensor in HBM.
//
// Launch 1, fused_scan_kernel, grid (n_splits, H_kv, B), 16 wavefronts per workgroup (8 where the register
// budget does not allow 1024 threads).  A workgroup owns L consecutive positions of one (sequence, kv-head)
// and all G query heads of that kv-head.  The page table of the split is read once into LDS.  Key and value
// rows are fetched in 64-position chunks with 16-byte loads whose lane addresses are consecutive inside a
// page, two chunks per wavefront in flight, staged in wavefront-private LDS and read back in the layout the
// arithmetic wants; barriers order LDS traffic only, so prefetched rows stay in flight across them.
//   phase A  Q.K^T on v_mfma_i32_16x16x64_i8, tokens on the N side, rows = (head, limb or block):
//            INT3 keys: the bf16 query as exact 23-bit fixed point in three int8 limbs, codes spread from the
//                       byte planes with shift/mask on dwords, a second contraction with the indicator of
//                       codes +-3 reproduces the reference's bf16 rounding of the dequantised key.
//            INT2 keys: the same limbs against the four-codes-per-byte rows; no second contraction, every
//                       dequantised INT2 key is exact in bf16.
//            INT4 keys: int8-quantised Q, exact nibble codes, one accumulator row per 32-channel block, the
//                       reference's fp32 rescale order (bit-equal to the split-form kernel).
//            scores[G][L] -> LDS (fp32), running max / min per head.
//   phase B  P.V on the same MFMA.  p = exp(s - m_split) is known exactly because phase A is complete, so
//            w = p * v_scale is converted to 23-bit fixed point once (fma with 2^23), the four bytes of the
//            converted word are the A-operand rows (head, limb 0..2 and the constant exponent byte), and the
//            int32 accumulators live for the whole split: every product is exact.  V codes are transposed by
//            ds_read_b64_tr_b4, weight rows by ds_read_b64_tr_b8.
//            The same pass drops every score into one of 256 linear buckets per (head, segment).
//   phase C  one wavefront per (head, segment): from the bucket histograms the smallest bucket range that holds
//            the split's top min(K, n) scores and fits the candidate buffer (every wavefront of a head finds it
//            itself); its positions are emitted as (key, position) in ascending position, sixteen consecutive
//            scores per lane and block.  Heavily tied scores fall back to a radix select.
//   sum of the wavefronts' integer accumulators with LDS integer atomics (issued along the emission's
//   comparisons), exact int64 recombination -> partial o.
// Launch 2, fused_merge_kernel, grid (B, H_q): selects the global top-k among the candidates (ties to
// the lower position, ascending output), merges the split partials
//   M = max m_i, l = sum l_i e^{m_i-M}, o_hat = sum o_i e^{m_i-M} / l
// (the split-KV combine of jetfire_vllm/csrc/fused_decode_wmma.cu:1226-1253), and computes the
// pre-correction terms o_old_unnorm, W over the winners (jetfire_vllm/csrc/int2_softmax_v.cu:738-788).
// Both kernels take a template argument MODE: the whole step, or one stage alone (Stage A: scores written out,
// top-k, statistics; Stage B: scores and winners given, value stream; selection alone), for callers that keep the
// reference's separate operators.
//
// This header holds the kernels, the launch planner and the launcher; it is included by the translation units that
// instantiate them (fused_scan.hip and the stage-wise forms), each for its own set of template arguments.
#pragma once
#include "common.h"

#include <atomic>
#include <type_traits>
#include <mutex>
#include <vector>

namespace jf {

#ifdef JF_DEBUG_HOOKS
// Process-wide measurement / test switches shared by those translation units (defined in fused_scan.hip),
// reachable from the debug entry points of jetfire_amd_debug.h; a library built without JF_DEBUG_HOOKS has none of
// them.  The event list has its own lock, the two scalars are atomics (a launch reads each once).
// Optional measurement hook: when armed, every fused_scan_kernel launch is bracketed by a pair of HIP
// events on its own stream, so a benchmark can read the kernel's device time without a profiler.
struct ScanProfile {
  std::vector<hipEvent_t> ev;
  int used = 0;
  std::atomic<bool> armed{false};
};
extern ScanProfile g_prof;
extern std::mutex g_prof_mu;
extern std::atomic<long long*> g_phase_clock;
extern std::atomic<int> g_force_split_len;  // test / measurement aid: overrides the planner's split length when positive
constexpr bool kDebugHooks = true;
// clock of the phase stamps: the wavefront's own cycle counter, or (JF_STAMP_WALL_CLOCK) the constant 100 MHz counter
// that every XCD shares, for comparing workgroups on different XCDs (their cycle counters run at different rates)
#ifdef JF_STAMP_WALL_CLOCK
#define JF_CLK() ((long long)wall_clock64())
#else
#define JF_CLK() clock64()
#endif
#else
#define JF_CLK() 0ll
constexpr bool kDebugHooks = false;
#endif
// Compute units of the current device (the planner balances workgroups over them); 256, the MI355X count, when
// no device can be asked (planning on a host without a GPU).
int device_cus();
// The one-pass scan kernels are instantiated in four translation units (fused_full_*.hip), one per family of
// schemes, so that they compile side by side; `params` points to the launcher's FusedParams.
int launch_full_scan_a(int scheme, int G, int NG, const void* params, void* stream);  // K3V2, K4V4, K3V4, K4V2
int launch_full_scan_b(int scheme, int G, int NG, const void* params, void* stream);  // K2V2, K2V3, K2V4
int launch_full_scan_c(int scheme, int G, int NG, const void* params, void* stream);  // K3V3, K4V3
int launch_full_scan_d(int scheme, int G, int NG, const void* params, void* stream);  // A2V2, A2V3, A2V4
int launch_full_scan_e(int scheme, int G, int NG, const void* params, void* stream);  // B4V2, B4V3, B4V4

namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v3i __attribute__((ext_vector_type(3)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

// Forms of the step (template argument MODE of both kernels):
//   FS_FULL     Stage A + Stage B + top-k in one pass (keys and values streamed once, scores never in HBM)
//   FS_STAGE_A  Stage A alone: scores (optionally written out), top-k, softmax statistics; no value stream
//   FS_STAGE_B  Stage B alone: scores and winners are inputs; value stream, o_hat and the pre-correction terms
//   FS_TOPK     selection alone: scores are an input; top-k, slots and softmax statistics (scan kernel only; its
//               merge is the FS_STAGE_A one)
constexpr int FS_FULL = 0, FS_STAGE_A = 1, FS_STAGE_B = 2, FS_TOPK = 3;

constexpr int FS_MAX_TOPK = 8192;      // widest correction
constexpr int FS_LDS_TOPK = 2048;      // winners the merge kernel keeps in static LDS; wider ones go to dynamic LDS
constexpr long long FS_MAX_SLOTS = 1ll << 26;  // slots per kv-head tensor: 64-byte rows, 32-bit row offsets (4 GB)
constexpr int FS_CAND_SLACK = 256;     // extra candidate slots per (row, split): room for the whole cut bucket

struct FusedParams {
  const uint16_t* q;
  const uint8_t* k_data;
  const uint16_t* k_scales;
  const uint16_t* k_zp;  // asymmetric INT2 keys only: zero-points, shaped like k_scales
  const uint8_t* v_data;
  const uint16_t* v_scales;
  const int64_t* block_table;
  const int32_t* seq_lens;
  int B, H_q, H_kv, max_S, max_blocks;
  int g_act;  // query heads per kv-head (H_q / H_kv); the kernel's G is this rounded up to 1, 2, 4, 8 or 16
  int64_t num_slots;
  float attn_scale;
  int top_k;
  int L, n_splits, Kc;
  float* scores;  // optional (B, H_q, max_S)
  const float* scores_in;  // FS_STAGE_B: the scores (B, H_q, max_S)
  const float* stats_m;    // FS_STAGE_B merge, optional: softmax statistics (B, H_q) that replace the ones derived
  const float* stats_iz;   //   from the split partials (pre-correction terms alone: n_splits == 0, o_hat == NULL)
  int scores_only;         // FS_STAGE_A: stop after writing `scores`
  float* part_m;  // (B, H_q, NS)
  float* part_l;  // (B, H_q, NS)
  float* part_o;  // (B, H_q, NS, D)
  uint32_t* cand_key;  // (B, H_q, NS, Kc)
  int32_t* cand_idx;   // (B, H_q, NS, Kc)
  int32_t* cand_cnt;   // (B, H_q, NS)
  // two-stage merge (long contexts): `mg_parts` workgroups per row first reduce `mg_spp` consecutive
  // candidate lists each to the row's top_k among them; the final merge then reads those lists
  int mg_parts, mg_spp;
  uint32_t* key2;      // (B, H_q, mg_parts, top_k)
  int32_t* idx2;       // (B, H_q, mg_parts, top_k)
  int32_t* cnt2;       // (B, H_q, mg_parts)
  // merge outputs
  int64_t* topk_idx;
  int64_t* topk_slots;
  float* o_hat;
  float* o_old;
  float* W;
  float* softmax_m;
  float* softmax_inv_z;
  // optional merge epilogue: out = bf16(fma(W, o_new, o_hat) - o_old_unnorm), both (B, H_q, D) bf16
  const uint16_t* blend_o_new;
  uint16_t* blend_out;
  long long* phase_clock;  // optional: 10 s_memtime stamps per scan workgroup, 8 per merge workgroup (measurement aid)
};

// Phase-A constants of the INT3 path, built once per workgroup in LDS.
template <int NSET>
struct K3Prep {
  int8_t aop[NSET][16][4][2][16];  // A operand bytes: [set][row = 4*head + limb][k-block][MFMA][byte]
  int sq4[NSET * 4][2];            // 4 * sum of the fixed-point query over the scale group
  float qsc[NSET * 4][2];          // 2^(e-22) * attn_scale of the (head, group)
  float amax_w[NSET * 8];          // per 64-channel half row: |q| maximum, fixed-point sum, exponent
  int sum_w[NSET * 8];
  int exp_w[NSET * 8];
};

// Phase-A constants of the INT4 path: the int8-quantised query rows as MFMA A operand.  Row 4*head + kk holds
// the head's values of 32-channel block kk and zeros elsewhere, so one accumulator register per block.
template <int NSET>
struct QInt8F {
  int8_t aop[NSET][16][4][2][16];  // [set][row = 4*head + block][k-block][MFMA][byte]
  float qs[NSET * 4][4];           // query scale of (head, block)
  int sum8[NSET * 4][4];           // 8 * sum of the int8 query over the block (the codes carry an offset of 8)
};

// LDS carve-up shared by the kernel and its launcher.
//   sc     [G][L] fp32 scores of the split
//   sbase  [L/16] first slot of every 16-position page
//   aux    phase A: query constants (K3Prep / QInt8F); afterwards: selection histograms [G][SEG][256]
//   stage  one private staging area per wavefront: key rows in phase A, V rows + weight rows in phase B
// After phase B the staging area holds the sum of the wavefronts' P.V accumulators.
template <int SCHEME, int G, int NG>
struct ScanLds {
  // SCHEME = 10 * key bits + value bits (key digit 1: asymmetric INT2; 5: INT4 with the bf16 model): the key side (staging, query constants, phase A) and the value side
  // (staging, phase B) are chosen independently
  static constexpr bool K3 = (SCHEME / 10 == 3);
  static constexpr bool KA = (SCHEME / 10 == 1);        // INT2 keys with a zero-point per group (four levels)
  static constexpr bool K2 = (SCHEME / 10 == 2) || KA;  // four codes per byte
  static constexpr bool KB4 = (SCHEME / 10 == 5);       // INT4 keys scored with the bf16 model (any group size)
  static constexpr bool KLIMB = K2 || K3 || KB4;  // keys with the bf16 model: fixed-point query limbs against integer codes
  static constexpr bool V2 = (SCHEME % 10 == 2);
  static constexpr bool V3 = (SCHEME % 10 == 3);
  static_assert((KLIMB || SCHEME / 10 == 4) && (V2 || V3 || SCHEME % 10 == 4), "keys and values are INT2, INT3 or INT4");
  static constexpr int NSET = (G + 3) / 4;
  // wavefronts per workgroup: sixteen where the register budget allows (128 VGPRs at 1024 threads), else eight
  static constexpr int NW = (G <= 4) ? 16 : 8;
  static constexpr int NT = NW * 64;
  static constexpr int LMAX = NW * 256;  // four 64-position chunks per wavefront
  // emission segments per head (one wavefront each)
  static constexpr int SEG = (NW / G >= 4) ? 4 : ((NW / G >= 2) ? 2 : 1);
  static constexpr int KP = K2 ? 32 : (K3 ? 48 : 64);
  static constexpr int KROW = K2 ? 40 : (K3 ? 48 : 80);  // LDS pitch of a staged key row (INT2, INT4: padded against bank conflicts)
  static constexpr int VP = V2 ? 32 : (V3 ? 48 : 64);
  // LDS pitch of a staged V row.  INT2 rows (32 bytes) are padded so that 16 consecutive rows hit 16 distinct
  // bank pairs; INT4 rows (64 bytes) keep their pitch and swap their 16-byte quarters instead (quarter q of row r
  // sits at q ^ ((r >> 2) & 3)), which has the same effect without the padding bytes.  INT3 rows (48 bytes: 16
  // consecutive rows already hit distinct bank pairs) swap the 8-byte halves of every plane in rows 16..31 and
  // 48..63, so that the two 16-row groups one 8-byte read serves in a cycle do not meet either.
  static constexpr bool VSWZ = !(V2 || V3);
  static constexpr int VROW = (VSWZ || V3) ? VP : VP + 8;
  static constexpr int VST = 64 * VROW;
  static constexpr int WL = NG * NSET * 64 * 16;  // per (group, set): one 16-byte weight row per token
  static constexpr int KST = 64 * KROW;
  static constexpr int WAVE_STAGE = (VST + WL > KST) ? (VST + WL) : KST;
  // INT3 / symmetric INT2 keys: the scale word of a token is loaded once (lane = token) and turned into the floats
  // phase A multiplies by -- the group scales and the rounding coefficients -- in a table behind the staged key rows,
  // 8 * NG bytes per token, instead of by every one of the four lanes that handle the token's heads
  static constexpr int SCT = 8 * NG;
  static constexpr bool SPREP = (K3 || (K2 && !KA)) && (WAVE_STAGE >= KST + 64 * SCT);
  static constexpr int ACC_REGS = 8 + NG;                   // v4i accumulators per set: 8 channel tiles + NG weight sums
  // sum of the wavefronts' accumulators: one int per (set, accumulator register, component, lane), in the staging
  // area (dead after phase B), followed by one kilobyte per wavefront for the exact selection's histogram
  static constexpr int XACC = NSET * ACC_REGS * 4 * 64 * 4;
  static constexpr int PREP = KLIMB ? (int)sizeof(K3Prep<NSET>) : (int)sizeof(QInt8F<NSET>);
  // selection histograms: 32-bit counters, or (any INT4 side, where the staging areas are larger and LDS is
  // tighter) two 16-bit counters per word: a (head, segment) histogram counts at most LMAX / SEG <= 4096 positions
  static constexpr bool H16 = !(KLIMB && V2);
  static constexpr int HIST = G * SEG * 256 * (H16 ? 2 : 4);
  static constexpr int AUX = ((PREP > HIST ? PREP : HIST) + 15) & ~15;
  __host__ __device__ static constexpr int stage_bytes() { return NW * WAVE_STAGE; }
  static_assert(NW * WAVE_STAGE >= XACC + NW * 1024, "the staging area must hold the accumulator sums and the selection scratch");
  __host__ __device__ static constexpr size_t per_position() { return (size_t)G * 4; }
  __host__ __device__ static size_t aux_offset(int L) { return (per_position() * L + (size_t)(L / 16) * 4 + 15) & ~(size_t)15; }
  __host__ __device__ static size_t total(int L) {
    return aux_offset(L) + AUX + stage_bytes() + 64;
  }
};

__device__ inline float key_to_score(uint32_t key) {
  const uint32_t u = (key & 0x80000000u) ? (key & 0x7fffffffu) : ~key;
  return __builtin_bit_cast(float, u);
}

// Orders this wavefront's earlier LDS writes before its later LDS reads (the LDS pipe executes one
// wavefront's instructions in order; this only stops the compiler from moving them).
__device__ inline void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup barrier that orders LDS traffic only: unlike __syncthreads() it does not wait for global loads
// that are still in flight (the prefetched key / value rows), which no other wavefront consumes.
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// A copy the compiler cannot see through: the source register is dead afterwards, so a load issued next can
// write it directly instead of a temporary that is moved into place (after a wait) at the end of the block.
__device__ inline uint32_t reg_copy(uint32_t v) {
  uint32_t r;
  asm volatile("v_mov_b32 %0, %1" : "=v"(r) : "v"(v));
  return r;
}

// (hi * 256 + mid) * 256 + lo as two v_lshl_add_u32.  Written as plain shifts and adds the compiler re-associates
// it into two shifts and a three-operand add, one instruction more, in the innermost loop of the key stream; the
// empty statement makes the intermediate opaque.  (The instructions themselves stay the compiler's: it alone knows
// how long after an MFMA its results may be read.)
__device__ inline int join_limbs(int hi, int mid, int lo) {
  int t = (hi << 8) + mid;
  asm("" : "+v"(t));
  return (t << 8) + lo;
}

// s_setprio takes an immediate; `p` is a compile-time constant after unrolling
__device__ inline void set_wave_prio(int p) {
  if (p >= 3) __builtin_amdgcn_s_setprio(3);
  else if (p == 2) __builtin_amdgcn_s_setprio(2);
  else if (p == 1) __builtin_amdgcn_s_setprio(1);
  else __builtin_amdgcn_s_setprio(0);
}

__device__ inline float uniform_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// ---------------------------------------------------------------------------------------------------
template <int MODE, int SCHEME, int G, int NG>
__global__ __launch_bounds__((ScanLds<SCHEME, G, NG>::NT)) void fused_scan_kernel(FusedParams p) {
  using Lds = ScanLds<SCHEME, G, NG>;
  constexpr bool HAS_K = (MODE == FS_FULL || MODE == FS_STAGE_A);  // key stream and phase A
  constexpr bool HAS_V = (MODE == FS_FULL || MODE == FS_STAGE_B);  // value stream and the P.V part of phase B
  constexpr bool HAS_TOPK = (MODE != FS_STAGE_B);                  // histograms and phase C
  constexpr bool K3 = Lds::K3, KLIMB = Lds::KLIMB, KA = Lds::KA, KB4 = Lds::KB4;
  constexpr bool V2 = Lds::V2, V3 = Lds::V3;
  constexpr int NSET = Lds::NSET;
  constexpr int SEG = Lds::SEG;
  constexpr int KP = Lds::KP;
  constexpr int KROW = Lds::KROW;
  constexpr int VP = Lds::VP;
  constexpr int VROW = Lds::VROW;
  constexpr int VOFF = V2 ? 2 : (V3 ? 4 : 8);  // code offset of the V format
  constexpr int NTILE = 8;          // 8 MFMA column tiles of 16 channels
  constexpr int AR = Lds::ACC_REGS;
  constexpr float LOG2E = 1.44269504088896340736f;
  constexpr int NW = Lds::NW, NT = Lds::NT;
  constexpr int MAXIT = Lds::LMAX / 64 / NW;  // chunks per wavefront

  extern __shared__ __align__(16) uint8_t smem[];
  const int L = p.L;
  float* sc = reinterpret_cast<float*>(smem);                     // [G][L]
  int* sbase = reinterpret_cast<int*>(smem + (size_t)G * L * 4);  // [L/16] first slot of each page
  uint8_t* aux = smem + Lds::aux_offset(L);
  uint8_t* stage = aux + Lds::AUX;
  int* hist = reinterpret_cast<int*>(aux);  // [G][SEG][256], valid after phase A
  __shared__ float red_f[NW][2 * G];
  __shared__ uint32_t vmax_sh[NW][2];
  __shared__ float m_sh[G], bin_a_sh[G], bin_b_sh[G], lsum_sh[NW][G];
  __shared__ int e_sh[2];
  // rounding coefficients 256 * (bf16(c s) - c s) / s for s = 1 + m/128 (INT3: c = 3; INT4, bf16 model: c = 3, 5, 7).
  // Static, so that a look-up's address is the index plus a constant the instruction carries.
  __shared__ float eps_sh[KB4 ? 3 : 1][128];
  __shared__ unsigned long long tmax_sh;
  if (threadIdx.x == 0) tmax_sh = 0ull;

  const int split = blockIdx.x, hkv = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: keeps wave-derived addresses in SGPRs
  const int S = max(0, min(p.max_S, p.seq_lens[b]));
  const int s0 = split * L;
  const int s1 = min(s0 + L, S);
  const int n = max(0, s1 - s0);
  const int s_cover = min(s0 + L, p.max_S);
  const int n_cover = max(0, s_cover - s0);
  const int64_t* bt = p.block_table + (size_t)b * p.max_blocks;
  // GA query heads belong to this kv-head; the template's G may be larger (the next of 1, 2, 4, 8, 16): the heads
  // past GA are zero query rows whose arithmetic runs along and whose results are never stored
  const int GA = p.g_act;
  const size_t head0 = (size_t)b * p.H_q + (size_t)hkv * GA;
  const size_t part_base = head0 * p.n_splits + split;  // + h * n_splits
  const uint8_t* kbase = p.k_data + (size_t)hkv * p.num_slots * KP;
  const uint8_t* vbase = p.v_data + (size_t)hkv * p.num_slots * VP;
  const uint8_t* vsbase = reinterpret_cast<const uint8_t*>(p.v_scales + (size_t)hkv * p.num_slots * NG);

  long long* clk = (kDebugHooks && p.phase_clock) ? p.phase_clock + (((size_t)b * p.H_kv + hkv) * p.n_splits + split) * 10 : nullptr;
  if (clk && tid == 0) clk[0] = JF_CLK();

  // The page-table entry and the query elements of this thread do not depend on the sequence length: they
  // are requested first, so their latency runs in parallel with the load of seq_lens[b] instead of after it.
  const int nch_cover = (n_cover + 63) >> 6;
  // (both unconditional, on clamped indices: under a condition the compiler waits for each load inside its branch,
  // one cold miss after the other)
  const int64_t bt_mine = bt[min((s0 >> 4) + tid, p.max_blocks - 1)];  // LMAX / 16 <= NT: one entry per thread covers the split
  constexpr int QN = NSET * 4 * D;               // elements of the padded query block (whole head sets)
  constexpr int QPT = (QN + NT - 1) / NT;
  uint16_t qraw[QPT];
#pragma unroll
  for (int it = 0; it < QPT; ++it) qraw[it] = HAS_K ? p.q[head0 * D + min(it * NT + tid, GA * D - 1)] : (uint16_t)0;
  auto q_elem = [&](int it) -> float { return (it * NT + tid < GA * D) ? bf16_to_f32(qraw[it]) : 0.f; };

  if (n == 0) {  // nothing valid in this split: padding scores, empty partials
    if (p.scores)
      for (int i = tid; i < GA * n_cover; i += NT)
        p.scores[(head0 + i / n_cover) * (size_t)p.max_S + s0 + (i % n_cover)] = -INFINITY;
    if constexpr (MODE == FS_STAGE_A)
      if (p.scores_only) return;
    for (int i = tid; i < GA * D; i += NT) p.part_o[(part_base + (size_t)(i / D) * p.n_splits) * D + (i % D)] = 0.f;
    if (tid < GA) {
      p.part_m[part_base + (size_t)tid * p.n_splits] = -INFINITY;
      p.part_l[part_base + (size_t)tid * p.n_splits] = 0.f;
      p.cand_cnt[part_base + (size_t)tid * p.n_splits] = 0;
    }
    for (int i = tid; i < GA * p.Kc; i += NT)  // unused candidate slots hold key 0 (no score maps to it)
      p.cand_key[(part_base + (size_t)(i / p.Kc) * p.n_splits) * p.Kc + (i % p.Kc)] = 0u;
    return;
  }

  // Page table of the split: one entry per 16 positions of every 64-token chunk that is touched.  Table
  // entries past the last valid position may hold anything: those pages read slot 0 instead, so every row
  // address formed below is in bounds (those rows' scores are masked to -inf, their softmax weights are
  // exactly zero).
  const int nch = (n + 63) >> 6;
  if (tid < nch_cover * 4) sbase[tid] = (tid <= ((n - 1) >> 4)) ? (int)(bt_mine * BS) : 0;
  lds_barrier();

  // ---- key stream, set-up.  A chunk is 64 consecutive positions = 4 pages; its rows are fetched with
  // 16-byte loads whose lane addresses are consecutive inside a page, staged in this wavefront's LDS area
  // in position order, and read back in the layout the arithmetic wants.
  uint8_t* kst = stage + wave * Lds::WAVE_STAGE;
  constexpr int KLD = KP / 16;  // 16-byte loads per lane and chunk
  uint32_t kl_page[KLD], kl_off[KLD], kl_lds[KLD];
#pragma unroll
  for (int i = 0; i < KLD; ++i) {
    const int o = 1024 * i + 16 * lane;  // byte offset inside the chunk's 64 rows
    kl_page[i] = (uint32_t)(o / (16 * KP));
    kl_off[i] = (uint32_t)(o % (16 * KP));
    kl_lds[i] = (uint32_t)((o / KP) * KROW + (o % KP));
  }
  const uint8_t* ksb = reinterpret_cast<const uint8_t*>(p.k_scales + (size_t)hkv * p.num_slots * (KLIMB ? NG : 1));
  const uint8_t* kzb = KA ? reinterpret_cast<const uint8_t*>(p.k_zp + (size_t)hkv * p.num_slots * NG) : nullptr;
  constexpr bool SPREP = HAS_K && Lds::SPREP;
  struct KBuf {
    v4u r[KLD];
    uint32_t s[SPREP ? 1 : 4];   // scale words: of the lane's token (SPREP), or of token t16 of each of the four pages
    uint32_t z[KA ? 4 : 1];  // zero-points of the asymmetric keys, packed like the scales
  };
  const int t16 = lane & 15, lg = lane >> 4;
  auto issue_k = [&](int chunk) -> KBuf {
    KBuf kbuf;
    constexpr int KNG = KLIMB ? NG : 1;  // key scales per row
    // (the scales first: they are copied out of the buffer one chunk earlier than the rows are, and loads return in order)
    if constexpr (SPREP) {
      const int tl = chunk * 64 + lane;
      const uint32_t slot = (uint32_t)(sbase[tl >> 4] + (tl & 15));
      if (KNG == 2) kbuf.s[0] = *reinterpret_cast<const uint32_t*>(ksb + (size_t)(slot * 4u));
      else kbuf.s[0] = (uint32_t) * reinterpret_cast<const uint16_t*>(ksb + (size_t)(slot * 2u));
    }
#pragma unroll
    for (int j = 0; j < (SPREP ? 0 : 4); ++j) {
      const int sb = __builtin_amdgcn_readfirstlane(sbase[chunk * 4 + j]);  // first slot of the page (uniform)
      const uint8_t* srow = ksb + (size_t)sb * (KNG * 2) + t16 * (KNG * 2);
      if (KNG == 2) kbuf.s[SPREP ? 0 : j] = *reinterpret_cast<const uint32_t*>(srow);
      else kbuf.s[SPREP ? 0 : j] = *reinterpret_cast<const uint16_t*>(srow);
      if constexpr (KA) {
        const uint8_t* zrow = kzb + (size_t)sb * (KNG * 2) + t16 * (KNG * 2);
        if (KNG == 2) kbuf.z[j] = *reinterpret_cast<const uint32_t*>(zrow);
        else kbuf.z[j] = *reinterpret_cast<const uint16_t*>(zrow);
      }
    }
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const uint32_t sb = (uint32_t)sbase[chunk * 4 + kl_page[i]];
      // (streaming hint: a key row is read exactly once; measured 0.6 - 2 us per launch against plain loads.  The
      // value rows keep the default policy: the merge kernel gathers the winners' rows again.)
      kbuf.r[i] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(kbase + (size_t)(sb * (uint32_t)KP + kl_off[i])));
    }
    return kbuf;
  };
  auto stash_k = [&](const KBuf& kbuf) {
#pragma unroll
    for (int i = 0; i < KLD; ++i) *reinterpret_cast<v4u*>(kst + kl_lds[i]) = kbuf.r[i];
  };
  // first two chunks of this wavefront and the V scales of the split start now, before the query set-up
  KBuf Ka = {}, Kb = {};
  // (every wavefront requests, on a clamped chunk if it has none of its own: the number of loads in flight at each
  // later wait is then the same on every path, and the compiler's waits leave the younger loads in flight)
  if constexpr (HAS_K) Ka = issue_k(min(wave, nch_cover - 1));
  constexpr int VSPT = Lds::LMAX / NT;
  // (positions past the split's end read the scale of its last row again: straight-line code whose loads leave
  // together, and the only use of these values is their maximum)
  uint32_t vsw[VSPT], vs_slot[VSPT];
#pragma unroll
  for (int i = 0; i < VSPT; ++i) {
    const int t = min(tid + i * NT, n - 1);
    vs_slot[i] = HAS_V ? (uint32_t)(sbase[t >> 4] + (t & 15)) : 0u;
  }
#pragma unroll
  for (int i = 0; i < VSPT; ++i) {
    vsw[i] = 0u;
    if constexpr (HAS_V) {
      if (NG == 2) vsw[i] = *reinterpret_cast<const uint32_t*>(vsbase + (size_t)(vs_slot[i] * 4u));
      else vsw[i] = (uint32_t) * reinterpret_cast<const uint16_t*>(vsbase + (size_t)(vs_slot[i] * 2u));
    }
  }
  if constexpr (!HAS_K) {
    // the scores are an input: no query constants
  } else if constexpr (KLIMB) {
    // Query rows -> 23-bit fixed point per (head, scale group), three balanced int8 limbs, written in the
    // byte order of the MFMA A operand.  One element per thread; group statistics by wavefront reductions.
    K3Prep<NSET>* prep = reinterpret_cast<K3Prep<NSET>*>(aux);
    // (the rounding table is built by two wavefronts that have no query rows to prepare, where there are such)
    constexpr int EPS_T0 = (QN / 64 <= NW - 2) ? NT - 128 : 0;
    if ((K3 || KB4) && tid >= EPS_T0 && tid < EPS_T0 + 128) {
      const int m = tid - EPS_T0;
      const float sm = 1.0f + (float)m * (1.0f / 128.0f);
#pragma unroll
      for (int i = 0; i < (KB4 ? 3 : 1); ++i) {
        const float t = (float)(3 + 2 * i) * sm;  // 3 s, 5 s, 7 s: exact in fp32
        eps_sh[i][m] = 256.0f * ((bf16_to_f32(f32_to_bf16(t)) - t) / sm);
      }
    }
    // stores the three limbs of element (h, d) in the byte order of the MFMA A operand
    auto put_limbs = [&](int h, int d, int qf) {
      const int l0 = (int)(int8_t)(qf & 255);
      const int r1 = (qf - l0) >> 8;
      const int l1 = (int)(int8_t)(r1 & 255);
      const int l2 = (r1 - l1) >> 8;
      const int set = h >> 2, hh = h & 3;
      // A lane of phase A spreads the 32 channels 32*lg .. 32*lg+31 of its token into two 16-byte operands u = 0, 1
      // (dword e, byte b).  INT3 (plane spread): channel 8b + 4u + e; INT2 (four codes per byte): channel 16u + 4b + e;
      // INT4 (nibble spread of the lane's four dwords): channel 16u + 8(e >> 1) + 2b + (e & 1).
      // With two scale groups MFMA g covers group g only (see the lane swap in phase A).
      const int u = K3 ? ((d >> 2) & 1) : ((d >> 4) & 1);
      const int mi = (NG == 2) ? (d >> 6) : u;
      const int kb = (NG == 2) ? (((d >> 5) & 1) + 2 * u) : (d >> 5);
      const int by = KB4 ? (4 * (2 * ((d >> 3) & 1) + (d & 1)) + ((d >> 1) & 3))
                         : (4 * (d & 3) + (K3 ? ((d >> 3) & 3) : ((d >> 2) & 3)));
      prep->aop[set][4 * hh + 0][kb][mi][by] = (int8_t)l0;
      prep->aop[set][4 * hh + 1][kb][mi][by] = (int8_t)l1;
      prep->aop[set][4 * hh + 2][kb][mi][by] = (int8_t)l2;
      prep->aop[set][4 * hh + 3][kb][mi][by] = 0;
    };
    constexpr int CODE_OFF4 = KB4 ? 8 : (K3 ? 4 : 2);  // the codes are used unsigned: offset 8 (INT4), 4 (INT3) or 2 (INT2)
    if constexpr (NG == 2) {
      // a wavefront's 64 elements are one scale group of one head: its statistics never leave the wavefront
#pragma unroll
      for (int it = 0; it < QPT; ++it) {
        const int c = it * NW + wave;  // 64-channel half row of this wavefront
        if (c * 64 >= QN) continue;    // uniform per wavefront
        const int i = it * NT + tid, h = i >> 7, d = i & 127;
        const float x = q_elem(it);
        const float amax = wave_max(fabsf(x));
        int e = 0;
        if (amax > 0.f && isfinite(amax)) (void)frexpf(amax, &e);  // amax = f * 2^e, f in [0.5, 1)
        const int qf = (int)rintf(ldexpf(x, 22 - e));
        const int sum = wave_sum_i(qf);
        put_limbs(h, d, qf);
        if (lane == 0) {
          prep->sq4[h][c & 1] = CODE_OFF4 * sum;
          prep->qsc[h][c & 1] = ldexpf(p.attn_scale, e - 22);
        }
      }
    } else {
#pragma unroll
      for (int it = 0; it < QPT; ++it) {
        const int c = it * NW + wave;  // 64-channel half row of this wavefront
        if (c * 64 < QN) {             // uniform per wavefront
          const float am = wave_max(fabsf(q_elem(it)));
          if (lane == 0) prep->amax_w[c] = am;
        }
      }
      lds_barrier();
#pragma unroll
      for (int it = 0; it < QPT; ++it) {
        const int i = it * NT + tid, h = i >> 7, d = i & 127;
        const float x = q_elem(it);
        const int c = it * NW + wave;
        if (c * 64 >= QN) continue;
        const float amax = fmaxf(prep->amax_w[c & ~1], prep->amax_w[c | 1]);
        int e = 0;
        if (amax > 0.f && isfinite(amax)) (void)frexpf(amax, &e);  // amax = f * 2^e, f in [0.5, 1)
        const int qf = (int)rintf(ldexpf(x, 22 - e));
        const int s = wave_sum_i(qf);
        if (lane == 0) {
          prep->sum_w[c] = s;
          prep->exp_w[c] = e;
        }
        put_limbs(h, d, qf);
      }
      lds_barrier();
      if (tid < NSET * 4) {
        const int h = tid;
        prep->sq4[h][0] = CODE_OFF4 * (prep->sum_w[2 * h] + prep->sum_w[2 * h + 1]);
        prep->qsc[h][0] = ldexpf(p.attn_scale, prep->exp_w[2 * h] - 22);
      }
    }
  } else {
    // int8 quantisation of the query rows per 32 channels (int8tc_qk_scores.cu:250-290), one element per thread;
    // heads past G are zero rows
    QInt8F<NSET>* qsh = reinterpret_cast<QInt8F<NSET>*>(aux);
#pragma unroll
    for (int it = 0; it < QPT; ++it) {
      const int i = it * NT + tid;
      if (i < QN) {  // uniform per wavefront: QN is a multiple of 64
        const int h = i >> 7, d = i & 127, kk = d >> 5;
        const float x = q_elem(it);
        float a = fabsf(x);
#pragma unroll
        for (int off = 16; off >= 1; off >>= 1) a = fmaxf(a, __shfl_xor(a, off));
        const float sq = fmaxf(a / 127.0f, 1e-12f);
        const float inv = 1.0f / sq;
        const int v = max(-128, min(127, (int)rintf(x * inv)));
        int sv = v;
#pragma unroll
        for (int off = 16; off >= 1; off >>= 1) sv += __shfl_xor(sv, off);
        // channel d sits in MFMA d>>6, k-block (d>>4)&3; inside the k-block's 16 bytes the nibble spread of two
        // packed dwords yields: even channels of bytes 0-3, odd channels of bytes 0-3, then the same for bytes 4-7
        const int set = h >> 2, hh = h & 3, mi = d >> 6, kb = (d >> 4) & 3;
        const int j2 = (d & 15) >> 1, odd = d & 1;
        const int by = (j2 >> 2) * 8 + odd * 4 + (j2 & 3);
#pragma unroll
        for (int r = 0; r < 4; ++r) qsh->aop[set][4 * hh + r][kb][mi][by] = (r == kk) ? (int8_t)v : (int8_t)0;
        if ((lane & 31) == 0) {
          qsh->qs[h][kk] = sq;
          qsh->sum8[h][kk] = 8 * sv;
        }
      }
    }
  }
  lds_barrier();
  if constexpr (HAS_K) Kb = issue_k(min(wave + NW, nch_cover - 1));
  if (clk && tid == 0) clk[7] = JF_CLK();

  // ---- V stream, set-up (same scheme as the key stream)
  uint8_t* vst = stage + wave * Lds::WAVE_STAGE;  // [64][VROW], this wavefront only
  uint8_t* wl = vst + Lds::VST;                   // [NG][NSET][64 tokens][16]
  constexpr int VLD = VP / 16;
  uint32_t vl_page[VLD], vl_off[VLD], vl_lds[VLD];
#pragma unroll
  for (int i = 0; i < VLD; ++i) {
    const int o = 1024 * i + 16 * lane;
    vl_page[i] = (uint32_t)(o / (16 * VP));
    vl_off[i] = (uint32_t)(o % (16 * VP));
    const int row = o / VP, q16 = (o % VP) / 16;
    vl_lds[i] = Lds::VSWZ ? (uint32_t)(row * VROW + ((q16 ^ ((row >> 2) & 3)) * 16))
                          : (uint32_t)(row * VROW + (o % VP) + (V3 ? 8 * ((row >> 4) & 1) : 0));  // (INT3: first half's place)
  }
  // (the V scales of a chunk are not fetched again: position chunk * 64 + lane of step `it` is tid + it * NT, whose
  // scale word this thread has held in vsw[it] since the set-up)
  struct VBuf {
    v4u r[VLD];
  };
  auto issue_v = [&](int chunk) -> VBuf {
    VBuf vbuf;
#pragma unroll
    for (int i = 0; i < VLD; ++i) {
      const uint32_t sb = (uint32_t)sbase[chunk * 4 + vl_page[i]];
      vbuf.r[i] = *reinterpret_cast<const v4u*>(vbase + (size_t)(sb * (uint32_t)VP + vl_off[i]));
    }
    return vbuf;
  };
  // the first two V chunks are requested while the last key chunks are being worked on
  VBuf Va = {}, Vb = {};
  bool va_requested = false, vb_requested = false;  // (uniform per wavefront)
  auto prefetch_v = [&](int it) {
    if constexpr (MODE == FS_FULL) {
      if (it == MAXIT - 2) {
        Va = issue_v(min(wave, nch - 1));
        va_requested = true;
      }
      if (it == MAXIT - 1) {
        Vb = issue_v(min(wave + NW, nch - 1));
        vb_requested = true;
      }
    }
  };
  if constexpr (MODE == FS_STAGE_B) {  // nothing to wait for: the value stream starts at once
    Va = issue_v(min(wave, nch - 1));
    Vb = issue_v(min(wave + NW, nch - 1));
  }


  // A chunk the sequence ends in (0 < n_local < 64 valid rows; uniform): the staged rows past the end and their
  // scale words become copies of the last valid row, so the stream's arithmetic runs without a validity select per
  // score (a copy of a valid score changes neither extremum), and `mask_tail` afterwards stores -inf over what those
  // positions produced.  A chunk past the end (n_local <= 0) is not worked through at all.
  auto clone_last_row = [&](int n_local, uint32_t (&Sx)[4], uint32_t (&Zx)[4]) {
    const int last = n_local - 1, jl = last >> 4;
    if constexpr (SPREP) {  // one scale word per lane (= token): Sx[0]
      const uint32_t sl = (uint32_t)__builtin_amdgcn_readlane((int)Sx[0], last);
      Sx[0] = (lane >= n_local) ? sl : Sx[0];
    } else {
      uint32_t sl = Sx[0], zl = Zx[0];
#pragma unroll
      for (int j = 1; j < 4; ++j) {
        sl = (jl == j) ? Sx[j] : sl;
        zl = (jl == j) ? Zx[j] : zl;
      }
      sl = (uint32_t)__builtin_amdgcn_readlane((int)sl, last & 15);
      zl = (uint32_t)__builtin_amdgcn_readlane((int)zl, last & 15);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool past = 16 * j + (lane & 15) >= n_local;
        Sx[j] = past ? sl : Sx[j];
        Zx[j] = past ? zl : Zx[j];
      }
    }
    constexpr int RDW = KP / 4;  // dwords per staged row
    const uint8_t* src = kst + last * KROW;
    for (int i = lane; i < (64 - n_local) * RDW; i += 64) {
      const int r = n_local + i / RDW, dw = i % RDW;
      *reinterpret_cast<uint32_t*>(kst + r * KROW + 4 * dw) = *reinterpret_cast<const uint32_t*>(src + 4 * dw);
    }
    wave_lds_fence();
  };
  auto mask_tail = [&](int chunk, int n_local) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int tl = 16 * j + (lane & 15);
      if (tl >= n_local) {
#pragma unroll
        for (int set = 0; set < NSET; ++set) {
          const int h = set * 4 + (lane >> 4);
          if ((G % 4 == 0) || h < G) sc[h * L + chunk * 64 + tl] = -INFINITY;
        }
      }
    }
  };

  // ------------------------------------------------------------------ phase A
  if constexpr (!HAS_K) {
    // the split's scores come from the caller's (B, H_q, max_S) tensor: -> LDS, running maximum per head;
    // positions past the sequence (and the rest of the last chunk) become -inf
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const float* srow = p.scores_in + (head0 + min(h, GA - 1)) * (size_t)p.max_S + s0;  // (past GA: a copy, unused)
      float mx = -INFINITY, mn = INFINITY;
      for (int t = tid; t < nch * 64; t += NT) {
        const float v = (t < n) ? srow[t] : -INFINITY;
        sc[h * L + t] = v;
        mx = fmaxf(mx, v);
        mn = fminf(mn, (t < n) ? v : INFINITY);
      }
      mx = wave_max(mx);
      mn = -wave_max(-mn);
      if (lane == 0) {
        red_f[wave][h] = mx;
        red_f[wave][G + h] = mn;  // (the minimum shapes the selection buckets)
      }
    }
  } else if constexpr (KLIMB) {
    // INT2 keys: the same scheme without the second contraction: (code - 2) * scale is exact in bf16 for every code,
    // so the reference's rounding (int2_qk_scores.cu:66-79) changes nothing; the codes sit four to a byte, MSB first.
    // INT3 keys on v_mfma_i32_16x16x64_i8.  The bf16 query row is held exactly as a 23-bit fixed-point number
    // per (head, scale group), split into three balanced int8 limbs that sit in different A-operand rows
    // (row = 4*head + limb), so one MFMA yields the three integer partial sums of a (token, head) in the
    // registers of one lane.  K codes are spread from the three byte planes to one byte per code with
    // shift/mask on whole dwords (4 codes per VALU operation) and used unsigned; the -4 offset is removed with
    // the per-row constant 4*sum(q).  Lane (token, k-block lg) holds channels 32*lg .. 32*lg+31, i.e. lanes
    // 0-31 hold scale group 0 and lanes 32-63 group 1; one v_permlane32_swap per dword regroups them so that
    // each MFMA contracts over exactly one scale group.  The reference rounds every dequantised key to bf16
    // (int3_qk_scores.cu:90-99); only codes +-3 are inexact, so that rounding is reproduced by a second
    // contraction with the indicator (+1 for code 7, -1 for code 1, byte LUT through v_perm_b32) weighted by
    // eps = (bf16(3s) - 3s) / s, which depends on the 7 mantissa bits of the scale only (128-entry table).
    const K3Prep<NSET>* prep = reinterpret_cast<const K3Prep<NSET>*>(aux);
    v4i Aop[NSET][2];
    int sq4[NSET][NG];
    float qsc[NSET][NG];
#pragma unroll
    for (int set = 0; set < NSET; ++set) {
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) Aop[set][mi] = *reinterpret_cast<const v4i*>(&prep->aop[set][t16][lg][mi][0]);
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        sq4[set][g] = prep->sq4[set * 4 + lg][g];
        qsc[set][g] = prep->qsc[set * 4 + lg][g];
      }
    }
    // this lane's plane dwords (INT2: its 8 bytes, INT4: its 16 bytes) of token t16 of a page
    const uint8_t* krd = kst + t16 * KROW + lg * (K3 ? 4 : (KB4 ? 16 : 8));
    float mxl[NSET], mnl[NSET];
#pragma unroll
    for (int set = 0; set < NSET; ++set) {
      mxl[set] = -INFINITY;
      mnl[set] = INFINITY;
    }
    float sumq[NSET][NG];  // fixed-point sum of the query over the scale group (asymmetric keys)
#pragma unroll
    for (int set = 0; set < NSET; ++set)
#pragma unroll
      for (int g = 0; g < NG; ++g) sumq[set][g] = (float)(sq4[set][g] / 2);
    (void)sumq;
    // (the offset term -sq4 of the limb-0 sum enters as the accumulator's initial value: exact, and one subtraction
    // per token, head and group less)
    v4i Cin[NSET][NG];
#pragma unroll
    for (int set = 0; set < NSET; ++set)
#pragma unroll
      for (int g = 0; g < NG; ++g) Cin[set][g] = (v4i){-sq4[set][g], 0, 0, 0};
    auto body = [&](int chunk, const uint32_t (&Sx)[4], const uint32_t (&Zx)[4]) {
      (void)Zx;
      // all LDS reads of the chunk first (plane dwords of the four pages, rounding coefficients), then arithmetic
      uint32_t Pj[4][KB4 ? 4 : 3];
      float sgj[4][NG], egj[4][NG];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint8_t* rp = krd + j * 16 * KROW;
        if constexpr (K3) {
          Pj[j][0] = *reinterpret_cast<const uint32_t*>(rp);
          Pj[j][1] = *reinterpret_cast<const uint32_t*>(rp + 16);
          Pj[j][2] = *reinterpret_cast<const uint32_t*>(rp + 32);
        } else if constexpr (KB4) {
          const v4u x = *reinterpret_cast<const v4u*>(rp);
#pragma unroll
          for (int i = 0; i < 4; ++i) Pj[j][KB4 ? i : 0] = x[i];
        } else {
          const v2u x = *reinterpret_cast<const v2u*>(rp);
          Pj[j][0] = x[0];
          Pj[j][1] = x[1];
          Pj[j][2] = 0u;
        }
        if constexpr (SPREP) {  // the token's entry of the table the wavefront has just written
          const uint8_t* sp = kst + Lds::KST + (16 * j + t16) * Lds::SCT;
          if (NG == 2) {
            const v4f x = *reinterpret_cast<const v4f*>(sp);
            sgj[j][0] = x[0];
            sgj[j][NG - 1] = x[1];
            egj[j][0] = x[2];
            egj[j][NG - 1] = x[3];
          } else {
            const v2f x = *reinterpret_cast<const v2f*>(sp);
            sgj[j][0] = x[0];
            egj[j][0] = x[1];
          }
        } else {
          const uint32_t sw = Sx[j];
          sgj[j][0] = bf16_to_f32((uint16_t)(sw & 0xffffu));
          egj[j][0] = K3 ? eps_sh[0][sw & 0x7fu] : 0.f;  // (INT4: three coefficients, read where they are used)
          if (NG == 2) {
            sgj[j][NG - 1] = bf16_to_f32((uint16_t)(sw >> 16));
            egj[j][NG - 1] = K3 ? eps_sh[0][(sw >> 16) & 0x7fu] : 0.f;
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t P0 = Pj[j][0], P1 = Pj[j][1], P2 = Pj[j][2];
        v4i Bc[2], Br[2];
        if constexpr (KB4) {  // two codes per byte, the even channel in the high nibble
          const uint32_t P3 = Pj[j][KB4 ? 3 : 0];
          Bc[0] = (v4i){(int)((P0 >> 4) & 0x0f0f0f0fu), (int)(P0 & 0x0f0f0f0fu), (int)((P1 >> 4) & 0x0f0f0f0fu), (int)(P1 & 0x0f0f0f0fu)};
          Bc[1] = (v4i){(int)((P2 >> 4) & 0x0f0f0f0fu), (int)(P2 & 0x0f0f0f0fu), (int)((P3 >> 4) & 0x0f0f0f0fu), (int)(P3 & 0x0f0f0f0fu)};
        } else if constexpr (K3) {
          Bc[0][0] = (int)((P0 >> 5) & 0x07070707u);
          Bc[0][1] = (int)((P0 >> 2) & 0x07070707u);
          Bc[0][2] = (int)(((P0 << 1) & 0x06060606u) | ((P1 >> 7) & 0x01010101u));
          Bc[0][3] = (int)((P1 >> 4) & 0x07070707u);
          Bc[1][0] = (int)((P1 >> 1) & 0x07070707u);
          Bc[1][1] = (int)(((P1 << 2) & 0x04040404u) | ((P2 >> 6) & 0x03030303u));
          Bc[1][2] = (int)((P2 >> 3) & 0x07070707u);
          Bc[1][3] = (int)(P2 & 0x07070707u);
        } else {  // four codes per byte, MSB first: dword e of operand u holds code e of each of the four bytes
          (void)P2;
          Bc[0] = (v4i){(int)((P0 >> 6) & 0x03030303u), (int)((P0 >> 4) & 0x03030303u), (int)((P0 >> 2) & 0x03030303u), (int)(P0 & 0x03030303u)};
          Bc[1] = (v4i){(int)((P1 >> 6) & 0x03030303u), (int)((P1 >> 4) & 0x03030303u), (int)((P1 >> 2) & 0x03030303u), (int)(P1 & 0x03030303u)};
        }
        if (NG == 2) {
          // Bc[0] <- lanes 0-31 keep their first half, lanes 32-63 receive the second half of lane-32;
          // Bc[1] <- lanes 0-31 receive the first half of lane+32, lanes 32-63 keep their second half
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const auto sw = __builtin_amdgcn_permlane32_swap((uint32_t)Bc[0][e], (uint32_t)Bc[1][e], false, false);
            Bc[0][e] = (int)sw[0];
            Bc[1][e] = (int)sw[1];
          }
        }
        if constexpr (KB4) {
          // khat = bf16((u - 8) s) for the unsigned nibble u: exact for |u - 8| in {0, 1, 2, 4, 8}; for 3, 5, 7 (and 6 =
          // 2 * 3) the rounding is eps_c(s) * s with the sign of the code, eps_c a function of the scale's mantissa
          // alone.  So next to the code contraction there are three with the signed indicators r3 = [c = +-3] +
          // 2 [c = +-6], r5 = [c = +-5], r7 = [c = +-7], made by byte look-ups: one table for the codes >= 0 (u >= 8,
          // selector u - 8 = c) and one for the codes < 0 (selector u = c + 8), chosen per byte by bit 3 of u.
          const int tok = chunk * 64 + 16 * j + t16;
          float acc_s[NSET][NG];
#pragma unroll
          for (int set = 0; set < NSET; ++set)
#pragma unroll
            for (int g = 0; g < NG; ++g) {
              const v4i zero = {0, 0, 0, 0};
              v4i Dc;
              if (NG == 2) {
                Dc = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], Bc[g], Cin[set][g], 0, 0, 0);
              } else {
                Dc = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][0], Bc[0], Cin[set][0], 0, 0, 0);
                Dc = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][1], Bc[1], Dc, 0, 0, 0);
              }
              (void)zero;
              acc_s[set][g] = (float)join_limbs(Dc[2], Dc[1], Dc[0]);
            }
#pragma unroll
          for (int c = 0; c < 3; ++c) {  // c = 0, 1, 2: the indicators of +-3 (and +-6), +-5, +-7
            const uint32_t pos_hi = (c == 0) ? 0x00020000u : ((c == 1) ? 0x00000100u : 0x01000000u);  // selectors 4..7
            const uint32_t pos_lo = (c == 0) ? 0x01000000u : 0u;                                       // selectors 0..3
            const uint32_t neg_hi = (c == 0) ? 0x0000ff00u : 0u;
            const uint32_t neg_lo = (c == 0) ? 0x00fe0000u : ((c == 1) ? 0xff000000u : 0x0000ff00u);
            v4i Bi[2];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const uint32_t x = (uint32_t)Bc[u][e], sel = x & 0x07070707u;
                const uint32_t t = (x >> 3) & 0x01010101u, hm = (t << 8) - t;  // 0xff in the bytes whose code is >= 0
                const uint32_t rp_ = __builtin_amdgcn_perm(pos_hi, pos_lo, sel), rn_ = __builtin_amdgcn_perm(neg_hi, neg_lo, sel);
                Bi[u][e] = (int)((rp_ & hm) | (rn_ & ~hm));
              }
#pragma unroll
            for (int set = 0; set < NSET; ++set)
#pragma unroll
              for (int g = 0; g < NG; ++g) {
                const v4i zero = {0, 0, 0, 0};
                v4i Dr;
                if (NG == 2) {
                  Dr = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], Bi[g], zero, 0, 0, 0);
                } else {
                  Dr = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][0], Bi[0], zero, 0, 0, 0);
                  Dr = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][1], Bi[1], Dr, 0, 0, 0);
                }
                const float ec = eps_sh[c][((g == 0) ? Sx[j] : (Sx[j] >> 16)) & 0x7fu];
                acc_s[set][g] = __builtin_fmaf(ec, (float)((Dr[2] << 8) + Dr[1]), acc_s[set][g]);
              }
          }
#pragma unroll
          for (int set = 0; set < NSET; ++set) {
            float score = 0.f;
#pragma unroll
            for (int g = 0; g < NG; ++g) score = __builtin_fmaf(acc_s[set][g], sgj[j][g] * qsc[set][g], score);
            const int h = set * 4 + lg;
            if ((G % 4 == 0) || h < G) {
              sc[h * L + tok] = score;
              mxl[set] = fmaxf(mxl[set], score);
              mnl[set] = fminf(mnl[set], score);
            }
          }
          continue;
        }
        if constexpr (KA) {
          // Four levels per group: khat(code) = bf16(fma(code - 2, scale, zp)) (int2_qk_scores.cu:66-79) is any function
          // of the code's two bits b1 b0, so with the indicator bytes x0 = b0, x1 = b1, x01 = b0 & b1
          //   khat = v0 + (v1 - v0) x0 + (v2 - v0) x1 + (v3 - v2 - v1 + v0) x01,   v_c = khat(c),
          // and q . khat is four exact fixed-point sums (the query's own, and the three contractions with the
          // indicators) combined in fp32 with coefficients that are exact differences of bf16 values.
          v4i X0[2], X1[2], X01[2];
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const uint32_t c = (uint32_t)Bc[u][e];
              const uint32_t b0 = c & 0x01010101u, b1 = (c >> 1) & 0x01010101u;
              X0[u][e] = (int)b0;
              X1[u][e] = (int)b1;
              X01[u][e] = (int)(b0 & b1);
            }
          float coef[NG][4];
#pragma unroll
          for (int g = 0; g < NG; ++g) {
            const float sc_g = sgj[j][g];
            const float zp_g = bf16_to_f32((uint16_t)((g == 0) ? (Zx[j] & 0xffffu) : (Zx[j] >> 16)));
            float v[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) v[c] = bf16_to_f32(f32_to_bf16(__builtin_fmaf((float)(c - 2), sc_g, zp_g)));
            coef[g][0] = v[0];
            coef[g][1] = v[1] - v[0];
            coef[g][2] = v[2] - v[0];
            coef[g][3] = (v[3] - v[2]) - (v[1] - v[0]);
          }
          const int tok = chunk * 64 + 16 * j + t16;
#pragma unroll
          for (int set = 0; set < NSET; ++set) {
            const v4i zero = {0, 0, 0, 0};
            float score = 0.f;
#pragma unroll
            for (int g = 0; g < NG; ++g) {
              v4i D0, D1, D01;
              if (NG == 2) {
                D0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], X0[g], zero, 0, 0, 0);
                D1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], X1[g], zero, 0, 0, 0);
                D01 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], X01[g], zero, 0, 0, 0);
              } else {
                D0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][0], X0[0], zero, 0, 0, 0);
                D0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][1], X0[1], D0, 0, 0, 0);
                D1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][0], X1[0], zero, 0, 0, 0);
                D1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][1], X1[1], D1, 0, 0, 0);
                D01 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][0], X01[0], zero, 0, 0, 0);
                D01 = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][1], X01[1], D01, 0, 0, 0);
              }
              const float s0f = (float)join_limbs(D0[2], D0[1], D0[0]);
              const float s1f = (float)join_limbs(D1[2], D1[1], D1[0]);
              const float s01f = (float)join_limbs(D01[2], D01[1], D01[0]);
              float v = coef[g][0] * sumq[set][g];
              v = __builtin_fmaf(coef[g][1], s0f, v);
              v = __builtin_fmaf(coef[g][2], s1f, v);
              v = __builtin_fmaf(coef[g][3], s01f, v);
              score = __builtin_fmaf(v, qsc[set][g], score);
            }
            const int h = set * 4 + lg;
            if ((G % 4 == 0) || h < G) {
              sc[h * L + tok] = score;
              mxl[set] = fmaxf(mxl[set], score);
              mnl[set] = fminf(mnl[set], score);
            }
          }
          continue;
        }
        if constexpr (K3) {
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              Br[u][e] = (int)__builtin_amdgcn_perm(0x01000000u, 0x0000ff00u, (uint32_t)Bc[u][e]);
        }
        // per-token scales (both groups) and the rounding coefficient
        float sg[NG], eg[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          sg[g] = sgj[j][g];
          eg[g] = egj[j][g];
        }
        const int tok = chunk * 64 + 16 * j + t16;
        if constexpr (NG == 2 && NSET >= 2) {
          // Two head sets: with two wavefronts per SIMD little else hides the wait for an MFMA's results, so all of a
          // token group's products are issued first and read afterwards.
          const v4i zero = {0, 0, 0, 0};
          v4i Dc_all[NSET][NG], Dr_all[NSET][NG];
#pragma unroll
          for (int set = 0; set < NSET; ++set)
#pragma unroll
            for (int g = 0; g < NG; ++g) {
              Dc_all[set][g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], Bc[g], Cin[set][g], 0, 0, 0);
              Dr_all[set][g] = K3 ? __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], Br[g], zero, 0, 0, 0) : zero;
            }
#pragma unroll
          for (int set = 0; set < NSET; ++set) {
            float score = 0.f;
#pragma unroll
            for (int g = 0; g < NG; ++g) {
              const int xc = join_limbs(Dc_all[set][g][2], Dc_all[set][g][1], Dc_all[set][g][0]);
              float v = (float)xc;
              if constexpr (K3) v = __builtin_fmaf(eg[g], (float)((Dr_all[set][g][2] << 8) + Dr_all[set][g][1]), v);
              score = __builtin_fmaf(v, sg[g] * qsc[set][g], score);
            }
            const int h = set * 4 + lg;
            if ((G % 4 == 0) || h < G) {
              sc[h * L + tok] = score;
              mxl[set] = fmaxf(mxl[set], score);
              mnl[set] = fminf(mnl[set], score);
            }
          }
          continue;
        }
#pragma unroll
        for (int set = 0; set < NSET; ++set) {
          float score = 0.f;
          const v4i zero = {0, 0, 0, 0};
          if (NG == 2) {
#pragma unroll
            for (int g = 0; g < NG; ++g) {
              const v4i Dc = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], Bc[g], Cin[set][g], 0, 0, 0);
              const int xc = join_limbs(Dc[2], Dc[1], Dc[0]);
              float v = (float)xc;
              if constexpr (K3) {
                const v4i Dr = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][g], Br[g], zero, 0, 0, 0);
                const int xr = (Dr[2] << 8) + Dr[1];
                v = __builtin_fmaf(eg[g], (float)xr, v);
              }
              score = __builtin_fmaf(v, sg[g] * qsc[set][g], score);
            }
          } else {
            v4i Dc = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][0], Bc[0], Cin[set][0], 0, 0, 0);
            Dc = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][1], Bc[1], Dc, 0, 0, 0);
            const int xc = join_limbs(Dc[2], Dc[1], Dc[0]);
            float v = (float)xc;
            if constexpr (K3) {
              v4i Dr = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][0], Br[0], zero, 0, 0, 0);
              Dr = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][1], Br[1], Dr, 0, 0, 0);
              const int xr = (Dr[2] << 8) + Dr[1];
              v = __builtin_fmaf(eg[0], (float)xr, v);
            }
            score = __builtin_fmaf(v, sg[0] * qsc[set][0], score);
          }
          const int h = set * 4 + lg;
          if ((G % 4 == 0) || h < G) {
            sc[h * L + tok] = score;
            mxl[set] = fmaxf(mxl[set], score);
            mnl[set] = fminf(mnl[set], score);
          }
        }
      }
    };
    // at most Lds::LMAX / 64 / NW chunks per wavefront: straight-line code, so that the wait for a chunk's
    // loads leaves the loads of the following chunks in flight
    // (step it + 1 sits inside step it's block, and the chunk two ahead is requested unconditionally, clamped: no
    // two paths with different numbers of loads in flight meet before a wait)
    auto key_step = [&](auto self, auto it_tag) -> void {
      constexpr int it = decltype(it_tag)::value;
      const int chunk = wave + it * NW;
      prefetch_v(it);
      if (chunk < nch_cover) {
        set_wave_prio(3 - it);  // wavefronts that are behind get the issue slots first
        KBuf& cur = (it & 1) ? Kb : Ka;
        stash_k(cur);
        wave_lds_fence();
        uint32_t Sc[4] = {0u, 0u, 0u, 0u}, Zc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (!SPREP || j == 0) Sc[j] = reg_copy(cur.s[SPREP ? 0 : j]);
          Zc[j] = KA ? reg_copy(cur.z[KA ? j : 0]) : 0u;
        }
        if constexpr (it + 2 < MAXIT) cur = issue_k(min(chunk + 2 * NW, nch_cover - 1));
        const int n_local = n - chunk * 64;  // (uniform)
        if (n_local > 0) {
          if (n_local < 64) clone_last_row(n_local, Sc, Zc);
          if constexpr (SPREP) {  // lane = token: scales and rounding coefficients of the chunk -> table
            const uint32_t sw = Sc[0];
            uint8_t* sp = kst + Lds::KST + lane * Lds::SCT;
            const float s0f = bf16_to_f32((uint16_t)(sw & 0xffffu));
            const float e0f = K3 ? eps_sh[0][sw & 0x7fu] : 0.f;
            if (NG == 2) {
              const float s1f = bf16_to_f32((uint16_t)(sw >> 16));
              const float e1f = K3 ? eps_sh[0][(sw >> 16) & 0x7fu] : 0.f;
              *reinterpret_cast<v4f*>(sp) = (v4f){s0f, s1f, e0f, e1f};
            } else {
              *reinterpret_cast<v2f*>(sp) = (v2f){s0f, e0f};
            }
            wave_lds_fence();
          }
          body(chunk, Sc, Zc);
        }
        if (n_local < 64) mask_tail(chunk, n_local);
        wave_lds_fence();
        if constexpr (it + 1 < MAXIT) self(self, std::integral_constant<int, it + 1>{});
      }
    };
    key_step(key_step, std::integral_constant<int, 0>{});
    // lanes of 16-lane row lg hold the running extrema of head set*4 + lg: reduce inside the rows (lane 15 of
    // a row ends up with the row's result) and publish them
#pragma unroll
    for (int set = 0; set < NSET; ++set) {
      float a = mxl[set], c = -mnl[set];
      JF_DPP_ROW_REDUCE(a, op_fmax, float, -INFINITY);
      JF_DPP_ROW_REDUCE(c, op_fmax, float, -INFINITY);
      const int h = set * 4 + lg;
      if (t16 == 15 && h < G) {
        red_f[wave][h] = a;
        red_f[wave][G + h] = -c;
      }
    }
  } else {
    // INT4 keys, int8-Q model on v_mfma_i32_16x16x64_i8: exact nibble codes (offset 8 removed through the
    // per-block constant), int32 block sums, the reference's four-term fp32 rescale in its order
    // (int8tc_qk_scores.cu:455-468).  Lane (token, k-block lg) spreads the 16 channels 64*m + 16*lg .. +15 of
    // both 64-channel spans m; its accumulator registers are the four 32-channel blocks of head lg.
    const QInt8F<NSET>* qsh = reinterpret_cast<const QInt8F<NSET>*>(aux);
    v4i Aop[NSET][2];
    v4i nsum8[NSET];  // minus the block sums: the accumulators' initial values
    float qs[NSET][4];
#pragma unroll
    for (int set = 0; set < NSET; ++set) {
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) Aop[set][mi] = *reinterpret_cast<const v4i*>(&qsh->aop[set][t16][lg][mi][0]);
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        nsum8[set][kk] = -qsh->sum8[set * 4 + lg][kk];
        qs[set][kk] = qsh->qs[set * 4 + lg][kk];
      }
    }
    const uint8_t* krd = kst + t16 * KROW + lg * 8;
    float mxl[NSET], mnl[NSET];
#pragma unroll
    for (int set = 0; set < NSET; ++set) {
      mxl[set] = -INFINITY;
      mnl[set] = INFINITY;
    }
    auto body = [&](int chunk, const uint32_t (&Sx)[4]) {
      v2u Xj[4][2];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint8_t* rp = krd + j * 16 * KROW;
        Xj[j][0] = *reinterpret_cast<const v2u*>(rp);
        Xj[j][1] = *reinterpret_cast<const v2u*>(rp + 32);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v4i Bm[2];
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) {
          const uint32_t x0 = Xj[j][mi][0], x1 = Xj[j][mi][1];
          Bm[mi] = (v4i){(int)((x0 >> 4) & 0x0f0f0f0fu), (int)(x0 & 0x0f0f0f0fu), (int)((x1 >> 4) & 0x0f0f0f0fu), (int)(x1 & 0x0f0f0f0fu)};
        }
        const float ks = bf16_to_f32((uint16_t)Sx[j]);
        const int tok = chunk * 64 + 16 * j + t16;
#pragma unroll
        for (int set = 0; set < NSET; ++set) {
          // (the -8 * sum of the block's query values, the codes being used unsigned, enters as the accumulator's
          // initial value: exact, and four subtractions per token and head less)
          v4i Dq = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][0], Bm[0], nsum8[set], 0, 0, 0);
          Dq = __builtin_amdgcn_mfma_i32_16x16x64_i8(Aop[set][1], Bm[1], Dq, 0, 0, 0);
          float sacc = (float)Dq[0] * qs[set][0];
#pragma unroll
          for (int kk = 1; kk < 4; ++kk) sacc = __builtin_fmaf((float)Dq[kk], qs[set][kk], sacc);
          const float a = __fmul_rn(__fmul_rn(sacc, ks), p.attn_scale);
          const int h = set * 4 + lg;
          if ((G % 4 == 0) || h < G) {
            sc[h * L + tok] = a;
            mxl[set] = fmaxf(mxl[set], a);
            mnl[set] = fminf(mnl[set], a);
          }
        }
      }
    };
    auto key_step = [&](auto self, auto it_tag) -> void {  // (nested, as for the other key formats)
      constexpr int it = decltype(it_tag)::value;
      const int chunk = wave + it * NW;
      prefetch_v(it);
      if (chunk < nch_cover) {
        set_wave_prio(3 - it);
        KBuf& cur = (it & 1) ? Kb : Ka;
        stash_k(cur);
        wave_lds_fence();
        uint32_t Sc[4], Zc[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 4; ++j) Sc[j] = reg_copy(cur.s[j]);
        if constexpr (it + 2 < MAXIT) cur = issue_k(min(chunk + 2 * NW, nch_cover - 1));
        const int n_local = n - chunk * 64;  // (uniform)
        if (n_local > 0) {
          if (n_local < 64) clone_last_row(n_local, Sc, Zc);
          body(chunk, Sc);
        }
        if (n_local < 64) mask_tail(chunk, n_local);
        wave_lds_fence();
        if constexpr (it + 1 < MAXIT) self(self, std::integral_constant<int, it + 1>{});
      }
    };
    key_step(key_step, std::integral_constant<int, 0>{});
#pragma unroll
    for (int set = 0; set < NSET; ++set) {
      float a = mxl[set], c = -mnl[set];
      JF_DPP_ROW_REDUCE(a, op_fmax, float, -INFINITY);
      JF_DPP_ROW_REDUCE(c, op_fmax, float, -INFINITY);
      const int h = set * 4 + lg;
      if (t16 == 15 && h < G) {
        red_f[wave][h] = a;
        red_f[wave][G + h] = -c;
      }
    }
  }

  if (clk && tid == 0) clk[9] = JF_CLK();  // wavefront 0 finished its chunks
  if (clk && lane == 0) atomicMax(&tmax_sh, (unsigned long long)JF_CLK());
  __builtin_amdgcn_s_setprio(0);
  // split extrema per head; fixed-point exponent of the V scales; selection buckets
  if constexpr (HAS_V) {
    uint32_t vm0 = 0u, vm1 = 0u;
#pragma unroll
    for (int i = 0; i < VSPT; ++i) {
      vm0 = max(vm0, vsw[i] & 0x7fffu);
      vm1 = max(vm1, (vsw[i] >> 16) & 0x7fffu);
    }
    vm0 = wave_max_u(vm0);
    vm1 = wave_max_u(vm1);
    if (lane == 0) {
      vmax_sh[wave][0] = vm0;
      vmax_sh[wave][1] = vm1;
    }
  }
  lds_barrier();  // phase A complete: the query constants are dead, their space becomes the histograms
  if (clk && tid == 0) { clk[8] = JF_CLK(); clk[5] = (long long)tmax_sh; }
  if (p.scores)  // validation output
    for (int i = tid; i < GA * n_cover; i += NT) {
      const int h = i / n_cover, t = i - h * n_cover;
      p.scores[(head0 + h) * (size_t)p.max_S + s0 + t] = sc[h * L + t];
    }
  if constexpr (MODE == FS_STAGE_A)
    if (p.scores_only) return;
  if constexpr (HAS_TOPK)
    for (int i = tid; i < Lds::HIST / 4; i += NT) hist[i] = 0;
  if (tid < G) {
    float m = red_f[0][tid], lo = red_f[0][G + tid];
#pragma unroll
    for (int w = 1; w < NW; ++w) {
      m = fmaxf(m, red_f[w][tid]);
      lo = fminf(lo, red_f[w][G + tid]);
    }
    m_sh[tid] = m;
    // bucket of a score: min(255, (m - s) * 255 / (m - lo)), bucket 0 = largest; monotone in s
    const float range = m - lo;
    const float iw = (range > 0.f && isfinite(range)) ? 254.99f / range : 0.f;
    bin_a_sh[tid] = -iw;
    bin_b_sh[tid] = isfinite(m) ? m * iw : 0.f;
  }
  if (HAS_V && tid >= 64 && tid < 64 + NG) {
    const int g = tid - 64;
    uint32_t vb = vmax_sh[0][g];
#pragma unroll
    for (int w = 1; w < NW; ++w) vb = max(vb, vmax_sh[w][g]);
    const float v = bf16_to_f32((uint16_t)vb);
    int e = 0;
    if (v > 0.f && isfinite(v)) (void)frexpf(v, &e);  // v = f * 2^e, f in [0.5, 1)
    e_sh[g] = 23 - e;                                 // v * 2^E in [2^22, 2^23): the weights use all 23 mantissa bits
  }
  lds_barrier();
  if (clk && tid == 0) clk[1] = JF_CLK();

  // ------------------------------------------------------------------ phase B: P.V on v_mfma_i32_16x16x64_i8
  // p = exp(s - m_split) is known exactly because phase A is complete, so w = p * v_scale is converted to
  // 23-bit fixed point once (fma with 2^23: p <= 1 and the largest V scale below 2^e keep the sum below 2^24, where
  // floats are integers); its three bytes, the lower two balanced around zero, are rows (limb, head) of
  // the A operand.  Lane = token stores the four heads' converted words as one 16-byte row per scale group (head-major;
  // the word's top byte is the constant 75 and becomes a constant row), and ds_read_b64_tr_b8 turns 8 token rows into the per-row byte runs the MFMA
  // wants.  V codes are staged packed in wavefront-private LDS and transposed by ds_read_b64_tr_b4 (16
  // tokens of one channel pair per lane), then spread.  sum_t w_t*(code - off) = sum_t w_t*code - off*sum_t w_t:
  // the constant row gives 75 * sum_t code (needed because the limbs are balanced), a ones B tile gives sum_t w_t.
  // Every accumulation is an exact integer.  The same pass drops every score into one of 256 linear buckets
  // per (head, half of the split) for the candidate selection.
  int E[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) E[g] = HAS_V ? __builtin_amdgcn_readfirstlane(e_sh[g]) : 0;
  v4i acc[NSET][NTILE], accw[NSET][NG];
#pragma unroll
  for (int set = 0; set < NSET; ++set) {
#pragma unroll
    for (int t = 0; t < NTILE; ++t) acc[set][t] = (v4i){0, 0, 0, 0};
#pragma unroll
    for (int g = 0; g < NG; ++g) accw[set][g] = (v4i){0, 0, 0, 0};
  }
  float lsum[G], nml[G], bin_a[G], bin_b[G];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    lsum[h] = 0.f;
    nml[h] = uniform_f(-(m_sh[h] * LOG2E));
    bin_a[h] = uniform_f(bin_a_sh[h]);
    bin_b[h] = uniform_f(bin_b_sh[h]);
  }
  // The bucket of a score is fma(s, a, b) clamped to [0, 255] with a and b uniform: an instruction takes one scalar
  // operand only, and left alone the compiler copies b (and 255.0, and the increment) into a vector register again
  // for every head of every chunk.  Copies it cannot see through stay in their registers through the stream.
  float bin_bv[G], clamp_hi = 255.f;
#pragma unroll
  for (int h = 0; h < G; ++h) {
    bin_bv[h] = bin_b[h];
    asm volatile("" : "+v"(bin_bv[h]));
  }
  asm volatile("" : "+v"(clamp_hi));
  v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};  // all-ones B tile of the weight sums (kept, like the above)
  asm volatile("" : "+v"(ones));
  const int r16 = lane & 15, kb4 = lane >> 4;
  // transposed weight read: 16-lane group kb4 fetches the rows of tokens 16*kb4 .. +15; the lane pair (2j, 2j+1)
  // supplies the two halves of the row that must land in byte j, i.e. of the token whose byte position in the
  // V operand (see below) is j
  const int tr_tok = (((r16 >> 1) & 3) << 1) | ((r16 >> 3) & 1);
  const uint8_t* wrow = wl + (kb4 * 16 + tr_tok) * 16 + (r16 & 1) * 8;
  const int seg_chunks = L / 64 / SEG;  // chunks per emission segment
  auto body_v = [&](int chunk, uint32_t vsw) {
    const int t = chunk * 64 + lane;
    float vsf[NG];
    vsf[0] = ldexpf(bf16_to_f32((uint16_t)(vsw & 0xffffu)), E[0]);
    if (NG == 2) vsf[NG - 1] = ldexpf(bf16_to_f32((uint16_t)(vsw >> 16)), E[NG - 1]);
    int* hb = hist + ((SEG == 1) ? 0 : (chunk / seg_chunks) * (Lds::H16 ? 128 : 256));
    const bool tv = t < n;
    const int inc = tv ? 1 : 0;
    (void)inc;
    uint32_t bits[NSET * 4][NG];
#pragma unroll
    for (int h = 0; h < NSET * 4; ++h) {
      if (h < G) {
        const float s = sc[h * L + t];
        // masked positions hold -inf: their weight is exactly zero
        const float pw = __builtin_amdgcn_exp2f(__builtin_fmaf(s, LOG2E, nml[h]));
        lsum[h] += pw;
#pragma unroll
        for (int g = 0; g < NG; ++g) bits[h][g] = __builtin_bit_cast(uint32_t, __builtin_fmaf(pw, vsf[g], 8388608.0f));
        if constexpr (HAS_TOPK) {
          // (positions past the end add zero instead of branching around the add: their score is -inf or, with a
          // degenerate range, gives a NaN, and either clamps to a bucket inside the table)
          const uint32_t bin = (uint32_t)__builtin_amdgcn_fmed3f(__builtin_fmaf(s, bin_a[h], bin_bv[h]), 0.f, clamp_hi);
          if (Lds::H16) atomicAdd(hb + ((h * (SEG * 256) + (int)bin) >> 1), inc << ((bin & 1u) << 4));
          else atomicAdd(hb + h * (SEG * 256) + (int)bin, inc);
        }
      } else {
#pragma unroll
        for (int g = 0; g < NG; ++g) bits[h][g] = 0x4b000000u;
      }
    }
    if constexpr (!HAS_V) return;  // Stage A alone: the weights' sums and the selection buckets were all
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int set = 0; set < NSET; ++set) {
        // one 16-byte row per token: byte 4h + l = limb l of head h (limbs 0 and 1 balanced around zero, limb 2 < 128),
        // byte 4h + 3 = 75, the exponent byte of the fixed-point conversion, which serves as the constant row that
        // yields the code sums
        v4i row;
#pragma unroll
        for (int hh = 0; hh < 4; ++hh) row[hh] = (int)(bits[set * 4 + hh][g] ^ 0x00008080u);
        *reinterpret_cast<v4i*>(wl + ((g * NSET + set) * 64 + lane) * 16) = row;
      }
    wave_lds_fence();
    v4i A[NG][NSET];
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int set = 0; set < NSET; ++set) {
        const uint8_t* src = wrow + (g * NSET + set) * 1024;
        const v2i x0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i*)(src));
        const v2i x1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i*)(src + 128));
        A[g][set] = (v4i){x0[0], x0[1], x1[0], x1[1]};
      }
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int set = 0; set < NSET; ++set)
        accw[set][g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[g][set], ones, accw[set][g], 0, 0, 0);
    // the nibble spread of a transposed V dword yields tokens 0,2,4,6 | 1,3,5,7 | 8,10,12,14 | 9,11,13,15 of the
    // lane group's 16 tokens: token r sits in byte (r&8) | ((r&1)<<2) | ((r>>1)&3)
    const uint8_t* vrow = vst + lane * VROW;
    if (V2) {
#pragma unroll
      for (int qc = 0; qc < 4; ++qc) {
        const v2i x = __builtin_amdgcn_ds_read_tr4_b64_v2i32((__attribute__((address_space(3))) v2i*)(vrow + 8 * qc));
        const uint32_t x0 = (uint32_t)x[0], x1 = (uint32_t)x[1], y0 = x0 >> 4, y1 = x1 >> 4;
        // the upper code of every nibble stays where it is: tile 2*qc accumulates 4 * code (undone in `combine`)
        const v4i Ba = {(int)(x0 & 0x0c0c0c0cu), (int)(y0 & 0x0c0c0c0cu), (int)(x1 & 0x0c0c0c0cu), (int)(y1 & 0x0c0c0c0cu)};
        const v4i Bb = {(int)(x0 & 0x03030303u), (int)(y0 & 0x03030303u), (int)(x1 & 0x03030303u), (int)(y1 & 0x03030303u)};
        const int g = (NG == 1) ? 0 : (qc >> 1);
#pragma unroll
        for (int set = 0; set < NSET; ++set) {
          acc[set][2 * qc] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[g][set], Ba, acc[set][2 * qc], 0, 0, 0);
          acc[set][2 * qc + 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[g][set], Bb, acc[set][2 * qc + 1], 0, 0, 0);
        }
      }
    } else if (V3) {
      // Planar INT3: bytes j of the three 16-byte planes form the 24-bit word of channels 8j .. 8j+7, code i at
      // bits 23-3i .. 21-3i.  A transposed read of one plane's 8-byte half hands lane c the nibble c of 16 tokens:
      // odd lanes the high nibbles of byte c >> 1, even lanes the low ones.  With one exchange inside the lane
      // pair (the odd lane needs its partner's plane-0 nibble, the even lane its partner's plane-2 nibble) the odd
      // lane holds what codes 0..3 of the word are made of and the even lane what codes 4..7 are made of, in the
      // same three positions: a = [c0 c0 c0 c1], b = [c1 c1 c2 c2], c = [c2 c3 c3 c3] (msb first).
      const bool odd = (lane & 1) != 0;
      const int hsw = 8 * ((lane >> 4) & 1);  // rows 16..31, 48..63 keep their plane halves swapped
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const uint8_t* src = vrow + (w ? 8 - hsw : hsw);
        const v2i x0 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((__attribute__((address_space(3))) v2i*)(src));
        const v2i x1 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((__attribute__((address_space(3))) v2i*)(src + 16));
        const v2i x2 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((__attribute__((address_space(3))) v2i*)(src + 32));
        v4i Bc[4];
#pragma unroll
        for (int hw = 0; hw < 2; ++hw) {  // tokens 0..7 and 8..15 of the lane group, one nibble each
          const int send = odd ? x2[hw] : x0[hw];
          const uint32_t b = (uint32_t)dpp_mov<0xb1, 0xf>(0, send);  // quad_perm [1,0,3,2]: the pair partner's value
          const uint32_t a = (uint32_t)(odd ? x0[hw] : x1[hw]), c = (uint32_t)(odd ? x1[hw] : x2[hw]);
          // per nibble (bit 3 of the two middle codes is cleared by the byte masks below)
          const uint32_t n1 = ((b >> 2) & 0x33333333u) | ((a << 2) & ~0x33333333u);
          const uint32_t n2 = ((c >> 3) & 0x11111111u) | ((b << 1) & ~0x11111111u);
          Bc[0][2 * hw] = (int)((a >> 1) & 0x07070707u);
          Bc[0][2 * hw + 1] = (int)((a >> 5) & 0x07070707u);
          Bc[1][2 * hw] = (int)(n1 & 0x07070707u);
          Bc[1][2 * hw + 1] = (int)((n1 >> 4) & 0x07070707u);
          Bc[2][2 * hw] = (int)(n2 & 0x07070707u);
          Bc[2][2 * hw + 1] = (int)((n2 >> 4) & 0x07070707u);
          Bc[3][2 * hw] = (int)(c & 0x07070707u);
          Bc[3][2 * hw + 1] = (int)((c >> 4) & 0x07070707u);
        }
        const int g = (NG == 1) ? 0 : w;
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
          for (int set = 0; set < NSET; ++set)
            acc[set][4 * w + m] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[g][set], Bc[m], acc[set][4 * w + m], 0, 0, 0);
      }
    } else {
      const int vx = 16 * ((lane >> 2) & 3);  // quarter swap of this lane's row
#pragma unroll
      for (int qc = 0; qc < 8; ++qc) {
        const v2i x = __builtin_amdgcn_ds_read_tr4_b64_v2i32((__attribute__((address_space(3))) v2i*)(vrow + (Lds::VSWZ ? ((8 * qc) ^ vx) : 8 * qc)));
        const uint32_t x0 = (uint32_t)x[0], x1 = (uint32_t)x[1];
        const v4i Bv = {(int)(x0 & 0x0f0f0f0fu), (int)((x0 >> 4) & 0x0f0f0f0fu),
                        (int)(x1 & 0x0f0f0f0fu), (int)((x1 >> 4) & 0x0f0f0f0fu)};
        const int g = (NG == 1) ? 0 : (qc >> 2);
#pragma unroll
        for (int set = 0; set < NSET; ++set)
          acc[set][qc] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[g][set], Bv, acc[set][qc], 0, 0, 0);
      }
    }
    wave_lds_fence();
  };
  auto stash_v = [&](const VBuf& vbuf) {
#pragma unroll
    for (int i = 0; i < VLD; ++i) {
      if (Lds::VSWZ) {
        *reinterpret_cast<v4u*>(vst + vl_lds[i]) = vbuf.r[i];  // 16-byte aligned with the unpadded pitch
      } else {
        *reinterpret_cast<v2u*>(vst + vl_lds[i]) = (v2u){vbuf.r[i][0], vbuf.r[i][1]};
        *reinterpret_cast<v2u*>(vst + (V3 ? (vl_lds[i] ^ 8u) : (vl_lds[i] + 8u))) = (v2u){vbuf.r[i][2], vbuf.r[i][3]};
      }
    }
  };
  if constexpr (MODE == FS_FULL) {  // (wavefronts that left the key stream before its last two steps)
    if (!va_requested) Va = issue_v(min(wave, nch - 1));
    if (!vb_requested) Vb = issue_v(min(wave + NW, nch - 1));
  }
  auto value_step = [&](auto self, auto it_tag) -> void {  // (nested like the key stream's steps)
    constexpr int it = decltype(it_tag)::value;
    const int chunk = wave + it * NW;
    if (chunk < nch) {
      set_wave_prio(3 - it);
      uint32_t vw = 0u;
      if constexpr (HAS_V) {
        VBuf& cur = (it & 1) ? Vb : Va;
        stash_v(cur);
        static_assert(VSPT == MAXIT, "one V scale word per thread and step");
        vw = vsw[it];
        if constexpr (it + 2 < MAXIT) cur = issue_v(min(chunk + 2 * NW, nch - 1));
      }
      body_v(chunk, vw);
      if constexpr (it + 1 < MAXIT) self(self, std::integral_constant<int, it + 1>{});
    }
  };
  value_step(value_step, std::integral_constant<int, 0>{});
  __builtin_amdgcn_s_setprio(0);
#pragma unroll
  for (int h = 0; h < G; ++h) {
    const float ls = wave_sum(lsum[h]);
    if (lane == 0) lsum_sh[wave][h] = ls;  // summed in wavefront order below: run-to-run deterministic
  }
  if constexpr (HAS_V) {
    // The accumulator sums below live at the start of the staging area: each wavefront clears what lies in its own
    // part (it is done with it), so the array is zero behind the barrier.
    const int z0 = wave * Lds::WAVE_STAGE;
    const int z1 = min(z0 + Lds::WAVE_STAGE, Lds::XACC);
    for (int o = z0 + lane * 16; o < z1; o += 1024) *reinterpret_cast<v4i*>(stage + o) = (v4i){0, 0, 0, 0};
  }
  lds_barrier();
  if (clk && tid == 0) clk[2] = JF_CLK();

  // ---- sum of the integer accumulators over the wavefronts: LDS integer atomics into one array at the start of
  // the staging area (cleared before the barrier above), read by `combine` after the candidates have been emitted.
  // Integer sums: exact and independent of the order.  The atomics return nothing, so a wavefront issues them a few
  // at a time along the comparisons of its first emission blocks: they drain in the LDS pipe while the vector ALU
  // works.
  // D layout: row r of a tile sits in lane 16*(r>>2) + column, register r&3; row 4*head + l is limb l for l < 3 and
  // the constant row (75 * sum of codes) for l = 3.  Item j = (register i = j >> 2 of set i / AR, component j & 3)
  // lives at xacc[j * 64 + lane].
  int* xacc = reinterpret_cast<int*>(stage);
  constexpr int ACC_TOTAL = NSET * AR, ACC_HALF = (ACC_TOTAL + 1) / 2;
  bool acc_issued = false;  // (uniform) this wavefront's sums are on their way
  auto add_acc_range = [&](const int first, const int last) {  // (constants once the caller's loop is unrolled)
#pragma unroll
    for (int j = 0; j < ACC_TOTAL * 4; ++j) {
      if (j < first || j >= last) continue;
      const int i = j >> 2, c = j & 3, set = i / AR, r = i % AR;
      const v4i v = (r < NTILE) ? acc[set][r < NTILE ? r : 0] : accw[set][r >= NTILE ? r - NTILE : 0];
      atomicAdd(xacc + j * 64 + lane, v[c]);
    }
  };
  auto combine = [&](int set) {
    // thread -> (tile, head, column)
    for (int i = tid; i < 4 * D; i += NT) {
      const int col = i & 15, hh = (i >> 4) & 3, tile = i >> 6;
      const int h = set * 4 + hh;
      if (h >= GA) continue;
      int d;
      if (V2) {
        const int e = ((col & 1) ? 0 : 2) + (tile & 1);
        d = (tile >> 1) * 32 + (col >> 1) * 4 + e;
      } else if (V3) {  // tile = 4 * (64-channel half) + code within the lane's four; odd columns hold codes 0..3
        d = (tile >> 2) * 64 + (col >> 1) * 8 + ((col & 1) ? 0 : 4) + (tile & 3);
      } else {
        d = tile * 16 + 2 * (col >> 1) + (1 - (col & 1));
      }
      const int g = (NG == 1) ? 0 : (d / (D / NG));
      const int* ta = xacc + ((set * AR + tile) * 4) * 64 + 16 * hh + col;   // row 4*hh + l of the tile: component l, lane 16*hh + col
      const int* wa = xacc + ((set * AR + NTILE + g) * 4) * 64 + 16 * hh;    // weight sums: any column of the all-ones tile
      int i0 = ta[0], i1 = ta[64], i2 = ta[128], cs = ta[192] / 75;          // (row 4*hh + 3 holds 75 * sum of the codes)
      if (V2 && !(tile & 1)) {  // even INT2 tiles hold four times their sums (exact multiples)
        i0 >>= 2;
        i1 >>= 2;
        i2 >>= 2;
        cs >>= 2;
      }
      const int w0 = wa[0], w1 = wa[64], w2 = wa[128];   // |sum| < 2^24: no overflow
      const long long wsum = (long long)w2 * 65536ll + (long long)w1 * 256ll + (long long)w0 + 32896ll * 64ll * (long long)nch;
      const long long tot = (long long)i2 * 65536ll + (long long)i1 * 256ll + (long long)i0 + 32896ll * (long long)cs - (long long)VOFF * wsum;
      p.part_o[(part_base + (size_t)h * p.n_splits) * D + d] = (float)ldexp((double)tot, -E[g]);
    }
  };

  // ------------------------------------------------------------------ phase C: candidates of the split
  // The merge kernel needs a superset of the split's top Kt = min(top_k, n) scores per head that fits the
  // candidate buffer (Kcap entries), in ascending position.  From the histograms: the smallest bucket index
  // `cut` with count(bucket <= cut) >= Kt.  If that count fits, every position whose bucket is <= cut is
  // emitted, one wavefront per (head, segment of the split), each segment starting where the counts of the segments
  // before it end.  Otherwise (heavily tied scores) one wavefront falls back to an exact radix select over the keys.
  const int Kcap = p.Kc;
  const int Kt = min(p.top_k, n);
  for (int hs = wave; HAS_TOPK && hs < G * SEG; hs += NW) {
    const int h = hs / SEG, seg = hs % SEG;
    if (h >= GA) continue;
    // Every wavefront of a head searches the cut itself (same histograms, same result): no exchange, no barrier
    // between the search and the emission.
    const float ba = uniform_f(bin_a_sh[h]);
    float bb = uniform_f(bin_b_sh[h]);
    asm volatile("" : "+v"(bb));  // (kept in a vector register: the multiply-add takes one scalar operand only)
    const int* h0 = hist + h * (SEG * 256) / (Lds::H16 ? 2 : 1);
    // lane l owns buckets 4l .. 4l+3 (ascending bucket = descending score) of every segment's histogram
    int cs[SEG][4], c[4], mine;
#pragma unroll
    for (int sg = 0; sg < SEG; ++sg) {
      if (Lds::H16) {
        const uint32_t w0 = (uint32_t)h0[sg * 128 + 2 * lane], w1 = (uint32_t)h0[sg * 128 + 2 * lane + 1];
        cs[sg][0] = (int)(w0 & 0xffffu);
        cs[sg][1] = (int)(w0 >> 16);
        cs[sg][2] = (int)(w1 & 0xffffu);
        cs[sg][3] = (int)(w1 >> 16);
      } else {
        const v4i x = *reinterpret_cast<const v4i*>(h0 + sg * 256 + 4 * lane);
#pragma unroll
        for (int u = 0; u < 4; ++u) cs[sg][u] = x[u];
      }
    }
    // c[u]: the bucket's count over all segments; cum[u]: over the segments before this wavefront's
    int cum[4] = {0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < 4; ++u) c[u] = 0;
#pragma unroll
    for (int sg = 0; sg < SEG; ++sg) {
      if (sg == seg) {  // (uniform)
#pragma unroll
        for (int u = 0; u < 4; ++u) cum[u] = c[u];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) c[u] += cs[sg][u];
    }
    mine = (c[0] + c[1]) + (c[2] + c[3]);
    const int cumt = (cum[0] + cum[1]) + (cum[2] + cum[3]);
    // one scan for both: the totals in the low half, the earlier segments' in the high half (each sum <= 4096)
    const int packed = mine | (cumt << 16);
    const int incl = wave_incl_scan_i(packed);
    // the first lane whose inclusive total reaches Kt holds the cut bucket; the rest is scalar arithmetic on that
    // lane's four counts
    const unsigned long long who = __ballot((incl & 0xffff) >= Kt);
    bool ok = false;
    int cut = 255, tot = 0, before_me = 0;
    if (who != 0ull) {
      const int src = __ffsll((long long)who) - 1;
      const int ex = __builtin_amdgcn_readlane(incl - packed, src);  // exclusive sums at that lane
      int run = ex & 0xffff;
      before_me = ex >> 16;
      bool found = false;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int cu = __builtin_amdgcn_readlane(c[u], src), mu = __builtin_amdgcn_readlane(cum[u], src);
        if (!found) {
          run += cu;
          before_me += mu;
          if (run >= Kt) {
            found = true;
            cut = 4 * src + u;
            tot = run;
          }
        }
      }
      ok = tot <= Kcap;
    }
    if (clk && tid == 0) clk[6] = JF_CLK();
    const float* srow = sc + h * L;
    uint32_t* ck = p.cand_key + (part_base + (size_t)h * p.n_splits) * Kcap;
    int32_t* ci = p.cand_idx + (part_base + (size_t)h * p.n_splits) * Kcap;
    if (ok) {
      // bucket(s) <= cut  <=>  not (s * ba + bb >= cut + 1): the bucket is the floor of that value clamped to
      // [0, 255]; with cut = 255 every position qualifies
      const float thr = uniform_f((cut >= 255) ? INFINITY : (float)(cut + 1));
      const int tb = seg * (L / SEG);
      const int te = min(n, (seg + 1) * (L / SEG));
      // the emitted total is at most Kcap by construction of the cut
      int count = __builtin_amdgcn_readfirstlane(before_me);
      // unused slots hold key 0 (no score maps to it); the planned total is known, so the head's wavefronts
      // share the padding and its stores leave before the emission's
      const int etot = min(Kcap, tot);
      for (int i = etot + seg * 64 + lane; i < Kcap; i += SEG * 64) ck[i] = 0u;
      // Blocks of 1024 positions, 16 consecutive ones per lane: the lane's candidates are consecutive in the output,
      // so a block costs one comparison per position, one wavefront scan of the lanes' counts, and a loop over the
      // few set bits of every lane.  The lane reads its four 16-byte quads starting at quad (lane >> 2) & 3 (the
      // four lanes that share a bank group then read different banks) and rotates its bit mask back afterwards.
      const int rot4 = ((lane >> 2) & 3) * 4;
      auto emit_block = [&](int t0, auto acc_tag) {
        constexpr int ACCSEL = decltype(acc_tag)::value;  // accumulator sums issued along the comparisons: -1 none, 0 / 1 a half, 2 all
        constexpr int A_LO = (ACCSEL == 1) ? ACC_HALF * 4 : 0;
        constexpr int A_HI = (ACCSEL < 0) ? 0 : ((ACCSEL == 0) ? ACC_HALF * 4 : ACC_TOTAL * 4);
        constexpr int PER = (A_HI - A_LO + 15) / 16;      // a few behind every comparison: the LDS queue never fills
        const int lt = t0 + 16 * lane;                    // first position of this lane
        const float* lp = srow + lt;
        v4f x[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) x[q] = *reinterpret_cast<const v4f*>(lp + ((4 * q + rot4) & 15));
        uint32_t ge = 0u;  // bit 4q + e set: element e of quad register q falls behind the cut (not emitted)
#pragma unroll
        for (int bi = 15; bi >= 0; --bi) {
          // ge = 2 * ge + [value >= thr]: the comparison's lane mask is the carry of one add
          const unsigned long long c = __builtin_amdgcn_ballot_w64(__builtin_fmaf(x[bi >> 2][bi & 3], ba, bb) >= thr);
          // (the two wait states between a vector instruction's scalar result and a vector instruction that reads it
          // are the compiler's job everywhere else; it does not look inside an asm statement)
          asm("s_nop 1\n\tv_addc_co_u32_e64 %0, vcc, %1, %1, %2" : "=v"(ge) : "v"(ge), "s"(c) : "vcc");
          if constexpr (HAS_V && PER > 0) {
            const int lo = A_LO + (15 - bi) * PER;
            if (lo < A_HI) {
              add_acc_range(lo, (lo + PER < A_HI) ? lo + PER : A_HI);
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
        // register bit b is position (b + rot4) mod 16 of the lane's run
        uint32_t m2 = ~ge & 0xffffu;
        m2 |= m2 << 16;
        uint32_t mask = (m2 >> (16 - rot4)) & 0xffffu;
        const int nvalid = max(0, min(16, te - lt));
        mask &= (1u << nvalid) - 1u;
        const int mine = __popc(mask);
        const int incl = wave_incl_scan_i(mine);
        uint32_t o = (uint32_t)(count + incl - mine);
        count += __builtin_amdgcn_readlane(incl, 63);
        // (the score of the next set bit is requested before the current one is stored: one LDS latency per lane run,
        // not one per candidate)
        int i = (mask != 0u) ? __ffs((int)mask) - 1 : 0;
        float sco = lp[i];
        while (mask != 0u) {
          mask &= mask - 1u;
          const int i_next = (mask != 0u) ? __ffs((int)mask) - 1 : 0;
          const float s_next = lp[i_next];
          if (o < (uint32_t)Kcap) {  // the bound only matters for non-finite scores
            ck[o] = score_key(sco);
            ci[o] = s0 + lt + i;
          }
          ++o;
          i = i_next;
          sco = s_next;
        }
      };
      constexpr std::integral_constant<int, -1> plain{};
      int t0 = tb;
      if (HAS_V && !acc_issued && te > tb) {  // the first block (or the first two) of this wavefront carry the sums
        if (te - tb > 1024) {
          emit_block(tb, std::integral_constant<int, 0>{});
          emit_block(tb + 1024, std::integral_constant<int, 1>{});
          t0 = tb + 2048;
        } else {
          emit_block(tb, std::integral_constant<int, 2>{});
          t0 = tb + 1024;
        }
        acc_issued = true;
      }
      for (; t0 < te; t0 += 1024) emit_block(t0, plain);
      if (seg == SEG - 1) {
        if (lane == 0) p.cand_cnt[part_base + (size_t)h * p.n_splits] = min(Kcap, count);
        for (int i = count + lane; i < etot; i += 64) ck[i] = 0u;  // (only if a segment emitted less than planned)
      }
    } else if (seg == 0) {
      // exact fallback: 8-bit radix select over the order-preserving keys (bits shared by every key skipped),
      // then the keys above the K-th and the lowest-position ties that fill the quota
      int* rh = reinterpret_cast<int*>(stage + Lds::XACC + wave * 1024);
      uint32_t T = 0;
      int quota = 0;
      uint32_t kmin = 0xffffffffu, kmax = 0u;
      for (int t = lane; t < n; t += 64) {
        const uint32_t k = score_key(srow[t]);
        kmin = min(kmin, k);
        kmax = max(kmax, k);
      }
      kmin = wave_min_u(kmin);
      kmax = wave_max_u(kmax);
      const uint32_t diff = kmin ^ kmax;
      if (diff == 0u) {  // every key equal: the lowest positions win
        T = kmax;
        quota = Kt;
      } else {
        int bits_left = 32 - __clz((int)diff);  // number of low bits that vary
        uint32_t prefix = (bits_left == 32) ? 0u : (kmax >> bits_left);
        int k_rem = Kt;
        while (bits_left > 0) {
          const int nb = min(8, bits_left);
          const int shift = bits_left - nb;
          const uint32_t dmask = (1u << nb) - 1u;
          for (int i = lane; i < 256; i += 64) rh[i] = 0;
          const bool first = (bits_left == 32);
          const int hi_shift = first ? 0 : bits_left;
          for (int t0 = 0; t0 < n; t0 += 64) {
            const int t = t0 + lane;
            const uint32_t k = (t < n) ? score_key(srow[t]) : 0u;
            const bool inpre = (t < n) && (first || ((k >> hi_shift) == prefix));
            if (inpre) atomicAdd(&rh[(int)((k >> shift) & dmask)], 1);
          }
          // lane l owns bins 255-4l .. 252-4l (descending), so a prefix scan over lanes counts the bins above
          const int c3 = rh[255 - 4 * lane], c2 = rh[254 - 4 * lane], c1 = rh[253 - 4 * lane], c0 = rh[252 - 4 * lane];
          const int mine = c0 + c1 + c2 + c3;
          const int e3 = wave_incl_scan_i(mine) - mine;  // keys in bins above 255-4l
          const int e2 = e3 + c3, e1 = e2 + c2, e0 = e1 + c1;
          int cut = -1, above = 0;
          if (e3 < k_rem && k_rem <= e3 + c3) { cut = 255 - 4 * lane; above = e3; }
          else if (e2 < k_rem && k_rem <= e2 + c2) { cut = 254 - 4 * lane; above = e2; }
          else if (e1 < k_rem && k_rem <= e1 + c1) { cut = 253 - 4 * lane; above = e1; }
          else if (e0 < k_rem && k_rem <= e0 + c0) { cut = 252 - 4 * lane; above = e0; }
          const unsigned long long who = __ballot(cut >= 0);
          const int src = __ffsll((long long)who) - 1;
          cut = __builtin_amdgcn_readlane(cut, src);
          above = __builtin_amdgcn_readlane(above, src);
          prefix = (prefix << nb) | (uint32_t)cut;
          k_rem -= above;
          bits_left = shift;
        }
        T = prefix;
        quota = k_rem;
      }
      int count = 0, base_tie = 0;
      for (int t0 = 0; t0 < n; t0 += 64) {
        const int t = t0 + lane;
        const uint32_t k = (t < n) ? score_key(srow[t]) : 0u;
        const bool above = (t < n) && (k > T), tie = (t < n) && (k == T);
        const unsigned long long ma = __ballot(above), mt = __ballot(tie);
        const int pa = count + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(ma >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)ma, 0u));
        const int pt = base_tie + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mt >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mt, 0u));
        if (above || (tie && pt < quota)) {
          const int pos = pa + min(pt, quota);
          if (pos < Kcap) {
            ck[pos] = k;
            ci[pos] = s0 + t;
          }
        }
        count += __popcll(ma);
        base_tie += __popcll(mt);
      }
      count += min(base_tie, quota);
      if (lane == 0) p.cand_cnt[part_base + (size_t)h * p.n_splits] = min(Kcap, count);
      for (int i = count + lane; i < Kcap; i += 64) ck[i] = 0u;
    }
  }
  if (clk && tid == 0) clk[3] = JF_CLK();

  if constexpr (HAS_V) {  // whatever the emission did not carry (no batch of this wavefront, a short split, the exact selection)
    if (!acc_issued) add_acc_range(0, ACC_TOTAL * 4);
    lds_barrier();
  }
  float lfin = 0.f;
  if (tid < G) {
#pragma unroll
    for (int w = 0; w < NW; ++w) lfin += lsum_sh[w][tid];
  }
#pragma unroll
  for (int set = 0; set < NSET; ++set)
    if constexpr (HAS_V) combine(set);
  if (tid < GA) {
    p.part_m[part_base + (size_t)tid * p.n_splits] = m_sh[tid];
    p.part_l[part_base + (size_t)tid * p.n_splits] = lfin;
  }
  if (clk && tid == 0) clk[4] = JF_CLK();
}

// Reductions over one value per wavefront (at most sixteen, in LDS): lane w of the first 16-lane row takes
// wavefront w's value, the row reduces on the DPP network and the result is read from lane 15 -- a handful of
// instructions instead of a loop over the sixteen entries in every thread.  Integer and min/max only: the result
// does not depend on the order.
template <int NWV>
__device__ inline float waves_max_f(const float* arr, int lane) {
  float v = (lane < NWV) ? arr[lane] : -INFINITY;
  JF_DPP_ROW_REDUCE(v, op_fmax, float, -INFINITY);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 15));
}
template <int NWV>
__device__ inline uint32_t waves_max_u(const uint32_t* arr, int lane) {
  uint32_t v = (lane < NWV) ? arr[lane] : 0u;
  JF_DPP_ROW_REDUCE(v, op_umax, uint32_t, 0u);
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 15);
}
template <int NWV>
__device__ inline uint32_t waves_min_u(const uint32_t* arr, int lane) {
  uint32_t v = (lane < NWV) ? arr[lane] : 0xffffffffu;
  JF_DPP_ROW_REDUCE(v, op_umin, uint32_t, 0xffffffffu);
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 15);
}
// sum of the entries before wavefront `wave` (uniform) and of all entries
template <int NWV>
__device__ inline void waves_prefix_i(const int* arr, int lane, int wave, int* before, int* all) {
  const int own = (lane < NWV) ? arr[lane] : 0;
  int v = own;
  JF_DPP_ROW_REDUCE(v, op_iadd, int, 0);  // inclusive scan inside the row
  *before = __builtin_amdgcn_readlane(v - own, wave);
  *all = __builtin_amdgcn_readlane(v, 15);
}

// ---------------------------------------------------------------------------------------------------
constexpr int MG_MAX_SPLITS = 256;
constexpr int MG_BINS = 1024;      // linear score buckets of the threshold search
constexpr int MG_LIST = 1024;      // members of the cut bucket resolved by rank counting
constexpr int MG_BT_LDS = 4096;    // block-table entries cached in LDS (65536 positions)
constexpr int MG_LIGHT_THREADS = 256, MG_LIGHT_REGK = 16, MG_LIGHT_TOPK = 512;  // the light shape of the merge

// Launch 2: one workgroup per (sequence, query head).
//   1. split statistics -> M, l, o_hat
//   2. the K-th largest candidate key tau (and how many keys equal to tau still belong to the top K): the
//      candidates are dropped into MG_BINS linear score buckets between the smallest and the largest, a scan
//      finds the bucket that holds the K-th largest, and the few members of that bucket are ranked against
//      each other (a bisection over the key range covers the case of more than MG_LIST members)
//   3. ordered compaction of the winners (key > tau, or key == tau while the quota lasts; candidates are stored
//      in position order, so ties resolve to the lower position and the output is ascending)
//   4. slots, softmax weights, and the pre-correction terms over the winners' V rows.
// The first MG_REGK * MG_THREADS candidates stay in registers from a single load; anything beyond that is
// re-read from global memory in every pass.
// Two shapes: 1024 threads x 8 register-resident candidates each (up to 8192 candidates, the common case;
// the phases are chains of LDS round trips and barriers, so more, lighter threads beat fewer, heavier ones)
// and 1024 x 32 for first-stage parts that exceed it.
// PARTIAL = true is the first stage of the two-stage merge: blockIdx.z selects a run of mg_spp candidate
// lists, steps 2 and 3 run on those alone and the winners (still in position order) are written out as one
// new candidate list; the final merge (PARTIAL = false, mg_parts > 1) reads these lists instead of the
// scan's.  The top K of a union is the top K of the parts' top K's, ties included: a candidate that a part
// drops is beaten by K candidates of that part.
template <int MODE, int VBITS, int NG, int MG_THREADS, int MG_REGK, bool PARTIAL, bool WIDE = false>
__global__ __launch_bounds__(MG_THREADS) void fused_merge_kernel(FusedParams p) {
  static_assert(!(PARTIAL && MODE == FS_STAGE_B), "Stage B alone selects nothing");
  constexpr int MG_WAVES = MG_THREADS / 64;
  constexpr int VP = D * VBITS / 8;
  // lanes per winner row and codes per lane: a dword of the row each (INT2, INT4), or (INT3, planar) two bytes of
  // each of the three planes = 16 codes
  constexpr int DW = (VBITS == 3) ? 8 : VP / 4;
  constexpr int CPD = (VBITS == 3) ? 16 : 32 / VBITS;
  constexpr int WPI = 64 / DW;          // winners per wavefront instruction
  // The floating-point sums (o_hat over the splits, the pre-correction terms over the winners) are organised
  // as if eight thread groups of 128 and sixteen wavefronts were at work, whatever MG_THREADS is: a smaller
  // workgroup takes several of those roles one after the other, so every shape of this kernel adds the same
  // numbers in the same order and the results do not depend on which shape the launcher picks.
  constexpr int VGRP = 8, VWAVES = 16;
  static_assert(MG_THREADS % D == 0 && VGRP % (MG_THREADS / D) == 0 && VWAVES % MG_WAVES == 0, "whole roles per thread group / wavefront");
  // the light shape (many rows per launch, few candidates per row) trades table sizes for workgroups per CU
  constexpr int MG_BT = (MG_THREADS >= 1024) ? MG_BT_LDS : 1024;  // block-table entries cached in LDS
  constexpr int MG_WIN = (MG_THREADS >= 1024) ? FS_LDS_TOPK : 512;  // widest correction of this shape (WIDE: any)
  __shared__ int hist[MG_BINS];
  __shared__ uint32_t lkey[MG_LIST];
  __shared__ float coef_sh[MG_MAX_SPLITS];
  __shared__ int cnt_sh[MG_MAX_SPLITS];
  __shared__ int bt_sh[MG_BT];
  // winners: key and position while they are selected; the thread that turns winner r into its softmax weight and
  // paged slot overwrites the two entries in place (weight bits over the key, slot over the position)
  // (WIDE, corrections beyond FS_LDS_TOPK: the two arrays are the launch's dynamic LDS, top_k entries each)
  __shared__ uint32_t win_key_s[WIDE ? 1 : MG_WIN];
  __shared__ int win_idx_s[WIDE ? 1 : MG_WIN];
  extern __shared__ __align__(16) uint32_t win_dyn[];
  uint32_t* const win_key = WIDE ? win_dyn : win_key_s;
  int* const win_idx = WIDE ? reinterpret_cast<int*>(win_dyn + p.top_k) : win_idx_s;
  __shared__ uint32_t cnt_a[MG_REGK / 4 * MG_WAVES];  // packed (winners, ties) per (group, wavefront)
  __shared__ float red_sh[VGRP][D];
  __shared__ float old_sh[VWAVES][D];
  __shared__ float w_sh[VWAVES];
  __shared__ float wred_f[MG_WAVES];
  __shared__ uint32_t wred_u[MG_WAVES], wred_k[MG_WAVES];
  __shared__ float wred_g[MG_WAVES];
  __shared__ int wred_i[MG_WAVES], wred_j[MG_WAVES];
  __shared__ int lcount_sh, cut_sh, above_sh, quota_sh;
  __shared__ uint32_t tau_sh;

  const int b = blockIdx.x, hq = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const size_t bh = (size_t)b * p.H_q + hq;
  const int NS = p.n_splits, K = p.top_k;
  const int hkv = hq / (p.H_q / p.H_kv);
  // candidate lists of this workgroup: NL lists of capacity Kc
  const bool staged = !PARTIAL && p.mg_parts > 1;
  const int part = PARTIAL ? (int)blockIdx.z : 0;
  const int l0 = PARTIAL ? part * p.mg_spp : 0;
  // (Stage B alone: the winners are an input, there are no candidate lists)
  const int NL = (MODE == FS_STAGE_B) ? 0 : (PARTIAL ? min(p.mg_spp, NS - l0) : (staged ? p.mg_parts : NS));
  const int Kc = staged ? K : p.Kc;
  const uint32_t* ck = staged ? p.key2 + bh * p.mg_parts * K : p.cand_key + (bh * NS + l0) * Kc;
  const int32_t* ci = staged ? p.idx2 + bh * p.mg_parts * K : p.cand_idx + (bh * NS + l0) * Kc;
  const int32_t* cc = staged ? p.cnt2 + bh * p.mg_parts : p.cand_cnt + bh * NS + l0;
  const int64_t* bt = p.block_table + (size_t)b * p.max_blocks;
  int64_t* out_idx = p.topk_idx + bh * (size_t)K;
  int64_t* out_slot = p.topk_slots + bh * (size_t)K;
  const int flat = NL * Kc;
  const int rounds = (flat + MG_THREADS - 1) / MG_THREADS;
  const int nblk_lds = min(p.max_blocks, MG_BT);

  long long* mclk = (kDebugHooks && p.phase_clock && !PARTIAL) ? p.phase_clock + (size_t)p.B * p.H_kv * p.n_splits * 10 + bh * 8 : nullptr;
  if (mclk && tid == 0) mclk[0] = JF_CLK();

  // ---- everything that does not depend on anything else is requested first, in the order of its use.  Every load
  // is unconditional, on a clamped index, and its mask is applied further down: under a condition the compiler waits
  // for a load inside its branch, and these loads (first touches of what other XCDs wrote) would cost one round trip
  // after the other instead of one for all.
  constexpr bool HAS_LISTS = (MODE != FS_STAGE_B);
  float pm = -INFINITY, pl = 0.f;
  int my_cnt = 0;
  // (given statistics, jf_stage_b_softmax_v: no partial results at all, NS = 0 and the pointers are null; those
  // loads then read the page table, which every caller of this kernel passes, and every one of them is masked)
  const bool has_parts = NS > 0;
  const float* dummy_f = reinterpret_cast<const float*>(bt);
  // The first MG_REGK * MG_THREADS candidates live in registers: group g = r / 4 of a thread holds the four
  // consecutive candidates (g * MG_THREADS + tid) * 4 + (r % 4), fetched with one 16-byte load.  Candidate
  // order = (group, thread, element).  Slots past a list's count hold key 0 (written by the producer).
  static_assert(MG_REGK % 4 == 0, "register candidates come in groups of four");
  constexpr int NGRP = MG_REGK / 4;
  const int rreg = min((flat + 4 * MG_THREADS - 1) / (4 * MG_THREADS), NGRP) * 4;  // register slots in use (uniform)
  uint32_t kreg[MG_REGK];
  int ireg[MG_REGK];
  v4u k4[NGRP];
  v4i i4[NGRP];
  // what the first barrier interval needs goes first (loads return in order): the split maxima, the list counts,
  // the candidate keys
  if constexpr (!PARTIAL) pm = *(has_parts ? p.part_m + bh * NS + min(tid, NS - 1) : dummy_f);
  if constexpr (HAS_LISTS) my_cnt = cc[min(tid, NL - 1)];
#pragma unroll
  for (int g = 0; g < NGRP; ++g) {
    k4[g] = (v4u){0u, 0u, 0u, 0u};
    if constexpr (HAS_LISTS)  // (flat is a multiple of 4; groups past the end are not requested)
      if (g == 0 || 4 * g < rreg) k4[g] = *reinterpret_cast<const v4u*>(ck + min((g * MG_THREADS + tid) * 4, flat - 4));
  }
  if constexpr (!PARTIAL) pl = *(has_parts ? p.part_l + bh * NS + min(tid, NS - 1) : dummy_f);
#pragma unroll
  for (int g = 0; g < NGRP; ++g) {
    i4[g] = (v4i){0, 0, 0, 0};
    if constexpr (HAS_LISTS)
      if (g == 0 || 4 * g < rreg) i4[g] = *reinterpret_cast<const v4i*>(ci + min((g * MG_THREADS + tid) * 4, flat - 4));
  }
  uint16_t blend_raw = 0;
  float blend_new = 0.f, blend_hat = 0.f;
  if constexpr (MODE == FS_FULL && !PARTIAL)  // (no blend: any readable address)
    blend_raw = *(p.blend_out ? p.blend_o_new + bh * D + (tid & (D - 1)) : reinterpret_cast<const uint16_t*>(ck));
  // o_hat: the thread groups of 128 take the splits round-robin (first terms requested now)
  constexpr int PO_PRE = 2, PO_GRP = MG_THREADS / D;
  float po[PO_PRE];
  {
    const int d = tid & (D - 1), q4 = tid >> 7;
#pragma unroll
    for (int i = 0; i < PO_PRE; ++i) {
      po[i] = 0.f;
      if constexpr (MODE != FS_STAGE_A && !PARTIAL)
        po[i] = *(has_parts ? p.part_o + (bh * NS + min(q4 + VGRP * i, NS - 1)) * D + d : dummy_f);
    }
  }
  // page-table entries for the table in LDS: stored after the first barrier, so that the wait for them (the
  // youngest loads) is not part of the first interval
  constexpr int BTPT = (MG_BT + MG_THREADS - 1) / MG_THREADS;
  int bt_mine[BTPT];
#pragma unroll
  for (int i = 0; i < BTPT; ++i) {
    bt_mine[i] = 0;
    // (the low half of the 64-bit entry only: the unused half of a wider load is a register the compiler hands out
    // again at once, and writing it has to wait for the load)
    if constexpr (!PARTIAL) bt_mine[i] = reinterpret_cast<const int*>(bt)[2 * min(tid + i * MG_THREADS, p.max_blocks - 1)];
  }
  for (int i = tid; i < MG_BINS; i += MG_THREADS) hist[i] = 0;
  if (tid == 0) lcount_sh = 0;
  // the masks of the loads the first interval uses (the others follow its barrier)
  if (tid >= NS) pm = -INFINITY;
  if (tid >= NL) my_cnt = 0;
#pragma unroll
  for (int g = 0; g < NGRP; ++g) {
    const bool in = (g * MG_THREADS + tid) * 4 < flat;
#pragma unroll
    for (int j = 0; j < 4; ++j) kreg[4 * g + j] = in ? k4[g][j] : 0u;
  }
  if (tid < NL) cnt_sh[tid] = my_cnt;

  // key of candidate f in pass-over-all-candidates loops: registers first, global memory beyond
  auto key_of = [&](int r) -> uint32_t {
    const int f = r * MG_THREADS + tid;
    return (f < flat) ? ck[f] : 0u;
  };
  // number of candidates with key >= x (x > 0), identical in every thread
  auto count_ge = [&](uint32_t x) -> int {
    int c = 0;
#pragma unroll
    for (int r = 0; r < MG_REGK; ++r)
      if (r < rreg) c += __popcll(__builtin_amdgcn_ballot_w64(kreg[r] >= x));
    for (int r = MG_REGK; r < rounds; ++r) c += __popcll(__builtin_amdgcn_ballot_w64(key_of(r) >= x));
    lds_barrier();
    if (lane == 0) wred_i[wave] = c;
    lds_barrier();
    int before, t;
    waves_prefix_i<MG_WAVES>(wred_i, lane, 0, &before, &t);
    return t;
  };

  // The split statistics (M, coefficients e^{m_i - M}, l, o_hat) and the threshold search (range of the candidate
  // keys, bucket histogram, bucket scan) do not depend on each other: their steps share the barrier intervals.
  // ---- interval 1: per-wavefront maximum of the split maxima and range of the candidate keys
  if (!PARTIAL) {
    const float v = wave_max(pm);
    if (lane == 0) wred_f[wave] = v;
  }
  uint32_t kmin = 0xffffffffu, kmax = 0u;
#pragma unroll
  for (int r = 0; r < MG_REGK; ++r)
    if (r < rreg && kreg[r] != 0u) { kmin = min(kmin, kreg[r]); kmax = max(kmax, kreg[r]); }
  for (int r = MG_REGK; r < rounds; ++r) {
    const uint32_t k = key_of(r);
    if (k != 0u) { kmin = min(kmin, k); kmax = max(kmax, k); }
  }
  kmin = wave_min_u(kmin);
  kmax = wave_max_u(kmax);
  if (lane == 0) { wred_u[wave] = kmin; wred_k[wave] = kmax; }
  lds_barrier();
  if (mclk && tid == 0) mclk[6] = JF_CLK();
  if (tid >= NS) pl = 0.f;
  if (MODE == FS_FULL && !PARTIAL && p.blend_out && tid < D) blend_new = bf16_to_f32(blend_raw);
#pragma unroll
  for (int g = 0; g < NGRP; ++g) {
    const bool in = (g * MG_THREADS + tid) * 4 < flat;
#pragma unroll
    for (int j = 0; j < 4; ++j) ireg[4 * g + j] = in ? i4[g][j] : 0;
  }
  if constexpr (!PARTIAL) {  // (first read long after the next barrier)
#pragma unroll
    for (int i = 0; i < BTPT; ++i)
      if (tid + i * MG_THREADS < nblk_lds) bt_sh[tid + i * MG_THREADS] = bt_mine[i];
  }
  // ---- interval 2: M, the coefficients, per-wavefront sums of l; the candidates drop into MG_BINS linear buckets
  float M = -INFINITY;
  if (!PARTIAL) {
    M = waves_max_f<MG_WAVES>(wred_f, lane);
    if (!isfinite(M)) M = 0.f;
    const float coef = (pm == -INFINITY) ? 0.f : __expf(pm - M);
    if (tid < NS) coef_sh[tid] = coef;
    const float v = wave_sum(pl * coef);  // fixed reduction tree: deterministic
    if (lane == 0) wred_g[wave] = v;
  }
  int total = 0;
  for (int s2 = 0; s2 < NL; ++s2) total += cnt_sh[s2];
  kmin = waves_min_u<MG_WAVES>(wred_u, lane);
  kmax = waves_max_u<MG_WAVES>(wred_k, lane);
  const float hi = key_to_score(kmax), lo = key_to_score(kmin);
  const float range = hi - lo;
  const float iw = (range > 0.f && isfinite(range)) ? ((float)MG_BINS - 0.01f) / range : 0.f;
  const float ba = -iw, bb = isfinite(hi) ? hi * iw : 0.f;
  auto bin_of = [&](uint32_t k) -> int {
    return (int)__builtin_amdgcn_fmed3f(__builtin_fmaf(key_to_score(k), ba, bb), 0.f, (float)(MG_BINS - 1));
  };
  const bool take_all = (total <= K);  // (uniform) every candidate wins: no threshold
  if (!take_all) {
#pragma unroll
    for (int r = 0; r < MG_REGK; ++r)
      if (r < rreg && kreg[r] != 0u) atomicAdd(&hist[bin_of(kreg[r])], 1);
    for (int r = MG_REGK; r < rounds; ++r) {
      const uint32_t k = key_of(r);
      if (k != 0u) atomicAdd(&hist[bin_of(k)], 1);
    }
  }
  lds_barrier();
  if (mclk && tid == 0) mclk[7] = JF_CLK();
  // ---- interval 3: 1/l, the partial sums of o_hat; first half of the bucket scan
  float inv_z = 0.f;
  if (!PARTIAL) {
    float lsum = 0.f;
#pragma unroll
    for (int w = 0; w < MG_WAVES; ++w) lsum += wred_g[w];
    inv_z = (lsum > 0.f) ? 1.0f / lsum : 0.f;
    if (tid == 0 && p.softmax_m) {
      p.softmax_m[bh] = M;
      p.softmax_inv_z[bh] = inv_z;
    }
  }
  if constexpr (MODE == FS_STAGE_B) {
    if (p.stats_m) {  // (uniform) the caller's statistics
      M = p.stats_m[bh];
      inv_z = p.stats_iz[bh];
    }
  }
  // thread t owns buckets BPT*t .. BPT*t + BPT-1 (bucket 0 = largest scores): which bucket holds the K-th largest
  constexpr int BPT = MG_BINS / MG_THREADS;
  int cb[BPT], mine = 0;
#pragma unroll
  for (int u = 0; u < BPT; ++u) {
    cb[u] = hist[BPT * tid + u];
    mine += cb[u];
  }
  const int incl = wave_incl_scan_i(mine);
  if (lane == 63) wred_j[wave] = incl;
  if constexpr (!PARTIAL && MODE != FS_STAGE_A) {
    // o_hat: group vg of the eight takes every eighth split, then a fixed-order sum
    const int d = tid & (D - 1), q4 = tid >> 7;
    for (int vg = q4; vg < VGRP; vg += PO_GRP) {
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < PO_PRE; ++i) {
        const int sp = vg + VGRP * i;
        if (sp < NS) o = __builtin_fmaf((vg == q4) ? po[i] : p.part_o[(bh * NS + sp) * D + d], coef_sh[sp], o);
      }
      // the remaining splits eight at a time: the loads of a batch are in flight together, the sum keeps its order
      constexpr int PO_B = 8;
      for (int sp0 = vg + VGRP * PO_PRE; sp0 < NS; sp0 += VGRP * PO_B) {
        float v[PO_B];
#pragma unroll
        for (int u = 0; u < PO_B; ++u) {
          const int sp = sp0 + VGRP * u;
          v[u] = (sp < NS) ? p.part_o[(bh * NS + sp) * D + d] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < PO_B; ++u) {
          const int sp = sp0 + VGRP * u;
          if (sp < NS) o = __builtin_fmaf(v[u], coef_sh[sp], o);
        }
      }
      red_sh[vg][d] = o;
    }
  }
  lds_barrier();
  // ---- interval 4: o_hat; the bucket of the K-th largest candidate
  if constexpr (!PARTIAL && MODE != FS_STAGE_A) {
    if (tid < D) {
      float o2 = red_sh[0][tid];
#pragma unroll
      for (int q = 1; q < VGRP; ++q) o2 += red_sh[q][tid];  // fixed order
      blend_hat = o2 * inv_z;
      if (MODE != FS_STAGE_B || p.o_hat) p.o_hat[bh * D + tid] = blend_hat;
    }
  }
  if (mclk && tid == 0) mclk[1] = JF_CLK();

  uint32_t tau = 0;
  int quota = 0;
  if (!take_all) {
    {
      int run, all_waves;
      waves_prefix_i<MG_WAVES>(wred_j, lane, wave, &run, &all_waves);
      run += incl - mine;
#pragma unroll
      for (int u = 0; u < BPT; ++u) {
        if (run < K && K <= run + cb[u]) { cut_sh = BPT * tid + u; above_sh = run; }
        run += cb[u];
      }
    }
    lds_barrier();
    const int cut = cut_sh, need = K - above_sh;  // `need` of the cut bucket's members belong to the top K
#pragma unroll
    for (int r = 0; r < MG_REGK; ++r)
      if (r < rreg && kreg[r] != 0u && bin_of(kreg[r]) == cut) {
        const int i = atomicAdd(&lcount_sh, 1);
        if (i < MG_LIST) lkey[i] = kreg[r];
      }
    for (int r = MG_REGK; r < rounds; ++r) {
      const uint32_t k = key_of(r);
      if (k != 0u && bin_of(k) == cut) {
        const int i = atomicAdd(&lcount_sh, 1);
        if (i < MG_LIST) lkey[i] = k;
      }
    }
    lds_barrier();
    const int m = lcount_sh;
    if (m <= MG_LIST) {
      // rank counting: the member with fewer than `need` larger members and at least `need` members >= it
      for (int i = tid; i < m; i += MG_THREADS) {
        const uint32_t k = lkey[i];
        int gt = 0, ge = 0;
        for (int j = 0; j < m; ++j) {
          const uint32_t o = lkey[j];
          gt += (o > k) ? 1 : 0;
          ge += (o >= k) ? 1 : 0;
        }
        if (gt < need && need <= ge) {  // every thread that gets here writes the same pair
          tau_sh = k;
          quota_sh = need - gt;
        }
      }
      lds_barrier();
      tau = tau_sh;
      quota = quota_sh;
    } else {
      // bisection over the key range: largest x with count(key >= x) >= K
      uint32_t lo_k = kmin, hi_k = kmax;  // invariant: count_ge(lo_k) >= K
      while (lo_k < hi_k) {
        const uint32_t mid = lo_k + (hi_k - lo_k + 1u) / 2u;
        if (count_ge(mid) >= K) lo_k = mid;
        else hi_k = mid - 1u;
      }
      tau = lo_k;
      quota = K - ((tau == 0xffffffffu) ? 0 : count_ge(tau + 1u));
    }
  }
  if (mclk && tid == 0) mclk[2] = JF_CLK();

  // ---- ordered compaction.  Register candidates: every thread counts its winners and ties per group, a
  // wavefront scan plus the wavefront totals in LDS give the thread's first place, and the thread places its
  // (consecutive) candidates one after the other.  The owner of a winner stores its key and position.
  int base_above = 0, base_tie = 0;
  {
    int cnt_g[NGRP];  // low half: winners, high half: ties of this thread in group g
    int scan_g[NGRP];
#pragma unroll
    for (int g = 0; g < NGRP; ++g) {
      int c = 0;
      if (4 * g < rreg) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t key = kreg[4 * g + j];
          const bool above = (key != 0u) && (take_all || key > tau), tie = (key != 0u) && !take_all && key == tau;
          c += (above ? 1 : 0) + (tie ? 0x10000 : 0);
        }
      }
      cnt_g[g] = c;
      scan_g[g] = wave_incl_scan_i(c);  // at most 4 * 64 per half: no carry between the halves
      if (lane == 63) cnt_a[g * MG_WAVES + wave] = (uint32_t)scan_g[g];
    }
    lds_barrier();
    uint32_t run = 0u;  // packed totals of the groups before g (each half stays below 2^16: at most 32768 candidates)
#pragma unroll
    for (int g = 0; g < NGRP; ++g) {
      int before_i, all_i;  // (packed pairs: each half stays below 2^16, so the halves never carry into each other)
      waves_prefix_i<MG_WAVES>(reinterpret_cast<const int*>(cnt_a) + g * MG_WAVES, lane, wave, &before_i, &all_i);
      const uint32_t before = (uint32_t)before_i, all = (uint32_t)all_i;
      if (4 * g < rreg) {
        const uint32_t start = run + before + (uint32_t)(scan_g[g] - cnt_g[g]);
        int pa = (int)(start & 0xffffu), pt = (int)(start >> 16);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t key = kreg[4 * g + j];
          const bool above = (key != 0u) && (take_all || key > tau), tie = (key != 0u) && !take_all && key == tau;
          if (above || (tie && pt < quota)) {
            const int pos = pa + min(pt, quota);
            if (pos < K) {
              win_key[pos] = key;
              win_idx[pos] = ireg[4 * g + j];
            }
          }
          pa += above ? 1 : 0;
          pt += tie ? 1 : 0;
        }
      }
      run += all;
    }
    base_above = (int)(run & 0xffffu);
    base_tie = (int)(run >> 16);
    lds_barrier();
  }
  for (int r = MG_REGK; r < rounds; ++r) {  // candidates beyond the register-resident ones, one round at a time
    const int f = r * MG_THREADS + tid;
    const uint32_t key = key_of(r);
    const bool above = (key != 0u) && (take_all || key > tau), tie = (key != 0u) && !take_all && key == tau;
    const unsigned long long ma = __builtin_amdgcn_ballot_w64(above), mt = __builtin_amdgcn_ballot_w64(tie);
    if (lane == 0) {
      wred_i[wave] = __popcll(ma);
      wred_j[wave] = __popcll(mt);
    }
    lds_barrier();
    int pa = base_above + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(ma >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)ma, 0u));
    int pt = base_tie + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mt >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mt, 0u));
    int tot_a = 0, tot_t = 0;
#pragma unroll
    for (int w = 0; w < MG_WAVES; ++w) {
      if (w < wave) { pa += wred_i[w]; pt += wred_j[w]; }
      tot_a += wred_i[w];
      tot_t += wred_j[w];
    }
    if (above || (tie && pt < quota)) {
      const int pos = pa + min(pt, quota);
      if (pos < K) {
        win_key[pos] = key;
        win_idx[pos] = ci[f];
      }
    }
    base_above += tot_a;
    base_tie += tot_t;
    lds_barrier();
  }
  int n_out = min(K, base_above + min(base_tie, quota));
  if constexpr (MODE == FS_STAGE_B) {
    // the winners are given (ascending positions, -1 padded, possibly none at all): their keys come from the
    // caller's score tensor
    n_out = p.topk_idx ? K : 0;
    const int64_t s_len = max(0, min(p.max_S, p.seq_lens[b]));
    for (int r = tid; r < n_out; r += MG_THREADS) {
      const int64_t pos = p.topk_idx[bh * (size_t)K + r];
      const bool ok = pos >= 0 && pos < s_len;
      win_idx[r] = ok ? (int)pos : -1;
      win_key[r] = ok ? score_key(p.scores_in[bh * (size_t)p.max_S + pos]) : 0u;
    }
    lds_barrier();
  }
  if (mclk && tid == 0) mclk[3] = JF_CLK();
  if (PARTIAL) {  // the winners become one candidate list of the final merge
    const size_t lo = (bh * p.mg_parts + part) * (size_t)K;
    for (int r = tid; r < K; r += MG_THREADS) {
      p.key2[lo + r] = (r < n_out) ? win_key[r] : 0u;  // unused slots: key 0
      if (r < n_out) p.idx2[lo + r] = win_idx[r];
    }
    if (tid == 0) p.cnt2[bh * p.mg_parts + part] = n_out;
    return;
  }

  // one thread per winner: position, paged slot, softmax weight
  for (int r = tid; r < K; r += MG_THREADS) {
    int64_t position = -1, slot = -1;
    int wslot = -1;
    float ww = 0.f;
    if (r < n_out && win_idx[r] >= 0) {
      position = win_idx[r];
      const int blk = (int)(position / BS);
      if (blk < p.max_blocks) slot = (int64_t)((blk < nblk_lds) ? (int64_t)bt_sh[blk] : bt[blk]) * BS + (position % BS);
      wslot = (slot >= 0 && slot < p.num_slots) ? (int)slot : -1;
      ww = __expf(key_to_score(win_key[r]) - M) * inv_z;
    }
    if constexpr (MODE != FS_STAGE_B) {
      out_idx[r] = position;
      out_slot[r] = slot;
    }
    win_idx[r] = wslot;
    win_key[r] = __builtin_bit_cast(uint32_t, ww);
  }
  if constexpr (MODE == FS_STAGE_A) return;  // Stage A alone ends with the winners and the statistics
  lds_barrier();
  if (mclk && tid == 0) mclk[4] = JF_CLK();

  // ---- pre-correction over the winners.  One winner row per DW lanes: lane (w_in, dwi) holds dword dwi of
  // the winner's packed V row (CPD codes) and accumulates its CPD channels; winners are visited in a fixed
  // order, so the sums are run-to-run deterministic.  UNR rows per lane are requested before any is used.
  const uint8_t* vbase = p.v_data + (size_t)hkv * p.num_slots * VP;
  const uint8_t* vsbase = reinterpret_cast<const uint8_t*>(p.v_scales + (size_t)hkv * p.num_slots * NG);
  const int dwi = lane % DW, w_in = lane / DW;
  const int g_of_lane = (NG == 1) ? 0 : ((dwi * CPD) / (D / NG));
  constexpr int UNR = (256 / (VWAVES * WPI) > 0) ? 256 / (VWAVES * WPI) : 1;  // 256 winners per pass
  for (int vw = wave; vw < VWAVES; vw += MG_WAVES) {  // (one turn unless the workgroup has fewer than sixteen wavefronts)
  float acc[CPD];
#pragma unroll
  for (int c = 0; c < CPD; ++c) acc[c] = 0.f;
  float accw = 0.f;
  for (int k0 = vw * WPI; k0 < n_out; k0 += UNR * VWAVES * WPI) {
    uint32_t word[UNR], word_b[UNR];  // (word_b: INT3 only)
    uint16_t sbits[UNR];
    float wv[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int k = k0 + u * VWAVES * WPI + w_in;
      const int slot = (k < n_out) ? win_idx[k] : -1;
      wv[u] = (slot >= 0) ? __builtin_bit_cast(float, win_key[k]) : 0.f;
      const uint32_t sl = (uint32_t)max(slot, 0);
      if constexpr (VBITS == 3) {  // bytes 2*dwi, 2*dwi+1 of every plane -> the 24-bit words of two 8-code groups
        const uint8_t* row = vbase + (size_t)(sl * (uint32_t)VP) + dwi * 2;
        const uint32_t h0 = *reinterpret_cast<const uint16_t*>(row), h1 = *reinterpret_cast<const uint16_t*>(row + 16),
                       h2 = *reinterpret_cast<const uint16_t*>(row + 32);
        word[u] = ((h0 & 0xffu) << 16) | ((h1 & 0xffu) << 8) | (h2 & 0xffu);
        word_b[u] = ((h0 >> 8) << 16) | ((h1 >> 8) << 8) | (h2 >> 8);
      } else {
        word[u] = *reinterpret_cast<const uint32_t*>(vbase + (size_t)(sl * (uint32_t)VP) + dwi * 4);
        word_b[u] = 0;
      }
      sbits[u] = *reinterpret_cast<const uint16_t*>(vsbase + (size_t)(sl * (uint32_t)(NG * 2)) + g_of_lane * 2);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const float ws = wv[u] * bf16_to_f32(sbits[u]);  // zero for padding rows
      // byte `byte` of the dword holds its codes MSB first; channel of code c in the dword = dwi*CPD + c.
      // code - VOFF is the code with its top bit flipped, read as a two's complement field: one signed bit-field
      // extract per code after one exclusive-or per word.
      constexpr uint32_t FLIP = (VBITS == 3) ? 0x00924924u : ((VBITS == 2) ? 0xaaaaaaaau : 0x88888888u);
      const uint32_t xa = word[u] ^ FLIP, xb = word_b[u] ^ FLIP;
#pragma unroll
      for (int c = 0; c < CPD; ++c) {
        int sh;
        if constexpr (VBITS == 3) {
          sh = 21 - 3 * (c & 7);
        } else {
          const int byte = c / (8 / VBITS), inb = c % (8 / VBITS);
          sh = 8 * byte + (8 - VBITS * (inb + 1));
        }
        const uint32_t x = (VBITS == 3 && c >= 8) ? xb : xa;
        const int code = (int)(x << (32 - VBITS - sh)) >> (32 - VBITS);
        acc[c] = __builtin_fmaf(ws, (float)code, acc[c]);
      }
      if (dwi == 0) accw += wv[u];
    }
  }
  // reduce over the WPI winners of a wavefront instruction (lanes with equal dwi): every exchange step halves
  // the channels a lane is responsible for (the lane whose offset bit is clear keeps the lower half), so after
  // log2(WPI) steps every lane holds the sums of CPD / WPI = 2 channels; then over wavefronts through LDS
  {
    int chan = dwi * CPD;
    auto halve = [&](auto off_c, auto n_c) {
      constexpr int OFF = decltype(off_c)::value, N = decltype(n_c)::value;
      const bool upper = (lane & OFF) != 0;
#pragma unroll
      for (int i = 0; i < N / 2; ++i) {
        if constexpr (OFF == 32) {  // one half-wave swap serves both directions
          const auto sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, acc[i]), __builtin_bit_cast(uint32_t, acc[i + N / 2]), false, false);
          acc[i] = __builtin_bit_cast(float, (uint32_t)sw[0]) + __builtin_bit_cast(float, (uint32_t)sw[1]);
        } else {
          const float keep = upper ? acc[i + N / 2] : acc[i];
          const int send = __builtin_bit_cast(int, upper ? acc[i] : acc[i + N / 2]);
          // lane ^ 8: rotation by 8 inside the 16-lane row; lane ^ 16: swizzle inside 32 lanes
          const int recv = (OFF == 8) ? dpp_mov<0x128, 0xf>(0, send) : __builtin_amdgcn_ds_swizzle(send, 0x401F);
          acc[i] = keep + __builtin_bit_cast(float, recv);
        }
      }
      chan += upper ? N / 2 : 0;
    };
    static_assert(DW == 8 || DW == 16, "eight or sixteen lanes per V row");
    if constexpr (DW == 8) {
      halve(std::integral_constant<int, 8>{}, std::integral_constant<int, CPD>{});
      halve(std::integral_constant<int, 16>{}, std::integral_constant<int, CPD / 2>{});
      halve(std::integral_constant<int, 32>{}, std::integral_constant<int, CPD / 4>{});
    } else {
      halve(std::integral_constant<int, 16>{}, std::integral_constant<int, CPD>{});
      halve(std::integral_constant<int, 32>{}, std::integral_constant<int, CPD / 2>{});
    }
    static_assert(CPD / WPI == 2, "two channels per lane after the exchange");
    old_sh[vw][chan] = acc[0];
    old_sh[vw][chan + 1] = acc[1];
    const float wsum = wave_sum(accw);  // only the dwi == 0 lanes hold weights
    if (lane == 0) w_sh[vw] = wsum;
  }
  }
  lds_barrier();
  if (tid < D) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < VWAVES; ++w) o += old_sh[w][tid];  // fixed order
    p.o_old[bh * D + tid] = o;
    float wt = 0.f;
#pragma unroll
    for (int w = 0; w < VWAVES; ++w) wt += w_sh[w];  // fixed order: the same value in every thread
    if (tid == 0) p.W[bh] = wt;
    // the blend of jetfire_vllm/csrc/blend.cu:202-226 for callers that hold o_new already
    if (MODE == FS_FULL && p.blend_out) p.blend_out[bh * D + tid] = f32_to_bf16(__builtin_fmaf(wt, blend_new, blend_hat) - o);
  }
  if (mclk && tid == 0) mclk[5] = JF_CLK();
}

constexpr size_t LDS_BUDGET_2WG = 80 * 1024 - 512;    // two workgroups per CU (160 KB LDS)
constexpr size_t LDS_BUDGET_1WG = 160 * 1024 - 1024;

template <int SCHEME, int G, int NG>
int lmax_for() {
  using Lds = ScanLds<SCHEME, G, NG>;
  const size_t budget = (G <= 4 && Lds::NW == 8) ? LDS_BUDGET_2WG : LDS_BUDGET_1WG;
  const size_t fixed = Lds::AUX + Lds::stage_bytes() + 64 + 832 + (Lds::KB4 ? 1536 : (Lds::K3 ? 512 : 0));  // + static LDS of the kernel (incl. the rounding tables)
  long lm = (long)((budget - fixed) / (Lds::per_position() + 1));  // +1: page table (4 bytes per 16 positions)
  lm = lm / 256 * 256;
  if (lm > Lds::LMAX) lm = Lds::LMAX;
  if (lm < 256) lm = 256;
  return (int)lm;
}

inline int lmax_dispatch(int scheme, int G, int NG) {
#define JF_LMAX_CASE(SCH, GG, NGG) if (scheme == SCH && G == GG && NG == NGG) return lmax_for<SCH, GG, NGG>()
  JF_LMAX_CASE(JF_SCHEME_K3V2, 1, 1); JF_LMAX_CASE(JF_SCHEME_K3V2, 2, 1); JF_LMAX_CASE(JF_SCHEME_K3V2, 4, 1);
  JF_LMAX_CASE(JF_SCHEME_K3V2, 8, 1); JF_LMAX_CASE(JF_SCHEME_K3V2, 16, 1);
  JF_LMAX_CASE(JF_SCHEME_K3V2, 1, 2); JF_LMAX_CASE(JF_SCHEME_K3V2, 2, 2); JF_LMAX_CASE(JF_SCHEME_K3V2, 4, 2);
  JF_LMAX_CASE(JF_SCHEME_K3V2, 8, 2); JF_LMAX_CASE(JF_SCHEME_K3V2, 16, 2);
  JF_LMAX_CASE(JF_SCHEME_K4V4, 1, 1); JF_LMAX_CASE(JF_SCHEME_K4V4, 2, 1); JF_LMAX_CASE(JF_SCHEME_K4V4, 4, 1);
  JF_LMAX_CASE(JF_SCHEME_K4V4, 8, 1); JF_LMAX_CASE(JF_SCHEME_K4V4, 16, 1);
  JF_LMAX_CASE(JF_SCHEME_K3V4, 1, 1); JF_LMAX_CASE(JF_SCHEME_K3V4, 2, 1); JF_LMAX_CASE(JF_SCHEME_K3V4, 4, 1);
  JF_LMAX_CASE(JF_SCHEME_K3V4, 8, 1); JF_LMAX_CASE(JF_SCHEME_K3V4, 16, 1);
  JF_LMAX_CASE(JF_SCHEME_K4V2, 1, 1); JF_LMAX_CASE(JF_SCHEME_K4V2, 2, 1); JF_LMAX_CASE(JF_SCHEME_K4V2, 4, 1);
  JF_LMAX_CASE(JF_SCHEME_K4V2, 8, 1); JF_LMAX_CASE(JF_SCHEME_K4V2, 16, 1);
  JF_LMAX_CASE(JF_SCHEME_K2V2, 1, 1); JF_LMAX_CASE(JF_SCHEME_K2V2, 2, 1); JF_LMAX_CASE(JF_SCHEME_K2V2, 4, 1);
  JF_LMAX_CASE(JF_SCHEME_K2V2, 8, 1); JF_LMAX_CASE(JF_SCHEME_K2V2, 16, 1);
  JF_LMAX_CASE(JF_SCHEME_K2V2, 1, 2); JF_LMAX_CASE(JF_SCHEME_K2V2, 2, 2); JF_LMAX_CASE(JF_SCHEME_K2V2, 4, 2);
  JF_LMAX_CASE(JF_SCHEME_K2V2, 8, 2); JF_LMAX_CASE(JF_SCHEME_K2V2, 16, 2);
  JF_LMAX_CASE(JF_SCHEME_K2V4, 1, 1); JF_LMAX_CASE(JF_SCHEME_K2V4, 2, 1); JF_LMAX_CASE(JF_SCHEME_K2V4, 4, 1);
  JF_LMAX_CASE(JF_SCHEME_K2V4, 8, 1); JF_LMAX_CASE(JF_SCHEME_K2V4, 16, 1);
#define JF_LMAX_ALL_G(SCH, NGG)                                                                      \
  JF_LMAX_CASE(SCH, 1, NGG); JF_LMAX_CASE(SCH, 2, NGG); JF_LMAX_CASE(SCH, 4, NGG); JF_LMAX_CASE(SCH, 8, NGG); \
  JF_LMAX_CASE(SCH, 16, NGG)
  JF_LMAX_ALL_G(JF_SCHEME_K2V3, 1); JF_LMAX_ALL_G(JF_SCHEME_K2V3, 2);
  JF_LMAX_ALL_G(JF_SCHEME_K3V3, 1); JF_LMAX_ALL_G(JF_SCHEME_K3V3, 2);
  JF_LMAX_ALL_G(JF_SCHEME_K4V3, 1);
  JF_LMAX_ALL_G(JF_SCHEME_A2V2, 1); JF_LMAX_ALL_G(JF_SCHEME_A2V2, 2);
  JF_LMAX_ALL_G(JF_SCHEME_A2V3, 1); JF_LMAX_ALL_G(JF_SCHEME_A2V3, 2);
  JF_LMAX_ALL_G(JF_SCHEME_A2V4, 1);
  JF_LMAX_ALL_G(JF_SCHEME_K3V4, 2); JF_LMAX_ALL_G(JF_SCHEME_K2V4, 2); JF_LMAX_ALL_G(JF_SCHEME_A2V4, 2);
  JF_LMAX_ALL_G(JF_SCHEME_B4V2, 1); JF_LMAX_ALL_G(JF_SCHEME_B4V2, 2); JF_LMAX_ALL_G(JF_SCHEME_B4V3, 1);
  JF_LMAX_ALL_G(JF_SCHEME_B4V3, 2); JF_LMAX_ALL_G(JF_SCHEME_B4V4, 1); JF_LMAX_ALL_G(JF_SCHEME_B4V4, 2);
#undef JF_LMAX_ALL_G
#undef JF_LMAX_CASE
  return 256;
}

// Estimated microseconds of the merge (fitted on MI355X): a fixed part per launch plus a part proportional to
// the candidates one workgroup visits.
constexpr double kMergeFixed = 8.5, kPartialFixed = 7.5, kPerCand = 0.0004, kPerCandBig = 0.001;
constexpr int MG_REG_CANDS = 8192;  // candidates the common merge shape keeps in registers
inline double merge_pass_us(double fixed, long cands) {
  return cands <= MG_REG_CANDS ? fixed + kPerCand * (double)cands : fixed + 1.5 + kPerCandBig * (double)cands;
}

// Two-stage merge when one workgroup per row would face more than MG_REG_CANDS candidates: the number of
// parts (at most MG_REG_CANDS / top_k, so that the final merge keeps its candidates in registers, and at least
// two lists per part) with the smallest estimated time.  parts == 1: single stage.
inline double merge_plan(int rows, int ns, int kc, int top_k, int* parts_out, int* spp_out) {
  *parts_out = 1;
  *spp_out = ns;
  const double wide = 1.5 * (top_k > 256 ? (double)top_k / 256.0 - 1.0 : 0.0);  // slots and pre-correction of the winners
  double best = merge_pass_us(kMergeFixed, (long)ns * kc) + wide;
  if ((long long)ns * kc <= MG_REG_CANDS || ns < 4) return best;
  // (wide corrections run the 32-register shape throughout: its 32768 candidates bound the final merge)
  int cap = (top_k > FS_LDS_TOPK ? 4 * MG_REG_CANDS : MG_REG_CANDS) / top_k;
  if (cap > ns / 2) cap = ns / 2;
  for (int parts = 2; parts <= cap; ++parts) {
    const int spp = (ns + parts - 1) / parts;
    if ((ns + spp - 1) / spp != parts) continue;  // the same spp as a smaller number of parts
    const long wgs = (long)(rows > 0 ? rows : 1) * parts;
    const double rounds = (double)((wgs + 511) / 512);  // two workgroups per CU
    const double us = kPartialFixed + rounds * (merge_pass_us(kPartialFixed, (long)spp * kc) - kPartialFixed) +
                      merge_pass_us(kMergeFixed, (long)parts * top_k) + wide;
    if (us < best) {
      best = us;
      *parts_out = parts;
      *spp_out = spp;
    }
  }
  return best;
}

inline int padded_group(int g) { return g <= 2 ? g : (g <= 4 ? 4 : (g <= 8 ? 8 : 16)); }

inline void fused_plan(int scheme, int NG, int B, int H_q, int H_kv, int max_S, int top_k, int* L_out, int* ns_out,
                       int* kc_out) {
  const int G = padded_group(H_q / H_kv);
  const int units = B * H_kv > 0 ? B * H_kv : 1;
  const int rows = B * H_q > 0 ? B * H_q : 1;
  // One scan workgroup is resident per CU (256 CUs).  Among the split lengths that fit LDS pick the one with
  // the smallest estimated time of scan + merge.  The constants are microseconds fitted to measurements on
  // MI355X: a scan workgroup costs a fixed part plus a part proportional to the 64-position chunks each of
  // its wavefronts works through; a last, partly filled round of workgroups runs faster than a full one; the
  // merge costs a fixed part per launch plus a part proportional to the candidates one workgroup visits.
  const int lmax = lmax_dispatch(scheme, G, NG);
  const int nw = (G <= 4) ? 16 : 8;
  const int kCUs = device_cus();
  constexpr double kScanFixed = 8.5;
  // one chunk per wavefront, all wavefronts; the mixed schemes are priced like the wider one
  const double per_chunk = (scheme == JF_SCHEME_K3V2 || scheme == JF_SCHEME_K2V2) ? 5.9 : 6.6;  // (INT3 values, asymmetric keys: as INT4)
  int L = 256;
  double best = -1.0;
  for (int cand = 256; cand <= lmax; cand += 256) {
    const long nsp = (max_S + cand - 1) / cand > 0 ? (max_S + cand - 1) / cand : 1;
    if (nsp > MG_MAX_SPLITS && cand < lmax) continue;
    const long nwg = nsp * units;
    const long full = nwg / kCUs, rem = nwg % kCUs;
    const double stream = per_chunk * (double)cand / (64.0 * nw);
    double cost = (double)full * (kScanFixed + stream);
    if (rem > 0) cost += kScanFixed + stream * (0.5 + 0.5 * (double)rem / kCUs);
    const int kc = (top_k + FS_CAND_SLACK) < cand ? (top_k + FS_CAND_SLACK) : cand;
    int parts, spp;
    cost += merge_plan(rows, (int)nsp, kc, top_k, &parts, &spp);
    if (best < 0.0 || cost <= best) {
      best = cost;
      L = cand;
    }
    if (cand >= max_S) break;
  }
#ifdef JF_DEBUG_HOOKS
  if (const int forced = g_force_split_len.load(std::memory_order_relaxed); forced > 0) {
    L = (forced + 255) / 256 * 256;
    if (L > lmax) L = lmax;
    while ((max_S + L - 1) / L > MG_MAX_SPLITS && L < lmax) L += 256;
  }
#endif
  int ns = (max_S + L - 1) / L;
  if (ns < 1) ns = 1;
  *L_out = L;
  *ns_out = ns;
  const int cap = top_k + FS_CAND_SLACK;  // the split may emit a superset of its top-k (see phase C)
  *kc_out = cap < L ? cap : L;
}

struct WsLayout {
  size_t off_m, off_l, off_o, off_key, off_idx, off_cnt, off_key2, off_idx2, off_cnt2, total;
};
inline WsLayout ws_layout(int B, int H_q, int ns, int kc, int parts, int top_k) {
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
  w.off_key2 = w.off_idx2 = w.off_cnt2 = 0;
  if (parts > 1) {
    w.off_key2 = take(rows * parts * top_k * 4);
    w.off_idx2 = take(rows * parts * top_k * 4);
    w.off_cnt2 = take(rows * parts * 4);
  }
  w.total = o + 256;
  return w;
}

template <int MODE, int SCHEME, int G, int NG>
int launch_scan(const FusedParams& p, hipStream_t st) {
  const size_t smem = ScanLds<SCHEME, G, NG>::total(p.L);
  auto kern = fused_scan_kernel<MODE, SCHEME, G, NG>;
  // per instantiation: raise the dynamic-LDS limit only when it grows (launches may come from several threads)
  static std::mutex attr_mu;
  static size_t attr_smem = 0;
  {
    std::lock_guard<std::mutex> lock(attr_mu);
    if (smem > attr_smem) {
      JF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
      attr_smem = smem;
    }
  }
#ifdef JF_DEBUG_HOOKS
  std::unique_lock<std::mutex> plock(g_prof_mu, std::defer_lock);
  bool prof = false;
  if (g_prof.armed) {  // (read without the lock: arming happens-before the launches a benchmark times)
    plock.lock();
    prof = g_prof.armed && g_prof.used + 2 <= (int)g_prof.ev.size();
    if (!prof) plock.unlock();
  }
  if (prof) JF_CHECK_HIP(hipEventRecord(g_prof.ev[g_prof.used], st));
#endif
  hipLaunchKernelGGL(kern, dim3(p.n_splits, p.H_kv, p.B), dim3(ScanLds<SCHEME, G, NG>::NT), smem, st, p);
  JF_CHECK_LAUNCH();
#ifdef JF_DEBUG_HOOKS
  if (prof) {
    JF_CHECK_HIP(hipEventRecord(g_prof.ev[g_prof.used + 1], st));
    g_prof.used += 2;
  }
#endif
  return JF_OK;
}

// One scheme of the one-pass form: the GQA group picks the instantiation.
template <int SCHEME, int NG>
int launch_full_by_group(int G, const void* params, void* stream) {
  const FusedParams& p = *static_cast<const FusedParams*>(params);
  hipStream_t st = (hipStream_t)stream;
  switch (G) {
    case 1: return launch_scan<FS_FULL, SCHEME, 1, NG>(p, st);
    case 2: return launch_scan<FS_FULL, SCHEME, 2, NG>(p, st);
    case 4: return launch_scan<FS_FULL, SCHEME, 4, NG>(p, st);
    case 8: return launch_scan<FS_FULL, SCHEME, 8, NG>(p, st);
    default: return launch_scan<FS_FULL, SCHEME, 16, NG>(p, st);
  }
}

inline bool scheme_has_zp(int scheme) {  // asymmetric INT2 keys
  return scheme == JF_SCHEME_A2V2 || scheme == JF_SCHEME_A2V3 || scheme == JF_SCHEME_A2V4;
}
inline bool known_scheme(int scheme) {
  return scheme == JF_SCHEME_K3V2 || scheme == JF_SCHEME_K4V4 || scheme == JF_SCHEME_K3V4 || scheme == JF_SCHEME_K4V2 ||
         scheme == JF_SCHEME_K2V2 || scheme == JF_SCHEME_K2V4 || scheme == JF_SCHEME_K2V3 || scheme == JF_SCHEME_K3V3 ||
         scheme == JF_SCHEME_K4V3 || scheme_has_zp(scheme) || scheme == JF_SCHEME_B4V2 || scheme == JF_SCHEME_B4V3 ||
         scheme == JF_SCHEME_B4V4;
}
// scale groups per row: every scheme but those with INT4 keys (int8-Q model: one key scale per row) may use
// 64-channel groups
inline bool scheme_any_group(int scheme) { return known_scheme(scheme) && scheme / 10 != 4; }
inline int scheme_ng(int scheme, int group_size) { return scheme_any_group(scheme) ? D / group_size : 1; }


// A merge kernel whose winners live in dynamic LDS (corrections wider than FS_LDS_TOPK): 8 bytes per winner; the
// dynamic-LDS limit of the instantiation is raised once.
template <void (*KERN)(FusedParams)>
int launch_wide_merge(dim3 grid, const FusedParams& p, hipStream_t st) {
  static std::mutex mu;
  static bool raised = false;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!raised) {
      JF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(KERN), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       FS_MAX_TOPK * 8));
      raised = true;
    }
  }
  hipLaunchKernelGGL(KERN, grid, dim3(1024), (size_t)p.top_k * 8, st, p);
  return JF_OK;
}

// The whole step on caller-provided workspace memory; every public entry point of the fused forms ends here.
// MODE FS_FULL: all arguments as in jf_fused_scan_topk.  FS_STAGE_A: the value side, o_hat, o_old_unnorm, W are
// unused; top_k == 0 asks for the scores alone (then nothing but `scores` is written and no workspace is needed).
// FS_STAGE_B: q and the key side are unused, `scores_in` and `topk_idx` are inputs (topk_idx may be NULL: o_hat only,
// zeros for the pre-correction terms), topk_slots is unused.
template <int MODE>
static int fused_run(int scheme, int group_size, const uint16_t* q, const uint8_t* k_data,
                     const uint16_t* k_scales, const uint16_t* k_zp, const uint8_t* v_data, const uint16_t* v_scales,
                     const int64_t* block_table, const int32_t* seq_lens, int B, int H_q, int H_kv,
                     int max_S, int max_blocks, int64_t num_slots, int block_size, float attn_scale,
                     int top_k, int64_t* topk_idx, int64_t* topk_slots, float* o_hat,
                     float* o_old_unnorm, float* W, float* softmax_m, float* softmax_inv_z, float* scores,
                     const float* scores_in, const uint16_t* blend_o_new, uint16_t* blend_out, void* workspace,
                     size_t workspace_bytes, void* stream) {
  JF_CHECK_ARG(known_scheme(scheme), "fused_scan: unknown scheme %d", scheme);
  JF_CHECK_ARG(MODE == FS_FULL || scheme == JF_SCHEME_K3V2 || scheme == JF_SCHEME_K4V4 ||
                   (MODE == FS_STAGE_A && (scheme == JF_SCHEME_K2V2 || scheme == JF_SCHEME_A2V2 || scheme == JF_SCHEME_B4V2)) ||
                   (MODE == FS_STAGE_B && (scheme == JF_SCHEME_K3V3 || scheme == JF_SCHEME_K3V4)),
               "fused_scan: the stage-wise forms take the K3V2 or K4V4 side formats (Stage A also K2V2 and A2V2, Stage B also K3V3)");
  JF_CHECK_ARG(!(MODE == FS_FULL || MODE == FS_STAGE_A) || scheme_has_zp(scheme) == (k_zp != nullptr) || B == 0,
               "fused_scan: zero-points go with the asymmetric INT2 key formats, and only with them");
  constexpr bool HAS_K = (MODE == FS_FULL || MODE == FS_STAGE_A), HAS_V = (MODE == FS_FULL || MODE == FS_STAGE_B);
  JF_CHECK_ARG(MODE != FS_TOPK || scheme == JF_SCHEME_K4V4, "fused_scan: the selection-only form uses the K4V4 layout");
  JF_CHECK_ARG((blend_o_new == nullptr) == (blend_out == nullptr), "fused_scan: o_new and out go together");
  JF_CHECK_ARG(B >= 0 && H_q > 0 && H_kv > 0 && max_S >= 0 && H_q % H_kv == 0, "fused_scan: bad shape");
  const int g_act = H_q / H_kv;
  JF_CHECK_ARG(g_act >= 1 && g_act <= 16, "fused_scan: GQA group %d not in 1..16", g_act);
  const int G = padded_group(g_act);  // the kernels come for 1, 2, 4, 8 and 16 query heads per kv-head
  JF_CHECK_ARG(block_size == 16, "fused_scan only supports block_size=16");
  JF_CHECK_ARG(group_size == 64 || group_size == 128, "fused_scan: group_size must be 64 or 128 (got %d)", group_size);
  JF_CHECK_ARG(scheme_any_group(scheme) || group_size == 128,
               "fused_scan: the INT4 sides (int8-Q keys, INT4 values) need group_size 128");
  const bool scores_only = (MODE == FS_STAGE_A) && top_k == 0;
  if (scores_only) top_k = 32;  // (any valid width: the plan depends on it, the kernel stops before using it)
  JF_CHECK_ARG(is_pow2(top_k) && top_k >= 32 && top_k <= FS_MAX_TOPK,
               "fused_scan: unsupported top_k=%d (supported: the powers of two from 32 to 8192)", top_k);
  JF_CHECK_ARG(max_S <= 262144, "fused_scan: max_S=%d exceeds supported limit (262144)", max_S);
  JF_CHECK_ARG((int64_t)max_blocks * block_size >= max_S, "fused_scan: block_table does not cover max_S");
  // (a row's byte offset inside one kv-head's tensor is formed in 32 bits: rows of at most 64 bytes)
  JF_CHECK_ARG(num_slots > 0 && num_slots <= FS_MAX_SLOTS, "fused_scan: num_slots out of range (at most 2^26: row offsets are 32-bit)");
  JF_CHECK_ARG((softmax_m == nullptr) == (softmax_inv_z == nullptr), "fused_scan: softmax_m and softmax_inv_z go together");
  if (B == 0) return JF_OK;
  JF_CHECK_ARG(block_table && seq_lens, "fused_scan: null input");
  if (HAS_K) {
    JF_CHECK_ARG(q && k_data && k_scales, "fused_scan: null input");
    JF_CHECK_ARG(((uintptr_t)k_data & 15) == 0 && ((uintptr_t)q & 15) == 0, "fused_scan: q and k_data must be 16-byte aligned");
    JF_CHECK_ARG(((uintptr_t)k_scales & 3) == 0 && ((uintptr_t)k_zp & 3) == 0, "fused_scan: k_scales and k_zp must be 4-byte aligned");
  }
  if (MODE != FS_STAGE_B) JF_CHECK_ARG(scores_only ? scores != nullptr : (topk_idx && topk_slots), "fused_scan: null output");
  if (HAS_V) {
    JF_CHECK_ARG(v_data && v_scales, "fused_scan: null input");
    JF_CHECK_ARG(((uintptr_t)v_data & 15) == 0 && ((uintptr_t)v_scales & 3) == 0,
                 "fused_scan: v_data must be 16-byte aligned, v_scales 4-byte aligned");
    JF_CHECK_ARG(o_hat && o_old_unnorm && W, "fused_scan: null output");
  }
  if (!HAS_K) JF_CHECK_ARG(scores_in != nullptr, "fused_scan: null scores");
  const int NGv = scheme_ng(scheme, group_size);
  FusedParams p;
  p.q = q; p.k_data = k_data; p.k_scales = k_scales; p.k_zp = k_zp; p.v_data = v_data; p.v_scales = v_scales;
  p.block_table = block_table; p.seq_lens = seq_lens;
  p.B = B; p.H_q = H_q; p.H_kv = H_kv; p.max_S = max_S; p.max_blocks = max_blocks; p.num_slots = num_slots;
  p.g_act = g_act;
  p.attn_scale = attn_scale; p.top_k = top_k;
  fused_plan(scheme, NGv, B, H_q, H_kv, max_S, top_k, &p.L, &p.n_splits, &p.Kc);
  JF_CHECK_ARG(p.n_splits <= MG_MAX_SPLITS, "fused_scan: too many splits (%d > %d)", p.n_splits, MG_MAX_SPLITS);
  merge_plan(B * H_q, p.n_splits, p.Kc, top_k, &p.mg_parts, &p.mg_spp);
  if (MODE == FS_STAGE_B) { p.mg_parts = 1; p.mg_spp = p.n_splits; }
  const WsLayout wl = ws_layout(B, H_q, p.n_splits, p.Kc, p.mg_parts, top_k);
  if (!scores_only) {
    JF_CHECK_ARG(workspace && workspace_bytes >= wl.total, "fused_scan: workspace too small (%zu < %zu)", workspace_bytes, wl.total);
    JF_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fused_scan: workspace must be 256-byte aligned");
  }
  uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
  p.scores = HAS_K ? scores : nullptr;
  p.scores_in = scores_in;
  p.stats_m = p.stats_iz = nullptr;
  p.scores_only = scores_only ? 1 : 0;
  p.part_m = reinterpret_cast<float*>(ws + wl.off_m);
  p.part_l = reinterpret_cast<float*>(ws + wl.off_l);
  p.part_o = reinterpret_cast<float*>(ws + wl.off_o);
  p.cand_key = reinterpret_cast<uint32_t*>(ws + wl.off_key);
  p.cand_idx = reinterpret_cast<int32_t*>(ws + wl.off_idx);
  p.cand_cnt = reinterpret_cast<int32_t*>(ws + wl.off_cnt);
  p.key2 = reinterpret_cast<uint32_t*>(ws + wl.off_key2);
  p.idx2 = reinterpret_cast<int32_t*>(ws + wl.off_idx2);
  p.cnt2 = reinterpret_cast<int32_t*>(ws + wl.off_cnt2);
  p.topk_idx = topk_idx; p.topk_slots = topk_slots; p.o_hat = o_hat; p.o_old = o_old_unnorm; p.W = W;
  p.softmax_m = softmax_m; p.softmax_inv_z = softmax_inv_z;
  p.blend_o_new = blend_o_new; p.blend_out = blend_out;
#ifdef JF_DEBUG_HOOKS
  p.phase_clock = g_phase_clock.load(std::memory_order_relaxed);
#else
  p.phase_clock = nullptr;
#endif
  hipStream_t st = (hipStream_t)stream;
  int rc = JF_OK;
#define JF_FUSED_CASE(SCH, GG, NGG) rc = launch_scan<MODE, SCH, GG, NGG>(p, st)
#define JF_FUSED_BY_G(SCH, NGG)                        \
  switch (G) {                                         \
    case 1: JF_FUSED_CASE(SCH, 1, NGG); break;         \
    case 2: JF_FUSED_CASE(SCH, 2, NGG); break;         \
    case 4: JF_FUSED_CASE(SCH, 4, NGG); break;         \
    case 8: JF_FUSED_CASE(SCH, 8, NGG); break;         \
    default: JF_FUSED_CASE(SCH, 16, NGG); break;       \
  }
  if constexpr (MODE == FS_FULL) {  // (instantiated elsewhere, by family)
    if (scheme_has_zp(scheme)) rc = launch_full_scan_d(scheme, G, NGv, &p, stream);
    else if (scheme / 10 == 5) rc = launch_full_scan_e(scheme, G, NGv, &p, stream);
    else if (scheme / 10 == 2) rc = launch_full_scan_b(scheme, G, NGv, &p, stream);
    else if (scheme == JF_SCHEME_K3V3 || scheme == JF_SCHEME_K4V3) rc = launch_full_scan_c(scheme, G, NGv, &p, stream);
    else rc = launch_full_scan_a(scheme, G, NGv, &p, stream);
  } else if constexpr (MODE == FS_TOPK) {
    JF_FUSED_BY_G(JF_SCHEME_K4V4, 1)
  } else if (scheme == JF_SCHEME_K3V2) {
    if (NGv == 2) JF_FUSED_BY_G(JF_SCHEME_K3V2, 2) else JF_FUSED_BY_G(JF_SCHEME_K3V2, 1)
  } else if (scheme == JF_SCHEME_K4V4) {
    JF_FUSED_BY_G(JF_SCHEME_K4V4, 1)
  } else if constexpr (MODE == FS_STAGE_B) {
    if (scheme == JF_SCHEME_K3V4) {  // INT4 values with either group size (one group: the K4V4 instantiation)
      if (NGv == 2) JF_FUSED_BY_G(JF_SCHEME_K3V4, 2) else JF_FUSED_BY_G(JF_SCHEME_K4V4, 1)
    } else if (NGv == 2) JF_FUSED_BY_G(JF_SCHEME_K3V3, 2) else JF_FUSED_BY_G(JF_SCHEME_K3V3, 1)
  } else if (scheme == JF_SCHEME_K2V2) {  // (Stage A)
    if (NGv == 2) JF_FUSED_BY_G(JF_SCHEME_K2V2, 2) else JF_FUSED_BY_G(JF_SCHEME_K2V2, 1)
  } else if (scheme == JF_SCHEME_B4V2) {
    if (NGv == 2) JF_FUSED_BY_G(JF_SCHEME_B4V2, 2) else JF_FUSED_BY_G(JF_SCHEME_B4V2, 1)
  } else {
    if (NGv == 2) JF_FUSED_BY_G(JF_SCHEME_A2V2, 2) else JF_FUSED_BY_G(JF_SCHEME_A2V2, 1)
  }
#undef JF_FUSED_BY_G
#undef JF_FUSED_CASE
  if (rc != JF_OK || scores_only) return rc;
  dim3 mgrid(B, H_q);
  const bool wide = top_k > FS_LDS_TOPK;  // the winners' arrays do not fit the kernels' static LDS
  if (p.mg_parts > 1) {  // first stage: every part's top_k, as new candidate lists (the same kernel for every form)
    const dim3 pgrid(B, H_q, p.mg_parts);
    if (wide) rc = launch_wide_merge<fused_merge_kernel<FS_FULL, 4, 1, 1024, 32, true, true>>(pgrid, p, st);
    else if ((long long)p.mg_spp * p.Kc > MG_REG_CANDS) hipLaunchKernelGGL((fused_merge_kernel<FS_FULL, 4, 1, 1024, 32, true>), pgrid, dim3(1024), 0, st, p);
    else hipLaunchKernelGGL((fused_merge_kernel<FS_FULL, 4, 1, 1024, 8, true>), pgrid, dim3(1024), 0, st, p);
    if (rc != JF_OK) return rc;
    JF_CHECK_LAUNCH();
  }
  const bool big = (MODE != FS_STAGE_B) &&
                   (p.mg_parts > 1 ? (long long)p.mg_parts * top_k : (long long)p.n_splits * p.Kc) > MG_REG_CANDS;
  // Many rows with few candidates each (large batches of short or medium sequences): four wavefronts per row and
  // small tables, so that five rows share a CU instead of one (measured from 257 rows up: 42.5 against 47.5 us per
  // layer at 384 rows of 2048 candidates, 38 against 57 at 1024 rows of 512).  Same results (see VGRP / VWAVES in
  // the kernel).
  const bool light = (MODE == FS_FULL) && !big && p.mg_parts == 1 && top_k <= MG_LIGHT_TOPK &&
                     (long long)B * H_q > (long long)device_cus() && (long long)p.n_splits * p.Kc <= MG_LIGHT_THREADS * MG_LIGHT_REGK;
#define JF_MERGE(VB, NGG)                                                                                            \
  do {                                                                                                               \
    if (wide) {                                                                                                      \
      if constexpr (MODE == FS_STAGE_B) rc = launch_wide_merge<fused_merge_kernel<MODE, VB, NGG, 1024, 8, false, true>>(mgrid, p, st); \
      else rc = launch_wide_merge<fused_merge_kernel<MODE, VB, NGG, 1024, 32, false, true>>(mgrid, p, st);            \
    } else if (big) hipLaunchKernelGGL((fused_merge_kernel<MODE, VB, NGG, 1024, 32, false>), mgrid, dim3(1024), 0, st, p); \
    else if (light) {                                                                                                \
      if constexpr (MODE == FS_FULL)                                                                                 \
        hipLaunchKernelGGL((fused_merge_kernel<FS_FULL, VB, NGG, MG_LIGHT_THREADS, MG_LIGHT_REGK, false>), mgrid, dim3(MG_LIGHT_THREADS), 0, st, p); \
    } else hipLaunchKernelGGL((fused_merge_kernel<MODE, VB, NGG, 1024, 8, false>), mgrid, dim3(1024), 0, st, p);       \
  } while (0)
  if constexpr (MODE == FS_STAGE_A || MODE == FS_TOPK) {  // no value rows are read: one instantiation serves every format
    if (wide) rc = launch_wide_merge<fused_merge_kernel<FS_STAGE_A, 4, 1, 1024, 32, false, true>>(mgrid, p, st);
    else if (big) hipLaunchKernelGGL((fused_merge_kernel<FS_STAGE_A, 4, 1, 1024, 32, false>), mgrid, dim3(1024), 0, st, p);
    else hipLaunchKernelGGL((fused_merge_kernel<FS_STAGE_A, 4, 1, 1024, 8, false>), mgrid, dim3(1024), 0, st, p);
  } else if (scheme % 10 == 2) {  // INT2 values
    if (NGv == 2) JF_MERGE(2, 2);
    else JF_MERGE(2, 1);
  } else if (scheme % 10 == 3) {  // INT3 values
    if (NGv == 2) JF_MERGE(3, 2);
    else JF_MERGE(3, 1);
  } else {
    if (NGv == 2) JF_MERGE(4, 2);
    else JF_MERGE(4, 1);
  }
#undef JF_MERGE
  if (rc != JF_OK) return rc;
  JF_CHECK_LAUNCH();
  return JF_OK;
}

// The pre-correction terms alone (Stage B merge kernel with the caller's softmax statistics):
//   W = sum_j p_j, o_old_unnorm = sum_j p_j * Vhat_j over the given winners, p_j = exp(score_j - m) * inv_z.
template <int VBITS, int NG>
static int launch_precorr_given_stats(const float* scores, const float* softmax_m, const float* softmax_inv_z,
                                      const uint8_t* v_data, const uint16_t* v_scales, const int64_t* block_table,
                                      const int32_t* seq_lens, const int64_t* topk_idx, int B, int H_q, int H_kv,
                                      int max_S, int max_blocks, int64_t num_slots, int top_k, float* o_old_unnorm,
                                      float* W, hipStream_t st) {
  FusedParams p = {};
  p.v_data = v_data; p.v_scales = v_scales; p.block_table = block_table; p.seq_lens = seq_lens;
  p.B = B; p.H_q = H_q; p.H_kv = H_kv; p.max_S = max_S; p.max_blocks = max_blocks; p.num_slots = num_slots;
  p.top_k = top_k;
  p.n_splits = 0; p.mg_parts = 1; p.mg_spp = 0; p.Kc = 0;
  p.scores_in = scores; p.stats_m = softmax_m; p.stats_iz = softmax_inv_z;
  p.topk_idx = const_cast<int64_t*>(topk_idx);
  p.o_old = o_old_unnorm; p.W = W;
  hipLaunchKernelGGL((fused_merge_kernel<FS_STAGE_B, VBITS, NG, 1024, 8, false>), dim3(B, H_q), dim3(1024), 0, st, p);
  JF_CHECK_LAUNCH();
  return JF_OK;
}

}  // namespace
}  // namespace jf
