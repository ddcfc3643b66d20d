// Quantise-on-append: bf16 K/V rows -> INT2/3/4 symmetric codes in the reference wire format,
// scattered into the paged cache.  One wavefront owns one (token, kv-head) row of 128 channels:
// lane l holds channels 2l and 2l+1 (one dword load), group maxima are wave reductions, and the
// packed row leaves as 8 (INT2), 12 (INT3) or 16 (INT4) dword stores.
//
// Arithmetic follows the reference quantiser exactly (jetfire_vllm/kernels/intN_pack.py:84-98):
// fp32 amax / qmax (IEEE division), clamp at 1e-8, round to bf16, IEEE divide by the bf16 scale,
// round-half-even, clamp, add the code offset.
#include "common.h"

namespace jf {
namespace {

struct RowDst {
  uint8_t* data;            // cache base
  int64_t data_stride_h;    // bytes
  int64_t data_stride_slot; // bytes
  uint16_t* scale;
  int64_t scale_stride_h;   // elements
  int64_t scale_stride_slot;
};
struct RowSrc {
  const uint16_t* x;
  int64_t stride_t, stride_h;  // elements
};

template <int NBITS>
__device__ inline void quant_row(const uint16_t* __restrict__ xrow, uint8_t* __restrict__ drow,
                                 uint16_t* __restrict__ srow, int group_size, int lane) {
  constexpr int QMAX = (1 << (NBITS - 1)) - 1;
  constexpr int OFF = 1 << (NBITS - 1);
  const uint32_t pair = reinterpret_cast<const uint32_t*>(xrow)[lane];
  const float x0 = bf16_to_f32((uint16_t)(pair & 0xffffu));
  const float x1 = bf16_to_f32((uint16_t)(pair >> 16));
  float amax = fmaxf(fabsf(x0), fabsf(x1));
  const int lanes_per_group = group_size >> 1;
  for (int off = 1; off < lanes_per_group; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  const float sraw = fmaxf(amax / (float)QMAX, 1e-8f);
  const uint16_t sb = f32_to_bf16(sraw);
  const float sf = bf16_to_f32(sb);
  if ((lane & (lanes_per_group - 1)) == 0) srow[lane / lanes_per_group] = sb;
  const int c0 = (int)fminf(fmaxf(rintf(x0 / sf), (float)-QMAX), (float)QMAX) + OFF;
  const int c1 = (int)fminf(fmaxf(rintf(x1 / sf), (float)-QMAX), (float)QMAX) + OFF;

  if (NBITS == 4) {
    // byte l = (c[2l] << 4) | c[2l+1]; four lanes make one dword.
    const uint32_t b = (uint32_t)((c0 << 4) | c1);
    uint32_t v = b;
    v |= (uint32_t)__shfl_down((int)b, 1) << 8;
    v |= (uint32_t)__shfl_down((int)b, 2) << 16;
    v |= (uint32_t)__shfl_down((int)b, 3) << 24;
    if ((lane & 3) == 0) reinterpret_cast<uint32_t*>(drow)[lane >> 2] = v;
  } else if (NBITS == 2) {
    // nibble l = (c[2l] << 2) | c[2l+1]; byte j = nibble[2j] << 4 | nibble[2j+1]; eight lanes per dword.
    const uint32_t n = (uint32_t)((c0 << 2) | c1);
    uint32_t v = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t ni = (i == 0) ? n : (uint32_t)__shfl_down((int)n, i);
      v |= ni << (8 * (i >> 1) + ((i & 1) ? 0 : 4));
    }
    if ((lane & 7) == 0) reinterpret_cast<uint32_t*>(drow)[lane >> 3] = v;
  } else {
    // INT3 planar: 8 codes (4 lanes) -> 24-bit word, MSB first; byte planes of 16 bytes each.
    const uint32_t p = (uint32_t)((c0 << 3) | c1);
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t pi = (i == 0) ? p : (uint32_t)__shfl_down((int)p, i);
      w |= pi << (18 - 6 * i);
    }
    // lane 4g now holds word g.  Plane dword j = bytes of words 4j..4j+3 -> lanes 16j, 16j+4, 16j+8, 16j+12.
    const uint32_t w1 = (uint32_t)__shfl_down((int)w, 4);
    const uint32_t w2 = (uint32_t)__shfl_down((int)w, 8);
    const uint32_t w3 = (uint32_t)__shfl_down((int)w, 12);
    if ((lane & 15) == 0) {
      const int j = lane >> 4;
      uint32_t* d32 = reinterpret_cast<uint32_t*>(drow);
      d32[0 + j] = ((w >> 16) & 255u) | (((w1 >> 16) & 255u) << 8) | (((w2 >> 16) & 255u) << 16) | (((w3 >> 16) & 255u) << 24);
      d32[4 + j] = ((w >> 8) & 255u) | (((w1 >> 8) & 255u) << 8) | (((w2 >> 8) & 255u) << 16) | (((w3 >> 8) & 255u) << 24);
      d32[8 + j] = (w & 255u) | ((w1 & 255u) << 8) | ((w2 & 255u) << 16) | ((w3 & 255u) << 24);
    }
  }
}

// Fast path (16-byte aligned rows): sixteen lanes own one row, lane l holds channels 8l .. 8l+7 (one 16-byte
// load), group maxima are DPP reductions inside the 16-lane row, and the packed row leaves as dword stores
// that are contiguous across the lanes of a row.  A wavefront converts four rows at a time.
template <int CTRL>
__device__ inline uint32_t dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
template <int CTRL>
__device__ inline float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Grid: x = blocks of 16 tokens, y = kv-head, z = tensor (K or V of the fused launch): no index arithmetic
// beyond adds, and the 16 rows of a block leave as one contiguous run when their slots are consecutive.
template <int NBITS>
__global__ __launch_bounds__(256) void quant_write16_kernel(RowSrc s0, RowDst d0, RowSrc s1, RowDst d1,
                                                            const int64_t* __restrict__ slots, int64_t T,
                                                            int H_kv, int n_tensors, int group_size) {
  constexpr int QMAX = (1 << (NBITS - 1)) - 1;
  constexpr int OFF = 1 << (NBITS - 1);
  const int l16 = threadIdx.x & 15;
  const uint32_t r = threadIdx.x >> 4;
  const int64_t t0 = (int64_t)blockIdx.x * 16;  // first token of the block (uniform: its products stay on the scalar unit)
  const int h = blockIdx.y;
  const int which = blockIdx.z;
  // rows past the end still take part in the cross-lane steps (they re-read the block's first row); the row is
  // requested without waiting for its slot, so the two loads are in flight together; masked rows (slot < 0) only
  // skip the stores
  const bool inside = t0 + r < T;
  const uint32_t re = inside ? r : 0u;
  const int64_t slot = slots[t0 + re];
  const RowSrc& s = which ? s1 : s0;
  const RowDst& d = which ? d1 : d0;
  // (the launcher takes this kernel only when the strides fit 32 bits: per-thread products are one 32 x 32 -> 64
  // multiply-add instead of a 64 x 64 multiplication)
  const uint16_t* xrow = s.x + t0 * s.stride_t + (int64_t)h * s.stride_h + (uint64_t)re * (uint32_t)s.stride_t;
  const uint4 raw = reinterpret_cast<const uint4*>(xrow)[l16];
  // (a slot index takes 32 bits: negative = masked row; anything beyond 2^32 cannot be a row of a cache and is
  // skipped like a masked row)
  const bool live = inside && (uint64_t)slot < ((uint64_t)1 << 32);
  float x[8];
  x[0] = bf16_to_f32((uint16_t)(raw.x & 0xffffu)); x[1] = bf16_to_f32((uint16_t)(raw.x >> 16));
  x[2] = bf16_to_f32((uint16_t)(raw.y & 0xffffu)); x[3] = bf16_to_f32((uint16_t)(raw.y >> 16));
  x[4] = bf16_to_f32((uint16_t)(raw.z & 0xffffu)); x[5] = bf16_to_f32((uint16_t)(raw.z >> 16));
  x[6] = bf16_to_f32((uint16_t)(raw.w & 0xffffu)); x[7] = bf16_to_f32((uint16_t)(raw.w >> 16));
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(x[i]));
  // all-reduce over the lanes of one scale group: 4, 8 or 16 lanes
  amax = fmaxf(amax, dpp_f32<0xB1>(amax));   // quad_perm [1,0,3,2]
  amax = fmaxf(amax, dpp_f32<0x4E>(amax));   // quad_perm [2,3,0,1]
  if (group_size >= 64) amax = fmaxf(amax, dpp_f32<0x141>(amax));   // row_half_mirror: lane i <-> 7 - i
  if (group_size >= 128) amax = fmaxf(amax, dpp_f32<0x140>(amax));  // row_mirror: lane i <-> 15 - i
  // scale = bf16(max(amax / QMAX, 1e-8)).  amax is a bf16 value M * 2^e with an 8-bit M, so the exact quotient by 3
  // or 7 is either an 8-bit value itself or has a binary tail of k/3 (k/7) of the unit it is cut at: at least 1/6
  // (1/14) of a bf16 ulp away from every bf16 rounding boundary.  The product with the fp32 reciprocal is within one
  // fp32 ulp of the quotient, i.e. rounds to the same bf16 value as the correctly rounded division (the floor 1e-8
  // is not within an fp32 ulp of a boundary either); checked for every mantissa by the tests.
  constexpr float RQ = 1.0f / (float)QMAX;
  const float sraw = fmaxf(amax * RQ, 1e-8f);
  const uint16_t sb = f32_to_bf16(sraw);
  const float sf = bf16_to_f32(sb);
  // code = clamp(rint(x / sf)).  x and sf are bf16 values (8 significant bits each), so the exact quotient is
  // either exactly a half-integer or at least 1/2040 away from one (for |q| >= 1/2): rint of the fp32-rounded
  // quotient equals rint of ANY value within a few ulp of the exact quotient, provided exact half-integers come
  // out exact.  q0 = x * rcp(sf) is within 2 ulp; one correction with the exact residual r = x - sf * q0 (an
  // fma) gives the exact quotient up to ~2^-45 relative, which rounds to the half-integer itself in a tie.
  // One reciprocal per lane replaces eight correctly rounded divisions.  The clamp comes before the rounding (the
  // bounds are integers: same result), and the rounding is the addition of 2^23 + OFF: the sum lies in
  // [2^23 + 1, 2^23 + 2 OFF - 1], where floats are the integers, so the addition rounds to nearest-even like rint
  // and leaves code = rint(q) + OFF in the low bits of the sum's pattern 0x4B000000 | code.  The pattern's own bits
  // start at bit 24: the packing below shifts and merges the patterns as they are and only ever keeps bits that
  // the codes alone reach.
  const float ry = __builtin_amdgcn_rcpf(sf);
  uint32_t c[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float q0 = x[i] * ry;
    const float q = __builtin_fmaf(__builtin_fmaf(-sf, q0, x[i]), ry, q0);
    const float qc = fminf(fmaxf(q, (float)-QMAX), (float)QMAX);
    c[i] = __builtin_bit_cast(uint32_t, qc + (8388608.0f + (float)OFF));
  }
  const uint64_t so = (uint64_t)(uint32_t)slot;
  uint8_t* drow = d.data + (int64_t)h * d.data_stride_h + so * (uint32_t)d.data_stride_slot;
  uint16_t* srow = d.scale + (int64_t)h * d.scale_stride_h + so * (uint32_t)d.scale_stride_slot;
  const int lpg = group_size >> 3;  // lanes per scale group: 4, 8 or 16
  const int lpg_shift = (group_size >= 128) ? 4 : ((group_size >= 64) ? 3 : 2);
  if (live && (l16 & (lpg - 1)) == 0) srow[l16 >> lpg_shift] = sb;
  if (NBITS == 4) {
    // byte j of the lane's dword = (c[2j] << 4) | c[2j+1]: the low byte of each merged pair (v_perm_b32 gathers them)
    const uint32_t p0 = (c[0] << 4) | c[1], p1 = (c[2] << 4) | c[3], p2 = (c[4] << 4) | c[5], p3 = (c[6] << 4) | c[7];
    const uint32_t v = __builtin_amdgcn_perm(p1, p0, 0x0c0c0400u) | __builtin_amdgcn_perm(p3, p2, 0x04000c0cu);
    if (live) reinterpret_cast<uint32_t*>(drow)[l16] = v;
  } else if (NBITS == 2) {
    // the lane's 8 codes are two bytes, four codes each MSB first (the low bytes of the two merged quadruples);
    // lane pairs share a dword
    const uint32_t pa = (c[0] << 6) | (c[1] << 4) | (c[2] << 2) | c[3], pb = (c[4] << 6) | (c[5] << 4) | (c[6] << 2) | c[7];
    const uint32_t hw = __builtin_amdgcn_perm(pb, pa, 0x0c0c0400u);
    const uint32_t nb = dpp_u32<0xB1>(hw);  // neighbour inside the lane pair
    if (live && (l16 & 1) == 0) reinterpret_cast<uint32_t*>(drow)[l16 >> 1] = hw | (nb << 16);
  } else {
    // INT3 planar: the lane's 8 codes are the 24-bit word l16, MSB first (bits 0..23 of w; what lies above is the
    // patterns' own bits and is never extracted); plane p holds byte p of every word.
    // Lane (4j + p), p < 3, assembles dword j of plane p from the four words of its quad.
    const uint32_t w = (c[0] << 21) | (c[1] << 18) | (c[2] << 15) | (c[3] << 12) | (c[4] << 9) | (c[5] << 6) | (c[6] << 3) | c[7];
    const uint32_t w0 = dpp_u32<0x00>(w), w1 = dpp_u32<0x55>(w), w2 = dpp_u32<0xAA>(w), w3 = dpp_u32<0xFF>(w);  // quad broadcasts
    const int pl = l16 & 3;
    const int sh = 16 - 8 * pl;
    const uint32_t v = ((w0 >> sh) & 255u) | (((w1 >> sh) & 255u) << 8) | (((w2 >> sh) & 255u) << 16) | (((w3 >> sh) & 255u) << 24);
    if (live && pl < 3) reinterpret_cast<uint32_t*>(drow)[4 * pl + (l16 >> 2)] = v;
  }
}

// Asymmetric INT2 keys over the full codebook (jetfire_vllm/kernels/intN_pack.py:110-169,
// fused_quant_write.py:85-133): per group scale = bf16(max((xmax - xmin) / 3, 1e-8)),
// zp = bf16(xmin + 2 * scale_f32), code = clamp(rint((x - zp) / scale), -2, 1) + 2.  Same lane layout as
// quant_write16_kernel (sixteen lanes per row, eight channels per lane); the divisions are IEEE divisions:
// the numerator x - zp is not a bf16 value, so the reciprocal shortcut of the symmetric kernel does not apply.
__global__ __launch_bounds__(256) void quant_write16_int2_asym_kernel(RowSrc s, RowDst d, uint16_t* __restrict__ zp_out,
                                                                      int64_t zp_stride_h, int64_t zp_stride_slot,
                                                                      const int64_t* __restrict__ slots, int64_t T,
                                                                      int group_size) {
  const int l16 = threadIdx.x & 15;
  const int64_t tq = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int h = blockIdx.y;
  const bool inside = tq < T;
  const int64_t t = inside ? tq : 0;
  const int64_t slot = slots[t];
  const uint16_t* xrow = s.x + t * s.stride_t + (int64_t)h * s.stride_h;
  const uint4 raw = reinterpret_cast<const uint4*>(xrow)[l16];
  const bool live = inside && slot >= 0;
  float x[8];
  x[0] = bf16_to_f32((uint16_t)(raw.x & 0xffffu)); x[1] = bf16_to_f32((uint16_t)(raw.x >> 16));
  x[2] = bf16_to_f32((uint16_t)(raw.y & 0xffffu)); x[3] = bf16_to_f32((uint16_t)(raw.y >> 16));
  x[4] = bf16_to_f32((uint16_t)(raw.z & 0xffffu)); x[5] = bf16_to_f32((uint16_t)(raw.z >> 16));
  x[6] = bf16_to_f32((uint16_t)(raw.w & 0xffffu)); x[7] = bf16_to_f32((uint16_t)(raw.w >> 16));
  float xmax = x[0], xmin = x[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    xmax = fmaxf(xmax, x[i]);
    xmin = fminf(xmin, x[i]);
  }
  xmax = fmaxf(xmax, dpp_f32<0xB1>(xmax)); xmin = fminf(xmin, dpp_f32<0xB1>(xmin));
  xmax = fmaxf(xmax, dpp_f32<0x4E>(xmax)); xmin = fminf(xmin, dpp_f32<0x4E>(xmin));
  if (group_size >= 64) { xmax = fmaxf(xmax, dpp_f32<0x141>(xmax)); xmin = fminf(xmin, dpp_f32<0x141>(xmin)); }
  if (group_size >= 128) { xmax = fmaxf(xmax, dpp_f32<0x140>(xmax)); xmin = fminf(xmin, dpp_f32<0x140>(xmin)); }
  const float sraw = fmaxf((xmax - xmin) / 3.0f, 1e-8f);
  const float zraw = xmin + 2.0f * sraw;
  const uint16_t sb = f32_to_bf16(sraw), zb = f32_to_bf16(zraw);
  const float sf = bf16_to_f32(sb), zf = bf16_to_f32(zb);
  uint32_t c[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) c[i] = (uint32_t)((int)fminf(fmaxf(rintf((x[i] - zf) / sf), -2.0f), 1.0f) + 2);
  uint8_t* drow = d.data + (int64_t)h * d.data_stride_h + slot * d.data_stride_slot;
  const int lpg = group_size >> 3;
  if (live && (l16 & (lpg - 1)) == 0) {
    d.scale[(int64_t)h * d.scale_stride_h + slot * d.scale_stride_slot + l16 / lpg] = sb;
    zp_out[(int64_t)h * zp_stride_h + slot * zp_stride_slot + l16 / lpg] = zb;
  }
  const uint32_t hw = ((c[0] << 6) | (c[1] << 4) | (c[2] << 2) | c[3]) | (((c[4] << 6) | (c[5] << 4) | (c[6] << 2) | c[7]) << 8);
  const uint32_t nb = dpp_u32<0xB1>(hw);
  if (live && (l16 & 1) == 0) reinterpret_cast<uint32_t*>(drow)[l16 >> 1] = hw | (nb << 16);
}

// units = T * H_kv * n_tensors (n_tensors = 2 for the fused K+V INT4 launch)
template <int NBITS>
__global__ __launch_bounds__(256) void quant_write_kernel(RowSrc s0, RowDst d0, RowSrc s1, RowDst d1,
                                                          const int64_t* __restrict__ slots, int64_t T,
                                                          int H_kv, int n_tensors, int group_size) {
  const int lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t total = T * H_kv * n_tensors;
  if (unit >= total) return;
  const int which = (int)(unit / (T * H_kv));
  const int64_t rem = unit - (int64_t)which * T * H_kv;
  const int64_t t = rem / H_kv;
  const int h = (int)(rem - t * H_kv);
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const RowSrc& s = which ? s1 : s0;
  const RowDst& d = which ? d1 : d0;
  const uint16_t* xrow = s.x + t * s.stride_t + (int64_t)h * s.stride_h;
  uint8_t* drow = d.data + (int64_t)h * d.data_stride_h + slot * d.data_stride_slot;
  uint16_t* srow = d.scale + (int64_t)h * d.scale_stride_h + slot * d.scale_stride_slot;
  quant_row<NBITS>(xrow, drow, srow, group_size, lane);
}

inline bool rows_16b_aligned(const void* x, int64_t stride_t, int64_t stride_h) {
  return ((uintptr_t)x & 15) == 0 && stride_t % 8 == 0 && stride_h % 8 == 0;
}
// what quant_write16_kernel multiplies per thread with 32-bit operands
inline bool strides_fit_32(int64_t x_stride_t, int64_t data_stride_slot, int64_t scale_stride_slot) {
  const int64_t lim = (int64_t)1 << 32;
  return x_stride_t >= 0 && x_stride_t < lim && data_stride_slot >= 0 && data_stride_slot < lim &&
         scale_stride_slot >= 0 && scale_stride_slot < lim;
}

int check_common(const void* x, const int64_t* slots, int64_t T, int H_kv, int group_size,
                 int64_t data_stride_slot, int nbits, const void* data, const void* scale) {
  JF_CHECK_ARG(T >= 0 && H_kv > 0 && H_kv <= 65535, "quant_write: bad T=%lld H_kv=%d", (long long)T, H_kv);
  JF_CHECK_ARG(T <= (int64_t)16 * 0x7fffffff, "quant_write: T=%lld exceeds the launch grid", (long long)T);
  JF_CHECK_ARG(group_size == 32 || group_size == 64 || group_size == 128,
               "quant_write: group_size must be 32, 64 or 128 (got %d)", group_size);
  JF_CHECK_ARG(nbits == 2 || nbits == 3 || nbits == 4, "quant_write: nbits must be 2, 3 or 4 (got %d)", nbits);
  if (T == 0) return JF_OK;
  JF_CHECK_ARG(x && slots && data && scale, "quant_write: null pointer");
  JF_CHECK_ARG(((uintptr_t)x & 3) == 0 && ((uintptr_t)data & 3) == 0, "quant_write: x and cache must be 4-byte aligned");
  JF_CHECK_ARG(data_stride_slot % 4 == 0 && data_stride_slot >= D * nbits / 8,
               "quant_write: cache row stride %lld too small / unaligned for INT%d", (long long)data_stride_slot, nbits);
  return JF_OK;
}

}  // namespace
}  // namespace jf

using namespace jf;

extern "C" int jf_quant_write_sym(const uint16_t* x, int64_t x_stride_t, int64_t x_stride_h,
                                  const int64_t* slots, int64_t T, int H_kv,
                                  uint8_t* out_data, int64_t data_stride_h, int64_t data_stride_slot,
                                  uint16_t* out_scale, int64_t scale_stride_h, int64_t scale_stride_slot,
                                  int64_t num_slots, int group_size, int nbits, void* stream) {
  (void)num_slots;
  int rc = check_common(x, slots, T, H_kv, group_size, data_stride_slot, nbits, out_data, out_scale);
  if (rc != JF_OK || T == 0) return rc;
  JF_CHECK_ARG(x_stride_t % 2 == 0 && x_stride_h % 2 == 0, "quant_write: x strides must be even");
  RowSrc s{x, x_stride_t, x_stride_h};
  RowDst d{out_data, data_stride_h, data_stride_slot, out_scale, scale_stride_h, scale_stride_slot};
  const int64_t units = T * H_kv;
  hipStream_t st = (hipStream_t)stream;
  if (rows_16b_aligned(x, x_stride_t, x_stride_h) && strides_fit_32(x_stride_t, data_stride_slot, scale_stride_slot)) {
    dim3 grid16((unsigned)((T + 15) / 16), (unsigned)H_kv, 1), block16(256);
    if (nbits == 2) hipLaunchKernelGGL(quant_write16_kernel<2>, grid16, block16, 0, st, s, d, s, d, slots, T, H_kv, 1, group_size);
    else if (nbits == 3) hipLaunchKernelGGL(quant_write16_kernel<3>, grid16, block16, 0, st, s, d, s, d, slots, T, H_kv, 1, group_size);
    else hipLaunchKernelGGL(quant_write16_kernel<4>, grid16, block16, 0, st, s, d, s, d, slots, T, H_kv, 1, group_size);
    JF_CHECK_LAUNCH();
    return JF_OK;
  }
  dim3 grid((unsigned)((units + 3) / 4)), block(256);
  if (nbits == 2) hipLaunchKernelGGL(quant_write_kernel<2>, grid, block, 0, st, s, d, s, d, slots, T, H_kv, 1, group_size);
  else if (nbits == 3) hipLaunchKernelGGL(quant_write_kernel<3>, grid, block, 0, st, s, d, s, d, slots, T, H_kv, 1, group_size);
  else hipLaunchKernelGGL(quant_write_kernel<4>, grid, block, 0, st, s, d, s, d, slots, T, H_kv, 1, group_size);
  JF_CHECK_LAUNCH();
  return JF_OK;
}

extern "C" int jf_quant_write_int4_sym_kv(const uint16_t* key, int64_t k_stride_t, int64_t k_stride_h,
                                          const uint16_t* value, int64_t v_stride_t, int64_t v_stride_h,
                                          const int64_t* slots, int64_t T, int H_kv,
                                          uint8_t* k_data, int64_t k_data_stride_h, int64_t k_data_stride_slot,
                                          uint16_t* k_scale, int64_t k_scale_stride_h, int64_t k_scale_stride_slot,
                                          uint8_t* v_data, int64_t v_data_stride_h, int64_t v_data_stride_slot,
                                          uint16_t* v_scale, int64_t v_scale_stride_h, int64_t v_scale_stride_slot,
                                          int64_t num_slots, int group_size, void* stream) {
  (void)num_slots;
  int rc = check_common(key, slots, T, H_kv, group_size, k_data_stride_slot, 4, k_data, k_scale);
  if (rc != JF_OK) return rc;
  rc = check_common(value, slots, T, H_kv, group_size, v_data_stride_slot, 4, v_data, v_scale);
  if (rc != JF_OK || T == 0) return rc;
  JF_CHECK_ARG((k_stride_t | k_stride_h | v_stride_t | v_stride_h) % 2 == 0, "quant_write: x strides must be even");
  RowSrc s0{key, k_stride_t, k_stride_h}, s1{value, v_stride_t, v_stride_h};
  RowDst d0{k_data, k_data_stride_h, k_data_stride_slot, k_scale, k_scale_stride_h, k_scale_stride_slot};
  RowDst d1{v_data, v_data_stride_h, v_data_stride_slot, v_scale, v_scale_stride_h, v_scale_stride_slot};
  const int64_t units = T * H_kv * 2;
  if (rows_16b_aligned(key, k_stride_t, k_stride_h) && rows_16b_aligned(value, v_stride_t, v_stride_h) &&
      strides_fit_32(k_stride_t, k_data_stride_slot, k_scale_stride_slot) &&
      strides_fit_32(v_stride_t, v_data_stride_slot, v_scale_stride_slot)) {
    dim3 grid16((unsigned)((T + 15) / 16), (unsigned)H_kv, 2), block16(256);
    hipLaunchKernelGGL(quant_write16_kernel<4>, grid16, block16, 0, (hipStream_t)stream, s0, d0, s1, d1, slots, T, H_kv, 2, group_size);
    JF_CHECK_LAUNCH();
    return JF_OK;
  }
  dim3 grid((unsigned)((units + 3) / 4)), block(256);
  hipLaunchKernelGGL(quant_write_kernel<4>, grid, block, 0, (hipStream_t)stream, s0, d0, s1, d1, slots, T, H_kv, 2, group_size);
  JF_CHECK_LAUNCH();
  return JF_OK;
}

extern "C" int jf_quant_write_int2_asym(const uint16_t* x, int64_t x_stride_t, int64_t x_stride_h, const int64_t* slots,
                                        int64_t T, int H_kv, uint8_t* out_data, int64_t data_stride_h,
                                        int64_t data_stride_slot, uint16_t* out_scale, int64_t scale_stride_h,
                                        int64_t scale_stride_slot, uint16_t* out_zp, int64_t zp_stride_h,
                                        int64_t zp_stride_slot, int64_t num_slots, int group_size, void* stream) {
  (void)num_slots;
  int rc = check_common(x, slots, T, H_kv, group_size, data_stride_slot, 2, out_data, out_scale);
  if (rc != JF_OK || T == 0) return rc;
  JF_CHECK_ARG(out_zp, "quant_write_int2_asym: null zero-point tensor");
  JF_CHECK_ARG(rows_16b_aligned(x, x_stride_t, x_stride_h), "quant_write_int2_asym: token rows must be 16-byte aligned");
  RowSrc s{x, x_stride_t, x_stride_h};
  RowDst d{out_data, data_stride_h, data_stride_slot, out_scale, scale_stride_h, scale_stride_slot};
  dim3 grid((unsigned)((T + 15) / 16), (unsigned)H_kv, 1), block(256);
  hipLaunchKernelGGL(quant_write16_int2_asym_kernel, grid, block, 0, (hipStream_t)stream, s, d, out_zp, zp_stride_h,
                     zp_stride_slot, slots, T, group_size);
  JF_CHECK_LAUNCH();
  return JF_OK;
}
