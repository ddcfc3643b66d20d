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

int check_common(const void* x, const int64_t* slots, int64_t T, int H_kv, int group_size,
                 int64_t data_stride_slot, int nbits, const void* data, const void* scale) {
  JF_CHECK_ARG(T >= 0 && H_kv > 0, "quant_write: bad T=%lld H_kv=%d", (long long)T, H_kv);
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
  dim3 grid((unsigned)((units + 3) / 4)), block(256);
  hipStream_t st = (hipStream_t)stream;
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
  dim3 grid((unsigned)((units + 3) / 4)), block(256);
  hipLaunchKernelGGL(quant_write_kernel<4>, grid, block, 0, (hipStream_t)stream, s0, d0, s1, d1, slots, T, H_kv, 2, group_size);
  JF_CHECK_LAUNCH();
  return JF_OK;
}
