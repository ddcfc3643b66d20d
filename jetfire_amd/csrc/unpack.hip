// Dequantise packed INT2/3/4 rows back to bf16 (jetfire_vllm/kernels/intN_pack.py:227-311).
// Sixteen lanes own one row of 128 channels: lane l reads the 2 (INT2), 3 (INT3, one byte of each plane) or
// 4 (INT4) bytes that hold channels 8l .. 8l+7 and stores them as one 16-byte run, so a wavefront writes
// four whole rows per instruction.  HBM-bound: 256 bytes written per row against 34..68 read.
//
// Arithmetic as the reference: bf16(f32(code - offset) * f32(scale)); with zero-points the rounded product
// is widened again, the zero-point added in fp32 and the sum rounded to bf16 a second time (:251-256).
#include "common.h"

namespace jf {
namespace {

template <int NBITS, bool ZP>
__global__ __launch_bounds__(256) void unpack_rows_kernel(const uint8_t* __restrict__ data, int64_t data_stride,
                                                          const uint16_t* __restrict__ scales, int64_t scale_stride,
                                                          const uint16_t* __restrict__ zps, int64_t zp_stride,
                                                          int64_t rows, int group_shift, uint16_t* __restrict__ out,
                                                          int64_t out_stride) {
  constexpr int OFF = 1 << (NBITS - 1);
  const int l16 = threadIdx.x & 15;
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (row >= rows) return;
  const uint8_t* drow = data + row * data_stride;
  const int g = (8 * l16) >> group_shift;
  const float s = bf16_to_f32(scales[row * scale_stride + g]);
  float z = 0.0f;
  if (ZP) z = bf16_to_f32(zps[row * zp_stride + g]);

  uint32_t codes;   // eight codes, channel 8l+i in bits [4i, 4i+4)
  if (NBITS == 4) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(drow + 4 * l16);   // byte j = (c[2j] << 4) | c[2j+1]
    // channel 2j sits in the high nibble of byte j, channel 2j+1 in the low one: swap the nibbles of every byte
    codes = ((w & 0xf0f0f0f0u) >> 4) | ((w & 0x0f0f0f0fu) << 4);
  } else if (NBITS == 2) {
    const uint32_t w = *reinterpret_cast<const uint16_t*>(drow + 2 * l16);   // byte j = c[4j]<<6 | c[4j+1]<<4 | ...
    codes = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) codes |= ((w >> (8 * (i >> 2) + 6 - 2 * (i & 3))) & 3u) << (4 * i);
  } else {
    const uint32_t w = ((uint32_t)drow[l16] << 16) | ((uint32_t)drow[16 + l16] << 8) | (uint32_t)drow[32 + l16];
    codes = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) codes |= ((w >> (21 - 3 * i)) & 7u) << (4 * i);
  }

  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float q = (float)((int)((codes >> (4 * i)) & 15u) - OFF);
    uint16_t b = f32_to_bf16(q * s);
    if (ZP) b = f32_to_bf16(bf16_to_f32(b) + z);
    if (i & 1) o[i >> 1] |= (uint32_t)b << 16; else o[i >> 1] = b;
  }
  *reinterpret_cast<uint4*>(out + row * out_stride + 8 * l16) = make_uint4(o[0], o[1], o[2], o[3]);
}

template <int NBITS>
int launch_unpack(const uint8_t* data, int64_t data_stride, const uint16_t* scales, int64_t scale_stride,
                  const uint16_t* zps, int64_t zp_stride, int64_t rows, int group_shift, uint16_t* out,
                  int64_t out_stride, hipStream_t st) {
  dim3 grid((unsigned)((rows + 15) / 16)), block(256);
  if (zps)
    hipLaunchKernelGGL((unpack_rows_kernel<NBITS, true>), grid, block, 0, st, data, data_stride, scales, scale_stride,
                       zps, zp_stride, rows, group_shift, out, out_stride);
  else
    hipLaunchKernelGGL((unpack_rows_kernel<NBITS, false>), grid, block, 0, st, data, data_stride, scales, scale_stride,
                       zps, zp_stride, rows, group_shift, out, out_stride);
  JF_CHECK_LAUNCH();
  return JF_OK;
}

}  // namespace
}  // namespace jf

using namespace jf;

extern "C" int jf_unpack(const uint8_t* data, int64_t data_stride_row, const uint16_t* scales,
                         int64_t scale_stride_row, const uint16_t* zps, int64_t zp_stride_row, int64_t rows,
                         int group_size, int nbits, uint16_t* out, int64_t out_stride_row, void* stream) {
  JF_CHECK_ARG(rows >= 0 && rows < ((int64_t)1 << 31) * 16, "unpack: rows=%lld out of range", (long long)rows);
  if (rows == 0) return JF_OK;
  JF_CHECK_ARG(data && scales && out, "unpack: null tensor");
  JF_CHECK_ARG(nbits == 2 || nbits == 3 || nbits == 4, "unpack: nbits=%d (2, 3 or 4)", nbits);
  JF_CHECK_ARG(is_pow2(group_size) && group_size >= 8 && group_size <= D, "unpack: group_size=%d (8..128, power of 2)",
               group_size);
  JF_CHECK_ARG(data_stride_row >= D * nbits / 8, "unpack: data rows overlap");
  JF_CHECK_ARG(nbits == 3 || (((uintptr_t)data | (uintptr_t)data_stride_row) & (nbits == 4 ? 3 : 1)) == 0,
               "unpack: data rows must be %d-byte aligned", nbits == 4 ? 4 : 2);
  JF_CHECK_ARG((((uintptr_t)out | (uintptr_t)(out_stride_row * 2)) & 15) == 0 && out_stride_row >= D,
               "unpack: output rows must be 16-byte aligned and at least 128 elements apart");
  JF_CHECK_ARG(scale_stride_row >= D / group_size && (!zps || zp_stride_row >= D / group_size),
               "unpack: scale / zero-point rows overlap");
  int shift = 0;
  while ((1 << shift) < group_size) ++shift;
  hipStream_t st = (hipStream_t)stream;
  switch (nbits) {
    case 2: return launch_unpack<2>(data, data_stride_row, scales, scale_stride_row, zps, zp_stride_row, rows, shift, out, out_stride_row, st);
    case 3: return launch_unpack<3>(data, data_stride_row, scales, scale_stride_row, zps, zp_stride_row, rows, shift, out, out_stride_row, st);
    default: return launch_unpack<4>(data, data_stride_row, scales, scale_stride_row, zps, zp_stride_row, rows, shift, out, out_stride_row, st);
  }
}
