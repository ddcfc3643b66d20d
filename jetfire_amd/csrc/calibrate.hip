// Read-only streaming calibration: what a kernel that does nothing but 16-byte loads reaches on this machine.
// The decode scan is a read stream (its writes are ~4 % of its traffic), so this is the ceiling its
// `roofline.achieved` is compared with besides the published HBM peak.  Measurement aid, no counterpart in the
// reference.
#include "common.h"

#ifdef JF_DEBUG_HOOKS

namespace jf {
namespace {
typedef unsigned v4u __attribute__((ext_vector_type(4)));

// grid-stride over 16-byte items, eight loads in flight per lane; the xor of everything read is stored only if
// it equals a value it cannot take by construction of the caller's data (keeps the loads alive)
__global__ __launch_bounds__(256) void stream_read_kernel(const v4u* __restrict__ src, size_t n16, unsigned* sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  v4u acc = {0u, 0u, 0u, 0u};
  for (; i + 7 * stride < n16; i += 8 * stride) {
    v4u v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  for (; i < n16; i += stride) acc ^= src[i];
  const unsigned x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (x == 0x9e3779b9u && sink) *sink = x;
}
}  // namespace
}  // namespace jf

using namespace jf;

extern "C" int jf_calibrate_stream_read(const void* src, size_t bytes, void* sink, void* stream) {
  JF_CHECK_ARG(src && bytes >= 16 && ((uintptr_t)src & 15) == 0, "calibrate_stream_read: src must be 16-byte aligned, at least 16 bytes");
  const size_t n16 = bytes / 16;
  size_t blocks = (n16 + 256 * 8 - 1) / (256 * 8);
  if (blocks > 256 * 16) blocks = 256 * 16;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const v4u*>(src), n16, reinterpret_cast<unsigned*>(sink));
  JF_CHECK_LAUNCH();
  return JF_OK;
}
#endif  // JF_DEBUG_HOOKS
