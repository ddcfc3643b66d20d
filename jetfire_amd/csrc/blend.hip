// GPU-side merge of the approximate partials with the CPU correction:
//   out = bf16_rne(fma(W, f32(o_new), o_hat) - o_old_unnorm)
// (jetfire_vllm/csrc/blend.cu:202-226 evaluates `hat + w*n - old` left to right with the
// multiply-add contracted).  One thread per output element; the whole launch is B*H_q*D elements.
#include "common.h"

namespace jf {
namespace {
__global__ __launch_bounds__(256) void blend_unnorm_kernel(const float* __restrict__ o_hat,
                                                           const float* __restrict__ o_old,
                                                           const float* __restrict__ W,
                                                           const uint16_t* __restrict__ o_new,
                                                           uint16_t* __restrict__ out, int D, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float w = W[i / D];
  const float v = __builtin_fmaf(w, bf16_to_f32(o_new[i]), o_hat[i]) - o_old[i];
  out[i] = f32_to_bf16(v);
}
// The form with a normalised o_old (jetfire_vllm/csrc/blend.cu:44-66): out = bf16_rne(fma(W, f32(o_new) - o_old, o_hat)).
__global__ __launch_bounds__(256) void blend_kernel(const float* __restrict__ o_hat, const float* __restrict__ o_old,
                                                    const float* __restrict__ W, const uint16_t* __restrict__ o_new,
                                                    uint16_t* __restrict__ out, int D, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float w = W[i / D];
  out[i] = f32_to_bf16(__builtin_fmaf(w, bf16_to_f32(o_new[i]) - o_old[i], o_hat[i]));
}
}  // namespace
}  // namespace jf

using namespace jf;

extern "C" int jf_blend_unnorm(const float* o_hat, const float* o_old_unnorm, const float* W,
                               const uint16_t* o_new, uint16_t* out, int B, int H_q, int D, void* stream) {
  JF_CHECK_ARG(B >= 0 && H_q > 0 && D > 0, "blend_unnorm: bad shape B=%d H_q=%d D=%d", B, H_q, D);
  if (B == 0) return JF_OK;
  JF_CHECK_ARG(o_hat && o_old_unnorm && W && o_new && out, "blend_unnorm: null pointer");
  const int64_t total = (int64_t)B * H_q * D;
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  hipLaunchKernelGGL(blend_unnorm_kernel, grid, block, 0, (hipStream_t)stream, o_hat, o_old_unnorm, W, o_new, out, D, total);
  JF_CHECK_LAUNCH();
  return JF_OK;
}

extern "C" int jf_blend(const float* o_hat, const float* o_old, const float* W, const uint16_t* o_new, uint16_t* out,
                        int B, int H_q, int D, void* stream) {
  JF_CHECK_ARG(B >= 0 && H_q > 0 && D > 0, "blend: bad shape B=%d H_q=%d D=%d", B, H_q, D);
  if (B == 0) return JF_OK;
  JF_CHECK_ARG(o_hat && o_old && W && o_new && out, "blend: null pointer");
  const int64_t total = (int64_t)B * H_q * D;
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  hipLaunchKernelGGL(blend_kernel, grid, block, 0, (hipStream_t)stream, o_hat, o_old, W, o_new, out, D, total);
  JF_CHECK_LAUNCH();
  return JF_OK;
}
