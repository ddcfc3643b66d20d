// C entry points of the fused decode step (scan + top-k + merge) and the process-wide state its translation
// units share; the kernels and the launcher live in fused_scan_impl.h.
#include "fused_scan_impl.h"

namespace jf {
#ifdef JF_DEBUG_HOOKS
ScanProfile g_prof;
std::mutex g_prof_mu;
std::atomic<long long*> g_phase_clock{nullptr};
std::atomic<int> g_force_split_len{0};
#endif

int device_cus() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      return n;
    (void)hipGetLastError();
    return 256;
  }();
  return cus;
}
}  // namespace jf

using namespace jf;

extern "C" size_t jf_fused_workspace_bytes(int scheme, int B, int H_q, int H_kv, int max_S, int top_k) {
  if (B <= 0 || H_q <= 0 || H_kv <= 0 || H_q % H_kv != 0 || max_S < 0 || top_k <= 0) return 256;
  // the split length depends on the group size only through the LDS budget; size for the worst case
  size_t worst = 0;
  for (int ng = 1; ng <= (scheme_any_group(scheme) ? 2 : 1); ++ng) {
    int L, ns, kc;
    fused_plan(scheme, ng, B, H_q, H_kv, max_S, top_k, &L, &ns, &kc);
    int parts, spp;
    merge_plan(B * H_q, ns, kc, top_k, &parts, &spp);
    const size_t t = ws_layout(B, H_q, ns, kc, parts, top_k).total;
    if (t > worst) worst = t;
  }
  return worst;
}

extern "C" int jf_fused_plan(int scheme, int group_size, int B, int H_q, int H_kv, int max_S, int top_k,
                             int* split_len, int* n_splits, int* list_cap, int* merge_parts) {
  JF_CHECK_ARG(known_scheme(scheme), "fused_plan: unknown scheme %d", scheme);
  JF_CHECK_ARG(B > 0 && H_q > 0 && H_kv > 0 && H_q % H_kv == 0 && max_S >= 0 && top_k > 0, "fused_plan: bad shape");
  JF_CHECK_ARG(group_size == 64 || group_size == 128, "fused_plan: group_size must be 64 or 128");
  int L, ns, kc, parts, spp;
  fused_plan(scheme, scheme_ng(scheme, group_size), B, H_q, H_kv, max_S, top_k, &L, &ns, &kc);
  merge_plan(B * H_q, ns, kc, top_k, &parts, &spp);
  if (split_len) *split_len = L;
  if (n_splits) *n_splits = ns;
  if (list_cap) *list_cap = kc;
  if (merge_parts) *merge_parts = parts;
  return JF_OK;
}

extern "C" int jf_fused_scan_topk(int scheme, int group_size, const uint16_t* q, const uint8_t* k_data,
                                  const uint16_t* k_scales, const uint8_t* v_data, const uint16_t* v_scales,
                                  const int64_t* block_table, const int32_t* seq_lens, int B, int H_q, int H_kv,
                                  int max_S, int max_blocks, int64_t num_slots, int block_size, float attn_scale,
                                  int top_k, int64_t* topk_idx, int64_t* topk_slots, float* o_hat,
                                  float* o_old_unnorm, float* W, float* softmax_m, float* softmax_inv_z, float* scores,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  return fused_run<FS_FULL>(scheme, group_size, q, k_data, k_scales, nullptr, v_data, v_scales, block_table, seq_lens, B, H_q,
                            H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, top_k, topk_idx, topk_slots,
                            o_hat, o_old_unnorm, W, softmax_m, softmax_inv_z, scores, nullptr, nullptr, nullptr, workspace,
                            workspace_bytes, stream);
}

extern "C" int jf_fused_scan_topk_blend(int scheme, int group_size, const uint16_t* q, const uint8_t* k_data,
                                        const uint16_t* k_scales, const uint8_t* v_data, const uint16_t* v_scales,
                                        const int64_t* block_table, const int32_t* seq_lens, int B, int H_q, int H_kv,
                                        int max_S, int max_blocks, int64_t num_slots, int block_size, float attn_scale,
                                        int top_k, int64_t* topk_idx, int64_t* topk_slots, float* o_hat,
                                        float* o_old_unnorm, float* W, float* softmax_m, float* softmax_inv_z,
                                        float* scores, const uint16_t* o_new, uint16_t* out, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  JF_CHECK_ARG(B == 0 || (o_new && out), "fused_scan_blend: null o_new / out");
  return fused_run<FS_FULL>(scheme, group_size, q, k_data, k_scales, nullptr, v_data, v_scales, block_table, seq_lens, B, H_q,
                            H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, top_k, topk_idx, topk_slots,
                            o_hat, o_old_unnorm, W, softmax_m, softmax_inv_z, scores, nullptr, o_new, out, workspace,
                            workspace_bytes, stream);
}

// Asymmetric INT2 keys: the same step with the zero-points of the key groups (and, optionally, the blend).
extern "C" int jf_fused_scan_topk_asym(int scheme, int group_size, const uint16_t* q, const uint8_t* k_data,
                                       const uint16_t* k_scales, const uint16_t* k_zp, const uint8_t* v_data,
                                       const uint16_t* v_scales, const int64_t* block_table, const int32_t* seq_lens, int B,
                                       int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots, int block_size,
                                       float attn_scale, int top_k, int64_t* topk_idx, int64_t* topk_slots, float* o_hat,
                                       float* o_old_unnorm, float* W, float* softmax_m, float* softmax_inv_z,
                                       float* scores, const uint16_t* o_new, uint16_t* out, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  JF_CHECK_ARG(scheme_has_zp(scheme), "fused_scan_asym: scheme must be JF_SCHEME_A2V2, JF_SCHEME_A2V3 or JF_SCHEME_A2V4");
  JF_CHECK_ARG(B == 0 || k_zp != nullptr, "fused_scan_asym: null k_zp");
  return fused_run<FS_FULL>(scheme, group_size, q, k_data, k_scales, k_zp, v_data, v_scales, block_table, seq_lens, B, H_q,
                            H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, top_k, topk_idx, topk_slots,
                            o_hat, o_old_unnorm, W, softmax_m, softmax_inv_z, scores, nullptr, o_new, out, workspace,
                            workspace_bytes, stream);
}

// ---------------------------------------------------------------------------------------------------
// The same step for callers that may not allocate: the workspace is a fixed array in device memory that every
// GPU the library runs on holds until the process ends.  `scratch` names the array for the device code
// object only; host code never passes that name anywhere: it asks the runtime once per device for the array's
// address on that device and uses the returned pointer from then on.
static __device__ __align__(256) unsigned char scratch[JF_FUSED_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};  // address of `scratch` on each device, resolved on first use
}  // namespace

extern "C" int jf_fused_scan_topk_static(int scheme, int group_size, const uint16_t* q, const uint8_t* k_data,
                                         const uint16_t* k_scales, const uint8_t* v_data, const uint16_t* v_scales,
                                         const int64_t* block_table, const int32_t* seq_lens, int B, int H_q,
                                         int H_kv, int max_S, int max_blocks, int64_t num_slots, int block_size,
                                         float attn_scale, int top_k, int64_t* topk_idx, int64_t* topk_slots,
                                         float* o_hat, float* o_old_unnorm, float* W, float* softmax_m,
                                         float* softmax_inv_z, float* scores, void* stream) {
  JF_CHECK_ARG(known_scheme(scheme), "fused_scan_static: unknown scheme %d", scheme);
  JF_CHECK_ARG(!scheme_has_zp(scheme),
               "fused_scan_static: the asymmetric INT2 key formats need their zero-points: use jf_fused_scan_topk_asym");
  JF_CHECK_ARG(B >= 0 && H_q > 0 && H_kv > 0 && max_S >= 0 && H_q % H_kv == 0 && top_k > 0,
               "fused_scan_static: bad shape");
  const size_t need = jf_fused_workspace_bytes(scheme, B, H_q, H_kv, max_S, top_k);
  JF_CHECK_ARG(need <= (size_t)JF_FUSED_STATIC_SCRATCH_BYTES,
               "fused_scan_static: this shape needs %zu bytes of workspace, the built-in scratch holds %zu; use "
               "jf_fused_scan_topk with a caller-provided workspace",
               need, (size_t)JF_FUSED_STATIC_SCRATCH_BYTES);
  int dev = -1;
  JF_CHECK_HIP(hipGetDevice(&dev));
  JF_CHECK_ARG(dev >= 0 && dev < kMaxDevices, "fused_scan_static: device ordinal %d out of range", dev);
  void* ws = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {  // once per device, with that device current
      void* ptr = nullptr;
      JF_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
      JF_CHECK_ARG(ptr != nullptr, "fused_scan_static: the runtime returned no address for the scratch array");
      g_scratch_ptr[dev] = ptr;
    }
    ws = g_scratch_ptr[dev];
  }
  return fused_run<FS_FULL>(scheme, group_size, q, k_data, k_scales, nullptr, v_data, v_scales, block_table, seq_lens, B, H_q,
                            H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, top_k, topk_idx, topk_slots,
                            o_hat, o_old_unnorm, W, softmax_m, softmax_inv_z, scores, nullptr, nullptr, nullptr, ws,
                            (size_t)JF_FUSED_STATIC_SCRATCH_BYTES, stream);
}

#ifdef JF_DEBUG_HOOKS
extern "C" int jf_profile_scan_begin(int max_launches) {
  JF_CHECK_ARG(max_launches > 0 && max_launches <= (1 << 20), "profile_scan_begin: bad max_launches=%d", max_launches);
  std::lock_guard<std::mutex> lock(g_prof_mu);
  for (hipEvent_t e : g_prof.ev) (void)hipEventDestroy(e);
  g_prof.ev.assign((size_t)max_launches * 2, nullptr);
  for (auto& e : g_prof.ev) JF_CHECK_HIP(hipEventCreate(&e));
  g_prof.used = 0;
  g_prof.armed = true;
  return JF_OK;
}

extern "C" int jf_profile_scan_end(double* total_ms, int* launches) {
  JF_CHECK_ARG(total_ms && launches, "profile_scan_end: null output");
  std::lock_guard<std::mutex> lock(g_prof_mu);
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

extern "C" int jf_debug_phase_clock(void* device_buffer) {
  g_phase_clock.store(reinterpret_cast<long long*>(device_buffer));
  return JF_OK;
}

extern "C" int jf_debug_split_len(int split_len) {
  JF_CHECK_ARG(split_len >= 0, "debug_split_len: negative length");
  g_force_split_len.store(split_len);
  return JF_OK;
}
#endif  // JF_DEBUG_HOOKS
