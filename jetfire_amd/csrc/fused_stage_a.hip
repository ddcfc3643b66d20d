// Stage A alone on the kernels of the fused step: scores (written to HBM on request), exact top-k with slots, softmax
// statistics; the key stream only.  The fast form of the reference's int3_qk_scores / int3_qk_scores_topk
// (jetfire_vllm/csrc/int3_qk_scores.cu:640-655) and int8tc_qk_scores / ..._topk / ..._topk_stats
// (jetfire_vllm/csrc/int8tc_qk_scores.cu:2774-2798) for the shapes the fused step supports.
#include "fused_scan_impl.h"

using namespace jf;

extern "C" int jf_stage_a_topk(int key_format, int group_size, const uint16_t* q, const uint8_t* k_data,
                               const uint16_t* k_scales, const int64_t* block_table, const int32_t* seq_lens, int B,
                               int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots, int block_size,
                               float attn_scale, int top_k, float* scores, int64_t* topk_idx, int64_t* topk_slots,
                               float* softmax_m, float* softmax_inv_z, void* workspace, size_t workspace_bytes,
                               void* stream) {
  JF_CHECK_ARG(key_format == JF_SCHEME_K3V2 || key_format == JF_SCHEME_K4V4 || key_format == JF_SCHEME_K2V2 ||
                   key_format == JF_SCHEME_B4V2,
               "stage_a_topk: key_format must be JF_SCHEME_K3V2 (INT3 keys, bf16 model), JF_SCHEME_K2V2 (symmetric INT2 keys, "
               "bf16 model), JF_SCHEME_B4V2 (INT4 keys, bf16 model) or JF_SCHEME_K4V4 (INT4 keys, int8-Q model)");
  JF_CHECK_ARG(top_k >= 0, "stage_a_topk: negative top_k");
  return fused_run<FS_STAGE_A>(key_format, group_size, q, k_data, k_scales, nullptr, nullptr, nullptr, block_table, seq_lens,
                               B, H_q, H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, top_k, topk_idx,
                               topk_slots, nullptr, nullptr, nullptr, softmax_m, softmax_inv_z, scores, nullptr, nullptr,
                               nullptr, workspace, workspace_bytes, stream);
}

// Stage A for the asymmetric INT2 keys: int2_qk_scores / int2_qk_scores_topk with zero-points
// (jetfire_vllm/csrc/int2_qk_scores.cu:66-79, 663-680).
extern "C" int jf_stage_a_topk_asym(int group_size, const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                                    const uint16_t* k_zp, const int64_t* block_table, const int32_t* seq_lens, int B,
                                    int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots, int block_size,
                                    float attn_scale, int top_k, float* scores, int64_t* topk_idx, int64_t* topk_slots,
                                    float* softmax_m, float* softmax_inv_z, void* workspace, size_t workspace_bytes,
                                    void* stream) {
  JF_CHECK_ARG(top_k >= 0, "stage_a_topk_asym: negative top_k");
  JF_CHECK_ARG(B == 0 || k_zp != nullptr, "stage_a_topk_asym: null k_zp");
  return fused_run<FS_STAGE_A>(JF_SCHEME_A2V2, group_size, q, k_data, k_scales, k_zp, nullptr, nullptr, block_table,
                               seq_lens, B, H_q, H_kv, max_S, max_blocks, num_slots, block_size, attn_scale, top_k,
                               topk_idx, topk_slots, nullptr, nullptr, nullptr, softmax_m, softmax_inv_z, scores, nullptr,
                               nullptr, nullptr, workspace, workspace_bytes, stream);
}

// The selection alone (scores are an input): the fast form of jf_topk_slots.  The rows are grouped
// four (or two, or one) to a workgroup; nothing else depends on the grouping.
extern "C" int jf_topk_slots_fast(const float* scores, const int32_t* seq_lens, const int64_t* block_table, int B, int H_q,
                                  int max_S, int max_blocks, int block_size, int top_k, int64_t* topk_idx,
                                  int64_t* topk_slots, float* softmax_m, float* softmax_inv_z, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  JF_CHECK_ARG(H_q > 0 && top_k > 0, "topk_slots_fast: bad shape");
  const int G = (H_q % 4 == 0) ? 4 : ((H_q % 2 == 0) ? 2 : 1);
  return fused_run<FS_TOPK>(JF_SCHEME_K4V4, 128, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, block_table, seq_lens, B, H_q,
                            H_q / G, max_S, max_blocks, (int64_t)1 << 25, block_size, 0.0f, top_k, topk_idx, topk_slots,
                            nullptr, nullptr, nullptr, softmax_m, softmax_inv_z, nullptr, scores, nullptr, nullptr,
                            workspace, workspace_bytes, stream);
}

// Workspace of jf_topk_slots_fast (the grouping is its own).
extern "C" size_t jf_topk_slots_fast_workspace_bytes(int B, int H_q, int max_S, int top_k) {
  if (H_q <= 0) return 256;
  const int G = (H_q % 4 == 0) ? 4 : ((H_q % 2 == 0) ? 2 : 1);
  return jf_fused_workspace_bytes(JF_SCHEME_K4V4, B, H_q, H_q / G, max_S, top_k);
}
