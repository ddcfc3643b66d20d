// Stage B alone on the kernels of the fused step: the scores and the winners are inputs; one pass over the packed
// values yields o_hat and the pre-correction terms.  The fast form of the reference's
// int2_softmax_v_with_pre_corr_wvs2 (jetfire_vllm/csrc/int2_softmax_v.cu:792-901),
// int3_softmax_v_with_pre_corr_wvs2 (jetfire_vllm/csrc/int3_softmax_v.cu:752-860) and
// int4_softmax_v_with_pre_corr_wvs2_scores (jetfire_vllm/csrc/int4_softmax_v.cu:2203-2235) for the shapes the fused
// step supports.
#include "fused_scan_impl.h"

using namespace jf;

extern "C" int jf_stage_b_softmax_v(int value_format, int group_size, const float* scores, const uint8_t* v_data,
                                    const uint16_t* v_scales, const int64_t* block_table, const int32_t* seq_lens,
                                    const int64_t* topk_idx, int B, int H_q, int H_kv, int max_S, int max_blocks,
                                    int64_t num_slots, int block_size, int top_k, float* o_hat, float* o_old_unnorm,
                                    float* W, void* workspace, size_t workspace_bytes, void* stream) {
  JF_CHECK_ARG(value_format == JF_SCHEME_K3V2 || value_format == JF_SCHEME_K3V3 || value_format == JF_SCHEME_K4V4 ||
                   value_format == JF_SCHEME_K3V4,
               "stage_b_softmax_v: value_format must be JF_SCHEME_K3V2 (INT2 values), JF_SCHEME_K3V3 (INT3 values), "
               "JF_SCHEME_K4V4 (INT4 values, group 128) or JF_SCHEME_K3V4 (INT4 values, group 64 or 128)");
  return fused_run<FS_STAGE_B>(value_format, group_size, nullptr, nullptr, nullptr, nullptr, v_data, v_scales, block_table,
                               seq_lens, B, H_q, H_kv, max_S, max_blocks, num_slots, block_size, 0.0f, top_k,
                               const_cast<int64_t*>(topk_idx), nullptr, o_hat, o_old_unnorm, W, nullptr, nullptr, nullptr,
                               scores, nullptr, nullptr, workspace, workspace_bytes, stream);
}

int jf::precorr_int4_given_stats(const float* scores, const float* softmax_m, const float* softmax_inv_z,
                                 const uint8_t* v_data, const uint16_t* v_scales, const int64_t* block_table,
                                 const int32_t* seq_lens, const int64_t* topk_idx, int B, int H_q, int H_kv, int max_S,
                                 int max_blocks, int64_t num_slots, int top_k, float* o_old_unnorm, float* W,
                                 void* stream) {
  return launch_precorr_given_stats<4, 1>(scores, softmax_m, softmax_inv_z, v_data, v_scales, block_table, seq_lens,
                                          topk_idx, B, H_q, H_kv, max_S, max_blocks, num_slots, top_k, o_old_unnorm, W,
                                          (hipStream_t)stream);
}
