/*
 * jetfire_amd.h — C ABI of the MI355X (gfx950) implementation of JetFire's GPU
 * approximate-attention decode path.
 *
 * Every entry point takes plain device/host pointers, sizes and a HIP stream
 * (passed as void*; NULL = the default stream).  Kernels are enqueued
 * asynchronously on that stream.  Return value: 0 on success, a negative
 * JF_ERR_* code otherwise; jf_last_error() returns the message for the calling
 * thread (the reference raises RuntimeError through TORCH_CHECK at the same
 * places).
 *
 * Layouts are the reference's (jetfire_vllm/adapter/cache_store.py:240-284):
 *   K/V data   (H_kv, num_slots, P)  uint8, P = 32 (INT2) / 48 (INT3 planar) / 64 (INT4)
 *   K/V scales (H_kv, num_slots, NG) bf16,  NG = 128 / group_size
 *   block_table (B, max_blocks) int64, seq_lens (B,) int32, block size 16
 *   slot = block_table[b, pos / 16] * 16 + pos % 16
 * bf16 values are passed as uint16_t bit patterns.  head_dim is 128 throughout.
 */
#ifndef JETFIRE_AMD_H
#define JETFIRE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JF_OK 0
#define JF_ERR_ARG (-1)      /* unsupported shape / argument (reference: TORCH_CHECK) */
#define JF_ERR_HIP (-2)      /* HIP runtime error */
#define JF_ERR_STATE (-3)    /* bad handle / wrong call order */
#define JF_ERR_TIMEOUT (-4)  /* CPU correction did not finish in time */

#define JF_SCHEME_K3V2 32    /* INT3 keys, INT2 values  (SymInt3K_SymInt2V) */
#define JF_SCHEME_K4V4 44    /* INT4 keys, INT4 values  (SymInt4K_SymInt4V) */
#define JF_SCHEME_K3V4 34    /* INT3 keys, INT4 values  (SymInt3K_SymInt4V), group 64 or 128 */
#define JF_SCHEME_K4V2 42    /* INT4 keys, INT2 values  (SymInt4K_SymInt2V), group 128 */
#define JF_SCHEME_K2V2 22    /* INT2 keys, INT2 values  (SymInt2K_SymInt2V), group 64 or 128 */
#define JF_SCHEME_K2V4 24    /* INT2 keys, INT4 values  (SymInt2K_SymInt4V), group 64 or 128 */
#define JF_SCHEME_K2V3 23    /* INT2 keys, INT3 values  (SymInt2K_SymInt3V), group 64 or 128 */
#define JF_SCHEME_K3V3 33    /* INT3 keys, INT3 values  (SymInt3K_SymInt3V), group 64 or 128 */
#define JF_SCHEME_K4V3 43    /* INT4 keys, INT3 values  (SymInt4K_SymInt3V), group 128 */
/* asymmetric INT2 keys (four levels, a zero-point per group: k_zp), key digit 1 */
#define JF_SCHEME_A2V2 12    /* (AsymInt2K4Level_SymInt2V), group 64 or 128 */
#define JF_SCHEME_A2V3 13    /* (AsymInt2K4Level_SymInt3V), group 64 or 128 */
#define JF_SCHEME_A2V4 14    /* (AsymInt2K4Level_SymInt4V), group 64 or 128 */
/* INT4 keys scored with the bf16 model of int4_qk_scores (jetfire_vllm/csrc/int4_qk_scores.cu:68-80) instead of the
 * int8-Q model: what the reference runs for INT4 keys with 64-channel groups (decode_path.py:2016-2022); key digit 5 */
#define JF_SCHEME_B4V2 52    /* (SymInt4K_SymInt2V), group 64 or 128 */
#define JF_SCHEME_B4V3 53    /* (SymInt4K_SymInt3V), group 64 or 128 */
#define JF_SCHEME_B4V4 54    /* (SymInt4K_SymInt4V), group 64 or 128 */

const char* jf_last_error(void);
const char* jf_version(void);

/* ------------------------------------------------------------------ piece 1: quantise-on-append
 * Replaces fused_quant_write_int{2,3,4}_sym (jetfire_vllm/kernels/fused_quant_write.py:242-270,
 * 337-369, 746-781): per (token, kv-head) and per group: scale = bf16(max(amax/qmax, 1e-8)),
 * code = clamp(rint(x / f32(scale)), +-qmax) + 2^(nbits-1), packed in the reference wire format and
 * scattered to out_data[h, slots[t], :], out_scale[h, slots[t], g].  slots[t] < 0 skips the token.
 * x is (T, H_kv, 128) bf16 with element strides x_stride_t / x_stride_h (last dim contiguous).
 * Data strides are in bytes, scale strides in bf16 elements.  nbits in {2,3,4};
 * group_size in {32, 64, 128}. */
int jf_quant_write_sym(const uint16_t* x, int64_t x_stride_t, int64_t x_stride_h,
                       const int64_t* slots, int64_t T, int H_kv,
                       uint8_t* out_data, int64_t data_stride_h, int64_t data_stride_slot,
                       uint16_t* out_scale, int64_t scale_stride_h, int64_t scale_stride_slot,
                       int64_t num_slots, int group_size, int nbits, void* stream);

/* Asymmetric INT2 keys over the full codebook.  Replaces fused_quant_write_int2_asym
 * (jetfire_vllm/kernels/fused_quant_write.py:36-133,204-239; golden form quantize_and_pack_asym,
 * kernels/intN_pack.py:110-169): per group scale = bf16(max((xmax - xmin) / 3, 1e-8)),
 * zp = bf16(xmin + 2 * scale), code = clamp(rint((x - zp) / scale), -2, 1) + 2, INT2 wire format; out_zp is
 * (H_kv, num_slots, NG) bf16 with element strides.  Token rows must be 16-byte aligned. */
int jf_quant_write_int2_asym(const uint16_t* x, int64_t x_stride_t, int64_t x_stride_h, const int64_t* slots,
                             int64_t T, int H_kv, uint8_t* out_data, int64_t data_stride_h, int64_t data_stride_slot,
                             uint16_t* out_scale, int64_t scale_stride_h, int64_t scale_stride_slot,
                             uint16_t* out_zp, int64_t zp_stride_h, int64_t zp_stride_slot,
                             int64_t num_slots, int group_size, void* stream);

/* K and V of an INT4/INT4 cache in one launch.  Replaces fused_quant_write_int4_sym_kv
 * (jetfire_vllm/kernels/fused_quant_write.py:552-617). */
int jf_quant_write_int4_sym_kv(const uint16_t* key, int64_t k_stride_t, int64_t k_stride_h,
                               const uint16_t* value, int64_t v_stride_t, int64_t v_stride_h,
                               const int64_t* slots, int64_t T, int H_kv,
                               uint8_t* k_data, int64_t k_data_stride_h, int64_t k_data_stride_slot,
                               uint16_t* k_scale, int64_t k_scale_stride_h, int64_t k_scale_stride_slot,
                               uint8_t* v_data, int64_t v_data_stride_h, int64_t v_data_stride_slot,
                               uint16_t* v_scale, int64_t v_scale_stride_h, int64_t v_scale_stride_slot,
                               int64_t num_slots, int group_size, void* stream);

/* Dequantise packed rows back to bf16.  Replaces unpack (jetfire_vllm/kernels/intN_pack.py:227-311):
 * out[r, c] = bf16(f32(code - 2^(nbits-1)) * f32(scale[r, c / group_size])); when zps is not NULL the
 * rounded product is widened, f32(zp) added and the sum rounded to bf16 again (:251-256).  data is
 * (rows, 128 * nbits / 8) uint8 with a row stride in bytes; scales / zps are (rows, 128 / group_size) bf16 and
 * out is (rows, 128) bf16, their row strides in elements.  nbits in {2,3,4}; group_size a power of two in
 * 8..128; output rows 16-byte aligned, INT4 data rows 4-byte and INT2 data rows 2-byte aligned. */
int jf_unpack(const uint8_t* data, int64_t data_stride_row, const uint16_t* scales, int64_t scale_stride_row,
              const uint16_t* zps, int64_t zp_stride_row, int64_t rows, int group_size, int nbits,
              uint16_t* out, int64_t out_stride_row, void* stream);

/* Mirror of appended rows into the bf16 host shadow the CPU correction reads: k_shadow[h, slots[t], :] =
 * key[t, h, :], the same for V; slots[t] < 0 (padding) and slots[t] >= num_slots are skipped.  Replaces the
 * reference's shadow mirror: the serial host copy + index_copy_ (jetfire_vllm/adapter/cache_store.py:686-759),
 * the prefill pipeline's D2H into pinned staging buffers followed by a worker thread's scatter
 * (cache_store.py:1224-1338) and the graph-mode decode append (staging copies + host callback,
 * cache_store.py:531-642, jetfire_vllm/csrc/cpu_topk_attn.cpp:1611-1665).  Here the shadow is pinned host
 * memory the GPU addresses and ONE kernel stores the rows to it across PCIe; the launch is asynchronous, can
 * be captured in a HIP graph, and its rows are visible to the host when work enqueued after it on the same
 * stream runs (the hand-off's publish kernel) or the stream / an event recorded after it has been waited for.
 * key / value are (T, H_kv, 128) bf16 with element strides (last dim contiguous, rows 4-byte aligned);
 * k_shadow / v_shadow are DEVICE-VISIBLE addresses (jf_host_buffer_device_pointer) of (H_kv, num_slots, 128)
 * bf16 with element strides shadow_stride_h / shadow_stride_slot, rows 16-byte aligned. */
int jf_shadow_write(const uint16_t* key, int64_t k_stride_t, int64_t k_stride_h,
                    const uint16_t* value, int64_t v_stride_t, int64_t v_stride_h,
                    const int64_t* slots, int64_t T, int H_kv,
                    uint16_t* k_shadow, uint16_t* v_shadow, int64_t shadow_stride_h, int64_t shadow_stride_slot,
                    int64_t num_slots, void* stream);

/* Address under which the GPU reaches a pinned host buffer (hipHostMalloc, torch's pin_memory=True), or
 * JF_ERR_ARG when host_ptr is pageable or device memory.  The reference allocates its mapped buffers itself
 * (alloc_mapped_pinned_pair, jetfire_vllm/csrc/cpu_topk_attn.cpp:972-1023); here the caller owns them. */
int jf_host_buffer_device_pointer(const void* host_ptr, void** device_ptr);

/* ------------------------------------------------------------------ Stage A (split form)
 * scores[b, hq, s] for s < seq_len, -inf for seq_len <= s < max_S.
 * jf_int3_qk_scores replaces int3_qk_scores (jetfire_vllm/csrc/int3_qk_scores.cu:318-390):
 *   bf16 q times bf16-rounded dequantised INT3 keys, fp32 accumulate, times attn_scale.
 *   n_scale_groups in {1, 2}.
 * jf_int8tc_qk_scores replaces int8tc_qk_scores (jetfire_vllm/csrc/int8tc_qk_scores.cu:1263-1331):
 *   q quantised to int8 per (row, 32 channels), exact INT4 key codes, int32 accumulate,
 *   fp32 rescale  s = fma(a3,qs3, fma(a2,qs2, fma(a1,qs1, a0*qs0))); score = (s*ks)*attn_scale. */
int jf_int3_qk_scores(const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                      const int64_t* block_table, const int32_t* seq_lens,
                      int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                      int n_scale_groups, int block_size, float attn_scale,
                      float* scores, void* stream);
/* The bf16 model of jf_int3_qk_scores for any symmetric key width: k_nbits 2 replaces int2_qk_scores with an
 * empty k_zp (jetfire_vllm/csrc/int2_qk_scores.cu:279-420: codes - 2, four per byte MSB first), 3 is
 * jf_int3_qk_scores, 4 replaces int4_qk_scores (jetfire_vllm/csrc/int4_qk_scores.cu:280-420: nibbles - 8,
 * (even << 4) | odd).  k_data (H_kv, num_slots, 16 * k_nbits), k_scales (H_kv, num_slots, n_scale_groups).
 * k_zp: NULL for symmetric keys; for the asymmetric INT2 keys (AsymInt2K4Level schemes) the zero-points
 * (H_kv, num_slots, n_scale_groups) bf16: keys are bf16(fma(code - 2, scale, zp)). */
int jf_intn_qk_scores(int k_nbits, const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                      const uint16_t* k_zp, const int64_t* block_table, const int32_t* seq_lens, int B, int H_q, int H_kv,
                      int max_S, int max_blocks, int64_t num_slots, int n_scale_groups, int block_size,
                      float attn_scale, float* scores, void* stream);
int jf_int8tc_qk_scores(const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                        const int64_t* block_table, const int32_t* seq_lens,
                        int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                        int block_size, float attn_scale,
                        float* scores, void* stream);

/* Exact top-k per (b, query head) over scores[b, hq, :min(max_S, seq_len)] by radix select on the
 * order-preserving key of the fp32 score; ties at the threshold go to the lower position; winners
 * are written in ascending position, the rest of the K lanes are -1; topk_slots is the paged slot of
 * each winner.  Replaces topk_slots_kernel_v5 (jetfire_vllm/csrc/int3_qk_scores.cu:426-554), whose
 * emission order and tie choice are arbitrary.  If softmax_m / softmax_inv_z are non-NULL they
 * receive the row max (0 if not finite) and 1/sum(exp(s-m)) (0 if the sum is not positive), as
 * topk_slots_stats_kernel_v5 does (jetfire_vllm/csrc/int8tc_qk_scores.cu:1678-1823).
 * top_k must be a power of two in [32, 8192]; max_S <= 262144. */
int jf_topk_slots(const float* scores, const int32_t* seq_lens, const int64_t* block_table,
                  int B, int H_q, int max_S, int max_blocks, int block_size, int top_k,
                  int64_t* topk_idx, int64_t* topk_slots,
                  float* softmax_m, float* softmax_inv_z, void* stream);

/* ------------------------------------------------------------------ Stage B (split form)
 * o_hat = sum_s p_s Vhat_s, o_old_unnorm = sum_{s in topk} p_s Vhat_s, W = sum_{s in topk} p_s with
 * p = exp(score - m) * inv_z and Vhat = (code - offset) * f32(scale) (no bf16 rounding).
 * Replaces int2_softmax_v_with_pre_corr_wvs2 (jetfire_vllm/csrc/int2_softmax_v.cu:792-901) for
 * v_nbits == 2 and int4_softmax_v_with_pre_corr_wvs2_scores (jetfire_vllm/csrc/int4_softmax_v.cu:
 * 2203-2235) for v_nbits == 4.  softmax_m / softmax_inv_z may be NULL (computed internally), or the
 * Stage-A statistics (int4_softmax_v_with_pre_corr_wvs2_scores; the int8-weight form of
 * int8tc_softmax_v_with_pre_corr_reg_stats is jf_softmax_v_int8_tiles below).  topk_idx may be NULL (o_hat only).
 * Split partials are reduced in a fixed order, so the result is run-to-run deterministic.
 * workspace: jf_softmax_v_workspace_bytes() bytes of device memory. */
size_t jf_softmax_v_workspace_bytes(int B, int H_q, int max_S);
int jf_softmax_v_pre_corr(const float* scores, const float* softmax_m, const float* softmax_inv_z,
                          const uint8_t* v_data, const uint16_t* v_scales,
                          const int64_t* block_table, const int32_t* seq_lens, const int64_t* topk_idx,
                          int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                          int block_size, int top_k, int v_nbits, int n_scale_groups,
                          float* o_hat, float* o_old_unnorm, float* W,
                          void* workspace, size_t workspace_bytes, void* stream);

/* INT4 values with int8-quantised softmax weights: replaces int8tc_softmax_v_with_pre_corr_reg_stats
 * (jetfire_vllm/csrc/int8tc_softmax_v_fused.cu:1017-1401 kernel, :1591-1734 launcher) with its arithmetic: eight
 * ranges of ceil(max_S / 8) positions, tiles of two pages starting at the page of a range's first position, per
 * tile and row rs = max|p * v_scale| / 127, pq = clamp(rint(p * v_scale / rs), -127, 127), o_hat += f32(sum pq *
 * (nibble - 8)) * rs (:1203-1236, 1298-1311); o_old_unnorm and W with exact fp32 weights (:1340-1400).  Needs the
 * Stage-A statistics and one V scale per token (group 128).  The ranges' partial sums are added in ascending order
 * (the reference adds them with atomics).  workspace: jf_softmax_v_workspace_bytes() bytes. */
int jf_softmax_v_int8_tiles(const float* scores, const float* softmax_m, const float* softmax_inv_z,
                            const uint8_t* v_data, const uint16_t* v_scales,
                            const int64_t* block_table, const int32_t* seq_lens, const int64_t* topk_idx,
                            int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                            int block_size, int top_k,
                            float* o_hat, float* o_old_unnorm, float* W,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ pieces 2+3: fused decode scan + top-k
 * One pass over the packed K and V of every (sequence, kv-head): Q.K^T for the GQA group, softmax
 * statistics, P.V, and exact top-k, without a (B, H_q, max_S) score tensor in HBM.  Produces what the
 * reference's Stage A + Stage B pair produces (jetfire_vllm/adapter/decode_path.py:2081-2131,
 * 2785-2935): topk_idx, topk_slots, o_hat, o_old_unnorm, W, and optionally softmax_m / softmax_inv_z.
 * The reference's own single-call form of this contract is int2_fused_attn_topk
 * (jetfire_vllm/kernels/int2_fused_attn_topk.py:5-10).  scheme: any of the nine symmetric pairs JF_SCHEME_K{2,3,4}V{2,3,4}
 * (the reference's kernel sets jetfire_vllm/kernels/_dispatch/sym_int*_k_sym_int*_v.py); pairs with INT4 keys (one key
 * scale per row) take group 128, the others group 64 or 128.  INT3 and symmetric INT2 keys score with the bf16 model of
 * jf_int3_qk_scores / jf_intn_qk_scores (jetfire_vllm/csrc/int2_qk_scores.cu:66-79), INT4 keys with the int8-Q model
 * of jf_int8tc_qk_scores; INT3 values are the planar rows of jetfire_vllm/csrc/int3_softmax_v.cu:43,282-284.
 * top_k: power of two in [32, 8192]; num_slots at most 2^26 (row
 * offsets are 32-bit).  If scores is non-NULL the fp32 scores are also written (validation).
 * workspace: jf_fused_workspace_bytes() bytes of device memory. */
size_t jf_fused_workspace_bytes(int scheme, int B, int H_q, int H_kv, int max_S, int top_k);
int jf_fused_scan_topk(int scheme, int group_size,
                       const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                       const uint8_t* v_data, const uint16_t* v_scales,
                       const int64_t* block_table, const int32_t* seq_lens,
                       int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                       int block_size, float attn_scale, int top_k,
                       int64_t* topk_idx, int64_t* topk_slots,
                       float* o_hat, float* o_old_unnorm, float* W,
                       float* softmax_m, float* softmax_inv_z, float* scores,
                       void* workspace, size_t workspace_bytes, void* stream);

/* jf_fused_scan_topk followed by the blend of jf_blend_unnorm (jetfire_vllm/csrc/blend.cu:202-226) inside the
 * merge kernel, for callers that hold the correction term already when the step is enqueued (a path without CPU
 * correction passes zeros): out = bf16(fma(W, o_new, o_hat) - o_old_unnorm), o_new and out (B, H_q, 128) bf16.
 * Every other output is written as by jf_fused_scan_topk; out is bit-equal to the separate blend. */
int jf_fused_scan_topk_blend(int scheme, int group_size,
                             const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                             const uint8_t* v_data, const uint16_t* v_scales,
                             const int64_t* block_table, const int32_t* seq_lens,
                             int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                             int block_size, float attn_scale, int top_k,
                             int64_t* topk_idx, int64_t* topk_slots,
                             float* o_hat, float* o_old_unnorm, float* W,
                             float* softmax_m, float* softmax_inv_z, float* scores,
                             const uint16_t* o_new, uint16_t* out,
                             void* workspace, size_t workspace_bytes, void* stream);

/* The fused step for the asymmetric INT2 keys (the reference's kernel sets
 * jetfire_vllm/kernels/_dispatch/int2_asym_k_sym_v.py, int2_asym_k_sym_int3_v.py, int2_asym_k_sym_int4_v.py): scheme
 * JF_SCHEME_A2V2 / JF_SCHEME_A2V3 / JF_SCHEME_A2V4 (group 64 or 128); k_zp (H_kv, num_slots, 128/group)
 * bf16 holds the zero-points; keys score with khat = bf16(fma(code - 2, scale, zp))
 * (jetfire_vllm/csrc/int2_qk_scores.cu:66-79).  o_new / out as in jf_fused_scan_topk_blend, or both NULL (no blend).
 * Everything else as jf_fused_scan_topk. */
int jf_fused_scan_topk_asym(int scheme, int group_size,
                            const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales, const uint16_t* k_zp,
                            const uint8_t* v_data, const uint16_t* v_scales,
                            const int64_t* block_table, const int32_t* seq_lens,
                            int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                            int block_size, float attn_scale, int top_k,
                            int64_t* topk_idx, int64_t* topk_slots,
                            float* o_hat, float* o_old_unnorm, float* W,
                            float* softmax_m, float* softmax_inv_z, float* scores,
                            const uint16_t* o_new, uint16_t* out,
                            void* workspace, size_t workspace_bytes, void* stream);

/* Stage A alone and Stage B alone on the kernels of the fused step, for callers that keep the reference's two-call
 * structure (jetfire_vllm/adapter/decode_path.py:2081-2131 then :2804-2935): the same results as the split entry
 * points above for the shapes the fused step supports (head_dim 128, block_size 16, H_q/H_kv from 1 to 16,
 * num_slots <= 2^26), at a fraction of their time.  workspace: jf_fused_workspace_bytes(format, ...).
 *
 * jf_stage_a_topk replaces int3_qk_scores / int3_qk_scores_topk (jetfire_vllm/csrc/int3_qk_scores.cu:640-655;
 * key_format JF_SCHEME_K3V2: INT3 keys, bf16 model, group 64 or 128), int2_qk_scores / int2_qk_scores_topk with
 * symmetric keys (jetfire_vllm/csrc/int2_qk_scores.cu:663-680; key_format JF_SCHEME_K2V2) and int8tc_qk_scores / _topk / _topk_stats
 * (jetfire_vllm/csrc/int8tc_qk_scores.cu:2774-2798; key_format JF_SCHEME_K4V4: INT4 keys, int8-Q model, group 128).
 * scores (B, H_q, max_S) may be NULL (not written); softmax_m / softmax_inv_z may be NULL.  top_k == 0: scores alone
 * (topk_idx, topk_slots and the workspace are then unused). */
int jf_stage_a_topk(int key_format, int group_size,
                    const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                    const int64_t* block_table, const int32_t* seq_lens,
                    int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                    int block_size, float attn_scale, int top_k,
                    float* scores, int64_t* topk_idx, int64_t* topk_slots,
                    float* softmax_m, float* softmax_inv_z,
                    void* workspace, size_t workspace_bytes, void* stream);
/* jf_stage_a_topk for the asymmetric INT2 keys: int2_qk_scores / int2_qk_scores_topk with k_zp
 * (jetfire_vllm/csrc/int2_qk_scores.cu:66-79, 663-680); group 64 or 128; workspace:
 * jf_fused_workspace_bytes(JF_SCHEME_A2V2, ...). */
int jf_stage_a_topk_asym(int group_size,
                         const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales, const uint16_t* k_zp,
                         const int64_t* block_table, const int32_t* seq_lens,
                         int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                         int block_size, float attn_scale, int top_k,
                         float* scores, int64_t* topk_idx, int64_t* topk_slots,
                         float* softmax_m, float* softmax_inv_z,
                         void* workspace, size_t workspace_bytes, void* stream);
/* jf_topk_slots on the kernels of the fused step: the same outputs as jf_topk_slots, i.e.
 * topk_slots_kernel_v5 / topk_slots_stats_kernel_v5 (jetfire_vllm/csrc/int3_qk_scores.cu:426-554,
 * jetfire_vllm/csrc/int8tc_qk_scores.cu:1678-1823).  workspace: jf_topk_slots_fast_workspace_bytes(). */
size_t jf_topk_slots_fast_workspace_bytes(int B, int H_q, int max_S, int top_k);
int jf_topk_slots_fast(const float* scores, const int32_t* seq_lens, const int64_t* block_table,
                       int B, int H_q, int max_S, int max_blocks, int block_size, int top_k,
                       int64_t* topk_idx, int64_t* topk_slots, float* softmax_m, float* softmax_inv_z,
                       void* workspace, size_t workspace_bytes, void* stream);
/* jf_stage_b_softmax_v replaces int2_softmax_v_with_pre_corr_wvs2 (jetfire_vllm/csrc/int2_softmax_v.cu:792-901;
 * value_format JF_SCHEME_K3V2: INT2 values, group 64 or 128), int3_softmax_v_with_pre_corr_wvs2
 * (jetfire_vllm/csrc/int3_softmax_v.cu:752-860; value_format JF_SCHEME_K3V3: INT3 values, group 64 or 128) and
 * int4_softmax_v_with_pre_corr_wvs2_scores
 * (jetfire_vllm/csrc/int4_softmax_v.cu:2203-2235; value_format JF_SCHEME_K4V4: INT4 values, group 128, or
 * JF_SCHEME_K3V4: INT4 values, group 64 or 128), with exact
 * fp32 softmax weights computed from `scores`.  topk_idx (B, H_q, top_k), ascending and -1 padded, may be NULL
 * (o_hat only; o_old_unnorm and W are then zero). */
int jf_stage_b_softmax_v(int value_format, int group_size,
                         const float* scores, const uint8_t* v_data, const uint16_t* v_scales,
                         const int64_t* block_table, const int32_t* seq_lens, const int64_t* topk_idx,
                         int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                         int block_size, int top_k,
                         float* o_hat, float* o_old_unnorm, float* W,
                         void* workspace, size_t workspace_bytes, void* stream);

/* jf_fused_scan_topk without the workspace arguments, for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  The workspace is a fixed array of JF_FUSED_STATIC_SCRATCH_BYTES in device memory that each
 * GPU the library runs on holds until the process ends; its address is looked up once per device on the first
 * call there (make that call outside a capture).  The call itself allocates and frees nothing.  Shapes whose
 * jf_fused_workspace_bytes() exceeds the array are rejected with JF_ERR_ARG.  Every call on a GPU shares that
 * GPU's array, so calls that overlap on one GPU (two streams, two threads) race; calls ordered on one stream
 * are safe, and nothing in the array has to be cleared between calls (every call rewrites what it reads).
 * Same kernels, same results as jf_fused_scan_topk. */
#define JF_FUSED_STATIC_SCRATCH_BYTES (64u << 20)
int jf_fused_scan_topk_static(int scheme, int group_size,
                              const uint16_t* q, const uint8_t* k_data, const uint16_t* k_scales,
                              const uint8_t* v_data, const uint16_t* v_scales,
                              const int64_t* block_table, const int32_t* seq_lens,
                              int B, int H_q, int H_kv, int max_S, int max_blocks, int64_t num_slots,
                              int block_size, float attn_scale, int top_k,
                              int64_t* topk_idx, int64_t* topk_slots,
                              float* o_hat, float* o_old_unnorm, float* W,
                              float* softmax_m, float* softmax_inv_z, float* scores, void* stream);

/* Introspection with no counterpart in the reference: the launch geometry jf_fused_scan_topk uses for a
 * shape.  split_len positions per scan workgroup, n_splits = ceil(max_S / split_len) workgroups per
 * (sequence, kv-head), list_cap candidate slots per (row, split), merge_parts > 1 if the candidate lists are
 * first reduced by that many workgroups per row.  Any output pointer may be NULL.  Needs no GPU. */
int jf_fused_plan(int scheme, int group_size, int B, int H_q, int H_kv, int max_S, int top_k,
                  int* split_len, int* n_splits, int* list_cap, int* merge_parts);

/* Measurement and test hooks (kernel timing by HIP events, phase stamps, a forced split length, pool stalls ...)
 * are declared in jetfire_amd_debug.h and exist only in a library built with -DJF_DEBUG_HOOKS. */

/* ------------------------------------------------------------------ piece 4: merge
 * out = bf16_rne(fma(W, f32(o_new), o_hat) - o_old_unnorm).  Replaces blend_unnorm_into
 * (jetfire_vllm/csrc/blend.cu:202-290).  o_new / out are (B, H_q, D) bf16. */
int jf_blend_unnorm(const float* o_hat, const float* o_old_unnorm, const float* W,
                    const uint16_t* o_new, uint16_t* out, int B, int H_q, int D, void* stream);

/* out = bf16_rne(fma(W, f32(o_new) - o_old, o_hat)) with a NORMALISED o_old: replaces blend / blend_into
 * (jetfire_vllm/csrc/blend.cu:44-66, 68-190). */
int jf_blend(const float* o_hat, const float* o_old, const float* W,
             const uint16_t* o_new, uint16_t* out, int B, int H_q, int D, void* stream);

/* ------------------------------------------------------------------ piece 4: CPU correction + hand-off
 * Exact softmax attention over the top-k slots from the host bf16 shadow.  Replaces cpu_topk_attn
 * (jetfire_vllm/csrc/cpu_topk_attn.cpp:854-956; row kernel :602-690): invalid slots (<0 or
 * >= num_slots) score -inf, a row without a valid slot gives zeros, output rounded to bf16.
 * All pointers are host memory.  done_flag (nullable) is set to 1 after the outputs are visible. */
int jf_cpu_topk_attn(const uint16_t* q, const uint16_t* k_shadow, const uint16_t* v_shadow,
                     const int64_t* head_map, const int64_t* ts_buf, uint16_t* o_new,
                     int B, int H_q, int K, int H_kv, int64_t num_slots, float scale,
                     int64_t* done_flag);
int jf_set_cpu_attn_threads(int n);   /* set_cpu_attn_threads (cpu_topk_attn.cpp:2509-2530) */
int jf_get_cpu_attn_threads(void);

/* Pinned hand-off context: replaces create_cpu_topk_submit_ctx / stream_submit_cpu_topk_attn /
 * stream_wait_cpu_topk_attn (jetfire_vllm/csrc/cpu_topk_attn.cpp:2054-2163, 2239, 2302) and the
 * pinned copies around them (jetfire_vllm/adapter/decode_path.py:2243-2267, 3107-3114).
 * submit: enqueues one small kernel on `stream` that copies q and topk_slots (both 16-byte aligned,
 *         K a multiple of 4; the slots cross PCIe as 32-bit values) into pinned host buffers and then raises a sequence flag in pinned memory; a
 *         dispatcher thread of the context polls that flag and runs the CPU correction on the worker
 *         pool as soon as the GPU has reached it.  Returns at once.
 * wait:   blocks the calling host thread until the correction of the last submit has finished (as the
 *         reference blocks on its future; JETFIRE_CPU_FUTURE_TIMEOUT_S, default 30 s, then
 *         JF_ERR_TIMEOUT), then enqueues a small kernel on `stream` that brings o_new from the pinned
 *         buffer into o_new_dev (16-byte aligned).  Not capturable into a HIP graph.
 * One job per context may be in flight: a submit while the previous correction still runs is rejected
 * (JF_ERR_ARG); destroy waits for an outstanding one.  Leave two host cores
 * to the caller and the dispatcher when sizing the worker pool (jf_set_cpu_attn_threads). */
typedef struct jf_handoff jf_handoff;
jf_handoff* jf_handoff_create(int B, int H_q, int H_kv, int K, int64_t num_slots,
                              const uint16_t* k_shadow_host, const uint16_t* v_shadow_host, float scale);
int jf_handoff_submit(jf_handoff* h, const uint16_t* q_dev, const int64_t* topk_slots_dev, void* stream);
int jf_handoff_wait(jf_handoff* h, uint16_t* o_new_dev, void* stream);
int64_t jf_handoff_submit_count(const jf_handoff* h);
void jf_handoff_destroy(jf_handoff* h);

/* Stream mode of the same context: the graph-capturable pair.  Replaces the reference's host-callback
 * submit / join (graph_submit_callback / graph_join_callback and stream_write_value64 / stream_wait_value64,
 * jetfire_vllm/csrc/cpu_topk_attn.cpp:1805-2016, 1293-1344) without any host callback or stream memory
 * operation: both calls only enqueue kernels, so a captured graph replays them with no host code in between.
 * stream_submit: the publish kernel of jf_handoff_submit, except that the sequence number comes from a counter
 *         in device memory which the kernel advances itself; from the first call on, ONE poller thread of the
 *         process (shared by every stream-mode context: a model has one per layer and batch size) looks at the
 *         context's pinned flag, with sleeps that lengthen while the GPU is silent, and runs the correction.
 * stream_wait: one workgroup whose first lane polls the pinned "finished" word until the correction of the
 *         device's current sequence number is done, then copies o_new into o_new_dev.  The wait is bounded
 *         (min(JETFIRE_CPU_FUTURE_TIMEOUT_S, 10 s); jf_handoff_set_device_wait_limit_us): at the limit the
 *         kernel raises a status word, writes zeros to o_new_dev and ends; every later wait of the context
 *         falls through at once.  jf_handoff_status reports it (JF_ERR_TIMEOUT) after the stream has been
 *         synchronised; jf_handoff_stream_submit refuses a failed context.
 * A context serves one mode: mixing the pairs is JF_ERR_ARG.  Calls of one context must be ordered on one
 * stream (submit, wait, submit, ...).  Destroy a stream-mode context only when no graph that holds its kernels
 * will be replayed again; destroy synchronises the device first. */
int jf_handoff_stream_submit(jf_handoff* h, const uint16_t* q_dev, const int64_t* topk_slots_dev, void* stream);
int jf_handoff_stream_wait(jf_handoff* h, uint16_t* o_new_dev, void* stream);
/* stream_wait followed by the blend of jf_blend_unnorm in the same kernel: out = bf16(fma(W, o_new, o_hat) -
 * o_old_unnorm) on the elements as they arrive (at the wait's limit o_new counts as zero).  o_new_dev may be
 * NULL when the caller has no use for the correction itself. */
int jf_handoff_stream_wait_blend(jf_handoff* h, const float* o_hat, const float* o_old_unnorm, const float* W,
                                 uint16_t* out, uint16_t* o_new_dev, void* stream);
int jf_handoff_status(jf_handoff* h);
int jf_handoff_set_device_wait_limit_us(jf_handoff* h, int64_t us);
/* on != 0: jf_handoff_stream_wait_blend writes zero for every non-finite output element, the graph-mode guard of
 * _sanitize_decode_output_if_needed (jetfire_vllm/adapter/decode_path.py:1133-1149) folded into the blend. */
int jf_handoff_set_output_sanitize(jf_handoff* h, int on);

/* Row implementation of the CPU correction: 0 scalar (cpu_topk_attn.cpp:602-690), 1 AVX2+FMA, 2 AVX-512-BF16
 * (vdpbf16ps row, jetfire_vllm/csrc/cpu_topk_attn.cpp:316-479).  The widest one the host supports is used unless
 * JETFIRE_CPU_ATTN_ISA (scalar | avx2 | avx512bf16) or jf_set_cpu_attn_isa asks for a narrower one (-1: widest).
 * An output row that comes out non-finite is recomputed by the scalar row and zeroed if it still is; the count
 * of such rows is get_cpu_topk_sanitize_count (cpu_topk_attn.cpp:809-826, 2643). */
int jf_set_cpu_attn_isa(int isa);
int jf_get_cpu_attn_isa(void);
int64_t jf_cpu_topk_sanitize_count(void);

/* The reference's own submit-context interface (jetfire_vllm/csrc/cpu_topk_attn.cpp:2054-2163
 * create_cpu_topk_submit_ctx, :2239 stream_submit_cpu_topk_attn, :2302 stream_wait_cpu_topk_attn): the caller owns
 * pinned host buffers q (B, H_q, 128) bf16, head_map / ts_buf (B, H_q, K) int64 and o_new (B, H_q, 128) bf16 and
 * fills q / ts_buf with its own stream-ordered copies (jetfire_vllm/adapter/decode_path.py:2243-2267); a context
 * remembers the pointers.  stream_submit enqueues a one-lane kernel that raises the context's sequence flag in
 * pinned memory, in stream order behind those copies; the shared poller thread then runs the correction into
 * o_new and stores 1 to flag_host (nullable).  stream_wait enqueues the bounded device-side wait of
 * jf_handoff_stream_wait (without a copy: the caller's own H2D copy of o_new follows it).  Both are kernels only
 * and can be captured into a HIP graph.  Handles are positive integers, 0 on error; they stay valid until
 * jf_clear_graph_contexts.  jf_submit_ctx_status: as jf_handoff_status. */
int64_t jf_submit_ctx_create(const uint16_t* q_host, const uint16_t* k_shadow_host, const uint16_t* v_shadow_host,
                             const int64_t* head_map_host, const int64_t* ts_buf_host, uint16_t* o_new_host,
                             int B, int H_q, int K, int H_kv, int64_t num_slots, float scale, int64_t* flag_host);
int jf_submit_ctx_stream_submit(int64_t ctx, void* stream);
int jf_submit_ctx_stream_wait(int64_t ctx, void* stream);
int jf_submit_ctx_status(int64_t ctx);
/* stream_write_value64 / stream_wait_value64 (jetfire_vllm/csrc/cpu_topk_attn.cpp:1293-1344) as one-lane kernels:
 * store `value` to a device-visible word with system scope / poll it until it equals `value`.  The wait is bounded
 * by min(JETFIRE_CPU_FUTURE_TIMEOUT_S, 10 s); jf_stream_wait_timeouts counts waits that ran into the bound. */
int jf_stream_write_value64(void* stream, int64_t* flag_device, int64_t value);
int jf_stream_wait_value64(void* stream, const int64_t* flag_device, int64_t value);
int64_t jf_stream_wait_timeouts(void);
/* submit_cpu_topk_attn_async / wait_for_flag (jetfire_vllm/csrc/cpu_topk_attn.cpp:1184-1260): jf_cpu_topk_attn on an
 * executor thread, returns at once; 1 is stored to `flag` when o_new is complete.  wait_for_flag spins, then sleeps in
 * short steps, until the flag is non-zero (timeout_s <= 0: forever). */
int jf_cpu_topk_attn_async(const uint16_t* q, const uint16_t* k_shadow, const uint16_t* v_shadow,
                           const int64_t* head_map, const int64_t* ts_buf, uint16_t* o_new,
                           int B, int H_q, int K, int H_kv, int64_t num_slots, float scale, int64_t* flag);
int jf_wait_for_flag(const int64_t* flag, double timeout_s);
/* graph_pool_warmup[_threads], get_graph_submit_count, reset_graph_runtime_state, clear_graph_contexts
 * (jetfire_vllm/csrc/cpu_topk_attn.cpp:2620-2660): start (n_threads > 0: resize) the worker pool; number of
 * stream-mode submits the poller has served; reset the counters; destroy every submit context (only when no
 * graph that holds their kernels will be replayed again). */
int jf_graph_pool_warmup(int n_threads);
int64_t jf_graph_submit_count(void);
int jf_reset_graph_runtime_state(void);
int jf_clear_graph_contexts(void);
/* get_shadow_append_count (jetfire_vllm/csrc/cpu_topk_attn.cpp:2353-2355; read by jetfire_get_graph_stats,
 * jetfire_vllm/adapter/decode_path.py:1017-1023): launches of the shadow mirror kernel that have run on the current
 * device, replays from a HIP graph included (the reference counts its graph-mode append callbacks).  reset != 0
 * zeroes the counter after reading it.  Copies one word from the device: call it outside graph capture. */
int jf_shadow_append_count(int64_t* count, int reset);
/* reset_graph_submit_count (jetfire_vllm/csrc/cpu_topk_attn.cpp:2436-2470; called by reset_jetfire_graph_stats,
 * jetfire_vllm/adapter/decode_path.py:1041-1045): zeroes the submit, shadow-append and sanitise counters and the
 * timing statistics below. */
int jf_reset_graph_submit_count(void);
/* get_graph_timing_stats (jetfire_vllm/csrc/cpu_topk_attn.cpp:2361-2434) as an array of JF_GRAPH_TIMING_FIELDS
 * doubles: [0] topk_jobs (corrections run for hand-off contexts), [1] topk_done_avg_us, [2] topk_done_max_us (their
 * duration on the worker pool), [3] shadow_append_jobs, [4] join_jobs (host-blocking jf_handoff_wait calls),
 * [5] join_wait_avg_us, [6] join_wait_max_us, [7] pool_workers, [8] pool_done_count (jobs the pool has finished).
 * This library has no host callbacks, so the reference's submit-callback times and "last call" words do not exist. */
#define JF_GRAPH_TIMING_FIELDS 9
int jf_graph_timing_stats(double* out, int n);
/* No counterpart in the reference (its graph submit callback runs on a host thread and wakes the pool itself):
 * jf_pool_wake brings sleeping workers of the correction pool back to spinning for the next job; jf_pool_doorbell
 * enqueues a one-lane kernel on `stream` (capturable) that has the poller thread do the same when the GPU reaches
 * it - put it at the head of a decode step so that the first layer's correction does not pay the pool's wake-up. */
int jf_pool_wake(void);
int jf_pool_doorbell(void* stream);

#ifdef __cplusplus
}
#endif
#endif /* JETFIRE_AMD_H */
