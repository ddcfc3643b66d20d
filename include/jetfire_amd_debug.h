/* jetfire_amd_debug.h - measurement and test hooks of libjetfire_amd.so.
 *
 * None of these has a counterpart in the reference, and none belongs to the product interface: they are compiled
 * into the library only when it is built with -DJF_DEBUG_HOOKS (`python -m jetfire_amd.build --debug-hooks`, which
 * the test and benchmark build uses; jf_version() then ends in "+debug-hooks").  A library built without the macro
 * exports none of them, so no process-wide switch can change its launch geometry.
 */
#ifndef JETFIRE_AMD_DEBUG_H
#define JETFIRE_AMD_DEBUG_H

#include "jetfire_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid with no counterpart in the reference: between begin and end, every launch of the fused
 * scan kernel is bracketed by a pair of HIP events recorded on the launch stream (at most max_launches
 * launches); end synchronises them and returns the summed device time and the number of launches. */
int jf_profile_scan_begin(int max_launches);
int jf_profile_scan_end(double* total_ms, int* launches);
/* Measurement aid with no counterpart in the reference: one kernel that streams `bytes` bytes from src with 16-byte
 * loads and writes nothing (sink: 4 bytes of device memory, may be NULL).  Its rate is the read-stream ceiling of
 * this machine, the figure the scan's achieved bandwidth is put beside. */
int jf_calibrate_stream_read(const void* src, size_t bytes, void* sink, void* stream);
/* Measurement aid: if device_buffer is non-NULL, every fused-scan workgroup stores ten int64 s_memtime
 * stamps of its phase boundaries at device_buffer[((b * H_kv + hkv) * n_splits + split) * 10 ...], and every
 * merge workgroup eight at device_buffer[B * H_kv * n_splits * 10 + (b * H_q + hq) * 8 ...] (which stamp
 * marks which boundary is internal to the kernels and may change).  NULL switches it off. */
int jf_debug_phase_clock(void* device_buffer);
/* Test / measurement aid with no counterpart in the reference: a positive split_len (rounded up to a
 * multiple of 256 and clamped to what fits the kernel's LDS) replaces the planner's choice of the split
 * length in jf_fused_scan_topk and jf_fused_workspace_bytes; 0 restores the planner.  Process-wide. */
int jf_debug_split_len(int split_len);
/* Test aids for the CPU pool, no counterpart in the reference.  jf_debug_pool_stall: the worker that claims `row` of
 * the next correction job sleeps `microseconds` before it computes the row (one shot), as if it had lost its core.
 * jf_debug_pool_wait_stragglers(0): jf_cpu_topk_attn returns as soon as every row is committed, like the hand-off
 * jobs do, instead of also waiting for workers that are still inside a row (the caller must then keep its tensors
 * alive); 1 restores the default. */
int jf_debug_pool_stall(int64_t row, int microseconds);
int jf_debug_pool_wait_stragglers(int on);
/* Measurement aid: device_buffer (capacity + 1 int64 words of device memory, zeroed by the caller) makes every
 * device-side wait launched from now on (jf_handoff_stream_wait[_blend], jf_submit_ctx_stream_wait; a graph captured
 * from now on keeps the pointer) add one to word 0 and store the time it waited, in ticks of the 100 MHz clock, to
 * word 1 + (n mod capacity).  NULL switches it off for later launches; the buffer must outlive every graph that
 * holds it. */
int jf_debug_wait_log(void* device_buffer, int capacity);
/* Test aid: while on, the dispatcher ignores published flags of the context (a correction that never finishes,
 * without hanging anything: the device-side wait runs into its limit). */
int jf_handoff_debug_pause(jf_handoff* h, int on);

#ifdef __cplusplus
}
#endif
#endif /* JETFIRE_AMD_DEBUG_H */
