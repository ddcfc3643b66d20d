// Mirror of appended bf16 K/V rows into the host shadow the CPU correction reads.
//
// The shadow lives in pinned host memory that the GPU can address, so one kernel stores every appended row
// straight to shadow[h, slots[t], :] across PCIe: no staging buffer, no host-side scatter, no host callback,
// and the launch can be recorded into a HIP graph like any other kernel.  Rows are 256 bytes and leave as
// 16-byte stores that are contiguous across the sixteen lanes of a row (consecutive slots give longer runs).
// Writes to pinned host memory are visible to the host once the kernel has completed.
#include "common.h"

namespace jf {
namespace {

struct MirrorSrc {
  const uint16_t* x;
  int64_t stride_t, stride_h;  // elements
};

// LPR lanes own one row: 16 lanes x 16 bytes, or 64 lanes x 4 bytes for rows that are only 4-byte aligned.
// Grid: x = blocks of 256 / LPR tokens, y = kv-head, z = tensor (K, V).
// Mirror launches that have run on this device, replays from a HIP graph included (the reference counts its
// graph-mode append callbacks, jetfire_vllm/csrc/cpu_topk_attn.cpp:1611-1616); device code only.
__device__ unsigned long long shadow_appends;

template <int LPR>
__global__ __launch_bounds__(256) void shadow_write_kernel(MirrorSrc k, MirrorSrc v, uint16_t* __restrict__ k_shadow,
                                                           uint16_t* __restrict__ v_shadow, int64_t stride_h,
                                                           int64_t stride_slot, const int64_t* __restrict__ slots,
                                                           int64_t T, int64_t num_slots) {
  constexpr int RPB = 256 / LPR;
  if ((blockIdx.x | blockIdx.y | blockIdx.z | threadIdx.x) == 0) atomicAdd(&shadow_appends, 1ull);
  const int l = threadIdx.x % LPR;
  const int64_t t = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
  if (t >= T) return;
  const int64_t slot = slots[t];
  if (slot < 0 || slot >= num_slots) return;  // padding tokens; a slot outside the shadow is never stored to
  const int h = blockIdx.y;
  const MirrorSrc& s = blockIdx.z ? v : k;
  uint16_t* shadow = blockIdx.z ? v_shadow : k_shadow;
  const uint16_t* src = s.x + t * s.stride_t + (int64_t)h * s.stride_h;
  uint16_t* dst = shadow + (int64_t)h * stride_h + slot * stride_slot;
  if (LPR == 16) {
    const uint4 r = reinterpret_cast<const uint4*>(src)[l];
    uint32_t* d32 = reinterpret_cast<uint32_t*>(dst) + 4 * l;
    __builtin_nontemporal_store(r.x, d32);
    __builtin_nontemporal_store(r.y, d32 + 1);
    __builtin_nontemporal_store(r.z, d32 + 2);
    __builtin_nontemporal_store(r.w, d32 + 3);
  } else {
    __builtin_nontemporal_store(reinterpret_cast<const uint32_t*>(src)[l], reinterpret_cast<uint32_t*>(dst) + l);
  }
}

inline bool aligned16(const void* x, int64_t stride_t, int64_t stride_h) {
  return ((uintptr_t)x & 15) == 0 && stride_t % 8 == 0 && stride_h % 8 == 0;
}

}  // namespace
}  // namespace jf

using namespace jf;

extern "C" int jf_host_buffer_device_pointer(const void* host_ptr, void** device_ptr) {
  JF_CHECK_ARG(host_ptr && device_ptr, "host_buffer_device_pointer: null pointer");
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, host_ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // an unknown pointer is an answer, not a sticky error
    set_error("host_buffer_device_pointer: %p is not known to the HIP runtime (pageable host memory?): %s", host_ptr,
              hipGetErrorString(e));
    return JF_ERR_ARG;
  }
  JF_CHECK_ARG(attr.type == hipMemoryTypeHost && attr.devicePointer != nullptr,
               "host_buffer_device_pointer: %p is not pinned host memory the GPU can address (memory type %d)",
               host_ptr, (int)attr.type);
  *device_ptr = attr.devicePointer;
  return JF_OK;
}

extern "C" int jf_shadow_write(const uint16_t* key, int64_t k_stride_t, int64_t k_stride_h, const uint16_t* value,
                               int64_t v_stride_t, int64_t v_stride_h, const int64_t* slots, int64_t T, int H_kv,
                               uint16_t* k_shadow, uint16_t* v_shadow, int64_t shadow_stride_h,
                               int64_t shadow_stride_slot, int64_t num_slots, void* stream) {
  JF_CHECK_ARG(T >= 0 && H_kv > 0 && H_kv <= 65535, "shadow_write: bad T=%lld H_kv=%d", (long long)T, H_kv);
  JF_CHECK_ARG(T <= (int64_t)4 * 0x7fffffff, "shadow_write: T=%lld exceeds the launch grid", (long long)T);
  if (T == 0) return JF_OK;
  JF_CHECK_ARG(key && value && slots && k_shadow && v_shadow, "shadow_write: null pointer");
  JF_CHECK_ARG(num_slots > 0 && shadow_stride_slot >= D && shadow_stride_h >= shadow_stride_slot,
               "shadow_write: bad shadow geometry (num_slots=%lld, strides %lld / %lld)", (long long)num_slots,
               (long long)shadow_stride_h, (long long)shadow_stride_slot);
  JF_CHECK_ARG((k_stride_t | k_stride_h | v_stride_t | v_stride_h) % 2 == 0 && (((uintptr_t)key | (uintptr_t)value) & 3) == 0,
               "shadow_write: token rows must be 4-byte aligned");
  JF_CHECK_ARG((((uintptr_t)k_shadow | (uintptr_t)v_shadow) & 15) == 0 && shadow_stride_h % 8 == 0 && shadow_stride_slot % 8 == 0,
               "shadow_write: shadow rows must be 16-byte aligned");
  MirrorSrc k{key, k_stride_t, k_stride_h}, v{value, v_stride_t, v_stride_h};
  hipStream_t st = (hipStream_t)stream;
  if (aligned16(key, k_stride_t, k_stride_h) && aligned16(value, v_stride_t, v_stride_h)) {
    dim3 grid((unsigned)((T + 15) / 16), (unsigned)H_kv, 2);
    hipLaunchKernelGGL(shadow_write_kernel<16>, grid, dim3(256), 0, st, k, v, k_shadow, v_shadow, shadow_stride_h,
                       shadow_stride_slot, slots, T, num_slots);
  } else {
    dim3 grid((unsigned)((T + 3) / 4), (unsigned)H_kv, 2);
    hipLaunchKernelGGL(shadow_write_kernel<64>, grid, dim3(256), 0, st, k, v, k_shadow, v_shadow, shadow_stride_h,
                       shadow_stride_slot, slots, T, num_slots);
  }
  JF_CHECK_LAUNCH();
  return JF_OK;
}

extern "C" int jf_shadow_append_count(int64_t* count, int reset) {
  JF_CHECK_ARG(count, "shadow_append_count: null output");
  unsigned long long v = 0;
  JF_CHECK_HIP(hipMemcpyFromSymbol(&v, HIP_SYMBOL(shadow_appends), sizeof(v)));
  *count = (int64_t)v;
  if (reset) {
    const unsigned long long zero = 0;
    JF_CHECK_HIP(hipMemcpyToSymbol(HIP_SYMBOL(shadow_appends), &zero, sizeof(zero)));
  }
  return JF_OK;
}
