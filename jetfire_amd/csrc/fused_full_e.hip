// One-pass scan kernels of the fused decode step, INT4 keys with the bf16 scoring model
// (see launch_full_scan_* in fused_scan_impl.h).
#include "fused_scan_impl.h"

int jf::launch_full_scan_e(int scheme, int G, int NG, const void* params, void* stream) {
  if (scheme == JF_SCHEME_B4V2)
    return NG == 2 ? launch_full_by_group<JF_SCHEME_B4V2, 2>(G, params, stream)
                   : launch_full_by_group<JF_SCHEME_B4V2, 1>(G, params, stream);
  if (scheme == JF_SCHEME_B4V3)
    return NG == 2 ? launch_full_by_group<JF_SCHEME_B4V3, 2>(G, params, stream)
                   : launch_full_by_group<JF_SCHEME_B4V3, 1>(G, params, stream);
  if (scheme == JF_SCHEME_B4V4)
    return NG == 2 ? launch_full_by_group<JF_SCHEME_B4V4, 2>(G, params, stream)
                   : launch_full_by_group<JF_SCHEME_B4V4, 1>(G, params, stream);
  JF_CHECK_ARG(false, "fused_scan: scheme %d is not in this family", scheme);
  return JF_ERR_ARG;
}
