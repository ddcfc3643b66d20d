// One-pass scan kernels of the fused decode step, asymmetric INT2 keys
// (see launch_full_scan_* in fused_scan_impl.h).
#include "fused_scan_impl.h"

int jf::launch_full_scan_d(int scheme, int G, int NG, const void* params, void* stream) {
  if (scheme == JF_SCHEME_A2V2)
    return NG == 2 ? launch_full_by_group<JF_SCHEME_A2V2, 2>(G, params, stream)
                   : launch_full_by_group<JF_SCHEME_A2V2, 1>(G, params, stream);
  if (scheme == JF_SCHEME_A2V3)
    return NG == 2 ? launch_full_by_group<JF_SCHEME_A2V3, 2>(G, params, stream)
                   : launch_full_by_group<JF_SCHEME_A2V3, 1>(G, params, stream);
  if (scheme == JF_SCHEME_A2V4)
    return NG == 2 ? launch_full_by_group<JF_SCHEME_A2V4, 2>(G, params, stream)
                   : launch_full_by_group<JF_SCHEME_A2V4, 1>(G, params, stream);
  JF_CHECK_ARG(false, "fused_scan: scheme %d is not in this family", scheme);
  return JF_ERR_ARG;
}
