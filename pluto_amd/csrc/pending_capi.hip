// Entry points declared in pluto_hip.h whose kernels are not built yet.
#include "common.h"

extern "C" {

int pluto_hip_gdn_scan(void*, const pluto_hip_delta_params*, int, int, int,
                       const void*, const void*, const void*, const float*,
                       const float*, int, float, float*, void*, void*, size_t) {
  return PLUTO_HIP_EUNSUPPORTED;
}
size_t pluto_hip_gdn_scan_workspace_bytes(const pluto_hip_delta_params*, int, int, int) {
  return 0;
}
int pluto_hip_gdn_recurrence(void*, const pluto_hip_delta_params*, int, int,
                             const void*, const void*, const void*, const float*,
                             const float*, int, float, float*, void*, int) {
  return PLUTO_HIP_EUNSUPPORTED;
}
}  // extern "C"
