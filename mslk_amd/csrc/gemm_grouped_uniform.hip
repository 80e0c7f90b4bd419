// Grouped GEMM, uniform batch (f8f8bf16_rowwise_batched and the 3D-3D grouped_mm) with its bias variants, in a translation
// unit of its own (see gemm_grouped_device.h).  `p.unaligned` is already set by launch_device_groups().
#include "gemm_grouped_device.h"

namespace mslk_amd {

hipError_t launch_device_groups_uniform(const DeviceGroups& p, hipStream_t s) {
  if (p.bias_dtype == 1) return launch_device_layout<kGroupsUniform, 1>(p, s);
  if (p.bias_dtype == 2) return launch_device_layout<kGroupsUniform, 2>(p, s);
  return launch_device_layout<kGroupsUniform, 0>(p, s);
}

}  // namespace mslk_amd
