// Grouped GEMM, device-side extents: offsets over N (3D-2D), offsets over K (2D-2D) and the padded-rows form, in a
// translation unit of their own (see gemm_grouped_device.h).  `p.unaligned` is already set by launch_device_groups().
#include "gemm_grouped_device.h"

namespace mslk_amd {

hipError_t launch_device_groups_layouts(const DeviceGroups& p, int layout, hipStream_t s) {
  switch (layout) {
    case kGroupsOffsetsN: return launch_device_layout<kGroupsOffsetsN, 0>(p, s);
    case kGroupsOffsetsK: return launch_device_layout<kGroupsOffsetsK, 0>(p, s);
    case kGroupsPrepadM: return launch_device_layout<kGroupsPrepadM, 0>(p, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace mslk_amd
