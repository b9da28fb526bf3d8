// Decode kernel (mnb_skinny_kernels.hip.h): the kernels for 4-bit weights without zero points.
#include "mnb_skinny_kernels.hip.h"

hipError_t mnb_skinny_launch_w4(const void* params, const void* plan, hipStream_t s) {
  return launch_zp<4, false>(*static_cast<const SkinnyParams*>(params), *static_cast<const SkinnyPlan*>(plan), s);
}

MNB_STAMPS_READER(MnbCalibrationReadStamps_w4)
