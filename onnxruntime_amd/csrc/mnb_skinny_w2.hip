// Decode kernel (mnb_skinny_kernels.hip.h): the kernels for 2-bit weights streamed from the copy in their own width.
#include "mnb_skinny_kernels.hip.h"

hipError_t mnb_skinny_launch_w2(const void* params, const void* plan, hipStream_t s) {
  return launch_zp<2, true>(*static_cast<const SkinnyParams*>(params), *static_cast<const SkinnyPlan*>(plan), s);
}

MNB_STAMPS_READER(MnbCalibrationReadStamps_w2)
