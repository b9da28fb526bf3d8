// Decode kernel (mnb_skinny_kernels.hip.h): the kernels for 8-bit weights.
#include "mnb_skinny_kernels.hip.h"

hipError_t mnb_skinny_launch_w8(const void* params, const void* plan, bool has_zp, hipStream_t s) {
  return has_zp ? launch_zp<8, true>(*static_cast<const SkinnyParams*>(params), *static_cast<const SkinnyPlan*>(plan), s)
                : launch_zp<8, false>(*static_cast<const SkinnyParams*>(params), *static_cast<const SkinnyPlan*>(plan), s);
}

MNB_STAMPS_READER(MnbCalibrationReadStamps_w8)
