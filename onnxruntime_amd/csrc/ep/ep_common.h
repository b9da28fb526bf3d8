// Shared declarations of the MI355X plugin execution provider.
//
// The library is loaded by ONNX Runtime through the plugin-EP C ABI
// (include/onnxruntime/core/session/onnxruntime_ep_c_api.h: CreateEpApiFactoriesFn :2732, OrtEpFactory :2753,
// OrtEp :2164, OrtKernelImpl :730) and claims com.microsoft::MatMulNBits nodes, which it runs through the C ABI of
// libmnb_mi355x.so (include/mnb_mi355x.h).  Only the plain C API is used: no C++ wrapper headers, no exceptions
// across the boundary.  The ONNX Runtime headers are taken from the include path given at build time; they are
// not part of this source tree.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstring>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "onnxruntime_c_api.h"

#include "mnb_mi355x.h"

namespace mi355x_ep {

constexpr const char* kEpName = "Mi355xExecutionProvider";
constexpr const char* kEpVendor = "AMD";
constexpr uint32_t kAmdVendorId = 0x1002;
constexpr const char* kEpVersion = "0.1.0";
constexpr const char* kMsDomain = "com.microsoft";
constexpr const char* kOnnxDomain = "";

struct Apis {
  const OrtApi* ort = nullptr;
  const OrtEpApi* ep = nullptr;
  const OrtLogger* logger = nullptr;
};

#define MI_RETURN_IF_ERROR(expr)  \
  do {                            \
    OrtStatus* mi_status_ = (expr); \
    if (mi_status_ != nullptr) return mi_status_; \
  } while (0)

#define MI_RETURN_IF_HIP(apis, expr)                                                               \
  do {                                                                                             \
    hipError_t mi_hip_ = (expr);                                                                   \
    if (mi_hip_ != hipSuccess) {                                                                   \
      std::string mi_msg_ = std::string("HIP failure: ") + hipGetErrorString(mi_hip_) + " in " #expr; \
      return (apis).ort->CreateStatus(ORT_EP_FAIL, mi_msg_.c_str());                                \
    }                                                                                              \
  } while (0)

// An MnbStatus (whose numeric values are OrtErrorCode values) becomes an OrtStatus with the library's message.
inline OrtStatus* StatusFromMnb(const Apis& apis, int rc) {
  if (rc == MNB_OK) return nullptr;
  return apis.ort->CreateStatus(static_cast<OrtErrorCode>(rc), MnbGetLastErrorMessage());
}

// ---- device runtime (ep_device_runtime.cc)
OrtAllocator* CreateDeviceAllocator(const Apis& apis, const OrtMemoryInfo* info, int device, bool pinned_host);
void DestroyDeviceAllocator(OrtAllocator* allocator);
OrtDataTransferImpl* CreateDataTransfer(const Apis& apis);
OrtSyncStreamImpl* CreateSyncStream(const Apis& apis, int device, OrtStatus** status);

// ---- kernels (ep_kernels.cc)
OrtStatus* CreateKernelRegistry(const Apis& apis, const char* ep_name, OrtKernelRegistry** out);

// ---- EP (ep.cc)
class Factory;
OrtEp* CreateEp(Factory& factory, const Apis& apis, int device);
void DestroyEp(OrtEp* ep);

// ---- factory (ep_factory.cc)
OrtEpFactory* CreateFactory(const Apis& apis);
void DestroyFactory(OrtEpFactory* factory);

class Factory : public OrtEpFactory {
 public:
  explicit Factory(const Apis& apis);
  ~Factory();

  // The registry is built once and shared by every OrtEp the factory creates.
  OrtStatus* GetKernelRegistry(const OrtKernelRegistry** out);

  const Apis apis;

  struct DeviceEntry {
    int ordinal = 0;
    OrtMemoryInfo* device_memory = nullptr;  // hipMalloc memory of this GPU
    OrtMemoryInfo* pinned_memory = nullptr;  // hipHostMalloc memory visible to this GPU
  };
  std::mutex mutex;
  std::vector<DeviceEntry> devices;
  OrtKernelRegistry* registry = nullptr;
};

}  // namespace mi355x_ep
