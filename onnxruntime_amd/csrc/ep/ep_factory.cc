// OrtEpFactory of the MI355X plugin EP (include/onnxruntime/core/session/onnxruntime_ep_c_api.h:2753-3080).
//
// One OrtEpDevice is offered per AMD GPU that HIP can see.  ONNX Runtime's hardware enumeration does not expose
// HIP ordinals, so the n-th AMD GPU it reports is taken to be HIP device n, the same convention the reference's
// CUDA plugin factory uses for CUDA ordinals (onnxruntime/core/providers/cuda/plugin/cuda_ep_factory.cc:190-214).
#include "ep_common.h"

namespace mi355x_ep {

namespace {

Factory* Self(OrtEpFactory* p) { return static_cast<Factory*>(p); }
const Factory* Self(const OrtEpFactory* p) { return static_cast<const Factory*>(p); }

const char* ORT_API_CALL GetNameImpl(const OrtEpFactory*) noexcept { return kEpName; }
const char* ORT_API_CALL GetVendorImpl(const OrtEpFactory*) noexcept { return kEpVendor; }
uint32_t ORT_API_CALL GetVendorIdImpl(const OrtEpFactory*) noexcept { return kAmdVendorId; }
const char* ORT_API_CALL GetVersionImpl(const OrtEpFactory*) noexcept { return kEpVersion; }

struct HwEntry {
  const OrtHardwareDevice* hw;
  int ordinal;
};
// hardware device -> HIP ordinal, filled by GetSupportedDevices and read by CreateEp
std::mutex g_hw_mutex;
std::vector<HwEntry> g_hw_map;

OrtStatus* EnsureDeviceEntry(Factory& f, int ordinal, Factory::DeviceEntry** out) {
  for (auto& e : f.devices)
    if (e.ordinal == ordinal) {
      *out = &e;
      return nullptr;
    }
  Factory::DeviceEntry e;
  e.ordinal = ordinal;
  MI_RETURN_IF_ERROR(f.apis.ort->CreateMemoryInfo_V2("Mi355x", OrtMemoryInfoDeviceType_GPU, kAmdVendorId, ordinal,
                                                     OrtDeviceMemoryType_DEFAULT, /*alignment*/ 256,
                                                     OrtDeviceAllocator, &e.device_memory));
  OrtStatus* st = f.apis.ort->CreateMemoryInfo_V2("Mi355x_pinned", OrtMemoryInfoDeviceType_GPU, kAmdVendorId, ordinal,
                                                  OrtDeviceMemoryType_HOST_ACCESSIBLE, /*alignment*/ 256,
                                                  OrtDeviceAllocator, &e.pinned_memory);
  if (st != nullptr) {
    f.apis.ort->ReleaseMemoryInfo(e.device_memory);
    return st;
  }
  f.devices.push_back(e);
  *out = &f.devices.back();
  return nullptr;
}

OrtStatus* ORT_API_CALL GetSupportedDevicesImpl(OrtEpFactory* this_ptr, const OrtHardwareDevice* const* devices,
                                                size_t num_devices, OrtEpDevice** ep_devices, size_t max_ep_devices,
                                                size_t* num_ep_devices) noexcept {
  Factory& f = *Self(this_ptr);
  const Apis& a = f.apis;
  *num_ep_devices = 0;
  const int hip_devices = MnbGetDeviceCount();
  int next_ordinal = 0;
  std::lock_guard<std::mutex> lock(f.mutex);
  for (size_t i = 0; i < num_devices && *num_ep_devices < max_ep_devices; ++i) {
    const OrtHardwareDevice* hw = devices[i];
    if (a.ort->HardwareDevice_Type(hw) != OrtHardwareDeviceType_GPU) continue;
    const uint32_t vendor = a.ort->HardwareDevice_VendorId(hw);
    if (vendor != 0 && vendor != kAmdVendorId) continue;
    const int ordinal = next_ordinal++;
    if (ordinal >= hip_devices) continue;  // enumerated by the OS but hidden from HIP

    Factory::DeviceEntry* entry = nullptr;
    MI_RETURN_IF_ERROR(EnsureDeviceEntry(f, ordinal, &entry));
    OrtEpDevice* ep_device = nullptr;
    MI_RETURN_IF_ERROR(a.ep->CreateEpDevice(this_ptr, hw, nullptr, nullptr, &ep_device));
    OrtStatus* st = a.ep->EpDevice_AddAllocatorInfo(ep_device, entry->device_memory);
    if (st == nullptr) st = a.ep->EpDevice_AddAllocatorInfo(ep_device, entry->pinned_memory);
    if (st != nullptr) {
      a.ep->ReleaseEpDevice(ep_device);
      return st;
    }
    {
      std::lock_guard<std::mutex> hw_lock(g_hw_mutex);
      bool known = false;
      for (auto& h : g_hw_map)
        if (h.hw == hw) {
          h.ordinal = ordinal;
          known = true;
        }
      if (!known) g_hw_map.push_back({hw, ordinal});
    }
    ep_devices[(*num_ep_devices)++] = ep_device;
  }
  return nullptr;
}

OrtStatus* ORT_API_CALL CreateEpImpl(OrtEpFactory* this_ptr, const OrtHardwareDevice* const* devices,
                                     const OrtKeyValuePairs* const* /*ep_metadata_pairs*/, size_t num_devices,
                                     const OrtSessionOptions* /*session_options*/, const OrtLogger* /*logger*/,
                                     OrtEp** ep) noexcept {
  Factory& f = *Self(this_ptr);
  *ep = nullptr;
  if (num_devices != 1) {
    return f.apis.ort->CreateStatus(ORT_INVALID_ARGUMENT,
                                    "Mi355xExecutionProvider runs a session on exactly one GPU; "
                                    "select a single OrtEpDevice.");
  }
  int ordinal = -1;
  {
    std::lock_guard<std::mutex> hw_lock(g_hw_mutex);
    for (auto& h : g_hw_map)
      if (h.hw == devices[0]) ordinal = h.ordinal;
  }
  if (ordinal < 0) {
    return f.apis.ort->CreateStatus(ORT_INVALID_ARGUMENT,
                                    "The OrtHardwareDevice was not offered by Mi355xExecutionProvider.");
  }
  OrtEp* created = CreateEp(f, f.apis, ordinal);
  if (created == nullptr) return f.apis.ort->CreateStatus(ORT_FAIL, "out of memory creating Mi355xExecutionProvider");
  *ep = created;
  return nullptr;
}

void ORT_API_CALL ReleaseEpImpl(OrtEpFactory*, OrtEp* ep) noexcept { DestroyEp(ep); }

OrtStatus* ORT_API_CALL CreateAllocatorImpl(OrtEpFactory* this_ptr, const OrtMemoryInfo* memory_info,
                                            const OrtKeyValuePairs* /*allocator_options*/,
                                            OrtAllocator** allocator) noexcept {
  Factory& f = *Self(this_ptr);
  *allocator = nullptr;
  const OrtMemoryDevice* md = f.apis.ep->MemoryInfo_GetMemoryDevice(memory_info);
  const int ordinal = static_cast<int>(f.apis.ep->MemoryDevice_GetDeviceId(md));
  const bool pinned = f.apis.ep->MemoryDevice_GetMemoryType(md) == OrtDeviceMemoryType_HOST_ACCESSIBLE;
  std::lock_guard<std::mutex> lock(f.mutex);
  for (auto& e : f.devices) {
    if (e.ordinal != ordinal) continue;
    OrtAllocator* created = CreateDeviceAllocator(f.apis, pinned ? e.pinned_memory : e.device_memory, ordinal, pinned);
    if (created == nullptr) return f.apis.ort->CreateStatus(ORT_FAIL, "out of memory creating an allocator");
    *allocator = created;
    return nullptr;
  }
  return f.apis.ort->CreateStatus(ORT_INVALID_ARGUMENT,
                                  "CreateAllocator: the OrtMemoryInfo does not belong to Mi355xExecutionProvider.");
}

void ORT_API_CALL ReleaseAllocatorImpl(OrtEpFactory*, OrtAllocator* allocator) noexcept {
  DestroyDeviceAllocator(allocator);
}

OrtStatus* ORT_API_CALL CreateDataTransferImpl(OrtEpFactory* this_ptr, OrtDataTransferImpl** data_transfer) noexcept {
  Factory& f = *Self(this_ptr);
  *data_transfer = CreateDataTransfer(f.apis);
  if (*data_transfer == nullptr) return f.apis.ort->CreateStatus(ORT_FAIL, "out of memory creating the data transfer");
  return nullptr;
}

bool ORT_API_CALL IsStreamAwareImpl(const OrtEpFactory*) noexcept { return true; }

OrtStatus* ORT_API_CALL CreateSyncStreamForDeviceImpl(OrtEpFactory* this_ptr, const OrtMemoryDevice* memory_device,
                                                      const OrtKeyValuePairs* /*stream_options*/,
                                                      OrtSyncStreamImpl** stream) noexcept {
  Factory& f = *Self(this_ptr);
  OrtStatus* st = nullptr;
  *stream = CreateSyncStream(f.apis, static_cast<int>(f.apis.ep->MemoryDevice_GetDeviceId(memory_device)), &st);
  return st;
}

}  // namespace

Factory::Factory(const Apis& apis_in) : OrtEpFactory{}, apis(apis_in) {
  ort_version_supported = ORT_API_VERSION;
  GetName = GetNameImpl;
  GetVendor = GetVendorImpl;
  GetVendorId = GetVendorIdImpl;
  GetVersion = GetVersionImpl;
  GetSupportedDevices = GetSupportedDevicesImpl;
  CreateEp = CreateEpImpl;
  ReleaseEp = ReleaseEpImpl;
  CreateAllocator = CreateAllocatorImpl;
  ReleaseAllocator = ReleaseAllocatorImpl;
  CreateDataTransfer = CreateDataTransferImpl;
  IsStreamAware = IsStreamAwareImpl;
  CreateSyncStreamForDevice = CreateSyncStreamForDeviceImpl;
  // Members left NULL are optional: no compiled-model compatibility data, no custom-op domains, no external
  // resource import.
}

Factory::~Factory() {
  if (registry != nullptr) apis.ep->ReleaseKernelRegistry(registry);
  for (auto& e : devices) {
    if (e.device_memory) apis.ort->ReleaseMemoryInfo(e.device_memory);
    if (e.pinned_memory) apis.ort->ReleaseMemoryInfo(e.pinned_memory);
  }
}

OrtStatus* Factory::GetKernelRegistry(const OrtKernelRegistry** out) {
  std::lock_guard<std::mutex> lock(mutex);
  if (registry == nullptr) MI_RETURN_IF_ERROR(CreateKernelRegistry(apis, kEpName, &registry));
  *out = registry;
  return nullptr;
}

OrtEpFactory* CreateFactory(const Apis& apis) { return new (std::nothrow) Factory(apis); }
void DestroyFactory(OrtEpFactory* factory) { delete static_cast<Factory*>(factory); }

}  // namespace mi355x_ep
