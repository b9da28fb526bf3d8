// Device plumbing the MI355X plugin EP hands to ONNX Runtime: allocators (OrtAllocator,
// include/onnxruntime/core/session/onnxruntime_c_api.h:356-424), the data transfer (OrtDataTransferImpl,
// onnxruntime_ep_c_api.h:100-157) and stream objects (OrtSyncStreamImpl / OrtSyncNotificationImpl,
// onnxruntime_ep_c_api.h:158-262).  Everything is plain HIP host API; streams use the default priority.
#include "ep_common.h"

namespace mi355x_ep {

namespace {

// ------------------------------------------------------------------------------------------- allocator
struct DeviceAllocator : OrtAllocator {
  const OrtMemoryInfo* info;
  int device;
  bool pinned;
};

void* ORT_API_CALL AllocImpl(OrtAllocator* this_, size_t size) {
  auto* self = static_cast<DeviceAllocator*>(this_);
  if (size == 0) return nullptr;
  int current = -1;
  if (hipGetDevice(&current) != hipSuccess) return nullptr;
  if (current != self->device && hipSetDevice(self->device) != hipSuccess) return nullptr;
  void* p = nullptr;
  hipError_t err = self->pinned ? hipHostMalloc(&p, size, hipHostMallocDefault) : hipMalloc(&p, size);
  if (current != self->device) (void)hipSetDevice(current);
  if (err != hipSuccess) {
    (void)hipGetLastError();  // leave no sticky error behind; the caller sees NULL
    return nullptr;
  }
  return p;
}

void ORT_API_CALL FreeImpl(OrtAllocator* this_, void* p) {
  auto* self = static_cast<DeviceAllocator*>(this_);
  if (p == nullptr) return;
  if (self->pinned)
    (void)hipHostFree(p);
  else
    (void)hipFree(p);
}

const OrtMemoryInfo* ORT_API_CALL InfoImpl(const OrtAllocator* this_) {
  return static_cast<const DeviceAllocator*>(this_)->info;
}

void* ORT_API_CALL ReserveImpl(OrtAllocator* this_, size_t size) { return AllocImpl(this_, size); }

// ------------------------------------------------------------------------------------------- data transfer
struct DataTransfer : OrtDataTransferImpl {
  Apis apis;
};

bool IsOurGpu(const Apis& a, const OrtMemoryDevice* d) {
  return a.ep->MemoryDevice_GetDeviceType(d) == OrtMemoryInfoDeviceType_GPU &&
         a.ep->MemoryDevice_GetVendorId(d) == kAmdVendorId;
}

bool IsCpu(const Apis& a, const OrtMemoryDevice* d) {
  return a.ep->MemoryDevice_GetDeviceType(d) == OrtMemoryInfoDeviceType_CPU;
}

void ORT_API_CALL ReleaseDataTransferImpl(OrtDataTransferImpl* this_ptr) noexcept {
  delete static_cast<DataTransfer*>(this_ptr);
}

bool ORT_API_CALL CanCopyImpl(const OrtDataTransferImpl* this_ptr, const OrtMemoryDevice* src,
                              const OrtMemoryDevice* dst) noexcept {
  const Apis& a = static_cast<const DataTransfer*>(this_ptr)->apis;
  const bool src_gpu = IsOurGpu(a, src), dst_gpu = IsOurGpu(a, dst);
  if (src_gpu && dst_gpu) return true;
  if (src_gpu && IsCpu(a, dst)) return true;
  if (dst_gpu && IsCpu(a, src)) return true;
  return false;
}

OrtStatus* ORT_API_CALL CopyTensorsImpl(OrtDataTransferImpl* this_ptr, const OrtValue** src_tensors,
                                        OrtValue** dst_tensors, OrtSyncStream** streams,
                                        size_t num_tensors) noexcept {
  const Apis& a = static_cast<DataTransfer*>(this_ptr)->apis;
  for (size_t i = 0; i < num_tensors; ++i) {
    const void* src = nullptr;
    void* dst = nullptr;
    size_t bytes = 0;
    MI_RETURN_IF_ERROR(a.ort->GetTensorData(src_tensors[i], &src));
    MI_RETURN_IF_ERROR(a.ort->GetTensorMutableData(dst_tensors[i], &dst));
    MI_RETURN_IF_ERROR(a.ort->GetTensorSizeInBytes(src_tensors[i], &bytes));
    if (bytes == 0 || src == dst) continue;
    const OrtMemoryDevice* sd = a.ep->Value_GetMemoryDevice(src_tensors[i]);
    const OrtMemoryDevice* dd = a.ep->Value_GetMemoryDevice(dst_tensors[i]);
    const bool src_gpu = IsOurGpu(a, sd), dst_gpu = IsOurGpu(a, dd);
    hipMemcpyKind kind;
    if (src_gpu && dst_gpu)
      kind = hipMemcpyDeviceToDevice;
    else if (src_gpu)
      kind = hipMemcpyDeviceToHost;
    else if (dst_gpu)
      kind = hipMemcpyHostToDevice;
    else
      return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "Mi355x data transfer: neither tensor is on an AMD GPU");
    OrtSyncStream* sync = streams != nullptr ? streams[i] : nullptr;
    if (sync != nullptr) {
      hipStream_t stream = static_cast<hipStream_t>(a.ort->SyncStream_GetHandle(sync));
      MI_RETURN_IF_HIP(a, hipMemcpyAsync(dst, src, bytes, kind, stream));
      // A copy into pageable host memory must have landed when the caller reads it right after the call.
      if (kind == hipMemcpyDeviceToHost) MI_RETURN_IF_HIP(a, hipStreamSynchronize(stream));
    } else {
      MI_RETURN_IF_HIP(a, hipMemcpy(dst, src, bytes, kind));
      if (kind == hipMemcpyDeviceToDevice) MI_RETURN_IF_HIP(a, hipStreamSynchronize(nullptr));
    }
  }
  return nullptr;
}

// ------------------------------------------------------------------------------------------- streams
struct SyncStream : OrtSyncStreamImpl {
  Apis apis;
  int device;
  hipStream_t stream;
};

struct Notification : OrtSyncNotificationImpl {
  Apis apis;
  hipStream_t producer;
  hipEvent_t event;
};

void ORT_API_CALL ReleaseNotificationImpl(OrtSyncNotificationImpl* this_ptr) noexcept {
  auto* n = static_cast<Notification*>(this_ptr);
  if (n->event != nullptr) (void)hipEventDestroy(n->event);
  delete n;
}

OrtStatus* ORT_API_CALL ActivateImpl(OrtSyncNotificationImpl* this_ptr) noexcept {
  auto* n = static_cast<Notification*>(this_ptr);
  MI_RETURN_IF_HIP(n->apis, hipEventRecord(n->event, n->producer));
  return nullptr;
}

OrtStatus* ORT_API_CALL WaitOnDeviceImpl(OrtSyncNotificationImpl* this_ptr, OrtSyncStream* consumer) noexcept {
  auto* n = static_cast<Notification*>(this_ptr);
  hipStream_t s = static_cast<hipStream_t>(n->apis.ort->SyncStream_GetHandle(consumer));
  MI_RETURN_IF_HIP(n->apis, hipStreamWaitEvent(s, n->event, 0));
  return nullptr;
}

OrtStatus* ORT_API_CALL WaitOnHostImpl(OrtSyncNotificationImpl* this_ptr) noexcept {
  auto* n = static_cast<Notification*>(this_ptr);
  MI_RETURN_IF_HIP(n->apis, hipEventSynchronize(n->event));
  return nullptr;
}

void ORT_API_CALL ReleaseStreamImpl(OrtSyncStreamImpl* this_ptr) noexcept {
  auto* s = static_cast<SyncStream*>(this_ptr);
  if (s->stream != nullptr) {
    (void)hipStreamSynchronize(s->stream);
    (void)hipStreamDestroy(s->stream);
  }
  delete s;
}

void* ORT_API_CALL GetHandleImpl(OrtSyncStreamImpl* this_ptr) noexcept {
  return static_cast<SyncStream*>(this_ptr)->stream;
}

OrtStatus* ORT_API_CALL CreateNotificationImpl(OrtSyncStreamImpl* this_ptr,
                                               OrtSyncNotificationImpl** notification) noexcept {
  auto* s = static_cast<SyncStream*>(this_ptr);
  *notification = nullptr;
  auto* n = new (std::nothrow) Notification{};
  if (n == nullptr) return s->apis.ort->CreateStatus(ORT_FAIL, "out of memory creating a stream notification");
  n->ort_version_supported = ORT_API_VERSION;
  n->Release = ReleaseNotificationImpl;
  n->Activate = ActivateImpl;
  n->WaitOnDevice = WaitOnDeviceImpl;
  n->WaitOnHost = WaitOnHostImpl;
  n->apis = s->apis;
  n->producer = s->stream;
  n->event = nullptr;
  hipError_t err = hipEventCreateWithFlags(&n->event, hipEventDisableTiming);
  if (err != hipSuccess) {
    delete n;
    return s->apis.ort->CreateStatus(ORT_EP_FAIL, hipGetErrorString(err));
  }
  *notification = n;
  return nullptr;
}

OrtStatus* ORT_API_CALL FlushImpl(OrtSyncStreamImpl* this_ptr) noexcept {
  auto* s = static_cast<SyncStream*>(this_ptr);
  MI_RETURN_IF_HIP(s->apis, hipStreamSynchronize(s->stream));
  return nullptr;
}

OrtStatus* ORT_API_CALL OnSessionRunEndImpl(OrtSyncStreamImpl*) noexcept { return nullptr; }

}  // namespace

OrtAllocator* CreateDeviceAllocator(const Apis&, const OrtMemoryInfo* info, int device, bool pinned_host) {
  auto* a = new (std::nothrow) DeviceAllocator{};
  if (a == nullptr) return nullptr;
  a->version = ORT_API_VERSION;
  a->Alloc = AllocImpl;
  a->Free = FreeImpl;
  a->Info = InfoImpl;
  a->Reserve = ReserveImpl;
  a->GetStats = nullptr;
  a->AllocOnStream = nullptr;
  a->Shrink = nullptr;
  a->info = info;
  a->device = device;
  a->pinned = pinned_host;
  return a;
}

void DestroyDeviceAllocator(OrtAllocator* allocator) { delete static_cast<DeviceAllocator*>(allocator); }

OrtDataTransferImpl* CreateDataTransfer(const Apis& apis) {
  auto* d = new (std::nothrow) DataTransfer{};
  if (d == nullptr) return nullptr;
  d->ort_version_supported = ORT_API_VERSION;
  d->Release = ReleaseDataTransferImpl;
  d->CanCopy = CanCopyImpl;
  d->CopyTensors = CopyTensorsImpl;
  d->apis = apis;
  return d;
}

OrtSyncStreamImpl* CreateSyncStream(const Apis& apis, int device, OrtStatus** status) {
  *status = nullptr;
  auto* s = new (std::nothrow) SyncStream{};
  if (s == nullptr) {
    *status = apis.ort->CreateStatus(ORT_FAIL, "out of memory creating a stream");
    return nullptr;
  }
  s->ort_version_supported = ORT_API_VERSION;
  s->Release = ReleaseStreamImpl;
  s->GetHandle = GetHandleImpl;
  s->CreateNotification = CreateNotificationImpl;
  s->Flush = FlushImpl;
  s->OnSessionRunEnd = OnSessionRunEndImpl;
  s->apis = apis;
  s->device = device;
  s->stream = nullptr;
  hipError_t err = hipSetDevice(device);
  if (err == hipSuccess) err = hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking);
  if (err != hipSuccess) {
    *status = apis.ort->CreateStatus(ORT_EP_FAIL, hipGetErrorString(err));
    delete s;
    return nullptr;
  }
  return s;
}

}  // namespace mi355x_ep
