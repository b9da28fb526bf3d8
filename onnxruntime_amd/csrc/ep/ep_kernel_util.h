// Helpers shared by the kernel implementations of the MI355X plugin EP (ep_kernels.cc, ep_fused_kernels.cc):
// tensor descriptions, device views of constant initializers, kernel-definition plumbing.
#pragma once
#include "ep_common.h"

namespace mi355x_ep {

// Shape and element type of a tensor value.
struct TensorDesc {
  std::vector<int64_t> dims;
  ONNXTensorElementDataType type = ONNX_TENSOR_ELEMENT_DATA_TYPE_UNDEFINED;
  int64_t count() const {
    int64_t c = 1;
    for (int64_t d : dims) c *= d;
    return c;
  }
};

inline OrtStatus* Describe(const Apis& a, const OrtValue* value, TensorDesc* out) {
  OrtTensorTypeAndShapeInfo* info = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetTensorTypeAndShape(value, &info));
  size_t rank = 0;
  OrtStatus* st = a.ort->GetDimensionsCount(info, &rank);
  if (st == nullptr) {
    out->dims.assign(rank, 0);
    if (rank > 0) st = a.ort->GetDimensions(info, out->dims.data(), rank);
  }
  if (st == nullptr) st = a.ort->GetTensorElementType(info, &out->type);
  a.ort->ReleaseTensorTypeAndShapeInfo(info);
  return st;
}

inline MnbTensorInfo ToMnb(const TensorDesc* d) {
  MnbTensorInfo t{};
  if (d == nullptr) return t;  // absent optional input
  static const int64_t kNoDims = 0;
  t.dims = d->dims.empty() ? &kNoDims : d->dims.data();
  t.rank = d->dims.size();
  t.dtype = static_cast<int>(d->type);
  return t;
}

inline bool OnHost(const Apis& a, const OrtValue* v) {
  return a.ep->MemoryDevice_GetDeviceType(a.ep->Value_GetMemoryDevice(v)) == OrtMemoryInfoDeviceType_CPU;
}

// A device view of a constant tensor: the tensor's own storage when it already lives on the GPU, otherwise a
// temporary device copy that is freed with the object.
class DeviceView {
 public:
  DeviceView() = default;
  DeviceView(const DeviceView&) = delete;
  DeviceView& operator=(const DeviceView&) = delete;
  ~DeviceView() {
    if (owned_ != nullptr) (void)hipFree(owned_);
  }
  OrtStatus* Init(const Apis& a, const OrtValue* v) {
    const void* p = nullptr;
    MI_RETURN_IF_ERROR(a.ort->GetTensorData(v, &p));
    if (!OnHost(a, v)) {
      ptr_ = p;
      return nullptr;
    }
    size_t bytes = 0;
    MI_RETURN_IF_ERROR(a.ort->GetTensorSizeInBytes(v, &bytes));
    if (bytes == 0) return nullptr;
    MI_RETURN_IF_HIP(a, hipMalloc(&owned_, bytes));
    MI_RETURN_IF_HIP(a, hipMemcpy(owned_, p, bytes, hipMemcpyHostToDevice));
    ptr_ = owned_;
    return nullptr;
  }
  const void* get() const { return ptr_; }

 private:
  const void* ptr_ = nullptr;
  void* owned_ = nullptr;
};

// Device scratch that lives for one Compute call.  It comes from the session's allocator for the device that holds
// `like` (the node's output), the way the reference's own GPU providers take theirs: KernelContext_GetScratchBuffer
// (onnxruntime_c_api.h:5269), handed back through the allocator of KernelContext_GetAllocator (:4929) once the call's
// kernels are enqueued -- the arena keeps the chunk with the compute stream.  A host that offers neither call (an
// ONNX Runtime older than the calls, or one whose allocator declines) is served from HIP's stream-ordered pool.
class CallScratch {
 public:
  CallScratch() = default;
  CallScratch(const CallScratch&) = delete;
  CallScratch& operator=(const CallScratch&) = delete;
  ~CallScratch() { (void)Release(); }

  // bytes == 0 leaves get() NULL.  `alignment`: what the consumer of the buffer demands of its address.
  OrtStatus* Acquire(const Apis& a, OrtKernelContext* ctx, const OrtValue* like, size_t bytes, hipStream_t stream,
                     size_t alignment = 256) {
    (void)Release();
    apis_ = &a;
    stream_ = stream;
    if (bytes == 0) return nullptr;
    if (ctx != nullptr && like != nullptr && a.ort->KernelContext_GetScratchBuffer != nullptr &&
        a.ort->KernelContext_GetAllocator != nullptr && a.ort->GetTensorMemoryInfo != nullptr &&
        a.ort->ReleaseAllocator != nullptr) {
      const OrtMemoryInfo* mem = nullptr;
      OrtStatus* st = a.ort->GetTensorMemoryInfo(like, &mem);
      if (st == nullptr && mem != nullptr) st = a.ort->KernelContext_GetAllocator(ctx, mem, &allocator_);
      void* p = nullptr;
      if (st == nullptr && allocator_ != nullptr) st = a.ort->KernelContext_GetScratchBuffer(ctx, mem, bytes, &p);
      if (st != nullptr) {  // the host declined: not an error of the node
        a.ort->ReleaseStatus(st);
        p = nullptr;
      }
      if (p != nullptr && reinterpret_cast<uintptr_t>(p) % alignment != 0) {
        allocator_->Free(allocator_, p);
        p = nullptr;
      }
      if (p != nullptr) {
        ptr_ = p;
        return nullptr;
      }
      if (allocator_ != nullptr) a.ort->ReleaseAllocator(allocator_);
      allocator_ = nullptr;
    }
    MI_RETURN_IF_HIP(a, hipMallocAsync(&ptr_, bytes, stream));
    pooled_ = true;
    return nullptr;
  }

  // Hands the buffer back; the work that uses it has been enqueued on the stream by then.
  hipError_t Release() {
    hipError_t e = hipSuccess;
    if (ptr_ != nullptr) {
      if (pooled_)
        e = hipFreeAsync(ptr_, stream_);
      else
        allocator_->Free(allocator_, ptr_);
    }
    if (allocator_ != nullptr) apis_->ort->ReleaseAllocator(allocator_);
    ptr_ = nullptr;
    allocator_ = nullptr;
    pooled_ = false;
    return e;
  }

  void* get() const { return ptr_; }
  bool from_session() const { return ptr_ != nullptr && !pooled_; }

 private:
  const Apis* apis_ = nullptr;
  OrtAllocator* allocator_ = nullptr;
  void* ptr_ = nullptr;
  hipStream_t stream_ = nullptr;
  bool pooled_ = false;
};

inline bool InputExists(const Apis& a, const OrtKernelInfo* info, size_t index, size_t count) {
  if (index >= count) return false;
  size_t size = 0;
  OrtStatus* st = a.ort->KernelInfo_GetInputName(info, index, nullptr, &size);
  if (st != nullptr) {
    a.ort->ReleaseStatus(st);
    return false;
  }
  return size > 1;  // an omitted optional input has the empty name
}

struct DefBuilder {
  const Apis& a;
  OrtKernelDefBuilder* b = nullptr;
  explicit DefBuilder(const Apis& apis) : a(apis) {}
  ~DefBuilder() {
    if (b != nullptr) a.ep->ReleaseKernelDefBuilder(b);
  }
};

inline OrtStatus* TypeList(const Apis& a, const std::vector<ONNXTensorElementDataType>& elems,
                    std::vector<const OrtDataType*>* out) {
  out->clear();
  for (auto e : elems) {
    const OrtDataType* t = nullptr;
    MI_RETURN_IF_ERROR(a.ep->GetTensorDataType(e, &t));
    out->push_back(t);
  }
  return nullptr;
}

// ---- profiling (ep_profiler.cc)
OrtStatus* CreateEpProfiler(const Apis& a, OrtEpProfilerImpl** out);

// Times what the enclosing scope enqueues on `stream` when the calling thread is inside an ONNX Runtime event that
// a profiler of this provider is following; does nothing otherwise.
class KernelTimer {
 public:
  KernelTimer(hipStream_t stream, const char* op, const char* kernel_name, int64_t M, int64_t N, int64_t K);
  ~KernelTimer();
  KernelTimer(const KernelTimer&) = delete;
  KernelTimer& operator=(const KernelTimer&) = delete;

 private:
  hipStream_t stream_;
  void* pending_ = nullptr;   // the launch record, until the stop event is in the stream
  void* profiler_ = nullptr;
};

// ---- compiled subgraphs (ep_compile.cc): MatMulNBits + Add(bias) as one node
OrtStatus* ReadIntAttr(const Apis& a, const OrtNode* node, const char* name, int64_t* value, bool* found);  // ep.cc
OrtStatus* CompileFusedNodes(const Apis& a, const OrtGraph** graphs, const OrtNode** fused_nodes, size_t count,
                             OrtNodeComputeInfo** node_compute_infos);
void ReleaseFusedNode(OrtNodeComputeInfo* info);

// ---- fused projections (ep_fused_kernels.cc): MatMulNBitsMlp and MatMulNBitsQkv for float and float16
OrtStatus* AddFusedProjectionKernels(const Apis& a, const Apis* state, const char* ep_name, OrtKernelRegistry* registry);

}  // namespace mi355x_ep
