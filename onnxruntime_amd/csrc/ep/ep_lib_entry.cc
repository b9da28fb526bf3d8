// The two symbols ONNX Runtime looks up in a plugin execution-provider library
// (include/onnxruntime/core/session/onnxruntime_ep_c_api.h:2715-2747): CreateEpFactories and ReleaseEpFactory.
#include "ep_common.h"

#define MI_EP_EXPORT extern "C" __attribute__((visibility("default")))

MI_EP_EXPORT OrtStatus* CreateEpFactories(const char* /*registered_name*/, const OrtApiBase* ort_api_base,
                                          const OrtLogger* default_logger, OrtEpFactory** factories,
                                          size_t max_factories, size_t* num_factories) {
  if (ort_api_base == nullptr || factories == nullptr || num_factories == nullptr) return nullptr;
  *num_factories = 0;
  // The runtime answers NULL when it is older than the headers this library was compiled with.
  const OrtApi* ort = ort_api_base->GetApi(ORT_API_VERSION);
  if (ort == nullptr) return nullptr;  // no OrtApi, hence no way to build an OrtStatus: report zero factories
  mi355x_ep::Apis apis;
  apis.ort = ort;
  apis.ep = ort->GetEpApi();
  apis.logger = default_logger;
  if (apis.ep == nullptr) return ort->CreateStatus(ORT_FAIL, "OrtApi::GetEpApi returned NULL");
  if (max_factories < 1) {
    return ort->CreateStatus(ORT_INVALID_ARGUMENT, "Not enough space to return EP factory. Need at least one.");
  }
  OrtEpFactory* factory = mi355x_ep::CreateFactory(apis);
  if (factory == nullptr) return ort->CreateStatus(ORT_FAIL, "out of memory creating the MI355X EP factory");
  factories[0] = factory;
  *num_factories = 1;
  return nullptr;
}

MI_EP_EXPORT OrtStatus* ReleaseEpFactory(OrtEpFactory* factory) {
  mi355x_ep::DestroyFactory(factory);
  return nullptr;
}
