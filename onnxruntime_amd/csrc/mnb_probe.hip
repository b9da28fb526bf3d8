// Machine ceilings measured with the plainest possible kernels, for reading the roofline fractions of the real ones:
//   * what a kernel that only reads N bytes per launch achieves (launch ramp and tail included), and
//   * what a loop of nothing but v_mfma_f32_32x32x16_f16 achieves with constant and with random fp16 operands
//     (matrix-core power draw, hence the sustained clock, depends on how many operand bits toggle).
// Diagnostics only: nothing on the operator's path calls them.
#include <hip/hip_runtime.h>

#include <vector>

#include "mnb_device.cuh"
#include "mnb_internal.h"

namespace {

template <int U>
__global__ void __launch_bounds__(256) mnb_probe_read_kernel(const uint4* __restrict__ p, float* out, size_t n_vec) {
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  uint4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t i = tid + u * stride;
    v[u] = i < n_vec ? p[i] : make_uint4(0, 0, 0, 0);
  }
  uint32_t s = 0;
#pragma unroll
  for (int u = 0; u < U; ++u) s += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  if (s == 0x12345678u) out[0] = 1.f;  // keeps the loads alive; practically never taken
}

template <int RANDOM>
__global__ void __launch_bounds__(512, 2) mnb_probe_mfma_kernel(float* out, int iters) {
  f16_t acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  h8_t a[4], b[2];
  uint32_t x = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 1u;
  for (int t = 0; t < 4; ++t)
    for (int i = 0; i < 8; ++i) {
      x = x * 1664525u + 1013904223u;
      a[t][i] = RANDOM ? (_Float16)((float)(x >> 8) * (1.0f / 8388608.0f) - 1.0f) : (_Float16)1.0f;  // U(-1, 1)
    }
  for (int t = 0; t < 2; ++t)
    for (int i = 0; i < 8; ++i) {
      x = x * 1664525u + 1013904223u;
      b[t][i] = RANDOM ? (_Float16)((float)((x >> 8) & 15) * 0.01f - 0.08f) : (_Float16)0.5f;  // 4-bit grid
    }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i * 2 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i * 2 + j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace

// `launches` back-to-back kernels (one HIP graph), each reading its own `bytes` of device memory once.
hipError_t mnb_probe_read(size_t bytes, int launches, double* gb_per_s) {
  *gb_per_s = 0.0;
  const size_t n_vec = bytes / 16;
  if (n_vec == 0 || launches < 1) return hipErrorInvalidValue;
  std::vector<uint4*> bufs((size_t)launches, nullptr);
  float* out = nullptr;
  hipStream_t s = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipGraph_t g = nullptr;
  hipGraphExec_t ge = nullptr;
  hipError_t err = hipSuccess;
  auto ok = [&](hipError_t e) {
    if (err == hipSuccess && e != hipSuccess) err = e;
    return err == hipSuccess;
  };
  constexpr int U = 8;
  const unsigned blocks = (unsigned)((n_vec + 256 * U - 1) / (256 * U));
  if (ok(hipMalloc(&out, 256))) {
    for (int i = 0; i < launches && err == hipSuccess; ++i)
      if (ok(hipMalloc(&bufs[i], n_vec * 16))) ok(hipMemset(bufs[i], i + 1, n_vec * 16));
  }
  if (ok(hipStreamCreateWithFlags(&s, hipStreamNonBlocking)) && ok(hipEventCreate(&e0)) && ok(hipEventCreate(&e1)) &&
      ok(hipDeviceSynchronize()) && ok(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal))) {
    for (int i = 0; i < launches; ++i) mnb_probe_read_kernel<U><<<blocks, 256, 0, s>>>(bufs[i], out, n_vec);
    ok(hipStreamEndCapture(s, &g));
    if (ok(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0))) {
      for (int w = 0; w < 3; ++w) ok(hipGraphLaunch(ge, s));
      ok(hipStreamSynchronize(s));
      const int reps = 20;
      ok(hipEventRecord(e0, s));
      for (int r = 0; r < reps; ++r) ok(hipGraphLaunch(ge, s));
      ok(hipEventRecord(e1, s));
      ok(hipStreamSynchronize(s));
      float ms = 0.f;
      if (ok(hipEventElapsedTime(&ms, e0, e1)) && ms > 0.f)
        *gb_per_s = (double)(n_vec * 16) * launches * reps / (ms * 1e-3) / 1e9;
    }
  }
  if (ge) (void)hipGraphExecDestroy(ge);
  if (g) (void)hipGraphDestroy(g);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (s) (void)hipStreamDestroy(s);
  for (uint4* b : bufs)
    if (b) (void)hipFree(b);
  if (out) (void)hipFree(out);
  return err;
}

hipError_t mnb_probe_mfma(int random_operands, double* tflops) {
  *tflops = 0.0;
  int dev = 0, cus = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (err != hipSuccess) return err;
  float* out = nullptr;
  err = hipMalloc(&out, (size_t)cus * 512 * sizeof(float));
  if (err != hipSuccess) return err;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  // From idle the matrix-core clock needs about 15 ms of load to settle: one untimed launch of 25 ms, then the timed one.
  const int iters = 100000;
  auto launch = [&](int n) {
    if (random_operands)
      mnb_probe_mfma_kernel<1><<<cus, 512, 0, nullptr>>>(out, n);
    else
      mnb_probe_mfma_kernel<0><<<cus, 512, 0, nullptr>>>(out, n);
  };
  if ((err = hipEventCreate(&e0)) == hipSuccess && (err = hipEventCreate(&e1)) == hipSuccess) {
    launch(iters);
    if ((err = hipDeviceSynchronize()) == hipSuccess) {
      (void)hipEventRecord(e0, nullptr);
      launch(iters);
      (void)hipEventRecord(e1, nullptr);
      err = hipDeviceSynchronize();
      float ms = 0.f;
      if (err == hipSuccess && (err = hipEventElapsedTime(&ms, e0, e1)) == hipSuccess && ms > 0.f)
        *tflops = (double)cus * 8 * iters * 8 * 32768.0 / (ms * 1e-3) / 1e12;
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(out);
  return err;
}
