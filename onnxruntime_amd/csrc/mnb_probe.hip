// Machine ceilings measured with the plainest possible kernels, for reading the roofline fractions of the real ones:
//   * what a kernel that only reads N bytes per launch achieves (launch ramp and tail included), swept over workgroup
//     size, 16-byte loads in flight per thread and batches per thread, and
//   * what a loop of nothing but v_mfma_f32_32x32x16_f16 achieves with constant and with random fp16 operands
//     (matrix-core power draw, hence the sustained clock, depends on how many operand bits toggle).
// Built as a library of its own (libmnb_probe.so) that only the benchmark loads: diagnostics, not part of the
// operator's C ABI, and nothing on the operator's path calls them.
#include "mnb_probe.h"

#include <hip/hip_runtime.h>

#include <vector>

#include "mnb_buffer.hip.h"
#include "mnb_device.hip.h"

namespace {

// Each thread issues U independent 16-byte loads (a wavefront reads 1 KiB contiguous per load), `batches` times.
template <int U>
__global__ void mnb_probe_read_kernel(const uint4* __restrict__ p, float* out, size_t n_vec, int batches) {
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  uint32_t s = 0;
  for (int b = 0; b < batches; ++b) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = tid + ((size_t)b * U + u) * stride;
      v[u] = i < n_vec ? p[i] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) s += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (s == 0x12345678u) out[0] = 1.f;  // keeps the loads alive; practically never taken
}

// Values of one operand class (MnbProbeMfmaRateOperands): what the matrix cores see decides their switching activity,
// and with it the clock the power limit allows.
__device__ __forceinline__ _Float16 mnb_probe_operand(int kind, uint32_t x, int lane) {
  const float u = (float)(x >> 8) * (1.0f / 8388608.0f) - 1.0f;  // U(-1, 1)
  const int q = (x >> 8) & 15;
  switch (kind) {
    case 1: return (_Float16)u;
    case 2: return (_Float16)0.0f;
    case 3: {  // sum of three uniforms: bell-shaped, variance 1
      uint32_t y = x * 747796405u + 2891336453u;
      float v = u + ((float)(y >> 8) * (1.0f / 8388608.0f) - 1.0f);
      y = y * 747796405u + 2891336453u;
      return (_Float16)(v + ((float)(y >> 8) * (1.0f / 8388608.0f) - 1.0f));
    }
    case 4: {  // a dequantised 4-bit weight: (q - 8) times the scale of the lane's column
      const float s = 0.005f + 0.01f * (float)(((uint32_t)lane * 2654435761u >> 20) & 1023) * (1.0f / 1024.0f);
      return (_Float16)((float)(q - 8) * s);
    }
    case 5: return (_Float16)(float)(q - 8);     // the same weight before its scale: four significant bits
    case 6: return (_Float16)(float)(1024 + q);  // the raw "magic" half the decode kernel feeds
    case 7: return (_Float16)((float)q * 0.01f - 0.08f);  // 4-bit grid under one scale
    default: return (_Float16)1.0f;
  }
}

__global__ void __launch_bounds__(512, 2) mnb_probe_mfma_kernel(float* out, int iters, int kind_a, int kind_b) {
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
      a[t][i] = mnb_probe_operand(kind_a, x, threadIdx.x & 63);
    }
  for (int t = 0; t < 2; ++t)
    for (int i = 0; i < 8; ++i) {
      x = x * 1664525u + 1013904223u;
      b[t][i] = mnb_probe_operand(kind_b, x, threadIdx.x & 63);
    }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i * 2 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i * 2 + j], 0, 0, 0);
    if ((it & 63) == 63) {  // keeps the sums finite whatever the operands are
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] *= 0.0009765625f;
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// A loop of "slots": one v_mfma_f32_32x32x16_f16 (MFMA) followed by V packed-fp16 fused multiply-adds on registers
// the matrix instruction does not touch, every instruction independent of its neighbours.  Timed with and without
// either kind, it shows whether a SIMD overlaps the two or issues them one after the other.
template <int V, bool MFMA, int LDS2>
__global__ void __launch_bounds__(512, 2) mnb_probe_issue_kernel(float* out, int iters) {
  __shared__ __align__(16) unsigned char tile[32768];
  for (int i = threadIdx.x; i < 32768 / 16; i += blockDim.x)
    reinterpret_cast<uint4*>(tile)[i] = make_uint4(0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u);  // ones
  __syncthreads();
  const int lane = threadIdx.x & 63;
  h8_t fa[8];
  f16_t acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  h8_t a, b;
  for (int i = 0; i < 8; ++i) a[i] = (_Float16)1.0f, b[i] = (_Float16)0.5f;
#pragma unroll
  for (int i = 0; i < 8; ++i) fa[i] = a;
  typedef _Float16 h2v __attribute__((ext_vector_type(2)));
  h2v h[8];
  for (int i = 0; i < 8; ++i) h[i] = h2v{(_Float16)(threadIdx.x & 7), (_Float16)i};
  const h2v m = h2v{(_Float16)0.5f, (_Float16)0.25f}, c = h2v{(_Float16)1.0f, (_Float16)2.0f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // the operand of this slot was read from LDS eight slots ago, into a register set of its own (16 bytes per
      // lane, a different kilobyte each time): the reads have a whole iteration to land
      if constexpr (MFMA) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(LDS2 ? fa[i] : a, b, acc[i], 0, 0, 0);
      if constexpr (LDS2 != 0)
        if (LDS2 == 2 || (i & 1) == 0)
          fa[i] = *reinterpret_cast<const h8_t*>(tile + ((it * 8 + i) & 31) * 1024 + lane * 16);
#pragma unroll
      for (int v = 0; v < V; ++v) h[(i * V + v) & 7] = h[(i * V + v) & 7] * m + c;
      if constexpr (MFMA) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (LDS2 == 2 || (LDS2 == 1 && (i & 1) == 0)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if constexpr (V > 0) __builtin_amdgcn_sched_group_barrier(0x002, V, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    s += (float)h[i].x + (float)h[i].y;
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  }
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// The streaming kernel's instruction mix in isolation.  A step is what that kernel does per packed word and column
// tile at 64 rows: 13 vector instructions turn a 32-bit word of eight 4-bit weights into the B operand (one shift,
// four and-or, four packed adds, four packed multiplies), and four v_mfma_f32_16x16x32_f16 use it.
// MODE 0: the matrix instructions alone; 1: the vector instructions alone; 2: operand made right in front of the
// matrix instructions that read it; 3: the operand of the next step is made between the matrix instructions of this
// one (order stated through scheduling groups).
template <int MODE>
__global__ void __launch_bounds__(512, 2) mnb_probe_dequant16_kernel(float* out, const uint32_t* words, int iters) {
  typedef float f4v __attribute__((ext_vector_type(4)));
  typedef _Float16 h2v __attribute__((ext_vector_type(2)));
  f4v acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = f4v{0.f, 0.f, 0.f, 0.f};
  h8_t a[4];
  for (int t = 0; t < 4; ++t)
    for (int i = 0; i < 8; ++i) a[t][i] = (_Float16)1.0f;
  uint32_t w = words[threadIdx.x & 63];  // (zero: keeps the arithmetic finite, and unknown to the compiler)
  uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
  asm("s_mov_b32 %0, 0x000F000F" : "=s"(mask_lo));
  asm("s_mov_b32 %0, 0x00F000F0" : "=s"(mask_hi));
  asm("v_mov_b32 %0, 0x64006400" : "=v"(magic_lo));
  asm("v_mov_b32 %0, 0x54005400" : "=v"(magic_hi));
  const h2v z_lo = h2v{(_Float16)-1032.0f, (_Float16)-1032.0f}, z_hi = h2v{(_Float16)-72.0f, (_Float16)-72.0f};
  const h2v s2 = h2v{(_Float16)0.01f, (_Float16)0.01f};
  auto as_h2 = [](uint32_t x) { return __builtin_bit_cast(h2v, x); };
  auto as_u32 = [](h2v x) { return __builtin_bit_cast(uint32_t, x); };
  auto make = [&](uint32_t word) {
    const uint32_t w8 = word >> 8;
    u4_t r;
    r[0] = as_u32((as_h2((word & mask_lo) | magic_lo) + z_lo) * s2);
    r[1] = as_u32((as_h2((word & mask_hi) | magic_hi) + z_hi) * s2);
    r[2] = as_u32((as_h2((w8 & mask_lo) | magic_lo) + z_lo) * s2);
    r[3] = as_u32((as_h2((w8 & mask_hi) | magic_hi) + z_hi) * s2);
    return __builtin_bit_cast(h8_t, r);
  };
  h8_t b = make(w);
  uint32_t sink = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      w = w * 5u + 0x11111111u * (uint32_t)st;  // (one more vector instruction; the word changes from step to step)
      if constexpr (MODE == 1) {
        const h8_t nb = make(w);
        sink ^= __builtin_bit_cast(u4_t, nb)[0] ^ __builtin_bit_cast(u4_t, nb)[3];
      } else if constexpr (MODE == 0) {
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
          acc[st * 4 + mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[mt], b, acc[st * 4 + mt], 0, 0, 0);
      } else if constexpr (MODE == 2) {
        b = make(w);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
          acc[st * 4 + mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[mt], b, acc[st * 4 + mt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      } else {
        const h8_t nb = make(w);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
          acc[st * 4 + mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[mt], b, acc[st * 4 + mt], 0, 0, 0);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        }
        b = nb;
      }
    }
  }
  float s = (float)sink;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s + (float)b[0];
}

// One wavefront that watches two counters for a while: the shader clock's cycle counter and the constant 100 MHz
// counter.  Their ratio is the clock the chip runs at while other kernels are busy on it.
__global__ void __launch_bounds__(64) mnb_probe_clock_kernel(unsigned long long* out, unsigned long long ticks) {
  if (threadIdx.x != 0) return;
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_amdgcn_s_memtime();
  unsigned long long r1 = r0;
  for (int spins = 0; spins < (1 << 22) && r1 - r0 < ticks; ++spins) {  // bounded whatever the counters do
    __builtin_amdgcn_s_sleep(64);
    r1 = __builtin_amdgcn_s_memrealtime();
  }
  const unsigned long long c1 = __builtin_amdgcn_s_memtime();
  r1 = __builtin_amdgcn_s_memrealtime();
  out[0] = c1 - c0;
  out[1] = r1 - r0;
}

// Buffers of the read probe, kept between calls so that a sweep allocates once.
std::vector<uint4*> g_bufs;
size_t g_buf_vecs = 0;
float* g_out = nullptr;

void release_buffers() {
  for (uint4* b : g_bufs)
    if (b) (void)hipFree(b);
  g_bufs.clear();
  g_buf_vecs = 0;
  if (g_out) (void)hipFree(g_out);
  g_out = nullptr;
}

hipError_t ensure_buffers(size_t n_vec, int launches) {
  if (g_buf_vecs == n_vec && (int)g_bufs.size() == launches && g_out) return hipSuccess;
  release_buffers();
  hipError_t e = hipMalloc(&g_out, 256);
  if (e != hipSuccess) return e;
  g_bufs.assign((size_t)launches, nullptr);
  for (int i = 0; i < launches; ++i) {
    if ((e = hipMalloc(&g_bufs[i], n_vec * 16)) != hipSuccess) return e;
    if ((e = hipMemset(g_bufs[i], i + 1, n_vec * 16)) != hipSuccess) return e;
  }
  g_buf_vecs = n_vec;
  return hipSuccess;
}

template <int U>
void launch_read(unsigned blocks, int threads, hipStream_t s, const uint4* p, size_t n_vec, int batches) {
  mnb_probe_read_kernel<U><<<blocks, threads, 0, s>>>(p, g_out, n_vec, batches);
}

// `launches` back-to-back kernels (one HIP graph), each reading its own `bytes` of device memory once.
// same_buffer: every launch reads the first buffer again (30 MB stay in the 256 MB Infinity Cache between launches).
hipError_t probe_read(size_t bytes, int launches, int threads, int loads_in_flight, int batches, bool same_buffer,
                      double* gb_per_s) {
  *gb_per_s = 0.0;
  const size_t n_vec = bytes / 16;
  hipStream_t s = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipGraph_t g = nullptr;
  hipGraphExec_t ge = nullptr;
  hipError_t err = hipSuccess;
  auto ok = [&](hipError_t e) {
    if (err == hipSuccess && e != hipSuccess) err = e;
    return err == hipSuccess;
  };
  const size_t per_block = (size_t)threads * loads_in_flight * batches;
  const unsigned blocks = (unsigned)((n_vec + per_block - 1) / per_block);
  ok(ensure_buffers(n_vec, same_buffer ? 1 : launches));
  if (ok(err) && ok(hipStreamCreateWithFlags(&s, hipStreamNonBlocking)) && ok(hipEventCreate(&e0)) &&
      ok(hipEventCreate(&e1)) && ok(hipDeviceSynchronize()) &&
      ok(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal))) {
    for (int i = 0; i < launches; ++i) {
      switch (loads_in_flight) {
        case 2: launch_read<2>(blocks, threads, s, g_bufs[same_buffer ? 0 : i], n_vec, batches); break;
        case 4: launch_read<4>(blocks, threads, s, g_bufs[same_buffer ? 0 : i], n_vec, batches); break;
        case 8: launch_read<8>(blocks, threads, s, g_bufs[same_buffer ? 0 : i], n_vec, batches); break;
        case 16: launch_read<16>(blocks, threads, s, g_bufs[same_buffer ? 0 : i], n_vec, batches); break;
        default: launch_read<32>(blocks, threads, s, g_bufs[same_buffer ? 0 : i], n_vec, batches); break;
      }
    }
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
  return err;
}

hipError_t probe_mfma(int kind_a, int kind_b, double* tflops) {
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
  auto launch = [&](int n) { mnb_probe_mfma_kernel<<<cus, 512, 0, nullptr>>>(out, n, kind_a, kind_b); };
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

template <int V>
void launch_issue(bool mfma, int lds2, int cus, int threads, float* out, int n) {
  if (!mfma)
    mnb_probe_issue_kernel<V, false, 0><<<cus, threads, 0, nullptr>>>(out, n);
  else if (lds2 == 2)
    mnb_probe_issue_kernel<V, true, 2><<<cus, threads, 0, nullptr>>>(out, n);
  else if (lds2 == 1)
    mnb_probe_issue_kernel<V, true, 1><<<cus, threads, 0, nullptr>>>(out, n);
  else
    mnb_probe_issue_kernel<V, true, 0><<<cus, threads, 0, nullptr>>>(out, n);
}

hipError_t probe_issue(int valu_per_mfma, int with_mfma, int waves_per_simd, int lds2, double* ns_per_slot) {
  *ns_per_slot = 0.0;
  int dev = 0, cus = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (err != hipSuccess) return err;
  float* out = nullptr;
  err = hipMalloc(&out, (size_t)cus * 512 * sizeof(float));
  if (err != hipSuccess) return err;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  const int iters = 20000, threads = 256 * waves_per_simd;
  auto launch = [&](int n) {
    switch (valu_per_mfma) {
      case 0: launch_issue<0>(with_mfma, lds2, cus, threads, out, n); break;
      case 1: launch_issue<1>(with_mfma, lds2, cus, threads, out, n); break;
      case 2: launch_issue<2>(with_mfma, lds2, cus, threads, out, n); break;
      case 4: launch_issue<4>(with_mfma, lds2, cus, threads, out, n); break;
      default: launch_issue<8>(with_mfma, lds2, cus, threads, out, n); break;
    }
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
        *ns_per_slot = (double)ms * 1e6 / ((double)iters * 8);
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(out);
  return err;
}

hipError_t probe_dequant16(int mode, int waves_per_simd, double* ns_per_step) {
  *ns_per_step = 0.0;
  int dev = 0, cus = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (err != hipSuccess) return err;
  float* out = nullptr;
  uint32_t* words = nullptr;
  if ((err = hipMalloc(&out, (size_t)cus * 512 * sizeof(float))) != hipSuccess) return err;
  if ((err = hipMalloc(&words, 64 * sizeof(uint32_t))) != hipSuccess || (err = hipMemset(words, 0, 256)) != hipSuccess) {
    (void)hipFree(out);
    if (words) (void)hipFree(words);
    return err;
  }
  hipEvent_t e0 = nullptr, e1 = nullptr;
  const int iters = 40000, threads = 256 * waves_per_simd;
  auto launch = [&](int n) {
    switch (mode) {
      case 0: mnb_probe_dequant16_kernel<0><<<cus, threads, 0, nullptr>>>(out, words, n); break;
      case 1: mnb_probe_dequant16_kernel<1><<<cus, threads, 0, nullptr>>>(out, words, n); break;
      case 2: mnb_probe_dequant16_kernel<2><<<cus, threads, 0, nullptr>>>(out, words, n); break;
      default: mnb_probe_dequant16_kernel<3><<<cus, threads, 0, nullptr>>>(out, words, n); break;
    }
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
        *ns_per_step = (double)ms * 1e6 / ((double)iters * 4);
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(out);
  (void)hipFree(words);
  return err;
}

// state of a running clock sample
hipStream_t g_clock_stream = nullptr;
unsigned long long* g_clock_out = nullptr;

hipError_t clock_start(double sample_ms) {
  hipError_t err = hipSuccess;
  if (!g_clock_stream && (err = hipStreamCreateWithFlags(&g_clock_stream, hipStreamNonBlocking)) != hipSuccess) return err;
  if (!g_clock_out && (err = hipMalloc(&g_clock_out, 2 * sizeof(unsigned long long))) != hipSuccess) return err;
  mnb_probe_clock_kernel<<<1, 64, 0, g_clock_stream>>>(g_clock_out, (unsigned long long)(sample_ms * 1e5));
  return hipGetLastError();
}

hipError_t clock_finish(double* ghz, double* sampled_ms) {
  *ghz = 0.0;
  *sampled_ms = 0.0;
  if (!g_clock_stream || !g_clock_out) return hipErrorNotReady;
  hipError_t err = hipStreamSynchronize(g_clock_stream);
  if (err != hipSuccess) return err;
  unsigned long long v[2] = {0, 0};
  if ((err = hipMemcpy(v, g_clock_out, sizeof(v), hipMemcpyDeviceToHost)) != hipSuccess) return err;
  if (v[1] > 0) {
    *ghz = (double)v[0] / (double)v[1] * 0.1;  // cycles per 10 ns tick
    *sampled_ms = (double)v[1] * 1e-5;
  }
  return hipSuccess;
}

}  // namespace

extern "C" {

int MnbProbeReadBandwidth(size_t bytes_per_launch, int launches, int threads, int loads_in_flight, int batches,
                          double* gb_per_s) {
  const bool u_ok = loads_in_flight == 2 || loads_in_flight == 4 || loads_in_flight == 8 || loads_in_flight == 16 ||
                    loads_in_flight == 32;
  if (!gb_per_s || bytes_per_launch < 16 || launches < 1 || (double)bytes_per_launch * launches > 8e9 || !u_ok ||
      threads < 64 || threads > 1024 || threads % 64 != 0 || batches < 1 || batches > 64)
    return 2;
  return probe_read(bytes_per_launch, launches, threads, loads_in_flight, batches, false, gb_per_s) == hipSuccess ? 0 : 1;
}

int MnbProbeReadBandwidthResident(size_t bytes_per_launch, int launches, int threads, int loads_in_flight, int batches,
                                  double* gb_per_s) {
  const bool u_ok = loads_in_flight == 2 || loads_in_flight == 4 || loads_in_flight == 8 || loads_in_flight == 16 ||
                    loads_in_flight == 32;
  if (!gb_per_s || bytes_per_launch < 16 || launches < 1 || bytes_per_launch > ((size_t)1 << 31) || !u_ok ||
      threads < 64 || threads > 1024 || threads % 64 != 0 || batches < 1 || batches > 64)
    return 2;
  return probe_read(bytes_per_launch, launches, threads, loads_in_flight, batches, true, gb_per_s) == hipSuccess ? 0 : 1;
}

void MnbProbeRelease(void) { release_buffers(); }

int MnbProbeMfmaRate(int random_operands, double* tflops) {
  if (!tflops) return 2;
  // (random: uniform activations against a 4-bit grid under one scale, as this probe has always run)
  return probe_mfma(random_operands ? 1 : 0, random_operands ? 7 : 0, tflops) == hipSuccess ? 0 : 1;
}

int MnbProbeMfmaRateOperands(int a_class, int b_class, double* tflops) {
  if (!tflops || a_class < 0 || a_class > 7 || b_class < 0 || b_class > 7) return 2;
  return probe_mfma(a_class, b_class, tflops) == hipSuccess ? 0 : 1;
}

int MnbProbeIssueOverlap(int valu_per_mfma, int with_mfma, int waves_per_simd, int lds_reads_per_two_mfma,
                         double* ns_per_slot) {
  const bool v_ok = valu_per_mfma == 0 || valu_per_mfma == 1 || valu_per_mfma == 2 || valu_per_mfma == 4 ||
                    valu_per_mfma == 8;
  if (!ns_per_slot || !v_ok || (valu_per_mfma == 0 && !with_mfma) || (waves_per_simd != 1 && waves_per_simd != 2) ||
      lds_reads_per_two_mfma < 0 || lds_reads_per_two_mfma > 2 || (lds_reads_per_two_mfma && !with_mfma))
    return 2;
  return probe_issue(valu_per_mfma, with_mfma, waves_per_simd, lds_reads_per_two_mfma, ns_per_slot) == hipSuccess ? 0
                                                                                                                  : 1;
}

int MnbProbeDequantMfma16(int mode, int waves_per_simd, double* ns_per_step) {
  if (!ns_per_step || mode < 0 || mode > 3 || (waves_per_simd != 1 && waves_per_simd != 2)) return 2;
  return probe_dequant16(mode, waves_per_simd, ns_per_step) == hipSuccess ? 0 : 1;
}

int MnbProbeShaderClockStart(double sample_ms) {
  if (!(sample_ms > 0.0) || sample_ms > 1000.0) return 2;
  return clock_start(sample_ms) == hipSuccess ? 0 : 1;
}

int MnbProbeShaderClockFinish(double* ghz, double* sampled_ms) {
  if (!ghz || !sampled_ms) return 2;
  return clock_finish(ghz, sampled_ms) == hipSuccess ? 0 : 1;
}

}  // extern "C"
