// Buffer addressing, loads straight into LDS and hand-written wait counts: shared by the tile GEMMs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u4_t __attribute__((ext_vector_type(4)));  // plain register quad (HIP's uint4 struct resists SROA)
typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Buffer addressing: a 128-bit resource (uniform base, no range check: every offset is valid by construction) plus a
// 32-bit per-lane byte offset, so a load costs no 64-bit address arithmetic in the vector unit.  The host pass of the
// compiler knows these builtins but not the target features they need, and silently drops a whole kernel, launch
// stub included, that calls one: the calls are for the device pass only.
#if defined(__HIP_DEVICE_COMPILE__)
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t mnb_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, -1, 0x00020000);
}
__device__ __forceinline__ u2_t mnb_buffer_load_b64(rsrc_t r, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0);
}
__device__ __forceinline__ uint32_t mnb_buffer_load_b32(rsrc_t r, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0);
}
// 16 bytes per lane from the buffer straight into LDS: lane L's bytes land at `lds` (uniform) + 16 L.
__device__ __forceinline__ void mnb_buffer_load_lds_b128(rsrc_t r, uint32_t off, lds_ptr_t lds) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, lds, 16, (int)off, 0, 0, 0);
}
#else
struct rsrc_t {};
inline rsrc_t mnb_rsrc(const void*) { return {}; }
inline u2_t mnb_buffer_load_b64(rsrc_t, uint32_t) { return u2_t{0, 0}; }
inline uint32_t mnb_buffer_load_b32(rsrc_t, uint32_t) { return 0; }
inline void mnb_buffer_load_lds_b128(rsrc_t, uint32_t, lds_ptr_t) {}
#endif

// s_waitcnt immediate that waits until at most VM vector-memory operations are outstanding and every LDS operation
// of the wavefront has completed (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14).
constexpr int waitcnt_vm_lds0(int vm) { return (vm & 15) | (7 << 4) | (0 << 8) | ((vm >> 4) << 14); }
// The same for vector-memory operations only (LDS and scalar-memory counters untouched).
constexpr int waitcnt_vm(int vm) { return (vm & 15) | (7 << 4) | (15 << 8) | ((vm >> 4) << 14); }

