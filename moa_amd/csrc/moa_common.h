// Shared host/device helpers of libmoa_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/moa_hip.h"

namespace moa {

// ---- error string (thread local, host) -----------------------------------
char* error_buffer();
int fail(int code, const char* fmt, ...);

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MOA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return MOA_OK;
}

// Raises a kernel's dynamic LDS limit.  The attribute belongs to the function on the current device,
// so it is set once per device; `done` is the caller's per-kernel table.  Two threads racing here both
// set the same value.
constexpr int kMaxDevices = 64;
inline int reserve_lds(const void* kernel, size_t bytes, bool (&done)[kMaxDevices], const char* what) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MOA_ERR_LAUNCH, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (tracked && done[dev]) return MOA_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess)
    return fail(MOA_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS: %s", what, bytes, hipGetErrorString(e));
  if (tracked) done[dev] = true;
  return MOA_OK;
}

inline int elem_bytes(int dtype) {
  switch (dtype) {
    case MOA_DTYPE_F16: return 2;
    case MOA_DTYPE_BF16: return 2;
    case MOA_DTYPE_F32: return 4;
    default: return 0;
  }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ---- device helpers ---------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// torch's integer `%`: the result takes the sign of the divisor.
// A zero divisor (a head without a ring) yields 0 instead of undefined behaviour.
__device__ __forceinline__ int64_t py_mod(int64_t a, int64_t m) {
  if (m == 0) return 0;
  int64_t r = a % m;
  return (r != 0 && ((r < 0) != (m < 0))) ? r + m : r;
}

// DPP lane exchanges inside a row of 16 lanes.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
constexpr int DPP_QUAD_XOR1 = 0xB1;      // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;      // quad_perm [2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

// Sum over aligned groups of W lanes (W = 4, 8 or 16); every lane gets the sum.
template <int W>
__device__ __forceinline__ float group_sum(float x) {
  x += dpp_f32<DPP_QUAD_XOR1>(x);
  x += dpp_f32<DPP_QUAD_XOR2>(x);
  if (W >= 8) x += dpp_f32<DPP_ROW_HALF_MIRROR>(x);
  if (W >= 16) x += dpp_f32<DPP_ROW_MIRROR>(x);
  return x;
}

}  // namespace moa
