// Device helpers shared by the MFMA kernels of libmoa_hip.so (prefill, grouped-query decode):
// element types with their v_mfma_f32_32x32x16 wrapper, asynchronous global->LDS copies,
// LDS operand reads (plain and transposing), small wave-level utilities.  gfx950 only.
#pragma once
#include "moa_common.h"

namespace moa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));


struct PF16 {
  static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack_rne(float lo, float hi) {   // one v_cvt_pk_f16_f32
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 r = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, r);
  }
};
struct PBF16 {
  static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack_rne(float lo, float hi) {   // one v_cvt_pk_bf16_f32
    f32x2 x = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2v));
  }
};

// Asynchronous 16-byte-per-lane copy global -> LDS (global_load_lds_dwordx4): lane i of the wave
// reads base + byte_off(i) and lands at LDS byte address lds_addr + 16*i.  base and lds_addr are
// wave-uniform.  Written as inline assembly on purpose: the compiler cannot prove that these LDS
// writes do not alias the operand reads of the stage being computed and would otherwise put a
// full vmcnt(0) wait in front of every LDS read; completion is tracked by hand with wait_vm().
// Loads complete in order, so the compiler's own vmcnt bookkeeping for ordinary loads stays safe
// (it can only wait longer than it planned).
__device__ __forceinline__ void async_copy16(const void* base, uint32_t byte_off, uint32_t lds_addr) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %1"
      :
      : "v"(byte_off), "s"(base), "s"(__builtin_amdgcn_readfirstlane(lds_addr))
      : "memory");
}
// max of a value with its twin in the other half of the wave (lane ^ 32), without going through LDS
__device__ __forceinline__ float max_with_other_half(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}
__device__ __forceinline__ uint32_t lds_address(const char* p) {
  return (uint32_t)(uintptr_t)((const char __attribute__((address_space(3)))*)p);
}
// Wait until at most n of this wave's global loads / async copies are outstanding.
__device__ __forceinline__ void wait_vm(int n) {
  if (n >= 32) asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
  else if (n >= 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else if (n >= 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if (n >= 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else if (n >= 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else if (n == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
  else if (n == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
  else if (n == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// The same for a count known at compile time.
template <int N>
__device__ __forceinline__ void wait_vm_exact() {
  static_assert(N >= 0 && N < 64, "vmcnt holds 6 bits");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Work-group barrier WITHOUT the memory fence of __syncthreads(): the fence would make every wave
// wait for all of its outstanding async copies (vmcnt(0)) at each phase boundary and serialise the
// copy pipeline.  What must be visible at a barrier is waited for explicitly with wait_vm().
__device__ __forceinline__ void phase_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// sm_scale * log2(e) as the MFMA kernels take it.  They mask a score by setting it to -inf before
// the multiply-add with the scale, and -inf * 0 is NaN: a scale of exactly zero (uniform weights) is
// replaced by one so small that every finite score still maps to 2^0 = 1 exactly.
inline float mfma_softmax_scale(float sm_scale) {
  const float s = sm_scale * 1.4426950408889634f;
  return s == 0.f ? 1e-30f : s;
}

template <int P>
struct IC {
  static constexpr int value = P;
};

// LDS accesses by 32-bit LDS byte address (a VGPR) plus a compile-time offset, so that the stage
// and row selection of an operand costs no VALU instruction.
__device__ __forceinline__ u32x4 lds_load16(uint32_t addr, int imm) {
  typedef u32x4 __attribute__((address_space(3))) * lds_u32x4_ptr;
  return *(lds_u32x4_ptr)(uintptr_t)(addr + imm);
}
__device__ __forceinline__ void lds_store8(uint32_t addr, u32x2 v) {
  typedef u32x2 __attribute__((address_space(3))) * lds_u32x2_ptr;
  *(lds_u32x2_ptr)(uintptr_t)addr = v;
}
// The transposing read: 4 consecutive rows of one 16-bit column out of a row-major LDS tile.  Within
// each group of 16 lanes, lane i must point at (row0 + i/4, col0 + 4*(i%4)); it receives rows
// row0..row0+3 of column col0 + i.
__device__ __forceinline__ u32x2 lds_load_tr16(uint32_t addr, int imm) {
  typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
  s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(uintptr_t)(addr + imm));
  return __builtin_bit_cast(u32x2, r);
}

}  // namespace moa
