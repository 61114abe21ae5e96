// Shared device/host helpers for the gfx950 DSA kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/dsa_hip.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// ---- error plumbing (never throws across the C ABI) ------------------------------------
void dsa_set_error(const char* fmt, ...);
#define DSA_FAIL(code, ...) do { dsa_set_error(__VA_ARGS__); return (code); } while (0)
#define DSA_REQUIRE(cond, ...) do { if (!(cond)) DSA_FAIL(DSA_ERR_BAD_ARG, __VA_ARGS__); } while (0)
#define DSA_CHECK_LAUNCH(name) do { hipError_t e_ = hipGetLastError(); \
    if (e_ != hipSuccess) DSA_FAIL(DSA_ERR_LAUNCH, "%s: launch failed: %s", name, hipGetErrorString(e_)); } while (0)

// hipFuncSetAttribute(fn, MaxDynamicSharedMemorySize, bytes), once per kernel and device while `bytes` does not
// grow: the call costs several microseconds of host time, which a short kernel sequence cannot hide.
hipError_t dsa_reserve_lds(const void* fn, size_t bytes);

// ---- small device helpers ----------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(unsigned short h) {
  return __builtin_bit_cast(float, ((unsigned)h) << 16);
}
__device__ __forceinline__ unsigned short f32_to_bf16_bits(float f) {   // round-to-nearest-even
  unsigned u = __builtin_bit_cast(unsigned, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}
__device__ __forceinline__ unsigned pack_bf16x2(float lo, float hi) {
  return (unsigned)f32_to_bf16_bits(lo) | ((unsigned)f32_to_bf16_bits(hi) << 16);
}
// the same rounding in one instruction (v_cvt_pk_bf16_f32)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned cvt_pk_bf16(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2_t));
}
// v_permlane32_swap: the upper half-wave of a trades places with the lower half-wave of b.
__device__ __forceinline__ void swap_halves(unsigned& a, unsigned& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
// A 32 x 32 MFMA accumulator gives lane (r, g = lane / 32) the elements 8j + 4g .. +3 (j = 0..3) of row
// segment r: four 8-byte pieces once rounded to bf16.  The two half-waves trade pieces so that the lane
// ends up with elements 8 (jj + g) .. +7 for jj = 0 and jj = 2: two 16-byte values, o[0] and o[1].
// Every lane of the wave must take part.
__device__ __forceinline__ void acc_row_to_16B(const f32x16& acc, float scale, uint4 (&o)[2]) {
  unsigned pc[4][2];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    pc[j][0] = cvt_pk_bf16(acc[4 * j] * scale, acc[4 * j + 1] * scale);
    pc[j][1] = cvt_pk_bf16(acc[4 * j + 2] * scale, acc[4 * j + 3] * scale);
  }
#pragma unroll
  for (int jj = 0; jj < 4; jj += 2) {
    swap_halves(pc[jj][0], pc[jj + 1][0]);
    swap_halves(pc[jj][1], pc[jj + 1][1]);
    o[jj >> 1] = make_uint4(pc[jj][0], pc[jj][1], pc[jj + 1][0], pc[jj + 1][1]);
  }
}
// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding).
#define DSA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt((((n) & 0xf) | (((n) >> 4) << 14)) | (0x7 << 4) | (0xf << 8))

static inline int dsa_cdiv(long a, long b) { return (int)((a + b - 1) / b); }
