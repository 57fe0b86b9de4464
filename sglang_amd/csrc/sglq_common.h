// Shared device helpers for the gfx950 (CDNA4, wave64) W8A8 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sglq.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned short v2us __attribute__((ext_vector_type(2)));

#define SGLQ_DEV static __device__ __forceinline__
#define SGLQ_MEM __device__ __forceinline__

namespace sglq {

// Thread-local message behind sglq_last_error().
void set_error(const char* fmt, ...);

SGLQ_DEV float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
SGLQ_DEV uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// DPP lane exchanges inside a 16-lane row; all are full-rate VALU modifiers.
template <int CTRL>
SGLQ_DEV uint32_t dpp(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
constexpr int DPP_XOR1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int DPP_XOR2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141; // reverse within 8 lanes
constexpr int DPP_MIRROR = 0x140;      // reverse within 16 lanes

SGLQ_DEV uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

// Max over LANES (1,2,4,8,16) adjacent lanes of non-negative floats held as bit
// patterns: integer order equals float order there, and the integer max needs
// no NaN canonicalisation.  Every lane of the group ends with the group max.
template <int LANES>
SGLQ_DEV uint32_t group_umax(uint32_t v) {
  if constexpr (LANES >= 2) v = umax(v, dpp<DPP_XOR1>(v));
  if constexpr (LANES >= 4) v = umax(v, dpp<DPP_XOR2>(v));
  if constexpr (LANES >= 8) v = umax(v, dpp<DPP_HALF_MIRROR>(v));
  if constexpr (LANES >= 16) v = umax(v, dpp<DPP_MIRROR>(v));
  return v;
}

// Max over the whole 64-lane wavefront.
SGLQ_DEV uint32_t wave_umax(uint32_t v) {
  v = group_umax<16>(v);
  v = umax(v, (uint32_t)__shfl_xor((int)v, 16));
  v = umax(v, (uint32_t)__shfl_xor((int)v, 32));
  return v;
}

// Correctly rounded x / y given r = RN(1 / y): one multiply and two FMAs.
// Exact for every quotient that can reach an 8-bit code (searched on the CPU by
// tests/csrc/exact_div_check.c).
SGLQ_DEV float div_by(float x, float y, float r) {
  float q0 = x * r;
  float e = __builtin_fmaf(-q0, y, x);
  return __builtin_fmaf(e, r, q0);
}

// Two fp32 -> two OCP e4m3fn bytes (round to nearest even) in the low or high
// half of `old`.  gfx950 converts to the OCP format natively.
template <bool HI>
SGLQ_DEV uint32_t cvt_pk_e4m3(float a, float b, uint32_t old) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, HI);
}

SGLQ_DEV float clampf(float v, float lo, float hi) { return __builtin_amdgcn_fmed3f(v, lo, hi); }

// Buffer resource over a dense allocation: out-of-range lanes read zero.
SGLQ_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// 16-bit floats (dtype code SGLQ_BF16 or SGLQ_FP16) as raw bits <-> fp32, round to nearest even.
template <int DT>
SGLQ_DEV float to_f32_16(uint16_t h) {
  if constexpr (DT == SGLQ_BF16) return u2f((uint32_t)h << 16);
  else return (float)__builtin_bit_cast(_Float16, h);
}
template <int DT>
SGLQ_DEV uint16_t from_f32_16(float v) {
  if constexpr (DT == SGLQ_BF16) return __builtin_bit_cast(uint16_t, (__bf16)v);
  else return __builtin_bit_cast(uint16_t, (_Float16)v);
}

// silu(v) = v / (1 + exp(-v)) in fp32 with the hardware's exp2 and reciprocal (each within one
// unit in the last place; the reference writes v / (1 + expf(-v)),
// sgl-kernel/csrc/elementwise/activation.cu:57-60, and builds with -use_fast_math,
// sgl-kernel/CMakeLists.txt:190, which makes both approximate as well).  exp2 overflows to +inf for v below
// about -88, where the result is -0 like the exact quotient's.
SGLQ_DEV float silu_f32(float v) {
  const float e = __builtin_amdgcn_exp2f(v * -1.44269504088896340736f);
  return v * __builtin_amdgcn_rcpf(1.0f + e);
}

// T(T(silu(x)) * y): both roundings of the reference's activation kernel (activation.cu:57-60,85-103).
template <int DT>
SGLQ_DEV uint16_t silu_mul_16(uint16_t xb, uint16_t yb) {
  float s = silu_f32(to_f32_16<DT>(xb));
  // (keeps the product and its rounding to 16 bits apart: fused into one mixed-precision
  // multiply-add with a +0 addend, silu(-0) would come out as +0)
  asm volatile("" : "+v"(s));
  const float act = to_f32_16<DT>(from_f32_16<DT>(s));
  return from_f32_16<DT>(act * to_f32_16<DT>(yb));
}

}  // namespace sglq
