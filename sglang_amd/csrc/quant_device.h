// Device pieces of the activation quantizers that more than one translation unit uses: the
// group quantizer itself (quant.hip) and the GEMM that quantizes its activations on the fly
// (gemm.hip).  Both must produce the same codes and scales bit for bit, so both build them from
// these functions.
#pragma once
#include "sglq_common.h"

namespace sglq {

// ---------------------------------------------------------------------------
// 8 consecutive input elements -> 8 floats, plus the bit pattern of their abs-max
// ---------------------------------------------------------------------------
template <int DT>
struct Chunk8;

template <>
struct Chunk8<SGLQ_BF16> {
  v4u raw;
  static constexpr int kBytes = 16;
  SGLQ_MEM void load(const void* p) { raw = *reinterpret_cast<const v4u*>(p); }
  // for data that is read exactly once: the non-temporal hint keeps it from displacing what the
  // last-level cache holds for the kernels around this one
  SGLQ_MEM void load_once(const void* p) { raw = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p)); }
  SGLQ_MEM uint32_t amax_bits() const {
    // |bf16| orders like its low 15 bits taken as an integer: packed 16-bit max.
    v2us m = {0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t a = raw[i] & 0x7fff7fffu;
      m = __builtin_elementwise_max(m, __builtin_bit_cast(v2us, a));
    }
    uint32_t hi = m.x > m.y ? m.x : m.y;
    return hi << 16;
  }
  SGLQ_MEM float get(int i) const {
    uint32_t w = raw[i >> 1];
    return u2f((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
};

template <>
struct Chunk8<SGLQ_FP16> {
  v4u raw;
  static constexpr int kBytes = 16;
  SGLQ_MEM void load(const void* p) { raw = *reinterpret_cast<const v4u*>(p); }
  // for data that is read exactly once: the non-temporal hint keeps it from displacing what the
  // last-level cache holds for the kernels around this one
  SGLQ_MEM void load_once(const void* p) { raw = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p)); }
  SGLQ_MEM float get(int i) const {
    uint32_t w = raw[i >> 1];
    unsigned short h = (i & 1) ? (unsigned short)(w >> 16) : (unsigned short)(w & 0xffffu);
    return (float)__builtin_bit_cast(_Float16, h);
  }
  SGLQ_MEM uint32_t amax_bits() const {
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) m = umax(m, f2u(get(i)) & 0x7fffffffu);
    return m;
  }
};

template <>
struct Chunk8<SGLQ_FP32> {
  v4u raw[2];
  static constexpr int kBytes = 32;
  SGLQ_MEM void load(const void* p) {
    raw[0] = reinterpret_cast<const v4u*>(p)[0];
    raw[1] = reinterpret_cast<const v4u*>(p)[1];
  }
  SGLQ_MEM void load_once(const void* p) {
    raw[0] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p));
    raw[1] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p) + 1);
  }
  SGLQ_MEM float get(int i) const { return u2f(raw[i >> 2][i & 3]); }
  SGLQ_MEM uint32_t amax_bits() const {
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) m = umax(m, raw[i >> 2][i & 3] & 0x7fffffffu);
    return m;
  }
};

template <int DT>
constexpr int elem_bytes() {
  return DT == SGLQ_FP32 ? 4 : 2;
}

// 8 quantized floats -> 8 bytes
struct Fp8Pack {
  SGLQ_DEV v2u pack(const float (&v)[8]) {
    v2u o;
    uint32_t w = cvt_pk_e4m3<false>(v[0], v[1], 0);
    o.x = cvt_pk_e4m3<true>(v[2], v[3], w);
    w = cvt_pk_e4m3<false>(v[4], v[5], 0);
    o.y = cvt_pk_e4m3<true>(v[6], v[7], w);
    return o;
  }
};

struct I8Pack {
  // inputs are already integral (or to be truncated) and inside [-128, 127]
  SGLQ_DEV v2u pack(const float (&v)[8]) {
    v2u o;
    o.x = ((uint32_t)(int)v[0] & 0xffu) | (((uint32_t)(int)v[1] & 0xffu) << 8) |
          (((uint32_t)(int)v[2] & 0xffu) << 16) | ((uint32_t)(int)v[3] << 24);
    o.y = ((uint32_t)(int)v[4] & 0xffu) | (((uint32_t)(int)v[5] & 0xffu) << 8) |
          (((uint32_t)(int)v[6] & 0xffu) << 16) | ((uint32_t)(int)v[7] << 24);
    return o;
  }
};

// Division of a 32-bit index by a runtime-constant divisor (Granlund-Montgomery).
struct FastDiv {
  uint32_t d, magic, shift;
  void init(uint32_t div) {
    d = div;
    uint32_t l = 0;
    while ((1ull << l) < div) ++l;
    magic = (uint32_t)(((1ull << 32) * ((1ull << l) - div)) / div + 1);
    shift = l;
  }
  SGLQ_MEM uint32_t div(uint32_t n) const {
    uint32_t t = __umulhi(magic, n);
    // shift may be 0 (d == 1): split the shift so that no shift count is negative
    uint32_t s1 = shift > 0 ? 1u : 0u;
    return (t + ((n - t) >> s1)) >> (shift - s1);
  }
};

template <bool CLAMP>
SGLQ_DEV float quantize_elem(float x, float y_s, float r, float qmin, float qmax) {
  float q = div_by(x, y_s, r);
  if constexpr (CLAMP) q = clampf(q, qmin, qmax);
  return __builtin_copysignf(q, x);
}

}  // namespace sglq
