/* Scalar C restatement of the W8A8 quantized-linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * Plain IEEE-754 binary32 arithmetic, one element at a time, compiled with
 * -ffp-contract=off and without fast-math so that every divide and multiply is
 * the correctly rounded one.  It exists to check the torch restatement
 * (w8a8_oracle.py) with independently written code and is never linked into or
 * called by the shipped library.  Each function cites the reference lines it follows.
 *
 * Input dtype codes: 0 = bf16, 1 = fp16, 2 = fp32.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static float fp16_to_f32(uint16_t h) {
  uint32_t s = (uint32_t)(h & 0x8000) << 16;
  int e = (h >> 10) & 0x1f;
  uint32_t m = h & 0x3ff;
  uint32_t u;
  if (e == 0) {
    if (m == 0) {
      u = s;
    } else { /* subnormal: value = m * 2^-24 */
      float f = (float)m * 5.9604644775390625e-08f;
      memcpy(&u, &f, 4);
      u |= s;
    }
  } else if (e == 31) {
    u = s | 0x7f800000u | (m << 13);
  } else {
    u = s | ((uint32_t)(e + 112) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static float load_elem(const void* p, int dtype, int64_t i) {
  if (dtype == 0) return bf16_to_f32(((const uint16_t*)p)[i]);
  if (dtype == 1) return fp16_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

/* fp32 -> OCP e4m3fn, round to nearest even, written from the bit layouts.
 * |x| > 448 after rounding saturates to 448 here; callers clamp first, as the
 * reference does, so that branch is not reached on the path. */
uint8_t oracle_e4m3fn_encode(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint8_t)(sign | 0x7f); /* NaN */
  if (a >= 0x43e80000u) return (uint8_t)(sign | 0x7e); /* >= 464 rounds past 448: saturate */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  if (a < 0x00800000u) return sign;         /* fp32 subnormal: far below 2^-10 */
  int shift;                                /* bits to drop from the 24-bit significand */
  if (e >= -6) {
    shift = 20; /* keep 1+3 bits */
  } else {
    shift = 20 + (-6 - e); /* e4m3 subnormal: quantum fixed at 2^-9 */
    if (shift > 25) return sign;
  }
  uint32_t kept = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) kept += 1;
  uint32_t code;
  if (e >= -6) {
    /* kept in [8,16]; 16 carries into the exponent */
    code = ((uint32_t)(e + 7) << 3) + (kept - 8);
  } else {
    code = kept; /* 0..8; 8 is the smallest normal */
  }
  return (uint8_t)(sign | code);
}

/* per_token_group_quant_8bit.cu:45,72-113 (fp8 destination). */
void oracle_group_quant_fp8(const void* x, int dtype, int64_t num_groups, int group_size, float eps,
                            float fp8_min, float fp8_max, uint8_t* q, float* s) {
  for (int64_t g = 0; g < num_groups; ++g) {
    float amax = eps; /* :45 */
    for (int j = 0; j < group_size; ++j) {
      float v = load_elem(x, dtype, g * group_size + j);
      amax = fmaxf(amax, fabsf(v)); /* :78-80 */
    }
    float y_s = amax / fp8_max; /* :86 */
    s[g] = y_s;                 /* :99-101 */
    for (int j = 0; j < group_size; ++j) {
      float v = load_elem(x, dtype, g * group_size + j);
      float qv = fminf(fmaxf(v / y_s, fp8_min), fp8_max); /* :110 */
      q[g * group_size + j] = oracle_e4m3fn_encode(qv);    /* :111 */
    }
  }
}

/* int8_kernel.py:38-48: absmax floor 1e-10, scale = absmax/127,
 * q = round_half_away(x * (127/absmax)). */
void oracle_token_quant_int8(const void* x, int dtype, int64_t rows, int64_t cols, int8_t* q, float* s) {
  for (int64_t r = 0; r < rows; ++r) {
    float amax = 0.f;
    for (int64_t j = 0; j < cols; ++j) amax = fmaxf(amax, fabsf(load_elem(x, dtype, r * cols + j)));
    amax = fmaxf(amax, 1e-10f); /* :39 */
    s[r] = amax / 127.0f;       /* :40 */
    float rr = 127.0f / amax;   /* :41 */
    for (int64_t j = 0; j < cols; ++j) {
      float v = roundf(load_elem(x, dtype, r * cols + j) * rr); /* :41-42 */
      if (v > 127.f) v = 127.f;
      if (v < -128.f) v = -128.f;
      q[r * cols + j] = (int8_t)v;
    }
  }
}

/* per_token_quant_fp8.cu:35-71 (guarded-inverse variant). */
void oracle_token_quant_fp8(const void* x, int dtype, int64_t rows, int64_t cols, uint8_t* q, float* s) {
  for (int64_t r = 0; r < rows; ++r) {
    float amax = 0.f; /* :35 */
    for (int64_t j = 0; j < cols; ++j) amax = fmaxf(amax, fabsf(load_elem(x, dtype, r * cols + j)));
    float scale = amax / 448.0f;                         /* :52 */
    float inv = (scale == 0.f) ? 0.f : 1.0f / scale;     /* :57 */
    s[r] = scale;
    for (int64_t j = 0; j < cols; ++j) {
      float v = load_elem(x, dtype, r * cols + j) * inv; /* :68 */
      v = fmaxf(fminf(v, 448.0f), -448.0f);              /* :69 */
      q[r * cols + j] = oracle_e4m3fn_encode(v);
    }
  }
}

/* per_tensor_quant_fp8.cu:10-123.  is_static == 0: *s = max|x| / 448 first (:44). */
void oracle_tensor_quant_fp8(const void* x, int dtype, int64_t n, int is_static, uint8_t* q, float* s) {
  if (!is_static) {
    float amax = 0.f; /* :13 */
    for (int64_t j = 0; j < n; ++j) amax = fmaxf(amax, fabsf(load_elem(x, dtype, j)));
    *s = amax / 448.0f;
  }
  float inv = 1.0f / *s; /* :56 */
  for (int64_t j = 0; j < n; ++j) {
    float v = load_elem(x, dtype, j) * inv;
    v = fmaxf(fminf(v, 448.0f), -448.0f); /* :70; fminf(NaN, 448) = 448 */
    q[j] = oracle_e4m3fn_encode(v);
  }
}

static float e4m3fn_decode(uint8_t c) {
  int e = (c >> 3) & 0xf;
  int m = c & 7;
  float v;
  if ((c & 0x7f) == 0x7f) return NAN;
  if (e == 0)
    v = (float)m * 0.001953125f; /* 2^-9 */
  else
    v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return (c & 0x80) ? -v : v;
}

float oracle_e4m3fn_decode(uint8_t c) { return e4m3fn_decode(c); }

/* fp8_blockwise_gemm_kernel.cu:345-423 semantics, evaluated in double:
 * D[m,n] = sum_kb P[m,n,kb] * SFA[m,kb] * SFB[kb, n/128].
 * a row-major [M,K]; bt row-major [N,K] (= column-major [K,N]);
 * sfa row-major [M,KB]; sfb row-major [NB,KB] (= weight_scale_inv). */
void oracle_fp8_blockwise_mm(const uint8_t* a, const uint8_t* bt, const float* sfa, const float* sfb,
                             int64_t M, int64_t N, int64_t K, double* out) {
  int64_t KB = (K + 127) / 128;
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t kb = 0; kb < KB; ++kb) {
        double p = 0.0;
        int64_t k1 = (kb + 1) * 128 < K ? (kb + 1) * 128 : K;
        for (int64_t k = kb * 128; k < k1; ++k)
          p += (double)e4m3fn_decode(a[m * K + k]) * (double)e4m3fn_decode(bt[n * K + k]);
        acc += p * (double)sfa[m * KB + kb] * (double)sfb[(n / 128) * KB + kb];
      }
      out[m * N + n] = acc;
    }
}

/* int8_kernel.py:273-296 (w8a8_block_int8_matmul), evaluated in double:
 * C[m,n] = sum_kb (sum_{k in kb} a[m,k] * bt[n,k]) * sfa[m,kb] * sfb[n/128, kb];
 * a [M,K], bt [N,K], sfa [M,KB], sfb [NB,KB], all row-major. */
void oracle_int8_blockwise_mm(const int8_t* a, const int8_t* bt, const float* sfa, const float* sfb,
                              int64_t M, int64_t N, int64_t K, double* out) {
  int64_t KB = (K + 127) / 128;
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t kb = 0; kb < KB; ++kb) {
        int64_t p = 0;
        int64_t k1 = (kb + 1) * 128 < K ? (kb + 1) * 128 : K;
        for (int64_t k = kb * 128; k < k1; ++k) p += (int64_t)a[m * K + k] * (int64_t)bt[n * K + k];
        acc += (double)p * (double)sfa[m * KB + kb] * (double)sfb[(n / 128) * KB + kb];
      }
      out[m * N + n] = acc;
    }
}

/* int8_gemm_kernel.cu: int8 x int8 -> int32 accumulators, exact. */
void oracle_int8_mm_i32(const int8_t* a, const int8_t* bt, int64_t M, int64_t N, int64_t K, int32_t* out) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      int32_t acc = 0;
      for (int64_t k = 0; k < K; ++k) acc += (int32_t)a[m * K + k] * (int32_t)bt[n * K + k];
      out[m * N + n] = acc;
    }
}
