// Activation quantization kernels for gfx950: per-token-group FP8/INT8,
// per-token FP8 and per-token INT8.  All are HBM-bound: every element is read
// once with 128-bit loads, kept in registers across the abs-max reduction
// (DPP inside 16-lane rows), and written once.
//
// Arithmetic contract (bit-exact with the reference's definitions):
//   group  : amax = max(eps, max|x|); s = amax / max8; q = clamp(x / s)     (IEEE divides)
//   tok fp8: amax = max|x|; s = amax / 448; inv = s == 0 ? 0 : 1/s; q = clamp(x * inv)
//   tok i8 : amax = max(max|x|, 1e-10); s = amax / 127; q = roundf(x * (127 / amax))
// The per-element divide of the group kernel is evaluated as a multiply by the
// correctly rounded reciprocal plus an exact FMA remainder correction, which
// returns the IEEE quotient (see div_by).  NaN inputs are outside the contract.
#include "quant_device.h"
#include "sglq_common.h"

namespace sglq {

// ---------------------------------------------------------------------------
// Per-token-group quantization.  16 elements per lane as two 8-element chunks
// half a group apart, so every load instruction reads fully used 128-byte runs.
// ---------------------------------------------------------------------------
//
// CLAMP = false is the standard e4m3fn case (bounds -448/+448): |x| <= amax bounds
// the quotient by 448 * (1 + 2^-22), which rounds to the code of 448 anyway, so
// the explicit clamp is dropped.  The quotient's sign is copied from x so that
// -0.0 stays -0.0 (the remainder correction would turn it into +0.0).
// POW2: the scale is the smallest power of two >= max(amax / qmax, 1e-10) (the UE8M0 rule of
// per_token_group_quant_8bit.cu:86-89, see group_quant_ue8m0_kernel), stored as fp32; the codes are
// x times its exact inverse, clamped as that kernel clamps them.
template <int DT, int GROUP, int NCH, int UNROLL, bool STRIDED_SCALE, bool TO_INT8, bool CLAMP, bool STREAM_IN = false, bool POW2 = false>
__global__ __launch_bounds__(256) void group_quant_kernel(const char* __restrict__ x, char* __restrict__ q,
                                                          float* __restrict__ s, uint32_t num_groups,
                                                          FastDiv groups_per_row, int64_t s_stride_row,
                                                          int64_t s_stride_col, float eps, float qmin, float qmax,
                                                          float rqmax) {
  // NCH 8-element chunks per lane, GROUP / NCH elements apart, so that the lanes of a
  // group read (and write) one contiguous run per chunk index.
  constexpr int LPG = GROUP / (8 * NCH);  // lanes per group
  constexpr int GPB = 256 / LPG;          // groups per block per step
  constexpr int EB = elem_bytes<DT>();
  const uint32_t t = threadIdx.x;
  const uint32_t sub = t % LPG;
  const uint32_t g0 = blockIdx.x * (UNROLL * GPB) + t / LPG;

  Chunk8<DT> ch[UNROLL][NCH];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const uint32_t gid = g0 + u * GPB;
    if (gid < num_groups) {
      const char* p = x + ((int64_t)gid * GROUP + sub * 8) * EB;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        // (an input of half the last-level cache and more is read past it: what the cache holds for the
        // kernels around this one, often the previous GEMM's output still to be written back, stays put)
        if constexpr (STREAM_IN) ch[u][c].load_once(p + c * (GROUP / NCH) * EB);
        else ch[u][c].load(p + c * (GROUP / NCH) * EB);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const uint32_t gid = g0 + u * GPB;
    if (gid < num_groups) {
      uint32_t mb = ch[u][0].amax_bits();
#pragma unroll
      for (int c = 1; c < NCH; ++c) mb = umax(mb, ch[u][c].amax_bits());
      mb = group_umax<LPG>(mb);
      const float amax = u2f(umax(mb, f2u(eps)));
      float y_s = div_by(amax, qmax, rqmax);
      float r = 1.0f / y_s;
      if constexpr (POW2) {
        const uint32_t bits = f2u(__builtin_fmaxf(y_s, 1e-10f));  // positive and normal
        const uint32_t biased = (bits >> 23) + ((bits & 0x7fffffu) != 0 ? 1u : 0u);
        y_s = u2f(biased << 23);
        r = u2f((254u - biased) << 23);  // exact
      }
      char* qp = q + (int64_t)gid * GROUP + sub * 8;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        float v[8];
        v2u o;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if constexpr (POW2) v[i] = __builtin_fminf(__builtin_fmaxf(ch[u][c].get(i) * r, qmin), qmax);
          else v[i] = quantize_elem<CLAMP>(ch[u][c].get(i), y_s, r, qmin, qmax);
        }
        if constexpr (TO_INT8) o = I8Pack::pack(v); else o = Fp8Pack::pack(v);
        *reinterpret_cast<v2u*>(qp + c * (GROUP / NCH)) = o;
      }
      if (sub == 0) {
        if constexpr (STRIDED_SCALE) {
          const uint32_t row = groups_per_row.div(gid);
          const uint32_t col = gid - row * groups_per_row.d;
          s[row * s_stride_row + col * s_stride_col] = y_s;
        } else {
          s[gid] = y_s;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Per-token-group FP8 quantization (group 128) whose result goes straight to the expert-major
// rows an MoE layer gathers it into (python/sglang/srt/layers/moe/cutlass_moe.py:156-158:
// quantize once per token, then shuffle_rows codes and scales by a_map): token t's codes and
// row-major scales are written to every row slot_map[t * topk + j], j < topk, that lies in
// [0, num_dst_rows); other entries (slots routed to nobody) are skipped.  Same arithmetic as
// group_quant_kernel; each token is read once and written topk times instead of being
// written once, read topk times and written topk times.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void group_quant_scatter_kernel(const char* __restrict__ x, char* __restrict__ q,
                                                                  float* __restrict__ s, const int* __restrict__ slot_map,
                                                                  uint32_t num_groups, FastDiv groups_per_row, int topk,
                                                                  int64_t num_dst_rows, float eps, float qmax, float rqmax) {
  constexpr int GROUP = 128, NCH = 2, LPG = GROUP / (8 * NCH), GPB = 256 / LPG;
  constexpr int EB = elem_bytes<DT>();
  const uint32_t t = threadIdx.x;
  const uint32_t sub = t % LPG;
  const uint32_t gid = blockIdx.x * GPB + t / LPG;
  if (gid >= num_groups) return;
  const uint32_t row = groups_per_row.div(gid);
  const uint32_t col = gid - row * groups_per_row.d;
  const int64_t hidden = (int64_t)groups_per_row.d * GROUP;
  Chunk8<DT> ch[NCH];
  const char* px = x + ((int64_t)gid * GROUP + sub * 8) * EB;
#pragma unroll
  for (int c = 0; c < NCH; ++c) ch[c].load(px + c * (GROUP / NCH) * EB);
  uint32_t mb = umax(ch[0].amax_bits(), ch[1].amax_bits());
  mb = group_umax<LPG>(mb);
  const float amax = u2f(umax(mb, f2u(eps)));
  const float y_s = div_by(amax, qmax, rqmax);
  const float r = 1.0f / y_s;
  v2u o[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = quantize_elem<false>(ch[c].get(i), y_s, r, -qmax, qmax);
    o[c] = Fp8Pack::pack(v);
  }
  for (int j = 0; j < topk; ++j) {
    const int64_t dst = slot_map[(int64_t)row * topk + j];
    if (dst < 0 || dst >= num_dst_rows) continue;
    char* qp = q + dst * hidden + (int64_t)col * GROUP + sub * 8;
#pragma unroll
    for (int c = 0; c < NCH; ++c) *reinterpret_cast<v2u*>(qp + c * (GROUP / NCH)) = o[c];
    if (sub == 0) s[dst * groups_per_row.d + col] = y_s;
  }
}

// ---------------------------------------------------------------------------
// SiLU-and-multiply fused with the per-token-group FP8 quantization that follows it in an MoE
// expert layer (python/sglang/srt/layers/moe/cutlass_moe.py:187-194): input [tokens, 2 d] in a
// 16-bit type, codes [tokens, d] and row-major scales [tokens, d / 128] of
// t = T(T(silu(x[:, :d])) * x[:, d:]) quantized in groups of 128 exactly as
// group_quant_kernel quantizes a stored t.  The intermediate is never written: 4 bytes read
// and 1 written per element instead of 6 + 3 for the two kernels.  8 lanes per group, two
// 8-element chunks per lane half a group apart.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void silu_mul_group_quant_kernel(const char* __restrict__ x, char* __restrict__ q,
                                                                   float* __restrict__ s, uint32_t num_groups,
                                                                   FastDiv groups_per_row, float eps, float qmax,
                                                                   float rqmax) {
  static_assert(DT == SGLQ_BF16 || DT == SGLQ_FP16, "16-bit inputs");
  constexpr int GROUP = 128, NCH = 2, LPG = GROUP / (8 * NCH), GPB = 256 / LPG;
  const uint32_t t = threadIdx.x;
  const uint32_t sub = t % LPG;
  const uint32_t gid = blockIdx.x * GPB + t / LPG;
  if (gid >= num_groups) return;
  const uint32_t row = groups_per_row.div(gid);
  const uint32_t col = gid - row * groups_per_row.d;
  const int64_t d = (int64_t)groups_per_row.d * GROUP;
  const char* px = x + ((int64_t)row * 2 * d + (int64_t)col * GROUP + sub * 8) * 2;
  Chunk8<DT> ch[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const v4u xv = *reinterpret_cast<const v4u*>(px + c * (GROUP / NCH) * 2);
    const v4u yv = *reinterpret_cast<const v4u*>(px + d * 2 + c * (GROUP / NCH) * 2);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t lo = silu_mul_16<DT>((uint16_t)(xv[w] & 0xffffu), (uint16_t)(yv[w] & 0xffffu));
      const uint32_t hi = silu_mul_16<DT>((uint16_t)(xv[w] >> 16), (uint16_t)(yv[w] >> 16));
      ch[c].raw[w] = lo | (hi << 16);
    }
  }
  uint32_t mb = umax(ch[0].amax_bits(), ch[1].amax_bits());
  mb = group_umax<LPG>(mb);
  const float amax = u2f(umax(mb, f2u(eps)));
  const float y_s = div_by(amax, qmax, rqmax);
  const float r = 1.0f / y_s;
  char* qp = q + (int64_t)gid * GROUP + sub * 8;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = quantize_elem<false>(ch[c].get(i), y_s, r, -qmax, qmax);
    *reinterpret_cast<v2u*>(qp + c * (GROUP / NCH)) = Fp8Pack::pack(v);
  }
  if (sub == 0) s[gid] = y_s;
}

// ---------------------------------------------------------------------------
// Per-token-group FP8 quantization with power-of-two scales packed as exponent bytes
// (scale_ue8m0, per_token_group_quant_8bit.cu:86-105 and :50-65; groups of 128).  The scale
// is the smallest power of two >= max(amax / 448, 1e-10), which is what
// exp2f(ceilf(log2f(.))) (:87-89) yields wherever log2f's own rounding cannot cross an
// integer: always for bf16 / fp16 inputs (amax / 448 is then an exact power of two or at
// least 2^-9 away from one in relative terms), and for fp32 inputs except a quotient a few
// units in the last place above a power of two.  Byte g % 4 of 32-bit word
// [g / 4][row] of the output (word column stride s_stride_col) is the biased exponent of
// group g's scale (:57-64, :94).  16 lanes per group, 8 elements per lane.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void group_quant_ue8m0_kernel(const char* __restrict__ x, char* __restrict__ q,
                                                                unsigned char* __restrict__ s, uint32_t num_groups,
                                                                FastDiv groups_per_row, int64_t s_stride_col, float eps,
                                                                float qmin, float qmax, float rqmax) {
  constexpr int EB = elem_bytes<DT>();
  const uint32_t sub = threadIdx.x & 15;
  const uint32_t gid = blockIdx.x * 16 + (threadIdx.x >> 4);
  if (gid >= num_groups) return;
  Chunk8<DT> ch;
  ch.load(x + ((int64_t)gid * 128 + sub * 8) * EB);
  const uint32_t mb = group_umax<16>(ch.amax_bits());
  const float amax = u2f(umax(mb, f2u(eps)));
  const float y = __builtin_fmaxf(div_by(amax, qmax, rqmax), 1e-10f);
  const uint32_t bits = f2u(y);  // positive and normal (>= 1e-10)
  const uint32_t biased = (bits >> 23) + ((bits & 0x7fffffu) != 0 ? 1u : 0u);  // exponent of the power of two >= y
  const float inv = u2f((254u - biased) << 23);                                // 2^-(biased - 127), exact
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = __builtin_fminf(__builtin_fmaxf(ch.get(i) * inv, qmin), qmax);
  *reinterpret_cast<v2u*>(q + (int64_t)gid * 128 + sub * 8) = Fp8Pack::pack(v);
  if (sub == 0) {
    const uint32_t row = groups_per_row.div(gid);
    const uint32_t col = gid - row * groups_per_row.d;
    s[((int64_t)(col >> 2) * s_stride_col + row) * 4 + (col & 3)] = (unsigned char)biased;
  }
}

// ---------------------------------------------------------------------------
// Per-token (whole-row) quantization.  TEAM lanes share one row (64 = one
// wavefront, 256 = the block); each lane keeps V 16-byte chunks in registers.
// ---------------------------------------------------------------------------
constexpr int MODE_FP8 = 0;
constexpr int MODE_INT8 = 1;

template <int DT, int TEAM, int V, int MODE>
__global__ __launch_bounds__(256) void token_quant_kernel(const char* __restrict__ x, char* __restrict__ q,
                                                          float* __restrict__ s, void* __restrict__ row_sum,
                                                          int64_t rows, uint32_t chunks) {
  constexpr int EB = elem_bytes<DT>();
  constexpr int TEAMS = 256 / TEAM;
  __shared__ uint32_t red_max[4];
  __shared__ float red_sum[4];
  const uint32_t t = threadIdx.x % TEAM;
  const int64_t row = (int64_t)blockIdx.x * TEAMS + threadIdx.x / TEAM;
  const bool live = row < rows;
  const char* xr = x + row * (int64_t)chunks * 8 * EB;

  Chunk8<DT> c[V];
  uint32_t mb = 0;
  float sum = 0.f;
#pragma unroll
  for (int v = 0; v < V; ++v) {
    const uint32_t ci = t + v * TEAM;
    if (live && ci < chunks) c[v].load(xr + (int64_t)ci * 8 * EB);
  }
#pragma unroll
  for (int v = 0; v < V; ++v) {
    const uint32_t ci = t + v * TEAM;
    if (live && ci < chunks) {
      mb = umax(mb, c[v].amax_bits());
      if (MODE == MODE_INT8 && row_sum != nullptr) {
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += c[v].get(i);
      }
    }
  }
  mb = wave_umax(mb);
  if (MODE == MODE_INT8 && row_sum != nullptr) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
  }
  if constexpr (TEAM == 256) {
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
      red_max[w] = mb;
      red_sum[w] = sum;
    }
    __syncthreads();
    mb = umax(umax(red_max[0], red_max[1]), umax(red_max[2], red_max[3]));
    sum = (red_sum[0] + red_sum[1]) + (red_sum[2] + red_sum[3]);
  }
  if (!live) return;

  float scale, mul, lo, hi;
  if constexpr (MODE == MODE_FP8) {
    const float amax = u2f(mb);
    scale = amax / 448.0f;
    mul = (scale == 0.f) ? 0.f : 1.0f / scale;
    lo = -448.0f;
    hi = 448.0f;
  } else {
    const float amax = u2f(umax(mb, f2u(1e-10f)));
    scale = amax / 127.0f;
    mul = 127.0f / amax;
    lo = -128.0f;
    hi = 127.0f;
  }
  if (t == 0) {
    s[row] = scale;
    if (MODE == MODE_INT8 && row_sum != nullptr) {
      if constexpr (DT == SGLQ_BF16) reinterpret_cast<__bf16*>(row_sum)[row] = (__bf16)sum;
      else if constexpr (DT == SGLQ_FP16) reinterpret_cast<_Float16*>(row_sum)[row] = (_Float16)sum;
      else reinterpret_cast<float*>(row_sum)[row] = sum;
    }
  }
  char* qr = q + row * (int64_t)chunks * 8;
#pragma unroll
  for (int v = 0; v < V; ++v) {
    const uint32_t ci = t + v * TEAM;
    if (ci < chunks) {
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float y = c[v].get(i) * mul;
        if constexpr (MODE == MODE_INT8) y = __builtin_roundf(y);
        o[i] = clampf(y, lo, hi);
      }
      v2u pk;
      if constexpr (MODE == MODE_INT8) pk = I8Pack::pack(o); else pk = Fp8Pack::pack(o);
      *reinterpret_cast<v2u*>(qr + (int64_t)ci * 8) = pk;
    }
  }
}

// Rows of any length (also not a multiple of 8, or longer than the register
// budget of the kernel above): one block per row, two passes, scalar accesses.
template <int DT, int MODE>
__global__ __launch_bounds__(256) void token_quant_generic_kernel(const char* __restrict__ x,
                                                                  char* __restrict__ q, float* __restrict__ s,
                                                                  void* __restrict__ row_sum, int64_t hidden) {
  __shared__ uint32_t red_max[4];
  __shared__ float red_sum[4];
  const int64_t row = blockIdx.x;
  auto ld = [&](int64_t j) -> float {
    const int64_t idx = row * hidden + j;
    if constexpr (DT == SGLQ_BF16) return u2f((uint32_t)reinterpret_cast<const uint16_t*>(x)[idx] << 16);
    else if constexpr (DT == SGLQ_FP16) return (float)reinterpret_cast<const _Float16*>(x)[idx];
    else return reinterpret_cast<const float*>(x)[idx];
  };
  uint32_t mb = 0;
  float sum = 0.f;
  for (int64_t j = threadIdx.x; j < hidden; j += 256) {
    const float v = ld(j);
    mb = umax(mb, f2u(v) & 0x7fffffffu);
    sum += v;
  }
  mb = wave_umax(mb);
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
  if ((threadIdx.x & 63) == 0) {
    red_max[threadIdx.x >> 6] = mb;
    red_sum[threadIdx.x >> 6] = sum;
  }
  __syncthreads();
  mb = umax(umax(red_max[0], red_max[1]), umax(red_max[2], red_max[3]));
  sum = (red_sum[0] + red_sum[1]) + (red_sum[2] + red_sum[3]);
  float scale, mul, lo, hi;
  if constexpr (MODE == MODE_FP8) {
    scale = u2f(mb) / 448.0f;
    mul = (scale == 0.f) ? 0.f : 1.0f / scale;
    lo = -448.0f;
    hi = 448.0f;
  } else {
    const float amax = u2f(umax(mb, f2u(1e-10f)));
    scale = amax / 127.0f;
    mul = 127.0f / amax;
    lo = -128.0f;
    hi = 127.0f;
  }
  if (threadIdx.x == 0) {
    s[row] = scale;
    if (MODE == MODE_INT8 && row_sum != nullptr) {
      if constexpr (DT == SGLQ_BF16) reinterpret_cast<__bf16*>(row_sum)[row] = (__bf16)sum;
      else if constexpr (DT == SGLQ_FP16) reinterpret_cast<_Float16*>(row_sum)[row] = (_Float16)sum;
      else reinterpret_cast<float*>(row_sum)[row] = sum;
    }
  }
  for (int64_t j = threadIdx.x; j < hidden; j += 256) {
    float y = ld(j) * mul;
    if constexpr (MODE == MODE_INT8) {
      y = clampf(__builtin_roundf(y), lo, hi);
      q[row * hidden + j] = (char)(int)y;
    } else {
      y = clampf(y, lo, hi);
      q[row * hidden + j] = (char)(cvt_pk_e4m3<false>(y, y, 0) & 0xffu);
    }
  }
}

// ---------------------------------------------------------------------------
// Per-tensor FP8 quantization (sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu): one scale
// for the whole tensor.  Dynamic mode runs tensor_absmax_kernel first: every block folds
// its share of the input into one abs-max, divides by 448 and merges it into *s with an
// unsigned integer atomic max on the float's bit pattern (non-negative floats order like
// their bits; *s must be zero on entry, as the reference's caller allocates it).  Both
// modes then run tensor_quant_kernel: q = max(min(x * (1 / *s), 448), -448) -> e4m3fn.
// VEC = false: element-wise accesses, for buffers that are not 16-byte aligned.
// ---------------------------------------------------------------------------
template <int DT>
SGLQ_DEV float load_elem(const char* x, int64_t idx) {
  if constexpr (DT == SGLQ_BF16) return u2f((uint32_t)reinterpret_cast<const uint16_t*>(x)[idx] << 16);
  else if constexpr (DT == SGLQ_FP16) return (float)reinterpret_cast<const _Float16*>(x)[idx];
  else return reinterpret_cast<const float*>(x)[idx];
}

template <int DT, bool VEC>
__global__ __launch_bounds__(256) void tensor_absmax_kernel(const char* __restrict__ x, float* __restrict__ s, int64_t n) {
  __shared__ uint32_t red[4];
  const int64_t nchunks = VEC ? (n >> 3) : 0;
  const int64_t stride = (int64_t)gridDim.x * 256;
  uint32_t mb = 0;
  int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (; c + 3 * stride < nchunks; c += 4 * stride) {  // four independent loads in flight per lane
    Chunk8<DT> ch[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) ch[u].load(x + (c + u * stride) * Chunk8<DT>::kBytes);
#pragma unroll
    for (int u = 0; u < 4; ++u) mb = umax(mb, ch[u].amax_bits());
  }
  for (; c < nchunks; c += stride) {
    Chunk8<DT> ch;
    ch.load(x + c * Chunk8<DT>::kBytes);
    mb = umax(mb, ch.amax_bits());
  }
  for (int64_t j = (nchunks << 3) + (int64_t)blockIdx.x * 256 + threadIdx.x; j < n; j += stride)
    mb = umax(mb, f2u(load_elem<DT>(x, j)) & 0x7fffffffu);
  mb = wave_umax(mb);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mb;
  __syncthreads();
  if (threadIdx.x == 0) {
    mb = umax(umax(red[0], red[1]), umax(red[2], red[3]));
    const uint32_t mine = f2u(u2f(mb) / 448.0f);  // per_tensor_quant_fp8.cu:44
    // Atomics on one address serialise in L2 (about 12 ns each, measured): skip the update when the
    // value already there is not smaller.  It only ever grows, so a stale read costs an atomic, never a result.
    unsigned int* sp = reinterpret_cast<unsigned int*>(s);
    if (mine > __hip_atomic_load(sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(sp, mine);
  }
}

SGLQ_DEV float clamp_like_fminf_fmaxf(float v) {
  // fminf / fmaxf return the non-NaN operand: NaN (0 * inf, all-zero tensor in dynamic mode)
  // becomes +448 as in per_tensor_quant_fp8.cu:70; fmed3 would not do that.
  return __builtin_fmaxf(__builtin_fminf(v, 448.0f), -448.0f);
}

// `repeat` (optional): the scale broadcast to `repeat_n` floats, one per token, which is what
// static_quant_fp8 hands to a GEMM that takes per-token scales (fp8_kernel.py:431-432,458-465).
template <int DT, bool VEC>
__global__ __launch_bounds__(256) void tensor_quant_kernel(const char* __restrict__ x, char* __restrict__ q,
                                                           const float* __restrict__ s, int64_t n,
                                                           float* __restrict__ repeat, int64_t repeat_n) {
  const float scale = *s;
  const float inv = 1.0f / scale;  // per_tensor_quant_fp8.cu:56, fp8_kernel.py:428
  const int64_t nchunks = VEC ? (n >> 3) : 0;
  const int64_t stride = (int64_t)gridDim.x * 256;
  if (repeat)
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < repeat_n; t += stride) repeat[t] = scale;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += stride) {
    Chunk8<DT> ch;
    ch.load(x + c * Chunk8<DT>::kBytes);
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = clamp_like_fminf_fmaxf(ch.get(i) * inv);
    *reinterpret_cast<v2u*>(q + c * 8) = Fp8Pack::pack(v);
  }
  for (int64_t j = (nchunks << 3) + (int64_t)blockIdx.x * 256 + threadIdx.x; j < n; j += stride) {
    const float y = clamp_like_fminf_fmaxf(load_elem<DT>(x, j) * inv);
    q[j] = (char)(cvt_pk_e4m3<false>(y, y, 0) & 0xffu);
  }
}

// ---------------------------------------------------------------------------
// Host-side dispatch
// ---------------------------------------------------------------------------
static int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return SGLQ_ELAUNCH;
  }
  return SGLQ_OK;
}

// Measured on MI355X (8192 x 16384 bf16, graph-timed): two 8-element chunks per lane and
// one group per lane sustains 5.9-6.3 TB/s; one chunk per lane or more groups per lane
// (deeper unrolling) is 2-6 % slower, like a plain 2:1 read/write streaming kernel.
#ifndef SGLQ_GQ_NCH
#define SGLQ_GQ_NCH 2
#endif
#ifndef SGLQ_GQ_UNROLL
#define SGLQ_GQ_UNROLL 1
#endif

template <int DT, int GROUP, bool TO_INT8, bool CLAMP>
static void launch_group_quant(const void* x, void* q, float* s, uint32_t num_groups, uint32_t gpr, bool strided,
                               int64_t sr, int64_t sc, float eps, float qmin, float qmax, hipStream_t st) {
  constexpr int NCH = GROUP >= 16 * SGLQ_GQ_NCH ? SGLQ_GQ_NCH : 1;
  constexpr int GPB = 256 / (GROUP / (8 * NCH));
  FastDiv fd;
  fd.init(gpr);
  const float rq = 1.0f / qmax;
  // more groups per lane once there is enough work to fill the chip several times over
  const bool deep = SGLQ_GQ_UNROLL > 1 && num_groups >= (uint32_t)GPB * SGLQ_GQ_UNROLL * 2048;
  const char* xi = static_cast<const char*>(x);
  char* qo = static_cast<char*>(q);
  // measured on 4096 x 16384 bf16 (128 MiB) right behind a GEMM that wrote 268 MB: 49.3 -> 38.5 us; timed alone
  // 8192 x 16384 70.4 -> 64.3 us, 4096 x 28672 63.3 -> 61.2 us, but 8192 x 7168 (112 MiB) 33.3 -> 33.8 us and
  // 8192 x 1536 (24 MiB) 7.8 -> 9.0 us: hence the threshold
  const bool stream_in = (int64_t)num_groups * GROUP * elem_bytes<DT>() >= ((int64_t)128 << 20);
#define SGLQ_LAUNCH_GQ(U, STR, ONCE)                                                                        \
  group_quant_kernel<DT, GROUP, NCH, U, STR, TO_INT8, CLAMP, ONCE><<<dim3((num_groups + GPB * U - 1) / (GPB * U)), dim3(256), 0, st>>>( \
      xi, qo, s, num_groups, fd, sr, sc, eps, qmin, qmax, rq)
  if (stream_in) {
    if (strided) SGLQ_LAUNCH_GQ(SGLQ_GQ_UNROLL, true, true); else SGLQ_LAUNCH_GQ(SGLQ_GQ_UNROLL, false, true);
  } else if (deep) {
    if (strided) SGLQ_LAUNCH_GQ(SGLQ_GQ_UNROLL, true, false); else SGLQ_LAUNCH_GQ(SGLQ_GQ_UNROLL, false, false);
  } else {
    if (strided) SGLQ_LAUNCH_GQ(1, true, false); else SGLQ_LAUNCH_GQ(1, false, false);
  }
#undef SGLQ_LAUNCH_GQ
}

template <bool TO_INT8>
static int group_quant_entry(const char* name, const void* input, int in_dtype, void* output_q, float* output_s,
                             int64_t num_tokens, int64_t hidden, int group_size, int64_t sr, int64_t sc, float eps,
                             float qmin, float qmax, void* stream) {
  if (!input || !output_q || !output_s) {
    if (num_tokens == 0) return SGLQ_OK;
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (num_tokens < 0 || hidden <= 0 || group_size <= 0 || hidden % group_size != 0) {
    set_error("%s: hidden (%lld) must be a positive multiple of group_size (%d)", name, (long long)hidden, group_size);
    return SGLQ_EINVAL;
  }
  if (!(qmax > 0.f) || !(eps > 0.f)) {
    set_error("%s: eps and the 8-bit maximum must be positive", name);
    return SGLQ_EINVAL;
  }
  if ((reinterpret_cast<uintptr_t>(input) & 15) || (reinterpret_cast<uintptr_t>(output_q) & 7)) {
    set_error("%s: input must be 16-byte and output_q 8-byte aligned", name);
    return SGLQ_EINVAL;
  }
  const int64_t gpr = hidden / group_size;
  const int64_t ng = num_tokens * gpr;
  if (ng == 0) return SGLQ_OK;
  if (ng >= (1ll << 32) - 65536) {
    set_error("%s: too many groups (%lld)", name, (long long)ng);
    return SGLQ_EINVAL;
  }
  const bool strided = !(sc == 1 && sr == gpr);
  const bool standard = !TO_INT8 && qmin == -448.0f && qmax == 448.0f;
  hipStream_t st = static_cast<hipStream_t>(stream);
#define SGLQ_GQ_CASE(DT, G)                                                                                   \
  if (in_dtype == DT && group_size == G) {                                                                    \
    if (standard)                                                                                             \
      launch_group_quant<DT, G, TO_INT8, false>(input, output_q, output_s, (uint32_t)ng, (uint32_t)gpr, strided, sr, \
                                                sc, eps, qmin, qmax, st);                                     \
    else                                                                                                      \
      launch_group_quant<DT, G, TO_INT8, true>(input, output_q, output_s, (uint32_t)ng, (uint32_t)gpr, strided, sr, \
                                               sc, eps, qmin, qmax, st);                                      \
    return check_launch(name);                                                                                \
  }
#define SGLQ_GQ_DT(DT) SGLQ_GQ_CASE(DT, 128) SGLQ_GQ_CASE(DT, 64) SGLQ_GQ_CASE(DT, 32) SGLQ_GQ_CASE(DT, 16) SGLQ_GQ_CASE(DT, 8)
  SGLQ_GQ_DT(SGLQ_BF16)
  SGLQ_GQ_DT(SGLQ_FP16)
  SGLQ_GQ_DT(SGLQ_FP32)
#undef SGLQ_GQ_DT
#undef SGLQ_GQ_CASE
  set_error("%s: unsupported in_dtype %d / group_size %d (group sizes built: 8, 16, 32, 64, 128)", name, in_dtype,
            group_size);
  return SGLQ_EUNSUPPORTED;
}

// sgl_per_token_group_quant_fp8 with power-of-two scales stored as fp32 (group 128): group_quant_kernel<POW2>.
template <int DT>
static void launch_group_quant_pow2(const void* x, void* q, float* s, uint32_t num_groups, uint32_t gpr, bool strided, int64_t sr,
                                    int64_t sc, float eps, float qmin, float qmax, hipStream_t st) {
  constexpr int GROUP = 128, NCH = 2, GPB = 256 / (GROUP / (8 * NCH));
  FastDiv fd;
  fd.init(gpr);
  const float rq = 1.0f / qmax;
  const char* xi = static_cast<const char*>(x);
  char* qo = static_cast<char*>(q);
  const bool stream_in = (int64_t)num_groups * GROUP * elem_bytes<DT>() >= ((int64_t)128 << 20);  // (as launch_group_quant)
  const dim3 grid((num_groups + GPB - 1) / GPB), block(256);
#define SGLQ_LAUNCH_P2(STR, ONCE) \
  group_quant_kernel<DT, GROUP, NCH, 1, STR, false, false, ONCE, true><<<grid, block, 0, st>>>(xi, qo, s, num_groups, fd, sr, sc, eps, qmin, qmax, rq)
  if (stream_in) {
    if (strided) SGLQ_LAUNCH_P2(true, true); else SGLQ_LAUNCH_P2(false, true);
  } else {
    if (strided) SGLQ_LAUNCH_P2(true, false); else SGLQ_LAUNCH_P2(false, false);
  }
#undef SGLQ_LAUNCH_P2
}

static int group_quant_pow2_entry(const void* input, int in_dtype, void* output_q, float* output_s, int64_t num_tokens,
                                  int64_t hidden, int64_t sr, int64_t sc, float eps, float qmin, float qmax, void* stream) {
  const char* name = "sgl_per_token_group_quant_fp8 (power-of-two fp32 scales)";
  if (!input || !output_q || !output_s) {
    if (num_tokens == 0) return SGLQ_OK;
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (num_tokens < 0 || hidden <= 0 || hidden % 128 != 0) {
    set_error("%s: hidden (%lld) must be a positive multiple of 128", name, (long long)hidden);
    return SGLQ_EINVAL;
  }
  if (!(qmax > 0.f) || !(eps > 0.f)) {
    set_error("%s: eps and the 8-bit maximum must be positive", name);
    return SGLQ_EINVAL;
  }
  if ((reinterpret_cast<uintptr_t>(input) & 15) || (reinterpret_cast<uintptr_t>(output_q) & 7)) {
    set_error("%s: input must be 16-byte and output_q 8-byte aligned", name);
    return SGLQ_EINVAL;
  }
  const int64_t gpr = hidden / 128;
  const int64_t ng = num_tokens * gpr;
  if (ng == 0) return SGLQ_OK;
  if (ng >= (1ll << 32) - 65536) {
    set_error("%s: too many groups (%lld)", name, (long long)ng);
    return SGLQ_EINVAL;
  }
  const bool strided = !(sc == 1 && sr == gpr);
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (in_dtype) {
    case SGLQ_BF16: launch_group_quant_pow2<SGLQ_BF16>(input, output_q, output_s, (uint32_t)ng, (uint32_t)gpr, strided, sr, sc, eps, qmin, qmax, st); break;
    case SGLQ_FP16: launch_group_quant_pow2<SGLQ_FP16>(input, output_q, output_s, (uint32_t)ng, (uint32_t)gpr, strided, sr, sc, eps, qmin, qmax, st); break;
    case SGLQ_FP32: launch_group_quant_pow2<SGLQ_FP32>(input, output_q, output_s, (uint32_t)ng, (uint32_t)gpr, strided, sr, sc, eps, qmin, qmax, st); break;
    default:
      set_error("%s: unsupported in_dtype %d", name, in_dtype);
      return SGLQ_EUNSUPPORTED;
  }
  return check_launch(name);
}

static int group_quant_ue8m0_entry(const void* input, int in_dtype, void* output_q, void* output_s, int64_t num_tokens,
                                   int64_t hidden, int64_t s_stride_col, float eps, float qmin, float qmax, void* stream) {
  const char* name = "sgl_per_token_group_quant_fp8 (scale_ue8m0)";
  if (!input || !output_q || !output_s) {
    if (num_tokens == 0) return SGLQ_OK;
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (num_tokens < 0 || hidden <= 0 || hidden % 128 != 0) {
    set_error("%s: hidden (%lld) must be a positive multiple of 128", name, (long long)hidden);
    return SGLQ_EINVAL;
  }
  if (!(qmax > 0.f) || !(eps > 0.f) || s_stride_col < num_tokens) {
    set_error("%s: eps and the 8-bit maximum must be positive, the scale column stride at least num_tokens", name);
    return SGLQ_EINVAL;
  }
  if ((reinterpret_cast<uintptr_t>(input) & 15) || (reinterpret_cast<uintptr_t>(output_q) & 7) ||
      (reinterpret_cast<uintptr_t>(output_s) & 3)) {
    set_error("%s: input must be 16-byte, output_q 8-byte and output_s 4-byte aligned", name);
    return SGLQ_EINVAL;
  }
  const int64_t gpr = hidden / 128, ng = num_tokens * gpr;
  if (ng == 0) return SGLQ_OK;
  if (ng >= (1ll << 32) - 65536) {
    set_error("%s: too many groups (%lld)", name, (long long)ng);
    return SGLQ_EINVAL;
  }
  FastDiv fd;
  fd.init((uint32_t)gpr);
  const dim3 grid((uint32_t)((ng + 15) / 16)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const char* xi = static_cast<const char*>(input);
  char* qo = static_cast<char*>(output_q);
  unsigned char* so = static_cast<unsigned char*>(output_s);
  const float rq = 1.0f / qmax;
  switch (in_dtype) {
    case SGLQ_BF16: group_quant_ue8m0_kernel<SGLQ_BF16><<<grid, block, 0, st>>>(xi, qo, so, (uint32_t)ng, fd, s_stride_col, eps, qmin, qmax, rq); break;
    case SGLQ_FP16: group_quant_ue8m0_kernel<SGLQ_FP16><<<grid, block, 0, st>>>(xi, qo, so, (uint32_t)ng, fd, s_stride_col, eps, qmin, qmax, rq); break;
    case SGLQ_FP32: group_quant_ue8m0_kernel<SGLQ_FP32><<<grid, block, 0, st>>>(xi, qo, so, (uint32_t)ng, fd, s_stride_col, eps, qmin, qmax, rq); break;
    default:
      set_error("%s: input dtype must be bf16, fp16 or fp32", name);
      return SGLQ_EUNSUPPORTED;
  }
  return check_launch(name);
}

template <int DT, int MODE>
static int launch_token_quant(const char* name, const void* x, void* q, float* s, void* row_sum, int64_t rows,
                              int64_t hidden, hipStream_t st) {
  const char* xi = static_cast<const char*>(x);
  char* qo = static_cast<char*>(q);
  const int64_t chunks = hidden / 8;
  if (hidden % 8 != 0 || chunks > 256 * 8) {
    token_quant_generic_kernel<DT, MODE><<<dim3((uint32_t)rows), dim3(256), 0, st>>>(xi, qo, s, row_sum, hidden);
    return check_launch(name);
  }
#define SGLQ_TQ(TEAM, V)                                                                                         \
  token_quant_kernel<DT, TEAM, V, MODE><<<dim3((uint32_t)((rows + (256 / TEAM) - 1) / (256 / TEAM))), dim3(256), 0, st>>>( \
      xi, qo, s, row_sum, rows, (uint32_t)chunks)
  if (chunks <= 64) SGLQ_TQ(64, 1);
  else if (chunks <= 128) SGLQ_TQ(64, 2);
  else if (chunks <= 256) SGLQ_TQ(64, 4);
  else if (chunks <= 512) SGLQ_TQ(256, 2);
  else if (chunks <= 1024) SGLQ_TQ(256, 4);
  else SGLQ_TQ(256, 8);
#undef SGLQ_TQ
  return check_launch(name);
}

template <int MODE>
static int token_quant_entry(const char* name, const void* input, int in_dtype, void* output_q, float* output_s,
                             void* row_sum, int64_t num_tokens, int64_t hidden, void* stream) {
  if (num_tokens == 0) return SGLQ_OK;
  if (!input || !output_q || !output_s) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (num_tokens < 0 || hidden <= 0 || num_tokens >= (1ll << 31)) {
    set_error("%s: bad shape [%lld, %lld]", name, (long long)num_tokens, (long long)hidden);
    return SGLQ_EINVAL;
  }
  if (MODE == MODE_FP8 && hidden % 8 != 0) {
    set_error("%s: Hidden dimension must be divisible by 8, but got %lld", name, (long long)hidden);
    return SGLQ_EINVAL;
  }
  if (hidden % 8 == 0 &&
      ((reinterpret_cast<uintptr_t>(input) & 15) || (reinterpret_cast<uintptr_t>(output_q) & 7))) {
    set_error("%s: input must be 16-byte and output_q 8-byte aligned", name);
    return SGLQ_EINVAL;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (in_dtype) {
    case SGLQ_BF16: return launch_token_quant<SGLQ_BF16, MODE>(name, input, output_q, output_s, row_sum, num_tokens, hidden, st);
    case SGLQ_FP16: return launch_token_quant<SGLQ_FP16, MODE>(name, input, output_q, output_s, row_sum, num_tokens, hidden, st);
    case SGLQ_FP32: return launch_token_quant<SGLQ_FP32, MODE>(name, input, output_q, output_s, row_sum, num_tokens, hidden, st);
  }
  set_error("%s: unsupported in_dtype %d", name, in_dtype);
  return SGLQ_EUNSUPPORTED;
}

template <int DT>
static void launch_tensor_quant(const void* x, void* q, float* s, int64_t n, bool is_static, hipStream_t st,
                                float* repeat = nullptr, int64_t repeat_n = 0) {
  const bool vec = ((reinterpret_cast<uintptr_t>(x) & 15) == 0) && ((reinterpret_cast<uintptr_t>(q) & 7) == 0);
  const int64_t work = vec ? (n + 7) / 8 : n;
  int64_t blocks = (work + 255) / 256;
  if (blocks > 4096) blocks = 4096;  // grid-stride beyond that: 16 blocks per CU
  if (blocks < 1) blocks = 1;
  int64_t max_blocks = (work + 1023) / 1024;  // the abs-max pass: four chunks per lane and trip, one atomic per block
  if (max_blocks > 1024) max_blocks = 1024;
  if (max_blocks < 1) max_blocks = 1;
  const dim3 grid((uint32_t)blocks), grid_max((uint32_t)max_blocks), block(256);
  const char* xc = static_cast<const char*>(x);
  char* qc = static_cast<char*>(q);
  if (vec) {
    if (!is_static) tensor_absmax_kernel<DT, true><<<grid_max, block, 0, st>>>(xc, s, n);
    tensor_quant_kernel<DT, true><<<grid, block, 0, st>>>(xc, qc, s, n, repeat, repeat_n);
  } else {
    if (!is_static) tensor_absmax_kernel<DT, false><<<grid_max, block, 0, st>>>(xc, s, n);
    tensor_quant_kernel<DT, false><<<grid, block, 0, st>>>(xc, qc, s, n, repeat, repeat_n);
  }
}

static int tensor_quant_entry(const void* input, int in_dtype, void* output_q, float* output_s, int64_t num_elements,
                              int is_static, void* stream) {
  const char* name = "sgl_per_tensor_quant_fp8";
  if (num_elements < 0) {
    set_error("%s: negative element count", name);
    return SGLQ_EINVAL;
  }
  if (!output_s) {
    set_error("%s: null scale pointer", name);
    return SGLQ_EINVAL;
  }
  if (num_elements > 0 && (!input || !output_q)) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (num_elements == 0) return SGLQ_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (in_dtype) {
    case SGLQ_BF16: launch_tensor_quant<SGLQ_BF16>(input, output_q, output_s, num_elements, is_static != 0, st); break;
    case SGLQ_FP16: launch_tensor_quant<SGLQ_FP16>(input, output_q, output_s, num_elements, is_static != 0, st); break;
    case SGLQ_FP32: launch_tensor_quant<SGLQ_FP32>(input, output_q, output_s, num_elements, is_static != 0, st); break;
    default:
      set_error("%s: input dtype must be bf16, fp16 or fp32", name);
      return SGLQ_EUNSUPPORTED;
  }
  return check_launch(name);
}

static int static_quant_entry(const void* input, int in_dtype, void* output_q, const float* scale, float* scale_repeat,
                              int64_t num_tokens, int64_t hidden, void* stream) {
  const char* name = "static_quant_fp8";
  if (num_tokens < 0 || hidden < 0) {
    set_error("%s: negative shape", name);
    return SGLQ_EINVAL;
  }
  if (!scale) {
    set_error("%s: null scale pointer", name);
    return SGLQ_EINVAL;
  }
  const int64_t n = num_tokens * hidden;
  if (n > 0 && (!input || !output_q)) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (n == 0 && !(scale_repeat && num_tokens > 0)) return SGLQ_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* s = const_cast<float*>(scale);  // static mode only reads it
  switch (in_dtype) {
    case SGLQ_BF16: launch_tensor_quant<SGLQ_BF16>(input, output_q, s, n, true, st, scale_repeat, num_tokens); break;
    case SGLQ_FP16: launch_tensor_quant<SGLQ_FP16>(input, output_q, s, n, true, st, scale_repeat, num_tokens); break;
    case SGLQ_FP32: launch_tensor_quant<SGLQ_FP32>(input, output_q, s, n, true, st, scale_repeat, num_tokens); break;
    default:
      set_error("%s: input dtype must be bf16, fp16 or fp32", name);
      return SGLQ_EUNSUPPORTED;
  }
  return check_launch(name);
}

}  // namespace sglq

extern "C" int sglq_per_token_group_quant_fp8_scatter(const void* input, int in_dtype, void* output_q, float* output_s,
                                                      const int32_t* slot_map, int64_t num_tokens, int64_t hidden,
                                                      int64_t topk, int64_t num_dst_rows, float eps, void* stream) {
  using namespace sglq;
  const char* name = "per_token_group_quant_fp8_scatter";
  if (num_tokens < 0 || hidden <= 0 || hidden % 128 != 0 || topk <= 0 || topk >= (1 << 20) || num_dst_rows < 0) {
    set_error("%s: hidden (%lld) must be a positive multiple of 128, topk positive", name, (long long)hidden);
    return SGLQ_EINVAL;
  }
  if (num_tokens == 0 || num_dst_rows == 0) return SGLQ_OK;
  if (!input || !output_q || !output_s || !slot_map) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (!(eps > 0.f)) {
    set_error("%s: eps must be positive", name);
    return SGLQ_EINVAL;
  }
  if ((reinterpret_cast<uintptr_t>(input) & 15) || (reinterpret_cast<uintptr_t>(output_q) & 7)) {
    set_error("%s: input must be 16-byte and output_q 8-byte aligned", name);
    return SGLQ_EINVAL;
  }
  const int64_t gpr = hidden / 128, ng = num_tokens * gpr;
  if (ng >= (1ll << 32) - 65536) {
    set_error("%s: too many groups (%lld)", name, (long long)ng);
    return SGLQ_EINVAL;
  }
  FastDiv fd;
  fd.init((uint32_t)gpr);
  const float qmax = 448.0f;
  const dim3 grid((uint32_t)((ng + 31) / 32)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const char* xi = static_cast<const char*>(input);
  char* qo = static_cast<char*>(output_q);
#define SGLQ_SCATTER(DT)                                                                                               \
  group_quant_scatter_kernel<DT><<<grid, block, 0, st>>>(xi, qo, output_s, slot_map, (uint32_t)ng, fd, (int)topk, num_dst_rows, \
                                                         eps, qmax, 1.0f / qmax)
  if (in_dtype == SGLQ_BF16) SGLQ_SCATTER(SGLQ_BF16);
  else if (in_dtype == SGLQ_FP16) SGLQ_SCATTER(SGLQ_FP16);
  else if (in_dtype == SGLQ_FP32) SGLQ_SCATTER(SGLQ_FP32);
  else {
    set_error("%s: unsupported in_dtype %d", name, in_dtype);
    return SGLQ_EUNSUPPORTED;
  }
#undef SGLQ_SCATTER
  return check_launch(name);
}

extern "C" int sglq_silu_and_mul_group_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                                                 int64_t num_tokens, int64_t d, float eps, void* stream) {
  using namespace sglq;
  const char* name = "silu_and_mul_group_quant_fp8";
  if (num_tokens < 0 || d <= 0 || d % 128 != 0) {
    set_error("%s: d (%lld) must be a positive multiple of 128", name, (long long)d);
    return SGLQ_EINVAL;
  }
  if (num_tokens == 0) return SGLQ_OK;
  if (!input || !output_q || !output_s) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (!(eps > 0.f)) {
    set_error("%s: eps must be positive", name);
    return SGLQ_EINVAL;
  }
  if ((reinterpret_cast<uintptr_t>(input) & 15) || (reinterpret_cast<uintptr_t>(output_q) & 7)) {
    set_error("%s: input must be 16-byte and output_q 8-byte aligned", name);
    return SGLQ_EINVAL;
  }
  const int64_t gpr = d / 128, ng = num_tokens * gpr;
  if (ng >= (1ll << 32) - 65536) {
    set_error("%s: too many groups (%lld)", name, (long long)ng);
    return SGLQ_EINVAL;
  }
  FastDiv fd;
  fd.init((uint32_t)gpr);
  const float qmax = 448.0f;
  const dim3 grid((uint32_t)((ng + 31) / 32)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const char* xi = static_cast<const char*>(input);
  char* qo = static_cast<char*>(output_q);
  if (in_dtype == SGLQ_BF16) silu_mul_group_quant_kernel<SGLQ_BF16><<<grid, block, 0, st>>>(xi, qo, output_s, (uint32_t)ng, fd, eps, qmax, 1.0f / qmax);
  else if (in_dtype == SGLQ_FP16) silu_mul_group_quant_kernel<SGLQ_FP16><<<grid, block, 0, st>>>(xi, qo, output_s, (uint32_t)ng, fd, eps, qmax, 1.0f / qmax);
  else {
    set_error("%s: dtype must be Half or BFloat16", name);
    return SGLQ_EUNSUPPORTED;
  }
  return check_launch(name);
}

extern "C" int sglq_static_quant_fp8(const void* input, int in_dtype, void* output_q, const float* scale,
                                     float* scale_repeat, int64_t num_tokens, int64_t hidden, void* stream) {
  return sglq::static_quant_entry(input, in_dtype, output_q, scale, scale_repeat, num_tokens, hidden, stream);
}

extern "C" int sglq_per_token_group_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                                              int64_t num_tokens, int64_t hidden, int group_size,
                                              int64_t s_stride_row, int64_t s_stride_col, float eps, float fp8_min,
                                              float fp8_max, void* stream) {
  return sglq::group_quant_entry<false>("sgl_per_token_group_quant_fp8", input, in_dtype, output_q, output_s,
                                        num_tokens, hidden, group_size, s_stride_row, s_stride_col, eps, fp8_min,
                                        fp8_max, stream);
}

extern "C" int sglq_per_token_group_quant_fp8_ue8m0(const void* input, int in_dtype, void* output_q, void* output_s,
                                                    int64_t num_tokens, int64_t hidden, int64_t s_stride_col, float eps,
                                                    float fp8_min, float fp8_max, void* stream) {
  return sglq::group_quant_ue8m0_entry(input, in_dtype, output_q, output_s, num_tokens, hidden, s_stride_col, eps, fp8_min,
                                       fp8_max, stream);
}

extern "C" int sglq_per_token_group_quant_fp8_pow2(const void* input, int in_dtype, void* output_q, float* output_s,
                                                   int64_t num_tokens, int64_t hidden, int64_t s_stride_row, int64_t s_stride_col,
                                                   float eps, float fp8_min, float fp8_max, void* stream) {
  return sglq::group_quant_pow2_entry(input, in_dtype, output_q, output_s, num_tokens, hidden, s_stride_row, s_stride_col, eps,
                                      fp8_min, fp8_max, stream);
}

extern "C" int sglq_per_token_group_quant_int8(const void* input, int in_dtype, void* output_q, float* output_s,
                                               int64_t num_tokens, int64_t hidden, int group_size,
                                               int64_t s_stride_row, int64_t s_stride_col, float eps, float int8_min,
                                               float int8_max, void* stream) {
  return sglq::group_quant_entry<true>("sgl_per_token_group_quant_int8", input, in_dtype, output_q, output_s,
                                       num_tokens, hidden, group_size, s_stride_row, s_stride_col, eps, int8_min,
                                       int8_max, stream);
}

extern "C" int sglq_per_token_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                                        int64_t num_tokens, int64_t hidden, void* stream) {
  return sglq::token_quant_entry<sglq::MODE_FP8>("sgl_per_token_quant_fp8", input, in_dtype, output_q, output_s,
                                                 nullptr, num_tokens, hidden, stream);
}

extern "C" int sglq_per_token_quant_int8(const void* input, int in_dtype, void* output_q, float* output_s,
                                         void* row_sum, int64_t num_tokens, int64_t hidden, void* stream) {
  return sglq::token_quant_entry<sglq::MODE_INT8>("per_token_quant_int8", input, in_dtype, output_q, output_s,
                                                  row_sum, num_tokens, hidden, stream);
}

extern "C" int sglq_per_tensor_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                                         int64_t num_elements, int is_static, void* stream) {
  return sglq::tensor_quant_entry(input, in_dtype, output_q, output_s, num_elements, is_static, stream);
}
