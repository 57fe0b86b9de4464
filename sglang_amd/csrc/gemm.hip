// W8A8 GEMM kernels for gfx950 (CDNA4): C[M,N] = A[M,K] * B[K,N] with A row-major
// and B column-major, i.e. both operands K-contiguous ("NT").  One template serves
//   * block-scaled FP8   (per-token-group activation scales x 128x128 weight scales),
//   * per-row/per-column scaled FP8, and
//   * per-row/per-column scaled INT8 (exact INT32 accumulators),
// on v_mfma_f32_16x16x128_f8f6f4 / v_mfma_i32_16x16x64_i8.
//
// Layout of the computation.  The MFMA "row" operand is a 16x128-byte slab of the
// weight (16 values of n), the "column" operand a 16x128-byte slab of the
// activations (16 values of m), so lane l of a 16x16 result holds
//     C[m = l % 16][n = 4 * (l / 16) + j],  j = 0..3
// i.e. four consecutive n for one m: the per-token scale is one register per lane
// and the epilogue stores 8-byte runs.
//
// Tiles of BM x 128 B (activations) and BN x 128 B (weights) are staged in LDS,
// double buffered.  A row holds eight 16-byte chunks; chunk c of row r is stored
// at chunk position c ^ swz(r), swz(r) = (r & 7) ^ ((r >> 3) & 1), which makes the
// 16-byte MFMA operand reads of any 8 or 16 consecutive lanes hit distinct banks.
// Global -> LDS copies use buffer loads that write LDS directly (each wavefront
// instruction fills 1 KiB = 8 rows); rows past M/N and chunks past K read as zero
// through the buffer range check.
#include <atomic>
#include <mutex>
#include <shared_mutex>
#include <type_traits>

#include "quant_device.h"
#include "sglq_common.h"

namespace sglq {

constexpr int KIND_FP8_BLOCK = 0;   // a4: sum_kb P_kb * sfa[m,kb] * sfb[kb,n/128]
constexpr int KIND_FP8_ROWCOL = 1;  // a6: sa[m] * (sb[n] * acc) + bias[n]
constexpr int KIND_I8_ROWCOL = 2;   // a5: float(acc) * (sb[n] * sa[m]) + bias[n]
constexpr int KIND_I8_RAW = 3;      // INT32 accumulators
constexpr int KIND_I8_BLOCK = 4;    // block-scaled INT8: sum_kb float(P_kb) * sfa[m,kb] * sfb[kb,n/128]
// KIND_FP8_BLOCK whose scales are all powers of two (UE8M0 values held as fp32): the MFMA applies them itself
// (v_mfma_scale_f32_16x16x128_f8f6f4 takes an exponent byte per lane for each operand) and accumulates in place,
// so there is no scale-and-accumulate pass behind every MFMA.  Only the 256- and 128-row pipelined kernels are
// built for it; everywhere else such scales run as KIND_FP8_BLOCK (the same sums folded per K block: equal to the
// in-place accumulation up to the order of the additions, not bit for bit).
constexpr int KIND_FP8_BLOCK_POW2 = 5;

constexpr bool is_block(int kind) { return kind == KIND_FP8_BLOCK || kind == KIND_I8_BLOCK || kind == KIND_FP8_BLOCK_POW2; }
constexpr bool fp8_operands(int kind) { return kind == KIND_FP8_BLOCK || kind == KIND_FP8_ROWCOL || kind == KIND_FP8_BLOCK_POW2; }
// the biased exponent of a positive power of two = its UE8M0 code, in byte 0 as the scaled MFMA reads it
SGLQ_DEV int ue8m0_of(float pow2) { return (int)(__builtin_bit_cast(uint32_t, pow2) >> 23); }
// ... of an activation scale as the kernels hold it: the eight bits from `shift` on, 23 for an fp32 power of two, 8 (kb % 4)
// for a word of four UE8M0 codes (GemmArgs::sa_packed) and K block kb
SGLQ_DEV int ue8m0_at(float word, int shift) { return (int)((__builtin_bit_cast(uint32_t, word) >> shift) & 0xffu); }
constexpr bool float_acc(int kind) { return fp8_operands(kind) || kind == KIND_I8_BLOCK; }

constexpr uint32_t OOB = 0x80000000u;  // offset beyond any buffer this library accepts
constexpr uint32_t SC_NONE = 0x40000000u;  // scalar offset beyond any scale tensor (at most 2^31 / 32 bytes)

struct GemmArgs {
  const char* a;   // [M, K] bytes, row stride lda
  const char* b;   // [N, K] bytes, row stride ldb (column-major [K, N])
  const float* sa; // block: sfa; rowcol: scales_a [M]
  const float* sb; // block: sfb; rowcol: scales_b [N]
  const void* bias;
  void* out;
  int64_t sa_stride_m, sa_stride_k;  // block scales
  int64_t sb_stride_k, sb_stride_n;
  int64_t ldo;
  uint32_t lda, ldb;
  uint32_t a_bytes, b_bytes;
  int M, N, K;
  int tiles_m, tiles_n;
  void* ws;        // split-K partial sums [splits][M][N], fp32 or int32; grouped GEMM: the tile plan
  int splits;
  int64_t b_expert_stride, sb_expert_stride;  // grouped GEMM: bytes / floats between experts' weights / weight scales
  int num_experts;
  int stream_out;  // the output is larger than the last-level cache: store it with the non-temporal hint
  int pow2_scales;  // block-scaled FP8: every scale is a power of two (KIND_FP8_BLOCK_POW2 where it is built)
  // ... and the activation scales come as UE8M0 codes, four K blocks to an int32 word: word (m, kb / 4) sits at
  // sa[m * sa_stride_m + (kb / 4) * sa_stride_k], byte kb % 4 of it is K block kb's code (what
  // sglq_per_token_group_quant_fp8_ue8m0 writes).  Read as they are by the KIND_FP8_BLOCK_POW2 kernels; every
  // other kernel gets them expanded to fp32 first (expand_packed_scales).
  int sa_packed;
  float* sa_expanded;  // room for [M, K / 128] fp32 scales (sa_packed only)
  float quant_eps;  // fused quantization (gemm_stream_quant_kernel): lower bound of a group's abs-max
};

// Grouped GEMM tile plan in the workspace (int32): [0] = number of row tiles, then from [4] on
// one entry of four per row tile: expert, first row, end row (both absolute rows of A and C).
constexpr int PLAN_HEADER = 4, PLAN_ENTRY = 4;

// s_waitcnt immediate: wait until at most `vm` vector-memory loads are outstanding
// and all LDS / scalar-memory operations are done (vmcnt is split over bits 3:0 and 15:14).
constexpr int waitcnt_vm_lgkm0(int vm) { return (vm & 0xf) | (((vm >> 4) & 3) << 14) | (7 << 4); }
// ... and one that waits for LDS / scalar-memory operations only
// Tile rows per band of the tile walk (tile_of_block).  Measured with the profiler's FETCH_SIZE counter (bytes
// that miss the XCDs' L2s) on the 256-row kernels at M = 4096: bands of 4 rows fetch 6 % less than bands of 8
// on 7168 x 16384 (224-wide tiles) and 20 % less on 2112 x 7168 (192-wide tiles), the same on 24576 x 1536 and
// 4096 x 7168 (with 32 tiles in flight per XCD, 4 x 8 and 8 x 4 touch the same number of rows when the tile is
// square); bands of 16 fetch 40-70 % more.  Launch times move by less than 2 % between 4 and 8 and by +2-3 %
// with 16: these kernels are not bound by that traffic.
#ifndef SGLQ_GROUP_M
#define SGLQ_GROUP_M 4
#endif
#ifndef SGLQ_STREAM_NSTAGE
#define SGLQ_STREAM_NSTAGE 3
#endif
constexpr int waitcnt_lgkm0_only() { return 0xf | (3 << 14) | (7 << 4); }

// Global -> LDS copies written as assembly (16 or 4 bytes per lane; lane l lands at
// lds_dst + l * size).  The decode kernel keeps several stages of such copies in flight and
// waits for them with explicit vmcnt counts; copies issued through the compiler's builtin
// are tracked by its wait-count pass, which cannot tell the ring's stages apart and would
// drain every copy in flight before each LDS read.
SGLQ_DEV v4u make_rsrc_sgpr(const void* ptr, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(ptr);
  return v4u{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
             (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu)),
             (uint32_t)__builtin_amdgcn_readfirstlane((int)bytes), 0x00020000u};
}
SGLQ_DEV void lds_copy16(v4u rsrc, uint32_t lds_dst, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" : : "s"(lds_dst), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
SGLQ_DEV void lds_copy4(v4u rsrc, uint32_t lds_dst, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, %3 offen lds" : : "s"(lds_dst), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
SGLQ_DEV uint32_t lds_addr(const void* p) {
  return (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const char*)p);
}

SGLQ_DEV int swz(int r) { return (r & 7) ^ ((r >> 3) & 1); }

// One 128-byte K block of a block-scaled kind: the product of a weight and an activation
// fragment from a zero accumulator.  FP8: one MFMA, fp32 result.  INT8: two MFMAs, exact
// int32 result, returned as its bit pattern so that the conversion to float can wait until
// the result is folded into the accumulator (block_value) instead of stalling on the MFMA.
template <int KIND>
SGLQ_DEV v4f block_mfma(const v8i& w, const v8i& a) {
  if constexpr (KIND == KIND_I8_BLOCK) {
    const v4i w0 = {w[0], w[1], w[2], w[3]}, w1 = {w[4], w[5], w[6], w[7]};
    const v4i a0 = {a[0], a[1], a[2], a[3]}, a1 = {a[4], a[5], a[6], a[7]};
    v4i t = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, a0, v4i{0, 0, 0, 0}, 0, 0, 0);
    t = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, a1, t, 0, 0, 0);
    return __builtin_bit_cast(v4f, t);
  } else {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, a, v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
  }
}
template <int KIND>
SGLQ_DEV float block_value(float raw) {
  if constexpr (KIND == KIND_I8_BLOCK) return (float)__builtin_bit_cast(int, raw);
  else return raw;
}

template <int OUT_DT>
SGLQ_DEV void store4(void* out, int64_t idx, float v0, float v1, float v2, float v3) {
  if constexpr (OUT_DT == SGLQ_BF16) {
    typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
    bf4 o = {(__bf16)v0, (__bf16)v1, (__bf16)v2, (__bf16)v3};
    *reinterpret_cast<bf4*>(reinterpret_cast<__bf16*>(out) + idx) = o;
  } else {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    h4 o = {(_Float16)v0, (_Float16)v1, (_Float16)v2, (_Float16)v3};
    *reinterpret_cast<h4*>(reinterpret_cast<_Float16*>(out) + idx) = o;
  }
}

// fp32 -> output type -> fp32
template <int OUT_DT>
SGLQ_DEV float round_out(float v) {
  if constexpr (OUT_DT == SGLQ_BF16) return (float)(__bf16)v;
  else return (float)(_Float16)v;
}

template <int OUT_DT>
SGLQ_DEV void load_bias4(const void* bias, int n, float (&b)[4]) {
  if constexpr (OUT_DT == SGLQ_BF16) {
    const uint16_t* p = reinterpret_cast<const uint16_t*>(bias) + n;
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = u2f((uint32_t)p[j] << 16);
  } else {
    const _Float16* p = reinterpret_cast<const _Float16*>(bias) + n;
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = (float)p[j];
  }
}

// Map the linear block id to an output tile: consecutive ids are dealt round-robin
// to the 8 XCDs by the dispatcher, so give every XCD one contiguous range of tiles
// (its L2 then sees a compact set of A rows and B columns), and walk each range in
// bands of GROUP_M tile-rows.
SGLQ_DEV void tile_of_block(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  const int q = total >> 3, rem = total & 7;
  const int xcd = pid & 7, idx = pid >> 3;
  int tile = xcd * q + (xcd < rem ? xcd : rem) + idx;
  constexpr int GROUP_M = SGLQ_GROUP_M;
  const int width = GROUP_M * tiles_n;
  const int group = tile / width;
  const int first_m = group * GROUP_M;
  const int gsz = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_group = tile - group * width;
  tm = first_m + in_group % gsz;
  tn = in_group / gsz;
}

// Scale, add bias and store four consecutive outputs C[m][n..n+3] from their accumulators.
// BLOCK_BIAS (block-scaled kinds only): 1 / 0 = the caller knows at compile time that there
// is / is not a bias, -1 = look at p.bias.
template <int KIND, int OUT_DT, int BLOCK_BIAS = -1, typename acc_t>
SGLQ_DEV void finish4(const GemmArgs& p, int m, int n, const acc_t& a, float sam) {
  const int64_t idx = (int64_t)m * p.ldo + n;
  if constexpr (KIND == KIND_I8_RAW) {
    *reinterpret_cast<v4i*>(reinterpret_cast<int32_t*>(p.out) + idx) = a;
  } else if constexpr (is_block(KIND)) {
    if (BLOCK_BIAS == 1 || (BLOCK_BIAS == -1 && p.bias)) {
      // the caller's `output += bias` on the rounded GEMM result (fp8_utils.py:210-211), fused:
      // round to the output type, add the bias in fp32, round again
      float bv[4], o[4];
      load_bias4<OUT_DT>(p.bias, n, bv);
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = round_out<OUT_DT>(a[e]) + bv[e];
      store4<OUT_DT>(p.out, idx, o[0], o[1], o[2], o[3]);
    } else {
      store4<OUT_DT>(p.out, idx, a[0], a[1], a[2], a[3]);
    }
  } else {
    float o[4], bv[4] = {0.f, 0.f, 0.f, 0.f};
    const v4f sbn = *reinterpret_cast<const v4f*>(p.sb + n);
    if (p.bias) load_bias4<OUT_DT>(p.bias, n, bv);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if constexpr (KIND == KIND_I8_ROWCOL) o[e] = __builtin_fmaf((float)a[e], sbn[e] * sam, bv[e]);
      else o[e] = __builtin_fmaf(sam, sbn[e] * a[e], bv[e]);
    }
    store4<OUT_DT>(p.out, idx, o[0], o[1], o[2], o[3]);
  }
}

// Split-K: store a wave's raw accumulators as partial sums of split `split` in the
// workspace, laid out [split][M][N] (fp32 or int32); splitk_reduce_kernel finishes them.
template <int MI, int NI, typename acc_t>
SGLQ_DEV void store_partials(const GemmArgs& p, acc_t (&acc)[MI][NI], int split, int m_base, int n_base, int r16, int g) {
  asm volatile("" : "+v"(r16), "+v"(g));  // keep the address arithmetic here (see epilogue_via_lds)
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = m_base + i * 16 + r16;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int n = n_base + j * 16 + g * 4;
      if (n >= p.N) continue;
      acc_t* dst = reinterpret_cast<acc_t*>(reinterpret_cast<char*>(p.ws) + (((int64_t)split * p.M + m) * p.N + n) * 4);
      *dst = acc[i][j];
    }
  }
}

// The same for the 256-row kernels, as buffer stores that need neither branches nor 64-bit
// addresses: a row beyond M lies beyond the split's extent and is dropped by the bounds
// check, a column beyond N gets an offset that is.  The host keeps (M + 256) N 4 below 2 GiB.
template <int MI, int NI, typename acc_t>
SGLQ_DEV void store_partials_bounded(const GemmArgs& p, acc_t (&acc)[MI][NI], int split, int m_base, int n_base, int r16, int g) {
  asm volatile("" : "+v"(r16), "+v"(g));  // keep the address arithmetic here (see epilogue_via_lds)
  const uint32_t row_bytes = (uint32_t)p.N * 4u, split_bytes = (uint32_t)p.M * row_bytes;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(reinterpret_cast<char*>(p.ws) + (int64_t)split * split_bytes, split_bytes);
  const int n_lane = n_base + g * 4;
  const uint32_t off = (uint32_t)(m_base + r16) * row_bytes + (uint32_t)n_lane * 4u;
#pragma unroll
  for (int i = 0; i < MI; ++i) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const uint32_t voff = (n_lane + j * 16 < p.N) ? off + (uint32_t)(i * 16) * row_bytes + (uint32_t)(j * 64) : OOB;
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[i][j]), rw, voff, 0, 0);
    }
  }
}

// Scale, add bias and store a wave's accumulators.  acc[i][j][e] belongs to
// C[m_base + 16 i + r16][n_base + 16 j + 4 g + e].
template <int KIND, int OUT_DT, int MI, int NI, int BLOCK_BIAS = -1, typename acc_t>
SGLQ_DEV void epilogue(const GemmArgs& p, acc_t (&acc)[MI][NI], int m_base, int n_base, int r16, int g) {
  asm volatile("" : "+v"(r16), "+v"(g));  // keep the address arithmetic here (see epilogue_via_lds)
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = m_base + i * 16 + r16;
    if (m >= p.M) continue;
    float sam = 1.f;
    if constexpr (KIND == KIND_FP8_ROWCOL || KIND == KIND_I8_ROWCOL) sam = p.sa[m];
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int n = n_base + j * 16 + g * 4;
      if (n >= p.N) continue;  // N % 8 == 0 (% 4 for 32-bit outputs) is checked on the host: a run of 4 is in or out as a whole
      finish4<KIND, OUT_DT, BLOCK_BIAS>(p, m, n, acc[i][j], sam);
    }
  }
}

// Epilogue of the 256-row kernels for 16-bit outputs, in two halves of 128 rows: every
// wave converts one half of its accumulators (fragment rows i < MI / 2, then the rest; scales
// and bias applied) and drops them into a 128 x 512-byte image in one stage buffer, then all
// eight waves write the image out in rows, 16 bytes per lane, so that a wavefront store
// covers two full 512-byte row segments instead of sixteen 32-byte pieces.  A half is
// therefore the upper (lower) 8 MI rows of every wave row's 16 MI; splitting the tile into
// its upper and lower 128 rows instead leaves half of the waves idle while the others
// convert.  Chunk c (16 bytes) of image row r sits at chunk position c ^ (r & 31).  The other stage buffer is not touched: it is receiving the
// next tile's first K block.  The caller has made sure nobody reads `img` any more; on
// return every wave has passed a barrier after its last read of `img`.
template <int KIND, int OUT_DT, int MI, int NI, int BN, bool BIAS, int HALF_ROWS = 128, int PASSES = 2, typename acc_t>
SGLQ_DEV void epilogue_via_lds(const GemmArgs& p, acc_t (&acc)[MI][NI], char* img, float* col_lds, int m0, int n0,
                               int wm, int wn, int r16, int g, int lane, int wave) {
  constexpr int TN = NI * 16;
  // The addresses below depend on the lane only, not on the tile: left alone, the compiler
  // computes them once before the caller's tile loop and keeps dozens of registers alive
  // through every K step (and spills them inside the pipelined steps, where a scratch access
  // waits for all copies in flight).  Hide the lane-derived values' origin so that the
  // arithmetic stays here.
  asm volatile("" : "+v"(r16), "+v"(g), "+v"(lane));
  constexpr bool ROWCOL = KIND == KIND_FP8_ROWCOL || KIND == KIND_I8_ROWCOL;
  // Per-row / per-column kinds: the tile's 256 column scales and bias values go through LDS
  // (`col_lds`: bias in floats 0..255, scales in 256..511) and are read per column group while
  // converting, so that they do not occupy 8 NI registers next to the accumulators.
  if constexpr (ROWCOL) {
    const int t = (int)threadIdx.x & 255, nb = n0 + t;
    float v = 0.f;
    if (nb < p.N) {
      if (threadIdx.x >= 256) v = p.sb[nb];
      else if (p.bias) {
        if constexpr (OUT_DT == SGLQ_BF16) v = u2f((uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[nb] << 16);
        else v = (float)reinterpret_cast<const _Float16*>(p.bias)[nb];
      }
    }
    col_lds[threadIdx.x] = v;
    __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0_only());
    __builtin_amdgcn_s_barrier();
  }
  const int c = lane & 31;
  const int n = n0 + c * 8;
  char* out = reinterpret_cast<char*>(p.out);
  // Block-scaled kinds: the optional bias is the caller's `output += bias` on the rounded
  // result (fp8_utils.py:210-211), added to the image's values on their way out.  The tile's
  // 256 bias values wait in LDS behind the image (`col_lds`, written here and made
  // visible by the first barrier below), so that no register holds them across the epilogue.
  // (BIAS: a kernel variant of its own, launched only with a bias, so that the plain variant's
  // register allocation is not disturbed)
  constexpr bool add_bias = BIAS && is_block(KIND);
  if (add_bias && threadIdx.x < 256) {
    const int nb = n0 + (int)threadIdx.x;
    float b = 0.f;
    if (nb < p.N) {
      if constexpr (OUT_DT == SGLQ_BF16) b = u2f((uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[nb] << 16);
      else b = (float)reinterpret_cast<const _Float16*>(p.bias)[nb];
    }
    col_lds[threadIdx.x] = b;
  }
  constexpr int FR = MI / PASSES;  // fragment rows of a wave in one pass (two passes, the halves; three for 192-row tiles)
  constexpr int HR = FR * 16;      // rows of a wave row in one pass
  // The tile's part of the output as a buffer: rows m0 .. min(M, m0 + 256) - 1 from column n0
  // on.  Used when every 16-byte chunk of the tile's columns lies inside N and the extent fits
  // the 31-bit offsets (wave-uniform conditions).
  const uint32_t row_bytes = (uint32_t)p.ldo * 2u;
  const int rows_left = p.M - m0 < PASSES * HALF_ROWS ? p.M - m0 : PASSES * HALF_ROWS;
  const bool whole_chunks = n0 + BN <= p.N && p.ldo < (1 << 21);
  const __amdgpu_buffer_rsrc_t r_out =
      make_rsrc(out + ((int64_t)m0 * p.ldo + n0) * 2, whole_chunks ? (uint32_t)rows_left * row_bytes - (uint32_t)n0 * 2u : 0u);
  static_assert(MI % PASSES == 0 && (HR & (HR - 1)) == 0 && HALF_ROWS % HR == 0 && HALF_ROWS % 16 == 0, "the passes are split by fragment row");
  constexpr int RPW = HALF_ROWS / 8;  // image rows per wave in the store phase
#pragma unroll
  for (int half = 0; half < PASSES; ++half) {
    {
      float sam[FR];
#pragma unroll
      for (int ii = 0; ii < FR; ++ii) {
        sam[ii] = 1.f;
        if constexpr (ROWCOL) {
          const int m = m0 + wm * MI * 16 + half * HR + ii * 16 + r16;
          sam[ii] = (m < p.M) ? p.sa[m] : 0.f;
        }
      }
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        v4f bv = {0.f, 0.f, 0.f, 0.f}, sbv = bv;
        if constexpr (ROWCOL) {
          bv = *reinterpret_cast<const v4f*>(col_lds + wn * TN + j * 16 + g * 4);
          sbv = *reinterpret_cast<const v4f*>(col_lds + 256 + wn * TN + j * 16 + g * 4);
        }
        const int chunk = wn * (TN / 8) + j * 2 + (g >> 1);
#pragma unroll
        for (int ii = 0; ii < FR; ++ii) {
          const int i = half * FR + ii;
          const int ml = wm * HR + ii * 16 + r16;  // row inside the image
          float o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if constexpr (KIND == KIND_I8_ROWCOL) o[e] = __builtin_fmaf((float)acc[i][j][e], sbv[e] * sam[ii], bv[e]);
            else if constexpr (KIND == KIND_FP8_ROWCOL) o[e] = __builtin_fmaf(sam[ii], sbv[e] * acc[i][j][e], bv[e]);
            else o[e] = acc[i][j][e];
          }
          char* dst = img + ml * 512 + ((chunk ^ (ml & 31)) * 16) + (g & 1) * 8;
          if constexpr (OUT_DT == SGLQ_BF16) {
            typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
            *reinterpret_cast<bf4*>(dst) = bf4{(__bf16)o[0], (__bf16)o[1], (__bf16)o[2], (__bf16)o[3]};
          } else {
            typedef _Float16 h4 __attribute__((ext_vector_type(4)));
            *reinterpret_cast<h4*>(dst) = h4{(_Float16)o[0], (_Float16)o[1], (_Float16)o[2], (_Float16)o[3]};
          }
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0_only());
    __builtin_amdgcn_s_barrier();
    // 128 image rows, 8 waves: wave w writes rows 16 w .. 16 w + 15, two rows per store
    // instruction; image row ml is row ml % HR of wave row ml / HR's half.  All eight reads are
    // issued before the first store (one LDS latency instead of eight).
    v4i v[RPW / 2];
#pragma unroll
    for (int it = 0; it < RPW / 2; ++it) {
      const int ml = wave * RPW + it * 2 + (lane >> 5);
      v[it] = *reinterpret_cast<const v4i*>(img + ml * 512 + ((c ^ (ml & 31)) * 16));
    }
    if constexpr (add_bias) {
      const v4f blo = *reinterpret_cast<const v4f*>(col_lds + c * 8), bhi = *reinterpret_cast<const v4f*>(col_lds + c * 8 + 4);
      const float bias8[8] = {blo[0], blo[1], blo[2], blo[3], bhi[0], bhi[1], bhi[2], bhi[3]};
#pragma unroll
      for (int it = 0; it < RPW / 2; ++it) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t w = (uint32_t)v[it][q];
          float lo, hi;
          if constexpr (OUT_DT == SGLQ_BF16) {
            lo = u2f(w << 16) + bias8[2 * q];
            hi = u2f(w & 0xffff0000u) + bias8[2 * q + 1];
            typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
            v[it][q] = __builtin_bit_cast(int, bf2{(__bf16)lo, (__bf16)hi});
          } else {
            typedef _Float16 h2 __attribute__((ext_vector_type(2)));
            const h2 h = __builtin_bit_cast(h2, w);
            lo = (float)h[0] + bias8[2 * q];
            hi = (float)h[1] + bias8[2 * q + 1];
            v[it][q] = __builtin_bit_cast(int, h2{(_Float16)lo, (_Float16)hi});
          }
        }
      }
    }
    if (whole_chunks) {
      // bounds-checked buffer stores: rows past M and lanes past the tile's width get an offset
      // beyond the extent and are dropped; no branches, no 64-bit address arithmetic
#pragma unroll
      for (int it = 0; it < RPW / 2; ++it) {
        const int ml = wave * RPW + it * 2 + (lane >> 5);
        const uint32_t m_rel = (uint32_t)((ml / HR) * (PASSES * HR) + half * HR + (ml & (HR - 1)));
        const uint32_t voff = (c * 8 < BN) ? m_rel * row_bytes + (uint32_t)c * 16u : OOB;
        // (aux bit 1 = nt: a line that will not be read again before it leaves the caches)
        if (p.stream_out) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v[it]), r_out, voff, 0, 2);
        else __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v[it]), r_out, voff, 0, 0);
      }
    } else {
#pragma unroll
      for (int it = 0; it < RPW / 2; ++it) {
        const int ml = wave * RPW + it * 2 + (lane >> 5);
        const int m = m0 + (ml / HR) * (PASSES * HR) + half * HR + (ml & (HR - 1));
        if (m < p.M && c * 8 < BN) {
          char* row = out + ((int64_t)m * p.ldo + n) * 2;
          if (n + 8 <= p.N) *reinterpret_cast<v4i*>(row) = v[it];  // (N is a multiple of 8: a chunk is in or out as a whole)
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0_only());  // my reads of the image are complete
    __builtin_amdgcn_s_barrier();
  }
}

// Epilogue of PIPE_DIRECT: every wave turns its own accumulators into whole 128-byte row pieces through 2 KiB of
// LDS that no other wave touches, one fragment row (16 rows x 64 columns) at a time: four 8-byte writes per lane
// (the lane's four columns of each fragment), then two 16-byte reads and two stores of 8 rows x 128 bytes.  No
// block barrier and no stage buffer: LDS operations of a wave execute in order.  Chunk c (16 bytes) of row r sits
// at chunk position c ^ (r & 7) ^ (r >> 3).  Tiles cut by N (or rows too far apart for 31-bit offsets) take guarded
// stores and then wait for everything outstanding, so that the caller's count of younger operations stays an upper bound.
template <int OUT_DT, int MI, int NI, int BM, int BN, typename acc_t>
SGLQ_DEV void epilogue_direct(const GemmArgs& p, acc_t (&acc)[MI][NI], char* mine, int m0, int n0, int row0, int col0, int r16, int g,
                              int lane) {
  static_assert(NI == 4, "a wave's 64 columns are one 128-byte line of 16-bit outputs");
  asm volatile("" : "+v"(r16), "+v"(g), "+v"(lane));  // (keep the lane arithmetic here, as in epilogue_via_lds)
  char* out = reinterpret_cast<char*>(p.out);
  const uint32_t row_bytes = (uint32_t)p.ldo * 2u;
  const int rows_left = p.M - m0 < BM ? p.M - m0 : BM;
  const bool whole = n0 + BN <= p.N && p.ldo < (1 << 21);
  const __amdgpu_buffer_rsrc_t r_out =
      make_rsrc(out + ((int64_t)m0 * p.ldo + n0) * 2, whole ? (uint32_t)rows_left * row_bytes - (uint32_t)n0 * 2u : 0u);
  const int swz_w = (r16 & 7) ^ (r16 >> 3);
  char* const wr = mine + r16 * 128 + (g & 1) * 8;
  const int c = lane & 7, r8 = lane >> 3;
  // LDS operations of a wave execute in the order of the program: the reads of fragment row i see its writes and are
  // done before the writes of row i + 1 land, with no wait in between.  The only waits are the ones for the data of
  // row i's reads in front of its stores, which are issued behind the LDS operations of row i + 1 (the compiler places them).
  auto to_lds = [&](int i) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      char* dst = wr + (((j * 2 + (g >> 1)) ^ swz_w) * 16);
      if constexpr (OUT_DT == SGLQ_BF16) {
        typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<bf4*>(dst) = bf4{(__bf16)acc[i][j][0], (__bf16)acc[i][j][1], (__bf16)acc[i][j][2], (__bf16)acc[i][j][3]};
      } else {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<h4*>(dst) = h4{(_Float16)acc[i][j][0], (_Float16)acc[i][j][1], (_Float16)acc[i][j][2], (_Float16)acc[i][j][3]};
      }
    }
  };
  auto from_lds = [&](v4i (&v)[2]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = h * 8 + r8;
      v[h] = *reinterpret_cast<const v4i*>(mine + r * 128 + ((c ^ (r & 7) ^ (r >> 3)) * 16));
    }
  };
  auto to_memory = [&](int i, const v4i (&v)[2]) {
    if (whole) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t voff = (uint32_t)(row0 + i * 16 + h * 8 + r8) * row_bytes + (uint32_t)(col0 * 2 + c * 16);
        if (p.stream_out) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v[h]), r_out, voff, 0, 2);
        else __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v[h]), r_out, voff, 0, 0);
      }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int m = m0 + row0 + i * 16 + h * 8 + r8, n = n0 + col0 + c * 8;
        if (m < p.M && n + 8 <= p.N) *reinterpret_cast<v4i*>(out + ((int64_t)m * p.ldo + n) * 2) = v[h];
      }
    }
  };
  v4i v[2][2];
  to_lds(0);
  __builtin_amdgcn_wave_barrier();
  from_lds(v[0]);
#pragma unroll
  for (int i = 1; i < MI; ++i) {
    __builtin_amdgcn_wave_barrier();
    to_lds(i);
    __builtin_amdgcn_wave_barrier();
    from_lds(v[i & 1]);
    __builtin_amdgcn_sched_barrier(0);
    to_memory(i - 1, v[(i - 1) & 1]);
    __builtin_amdgcn_sched_barrier(0);
  }
  to_memory(MI - 1, v[(MI - 1) & 1]);
  if (!whole) __builtin_amdgcn_s_waitcnt(0);
}

// GROUPED: one launch for a group of problems that share N and K (the experts of an MoE
// layer).  Row tile t of the grid belongs to expert plan[t].expert and covers rows
// plan[t].row0 .. of A and C up to the expert's last row; B and its scales are the
// expert's.  Rows of the tile beyond the expert's are other experts' rows: they are
// computed and dropped by the epilogue's row bound.
template <int KIND, int BM, int BN, int WAVES_M, int WAVES_N, int OUT_DT, bool DMA, bool GROUPED = false>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, 2) void gemm_kernel(const GemmArgs p_in) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N;  // per-wave tile
  constexpr int MI = TM / 16, NI = TN / 16;
  constexpr int STAGE_BYTES = (BM + BN) * 128;
  constexpr int NLOAD = (BM + BN) / 8 / NW;  // 1 KiB copies per wave per stage
  constexpr bool IS_FP8 = fp8_operands(KIND);
  static_assert((BM + BN) % (8 * NW) == 0 && TM % 16 == 0 && TN % 16 == 0, "tile shape");
  static_assert(!is_block(KIND) || (128 % TN == 0), "a wave must stay inside one 128-wide scale block");

  __shared__ __attribute__((aligned(1024))) char smem[2 * STAGE_BYTES];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform by construction
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int r16 = lane & 15, g = lane >> 4;

  // blockIdx = split * tiles + tile; split s works on K blocks [kb_lo, kb_hi)
  GemmArgs p = p_in;
  const int tiles = p.tiles_m * p.tiles_n;
  const int split = GROUPED ? 0 : blockIdx.x / tiles;
  int tm, tn;
  tile_of_block(blockIdx.x - split * tiles, p.tiles_m, p.tiles_n, tm, tn);
  int m0 = tm * BM;
  const int n0 = tn * BN;
  if constexpr (GROUPED) {
    const int* plan = static_cast<const int*>(p.ws);
    if (tm >= plan[0]) return;  // the grid covers the largest possible number of row tiles
    const int* entry = plan + PLAN_HEADER + PLAN_ENTRY * tm;
    const int expert = entry[0];
    m0 = entry[1];
    p.M = entry[2];
    p.b += (int64_t)expert * p.b_expert_stride;
    p.sb += (int64_t)expert * p.sb_expert_stride;
  }

  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b, p.b_bytes);

  // ---- global -> LDS copy plan: copy i (of (BM+BN)/8) fills rows 8i..8i+7 of the stage
  uint32_t src_off[NLOAD];  // byte offset of this lane's 16-byte chunk at k0 = 0
  int src_k[NLOAD];         // its k offset inside the 128-byte K block
#pragma unroll
  for (int j = 0; j < NLOAD; ++j) {
    const int i = wave + j * NW;
    const int row = i * 8 + (lane >> 3);  // row inside the stage (A rows first, then B rows)
    const bool is_a = row < BM;
    const int rr = is_a ? row : row - BM;
    const int c = (lane & 7) ^ swz(rr);
    const int grow = is_a ? (m0 + rr) : (n0 + rr);
    const bool ok = is_a ? (grow < p.M) : (grow < p.N);
    src_k[j] = c * 16;
    src_off[j] = ok ? (uint32_t)grow * (is_a ? p.lda : p.ldb) + c * 16 : OOB;
  }

  auto issue_loads = [&](int stage, int k0) {
#pragma unroll
    for (int j = 0; j < NLOAD; ++j) {
      const int i = wave + j * NW;
      const bool is_a = (i * 8) < BM;  // uniform per wave instruction
      uint32_t off = (k0 + src_k[j] < p.K) ? src_off[j] + (uint32_t)k0 : OOB;
      if (src_off[j] == OOB) off = OOB;
      char* dst = smem + stage * STAGE_BYTES + i * 1024;
      if constexpr (DMA) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(is_a ? ra : rb, (__attribute__((address_space(3))) void*)dst, 16,
                                                 off, 0, 0, 0);
      } else {
        v4i v = __builtin_amdgcn_raw_buffer_load_b128(is_a ? ra : rb, off, 0, 0);
        *reinterpret_cast<v4i*>(dst + lane * 16) = v;
      }
    }
  };

  // ---- MFMA operand addresses in LDS
  const int sw = (r16 & 7) ^ (r16 >> 3);
  const int lane_off0 = r16 * 128 + (((2 * g) ^ sw) * 16);
  const int lane_off1 = lane_off0 ^ 16;
  const int a_base = (wm * TM) * 128;
  const int b_base = (BM + wn * TN) * 128;

  using acc_t = typename std::conditional<float_acc(KIND), v4f, v4i>::type;
  acc_t acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

  // ---- block scales: one activation scale per lane per 16-row fragment
  const int nkb_all = (p.K + 127) >> 7;
  const int kb_lo = (int)((int64_t)split * nkb_all / p.splits), nkb = (int)((int64_t)(split + 1) * nkb_all / p.splits);
  float sfa_next[MI];
  float sfb_next = 0.f;
  int sfa_row[MI];
  int nb = 0;
  if constexpr (is_block(KIND)) {
    const int nblocks = (p.N + 127) >> 7;
    nb = (n0 + wn * TN) >> 7;
    if (nb >= nblocks) nb = nblocks - 1;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      int m = m0 + wm * TM + i * 16 + r16;
      sfa_row[i] = m < p.M ? m : p.M - 1;
      sfa_next[i] = p.sa[sfa_row[i] * p.sa_stride_m + kb_lo * p.sa_stride_k];
    }
    sfb_next = p.sb[kb_lo * p.sb_stride_k + nb * p.sb_stride_n];
  }

  issue_loads(kb_lo & 1, kb_lo * 128);

  for (int kb = kb_lo; kb < nkb; ++kb) {
    const int cur = kb & 1;
    __builtin_amdgcn_s_waitcnt(0);  // this stage's copies (and prefetched scales) have landed
    __syncthreads();                // for every wave; and all waves are done reading the other stage
    if (kb + 1 < nkb) issue_loads(cur ^ 1, (kb + 1) * 128);

    float sc[MI];
    if constexpr (is_block(KIND)) {
#pragma unroll
      for (int i = 0; i < MI; ++i) sc[i] = sfa_next[i] * sfb_next;
      if (kb + 1 < nkb) {
#pragma unroll
        for (int i = 0; i < MI; ++i) sfa_next[i] = p.sa[sfa_row[i] * p.sa_stride_m + (kb + 1) * p.sa_stride_k];
        sfb_next = p.sb[(kb + 1) * p.sb_stride_k + nb * p.sb_stride_n];
      }
    }

    const char* st = smem + cur * STAGE_BYTES;
    v8i af[MI], bf[NI];
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const char* q = st + a_base + i * 16 * 128;
      v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
      v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
      af[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const char* q = st + b_base + j * 16 * 128;
      v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
      v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
      bf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }

#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        if constexpr (is_block(KIND)) {
          const v4f part = block_mfma<KIND>(bf[j], af[i]);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][j][e] = __builtin_fmaf(block_value<KIND>(part[e]), sc[i], acc[i][j][e]);
        } else if constexpr (KIND == KIND_FP8_ROWCOL) {
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[j], af[i], acc[i][j], 0, 0, 0, 0, 0, 0);
        } else {
          const v4i b0 = {bf[j][0], bf[j][1], bf[j][2], bf[j][3]}, b1 = {bf[j][4], bf[j][5], bf[j][6], bf[j][7]};
          const v4i a0 = {af[i][0], af[i][1], af[i][2], af[i][3]}, a1 = {af[i][4], af[i][5], af[i][6], af[i][7]};
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b0, a0, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b1, a1, acc[i][j], 0, 0, 0);
        }
      }
    }
  }

  if (p.splits > 1) store_partials<MI, NI>(p, acc, split, m0 + wm * TM, n0 + wn * TN, r16, g);
  else epilogue<KIND, OUT_DT, MI, NI>(p, acc, m0 + wm * TM, n0 + wn * TN, r16, g);
}

// ---------------------------------------------------------------------------
// Prefill kernel: 256 x 256 output tile, 8 wavefronts (2 per SIMD), each owning
// 128 (m) x 64 (n).  One K step (128 bytes) is 2 x 32 MFMAs x 32 cycles = 2048
// MFMA-pipe cycles per SIMD, about a microsecond, which is what hides the
// latency of the next stage's global -> LDS copies with only two 64 KiB stages.
// A wave keeps its four weight fragments of the step in registers and streams
// the eight activation fragments through a two-deep register queue, so each LDS
// byte is read once per wave and the 128 accumulator registers leave room for
// two waves per SIMD.
// ---------------------------------------------------------------------------
template <int KIND, int OUT_DT, bool BIAS>
__global__ __launch_bounds__(512) void gemm_big_kernel(const GemmArgs p) {
  constexpr int BM = 256, BN = 256, NW = 8, WAVES_N = 4;
  constexpr int TM = 128, TN = 64, MI = TM / 16, NI = TN / 16;
  constexpr int STAGE_BYTES = (BM + BN) * 128;
  constexpr int NLOAD = (BM + BN) / 8 / NW;  // 8 one-KiB copies per wave per stage: 4 of A, 4 of B
  constexpr bool IS_FP8 = fp8_operands(KIND);
  constexpr bool BLOCK = is_block(KIND);

  // One LDS object per kernel: with a second __shared__ array the compiler tells the arrays
  // apart by alias scopes and then orders every LDS read behind the direct-to-LDS copies in
  // flight (s_waitcnt vmcnt(0) throughout the K loop).  The epilogue's 512 floats (bias values
  // and column scales of the tile's columns) therefore live at the end of `smem`.
  __shared__ __attribute__((aligned(1024))) char smem[2 * STAGE_BYTES + 2048];
  float* const col_lds = reinterpret_cast<float*>(smem + 2 * STAGE_BYTES);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int r16 = lane & 15, g = lane >> 4;

  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b, p.b_bytes);

  // Copy j of this wave fills stage rows 8 (wave + 8 j) .. + 7; lane l brings row
  // l / 8 of those, chunk (l % 8) ^ swz(row).  swz depends on l / 8 and the parity
  // of the wave only, so all four A copies (and all four B copies) share one
  // per-lane offset and differ by a multiple of 64 rows.  Rows past M / N fall
  // beyond the buffer's extent and read as zero; the K offset travels in the
  // scalar operand (K is a multiple of 128 for this kernel).
  const int l8 = lane >> 3;
  const int c16 = (((lane & 7) ^ l8 ^ (wave & 1)) & 7) * 16;
  const uint32_t row_in_tile = (uint32_t)(wave * 8 + l8);
  uint32_t off_a = 0, off_b = 0;  // of the tile whose copies are being issued
  const uint32_t step_a = 64u * p.lda, step_b = 64u * p.ldb;
  auto issue_load = [&](int j, int stage, int k0) {
    const bool is_a = j < NLOAD / 2;
    const int i = wave + j * NW;
    char* dst = smem + stage * STAGE_BYTES + i * 1024;
    const uint32_t off = is_a ? off_a + (uint32_t)j * step_a : off_b + (uint32_t)(j - NLOAD / 2) * step_b;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(is_a ? ra : rb, (__attribute__((address_space(3))) void*)dst, 16, off, k0,
                                             0, 0);
  };

  const int sw = (r16 & 7) ^ (r16 >> 3);
  const int lane_off0 = r16 * 128 + (((2 * g) ^ sw) * 16);
  const int lane_off1 = lane_off0 ^ 16;
  const int a_base = (wm * TM) * 128;
  const int b_base = (BM + wn * TN) * 128;
  auto read_frag = [&](const char* q) -> v8i {
    v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
    v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  using acc_t = typename std::conditional<float_acc(KIND), v4f, v4i>::type;
  acc_t acc[MI][NI];

  // Block scales: row m of K block kb sits at sfa[m * stride_m + kb * stride_k].
  // A lane owns row r16 of each of the wave's 16-row fragments; rows past M read
  // as zero through the out-of-range offset (they are never stored).
  const int nkb = p.K >> 7;
  float sfa_cur[MI];
  float sfb_cur = 0.f, sfb_next = 0.f;
  __amdgpu_buffer_rsrc_t rs = ra;
  uint32_t sfa_off = 0, sfa_ok = 0;
  int sfa_frag = 0, sfa_step = 0, nb = 0;
  if constexpr (BLOCK) {
    const int64_t sfa_elems = (int64_t)(p.M - 1) * p.sa_stride_m + (int64_t)(nkb - 1) * p.sa_stride_k + 1;
    rs = make_rsrc(p.sa, (uint32_t)(sfa_elems * 4));
    sfa_frag = (int)(16 * p.sa_stride_m * 4);
    sfa_step = (int)(p.sa_stride_k * 4);
  }
  // Addressing of the tile whose copies and scales are issued from now on.
  auto set_tile = [&](int m0, int n0) {
    off_a = (uint32_t)(m0 + row_in_tile) * p.lda + c16;
    off_b = (uint32_t)(n0 + row_in_tile) * p.ldb + c16;
    if constexpr (BLOCK) {
      const int nblocks = (p.N + 127) >> 7;
      nb = (n0 + wn * TN) >> 7;
      if (nb >= nblocks) nb = nblocks - 1;
      nb = __builtin_amdgcn_readfirstlane(nb);
      const int mrow = m0 + wm * TM + r16;
      // a row past M must not alias a valid element of another K block: send it out of range
      sfa_off = mrow < p.M ? (uint32_t)(mrow * p.sa_stride_m * 4) : OOB;
      sfa_ok = 0;
#pragma unroll
      for (int i = 0; i < MI; ++i) sfa_ok |= (mrow + i * 16 < p.M ? 1u : 0u) << i;
    }
  };
  auto load_sfa = [&](int i, int kb) -> float {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                         rs, ((sfa_ok >> i) & 1) ? sfa_off + i * sfa_frag : OOB, kb * sfa_step, 0));
  };

  // One K step on stage `cur`.  With a `pre_tag`, the copies (into the other stage) and the
  // scales of K block `kn` of the tile that set_tile named last are issued here, in the
  // shadow of the MFMAs, so that no wave spends issue slots on them while the MFMA pipe is
  // idle: that is the next K block of this tile, or, in a tile's last step (`last_tag`),
  // the first K block of the block's next tile.
  auto k_step = [&](int cur, int kn, auto pre_tag, auto last_tag) {
    constexpr bool pre = decltype(pre_tag)::value;
    constexpr bool last = decltype(last_tag)::value;
    const char* st = smem + cur * STAGE_BYTES;
    v8i bf[NI];
    bf[0] = read_frag(st + b_base);
    v8i a_cur = read_frag(st + a_base);
#pragma unroll
    for (int j = 1; j < NI; ++j) bf[j] = read_frag(st + b_base + j * 16 * 128);
    float sc = 0.f, sc_prev = 0.f;
    __builtin_amdgcn_sched_barrier(0);

    v4f part_prev = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      v8i a_nxt = a_cur;
      if constexpr (BLOCK) {
        sc_prev = sc;
        sc = sfa_cur[i] * sfb_cur;
      }
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        const int idx = i * NI + j;
        if constexpr (BLOCK) {
          v4f part = block_mfma<KIND>(bf[j], a_cur);
          __builtin_amdgcn_sched_barrier(0);
          if (j == 0 && i + 1 < MI) a_nxt = read_frag(st + a_base + (i + 1) * 16 * 128);
          if (pre && idx < NLOAD) issue_load(idx, cur ^ 1, kn * 128);
          if (idx > 0) {  // scale-and-accumulate the previous MFMA's result while this one runs
            const int pi = (idx - 1) / NI, pj = (idx - 1) % NI;
            const float s_use = (pi == i) ? sc : sc_prev;
            acc[pi][pj][0] = __builtin_fmaf(block_value<KIND>(part_prev[0]), s_use, acc[pi][pj][0]);
            acc[pi][pj][1] = __builtin_fmaf(block_value<KIND>(part_prev[1]), s_use, acc[pi][pj][1]);
            acc[pi][pj][2] = __builtin_fmaf(block_value<KIND>(part_prev[2]), s_use, acc[pi][pj][2]);
            acc[pi][pj][3] = __builtin_fmaf(block_value<KIND>(part_prev[3]), s_use, acc[pi][pj][3]);
          }
          if (pre && idx == NLOAD) sfb_next = p.sb[kn * p.sb_stride_k + nb * p.sb_stride_n];
          // fragment i - 1's scale is dead once its last result is folded in (idx = 4 i): refill it
          if (pre && j == 1 && i >= 1) sfa_cur[i - 1] = load_sfa(i - 1, kn);
          part_prev = part;
        } else if constexpr (KIND == KIND_FP8_ROWCOL) {
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[j], a_cur, acc[i][j], 0, 0, 0, 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (j == 0 && i + 1 < MI) a_nxt = read_frag(st + a_base + (i + 1) * 16 * 128);
          if (pre && idx < NLOAD) issue_load(idx, cur ^ 1, kn * 128);
        } else {
          const v4i b0 = {bf[j][0], bf[j][1], bf[j][2], bf[j][3]}, b1 = {bf[j][4], bf[j][5], bf[j][6], bf[j][7]};
          const v4i a0 = {a_cur[0], a_cur[1], a_cur[2], a_cur[3]}, a1 = {a_cur[4], a_cur[5], a_cur[6], a_cur[7]};
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b0, a0, acc[i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (j == 0 && i + 1 < MI) a_nxt = read_frag(st + a_base + (i + 1) * 16 * 128);
          if (pre && idx < NLOAD) issue_load(idx, cur ^ 1, kn * 128);
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b1, a1, acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      a_cur = a_nxt;
    }
    if constexpr (BLOCK) {
      acc[MI - 1][NI - 1][0] = __builtin_fmaf(block_value<KIND>(part_prev[0]), sc, acc[MI - 1][NI - 1][0]);
      acc[MI - 1][NI - 1][1] = __builtin_fmaf(block_value<KIND>(part_prev[1]), sc, acc[MI - 1][NI - 1][1]);
      acc[MI - 1][NI - 1][2] = __builtin_fmaf(block_value<KIND>(part_prev[2]), sc, acc[MI - 1][NI - 1][2]);
      acc[MI - 1][NI - 1][3] = __builtin_fmaf(block_value<KIND>(part_prev[3]), sc, acc[MI - 1][NI - 1][3]);
      if constexpr (pre) {
        sfa_cur[MI - 1] = load_sfa(MI - 1, kn);
        sfb_cur = sfb_next;
      }
    }
    if constexpr (!last) {
      // The next stage's copies were the first eight vector-memory loads of this step and
      // vector-memory operations retire in order, so it is enough to wait until at most the
      // SCALE_LOADS_AFTER_COPIES younger ones (activation-scale refills, none for the other
      // kinds) are still in flight; lgkmcnt(0) covers this wave's LDS reads of the stage
      // that the next step overwrites.  A bare s_barrier: the waits above are the only
      // ordering needed, a fence would drain the scale refills as well.
      constexpr int SCALE_LOADS_AFTER_COPIES = BLOCK ? MI - 1 : 0;
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(SCALE_LOADS_AFTER_COPIES));
      __builtin_amdgcn_s_barrier();
    } else {
      // Last K block of a tile: wait for everything, so that the epilogue's stores are the
      // only vector-memory operations in flight when the next tile starts.  After the
      // barrier the next tile's first K block is visible to every wave and nobody reads
      // this stage any more (it becomes the epilogue's staging buffer).
      __builtin_amdgcn_s_waitcnt(0);
      __builtin_amdgcn_s_barrier();
    }
  };

  // ---- persistent walk over the tiles blockIdx, blockIdx + gridDim, ...
  const int total = p.tiles_m * p.tiles_n;
  int tile = blockIdx.x;
  int tm, tn;
  tile_of_block(tile, p.tiles_m, p.tiles_n, tm, tn);
  int m0 = tm * BM, n0 = tn * BN;
  int par = 0;  // stage that holds K block 0 of the current tile

  set_tile(m0, n0);
#pragma unroll
  for (int j = 0; j < NLOAD; ++j) issue_load(j, 0, 0);
  if constexpr (BLOCK) {
#pragma unroll
    for (int i = 0; i < MI; ++i) sfa_cur[i] = load_sfa(i, 0);
    sfb_cur = p.sb[nb * p.sb_stride_n];
  }
  __builtin_amdgcn_s_waitcnt(0);
  __builtin_amdgcn_s_barrier();

  while (true) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

    for (int kb = 0; kb + 1 < nkb; ++kb) k_step((kb + par) & 1, kb + 1, std::true_type{}, std::false_type{});

    const int next_tile = tile + (int)gridDim.x;
    const bool has_next = next_tile < total;
    const int last_stage = (nkb - 1 + par) & 1;
    const int cm0 = m0, cn0 = n0;
    // The tile's last step always prefetches: past the block's last tile it is pointed at
    // rows beyond M and N, which the buffer bounds turn into zero fill without memory traffic.
    tile_of_block(has_next ? next_tile : 0, p.tiles_m, p.tiles_n, tm, tn);
    m0 = has_next ? tm * BM : p.tiles_m * BM;
    n0 = has_next ? tn * BN : p.tiles_n * BN;
    set_tile(m0, n0);  // the current tile issues no more copies or scale loads
    k_step(last_stage, 0, std::true_type{}, std::true_type{});

    if constexpr (KIND == KIND_I8_RAW) {
      epilogue<KIND, OUT_DT, MI, NI>(p, acc, cm0 + wm * TM, cn0 + wn * TN, r16, g);
    } else {
      // (rows of 16-bit outputs are 16-byte aligned: checked on the host)
      epilogue_via_lds<KIND, OUT_DT, MI, NI, BN, BIAS>(p, acc, smem + last_stage * STAGE_BYTES, col_lds, cm0, cn0, wm, wn, r16, g, lane, wave);
    }
    if (!has_next) break;
    tile = next_tile;
    par = last_stage ^ 1;
  }
}

// ---------------------------------------------------------------------------
// 256 x 256 kernel, software-pipelined across K steps (K >= 384).  Same tile, wave grid
// and LDS layout as gemm_big_kernel; what differs is what is in registers when a step
// starts and how far ahead the copies run.  With u the running index of the K block:
//   * step u starts with block u's four weight fragments and first activation fragment in
//     registers.  Barrier 1, behind MFMA 3: every wave holds block u's weights in registers,
//     so the weight half of block u's stage is free and receives the weight copies of block
//     u + 2 (behind MFMAs 4..7): they have 1 3/4 steps to land.
//   * barrier 2, before the last activation fragment's four MFMAs (28..31): every wave has
//     completed its LDS reads of block u's activations, and block u + 1 has landed.  Behind
//     MFMAs 28..31 a wave reads the first fragments of block u + 1 (each weight fragment
//     right after its last use) and issues the activation copies of block u + 2 into the
//     half that just became free (one step to land).
//   * the block scales travel through LDS like the operands: per K block one dword per
//     activation row (four 64-row copies, waves 0..3) and the tile's two weight scales (wave
//     4), issued with the activation copies and read into registers behind MFMAs 28..31.
//     Vector-memory instructions are the scarce issue resource of this loop (a CU's 64
//     one-KiB copies per step already keep its address unit busy half of the time); loading
//     the scales per fragment and per wave took as many instructions again.
// A CU needs about a stage's worth of bytes in flight to cover the memory latency of a
// step; a plain two-stage ring has less than that most of the time.  The sequence of
// blocks runs across tile boundaries (the block's next tile follows the last K block of
// the current one); only the copies behind a tile's last step are deferred to the next
// tile's first step, because the freed stage stages the C tile.
// ---------------------------------------------------------------------------
// MODE selects one of three variants, each launched only where it is needed so that the
// plain one keeps its register allocation: 0 = whole tiles, 1 = split-K work units (raw
// partial sums to the workspace), 2 = whole tiles of a block-scaled kind with a bias,
// 3 = grouped GEMM (row tiles and their experts from the plan in the workspace).
constexpr int PIPE_PLAIN = 0, PIPE_SPLITK = 1, PIPE_BIAS = 2, PIPE_GROUPED = 3, PIPE_DIRECT = 4;
// 4 = whole tiles whose outputs every wave brings into row order by itself (epilogue_direct: 2 KiB of LDS per
// wave, no block barrier): no stage is needed at a tile's end, so the copies run on across tile boundaries without the deferral,
// and the next tile's first K blocks are older in the vector-memory queue than the tile's stores: the steps that
// wait for them do not wait for the stores (vector-memory operations retire in order).  For short K, where
// the stores of a 256 x 256 tile every four to twelve steps are what the other variants stall on.
// BM = 128: tiles of 128 rows (a wave owns 64 x 64, 16 MFMAs per step) for problems whose
// 256-row tiles would leave most of the chip idle; same schedule, half the activation copies.
template <int KIND, int OUT_DT, int MODE, int BM = 256>
__global__ __launch_bounds__(512) void gemm_pipe_kernel(const GemmArgs p) {
  constexpr int BN = 256, NW = 8, WAVES_N = 4;
  constexpr int TM = BM / 2, TN = 64, MI = TM / 16, NI = TN / 16;
  constexpr int STAGE_BYTES = (BM + BN) * 128;
  constexpr int NCOPY_A = BM / 64;  // activation copies per wave per stage
  constexpr bool IS_FP8 = fp8_operands(KIND);
  constexpr bool BLOCK = is_block(KIND);
  constexpr bool HW = KIND == KIND_FP8_BLOCK_POW2;  // the MFMA applies the block scales
  constexpr bool FOLD = BLOCK && !HW;               // they are applied to each MFMA's result
  constexpr bool DIRECT = MODE == PIPE_DIRECT;      // outputs stored from the accumulators; uniform steps across tile boundaries
  static_assert(NI == 4 && (MI == 8 || MI == 4), "the copy schedule below is written for 4 x 8 or 4 x 4 fragments");
  static_assert(!DIRECT || (MI == 8 && BLOCK), "PIPE_DIRECT is built for the block-scaled kinds on 256-row tiles");

  constexpr int SCALE_BYTES = 2048;  // per K block: 256 activation-row scales, then the tile's two weight scales
  // (one LDS object per kernel, see gemm_big_kernel: the epilogue's 512 floats sit at the end)
  // (PIPE_DIRECT: 2 KiB more per wave, the wave's own part of the epilogue)
  __shared__ __attribute__((aligned(1024))) char smem[2 * STAGE_BYTES + 2 * SCALE_BYTES + 2048 + (MODE == PIPE_DIRECT ? NW * 2048 : 0)];
  float* const col_lds = reinterpret_cast<float*>(smem + 2 * STAGE_BYTES + 2 * SCALE_BYTES);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int r16 = lane & 15, g = lane >> 4;

  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b, p.b_bytes);

  // Copy j (0..3) of a wave fills activation rows 8 (wave + 8 j) .. + 7 of the stage, and
  // the same rows of the weight half; lane l brings row l / 8 of those, chunk
  // (l % 8) ^ swz(row).  swz depends on l / 8 and the parity of the wave only, so the four
  // copies share one per-lane offset (lane_a / lane_b: the lane's row inside the tile and its
  // chunk) and everything else travels in the scalar operand: the tile's first row, the copy's
  // multiple of 64 rows and the K offset.  The buffer's range check covers the sum of both
  // offsets: rows past M / N fall beyond the extent and read as zero.
  const int l8 = lane >> 3;
  const int c16 = (((lane & 7) ^ l8 ^ (wave & 1)) & 7) * 16;
  const uint32_t row_in_tile = (uint32_t)(wave * 8 + l8);
  const uint32_t lane_a = row_in_tile * p.lda + c16, lane_b = row_in_tile * p.ldb + c16;
  const uint32_t step_a = 64u * p.lda, step_b = 64u * p.ldb;
  // off_a / off_b: tile of the block after the current one (copies deferred to a tile's first
  // step); off_a2 / off_b2: tile of the block two after the current one.  Scalars: byte offset
  // of the tile's first row.
  uint32_t off_a = 0, off_a2 = 0, off_b = 0, off_b2 = 0;
  auto copy_a = [&](int j, int stage, int k0, uint32_t off) {
    char* dst = smem + stage * STAGE_BYTES + (wave + j * NW) * 1024;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (__attribute__((address_space(3))) void*)dst, 16, lane_a,
                                             off + (uint32_t)j * step_a + (uint32_t)k0, 0, 0);
  };
  // Grouped mode: every tile has its expert's weight; b_cur / b_two are the weights of the
  // tiles of the block after the current one and of the block two after it (like off_b / off_b2).
  const char* b_cur = p.b;
  const char* b_two = p.b;
  auto copy_b = [&](int j, int stage, int k0, uint32_t off, bool two_ahead) {
    char* dst = smem + stage * STAGE_BYTES + BM * 128 + (wave + j * NW) * 1024;
    if constexpr (MODE == PIPE_GROUPED) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(make_rsrc(two_ahead ? b_two : b_cur, p.b_bytes),
                                               (__attribute__((address_space(3))) void*)dst, 16, lane_b,
                                               off + (uint32_t)j * step_b + (uint32_t)k0, 0, 0);
    } else {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void*)dst, 16, lane_b,
                                               off + (uint32_t)j * step_b + (uint32_t)k0, 0, 0);
    }
  };
  // (a tile past the last one: any offset beyond the extents; the sum with a lane's offset stays below 2^32)
  auto a_offset = [&](int m0) { return m0 < p.M ? (uint32_t)m0 * p.lda : OOB; };
  auto b_offset = [&](int n0) { return n0 < p.N ? (uint32_t)n0 * p.ldb : OOB; };

  const int sw = (r16 & 7) ^ (r16 >> 3);
  const int lane_off0 = r16 * 128 + (((2 * g) ^ sw) * 16);
  const int lane_off1 = lane_off0 ^ 16;
  const int a_base = (wm * TM) * 128;
  const int b_base = (BM + wn * TN) * 128;
  auto read_frag = [&](const char* q) -> v8i {
    v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
    v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  using acc_t = typename std::conditional<float_acc(KIND), v4f, v4i>::type;
  acc_t acc[MI][NI];
  v8i bf[NI];  // the step's weight fragments
  v8i a_cur;   // the activation fragment the next MFMAs use

  // Block scales.  Row m of K block kb sits at sfa[m * stride_m + kb * stride_k]; a lane owns
  // row r16 of each of the wave's 16-row fragments.  Every wave issues one 4-byte-per-lane
  // copy per K block: waves 0..3 the activation scales of tile rows 64 w + lane, wave 4 the
  // two weight scales of the tile's two 128-column blocks (lanes 0 and 1), waves 5..7 nothing
  // (all lanes out of range; kept so that the instruction stream has no branch).
  // lane_s: the lane's offset inside a tile's scales; sc_off / sc_off2 (scalars): those of the
  // tile of block u + 1 / u + 2.  Rows past M and a second column block past N are not singled
  // out: what they read (a value inside the scale tensor, or zero beyond it) only reaches
  // outputs that the epilogue drops.
  const int nkb_all = p.K >> 7;
  const int splits = MODE == PIPE_SPLITK ? p.splits : 1;
  const int nkb = nkb_all / splits;  // K blocks of one work unit (the host makes it divide)
  float sfa_cur[MI];
  float sfb_cur = 0.f;
  __amdgpu_buffer_rsrc_t rsc = ra;
  uint32_t lane_s = OOB, sc_off = SC_NONE, sc_off2 = SC_NONE;
  int sc_step = 0;
  const int sc_dst = 2 * STAGE_BYTES + wave * 256;  // waves 5..7 land behind the used part
  const int sfa_rd = 2 * STAGE_BYTES + (wm * TM + r16) * 4;
  const int sfb_rd = 2 * STAGE_BYTES + 1024 + (wn >> 1) * 4;
  if constexpr (BLOCK) {
    const int nblocks = (p.N + 127) >> 7;
    const int sa_last = (HW && p.sa_packed) ? (nkb_all - 1) >> 2 : nkb_all - 1;  // (packed: words of four K blocks)
    const int64_t sfa_elems = (int64_t)(p.M - 1) * p.sa_stride_m + (int64_t)sa_last * p.sa_stride_k + 1;
    int64_t sfb_elems = (int64_t)(nblocks - 1) * p.sb_stride_n + (int64_t)(nkb_all - 1) * p.sb_stride_k + 1;
    if constexpr (MODE == PIPE_GROUPED) sfb_elems += (int64_t)(p.num_experts - 1) * p.sb_expert_stride;
    rsc = wave < 4 ? make_rsrc(p.sa, (uint32_t)(sfa_elems * 4)) : make_rsrc(p.sb, (uint32_t)(sfb_elems * 4));
    sc_step = (int)((wave < 4 ? p.sa_stride_k : p.sb_stride_k) * 4);
    if (wave < 4) lane_s = wave * 64 < BM ? (uint32_t)((wave * 64 + lane) * p.sa_stride_m * 4) : OOB;
    else lane_s = (wave == 4 && lane < 2) ? (uint32_t)(lane * p.sb_stride_n * 4) : OOB;
  }
  // (SC_NONE: no tile; beyond both scale tensors, and its sum with OOB does not wrap)
  auto scale_offset = [&](int m0, int n0, int expert) -> uint32_t {
    if (m0 >= p.M || n0 >= p.N) return SC_NONE;
    if (wave < 4) return (uint32_t)(m0 * p.sa_stride_m * 4);
    return (uint32_t)(((n0 >> 7) * p.sb_stride_n + expert * p.sb_expert_stride) * 4);
  };
  // (packed activation scales: this wave's copy of K block kb fetches the word of K blocks 4 (kb / 4) .. + 3)
  const int sc_kshift = (HW && p.sa_packed && wave < 4) ? 2 : 0;
  const bool sa_packed = HW && p.sa_packed;
  auto code_shift = [&](int kb) { return sa_packed ? 8 * (kb & 3) : 23; };
  int sh_cur = 23;  // where the UE8M0 code of the K block in sfa_cur sits inside its word
  auto copy_scales = [&](int buf, int kb, uint32_t off) {
    char* dst = smem + buf * SCALE_BYTES + sc_dst;
    const int kw = HW ? kb >> sc_kshift : kb;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsc, (__attribute__((address_space(3))) void*)dst, 4, lane_s, (uint32_t)(kw * sc_step) + off, 0,
                                             0);
  };
  auto read_sfa = [&](int buf, int i) -> float {
    return *reinterpret_cast<const float*>(smem + buf * SCALE_BYTES + sfa_rd + i * 64);
  };
  auto read_sfb = [&](int buf) -> float { return *reinterpret_cast<const float*>(smem + buf * SCALE_BYTES + sfb_rd); };

  // One K step: block u sits in stage `cur` and its first fragments are in bf / a_cur.
  // kn: index, inside its tile, of block u + 1 (scales, and the copies deferred to a tile's
  // first step); kn2: that of block u + 2 (off_a2 / off_b2).
  // (PIPE_DIRECT: every step copies like a middle step; stores_tag: the tile before this first step has just
  // issued its 2 MI stores, which are younger than block u + 1's copies)
  auto k_step = [&](int cur, int kn, int kn2, auto first_tag, auto last_tag, auto stores_tag) {
    constexpr bool first = decltype(first_tag)::value;
    constexpr bool last = decltype(last_tag)::value;
    constexpr bool after_stores = decltype(stores_tag)::value;
    constexpr bool refill = !last;             // read block u + 1's first fragments and scales behind their last use
    constexpr bool copies = !last || DIRECT;   // issue the copies of block u + 2
    const char* st = smem + cur * STAGE_BYTES;
    const char* sn = smem + (cur ^ 1) * STAGE_BYTES;
    float sc = 0.f, sc_prev = 0.f;
    v4f part_prev = {0.f, 0.f, 0.f, 0.f};
    int ea = 0;                                 // HW: exponent byte of the fragment's activation scale (per lane: its row)
    const int eb = HW ? ue8m0_of(sfb_cur) : 0;  // ... and of the block's weight scale
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      v8i a_nxt = a_cur;
      if constexpr (FOLD) {
        sc_prev = sc;
        sc = sfa_cur[i] * sfb_cur;
      }
      if constexpr (HW) ea = ue8m0_at(sfa_cur[i], sh_cur);
      if (i == 1 && copies) {
        // barrier 1: MFMAs 0..3 have consumed this wave's weight fragments, so its LDS reads
        // of block u's weights are complete; behind the barrier that holds for every wave.
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
      if (i == MI - 1) {
        // barrier 2.  Vector-memory operations retire in order; block u + 1's last copy is
        // the activation copy behind MFMA 31 of the step before (MFMA 11 of this step in a
        // tile's first step).  Younger than it are only the four weight copies of block u + 2,
        // which stay in flight.  lgkmcnt(0): this wave's LDS reads of block u's activations
        // and scales are complete.  A bare s_barrier: these waits are all the ordering needed.
        // (with 16 MFMAs per step the first step's weight copies of block u + 2 come behind
        // this barrier, and what is in flight here are the deferred copies of block u + 1)
        constexpr int YOUNGER = DIRECT ? 4 + (after_stores ? 2 * MI : 0) : ((last || (first && MI == 4)) ? 0 : 4);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(YOUNGER));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        const int idx = i * NI + j;
        v4f part = {0.f, 0.f, 0.f, 0.f};
        if constexpr (FOLD) {
          part = block_mfma<KIND>(bf[j], a_cur);
        } else if constexpr (HW) {
          const v4f c0 = first ? v4f{0.f, 0.f, 0.f, 0.f} : acc[i][j];
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[j], a_cur, c0, 0, 0, 0, eb, 0, ea);
        } else if constexpr (KIND == KIND_FP8_ROWCOL) {
          // (a tile's first step starts from zero instead of clearing 128 registers beforehand)
          const v4f c0 = first ? v4f{0.f, 0.f, 0.f, 0.f} : acc[i][j];
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[j], a_cur, c0, 0, 0, 0, 0, 0, 0);
        } else {
          const v4i b0 = {bf[j][0], bf[j][1], bf[j][2], bf[j][3]};
          const v4i a0 = {a_cur[0], a_cur[1], a_cur[2], a_cur[3]};
          const v4i c0 = first ? v4i{0, 0, 0, 0} : acc[i][j];
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b0, a0, c0, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!IS_FP8 && !BLOCK) {
          const v4i b1 = {bf[j][4], bf[j][5], bf[j][6], bf[j][7]};
          const v4i a1 = {a_cur[4], a_cur[5], a_cur[6], a_cur[7]};
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b1, a1, acc[i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (i + 1 < MI) {
          if (j == 0) a_nxt = read_frag(st + a_base + (i + 1) * 16 * 128);
        } else {
          // weight fragment j has had its last use in this step: refill it from block u + 1
          // (not in a tile's last step: the next tile's first fragments and scales are read behind
          // the epilogue, which needs the registers)
          if constexpr (refill) {
            bf[j] = read_frag(sn + b_base + j * 16 * 128);
            if (j == 0) a_nxt = read_frag(sn + a_base);
          }
          if constexpr (copies) {
            if (j < NCOPY_A) copy_a(j, cur, kn2 * 128, off_a2);
          }
          if constexpr (BLOCK) {
            if constexpr (refill) {
              // scales i < MI - 1 had their last use when the last fragment's scale was formed; its own
              // scale and sfb_cur are dead as well: `sc` holds their product (HW: `ea` and `eb` their exponents)
#pragma unroll
              for (int q = 0; q < MI / NI; ++q) sfa_cur[(MI / NI) * j + q] = read_sfa(cur ^ 1, (MI / NI) * j + q);
              if (j == 0) sfb_cur = read_sfb(cur ^ 1);
            }
            if constexpr (copies) {
              if (j == 0) copy_scales(cur, kn2, sc_off2);
            }
          }
        }
        if constexpr (first && !DIRECT) {
          if (idx >= 4 && idx < 8) copy_b(idx - 4, cur ^ 1, kn * 128, off_b, false);
          if (idx >= 8 && idx < 8 + NCOPY_A) copy_a(idx - 8, cur ^ 1, kn * 128, off_a);
          if (BLOCK && idx == 11) copy_scales(cur ^ 1, kn, sc_off);
          if (idx >= 12 && idx < 16) copy_b(idx - 12, cur, kn2 * 128, off_b2, true);
        } else if constexpr (copies) {
          if (idx >= 4 && idx < 8) copy_b(idx - 4, cur, kn2 * 128, off_b2, true);
        }
        if constexpr (FOLD) {
          if (idx > 0) {  // scale-and-accumulate the previous MFMA's result while this one runs
            const int pi = (idx - 1) / NI, pj = (idx - 1) % NI;
            const float s_use = (pi == i) ? sc : sc_prev;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              acc[pi][pj][e] = first ? block_value<KIND>(part_prev[e]) * s_use
                                     : __builtin_fmaf(block_value<KIND>(part_prev[e]), s_use, acc[pi][pj][e]);
          }
          part_prev = part;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      a_cur = a_nxt;
    }
    if constexpr (FOLD) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        acc[MI - 1][NI - 1][e] = first ? block_value<KIND>(part_prev[e]) * sc
                                       : __builtin_fmaf(block_value<KIND>(part_prev[e]), sc, acc[MI - 1][NI - 1][e]);
    }
    if constexpr (HW && refill) sh_cur = code_shift(kn);  // sfa_cur now holds block u + 1's words
  };

  // ---- persistent walk over the work units blockIdx, blockIdx + gridDim, ...  A unit is an
  // output tile, or with split-K (p.splits > 1) one of a tile's p.splits contiguous K ranges,
  // whose raw partial sums go to the workspace for splitk_reduce_kernel.
  // Grouped mode: the row tiles come from the plan in the workspace (their number is device
  // data); a tile's rows end where its expert's rows end.
  const int* plan = static_cast<const int*>(p.ws);
  const int tiles_m = MODE == PIPE_GROUPED ? plan[0] : p.tiles_m;
  const int tiles = tiles_m * p.tiles_n;
  const int total = tiles * splits;
  auto unit_origin = [&](int u, int& um0, int& un0, int& ukb0, int& uexpert, int& um_end) {
    const int split = MODE == PIPE_SPLITK ? u / tiles : 0;
    int tm, tn;
    tile_of_block(u - split * tiles, tiles_m, p.tiles_n, tm, tn);
    um0 = tm * BM;
    un0 = tn * BN;
    ukb0 = split * nkb;
    uexpert = 0;
    um_end = p.M;
    if constexpr (MODE == PIPE_GROUPED) {
      const int* entry = plan + PLAN_HEADER + PLAN_ENTRY * tm;
      uexpert = entry[0];
      um0 = entry[1];
      um_end = entry[2];
    }
  };
  int unit = blockIdx.x;
  if (MODE == PIPE_GROUPED && unit >= total) return;  // the grid is sized for the largest possible plan
  int m0, n0, kb0, expert, m_end;
  unit_origin(unit, m0, n0, kb0, expert, m_end);
  int par = 0;  // stage that holds the unit's first K block

  off_a = off_a2 = a_offset(m0);
  off_b = off_b2 = b_offset(n0);
  if constexpr (MODE == PIPE_GROUPED) b_cur = b_two = p.b + (int64_t)expert * p.b_expert_stride;
  if constexpr (BLOCK) sc_off = sc_off2 = scale_offset(m0, n0, expert);
#pragma unroll
  for (int j = 0; j < NCOPY_A; ++j) copy_a(j, 0, kb0 * 128, off_a);
#pragma unroll
  for (int j = 0; j < 4; ++j) copy_b(j, 0, kb0 * 128, off_b, false);
  if constexpr (BLOCK) copy_scales(0, kb0, sc_off);
  __builtin_amdgcn_s_waitcnt(0);
  __builtin_amdgcn_s_barrier();
  // a unit's first weight fragments, activation fragment and scales, from stage `stage`
  auto read_first = [&](int stage) {
#pragma unroll
    for (int j = 0; j < NI; ++j) bf[j] = read_frag(smem + stage * STAGE_BYTES + b_base + j * 16 * 128);
    a_cur = read_frag(smem + stage * STAGE_BYTES + a_base);
    if constexpr (BLOCK) {
#pragma unroll
      for (int i = 0; i < MI; ++i) sfa_cur[i] = read_sfa(stage, i);
      sfb_cur = read_sfb(stage);
      if constexpr (HW) sh_cur = code_shift(kb0);
    }
  };
  read_first(0);
  if constexpr (DIRECT) {
    // the steps of this variant expect block u + 1's copies to be under way when step u starts
#pragma unroll
    for (int j = 0; j < 4; ++j) copy_b(j, 1, (kb0 + 1) * 128, off_b, false);
#pragma unroll
    for (int j = 0; j < NCOPY_A; ++j) copy_a(j, 1, (kb0 + 1) * 128, off_a);
    if constexpr (BLOCK) copy_scales(1, kb0 + 1, sc_off);
  }

  while (true) {
    // The block's next unit; past its last one the prefetches are pointed at rows beyond M
    // and N, which the buffer bounds turn into zero fill without memory traffic.
    const int next_unit = unit + (int)gridDim.x;
    const bool has_next = next_unit < total;
    int nm0, nn0, nkb0, nexpert, nm_end;
    unit_origin(has_next ? next_unit : 0, nm0, nn0, nkb0, nexpert, nm_end);
    if (!has_next) {
      nm0 = MODE == PIPE_GROUPED ? p.M : p.tiles_m * BM;
      nn0 = p.tiles_n * BN;
    }
    const char* b_next = p.b;
    if constexpr (MODE == PIPE_GROUPED) b_next = p.b + (int64_t)nexpert * p.b_expert_stride;

    // (a unit has at least three K blocks, so its first, last-but-one and last step are distinct)
    const uint32_t off_a_next = a_offset(nm0), off_b_next = b_offset(nn0);
    uint32_t sc_off_next = SC_NONE;
    if constexpr (BLOCK) sc_off_next = scale_offset(nm0, nn0, nexpert);
    if constexpr (DIRECT) {
      if (unit == (int)blockIdx.x) k_step(par, kb0 + 1, kb0 + 2, std::true_type{}, std::false_type{}, std::false_type{});
      else k_step(par, kb0 + 1, kb0 + 2, std::true_type{}, std::false_type{}, std::true_type{});  // behind the last tile's stores
    } else {
      k_step(par, kb0 + 1, kb0 + 2, std::true_type{}, std::false_type{}, std::false_type{});
    }
    for (int kb = 1; kb + 1 < nkb; ++kb) {
      const bool pen = kb + 2 == nkb;  // the block two ahead is the next unit's first
      off_a2 = pen ? off_a_next : off_a2;
      off_b2 = pen ? off_b_next : off_b2;
      sc_off2 = pen ? sc_off_next : sc_off2;
      if constexpr (MODE == PIPE_GROUPED) b_two = pen ? b_next : b_two;
      k_step((kb + par) & 1, kb0 + kb + 1, pen ? nkb0 : kb0 + kb + 2, std::false_type{}, std::false_type{}, std::false_type{});
    }
    // last K block: its copies (the next unit's second block) wait for the next unit's first step
    // (PIPE_DIRECT: they are issued here like any other step's)
    const int last_stage = (nkb - 1 + par) & 1;
    if constexpr (DIRECT) k_step(last_stage, nkb0, nkb0 + 1, std::false_type{}, std::true_type{}, std::false_type{});
    else k_step(last_stage, 0, 0, std::false_type{}, std::true_type{}, std::false_type{});
    off_a = off_a2;
    off_b = off_b2;
    sc_off = sc_off2;
    if constexpr (MODE == PIPE_GROUPED) b_cur = b_two;

    // Every wave has passed the last step's barrier: nobody reads `last_stage` any more and
    // nothing is being copied into it, so it stages the C tile.
    if constexpr (DIRECT) {
      // (pin the accumulators here: left alone, the compiler sinks the last folds into the epilogue's blocks and
      // spills their operands across the step's tail)
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) asm volatile("" : "+v"(acc[i][j]));
      epilogue_direct<OUT_DT, MI, NI, BM, BN>(p, acc, smem + 2 * STAGE_BYTES + 2 * SCALE_BYTES + 2048 + wave * 2048, m0, n0, wm * TM, wn * TN, r16, g,
                                              lane);
    } else if constexpr (MODE == PIPE_SPLITK) {
      store_partials_bounded<MI, NI>(p, acc, unit / tiles, m0 + wm * TM, n0 + wn * TN, r16, g);
    } else if constexpr (KIND == KIND_I8_RAW) {
      epilogue<KIND, OUT_DT, MI, NI>(p, acc, m0 + wm * TM, n0 + wn * TN, r16, g);
    } else if constexpr (MODE == PIPE_GROUPED) {
      GemmArgs q = p;
      q.M = m_end;  // rows past the expert's last one belong to other experts
      epilogue_via_lds<KIND, OUT_DT, MI, NI, BN, false, BM / 2>(q, acc, smem + last_stage * STAGE_BYTES, col_lds, m0, n0, wm, wn, r16, g, lane, wave);
    } else {
      // (rows of 16-bit outputs are 16-byte aligned: checked on the host)
      epilogue_via_lds<KIND, OUT_DT, MI, NI, BN, MODE == PIPE_BIAS, BM / 2>(p, acc, smem + last_stage * STAGE_BYTES, col_lds, m0, n0, wm, wn, r16,
                                                                             g, lane, wave);
    }
    if (!has_next) break;
    unit = next_unit;
    m0 = nm0;
    n0 = nn0;
    kb0 = nkb0;
    expert = nexpert;
    m_end = nm_end;
    par = last_stage ^ 1;
    read_first(par);  // (landed before the last step's second barrier)
  }
  // (PIPE_DIRECT: the last step's copies, pointed beyond the operands, still write zeros into LDS)
  if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0);
}

// ---------------------------------------------------------------------------
// 256 x (32 NI) kernel, NI = 6, 7 or 8 (tile widths 192, 224, 256), K >= 384: the same
// persistent, pipelined two-stage structure as gemm_pipe_kernel with the roles of the
// operands exchanged.  The eight waves form a 4 (M) x 2 (N) grid; a wave keeps its four
// activation fragments of the K step in registers and streams its NI weight fragments one
// ahead.  The tile width is chosen on the host so that the tile count fills whole rounds of
// the chip's CUs: 7168 columns are 32 tiles of 224 (two full rounds at M = 4096) instead
// of 28 tiles of 256 (one full round and a 3/4 one).  A wave's columns can straddle two
// 128-column scale blocks: the K steps are instantiated per position of that boundary among the
// wave's fragments and the tile loop dispatches on it once per tile.  Here the
// activation half of a stage is the one that is free early (barrier 1, behind MFMA 3: all
// four activation fragments are in registers) and is refilled two K blocks ahead; the
// weight copies of block u + 2 follow behind the last weight fragment's MFMAs.
// ---------------------------------------------------------------------------
template <int KIND, int OUT_DT, int NI, bool BIAS, int MI = 4>
__global__ __launch_bounds__(512) void gemm_wide_kernel(const GemmArgs p) {
  // (MI = 3: tiles of 192 rows, for row counts that 256-row tiles cover with a part-empty round of the CUs)
  constexpr int BM = 64 * MI, NW = 8, WAVES_N = 2;
  constexpr int TM = MI * 16, TN = NI * 16, BN = WAVES_N * TN;
  constexpr int STAGE_BYTES = 512 * 128;  // stage pitch; only (BM + BN) rows are filled
  constexpr int NB = BN / 8;              // one-KiB weight copies per stage
  constexpr int NBW = (NB + NW - 1) / NW; // ... per wave (the last one only for waves < NB % 8)
  constexpr bool IS_FP8 = fp8_operands(KIND);
  constexpr bool BLOCK = is_block(KIND);
  constexpr bool HW = KIND == KIND_FP8_BLOCK_POW2;  // the MFMA applies the block scales
  constexpr bool FOLD = BLOCK && !HW;               // they are applied to each MFMA's result
  static_assert(NBW <= 4 && NBW <= MI && NI >= 4 && (MI == 4 || MI == 3), "copy and scale-load slots below assume this");

  constexpr int SCALE_BYTES = 2048;  // per K block: 256 activation-row scales, then up to three weight scales
  // (one LDS object per kernel, see gemm_big_kernel: the epilogue's 512 floats sit at the end)
  __shared__ __attribute__((aligned(1024))) char smem[2 * STAGE_BYTES + 2 * SCALE_BYTES + 2048];
  float* const col_lds = reinterpret_cast<float*>(smem + 2 * STAGE_BYTES + 2 * SCALE_BYTES);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int r16 = lane & 15, g = lane >> 4;

  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b, p.b_bytes);

  // Copy j of a wave fills activation rows 8 (wave + 8 j) .. + 7 of the stage, or the same
  // rows of the weight part; lane l brings row l / 8 of those, chunk (l % 8) ^ swz(row).
  // swz depends on l / 8 and the parity of the wave only, so a wave's copies share one
  // per-lane offset (lane_a / lane_b: the lane's row inside the tile and its chunk); the tile's
  // first row, the copy's multiple of 64 rows and the K offset travel in the scalar operand.
  // The buffer's range check covers the sum of both offsets: rows past M / N fall beyond the
  // extent and read as zero.  A weight copy past the tile's width (224-wide tiles: the fourth
  // copy of waves 4..7) is sent out of range as well and zero-fills stage rows that nobody reads.
  const int l8 = lane >> 3;
  const int c16 = (((lane & 7) ^ l8 ^ (wave & 1)) & 7) * 16;
  const uint32_t row_in_tile = (uint32_t)(wave * 8 + l8);
  const uint32_t lane_a = row_in_tile * p.lda + c16, lane_b = row_in_tile * p.ldb + c16;
  const uint32_t step_a = 64u * p.lda, step_b = 64u * p.ldb;
  const bool last_b_ok = wave + (NBW - 1) * NW < NB;
  // off_a / off_b: tile of the block after the current one (copies deferred to a tile's first
  // step); off_a2 / off_b2: tile of the block two after the current one.  Scalars: byte offset
  // of the tile's first row.
  uint32_t off_a = 0, off_a2 = 0, off_b = 0, off_b2 = 0;
  auto copy_a = [&](int j, int stage, int k0, uint32_t off) {
    char* dst = smem + stage * STAGE_BYTES + (wave + j * NW) * 1024;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (__attribute__((address_space(3))) void*)dst, 16, lane_a,
                                             off + (uint32_t)j * step_a + (uint32_t)k0, 0, 0);
  };
  auto copy_b = [&](int j, int stage, int k0, uint32_t off_tile) {
    char* dst = smem + stage * STAGE_BYTES + BM * 128 + (wave + j * NW) * 1024;
    uint32_t off = off_tile + (uint32_t)j * step_b + (uint32_t)k0;
    if (j == NBW - 1 && NB % NW != 0) off = last_b_ok ? off : OOB;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void*)dst, 16, lane_b, off, 0, 0);
  };
  // (a tile past the last one: any offset beyond the extents; the sum with a lane's offset stays below 2^32)
  auto a_offset = [&](int m0) { return m0 < p.M ? (uint32_t)m0 * p.lda : OOB; };
  auto b_offset = [&](int n0) { return n0 < p.N ? (uint32_t)n0 * p.ldb : OOB; };

  const int sw = (r16 & 7) ^ (r16 >> 3);
  const int lane_off0 = r16 * 128 + (((2 * g) ^ sw) * 16);
  const int lane_off1 = lane_off0 ^ 16;
  const int a_base = (wm * TM) * 128;
  const int b_base = (BM + wn * TN) * 128;
  auto read_frag = [&](const char* q) -> v8i {
    v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
    v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  using acc_t = typename std::conditional<float_acc(KIND), v4f, v4i>::type;
  acc_t acc[MI][NI];
  v8i af[MI];  // the step's activation fragments
  v8i b_cur;   // the weight fragment the next MFMAs use

  // Block scales.  Row m of K block kb sits at sfa[m * stride_m + kb * stride_k]; a lane owns
  // row r16 of each of the wave's 16-row activation fragments.  Every wave issues one
  // 4-byte-per-lane copy per K block: waves 0..3 the activation scales of tile rows
  // 64 w + lane, wave 4 the weight scales of the (up to three) 128-column blocks the tile
  // touches (lanes 0..2), waves 5..7 nothing (all lanes out of range; kept so that the
  // instruction stream has no branch).  lane_s: the lane's offset inside a tile's scales;
  // sc_off / sc_off2 (scalars): those of the tile of block u + 1 / u + 2.  Rows past M and
  // column blocks past N are not singled out: what they read (a value inside the scale tensor,
  // or zero beyond it) only reaches outputs that the epilogue drops.  The wave's weight fragments 0 .. jsw - 1 lie in scale
  // block sb_lo of the tile's blocks, the others in sb_lo + 1.
  const int nkb = p.K >> 7;
  float sfa_cur[MI];
  float sfb_lo = 0.f, sfb_hi = 0.f;
  __amdgpu_buffer_rsrc_t rsc = ra;
  uint32_t lane_s = OOB, sc_off = SC_NONE, sc_off2 = SC_NONE;
  int sc_step = 0, jsw = NI;
  // jsw / sfb read offset of the tile whose scales are read next (two tiles can be in flight:
  // the values for the tile of block u + 1 are needed when its scales are read)
  int jsw_nxt = NI, sfb_rd_nxt = 0;
  const int sc_dst = 2 * STAGE_BYTES + wave * 256;  // waves 5..7 land behind the used part
  const int sfa_rd = 2 * STAGE_BYTES + (wm * TM + r16) * 4;
  if constexpr (BLOCK) {
    const int nblocks = (p.N + 127) >> 7;
    const int sa_last = (HW && p.sa_packed) ? (nkb - 1) >> 2 : nkb - 1;  // (packed: words of four K blocks)
    const int64_t sfa_elems = (int64_t)(p.M - 1) * p.sa_stride_m + (int64_t)sa_last * p.sa_stride_k + 1;
    const int64_t sfb_elems = (int64_t)(nblocks - 1) * p.sb_stride_n + (int64_t)(nkb - 1) * p.sb_stride_k + 1;
    rsc = wave < 4 ? make_rsrc(p.sa, (uint32_t)(sfa_elems * 4)) : make_rsrc(p.sb, (uint32_t)(sfb_elems * 4));
    sc_step = (int)((wave < 4 ? p.sa_stride_k : p.sb_stride_k) * 4);
    if (wave < 4) lane_s = wave * 64 < BM ? (uint32_t)((wave * 64 + lane) * p.sa_stride_m * 4) : OOB;
    else lane_s = (wave == 4 && lane < 3) ? (uint32_t)(lane * p.sb_stride_n * 4) : OOB;
  }
  // (SC_NONE: no tile; beyond both scale tensors, and its sum with OOB does not wrap)
  auto scale_offset = [&](int m0, int n0) -> uint32_t {
    if (m0 >= p.M || n0 >= p.N) return SC_NONE;
    if (wave < 4) return (uint32_t)(m0 * p.sa_stride_m * 4);
    return (uint32_t)((n0 >> 7) * p.sb_stride_n * 4);
  };
  // where this wave's columns start inside the tile's scale blocks
  auto set_scale_split = [&](int n0) {
    const int nw = n0 + wn * TN;
    const int nb_lo = nw >> 7;
    jsw_nxt = __builtin_amdgcn_readfirstlane(((nb_lo + 1) * 128 - nw) >> 4);
    sfb_rd_nxt = __builtin_amdgcn_readfirstlane(2 * STAGE_BYTES + 1024 + (nb_lo - (n0 >> 7)) * 4);
  };
  // (packed activation scales: this wave's copy of K block kb fetches the word of K blocks 4 (kb / 4) .. + 3)
  const int sc_kshift = (HW && p.sa_packed && wave < 4) ? 2 : 0;
  const bool sa_packed = HW && p.sa_packed;
  auto code_shift = [&](int kb) { return sa_packed ? 8 * (kb & 3) : 23; };
  int sh_cur = 23;  // where the UE8M0 code of the K block in sfa_cur sits inside its word
  auto copy_scales = [&](int buf, int kb, uint32_t off) {
    char* dst = smem + buf * SCALE_BYTES + sc_dst;
    const int kw = HW ? kb >> sc_kshift : kb;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsc, (__attribute__((address_space(3))) void*)dst, 4, lane_s, (uint32_t)(kw * sc_step) + off, 0,
                                             0);
  };
  auto read_sfa = [&](int buf, int i) -> float {
    return *reinterpret_cast<const float*>(smem + buf * SCALE_BYTES + sfa_rd + i * 64);
  };
  auto read_sfb = [&](int buf, int which) -> float {
    return *reinterpret_cast<const float*>(smem + buf * SCALE_BYTES + sfb_rd_nxt + which * 4);
  };

  // One K step: block u sits in stage `cur`, its activation fragments and first weight
  // fragment are in af / b_cur.  kn: index, inside its tile, of block u + 1 (the copies
  // deferred to a tile's first step); kn2: that of block u + 2 (off_a2 / off_b2).
  auto k_step = [&](int cur, int kn, int kn2, auto first_tag, auto last_tag, auto jsw_tag) __attribute__((always_inline)) {
    constexpr bool first = decltype(first_tag)::value;
    constexpr bool last = decltype(last_tag)::value;
    // Fragments j < JSW of this wave lie in the tile's scale block sb_lo, the others in sb_lo + 1.  JSW is a
    // compile-time constant here (the tile loop below dispatches on it once per tile): the scale of fragment
    // (i, j), sfa[i] * sfb of j's block, then takes 8 multiplies per K step and no selects instead of one
    // multiply and one select per MFMA.  The VALU port also issues the MFMAs and the folds and is the scarce
    // resource of this loop: with 28 multiplies and 8 selects fewer per step the launch is 5 % shorter.
    constexpr int JSW = decltype(jsw_tag)::value;
    const char* st = smem + cur * STAGE_BYTES;
    const char* sn = smem + (cur ^ 1) * STAGE_BYTES;
    float sc = 0.f, sc_prev = 0.f;
    float scv[MI] = {};  // sfa[i] * sfb of the scale block of the fragments being multiplied
    if constexpr (FOLD) {
#pragma unroll
      for (int i = 0; i < MI; ++i) scv[i] = sfa_cur[i] * sfb_lo;
    }
    // HW: the exponent bytes of the fragments' activation scales (per lane: its row) and of the two weight scales
    // (HW runs one instantiation of the step for every position of the boundary, JSW = NI, and selects per
    // fragment at run time: instantiated per position like the other block kinds, the accumulators change
    // registers between the instantiations and the kernel spills)
    int ea[MI] = {};
    const int eb_lo = HW ? ue8m0_of(sfb_lo) : 0, eb_hi = HW ? ue8m0_of(sfb_hi) : 0;
    const int jsw_now = jsw;
    if constexpr (HW) {
#pragma unroll
      for (int i = 0; i < MI; ++i) ea[i] = ue8m0_at(sfa_cur[i], sh_cur);
    }
    v4f part_prev = {0.f, 0.f, 0.f, 0.f};
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      v8i b_nxt = b_cur;
      if constexpr (FOLD) {
        if (j == JSW) {  // (compile-time: no branch) the fragments from here on lie in the next scale block
#pragma unroll
          for (int i = 0; i < MI; ++i) scv[i] = sfa_cur[i] * sfb_hi;
        }
      }
      if (j == 1 && !last) {
        // barrier 1: MFMAs 0..3 have consumed this wave's activation fragments, so its LDS
        // reads of block u's activations are complete; behind the barrier that holds for
        // every wave and the activation half of the stage is free.
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
      if (j == NI - 1) {
        // barrier 2.  Vector-memory operations retire in order; block u + 1's last copy is a
        // weight copy behind the last MFMAs of the step before (or a deferred one behind MFMA
        // 11 of a tile's first step).  Younger than it are only the four activation copies of
        // block u + 2, which stay in flight.  lgkmcnt(0): this wave's LDS reads of block u's
        // weights and scales are complete.  A bare s_barrier: these waits are all the
        // ordering that is needed.
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(last ? 0 : MI));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int idx = j * MI + i;
        v4f part = {0.f, 0.f, 0.f, 0.f};
        if constexpr (FOLD) {
          part = block_mfma<KIND>(b_cur, af[i]);
        } else if constexpr (HW) {
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b_cur, af[i], acc[i][j], 0, 0, 0, j < jsw_now ? eb_lo : eb_hi, 0, ea[i]);
        } else if constexpr (KIND == KIND_FP8_ROWCOL) {
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b_cur, af[i], acc[i][j], 0, 0, 0, 0, 0, 0);
        } else {
          const v4i b0 = {b_cur[0], b_cur[1], b_cur[2], b_cur[3]};
          const v4i a0 = {af[i][0], af[i][1], af[i][2], af[i][3]};
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b0, a0, acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!IS_FP8 && !BLOCK) {
          const v4i b1 = {b_cur[4], b_cur[5], b_cur[6], b_cur[7]};
          const v4i a1 = {af[i][4], af[i][5], af[i][6], af[i][7]};
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b1, a1, acc[i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (FOLD) {
          sc_prev = sc;
          sc = scv[i];
        }
        if (j + 1 < NI) {
          if (i == 0) b_nxt = read_frag(st + b_base + (j + 1) * 16 * 128);
        } else {
          // activation fragment i has had its last use in this step: refill it from block u + 1
          af[i] = read_frag(sn + a_base + i * 16 * 128);
          if (i == 0) b_nxt = read_frag(sn + b_base);
          if (!last && i < NBW) copy_b(i, cur, kn2 * 128, off_b2);
          if constexpr (BLOCK) {
            // so has its scale (`sc` holds the product), and the weight scales (`sfb_j`)
            sfa_cur[i] = read_sfa(cur ^ 1, i);
            if (i == 0) sfb_lo = read_sfb(cur ^ 1, 0);
            if (i == 1) sfb_hi = read_sfb(cur ^ 1, 1);
            if (i == 0 && !last) copy_scales(cur, kn2, sc_off2);
          }
        }
        if constexpr (first) {
          if (idx >= 4 && idx < 4 + MI) copy_a(idx - 4, cur ^ 1, kn * 128, off_a);
          if (idx >= 8 && idx < 8 + NBW) copy_b(idx - 8, cur ^ 1, kn * 128, off_b);
          if (BLOCK && idx == 11) copy_scales(cur ^ 1, kn, sc_off);
          if (idx >= 12 && idx < 12 + MI) copy_a(idx - 12, cur, kn2 * 128, off_a2);
        } else if constexpr (!last) {
          if (idx >= 4 && idx < 4 + MI) copy_a(idx - 4, cur, kn2 * 128, off_a2);
        }
        if constexpr (FOLD) {
          if (idx > 0) {  // scale-and-accumulate the previous MFMA's result while this one runs
            const int pj = (idx - 1) / MI, pi = (idx - 1) % MI;
            acc[pi][pj][0] = __builtin_fmaf(block_value<KIND>(part_prev[0]), sc_prev, acc[pi][pj][0]);
            acc[pi][pj][1] = __builtin_fmaf(block_value<KIND>(part_prev[1]), sc_prev, acc[pi][pj][1]);
            acc[pi][pj][2] = __builtin_fmaf(block_value<KIND>(part_prev[2]), sc_prev, acc[pi][pj][2]);
            acc[pi][pj][3] = __builtin_fmaf(block_value<KIND>(part_prev[3]), sc_prev, acc[pi][pj][3]);
          }
          part_prev = part;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      b_cur = b_nxt;
    }
    if constexpr (FOLD) {
      acc[MI - 1][NI - 1][0] = __builtin_fmaf(block_value<KIND>(part_prev[0]), sc, acc[MI - 1][NI - 1][0]);
      acc[MI - 1][NI - 1][1] = __builtin_fmaf(block_value<KIND>(part_prev[1]), sc, acc[MI - 1][NI - 1][1]);
      acc[MI - 1][NI - 1][2] = __builtin_fmaf(block_value<KIND>(part_prev[2]), sc, acc[MI - 1][NI - 1][2]);
      acc[MI - 1][NI - 1][3] = __builtin_fmaf(block_value<KIND>(part_prev[3]), sc, acc[MI - 1][NI - 1][3]);
    }
    if constexpr (BLOCK) jsw = jsw_nxt;
    if constexpr (HW) sh_cur = code_shift(kn);  // sfa_cur now holds block u + 1's words (a tile's last step: the next tile's block 0)
  };

  // ---- persistent walk over the tiles blockIdx, blockIdx + gridDim, ...
  const int total = p.tiles_m * p.tiles_n;
  int tile = blockIdx.x;
  int tm, tn;
  tile_of_block(tile, p.tiles_m, p.tiles_n, tm, tn);
  int m0 = tm * BM, n0 = tn * BN;
  int par = 0;  // stage that holds K block 0 of the current tile

  off_a = off_a2 = a_offset(m0);
  off_b = off_b2 = b_offset(n0);
  if constexpr (BLOCK) {
    sc_off = sc_off2 = scale_offset(m0, n0);
    set_scale_split(n0);
  }
#pragma unroll
  for (int j = 0; j < MI; ++j) copy_a(j, 0, 0, off_a);
#pragma unroll
  for (int j = 0; j < NBW; ++j) copy_b(j, 0, 0, off_b);
  if constexpr (BLOCK) copy_scales(0, 0, sc_off);
  __builtin_amdgcn_s_waitcnt(0);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < MI; ++i) af[i] = read_frag(smem + a_base + i * 16 * 128);
  b_cur = read_frag(smem + b_base);
  if constexpr (BLOCK) {
#pragma unroll
    for (int i = 0; i < MI; ++i) sfa_cur[i] = read_sfa(0, i);
    sfb_lo = read_sfb(0, 0);
    sfb_hi = read_sfb(0, 1);
    jsw = jsw_nxt;
    if constexpr (HW) sh_cur = code_shift(0);
  }

  while (true) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

    // The block's next tile; past its last tile the prefetches are pointed at rows beyond M
    // and N, which the buffer bounds turn into zero fill without memory traffic.
    const int next_tile = tile + (int)gridDim.x;
    const bool has_next = next_tile < total;
    tile_of_block(has_next ? next_tile : 0, p.tiles_m, p.tiles_n, tm, tn);
    const int nm0 = has_next ? tm * BM : p.tiles_m * BM;
    const int nn0 = has_next ? tn * BN : p.tiles_n * BN;

    // (K >= 384 for this kernel, so the first, the last-but-one and the last step are distinct)
    const uint32_t off_a_next = a_offset(nm0), off_b_next = b_offset(nn0);
    uint32_t sc_off_next = SC_NONE;
    if constexpr (BLOCK) sc_off_next = scale_offset(nm0, nn0);
    const int last_stage = (nkb - 1 + par) & 1;
    // the tile's K steps, instantiated for the position of the scale-block boundary among this wave's fragments
    auto tile_steps = [&](auto jsw_tag) __attribute__((always_inline)) {
      k_step(par, 1, 2, std::true_type{}, std::false_type{}, jsw_tag);
      for (int kb = 1; kb + 1 < nkb; ++kb) {
        const bool pen = kb + 2 == nkb;  // the block two ahead is the next tile's first
        off_a2 = pen ? off_a_next : off_a2;
        off_b2 = pen ? off_b_next : off_b2;
        sc_off2 = pen ? sc_off_next : sc_off2;
        k_step((kb + par) & 1, kb + 1, pen ? 0 : kb + 2, std::false_type{}, std::false_type{}, jsw_tag);
      }
      // last K block: the scales read behind its last MFMAs are the next tile's; its copies (the
      // next tile's second block) wait for the next tile's first step
      if constexpr (BLOCK) set_scale_split(nn0);
      k_step(last_stage, 0, 0, std::false_type{}, std::true_type{}, jsw_tag);
    };
    if constexpr (!BLOCK || NI == 8 || HW) {
      tile_steps(std::integral_constant<int, NI>{});  // (256-wide tiles: a wave's 128 columns are one scale block)
    } else if constexpr (NI == 6) {
      // 192-wide tiles start at multiples of 64 columns: the boundary is behind fragment 2, 4 or 6 (= none)
      if (jsw == 2) tile_steps(std::integral_constant<int, 2>{});
      else if (jsw == 4) tile_steps(std::integral_constant<int, 4>{});
      else tile_steps(std::integral_constant<int, 6>{});
    } else {
      // 224-wide tiles start at multiples of 32 columns, their second wave 112 columns later: any position
      switch (jsw) {
        case 1: tile_steps(std::integral_constant<int, 1>{}); break;
        case 2: tile_steps(std::integral_constant<int, 2>{}); break;
        case 3: tile_steps(std::integral_constant<int, 3>{}); break;
        case 4: tile_steps(std::integral_constant<int, 4>{}); break;
        case 5: tile_steps(std::integral_constant<int, 5>{}); break;
        case 6: tile_steps(std::integral_constant<int, 6>{}); break;
        default: tile_steps(std::integral_constant<int, 7>{}); break;
      }
    }
    off_a = off_a2;
    off_b = off_b2;
    sc_off = sc_off2;

    // Every wave has passed the last step's barrier: nobody reads `last_stage` any more and
    // nothing is being copied into it, so it stages the C tile.
    if constexpr (KIND == KIND_I8_RAW) {
      epilogue<KIND, OUT_DT, MI, NI>(p, acc, m0 + wm * TM, n0 + wn * TN, r16, g);
    } else {
      // (rows of 16-bit outputs are 16-byte aligned: checked on the host)
      epilogue_via_lds<KIND, OUT_DT, MI, NI, BN, BIAS, MI == 4 ? 128 : 64, MI == 4 ? 2 : 3>(p, acc, smem + last_stage * STAGE_BYTES, col_lds, m0, n0, wm, wn, r16, g, lane, wave);
    }
    if (!has_next) break;
    tile = next_tile;
    m0 = nm0;
    n0 = nn0;
    par = last_stage ^ 1;
  }
}

// ---------------------------------------------------------------------------
// Decode kernel (M <= 64): the weight matrix is streamed once from HBM, so the
// job is to keep enough bytes in flight.  A block owns 128 weight rows and a
// contiguous range of K blocks (split-K across blocks); its four waves take 32
// rows each.  Weight tiles (16 KiB), the activation tile and, for the block-scaled
// kind, the activation scales of each K block are copied global -> LDS through a
// ring of NSTAGE stages (80-100 KiB in flight per CU); a K block's fragments are read
// from LDS into registers one step before its MFMAs, so the block's stage is free for
// the copy NSTAGE blocks ahead as soon as the step starts, and the LDS reads, the
// copies and the scale-and-accumulate of each MFMA's result overlap the MFMAs (a block
// may be alone on its CU, one wave per SIMD).  All copies of a stage are vector-memory
// loads that retire in order, so "stage t has landed" is a vmcnt wait that leaves the
// younger stages' loads outstanding.  With splits > 1 the partial sums go to a workspace and
// splitk_reduce_kernel applies the epilogue.  For 64 < M <= 512 there are several 64-row
// tiles per weight tile; they run side by side on one XCD, so the weights still come from
// HBM once and from that XCD's L2 after that.
// ---------------------------------------------------------------------------
template <int KIND, int MI, int OUT_DT, int BN = 128>
// (two waves per SIMD asked for: with at most 256 registers per lane the MFMAs write plain
// VGPRs; given 512 the compiler puts their results into accumulation registers and copies
// each one out behind a full MFMA latency of wait states)
__global__ __launch_bounds__(256, 2) void gemm_skinny_kernel(const GemmArgs p) {
  static_assert(BN == 128 || BN == 64, "a wave takes 32 or 16 of the block's weight rows");
  constexpr int NI = BN / 64;
  constexpr int WCW = BN / 32;                     // weight copies per wave per stage
  constexpr int AR = MI * 16 < 32 ? 32 : MI * 16;  // activation rows staged (at least one copy per wave)
  constexpr int ACW = AR / 32;                     // activation copies per wave per stage
  constexpr bool BLOCK = is_block(KIND);
  constexpr int CPW = WCW + ACW + (BLOCK ? 2 : 0);  // vector-memory loads per wave per stage
  constexpr int W_BYTES = BN * 128, A_BYTES = AR * 128, S_BYTES = BLOCK ? 2048 : 0;  // 4 x 256 B of activation scales, then the weight scale
  constexpr int STAGE_BYTES = W_BYTES + A_BYTES + S_BYTES;
  // 60-78 KiB of LDS: two blocks (eight waves) per CU.  A ring of six stages (one block per CU,
  // five stages in flight) is slower wherever it was tried, also for launches of fewer blocks than
  // CUs whose blocks walk 56 K blocks each (64 x 2048 x 7168 without split-K: 29.5 us with three stages,
  // 32.9 with six): what a CU's load path delivers sets the step time, not the depth of the ring.
  constexpr int NSTAGE = BN == 64 ? 4 : 3;
  constexpr bool IS_FP8 = fp8_operands(KIND);

  __shared__ __attribute__((aligned(1024))) char smem[NSTAGE * STAGE_BYTES];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4, l8 = lane >> 3;

  // Block id -> (weight tile and split, row tile): the row tiles of one weight tile get ids 8 apart
  // inside a group of eight weight tiles, so they are dispatched together and (blocks go to the
  // eight XCDs round-robin) to the same XCD: its L2 serves the weight tile's second reader.
  const int cols = p.tiles_n * p.splits;
  const int group = (int)blockIdx.x / (8 * p.tiles_m);
  const int in_group = (int)blockIdx.x - group * 8 * p.tiles_m;
  const int width = cols - group * 8 < 8 ? cols - group * 8 : 8;
  const int col = group * 8 + in_group % width;
  const int tile_n = col % p.tiles_n, split = col / p.tiles_n;
  const int n0 = tile_n * BN;
  const int m_base = (in_group / width) * 64;
  const int nkb = p.K >> 7;
  // Split s takes the K blocks s, s + splits, s + 2 splits, ...: the blocks that share a
  // weight tile then read neighbouring 128-byte pieces of the same rows at about the same
  // time, which keeps DRAM pages open longer than giving each split one contiguous K range.
  const int kb0 = split, kstride = p.splits;
  const int nsteps = (nkb - split + p.splits - 1) / p.splits;

  const v4u ra = make_rsrc_sgpr(p.a, p.a_bytes);
  const v4u rb = make_rsrc_sgpr(p.b, p.b_bytes);
  v4u rs = ra, rsb = ra;

  // Same copy plan as the prefill kernel: lane l brings row l / 8 of an 8-row
  // group, chunk (l % 8) ^ swz(row); copies of one wave differ by 32 rows.
  const int c16 = (((lane & 7) ^ l8 ^ (wave & 1)) & 7) * 16;
  const uint32_t off_w = (uint32_t)(n0 + wave * 8 + l8) * p.ldb + c16;
  const uint32_t off_a = (uint32_t)(m_base + wave * 8 + l8) * p.lda + c16;
  const uint32_t step_w = 32u * p.ldb, step_a = 32u * p.lda;
  uint32_t off_s = 0, off_sb = OOB;
  int sfa_step = 0, sfb_step = 0;
  if constexpr (BLOCK) {
    const int64_t sfa_elems = (int64_t)(p.M - 1) * p.sa_stride_m + (int64_t)(nkb - 1) * p.sa_stride_k + 1;
    rs = make_rsrc_sgpr(p.sa, (uint32_t)(sfa_elems * 4));
    off_s = m_base + lane < p.M ? (uint32_t)((m_base + lane) * p.sa_stride_m * 4) : OOB;  // lane = activation row of the tile
    sfa_step = (int)(p.sa_stride_k * 4);
    // the weight scale of the block's 128 weight rows travels with every stage as well: one
    // dword, brought by lane 0 of wave 0 (the other lanes and waves are out of range; the
    // instruction stays so that every wave counts the same number of copies per stage)
    const int nblocks = (p.N + 127) >> 7;
    const int nb = (n0 >> 7) < nblocks ? (n0 >> 7) : nblocks - 1;
    const int64_t sfb_elems = (int64_t)(nblocks - 1) * p.sb_stride_n + (int64_t)(nkb - 1) * p.sb_stride_k + 1;
    rsb = make_rsrc_sgpr(p.sb, (uint32_t)(sfb_elems * 4));
    off_sb = (wave == 0 && lane == 0) ? (uint32_t)(nb * p.sb_stride_n * 4) : OOB;
    sfb_step = (int)(p.sb_stride_k * 4);
  }

  const uint32_t smem_base = lds_addr(smem);
  auto issue_group = [&](int t) {  // all copies of K block kb0 + t into stage t % NSTAGE
    const uint32_t st = smem_base + (uint32_t)(t % NSTAGE) * STAGE_BYTES;
    const uint32_t k0 = (uint32_t)(kb0 + t * kstride) * 128u;
#pragma unroll
    for (int j = 0; j < WCW; ++j) lds_copy16(rb, st + (wave + 4 * j) * 1024, off_w + j * step_w, k0);
#pragma unroll
    for (int j = 0; j < ACW; ++j) lds_copy16(ra, st + W_BYTES + (wave + 4 * j) * 1024, off_a + j * step_a, k0);
    // one dword per lane: its row's activation scale for this K block
    if constexpr (BLOCK) {
      lds_copy4(rs, st + W_BYTES + A_BYTES + wave * 256, off_s, (uint32_t)((kb0 + t * kstride) * sfa_step));
      lds_copy4(rsb, st + W_BYTES + A_BYTES + 1024 + wave * 256, off_sb, (uint32_t)((kb0 + t * kstride) * sfb_step));
    }
  };

  const int sw = (r16 & 7) ^ (r16 >> 3);
  const int lane_off0 = r16 * 128 + (((2 * g) ^ sw) * 16);
  const int lane_off1 = lane_off0 ^ 16;
  auto read_frag = [&](const char* q) -> v8i {
    v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
    v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  using acc_t = typename std::conditional<float_acc(KIND), v4f, v4i>::type;
  acc_t acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

  // Every stage of the ring is filled before the first MFMA; after that, step t runs on the
  // fragments of K block t that step t - 1 read from LDS into registers, and while its MFMAs
  // run it reads the fragments of block t + 1 and refills block t's stage with block t + NSTAGE.
  // Two register sets take turns (the loop below is unrolled by two), so nothing is moved.
  struct Frags {
    v8i f[NI + MI];  // weight fragments, then activation fragments
    float sa[MI], sb;
  };
  Frags fa, fb;
  auto read_one = [&](int t, Frags& d, int k) {  // k-th LDS read group of K block t
    const char* st = smem + (t % NSTAGE) * STAGE_BYTES;
    if (k < NI) d.f[k] = read_frag(st + (wave * (BN / 4) + k * 16) * 128);
    else if (k < NI + MI) d.f[k] = read_frag(st + W_BYTES + (k - NI) * 16 * 128);
    else if constexpr (BLOCK) {
      d.sb = *reinterpret_cast<const float*>(st + W_BYTES + A_BYTES + 1024);
      const float* sfa = reinterpret_cast<const float*>(st + W_BYTES + A_BYTES + wave * 256);
#pragma unroll
      for (int i = 0; i < MI; ++i) d.sa[i] = sfa[i * 16 + r16];
    }
  };
  constexpr int NREAD = NI + MI + 1;
  // "K block u has landed" with the blocks up to u + younger issued: copies retire in order
  static_assert((NSTAGE - 1) * CPW < 64, "vmcnt holds six bits");
  static_assert(NSTAGE <= 4, "wait_landed counts at most three younger blocks");
  auto wait_landed = [&](int younger) {
    if (younger >= 3) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(3 * CPW));
    else if (younger == 2) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(2 * CPW));
    else if (younger == 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(CPW));
    else __builtin_amdgcn_s_waitcnt(0);
  };

  auto step = [&](int t, Frags& cur, Frags& nxt) {
    // Block t + 1 has landed (the blocks up to t + NSTAGE - 1 are issued), and this wave's LDS
    // reads of block t are complete; behind the barrier both hold for every wave, so block t's
    // stage can be refilled.
    const int issued = t + NSTAGE - 1 < nsteps - 1 ? t + NSTAGE - 1 : nsteps - 1;
    wait_landed(issued - (t + 1));
    __builtin_amdgcn_s_barrier();
    if (t + NSTAGE < nsteps) issue_group(t + NSTAGE);
    float sc[MI];
    if constexpr (BLOCK) {
#pragma unroll
      for (int i = 0; i < MI; ++i) sc[i] = cur.sa[i] * cur.sb;
    }
    __builtin_amdgcn_sched_barrier(0);
    constexpr int NMFMA = MI * NI;
    // the result of MFMA idx is folded into the accumulator while MFMA idx + 1 runs
    v4f part[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int idx = 0; idx < NMFMA; ++idx) {
      const int i = idx / NI, j = idx % NI;
      if constexpr (BLOCK) {
        part[idx & 1] = block_mfma<KIND>(cur.f[j], cur.f[NI + i]);
      } else if constexpr (KIND == KIND_FP8_ROWCOL) {
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(cur.f[j], cur.f[NI + i], acc[i][j], 0, 0, 0, 0, 0, 0);
      } else {
        const v8i &w = cur.f[j], &a = cur.f[NI + i];
        const v4i b0 = {w[0], w[1], w[2], w[3]}, b1 = {w[4], w[5], w[6], w[7]};
        const v4i a0 = {a[0], a[1], a[2], a[3]}, a1 = {a[4], a[5], a[6], a[7]};
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b0, a0, acc[i][j], 0, 0, 0);
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b1, a1, acc[i][j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      // the LDS reads of block t + 1 are spread over the MFMAs (after the last block: of a stage
      // that holds an older block, unused)
#pragma unroll
      for (int k = 0; k < NREAD; ++k)
        if (k * NMFMA / NREAD == idx) read_one(t + 1, nxt, k);
      if constexpr (BLOCK) {
        if (idx > 0) {
          const int pi = (idx - 1) / NI, pj = (idx - 1) % NI;
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[pi][pj][e] = __builtin_fmaf(block_value<KIND>(part[(idx - 1) & 1][e]), sc[pi], acc[pi][pj][e]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (BLOCK) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        acc[MI - 1][NI - 1][e] = __builtin_fmaf(block_value<KIND>(part[(NMFMA - 1) & 1][e]), sc[MI - 1], acc[MI - 1][NI - 1][e]);
    }
  };

#pragma unroll
  for (int t = 0; t < NSTAGE; ++t)
    if (t < nsteps) issue_group(t);
  wait_landed(nsteps - 1 < NSTAGE - 1 ? nsteps - 1 : NSTAGE - 1);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int k = 0; k < NREAD; ++k) read_one(0, fa, k);

  for (int t = 0; t < nsteps; t += 2) {
    step(t, fa, fb);
    if (t + 1 < nsteps) step(t + 1, fb, fa);
  }

  if (p.splits == 1) epilogue<KIND, OUT_DT, MI, NI>(p, acc, m_base, n0 + wave * (BN / 4), r16, g);
  else store_partials<MI, NI>(p, acc, split, m_base, n0 + wave * (BN / 4), r16, g);
}

// ---------------------------------------------------------------------------
// Decode kernel for M <= 32 (M <= 64 with 16-row blocks) and N large enough to give every CU a block without
// splitting K across blocks: a block owns BN = 16 NIB weight rows and the whole of K; its
// four waves take the K blocks w, w + 4, w + 8, ... and add their partial sums through LDS
// at the end, so no workspace and no second launch are needed.  Every wave has a ring of
// NSTAGE stages of its own (weight rows, activation rows, activation scales and the weight
// scale of one K block), filled by global -> LDS copies that it issues and waits for itself:
// the loop has no barrier, and 4 x (NSTAGE - 1) stages are in flight per block.  A wave's
// copies retire in order, so "my stage t has landed" is a vmcnt wait that leaves the
// NSTAGE - 1 younger stages outstanding; past the wave's last K block the copies are pointed
// out of range (zero fill, no memory traffic), which keeps that count constant.
// ---------------------------------------------------------------------------
template <int KIND, int MI, int NIB, int OUT_DT, bool ROW_TILES = false>
__global__ __launch_bounds__(256) void gemm_stream_kernel(const GemmArgs p) {
  constexpr int BN = NIB * 16, AR = MI * 16;
  constexpr bool BLOCK = is_block(KIND);
  constexpr bool IS_FP8 = fp8_operands(KIND);
  constexpr int WC = BN / 8, AC = AR / 8;          // one-KiB copies per stage: weights, activations
  constexpr int CPW = WC + AC + (BLOCK ? 2 : 0);   // vector-memory loads per stage
  constexpr int W_BYTES = BN * 128, A_BYTES = AR * 128, S_BYTES = BLOCK ? 512 : 0;
  constexpr int STAGE_BYTES = W_BYTES + A_BYTES + S_BYTES;
  // (64 x 64 tiles: two stages of 16.5 KiB per wave, 132 KiB per block)
  constexpr int NSTAGE = MI * NIB >= 16 ? 2 : SGLQ_STREAM_NSTAGE;
  constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;
  static_assert((NSTAGE - 1) * CPW <= 63, "vmcnt holds 6 bits");
  static_assert(MI * NIB * 1024 <= RING_BYTES, "the partial sums are exchanged through a wave's ring");
  static_assert(4 * RING_BYTES <= 160 * 1024, "LDS of one CU");

  __shared__ __attribute__((aligned(1024))) char smem[4 * RING_BYTES];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4, l8 = lane >> 3;
  // ROW_TILES (M > 64): a second grid dimension of 64-row tiles.  The row tiles of one weight tile get block ids
  // 8 apart inside a group of eight weight tiles, so they are dispatched together and (blocks go to the eight
  // XCDs round-robin) to the same XCD, whose L2 serves the weight tile's later readers.
  int n0 = blockIdx.x * BN, m_base = 0;
  if constexpr (ROW_TILES) {
    const int group = (int)blockIdx.x / (8 * p.tiles_m);
    const int in_group = (int)blockIdx.x - group * 8 * p.tiles_m;
    const int width = p.tiles_n - group * 8 < 8 ? p.tiles_n - group * 8 : 8;
    n0 = (group * 8 + in_group % width) * BN;
    m_base = (in_group / width) * AR;
  }
  const int nkb = p.K >> 7;
  const int nsteps = (nkb - wave + 3) >> 2;  // K blocks wave, wave + 4, ...

  const v4u ra = make_rsrc_sgpr(p.a, p.a_bytes);
  const v4u rb = make_rsrc_sgpr(p.b, p.b_bytes);
  v4u rsa = ra, rsb = ra;

  // Copy gj brings rows 8 gj .. 8 gj + 7 of the operand: lane l row l / 8, chunk (l % 8) ^ swz(row),
  // swz(row) = (row & 7) ^ ((row >> 3) & 1) = (l / 8) ^ (gj & 1).
  const int c16_even = (((lane & 7) ^ l8) & 7) * 16, c16_odd = (((lane & 7) ^ l8 ^ 1) & 7) * 16;
  const uint32_t offw_even = (uint32_t)(n0 + l8) * p.ldb + c16_even, offw_odd = (uint32_t)(n0 + l8) * p.ldb + c16_odd;
  const uint32_t offa_even = (uint32_t)(m_base + l8) * p.lda + c16_even, offa_odd = (uint32_t)(m_base + l8) * p.lda + c16_odd;
  const uint32_t step_w = 8u * p.ldb, step_a = 8u * p.lda;
  uint32_t off_sa = OOB, off_sb = OOB;
  int sfa_step = 0, sfb_step = 0;
  if constexpr (BLOCK) {
    const int nblocks = (p.N + 127) >> 7;
    const int64_t sfa_elems = (int64_t)(p.M - 1) * p.sa_stride_m + (int64_t)(nkb - 1) * p.sa_stride_k + 1;
    const int64_t sfb_elems = (int64_t)(nblocks - 1) * p.sb_stride_n + (int64_t)(nkb - 1) * p.sb_stride_k + 1;
    rsa = make_rsrc_sgpr(p.sa, (uint32_t)(sfa_elems * 4));
    rsb = make_rsrc_sgpr(p.sb, (uint32_t)(sfb_elems * 4));
    off_sa = m_base + lane < p.M ? (uint32_t)((m_base + lane) * p.sa_stride_m * 4) : OOB;  // lane = activation row of the tile
    int nb = n0 >> 7;  // BN divides 128: one scale block per block of rows
    if (nb >= nblocks) nb = nblocks - 1;
    off_sb = lane == 0 ? (uint32_t)(nb * p.sb_stride_n * 4) : OOB;
    sfa_step = (int)(p.sa_stride_k * 4);
    sfb_step = (int)(p.sb_stride_k * 4);
  }

  const uint32_t ring = lds_addr(smem) + (uint32_t)wave * RING_BYTES;
  auto issue_group = [&](int t) {  // all copies of this wave's t-th K block into slot t % NSTAGE
    const uint32_t st = ring + (uint32_t)(t % NSTAGE) * STAGE_BYTES;
    const uint32_t kb = (uint32_t)(wave + 4 * t);
    const uint32_t kill = t < nsteps ? 0u : OOB;  // past the end: out of range, the K offset is not bounds-checked
    const uint32_t k0 = t < nsteps ? kb * 128u : 0u;
#pragma unroll
    for (int j = 0; j < WC; ++j)
      lds_copy16(rb, st + j * 1024, (((j & 1) ? offw_odd : offw_even) + j * step_w) | kill, k0);
#pragma unroll
    for (int j = 0; j < AC; ++j)
      lds_copy16(ra, st + W_BYTES + j * 1024, (((j & 1) ? offa_odd : offa_even) + j * step_a) | kill, k0);
    if constexpr (BLOCK) {
      lds_copy4(rsa, st + W_BYTES + A_BYTES, off_sa | kill, t < nsteps ? kb * (uint32_t)sfa_step : 0u);
      lds_copy4(rsb, st + W_BYTES + A_BYTES + 256, off_sb | kill, t < nsteps ? kb * (uint32_t)sfb_step : 0u);
    }
  };

  const int sw = (r16 & 7) ^ (r16 >> 3);
  const int lane_off0 = r16 * 128 + (((2 * g) ^ sw) * 16);
  const int lane_off1 = lane_off0 ^ 16;
  auto read_frag = [&](const char* q) -> v8i {
    v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
    v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  using acc_t = typename std::conditional<float_acc(KIND), v4f, v4i>::type;
  acc_t acc[MI][NIB];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NIB; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

#pragma unroll
  for (int t = 0; t < NSTAGE - 1; ++t) issue_group(t);

  char* my_ring = smem + wave * RING_BYTES;
  for (int t = 0; t < nsteps; ++t) {
    // slot (t - 1) % NSTAGE was read in the iteration before (its fragments went through the
    // MFMAs): refill it, then wait for stage t, leaving the NSTAGE - 1 younger groups in flight
    issue_group(t + NSTAGE - 1);
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSTAGE - 1) * CPW) : "memory");

    const char* st = my_ring + (t % NSTAGE) * STAGE_BYTES;
    v8i wf[NIB], af[MI];
#pragma unroll
    for (int j = 0; j < NIB; ++j) wf[j] = read_frag(st + j * 16 * 128);
#pragma unroll
    for (int i = 0; i < MI; ++i) af[i] = read_frag(st + W_BYTES + i * 16 * 128);
    float sc[MI];
    if constexpr (BLOCK) {
      const float* sfa = reinterpret_cast<const float*>(st + W_BYTES + A_BYTES);
      const float sfb = sfa[64];
#pragma unroll
      for (int i = 0; i < MI; ++i) sc[i] = sfa[i * 16 + r16] * sfb;
    }
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int j = 0; j < NIB; ++j) {
        if constexpr (BLOCK) {
          v4f part = block_mfma<KIND>(wf[j], af[i]);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][j][e] = __builtin_fmaf(block_value<KIND>(part[e]), sc[i], acc[i][j][e]);
        } else if constexpr (KIND == KIND_FP8_ROWCOL) {
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[j], af[i], acc[i][j], 0, 0, 0, 0, 0, 0);
        } else {
          const v4i b0 = {wf[j][0], wf[j][1], wf[j][2], wf[j][3]}, b1 = {wf[j][4], wf[j][5], wf[j][6], wf[j][7]};
          const v4i a0 = {af[i][0], af[i][1], af[i][2], af[i][3]}, a1 = {af[i][4], af[i][5], af[i][6], af[i][7]};
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b0, a0, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b1, a1, acc[i][j], 0, 0, 0);
        }
      }
    }
  }

  // The rings are done with (the copies still in flight are the zero fills past the end):
  // waves 1..3 leave their partial sums in their own ring, wave 0 adds them in wave order.
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
  if (wave != 0) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NIB; ++j) *reinterpret_cast<acc_t*>(my_ring + (i * NIB + j) * 1024 + lane * 16) = acc[i][j];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < 4; ++w)
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NIB; ++j) {
          const acc_t t = *reinterpret_cast<const acc_t*>(smem + w * RING_BYTES + (i * NIB + j) * 1024 + lane * 16);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][j][e] += t[e];
        }
    epilogue<KIND, OUT_DT, MI, NIB>(p, acc, m_base, n0, r16, g);
  }
}

// ---------------------------------------------------------------------------
// gemm_stream_kernel for M <= 8 with the activation quantization folded in: p.a holds the
// 16-bit activations (row stride p.lda BYTES) instead of FP8 codes and group scales.  A wave
// streams, next to the weight rows of its K blocks, the 8 x 128 activations of the same K
// blocks (8 rows x 256 bytes) through its ring, and turns them into the codes and the scale of
// per-token-group quantization with groups of 128 = one K block right before the block's MFMAs:
//   * lane l takes 16 elements (32 bytes) of row l / 8; the row's eight lanes are adjacent, so
//     the group's abs-max is three DPP steps, as in group_quant_kernel;
//   * scale and codes come from the same device functions as that kernel (quant_device.h):
//     bit-identical codes and scales;
//   * the 16 codes of a lane are one 16-byte chunk of the MFMA operand tile: they go to a
//     wave-private 8 x 128-byte tile in LDS in the swizzled layout of the MFMA operand reads, and
//     the operand is read back from there (the lanes of fragment rows 8..15, whose results are
//     never stored, read rows 0..7 again); the row's scale reaches the MFMA lanes of that row
//     with one cross-lane read.
// LDS accesses of one wave execute in order, so the tile needs no barrier.  Weight rows, K
// split over the waves and the order of every sum are those of gemm_stream_kernel<KIND, 1, NIB>:
// the output equals quantize-then-multiply through that kernel bit for bit, without the
// quantization launch and without the codes' round trip through memory.
// ---------------------------------------------------------------------------
template <int NIB, int OUT_DT, int IN_DT, int ROWS>
__global__ __launch_bounds__(256) void gemm_stream_quant_kernel(const GemmArgs p) {
  constexpr int KIND = KIND_FP8_BLOCK;
  constexpr int BN = NIB * 16, XR = 8;
  constexpr int WC = BN / 8, XC = XR * 256 / 1024;  // one-KiB copies per stage: weights, activations
  constexpr int CPW = WC + XC + 1;                  // ... and the weight scale
  constexpr int W_BYTES = BN * 128, X_BYTES = XR * 256, S_BYTES = 256;
  constexpr int STAGE_BYTES = W_BYTES + X_BYTES + S_BYTES;
  constexpr int NSTAGE = SGLQ_STREAM_NSTAGE;
  constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;
  constexpr int TILE_BYTES = 8 * 128;  // the quantized activations of the current K block
  // ROWS (1, 2, 4 or 8, at least M): rows that take part in the quantization.  A row's 128 elements are
  // spread over 64 / ROWS adjacent lanes, so that a wave spends 2 ROWS elements' worth of arithmetic
  // per lane and K block instead of 16 whatever M is.
  constexpr int LPR = 64 / ROWS, EPL = 128 / LPR, WPL = EPL / 2;  // lanes per row, elements and 32-bit words per lane
  static_assert(ROWS == 1 || ROWS == 2 || ROWS == 4 || ROWS == 8, "rows per wave");
  static_assert((NSTAGE - 1) * CPW <= 63, "vmcnt holds 6 bits");
  static_assert(NIB * 1024 <= RING_BYTES, "the partial sums are exchanged through a wave's ring");

  __shared__ __attribute__((aligned(1024))) char smem[4 * (RING_BYTES + TILE_BYTES)];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4, l8 = lane >> 3;
  const int n0 = blockIdx.x * BN;
  const int nkb = p.K >> 7;
  const int nsteps = (nkb - wave + 3) >> 2;  // K blocks wave, wave + 4, ...

  const v4u rx = make_rsrc_sgpr(p.a, p.a_bytes);
  const v4u rb = make_rsrc_sgpr(p.b, p.b_bytes);

  // weights: as gemm_stream_kernel (copy gj brings rows 8 gj .. 8 gj + 7, lane l row l / 8, chunk (l % 8) ^ swz(row))
  const int c16_even = (((lane & 7) ^ l8) & 7) * 16, c16_odd = (((lane & 7) ^ l8 ^ 1) & 7) * 16;
  const uint32_t offw_even = (uint32_t)(n0 + l8) * p.ldb + c16_even, offw_odd = (uint32_t)(n0 + l8) * p.ldb + c16_odd;
  const uint32_t step_w = 8u * p.ldb;
  // activations: copy j brings rows 4 j .. 4 j + 3 of the K block, lane l 16 bytes (8 elements) of row
  // 4 j + l / 16; rows past M are out of range and read as zero
  const uint32_t x_piece = (uint32_t)(lane & 15) * 16u;
  uint32_t offx[XC];
#pragma unroll
  for (int j = 0; j < XC; ++j) {
    const int row = 4 * j + (lane >> 4);
    offx[j] = row < p.M ? (uint32_t)row * p.lda + x_piece : OOB;
  }
  const int nblocks = (p.N + 127) >> 7;
  const int64_t sfb_elems = (int64_t)(nblocks - 1) * p.sb_stride_n + (int64_t)(nkb - 1) * p.sb_stride_k + 1;
  const v4u rsb = make_rsrc_sgpr(p.sb, (uint32_t)(sfb_elems * 4));
  int nb = n0 >> 7;  // BN divides 128: one scale block per block of rows
  if (nb >= nblocks) nb = nblocks - 1;
  const uint32_t off_sb = lane == 0 ? (uint32_t)(nb * p.sb_stride_n * 4) : OOB;
  const int sfb_step = (int)(p.sb_stride_k * 4);

  const uint32_t ring = lds_addr(smem) + (uint32_t)wave * RING_BYTES;
  auto issue_group = [&](int t) {  // all copies of this wave's t-th K block into slot t % NSTAGE
    const uint32_t st = ring + (uint32_t)(t % NSTAGE) * STAGE_BYTES;
    const uint32_t kb = (uint32_t)(wave + 4 * t);
    const uint32_t kill = t < nsteps ? 0u : OOB;  // past the end: out of range, the K offset is not bounds-checked
    const uint32_t k0 = t < nsteps ? kb * 128u : 0u;
#pragma unroll
    for (int j = 0; j < WC; ++j)
      lds_copy16(rb, st + j * 1024, (((j & 1) ? offw_odd : offw_even) + j * step_w) | kill, k0);
#pragma unroll
    for (int j = 0; j < XC; ++j) lds_copy16(rx, st + W_BYTES + j * 1024, offx[j] | kill, k0 * 2u);
    lds_copy4(rsb, st + W_BYTES + X_BYTES, off_sb | kill, t < nsteps ? kb * (uint32_t)sfb_step : 0u);
  };

  const int sw = (r16 & 7) ^ (r16 >> 3);
  const int lane_off0 = r16 * 128 + (((2 * g) ^ sw) * 16);
  const int lane_off1 = lane_off0 ^ 16;
  auto read_frag = [&](const char* q) -> v8i {
    v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
    v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  v4f acc[NIB];
#pragma unroll
  for (int j = 0; j < NIB; ++j) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};

  char* my_ring = smem + wave * RING_BYTES;
  char* my_tile = smem + 4 * RING_BYTES + wave * TILE_BYTES;
  // operand read of the tile: row r16 % ROWS (swz(row) = row for rows 0..7)
  const int t_row = r16 & (ROWS - 1);
  const int tile_off0 = t_row * 128 + (((2 * g) ^ t_row) * 16), tile_off1 = tile_off0 ^ 16;
  // quantization lanes: row l / LPR, elements EPL (l % LPR) .. + EPL - 1 of the K block; its codes are EPL
  // bytes of the row's 16-byte chunk EPL (l % LPR) / 16, which sits at chunk position chunk ^ swz(row) = chunk ^ row
  const int q_row = lane / LPR, q_first = (lane % LPR) * EPL;
  const int q_src = q_row * 256 + q_first * 2;
  const int q_dst = q_row * 128 + ((((q_first >> 4) ^ q_row) & 7) * 16) + (q_first & 15);
  // byte index of a lane that holds the scale of fragment row r16 (rows past ROWS repeat the rows below, like the codes)
  const int scale_from = ((r16 & (ROWS - 1)) * LPR) * 4;

#pragma unroll
  for (int t = 0; t < NSTAGE - 1; ++t) issue_group(t);

  for (int t = 0; t < nsteps; ++t) {
    issue_group(t + NSTAGE - 1);
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSTAGE - 1) * CPW) : "memory");

    const char* st = my_ring + (t % NSTAGE) * STAGE_BYTES;
    // ---- per-token-group quantization of this K block's ROWS x 128 activations
    uint32_t w[WPL];
    {
      const char* src = st + W_BYTES + q_src;
      if constexpr (WPL == 8) {
        const v4u lo = *reinterpret_cast<const v4u*>(src), hi = *reinterpret_cast<const v4u*>(src + 16);
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = lo[i], w[4 + i] = hi[i];
      } else if constexpr (WPL == 4) {
        const v4u lo = *reinterpret_cast<const v4u*>(src);
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = lo[i];
      } else if constexpr (WPL == 2) {
        const v2u lo = *reinterpret_cast<const v2u*>(src);
        w[0] = lo.x, w[1] = lo.y;
      } else {
        w[0] = *reinterpret_cast<const uint32_t*>(src);
      }
    }
    // |x| of a 16-bit float orders like its low 15 bits taken as an integer (bfloat16 and half alike)
    v2us m16 = {0, 0};
#pragma unroll
    for (int i = 0; i < WPL; ++i) m16 = __builtin_elementwise_max(m16, __builtin_bit_cast(v2us, w[i] & 0x7fff7fffu));
    uint32_t hmax = m16.x > m16.y ? m16.x : m16.y;
    if constexpr (LPR == 8) hmax = group_umax<8>(hmax);
    else if constexpr (LPR == 16) hmax = group_umax<16>(hmax);
    else if constexpr (LPR == 32) hmax = umax(group_umax<16>(hmax), (uint32_t)__shfl_xor((int)group_umax<16>(hmax), 16));
    else hmax = wave_umax(hmax);
    const float amax_x = to_f32_16<IN_DT>((uint16_t)hmax);
    const float amax = u2f(umax(f2u(amax_x), f2u(p.quant_eps)));
    const float y_s = div_by(amax, 448.0f, 1.0f / 448.0f);
    const float rcp = 1.0f / y_s;
    uint32_t codes[(EPL + 3) / 4];
#pragma unroll
    for (int i = 0; i < WPL; ++i) {
      const float lo = quantize_elem<false>(to_f32_16<IN_DT>((uint16_t)(w[i] & 0xffffu)), y_s, rcp, -448.0f, 448.0f);
      const float hi = quantize_elem<false>(to_f32_16<IN_DT>((uint16_t)(w[i] >> 16)), y_s, rcp, -448.0f, 448.0f);
      if (i & 1) codes[i >> 1] = cvt_pk_e4m3<true>(lo, hi, codes[i >> 1]);
      else codes[i >> 1] = cvt_pk_e4m3<false>(lo, hi, 0);
    }
    if constexpr (EPL == 16) *reinterpret_cast<v4u*>(my_tile + q_dst) = v4u{codes[0], codes[1], codes[2], codes[3]};
    else if constexpr (EPL == 8) *reinterpret_cast<v2u*>(my_tile + q_dst) = v2u{codes[0], codes[1]};
    else if constexpr (EPL == 4) *reinterpret_cast<uint32_t*>(my_tile + q_dst) = codes[0];
    else *reinterpret_cast<uint16_t*>(my_tile + q_dst) = (uint16_t)codes[0];
    // (executed by every lane: a cross-lane read only sees lanes that take part in it)
    const float sfa = u2f((uint32_t)__builtin_amdgcn_ds_bpermute(scale_from, (int)f2u(y_s)));

    v8i wf[NIB];
#pragma unroll
    for (int j = 0; j < NIB; ++j) wf[j] = read_frag(st + j * 16 * 128);
    const float sfb = *reinterpret_cast<const float*>(st + W_BYTES + X_BYTES);
    const v4i alo = *reinterpret_cast<const v4i*>(my_tile + tile_off0), ahi = *reinterpret_cast<const v4i*>(my_tile + tile_off1);
    const v8i af = v8i{alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
    const float sc = sfa * sfb;
#pragma unroll
    for (int j = 0; j < NIB; ++j) {
      const v4f part = block_mfma<KIND>(wf[j], af);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[j][e] = __builtin_fmaf(part[e], sc, acc[j][e]);
    }
  }

  // as gemm_stream_kernel: waves 1..3 leave their partial sums in their own ring, wave 0 adds them in wave order
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
  if (wave != 0) {
#pragma unroll
    for (int j = 0; j < NIB; ++j) *reinterpret_cast<v4f*>(my_ring + j * 1024 + lane * 16) = acc[j];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < 4; ++w)
#pragma unroll
      for (int j = 0; j < NIB; ++j) {
        const v4f t = *reinterpret_cast<const v4f*>(smem + w * RING_BYTES + j * 1024 + lane * 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[j][e] += t[e];
      }
    v4f out_acc[1][NIB];
#pragma unroll
    for (int j = 0; j < NIB; ++j) out_acc[0][j] = acc[j];
    epilogue<KIND, OUT_DT, 1, NIB>(p, out_acc, 0, n0, r16, g);
  }
}

// ---------------------------------------------------------------------------
// gemm_stream_kernel for M <= 8 with the per-token (per-row) activation quantization folded in, for the
// per-row / per-column scaled kinds: p.a holds the 16-bit activations (row stride p.lda BYTES).  A row's
// scale needs the whole row, so every block first reads its ROWS rows once (they come from L2 for every
// block but the first) and forms the rows' abs-max: 256 lanes stride over a row's 16-byte chunks, packed
// 16-bit integer max on the sign-stripped bit patterns, wave max, the four waves' values meet in LDS.  The
// first ring stages (weights and raw activations) are issued before that pass, so the weight stream starts
// with the kernel.  From the row maximum:
//   FP8  scale = max / 448, inv = scale == 0 ? 0 : 1 / scale, q = e4m3(clamp(x * inv))      (token_quant_kernel,
//   INT8 scale = max(max, 1e-10) / 127, mul = 127 / max(max, 1e-10), q = clamp(round(x * mul))  quant.hip)
// with the same expressions as the quantization kernel: bit-identical codes and scales.  The K loop is that
// of gemm_stream_quant_kernel (raw activations through the wave's ring, quantized into a wave-private
// 8 x 128-byte tile in the MFMA operand layout) with the accumulation of gemm_stream_kernel<KIND, 1, NIB>
// in place, and wave 0's epilogue takes the row scale from its register: the output equals
// quantize-then-multiply through that kernel bit for bit.
// ---------------------------------------------------------------------------
template <int KIND, int NIB, int OUT_DT, int IN_DT, int ROWS>
__global__ __launch_bounds__(256) void gemm_stream_tokenquant_kernel(const GemmArgs p) {
  static_assert(KIND == KIND_FP8_ROWCOL || KIND == KIND_I8_ROWCOL, "per-row / per-column scaled kinds");
  constexpr bool IS_FP8 = KIND == KIND_FP8_ROWCOL;
  constexpr int BN = NIB * 16, XR = 8;
  constexpr int WC = BN / 8, XC = XR * 256 / 1024;  // one-KiB copies per stage: weights, activations
  constexpr int CPW = WC + XC;
  constexpr int W_BYTES = BN * 128, X_BYTES = XR * 256;
  constexpr int STAGE_BYTES = W_BYTES + X_BYTES;
  constexpr int NSTAGE = SGLQ_STREAM_NSTAGE;
  constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;
  constexpr int TILE_BYTES = 8 * 128;  // the quantized activations of the current K block
  constexpr int LPR = 64 / ROWS, EPL = 128 / LPR, WPL = EPL / 2;  // lanes per row, elements and 32-bit words per lane
  static_assert(ROWS == 1 || ROWS == 2 || ROWS == 4 || ROWS == 8, "rows per wave");
  static_assert((NSTAGE - 1) * CPW <= 63, "vmcnt holds 6 bits");
  static_assert(NIB * 1024 <= RING_BYTES, "the partial sums are exchanged through a wave's ring");

  // (one LDS object: rings, the waves' code tiles, then the waves' row maxima)
  __shared__ __attribute__((aligned(1024))) char smem[4 * (RING_BYTES + TILE_BYTES) + 4 * ROWS * 4];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4, l8 = lane >> 3;
  const int n0 = blockIdx.x * BN;
  const int nkb = p.K >> 7;
  const int nsteps = (nkb - wave + 3) >> 2;  // K blocks wave, wave + 4, ...

  const v4u rx = make_rsrc_sgpr(p.a, p.a_bytes);
  const v4u rb = make_rsrc_sgpr(p.b, p.b_bytes);

  const int c16_even = (((lane & 7) ^ l8) & 7) * 16, c16_odd = (((lane & 7) ^ l8 ^ 1) & 7) * 16;
  const uint32_t offw_even = (uint32_t)(n0 + l8) * p.ldb + c16_even, offw_odd = (uint32_t)(n0 + l8) * p.ldb + c16_odd;
  const uint32_t step_w = 8u * p.ldb;
  const uint32_t x_piece = (uint32_t)(lane & 15) * 16u;
  uint32_t offx[XC];
#pragma unroll
  for (int j = 0; j < XC; ++j) {
    const int row = 4 * j + (lane >> 4);
    offx[j] = row < p.M ? (uint32_t)row * p.lda + x_piece : OOB;
  }

  const uint32_t ring = lds_addr(smem) + (uint32_t)wave * RING_BYTES;
  auto issue_group = [&](int t) {  // all copies of this wave's t-th K block into slot t % NSTAGE
    const uint32_t st = ring + (uint32_t)(t % NSTAGE) * STAGE_BYTES;
    const uint32_t kb = (uint32_t)(wave + 4 * t);
    const uint32_t kill = t < nsteps ? 0u : OOB;  // past the end: out of range, the K offset is not bounds-checked
    const uint32_t k0 = t < nsteps ? kb * 128u : 0u;
#pragma unroll
    for (int j = 0; j < WC; ++j)
      lds_copy16(rb, st + j * 1024, (((j & 1) ? offw_odd : offw_even) + j * step_w) | kill, k0);
#pragma unroll
    for (int j = 0; j < XC; ++j) lds_copy16(rx, st + W_BYTES + j * 1024, offx[j] | kill, k0 * 2u);
  };

  const int sw = (r16 & 7) ^ (r16 >> 3);
  const int lane_off0 = r16 * 128 + (((2 * g) ^ sw) * 16);
  const int lane_off1 = lane_off0 ^ 16;
  auto read_frag = [&](const char* q) -> v8i {
    v4i lo = *reinterpret_cast<const v4i*>(q + lane_off0);
    v4i hi = *reinterpret_cast<const v4i*>(q + lane_off1);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  using acc_t = typename std::conditional<IS_FP8, v4f, v4i>::type;
  acc_t acc[NIB];
#pragma unroll
  for (int j = 0; j < NIB; ++j) acc[j] = acc_t{0, 0, 0, 0};

  char* my_ring = smem + wave * RING_BYTES;
  char* my_tile = smem + 4 * RING_BYTES + wave * TILE_BYTES;
  uint32_t* red = reinterpret_cast<uint32_t*>(smem + 4 * (RING_BYTES + TILE_BYTES));
  const int t_row = r16 & (ROWS - 1);
  const int tile_off0 = t_row * 128 + (((2 * g) ^ t_row) * 16), tile_off1 = tile_off0 ^ 16;
  const int q_row = lane / LPR, q_first = (lane % LPR) * EPL;
  const int q_src = q_row * 256 + q_first * 2;
  const int q_dst = q_row * 128 + ((((q_first >> 4) ^ q_row) & 7) * 16) + (q_first & 15);

#pragma unroll
  for (int t = 0; t < NSTAGE - 1; ++t) issue_group(t);

  // ---- the rows' abs-max: every lane of the block strides over the 16-byte chunks of each row (rows past M and
  // chunks past K are out of range and read as zero)
  {
    const __amdgpu_buffer_rsrc_t rxa = make_rsrc(p.a, p.a_bytes);
    const uint32_t chunks = (uint32_t)p.K >> 3;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      v2us m16 = {0, 0};
      for (uint32_t c0 = 0; c0 < chunks; c0 += 1024) {
        v4u raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t c = c0 + (uint32_t)u * 256u + threadIdx.x;
          raw[u] = __builtin_amdgcn_raw_buffer_load_b128(rxa, c < chunks ? (uint32_t)r * p.lda + c * 16u : OOB, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) m16 = __builtin_elementwise_max(m16, __builtin_bit_cast(v2us, raw[u][i] & 0x7fff7fffu));
      }
      const uint32_t hmax = wave_umax(m16.x > m16.y ? (uint32_t)m16.x : (uint32_t)m16.y);
      if (lane == 0) red[wave * ROWS + r] = hmax;
    }
  }
  __syncthreads();
  // scale and multiplier of a row, from the same expressions as token_quant_kernel
  auto row_scale = [&](int r, float& scale, float& mul) {
    const uint32_t hmax = umax(umax(red[r], red[ROWS + r]), umax(red[2 * ROWS + r], red[3 * ROWS + r]));
    const float amax_x = to_f32_16<IN_DT>((uint16_t)hmax);
    if constexpr (IS_FP8) {
      scale = amax_x / 448.0f;
      mul = (scale == 0.f) ? 0.f : 1.0f / scale;
    } else {
      const float amax = u2f(umax(f2u(amax_x), f2u(1e-10f)));
      scale = amax / 127.0f;
      mul = 127.0f / amax;
    }
  };
  float q_scale, q_mul, out_scale, out_mul;
  row_scale(q_row, q_scale, q_mul);
  row_scale(t_row, out_scale, out_mul);

  for (int t = 0; t < nsteps; ++t) {
    issue_group(t + NSTAGE - 1);
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSTAGE - 1) * CPW) : "memory");

    const char* st = my_ring + (t % NSTAGE) * STAGE_BYTES;
    // ---- quantization of this K block's ROWS x 128 activations with the rows' scales
    uint32_t w[WPL];
    {
      const char* src = st + W_BYTES + q_src;
      if constexpr (WPL == 8) {
        const v4u lo = *reinterpret_cast<const v4u*>(src), hi = *reinterpret_cast<const v4u*>(src + 16);
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = lo[i], w[4 + i] = hi[i];
      } else if constexpr (WPL == 4) {
        const v4u lo = *reinterpret_cast<const v4u*>(src);
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = lo[i];
      } else if constexpr (WPL == 2) {
        const v2u lo = *reinterpret_cast<const v2u*>(src);
        w[0] = lo.x, w[1] = lo.y;
      } else {
        w[0] = *reinterpret_cast<const uint32_t*>(src);
      }
    }
    uint32_t codes[(EPL + 3) / 4];
#pragma unroll
    for (int i = 0; i < (EPL + 3) / 4; ++i) codes[i] = 0;
#pragma unroll
    for (int i = 0; i < WPL; ++i) {
      float lo = to_f32_16<IN_DT>((uint16_t)(w[i] & 0xffffu)) * q_mul;
      float hi = to_f32_16<IN_DT>((uint16_t)(w[i] >> 16)) * q_mul;
      if constexpr (IS_FP8) {
        lo = clampf(lo, -448.0f, 448.0f);
        hi = clampf(hi, -448.0f, 448.0f);
        if (i & 1) codes[i >> 1] = cvt_pk_e4m3<true>(lo, hi, codes[i >> 1]);
        else codes[i >> 1] = cvt_pk_e4m3<false>(lo, hi, 0);
      } else {
        const uint32_t blo = (uint32_t)(int)clampf(__builtin_roundf(lo), -128.0f, 127.0f) & 0xffu;
        const uint32_t bhi = (uint32_t)(int)clampf(__builtin_roundf(hi), -128.0f, 127.0f) & 0xffu;
        codes[i >> 1] |= (blo | (bhi << 8)) << ((i & 1) * 16);
      }
    }
    if constexpr (EPL == 16) *reinterpret_cast<v4u*>(my_tile + q_dst) = v4u{codes[0], codes[1], codes[2], codes[3]};
    else if constexpr (EPL == 8) *reinterpret_cast<v2u*>(my_tile + q_dst) = v2u{codes[0], codes[1]};
    else if constexpr (EPL == 4) *reinterpret_cast<uint32_t*>(my_tile + q_dst) = codes[0];
    else *reinterpret_cast<uint16_t*>(my_tile + q_dst) = (uint16_t)codes[0];

    v8i wf[NIB];
#pragma unroll
    for (int j = 0; j < NIB; ++j) wf[j] = read_frag(st + j * 16 * 128);
    const v4i alo = *reinterpret_cast<const v4i*>(my_tile + tile_off0), ahi = *reinterpret_cast<const v4i*>(my_tile + tile_off1);
    const v8i af = v8i{alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
#pragma unroll
    for (int j = 0; j < NIB; ++j) {
      if constexpr (IS_FP8) {
        acc[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[j], af, acc[j], 0, 0, 0, 0, 0, 0);
      } else {
        const v4i b0 = {wf[j][0], wf[j][1], wf[j][2], wf[j][3]}, b1 = {wf[j][4], wf[j][5], wf[j][6], wf[j][7]};
        acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b0, alo, acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b1, ahi, acc[j], 0, 0, 0);
      }
    }
  }

  // as gemm_stream_kernel: waves 1..3 leave their partial sums in their own ring, wave 0 adds them in wave order
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
  if (wave != 0) {
#pragma unroll
    for (int j = 0; j < NIB; ++j) *reinterpret_cast<acc_t*>(my_ring + j * 1024 + lane * 16) = acc[j];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < 4; ++w)
#pragma unroll
      for (int j = 0; j < NIB; ++j) {
        const acc_t t = *reinterpret_cast<const acc_t*>(smem + w * RING_BYTES + j * 1024 + lane * 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[j][e] += t[e];
      }
    int r = r16, gg = g;
    asm volatile("" : "+v"(r), "+v"(gg));
    if (r < p.M) {
#pragma unroll
      for (int j = 0; j < NIB; ++j) {
        const int n = n0 + j * 16 + gg * 4;
        if (n < p.N) finish4<KIND, OUT_DT>(p, r, n, acc[j], out_scale);
      }
    }
  }
}

// Sum the split-K partials in split order and apply the epilogue; one thread per
// run of four consecutive n.
template <int KIND, int OUT_DT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmArgs p) {
  constexpr bool IS_FP8 = fp8_operands(KIND);
  using acc_t = typename std::conditional<float_acc(KIND), v4f, v4i>::type;
  const int n4 = p.N >> 2;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)p.M * n4) return;
  const int m = (int)(id / n4), n = (int)(id % n4) * 4;
  const acc_t* src =
      reinterpret_cast<const acc_t*>(reinterpret_cast<const char*>(p.ws) + ((int64_t)m * p.N + n) * 4);
  const int64_t stride = (int64_t)p.M * p.N / 4;  // in acc_t units
  acc_t a = src[0];
  for (int s = 1; s < p.splits; ++s) a += src[s * stride];
  float sam = 1.f;
  if constexpr (KIND == KIND_FP8_ROWCOL || KIND == KIND_I8_ROWCOL) sam = p.sa[m];
  finish4<KIND, OUT_DT>(p, m, n, a, sam);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
// The test hooks (sglq_debug_*) are per calling thread: a test that forces a kernel cannot
// change what another thread's GEMM calls launch.
static thread_local bool g_use_dma = true;

// Compute units of the current device, rounded down to a multiple of 8 (keeps the persistent
// kernels' tile walk on one XCD per block).  The only process-wide state besides the tuned
// table: an immutable property, cached per device ordinal (a racing first call stores the same value).
constexpr int MAX_DEVICES = 64;
static int num_cus() {
  static std::atomic<int> cached[MAX_DEVICES];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) dev = 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    n = n >= 8 ? (n / 8) * 8 : n;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

static thread_local int g_force_splits = 0;  // test hook: > 0 fixes the split-K factor where split-K applies
// The selection in force for the call being launched on this thread: the test hooks, else a
// matching entry of the tuned table, else 0 = the built-in heuristics.
static thread_local int t_tile = 0, t_splits = 0;
static thread_local int g_grouped_tile = 0;  // test hook: 32 / 64 / 128 / 256 fixes the grouped GEMM's row tile, 130 = 128 rows pipelined (0 = from the average group)
static thread_local const char* g_last_kernel = "";  // which GEMM kernel the calling thread's last call launched
static thread_local bool g_last_hw_scaled = false;   // ... and whether its MFMAs applied the block scales (KIND_FP8_BLOCK_POW2)

template <int KIND, int OUT_DT>
static void launch_reduce(GemmArgs& p, hipStream_t st);
static void expand_packed_scales(GemmArgs& p, hipStream_t st);

// Tile plan of a grouped GEMM, from the experts' row counts and first rows in device memory
// (problem_sizes[e][0], expert_offsets[e]); one block.  Inconsistent inputs cannot make the
// GEMM leave its buffers: rows are clamped to [0, total_m] and tiles to the grid's count.
__global__ __launch_bounds__(256) void grouped_plan_kernel(const int* __restrict__ problem_sizes,
                                                          const int* __restrict__ expert_offsets, int num_experts,
                                                          int total_m, int bm, int max_tiles, int* __restrict__ plan) {
  __shared__ int scan[256];
  __shared__ int base_s;
  const int tid = threadIdx.x;
  if (tid == 0) base_s = 0;
  __syncthreads();
  for (int e0 = 0; e0 < num_experts; e0 += 256) {
    const int e = e0 + tid;
    int rows = 0, first = 0;
    if (e < num_experts) {
      first = expert_offsets[e];
      rows = problem_sizes[3 * e];
      if (first < 0) first = 0;
      if (first > total_m) first = total_m;
      if (rows < 0) rows = 0;
      if (rows > total_m - first) rows = total_m - first;
    }
    const int t = (rows + bm - 1) / bm;
    scan[tid] = t;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
      const int v = tid >= d ? scan[tid - d] : 0;
      __syncthreads();
      scan[tid] += v;
      __syncthreads();
    }
    const int begin = base_s + scan[tid] - t;
    for (int i = 0; i < t; ++i) {
      const int slot = begin + i;
      if (slot < max_tiles) {
        int* entry = plan + PLAN_HEADER + PLAN_ENTRY * slot;
        entry[0] = e;
        entry[1] = first + i * bm;
        entry[2] = first + rows;
        entry[3] = 0;
      }
    }
    __syncthreads();
    if (tid == 255) base_s += scan[255];
    __syncthreads();
  }
  if (tid == 0) plan[0] = base_s < max_tiles ? base_s : max_tiles;
}

template <int KIND, int BM, int BN, int WAVES_M, int WAVES_N, int OUT_DT>
static void launch_grouped_cfg(GemmArgs& p, int max_tiles, hipStream_t st) {
  p.tiles_m = max_tiles;
  p.tiles_n = (p.N + BN - 1) / BN;
  p.splits = 1;
  const dim3 grid((uint32_t)(p.tiles_m * p.tiles_n)), block(WAVES_M * WAVES_N * 64);
  gemm_kernel<KIND, BM, BN, WAVES_M, WAVES_N, OUT_DT, true, true><<<grid, block, 0, st>>>(p);
}

// 128 x 128 (and narrower) tiles.  When the tiles do not fill the chip (two blocks per
// CU), K is split across blocks as far as the workspace and the partial sums' traffic allow.
template <int KIND, int BM, int BN, int WAVES_M, int WAVES_N, int OUT_DT>
static void launch_cfg(GemmArgs& p, int64_t ws_bytes, hipStream_t st) {
  expand_packed_scales(p, st);
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int tiles = p.tiles_m * p.tiles_n;
  const int nkb = (p.K + 127) >> 7;
  int splits = 1;
  if (tiles < 384) {
    splits = (512 + tiles / 2) / tiles;
    const int by_steps = nkb / 4 > 0 ? nkb / 4 : 1;  // at least four K blocks per split
    // partial sums: 8 * M * N * splits bytes written and read, against (M + N) * K of operands
    const int64_t by_traffic = ((int64_t)(p.M + p.N) * p.K) / (8 * (int64_t)p.M * p.N / 2 + 1);
    if (splits > by_steps) splits = by_steps;
    if (splits > by_traffic) splits = (int)(by_traffic > 0 ? by_traffic : 1);
  }
  if (t_splits > 0) splits = t_splits < nkb ? t_splits : nkb;
  const int64_t per_split = (int64_t)p.M * p.N * 4;
  if (!p.ws || ws_bytes < per_split * 2) splits = 1;
  else if (splits * per_split > ws_bytes) splits = (int)(ws_bytes / per_split);
  if (splits < 1) splits = 1;
  p.splits = splits;
  dim3 grid((uint32_t)(tiles * splits)), block(WAVES_M * WAVES_N * 64);
  g_last_kernel = splits > 1 ? "gemm_kernel+splitk_reduce_kernel" : "gemm_kernel";
  if (g_use_dma) gemm_kernel<KIND, BM, BN, WAVES_M, WAVES_N, OUT_DT, true><<<grid, block, 0, st>>>(p);
  else gemm_kernel<KIND, BM, BN, WAVES_M, WAVES_N, OUT_DT, false><<<grid, block, 0, st>>>(p);
  if (splits > 1) launch_reduce<KIND, OUT_DT>(p, st);
}

// test hook: 0 = heuristic, 64 = the M <= 64 kernel where it applies, 128 = the 128 x 128 kernel,
// 256 = the plain 256 x 256 kernel, 258 = the pipelined one (K >= 384, else the plain one),
// 192 / 224 / 257 = the 4 x 2-wave kernel with tiles 192, 224, 256 wide (K >= 384, else as 258),
// 193 = that kernel on 192 x 192 tiles (block-scaled FP8 without a bias, K >= 384; else the heuristic),
// 259 = as 258 with the wave-private epilogue and copies that run on across tile boundaries (block-scaled FP8, no bias, no split),
// 130 = the pipelined kernel with 128-row tiles (K >= 384, else the 128 x 128 kernel)
static thread_local int g_force_tile = 0;
#ifndef SGLQ_DIRECT_MAX_K
#define SGLQ_DIRECT_MAX_K 4096
#endif

static double model_pipe_splits(const GemmArgs& p, int rows_per_tile, int64_t ws_bytes, int& splits);

// Whether this launch takes the kernels whose MFMAs apply the block scales (built for bf16 outputs without a
// fused bias, what the reference's call of that GEMM produces: fp8_utils.py:225-258).
template <int KIND, int OUT_DT>
static bool can_hw_scale(const GemmArgs& p) {
  return KIND == KIND_FP8_BLOCK && OUT_DT == SGLQ_BF16 && p.pow2_scales && !p.bias;
}
template <int KIND, int OUT_DT>
static bool hw_scaled(const GemmArgs& p) {
  const bool hw = can_hw_scale<KIND, OUT_DT>(p);
  if (hw) g_last_hw_scaled = true;
  return hw;
}

// Packed UE8M0 activation scales (GemmArgs::sa_packed) as fp32 powers of two, column-major [K / 128][M], for the
// kernels that multiply by the scales instead of handing their exponents to the matrix instruction.
__global__ __launch_bounds__(256) void expand_ue8m0_kernel(const uint32_t* __restrict__ packed, int64_t stride_m, int64_t stride_k4,
                                                          float* __restrict__ out, int M, int nkb) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * nkb) return;
  const int kb = (int)(idx / M), m = (int)(idx % M);
  const uint32_t word = packed[(int64_t)m * stride_m + (int64_t)(kb >> 2) * stride_k4];
  out[idx] = __builtin_bit_cast(float, ((word >> (8 * (kb & 3))) & 0xffu) << 23);
}
// Called by every launcher whose kernel does not read the packed form, before its launch.
static void expand_packed_scales(GemmArgs& p, hipStream_t st) {
  if (!p.sa_packed) return;
  const int nkb = p.K >> 7;
  const int64_t n = (int64_t)p.M * nkb;
  expand_ue8m0_kernel<<<dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, st>>>(reinterpret_cast<const uint32_t*>(p.sa), p.sa_stride_m, p.sa_stride_k,
                                                                            p.sa_expanded, p.M, nkb);
  p.sa = p.sa_expanded;
  p.sa_stride_m = 1;
  p.sa_stride_k = p.M;
  p.sa_packed = 0;
}

template <int KIND, int OUT_DT>
static void launch_big(GemmArgs& p, int64_t ws_bytes, hipStream_t st) {
  if (!(t_tile != 256 && p.K >= 384 && can_hw_scale<KIND, OUT_DT>(p))) expand_packed_scales(p, st);
  p.tiles_m = (p.M + 255) / 256;
  p.tiles_n = (p.N + 255) / 256;
  p.splits = 1;
  // persistent: one block per CU walks the tiles blockIdx, blockIdx + gridDim, ...
  const int tiles = p.tiles_m * p.tiles_n;
  // the pipelined kernel needs three K blocks; 256 forces the plain one (test hook)
  if (t_tile != 256 && p.K >= 384) {
    // Too few tiles for the chip: split K into equal contiguous ranges of at least four K
    // blocks, as many as fill the CUs and the workspace holds; the partial sums cost
    // 8 M N splits bytes of traffic, which must stay well under the operands'.
    const int nkb = p.K >> 7;
    int splits = 1;
    if (t_splits > 0) {
      int want = t_splits;
      const int64_t per_split = (int64_t)p.M * p.N * 4;
      // (the kernel addresses a split's partial sums, tile padding included, with 31 bits)
      if (!p.ws || ws_bytes < 2 * per_split || (int64_t)(p.M + 256) * p.N * 4 >= (int64_t)1 << 31) want = 1;
      else if (want * per_split > ws_bytes) want = (int)(ws_bytes / per_split);
      for (int s = want; s >= 2; --s)
        if (nkb % s == 0 && nkb / s >= 3) {
          splits = s;
          break;
        }
    } else if (2 * tiles <= num_cus()) {
      // too few tiles for the chip: equal contiguous K ranges, as many as the cost model favours
      model_pipe_splits(p, 256, ws_bytes, splits);
    }
    p.splits = splits;
    const int units = tiles * splits;
    const int blocks = units < num_cus() ? units : num_cus();
    g_last_kernel = splits > 1 ? "gemm_pipe_kernel+splitk_reduce_kernel" : "gemm_pipe_kernel";
    const dim3 grid((uint32_t)blocks), block(512);
    if (splits > 1) {
      if (hw_scaled<KIND, OUT_DT>(p)) {
        if constexpr (KIND == KIND_FP8_BLOCK && OUT_DT == SGLQ_BF16) gemm_pipe_kernel<KIND_FP8_BLOCK_POW2, OUT_DT, PIPE_SPLITK><<<grid, block, 0, st>>>(p);
      } else {
        gemm_pipe_kernel<KIND, OUT_DT, PIPE_SPLITK><<<grid, block, 0, st>>>(p);
      }
      launch_reduce<KIND, OUT_DT>(p, st);  // (adds the bias)
    } else if (is_block(KIND) && p.bias) {
      if constexpr (is_block(KIND)) gemm_pipe_kernel<KIND, OUT_DT, PIPE_BIAS><<<grid, block, 0, st>>>(p);
    } else if (hw_scaled<KIND, OUT_DT>(p)) {
      if constexpr (KIND == KIND_FP8_BLOCK && OUT_DT == SGLQ_BF16) {
        if (t_tile == 259 || (t_tile == 0 && p.K <= SGLQ_DIRECT_MAX_K)) {
          g_last_kernel = "gemm_pipe_kernel<direct stores>";
          gemm_pipe_kernel<KIND_FP8_BLOCK_POW2, OUT_DT, PIPE_DIRECT><<<grid, block, 0, st>>>(p);
        } else {
          gemm_pipe_kernel<KIND_FP8_BLOCK_POW2, OUT_DT, PIPE_PLAIN><<<grid, block, 0, st>>>(p);
        }
      }
    } else if (KIND == KIND_FP8_BLOCK && (t_tile == 259 || (t_tile == 0 && p.K <= SGLQ_DIRECT_MAX_K))) {
      // (measured against the plain variant at M = 4096: K = 1024 76.2 -> 70.4 us, 1536 149.2 -> 140.3, 2048 125.2 -> 117.7,
      // 3072 177.5 -> 176.2, 4096 222.4 -> 218.6, 7168 95.6 -> 95.1; K = 512 within 1 %: four steps per tile are too few
      // to keep the stores of one tile out of the way of the next)
      g_last_kernel = "gemm_pipe_kernel<direct stores>";
      if constexpr (KIND == KIND_FP8_BLOCK) gemm_pipe_kernel<KIND, OUT_DT, PIPE_DIRECT><<<grid, block, 0, st>>>(p);
    } else {
      gemm_pipe_kernel<KIND, OUT_DT, PIPE_PLAIN><<<grid, block, 0, st>>>(p);
    }
  } else {
    const int blocks = tiles < num_cus() ? tiles : num_cus();
    g_last_kernel = "gemm_big_kernel";
    if (is_block(KIND) && p.bias) {
      if constexpr (is_block(KIND)) gemm_big_kernel<KIND, OUT_DT, true><<<dim3((uint32_t)blocks), dim3(512), 0, st>>>(p);
    } else {
      gemm_big_kernel<KIND, OUT_DT, false><<<dim3((uint32_t)blocks), dim3(512), 0, st>>>(p);
    }
  }
}

// Split-K factor of the pipelined kernel by a cost model in microseconds, fitted to measurements
// over M = 256 ... 3072 on the DeepSeek-V3 and Llama-70B shapes: the work units (tiles x splits)
// run in rounds over the CUs; a unit costs its K steps (0.85 us each with 128-row tiles, 1.3 us
// with 256-row tiles) plus a fixed 8 / 10 us (the first blocks' arrival, the epilogue); splitting
// adds the reduction launch (4 us) and the partial sums' round trip (8 M N s bytes at 5 TB/s).
// Returns the modelled time; `splits` gets the factor (a divisor of the K blocks, at least four per unit).
static double model_pipe_splits(const GemmArgs& p, int rows_per_tile, int64_t ws_bytes, int& splits) {
  const int tiles = ((p.M + rows_per_tile - 1) / rows_per_tile) * ((p.N + 255) / 256);
  const int nkb = p.K >> 7;
  const double step_us = rows_per_tile == 128 ? 0.85 : 1.3, fixed_us = rows_per_tile == 128 ? 8.0 : 10.0;
  const int64_t per_split = (int64_t)p.M * p.N * 4;
  const bool can_split = p.ws && ws_bytes >= 2 * per_split && (int64_t)(p.M + 256) * p.N * 4 < ((int64_t)1 << 31);
  double best = 1e30;
  splits = 1;
  for (int s = 1; s <= 16; ++s) {
    if (s > 1 && (!can_split || nkb % s != 0 || nkb / s < 4 || s * per_split > ws_bytes)) continue;
    const int rounds = (tiles * s + num_cus() - 1) / num_cus();
    double cost = rounds * ((nkb / s) * step_us + fixed_us);
    if (s > 1) cost += 4.0 + 8.0 * p.M * p.N * s / 5e6;
    if (cost < best) {
      best = cost;
      splits = s;
    }
  }
  return best;
}

// The pipelined kernel with 128-row tiles: (tile, K range) work units.
template <int KIND, int OUT_DT>
static void launch_pipe128(GemmArgs& p, int64_t ws_bytes, hipStream_t st) {
  if (!can_hw_scale<KIND, OUT_DT>(p)) expand_packed_scales(p, st);
  p.tiles_m = (p.M + 127) / 128;
  p.tiles_n = (p.N + 255) / 256;
  const int tiles = p.tiles_m * p.tiles_n;
  const int nkb = p.K >> 7;
  int splits = 1;
  if (t_splits > 0) {
    const int64_t per_split = (int64_t)p.M * p.N * 4;
    int want = t_splits;
    if (!p.ws || ws_bytes < 2 * per_split || (int64_t)(p.M + 256) * p.N * 4 >= (int64_t)1 << 31) want = 1;
    else if (want * per_split > ws_bytes) want = (int)(ws_bytes / per_split);
    for (int s = want; s >= 2; --s)
      if (nkb % s == 0 && nkb / s >= 3) {
        splits = s;
        break;
      }
  } else {
    model_pipe_splits(p, 128, ws_bytes, splits);
  }
  p.splits = splits;
  const int units = tiles * splits;
  const dim3 grid((uint32_t)(units < num_cus() ? units : num_cus())), block(512);
  g_last_kernel = splits > 1 ? "gemm_pipe_kernel<128 rows>+splitk_reduce_kernel" : "gemm_pipe_kernel<128 rows>";
  if (splits > 1) {
    if (hw_scaled<KIND, OUT_DT>(p)) {
      if constexpr (KIND == KIND_FP8_BLOCK && OUT_DT == SGLQ_BF16) gemm_pipe_kernel<KIND_FP8_BLOCK_POW2, OUT_DT, PIPE_SPLITK, 128><<<grid, block, 0, st>>>(p);
    } else {
      gemm_pipe_kernel<KIND, OUT_DT, PIPE_SPLITK, 128><<<grid, block, 0, st>>>(p);
    }
    launch_reduce<KIND, OUT_DT>(p, st);  // (adds the bias)
  } else if (is_block(KIND) && p.bias) {
    if constexpr (is_block(KIND)) gemm_pipe_kernel<KIND, OUT_DT, PIPE_BIAS, 128><<<grid, block, 0, st>>>(p);
  } else if (hw_scaled<KIND, OUT_DT>(p)) {
    if constexpr (KIND == KIND_FP8_BLOCK && OUT_DT == SGLQ_BF16) gemm_pipe_kernel<KIND_FP8_BLOCK_POW2, OUT_DT, PIPE_PLAIN, 128><<<grid, block, 0, st>>>(p);
  } else {
    gemm_pipe_kernel<KIND, OUT_DT, PIPE_PLAIN, 128><<<grid, block, 0, st>>>(p);
  }
}

// 192 x 192 tiles (block-scaled FP8 without a fused bias): the tile for row and column counts that 256-row tiles
// cover with a part-empty round of the CUs (4096 x 2112: 242 tiles instead of 176 on 256 CUs).
template <int KIND, int OUT_DT>
static void launch_wide_192rows(GemmArgs& p, hipStream_t st) {
  expand_packed_scales(p, st);
  p.tiles_m = (p.M + 191) / 192;
  p.tiles_n = (p.N + 191) / 192;
  p.splits = 1;
  const int tiles = p.tiles_m * p.tiles_n;
  const int blocks = tiles < num_cus() ? tiles : num_cus();
  g_last_kernel = "gemm_wide_kernel<6, 192 rows>";
  if constexpr (KIND == KIND_FP8_BLOCK) gemm_wide_kernel<KIND, OUT_DT, 6, false, 3><<<dim3((uint32_t)blocks), dim3(512), 0, st>>>(p);
}

template <int KIND, int OUT_DT, int NI>
static void launch_wide(GemmArgs& p, hipStream_t st) {
  if (!can_hw_scale<KIND, OUT_DT>(p)) expand_packed_scales(p, st);
  p.tiles_m = (p.M + 255) / 256;
  p.tiles_n = (p.N + 32 * NI - 1) / (32 * NI);
  p.splits = 1;
  const int tiles = p.tiles_m * p.tiles_n;
  const int blocks = tiles < num_cus() ? tiles : num_cus();
  g_last_kernel = NI == 6 ? "gemm_wide_kernel<6>" : NI == 7 ? "gemm_wide_kernel<7>" : "gemm_wide_kernel<8>";
  if (is_block(KIND) && p.bias) {
    if constexpr (is_block(KIND)) gemm_wide_kernel<KIND, OUT_DT, NI, true><<<dim3((uint32_t)blocks), dim3(512), 0, st>>>(p);
  } else if (hw_scaled<KIND, OUT_DT>(p)) {
    if constexpr (KIND == KIND_FP8_BLOCK && OUT_DT == SGLQ_BF16) gemm_wide_kernel<KIND_FP8_BLOCK_POW2, OUT_DT, NI, false><<<dim3((uint32_t)blocks), dim3(512), 0, st>>>(p);
  } else {
    gemm_wide_kernel<KIND, OUT_DT, NI, false><<<dim3((uint32_t)blocks), dim3(512), 0, st>>>(p);
  }
}

// Tile width of the 256-row kernels.  Every CU works through ceil(tiles / CUs) tiles, each
// costing in proportion to its width: take the width with the least rounds x width (7168
// columns at M = 4096: 2 x 224 against 2 x 256; 2112 columns: 1 x 192 against 1 x 256).
// narrow_only: not the 256-wide kernel (block-scaled INT8 on short K, where its epilogue weighs most and its
// two MFMAs per K block leave no registers to spare: 4096 x 32768 x 512 163 us there, 120 us on 192-wide tiles;
// 4096 x 24576 x 1536 227 -> 197 us)
static int pick_tile_width(const GemmArgs& p, bool narrow_only = false) {
  const int tiles_m = (p.M + 255) / 256;
  const int widest = narrow_only ? 224 : 256;
  int best = widest;
  int64_t best_cost = 0;
  for (int bn = widest; bn >= 192; bn -= 32) {
    const int tiles = tiles_m * ((p.N + bn - 1) / bn);
    const int64_t cost = (int64_t)((tiles + num_cus() - 1) / num_cus()) * bn;
    if (bn == widest || cost < best_cost) {
      best = bn;
      best_cost = cost;
    }
  }
  return best;
}

template <int KIND, int OUT_DT>
static void launch_reduce(GemmArgs& p, hipStream_t st) {
  const int64_t work = (int64_t)p.M * (p.N >> 2);
  splitk_reduce_kernel<KIND, OUT_DT><<<dim3((uint32_t)((work + 255) / 256)), dim3(256), 0, st>>>(p);
}

template <int KIND, int MI, int OUT_DT, int BN = 128>
static void launch_skinny_mi(GemmArgs& p, hipStream_t st) {
  if (BN == 64) g_last_kernel = p.splits > 1 ? "gemm_skinny_kernel<64 columns>+splitk_reduce_kernel" : "gemm_skinny_kernel<64 columns>";
  else g_last_kernel = p.splits > 1 ? "gemm_skinny_kernel+splitk_reduce_kernel" : "gemm_skinny_kernel";
  const dim3 grid((uint32_t)(p.tiles_n * p.splits * p.tiles_m)), block(256);
  gemm_skinny_kernel<KIND, MI, OUT_DT, BN><<<grid, block, 0, st>>>(p);
  if (p.splits > 1) launch_reduce<KIND, OUT_DT>(p, st);
}

// Modelled time (us, without what every launch pays) of gemm_skinny_kernel on M > 64 rows with tiles of `bn` weight rows
// and `sp` splits of K.  Fitted to sweeps of M = 96 .. 512, N = 2048 .. 8192, K = 2048 .. 7168: a K step of a block
// that has its CU to itself takes 0.5 us with 128 weight rows and 0.32 us with 64 (0.4 / 0.24 us for the kinds
// without block scales), proportionally more once there are more blocks than CUs; a split costs 4 us for the second
// launch plus the partial sums written and read at 4 TB/s.
static double skinny_cost(int M, int N, int K, int bn, int sp) {
  const int tiles = ((M + 63) / 64) * ((N + bn - 1) / bn), nkb = K >> 7;
  const int blocks = tiles * sp;
  const double steps = (double)((nkb + sp - 1) / sp);
  // (more blocks than CUs: the CUs that hold two set the pace; with 64 weight rows per block a step then takes
  // 1.75 times as long at once, 288 .. 512 blocks alike)
  double crowd = blocks > 256 ? blocks / 256.0 : 1.0;
  if (bn == 64 && blocks > 256) crowd = crowd * 1.2 > 1.75 ? crowd * 1.2 : 1.75;
  double cost = steps * (bn == 64 ? 0.32 : 0.5) * crowd;
  if (sp > 1) cost += 4.0 + (double)M * N * 4.0 * sp * 2.0 / 4e6;
  return cost;
}

// The split-K factor of the decode path without the caller's workspace limits: so that every CU streams weights.
static int skinny_splits(int M, int N, int K, int bn = 128) {
  const int tiles_m = (M + 63) / 64, tiles = tiles_m * ((N + bn - 1) / bn);
  const int nkb = K >> 7;
  // Measured: the fastest split factor puts about one block on every CU (192-256 blocks);
  // more blocks only add partial-sum traffic.
  int splits = 256 / tiles;
  int by_steps = nkb / 2 > 0 ? nkb / 2 : 1;  // at least two K blocks per split
  if (tiles_m > 1) {
    // Several row tiles share a weight tile's traffic.  The split is the cheapest under a model fitted to
    // sweeps of the split factor (256 x 2048 x 7168, 64 tiles: 29.8 / 21.0 / 17.5 / 16.3 / 18.3 / 18.8 us with
    // 1 / 2 / 3 / 4 / 6 / 8 splits; 160 x 7168 x 2048, 168 tiles: 17.4 us with two splits, 12.7 us for the 224
    // tiles of 256 rows with one; 512 x 2112 x 7168, 136 tiles: 29.9 us with one, 24.2 with two): 0.5 us per K
    // block while the blocks fit one per CU, proportionally more beyond; with a split, 4 us for the second
    // launch plus the partial sums written and read at 4 TB/s.  At most eight splits, at least four K blocks each.
    const int max_splits = nkb / 4 > 8 ? 8 : (nkb / 4 > 0 ? nkb / 4 : 1);
    double best = 0.0;
    splits = 1;
    for (int sp = 1; sp <= max_splits; ++sp) {
      const double cost = skinny_cost(M, N, K, bn, sp);
      if (sp == 1 || cost < best) {
        best = cost;
        splits = sp;
      }
    }
    return splits;
  }
  if (splits > by_steps) splits = by_steps;
  // (a handful of weight tiles: 64 x 512 x 7168, four tiles, 15.2 us with 28 splits, 11.9 us with 8)
  if (tiles < 8 && splits > 8) splits = 8;
  return splits < 1 ? 1 : splits;
}

template <int KIND, int OUT_DT>
static void launch_skinny(GemmArgs& p, int64_t ws_bytes, hipStream_t st) {
  expand_packed_scales(p, st);
  // Weight rows per block: 128, or 64 where several row tiles share the weight tiles (M > 64) and the model above
  // says that twice as many blocks with two thirds of the bytes each are faster: up to about 200 tiles of 128.
  bool narrow = t_tile == 66 && p.M > 32;
  if (t_tile == 0 && p.M > 64) {
    const int sw = skinny_splits(p.M, p.N, p.K, 128), sn = skinny_splits(p.M, p.N, p.K, 64);
    narrow = skinny_cost(p.M, p.N, p.K, 64, sn) < skinny_cost(p.M, p.N, p.K, 128, sw);
  }
  // 33 .. 64 rows: 64 weight rows per block on narrow weights and on short K (64 x 2048 x 16384: 19.8 -> 18.2 us,
  // 64 x 7168 x 256: 4.8 -> 4.1 us); 128 on wide ones (64 x 10240 x 8192: 25.2 against 27.5 us)
  // ... and where 64-row blocks fill most of one round of the CUs without a split while 128-row blocks need two
  // splits and the second launch (64 x 14336 x 4096: 19.8 -> 16.0 us)
  if (t_tile == 0 && p.M > 32 && p.M <= 64) {
    const int t64 = (p.N + 63) / 64;
    narrow = p.N <= 4096 || p.K <= 512 || (4 * t64 > 3 * num_cus() && t64 <= num_cus() && (p.K >> 7) <= 40);
  }
  p.tiles_m = (p.M + 63) / 64;
  p.tiles_n = narrow ? (p.N + 63) / 64 : (p.N + 127) / 128;
  const int nkb = p.K >> 7;
  int splits = skinny_splits(p.M, p.N, p.K, narrow ? 64 : 128);
  if (t_splits > 0) splits = t_splits < nkb ? t_splits : nkb;
  const int64_t per_split = (int64_t)p.M * p.N * 4;
  if (!p.ws || ws_bytes < per_split * 2) splits = 1;
  else if (splits * per_split > ws_bytes) splits = (int)(ws_bytes / per_split);
  if (splits < 1) splits = 1;
  p.splits = splits;
  if (p.M <= 16) launch_skinny_mi<KIND, 1, OUT_DT>(p, st);
  else if (p.M <= 32) launch_skinny_mi<KIND, 2, OUT_DT>(p, st);
  else if (narrow) launch_skinny_mi<KIND, 4, OUT_DT, 64>(p, st);
  else launch_skinny_mi<KIND, 4, OUT_DT>(p, st);  // (64-row tiles for any M > 32)
}

// Decode path without split-K: blocks of 16 or 32 weight rows over the whole of K (M <= 32; M <= 64 on small weights).
// stream_rows: weight rows per block in units of 16 (1 or 2) that this kernel takes the problem with, 0 = it does not.
template <int KIND>
static int stream_rows(const GemmArgs& p) {
  if (p.M > 64 || p.K < 512) return 0;
  // Rows of weight per block (16 or 32; 0 = leave the shape to the split-K kernel), from a sweep over
  // N = 1024 ... 57344, K = 512 ... 28672 and M = 1 ... 64 with the weights rotated through more than the
  // last-level cache.  Against the split-K kernel this one saves the second launch and the partial sums,
  // which is worth a factor of up to two on small weights (1 x 3072 x 1536: 7.7 -> 4.3 us) and 5-15 % on
  // large ones; the split-K kernel is ahead where it needs no split (N >= 16384) and K is short, and for
  // more than 16 rows on large N, where this kernel's per-wave activation copies weigh more.
  int nib = 0;
  if (t_tile == 16) nib = 1;
  else if (t_tile == 32) nib = 2;
  else if (t_tile == 0) {
    // 32-row blocks move half the activation bytes per weight byte; they lose where they leave half of the
    // CUs idle (N <= 4096) or their last round is less than half full (N = 10240: 320 blocks on 256 CUs)
    const int blocks32 = (p.N + 31) / 32, rounds32 = (blocks32 + num_cus() - 1) / num_cus();
    const bool wide_ok = p.N > 4096 && (rounds32 * num_cus() - blocks32 < num_cus() / 2 || rounds32 > 3);
    // (more than 128 weight tiles: the split-K kernel then runs unsplit, one launch; at N = 16384 it splits in
    // two and loses, 16 x 16384 x 1024: 8.3 us against 5.5 us here)
    const bool short_k_no_split = p.K < 2048 && p.N > 16384;
    if (p.M <= 16) {
      if (short_k_no_split) nib = 0;
      // (long K: 16-row blocks except where they fill between one and one and a half rounds of the CUs;
      // 8 x 57344 x 8192: 83 against 93 us, 8 x 5120 x 13824: 19.1 against 16.3 us)
      else if (p.K >= 8192) nib = (p.N > 4096 && p.N <= 6144) ? 2 : 1;
      else nib = wide_ok ? 2 : 1;
    } else if (p.M <= 32) {
      if (short_k_no_split || p.N >= 18432 || (p.N >= 10240 && p.K >= 7168)) nib = 0;
      else if (p.K >= 8192) nib = p.N <= 4096 ? 1 : 2;
      else nib = wide_ok ? 2 : 1;
    } else {
      // 64 activation rows (8 KiB per K block and wave, one block per CU): on weights of up to 30 MB with few
      // enough blocks (64 x 4096 x 7168: 14.1 -> 10.3 us, 64 x 4096 x 4096: 14.8 -> 8.3 us; but
      // 64 x 8192 x 8192: 22 -> 27 us and 64 x 13824 x 2048: 14.4 -> 15.8 us)
      nib = ((int64_t)p.N * p.K <= (30 << 20) && p.N <= 10240) ? 1 : 0;
      // (32-row blocks where they fill most of one round: 64 x 6144 x 4096, 192 blocks, 13.4 -> 10.1 us)
      if (nib == 1 && 8 * blocks32 >= 5 * num_cus() && blocks32 <= num_cus()) nib = 2;
      // ... and with 32-row blocks where those fill exactly one round of the CUs (half the activation bytes per
      // weight byte of the 16-row blocks; 64 x 8192 x 8192: 21.3 us on the split-K kernel, 20.4 us here,
      // 33 x 8192 x 8192: 20.2 -> 18.5 us; with 224 blocks, 64 x 7168 x 16384, it loses: 32.7 -> 34.2 us)
      if (nib == 0 && p.K >= 8192 && blocks32 <= num_cus() && 16 * blocks32 > 15 * num_cus()) nib = 2;
    }
    if (nib == 2 && p.N < 2048) nib = 1;
    // narrow weights: 16-row blocks (8 x 512 x 7168: 14.2 us on the split-K kernel, two launches, 5.8 us here;
    // 32 x 256 x 7168: 14.1 -> 6.8 us; 64 x 512 x 7168: 11.4 -> 8.4 us, 64 x 768 x 2048: 9.2 -> 4.7 us)
    if (p.N < 1024) nib = 1;
  }
  return nib;
}

template <int KIND, int OUT_DT>
static bool launch_stream(GemmArgs& p, hipStream_t st) {
  const int nib = stream_rows<KIND>(p);
  if (nib == 0) return false;
  expand_packed_scales(p, st);
  p.splits = 1;
  p.tiles_m = 1;
  p.tiles_n = (p.N + 16 * nib - 1) / (16 * nib);
  const dim3 grid((uint32_t)p.tiles_n), block(256);
  g_last_kernel = nib == 1 ? "gemm_stream_kernel<16 rows>" : "gemm_stream_kernel<32 rows>";
  if (p.M <= 16) {
    if (nib == 1) gemm_stream_kernel<KIND, 1, 1, OUT_DT><<<grid, block, 0, st>>>(p);
    else gemm_stream_kernel<KIND, 1, 2, OUT_DT><<<grid, block, 0, st>>>(p);
  } else if (p.M <= 32) {
    if (nib == 1) gemm_stream_kernel<KIND, 2, 1, OUT_DT><<<grid, block, 0, st>>>(p);
    else gemm_stream_kernel<KIND, 2, 2, OUT_DT><<<grid, block, 0, st>>>(p);
  } else {
    if (nib == 1) gemm_stream_kernel<KIND, 4, 1, OUT_DT><<<grid, block, 0, st>>>(p);
    else gemm_stream_kernel<KIND, 4, 2, OUT_DT><<<grid, block, 0, st>>>(p);
  }
  return true;
}

// 64 < M <= 512 on the full-K decode kernel: 64 x 64 tiles, one block per tile (its four waves take every fourth K
// block each and read their operands from LDS once, where the split-K kernel's waves all read the tile's
// activation rows).  A K block takes 0.24 us there whatever the kind, against 0.32 us (block-scaled kinds) on the
// split-K kernel with 64 weight rows per block: it pays for the block-scaled kinds while the tiles fit one per CU
// (256 x 4096 x 7168: 23.1 -> 20.9 us, 512 x 2048 x 7168: 22.5 -> 19.0 us, 384 x 2048 x 4096: 14.3 -> 12.8 us), not beyond
// (one block per CU: 512 x 4096 x 4096 24.5 against 20.7 us) and not where the split-K kernel splits well
// (128 x 2048 x 7168: 20.1 against 13.7 us).  All times with the weights rotated past the last-level cache.
template <int KIND>
static int stream_tiles_choice(const GemmArgs& p) {  // 0: the split-K kernel; 68: 64 x 64 tiles; 69: 32 x 64 tiles
  if (p.M <= 64 || p.K < 512) return 0;
  const int nkb = p.K >> 7;
  const double wide = skinny_cost(p.M, p.N, p.K, 128, skinny_splits(p.M, p.N, p.K, 128));
  const double narrow = skinny_cost(p.M, p.N, p.K, 64, skinny_splits(p.M, p.N, p.K, 64));
  // (the split-K kernel's steps are a quarter shorter for the kinds without block scales than the model's)
  const double split_k = 0.95 * (is_block(KIND) ? 1.0 : 0.8) * (wide < narrow ? wide : narrow);
  // 32 x 64 tiles while those fit one per CU: three stages of 12.5 KiB per wave, 100 KiB in flight per CU instead of
  // 66, and a K block of half the work takes 0.17 us with the weights coming from HBM (256 x 2048 x 7168 block-FP8:
  // 16.7 us on the split-K kernel, 19.3 us on 64 x 64 tiles, 14.6 us here; 256 x 2048 x 4096: 14.3 / 12.9 / 10.2 us;
  // 128 x 4096 x 4096 per-channel FP8: 13.1 -> 11.2 us); any kind.  Few tiles and a long K stay with the split-K
  // kernel, which spreads the K blocks over the idle CUs (96 x 2048 x 7168: 12.6 us there, 15.2 us here).
  const int tiles32 = ((p.M + 31) / 32) * ((p.N + 63) / 64);
  if (tiles32 <= num_cus() && 1.0 + 0.17 * nkb < split_k) return 69;
  if (!is_block(KIND)) return 0;
  const int tiles = ((p.M + 63) / 64) * ((p.N + 63) / 64);
  if (tiles > num_cus()) return 0;
  // (few tiles and a long K: the split-K kernel spreads the K blocks over the CUs that this kernel leaves idle;
  // 128 x 4096 x 7168, 128 tiles: 18.9 us here, 16.4 us there with four splits)
  if (!(2 * tiles > num_cus() || (nkb <= 32 && 4 * tiles > num_cus()) || nkb <= 16)) return 0;
  // (1 us more than the split-K kernel per launch: the partial sums' way through LDS at the end)
  return 1.0 + 0.24 * nkb < split_k ? 68 : 0;
}

template <int KIND, int OUT_DT>
static void launch_stream_tiles(GemmArgs& p, hipStream_t st, bool half_rows = false) {
  expand_packed_scales(p, st);
  p.splits = 1;
  p.tiles_m = half_rows ? (p.M + 31) / 32 : (p.M + 63) / 64;
  p.tiles_n = (p.N + 63) / 64;
  const dim3 grid((uint32_t)(p.tiles_m * p.tiles_n)), block(256);
  if (half_rows) {
    g_last_kernel = "gemm_stream_kernel<32 x 64 tiles>";
    gemm_stream_kernel<KIND, 2, 4, OUT_DT, true><<<grid, block, 0, st>>>(p);
  } else {
    g_last_kernel = "gemm_stream_kernel<64 x 64 tiles>";
    gemm_stream_kernel<KIND, 4, 4, OUT_DT, true><<<grid, block, 0, st>>>(p);
  }
}

// Tuned kernel selections per problem, the counterpart of the reference's per-(N, K) JSON
// tables for its Triton kernels (python/sglang/srt/layers/quantization/fp8_kernel.py:738-776,
// layers/quantization/configs/): an entry names the kernel (a code of sglq_debug_force_tile)
// and the split-K factor for kind, N, K and a range of M.  Normally filled once at start-up through
// sglq_tuned_add; a reader/writer lock makes later additions safe against GEMM calls on other
// threads (an uncontended shared lock costs tens of nanoseconds per GEMM call).
struct TunedEntry {
  int kind;
  int64_t n, k, m_lo, m_hi;
  int tile, splits;
};
constexpr int MAX_TUNED = 1024;
static TunedEntry g_tuned[MAX_TUNED];
static int g_num_tuned = 0;
static std::shared_mutex g_tuned_lock;

static bool tuned_lookup(int kind, int64_t m, int64_t n, int64_t k, int& tile, int& splits) {
  std::shared_lock<std::shared_mutex> guard(g_tuned_lock);
  for (int i = 0; i < g_num_tuned; ++i) {
    const TunedEntry& e = g_tuned[i];
    if (e.kind == kind && e.n == n && e.k == k && m >= e.m_lo && m <= e.m_hi) {
      tile = e.tile;
      splits = e.splits;
      return true;
    }
  }
  return false;
}

// The selection in force for this call: the calling thread's test hooks, else a tuned entry.
static void pick_selection(int kind, const GemmArgs& p) {
  t_tile = g_force_tile;
  t_splits = g_force_splits;
  if (t_tile == 0 && t_splits == 0) {
    int tile = 0, splits = 0;
    if (tuned_lookup(kind, p.M, p.N, p.K, tile, splits)) {
      t_tile = tile;
      t_splits = splits;
    }
  }
}

// Whether the decode kernel without split-K takes this problem (and with how many weight rows per block).
template <int KIND>
static int stream_choice(const GemmArgs& p) {
  if ((p.K & 127) == 0 && p.M <= 64 && g_use_dma && (t_tile == 0 || t_tile == 16 || t_tile == 32)) return stream_rows<KIND>(p);
  return 0;
}

template <int KIND, int OUT_DT>
static void launch_kind(GemmArgs& p, int64_t ws_bytes, hipStream_t st) {
  pick_selection(KIND, p);
  if ((p.K & 127) == 0 && p.M <= 64 && g_use_dma && (t_tile == 0 || t_tile == 16 || t_tile == 32) &&
      launch_stream<KIND, OUT_DT>(p, st))
    return;
  // The same kernel with several 64-row tiles per weight tile (side by side on one XCD) takes up to 512 rows
  // from the 128-row kernels where its blocks fit the chip at once (two per CU), a block has at most 56 K
  // blocks to walk after the split, and, beyond two row tiles, the weights are small enough for the row tiles'
  // re-reads to stay in the caches.  Measured per kind over M = 96 ... 512 on 17 weight shapes, e.g. block-scaled
  // FP8 256 x 4096 x 7168: 24.6 us on the pipelined 128-row kernel, 21.8 us here; 512 x 4096 x 4096: 24.7 -> 19.7;
  // 128 x 14336 x 4096: 28.8 -> 22.3; but 160 x 14336 x 4096 (59 MB, three row tiles): 30.7 against 33.5,
  // 160 x 8192 x 8192 (64 K blocks per block): 31.2 against 35.2, 160 x 24576 x 1536 (576 tiles): 18.5 against 22.9;
  // with two row tiles up to 64 MB of weights (128 x 8192 x 8192: 29.8 -> 27.3 us, but 96 x 5120 x 13824, 68 MB:
  // 28.5 against 35.3, 96 x 18432 x 7168: 43.5 against 55.4).
  const int64_t weight_bytes = (int64_t)p.N * p.K;
  // (K blocks per block counted with no more blocks than CUs: 96 x 7168 x 16384 with three splits, 336 blocks of
  // 43 K blocks over 117 MB of weights, takes 50 us against 35; and, for the block-scaled kinds, not 41-56 K blocks on
  // fewer than 224 blocks: 384 x 4096 x 7168, 192 blocks, 30 us against 26-28, where the 256 blocks of 512 rows take 30
  // against 32; per-channel FP8 takes 23 us there against 28)
  const int skinny_tiles = ((p.M + 63) / 64) * ((p.N + 127) / 128);
  int skinny_fit = skinny_splits(p.M, p.N, p.K);
  if (skinny_fit * skinny_tiles > 256) skinny_fit = 256 / skinny_tiles > 0 ? 256 / skinny_tiles : 1;
  const int skinny_steps = ((p.K >> 7) + skinny_fit - 1) / skinny_fit;
  const bool skinny_mid = p.M <= 512 && skinny_tiles <= 512 && skinny_steps <= 56 && weight_bytes <= (p.M <= 128 ? (64 << 20) : (48 << 20) - 1) &&
                          !(is_block(KIND) && skinny_steps > 40 && skinny_fit * skinny_tiles < 224);
  if ((p.K & 127) == 0 && p.K >= 512 && g_use_dma && (t_tile == 68 || t_tile == 69) && p.M > 32 && p.M <= 1024) {
    launch_stream_tiles<KIND, OUT_DT>(p, st, t_tile == 69);
    return;
  }
  const bool skinny_rows = p.M <= 64 || skinny_mid || ((t_tile == 64 || t_tile == 66) && p.M <= 512);
  if ((p.K & 127) == 0 && g_use_dma && t_tile == 0 && p.M > 64 && p.M <= 512) {
    // (32 x 64 tiles also where the split-K kernel is not in the running: K blocks beyond its 56 per block)
    const int tiles_code = stream_tiles_choice<KIND>(p);
    if (tiles_code == 69 || (tiles_code == 68 && skinny_rows)) {
      launch_stream_tiles<KIND, OUT_DT>(p, st, tiles_code == 69);
      return;
    }
  }
  if ((p.K & 127) == 0 && skinny_rows && g_use_dma && (t_tile == 0 || t_tile == 64 || t_tile == 66)) {
    launch_skinny<KIND, OUT_DT>(p, ws_bytes, st);
    return;
  }
  // Measured crossover: the 256 x 256 kernel wins once its tiles cover more than half of
  // the 256 CUs (e.g. 144 tiles at M = 4096, N = 2112; 192 at M = 512, N = 24576); with
  // fewer tiles the 128 x 128 kernel with split-K keeps more CUs busy.
  const int big_tiles = ((p.M + 255) / 256) * ((p.N + 255) / 256);
  // ... unless the problem is large and deep enough for the pipelined kernel with K split over
  // (tile, K range) units: 512 x 7168 x 16384 90.6 -> 75.6 us, 1024 x 7168 x 16384 164.5 -> 122.6 us,
  // but 1024 x 4096 x 7168 49 -> 56 us (measured).
  bool deep = p.M > 256 && (p.K >> 7) >= 64 && 2.0 * p.M * p.N * p.K >= 1e11;
  if (deep && big_tiles < 140 && t_tile == 0 && p.K >= 384) {
    // ... and the 128-row tiles do not fill the chip better (1024 x 8192 x 8192: 81 us with 256-row tiles and
    // K split in two, 66 us with 128-row tiles, one per CU)
    int s128, s256;
    if (model_pipe_splits(p, 128, ws_bytes, s128) < model_pipe_splits(p, 256, ws_bytes, s256)) deep = false;
  }
  if (KIND == KIND_FP8_BLOCK && t_tile == 193 && (p.K & 127) == 0 && p.K >= 384 && !p.bias) {
    launch_wide_192rows<KIND, OUT_DT>(p, st);
    return;
  }
  const bool forced_256 = t_tile == 256 || t_tile == 258 || t_tile == 259 || t_tile == 192 || t_tile == 224 || t_tile == 257;
  // (up to 128 rows a 256-row tile is half empty: 96 x 36864 x 7168 73.2 us on 192-wide tiles, 65.1 us on 128-row
  // tiles; block-scaled INT8 with one or two K blocks runs 20-35 % faster on the 128 x 128 kernel than on the
  // unpipelined 256 x 256 one: 4096 x 7168 x 128 33.0 -> 27.3 us, 3072 x 7168 x 256 35.7 -> 26.2 us)
  // (block-INT8 with four K blocks and fewer than 2048 rows: 128-row tiles, 1024 x 32768 x 512 47.9 -> 32.4 us)
  const bool rows_256 = p.M > 128 && !(KIND == KIND_I8_BLOCK && (p.K < 384 || (p.K <= 512 && p.M < 2048)));
  if ((p.K & 127) == 0 && (forced_256 || (t_tile == 0 && g_use_dma && rows_256 && (big_tiles >= 140 || deep)))) {
    int width = t_tile == 0 ? (big_tiles >= 140 ? pick_tile_width(p, KIND == KIND_I8_BLOCK && p.K <= 2048 && p.M >= 2048) : 256) : t_tile;
    if (p.K < 384 && width != 256) width = 258;  // the 4 x 2-wave kernel needs three K blocks
    if (KIND == KIND_FP8_BLOCK && t_tile == 0 && big_tiles >= 140 && p.K >= 384 && !p.bias && !can_hw_scale<KIND, OUT_DT>(p)) {
      // 192 x 192 tiles where they fill the rounds of the CUs better: rounds x tile area, with 22 % more time per
      // area for the smaller tile when the chip is full (4096 x 2112 x 7168: 176 tiles of 256 x 192 take 66.2 us,
      // 242 of 192 x 192 61.4 us; 8192 x 2112 x 7168: 132.9 -> 117 us; 4096 x 4096 x 7168, two rounds of 192 x 192
      // against one of 256 x 256: 97 -> 116 us)
      const int cus = num_cus();
      const int t256 = ((p.M + 255) / 256) * ((p.N + width - 1) / (width == 258 ? 256 : width));
      const int t192 = ((p.M + 191) / 192) * ((p.N + 191) / 192);
      const double c256 = (double)((t256 + cus - 1) / cus) * 256.0 * (width == 258 || width == 257 ? 256 : width);
      const double c192 = (double)((t192 + cus - 1) / cus) * 192.0 * 192.0 * 1.22;
      if (c192 < c256) {
        launch_wide_192rows<KIND, OUT_DT>(p, st);
        return;
      }
    }
    if (width == 192) launch_wide<KIND, OUT_DT, 6>(p, st);
    else if (width == 224) launch_wide<KIND, OUT_DT, 7>(p, st);
    else if (width == 257) launch_wide<KIND, OUT_DT, 8>(p, st);
    else launch_big<KIND, OUT_DT>(p, ws_bytes, st);
    return;
  }
  // Between the two: the pipelined kernel with 128-row tiles and K split over work units.
  // Measured against the 128 x 128 kernel: 256 x 7168 x 16384 64 -> 44 us, 1024 x 7168 x 2048
  // 26 -> 20 us, 2048 x 4096 x 7168 74 -> 58 us, 2048 x 2112 x 7168 64 -> 48 us; below 256 rows
  // it only wins on large weights (256 x 24576 x 1536 22 -> 17 us, but 256 x 2112 x 7168 19 -> 21 us).
  // ... and on wide ones (160 x 12288 x 1536: 22.3 -> 13.7 us, 256 x 32768 x 512: 13.3 -> 11.2 us)
  const bool mid = p.M > 256 || (p.M > 128 && weight_bytes >= (24 << 20)) || (p.M > 64 && weight_bytes >= (48 << 20)) ||
                   (p.M > 128 && weight_bytes >= (16 << 20) && p.N >= 12288);
  if ((p.K & 127) == 0 && p.K >= 384 && (t_tile == 130 || (t_tile == 0 && g_use_dma && mid))) {
    launch_pipe128<KIND, OUT_DT>(p, ws_bytes, st);
    return;
  }
  if (p.M <= 32) launch_cfg<KIND, 32, 128, 1, 4, OUT_DT>(p, ws_bytes, st);
  else if (p.M <= 64) launch_cfg<KIND, 64, 128, 1, 4, OUT_DT>(p, ws_bytes, st);
  else launch_cfg<KIND, 128, 128, 2, 2, OUT_DT>(p, ws_bytes, st);
}

static int gemm_common_checks(const char* name, const void* a, int64_t lda, const void* b, int64_t ldb,
                              const void* out, int64_t ldo, int64_t M, int64_t N, int64_t K, int out_elem_bytes) {
  if (M < 0 || N < 0 || K < 0) {
    set_error("%s: negative dimension", name);
    return SGLQ_EINVAL;
  }
  if (M == 0 || N == 0) return -1;  // nothing to do
  if (!a || !b || !out) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (K == 0 || K % 16 != 0) {
    set_error("%s: K (%lld) must be a positive multiple of 16", name, (long long)K);
    return SGLQ_EINVAL;
  }
  if (lda % 16 != 0 || ldb % 16 != 0 || lda < K || ldb < K) {
    set_error("%s: lda/ldb must be multiples of 16 and >= K", name);
    return SGLQ_EINVAL;
  }
  if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15)) {
    set_error("%s: mat_a and mat_b must be 16-byte aligned", name);
    return SGLQ_EINVAL;
  }
  // Output rows are written in 16-byte pieces: N and ldo multiples of 16 bytes' worth of elements,
  // the base 16-byte aligned (the reference asks the same of its outputs: int8_gemm_kernel.cu:679,
  // fp8_gemm_kernel.cu:1108, fp8_blockwise_gemm_kernel.cu:383).
  const int64_t per16 = 16 / out_elem_bytes;
  if (N % per16 != 0 || ldo % per16 != 0 || ldo < N || (reinterpret_cast<uintptr_t>(out) & 15)) {
    set_error("%s: N (%lld) and ldo (%lld) must be multiples of %lld and out 16-byte aligned", name, (long long)N,
              (long long)ldo, (long long)per16);
    return SGLQ_EINVAL;
  }
  const int64_t a_bytes = (M - 1) * lda + K, b_bytes = (N - 1) * ldb + K;
  if (a_bytes >= (1ll << 31) || b_bytes >= (1ll << 31) || M >= (1 << 30) || N >= (1 << 30)) {
    set_error("%s: operand larger than 2 GiB is not supported", name);
    return SGLQ_EUNSUPPORTED;
  }
  return SGLQ_OK;
}

static void fill_common(GemmArgs& p, const void* a, int64_t lda, const void* b, int64_t ldb, void* out, int64_t ldo,
                        int64_t M, int64_t N, int64_t K) {
  p = GemmArgs{};
  p.a = static_cast<const char*>(a);
  p.b = static_cast<const char*>(b);
  p.out = out;
  p.lda = (uint32_t)lda;
  p.ldb = (uint32_t)ldb;
  p.ldo = ldo;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.a_bytes = (uint32_t)((M - 1) * lda + K);
  p.b_bytes = (uint32_t)((N - 1) * ldb + K);
  // 256 MB of last-level cache: an output well beyond it is written past the caches (8192 x 32768 x 512,
  // 537 MB: 236 -> 199 us); one that fits is better left there for the kernel that reads it next
  // (4096 x 32768 x 512, 268 MB: 97 -> 108 us with the hint)
  p.stream_out = 2 * M * N > (int64_t)384 << 20;
}

static int finish(const char* name) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", name, hipGetErrorString(e));
    return SGLQ_ELAUNCH;
  }
  return SGLQ_OK;
}

}  // namespace sglq

using namespace sglq;

// Test hook: choose between direct-to-LDS buffer loads (default) and loads staged
// through registers.  Both fill LDS identically.
extern "C" void sglq_debug_set_direct_lds(int on) { g_use_dma = on != 0; }
extern "C" void sglq_debug_force_tile(int tile) { g_force_tile = tile; }
extern "C" void sglq_debug_force_splits(int splits) { g_force_splits = splits; }
extern "C" int sglq_tuned_clear(void) {
  std::unique_lock<std::shared_mutex> guard(g_tuned_lock);
  g_num_tuned = 0;
  return SGLQ_OK;
}
extern "C" int sglq_tuned_add(int kind, int64_t N, int64_t K, int64_t m_lo, int64_t m_hi, int tile, int splits) {
  static const int tiles[] = {0, 16, 32, 64, 66, 68, 69, 128, 130, 192, 193, 224, 256, 257, 258, 259};
  bool known = false;
  for (int t : tiles) known = known || t == tile;
  if (kind < 0 || kind > 4 || N <= 0 || K <= 0 || m_lo < 0 || m_hi < m_lo || !known || splits < 0 || splits > 64) {
    set_error("tuned_add: kind 0..4, positive N and K, 0 <= m_lo <= m_hi, a known kernel code and 0 <= splits <= 64 expected");
    return SGLQ_EINVAL;
  }
  std::unique_lock<std::shared_mutex> guard(g_tuned_lock);
  if (g_num_tuned >= MAX_TUNED) {
    set_error("tuned_add: the table holds %d entries", MAX_TUNED);
    return SGLQ_EUNSUPPORTED;
  }
  g_tuned[g_num_tuned++] = TunedEntry{kind, N, K, m_lo, m_hi, tile, splits};
  return SGLQ_OK;
}

extern "C" void sglq_debug_grouped_tile(int rows) {
  g_grouped_tile = (rows == 32 || rows == 64 || rows == 128 || rows == 130 || rows == 256) ? rows : 0;
}
extern "C" const char* sglq_debug_last_gemm_kernel(void) { return g_last_kernel; }
extern "C" int sglq_debug_last_gemm_hw_scaled(void) { return g_last_hw_scaled ? 1 : 0; }

template <int KIND>
static int blockwise_entry(const char* name, const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                           int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb, int64_t sfb_stride_k,
                           int64_t sfb_stride_n, const void* bias, void* out, int64_t ldo, int out_dtype, int64_t M,
                           int64_t N, int64_t K, void* workspace, int64_t workspace_bytes, void* stream, bool pow2_scales = false,
                           bool sfa_packed = false) {
  int rc = gemm_common_checks(name, a, lda, b, ldb, out, ldo, M, N, K, 2);
  if (rc < 0) return SGLQ_OK;
  if (rc) return rc;
  if (!sfa || !sfb) {
    set_error("%s: null scale pointer", name);
    return SGLQ_EINVAL;
  }
  if (out_dtype != SGLQ_BF16 && out_dtype != SGLQ_FP16) {
    set_error("%s: out_dtype must be Half or BFloat16", name);
    return SGLQ_EINVAL;
  }
  GemmArgs p;
  fill_common(p, a, lda, b, ldb, out, ldo, M, N, K);
  p.sa = sfa;
  p.sb = sfb;
  p.bias = bias;
  p.sa_stride_m = sfa_stride_m;
  p.sa_stride_k = sfa_stride_k;
  p.sb_stride_k = sfb_stride_k;
  p.sb_stride_n = sfb_stride_n;
  if (sfa_packed) {
    // The head of the workspace takes the scales as fp32 for the kernels that do not read the packed words
    // (decode and split-K shapes, outputs other than bf16); split-K partial sums get the rest.
    if (K % 128 != 0) {
      set_error("%s: K (%lld) must be a multiple of 128 for packed scales", name, (long long)K);
      return SGLQ_EINVAL;
    }
    const int64_t need = (M * (K / 128) * 4 + 255) & ~(int64_t)255;
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 3)) {
      set_error("%s: the workspace must hold M * K / 128 floats (%lld bytes) for the expanded scales", name, (long long)need);
      return SGLQ_EINVAL;
    }
    p.sa_packed = 1;
    p.sa_expanded = static_cast<float*>(workspace);
    workspace = static_cast<char*>(workspace) + need;
    workspace_bytes -= need;
  }
  p.ws = workspace;
  p.pow2_scales = pow2_scales ? 1 : 0;
  g_last_hw_scaled = false;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (out_dtype == SGLQ_BF16) launch_kind<KIND, SGLQ_BF16>(p, workspace_bytes, st);
  else launch_kind<KIND, SGLQ_FP16>(p, workspace_bytes, st);
  return finish(name);
}

extern "C" int sglq_fp8_blockwise_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                            int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                            int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                            int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                            int64_t workspace_bytes, void* stream) {
  return blockwise_entry<KIND_FP8_BLOCK>("fp8_blockwise_scaled_mm", a, lda, b, ldb, sfa, sfa_stride_m, sfa_stride_k, sfb,
                                         sfb_stride_k, sfb_stride_n, nullptr, out, ldo, out_dtype, M, N, K, workspace,
                                         workspace_bytes, stream);
}

extern "C" int sglq_fp8_blockwise_scaled_mm_ue8m0(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                                  int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                                  int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                                  int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                                  int64_t workspace_bytes, void* stream) {
  return blockwise_entry<KIND_FP8_BLOCK>("fp8_blockwise_scaled_mm_ue8m0", a, lda, b, ldb, sfa, sfa_stride_m, sfa_stride_k, sfb,
                                         sfb_stride_k, sfb_stride_n, nullptr, out, ldo, out_dtype, M, N, K, workspace,
                                         workspace_bytes, stream, true);
}

extern "C" int sglq_fp8_blockwise_scaled_mm_ue8m0_packed(const void* a, int64_t lda, const void* b, int64_t ldb, const int32_t* sfa_packed,
                                                         int64_t sfa_stride_m, int64_t sfa_stride_k4, const float* sfb,
                                                         int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                                         int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                                         int64_t workspace_bytes, void* stream) {
  return blockwise_entry<KIND_FP8_BLOCK>("fp8_blockwise_scaled_mm_ue8m0_packed", a, lda, b, ldb, reinterpret_cast<const float*>(sfa_packed),
                                         sfa_stride_m, sfa_stride_k4, sfb, sfb_stride_k, sfb_stride_n, nullptr, out, ldo, out_dtype, M, N,
                                         K, workspace, workspace_bytes, stream, true, true);
}

extern "C" int sglq_fp8_blockwise_scaled_mm_bias(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                                 int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                                 int64_t sfb_stride_k, int64_t sfb_stride_n, const void* bias, void* out,
                                                 int64_t ldo, int out_dtype, int64_t M, int64_t N, int64_t K,
                                                 void* workspace, int64_t workspace_bytes, void* stream) {
  return blockwise_entry<KIND_FP8_BLOCK>("fp8_blockwise_scaled_mm_bias", a, lda, b, ldb, sfa, sfa_stride_m, sfa_stride_k,
                                         sfb, sfb_stride_k, sfb_stride_n, bias, out, ldo, out_dtype, M, N, K, workspace,
                                         workspace_bytes, stream);
}

extern "C" int sglq_fp8_blockwise_scaled_grouped_mm(const void* a, int64_t lda, const void* b, int64_t ldb,
                                                    int64_t b_expert_stride, const float* sfa, int64_t sfa_stride_m,
                                                    int64_t sfa_stride_k, const float* sfb, int64_t sfb_expert_stride,
                                                    int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                                    int out_dtype, const int32_t* problem_sizes,
                                                    const int32_t* expert_offsets, int64_t num_experts, int64_t total_m,
                                                    int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                                    void* stream) {
  using namespace sglq;
  const char* name = "fp8_blockwise_scaled_grouped_mm";
  if (num_experts < 0) {
    set_error("%s: negative number of experts", name);
    return SGLQ_EINVAL;
  }
  int rc = gemm_common_checks(name, a, lda, b, ldb, out, ldo, total_m, N, K, 2);
  if (rc < 0 || num_experts == 0) return SGLQ_OK;
  if (rc) return rc;
  if (!sfa || !sfb || !problem_sizes || !expert_offsets) {
    set_error("%s: null scale, problem_sizes or expert_offsets pointer", name);
    return SGLQ_EINVAL;
  }
  if (out_dtype != SGLQ_BF16 && out_dtype != SGLQ_FP16) {
    set_error("%s: output must be bfloat16 or half", name);
    return SGLQ_EINVAL;
  }
  if (K % 128 != 0) {
    set_error("%s: K (%lld) must be a multiple of 128", name, (long long)K);
    return SGLQ_EINVAL;
  }
  if (b_expert_stride % 16 != 0 || num_experts >= (1 << 20)) {
    set_error("%s: the experts' weights must be 16-byte aligned, fewer than 2^20 experts", name);
    return SGLQ_EINVAL;
  }
  // Row tile height from the average group: the experts' row counts are device data.
  // Measured with 256 experts of 4096 x 7168 (one launch streams every expert's weight once,
  // 7.5 GB) and equal groups: below about 12 rows per expert the 128-row kernel's 64-row tiles
  // are fastest (1.30-1.32 ms, 5.7-5.8 TB/s, against 1.43-1.45 ms); from there to 128 rows per
  // expert the pipelined kernel with 128-row tiles (1.46 ms at 16 rows, 1.57 ms at 64, 1.76 ms
  // at 128, where the unpipelined 128-row tiles need 1.48, 2.23 and 3.99 ms and the pipelined
  // 256-row ones 2.1-2.2 ms whatever their fill); above 128 rows per expert two 128-row tiles
  // cost what one 256-row tile costs and the 256-row tile computes faster (2.26 against
  // 2.51 ms at 256 rows, 7.7 against 8.1 ms at 1024).
  const int64_t avg = total_m / num_experts;
  bool pipelined;
  int bm;
  if (g_grouped_tile) {  // test hook; 130 = the pipelined kernel with 128-row tiles
    pipelined = g_grouped_tile == 256 || g_grouped_tile == 130;
    bm = g_grouped_tile == 130 ? 128 : g_grouped_tile;
  } else {
    pipelined = avg >= 12 && K >= 384;
    bm = pipelined ? (avg > 128 ? 256 : 128) : avg < 12 ? 64 : 128;
  }
  if (pipelined && K < 384) {
    set_error("%s: the pipelined kernel needs K >= 384", name);
    return SGLQ_EINVAL;
  }
  const int64_t max_tiles = total_m / bm + num_experts;
  const int64_t need = (int64_t)(PLAN_HEADER + PLAN_ENTRY * max_tiles) * 4;
  if (!workspace || workspace_bytes < need) {
    set_error("%s: workspace of %lld bytes needed for the tile plan (%lld given)", name, (long long)need,
              (long long)workspace_bytes);
    return SGLQ_EINVAL;
  }
  if (max_tiles * ((N + 127) / 128) >= (1ll << 31)) {
    set_error("%s: too many tiles", name);
    return SGLQ_EUNSUPPORTED;
  }
  GemmArgs p;
  fill_common(p, a, lda, b, ldb, out, ldo, total_m, N, K);
  p.sa = sfa;
  p.sb = sfb;
  p.sa_stride_m = sfa_stride_m;
  p.sa_stride_k = sfa_stride_k;
  p.sb_stride_k = sfb_stride_k;
  p.sb_stride_n = sfb_stride_n;
  p.b_expert_stride = b_expert_stride;
  p.sb_expert_stride = sfb_expert_stride;
  p.num_experts = (int)num_experts;
  p.ws = workspace;
  hipStream_t st = static_cast<hipStream_t>(stream);
  grouped_plan_kernel<<<dim3(1), dim3(256), 0, st>>>(problem_sizes, expert_offsets, (int)num_experts, (int)total_m, bm,
                                                     (int)max_tiles, static_cast<int*>(workspace));
  if (pipelined) {
    g_last_kernel = bm == 256 ? "grouped_plan_kernel+gemm_pipe_kernel<grouped>" : "grouped_plan_kernel+gemm_pipe_kernel<grouped, 128 rows>";
    p.tiles_m = (int)max_tiles;
    p.tiles_n = (int)((N + 255) / 256);
    p.splits = 1;
    const int64_t units = max_tiles * p.tiles_n;
    const dim3 grid((uint32_t)(units < num_cus() ? units : num_cus())), block(512);
    if (bm == 256) {
      if (out_dtype == SGLQ_BF16) gemm_pipe_kernel<KIND_FP8_BLOCK, SGLQ_BF16, PIPE_GROUPED><<<grid, block, 0, st>>>(p);
      else gemm_pipe_kernel<KIND_FP8_BLOCK, SGLQ_FP16, PIPE_GROUPED><<<grid, block, 0, st>>>(p);
    } else {
      if (out_dtype == SGLQ_BF16) gemm_pipe_kernel<KIND_FP8_BLOCK, SGLQ_BF16, PIPE_GROUPED, 128><<<grid, block, 0, st>>>(p);
      else gemm_pipe_kernel<KIND_FP8_BLOCK, SGLQ_FP16, PIPE_GROUPED, 128><<<grid, block, 0, st>>>(p);
    }
    return finish(name);
  }
  g_last_kernel = "grouped_plan_kernel+gemm_kernel<grouped>";
  if (out_dtype == SGLQ_BF16) {
    if (bm == 32) launch_grouped_cfg<KIND_FP8_BLOCK, 32, 128, 1, 4, SGLQ_BF16>(p, (int)max_tiles, st);
    else if (bm == 64) launch_grouped_cfg<KIND_FP8_BLOCK, 64, 128, 1, 4, SGLQ_BF16>(p, (int)max_tiles, st);
    else launch_grouped_cfg<KIND_FP8_BLOCK, 128, 128, 2, 2, SGLQ_BF16>(p, (int)max_tiles, st);
  } else {
    if (bm == 32) launch_grouped_cfg<KIND_FP8_BLOCK, 32, 128, 1, 4, SGLQ_FP16>(p, (int)max_tiles, st);
    else if (bm == 64) launch_grouped_cfg<KIND_FP8_BLOCK, 64, 128, 1, 4, SGLQ_FP16>(p, (int)max_tiles, st);
    else launch_grouped_cfg<KIND_FP8_BLOCK, 128, 128, 2, 2, SGLQ_FP16>(p, (int)max_tiles, st);
  }
  return finish(name);
}

extern "C" int sglq_int8_blockwise_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                             int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                             int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                             int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                             int64_t workspace_bytes, void* stream) {
  return blockwise_entry<KIND_I8_BLOCK>("w8a8_block_int8_matmul", a, lda, b, ldb, sfa, sfa_stride_m, sfa_stride_k, sfb,
                                        sfb_stride_k, sfb_stride_n, nullptr, out, ldo, out_dtype, M, N, K, workspace,
                                        workspace_bytes, stream);
}

extern "C" int sglq_int8_blockwise_scaled_mm_bias(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                                  int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                                  int64_t sfb_stride_k, int64_t sfb_stride_n, const void* bias, void* out,
                                                  int64_t ldo, int out_dtype, int64_t M, int64_t N, int64_t K,
                                                  void* workspace, int64_t workspace_bytes, void* stream) {
  return blockwise_entry<KIND_I8_BLOCK>("w8a8_block_int8_matmul_bias", a, lda, b, ldb, sfa, sfa_stride_m, sfa_stride_k, sfb,
                                        sfb_stride_k, sfb_stride_n, bias, out, ldo, out_dtype, M, N, K, workspace,
                                        workspace_bytes, stream);
}

static int rowcol_entry(const char* name, bool fp8, const void* a, int64_t lda, const void* b, int64_t ldb,
                        const float* scales_a, const float* scales_b, const void* bias, void* out, int64_t ldo,
                        int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                        void* stream) {
  int rc = gemm_common_checks(name, a, lda, b, ldb, out, ldo, M, N, K, 2);
  if (rc < 0) return SGLQ_OK;
  if (rc) return rc;
  if (!scales_a || !scales_b) {
    set_error("%s: null scale pointer", name);
    return SGLQ_EINVAL;
  }
  if (reinterpret_cast<uintptr_t>(scales_b) & 15) {
    set_error("%s: scales_b must be 16-byte aligned", name);
    return SGLQ_EINVAL;
  }
  if (out_dtype != SGLQ_BF16 && out_dtype != SGLQ_FP16) {
    set_error("%s: out_dtype must be Half or BFloat16", name);
    return SGLQ_EINVAL;
  }
  GemmArgs p;
  fill_common(p, a, lda, b, ldb, out, ldo, M, N, K);
  p.sa = scales_a;
  p.sb = scales_b;
  p.bias = bias;
  p.ws = workspace;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (fp8) {
    if (out_dtype == SGLQ_BF16) launch_kind<KIND_FP8_ROWCOL, SGLQ_BF16>(p, workspace_bytes, st);
    else launch_kind<KIND_FP8_ROWCOL, SGLQ_FP16>(p, workspace_bytes, st);
  } else {
    if (out_dtype == SGLQ_BF16) launch_kind<KIND_I8_ROWCOL, SGLQ_BF16>(p, workspace_bytes, st);
    else launch_kind<KIND_I8_ROWCOL, SGLQ_FP16>(p, workspace_bytes, st);
  }
  return finish(name);
}

extern "C" int sglq_int8_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* scales_a,
                                   const float* scales_b, const void* bias, void* out, int64_t ldo, int out_dtype,
                                   int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                   void* stream) {
  return rowcol_entry("int8_scaled_mm", false, a, lda, b, ldb, scales_a, scales_b, bias, out, ldo, out_dtype, M, N, K,
                      workspace, workspace_bytes, stream);
}

extern "C" int sglq_fp8_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* scales_a,
                                  const float* scales_b, const void* bias, void* out, int64_t ldo, int out_dtype,
                                  int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                  void* stream) {
  return rowcol_entry("fp8_scaled_mm", true, a, lda, b, ldb, scales_a, scales_b, bias, out, ldo, out_dtype, M, N, K,
                      workspace, workspace_bytes, stream);
}

extern "C" int sglq_int8_mm_i32(const void* a, int64_t lda, const void* b, int64_t ldb, int32_t* out, int64_t ldo,
                                int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                void* stream) {
  const char* name = "int8_mm_i32";
  int rc = gemm_common_checks(name, a, lda, b, ldb, out, ldo, M, N, K, 4);
  if (rc < 0) return SGLQ_OK;
  if (rc) return rc;
  GemmArgs p;
  fill_common(p, a, lda, b, ldb, out, ldo, M, N, K);
  p.ws = workspace;
  launch_kind<KIND_I8_RAW, SGLQ_BF16>(p, workspace_bytes, static_cast<hipStream_t>(stream));
  return finish(name);
}

// ---------------------------------------------------------------------------
// Quantize-and-multiply in one call: per-token-group FP8 quantization (groups of 128) of 16-bit
// activations followed by the block-scaled FP8 GEMM, the pair of calls of
// cutlass_w8a8_block_fp8_linear_with_fallback (fp8_utils.py:204-209).  For M <= 4 on the shapes that the
// full-K decode kernel takes with one to 2.5 blocks per compute unit, one launch does both
// (gemm_stream_quant_kernel; for M <= 8 on any of that kernel's shapes when a 16- or 32-row block is forced
// through the test hook); otherwise the two kernels run one after the other with the codes and scales in the
// workspace.
// Either way the output is bit-identical to the two operators called in turn.
// ---------------------------------------------------------------------------
template <int OUT_DT>
static void launch_stream_quant(GemmArgs& p, int nib, int in_dtype, hipStream_t st) {
  p.splits = 1;
  p.tiles_m = 1;
  p.tiles_n = (p.N + 16 * nib - 1) / (16 * nib);
  const dim3 grid((uint32_t)p.tiles_n), block(256);
  g_last_kernel = nib == 1 ? "gemm_stream_quant_kernel<16 rows>" : "gemm_stream_quant_kernel<32 rows>";
  auto launch = [&](auto nib_tag, auto in_tag) {
    constexpr int NIB = decltype(nib_tag)::value, IN_DT = decltype(in_tag)::value;
    if (p.M <= 1) gemm_stream_quant_kernel<NIB, OUT_DT, IN_DT, 1><<<grid, block, 0, st>>>(p);
    else if (p.M <= 2) gemm_stream_quant_kernel<NIB, OUT_DT, IN_DT, 2><<<grid, block, 0, st>>>(p);
    else if (p.M <= 4) gemm_stream_quant_kernel<NIB, OUT_DT, IN_DT, 4><<<grid, block, 0, st>>>(p);
    else gemm_stream_quant_kernel<NIB, OUT_DT, IN_DT, 8><<<grid, block, 0, st>>>(p);
  };
  using one = std::integral_constant<int, 1>;
  using two = std::integral_constant<int, 2>;
  using bf16 = std::integral_constant<int, SGLQ_BF16>;
  using fp16 = std::integral_constant<int, SGLQ_FP16>;
  if (in_dtype == SGLQ_BF16) {
    if (nib == 1) launch(one{}, bf16{});
    else launch(two{}, bf16{});
  } else {
    if (nib == 1) launch(one{}, fp16{});
    else launch(two{}, fp16{});
  }
}

extern "C" int sglq_w8a8_block_fp8_linear(const void* x, int in_dtype, const void* b, int64_t ldb, const float* sfb,
                                          int64_t sfb_stride_k, int64_t sfb_stride_n, const void* bias, void* out,
                                          int64_t ldo, int out_dtype, int64_t M, int64_t N, int64_t K, float eps,
                                          void* workspace, int64_t workspace_bytes, void* stream) {
  const char* name = "w8a8_block_fp8_linear";
  if (in_dtype != SGLQ_BF16 && in_dtype != SGLQ_FP16 && in_dtype != SGLQ_FP32) {
    set_error("%s: activations must be BFloat16, Half or Float", name);
    return SGLQ_EUNSUPPORTED;
  }
  if (K > 0 && K % 128 != 0) {
    set_error("%s: K (%lld) must be a multiple of the quantization group, 128", name, (long long)K);
    return SGLQ_EINVAL;
  }
  // (x stands in for the codes: same row count, contiguous rows of K elements)
  int rc = gemm_common_checks(name, x, K, b, ldb, out, ldo, M, N, K, 2);
  if (rc < 0) return SGLQ_OK;
  if (rc) return rc;
  if (!sfb) {
    set_error("%s: null scale pointer", name);
    return SGLQ_EINVAL;
  }
  if (out_dtype != SGLQ_BF16 && out_dtype != SGLQ_FP16) {
    set_error("%s: out_dtype must be Half or BFloat16", name);
    return SGLQ_EINVAL;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (M <= 8 && in_dtype != SGLQ_FP32 && M * K * 2 < (1ll << 31)) {
    GemmArgs p;
    fill_common(p, x, K, b, ldb, out, ldo, M, N, K);
    p.sb = sfb;
    p.bias = bias;
    p.sb_stride_k = sfb_stride_k;
    p.sb_stride_n = sfb_stride_n;
    pick_selection(KIND_FP8_BLOCK, p);
    const int nib = stream_choice<KIND_FP8_BLOCK>(p);
    // Measured against the two launches (graph-timed, weights rotated past the last-level cache, DeepSeek-V3 and
    // Llama-70B shapes): the single kernel wins for M <= 4 where its blocks fill one to two and a half rounds of the
    // CUs (1 x 7168 x 16384: 27.8 -> 26.3 us, 4 x 4096 x 7168: 9.0 -> 8.2 us, 4 x 8192 x 8192: 17.1 -> 15.4 us); with
    // fewer blocks the quantization's latency is exposed (1 x 2112 x 7168: 7.5 -> 8.2 us), with many more its
    // arithmetic, repeated by every block, costs more than the launch it saves (4 x 57344 x 8192: 83.9 -> 86.7 us),
    // and from 5 rows on it loses nearly everywhere (8 x 4096 x 7168: 9.2 -> 10.1 us).  A forced 16- or 32-row
    // block (test hook) takes the single kernel for any M <= 8.
    const int blocks = nib > 0 ? (int)((N + 16 * nib - 1) / (16 * nib)) : 0;
    const bool pays = g_force_tile != 0 || (M <= 4 && blocks >= num_cus() && 2 * blocks <= 5 * num_cus());
    if (nib > 0 && pays) {
      p.lda = (uint32_t)(K * 2);  // row stride of the 16-bit activations in bytes
      p.a_bytes = (uint32_t)(M * K * 2);
      p.quant_eps = eps;
      if (out_dtype == SGLQ_BF16) launch_stream_quant<SGLQ_BF16>(p, nib, in_dtype, st);
      else launch_stream_quant<SGLQ_FP16>(p, nib, in_dtype, st);
      return finish(name);
    }
  }
  // two launches: codes [M, K] and column-major scales [M, K / 128] at the head of the workspace
  const int64_t code_bytes = (M * K + 255) / 256 * 256, scale_bytes = (M * (K / 128) * 4 + 255) / 256 * 256;
  if (!workspace || workspace_bytes < code_bytes + scale_bytes || (reinterpret_cast<uintptr_t>(workspace) & 15)) {
    set_error("%s: a 16-byte aligned workspace of at least %lld bytes is needed for the quantized activations of this shape (%lld given)",
              name, (long long)(code_bytes + scale_bytes), (long long)workspace_bytes);
    return SGLQ_EINVAL;
  }
  char* ws = static_cast<char*>(workspace);
  float* scales = reinterpret_cast<float*>(ws + code_bytes);
  rc = sglq_per_token_group_quant_fp8(x, in_dtype, ws, scales, M, K, 128, 1, M, eps, -448.0f, 448.0f, stream);
  if (rc) return rc;
  return blockwise_entry<KIND_FP8_BLOCK>(name, ws, K, b, ldb, scales, 1, M, sfb, sfb_stride_k, sfb_stride_n, bias, out, ldo, out_dtype,
                                         M, N, K, ws + code_bytes + scale_bytes, workspace_bytes - code_bytes - scale_bytes, stream);
}

// ---------------------------------------------------------------------------
// Quantize-and-multiply in one call for the per-token kinds: per-token INT8 quantization + int8_scaled_mm
// (the pair of calls of W8A8Int8LinearMethod.apply, w8a8_int8.py:387-391) and per-token FP8 quantization +
// fp8_scaled_mm (apply_fp8_linear's dynamic per-token branch, fp8_utils.py:693,725-732); the fused form is the
// reference's CPU backend's int8_scaled_mm_with_quant (sgl-kernel/csrc/cpu/gemm_int8.cpp:423-489).  For decode
// rows on the shapes that the full-K decode kernel takes, one launch does both
// (gemm_stream_tokenquant_kernel); otherwise the two kernels run one after the other with the codes and the
// row scales at the head of the workspace.  Either way the output is bit-identical to the two operators
// called in turn.
// ---------------------------------------------------------------------------
template <int KIND, int OUT_DT>
static void launch_stream_tokenquant(GemmArgs& p, int nib, int in_dtype, hipStream_t st) {
  p.splits = 1;
  p.tiles_m = 1;
  p.tiles_n = (p.N + 16 * nib - 1) / (16 * nib);
  const dim3 grid((uint32_t)p.tiles_n), block(256);
  g_last_kernel = nib == 1 ? "gemm_stream_tokenquant_kernel<16 rows>" : "gemm_stream_tokenquant_kernel<32 rows>";
  auto launch = [&](auto nib_tag, auto in_tag) {
    constexpr int NIB = decltype(nib_tag)::value, IN_DT = decltype(in_tag)::value;
    if (p.M <= 1) gemm_stream_tokenquant_kernel<KIND, NIB, OUT_DT, IN_DT, 1><<<grid, block, 0, st>>>(p);
    else if (p.M <= 2) gemm_stream_tokenquant_kernel<KIND, NIB, OUT_DT, IN_DT, 2><<<grid, block, 0, st>>>(p);
    else if (p.M <= 4) gemm_stream_tokenquant_kernel<KIND, NIB, OUT_DT, IN_DT, 4><<<grid, block, 0, st>>>(p);
    else gemm_stream_tokenquant_kernel<KIND, NIB, OUT_DT, IN_DT, 8><<<grid, block, 0, st>>>(p);
  };
  using one = std::integral_constant<int, 1>;
  using two = std::integral_constant<int, 2>;
  using bf16 = std::integral_constant<int, SGLQ_BF16>;
  using fp16 = std::integral_constant<int, SGLQ_FP16>;
  if (in_dtype == SGLQ_BF16) {
    if (nib == 1) launch(one{}, bf16{});
    else launch(two{}, bf16{});
  } else {
    if (nib == 1) launch(one{}, fp16{});
    else launch(two{}, fp16{});
  }
}

// Rows up to which the single kernel is taken without the test hook (see the measurements in tokenquant_linear_entry)
#ifndef SGLQ_TOKENQUANT_FUSED_ROWS
#define SGLQ_TOKENQUANT_FUSED_ROWS 2
#endif

template <int KIND>
static int tokenquant_linear_entry(const char* name, const void* x, int in_dtype, const void* b, int64_t ldb,
                                   const float* scales_b, const void* bias, void* out, int64_t ldo, int out_dtype,
                                   int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                   void* stream) {
  constexpr bool IS_FP8 = KIND == KIND_FP8_ROWCOL;
  if (in_dtype != SGLQ_BF16 && in_dtype != SGLQ_FP16 && in_dtype != SGLQ_FP32) {
    set_error("%s: activations must be BFloat16, Half or Float", name);
    return SGLQ_EUNSUPPORTED;
  }
  // (x stands in for the codes: same row count, contiguous rows of K elements)
  int rc = gemm_common_checks(name, x, K, b, ldb, out, ldo, M, N, K, 2);
  if (rc < 0) return SGLQ_OK;
  if (rc) return rc;
  if (!scales_b) {
    set_error("%s: null scale pointer", name);
    return SGLQ_EINVAL;
  }
  if (reinterpret_cast<uintptr_t>(scales_b) & 15) {
    set_error("%s: scales_b must be 16-byte aligned", name);
    return SGLQ_EINVAL;
  }
  if (out_dtype != SGLQ_BF16 && out_dtype != SGLQ_FP16) {
    set_error("%s: out_dtype must be Half or BFloat16", name);
    return SGLQ_EINVAL;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (M <= 8 && in_dtype != SGLQ_FP32 && K % 128 == 0 && M * K * 2 < (1ll << 31)) {
    GemmArgs p;
    fill_common(p, x, K, b, ldb, out, ldo, M, N, K);
    p.sb = scales_b;
    p.bias = bias;
    pick_selection(KIND, p);
    const int nib = stream_choice<KIND>(p);
    // Every block reads the M rows once more for their maxima (M K 2 bytes from L2 per block) before its first
    // MFMA; against that stand the quantization launch (2.4-2.8 us) and the codes' round trip.  A forced 16- or
    // 32-row block (test hook) takes the single kernel for any M <= 8.
    const bool pays = g_force_tile != 0 || M <= SGLQ_TOKENQUANT_FUSED_ROWS;
    if (nib > 0 && pays) {
      p.lda = (uint32_t)(K * 2);  // row stride of the 16-bit activations in bytes
      p.a_bytes = (uint32_t)(M * K * 2);
      if (out_dtype == SGLQ_BF16) launch_stream_tokenquant<KIND, SGLQ_BF16>(p, nib, in_dtype, st);
      else launch_stream_tokenquant<KIND, SGLQ_FP16>(p, nib, in_dtype, st);
      return finish(name);
    }
  }
  // two launches: codes [M, K] and the row scales [M] at the head of the workspace
  const int64_t code_bytes = (M * K + 255) / 256 * 256, scale_bytes = (M * 4 + 255) / 256 * 256;
  if (!workspace || workspace_bytes < code_bytes + scale_bytes || (reinterpret_cast<uintptr_t>(workspace) & 15)) {
    set_error("%s: a 16-byte aligned workspace of at least %lld bytes is needed for the quantized activations of this shape (%lld given)",
              name, (long long)(code_bytes + scale_bytes), (long long)workspace_bytes);
    return SGLQ_EINVAL;
  }
  char* ws = static_cast<char*>(workspace);
  float* scales = reinterpret_cast<float*>(ws + code_bytes);
  if (IS_FP8) rc = sglq_per_token_quant_fp8(x, in_dtype, ws, scales, M, K, stream);
  else rc = sglq_per_token_quant_int8(x, in_dtype, ws, scales, nullptr, M, K, stream);
  if (rc) return rc;
  return rowcol_entry(name, IS_FP8, ws, K, b, ldb, scales, scales_b, bias, out, ldo, out_dtype, M, N, K, ws + code_bytes + scale_bytes,
                      workspace_bytes - code_bytes - scale_bytes, stream);
}

extern "C" int sglq_w8a8_int8_linear(const void* x, int in_dtype, const void* b, int64_t ldb, const float* scales_b,
                                     const void* bias, void* out, int64_t ldo, int out_dtype, int64_t M, int64_t N,
                                     int64_t K, void* workspace, int64_t workspace_bytes, void* stream) {
  return tokenquant_linear_entry<KIND_I8_ROWCOL>("w8a8_int8_linear", x, in_dtype, b, ldb, scales_b, bias, out, ldo, out_dtype, M, N, K,
                                                 workspace, workspace_bytes, stream);
}

extern "C" int sglq_w8a8_fp8_linear(const void* x, int in_dtype, const void* b, int64_t ldb, const float* scales_b,
                                    const void* bias, void* out, int64_t ldo, int out_dtype, int64_t M, int64_t N,
                                    int64_t K, void* workspace, int64_t workspace_bytes, void* stream) {
  return tokenquant_linear_entry<KIND_FP8_ROWCOL>("w8a8_fp8_linear", x, in_dtype, b, ldb, scales_b, bias, out, ldo, out_dtype, M, N, K,
                                                  workspace, workspace_bytes, stream);
}

// ---------------------------------------------------------------------------
// The block-scaled FP8 GEMM for callers that cannot allocate device memory (code under HIP
// graph capture, serving loops, harnesses that forbid it): the split-K partial sums pass through
// a fixed array in device memory instead of a caller workspace.  Every GPU the library runs on
// holds its own copy of the array, at its own address, until the process ends.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[SGLQ_NOALLOC_SCRATCH_BYTES];

// In host code `scratch` is a stand-in for the symbol, not a device address: the address of the
// current device's copy comes from hipGetSymbolAddress, once per device.
static std::mutex g_scratch_lock;
static void* g_scratch_ptr[sglq::MAX_DEVICES];

static int scratch_of_current_device(const char* name, void** ptr_out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("%s: hipGetDevice failed: %s", name, hipGetErrorString(e));
    return SGLQ_ELAUNCH;
  }
  if (dev < 0 || dev >= sglq::MAX_DEVICES) {
    set_error("%s: device ordinal %d is beyond the %d this library keeps scratch addresses for", name, dev, sglq::MAX_DEVICES);
    return SGLQ_EUNSUPPORTED;
  }
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", name, dev, hipGetErrorString(e));
      return SGLQ_ELAUNCH;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *ptr_out = g_scratch_ptr[dev];
  return SGLQ_OK;
}

extern "C" int sglq_init(void) {
  void* ptr = nullptr;
  return scratch_of_current_device("sglq_init", &ptr);
}

extern "C" int sglq_fp8_blockwise_scaled_mm_noalloc(const void* a, int64_t lda, const void* b, int64_t ldb,
                                                    const float* sfa, int64_t sfa_stride_m, int64_t sfa_stride_k,
                                                    const float* sfb, int64_t sfb_stride_k, int64_t sfb_stride_n,
                                                    void* out, int64_t ldo, int out_dtype, int64_t M, int64_t N,
                                                    int64_t K, void* stream) {
  const char* name = "fp8_blockwise_scaled_mm_noalloc";
  // The scratch holds split-K partial sums: two fp32 per output must fit for K to be split at all, i.e. up to
  // SGLQ_NOALLOC_MAX_OUTPUTS outputs.  Larger outputs run unsplit and do not touch the scratch (the launchers fall
  // back to one split when the workspace is too small, exactly as the workspace entry point does with a workspace
  // of this size), so they are served as well; sizes beyond what the library addresses at all (operands of 2 GiB,
  // 2^30 rows or columns) are rejected by the common checks with their message.
  void* ws = nullptr;
  const int rc = scratch_of_current_device(name, &ws);
  if (rc) return rc;
  // The partial sums of a split are written in full before the reduction reads them, so nothing
  // in the scratch has to start at zero and no clearing pass is needed.
  return blockwise_entry<KIND_FP8_BLOCK>(name, a, lda, b, ldb, sfa, sfa_stride_m, sfa_stride_k, sfb, sfb_stride_k, sfb_stride_n,
                                         nullptr, out, ldo, out_dtype, M, N, K, ws, SGLQ_NOALLOC_SCRATCH_BYTES, stream);
}
