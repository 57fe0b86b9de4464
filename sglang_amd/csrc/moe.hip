// The data movement around the grouped (MoE) block-scaled FP8 GEMM on gfx950: routing
// tables from the top-k expert ids, row gathers into expert-major order, SiLU-and-multiply
// between the two GEMMs, and the weighted combine back to token order.  All HBM-bound.
#include "sglq_common.h"

namespace sglq {

static int check_moe_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return SGLQ_ELAUNCH;
  }
  return SGLQ_OK;
}

// ---------------------------------------------------------------------------
// prepare_moe_input (sgl-kernel/csrc/moe/prepare_moe_input.cu:13-139): from topk_ids
// [topk_length] (token-major: slot i belongs to token i / topk) build
//   problem_sizes1[e] = (count_e, 2 n, k), problem_sizes2[e] = (count_e, k, n)       (:31-38)
//   expert_offsets[0 .. E] = running sum of the counts                                (:41-54)
//   blockscale_offsets[0 .. E] (optional) = running sum of the counts rounded up to 128 (:56-76)
//   input_permutation[p] = token of the slot that lands in expert-major position p     (:93)
//   output_permutation[i] = expert-major position of slot i                            (:94)
// The reference hands out positions inside an expert with atomicAdd, in whatever order the
// threads arrive; here slots keep their order (position = number of earlier slots of the same
// expert), so the tables are the same on every run.  Ids outside [0, E) belong to nobody: their
// output_permutation entries are left as they are, as in the reference.
// The counts of every expert must be known before any offset, hence three launches: count
// (one block per expert), offsets (one block scanning E values), place.  A thread looks at
// four consecutive slots at a time, a block of 1024 threads at 4096.
// ---------------------------------------------------------------------------
constexpr int MOE_THREADS = 1024, MOE_SWEEP = 4 * MOE_THREADS;

// Slots i .. i + 3; slots past the end read as -1, which is nobody's id.
SGLQ_DEV v4i load_ids4(const int* __restrict__ ids, int64_t i, int64_t n, bool aligned) {
  if (aligned && i + 3 < n) return *reinterpret_cast<const v4i*>(ids + i);
  v4i v = {-1, -1, -1, -1};
#pragma unroll
  for (int q = 0; q < 4; ++q)
    if (i + q < n) v[q] = ids[i + q];
  return v;
}

// Number of slots in [0, end) that name expert e; every thread of the block gets the sum.
SGLQ_DEV int block_count_ids(const int* __restrict__ ids, int64_t end, int e, bool aligned, int* red) {
  int c = 0;
#pragma unroll 4
  for (int64_t i = 4 * (int64_t)threadIdx.x; i < end; i += MOE_SWEEP) {
    const v4i v = load_ids4(ids, i, end, aligned);
    c += (v[0] == e) + (v[1] == e) + (v[2] == e) + (v[3] == e);
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) c += __shfl_xor(c, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
  __syncthreads();
  c = 0;
#pragma unroll
  for (int w = 0; w < MOE_THREADS / 64; ++w) c += red[w];
  __syncthreads();
  return c;
}

__global__ __launch_bounds__(MOE_THREADS) void moe_count_kernel(const int* __restrict__ topk_ids, int* __restrict__ ps1,
                                                                int* __restrict__ ps2, int64_t topk_length, int n, int k,
                                                                int aligned) {
  __shared__ int red[MOE_THREADS / 64];
  const int e = blockIdx.x;
  const int c = block_count_ids(topk_ids, topk_length, e, aligned != 0, red);
  if (threadIdx.x == 0) {
    ps1[3 * e] = c;
    ps1[3 * e + 1] = 2 * n;
    ps1[3 * e + 2] = k;
    ps2[3 * e] = c;
    ps2[3 * e + 1] = k;
    ps2[3 * e + 2] = n;
  }
}

__global__ __launch_bounds__(256) void moe_offsets_kernel(const int* __restrict__ ps1, int* __restrict__ expert_offsets,
                                                          int* __restrict__ blockscale_offsets, int num_experts) {
  __shared__ int scan[256], scan_r[256];
  __shared__ int base, base_r;
  const int tid = threadIdx.x;
  if (tid == 0) {
    base = 0;
    base_r = 0;
    expert_offsets[0] = 0;
    if (blockscale_offsets) blockscale_offsets[0] = 0;
  }
  __syncthreads();
  for (int e0 = 0; e0 < num_experts; e0 += 256) {
    const int e = e0 + tid;
    const int c = e < num_experts ? ps1[3 * e] : 0;
    const int r = (c + 127) / 128 * 128;
    scan[tid] = c;
    scan_r[tid] = r;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
      const int v = tid >= d ? scan[tid - d] : 0, vr = tid >= d ? scan_r[tid - d] : 0;
      __syncthreads();
      scan[tid] += v;
      scan_r[tid] += vr;
      __syncthreads();
    }
    if (e < num_experts) {
      expert_offsets[e + 1] = base + scan[tid];
      if (blockscale_offsets) blockscale_offsets[e + 1] = base_r + scan_r[tid];
    }
    __syncthreads();
    if (tid == 255) {
      base += scan[255];
      base_r += scan_r[255];
    }
    __syncthreads();
  }
}

// Block (e, part) places expert e's slots of the part-th range of `span` slots (a multiple of
// 4096); it first counts the expert's slots in the ranges before its own, which is where its
// positions start.  Inside a sweep a slot's position follows from the matches before it:
// those of earlier waves, of earlier lanes of its wave (one ballot per slot of the four), and
// of the thread's own earlier slots.
__global__ __launch_bounds__(MOE_THREADS) void moe_place_kernel(const int* __restrict__ topk_ids,
                                                                const int* __restrict__ expert_offsets,
                                                                int* __restrict__ input_permutation,
                                                                int* __restrict__ output_permutation, int64_t topk_length,
                                                                int topk, int64_t span, int aligned) {
  __shared__ int red[MOE_THREADS / 64];
  __shared__ int wave_count[2][MOE_THREADS / 64];
  const int e = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t begin = (int64_t)blockIdx.y * span;
  if (begin >= topk_length) return;
  const int64_t end = begin + span < topk_length ? begin + span : topk_length;
  int next = expert_offsets[e] + block_count_ids(topk_ids, begin, e, aligned != 0, red);
  const uint64_t below = (1ull << lane) - 1ull;
  int buf = 0;
  v4i v = load_ids4(topk_ids, begin + 4 * (int64_t)threadIdx.x, end, aligned != 0);
  for (int64_t i0 = begin; i0 < end; i0 += MOE_SWEEP, buf ^= 1) {
    const int64_t i = i0 + 4 * (int64_t)threadIdx.x;
    const v4i cur = v;
    if (i0 + MOE_SWEEP < end) v = load_ids4(topk_ids, i + MOE_SWEEP, end, aligned != 0);  // the next sweep's, ahead of the barrier
    int before = 0, in_wave = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint64_t ballot = __ballot(cur[q] == e);
      before += __popcll(ballot & below);
      in_wave += __popcll(ballot);
    }
    if (lane == 0) wave_count[buf][wave] = in_wave;
    __syncthreads();  // (the buffer written two sweeps ago was last read before the previous sweep's barrier)
    int earlier_waves = 0, total = 0;
#pragma unroll
    for (int w = 0; w < MOE_THREADS / 64; ++w) {
      const int c = wave_count[buf][w];
      earlier_waves += w < wave ? c : 0;
      total += c;
    }
    int pos = next + earlier_waves + before;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (cur[q] == e) {
        input_permutation[pos] = (int)((i + q) / topk);
        output_permutation[i + q] = pos;
        ++pos;
      }
    }
    next += total;
  }
}

// ---------------------------------------------------------------------------
// shuffle_rows (prepare_moe_input.cu:168-244): output[d] = input[dst2src_map[d]], rows of
// row_bytes bytes.  16-byte pieces when rows and pointers allow, 4-byte or single bytes
// otherwise; a linear walk over (row, piece) pairs, so short rows (the 224-byte scale rows)
// use the lanes as well as long ones.
// ---------------------------------------------------------------------------
template <typename PIECE>
__global__ __launch_bounds__(256) void shuffle_rows_kernel(const char* __restrict__ in, const int* __restrict__ map,
                                                           char* __restrict__ out, int64_t num_src_rows,
                                                           int64_t num_dst_rows, int64_t row_bytes) {
  const int64_t ppr = row_bytes / (int64_t)sizeof(PIECE);  // pieces per row
  const int64_t total = num_dst_rows * ppr;
  for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
    const int64_t d = id / ppr, c = id - d * ppr;
    const int64_t s = map[d];
    if (s < 0 || s >= num_src_rows) continue;  // a map entry that names no row: the destination row is left alone
    reinterpret_cast<PIECE*>(out + d * row_bytes)[c] = reinterpret_cast<const PIECE*>(in + s * row_bytes)[c];
  }
}

// ---------------------------------------------------------------------------
// silu_and_mul (sgl-kernel/csrc/elementwise/activation.cu:57-60,85-103, the flashinfer
// act_and_mul kernel it instantiates): out[t, j] = T(silu(x[t, j])) * x[t, d + j] with the
// product rounded to T again; silu(v) = v / (1 + expf(-v)) in fp32.  16 bytes per lane.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                           int64_t tokens, int64_t d) {
  const int64_t cpr = d >> 3;  // 8-element chunks per output row
  const int64_t total = tokens * cpr;
  for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
    const int64_t t = id / cpr, c = id - t * cpr;
    const v4u xv = *reinterpret_cast<const v4u*>(in + t * 2 * d + c * 8);
    const v4u yv = *reinterpret_cast<const v4u*>(in + t * 2 * d + d + c * 8);
    v4u o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t w = 0;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        w |= (uint32_t)silu_mul_16<DT>((uint16_t)(xv[q] >> (16 * h)), (uint16_t)(yv[q] >> (16 * h))) << (16 * h);
      }
      o[q] = w;
    }
    *reinterpret_cast<v4u*>(out + t * d + c * 8) = o;
  }
}

// Rows whose halves are not 16-byte aligned (d not a multiple of 8): one element per lane.
template <int DT>
__global__ __launch_bounds__(256) void silu_and_mul_scalar_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                                  int64_t tokens, int64_t d) {
  const int64_t total = tokens * d;
  for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
    const int64_t t = id / d, c = id - t * d;
    out[id] = silu_mul_16<DT>(in[t * 2 * d + c], in[t * 2 * d + d + c]);
  }
}

// ---------------------------------------------------------------------------
// apply_shuffle_mul_sum (prepare_moe_input.cu:258-392): output[i, :] = sum over j < topk of
// factors[i * topk + j] * input[permutation[i * topk + j], :], accumulated in fp32 in j order
// with one fused multiply-add per term (:293-295), rounded once to the 16-bit type.
// A lane owns 8 consecutive elements of one output row; lanes walk (row, chunk) pairs linearly,
// so rows of any length fill the waves.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void shuffle_mul_sum_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                              const int* __restrict__ perm,
                                                              const uint16_t* __restrict__ factors, int64_t m, int topk,
                                                              int64_t row, int64_t num_src_rows) {
  const int64_t cpr = row >> 3;  // chunks per row
  const int64_t total = m * cpr;
  for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
    const int64_t i = id / cpr, c = id - i * cpr;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // Eight slots at a time: their table entries, then their rows, are loaded together so that one
    // memory round trip covers eight terms; the sum still runs in slot order.  A slot that names
    // no row (routed to nobody, or past topk) reads row 0 and enters as 0 * 0, which leaves the
    // sum as it is (the sum is never -0: it starts from +0).
    for (int j0 = 0; j0 < topk; j0 += 8) {
      int64_t src[8];
      float f[8];
      bool ok[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int64_t slot = i * topk + (j0 + u < topk ? j0 + u : topk - 1);
        src[u] = perm[slot];
        f[u] = factors ? to_f32_16<DT>(factors[slot]) : 1.0f;
      }
      v4u v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        ok[u] = j0 + u < topk && src[u] >= 0 && src[u] < num_src_rows;
        v[u] = *reinterpret_cast<const v4u*>(in + (ok[u] ? src[u] : 0) * row + c * 8);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float fu = ok[u] ? f[u] : 0.f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t w = ok[u] ? v[u][q] : 0u;
          acc[2 * q] = __builtin_fmaf(fu, to_f32_16<DT>((uint16_t)(w & 0xffffu)), acc[2 * q]);
          acc[2 * q + 1] = __builtin_fmaf(fu, to_f32_16<DT>((uint16_t)(w >> 16)), acc[2 * q + 1]);
        }
      }
    }
    v4u o;
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = (uint32_t)from_f32_16<DT>(acc[2 * q]) | ((uint32_t)from_f32_16<DT>(acc[2 * q + 1]) << 16);
    *reinterpret_cast<v4u*>(out + i * row + c * 8) = o;
  }
}

}  // namespace sglq

using namespace sglq;

extern "C" int sglq_prepare_moe_input(const int32_t* topk_ids, int32_t* expert_offsets, int32_t* blockscale_offsets,
                                      int32_t* problem_sizes1, int32_t* problem_sizes2, int32_t* input_permutation,
                                      int32_t* output_permutation, int64_t topk_length, int64_t topk, int64_t num_experts,
                                      int64_t n, int64_t k, void* stream) {
  const char* name = "prepare_moe_input";
  if (topk_length < 0 || topk <= 0 || num_experts < 0 || num_experts >= (1 << 20) || n < 0 || k < 0 ||
      n >= (1ll << 30) || k >= (1ll << 31) || topk_length >= (1ll << 31)) {
    set_error("%s: bad sizes", name);
    return SGLQ_EINVAL;
  }
  if (num_experts == 0) return SGLQ_OK;
  if (!expert_offsets || !problem_sizes1 || !problem_sizes2 || (topk_length > 0 && (!topk_ids || !input_permutation || !output_permutation))) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int aligned = (reinterpret_cast<uintptr_t>(topk_ids) & 15) == 0;
  moe_count_kernel<<<dim3((uint32_t)num_experts), dim3(MOE_THREADS), 0, st>>>(topk_ids, problem_sizes1, problem_sizes2, topk_length,
                                                                              (int)n, (int)k, aligned);
  moe_offsets_kernel<<<dim3(1), dim3(256), 0, st>>>(problem_sizes1, expert_offsets, blockscale_offsets, (int)num_experts);
  if (topk_length > 0) {
    // few experts: several blocks per expert, each with its own range of slots (about one block per CU in all)
    const int64_t sweeps = (topk_length + MOE_SWEEP - 1) / MOE_SWEEP;
    int64_t parts = 256 / num_experts;
    if (parts > sweeps) parts = sweeps;
    if (parts < 1) parts = 1;
    const int64_t span = (sweeps + parts - 1) / parts * MOE_SWEEP;
    moe_place_kernel<<<dim3((uint32_t)num_experts, (uint32_t)parts), dim3(MOE_THREADS), 0, st>>>(
        topk_ids, expert_offsets, input_permutation, output_permutation, topk_length, (int)topk, span, aligned);
  }
  return check_moe_launch(name);
}

extern "C" int sglq_shuffle_rows(const void* input, const int32_t* dst2src_map, void* output, int64_t num_src_rows,
                                 int64_t num_dst_rows, int64_t row_bytes, void* stream) {
  const char* name = "shuffle_rows";
  if (num_src_rows < 0 || num_dst_rows < 0 || row_bytes < 0) {
    set_error("%s: negative size", name);
    return SGLQ_EINVAL;
  }
  if (num_dst_rows == 0 || row_bytes == 0) return SGLQ_OK;
  if (!input || !dst2src_map || !output) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const char* in = static_cast<const char*>(input);
  char* out = static_cast<char*>(output);
  const uintptr_t align = reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(output) | (uintptr_t)row_bytes;
  const int piece = (align & 15) == 0 ? 16 : (align & 3) == 0 ? 4 : 1;
  const int64_t total = num_dst_rows * (row_bytes / piece);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  const dim3 grid((uint32_t)blocks), block(256);
  if (piece == 16) shuffle_rows_kernel<v4u><<<grid, block, 0, st>>>(in, dst2src_map, out, num_src_rows, num_dst_rows, row_bytes);
  else if (piece == 4) shuffle_rows_kernel<uint32_t><<<grid, block, 0, st>>>(in, dst2src_map, out, num_src_rows, num_dst_rows, row_bytes);
  else shuffle_rows_kernel<unsigned char><<<grid, block, 0, st>>>(in, dst2src_map, out, num_src_rows, num_dst_rows, row_bytes);
  return check_moe_launch(name);
}

extern "C" int sglq_silu_and_mul(const void* input, int dtype, void* output, int64_t num_tokens, int64_t d, void* stream) {
  const char* name = "silu_and_mul";
  if (num_tokens < 0 || d < 0) {
    set_error("%s: negative size", name);
    return SGLQ_EINVAL;
  }
  if (num_tokens == 0 || d == 0) return SGLQ_OK;
  if (!input || !output) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (dtype != SGLQ_BF16 && dtype != SGLQ_FP16) {
    set_error("%s: dtype must be Half or BFloat16", name);
    return SGLQ_EUNSUPPORTED;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool wide = d % 8 == 0 && !(reinterpret_cast<uintptr_t>(input) & 15) && !(reinterpret_cast<uintptr_t>(output) & 15);
  const int64_t total = wide ? num_tokens * (d / 8) : num_tokens * d;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  const dim3 grid((uint32_t)blocks), block(256);
  const uint16_t* in = static_cast<const uint16_t*>(input);
  uint16_t* out = static_cast<uint16_t*>(output);
  if (wide) {
    if (dtype == SGLQ_BF16) silu_and_mul_kernel<SGLQ_BF16><<<grid, block, 0, st>>>(in, out, num_tokens, d);
    else silu_and_mul_kernel<SGLQ_FP16><<<grid, block, 0, st>>>(in, out, num_tokens, d);
  } else {
    if (dtype == SGLQ_BF16) silu_and_mul_scalar_kernel<SGLQ_BF16><<<grid, block, 0, st>>>(in, out, num_tokens, d);
    else silu_and_mul_scalar_kernel<SGLQ_FP16><<<grid, block, 0, st>>>(in, out, num_tokens, d);
  }
  return check_moe_launch(name);
}

extern "C" int sglq_apply_shuffle_mul_sum(const void* input, void* output, const int32_t* permutation, const void* factors,
                                          int dtype, int64_t m, int64_t topk, int64_t row, int64_t num_src_rows,
                                          void* stream) {
  const char* name = "apply_shuffle_mul_sum";
  if (m < 0 || topk <= 0 || row < 0 || num_src_rows < 0 || topk >= (1 << 20) || m >= (1ll << 31)) {
    set_error("%s: bad sizes", name);
    return SGLQ_EINVAL;
  }
  if (m == 0 || row == 0) return SGLQ_OK;
  if (num_src_rows == 0) {
    set_error("%s: input has no rows", name);
    return SGLQ_EINVAL;
  }
  if (!input || !output || !permutation) {
    set_error("%s: null pointer", name);
    return SGLQ_EINVAL;
  }
  if (row % 8 != 0 || (reinterpret_cast<uintptr_t>(input) & 15) || (reinterpret_cast<uintptr_t>(output) & 15)) {
    set_error("%s: rows must be multiples of 8 elements and 16-byte aligned", name);
    return SGLQ_EINVAL;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  int64_t blocks = (m * (row / 8) + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  const dim3 grid((uint32_t)blocks), block(256);
  const uint16_t* in = static_cast<const uint16_t*>(input);
  uint16_t* out = static_cast<uint16_t*>(output);
  const uint16_t* f = static_cast<const uint16_t*>(factors);
  if (dtype == SGLQ_BF16) shuffle_mul_sum_kernel<SGLQ_BF16><<<grid, block, 0, st>>>(in, out, permutation, f, m, (int)topk, row, num_src_rows);
  else if (dtype == SGLQ_FP16) shuffle_mul_sum_kernel<SGLQ_FP16><<<grid, block, 0, st>>>(in, out, permutation, f, m, (int)topk, row, num_src_rows);
  else {
    set_error("%s: dtype must be Half or BFloat16", name);
    return SGLQ_EUNSUPPORTED;
  }
  return check_moe_launch(name);
}
