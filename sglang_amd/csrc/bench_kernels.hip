// Measurement kernels for gfx950 (built into libsglq_bench.so, not into the operator library):
//   * a register-only MFMA loop, the ceiling that the matrix pipe sustains on real operand
//     bytes at the clock the chip settles to under that load,
//   * a clock probe (shader-clock and constant-rate counters per compute unit), from which a harness
//     derives the average shader clock over a timed region,
//   * a plain copy and a read-only / write-only pass of known size, the yardsticks for the
//     FETCH_SIZE / WRITE_SIZE profiler counters and for the memory system's streaming rate,
//   * a global -> LDS copy loop without arithmetic: what the compute units take in through their LDS from the
//     L2s, the last-level cache or HBM with the GEMM kernels' copy instruction and tile shapes.
// C ABI, raw pointers, nothing allocated; every kernel runs a bounded loop.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

namespace {

// Variants of the MFMA loop.  One iteration is the K step of a 128 x 64 wave tile:
// 32 x v_mfma_f32_16x16x128_f8f6f4 or 16 x v_mfma_f32_32x32x64_f8f6f4 = 2 097 152 flop per wave.
constexpr int ACCUMULATE_16 = 0;  // 16x16x128, accumulating in place (per-row/per-column kinds)
constexpr int FOLD_16 = 1;        // 16x16x128 from a zero accumulator, result folded in with 4 FMAs (block-scaled kind)
constexpr int ACCUMULATE_32 = 2;  // 32x32x64, accumulating in place
constexpr int FOLD_32 = 3;        // 32x32x64 in pairs (one 128-byte K block), the pair's result folded in with 16 FMAs
constexpr int SCALED_16 = 4;      // 16x16x128 with an exponent byte per lane for each operand, accumulating in place (power-of-two block scales)

struct ClockSample {
  uint64_t shader_cycles, realtime_ticks;
};

__device__ __forceinline__ ClockSample read_clocks() {
  ClockSample s;
  s.shader_cycles = __builtin_readcyclecounter();      // s_memtime: counts at the shader clock
  s.realtime_ticks = __builtin_amdgcn_s_memrealtime(); // constant-rate reference counter
  return s;
}

template <int VARIANT>
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(const v8i* __restrict__ operands, int iters, float* __restrict__ sink,
                                                           uint64_t* __restrict__ clocks) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // six operand registers' worth of bytes per lane, distinct per wave (6 x 512 x 32 B = 96 KiB are read)
  v8i a[2], b[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) a[i] = operands[(i * 8 + wave) * 64 + lane];
#pragma unroll
  for (int j = 0; j < 4; ++j) b[j] = operands[((2 + j) * 8 + wave) * 64 + lane];
  const float scale = 1.0f + 1e-6f * (float)lane;

  ClockSample t0 = read_clocks();
  if constexpr (VARIANT == ACCUMULATE_16 || VARIANT == FOLD_16 || VARIANT == SCALED_16) {
    int sa[8], sb = 125 + (iters & 1);  // exponent bytes near 127 (2^0), per fragment as in the kernels
#pragma unroll
    for (int i = 0; i < 8; ++i) sa[i] = 124 + ((lane + i) & 7);
    v4f acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
      // the operands are opaque to the compiler in every iteration: nothing is hoisted
      asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
      v4f prev = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        asm volatile("" : "+v"(a[i & 1]));  // a new activation fragment as far as the compiler knows
        if constexpr (VARIANT == SCALED_16) asm volatile("" : "+v"(sa[i]), "+v"(sb));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (VARIANT == ACCUMULATE_16) {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[j], a[i & 1], acc[i][j], 0, 0, 0, 0, 0, 0);
          } else if constexpr (VARIANT == SCALED_16) {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[j], a[i & 1], acc[i][j], 0, 0, 0, sb, 0, sa[i]);
          } else {
            const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[j], a[i & 1], v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
            const int idx = i * 4 + j;
            if (idx > 0) {  // fold the previous result while this MFMA runs
              const int pi = (idx - 1) / 4, pj = (idx - 1) % 4;
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[pi][pj][e] = __builtin_fmaf(prev[e], scale, acc[pi][pj][e]);
            }
            prev = part;
          }
        }
      }
      if constexpr (VARIANT == FOLD_16) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[7][3][e] = __builtin_fmaf(prev[e], scale, acc[7][3][e]);
      }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) s += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    sink[blockIdx.x * 512 + threadIdx.x] = s;
  } else {
    v16f acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
      asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
      v16f prev;
#pragma unroll
      for (int e = 0; e < 16; ++e) prev[e] = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        asm volatile("" : "+v"(a[0]), "+v"(a[1]));
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if constexpr (VARIANT == ACCUMULATE_32) {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[j], a[i & 1], acc[i][j], 0, 0, 0, 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[2 + j], a[(i + 1) & 1], acc[i][j], 0, 0, 0, 0, 0, 0);
          } else {
            v16f zero;
#pragma unroll
            for (int e = 0; e < 16; ++e) zero[e] = 0.f;
            v16f part = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[j], a[i & 1], zero, 0, 0, 0, 0, 0, 0);
            part = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[2 + j], a[(i + 1) & 1], part, 0, 0, 0, 0, 0, 0);
            const int idx = i * 2 + j;
            if (idx > 0) {
              const int pi = (idx - 1) / 2, pj = (idx - 1) % 2;
#pragma unroll
              for (int e = 0; e < 16; ++e) acc[pi][pj][e] = __builtin_fmaf(prev[e], scale, acc[pi][pj][e]);
            }
            prev = part;
          }
        }
      }
      if constexpr (VARIANT == FOLD_32) {
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[3][1][e] = __builtin_fmaf(prev[e], scale, acc[3][1][e]);
      }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[i][j][e];
    sink[blockIdx.x * 512 + threadIdx.x] = s;
  }
  ClockSample t1 = read_clocks();
  if (threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = t1.shader_cycles - t0.shader_cycles;
    clocks[2 * blockIdx.x + 1] = t1.realtime_ticks - t0.realtime_ticks;
  }
}

// One sample of both counters per compute unit: slot = (XCC id, shader engine, shader array, CU) of the
// CU the block runs on (4096 slots).  The shader-cycle counters of different CUs are not aligned with each
// other, so only differences between two samples of the same slot mean anything.  Blocks on the same CU write
// nearly identical values; the last writer stays.
__global__ __launch_bounds__(64) void clock_probe_kernel(uint64_t* __restrict__ out) {
  if (threadIdx.x != 0) return;
  const ClockSample s = read_clocks();
  // HW_REG_XCC_ID (hardware register 20) bits 3:0; HW_REG_HW_ID (register 4): CU id bits 11:8, SH id bit 12, SE id bits 15:13
  const uint32_t xcc = __builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11)) & 15u;
  const uint32_t cu = __builtin_amdgcn_s_getreg(4 | (8 << 6) | ((8 - 1) << 11)) & 255u;
  const uint32_t slot = (xcc << 8) | cu;
  out[2 * slot] = s.shader_cycles;
  out[2 * slot + 1] = s.realtime_ticks;
}

// mode 0: dst = src; 1: read src only (one value per block written at the end); 2: write dst only
template <int MODE>
__global__ __launch_bounds__(256) void stream_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst, int64_t n16, int* __restrict__ sink) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  v4i keep = {0, 0, 0, 0};
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) {
    if constexpr (MODE == 0) dst[i] = src[i];
    if constexpr (MODE == 1) {
      const v4i v = src[i];
      keep[0] ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
    if constexpr (MODE == 2) dst[i] = v4i{(int)i, 1, 2, 3};
  }
  if constexpr (MODE == 1) {
    if (keep[0] == 0x5a5a5a5a) sink[blockIdx.x] = keep[0];  // practically never: keeps the loads alive
  }
}

// What a compute unit can take in through its LDS: the GEMM kernels' global -> LDS copies and nothing else.
// 8 waves per block, one block per CU; a "stage" is `rows` rows of 128 bytes (rows a multiple of 64: every wave
// issues rows / 64 one-KiB copies per stage, lane l bringing 16 bytes of row l / 8 as in the GEMM kernels), the rows
// `pitch` bytes apart.  Every wave keeps NSTAGE - 1 stages of its own copies in flight (copies retire in order:
// one vmcnt wait per stage) and nothing synchronises the waves.  Stage t of a block starts at byte
// (t % steps) * 128 of its window's rows: a block walks its window along the rows like a GEMM block walks K.
// Blocks b and b + 8, ..., b + 8 (share - 1) read the same window (the dispatcher deals blocks to the eight XCDs
// round-robin, so they share an L2); windows are `window_bytes` apart.
typedef unsigned int v4u_b __attribute__((ext_vector_type(4)));
template <int NSTAGE>
__global__ __launch_bounds__(512) void lds_fill_kernel(const char* __restrict__ src, int rows, uint32_t pitch, int steps, int64_t window_bytes,
                                                       int share, int iters, uint64_t* __restrict__ clocks, int* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(1024))) char fill_smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int cpw = rows / 64;  // copies per wave and stage
  const int stage_bytes = rows * 128;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int64_t window = (int64_t)((idx / share) * 8 + xcd);
  const char* base = src + window * window_bytes;
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  const uint32_t extent = (uint32_t)((rows - 1) * (int64_t)pitch + (int64_t)steps * 128);
  const v4u_b rsrc = {(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a), (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu)),
                      (uint32_t)__builtin_amdgcn_readfirstlane((int)extent), 0x00020000u};
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const char*)fill_smem);
  const uint32_t lane_off = (uint32_t)(wave * 8 + (lane >> 3)) * pitch + (uint32_t)(lane & 7) * 16u;
  auto issue = [&](int t) {
    const uint32_t st = lds0 + (uint32_t)(t % NSTAGE) * (uint32_t)stage_bytes;
    const uint32_t k0 = (uint32_t)(t % steps) * 128u;
    for (int j = 0; j < cpw; ++j) {
      const uint32_t dst = st + (uint32_t)(wave + 8 * j) * 1024u;
      const uint32_t voff = lane_off + (uint32_t)(64 * j) * pitch;
      asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" : : "s"(dst), "v"(voff), "s"(rsrc), "s"(k0) : "memory");
    }
  };
  const ClockSample t0 = read_clocks();
  for (int t = 0; t < NSTAGE - 1; ++t) issue(t);
  for (int t = 0; t < iters; ++t) {
    issue(t + NSTAGE - 1);
    // (stage t has landed: at most the NSTAGE - 1 younger stages' copies are outstanding; cpw is 1, 2, 3, 4 or 6)
    if (cpw == 1) asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSTAGE - 1) * 1) : "memory");
    else if (cpw == 2) asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSTAGE - 1) * 2) : "memory");
    else if (cpw == 3) asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSTAGE - 1) * 3) : "memory");
    else if (cpw == 4) asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSTAGE - 1) * 4) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSTAGE - 1) * 6) : "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
  const ClockSample t1 = read_clocks();
  __syncthreads();
  if (threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = t1.shader_cycles - t0.shader_cycles;
    clocks[2 * blockIdx.x + 1] = t1.realtime_ticks - t0.realtime_ticks;
    if (fill_smem[lane] == 0x5a && fill_smem[1024] == 0x5a) sink[blockIdx.x] = 1;  // keeps the stages observable
  }
}

}  // namespace

extern "C" {

// The LDS fill loop: `blocks` blocks of 512 lanes, `stages` (2, 3 or 4) stages of rows x 128 bytes in LDS (rows in
// {64, 128, 192, 256, 384}; stages * rows * 128 <= 160 KiB), `iters` stages per wave.  src must hold
// ceil(blocks / 8 / share) * 8 windows of window_bytes each, a window at least (rows - 1) * pitch + steps * 128 bytes.
// clocks: blocks x 2 uint64 (shader cycles, 100 MHz ticks of each block's loop).
int sglqb_lds_fill(int stages, const void* src, int rows, int64_t pitch, int steps, int64_t window_bytes, int share, int iters,
                   uint64_t* clocks, int* sink, int blocks, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!src || !clocks || !sink || blocks <= 0 || iters <= 0 || steps <= 0 || share <= 0) return -1;
  if (rows != 64 && rows != 128 && rows != 192 && rows != 256 && rows != 384) return -1;
  const int64_t lds = (int64_t)stages * rows * 128;
  if (lds > 160 * 1024 || pitch < 128 || pitch % 16 != 0 || (rows - 1) * pitch + (int64_t)steps * 128 > window_bytes ||
      (rows - 1) * pitch + (int64_t)steps * 128 >= (1ll << 31))
    return -1;
  const char* s = static_cast<const char*>(src);
  hipError_t e = hipSuccess;
  if (stages == 2) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(lds_fill_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess) lds_fill_kernel<2><<<blocks, 512, lds, st>>>(s, rows, (uint32_t)pitch, steps, window_bytes, share, iters, clocks, sink);
  } else if (stages == 3) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(lds_fill_kernel<3>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess) lds_fill_kernel<3><<<blocks, 512, lds, st>>>(s, rows, (uint32_t)pitch, steps, window_bytes, share, iters, clocks, sink);
  } else if (stages == 4) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(lds_fill_kernel<4>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess) lds_fill_kernel<4><<<blocks, 512, lds, st>>>(s, rows, (uint32_t)pitch, steps, window_bytes, share, iters, clocks, sink);
  } else {
    return -1;
  }
  if (e != hipSuccess) return (int)e;
  return (int)hipGetLastError();
}

// variant 0..3 (see above); operands: 96 KiB of e4m3 bytes (no NaN codes); sink: blocks * 512 floats;
// clocks: blocks * 2 uint64 (shader cycles, constant-rate ticks of each block).  8 waves per block,
// one block per CU when blocks = the CU count.  Returns the HIP error code of the launch.
int sglqb_mfma_ceiling(int variant, int iters, const void* operands, float* sink, uint64_t* clocks, int blocks, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  const v8i* ops = static_cast<const v8i*>(operands);
  if (blocks <= 0 || iters < 0 || !operands || !sink || !clocks) return -1;
  switch (variant) {
    case ACCUMULATE_16: mfma_ceiling_kernel<ACCUMULATE_16><<<blocks, 512, 0, st>>>(ops, iters, sink, clocks); break;
    case FOLD_16: mfma_ceiling_kernel<FOLD_16><<<blocks, 512, 0, st>>>(ops, iters, sink, clocks); break;
    case ACCUMULATE_32: mfma_ceiling_kernel<ACCUMULATE_32><<<blocks, 512, 0, st>>>(ops, iters, sink, clocks); break;
    case FOLD_32: mfma_ceiling_kernel<FOLD_32><<<blocks, 512, 0, st>>>(ops, iters, sink, clocks); break;
    case SCALED_16: mfma_ceiling_kernel<SCALED_16><<<blocks, 512, 0, st>>>(ops, iters, sink, clocks); break;
    default: return -1;
  }
  return (int)hipGetLastError();
}

// out: 4096 x 2 uint64 (per CU slot: shader cycles, constant-rate ticks), zero-filled by the caller.
int sglqb_clock_probe(uint64_t* out, int blocks, void* stream) {
  if (!out || blocks <= 0) return -1;
  clock_probe_kernel<<<blocks, 64, 0, static_cast<hipStream_t>(stream)>>>(out);
  return (int)hipGetLastError();
}

// mode 0 copy, 1 read only, 2 write only over `bytes` (a multiple of 16); sink: `blocks` ints.
int sglqb_stream(int mode, const void* src, void* dst, int64_t bytes, int* sink, int blocks, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (bytes < 0 || bytes % 16 != 0 || blocks <= 0) return -1;
  const v4i* s = static_cast<const v4i*>(src);
  v4i* d = static_cast<v4i*>(dst);
  if (mode == 0) stream_kernel<0><<<blocks, 256, 0, st>>>(s, d, bytes / 16, sink);
  else if (mode == 1) stream_kernel<1><<<blocks, 256, 0, st>>>(s, d, bytes / 16, sink);
  else if (mode == 2) stream_kernel<2><<<blocks, 256, 0, st>>>(s, d, bytes / 16, sink);
  else return -1;
  return (int)hipGetLastError();
}

}  // extern "C"
