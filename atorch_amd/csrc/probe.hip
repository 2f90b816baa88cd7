// Measurement aids of the library (no counterpart in the reference): the shader clock under load and
// what the fp8 matrix pipes deliver from registers alone, with and without the block-scale fold.
#include "common.hpp"

namespace aamd {

typedef float v16f __attribute__((ext_vector_type(16)));

// One wavefront: spins until the shader cycle counter has advanced by min_cycles (the iteration
// bound ends the loop even if the counter stood still).
__global__ void clock_probe_kernel(unsigned long long* out, long long min_cycles) {
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  unsigned long long c1 = c0;
  for (long long it = 0; it < min_cycles && (long long)(c1 - c0) < min_cycles; it++) {
    __builtin_amdgcn_s_sleep(8);
    c1 = __builtin_readcyclecounter();
  }
  const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0) {
    out[0] = c1 - c0;
    out[1] = r1 - r0;
  }
}

// The GEMM's inner loop without any memory traffic: eight waves per workgroup (two per SIMD), each
// with the fragments of a 128 x 64 wave tile in registers, issue per iteration the sixteen
// v_mfma_f32_32x32x64_f8f6f4 of one 128-deep step.  FOLD: every pair's raw product is folded into the
// accumulator with sixteen FMAs (the block-scale step); otherwise the MFMAs accumulate directly.
template <bool FOLD>
__global__ __launch_bounds__(512, 1) void mfma_probe_kernel(const int* __restrict__ src, float* __restrict__ out,
                                                             int iters, unsigned long long* cyc) {
  const int tid = threadIdx.x;
  v8i lf[2][2], rf[4][2];
  const v8i* s8 = reinterpret_cast<const v8i*>(src) + (size_t)(blockIdx.x % 64) * 512 * 12 + tid;
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int h = 0; h < 2; h++) lf[j][h] = s8[(j * 2 + h) * 512];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int h = 0; h < 2; h++) rf[i][h] = s8[(4 + i * 2 + h) * 512];
  v16f acc[4][2], zero;
#pragma unroll
  for (int r = 0; r < 16; r++) zero[r] = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) acc[i][j] = zero;
  const float sc = 1.0f + 1e-7f * (float)(tid & 3);
  const unsigned long long t0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        if constexpr (FOLD) {
          v16f pr = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(rf[i][0], lf[j][0], zero, 0, 0, 0, 0, 0, 0);
          pr = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(rf[i][1], lf[j][1], pr, 0, 0, 0, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] = __builtin_fmaf(pr[r], sc, acc[i][j][r]);
        } else {
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(rf[i][0], lf[j][0], acc[i][j], 0, 0, 0, 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(rf[i][1], lf[j][1], acc[i][j], 0, 0, 0, 0, 0, 0);
        }
        asm volatile("" : "+v"(acc[i][j]));
      }
  }
  const unsigned long long t1 = __builtin_readcyclecounter();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) s += acc[i][j][r];
  out[(size_t)blockIdx.x * 512 + tid] = s;
  if (tid == 64 && blockIdx.x == 0) cyc[0] = t1 - t0;  // a wave that shares its SIMD's pipe for the whole run
}

// Streaming probe: what this GPU's memory system delivers for a given mix of read and write streams with
// nothing else in the way.  Every lane handles 16-byte words: per unit of work it reads one word from
// each of R input streams and writes one word to each of W output streams (streams are disjoint
// `stride_words`-long arrays laid out one after the other), all accesses streaming (nontemporal),
// two units in flight per lane.
template <int R, int W>
__global__ __launch_bounds__(256) void stream_probe_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst,
                                                          int64_t stride_words, int64_t units) {
  const int64_t step = (int64_t)gridDim.x * 256;
  int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (; u + step < units; u += 2 * step) {
    v4i a = {0, 0, 0, 0}, b = {0, 0, 0, 0};
    v4i ra[R > 0 ? R : 1], rb[R > 0 ? R : 1];
#pragma unroll
    for (int r = 0; r < R; r++) {
      ra[r] = __builtin_nontemporal_load(src + r * stride_words + u);
      rb[r] = __builtin_nontemporal_load(src + r * stride_words + u + step);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
      a ^= ra[r];
      b ^= rb[r];
    }
    if constexpr (W > 0) {
#pragma unroll
      for (int w = 0; w < W; w++) {
        __builtin_nontemporal_store(a + w, dst + w * stride_words + u);
        __builtin_nontemporal_store(b + w, dst + w * stride_words + u + step);
      }
    } else {
      if ((a[0] ^ b[0]) == 0x7fffffff && (a[1] ^ b[1]) == 0x12345678) dst[0] = a;  // keeps the loads alive
    }
  }
  for (; u < units; u += step) {
    v4i a = {0, 0, 0, 0};
#pragma unroll
    for (int r = 0; r < R; r++) a ^= __builtin_nontemporal_load(src + r * stride_words + u);
    if constexpr (W > 0) {
#pragma unroll
      for (int w = 0; w < W; w++) __builtin_nontemporal_store(a + w, dst + w * stride_words + u);
    } else {
      if (a[0] == 0x7fffffff && a[1] == 0x12345678) dst[0] = a;
    }
  }
}

template <int R, int W>
static int launch_stream_probe(const void* src, void* dst, int64_t stride_words, int64_t units, hipStream_t st) {
  int64_t blocks = (units + 511) / 512;
  if (blocks > (1 << 20)) blocks = 1 << 20;
  stream_probe_kernel<R, W><<<(unsigned)blocks, 256, 0, st>>>((const v4i*)src, (v4i*)dst, stride_words, units);
  AAMD_LAUNCH_CHECK("stream_probe");
  return AAMD_OK;
}

}  // namespace aamd

extern "C" int aamd_stream_probe(const void* src, void* dst, int reads, int writes, int64_t stride_bytes,
                                 int64_t units, void* stream) {
  using namespace aamd;
  AAMD_REQUIRE(src && dst, "stream_probe: null pointer");
  AAMD_REQUIRE(stride_bytes > 0 && stride_bytes % 16 == 0 && units > 0 && units * 16 <= stride_bytes,
               "stream_probe: every stream holds `units` 16-byte words inside its stride");
  AAMD_REQUIRE(((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0, "stream_probe: alignment");
  hipStream_t st = (hipStream_t)stream;
  const int64_t sw = stride_bytes / 16;
#define AAMD_SP(R, W) \
  if (reads == R && writes == W) return launch_stream_probe<R, W>(src, dst, sw, units, st);
  AAMD_SP(1, 0) AAMD_SP(0, 1) AAMD_SP(1, 1) AAMD_SP(2, 1) AAMD_SP(1, 2) AAMD_SP(1, 4) AAMD_SP(4, 1) AAMD_SP(8, 1)
  AAMD_SP(3, 2) AAMD_SP(2, 2)
#undef AAMD_SP
  AAMD_REQUIRE(false, "stream_probe: mix %d:%d is not built (1:0 0:1 1:1 2:1 1:2 1:4 4:1 8:1 3:2 2:2 are)", reads, writes);
  return AAMD_OK;
}

extern "C" int aamd_clock_probe(uint64_t* out, int64_t min_cycles, void* stream) {
  AAMD_REQUIRE(out != nullptr, "clock_probe: null pointer");
  AAMD_REQUIRE(min_cycles >= 0 && min_cycles <= (1LL << 31), "clock_probe: min_cycles out of range");
  aamd::clock_probe_kernel<<<1, 64, 0, (hipStream_t)stream>>>(reinterpret_cast<unsigned long long*>(out), min_cycles);
  AAMD_LAUNCH_CHECK("clock_probe");
  return AAMD_OK;
}

extern "C" int aamd_mfma_probe(const void* operands, int fold, int iters, int workgroups, float* out, uint64_t* cycles,
                               void* stream) {
  AAMD_REQUIRE(operands && out && cycles, "mfma_probe: null pointer");
  AAMD_REQUIRE(iters >= 1 && iters <= (1 << 20) && workgroups >= 1 && workgroups <= (1 << 16), "mfma_probe: bad sizes");
  AAMD_REQUIRE((reinterpret_cast<uintptr_t>(operands) & 31) == 0, "mfma_probe: operands must be 32-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (fold)
    aamd::mfma_probe_kernel<true><<<workgroups, 512, 0, st>>>((const int*)operands, out, iters, (unsigned long long*)cycles);
  else
    aamd::mfma_probe_kernel<false><<<workgroups, 512, 0, st>>>((const int*)operands, out, iters, (unsigned long long*)cycles);
  AAMD_LAUNCH_CHECK("mfma_probe");
  return AAMD_OK;
}
