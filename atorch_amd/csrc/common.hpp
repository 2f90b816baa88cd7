// Shared device helpers for the gfx950 FP8 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "../../include/atorch_amd_fp8.h"

namespace aamd {

constexpr int kTile = 128;       // quantisation tile / block edge
constexpr float kFp8Max = 448.f;  // largest finite e4m3fn magnitude

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short u16;

// ---- error plumbing -------------------------------------------------------
void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define AAMD_REQUIRE(cond, ...)      \
  do {                               \
    if (!(cond)) {                   \
      aamd::set_error(__VA_ARGS__);  \
      return AAMD_ERR_ARG;           \
    }                                \
  } while (0)

#define AAMD_LAUNCH_CHECK(what)                              \
  do {                                                       \
    hipError_t e__ = hipGetLastError();                      \
    if (e__ != hipSuccess) return aamd::hip_fail(e__, what); \
  } while (0)

// ---- scalar conversions ---------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 bits, round to nearest even: gfx950 has the conversion in hardware
// (v_cvt_pk_bf16_f32, two values per instruction).
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack_bf16x2(f, 0.f) & 0xffffu; }

// Input element loaders: 8 consecutive elements -> 8 floats.
struct BF16 {
  typedef u16 elem;
};
// bf16 rows [a | b] of a gated linear unit: the element read at column c is
// h = bf16(bf16(silu(a[c])) * b[c]) with b = a + gate_off (grouped_gemm_moe.py:331-334).
struct GLU {
  typedef u16 elem;
};
// bf16 values x read as h = bf16(gelu(x)), gelu(x) = x/2 (1 + erf(x / sqrt 2)) in fp32: the default
// activation of the expert MLP (grouped_gemm_moe.py:449, torch.nn.functional.gelu).
struct GELU {
  typedef u16 elem;
};
// Its backward: values x plus the gradient dh of h (at a fixed element offset from x: both are dense
// [M, F] tensors); the element read is bf16(dh (cdf(x) + x pdf(x))), autograd's gelu_backward.
struct GELUB {
  typedef u16 elem;
};
struct F32 {
  typedef float elem;
};
struct F16 {
  typedef u16 elem;
};
// Inputs whose values are bf16 numbers: quotients by the scale of a bf16 maximum may take the
// checked two-instruction division (see Divider); fp32 and fp16 inputs take the plain one.
template <typename IN>
constexpr bool kBf16Values = !std::is_same<IN, F32>::value && !std::is_same<IN, F16>::value;

__device__ __forceinline__ void unpack8(const v4i& raw, float* v) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    uint32_t w = (uint32_t)raw[i];
    v[2 * i] = __uint_as_float(w << 16);
    v[2 * i + 1] = __uint_as_float(w & 0xffff0000u);
  }
}

// ---- 16-lane (one DPP row) max reduction: every lane of the row gets the max
// Maximum over the 16 lanes of a DPP row of values that are not negative: such floats order like their bit
// patterns, and the integer maximum takes its second operand straight from the neighbouring lane (the float
// one would first canonicalise it).  A NaN orders above every number and is kept.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
  const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
  return o > v ? o : v;
}
__device__ __forceinline__ float row16_max(float v) {
  uint32_t u = __float_as_uint(v);
  u = dpp_max_u32<0xB1>(u);   // quad_perm [1,0,3,2]
  u = dpp_max_u32<0x4E>(u);   // quad_perm [2,3,0,1]
  u = dpp_max_u32<0x141>(u);  // row_half_mirror
  u = dpp_max_u32<0x140>(u);  // row_mirror
  return __uint_as_float(u);
}

// Two floats -> two e4m3fn codes in the low or high half of `old` (RNE, v_cvt_pk_fp8_f32).
// No clamp ahead of the encoder: a quotient x / s with s = RN(max(amax, eps) / 448) and
// |x| <= amax is at most 448 (1 + 2^-23), which RNE maps to 448 (the encoder's own overflow
// handling starts above 464).
template <bool HI>
__device__ __forceinline__ int pack2_fp8(float a, float b, int old) {
  return __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, HI);
}

// The scale of a tile, s = max(amax, eps) / 448 with 0 -> 1, and what divides the tile's values by it.
// Scale and quotients are part of the bit-exact contract: they are the correctly rounded (IEEE) ones.
//
// `plain` takes the hardware's division sequences, a dozen instructions per quotient.  Without it (amax and
// the values are bf16 numbers, eps is zero):
//   scale: the tail of the division sequence with the constant's reciprocal, y = RN(1 / 448): q = a y,
//     r = a - 448 q (exact in an FMA), s = q + r y (Markstein); checked against a / 448 for every bf16 a.
//   quotients, two instructions per value: the reciprocal of s is held as an unevaluated sum yh + yl.  yh
//     lies two units in the last place below the hardware reciprocal, so below 1 / s, and with
//     e = 1 - s yh > 0 (one FMA), yl = yh (e + e^2) >= +0 makes yh + yl = 1 / s to about 2^-60.  Then
//     fma(x, yh, x yl) rounds x (yh + yl) once (the small product carries a relative error of 2^-24 on a
//     term 2^-21 of the sum), and both products of a zero x have its sign, so a negative zero stays one.
//     That is no proof of a correctly rounded quotient: the scheme is used where every case has been
//     enumerated and gives the code of the plain division: all pairs of a bf16 value and a bf16 maximum,
//     about 10^9.
// Maxima outside 2^-90 .. 2^100 (zero among them) take the plain path, where a residual or a reciprocal
// could leave the normal range.
struct Divider {
  float s, yh, yl;
  bool plain;
};
__device__ __forceinline__ Divider make_scale(float amax, float eps, bool plain) {
  const float a = fmaxf(amax, eps);
  Divider d;
  // 2^-90 <= a < 2^100 as one unsigned comparison of the bit patterns (a is not negative; zero, NaN and
  // infinity fall outside)
  d.plain = plain || __float_as_uint(a) - 0x12800000u >= 0x71800000u - 0x12800000u;
  if (__builtin_expect(d.plain, 0)) {
    const float s = a / kFp8Max;
    d.s = s == 0.f ? 1.f : s;
    d.yh = d.yl = 0.f;
  } else {
    constexpr float y = 1.0f / kFp8Max;
    const float q = a * y;
    const float r = __builtin_fmaf(-kFp8Max, q, a);
    d.s = __builtin_fmaf(r, y, q);  // not zero: a >= 2^-90
    d.yh = __uint_as_float(__float_as_uint(__builtin_amdgcn_rcpf(d.s)) - 2u);
    const float e = __builtin_fmaf(-d.s, d.yh, 1.0f);
    d.yl = __builtin_fmaf(e, e, e) * d.yh;
  }
  return d;
}
__device__ __forceinline__ v2i pack8_fp8(const float* t) {
  v2i o;
  int w = pack2_fp8<false>(t[0], t[1], 0);
  o[0] = pack2_fp8<true>(t[2], t[3], w);
  w = pack2_fp8<false>(t[4], t[5], 0);
  o[1] = pack2_fp8<true>(t[6], t[7], w);
  return o;
}
// the plain path, out of line: a hundred instructions that the kernels of bf16 inputs almost never run
__device__ __attribute__((noinline)) v2i quant8_plain(float v0, float v1, float v2, float v3, float v4, float v5, float v6,
                                                      float v7, float s) {
  const float t[8] = {v0 / s, v1 / s, v2 / s, v3 / s, v4 / s, v5 / s, v6 / s, v7 / s};
  return pack8_fp8(t);
}
// 8 values / one scale -> 8 codes in two dwords.  CALL_PLAIN: the plain path is a function call (values that live
// across a call sit in the callee-saved half of the register file, which costs a kernel with many live values
// its occupancy: such kernels keep the path in line)
template <bool CALL_PLAIN = true>
__device__ __forceinline__ v2i quant8(const float* v, const Divider& d) {
  if (__builtin_expect(d.plain, 0)) {
    if constexpr (CALL_PLAIN) {
      return quant8_plain(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], d.s);
    } else {
      const float t[8] = {v[0] / d.s, v[1] / d.s, v[2] / d.s, v[3] / d.s, v[4] / d.s, v[5] / d.s, v[6] / d.s, v[7] / d.s};
      return pack8_fp8(t);
    }
  }
  float t[8];
#pragma unroll
  for (int i = 0; i < 8; i++) t[i] = __builtin_fmaf(v[i], d.yh, v[i] * d.yl);
  return pack8_fp8(t);
}

__device__ __forceinline__ float amax8(const float* v) {
  float m = fmaxf(fabsf(v[0]), fabsf(v[1]));
#pragma unroll
  for (int i = 2; i < 8; i++) m = fmaxf(m, fabsf(v[i]));
  return m;
}

// Which group does padded tile `t` belong to?  tile_off[E+1] is an exclusive prefix of
// per-group tile counts.  All threads of the block take part; returns the same g in every
// thread (E+1 if t is beyond the last tile).  `slot` is one int of shared memory.
__device__ __forceinline__ int find_group(const int32_t* __restrict__ tile_off, int E, int t, int* slot) {
  if (threadIdx.x == 0) *slot = E + 1;
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int lo = tile_off[e], hi = tile_off[e + 1];
    if (t >= lo && t < hi) *slot = e;
  }
  __syncthreads();
  return *slot;
}

}  // namespace aamd
