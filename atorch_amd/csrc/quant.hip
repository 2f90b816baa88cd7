// Memory-bound quantisation kernels for gfx950: 1x128 tile quant (optionally with the token
// permute fused in as a scatter), row-wise + transposed quant of ragged groups in one pass,
// 128x128 block quant with the transposed copy, and dequant.
//
// All of them stream HBM with 128-bit accesses; amax reductions over a 128-element tile run
// inside one 16-lane DPP row.  Scales and codes are part of a bit-exact contract, so every
// quotient gives the code of the correctly rounded one (the IEEE division or its checked two-instruction form).
#include "common.hpp"

namespace aamd {

// ---------------------------------------------------------------------------------------
// tile loaders: 8 consecutive elements per lane
// ---------------------------------------------------------------------------------------
// 16 bytes at a byte offset from a base pointer.  With a base that is the same in every lane the
// address is a scalar register pair plus a 32-bit lane offset: no 64-bit arithmetic per access.
template <typename T>
__device__ __forceinline__ v4i ld16(const T* base, uint32_t boff) {
  return *reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(base) + boff);
}
template <typename T>
__device__ __forceinline__ v4i ld16_nt(const T* base, uint32_t boff) {
  return __builtin_nontemporal_load(reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(base) + boff));
}
template <typename V, typename T>
__device__ __forceinline__ void st_nt(T* base, uint32_t boff, V val) {
  __builtin_nontemporal_store(val, reinterpret_cast<V*>(reinterpret_cast<char*>(base) + boff));
}

template <typename IN>
struct Raw8;
template <>
struct Raw8<BF16> {
  v4i a;
  __device__ __forceinline__ void load(const u16* p, uint32_t boff, int64_t) { a = ld16_nt(p, boff); }
  __device__ __forceinline__ void zero() { a = v4i{0, 0, 0, 0}; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(a)); }
  __device__ __forceinline__ void get(float* v) const { unpack8(a, v); }
};
template <>
struct Raw8<F32> {
  v4i a, b;
  __device__ __forceinline__ void load(const float* p, uint32_t boff, int64_t) {
    a = ld16_nt(p, boff);
    b = ld16_nt(p + 4, boff);
  }
  __device__ __forceinline__ void zero() { a = b = v4i{0, 0, 0, 0}; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(a), "+v"(b)); }
  __device__ __forceinline__ void get(float* v) const {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[i] = __int_as_float(a[i]);
      v[4 + i] = __int_as_float(b[i]);
    }
  }
};

template <>
struct Raw8<F16> {
  v4i a;
  __device__ __forceinline__ void load(const u16* p, uint32_t boff, int64_t) { a = ld16_nt(p, boff); }
  __device__ __forceinline__ void zero() { a = v4i{0, 0, 0, 0}; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(a)); }
  __device__ __forceinline__ void get(float* v) const {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t w = (uint32_t)a[i];
      v[2 * i] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w & 0xffffu));
      v[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w >> 16));
    }
  }
};

// sigmoid on the hardware transcendental units, one v_exp_f32 and one v_rcp_f32 per value.  Both
// flush results below the normal range, and 1 / (1 + e^-x) gets there for x below about -87 while
// x times it is still a normal number, so the reciprocal is taken of the sum scaled by 2^-16
// (x r' stays finite for |x| < 2^112):
//   e = e^-x (inf where it overflows, 0 where it leaves the normal range), r' = 1 / (2^-16 + 2^-16 e)
//   = 2^16 sigmoid(x).
// silu(x) = (x r') 2^-16, sigmoid(x) = r' 2^-16.  A few fp32 ulps of error (more for |x| in the tens,
// where x log2(e) itself is rounded), far below the bf16 rounding that follows; e^-x = inf gives
// r' = 0 and silu = -0 as in fp32 arithmetic.
__device__ __forceinline__ float sigmoid_scaled(float x) {
  const float e = __builtin_amdgcn_exp2f(x * -1.4426950408889634f);
  return __builtin_amdgcn_rcpf(__builtin_fmaf(e, 0x1p-16f, 0x1p-16f));
}
__device__ __forceinline__ float silu_from(float x, float r_scaled) { return (x * r_scaled) * 0x1p-16f; }

// SwiGLU on load: a and b halves of a row, h = silu(a) * b with both roundings to bf16 that the
// reference's two torch ops make (F.silu on a bf16 tensor, then the product; fp32 inside).
template <>
struct Raw8<GLU> {
  v4i a, b;
  __device__ __forceinline__ void load(const u16* p, uint32_t boff, int64_t gate_off) {
    a = ld16_nt(p, boff);
    b = ld16_nt(p + gate_off, boff);
  }
  __device__ __forceinline__ void zero() { a = b = v4i{0, 0, 0, 0}; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(a), "+v"(b)); }
  __device__ __forceinline__ void get(float* v) const {
    float fa[8], fb[8];
    unpack8(a, fa);
    unpack8(b, fb);
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      const float s0 = silu_from(fa[i], sigmoid_scaled(fa[i]));
      const float s1 = silu_from(fa[i + 1], sigmoid_scaled(fa[i + 1]));
      const uint32_t sl = pack_bf16x2(s0, s1);
      const uint32_t h = pack_bf16x2(__uint_as_float(sl << 16) * fb[i], __uint_as_float(sl & 0xffff0000u) * fb[i + 1]);
      v[i] = __uint_as_float(h << 16);
      v[i + 1] = __uint_as_float(h & 0xffff0000u);
    }
  }
};

// GELU on load, h = bf16(x Phi(x)), and its backward dh (Phi(x) + x pdf(x)), pdf = exp(-x^2 / 2) / sqrt(2 pi).
// The reference evaluates Phi as (1 + erf(x / sqrt 2)) / 2 in fp32 (torch.nn.functional.gelu on a bf16 tensor).
// Here Phi comes from the complementary function, without branches and without the cancellation of 1 + erf
// for negative x:
//   erfc(t) / 2 = exp(-t^2) q(u),  u = 1 / (1 + t / 2),  t = |x| / sqrt 2,
// q a polynomial of degree 7 (a least-squares fit of erfcx(t) / 2 at Chebyshev nodes of u over 0 <= t <= 4.3,
// relative error 6e-8; beyond 4.3, where erfc / 2 is below 1e-9, q stays at its value there), Phi(x) = erfc(t) / 2
// for x < 0 and 1 - erfc(t) / 2 otherwise.  With s = |x| sqrt(log2(e) / 2) the exponential is exp2(-s^2) and
// t / 2 = 0.41628 s: one v_rcp_f32, one v_exp_f32 and a dozen multiply-adds against the three divergent ranges of
// the library's erff.  In fp32 arithmetic x Phi(x) comes out within 2.3e-6 of its value for |x| <= 6: rounded to
// bf16 it equals the correctly rounded product for every normal bf16 x >= -4, and below that it keeps digits
// where 1 + erf(x / sqrt 2) has lost them.  Infinities and NaNs give what the reference's formula gives.
__device__ __forceinline__ float gelu_phi(float x, float* exp_neg_half_sq = nullptr) {
  const float s = fabsf(x) * 0.8493217825889587f;  // sqrt(log2(e) / 2) |x|
  const float u = __builtin_amdgcn_rcpf(__builtin_fmaf(fminf(s, 5.164826393127441f), 0.41627731919288635f, 1.0f));
  float q = 0.042140234261751175f;
  q = __builtin_fmaf(q, u, -0.16624070703983307f);
  q = __builtin_fmaf(q, u, 0.1660318523645401f);
  q = __builtin_fmaf(q, u, 0.05331931263208389f);
  q = __builtin_fmaf(q, u, 0.11762023717164993f);
  q = __builtin_fmaf(q, u, 0.14757198095321655f);
  q = __builtin_fmaf(q, u, 0.13941511511802673f);
  q = __builtin_fmaf(q, u, 0.00014206925698090345f);
  const float e = __builtin_amdgcn_exp2f(-(s * s));  // exp(-x^2 / 2) = exp(-t^2)
  if (exp_neg_half_sq) *exp_neg_half_sq = e;
  const float h = q * e;  // erfc(t) / 2
  return x < 0.f ? h : 1.0f - h;
}
// Both GELU forms are functions of one bf16 value, x Phi(x) rounded to bf16 and Phi(x) + x pdf(x) in fp32, and cost
// two dozen vector instructions per value, which is what bounds the fused kernels.  The dual kernels therefore read
// them from tables in LDS indexed by the bits of x, for |x| in [2^-14, 2^3) (17 binades x 128 x 2 signs); values
// outside (exact zeros, outliers) take the arithmetic.  The tables are filled by the same functions, by a small
// kernel ahead of every launch, into arrays of the library on the device: every call writes the same values, so
// calls that overlap do not disturb each other.
constexpr uint32_t kLutLo = (uint32_t)(127 - 14) << 7;        // first magnitude (bits without the sign) of the tables
constexpr uint32_t kLutN = (uint32_t)(14 + 3) << 7;           // magnitudes per sign
static __device__ __attribute__((aligned(16))) u16 g_gelu_lut[2 * kLutN];
static __device__ __attribute__((aligned(16))) float g_gelub_lut[2 * kLutN];
__device__ __forceinline__ float gelu_grad_factor(float x) {
  float e;  // exp(-x^2 / 2)
  const float cdf = gelu_phi(x, &e);
  const float pdf = 0.39894228040143267794f * e;
  return cdf + x * pdf;
}
__global__ __launch_bounds__(256) void gelu_lut_kernel() {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= 2 * kLutN) return;
  const uint32_t sign = i >= kLutN ? 1u : 0u;
  const float x = __uint_as_float(((sign << 15) | (kLutLo + i - sign * kLutN)) << 16);
  g_gelu_lut[i] = (u16)f32_to_bf16_bits(x * gelu_phi(x));
  g_gelub_lut[i] = gelu_grad_factor(x);
}
// a pair of values outside the tables: out of line, these are rare
__device__ __attribute__((noinline)) uint32_t gelu_pair_plain(uint32_t w) {
  const float x0 = __uint_as_float(w << 16), x1 = __uint_as_float(w & 0xffff0000u);
  return pack_bf16x2(x0 * gelu_phi(x0), x1 * gelu_phi(x1));
}
__device__ __attribute__((noinline)) uint32_t gelu_grad_pair_plain(uint32_t w, uint32_t gw) {
  const float x0 = __uint_as_float(w << 16), x1 = __uint_as_float(w & 0xffff0000u);
  const float g0 = __uint_as_float(gw << 16), g1 = __uint_as_float(gw & 0xffff0000u);
  return pack_bf16x2(g0 * gelu_grad_factor(x0), g1 * gelu_grad_factor(x1));
}
// Table position of the bf16 value whose magnitude bits are `mag` and whose sign is `sign` (0 / 1); `ok` is cleared
// when the value lies outside the tables (position 0 is returned then, so the read that follows stays inside).
__device__ __forceinline__ uint32_t lut_index(uint32_t mag, uint32_t sign, bool& ok) {
  const uint32_t m = mag - kLutLo;
  const bool in = m < kLutN;
  ok = ok && in;
  return in ? m + sign * kLutN : 0u;
}
template <typename IN>
constexpr uint32_t kLutBytes = 0;
template <>
constexpr uint32_t kLutBytes<GELU> = 2 * kLutN * sizeof(u16);
template <>
constexpr uint32_t kLutBytes<GELUB> = 2 * kLutN * sizeof(float);

template <>
struct Raw8<GELU> {
  v4i a;
  __device__ __forceinline__ void load(const u16* p, uint32_t boff, int64_t) { a = ld16_nt(p, boff); }
  __device__ __forceinline__ void zero() { a = v4i{0, 0, 0, 0}; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(a)); }
  __device__ __forceinline__ void get(float* v) const {
    float x[8];
    unpack8(a, x);
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      const float g0 = x[i] * gelu_phi(x[i]);
      const float g1 = x[i + 1] * gelu_phi(x[i + 1]);
      const uint32_t h = pack_bf16x2(g0, g1);
      v[i] = __uint_as_float(h << 16);
      v[i + 1] = __uint_as_float(h & 0xffff0000u);
    }
  }
  // the same values from the table (a copy of g_gelu_lut in LDS): all eight reads are issued together, and a
  // value outside the table, which is rare, sends its pair through the arithmetic afterwards
  __device__ __forceinline__ void get(float* v, const void* lut) const {
    const u16* const T = static_cast<const u16*>(lut);
    uint32_t t[8], h[4];
    bool ok = true;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t w = (uint32_t)a[i];
      t[2 * i] = lut_index(w & 0x7fffu, (w >> 15) & 1u, ok);
      t[2 * i + 1] = lut_index((w >> 16) & 0x7fffu, w >> 31, ok);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) h[i] = (uint32_t)T[t[2 * i]] | ((uint32_t)T[t[2 * i + 1]] << 16);
    if (__builtin_expect(!ok, 0)) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t w = (uint32_t)a[i];
        if ((w & 0x7fffu) - kLutLo >= kLutN || ((w >> 16) & 0x7fffu) - kLutLo >= kLutN) h[i] = gelu_pair_plain(w);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[2 * i] = __uint_as_float(h[i] << 16);
      v[2 * i + 1] = __uint_as_float(h[i] & 0xffff0000u);
    }
  }
};
template <>
struct Raw8<GELUB> {
  v4i a, d;
  __device__ __forceinline__ void load(const u16* p, uint32_t boff, int64_t dh_off) {
    a = ld16_nt(p, boff);
    d = ld16_nt(p + dh_off, boff);
  }
  __device__ __forceinline__ void zero() { a = d = v4i{0, 0, 0, 0}; }
  __device__ __forceinline__ void pin() { asm volatile("" : "+v"(a), "+v"(d)); }
  __device__ __forceinline__ void get(float* v) const {
    float x[8], g[8];
    unpack8(a, x);
    unpack8(d, g);
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      const uint32_t h = pack_bf16x2(g[i] * gelu_grad_factor(x[i]), g[i + 1] * gelu_grad_factor(x[i + 1]));
      v[i] = __uint_as_float(h << 16);
      v[i + 1] = __uint_as_float(h & 0xffff0000u);
    }
  }
  // the same values with the factor from the table (a copy of g_gelub_lut in LDS), read like the forward's
  __device__ __forceinline__ void get(float* v, const void* lut) const {
    const float* const T = static_cast<const float*>(lut);
    uint32_t t[8], h[4];
    float f[8];
    bool ok = true;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t w = (uint32_t)a[i];
      t[2 * i] = lut_index(w & 0x7fffu, (w >> 15) & 1u, ok);
      t[2 * i + 1] = lut_index((w >> 16) & 0x7fffu, w >> 31, ok);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = T[t[i]];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t gw = (uint32_t)d[i];
      h[i] = pack_bf16x2(__uint_as_float(gw << 16) * f[2 * i], __uint_as_float(gw & 0xffff0000u) * f[2 * i + 1]);
    }
    if (__builtin_expect(!ok, 0)) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t w = (uint32_t)a[i];
        if ((w & 0x7fffu) - kLutLo >= kLutN || ((w >> 16) & 0x7fffu) - kLutLo >= kLutN)
          h[i] = gelu_grad_pair_plain(w, (uint32_t)d[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[2 * i] = __uint_as_float(h[i] << 16);
      v[2 * i + 1] = __uint_as_float(h[i] & 0xffff0000u);
    }
  }
};

// 8 values that are bf16-representable -> 16 bytes
__device__ __forceinline__ v4i pack8_bf16(const float* v) {
  v4i w;
#pragma unroll
  for (int i = 0; i < 4; i++) w[i] = (int)pack_bf16x2(v[2 * i], v[2 * i + 1]);
  return w;
}

// ---------------------------------------------------------------------------------------
// 1x128 quant, 16 lanes per tile, U tiles per lane group.  SCATTER: write each quantised
// row to its topk destinations (row_map), reading it once.
// ---------------------------------------------------------------------------------------
// floor(n / d) for n < 2^31 as one widening multiply and a shift: magic = floor(2^sh / d) + 1, sh = 31 + ceil(log2 d)
struct FastDiv {
  uint32_t magic;
  int sh;
  __device__ __forceinline__ uint32_t div(uint32_t n) const { return (uint32_t)(((uint64_t)n * magic) >> sh); }
};
static FastDiv make_fastdiv(uint32_t d) {
  int l = 0;
  while (((uint64_t)1 << l) < d) l++;
  FastDiv f;
  f.sh = 31 + l;
  f.magic = (uint32_t)((((uint64_t)1 << f.sh) / (uint64_t)d) + 1);
  return f;
}

// tiles per 16-lane group and pass: two keep enough loads in flight (one and four measured slower)
constexpr int kQuantU = 2;
constexpr int64_t kMaxRowLd = (int64_t)1 << 24;  // row strides (elements) of the row-wise quantisers' inputs
// A workgroup takes 16 U consecutive tiles of the row-major tile order.  These kernels run close to the rate at
// which the vector ALUs issue, so nothing that is the same in every lane is computed in the lanes: the position
// of the block's first tile comes from the scalar unit, a lane adds its small tile number to it, and every
// access is a scalar base plus a 32-bit lane offset.  The outputs are dense, so tile t of the order lies at
// byte 128 t of q; the input needs (row, column tile) only where its rows are strided.
// (the launchers keep ldx below 2^24: 16 U rows of it stay within the 32-bit offset)
template <typename IN, bool SCATTER, int U>
__global__ __launch_bounds__(256) void quant_1x128_kernel(const typename IN::elem* __restrict__ x, int64_t ldx,
                                                          int nt, FastDiv nt_div, int64_t total_tiles,
                                                          const int32_t* __restrict__ row_map, int topk,
                                                          int64_t M_out, uint8_t* __restrict__ q,
                                                          float* __restrict__ s, float eps, int64_t gate_off,
                                                          u16* __restrict__ h_out) {
  // the short division is checked for bf16 values over scales of bf16 maxima only
  const bool plain_div = !kBf16Values<IN> || eps != 0.f;
  const int grp = threadIdx.x >> 4, l = threadIdx.x & 15;
  constexpr uint32_t kEl = sizeof(typename IN::elem);
  const int64_t base = (int64_t)blockIdx.x * (16 * U);  // first tile of the block: the same in every lane
  const int64_t tiles_left = total_tiles - base;
  const uint32_t left = tiles_left < 16 * U ? (uint32_t)tiles_left : 16u * U;  // >= 1
  const int64_t cols = (int64_t)nt * kTile;
  const bool dense = !SCATTER && ldx == cols;
  int64_t row0 = 0;
  uint32_t tc0 = 0;
  if (!dense) {
    row0 = total_tiles < ((int64_t)1 << 31) ? (int64_t)nt_div.div((uint32_t)base) : base / nt;
    tc0 = (uint32_t)(base - row0 * nt);
  }
  const typename IN::elem* const xb = dense ? x + base * kTile : x + row0 * ldx;

  Raw8<IN> raw[U];
  uint32_t jt[U], wrow[U], tc[U];
  bool valid[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    uint32_t j = (uint32_t)(u * 16 + grp);
    valid[u] = j < left;
    if (!valid[u]) j = left - 1;
    jt[u] = j;
    uint32_t xoff;  // elements from xb
    if (dense) {
      xoff = j * kTile;
      wrow[u] = tc[u] = 0;
    } else {
      const uint32_t t = tc0 + j;  // below nt + 16 U
      wrow[u] = nt >= 16 * U ? (t >= (uint32_t)nt ? 1u : 0u) : nt_div.div(t);
      tc[u] = t - wrow[u] * (uint32_t)nt;
      xoff = wrow[u] * (uint32_t)ldx + tc[u] * kTile;
    }
    raw[u].load(xb, (xoff + (uint32_t)l * 8) * kEl, gate_off);
  }
  u16* const hb = h_out ? h_out + base * kTile : nullptr;
  uint8_t* const qb = q + base * kTile;
  float* const sb = s + base;
#pragma unroll
  for (int u = 0; u < U; u++) {
    float v[8];
    raw[u].get(v);
    const Divider dv = make_scale(row16_max(amax8(v)), eps, plain_div);
    const float sc = dv.s;
    const v2i codes = quant8(v, dv);
    if (!valid[u]) continue;
    const uint32_t off = jt[u] * kTile + (uint32_t)l * 8;  // element of the dense outputs, from the block's first tile
    if (h_out != nullptr) st_nt(hb, off * 2, pack8_bf16(v));  // the activation itself, for callers that keep it
    // the codes are not read again by this kernel: streaming stores keep them out of the way
    if constexpr (!SCATTER) {
      st_nt(qb, off, codes);
      if (l == 0) sb[jt[u]] = sc;
    } else {
      const int64_t row = row0 + wrow[u];
      for (int j = 0; j < topk; j++) {
        const int64_t dst = row_map[row * topk + j];
        if (dst < 0 || dst >= M_out) continue;
        __builtin_nontemporal_store(codes, reinterpret_cast<v2i*>(q + dst * cols + (int64_t)tc[u] * kTile + l * 8));
        if (l == 0) s[dst * nt + tc[u]] = sc;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// 128x128 register tile shared by the dual (row + transposed) quant and the block quant:
// 256 threads, thread (gr = tid/16, c = tid%16) holds rows gr*8 .. gr*8+7, columns c*8 .. c*8+7.
// ---------------------------------------------------------------------------------------
constexpr int kTLd = kTile + 16;  // LDS row stride (bytes) of the transposed code tile
// 128 rows of a tile are addressed with 32-bit byte offsets: row strides (elements, at most 4 bytes each) stay below this
constexpr int64_t kMaxTileLd = (int64_t)1 << 22;

// `x` is the tile's origin, the same in every lane; FULL: all 128 rows are valid
template <typename IN, bool FULL>
__device__ __forceinline__ void issue_tile_loads(const typename IN::elem* __restrict__ x, uint32_t ldx, int rows_valid,
                                                 Raw8<IN> (&raw)[8], int64_t gate_off = 0) {
  const int gr = (int)threadIdx.x >> 4, c = (int)threadIdx.x & 15;
  constexpr uint32_t kEl = sizeof(typename IN::elem);
  const uint32_t off0 = ((uint32_t)(gr * 8) * ldx + (uint32_t)c * 8) * kEl;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    if (FULL || gr * 8 + i < rows_valid)
      raw[i].load(x, off0 + (uint32_t)i * ldx * kEl, gate_off);
    else
      raw[i].zero();
  }
}
template <typename IN, bool FULL>
__device__ __forceinline__ void load_tile(const typename IN::elem* __restrict__ x, uint32_t ldx, int rows_valid,
                                          float (&v)[8][8], int64_t gate_off = 0) {
  Raw8<IN> raw[8];
  issue_tile_loads<IN, FULL>(x, ldx, rows_valid, raw, gate_off);
#pragma unroll
  for (int i = 0; i < 8; i++) raw[i].get(v[i]);
}

// Byte `b` of row `r` of the staged code tile.  A thread writes the few codes it holds of a row, and the lanes
// c = 0..15 of a wave do so in rows eight apart: 8 * 144 bytes is a multiple of 128, so without more ado sixteen
// lanes would meet in one or two LDS banks.  The 16-byte chunk index inside the row is therefore XORed with three
// bits of the row: the 64 lanes of a write then spread evenly over all banks, and a row is still read back as
// eight whole 16-byte chunks, in permuted order.
__device__ __forceinline__ int staged_off(int r, int b) { return r * kTLd + (b ^ (((r >> 4) & 7) << 4)); }

// the staged 128 x 128 code tile written as rows of 128 bytes, one 16-byte store per lane
// (`out`: the tile's origin, the same in every lane; 128 ld_out < 2^32)
__device__ __forceinline__ void store_staged_tile(const uint8_t* tile_t, uint8_t* __restrict__ out, uint32_t ld_out) {
  __syncthreads();
#pragma unroll
  for (int n = 0; n < 4; n++) {
    const int idx = (int)threadIdx.x + 256 * n;
    const int r = idx >> 3, ch = idx & 7;
    st_nt(out, (uint32_t)r * ld_out + (uint32_t)ch * 16, *reinterpret_cast<const v4i*>(tile_t + staged_off(r, ch * 16)));
  }
}

// Where tile (token tile pt, column tile kc) of the transposed codes goes, and the stride of its 128 rows.
// Layout 0: q_t is [cols, ld_t], a row per column of x; layout 1 (AAMD_QT_BLOCKED): q_t is [ld_t / 128, cols, 128],
// token-block-major, so that a tile is 16 KB of consecutive bytes and the tiles of a token block follow each other:
// the kernel then writes the transposed codes as one sequential sweep instead of 128-byte pieces ld_t apart.
__device__ __forceinline__ uint8_t* qt_tile(uint8_t* q_t, int blocked, int64_t cols, uint32_t ld_t, int pt, int kc, uint32_t* ld) {
  *ld = blocked ? (uint32_t)kTile : ld_t;
  return blocked ? q_t + ((int64_t)pt * cols + (int64_t)kc * kTile) * kTile
                 : q_t + (int64_t)kc * kTile * ld_t + (int64_t)pt * kTile;
}

// One 128 x 128 tile of the dual quantiser: token tile pt of group g, column tile kc.  Everything that
// locates the tile is the same in every lane, so each access is a scalar base plus a 32-bit lane offset
// (the launchers bound the row strides so that 128 rows stay below 2^32 bytes).
// GATHER: row r of the tile is source row src_row[r] of x (the token permute fused in: x is in token order,
// the outputs in expert-contiguous order); src_row lives in LDS and holds every valid row of the tile.
template <typename IN, bool FULL, bool GATHER = false>
__device__ __forceinline__ void dual_tile(const typename IN::elem* __restrict__ x, uint32_t ldx, int nt, int64_t m0,
                                          int mvalid, int pt, int kc, uint8_t* __restrict__ q, float* __restrict__ s,
                                          uint8_t* __restrict__ q_t, float* __restrict__ s_t, uint32_t ld_t, int blocked,
                                          float eps, int64_t gate_off, u16* __restrict__ h_out, uint8_t* tile_t,
                                          Divider* cdiv, const uint32_t* src_row = nullptr, const void* lut = nullptr) {
  const bool plain_div = !kBf16Values<IN> || eps != 0.f;  // see make_scale
  float (*part)[kTile] = reinterpret_cast<float (*)[kTile]>(tile_t);
  const int64_t cols = (int64_t)nt * kTile;
  const int gr = (int)threadIdx.x >> 4, c = (int)threadIdx.x & 15;

  // The GELU kernels hold their results, which are bf16 numbers, packed two to a register until the column pass
  // (the erf evaluation needs the registers: unpacked, two workgroups fit on a CU instead of four).  For the other
  // inputs the 64 values of a thread stay in fp32: the packed form compiles to more registers there, not fewer.
  constexpr bool kPacked = std::is_same<IN, GELU>::value || std::is_same<IN, GELUB>::value;
  Raw8<IN> raw[8];
  if constexpr (GATHER) {
    // a row's 256-byte segment (16 lanes x 16 bytes) stays one coalesced access; only its base is looked up
    constexpr uint32_t kEl = sizeof(typename IN::elem);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if (FULL || gr * 8 + i < mvalid)
        raw[i].load(x + (int64_t)src_row[gr * 8 + i] * ldx + (int64_t)kc * kTile, (uint32_t)c * 8 * kEl, gate_off);
      else
        raw[i].zero();
    }
  } else {
    issue_tile_loads<IN, FULL>(x + m0 * ldx + (int64_t)kc * kTile, ldx, mvalid, raw, gate_off);
  }
  float v[kPacked ? 1 : 8][8];
  uint32_t vp[kPacked ? 8 : 1][4];

  // row-wise 1x128 codes and scales (a tile row lives in one 16-lane DPP row)
  u16* const hb = h_out ? h_out + m0 * cols + (int64_t)kc * kTile : nullptr;
  uint8_t* const qb = q ? q + m0 * cols + (int64_t)kc * kTile : nullptr;
  float* const sb = q ? s + m0 * nt + kc : nullptr;
  const uint32_t ucols = (uint32_t)cols;
  float cm[8];
#pragma unroll
  for (int j = 0; j < 8; j++) cm[j] = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const uint32_t r = (uint32_t)(gr * 8 + i);
    const bool live = FULL || (int)r < mvalid;
    float (&vi)[8] = v[kPacked ? 0 : i];
    // (a row is unpacked where its turn comes: hoisted to the top, the rows of the whole tile would be live unpacked)
    if constexpr (kPacked) {
      raw[i].pin();
      raw[i].get(vi, lut);  // the activation from its table in LDS
    } else {
      raw[i].get(vi);
    }
    if constexpr (kPacked) {
      const v4i pk = pack8_bf16(vi);
#pragma unroll
      for (int k = 0; k < 4; k++) vp[i][k] = (uint32_t)pk[k];
#pragma unroll
      for (int j = 0; j < 8; j++) cm[j] = fmaxf(cm[j], fabsf(vi[j]));
    }
    if (hb != nullptr && live) st_nt(hb, (r * ucols + (uint32_t)c * 8) * 2, pack8_bf16(vi));
    if (qb != nullptr) {
      const Divider dv = make_scale(row16_max(amax8(vi)), eps, plain_div);
      const v2i codes = quant8(vi, dv);
      if (live) {
        st_nt(qb, r * ucols + (uint32_t)c * 8, codes);
        if (c == 0) *reinterpret_cast<float*>(reinterpret_cast<char*>(sb) + r * (uint32_t)nt * 4) = dv.s;
      }
    }
    if constexpr (kPacked) {
#pragma unroll
      for (int k = 0; k < 4; k++) asm volatile("" : "+v"(vp[i][k]));  // the row is finished before the next one is unpacked
    }
  }
  // column amax over the 128 tokens of the tile (two rows per three-operand maximum)
#pragma unroll
  for (int j = 0; j < 8; j++) {
    if constexpr (!kPacked) {
#pragma unroll
      for (int i = 0; i < 8; i += 2) cm[j] = fmaxf(fmaxf(cm[j], fabsf(v[i][j])), fabsf(v[i + 1][j]));
    }
    part[gr][c * 8 + j] = cm[j];
  }
  __syncthreads();
  if ((int)threadIdx.x < kTile) {
    float m = part[0][(int)threadIdx.x];
#pragma unroll
    for (int i = 1; i < 16; i++) m = fmaxf(m, part[i][(int)threadIdx.x]);
    const Divider dv = make_scale(m, eps, plain_div);
    cdiv[((int)threadIdx.x & 7) * 16 + ((int)threadIdx.x >> 3)] = dv;  // [column % 8][column / 8]: lanes of a row read 16 neighbours
    (s_t + (int64_t)pt * cols + (int64_t)kc * kTile)[(int)threadIdx.x] = dv.s;
  }
  __syncthreads();
  // codes of the 8x8 register block, transposed through LDS, written as rows of 128 bytes
#pragma unroll
  for (int j = 0; j < 8; j++) {
    float col[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if constexpr (kPacked) col[i] = __uint_as_float(j & 1 ? vp[i][j / 2] & 0xffff0000u : vp[i][j / 2] << 16);
      else col[i] = v[i][j];
    }
    *reinterpret_cast<v2i*>(tile_t + staged_off(c * 8 + j, gr * 8)) = quant8(col, cdiv[j * 16 + c]);
  }
  uint32_t ld_out;
  uint8_t* const out_t = qt_tile(q_t, blocked, cols, ld_t, pt, kc, &ld_out);
  store_staged_tile(tile_t, out_t, ld_out);
}

template <typename IN>
__global__ __launch_bounds__(256) void quant_dual_grouped_kernel(
    const typename IN::elem* __restrict__ x, int64_t ldx, int nt, const int64_t* __restrict__ goff,
    const int32_t* __restrict__ tile_off, int E, uint8_t* __restrict__ q, float* __restrict__ s,
    uint8_t* __restrict__ q_t, float* __restrict__ s_t, int64_t ld_t, int blocked, float eps, int64_t gate_off,
    u16* __restrict__ h_out) {
  // the per-row-group column maxima are dead before the transposed codes are staged: one region
  __shared__ __attribute__((aligned(16))) uint8_t tile_t[kTile * kTLd];
  static_assert(sizeof(float) * 16 * kTile <= sizeof(tile_t), "the column maxima fit in the staging region");
  __shared__ Divider cdiv[kTile];  // scale and divider of every column of the tile
  __shared__ int slot;
  // the activation's table (GELU forms only), copied from the library's array; find_group's barriers order the
  // copy before the tile's reads
  __shared__ __attribute__((aligned(16))) uint8_t lut_s[kLutBytes<IN> ? kLutBytes<IN> : 16];
  if constexpr (kLutBytes<IN> != 0) {
    const v4i* const src = reinterpret_cast<const v4i*>(std::is_same<IN, GELU>::value ? (const void*)g_gelu_lut : (const void*)g_gelub_lut);
    for (uint32_t i = threadIdx.x; i < kLutBytes<IN> / 16; i += 256) reinterpret_cast<v4i*>(lut_s)[i] = src[i];
  }

  // Workgroups go to the eight XCDs in turn, and the row-wise scales of a tile are 128 single floats, one
  // per row: with tile = workgroup index, the eight floats of a 32-byte sector would come from eight
  // different L2 caches and reach memory as eight partial writes.  The index is therefore re-dealt so
  // that eight consecutive workgroups of one XCD take eight consecutive column tiles of one token tile.
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  {
    const uint32_t ntx = gridDim.x, per_row = ntx >> 3;
    const uint32_t lin = by * ntx + bx, chunks = gridDim.y * per_row;
    if ((ntx & 7) == 0 && lin < (chunks & ~7u) * 8) {
      const uint32_t j = lin >> 3, chunk = (j & ~7u) + (lin & 7);
      by = chunk / per_row;
      bx = (chunk - by * per_row) * 8 + (j & 7);
    }
  }
  const int pt = (int)by, kc = (int)bx;
  const int g = __builtin_amdgcn_readfirstlane(find_group(tile_off, E, pt, &slot));
  if (g >= E) return;
  const int64_t m0 = goff[g] + (int64_t)(pt - tile_off[g]) * kTile;
  const int64_t left = goff[g + 1] - m0;
  const int mvalid = left < kTile ? (int)left : kTile;
  if (mvalid == kTile)
    dual_tile<IN, true>(x, (uint32_t)ldx, nt, m0, mvalid, pt, kc, q, s, q_t, s_t, (uint32_t)ld_t, blocked, eps, gate_off, h_out, tile_t, cdiv, nullptr, lut_s);
  else
    dual_tile<IN, false>(x, (uint32_t)ldx, nt, m0, mvalid, pt, kc, q, s, q_t, s_t, (uint32_t)ld_t, blocked, eps, gate_off, h_out, tile_t, cdiv, nullptr, lut_s);
}

// The dual quantiser with the token permute fused in: x holds the tokens in their original order, and permuted
// row j (the rows of every output) is a copy of token sorted_idx[j] / topk, the stable order of the router
// preprocess.  A workgroup looks up the source rows of its 128 permuted rows once (flat index / topk by a
// multiply and a shift: magic = floor(2^sh / topk) + 1 with 2^(sh - 31) >= topk, exact for indices below 2^31)
// and then runs the tile of the grouped kernel on gathered rows.  Source rows are clamped to the token count,
// so a corrupt index reads a wrong row, never beyond x.
template <typename IN>
__global__ __launch_bounds__(256) void quant_dual_gather_kernel(
    const typename IN::elem* __restrict__ x, int64_t ldx, int nt, const int64_t* __restrict__ sorted_idx,
    uint32_t magic, int sh, uint32_t T, const int64_t* __restrict__ goff, const int32_t* __restrict__ tile_off, int E,
    uint8_t* __restrict__ q, float* __restrict__ s, uint8_t* __restrict__ q_t, float* __restrict__ s_t, int64_t ld_t,
    int blocked, float eps) {
  __shared__ __attribute__((aligned(16))) uint8_t tile_t[kTile * kTLd];
  __shared__ Divider cdiv[kTile];
  __shared__ uint32_t src_row[kTile];
  __shared__ int slot;
  uint32_t bx = blockIdx.x, by = blockIdx.y;  // eight column tiles of a token tile on one XCD: see quant_dual_grouped_kernel
  {
    const uint32_t ntx = gridDim.x, per_row = ntx >> 3;
    const uint32_t lin = by * ntx + bx, chunks = gridDim.y * per_row;
    if ((ntx & 7) == 0 && lin < (chunks & ~7u) * 8) {
      const uint32_t j = lin >> 3, chunk = (j & ~7u) + (lin & 7);
      by = chunk / per_row;
      bx = (chunk - by * per_row) * 8 + (j & 7);
    }
  }
  const int pt = (int)by, kc = (int)bx;
  const int g = __builtin_amdgcn_readfirstlane(find_group(tile_off, E, pt, &slot));
  if (g >= E) return;
  const int64_t m0 = goff[g] + (int64_t)(pt - tile_off[g]) * kTile;
  const int64_t left = goff[g + 1] - m0;
  const int mvalid = left < kTile ? (int)left : kTile;
  if ((int)threadIdx.x < mvalid) {
    const uint32_t flat = (uint32_t)sorted_idx[m0 + (int)threadIdx.x];
    const uint32_t tok = (uint32_t)(((uint64_t)flat * magic) >> sh);
    src_row[threadIdx.x] = tok < T ? tok : T - 1;
  }
  __syncthreads();
  if (mvalid == kTile)
    dual_tile<IN, true, true>(x, (uint32_t)ldx, nt, m0, mvalid, pt, kc, q, s, q_t, s_t, (uint32_t)ld_t, blocked, eps, 0, nullptr, tile_t, cdiv, src_row);
  else
    dual_tile<IN, false, true>(x, (uint32_t)ldx, nt, m0, mvalid, pt, kc, q, s, q_t, s_t, (uint32_t)ld_t, blocked, eps, 0, nullptr, tile_t, cdiv, src_row);
}

// ---------------------------------------------------------------------------------------
// SwiGLU backward with both quantisations: rows [a | b] plus the gradient dh of h give the [da | db] row,
//   da = bf16(bf16(dh*b) * sig(a) * (1 + a*(1 - sig(a)))),  db = bf16(dh * bf16(silu(a))),
// what autograd makes of the two torch ops on bf16 tensors (grouped_gemm_moe.py:331-334).  One workgroup of 512
// threads per 128 tokens x 128 features makes the da tile and the db tile of those features from one read of a, b
// and dh and one sigmoid per position.
// Thread (gr = tid / 16, c = tid % 16) holds rows gr*4 .. gr*4+3, columns c*8 .. c*8+7 of both tiles.
// ---------------------------------------------------------------------------------------
// sigmoid(a) in fp32 per bf16 value a, for |a| in [2^-14, 2^4), read from LDS like the GELU tables (filled ahead of
// every launch by the kernel's own sigmoid; inside the table range a sigmoid(a) equals the scaled form's silu bit
// for bit: neither product leaves the normal range there)
constexpr uint32_t kSigLo = (uint32_t)(127 - 14) << 7;
constexpr uint32_t kSigN = (uint32_t)(14 + 4) << 7;
static __device__ __attribute__((aligned(16))) float g_sigmoid_lut[2 * kSigN];
__global__ __launch_bounds__(256) void sigmoid_lut_kernel() {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= 2 * kSigN) return;
  const uint32_t sign = i >= kSigN ? 1u : 0u;
  const float x = __uint_as_float(((sign << 15) | (kSigLo + i - sign * kSigN)) << 16);
  g_sigmoid_lut[i] = sigmoid_scaled(x) * 0x1p-16f;
}

// 4 values / one scale -> 4 codes in one dword
__device__ __forceinline__ int quant4(const float* v, const Divider& d) {
  float t[4];
  if (__builtin_expect(d.plain, 0)) {
#pragma unroll
    for (int i = 0; i < 4; i++) t[i] = v[i] / d.s;
    return pack2_fp8<true>(t[2], t[3], pack2_fp8<false>(t[0], t[1], 0));
  }
#pragma unroll
  for (int i = 0; i < 4; i++) t[i] = __builtin_fmaf(v[i], d.yh, v[i] * d.yl);
  return pack2_fp8<true>(t[2], t[3], pack2_fp8<false>(t[0], t[1], 0));
}

template <bool FULL>
__device__ __forceinline__ void swiglu_bwd_dual_tile(const u16* __restrict__ xa /* a at the tile's origin */, uint32_t ld,
                                                     int64_t gate_off, const u16* __restrict__ xd, uint32_t ld_dh, int nt,
                                                     int64_t m0, int mvalid, int pt, int f, uint8_t* __restrict__ q,
                                                     float* __restrict__ s, uint8_t* __restrict__ q_t,
                                                     float* __restrict__ s_t, uint32_t ld_t, int blocked,
                                                     u16* __restrict__ g_out, uint8_t (*tile_t)[kTile * kTLd],
                                                     Divider (*cdiv)[kTile], const float* sig_lut) {
  const int tid = threadIdx.x, gr = tid >> 4, c = tid & 15;
  const int half = nt / 2;
  const int64_t cols = (int64_t)nt * kTile;
  const uint32_t ucols = (uint32_t)cols;
  // ---- loads, then da and db of the thread's 4 x 8 positions
  v4i ra[4], rb[4], rd[4];
  {
    const uint32_t off0 = ((uint32_t)(gr * 4) * ld + (uint32_t)c * 8) * 2, off0d = ((uint32_t)(gr * 4) * ld_dh + (uint32_t)c * 8) * 2;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (FULL || gr * 4 + i < mvalid) {
        ra[i] = ld16_nt(xa, off0 + (uint32_t)i * ld * 2);
        rb[i] = ld16_nt(xa + gate_off, off0 + (uint32_t)i * ld * 2);
        rd[i] = ld16_nt(xd, off0d + (uint32_t)i * ld_dh * 2);
      } else {
        ra[i] = rb[i] = rd[i] = v4i{0, 0, 0, 0};
      }
    }
  }
  uint32_t vp[2][4][4];  // [da | db][row][column pair]: the results are bf16 numbers and wait for the column pass packed
  float (*part)[32][kTile] = reinterpret_cast<float (*)[32][kTile]>(&tile_t[0][0]);  // [2][32][128] floats: dead before the staging
  static_assert(sizeof(float) * 2 * 32 * kTile <= 2 * sizeof(tile_t[0]), "the column maxima fit in the staging regions");
  float cm[2][8];
#pragma unroll
  for (int w = 0; w < 2; w++)
#pragma unroll
    for (int j = 0; j < 8; j++) cm[w][j] = 0.f;
  // one row at a time, from the packed inputs to the stored codes of both tiles
#pragma unroll
  for (int i = 0; i < 4; i++) {
    float fa[8], fb[8], fd[8], v[2][8];
    unpack8(ra[i], fa);
    unpack8(rb[i], fb);
    unpack8(rd[i], fd);
    // sigmoid(a) of the row's eight values from the table, all reads issued together; silu = a sigmoid(a)
    float sg[8], sil[8];
    {
      uint32_t t[8];
      bool ok = true;
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const uint32_t w = (uint32_t)ra[i][k];
        const uint32_t m0 = (w & 0x7fffu) - kSigLo, m1 = ((w >> 16) & 0x7fffu) - kSigLo;
        ok = ok && m0 < kSigN && m1 < kSigN;
        t[2 * k] = m0 < kSigN ? m0 + ((w >> 15) & 1u) * kSigN : 0u;
        t[2 * k + 1] = m1 < kSigN ? m1 + (w >> 31) * kSigN : 0u;
      }
#pragma unroll
      for (int k = 0; k < 8; k++) sg[k] = sig_lut[t[k]];
#pragma unroll
      for (int k = 0; k < 8; k++) sil[k] = fa[k] * sg[k];
      if (__builtin_expect(!ok, 0)) {  // values outside the table (zeros, outliers): the arithmetic
#pragma unroll
        for (int k = 0; k < 8; k++) {
          if ((__float_as_uint(fa[k]) >> 16 & 0x7fffu) - kSigLo >= kSigN) {
            const float rs = sigmoid_scaled(fa[k]);
            sg[k] = rs * 0x1p-16f;
            sil[k] = silu_from(fa[k], rs);
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < 8; k += 2) {
      // db = bf16(dh * bf16(silu(a)))
      const uint32_t sl = pack_bf16x2(sil[k], sil[k + 1]);
      const uint32_t ob = pack_bf16x2(fd[k] * __uint_as_float(sl << 16), fd[k + 1] * __uint_as_float(sl & 0xffff0000u));
      vp[1][i][k / 2] = ob;
      v[1][k] = __uint_as_float(ob << 16);
      v[1][k + 1] = __uint_as_float(ob & 0xffff0000u);
      // da = bf16(bf16(dh * b) * sig(a) * (1 + a * (1 - sig(a))))
      const float sg0 = sg[k], sg1 = sg[k + 1];
      const uint32_t gb = pack_bf16x2(fd[k] * fb[k], fd[k + 1] * fb[k + 1]);
      const uint32_t oa = pack_bf16x2((__uint_as_float(gb << 16) * sg0) * (1.0f + fa[k] * (1.0f - sg0)),
                                      (__uint_as_float(gb & 0xffff0000u) * sg1) * (1.0f + fa[k + 1] * (1.0f - sg1)));
      vp[0][i][k / 2] = oa;
      v[0][k] = __uint_as_float(oa << 16);
      v[0][k + 1] = __uint_as_float(oa & 0xffff0000u);
    }
    const uint32_t r = (uint32_t)(gr * 4 + i);
    const bool live = FULL || (int)r < mvalid;
#pragma unroll
    for (int w = 0; w < 2; w++) {
      const int kc = w == 0 ? f : half + f;
#pragma unroll
      for (int j = 0; j < 8; j++) cm[w][j] = fmaxf(cm[w][j], fabsf(v[w][j]));
      if (g_out != nullptr && live)
        st_nt(g_out + m0 * cols + (int64_t)kc * kTile, (r * ucols + (uint32_t)c * 8) * 2,
              v4i{(int)vp[w][i][0], (int)vp[w][i][1], (int)vp[w][i][2], (int)vp[w][i][3]});
      if (q != nullptr) {
        const Divider dv = make_scale(row16_max(amax8(v[w])), 0.f, false);
        const v2i codes = quant8<false>(v[w], dv);
        if (live) {
          st_nt(q + m0 * cols + (int64_t)kc * kTile, r * ucols + (uint32_t)c * 8, codes);
          if (c == 0) *reinterpret_cast<float*>(reinterpret_cast<char*>(s + m0 * nt + kc) + r * (uint32_t)nt * 4) = dv.s;
        }
      }
    }
#pragma unroll
    for (int w = 0; w < 2; w++)
#pragma unroll
      for (int j = 0; j < 4; j++) asm volatile("" : "+v"(vp[w][i][j]));  // the row is finished before the next one starts
  }
#pragma unroll
  for (int w = 0; w < 2; w++)
#pragma unroll
    for (int j = 0; j < 8; j++) part[w][gr][c * 8 + j] = cm[w][j];
  __syncthreads();
  if (tid < 2 * kTile) {
    const int w = tid >> 7, col = tid & (kTile - 1);
    float m = part[w][0][col];
#pragma unroll
    for (int i = 1; i < 32; i++) m = fmaxf(m, part[w][i][col]);
    const Divider dv = make_scale(m, 0.f, false);
    cdiv[w][(col & 7) * 16 + (col >> 3)] = dv;  // [column % 8][column / 8]: lanes of a row read 16 neighbours
    (s_t + (int64_t)pt * cols + (int64_t)(w == 0 ? f : half + f) * kTile)[col] = dv.s;
  }
  __syncthreads();
  // ---- transposed codes through the LDS
#pragma unroll
  for (int w = 0; w < 2; w++)
#pragma unroll
    for (int j = 0; j < 8; j++) {
      float col[4];
#pragma unroll
      for (int i = 0; i < 4; i++) col[i] = __uint_as_float(j & 1 ? vp[w][i][j / 2] & 0xffff0000u : vp[w][i][j / 2] << 16);
      *reinterpret_cast<int*>(&tile_t[w][staged_off(c * 8 + j, gr * 4)]) = quant4(col, cdiv[w][j * 16 + c]);
      if (j % 4 == 3) __builtin_amdgcn_sched_barrier(0);  // a few dividers at a time: sixteen of them are 64 registers
    }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < 2; w++) {
    uint32_t ld_out;
    uint8_t* const out = qt_tile(q_t, blocked, cols, ld_t, pt, w == 0 ? f : half + f, &ld_out);
#pragma unroll
    for (int n = 0; n < 2; n++) {
      const int idx = tid + 512 * n;
      const int r = idx >> 3, ch = idx & 7;
      st_nt(out, (uint32_t)r * ld_out + (uint32_t)ch * 16, *reinterpret_cast<const v4i*>(&tile_t[w][staged_off(r, ch * 16)]));
    }
  }
}

__global__ __launch_bounds__(512, 4) void swiglu_bwd_dual_kernel(const u16* __restrict__ fc1, int64_t ld, int64_t gate_off,
                                                              const u16* __restrict__ dh, int64_t ld_dh, int nt,
                                                              const int64_t* __restrict__ goff,
                                                              const int32_t* __restrict__ tile_off, int E,
                                                              uint8_t* __restrict__ q, float* __restrict__ s,
                                                              uint8_t* __restrict__ q_t, float* __restrict__ s_t,
                                                              int64_t ld_t, int blocked, u16* __restrict__ g_out) {
  __shared__ __attribute__((aligned(16))) uint8_t tile_ts[2][kTile * kTLd];
  __shared__ Divider cdivs[2][kTile];
  __shared__ int slot;
  __shared__ __attribute__((aligned(16))) float sig_s[2 * kSigN];  // find_group's barriers order the copy before its reads
  for (uint32_t i = threadIdx.x; i < 2 * kSigN / 4; i += 512)
    reinterpret_cast<v4i*>(sig_s)[i] = reinterpret_cast<const v4i*>(g_sigmoid_lut)[i];
  // consecutive workgroups of one XCD take the eight consecutive feature tiles of a scale sector
  // (see quant_dual_grouped_kernel)
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  {
    const uint32_t ntx = gridDim.x, per_row = ntx >> 3;
    const uint32_t lin = by * ntx + bx, chunks = gridDim.y * per_row;
    if ((ntx & 7) == 0 && lin < (chunks & ~7u) * 8) {
      const uint32_t j = lin >> 3, chunk = (j & ~7u) + (lin & 7);
      by = chunk / per_row;
      bx = (chunk - by * per_row) * 8 + (j & 7);
    }
  }
  const int pt = (int)by, f = (int)bx;
  const int g = __builtin_amdgcn_readfirstlane(find_group(tile_off, E, pt, &slot));
  if (g >= E) return;
  const int64_t m0 = goff[g] + (int64_t)(pt - tile_off[g]) * kTile;
  const int64_t left = goff[g + 1] - m0;
  const int mvalid = left < kTile ? (int)left : kTile;
  const u16* const xa = fc1 + m0 * ld + (int64_t)f * kTile;
  const u16* const xd = dh + m0 * ld_dh + (int64_t)f * kTile;
  if (mvalid == kTile)
    swiglu_bwd_dual_tile<true>(xa, (uint32_t)ld, gate_off, xd, (uint32_t)ld_dh, nt, m0, mvalid, pt, f, q, s, q_t, s_t,
                               (uint32_t)ld_t, blocked, g_out, tile_ts, cdivs, sig_s);
  else
    swiglu_bwd_dual_tile<false>(xa, (uint32_t)ld, gate_off, xd, (uint32_t)ld_dh, nt, m0, mvalid, pt, f, q, s, q_t, s_t,
                                (uint32_t)ld_t, blocked, g_out, tile_ts, cdivs, sig_s);
}

// The 8x8 byte matrix held as eight rows of two dwords, transposed with byte permutes: cols[j]
// holds byte j of rows 0..7.  (v_perm_b32 selects bytes 0-3 from its second source, 4-7 from the first.)
__device__ __forceinline__ void transpose8x8_bytes(const v2i (&rows)[8], v2i (&cols)[8]) {
#pragma unroll
  for (int jb = 0; jb < 2; jb++)
#pragma unroll
    for (int ib = 0; ib < 2; ib++) {
      const uint32_t a = (uint32_t)rows[4 * ib][jb], b = (uint32_t)rows[4 * ib + 1][jb];
      const uint32_t c = (uint32_t)rows[4 * ib + 2][jb], d = (uint32_t)rows[4 * ib + 3][jb];
      const uint32_t x0 = __builtin_amdgcn_perm(b, a, 0x05010400u);  // a0 b0 a1 b1
      const uint32_t x1 = __builtin_amdgcn_perm(b, a, 0x07030602u);  // a2 b2 a3 b3
      const uint32_t y0 = __builtin_amdgcn_perm(d, c, 0x05010400u);
      const uint32_t y1 = __builtin_amdgcn_perm(d, c, 0x07030602u);
      cols[4 * jb + 0][ib] = (int)__builtin_amdgcn_perm(y0, x0, 0x05040100u);  // a0 b0 c0 d0
      cols[4 * jb + 1][ib] = (int)__builtin_amdgcn_perm(y0, x0, 0x07060302u);
      cols[4 * jb + 2][ib] = (int)__builtin_amdgcn_perm(y1, x1, 0x05040100u);
      cols[4 * jb + 3][ib] = (int)__builtin_amdgcn_perm(y1, x1, 0x07060302u);
    }
}

template <typename IN>
__global__ __launch_bounds__(256) void quant_128x128_kernel(const typename IN::elem* __restrict__ w,
                                                            int64_t expert_stride, int64_t N, int64_t K,
                                                            uint8_t* __restrict__ q, float* __restrict__ s,
                                                            uint8_t* __restrict__ q_t, float* __restrict__ s_t,
                                                            float eps) {
  const bool plain_div = !kBf16Values<IN> || eps != 0.f;  // see make_scale
  __shared__ float part[16];
  __shared__ __attribute__((aligned(16))) uint8_t tile_t[kTile * kTLd];
  const int kb = blockIdx.x, nb = blockIdx.y, e = blockIdx.z;
  const int nkb = (int)(K / kTile), nnb = (int)(N / kTile);
  const int gr = threadIdx.x >> 4, c = threadIdx.x & 15;

  float v[8][8];
  load_tile<IN, true>(w + e * expert_stride + (int64_t)nb * kTile * K + (int64_t)kb * kTile, (uint32_t)K, kTile, v);
  float m = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) m = fmaxf(m, amax8(v[i]));
  m = row16_max(m);
  if (c == 0) part[gr] = m;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; i++) m = fmaxf(m, part[i]);
  const Divider dv = make_scale(m, eps, plain_div);
  const float sc = dv.s;
  if (threadIdx.x == 0) {
    s[((int64_t)e * nnb + nb) * nkb + kb] = sc;
    if (s_t != nullptr) s_t[((int64_t)e * nkb + kb) * nnb + nb] = sc;
  }
  uint8_t* qe = q + (int64_t)e * N * K + (int64_t)nb * kTile * K + (int64_t)kb * kTile;
  v2i codes[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    codes[i] = quant8(v[i], dv);
    st_nt(qe, (uint32_t)(gr * 8 + i) * (uint32_t)K + (uint32_t)c * 8, codes[i]);
  }
  if (q_t != nullptr) {
    // one scale for the whole block: the transposed copy holds the same codes, so the 8x8 block of
    // this thread is transposed bytewise instead of being quantised a second time
    v2i cols[8];
    transpose8x8_bytes(codes, cols);
#pragma unroll
    for (int j = 0; j < 8; j++) *reinterpret_cast<v2i*>(tile_t + staged_off(c * 8 + j, gr * 8)) = cols[j];
    store_staged_tile(tile_t, q_t + (int64_t)e * N * K + (int64_t)kb * kTile * N + (int64_t)nb * kTile, (uint32_t)N);
  }
}

template <typename OUT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ q, const float* __restrict__ s,
                                                      int64_t M, int64_t N, int tile_scale,
                                                      OUT* __restrict__ y) {
  // one lane: 16 consecutive codes of one row
  const int64_t chunks_per_row = N / 16;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= M * chunks_per_row) return;
  const int64_t r = idx / chunks_per_row, ch = idx - r * chunks_per_row;
  const int64_t nt = N / kTile;
  const float sc = tile_scale ? s[r * nt + ch / 8] : s[(r / kTile) * nt + ch / 8];
  const v4i raw = *reinterpret_cast<const v4i*>(q + r * N + ch * 16);
  float o[16];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(raw[i], false);
    auto hi = __builtin_amdgcn_cvt_pk_f32_fp8(raw[i], true);
    o[4 * i] = lo[0] * sc;
    o[4 * i + 1] = lo[1] * sc;
    o[4 * i + 2] = hi[0] * sc;
    o[4 * i + 3] = hi[1] * sc;
  }
  OUT* dst = y + r * N + ch * 16;
  if constexpr (sizeof(OUT) == 4) {
#pragma unroll
    for (int i = 0; i < 4; i++)
      reinterpret_cast<v4f*>(dst)[i] = v4f{o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
  } else {
    v4i w0, w1;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      w0[i] = (int)pack_bf16x2(o[2 * i], o[2 * i + 1]);
      w1[i] = (int)pack_bf16x2(o[8 + 2 * i], o[8 + 2 * i + 1]);
    }
    reinterpret_cast<v4i*>(dst)[0] = w0;
    reinterpret_cast<v4i*>(dst)[1] = w1;
  }
}

int launch_group_tile_offsets(const int64_t* goff, int E, int tile, int32_t* tile_off, hipStream_t st);

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace aamd

using namespace aamd;

extern "C" int aamd_quant_1x128(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ldx, uint8_t* q,
                                float* s, float eps, void* stream) {
  return aamd_permute_quant_1x128(x, x_dtype, rows, cols, ldx, nullptr, 1, rows, q, s, eps, stream);
}

extern "C" int aamd_permute_quant_1x128(const void* x, int x_dtype, int64_t T, int64_t cols, int64_t ldx,
                                        const int32_t* row_map, int topk, int64_t M_out, uint8_t* q, float* s,
                                        float eps, void* stream) {
  AAMD_REQUIRE(x_dtype == AAMD_BF16 || x_dtype == AAMD_F32 || x_dtype == AAMD_F16, "quant_1x128: unsupported dtype %d", x_dtype);
  AAMD_REQUIRE(T >= 0 && cols >= 0 && cols % kTile == 0, "quant_1x128: cols=%lld must be a multiple of 128",
               (long long)cols);
  AAMD_REQUIRE(ldx >= cols && ldx % 8 == 0 && ldx < kMaxRowLd, "quant_1x128: ldx=%lld must be >= cols, a multiple of 8 and below 2^24",
               (long long)ldx);
  AAMD_REQUIRE(topk >= 1 && M_out >= 0, "quant_1x128: bad topk/M_out");
  if (T == 0 || cols == 0) return AAMD_OK;
  AAMD_REQUIRE(x && q && s, "quant_1x128: null pointer");
  AAMD_REQUIRE(aligned16(x) && aligned16(q), "quant_1x128: x and q must be 16-byte aligned");
  const int nt = (int)(cols / kTile);
  const int64_t total = T * nt;
  AAMD_REQUIRE(total < (int64_t)1 << 40, "quant_1x128: too many tiles");
  hipStream_t st = (hipStream_t)stream;
  constexpr int U = kQuantU;
  const int64_t blocks = (total + 16 * U - 1) / (16 * U);
  AAMD_REQUIRE(blocks < 0x7fffffffLL, "quant_1x128: grid too large");
  dim3 grid((unsigned)blocks), block(256);
  const FastDiv nd = make_fastdiv((uint32_t)nt);
  if (row_map == nullptr) {
    if (x_dtype == AAMD_BF16)
      quant_1x128_kernel<BF16, false, U><<<grid, block, 0, st>>>((const u16*)x, ldx, nt, nd, total, nullptr, 1, M_out, q, s, eps, 0, nullptr);
    else if (x_dtype == AAMD_F16)
      quant_1x128_kernel<F16, false, U><<<grid, block, 0, st>>>((const u16*)x, ldx, nt, nd, total, nullptr, 1, M_out, q, s, eps, 0, nullptr);
    else
      quant_1x128_kernel<F32, false, U><<<grid, block, 0, st>>>((const float*)x, ldx, nt, nd, total, nullptr, 1, M_out, q, s, eps, 0, nullptr);
  } else {
    if (x_dtype == AAMD_BF16)
      quant_1x128_kernel<BF16, true, U><<<grid, block, 0, st>>>((const u16*)x, ldx, nt, nd, total, row_map, topk, M_out, q, s, eps, 0, nullptr);
    else if (x_dtype == AAMD_F16)
      quant_1x128_kernel<F16, true, U><<<grid, block, 0, st>>>((const u16*)x, ldx, nt, nd, total, row_map, topk, M_out, q, s, eps, 0, nullptr);
    else
      quant_1x128_kernel<F32, true, U><<<grid, block, 0, st>>>((const float*)x, ldx, nt, nd, total, row_map, topk, M_out, q, s, eps, 0, nullptr);
  }
  AAMD_LAUNCH_CHECK("quant_1x128");
  return AAMD_OK;
}

extern "C" int aamd_quant_1x128_dual_grouped(const void* x, int x_dtype, int64_t M, int64_t cols, int64_t ldx,
                                             const int64_t* group_offsets, int E, int32_t* tile_ws, uint8_t* q,
                                             float* s, uint8_t* q_t, float* s_t, int64_t ld_t, int q_t_layout,
                                             float eps, void* stream) {
  AAMD_REQUIRE(x_dtype == AAMD_BF16 || x_dtype == AAMD_F32 || x_dtype == AAMD_F16, "quant_dual: unsupported dtype %d", x_dtype);
  AAMD_REQUIRE(q_t_layout == AAMD_QT_ROWS || q_t_layout == AAMD_QT_BLOCKED, "quant_dual: unknown q_t layout %d", q_t_layout);
  AAMD_REQUIRE(M >= 0 && cols >= 0 && cols % kTile == 0, "quant_dual: cols=%lld must be a multiple of 128",
               (long long)cols);
  AAMD_REQUIRE(ldx >= cols && ldx % 8 == 0 && ldx < kMaxTileLd, "quant_dual: bad ldx=%lld", (long long)ldx);
  AAMD_REQUIRE(ld_t < kMaxTileLd, "quant_dual: ld_t=%lld too large", (long long)ld_t);
  AAMD_REQUIRE(E >= 1 && group_offsets && tile_ws, "quant_dual: group_offsets / tile_ws required");
  AAMD_REQUIRE(ld_t % kTile == 0 && ld_t >= 0, "quant_dual: ld_t=%lld must be a multiple of 128", (long long)ld_t);
  AAMD_REQUIRE((q == nullptr) == (s == nullptr), "quant_dual: q and s go together");
  AAMD_REQUIRE(q_t && s_t, "quant_dual: q_t / s_t required");
  if (cols == 0) return AAMD_OK;
  // The padded tile count sum_g ceil(M_g/128) is known only on the device; floor(M/128) + E bounds
  // it.  The grid covers min(bound, ld_t/128) tiles, so no tile can land beyond column ld_t of the
  // transposed outputs; tiles past the real total find no group and exit.
  const int64_t max_tiles = M / kTile + E;
  const int64_t grid_tiles = ld_t / kTile < max_tiles ? ld_t / kTile : max_tiles;
  if (grid_tiles == 0) return AAMD_OK;
  AAMD_REQUIRE(aligned16(x) && aligned16(q_t) && (!q || aligned16(q)), "quant_dual: pointers must be 16-byte aligned");
  AAMD_REQUIRE(grid_tiles <= 65535, "quant_dual: more than 65535 token tiles");
  hipStream_t st = (hipStream_t)stream;
  int rc = launch_group_tile_offsets(group_offsets, E, kTile, tile_ws, st);
  if (rc) return rc;
  dim3 grid((unsigned)(cols / kTile), (unsigned)grid_tiles), block(256);
  const int nt = (int)(cols / kTile);
  if (x_dtype == AAMD_BF16)
    quant_dual_grouped_kernel<BF16><<<grid, block, 0, st>>>((const u16*)x, ldx, nt, group_offsets, tile_ws, E, q, s, q_t, s_t, ld_t, q_t_layout, eps, 0, nullptr);
  else if (x_dtype == AAMD_F16)
    quant_dual_grouped_kernel<F16><<<grid, block, 0, st>>>((const u16*)x, ldx, nt, group_offsets, tile_ws, E, q, s, q_t, s_t, ld_t, q_t_layout, eps, 0, nullptr);
  else
    quant_dual_grouped_kernel<F32><<<grid, block, 0, st>>>((const float*)x, ldx, nt, group_offsets, tile_ws, E, q, s, q_t, s_t, ld_t, q_t_layout, eps, 0, nullptr);
  AAMD_LAUNCH_CHECK("quant_dual_grouped");
  return AAMD_OK;
}

extern "C" int aamd_permute_quant_1x128_dual_grouped(const void* x, int x_dtype, int64_t T, int64_t cols, int64_t ldx,
                                                     const int64_t* sorted_idx, int topk, int64_t M,
                                                     const int64_t* group_offsets, int E, int32_t* tile_ws, uint8_t* q,
                                                     float* s, uint8_t* q_t, float* s_t, int64_t ld_t, int q_t_layout,
                                                     float eps, void* stream) {
  AAMD_REQUIRE(x_dtype == AAMD_BF16 || x_dtype == AAMD_F32 || x_dtype == AAMD_F16, "permute_quant_dual: unsupported dtype %d", x_dtype);
  AAMD_REQUIRE(q_t_layout == AAMD_QT_ROWS || q_t_layout == AAMD_QT_BLOCKED, "permute_quant_dual: unknown q_t layout %d", q_t_layout);
  AAMD_REQUIRE(T >= 0 && M >= 0 && cols >= 0 && cols % kTile == 0, "permute_quant_dual: cols=%lld must be a multiple of 128",
               (long long)cols);
  AAMD_REQUIRE(ldx >= cols && ldx % 8 == 0, "permute_quant_dual: bad ldx=%lld", (long long)ldx);
  AAMD_REQUIRE(topk >= 1 && topk <= 32768, "permute_quant_dual: topk=%d out of range", topk);
  AAMD_REQUIRE(T * topk < ((int64_t)1 << 31) && M <= T * topk, "permute_quant_dual: T * topk must stay below 2^31 and M within it");
  AAMD_REQUIRE(ld_t < kMaxTileLd && cols < kMaxTileLd, "permute_quant_dual: ld_t=%lld too large", (long long)ld_t);
  AAMD_REQUIRE(E >= 1 && group_offsets && tile_ws, "permute_quant_dual: group_offsets / tile_ws required");
  AAMD_REQUIRE(ld_t % kTile == 0 && ld_t >= 0, "permute_quant_dual: ld_t=%lld must be a multiple of 128", (long long)ld_t);
  AAMD_REQUIRE((q == nullptr) == (s == nullptr), "permute_quant_dual: q and s go together");
  AAMD_REQUIRE(q_t && s_t, "permute_quant_dual: q_t / s_t required");
  if (cols == 0 || M == 0) return AAMD_OK;
  AAMD_REQUIRE(T > 0 && x && sorted_idx, "permute_quant_dual: null input");
  const int64_t max_tiles = M / kTile + E;
  const int64_t grid_tiles = ld_t / kTile < max_tiles ? ld_t / kTile : max_tiles;
  if (grid_tiles == 0) return AAMD_OK;
  AAMD_REQUIRE(aligned16(x) && aligned16(q_t) && (!q || aligned16(q)), "permute_quant_dual: pointers must be 16-byte aligned");
  AAMD_REQUIRE(grid_tiles <= 65535, "permute_quant_dual: more than 65535 token tiles");
  // flat / topk == (flat * magic) >> sh for flat < 2^31: magic = floor(2^sh / topk) + 1, sh = 31 + ceil(log2 topk)
  int l = 0;
  while ((1 << l) < topk) l++;
  const int sh = 31 + l;
  const uint32_t magic = (uint32_t)((((uint64_t)1 << sh) / (uint64_t)topk) + 1);
  hipStream_t st = (hipStream_t)stream;
  int rc = launch_group_tile_offsets(group_offsets, E, kTile, tile_ws, st);
  if (rc) return rc;
  dim3 grid((unsigned)(cols / kTile), (unsigned)grid_tiles), block(256);
  const int nt = (int)(cols / kTile);
  if (x_dtype == AAMD_BF16)
    quant_dual_gather_kernel<BF16><<<grid, block, 0, st>>>((const u16*)x, ldx, nt, sorted_idx, magic, sh, (uint32_t)T, group_offsets, tile_ws, E, q, s, q_t, s_t, ld_t, q_t_layout, eps);
  else if (x_dtype == AAMD_F16)
    quant_dual_gather_kernel<F16><<<grid, block, 0, st>>>((const u16*)x, ldx, nt, sorted_idx, magic, sh, (uint32_t)T, group_offsets, tile_ws, E, q, s, q_t, s_t, ld_t, q_t_layout, eps);
  else
    quant_dual_gather_kernel<F32><<<grid, block, 0, st>>>((const float*)x, ldx, nt, sorted_idx, magic, sh, (uint32_t)T, group_offsets, tile_ws, E, q, s, q_t, s_t, ld_t, q_t_layout, eps);
  AAMD_LAUNCH_CHECK("permute_quant_dual_grouped");
  return AAMD_OK;
}

// ---------------------------------------------------------------------------------------
// SwiGLU fused into the quantisation of the intermediate activations
// ---------------------------------------------------------------------------------------
extern "C" int aamd_swiglu_quant_1x128(const void* fc1, int64_t rows, int64_t F, int64_t ld, void* h_out, uint8_t* q,
                                       float* s, void* stream) {
  AAMD_REQUIRE(rows >= 0 && F >= 0 && F % kTile == 0, "swiglu_quant: F=%lld must be a multiple of 128", (long long)F);
  AAMD_REQUIRE(ld >= 2 * F && ld % 8 == 0 && ld < kMaxRowLd, "swiglu_quant: ld=%lld must be >= 2F, a multiple of 8 and below 2^24", (long long)ld);
  if (rows == 0 || F == 0) return AAMD_OK;
  AAMD_REQUIRE(fc1 && q && s, "swiglu_quant: null pointer");
  AAMD_REQUIRE(aligned16(fc1) && aligned16(q) && aligned16(h_out), "swiglu_quant: pointers must be 16-byte aligned");
  const int nt = (int)(F / kTile);
  const int64_t total = rows * nt;
  AAMD_REQUIRE(total < (int64_t)1 << 40, "swiglu_quant: too many tiles");
  constexpr int U = kQuantU;
  const int64_t blocks = (total + 16 * U - 1) / (16 * U);
  AAMD_REQUIRE(blocks < 0x7fffffffLL, "swiglu_quant: grid too large");
  quant_1x128_kernel<GLU, false, U><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
      (const u16*)fc1, ld, nt, make_fastdiv((uint32_t)nt), total, nullptr, 1, rows, q, s, 0.f, F, (u16*)h_out);
  AAMD_LAUNCH_CHECK("swiglu_quant_1x128");
  return AAMD_OK;
}

extern "C" int aamd_swiglu_quant_1x128_dual_grouped(const void* fc1, int64_t M, int64_t F, int64_t ld,
                                                    const int64_t* group_offsets, int E, int32_t* tile_ws,
                                                    void* h_out, uint8_t* q, float* s, uint8_t* q_t, float* s_t,
                                                    int64_t ld_t, int q_t_layout, void* stream) {
  AAMD_REQUIRE(q_t_layout == AAMD_QT_ROWS || q_t_layout == AAMD_QT_BLOCKED, "swiglu_quant_dual: unknown q_t layout %d", q_t_layout);
  AAMD_REQUIRE(M >= 0 && F >= 0 && F % kTile == 0, "swiglu_quant_dual: F=%lld must be a multiple of 128", (long long)F);
  AAMD_REQUIRE(ld >= 2 * F && ld % 8 == 0 && ld < kMaxTileLd && ld_t < kMaxTileLd, "swiglu_quant_dual: bad ld=%lld", (long long)ld);
  AAMD_REQUIRE(E >= 1 && group_offsets && tile_ws, "swiglu_quant_dual: group_offsets / tile_ws required");
  AAMD_REQUIRE(ld_t % kTile == 0 && ld_t >= 0, "swiglu_quant_dual: ld_t=%lld must be a multiple of 128", (long long)ld_t);
  AAMD_REQUIRE((q == nullptr) == (s == nullptr), "swiglu_quant_dual: q and s go together");
  AAMD_REQUIRE(q_t && s_t, "swiglu_quant_dual: q_t / s_t required");
  if (F == 0) return AAMD_OK;
  const int64_t max_tiles = M / kTile + E;
  const int64_t grid_tiles = ld_t / kTile < max_tiles ? ld_t / kTile : max_tiles;
  if (grid_tiles == 0) return AAMD_OK;
  AAMD_REQUIRE(aligned16(fc1) && aligned16(q_t) && (!q || aligned16(q)) && aligned16(h_out),
               "swiglu_quant_dual: pointers must be 16-byte aligned");
  AAMD_REQUIRE(grid_tiles <= 65535, "swiglu_quant_dual: more than 65535 token tiles");
  hipStream_t st = (hipStream_t)stream;
  int rc = launch_group_tile_offsets(group_offsets, E, kTile, tile_ws, st);
  if (rc) return rc;
  dim3 grid((unsigned)(F / kTile), (unsigned)grid_tiles), block(256);
  quant_dual_grouped_kernel<GLU><<<grid, block, 0, st>>>((const u16*)fc1, ld, (int)(F / kTile), group_offsets, tile_ws, E,
                                                         q, s, q_t, s_t, ld_t, q_t_layout, 0.f, F, (u16*)h_out);
  AAMD_LAUNCH_CHECK("swiglu_quant_dual_grouped");
  return AAMD_OK;
}

// GELU fused into the quantisers: same launches with the GELU / GELU-backward loaders
extern "C" int aamd_gelu_quant_1x128(const void* x, int64_t rows, int64_t F, int64_t ld, void* h_out, uint8_t* q, float* s,
                                     void* stream) {
  AAMD_REQUIRE(rows >= 0 && F >= 0 && F % kTile == 0, "gelu_quant: F=%lld must be a multiple of 128", (long long)F);
  AAMD_REQUIRE(ld >= F && ld % 8 == 0 && ld < kMaxRowLd, "gelu_quant: ld=%lld must be >= F, a multiple of 8 and below 2^24", (long long)ld);
  if (rows == 0 || F == 0) return AAMD_OK;
  AAMD_REQUIRE(x && q && s, "gelu_quant: null pointer");
  AAMD_REQUIRE(aligned16(x) && aligned16(q) && aligned16(h_out), "gelu_quant: pointers must be 16-byte aligned");
  const int nt = (int)(F / kTile);
  const int64_t total = rows * nt;
  AAMD_REQUIRE(total < (int64_t)1 << 40, "gelu_quant: too many tiles");
  constexpr int U = kQuantU;
  const int64_t blocks = (total + 16 * U - 1) / (16 * U);
  AAMD_REQUIRE(blocks < 0x7fffffffLL, "gelu_quant: grid too large");
  quant_1x128_kernel<GELU, false, U><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
      (const u16*)x, ld, nt, make_fastdiv((uint32_t)nt), total, nullptr, 1, rows, q, s, 0.f, 0, (u16*)h_out);
  AAMD_LAUNCH_CHECK("gelu_quant_1x128");
  return AAMD_OK;
}

// dh == nullptr: forward (h = gelu(x)); else backward (g = dh * gelu'(x)), dh dense with the row stride of x
extern "C" int aamd_gelu_quant_1x128_dual_grouped(const void* x, const void* dh, int64_t M, int64_t F, int64_t ld,
                                                  const int64_t* group_offsets, int E, int32_t* tile_ws, void* h_out,
                                                  uint8_t* q, float* s, uint8_t* q_t, float* s_t, int64_t ld_t,
                                                  int q_t_layout, void* stream) {
  AAMD_REQUIRE(q_t_layout == AAMD_QT_ROWS || q_t_layout == AAMD_QT_BLOCKED, "gelu_quant_dual: unknown q_t layout %d", q_t_layout);
  AAMD_REQUIRE(M >= 0 && F >= 0 && F % kTile == 0, "gelu_quant_dual: F=%lld must be a multiple of 128", (long long)F);
  AAMD_REQUIRE(ld >= F && ld % 8 == 0 && ld < kMaxTileLd && ld_t < kMaxTileLd, "gelu_quant_dual: bad ld=%lld", (long long)ld);
  AAMD_REQUIRE(E >= 1 && group_offsets && tile_ws, "gelu_quant_dual: group_offsets / tile_ws required");
  AAMD_REQUIRE(ld_t % kTile == 0 && ld_t >= 0, "gelu_quant_dual: ld_t=%lld must be a multiple of 128", (long long)ld_t);
  AAMD_REQUIRE((q == nullptr) == (s == nullptr), "gelu_quant_dual: q and s go together");
  AAMD_REQUIRE(q_t && s_t, "gelu_quant_dual: q_t / s_t required");
  if (F == 0) return AAMD_OK;
  const int64_t max_tiles = M / kTile + E;
  const int64_t grid_tiles = ld_t / kTile < max_tiles ? ld_t / kTile : max_tiles;
  if (grid_tiles == 0) return AAMD_OK;
  AAMD_REQUIRE(x != nullptr, "gelu_quant_dual: null input");
  AAMD_REQUIRE(aligned16(x) && aligned16(dh) && aligned16(q_t) && (!q || aligned16(q)) && aligned16(h_out),
               "gelu_quant_dual: pointers must be 16-byte aligned");
  AAMD_REQUIRE(grid_tiles <= 65535, "gelu_quant_dual: more than 65535 token tiles");
  hipStream_t st = (hipStream_t)stream;
  int rc = launch_group_tile_offsets(group_offsets, E, kTile, tile_ws, st);
  if (rc) return rc;
  dim3 grid((unsigned)(F / kTile), (unsigned)grid_tiles), block(256);
  gelu_lut_kernel<<<dim3((2 * kLutN + 255) / 256), dim3(256), 0, st>>>();
  if (dh == nullptr) {
    quant_dual_grouped_kernel<GELU><<<grid, block, 0, st>>>((const u16*)x, ld, (int)(F / kTile), group_offsets, tile_ws, E, q, s,
                                                            q_t, s_t, ld_t, q_t_layout, 0.f, 0, (u16*)h_out);
  } else {
    const int64_t dh_off = (const u16*)dh - (const u16*)x;  // elements; the loader reads dh at x + dh_off
    quant_dual_grouped_kernel<GELUB><<<grid, block, 0, st>>>((const u16*)x, ld, (int)(F / kTile), group_offsets, tile_ws, E, q, s,
                                                             q_t, s_t, ld_t, q_t_layout, 0.f, dh_off, (u16*)h_out);
  }
  AAMD_LAUNCH_CHECK("gelu_quant_dual_grouped");
  return AAMD_OK;
}

extern "C" int aamd_swiglu_bwd_quant_1x128_dual_grouped(const void* dh, int64_t ld_dh, const void* fc1, int64_t ld,
                                                        int64_t M, int64_t F, const int64_t* group_offsets, int E,
                                                        int32_t* tile_ws, void* g_out, uint8_t* q, float* s,
                                                        uint8_t* q_t, float* s_t, int64_t ld_t, int q_t_layout,
                                                        void* stream) {
  AAMD_REQUIRE(q_t_layout == AAMD_QT_ROWS || q_t_layout == AAMD_QT_BLOCKED, "swiglu_bwd_quant_dual: unknown q_t layout %d", q_t_layout);
  AAMD_REQUIRE(M >= 0 && F >= 0 && F % kTile == 0, "swiglu_bwd_quant_dual: F=%lld must be a multiple of 128", (long long)F);
  AAMD_REQUIRE(ld >= 2 * F && ld % 8 == 0 && ld_dh >= F && ld_dh % 8 == 0 && ld < kMaxTileLd && ld_dh < kMaxTileLd && ld_t < kMaxTileLd,
               "swiglu_bwd_quant_dual: bad ld=%lld / ld_dh=%lld",
               (long long)ld, (long long)ld_dh);
  AAMD_REQUIRE(E >= 1 && group_offsets && tile_ws, "swiglu_bwd_quant_dual: group_offsets / tile_ws required");
  AAMD_REQUIRE(ld_t % kTile == 0 && ld_t >= 0, "swiglu_bwd_quant_dual: ld_t=%lld must be a multiple of 128", (long long)ld_t);
  AAMD_REQUIRE((q == nullptr) == (s == nullptr), "swiglu_bwd_quant_dual: q and s go together");
  AAMD_REQUIRE(q_t && s_t, "swiglu_bwd_quant_dual: q_t / s_t required");
  if (F == 0) return AAMD_OK;
  const int64_t max_tiles = M / kTile + E;
  const int64_t grid_tiles = ld_t / kTile < max_tiles ? ld_t / kTile : max_tiles;
  if (grid_tiles == 0) return AAMD_OK;
  AAMD_REQUIRE(dh && fc1, "swiglu_bwd_quant_dual: null input");
  AAMD_REQUIRE(aligned16(fc1) && aligned16(dh) && aligned16(q_t) && (!q || aligned16(q)) && aligned16(g_out),
               "swiglu_bwd_quant_dual: pointers must be 16-byte aligned");
  AAMD_REQUIRE(grid_tiles <= 65535, "swiglu_bwd_quant_dual: more than 65535 token tiles");
  hipStream_t st = (hipStream_t)stream;
  int rc = launch_group_tile_offsets(group_offsets, E, kTile, tile_ws, st);
  if (rc) return rc;
  const int nt = (int)(2 * F / kTile);
  dim3 grid((unsigned)(nt / 2), (unsigned)grid_tiles), block(512);  // two teams: the da and the db tile of a feature tile
  sigmoid_lut_kernel<<<dim3((2 * kSigN + 255) / 256), dim3(256), 0, st>>>();
  swiglu_bwd_dual_kernel<<<grid, block, 0, st>>>((const u16*)fc1, ld, F, (const u16*)dh, ld_dh, nt, group_offsets, tile_ws, E,
                                                 q, s, q_t, s_t, ld_t, q_t_layout, (u16*)g_out);
  AAMD_LAUNCH_CHECK("swiglu_bwd_quant_dual_grouped");
  return AAMD_OK;
}

extern "C" int aamd_quant_128x128(const void* w, int w_dtype, int64_t E, int64_t N, int64_t K,
                                  int64_t expert_stride, uint8_t* q, float* s, uint8_t* q_t, float* s_t, float eps,
                                  void* stream) {
  AAMD_REQUIRE(w_dtype == AAMD_BF16 || w_dtype == AAMD_F32 || w_dtype == AAMD_F16, "quant_128x128: unsupported dtype %d", w_dtype);
  AAMD_REQUIRE(E >= 0 && N >= 0 && K >= 0 && N % kTile == 0 && K % kTile == 0,
               "quant_128x128: N=%lld and K=%lld must be multiples of 128", (long long)N, (long long)K);
  AAMD_REQUIRE((q_t == nullptr) == (s_t == nullptr), "quant_128x128: q_t and s_t go together");
  AAMD_REQUIRE(N < kMaxTileLd && K < kMaxTileLd, "quant_128x128: N=%lld or K=%lld too large", (long long)N, (long long)K);
  if (E == 0 || N == 0 || K == 0) return AAMD_OK;
  AAMD_REQUIRE(w && q && s, "quant_128x128: null pointer");
  AAMD_REQUIRE(expert_stride >= N * K && expert_stride % 8 == 0, "quant_128x128: bad expert stride");
  AAMD_REQUIRE(aligned16(w) && aligned16(q) && (!q_t || aligned16(q_t)), "quant_128x128: pointers must be 16-byte aligned");
  AAMD_REQUIRE(N / kTile <= 65535 && E <= 65535, "quant_128x128: grid too large");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)(K / kTile), (unsigned)(N / kTile), (unsigned)E), block(256);
  if (w_dtype == AAMD_BF16)
    quant_128x128_kernel<BF16><<<grid, block, 0, st>>>((const u16*)w, expert_stride, N, K, q, s, q_t, s_t, eps);
  else if (w_dtype == AAMD_F16)
    quant_128x128_kernel<F16><<<grid, block, 0, st>>>((const u16*)w, expert_stride, N, K, q, s, q_t, s_t, eps);
  else
    quant_128x128_kernel<F32><<<grid, block, 0, st>>>((const float*)w, expert_stride, N, K, q, s, q_t, s_t, eps);
  AAMD_LAUNCH_CHECK("quant_128x128");
  return AAMD_OK;
}

extern "C" int aamd_dequant(const uint8_t* q, const float* s, int64_t M, int64_t N, int tile_scale, void* y,
                            int y_dtype, void* stream) {
  AAMD_REQUIRE(y_dtype == AAMD_BF16 || y_dtype == AAMD_F32, "dequant: unsupported dtype %d", y_dtype);
  AAMD_REQUIRE(M >= 0 && N >= 0 && N % kTile == 0, "dequant: N=%lld must be a multiple of 128", (long long)N);
  AAMD_REQUIRE(tile_scale || M % kTile == 0, "dequant: block scales need M %% 128 == 0");
  if (M == 0 || N == 0) return AAMD_OK;
  AAMD_REQUIRE(q && s && y && aligned16(q) && aligned16(y), "dequant: null or unaligned pointer");
  const int64_t n = M * (N / 16);
  const int64_t blocks = (n + 255) / 256;
  AAMD_REQUIRE(blocks < 0x7fffffffLL, "dequant: grid too large");
  hipStream_t st = (hipStream_t)stream;
  if (y_dtype == AAMD_F32)
    dequant_kernel<float><<<(unsigned)blocks, 256, 0, st>>>(q, s, M, N, tile_scale, (float*)y);
  else
    dequant_kernel<u16><<<(unsigned)blocks, 256, 0, st>>>(q, s, M, N, tile_scale, (u16*)y);
  AAMD_LAUNCH_CHECK("dequant");
  return AAMD_OK;
}
