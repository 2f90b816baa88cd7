// Ragged grouped block-scaled FP8 GEMM for gfx950 (forward, dgrad, wgrad and the dense case).
//
// One kernel template covers the three GEMM families.  Both operands are "K-major" byte
// matrices (rows of fp8 codes along the contraction), called L and R here:
//
//   L = the operand whose row index ends up on the MFMA column / lane axis
//       (forward+dgrad: the token rows; wgrad: the rows of dY^T),
//   R = the operand whose row index ends up on the MFMA row / register axis
//       (forward+dgrad: the weight rows of the group's expert; wgrad: the rows of X^T).
//
// Output is C[l, r] with r contiguous, so the four consecutive MFMA rows a lane owns are
// four consecutive output elements.  A workgroup of 256 threads (4 waves, 2x2) computes a
// 128 x 128 tile; each wave a 64 x 64 sub-tile as 4 x 4 v_mfma_f32_16x16x128_f8f6f4 (one MFMA
// = one full 128-deep scale block, so the raw dot product never needs a second instruction).
// The raw product is folded into the fp32 accumulator with the scales of that block:
//   acc += p * (l_scale[l, kb] * r_scale)      r_scale per 128x128 block (one scalar) or per row.
// The per-lane l_scale sits in a VGPR because the L row is the lane axis.
//
// Tiles of 128 contraction bytes are staged global -> VGPR -> LDS (double buffered, one
// barrier per step) with an XOR swizzle of the 16-byte chunks so that both the 16-byte
// stores and the MFMA operand reads are bank-conflict free.
#include <stdlib.h>

#include "common.hpp"

namespace aamd {

constexpr int kBK = 128;  // contraction bytes per step == scale block

enum GemmMode { kRaggedRows = 0, kRaggedK = 1 };

// XOR swizzle of the 16-byte chunk index inside a 128-byte LDS row.
#ifndef AAMD_SWZ_SHIFT
#define AAMD_SWZ_SHIFT 1
#endif
__device__ __forceinline__ int swz(int row) { return (row >> AAMD_SWZ_SHIFT) & 7; }

struct GemmParams {
  const uint8_t* L;
  const uint8_t* R;
  const float* Ls;
  const float* Rs;
  void* C;
  const void* bias;
  const int64_t* goff;      // [E+1] rows per group prefix (device); nullptr: one group [0, Lrows)
  const int32_t* tile_off;  // [E+1] 128-row tile prefix (device)
  int64_t ldl, ldr;                          // row strides of L and R (bytes)
  int64_t r_group_stride;                    // bytes between the R matrices of consecutive groups
  int64_t ls_row_stride, ls_blk_stride;      // L scale (row, block) strides, floats
  int64_t rs_row_stride, rs_blk_stride, rs_group_stride;
  int64_t ldc, c_group_stride;               // elements
  int64_t bias_group_stride;
  int64_t Lrows;   // kRaggedRows: total token rows; kRaggedK: rows of L (= N of dW)
  int64_t Rrows;   // rows of R per group
  int nkb;         // kRaggedRows: K / 128
  int E;
  int nRt;         // Rrows / 128
  int nLt;         // kRaggedK: Lrows / 128
  int max_kb;      // kRaggedK: contraction blocks the operand buffers hold (ld_t / 128)
  int accumulate;
  int bias_dtype;
};

__device__ __forceinline__ v4f mfma_fp8_16x16x128(const v8i& a, const v8i& b) {
  const v4f z = {0.f, 0.f, 0.f, 0.f};
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, z, 0, 0, 0, 0, 0, 0);
}

template <typename OUT>
__device__ __forceinline__ void store4(OUT* dst, const v4f& v, bool accumulate) {
  if constexpr (sizeof(OUT) == 4) {
    v4f o = v;
    if (accumulate) {
      const v4f old = *reinterpret_cast<const v4f*>(dst);
      o += old;
    }
    *reinterpret_cast<v4f*>(dst) = o;
  } else {
    v4f o = v;
    if (accumulate) {
      const v2i old = *reinterpret_cast<const v2i*>(dst);
      o[0] += bf16_bits_to_f32((uint32_t)old[0] & 0xffffu);
      o[1] += bf16_bits_to_f32((uint32_t)old[0] >> 16);
      o[2] += bf16_bits_to_f32((uint32_t)old[1] & 0xffffu);
      o[3] += bf16_bits_to_f32((uint32_t)old[1] >> 16);
    }
    v2i w;
    w[0] = (int)(f32_to_bf16_bits(o[0]) | (f32_to_bf16_bits(o[1]) << 16));
    w[1] = (int)(f32_to_bf16_bits(o[2]) | (f32_to_bf16_bits(o[3]) << 16));
    *reinterpret_cast<v2i*>(dst) = w;
  }
}

// Tile configuration: WR x WL waves, each computing (WTR*16) R rows x (WTL*16) L rows.
template <int WR_, int WL_, int WTR_, int WTL_>
struct Cfg {
  static constexpr int WR = WR_, WL = WL_, WTR = WTR_, WTL = WTL_;
  static constexpr int NT = 64 * WR * WL;   // threads
  static constexpr int BM = WL * WTL * 16;  // L rows per workgroup tile
  static constexpr int BN = WR * WTR * 16;  // R rows per workgroup tile
  static constexpr int LCH = BM * 8 / NT;   // 16-byte chunks per thread and step (L)
  static constexpr int RCH = BN * 8 / NT;
  static_assert(NT >= BM + BN, "one thread per scale value");
  static_assert((WTR * 16) % 128 == 0 || BN == 128, "a wave's R rows stay inside one 128-row scale block");
};
typedef Cfg<2, 2, 4, 4> CfgSmall;  // 256 threads, 128 x 128
typedef Cfg<2, 4, 8, 4> CfgLarge;  // 512 threads, 256 x 256

// A 64-bit offset the compiler can keep in scalar registers (it is the same in every lane).
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)(uint64_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

template <int MODE, bool R_PER_ROW, typename OUT, typename C>
__global__ __launch_bounds__(C::NT, C::NT == 256 ? 2 : 1) void grouped_gemm_kernel(const GemmParams p) {
  constexpr int BM = C::BM, BN = C::BN, NT = C::NT;
  __shared__ __attribute__((aligned(16))) uint8_t Lbuf[2][BM * kBK];
  __shared__ __attribute__((aligned(16))) uint8_t Rbuf[2][BN * kBK];
  __shared__ __attribute__((aligned(16))) float Sc[2][BM + BN];  // [buf][L rows | R rows or R blocks]
  __shared__ int slot;

  const int tid = threadIdx.x;

  // ---- which tile -------------------------------------------------------------------
  // Workgroup ids go round-robin over the 8 XCDs; give every XCD one contiguous range of
  // tile ids so that tiles sharing operand panels meet in the same L2.
  int g, lt, rt;
  {
    const int total_lt = MODE == kRaggedRows ? (p.goff ? p.tile_off[p.E] : (int)((p.Lrows + BM - 1) / BM))
                                             : p.nLt * p.E;
    const int64_t ntot = (int64_t)total_lt * p.nRt;
    const int64_t bid = blockIdx.x;
    if (bid >= ntot) return;
    const int64_t per = ntot / 8, rem = ntot % 8;
    const int64_t xcd = bid % 8, idx = bid / 8;
    const int64_t pid = xcd < rem ? xcd * (per + 1) + idx : rem * (per + 1) + (xcd - rem) * per + idx;
    // inside the range: groups of GL L tiles, R tile index outer, L tile inner
    constexpr int GL = 8;
    const int64_t width = (int64_t)GL * p.nRt;
    const int first = (int)(pid / width) * GL;
    const int gsz = total_lt - first < GL ? total_lt - first : GL;
    const int in_grp = (int)(pid % width);
    lt = first + in_grp % gsz;
    rt = in_grp / gsz;
  }

  int64_t l0;     // first L row of the tile
  int lvalid;     // valid L rows in the tile
  int kb0, nkb;   // contraction blocks [kb0, kb0 + nkb)
  if constexpr (MODE == kRaggedRows) {
    if (p.goff) {
      g = find_group(p.tile_off, p.E, lt, &slot);
      if (g >= p.E) return;
      l0 = p.goff[g] + (int64_t)(lt - p.tile_off[g]) * BM;
      const int64_t left = p.goff[g + 1] - l0;
      lvalid = left < BM ? (int)left : BM;
    } else {
      g = 0;
      l0 = (int64_t)lt * BM;
      const int64_t left = p.Lrows - l0;
      lvalid = left < BM ? (int)left : BM;
    }
    kb0 = 0;
    nkb = p.nkb;
  } else {
    g = lt / p.nLt;
    lt -= g * p.nLt;
    l0 = (int64_t)lt * BM;
    const int64_t left = p.Lrows - l0;
    lvalid = left < BM ? (int)left : BM;
    kb0 = p.tile_off[g];
    nkb = p.tile_off[g + 1] - kb0;
    if (kb0 + nkb > p.max_kb) nkb = p.max_kb > kb0 ? p.max_kb - kb0 : 0;  // never read past the buffers
  }
  g = __builtin_amdgcn_readfirstlane(g);
  const int64_t r0 = (int64_t)rt * BN;
  const int64_t rleft = p.Rrows - r0;
  const int rvalid = rleft < BN ? (int)rleft : BN;  // a multiple of 128

  // uniform tile bases + per-thread 32-bit offsets
  const uint8_t* Lbase = p.L + uniform_i64(l0 * p.ldl + (int64_t)kb0 * kBK);
  const uint8_t* Rbase = p.R + uniform_i64((int64_t)g * p.r_group_stride + r0 * p.ldr + (int64_t)kb0 * kBK);
  const float* Lsg = p.Ls + (int64_t)kb0 * p.ls_blk_stride;
  const float* Rsg = p.Rs + (int64_t)g * p.rs_group_stride + (int64_t)kb0 * p.rs_blk_stride;

  // ---- global -> register staging: LCH + RCH chunks of 16 bytes per thread -----------------
  const int ld_row = tid >> 3, ld_ch = tid & 7;
  int loff[C::LCH], roff[C::RCH], lds_loff[C::LCH], lds_roff[C::RCH];
#pragma unroll
  for (int n = 0; n < C::LCH; n++) {
    const int row = ld_row + (NT / 8) * n;
    const int lrow = row < lvalid ? row : lvalid - 1;
    loff[n] = lrow * (int)p.ldl + ld_ch * 16;
    lds_loff[n] = row * kBK + ((ld_ch ^ swz(row)) << 4);
  }
#pragma unroll
  for (int n = 0; n < C::RCH; n++) {
    const int row = ld_row + (NT / 8) * n;
    const int rrow = row < rvalid ? row : rvalid - 1;
    roff[n] = rrow * (int)p.ldr + ld_ch * 16;
    lds_roff[n] = row * kBK + ((ld_ch ^ swz(row)) << 4);
  }
  // scales: thread t < BM fetches the L scale of row t; thread BM + t the R scale of row t
  // (per-row scales) or of 128-row block t (block scales)
  const float* sptr = Lsg + l0 * p.ls_row_stride;  // threads without a scale re-read a valid one
  int64_t s_step = 0;
  if (tid < BM) {
    const int lrow = tid < lvalid ? tid : lvalid - 1;
    sptr = Lsg + (l0 + lrow) * p.ls_row_stride;
    s_step = p.ls_blk_stride;
  } else if (tid < BM + BN) {
    const int t = tid - BM;
    if (R_PER_ROW) {
      const int rrow = t < rvalid ? t : rvalid - 1;
      sptr = Rsg + (r0 + rrow) * p.rs_row_stride;
      s_step = p.rs_blk_stride;
    } else if (t < BN / kTile) {
      const int blk = t * kTile < rvalid ? t : rvalid / kTile - 1;
      sptr = Rsg + (r0 / kTile + blk) * p.rs_row_stride;
      s_step = p.rs_blk_stride;
    }
  }
  const int s_slot = tid < BM + BN ? tid : 0;  // NT == BM + BN for the shipped configurations

  v4i lreg[C::LCH], rreg[C::RCH];
  float sreg = 0.f;
  auto g_load = [&](int kb) {
    const uint8_t* lb = Lbase + (int64_t)kb * kBK;
    const uint8_t* rb = Rbase + (int64_t)kb * kBK;
#pragma unroll
    for (int n = 0; n < C::LCH; n++) lreg[n] = *reinterpret_cast<const v4i*>(lb + loff[n]);
#pragma unroll
    for (int n = 0; n < C::RCH; n++) rreg[n] = *reinterpret_cast<const v4i*>(rb + roff[n]);
    sreg = sptr[(int64_t)kb * s_step];
  };
  auto s_store = [&](int buf) {
#pragma unroll
    for (int n = 0; n < C::LCH; n++) *reinterpret_cast<v4i*>(&Lbuf[buf][lds_loff[n]]) = lreg[n];
#pragma unroll
    for (int n = 0; n < C::RCH; n++) *reinterpret_cast<v4i*>(&Rbuf[buf][lds_roff[n]]) = rreg[n];
    Sc[buf][s_slot] = sreg;
  };

  // ---- MFMA tiling ------------------------------------------------------------------------
  const int wave = tid >> 6, lane = tid & 63;
  const int wr = wave / C::WL, wl = wave % C::WL;
  const int l16 = lane & 15, lg = lane >> 4;
  const int sw = swz(l16);
  const int ch0 = ((2 * lg) ^ sw) << 4, ch1 = ((2 * lg + 1) ^ sw) << 4;
  const int wrow0 = wr * C::WTR * 16;            // first R row of this wave inside the tile
  const int wlrow0 = wl * C::WTL * 16;           // first L row of this wave inside the tile
  const bool wave_active = wrow0 < rvalid;        // whole wave in or out: rvalid % 128 == 0

  v4f acc[C::WTR][C::WTL];
#pragma unroll
  for (int i = 0; i < C::WTR; i++)
#pragma unroll
    for (int j = 0; j < C::WTL; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  if (nkb > 0) {
    g_load(0);
    s_store(0);
  }
  __syncthreads();

  // Software pipeline inside the wave, pinned with scheduling barriers: the MFMA of sub-tile t
  // is issued, then the four scale-and-accumulate FMAs of sub-tile t-1 run in its shadow (the
  // waves of a workgroup move in lock step between barriers, so MFMA and VALU work must
  // overlap inside one wave, not across waves).  The loop body is branch free: the prefetch of
  // the last step re-reads the last block, and waves outside a partial R tile compute on
  // clamped rows and skip only the final store.
  for (int kb = 0; kb < nkb; kb++) {
    const int cur = kb & 1;
    g_load(kb + 1 < nkb ? kb + 1 : kb);

    const uint8_t* Lt = Lbuf[cur];
    const uint8_t* Rt = Rbuf[cur];
    const float* Lsc = &Sc[cur][0];
    const float* Rsc = &Sc[cur][BM];
    v8i lf[C::WTL];
    float cs[C::WTL];
    const float rblk = R_PER_ROW ? 1.f : Rsc[wrow0 / kTile];
#pragma unroll
    for (int j = 0; j < C::WTL; j++) {
      const int row = wlrow0 + j * 16 + l16;
      const v4i lo = *reinterpret_cast<const v4i*>(Lt + row * kBK + ch0);
      const v4i hi = *reinterpret_cast<const v4i*>(Lt + row * kBK + ch1);
      lf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      cs[j] = Lsc[row] * rblk;
    }
    auto load_rf = [&](int i) {
      const int row = wrow0 + i * 16 + l16;
      const v4i lo = *reinterpret_cast<const v4i*>(Rt + row * kBK + ch0);
      const v4i hi = *reinterpret_cast<const v4i*>(Rt + row * kBK + ch1);
      return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    auto load_rs = [&](int i) {
      v4f r = {1.f, 1.f, 1.f, 1.f};
      if constexpr (R_PER_ROW) r = *reinterpret_cast<const v4f*>(&Rsc[wrow0 + i * 16 + 4 * lg]);
      return r;
    };
    v8i rf[2];
    v4f rs4[2];
    rf[0] = load_rf(0);
    rs4[0] = load_rs(0);
    v4f pprev = {0.f, 0.f, 0.f, 0.f};
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < C::WTR; i++) {
#pragma unroll
      for (int j = 0; j < C::WTL; j++) {
        const v4f pcur = mfma_fp8_16x16x128(rf[i & 1], lf[j]);
        if (i > 0 || j > 0) {
          const int pi = j > 0 ? i : i - 1, pj = j > 0 ? j - 1 : C::WTL - 1;
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const float sc = R_PER_ROW ? cs[pj] * rs4[pi & 1][r] : cs[pj];
            acc[pi][pj][r] = __builtin_fmaf(pprev[r], sc, acc[pi][pj][r]);
          }
        }
        pprev = pcur;
        // the fragments of the next R row tile are fetched once the last FMA that needed the
        // previous row tile's scales has been placed
        if (j == 0 && i + 1 < C::WTR) {
          rf[(i + 1) & 1] = load_rf(i + 1);
          rs4[(i + 1) & 1] = load_rs(i + 1);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const float sc = R_PER_ROW ? cs[C::WTL - 1] * rs4[(C::WTR - 1) & 1][r] : cs[C::WTL - 1];
      acc[C::WTR - 1][C::WTL - 1][r] = __builtin_fmaf(pprev[r], sc, acc[C::WTR - 1][C::WTL - 1][r]);
    }

    s_store(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue ------------------------------------------------------------------------------
  if (MODE == kRaggedK && nkb == 0 && p.accumulate) return;  // empty group: leave dW untouched
  if (!wave_active) return;
  OUT* Cg = reinterpret_cast<OUT*>(p.C) + (int64_t)g * p.c_group_stride;
#pragma unroll
  for (int i = 0; i < C::WTR; i++) {
    const int64_t rcol = r0 + wrow0 + i * 16 + 4 * lg;
    v4f b4 = {0.f, 0.f, 0.f, 0.f};
    if (MODE == kRaggedRows && p.bias != nullptr) {
      if (p.bias_dtype == AAMD_F32) {
        b4 = *reinterpret_cast<const v4f*>(reinterpret_cast<const float*>(p.bias) + g * p.bias_group_stride + rcol);
      } else {
        const v2i raw = *reinterpret_cast<const v2i*>(reinterpret_cast<const u16*>(p.bias) + g * p.bias_group_stride + rcol);
        b4[0] = bf16_bits_to_f32((uint32_t)raw[0] & 0xffffu);
        b4[1] = bf16_bits_to_f32((uint32_t)raw[0] >> 16);
        b4[2] = bf16_bits_to_f32((uint32_t)raw[1] & 0xffffu);
        b4[3] = bf16_bits_to_f32((uint32_t)raw[1] >> 16);
      }
    }
#pragma unroll
    for (int j = 0; j < C::WTL; j++) {
      const int lrow = wlrow0 + j * 16 + l16;
      if (lrow < lvalid) store4<OUT>(Cg + (l0 + lrow) * p.ldc + rcol, acc[i][j] + b4, p.accumulate != 0);
    }
  }
}

int launch_group_tile_offsets(const int64_t* goff, int E, int tile, int32_t* tile_off, hipStream_t st);

template <int MODE, bool R_PER_ROW, typename C>
static int launch_gemm(const GemmParams& p, int c_dtype, int64_t blocks, hipStream_t st) {
  if (blocks <= 0) return AAMD_OK;
  AAMD_REQUIRE(blocks < 0x7fffffffLL, "grouped_gemm: grid too large");
  dim3 grid((unsigned)blocks), block(C::NT);
  if (c_dtype == AAMD_BF16)
    grouped_gemm_kernel<MODE, R_PER_ROW, u16, C><<<grid, block, 0, st>>>(p);
  else
    grouped_gemm_kernel<MODE, R_PER_ROW, float, C><<<grid, block, 0, st>>>(p);
  AAMD_LAUNCH_CHECK("grouped_gemm");
  return AAMD_OK;
}

// Large tiles whenever the problem has enough of them to fill the chip; AAMD_GEMM_TILE=small|large overrides.
static bool use_large_tiles(int64_t l_rows, int64_t r_rows, int64_t groups) {
  const char* env = getenv("AAMD_GEMM_TILE");
  if (env && env[0] == 's') return false;
  if (env && env[0] == 'l') return true;
  const int64_t tiles = ((l_rows + 255) / 256) * ((r_rows + 255) / 256) * groups;
  return tiles >= 512;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace aamd

using namespace aamd;

extern "C" int aamd_grouped_gemm_fp8_nt(const uint8_t* a, int64_t lda, const float* a_s, const uint8_t* b,
                                        const float* b_s, int b_tile_scaled, const int64_t* group_offsets, int E,
                                        int32_t* tile_ws, int64_t M, int64_t N, int64_t K, void* c, int c_dtype,
                                        int64_t ldc, const void* bias, int bias_dtype, void* stream) {
  AAMD_REQUIRE(c_dtype == AAMD_BF16 || c_dtype == AAMD_F32, "grouped_gemm_nt: unsupported output dtype %d", c_dtype);
  AAMD_REQUIRE(M >= 0 && N >= 0 && K >= 0, "grouped_gemm_nt: negative size");
  AAMD_REQUIRE(K % kBK == 0 && N % kTile == 0, "grouped_gemm_nt: K=%lld and N=%lld must be multiples of 128",
               (long long)K, (long long)N);
  AAMD_REQUIRE(E >= 1, "grouped_gemm_nt: E must be >= 1");
  AAMD_REQUIRE(group_offsets != nullptr || E == 1, "grouped_gemm_nt: group_offsets required when E > 1");
  AAMD_REQUIRE(group_offsets == nullptr || tile_ws != nullptr, "grouped_gemm_nt: tile_ws required");
  AAMD_REQUIRE(bias == nullptr || bias_dtype == AAMD_BF16 || bias_dtype == AAMD_F32, "grouped_gemm_nt: bad bias dtype");
  if (M == 0 || N == 0) return AAMD_OK;
  AAMD_REQUIRE(a && a_s && b && b_s && c, "grouped_gemm_nt: null pointer");
  AAMD_REQUIRE(lda >= K && lda % 16 == 0 && aligned16(a) && aligned16(b), "grouped_gemm_nt: operands must be 16-byte aligned");
  AAMD_REQUIRE(ldc >= N && ldc % 4 == 0 && aligned16(c), "grouped_gemm_nt: output must be 16-byte aligned");
  AAMD_REQUIRE(K > 0, "grouped_gemm_nt: K must be positive");
  hipStream_t st = (hipStream_t)stream;
  const bool large = use_large_tiles(M, N, 1);
  const int BM = large ? CfgLarge::BM : CfgSmall::BM, BN = large ? CfgLarge::BN : CfgSmall::BN;
  if (group_offsets) {
    int rc = launch_group_tile_offsets(group_offsets, E, BM, tile_ws, st);
    if (rc) return rc;
  }
  GemmParams p = {};
  p.L = a; p.ldl = lda; p.Ls = a_s; p.ls_row_stride = K / kBK; p.ls_blk_stride = 1;
  p.R = b; p.ldr = K; p.r_group_stride = N * K;
  p.Rs = b_s;
  p.rs_row_stride = K / kBK; p.rs_blk_stride = 1;
  p.rs_group_stride = b_tile_scaled ? N * (K / kBK) : (N / kTile) * (K / kBK);
  p.C = c; p.ldc = ldc; p.c_group_stride = 0;
  p.bias = bias; p.bias_dtype = bias_dtype; p.bias_group_stride = N;
  p.goff = group_offsets; p.tile_off = tile_ws;
  p.Lrows = M; p.Rrows = N; p.nkb = (int)(K / kBK); p.E = E; p.nRt = (int)((N + BN - 1) / BN); p.nLt = 0;
  p.accumulate = 0;
  const int64_t max_lt = group_offsets ? M / BM + E : (M + BM - 1) / BM;
  const int64_t blocks = max_lt * p.nRt;
  if (large)
    return b_tile_scaled ? launch_gemm<kRaggedRows, true, CfgLarge>(p, c_dtype, blocks, st)
                         : launch_gemm<kRaggedRows, false, CfgLarge>(p, c_dtype, blocks, st);
  return b_tile_scaled ? launch_gemm<kRaggedRows, true, CfgSmall>(p, c_dtype, blocks, st)
                       : launch_gemm<kRaggedRows, false, CfgSmall>(p, c_dtype, blocks, st);
}

extern "C" int aamd_grouped_gemm_fp8_wgrad(const uint8_t* dyt, const float* sdyt, const uint8_t* xt,
                                           const float* sxt, int64_t ld_t, const int64_t* group_offsets, int E,
                                           int32_t* tile_ws, int64_t N, int64_t K, void* dw, int dw_dtype,
                                           int64_t expert_stride, int accumulate, void* stream) {
  AAMD_REQUIRE(dw_dtype == AAMD_BF16 || dw_dtype == AAMD_F32, "grouped_gemm_wgrad: unsupported output dtype %d", dw_dtype);
  AAMD_REQUIRE(N >= 0 && K >= 0 && N % kTile == 0 && K % kTile == 0,
               "grouped_gemm_wgrad: N=%lld and K=%lld must be multiples of 128", (long long)N, (long long)K);
  AAMD_REQUIRE(E >= 1 && group_offsets && tile_ws, "grouped_gemm_wgrad: group_offsets / tile_ws required");
  AAMD_REQUIRE(ld_t >= 0 && ld_t % kBK == 0, "grouped_gemm_wgrad: ld_t=%lld must be a multiple of 128", (long long)ld_t);
  if (N == 0 || K == 0) return AAMD_OK;
  AAMD_REQUIRE(dw && (ld_t == 0 || (dyt && sdyt && xt && sxt)), "grouped_gemm_wgrad: null pointer");
  AAMD_REQUIRE(aligned16(dyt) && aligned16(xt) && aligned16(dw), "grouped_gemm_wgrad: pointers must be 16-byte aligned");
  AAMD_REQUIRE(expert_stride >= N * K && expert_stride % 4 == 0, "grouped_gemm_wgrad: bad expert stride");
  hipStream_t st = (hipStream_t)stream;
  int rc = launch_group_tile_offsets(group_offsets, E, kBK, tile_ws, st);
  if (rc) return rc;
  GemmParams p = {};
  p.L = dyt; p.ldl = ld_t; p.Ls = sdyt; p.ls_row_stride = 1; p.ls_blk_stride = N;
  p.R = xt; p.ldr = ld_t; p.r_group_stride = 0;
  p.Rs = sxt; p.rs_row_stride = 1; p.rs_blk_stride = K; p.rs_group_stride = 0;
  p.C = dw; p.ldc = K; p.c_group_stride = expert_stride;
  p.bias = nullptr; p.bias_dtype = AAMD_NONE; p.bias_group_stride = 0;
  p.goff = group_offsets; p.tile_off = tile_ws;
  const bool large = use_large_tiles(N, K, E);
  const int BM = large ? CfgLarge::BM : CfgSmall::BM, BN = large ? CfgLarge::BN : CfgSmall::BN;
  p.Lrows = N; p.Rrows = K; p.nkb = 0; p.E = E; p.nRt = (int)((K + BN - 1) / BN); p.nLt = (int)((N + BM - 1) / BM);
  p.max_kb = (int)(ld_t / kBK);
  p.accumulate = accumulate;
  const int64_t blocks = (int64_t)E * p.nLt * p.nRt;
  return large ? launch_gemm<kRaggedK, true, CfgLarge>(p, dw_dtype, blocks, st)
               : launch_gemm<kRaggedK, true, CfgSmall>(p, dw_dtype, blocks, st);
}
