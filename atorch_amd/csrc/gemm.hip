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
// Output is C[l, r] with r contiguous, so the four consecutive MFMA rows a lane owns are four
// consecutive output elements.  The contraction advances in steps of 128 bytes = one scale
// block.  Per step and 32x32 sub-tile two chained v_mfma_f32_32x32x64_f8f6f4 give the raw
// 128-deep dot products, which are folded into the fp32 accumulator with the step's scales:
//   acc += p * (l_scale[l, kb] * r_scale)      r_scale per 128x128 block (one scalar) or per row.
// The per-lane l_scale sits in one VGPR because the L row is the lane axis.
//
// Why this shape of MFMA: measured on MI355X, VALU instructions co-execute with the 16-pass
// 32x32x64 MFMA (8 FMAs per MFMA cost ~4 %), but not with the 8-pass 16x16x128 one (there every
// FMA adds its full 4 cycles).  The fold needs 8 FMAs per MFMA, so only the former keeps the
// matrix pipe busy.
//
// Data path: global -> LDS directly (global_load_lds, 16 bytes per lane, no register stop),
// two stages, one workgroup barrier per step (two in the 256x256 configuration, whose L tile is
// requested two steps ahead).  Rows are 128 bytes; the 16-byte chunks of a row
// are XOR-swizzled so that the linear 1 KB writes of the direct loads and the 32-row MFMA
// operand reads are both bank-conflict free on the 64-bank LDS (measured: ~235 of 256 B/clk).
#include <stdlib.h>
#include <string.h>

#include <atomic>

#include "common.hpp"
#ifdef AAMD_TUNING
#include "../../include/atorch_amd_probes.h"
#endif

namespace aamd {

constexpr int kBK = 128;  // contraction bytes per step == scale block

enum GemmMode { kRaggedRows = 0, kRaggedK = 1 };

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef float v16f __attribute__((ext_vector_type(16)));

// XOR swizzle of the 16-byte chunk index inside a 128-byte LDS row (depends on row % 16 only).
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

struct GemmParams {
  const uint8_t* L;
  const uint8_t* R;
  const float* Ls;
  const float* Rs;
  void* C;
  const void* bias;
  const int64_t* goff;      // [E+1] rows per group prefix (device); nullptr: one group [0, Lrows)
  const int32_t* tile_off;  // [E+1] tile prefix (device)
  int64_t ldl, ldr;                          // row strides of L and R (bytes)
  int64_t l_kb_stride, r_kb_stride;          // bytes between consecutive 128-wide contraction blocks of a row
  int64_t r_group_stride;                    // bytes between the R matrices of consecutive groups
  int64_t ls_row_stride, ls_blk_stride;      // L scale (row, block) strides, floats
  int64_t rs_row_stride, rs_blk_stride, rs_group_stride;
  int64_t ldc, c_group_stride;               // elements
  int64_t bias_group_stride;
  int64_t Lrows;   // kRaggedRows: total token rows; kRaggedK: rows of L (= N of dW)
  int64_t Rrows;   // rows of R per group
  int nkb;         // kRaggedRows: K / 128
  int E;
  int nRt;         // R tiles
  int nLt;         // kRaggedK: L tiles
  int max_kb;      // kRaggedK: contraction blocks the operand buffers hold (ld_t / 128)
  int accumulate;
  int group_r;     // the tile order groups R tiles (inside each group of rows / expert) instead of L tiles
  int bias_dtype;
  int gl;          // L tiles that share an R panel in the tile order
  int ls_batch;    // kRaggedRows: L scales are fetched eight contraction blocks at a time
};

__device__ __forceinline__ v16f mfma_fp8_32x32x64(const v8i& a, const v8i& b, const v16f& c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

template <typename OUT>
__device__ __forceinline__ void store4(OUT* dst, v4f o, bool accumulate) {
  if constexpr (sizeof(OUT) == 4) {
    if (accumulate) o += *reinterpret_cast<const v4f*>(dst);
    *reinterpret_cast<v4f*>(dst) = o;
  } else {
    if (accumulate) {
      const v2i old = *reinterpret_cast<const v2i*>(dst);
      o[0] += bf16_bits_to_f32((uint32_t)old[0] & 0xffffu);
      o[1] += bf16_bits_to_f32((uint32_t)old[0] >> 16);
      o[2] += bf16_bits_to_f32((uint32_t)old[1] & 0xffffu);
      o[3] += bf16_bits_to_f32((uint32_t)old[1] >> 16);
    }
    v2i w;
    w[0] = (int)pack_bf16x2(o[0], o[1]);
    w[1] = (int)pack_bf16x2(o[2], o[3]);
    *reinterpret_cast<v2i*>(dst) = w;
  }
}

// Tile configuration: WR x WL waves, each computing (WTR*32) R rows x (WTL*32) L rows.
template <int WR_, int WL_, int WTR_, int WTL_, int PRB_ = 2, bool LAHEAD_ = false>
struct Cfg {
  static constexpr bool LAHEAD = LAHEAD_;  // load the L tile two steps ahead (extra barrier per step)
  static constexpr int WR = WR_, WL = WL_, WTR = WTR_, WTL = WTL_;
  static constexpr int PRB = PRB_;  // raw-product buffers: 2 folds a sub-tile under the next one's MFMAs
  static constexpr int NT = 64 * WR * WL;   // threads
  static constexpr int BM = WL * WTL * 32;  // L rows per workgroup tile
  static constexpr int BN = WR * WTR * 32;  // R rows per workgroup tile
  static constexpr int LCH = BM * 8 / NT;   // 16-byte chunks per thread and step (L)
  static constexpr int RCH = BN * 8 / NT;
  static_assert(NT >= BM + BN, "one thread per scale value");
  static_assert(BM % 64 == 0 && BN % 128 == 0, "whole waves per scale side; R tiles cover whole scale blocks");
  static_assert((WTR * 32) % 128 == 0 || BN == 128, "a wave's R rows stay inside one 128-row scale block");
  static_assert(LCH * NT == BM * 8 && RCH * NT == BN * 8, "tile rows divide evenly over the threads");
  static_assert((NT / 8) % 16 == 0, "the swizzle of a slab depends on the wave only");
};
typedef Cfg<2, 2, 2, 2, 3> CfgSmall;  // 256 threads, 128 (L) x 128 (R), two workgroups per CU
typedef Cfg<2, 4, 4, 2, 1, true> CfgLarge;  // 512 threads, 256 (L) x 256 (R); one product buffer: 256 registers per lane
typedef Cfg<2, 4, 2, 2> CfgWgrad;  // 512 threads, 256 (L) x 128 (R): room for the per-row R scales

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant
// expression inside the body.
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// A 64-bit offset the compiler can keep in scalar registers (it is the same in every lane).
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)(uint64_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

template <int MODE, bool R_PER_ROW, typename OUT, typename C>
__global__ __launch_bounds__(C::NT, C::NT == 256 ? 2 : 1) void grouped_gemm_kernel(const GemmParams p) {
  constexpr int BM = C::BM, BN = C::BN, NT = C::NT;
  // LDS: two stages of an L tile and an R tile of 128-byte rows, then the two stages' scales
  // ([L rows | R rows or R blocks | unused], NT floats each).  After the contraction loop the same
  // memory stages the output tile for the row-contiguous stores of the epilogue.
  constexpr int kStage = (BM + BN) * kBK;
  constexpr int kStgBytes = 64 * 144;  // per-wave epilogue staging: 64 rows x (128 + 16) bytes
  static_assert(2 * kStage >= (NT / 64) * kStgBytes, "the epilogue staging fits in the stage buffers");
  // kRaggedRows keeps two batches of L scales besides: [BM rows][8 contraction blocks] floats each.
  constexpr int kLsBatch = MODE == kRaggedRows ? BM * 8 * 4 : 0;
  static_assert(NT == 2 * BM, "two threads fetch the 32 bytes of a row's scale batch");
  __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kStage + 2 * NT * 4 + 2 * kLsBatch];
  // both L stages first, then both R stages: every fragment of a side is within 64 KB of one base
  // address, so the stage and the sub-tile row go into the immediate offset of the LDS reads
  uint8_t* const Lbuf0 = lds;
  uint8_t* const Lbuf1 = lds + BM * kBK;
  uint8_t* const Rbuf0 = lds + 2 * BM * kBK;
  uint8_t* const Rbuf1 = lds + 2 * BM * kBK + BN * kBK;
  static_assert(2 * BM * kBK <= 65536 && 2 * BN * kBK <= 65536, "immediate LDS offsets are 16 bits");
  float* const Sc0 = reinterpret_cast<float*>(lds + 2 * kStage);
  float* const Sc1 = Sc0 + NT;
  float* const LsB0 = Sc1 + NT;  // scale batches (kRaggedRows)

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, lives in an SGPR
  const int lane = tid & 63;

  // ---- which tile -------------------------------------------------------------------------
  // One tile per workgroup (a loop over tiles inside the kernel costs registers and the
  // hardware's own dispatch balances ragged tiles better).  Workgroup ids go round-robin over
  // the 8 XCDs; every XCD gets one contiguous range of tile ids so that tiles sharing operand
  // panels meet in the same L2.
  // Row-ragged launches look their group up in the device-side offsets.  Every wave does it on its
  // own, without LDS or barriers: lane e fetches the tile range and the row range of group e (all
  // loads go out before the first wait: one trip to memory instead of three dependent ones, tile
  // count -> tile index -> matching group -> its row offsets), the lane whose group holds the tile
  // is found with a ballot and its values are broadcast with readlane.
  int total_lt;
  int t_lo = 0, t_hi = 0;
  int64_t r_lo = 0, r_hi = 0;
  if (MODE == kRaggedRows && p.goff != nullptr) {
    if (lane < p.E) {
      t_lo = p.tile_off[lane];
      t_hi = p.tile_off[lane + 1];
      r_lo = p.goff[lane];
      r_hi = p.goff[lane + 1];
    }
    total_lt = p.tile_off[p.E];
  } else {
    total_lt = MODE == kRaggedRows ? (int)((p.Lrows + BM - 1) / BM) : p.nLt * p.E;
  }
  const int64_t ntot = (int64_t)total_lt * p.nRt;
  const int64_t bid = blockIdx.x;
  if (bid >= ntot) return;
  int g, lt, rt;
  const int64_t per = ntot / 8, rem = ntot % 8;
  const int64_t xcd = bid % 8, idx = bid / 8;
  const int64_t pid = xcd < rem ? xcd * (per + 1) + idx : rem * (per + 1) + (xcd - rem) * per + idx;
  const int GL = p.gl;
  const bool by_group = MODE == kRaggedRows && p.goff != nullptr && p.group_r;  // tile order per group, below
  {
    // inside the range: groups of GL L tiles, R tile index outer, L tile inner
    if (MODE == kRaggedK && p.group_r) {
      // wgrad with more R tiles than L tiles: groups of GL R tiles, all L tiles of the expert inside
      const int64_t per_e = (int64_t)p.nLt * p.nRt;
      const int e = (int)(pid / per_e);
      const int64_t pe = pid - e * per_e;
      const int64_t width = (int64_t)GL * p.nLt;
      const int first = (int)(pe / width) * GL;
      const int gsz = p.nRt - first < GL ? p.nRt - first : GL;
      const int in_grp = (int)(pe % width);
      rt = first + in_grp % gsz;
      lt = e * p.nLt + in_grp / gsz;
    } else {
      const int64_t width = (int64_t)GL * p.nRt;
      const int first = (int)(pid / width) * GL;
      const int gsz = total_lt - first < GL ? total_lt - first : GL;
      const int in_grp = (int)(pid % width);
      lt = first + in_grp % gsz;
      rt = in_grp / gsz;
    }
  }

  int64_t l0;     // first L row of the tile
  int lvalid;     // valid L rows in the tile
  int kb0, nkb;   // contraction blocks [kb0, kb0 + nkb)
  bool short_operands = false;
  if constexpr (MODE == kRaggedRows) {
    if (p.goff) {
      // exactly one group holds tile lt (empty groups hold none)
      // With group_r the tile ids of a group are contiguous and ordered in batches of GL R tiles,
      // all L tiles of the group inside a batch, R index fastest: the weights of the group, the
      // large operand, are then fetched once, and the group's few L panels are what gets re-read.
      g = p.E;
      l0 = 0;
      lvalid = 0;
      for (int base = 0; base < p.E; base += 64) {
        if (base > 0) {  // more than 64 groups: the next 64
          const int e = base + lane;
          t_lo = t_hi = 0;
          if (e < p.E) {
            t_lo = p.tile_off[e];
            t_hi = p.tile_off[e + 1];
            r_lo = p.goff[e];
            r_hi = p.goff[e + 1];
          }
        }
        int my_lt = lt, my_rt = 0;
        bool mine = lt >= t_lo && lt < t_hi;  // empty groups (and lanes past E) hold no tile
        if (by_group) {
          const int64_t p_lo = (int64_t)t_lo * p.nRt, p_hi = (int64_t)t_hi * p.nRt;
          mine = pid >= p_lo && pid < p_hi;
          const int nl = mine ? t_hi - t_lo : 1;
          const int64_t pe = pid - p_lo, width = (int64_t)GL * nl;
          const int first_r = (int)(pe / width) * GL;
          const int gsz = p.nRt - first_r < GL ? p.nRt - first_r : GL;
          const int in_grp = (int)(pe % width);
          my_rt = first_r + in_grp % (gsz > 0 ? gsz : 1);
          my_lt = t_lo + in_grp / (gsz > 0 ? gsz : 1);
        }
        const unsigned long long hit = __ballot(mine);
        if (hit != 0) {  // exactly one group holds the tile
          const int src = __builtin_ctzll(hit);
          const int64_t first = r_lo + (int64_t)(my_lt - t_lo) * BM, left = r_hi - first;
          const int lv = left < BM ? (int)left : BM;
          g = base + src;
          l0 = (int64_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)((uint64_t)first >> 32), src) << 32) |
                         (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(uint64_t)first, src));
          lvalid = __builtin_amdgcn_readlane(lv, src);
          if (by_group) rt = __builtin_amdgcn_readlane(my_rt, src);
          break;
        }
      }
      if (g >= p.E) return;
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
    // Operand buffers too short for the padded token count (ld_t below the device-side total): never
    // read past them, and make the failure visible: the group's gradient tile is written as NaN.
    if (kb0 + nkb > p.max_kb) {
      nkb = 0;
      short_operands = true;
    }
  }
  g = __builtin_amdgcn_readfirstlane(g);
  const int64_t r0 = (int64_t)rt * BN;
  const int64_t rleft = p.Rrows - r0;
  const int rvalid = rleft < BN ? (int)rleft : BN;  // a multiple of 128

  // uniform tile bases + per-thread 32-bit offsets
  const uint8_t* Lbase = p.L + uniform_i64(l0 * p.ldl + (int64_t)kb0 * p.l_kb_stride);
  const uint8_t* Rbase = p.R + uniform_i64((int64_t)g * p.r_group_stride + r0 * p.ldr + (int64_t)kb0 * p.r_kb_stride);
  const float* Lsg = p.Ls + (int64_t)kb0 * p.ls_blk_stride;
  const float* Rsg = p.Rs + (int64_t)g * p.rs_group_stride + (int64_t)kb0 * p.rs_blk_stride;

  // ---- global -> LDS without a register stop ---------------------------------------------------
  // One wave instruction of the direct load writes 1 KB of LDS, lane l at base + 16 l: eight
  // tile rows of 128 bytes.  Lane l owns LDS position (row l/8, chunk l%8) and fetches the
  // global chunk the swizzle assigns to that position.
  // A wave instruction n covers the 8-row slab starting at tile row wave*8 + (NT/8)*n.  The lane
  // part of the address (row inside the slab, swizzled chunk) is the same for every slab of a
  // wave: (row & 7) is lane/8 and ((row >> 3) & 1) is wave & 1 because NT/8 is a multiple of 16.
  // The slab part is wave-uniform and lives in scalar registers.  Rows past the valid part of a
  // tile are never stored, so they may read whatever follows them in the operand; only the end
  // of the operand itself must not be crossed: slabs beyond the last readable row are moved onto
  // the last slab that holds one, and that slab clamps its rows per lane.
  const int r8 = lane >> 3;
  const uint32_t chunk = (uint32_t)(((lane & 7) ^ r8 ^ (wave & 1)) << 4);
  const int64_t l_rows_left = p.Lrows - l0;
  const int availL = l_rows_left < BM ? (int)l_rows_left : BM;  // >= 1
  const int bmaxL = ((availL - 1) >> 3) << 3, tailL = availL - bmaxL;
  const uint32_t voffL = (uint32_t)r8 * (uint32_t)p.ldl + chunk;
  const uint32_t voffLt = (uint32_t)(r8 < tailL ? r8 : tailL - 1) * (uint32_t)p.ldl + chunk;
  const uint32_t voffR = (uint32_t)r8 * (uint32_t)p.ldr + chunk;  // rvalid is a multiple of 128: whole slabs
  uint32_t lslab[C::LCH], rslab[C::RCH];  // scalar byte offsets of the slabs
  bool ltail[C::LCH];
#pragma unroll
  for (int n = 0; n < C::LCH; n++) {
    const int b = wave * 8 + (NT / 8) * n;
    ltail[n] = b >= bmaxL;
    lslab[n] = __builtin_amdgcn_readfirstlane((uint32_t)(ltail[n] ? bmaxL : b) * (uint32_t)p.ldl);
  }
#pragma unroll
  for (int n = 0; n < C::RCH; n++) {
    const int b = wave * 8 + (NT / 8) * n;
    rslab[n] = __builtin_amdgcn_readfirstlane((uint32_t)(b < rvalid ? b : rvalid - 8) * (uint32_t)p.ldr);
  }
  // scales: thread t < BM fetches the L scale of row t; thread BM + t the R scale of row t
  // (per-row scales) or of 128-row block t (block scales); the rest re-read a valid value.
  // Whole waves are on one side (BM is a multiple of 64), so base and step are wave-uniform.
  const bool l_side = wave < BM / 64;
  const float* sbase = l_side ? Lsg + l0 * p.ls_row_stride : Rsg + (R_PER_ROW ? r0 : r0 / kTile) * p.rs_row_stride;
  const int64_t s_step = l_side ? p.ls_blk_stride : p.rs_blk_stride;
  uint32_t soff;  // element offset of this thread's scale from sbase
  if (l_side) {
    const int lrow = tid < lvalid ? tid : lvalid - 1;
    soff = (uint32_t)lrow * (uint32_t)p.ls_row_stride;
  } else {
    const int t = tid - BM;
    const int nvalid = R_PER_ROW ? rvalid : rvalid / kTile;
    const int rr = t < nvalid ? t : nvalid - 1;
    soff = (uint32_t)rr * (uint32_t)p.rs_row_stride;
  }

  // All loads of the contraction loop are issued from inline assembly, with the wait counts kept
  // by hand: the compiler's own bookkeeping of direct-to-LDS loads is conservative (it tracks
  // eight of them individually and otherwise waits for every outstanding load).  Per step and
  // thread: LCH + RCH 16-byte tile loads and the scale loads; all of them write LDS only,
  // so no VGPR is ever written behind the compiler's back.
  auto lds_addr = [](const void* q) { return (uint32_t)(uintptr_t)(lds_ptr_t)q; };
  const uint32_t soff_b = soff * 4u;
  // L scales of a row-major [rows, K/128] operand: one 4-byte value per row and step would touch
  // as many cache lines as the tile itself.  Instead 32 bytes per row (eight contraction blocks)
  // are fetched every eighth step, 16 bytes per thread, into [row][8] floats.  The last batch is
  // shifted back so that it ends at the last block.
  const bool batch = MODE == kRaggedRows && p.ls_batch != 0;  // uniform; implies nkb >= 8
  // this wave loads a scale every step (never in the configuration that takes all its scales in batches)
  const bool step_scale = !C::LAHEAD && !(batch && l_side);
  const int brow = (tid >> 1) < lvalid ? (tid >> 1) : lvalid - 1;
  const uint32_t boff = ((uint32_t)brow * (uint32_t)p.ls_row_stride + (uint32_t)(tid & 1) * 4u) * 4u;
  auto batch_start = [&](int b) { return 8 * b + 8 <= nkb ? 8 * b : nkb - 8; };
  auto dma_scale_batch = [&](int b) {
    if constexpr (MODE == kRaggedRows) {
      const uint8_t* sb = reinterpret_cast<const uint8_t*>(Lsg + uniform_i64(l0 * p.ls_row_stride + batch_start(b)));
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   ::"v"(boff), "s"(sb), "s"(lds_addr(LsB0 + (b & 1) * (BM * 8)) + (uint32_t)(wave * 1024))
                   : "memory");
    }
  };
  auto dma_scale = [&](int kb, float* Sd) {
    const uint8_t* sb = reinterpret_cast<const uint8_t*>(sbase + (int64_t)kb * s_step);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                   ::"v"(soff_b), "s"(sb), "s"(lds_addr(Sd) + (uint32_t)(wave * 256))
                   : "memory");
  };
  // One wave instruction of the L (R) tile of a step; the last one of a half also carries that
  // half's scale loads.  L half: the L tile and, from the waves that own them, the L scales.
  auto dmaL_tile = [&](int n, int kb, uint8_t* Ld) {
    const uint8_t* lb = Lbase + (int64_t)kb * p.l_kb_stride;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 ::"v"(ltail[n] ? voffLt : voffL), "s"(lb + lslab[n]),
                   "s"(lds_addr(Ld) + (uint32_t)((wave * 8 + (NT / 8) * n) * kBK))
                 : "memory");
  };
  auto dmaL_scales = [&](int kb, float* Sd) {
    if (l_side && step_scale) dma_scale(kb, Sd);
  };
  auto dmaR_tile = [&](int n, int kb, uint8_t* Rd) {
    const uint8_t* rb = Rbase + (int64_t)kb * p.r_kb_stride;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 ::"v"(voffR), "s"(rb + rslab[n]),
                   "s"(lds_addr(Rd) + (uint32_t)((wave * 8 + (NT / 8) * n) * kBK))
                 : "memory");
  };
  auto dmaR_scales = [&](int kb, float* Sd) {
    if constexpr (!C::LAHEAD) {
      if (!l_side) dma_scale(kb, Sd);
      if (batch && (kb & 7) == 0) dma_scale_batch(kb >> 3);  // lands a step before its first use
    }
  };
  auto dmaL_one = [&](int n, int kb, uint8_t* Ld, float* Sd) {
    dmaL_tile(n, kb, Ld);
    if (n == C::LCH - 1) dmaL_scales(kb, Sd);
  };
  auto dmaR_one = [&](int n, int kb, uint8_t* Rd, float* Sd) {
    dmaR_tile(n, kb, Rd);
    if (n == C::RCH - 1) dmaR_scales(kb, Sd);
  };
  auto dmaL = [&](int kb, uint8_t* Ld, float* Sd) {
#pragma unroll
    for (int n = 0; n < C::LCH; n++) dmaL_one(n, kb, Ld, Sd);
  };
  auto dmaR = [&](int kb, uint8_t* Rd, float* Sd) {
#pragma unroll
    for (int n = 0; n < C::RCH; n++) dmaR_one(n, kb, Rd, Sd);
  };
  auto dma = [&](int kb, uint8_t* Ld, uint8_t* Rd, float* Sd) {
    dmaL(kb, Ld, Sd);
    dmaR(kb, Rd, Sd);
  };
  // End of a step: this thread's loads have landed, then the workgroup barrier.
  auto dma_wait_and_sync = [&]() {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };

  // ---- MFMA tiling ------------------------------------------------------------------------
  // v_mfma_f32_32x32x64_f8f6f4: lane l supplies operand row l%32 and 32 contraction bytes chosen
  // by l/32; with two MFMAs per 128-byte step a lane reads, per row and K half h, the logical
  // chunks 4h + 2(l/32) and 4h + 2(l/32) + 1.  Any assignment works as long as L and R use the
  // same one.  D: lane l holds column l%32, rows 8(r/4) + 4(l/32) + r%4 for r = 0..15.
  // Wave w runs on SIMD w % 4.  With eight waves the two on a SIMD share their R half and take L
  // row blocks half a tile apart, so that in a tile whose valid rows end in the first half every
  // SIMD keeps one wave with work and one that only loads: such a tile finishes in about two
  // thirds of the time instead of leaving two SIMDs idle and two fully loaded (measured +2 % on a
  // Zipf-ragged 64-group launch; pairs that differ in both halves measured 1 % slower overall).
  constexpr bool kRemap = NT == 512 && C::WR == 2 && C::WL == 4;
  const int wr = kRemap ? wave & 1 : wave / C::WL;
  const int wl = kRemap ? ((wave & 3) >> 1) + 2 * (wave >> 2) : wave % C::WL;
  const int l32 = lane & 31, hg = lane >> 5;
  const int sw = swz(l32);
  int chk[2][2];  // byte offset of the two chunks of K half h inside this lane's row
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int c = 0; c < 2; c++) chk[h][c] = ((4 * h + 2 * hg + c) ^ sw) << 4;
  const int wrow0 = wr * C::WTR * 32;            // first R row of this wave inside the tile
  const int wlrow0 = wl * C::WTL * 32;           // first L row of this wave inside the tile
  // LDS byte addresses of this lane's four chunks in its row of the wave's first sub-tile, stage 0.
  // Kept opaque: every fragment read is one of these plus a compile-time offset.
  uint32_t la[2][2], ra[2][2];
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int c = 0; c < 2; c++) {
      la[h][c] = (uint32_t)(uintptr_t)(lds_ptr_t)Lbuf0 + (uint32_t)((wlrow0 + l32) * kBK + chk[h][c]);
      ra[h][c] = (uint32_t)(uintptr_t)(lds_ptr_t)Rbuf0 + (uint32_t)((wrow0 + l32) * kBK + chk[h][c]);
      asm volatile("" : "+v"(la[h][c]));
      asm volatile("" : "+v"(ra[h][c]));
    }
  const bool wave_active = wrow0 < rvalid;        // whole wave in or out: rvalid % 128 == 0
  // a wave none of whose L rows or R rows is valid takes part in loads and barriers only
  const bool has_work = __builtin_amdgcn_readfirstlane((int)(wave_active && wlrow0 < lvalid)) != 0;

  v16f acc[C::WTR][C::WTL];
#pragma unroll
  for (int i = 0; i < C::WTR; i++)
#pragma unroll
    for (int j = 0; j < C::WTL; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = short_operands ? __builtin_nanf("") : 0.f;

  // One 128-deep step on the stage (Lt, Rt, Sct).  Per 32x32 sub-tile t: two chained MFMAs, then
  // the 16 scale-and-accumulate FMAs of sub-tile t-1 run in their shadow.  The wanted issue
  // order is described to the scheduler with group barriers and fenced with scheduling
  // barriers; the accumulators are tied to the end of the step so the FMAs cannot drift past
  // the workgroup barrier.  Branch free: waves outside a partial R tile compute on clamped
  // rows and skip only the final store.
  constexpr int NTILES = C::WTR * C::WTL;
  auto compute = [&](int kb, int stage, const float* Sct, auto&& after_l_reads, auto&& per_tile) {
    __builtin_amdgcn_sched_barrier(0);
    // L scale of tile row r: Lsc[r * lsc_stride]
    const int bsel = kb >> 3;
    const float* Lsc = batch ? LsB0 + (bsel & 1) * (BM * 8) + (kb - batch_start(bsel)) : Sct;
    const int lsc_stride = batch ? 8 : 1;
    const float* Rsc = Sct + BM;
    // fragment of sub-tile row `sub` (32 rows each) of one side, K half h
    typedef const __attribute__((address_space(3))) v4i* lds_v4i_t;
    auto load_frag = [&](const uint32_t (&base)[2][2], int rows_per_stage, int sub, int h) {
      const uint32_t delta = (uint32_t)((stage * rows_per_stage + sub * 32) * kBK);
      const v4i lo = *(lds_v4i_t)(uintptr_t)(base[h][0] + delta);
      const v4i hi = *(lds_v4i_t)(uintptr_t)(base[h][1] + delta);
      return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    v8i lf[C::WTL][2];
    float cs[C::WTL];
    const float rblk = R_PER_ROW ? 1.f : Rsc[wrow0 / kTile];
    v8i rf[2][2];
    // LDS reads in the order of first use: the first MFMA waits for two fragments only, the rest
    // arrive in its shadow
    lf[0][0] = load_frag(la, BM, 0, 0);
    rf[0][0] = load_frag(ra, BN, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    lf[0][1] = load_frag(la, BM, 0, 1);
    rf[0][1] = load_frag(ra, BN, 0, 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < C::WTL; j++) {
      const int row = wlrow0 + j * 32 + l32;
      if (j > 0) {
        lf[j][0] = load_frag(la, BM, j, 0);
        lf[j][1] = load_frag(la, BM, j, 1);
      }
      cs[j] = Lsc[row * lsc_stride] * rblk;
    }
    v4f rs[2][4];  // R_PER_ROW: scales of the 16 R rows this lane holds in a sub-tile
    auto load_r = [&](int i) {
      if (i > 0) {
        rf[i & 1][0] = load_frag(ra, BN, i, 0);
        rf[i & 1][1] = load_frag(ra, BN, i, 1);
      }
      if constexpr (R_PER_ROW) {
#pragma unroll
        for (int q = 0; q < 4; q++)
          rs[i & 1][q] = *reinterpret_cast<const v4f*>(&Rsc[wrow0 + i * 32 + 8 * q + 4 * hg]);
      }
    };
    // raw-product buffers: sub-tile t's fold runs D = PRB - 1 sub-tiles later (0: right after it).
    // Per-row R scales live in a two-slot ring that allows at most D = 1.
    constexpr int PRB = R_PER_ROW && C::PRB > 2 ? 2 : C::PRB;
    constexpr int D = PRB - 1;
    v16f pr[PRB];
    load_r(0);
    // acc of sub-tile t += raw product * scales, registers [8*half, 8*half + 8) of the sub-tile
    auto fold_half = [&](int t, int half) {
      const int i = t / C::WTL, j = t % C::WTL;
#pragma unroll
      for (int r = 8 * half; r < 8 * half + 8; r++) {
        const float sc = R_PER_ROW ? cs[j] * rs[i & 1][r / 4][r % 4] : cs[j];
        acc[i][j][r] = __builtin_fmaf(pr[t % PRB][r], sc, acc[i][j][r]);
      }
    };
    v16f zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.f;
    // Issue order per sub-tile, kept by full scheduling barriers: first MFMA, half of the previous
    // sub-tile's fold, second MFMA, the other half, then the LDS reads of the next R row.  Each MFMA
    // (16 passes) covers its own issue plus eight FMAs of another sub-tile.
    static_for<NTILES>([&](auto T) {
      constexpr int t = decltype(T)::value;
      constexpr int i = t / C::WTL, j = t % C::WTL;
      __builtin_amdgcn_sched_barrier(0);
      pr[t % PRB] = mfma_fp8_32x32x64(rf[i & 1][0], lf[j][0], zero);
      __builtin_amdgcn_sched_barrier(0);
      if (D >= 1 && t >= D) fold_half(t - D, 0);
      __builtin_amdgcn_sched_barrier(0);
      pr[t % PRB] = mfma_fp8_32x32x64(rf[i & 1][1], lf[j][1], pr[t % PRB]);
      __builtin_amdgcn_sched_barrier(0);
      if (D >= 1 && t >= D) fold_half(t - D, 1);
      if (D == 0) {
        fold_half(t, 0);
        fold_half(t, 1);
      }
      __builtin_amdgcn_sched_barrier(0);
      // the next R row overwrites the fragment and scale slot of row i - 1, whose last fold is done
      if (j == 0 && i + 1 < C::WTR) load_r(i + 1);
      __builtin_amdgcn_sched_barrier(0);
      // every L fragment has been an MFMA operand by now, so it has left the LDS: the hook (a
      // barrier and the next L loads) costs no extra wait here
      per_tile(T);
      if (t == C::WTL - 1) after_l_reads();
    });
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = NTILES - D; t < NTILES; t++) {
      fold_half(t, 0);
      fold_half(t, 1);
    }
    // tie the accumulators to this point: the FMAs above may not drift past the barrier below
#pragma unroll
    for (int i = 0; i < C::WTR; i++)
#pragma unroll
      for (int j = 0; j < C::WTL; j++) asm volatile("" : "+v"(acc[i][j]));
    __builtin_amdgcn_sched_barrier(0);
  };

  auto nothing = [] {};
  auto no_feed = [](auto) {};
  // Two workgroups per CU: the loads of a step go out in one burst after the barrier (issued a few
  // at a time behind the sub-tiles they measured 6 % slower here: they have less time to arrive,
  // and the other workgroup already fills the issue gap).
  if constexpr (!C::LAHEAD) {
    if (nkb > 0) dma(0, Lbuf0, Rbuf0, Sc0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // a wave without valid rows runs its own copy of the loop, loads and barriers only
    auto loop = [&](auto W) {
      constexpr bool kWork = decltype(W)::value;
      int kb = 0;
      for (; kb + 1 < nkb; kb += 2) {  // two steps per trip: the stage addresses are compile-time constants
        dma(kb + 1, Lbuf1, Rbuf1, Sc1);
        if constexpr (kWork) compute(kb, 0, Sc0, nothing, no_feed);
        dma_wait_and_sync();
        dma(kb + 2 < nkb ? kb + 2 : kb + 1, Lbuf0, Rbuf0, Sc0);  // the last prefetch re-reads a valid block
        if constexpr (kWork) compute(kb + 1, 1, Sc1, nothing, no_feed);
        dma_wait_and_sync();
      }
      if constexpr (kWork)
        if (kb < nkb) compute(kb, 0, Sc0, nothing, no_feed);  // odd number of steps
    };
    if (has_work) loop(std::true_type{});
    else loop(std::false_type{});
  } else {
    // One workgroup per CU, eight waves, two per SIMD.  The matrix pipe of a SIMD idles whenever both
    // of its waves are away from their MFMAs at the same time, which is what a workgroup barrier
    // followed by LDS reads produces.  So the two barriers of a step stand where register-resident
    // MFMA work follows them:
    //   Q (start of step k): every wave holds the L fragments of step k, so the L half of stage k is
    //     free and the L tile of step k+2 is requested behind the first sub-tiles;
    //   P (before the last R row of sub-tiles): every wave has read the last fragments of stage k
    //     and the tiles of step k+1 have landed; behind it the R tile of step k+2 is requested and
    //     the first fragments of step k+1 are read from the LDS while the last R row, whose operands
    //     are already in registers, runs on the matrix pipe.  The fragment registers of step k are
    //     reused as they die, so the prefetch costs no registers.
    // The fold of the sub-tile in front of a barrier is issued behind it: the wave that arrives last
    // has just issued its MFMAs, and the one that waited folds while those still run.
    // Loads complete in issue order, so "all but the newest L group" is one wait count.  Past the
    // end the loads re-read the last block to keep the counts uniform.
    static_assert(!R_PER_ROW && MODE == kRaggedRows, "the two-barrier pipeline is written for block-scaled R operands");
    static_assert(C::PRB == 1 && C::WTR % 2 == 0 && C::RCH % C::WTL == 0 && C::LCH <= NTILES, "pipeline shape");
    constexpr int PT = (C::WTR - 1) * C::WTL - 1;  // the sub-tile in front of barrier P
    constexpr int RPER = C::RCH / C::WTL;
    auto kclamp = [&](int k) { return k < nkb ? k : nkb - 1; };
    typedef const __attribute__((address_space(3))) v4i* lds_v4i_t;
    auto frag = [&](const uint32_t (&base)[2][2], int stage, int rows_per_stage, int sub, int h) {
      const uint32_t delta = (uint32_t)((stage * rows_per_stage + sub * 32) * kBK);
      const v4i lo = *(lds_v4i_t)(uintptr_t)(base[h][0] + delta);
      const v4i hi = *(lds_v4i_t)(uintptr_t)(base[h][1] + delta);
      return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    // Scales of this pipeline come in batches of eight contraction blocks only (the launcher takes the other
    // configuration when K has fewer than eight blocks), so a
    // step issues no scale load and takes no branch: batch b (blocks 8 b .. 8 b + 7, the last one shifted
    // back to end at the last block) is requested behind barrier P of step 8 (b - 1), eight steps before
    // its first use.  L scales: every wave fetches 32 rows x 32 bytes into LsB[b & 1][row][8]; R block
    // scales: wave 0 fetches the tile's two 128-row blocks x 32 bytes into RsB[b & 1][block][8] (lanes past
    // the fourth repeat those addresses: the direct-to-LDS load always writes 1 KB).
    // Scale rows that are not 16-byte aligned (a number of contraction blocks that is not a multiple of four, an
    // unaligned base) take 4-byte loads instead: four per wave and batch for the L scales (lane l of load q fetches
    // float 64 q + l of the wave's 32 rows x 8 floats), one for the R scales.
    float* const RsB0 = Sc0;  // [2][NT] floats, the first 16 of each in use
    const bool x4 = p.ls_batch == 1;
    const int rblocks = rvalid / kTile;
    const int rlane_blk = ((lane >> 1) & 1) < rblocks ? (lane >> 1) & 1 : rblocks - 1;
    const uint32_t roff = ((uint32_t)rlane_blk * (uint32_t)p.rs_row_stride + (uint32_t)(lane & 1) * 4u) * 4u;
    const int rlane_blk1 = ((lane >> 3) & 1) < rblocks ? (lane >> 3) & 1 : rblocks - 1;
    const uint32_t roff1 = ((uint32_t)rlane_blk1 * (uint32_t)p.rs_row_stride + (uint32_t)(lane & 7)) * 4u;
    uint32_t boff1[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int row = wave * 32 + q * 8 + (lane >> 3);
      boff1[q] = ((uint32_t)(row < lvalid ? row : lvalid - 1) * (uint32_t)p.ls_row_stride + (uint32_t)(lane & 7)) * 4u;
    }
    auto dma_batches = [&](int b) {
      const uint8_t* lsb = reinterpret_cast<const uint8_t*>(Lsg + uniform_i64(l0 * p.ls_row_stride + batch_start(b)));
      const uint8_t* rsb = reinterpret_cast<const uint8_t*>(Rsg + uniform_i64((r0 / kTile) * p.rs_row_stride + batch_start(b)));
      const uint32_t ldst = lds_addr(LsB0 + (b & 1) * (BM * 8)) + (uint32_t)(wave * 1024);
      const uint32_t rdst = lds_addr(RsB0 + (b & 1) * NT);
      if (x4) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(boff), "s"(lsb), "s"(ldst) : "memory");
        if (wave == 0)
          asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(roff), "s"(rsb), "s"(rdst) : "memory");
      } else {
#pragma unroll
        for (int q = 0; q < 4; q++)
          asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(boff1[q]), "s"(lsb), "s"(ldst + (uint32_t)(q * 256)) : "memory");
        if (wave == 0)
          asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(roff1), "s"(rsb), "s"(rdst) : "memory");
      }
    };
    if (nkb > 0) {
      dmaL(0, Lbuf0, Sc0);  // (the per-step scale hooks of these helpers are off: see step_scale)
      dmaR(0, Rbuf0, Sc0);
      dma_batches(0);
      dmaL(kclamp(1), Lbuf1, Sc1);
      dmaR(kclamp(1), Rbuf1, Sc1);
      // the tiles of step 0 and the first scale batch have landed; those of step 1 may still be on their way
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(C::LCH + C::RCH) : "memory");
      auto barrier_q = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
      // all but this step's L tile loads have landed (loads complete in issue order)
      auto barrier_p = [&]() { asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(C::LCH) : "memory"); };
      if (has_work) {
        v8i lf[C::WTL][2], rf[2][2];
        float cs[C::WTL], csn[C::WTL], rblkn;
        float cs_last = 0.f;  // scale of the sub-tile whose fold is still owed (the last one of the step before)
        v16f pr, zero;
#pragma unroll
        for (int r = 0; r < 16; r++) zero[r] = pr[r] = 0.f;
        // scales of step kb: the lane's L row scales and the R block scale of the wave; their product is
        // formed where it is first needed, not where the reads are issued
        auto read_scales = [&](int kb, float (&dst)[C::WTL], float& rblk) {
          const int b = kb >> 3, in_batch = kb - batch_start(b);
          const float* Lsc = LsB0 + (b & 1) * (BM * 8) + in_batch;
          rblk = RsB0[(b & 1) * NT + (wrow0 / kTile) * 8 + in_batch];
#pragma unroll
          for (int j = 0; j < C::WTL; j++) dst[j] = Lsc[(wlrow0 + j * 32 + l32) * 8];
        };
        // (the empty volatile statements pin MFMAs and folds between the memory instructions around
        // them: plain arithmetic is otherwise free to drift past inline assembly)
        auto fold = [&](int i, int j, float sc) {
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] = __builtin_fmaf(pr[r], sc, acc[i][j][r]);
          asm volatile("" : "+v"(acc[i][j]));
        };
        // fragments and scales of step 0
#pragma unroll
        for (int h = 0; h < 2; h++) {
          lf[0][h] = frag(la, 0, BM, 0, h);
          rf[0][h] = frag(ra, 0, BN, 0, h);
        }
#pragma unroll
        for (int j = 1; j < C::WTL; j++)
#pragma unroll
          for (int h = 0; h < 2; h++) lf[j][h] = frag(la, 0, BM, j, h);
        read_scales(0, cs, rblkn);
#pragma unroll
        for (int j = 0; j < C::WTL; j++) cs[j] *= rblkn;
        // FIRST: the first step of a run of eight, which requests the next scale batch behind barrier P
        auto step = [&](int kb, auto S, auto FIRST) {
          constexpr int s = decltype(S)::value;
          constexpr bool kFirst = decltype(FIRST)::value;
          uint8_t* const Lc = s ? Lbuf1 : Lbuf0;
          uint8_t* const Rc = s ? Rbuf1 : Rbuf0;
          const int k2 = kclamp(kb + 2);
          __builtin_amdgcn_sched_barrier(0);
          barrier_q();
          __builtin_amdgcn_sched_barrier(0);
          fold(C::WTR - 1, C::WTL - 1, cs_last);  // owed by the step before (adds zero in the first step)
          static_for<NTILES>([&](auto T) {
            constexpr int t = decltype(T)::value;
            constexpr int i = t / C::WTL, j = t % C::WTL;
            __builtin_amdgcn_sched_barrier(0);
            pr = mfma_fp8_32x32x64(rf[i & 1][0], lf[j][0], zero);
            pr = mfma_fp8_32x32x64(rf[i & 1][1], lf[j][1], pr);
            asm volatile("" : "+v"(pr));
            __builtin_amdgcn_sched_barrier(0);
            // memory instructions go out while the MFMAs run, ahead of the fold that waits for them
            if constexpr (t < C::LCH) dmaL_tile(t, k2, Lc);
            if constexpr (j == 0 && i + 1 < C::WTR) {
#pragma unroll
              for (int h = 0; h < 2; h++) rf[(i + 1) & 1][h] = frag(ra, s, BN, i + 1, h);
            }
            if constexpr (t == PT) {
              __builtin_amdgcn_sched_barrier(0);
              barrier_p();
              __builtin_amdgcn_sched_barrier(0);
              if constexpr (kFirst) {
                if (kb + 8 < nkb) dma_batches((kb >> 3) + 1);
              }
              // row C::WTR - 2 has been consumed: its registers take the first R row of the next step
#pragma unroll
              for (int h = 0; h < 2; h++) rf[0][h] = frag(ra, s ^ 1, BN, 0, h);
              read_scales(kclamp(kb + 1), csn, rblkn);
            }
            if constexpr (t > PT) {
              constexpr int jn = t - PT - 1;  // == j: this sub-tile was the last user of lf[j]
              static_for<RPER>([&](auto N) { dmaR_tile(jn * RPER + decltype(N)::value, k2, Rc); });
#pragma unroll
              for (int h = 0; h < 2; h++) lf[jn][h] = frag(la, s ^ 1, BM, jn, h);
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (t + 1 < NTILES) fold(i, j, cs[j]);
          });
          cs_last = cs[C::WTL - 1];
#pragma unroll
          for (int j = 0; j < C::WTL; j++) cs[j] = csn[j] * rblkn;
        };
        // runs of eight steps (the contraction has at least eight blocks; the last run may be shorter), two
        // steps per trip so that the stage addresses are compile-time constants
        constexpr std::integral_constant<int, 0> S0{};
        constexpr std::integral_constant<int, 1> S1{};
        for (int kb = 0; kb < nkb; kb += 8) {
          const int n = nkb - kb < 8 ? nkb - kb : 8;
          step(kb, S0, std::true_type{});
          if (n > 1) step(kb + 1, S1, std::false_type{});
          int kk = 2;
          for (; kk + 1 < n; kk += 2) {
            step(kb + kk, S0, std::false_type{});
            step(kb + kk + 1, S1, std::false_type{});
          }
          if (kk < n) step(kb + kk, S0, std::false_type{});  // odd number of steps
        }
        __builtin_amdgcn_sched_barrier(0);
        fold(C::WTR - 1, C::WTL - 1, cs_last);
      } else {
        // a wave without valid rows: loads and barriers only, in the order of the working waves
        auto step = [&](int kb, uint8_t* Lc, uint8_t* Rc, bool first) {
          const int k2 = kclamp(kb + 2);
          barrier_q();
#pragma unroll
          for (int n = 0; n < C::LCH; n++) dmaL_tile(n, k2, Lc);
          barrier_p();
          if (first && kb + 8 < nkb) dma_batches((kb >> 3) + 1);
#pragma unroll
          for (int n = 0; n < C::RCH; n++) dmaR_tile(n, k2, Rc);
        };
        int kb = 0;
        for (; kb + 1 < nkb; kb += 2) {
          step(kb, Lbuf0, Rbuf0, (kb & 7) == 0);
          step(kb + 1, Lbuf1, Rbuf1, false);
        }
        if (kb < nkb) step(kb, Lbuf0, Rbuf0, (kb & 7) == 0);
      }
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // the trailing loads must not land in the epilogue's staging
    }
  }

  // ---- epilogue ------------------------------------------------------------------------------
  // A lane holds, for one output row, groups of four consecutive columns; stored directly that
  // would be 8-byte pieces in 32 different rows per instruction.  Each wave instead transposes its
  // tile through its own LDS region and writes 128-byte row segments: 8 lanes x 16 bytes per row.
  if (MODE == kRaggedK && nkb == 0 && p.accumulate && !short_operands) return;  // empty group: leave dW untouched
  __syncthreads();  // every wave is done with the stage buffers
  if (!has_work) return;
  OUT* Cg = reinterpret_cast<OUT*>(p.C) + (int64_t)g * p.c_group_stride;
  uint8_t* const stg = lds + wave * kStgBytes;
  constexpr int WROWS = C::WTL * 32;
  static_assert(WROWS <= 64 && WROWS % 8 == 0, "the staging region holds 64 rows");
  // (the bias is a compile-time case: without one the staging is two conversions and a write per
  // four values instead of a uniform branch, four adds and the moves that feed them)
  auto flush = [&](auto tag, auto with_bias) {
    using ST = decltype(tag);  // staging type: OUT, or float when the old output is added in fp32
    constexpr bool kBias = decltype(with_bias)::value;
    constexpr int CW = 128 / (int)sizeof(ST);  // columns per chunk
    constexpr int SUBS = CW / 32;              // 32-column sub-tiles per chunk
    constexpr int PITCH = 128 + (sizeof(ST) == 2 ? 8 : 16);
    constexpr int VL = 16 / (int)sizeof(ST);   // columns per lane in the store phase
    static_assert(C::WTR % SUBS == 0, "chunks cover whole sub-tiles");
#pragma unroll
    for (int ci = 0; ci < C::WTR / SUBS; ci++) {
#pragma unroll
      for (int si = 0; si < SUBS; si++) {
        const int i = ci * SUBS + si;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int64_t rcol = r0 + wrow0 + i * 32 + 8 * q + 4 * hg;
          v4f b4 = {0.f, 0.f, 0.f, 0.f};
          if constexpr (kBias) {
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
            v4f o = v4f{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
            if constexpr (kBias) o += b4;
            uint8_t* dst = stg + (j * 32 + l32) * PITCH + (si * 32 + 8 * q + 4 * hg) * (int)sizeof(ST);
            if constexpr (sizeof(ST) == 4) {
              *reinterpret_cast<v4f*>(dst) = o;
            } else {
              v2i w;
              w[0] = (int)pack_bf16x2(o[0], o[1]);
              w[1] = (int)pack_bf16x2(o[2], o[3]);
              *reinterpret_cast<v2i*>(dst) = w;
            }
          }
        }
      }
      __builtin_amdgcn_wave_barrier();  // same wave, in-order LDS: the reads below see the writes above
      const int64_t col = r0 + wrow0 + ci * CW + (lane & 7) * VL;
      // all rows of the chunk leave the LDS before the first store: inside the row-valid branches
      // each read would be followed by its own wait.  One 64-bit row address per chunk, then steps
      // of eight rows.
      v4i raws[WROWS / 8];
#pragma unroll
      for (int ps = 0; ps < WROWS / 8; ps++)
        raws[ps] = *reinterpret_cast<const v4i*>(stg + (ps * 8 + (lane >> 3)) * PITCH + (lane & 7) * 16);
#pragma unroll
      for (int ps = 0; ps < WROWS / 8; ps++) asm volatile("" : "+v"(raws[ps]));
      OUT* const out_row0 = Cg + (l0 + wlrow0 + (lane >> 3)) * p.ldc + col;
      const int64_t row_step = 8 * p.ldc;
      // accumulation into an fp32 output: the old values of all rows are requested before the
      // first is used (one trip to memory per chunk instead of one per row)
      constexpr bool kAddF32 = sizeof(ST) == sizeof(OUT) && sizeof(OUT) == 4;
      v4f olds[kAddF32 ? WROWS / 8 : 1];
      if constexpr (kAddF32) {
        if (p.accumulate) {
          OUT* o_row = out_row0;
#pragma unroll
          for (int ps = 0; ps < WROWS / 8; ps++) {
            olds[ps] = v4f{0.f, 0.f, 0.f, 0.f};
            if (wlrow0 + ps * 8 + (lane >> 3) < lvalid) olds[ps] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(o_row));
            o_row += row_step;
          }
#pragma unroll
          for (int ps = 0; ps < WROWS / 8; ps++) asm volatile("" : "+v"(olds[ps]));
        }
      }
      OUT* out_row = out_row0;
#pragma unroll
      for (int ps = 0; ps < WROWS / 8; ps++) {
        const int lrow = wlrow0 + ps * 8 + (lane >> 3);
        const v4i raw = raws[ps];
        OUT* out = out_row;
        out_row += row_step;
        if (lrow < lvalid) {
          if constexpr (sizeof(ST) == sizeof(OUT)) {
            if constexpr (sizeof(OUT) == 4) {
              // the output is not read again by this launch: streaming stores keep it from
              // evicting operand panels from L2 (measured +1-2 % where the output is large)
              if (p.accumulate) {
                const v4f o = __builtin_bit_cast(v4f, raw) + olds[ps];
                __builtin_nontemporal_store(o, reinterpret_cast<v4f*>(out));
              } else {
                __builtin_nontemporal_store(raw, reinterpret_cast<v4i*>(out));
              }
            } else {
              __builtin_nontemporal_store(raw, reinterpret_cast<v4i*>(out));
            }
          } else {  // fp32 staging, bf16 output with accumulation
            store4<OUT>(out, __builtin_bit_cast(v4f, raw), true);
          }
        }
      }
      __builtin_amdgcn_wave_barrier();  // the next chunk overwrites the region
    }
  };
  const bool with_bias = MODE == kRaggedRows && p.bias != nullptr;
  auto flush_as = [&](auto tag) {
    if constexpr (MODE == kRaggedRows) {
      if (with_bias) flush(tag, std::true_type{});
      else flush(tag, std::false_type{});
    } else {
      flush(tag, std::false_type{});
    }
  };
  if constexpr (sizeof(OUT) == 4) {
    flush_as(float{});
  } else {
    if (p.accumulate) flush_as(float{});
    else flush_as(u16{});
  }
}

int launch_group_tile_offsets(const int64_t* goff, int E, int tile, int32_t* tile_off, hipStream_t st);

// Launch choices a caller of the measurement build may pin per call (-1 = the library chooses, which is
// all the product entry points ever pass).
struct GemmOptions {
  int tile = -1;      // 0: 128x128 tiles, 1: the large configuration
  int group_r = -1;   // tile order groups R tiles (1) or L tiles (0)
  int gl = -1;        // tiles that share a panel in the tile order
  int ls_batch = -1;  // 0: L scales fetched one contraction block at a time
};

template <int MODE, bool R_PER_ROW, typename C>
static int launch_gemm(GemmParams p, int c_dtype, int64_t blocks, hipStream_t st, const GemmOptions& g_opt) {
  if (blocks <= 0) return AAMD_OK;
  // L tiles per group of the tile order: 8 for the row-ragged launches; 4 for wgrad, whose operand
  // panels run over all tokens of an expert and are several times larger (measured: 5 % faster
  // at 4096 tokens per expert and 28672 x 4096 outputs, within 3 % either way elsewhere)
  p.gl = MODE == kRaggedK ? 4 : 8;
  // group along the side with more tiles per expert (row-ragged launches: batches of 4 R tiles measured 1 % faster
  // than the L grouping with many small groups, the same with few large ones)
  if (MODE == kRaggedK) p.group_r = p.nRt > p.nLt;
  else p.group_r = p.goff != nullptr && (int64_t)p.nRt * C::BM * p.E > p.Lrows;
  if (MODE == kRaggedRows && p.group_r) p.gl = 4;
  // per-call overrides (measurement build only)
  if (g_opt.group_r >= 0) p.group_r = g_opt.group_r != 0 && (MODE == kRaggedK || p.goff != nullptr);
  if (g_opt.gl > 0) p.gl = g_opt.gl;

  AAMD_REQUIRE(blocks < 0x7fffffffLL, "grouped_gemm: grid too large");
  dim3 grid((unsigned)blocks), block(C::NT);
  if (c_dtype == AAMD_BF16)
    grouped_gemm_kernel<MODE, R_PER_ROW, u16, C><<<grid, block, 0, st>>>(p);
  else
    grouped_gemm_kernel<MODE, R_PER_ROW, float, C><<<grid, block, 0, st>>>(p);
  AAMD_LAUNCH_CHECK("grouped_gemm");
  return AAMD_OK;
}

// Tile choice: large tiles whenever the problem has enough of them to fill the chip
// (option "tile": 0 forces the small configuration, 1 the large one).
static bool use_large_tiles(int64_t tiles_256, bool by_default, const GemmOptions& g_opt) {
  if (g_opt.tile == 0) return false;
  if (g_opt.tile == 1) return true;
  // 256x256 tiles halve the bytes every CU pulls from L2 and measured faster wherever the launch
  // still fills the GPU with them; small launches keep the 128x128 tiles (two workgroups per CU).
  return by_default && tiles_256 >= 512;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace aamd

using namespace aamd;

static int gemm_nt_impl(const uint8_t* a, int64_t lda, const float* a_s, const uint8_t* b, const float* b_s,
                        int b_tile_scaled, const int64_t* group_offsets, int E, int32_t* tile_ws, int64_t M, int64_t N,
                        int64_t K, void* c, int c_dtype, int64_t ldc, const void* bias, int bias_dtype, void* stream,
                        const GemmOptions& g_opt = GemmOptions()) {
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
  AAMD_REQUIRE(ldc >= N && (ldc * (c_dtype == AAMD_BF16 ? 2 : 4)) % 16 == 0 && aligned16(c),
               "grouped_gemm_nt: output rows must be 16-byte aligned");
  AAMD_REQUIRE(K > 0, "grouped_gemm_nt: K must be positive");
  AAMD_REQUIRE(lda < (1LL << 23) && K < (1LL << 23), "grouped_gemm_nt: row stride too large");
  hipStream_t st = (hipStream_t)stream;
  // scale batches of eight contraction blocks; their 16-byte loads need aligned rows and whole groups of four blocks
  const bool batches = (K / kBK) >= 8 && g_opt.ls_batch != 0;
  const bool batches16 = batches && (K / kBK) % 4 == 0 && aligned16(a_s);
  // tile-scaled B carries per-row R scales: use the configuration that has room for them; the 256x256
  // configuration takes all its scales in batches (with 4-byte loads where the rows are not aligned)
  const bool large = use_large_tiles(((M + 255) / 256 + (group_offsets ? E : 0)) * ((N + 255) / 256), true, g_opt) &&
                     (b_tile_scaled || batches);
  const int BM = large ? CfgLarge::BM : CfgSmall::BM;
  const int BN = large ? (b_tile_scaled ? CfgWgrad::BN : CfgLarge::BN) : CfgSmall::BN;
  if (group_offsets) {
    int rc = launch_group_tile_offsets(group_offsets, E, BM, tile_ws, st);
    if (rc) return rc;
  }
  GemmParams p = {};
  p.L = a; p.ldl = lda; p.Ls = a_s; p.ls_row_stride = K / kBK; p.ls_blk_stride = 1;
  p.l_kb_stride = p.r_kb_stride = kBK;
  // 1: batches by 16-byte loads; 2 (256x256 configuration only): by 4-byte loads
  p.ls_batch = large && !b_tile_scaled ? (batches16 && aligned16(b_s) ? 1 : 2) : (batches16 ? 1 : 0);
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
    return b_tile_scaled ? launch_gemm<kRaggedRows, true, CfgWgrad>(p, c_dtype, blocks, st, g_opt)
                         : launch_gemm<kRaggedRows, false, CfgLarge>(p, c_dtype, blocks, st, g_opt);
  return b_tile_scaled ? launch_gemm<kRaggedRows, true, CfgSmall>(p, c_dtype, blocks, st, g_opt)
                       : launch_gemm<kRaggedRows, false, CfgSmall>(p, c_dtype, blocks, st, g_opt);
}

#ifndef AAMD_TUNING
extern "C" int aamd_grouped_gemm_fp8_nt(const uint8_t* a, int64_t lda, const float* a_s, const uint8_t* b,
                                        const float* b_s, int b_tile_scaled, const int64_t* group_offsets, int E,
                                        int32_t* tile_ws, int64_t M, int64_t N, int64_t K, void* c, int c_dtype,
                                        int64_t ldc, const void* bias, int bias_dtype, void* stream) {
  return gemm_nt_impl(a, lda, a_s, b, b_s, b_tile_scaled, group_offsets, E, tile_ws, M, N, K, c, c_dtype, ldc, bias,
                      bias_dtype, stream);
}

// The same GEMM for callers that cannot allocate: the tile prefix lives in a file-scope device
// array, one copy per GPU, whose address is looked up once per device.
namespace aamd {
constexpr int kStaticMaxGroups = AAMD_STATIC_MAX_GROUPS;
static __device__ __align__(256) int32_t scratch[kStaticMaxGroups + 1];
constexpr int kMaxDevices = 64;
static std::atomic<int32_t*> g_scratch_ptr[kMaxDevices];

// Device address of this GPU's copy of `scratch` (the array's name is only a host-side handle).
static int scratch_of_current_device(int32_t** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  AAMD_REQUIRE(dev >= 0 && dev < kMaxDevices, "grouped_gemm_nt_static: device index %d out of range", dev);
  int32_t* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    AAMD_REQUIRE(ptr != nullptr, "grouped_gemm_nt_static: no device address for the scratch array");
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // every thread finds the same address
  }
  *out = ptr;
  return AAMD_OK;
}
}  // namespace aamd

extern "C" int aamd_grouped_gemm_fp8_nt_static(const uint8_t* a, int64_t lda, const float* a_s, const uint8_t* b,
                                               const float* b_s, int b_tile_scaled, const int64_t* group_offsets,
                                               int E, int64_t M, int64_t N, int64_t K, void* c, int c_dtype,
                                               int64_t ldc, const void* bias, int bias_dtype, void* stream) {
  AAMD_REQUIRE(E >= 1 && E <= kStaticMaxGroups, "grouped_gemm_nt_static: E=%d exceeds the %d groups the static scratch holds",
               E, kStaticMaxGroups);
  int32_t* ws = nullptr;
  if (group_offsets != nullptr) {
    const int rc = scratch_of_current_device(&ws);
    if (rc) return rc;
  }
  // the tile prefix is rewritten in full (E + 1 entries) by the first kernel of every call
  return gemm_nt_impl(a, lda, a_s, b, b_s, b_tile_scaled, group_offsets, E, ws, M, N, K, c, c_dtype, ldc, bias,
                      bias_dtype, stream);
}
#endif  // !AAMD_TUNING

static int wgrad_impl(const uint8_t* dyt, const float* sdyt, const uint8_t* xt, const float* sxt, int64_t ld_t,
                      int q_t_layout, const int64_t* group_offsets, int E, int32_t* tile_ws, int64_t N, int64_t K, void* dw,
                      int dw_dtype, int64_t expert_stride, int accumulate, void* stream,
                      const GemmOptions& g_opt = GemmOptions()) {
  AAMD_REQUIRE(dw_dtype == AAMD_BF16 || dw_dtype == AAMD_F32, "grouped_gemm_wgrad: unsupported output dtype %d", dw_dtype);
  AAMD_REQUIRE(N >= 0 && K >= 0 && N % kTile == 0 && K % kTile == 0,
               "grouped_gemm_wgrad: N=%lld and K=%lld must be multiples of 128", (long long)N, (long long)K);
  AAMD_REQUIRE(E >= 1 && group_offsets && tile_ws, "grouped_gemm_wgrad: group_offsets / tile_ws required");
  AAMD_REQUIRE(ld_t >= 0 && ld_t % kBK == 0, "grouped_gemm_wgrad: ld_t=%lld must be a multiple of 128", (long long)ld_t);
  AAMD_REQUIRE(ld_t < (1LL << 23), "grouped_gemm_wgrad: ld_t too large");
  AAMD_REQUIRE(q_t_layout == AAMD_QT_ROWS || q_t_layout == AAMD_QT_BLOCKED, "grouped_gemm_wgrad: unknown operand layout %d", q_t_layout);
  if (N == 0 || K == 0) return AAMD_OK;
  AAMD_REQUIRE(dw && (ld_t == 0 || (dyt && sdyt && xt && sxt)), "grouped_gemm_wgrad: null pointer");
  AAMD_REQUIRE(aligned16(dyt) && aligned16(xt) && aligned16(dw), "grouped_gemm_wgrad: pointers must be 16-byte aligned");
  AAMD_REQUIRE(expert_stride >= N * K && expert_stride % 4 == 0, "grouped_gemm_wgrad: bad expert stride");
  hipStream_t st = (hipStream_t)stream;
  int rc = launch_group_tile_offsets(group_offsets, E, kBK, tile_ws, st);
  if (rc) return rc;
  GemmParams p = {};
  p.L = dyt; p.Ls = sdyt; p.ls_row_stride = 1; p.ls_blk_stride = N;
  p.R = xt; p.r_group_stride = 0;
  if (q_t_layout == AAMD_QT_BLOCKED) {  // [ld_t / 128, rows, 128]: a contraction block of all rows is one slab
    p.ldl = p.ldr = kBK;
    p.l_kb_stride = N * kBK; p.r_kb_stride = K * kBK;
  } else {
    p.ldl = p.ldr = ld_t;
    p.l_kb_stride = p.r_kb_stride = kBK;
  }
  p.Rs = sxt; p.rs_row_stride = 1; p.rs_blk_stride = K; p.rs_group_stride = 0;
  p.C = dw; p.ldc = K; p.c_group_stride = expert_stride;
  p.bias = nullptr; p.bias_dtype = AAMD_NONE; p.bias_group_stride = 0;
  p.goff = group_offsets; p.tile_off = tile_ws;
  // per-row scales on both operands: the 128x128 configuration measured faster for wgrad
  // (measurement build: tile 1 = 256 x 128)
  const int cfg = g_opt.tile > 0 ? 1 : 0;
  const int BM = cfg ? CfgWgrad::BM : CfgSmall::BM;
  const int BN = cfg ? CfgWgrad::BN : CfgSmall::BN;
  p.Lrows = N; p.Rrows = K; p.nkb = 0; p.E = E; p.nRt = (int)((K + BN - 1) / BN); p.nLt = (int)((N + BM - 1) / BM);
  p.max_kb = (int)(ld_t / kBK);
  p.accumulate = accumulate;
  const int64_t blocks = (int64_t)E * p.nLt * p.nRt;
#ifdef AAMD_TUNING
  if (cfg == 1) return launch_gemm<kRaggedK, true, CfgWgrad>(p, dw_dtype, blocks, st, g_opt);
#endif
  return launch_gemm<kRaggedK, true, CfgSmall>(p, dw_dtype, blocks, st, g_opt);
}

#ifndef AAMD_TUNING
extern "C" int aamd_grouped_gemm_fp8_wgrad(const uint8_t* dyt, const float* sdyt, const uint8_t* xt,
                                           const float* sxt, int64_t ld_t, int q_t_layout,
                                           const int64_t* group_offsets, int E, int32_t* tile_ws, int64_t N,
                                           int64_t K, void* dw, int dw_dtype, int64_t expert_stride, int accumulate,
                                           void* stream) {
  return wgrad_impl(dyt, sdyt, xt, sxt, ld_t, q_t_layout, group_offsets, E, tile_ws, N, K, dw, dw_dtype, expert_stride, accumulate,
                    stream);
}
#else
// Measurement build (libatorch_amd_probes.so): the same two GEMMs with the launch choices pinned per call.
// opts = {tile, group_r, gl, ls_batch}, -1 = the library's own choice.
extern "C" int aamd_tuning_grouped_gemm_fp8_nt(const uint8_t* a, int64_t lda, const float* a_s, const uint8_t* b,
                                               const float* b_s, int b_tile_scaled, const int64_t* group_offsets,
                                               int E, int32_t* tile_ws, int64_t M, int64_t N, int64_t K, void* c,
                                               int c_dtype, int64_t ldc, const void* bias, int bias_dtype,
                                               const int* opts, void* stream) {
  AAMD_REQUIRE(opts != nullptr, "tuning_grouped_gemm_nt: null options");
  GemmOptions o;
  o.tile = opts[0]; o.group_r = opts[1]; o.gl = opts[2]; o.ls_batch = opts[3];
  return gemm_nt_impl(a, lda, a_s, b, b_s, b_tile_scaled, group_offsets, E, tile_ws, M, N, K, c, c_dtype, ldc, bias,
                      bias_dtype, stream, o);
}
extern "C" int aamd_tuning_grouped_gemm_fp8_wgrad(const uint8_t* dyt, const float* sdyt, const uint8_t* xt,
                                                  const float* sxt, int64_t ld_t, int q_t_layout,
                                                  const int64_t* group_offsets, int E, int32_t* tile_ws, int64_t N,
                                                  int64_t K, void* dw, int dw_dtype, int64_t expert_stride,
                                                  int accumulate, const int* opts, void* stream) {
  AAMD_REQUIRE(opts != nullptr, "tuning_grouped_gemm_wgrad: null options");
  GemmOptions o;
  o.tile = opts[0]; o.group_r = opts[1]; o.gl = opts[2]; o.ls_batch = opts[3];
  return wgrad_impl(dyt, sdyt, xt, sxt, ld_t, q_t_layout, group_offsets, E, tile_ws, N, K, dw, dw_dtype, expert_stride,
                    accumulate, stream, o);
}
#endif
