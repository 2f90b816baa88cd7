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
#include "common.hpp"

namespace aamd {

constexpr int kBM = 128;  // L rows per workgroup tile
constexpr int kBN = 128;  // R rows per workgroup tile
constexpr int kBK = 128;  // contraction bytes per step == scale block

enum GemmMode { kRaggedRows = 0, kRaggedK = 1 };

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

template <int MODE, bool R_PER_ROW, typename OUT>
__global__ __launch_bounds__(256, 2) void grouped_gemm_kernel(const GemmParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t Lbuf[2][kBM * kBK];
  __shared__ __attribute__((aligned(16))) uint8_t Rbuf[2][kBN * kBK];
  __shared__ __attribute__((aligned(16))) float Lsc[2][kBM];
  __shared__ __attribute__((aligned(16))) float Rsc[2][kBN];
  __shared__ int slot;

  const int tid = threadIdx.x;

  // ---- which tile -------------------------------------------------------------------
  // Workgroup ids go round-robin over the 8 XCDs; give every XCD one contiguous range of
  // tile ids so that tiles sharing operand panels meet in the same L2.
  int g, lt, rt;
  {
    const int total_lt = MODE == kRaggedRows ? (p.goff ? p.tile_off[p.E] : (int)((p.Lrows + kBM - 1) / kBM))
                                             : p.nLt * p.E;
    const int64_t ntot = (int64_t)total_lt * p.nRt;
    const int64_t bid = blockIdx.x;
    if (bid >= ntot) return;
    const int64_t per = ntot / 8, rem = ntot % 8;
    const int64_t xcd = bid % 8, idx = bid / 8;
    const int64_t pid = xcd < rem ? xcd * (per + 1) + idx : rem * (per + 1) + (xcd - rem) * per + idx;
    // inside the range: groups of 8 L tiles, R tile index outer, L tile inner
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
      l0 = p.goff[g] + (int64_t)(lt - p.tile_off[g]) * kBM;
      const int64_t left = p.goff[g + 1] - l0;
      lvalid = left < kBM ? (int)left : kBM;
    } else {
      g = 0;
      l0 = (int64_t)lt * kBM;
      const int64_t left = p.Lrows - l0;
      lvalid = left < kBM ? (int)left : kBM;
    }
    kb0 = 0;
    nkb = p.nkb;
  } else {
    g = lt / p.nLt;
    lt -= g * p.nLt;
    l0 = (int64_t)lt * kBM;
    lvalid = kBM;
    kb0 = p.tile_off[g];
    nkb = p.tile_off[g + 1] - kb0;
    if (kb0 + nkb > p.max_kb) nkb = p.max_kb > kb0 ? p.max_kb - kb0 : 0;  // never read past the buffers
  }
  g = __builtin_amdgcn_readfirstlane(g);
  const int64_t r0 = (int64_t)rt * kBN;

  const uint8_t* Lg = p.L + (int64_t)kb0 * kBK;
  const uint8_t* Rg = p.R + (int64_t)g * p.r_group_stride + (int64_t)kb0 * kBK;
  const float* Lsg = p.Ls + (int64_t)kb0 * p.ls_blk_stride;
  const float* Rsg = p.Rs + (int64_t)g * p.rs_group_stride + (int64_t)kb0 * p.rs_blk_stride;

  // ---- global -> register staging: 4 L chunks + 4 R chunks of 16 bytes per thread ------
  const int ld_row = tid >> 3, ld_ch = tid & 7;  // + 32 rows per step
  const uint8_t* lptr[4];
  const uint8_t* rptr[4];
  int lds_off[4];
#pragma unroll
  for (int n = 0; n < 4; n++) {
    const int row = ld_row + 32 * n;
    const int lrow = row < lvalid ? row : lvalid - 1;
    lptr[n] = Lg + (l0 + lrow) * p.ldl + ld_ch * 16;
    rptr[n] = Rg + (r0 + row) * p.ldr + ld_ch * 16;
    lds_off[n] = row * kBK + ((ld_ch ^ (row & 7)) << 4);
  }
  // scales: threads 0..127 fetch the L scale of row tid; threads 128..255 the per-row R scale
  const float* sptr;
  if (tid < kBM) {
    const int lrow = tid < lvalid ? tid : lvalid - 1;
    sptr = Lsg + (l0 + lrow) * p.ls_row_stride;
  } else {
    sptr = R_PER_ROW ? Rsg + (r0 + (tid - kBM)) * p.rs_row_stride : Rsg + rt * p.rs_row_stride;
  }
  const int64_t s_step = tid < kBM ? p.ls_blk_stride : p.rs_blk_stride;

  v4i lreg[4], rreg[4];
  float sreg = 0.f;
  auto g_load = [&](int kb) {
#pragma unroll
    for (int n = 0; n < 4; n++) {
      lreg[n] = *reinterpret_cast<const v4i*>(lptr[n] + (int64_t)kb * kBK);
      rreg[n] = *reinterpret_cast<const v4i*>(rptr[n] + (int64_t)kb * kBK);
    }
    sreg = sptr[(int64_t)kb * s_step];
  };
  auto s_store = [&](int buf) {
#pragma unroll
    for (int n = 0; n < 4; n++) {
      *reinterpret_cast<v4i*>(&Lbuf[buf][lds_off[n]]) = lreg[n];
      *reinterpret_cast<v4i*>(&Rbuf[buf][lds_off[n]]) = rreg[n];
    }
    if (tid < kBM)
      Lsc[buf][tid] = sreg;
    else
      Rsc[buf][tid - kBM] = sreg;
  };

  // ---- MFMA tiling ------------------------------------------------------------------------
  const int wave = tid >> 6, lane = tid & 63;
  const int wr = wave >> 1, wl = wave & 1;
  const int l16 = lane & 15, lg = lane >> 4;
  const int sw = l16 & 7;
  const int ch0 = ((2 * lg) ^ sw) << 4, ch1 = ((2 * lg + 1) ^ sw) << 4;

  v4f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  if (nkb > 0) {
    g_load(0);
    s_store(0);
  }
  __syncthreads();

  for (int kb = 0; kb < nkb; kb++) {
    const int cur = kb & 1;
    if (kb + 1 < nkb) g_load(kb + 1);

    const uint8_t* Lt = Lbuf[cur];
    const uint8_t* Rt = Rbuf[cur];
    v8i lf[4];
    float cs[4];
    const float rblk = R_PER_ROW ? 1.f : Rsc[cur][0];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int row = wl * 64 + j * 16 + l16;
      const v4i lo = *reinterpret_cast<const v4i*>(Lt + row * kBK + ch0);
      const v4i hi = *reinterpret_cast<const v4i*>(Lt + row * kBK + ch1);
      lf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      cs[j] = Lsc[cur][row] * rblk;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = wr * 64 + i * 16 + l16;
      const v4i lo = *reinterpret_cast<const v4i*>(Rt + row * kBK + ch0);
      const v4i hi = *reinterpret_cast<const v4i*>(Rt + row * kBK + ch1);
      const v8i rf = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      v4f rs4 = {1.f, 1.f, 1.f, 1.f};
      if constexpr (R_PER_ROW) rs4 = *reinterpret_cast<const v4f*>(&Rsc[cur][wr * 64 + i * 16 + 4 * lg]);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const v4f pr = mfma_fp8_16x16x128(rf, lf[j]);
        if constexpr (R_PER_ROW) {
#pragma unroll
          for (int r = 0; r < 4; r++) acc[i][j][r] = __builtin_fmaf(pr[r], cs[j] * rs4[r], acc[i][j][r]);
        } else {
#pragma unroll
          for (int r = 0; r < 4; r++) acc[i][j][r] = __builtin_fmaf(pr[r], cs[j], acc[i][j][r]);
        }
      }
    }

    if (kb + 1 < nkb) s_store(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue ------------------------------------------------------------------------------
  if (MODE == kRaggedK && nkb == 0 && p.accumulate) return;  // empty group: leave dW untouched
  OUT* Cg = reinterpret_cast<OUT*>(p.C) + (int64_t)g * p.c_group_stride;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int64_t rcol = r0 + wr * 64 + i * 16 + 4 * lg;
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
    for (int j = 0; j < 4; j++) {
      const int lrow = wl * 64 + j * 16 + l16;
      if (lrow < lvalid) store4<OUT>(Cg + (l0 + lrow) * p.ldc + rcol, acc[i][j] + b4, p.accumulate != 0);
    }
  }
}

int launch_group_tile_offsets(const int64_t* goff, int E, int tile, int32_t* tile_off, hipStream_t st);

template <int MODE, bool R_PER_ROW>
static int launch_gemm(const GemmParams& p, int c_dtype, int64_t blocks, hipStream_t st) {
  if (blocks <= 0) return AAMD_OK;
  AAMD_REQUIRE(blocks < 0x7fffffffLL, "grouped_gemm: grid too large");
  dim3 grid((unsigned)blocks), block(256);
  if (c_dtype == AAMD_BF16)
    grouped_gemm_kernel<MODE, R_PER_ROW, u16><<<grid, block, 0, st>>>(p);
  else
    grouped_gemm_kernel<MODE, R_PER_ROW, float><<<grid, block, 0, st>>>(p);
  AAMD_LAUNCH_CHECK("grouped_gemm");
  return AAMD_OK;
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
  AAMD_REQUIRE(K % kBK == 0 && N % kBN == 0, "grouped_gemm_nt: K=%lld and N=%lld must be multiples of 128",
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
  if (group_offsets) {
    int rc = launch_group_tile_offsets(group_offsets, E, kBM, tile_ws, st);
    if (rc) return rc;
  }
  GemmParams p = {};
  p.L = a; p.ldl = lda; p.Ls = a_s; p.ls_row_stride = K / kBK; p.ls_blk_stride = 1;
  p.R = b; p.ldr = K; p.r_group_stride = N * K;
  p.Rs = b_s;
  p.rs_row_stride = K / kBK; p.rs_blk_stride = 1;
  p.rs_group_stride = b_tile_scaled ? N * (K / kBK) : (N / kBN) * (K / kBK);
  p.C = c; p.ldc = ldc; p.c_group_stride = 0;
  p.bias = bias; p.bias_dtype = bias_dtype; p.bias_group_stride = N;
  p.goff = group_offsets; p.tile_off = tile_ws;
  p.Lrows = M; p.Rrows = N; p.nkb = (int)(K / kBK); p.E = E; p.nRt = (int)(N / kBN); p.nLt = 0;
  p.accumulate = 0;
  const int64_t max_lt = group_offsets ? M / kBM + E : (M + kBM - 1) / kBM;
  const int64_t blocks = max_lt * p.nRt;
  return b_tile_scaled ? launch_gemm<kRaggedRows, true>(p, c_dtype, blocks, st)
                       : launch_gemm<kRaggedRows, false>(p, c_dtype, blocks, st);
}

extern "C" int aamd_grouped_gemm_fp8_wgrad(const uint8_t* dyt, const float* sdyt, const uint8_t* xt,
                                           const float* sxt, int64_t ld_t, const int64_t* group_offsets, int E,
                                           int32_t* tile_ws, int64_t N, int64_t K, void* dw, int dw_dtype,
                                           int64_t expert_stride, int accumulate, void* stream) {
  AAMD_REQUIRE(dw_dtype == AAMD_BF16 || dw_dtype == AAMD_F32, "grouped_gemm_wgrad: unsupported output dtype %d", dw_dtype);
  AAMD_REQUIRE(N >= 0 && K >= 0 && N % kBM == 0 && K % kBN == 0,
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
  p.Lrows = N; p.Rrows = K; p.nkb = 0; p.E = E; p.nRt = (int)(K / kBN); p.nLt = (int)(N / kBM);
  p.max_kb = (int)(ld_t / kBK);
  p.accumulate = accumulate;
  const int64_t blocks = (int64_t)E * p.nLt * p.nRt;
  return launch_gemm<kRaggedK, true>(p, dw_dtype, blocks, st);
}
