// Token routing kernels for gfx950: device-side router preprocess (histogram, scan, stable
// counting sort), inverse permutation, and the fused unpermute + weighted combine.
#include "common.hpp"

// The combine reproduces "multiply, round, then sum": no fused multiply-add in this file.
#pragma clang fp contract(off)

namespace aamd {

// ---------------------------------------------------------------------------------------
// unpermute + combine: one workgroup per token, 16-byte gathers of the topk source rows.
// PD: dtype of probs (AAMD_NONE / AAMD_BF16 / AAMD_F32).
// ---------------------------------------------------------------------------------------
constexpr int kMaxTopk = 64;

// YT: element type of the permuted rows (BF16 or F32); the result has the promoted type of rows and
// probs (fp32 rows, or fp32 probs, give fp32).
template <typename YT, int PD>
__global__ __launch_bounds__(1024) void unpermute_combine_kernel(const typename YT::elem* __restrict__ y, int64_t M, int H8,
                                                                const int32_t* __restrict__ row_map,
                                                                const void* __restrict__ probs, int topk,
                                                                void* __restrict__ out) {
  constexpr bool kRowsF32 = std::is_same<YT, F32>::value;
  constexpr int VL = kRowsF32 ? 4 : 8;                      // elements per 16-byte chunk (H8 counts chunks)
  constexpr bool kRoundProducts = !kRowsF32 && PD == AAMD_BF16;  // products are bf16 tensors in the reference
  constexpr bool kOutF32 = kRowsF32 || PD == AAMD_F32;
  __shared__ int srow[kMaxTopk];
  __shared__ float sprob[kMaxTopk];
  const int64_t t = blockIdx.x;
  if ((int)threadIdx.x < topk) {
    int r = row_map[t * topk + threadIdx.x];
    if (r >= M) r = -1;
    srow[threadIdx.x] = r;
    float pv = 1.f;
    if constexpr (PD == AAMD_BF16) pv = bf16_bits_to_f32(reinterpret_cast<const u16*>(probs)[t * topk + threadIdx.x]);
    if constexpr (PD == AAMD_F32) pv = reinterpret_cast<const float*>(probs)[t * topk + threadIdx.x];
    sprob[threadIdx.x] = pv;
  }
  __syncthreads();
  const int64_t H = (int64_t)H8 * VL;
  for (int c = threadIdx.x; c < H8; c += blockDim.x) {
    // torch's reduction of a strided dimension, which the reference runs: four accumulators, slot j
    // goes to accumulator j mod 4, the total is ((a0 + a1) + a2) + a3
    float acc[4][VL];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
      for (int i = 0; i < VL; i++) acc[a][i] = 0.f;
    // Eight gathered rows at a time: their loads are issued together, then folded in slot order.  (A plain loop
    // over the slots compiles to one load in flight per lane.)  Row and weight are the same in every lane: held in
    // scalar registers, the row address is scalar base + lane offset; slots past topk are skipped by branches the
    // whole wave takes, a dropped copy contributes the zeros the reference multiplies there.  Streaming loads: a
    // permuted row is read exactly once.
    for (int j0 = 0; j0 < topk; j0 += 8) {
      v4i raw[8];
      float pv[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const bool on = j0 + u < topk;
        const int r = on ? __builtin_amdgcn_readfirstlane(srow[on ? j0 + u : 0]) : -1;
        pv[u] = on ? __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(sprob[on ? j0 + u : 0]))) : 0.f;
        if (r >= 0) raw[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(y + (int64_t)r * H) + c);
        else raw[u] = v4i{0, 0, 0, 0};
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        if (j0 + u >= topk) break;
        float v[VL];
        if constexpr (kRowsF32) {
#pragma unroll
          for (int i = 0; i < 4; i++) v[i] = __int_as_float(raw[u][i]);
        } else {
          unpack8(raw[u], v);
        }
        // separate multiply and add (no FMA contraction): the reference multiplies, rounds the
        // product to the promoted dtype, then sums
#pragma unroll
        for (int i = 0; i < VL; i += 2) {
          float p0 = v[i], p1 = v[i + 1];
          if constexpr (kRoundProducts) {
            const uint32_t pk = pack_bf16x2(v[i] * pv[u], v[i + 1] * pv[u]);
            p0 = __uint_as_float(pk << 16);
            p1 = __uint_as_float(pk & 0xffff0000u);
          } else if constexpr (PD != AAMD_NONE) {
            p0 = v[i] * pv[u];
            p1 = v[i + 1] * pv[u];
          }
          acc[u & 3][i] = acc[u & 3][i] + p0;  // slot j0 + u, j0 a multiple of 8
          acc[u & 3][i + 1] = acc[u & 3][i + 1] + p1;
        }
      }
    }
    float tot[VL];
#pragma unroll
    for (int i = 0; i < VL; i++) tot[i] = ((acc[0][i] + acc[1][i]) + acc[2][i]) + acc[3][i];
    if constexpr (kOutF32) {
      float* dst = reinterpret_cast<float*>(out) + t * H + c * VL;
      // streaming stores: 5 % faster than plain ones here
      __builtin_nontemporal_store(v4f{tot[0], tot[1], tot[2], tot[3]}, reinterpret_cast<v4f*>(dst));
      if constexpr (VL == 8) __builtin_nontemporal_store(v4f{tot[4], tot[5], tot[6], tot[7]}, reinterpret_cast<v4f*>(dst) + 1);
    } else {
      if constexpr (VL == 8) {
        v4i w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (int)pack_bf16x2(tot[2 * i], tot[2 * i + 1]);
        __builtin_nontemporal_store(w, reinterpret_cast<v4i*>(reinterpret_cast<u16*>(out) + t * H + c * 8));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// plain row permute: 16-byte chunks, each source row read once and written topk times
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void permute_rows_kernel(const v4i* __restrict__ x, int chunks,
                                                           const int32_t* __restrict__ row_map, int topk,
                                                           int64_t M_out, v4i* __restrict__ out) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
    const v4i v = __builtin_nontemporal_load(x + t * chunks + c);
    for (int j = 0; j < topk; j++) {
      const int64_t dst = row_map[t * topk + j];
      if (dst >= 0 && dst < M_out) __builtin_nontemporal_store(v, out + dst * chunks + c);
    }
  }
}

// ---------------------------------------------------------------------------------------
// row permute with a weight per copy and a conversion: out[row_map[t*k+j]] = OUT(x[t] * probs[t, j]).
// The gradient of the combine with respect to the permuted rows (what autograd makes of the
// multiply in token_dispatcher.py:156-158: the product in the promoted type, cast to the rows' type).
// ---------------------------------------------------------------------------------------
template <typename IN, typename OUT, int PD>
__global__ __launch_bounds__(256) void permute_rows_scaled_kernel(const typename IN::elem* __restrict__ x, int64_t cols,
                                                                  const int32_t* __restrict__ row_map, int topk,
                                                                  const void* __restrict__ probs, int64_t M_out,
                                                                  typename OUT::elem* __restrict__ out) {
  const int64_t t = blockIdx.x;
  for (int64_t c = (int64_t)threadIdx.x * 8; c < cols; c += (int64_t)blockDim.x * 8) {
    float v[8];
    if constexpr (std::is_same<IN, F32>::value) {
      const v4f a = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x + t * cols + c));
      const v4f b = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x + t * cols + c) + 1);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        v[i] = a[i];
        v[4 + i] = b[i];
      }
    } else {
      unpack8(__builtin_nontemporal_load(reinterpret_cast<const v4i*>(x + t * cols + c)), v);
    }
    for (int j = 0; j < topk; j++) {
      const int64_t dst = row_map[t * topk + j];
      if (dst < 0 || dst >= M_out) continue;
      float pv = 1.f;
      if constexpr (PD == AAMD_BF16) pv = bf16_bits_to_f32(reinterpret_cast<const u16*>(probs)[t * topk + j]);
      if constexpr (PD == AAMD_F32) pv = reinterpret_cast<const float*>(probs)[t * topk + j];
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; i++) o[i] = v[i] * pv;
      if constexpr (std::is_same<OUT, F32>::value) {
        __builtin_nontemporal_store(v4f{o[0], o[1], o[2], o[3]}, reinterpret_cast<v4f*>(out + dst * cols + c));
        __builtin_nontemporal_store(v4f{o[4], o[5], o[6], o[7]}, reinterpret_cast<v4f*>(out + dst * cols + c) + 1);
      } else {
        v4i w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (int)pack_bf16x2(o[2 * i], o[2 * i + 1]);
        __builtin_nontemporal_store(w, reinterpret_cast<v4i*>(out + dst * cols + c));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// gradient of the combine with respect to the weights: dprobs[t, j] = <dout[t], y[row_map[t*k+j]]>
// (fp32 products and sums).  One workgroup per token, as in the combine: a lane holds 8 columns of dout per trip
// over the row, the gathers of up to eight slots are issued together, every lane keeps their partial sums, and the
// workgroup reduces them once at the end (lanes of a wave by shuffles, waves in a fixed order through the LDS).
// H8: columns / 8.
// ---------------------------------------------------------------------------------------
template <typename DT, typename YT>
__global__ __launch_bounds__(1024) void unpermute_probs_grad_kernel(const typename DT::elem* __restrict__ dout,
                                                                    const typename YT::elem* __restrict__ y, int64_t M,
                                                                    int H8, const int32_t* __restrict__ row_map,
                                                                    int topk, float* __restrict__ dprobs) {
  constexpr bool kYF32 = std::is_same<YT, F32>::value;
  __shared__ int srow[kMaxTopk];
  __shared__ float red[16][kMaxTopk];
  const int64_t t = blockIdx.x;
  const int wave = (int)threadIdx.x >> 6, nwaves = (int)blockDim.x >> 6;
  if ((int)threadIdx.x < topk) {
    const int r = row_map[t * topk + threadIdx.x];
    srow[threadIdx.x] = r >= 0 && r < M ? r : -1;  // a dropped copy: gradient 0
  }
  __syncthreads();
  const int64_t H = (int64_t)H8 * 8;
  for (int j0 = 0; j0 < topk; j0 += 8) {
    float part[8];
#pragma unroll
    for (int u = 0; u < 8; u++) part[u] = 0.f;
    for (int c = threadIdx.x; c < H8; c += blockDim.x) {
      float a[8];
      if constexpr (std::is_same<DT, F32>::value) {
        const v4f lo = *reinterpret_cast<const v4f*>(dout + t * H + (int64_t)c * 8);
        const v4f hi = *(reinterpret_cast<const v4f*>(dout + t * H + (int64_t)c * 8) + 1);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          a[i] = lo[i];
          a[4 + i] = hi[i];
        }
      } else {
        unpack8(*reinterpret_cast<const v4i*>(dout + t * H + (int64_t)c * 8), a);
      }
      v4i raw[8][kYF32 ? 2 : 1];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        // the row is the same in every lane (scalar base + lane offset); slots past topk and dropped copies are
        // skipped by a branch the whole wave takes
        const int r = j0 + u < topk ? __builtin_amdgcn_readfirstlane(srow[j0 + u < topk ? j0 + u : 0]) : -1;
        const v4i* src = reinterpret_cast<const v4i*>(y + (int64_t)(r < 0 ? 0 : r) * H + (int64_t)c * 8);
#pragma unroll
        for (int w = 0; w < (kYF32 ? 2 : 1); w++) {
          if (r >= 0) raw[u][w] = __builtin_nontemporal_load(src + w);
          else raw[u][w] = v4i{0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        if (j0 + u >= topk) break;
        float b[8];
        if constexpr (kYF32) {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            b[i] = __int_as_float(raw[u][0][i]);
            b[4 + i] = __int_as_float(raw[u][kYF32 ? 1 : 0][i]);
          }
        } else {
          unpack8(raw[u][0], b);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) part[u] = part[u] + a[i] * b[i];
      }
    }
#pragma unroll
    for (int u = 0; u < 8; u++) {
      if (j0 + u >= topk) break;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) part[u] += __shfl_xor(part[u], off);
      if ((threadIdx.x & 63) == 0) red[wave][j0 + u] = part[u];
    }
  }
  __syncthreads();
  if ((int)threadIdx.x < topk) {
    float sum = 0.f;
    for (int w = 0; w < nwaves; w++) sum += red[w][threadIdx.x];
    dprobs[t * topk + threadIdx.x] = sum;
  }
}

// ---------------------------------------------------------------------------------------
// inverse permutation
// ---------------------------------------------------------------------------------------
__global__ void fill_i32_kernel(int32_t* __restrict__ p, int64_t n, int32_t v) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
__global__ void invert_permutation_kernel(const int64_t* __restrict__ sorted_idx, int64_t n_perm, int64_t n_flat,
                                          int32_t* __restrict__ row_map) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j < n_perm) {
    const int64_t f = sorted_idx[j];
    if (f >= 0 && f < n_flat) row_map[f] = (int32_t)j;
  }
}

// ---------------------------------------------------------------------------------------
// router preprocess: stable counting sort by expert id.
//   chunk  = 1024 consecutive flat indices handled by one workgroup (4 rounds of 256)
//   hist   [E][nchunk]: ids of expert e in chunk b            (kernel 1)
//   scan   rows of hist -> exclusive prefix along chunks, row totals      (kernel 2)
//   goff   exclusive prefix of the row totals                              (kernel 3)
//   place  position = goff[e] + hist_prefix[e][b] + rank inside the chunk  (kernel 4)
// ---------------------------------------------------------------------------------------
constexpr int kChunk = 1024;

template <typename ID>
__device__ __forceinline__ int load_id(const ID* ids, int64_t i, int64_t n, int E) {
  if (i >= n) return -1;
  const int64_t e = (int64_t)ids[i];
  return (e >= 0 && e < E) ? (int)e : -1;  // out-of-range ids are dropped (row_map -1)
}

template <typename ID>
__global__ __launch_bounds__(256) void route_hist_kernel(const ID* __restrict__ ids, int64_t n, int E, int nchunk,
                                                         int32_t* __restrict__ hist) {
  extern __shared__ int cnt[];
  for (int e = threadIdx.x; e < E; e += 256) cnt[e] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kChunk;
#pragma unroll
  for (int it = 0; it < kChunk / 256; it++) {
    const int e = load_id(ids, base + it * 256 + threadIdx.x, n, E);
    if (e >= 0) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256) hist[(int64_t)e * nchunk + blockIdx.x] = cnt[e];
}

__global__ __launch_bounds__(256) void route_rowscan_kernel(int32_t* __restrict__ hist, int nchunk,
                                                            int32_t* __restrict__ totals) {
  __shared__ int buf[256];
  __shared__ int carry;
  int32_t* row = hist + (int64_t)blockIdx.x * nchunk;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < nchunk; base += 256) {
    const int i = base + threadIdx.x;
    const int v = i < nchunk ? row[i] : 0;
    buf[threadIdx.x] = v;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
      const int t = (int)threadIdx.x >= d ? buf[threadIdx.x - d] : 0;
      __syncthreads();
      buf[threadIdx.x] += t;
      __syncthreads();
    }
    if (i < nchunk) row[i] = carry + buf[threadIdx.x] - v;
    __syncthreads();
    if (threadIdx.x == 255) carry += buf[255];
    __syncthreads();
  }
  if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

__global__ __launch_bounds__(256) void route_goff_kernel(const int32_t* __restrict__ totals, int E,
                                                         int64_t* __restrict__ goff) {
  __shared__ int buf[256];
  __shared__ long long carry;
  if (threadIdx.x == 0) {
    carry = 0;
    goff[0] = 0;
  }
  __syncthreads();
  for (int base = 0; base < E; base += 256) {
    const int e = base + threadIdx.x;
    buf[threadIdx.x] = e < E ? totals[e] : 0;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
      const int t = (int)threadIdx.x >= d ? buf[threadIdx.x - d] : 0;
      __syncthreads();
      buf[threadIdx.x] += t;
      __syncthreads();
    }
    if (e < E) goff[e + 1] = carry + buf[threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 255) carry += buf[255];
    __syncthreads();
  }
}

template <typename ID>
__global__ __launch_bounds__(256) void route_place_kernel(const ID* __restrict__ ids, int64_t n, int E, int nchunk,
                                                          const int32_t* __restrict__ hist,
                                                          const int64_t* __restrict__ goff,
                                                          int64_t* __restrict__ sorted_idx,
                                                          int32_t* __restrict__ row_map) {
  // slot = round * 4 + wave, 16 slots of 64 consecutive flat indices each
  extern __shared__ int h[];  // [16][E]
  constexpr int kSlots = kChunk / 64;
  for (int i = threadIdx.x; i < kSlots * E; i += 256) h[i] = 0;
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t base = (int64_t)blockIdx.x * kChunk;
  int eid[kChunk / 256], rank[kChunk / 256];
#pragma unroll
  for (int it = 0; it < kChunk / 256; it++) {
    const int e = load_id(ids, base + it * 256 + threadIdx.x, n, E);
    // lanes of this wave holding the same expert id
    unsigned long long peers = __ballot(e >= 0);
    if (e < 0) peers = ~peers;
    for (int b = 0; (1 << b) < E; b++) {
      const unsigned long long vote = __ballot((e >> b) & 1);
      peers &= ((e >> b) & 1) ? vote : ~vote;
    }
    const unsigned long long below = peers & ((1ull << lane) - 1ull);
    eid[it] = e;
    rank[it] = __popcll(below);
    if (e >= 0 && below == 0) h[(it * 4 + wave) * E + e] = __popcll(peers);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256) {
    int64_t run = goff[e] + hist[(int64_t)e * nchunk + blockIdx.x];
    for (int sl = 0; sl < kSlots; sl++) {
      const int c = h[sl * E + e];
      h[sl * E + e] = (int)run;
      run += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < kChunk / 256; it++) {
    const int64_t flat = base + it * 256 + threadIdx.x;
    if (flat >= n) continue;
    if (eid[it] < 0) {
      row_map[flat] = -1;
      continue;
    }
    const int pos = h[(it * 4 + wave) * E + eid[it]] + rank[it];
    row_map[flat] = pos;
    if (sorted_idx) sorted_idx[pos] = flat;
  }
}

// ---------------------------------------------------------------------------------------
// Per-expert bias on expert-tagged rows: out[t] = inp[t] + bias[bin_ids[t]] and its bias gradient
// ---------------------------------------------------------------------------------------
template <typename ID>
__global__ __launch_bounds__(256) void bias_gather_add_kernel(const v4i* __restrict__ inp, const v4i* __restrict__ bias,
                                                              const ID* __restrict__ bin_ids, int64_t chunks, int row_chunks,
                                                              int E, bool is_bf16, v4i* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= chunks) return;
  const int64_t t = i / row_chunks;
  const int c = (int)(i - t * row_chunks);
  const int64_t e = (int64_t)bin_ids[t];
  const v4i a = __builtin_nontemporal_load(inp + i);
  v4i r = a;
  if (e >= 0 && e < E) {
    const v4i b = bias[e * row_chunks + c];
    if (is_bf16) {
      float fa[8], fb[8];
      unpack8(a, fa);
      unpack8(b, fb);
#pragma unroll
      for (int k = 0; k < 4; k++) r[k] = (int)pack_bf16x2(fa[2 * k] + fb[2 * k], fa[2 * k + 1] + fb[2 * k + 1]);
    } else {
#pragma unroll
      for (int k = 0; k < 4; k++) r[k] = __float_as_int(__int_as_float(a[k]) + __int_as_float(b[k]));
    }
  }
  __builtin_nontemporal_store(r, out + i);
}

__global__ __launch_bounds__(256) void fill_zero_f32_kernel(float* __restrict__ p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// bgrad[e, :] += sum of the rows tagged e.  A workgroup walks rows_per_wg consecutive rows (a multiple of 8, chosen
// by the launcher); a thread owns one 16-byte chunk of columns and keeps the running sum of the current expert in
// registers, so rows grouped by expert cost one set of atomics per workgroup and expert.
constexpr int kBgRowsMin = 32, kBgRowsMax = 4096;
template <typename ID>
__global__ __launch_bounds__(512) void bias_gather_bgrad_kernel(const v4i* __restrict__ grad, const ID* __restrict__ bin_ids,
                                                                int64_t T, int row_chunks, int E, bool is_bf16,
                                                                float* __restrict__ bgrad, int rows_per_wg) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= row_chunks) return;
  const int64_t t0 = (int64_t)blockIdx.y * rows_per_wg;
  const int64_t t1 = t0 + rows_per_wg < T ? t0 + rows_per_wg : T;
  const int W = is_bf16 ? 8 : 4;  // columns per chunk
  float acc[8];
#pragma unroll
  for (int k = 0; k < 8; k++) acc[k] = 0.f;
  int64_t cur = -1;
  auto flush = [&]() {
    if (cur < 0 || cur >= E) return;
    float* dst = bgrad + cur * (int64_t)row_chunks * W + (int64_t)c * W;
    for (int k = 0; k < W; k++) atomicAdd(dst + k, acc[k]);
  };
  constexpr int B = 8;  // rows in flight per thread
  for (int64_t tb = t0; tb < t1; tb += B) {
    v4i g[B];
    int64_t e[B];
#pragma unroll
    for (int u = 0; u < B; u++) {
      const int64_t t = tb + u < t1 ? tb + u : t1 - 1;
      e[u] = tb + u < t1 ? (int64_t)bin_ids[t] : -2;  // -2: past the end, skipped below
      g[u] = __builtin_nontemporal_load(grad + t * row_chunks + c);
    }
#pragma unroll
    for (int u = 0; u < B; u++) {
      if (e[u] == -2) continue;
      if (e[u] != cur) {
        flush();
#pragma unroll
        for (int k = 0; k < 8; k++) acc[k] = 0.f;
        cur = e[u];
      }
      if (is_bf16) {
        float f[8];
        unpack8(g[u], f);
#pragma unroll
        for (int k = 0; k < 8; k++) acc[k] += f[k];
      } else {
#pragma unroll
        for (int k = 0; k < 4; k++) acc[k] += __int_as_float(g[u][k]);
      }
    }
  }
  flush();
}

}  // namespace aamd

using namespace aamd;

// Workgroup size for kernels that walk a row in 16-byte chunks, one chunk per lane and trip: 256 lanes unless
// another multiple of 64 leaves fewer lanes idle in the last trip (7168 columns of bf16 are 896 chunks: 448 lanes
// make two full trips, 256 would leave the fourth half empty).
static int threads_for_row_chunks(int64_t chunks) {
  int threads = 256;
  int64_t waste = (chunks + 255) / 256 * 256 - chunks;
  for (int b = 512; b >= 128; b -= 64) {
    const int64_t w = (chunks + b - 1) / b * b - chunks;
    if (w < waste) { waste = w; threads = b; }
  }
  return threads;
}

// Workgroup size for the one-workgroup-per-token kernels, a lane handling one chunk of the row per trip: as few
// trips as 1024 lanes allow, the lanes spread evenly over them, so that all the loads of a token are in flight at
// once (7168 columns of bf16 in 16-byte chunks: 896 lanes and one trip; the combine runs at 74 % of the HBM rate
// that way against 68 % with two trips of 448 lanes).
static int threads_for_one_row(int64_t chunks) {
  if (chunks <= 64) return 64;
  const int64_t trips = (chunks + 1023) / 1024;
  return (int)(((chunks + trips - 1) / trips + 63) / 64 * 64);
}

extern "C" int aamd_bias_gather_add(const void* inp, const void* bias, const void* bin_ids, int ids_are_i64, int64_t T,
                                    int64_t H, int E, int dtype, void* out, void* stream) {
  AAMD_REQUIRE(dtype == AAMD_BF16 || dtype == AAMD_F32, "bias_gather_add: unsupported dtype %d", dtype);
  const int64_t row_bytes = H * (dtype == AAMD_BF16 ? 2 : 4);
  AAMD_REQUIRE(T >= 0 && H >= 0 && E >= 1 && row_bytes % 16 == 0, "bias_gather_add: row size must be a multiple of 16 bytes");
  if (T == 0 || H == 0) return AAMD_OK;
  AAMD_REQUIRE(inp && bias && bin_ids && out, "bias_gather_add: null pointer");
  AAMD_REQUIRE(((uintptr_t)inp & 15) == 0 && ((uintptr_t)bias & 15) == 0 && ((uintptr_t)out & 15) == 0,
               "bias_gather_add: pointers must be 16-byte aligned");
  const int64_t rc = row_bytes / 16, chunks = T * rc;
  AAMD_REQUIRE(rc < 0x7fffffffLL && (chunks + 255) / 256 < 0x7fffffffLL, "bias_gather_add: too large");
  const unsigned blocks = (unsigned)((chunks + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (ids_are_i64)
    bias_gather_add_kernel<int64_t><<<blocks, 256, 0, st>>>((const v4i*)inp, (const v4i*)bias, (const int64_t*)bin_ids, chunks,
                                                            (int)rc, E, dtype == AAMD_BF16, (v4i*)out);
  else
    bias_gather_add_kernel<int32_t><<<blocks, 256, 0, st>>>((const v4i*)inp, (const v4i*)bias, (const int32_t*)bin_ids, chunks,
                                                            (int)rc, E, dtype == AAMD_BF16, (v4i*)out);
  AAMD_LAUNCH_CHECK("bias_gather_add");
  return AAMD_OK;
}

extern "C" int aamd_bias_gather_add_bgrad(const void* grad, const void* bin_ids, int ids_are_i64, int64_t T, int64_t H,
                                          int E, int dtype, float* bgrad, void* stream) {
  AAMD_REQUIRE(dtype == AAMD_BF16 || dtype == AAMD_F32, "bias_gather_add_bgrad: unsupported dtype %d", dtype);
  const int64_t row_bytes = H * (dtype == AAMD_BF16 ? 2 : 4);
  AAMD_REQUIRE(T >= 0 && H >= 0 && E >= 1 && row_bytes % 16 == 0,
               "bias_gather_add_bgrad: row size must be a multiple of 16 bytes");
  if (H == 0) return AAMD_OK;
  AAMD_REQUIRE(bgrad != nullptr, "bias_gather_add_bgrad: null output");
  hipStream_t st = (hipStream_t)stream;
  const int64_t n = (int64_t)E * H;
  AAMD_REQUIRE((n + 255) / 256 < 0x7fffffffLL, "bias_gather_add_bgrad: too large");
  fill_zero_f32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(bgrad, n);  // a kernel, so callers may capture it
  AAMD_LAUNCH_CHECK("bias_gather_add_bgrad (clear)");
  if (T == 0) return AAMD_OK;
  AAMD_REQUIRE(grad && bin_ids, "bias_gather_add_bgrad: null pointer");
  AAMD_REQUIRE(((uintptr_t)grad & 15) == 0, "bias_gather_add_bgrad: grad must be 16-byte aligned");
  const int64_t rc = row_bytes / 16;
  const int threads = threads_for_row_chunks(rc);
  // Rows per workgroup: every workgroup ends with one atomic add per column and expert it met, and those adds, not
  // the reads, bound the launch when workgroups are short (128 rows each: 63 % of the HBM rate on 524288 x 7168
  // bf16; 4096 rows each: 84 %).  About one workgroup per CU keeps enough loads in flight (half as many: 63 % again).
  const int64_t col_blocks = (rc + threads - 1) / threads;
  int64_t rows_per_wg = T * col_blocks / 256 / 8 * 8;
  rows_per_wg = rows_per_wg < kBgRowsMin ? kBgRowsMin : rows_per_wg > kBgRowsMax ? kBgRowsMax : rows_per_wg;
  const int64_t row_blocks = (T + rows_per_wg - 1) / rows_per_wg;
  AAMD_REQUIRE(rc < 0x7fffffffLL && row_blocks <= 65535, "bias_gather_add_bgrad: more than 65535 * 4096 rows");
  dim3 grid((unsigned)col_blocks, (unsigned)row_blocks), block((unsigned)threads);
  if (ids_are_i64)
    bias_gather_bgrad_kernel<int64_t><<<grid, block, 0, st>>>((const v4i*)grad, (const int64_t*)bin_ids, T, (int)rc, E,
                                                              dtype == AAMD_BF16, bgrad, (int)rows_per_wg);
  else
    bias_gather_bgrad_kernel<int32_t><<<grid, block, 0, st>>>((const v4i*)grad, (const int32_t*)bin_ids, T, (int)rc, E,
                                                              dtype == AAMD_BF16, bgrad, (int)rows_per_wg);
  AAMD_LAUNCH_CHECK("bias_gather_add_bgrad");
  return AAMD_OK;
}

extern "C" int aamd_unpermute_combine(const void* y, int y_dtype, int64_t M, int64_t H, const int32_t* row_map,
                                      const void* probs, int probs_dtype, int64_t T, int topk, void* out,
                                      void* stream) {
  AAMD_REQUIRE(y_dtype == AAMD_BF16 || y_dtype == AAMD_F32, "unpermute_combine: unsupported row dtype %d", y_dtype);
  AAMD_REQUIRE(probs_dtype == AAMD_NONE || probs_dtype == AAMD_BF16 || probs_dtype == AAMD_F32,
               "unpermute_combine: unsupported probs dtype %d", probs_dtype);
  AAMD_REQUIRE(M >= 0 && H >= 0 && T >= 0 && H % 8 == 0, "unpermute_combine: H=%lld must be a multiple of 8",
               (long long)H);
  AAMD_REQUIRE(topk >= 1 && topk <= kMaxTopk, "unpermute_combine: topk=%d out of range [1, %d]", topk, kMaxTopk);
  AAMD_REQUIRE(M < 0x7fffffffLL && T < 0x7fffffffLL, "unpermute_combine: too many rows");
  if (T == 0 || H == 0) return AAMD_OK;
  AAMD_REQUIRE(row_map && out && (y || M == 0), "unpermute_combine: null pointer");
  AAMD_REQUIRE(probs_dtype == AAMD_NONE || probs != nullptr, "unpermute_combine: probs missing");
  AAMD_REQUIRE(((uintptr_t)y & 15) == 0 && ((uintptr_t)out & 15) == 0, "unpermute_combine: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  // one workgroup per token, one 16-byte chunk of the row per lane and trip
  dim3 grid((unsigned)T), block((unsigned)threads_for_one_row(H / (y_dtype == AAMD_BF16 ? 8 : 4)));
  if (y_dtype == AAMD_BF16) {
    const int H8 = (int)(H / 8);
    if (probs_dtype == AAMD_BF16)
      unpermute_combine_kernel<BF16, AAMD_BF16><<<grid, block, 0, st>>>((const u16*)y, M, H8, row_map, probs, topk, out);
    else if (probs_dtype == AAMD_F32)
      unpermute_combine_kernel<BF16, AAMD_F32><<<grid, block, 0, st>>>((const u16*)y, M, H8, row_map, probs, topk, out);
    else
      unpermute_combine_kernel<BF16, AAMD_NONE><<<grid, block, 0, st>>>((const u16*)y, M, H8, row_map, probs, topk, out);
  } else {
    const int H4 = (int)(H / 4);
    if (probs_dtype == AAMD_BF16)
      unpermute_combine_kernel<F32, AAMD_BF16><<<grid, block, 0, st>>>((const float*)y, M, H4, row_map, probs, topk, out);
    else if (probs_dtype == AAMD_F32)
      unpermute_combine_kernel<F32, AAMD_F32><<<grid, block, 0, st>>>((const float*)y, M, H4, row_map, probs, topk, out);
    else
      unpermute_combine_kernel<F32, AAMD_NONE><<<grid, block, 0, st>>>((const float*)y, M, H4, row_map, probs, topk, out);
  }
  AAMD_LAUNCH_CHECK("unpermute_combine");
  return AAMD_OK;
}

extern "C" int aamd_permute_rows_scaled(const void* x, int x_dtype, int64_t T, int64_t cols, const int32_t* row_map,
                                        int topk, const void* probs, int probs_dtype, int64_t M_out, void* out,
                                        int out_dtype, void* stream) {
  AAMD_REQUIRE((x_dtype == AAMD_BF16 || x_dtype == AAMD_F32) && (out_dtype == AAMD_BF16 || out_dtype == AAMD_F32),
               "permute_rows_scaled: unsupported dtype %d -> %d", x_dtype, out_dtype);
  AAMD_REQUIRE(!(x_dtype == AAMD_BF16 && out_dtype == AAMD_F32), "permute_rows_scaled: bf16 -> fp32 is not a case of the combine's gradient");
  AAMD_REQUIRE(probs_dtype == AAMD_NONE || probs_dtype == AAMD_BF16 || probs_dtype == AAMD_F32,
               "permute_rows_scaled: unsupported probs dtype %d", probs_dtype);
  AAMD_REQUIRE(T >= 0 && cols >= 0 && cols % 8 == 0, "permute_rows_scaled: cols=%lld must be a multiple of 8", (long long)cols);
  AAMD_REQUIRE(topk >= 1 && M_out >= 0 && T < 0x7fffffffLL, "permute_rows_scaled: bad topk / sizes");
  if (T == 0 || cols == 0) return AAMD_OK;
  AAMD_REQUIRE(x && out && row_map && (probs || probs_dtype == AAMD_NONE), "permute_rows_scaled: null pointer");
  AAMD_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0, "permute_rows_scaled: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  // (write bound: 256 lanes and several trips over the row measured faster at top-8 than one trip of up to 1024)
  dim3 grid((unsigned)T), block(256);
#define AAMD_PRS(IN_, OUT_, PD_)                                                                                          \
  permute_rows_scaled_kernel<IN_, OUT_, PD_><<<grid, block, 0, st>>>((const IN_::elem*)x, cols, row_map, topk, probs, M_out, \
                                                                     (OUT_::elem*)out)
#define AAMD_PRS_P(IN_, OUT_)                                  \
  do {                                                         \
    if (probs_dtype == AAMD_BF16) AAMD_PRS(IN_, OUT_, AAMD_BF16); \
    else if (probs_dtype == AAMD_F32) AAMD_PRS(IN_, OUT_, AAMD_F32); \
    else AAMD_PRS(IN_, OUT_, AAMD_NONE);                        \
  } while (0)
  if (x_dtype == AAMD_BF16) AAMD_PRS_P(BF16, BF16);
  else if (out_dtype == AAMD_BF16) AAMD_PRS_P(F32, BF16);
  else AAMD_PRS_P(F32, F32);
#undef AAMD_PRS_P
#undef AAMD_PRS
  AAMD_LAUNCH_CHECK("permute_rows_scaled");
  return AAMD_OK;
}

extern "C" int aamd_unpermute_probs_grad(const void* dout, int dout_dtype, const void* y, int y_dtype, int64_t M, int64_t H,
                                         const int32_t* row_map, int64_t T, int topk, float* dprobs, void* stream) {
  AAMD_REQUIRE((dout_dtype == AAMD_BF16 || dout_dtype == AAMD_F32) && (y_dtype == AAMD_BF16 || y_dtype == AAMD_F32),
               "unpermute_probs_grad: unsupported dtype");
  AAMD_REQUIRE(M >= 0 && H >= 0 && T >= 0 && H % 8 == 0, "unpermute_probs_grad: H=%lld must be a multiple of 8", (long long)H);
  AAMD_REQUIRE(topk >= 1 && topk <= kMaxTopk && T < 0x7fffffffLL, "unpermute_probs_grad: bad topk / sizes");
  if (T == 0) return AAMD_OK;
  AAMD_REQUIRE(dout && row_map && dprobs && (y || M == 0), "unpermute_probs_grad: null pointer");
  AAMD_REQUIRE(((uintptr_t)y & 15) == 0 && ((uintptr_t)dout & 15) == 0, "unpermute_probs_grad: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (M == 0) {  // every copy was dropped: no row to read (y may be null)
    const int64_t n = T * topk;
    AAMD_REQUIRE((n + 255) / 256 < 0x7fffffffLL, "unpermute_probs_grad: too large");
    fill_zero_f32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(dprobs, n);
    AAMD_LAUNCH_CHECK("unpermute_probs_grad (clear)");
    return AAMD_OK;
  }
  const int H8 = (int)(H / 8);
  dim3 grid((unsigned)T), block((unsigned)threads_for_one_row(H8));
  if (dout_dtype == AAMD_BF16 && y_dtype == AAMD_BF16)
    unpermute_probs_grad_kernel<BF16, BF16><<<grid, block, 0, st>>>((const u16*)dout, (const u16*)y, M, H8, row_map, topk, dprobs);
  else if (dout_dtype == AAMD_F32 && y_dtype == AAMD_BF16)
    unpermute_probs_grad_kernel<F32, BF16><<<grid, block, 0, st>>>((const float*)dout, (const u16*)y, M, H8, row_map, topk, dprobs);
  else if (dout_dtype == AAMD_F32 && y_dtype == AAMD_F32)
    unpermute_probs_grad_kernel<F32, F32><<<grid, block, 0, st>>>((const float*)dout, (const float*)y, M, H8, row_map, topk, dprobs);
  else
    unpermute_probs_grad_kernel<BF16, F32><<<grid, block, 0, st>>>((const u16*)dout, (const float*)y, M, H8, row_map, topk, dprobs);
  AAMD_LAUNCH_CHECK("unpermute_probs_grad");
  return AAMD_OK;
}

extern "C" int aamd_permute_rows(const void* x, int x_dtype, int64_t T, int64_t cols, const int32_t* row_map,
                                 int topk, int64_t M_out, void* out, void* stream) {
  AAMD_REQUIRE(x_dtype == AAMD_BF16 || x_dtype == AAMD_F32, "permute_rows: unsupported dtype %d", x_dtype);
  const int64_t row_bytes = cols * (x_dtype == AAMD_BF16 ? 2 : 4);
  AAMD_REQUIRE(T >= 0 && cols >= 0 && row_bytes % 16 == 0, "permute_rows: row size must be a multiple of 16 bytes");
  AAMD_REQUIRE(topk >= 1 && M_out >= 0 && T < 0x7fffffffLL, "permute_rows: bad topk / sizes");
  if (T == 0 || cols == 0) return AAMD_OK;
  AAMD_REQUIRE(x && out && row_map, "permute_rows: null pointer");
  AAMD_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0, "permute_rows: pointers must be 16-byte aligned");
  permute_rows_kernel<<<(unsigned)T, 256, 0, (hipStream_t)stream>>>((const v4i*)x, (int)(row_bytes / 16), row_map, topk,
                                                                    M_out, (v4i*)out);
  AAMD_LAUNCH_CHECK("permute_rows");
  return AAMD_OK;
}

extern "C" int aamd_invert_permutation(const int64_t* sorted_idx, int64_t n_perm, int64_t n_flat, int32_t* row_map,
                                       void* stream) {
  AAMD_REQUIRE(n_perm >= 0 && n_flat >= 0 && n_perm <= n_flat, "invert_permutation: bad sizes");
  AAMD_REQUIRE(n_flat < 0x7fffffffLL, "invert_permutation: too many rows");
  if (n_flat == 0) return AAMD_OK;
  AAMD_REQUIRE(row_map && (sorted_idx || n_perm == 0), "invert_permutation: null pointer");
  hipStream_t st = (hipStream_t)stream;
  if (n_perm < n_flat) {
    fill_i32_kernel<<<(unsigned)((n_flat + 255) / 256), 256, 0, st>>>(row_map, n_flat, -1);
    AAMD_LAUNCH_CHECK("fill_i32");
  }
  if (n_perm > 0) {
    invert_permutation_kernel<<<(unsigned)((n_perm + 255) / 256), 256, 0, st>>>(sorted_idx, n_perm, n_flat, row_map);
    AAMD_LAUNCH_CHECK("invert_permutation");
  }
  return AAMD_OK;
}

extern "C" int64_t aamd_moe_preprocess_ws_ints(int64_t n, int E) {
  if (n < 0 || E < 1) return 0;
  const int64_t nchunk = (n + kChunk - 1) / kChunk;
  return (int64_t)E * (nchunk > 0 ? nchunk : 1) + E;
}

extern "C" int aamd_moe_preprocess(const void* expert_ids, int ids_are_i64, int64_t n, int E, int64_t* sorted_idx,
                                   int32_t* row_map, int64_t* group_offsets, int32_t* ws, void* stream) {
  AAMD_REQUIRE(n >= 0 && n < 0x7fffffffLL, "moe_preprocess: n out of range");
  AAMD_REQUIRE(E >= 1 && E <= 1024, "moe_preprocess: E=%d out of range [1, 1024]", E);
  AAMD_REQUIRE(group_offsets && ws, "moe_preprocess: group_offsets / ws required");
  AAMD_REQUIRE(n == 0 || (expert_ids && row_map), "moe_preprocess: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const int nchunk = (int)((n + kChunk - 1) / kChunk);
  const int nc = nchunk > 0 ? nchunk : 1;
  int32_t* hist = ws;
  int32_t* totals = ws + (int64_t)E * nc;
  if (nchunk == 0) {
    fill_i32_kernel<<<(unsigned)((E + 255) / 256), 256, 0, st>>>(hist, E, 0);
    AAMD_LAUNCH_CHECK("fill_i32");
  } else if (ids_are_i64) {
    route_hist_kernel<int64_t><<<nchunk, 256, E * sizeof(int), st>>>((const int64_t*)expert_ids, n, E, nc, hist);
  } else {
    route_hist_kernel<int32_t><<<nchunk, 256, E * sizeof(int), st>>>((const int32_t*)expert_ids, n, E, nc, hist);
  }
  AAMD_LAUNCH_CHECK("route_hist");
  route_rowscan_kernel<<<E, 256, 0, st>>>(hist, nc, totals);
  AAMD_LAUNCH_CHECK("route_rowscan");
  route_goff_kernel<<<1, 256, 0, st>>>(totals, E, group_offsets);
  AAMD_LAUNCH_CHECK("route_goff");
  if (nchunk > 0) {
    const size_t sh = (size_t)(kChunk / 64) * E * sizeof(int);
    if (ids_are_i64)
      route_place_kernel<int64_t><<<nchunk, 256, sh, st>>>((const int64_t*)expert_ids, n, E, nc, hist, group_offsets, sorted_idx, row_map);
    else
      route_place_kernel<int32_t><<<nchunk, 256, sh, st>>>((const int32_t*)expert_ids, n, E, nc, hist, group_offsets, sorted_idx, row_map);
    AAMD_LAUNCH_CHECK("route_place");
  }
  return AAMD_OK;
}
