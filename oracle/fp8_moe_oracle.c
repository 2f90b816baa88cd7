/*
 * CPU oracle for the FP8 grouped-linear MoE expert path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is a scalar restatement of the
 * reference arithmetic; nothing in the shipped package may link, import or
 * call it.  Only the test-suite, the smoke check and the CPU-baseline leg of
 * the benchmark use it, and only as the checker.
 *
 * Every function cites the reference file:line it restates (paths relative
 * to the reference tree root).  The e4m3fn encoder is written with integer
 * arithmetic only so that it is independent of any library cast; the tests
 * pin it against torch's CPU cast over all 2^16 bf16 patterns and against an
 * exact rational-arithmetic rounder.
 *
 * Parity status: what pins each function (tests/test_oracle.py, tests/test_golden.py)
 *   oracle_f32_to_e4m3fn / oracle_e4m3fn_to_f32   pinned: torch's CPU cast on all 2^16 bf16 patterns and
 *       10^6 random fp32 values, an exact rational rounder on ties / subnormals / the 448-464-465 edge,
 *       round trip over all 256 codes
 *   f32_to_bf16                                   pinned: torch's cast on 2*10^5 random values
 *   oracle_tile_quant / oracle_block_quant        pinned: closed form s = fl(max(amax,eps)/448) and exact
 *       rational rounding of fl(x/s); the reference tests' known answers (zeros, ones, 1000, -512, the 1e4
 *       outlier); independent torch restatement; error bound; transpose and row-permutation invariants
 *   oracle_tile_quant_t_grouped                   pinned: equals tile quant of the zero padded transpose of
 *       each group (torch restatement), partial tiles and empty groups included
 *   oracle_fp8_gemm                               pinned: float64 dequantise-and-matmul (library routine),
 *       pure-Python brute force in the reference's accumulation order, linearity / accumulate,
 *       grouped == per-expert loop, fp64 autograd of the unquantised problem (roles and transposes)
 *   oracle_permute_indices                        pinned: torch.argsort(stable=True), bincount
 *   oracle_swiglu_bf16                            pinned: torch's CPU F.silu and multiply on bf16 tensors, bit for
 *       bit over every finite bf16 a; closed forms silu(0) = 0, silu(x) -> x and -> -0 for large |x|;
 *       h == b * silu(a) in double within two bf16 roundings
 *   oracle_swiglu_bwd_bf16                        pinned: torch's CPU autograd of the same two ops, bit for bit
 *       over every finite bf16 a; float64 central differences; da(0) = dh b / 2, db = dh silu(a)
 *   oracle_bias_gather_add / _bgrad               pinned: torch's inp + bias[ids] bit for bit, index_add_ in
 *       float64, integer-valued data whose fp32 sums are exact in any order
 *   oracle_unpermute_combine                      pinned: brute force, torch restatement (index_copy_,
 *       multiply, sum) bit-exact for bf16 weights, inverse-of-permute property; the summation order
 *       (four interleaved accumulators) is pinned against torch's own sum on the GPU by a GPU test
 * Parity unpinned (nothing available here can pin it; the oracle's choice is stated instead):
 *   - the exact fp32 rounding of the reference's compiled Triton division x / s on its GPU: the oracle
 *     is defined as IEEE round-to-nearest division;
 *   - the numerics and layouts of the external `kitchen` package behind quantize_op (not in the
 *     reference tree, no version pinned): the in-tree Triton formulas are the anchor instead.
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off -shared -fPIC (see Makefile).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define TILE 128

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even (what torch's .to(bfloat16) does). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40); /* quiet NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/*
 * fp32 -> OCP e4m3fn code, round to nearest even, NOT saturating: magnitudes
 * that round above 448 become NaN (0x7f), as torch's CPU cast does.  This is
 * the `y.to(y_ptr.dtype.element_ty)` step of
 * atorch/modules/fp8/triton_kernel.py:36 and :122.
 */
uint8_t oracle_f32_to_e4m3fn(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 31) << 7);
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return (uint8_t)(sign | 0x7f); /* inf, NaN -> NaN */
    uint32_t exp = a >> 23;
    uint32_t man = a & 0x7fffffu;
    if (exp == 0) return sign; /* fp32 zero / subnormal: far below 2^-10 */
    int E = (int)exp - 127;
    if (E >= -6) {
        uint32_t m = man >> 20;
        uint32_t rem = man & 0xfffffu;
        if (rem > 0x80000u || (rem == 0x80000u && (m & 1u))) m++;
        if (m == 8) {
            m = 0;
            E++;
        }
        if (E > 8 || (E == 8 && m == 7)) return (uint8_t)(sign | 0x7f);
        return (uint8_t)(sign | ((uint32_t)(E + 7) << 3) | m);
    }
    /* result is subnormal in e4m3fn: quantum 2^-9 */
    int shift = 14 - E; /* >= 21 */
    if (shift > 24) return sign; /* < 2^-10: rounds to zero */
    uint32_t full = man | 0x800000u;
    uint32_t q = full >> shift;
    uint32_t rem = full & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint8_t)(sign | q); /* q == 8 is the smallest normal, 0x08 */
}

/* e4m3fn code -> fp32 (exact). Used by dequant: triton_kernel.py:58-60,74-76. */
float oracle_e4m3fn_to_f32(uint8_t c) {
    uint32_t e = (c >> 3) & 0xf, m = c & 7;
    float v;
    if (e == 0xf && m == 7) return NAN;
    if (e == 0)
        v = ldexpf((float)m, -9);
    else
        v = ldexpf((float)(8 + m), (int)e - 10);
    return (c & 0x80) ? -v : v;
}

void oracle_e4m3fn_to_f32_array(const uint8_t *c, int64_t n, float *out) {
    for (int64_t i = 0; i < n; i++) out[i] = oracle_e4m3fn_to_f32(c[i]);
}
void oracle_f32_to_e4m3fn_array(const float *x, int64_t n, uint8_t *out) {
    for (int64_t i = 0; i < n; i++) out[i] = oracle_f32_to_e4m3fn(x[i]);
}
void oracle_bf16_to_f32_array(const uint16_t *x, int64_t n, float *out) {
    for (int64_t i = 0; i < n; i++) out[i] = bf16_to_f32(x[i]);
}
void oracle_f32_to_bf16_array(const float *x, int64_t n, uint16_t *out) {
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_bf16(x[i]);
}

/* s = max(amax, eps) / 448 ; s == 0 -> 1   (triton_kernel.py:31-33, 106-108) */
static inline float scale_from_amax(float amax, float eps) {
    float s = fmaxf(amax, eps) / 448.0f;
    if (s == 0.0f) s = 1.0f;
    return s;
}

/*
 * 1x128 tile quantisation (atorch/modules/fp8/triton_kernel.py:94-140):
 * x [rows, cols] fp32 (the kernel casts its input to fp32 first, :105),
 * cols % 128 == 0 (:135); q [rows, cols] codes, s [rows, cols/128] fp32.
 */
int oracle_tile_quant(const float *x, int64_t rows, int64_t cols, float eps, uint8_t *q, float *s) {
    if (cols % TILE) return 1;
    int64_t nt = cols / TILE;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t t = 0; t < nt; t++) {
            const float *p = x + r * cols + t * TILE;
            float amax = 0.0f;
            for (int j = 0; j < TILE; j++) amax = fmaxf(amax, fabsf(p[j]));
            float sc = scale_from_amax(amax, eps);
            s[r * nt + t] = sc;
            for (int j = 0; j < TILE; j++) q[r * cols + t * TILE + j] = oracle_f32_to_e4m3fn(p[j] / sc);
        }
    return 0;
}

/*
 * 128x128 block quantisation (triton_kernel.py:21-46): x [N, K] fp32, both
 * multiples of 128 (scale tensor is [N//128, K//128], :43).
 */
int oracle_block_quant(const float *x, int64_t N, int64_t K, float eps, uint8_t *q, float *s) {
    if (N % TILE || K % TILE) return 1;
    int64_t nb = N / TILE, kb = K / TILE;
    for (int64_t bi = 0; bi < nb; bi++)
        for (int64_t bj = 0; bj < kb; bj++) {
            float amax = 0.0f;
            for (int i = 0; i < TILE; i++)
                for (int j = 0; j < TILE; j++)
                    amax = fmaxf(amax, fabsf(x[(bi * TILE + i) * K + bj * TILE + j]));
            float sc = scale_from_amax(amax, eps);
            s[bi * kb + bj] = sc;
            for (int i = 0; i < TILE; i++)
                for (int j = 0; j < TILE; j++) {
                    int64_t o = (bi * TILE + i) * K + bj * TILE + j;
                    q[o] = oracle_f32_to_e4m3fn(x[o] / sc);
                }
        }
    return 0;
}

/*
 * Transposed 1x128 quantisation of ragged groups.  The in-tree definition is
 * tile_quant(x_i.t().contiguous()) (atorch/modules/fp8/scaled_linear.py:402-414,
 * 431-446); a partial last token tile (M_i % 128 != 0) is zero padded, i.e.
 * amax runs over the valid tokens only.
 *
 * x [M, R] fp32 row major, splits[E] rows per group (sum = M).
 * Padded column offset of group i: poff_i = sum_{j<i} ceil(M_j/128)*128.
 * q_t [R, ld_t] codes, q_t[r, poff_i + m] = code(x[off_i + m, r]); pad
 *      columns inside a group's padded range are written as 0.
 * s_t [ld_t/128 (at least poff_E/128), R] fp32, s_t[poff_i/128 + m/128, r].
 */
int oracle_tile_quant_t_grouped(const float *x, int64_t M, int64_t R, const int64_t *splits, int64_t E,
                                float eps, uint8_t *q_t, float *s_t, int64_t ld_t) {
    int64_t off = 0, poff = 0;
    for (int64_t g = 0; g < E; g++) {
        int64_t Mi = splits[g];
        int64_t nb = (Mi + TILE - 1) / TILE;
        if (poff + nb * TILE > ld_t) return 2;
        for (int64_t b = 0; b < nb; b++) {
            int64_t m0 = b * TILE, m1 = m0 + TILE < Mi ? m0 + TILE : Mi;
            for (int64_t r = 0; r < R; r++) {
                float amax = 0.0f;
                for (int64_t m = m0; m < m1; m++) amax = fmaxf(amax, fabsf(x[(off + m) * R + r]));
                float sc = scale_from_amax(amax, eps);
                s_t[(poff / TILE + b) * R + r] = sc;
                for (int64_t m = m0; m < m0 + TILE; m++)
                    q_t[r * ld_t + poff + m] = m < m1 ? oracle_f32_to_e4m3fn(x[(off + m) * R + r] / sc) : 0;
            }
        }
        off += Mi;
        poff += nb * TILE;
    }
    return off == M ? 0 : 3;
}

/*
 * Block-scaled fp8 GEMM, arithmetic definition of triton_kernel.py:151-195:
 *   C[m,n] = sum_kb ( dot(A[m,kb], B[n,kb]) * a_s[m,kb] * b_s[n/div,kb] )
 * with the product order (dot * a_s) * b_s then += into an fp32 accumulator
 * (:185).  The 128-long dot is summed exactly (in double: every product of
 * two e4m3 values is a multiple of 2^-18 below 2^18, so 128 of them fit 53
 * bits) and rounded to fp32 once - tl.dot's own summation order is not
 * defined, so this is the order-free ideal of it.
 *
 * a [M, lda] codes (K valid), a_s element (m,kb) at a_s[m*as_rs + kb*as_cs];
 * b [N, ldb] codes, b_s element (n/b_div, kb) at b_s[(n/b_div)*bs_rs + kb*bs_cs];
 * b_div = 128 for block-scaled B, 1 for tile-scaled B (:167,177,208).
 * c [M, ldc] fp32.  accumulate != 0 adds into c.
 */
int oracle_fp8_gemm(const uint8_t *a, int64_t lda, const float *a_s, int64_t as_rs, int64_t as_cs,
                    const uint8_t *b, int64_t ldb, const float *b_s, int64_t bs_rs, int64_t bs_cs,
                    int64_t b_div, int64_t M, int64_t N, int64_t K, float *c, int64_t ldc, int accumulate) {
    if (K % TILE) return 1;
    static float lut[256];
    static int lut_ok = 0;
    if (!lut_ok) {
        for (int i = 0; i < 256; i++) lut[i] = oracle_e4m3fn_to_f32((uint8_t)i);
        lut_ok = 1;
    }
    int64_t nkb = K / TILE;
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int64_t kb = 0; kb < nkb; kb++) {
                const uint8_t *pa = a + m * lda + kb * TILE, *pb = b + n * ldb + kb * TILE;
                double d = 0.0;
                for (int j = 0; j < TILE; j++) d += (double)lut[pa[j]] * (double)lut[pb[j]];
                float dot = (float)d;
                acc += dot * a_s[m * as_rs + kb * as_cs] * b_s[(n / b_div) * bs_rs + kb * bs_cs];
            }
            if (accumulate)
                c[m * ldc + n] += acc;
            else
                c[m * ldc + n] = acc;
        }
    return 0;
}

/*
 * permute (atorch/modules/moe/token_dispatcher.py:89-116): stable argsort of
 * the flattened [T, topk] expert ids.  sorted_idx[j] = flat (token*topk+slot)
 * index of permuted row j; the permuted row is tokens[sorted_idx[j] / topk].
 * counts[E] receives tokens per expert (the histc of :310).
 */
int oracle_permute_indices(const int64_t *ids, int64_t n, int64_t E, int64_t *sorted_idx, int64_t *counts) {
    int64_t *pos = (int64_t *)calloc((size_t)E + 1, sizeof(int64_t));
    if (!pos) return 4;
    for (int64_t i = 0; i < n; i++) {
        if (ids[i] < 0 || ids[i] >= E) {
            free(pos);
            return 1;
        }
        pos[ids[i] + 1]++;
    }
    for (int64_t e = 0; e < E; e++) {
        counts[e] = pos[e + 1];
        pos[e + 1] += pos[e];
    }
    for (int64_t i = 0; i < n; i++) sorted_idx[pos[ids[i]]++] = i;
    free(pos);
    return 0;
}

/*
 * unpermute + weighted combine (token_dispatcher.py:119-161) on bf16 data:
 *   buf = zeros[M,H]; buf[sorted_idx[j]] = y[j]            (:146-155)
 *   buf.reshape(T,k,H) * probs[T,k,1]                      (:156-158) -> each
 *       product rounded to the promoted dtype
 *   .sum(dim=1)                                            (:159) -> fp32
 *       accumulate, one final rounding
 * probs_is_bf16: probs bf16 -> products and result bf16 (out_bf16 written);
 * else probs fp32 -> products and result fp32 (out_f32 written).
 * The fp32 accumulation follows torch's GPU reduction of a strided dimension, which is what the
 * reference executes: four accumulators, slot j goes to accumulator j mod 4 in slot order, then
 * ((a0 + a1) + a2) + a3.  (For k <= 4 that is the plain left-to-right sum.)  A GPU test checks this
 * order against torch's own sum on the device.
 * probs == NULL: topk = 1, plain inverse permutation (:141-144).
 * n_perm may be smaller than T*k (rows dropped): missing rows count as 0.
 */
int oracle_unpermute_combine(const uint16_t *y, int64_t n_perm, int64_t H, const int64_t *sorted_idx,
                             const void *probs, int probs_is_bf16, int64_t T, int64_t k, uint16_t *out_bf16,
                             float *out_f32) {
    int64_t n_flat = T * k;
    int64_t *inv = (int64_t *)malloc((size_t)n_flat * sizeof(int64_t));
    if (!inv) return 4;
    for (int64_t i = 0; i < n_flat; i++) inv[i] = -1;
    for (int64_t j = 0; j < n_perm; j++) {
        if (sorted_idx[j] < 0 || sorted_idx[j] >= n_flat) {
            free(inv);
            return 1;
        }
        inv[sorted_idx[j]] = j;
    }
    for (int64_t t = 0; t < T; t++)
        for (int64_t h = 0; h < H; h++) {
            float acc4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int64_t j = 0; j < k; j++) {
                int64_t row = inv[t * k + j];
                float v = row < 0 ? 0.0f : bf16_to_f32(y[row * H + h]);
                if (probs) {
                    if (probs_is_bf16) {
                        float p = bf16_to_f32(((const uint16_t *)probs)[t * k + j]);
                        v = bf16_to_f32(f32_to_bf16(v * p));
                    } else {
                        v = v * ((const float *)probs)[t * k + j];
                    }
                }
                acc4[j & 3] += v;
            }
            const float acc = ((acc4[0] + acc4[1]) + acc4[2]) + acc4[3];
            if (probs && !probs_is_bf16)
                out_f32[t * H + h] = acc;
            else
                out_bf16[t * H + h] = f32_to_bf16(acc);
        }
    free(inv);
    return 0;
}

/*
 * Per-expert bias on expert-tagged rows, atorch/kernels/triton_jit/bias_gather_add.py:24-47 (forward:
 * out[t] = inp[t] + bias[bin_ids[t]], in the tensors' dtype: a bf16 sum is the fp32 sum rounded) and
 * :80-98 (backward: bgrad[e] = fp32 sum of the rows tagged e; the reference adds atomically in no
 * fixed order, here in row order).  is_bf16 selects bf16 bit patterns or fp32 for inp / bias / out / grad.
 */
int oracle_bias_gather_add(const void *inp, const void *bias, const int64_t *bin_ids, int64_t T, int64_t H, int E,
                           int is_bf16, void *out) {
    if (T < 0 || H < 0 || E < 1) return 1;
    for (int64_t t = 0; t < T; t++) {
        const int64_t e = bin_ids[t];
        if (e < 0 || e >= E) return 2;
        for (int64_t c = 0; c < H; c++) {
            if (is_bf16) {
                const float a = bf16_to_f32(((const uint16_t *)inp)[t * H + c]);
                const float b = bf16_to_f32(((const uint16_t *)bias)[e * H + c]);
                ((uint16_t *)out)[t * H + c] = f32_to_bf16(a + b);
            } else {
                ((float *)out)[t * H + c] = ((const float *)inp)[t * H + c] + ((const float *)bias)[e * H + c];
            }
        }
    }
    return 0;
}

int oracle_bias_gather_bgrad(const void *grad, const int64_t *bin_ids, int64_t T, int64_t H, int E, int is_bf16,
                             float *bgrad) {
    if (T < 0 || H < 0 || E < 1) return 1;
    for (int64_t i = 0; i < (int64_t)E * H; i++) bgrad[i] = 0.0f;
    for (int64_t t = 0; t < T; t++) {
        const int64_t e = bin_ids[t];
        if (e < 0 || e >= E) return 2;
        for (int64_t c = 0; c < H; c++) {
            const float g = is_bf16 ? bf16_to_f32(((const uint16_t *)grad)[t * H + c]) : ((const float *)grad)[t * H + c];
            bgrad[e * H + c] += g;
        }
    }
    return 0;
}

/*
 * SwiGLU of rows [a | b] (bf16 bit patterns), atorch/modules/moe/grouped_gemm_moe.py:331-334:
 * torch.chunk(x, 2, -1); F.silu(x[0]) * x[1].  Two torch ops on bf16 tensors: silu is evaluated in
 * fp32 as x / (1 + exp(-x)) and rounded to bf16, the product is formed in fp32 and rounded to bf16.
 * The fp32 formula is followed operation by operation with a correctly rounded expf (so exp(-x)
 * overflows to inf, and silu to -0, below about -88.7 as it does in fp32); an implementation whose
 * expf is off by an ulp may differ by one bf16 unit in the last place on rare inputs.
 */
int oracle_swiglu_bf16(const uint16_t *fc1, int64_t rows, int64_t F, int64_t ld, uint16_t *h) {
    if (rows < 0 || F < 0 || ld < 2 * F) return 1;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < F; c++) {
            const float a = bf16_to_f32(fc1[r * ld + c]);
            const float b = bf16_to_f32(fc1[r * ld + F + c]);
            const float e = (float)exp(-(double)a); /* correctly rounded expf; overflows to inf like fp32 */
            const float sl32 = a / (1.0f + e);
            const float sl = bf16_to_f32(f32_to_bf16(sl32));
            h[r * F + c] = f32_to_bf16(sl * b);
        }
    return 0;
}

/*
 * Backward of the same two torch ops under autograd (grouped_gemm_moe.py:331-334 differentiated:
 * mul backward, then silu_backward), all tensors bf16:
 *   db = bf16(dh * bf16(silu(a)))                       grad of the product w.r.t. b: dh * saved silu output
 *   g  = bf16(dh * b)                                   grad w.r.t. the silu output
 *   da = bf16(g * sig * (1 + a * (1 - sig))),  sig = 1 / (1 + exp(-a))   silu_backward, fp32 inside,
 * evaluated left to right as torch's kernel writes it: (g * sig) * (1 + a * (1 - sig)).
 * dfc1 rows are [da | db] like fc1's [a | b].  Correctly rounded expf as in oracle_swiglu_bf16.
 */
int oracle_swiglu_bwd_bf16(const uint16_t *dh, const uint16_t *fc1, int64_t rows, int64_t F, int64_t ld,
                           uint16_t *dfc1) {
    if (rows < 0 || F < 0 || ld < 2 * F) return 1;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < F; c++) {
            const float a = bf16_to_f32(fc1[r * ld + c]);
            const float b = bf16_to_f32(fc1[r * ld + F + c]);
            const float d = bf16_to_f32(dh[r * F + c]);
            const float e = (float)exp(-(double)a);
            const float sl = bf16_to_f32(f32_to_bf16(a / (1.0f + e)));
            const float sig = 1.0f / (1.0f + e);
            const float g = bf16_to_f32(f32_to_bf16(d * b));
            const float t = g * sig;
            const float u = 1.0f + a * (1.0f - sig);
            dfc1[r * 2 * F + c] = f32_to_bf16(t * u);
            dfc1[r * 2 * F + F + c] = f32_to_bf16(d * sl);
        }
    return 0;
}
