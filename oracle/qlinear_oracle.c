/*
 * CPU oracle for the quantized-Linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic the reference's x86 CPU backend
 * performs for a Linear layer with Q4_0 / Q8_0 weights, plus closed-form
 * restatements of the W4A16 (group-128, zero-point) and W8A8 (per-token dynamic)
 * paths and of the MoE expert loop.  It is the checker the GPU kernels are
 * compared against.  Nothing in the shipped library links, loads or calls it:
 * only tests, the smoke check and the benchmark's cpu_baseline leg may.
 *
 * Every function cites the reference file:line it follows (paths are relative
 * to the reference checkout root).
 *
 * Pinning status (what independently fixes each function; see tests/test_oracle_*.py):
 *   orc_fp16_to_fp32 / orc_fp32_to_fp16      exhaustive vs numpy float16 and vs the compiled reference macros
 *   orc_x86_scale_bits                       exhaustive (65 536 patterns) vs the compiled reference's store/load round trip
 *   orc_quantize_row_q8_0                    bit-exact vs the compiled reference quantize_row_q8_0 (AVX2 branch)
 *   orc_dequantize_row_q4_0 / _q8_0          bit-exact vs the compiled reference
 *   orc_vec_dot_q4_0_q8_0 / _q8_0_q8_0       bit-exact vs the compiled reference vec_dot_* (same 8-lane fma + hsum order)
 *   orc_linear_q                             composition of the above; llamafile_sgemm itself is unbuildable here
 *                                            (needs fmt through mllm/utils/Common.hpp), its tile kernel is restated and
 *                                            pinned through vec_dot (identical lane layout, fma and hsum) and a double
 *                                            precision brute force
 *   orc_w4a16_*  orc_w8a8_*  orc_per_token_quant_int8
 *                                            the reference has no CPU implementation (CUDA-only third-party kernels):
 *                                            parity unpinned by the reference; pinned here by the closed forms its tests
 *                                            state, brute force in int64/float64 and special cases
 *   orc_moe_ffn                              composition + permutation invariance + hand-built micro case
 *   orc_exp_poly / orc_silu_array / orc_rmsnorm / orc_softmax_rows / orc_topk_rows / orc_moe_gate
 *                                            the x86 kernels they restate need Highway, which the reference does not
 *                                            vendor: unbuildable here.  Pinned by closed forms in float64 (exp_poly
 *                                            against exp(x) * exp(n * 2.1219444e-4), which is what the reference's
 *                                            reduction constants produce; rmsnorm, softmax, silu against their
 *                                            definitions), by numpy sort for top-k, and by the properties the reference's
 *                                            own TopK test checks (shapes of tests/cpu/KernelTest.cpp:686, descending order)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK 32
#define ORC_API __attribute__((visibility("default")))

enum { ORC_Q4_0 = 0, ORC_Q8_0 = 1 };
enum { ORC_SCALE_IEEE = 0, ORC_SCALE_X86_REF = 1 };

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ------------------------------------------------------------------------------------------------
 * fp16 <-> fp32.  The x86 reference uses F16C: _cvtsh_ss / _cvtss_sh(x, 0) (round to nearest even)
 * mllm/backends/cpu/kernels/common/ggml/quantize/quantize.hpp:108-109
 * ---------------------------------------------------------------------------------------------- */
ORC_API float orc_fp16_to_fp32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff;
  if (e == 0) {
    float v = (float)m * 0x1p-24f; /* subnormal or zero: exact */
    return sign ? -v : v;
  }
  if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

ORC_API uint16_t orc_fp32_to_fp16(float f) {
  uint32_t x = f2u(f);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  x &= 0x7fffffffu;
  if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x3ffu)); /* NaN -> quiet NaN */
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                        /* >= 65520 rounds to inf */
  if (x < 0x38800000u) {                                                          /* below 2^-14: subnormal half */
    float v = u2f(x) * 0x1p24f;                                                   /* exact scaling */
    return (uint16_t)(sign | (uint16_t)lrintf(v));                                /* RNE in the default rounding mode */
  }
  uint32_t e = (x >> 23) - 112u, m = x & 0x7fffffu;
  uint32_t h = (e << 10) | (m >> 13), rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++; /* a carry into the exponent is the right answer */
  return (uint16_t)(sign | h);
}

/* bf16 helpers (the prefill paths take bf16 activations; the decode path up-casts bf16 exactly) */
ORC_API float orc_bf16_to_fp32(uint16_t b) { return u2f((uint32_t)b << 16); }
ORC_API uint16_t orc_fp32_to_bf16(float f) {
  uint32_t x = f2u(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

/* ------------------------------------------------------------------------------------------------
 * The x86 build of the reference stores a block scale through two mismatched types: the macro
 * MLLM_FP32_TO_FP16 yields the raw 16-bit pattern `b` as an integer (quantize.hpp:109,133), which is
 * assigned to a half_float::half field (mllm/core/DataTypes.hpp:26) -> the field holds the NUMBER b rounded
 * to half precision (11 significant bits, nearest even).  Reading goes half -> float -> uint16_t -> table
 * lookup (quantize.hpp:114-130), so the scale that takes part in the arithmetic is fp16_to_fp32(b') with
 * b' = RNE(b to 11 significant bits).  Patterns >= 65520 become +inf as a half; converting that to uint16_t
 * is undefined in C++ and never occurs for finite scales (b < 0x7c00), we return 0xffff for them.
 * ---------------------------------------------------------------------------------------------- */
ORC_API uint16_t orc_x86_scale_bits(uint16_t b) {
  if (b < 2048) return b;
  if (b >= 65520) return 0xffff;
  int p = 31 - __builtin_clz((unsigned)b); /* b in [2^p, 2^(p+1)) */
  int sh = p - 10;
  uint32_t q = b >> sh, rem = b & ((1u << sh) - 1u), half = 1u << (sh - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  return (uint16_t)(q << sh);
}

static inline float scale_value(uint16_t bits, int scale_mode) {
  return orc_fp16_to_fp32(scale_mode == ORC_SCALE_X86_REF ? orc_x86_scale_bits(bits) : bits);
}

/* ------------------------------------------------------------------------------------------------
 * Q8_0 activation quantization, AVX2 branch of quantize_row_q8_0
 * mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.cpp:106-190
 *   amax = max|x| ; d = amax/127 ; id = amax != 0 ? 127/amax : 0 ; q = int8_sat(rne(x*id)) ; d -> fp16 RNE
 * Output is structure-of-arrays: codes[k], scale bit patterns[k/32] as the F16C conversion produces them
 * (the x86 storage rounding is applied where the scale is USED, see scale_value()).
 * ---------------------------------------------------------------------------------------------- */
ORC_API void orc_quantize_row_q8_0(const float* x, int8_t* qs, uint16_t* d_bits, int k) {
  int nb = k / QK;
  for (int i = 0; i < nb; i++) {
    const float* xb = x + (size_t)i * QK;
    float amax = 0.0f;
    for (int j = 0; j < QK; j++) {
      float a = fabsf(xb[j]);
      amax = a > amax ? a : amax;
    }
    const float d = amax / 127.f;
    const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;
    d_bits[i] = orc_fp32_to_fp16(d);
    for (int j = 0; j < QK; j++) {
      float v = rintf(xb[j] * id); /* _mm256_round_ps(_MM_ROUND_NEAREST) = half to even */
      int q = (int)v;
      q = q > 127 ? 127 : (q < -128 ? -128 : q); /* packs_epi32 / packs_epi16 saturate */
      qs[(size_t)i * QK + j] = (int8_t)q;
    }
  }
}

/* ------------------------------------------------------------------------------------------------
 * Offline weight quantizers: fp32 rows -> reference blocks (array of 18 / 34-byte structs).
 *   Q4_0   quantize_row_q4_0_reference, mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q4.cpp:33-68
 *          max = the element of largest magnitude, WITH its sign ; d = max / -8 ; id = d ? 1/d : 0 ;
 *          code = min(15, (int8)(x*id + 8.5)) (truncation) ; element j in the low nibble of byte j, 16+j in the high one
 *   Q8_0   quantize_row_q8_0 (the same routine the activations go through), quantize_q8.cpp:106-190
 * The 2-byte scale field: scale_mode IEEE stores the fp16 pattern P of d; X86_REF stores what the x86 build of the
 * reference leaves in the file, the half-precision ENCODING OF THE NUMBER P (DataTypes.hpp:26 with quantize.hpp:108-134),
 * which a later x86 read turns into P rounded to 11 significant bits.  For a negative d (positive maximum) P >= 0x8000
 * and that rounding drops up to five low bits of the scale pattern.
 * Pinned: codes and decoded scale pattern bit-exact against the compiled reference (tests/test_oracle_vs_reference.py).
 * ---------------------------------------------------------------------------------------------- */
static uint16_t store_scale_field(uint16_t pattern, int scale_mode) {
  return scale_mode == ORC_SCALE_X86_REF ? orc_fp32_to_fp16((float)pattern) : pattern;
}
ORC_API void orc_quantize_row_q4_0(const float* x, uint8_t* blocks, int k, int scale_mode) {
  int nb = k / QK;
  for (int i = 0; i < nb; i++) {
    const float* xb = x + (size_t)i * QK;
    uint8_t* y = blocks + (size_t)i * 18;
    float amax = 0.0f, max = 0.0f;
    for (int j = 0; j < QK; j++) {
      const float v = xb[j];
      if (amax < fabsf(v)) {
        amax = fabsf(v);
        max = v;
      }
    }
    const float d = max / -8;
    const float id = d ? 1.0f / d : 0.0f;
    const uint16_t field = store_scale_field(orc_fp32_to_fp16(d), scale_mode);
    memcpy(y, &field, 2);
    for (int j = 0; j < QK / 2; j++) {
      const float x0 = xb[j] * id, x1 = xb[QK / 2 + j] * id;
      int q0 = (int8_t)(x0 + 8.5f), q1 = (int8_t)(x1 + 8.5f);
      q0 = q0 < 15 ? q0 : 15;
      q1 = q1 < 15 ? q1 : 15;
      y[2 + j] = (uint8_t)((uint8_t)q0 | ((uint8_t)q1 << 4));
    }
  }
}
ORC_API void orc_quantize_row_q8_0_blocks(const float* x, uint8_t* blocks, int k, int scale_mode) {
  int nb = k / QK;
  for (int i = 0; i < nb; i++) {
    int8_t qs[QK];
    uint16_t bits;
    orc_quantize_row_q8_0(x + (size_t)i * QK, qs, &bits, QK);
    const uint16_t field = store_scale_field(bits, scale_mode);
    memcpy(blocks + (size_t)i * 34, &field, 2);
    memcpy(blocks + (size_t)i * 34 + 2, qs, QK);
  }
}

/* Reference array-of-structures block layouts, mllm/core/DataTypes.hpp:110-121,164-170 (pack(1)):
 *   block_q4_0 = { fp16 d; uint8 qs[16] }  18 bytes; element j in the low nibble of qs[j], element j+16 in the high one
 *   block_q8_0 = { fp16 d; int8 qs[32] }   34 bytes
 * Here `d` is always the IEEE fp16 bit pattern. */
static inline uint16_t blk_d(const uint8_t* blk) { uint16_t d; memcpy(&d, blk, 2); return d; }
static inline int blk_bytes(int wtype) { return wtype == ORC_Q4_0 ? 18 : 34; }

static inline void unpack_block(const uint8_t* blk, int wtype, int8_t w[QK]) {
  if (wtype == ORC_Q4_0) {
    for (int j = 0; j < 16; j++) {
      w[j] = (int8_t)((blk[2 + j] & 0x0f) - 8);
      w[j + 16] = (int8_t)((blk[2 + j] >> 4) - 8);
    }
  } else {
    memcpy(w, blk + 2, QK);
  }
}

/* dequantize_row_q4_0: quantize_q4.cpp:74-93 ; dequantize_row_q8_0: quantize_q8.cpp:197-211 */
ORC_API void orc_dequantize_row(const uint8_t* blocks, int wtype, float* y, int k, int scale_mode) {
  int nb = k / QK, bb = blk_bytes(wtype);
  for (int i = 0; i < nb; i++) {
    const uint8_t* blk = blocks + (size_t)i * bb;
    float d = scale_value(blk_d(blk), scale_mode);
    int8_t w[QK];
    unpack_block(blk, wtype, w);
    for (int j = 0; j < QK; j++) y[(size_t)i * QK + j] = (float)w[j] * d;
  }
}

/* One weight row times one quantized activation row.
 *   vec_dot_q4_0_q8_0 (AVX2): ggml/vec_dot.cpp:132-162, helpers ggml/vec_dot.hpp:244-295
 *   vec_dot_q8_0_q8_0 (AVX2): ggml/vec_dot.cpp:1572-1593
 *   tinyBLAS_Q0_AVX::gemm   : llamafile/llamafile_sgemm.cpp:697-743 (identical per-output arithmetic)
 * Eight fp32 lanes; lane L holds sum_blocks fma(dW*dX, float(int32 sum of elements 4L..4L+3), lane) and the
 * horizontal sum is ((l0+l4)+(l2+l6)) + ((l1+l5)+(l3+l7)).  isum (optional) receives the exact per-block int32 sums. */
static float dot_row(const uint8_t* wrow, int wtype, const int8_t* xq, const uint16_t* xd, int nb, int scale_mode,
                     int32_t* isum) {
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int bb = blk_bytes(wtype);
  for (int b = 0; b < nb; b++) {
    const uint8_t* blk = wrow + (size_t)b * bb;
    int8_t w[QK];
    unpack_block(blk, wtype, w);
    const int8_t* xb = xq + (size_t)b * QK;
    const float d = scale_value(blk_d(blk), scale_mode) * scale_value(xd[b], scale_mode);
    int32_t tot = 0;
    for (int L = 0; L < 8; L++) {
      int32_t s = 0;
      for (int j = 0; j < 4; j++) s += (int32_t)w[4 * L + j] * (int32_t)xb[4 * L + j];
      tot += s;
      acc[L] = fmaf(d, (float)s, acc[L]);
    }
    if (isum) isum[b] = tot;
  }
  float t0 = acc[4] + acc[0], t1 = acc[5] + acc[1], t2 = acc[6] + acc[2], t3 = acc[7] + acc[3];
  float u0 = t0 + t2, u1 = t1 + t3;
  return u0 + u1;
}

ORC_API float orc_vec_dot(const uint8_t* wrow, int wtype, const int8_t* xq, const uint16_t* xd, int k, int scale_mode) {
  return dot_row(wrow, wtype, xq, xd, k / QK, scale_mode, NULL);
}

/* Exact per-block integer dot products isum[n][m][b] (the int32 accumulators the GPU must match bit for bit). */
ORC_API void orc_block_isums(const uint8_t* W, int wtype, const int8_t* xq, int M, int N, int K, int32_t* isum) {
  int nb = K / QK, bb = blk_bytes(wtype);
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; n++)
    for (int m = 0; m < M; m++)
      for (int b = 0; b < nb; b++) {
        int8_t w[QK];
        unpack_block(W + ((size_t)n * nb + b) * bb, wtype, w);
        const int8_t* xb = xq + ((size_t)m * nb + b) * QK;
        int32_t s = 0;
        for (int j = 0; j < QK; j++) s += (int32_t)w[j] * (int32_t)xb[j];
        isum[((size_t)n * M + m) * nb + b] = s;
      }
}

/* Quantized Linear as the x86 CPU backend runs it:
 *   CPULinearOp::forward -> ggml::mat_mul(x, W, y, bias, false, true)      backends/cpu/ops/LinearOp.cpp:100-128,282-288
 *   mat_mul: quantize every activation row to Q8_0, then llamafile_sgemm   ggml/matmul.cpp:148-206
 *   y[m][n] = bias[n] + hsum(...)                                          llamafile_sgemm.cpp:735-741
 * x fp32 [M][K]; W reference blocks [N][K/32]; bias fp32 [N] or NULL; y fp32 [M][N].
 * xq_out / xd_out (optional) receive the activation codes [M][K] and scale patterns [M][K/32]. */
ORC_API int orc_linear_q(const float* x, const uint8_t* W, int wtype, const float* bias, float* y, int M, int N, int K,
                         int scale_mode, int8_t* xq_out, uint16_t* xd_out) {
  if (K % QK != 0 || M < 0 || N < 0) return -1;
  int nb = K / QK, bb = blk_bytes(wtype);
  int8_t* xq = xq_out ? xq_out : (int8_t*)malloc((size_t)M * K);
  uint16_t* xd = xd_out ? xd_out : (uint16_t*)malloc((size_t)M * nb * 2);
  if (!xq || !xd) return -2;
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; m++) orc_quantize_row_q8_0(x + (size_t)m * K, xq + (size_t)m * K, xd + (size_t)m * nb, K);
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; n++) {
    const uint8_t* wrow = W + (size_t)n * nb * bb;
    for (int m = 0; m < M; m++) {
      float v = dot_row(wrow, wtype, xq + (size_t)m * K, xd + (size_t)m * nb, nb, scale_mode, NULL);
      y[(size_t)m * N + n] = bias ? bias[n] + v : v;
    }
  }
  if (!xq_out) free(xq);
  if (!xd_out) free(xd);
  return 0;
}

/* ------------------------------------------------------------------------------------------------
 * The same Linear with the vector instructions and the work split of the reference's x86 path: the form whose
 * speed stands for "the reference's CPU path" when it is timed next to the GPU.
 *   tinyBLAS_Q0_AVX<block_q4_0 | block_q8_0, block_q8_0, float>   llamafile/llamafile_sgemm.cpp:579-790
 *     mnpack (tile shapes of a 16-register build, VECTOR_REGISTERS == 16)      :588-695
 *     gemm<RM, RN>: jobs = tiles, duty = ceil(tiles / nth), thread ith takes jobs [duty * ith, duty * (ith + 1))   :697-705
 *       per block l:  Cv[j][i] = fmadd(set1(dW * dX), cvtepi32_ps(madd_epi16(1, maddubs_epi16(|w|, sign(x, w)))), Cv[j][i])
 *       C[ldc * (jj + j) + ii + i] = bias[ii + i] + hsum(Cv[j][i])                                                 :706-741
 *     loaders: Q4_0 nibbles -> bytes - 8 (denibble), Q8_0 as stored          :745-778
 *   called once per thread id under an OpenMP parallel-for over [0, threads)  ggml/matmul.cpp:197-206
 * Weights and activations are arrays of blocks as in the reference (the activations are repacked from this file's
 * structure-of-arrays quantizer output into block_q8_0 records first).  The scale of a block is read through
 * scale_value(), i.e. with the x86 build's storage rounding when scale_mode says so.
 * Every output goes through exactly the operations of dot_row() above (same eight lanes, same fused multiply-add, same
 * horizontal sum), so the two must agree bit for bit: tests/test_oracle_golden.py checks that.
 * ---------------------------------------------------------------------------------------------- */
#if defined(__AVX2__) && defined(__FMA__)
#include <immintrin.h>
#include <omp.h>

typedef struct {
  const uint8_t* A; /* weight blocks [m rows][k blocks] */
  const uint8_t* B; /* activation blocks (34 bytes each) [n rows][k blocks] */
  const float* bias;
  float* C;
  int64_t k, lda, ldb, ldc;
  int ith, nth, wtype, scale_mode, abytes;
} tb_q0;

static inline float tb_hsum(__m256 x) { /* llamafile_sgemm.cpp:161-177 */
  __m128 v = _mm_add_ps(_mm256_extractf128_ps(x, 1), _mm256_castps256_ps128(x));
  v = _mm_add_ps(v, _mm_movehl_ps(v, v));
  v = _mm_add_ss(v, _mm_movehdup_ps(v));
  return _mm_cvtss_f32(v);
}
static inline __m256i tb_load_w(const tb_q0* t, const uint8_t* blk) {
  if (t->wtype == ORC_Q4_0) { /* denibble(qs) - 8, :757,774-777 */
    __m128i x = _mm_loadu_si128((const __m128i*)(blk + 2));
    __m256i n = _mm256_and_si256(_mm256_set1_epi8(15), _mm256_insertf128_si256(_mm256_castsi128_si256(x), _mm_srli_epi16(x, 4), 1));
    return _mm256_sub_epi8(n, _mm256_set1_epi8(8));
  }
  return _mm256_loadu_si256((const __m256i*)(blk + 2));
}
static inline __m256 tb_updot(__m256i u, __m256i s) { /* :762-772, the branch without VNNI */
  return _mm256_cvtepi32_ps(_mm256_madd_epi16(_mm256_set1_epi16(1), _mm256_maddubs_epi16(u, s)));
}

#define TB_GEMM(RM, RN)                                                                                                  \
  static void tb_gemm_##RM##x##RN(const tb_q0* t, int64_t m0, int64_t m, int64_t n0, int64_t n) {                        \
    const int64_t ytiles = (m - m0) / RM, xtiles = (n - n0) / RN, tiles = xtiles * ytiles;                               \
    const int64_t duty = (tiles + t->nth - 1) / t->nth, start = duty * t->ith;                                           \
    int64_t end = start + duty;                                                                                          \
    if (end > tiles) end = tiles;                                                                                        \
    for (int64_t job = start; job < end; ++job) {                                                                        \
      const int64_t ii = m0 + job / xtiles * RM, jj = n0 + job % xtiles * RN;                                            \
      __m256 Cv[RN][RM];                                                                                                 \
      for (int j = 0; j < RN; ++j)                                                                                       \
        for (int i = 0; i < RM; ++i) Cv[j][i] = _mm256_setzero_ps();                                                     \
      for (int64_t l = 0; l < t->k; ++l)                                                                                 \
        for (int j = 0; j < RN; ++j)                                                                                     \
          for (int i = 0; i < RM; ++i) {                                                                                 \
            const uint8_t* ab = t->A + (t->lda * (ii + i) + l) * t->abytes;                                              \
            const uint8_t* bb = t->B + (t->ldb * (jj + j) + l) * 34;                                                     \
            const __m256i a = tb_load_w(t, ab), b = _mm256_loadu_si256((const __m256i*)(bb + 2));                        \
            const __m256 ud = tb_updot(_mm256_sign_epi8(a, a), _mm256_sign_epi8(b, a));                                  \
            const float d = scale_value(blk_d(ab), t->scale_mode) * scale_value(blk_d(bb), t->scale_mode);               \
            Cv[j][i] = _mm256_fmadd_ps(_mm256_set1_ps(d), ud, Cv[j][i]);                                                 \
          }                                                                                                              \
      for (int j = 0; j < RN; ++j)                                                                                       \
        for (int i = 0; i < RM; ++i) {                                                                                   \
          const float v = tb_hsum(Cv[j][i]);                                                                             \
          t->C[t->ldc * (jj + j) + (ii + i)] = t->bias ? t->bias[ii + i] + v : v;                                        \
        }                                                                                                                \
    }                                                                                                                    \
  }
TB_GEMM(4, 2) TB_GEMM(2, 4) TB_GEMM(3, 2) TB_GEMM(2, 3) TB_GEMM(4, 1) TB_GEMM(2, 2) TB_GEMM(1, 4) TB_GEMM(3, 1)
TB_GEMM(1, 3) TB_GEMM(2, 1) TB_GEMM(1, 2) TB_GEMM(1, 1)
#undef TB_GEMM

static void tb_mnpack(const tb_q0* t, int64_t m0, int64_t m, int64_t n0, int64_t n) { /* :588-695, VECTOR_REGISTERS == 16 */
  int64_t mc, nc;
  const int64_t dm = m - m0 < 4 ? m - m0 : 4, dn = n - n0 < 4 ? n - n0 : 4;
  switch ((int)((dm << 4) | dn)) {
    case 0x44: case 0x43: case 0x42: mc = 4; nc = 2; tb_gemm_4x2(t, m0, m, n0, n); break;
    case 0x34: case 0x24: mc = 2; nc = 4; tb_gemm_2x4(t, m0, m, n0, n); break;
    case 0x33: case 0x32: mc = 3; nc = 2; tb_gemm_3x2(t, m0, m, n0, n); break;
    case 0x23: mc = 2; nc = 3; tb_gemm_2x3(t, m0, m, n0, n); break;
    case 0x41: mc = 4; nc = 1; tb_gemm_4x1(t, m0, m, n0, n); break;
    case 0x22: mc = 2; nc = 2; tb_gemm_2x2(t, m0, m, n0, n); break;
    case 0x14: mc = 1; nc = 4; tb_gemm_1x4(t, m0, m, n0, n); break;
    case 0x31: mc = 3; nc = 1; tb_gemm_3x1(t, m0, m, n0, n); break;
    case 0x13: mc = 1; nc = 3; tb_gemm_1x3(t, m0, m, n0, n); break;
    case 0x21: mc = 2; nc = 1; tb_gemm_2x1(t, m0, m, n0, n); break;
    case 0x12: mc = 1; nc = 2; tb_gemm_1x2(t, m0, m, n0, n); break;
    case 0x11: mc = 1; nc = 1; tb_gemm_1x1(t, m0, m, n0, n); break;
    default: return;
  }
  const int64_t mp = m0 + (m - m0) / mc * mc, np = n0 + (n - n0) / nc * nc;
  tb_mnpack(t, mp, m, n0, np);
  tb_mnpack(t, m0, m, np, n);
}

/* x fp32 [M][K]; W reference blocks [N][K/32]; y fp32 [M][N]; nth threads as the op's `threads` option (default 8,
 * mllm/core/BaseOp.hpp:77).  work: M * (K/32) * 34 bytes for the activation blocks, or NULL (allocated per call, as
 * mat_mul allocates its temporary, ggml/matmul.cpp:148-153). */
ORC_API int orc_linear_q_tiles(const float* x, const uint8_t* W, int wtype, const float* bias, float* y, int M, int N, int K,
                               int scale_mode, int nth, uint8_t* work) {
  if (K % QK != 0 || M < 0 || N < 0 || nth < 1) return -1;
  const int nb = K / QK;
  uint8_t* B = work ? work : (uint8_t*)malloc((size_t)M * nb * 34 + 64);
  if (!B) return -2;
  /* quantize_row_q8_0 per activation row, rows spread over the threads (ggml/matmul.cpp:173-187) */
#pragma omp parallel for schedule(static) num_threads(nth)
  for (int mrow = 0; mrow < M; mrow++) {
    int8_t q[QK];
    uint16_t d;
    for (int b = 0; b < nb; b++) {
      orc_quantize_row_q8_0(x + (size_t)mrow * K + (size_t)b * QK, q, &d, QK);
      uint8_t* blk = B + ((size_t)mrow * nb + b) * 34;
      memcpy(blk, &d, 2);
      memcpy(blk + 2, q, QK);
    }
  }
#pragma omp parallel num_threads(nth)
  {
    tb_q0 t = {W, B, bias, y, nb, nb, nb, N, omp_get_thread_num(), omp_get_num_threads(), wtype, scale_mode, blk_bytes(wtype)};
    tb_mnpack(&t, 0, N, 0, M);
  }
  if (!work) free(B);
  return 0;
}
#else
ORC_API int orc_linear_q_tiles(const float* x, const uint8_t* W, int wtype, const float* bias, float* y, int M, int N, int K,
                               int scale_mode, int nth, uint8_t* work) {
  (void)nth; (void)work;
  return orc_linear_q(x, W, wtype, bias, y, M, N, K, scale_mode, NULL, NULL);
}
#endif

/* ------------------------------------------------------------------------------------------------
 * W4A16, group 128 along K, uint4 codes with uint4 zero-points and fp16 scales (AWQ/Marlin semantics):
 *   w = (q - zp) * scale, computed in the activation dtype   mllm-kernel/mllm_kernel/cuda/csrc/gemm/marlin/dequant.h:18-26,
 *                                                            marlin_template.h:153-168
 *   test formula (q - 8) * scale for the symmetric variant   mllm-kernel/tests/test_gptq_marlin.py:143-146
 * Canonical restatement used by the GPU kernel and by this oracle:
 *   w_bf16[n][k] = bf16_rne( float(q[n][k] - zp[n][k/128]) * fp16_to_fp32(s[n][k/128]) )
 *   C[m][n]      = bf16_rne( sum_k float(A[m][k]) * float(w_bf16[n][k]) )      (products are exact in fp32)
 * The sum is taken in double here (order-free anchor); the kernel accumulates in fp32.
 * Storage: qw u8 [N][K/2], element 2j in the low nibble of byte j; zp u8 [N][ceil(G/2)], group 2g low nibble;
 * s fp16 bits [N][G], G = K/128.
 * ---------------------------------------------------------------------------------------------- */
static inline int nib(const uint8_t* p, size_t i) { return (i & 1) ? (p[i >> 1] >> 4) : (p[i >> 1] & 0x0f); }

ORC_API void orc_w4a16_dequant(const uint8_t* qw, const uint16_t* s, const uint8_t* zp, int N, int K, int group,
                               uint16_t* w_bf16) {
  int G = K / group, zpb = (G + 1) / 2;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; n++)
    for (int k = 0; k < K; k++) {
      int g = k / group;
      int q = nib(qw + (size_t)n * (K / 2), (size_t)k);
      int z = nib(zp + (size_t)n * zpb, (size_t)g);
      float w = (float)(q - z) * orc_fp16_to_fp32(s[(size_t)n * G + g]);
      w_bf16[(size_t)n * K + k] = orc_fp32_to_bf16(w);
    }
}

ORC_API int orc_w4a16_gemm(const uint16_t* A_bf16, const uint8_t* qw, const uint16_t* s, const uint8_t* zp,
                           const uint16_t* bias_bf16, uint16_t* C_bf16, int M, int N, int K, int group) {
  if (K % group != 0 || K % 2 != 0) return -1;
  uint16_t* w = (uint16_t*)malloc((size_t)N * K * 2);
  float* af = (float*)malloc((size_t)M * K * 4);
  if (!w || !af) return -2;
  orc_w4a16_dequant(qw, s, zp, N, K, group, w);
  for (size_t i = 0; i < (size_t)M * K; i++) af[i] = orc_bf16_to_fp32(A_bf16[i]);
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; n++) {
    float* wf = (float*)malloc((size_t)K * 4);
    for (int k = 0; k < K; k++) wf[k] = orc_bf16_to_fp32(w[(size_t)n * K + k]);
    for (int m = 0; m < M; m++) {
      double acc = 0.0;
      const float* a = af + (size_t)m * K;
      for (int k = 0; k < K; k++) acc += (double)a[k] * (double)wf[k];
      float r = (float)acc;
      if (bias_bf16) r += orc_bf16_to_fp32(bias_bf16[n]);
      C_bf16[(size_t)m * N + n] = orc_fp32_to_bf16(r);
    }
    free(wf);
  }
  free(w);
  free(af);
  return 0;
}

/* ------------------------------------------------------------------------------------------------
 * Per-token dynamic int8 activation quantization (torch form):
 *   absmax = max(amax|x|, 1e-10); scale = absmax / 127; q = clamp(round_half_even(x / scale), -128, 127)
 *   pymllm/tests/bench_w8a8_activation_quant.py:20-26
 * x fp32 [M][K] (a bf16 activation is up-cast exactly first); q int8 [M][K]; scale fp32 [M].
 * ---------------------------------------------------------------------------------------------- */
ORC_API void orc_per_token_quant_int8(const float* x, int8_t* q, float* scale, int M, int K) {
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; m++) {
    const float* xr = x + (size_t)m * K;
    float amax = 0.0f;
    for (int k = 0; k < K; k++) {
      float a = fabsf(xr[k]);
      amax = a > amax ? a : amax;
    }
    if (amax < 1e-10f) amax = 1e-10f;
    const float sc = amax / 127.0f;
    scale[m] = sc;
    for (int k = 0; k < K; k++) {
      float v = rintf(xr[k] / sc);
      v = v > 127.f ? 127.f : (v < -128.f ? -128.f : v);
      q[(size_t)m * K + k] = (int8_t)v;
    }
  }
}

/* W8A8 GEMM: acc[m][n] = sum_k xq[m][k] * W[n][k] in int32 (exact), then
 *   y = out_dtype( float(acc) * (w_scale[n] * x_scale[m]) + bias[n] )
 *   mllm-kernel/mllm_kernel/cuda/csrc/cutlass_extensions/epilogue/epilogue_per_row_per_col_scale.h:234-253,273-280
 *   CPU-style references: tests/ascend/AscendLinearKernelTest.hpp:289-303, mllm-kernel/tests/test_int8_scaled_mm_cutlass.py:22-35
 * acc_out (optional) int32 [M][N]; y bf16 bits [M][N] (optional). */
ORC_API void orc_w8a8_gemm(const int8_t* xq, const float* x_scale, const int8_t* W, const float* w_scale,
                           const float* bias, int32_t* acc_out, uint16_t* y_bf16, int M, int N, int K) {
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; m++)
    for (int n = 0; n < N; n++) {
      const int8_t* a = xq + (size_t)m * K;
      const int8_t* w = W + (size_t)n * K;
      int32_t acc = 0;
      for (int k = 0; k < K; k++) acc += (int32_t)a[k] * (int32_t)w[k];
      if (acc_out) acc_out[(size_t)m * N + n] = acc;
      if (y_bf16) {
        float r = (float)acc * (w_scale[n] * x_scale[m]);
        if (bias) r += bias[n];
        y_bf16[(size_t)m * N + n] = orc_fp32_to_bf16(r);
      }
    }
}

/* ------------------------------------------------------------------------------------------------
 * MoE expert FFN over expert-sorted tokens.
 *   Qwen3MoE::moeInfer      mllm/models/qwen3_moe/modeling_qwen3_moe_fa2.hpp:175-238
 *   Qwen3MoeMLP::forward    :98-100     down(silu(gate(x)) * up(x)), every Linear = orc_linear_q
 *   SiLU                    mllm/backends/cpu/kernels/x86/silu.cpp:16-56 (orc_silu_array, declared below)
 * x fp32 [T][H]; topk_ids int32 [T][k]; topk_w fp32 [T][k]; expert e weights: Wg,Wu blocks [I][H/32], Wd blocks [H][I/32],
 * stored per expert contiguously.  y fp32 [T][H] = sum_j topk_w[t][j] * expert_{ids[t][j]}(x[t]), j ascending.
 * ---------------------------------------------------------------------------------------------- */
ORC_API float orc_silu(float x) { return x / (1.0f + expf(-x)); }
ORC_API void orc_silu_array(const float* x, float* y, int64_t len);

/* exp as the x86 kernels compute it: vexpq_fast_f32, mllm/backends/cpu/kernels/x86/math.hpp:19-72, one lane of it.
 * MulAdd is a fused multiply-add on the AVX2/FMA targets the reference builds for.  Note the argument reduction as the
 * reference writes it: C1 is the full ln 2 (std::numbers::ln2_v<float>) and the Cephes correction C2 is still
 * subtracted, so the reduced argument is off by n * 2.1219444e-4 and the result is exp(x) * exp(n * 2.1219444e-4),
 * n = floor(x * log2(e) + 0.5).  Restated as written. */
ORC_API float orc_exp_poly(float x) {
  x = fminf(fmaxf(x, -88.3762626647949f), 88.3762626647949f);
  float fx = fmaf(x, 1.44269504088896341f, 0.5f);
  float tmp = floorf(fx);
  fx = tmp - (tmp > fx ? 1.0f : 0.0f);
  float tmp2 = fx * 0.693147180559945309f;
  float z = fx * -2.12194440e-4f;
  x = (x - tmp2) - z;
  z = x * x;
  float y = 1.9875691500E-4f;
  y = fmaf(y, x, 1.3981999507E-3f);
  y = fmaf(y, x, 8.3334519073E-3f);
  y = fmaf(y, x, 4.1665795894E-2f);
  y = fmaf(y, x, 1.6666665459E-1f);
  y = fmaf(y, x, 5.0000001201E-1f);
  y = fmaf(y, z, x);
  y = y + 1.0f;
  int32_t n = (int32_t)fx + 0x7f;
  return y * u2f((uint32_t)n << 23);
}

/* silu_fp32, mllm/backends/cpu/kernels/x86/silu.cpp:16-56: whole vectors of 8 floats (AVX2) take
 * x * (1 / (1 + exp_poly(-x))), the remaining len % 8 elements x / (1 + exp(-x)). */
ORC_API void orc_silu_array(const float* x, float* y, int64_t len) {
  int64_t aligned = len - (len % 8);
  for (int64_t i = 0; i < aligned; i++) y[i] = x[i] * (1.0f / (1.0f + orc_exp_poly(-x[i])));
  for (int64_t i = aligned; i < len; i++) y[i] = x[i] / (1.0f + expf(-x[i]));
}

/* rmsnorm_fp32, mllm/backends/cpu/kernels/x86/rmsnorm.cpp:17-52 with vsquare_mean_fp32, math.hpp:75-90:
 * eight partial sums (AVX2 lanes) over whole vectors, reduced, then the tail; y = x * (w * rms) in whole vectors,
 * x * rms * w in the tail. */
ORC_API void orc_rmsnorm(const float* x, const float* w, float* y, int64_t rows, int D, float eps, int add_unit_offset) {
  for (int64_t r = 0; r < rows; r++) {
    const float* xr = x + r * D;
    float* yr = y + r * D;
    float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int i = 0;
    for (; i + 8 <= D; i += 8)
      for (int l = 0; l < 8; l++) lanes[l] = lanes[l] + xr[i + l] * xr[i + l];
    /* hn::ReduceSum on AVX2: pairwise over the lanes */
    float acc = ((lanes[0] + lanes[4]) + (lanes[2] + lanes[6])) + ((lanes[1] + lanes[5]) + (lanes[3] + lanes[7]));
    for (; i < D; i++) acc += xr[i] * xr[i];
    float rms = 1.0f / sqrtf(acc / (float)D + eps);
    i = 0;
    for (; i + 8 <= D; i += 8)
      for (int l = 0; l < 8; l++) {
        float m = add_unit_offset ? (w[i + l] + 1.0f) * rms : w[i + l] * rms;
        yr[i + l] = xr[i + l] * m;
      }
    for (; i < D; i++) yr[i] = add_unit_offset ? xr[i] * rms * (w[i] + 1.0f) : xr[i] * rms * w[i];
  }
}

/* softmax_v1_fp32 over contiguous rows, mllm/backends/cpu/kernels/x86/softmax.cpp:18-76: rows of at most 16 elements
 * use expf, longer ones exp_poly on whole vectors of 8 and expf on the tail; the sum runs in 8 lanes. */
ORC_API void orc_softmax_rows(const float* x, float* y, int64_t rows, int len) {
  for (int64_t r = 0; r < rows; r++) {
    const float* xr = x + r * len;
    float* yr = y + r * len;
    float mx = -3.402823466e+38f;
    for (int i = 0; i < len; i++) mx = fmaxf(mx, xr[i]);
    float sum;
    if (len <= 16) {
      sum = 0.f;
      for (int i = 0; i < len; i++) {
        yr[i] = expf(xr[i] - mx);
        sum += yr[i];
      }
    } else {
      float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      int i = 0;
      for (; i + 8 <= len; i += 8)
        for (int l = 0; l < 8; l++) {
          yr[i + l] = orc_exp_poly(xr[i + l] - mx);
          lanes[l] += yr[i + l];
        }
      sum = ((lanes[0] + lanes[4]) + (lanes[2] + lanes[6])) + ((lanes[1] + lanes[5]) + (lanes[3] + lanes[7]));
      for (; i < len; i++) {
        yr[i] = expf(xr[i] - mx);
        sum += yr[i];
      }
    }
    sum = 1.f / sum;
    for (int i = 0; i < len; i++) yr[i] *= sum;
  }
}

/* topk_impl over the last axis, mllm/backends/cpu/ops/TopKOp.cpp:20-72: a candidate replaces the weakest kept element
 * only when it is strictly better, the kept set is then ordered by value (sorted) or by index.  The order among EQUAL
 * values is left to std::priority_queue / std::sort there; here equal values are kept lowest index first and a stable
 * order is used (tests use rows without ties, plus tie cases checked as sets). */
ORC_API void orc_topk_rows(const float* x, float* values, int32_t* indices, int64_t rows, int len, int k, int largest,
                           int sorted) {
  for (int64_t r = 0; r < rows; r++) {
    const float* xr = x + r * len;
    float* v = values + r * k;
    int32_t* id = indices + r * k;
    int n = 0;
    for (int i = 0; i < len; i++) { /* kept set ordered best first (insertion keeps earlier indices ahead on ties) */
      float c = xr[i];
      int pos = n;
      while (pos > 0 && (largest ? c > v[pos - 1] : c < v[pos - 1])) pos--;
      if (pos >= k) continue;
      int last = n < k ? n : k - 1;
      for (int j = last; j > pos; j--) {
        v[j] = v[j - 1];
        id[j] = id[j - 1];
      }
      v[pos] = c;
      id[pos] = i;
      if (n < k) n++;
    }
    if (!sorted) { /* by index */
      for (int a = 1; a < k; a++) {
        float tv = v[a];
        int32_t ti = id[a];
        int b = a - 1;
        while (b >= 0 && id[b] > ti) {
          v[b + 1] = v[b];
          id[b + 1] = id[b];
          b--;
        }
        v[b + 1] = tv;
        id[b + 1] = ti;
      }
    }
  }
}

/* MoEGate::forward, mllm/models/qwen3_moe/modeling_qwen3_moe_fa2.hpp:121-139: logits = x . W^T in fp32, softmax, topk
 * (largest, not sorted: index order), optionally weights / sum(weights).  The fp32 matmul's summation order on the CPU
 * depends on the BLAS in use; here: sequential fp32 over H. */
ORC_API void orc_moe_gate(const float* x, const float* w, int32_t* ids, float* weights, float* scores, int64_t M, int H, int E,
                          int k, int norm) {
  float* logit = (float*)malloc(sizeof(float) * (size_t)E);
  float* prob = (float*)malloc(sizeof(float) * (size_t)E);
  for (int64_t t = 0; t < M; t++) {
    for (int e = 0; e < E; e++) {
      float acc = 0.f;
      for (int h = 0; h < H; h++) acc = fmaf(x[t * H + h], w[(size_t)e * H + h], acc);
      logit[e] = acc;
    }
    orc_softmax_rows(logit, prob, 1, E);
    if (scores) memcpy(scores + t * E, prob, sizeof(float) * (size_t)E);
    orc_topk_rows(prob, weights + t * k, ids + t * k, 1, E, k, 1, 0);
    if (norm) {
      float s = 0.f;
      for (int j = 0; j < k; j++) s += weights[t * k + j];
      for (int j = 0; j < k; j++) weights[t * k + j] = weights[t * k + j] / s;
    }
  }
  free(logit);
  free(prob);
}

ORC_API int orc_moe_ffn(const float* x, const int32_t* topk_ids, const float* topk_w, const uint8_t* Wg,
                        const uint8_t* Wu, const uint8_t* Wd, int wtype, float* y, int T, int H, int I, int E, int k,
                        int scale_mode) {
  if (H % QK || I % QK) return -1;
  int bb = blk_bytes(wtype);
  size_t gu_bytes = (size_t)I * (H / QK) * bb, d_bytes = (size_t)H * (I / QK) * bb;
  float* per = (float*)calloc((size_t)T * k * H, 4); /* output of the expert for (token, slot) */
  if (!per) return -2;
  for (int e = 0; e < E; e++) {
    int cnt = 0;
    for (int i = 0; i < T * k; i++) cnt += (topk_ids[i] == e);
    if (!cnt) continue;
    int* rows = (int*)malloc(sizeof(int) * cnt);
    float* xe = (float*)malloc((size_t)cnt * H * 4);
    float* g = (float*)malloc((size_t)cnt * I * 4);
    float* u = (float*)malloc((size_t)cnt * I * 4);
    float* o = (float*)malloc((size_t)cnt * H * 4);
    int c = 0;
    for (int i = 0; i < T * k; i++)
      if (topk_ids[i] == e) {
        rows[c] = i;
        memcpy(xe + (size_t)c * H, x + (size_t)(i / k) * H, (size_t)H * 4);
        c++;
      }
    orc_linear_q(xe, Wg + e * gu_bytes, wtype, NULL, g, cnt, I, H, scale_mode, NULL, NULL);
    orc_linear_q(xe, Wu + e * gu_bytes, wtype, NULL, u, cnt, I, H, scale_mode, NULL, NULL);
    orc_silu_array(g, g, (int64_t)cnt * I); /* the SiLU operator over the whole [cnt, I] tensor, then the product */
    for (size_t i = 0; i < (size_t)cnt * I; i++) g[i] = g[i] * u[i];
    orc_linear_q(g, Wd + e * d_bytes, wtype, NULL, o, cnt, H, I, scale_mode, NULL, NULL);
    for (c = 0; c < cnt; c++) memcpy(per + (size_t)rows[c] * H, o + (size_t)c * H, (size_t)H * 4);
    free(rows); free(xe); free(g); free(u); free(o);
  }
#pragma omp parallel for schedule(static)
  for (int t = 0; t < T; t++)
    for (int h = 0; h < H; h++) {
      float acc = 0.0f;
      for (int j = 0; j < k; j++) acc += per[((size_t)t * k + j) * H + h] * topk_w[(size_t)t * k + j];
      y[(size_t)t * H + h] = acc;
    }
  free(per);
  return 0;
}

/* ================================================================================================
 * K-quants: Q4_K / Q6_K weights with Q8_K activations (the formats of the shipped Qwen3-MoE recipe).
 *   block_q4_K (144 B): fp16 d, fp16 dmin, 12 B of 6-bit scales and mins, 128 B of nibbles   mllm/core/DataTypes.hpp:139-147
 *   block_q6_K (210 B): 128 B low nibbles, 64 B high bit pairs, 16 int8 scales, fp16 d        mllm/core/DataTypes.hpp:153-160
 *   block_q8_K        : fp32 d, 256 int8, 16 int16 sums of 16                                 mllm/core/DataTypes.hpp:188-194
 * Weight blocks are passed as the reference's byte layout with IEEE fp16 patterns in the fp16 fields; scale_mode
 * X86_REF applies the x86 build's storage rounding to them where they are used (scale_value()).
 * Pinned bit for bit against the compiled reference (quantize_row_q8_K, dequantize_row_q4_K / _q6_K, vec_dot_q4_K_q8_K,
 * vec_dot_q6_K_q8_K) in tests/test_oracle_vs_reference.py.
 * ============================================================================================== */
#define QK_K 256
enum { ORC_Q4_K = 2, ORC_Q6_K = 3 };
static inline int kblk_bytes(int wtype) { return wtype == ORC_Q4_K ? 144 : 210; }

/* quantize_row_q8_K_reference, quantize_q8.cpp:215-248.  nearest_int (quantize.hpp:261-267) is round-half-even. */
ORC_API void orc_quantize_row_q8_K(const float* x, int8_t* qs, float* d, int16_t* bsums, int k) {
  int nb = k / QK_K;
  for (int i = 0; i < nb; i++) {
    const float* xb = x + (size_t)i * QK_K;
    int8_t* q = qs + (size_t)i * QK_K;
    float max = 0, amax = 0;
    for (int j = 0; j < QK_K; j++) {
      float ax = fabsf(xb[j]);
      if (ax > amax) {
        amax = ax;
        max = xb[j];
      }
    }
    if (amax == 0.0f) {
      d[i] = 0;
      memset(q, 0, QK_K);
      /* the reference leaves bsums of such a block untouched (uninitialised memory of a fresh tensor); zero here */
      memset(bsums + (size_t)i * 16, 0, 32);
      continue;
    }
    const float iscale = -128.f / max;
    for (int j = 0; j < QK_K; j++) {
      int v = (int)rintf(iscale * xb[j]);
      q[j] = (int8_t)(v < 127 ? v : 127);
    }
    for (int j = 0; j < 16; j++) {
      int sum = 0;
      for (int ii = 0; ii < 16; ii++) sum += q[j * 16 + ii];
      bsums[(size_t)i * 16 + j] = (int16_t)sum;
    }
    d[i] = 1 / iscale;
  }
}

/* get_scale_min_k4, quantize.hpp */
static inline void scale_min_k4(int j, const uint8_t* q, uint8_t* d, uint8_t* m) {
  if (j < 4) {
    *d = q[j] & 63;
    *m = q[j + 4] & 63;
  } else {
    *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
    *m = (uint8_t)((q[j + 4] >> 4) | ((q[j - 0] >> 6) << 4));
  }
}
static inline uint16_t rd16(const uint8_t* p) { uint16_t v; memcpy(&v, p, 2); return v; }

/* dequantize_row_q4_K, quantize_q4.cpp:284-312: y = (d * sc) * q - (dmin * m), each product rounded to fp32 */
ORC_API void orc_dequantize_row_q4_K(const uint8_t* blocks, float* y, int k, int scale_mode) {
  int nb = k / QK_K;
  for (int i = 0; i < nb; i++) {
    const uint8_t* b = blocks + (size_t)i * 144;
    const float d = scale_value(rd16(b), scale_mode), min = scale_value(rd16(b + 2), scale_mode);
    const uint8_t* q = b + 16;
    int is = 0;
    for (int j = 0; j < QK_K; j += 64) {
      uint8_t sc, m;
      scale_min_k4(is + 0, b + 4, &sc, &m);
      const float d1 = d * sc, m1 = min * m;
      scale_min_k4(is + 1, b + 4, &sc, &m);
      const float d2 = d * sc, m2 = min * m;
      for (int l = 0; l < 32; l++) *y++ = d1 * (q[l] & 0xF) - m1;
      for (int l = 0; l < 32; l++) *y++ = d2 * (q[l] >> 4) - m2;
      q += 32;
      is += 2;
    }
  }
}

/* the 6-bit value (minus 32) of element e of a q6_K block, dequantize_row_q6_K, quantize_q6.cpp:108-133 */
static inline int q6_value(const uint8_t* b, int e) {
  const uint8_t* ql = b + 64 * (e / 128);
  const uint8_t* qh = b + 128 + 32 * (e / 128);
  int r = e % 128, g = r / 32, l = r % 32;
  int lo = (g & 1) ? ql[l + 32] : ql[l];
  lo = (g >= 2) ? (lo >> 4) : (lo & 0xF);
  int hi = (qh[l] >> (2 * g)) & 3;
  return (int8_t)(lo | (hi << 4)) - 32;
}
ORC_API void orc_dequantize_row_q6_K(const uint8_t* blocks, float* y, int k, int scale_mode) {
  int nb = k / QK_K;
  for (int i = 0; i < nb; i++) {
    const uint8_t* b = blocks + (size_t)i * 210;
    const float d = scale_value(rd16(b + 208), scale_mode);
    const int8_t* sc = (const int8_t*)(b + 192);
    for (int e = 0; e < QK_K; e++) y[(size_t)i * QK_K + e] = d * sc[e / 16] * q6_value(b, e);
  }
}

static inline float hsum8(const float* a) { /* hsum_float_8 */
  float t0 = a[4] + a[0], t1 = a[5] + a[1], t2 = a[6] + a[2], t3 = a[7] + a[3];
  float u0 = t0 + t2, u1 = t1 + t3;
  return u0 + u1;
}

/* vec_dot_q4_K_q8_K, AVX2 branch, vec_dot.cpp:498-560 (QK_K == 256).  Eight int32 lanes: lane u collects, over the eight
 * sub-blocks, scale * (sum over elements 4u..4u+3 of the sub-block); acc[u] = fma(d, float(lane), acc[u]) per super-block.
 * Mins: four lanes, lane v = m[2v] * bsum32[2v] + m[2v+1] * bsum32[2v+1], acc_m[v] = fma(dmin, float(lane), acc_m[v]),
 * reduced as (a0 + a2) + (a1 + a3).  isum / msum (optional) receive the exact per-super-block integers. */
ORC_API float orc_vec_dot_q4_K_q8_K(const uint8_t* wrow, const int8_t* xq, const float* xd, const int16_t* xbs, int k, int scale_mode,
                                    int32_t* isum, int32_t* msum) {
  int nb = k / QK_K;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}, acc_m[4] = {0, 0, 0, 0};
  for (int i = 0; i < nb; i++) {
    const uint8_t* b = wrow + (size_t)i * 144;
    const float d = xd[i] * scale_value(rd16(b), scale_mode);
    const float dmin = -xd[i] * scale_value(rd16(b + 2), scale_mode);
    uint8_t sc[8], mn[8];
    for (int j = 0; j < 8; j++) scale_min_k4(j, b + 4, &sc[j], &mn[j]);
    const int16_t* bs = xbs + (size_t)i * 16;
    int32_t mtot = 0;
    for (int v = 0; v < 4; v++) {
      int32_t p = (int32_t)mn[2 * v] * (bs[4 * v] + bs[4 * v + 1]) + (int32_t)mn[2 * v + 1] * (bs[4 * v + 2] + bs[4 * v + 3]);
      mtot += p;
      acc_m[v] = fmaf(dmin, (float)p, acc_m[v]);
    }
    int32_t lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const uint8_t* q4 = b + 16;
    const int8_t* q8 = xq + (size_t)i * QK_K;
    for (int j = 0; j < 4; j++) {
      for (int u = 0; u < 8; u++) {
        int32_t lo = 0, hi = 0;
        for (int e = 4 * u; e < 4 * u + 4; e++) {
          lo += (int32_t)(q4[32 * j + e] & 0xF) * q8[64 * j + e];
          hi += (int32_t)(q4[32 * j + e] >> 4) * q8[64 * j + 32 + e];
        }
        lanes[u] += sc[2 * j] * lo + sc[2 * j + 1] * hi;
      }
    }
    int32_t tot = 0;
    for (int u = 0; u < 8; u++) {
      tot += lanes[u];
      acc[u] = fmaf(d, (float)lanes[u], acc[u]);
    }
    if (isum) isum[i] = tot;
    if (msum) msum[i] = mtot;
  }
  float am0 = acc_m[0] + acc_m[2], am1 = acc_m[1] + acc_m[3];
  return hsum8(acc) + (am0 + am1);
}

/* vec_dot_q6_K_q8_K, AVX2 branch, vec_dot.cpp:955-1044.  Lane u of group g covers elements 4u..4u+3 of the group's 32. */
ORC_API float orc_vec_dot_q6_K_q8_K(const uint8_t* wrow, const int8_t* xq, const float* xd, int k, int scale_mode, int32_t* isum) {
  int nb = k / QK_K;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int i = 0; i < nb; i++) {
    const uint8_t* b = wrow + (size_t)i * 210;
    const float d = xd[i] * scale_value(rd16(b + 208), scale_mode);
    const int8_t* sc = (const int8_t*)(b + 192);
    const int8_t* q8 = xq + (size_t)i * QK_K;
    int32_t lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int grp = 0; grp < 8; grp++) /* 8 groups of 32 elements */
      for (int u = 0; u < 8; u++) {
        int32_t s = 0;
        for (int e = 32 * grp + 4 * u; e < 32 * grp + 4 * u + 4; e++) s += q6_value(b, e) * q8[e];
        lanes[u] += sc[2 * grp + (u >= 4)] * s;
      }
    int32_t tot = 0;
    for (int u = 0; u < 8; u++) {
      tot += lanes[u];
      acc[u] = fmaf(d, (float)lanes[u], acc[u]);
    }
    if (isum) isum[i] = tot;
  }
  return hsum8(acc);
}

/* Linear with Q4_K / Q6_K weights: ggml::mat_mul's generic branch, matmul.cpp:147-189 (rows of x to Q8_K), :300-360
 * (vec_dot per output element), bias added afterwards with mllm_add_fp32 (:280-290). */
ORC_API int orc_linear_kq(const float* x, const uint8_t* W, int wtype, const float* bias, float* y, int M, int N, int K, int scale_mode) {
  if (K % QK_K || (wtype != ORC_Q4_K && wtype != ORC_Q6_K)) return -1;
  int nb = K / QK_K, bb = kblk_bytes(wtype);
  int8_t* xq = (int8_t*)malloc((size_t)M * K);
  float* xd = (float*)malloc(sizeof(float) * (size_t)M * nb);
  int16_t* xbs = (int16_t*)malloc(sizeof(int16_t) * (size_t)M * nb * 16);
  if (!xq || !xd || !xbs) return -2;
  for (int m = 0; m < M; m++) orc_quantize_row_q8_K(x + (size_t)m * K, xq + (size_t)m * K, xd + (size_t)m * nb, xbs + (size_t)m * nb * 16, K);
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; n++)
    for (int m = 0; m < M; m++) {
      const uint8_t* wrow = W + (size_t)n * nb * bb;
      float v = wtype == ORC_Q4_K
                    ? orc_vec_dot_q4_K_q8_K(wrow, xq + (size_t)m * K, xd + (size_t)m * nb, xbs + (size_t)m * nb * 16, K, scale_mode, NULL, NULL)
                    : orc_vec_dot_q6_K_q8_K(wrow, xq + (size_t)m * K, xd + (size_t)m * nb, K, scale_mode, NULL);
      y[(size_t)m * N + n] = bias ? v + bias[n] : v;
    }
  free(xq); free(xd); free(xbs);
  return 0;
}

/* ================================================================================================
 * Offline K-quant weight quantizers: fp32 rows -> reference super-blocks
 *   Q4_K  quantize_row_q4_K_reference with make_qkx2_quants(32, 15, ..., rmin -1, rdelta 0.1, nstep 20, squared error),
 *         mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q4.cpp:97-168 (the search), :184-282 (the super-block)
 *   Q6_K  quantize_row_q6_K_reference with make_qx_quants(16, 32, ..., rmse_type 1), quantize_q6.cpp:34-106,
 *         quantize.hpp:268-325 (the search); nearest_int quantize.hpp:261-267
 * Every fp32 operation is written in the reference's order (no contraction in either build): sums run element by element,
 * `w * l * l` is (w * l) * l, and so on.  The fp16 fields d / dmin: scale_mode IEEE stores the fp16 pattern P and the final
 * code pass reads its value; X86_REF stores what the x86 build leaves in the file, the half-precision encoding of the NUMBER P,
 * and the final code pass reads what that build reads back, P rounded to 11 significant bits (orc_x86_scale_bits) -- so
 * the codes themselves can differ between the two modes.
 * Pinned: bytes (codes, 6-bit / int8 scales) and decoded d / dmin patterns bit-exact against the compiled reference
 * quantizers in X86_REF mode (tests/test_oracle_vs_reference.py); the IEEE mode differs only in the two lines named above.
 * ============================================================================================== */
static inline int orc_nearest_int(float fval) {
  float val = fval + 12582912.f;
  int i;
  memcpy(&i, &val, sizeof(int));
  return (i & 0x007fffff) - 0x00400000;
}

/* one sub-block of n weights -> codes L (0..nmax), returns the scale, *the_min = -offset (>= 0) */
static float orc_qkx2_search(int n, int nmax, const float* x, const float* weights, uint8_t* L, float* the_min, uint8_t* Laux,
                             float rmin, float rdelta, int nstep) {
  float min = x[0], max = x[0];
  float sum_w = weights[0];
  float sum_x = sum_w * x[0];
  for (int i = 1; i < n; i++) {
    if (x[i] < min) min = x[i];
    if (x[i] > max) max = x[i];
    const float w = weights[i];
    sum_w += w;
    sum_x += w * x[i];
  }
  if (min > 0) min = 0;
  if (max == min) {
    for (int i = 0; i < n; i++) L[i] = 0;
    *the_min = -min;
    return 0.f;
  }
  float iscale = nmax / (max - min);
  float scale = 1 / iscale;
  float best = 0;
  for (int i = 0; i < n; i++) {
    int l = orc_nearest_int(iscale * (x[i] - min));
    l = l < 0 ? 0 : (l > nmax ? nmax : l);
    L[i] = (uint8_t)l;
    float diff = scale * L[i] + min - x[i];
    diff = diff * diff;
    best += weights[i] * diff;
  }
  for (int is = 0; is <= nstep; is++) {
    iscale = (rmin + rdelta * is + nmax) / (max - min);
    float sum_l = 0, sum_l2 = 0, sum_xl = 0;
    for (int i = 0; i < n; i++) {
      int l = orc_nearest_int(iscale * (x[i] - min));
      l = l < 0 ? 0 : (l > nmax ? nmax : l);
      Laux[i] = (uint8_t)l;
      const float w = weights[i];
      sum_l += w * l;
      sum_l2 += w * l * l;
      sum_xl += w * l * x[i];
    }
    const float D = sum_w * sum_l2 - sum_l * sum_l;
    if (D > 0) {
      float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
      float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
      if (this_min > 0) {
        this_min = 0;
        this_scale = sum_xl / sum_l2;
      }
      float err = 0;
      for (int i = 0; i < n; i++) {
        float diff = this_scale * Laux[i] + this_min - x[i];
        diff = diff * diff;
        err += weights[i] * diff;
      }
      if (err < best) {
        for (int i = 0; i < n; i++) L[i] = Laux[i];
        best = err;
        scale = this_scale;
        min = this_min;
      }
    }
  }
  *the_min = -min;
  return scale;
}

ORC_API void orc_quantize_row_q4_K(const float* x, uint8_t* blocks, int k, int scale_mode) {
  const int nb = k / QK_K;
  for (int i = 0; i < nb; i++, x += QK_K) {
    uint8_t* y = blocks + (size_t)i * 144;
    uint8_t L[QK_K], Laux[32];
    float weights[32], mins[8], scales[8];
    float max_scale = 0, max_min = 0;
    for (int j = 0; j < 8; j++) {
      const float* xs = x + 32 * j;
      float sum_x2 = 0;
      for (int l = 0; l < 32; l++) sum_x2 += xs[l] * xs[l];
      const float av_x = sqrtf(sum_x2 / 32);
      for (int l = 0; l < 32; l++) weights[l] = av_x + fabsf(xs[l]);
      scales[j] = orc_qkx2_search(32, 15, xs, weights, L + 32 * j, &mins[j], Laux, -1.f, 0.1f, 20);
      if (scales[j] > max_scale) max_scale = scales[j];
      if (mins[j] > max_min) max_min = mins[j];
    }
    const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
    const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
    uint8_t* sc12 = y + 4;
    memset(sc12, 0, 12);
    uint8_t ls6[8], lm6[8];
    for (int j = 0; j < 8; j++) {
      uint8_t ls = (uint8_t)orc_nearest_int(inv_scale * scales[j]);
      uint8_t lm = (uint8_t)orc_nearest_int(inv_min * mins[j]);
      ls = ls < 63 ? ls : 63;
      lm = lm < 63 ? lm : 63;
      ls6[j] = ls;
      lm6[j] = lm;
      if (j < 4) {
        sc12[j] = ls;
        sc12[j + 4] = lm;
      } else {
        sc12[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
        sc12[j - 4] |= (uint8_t)((ls >> 4) << 6);
        sc12[j] |= (uint8_t)((lm >> 4) << 6);
      }
    }
    const uint16_t pd = orc_fp32_to_fp16(max_scale / 63.f), pm = orc_fp32_to_fp16(max_min / 63.f);
    const uint16_t fd = store_scale_field(pd, scale_mode), fm = store_scale_field(pm, scale_mode);
    memcpy(y, &fd, 2);
    memcpy(y + 2, &fm, 2);
    const float dv = scale_value(pd, scale_mode), mv = scale_value(pm, scale_mode);
    for (int j = 0; j < 8; j++) {
      const float d = dv * ls6[j];  /* the 6-bit values read back (get_scale_min_k4) are the ones just packed */
      if (d == 0.0f) continue;
      const float dm = mv * lm6[j];
      for (int ii = 0; ii < 32; ii++) {
        int l = orc_nearest_int((x[32 * j + ii] + dm) / d);
        L[32 * j + ii] = (uint8_t)(l < 0 ? 0 : (l > 15 ? 15 : l));
      }
    }
    uint8_t* q = y + 16;
    for (int j = 0; j < QK_K; j += 64, q += 32)
      for (int l = 0; l < 32; l++) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
  }
}

/* one group of n weights -> codes L (0 .. 2 nmax - 1, offset nmax), returns the scale; weights x^2 (rmse_type 1) */
static float orc_qx_search(int n, int nmax, const float* x, int8_t* L) {
  float max = 0, amax = 0;
  for (int i = 0; i < n; i++) {
    const float ax = fabsf(x[i]);
    if (ax > amax) {
      amax = ax;
      max = x[i];
    }
  }
  if (amax < 1e-30f) {
    for (int i = 0; i < n; i++) L[i] = 0;
    return 0.f;
  }
  float iscale = -nmax / max;
  float sumlx = 0, suml2 = 0;
  for (int i = 0; i < n; i++) {
    int l = orc_nearest_int(iscale * x[i]);
    l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
    L[i] = (int8_t)(l + nmax);
    const float w = x[i] * x[i];
    sumlx += w * x[i] * l;
    suml2 += w * l * l;
  }
  float scale = sumlx / suml2;
  float best = scale * sumlx;
  for (int is = -9; is <= 9; is++) {
    if (is == 0) continue;
    iscale = -(nmax + 0.1f * is) / max;
    sumlx = suml2 = 0;
    for (int i = 0; i < n; i++) {
      int l = orc_nearest_int(iscale * x[i]);
      l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
      const float w = x[i] * x[i];
      sumlx += w * x[i] * l;
      suml2 += w * l * l;
    }
    if (suml2 > 0 && sumlx * sumlx > best * suml2) {
      for (int i = 0; i < n; i++) {
        int l = orc_nearest_int(iscale * x[i]);
        l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
        L[i] = (int8_t)(nmax + l);
      }
      scale = sumlx / suml2;
      best = scale * sumlx;
    }
  }
  return scale;
}

ORC_API void orc_quantize_row_q6_K(const float* x, uint8_t* blocks, int k, int scale_mode) {
  const int nb = k / QK_K;
  for (int i = 0; i < nb; i++, x += QK_K) {
    uint8_t* y = blocks + (size_t)i * 210;
    int8_t L[QK_K];
    float scales[16];
    float max_scale = 0, max_abs_scale = 0;
    for (int ib = 0; ib < 16; ib++) {
      const float scale = orc_qx_search(16, 32, x + 16 * ib, L + 16 * ib);
      scales[ib] = scale;
      const float a = fabsf(scale);
      if (a > max_abs_scale) {
        max_abs_scale = a;
        max_scale = scale;
      }
    }
    if (!max_abs_scale) {
      memset(y, 0, 210);  /* the fp16 pattern of 0.0 is 0 in either storage mode */
      continue;
    }
    const float iscale = -128.f / max_scale;
    const uint16_t pd = orc_fp32_to_fp16(1 / iscale);
    const uint16_t fd = store_scale_field(pd, scale_mode);
    memcpy(y + 208, &fd, 2);
    int8_t* sc = (int8_t*)(y + 192);
    for (int ib = 0; ib < 16; ib++) {
      const int v = orc_nearest_int(iscale * scales[ib]);
      sc[ib] = (int8_t)(v < 127 ? v : 127);
    }
    const float dv = scale_value(pd, scale_mode);
    for (int j = 0; j < 16; j++) {
      const float d = dv * sc[j];
      if (!d) continue;
      for (int ii = 0; ii < 16; ii++) {
        int l = orc_nearest_int(x[16 * j + ii] / d);
        l = l < -32 ? -32 : (l > 31 ? 31 : l);
        L[16 * j + ii] = (int8_t)(l + 32);
      }
    }
    uint8_t* ql = y;
    uint8_t* qh = y + 128;
    for (int j = 0; j < QK_K; j += 128, ql += 64, qh += 32)
      for (int l = 0; l < 32; l++) {
        const uint8_t q1 = L[j + l] & 0xF, q2 = L[j + l + 32] & 0xF, q3 = L[j + l + 64] & 0xF, q4 = L[j + l + 96] & 0xF;
        ql[l] = (uint8_t)(q1 | (q3 << 4));
        ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
        qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) | ((L[j + l + 64] >> 4) << 4) | ((L[j + l + 96] >> 4) << 6));
      }
  }
}
