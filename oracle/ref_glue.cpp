// extern "C" wrappers over the reference's own kernel functions.  TEST INFRASTRUCTURE ONLY.
//
// Compiled together with the reference's translation units
//   mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.cpp
//   mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q4.cpp
//   mllm/backends/cpu/kernels/common/ggml/vec_dot.cpp
// straight from the reference checkout (see oracle/Makefile) into oracle/_ref/libmllm_ref.so.  It exists so that the
// tests can pin oracle/qlinear_oracle.c against the real reference arithmetic.  Nothing here restates arithmetic: each
// wrapper only converts between plain arrays and the reference's block structs and calls the reference function.
//
// Scale encoding: on x86 the reference's block field `d` is a half_float::half that holds the NUMBER
// float(bit pattern) (see qlinear_oracle.c, orc_x86_scale_bits).  Wrappers that take an IEEE fp16 bit pattern `b`
// store half(float(b)), exactly what the reference quantizer's own assignment `y[i].d = MLLM_FP32_TO_FP16(d)` does.
#include <cstdint>
#include <cstring>
#include <vector>

#include "mllm/core/DataTypes.hpp"
#include "mllm/backends/cpu/kernels/common/ggml/quantize/quantize.hpp"
#include "mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q4.hpp"
#include "mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.hpp"
#include "mllm/backends/cpu/kernels/common/ggml/vec_dot.hpp"

using namespace mllm;
using namespace mllm::cpu;
using namespace mllm::cpu::ggml;

#define REF_API extern "C" __attribute__((visibility("default")))

static_assert(sizeof(block_q4_0) == 18, "block_q4_0 must be 18 bytes");
static_assert(sizeof(block_q8_0) == 34, "block_q8_0 must be 34 bytes");

// raw macro results
REF_API uint16_t ref_fp32_to_fp16_bits(float f) { return (uint16_t)MLLM_FP32_TO_FP16(f); }
REF_API float ref_fp16_bits_to_fp32(uint16_t b) { return MLLM_FP16_TO_FP32(b); }

// The value a scale takes part with after the reference stored pattern `b` into a block and read it back.
REF_API float ref_scale_store_load(uint16_t b) {
  block_q8_0 blk;
  blk.d = b;  // same implicit conversion as `y[i].d = MLLM_FP32_TO_FP16(d)`
  return MLLM_FP16_TO_FP32(blk.d);
}

// quantize_row_q8_0 -> codes and the EFFECTIVE scale value (what a later read of the block yields)
REF_API void ref_quantize_row_q8_0(const float* x, int8_t* qs, float* d_eff, int k) {
  int nb = k / QK8_0;
  std::vector<block_q8_0> y(nb);
  quantize_row_q8_0(x, y.data(), k);
  for (int i = 0; i < nb; i++) {
    std::memcpy(qs + (size_t)i * QK8_0, y[i].qs, QK8_0);
    d_eff[i] = MLLM_FP16_TO_FP32(y[i].d);
  }
}

static void to_ref_q4(const uint8_t* canon, int nb, std::vector<block_q4_0>& out) {
  out.resize(nb);
  for (int i = 0; i < nb; i++) {
    uint16_t b;
    std::memcpy(&b, canon + (size_t)i * 18, 2);
    out[i].d = b;
    std::memcpy(out[i].qs, canon + (size_t)i * 18 + 2, 16);
  }
}
static void to_ref_q8(const uint8_t* canon, int nb, std::vector<block_q8_0>& out) {
  out.resize(nb);
  for (int i = 0; i < nb; i++) {
    uint16_t b;
    std::memcpy(&b, canon + (size_t)i * 34, 2);
    out[i].d = b;
    std::memcpy(out[i].qs, canon + (size_t)i * 34 + 2, 32);
  }
}

// wtype: 0 = Q4_0, 1 = Q8_0.  `canon` = blocks whose d field is an IEEE fp16 bit pattern.
REF_API void ref_dequantize_row(const uint8_t* canon, int wtype, float* y, int k) {
  int nb = k / 32;
  if (wtype == 0) {
    std::vector<block_q4_0> w;
    to_ref_q4(canon, nb, w);
    dequantize_row_q4_0(w.data(), y, k);
  } else {
    std::vector<block_q8_0> w;
    to_ref_q8(canon, nb, w);
    dequantize_row_q8_0(w.data(), y, k);
  }
}

// Quantized Linear the way ggml::mat_mul's vec_dot fallback runs it (ggml/matmul.cpp:148-193,295-351):
// reference quantize_row_q8_0 on every activation row, reference vec_dot per output, then + bias.
REF_API void ref_linear_q(const float* x, const uint8_t* W_canon, int wtype, const float* bias, float* y, int M, int N,
                          int K) {
  int nb = K / 32;
  std::vector<block_q8_0> xq((size_t)M * nb);
  for (int m = 0; m < M; m++) quantize_row_q8_0(x + (size_t)m * K, xq.data() + (size_t)m * nb, K);
  std::vector<block_q4_0> w4;
  std::vector<block_q8_0> w8;
  for (int n = 0; n < N; n++) {
    if (wtype == 0) to_ref_q4(W_canon + (size_t)n * nb * 18, nb, w4);
    else to_ref_q8(W_canon + (size_t)n * nb * 34, nb, w8);
    for (int m = 0; m < M; m++) {
      float s = 0.f;
      if (wtype == 0) vec_dot_q4_0_q8_0(K, &s, w4.data(), xq.data() + (size_t)m * nb);
      else vec_dot_q8_0_q8_0(K, &s, w8.data(), xq.data() + (size_t)m * nb, 0, 0, 0);
      y[(size_t)m * N + n] = bias ? s + bias[n] : s;
    }
  }
}

// Reference Q4_0 weight quantizer (quantize_q4.cpp:33-72) -> canonical blocks carrying the EFFECTIVE scale pattern.
REF_API void ref_quantize_row_q4_0(const float* x, uint8_t* canon, int k) {
  int nb = k / 32;
  std::vector<block_q4_0> y(nb);
  quantize_row_q4_0(x, y.data(), k);
  for (int i = 0; i < nb; i++) {
    uint16_t b = (uint16_t)(float)y[i].d;
    std::memcpy(canon + (size_t)i * 18, &b, 2);
    std::memcpy(canon + (size_t)i * 18 + 2, y[i].qs, 16);
  }
}

// ---- K-quants ------------------------------------------------------------------------------------------------------
#include "mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q6.hpp"
static_assert(sizeof(block_q4_K) == 144, "block_q4_K must be 144 bytes");
static_assert(sizeof(block_q6_K) == 210, "block_q6_K must be 210 bytes");

static void to_ref_q4k(const uint8_t* canon, int nb, std::vector<block_q4_K>& out) {
  out.resize(nb);
  for (int i = 0; i < nb; i++) {
    uint16_t d, m;
    std::memcpy(&d, canon + (size_t)i * 144, 2);
    std::memcpy(&m, canon + (size_t)i * 144 + 2, 2);
    out[i].d = d;  // implicit conversion, as in the quantizer's `y[i].d = MLLM_FP32_TO_FP16(...)`
    out[i].dmin = m;
    std::memcpy(out[i].scales, canon + (size_t)i * 144 + 4, 12);
    std::memcpy(out[i].qs, canon + (size_t)i * 144 + 16, 128);
  }
}
static void to_ref_q6k(const uint8_t* canon, int nb, std::vector<block_q6_K>& out) {
  out.resize(nb);
  for (int i = 0; i < nb; i++) {
    std::memcpy(out[i].ql, canon + (size_t)i * 210, 128);
    std::memcpy(out[i].qh, canon + (size_t)i * 210 + 128, 64);
    std::memcpy(out[i].scales, canon + (size_t)i * 210 + 192, 16);
    uint16_t d;
    std::memcpy(&d, canon + (size_t)i * 210 + 208, 2);
    out[i].d = d;
  }
}

// quantize_row_q8_K -> codes, fp32 scales, sums of 16
REF_API void ref_quantize_row_q8_K(const float* x, int8_t* qs, float* d, int16_t* bsums, int k) {
  int nb = k / QK_K;
  std::vector<block_q8_K> y(nb);
  std::memset(y.data(), 0, sizeof(block_q8_K) * nb);
  quantize_row_q8_K(x, y.data(), k);
  for (int i = 0; i < nb; i++) {
    std::memcpy(qs + (size_t)i * QK_K, y[i].qs, QK_K);
    d[i] = y[i].d;
    std::memcpy(bsums + (size_t)i * 16, y[i].bsums, 32);
  }
}

// wtype: 2 = Q4_K, 3 = Q6_K; canonical blocks (IEEE fp16 patterns in the fp16 fields)
REF_API void ref_dequantize_row_k(const uint8_t* canon, int wtype, float* y, int k) {
  int nb = k / QK_K;
  if (wtype == 2) {
    std::vector<block_q4_K> w;
    to_ref_q4k(canon, nb, w);
    dequantize_row_q4_K(w.data(), y, k);
  } else {
    std::vector<block_q6_K> w;
    to_ref_q6k(canon, nb, w);
    dequantize_row_q6_K(w.data(), y, k);
  }
}

// Linear the way ggml::mat_mul's generic branch runs it: quantize_row_q8_K per activation row, vec_dot per output, + bias
REF_API void ref_linear_kq(const float* x, const uint8_t* W_canon, int wtype, const float* bias, float* y, int M, int N, int K) {
  int nb = K / QK_K;
  std::vector<block_q8_K> xq((size_t)M * nb);
  std::memset(xq.data(), 0, sizeof(block_q8_K) * xq.size());
  for (int m = 0; m < M; m++) quantize_row_q8_K(x + (size_t)m * K, xq.data() + (size_t)m * nb, K);
  std::vector<block_q4_K> w4;
  std::vector<block_q6_K> w6;
  for (int n = 0; n < N; n++) {
    if (wtype == 2) to_ref_q4k(W_canon + (size_t)n * nb * 144, nb, w4);
    else to_ref_q6k(W_canon + (size_t)n * nb * 210, nb, w6);
    for (int m = 0; m < M; m++) {
      float s = 0.f;
      if (wtype == 2) vec_dot_q4_K_q8_K(K, &s, w4.data(), xq.data() + (size_t)m * nb);
      else vec_dot_q6_K_q8_K(K, &s, w6.data(), xq.data() + (size_t)m * nb);
      y[(size_t)m * N + n] = bias ? s + bias[n] : s;
    }
  }
}

// The reference's offline quantizers (quantize_q4.cpp:184-282, quantize_q6.cpp:34-106) -> canonical blocks carrying the
// EFFECTIVE scale patterns (what an x86 read of the stored field yields), used to make realistic fixtures.
REF_API void ref_quantize_row_k(const float* x, uint8_t* canon, int wtype, int k) {
  int nb = k / QK_K;
  if (wtype == 2) {
    std::vector<block_q4_K> y(nb);
    quantize_row_q4_K(x, y.data(), k);
    for (int i = 0; i < nb; i++) {
      uint16_t d = (uint16_t)(float)y[i].d, m = (uint16_t)(float)y[i].dmin;
      std::memcpy(canon + (size_t)i * 144, &d, 2);
      std::memcpy(canon + (size_t)i * 144 + 2, &m, 2);
      std::memcpy(canon + (size_t)i * 144 + 4, y[i].scales, 12);
      std::memcpy(canon + (size_t)i * 144 + 16, y[i].qs, 128);
    }
  } else {
    std::vector<block_q6_K> y(nb);
    quantize_row_q6_K(x, y.data(), k);
    for (int i = 0; i < nb; i++) {
      std::memcpy(canon + (size_t)i * 210, y[i].ql, 128);
      std::memcpy(canon + (size_t)i * 210 + 128, y[i].qh, 64);
      std::memcpy(canon + (size_t)i * 210 + 192, y[i].scales, 16);
      uint16_t d = (uint16_t)(float)y[i].d;
      std::memcpy(canon + (size_t)i * 210 + 208, &d, 2);
    }
  }
}
