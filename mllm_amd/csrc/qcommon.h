// Device-side helpers shared by the gfx950 quantized-Linear kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mllm_hip_qlinear.h"

#define QK 32
#define MLLM_API extern "C" __attribute__((visibility("default")))

#define HIP_RET(expr)                    \
  do {                                   \
    hipError_t e__ = (expr);             \
    if (e__ != hipSuccess) return (int)e__; \
  } while (0)
// the same for calls of this library that return its own int codes (0 = success)
#define RC_RET(expr)         \
  do {                       \
    int rc__ = (expr);       \
    if (rc__ != 0) return rc__; \
  } while (0)

namespace mllmhip {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte load
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---- bit casts / small conversions ---------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {  // round to nearest even, NaN kept quiet
  uint32_t x = __float_as_uint(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {  // two floats -> one dword of bf16, a in the low half
  f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // v_cvt_pk_bf16_f32, nearest even
}
__device__ __forceinline__ float f16bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f32_to_f16bits(float f) {  // v_cvt_f16_f32, round to nearest even
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}
// What an fp16 scale pattern reads back as after the reference's x86 build stored it in a block: the pattern, taken as
// a number, rounded to half precision (11 significant bits).  Mirrors the mechanism itself: number -> half -> number.
__device__ __forceinline__ uint16_t x86_scale_bits(uint16_t b) {
  return (uint16_t)(uint32_t)(float)(_Float16)(float)(uint32_t)b;
}

// ---- exp as the reference's x86 kernels compute it ------------------------------------------------------------
// vexpq_fast_f32, mllm/backends/cpu/kernels/x86/math.hpp:19-72 (Cephes polynomial; fmaf where the reference uses MulAdd).
// As the reference writes the argument reduction (the full ln 2 and the Cephes correction term both subtracted), the
// result is exp(x) * exp(n * 2.1219444e-4), n = round(x / ln 2): restated as written, not repaired.
__device__ __forceinline__ float exp_poly(float x) {
  x = fminf(fmaxf(x, -88.3762626647949f), 88.3762626647949f);
  float fx = fmaf(x, 1.44269504088896341f, 0.5f);
  const float tmp = floorf(fx);
  fx = tmp - (tmp > fx ? 1.0f : 0.0f);
  const float t2 = fx * 0.693147180559945309f;
  const float z0 = fx * -2.12194440e-4f;
  x = (x - t2) - z0;
  const float z = x * x;
  float y = 1.9875691500E-4f;
  y = fmaf(y, x, 1.3981999507E-3f);
  y = fmaf(y, x, 8.3334519073E-3f);
  y = fmaf(y, x, 4.1665795894E-2f);
  y = fmaf(y, x, 1.6666665459E-1f);
  y = fmaf(y, x, 5.0000001201E-1f);
  y = fmaf(y, z, x);
  y = y + 1.0f;
  const int n = (int)fx + 0x7f;
  return y * __int_as_float(n << 23);
}
// ---- wavefront reductions with DPP (64-wide waves; a DPP row is 16 lanes) -------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// Sum over aligned groups of G consecutive lanes; every lane of the group ends up with the total.
template <int G>
__device__ __forceinline__ float group_sum(float v) {
  if (G >= 2) v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  if (G >= 4) v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  if (G >= 8) v += dpp_f<0x141>(v);  // row_half_mirror
  if (G >= 16) v += dpp_f<0x140>(v); // row_mirror
  if (G >= 32) v += __shfl_xor(v, 16, 64);
  if (G >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

// ---- the two divisions of the Q8_0 rule, in fewer instructions, with the bits of IEEE division ------------------------
// amax / 127 and 127 / amax must come out as the correctly rounded quotients (the scale pattern and every code depend on
// them); the compiler's IEEE division is about ten instructions each.  Division by the constant: q0 = amax * RN(1/127), one
// residual, one correction -- equal to amax / 127.f for EVERY positive finite fp32 amax, denormals included.  The reciprocal
// form: v_rcp_f32, one residual, one correction -- equal to 127.f / amax for every amax in [2^-100, 2^100] (1 677 721 600
// values; it differs outside, where the quotient or the reciprocal leaves the normal range).  Both were compared with IEEE
// division over all 2^31 - 2^23 positive finite bit patterns on the GPU.  A wave takes the IEEE division when one of its
// lanes holds a nonzero amax outside that range, an infinity or a NaN (a uniform branch: no lane ever sees a quotient of the
// short forms there).
__device__ __forceinline__ void q8_scales(float amax, float& d, float& id) {
  const bool far = amax != 0.f && !(amax >= 0x1p-100f && amax <= 0x1p100f);  // (infinities and NaN: far)
  if (__builtin_expect(__ballot(far) != 0ull, 0)) {
    d = amax / 127.f;
    id = (amax != 0.f) ? 127.f / amax : 0.f;
    return;
  }
  const float c = 1.0f / 127.0f;
  const float q0 = amax * c;
  d = __builtin_fmaf(__builtin_fmaf(-127.0f, q0, amax), c, q0);
  const float y0 = __builtin_amdgcn_rcpf(amax);
  const float p0 = 127.0f * y0;
  const float q = __builtin_fmaf(__builtin_fmaf(-amax, p0, 127.0f), y0, p0);
  id = (amax != 0.f) ? q : 0.f;
}

// ---- Q8_0 quantization of one 32-element block held in registers ----------------------------------------
// quantize_row_q8_0, AVX2 branch (mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.cpp:106-190):
//   amax = max|v| ; d = amax / 127 ; id = amax != 0 ? 127 / amax : 0 ; q = sat_int8(round_half_even(v * id)).
// q[8] receives the codes, four per dword in element order; returns the fp16 pattern of d; sum = sum of the codes.
__device__ __forceinline__ uint16_t quantize_block_q8_0(const float (&v)[32], uint32_t (&q)[8], int& sum) {
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(v[j]));
  const float d = amax / 127.f;
  const float id = (amax != 0.f) ? 127.f / amax : 0.f;
  int s = 0;
#pragma unroll
  for (int w = 0; w < 8; w++) {
    uint32_t pk = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      int qi = (int)rintf(v[4 * w + j] * id);
      qi = min(127, max(-128, qi));
      s += qi;
      pk |= ((uint32_t)qi & 0xffu) << (8 * j);
    }
    q[w] = pk;
  }
  sum = s;
  return f32_to_f16bits(d);
}

// Four Q8_0 codes rint(v[e] * idv) packed into a dword, for |v[e] * idv| <= 127 (idv = 127 / amax of the block): adding
// 1.5 * 2^23 rounds to nearest-even exactly as rintf does and leaves the two's-complement code in the low byte of the sum,
// so round / convert / clamp / shift-or become one add and three byte permutes.  The product is rounded to fp32 first, as
// in the reference (the build never contracts a * b + c).
__device__ __forceinline__ uint32_t q8_pack4(const float* v, float idv) {
  uint32_t b[4];
#pragma unroll
  for (int e = 0; e < 4; e++) b[e] = __float_as_uint(v[e] * idv + 12582912.0f);
  return __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u) | __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
}

// The Q8_0 image of activation rows that the decode GEMV copies into LDS: for MT rows of nb blocks, 16-byte planes of
// elements 0..15 and 16..31 of every block, then the fp32 effective scales, then -8 * sum(codes).
struct QImage {
  unsigned char* base;  // null: no image wanted
  int MT, nb, x86_scale;
};
// Four neighbouring lanes (a quad) hold the four eighths of one 32-element block: lane j of the quad has elements
// 8j..8j+7.  Same arithmetic as quantize_row_q8_0 (quantize_q8.cpp:106-190), same image as quant_image_kernel writes.
__device__ __forceinline__ void quad_quantize_to_image(const float (&v)[8], const QImage& q, int m, int blk, int j, bool write) {
  float amax = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[e]));
  amax = fmaxf(amax, dpp_f<0xB1>(amax));
  amax = fmaxf(amax, dpp_f<0x4E>(amax));
  const float d = amax / 127.f;
  const float idv = (amax != 0.f) ? 127.f / amax : 0.f;
  const uint32_t pk[2] = {q8_pack4(&v[0], idv), q8_pack4(&v[4], idv)};
  int sum = __builtin_amdgcn_sdot4((int)pk[0], 0x01010101, 0, false);
  sum = __builtin_amdgcn_sdot4((int)pk[1], 0x01010101, sum, false);
  sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xf, 0xf, true);
  sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xf, 0xf, true);
  if (!write) return;
  const int mnb = q.MT * q.nb;
  const int id = m * q.nb + blk;
  u32x4* lo = reinterpret_cast<u32x4*>(q.base);
  u32x4* hi = lo + mnb;
  float* sd = reinterpret_cast<float*>(hi + mnb);
  int* sn = reinterpret_cast<int*>(sd + mnb);
  u32x2* dst = reinterpret_cast<u32x2*>((j < 2 ? lo : hi) + id) + (j & 1);
  *dst = u32x2{pk[0], pk[1]};
  if (j == 0) {
    uint16_t bits = f32_to_f16bits(d);
    if (q.x86_scale) bits = x86_scale_bits(bits);
    sd[id] = f16bits_to_f32(bits);
    sn[id] = -8 * sum;
  }
}
// rows of the image beyond the real ones read as zero blocks
__device__ __forceinline__ void image_zero_row(const QImage& q, int m, int tid, int nthreads) {
  const int mnb = q.MT * q.nb;
  u32x4* lo = reinterpret_cast<u32x4*>(q.base);
  u32x4* hi = lo + mnb;
  float* sd = reinterpret_cast<float*>(hi + mnb);
  int* sn = reinterpret_cast<int*>(sd + mnb);
  for (int b = tid; b < q.nb; b += nthreads) {
    lo[m * q.nb + b] = u32x4{0, 0, 0, 0};
    hi[m * q.nb + b] = u32x4{0, 0, 0, 0};
    sd[m * q.nb + b] = 0.f;
    sn[m * q.nb + b] = 0;
  }
}

// One 32-element activation block, raw: fp32 input = 8 x 16 B, bf16 input = 4 x 16 B.  Loading and converting are
// separate steps so that a caller can issue other loads in between.
template <int XT>
__device__ __forceinline__ void load_block_raw_t(const void* x, int64_t elem_offset, u32x4 (&raw)[XT == MLLM_HIP_F32 ? 8 : 4]) {
  if (XT == MLLM_HIP_F32) {
    const u32x4* p = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(x) + elem_offset);
#pragma unroll
    for (int i = 0; i < 8; i++) raw[i] = p[i];
  } else {
    const u32x4* p = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(x) + elem_offset);
#pragma unroll
    for (int i = 0; i < 4; i++) raw[i] = p[i];
  }
}
template <int XT>
__device__ __forceinline__ void block_raw_to_f32_t(const u32x4 (&raw)[XT == MLLM_HIP_F32 ? 8 : 4], float (&v)[32]) {
  if (XT == MLLM_HIP_F32) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      v[4 * i + 0] = __uint_as_float(raw[i].x); v[4 * i + 1] = __uint_as_float(raw[i].y);
      v[4 * i + 2] = __uint_as_float(raw[i].z); v[4 * i + 3] = __uint_as_float(raw[i].w);
    }
  } else {  // bf16 -> fp32 is exact
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t w[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
      for (int j = 0; j < 4; j++) {
        v[8 * i + 2 * j + 0] = __uint_as_float(w[j] << 16);
        v[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
    }
  }
}
__device__ __forceinline__ void load_block_raw(const void* x, int x_dtype, int64_t elem_offset, u32x4 (&raw)[8]) {
  if (x_dtype == MLLM_HIP_F32) {
    const u32x4* p = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(x) + elem_offset);
#pragma unroll
    for (int i = 0; i < 8; i++) raw[i] = p[i];
  } else {
    const u32x4* p = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(x) + elem_offset);
#pragma unroll
    for (int i = 0; i < 4; i++) raw[i] = p[i];
  }
}
__device__ __forceinline__ void block_raw_to_f32(const u32x4 (&raw)[8], int x_dtype, float (&v)[32]) {
  if (x_dtype == MLLM_HIP_F32) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      v[4 * i + 0] = __uint_as_float(raw[i].x); v[4 * i + 1] = __uint_as_float(raw[i].y);
      v[4 * i + 2] = __uint_as_float(raw[i].z); v[4 * i + 3] = __uint_as_float(raw[i].w);
    }
  } else {  // bf16 -> fp32 is exact
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t w[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
      for (int j = 0; j < 4; j++) {
        v[8 * i + 2 * j + 0] = __uint_as_float(w[j] << 16);
        v[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
    }
  }
}
__device__ __forceinline__ void load_block_f32(const void* x, int x_dtype, int64_t elem_offset, float (&v)[32]) {
  u32x4 raw[8];
  load_block_raw(x, x_dtype, elem_offset, raw);
  block_raw_to_f32(raw, x_dtype, v);
}

// packed weight layout: code planes of 16 B per block (Q4_0: one plane, Q8_0: two), then the fp16 scales [N][nbp]
struct PackedView {
  const u32x4* q0;      // Q4_0: 32 nibbles of the block; Q8_0: elements 0..15
  const u32x4* q1;      // Q8_0: elements 16..31 (unused for Q4_0)
  const uint16_t* d;    // IEEE fp16 patterns
};
__host__ __device__ inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
__host__ __device__ inline size_t packed_plane_bytes(int64_t N, int64_t K) { return align_up((size_t)N * (K / QK) * 16, 256); }
// scale rows are padded to a multiple of 8 entries (16 bytes) so that a row's scales can be fetched with 16-byte loads
__host__ __device__ inline int64_t scale_row_stride(int64_t K) { return (int64_t)align_up((size_t)(K / QK), 8); }
__host__ __device__ inline size_t packed_bytes(int wtype, int64_t N, int64_t K) {
  return packed_plane_bytes(N, K) * (wtype == MLLM_HIP_Q4_0 ? 1 : 2) + align_up((size_t)N * scale_row_stride(K) * 2, 256);
}
__host__ __device__ inline PackedView packed_view(int wtype, const void* packed, int64_t N, int64_t K) {
  const char* p = reinterpret_cast<const char*>(packed);
  size_t pl = packed_plane_bytes(N, K);
  PackedView v;
  v.q0 = reinterpret_cast<const u32x4*>(p);
  v.q1 = reinterpret_cast<const u32x4*>(p + pl);
  v.d = reinterpret_cast<const uint16_t*>(p + pl * (wtype == MLLM_HIP_Q4_0 ? 1 : 2));
  return v;
}

}  // namespace mllmhip
