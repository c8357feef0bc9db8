// Offline K-quant weight quantizers on the GPU: fp32 rows -> the reference's super-blocks (256 weights)
//   Q4_K (144 B)  quantize_row_q4_K_reference, mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q4.cpp:184-282, with the
//                 per-sub-block search make_qkx2_quants (:97-168; 32 weights, 4 bits, 21 candidate scales, squared error
//                 weighted by sqrt(mean x^2) + |x|)
//   Q6_K (210 B)  quantize_row_q6_K_reference, quantize_q6.cpp:34-106, with make_qx_quants (quantize.hpp:268-325; 16 weights,
//                 weights x^2, 18 candidate scales)
// used by the reference's model converter (tools/mllm-quantizer/schema/gguf.cpp:211-250).
//
// Byte-exact with the CPU code: a sub-block's search is one thread that performs the reference's fp32 operations in the
// reference's order (the build never contracts a * b + c and divides / takes square roots correctly rounded); what the
// reference then does per super-block (largest scale, 6-bit / int8 sub-block scales, the fp16 fields, the final codes, the
// interleaved code bytes) goes through LDS between the threads of that super-block.  A load-time tool: one launch for a
// whole matrix, nothing tuned beyond keeping every lane busy.
#include "qcommon.h"

namespace mllmhip {

// round to nearest even through the 1.5 * 2^23 constant (quantize.hpp:261-267)
__device__ __forceinline__ int kq_nearest_int(float fval) {
  const float val = fval + 12582912.f;
  return (int)(__float_as_uint(val) & 0x007fffffu) - 0x00400000;
}

// how a computed fp16 pattern is left in the file, and what the quantizer reads back from it
__device__ __forceinline__ uint16_t kq_store_field(uint16_t pattern, int x86) { return x86 ? f32_to_f16bits((float)pattern) : pattern; }
__device__ __forceinline__ float kq_field_value(uint16_t pattern, int x86) { return f16bits_to_f32(x86 ? x86_scale_bits(pattern) : pattern); }

// ---- Q4_K ---------------------------------------------------------------------------------------------------------
constexpr int Q4K_SB_PER_WG = 32;  // 256 threads = 32 super-blocks x 8 sub-blocks

__global__ __launch_bounds__(256) void quantize_q4k_kernel(const float* __restrict__ w, unsigned char* __restrict__ blocks, int64_t nsb, int x86) {
  __shared__ float s_scale[Q4K_SB_PER_WG][8], s_min[Q4K_SB_PER_WG][8];
  __shared__ unsigned char s_ls[Q4K_SB_PER_WG][8], s_lm[Q4K_SB_PER_WG][8];
  __shared__ __align__(16) unsigned char s_L[Q4K_SB_PER_WG][256];
  const int tid = threadIdx.x, sl = tid >> 3, j = tid & 7;
  const int64_t sb = (int64_t)blockIdx.x * Q4K_SB_PER_WG + sl;
  const bool live = sb < nsb;
  float x[32];
  {
    const f32x4* p = reinterpret_cast<const f32x4*>(w + (live ? sb : 0) * 256 + 32 * j);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const f32x4 v = p[i];
      x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
    }
  }
  // weights of the squared error: sqrt(mean of x^2) + |x|
  float sum_x2 = 0;
#pragma unroll
  for (int l = 0; l < 32; l++) sum_x2 += x[l] * x[l];
  const float av_x = sqrtf(sum_x2 / 32);
  float wt[32];
#pragma unroll
  for (int l = 0; l < 32; l++) wt[l] = av_x + fabsf(x[l]);

  // ---- the search over this sub-block (nmax 15, rmin -1, rdelta 0.1, 20 steps) ----
  unsigned char L[32];
  float scale, the_min;
  {
    float mn = x[0], mx = x[0];
    float sum_w = wt[0];
    float sum_x = sum_w * x[0];
#pragma unroll
    for (int i = 1; i < 32; i++) {
      if (x[i] < mn) mn = x[i];
      if (x[i] > mx) mx = x[i];
      sum_w += wt[i];
      sum_x += wt[i] * x[i];
    }
    if (mn > 0) mn = 0;
    if (mx == mn) {
#pragma unroll
      for (int i = 0; i < 32; i++) L[i] = 0;
      the_min = -mn;
      scale = 0.f;
    } else {
      float iscale = 15 / (mx - mn);
      scale = 1 / iscale;
      float best = 0;
#pragma unroll
      for (int i = 0; i < 32; i++) {
        int l = kq_nearest_int(iscale * (x[i] - mn));
        l = max(0, min(15, l));
        L[i] = (unsigned char)l;
        float diff = scale * (float)l + mn - x[i];
        diff = diff * diff;
        best += wt[i] * diff;
      }
      for (int is = 0; is <= 20; is++) {
        iscale = (-1.f + 0.1f * is + 15) / (mx - mn);  // (mn is the best candidate's offset so far, as in the reference)
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        unsigned char Laux[32];
#pragma unroll
        for (int i = 0; i < 32; i++) {
          int l = kq_nearest_int(iscale * (x[i] - mn));
          l = max(0, min(15, l));
          Laux[i] = (unsigned char)l;
          const float wl = wt[i] * (float)l;
          sum_l += wl;
          sum_l2 += wl * (float)l;
          sum_xl += wl * x[i];
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
#pragma unroll
          for (int i = 0; i < 32; i++) {
            float diff = this_scale * (float)Laux[i] + this_min - x[i];
            diff = diff * diff;
            err += wt[i] * diff;
          }
          if (err < best) {
#pragma unroll
            for (int i = 0; i < 32; i++) L[i] = Laux[i];
            best = err;
            scale = this_scale;
            mn = this_min;
          }
        }
      }
      the_min = -mn;
    }
  }
  s_scale[sl][j] = scale;
  s_min[sl][j] = the_min;
  __syncthreads();

  // ---- the super-block: largest scale and offset, 6-bit sub-block values, the two fp16 fields ----
  float max_scale = 0, max_min = 0;
#pragma unroll
  for (int u = 0; u < 8; u++) {
    if (s_scale[sl][u] > max_scale) max_scale = s_scale[sl][u];
    if (s_min[sl][u] > max_min) max_min = s_min[sl][u];
  }
  const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
  const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
  unsigned char ls = (unsigned char)kq_nearest_int(inv_scale * scale);
  unsigned char lm = (unsigned char)kq_nearest_int(inv_min * the_min);
  ls = ls < 63 ? ls : 63;
  lm = lm < 63 ? lm : 63;
  s_ls[sl][j] = ls;
  s_lm[sl][j] = lm;
  const uint16_t pd = f32_to_f16bits(max_scale / 63.f), pm = f32_to_f16bits(max_min / 63.f);
  // final codes of this sub-block against the stored scale and offset (a sub-block whose scale came out 0 keeps the search's)
  const float d = kq_field_value(pd, x86) * (float)ls;
  if (d != 0.0f) {
    const float dm = kq_field_value(pm, x86) * (float)lm;
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const int l = kq_nearest_int((x[i] + dm) / d);
      L[i] = (unsigned char)max(0, min(15, l));
    }
  }
#pragma unroll
  for (int i = 0; i < 8; i++)
    reinterpret_cast<uint32_t*>(&s_L[sl][32 * j])[i] =
        (uint32_t)L[4 * i] | ((uint32_t)L[4 * i + 1] << 8) | ((uint32_t)L[4 * i + 2] << 16) | ((uint32_t)L[4 * i + 3] << 24);
  __syncthreads();
  if (!live) return;

  unsigned char* y = blocks + sb * 144;  // 144 = 9 x 16: a block keeps the 16-byte alignment of the buffer
  if (j == 0) {
    // d, dmin, then the twelve bytes of 6-bit values: scales 0..3 and mins 0..3 in the low six bits of bytes 0..7, scales / mins
    // 4..7 as nibbles of bytes 8..11 with their two high bits on top of bytes 0..7
    unsigned char sc[12];
#pragma unroll
    for (int u = 0; u < 12; u++) sc[u] = 0;
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const unsigned char a = s_ls[sl][u], b = s_lm[sl][u];
      if (u < 4) {
        sc[u] = a;
        sc[u + 4] = b;
      } else {
        sc[u + 4] = (unsigned char)((a & 0xF) | ((b & 0xF) << 4));
        sc[u - 4] |= (unsigned char)((a >> 4) << 6);
        sc[u] |= (unsigned char)((b >> 4) << 6);
      }
    }
    uint32_t o[4];
    o[0] = (uint32_t)kq_store_field(pd, x86) | ((uint32_t)kq_store_field(pm, x86) << 16);
#pragma unroll
    for (int u = 0; u < 3; u++)
      o[1 + u] = (uint32_t)sc[4 * u] | ((uint32_t)sc[4 * u + 1] << 8) | ((uint32_t)sc[4 * u + 2] << 16) | ((uint32_t)sc[4 * u + 3] << 24);
    *reinterpret_cast<u32x4*>(y) = u32x4{o[0], o[1], o[2], o[3]};
  }
  // code bytes 16 j .. 16 j + 15: byte b of the 128 = element 64 (b / 32) + b % 32 in the low nibble, that element + 32 in the high one
  {
    const int g = j >> 1, l0 = 16 * (j & 1);
    const u32x4 lo = *reinterpret_cast<const u32x4*>(&s_L[sl][64 * g + l0]);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(&s_L[sl][64 * g + 32 + l0]);
    *reinterpret_cast<u32x4*>(y + 16 + 16 * j) = u32x4{lo.x | (hi.x << 4), lo.y | (hi.y << 4), lo.z | (hi.z << 4), lo.w | (hi.w << 4)};
  }
}

// ---- Q6_K ---------------------------------------------------------------------------------------------------------
constexpr int Q6K_SB_PER_WG = 16;  // 256 threads = 16 super-blocks x 16 groups of 16 weights

__global__ __launch_bounds__(256) void quantize_q6k_kernel(const float* __restrict__ w, unsigned char* __restrict__ blocks, int64_t nsb, int x86) {
  __shared__ float s_scale[Q6K_SB_PER_WG][16];
  __shared__ __align__(16) unsigned char s_L[Q6K_SB_PER_WG][256];
  const int tid = threadIdx.x, sl = tid >> 4, ib = tid & 15;
  const int64_t sb = (int64_t)blockIdx.x * Q6K_SB_PER_WG + sl;
  const bool live = sb < nsb;
  float x[16];
  {
    const f32x4* p = reinterpret_cast<const f32x4*>(w + (live ? sb : 0) * 256 + 16 * ib);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const f32x4 v = p[i];
      x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
    }
  }
  // ---- the search over this group (nmax 32, error weights x^2, candidate scales -(32 + 0.1 is) / max, is = -9 .. 9) ----
  int L[16];  // codes with the offset of 32 applied: 0 .. 63
  float scale;
  {
    float mx = 0, amax = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const float ax = fabsf(x[i]);
      if (ax > amax) {
        amax = ax;
        mx = x[i];
      }
    }
    if (amax < 1e-30f) {
#pragma unroll
      for (int i = 0; i < 16; i++) L[i] = 0;
      scale = 0.f;
    } else {
      float iscale = -32 / mx;
      float sumlx = 0, suml2 = 0;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        int l = kq_nearest_int(iscale * x[i]);
        l = max(-32, min(31, l));
        L[i] = l + 32;
        const float wx = x[i] * x[i];
        sumlx += wx * x[i] * (float)l;
        suml2 += wx * (float)l * (float)l;
      }
      scale = sumlx / suml2;
      float best = scale * sumlx;
      for (int is = -9; is <= 9; is++) {
        if (is == 0) continue;
        iscale = -(32 + 0.1f * is) / mx;
        sumlx = 0;
        suml2 = 0;
        int Lt[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
          int l = kq_nearest_int(iscale * x[i]);
          l = max(-32, min(31, l));
          Lt[i] = l + 32;
          const float wx = x[i] * x[i];
          sumlx += wx * x[i] * (float)l;
          suml2 += wx * (float)l * (float)l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
#pragma unroll
          for (int i = 0; i < 16; i++) L[i] = Lt[i];
          scale = sumlx / suml2;
          best = scale * sumlx;
        }
      }
    }
  }
  s_scale[sl][ib] = scale;
  __syncthreads();

  // ---- the super-block: the scale of largest magnitude (the first one of that magnitude), int8 group scales, fp16 d ----
  float max_scale = 0, max_abs = 0;
#pragma unroll
  for (int u = 0; u < 16; u++) {
    const float s = s_scale[sl][u], a = fabsf(s);
    if (a > max_abs) {
      max_abs = a;
      max_scale = s;
    }
  }
  const bool zero_block = max_abs == 0.f;
  int sc = 0;
  uint16_t pd = 0;
  if (!zero_block) {
    const float iscale = -128.f / max_scale;
    pd = f32_to_f16bits(1 / iscale);
    sc = min(127, kq_nearest_int(iscale * scale));
    sc = (int)(int8_t)sc;
    const float d = kq_field_value(pd, x86) * (float)sc;
    if (d != 0.f) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        int l = kq_nearest_int(x[i] / d);
        l = max(-32, min(31, l));
        L[i] = l + 32;
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 16; i++) L[i] = 0;
  }
#pragma unroll
  for (int i = 0; i < 4; i++)
    reinterpret_cast<uint32_t*>(&s_L[sl][16 * ib])[i] =
        (uint32_t)L[4 * i] | ((uint32_t)L[4 * i + 1] << 8) | ((uint32_t)L[4 * i + 2] << 16) | ((uint32_t)L[4 * i + 3] << 24);
  __syncthreads();
  if (!live) return;

  // 210-byte blocks are only 2-byte aligned: two-byte stores.  Thread ib writes bytes 8 ib .. 8 ib + 7 of the low nibbles, 4 ib ..
  // 4 ib + 3 of the high bit pairs, its own scale; thread 0 also d.
  unsigned char* y = blocks + sb * 210;
  const unsigned char* Ls = s_L[sl];
  uint16_t* ql = reinterpret_cast<uint16_t*>(y) + 4 * ib;
#pragma unroll
  for (int h = 0; h < 4; h++) {
    uint32_t pair = 0;
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const int b = 8 * ib + 2 * h + e, n = b >> 6, c = b & 63;
      const int base = 128 * n + c;  // c < 32: elements c and c + 64 of the half; else, with l = c - 32, elements l + 32 and l + 96
      const unsigned char v = (unsigned char)((Ls[base] & 0xF) | ((Ls[base + 64] & 0xF) << 4));
      pair |= (uint32_t)v << (8 * e);
    }
    ql[h] = (uint16_t)pair;
  }
  uint16_t* qh = reinterpret_cast<uint16_t*>(y + 128) + 2 * ib;
#pragma unroll
  for (int h = 0; h < 2; h++) {
    uint32_t pair = 0;
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const int b = 4 * ib + 2 * h + e, n = b >> 5, l = b & 31;
      const unsigned char* q = Ls + 128 * n + l;
      const unsigned char v = (unsigned char)((q[0] >> 4) | ((q[32] >> 4) << 2) | ((q[64] >> 4) << 4) | ((q[96] >> 4) << 6));
      pair |= (uint32_t)v << (8 * e);
    }
    qh[h] = (uint16_t)pair;
  }
  y[192 + ib] = (unsigned char)(int8_t)sc;
  if (ib == 0) *reinterpret_cast<uint16_t*>(y + 208) = zero_block ? (uint16_t)0 : kq_store_field(pd, x86);
}

}  // namespace mllmhip

using namespace mllmhip;

MLLM_API int mllm_hip_kq_quantize_weight_blocks(int wtype, const float* w, void* blocks, int weight_scale_mode, int64_t N, int64_t K,
                                                void* stream) {
  if ((wtype != MLLM_HIP_Q4_K && wtype != MLLM_HIP_Q6_K) || !w || !blocks || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (weight_scale_mode != MLLM_HIP_SCALE_IEEE && weight_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (K % 256) return MLLM_HIP_E_SHAPE;
  const int64_t nsb = N * (K / 256);
  if (nsb > ((int64_t)1 << 31) * 16) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(w) % 16 || reinterpret_cast<uintptr_t>(blocks) % (wtype == MLLM_HIP_Q4_K ? 16 : 2)) return MLLM_HIP_E_ALIGN;
  const int x86 = weight_scale_mode == MLLM_HIP_SCALE_X86_REF;
  if (wtype == MLLM_HIP_Q4_K)
    hipLaunchKernelGGL(quantize_q4k_kernel, dim3((unsigned)((nsb + Q4K_SB_PER_WG - 1) / Q4K_SB_PER_WG)), dim3(256), 0, (hipStream_t)stream, w,
                       static_cast<unsigned char*>(blocks), nsb, x86);
  else
    hipLaunchKernelGGL(quantize_q6k_kernel, dim3((unsigned)((nsb + Q6K_SB_PER_WG - 1) / Q6K_SB_PER_WG)), dim3(256), 0, (hipStream_t)stream, w,
                       static_cast<unsigned char*>(blocks), nsb, x86);
  return (int)hipGetLastError();
}
