// Q4_K / Q6_K Linear for gfx950: super-block formats of 256 weights with Q8_K activations (the formats the shipped
// Qwen3-MoE recipe quantizes to).  Decode GEMV for up to eight activation rows; more rows run as groups of eight.
//
// Arithmetic follows the reference's x86 CPU path:
//   activation quantization  quantize_row_q8_K_reference   mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.cpp:215-248
//   Q4_K dot                 vec_dot_q4_K_q8_K (AVX2)       mllm/backends/cpu/kernels/common/ggml/vec_dot.cpp:498-560
//   Q6_K dot                 vec_dot_q6_K_q8_K (AVX2)       mllm/backends/cpu/kernels/common/ggml/vec_dot.cpp:955-1044
//   dequantization probes    dequantize_row_q4_K / _q6_K    quantize_q4.cpp:284-312, quantize_q6.cpp:108-133
//   call site                ggml::mat_mul generic branch    mllm/backends/cpu/kernels/common/ggml/matmul.cpp:147-189,300-360
// The integer work (codes, sums of 16, sub-block-scaled dot products per super-block) is exact; the fp32 accumulation
// runs per lane and is reduced over the lanes of a row, a different order than the CPU's eight lanes.
//
// HBM-bound like the Q4_0 / Q8_0 GEMV: a launch streams 144 (Q4_K) or 210 (Q6_K) bytes per 256 weights once, as 16-byte
// loads that are contiguous across the lanes of a group.  The reference's array-of-structures blocks (210 is not even a
// multiple of 4) are split at load time into planes of 16-byte records.
#include <initializer_list>

#include "qcommon.h"
#include "qgemm_layout.h"

#include "kquant_layout.h"

namespace mllmhip {

// what an fp16 field reads as: the IEEE pattern itself, or (files of the x86 build) the number stored there taken as
// the pattern
__device__ __forceinline__ uint16_t field_bits(const uint8_t* p, int x86) {
  const uint16_t raw = (uint16_t)p[0] | ((uint16_t)p[1] << 8);
  if (!x86) return raw;
  const float num = f16bits_to_f32(raw);
  return (num >= 0.f && num < 65536.f) ? (uint16_t)(uint32_t)num : (uint16_t)0;
}
__device__ __forceinline__ uint32_t bytes_u32(const uint8_t* p) {
  return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

// ---- scale decoding ----------------------------------------------------------------------------------------------------
// the 6-bit scales and mins of a Q4_K super-block as bytes: sc[0..7] in (lo, hi) of `sc`, mins likewise
// (get_scale_min_k4, quantize.hpp; the same bit shuffle as vec_dot.cpp:507-512)
struct K4Scales {
  uint32_t sc0, sc1, mn0, mn1;
};
__device__ __forceinline__ K4Scales k4_scales(uint32_t u0, uint32_t u1, uint32_t u2) {
  K4Scales r;
  r.mn1 = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
  r.mn0 = u1 & 0x3f3f3f3fu;
  r.sc1 = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
  r.sc0 = u0 & 0x3f3f3f3fu;
  return r;
}
__device__ __forceinline__ int byte_of(uint32_t lo, uint32_t hi, int k) {  // k = 0..7
  return (int)(((k < 4 ? lo : hi) >> (8 * (k & 3))) & 0xffu);
}

// one thread per 16-byte record of plane A (Q4_K: 8 per super-block; Q6_K: 8 per super-block); thread 0 of a super-block
// also writes the small planes
__global__ void kq_prepack_kernel(int wtype, const uint8_t* __restrict__ blocks, int x86, KView v, int64_t nsb_total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t sb = i >> 3;
  const int c = (int)(i & 7);
  if (sb >= nsb_total) return;
  u32x4* A = const_cast<u32x4*>(v.a);
  u32x4* S = const_cast<u32x4*>(v.s);
  if (wtype == MLLM_HIP_Q4_K) {
    const uint8_t* b = blocks + sb * 144;
    const uint8_t* q = b + 16 + 16 * c;
    A[sb * 8 + c] = u32x4{bytes_u32(q), bytes_u32(q + 4), bytes_u32(q + 8), bytes_u32(q + 12)};
    if (c == 0) {
      const K4Scales k = k4_scales(bytes_u32(b + 4), bytes_u32(b + 8), bytes_u32(b + 12));
      uint32_t rec[4];
#pragma unroll
      for (int p = 0; p < 4; p++)
        rec[p] = (uint32_t)byte_of(k.sc0, k.sc1, 2 * p) | ((uint32_t)byte_of(k.sc0, k.sc1, 2 * p + 1) << 8) |
                 ((uint32_t)byte_of(k.mn0, k.mn1, 2 * p) << 16) | ((uint32_t)byte_of(k.mn0, k.mn1, 2 * p + 1) << 24);
      S[sb] = u32x4{rec[0], rec[1], rec[2], rec[3]};
      reinterpret_cast<uint32_t*>(const_cast<uint16_t*>(v.d))[sb] = (uint32_t)field_bits(b, x86) | ((uint32_t)field_bits(b + 2, x86) << 16);
    }
  } else {
    const uint8_t* b = blocks + sb * 210;
    const uint8_t* q = b + 16 * c;
    A[sb * 8 + c] = u32x4{bytes_u32(q), bytes_u32(q + 4), bytes_u32(q + 8), bytes_u32(q + 12)};
    if (c < 4) {
      const uint8_t* hq = b + 128 + 16 * c;
      const_cast<u32x4*>(v.h)[sb * 4 + c] = u32x4{bytes_u32(hq), bytes_u32(hq + 4), bytes_u32(hq + 8), bytes_u32(hq + 12)};
    }
    if (c == 0) {
      const uint8_t* s = b + 192;
      S[sb] = u32x4{bytes_u32(s), bytes_u32(s + 4), bytes_u32(s + 8), bytes_u32(s + 12)};
      const_cast<uint16_t*>(v.d)[sb] = field_bits(b + 208, x86);
    }
  }
}

// ---- dequantization probe ------------------------------------------------------------------------------------------------
__global__ void kq_dequantize_kernel(int wtype, KView v, float* __restrict__ w, int64_t nsb_total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // one thread per element
  const int64_t sb = i >> 8;
  const int e = (int)(i & 255);
  if (sb >= nsb_total) return;
  const uint8_t* A = reinterpret_cast<const uint8_t*>(v.a) + sb * 128;
  if (wtype == MLLM_HIP_Q4_K) {
    const uint32_t dd = reinterpret_cast<const uint32_t*>(v.d)[sb];
    const float d = f16bits_to_f32((uint16_t)(dd & 0xffff)), mn = f16bits_to_f32((uint16_t)(dd >> 16));
    const int j = e >> 5, l = e & 31;  // sub-block, element
    const uint32_t rec = reinterpret_cast<const uint32_t*>(v.s)[sb * 4 + (j >> 1)];
    const int q = (j & 1) ? (A[32 * (j >> 1) + l] >> 4) : (A[32 * (j >> 1) + l] & 0xF);
    const float d1 = d * (float)((rec >> (8 * (j & 1))) & 0xffu), m1 = mn * (float)((rec >> (16 + 8 * (j & 1))) & 0xffu);
    w[i] = d1 * (float)q - m1;
  } else {
    const uint8_t* H = reinterpret_cast<const uint8_t*>(v.h) + sb * 64;
    const int8_t* sc = reinterpret_cast<const int8_t*>(v.s) + sb * 16;
    const int n = e >> 7, r = e & 127, g = r >> 5, l = r & 31;
    int lo = A[64 * n + ((g & 1) ? 32 : 0) + l];
    lo = (g >= 2) ? (lo >> 4) : (lo & 0xF);
    const int hi = (H[32 * n + l] >> (2 * g)) & 3;
    const int q = (int)(int8_t)(lo | (hi << 4)) - 32;
    const float d = f16bits_to_f32(v.d[sb]);
    w[i] = d * (float)sc[e >> 4] * (float)q;
  }
}

// ---- Q8_K quantization of activations ---------------------------------------------------------------------------------------
// 32 neighbouring lanes (half a wave) hold one super-block, eight consecutive elements per lane; both halves of the wave
// must be active or idle as a whole.  The reference takes the element of largest magnitude WITH its sign, the first one
// when several are equal: the magnitude goes through a plain max butterfly, the sign comes from the first lane (lowest set
// bit of a ballot) that holds an element of that magnitude and, in it, the first such element.  Codes: the product is
// rounded to fp32, then adding 1.5 * 2^23 rounds to nearest-even as rintf does and leaves the two's-complement code in the
// low byte; the clamp to 127 is an integer min on the bits of that (positive) sum.  Outputs of a lane: its eight codes (two dwords), the sum of its
// eight codes, the block scale.
struct Q8KItem {
  uint32_t q0, q1;
  int sum8;
  float d;
};
__device__ __forceinline__ Q8KItem quantize_q8k_item(const float (&v)[8], int lane) {
  // magnitudes compare as their bit patterns: the butterfly runs on unsigned integers
  uint32_t am = 0u;
#pragma unroll
  for (int e = 0; e < 8; e++) am = max(am, __float_as_uint(v[e]) & 0x7fffffffu);
  am = max(am, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)am, 0xB1, 0xf, 0xf, true));   // lane ^ 1
  am = max(am, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)am, 0x4E, 0xf, 0xf, true));   // lane ^ 2
  am = max(am, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)am, 0x141, 0xf, 0xf, true));  // half-row mirror
  am = max(am, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)am, 0x140, 0xf, 0xf, true));  // row mirror
  am = max(am, (uint32_t)__shfl_xor((int)am, 16, 64));
  const float amax = __uint_as_float(am);
  float sel = 0.f;  // the lane's first element of that magnitude
#pragma unroll
  for (int e = 7; e >= 0; e--) sel = ((__float_as_uint(v[e]) & 0x7fffffffu) == am) ? v[e] : sel;
  const bool hit = (__float_as_uint(sel) & 0x7fffffffu) == am, neg = (__float_as_uint(sel) >> 31) != 0u;
  const unsigned long long mh = __ballot(hit), mn = __ballot(hit && neg);
  const uint32_t h32 = (lane & 32) ? (uint32_t)(mh >> 32) : (uint32_t)mh;
  const uint32_t n32 = (lane & 32) ? (uint32_t)(mn >> 32) : (uint32_t)mn;
  const bool negative = (n32 & (h32 & (0u - h32))) != 0u;
  Q8KItem r{0u, 0u, 0, 0.f};
  if (amax == 0.f) return r;
  const float iscale = -128.f / (negative ? -amax : amax);
  uint32_t b[8];
#pragma unroll
  for (int e = 0; e < 8; e++) b[e] = (uint32_t)min((int)__float_as_uint(iscale * v[e] + 12582912.0f), 0x4B40007F);  // bits of 1.5 * 2^23 + 127
  r.q0 = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u) | __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
  r.q1 = __builtin_amdgcn_perm(b[5], b[4], 0x0c0c0400u) | __builtin_amdgcn_perm(b[7], b[6], 0x04000c0cu);
  r.sum8 = __builtin_amdgcn_sdot4((int)r.q1, 0x01010101, __builtin_amdgcn_sdot4((int)r.q0, 0x01010101, 0, false), false);
  r.d = 1.f / iscale;
  return r;
}

template <int XT>
__device__ __forceinline__ void load8(const void* x, int64_t elem, float (&v)[8]) {
  if (XT == MLLM_HIP_F32) {
    const f32x4* p = reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(x) + elem);
    const f32x4 a = p[0], b = p[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    const u32x4 r = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(x) + elem);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      v[2 * j + 0] = __uint_as_float(w[j] << 16);
      v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}

// stand-alone form: codes int8 [rows][K], d fp32 [rows][K/256], sums of 16 int16 [rows][K/16]; items from `valid` on
// (rows beyond the real ones) are written as zeros.  Used as parity probe and, with the three arrays back to back, to
// write the image the GEMV copies into LDS.
constexpr int KQ_IMAGE = 2;  // activation "type": the quantized image instead of activations
__global__ __launch_bounds__(256) void quantize_q8k_kernel(const void* __restrict__ x, int x_dtype, int8_t* __restrict__ codes,
                                                           float* __restrict__ d, int16_t* __restrict__ bsums, int64_t nitems,
                                                           int64_t valid) {
  const int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x;  // nitems is a multiple of 32: whole half-waves
  if (it >= nitems) return;
  float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (it < valid) {
    if (x_dtype == MLLM_HIP_F32) load8<MLLM_HIP_F32>(x, it * 8, v);
    else load8<MLLM_HIP_BF16>(x, it * 8, v);
  }
  const Q8KItem r = quantize_q8k_item(v, threadIdx.x & 63);
  *reinterpret_cast<u32x2*>(codes + it * 8) = u32x2{r.q0, r.q1};
  const int s16 = r.sum8 + __builtin_amdgcn_update_dpp(0, r.sum8, 0xB1, 0xf, 0xf, true);  // with the neighbouring lane
  if ((it & 1) == 0) bsums[it >> 1] = (int16_t)s16;
  if ((it & 31) == 0) d[it >> 5] = r.d;
}

// ---- GEMV -------------------------------------------------------------------------------------------------------------
// One launch serves up to four weight matrices that share the activations and K (sibling projections): workgroups
// [wg_start[p], wg_start[p + 1]) belong to part p.
constexpr int KQ_MAX_PARTS = 4;
struct KGemvPart {
  KView w;
  const float* bias;
  float* y;
  int N;
};
struct KGemvArgs {
  KGemvPart part[KQ_MAX_PARTS];
  int wg_start[KQ_MAX_PARTS + 1];
  int nparts;
  const void* x;
  int M, nsb;  // nsb = K / 256
  // MoE slots (M = 1 only): blockIdx.y = slot; its expert's matrices lie slot_ids[slot] * estride bytes further in every plane,
  // its activation row is slot / slot_div, its output row is the slot.  slot_ids == null: a plain Linear.
  const int32_t* slot_ids;
  const float* x2;       // slots with fp32 x only: the activation is silu(x) * x2 (the MLP's product folded into the down GEMV)
  int silu_accurate;     // expf instead of the reference's polynomial (mllm_hip_set_exp_mode)
  int slot_E, slot_div, slot_div_slots;  // experts, pairs per activation row, number of slots (grid y)
  size_t estride;
  // MoE row tiles (matrix-core kernels, quantized image as input): blockIdx.y = a tile of up to eight expert-sorted positions
  // that share an expert.  The image holds img_rows rows; tile row m reads image row row_ids[row0 + m] / row_div (row_ids
  // null: row0 + m) and writes output row out_ids[row0 + m] (null: row0 + m).  tile_expert == null: a plain Linear.
  const int* tile_expert;
  const int* tile_row0;
  const int* tile_rows;
  const int* ntiles;
  const int* row_ids;
  const int* out_ids;
  int row_div;
  int img_rows;  // rows of the image (0: the kernel's row tile MT)
};
// the tile of this workgroup: how many rows it has, where they start, where the expert's matrices lie
struct KTile {
  int rows, row0;
  size_t eoff;
  bool active;
};
__device__ __forceinline__ KTile kq_tile(const KGemvArgs& a) {
  KTile t{a.M, 0, 0, true};
  if (a.tile_expert) {
    const int ti = blockIdx.y;
    if (ti >= min(a.ntiles[0], (int)gridDim.y)) {
      t.active = false;
      return t;
    }
    t.rows = a.tile_rows[ti];
    t.row0 = a.tile_row0[ti];
    t.eoff = (size_t)a.tile_expert[ti] * a.estride;
  }
  return t;
}
__device__ __forceinline__ int kq_tile_in_row(const KGemvArgs& a, const KTile& t, int m) {
  if (!a.tile_expert) return m;
  const int pos = t.row0 + min(m, t.rows - 1);  // rows past the tile repeat its last row; their results are dropped
  return a.row_ids ? a.row_ids[pos] / a.row_div : pos;
}
__device__ __forceinline__ int kq_tile_out_row(const KGemvArgs& a, const KTile& t, int m) {
  if (!a.tile_expert) return m;
  return a.out_ids ? a.out_ids[t.row0 + m] : t.row0 + m;
}
template <typename T>
__device__ __forceinline__ const T* kq_at(const T* p, size_t byte_offset) {
  return reinterpret_cast<const T*>(reinterpret_cast<const char*>(p) + byte_offset);
}
#define KBUF_OOB 0xffffffffu
#define KBUF_NT 2

// A unit = what one lane takes per step.  Q4_K: one 16-byte chunk of nibbles = 32 weights (eight units per super-block).
// Q6_K: one 16-byte chunk of high bits with its two chunks of low nibbles = 64 weights (four units per super-block).
template <int WT>
struct KUnit {
  u32x4 a, b, h, s;
  uint16_t d;
};
struct KRsrc {
  __amdgpu_buffer_rsrc_t a, h, s, d;
};

template <int WT>
__device__ __forceinline__ void load_unit(KUnit<WT>& u, const KRsrc& r, uint32_t sb_base, int unit, int units, bool row_ok) {
  const bool ok = row_ok && unit < units;
  if (WT == MLLM_HIP_Q4_K) {
    const uint32_t sb = sb_base + (uint32_t)(unit >> 3);
    u.a = __builtin_amdgcn_raw_buffer_load_b128(r.a, ok ? (sb * 8u + (uint32_t)(unit & 7)) * 16u : KBUF_OOB, 0, KBUF_NT);
    u.s.x = __builtin_amdgcn_raw_buffer_load_b32(r.s, ok ? sb * 16u + (uint32_t)((unit >> 1) & 3) * 4u : KBUF_OOB, 0, KBUF_NT);  // its pair's scales
    u.s.y = __builtin_amdgcn_raw_buffer_load_b32(r.d, ok ? sb * 4u : KBUF_OOB, 0, KBUF_NT);                                      // d, dmin
  } else {
    const uint32_t sb = sb_base + (uint32_t)(unit >> 2);
    const uint32_t n = (uint32_t)(unit >> 1) & 1u, t = (uint32_t)unit & 1u;
    u.a = __builtin_amdgcn_raw_buffer_load_b128(r.a, ok ? (sb * 8u + 4u * n + t) * 16u : KBUF_OOB, 0, KBUF_NT);
    u.b = __builtin_amdgcn_raw_buffer_load_b128(r.a, ok ? (sb * 8u + 4u * n + 2u + t) * 16u : KBUF_OOB, 0, KBUF_NT);
    u.h = __builtin_amdgcn_raw_buffer_load_b128(r.h, ok ? (sb * 4u + 2u * n + t) * 16u : KBUF_OOB, 0, KBUF_NT);
    u.s = __builtin_amdgcn_raw_buffer_load_b128(r.s, ok ? sb * 16u : KBUF_OOB, 0, KBUF_NT);
    u.d = __builtin_amdgcn_raw_buffer_load_b16(r.d, ok ? sb * 2u : KBUF_OOB, 0, KBUF_NT);
  }
}

__device__ __forceinline__ int dot16(const u32x4& w, const u32x4& x) {
  int acc = __builtin_amdgcn_sdot4((int)w.x, (int)x.x, 0, false);
  acc = __builtin_amdgcn_sdot4((int)w.y, (int)x.y, acc, false);
  acc = __builtin_amdgcn_sdot4((int)w.z, (int)x.z, acc, false);
  acc = __builtin_amdgcn_sdot4((int)w.w, (int)x.w, acc, false);
  return acc;
}
__device__ __forceinline__ int half16(uint32_t pair, int hi) { return (int)(int16_t)(hi ? (pair >> 16) : (pair & 0xffffu)); }

__device__ __forceinline__ void silu_mul8(float (&v)[8], const float* u, bool accurate) {
  const f32x4 a = reinterpret_cast<const f32x4*>(u)[0], b = reinterpret_cast<const f32x4*>(u)[1];
  const float uu[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
  for (int e = 0; e < 8; e++) v[e] = v[e] * (1.0f / (1.0f + (accurate ? expf(-v[e]) : exp_poly(-v[e])))) * uu[e];
}

// Workgroup = NW waves; a wave is cut into 64 / G groups of G lanes; a group owns R consecutive weight rows and its lanes
// stride over the row's units.  x is quantized to Q8_K once per workgroup into LDS: codes [MT][K], scales [MT][nsb], sums
// of 16 as int16 [MT][nsb][16].
// U = units a lane keeps in flight per row and trip.
// ONE: the row's units fit one trip (units <= G U): no second set of registers for the next trip.
template <int WT, int XT, int MT, int G, int R, int U, int LB = 256, bool ONE = false>
__global__ __launch_bounds__(LB) void kq_gemv_kernel(KGemvArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int nsb = a.nsb;
  const int K = nsb * QK_K;
  u32x4* s_q = reinterpret_cast<u32x4*>(smem);                         // [MT][K / 16]
  uint32_t* s_bs = reinterpret_cast<uint32_t*>(smem + (size_t)MT * K);  // [MT][nsb][8] pairs of int16 (sums of 16)
  float* s_d = reinterpret_cast<float*>(s_bs + (size_t)MT * nsb * 8);   // [MT][nsb]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int GROUPS = 64 / G;
  const int grp = lane / G, c0 = lane % G;
  const int nthreads = blockDim.x;  // 64 .. LB
  int pidx = 0;  // uniform: which matrix this workgroup works on
#pragma unroll
  for (int p = 1; p < KQ_MAX_PARTS; p++)
    if (p < a.nparts && (int)blockIdx.x >= a.wg_start[p]) pidx = p;
  const KGemvPart& pt = a.part[pidx];
  const int64_t row0 = ((int64_t)(blockIdx.x - a.wg_start[pidx]) * (nthreads >> 6) + wave) * (GROUPS * R) + (int64_t)grp * R;
  constexpr int UPS = WT == MLLM_HIP_Q4_K ? 8 : 4;  // units per super-block
  const int units = nsb * UPS;

  // MoE slot (uniform): expert offset of the weight planes, activation row, output row.  A slot whose expert id is outside
  // [0, E) computes with expert 0 and its row is never read (the combine pass skips it).
  size_t eoff = 0;
  int64_t xrow = 0, yrow = 0;
  if (MT == 1 && a.slot_ids) {
    const int slot = blockIdx.y;
    const int e = a.slot_ids[slot];
    eoff = (size_t)((e >= 0 && e < a.slot_E) ? e : 0) * a.estride;
    xrow = slot / a.slot_div;
    yrow = slot;
  }
  const char* xp = reinterpret_cast<const char*>(a.x) + xrow * K * (XT == MLLM_HIP_BF16 ? 2 : 4);
  const float* x2p = (XT == MLLM_HIP_F32 && MT == 1 && a.x2) ? a.x2 + xrow * K : nullptr;  // uniform
  KRsrc rs;
  {
    const uint32_t sbt = (uint32_t)pt.N * (uint32_t)nsb;
    auto at = [&](const void* base) { return const_cast<char*>(reinterpret_cast<const char*>(base) + eoff); };
    rs.a = __builtin_amdgcn_make_buffer_rsrc(at(pt.w.a), 0, sbt * 128u, 0x00020000);
    rs.h = __builtin_amdgcn_make_buffer_rsrc(at(WT == MLLM_HIP_Q6_K ? pt.w.h : pt.w.a), 0, sbt * 64u, 0x00020000);
    rs.s = __builtin_amdgcn_make_buffer_rsrc(at(pt.w.s), 0, sbt * 16u, 0x00020000);
    rs.d = __builtin_amdgcn_make_buffer_rsrc(at(pt.w.d), 0, sbt * (WT == MLLM_HIP_Q4_K ? 4u : 2u), 0x00020000);
  }
  // Memory requests return in order: the activations a thread will quantize (its first two items) are requested first,
  // then the first trip of weights, so that the quantization runs while the weights are still on their way.
  const int nitems = MT * (K >> 3);
  const int valid = a.M * (K >> 3);
  constexpr int XL = XT == KQ_IMAGE ? MLLM_HIP_F32 : XT;
  // (two rows: four items, or rows of 2560 elements leave half an item per thread to the loop further down, where it comes
  // back behind the weights)
  constexpr int NPRE = MT == 2 ? 4 : 2;
  u32x4 raw[NPRE][XL == MLLM_HIP_F32 ? 2 : 1];
  u32x4 raw2[2][2];
  if (XT != KQ_IMAGE) {
#pragma unroll
    for (int k = 0; k < NPRE; k++) {
      const int it = min(tid + k * nthreads, valid - 1);
      if (XL == MLLM_HIP_F32) {
        const u32x4* p = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(xp) + (int64_t)it * 8);
        raw[k][0] = p[0];
        raw[k][XL == MLLM_HIP_F32 ? 1 : 0] = p[1];
      } else {
        raw[k][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(xp) + (int64_t)it * 8);
      }
    }
    if (XT == MLLM_HIP_F32 && MT == 1 && x2p) {  // the second factor with the first (ahead of the weights: requests return in order)
#pragma unroll
      for (int k = 0; k < 2; k++) {
        const u32x4* p = reinterpret_cast<const u32x4*>(x2p + (int64_t)min(tid + k * nthreads, valid - 1) * 8);
        raw2[k][0] = p[0];
        raw2[k][1] = p[1];
      }
    }
    __asm__ volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  }
  KUnit<WT> cur[U][R];
#pragma unroll
  for (int uu = 0; uu < U; uu++)
#pragma unroll
    for (int r = 0; r < R; r++) load_unit<WT>(cur[uu][r], rs, (uint32_t)((row0 + r) * nsb), uu * G + c0, units, row0 + r < pt.N);

  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  // ---- activations -> Q8_K in LDS (rows m >= M are zero) ----
  if (XT == KQ_IMAGE) {  // codes | sums | scales, written by quantize_q8k_kernel in exactly this layout
    const int n16 = MT * (K >> 4), n4 = MT * nsb * 9;
    for (int c = tid; c < n16; c += nthreads) s_q[c] = reinterpret_cast<const u32x4*>(a.x)[c];
    const uint32_t* tail = reinterpret_cast<const uint32_t*>(a.x) + (size_t)n16 * 4;
    for (int c = tid; c < n4; c += nthreads) s_bs[c] = tail[c];
  }
  auto quantize_to_lds = [&](int it, const float (&v)[8]) {
    const Q8KItem q = quantize_q8k_item(v, lane);
    reinterpret_cast<u32x2*>(s_q)[it] = u32x2{q.q0, q.q1};
    const int s16 = q.sum8 + __builtin_amdgcn_update_dpp(0, q.sum8, 0xB1, 0xf, 0xf, true);
    const int s16b = __builtin_amdgcn_update_dpp(0, s16, 0x4E, 0xf, 0xf, true);  // the other pair of the quad
    if ((it & 3) == 0) s_bs[it >> 2] = ((uint32_t)s16 & 0xffffu) | ((uint32_t)s16b << 16);
    if ((it & 31) == 0) s_d[it >> 5] = q.d;
  };
  if (XT != KQ_IMAGE) {
#pragma unroll
    for (int k = 0; k < NPRE; k++) {  // whole half-waves: nitems is a multiple of 32
      const int it = tid + k * nthreads;
      if (it < nitems) {
        float v[8];
        if (XL == MLLM_HIP_F32) {
          const u32x4 p = raw[k][0], q = raw[k][XL == MLLM_HIP_F32 ? 1 : 0];
          v[0] = __uint_as_float(p.x); v[1] = __uint_as_float(p.y); v[2] = __uint_as_float(p.z); v[3] = __uint_as_float(p.w);
          v[4] = __uint_as_float(q.x); v[5] = __uint_as_float(q.y); v[6] = __uint_as_float(q.z); v[7] = __uint_as_float(q.w);
        } else {
          const uint32_t w[4] = {raw[k][0].x, raw[k][0].y, raw[k][0].z, raw[k][0].w};
#pragma unroll
          for (int j = 0; j < 4; j++) {
            v[2 * j + 0] = __uint_as_float(w[j] << 16);
            v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
          }
        }
        if (it >= valid) {
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = 0.f;
        }
        if (XT == MLLM_HIP_F32 && MT == 1 && x2p) silu_mul8(v, reinterpret_cast<const float*>(&raw2[k < 2 ? k : 0][0]), a.silu_accurate);
        quantize_to_lds(it, v);
      }
    }
    for (int it = tid + NPRE * nthreads; it < nitems; it += nthreads) {
      float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (it < valid) load8<XL>(xp, (int64_t)it * 8, v);
      if (XT == MLLM_HIP_F32 && MT == 1 && x2p) silu_mul8(v, x2p + (int64_t)min(it, valid - 1) * 8, a.silu_accurate);
      quantize_to_lds(it, v);
    }
  }
  __syncthreads();

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < MT; m++) acc[r][m] = 0.f;

  for (int u0 = 0; u0 < units; u0 += G * U) {
    KUnit<WT> nxt[U][R];
    const bool more = !ONE && u0 + G * U < units;  // uniform
    if (more) {
#pragma unroll
      for (int uu = 0; uu < U; uu++)
#pragma unroll
        for (int r = 0; r < R; r++)
          load_unit<WT>(nxt[uu][r], rs, (uint32_t)((row0 + r) * nsb), u0 + G * U + uu * G + c0, units, row0 + r < pt.N);
    }
#pragma unroll
    for (int uu = 0; uu < U; uu++) {
    const KUnit<WT>(&cu)[R] = cur[uu];
    const int unit = u0 + uu * G + c0;
    if (unit < units) {
      if (WT == MLLM_HIP_Q4_K) {
        const int sb = unit >> 3, c = unit & 7, jp = c >> 1, hh = c & 1;
        int sc_lo[R], sc_hi[R], mn_lo[R], mn_hi[R];
        float dw[R], dmw[R];
        u32x4 wlo[R], whi[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
          const uint32_t rec = cu[r].s.x;  // {sc[2jp], sc[2jp+1], m[2jp], m[2jp+1]}
          sc_lo[r] = (int)(rec & 0xffu);
          sc_hi[r] = (int)((rec >> 8) & 0xffu);
          mn_lo[r] = (int)((rec >> 16) & 0xffu);
          mn_hi[r] = (int)(rec >> 24);
          dw[r] = f16bits_to_f32((uint16_t)(cu[r].s.y & 0xffffu));
          dmw[r] = f16bits_to_f32((uint16_t)(cu[r].s.y >> 16));
          const uint32_t m4 = 0x0f0f0f0fu;
          wlo[r] = u32x4{cu[r].a.x & m4, cu[r].a.y & m4, cu[r].a.z & m4, cu[r].a.w & m4};
          whi[r] = u32x4{(cu[r].a.x >> 4) & m4, (cu[r].a.y >> 4) & m4, (cu[r].a.z >> 4) & m4, (cu[r].a.w >> 4) & m4};
        }
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const int qb = m * (K >> 4) + sb * 16 + 4 * jp + hh;  // 16-byte chunk of the sub-block pair's low half
          const u32x4 xlo = s_q[qb], xhi = s_q[qb + 2];
          const float yd = s_d[m * nsb + sb];
          const u32x2 bp = reinterpret_cast<const u32x2*>(s_bs)[(m * nsb + sb) * 4 + jp];  // sums 4jp..4jp+3
          const int bs_lo = half16(bp.x, hh), bs_hi = half16(bp.y, hh);
#pragma unroll
          for (int r = 0; r < R; r++) {
            const int isum = sc_lo[r] * dot16(wlo[r], xlo) + sc_hi[r] * dot16(whi[r], xhi);
            const int msum = mn_lo[r] * bs_lo + mn_hi[r] * bs_hi;
            acc[r][m] = fmaf(yd * dw[r], (float)isum, acc[r][m]);
            acc[r][m] = fmaf(-yd * dmw[r], (float)msum, acc[r][m]);
          }
        }
      } else {
        const int sb = unit >> 2, n = (unit >> 1) & 1, t = unit & 1;
        u32x4 wv[R][4];
        int sc[R][4];
        float dw[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
          dw[r] = f16bits_to_f32(cu[r].d);
          const uint32_t sw[4] = {cu[r].s.x, cu[r].s.y, cu[r].s.z, cu[r].s.w};
#pragma unroll
          for (int g = 0; g < 4; g++) {
            const u32x4& src = (g & 1) ? cu[r].b : cu[r].a;
            const int sh = (g >= 2) ? 4 : 0;
            const uint32_t m4 = 0x0f0f0f0fu, m2 = 0x03030303u;
            wv[r][g] = u32x4{((src.x >> sh) & m4) | (((cu[r].h.x >> (2 * g)) & m2) << 4), ((src.y >> sh) & m4) | (((cu[r].h.y >> (2 * g)) & m2) << 4),
                             ((src.z >> sh) & m4) | (((cu[r].h.z >> (2 * g)) & m2) << 4), ((src.w >> sh) & m4) | (((cu[r].h.w >> (2 * g)) & m2) << 4)};
            const int si = 8 * n + 2 * g + t;  // scale of these 16 weights
            sc[r][g] = (int)(int8_t)((sw[si >> 2] >> (8 * (si & 3))) & 0xffu);
          }
        }
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const float yd = s_d[m * nsb + sb];
          const u32x4 bq = reinterpret_cast<const u32x4*>(s_bs)[(m * nsb + sb) * 2 + n];  // sums 8n..8n+7
          const uint32_t bw[4] = {bq.x, bq.y, bq.z, bq.w};
          int tot[R];
#pragma unroll
          for (int r = 0; r < R; r++) tot[r] = 0;
#pragma unroll
          for (int g = 0; g < 4; g++) {
            const u32x4 xq = s_q[m * (K >> 4) + sb * 16 + 8 * n + 2 * g + t];
            const int bs = half16(bw[g], t);
#pragma unroll
            for (int r = 0; r < R; r++) tot[r] += sc[r][g] * (dot16(wv[r][g], xq) - 32 * bs);
          }
#pragma unroll
          for (int r = 0; r < R; r++) acc[r][m] = fmaf(yd * dw[r], (float)tot[r], acc[r][m]);
        }
      }
    }
    }
    if (more) {
#pragma unroll
      for (int uu = 0; uu < U; uu++)
#pragma unroll
        for (int r = 0; r < R; r++) cur[uu][r] = nxt[uu][r];
    }
  }

#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < MT; m++) {
      const float v = group_sum<G>(acc[r][m]);
      const int64_t row = row0 + r;
      if (c0 == 0 && row < pt.N && m < a.M) pt.y[(yrow + m) * pt.N + row] = pt.bias ? v + pt.bias[row] : v;
    }
}

static int g_kq_G = 0, g_kq_NW = 0, g_kq_U = 0;  // tuning overrides (0 = heuristic)

// R1: one weight row per lane group and up to 16 waves per workgroup (few rows of many units: o_proj, down_proj).  The
// quantization of x is the long part of such a workgroup, so it is shared by as many rows as still fill the CUs.
template <int WT, int XT, int MT, int G, int U, bool R1 = false, bool ONE = false>
static int launch_kq_u(const KGemvArgs& a_in, int NW, hipStream_t st) {
  constexpr int R = R1 ? 1 : (WT == MLLM_HIP_Q4_K && MT >= 4) ? 4 : 2;  // wider row tiles reuse every LDS read for more weight rows
  constexpr int LB = R1 ? 1024 : 256;
  if (NW < 1 || NW * 64 > LB) return MLLM_HIP_E_BADARG;  // the kernel is compiled for at most LB threads
  const int rows_per_wg = NW * (64 / G) * R;
  const int K = a_in.nsb * QK_K;
  const size_t lds = (size_t)MT * K + (size_t)MT * a_in.nsb * 4 + (size_t)MT * a_in.nsb * 32;
  if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
  KGemvArgs a = a_in;
  unsigned grid = 0;
  for (int p = 0; p < a.nparts; p++) {
    a.wg_start[p] = (int)grid;
    grid += (unsigned)((a.part[p].N + rows_per_wg - 1) / rows_per_wg);
  }
  a.wg_start[a.nparts] = (int)grid;
  if (ONE && a_in.nsb * (WT == MLLM_HIP_Q4_K ? 8 : 4) > G * U) return MLLM_HIP_E_BADARG;
  auto kern = kq_gemv_kernel<WT, XT, MT, G, R, U, LB, ONE>;
  if (lds > 64 * 1024)
    HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  const unsigned slots = (MT == 1 && a.slot_ids) ? (unsigned)a.slot_div_slots : 1u;
  hipLaunchKernelGGL(kern, dim3(grid, slots), dim3(NW * 64), lds, st, a);
  return (int)hipGetLastError();
}
template <int WT, int XT, int MT, int G>
static int launch_kq_g(const KGemvArgs& a, int NW, int U, bool r1, hipStream_t st) {
  // Q4_K, one or two rows, 32 lanes per weight row: a row of up to 96 (128 in the large workgroups) units is requested whole
  // before the quantization of x, three (four) units per lane, instead of one trip ahead of the dot loop -- time stamps put
  // a round trip to memory into every further trip (2560-element rows: 2.0 to 2.9 us of loop for three trips)
  if constexpr (WT == MLLM_HIP_Q4_K && MT <= 2 && G == 32) {
    const int units = a.nsb * 8;
    if (!g_kq_U) {  // (a tuning override of the units in flight keeps the trips)
      if (r1 && units <= 4 * G) return launch_kq_u<WT, XT, MT, G, 4, true, true>(a, NW, st);
      // (one row only: with two, no gain.  117 registers = four waves per SIMD, so the 1216 workgroups of gate + up come in
      // two rounds; asking the compiler for five waves, 96 registers, measured slower: gate + up 8.7 -> 9.1 us, q+k+v 5.35 -> 5.65)
      if constexpr (MT == 1)
        if (!r1 && units > 2 * G && units <= 3 * G) return launch_kq_u<WT, XT, MT, G, 3, false, true>(a, NW, st);
    }
  }
  if (r1 && MT <= 2 && G >= 32) return launch_kq_u<WT, XT, MT, G, (MT <= 2 && G >= 32 && WT == MLLM_HIP_Q4_K) ? 4 : 1, (MT <= 2 && G >= 32)>(a, NW, st);
  if (WT == MLLM_HIP_Q4_K && U >= 4 && MT <= 2) return launch_kq_u<WT, XT, MT, G, (WT == MLLM_HIP_Q4_K && MT <= 2) ? 4 : 1>(a, NW, st);
  if (U >= 2 && MT <= 2) return launch_kq_u<WT, XT, MT, G, MT <= 2 ? 2 : 1>(a, NW, st);
  return launch_kq_u<WT, XT, MT, G, 1>(a, NW, st);
}
template <int WT, int XT, int MT>
static int launch_kq_m(const KGemvArgs& a, hipStream_t st) {
  // Measured on MI355X over the Qwen3-4B projection shapes (lanes per row x waves x units in flight swept): Q4_K rows want 32
  // lanes, Q6_K rows (units twice as heavy) the whole wave; four waves per workgroup share the activation quantization;
  // a grid of about one workgroup per CU keeps four units per lane in flight, a larger grid gets its bytes in flight
  // from occupancy and keeps one.
  const int units = a.nsb * (WT == MLLM_HIP_Q4_K ? 8 : 4);
  int best = WT == MLLM_HIP_Q4_K ? 32 : 64;
  while (best > 8 && best / 2 >= units) best >>= 1;
  int NW = 4;
  int64_t rows = 0;
  for (int p = 0; p < a.nparts; p++) rows += a.part[p].N;
  // (MoE slots multiply the grid: the shape rules below look at the whole launch)
  const int grid = (int)((rows + NW * (64 / best) * 2 - 1) / (NW * (64 / best) * 2)) * ((MT == 1 && a.slot_ids) ? a.slot_div_slots : 1);
  int U = 1;  // (four units in flight only in the large workgroups below: the 384-workgroup q/k/v launch measured 5.8 us with
              // one unit against 6.4 us with four)
  // few rows of many units (o_proj, down_proj): large workgroups of one row per lane group, the whole wave on a row when it is
  // long enough to keep 64 lanes busy for a trip
  // (only with at least 32 lanes per row: the narrower shapes have no such variant and keep their 256-thread workgroups)
  const bool r1 = MT <= 2 && grid < (WT == MLLM_HIP_Q4_K ? 256 : 512) && best >= 32 && !g_kq_NW && !g_kq_G;
  if (r1) {
    if (units >= 64 * 4) best = 64;
    NW = best == 64 ? 16 : 8;  // 16 rows per workgroup either way
    // ... or fewer, so that the grid is about one workgroup per CU (the Q4_0 kernel's finding: 2560 rows of 9728 elements
    // as 160 workgroups of 16 waves or as 256 of 10)
    const int rpw = 64 / best;  // rows per wave
    const int want = (int)((rows / rpw + 255) / 256);
    if (want >= 4 && want < NW) NW = want;
  }  // (many rows, K = 2560: eight waves per workgroup measured slower than four, 11.0 against 9.6 us for gate + up)
  // Q6_K rows whose units leave most of a 64-lane trip idle (K = 2560: 40 units): 16 lanes per row, two waves, where that still
  // makes a thousand workgroups (gate + up 15.8 -> 13.5 us; the smaller q/k/v launch stays faster with the whole wave)
  if (WT == MLLM_HIP_Q6_K && MT <= 2 && !r1 && !g_kq_G && !g_kq_NW && best == 64 && rows / 16 >= 1024 &&
      2 * ((units + 15) / 16 * 16 - units) < (units + 63) / 64 * 64 - units) {
    best = 16;
    NW = 2;
  }
  // MoE slots (thousands of small workgroups, each quantizing its token's x): 16 lanes per row make the workgroups twice as
  // tall, two units in flight (Qwen3-30B-A3B experts, eight tokens: 54.6 -> 45.1 us for the layer)
  if (MT == 1 && a.slot_ids && a.slot_div_slots > 1 && best >= 16 && !r1) {
    best = 16;
    U = 2;
  }
  if (g_kq_G) best = g_kq_G;
  if (g_kq_NW) NW = g_kq_NW;
  if (g_kq_U) U = g_kq_U;
  if (best == 64) return launch_kq_g<WT, XT, MT, 64>(a, NW, U, r1, st);
  if (best == 32) return launch_kq_g<WT, XT, MT, 32>(a, NW, U, r1, st);
  if (best == 16) return launch_kq_g<WT, XT, MT, 16>(a, NW, U, r1, st);
  return launch_kq_g<WT, XT, MT, 8>(a, NW, U, r1, st);
}
template <int WT, int XT>
static int launch_kq(const KGemvArgs& a, hipStream_t st) {
  if (a.M <= 1) return launch_kq_m<WT, XT, 1>(a, st);
  if (a.M <= 2) return launch_kq_m<WT, XT, 2>(a, st);
  if (a.M <= 4) return launch_kq_m<WT, XT, 4>(a, st);
  return launch_kq_m<WT, XT, 8>(a, st);
}


// ---- Q4_K, three to eight rows: sub-block sums on the matrix cores ---------------------------------------------------------
// The dot4 kernel above needs the activation codes of every row from LDS for every weight unit and is bound by those reads
// from three rows on (17 us per 9728 x 2560 projection at eight rows against 7 at one).  Here v_mfma_i32_16x16x64_i8 makes
// the sums of one 32-element sub-block, as in the Q4_0 kernel of this kind (qgemv_mfma.hip): the instruction sums over
// K = 64, and the sums of different sub-blocks are kept apart by the activation operand.  A 16-byte record of the nibble
// plane holds 16 elements of sub-block 2c (low nibbles) and the same 16 of sub-block 2c+1 (high nibbles); lane group g of
// the weight operand holds record 4j + g of the lane's weight row, so the low-nibble instruction sees sub-block 4j in
// groups 0,1 and sub-block 4j+2 in groups 2,3 (the high-nibble instruction 4j+1 and 4j+3).  Output column 8 q + t gets the
// codes of (that sub-block, activation row t) in groups 2q, 2q+1 and zeros in the other two: one instruction = the sums of
// two sub-blocks for eight rows, every lane of the result useful.
// Scaling per lane (four consecutive weight rows of one activation row):
//   acc = fma(fp32(d*sc) * dx, float(isum), acc);  acc = fma(-(fp32(dmin*m) * dx), float(sum of the row's 32 codes), acc)
// the reference's sum (vec_dot_q4_K_q8_K: integer sums per super-block, then d*dx and dmin*dx) regrouped; the integer parts
// are exact, the fp32 roundings differ in order only.
// Order and batching of the requests in front of the loop (measured on the 4B layer shapes; the values compiled in are the
// fastest): KMF_WEIGHTS_FIRST 1 asks for the slice's weights before the quantized image is copied -- the image, which every
// wave needs before the first barrier, then comes back behind them (layer at eight rows 58.3 us against 54.2);
// KMF_COPY_UNROLL = image pieces a thread requests before it stores the first (10: the down projection gets slower);
// KMF_QUANT_BATCH = activation items a thread requests before it quantizes the first.
#ifndef KMF_WEIGHTS_FIRST
#define KMF_WEIGHTS_FIRST 0
#endif
#ifndef KMF_QUANT_BATCH
#define KMF_QUANT_BATCH 4
#endif
#ifndef KMF_COPY_UNROLL
#define KMF_COPY_UNROLL 5
#endif
typedef int kv4i __attribute__((ext_vector_type(4)));
constexpr int KMF_NG = 10;  // groups of four sub-blocks per trip, at most (the launcher takes 6 or 8 for shorter slices)

static int kmf_slices(int nb32) {
  int s = 1;
  while (s < 8 && nb32 > 40 * s) s *= 2;
  return s;
}

// blockDim = nwaves * 64; a workgroup holds nwaves / S row tiles (16 weight rows), S K-slices each; nbs = sub-blocks per slice
// (a multiple of 8: whole super-blocks).
// LDS: xc [nb32 + xpad][MT] 32 bytes: the 32 codes of (sub-block, row); xs [nb32 + xpad][MT] {dx, sum of the 32 codes}
//      (xpad = how far the last trip of the last slice reaches past the row: zeros); one zero record;
//      ws per wave [whole trips][16 rows] fp32 d*sc, then the same of dmin*m (after the loop: the wave's four sums for the
//      wave of slice 0).
// NG = groups of four sub-blocks per trip: the slice in one trip where it fits (6, 8 or 10), so that neither registers nor
// LDS rows are held for sub-blocks the slice does not have -- with K = 2048 three workgroups fit a CU instead of two.
// K slices spread over workgroups (blockIdx.z = slice group): where they meet.  SG = 1: all slices of a tile in one workgroup.
struct KMeet {
  int SG;              // slice groups (= gridDim.z); a workgroup holds slices [z S, z S + S)
  int lrows;           // sub-blocks a workgroup keeps in LDS: its slices' plus what their last trips reach past them
  float* part;         // [x column of the grid][wave][slice group][32 lanes] four partial sums
  unsigned* counters;  // one per x column (cstride counters apart), zero between launches
  int cstride;
};
// host side: what a caller's workspace offers for it (key = the workspace address that owns the counter block)
struct KMeetRoom {
  const void* key;
  void* part;
  size_t part_bytes;
};
int gemv_counter_block(const void* workspace, hipStream_t st, unsigned** out);  // qgemv_mfma.hip
constexpr int KQ_NOT_TAKEN = 1;  // a launcher's answer when the launch does not suit it (also gemv_counter_block's when no block is free)
template <int XT, int MT, int NG = KMF_NG>
__global__ __launch_bounds__(512) void kq4_gemv_mfma_kernel(KGemvArgs a, int S, int nbs, KMeet km) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int TRIP = 4 * NG;
  const int nsb = a.nsb, nb32 = nsb * 8, K = nsb * QK_K;
  const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int pidx = 0;
#pragma unroll
  for (int p = 1; p < KQ_MAX_PARTS; p++)
    if (p < a.nparts && (int)blockIdx.x >= a.wg_start[p]) pidx = p;
  const KGemvPart& pt = a.part[pidx];
  const KTile mt = kq_tile(a);
  if (!mt.active) return;  // uniform, ahead of every barrier
  const int N = pt.N;
  const int tiles_wg = nwaves / S;
  const int tile = ((int)blockIdx.x - a.wg_start[pidx]) * tiles_wg + wave / S;
  const int sg = km.SG > 1 ? (int)blockIdx.z : 0;
  const int slice = sg * S + wave % S;
  const int row0 = tile * 16;
  const bool tile_ok = row0 < N;
  const int b0 = slice * nbs, b1 = min(nb32, b0 + nbs);
  const int kb0 = min(nb32, sg * S * nbs), kb1 = min(nb32, kb0 + S * nbs);  // the workgroup's sub-blocks; LDS rows count from kb0
  const int nloc = kb1 - kb0, lrows = km.lrows;

  const int wsb = (nbs + TRIP - 1) / TRIP * TRIP;
  u32x4* xc = reinterpret_cast<u32x4*>(smem);                        // [((sb - kb0) * MT + m) * 2 + half]
  u32x4* zrec = xc + (size_t)lrows * MT * 2;
  u32x2* xs = reinterpret_cast<u32x2*>(zrec + 1);                    // [(sb - kb0) * MT + m]
  float* ws_all = reinterpret_cast<float*>(xs + (size_t)lrows * MT);
  float* ws_ds = ws_all + (size_t)wave * 2 * wsb * 16;
  float* ws_dm = ws_ds + (size_t)wsb * 16;
  f32x4* red = reinterpret_cast<f32x4*>(ws_ds);  // the wave's scale table, dead after the loop (2 wsb x 64 bytes >= 1 KB)
  int* s_flag = reinterpret_cast<int*>(ws_all + (size_t)nwaves * 2 * wsb * 16);

  // ---- 1. weight scale records of the tile and slice: one 16-byte record per (row, super-block) --------------------------
  const uint32_t sbt = (uint32_t)N * (uint32_t)nsb;
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(kq_at(pt.w.a, mt.eoff)), 0, sbt * 128u, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsc = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(kq_at(pt.w.s, mt.eoff)), 0, sbt * 16u, 0x00020000);
  const int spb = nbs >> 3;  // super-blocks per slice (at most 8)
  const __amdgpu_buffer_rsrc_t rdd = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(kq_at(pt.w.d, mt.eoff)), 0, sbt * 4u, 0x00020000);
  u32x4 sc[2];
  uint32_t scd[2];
#pragma unroll
  for (int k = 0; k < 2; k++) {
    const int ch = lane + 64 * k;
    const int r = ch / spb, si = ch - r * spb;
    const int sb256 = (b0 >> 3) + si;
    const bool ok = tile_ok && r < 16 && row0 + r < N && sb256 < nsb;
    const uint32_t rec = (uint32_t)(row0 + r) * (uint32_t)nsb + (uint32_t)sb256;
    sc[k] = __builtin_amdgcn_raw_buffer_load_b128(rsc, ok ? rec * 16u : KBUF_OOB, 0, KBUF_NT);
    scd[k] = __builtin_amdgcn_raw_buffer_load_b32(rdd, ok ? rec * 4u : KBUF_OOB, 0, KBUF_NT);
  }
  // ---- 2. weight codes: lane (row c, group g) takes records b0 + 4 j + g ------------------------------------------------------
  const int c = lane & 15, g = lane >> 4;
  const bool row_ok = tile_ok && row0 + c < N;
  const uint32_t rbase = (uint32_t)(row0 + c) * (uint32_t)nb32;
  u32x4 wq[NG];
  auto load_groups = [&](int bb) {
#pragma unroll
    for (int j = 0; j < NG; j++) {
      const int b = bb + 4 * j + g;
      wq[j] = __builtin_amdgcn_raw_buffer_load_b128(ra, (row_ok && b < b1) ? (rbase + (uint32_t)b) * 16u : KBUF_OOB, 0, KBUF_NT);
    }
  };
  if (KMF_WEIGHTS_FIRST && XT == KQ_IMAGE) load_groups(b0);
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // ---- 3. activations into LDS -------------------------------------------------------------------------------------------------
  if (XT == KQ_IMAGE) {  // codes [R][K], sums of 16 as int16 [R][K/16], scales [R][nsb]; R = MT, or the rows of a MoE image
    const size_t R = a.img_rows ? (size_t)a.img_rows : (size_t)MT;
    const u32x4* codes = reinterpret_cast<const u32x4*>(a.x);
    const uint32_t* pairs = reinterpret_cast<const uint32_t*>(reinterpret_cast<const char*>(a.x) + R * K);
    const float* dd = reinterpret_cast<const float*>(reinterpret_cast<const char*>(a.x) + R * K + R * nsb * 32);
    // Thread (row m = tid % MT, piece tid / MT): a wave reads 128 contiguous bytes of each of its rows and writes 1 KB of
    // contiguous LDS.  The pieces of a batch are all requested before the first is stored, and the sums and scales before
    // the codes: one round trip to memory per batch, where a copy row by row and pass by pass took one per pass.
    const int m = tid & (MT - 1), p0 = tid / MT, pstep = nthreads / MT;
    const size_t src = (size_t)kq_tile_in_row(a, mt, m);
    constexpr int CS = 3;
    uint32_t pr[CS];
    float dv[CS];
#pragma unroll
    for (int u = 0; u < CS; u++) {
      const int sb = p0 + u * pstep;
      if (sb < nloc) {
        pr[u] = pairs[src * nb32 + kb0 + sb];
        dv[u] = dd[src * nsb + ((kb0 + sb) >> 3)];
      }
    }
    for (int r0 = p0; r0 < 2 * nloc; r0 += pstep * KMF_COPY_UNROLL) {
      u32x4 cv[KMF_COPY_UNROLL];
#pragma unroll
      for (int u = 0; u < KMF_COPY_UNROLL; u++) {
        const int r = r0 + u * pstep;
        if (r < 2 * nloc) cv[u] = codes[(src * nb32 + kb0) * 2 + r];
      }
#pragma unroll
      for (int u = 0; u < KMF_COPY_UNROLL; u++) {
        const int r = r0 + u * pstep;
        if (r < 2 * nloc) xc[((size_t)(r >> 1) * MT + m) * 2 + (r & 1)] = cv[u];
      }
    }
    auto put_sums = [&](int sb, uint32_t pair, float d) {
      const int bsum = (int)(int16_t)(pair & 0xffffu) + (int)(int16_t)(pair >> 16);
      xs[(size_t)sb * MT + m] = u32x2{__float_as_uint(d), (uint32_t)bsum};
    };
#pragma unroll
    for (int u = 0; u < CS; u++)
      if (p0 + u * pstep < nloc) put_sums(p0 + u * pstep, pr[u], dv[u]);
    for (int sb = p0 + CS * pstep; sb < nloc; sb += pstep) put_sums(sb, pairs[src * nb32 + kb0 + sb], dd[src * nsb + ((kb0 + sb) >> 3)]);
  } else {
    const int ipr = K >> 3;     // items (eight elements) per row; 32 consecutive items = one super-block
    const int iwg = nloc << 2;  // of them in this workgroup's sub-blocks (whole super-blocks)
    const int nitems = MT * iwg;
    const float inv_iwg = 1.0f / (float)iwg;
    // (the items of a batch are all requested before the first is quantized: one round trip to memory per batch)
    constexpr int QI = KMF_QUANT_BATCH;
    for (int it0 = tid; it0 < nitems; it0 += nthreads * QI) {  // whole half-waves: nitems and nthreads are multiples of 32
      float v[QI][8];
#pragma unroll
      for (int u = 0; u < QI; u++) {
        const int it = it0 + u * nthreads;
        const int m = (int)(((float)it + 0.5f) * inv_iwg), i = it - m * iwg;  // it / iwg: far from rounding trouble
#pragma unroll
        for (int e = 0; e < 8; e++) v[u][e] = 0.f;
        if (it < nitems && m < a.M) load8<XT == KQ_IMAGE ? MLLM_HIP_F32 : XT>(a.x, ((int64_t)m * ipr + 4 * kb0 + i) * 8, v[u]);
      }
      if (it0 == tid) load_groups(b0);  // the weights right behind the first batch: they arrive while it is quantized
#pragma unroll
      for (int u = 0; u < QI; u++) {
        const int it = it0 + u * nthreads;
        if (it >= nitems) break;
        const int m = (int)(((float)it + 0.5f) * inv_iwg), i = it - m * iwg;
        const Q8KItem qi = quantize_q8k_item(v[u], lane);
        int s32 = qi.sum8 + __builtin_amdgcn_update_dpp(0, qi.sum8, 0xB1, 0xf, 0xf, true);
        s32 += __builtin_amdgcn_update_dpp(0, s32, 0x4E, 0xf, 0xf, true);
        const int sb = i >> 2, part = i & 3;  // sub-block (from kb0), which 8 of its 32 codes
        reinterpret_cast<u32x2*>(xc + ((size_t)sb * MT + m) * 2 + (part >> 1))[part & 1] = u32x2{qi.q0, qi.q1};
        if (part == 0) xs[(size_t)sb * MT + m] = u32x2{__float_as_uint(qi.d), (uint32_t)s32};
      }
    }
  }
  if (!KMF_WEIGHTS_FIRST && XT == KQ_IMAGE) load_groups(b0);
  if (XT != KQ_IMAGE && tid >= (nloc << 2) * MT) load_groups(b0);  // (threads without an item to quantize)
  if (tid == 0) zrec[0] = u32x4{0u, 0u, 0u, 0u};
  for (int i = tid; i < (lrows - nloc) * MT * 2; i += nthreads) xc[(size_t)nloc * MT * 2 + i] = u32x4{0u, 0u, 0u, 0u};
  for (int i = tid; i < (lrows - nloc) * MT; i += nthreads) xs[(size_t)nloc * MT + i] = u32x2{0u, 0u};
  // weight scales: fp32 d*sc and dmin*m per (sub-block of the slice, row); zero past the row and in the rest of the last trip
#pragma unroll
  for (int k = 0; k < 2; k++) {
    const int ch = lane + 64 * k;
    const int r = ch / spb, si = ch - r * spb;
    if (r < 16) {
      const bool in = (b0 >> 3) + si < nsb;
      const float d = f16bits_to_f32((uint16_t)(scd[k] & 0xffffu)), dmin = f16bits_to_f32((uint16_t)(scd[k] >> 16));
      const uint32_t rec[4] = {sc[k].x, sc[k].y, sc[k].z, sc[k].w};  // per pair of sub-blocks {sc, sc, m, m}
#pragma unroll
      for (int j = 0; j < 8; j++) {
        ws_ds[(8 * si + j) * 16 + r] = in ? d * (float)((rec[j >> 1] >> (8 * (j & 1))) & 0xffu) : 0.f;
        ws_dm[(8 * si + j) * 16 + r] = in ? dmin * (float)((rec[j >> 1] >> (16 + 8 * (j & 1))) & 0xffu) : 0.f;
      }
    }
  }
  for (int i = nbs * 16 + lane; i < wsb * 16; i += 64) {
    ws_ds[i] = 0.f;
    ws_dm[i] = 0.f;
  }
  __syncthreads();

  // ---- 4. sub-block sums on the matrix cores, scaling on the vector ALU (software-pipelined over groups of four) --------------
  const int q2 = (lane & 15) >> 3, t = lane & 7, tm = t & (MT - 1);
  const bool mine = (g >> 1) == q2;  // the lane groups that supply this column's codes
  const int half = g & 1;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int bb = b0; bb < b1; bb += TRIP) {
    if (bb != b0) load_groups(bb);
    const u32x4* bl = mine ? xc + ((size_t)(bb - kb0 + 2 * q2) * MT + tm) * 2 + half : zrec;
    const int bstep = mine ? 8 * MT : 0;  // four sub-blocks further per group
    const u32x2* xsl = xs + (size_t)(bb - kb0 + 2 * q2) * MT + tm;
    const float* dsl = ws_ds + (bb - b0 + 2 * q2) * 16 + 4 * g;
    const float* dml = ws_dm + (bb - b0 + 2 * q2) * 16 + 4 * g;
    u32x4 Bl[2], Bh[2];
    u32x2 sx[2][2];
    f32x4 ds[2][2], dm[2][2];
    kv4i D[2][2];
    auto fetch_b = [&](int set, int j) {
      Bl[set] = bl[j * bstep];
      Bh[set] = bl[j * bstep + (mine ? 2 * MT : 0)];
    };
    auto fetch_s = [&](int set, int j) {
#pragma unroll
      for (int h = 0; h < 2; h++) {
        sx[set][h] = xsl[(4 * j + h) * MT];
        ds[set][h] = *reinterpret_cast<const f32x4*>(dsl + (4 * j + h) * 16);
        dm[set][h] = *reinterpret_cast<const f32x4*>(dml + (4 * j + h) * 16);
      }
    };
    auto issue = [&](int set, int j) {
      const u32x4 w = wq[j];
      const kv4i Al = {(int)(w.x & 0x0f0f0f0fu), (int)(w.y & 0x0f0f0f0fu), (int)(w.z & 0x0f0f0f0fu), (int)(w.w & 0x0f0f0f0fu)};
      const kv4i Ah = {(int)((w.x >> 4) & 0x0f0f0f0fu), (int)((w.y >> 4) & 0x0f0f0f0fu), (int)((w.z >> 4) & 0x0f0f0f0fu),
                       (int)((w.w >> 4) & 0x0f0f0f0fu)};
      D[set][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Al, __builtin_bit_cast(kv4i, Bl[set]), kv4i{0, 0, 0, 0}, 0, 0, 0);
      D[set][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Ah, __builtin_bit_cast(kv4i, Bh[set]), kv4i{0, 0, 0, 0}, 0, 0, 0);
    };
    auto scale = [&](int set, int j) {
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const bool live = bb + 4 * j + 2 * q2 + h < b1;
        const float dx = live ? __uint_as_float(sx[set][h].x) : 0.f;
        const float bs = (float)(int)sx[set][h].y;
        acc.x = fmaf(ds[set][h].x * dx, (float)D[set][h].x, acc.x);
        acc.y = fmaf(ds[set][h].y * dx, (float)D[set][h].y, acc.y);
        acc.z = fmaf(ds[set][h].z * dx, (float)D[set][h].z, acc.z);
        acc.w = fmaf(ds[set][h].w * dx, (float)D[set][h].w, acc.w);
        acc.x = fmaf(-(dm[set][h].x * dx), bs, acc.x);
        acc.y = fmaf(-(dm[set][h].y * dx), bs, acc.y);
        acc.z = fmaf(-(dm[set][h].z * dx), bs, acc.z);
        acc.w = fmaf(-(dm[set][h].w * dx), bs, acc.w);
      }
    };
    fetch_b(0, 0);
#pragma unroll
    for (int j = 0; j < NG; j++) {
      issue(j & 1, j);
      if (j + 1 < NG) fetch_b((j + 1) & 1, j + 1);
      fetch_s(j & 1, j);
      __builtin_amdgcn_sched_barrier(0);
      if (j > 0) scale((j - 1) & 1, j - 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    scale((NG - 1) & 1, NG - 1);
  }
  {  // the two lanes of an activation row (sub-blocks = 0,1 and 2,3 mod 4)
    acc.x += __shfl_xor(acc.x, 8, 64);
    acc.y += __shfl_xor(acc.y, 8, 64);
    acc.z += __shfl_xor(acc.z, 8, 64);
    acc.w += __shfl_xor(acc.w, 8, 64);
  }

  // ---- 5. slices of a tile in slice order, bias ------------------------------------------------------------------------------
  if (S > 1) {
    red[lane] = acc;
    __syncthreads();
    if (wave % S != 0) return;
    for (int s = 1; s < S; s++) {
      const f32x4 o = reinterpret_cast<const f32x4*>(ws_ds + (size_t)s * 2 * wsb * 16)[lane];  // the table of wave + s
      acc.x += o.x; acc.y += o.y; acc.z += o.z; acc.w += o.w;
    }
  }
  if (km.SG > 1) {
    // The slice groups of a grid column meet in global memory (S = 1 here: every wave is a tile).  Ordering, step by step:
    // partial sums leave with device-scope stores; every wave waits until the memory system has acknowledged its stores
    // (s_waitcnt vmcnt(0): stores count in vmcnt until acknowledged); the workgroup barrier; thread 0 counts the workgroup
    // in with a device-scope atomic add; the workgroup that sees the last count reads all partial sums with device-scope
    // loads issued after a second barrier, and adds them in slice order: the bits of the one-workgroup form.
    const int SG = km.SG;
    const int li = 8 * g + t;
    float* pbase = km.part + (((size_t)blockIdx.x * nwaves + wave) * SG) * 128;
    if (q2 == 0) {
      float* dst = pbase + (size_t)sg * 128 + 4 * li;
      __hip_atomic_store(dst + 0, acc.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + 1, acc.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + 2, acc.z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + 3, acc.w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      unsigned* cnt = km.counters + (size_t)blockIdx.x * km.cstride;
      const unsigned old = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int last = old == (unsigned)(SG - 1);
      if (last) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
      *s_flag = last;
    }
    __syncthreads();
    if (!*s_flag) return;
    if (q2 == 0) {  // (at most eight slice groups; their loads are in flight together)
      float pv[8][4];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const float* src = pbase + (size_t)min(u, SG - 1) * 128 + 4 * li;
#pragma unroll
        for (int e = 0; e < 4; e++) pv[u][e] = __hip_atomic_load(src + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      acc = f32x4{pv[0][0], pv[0][1], pv[0][2], pv[0][3]};
#pragma unroll
      for (int u = 1; u < 8; u++)
        if (u < SG) { acc.x += pv[u][0]; acc.y += pv[u][1]; acc.z += pv[u][2]; acc.w += pv[u][3]; }
    }
  }
  if (!tile_ok || q2 != 0 || t >= MT || t >= mt.rows) return;
  const int n = row0 + 4 * g;
  const float v[4] = {acc.x, acc.y, acc.z, acc.w};
  float* yrow = pt.y + (int64_t)kq_tile_out_row(a, mt, t) * N;
#pragma unroll
  for (int e = 0; e < 4; e++)
    if (n + e < N) yrow[n + e] = pt.bias ? v[e] + pt.bias[n + e] : v[e];
}

static int kmf_groups(int nbs) { return nbs <= 24 ? 6 : (nbs <= 32 ? 8 : KMF_NG); }
// how far the last trip of a slice reads past the row's nb32 sub-blocks (whole trips from the slice's first sub-block)
static int kmf_xpad(int nb32, int S, int nbs) {
  const int trip = 4 * kmf_groups(nbs);
  int pad = 0;
  for (int s = 0; s < S; s++) {
    const int b0 = s * nbs, b1 = std::min(nb32, b0 + nbs);
    if (b1 > b0) pad = std::max(pad, b0 + ((b1 - b0 - 1) / trip + 1) * trip - nb32);
  }
  return pad;
}
template <int MT>
static size_t kmf_lds_bytes(int nb32, int nbs, int nwaves, int S) {
  const int trip = 4 * kmf_groups(nbs);
  const int wsb = (nbs + trip - 1) / trip * trip, rows = nb32 + kmf_xpad(nb32, S, nbs);
  return (size_t)rows * MT * 32 + 16 + (size_t)rows * MT * 8 + (size_t)nwaves * 2 * wsb * 64 + 16;
}
// the same with one slice per workgroup (slice groups over the grid's z): the slice's sub-blocks in whole trips
template <int MT>
static size_t kmf_lds_bytes_z(int nbs, int nwaves) {
  const int trip = 4 * kmf_groups(nbs);
  const int wsb = (nbs + trip - 1) / trip * trip;
  return (size_t)wsb * MT * 32 + 16 + (size_t)wsb * MT * 8 + (size_t)nwaves * 2 * wsb * 64 + 16;
}
static bool kq4_mfma_fits(int MT, int nsb) {
  const int nb32 = nsb * 8;
  if (nb32 > 512) return false;  // scale records: at most 128 per wave
  const int S = kmf_slices(nb32);
  const int nbs = ((nb32 + S - 1) / S + 7) / 8 * 8;
  return (MT == 4 ? kmf_lds_bytes<4>(nb32, nbs, 8, S) : kmf_lds_bytes<8>(nb32, nbs, 8, S)) <= 160 * 1024;
}
// room for the partial sums of a launch whose slices meet in global memory (0: its slices share a workgroup anyway)
static size_t kmf_part_bytes(int nsb, int64_t n_total, int nparts) {
  const int S = std::max(kmf_slices(nsb * 8), nsb > 5 ? (nsb > 10 ? (nsb > 20 ? 8 : 4) : 2) : 1);  // (Q4_K's slices, Q6_K's: k6mf_split)
  if (S < 2) return 0;
  return (size_t)((n_total + 15) / 16 + (int64_t)nparts * 8) * S * 512;
}
int g_kq_meet = -1, g_kq_meet_waves = 0, g_kq_meet_min = 4;  // (mllm_hip_kq_set_slice_meeting)
// row tiles (= waves) per workgroup of a launch whose K slices meet in memory: four to six, the first that needs the fewest
// rounds of 256 workgroups (measured with Q4_K on 2560 x 9728 with eight slices: 12.6 / 11.4 / 12.4 us with four / five /
// six at four rows, five = exactly 256 workgroups; 2560 x 4096 with four slices: 8.8 / 8.9 / 9.8, and 9.2 with three)
static int kq_meet_waves(const KGemvArgs& a, int SG) {
  int nwaves = g_kq_meet_waves;
  if (!nwaves) {
    int64_t best = 0;
    for (int nw = 4; nw <= 6; nw++) {
      int64_t wgs = 0;
      for (int p = 0; p < a.nparts; p++) wgs += ((a.part[p].N + 15) / 16 + nw - 1) / nw;
      const int64_t rounds = (wgs * SG + 255) / 256;
      if (!best || rounds < best) {
        best = rounds;
        nwaves = nw;
      }
    }
  }
  return nwaves;
}
template <int XT, int MT>
static int launch_kq4_mfma_z(const KGemvArgs& a_in, const KMeetRoom& room, hipStream_t st) {
  KGemvArgs a = a_in;
  const int nb32 = a.nsb * 8;
  const int SG = kmf_slices(nb32);
  const int nbs = ((nb32 + SG - 1) / SG + 7) / 8 * 8;
  const int nwaves = kq_meet_waves(a, SG);
  unsigned grid = 0;
  for (int p = 0; p < a.nparts; p++) {
    a.wg_start[p] = (int)grid;
    grid += (unsigned)(((a.part[p].N + 15) / 16 + nwaves - 1) / nwaves);
  }
  a.wg_start[a.nparts] = (int)grid;
  if (SG < 2 || g_kq_meet == 0 || !room.part || (size_t)grid * nwaves * SG * 512 > room.part_bytes || grid > 1024u) return KQ_NOT_TAKEN;
  KMeet km{};
  km.SG = SG;
  const int trip = 4 * kmf_groups(nbs);
  km.lrows = (nbs + trip - 1) / trip * trip;
  km.part = static_cast<float*>(room.part);
  RC_RET(gemv_counter_block(room.key, st, &km.counters));
  km.cstride = 1;
  while (km.cstride < 32 && (size_t)grid * km.cstride * 2 <= 1024u) km.cstride *= 2;
  const size_t lds = kmf_lds_bytes_z<MT>(nbs, nwaves);
  auto go = [&](auto kern) {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3(grid, 1, (unsigned)SG), dim3(nwaves * 64), lds, st, a, 1, nbs, km);
    return (int)hipGetLastError();
  };
  switch (kmf_groups(nbs)) {
    case 6: return go(kq4_gemv_mfma_kernel<XT, MT, 6>);
    case 8: return go(kq4_gemv_mfma_kernel<XT, MT, 8>);
    default: return go(kq4_gemv_mfma_kernel<XT, MT, KMF_NG>);
  }
}
template <int XT, int MT>
static int launch_kq4_mfma_t(const KGemvArgs& a_in, hipStream_t st, unsigned grid_y = 1) {
  KGemvArgs a = a_in;
  const int nb32 = a.nsb * 8;
  const int S = kmf_slices(nb32);
  const int nbs = ((nb32 + S - 1) / S + 7) / 8 * 8;
  // (MoE row tiles, grid_y > 1: the tile's eight image rows are staged once per workgroup; eight waves = 64 weight rows per
  // staging instead of 32: Q4_K 512 tokens 491 -> 458 us.  The Q6_K kernel, with two waves per SIMD, loses with eight: 780 -> 915)
  int nwaves = XT == KQ_IMAGE ? (grid_y > 1 ? (g_kq_NW ? g_kq_NW : 8) : 4) : 8;
  if (nwaves < S) nwaves = S;
  const int tiles_wg = nwaves / S;
  unsigned grid = 0;
  for (int p = 0; p < a.nparts; p++) {
    a.wg_start[p] = (int)grid;
    grid += (unsigned)(((a.part[p].N + 15) / 16 + tiles_wg - 1) / tiles_wg);
  }
  a.wg_start[a.nparts] = (int)grid;
  const size_t lds = kmf_lds_bytes<MT>(nb32, nbs, nwaves, S);
  if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
  KMeet km{};
  km.SG = 1;
  km.lrows = nb32 + kmf_xpad(nb32, S, nbs);
  auto go = [&](auto kern) {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3(grid, grid_y), dim3(nwaves * 64), lds, st, a, S, nbs, km);
    return (int)hipGetLastError();
  };
  switch (kmf_groups(nbs)) {
    case 6: return go(kq4_gemv_mfma_kernel<XT, MT, 6>);
    case 8: return go(kq4_gemv_mfma_kernel<XT, MT, 8>);
    default: return go(kq4_gemv_mfma_kernel<XT, MT, KMF_NG>);
  }
}
template <int XT>
static int launch_kq4_mfma(const KGemvArgs& a, hipStream_t st) {
  return a.M <= 4 ? launch_kq4_mfma_t<XT, 4>(a, st) : launch_kq4_mfma_t<XT, 8>(a, st);
}
// ---- Q6_K, three to eight rows: the same on 16-element units -------------------------------------------------------------------
// Q6_K scales 16 elements at a time, which is exactly what one lane supplies to the K = 64 instruction: lane group g of the
// weight operand holds one 16-element unit, and output column 4 q + t gets the codes of (unit q of the four, activation row
// t) in lane group q and zeros elsewhere: one instruction = the sums of four units for four rows.  A 16-byte record of the
// low-nibble plane serves two units (low and high nibbles) with the matching 16 bytes of the bit-pair plane; the codes stay
// unsigned (0..63) and the offset of 32 goes into the sum as -32 * (sum of the unit's 16 activation codes), which the Q8_K
// quantization delivers anyway.  Scaling per lane: acc = fma(fp32(d * sc) * dx, float(isum - 32 * bsum), acc).
// Step st of a trip = half a super-block (records 4 (st & 1) + g of super-block st / 2): low nibbles are units 8 (st & 1) + g,
// high nibbles units 8 (st & 1) + 4 + g.
constexpr int K6_ST = 10;  // steps per trip, at most: five super-blocks (the launcher takes fewer for shorter slices)
// ST = steps per trip: the slice in one trip where it fits (6, 8 or 10); xpad = super-blocks the last trip of a slice reaches
// past the row (zeros in LDS)
template <int XT, int MT, int ST = K6_ST>
__global__ __launch_bounds__(512) void kq6_gemv_mfma_kernel(KGemvArgs a, int S, int sps, KMeet km) {  // sps = super-blocks per slice; km.lrows in super-blocks
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int TH = MT / 4;
  constexpr int TSB = ST / 2;  // super-blocks per trip
  const int nsb = a.nsb, nu = nsb * 16, K = nsb * QK_K;
  const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int pidx = 0;
#pragma unroll
  for (int p = 1; p < KQ_MAX_PARTS; p++)
    if (p < a.nparts && (int)blockIdx.x >= a.wg_start[p]) pidx = p;
  const KGemvPart& pt = a.part[pidx];
  const KTile mt = kq_tile(a);
  if (!mt.active) return;  // uniform, ahead of every barrier
  const int N = pt.N;
  const int tiles_wg = nwaves / S;
  const int tile = ((int)blockIdx.x - a.wg_start[pidx]) * tiles_wg + wave / S;
  const int sg = km.SG > 1 ? (int)blockIdx.z : 0;  // slice group: the workgroup's slices are [sg S, sg S + S)
  const int slice = sg * S + wave % S;
  const int row0 = tile * 16;
  const bool tile_ok = row0 < N;
  const int s0 = slice * sps, s1 = min(nsb, s0 + sps);  // this wave's super-blocks
  const int ks0 = min(nsb, sg * S * sps), ks1 = min(nsb, ks0 + S * sps);  // the workgroup's; LDS rows count from ks0
  const int nloc = ks1 - ks0, lsb = km.lrows, nul = nloc * 16;

  const int wsu = (sps + TSB - 1) / TSB * TSB * 16;  // units of weight scales per wave: whole trips
  u32x4* xc = reinterpret_cast<u32x4*>(smem);                     // [(unit - 16 ks0) * MT + m] the unit's 16 codes
  u32x4* zrec = xc + (size_t)lsb * 16 * MT;
  int* bs16 = reinterpret_cast<int*>(zrec + 1);                   // [(unit - 16 ks0) * MT + m] sum of the unit's codes
  float* dxs = reinterpret_cast<float*>(bs16 + (size_t)lsb * 16 * MT);  // [(super-block - ks0) * MT + m]
  float* ws_all = dxs + (size_t)lsb * MT;
  float* ws = ws_all + (size_t)wave * wsu * 16;
  int* s_flag = reinterpret_cast<int*>(ws_all + (size_t)nwaves * wsu * 16);
  f32x4* red = reinterpret_cast<f32x4*>(smem) + (size_t)wave * TH * 64;  // takes the place of the codes once every wave is done with them

  const uint32_t sbt = (uint32_t)N * (uint32_t)nsb;
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(kq_at(pt.w.a, mt.eoff)), 0, sbt * 128u, 0x00020000);
  const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(kq_at(pt.w.h, mt.eoff)), 0, sbt * 64u, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsc = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(kq_at(pt.w.s, mt.eoff)), 0, sbt * 16u, 0x00020000);
  const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(kq_at(pt.w.d, mt.eoff)), 0, sbt * 2u, 0x00020000);
  // ---- 1. weight scales of the tile and slice: 16 int8 and one fp16 per (row, super-block) -------------------------------------
  u32x4 sc[2];
  uint16_t scd[2];
#pragma unroll
  for (int k = 0; k < 2; k++) {
    const int ch = lane + 64 * k;
    const int r = ch / sps, si = ch - r * sps;
    const bool ok = tile_ok && r < 16 && row0 + r < N && s0 + si < nsb;
    const uint32_t idx = (uint32_t)(row0 + r) * (uint32_t)nsb + (uint32_t)(s0 + si);
    sc[k] = __builtin_amdgcn_raw_buffer_load_b128(rsc, ok ? idx * 16u : KBUF_OOB, 0, KBUF_NT);
    scd[k] = __builtin_amdgcn_raw_buffer_load_b16(rd, ok ? idx * 2u : KBUF_OOB, 0, KBUF_NT);
  }
  // ---- 2. weight codes: lane (row c, group g), step st: low-nibble record 4 (st & 1) + g and bit-pair record 2 (st & 1) + (g & 1)
  const int c = lane & 15, g = lane >> 4;
  const bool row_ok = tile_ok && row0 + c < N;
  const uint32_t rbase = (uint32_t)(row0 + c) * (uint32_t)nsb;
  u32x4 wl[ST], wh[ST];
  auto load_steps = [&](int sb0) {
#pragma unroll
    for (int st = 0; st < ST; st++) {
      const int sb = sb0 + (st >> 1);
      const bool ok = row_ok && sb < s1;
      wl[st] = __builtin_amdgcn_raw_buffer_load_b128(ra, ok ? ((rbase + (uint32_t)sb) * 8u + 4u * (st & 1) + (uint32_t)g) * 16u : KBUF_OOB, 0, KBUF_NT);
      wh[st] = __builtin_amdgcn_raw_buffer_load_b128(rh, ok ? ((rbase + (uint32_t)sb) * 4u + 2u * (st & 1) + (uint32_t)(g & 1)) * 16u : KBUF_OOB, 0, KBUF_NT);
    }
  };
  // (MoE row tiles -- short rows, the slice is one trip -- ask for the weights first: behind the image copy they would be a
  // second round trip to memory in a kernel that is little more than its prologue; all-Q6_K experts, 512 tokens: 250 us this
  // way, 256 the other)
  const bool wfirst = KMF_WEIGHTS_FIRST || a.tile_expert != nullptr;  // uniform
  if (wfirst && XT == KQ_IMAGE) load_steps(s0);
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // ---- 3. activations into LDS -------------------------------------------------------------------------------------------------
  if (XT == KQ_IMAGE) {  // codes [R][K], sums of 16 as int16 [R][K/16], scales [R][nsb]; R = MT, or the rows of a MoE image
    const size_t R = a.img_rows ? (size_t)a.img_rows : (size_t)MT;
    const u32x4* codes = reinterpret_cast<const u32x4*>(a.x);
    const int16_t* sums = reinterpret_cast<const int16_t*>(reinterpret_cast<const char*>(a.x) + R * K);
    const float* dd = reinterpret_cast<const float*>(reinterpret_cast<const char*>(a.x) + R * K + R * nsb * 32);
    // thread (row m = tid % MT, unit tid / MT), a batch of units requested before the first is stored, as in the Q4_K kernel
    const int m = tid & (MT - 1), p0 = tid / MT, pstep = nthreads / MT;
    const size_t src = (size_t)kq_tile_in_row(a, mt, m);
    float dv[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
      if (p0 + i * pstep < nloc) dv[i] = dd[src * nsb + ks0 + p0 + i * pstep];
    for (int u0 = p0; u0 < nul; u0 += pstep * KMF_COPY_UNROLL) {
      u32x4 cv[KMF_COPY_UNROLL];
      int16_t sv[KMF_COPY_UNROLL];
#pragma unroll
      for (int i = 0; i < KMF_COPY_UNROLL; i++) {
        const int u = u0 + i * pstep;
        if (u < nul) {
          cv[i] = codes[src * nu + ks0 * 16 + u];
          sv[i] = sums[src * nu + ks0 * 16 + u];
        }
      }
#pragma unroll
      for (int i = 0; i < KMF_COPY_UNROLL; i++) {
        const int u = u0 + i * pstep;
        if (u < nul) {
          xc[(size_t)u * MT + m] = cv[i];
          bs16[(size_t)u * MT + m] = (int)sv[i];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
      if (p0 + i * pstep < nloc) dxs[(p0 + i * pstep) * MT + m] = dv[i];
    for (int sb = p0 + 2 * pstep; sb < nloc; sb += pstep) dxs[sb * MT + m] = dd[src * nsb + ks0 + sb];
  } else {
    const int ipr = K >> 3;      // items (eight elements) per row
    const int iwg = nloc << 5;   // of them in this workgroup's super-blocks
    const int nitems = MT * iwg;
    const float inv_iwg = 1.0f / (float)iwg;
    constexpr int QI = KMF_QUANT_BATCH;  // (a batch of items is requested before the first is quantized)
    for (int it0 = tid; it0 < nitems; it0 += nthreads * QI) {  // whole half-waves
      float v[QI][8];
#pragma unroll
      for (int b = 0; b < QI; b++) {
        const int it = it0 + b * nthreads;
        const int m = (int)(((float)it + 0.5f) * inv_iwg), i = it - m * iwg;
#pragma unroll
        for (int e = 0; e < 8; e++) v[b][e] = 0.f;
        if (it < nitems && m < a.M) load8<XT == KQ_IMAGE ? MLLM_HIP_F32 : XT>(a.x, ((int64_t)m * ipr + 32 * ks0 + i) * 8, v[b]);
      }
      if (it0 == tid) load_steps(s0);  // the weights right behind the first batch: they arrive while it is quantized
#pragma unroll
      for (int b = 0; b < QI; b++) {
        const int it = it0 + b * nthreads;
        if (it >= nitems) break;
        const Q8KItem qi = quantize_q8k_item(v[b], lane);
        const int s16 = qi.sum8 + __builtin_amdgcn_update_dpp(0, qi.sum8, 0xB1, 0xf, 0xf, true);
        const int m = (int)(((float)it + 0.5f) * inv_iwg), i = it - m * iwg;
        const int u = i >> 1;
        reinterpret_cast<u32x2*>(xc + (size_t)u * MT + m)[i & 1] = u32x2{qi.q0, qi.q1};
        if ((i & 1) == 0) bs16[(size_t)u * MT + m] = s16;
        if ((i & 31) == 0) dxs[(i >> 5) * MT + m] = qi.d;
      }
    }
  }
  if (!wfirst && XT == KQ_IMAGE) load_steps(s0);
  if (XT != KQ_IMAGE && tid >= (nloc << 5) * MT) load_steps(s0);  // (threads without an item to quantize)
  if (tid == 0) zrec[0] = u32x4{0u, 0u, 0u, 0u};
  for (int i = tid; i < (lsb - nloc) * 16 * MT; i += nthreads) {
    xc[(size_t)nul * MT + i] = u32x4{0u, 0u, 0u, 0u};
    bs16[(size_t)nul * MT + i] = 0;
  }
  for (int i = tid; i < (lsb - nloc) * MT; i += nthreads) dxs[nloc * MT + i] = 0.f;
#pragma unroll
  for (int k = 0; k < 2; k++) {
    const int ch = lane + 64 * k;
    const int r = ch / sps, si = ch - r * sps;
    if (r < 16) {
      const float d = (s0 + si < nsb) ? f16bits_to_f32(scd[k]) : 0.f;
      const uint32_t wds[4] = {sc[k].x, sc[k].y, sc[k].z, sc[k].w};
#pragma unroll
      for (int j = 0; j < 16; j++) ws[(16 * si + j) * 16 + r] = d * (float)(int8_t)(wds[j >> 2] >> (8 * (j & 3)));
    }
  }
  for (int i = sps * 256 + lane; i < wsu * 16; i += 64) ws[i] = 0.f;
  __syncthreads();

  // ---- 4. unit sums on the matrix cores, scaling on the vector ALU ----------------------------------------------------------------
  const int q = (lane & 15) >> 2, tt = lane & 3;
  const bool mine = g == q;
  const int shl = 2 * (g >> 1);  // this lane's low-nibble units take bit pair g / 2 of the high plane, its high-nibble units g / 2 + 2
  f32x4 acc[TH];
#pragma unroll
  for (int h = 0; h < TH; h++) acc[h] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int sb0 = s0; sb0 < s1; sb0 += TSB) {
    if (sb0 != s0) load_steps(sb0);
    const int u0 = (sb0 - ks0) * 16;  // first unit of the trip in LDS
    const u32x4* bl[TH];
    const int* bsl[TH];
    const float* dxl[TH];
#pragma unroll
    for (int h = 0; h < TH; h++) {
      bl[h] = mine ? xc + (size_t)(u0 + q) * MT + 4 * h + tt : zrec;
      bsl[h] = bs16 + (size_t)(u0 + q) * MT + 4 * h + tt;
      dxl[h] = dxs + (sb0 - ks0) * MT + 4 * h + tt;
    }
    const int bstep = mine ? MT : 0;
    const float* wsl = ws + (size_t)((sb0 - s0) * 16 + q) * 16 + 4 * g;
    u32x4 B[2][2][TH];
    int bs[2][2][TH];
    float dxv[2][TH];
    f32x4 dsv[2][2];
    kv4i D[2][2][TH];
    auto fetch_b = [&](int set, int st) {  // units 8 st + q (low nibbles) and 8 st + 4 + q (high)
#pragma unroll
      for (int h = 0; h < TH; h++) {
        B[set][0][h] = bl[h][(8 * st) * bstep];
        B[set][1][h] = bl[h][(8 * st + 4) * bstep];
      }
    };
    auto fetch_s = [&](int set, int st) {
#pragma unroll
      for (int h = 0; h < TH; h++) {
        bs[set][0][h] = bsl[h][(8 * st) * MT];
        bs[set][1][h] = bsl[h][(8 * st + 4) * MT];
        dxv[set][h] = dxl[h][(st >> 1) * MT];
      }
      dsv[set][0] = *reinterpret_cast<const f32x4*>(wsl + (8 * st) * 16);
      dsv[set][1] = *reinterpret_cast<const f32x4*>(wsl + (8 * st + 4) * 16);
    };
    auto issue = [&](int set, int st) {
      const uint32_t l4[4] = {wl[st].x, wl[st].y, wl[st].z, wl[st].w};
      const uint32_t h4[4] = {wh[st].x, wh[st].y, wh[st].z, wh[st].w};
      kv4i Alo, Ahi;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t hs = h4[e] >> shl;
        Alo[e] = (int)((l4[e] & 0x0f0f0f0fu) | ((hs & 0x03030303u) << 4));
        Ahi[e] = (int)(((l4[e] >> 4) & 0x0f0f0f0fu) | (((hs >> 4) & 0x03030303u) << 4));
      }
#pragma unroll
      for (int h = 0; h < TH; h++) {
        D[set][0][h] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Alo, __builtin_bit_cast(kv4i, B[set][0][h]), kv4i{0, 0, 0, 0}, 0, 0, 0);
        D[set][1][h] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Ahi, __builtin_bit_cast(kv4i, B[set][1][h]), kv4i{0, 0, 0, 0}, 0, 0, 0);
      }
    };
    auto scale = [&](int set, int st) {
      const bool live = sb0 + (st >> 1) < s1;  // uniform
#pragma unroll
      for (int h = 0; h < TH; h++) {
        const float dx = live ? dxv[set][h] : 0.f;
#pragma unroll
        for (int w = 0; w < 2; w++) {
          const int corr = -32 * bs[set][w][h];  // the codes went in as 0..63
          acc[h].x = fmaf(dsv[set][w].x * dx, (float)(D[set][w][h].x + corr), acc[h].x);
          acc[h].y = fmaf(dsv[set][w].y * dx, (float)(D[set][w][h].y + corr), acc[h].y);
          acc[h].z = fmaf(dsv[set][w].z * dx, (float)(D[set][w][h].z + corr), acc[h].z);
          acc[h].w = fmaf(dsv[set][w].w * dx, (float)(D[set][w][h].w + corr), acc[h].w);
        }
      }
    };
    fetch_b(0, 0);
#pragma unroll
    for (int st = 0; st < ST; st++) {
      issue(st & 1, st);
      if (st + 1 < ST) fetch_b((st + 1) & 1, st + 1);
      fetch_s(st & 1, st);
      __builtin_amdgcn_sched_barrier(0);
      if (st > 0) scale((st - 1) & 1, st - 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    scale((ST - 1) & 1, ST - 1);
  }
#pragma unroll
  for (int h = 0; h < TH; h++) {  // the four lanes of an activation row (units = 0..3 mod 4)
    float v[4] = {acc[h].x, acc[h].y, acc[h].z, acc[h].w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
      v[e] += __shfl_xor(v[e], 4, 64);
      v[e] += __shfl_xor(v[e], 8, 64);
    }
    acc[h] = f32x4{v[0], v[1], v[2], v[3]};
  }

  // ---- 5. slices of a tile in slice order, bias ------------------------------------------------------------------------------
  if (S > 1) {
    __syncthreads();
#pragma unroll
    for (int h = 0; h < TH; h++) red[h * 64 + lane] = acc[h];
    __syncthreads();
    if (wave % S != 0) return;
    for (int s = 1; s < S; s++)
#pragma unroll
      for (int h = 0; h < TH; h++) {
        const f32x4 o = red[(size_t)s * TH * 64 + h * 64 + lane];
        acc[h].x += o.x; acc[h].y += o.y; acc[h].z += o.z; acc[h].w += o.w;
      }
  }
  if (km.SG > 1) {  // the slice groups of a grid column meet in global memory, as in the Q4_K kernel (S = 1 here: every wave is a tile)
    const int SG = km.SG;
    const int li = 4 * g + tt;
    float* pbase = km.part + (((size_t)blockIdx.x * nwaves + wave) * SG) * 128;
    if (q == 0) {
#pragma unroll
      for (int h = 0; h < TH; h++) {
        float* dst = pbase + (size_t)sg * 128 + (16 * h + li) * 4;
        __hip_atomic_store(dst + 0, acc[h].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(dst + 1, acc[h].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(dst + 2, acc[h].z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(dst + 3, acc[h].w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      unsigned* cnt = km.counters + (size_t)blockIdx.x * km.cstride;
      const unsigned old = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int last = old == (unsigned)(SG - 1);
      if (last) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
      *s_flag = last;
    }
    __syncthreads();
    if (!*s_flag) return;
    if (q == 0) {
#pragma unroll
      for (int h = 0; h < TH; h++) {
        float pv[8][4];
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const float* src = pbase + (size_t)min(u, SG - 1) * 128 + (16 * h + li) * 4;
#pragma unroll
          for (int e = 0; e < 4; e++) pv[u][e] = __hip_atomic_load(src + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        acc[h] = f32x4{pv[0][0], pv[0][1], pv[0][2], pv[0][3]};
#pragma unroll
        for (int u = 1; u < 8; u++)
          if (u < SG) { acc[h].x += pv[u][0]; acc[h].y += pv[u][1]; acc[h].z += pv[u][2]; acc[h].w += pv[u][3]; }
      }
    }
  }
  if (!tile_ok || q != 0) return;
  const int n = row0 + 4 * g;
#pragma unroll
  for (int h = 0; h < TH; h++) {
    const int t = 4 * h + tt;
    if (t >= mt.rows) continue;
    const float v[4] = {acc[h].x, acc[h].y, acc[h].z, acc[h].w};
    float* yrow = pt.y + (int64_t)kq_tile_out_row(a, mt, t) * N;
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (n + e < N) yrow[n + e] = pt.bias ? v[e] + pt.bias[n + e] : v[e];
  }
}

static int k6mf_steps(int sps) { return sps <= 3 ? 6 : (sps <= 4 ? 8 : K6_ST); }
// super-blocks the last trip of a slice reads past the row (whole trips from the slice's first super-block)
static int k6mf_xpad(int nsb, int S, int sps) {
  const int tsb = k6mf_steps(sps) / 2;
  int pad = 0;
  for (int s = 0; s < S; s++) {
    const int s0 = s * sps, s1 = std::min(nsb, s0 + sps);
    if (s1 > s0) pad = std::max(pad, s0 + ((s1 - s0 - 1) / tsb + 1) * tsb - nsb);
  }
  return pad;
}
template <int MT>
static size_t k6mf_lds_bytes(int nsb, int sps, int nwaves, int S) {
  const int tsb = k6mf_steps(sps) / 2, rows = nsb + k6mf_xpad(nsb, S, sps);
  const int wsu = (sps + tsb - 1) / tsb * tsb * 16;
  const size_t need = (size_t)rows * 16 * MT * 16 + 16 + (size_t)rows * 16 * MT * 4 + (size_t)rows * MT * 4 + (size_t)nwaves * wsu * 64 + 16;
  // the partial sums of the slices reuse the code area: it must hold them
  return std::max(need, (size_t)nwaves * (MT / 4) * 1024);
}
// the same with one slice per workgroup (slice groups over the grid's z): the slice's super-blocks in whole trips
template <int MT>
static size_t k6mf_lds_bytes_z(int sps, int nwaves) {
  const int tsb = k6mf_steps(sps) / 2, rows = (sps + tsb - 1) / tsb * tsb;
  return (size_t)rows * 16 * MT * 16 + 16 + (size_t)rows * 16 * MT * 4 + (size_t)rows * MT * 4 + (size_t)nwaves * rows * 16 * 64 + 16;
}
static void k6mf_split(int nsb, int& S, int& sps) {
  S = 1;
  while (S < 8 && nsb > 5 * S) S *= 2;
  sps = (nsb + S - 1) / S;
}
static bool kq6_mfma_fits(int MT, int nsb) {
  int S, sps;
  k6mf_split(nsb, S, sps);
  if (sps > 8) return false;  // scale records: at most 128 per wave
  return (MT == 4 ? k6mf_lds_bytes<4>(nsb, sps, 8, S) : k6mf_lds_bytes<8>(nsb, sps, 8, S)) <= 160 * 1024;
}
static int kq_meet_waves(const KGemvArgs& a, int SG);
// every K slice a workgroup of its own (four to six row tiles), meeting in the caller's workspace: as launch_kq4_mfma_z
template <int XT, int MT>
static int launch_kq6_mfma_z(const KGemvArgs& a_in, const KMeetRoom& room, hipStream_t st) {
  KGemvArgs a = a_in;
  int SG, sps;
  k6mf_split(a.nsb, SG, sps);
  const int nwaves = kq_meet_waves(a, SG);
  unsigned grid = 0;
  for (int p = 0; p < a.nparts; p++) {
    a.wg_start[p] = (int)grid;
    grid += (unsigned)(((a.part[p].N + 15) / 16 + nwaves - 1) / nwaves);
  }
  a.wg_start[a.nparts] = (int)grid;
  if (SG < 2 || sps > 8 || g_kq_meet == 0 || !room.part || (size_t)grid * nwaves * SG * 512 > room.part_bytes || grid > 1024u) return KQ_NOT_TAKEN;
  KMeet km{};
  km.SG = SG;
  const int tsb = k6mf_steps(sps) / 2;
  km.lrows = (sps + tsb - 1) / tsb * tsb;
  km.part = static_cast<float*>(room.part);
  RC_RET(gemv_counter_block(room.key, st, &km.counters));
  km.cstride = 1;
  while (km.cstride < 32 && (size_t)grid * km.cstride * 2 <= 1024u) km.cstride *= 2;
  const size_t lds = k6mf_lds_bytes_z<MT>(sps, nwaves);
  auto go = [&](auto kern) {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3(grid, 1, (unsigned)SG), dim3(nwaves * 64), lds, st, a, 1, sps, km);
    return (int)hipGetLastError();
  };
  switch (k6mf_steps(sps)) {
    case 6: return go(kq6_gemv_mfma_kernel<XT, MT, 6>);
    case 8: return go(kq6_gemv_mfma_kernel<XT, MT, 8>);
    default: return go(kq6_gemv_mfma_kernel<XT, MT, K6_ST>);
  }
}
template <int XT, int MT>
static int launch_kq6_mfma_t(const KGemvArgs& a_in, hipStream_t st, unsigned grid_y = 1) {
  KGemvArgs a = a_in;
  int S, sps;
  k6mf_split(a.nsb, S, sps);
  int nwaves = XT == KQ_IMAGE ? 4 : 8;
  if (nwaves < S) nwaves = S;
  const int tiles_wg = nwaves / S;
  unsigned grid = 0;
  for (int p = 0; p < a.nparts; p++) {
    a.wg_start[p] = (int)grid;
    grid += (unsigned)(((a.part[p].N + 15) / 16 + tiles_wg - 1) / tiles_wg);
  }
  a.wg_start[a.nparts] = (int)grid;
  const size_t lds = k6mf_lds_bytes<MT>(a.nsb, sps, nwaves, S);
  if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
  KMeet km{};
  km.SG = 1;
  km.lrows = a.nsb + k6mf_xpad(a.nsb, S, sps);
  auto go = [&](auto kern) {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3(grid, grid_y), dim3(nwaves * 64), lds, st, a, S, sps, km);
    return (int)hipGetLastError();
  };
  switch (k6mf_steps(sps)) {
    case 6: return go(kq6_gemv_mfma_kernel<XT, MT, 6>);
    case 8: return go(kq6_gemv_mfma_kernel<XT, MT, 8>);
    default: return go(kq6_gemv_mfma_kernel<XT, MT, K6_ST>);
  }
}
template <int XT>
static int launch_kq6_mfma(const KGemvArgs& a, hipStream_t st) {
  return a.M <= 4 ? launch_kq6_mfma_t<XT, 4>(a, st) : launch_kq6_mfma_t<XT, 8>(a, st);
}

static int g_kq_path = 0;  // 1: always the dot4 kernel, 2: the matrix-core kernels wherever they fit (comparison runs and tests)


// ---- many rows: the matrix-core GEMM of the block formats (moe.hip, qg_kernel) with these weights -------------------------
// Same scheme as for Q4_0 / Q8_0: both operands as fp16 with their scales folded in, fp32 accumulation in
// v_mfma_f32_32x32x16_f16.  Activations: the Q8_K round trip xh = fp16(d * q) (codes and d bit-exact, the product rounded
// once).  Weights: Q4_K as 4-bit codes q with the sub-block's fp16(d * sc) and fp16(dmin * m), value = fma(q, ds, -dm)
// rounded once; Q6_K as int8 codes q - 32 with fp16(d * sc) per 16 elements.  Within about 5e-4 relative L2 of the
// reference's integer / fp32 arithmetic.
//
// code area, Q4_K: one output dword per thread, in the order of the Q4_0 gemm layout
template <int WT>
__global__ __launch_bounds__(256) void kqg_prepack_q_kernel(const uint8_t* __restrict__ blocks, uint32_t* __restrict__ P, int N, int K,
                                                            int64_t words) {
  const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (w >= words) return;
  const int kbs = K / 64, nsb = K / QK_K;
  uint32_t v = 0;
  if (WT == MLLM_HIP_Q4_K) {
    const int d = (int)(w % 4), l = (int)((w / 4) % 64);
    const int64_t blk = w / 256;
    const int kb = (int)(blk % kbs), nb = (int)(blk / kbs);
    const int n = nb * 32 + (l & 31), k0 = kb * 64 + d * 16 + (l >> 5) * 8;
    if (n < N) {
      const uint8_t* qs = blocks + ((int64_t)n * nsb + k0 / QK_K) * 144 + 16;
      const int e = k0 % QK_K, c = e >> 6, p = e & 63;  // 64-element chunk, position: low nibbles first, then high
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const uint32_t byte = qs[32 * c + (p & 31) + i];
        const uint32_t q = p < 32 ? (byte & 15u) : (byte >> 4);
        v |= q << (4 * ((i >> 1) + 4 * (i & 1)));
      }
    }
  } else {
    const int x = (int)(w % 4), l = (int)((w / 4) % 64), pl = (int)((w / 256) % 2);
    const int64_t blk = w / 512;
    const int kb = (int)(blk % kbs), nb = (int)(blk / kbs);
    const int d = 2 * pl + x / 2;
    const int n = nb * 32 + (l & 31), k0 = kb * 64 + d * 16 + (l >> 5) * 8 + 4 * (x % 2);
    if (n < N) {
      const uint8_t* b = blocks + ((int64_t)n * nsb + k0 / QK_K) * 210;
      uint32_t c[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {  // dequantize_row_q6_K's element order: halves of 128, quarters of 32
        const int e = k0 % QK_K + i, h = e >> 7, r = e & 127, g = r >> 5, ll = r & 31;
        int lo = b[64 * h + ((g & 1) ? 32 : 0) + ll];
        lo = g >= 2 ? (lo >> 4) : (lo & 15);
        const int hi = (b[128 + 32 * h + ll] >> (2 * g)) & 3;
        c[i] = (uint32_t)((lo | (hi << 4)) - 32) & 0xffu;
      }
      v = c[0] | (c[2] << 8) | (c[1] << 16) | (c[3] << 24);
    }
  }
  P[w] = v;
}
// scale records: one thread per (32-row group, 64-element step, row)
template <int WT>
__global__ __launch_bounds__(256) void kqg_prepack_s_kernel(const uint8_t* __restrict__ blocks, u32x2* __restrict__ S, int N, int K, int x86,
                                                            int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  const int kbs = K / 64, nsb = K / QK_K;
  const int row = (int)(i % 32), kb = (int)((i / 32) % kbs), nb = (int)(i / 32 / kbs);
  const int n = nb * 32 + row;
  u32x2 v{0u, 0u};
  if (n < N) {
    if (WT == MLLM_HIP_Q4_K) {
      const uint8_t* b = blocks + ((int64_t)n * nsb + kb / 4) * 144;
      const float d = f16bits_to_f32(field_bits(b, x86)), dmin = f16bits_to_f32(field_bits(b + 2, x86));
      const K4Scales k = k4_scales(bytes_u32(b + 4), bytes_u32(b + 8), bytes_u32(b + 12));
      const int j = 2 * (kb % 4);
      v.x = (uint32_t)f32_to_f16bits(d * (float)byte_of(k.sc0, k.sc1, j)) | ((uint32_t)f32_to_f16bits(d * (float)byte_of(k.sc0, k.sc1, j + 1)) << 16);
      v.y = (uint32_t)f32_to_f16bits(dmin * (float)byte_of(k.mn0, k.mn1, j)) | ((uint32_t)f32_to_f16bits(dmin * (float)byte_of(k.mn0, k.mn1, j + 1)) << 16);
    } else {
      const uint8_t* b = blocks + ((int64_t)n * nsb + kb / 4) * 210;
      const float d = f16bits_to_f32(field_bits(b + 208, x86));
      const int8_t* sc = reinterpret_cast<const int8_t*>(b + 192) + 4 * (kb % 4);
      v.x = (uint32_t)f32_to_f16bits(d * (float)sc[0]) | ((uint32_t)f32_to_f16bits(d * (float)sc[1]) << 16);
      v.y = (uint32_t)f32_to_f16bits(d * (float)sc[2]) | ((uint32_t)f32_to_f16bits(d * (float)sc[3]) << 16);
    }
  }
  S[i] = v;
}
// activations: Q8_K quantization and back to fp16 in one pass, xh[rows][K]
__global__ __launch_bounds__(256) void kq_act_f16_kernel(const void* __restrict__ x, int x_dtype, uint16_t* __restrict__ xh, int64_t nitems) {
  const int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x;  // nitems is a multiple of 32: whole half-waves
  if (it >= nitems) return;
  float v[8];
  if (x_dtype == MLLM_HIP_F32) load8<MLLM_HIP_F32>(x, it * 8, v);
  else load8<MLLM_HIP_BF16>(x, it * 8, v);
  const Q8KItem r = quantize_q8k_item(v, threadIdx.x & 63);
  uint32_t o[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const uint32_t word = j < 2 ? r.q0 : r.q1;
    const float a = r.d * (float)(int8_t)(word >> (16 * (j & 1)));
    const float b = r.d * (float)(int8_t)(word >> (16 * (j & 1) + 8));
    o[j] = (uint32_t)f32_to_f16bits(a) | ((uint32_t)f32_to_f16bits(b) << 16);
  }
  *reinterpret_cast<u32x4*>(xh + it * 8) = u32x4{o[0], o[1], o[2], o[3]};
}

}  // namespace mllmhip

using namespace mllmhip;

static int kq_check(int wtype, const void* packed, int64_t N, int64_t K) {
  if (wtype != MLLM_HIP_Q4_K && wtype != MLLM_HIP_Q6_K) return MLLM_HIP_E_BADARG;
  if (!packed || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (K % QK_K) return MLLM_HIP_E_SHAPE;
  if (N > INT32_MAX || N * (K / QK_K) * 128 >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;  // 32-bit buffer offsets
  if (reinterpret_cast<uintptr_t>(packed) % 256) return MLLM_HIP_E_ALIGN;
  return 0;
}

MLLM_API int mllm_hip_kq_set_path(int path) {
  if (path != 0 && path != 1 && path != 2) return MLLM_HIP_E_BADARG;
  g_kq_path = path;
  return 0;
}
MLLM_API int mllm_hip_kq_set_slice_meeting(int mode, int waves_per_wg) {
  if (mode < -1 || mode > 1 || (waves_per_wg != 0 && (waves_per_wg < 1 || waves_per_wg > 8))) return MLLM_HIP_E_BADARG;
  g_kq_meet = mode;
  g_kq_meet_min = mode == 1 ? 2 : 4;
  g_kq_meet_waves = waves_per_wg;
  return 0;
}

MLLM_API int mllm_hip_kq_set_tuning(int lanes_per_row, int waves_per_wg, int units_in_flight) {
  auto ok = [](int v, std::initializer_list<int> allowed) {
    for (int x : allowed)
      if (v == x) return true;
    return false;
  };
  if (!ok(lanes_per_row, {0, 8, 16, 32, 64}) || !ok(waves_per_wg, {0, 1, 2, 4}) || !ok(units_in_flight, {0, 1, 2, 4})) return MLLM_HIP_E_BADARG;
  g_kq_G = lanes_per_row;
  g_kq_NW = waves_per_wg;
  g_kq_U = units_in_flight;
  return 0;
}

MLLM_API size_t mllm_hip_kq_packed_bytes(int wtype, int64_t N, int64_t K) {
  if ((wtype != MLLM_HIP_Q4_K && wtype != MLLM_HIP_Q6_K) || N <= 0 || K <= 0 || K % QK_K) return 0;
  return kq_packed_bytes(wtype, N, K);
}

MLLM_API int mllm_hip_kq_prepack(int wtype, const void* blocks, int weight_scale_mode, void* packed, int64_t N, int64_t K, void* stream) {
  int rc = kq_check(wtype, packed, N, K);
  if (rc) return rc;
  if (!blocks || (weight_scale_mode != MLLM_HIP_SCALE_IEEE && weight_scale_mode != MLLM_HIP_SCALE_X86_REF)) return MLLM_HIP_E_BADARG;
  const int64_t nsb = N * (K / QK_K);
  hipLaunchKernelGGL(kq_prepack_kernel, dim3((unsigned)((nsb * 8 + 255) / 256)), dim3(256), 0, (hipStream_t)stream, wtype,
                     (const uint8_t*)blocks, weight_scale_mode == MLLM_HIP_SCALE_X86_REF, kq_view(wtype, packed, N, K), nsb);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_kq_dequantize(int wtype, const void* packed, float* w, int64_t N, int64_t K, void* stream) {
  int rc = kq_check(wtype, packed, N, K);
  if (rc) return rc;
  if (!w) return MLLM_HIP_E_BADARG;
  const int64_t nsb = N * (K / QK_K);
  hipLaunchKernelGGL(kq_dequantize_kernel, dim3((unsigned)nsb), dim3(256), 0, (hipStream_t)stream, wtype, kq_view(wtype, packed, N, K), w, nsb);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_quantize_q8_K(const void* x, int x_dtype, int8_t* codes, float* d, int16_t* bsums, int64_t M, int64_t K, void* stream) {
  if (!x || !codes || !d || !bsums || M <= 0 || K <= 0 || (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16)) return MLLM_HIP_E_BADARG;
  if (K % QK_K) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(codes) % 8) return MLLM_HIP_E_ALIGN;
  const int64_t nitems = M * K / 8;
  hipLaunchKernelGGL(quantize_q8k_kernel, dim3((unsigned)((nitems + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, x_dtype, codes, d,
                     bsums, nitems, nitems);
  return (int)hipGetLastError();
}

MLLM_API size_t mllm_hip_kq_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || K % QK_K) return 0;
  return (size_t)8 * K + (size_t)8 * (K / QK_K) * 36;  // one group of eight rows: codes, sums of 16, scales
}

MLLM_API size_t mllm_hip_kq_workspace_bytes_n(int64_t M, int64_t K, int64_t N_total) {
  const size_t img = mllm_hip_kq_workspace_bytes(M, K);
  if (!img || N_total <= 0) return img;
  return align_up(img, 256) + kmf_part_bytes((int)(K / QK_K), N_total, KQ_MAX_PARTS);
}

MLLM_API int mllm_hip_linear_kq_multi(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype, int64_t M,
                                      int64_t K, void* workspace, void* stream) {
  return mllm_hip_linear_kq_multi_ws(wtype, nparts, parts, x, x_dtype, M, K, workspace, workspace ? mllm_hip_kq_workspace_bytes(M, K) : 0,
                                     stream);
}

MLLM_API int mllm_hip_linear_kq_multi_ws(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype, int64_t M,
                                         int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  if (nparts < 1 || nparts > KQ_MAX_PARTS || !parts) return MLLM_HIP_E_BADARG;
  if (!x || M <= 0 || (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16)) return MLLM_HIP_E_BADARG;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16) return MLLM_HIP_E_ALIGN;
  for (int p = 0; p < nparts; p++) {
    int rc = kq_check(wtype, parts[p].packed, parts[p].N, K);
    if (rc) return rc;
    if (!parts[p].y) return MLLM_HIP_E_BADARG;
  }
  const size_t xrow = (size_t)K * (x_dtype == MLLM_HIP_F32 ? 4 : 2);
  const int nsb = (int)(K / QK_K);
  hipStream_t st = (hipStream_t)stream;
  int rc = 0;
  const size_t img_bytes = mllm_hip_kq_workspace_bytes(M, K);
  if (workspace && workspace_bytes < img_bytes) return MLLM_HIP_E_BADARG;
  // what lies behind the image serves the partial sums of K slices that meet in global memory
  KMeetRoom room{workspace, nullptr, 0};
  if (workspace && workspace_bytes > align_up(img_bytes, 256)) {
    room.part = reinterpret_cast<char*>(workspace) + align_up(img_bytes, 256);
    room.part_bytes = workspace_bytes - align_up(img_bytes, 256);
  }
  for (int64_t m0 = 0; m0 < M; m0 += 8) {  // more than eight rows: groups of eight (each streams the weights again)
    const int rows = (int)(M - m0 < 8 ? M - m0 : 8);
    const void* xg = reinterpret_cast<const char*>(x) + m0 * xrow;
    KGemvArgs a{};
    for (int p = 0; p < nparts; p++)
      a.part[p] = KGemvPart{kq_view(wtype, parts[p].packed, parts[p].N, K), parts[p].bias, parts[p].y + m0 * parts[p].N, (int)parts[p].N};
    a.nparts = nparts;
    a.x = xg;
    a.M = rows;
    a.nsb = nsb;
    // Q4_K: from three rows on.  Q6_K (heavier unpacking, 200 registers): from five rows on, and with three or four rows of
    // more than 4096 elements (4B layer shapes q+k+v / o / gate+up / down, dot4 -> matrix cores: eight rows 14.8 / 13.8 / 33.3 /
    // 19.7 -> 13.8 / 12.6 / 25.0 / 19.7 us; four rows 11.1 / 10.1 / 24.1 / 17.8 -> 12.1 / 10.6 / 21.3 / 16.2).
    // The rule looks at the weight type, the number of rows and the row length only: a projection gives the same bits alone
    // and as a part of a launch.
    const bool mfma = rows >= 3 && g_kq_path != 1 &&
                      (wtype == MLLM_HIP_Q4_K ? kq4_mfma_fits(rows <= 4 ? 4 : 8, nsb)
                                              : (rows > 4 || nsb > 16 || g_kq_path == 2) && kq6_mfma_fits(rows <= 4 ? 4 : 8, nsb));
    int k6S = 1, k6sps = 0;
    k6mf_split(nsb, k6S, k6sps);
    // (Q6_K: from eight slices on; with four, 2560 x 4096 at eight rows, the one-workgroup form measured 12.7 us against 13.4)
    if (mfma && room.part && g_kq_meet != 0 &&
        (wtype == MLLM_HIP_Q4_K ? kmf_slices(nsb * 8) >= g_kq_meet_min : k6S >= (g_kq_meet == 1 ? 2 : 8))) {
      // long rows: every workgroup takes one K slice and quantizes just that part of x itself; the slices meet in the workspace
      const bool f32 = x_dtype == MLLM_HIP_F32, r4 = rows <= 4;
      if (wtype == MLLM_HIP_Q4_K)
        rc = r4 ? (f32 ? launch_kq4_mfma_z<MLLM_HIP_F32, 4>(a, room, st) : launch_kq4_mfma_z<MLLM_HIP_BF16, 4>(a, room, st))
                : (f32 ? launch_kq4_mfma_z<MLLM_HIP_F32, 8>(a, room, st) : launch_kq4_mfma_z<MLLM_HIP_BF16, 8>(a, room, st));
      else
        rc = r4 ? (f32 ? launch_kq6_mfma_z<MLLM_HIP_F32, 4>(a, room, st) : launch_kq6_mfma_z<MLLM_HIP_BF16, 4>(a, room, st))
                : (f32 ? launch_kq6_mfma_z<MLLM_HIP_F32, 8>(a, room, st) : launch_kq6_mfma_z<MLLM_HIP_BF16, 8>(a, room, st));
      if (rc == 0) continue;
      if (rc != KQ_NOT_TAKEN) return rc;
    }
    if (workspace && rows >= 3) {
      // several rows: quantize once for all workgroups; the GEMV then copies the image instead of quantizing
      const int MT = rows <= 4 ? 4 : 8;
      int8_t* img = reinterpret_cast<int8_t*>(workspace);
      const int64_t nitems = (int64_t)MT * K / 8;
      hipLaunchKernelGGL(quantize_q8k_kernel, dim3((unsigned)((nitems + 255) / 256)), dim3(256), 0, st, xg, x_dtype, img,
                         reinterpret_cast<float*>(img + (size_t)MT * K + (size_t)MT * nsb * 32),
                         reinterpret_cast<int16_t*>(img + (size_t)MT * K), nitems, (int64_t)rows * K / 8);
      a.x = img;
      if (mfma) rc = wtype == MLLM_HIP_Q4_K ? launch_kq4_mfma<KQ_IMAGE>(a, st) : launch_kq6_mfma<KQ_IMAGE>(a, st);
      else rc = wtype == MLLM_HIP_Q4_K ? launch_kq<MLLM_HIP_Q4_K, KQ_IMAGE>(a, st) : launch_kq<MLLM_HIP_Q6_K, KQ_IMAGE>(a, st);
    } else if (mfma && wtype == MLLM_HIP_Q4_K) {
      rc = x_dtype == MLLM_HIP_F32 ? launch_kq4_mfma<MLLM_HIP_F32>(a, st) : launch_kq4_mfma<MLLM_HIP_BF16>(a, st);
    } else if (mfma) {
      rc = x_dtype == MLLM_HIP_F32 ? launch_kq6_mfma<MLLM_HIP_F32>(a, st) : launch_kq6_mfma<MLLM_HIP_BF16>(a, st);
    } else if (wtype == MLLM_HIP_Q4_K) {
      rc = x_dtype == MLLM_HIP_F32 ? launch_kq<MLLM_HIP_Q4_K, MLLM_HIP_F32>(a, st) : launch_kq<MLLM_HIP_Q4_K, MLLM_HIP_BF16>(a, st);
    } else {
      rc = x_dtype == MLLM_HIP_F32 ? launch_kq<MLLM_HIP_Q6_K, MLLM_HIP_F32>(a, st) : launch_kq<MLLM_HIP_Q6_K, MLLM_HIP_BF16>(a, st);
    }
    if (rc) return rc;
  }
  return 0;
}

MLLM_API int mllm_hip_linear_kq(int wtype, const void* packed, const void* x, int x_dtype, const float* bias, float* y, int64_t M,
                                int64_t N, int64_t K, void* workspace, void* stream) {
  if (!y) return MLLM_HIP_E_BADARG;
  mllm_hip_gemv_part part{packed, bias, y, N};
  return mllm_hip_linear_kq_multi(wtype, 1, &part, x, x_dtype, M, K, workspace, stream);
}

// ---- MoE slots: one GEMV row per (token, expert) pair ---------------------------------------------------------------------------
// nparts sibling matrices per expert (gate and up, or down alone), packed0[p] = expert 0's matrix of part p, the experts'
// matrices mllm_hip_kq_packed_bytes(wtype, N, K) apart; slot s multiplies activation row s / slot_div by the matrices of
// expert ids[s] and writes row s of ys[p] ([slots][N]).  x2 (fp32, same rows as x): the activation is silu(x) * x2.
namespace mllmhip {
int exp_mode_accurate();  // layer_ops.hip: the setting of mllm_hip_set_exp_mode
int kq_moe_gemv(int wtype, int nparts, const void* const* packed0, float* const* ys, int64_t N, int64_t K, const void* x, int x_dtype,
                const float* x2, const int32_t* ids, int E, int slots, int slot_div, hipStream_t st) {
  if (x2 && x_dtype != MLLM_HIP_F32) return MLLM_HIP_E_BADARG;
  if (nparts < 1 || nparts > KQ_MAX_PARTS || slots < 1 || slots > 65535) return MLLM_HIP_E_SHAPE;
  KGemvArgs a{};
  for (int p = 0; p < nparts; p++) a.part[p] = KGemvPart{kq_view(wtype, packed0[p], N, K), nullptr, ys[p], (int)N};
  a.nparts = nparts;
  a.x = x;
  a.M = 1;
  a.nsb = (int)(K / QK_K);
  a.slot_ids = ids;
  a.x2 = x2;
  a.silu_accurate = exp_mode_accurate();
  a.slot_E = E;
  a.slot_div = slot_div;
  a.slot_div_slots = slots;
  a.estride = kq_packed_bytes(wtype, N, K);
  if (wtype == MLLM_HIP_Q4_K)
    return x_dtype == MLLM_HIP_F32 ? launch_kq<MLLM_HIP_Q4_K, MLLM_HIP_F32>(a, st) : launch_kq<MLLM_HIP_Q4_K, MLLM_HIP_BF16>(a, st);
  return x_dtype == MLLM_HIP_F32 ? launch_kq<MLLM_HIP_Q6_K, MLLM_HIP_F32>(a, st) : launch_kq<MLLM_HIP_Q6_K, MLLM_HIP_BF16>(a, st);
}

// The Q8_K image of `rows` activation rows of K elements (codes [rows][K], sums of 16 [rows][K/16] int16, scales
// [rows][K/256]) at `image`: what the matrix-core kernels copy into LDS.
size_t kq_image_bytes(int64_t rows, int64_t K) { return (size_t)rows * K + (size_t)rows * (K / 16) * 2 + (size_t)rows * (K / QK_K) * 4; }
int kq_quantize_image(const void* x, int x_dtype, void* image, int64_t rows, int64_t K, hipStream_t st) {
  const int64_t nitems = rows * K / 8;
  int8_t* codes = reinterpret_cast<int8_t*>(image);
  int16_t* bsums = reinterpret_cast<int16_t*>(codes + rows * K);
  float* d = reinterpret_cast<float*>(codes + rows * K + rows * (K / 16) * 2);
  hipLaunchKernelGGL(quantize_q8k_kernel, dim3((unsigned)((nitems + 255) / 256)), dim3(256), 0, st, x, x_dtype, codes, d, bsums, nitems,
                     nitems);
  return (int)hipGetLastError();
}
bool kq_moe_tiles_fit(int wtype, int64_t K) {
  return wtype == MLLM_HIP_Q4_K ? kq4_mfma_fits(8, (int)(K / QK_K)) : kq6_mfma_fits(8, (int)(K / QK_K));
}
// MoE row tiles on the matrix-core kernels: tile t (blockIdx.y) = up to eight expert-sorted positions of expert tile_expert[t];
// its rows read image rows row_ids[pos] / row_div (null: pos) and write rows out_ids[pos] (null: pos) of ys[p].
int kq_moe_tiles_gemv(int wtype, int nparts, const void* const* packed0, float* const* ys, int64_t N, int64_t K, const void* image,
                      int64_t img_rows, const int* tile_expert, const int* tile_row0, const int* tile_rows, const int* ntiles,
                      unsigned max_tiles, const int* row_ids, int row_div, const int* out_ids, hipStream_t st) {
  if (nparts < 1 || nparts > KQ_MAX_PARTS || max_tiles < 1 || max_tiles > 65535) return MLLM_HIP_E_SHAPE;
  KGemvArgs a{};
  for (int p = 0; p < nparts; p++) a.part[p] = KGemvPart{kq_view(wtype, packed0[p], N, K), nullptr, ys[p], (int)N};
  a.nparts = nparts;
  a.x = image;
  a.M = 8;
  a.nsb = (int)(K / QK_K);
  a.estride = kq_packed_bytes(wtype, N, K);
  a.tile_expert = tile_expert; a.tile_row0 = tile_row0; a.tile_rows = tile_rows; a.ntiles = ntiles;
  a.row_ids = row_ids; a.out_ids = out_ids; a.row_div = row_div > 0 ? row_div : 1;
  a.img_rows = (int)img_rows;
  return wtype == MLLM_HIP_Q4_K ? launch_kq4_mfma_t<KQ_IMAGE, 8>(a, st, max_tiles) : launch_kq6_mfma_t<KQ_IMAGE, 8>(a, st, max_tiles);
}
}  // namespace mllmhip

// ---- many rows on the matrix cores ------------------------------------------------------------------------------------------
static bool kq_type(int wtype) { return wtype == MLLM_HIP_Q4_K || wtype == MLLM_HIP_Q6_K; }
MLLM_API size_t mllm_hip_kq_gemm_packed_bytes(int wtype, int64_t N, int64_t K) {
  if (!kq_type(wtype) || N <= 0 || K <= 0 || K % QK_K) return 0;
  return (size_t)qg_bytes(wtype, N, K);
}
MLLM_API int mllm_hip_kq_gemm_prepack(int wtype, const void* blocks, int weight_scale_mode, void* gemm_packed, int64_t N, int64_t K,
                                      void* stream) {
  if (!kq_type(wtype) || !blocks || !gemm_packed || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (weight_scale_mode != MLLM_HIP_SCALE_IEEE && weight_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (K % QK_K || N > INT32_MAX || K > INT32_MAX || qg_bytes(wtype, N, K) >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(gemm_packed) % 16) return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int64_t words = qg_qbytes(wtype, N, K) / 4, count = qg_np(N) * (K / 64);
  const uint8_t* b = reinterpret_cast<const uint8_t*>(blocks);
  uint32_t* q = reinterpret_cast<uint32_t*>(gemm_packed);
  u32x2* sc = reinterpret_cast<u32x2*>(reinterpret_cast<char*>(gemm_packed) + qg_qbytes(wtype, N, K));
  const int x86 = weight_scale_mode == MLLM_HIP_SCALE_X86_REF;
  const dim3 gq((unsigned)((words + 255) / 256)), gs((unsigned)((count + 255) / 256));
  if (wtype == MLLM_HIP_Q4_K) {
    hipLaunchKernelGGL(kqg_prepack_q_kernel<MLLM_HIP_Q4_K>, gq, dim3(256), 0, st, b, q, (int)N, (int)K, words);
    hipLaunchKernelGGL(kqg_prepack_s_kernel<MLLM_HIP_Q4_K>, gs, dim3(256), 0, st, b, sc, (int)N, (int)K, x86, count);
  } else {
    hipLaunchKernelGGL(kqg_prepack_q_kernel<MLLM_HIP_Q6_K>, gq, dim3(256), 0, st, b, q, (int)N, (int)K, words);
    hipLaunchKernelGGL(kqg_prepack_s_kernel<MLLM_HIP_Q6_K>, gs, dim3(256), 0, st, b, sc, (int)N, (int)K, x86, count);
  }
  return (int)hipGetLastError();
}
MLLM_API size_t mllm_hip_linear_kq_gemm_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || K % QK_K) return 0;
  return align_up((size_t)M * K * 2, 256) + qg_route_bytes(M);
}
MLLM_API int mllm_hip_linear_kq_gemm(int wtype, const void* gemm_packed, const void* x, int x_dtype, const float* bias, float* y, int64_t M,
                                     int64_t N, int64_t K, void* workspace, void* stream) {
  if (!kq_type(wtype) || !gemm_packed || !x || !y || !workspace || M <= 0 || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (K % QK_K || M * K * 2 >= ((int64_t)1 << 32) || N > INT32_MAX || qg_bytes(wtype, N, K) >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16 || reinterpret_cast<uintptr_t>(gemm_packed) % 16 ||
      reinterpret_cast<uintptr_t>(y) % 16)
    return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  uint16_t* xh = reinterpret_cast<uint16_t*>(workspace);
  const int64_t nitems = M * K / 8;
  hipLaunchKernelGGL(kq_act_f16_kernel, dim3((unsigned)((nitems + 255) / 256)), dim3(256), 0, st, x, x_dtype, xh, nitems);
  return qg_linear_run(wtype, gemm_packed, xh, bias, y, M, N, K, reinterpret_cast<char*>(workspace) + align_up((size_t)M * K * 2, 256), nullptr, st);
}

// the same for short batches (M <= 256 gains; any M is accepted): K cut into ranges that run as separate workgroups
MLLM_API size_t mllm_hip_linear_kq_gemm_short_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % QK_K) return 0;
  return align_up(mllm_hip_linear_kq_gemm_workspace_bytes(M, K), 256) + qg_partial_bytes(M, N, K);
}
MLLM_API int mllm_hip_linear_kq_gemm_short(int wtype, const void* gemm_packed, const void* x, int x_dtype, const float* bias, float* y,
                                           int64_t M, int64_t N, int64_t K, void* workspace, void* stream) {
  if (!kq_type(wtype) || !gemm_packed || !x || !y || !workspace || M <= 0 || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (K % QK_K || M * K * 2 >= ((int64_t)1 << 32) || N > INT32_MAX || qg_bytes(wtype, N, K) >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 256 || reinterpret_cast<uintptr_t>(gemm_packed) % 16 ||
      reinterpret_cast<uintptr_t>(y) % 16)
    return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  uint16_t* xh = reinterpret_cast<uint16_t*>(workspace);
  const int64_t nitems = M * K / 8;
  hipLaunchKernelGGL(kq_act_f16_kernel, dim3((unsigned)((nitems + 255) / 256)), dim3(256), 0, st, x, x_dtype, xh, nitems);
  char* base = reinterpret_cast<char*>(workspace);
  void* partial = qg_partial_bytes(M, N, K) ? base + align_up(mllm_hip_linear_kq_gemm_workspace_bytes(M, K), 256) : nullptr;
  return qg_linear_run(wtype, gemm_packed, xh, bias, y, M, N, K, base + align_up((size_t)M * K * 2, 256), partial, st);
}
