// The operators either side of a quantized Linear in a decoder layer, for gfx950: RMSNorm, SiLU, elementwise add / mul,
// SiLU(gate) * up, softmax, top-k and the whole MoE gate (logits -> softmax -> top-k -> normalise).
//
// Arithmetic follows the reference's x86 CPU kernels:
//   RMSNorm   mllm/backends/cpu/kernels/x86/rmsnorm.cpp:17-52      y = x * (w * rms), rms = 1 / sqrt(mean(x^2) + eps)
//   SiLU      mllm/backends/cpu/kernels/x86/silu.cpp:16-27         x * (1 / (1 + exp_poly(-x)))
//   exp_poly  mllm/backends/cpu/kernels/x86/math.hpp:19-72         Cephes polynomial
//   softmax   mllm/backends/cpu/kernels/x86/softmax.cpp:18-76      exp_poly(x - max) * (1 / sum); expf for len <= 16
//   top-k     mllm/backends/cpu/ops/TopKOp.cpp:20-72               k extreme values, by value or by index
//   MoE gate  mllm/models/qwen3_moe/modeling_qwen3_moe_fa2.hpp:121-139
// Sums run in a different order than the CPU's vector lanes; everything elementwise is the same fp32 operation
// sequence.
//
// All of these are HBM- or latency-bound.  What they add for this GPU: the kernels that produce the input of a decode
// GEMV (RMSNorm, SiLU*up) can also write that input's Q8_0 image in the form the GEMV kernel copies into LDS, so the
// GEMV of every workgroup skips the quantization.
#include "qcommon.h"

namespace mllmhip {

// `accurate` replaces the polynomial (whose argument reduction, as written in the reference, leaves a relative error of
// about 2.1e-4 per unit of the binary exponent of the result) by expf.
__device__ __forceinline__ float silu_ref(float x, bool accurate) { return x * (1.0f / (1.0f + (accurate ? expf(-x) : exp_poly(-x)))); }

// ---- eight consecutive elements per lane ------------------------------------------------------------------------------
template <int XT>
struct Item8 {
  u32x4 r[XT == MLLM_HIP_F32 ? 2 : 1];
};
template <int XT>
__device__ __forceinline__ void item_load(const void* p, int64_t elem, Item8<XT>& it) {
  if (XT == MLLM_HIP_F32) {
    const u32x4* q = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(p) + elem);
    it.r[0] = q[0];
    it.r[XT == MLLM_HIP_F32 ? 1 : 0] = q[1];
  } else {
    it.r[0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p) + elem);
  }
}
template <int XT>
__device__ __forceinline__ void item_to_f32(const Item8<XT>& it, float (&v)[8]) {
  if (XT == MLLM_HIP_F32) {
    const u32x4 a = it.r[0], b = it.r[XT == MLLM_HIP_F32 ? 1 : 0];
    v[0] = __uint_as_float(a.x); v[1] = __uint_as_float(a.y); v[2] = __uint_as_float(a.z); v[3] = __uint_as_float(a.w);
    v[4] = __uint_as_float(b.x); v[5] = __uint_as_float(b.y); v[6] = __uint_as_float(b.z); v[7] = __uint_as_float(b.w);
  } else {
    const uint32_t w[4] = {it.r[0].x, it.r[0].y, it.r[0].z, it.r[0].w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      v[2 * j + 0] = __uint_as_float(w[j] << 16);
      v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}
// stores v in the tensor's type and leaves in v what a reader of the tensor will see (bf16: the rounded values)
template <int XT>
__device__ __forceinline__ void item_store(void* p, int64_t elem, float (&v)[8]) {
  if (XT == MLLM_HIP_F32) {
    u32x4* q = reinterpret_cast<u32x4*>(reinterpret_cast<float*>(p) + elem);
    q[0] = u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])};
    q[1] = u32x4{__float_as_uint(v[4]), __float_as_uint(v[5]), __float_as_uint(v[6]), __float_as_uint(v[7])};
  } else {
    u32x4 o = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
    *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(p) + elem) = o;
    const uint32_t w[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      v[2 * j + 0] = __uint_as_float(w[j] << 16);
      v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}

__device__ __forceinline__ float wave_sum(float v) { return group_sum<64>(v); }
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));
  v = fmaxf(v, dpp_f<0x4E>(v));
  v = fmaxf(v, dpp_f<0x141>(v));
  v = fmaxf(v, dpp_f<0x140>(v));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

// ---- RMSNorm ----------------------------------------------------------------------------------------------------------
struct RmsArgs {
  const void* x;
  const float* w;
  void* y;
  int64_t rows;
  int D;
  float eps;
  int add_unit_offset;
  QImage img;
};
// One workgroup per row; a lane keeps NI items of eight elements in registers between the two passes.
template <int XT, int NI>
__global__ __launch_bounds__(256) void rmsnorm_kernel(RmsArgs a) {
  __shared__ float s_grp[4 * NI];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t row = blockIdx.x;
  if (row >= a.rows) {  // only launched for the zero rows of an image
    image_zero_row(a.img, (int)row, tid, 256);
    return;
  }
  const int nitems = a.D >> 3;
  Item8<XT> raw[NI];
  Item8<MLLM_HIP_F32> wraw[NI];
#pragma unroll
  for (int k = 0; k < NI; k++) {
    const int it = min(tid + 256 * k, nitems - 1);
    item_load<XT>(a.x, row * a.D + (int64_t)it * 8, raw[k]);
  }
#pragma unroll
  for (int k = 0; k < NI; k++) {
    const int it = min(tid + 256 * k, nitems - 1);
    item_load<MLLM_HIP_F32>(a.w, (int64_t)it * 8, wraw[k]);
  }
  // Sum of squares in a fixed order (per item an fma chain, the 64 items of a group through the wave butterfly, the
  // groups one after the other): a function of the row alone, not of how rows are spread over workgroups.
  float v[NI][8];
#pragma unroll
  for (int k = 0; k < NI; k++) {
    item_to_f32<XT>(raw[k], v[k]);
    float p = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) p = fmaf(v[k][e], v[k][e], p);
    p = wave_sum(tid + 256 * k < nitems ? p : 0.f);
    if (lane == 0) s_grp[wave + 4 * k] = p;
  }
  __syncthreads();
  const int ngroups = (nitems + 63) >> 6;
  float total = 0.f;
  for (int g = 0; g < ngroups; g++) total += s_grp[g];
  const float rms = 1.0f / sqrtf(total / (float)a.D + a.eps);
#pragma unroll
  for (int k = 0; k < NI; k++) {
    const int it = tid + 256 * k;
    const bool valid = it < nitems;
    float wv[8], o[8];
    item_to_f32<MLLM_HIP_F32>(wraw[k], wv);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float mult = (a.add_unit_offset ? wv[e] + 1.0f : wv[e]) * rms;
      o[e] = valid ? v[k][e] * mult : 0.f;
    }
    if (valid) item_store<XT>(a.y, row * a.D + (int64_t)it * 8, o);
    if (a.img.base) quad_quantize_to_image(o, a.img, (int)row, it >> 2, it & 3, valid);
  }
}

// ---- elementwise: SiLU, SiLU(gate) * up, add, mul ---------------------------------------------------------------------
enum { EW_SILU = 0, EW_SILU_MUL = 1, EW_ADD = 2, EW_MUL = 3 };
struct EwArgs {
  const void* a;
  const void* b;
  void* y;
  int64_t rows;  // image: rows of D elements; without image rows * D is just the element count
  int D;
  int exp_accurate;
  QImage img;
};
template <int XT, int OP>
__global__ __launch_bounds__(256) void elementwise_kernel(EwArgs a) {
  const int ipr = a.D >> 3;  // items per row
  const int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = it / ipr;
  const int col = (int)(it - row * ipr);
  const int64_t total_rows = a.img.base ? max((int64_t)a.img.MT, a.rows) : a.rows;
  if (row >= total_rows) return;  // whole quads leave together: ipr is a multiple of 4 whenever an image is written
  float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const bool valid = row < a.rows;
  if (valid) {
    Item8<XT> ra, rb;
    float va[8], vb[8];
    item_load<XT>(a.a, it * 8, ra);
    if (OP != EW_SILU) item_load<XT>(a.b, it * 8, rb);
    item_to_f32<XT>(ra, va);
    if (OP != EW_SILU) item_to_f32<XT>(rb, vb);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      if (OP == EW_SILU) o[e] = silu_ref(va[e], a.exp_accurate);
      if (OP == EW_SILU_MUL) {
        // the reference runs SiLU and the product as two operators: the SiLU result is stored in the tensor's type first
        float s = silu_ref(va[e], a.exp_accurate);
        if (XT != MLLM_HIP_F32) s = bf16_to_f32(f32_to_bf16(s));
        o[e] = s * vb[e];
      }
      if (OP == EW_ADD) o[e] = va[e] + vb[e];
      if (OP == EW_MUL) o[e] = va[e] * vb[e];
    }
    item_store<XT>(a.y, it * 8, o);
  }
  if (a.img.base) quad_quantize_to_image(o, a.img, (int)row, col >> 2, col & 3, true);
}

// ---- softmax over the last axis, one wave per row ----------------------------------------------------------------------
// rows of at most 16 elements use expf like the reference's short-row branch (softmax.cpp:19-31); in longer rows the
// whole vectors of eight take the polynomial and the len % 8 tail elements expf (softmax.cpp:44-57)
__device__ __forceinline__ float softmax_exp(float x, bool poly) { return poly ? exp_poly(x) : expf(x); }

__global__ __launch_bounds__(256) void softmax_rows_kernel(const float* __restrict__ x, float* __restrict__ y, int64_t rows, int len,
                                                           int exp_accurate) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* xr = x + row * len;
  float* yr = y + row * len;
  const bool poly = len > 16 && !exp_accurate;
  float mx = -3.402823466e+38f;
  for (int i = lane; i < len; i += 64) mx = fmaxf(mx, xr[i]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int i = lane; i < len; i += 64) {
    const float e = softmax_exp(xr[i] - mx, poly && i < (len & ~7));
    yr[i] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  const float inv = 1.f / sum;
  for (int i = lane; i < len; i += 64) yr[i] *= inv;  // each lane re-reads what it wrote itself
}

// Rows of up to 64 NR elements: the lane keeps its elements (index lane + 64 j) in registers -- one pass over memory, every
// load requested before the first is used (the loops above are a load per iteration, three times over) -- and sums them in
// the same order: the same bits.  32 rows of 1024 (the attention of a decode token): 11.7 -> 3.6 us.
template <int NR>
__global__ __launch_bounds__(256) void softmax_rows_reg_kernel(const float* __restrict__ x, float* __restrict__ y, int64_t rows, int len,
                                                               int exp_accurate) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* xr = x + row * len;
  float* yr = y + row * len;
  const bool poly = len > 16 && !exp_accurate;
  float v[NR];
#pragma unroll
  for (int j = 0; j < NR; j++) v[j] = lane + 64 * j < len ? xr[lane + 64 * j] : -3.402823466e+38f;
  float mx = -3.402823466e+38f;
#pragma unroll
  for (int j = 0; j < NR; j++) mx = fmaxf(mx, v[j]);
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < NR; j++) {
    const int i = lane + 64 * j;
    if (i < len) {
      v[j] = softmax_exp(v[j] - mx, poly && i < (len & ~7));
      sum += v[j];
    }
  }
  sum = wave_sum(sum);
  const float inv = 1.f / sum;
#pragma unroll
  for (int j = 0; j < NR; j++)
    if (lane + 64 * j < len) yr[lane + 64 * j] = v[j] * inv;
}
// Long rows (a vocabulary): a workgroup of sixteen waves per row, three passes with eight loads in flight per thread; maxima
// and sums meet in LDS (per thread in index order, then the waves in order).  Eight rows of 151 936: 1993 -> about 60 us.
constexpr int SOFTMAX_WG = 1024;
__global__ __launch_bounds__(SOFTMAX_WG) void softmax_long_rows_kernel(const float* __restrict__ x, float* __restrict__ y, int len,
                                                                      int exp_accurate) {
  __shared__ float s_red[SOFTMAX_WG / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* xr = x + (int64_t)blockIdx.x * len;
  float* yr = y + (int64_t)blockIdx.x * len;
  const bool poly = !exp_accurate;
  constexpr int UB = 8;
  float mx = -3.402823466e+38f;
  for (int i0 = tid; i0 < len; i0 += SOFTMAX_WG * UB) {
    float v[UB];
#pragma unroll
    for (int u = 0; u < UB; u++) v[u] = i0 + SOFTMAX_WG * u < len ? xr[i0 + SOFTMAX_WG * u] : -3.402823466e+38f;
#pragma unroll
    for (int u = 0; u < UB; u++) mx = fmaxf(mx, v[u]);
  }
  mx = wave_max(mx);
  if (lane == 0) s_red[wave] = mx;
  __syncthreads();
  mx = s_red[0];
#pragma unroll
  for (int w = 1; w < SOFTMAX_WG / 64; w++) mx = fmaxf(mx, s_red[w]);
  __syncthreads();
  float sum = 0.f;
  for (int i0 = tid; i0 < len; i0 += SOFTMAX_WG * UB) {
    float v[UB];
#pragma unroll
    for (int u = 0; u < UB; u++) v[u] = i0 + SOFTMAX_WG * u < len ? xr[i0 + SOFTMAX_WG * u] : 0.f;
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int i = i0 + SOFTMAX_WG * u;
      if (i < len) {
        const float e = softmax_exp(v[u] - mx, poly && i < (len & ~7));
        yr[i] = e;
        sum += e;
      }
    }
  }
  sum = wave_sum(sum);
  if (lane == 0) s_red[wave] = sum;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < SOFTMAX_WG / 64; w++) total += s_red[w];
  const float inv = 1.f / total;
  for (int i0 = tid; i0 < len; i0 += SOFTMAX_WG * UB) {  // each thread re-reads what it wrote itself
    float v[UB];
#pragma unroll
    for (int u = 0; u < UB; u++) v[u] = i0 + SOFTMAX_WG * u < len ? yr[i0 + SOFTMAX_WG * u] : 0.f;
#pragma unroll
    for (int u = 0; u < UB; u++)
      if (i0 + SOFTMAX_WG * u < len) yr[i0 + SOFTMAX_WG * u] = v[u] * inv;
  }
}

// Rows between the two (2049 to 16 384 elements: the keys of an attention row): a workgroup of four waves per row, the row in
// registers (16, 32 or 64 elements per thread), one pass over memory; maxima and sums meet in LDS.
template <int R>
__global__ __launch_bounds__(256) void softmax_wg_rows_kernel(const float* __restrict__ x, float* __restrict__ y, int len, int exp_accurate) {
  __shared__ float s_red[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* xr = x + (int64_t)blockIdx.x * len;
  float* yr = y + (int64_t)blockIdx.x * len;
  const bool poly = !exp_accurate;
  float v[R];
#pragma unroll
  for (int j = 0; j < R; j++) v[j] = tid + 256 * j < len ? xr[tid + 256 * j] : -3.402823466e+38f;
  float mx = v[0];
#pragma unroll
  for (int j = 1; j < R; j++) mx = fmaxf(mx, v[j]);
  mx = wave_max(mx);
  if (lane == 0) s_red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
  __syncthreads();
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < R; j++) {
    const int i = tid + 256 * j;
    if (i < len) {
      v[j] = softmax_exp(v[j] - mx, poly && i < (len & ~7));
      sum += v[j];
    }
  }
  sum = wave_sum(sum);
  if (lane == 0) s_red[wave] = sum;
  __syncthreads();
  const float inv = 1.f / (((s_red[0] + s_red[1]) + s_red[2]) + s_red[3]);
#pragma unroll
  for (int j = 0; j < R; j++)
    if (tid + 256 * j < len) yr[tid + 256 * j] = v[j] * inv;
}

// ---- top-k over the last axis, one wave per row -------------------------------------------------------------------------
// Selection by repeated wave-wide extreme: round r takes the best element that comes after the one taken in round r-1
// in the order (value descending [ascending for smallest], index ascending).  Equal values are taken lowest index
// first (the reference's order among equal values is whatever its heap and std::sort leave).
struct KeyIdx {
  float v;
  int i;
};
__device__ __forceinline__ bool comes_before(float va, int ia, float vb, int ib, bool largest) {
  if (va != vb) return largest ? va > vb : va < vb;
  return ia < ib;
}
__device__ __forceinline__ KeyIdx wave_best(KeyIdx k, bool largest) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const float ov = __shfl_xor(k.v, off, 64);
    const int oi = __shfl_xor(k.i, off, 64);
    if (oi >= 0 && (k.i < 0 || comes_before(ov, oi, k.v, k.i, largest))) {
      k.v = ov;
      k.i = oi;
    }
  }
  return k;
}
// rows of `vals` may live in global memory or in LDS; out arrays are written by lane 0.  sorted == 0: by index.
__device__ __forceinline__ void wave_topk(const float* vals, int len, int k, bool largest, bool sorted, float* out_v, int* out_i,
                                          int lane) {
  float pv = 0.f;
  int pi = -1;  // previous pick
  for (int r = 0; r < k; r++) {
    KeyIdx best{0.f, -1};
    for (int i = lane; i < len; i += 64) {
      const float v = vals[i];
      const bool after_prev = pi < 0 || comes_before(pv, pi, v, i, largest);
      if (after_prev && (best.i < 0 || comes_before(v, i, best.v, best.i, largest))) {
        best.v = v;
        best.i = i;
      }
    }
    best = wave_best(best, largest);
    pv = best.v;
    pi = best.i;
    if (lane == 0) {
      out_v[r] = best.v;
      out_i[r] = best.i;
    }
  }
  if (!sorted && lane == 0) {  // by index: insertion sort of k entries
    for (int a = 1; a < k; a++) {
      const float v = out_v[a];
      const int i = out_i[a];
      int b = a - 1;
      while (b >= 0 && out_i[b] > i) {
        out_v[b + 1] = out_v[b];
        out_i[b + 1] = out_i[b];
        b--;
      }
      out_v[b + 1] = v;
      out_i[b + 1] = i;
    }
  }
}

// The same selection for a row of up to 64 R elements in LDS, by rank: a lane keeps its R elements (index lane + 64 j) and counts,
// over one pass of broadcast reads, how many elements of the row come before each of them in the order above; the elements
// of rank < k are the selection, rank = place by value, and the place by index is a count over ballots.  One pass instead of
// k rounds of wave-wide extremes (each six exchanges through the LDS pipe): the gate's 8 of 128 take a fifth of the time.
// (value, index) as one unsigned key, larger = earlier in that order: the float's bits made monotonic (-0 counts as +0, as it
// compares equal), inverted for "smallest first"; below it the inverted index, so that equal values go lowest index first
__device__ __forceinline__ unsigned long long order_key(float v, int i, bool largest) {
  uint32_t b = __float_as_uint(v + 0.f);
  b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  if (!largest) b = ~b;
  return ((unsigned long long)b << 32) | (uint32_t)~(uint32_t)i;
}
template <int R>
__device__ __forceinline__ void wave_topk_ranked(const float* vals, int len, int k, bool largest, bool sorted, float* out_v, int* out_i,
                                                 int lane) {
  float v[R];
  unsigned long long key[R];
  int rank[R];
#pragma unroll
  for (int j = 0; j < R; j++) {
    v[j] = lane + 64 * j < len ? vals[lane + 64 * j] : 0.f;
    key[j] = order_key(v[j], lane + 64 * j, largest);
    rank[j] = 0;
  }
#pragma unroll 8
  for (int o = 0; o < len; o++) {  // (eight reads in flight: one at a time, their latency is the whole cost)
    const unsigned long long ok = order_key(vals[o], o, largest);  // every lane the same address
#pragma unroll
    for (int j = 0; j < R; j++) rank[j] += ok > key[j] ? 1 : 0;
  }
  unsigned long long m[R];
#pragma unroll
  for (int j = 0; j < R; j++) m[j] = __ballot(lane + 64 * j < len && rank[j] < k);
  int before = 0;  // selected elements of the lower sixty-fours
#pragma unroll
  for (int j = 0; j < R; j++) {
    if (lane + 64 * j < len && rank[j] < k) {
      const int pos = sorted ? rank[j] : before + __popcll(m[j] & ((1ull << lane) - 1ull));
      out_v[pos] = v[j];
      out_i[pos] = lane + 64 * j;
    }
    before += __popcll(m[j]);
  }
}

__global__ __launch_bounds__(256) void topk_rows_kernel(const float* __restrict__ x, float* __restrict__ values, int32_t* __restrict__ indices,
                                                        int64_t rows, int len, int k, int largest, int sorted) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;  // (no workgroup barrier below)
  if (len <= 256) {  // short rows -- the experts of an MoE gate -- by rank in one pass over a copy of the row in LDS
    __shared__ float s_row[4][256];
    float* sr = s_row[threadIdx.x >> 6];
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = lane + 64 * j < len ? x[row * len + lane + 64 * j] : 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) sr[lane + 64 * j] = v[j];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (len <= 128) wave_topk_ranked<2>(sr, len, k, largest != 0, sorted != 0, values + row * k, indices + row * k, lane);
    else wave_topk_ranked<4>(sr, len, k, largest != 0, sorted != 0, values + row * k, indices + row * k, lane);
    return;
  }
  wave_topk(x + row * len, len, k, largest != 0, sorted != 0, values + row * k, indices + row * k, lane);
}

// Long rows (a vocabulary): a workgroup of sixteen waves per row runs the same k rounds, every thread scanning its share of
// the row with eight loads in flight, the waves' candidates meeting in LDS.  20 of 151 936: 11.3 ms with one wave -> 0.2 ms.
constexpr int TOPK_WG = 1024;
__global__ __launch_bounds__(TOPK_WG) void topk_long_rows_kernel(const float* __restrict__ x, float* __restrict__ values,
                                                                int32_t* __restrict__ indices, int len, int k, int largest, int sorted) {
  __shared__ float s_v[TOPK_WG / 64];
  __shared__ int s_i[TOPK_WG / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t row = blockIdx.x;
  const float* xr = x + row * len;
  float* out_v = values + row * k;
  int32_t* out_i = indices + row * k;
  const bool lg = largest != 0;
  float pv = 0.f;
  int pi = -1;  // previous pick
  constexpr int UB = 8;
  for (int r = 0; r < k; r++) {
    KeyIdx best{0.f, -1};
    for (int i0 = tid; i0 < len; i0 += TOPK_WG * UB) {
      float v[UB];
#pragma unroll
      for (int u = 0; u < UB; u++) v[u] = i0 + TOPK_WG * u < len ? xr[i0 + TOPK_WG * u] : 0.f;
#pragma unroll
      for (int u = 0; u < UB; u++) {
        const int i = i0 + TOPK_WG * u;
        if (i < len) {
          const bool after_prev = pi < 0 || comes_before(pv, pi, v[u], i, lg);
          if (after_prev && (best.i < 0 || comes_before(v[u], i, best.v, best.i, lg))) {
            best.v = v[u];
            best.i = i;
          }
        }
      }
    }
    best = wave_best(best, lg);
    if (lane == 0) {
      s_v[wave] = best.v;
      s_i[wave] = best.i;
    }
    __syncthreads();
    best = KeyIdx{s_v[0], s_i[0]};
#pragma unroll
    for (int w = 1; w < TOPK_WG / 64; w++) {
      const float ov = s_v[w];
      const int oi = s_i[w];
      if (oi >= 0 && (best.i < 0 || comes_before(ov, oi, best.v, best.i, lg))) best = KeyIdx{ov, oi};
    }
    __syncthreads();
    pv = best.v;
    pi = best.i;
    if (tid == 0) {
      out_v[r] = best.v;
      out_i[r] = best.i;
    }
  }
  if (!sorted && tid == 0) {  // by index: insertion sort of k entries (thread 0 wrote them itself)
    for (int a = 1; a < k; a++) {
      const float v = out_v[a];
      const int i = out_i[a];
      int b = a - 1;
      while (b >= 0 && out_i[b] > i) {
        out_v[b + 1] = out_v[b];
        out_i[b + 1] = out_i[b];
        b--;
      }
      out_v[b + 1] = v;
      out_i[b + 1] = i;
    }
  }
}

// Rows longer than 256 elements, k up to TOPK_SEL_MAX: radix select.  (value, index) pairs are ordered by order_key(); the
// key of the k-th pair is found a digit at a time (four bytes, or 12, 12 and 8 bits), highest first: a histogram of that digit
// over the elements that agree with the digits found so far (LDS counters; lanes of a wave that hold the same digit add once),
// then the bin in which the k-th falls.  These counting passes give the value's key; where more elements share that value
// than are still wanted, as many again over the inverted index choose the lowest indices among them.  Every pair at or above the k-th key is then collected
// in LDS and placed by its rank among the k.  The passes read the row again (eight 16-byte loads in flight per thread) or,
// for rows of up to eight such loads per thread, keep the keys in registers.  The cost does not depend on k.
constexpr int TOPK_SEL_MAX = 2048;
#ifndef TOPK_LEADERS
#define TOPK_LEADERS 2
#endif
template <int VEC> struct TopkVec;
template <> struct TopkVec<1> { typedef float T; };
template <> struct TopkVec<4> { typedef float4 T; };
template <int NT, int VEC, int R, bool WIDE>
__global__ __launch_bounds__(NT) void topk_select_rows_kernel(const float* __restrict__ x, float* __restrict__ values,
                                                              int32_t* __restrict__ indices, int len, int k, int largest, int sorted) {
  typedef typename TopkVec<VEC>::T VT;
  __shared__ unsigned s_hist[WIDE ? 4096 : 256];
  __shared__ unsigned s_pick[4];  // chosen digit, pairs still wanted inside its bin, the bin's count; [3]: pairs collected
  __shared__ unsigned long long s_sel[TOPK_SEL_MAX];
  const int tid = threadIdx.x, lane = tid & 63;
  const int64_t row = blockIdx.x;
  const float* xr = x + row * len;
  const bool lg = largest != 0;
  const int nunits = len / VEC;  // (VEC divides len)
  const bool inreg = nunits <= NT * R;
  uint32_t kreg[R][VEC];
  auto vkey = [&](float v) {
    uint32_t b = __float_as_uint(v + 0.f);
    b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return lg ? b : ~b;
  };
  auto load_keys = [&](int base, uint32_t (&kk)[R][VEC]) {
    VT v[R];
#pragma unroll
    for (int j = 0; j < R; j++) {
      const int u = base + tid + NT * j;
      if (u < nunits) v[j] = reinterpret_cast<const VT*>(xr)[u];
      else v[j] = VT{};
    }
#pragma unroll
    for (int j = 0; j < R; j++) {
      const float* f = reinterpret_cast<const float*>(&v[j]);
#pragma unroll
      for (int e = 0; e < VEC; e++) kk[j][e] = vkey(f[e]);
    }
  };
  if (inreg) load_keys(0, kreg);
  // f(key, index, valid) for every element of the row, by all lanes of every wave together (f holds wave-wide operations)
  auto scan = [&](auto&& f) {
    if (inreg) {
#pragma unroll
      for (int j = 0; j < R; j++) {
        const int u = tid + NT * j;
#pragma unroll
        for (int e = 0; e < VEC; e++) f(kreg[j][e], u * VEC + e, u < nunits);
      }
    } else {
      for (int base = 0; base < nunits; base += NT * R) {
        uint32_t kk[R][VEC];
        load_keys(base, kk);
#pragma unroll
        for (int j = 0; j < R; j++) {
          const int u = base + tid + NT * j;
#pragma unroll
          for (int e = 0; e < VEC; e++) f(kk[j][e], u * VEC + e, u < nunits);
        }
      }
    }
  };
  auto hist_add = [&](bool match, uint32_t digit) {
    unsigned long long m = __ballot(match);
    for (int it = 0; it < TOPK_LEADERS && m; it++) {  // (m is the same in every lane)
      const int leader = __ffsll((long long)m) - 1;
      const uint32_t d0 = (uint32_t)__builtin_amdgcn_readlane((int)digit, leader);
      const bool mine = match && digit == d0;
      const unsigned long long same = __ballot(mine);
      if (lane == leader) atomicAdd(&s_hist[d0], (unsigned)__popcll(same));
      match = match && !mine;
      m &= ~same;
    }
    if (match) atomicAdd(&s_hist[digit], 1u);
  };
  // the bin of the `need`-th largest digit among nb bins: wave 0, a lane per nb / 64 bins
  auto pick = [&](uint32_t need, int nb) {
    if (tid < 64) {
      const int per = nb >> 6, b0 = lane * per;
      uint32_t tot = 0;
      for (int q = 0; q < per; q++) tot += s_hist[b0 + ((q + lane) & (per - 1))];  // (the lanes on different banks)
      uint32_t incl = tot;  // this lane's bins and all higher ones
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const uint32_t o = (uint32_t)__shfl_down((int)incl, off, 64);
        if (lane + off < 64) incl += o;
      }
      uint32_t a = incl - tot;
      if (a < need && need <= incl) {
        for (int q = per - 1; q >= 0; q--) {
          const uint32_t c = s_hist[b0 + q];
          if (a + c >= need) {
            s_pick[0] = (uint32_t)(b0 + q);
            s_pick[1] = need - a;
            s_pick[2] = c;
            break;
          }
          a += c;
        }
      }
    }
  };
  // one counting pass over the digit of `bits` bits at `shift`: keyof(key, index, valid, &k32) says whether the element still
  // agrees with the digits found so far and gives the 32 bits the digit is taken from
  auto count_pass = [&](int shift, int bits, uint32_t need, auto&& keyof) {
    const int nb = 1 << bits;
    for (int b = tid; b < nb; b += NT) s_hist[b] = 0;
    __syncthreads();
    scan([&](uint32_t key, int idx, bool ok) {
      uint32_t k32;
      const bool mt = keyof(key, idx, ok, k32);
      hist_add(mt, (k32 >> shift) & (uint32_t)(nb - 1));
    });
    __syncthreads();
    pick(need, nb);
    __syncthreads();
  };
  // rows read again per pass: 12 + 12 + 8 bits (a pass over memory less); rows in registers: four bytes (256 counters to clear
  // and to walk per pass instead of 4096)
  constexpr int NPASS = WIDE ? 3 : 4;
  const int p_shift[4] = {WIDE ? 20 : 24, WIDE ? 8 : 16, WIDE ? 0 : 8, 0}, p_bits[4] = {WIDE ? 12 : 8, WIDE ? 12 : 8, 8, 8};
  uint32_t need = (uint32_t)k, t_val = 0, mask = 0, ties = 0;
  if (tid == 0) s_pick[3] = 0;
#pragma unroll
  for (int p = 0; p < NPASS; p++) {
    count_pass(p_shift[p], p_bits[p], need, [&](uint32_t key, int, bool ok, uint32_t& k32) {
      k32 = key;
      return ok && (key & mask) == t_val;
    });
    t_val |= s_pick[0] << p_shift[p];
    mask |= ((1u << p_bits[p]) - 1u) << p_shift[p];
    need = s_pick[1];
    ties = s_pick[2];
  }
  uint32_t t_idx = 0;  // pairs of the k-th value are taken down to this inverted index
  if (ties != need) {   // (the same in every thread)
    mask = 0;
#pragma unroll
    for (int p = 0; p < NPASS; p++) {
      count_pass(p_shift[p], p_bits[p], need, [&](uint32_t key, int idx, bool ok, uint32_t& k32) {
        k32 = ~(uint32_t)idx;
        return ok && key == t_val && (k32 & mask) == t_idx;
      });
      t_idx |= s_pick[0] << p_shift[p];
      mask |= ((1u << p_bits[p]) - 1u) << p_shift[p];
      need = s_pick[1];
    }
  }
  scan([&](uint32_t key, int idx, bool ok) {
    const uint32_t ni = ~(uint32_t)idx;
    if (ok && (key > t_val || (key == t_val && ni >= t_idx))) {
      const unsigned pos = atomicAdd(&s_pick[3], 1u);
      if (pos < (unsigned)TOPK_SEL_MAX) s_sel[pos] = ((unsigned long long)key << 32) | ni;
    }
  });
  __syncthreads();
  const bool by_value = sorted != 0;
  for (int t = tid; t < k; t += NT) {
    const unsigned long long my = s_sel[t];
    const unsigned long long mc = by_value ? my : (my << 32);  // by index: the inverted index alone, larger = earlier
    int rank = 0;
    for (int j = 0; j < k; j++) {
      const unsigned long long o = s_sel[j];
      rank += (by_value ? o : (o << 32)) > mc ? 1 : 0;
    }
    const int idx = (int)~(uint32_t)my;
    values[row * k + rank] = xr[idx];
    indices[row * k + rank] = idx;
  }
}

// ---- MoE gate: logits = x . W^T (fp32), softmax, top-k, optional normalisation ------------------------------------------
// A workgroup of sixteen waves takes four tokens: the tokens' activations sit in LDS, every wave walks a sixteenth of the
// experts (16-byte loads along H, the tokens share each weight load), then wave t finishes token t.
// A lane requests eight pieces of an expert's row before it multiplies the first (a row of 2048 elements is one such batch,
// a round trip to memory per expert instead of one per piece), and only the workgroup's real tokens are multiplied.  One
// decode token of a 128-expert layer (1 MB of gate weights through one workgroup): 109 us with four waves and a load per
// iteration, an order of magnitude less this way; the sums run in the same order per lane (same logits bit for bit).
struct GateArgs {
  const void* x;
  const float* w;  // [E, H]
  int32_t* ids;    // [M, k]
  float* weights;  // [M, k]
  float* scores;   // [M, E] or null
  int64_t M;
  int H, E, k, norm, exp_accurate;
};
constexpr int GATE_TOK = 4;
constexpr int GATE_WAVES = 16;
// x of the workgroup's ntok tokens -> fp32 in LDS
template <int XT>
__device__ __forceinline__ void gate_stage_x(const GateArgs& a, int64_t tok0, int ntok, float* s_x, int tid, int nthreads) {
  const int ipr = a.H >> 3, nitems = ntok * ipr;
  for (int it = tid; it < nitems; it += nthreads) {  // (four tokens of 2048 elements, 1024 threads: one item per thread)
    const int t = it / ipr, c = it - t * ipr;
    float v[8];
    Item8<XT> r;
    item_load<XT>(a.x, (tok0 + t) * a.H + (int64_t)c * 8, r);
    item_to_f32<XT>(r, v);
    f32x4* dst = reinterpret_cast<f32x4*>(s_x + (size_t)t * a.H + c * 8);
    dst[0] = f32x4{v[0], v[1], v[2], v[3]};
    dst[1] = f32x4{v[4], v[5], v[6], v[7]};
  }
}
// logits of experts e0 + wave, e0 + wave + nwaves, ... < e1 for the ntok tokens in s_x; out[t * ostride + e]
__device__ __forceinline__ void gate_logits(const GateArgs& a, const float* s_x, int ntok, int e0, int e1, int wave, int nwaves, int lane,
                                            float* out, size_t ostride) {
  constexpr int CB = 8;  // pieces of a row a lane requests before it multiplies the first
  const int nc = a.H >> 2;
  for (int e = e0 + wave; e < e1; e += nwaves) {
    float acc[GATE_TOK] = {0.f, 0.f, 0.f, 0.f};
    const f32x4* wr = reinterpret_cast<const f32x4*>(a.w + (size_t)e * a.H);
    for (int c0 = lane; c0 < nc; c0 += 64 * CB) {
      f32x4 wv[CB];
#pragma unroll
      for (int u = 0; u < CB; u++)
        if (c0 + 64 * u < nc) wv[u] = wr[c0 + 64 * u];
#pragma unroll
      for (int u = 0; u < CB; u++) {
        const int c = c0 + 64 * u;
        if (c < nc) {
#pragma unroll
          for (int t = 0; t < GATE_TOK; t++) {
            if (t < ntok) {  // uniform
              const f32x4 xv = reinterpret_cast<const f32x4*>(s_x + (size_t)t * a.H)[c];
              acc[t] = fmaf(xv.x, wv[u].x, acc[t]);
              acc[t] = fmaf(xv.y, wv[u].y, acc[t]);
              acc[t] = fmaf(xv.z, wv[u].z, acc[t]);
              acc[t] = fmaf(xv.w, wv[u].w, acc[t]);
            }
          }
        }
      }
    }
#pragma unroll
    for (int t = 0; t < GATE_TOK; t++) {
      if (t < ntok) {
        const float s = wave_sum(acc[t]);
        if (lane == 0) out[t * ostride + e] = s;
      }
    }
  }
}
// one wave finishes one token: softmax over its E logits in lg (LDS, overwritten), the k largest in index order, weights
__device__ __forceinline__ void gate_select(const GateArgs& a, float* lg, int64_t tok, float* tv, int* ti, int lane) {
  const bool poly = a.E > 16 && !a.exp_accurate;
  float mx = -3.402823466e+38f;
  for (int i = lane; i < a.E; i += 64) mx = fmaxf(mx, lg[i]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int i = lane; i < a.E; i += 64) {
    const float ex = softmax_exp(lg[i] - mx, poly && i < (a.E & ~7));
    lg[i] = ex;
    sum += ex;
  }
  sum = wave_sum(sum);
  const float inv = 1.f / sum;
  for (int i = lane; i < a.E; i += 64) {
    const float p = lg[i] * inv;
    lg[i] = p;
    if (a.scores) a.scores[tok * a.E + i] = p;
  }
  // LDS writes of this wave are read back by other lanes of the same wave only
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  if (a.E <= 128) wave_topk_ranked<2>(lg, a.E, a.k, true, false, tv, ti, lane);
  else if (a.E <= 256) wave_topk_ranked<4>(lg, a.E, a.k, true, false, tv, ti, lane);
  else wave_topk(lg, a.E, a.k, true, false, tv, ti, lane);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  // topk(..., largest = true, sorted = false): by index; then weight / sum(weights) in index order
  float tsum = 0.f;
  for (int r = 0; r < a.k; r++) tsum += tv[r];
  for (int r = lane; r < a.k; r += 64) {
    const float wv = tv[r];
    a.weights[tok * a.k + r] = a.norm ? wv / tsum : wv;
    a.ids[tok * a.k + r] = ti[r];
  }
}
// everything in one launch: a workgroup per four tokens (callers that pass no scores buffer)
template <int XT>
__global__ __launch_bounds__(GATE_WAVES * 64) void moe_gate_kernel(GateArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_x = reinterpret_cast<float*>(smem);     // [GATE_TOK][H]
  float* s_logit = s_x + (size_t)GATE_TOK * a.H;   // [GATE_TOK][E]
  float* s_tv = s_logit + (size_t)GATE_TOK * a.E;  // [GATE_TOK][k]
  int* s_ti = reinterpret_cast<int*>(s_tv + (size_t)GATE_TOK * a.k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t tok0 = (int64_t)blockIdx.x * GATE_TOK;
  const int ntok = (int)min((int64_t)GATE_TOK, a.M - tok0);  // uniform
  gate_stage_x<XT>(a, tok0, ntok, s_x, tid, GATE_WAVES * 64);
  __syncthreads();
  gate_logits(a, s_x, ntok, 0, a.E, wave, GATE_WAVES, lane, s_logit, (size_t)a.E);
  __syncthreads();
  if (wave >= ntok) return;
  gate_select(a, s_logit + wave * a.E, tok0 + wave, s_tv + wave * a.k, s_ti + wave * a.k, lane);
}
// The same in two launches for callers that pass a scores buffer, which holds the logits in between: with few tokens one
// workgroup per four tokens leaves the chip to one CU (a decode token: 1 MB of gate weights through one workgroup), so the
// experts are spread over the grid's y -- epg experts and as many waves per workgroup -- and a second, small launch
// finishes each token.  Same logits, same selection.
template <int XT>
__global__ __launch_bounds__(GATE_WAVES * 64) void moe_gate_logits_kernel(GateArgs a, int epg) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_x = reinterpret_cast<float*>(smem);  // [GATE_TOK][H]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x;
  const int64_t tok0 = (int64_t)blockIdx.x * GATE_TOK;
  const int ntok = (int)min((int64_t)GATE_TOK, a.M - tok0);  // uniform
  gate_stage_x<XT>(a, tok0, ntok, s_x, tid, nthreads);
  __syncthreads();
  const int e0 = (int)blockIdx.y * epg;
  gate_logits(a, s_x, ntok, e0, min(a.E, e0 + epg), wave, nthreads >> 6, lane, a.scores + tok0 * a.E, (size_t)a.E);
}
__global__ __launch_bounds__(GATE_TOK * 64) void moe_gate_select_kernel(GateArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_logit = reinterpret_cast<float*>(smem);  // [GATE_TOK][E]
  float* s_tv = s_logit + (size_t)GATE_TOK * a.E;   // [GATE_TOK][k]
  int* s_ti = reinterpret_cast<int*>(s_tv + (size_t)GATE_TOK * a.k);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t tok = (int64_t)blockIdx.x * GATE_TOK + wave;
  if (tok >= a.M) return;  // (no workgroup barrier below)
  float* lg = s_logit + wave * a.E;
  for (int i = lane; i < a.E; i += 64) lg[i] = a.scores[tok * a.E + i];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  gate_select(a, lg, tok, s_tv + wave * a.k, s_ti + wave * a.k, lane);
}

}  // namespace mllmhip

using namespace mllmhip;

static int g_exp_accurate = 0;
namespace mllmhip {
int exp_mode_accurate() { return g_exp_accurate; }
}
MLLM_API int mllm_hip_set_exp_mode(int accurate) {
  if (accurate != 0 && accurate != 1) return MLLM_HIP_E_BADARG;
  g_exp_accurate = accurate;
  return 0;
}

static bool dtype_ok(int t) { return t == MLLM_HIP_F32 || t == MLLM_HIP_BF16; }
static bool al16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// image argument checks shared by the producers: rows <= 8, D a multiple of 32
static int make_image(void* q_image, int64_t rows, int64_t D, int act_scale_mode, QImage& q) {
  q = QImage{nullptr, 0, 0, 0};
  if (!q_image) return 0;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (rows < 1 || rows > 8 || D % QK) return MLLM_HIP_E_SHAPE;
  if (!al16(q_image)) return MLLM_HIP_E_ALIGN;
  q.base = reinterpret_cast<unsigned char*>(q_image);
  q.MT = rows <= 1 ? 1 : (rows <= 2 ? 2 : (rows <= 4 ? 4 : 8));
  q.nb = (int)(D / QK);
  q.x86_scale = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  return 0;
}

MLLM_API int mllm_hip_rmsnorm(const void* x, int dtype, const float* weight, void* y, int64_t rows, int64_t D, float epsilon,
                              int add_unit_offset, void* q_image, int act_scale_mode, void* stream) {
  if (!x || !weight || !y || !dtype_ok(dtype) || rows <= 0 || D <= 0) return MLLM_HIP_E_BADARG;
  if (D % 8 || D > 8 * 256 * 8 || rows > 0x7fffffff) return MLLM_HIP_E_SHAPE;
  if (!al16(x) || !al16(y) || !al16(weight)) return MLLM_HIP_E_ALIGN;
  RmsArgs a{x, weight, y, rows, (int)D, epsilon, add_unit_offset, {}};
  int rc = make_image(q_image, rows, D, act_scale_mode, a.img);
  if (rc) return rc;
  const unsigned grid = (unsigned)(a.img.base ? a.img.MT : rows);
  const int ni = (int)((D / 8 + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
#define RMS(XT_, NI_) hipLaunchKernelGGL((rmsnorm_kernel<XT_, NI_>), dim3(grid), dim3(256), 0, st, a)
#define RMS_T(XT_)        \
  if (ni <= 1) RMS(XT_, 1); \
  else if (ni <= 2) RMS(XT_, 2); \
  else if (ni <= 4) RMS(XT_, 4); \
  else RMS(XT_, 8)
  if (dtype == MLLM_HIP_F32) {
    RMS_T(MLLM_HIP_F32);
  } else {
    RMS_T(MLLM_HIP_BF16);
  }
#undef RMS_T
#undef RMS
  return (int)hipGetLastError();
}

template <int OP>
static int launch_elementwise(const void* a_, const void* b_, void* y, int dtype, int64_t rows, int64_t D, void* q_image,
                              int act_scale_mode, void* stream) {
  if (!a_ || (OP != EW_SILU && !b_) || !y || !dtype_ok(dtype) || rows <= 0 || D <= 0) return MLLM_HIP_E_BADARG;
  if (D % 8 || D > 0x7fffffff) return MLLM_HIP_E_SHAPE;
  if (!al16(a_) || !al16(b_) || !al16(y)) return MLLM_HIP_E_ALIGN;
  EwArgs a{a_, b_, y, rows, (int)D, g_exp_accurate, {}};
  int rc = make_image(q_image, rows, D, act_scale_mode, a.img);
  if (rc) return rc;
  const int64_t total_rows = a.img.base ? a.img.MT : rows;
  const int64_t items = total_rows * (D / 8);
  if ((items + 255) / 256 > 0x7fffffff) return MLLM_HIP_E_SHAPE;
  const unsigned grid = (unsigned)((items + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MLLM_HIP_F32)
    hipLaunchKernelGGL((elementwise_kernel<MLLM_HIP_F32, OP>), dim3(grid), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((elementwise_kernel<MLLM_HIP_BF16, OP>), dim3(grid), dim3(256), 0, st, a);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_silu(const void* x, void* y, int dtype, int64_t n, void* stream) {
  if (n <= 0 || n % 8) return n <= 0 ? MLLM_HIP_E_BADARG : MLLM_HIP_E_SHAPE;
  return launch_elementwise<EW_SILU>(x, nullptr, y, dtype, n / 8, 8, nullptr, 0, stream);
}
MLLM_API int mllm_hip_add(const void* a, const void* b, void* y, int dtype, int64_t rows, int64_t D, void* q_image,
                          int act_scale_mode, void* stream) {
  return launch_elementwise<EW_ADD>(a, b, y, dtype, rows, D, q_image, act_scale_mode, stream);
}
MLLM_API int mllm_hip_mul(const void* a, const void* b, void* y, int dtype, int64_t rows, int64_t D, void* q_image,
                          int act_scale_mode, void* stream) {
  return launch_elementwise<EW_MUL>(a, b, y, dtype, rows, D, q_image, act_scale_mode, stream);
}
MLLM_API int mllm_hip_silu_mul(const void* gate, const void* up, void* y, int dtype, int64_t rows, int64_t D, void* q_image,
                               int act_scale_mode, void* stream) {
  return launch_elementwise<EW_SILU_MUL>(gate, up, y, dtype, rows, D, q_image, act_scale_mode, stream);
}

MLLM_API int mllm_hip_softmax(const float* x, float* y, int64_t rows, int64_t len, void* stream) {
  if (!x || !y || rows <= 0 || len <= 0) return MLLM_HIP_E_BADARG;
  if (len > 0x7fffffff || (rows + 3) / 4 > 0x7fffffff) return MLLM_HIP_E_SHAPE;
  const dim3 grid4((unsigned)((rows + 3) / 4));
  hipStream_t st = (hipStream_t)stream;
  if (len <= 256) hipLaunchKernelGGL(softmax_rows_reg_kernel<4>, grid4, dim3(256), 0, st, x, y, rows, (int)len, g_exp_accurate);
  else if (len <= 1024) hipLaunchKernelGGL(softmax_rows_reg_kernel<16>, grid4, dim3(256), 0, st, x, y, rows, (int)len, g_exp_accurate);
  else if (len <= 2048) hipLaunchKernelGGL(softmax_rows_reg_kernel<32>, grid4, dim3(256), 0, st, x, y, rows, (int)len, g_exp_accurate);
  else if (len <= 4096 && rows <= 0x7fffffff) hipLaunchKernelGGL(softmax_wg_rows_kernel<16>, dim3((unsigned)rows), dim3(256), 0, st, x, y, (int)len, g_exp_accurate);
  else if (len <= 8192 && rows <= 0x7fffffff) hipLaunchKernelGGL(softmax_wg_rows_kernel<32>, dim3((unsigned)rows), dim3(256), 0, st, x, y, (int)len, g_exp_accurate);
  else if (len <= 16384 && rows <= 0x7fffffff) hipLaunchKernelGGL(softmax_wg_rows_kernel<64>, dim3((unsigned)rows), dim3(256), 0, st, x, y, (int)len, g_exp_accurate);
  else if (len >= 16384 && rows <= 0x7fffffff) hipLaunchKernelGGL(softmax_long_rows_kernel, dim3((unsigned)rows), dim3(SOFTMAX_WG), 0, st, x, y, (int)len, g_exp_accurate);
  else hipLaunchKernelGGL(softmax_rows_kernel, grid4, dim3(256), 0, st, x, y, rows, (int)len, g_exp_accurate);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_topk(const float* x, float* values, int32_t* indices, int64_t rows, int64_t len, int k, int largest,
                           int sorted, void* stream) {
  if (!x || !values || !indices || rows <= 0 || len <= 0) return MLLM_HIP_E_BADARG;
  if (k < 1 || k > len || len > 0x7fffffff || (rows + 3) / 4 > 0x7fffffff) return MLLM_HIP_E_SHAPE;
  if (len > 256 && k <= TOPK_SEL_MAX && rows <= 0x7fffffff) {
    const bool vec = len % 4 == 0 && ((uintptr_t)x & 15) == 0;
    const int64_t units = vec ? len / 4 : len;
    const dim3 grid((unsigned)rows);
    hipStream_t st = (hipStream_t)stream;
#define TOPK_SELECT(NT, R, WIDE) \
  do { \
    if (vec) hipLaunchKernelGGL((topk_select_rows_kernel<NT, 4, R, WIDE>), grid, dim3(NT), 0, st, x, values, indices, (int)len, k, largest, sorted); \
    else hipLaunchKernelGGL((topk_select_rows_kernel<NT, 1, R, WIDE>), grid, dim3(NT), 0, st, x, values, indices, (int)len, k, largest, sorted); \
  } while (0)
    if (units <= 256) TOPK_SELECT(256, 1, false);  // (loads per thread that hold the row: no empty slots to step over)
    else if (units <= 512) TOPK_SELECT(256, 2, false);
    else if (units <= 1024) TOPK_SELECT(256, 4, false);
    else if (units <= 2048) TOPK_SELECT(256, 8, false);
    else if (units <= 4096) TOPK_SELECT(1024, 4, false);
    else if (units <= 8192) TOPK_SELECT(1024, 8, false);
    else TOPK_SELECT(1024, 8, true);
#undef TOPK_SELECT
  } else if (len >= 8192 && rows <= 0x7fffffff)
    hipLaunchKernelGGL(topk_long_rows_kernel, dim3((unsigned)rows), dim3(TOPK_WG), 0, (hipStream_t)stream, x, values, indices, (int)len, k,
                       largest, sorted);
  else
    hipLaunchKernelGGL(topk_rows_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream, x, values, indices, rows,
                       (int)len, k, largest, sorted);
  return (int)hipGetLastError();
}

static int g_gate_two_launches = 1;  // 0: the one-launch form also where a scores buffer is given (comparison runs and tests)
MLLM_API int mllm_hip_moe_gate_set_form(int two_launches) {
  if (two_launches != 0 && two_launches != 1) return MLLM_HIP_E_BADARG;
  g_gate_two_launches = two_launches;
  return 0;
}

MLLM_API int mllm_hip_moe_gate(const void* x, int x_dtype, const float* gate_weight, int32_t* topk_ids, float* topk_weights,
                               float* scores, int64_t M, int64_t H, int64_t E, int k, int norm_topk_prob, void* stream) {
  if (!x || !gate_weight || !topk_ids || !topk_weights || !dtype_ok(x_dtype) || M <= 0 || H <= 0 || E <= 0) return MLLM_HIP_E_BADARG;
  if (k < 1 || k > E || H % 8 || (M + GATE_TOK - 1) / GATE_TOK > 0x7fffffff) return MLLM_HIP_E_SHAPE;
  if (!al16(x) || !al16(gate_weight)) return MLLM_HIP_E_ALIGN;
  const size_t lds = ((size_t)GATE_TOK * H + (size_t)GATE_TOK * E + (size_t)2 * GATE_TOK * k) * 4;
  if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
  GateArgs a{x, gate_weight, topk_ids, topk_weights, scores, M, (int)H, (int)E, k, norm_topk_prob, g_exp_accurate};
  const unsigned grid = (unsigned)((M + GATE_TOK - 1) / GATE_TOK);
  hipStream_t st = (hipStream_t)stream;
  if (scores && g_gate_two_launches) {
    // experts per workgroup: four (one per wave) while the token groups alone do not fill the chip, else sixteen
    const int epg = grid >= 64 ? 16 : 4;
    const size_t lds1 = (size_t)GATE_TOK * H * 4, lds2 = ((size_t)GATE_TOK * E + (size_t)2 * GATE_TOK * k) * 4;
    auto go = [&](auto kern) -> int {
      if (lds1 > 64 * 1024)
        HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds1));
      hipLaunchKernelGGL(kern, dim3(grid, (unsigned)((E + epg - 1) / epg)), dim3(64 * epg), lds1, st, a, epg);
      return (int)hipGetLastError();
    };
    RC_RET(x_dtype == MLLM_HIP_F32 ? go(moe_gate_logits_kernel<MLLM_HIP_F32>) : go(moe_gate_logits_kernel<MLLM_HIP_BF16>));
    if (lds2 > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(moe_gate_select_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds2));
    hipLaunchKernelGGL(moe_gate_select_kernel, dim3(grid), dim3(GATE_TOK * 64), lds2, st, a);
    return (int)hipGetLastError();
  }
  auto launch = [&](auto kern) -> int {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GATE_WAVES * 64), lds, st, a);
    return (int)hipGetLastError();
  };
  return x_dtype == MLLM_HIP_F32 ? launch(moe_gate_kernel<MLLM_HIP_F32>) : launch(moe_gate_kernel<MLLM_HIP_BF16>);
}
