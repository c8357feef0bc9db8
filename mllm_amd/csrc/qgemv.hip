// Q4_0 / Q8_0 Linear for decode (M = 1..8) on gfx950: weight pre-pack, fused Q8_0 activation quantization + block-dot
// GEMV, and the parity probes.  HBM-bound: every weight byte is read once with 16-byte fully coalesced loads.
//
// Arithmetic follows the reference's x86 CPU path:
//   activation quantization  mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.cpp:106-190
//   block dot + scaling       mllm/backends/cpu/kernels/common/llamafile/llamafile_sgemm.cpp:697-743
//   flow                      mllm/backends/cpu/kernels/common/ggml/matmul.cpp:148-206
// The int32 block sums are exact; the fp32 accumulation order differs from the CPU's 8-lane order (tolerance 1e-3 rel-L2).
#include "qcommon.h"

#include <string.h>

#include <initializer_list>

namespace mllmhip {

// =========================================================================================================
// pre-pack: reference blocks (AoS) -> code planes + scale array
// =========================================================================================================
__global__ void prepack_kernel(int wtype, const uint8_t* __restrict__ blocks, int x86_scale, u32x4* __restrict__ q0,
                               u32x4* __restrict__ q1, uint16_t* __restrict__ d, int64_t nblocks) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  const int bb = wtype == MLLM_HIP_Q4_0 ? 18 : 34;
  const uint8_t* b = blocks + i * bb;
  uint16_t raw = (uint16_t)b[0] | ((uint16_t)b[1] << 8);
  uint16_t bits = raw;
  if (x86_scale) {
    // the field holds the pattern as a half-precision NUMBER: number -> integer gives the pattern that is looked up
    float num = f16bits_to_f32(raw);
    bits = (num >= 0.f && num < 65536.f) ? (uint16_t)(uint32_t)num : (uint16_t)0;
  }
  d[i] = bits;
  uint32_t w[8];
  const int nw = wtype == MLLM_HIP_Q4_0 ? 4 : 8;
  for (int j = 0; j < nw; j++) {
    const uint8_t* p = b + 2 + 4 * j;  // blocks are only 2-byte aligned: assemble from bytes
    w[j] = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
  }
  q0[i] = u32x4{w[0], w[1], w[2], w[3]};
  if (wtype == MLLM_HIP_Q8_0) q1[i] = u32x4{w[4], w[5], w[6], w[7]};
}

// =========================================================================================================
// GEMV
// =========================================================================================================
struct GemvArgs {
  PackedView w;
  const void* x;
  const float* bias;
  float* y;
  int x_dtype;
  int M;          // actual rows of x (<= MT)
  int N;
  int nb;         // K / 32
  int x86_scale;  // reproduce the x86 storage rounding of the activation scale
};

// exact int32 dot product of one weight block with one quantized activation block
template <int WT>
__device__ __forceinline__ int block_dot(const u32x4& w0, const u32x4& w1, const u32x4& xlo, const u32x4& xhi, int neg8sum) {
  if (WT == MLLM_HIP_Q4_0) {
    // dword j of the block: low nibbles = elements 4j..4j+3, high nibbles = elements 16+4j..16+4j+3.
    // nibbles stay unsigned (0..15); the -8 offset is folded in as -8 * sum(x codes), precomputed per activation block.
    const uint32_t m = 0x0f0f0f0fu;
    int acc = neg8sum;
    acc = __builtin_amdgcn_sdot4((int)(w0.x & m), (int)xlo.x, acc, false);
    acc = __builtin_amdgcn_sdot4((int)(w0.y & m), (int)xlo.y, acc, false);
    acc = __builtin_amdgcn_sdot4((int)(w0.z & m), (int)xlo.z, acc, false);
    acc = __builtin_amdgcn_sdot4((int)(w0.w & m), (int)xlo.w, acc, false);
    acc = __builtin_amdgcn_sdot4((int)((w0.x >> 4) & m), (int)xhi.x, acc, false);
    acc = __builtin_amdgcn_sdot4((int)((w0.y >> 4) & m), (int)xhi.y, acc, false);
    acc = __builtin_amdgcn_sdot4((int)((w0.z >> 4) & m), (int)xhi.z, acc, false);
    acc = __builtin_amdgcn_sdot4((int)((w0.w >> 4) & m), (int)xhi.w, acc, false);
    return acc;
  } else {
    int acc = 0;
    acc = __builtin_amdgcn_sdot4((int)w0.x, (int)xlo.x, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w0.y, (int)xlo.y, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w0.z, (int)xlo.z, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w0.w, (int)xlo.w, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w1.x, (int)xhi.x, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w1.y, (int)xhi.y, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w1.z, (int)xhi.z, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w1.w, (int)xhi.w, acc, false);
    return acc;
  }
}

// One loop trip's worth of weight data of a lane: U block columns x R rows.
template <int WT, int R, int U>
struct WChunk {
  u32x4 w0[U][R];
  u32x4 w1[WT == MLLM_HIP_Q8_0 ? U : 1][R];
  uint16_t dw[U][R];
};

template <int WT, int G, int R, int U>
__device__ __forceinline__ void load_chunk(WChunk<WT, R, U>& c, const PackedView& w, const int64_t (&rbase)[R], int t0,
                                           int c0, int nb) {
#pragma unroll
  for (int u = 0; u < U; u++) {
    const int col = t0 + u * G + c0;
#pragma unroll
    for (int r = 0; r < R; r++) {
      c.w0[u][r] = u32x4{0, 0, 0, 0};
      if (WT == MLLM_HIP_Q8_0) c.w1[u][r] = u32x4{0, 0, 0, 0};
      c.dw[u][r] = 0;
      if (col < nb) {  // lanes past the end of the row issue nothing
        c.w0[u][r] = __builtin_nontemporal_load(&w.q0[rbase[r] + col]);
        if (WT == MLLM_HIP_Q8_0) c.w1[u][r] = __builtin_nontemporal_load(&w.q1[rbase[r] + col]);
        c.dw[u][r] = __builtin_nontemporal_load(&w.d[rbase[r] + col]);
      }
    }
  }
}

// Workgroup = NW waves.  Each wave is cut into 64/G groups of G lanes; a group owns R consecutive weight rows and its
// lanes stride over the row's blocks (lane c takes blocks c, c+G, ...), so one load instruction of a group reads G*16
// contiguous bytes.  All of x is quantized once per workgroup into LDS (codes in two 16-byte planes so that neighbouring
// lanes read neighbouring 16-byte words, plus the fp32 scale and -8*sum(codes) per block).
// U = how many block columns a lane keeps in flight per loop trip.  The first trip's weight loads are issued before the
// activation quantization so that HBM latency overlaps it; later trips are double-buffered.
template <int WT, int MT, int G, int R, int U>
__global__ __launch_bounds__(256) void gemv_q_kernel(GemvArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int nb = a.nb;
  const int mnb = MT * nb;
  u32x4* s_lo = reinterpret_cast<u32x4*>(smem);
  u32x4* s_hi = s_lo + mnb;
  float* s_d = reinterpret_cast<float*>(s_hi + mnb);
  int* s_n8 = reinterpret_cast<int*>(s_d + mnb);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int nwaves = blockDim.x >> 6;
  constexpr int GROUPS = 64 / G;
  const int grp = lane / G;
  const int c0 = lane % G;
  const int64_t row0 = ((int64_t)blockIdx.x * nwaves + wave) * (GROUPS * R) + (int64_t)grp * R;

  // rows past N are clamped for the loads and dropped at the store
  int64_t rbase[R];
#pragma unroll
  for (int r = 0; r < R; r++) rbase[r] = min(row0 + r, (int64_t)a.N - 1) * nb;

  WChunk<WT, R, U> cur;
  load_chunk<WT, G, R, U>(cur, a.w, rbase, 0, c0, nb);

  // ---- activation quantization into LDS (rows m >= M are zero-filled so the unrolled MT loop is harmless) ----
  for (int id = tid; id < mnb; id += blockDim.x) {
    const int m = id / nb, b = id - m * nb;
    uint32_t q[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    float dx = 0.f;
    int sum = 0;
    if (m < a.M) {
      float v[32];
      load_block_f32(a.x, a.x_dtype, (int64_t)m * nb * QK + (int64_t)b * QK, v);
      uint16_t bits = quantize_block_q8_0(v, q, sum);
      if (a.x86_scale) bits = x86_scale_bits(bits);
      dx = f16bits_to_f32(bits);
    }
    s_lo[id] = u32x4{q[0], q[1], q[2], q[3]};
    s_hi[id] = u32x4{q[4], q[5], q[6], q[7]};
    s_d[id] = dx;
    s_n8[id] = -8 * sum;
  }
  __syncthreads();

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < MT; m++) acc[r][m] = 0.f;

  for (int t0 = 0; t0 < nb; t0 += G * U) {
    WChunk<WT, R, U> nxt;
    const bool more = t0 + G * U < nb;  // uniform
    if (more) load_chunk<WT, G, R, U>(nxt, a.w, rbase, t0 + G * U, c0, nb);
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = t0 + u * G + c0;
      if (col < nb) {
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const u32x4 xlo = s_lo[m * nb + col];
          const u32x4 xhi = s_hi[m * nb + col];
          const float dx = s_d[m * nb + col];
          const int n8 = s_n8[m * nb + col];
#pragma unroll
          for (int r = 0; r < R; r++) {
            const int isum = block_dot<WT>(cur.w0[u][r], cur.w1[WT == MLLM_HIP_Q8_0 ? u : 0][r], xlo, xhi, n8);
            const float d = f16bits_to_f32(cur.dw[u][r]) * dx;
            acc[r][m] = fmaf(d, (float)isum, acc[r][m]);
          }
        }
      }
    }
    if (more) cur = nxt;
  }

#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < MT; m++) {
      float v = group_sum<G>(acc[r][m]);
      const int64_t row = row0 + r;
      if (c0 == 0 && row < a.N && m < a.M) a.y[(int64_t)m * a.N + row] = a.bias ? a.bias[row] + v : v;
    }
}

// =========================================================================================================
// stand-alone activation quantization, probes
// =========================================================================================================
__global__ void quantize_q8_0_kernel(const void* __restrict__ x, int x_dtype, int8_t* __restrict__ codes,
                                     uint16_t* __restrict__ d_bits, int64_t nblocks) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  float v[32];
  uint32_t q[8];
  int sum;
  load_block_f32(x, x_dtype, i * QK, v);
  d_bits[i] = quantize_block_q8_0(v, q, sum);
  u32x4* out = reinterpret_cast<u32x4*>(codes + i * QK);
  out[0] = u32x4{q[0], q[1], q[2], q[3]};
  out[1] = u32x4{q[4], q[5], q[6], q[7]};
}

__global__ void dequantize_kernel(int wtype, PackedView w, float* __restrict__ out, int64_t nblocks) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  const float d = f16bits_to_f32(w.d[i]);
  const u32x4 a = w.q0[i];
  const uint32_t aw[4] = {a.x, a.y, a.z, a.w};
  float* o = out + i * QK;
  if (wtype == MLLM_HIP_Q4_0) {
    for (int j = 0; j < 16; j++) {
      const uint32_t byte = (aw[j >> 2] >> (8 * (j & 3))) & 0xffu;
      o[j] = (float)((int)(byte & 15u) - 8) * d;
      o[j + 16] = (float)((int)(byte >> 4) - 8) * d;
    }
  } else {
    const u32x4 b = w.q1[i];
    const uint32_t bw[4] = {b.x, b.y, b.z, b.w};
    for (int j = 0; j < 16; j++) {
      o[j] = (float)(int8_t)((aw[j >> 2] >> (8 * (j & 3))) & 0xffu) * d;
      o[j + 16] = (float)(int8_t)((bw[j >> 2] >> (8 * (j & 3))) & 0xffu) * d;
    }
  }
}

// one thread per (n, m, b)
__global__ void block_isums_kernel(int wtype, PackedView w, const int8_t* __restrict__ codes, int32_t* __restrict__ out,
                                   int64_t M, int64_t N, int64_t nb) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * M * nb) return;
  const int64_t b = i % nb, m = (i / nb) % M, n = i / (nb * M);
  const u32x4* xq = reinterpret_cast<const u32x4*>(codes + (m * nb + b) * QK);
  const u32x4 xlo = xq[0], xhi = xq[1];
  const u32x4 w0 = w.q0[n * nb + b];
  u32x4 w1 = w0;
  int isum;
  if (wtype == MLLM_HIP_Q4_0) {
    const uint32_t xs[8] = {xlo.x, xlo.y, xlo.z, xlo.w, xhi.x, xhi.y, xhi.z, xhi.w};
    int s = 0;
    for (int j = 0; j < 8; j++) s = __builtin_amdgcn_sdot4((int)xs[j], 0x01010101, s, false);
    isum = block_dot<MLLM_HIP_Q4_0>(w0, w1, xlo, xhi, -8 * s);
  } else {
    w1 = w.q1[n * nb + b];
    isum = block_dot<MLLM_HIP_Q8_0>(w0, w1, xlo, xhi, 0);
  }
  out[i] = isum;
}

// ---- launch-shape selection ------------------------------------------------------------------------------
static int g_tune_G = 0, g_tune_R = 0, g_tune_NW = 0;

struct GemvShape { int G, R, NW; };

static GemvShape pick_shape(int MT, int64_t N, int nb) {
  GemvShape s;
  s.R = MT >= 8 ? 4 : (MT >= 4 ? 2 : 1);
  s.NW = 4;
  // lanes per row: the narrowest power of two that yields >= ~2048 waves (8 per CU), never wider than the row
  s.G = 8;
  while (s.G < 64 && N * s.G / (64 * s.R) < 2048 && s.G * 2 <= (nb > 8 ? nb : 8)) s.G *= 2;
  if (g_tune_G) s.G = g_tune_G;
  if (g_tune_R) s.R = g_tune_R;
  if (g_tune_NW) s.NW = g_tune_NW;
  return s;
}

template <int WT, int MT, int G, int R>
static int launch_gemv_u(const GemvArgs& a, int NW, hipStream_t st) {
  constexpr int U = ((R >= 4) ? 1 : (R == 2 ? 2 : 4)) * (WT == MLLM_HIP_Q4_0 ? 2 : 1);
  const int rows_per_wg = NW * (64 / G) * R;
  const unsigned grid = (unsigned)((a.N + rows_per_wg - 1) / rows_per_wg);
  const size_t lds = (size_t)MT * a.nb * 40;
  auto kern = gemv_q_kernel<WT, MT, G, R, U>;
  if (lds > 64 * 1024) {
    if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
    HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, st, a);
  return (int)hipGetLastError();
}

template <int WT, int MT>
static int launch_gemv_m(const GemvArgs& a, GemvShape s, hipStream_t st) {
#define CASE(G_, R_) \
  if (s.G == G_ && s.R == R_) return launch_gemv_u<WT, MT, G_, R_>(a, s.NW, st);
  CASE(8, 1) CASE(16, 1) CASE(32, 1) CASE(64, 1)
  CASE(8, 2) CASE(16, 2) CASE(32, 2) CASE(64, 2)
  CASE(8, 4) CASE(16, 4) CASE(32, 4) CASE(64, 4)
#undef CASE
  return MLLM_HIP_E_BADARG;
}

template <int WT>
static int launch_gemv_w(const GemvArgs& a, hipStream_t st) {
  const int MT = a.M <= 1 ? 1 : (a.M <= 2 ? 2 : (a.M <= 4 ? 4 : 8));
  GemvShape s = pick_shape(MT, a.N, a.nb);
  switch (MT) {
    case 1: return launch_gemv_m<WT, 1>(a, s, st);
    case 2: return launch_gemv_m<WT, 2>(a, s, st);
    case 4: return launch_gemv_m<WT, 4>(a, s, st);
    default: return launch_gemv_m<WT, 8>(a, s, st);
  }
}

}  // namespace mllmhip

using namespace mllmhip;

// =========================================================================================================
// C ABI
// =========================================================================================================
MLLM_API const char* mllm_hip_version(void) { return "mllm-hip-qlinear 0.1 (gfx950)"; }

MLLM_API int mllm_hip_init(int device) {
  int count = 0;
  HIP_RET(hipGetDeviceCount(&count));
  if (device < 0 || device >= count) return MLLM_HIP_E_NODEVICE;
  hipDeviceProp_t prop;
  HIP_RET(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return MLLM_HIP_E_NODEVICE;
  return 0;
}

MLLM_API int mllm_hip_gemv_set_tuning(int lanes_per_row, int rows_per_group, int waves_per_wg) {
  auto ok = [](int v, std::initializer_list<int> allowed) {
    for (int a : allowed)
      if (v == a) return true;
    return false;
  };
  if (!ok(lanes_per_row, {0, 8, 16, 32, 64}) || !ok(rows_per_group, {0, 1, 2, 4}) || waves_per_wg < 0 || waves_per_wg > 4)
    return MLLM_HIP_E_BADARG;
  g_tune_G = lanes_per_row;
  g_tune_R = rows_per_group;
  g_tune_NW = waves_per_wg;
  return 0;
}

MLLM_API size_t mllm_hip_q_packed_bytes(int wtype, int64_t N, int64_t K) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || N <= 0 || K <= 0 || K % QK) return 0;
  return packed_bytes(wtype, N, K);
}

static int check_w(int wtype, const void* packed, int64_t N, int64_t K) {
  if (wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) return MLLM_HIP_E_BADARG;
  if (!packed || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (K % QK) return MLLM_HIP_E_SHAPE;
  if (N > INT32_MAX || K > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(packed) % 16) return MLLM_HIP_E_ALIGN;
  return 0;
}

MLLM_API int mllm_hip_q_prepack(int wtype, const void* blocks, int weight_scale_mode, void* packed, int64_t N, int64_t K,
                                void* stream) {
  int rc = check_w(wtype, packed, N, K);
  if (rc) return rc;
  if (!blocks || (weight_scale_mode != MLLM_HIP_SCALE_IEEE && weight_scale_mode != MLLM_HIP_SCALE_X86_REF))
    return MLLM_HIP_E_BADARG;
  const int64_t nblocks = N * (K / QK);
  PackedView v = packed_view(wtype, packed, N, K);
  hipLaunchKernelGGL(prepack_kernel, dim3((unsigned)((nblocks + 255) / 256)), dim3(256), 0, (hipStream_t)stream, wtype,
                     (const uint8_t*)blocks, weight_scale_mode == MLLM_HIP_SCALE_X86_REF, const_cast<u32x4*>(v.q0),
                     const_cast<u32x4*>(v.q1), const_cast<uint16_t*>(v.d), nblocks);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_linear_q_gemv(int wtype, const void* packed, const void* x, int x_dtype, const float* bias,
                                    float* y, int M, int64_t N, int64_t K, int act_scale_mode, void* stream) {
  int rc = check_w(wtype, packed, N, K);
  if (rc) return rc;
  if (!x || !y || (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16)) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (M < 1 || M > 8) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16) return MLLM_HIP_E_ALIGN;
  GemvArgs a;
  a.w = packed_view(wtype, packed, N, K);
  a.x = x;
  a.bias = bias;
  a.y = y;
  a.x_dtype = x_dtype;
  a.M = M;
  a.N = (int)N;
  a.nb = (int)(K / QK);
  a.x86_scale = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  return wtype == MLLM_HIP_Q4_0 ? launch_gemv_w<MLLM_HIP_Q4_0>(a, (hipStream_t)stream)
                                : launch_gemv_w<MLLM_HIP_Q8_0>(a, (hipStream_t)stream);
}

MLLM_API int mllm_hip_quantize_q8_0(const void* x, int x_dtype, int8_t* codes, uint16_t* d_bits, int64_t M, int64_t K,
                                    void* stream) {
  if (!x || !codes || !d_bits || M <= 0 || K <= 0 || (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16))
    return MLLM_HIP_E_BADARG;
  if (K % QK) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(codes) % 16) return MLLM_HIP_E_ALIGN;
  const int64_t nblocks = M * (K / QK);
  hipLaunchKernelGGL(quantize_q8_0_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, (hipStream_t)stream, x,
                     x_dtype, codes, d_bits, nblocks);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_q_dequantize(int wtype, const void* packed, float* w, int64_t N, int64_t K, void* stream) {
  int rc = check_w(wtype, packed, N, K);
  if (rc) return rc;
  if (!w) return MLLM_HIP_E_BADARG;
  const int64_t nblocks = N * (K / QK);
  hipLaunchKernelGGL(dequantize_kernel, dim3((unsigned)((nblocks + 255) / 256)), dim3(256), 0, (hipStream_t)stream, wtype,
                     packed_view(wtype, packed, N, K), w, nblocks);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_q_block_isums(int wtype, const void* packed, const int8_t* codes, int32_t* isums, int64_t M,
                                    int64_t N, int64_t K, void* stream) {
  int rc = check_w(wtype, packed, N, K);
  if (rc) return rc;
  if (!codes || !isums || M <= 0) return MLLM_HIP_E_BADARG;
  if (reinterpret_cast<uintptr_t>(codes) % 16) return MLLM_HIP_E_ALIGN;
  const int64_t total = N * M * (K / QK);
  hipLaunchKernelGGL(block_isums_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, wtype,
                     packed_view(wtype, packed, N, K), codes, isums, M, N, K / QK);
  return (int)hipGetLastError();
}
