// W8A8 Linear for prefill on gfx950: per-token dynamic int8 activation quantization + int8 MFMA GEMM with int32
// accumulation and a per-token x per-channel scale epilogue.
//
// Semantics (the reference's CUDA path, restated):
//   activation quant   pymllm/tests/bench_w8a8_activation_quant.py:20-26
//                      absmax = max(amax|x|, 1e-10); scale = absmax/127; q = clamp(round_half_even(x/scale), -128, 127)
//   GEMM + epilogue    pymllm/quantization/methods/compressed_tensors.py:450-468 (apply)
//                      mllm-kernel/mllm_kernel/cuda/csrc/cutlass_extensions/epilogue/epilogue_per_row_per_col_scale.h:273-280
//                      y = out_dtype( float(acc_int32) * (w_scale[n] * x_scale[m]) + bias[n] )
// The int32 accumulators are exact, so they match any other exact implementation bit for bit.
#include "qcommon.h"

namespace mllmhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// =========================================================================================================
// per-token dynamic quantization: one workgroup per row
// =========================================================================================================
template <int XT>
__device__ __forceinline__ float load_x1(const void* x, int64_t i) {
  return XT == MLLM_HIP_F32 ? reinterpret_cast<const float*>(x)[i] : bf16_to_f32(reinterpret_cast<const uint16_t*>(x)[i]);
}
template <int XT>
__device__ __forceinline__ void load_x8v(const void* x, int64_t i, float (&v)[8]) {
  if (XT == MLLM_HIP_F32) {
    const float4* p = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(x) + i);
    const float4 a = p[0], b = p[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    const u32x4 r = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(x) + i);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      v[2 * j] = __uint_as_float(w[j] << 16);
      v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}
__device__ __forceinline__ int quant1(float x, float scale) {
  float r = rintf(x / scale);  // IEEE division, round half to even
  r = fminf(127.f, fmaxf(-128.f, r));
  return (int)r;
}

template <int XT>
__global__ __launch_bounds__(256) void per_token_quant_kernel(const void* __restrict__ x, int8_t* __restrict__ q,
                                                              float* __restrict__ scale, int K) {
  __shared__ float s_max[4];
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x;
  const bool vec = (K % 8) == 0;
  const int64_t base = row * K;
  float amax = 0.f;
  if (vec) {
    for (int k = tid * 8; k < K; k += 256 * 8) {
      float v[8];
      load_x8v<XT>(x, base + k, v);
#pragma unroll
      for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[e]));
    }
  } else {
    for (int k = tid; k < K; k += 256) amax = fmaxf(amax, fabsf(load_x1<XT>(x, base + k)));
  }
  // wave max with DPP, then across the four waves through LDS
  amax = fmaxf(amax, dpp_f<0xB1>(amax));
  amax = fmaxf(amax, dpp_f<0x4E>(amax));
  amax = fmaxf(amax, dpp_f<0x141>(amax));
  amax = fmaxf(amax, dpp_f<0x140>(amax));
  amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
  amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
  if ((tid & 63) == 0) s_max[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
  amax = fmaxf(amax, 1e-10f);
  const float sc = amax / 127.0f;
  if (tid == 0) scale[row] = sc;
  if (vec) {
    for (int k = tid * 8; k < K; k += 256 * 8) {
      float v[8];
      load_x8v<XT>(x, base + k, v);
      uint32_t pk[2] = {0, 0};
#pragma unroll
      for (int e = 0; e < 8; e++) pk[e >> 2] |= ((uint32_t)quant1(v[e], sc) & 0xffu) << (8 * (e & 3));
      *reinterpret_cast<uint2*>(q + base + k) = make_uint2(pk[0], pk[1]);
    }
  } else {
    for (int k = tid; k < K; k += 256) q[base + k] = (int8_t)quant1(load_x1<XT>(x, base + k), sc);
  }
}

// =========================================================================================================
// int8 GEMM  C[m][n] = sum_k A[m][k] * W[n][k]   (both operands K-contiguous)
// =========================================================================================================
struct W8A8Args {
  const int8_t* A;      // [M][K]
  const int8_t* W;      // [N][K]
  const float* xs;      // [M]
  const float* ws;      // [N]
  const float* bias;    // [N] or null
  uint16_t* C;          // bf16 [M][N] or null
  int32_t* acc;         // int32 [M][N] or null
  int M, N, K;
};

// Workgroup tile BM x BN, K step 64 bytes; waves laid out (BM/WM) x (BN/WN), each owning WM x WN as 32x32 MFMA tiles
// (v_mfma_i32_32x32x32_i8: every lane supplies 16 consecutive k of one row of A and of one row of W).
// Global -> registers -> LDS with the next K step's loads in flight during the MFMAs; LDS rows are padded from 64 to 80
// bytes so that the 16-byte operand reads of 16 neighbouring rows fall into distinct banks.
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void w8a8_gemm_kernel(W8A8Args a) {
  constexpr int BK = 64, LDK = 80;
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  constexpr int CA = BM * 4 / NT, CB = BN * 4 / NT;  // 16-byte chunks per thread and K step
  static_assert(BM * 4 % NT == 0 && BN * 4 % NT == 0, "tile must split evenly over the threads");
  constexpr int TM = WM / 32, TN = WN / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int STAGE = (BM + BN) * LDK;  // one K step: A rows then W rows

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / (BN / WN), wn = wave % (BN / WN);

  // XCD-aware tile order: workgroup i runs on XCD i % 8, so give each XCD a contiguous run of tiles (same A panel)
  const int tilesN = (a.N + BN - 1) / BN, tilesM = (a.M + BM - 1) / BM;
  const int total = tilesM * tilesN;
  int tile = blockIdx.x;
  if (total % 8 == 0) tile = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;
  const int m0 = (tile / tilesN) * BM, n0 = (tile % tilesN) * BN;

  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.A), 0, (uint32_t)((int64_t)a.M * a.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t rW = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.W), 0, (uint32_t)((int64_t)a.N * a.K), 0x00020000);

  // chunk c of a thread: row = (tid + c*NT) / 4, 16-byte column = (tid + c*NT) % 4
  uint32_t offA[CA], offB[CB];
#pragma unroll
  for (int c = 0; c < CA; c++) {
    const int idx = tid + c * NT, row = m0 + idx / 4;
    offA[c] = row < a.M ? (uint32_t)((int64_t)row * a.K + (idx % 4) * 16) : 0xffffffffu;
  }
#pragma unroll
  for (int c = 0; c < CB; c++) {
    const int idx = tid + c * NT, row = n0 + idx / 4;
    offB[c] = row < a.N ? (uint32_t)((int64_t)row * a.K + (idx % 4) * 16) : 0xffffffffu;
  }
  u32x4 gA[CA], gB[CB];
  auto gload = [&](int k0) {
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const bool ok = offA[c] != 0xffffffffu && k0 + ((tid + c * NT) % 4) * 16 < a.K;
      gA[c] = __builtin_amdgcn_raw_buffer_load_b128(rA, ok ? offA[c] + k0 : 0xffffffffu, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < CB; c++) {
      const bool ok = offB[c] != 0xffffffffu && k0 + ((tid + c * NT) % 4) * 16 < a.K;
      gB[c] = __builtin_amdgcn_raw_buffer_load_b128(rW, ok ? offB[c] + k0 : 0xffffffffu, 0, 0);
    }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const int idx = tid + c * NT;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + (idx / 4) * LDK + (idx % 4) * 16) = gA[c];
    }
#pragma unroll
    for (int c = 0; c < CB; c++) {
      const int idx = tid + c * NT;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + (BM + idx / 4) * LDK + (idx % 4) * 16) = gB[c];
    }
  };

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

  const int KT = (a.K + BK - 1) / BK;
  gload(0);
  sstore(0);
  __syncthreads();
  const int lrow = lane & 31, lk = (lane >> 5) * 16;
  for (int kt = 0; kt < KT; kt++) {
    const int buf = kt & 1;
    if (kt + 1 < KT) gload((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      v4i fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; i++)
        fa[i] = *reinterpret_cast<const v4i*>(smem + buf * STAGE + (wm * WM + i * 32 + lrow) * LDK + ks * 32 + lk);
#pragma unroll
      for (int j = 0; j < TN; j++)
        fb[j] = *reinterpret_cast<const v4i*>(smem + buf * STAGE + (BM + wn * WN + j * 32 + lrow) * LDK + ks * 32 + lk);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) sstore(buf ^ 1);
    __syncthreads();
  }

  // epilogue.  32x32 accumulator layout: register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32.
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int n = n0 + wn * WN + j * 32 + lrow;
    const bool nok = n < a.N;
    const float wsn = nok ? a.ws[n] : 0.f;
    const float bn = (nok && a.bias) ? a.bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
        if (nok && m < a.M) {
          const int v = acc[i][j][r];
          if (a.acc) a.acc[(int64_t)m * a.N + n] = v;
          if (a.C) {
            float f = (float)v * (wsn * a.xs[m]);
            if (a.bias) f += bn;
            a.C[(int64_t)m * a.N + n] = f32_to_bf16(f);
          }
        }
      }
    }
  }
}

template <int BM, int BN, int WM, int WN>
static int launch_w8a8(const W8A8Args& a, hipStream_t st) {
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  const size_t lds = 2 * (size_t)(BM + BN) * 80;
  const unsigned grid = (unsigned)(((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN));
  auto kern = w8a8_gemm_kernel<BM, BN, WM, WN>;
  if (lds > 64 * 1024)
    HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), lds, st, a);
  return (int)hipGetLastError();
}

static int g_w8a8_tile = 0;  // 0 = heuristic, 1 = 256x192, 2 = 128x128, 3 = 64x64

}  // namespace mllmhip

using namespace mllmhip;

MLLM_API int mllm_hip_w8a8_set_tuning(int tile) {
  if (tile < 0 || tile > 3) return MLLM_HIP_E_BADARG;
  g_w8a8_tile = tile;
  return 0;
}

MLLM_API int mllm_hip_per_token_quant_int8(const void* x, int x_dtype, int8_t* q, float* scale, int64_t M, int64_t K,
                                           void* stream) {
  if (!x || !q || !scale || M <= 0 || K <= 0 || (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16))
    return MLLM_HIP_E_BADARG;
  if (M > INT32_MAX || K > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (K % 8 == 0 && (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(q) % 8)) return MLLM_HIP_E_ALIGN;
  if (x_dtype == MLLM_HIP_F32)
    hipLaunchKernelGGL(per_token_quant_kernel<MLLM_HIP_F32>, dim3((unsigned)M), dim3(256), 0, (hipStream_t)stream, x, q, scale, (int)K);
  else
    hipLaunchKernelGGL(per_token_quant_kernel<MLLM_HIP_BF16>, dim3((unsigned)M), dim3(256), 0, (hipStream_t)stream, x, q, scale, (int)K);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_w8a8_gemm(const int8_t* xq, const float* x_scale, const int8_t* W, const float* w_scale,
                                const float* bias, void* out_bf16, int32_t* acc_out, int64_t M, int64_t N, int64_t K,
                                void* stream) {
  if (!xq || !W || M <= 0 || N <= 0 || K <= 0 || (!out_bf16 && !acc_out)) return MLLM_HIP_E_BADARG;
  if (out_bf16 && (!x_scale || !w_scale)) return MLLM_HIP_E_BADARG;
  if (K % 16) return MLLM_HIP_E_SHAPE;
  if (M * K >= ((int64_t)1 << 32) || N * K >= ((int64_t)1 << 32) || M > INT32_MAX || N > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(xq) % 16 || reinterpret_cast<uintptr_t>(W) % 16) return MLLM_HIP_E_ALIGN;
  W8A8Args a{xq, W, x_scale, w_scale, bias, (uint16_t*)out_bf16, acc_out, (int)M, (int)N, (int)K};
  hipStream_t st = (hipStream_t)stream;
  int tile = g_w8a8_tile;
  if (!tile) {
    const int64_t big = ((M + 255) / 256) * ((N + 191) / 192);
    const int64_t mid = ((M + 127) / 128) * ((N + 127) / 128);
    (void)big;  // the 256x192 tile is compiled and tested but measured slower than 128x128 so far
    tile = mid >= 128 ? 2 : 3;
  }
  switch (tile) {
    case 1: return launch_w8a8<256, 192, 128, 96>(a, st);
    case 2: return launch_w8a8<128, 128, 64, 64>(a, st);
    default: return launch_w8a8<64, 64, 32, 32>(a, st);
  }
}

MLLM_API size_t mllm_hip_w8a8_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0) return 0;
  return align_up((size_t)M * K, 256) + align_up((size_t)M * 4, 256);
}

MLLM_API int mllm_hip_w8a8_linear(const void* x, int x_dtype, const int8_t* W, const float* w_scale, const float* bias,
                                  void* out_bf16, int64_t M, int64_t N, int64_t K, void* workspace, void* stream) {
  if (!workspace) return MLLM_HIP_E_BADARG;
  if (reinterpret_cast<uintptr_t>(workspace) % 16) return MLLM_HIP_E_ALIGN;
  int8_t* q = reinterpret_cast<int8_t*>(workspace);
  float* xs = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + align_up((size_t)M * K, 256));
  int rc = mllm_hip_per_token_quant_int8(x, x_dtype, q, xs, M, K, stream);
  if (rc) return rc;
  return mllm_hip_w8a8_gemm(q, xs, W, w_scale, bias, out_bf16, nullptr, M, N, K, stream);
}
