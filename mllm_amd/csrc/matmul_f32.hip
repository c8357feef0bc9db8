// Activation x activation MatMul in fp32 (the kMatMul factory slot of the backend: attention scores / MoE gate logits in
// the reference run through it, mllm/backends/cpu/ops/MatMulOp.cpp:47-61).  Not a quantized path and not tuned: a
// 64x64 LDS-tiled kernel that keeps the op on the device.
#include "qcommon.h"

namespace mllmhip {

template <bool TA, bool TB>
__global__ __launch_bounds__(256) void matmul_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                         float* __restrict__ C, int M, int N, int K) {
  __shared__ float sA[16][64 + 1];
  __shared__ float sB[16][64 + 1];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int i = threadIdx.x; i < 16 * 64; i += 256) {
      const int kk = i / 64, r = i % 64;
      const int m = m0 + r, n = n0 + r, k = k0 + kk;
      sA[kk][r] = (m < M && k < K) ? (TA ? A[(int64_t)k * M + m] : A[(int64_t)m * K + k]) : 0.f;
      sB[kk][r] = (n < N && k < K) ? (TB ? B[(int64_t)n * K + k] : B[(int64_t)k * N + n]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; kk++)
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = fmaf(sA[kk][ty * 4 + i], sB[kk][tx * 4 + j], acc[i][j]);
    __syncthreads();
  }
  for (int i = 0; i < 4; i++)
    for (int j = 0; j < 4; j++) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < M && n < N) C[(int64_t)m * N + n] = acc[i][j];
    }
}

}  // namespace mllmhip

using namespace mllmhip;

MLLM_API int mllm_hip_matmul_f32(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K, int transpose_a,
                                 int transpose_b, void* stream) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return MLLM_HIP_E_SHAPE;
  const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
  hipStream_t st = (hipStream_t)stream;
  if (transpose_a && transpose_b) hipLaunchKernelGGL((matmul_f32_kernel<true, true>), grid, dim3(256), 0, st, A, B, C, (int)M, (int)N, (int)K);
  else if (transpose_a) hipLaunchKernelGGL((matmul_f32_kernel<true, false>), grid, dim3(256), 0, st, A, B, C, (int)M, (int)N, (int)K);
  else if (transpose_b) hipLaunchKernelGGL((matmul_f32_kernel<false, true>), grid, dim3(256), 0, st, A, B, C, (int)M, (int)N, (int)K);
  else hipLaunchKernelGGL((matmul_f32_kernel<false, false>), grid, dim3(256), 0, st, A, B, C, (int)M, (int)N, (int)K);
  return (int)hipGetLastError();
}
