// Sizes of the "gemm-packed" weight layout of the matrix-core GEMM (moe.hip) and the entry into that GEMM for callers
// that bring their own fp16 activations (kquant.hip: Q4_K / Q6_K weights with the Q8_K round trip of the activations).
//
//   codes   4-bit types (Q4_0, Q4_K): [N/32][K/64][64 lanes][16 B]; 8-bit types (Q8_0; Q6_K with its codes widened to
//           int8): [N/32][K/64][2][64 lanes][16 B]; N padded to 32 rows, K to 128 elements
//   scales  [N/32][K/64][32 rows] records of one dword (Q4_0 / Q8_0: the fp16 scales of the step's two blocks) or two
//           (Q4_K: the two sub-block scales d*sc, then the two offsets dmin*m; Q6_K: the step's four 16-element scales d*sc)
#pragma once
#include "qcommon.h"

namespace mllmhip {

__host__ __device__ inline int64_t qg_kp(int64_t K) { return (K + 127) / 128 * 128; }
__host__ __device__ inline int64_t qg_np(int64_t N) { return (N + 31) / 32 * 32; }
__host__ __device__ constexpr bool qg_nibbles(int wtype) { return wtype == MLLM_HIP_Q4_0 || wtype == MLLM_HIP_Q4_K; }
__host__ __device__ constexpr int qg_scale_dwords(int wtype) { return (wtype == MLLM_HIP_Q4_K || wtype == MLLM_HIP_Q6_K) ? 2 : 1; }
__host__ __device__ inline int64_t qg_qbytes(int wtype, int64_t N, int64_t K) {
  return qg_nibbles(wtype) ? qg_np(N) * qg_kp(K) / 2 : qg_np(N) * qg_kp(K);
}
__host__ __device__ inline int64_t qg_bytes(int wtype, int64_t N, int64_t K) {
  return qg_qbytes(wtype, N, K) + qg_np(N) * (qg_kp(K) / 64) * 4 * qg_scale_dwords(wtype);
}

// y[M][N] fp32 = xh[M][K] (fp16) * W^T + bias on the matrix cores; route_ws: qg_route_bytes(M) bytes, 16-byte aligned
// partial_ws: null, or qg_partial_bytes(M, N, K) bytes (256-byte aligned) for short batches: K is then cut into ranges that
// run as separate workgroups (qg_partial_bytes returns 0 where that does not pay; pass null then)
size_t qg_route_bytes(int64_t M);
size_t qg_partial_bytes(int64_t M, int64_t N, int64_t K);
int qg_linear_run(int wtype, const void* gemm_packed, const uint16_t* xh, const float* bias, float* y, int64_t M, int64_t N,
                  int64_t K, void* route_ws, void* partial_ws, hipStream_t st);

}  // namespace mllmhip
