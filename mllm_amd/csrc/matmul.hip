// Activation x activation MatMul on the matrix cores (the kMatMul factory slot of the backend: attention scores, attention
// x values and the MoE gate logits of the reference run through it, mllm/backends/cpu/ops/MatMulOp.cpp:27-61 with the batch
// loop of mllm/backends/cpu/kernels/common/ggml/matmul.cpp / mllm_blas).  Not a quantized path.
//   fp32 operands   v_mfma_f32_32x32x2f32: exact fp32 products, fp32 accumulation (the CPU's arithmetic in another order)
//   bf16 / fp16     v_mfma_f32_32x32x16_{bf16,f16}: exact products, fp32 accumulation, one rounding of the result
// One launch covers the whole batch (blockIdx.z walks it; a stride of 0 broadcasts an operand).
//
// Workgroup = 2 x 2 waves, each wave (32 TM) x (32 TN) outputs, K step 32.  Both operand tiles sit in LDS as [row][k] with
// 16 bytes of padding per row, whichever way the tensor is laid out in memory (an operand that is contiguous along its row
// index is transposed on its way into LDS).  Inside a K step lane half h takes k = 16 h .. 16 h + 15 of its row, for both
// operands alike: the order in which an MFMA walks k is free, and this way every lane fetches its operands of the whole
// step with 16-byte LDS reads.
#include <algorithm>

#include "qcommon.h"

namespace mllmhip {

typedef __bf16 mm_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 mm_f16x8 __attribute__((ext_vector_type(8)));
typedef float mm_f32x16 __attribute__((ext_vector_type(16)));

struct MMArgs {
  const void* A;
  const void* B;
  void* C;
  int M, N, K, batch;
  int64_t sA, sB, sC;  // batch strides in elements
  int vecA, vecB;      // 16-byte loads allowed (base, leading dimension and batch stride all multiples of 16 bytes)
};

template <int DT>
struct MMElem {
  using type = uint16_t;
};
template <>
struct MMElem<MLLM_HIP_F32> {
  using type = float;
};

// One operand tile of ROWS x 32 elements from global memory into registers, then into LDS as [row][k].
// CONTIG_K: the tensor is [rows][K] (k contiguous); otherwise it is [K][rows].
template <typename E, int ROWS, bool CONTIG_K>
struct MMTile {
  static constexpr int VE = 16 / (int)sizeof(E);
  static constexpr int LDK = 32 + VE;
  static constexpr int NV = ROWS * 32 / VE / 256;  // 16-byte vectors per thread
  static_assert(ROWS * 32 / VE % 256 == 0, "tile must split evenly over 256 threads");
  u32x4 v[NV];

  static __device__ __forceinline__ uint32_t bits(E e) {
    if constexpr (sizeof(E) == 4) return __builtin_bit_cast(uint32_t, e);
    else return (uint32_t)e;
  }
  // j is a compile-time constant after unrolling; the element goes through a plain dword first (a bit cast applied directly
  // to q[j] was compiled as a read of element 0)
  static __device__ __forceinline__ E elem(u32x4 q, int j) {
    const uint32_t d = sizeof(E) == 4 ? q[j] : (q[j >> 1] >> (16 * (j & 1)));
    if constexpr (sizeof(E) == 4) return __builtin_bit_cast(E, d);
    else return (E)d;
  }

  __device__ __forceinline__ void load(const E* __restrict__ X, int row0, int k0, int rows, int K, bool vec) {
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int idx = c * 256 + (int)threadIdx.x;
      int r, k;
      int64_t off;
      if (CONTIG_K) {
        r = row0 + idx / (32 / VE), k = k0 + (idx % (32 / VE)) * VE;
        off = (int64_t)r * K + k;
      } else {
        k = k0 + idx / (ROWS / VE), r = row0 + (idx % (ROWS / VE)) * VE;
        off = (int64_t)k * rows + r;
      }
      if (vec) {
        u32x4 q = {0u, 0u, 0u, 0u};
        if (r < rows && k < K) q = *reinterpret_cast<const u32x4*>(X + off);
        v[c] = q;
      } else {
        u32x4 q = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < VE; ++j) {
          const bool ok = CONTIG_K ? (r < rows && k + j < K) : (r + j < rows && k < K);
          const uint32_t e = ok ? bits(X[off + j]) : 0u;
          if constexpr (sizeof(E) == 4) q[j] = e;
          else q[j >> 1] |= e << (16 * (j & 1));
        }
        v[c] = q;
      }
    }
  }
  __device__ __forceinline__ void store(E* __restrict__ s) const {
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int idx = c * 256 + (int)threadIdx.x;
      if (CONTIG_K) {
        const int r = idx / (32 / VE), k = (idx % (32 / VE)) * VE;
        *reinterpret_cast<u32x4*>(s + r * LDK + k) = v[c];
      } else {
        const int k = idx / (ROWS / VE), r = (idx % (ROWS / VE)) * VE;
#pragma unroll
        for (int j = 0; j < VE; ++j) s[(r + j) * LDK + k] = elem(v[c], j);
      }
    }
  }
};

template <int DT, bool TA, bool TB, int TM, int TN>
__global__ __launch_bounds__(256) void matmul_kernel(MMArgs a) {
  using E = typename MMElem<DT>::type;
  constexpr int VE = 16 / (int)sizeof(E), LDK = 32 + VE;
  constexpr int BM = 64 * TM, BN = 64 * TN;
  __shared__ __align__(16) E sA[BM * LDK];
  __shared__ __align__(16) E sB[BN * LDK];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1, r = lane & 31, h = lane >> 5;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int KT = (a.K + 31) / 32;

  for (int z = blockIdx.z; z < a.batch; z += gridDim.z) {
    const E* A = reinterpret_cast<const E*>(a.A) + z * a.sA;
    const E* B = reinterpret_cast<const E*>(a.B) + z * a.sB;
    E* C = reinterpret_cast<E*>(a.C) + z * a.sC;

    // A is [M][K], or [K][M] when transposed; B is [K][N], or [N][K] when transposed
    MMTile<E, BM, !TA> ta;
    MMTile<E, BN, TB> tb;
    mm_f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    ta.load(A, m0, 0, a.M, a.K, a.vecA);
    tb.load(B, n0, 0, a.N, a.K, a.vecB);
    for (int kt = 0; kt < KT; ++kt) {
      __syncthreads();  // the previous step's LDS reads are done
      ta.store(sA);
      tb.store(sB);
      __syncthreads();
      if (kt + 1 < KT) {
        ta.load(A, m0, (kt + 1) * 32, a.M, a.K, a.vecA);
        tb.load(B, n0, (kt + 1) * 32, a.N, a.K, a.vecB);
      }
      if constexpr (DT == MLLM_HIP_F32) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {  // four k of this lane's sixteen at a time
          f32x4 fa[TM], fb[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const f32x4*>(sA + (wm * 32 * TM + i * 32 + r) * LDK + 16 * h + 4 * q);
#pragma unroll
          for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const f32x4*>(sB + (wn * 32 * TN + j * 32 + r) * LDK + 16 * h + 4 * q);
#pragma unroll
          for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
              for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          u32x4 fa[TM], fb[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const u32x4*>(sA + (wm * 32 * TM + i * 32 + r) * LDK + 16 * h + 8 * q);
#pragma unroll
          for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const u32x4*>(sB + (wn * 32 * TN + j * 32 + r) * LDK + 16 * h + 8 * q);
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
              if constexpr (DT == MLLM_HIP_BF16)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(mm_bf16x8, fa[i]),
                                                                    __builtin_bit_cast(mm_bf16x8, fb[j]), acc[i][j], 0, 0, 0);
              else
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(mm_f16x8, fa[i]),
                                                                   __builtin_bit_cast(mm_f16x8, fb[j]), acc[i][j], 0, 0, 0);
            }
        }
      }
    }

    // 32x32 accumulator layout: register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4, column l % 32
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * 32 * TN + j * 32 + r;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m0 + wm * 32 * TM + i * 32 + 8 * (v / 4) + 4 * h + (v % 4);
          if (n < a.N && m < a.M) {
            const float f = acc[i][j][v];
            if constexpr (DT == MLLM_HIP_F32) C[(int64_t)m * a.N + n] = f;
            else if constexpr (DT == MLLM_HIP_BF16) C[(int64_t)m * a.N + n] = f32_to_bf16(f);
            else C[(int64_t)m * a.N + n] = f32_to_f16bits(f);
          }
        }
    }
  }
}

// Up to four rows of A [M][K] against B [K][N] (attention probabilities x values of a decode token): a GEMV per row, bound by
// reading B once, which the tile kernel above walks with one workgroup per 64 columns and a K step at a time (32 heads x
// 8192 x 128 bf16: 158 us, 0.43 TB/s).  Here a workgroup of sixteen waves takes 2^lpr_log2 x VE columns (VE elements = 16
// bytes per lane); a wave reads 64 >> lpr_log2 rows of B per pass, the waves stride over K, four passes requested before the
// first is multiplied; fp32 sums per lane, then over the lanes of a column (wave shuffles), then over the waves in order
// through LDS.  Exact products, fp32 sums in another order than the tile kernel's.
template <int DT>
__device__ __forceinline__ float mm_to_f32(typename MMElem<DT>::type e) {
  if constexpr (DT == MLLM_HIP_F32) return e;
  else if constexpr (DT == MLLM_HIP_BF16) return bf16_to_f32(e);
  else return f16bits_to_f32(e);
}
constexpr int MMR_WAVES = 16;
template <int DT, int MR>
__global__ __launch_bounds__(MMR_WAVES * 64) void matmul_rows_kernel(MMArgs a, int lpr_log2) {
  using E = typename MMElem<DT>::type;
  constexpr int VE = 16 / (int)sizeof(E);
  extern __shared__ __align__(16) unsigned char mmr_smem[];
  float* s_part = reinterpret_cast<float*>(mmr_smem);  // [wave][row][column of the workgroup]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lpr = 1 << lpr_log2, rpw = 64 >> lpr_log2, ncols = lpr * VE;
  const int col = (lane & (lpr - 1)) * VE, sub = lane >> lpr_log2;
  const int n0 = (int)blockIdx.x * ncols + col;
  const int kstep = MMR_WAVES * rpw;
  constexpr int UB = 4;
  for (int z = blockIdx.y; z < a.batch; z += gridDim.y) {
    const E* A = reinterpret_cast<const E*>(a.A) + z * a.sA;
    const E* B = reinterpret_cast<const E*>(a.B) + z * a.sB;
    E* C = reinterpret_cast<E*>(a.C) + z * a.sC;
    float acc[MR][VE];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
      for (int j = 0; j < VE; j++) acc[m][j] = 0.f;
    for (int k0 = wave * rpw + sub; k0 < a.K; k0 += kstep * UB) {
      u32x4 bv[UB];
      E av[UB][MR];
#pragma unroll
      for (int u = 0; u < UB; u++) {
        const int k = k0 + u * kstep;
        const bool ok = k < a.K && n0 < a.N;  // (N is a multiple of VE here: a lane's columns are all inside or all outside)
        bv[u] = u32x4{0u, 0u, 0u, 0u};
        if (ok) bv[u] = *reinterpret_cast<const u32x4*>(B + (int64_t)k * a.N + n0);
#pragma unroll
        for (int m = 0; m < MR; m++) av[u][m] = (ok && m < a.M) ? A[(int64_t)m * a.K + k] : (E)0;
      }
#pragma unroll
      for (int u = 0; u < UB; u++)
#pragma unroll
        for (int m = 0; m < MR; m++) {
          const float am = mm_to_f32<DT>(av[u][m]);
#pragma unroll
          for (int j = 0; j < VE; j++) acc[m][j] = fmaf(am, mm_to_f32<DT>(MMTile<E, 64, true>::elem(bv[u], j)), acc[m][j]);
        }
    }
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
      for (int j = 0; j < VE; j++) {
        float v = acc[m][j];
        for (int off = lpr; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
        if (sub == 0) s_part[((size_t)wave * MR + m) * ncols + col + j] = v;
      }
    __syncthreads();
    for (int i = tid; i < MR * ncols; i += MMR_WAVES * 64) {
      const int m = i / ncols, c = i - m * ncols, n = (int)blockIdx.x * ncols + c;
      if (m < a.M && n < a.N) {
        float f = 0.f;
#pragma unroll
        for (int w = 0; w < MMR_WAVES; w++) f += s_part[((size_t)w * MR + m) * ncols + c];
        if constexpr (DT == MLLM_HIP_F32) C[(int64_t)m * a.N + n] = f;
        else if constexpr (DT == MLLM_HIP_BF16) C[(int64_t)m * a.N + n] = f32_to_bf16(f);
        else C[(int64_t)m * a.N + n] = f32_to_f16bits(f);
      }
    }
    __syncthreads();
  }
}
// the launch shape of the kernel above; false where it does not apply (the tile kernel then)
template <int DT>
static bool launch_matmul_rows(const MMArgs& a, hipStream_t st, int* rc) {
  constexpr int VE = 16 / (int)sizeof(typename MMElem<DT>::type);
  if (a.M > 4 || !a.vecB || a.N % VE || a.K < 256) return false;
  int lg = 0;
  while (lg < 6 && (VE << lg) < a.N) lg++;
  // narrower column blocks while the launch has fewer than 128 workgroups, down to 64 bytes of a row per workgroup
  while (lg > 2 && (int64_t)a.batch * ((a.N + (VE << lg) - 1) / (VE << lg)) < 128) lg--;
  const int mr = a.M <= 1 ? 1 : (a.M <= 2 ? 2 : 4);
  while (lg > 0 && (size_t)MMR_WAVES * mr * (VE << lg) * sizeof(float) > 64 * 1024) lg--;  // the waves' partial sums fit 64 KB of LDS
  const int ncols = VE << lg;
  const dim3 grid((unsigned)((a.N + ncols - 1) / ncols), (unsigned)std::min(a.batch, 65535));
  const size_t lds = (size_t)MMR_WAVES * 4 * ncols * sizeof(float);
  if (a.M <= 1) hipLaunchKernelGGL((matmul_rows_kernel<DT, 1>), grid, dim3(MMR_WAVES * 64), lds / 4, st, a, lg);
  else if (a.M <= 2) hipLaunchKernelGGL((matmul_rows_kernel<DT, 2>), grid, dim3(MMR_WAVES * 64), lds / 2, st, a, lg);
  else hipLaunchKernelGGL((matmul_rows_kernel<DT, 4>), grid, dim3(MMR_WAVES * 64), lds, st, a, lg);
  *rc = (int)hipGetLastError();
  return true;
}

template <int DT, bool TA, bool TB>
static int launch_matmul(const MMArgs& a, hipStream_t st) {
  if constexpr (!TA && !TB) {
    int rc = 0;
    if (launch_matmul_rows<DT>(a, st, &rc)) return rc;
  }
  // the small tile where the large one would leave most of the 256 CUs without a workgroup
  const int64_t big = (int64_t)((a.M + 127) / 128) * ((a.N + 127) / 128) * a.batch;
  const unsigned gz = (unsigned)std::min(a.batch, 65535);
  if (big >= 256 && a.M > 64 && a.N > 64) {
    hipLaunchKernelGGL((matmul_kernel<DT, TA, TB, 2, 2>), dim3((unsigned)((a.N + 127) / 128), (unsigned)((a.M + 127) / 128), gz),
                       dim3(256), 0, st, a);
  } else {
    hipLaunchKernelGGL((matmul_kernel<DT, TA, TB, 1, 1>), dim3((unsigned)((a.N + 63) / 64), (unsigned)((a.M + 63) / 64), gz),
                       dim3(256), 0, st, a);
  }
  return (int)hipGetLastError();
}

template <int DT>
static int launch_matmul_t(const MMArgs& a, int ta, int tb, hipStream_t st) {
  if (ta && tb) return launch_matmul<DT, true, true>(a, st);
  if (ta) return launch_matmul<DT, true, false>(a, st);
  if (tb) return launch_matmul<DT, false, true>(a, st);
  return launch_matmul<DT, false, false>(a, st);
}

}  // namespace mllmhip

using namespace mllmhip;

MLLM_API int mllm_hip_matmul_batched(const void* A, const void* B, void* C, int dtype, int64_t batch, int64_t M, int64_t N,
                                     int64_t K, int64_t stride_a, int64_t stride_b, int64_t stride_c, int transpose_a,
                                     int transpose_b, void* stream) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0 || batch <= 0 || stride_a < 0 || stride_b < 0 || stride_c < 0)
    return MLLM_HIP_E_BADARG;
  if (dtype != MLLM_HIP_F32 && dtype != MLLM_HIP_BF16 && dtype != MLLM_HIP_F16) return MLLM_HIP_E_BADARG;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX || batch > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if ((M + 63) / 64 > 65535) return MLLM_HIP_E_SHAPE;
  if (batch > 1 && stride_c < M * N) return MLLM_HIP_E_SHAPE;  // outputs of different batch entries must not overlap
  const int es = dtype == MLLM_HIP_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(A) % es || reinterpret_cast<uintptr_t>(B) % es || reinterpret_cast<uintptr_t>(C) % es)
    return MLLM_HIP_E_ALIGN;
  const int ve = 16 / es;
  auto vec_ok = [&](const void* p, int64_t ld, int64_t stride) {
    return reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % ve == 0 && (batch == 1 || stride % ve == 0);
  };
  MMArgs a{A, B, C, (int)M, (int)N, (int)K, (int)batch, stride_a, stride_b, stride_c,
           vec_ok(A, transpose_a ? M : K, stride_a) ? 1 : 0, vec_ok(B, transpose_b ? K : N, stride_b) ? 1 : 0};
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case MLLM_HIP_F32: return launch_matmul_t<MLLM_HIP_F32>(a, transpose_a, transpose_b, st);
    case MLLM_HIP_BF16: return launch_matmul_t<MLLM_HIP_BF16>(a, transpose_a, transpose_b, st);
    default: return launch_matmul_t<MLLM_HIP_F16>(a, transpose_a, transpose_b, st);
  }
}

MLLM_API int mllm_hip_matmul_f32(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K, int transpose_a,
                                 int transpose_b, void* stream) {
  return mllm_hip_matmul_batched(A, B, C, MLLM_HIP_F32, 1, M, N, K, 0, 0, 0, transpose_a, transpose_b, stream);
}
