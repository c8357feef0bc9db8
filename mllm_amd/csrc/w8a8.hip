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

// NI > 0: the row (K <= NI * 2048, K % 8 == 0) stays in registers between the maximum and the rounding, eight elements per
// lane and item; NI == 0: any K, the row is read twice (the second time from cache).
template <int XT, int NI>
__global__ __launch_bounds__(256) void per_token_quant_kernel(const void* __restrict__ x, int8_t* __restrict__ q,
                                                              float* __restrict__ scale, int K) {
  __shared__ float s_max[4];
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x;
  const bool vec = (K % 8) == 0;
  const int64_t base = row * K;
  float amax = 0.f;
  float held[NI > 0 ? NI : 1][8];
  if (NI > 0) {
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const int k = (tid + 256 * i) * 8;
      load_x8v<XT>(x, base + (k < K ? k : K - 8), held[i]);  // clamped: lanes past the row re-read its tail and are not stored
#pragma unroll
      for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(held[i][e]));
    }
  } else if (vec) {
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
  if (NI > 0) {
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const int k = (tid + 256 * i) * 8;
      uint32_t pk[2] = {0, 0};
#pragma unroll
      for (int e = 0; e < 8; e++) pk[e >> 2] |= ((uint32_t)quant1(held[i][e], sc) & 0xffu) << (8 * (e & 3));
      if (k < K) *reinterpret_cast<uint2*>(q + base + k) = make_uint2(pk[0], pk[1]);
    }
  } else if (vec) {
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
// Global -> registers -> LDS with the loads of the next D K steps in flight during the MFMAs.  LDS rows are 64 bytes,
// unpadded: measured on MI355X, 16-byte operand reads run at the full LDS rate (about 64 B/clk/CU) for every row stride
// except multiples of 128 bytes.
template <int BM, int BN, int WM, int WN, int D>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void w8a8_gemm_kernel(W8A8Args a) {
  constexpr int BK = 64, LDK = 64;
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
  // D register sets hold the global loads of the next D K steps while they are in flight (HBM/L2 latency is several
  // K steps of MFMA work); loads are issued unconditionally (past K they are out of range or unused) so that the
  // hardware wait counters stay exact.
  u32x4 gA[D][CA], gB[D][CB];
  auto gload = [&](int k0, u32x4 (&ga)[CA], u32x4 (&gb)[CB]) {
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const bool ok = offA[c] != 0xffffffffu && k0 + ((tid + c * NT) % 4) * 16 < a.K;
      ga[c] = __builtin_amdgcn_raw_buffer_load_b128(rA, ok ? offA[c] + k0 : 0xffffffffu, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < CB; c++) {
      const bool ok = offB[c] != 0xffffffffu && k0 + ((tid + c * NT) % 4) * 16 < a.K;
      gb[c] = __builtin_amdgcn_raw_buffer_load_b128(rW, ok ? offB[c] + k0 : 0xffffffffu, 0, 0);
    }
  };
  auto sstore = [&](int buf, const u32x4 (&ga)[CA], const u32x4 (&gb)[CB]) {
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const int idx = tid + c * NT;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + (idx / 4) * LDK + (idx % 4) * 16) = ga[c];
    }
#pragma unroll
    for (int c = 0; c < CB; c++) {
      const int idx = tid + c * NT;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + (BM + idx / 4) * LDK + (idx % 4) * 16) = gb[c];
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
  // K step s lives in register set s % D from its issue until it is written to LDS buffer s % 2 one step before use
#pragma unroll
  for (int d = 0; d < D; d++) gload(d * BK, gA[d], gB[d]);
  sstore(0, gA[0], gB[0]);
  __syncthreads();
  const int lrow = lane & 31, lk = (lane >> 5) * 16;
  for (int kt0 = 0; kt0 < KT; kt0 += D) {
#pragma unroll
    for (int d = 0; d < D; d++) {
      const int kt = kt0 + d;
      if (kt < KT) {  // uniform
        const int buf = kt & 1;
        gload((kt + D) * BK, gA[d], gB[d]);  // set d was written to LDS one step ago: free again
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
        sstore(buf ^ 1, gA[(d + 1) % D], gB[(d + 1) % D]);  // K step kt + 1
        __syncthreads();
      }
    }
  }

  // epilogue.  32x32 accumulator layout: register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32.
  // The row / column scales and the bias of the tile go through LDS once (the staging buffers are free after the last
  // barrier), so the per-element work is three fp32 operations and a store, with no loads or branches on full tiles.
  float* sXs = reinterpret_cast<float*>(smem);
  float* sWs = sXs + BM;
  float* sBi = sWs + BN;
  for (int i = tid; i < BM; i += NT) sXs[i] = (a.xs && m0 + i < a.M) ? a.xs[m0 + i] : 0.f;
  for (int i = tid; i < BN; i += NT) {
    sWs[i] = (a.ws && n0 + i < a.N) ? a.ws[n0 + i] : 0.f;
    sBi[i] = (a.bias && n0 + i < a.N) ? a.bias[n0 + i] : 0.f;
  }
  __syncthreads();
  const bool full = m0 + BM <= a.M && n0 + BN <= a.N;
  const int hi4 = 4 * (lane >> 5);
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int cn = wn * WN + j * 32 + lrow;
    const int n = n0 + cn;
    const bool nok = n < a.N;
    const float wsn = sWs[cn], bn = sBi[cn];
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int rm = wm * WM + i * 32 + 8 * g + hi4;  // first of four consecutive rows
        const f32x4 xs4 = *reinterpret_cast<const f32x4*>(&sXs[rm]);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int m = m0 + rm + e;
          const int v = acc[i][j][4 * g + e];
          if (full || (nok && m < a.M)) {
            if (a.acc) a.acc[(int64_t)m * a.N + n] = v;
            if (a.C) {
              float f = (float)v * (wsn * xs4[e]);
              if (a.bias) f += bn;
              a.C[(int64_t)m * a.N + n] = f32_to_bf16(f);
            }
          }
        }
      }
    }
  }
}

// Weight layout for the large-problem kernel below: the matrix in v_mfma_i32_32x32x32_i8 operand order.  Block (nb, kb)
// of 32 rows x 32 bytes is 1 KB, lane l = (row l%32, k-half l/32) owns bytes [16 l, 16 l + 16); blocks are ordered
// [nb][kb] with N padded to 32 and K to 128 by zeros.  A wave's 16-byte operand load then reads one contiguous KB
// (8 cache lines) instead of 32 bytes from each of 32 rows (32 cache lines, each touched again by the next three loads).
__host__ __device__ inline int64_t w8a8_packed_k(int64_t K) { return (K + 127) / 128 * 128; }
__host__ __device__ inline int64_t w8a8_packed_n(int64_t N) { return (N + 31) / 32 * 32; }

__global__ __launch_bounds__(256) void w8a8_prepack_kernel(const int8_t* __restrict__ W, u32x4* __restrict__ P, int N, int K,
                                                           int64_t chunks) {
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one 16-byte piece of the packed matrix
  if (c >= chunks) return;
  const int kbs = (int)(w8a8_packed_k(K) / 32);
  const int l = (int)(c % 64);
  const int64_t blk = c / 64;
  const int kb = (int)(blk % kbs), nb = (int)(blk / kbs);
  const int n = nb * 32 + (l & 31), k = kb * 32 + (l >> 5) * 16;
  u32x4 v = {0, 0, 0, 0};
  if (n < N && k < K) v = *reinterpret_cast<const u32x4*>(W + (int64_t)n * K + k);  // K % 16 == 0
  P[c] = v;
}

// Large-problem kernel.  Measured on this part: a 16-byte LDS read of a whole wave occupies the CU's LDS pipe for 16
// cycles (64 B/clk/CU) while one v_mfma_i32_32x32x32_i8 occupies a SIMD for 32, so a wave that pulls both operands of a
// 64x64 tile through LDS is LDS-bound at under half the matrix rate.  Here only the activation tile goes through LDS;
// the four waves of a workgroup sit side by side along N, each owns (32 TM) x (32 TN) outputs and fetches ITS weight
// operands straight from global memory into registers in MFMA layout, one K step (128 bytes) ahead: every operand
// register is reloaded for the next step right after its last use.  PK: weights in the prepacked layout above; else
// the plain [N][K] matrix with K % 128 == 0.
// The weights are the MFMA's first operand, so that a lane ends up with four CONSECUTIVE output columns per row.
// Scheduling barriers pin the hand-made software pipeline: left alone, the compiler sinks all global loads to the end
// of the loop body and exposes their latency.
// WPS: waves per SIMD the register budget is held to (workgroups of 4 waves: WPS workgroups per CU).
template <int TM, int TN, bool PK, int WPS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WPS, WPS))) void w8a8_gemm_nsplit_kernel(W8A8Args a) {
  constexpr int BK = 128, LDK = 144, KS = BK / 32;
  constexpr int BM = TM * 32, WN = TN * 32, BN = 4 * WN;
  constexpr int CA = BM * (BK / 16) / 256;  // 16-byte activation chunks per thread and K step
  constexpr int STAGE = BM * LDK;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, hi = lane >> 5;
  const int tilesN = (a.N + BN - 1) / BN, tilesM = (a.M + BM - 1) / BM;
  const int total = tilesM * tilesN;
  int tile = blockIdx.x;
  if (total % 8 == 0) tile = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;  // one run of tiles per XCD ...
  const int m0 = (tile % tilesM) * BM, n0 = (tile / tilesM) * BN;              // ... that shares a slice of the weights

  // Rows past the end are clamped to the last row (their results are never stored).  Activation bytes past K belong to
  // the next row and meet zero weights (PK) or do not occur (K % 128 == 0); reads past the buffers return zero.
  const int Kw = PK ? (int)w8a8_packed_k(a.K) : a.K;
  const int64_t wbytes = PK ? w8a8_packed_n(a.N) * Kw : (int64_t)a.N * a.K;
  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.A), 0, (uint32_t)((int64_t)a.M * a.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t rW = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.W), 0, (uint32_t)wbytes, 0x00020000);
  uint32_t offA[CA];
#pragma unroll
  for (int c = 0; c < CA; c++) {
    const int idx = tid + c * 256;
    offA[c] = (uint32_t)((int64_t)min(m0 + idx / 8, a.M - 1) * a.K + (idx % 8) * 16);
  }
  uint32_t offB[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int nrow = n0 + wave * WN + j * 32;
    offB[j] = PK ? (uint32_t)((int64_t)min(nrow, (int)w8a8_packed_n(a.N) - 32) * Kw + lane * 16)
                 : (uint32_t)((int64_t)min(nrow + lrow, a.N - 1) * a.K + hi * 16);
  }

  auto loadA = [&](int k0, u32x4 (&ga)[CA]) {
#pragma unroll
    for (int c = 0; c < CA; c++) ga[c] = __builtin_amdgcn_raw_buffer_load_b128(rA, offA[c], k0, 0);
  };
  auto storeA = [&](int buf, const u32x4 (&ga)[CA]) {
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const int idx = tid + c * 256;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + (idx / 8) * LDK + (idx % 8) * 16) = ga[c];
    }
  };
  auto loadB = [&](int k0, int ks, int j) -> v4i {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rW, offB[j], (k0 + ks * 32) * (PK ? 32 : 1), 0);
    return v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
  };
  auto readA = [&](int buf, int ks, v4i (&fa)[TM]) {
#pragma unroll
    for (int i = 0; i < TM; i++)
      fa[i] = *reinterpret_cast<const v4i*>(smem + buf * STAGE + (i * 32 + lrow) * LDK + ks * 32 + hi * 16);
  };

  v16i acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; j++)
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[j][i][r] = 0;

  const int KT = Kw / BK;
  u32x4 ga[CA];
  v4i fb[KS][TN];
  v4i fa[2][TM];
  loadA(0, ga);
#pragma unroll
  for (int ks = 0; ks < KS; ks++)
#pragma unroll
    for (int j = 0; j < TN; j++) fb[ks][j] = loadB(0, ks, j);
  storeA(0, ga);
  __syncthreads();
  readA(0, 0, fa[0]);

  for (int kt = 0; kt < KT; kt++) {
    const int buf = kt & 1, k1 = (kt + 1) * BK;
    loadA(k1, ga);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (ks < KS - 1) {
        readA(buf, ks + 1, fa[(ks + 1) & 1]);  // the next sub-step's activations while this one's MFMAs run
      } else {
        storeA(buf ^ 1, ga);  // free since the previous barrier; its loads were issued a whole K step ago
        __syncthreads();
        readA(buf ^ 1, 0, fa[(ks + 1) & 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int i = 0; i < TM; i++)
          acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ks][j], fa[ks & 1][i], acc[j][i], 0, 0, 0);
        fb[ks][j] = loadB(k1, ks, j);  // the operand of the next K step, into the register that just became free
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  __syncthreads();  // all LDS reads done before the scales overwrite the tiles

  // acc[j][i][4g+e] = C[m0 + 32i + lrow][n0 + wave*WN + 32j + 8g + 4hi + e]
  float* sXs = reinterpret_cast<float*>(smem);
  float* sWs = sXs + BM;
  float* sBi = sWs + BN;
  for (int i = tid; i < BM; i += 256) sXs[i] = (a.xs && m0 + i < a.M) ? a.xs[m0 + i] : 0.f;
  for (int i = tid; i < BN; i += 256) {
    sWs[i] = (a.ws && n0 + i < a.N) ? a.ws[n0 + i] : 0.f;
    sBi[i] = (a.bias && n0 + i < a.N) ? a.bias[n0 + i] : 0.f;
  }
  __syncthreads();
  // Full tiles with bf16 output only take a branch-free path: the column scales sit in registers, and each 32-row slab
  // of results is turned through LDS so that a wave stores whole rows of the workgroup's BN columns (runs of whole
  // cache lines, 16 bytes per lane).
  constexpr int ROWB = 2 * BN + 16;
  unsigned char* patch = smem + 4096;
  static_assert((BM + 2 * BN) * 4 <= 4096, "scales overlap the store patch");
  const bool full = m0 + BM <= a.M && n0 + BN <= a.N && a.N % 8 == 0 && reinterpret_cast<uintptr_t>(a.C) % 16 == 0;
  if (full && a.C && !a.acc) {
    f32x4 ws4[TN][4], bi4[TN][4];
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        ws4[j][g] = *reinterpret_cast<const f32x4*>(&sWs[wave * WN + j * 32 + 8 * g + 4 * hi]);
        bi4[j][g] = *reinterpret_cast<const f32x4*>(&sBi[wave * WN + j * 32 + 8 * g + 4 * hi]);
      }
    const bool has_bias = a.bias != nullptr;
    constexpr int CPR = BN / 8;  // 16-byte pieces per row
    static_assert((8 * CPR) % 64 == 0, "a wave stores whole rows");
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const float xsm = sXs[i * 32 + lrow];
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          float f[4];
#pragma unroll
          for (int e = 0; e < 4; e++) f[e] = (float)acc[j][i][4 * g + e] * (ws4[j][g][e] * xsm);
          if (has_bias) {
#pragma unroll
            for (int e = 0; e < 4; e++) f[e] += bi4[j][g][e];
          }
          *reinterpret_cast<uint2*>(patch + lrow * ROWB + (wave * WN + j * 32 + 8 * g + 4 * hi) * 2) =
              uint2{pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3])};
        }
      __syncthreads();
#pragma unroll
      for (int t = 0; t < 8 * CPR / 64; t++) {  // wave w stores rows 8w .. 8w+7
        const int c = lane + 64 * t;
        const int row = wave * 8 + c / CPR, cc = c % CPR;
        const u32x4 v = *reinterpret_cast<const u32x4*>(patch + row * ROWB + cc * 16);
        *reinterpret_cast<u32x4*>(&a.C[(int64_t)(m0 + i * 32 + row) * a.N + n0 + cc * 8]) = v;
      }
      if (i + 1 < TM) __syncthreads();
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; i++) {
    const int m = m0 + i * 32 + lrow;
    const float xsm = sXs[i * 32 + lrow];
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int cn = wave * WN + j * 32 + 8 * g + 4 * hi;
        const int n = n0 + cn;
        const f32x4 ws4 = *reinterpret_cast<const f32x4*>(&sWs[cn]);
        const f32x4 bi4 = *reinterpret_cast<const f32x4*>(&sBi[cn]);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          if (m < a.M && n + e < a.N) {
            const int v = acc[j][i][4 * g + e];
            if (a.acc) a.acc[(int64_t)m * a.N + n + e] = v;
            if (a.C) {
              float f = (float)v * (ws4[e] * xsm);
              if (a.bias) f += bi4[e];
              a.C[(int64_t)m * a.N + n + e] = (uint16_t)pack_bf16(f, 0.f);
            }
          }
        }
      }
    }
  }
}

template <int TM, int TN, bool PK, int WPS>
static int launch_w8a8_nsplit(const W8A8Args& a, hipStream_t st) {
  constexpr int BM = TM * 32, BN = 4 * TN * 32;
  constexpr size_t stage = 2 * (size_t)BM * 144, patch = 4096 + 32 * (2 * (size_t)BN + 16);
  const size_t lds = stage > patch ? stage : patch;
  const unsigned grid = (unsigned)(((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN));
  hipLaunchKernelGGL((w8a8_gemm_nsplit_kernel<TM, TN, PK, WPS>), dim3(grid), dim3(256), lds, st, a);
  return (int)hipGetLastError();
}

static int g_w8a8_ntile = 0;  // weights-from-global kernel: 0 = heuristic, 1 = 128x384, 2 = 64x384, 3 = 128x128, 4 = 64x128, 5 = 128x256

// Tile choice for the weights-from-global kernel: the biggest tile that still gives every CU work.
template <bool PK>
static int launch_w8a8_nsplit_auto(const W8A8Args& a, hipStream_t st) {
  auto tiles = [&](int bm, int bn) { return (int64_t)((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn); };
  int t = g_w8a8_ntile;
  if (!t) {
    if (a.M > 64 && tiles(128, 384) >= 192) t = 1;
    else if (tiles(64, 384) >= 192 || a.N <= 128) t = 2;
    else if (a.M > 64 && tiles(128, 128) >= 192) t = 3;
    else t = 4;
  }
  switch (t) {
    case 1: return launch_w8a8_nsplit<4, 3, PK, 1>(a, st);
    case 2: return launch_w8a8_nsplit<2, 3, PK, 2>(a, st);
    case 3: return launch_w8a8_nsplit<4, 1, PK, 2>(a, st);
    case 5: return launch_w8a8_nsplit<4, 2, PK, 2>(a, st);
    default: return launch_w8a8_nsplit<2, 1, PK, 2>(a, st);
  }
}

template <int BM, int BN, int WM, int WN, int D>
static int launch_w8a8(const W8A8Args& a, hipStream_t st) {
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  const size_t lds = 2 * (size_t)(BM + BN) * 64;
  const unsigned grid = (unsigned)(((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN));
  auto kern = w8a8_gemm_kernel<BM, BN, WM, WN, D>;
  if (lds > 64 * 1024)
    HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), lds, st, a);
  return (int)hipGetLastError();
}

static int g_w8a8_tile = 0;  // 0 = heuristic, 1 = 256x192, 2 = 128x128, 3 = 64x64, 4 = weights-from-global tiles

}  // namespace mllmhip

using namespace mllmhip;

MLLM_API int mllm_hip_w8a8_set_tuning(int tile) {
  if (tile < 0 || tile > 4) return MLLM_HIP_E_BADARG;
  g_w8a8_tile = tile;
  return 0;
}

// ---- decode: up to eight tokens against the prepacked weights --------------------------------------------------------------
// The tile kernels above spend a 128-row tile on a decode token and leave most CUs idle (9728 x 2560 at one token: 16 us;
// 2560 x 9728: 41 us).  Here a workgroup takes one block row of the packed matrix (32 weight rows) and its waves stride over
// the K blocks, eight 1 KB blocks requested per wave before the first is multiplied (the first batch ahead of the copy of
// the tokens' codes into LDS, which it does not depend on); v_dot4_i32_i8 sums, the two K halves of a block met by a wave
// shuffle, the waves through LDS.  Integer sums are exact: the epilogue is the tile kernels' and so are the bits.
constexpr int W8G_MAXW = 16;
template <int MT>
__global__ __launch_bounds__(W8G_MAXW * 64) void w8a8_gemv_packed_kernel(W8A8Args a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int Kp = (int)w8a8_packed_k(a.K), kbs = Kp / 32;
  u32x4* sx = reinterpret_cast<u32x4*>(smem);                          // [MT][Kp / 16] the tokens' codes, zero past K and M
  int* s_part = reinterpret_cast<int*>(smem + (size_t)MT * Kp);        // [wave][MT][32]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int nb = blockIdx.x;
  const u32x4* P = reinterpret_cast<const u32x4*>(a.W) + (size_t)nb * kbs * 64 + lane;
  constexpr int UB = 8;
  u32x4 wv[UB];
  auto load_batch = [&](int kb0) {
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int kb = kb0 + u * nwaves;
      wv[u] = u32x4{0u, 0u, 0u, 0u};
      if (kb < kbs) wv[u] = P[(size_t)kb * 64];
    }
  };
  load_batch(wave);
  const int cpr = Kp / 16;  // 16-byte pieces per token
  for (int i = tid; i < MT * cpr; i += nthreads) {
    const int m = i / cpr, c = i - m * cpr;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (m < a.M && c * 16 < a.K) v = *reinterpret_cast<const u32x4*>(a.A + (size_t)m * a.K + c * 16);  // K % 16 == 0
    sx[i] = v;
  }
  __syncthreads();
  int acc[MT];
#pragma unroll
  for (int m = 0; m < MT; m++) acc[m] = 0;
  for (int kb0 = wave; kb0 < kbs; kb0 += nwaves * UB) {
    if (kb0 != wave) load_batch(kb0);
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int kb = kb0 + u * nwaves;
      if (kb < kbs) {  // uniform
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const u32x4 xv = sx[m * cpr + kb * 2 + h];
          int s = acc[m];
          s = __builtin_amdgcn_sdot4((int)wv[u].x, (int)xv.x, s, false);
          s = __builtin_amdgcn_sdot4((int)wv[u].y, (int)xv.y, s, false);
          s = __builtin_amdgcn_sdot4((int)wv[u].z, (int)xv.z, s, false);
          s = __builtin_amdgcn_sdot4((int)wv[u].w, (int)xv.w, s, false);
          acc[m] = s;
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MT; m++) {
    acc[m] += __shfl_xor(acc[m], 32, 64);
    if (h == 0) s_part[(wave * MT + m) * 32 + r] = acc[m];
  }
  __syncthreads();
  for (int i = tid; i < MT * 32; i += nthreads) {
    const int m = i >> 5, n = nb * 32 + (i & 31);
    if (m < a.M && n < a.N) {
      int v = 0;
      for (int w = 0; w < nwaves; w++) v += s_part[(w * MT + m) * 32 + (i & 31)];
      if (a.acc) a.acc[(int64_t)m * a.N + n] = v;
      if (a.C) {
        float f = (float)v * (a.ws[n] * a.xs[m]);
        if (a.bias) f += a.bias[n];
        a.C[(int64_t)m * a.N + n] = (uint16_t)pack_bf16(f, 0.f);
      }
    }
  }
}
// The same walk with the sums on the matrix cores: the 16 bytes a lane holds of a packed block ARE its operand of one
// v_mfma_i32_32x32x32_i8 (row l % 32, sixteen consecutive k of half l / 32), the other operand the same sixteen k of token
// l % 32 from LDS (lanes past the MT tokens staged pass zeros): one matrix instruction per block whatever the token count, no
// vector arithmetic in the loop.  The tokens' codes sit in LDS in runs of cb K blocks (all of them where the rows fit whole).
// acc[4g + e] = C[token l % 32][row 8g + 4 (l / 32) + e]; integer sums, so the same bits as every other form.
template <int MT>
__global__ __launch_bounds__(W8G_MAXW * 64) void w8a8_gemv_mfma_packed_kernel(W8A8Args a, int cb) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int Kp = (int)w8a8_packed_k(a.K), kbs = Kp / 32;
  u32x4* sx = reinterpret_cast<u32x4*>(smem);   // [MT][2 cb] the tokens' codes of the cb blocks in work, zero past K and M
  int* s_part = reinterpret_cast<int*>(smem);   // [wave][MT][32], after the loop
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int nb = blockIdx.x;
  const u32x4* P = reinterpret_cast<const u32x4*>(a.W) + (size_t)nb * kbs * 64 + lane;
  constexpr int UB = 8;
  u32x4 wv[UB];
  auto load_batch = [&](int kb0, int c1) {
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int kb = kb0 + u * nwaves;
      wv[u] = u32x4{0u, 0u, 0u, 0u};
      if (kb < c1) wv[u] = P[(size_t)kb * 64];
    }
  };
  const int cpr = cb * 2;  // 16-byte pieces per token in LDS
  v16i acc;
#pragma unroll
  for (int j = 0; j < 16; j++) acc[j] = 0;
  const bool staged = r < MT;
  const u32x4* sxr = sx + (size_t)(staged ? r : 0) * cpr + h;
  for (int c0 = 0; c0 < kbs; c0 += cb) {
    const int c1 = min(c0 + cb, kbs);
    load_batch(c0 + wave, c1);  // ahead of the copy of the codes
    if (c0) __syncthreads();    // every wave is done with the previous run's codes
    for (int i = tid; i < MT * cpr; i += nthreads) {
      const int m = i / cpr, c = i - m * cpr, gc = c0 * 2 + c;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (m < a.M && gc * 16 < a.K) v = *reinterpret_cast<const u32x4*>(a.A + (size_t)m * a.K + gc * 16);  // K % 16 == 0
      sx[i] = v;
    }
    __syncthreads();
    for (int kb0 = c0 + wave; kb0 < c1; kb0 += nwaves * UB) {
      if (kb0 != c0 + wave) load_batch(kb0, c1);
#pragma unroll
      for (int u = 0; u < UB; u++) {
        const int kb = kb0 + u * nwaves;
        if (kb < c1) {  // uniform
          u32x4 xv = {0u, 0u, 0u, 0u};
          if (staged) xv = sxr[(kb - c0) * 2];
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(v4i, wv[u]), __builtin_bit_cast(v4i, xv), acc, 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();  // every wave is done with the codes
  if (staged) {
#pragma unroll
    for (int g = 0; g < 4; g++)
      *reinterpret_cast<v4i*>(&s_part[(wave * MT + r) * 32 + 8 * g + 4 * h]) = v4i{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
  }
  __syncthreads();
  for (int i = tid; i < MT * 32; i += nthreads) {
    const int m = i >> 5, n = nb * 32 + (i & 31);
    if (m < a.M && n < a.N) {
      int v = 0;
      for (int w = 0; w < nwaves; w++) v += s_part[(w * MT + m) * 32 + (i & 31)];
      if (a.acc) a.acc[(int64_t)m * a.N + n] = v;
      if (a.C) {
        float f = (float)v * (a.ws[n] * a.xs[m]);
        if (a.bias) f += a.bias[n];
        a.C[(int64_t)m * a.N + n] = (uint16_t)pack_bf16(f, 0.f);
      }
    }
  }
}
// false where the kernels above do not apply
static int g_w8a8_decode = 1;  // 0: the tile kernels also for a few tokens (comparison runs and tests)
static int g_w8a8_decode_mfma_from = 5;  // token counts from this one up take the matrix-core form (two to four: the dot form is
                                         // faster, 9728 x 2560 at four tokens 11.3 against 12.9 us)
static bool launch_w8a8_gemv_packed(const W8A8Args& a, hipStream_t st, int* rc) {
  if (a.M > 32 || !g_w8a8_decode) return false;
  const int Kp = (int)w8a8_packed_k(a.K), kbs = Kp / 32;
  const int nwaves = kbs >= 32 ? W8G_MAXW : 4;
  if (a.M >= g_w8a8_decode_mfma_from) {
    // 17 to 32 tokens: every lane reads its own token's codes from LDS, and the tile kernels win where N gives them enough
    // tiles (9728 x 2560 at 32 tokens: 21.6 us here, 17.1 there; 2560 x 9728: 28.4 against 43.5)
    if (a.M > 16 && a.N > 8192) return false;
    const int MT = a.M <= 8 ? 8 : (a.M <= 16 ? 16 : 32);
    const int cap = 152 * 1024 / (MT * 32);  // K blocks of MT tokens in 152 KB
    const int cb = kbs < cap ? kbs : cap;
    const size_t x_bytes = (size_t)MT * cb * 32, part_bytes = (size_t)nwaves * MT * 32 * 4;
    const size_t lds = x_bytes > part_bytes ? x_bytes : part_bytes;
    const dim3 grid((unsigned)(w8a8_packed_n(a.N) / 32));
    auto go = [&](auto kern) {
      if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return (int)hipGetLastError();
      hipLaunchKernelGGL(kern, grid, dim3(nwaves * 64), lds, st, a, cb);
      return (int)hipGetLastError();
    };
    *rc = MT == 8 ? go(w8a8_gemv_mfma_packed_kernel<8>) : MT == 16 ? go(w8a8_gemv_mfma_packed_kernel<16>) : go(w8a8_gemv_mfma_packed_kernel<32>);
    return true;
  }
  if (a.M > 8) return false;
  const int MT = a.M <= 1 ? 1 : (a.M <= 2 ? 2 : (a.M <= 4 ? 4 : 8));
  const size_t lds = (size_t)MT * Kp + (size_t)nwaves * MT * 32 * 4;
  if (lds > 160 * 1024) return false;
  const dim3 grid((unsigned)(w8a8_packed_n(a.N) / 32));
  auto go = [&](auto kern) {
    if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return (int)hipGetLastError();
    hipLaunchKernelGGL(kern, grid, dim3(nwaves * 64), lds, st, a);
    return (int)hipGetLastError();
  };
  *rc = MT == 1 ? go(w8a8_gemv_packed_kernel<1>) : MT == 2 ? go(w8a8_gemv_packed_kernel<2>) : MT == 4 ? go(w8a8_gemv_packed_kernel<4>) : go(w8a8_gemv_packed_kernel<8>);
  return true;
}
MLLM_API int mllm_hip_w8a8_set_decode(int gemv) {
  if (gemv != 0 && gemv != 1) return MLLM_HIP_E_BADARG;
  g_w8a8_decode = gemv;
  return 0;
}
MLLM_API int mllm_hip_w8a8_set_decode_mfma_from(int tokens) {
  if (tokens < 1 || tokens > 33) return MLLM_HIP_E_BADARG;
  g_w8a8_decode_mfma_from = tokens;
  return 0;
}

MLLM_API int mllm_hip_w8a8_nsplit_set_tuning(int tile) {
  if (tile < 0 || tile > 5) return MLLM_HIP_E_BADARG;
  g_w8a8_ntile = tile;
  return 0;
}

MLLM_API int mllm_hip_per_token_quant_int8(const void* x, int x_dtype, int8_t* q, float* scale, int64_t M, int64_t K,
                                           void* stream) {
  if (!x || !q || !scale || M <= 0 || K <= 0 || (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16))
    return MLLM_HIP_E_BADARG;
  if (M > INT32_MAX || K > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (K % 8 == 0 && (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(q) % 8)) return MLLM_HIP_E_ALIGN;
  const int ni = (K % 8 == 0 && K >= 8 && K <= 4 * 2048) ? (K <= 2048 ? 1 : (K <= 4096 ? 2 : 4)) : 0;
#define PTQ(XT_, NI_) \
  hipLaunchKernelGGL((per_token_quant_kernel<XT_, NI_>), dim3((unsigned)M), dim3(256), 0, (hipStream_t)stream, x, q, scale, (int)K)
#define PTQ_T(XT_)          \
  if (ni == 1) PTQ(XT_, 1); \
  else if (ni == 2) PTQ(XT_, 2); \
  else if (ni == 4) PTQ(XT_, 4); \
  else PTQ(XT_, 0)
  if (x_dtype == MLLM_HIP_F32) {
    PTQ_T(MLLM_HIP_F32);
  } else {
    PTQ_T(MLLM_HIP_BF16);
  }
#undef PTQ_T
#undef PTQ
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
    const int64_t mid = ((M + 127) / 128) * ((N + 127) / 128);
    // the 256x192 tile is compiled and tested but measured slower than 128x128
    tile = (K % 128 == 0 && mid >= 256) ? 4 : mid >= 128 ? 2 : 3;
  }
  if (tile == 4 && K % 128) tile = 2;
  switch (tile) {
    case 4: return launch_w8a8_nsplit_auto<false>(a, st);
    case 1: return launch_w8a8<256, 192, 128, 96, 4>(a, st);
    case 2: return launch_w8a8<128, 128, 64, 64, 4>(a, st);
    default: return launch_w8a8<64, 64, 32, 32, 2>(a, st);
  }
}

MLLM_API size_t mllm_hip_w8a8_packed_bytes(int64_t N, int64_t K) {
  if (N <= 0 || K <= 0) return 0;
  return (size_t)(w8a8_packed_n(N) * w8a8_packed_k(K));
}

MLLM_API int mllm_hip_w8a8_prepack(const int8_t* W, int64_t N, int64_t K, void* packed, void* stream) {
  if (!W || !packed || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (K % 16 || N > INT32_MAX || K > INT32_MAX || w8a8_packed_n(N) * w8a8_packed_k(K) >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(W) % 16 || reinterpret_cast<uintptr_t>(packed) % 16) return MLLM_HIP_E_ALIGN;
  const int64_t chunks = w8a8_packed_n(N) * w8a8_packed_k(K) / 16;
  hipLaunchKernelGGL(w8a8_prepack_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, (hipStream_t)stream, W,
                     reinterpret_cast<u32x4*>(packed), (int)N, (int)K, chunks);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_w8a8_gemm_packed(const int8_t* xq, const float* x_scale, const void* W_packed, const float* w_scale,
                                       const float* bias, void* out_bf16, int32_t* acc_out, int64_t M, int64_t N,
                                       int64_t K, void* stream) {
  if (!xq || !W_packed || M <= 0 || N <= 0 || K <= 0 || (!out_bf16 && !acc_out)) return MLLM_HIP_E_BADARG;
  if (out_bf16 && (!x_scale || !w_scale)) return MLLM_HIP_E_BADARG;
  if (K % 16) return MLLM_HIP_E_SHAPE;
  if (M * K >= ((int64_t)1 << 32) || w8a8_packed_n(N) * w8a8_packed_k(K) >= ((int64_t)1 << 32) || M > INT32_MAX || N > INT32_MAX)
    return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(xq) % 16 || reinterpret_cast<uintptr_t>(W_packed) % 16) return MLLM_HIP_E_ALIGN;
  W8A8Args a{xq, reinterpret_cast<const int8_t*>(W_packed), x_scale, w_scale, bias, (uint16_t*)out_bf16, acc_out, (int)M, (int)N, (int)K};
  int rc = 0;
  if (launch_w8a8_gemv_packed(a, (hipStream_t)stream, &rc)) return rc;  // up to 32 tokens
  return launch_w8a8_nsplit_auto<true>(a, (hipStream_t)stream);
}

MLLM_API size_t mllm_hip_w8a8_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0) return 0;
  return align_up((size_t)M * K, 256) + align_up((size_t)M * 4, 256);
}

MLLM_API int mllm_hip_w8a8_linear(const void* x, int x_dtype, const int8_t* W, const float* w_scale, const float* bias,
                                  void* out_bf16, int64_t M, int64_t N, int64_t K, void* workspace, void* stream) {
  // everything the second step would reject is rejected before the first one is launched
  if (!workspace || !W || !w_scale || !out_bf16 || N <= 0) return MLLM_HIP_E_BADARG;
  if (K > 0 && K % 16) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(workspace) % 16 || reinterpret_cast<uintptr_t>(W) % 16) return MLLM_HIP_E_ALIGN;
  int8_t* q = reinterpret_cast<int8_t*>(workspace);
  float* xs = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + align_up((size_t)M * K, 256));
  int rc = mllm_hip_per_token_quant_int8(x, x_dtype, q, xs, M, K, stream);
  if (rc) return rc;
  return mllm_hip_w8a8_gemm(q, xs, W, w_scale, bias, out_bf16, nullptr, M, N, K, stream);
}

MLLM_API int mllm_hip_w8a8_linear_packed(const void* x, int x_dtype, const void* W_packed, const float* w_scale,
                                         const float* bias, void* out_bf16, int64_t M, int64_t N, int64_t K,
                                         void* workspace, void* stream) {
  // everything the second step would reject is rejected before the first one is launched
  if (!workspace || !W_packed || !w_scale || !out_bf16 || N <= 0) return MLLM_HIP_E_BADARG;
  if (K > 0 && K % 16) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(workspace) % 16 || reinterpret_cast<uintptr_t>(W_packed) % 16) return MLLM_HIP_E_ALIGN;
  int8_t* q = reinterpret_cast<int8_t*>(workspace);
  float* xs = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + align_up((size_t)M * K, 256));
  int rc = mllm_hip_per_token_quant_int8(x, x_dtype, q, xs, M, K, stream);
  if (rc) return rc;
  return mllm_hip_w8a8_gemm_packed(q, xs, W_packed, w_scale, bias, out_bf16, nullptr, M, N, K, stream);
}
