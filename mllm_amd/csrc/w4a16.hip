// W4A16 Linear for prefill on gfx950: bf16 activations x uint4 weights with per-group fp16 scales and uint4 zero-points
// (group size a multiple of 64 along K, 128 in the checkpoints), fp32 accumulation, bf16 output.
//
// Semantics (the reference runs this on CUDA through Marlin; restated in closed form):
//   dequantization      mllm-kernel/mllm_kernel/cuda/csrc/gemm/marlin/dequant.h:18-26 (q - zp), marlin_template.h:153-168 (x scale)
//   checkpoint scheme   pymllm/quantization/methods/awq_marlin.py:274-449
//   test formula        mllm-kernel/tests/test_gptq_marlin.py:143-146
//   w_bf16[n][k] = bf16_rne( float(q[n][k] - zp[n][k/g]) * fp32(scale[n][k/g]) )   (the product is exact in fp32: <= 16 bits)
//   C[m][n]      = bf16_rne( sum_k A[m][k] * w_bf16[n][k]  (+ bias[n]) ),  fp32 accumulate on the matrix cores
// Storage: qw uint8 [N][K/2], element 2j in the low nibble of byte j; scales fp16 [N][K/g]; zero-points uint8
// [N][ceil(K/g/2)], group 2i in the low nibble of byte i.
//
// Weights are fetched packed (16 bytes = 32 elements per lane), dequantized once per workgroup in registers and staged
// as bf16 in LDS next to the activation tile; the matrix cores read both operands from LDS.
#include "qcommon.h"

namespace mllmhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

// eight elements of one packed dword -> four dwords of bf16 pairs, element order kept.
// (q - zp) * s == fma(q, s, -zp*s) exactly: both products and their sum need at most 16 significant bits.
// One conversion (v_cvt_f32_ubyteN reads byte N of a dword), one fma and half a pack per element.  The empty asm hides
// from the optimizer that only four bits of each byte can be set; knowing it, the compiler replaces mask + byte
// conversion by one bit-field extract PER ELEMENT plus the conversion.
__device__ __forceinline__ void dequant8(uint32_t w, float s, float nzs, uint32_t (&out)[4]) {
  uint32_t lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu;  // bytes: elements 0,2,4,6 / 1,3,5,7
  asm("" : "+v"(lo));
  asm("" : "+v"(hi));
#pragma unroll
  for (int b = 0; b < 4; b++) {
    const float e0 = fmaf((float)((lo >> (8 * b)) & 0xffu), s, nzs);
    const float e1 = fmaf((float)((hi >> (8 * b)) & 0xffu), s, nzs);
    out[b] = pack_bf16(e0, e1);
  }
}

struct W4A16Args {
  const uint16_t* A;    // bf16 [M][K]
  const uint8_t* qw;    // [N][K/2]
  const uint16_t* s;    // fp16 [N][G]
  const uint8_t* zp;    // [N][(G+1)/2]
  const uint16_t* bias; // bf16 [N] or null
  uint16_t* C;          // bf16 [M][N]
  int M, N, K, group;
};

// Workgroup tile BM x BN, K step 64 elements; waves (BM/WM) x (BN/WN), each WM x WN as 32x32 tiles of
// v_mfma_f32_32x32x16_bf16 (every lane supplies 8 consecutive k of one row of A and of one row of W).
// LDS rows hold 64 bf16 = 128 bytes, padded to 144 so that 16-byte reads of 16 neighbouring rows hit distinct banks.
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void w4a16_gemm_kernel(W4A16Args a) {
  constexpr int BK = 64, LDK = 144;
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  constexpr int CA = BM * 8 / NT;                 // 16-byte activation chunks (8 bf16) per thread and K step
  constexpr int CB = (BN * 2 + NT - 1) / NT;      // 16-byte packed weight chunks (32 elements) per thread and K step
  static_assert(BM * 8 % NT == 0, "activation tile must split evenly over the threads");
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int STAGE = (BM + BN) * LDK;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / (BN / WN), wn = wave % (BN / WN);
  const int G = a.K / a.group, zpb = (G + 1) / 2;

  const int tilesN = (a.N + BN - 1) / BN, tilesM = (a.M + BM - 1) / BM;
  const int total = tilesM * tilesN;
  int tile = blockIdx.x;
  if (total % 8 == 0) tile = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;  // one run of tiles per XCD
  const int m0 = (tile / tilesN) * BM, n0 = (tile % tilesN) * BN;

  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.A), 0, (uint32_t)((int64_t)a.M * a.K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rW = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.qw), 0, (uint32_t)((int64_t)a.N * a.K / 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rS = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.s), 0, (uint32_t)((int64_t)a.N * G * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rZ = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.zp), 0, (uint32_t)((int64_t)a.N * zpb), 0x00020000);

  // activation chunk c: row = idx / 8, 16-byte column = idx % 8 ; weight chunk c: row = idx / 2, half = idx % 2
  uint32_t offA[CA];
#pragma unroll
  for (int c = 0; c < CA; c++) {
    const int idx = tid + c * NT, row = m0 + idx / 8;
    offA[c] = row < a.M ? (uint32_t)(((int64_t)row * a.K + (idx % 8) * 8) * 2) : 0xffffffffu;
  }
  int wrow[CB];
  bool wok[CB];
#pragma unroll
  for (int c = 0; c < CB; c++) {
    const int idx = tid + c * NT;
    wrow[c] = n0 + idx / 2;
    wok[c] = idx < BN * 2 && wrow[c] < a.N;
  }
  u32x4 gA[CA], gW[CB];
  uint16_t gS[CB];
  uint8_t gZ[CB];
  auto gload = [&](int k0) {
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const bool ok = offA[c] != 0xffffffffu && k0 + ((tid + c * NT) % 8) * 8 < a.K;
      gA[c] = __builtin_amdgcn_raw_buffer_load_b128(rA, ok ? offA[c] + (uint32_t)k0 * 2u : 0xffffffffu, 0, 0);
    }
    const int g = k0 / a.group;
#pragma unroll
    for (int c = 0; c < CB; c++) {
      const int half = (tid + c * NT) & 1;
      const bool ok = wok[c] && k0 + half * 32 < a.K;
      gW[c] = __builtin_amdgcn_raw_buffer_load_b128(rW, ok ? (uint32_t)(((int64_t)wrow[c] * a.K + k0 + half * 32) / 2) : 0xffffffffu, 0, 0);
      gS[c] = __builtin_amdgcn_raw_buffer_load_b16(rS, ok ? (uint32_t)(((int64_t)wrow[c] * G + g) * 2) : 0xffffffffu, 0, 0);
      gZ[c] = __builtin_amdgcn_raw_buffer_load_b8(rZ, ok ? (uint32_t)((int64_t)wrow[c] * zpb + (g >> 1)) : 0xffffffffu, 0, 0);
    }
  };
  auto sstore = [&](int buf, int k0) {
    unsigned char* base = smem + buf * STAGE;
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const int idx = tid + c * NT;
      *reinterpret_cast<u32x4*>(base + (idx / 8) * LDK + (idx % 8) * 16) = gA[c];
    }
    const int g = k0 / a.group;
#pragma unroll
    for (int c = 0; c < CB; c++) {
      const int idx = tid + c * NT;
      if (idx < BN * 2) {
        const float s = f16bits_to_f32(gS[c]);
        const float z = (float)((g & 1) ? (gZ[c] >> 4) : (gZ[c] & 15));
        const float nzs = -(z * s);  // exact: 4-bit integer times an 11-bit significand
        const uint32_t w[4] = {gW[c].x, gW[c].y, gW[c].z, gW[c].w};
        unsigned char* dst = base + (BM + idx / 2) * LDK + (idx & 1) * 64;
#pragma unroll
        for (int j = 0; j < 4; j++) {
          uint32_t o[4];
          dequant8(w[j], s, nzs, o);
          *reinterpret_cast<u32x4*>(dst + j * 16) = u32x4{o[0], o[1], o[2], o[3]};
        }
      }
    }
  };

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int KT = (a.K + BK - 1) / BK;
  gload(0);
  sstore(0, 0);
  __syncthreads();
  const int lrow = lane & 31, lk = (lane >> 5) * 16;
  for (int kt = 0; kt < KT; kt++) {
    const int buf = kt & 1;
    if (kt + 1 < KT) gload((kt + 1) * BK);
    const unsigned char* base = smem + buf * STAGE;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      bf16x8 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; i++)
        fa[i] = *reinterpret_cast<const bf16x8*>(base + (wm * WM + i * 32 + lrow) * LDK + ks * 32 + lk);
#pragma unroll
      for (int j = 0; j < TN; j++)
        fb[j] = *reinterpret_cast<const bf16x8*>(base + (BM + wn * WN + j * 32 + lrow) * LDK + ks * 32 + lk);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) sstore(buf ^ 1, (kt + 1) * BK);
    __syncthreads();
  }

  // epilogue.  32x32 accumulator layout: register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32.
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int n = n0 + wn * WN + j * 32 + lrow;
    const bool nok = n < a.N;
    const float bn = (nok && a.bias) ? bf16_to_f32(a.bias[n]) : 0.f;
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
        if (nok && m < a.M) {
          float f = acc[i][j][r];
          if (a.bias) f += bn;
          a.C[(int64_t)m * a.N + n] = f32_to_bf16(f);
        }
      }
    }
  }
}

// dequantized weight table (parity probe and the definition of "dequantized weight values")
__global__ void w4a16_dequant_kernel(const uint8_t* __restrict__ qw, const uint16_t* __restrict__ s,
                                     const uint8_t* __restrict__ zp, uint16_t* __restrict__ w, int64_t N, int64_t K, int group) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // one packed dword = 8 elements
  if (i >= N * K / 8) return;
  const int64_t n = i / (K / 8), k = (i % (K / 8)) * 8;
  const int G = (int)(K / group), zpb = (G + 1) / 2, g = (int)(k / group);
  const float sc = f16bits_to_f32(s[n * G + g]);
  const uint8_t zb = zp[n * zpb + (g >> 1)];
  const float z = (float)((g & 1) ? (zb >> 4) : (zb & 15));
  const uint32_t word = *reinterpret_cast<const uint32_t*>(qw + (n * K + k) / 2);
  uint32_t o[4];
  dequant8(word, sc, -(z * sc), o);
  *reinterpret_cast<u32x4*>(w + n * K + k) = u32x4{o[0], o[1], o[2], o[3]};
}

// ---------------------------------------------------------------------------------------------------------
// Prepacked weights + weights-from-global kernel (the fast path for prefill-sized M).
//
// Measured on this part: a 16-byte LDS read of a whole wave occupies the CU's LDS pipe for 16 cycles (64 B/clk/CU) while
// one v_mfma_f32_32x32x16_bf16 occupies a SIMD for 32, so a wave that pulls both operands of a 64x64 tile through LDS is
// LDS-bound at under half the matrix rate, and dequantized weights staged in LDS cost that bandwidth twice (write +
// reads).  Here only the activation tile goes through LDS.  The four waves of a workgroup sit side by side along N, each
// owns (32 TM) x (32 TN) outputs, loads ITS packed 4-bit weights straight from global memory (16 bytes per lane = the
// lane's operands of four MFMA K steps), dequantizes them in registers one MFMA step ahead of their use, and no weight
// is dequantized twice inside a workgroup.
//
// Packed layout (one pass over the checkpoint tensors, mllm_hip_w4a16_prepack):
//   q   [N/32][K/64][64 lanes][16 bytes]: lane l = (row l%32, half l/32); dword d of its 16 bytes holds the eight
//       elements k = 64 kb + 16 d + 8 (l/32) + 0..7 of its row, element e in nibble e (the checkpoint's own dword).
//       N is padded to 32 rows and K to 128 elements with zeros.
//   sz  [N/32][K/group][32 rows][2 floats]: (scale, -zero_point * scale) of the row's group, both exact in fp32.
__host__ __device__ inline int64_t w4a16_packed_n(int64_t N) { return (N + 31) / 32 * 32; }
__host__ __device__ inline int64_t w4a16_packed_k(int64_t K) { return (K + 127) / 128 * 128; }
__host__ __device__ inline int64_t w4a16_packed_qbytes(int64_t N, int64_t K) { return w4a16_packed_n(N) * w4a16_packed_k(K) / 2; }

__global__ __launch_bounds__(256) void w4a16_prepack_q_kernel(const uint8_t* __restrict__ qw, uint32_t* __restrict__ P, int N,
                                                              int K, int64_t words) {
  const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one dword = 8 elements of the packed matrix
  if (w >= words) return;
  const int kbs = (int)(w4a16_packed_k(K) / 64);
  const int d = (int)(w % 4), l = (int)((w / 4) % 64);
  const int64_t blk = w / 256;
  const int kb = (int)(blk % kbs), nb = (int)(blk / kbs);
  const int n = nb * 32 + (l & 31), k = kb * 64 + d * 16 + (l >> 5) * 8;
  uint32_t v = 0;
  if (n < N && k < K) v = *reinterpret_cast<const uint32_t*>(qw + ((int64_t)n * K + k) / 2);
  P[w] = v;
}
__global__ __launch_bounds__(256) void w4a16_prepack_sz_kernel(const uint16_t* __restrict__ s, const uint8_t* __restrict__ zp,
                                                               float2* __restrict__ SZ, int N, int G, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // (nb, g, row)
  if (i >= count) return;
  const int row = (int)(i % 32), g = (int)((i / 32) % G), nb = (int)(i / 32 / G);
  const int n = nb * 32 + row;
  float2 v = {0.f, 0.f};
  if (n < N) {
    const float sc = f16bits_to_f32(s[(int64_t)n * G + g]);
    const uint8_t zb = zp[(int64_t)n * ((G + 1) / 2) + (g >> 1)];
    const float z = (float)((g & 1) ? (zb >> 4) : (zb & 15));
    v = float2{sc, -(z * sc)};
  }
  SZ[i] = v;
}

struct W4A16PArgs {
  const uint16_t* A;     // bf16 [M][K]
  const uint8_t* P;      // packed q then sz
  const uint16_t* bias;  // bf16 [N] or null
  uint16_t* C;           // bf16 [M][N]
  int M, N, K, group;
};


// One output tile (32 TM rows from m0) x (128 TN columns from n0) by the four waves of a workgroup.
template <int TM, int TN, int BK>
__device__ __forceinline__ void w4a16_nsplit_tile(const W4A16PArgs& a, const int m0, const int n0, unsigned char* smem) {
  static_assert(BK == 64 || BK == 128, "K step of one or two 64-element weight blocks");
  constexpr int LDK = 2 * BK + 16, KS = BK / 16, NH = BK / 64;  // LDS row in bytes; MFMA steps; weight blocks per K step
  constexpr int CPRA = BK / 8;                                  // 16-byte activation chunks per row and K step
  constexpr int BM = TM * 32, WN = TN * 32, BN = 4 * WN;
  constexpr int CA = BM * (2 * BK / 16) / 256;  // 16-byte activation chunks per thread and K step
  static_assert(CA >= 1, "tile too small for 256 threads");
  constexpr int STAGE = BM * LDK;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, hi = lane >> 5;

  const int Kp = (int)w4a16_packed_k(a.K), kbs = Kp / 64, G = a.K / a.group, g64 = a.group / 64;
  const int64_t qbytes = w4a16_packed_qbytes(a.N, a.K);
  const int nbs = (int)(w4a16_packed_n(a.N) / 32);
  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.A), 0, (uint32_t)((int64_t)a.M * a.K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rQ = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.P), 0, (uint32_t)qbytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rS = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.P + qbytes), 0, (uint32_t)((int64_t)nbs * G * 256), 0x00020000);

  // activation chunk: row idx / CPRA, 16-byte column idx % CPRA.  Rows past M are clamped (never stored); columns past K
  // read as zeros so that the zero-padded tail of the weights never meets another row's values.
  uint32_t offA[CA];
  int colA[CA];
#pragma unroll
  for (int c = 0; c < CA; c++) {
    const int idx = tid + c * 256;
    colA[c] = (idx % CPRA) * 8;
    offA[c] = (uint32_t)(((int64_t)min(m0 + idx / CPRA, a.M - 1) * a.K + colA[c]) * 2);
  }
  uint32_t offQ[TN], offS[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int nb = min((n0 + wave * WN) / 32 + j, nbs - 1);
    offQ[j] = (uint32_t)((int64_t)nb * kbs * 1024 + lane * 16);
    offS[j] = (uint32_t)(((int64_t)nb * G * 32 + lrow) * 8);
  }
  auto loadA = [&](int k0, u32x4 (&ga)[CA]) {
#pragma unroll
    for (int c = 0; c < CA; c++)
      ga[c] = __builtin_amdgcn_raw_buffer_load_b128(rA, k0 + colA[c] < a.K ? offA[c] : 0xffffffffu, k0 * 2, 0);
  };
  auto storeA = [&](int buf, const u32x4 (&ga)[CA]) {
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const int idx = tid + c * 256;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + (idx / CPRA) * LDK + (idx % CPRA) * 16) = ga[c];
    }
  };
  auto readA = [&](int buf, int ks, bf16x8 (&fa)[TM]) {
#pragma unroll
    for (int i = 0; i < TM; i++)
      fa[i] = *reinterpret_cast<const bf16x8*>(smem + buf * STAGE + (i * 32 + lrow) * LDK + ks * 32 + hi * 16);
  };
  // the packed weights and the (scale, -zp*scale) pair of 64-element block kb of column block j
  auto loadQ = [&](int kb, int j) -> u32x4 { return __builtin_amdgcn_raw_buffer_load_b128(rQ, offQ[j], kb * 1024, 0); };
  auto loadS = [&](int kb, int j) -> u32x2 {
    return __builtin_amdgcn_raw_buffer_load_b64(rS, offS[j], min(kb / g64, G - 1) * 256, 0);
  };
  auto dequant = [&](const u32x4& q, const u32x2& sz, int d) -> bf16x8 {
    uint32_t o[4];
    dequant8(q[d], __uint_as_float(sz.x), __uint_as_float(sz.y), o);
    return __builtin_bit_cast(bf16x8, u32x4{o[0], o[1], o[2], o[3]});
  };

  v16f acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; j++)
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[j][i][r] = 0.f;

  const int KT = Kp / BK;
  u32x4 ga[CA];
  u32x4 rq[NH][TN];  // packed weights of the 64-element blocks of a K step
  u32x2 rs[NH][TN];
  bf16x8 fb[2][TN];  // dequantized operands of MFMA step ks (set ks & 1)
  bf16x8 fa[2][TM];
  loadA(0, ga);
#pragma unroll
  for (int h = 0; h < NH; h++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      rq[h][j] = loadQ(h, j);
      rs[h][j] = loadS(h, j);
    }
  storeA(0, ga);
  __syncthreads();
  readA(0, 0, fa[0]);
#pragma unroll
  for (int j = 0; j < TN; j++) fb[0][j] = dequant(rq[0][j], rs[0][j], 0);

  for (int kt = 0; kt < KT; kt++) {
    const int buf = kt & 1, k1 = (kt + 1) * BK;
    loadA(k1, ga);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (ks < KS - 1) {
        readA(buf, ks + 1, fa[(ks + 1) & 1]);  // the next step's activations while this one's MFMAs run
      } else {
        storeA(buf ^ 1, ga);  // free since the previous barrier; its loads were issued a whole K step ago
        __syncthreads();
        readA(buf ^ 1, 0, fa[(ks + 1) & 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
      const int nh = ((ks + 1) / 4) % NH, nd = (ks + 1) % 4;  // block and dword of the NEXT MFMA step's weights
#pragma unroll
      for (int j = 0; j < TN; j++) {
        // One wave per SIMD issues in order: the dequantization of the next step's operand (23 VALU instructions) is
        // cut into TM pieces, one in the shadow of each MFMA (32 cycles), and pinned there; left to the scheduler, the
        // MFMAs queue up back to back and the matrix pipe idles behind them while the VALU work runs.
        uint32_t lo = rq[nh][j][nd] & 0x0f0f0f0fu, hi = (rq[nh][j][nd] >> 4) & 0x0f0f0f0fu;
        asm("" : "+v"(lo));
        asm("" : "+v"(hi));
        const float sc = __uint_as_float(rs[nh][j].x), nzs = __uint_as_float(rs[nh][j].y);
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < TM; i++) {
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[ks & 1][j], fa[ks & 1][i], acc[j][i], 0, 0, 0);
#pragma unroll
          for (int b = i * 4 / TM; b < (i + 1) * 4 / TM; b++)
            o[b] = pack_bf16(fmaf((float)((lo >> (8 * b)) & 0xffu), sc, nzs), fmaf((float)((hi >> (8 * b)) & 0xffu), sc, nzs));
          __builtin_amdgcn_sched_barrier(0);
        }
        fb[(ks + 1) & 1][j] = __builtin_bit_cast(bf16x8, u32x4{o[0], o[1], o[2], o[3]});
        if (nd == 3) {  // last dword of that half consumed: fetch the same half of the next K step into its registers
          rq[nh][j] = loadQ((kt + 1) * NH + nh, j);
          rs[nh][j] = loadS((kt + 1) * NH + nh, j);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  __syncthreads();  // all LDS reads done before the epilogue reuses the tiles

  // acc[j][i][4g+e] = C[m0 + 32i + lrow][n0 + wave*WN + 32j + 8g + 4hi + e]
  float* sBi = reinterpret_cast<float*>(smem);
  for (int i = tid; i < BN; i += 256) sBi[i] = (a.bias && n0 + i < a.N) ? bf16_to_f32(a.bias[n0 + i]) : 0.f;
  __syncthreads();
  constexpr int ROWB = 2 * BN + 16;
  unsigned char* patch = smem + 4096;
  static_assert(BN * 4 <= 4096, "bias overlaps the store patch");
  const bool has_bias = a.bias != nullptr;
  const bool full = m0 + BM <= a.M && n0 + BN <= a.N && a.N % 8 == 0 && reinterpret_cast<uintptr_t>(a.C) % 16 == 0;
  if (full) {
    // branch-free path: each 32-row slab of results is turned through LDS so that a wave stores whole rows of the
    // workgroup's BN columns (runs of whole cache lines, 16 bytes per lane)
    f32x4 bi4[TN][4];
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) bi4[j][g] = *reinterpret_cast<const f32x4*>(&sBi[wave * WN + j * 32 + 8 * g + 4 * hi]);
    constexpr int CPR = BN / 8;  // 16-byte pieces per row
    static_assert((8 * CPR) % 64 == 0, "a wave stores whole rows");
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          float f[4];
#pragma unroll
          for (int e = 0; e < 4; e++) f[e] = acc[j][i][4 * g + e];
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
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int cn = wave * WN + j * 32 + 8 * g + 4 * hi;
        const f32x4 bi4 = *reinterpret_cast<const f32x4*>(&sBi[cn]);
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (m < a.M && n0 + cn + e < a.N) {
            float f = acc[j][i][4 * g + e];
            if (has_bias) f += bi4[e];
            a.C[(int64_t)m * a.N + n0 + cn + e] = (uint16_t)pack_bf16(f, 0.f);
          }
      }
  }
}

// Tile schedule.  Full tiles (32 TM rows) cover the first `big_cols` column tiles, half-height tiles the remaining column
// tiles.  The host picks big_cols so that the full tiles fill whole rounds of the chip's workgroup slots and the remainder,
// which would otherwise occupy a whole further round at a fraction of the chip, runs as twice as many tiles of half the
// duration; the half-height tiles are the FIRST workgroups of the grid (2048 x 9728 x 2560: 108 -> 101 us; as the last
// workgroups 107).
// WPS: waves per SIMD the register budget is held to (workgroups of 4 waves: WPS workgroups per CU).
template <int TM, int TN, int BK, int WPS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WPS, WPS))) void w4a16_gemm_nsplit_kernel(W4A16PArgs a, int big_cols) {
  constexpr int BM = TM * 32, BN = 4 * TN * 32;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tilesM = (a.M + BM - 1) / BM;
  const int nbig = tilesM * big_cols;
  // The half-height tiles come FIRST in the grid: at the start every CU holds two workgroups, half-height ones beside full
  // ones, and the slots they free take full tiles; as the last round of the launch the half-height tiles ran one to a CU, a
  // wave alone on its SIMD (whose vector and matrix instructions do not overlap).
  constexpr int HM = BM / 2;
  const int tilesH = (a.M + HM - 1) / HM;
  const int nsmall = TM >= 2 ? (int)gridDim.x - nbig : 0;
  int b = (int)blockIdx.x - nsmall;
  if (b >= 0) {
    // Workgroup b runs on XCD b % 8, and every XCD has its own L2.  An XCD takes a block of the tile grid, two blocks along
    // M by four along N where the counts divide: it then reads half of the activations and a quarter of the weights
    // (a run of whole tile columns per XCD reads ALL of the activations and an eighth of the weights: for 2048 x 9728 x 2560
    // 11.8 MB per XCD against 7.9)
    int tm = b % tilesM, tn = b / tilesM;
    if (tilesM % 2 == 0 && big_cols % 4 == 0) {
      const int xcd = b & 7, seq = b >> 3, hm = tilesM / 2, qn = big_cols / 4;
      tm = (xcd & 1) * hm + seq % hm;
      tn = (xcd >> 1) * qn + seq / hm;
    } else if (nbig % 8 == 0) {
      b = (b % 8) * (nbig / 8) + b / 8;  // one run of tiles per XCD that shares a slice of the weights
      tm = b % tilesM;
      tn = b / tilesM;
    }
    w4a16_nsplit_tile<TM, TN, BK>(a, tm * BM, tn * BN, smem);
  } else {
    if constexpr (TM >= 2) {
      b = (int)blockIdx.x;
      w4a16_nsplit_tile<TM / 2, TN, BK>(a, (b % tilesH) * HM, (big_cols + b / tilesH) * BN, smem);
    }
  }
}

// dequantized weight table from the PACKED form, through the same dequant8 and (scale, -zp*scale) pairs as the GEMM
__global__ void w4a16_dequant_packed_kernel(const uint8_t* __restrict__ P, uint16_t* __restrict__ w, int N, int K, int group) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // one dword = 8 elements of the table
  if (i >= (int64_t)N * K / 8) return;
  const int n = (int)(i / (K / 8)), k = (int)(i % (K / 8)) * 8;
  const int kbs = (int)(w4a16_packed_k(K) / 64), G = K / group;
  const int nb = n / 32, row = n % 32, kb = k / 64, d = (k % 64) / 16, hi = (k % 16) / 8;
  const uint32_t word = reinterpret_cast<const uint32_t*>(P)[(((int64_t)nb * kbs + kb) * 64 + hi * 32 + row) * 4 + d];
  const float2 sz = reinterpret_cast<const float2*>(P + w4a16_packed_qbytes(N, K))[((int64_t)nb * G + k / group) * 32 + row];
  uint32_t o[4];
  dequant8(word, sz.x, sz.y, o);
  *reinterpret_cast<u32x4*>(w + (int64_t)n * K + k) = u32x4{o[0], o[1], o[2], o[3]};
}

static int g_w4a16_tail = 1;  // half-height tiles for a short last round (0 switches the schedule off: tuning/tests)

template <int TM, int TN, int BK, int WPS>
static int launch_w4a16_nsplit(const W4A16PArgs& a, hipStream_t st) {
  constexpr int BM = TM * 32, BN = 4 * TN * 32;
  constexpr size_t stage = 2 * (size_t)BM * (2 * BK + 16), patch = 4096 + 32 * (2 * (size_t)BN + 16);
  const size_t lds = stage > patch ? stage : patch;
  auto kern = w4a16_gemm_nsplit_kernel<TM, TN, BK, WPS>;
  static int slots = 0;  // workgroups the chip holds at once
  if (!slots) {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    int dev = 0, cus = 0, per_cu = 0;
    HIP_RET(hipGetDevice(&dev));
    HIP_RET(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    HIP_RET(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), 256, lds));
    slots = cus * (per_cu > 0 ? per_cu : 1);
  }
  const int tilesM = (a.M + BM - 1) / BM, tilesN = (a.N + BN - 1) / BN;
  const int64_t total = (int64_t)tilesM * tilesN;
  int big_cols = tilesN;
  if (g_w4a16_tail && TM >= 2 && total > slots && total % slots) {
    // columns whose full tiles fit into whole rounds; the remaining columns as half tiles if that ends earlier
    const int cols = (int)(total / slots * slots / tilesM);
    const int64_t halves = (int64_t)(tilesN - cols) * ((a.M + BM / 2 - 1) / (BM / 2));
    const double as_full = (double)((total + slots - 1) / slots);
    // a half tile takes about 0.6 of a full one: it dequantizes the same weights for half the rows
    const double with_tail = (double)(((int64_t)cols * tilesM + slots - 1) / slots) + 0.6 * (double)((halves + slots - 1) / slots);
    if (with_tail < as_full) big_cols = cols;
  }
  const int64_t grid = (int64_t)tilesM * big_cols + (int64_t)(tilesN - big_cols) * ((a.M + BM / 2 - 1) / (BM / 2));
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, st, a, big_cols);
  return (int)hipGetLastError();
}

static int g_w4a16_ptile = 0;  // packed path: 0 = heuristic, 1 = 128x384, 2 = 64x384, 3 = 128x128, 4 = 64x128, 5 = 128x256

// Tile choice for the weights-from-global kernel.  128x256 with two workgroups per CU measured best on large problems
// (one wave's dequantization runs beside the other's MFMAs); smaller tiles only to give every CU work.
static int launch_w4a16_nsplit_auto(const W4A16PArgs& a, hipStream_t st) {
  auto tiles = [&](int bm, int bn) { return (int64_t)((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn); };
  int t = g_w4a16_ptile;
  if (!t) {
    if (a.M > 64) t = tiles(128, 256) >= 256 ? 5 : tiles(128, 128) >= 128 ? 3 : 4;
    else t = tiles(64, 384) >= 192 ? 2 : 4;
  }
  switch (t) {
    case 1: return launch_w4a16_nsplit<4, 3, 128, 1>(a, st);
    case 2: return launch_w4a16_nsplit<2, 3, 128, 2>(a, st);
    case 3: return launch_w4a16_nsplit<4, 1, 64, 3>(a, st);
    case 5: return launch_w4a16_nsplit<4, 2, 64, 2>(a, st);
    default: return launch_w4a16_nsplit<2, 1, 128, 2>(a, st);
  }
}

template <int BM, int BN, int WM, int WN>
static int launch_w4a16(const W4A16Args& a, hipStream_t st) {
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  const size_t lds = 2 * (size_t)(BM + BN) * 144;
  const unsigned grid = (unsigned)(((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN));
  auto kern = w4a16_gemm_kernel<BM, BN, WM, WN>;
  if (lds > 64 * 1024)
    HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), lds, st, a);
  return (int)hipGetLastError();
}

static int g_w4a16_tile = 0;  // 0 = heuristic, 1 = 256x192, 2 = 128x128, 3 = 64x64

}  // namespace mllmhip

using namespace mllmhip;

MLLM_API int mllm_hip_w4a16_set_tuning(int tile) {
  if (tile < 0 || tile > 3) return MLLM_HIP_E_BADARG;
  g_w4a16_tile = tile;
  return 0;
}

MLLM_API int mllm_hip_w4a16_packed_set_tuning(int tile) {
  if (tile < 0 || (tile & 15) > 5 || tile > 31) return MLLM_HIP_E_BADARG;
  g_w4a16_ptile = tile & 15;
  g_w4a16_tail = !(tile & 16);
  return 0;
}

static int check_w4a16(const void* qw, const void* s, const void* zp, int64_t N, int64_t K, int group) {
  if (!qw || !s || !zp || N <= 0 || K <= 0 || group <= 0) return MLLM_HIP_E_BADARG;
  if (group % 64 || K % group) return MLLM_HIP_E_SHAPE;
  if (N * K / 2 >= ((int64_t)1 << 32) || N > INT32_MAX || K > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(qw) % 16) return MLLM_HIP_E_ALIGN;
  return 0;
}

MLLM_API int mllm_hip_w4a16_gemm(const void* a_bf16, const uint8_t* qw, const uint16_t* scales, const uint8_t* zeros,
                                 const void* bias_bf16, void* c_bf16, int64_t M, int64_t N, int64_t K, int group,
                                 void* stream) {
  int rc = check_w4a16(qw, scales, zeros, N, K, group);
  if (rc) return rc;
  if (!a_bf16 || !c_bf16 || M <= 0) return MLLM_HIP_E_BADARG;
  if (M * K * 2 >= ((int64_t)1 << 32) || M > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(a_bf16) % 16) return MLLM_HIP_E_ALIGN;
  W4A16Args a{(const uint16_t*)a_bf16, qw, scales, zeros, (const uint16_t*)bias_bf16, (uint16_t*)c_bf16,
              (int)M, (int)N, (int)K, group};
  hipStream_t st = (hipStream_t)stream;
  int tile = g_w4a16_tile;
  if (!tile) {
    const int64_t big = ((M + 255) / 256) * ((N + 191) / 192);
    const int64_t mid = ((M + 127) / 128) * ((N + 127) / 128);
    (void)big;  // the 256x192 tile is compiled and tested but measured slower than 128x128 so far
    tile = mid >= 128 ? 2 : 3;
  }
  switch (tile) {
    case 1: return launch_w4a16<256, 192, 128, 96>(a, st);
    case 2: return launch_w4a16<128, 128, 64, 64>(a, st);
    default: return launch_w4a16<64, 64, 32, 32>(a, st);
  }
}

MLLM_API int mllm_hip_w4a16_dequantize(const uint8_t* qw, const uint16_t* scales, const uint8_t* zeros, void* w_bf16,
                                       int64_t N, int64_t K, int group, void* stream) {
  int rc = check_w4a16(qw, scales, zeros, N, K, group);
  if (rc) return rc;
  if (!w_bf16) return MLLM_HIP_E_BADARG;
  const int64_t words = N * K / 8;
  hipLaunchKernelGGL(w4a16_dequant_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, (hipStream_t)stream, qw,
                     scales, zeros, (uint16_t*)w_bf16, N, K, group);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------
// AWQ checkpoint tensors -> the row-major layout of this file (the unpacking half of what the reference does in
// AWQMarlinLinearMethod.process_weights_after_loading, pymllm/quantization/methods/awq_marlin.py:366-410).
//   qweight int32 [K][N/8], qzeros int32 [K/group][N/8]: eight 4-bit codes of eight neighbouring output columns per dword,
//   nibble position p holding column 8 j + {0,2,4,6,1,3,5,7}[p] (awq_marlin.py:202-213 unpack_cols followed by the
//   undo_interleave of :248-257; awq_marlin_repack.cuh:108-110 reads column c from nibble {0,4,1,5,2,6,3,7}[c]);
//   scales fp16 [K/group][N].
// The weight codes are transposed through LDS in 64 x 64 tiles so that both the checkpoint reads and the [N][K/2] writes
// are whole 32-byte runs.
__device__ __forceinline__ int awq_nibble_of_column(int c) { return ((c & 1) << 2) | (c >> 1); }  // {0,4,1,5,2,6,3,7}[c]

__global__ __launch_bounds__(256) void awq_unpack_q_kernel(const uint32_t* __restrict__ qweight, uint32_t* __restrict__ qw,
                                                           int N, int K) {
  __shared__ uint32_t tile[64][9];  // [k][column dword], one pad dword against bank conflicts of the column reads
  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64, t = threadIdx.x;
  const int nd = N / 8;
  for (int i = t; i < 512; i += 256) {
    const int k = k0 + i / 8, j = n0 / 8 + i % 8;
    tile[i / 8][i % 8] = (k < K && j < nd) ? qweight[(int64_t)k * nd + j] : 0u;
  }
  __syncthreads();
  for (int i = t; i < 512; i += 256) {
    const int r = i / 8, kd = i % 8;  // output row n0 + r, its dword of elements k0 + 8 kd .. + 7
    const int n = n0 + r, k = k0 + kd * 8;
    if (n >= N || k >= K) continue;
    const int sh = 4 * awq_nibble_of_column(r & 7);
    uint32_t v = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) v |= ((tile[kd * 8 + e][r >> 3] >> sh) & 15u) << (4 * e);
    qw[((int64_t)n * K + k) / 8] = v;
  }
}

__global__ __launch_bounds__(256) void awq_unpack_sz_kernel(const uint32_t* __restrict__ qzeros, const uint16_t* __restrict__ s_in,
                                                            uint16_t* __restrict__ s_out, uint8_t* __restrict__ z_out, int N,
                                                            int G) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // (group, n): neighbouring threads read neighbouring columns
  if (i >= (int64_t)N * G) return;
  const int n = (int)(i % N), g = (int)(i / N);
  s_out[(int64_t)n * G + g] = s_in[(int64_t)g * N + n];
  if (g & 1) return;  // one thread per byte of zero points: groups g (low nibble) and g + 1 (high nibble)
  const int sh = 4 * awq_nibble_of_column(n & 7), nd = N / 8;
  uint32_t z = (qzeros[(int64_t)g * nd + n / 8] >> sh) & 15u;
  if (g + 1 < G) z |= ((qzeros[(int64_t)(g + 1) * nd + n / 8] >> sh) & 15u) << 4;
  z_out[(int64_t)n * ((G + 1) / 2) + g / 2] = (uint8_t)z;
}

MLLM_API int mllm_hip_w4a16_from_awq(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales, int64_t N,
                                     int64_t K, int group, uint8_t* qw, uint16_t* scales_out, uint8_t* zeros_out,
                                     void* stream) {
  if (!qweight || !qzeros || !scales || !qw || !scales_out || !zeros_out || N <= 0 || K <= 0 || group <= 0)
    return MLLM_HIP_E_BADARG;
  if (N % 8 || K % 8 || K % group) return MLLM_HIP_E_SHAPE;
  if (N * K / 2 >= ((int64_t)1 << 32) || N > INT32_MAX || K > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(qw) % 4 || reinterpret_cast<uintptr_t>(qweight) % 4 ||
      reinterpret_cast<uintptr_t>(qzeros) % 4)
    return MLLM_HIP_E_ALIGN;
  const int G = (int)(K / group);
  if ((K + 63) / 64 > 65535) return MLLM_HIP_E_SHAPE;
  hipLaunchKernelGGL(awq_unpack_q_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64)), dim3(256), 0,
                     (hipStream_t)stream, reinterpret_cast<const uint32_t*>(qweight), reinterpret_cast<uint32_t*>(qw), (int)N,
                     (int)K);
  hipLaunchKernelGGL(awq_unpack_sz_kernel, dim3((unsigned)((N * G + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const uint32_t*>(qzeros), scales, scales_out, zeros_out, (int)N, G);
  return (int)hipGetLastError();
}

MLLM_API size_t mllm_hip_w4a16_packed_bytes(int64_t N, int64_t K, int group) {
  if (N <= 0 || K <= 0 || group <= 0 || group % 64 || K % group) return 0;
  return (size_t)(w4a16_packed_qbytes(N, K) + w4a16_packed_n(N) * (K / group) * 8);
}

MLLM_API int mllm_hip_w4a16_prepack(const uint8_t* qw, const uint16_t* scales, const uint8_t* zeros, int64_t N, int64_t K,
                                    int group, void* packed, void* stream) {
  int rc = check_w4a16(qw, scales, zeros, N, K, group);
  if (rc) return rc;
  if (!packed) return MLLM_HIP_E_BADARG;
  if (reinterpret_cast<uintptr_t>(packed) % 16) return MLLM_HIP_E_ALIGN;
  if (mllm_hip_w4a16_packed_bytes(N, K, group) >= ((size_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  const int64_t words = w4a16_packed_qbytes(N, K) / 4;
  hipLaunchKernelGGL(w4a16_prepack_q_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, (hipStream_t)stream, qw,
                     reinterpret_cast<uint32_t*>(packed), (int)N, (int)K, words);
  const int G = (int)(K / group);
  const int64_t count = w4a16_packed_n(N) * G;
  hipLaunchKernelGGL(w4a16_prepack_sz_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, (hipStream_t)stream, scales,
                     zeros, reinterpret_cast<float2*>(reinterpret_cast<char*>(packed) + w4a16_packed_qbytes(N, K)), (int)N, G,
                     count);
  return (int)hipGetLastError();
}

// ---- decode: up to 32 tokens against the packed weights ------------------------------------------------------------------
// The tile kernels spend a 128-row tile on a decode token (9728 x 2560 at one token: 20 us; 2560 x 9728: 65 us).  Here a
// workgroup takes one block row of the packed matrix (32 weight rows), its waves stride over the 64-element K blocks, eight
// blocks requested per wave before the first is dequantized (the first batch ahead of the copy of the tokens' activations
// into LDS); weights go to bf16 exactly as in the tile kernels (dequant8), the products (exact in fp32) are added by fp32
// FMAs, the two K halves of a block meet through a wave shuffle, the waves through LDS.  Same rounding points as the tile
// kernels (weights to bf16, the sum + bias to bf16), fp32 sums in another order.  The kernel is bound by its vector ALU
// work, which grows with the tokens (9728 x 2560: 12.5 / 14.0 / 17.9 / 25.5 us at one / two / four / eight tokens against 20 us
// for the tile kernels): it serves one token, the matrix-core form below two and more.
constexpr int W4G_MAXW = 16;
template <int MT>
__global__ __launch_bounds__(W4G_MAXW * 64) void w4a16_gemv_packed_kernel(W4A16PArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int Kp = (int)w4a16_packed_k(a.K), kbs = Kp / 64, G = a.K / a.group, g64 = a.group / 64;
  u32x4* sx = reinterpret_cast<u32x4*>(smem);                         // [MT][Kp / 8] bf16 activations, zero past K and M
  float* s_part = reinterpret_cast<float*>(smem + (size_t)MT * Kp * 2);  // [wave][MT][32]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int nb = blockIdx.x;
  const int64_t qbytes = w4a16_packed_qbytes(a.N, a.K);
  const u32x4* Q = reinterpret_cast<const u32x4*>(a.P) + (size_t)nb * kbs * 64 + lane;
  const float2* SZ = reinterpret_cast<const float2*>(a.P + qbytes) + (size_t)nb * G * 32 + r;
  constexpr int UB = 8;
  u32x4 wv[UB];
  float2 sz[UB];
  auto load_batch = [&](int kb0) {
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int kb = kb0 + u * nwaves;
      wv[u] = u32x4{0u, 0u, 0u, 0u};
      sz[u] = float2{0.f, 0.f};
      if (kb < kbs) {
        wv[u] = Q[(size_t)kb * 64];
        sz[u] = SZ[(size_t)min(kb / g64, G - 1) * 32];  // (blocks of the zero padding past K: their codes are zero, as are the activations)
      }
    }
  };
  load_batch(wave);
  const int cpr = Kp / 8;  // 16-byte pieces (eight elements) per token
  for (int i = tid; i < MT * cpr; i += nthreads) {
    const int m = i / cpr, c = i - m * cpr;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (m < a.M && c * 8 < a.K) v = *reinterpret_cast<const u32x4*>(a.A + (size_t)m * a.K + c * 8);  // K % 64 == 0
    sx[i] = v;
  }
  __syncthreads();
  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; m++) acc[m] = 0.f;
  for (int kb0 = wave; kb0 < kbs; kb0 += nwaves * UB) {
    if (kb0 != wave) load_batch(kb0);
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int kb = kb0 + u * nwaves;
      if (kb < kbs) {  // uniform
        const uint32_t wd[4] = {wv[u].x, wv[u].y, wv[u].z, wv[u].w};
#pragma unroll
        for (int d = 0; d < 4; d++) {  // elements k = 64 kb + 16 d + 8 h + 0..7
          uint32_t wb[4];
          dequant8(wd[d], sz[u].x, sz[u].y, wb);
#pragma unroll
          for (int m = 0; m < MT; m++) {
            const u32x4 xv = sx[m * cpr + kb * 8 + 2 * d + h];
            float s = acc[m];
            const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int p = 0; p < 4; p++) {
              s = fmaf(__uint_as_float(wb[p] << 16), __uint_as_float(xw[p] << 16), s);
              s = fmaf(__uint_as_float(wb[p] & 0xffff0000u), __uint_as_float(xw[p] & 0xffff0000u), s);
            }
            acc[m] = s;
          }
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
      float f = 0.f;
      for (int w = 0; w < nwaves; w++) f += s_part[(w * MT + m) * 32 + (i & 31)];
      if (a.bias) f += bf16_to_f32(a.bias[n]);
      a.C[(int64_t)m * a.N + n] = (uint16_t)pack_bf16(f, 0.f);
    }
  }
}
// The same walk with the products on the matrix cores: the packed dword d of a lane IS its operand of the d-th
// v_mfma_f32_32x32x16_bf16 of the block (row l % 32, eight consecutive k of half l / 32), the other operand the same eight k of
// token l % 32 from LDS (lanes past the MT tokens staged pass zeros), so a block costs four matrix instructions whatever the
// token count and the vector ALU does the dequantization only.  acc[4g + e] = C[token l % 32][row 8g + 4 (l / 32) + e]; the
// waves' sums meet in LDS where the activations were (after a barrier).
template <int MT>
__global__ __launch_bounds__(W4G_MAXW * 64) void w4a16_gemv_mfma_packed_kernel(W4A16PArgs a, int cb) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int Kp = (int)w4a16_packed_k(a.K), kbs = Kp / 64, G = a.K / a.group, g64 = a.group / 64;
  u32x4* sx = reinterpret_cast<u32x4*>(smem);       // [MT][8 cb] bf16 activations of the cb blocks in work, zero past K and M
  float* s_part = reinterpret_cast<float*>(smem);   // [wave][MT][32], after the loop
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int nb = blockIdx.x;
  const int64_t qbytes = w4a16_packed_qbytes(a.N, a.K);
  const u32x4* Q = reinterpret_cast<const u32x4*>(a.P) + (size_t)nb * kbs * 64 + lane;
  const float2* SZ = reinterpret_cast<const float2*>(a.P + qbytes) + (size_t)nb * G * 32 + r;
  constexpr int UB = 8;
  u32x4 wv[UB];
  float2 sz[UB];
  auto load_batch = [&](int kb0, int c1) {
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int kb = kb0 + u * nwaves;
      wv[u] = u32x4{0u, 0u, 0u, 0u};
      sz[u] = float2{0.f, 0.f};
      if (kb < c1) {
        wv[u] = Q[(size_t)kb * 64];
        sz[u] = SZ[(size_t)min(kb / g64, G - 1) * 32];
      }
    }
  };
  const int cpr = cb * 8;  // 16-byte pieces (eight elements) per token in LDS
  v16f acc;
#pragma unroll
  for (int j = 0; j < 16; j++) acc[j] = 0.f;
  const bool staged = r < MT;
  const u32x4* sxr = sx + (size_t)(staged ? r : 0) * cpr + h;
  // the K blocks in runs of cb (all of them where the tokens' rows fit LDS whole)
  for (int c0 = 0; c0 < kbs; c0 += cb) {
  const int c1 = min(c0 + cb, kbs);
  load_batch(c0 + wave, c1);  // ahead of the copy of the activations
  if (c0) __syncthreads();    // every wave is done with the previous run's activations
  for (int i = tid; i < MT * cpr; i += nthreads) {
    const int m = i / cpr, c = i - m * cpr, gc = c0 * 8 + c;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (m < a.M && gc * 8 < a.K) v = *reinterpret_cast<const u32x4*>(a.A + (size_t)m * a.K + gc * 8);
    sx[i] = v;
  }
  __syncthreads();
  for (int kb0 = c0 + wave; kb0 < c1; kb0 += nwaves * UB) {
    if (kb0 != c0 + wave) load_batch(kb0, c1);
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int kb = kb0 + u * nwaves;
      if (kb < c1) {  // uniform
        const uint32_t wd[4] = {wv[u].x, wv[u].y, wv[u].z, wv[u].w};
#pragma unroll
        for (int d = 0; d < 4; d++) {  // elements k = 64 kb + 16 d + 8 h + 0..7
          uint32_t wb[4];
          dequant8(wd[d], sz[u].x, sz[u].y, wb);
          u32x4 xv = {0u, 0u, 0u, 0u};
          if (staged) xv = sxr[(kb - c0) * 8 + 2 * d];
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, u32x4{wb[0], wb[1], wb[2], wb[3]}),
                                                        __builtin_bit_cast(bf16x8, xv), acc, 0, 0, 0);
        }
      }
    }
  }
  }
  __syncthreads();  // every wave is done with the activations
  if (staged) {
#pragma unroll
    for (int g = 0; g < 4; g++)
      *reinterpret_cast<f32x4*>(&s_part[(wave * MT + r) * 32 + 8 * g + 4 * h]) = f32x4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
  }
  __syncthreads();
  for (int i = tid; i < MT * 32; i += nthreads) {
    const int m = i >> 5, n = nb * 32 + (i & 31);
    if (m < a.M && n < a.N) {
      float f = 0.f;
      for (int w = 0; w < nwaves; w++) f += s_part[(w * MT + m) * 32 + (i & 31)];
      if (a.bias) f += bf16_to_f32(a.bias[n]);
      a.C[(int64_t)m * a.N + n] = (uint16_t)pack_bf16(f, 0.f);
    }
  }
}
static int g_w4a16_decode = 1;  // 0: the tile kernels also for a few tokens (comparison runs and tests)
static int g_w4a16_decode_mfma_from = 2;  // token counts from this one up take the matrix-core form
static bool launch_w4a16_gemv_packed(const W4A16PArgs& a, hipStream_t st, int* rc) {
  if (a.M > 32 || !g_w4a16_decode) return false;
  const int Kp = (int)w4a16_packed_k(a.K), kbs = Kp / 64;
  const int nwaves = kbs >= 32 ? W4G_MAXW : 4;
  const dim3 grid((unsigned)(w4a16_packed_n(a.N) / 32));
  if (a.M >= g_w4a16_decode_mfma_from) {
    // 17 to 32 tokens: every lane reads its own token's activations from LDS, and the tile kernels win where N gives them
    // enough tiles (9728 x 2560 at 32 tokens: 24 us here, 20 there; 6144 x 2048: 11.6 against 16.9)
    if (a.M > 16 && a.N > 8192) return false;
    const int MT = a.M <= 8 ? 8 : (a.M <= 16 ? 16 : 32);
    const int cap = 152 * 1024 / (MT * 128);  // K blocks of MT tokens in 152 KB
    const int cb = kbs < cap ? kbs : cap;
    const size_t x_bytes = (size_t)MT * cb * 128, part_bytes = (size_t)nwaves * MT * 32 * 4;
    const size_t lds = x_bytes > part_bytes ? x_bytes : part_bytes;
    auto go = [&](auto kern) {
      if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return (int)hipGetLastError();
      hipLaunchKernelGGL(kern, grid, dim3(nwaves * 64), lds, st, a, cb);
      return (int)hipGetLastError();
    };
    *rc = MT == 8 ? go(w4a16_gemv_mfma_packed_kernel<8>) : MT == 16 ? go(w4a16_gemv_mfma_packed_kernel<16>) : go(w4a16_gemv_mfma_packed_kernel<32>);
    return true;
  }
  if (a.M > 4) return false;
  const int MT = a.M <= 1 ? 1 : (a.M <= 2 ? 2 : 4);
  const size_t lds = (size_t)MT * Kp * 2 + (size_t)nwaves * MT * 32 * 4;
  if (lds > 160 * 1024) return false;
  auto go = [&](auto kern) {
    if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return (int)hipGetLastError();
    hipLaunchKernelGGL(kern, grid, dim3(nwaves * 64), lds, st, a);
    return (int)hipGetLastError();
  };
  *rc = MT == 1 ? go(w4a16_gemv_packed_kernel<1>) : MT == 2 ? go(w4a16_gemv_packed_kernel<2>) : go(w4a16_gemv_packed_kernel<4>);
  return true;
}
MLLM_API int mllm_hip_w4a16_set_decode(int gemv) {
  if (gemv != 0 && gemv != 1) return MLLM_HIP_E_BADARG;
  g_w4a16_decode = gemv;
  return 0;
}
MLLM_API int mllm_hip_w4a16_set_decode_mfma_from(int tokens) {
  if (tokens < 1 || tokens > 33) return MLLM_HIP_E_BADARG;
  g_w4a16_decode_mfma_from = tokens;
  return 0;
}

MLLM_API int mllm_hip_w4a16_gemm_packed(const void* a_bf16, const void* packed, const void* bias_bf16, void* c_bf16,
                                        int64_t M, int64_t N, int64_t K, int group, void* stream) {
  if (!a_bf16 || !packed || !c_bf16 || M <= 0 || N <= 0 || K <= 0 || group <= 0) return MLLM_HIP_E_BADARG;
  if (group % 64 || K % group) return MLLM_HIP_E_SHAPE;
  if (M * K * 2 >= ((int64_t)1 << 32) || M > INT32_MAX || N > INT32_MAX ||
      mllm_hip_w4a16_packed_bytes(N, K, group) >= ((size_t)1 << 32))
    return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(a_bf16) % 16 || reinterpret_cast<uintptr_t>(packed) % 16) return MLLM_HIP_E_ALIGN;
  W4A16PArgs a{(const uint16_t*)a_bf16, (const uint8_t*)packed, (const uint16_t*)bias_bf16, (uint16_t*)c_bf16,
               (int)M, (int)N, (int)K, group};
  int rc = 0;
  if (launch_w4a16_gemv_packed(a, (hipStream_t)stream, &rc)) return rc;  // up to 32 tokens
  return launch_w4a16_nsplit_auto(a, (hipStream_t)stream);
}

MLLM_API int mllm_hip_w4a16_dequantize_packed(const void* packed, void* w_bf16, int64_t N, int64_t K, int group, void* stream) {
  if (!packed || !w_bf16 || N <= 0 || K <= 0 || group <= 0) return MLLM_HIP_E_BADARG;
  if (group % 64 || K % group || N > INT32_MAX || K > INT32_MAX) return MLLM_HIP_E_SHAPE;
  const int64_t words = N * K / 8;
  hipLaunchKernelGGL(w4a16_dequant_packed_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)packed, (uint16_t*)w_bf16, (int)N, (int)K, group);
  return (int)hipGetLastError();
}
