// Block-quantized GEMM for many activation rows on gfx950, and the MoE expert FFN built on it.
//
//   y[row][n] = sum_b fp32(dW[n][b] * dX[row][b]) * int32(sum_32 qW * qX)       (every Linear of the reference's CPU path)
//
// Reference semantics:
//   expert loop           mllm/models/qwen3_moe/modeling_qwen3_moe_fa2.hpp:175-238 (moeInfer), :98-100 (Qwen3MoeMLP)
//   each Linear           mllm/backends/cpu/kernels/common/ggml/matmul.cpp:148-206 (Q8_0 activations, block dots)
//   SiLU                  mllm/backends/cpu/kernels/x86/silu.cpp:41   x / (1 + exp(-x))
// The per-block int32 sums come from v_mfma_i32_32x32x32_i8 (K = 32 = one quantization block per instruction, exact);
// they are scaled and accumulated in fp32 on the vector ALU.  Tokens are the MFMA rows, weight rows the MFMA columns, so
// a lane owns one output channel: its weight scale is a scalar per block and stores are contiguous across lanes.
#include "qgemv_kernel.h"

namespace mllmhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int TOK_TILE = 64;    // activation rows per workgroup tile (2 MFMA row tiles)
constexpr int TT = TOK_TILE / 32;
constexpr int KCH = 8;          // blocks per K chunk staged in LDS

// ---------------------------------------------------------------------------------------------------------
// routing: histogram, offsets, expert-sorted order and the tile list, one workgroup
// ---------------------------------------------------------------------------------------------------------
struct RouteOut {
  int* counts;       // [E]
  int* offsets;      // [E + 1]
  int* sorted_idx;   // [T*k]  flat index t*k + j of the entry at each expert-sorted position
  int* tile_expert;  // [max_tiles]
  int* tile_row0;    // [max_tiles]  first sorted position of the tile
  int* tile_rows;    // [max_tiles]  rows in the tile (<= TOK_TILE)
  int* ntiles;       // [1]
};

__global__ __launch_bounds__(1024) void moe_route_kernel(const int32_t* __restrict__ ids, int n, int E, RouteOut o) {
  extern __shared__ int s_cnt[];  // [E] counts, then [E] cursors
  int* s_cur = s_cnt + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) s_cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) atomicAdd(&s_cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0, nt = 0;
    for (int e = 0; e < E; e++) {
      const int c = s_cnt[e];
      o.counts[e] = c;
      o.offsets[e] = off;
      s_cur[e] = off;
      off += c;
    }
    o.offsets[E] = off;
    // tile list, full tiles first so that the long-running workgroups start early
    for (int pass = 0; pass < 2; pass++)
      for (int e = 0; e < E; e++) {
        const int c = s_cnt[e], base = o.offsets[e];
        for (int r = 0; r < c; r += TOK_TILE) {
          const int rows = min(TOK_TILE, c - r);
          if ((rows == TOK_TILE) == (pass == 0)) {
            o.tile_expert[nt] = e;
            o.tile_row0[nt] = base + r;
            o.tile_rows[nt] = rows;
            nt++;
          }
        }
      }
    o.ntiles[0] = nt;
  }
  __syncthreads();
  // the order inside an expert does not matter: every row is computed independently of its neighbours
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) o.sorted_idx[atomicAdd(&s_cur[e], 1)] = i;
  }
}

// identity routing for a plain Linear over M rows
__global__ void identity_tiles_kernel(int M, RouteOut o) {
  const int nt = (M + TOK_TILE - 1) / TOK_TILE;
  for (int t = threadIdx.x; t < nt; t += blockDim.x) {
    o.tile_expert[t] = 0;
    o.tile_row0[t] = t * TOK_TILE;
    o.tile_rows[t] = min(TOK_TILE, M - t * TOK_TILE);
  }
  if (threadIdx.x == 0) o.ntiles[0] = nt;
}

// ---------------------------------------------------------------------------------------------------------
// Q8_0 activation quantization to codes + the fp32 scale that takes part in the arithmetic
// (quantize_row_q8_0, AVX2 branch, ggml/quantize/quantize_q8.cpp:106-190)
// ---------------------------------------------------------------------------------------------------------
__global__ void quant_rows_kernel(const void* __restrict__ x, int x_dtype, int8_t* __restrict__ codes,
                                  float* __restrict__ deff, int64_t nblocks, int x86_scale) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  float v[32];
  uint32_t q[8];
  int sum;
  load_block_f32(x, x_dtype, i * QK, v);
  uint16_t bits = quantize_block_q8_0(v, q, sum);
  if (x86_scale) bits = x86_scale_bits(bits);
  deff[i] = f16bits_to_f32(bits);
  u32x4* out = reinterpret_cast<u32x4*>(codes + i * QK);
  out[0] = u32x4{q[0], q[1], q[2], q[3]};
  out[1] = u32x4{q[4], q[5], q[6], q[7]};
}

// ---------------------------------------------------------------------------------------------------------
// the tile kernel
// ---------------------------------------------------------------------------------------------------------
struct QGemmArgs {
  const char* W0;        // packed weights of matrix 0 (gate, or the only matrix), expert e at W0 + e * wstride
  const char* W1;        // packed weights of matrix 1 (up) for the fused gate/up mode
  size_t wstride;
  const int8_t* aq;      // activation codes  [rows][K]
  const float* ad;       // activation scales [rows][K/32]
  const int* a_index;    // activation row of each sorted position is a_index[pos] / a_div ; null: the position itself
  int a_div;
  int a_rows;            // rows of aq
  const int* o_index;    // output row of each sorted position (null: the position itself)
  float* out;            // fp32 [..][N]   (plain / down mode)
  const float* bias;     // [N] or null    (plain mode)
  int8_t* hq;            // gate/up mode: int8 codes of silu(g)*u  [rows][N]
  float* hd;             // gate/up mode: their scales              [rows][N/32]
  const int* tile_expert;
  const int* tile_row0;
  const int* tile_rows;
  const int* ntiles;
  int N, K;
  int x86_scale;
};

// weight codes of one block for the lane's output channel as signed int8: lanes 0..31 supply elements 0..15, lanes 32..63
// elements 16..31 (Q4_0: low / high nibbles of the same 16 bytes; Q8_0: first / second code plane).
template <int WT>
__device__ __forceinline__ v4i weight_operand(const u32x4& q, int hi) {
  if (WT == MLLM_HIP_Q4_0) {
    const uint32_t sh = hi ? 4u : 0u;
    const uint32_t d[4] = {q.x, q.y, q.z, q.w};
    v4i r;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint32_t nib = (d[j] >> sh) & 0x0f0f0f0fu;                    // bytes 0..15
      r[j] = (int)(((nib | 0x80808080u) - 0x08080808u) ^ 0x80808080u);    // per-byte (v - 8), no borrow between bytes
    }
    return r;
  } else {
    return v4i{(int)q.x, (int)q.y, (int)q.z, (int)q.w};
  }
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }

constexpr int PLANE = TOK_TILE * 16 + 16;          // LDS bytes of one (block, half) plane of activation codes, padded
constexpr int SA_BYTES = KCH * 2 * PLANE;
constexpr int SDX_BYTES = KCH * TOK_TILE * 4;
constexpr int SU_LD = 128 + 4;                     // row stride (floats) of the up -> gate hand-over tile
constexpr int SU_BYTES = TOK_TILE * SU_LD * 4;

// Workgroup tile: up to TOK_TILE activation rows x 128 output channels; a wave owns 32 channels (one MFMA column tile) and
// all 32-row tiles.  K is walked in chunks of 8 blocks:
//   * the rows' int8 codes (128 x 256 B) and fp32 scales of the chunk are staged in LDS once per workgroup, laid out as
//     [block][half][row] 16-byte words so that operand reads of neighbouring rows are neighbouring words;
//   * each lane keeps its channel's 8 weight blocks and 8 scales of the chunk in registers;
//   * the next chunk's global loads (activations and weights) are in flight while the current chunk is computed.
// MODE 0: one weight matrix, out[o_index[pos]][n] = acc (+ bias).
// MODE 1: eight waves; waves 0..3 run the gate matrix, waves 4..7 the up matrix over the same channels; the up
//         accumulators are handed over through LDS and the gate waves emit h = silu(g) * u quantized to Q8_0 (the 32
//         channels of a wave are exactly one block of the next Linear's input).
template <int WT, int MODE>
__global__ __launch_bounds__(MODE == 1 ? 512 : 256) void qgemm_tile_kernel(QGemmArgs a) {
  constexpr int NT = MODE == 1 ? 512 : 256;
  constexpr int UA = TOK_TILE * 16 / NT;  // 16-byte activation words per thread and chunk
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sA = smem;
  float* sDx = reinterpret_cast<float*>(smem + SA_BYTES);
  float* sU = reinterpret_cast<float*>(smem);  // MODE 1 hand-over tile, reuses the staging area after the last chunk

  const int tile = blockIdx.x;
  if (tile >= a.ntiles[0]) return;
  const int e = a.tile_expert[tile], row0 = a.tile_row0[tile], rows = a.tile_rows[tile];
  const int ntt = (rows + 31) >> 5;
  const int last_njg = (rows - 32 * (ntt - 1) + 7) >> 3;  // 8-row groups in the last 32-row tile
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, hi = lane >> 5;
  const int nb = a.K / QK, nbp = (int)scale_row_stride(a.K);
  const int mat = MODE == 1 ? (wave >> 2) : 0;
  const int nt = blockIdx.y * 4 + (wave & 3);  // this wave's tile of 32 output channels
  const bool nvalid = nt * 32 < a.N;
  const int n = min(nt * 32 + lrow, a.N - 1);

  const PackedView w = packed_view(WT, (mat ? a.W1 : a.W0) + (size_t)e * a.wstride, a.N, a.K);
  const u32x4* wq = (WT == MLLM_HIP_Q8_0 && hi) ? w.q1 : w.q0;

  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.aq), 0, (uint32_t)((int64_t)a.a_rows * a.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t rD = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.ad), 0, (uint32_t)((int64_t)a.a_rows * nb * 4), 0x00020000);

  // staging assignment: word u = tid + i*NT of the chunk -> row u/16, 16-byte column u%16 (= block*2 + half)
  uint32_t abase[UA];
#pragma unroll
  for (int i = 0; i < UA; i++) {
    const int u = tid + i * NT, p = u >> 4;
    uint32_t off = 0xffffffffu;
    if (p < rows) {
      const int r = a.a_index ? a.a_index[row0 + p] / a.a_div : row0 + p;
      off = (uint32_t)((int64_t)r * a.K + (u & 15) * 16);
    }
    abase[i] = off;
  }
  // scales: thread t < 2*TOK_TILE -> row t/2, blocks (t%2)*4 .. +4 of the chunk
  uint32_t dbase = 0xffffffffu;
  if (tid < 2 * TOK_TILE && (tid >> 1) < rows) {
    const int p = tid >> 1;
    const int r = a.a_index ? a.a_index[row0 + p] / a.a_div : row0 + p;
    dbase = (uint32_t)(((int64_t)r * nb + (tid & 1) * 4) * 4);
  }

  u32x4 pa[UA];
  float pd[4];
  u32x4 bq[KCH], bqn[KCH], bs, bsn;
  auto gload_act = [&](int b0) {
#pragma unroll
    for (int i = 0; i < UA; i++) {
      const int blk = ((tid + i * NT) & 15) >> 1;
      const bool ok = abase[i] != 0xffffffffu && b0 + blk < nb;
      pa[i] = __builtin_amdgcn_raw_buffer_load_b128(rA, ok ? abase[i] + (uint32_t)b0 * QK : 0xffffffffu, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const bool ok = dbase != 0xffffffffu && b0 + (tid & 1) * 4 + j < nb;
      pd[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rD, ok ? dbase + (uint32_t)(b0 + j) * 4 : 0xffffffffu, 0, 0));
    }
  };
  auto sstore_act = [&]() {
#pragma unroll
    for (int i = 0; i < UA; i++) {
      const int u = tid + i * NT;
      *reinterpret_cast<u32x4*>(sA + (u & 15) * PLANE + (u >> 4) * 16) = pa[i];
    }
    if (tid < 2 * TOK_TILE) {
#pragma unroll
      for (int j = 0; j < 4; j++) sDx[((tid & 1) * 4 + j) * TOK_TILE + (tid >> 1)] = pd[j];
    }
  };
  auto gload_w = [&](int b0, u32x4 (&q)[KCH], u32x4& sc) {
#pragma unroll
    for (int k = 0; k < KCH; k++) q[k] = wq[(int64_t)n * nb + min(b0 + k, nb - 1)];
    sc = *reinterpret_cast<const u32x4*>(w.d + (int64_t)n * nbp + min(b0, nbp - KCH));
  };

  float acc[TT][16];
#pragma unroll
  for (int tt = 0; tt < TT; tt++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[tt][r] = 0.f;

  gload_act(0);
  gload_w(0, bq, bs);
  sstore_act();
  __syncthreads();

  for (int b0 = 0; b0 < nb; b0 += KCH) {
    // the next chunk's loads are issued unconditionally (past the end they are clamped or out of range and unused): a
    // branch around them would leave the number of loads in flight unknown and force a full wait before the MFMAs
    const bool more = b0 + KCH < nb;
    gload_act(b0 + KCH);
    gload_w(b0 + KCH, bqn, bsn);
    if (nvalid) {
      const uint32_t sw[4] = {bs.x, bs.y, bs.z, bs.w};
#pragma unroll
      for (int k = 0; k < KCH; k++) {
        if (b0 + k < nb) {
          const v4i fb = weight_operand<WT>(bq[k], hi);
          const float dw = f16bits_to_f32((uint16_t)(sw[k >> 1] >> (16 * (k & 1))));
#pragma unroll
          for (int tt = 0; tt < TT; tt++) {
            if (tt < ntt) {
              const v4i fa = *reinterpret_cast<const v4i*>(sA + (k * 2 + hi) * PLANE + (tt * 32 + lrow) * 16);
              v16i z;
#pragma unroll
              for (int r = 0; r < 16; r++) z[r] = 0;
              const v16i is = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, z, 0, 0, 0);
              const int njg = (tt == ntt - 1) ? last_njg : 4;
              // accumulator register r of lane l: row 8*(r/4) + 4*(l/32) + r%4, column l%32
#pragma unroll
              for (int j = 0; j < 4; j++) {
                if (j < njg) {
                  const f32x4 dx = *reinterpret_cast<const f32x4*>(&sDx[k * TOK_TILE + tt * 32 + 8 * j + 4 * hi]);
#pragma unroll
                  for (int i = 0; i < 4; i++) acc[tt][4 * j + i] = fmaf(dw * dx[i], (float)is[4 * j + i], acc[tt][4 * j + i]);
                }
              }
            }
          }
        }
      }
    }
    __syncthreads();  // every wave is done with the staged chunk
    if (more) {
      sstore_act();
#pragma unroll
      for (int k = 0; k < KCH; k++) bq[k] = bqn[k];
      bs = bsn;
    }
    __syncthreads();
  }

  if (MODE == 1) {
    // up waves hand their accumulators to the gate waves of the same channels (the staging area is free now)
    if (mat == 1 && nvalid) {
#pragma unroll
      for (int tt = 0; tt < TT; tt++)
        if (tt < ntt)
#pragma unroll
          for (int r = 0; r < 16; r++)
            sU[(tt * 32 + 8 * (r / 4) + 4 * hi + (r % 4)) * SU_LD + (wave & 3) * 32 + lrow] = acc[tt][r];
    }
    __syncthreads();
    if (mat == 1 || !nvalid) return;
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
      if (tt >= ntt) continue;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int p = tt * 32 + 8 * (r / 4) + 4 * hi + (r % 4);  // row within the tile, same for the 32 lanes of a half
        const float h = silu_f(acc[tt][r]) * sU[p * SU_LD + (wave & 3) * 32 + lrow];
        float amax = fabsf(h);
        amax = fmaxf(amax, dpp_f<0xB1>(amax));
        amax = fmaxf(amax, dpp_f<0x4E>(amax));
        amax = fmaxf(amax, dpp_f<0x141>(amax));
        amax = fmaxf(amax, dpp_f<0x140>(amax));
        amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
        const float d = amax / 127.f;
        const float idv = (amax != 0.f) ? 127.f / amax : 0.f;
        int qi = (int)rintf(h * idv);
        qi = min(127, max(-128, qi));
        if (p < rows) {
          a.hq[(int64_t)(row0 + p) * a.N + n] = (int8_t)qi;
          if (lrow == 0) {
            uint16_t bits = f32_to_f16bits(d);
            if (a.x86_scale) bits = x86_scale_bits(bits);
            a.hd[(int64_t)(row0 + p) * (a.N / QK) + nt] = f16bits_to_f32(bits);
          }
        }
      }
    }
  } else {
    if (!nvalid) return;
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
      if (tt >= ntt) continue;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int p = tt * 32 + 8 * (r / 4) + 4 * hi + (r % 4);
        if (p < rows && nt * 32 + lrow < a.N) {
          const int64_t orow = a.o_index ? a.o_index[row0 + p] : row0 + p;
          float v = acc[tt][r];
          if (a.bias) v = a.bias[n] + v;
          a.out[orow * a.N + n] = v;
        }
      }
    }
  }
}

// y[t][h] = sum_j per[t*k + j][h] * w[t][j]   (multiply, then add in j order: modeling_qwen3_moe_fa2.hpp:233-236)
__global__ void moe_combine_kernel(const float* __restrict__ per, const float* __restrict__ w, const int32_t* __restrict__ ids,
                                   float* __restrict__ y, int64_t T, int H, int k, int E) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * H) return;
  const int64_t t = i / H;
  const int h = (int)(i % H);
  float acc = 0.f;
  for (int j = 0; j < k; j++) {
    const int e = ids[t * k + j];
    if (e >= 0 && e < E) acc = acc + per[(t * k + j) * H + h] * w[t * k + j];
  }
  y[i] = acc;
}

// ---- workspace carving ---------------------------------------------------------------------------------------
struct Carver {
  char* p;
  size_t used = 0;
  explicit Carver(void* base) : p(reinterpret_cast<char*>(base)) {}
  template <typename T>
  T* take(size_t count) {
    T* r = reinterpret_cast<T*>(p ? p + used : nullptr);
    used += align_up(count * sizeof(T), 256);
    return r;
  }
};
static RouteOut carve_route(Carver& c, int E, int64_t entries) {
  RouteOut o;
  const size_t max_tiles = (size_t)E + (size_t)(entries / TOK_TILE) + 1;
  o.counts = c.take<int>(E);
  o.offsets = c.take<int>(E + 1);
  o.sorted_idx = c.take<int>(entries);
  o.tile_expert = c.take<int>(max_tiles);
  o.tile_row0 = c.take<int>(max_tiles);
  o.tile_rows = c.take<int>(max_tiles);
  o.ntiles = c.take<int>(1);
  return o;
}

template <int MODE>
static int launch_tiles(int wtype, const QGemmArgs& a, unsigned max_tiles, hipStream_t st) {
  const dim3 grid(max_tiles, (unsigned)((a.N + 127) / 128));
  const size_t lds = (MODE == 1 && SU_BYTES > SA_BYTES + SDX_BYTES) ? (size_t)SU_BYTES : (size_t)(SA_BYTES + SDX_BYTES);
  auto launch = [&](auto kern) -> int {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, grid, dim3(MODE == 1 ? 512 : 256), lds, st, a);
    return (int)hipGetLastError();
  };
  return wtype == MLLM_HIP_Q4_0 ? launch(qgemm_tile_kernel<MLLM_HIP_Q4_0, MODE>) : launch(qgemm_tile_kernel<MLLM_HIP_Q8_0, MODE>);
}

}  // namespace mllmhip

using namespace mllmhip;

// =========================================================================================================
// C ABI
// =========================================================================================================
MLLM_API size_t mllm_hip_linear_q_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || K % QK) return 0;
  Carver c(nullptr);
  c.take<int8_t>((size_t)M * K);
  c.take<float>((size_t)M * (K / QK));
  carve_route(c, 1, M);
  return c.used;
}

MLLM_API int mllm_hip_linear_q(int wtype, const void* packed, const void* x, int x_dtype, const float* bias, float* y,
                               int64_t M, int64_t N, int64_t K, int act_scale_mode, void* workspace, void* stream) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || !packed || !x || !y || !workspace || M <= 0 || N <= 0 || K <= 0)
    return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (K % QK || M * K >= ((int64_t)1 << 32) || N > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16 || reinterpret_cast<uintptr_t>(packed) % 16)
    return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  Carver c(workspace);
  int8_t* aq = c.take<int8_t>((size_t)M * K);
  float* ad = c.take<float>((size_t)M * (K / QK));
  RouteOut ro = carve_route(c, 1, M);
  const int64_t nblocks = M * (K / QK);
  hipLaunchKernelGGL(quant_rows_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, st, x, x_dtype, aq, ad, nblocks,
                     act_scale_mode == MLLM_HIP_SCALE_X86_REF);
  hipLaunchKernelGGL(identity_tiles_kernel, dim3(1), dim3(256), 0, st, (int)M, ro);
  QGemmArgs a{};
  a.W0 = a.W1 = reinterpret_cast<const char*>(packed);
  a.wstride = 0;
  a.aq = aq; a.ad = ad; a.a_index = nullptr; a.a_div = 1; a.a_rows = (int)M;
  a.o_index = nullptr; a.out = y; a.bias = bias;
  a.tile_expert = ro.tile_expert; a.tile_row0 = ro.tile_row0; a.tile_rows = ro.tile_rows; a.ntiles = ro.ntiles;
  a.N = (int)N; a.K = (int)K; a.x86_scale = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  return launch_tiles<0>(wtype, a, (unsigned)((M + TOK_TILE - 1) / TOK_TILE), st);
}

MLLM_API size_t mllm_hip_moe_workspace_bytes(int64_t T, int64_t H, int64_t I, int E, int k) {
  if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || k <= 0 || H % QK || I % QK) return 0;
  Carver c(nullptr);
  c.take<int8_t>((size_t)T * H);
  c.take<float>((size_t)T * (H / QK));
  c.take<int8_t>((size_t)T * k * I);
  c.take<float>((size_t)T * k * (I / QK));
  c.take<float>((size_t)T * k * H);
  carve_route(c, E, T * k);
  return c.used;
}

MLLM_API int mllm_hip_moe_route(const int32_t* topk_ids, int64_t T, int E, int k, int32_t* counts, int32_t* offsets,
                                int32_t* sorted_idx, void* workspace, void* stream) {
  if (!topk_ids || !workspace || T <= 0 || E <= 0 || E > 4096 || k <= 0) return MLLM_HIP_E_BADARG;
  hipStream_t st = (hipStream_t)stream;
  Carver c(workspace);
  RouteOut ro = carve_route(c, E, T * k);
  hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(1024), 2 * E * sizeof(int), st, topk_ids, (int)(T * k), E, ro);
  HIP_RET(hipGetLastError());
  if (counts) HIP_RET(hipMemcpyAsync(counts, ro.counts, E * sizeof(int), hipMemcpyDeviceToDevice, st));
  if (offsets) HIP_RET(hipMemcpyAsync(offsets, ro.offsets, (E + 1) * sizeof(int), hipMemcpyDeviceToDevice, st));
  if (sorted_idx) HIP_RET(hipMemcpyAsync(sorted_idx, ro.sorted_idx, T * k * sizeof(int), hipMemcpyDeviceToDevice, st));
  return 0;
}

MLLM_API int mllm_hip_moe_ffn_q(int wtype, const void* gate_packed, const void* up_packed, const void* down_packed,
                                const void* x, int x_dtype, const int32_t* topk_ids, const float* topk_w, float* y,
                                int64_t T, int64_t H, int64_t I, int E, int k, int act_scale_mode, void* workspace,
                                void* stream) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || !gate_packed || !up_packed || !down_packed || !x || !topk_ids ||
      !topk_w || !y || !workspace || T <= 0 || E <= 0 || E > 4096 || k <= 0)
    return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (H <= 0 || I <= 0 || H % QK || I % QK) return MLLM_HIP_E_SHAPE;
  if (T * H >= ((int64_t)1 << 32) || T * k * I >= ((int64_t)1 << 32) || T * k > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16) return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int x86 = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  Carver c(workspace);
  int8_t* xq = c.take<int8_t>((size_t)T * H);
  float* xd = c.take<float>((size_t)T * (H / QK));
  int8_t* hq = c.take<int8_t>((size_t)T * k * I);
  float* hd = c.take<float>((size_t)T * k * (I / QK));
  float* per = c.take<float>((size_t)T * k * H);
  RouteOut ro = carve_route(c, E, T * k);
  const unsigned max_tiles = (unsigned)(E + (T * k) / TOK_TILE + 1);

  hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(1024), 2 * E * sizeof(int), st, topk_ids, (int)(T * k), E, ro);
  const int64_t nblocks = T * (H / QK);
  hipLaunchKernelGGL(quant_rows_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, st, x, x_dtype, xq, xd, nblocks, x86);

  QGemmArgs a{};
  a.tile_expert = ro.tile_expert; a.tile_row0 = ro.tile_row0; a.tile_rows = ro.tile_rows; a.ntiles = ro.ntiles;
  a.x86_scale = x86;
  // gate & up -> silu(g)*u -> Q8_0, rows in expert-sorted order
  a.W0 = reinterpret_cast<const char*>(gate_packed);
  a.W1 = reinterpret_cast<const char*>(up_packed);
  a.wstride = packed_bytes(wtype, I, H);
  a.aq = xq; a.ad = xd; a.a_index = ro.sorted_idx; a.a_div = k; a.a_rows = (int)T;
  a.hq = hq; a.hd = hd;
  a.N = (int)I; a.K = (int)H;
  int rc = launch_tiles<1>(wtype, a, max_tiles, st);
  if (rc) return rc;
  // down -> per-(token, slot) rows
  a.W0 = a.W1 = reinterpret_cast<const char*>(down_packed);
  a.wstride = packed_bytes(wtype, H, I);
  a.aq = hq; a.ad = hd; a.a_index = nullptr; a.a_div = 1; a.a_rows = (int)(T * k);
  a.o_index = ro.sorted_idx; a.out = per; a.bias = nullptr; a.hq = nullptr; a.hd = nullptr;
  a.N = (int)H; a.K = (int)I;
  rc = launch_tiles<0>(wtype, a, max_tiles, st);
  if (rc) return rc;
  const int64_t total = T * H;
  hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, per, topk_w, topk_ids, y, T,
                     (int)H, k, E);
  return (int)hipGetLastError();
}
