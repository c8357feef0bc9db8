// Block-quantized GEMM for many activation rows on gfx950, and the MoE expert FFN built on it.
//
//   y[row][n] = sum_b fp32(dW[n][b] * dX[row][b]) * int32(sum_32 qW * qX)       (every Linear of the reference's CPU path)
//
// Reference semantics:
//   expert loop           mllm/models/qwen3_moe/modeling_qwen3_moe_fa2.hpp:175-238 (moeInfer), :98-100 (Qwen3MoeMLP)
//   each Linear           mllm/backends/cpu/kernels/common/ggml/matmul.cpp:148-206 (Q8_0 activations, block dots)
//   SiLU                  mllm/backends/cpu/kernels/x86/silu.cpp:16-27   x * (1 / (1 + exp_poly(-x))), math.hpp:19-72
// The per-block int32 sums come from v_mfma_i32_32x32x32_i8 (K = 32 = one quantization block per instruction, exact);
// they are scaled and accumulated in fp32 on the vector ALU.  Tokens are the MFMA rows, weight rows the MFMA columns, so
// a lane owns one output channel: its weight scale is a scalar per block and stores are contiguous across lanes.
#include "qgemv_kernel.h"
#include "qgemm_layout.h"

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

// GROUPED: an expert's tiles are neighbours in the list (full tiles, then its partial tile), the experts in the order of
// their numbers; otherwise all full tiles come first.  (Measured and dropped for the grouped list: experts in order of
// falling row counts, so that the short tiles end a launch: 4 % slower on 512 tokens x 8 of 128 experts -- the heavy
// experts' tiles are bound by arithmetic and the light ones by memory, and a list that mixes them overlaps the two.)
template <bool GROUPED = false>
__device__ __forceinline__ void moe_route_body(const int32_t* __restrict__ ids, int n, int E, int tile_h, const RouteOut& o, int* s_cnt) {
  // s_cnt: [E] counts, [E] cursors, [E] scan scratch x 3
  int* s_cur = s_cnt + E;
  int* s_off = s_cur + E;   // exclusive scan of the counts
  int* s_full = s_off + E;  // exclusive scan of the full-tile counts
  int* s_part = s_full + E; // exclusive scan of the partial-tile flags
  __shared__ int s_tot[3];
  for (int e = threadIdx.x; e < E; e += blockDim.x) s_cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) atomicAdd(&s_cnt[e], 1);
  }
  __syncthreads();
  // three exclusive scans over the experts, one wave each (E is at most a few thousand: 64 experts per step)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (wave < 3) {
    int* dst = wave == 0 ? s_off : wave == 1 ? s_full : s_part;
    int run = 0;
    for (int base = 0; base < E; base += 64) {
      const int e = base + lane;
      const int c = e < E ? s_cnt[e] : 0;
      const int v = wave == 0 ? c : wave == 1 ? c / tile_h : (c % tile_h != 0);
      int incl = v;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int t = __shfl_up(incl, d, 64);
        if (lane >= d) incl += t;
      }
      if (e < E) dst[e] = run + incl - v;
      run += __shfl(incl, 63, 64);
    }
    if (lane == 0) s_tot[wave] = run;
  }
  __syncthreads();
  // tile list, full tiles first so that the long-running workgroups start early (GROUPED: expert by expert)
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    const int c = s_cnt[e], base = s_off[e];
    o.counts[e] = c;
    o.offsets[e] = base;
    s_cur[e] = base;
    const int nf = c / tile_h;
    for (int t = 0; t < nf; t++) {
      const int slot = s_full[e] + t + (GROUPED ? s_part[e] : 0);
      o.tile_expert[slot] = e;
      o.tile_row0[slot] = base + t * tile_h;
      o.tile_rows[slot] = tile_h;
    }
    if (c % tile_h) {
      const int slot = GROUPED ? s_full[e] + nf + s_part[e] : s_tot[1] + s_part[e];
      o.tile_expert[slot] = e;
      o.tile_row0[slot] = base + nf * tile_h;
      o.tile_rows[slot] = c % tile_h;
    }
  }
  if (threadIdx.x == 0) {
    o.offsets[E] = s_tot[0];
    o.ntiles[0] = s_tot[1] + s_tot[2];
  }
  __syncthreads();
  // the order inside an expert does not matter: every row is computed independently of its neighbours
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) o.sorted_idx[atomicAdd(&s_cur[e], 1)] = i;
  }
}

__global__ __launch_bounds__(1024) void moe_route_kernel(const int32_t* __restrict__ ids, int n, int E, int tile_h, RouteOut o) {
  extern __shared__ int s_route[];
  moe_route_body(ids, n, E, tile_h, o, s_route);
}

// identity routing for a plain Linear over M rows
__global__ void identity_tiles_kernel(int M, int tile_h, RouteOut o) {
  const int nt = (M + tile_h - 1) / tile_h;
  for (int t = threadIdx.x; t < nt; t += blockDim.x) {
    o.tile_expert[t] = 0;
    o.tile_row0[t] = t * tile_h;
    o.tile_rows[t] = min(tile_h, M - t * tile_h);
  }
  if (threadIdx.x == 0) o.ntiles[0] = nt;
}

// The routing pass keeps five int arrays of E entries in LDS: E is limited to what fits the 64 KB a launch gets without
// raising the kernel's dynamic-LDS attribute.  The launch status is read before anything that consumes the tile list is
// queued: a consumer must never walk a list the routing pass did not write.
constexpr int MOE_MAX_EXPERTS = 3072;
static int launch_route(const int32_t* ids, int64_t entries, int E, int tile_h, const RouteOut& ro, hipStream_t st) {
  if (E <= 0 || E > MOE_MAX_EXPERTS) return MLLM_HIP_E_SHAPE;
  hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(1024), 5 * (size_t)E * sizeof(int), st, ids, (int)entries, E, tile_h, ro);
  return (int)hipGetLastError();
}
static int launch_identity_tiles(int64_t M, int tile_h, const RouteOut& ro, hipStream_t st) {
  hipLaunchKernelGGL(identity_tiles_kernel, dim3(1), dim3(256), 0, st, (int)M, tile_h, ro);
  return (int)hipGetLastError();
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

// the SiLU operator runs over whole [rows, I] tensors with I a multiple of 32: always the vector form
__device__ __forceinline__ float silu_f(float x) { return x * (1.0f / (1.0f + exp_poly(-x))); }

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
  if (tile >= min(a.ntiles[0], (int)gridDim.x)) return;
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

// =========================================================================================================
// Matrix-core path for many rows: fp16 operands with the block scales folded in
//
//   y[row][n] = sum_k xh[row][k] * wh[n][k],   xh = fp16(dX * qX) (the Q8_0 round trip of the activations, exact product
//   rounded once to fp16), wh = fp16(dW * qW) (likewise), fp32 accumulation in v_mfma_f32_32x32x16_f16.
//
// The block-dot form above needs three vector-ALU operations per (row, channel, block) to scale and add the int32 block
// sums, which bounds it far below the matrix rate.  Folding the scales into 16-bit operands moves that work to the
// operands: about two operations per WEIGHT element per 32*TM rows, nothing per accumulator.  Both roundings are to 11
// significant bits (relative error <= 2^-12 each), which keeps the result within about 3e-4 relative L2 of the
// reference's fp32 block arithmetic.  |dX*qX| and |dW*qW| must stay below 65504 (fp16).
//
// Weight layout ("gemm-packed", mllm_hip_q_gemm_prepack): codes in v_mfma_*_32x32x16 operand order, N padded to 32 rows
// and K to 128 elements with zero blocks;
//   Q4_0  q  [N/32][K/64][64 lanes][16 B]: lane l = (row l%32, half l/32); dword d of its 16 bytes holds the eight
//            elements k = 64 kb + 16 d + 8 (l/32) + 0..7: element 2i in nibble i, element 2i+1 in nibble 4+i (so that
//            (dword >> 4i) & 0x000f000f is the pair (2i, 2i+1) in the two halves of a register)
//   Q8_0  q  [N/32][K/64][2][64 lanes][16 B]: plane p holds d = 2p, 2p+1; each d is two dwords of four codes in byte
//            order e0, e2, e1, e3
//   scales   [N/32][K/64][32 rows] dwords: fp16 scale of block 2kb | fp16 scale of block 2kb+1 << 16, after the
//            weight_scale_mode decoding
// Kernel structure as the W4A16 weights-from-global kernel: four waves side by side along N, activations via LDS,
// weights straight from global memory two K steps ahead, dequantized one MFMA step ahead in the shadows of the MFMAs.
// =========================================================================================================
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));


// one output dword of the code area per thread
template <int WT>
__global__ __launch_bounds__(256) void qg_prepack_q_kernel(const unsigned char* __restrict__ blocks, uint32_t* __restrict__ P,
                                                           int N, int K, int64_t words) {
  const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (w >= words) return;
  const int kbs = (int)(qg_kp(K) / 64), nblk = K / QK;
  constexpr int BS = WT == MLLM_HIP_Q4_0 ? 18 : 34;
  uint32_t v = 0;
  if (WT == MLLM_HIP_Q4_0) {
    const int d = (int)(w % 4), l = (int)((w / 4) % 64);
    const int64_t blk = w / 256;
    const int kb = (int)(blk % kbs), nb = (int)(blk / kbs);
    const int n = nb * 32 + (l & 31), k0 = kb * 64 + d * 16 + (l >> 5) * 8;
    if (n < N && k0 < K) {
      const unsigned char* qs = blocks + ((int64_t)n * nblk + k0 / QK) * BS + 2;
      const int o = k0 % QK;  // 0, 8, 16, 24: elements o..o+7 are the low (o < 16) or high nibbles of qs[o % 16 ..]
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const uint32_t byte = qs[(o & 15) + i];
        const uint32_t e = o < 16 ? (byte & 15u) : (byte >> 4);
        v |= e << (4 * ((i >> 1) + 4 * (i & 1)));
      }
    }
  } else {
    const int x = (int)(w % 4), l = (int)((w / 4) % 64), pl = (int)((w / 256) % 2);
    const int64_t blk = w / 512;
    const int kb = (int)(blk % kbs), nb = (int)(blk / kbs);
    const int d = 2 * pl + x / 2;
    const int n = nb * 32 + (l & 31), k0 = kb * 64 + d * 16 + (l >> 5) * 8 + 4 * (x % 2);
    if (n < N && k0 < K) {
      const unsigned char* qs = blocks + ((int64_t)n * nblk + k0 / QK) * BS + 2 + k0 % QK;
      v = (uint32_t)qs[0] | ((uint32_t)qs[2] << 8) | ((uint32_t)qs[1] << 16) | ((uint32_t)qs[3] << 24);
    }
  }
  P[w] = v;
}
template <int WT>
__global__ __launch_bounds__(256) void qg_prepack_s_kernel(const unsigned char* __restrict__ blocks, uint32_t* __restrict__ S,
                                                           int N, int K, int x86_scale, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // (nb, kb, row)
  if (i >= count) return;
  const int kbs = (int)(qg_kp(K) / 64), nblk = K / QK;
  constexpr int BS = WT == MLLM_HIP_Q4_0 ? 18 : 34;
  const int row = (int)(i % 32), kb = (int)((i / 32) % kbs), nb = (int)(i / 32 / kbs);
  const int n = nb * 32 + row;
  uint32_t v = 0;
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const int b = 2 * kb + h;
    if (n < N && b < nblk) {
      const unsigned char* p = blocks + ((int64_t)n * nblk + b) * BS;
      uint16_t bits = (uint16_t)(p[0] | (p[1] << 8));
      if (x86_scale) {  // as mllm_hip_q_prepack: the field holds the pattern as a half-precision NUMBER
        const float num = f16bits_to_f32(bits);
        bits = (num >= 0.f && num < 65536.f) ? (uint16_t)(uint32_t)num : (uint16_t)0;
      }
      v |= (uint32_t)bits << (16 * h);
    }
  }
  S[i] = v;
}

// activations: Q8_0 quantization (bit-exact codes and scale) and back to fp16 in one pass
// (xl, when asked for: the rounding residual dX*qX - xh, exact in fp16, for the two-term gate/up path)
__global__ void qg_act_kernel(const void* __restrict__ x, int x_dtype, uint16_t* __restrict__ xh, uint16_t* __restrict__ xl,
                              int64_t nblocks, int x86_scale) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  float v[32];
  uint32_t q[8];
  int sum;
  load_block_f32(x, x_dtype, i * QK, v);
  uint16_t bits = quantize_block_q8_0(v, q, sum);
  if (x86_scale) bits = x86_scale_bits(bits);
  const float d = f16bits_to_f32(bits);
  uint32_t o[16], ol[16];
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const float a = d * (float)(int8_t)(q[j / 2] >> (16 * (j & 1)));       // exact in fp32: 11 x 8 bits
    const float b = d * (float)(int8_t)(q[j / 2] >> (16 * (j & 1) + 8));
    const uint16_t ha = f32_to_f16bits(a), hb = f32_to_f16bits(b);
    o[j] = (uint32_t)ha | ((uint32_t)hb << 16);
    ol[j] = (uint32_t)f32_to_f16bits(a - f16bits_to_f32(ha)) | ((uint32_t)f32_to_f16bits(b - f16bits_to_f32(hb)) << 16);
  }
  u32x4* out = reinterpret_cast<u32x4*>(xh + i * QK);
#pragma unroll
  for (int j = 0; j < 4; j++) out[j] = u32x4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
  if (xl) {
    u32x4* outl = reinterpret_cast<u32x4*>(xl + i * QK);
#pragma unroll
    for (int j = 0; j < 4; j++) outl[j] = u32x4{ol[4 * j], ol[4 * j + 1], ol[4 * j + 2], ol[4 * j + 3]};
  }
}

struct QG2Args {
  const char* W0;        // gemm-packed weights of matrix 0 (gate, or the only matrix), expert e at W0 + e * wstride
  const char* W1;        // gemm-packed weights of matrix 1 (up) in the fused gate/up mode
  size_t wstride;
  const uint16_t* xh;    // fp16 activations [a_rows][K]
  const uint16_t* xl;    // their rounding residuals, same shape (two-term mode only)
  const int* a_index;    // activation row of sorted position pos is a_index[pos] / a_div ; null: pos itself
  int a_div;
  int a_rows;
  const int* o_index;    // output row of sorted position pos (null: pos itself)
  float* out;            // fp32 [..][N]       (one-matrix mode)
  const float* bias;     // [N] or null        (one-matrix mode)
  uint16_t* hh;          // gate/up mode: fp16 Q8_0 round trip of silu(g)*u, [rows][N]
  const int* tile_expert;
  const int* tile_row0;
  const int* tile_rows;
  const int* ntiles;
  int N, K;
  int wtype;
  int x86_scale;
  int ksplit;            // one-matrix mode: K is cut into this many ranges (blockIdx.z), each writing its own partial result
  float* partial;        // [ksplit][a_rows][N] when ksplit > 1
};

// pair `b` (elements 2b, 2b+1) of the eight weights of one MFMA step, scaled: one dword of two fp16.  With PREC == 2 also
// the rounding residual of the product (exact: the error of a product of two fp16 numbers is an fp16 number).
// Q4_K: the sub-block's value is ds * q - dm (q = 0..15): one fused multiply-add, one rounding; Q6_K: codes widened to
// int8 at load time, ds the scale of the step's 16 elements: the Q8_0 arithmetic.
template <int WT, int PREC>
__device__ __forceinline__ uint32_t qg_pair(const u32x4 (&rq)[qg_nibbles(WT) ? 1 : 2], int d, int b, f16x2 dd, f16x2 dm, uint32_t& lo) {
  uint32_t t;
  f16x2 off;
  if (WT == MLLM_HIP_Q4_K) {
    static_assert(WT != MLLM_HIP_Q4_K || PREC == 1, "one-term operands only");
    t = ((rq[0][d] >> (4 * b)) & 0x000f000fu) | 0x64006400u;       // (1024 + q) in both halves
    const f16x2 c = __builtin_bit_cast(f16x2, t) - f16x2{(_Float16)1024.f, (_Float16)1024.f};  // q, exact
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(c, dd, -dm));                // v_pk_fma_f16
  }
  if (WT == MLLM_HIP_Q4_0) {
    t = ((rq[0][d] >> (4 * b)) & 0x000f000fu) | 0x64006400u;       // (1024 + q) in both halves
    off = f16x2{(_Float16)1032.f, (_Float16)1032.f};               // ... - 1032 = q - 8, exact
  } else {
    const uint32_t w = rq[d >> 1][2 * (d & 1) + (b >> 1)] ^ 0x80808080u;  // codes + 128, bytes e0 e2 e1 e3
    t = ((w >> (8 * (b & 1))) & 0x00ff00ffu) | 0x64006400u;
    off = f16x2{(_Float16)1152.f, (_Float16)1152.f};
  }
  const f16x2 c = __builtin_bit_cast(f16x2, t) - off;              // v_pk_add_f16, exact
  const f16x2 r = c * dd;                                          // v_pk_mul_f16: one rounding
  if (PREC == 2) lo = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(c, dd, -r));  // v_pk_fma_f16
  return __builtin_bit_cast(uint32_t, r);
}

// One tile: `rows` (<= 32 TM) sorted positions from row0 x 128 TN channels from n0, NW weight matrices (1, or gate + up).
// PREC == 2 carries both operands as fp16 value + fp16 residual and adds the two first-order cross terms
// (wh*xh + wl*xh + wh*xl): the operands are then exact and the result is the fp32 sum of exact products.  The gate/up
// stage needs it: its output is re-quantized to Q8_0, and a relative perturbation eps of the values in front of that
// rounding step flips codes often enough to come out as about sqrt(eps/40) in relative L2.
template <int WT, int NW, int TM, int TN, int PREC>
__device__ __forceinline__ void qg_tile(const QG2Args& a, const int e, const int row0, const int rows, const int n0,
                                        unsigned char* smem) {
  constexpr int BK = 64, LDK = 2 * BK + 16, KS = BK / 16;
  constexpr int BM = TM * 32, WN = TN * 32;
  constexpr int CA = TM;  // 16-byte activation chunks per thread and K step: 32 TM rows x 8 chunks over 256 threads
  constexpr int STAGE = PREC * BM * LDK;  // value rows, then residual rows
  constexpr int QW = qg_nibbles(WT) ? 1 : 2;
  constexpr int SDW = qg_scale_dwords(WT);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, hi = lane >> 5;
  const int Kp = (int)qg_kp(a.K), kbs = Kp / 64, nbs = (int)(qg_np(a.N) / 32);
  const int64_t qbytes = qg_qbytes(WT, a.N, a.K), wbytes = qg_bytes(WT, a.N, a.K);

  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.xh), 0, (uint32_t)((int64_t)a.a_rows * a.K * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rW[NW];
  rW[0] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a.W0 + (size_t)e * a.wstride), 0, (uint32_t)wbytes, 0x00020000);
  if (NW == 2) rW[NW - 1] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a.W1 + (size_t)e * a.wstride), 0, (uint32_t)wbytes, 0x00020000);

  // activation chunk c of a thread: tile row (tid + 256 c) / 8, 16-byte column (tid + 256 c) % 8.  Rows past `rows` repeat
  // the last one (never stored); columns past K read as zeros so that the zero-padded weight tail meets no other row.
  uint32_t offA[CA];
  const int colA = (tid % 8) * 8;
#pragma unroll
  for (int c = 0; c < CA; c++) {
    const int pos = row0 + min((tid + c * 256) / 8, rows - 1);
    const int arow = a.a_index ? a.a_index[pos] / a.a_div : pos;
    offA[c] = (uint32_t)(((int64_t)arow * a.K + colA) * 2);
  }
  uint32_t offQ[TN], offS[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int nb = min((n0 + wave * WN) / 32 + j, nbs - 1);
    offQ[j] = (uint32_t)((int64_t)nb * kbs * (1024 * QW) + lane * 16);
    offS[j] = (uint32_t)(qbytes + ((int64_t)nb * kbs * 32 + lrow) * 4 * SDW);
  }
  const __amdgpu_buffer_rsrc_t rAl = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(PREC == 2 ? a.xl : a.xh), 0, (uint32_t)((int64_t)a.a_rows * a.K * 2), 0x00020000);
  auto loadA = [&](int k0, u32x4 (&ga)[PREC][CA]) {
    const bool ok = k0 + colA < a.K;
#pragma unroll
    for (int c = 0; c < CA; c++) {
      ga[0][c] = __builtin_amdgcn_raw_buffer_load_b128(rA, ok ? offA[c] : 0xffffffffu, k0 * 2, 0);
      if (PREC == 2) ga[PREC - 1][c] = __builtin_amdgcn_raw_buffer_load_b128(rAl, ok ? offA[c] : 0xffffffffu, k0 * 2, 0);
    }
  };
  auto storeA = [&](int buf, const u32x4 (&ga)[PREC][CA]) {
#pragma unroll
    for (int p = 0; p < PREC; p++)
#pragma unroll
      for (int c = 0; c < CA; c++) {
        const int idx = tid + c * 256;
        *reinterpret_cast<u32x4*>(smem + buf * STAGE + (p * BM + idx / 8) * LDK + (idx % 8) * 16) = ga[p][c];
      }
  };
  auto readA = [&](int buf, int ks, f16x8 (&fa)[PREC][TM]) {
#pragma unroll
    for (int p = 0; p < PREC; p++)
#pragma unroll
      for (int i = 0; i < TM; i++)
        fa[p][i] = *reinterpret_cast<const f16x8*>(smem + buf * STAGE + (p * BM + i * 32 + lrow) * LDK + ks * 32 + hi * 16);
  };

  v16f acc[NW][TN][TM];
#pragma unroll
  for (int w = 0; w < NW; w++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[w][j][i][r] = 0.f;

  u32x4 ga[PREC][CA];
  u32x4 rq[2][NW][TN][QW];      // packed codes of K steps kt (set kt & 1) and kt + 1
  uint32_t rs[2][NW][TN][SDW];  // their scale records
  f16x8 fb[2][NW][TN][PREC];    // dequantized operands of MFMA step ks (set ks & 1): value, residual
  f16x8 fa[2][PREC][TM];
  auto loadS = [&](uint32_t (&r)[SDW], int w, int j, int kb) {
    if (SDW == 1) {
      r[0] = __builtin_amdgcn_raw_buffer_load_b32(rW[w], offS[j], kb * 128, 0);
    } else {
      const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rW[w], offS[j], kb * 256, 0);
      r[0] = v.x;
      r[SDW - 1] = v.y;
    }
  };
  auto loadW = [&](int set, int kb) {
#pragma unroll
    for (int w = 0; w < NW; w++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int p = 0; p < QW; p++) rq[set][w][j][p] = __builtin_amdgcn_raw_buffer_load_b128(rW[w], offQ[j], (kb * QW + p) * 1024, 0);
        loadS(rs[set][w][j], w, j, kb);
      }
  };
  // the scale of dword d (K elements 16 d .. 16 d + 15 of the step) in both halves; for Q4_K also the offset
  auto scale2 = [&](const uint32_t (&s)[SDW], int d) -> f16x2 {
    uint32_t h;
    if constexpr (WT == MLLM_HIP_Q6_K) {
      const uint32_t v = s[d >> 1];
      h = (d & 1) ? (v >> 16) : (v & 0xffffu);
    } else {
      h = d < 2 ? (s[0] & 0xffffu) : (s[0] >> 16);
    }
    return __builtin_bit_cast(f16x2, h | (h << 16));
  };
  auto offset2 = [&](const uint32_t (&s)[SDW], int d) -> f16x2 {
    const uint32_t h = d < 2 ? (s[SDW - 1] & 0xffffu) : (s[SDW - 1] >> 16);
    return __builtin_bit_cast(f16x2, h | (h << 16));
  };
  // K range of this workgroup: all of it, or (short batches, one matrix) range blockIdx.z of a.ksplit, written to its own
  // partial result; the ranges start at even K steps
  int kt0 = 0, kt1 = Kp / BK;  // even
  float* outp = a.out;
  const float* biasp = a.bias;
  if (NW == 1 && a.ksplit > 1) {
    const int per = ((kt1 + a.ksplit - 1) / a.ksplit + 1) / 2 * 2;
    kt0 = (int)blockIdx.z * per;
    kt1 = min(kt1, kt0 + per);
    outp = a.partial + (size_t)blockIdx.z * a.a_rows * a.N;
    biasp = nullptr;
  }
  loadA(kt0 * BK, ga);
  loadW(0, kt0);
  loadW(1, kt0 + 1);
  storeA(0, ga);
  __syncthreads();
  readA(0, 0, fa[0]);
#pragma unroll
  for (int w = 0; w < NW; w++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const f16x2 dd = scale2(rs[0][w][j], 0), dm = offset2(rs[0][w][j], 0);
      uint32_t o[4], ol[4] = {0, 0, 0, 0};
#pragma unroll
      for (int b = 0; b < 4; b++) o[b] = qg_pair<WT, PREC>(rq[0][w][j], 0, b, dd, dm, ol[b]);
      fb[0][w][j][0] = __builtin_bit_cast(f16x8, u32x4{o[0], o[1], o[2], o[3]});
      if (PREC == 2) fb[0][w][j][PREC - 1] = __builtin_bit_cast(f16x8, u32x4{ol[0], ol[1], ol[2], ol[3]});
    }

  // one K step (64 elements) with its weights in register set CUR; refills that set with K step kt + 2 when done with it
  auto kstep = [&](auto cur_tag, int kt) {
    constexpr int CUR = decltype(cur_tag)::value;
    const int buf = kt & 1;
    loadA((kt + 1) * BK, ga);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (ks < KS - 1) {
        readA(buf, ks + 1, fa[(ks + 1) & 1]);  // the next step's activations while this one's MFMAs run
      } else {
        storeA(buf ^ 1, ga);
        __syncthreads();
        readA(buf ^ 1, 0, fa[(ks + 1) & 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
      const int ns = ks < KS - 1 ? CUR : CUR ^ 1, nd = (ks + 1) % KS;  // register set and dword of the NEXT step's weights
#pragma unroll
      for (int w = 0; w < NW; w++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
          // the dequantization of the next step's operand is cut into TM pieces, one pinned into the shadow of each MFMA
          const f16x2 dd = scale2(rs[ns][w][j], nd), dm = offset2(rs[ns][w][j], nd);
          uint32_t o[4], ol[4] = {0, 0, 0, 0};
#pragma unroll
          for (int i = 0; i < TM; i++) {
            acc[w][j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ks & 1][w][j][0], fa[ks & 1][0][i], acc[w][j][i], 0, 0, 0);
            if (PREC == 2) {
              acc[w][j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ks & 1][w][j][PREC - 1], fa[ks & 1][0][i], acc[w][j][i], 0, 0, 0);
              acc[w][j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ks & 1][w][j][0], fa[ks & 1][PREC - 1][i], acc[w][j][i], 0, 0, 0);
            }
#pragma unroll
            for (int b = i * 4 / TM; b < (i + 1) * 4 / TM; b++) o[b] = qg_pair<WT, PREC>(rq[ns][w][j], nd, b, dd, dm, ol[b]);
            __builtin_amdgcn_sched_barrier(0);
          }
          fb[(ks + 1) & 1][w][j][0] = __builtin_bit_cast(f16x8, u32x4{o[0], o[1], o[2], o[3]});
          if (PREC == 2) fb[(ks + 1) & 1][w][j][PREC - 1] = __builtin_bit_cast(f16x8, u32x4{ol[0], ol[1], ol[2], ol[3]});
          if (ks == KS - 2) {  // the set's last dword is consumed: fetch K step kt + 2 into it
#pragma unroll
            for (int p = 0; p < QW; p++)
              rq[CUR][w][j][p] = __builtin_amdgcn_raw_buffer_load_b128(rW[w], offQ[j], ((kt + 2) * QW + p) * 1024, 0);
            loadS(rs[CUR][w][j], w, j, kt + 2);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
    }
  };
  for (int kt = kt0; kt < kt1; kt += 2) {
    kstep(std::integral_constant<int, 0>{}, kt);
    kstep(std::integral_constant<int, 1>{}, kt + 1);
  }
  __syncthreads();

  // acc[w][j][i][4g+e] = result[row0 + 32i + lrow][n0 + wave*WN + 32j + 8g + 4hi + e]
  if (NW == 1) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int r = i * 32 + lrow;
      if (r < rows) {
        const int pos = row0 + r;
        float* orow = outp + (int64_t)(a.o_index ? a.o_index[pos] : pos) * a.N;
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            const int n = n0 + wave * WN + j * 32 + 8 * g + 4 * hi;
            f32x4 v = {acc[0][j][i][4 * g], acc[0][j][i][4 * g + 1], acc[0][j][i][4 * g + 2], acc[0][j][i][4 * g + 3]};
            if (n + 3 < a.N && a.N % 4 == 0) {
              if (biasp) v += *reinterpret_cast<const f32x4*>(biasp + n);
              *reinterpret_cast<f32x4*>(orow + n) = v;
            } else {
#pragma unroll
              for (int e2 = 0; e2 < 4; e2++)
                if (n + e2 < a.N) orow[n + e2] = biasp ? v[e2] + biasp[n + e2] : v[e2];
            }
          }
      }
    }
  } else {
    // h = silu(gate) * up, Q8_0 round trip over each block of 32 channels (a block is one column tile j: 16 channels in
    // this lane, 16 in lane ^ 32), written as fp16 for the next Linear
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int r = i * 32 + lrow;
#pragma unroll
      for (int j = 0; j < TN; j++) {
        float h[16];
        float amax = 0.f;
#pragma unroll
        for (int q = 0; q < 16; q++) {
          h[q] = silu_f(acc[0][j][i][q]) * acc[NW - 1][j][i][q];
          amax = fmaxf(amax, fabsf(h[q]));
        }
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        const float d = amax / 127.f;
        const float idv = (amax != 0.f) ? 127.f / amax : 0.f;
        uint16_t bits = f32_to_f16bits(d);
        if (a.x86_scale) bits = x86_scale_bits(bits);
        const float deff = f16bits_to_f32(bits);
        if (r < rows) {
          uint16_t* hrow = a.hh + (int64_t)(row0 + r) * a.N;
#pragma unroll
          for (int g = 0; g < 4; g++) {
            const int n = n0 + wave * WN + j * 32 + 8 * g + 4 * hi;
            uint32_t o[2];
#pragma unroll
            for (int e2 = 0; e2 < 2; e2++) {
              const int q0 = min(127, max(-128, (int)rintf(h[4 * g + 2 * e2] * idv)));
              const int q1 = min(127, max(-128, (int)rintf(h[4 * g + 2 * e2 + 1] * idv)));
              o[e2] = (uint32_t)f32_to_f16bits(deff * (float)q0) | ((uint32_t)f32_to_f16bits(deff * (float)q1) << 16);
            }
            if (n + 3 < a.N) *reinterpret_cast<uint2*>(hrow + n) = uint2{o[0], o[1]};
          }
        }
      }
    }
  }
}

// MODE 0: one matrix, 128 x 256 tiles, one-term operands.  MODE 1: gate and up together with two-term operands; a tile of
// the list is cut into halves of 64 rows (blockIdx.z) x 128 channels.
// The tile height follows the rows the tile really has: short tiles skip the MFMAs of empty row blocks.
template <int WT, int MODE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void qg_kernel(QG2Args a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int t = blockIdx.x;
  if (t >= min(a.ntiles[0], (int)gridDim.x)) return;
  const int e = a.tile_expert[t];
  int row0 = a.tile_row0[t], rows = a.tile_rows[t];
  if constexpr (MODE == 1) {
    const int n0 = blockIdx.y * 128;
    row0 += 64 * blockIdx.z;
    rows -= 64 * blockIdx.z;
    if (rows <= 0) return;
    if (rows > 32) qg_tile<WT, 2, 2, 1, 2>(a, e, row0, min(rows, 64), n0, smem);
    else qg_tile<WT, 2, 1, 1, 2>(a, e, row0, rows, n0, smem);
  } else {
    const int n0 = blockIdx.y * 256;
    if (rows > 64) qg_tile<WT, 1, 4, 2, 1>(a, e, row0, rows, n0, smem);
    else if (rows > 32) qg_tile<WT, 1, 2, 2, 1>(a, e, row0, rows, n0, smem);
    else qg_tile<WT, 1, 1, 2, 1>(a, e, row0, rows, n0, smem);
  }
}

constexpr int QG_TILE_H = 128;

template <int MODE>
static int launch_qg(const QG2Args& a, unsigned max_tiles, hipStream_t st) {
  constexpr int TN = MODE == 1 ? 1 : 2;
  const dim3 grid(max_tiles, (unsigned)((a.N + 128 * TN - 1) / (128 * TN)), MODE == 1 ? 2 : (unsigned)(a.ksplit > 1 ? a.ksplit : 1));
  const size_t lds = 2 * (size_t)QG_TILE_H * (2 * 64 + 16);  // MODE 1: half the rows, value + residual
  if (a.wtype == MLLM_HIP_Q4_0) hipLaunchKernelGGL((qg_kernel<MLLM_HIP_Q4_0, MODE>), grid, dim3(256), lds, st, a);
  else if (a.wtype == MLLM_HIP_Q8_0) hipLaunchKernelGGL((qg_kernel<MLLM_HIP_Q8_0, MODE>), grid, dim3(256), lds, st, a);
  else if constexpr (MODE == 0) {  // the super-block formats: plain Linear only
    if (a.wtype == MLLM_HIP_Q4_K) hipLaunchKernelGGL((qg_kernel<MLLM_HIP_Q4_K, 0>), grid, dim3(256), lds, st, a);
    else hipLaunchKernelGGL((qg_kernel<MLLM_HIP_Q6_K, 0>), grid, dim3(256), lds, st, a);
  } else return MLLM_HIP_E_BADARG;
  return (int)hipGetLastError();
}

// =========================================================================================================
// Exact block sums on the matrix cores ("qx"): the reference's arithmetic itself for many rows
//
//   y[row][n] = sum_b fp32(dW[n][b] * dX[row][b]) * float(sum_32 qW * qX)
//
// (llamafile_sgemm.cpp:697-743: Cv += set1(dW * dX) * float(int32 block sum)).  Per 32-row x 32-channel tile and block,
// four v_mfma_f32_32x32x16_f16 and sixteen fp32 FMAs:
//   * the block sum: two MFMAs whose operands are integers held as fp16 numbers.  The activation codes are stored that
//     way; a weight code is OR-ed into the mantissa of 1024.0 (nibble at bits 0..3 of a half-word) or of 64.0 (bits
//     4..7), i.e. it enters as 1024 + q or 64 + q (q = 0..15; Q8_0: 1024 + 128 + q), which costs five operations per
//     eight 4-bit codes.  A third MFMA puts the correction in front: its operands are the constants -(1024 + 8),
//     -(64 + 8) and the sums of the activation codes that meet each constant (two per row and block, from the producer
//     of the activations), so the chain starts at -sum(offset * qX) and ends at sum((q - 8) * qX).  Every product and
//     every partial sum is an integer below 2^24: the fp32 result IS the int32 block sum, already a float.
//   * the 32 x 32 scale products dW[n] * dX[row]: a fourth MFMA, an outer product of the two fp16 scales sitting in one
//     K slot of otherwise zero operands; an 11-bit by 11-bit product is exact in fp32.
//   * acc = fma(dW * dX, block sum, acc): the reference's operation.  Only the order in which blocks are added differs
//     from the CPU path.
// Same gemm-packed weights and tile list as the fp16-operand kernel.  Activations: Q8_0 codes as fp16 integers
// [rows][K] and one record of three dwords per row and K step of 64: the fp16 scales of the step's two blocks, then per
// block the two partial code sums (elements with bit 1 of k clear | set) as fp16 integers.
// =========================================================================================================
struct QXArgs {
  const char* W0;        // gemm-packed weights of matrix 0 (gate, or the only matrix), expert e at W0 + e * wstride
  const char* W1;        // matrix 1 (up) in the gate/up mode
  size_t wstride;
  const uint16_t* xq;    // Q8_0 codes of the activations as fp16 integers [a_rows][K]
  const uint32_t* xd;    // [a_rows][KD][3] dwords: fp16 scales of blocks 2j | 2j+1, then per block fp16(sum of the codes
                         // with (k & 2) == 0) | fp16(sum of the others) << 16; zeros past the end
  const int* a_index;    // activation row of sorted position pos is a_index[pos] / a_div ; null: pos itself
  int a_div;
  int a_rows;
  const int* o_index;    // output row of sorted position pos (null: pos itself)
  float* out;            // fp32 [..][N]       (one-matrix mode)
  const float* bias;     // [N] or null        (one-matrix mode)
  uint16_t* hq;          // gate/up mode: Q8_0 codes of silu(g)*u as fp16 integers [rows][N]
  uint32_t* hd;          // gate/up mode: their records [rows][ceil(N/64)][3], as xd
  const int* tile_expert;
  const int* tile_row0;
  const int* tile_rows;
  const int* ntiles;
  int N, K;
  int x86_scale;
  int half_tiles;        // tiles of at most sixteen rows take the 16-row form (same bits; 0: comparison runs and tests)
};

// masks and exponent patterns of qx_codes, kept in registers (v_and_or_b32 takes no literal constants)
struct QXConst {
  uint32_t m_lo, m_hi, e_1024, e_64;
};
__device__ __forceinline__ QXConst qx_const(int wtype) {
  QXConst c{wtype == MLLM_HIP_Q4_0 ? 0x000f000fu : 0x00ff00ffu, 0x00f000f0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+v"(c.m_lo), "+v"(c.m_hi), "+v"(c.e_1024), "+v"(c.e_64));
  return c;
}
// the eight weight codes of MFMA step d (16 K elements, this lane's half) as fp16 numbers offset + code:
// Q4_0: 1024 + q for the elements with (k & 2) == 0, 64 + q for the others (q = 0..15); Q8_0: 1152 + q (q = -128..127)
// ... from the dwords themselves: Q4_0 one dword (v1 unused), Q8_0 two
template <int WT>
__device__ __forceinline__ f16x8 qx_codes_dw(uint32_t v0, uint32_t v1, const QXConst& c) {
  uint32_t o[4];
  if (WT == MLLM_HIP_Q4_0) {
    // pair i of the dword sits in nibbles i and 4 + i.  Nibbles at bits 0..3 of a half-word land in the mantissa of 1024.0
    // (unit 1), nibbles at bits 4..7 in the mantissa of 64.0 (unit 1/16): pairs 0 and 1 need no shift, pairs 2 and 3 one
    // shift by 8 for both.
    const uint32_t t = v0 >> 8;
    o[0] = (v0 & c.m_lo) | c.e_1024;
    o[1] = (v0 & c.m_hi) | c.e_64;
    o[2] = (t & c.m_lo) | c.e_1024;
    o[3] = (t & c.m_hi) | c.e_64;
  } else {
    // two dwords of four codes each in byte order e0 e2 e1 e3; + 128 makes them unsigned
    const uint32_t w0 = v0 ^ 0x80808080u, w1 = v1 ^ 0x80808080u;
    o[0] = (w0 & c.m_lo) | c.e_1024;
    o[1] = ((w0 >> 8) & c.m_lo) | c.e_1024;
    o[2] = (w1 & c.m_lo) | c.e_1024;
    o[3] = ((w1 >> 8) & c.m_lo) | c.e_1024;
  }
  return __builtin_bit_cast(f16x8, u32x4{o[0], o[1], o[2], o[3]});
}
template <int WT>
__device__ __forceinline__ f16x8 qx_codes(const u32x4 (&rq)[WT == MLLM_HIP_Q4_0 ? 1 : 2], int d, const QXConst& c) {
  if (WT == MLLM_HIP_Q4_0) return qx_codes_dw<WT>(rq[0][d], 0u, c);
  return qx_codes_dw<WT>(rq[d >> 1][2 * (d & 1)], rq[d >> 1][2 * (d & 1) + 1], c);
}
// fp16 pair (-offset of the elements with (k & 2) == 0, -offset of the others) including the 8 of Q4_0's code offset
__host__ __device__ constexpr uint32_t qx_offsets(int wtype) { return wtype == MLLM_HIP_Q4_0 ? 0xD480E408u : 0xE480E480u; }

// One tile: `rows` (<= 32 TM) sorted positions from row0 x 128 TN channels from n0, NW weight matrices (1, or gate + up).
template <int WT, int NW, int TM, int TN>
__device__ __forceinline__ void qx_tile(const QXArgs& a, const int e, const int row0, const int rows, const int n0,
                                        unsigned char* smem) {
  constexpr int BK = 64, LDK = 2 * BK + 16;
  constexpr int BM = TM * 32, WN = TN * 32;
  constexpr int CA = TM;                      // 16-byte activation chunks per thread and K step
  constexpr int STAGE = BM * LDK + BM * 48;   // code rows, then per row the record's three dwords, each the first of a
                                              // 16-byte MFMA operand whose other K slots are zero
  constexpr int QW = WT == MLLM_HIP_Q4_0 ? 1 : 2;
  constexpr int ST = 4;                       // K steps of weights in flight per wave

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, hi = lane >> 5;
  const int Kp = (int)qg_kp(a.K), kbs = Kp / 64, nbs = (int)(qg_np(a.N) / 32), KD = (a.K + 63) / 64;
  const int64_t qbytes = qg_qbytes(WT, a.N, a.K), wbytes = qg_bytes(WT, a.N, a.K);

  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.xq), 0, (uint32_t)((int64_t)a.a_rows * a.K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rD = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(a.xd), 0, (uint32_t)((int64_t)a.a_rows * KD * 12), 0x00020000);
  __amdgpu_buffer_rsrc_t rW[NW];
  rW[0] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a.W0 + (size_t)e * a.wstride), 0, (uint32_t)wbytes, 0x00020000);
  if (NW == 2) rW[NW - 1] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a.W1 + (size_t)e * a.wstride), 0, (uint32_t)wbytes, 0x00020000);

  // activation chunk c of a thread: tile row (tid + 256 c) / 8, 16-byte column (tid + 256 c) % 8.  Rows past `rows` repeat
  // the last one (never stored); columns past K read as zeros (out-of-range buffer offsets).
  uint32_t offA[CA];
  const int colA = (tid % 8) * 8;
#pragma unroll
  for (int c = 0; c < CA; c++) {
    const int pos = row0 + min((tid + c * 256) / 8, rows - 1);
    const int arow = a.a_index ? a.a_index[pos] / a.a_div : pos;
    offA[c] = (uint32_t)(((int64_t)arow * a.K + colA) * 2);
  }
  // the record of a row and K step: threads 0 .. BM-1, one row each
  uint32_t offD = 0xffffffffu;
  if (tid < BM) {
    const int pos = row0 + min(tid, rows - 1);
    const int arow = a.a_index ? a.a_index[pos] / a.a_div : pos;
    offD = (uint32_t)((int64_t)arow * KD * 12);
  }
  uint32_t offQ[TN], offS[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int nb = min((n0 + wave * WN) / 32 + j, nbs - 1);
    offQ[j] = (uint32_t)((int64_t)nb * kbs * (1024 * QW) + lane * 16);
    offS[j] = (uint32_t)(qbytes + ((int64_t)nb * kbs * 32 + lrow) * 4);
  }
  typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
  // Activations travel two K steps ahead of their use, in two register sets.  Vector memory returns in order: the wait for
  // a step's activations also waits for every load issued before them, so loading them only one step ahead would cut
  // the weights' lead (ST steps) down to one step as well.
  u32x4 ga[2][CA];
  u32x3 gd[2] = {{0u, 0u, 0u}, {0u, 0u, 0u}};
  auto loadA = [&](int set, int kt) {
    const bool ok = kt * BK + colA < a.K;
#pragma unroll
    for (int c = 0; c < CA; c++) ga[set][c] = __builtin_amdgcn_raw_buffer_load_b128(rA, ok ? offA[c] : 0xffffffffu, kt * BK * 2, 0);
    if (tid < BM) gd[set] = __builtin_amdgcn_raw_buffer_load_b96(rD, kt < KD ? offD : 0xffffffffu, kt * 12, 0);
  };
  auto storeA = [&](int set, int buf) {
#pragma unroll
    for (int c = 0; c < CA; c++) {
      const int idx = tid + c * 256;
      *reinterpret_cast<u32x4*>(smem + buf * STAGE + (idx / 8) * LDK + (idx % 8) * 16) = ga[set][c];
    }
    if (tid < BM) {
      u32x4* rec = reinterpret_cast<u32x4*>(smem + buf * STAGE + BM * LDK + tid * 48);
      rec[0] = u32x4{gd[set].x, 0u, 0u, 0u};
      rec[1] = u32x4{gd[set].y, 0u, 0u, 0u};
      rec[2] = u32x4{gd[set].z, 0u, 0u, 0u};
    }
  };

  v16f acc[NW][TN][TM];
#pragma unroll
  for (int w = 0; w < NW; w++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[w][j][i][r] = 0.f;

  u32x4 rq[ST][NW][TN][QW];  // packed codes of the K steps in flight (ring, slot = step % ST)
  uint32_t rs[ST][NW][TN];   // their scale dwords
  auto loadW = [&](int slot, int kt) {
    const bool ok = kt < kbs;  // steps past the end read nothing (zeros): the ring is always full
#pragma unroll
    for (int w = 0; w < NW; w++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int p = 0; p < QW; p++)
          rq[slot][w][j][p] = __builtin_amdgcn_raw_buffer_load_b128(rW[w], ok ? offQ[j] : 0xffffffffu, (kt * QW + p) * 1024, 0);
        rs[slot][w][j] = __builtin_amdgcn_raw_buffer_load_b32(rW[w], ok ? offS[j] : 0xffffffffu, kt * 128, 0);
      }
  };
  // Scale operand of the weights: the fp16 scale of the step's first block in K slot 0 (low half of the first register), of
  // its second block in K slot 1 (high half), in the lanes of the low K half only; every other K slot is zero.  The
  // activations' scale pair and code sums are used as they come (first register of an otherwise zero operand): what a K
  // slot holds does not matter where the other operand is zero.
  static_assert(TM == 1, "one row tile per workgroup");
  const uint32_t msk0 = hi ? 0u : 0x0000ffffu, msk1 = hi ? 0u : 0xffff0000u;
  const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const QXConst kc = qx_const(WT);
  const f16x8 off_op = __builtin_bit_cast(f16x8, u32x4{hi ? 0u : qx_offsets(WT), 0u, 0u, 0u});

  // A "group" is one (block, matrix, column tile): four MFMAs (offset correction, shared by the matrices of a block; two
  // for the block sum; the scale product) and sixteen FMAs.  A wave issues in order and a dependent MFMA holds it until its
  // input is ready, so everything else is slotted between the MFMAs of one group: the unpacking of the NEXT group's weight
  // codes and the FMAs of the PREVIOUS group (whose MFMA results sit in the other of two register sets).  The matrix pipe
  // then runs back to back while the vector ALU works in its shadow, within one wave.
  constexpr int G = 2 * NW * TN;  // groups per K step: block-major, then matrix, then column tile
  f16x8 fw[2][2];                 // unpacked codes of the current / next group (two MFMA steps each)
  u32x4 sw[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};  // their scale operands
  v16f T[2], S[2];                // block sums and scale products of the current / previous group
  T[1] = zero16;
  S[1] = zero16;

  const int nsteps = (kbs + ST - 1) / ST * ST;
  loadA(0, 0);
  loadA(1, 1);
#pragma unroll
  for (int s = 0; s < ST; s++) loadW(s, s);
  storeA(0, 0);
  // the first group's operands
  fw[0][0] = qx_codes<WT>(rq[0][0][0], 0, kc);
  fw[0][1] = qx_codes<WT>(rq[0][0][0], 1, kc);
  sw[0].x = rs[0][0][0] & msk0;
  __syncthreads();

  // one K step (64 elements = two blocks) with its weights in ring slot SLOT; refills the slot with step kt + ST
  auto kstep = [&](auto slot_tag, int kt) {
    constexpr int SLOT = decltype(slot_tag)::value;
    constexpr int NSLOT = (SLOT + 1) % ST;
    const int buf = kt & 1;
    loadA(SLOT & 1, kt + 2);  // the set whose step (kt) is in LDS already
    f16x8 fb[2][2];
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int d = 0; d < 2; d++)
        fb[b][d] = *reinterpret_cast<const f16x8*>(smem + buf * STAGE + lrow * LDK + (2 * b + d) * 32 + hi * 16);
    // the row's scale pair (both scales: the weight operand is zero in the other block's K slot) and its two code-sum pairs,
    // each already an operand
    f16x8 rec[3];
#pragma unroll
    for (int q = 0; q < 3; q++) rec[q] = *reinterpret_cast<const f16x8*>(smem + buf * STAGE + BM * LDK + lrow * 48 + q * 16);
    v16f tc = zero16;
#pragma unroll
    for (int g = 0; g < G; g++) {
      constexpr int cur = 0;  // the register sets alternate by the parity of g (G is even)
      const int c = (g + cur) & 1, n = c ^ 1;
      const int b = g / (NW * TN), w = (g / TN) % NW, j = g % TN;
      // the next group: (b', w', j') in this step, or the first group of the next step (ring slot NSLOT)
      const bool last = g == G - 1;
      const int gn = last ? 0 : g + 1;
      const int bn = gn / (NW * TN), wn = (gn / TN) % NW, jn = gn % TN;
      __builtin_amdgcn_sched_barrier(0);
      if (w == 0 && j == 0) {  // the block's correction, shared by all its groups
        tc = __builtin_amdgcn_mfma_f32_32x32x16_f16(off_op, rec[1 + b], zero16, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (last) fw[n][0] = qx_codes<WT>(rq[NSLOT][wn][jn], 2 * bn, kc);
      else fw[n][0] = qx_codes<WT>(rq[SLOT][wn][jn], 2 * bn, kc);
      __builtin_amdgcn_sched_barrier(0);
      T[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[c][0], fb[b][0], tc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (last) {
        fw[n][1] = qx_codes<WT>(rq[NSLOT][wn][jn], 2 * bn + 1, kc);
        sw[n].x = rs[NSLOT][wn][jn] & msk0;
      } else {
        fw[n][1] = qx_codes<WT>(rq[SLOT][wn][jn], 2 * bn + 1, kc);
        sw[n].x = rs[SLOT][wn][jn] & (bn ? msk1 : msk0);
        if (bn == 1) {  // both blocks of (wn, jn) are unpacked: its ring registers are free, fetch K step kt + ST into them
#pragma unroll
          for (int p = 0; p < QW; p++)
            rq[SLOT][wn][jn][p] = __builtin_amdgcn_raw_buffer_load_b128(rW[wn], kt + ST < kbs ? offQ[jn] : 0xffffffffu, ((kt + ST) * QW + p) * 1024, 0);
          rs[SLOT][wn][jn] = __builtin_amdgcn_raw_buffer_load_b32(rW[wn], kt + ST < kbs ? offS[jn] : 0xffffffffu, (kt + ST) * 128, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      S[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, sw[c]), rec[0], zero16, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      // the FMAs of the previous group (of the previous step's last group when g == 0): first half
      const int pg = g == 0 ? G - 1 : g - 1;
      const int pw = (pg / TN) % NW, pj = pg % TN;
#pragma unroll
      for (int r = 0; r < 8; r++) acc[pw][pj][0][r] = fmaf(S[n][r], T[n][r], acc[pw][pj][0][r]);
      asm volatile("" : "+v"(acc[pw][pj][0]));  // pins the FMAs here (the compiler otherwise sinks them to the end of the body)
      __builtin_amdgcn_sched_barrier(0);
      T[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[c][1], fb[b][1], T[c], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 8; r < 16; r++) acc[pw][pj][0][r] = fmaf(S[n][r], T[n][r], acc[pw][pj][0][r]);
      asm volatile("" : "+v"(acc[pw][pj][0]));
      __builtin_amdgcn_sched_barrier(0);
    }
    storeA((SLOT & 1) ^ 1, buf ^ 1);
    __syncthreads();
  };
  for (int kt = 0; kt < nsteps; kt += ST) {
    kstep(std::integral_constant<int, 0>{}, kt);
    kstep(std::integral_constant<int, 1>{}, kt + 1);
    kstep(std::integral_constant<int, 2>{}, kt + 2);
    kstep(std::integral_constant<int, 3>{}, kt + 3);
  }
  // the last group's FMAs (G even: its results are in set 1)
#pragma unroll
  for (int r = 0; r < 16; r++) acc[NW - 1][TN - 1][0][r] = fmaf(S[1][r], T[1][r], acc[NW - 1][TN - 1][0][r]);

  // acc[w][j][i][4g+e] = result[row0 + 32i + lrow][n0 + wave*WN + 32j + 8g + 4hi + e]
  if (NW == 1) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int r = i * 32 + lrow;
      if (r < rows) {
        const int pos = row0 + r;
        float* orow = a.out + (int64_t)(a.o_index ? a.o_index[pos] : pos) * a.N;
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            const int n = n0 + wave * WN + j * 32 + 8 * g + 4 * hi;
            f32x4 v = {acc[0][j][i][4 * g], acc[0][j][i][4 * g + 1], acc[0][j][i][4 * g + 2], acc[0][j][i][4 * g + 3]};
            if (n + 3 < a.N && a.N % 4 == 0) {
              if (a.bias) v += *reinterpret_cast<const f32x4*>(a.bias + n);
              *reinterpret_cast<f32x4*>(orow + n) = v;
            } else {
#pragma unroll
              for (int e2 = 0; e2 < 4; e2++)
                if (n + e2 < a.N) orow[n + e2] = a.bias ? v[e2] + a.bias[n + e2] : v[e2];
            }
          }
      }
    }
  } else {
    // h = silu(gate) * up, quantized to Q8_0 over each block of 32 channels (a block is one column tile j: 16 channels in
    // this lane, 16 in lane ^ 32): codes as fp16 integers and the fp16 scale, the next Linear's activation format
    const int nblk = a.N / QK, KDo = (a.N + 63) / 64;
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int r = i * 32 + lrow;
#pragma unroll
      for (int j = 0; j < TN; j++) {
        float h[16];
        float amax = 0.f;
#pragma unroll
        for (int q = 0; q < 16; q++) {
          h[q] = silu_f(acc[0][j][i][q]) * acc[NW - 1][j][i][q];
          amax = fmaxf(amax, fabsf(h[q]));
        }
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        const float d = amax / 127.f;
        const float idv = (amax != 0.f) ? 127.f / amax : 0.f;
        uint16_t bits = f32_to_f16bits(d);
        if (a.x86_scale) bits = x86_scale_bits(bits);
        const int blk = (n0 + wave * WN) / 32 + j;
        // element 8g + 4hi + e of the block: bit 1 of its index is bit 1 of e
        int qv[16], sa = 0, sb = 0;
#pragma unroll
        for (int q = 0; q < 16; q++) {
          qv[q] = min(127, max(-128, (int)rintf(h[q] * idv)));
          if (q & 2) sb += qv[q];
          else sa += qv[q];
        }
        sa += __shfl_xor(sa, 32, 64);
        sb += __shfl_xor(sb, 32, 64);
        if (r < rows && blk < nblk) {
          uint16_t* hrow = a.hq + (int64_t)(row0 + r) * a.N;
#pragma unroll
          for (int g = 0; g < 4; g++) {
            const int n = n0 + wave * WN + j * 32 + 8 * g + 4 * hi;
            uint32_t o[2];
#pragma unroll
            for (int e2 = 0; e2 < 2; e2++)
              o[e2] = (uint32_t)f32_to_f16bits((float)qv[4 * g + 2 * e2]) | ((uint32_t)f32_to_f16bits((float)qv[4 * g + 2 * e2 + 1]) << 16);
            *reinterpret_cast<uint2*>(hrow + n) = uint2{o[0], o[1]};
          }
          if (hi == 0) {
            uint32_t* recp = a.hd + ((int64_t)(row0 + r) * KDo + (blk >> 1)) * 3;
            reinterpret_cast<uint16_t*>(recp)[blk & 1] = bits;
            recp[1 + (blk & 1)] = (uint32_t)f32_to_f16bits((float)sa) | ((uint32_t)f32_to_f16bits((float)sb) << 16);
            if (blk == nblk - 1 && (nblk & 1)) {  // the unused half of the last record
              reinterpret_cast<uint16_t*>(recp)[1] = 0;
              recp[2] = 0;
            }
          }
        }
      }
    }
  }
}


// The same tile for at most SIXTEEN sorted positions: v_mfma_f32_16x16x32_f16 takes a whole block of 32 elements per
// instruction for 16 channels x 16 rows, so a tile of up to 16 rows costs half the matrix time (and half the FMAs) of the
// 32-row form above, which would pad it to 32.  Same packed weights: a lane of the 32-row layout holds, of channel lane % 32,
// the block's elements 8 hi .. 8 hi + 7 (MFMA step 0) and 16 + 8 hi .. (step 1); the 16-row operand wants, in lane
// (channel c, K group kg), eight elements of channel c [+ 16].  v_permlane16_swap on the PACKED dwords (step 0 as first
// operand, step 1 as second) leaves in the first the channels 0..15 and in the second the channels 16..31, each with K
// groups (hi 0, step 0), (hi 0, step 1), (hi 1, step 0), (hi 1, step 1); the activation operand is read from LDS in that
// order of K, so the products that meet are the same and every sum is the same exact integer.  Same scale products,
// same FMAs per block, same order of blocks: the same bits as the 32-row form row by row.
template <int WT, int NW, int TN>
__device__ __forceinline__ void qx_tile16(const QXArgs& a, const int e, const int row0, const int rows, const int n0,
                                          unsigned char* smem) {
  constexpr int BK = 64, LDK = 2 * BK + 16;
  constexpr int BM = 16, WN = TN * 32;
  constexpr int STAGE = BM * LDK + BM * 48;
  constexpr int QW = WT == MLLM_HIP_Q4_0 ? 1 : 2;
  constexpr int ST = 4;  // K steps of weights in flight per wave

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31;             // channel of this lane in the packed layout
  const int c16 = lane & 15, kg = lane >> 4;  // 16-row operands: channel / row c16, K group kg
  const int Kp = (int)qg_kp(a.K), kbs = Kp / 64, nbs = (int)(qg_np(a.N) / 32), KD = (a.K + 63) / 64;
  const int64_t qbytes = qg_qbytes(WT, a.N, a.K), wbytes = qg_bytes(WT, a.N, a.K);

  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.xq), 0, (uint32_t)((int64_t)a.a_rows * a.K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rD = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(a.xd), 0, (uint32_t)((int64_t)a.a_rows * KD * 12), 0x00020000);
  __amdgpu_buffer_rsrc_t rW[NW];
  rW[0] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a.W0 + (size_t)e * a.wstride), 0, (uint32_t)wbytes, 0x00020000);
  if (NW == 2) rW[NW - 1] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a.W1 + (size_t)e * a.wstride), 0, (uint32_t)wbytes, 0x00020000);

  // activation chunk of threads 0 .. 127: tile row tid / 8, 16-byte column tid % 8; record of a row: threads 0 .. 15.
  // Rows past `rows` repeat the last one (never stored); columns past K read as zeros.
  const bool ldA = tid < BM * 8;
  const int colA = (tid % 8) * 8;
  uint32_t offA = 0xffffffffu, offD = 0xffffffffu;
  if (ldA) {
    const int pos = row0 + min(tid / 8, rows - 1);
    const int arow = a.a_index ? a.a_index[pos] / a.a_div : pos;
    offA = (uint32_t)(((int64_t)arow * a.K + colA) * 2);
  }
  if (tid < BM) {
    const int pos = row0 + min(tid, rows - 1);
    const int arow = a.a_index ? a.a_index[pos] / a.a_div : pos;
    offD = (uint32_t)((int64_t)arow * KD * 12);
  }
  uint32_t offQ[TN], offS[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int nb = min((n0 + wave * WN) / 32 + j, nbs - 1);
    offQ[j] = (uint32_t)((int64_t)nb * kbs * (1024 * QW) + lane * 16);
    offS[j] = (uint32_t)(qbytes + ((int64_t)nb * kbs * 32 + lrow) * 4);
  }
  typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
  u32x4 ga[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
  u32x3 gd[2] = {{0u, 0u, 0u}, {0u, 0u, 0u}};
  auto loadA = [&](int set, int kt) {  // two K steps ahead of their use, as in the 32-row form
    if (ldA) ga[set] = __builtin_amdgcn_raw_buffer_load_b128(rA, kt * BK + colA < a.K ? offA : 0xffffffffu, kt * BK * 2, 0);
    if (tid < BM) gd[set] = __builtin_amdgcn_raw_buffer_load_b96(rD, kt < KD ? offD : 0xffffffffu, kt * 12, 0);
  };
  auto storeA = [&](int set, int buf) {
    if (ldA) *reinterpret_cast<u32x4*>(smem + buf * STAGE + (tid / 8) * LDK + (tid % 8) * 16) = ga[set];
    if (tid < BM) {
      u32x4* rec = reinterpret_cast<u32x4*>(smem + buf * STAGE + BM * LDK + tid * 48);
      rec[0] = u32x4{gd[set].x, 0u, 0u, 0u};
      rec[1] = u32x4{gd[set].y, 0u, 0u, 0u};
      rec[2] = u32x4{gd[set].z, 0u, 0u, 0u};
    }
  };

  f32x4 acc[NW][TN][2];  // [matrix][column tile][channel half]
#pragma unroll
  for (int w = 0; w < NW; w++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int h = 0; h < 2; h++) acc[w][j][h] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 rq[ST][NW][TN][QW];
  uint32_t rs[ST][NW][TN];
  auto loadW = [&](int slot, int kt) {
    const bool ok = kt < kbs;
#pragma unroll
    for (int w = 0; w < NW; w++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int p = 0; p < QW; p++)
          rq[slot][w][j][p] = __builtin_amdgcn_raw_buffer_load_b128(rW[w], ok ? offQ[j] : 0xffffffffu, (kt * QW + p) * 1024, 0);
        rs[slot][w][j] = __builtin_amdgcn_raw_buffer_load_b32(rW[w], ok ? offS[j] : 0xffffffffu, kt * 128, 0);
      }
  };
  // scale operands: the fp16 scale of the step's first block in K slot 0, of its second block in K slot 1, in the lanes of K
  // group 0; everything else zero
  const uint32_t msk0 = kg ? 0u : 0x0000ffffu, msk1 = kg ? 0u : 0xffff0000u;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const QXConst kc = qx_const(WT);
  const f16x8 off_op = __builtin_bit_cast(f16x8, u32x4{kg ? 0u : qx_offsets(WT), 0u, 0u, 0u});

  // the operands of one (block, matrix, column tile) from the packed registers: codes of the channels 0..15 | 16..31
  auto unpack = [&](const u32x4 (&q)[QW], int b, f16x8 (&fw)[2]) {
    if (WT == MLLM_HIP_Q4_0) {
      const auto r = __builtin_amdgcn_permlane16_swap(q[0][2 * b], q[0][2 * b + 1], false, false);
      fw[0] = qx_codes_dw<WT>(r[0], 0u, kc);
      fw[1] = qx_codes_dw<WT>(r[1], 0u, kc);
    } else {
      // block b: steps 2b (dwords 0, 1 of register b) and 2b + 1 (dwords 2, 3)
      const auto r0 = __builtin_amdgcn_permlane16_swap(q[QW - 1 ? b : 0][0], q[QW - 1 ? b : 0][2], false, false);
      const auto r1 = __builtin_amdgcn_permlane16_swap(q[QW - 1 ? b : 0][1], q[QW - 1 ? b : 0][3], false, false);
      fw[0] = qx_codes_dw<WT>(r0[0], r1[0], kc);
      fw[1] = qx_codes_dw<WT>(r0[1], r1[1], kc);
    }
  };
  auto scales = [&](uint32_t s, int b, u32x4 (&sw)[2]) {
    const uint32_t up = __builtin_amdgcn_permlane16_swap(s, s, false, false)[1];  // lanes 0..15 <- lanes 16..31
    const uint32_t m = b ? msk1 : msk0;
    sw[0].x = s & m;
    sw[1].x = up & m;
  };

  constexpr int G = 2 * NW * TN;  // groups per K step: block-major, then matrix, then column tile
  f16x8 fw[2][2];                 // [current | next group][channel half]
  u32x4 sw[2][2] = {{{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}}, {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}}};
  f32x4 T[2][2], S[2][2];         // block sums and scale products of the current / previous group
  T[1][0] = T[1][1] = S[1][0] = S[1][1] = zero4;

  const int nsteps = (kbs + ST - 1) / ST * ST;
  loadA(0, 0);
  loadA(1, 1);
#pragma unroll
  for (int s = 0; s < ST; s++) loadW(s, s);
  storeA(0, 0);
  unpack(rq[0][0][0], 0, fw[0]);
  scales(rs[0][0][0], 0, sw[0]);
  __syncthreads();

  auto kstep = [&](auto slot_tag, int kt) {
    constexpr int SLOT = decltype(slot_tag)::value;
    constexpr int NSLOT = (SLOT + 1) % ST;
    const int buf = kt & 1;
    loadA(SLOT & 1, kt + 2);
    f16x8 fb[2];
#pragma unroll
    for (int b = 0; b < 2; b++)
      fb[b] = *reinterpret_cast<const f16x8*>(smem + buf * STAGE + c16 * LDK + (2 * b + (kg & 1)) * 32 + (kg >> 1) * 16);
    f16x8 rec[3];
#pragma unroll
    for (int q = 0; q < 3; q++) rec[q] = *reinterpret_cast<const f16x8*>(smem + buf * STAGE + BM * LDK + c16 * 48 + q * 16);
    f32x4 tc = zero4;
#pragma unroll
    for (int g = 0; g < G; g++) {
      const int c = g & 1, n = c ^ 1;  // the register sets alternate (G is even)
      const int b = g / (NW * TN);
      const bool last = g == G - 1;
      const int gn = last ? 0 : g + 1;
      const int bn = gn / (NW * TN), wn = (gn / TN) % NW, jn = gn % TN;
      const int pg = g == 0 ? G - 1 : g - 1;
      const int pw = (pg / TN) % NW, pj = pg % TN;
      __builtin_amdgcn_sched_barrier(0);
      if (g % (NW * TN) == 0) tc = __builtin_amdgcn_mfma_f32_16x16x32_f16(off_op, rec[1 + b], zero4, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (last) unpack(rq[NSLOT][wn][jn], bn, fw[n]);
      else unpack(rq[SLOT][wn][jn], bn, fw[n]);
      __builtin_amdgcn_sched_barrier(0);
      T[c][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fw[c][0], fb[b], tc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      S[c][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, sw[c][0]), rec[0], zero4, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (last) {
        scales(rs[NSLOT][wn][jn], bn, sw[n]);
      } else {
        scales(rs[SLOT][wn][jn], bn, sw[n]);
        if (bn == 1) {  // both blocks of (wn, jn) are unpacked: fetch K step kt + ST into its ring registers
#pragma unroll
          for (int p = 0; p < QW; p++)
            rq[SLOT][wn][jn][p] = __builtin_amdgcn_raw_buffer_load_b128(rW[wn], kt + ST < kbs ? offQ[jn] : 0xffffffffu, ((kt + ST) * QW + p) * 1024, 0);
          rs[SLOT][wn][jn] = __builtin_amdgcn_raw_buffer_load_b32(rW[wn], kt + ST < kbs ? offS[jn] : 0xffffffffu, (kt + ST) * 128, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      T[c][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fw[c][1], fb[b], tc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      // the FMAs of the previous group (of the previous step's last group when g == 0)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[pw][pj][0][r] = fmaf(S[n][0][r], T[n][0][r], acc[pw][pj][0][r]);
      asm volatile("" : "+v"(acc[pw][pj][0]));
      __builtin_amdgcn_sched_barrier(0);
      S[c][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, sw[c][1]), rec[0], zero4, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < 4; r++) acc[pw][pj][1][r] = fmaf(S[n][1][r], T[n][1][r], acc[pw][pj][1][r]);
      asm volatile("" : "+v"(acc[pw][pj][1]));
      __builtin_amdgcn_sched_barrier(0);
    }
    storeA((SLOT & 1) ^ 1, buf ^ 1);
    __syncthreads();
  };
  for (int kt = 0; kt < nsteps; kt += ST) {
    kstep(std::integral_constant<int, 0>{}, kt);
    kstep(std::integral_constant<int, 1>{}, kt + 1);
    kstep(std::integral_constant<int, 2>{}, kt + 2);
    kstep(std::integral_constant<int, 3>{}, kt + 3);
  }
  // the last group's FMAs (G even: its results are in set 1)
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int r = 0; r < 4; r++) acc[NW - 1][TN - 1][h][r] = fmaf(S[1][h][r], T[1][h][r], acc[NW - 1][TN - 1][h][r]);

  // acc[w][j][h][e] = result[row0 + c16][n0 + wave*WN + 32j + 16h + 4kg + e]
  if (NW == 1) {
    if (c16 < rows) {
      const int pos = row0 + c16;
      float* orow = a.out + (int64_t)(a.o_index ? a.o_index[pos] : pos) * a.N;
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const int n = n0 + wave * WN + j * 32 + 16 * h + 4 * kg;
          f32x4 v = acc[0][j][h];
          if (n + 3 < a.N && a.N % 4 == 0) {
            if (a.bias) v += *reinterpret_cast<const f32x4*>(a.bias + n);
            *reinterpret_cast<f32x4*>(orow + n) = v;
          } else {
#pragma unroll
            for (int e2 = 0; e2 < 4; e2++)
              if (n + e2 < a.N) orow[n + e2] = a.bias ? v[e2] + a.bias[n + e2] : v[e2];
          }
        }
    }
  } else {
    // h = silu(gate) * up, quantized to Q8_0 over each block of 32 channels (one column tile j: eight channels in each of the
    // four lanes of a row), written in the next Linear's activation format
    const int nblk = a.N / QK, KDo = (a.N + 63) / 64;
#pragma unroll
    for (int j = 0; j < TN; j++) {
      float hv[8];
      float amax = 0.f;
#pragma unroll
      for (int q = 0; q < 8; q++) {
        hv[q] = silu_f(acc[0][j][q >> 2][q & 3]) * acc[NW - 1][j][q >> 2][q & 3];
        amax = fmaxf(amax, fabsf(hv[q]));
      }
      amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
      amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
      const float d = amax / 127.f;
      const float idv = (amax != 0.f) ? 127.f / amax : 0.f;
      uint16_t bits = f32_to_f16bits(d);
      if (a.x86_scale) bits = x86_scale_bits(bits);
      const int blk = (n0 + wave * WN) / 32 + j;
      // element 16h + 4kg + e of the block: bit 1 of its index is bit 1 of e
      int qv[8], sa = 0, sb = 0;
#pragma unroll
      for (int q = 0; q < 8; q++) {
        qv[q] = min(127, max(-128, (int)rintf(hv[q] * idv)));
        if (q & 2) sb += qv[q];
        else sa += qv[q];
      }
      sa += __shfl_xor(sa, 16, 64);
      sa += __shfl_xor(sa, 32, 64);
      sb += __shfl_xor(sb, 16, 64);
      sb += __shfl_xor(sb, 32, 64);
      if (c16 < rows && blk < nblk) {
        uint16_t* hrow = a.hq + (int64_t)(row0 + c16) * a.N;
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const int n = n0 + wave * WN + j * 32 + 16 * h + 4 * kg;
          uint32_t o[2];
#pragma unroll
          for (int e2 = 0; e2 < 2; e2++)
            o[e2] = (uint32_t)f32_to_f16bits((float)qv[4 * h + 2 * e2]) | ((uint32_t)f32_to_f16bits((float)qv[4 * h + 2 * e2 + 1]) << 16);
          *reinterpret_cast<uint2*>(hrow + n) = uint2{o[0], o[1]};
        }
        if (kg == 0) {
          uint32_t* recp = a.hd + ((int64_t)(row0 + c16) * KDo + (blk >> 1)) * 3;
          reinterpret_cast<uint16_t*>(recp)[blk & 1] = bits;
          recp[1 + (blk & 1)] = (uint32_t)f32_to_f16bits((float)sa) | ((uint32_t)f32_to_f16bits((float)sb) << 16);
          if (blk == nblk - 1 && (nblk & 1)) {  // the unused half of the last record
            reinterpret_cast<uint16_t*>(recp)[1] = 0;
            recp[2] = 0;
          }
        }
      }
    }
  }
}

constexpr int QX_TILE_H = 32;
constexpr int QX_DOWN_TN = 2;  // column tiles per wave in the one-matrix mode
constexpr int QX_GROUP = 8;    // tiles per group of work items (see qx_kernel)
// MODE 0: one matrix, up to 32 rows x 256 channels per workgroup.  MODE 1: gate and up together, 32 rows x 128 channels.
template <int WT, int MODE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void qx_kernel(QXArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  // Work items in groups of QX_GROUP tiles (list order: an expert's tiles are neighbours) x all column blocks, inside a
  // group the tile index fastest.  Workgroup L runs on XCD L % 8, and every XCD has its own L2: XCD x takes a contiguous
  // eighth of the work items, so that the tiles of one expert and column block -- which read the same weights -- and the
  // column blocks of one tile -- which read the same activation rows -- run on one XCD at about the same time.
  // (512 tokens x 8 of 128 experts, whole FFN: column block slowest over the whole list 167.5 us, groups of eight tiles
  // 162.3; 8192 tokens 1352 -> 1330.)
  const int nt = min(a.ntiles[0], (int)gridDim.x), ny = (int)gridDim.y;
  const int L = (int)(blockIdx.x + gridDim.x * blockIdx.y);
  const int nw = nt * ny, base = nw >> 3, rem = nw & 7;  // XCD x takes base + (x < rem) items
  const int xcd = L & 7, seq = L >> 3;
  if (seq >= base + (xcd < rem)) return;
  const int w = xcd * base + min(xcd, rem) + seq;
  const int per = QX_GROUP * ny, g = w / per, r0 = w - g * per;
  const int gt = min(QX_GROUP, nt - g * QX_GROUP);  // tiles in this group (the last one may be short)
  const int by = r0 / gt, t = g * QX_GROUP + (r0 - by * gt);
  const int e = a.tile_expert[t], row0 = a.tile_row0[t], rows = a.tile_rows[t];
  if constexpr (MODE == 1) {
    const int n0 = by * 128;
    if (rows <= 16 && a.half_tiles) qx_tile16<WT, 2, 1>(a, e, row0, rows, n0, smem);
    else qx_tile<WT, 2, 1, 1>(a, e, row0, rows, n0, smem);
  } else {
    const int n0 = by * (128 * QX_DOWN_TN);
    if (rows <= 16 && a.half_tiles) qx_tile16<WT, 1, QX_DOWN_TN>(a, e, row0, rows, n0, smem);
    else qx_tile<WT, 1, 1, QX_DOWN_TN>(a, e, row0, rows, n0, smem);
  }
}



template <int MODE>
static int launch_qx(int wtype, const QXArgs& a, unsigned max_tiles, hipStream_t st) {
  const int wg_n = MODE == 1 ? 128 : 128 * QX_DOWN_TN;
  const dim3 grid(max_tiles, (unsigned)((a.N + wg_n - 1) / wg_n));
  const size_t lds = 2 * (size_t)(QX_TILE_H * (2 * 64 + 16) + QX_TILE_H * 48);
  if (wtype == MLLM_HIP_Q4_0) hipLaunchKernelGGL((qx_kernel<MLLM_HIP_Q4_0, MODE>), grid, dim3(256), lds, st, a);
  else hipLaunchKernelGGL((qx_kernel<MLLM_HIP_Q8_0, MODE>), grid, dim3(256), lds, st, a);
  return (int)hipGetLastError();
}

// activations for the kernel above: Q8_0 quantization (bit-exact codes and scale); codes as fp16 integers, and per row and K
// step of 64 a record of three dwords: the two blocks' fp16 scales, then per block the code sums over the elements with
// bit 1 of k clear | set, as fp16 integers (at most 16 x 127 each: exact).  The second half of a last, incomplete record is zero.
__device__ __forceinline__ void qx_act_block(const void* __restrict__ x, int x_dtype, uint16_t* __restrict__ xq, uint32_t* __restrict__ xd,
                                             int64_t i, int nb, int x86_scale) {
  float v[32];
  uint32_t q[8];
  int sum;
  load_block_f32(x, x_dtype, i * QK, v);
  uint16_t bits = quantize_block_q8_0(v, q, sum);
  if (x86_scale) bits = x86_scale_bits(bits);
  uint32_t o[16];
  int sa = 0, sb = 0;
#pragma unroll
  for (int j = 0; j < 16; j++) {  // elements 2j, 2j+1
    const int c0 = (int8_t)(q[j / 2] >> (16 * (j & 1))), c1 = (int8_t)(q[j / 2] >> (16 * (j & 1) + 8));
    o[j] = (uint32_t)f32_to_f16bits((float)c0) | ((uint32_t)f32_to_f16bits((float)c1) << 16);
    if (j & 1) sb += c0 + c1;
    else sa += c0 + c1;
  }
  u32x4* out = reinterpret_cast<u32x4*>(xq + i * QK);
#pragma unroll
  for (int j = 0; j < 4; j++) out[j] = u32x4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
  const int64_t row = i / nb;
  const int b = (int)(i - row * nb), KD = (nb + 1) / 2;
  uint32_t* rec = xd + (row * KD + (b >> 1)) * 3;
  reinterpret_cast<uint16_t*>(rec)[b & 1] = bits;
  rec[1 + (b & 1)] = (uint32_t)f32_to_f16bits((float)sa) | ((uint32_t)f32_to_f16bits((float)sb) << 16);
  if (b == nb - 1 && (nb & 1)) {
    reinterpret_cast<uint16_t*>(rec)[1] = 0;
    rec[2] = 0;
  }
}

// the two independent preparations of the grouped FFN in one launch: workgroup 0 routes, the others quantize x
__global__ __launch_bounds__(1024) void qx_prepare_kernel(const int32_t* __restrict__ ids, int n, int E, int tile_h, RouteOut o,
                                                          const void* __restrict__ x, int x_dtype, uint16_t* __restrict__ xq,
                                                          uint32_t* __restrict__ xd, int64_t nblocks, int nb, int x86_scale) {
  extern __shared__ int s_route[];
  if (blockIdx.x == 0) {
    moe_route_body<true>(ids, n, E, tile_h, o, s_route);
    return;
  }
  const int64_t i = (int64_t)(blockIdx.x - 1) * 1024 + threadIdx.x;
  if (i < nblocks) qx_act_block(x, x_dtype, xq, xd, i, nb, x86_scale);
}

// y[t][h] = sum_j per[t*k + j][h] * w[t][j]   (multiply, then add in j order: modeling_qwen3_moe_fa2.hpp:233-236)
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ per, const float* __restrict__ w, const int32_t* __restrict__ ids,
                                                          float* __restrict__ y, int64_t T, int H, int k, int E) {
  // four consecutive channels per thread (H % 4 == 0: H is a multiple of the block size), all k rows requested before the
  // first is used; the sum itself runs in slot order
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= T * H) return;
  const int64_t t = i / H;
  const int h = (int)(i - t * H);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int j0 = 0; j0 < k; j0 += 8) {
    // every load is unconditional (slots past k repeat the last one; the row of a slot without expert was never written
    // but is readable memory): nothing waits on a branch, and what must not count is dropped by a select
    int e[8];
    float wj[8];
    f32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const int64_t s = t * k + min(j0 + u, k - 1);
      e[u] = ids[s];
      wj[u] = w[s];
      v[u] = *reinterpret_cast<const f32x4*>(per + s * H + h);
    }
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const f32x4 nx = acc + v[u] * wj[u];
      const bool ok = j0 + u < k && e[u] >= 0 && e[u] < E;
      acc.x = ok ? nx.x : acc.x;
      acc.y = ok ? nx.y : acc.y;
      acc.z = ok ? nx.z : acc.z;
      acc.w = ok ? nx.w : acc.w;
    }
  }
  *reinterpret_cast<f32x4*>(y + i) = acc;
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
static RouteOut carve_route(Carver& c, int E, int64_t entries, int tile_h = TOK_TILE) {
  RouteOut o;
  const size_t max_tiles = (size_t)E + (size_t)(entries / tile_h) + 1;
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

// y = sum over the K ranges of their partial results (in range order) + bias
__global__ __launch_bounds__(256) void qg_reduce_kernel(const float* __restrict__ partial, int Z, int64_t MN, int N, const float* __restrict__ bias,
                                                        float* __restrict__ y) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;  // N % 4 == 0 on this path
  if (i >= MN) return;
  f32x4 v = *reinterpret_cast<const f32x4*>(partial + i);
  for (int z = 1; z < Z; z++) v += *reinterpret_cast<const f32x4*>(partial + (size_t)z * MN + i);
  if (bias) v += *reinterpret_cast<const f32x4*>(bias + i % N);
  *reinterpret_cast<f32x4*>(y + i) = v;
}

// Short batches: a Linear of a few hundred rows has M/128 x N/256 tiles, far fewer than the chip has CUs (gate projection of
// the 4B layer at 128 rows: 38 workgroups, down: 10), and each streams its weights two K steps ahead only.  K is therefore
// cut into up to eight ranges that run as separate workgroups and leave partial results, summed by a small second kernel
// in range order.  Number of ranges: enough for about one workgroup per CU, at most 24 MB of partial results (their round trip through memory is what the second kernel costs); up to 1024 rows.
int qg_short_splits(int64_t M, int64_t N, int64_t K) {
  if (M > 1024 || N % 4) return 1;
  const int64_t tiles = ((M + QG_TILE_H - 1) / QG_TILE_H) * ((N + 255) / 256);
  const int KT = (int)(qg_kp(K) / 64);
  int z = (int)((256 + tiles - 1) / tiles);
  if (z > 8) z = 8;
  while (z > 1 && (int64_t)z * M * N * 4 > (24 << 20)) z--;
  if (z <= 1) return 1;
  const int per = ((KT + z - 1) / z + 1) / 2 * 2;
  return (KT + per - 1) / per;  // no empty range
}
size_t qg_partial_bytes(int64_t M, int64_t N, int64_t K) {
  const int z = qg_short_splits(M, N, K);
  return z > 1 ? align_up((size_t)z * M * N * 4, 256) : 0;
}

size_t qg_route_bytes(int64_t M) {
  Carver c(nullptr);
  carve_route(c, 1, M);
  return c.used;
}
int qg_linear_run(int wtype, const void* gemm_packed, const uint16_t* xh, const float* bias, float* y, int64_t M, int64_t N,
                  int64_t K, void* route_ws, void* partial_ws, hipStream_t st) {
  Carver c(route_ws);
  RouteOut ro = carve_route(c, 1, M);
  RC_RET(launch_identity_tiles(M, QG_TILE_H, ro, st));
  QG2Args a{};
  a.W0 = a.W1 = reinterpret_cast<const char*>(gemm_packed);
  a.wstride = 0;
  a.xh = xh; a.a_index = nullptr; a.a_div = 1; a.a_rows = (int)M;
  a.o_index = nullptr; a.out = y; a.bias = bias;
  a.tile_expert = ro.tile_expert; a.tile_row0 = ro.tile_row0; a.tile_rows = ro.tile_rows; a.ntiles = ro.ntiles;
  a.N = (int)N; a.K = (int)K; a.wtype = wtype; a.x86_scale = 0;
  a.ksplit = partial_ws ? qg_short_splits(M, N, K) : 1;
  a.partial = reinterpret_cast<float*>(partial_ws);
  const int rc = launch_qg<0>(a, (unsigned)((M + QG_TILE_H - 1) / QG_TILE_H), st);
  if (rc || a.ksplit <= 1) return rc;
  hipLaunchKernelGGL(qg_reduce_kernel, dim3((unsigned)((M * N / 4 + 255) / 256)), dim3(256), 0, st, a.partial, a.ksplit, M * N, (int)N, bias, y);
  return (int)hipGetLastError();
}

}  // namespace mllmhip

using namespace mllmhip;

// =========================================================================================================
// C ABI
// =========================================================================================================
// rows up to which mllm_hip_linear_q runs as passes of the eight-row GEMV
constexpr int64_t LINEAR_Q_GEMV_ROWS = 16;
MLLM_API size_t mllm_hip_linear_q_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || K % QK) return 0;
  Carver c(nullptr);
  c.take<int8_t>((size_t)M * K);
  c.take<float>((size_t)M * (K / QK));
  carve_route(c, 1, M);
  // short batches run as passes of the decode GEMV, which keeps the quantized image of eight rows here
  const size_t gemv = M <= LINEAR_Q_GEMV_ROWS ? mllm_hip_gemv_workspace_bytes(8, K) : 0;
  return c.used > gemv ? c.used : gemv;
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
  if (M <= LINEAR_Q_GEMV_ROWS) {
    // same block arithmetic, the weights streamed once per eight rows: measured against the tile kernel below on the
    // Qwen3-4B projections, 16 rows: 15-22 us against 40-127 (the tile kernel's workgroup is one row tile x 128 channels
    // whatever the row count, and walks all of K alone)
    const mllm_hip_gemv_part part{packed, bias, y, N};
    return mllm_hip_linear_q_gemv_multi_wsn(wtype, 1, &part, x, x_dtype, (int)M, K, act_scale_mode, workspace,
                                            mllm_hip_gemv_workspace_bytes(8, K), stream);
  }
  Carver c(workspace);
  int8_t* aq = c.take<int8_t>((size_t)M * K);
  float* ad = c.take<float>((size_t)M * (K / QK));
  RouteOut ro = carve_route(c, 1, M);
  const int64_t nblocks = M * (K / QK);
  hipLaunchKernelGGL(quant_rows_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, st, x, x_dtype, aq, ad, nblocks,
                     act_scale_mode == MLLM_HIP_SCALE_X86_REF);
  RC_RET(launch_identity_tiles(M, TOK_TILE, ro, st));
  QGemmArgs a{};
  a.W0 = a.W1 = reinterpret_cast<const char*>(packed);
  a.wstride = 0;
  a.aq = aq; a.ad = ad; a.a_index = nullptr; a.a_div = 1; a.a_rows = (int)M;
  a.o_index = nullptr; a.out = y; a.bias = bias;
  a.tile_expert = ro.tile_expert; a.tile_row0 = ro.tile_row0; a.tile_rows = ro.tile_rows; a.ntiles = ro.ntiles;
  a.N = (int)N; a.K = (int)K; a.x86_scale = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  return launch_tiles<0>(wtype, a, (unsigned)((M + TOK_TILE - 1) / TOK_TILE), st);
}

// decode path (moe_decode.hip): up to eight tokens as GEMVs, two launches
namespace mllmhip {
size_t moe_decode_workspace_bytes(int64_t T, int64_t I, int k);
bool moe_decode_applies(int64_t T, int64_t H, int64_t I, int E, int k);
int moe_decode_set_tokens(int tokens);
bool moe_rows_applies(int64_t T, int64_t H, int64_t I, int E, int k);
int moe_rows_set_tokens(int tokens);
int moe_rows_tile();
int launch_moe_rows(int wtype, const void* gate, const void* up, const void* down, const void* x, int x_dtype, const int* tile_expert,
                    const int* tile_row0, const int* tile_rows, const int* ntiles, const int* sorted_idx, void* img, float* per,
                    int64_t T, int64_t H, int64_t I, int E, int k, int x86, unsigned max_tiles, hipStream_t st);

// workspace of the row-tile path: images of h, one down result per pair, routing with tiles of moe_rows_tile() rows
struct RowsCarve {
  unsigned char* img;
  float* per;
  RouteOut ro;
};
static RowsCarve carve_rows(Carver& c, int64_t T, int64_t H, int64_t I, int E, int k) {
  RowsCarve r;
  r.img = c.take<unsigned char>(moe_decode_workspace_bytes(T, I, k));
  r.per = c.take<float>((size_t)T * k * H);
  r.ro = carve_route(c, E, T * k, moe_rows_tile());
  return r;
}
int launch_moe_decode(int wtype, const void* gate, const void* up, const void* down, const void* x, int x_dtype, const int32_t* ids,
                      const float* w, float* y, int64_t T, int64_t H, int64_t I, int E, int k, int x86, void* workspace,
                      hipStream_t st);
}  // namespace mllmhip

MLLM_API size_t mllm_hip_moe_workspace_bytes(int64_t T, int64_t H, int64_t I, int E, int k) {
  if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || k <= 0 || H % QK || I % QK) return 0;
  Carver c(nullptr);
  c.take<int8_t>((size_t)T * H);
  c.take<float>((size_t)T * (H / QK));
  c.take<int8_t>((size_t)T * k * I);
  c.take<float>((size_t)T * k * (I / QK));
  c.take<float>((size_t)T * k * H);
  carve_route(c, E, T * k);
  // whichever path the call then takes
  const size_t decode = moe_decode_workspace_bytes(T, I, k);
  Carver cr(nullptr);
  carve_rows(cr, T, H, I, E, k);
  const size_t most = c.used > cr.used ? c.used : cr.used;
  return most > decode ? most : decode;
}

MLLM_API int mllm_hip_moe_set_tuning(int pair_tokens, int row_tokens) {
  if (pair_tokens < 0 || pair_tokens > 4096 || row_tokens < 0 || row_tokens > 65536) return MLLM_HIP_E_BADARG;
  moe_decode_set_tokens(pair_tokens);
  moe_rows_set_tokens(row_tokens);
  return 0;
}

MLLM_API int mllm_hip_moe_route(const int32_t* topk_ids, int64_t T, int E, int k, int32_t* counts, int32_t* offsets,
                                int32_t* sorted_idx, void* workspace, void* stream) {
  if (!topk_ids || !workspace || T <= 0 || E <= 0 || k <= 0) return MLLM_HIP_E_BADARG;
  hipStream_t st = (hipStream_t)stream;
  Carver c(workspace);
  RouteOut ro = carve_route(c, E, T * k);
  RC_RET(launch_route(topk_ids, T * k, E, TOK_TILE, ro, st));
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
      !topk_w || !y || !workspace || T <= 0 || E <= 0 || k <= 0)
    return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (H <= 0 || I <= 0 || H % QK || I % QK || E > MOE_MAX_EXPERTS) return MLLM_HIP_E_SHAPE;
  if (T * H >= ((int64_t)1 << 32) || T * k * I >= ((int64_t)1 << 32) || T * k > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16 || reinterpret_cast<uintptr_t>(y) % 16) return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int x86 = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  // few pairs per expert: every (token, expert) pair is one GEMV row; two launches instead of five
  if (moe_decode_applies(T, H, I, E, k))
    return launch_moe_decode(wtype, gate_packed, up_packed, down_packed, x, x_dtype, topk_ids, topk_w, y, T, H, I, E, k, x86, workspace, st);
  // a few pairs per expert: the pairs sorted by expert, tiles of eight rows that share the expert's weights
  if (moe_rows_applies(T, H, I, E, k)) {
    Carver cr(workspace);
    RowsCarve rc = carve_rows(cr, T, H, I, E, k);
    const unsigned max_tiles = (unsigned)(E + (T * k) / moe_rows_tile() + 1);
    RC_RET(launch_route(topk_ids, T * k, E, moe_rows_tile(), rc.ro, st));
    int r = launch_moe_rows(wtype, gate_packed, up_packed, down_packed, x, x_dtype, rc.ro.tile_expert, rc.ro.tile_row0, rc.ro.tile_rows,
                            rc.ro.ntiles, rc.ro.sorted_idx, rc.img, rc.per, T, H, I, E, k, x86, max_tiles, st);
    if (r) return r;
    const int64_t total = T * H;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, st, rc.per, topk_w, topk_ids, y, T,
                       (int)H, k, E);
    return (int)hipGetLastError();
  }
  Carver c(workspace);
  int8_t* xq = c.take<int8_t>((size_t)T * H);
  float* xd = c.take<float>((size_t)T * (H / QK));
  int8_t* hq = c.take<int8_t>((size_t)T * k * I);
  float* hd = c.take<float>((size_t)T * k * (I / QK));
  float* per = c.take<float>((size_t)T * k * H);
  RouteOut ro = carve_route(c, E, T * k);
  const unsigned max_tiles = (unsigned)(E + (T * k) / TOK_TILE + 1);

  RC_RET(launch_route(topk_ids, T * k, E, TOK_TILE, ro, st));
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
  hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, st, per, topk_w, topk_ids, y, T,
                     (int)H, k, E);
  return (int)hipGetLastError();
}

// ---- matrix-core path (gemm-packed weights) -------------------------------------------------------------------
MLLM_API size_t mllm_hip_q_gemm_packed_bytes(int wtype, int64_t N, int64_t K) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || N <= 0 || K <= 0 || K % QK) return 0;
  return (size_t)qg_bytes(wtype, N, K);
}

MLLM_API int mllm_hip_q_gemm_prepack(int wtype, const void* blocks, int weight_scale_mode, void* packed, int64_t N, int64_t K,
                                     void* stream) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || !blocks || !packed || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (weight_scale_mode != MLLM_HIP_SCALE_IEEE && weight_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (K % QK || N > INT32_MAX || K > INT32_MAX || qg_bytes(wtype, N, K) >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(packed) % 16) return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int64_t words = qg_qbytes(wtype, N, K) / 4, count = qg_np(N) * (qg_kp(K) / 64);
  const unsigned char* b = reinterpret_cast<const unsigned char*>(blocks);
  uint32_t* q = reinterpret_cast<uint32_t*>(packed);
  uint32_t* sc = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(packed) + qg_qbytes(wtype, N, K));
  const int x86 = weight_scale_mode == MLLM_HIP_SCALE_X86_REF;
  if (wtype == MLLM_HIP_Q4_0) {
    hipLaunchKernelGGL(qg_prepack_q_kernel<MLLM_HIP_Q4_0>, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st, b, q, (int)N, (int)K, words);
    hipLaunchKernelGGL(qg_prepack_s_kernel<MLLM_HIP_Q4_0>, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st, b, sc, (int)N, (int)K, x86, count);
  } else {
    hipLaunchKernelGGL(qg_prepack_q_kernel<MLLM_HIP_Q8_0>, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st, b, q, (int)N, (int)K, words);
    hipLaunchKernelGGL(qg_prepack_s_kernel<MLLM_HIP_Q8_0>, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st, b, sc, (int)N, (int)K, x86, count);
  }
  return (int)hipGetLastError();
}

MLLM_API size_t mllm_hip_linear_q_gemm_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || K % QK) return 0;
  Carver c(nullptr);
  c.take<uint16_t>((size_t)M * K);
  carve_route(c, 1, M);
  return c.used;
}

MLLM_API int mllm_hip_linear_q_gemm(int wtype, const void* gemm_packed, const void* x, int x_dtype, const float* bias,
                                    float* y, int64_t M, int64_t N, int64_t K, int act_scale_mode, void* workspace,
                                    void* stream) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || !gemm_packed || !x || !y || !workspace || M <= 0 || N <= 0 || K <= 0)
    return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (K % QK || M * K * 2 >= ((int64_t)1 << 32) || N > INT32_MAX || qg_bytes(wtype, N, K) >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16 ||
      reinterpret_cast<uintptr_t>(gemm_packed) % 16 || reinterpret_cast<uintptr_t>(y) % 16)
    return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  Carver c(workspace);
  uint16_t* xh = c.take<uint16_t>((size_t)M * K);
  const int64_t nblocks = M * (K / QK);
  hipLaunchKernelGGL(qg_act_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, st, x, x_dtype, xh,
                     (uint16_t*)nullptr, nblocks, act_scale_mode == MLLM_HIP_SCALE_X86_REF);
  return qg_linear_run(wtype, gemm_packed, xh, bias, y, M, N, K, c.p + c.used, nullptr, st);
}

// the same for short batches (M <= 256 gains; any M is accepted): K cut into ranges, see qg_short_splits
MLLM_API size_t mllm_hip_linear_q_gemm_short_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % QK) return 0;
  return mllm_hip_linear_q_gemm_workspace_bytes(M, K) + qg_partial_bytes(M, N, K);
}
MLLM_API int mllm_hip_linear_q_gemm_short(int wtype, const void* gemm_packed, const void* x, int x_dtype, const float* bias, float* y,
                                          int64_t M, int64_t N, int64_t K, int act_scale_mode, void* workspace, void* stream) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || !gemm_packed || !x || !y || !workspace || M <= 0 || N <= 0 || K <= 0)
    return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (K % QK || M * K * 2 >= ((int64_t)1 << 32) || N > INT32_MAX || qg_bytes(wtype, N, K) >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 256 ||
      reinterpret_cast<uintptr_t>(gemm_packed) % 16 || reinterpret_cast<uintptr_t>(y) % 16)
    return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  Carver c(workspace);
  uint16_t* xh = c.take<uint16_t>((size_t)M * K);
  const int64_t nblocks = M * (K / QK);
  hipLaunchKernelGGL(qg_act_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, st, x, x_dtype, xh,
                     (uint16_t*)nullptr, nblocks, act_scale_mode == MLLM_HIP_SCALE_X86_REF);
  void* route = c.p + c.used;
  void* partial = qg_partial_bytes(M, N, K) ? c.p + mllm_hip_linear_q_gemm_workspace_bytes(M, K) : nullptr;
  return qg_linear_run(wtype, gemm_packed, xh, bias, y, M, N, K, route, partial, st);
}

namespace mllmhip {
struct QXCarve {
  uint16_t* xq;
  uint32_t* xd;
  uint16_t* hq;
  uint32_t* hd;
  float* per;
  RouteOut ro;
};
static QXCarve carve_qx(Carver& c, int64_t T, int64_t H, int64_t I, int E, int k) {
  QXCarve r;
  r.xq = c.take<uint16_t>((size_t)T * H);
  r.xd = c.take<uint32_t>((size_t)T * 3 * ((H + 63) / 64));
  r.hq = c.take<uint16_t>((size_t)T * k * I);
  r.hd = c.take<uint32_t>((size_t)T * k * 3 * ((I + 63) / 64));
  r.per = c.take<float>((size_t)T * k * H);
  r.ro = carve_route(c, E, T * k, QX_TILE_H);
  return r;
}
// 0: exact block sums (qx_kernel); 1: fp16 operands with the block scales folded in (qg_kernel); 2: as 0 with every tile in
// the 32-row form (the comparison for the 16-row form: same bits)
static int g_moe_gemm_path = 0;
}  // namespace mllmhip

MLLM_API int mllm_hip_moe_gemm_set_path(int path) {
  if (path < 0 || path > 2) return MLLM_HIP_E_BADARG;
  g_moe_gemm_path = path;
  return 0;
}

// The grouped expert FFN with the reference's own block arithmetic on the matrix cores (qx_kernel): route, quantize x,
// gate + up + SiLU * up + re-quantization in one launch, down, weighted sum in slot order.
static int moe_ffn_qx(int wtype, const void* gate_packed, const void* up_packed, const void* down_packed, const void* x, int x_dtype,
                      const int32_t* topk_ids, const float* topk_w, float* y, int64_t T, int64_t H, int64_t I, int E, int k, int x86,
                      void* workspace, hipStream_t st) {
  Carver c(workspace);
  QXCarve w = carve_qx(c, T, H, I, E, k);
  const unsigned max_tiles = (unsigned)(E + (T * k) / QX_TILE_H + 1);
  if (E > MOE_MAX_EXPERTS) return MLLM_HIP_E_SHAPE;
  const int64_t nblocks = T * (H / QK);
  hipLaunchKernelGGL(qx_prepare_kernel, dim3((unsigned)(1 + (nblocks + 1023) / 1024)), dim3(1024), 5 * (size_t)E * sizeof(int), st,
                     topk_ids, (int)(T * k), E, QX_TILE_H, w.ro, x, x_dtype, w.xq, w.xd, nblocks, (int)(H / QK), x86);
  HIP_RET(hipGetLastError());
  QXArgs a{};
  a.tile_expert = w.ro.tile_expert; a.tile_row0 = w.ro.tile_row0; a.tile_rows = w.ro.tile_rows; a.ntiles = w.ro.ntiles;
  a.x86_scale = x86;
  a.half_tiles = g_moe_gemm_path != 2;
  a.W0 = reinterpret_cast<const char*>(gate_packed);
  a.W1 = reinterpret_cast<const char*>(up_packed);
  a.wstride = (size_t)qg_bytes(wtype, I, H);
  a.xq = w.xq; a.xd = w.xd; a.a_index = w.ro.sorted_idx; a.a_div = k; a.a_rows = (int)T;
  a.hq = w.hq; a.hd = w.hd;
  a.N = (int)I; a.K = (int)H;
  RC_RET(launch_qx<1>(wtype, a, max_tiles, st));
  a.W0 = a.W1 = reinterpret_cast<const char*>(down_packed);
  a.wstride = (size_t)qg_bytes(wtype, H, I);
  a.xq = w.hq; a.xd = w.hd; a.a_index = nullptr; a.a_div = 1; a.a_rows = (int)(T * k);
  a.o_index = w.ro.sorted_idx; a.out = w.per; a.bias = nullptr; a.hq = nullptr; a.hd = nullptr;
  a.N = (int)H; a.K = (int)I;
  RC_RET(launch_qx<0>(wtype, a, max_tiles, st));
  const int64_t total = T * H;
  hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, st, w.per, topk_w, topk_ids, y, T,
                     (int)H, k, E);
  return (int)hipGetLastError();
}

MLLM_API size_t mllm_hip_moe_gemm_workspace_bytes(int64_t T, int64_t H, int64_t I, int E, int k) {
  if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || k <= 0 || H % QK || I % QK) return 0;
  Carver c(nullptr);
  c.take<uint16_t>((size_t)T * H);
  c.take<uint16_t>((size_t)T * H);
  c.take<uint16_t>((size_t)T * k * I);
  c.take<float>((size_t)T * k * H);
  carve_route(c, E, T * k);
  // the exact form: codes as fp16 integers + scale pairs for x and for h, the per-pair rows, routing
  Carver cx(nullptr);
  carve_qx(cx, T, H, I, E, k);
  return c.used > cx.used ? c.used : cx.used;
}

MLLM_API int mllm_hip_moe_ffn_q_gemm(int wtype, const void* gate_packed, const void* up_packed, const void* down_packed,
                                     const void* x, int x_dtype, const int32_t* topk_ids, const float* topk_w, float* y,
                                     int64_t T, int64_t H, int64_t I, int E, int k, int act_scale_mode, void* workspace,
                                     void* stream) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || !gate_packed || !up_packed || !down_packed || !x || !topk_ids ||
      !topk_w || !y || !workspace || T <= 0 || E <= 0 || k <= 0)
    return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (H <= 0 || I <= 0 || H % QK || I % QK || E > MOE_MAX_EXPERTS) return MLLM_HIP_E_SHAPE;
  if (T * H * 2 >= ((int64_t)1 << 32) || T * k * I * 2 >= ((int64_t)1 << 32) || T * k > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16 || reinterpret_cast<uintptr_t>(y) % 16) return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int x86 = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  if (g_moe_gemm_path != 1)
    return moe_ffn_qx(wtype, gate_packed, up_packed, down_packed, x, x_dtype, topk_ids, topk_w, y, T, H, I, E, k, x86, workspace, st);
  Carver c(workspace);
  uint16_t* xh = c.take<uint16_t>((size_t)T * H);
  uint16_t* xl = c.take<uint16_t>((size_t)T * H);
  uint16_t* hh = c.take<uint16_t>((size_t)T * k * I);
  float* per = c.take<float>((size_t)T * k * H);
  RouteOut ro = carve_route(c, E, T * k);
  const unsigned max_tiles = (unsigned)(E + (T * k) / QG_TILE_H + 1);

  RC_RET(launch_route(topk_ids, T * k, E, QG_TILE_H, ro, st));
  const int64_t nblocks = T * (H / QK);
  hipLaunchKernelGGL(qg_act_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, st, x, x_dtype, xh, xl, nblocks, x86);

  QG2Args a{};
  a.tile_expert = ro.tile_expert; a.tile_row0 = ro.tile_row0; a.tile_rows = ro.tile_rows; a.ntiles = ro.ntiles;
  a.wtype = wtype; a.x86_scale = x86;
  // gate & up -> silu(g)*u -> Q8_0 round trip in fp16, rows in expert-sorted order
  a.W0 = reinterpret_cast<const char*>(gate_packed);
  a.W1 = reinterpret_cast<const char*>(up_packed);
  a.wstride = (size_t)qg_bytes(wtype, I, H);
  a.xh = xh; a.xl = xl; a.a_index = ro.sorted_idx; a.a_div = k; a.a_rows = (int)T;
  a.hh = hh;
  a.N = (int)I; a.K = (int)H;
  int rc = launch_qg<1>(a, max_tiles, st);
  if (rc) return rc;
  // down -> per-(token, slot) rows
  a.W0 = a.W1 = reinterpret_cast<const char*>(down_packed);
  a.wstride = (size_t)qg_bytes(wtype, H, I);
  a.xh = hh; a.xl = nullptr; a.a_index = nullptr; a.a_div = 1; a.a_rows = (int)(T * k);
  a.o_index = ro.sorted_idx; a.out = per; a.bias = nullptr; a.hh = nullptr;
  a.N = (int)H; a.K = (int)I;
  rc = launch_qg<0>(a, max_tiles, st);
  if (rc) return rc;
  const int64_t total = T * H;
  hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, st, per, topk_w, topk_ids, y, T,
                     (int)H, k, E);
  return (int)hipGetLastError();
}

// ---- experts in the super-block formats (kquant.hip) ----------------------------------------------------------------------
// The shipped Qwen3-MoE recipe quantizes the experts to Q4_K / Q6_K.  Every (token, expert) pair is one row of the K-quant
// GEMV: gate and up in one launch (the workgroup quantizes the token's x to Q8_K), silu(g) * u, the down GEMV (quantizing h),
// the weighted sum in slot order.  Three or four launches for any T; the weights of an expert are read once per pair that uses it,
// so this is the decode form.  With more than two pairs per expert the pairs are sorted by expert and run as tiles of eight
// rows on the matrix-core kernels instead (the grouped form).
namespace mllmhip {
int kq_moe_gemv(int wtype, int nparts, const void* const* packed0, float* const* ys, int64_t N, int64_t K, const void* x, int x_dtype,
                const float* x2, const int32_t* ids, int E, int slots, int slot_div, hipStream_t st);
size_t kq_image_bytes(int64_t rows, int64_t K);
int kq_quantize_image(const void* x, int x_dtype, void* image, int64_t rows, int64_t K, hipStream_t st);
bool kq_moe_tiles_fit(int wtype, int64_t K);
int kq_moe_tiles_gemv(int wtype, int nparts, const void* const* packed0, float* const* ys, int64_t N, int64_t K, const void* image,
                      int64_t img_rows, const int* tile_expert, const int* tile_row0, const int* tile_rows, const int* ntiles,
                      unsigned max_tiles, const int* row_ids, int row_div, const int* out_ids, hipStream_t st);
bool kx_moe_tiles_fit(int wtype, int64_t N, int64_t K);
int kx_tile_rows();
int kx_moe_tiles(int wtype, int nparts, const void* const* packed0, float* const* ys, int64_t N, int64_t K, const void* image,
                 int64_t img_rows, const int* tile_expert, const int* tile_row0, const int* tile_rows, const int* ntiles,
                 unsigned max_tiles, const int* row_ids, int row_div, const int* out_ids, int silu_mul, hipStream_t st);
// 0: by the number of pairs per expert; 1: always pairs as GEMV rows; 2: always tiles of eight rows; 3: always tiles of 32 rows
// (where the format has them)
static int g_moe_kq_path = 0;
constexpr int KQ_MOE_TILE = 8;
struct KqMoeCarve {
  float *g, *u, *h, *per;
  char *ximg, *himg;
  RouteOut ro;
};
static KqMoeCarve carve_kq_moe(Carver& c, int64_t T, int64_t H, int64_t I, int E, int k) {
  KqMoeCarve r;
  const size_t slots = (size_t)T * k;
  r.g = c.take<float>(slots * I);
  r.u = c.take<float>(slots * I);
  r.h = c.take<float>(slots * I);
  r.per = c.take<float>(slots * H);
  r.ximg = c.take<char>(kq_image_bytes(T, H));
  r.himg = c.take<char>(kq_image_bytes((int64_t)slots, I));
  r.ro = carve_route(c, E, (int64_t)slots, KQ_MOE_TILE);
  return r;
}
}  // namespace mllmhip

MLLM_API int mllm_hip_moe_kq_set_path(int path) {
  if (path < 0 || path > 3) return MLLM_HIP_E_BADARG;
  g_moe_kq_path = path;
  return 0;
}

MLLM_API size_t mllm_hip_moe_kq_workspace_bytes(int64_t T, int64_t H, int64_t I, int E, int k) {
  if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || k <= 0 || H % 256 || I % 256) return 0;
  Carver c(nullptr);
  carve_kq_moe(c, T, H, I, E, k);
  return c.used;
}

MLLM_API int mllm_hip_moe_ffn_kq2(int wtype, int wtype_down, const void* gate_packed, const void* up_packed, const void* down_packed,
                                  const void* x, int x_dtype, const int32_t* topk_ids, const float* topk_w, float* y, int64_t T,
                                  int64_t H, int64_t I, int E, int k, void* workspace, void* stream) {
  if ((wtype != MLLM_HIP_Q4_K && wtype != MLLM_HIP_Q6_K) || (wtype_down != MLLM_HIP_Q4_K && wtype_down != MLLM_HIP_Q6_K) || !gate_packed || !up_packed || !down_packed || !x || !topk_ids ||
      !topk_w || !y || !workspace || T <= 0 || E <= 0 || k <= 0)
    return MLLM_HIP_E_BADARG;
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  if (H <= 0 || I <= 0 || H % 256 || I % 256 || T * k > 65535) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16 ||
      reinterpret_cast<uintptr_t>(gate_packed) % 16 || reinterpret_cast<uintptr_t>(up_packed) % 16 ||
      reinterpret_cast<uintptr_t>(down_packed) % 16 || reinterpret_cast<uintptr_t>(y) % 16)
    return MLLM_HIP_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int slots = (int)(T * k);
  Carver c(workspace);
  const KqMoeCarve w = carve_kq_moe(c, T, H, I, E, k);
  float *g = w.g, *u = w.u, *h = w.h, *per = w.per;
  // More than about one pair per expert (Q6_K: half a pair): the pairs are sorted by expert and run as tiles of eight rows on the matrix-core
  // kernels, so an expert's matrices are streamed once per eight pairs instead of once per pair (the grouped form).
  // x and h are quantized to Q8_K once (bit-exact images), the tiles gather their rows from the images.
  const bool tiles_ok = E <= MOE_MAX_EXPERTS && kq_moe_tiles_fit(wtype, H) && kq_moe_tiles_fit(wtype_down, I) &&
                        (size_t)E + (size_t)slots / KQ_MOE_TILE + 1 <= 65535;
  // measured at 128 experts, top-8 (pairs / tiles, us): Q4_K 16 tokens 80 / 84, 24: 112 / 97, 32: 145 / 112, 64: 289 / 153,
  // 512: 2182 / 480; Q6_K 8 tokens 79 / 77, 16: 142 / 126, 32: 260 / 165, 512: 3976 / 760
  const bool many = (wtype == MLLM_HIP_Q4_K && wtype_down == MLLM_HIP_Q4_K) ? slots > E : 2 * slots > E;
  // Four pairs per expert and more: tiles of 32 rows, weights as the second operand of 32 x 32 matrix instructions (one pass
  // over an expert's weights per 32 pairs, one unpacking per 32 rows).  Same integer arithmetic; silu(gate) * up is formed where
  // the two results leave their kernel (six launches).
  const bool tiles32_ok = E <= MOE_MAX_EXPERTS && kx_moe_tiles_fit(wtype, I, H) && kx_moe_tiles_fit(wtype_down, H, I);
  if (tiles32_ok && (g_moe_kq_path == 3 || (g_moe_kq_path == 0 && slots >= 4 * E))) {
    const int th = kx_tile_rows();
    const unsigned max_tiles = (unsigned)(E + slots / th + 1);
    RC_RET(launch_route(topk_ids, slots, E, th, w.ro, st));
    RC_RET(kq_quantize_image(x, x_dtype, w.ximg, T, H, st));
    const void* gu2[2] = {gate_packed, up_packed};
    float* guy2[2] = {h, u};  // silu(gate) * up, rows in expert-sorted order
    RC_RET(kx_moe_tiles(wtype, 2, gu2, guy2, I, H, w.ximg, T, w.ro.tile_expert, w.ro.tile_row0, w.ro.tile_rows, w.ro.ntiles, max_tiles,
                        w.ro.sorted_idx, k, nullptr, 1, st));
    RC_RET(kq_quantize_image(h, MLLM_HIP_F32, w.himg, slots, I, st));
    const void* dn2[1] = {down_packed};
    float* dny2[1] = {per};  // row t * k + j
    RC_RET(kx_moe_tiles(wtype_down, 1, dn2, dny2, H, I, w.himg, slots, w.ro.tile_expert, w.ro.tile_row0, w.ro.tile_rows, w.ro.ntiles,
                        max_tiles, nullptr, 1, w.ro.sorted_idx, 0, st));
    const int64_t total2 = T * H;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total2 / 4 + 255) / 256)), dim3(256), 0, st, per, topk_w, topk_ids, y, T,
                       (int)H, k, E);
    return (int)hipGetLastError();
  }
  if (tiles_ok && (g_moe_kq_path == 2 || ((g_moe_kq_path == 0 || g_moe_kq_path == 3) && many))) {
    const unsigned max_tiles = (unsigned)(E + slots / KQ_MOE_TILE + 1);
    RC_RET(launch_route(topk_ids, slots, E, KQ_MOE_TILE, w.ro, st));
    RC_RET(kq_quantize_image(x, x_dtype, w.ximg, T, H, st));
    const void* gu2[2] = {gate_packed, up_packed};
    float* guy2[2] = {g, u};  // rows in expert-sorted order
    RC_RET(kq_moe_tiles_gemv(wtype, 2, gu2, guy2, I, H, w.ximg, T, w.ro.tile_expert, w.ro.tile_row0, w.ro.tile_rows, w.ro.ntiles,
                             max_tiles, w.ro.sorted_idx, k, nullptr, st));
    // positions past the last valid pair (invalid expert ids) are never written nor read: the tiles cover offsets[E] rows
    RC_RET(mllm_hip_silu_mul(g, u, h, MLLM_HIP_F32, slots, I, nullptr, MLLM_HIP_SCALE_IEEE, stream));
    RC_RET(kq_quantize_image(h, MLLM_HIP_F32, w.himg, slots, I, st));
    const void* dn2[1] = {down_packed};
    float* dny2[1] = {per};  // row t * k + j
    RC_RET(kq_moe_tiles_gemv(wtype_down, 1, dn2, dny2, H, I, w.himg, slots, w.ro.tile_expert, w.ro.tile_row0, w.ro.tile_rows,
                             w.ro.ntiles, max_tiles, nullptr, 1, w.ro.sorted_idx, st));
    const int64_t total2 = T * H;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total2 / 4 + 255) / 256)), dim3(256), 0, st, per, topk_w, topk_ids, y, T,
                       (int)H, k, E);
    return (int)hipGetLastError();
  }
  const void* gu[2] = {gate_packed, up_packed};
  float* guy[2] = {g, u};
  int rc = kq_moe_gemv(wtype, 2, gu, guy, I, H, x, x_dtype, nullptr, topk_ids, E, slots, k, st);
  if (rc) return rc;
  // silu(g) * u: up to 32 pairs it is formed where the down GEMV reads its activations (same fp32 operations; one launch
  // fewer: one token 17.8 -> 16.4 us); with more pairs every down workgroup reading g and u costs more than the elementwise
  // launch (eight tokens 50 against 48 us)
  const void* dn[1] = {down_packed};
  float* dny[1] = {per};
  if (slots <= 32) {
    rc = kq_moe_gemv(wtype_down, 1, dn, dny, H, I, g, MLLM_HIP_F32, u, topk_ids, E, slots, 1, st);
  } else {
    rc = mllm_hip_silu_mul(g, u, h, MLLM_HIP_F32, slots, I, nullptr, MLLM_HIP_SCALE_IEEE, stream);
    if (rc) return rc;
    rc = kq_moe_gemv(wtype_down, 1, dn, dny, H, I, h, MLLM_HIP_F32, nullptr, topk_ids, E, slots, 1, st);
  }
  if (rc) return rc;
  const int64_t total = T * H;
  hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, st, per, topk_w, topk_ids, y, T,
                     (int)H, k, E);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_moe_ffn_kq(int wtype, const void* gate_packed, const void* up_packed, const void* down_packed, const void* x,
                                 int x_dtype, const int32_t* topk_ids, const float* topk_w, float* y, int64_t T, int64_t H,
                                 int64_t I, int E, int k, void* workspace, void* stream) {
  return mllm_hip_moe_ffn_kq2(wtype, wtype, gate_packed, up_packed, down_packed, x, x_dtype, topk_ids, topk_w, y, T, H, I, E, k, workspace,
                              stream);
}
