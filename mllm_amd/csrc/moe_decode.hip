// MoE expert FFN for a handful of tokens (decode): two launches, no routing pass.
//
//   reference: Qwen3MoE::moeInfer + Qwen3MoeMLP::forward, mllm/models/qwen3_moe/modeling_qwen3_moe_fa2.hpp:98-100,175-238 -- per
//   active expert three small Linears (CPULinearOp -> quantize_row_q8_0 + block dots), SiLU and product in between, the
//   weighted sum over the token's experts at the end.
//
// With up to eight tokens every (token, expert) pair is one activation row, so the path is a set of GEMVs and HBM-bound:
// 8 experts x 3 matrices x 0.88 MB for one Qwen3-30B-A3B token.  The grouped-GEMM path spends five launches and 128-row
// tiles on it.  Here:
//   launch 1  one workgroup per (slot, 32 intermediate channels): quantizes the token's x (Q8_0, bit-exact), gate and up
//             rows of the slot's expert as PAIRED rows of a lane group, h = silu(g) * u, and the Q8_0 image of those 32
//             values of h (exactly one block) for launch 2;
//   launch 2  one workgroup per (token, 16 output rows): copies the images of the token's k slots into LDS and walks the
//             experts in slot order, acc += w_j * (W_down,e_j . h_j), the weights of the next eight experts in flight
//             while one is multiplied.  The sum runs in the reference's order (slot j ascending), no atomics.
// Arithmetic as in the GEMV kernel: exact int32 block dots, fp32 fma with dW * dX.
#include "qgemv_kernel.h"

namespace mllmhip {

__device__ __forceinline__ float silu_vec(float x) { return x * (1.0f / (1.0f + exp_poly(-x))); }

struct MoeDecodeArgs {
  const char* gate;  // E packed [I][H] matrices back to back
  const char* up;
  const char* down;  // E packed [H][I]
  size_t gu_stride, d_stride;
  const void* x;     // [T][H]
  const int32_t* ids;  // [T][k]
  const float* w;      // [T][k]
  unsigned char* img;  // per slot: Q8_0 image of h (one activation row of I elements), img_stride bytes apart
  float* y;            // [T][H]
  int img_stride;
  int T, H, I, E, k, x86;
};

// ---- launch 1: gate / up / SiLU * up / re-quantization ----------------------------------------------------------------
// 512 threads: wave w, lane group grp (16 lanes) -> intermediate channel n = n0 + 4 w + grp; row 0 of the group is the gate
// row, row 1 the up row; lanes stride over the block columns.
template <int WT, int XT>
__global__ __launch_bounds__(512) void moe_decode_gateup_kernel(MoeDecodeArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int nb = a.H / QK, nbp = (int)scale_row_stride(a.H);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slot = blockIdx.y;
  const int tok = slot / a.k;
  const int e = a.ids[slot];
  const int n0 = blockIdx.x * 32;
  const QImage out{a.img + (size_t)slot * a.img_stride, 1, a.I / QK, a.x86};
  float* s_h = reinterpret_cast<float*>(smem + align_up((size_t)nb * 40, 16));
  // activations of the token first, weights behind them (requests return in order); the activations do not wait for the
  // slot's expert id either, which the weight addresses need
  const int nitems = nb * 4;
  XRaw<XT> raw;
  load_x8<XT>(a.x, ((int64_t)tok * nb * 4 + min(tid, nitems - 1)) * 8, raw);
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  if (e < 0 || e >= a.E) {  // uniform: this slot contributes nothing; its image block reads as zeros
    if (tid < 4) {
      const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      quad_quantize_to_image(z, out, 0, n0 / QK, tid, true);
    }
    return;
  }

  const int grp = lane >> 4, c0 = lane & 15;
  const int n = n0 + 4 * wave + grp;
  const PackedView wv[2] = {packed_view(WT, a.gate + (size_t)e * a.gu_stride, a.I, a.H), packed_view(WT, a.up + (size_t)e * a.gu_stride, a.I, a.H)};
  constexpr int U = 4;  // block columns per lane and trip: 64 columns per trip
  u32x4 w0[U][2], w1[WT == MLLM_HIP_Q8_0 ? U : 1][2];
  uint16_t dw[U][2];
  auto load_trip = [&](int t0) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = min(t0 + 16 * u + c0, nb - 1);  // clamped: columns past the row are loaded twice and not used
#pragma unroll
      for (int r = 0; r < 2; r++) {
        const size_t blk = (size_t)n * nb + col;
        w0[u][r] = wv[r].q0[blk];
        if (WT == MLLM_HIP_Q8_0) w1[WT == MLLM_HIP_Q8_0 ? u : 0][r] = wv[r].q1[blk];
        dw[u][r] = wv[r].d[(size_t)n * nbp + col];
      }
    }
  };
  load_trip(0);
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // x -> Q8_0 in LDS, laid out like the GEMV kernel's image (one activation row)
  const QImage xi{smem, 1, nb, a.x86};
  {
    float v[8];
    x8_to_f32<XT>(raw, v);
    if (tid < nitems) quad_quantize_to_image(v, xi, 0, tid >> 2, tid & 3, true);  // whole quads: nitems is a multiple of 4
    for (int it = tid + 512; it < nitems; it += 512) {
      XRaw<XT> rw;
      load_x8<XT>(a.x, ((int64_t)tok * nb * 4 + it) * 8, rw);
      x8_to_f32<XT>(rw, v);
      quad_quantize_to_image(v, xi, 0, it >> 2, it & 3, true);
    }
  }
  __syncthreads();
  const u32x4* s_lo = reinterpret_cast<const u32x4*>(smem);
  const u32x4* s_hi = s_lo + nb;
  const float* s_d = reinterpret_cast<const float*>(s_hi + nb);
  const int* s_n8 = reinterpret_cast<const int*>(s_d + nb);

  float acc[2] = {0.f, 0.f};
  for (int t0 = 0; t0 < nb; t0 += 16 * U) {
    if (t0) load_trip(t0);
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = t0 + 16 * u + c0;
      if (col < nb) {
        const u32x4 xlo = s_lo[col], xhi = s_hi[col];
        const float dx = s_d[col];
        const int n8 = s_n8[col];
#pragma unroll
        for (int r = 0; r < 2; r++) {
          const int isum = block_dot<WT>(w0[u][r], w1[WT == MLLM_HIP_Q8_0 ? u : 0][r], xlo, xhi, n8);
          acc[r] = fmaf(f16bits_to_f32(dw[u][r]) * dx, (float)isum, acc[r]);
        }
      }
    }
  }
  const float g = group_sum<16>(acc[0]), u = group_sum<16>(acc[1]);
  if (c0 == 0) s_h[4 * wave + grp] = silu_vec(g) * u;
  __syncthreads();
  if (tid < 4) {  // one quad: the 32 values are exactly one Q8_0 block of h
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = s_h[8 * tid + i];
    quad_quantize_to_image(v, out, 0, n0 / QK, tid, true);
  }
}

// ---- launch 2: down projection and the weighted sum over the token's experts -------------------------------------------
// DNW waves per workgroup: wave w, lane group grp (8 lanes) -> output row n = n0 + 8 w + grp; lanes stride over the block
// columns (up to 32 of them: I <= 1024).
constexpr int DNW = 2;  // measured: one wave per workgroup is 6 % slower at one and at eight tokens
template <int WT>
__global__ __launch_bounds__(DNW * 64) void moe_decode_down_kernel(MoeDecodeArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int nb = a.I / QK, nbp = (int)scale_row_stride(a.I);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tok = blockIdx.y;
  const int grp = lane >> 3, c0 = lane & 7;
  const int n = blockIdx.x * (8 * DNW) + 8 * wave + grp;
  constexpr int U = 4;
  struct Chunk {
    u32x4 w0[U];
    u32x4 w1[WT == MLLM_HIP_Q8_0 ? U : 1];
    uint16_t dw[U];
    int e;     // the slot's expert id as routed (may be invalid)
    float wt;  // and its weight: read with the id, not in the walk over the experts below (a wait for scalar memory per expert)
  };
  auto load_expert = [&](int j, Chunk& c) {
    int e = a.ids[tok * a.k + min(j, a.k - 1)];
    c.e = e;
    c.wt = a.w[tok * a.k + min(j, a.k - 1)];
    e = min(max(e, 0), a.E - 1);  // an invalid slot loads some expert's rows and is skipped at the sum
    const PackedView v = packed_view(WT, a.down + (size_t)e * a.d_stride, a.H, a.I);
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = min(8 * u + c0, nb - 1);
      const size_t blk = (size_t)n * nb + col;
      c.w0[u] = v.q0[blk];
      if (WT == MLLM_HIP_Q8_0) c.w1[WT == MLLM_HIP_Q8_0 ? u : 0] = v.q1[blk];
      c.dw[u] = v.d[(size_t)n * nbp + col];
    }
  };
  // the weights of the next PF experts are in flight while one is multiplied: with only the next one requested the walk over a
  // token's experts is a chain of exposed load latencies (8.8 us for eight experts, 7 MB)
  constexpr int PF = WT == MLLM_HIP_Q4_0 ? 8 : 4;
  Chunk buf[PF];
  // the images of this token's k slots are contiguous; their first pieces are requested ahead of the weights (requests
  // return in order, and the addresses of the weights wait for the expert ids)
  const int n16 = a.k * a.img_stride / 16;
  const u32x4* src = reinterpret_cast<const u32x4*>(a.img + (size_t)tok * a.k * a.img_stride);
  constexpr int IP = 4;
  u32x4 ip[IP];
#pragma unroll
  for (int i = 0; i < IP; i++)
    if (tid + i * DNW * 64 < n16) ip[i] = src[tid + i * DNW * 64];
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int p = 0; p < PF; p++) load_expert(p, buf[p]);  // slots past k load the last expert again and are not used
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < IP; i++)
    if (tid + i * DNW * 64 < n16) reinterpret_cast<u32x4*>(smem)[tid + i * DNW * 64] = ip[i];
  for (int c = tid + IP * DNW * 64; c < n16; c += DNW * 64) reinterpret_cast<u32x4*>(smem)[c] = src[c];
  __syncthreads();

  float total = 0.f;
  for (int j0 = 0; j0 < a.k; j0 += PF) {
#pragma unroll
    for (int p = 0; p < PF; p++) {
      const int j = j0 + p;
      if (j < a.k) {  // uniform
        const unsigned char* im = smem + (size_t)j * a.img_stride;
        const u32x4* s_lo = reinterpret_cast<const u32x4*>(im);
        const u32x4* s_hi = s_lo + nb;
        const float* s_d = reinterpret_cast<const float*>(s_hi + nb);
        const int* s_n8 = reinterpret_cast<const int*>(s_d + nb);
        float acc = 0.f;
#pragma unroll
        for (int u = 0; u < U; u++) {
          const int col = 8 * u + c0;
          if (col < nb) {
            const int isum = block_dot<WT>(buf[p].w0[u], buf[p].w1[WT == MLLM_HIP_Q8_0 ? u : 0], s_lo[col], s_hi[col], s_n8[col]);
            acc = fmaf(f16bits_to_f32(buf[p].dw[u]) * s_d[col], (float)isum, acc);
          }
        }
        const float v = group_sum<8>(acc);
        if (buf[p].e >= 0 && buf[p].e < a.E) total = total + v * buf[p].wt;
        if (j + PF < a.k) load_expert(j + PF, buf[p]);  // uniform: refill the slot just used
      }
    }
  }
  if (c0 == 0) a.y[(size_t)tok * a.H + n] = total;
}

// image bytes of one slot, padded to 16
__host__ __device__ inline int moe_decode_img_stride(int64_t I) { return (int)align_up((size_t)(I / QK) * 40, 16); }

size_t moe_decode_workspace_bytes(int64_t T, int64_t I, int k) { return (size_t)T * k * moe_decode_img_stride(I); }

// Whether the per-pair kernels run.  They read an expert's matrices once per pair that uses it; measured at 128 experts,
// top-8 (2048 x 768) they are the fastest form up to one pair per expert (16 tokens: 54 us; the eight-row tiles below 53 us, the
// grouped 64-row tiles 144 us), and the row tiles from there on (32 tokens: 97 vs 76 us).
// g_moe_decode_tokens > 0 replaces the rule by a token limit (comparison runs, tests).
static int g_moe_decode_tokens = 0;
int moe_decode_set_tokens(int tokens) {
  if (tokens < 0 || tokens > 4096) return MLLM_HIP_E_BADARG;
  g_moe_decode_tokens = tokens;
  return 0;
}

bool moe_decode_applies(int64_t T, int64_t H, int64_t I, int E, int k) {
  const bool few = g_moe_decode_tokens > 0 ? T <= g_moe_decode_tokens : (T <= 8 || (T <= 4096 && T * k <= (int64_t)E));
  return few && I % 32 == 0 && I / QK <= 32 && H % 32 == 0 && k <= 64 && H / QK * 40 + 256 <= 64 * 1024 &&
         (int64_t)k * moe_decode_img_stride(I) <= 64 * 1024 && T * k <= 65535;
}

int launch_moe_decode(int wtype, const void* gate, const void* up, const void* down, const void* x, int x_dtype, const int32_t* ids,
                      const float* w, float* y, int64_t T, int64_t H, int64_t I, int E, int k, int x86, void* workspace,
                      hipStream_t st) {
  MoeDecodeArgs a{};
  a.gate = reinterpret_cast<const char*>(gate);
  a.up = reinterpret_cast<const char*>(up);
  a.down = reinterpret_cast<const char*>(down);
  a.gu_stride = packed_bytes(wtype, I, H);
  a.d_stride = packed_bytes(wtype, H, I);
  a.x = x;
  a.ids = ids;
  a.w = w;
  a.img = reinterpret_cast<unsigned char*>(workspace);
  a.y = y;
  a.img_stride = moe_decode_img_stride(I);
  a.T = (int)T; a.H = (int)H; a.I = (int)I; a.E = E; a.k = k; a.x86 = x86;
  const size_t lds1 = align_up((size_t)(H / QK) * 40, 16) + 32 * sizeof(float);
  const dim3 g1((unsigned)(I / 32), (unsigned)(T * k));
#define GU(WT_, XT_) hipLaunchKernelGGL((moe_decode_gateup_kernel<WT_, XT_>), g1, dim3(512), lds1, st, a)
  if (wtype == MLLM_HIP_Q4_0) {
    if (x_dtype == MLLM_HIP_F32) GU(MLLM_HIP_Q4_0, MLLM_HIP_F32); else GU(MLLM_HIP_Q4_0, MLLM_HIP_BF16);
  } else {
    if (x_dtype == MLLM_HIP_F32) GU(MLLM_HIP_Q8_0, MLLM_HIP_F32); else GU(MLLM_HIP_Q8_0, MLLM_HIP_BF16);
  }
#undef GU
  HIP_RET(hipGetLastError());
  const size_t lds2 = (size_t)k * a.img_stride;
  const dim3 g2((unsigned)(H / (8 * DNW)), (unsigned)T);
  if (wtype == MLLM_HIP_Q4_0) hipLaunchKernelGGL((moe_decode_down_kernel<MLLM_HIP_Q4_0>), g2, dim3(DNW * 64), lds2, st, a);
  else hipLaunchKernelGGL((moe_decode_down_kernel<MLLM_HIP_Q8_0>), g2, dim3(DNW * 64), lds2, st, a);
  return (int)hipGetLastError();
}

// ---- a few rows per expert ------------------------------------------------------------------------------------------------
// Between decode and prefill (up to about eight pairs per expert) the per-pair kernels read an expert's matrices once per
// pair and the 64-row tiles of the grouped path are mostly empty.  Here the pairs are sorted by expert (the routing pass of
// the grouped path with tiles of eight rows) and one workgroup serves the rows of one tile: the weights are read once per
// tile, each row has its own Q8_0 image in LDS and its own accumulators.  Same block arithmetic and the same two stages as
// above; the down stage writes one row per pair and the weighted sum over a token's slots is the grouped path's combine pass
// (slot order, no atomics).
constexpr int MOE_ROWS = 8;  // rows of a tile

struct MoeRowsArgs {
  MoeDecodeArgs d;
  const int* tile_expert;
  const int* tile_row0;
  const int* tile_rows;
  const int* ntiles;
  const int* sorted_idx;  // flat index t*k + j at every expert-sorted position
  float* per;             // [T*k][H] down results by flat index
  int x_stride;           // bytes of one row's image of x in LDS
};

// gate / up / SiLU * up / re-quantization for the R (>= rows) rows of one tile; thread roles as in moe_decode_gateup_kernel
template <int WT, int XT, int R>
__device__ __forceinline__ void moe_rows_gateup(const MoeRowsArgs& b, const int e, const int row0, const int rows, unsigned char* smem) {
  const MoeDecodeArgs& a = b.d;
  const int nb = a.H / QK, nbp = (int)scale_row_stride(a.H);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * 32;
  const int grp = lane >> 4, c0 = lane & 15;
  const int n = n0 + 4 * wave + grp;
  float* s_h = reinterpret_cast<float*>(smem + (size_t)MOE_ROWS * b.x_stride);

  const PackedView wv[2] = {packed_view(WT, a.gate + (size_t)e * a.gu_stride, a.I, a.H), packed_view(WT, a.up + (size_t)e * a.gu_stride, a.I, a.H)};
  constexpr int U = (R > 4 || (R > 2 && WT == MLLM_HIP_Q8_0)) ? 1 : 2;  // block columns per lane and trip, as 128 registers allow
  // two register sets: the next trip's weights are requested before the current trip is multiplied
  u32x4 w0[U][2], w1[WT == MLLM_HIP_Q8_0 ? U : 1][2], w0n[U][2], w1n[WT == MLLM_HIP_Q8_0 ? U : 1][2];
  uint16_t dw[U][2], dwn[U][2];
  auto load_trip = [&](int t0) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = min(t0 + 16 * u + c0, nb - 1);
#pragma unroll
      for (int r = 0; r < 2; r++) {
        const size_t blk = (size_t)n * nb + col;
        w0n[u][r] = wv[r].q0[blk];
        if (WT == MLLM_HIP_Q8_0) w1n[WT == MLLM_HIP_Q8_0 ? u : 0][r] = wv[r].q1[blk];
        dwn[u][r] = wv[r].d[(size_t)n * nbp + col];
      }
    }
  };
  // the rows' activations -> Q8_0 images in LDS, four requests in flight per thread; items are eighths of a block, so the four
  // lanes of a quad always hold one block of one row.  The first trip of weights is requested right behind the first batch
  // of activations (requests return in order: ahead of them it would hold the activations back, whose addresses already
  // wait for the sorted positions; 32 / 64 tokens of the 128-expert layer: 63.0 / 93.0 -> 61.4 / 90.5 us)
  const int nitems = nb * 4, total = rows * nitems;
  if (tid >= total) load_trip(0);  // (threads without an item)
  for (int it0 = tid; it0 < total; it0 += 512 * 4) {
    XRaw<XT> raw[4];
    int rr[4], ii[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int it = min(it0 + 512 * q, total - 1);
      rr[q] = it / nitems;
      ii[q] = it - rr[q] * nitems;
      const int tok = b.sorted_idx[row0 + rr[q]] / a.k;
      load_x8<XT>(a.x, ((int64_t)tok * nitems + ii[q]) * 8, raw[q]);
    }
    if (it0 == tid) load_trip(0);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      if (it0 + 512 * q < total) {  // the same answer in the four lanes of a quad: total and the strides are multiples of 4
        float v[8];
        x8_to_f32<XT>(raw[q], v);
        quad_quantize_to_image(v, QImage{smem + (size_t)rr[q] * b.x_stride, 1, nb, a.x86}, 0, ii[q] >> 2, ii[q] & 3, true);
      }
    }
  }
  __syncthreads();

  float acc[R][2];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r][0] = acc[r][1] = 0.f;
  for (int t0 = 0; t0 < nb; t0 += 16 * U) {
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
      for (int r = 0; r < 2; r++) {
        w0[u][r] = w0n[u][r];
        if (WT == MLLM_HIP_Q8_0) w1[WT == MLLM_HIP_Q8_0 ? u : 0][r] = w1n[WT == MLLM_HIP_Q8_0 ? u : 0][r];
        dw[u][r] = dwn[u][r];
      }
    if (t0 + 16 * U < nb) load_trip(t0 + 16 * U);  // uniform
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = t0 + 16 * u + c0;
      if (col < nb) {
        const float dg = f16bits_to_f32(dw[u][0]), du = f16bits_to_f32(dw[u][1]);
#pragma unroll
        for (int r = 0; r < R; r++) {
          if (r < rows) {  // uniform
            const unsigned char* im = smem + (size_t)r * b.x_stride;
            const u32x4* s_lo = reinterpret_cast<const u32x4*>(im);
            const u32x4 xlo = s_lo[col], xhi = s_lo[nb + col];
            const float dx = reinterpret_cast<const float*>(s_lo + 2 * nb)[col];
            const int n8 = reinterpret_cast<const int*>(s_lo + 2 * nb)[nb + col];
            const int ig = block_dot<WT>(w0[u][0], w1[WT == MLLM_HIP_Q8_0 ? u : 0][0], xlo, xhi, n8);
            const int iu = block_dot<WT>(w0[u][1], w1[WT == MLLM_HIP_Q8_0 ? u : 0][1], xlo, xhi, n8);
            acc[r][0] = fmaf(dg * dx, (float)ig, acc[r][0]);
            acc[r][1] = fmaf(du * dx, (float)iu, acc[r][1]);
          }
          __builtin_amdgcn_sched_barrier(0);  // one row's image block in registers at a time: two workgroups fit a CU
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; r++) {
    if (r < rows) {
      const float g = group_sum<16>(acc[r][0]), u = group_sum<16>(acc[r][1]);
      if (c0 == 0) s_h[r * 32 + 4 * wave + grp] = silu_vec(g) * u;
    }
  }
  __syncthreads();
  if (tid < 4 * rows) {  // one quad per row: the 32 values are exactly one Q8_0 block of that row's h
    const int r = tid >> 2, j = tid & 3;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = s_h[r * 32 + 8 * j + i];
    quad_quantize_to_image(v, QImage{a.img + (size_t)(row0 + r) * a.img_stride, 1, a.I / QK, a.x86}, 0, n0 / QK, j, true);
  }
}

template <int WT, int XT>
__global__ __launch_bounds__(512, 4) void moe_rows_gateup_kernel(MoeRowsArgs b) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int t = blockIdx.y;
  if (t >= min(b.ntiles[0], (int)gridDim.y)) return;
  const int e = b.tile_expert[t], row0 = b.tile_row0[t], rows = b.tile_rows[t];
  if (rows <= 2) moe_rows_gateup<WT, XT, 2>(b, e, row0, rows, smem);
  else if (rows <= 4) moe_rows_gateup<WT, XT, 4>(b, e, row0, rows, smem);
  else moe_rows_gateup<WT, XT, MOE_ROWS>(b, e, row0, rows, smem);
}

// down projection of the rows of one tile: NW waves, wave w, lane group grp (8 lanes) -> output row n = n0 + 8 w + grp
template <int WT, int NW>
__global__ __launch_bounds__(NW * 64) void moe_rows_down_kernel(MoeRowsArgs b) {
  extern __shared__ __align__(16) unsigned char smem[];
  const MoeDecodeArgs& a = b.d;
  const int t = blockIdx.y;
  if (t >= min(b.ntiles[0], (int)gridDim.y)) return;
  const int e = b.tile_expert[t], row0 = b.tile_row0[t], rows = b.tile_rows[t];
  const int nb = a.I / QK, nbp = (int)scale_row_stride(a.I);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = lane >> 3, c0 = lane & 7;
  const int n = blockIdx.x * (8 * NW) + 8 * wave + grp;
  constexpr int U = 4;
  u32x4 w0[U], w1[WT == MLLM_HIP_Q8_0 ? U : 1];
  uint16_t dw[U];
  const PackedView v = packed_view(WT, a.down + (size_t)e * a.d_stride, a.H, a.I);
#pragma unroll
  for (int u = 0; u < U; u++) {
    const int col = min(8 * u + c0, nb - 1);
    const size_t blk = (size_t)n * nb + col;
    w0[u] = v.q0[blk];
    if (WT == MLLM_HIP_Q8_0) w1[WT == MLLM_HIP_Q8_0 ? u : 0] = v.q1[blk];
    dw[u] = v.d[(size_t)n * nbp + col];
  }
  // the images of the tile's rows are contiguous (sorted positions row0 .. row0 + rows - 1)
  const int n16 = rows * a.img_stride / 16;
  const u32x4* src = reinterpret_cast<const u32x4*>(a.img + (size_t)row0 * a.img_stride);
  for (int c = tid; c < n16; c += NW * 64) reinterpret_cast<u32x4*>(smem)[c] = src[c];
  __syncthreads();
  // (the rows' destinations read ahead of this loop, all at once: measured slower, 32 tokens 62 -> 65 us)
  for (int r = 0; r < rows; r++) {  // uniform
    const unsigned char* im = smem + (size_t)r * a.img_stride;
    const u32x4* s_lo = reinterpret_cast<const u32x4*>(im);
    const float* s_d = reinterpret_cast<const float*>(s_lo + 2 * nb);
    const int* s_n8 = reinterpret_cast<const int*>(s_d + nb);
    float acc = 0.f;
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = 8 * u + c0;
      if (col < nb) {
        const int isum = block_dot<WT>(w0[u], w1[WT == MLLM_HIP_Q8_0 ? u : 0], s_lo[col], s_lo[nb + col], s_n8[col]);
        acc = fmaf(f16bits_to_f32(dw[u]) * s_d[col], (float)isum, acc);
      }
    }
    const float val = group_sum<8>(acc);
    if (c0 == 0) b.per[(size_t)b.sorted_idx[row0 + r] * a.H + n] = val;
  }
}

// The row tiles run up to ten pairs per expert (measured as above: 64 tokens 105 us against 175 us for the grouped 64-row
// tiles, 160 tokens 181 against 194 us, 192 tokens 215 against 198 us); a token limit > 0 replaces the rule.
static int g_moe_rows_tokens = 0;
int moe_rows_set_tokens(int tokens) {
  if (tokens < 0 || tokens > 65536) return MLLM_HIP_E_BADARG;
  g_moe_rows_tokens = tokens;
  return 0;
}
static size_t moe_rows_x_stride(int64_t H) { return align_up((size_t)(H / QK) * 40, 16); }
bool moe_rows_applies(int64_t T, int64_t H, int64_t I, int E, int k) {
  const bool few = g_moe_rows_tokens > 0 ? T <= g_moe_rows_tokens : T * k <= 10 * (int64_t)E;
  return few && I % 32 == 0 && I / QK <= 32 && H % 32 == 0 && MOE_ROWS * moe_rows_x_stride(H) + MOE_ROWS * 32 * 4 <= 64 * 1024 &&
         E + T * k / MOE_ROWS + 1 <= 65535;
}
int moe_rows_tile() { return MOE_ROWS; }

// the two stages between the routing pass and the combine pass; img: T*k images of h (moe_decode_workspace_bytes)
int launch_moe_rows(int wtype, const void* gate, const void* up, const void* down, const void* x, int x_dtype, const int* tile_expert,
                    const int* tile_row0, const int* tile_rows, const int* ntiles, const int* sorted_idx, void* img, float* per,
                    int64_t T, int64_t H, int64_t I, int E, int k, int x86, unsigned max_tiles, hipStream_t st) {
  MoeRowsArgs b{};
  MoeDecodeArgs& a = b.d;
  a.gate = reinterpret_cast<const char*>(gate);
  a.up = reinterpret_cast<const char*>(up);
  a.down = reinterpret_cast<const char*>(down);
  a.gu_stride = packed_bytes(wtype, I, H);
  a.d_stride = packed_bytes(wtype, H, I);
  a.x = x;
  a.img = reinterpret_cast<unsigned char*>(img);
  a.img_stride = moe_decode_img_stride(I);
  a.T = (int)T; a.H = (int)H; a.I = (int)I; a.E = E; a.k = k; a.x86 = x86;
  b.tile_expert = tile_expert; b.tile_row0 = tile_row0; b.tile_rows = tile_rows; b.ntiles = ntiles; b.sorted_idx = sorted_idx;
  b.per = per;
  b.x_stride = (int)moe_rows_x_stride(H);
  const size_t lds1 = (size_t)MOE_ROWS * b.x_stride + MOE_ROWS * 32 * sizeof(float);
  const dim3 g1((unsigned)(I / 32), max_tiles);
#define GU(WT_, XT_) hipLaunchKernelGGL((moe_rows_gateup_kernel<WT_, XT_>), g1, dim3(512), lds1, st, b)
  if (wtype == MLLM_HIP_Q4_0) {
    if (x_dtype == MLLM_HIP_F32) GU(MLLM_HIP_Q4_0, MLLM_HIP_F32); else GU(MLLM_HIP_Q4_0, MLLM_HIP_BF16);
  } else {
    if (x_dtype == MLLM_HIP_F32) GU(MLLM_HIP_Q8_0, MLLM_HIP_F32); else GU(MLLM_HIP_Q8_0, MLLM_HIP_BF16);
  }
#undef GU
  HIP_RET(hipGetLastError());
  const size_t lds2 = (size_t)MOE_ROWS * a.img_stride;
  // 64 output rows per workgroup where H allows (a tile's images are copied into LDS once per workgroup, and eight times
  // fewer workgroups are dispatched), else 16
  if (H % 64 == 0) {
    const dim3 g2((unsigned)(H / 64), max_tiles);
    if (wtype == MLLM_HIP_Q4_0) hipLaunchKernelGGL((moe_rows_down_kernel<MLLM_HIP_Q4_0, 8>), g2, dim3(512), lds2, st, b);
    else hipLaunchKernelGGL((moe_rows_down_kernel<MLLM_HIP_Q8_0, 8>), g2, dim3(512), lds2, st, b);
  } else {
    const dim3 g2((unsigned)(H / 16), max_tiles);
    if (wtype == MLLM_HIP_Q4_0) hipLaunchKernelGGL((moe_rows_down_kernel<MLLM_HIP_Q4_0, 2>), g2, dim3(128), lds2, st, b);
    else hipLaunchKernelGGL((moe_rows_down_kernel<MLLM_HIP_Q8_0, 2>), g2, dim3(128), lds2, st, b);
  }
  return (int)hipGetLastError();
}

}  // namespace mllmhip
