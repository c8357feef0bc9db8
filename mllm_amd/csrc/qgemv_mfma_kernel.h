// Q4_0 / Q8_0 decode GEMV for three to eight activation rows on the matrix cores.
//
// Same arithmetic as the one- and two-row kernel (qgemv_kernel.h; reference: quantize_q8.cpp:106-190 for the activations,
// llamafile_sgemm.cpp:697-743 for block dot + scaling): exact int32 block sums, acc = fma(fp32(dW * dX), float(isum), acc).
// With several rows the vector-ALU form (one dot4 chain and two 16-byte LDS reads per row and block) is bound by LDS reads
// and their latency: 24 us for the gate + up launch of the 4B layer at eight rows against 7 us at one.
//
// Here v_mfma_i32_16x16x64_i8 produces the block sums.  The instruction sums over K = 64, a block has 32 elements and every
// block carries its own scales, so the sums of different blocks must not mix.  They are kept apart by the ACTIVATION
// operand: lane group g (16 lanes, 16 bytes of K each) of the weight operand holds half a block of block 4j + g of the
// lane's weight row -- simply the 16 bytes that lane loaded, low nibbles for the first instruction, high nibbles for the
// second -- and output column 4q + t gets activation codes only in lane group q (block 4j + q, activation row t), zeros in
// the other three groups.  Column 4q + t of the result is then the block sum of (block 4j + q, row t) alone: two
// instructions per four blocks and four activation rows, every lane of the result useful, no data movement between
// lanes.  Rows 4..7 take a second pair of instructions with the same weight operands.
//
// Result layout: lane l holds weight rows 4 (l / 16) + 0..3 of column l % 16, so the scaling is four fused multiply-adds per
// lane and instruction pair; a lane accumulates the blocks = q mod 4 of one activation row, the four partial sums meet in a
// two-step butterfly at the end.
//
// Work split: a wave owns 16 weight rows and one K slice of at most 40 blocks (all of it requested up front); the S slices
// of a row tile are waves of one workgroup and are summed through LDS in slice order.  S depends on the row length only,
// so a matrix gives the same bits alone or as part of a multi-matrix launch.
#pragma once
#include "qgemv_kernel.h"

namespace mllmhip {

typedef int v4i_t __attribute__((ext_vector_type(4)));

constexpr int MF_NG = 10;  // groups of four blocks per trip: 40 blocks, all in flight

// quantization of eight elements by one lane of a quad (the four lanes share a block): codes, effective scale, -8 * sum
__device__ __forceinline__ void quad_quantize(const float (&v)[8], int x86, uint32_t (&pk)[2], float& deff, int& n8) {
  float amax = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[e]));
  amax = fmaxf(amax, dpp_f<0xB1>(amax));
  amax = fmaxf(amax, dpp_f<0x4E>(amax));
  float d, idv;
  q8_scales(amax, d, idv);
  pk[0] = q8_pack4(&v[0], idv);  // |v| <= amax: within -127 .. 127, the reference's saturation never acts
  pk[1] = q8_pack4(&v[4], idv);
  int sum = __builtin_amdgcn_sdot4((int)pk[0], 0x01010101, 0, false);
  sum = __builtin_amdgcn_sdot4((int)pk[1], 0x01010101, sum, false);
  sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xf, 0xf, true);
  sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xf, 0xf, true);
  uint16_t bits = f32_to_f16bits(d);
  if (x86) bits = x86_scale_bits(bits);
  deff = f16bits_to_f32(bits);
  n8 = -8 * sum;
}

// row stride of the activation code planes in 16-byte units: = 4 mod 16, so that the 16 addresses (4 blocks x 4 rows) of one
// operand read fall into 16 different bank groups
__host__ __device__ inline int mf_row_stride(int nb) { return nb + ((4 - nb % 16) + 16) % 16; }

// blockDim = NWV * 64; a workgroup holds NWV / S row tiles, S slices each.  nbs = blocks per slice (a multiple of 8).
// LDS: xlo [MT][rs] 16 bytes: codes of elements 0..15 of (row, block); xhi likewise elements 16..31; 40 blocks of slack;
//      zrow [nb + 40] zero blocks (the operand of the lane groups that must not contribute)
//      xs [MT][nb] {effective scale, -8 * sum}, 40 entries of slack
//      ws per wave [whole trips][16 rows] fp32 weight scales of its tile and slice, zero past the slice
//      red per wave [MT / 4][64] four partial sums
// PAIR (the MLP front half, mlp_mfma.hip): parts 0 and 1 are the gate and the up projection with the same N; a workgroup
// holds whole 32-channel blocks of h = silu(gate) * up: per row tile 2 S waves (gate slices, then up slices).  The wave of
// gate slice 0 sums both sets of slices, forms h, stores it and / or hands it to the quads that write its Q8_0 image.
struct MfmaMlpOut {
  float* h;              // fp32 [M][N] or null
  unsigned char* image;  // image of h for MT rows or null
  int exp_accurate;
};
template <int WT, int XT, int MT, bool PAIR>
__global__ __launch_bounds__(PAIR ? 1024 : 512) void gemv_mfma_kernel(GemvArgs a, int S, int nbs, MfmaMlpOut mo) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int TH = MT / 4;  // groups of four activation rows
  constexpr int TRIP = 4 * MF_NG;
  const int nb = a.nb, nbp = a.nbp;
  const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: slice bounds and LDS offsets below are uniform
  int pidx = 0;  // uniform: which matrix this workgroup (PAIR: this wave) works on
  if (PAIR) {
    pidx = (wave / S) & 1;
  } else {
#pragma unroll
    for (int p = 1; p < GEMV_MAX_PARTS; p++)
      if (p < a.nparts && (int)blockIdx.x >= a.wg_start[p]) pidx = p;
  }
  const GemvPart& pt = a.part[pidx];
  const int N = pt.N;
  const int tiles_wg = PAIR ? nwaves / (2 * S) : nwaves / S;
  const int tile_l = PAIR ? wave / (2 * S) : wave / S;  // row tile within the workgroup
  const int tile = ((int)blockIdx.x - (PAIR ? 0 : a.wg_start[pidx])) * tiles_wg + tile_l;  // uniform per wave
  const int slice = wave % S;
  const int row0 = tile * 16;
  const bool tile_ok = row0 < N;
  const int b0 = slice * nbs, b1 = min(nb, b0 + nbs);  // this wave's blocks

  const int rs = mf_row_stride(nb);
  const int wsb = (nbs + TRIP - 1) / TRIP * TRIP;
  u32x4* xlo = reinterpret_cast<u32x4*>(smem);
  u32x4* xhi = xlo + (size_t)MT * rs;
  u32x4* zrow = xhi + (size_t)MT * rs + TRIP;
  u32x2* xs = reinterpret_cast<u32x2*>(zrow + nb + TRIP);
  float* ws_all = reinterpret_cast<float*>(xs + (size_t)MT * nb + TRIP);
  float* ws = ws_all + (size_t)wave * wsb * 16;
  f32x4* red = reinterpret_cast<f32x4*>(ws_all + (size_t)nwaves * wsb * 16) + (size_t)wave * TH * 64;

  // ---- 1. activation requests (return first) ---------------------------------------------------------------------
  // image (rows m, blocks b): planes lo [m][b] 16 B, hi [m][b] 16 B, scales [m][b], -8 sums [m][b].  Wave w copies rows
  // w, w + nwaves, ...; the first two 64-block stretches of each row are requested here, the rest after the weights.
  const int mnb = MT * nb;
  const u32x4* img_lo = reinterpret_cast<const u32x4*>(a.x);
  const u32x4* img_hi = img_lo + mnb;
  const float* img_d = reinterpret_cast<const float*>(img_hi + mnb);
  const int* img_n8 = reinterpret_cast<const int*>(img_d + mnb);
  constexpr int RW = MT / 4;  // rows per wave with four waves (eight waves: at most one)
  constexpr int XTT = XT == GEMV_PREQ ? MLLM_HIP_BF16 : XT;
  u32x4 plo[RW][2], phi[RW][2];
  float pd[RW][2];
  int pn[RW][2];
  const int nitems = mnb * 4, valid = a.M * nb * 4;
  constexpr int NPRE = 4;  // activation items a thread requests at a time (the first batch ahead of the weights)
  XRaw<XTT> raw[NPRE];
  if (XT == GEMV_PREQ) {
#pragma unroll
    for (int r = 0; r < RW; r++)
#pragma unroll
      for (int k = 0; k < 2; k++) {
        const int m = wave + r * nwaves, b = lane + 64 * k;
        const int it = min(m, MT - 1) * nb + min(b, nb - 1);
        plo[r][k] = img_lo[it]; phi[r][k] = img_hi[it]; pd[r][k] = img_d[it]; pn[r][k] = img_n8[it];
      }
  } else {
#pragma unroll
    for (int k = 0; k < NPRE; k++) load_x8<XTT>(a.x, (int64_t)min(tid + k * nthreads, valid - 1) * 8, raw[k]);
  }

  // ---- 2. weight scales of the tile and slice: 16-byte pieces of eight ----------------------------------------------------
  const WRsrc wr = make_wrsrc(pt.w, WT, N, nb, nbp);
  const int cps = nbs >> 3;  // pieces per row and slice
  u32x4 sc[2];
#pragma unroll
  for (int k = 0; k < 2; k++) {
    const int ch = lane + 64 * k;
    const int r = ch / cps, cc = ch - r * cps;
    const bool ok = tile_ok && r < 16 && row0 + r < N && b0 + 8 * cc < nbp;
    sc[k] = __builtin_amdgcn_raw_buffer_load_b128(wr.d, ok ? (uint32_t)(((int64_t)(row0 + r) * nbp + b0 + 8 * cc) * 2) : BUF_OOB, 0, BUF_NT);
  }
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // ---- 3. weight codes: lane (row c, group g) takes blocks b0 + 4 j + g, j = 0 .. MF_NG - 1 ---------------------------------
  const int c = lane & 15, g = lane >> 4;
  const bool row_ok = tile_ok && row0 + c < N;
  const uint32_t rbase = (uint32_t)(row0 + c) * (uint32_t)nb;
  u32x4 wq[MF_NG][WT == MLLM_HIP_Q8_0 ? 2 : 1];
  auto load_groups = [&](int bb) {
#pragma unroll
    for (int j = 0; j < MF_NG; j++) {
      const int b = bb + 4 * j + g;
      const uint32_t off = (row_ok && b < b1) ? (rbase + (uint32_t)b) * 16u : BUF_OOB;
      wq[j][0] = __builtin_amdgcn_raw_buffer_load_b128(wr.q0, off, 0, BUF_NT);
      if (WT == MLLM_HIP_Q8_0) wq[j][WT == MLLM_HIP_Q8_0 ? 1 : 0] = __builtin_amdgcn_raw_buffer_load_b128(wr.q1, off, 0, BUF_NT);
    }
  };
  load_groups(b0);
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // ---- 4. activations into LDS ---------------------------------------------------------------------------------------------
  if (XT == GEMV_PREQ) {
#pragma unroll
    for (int r = 0; r < RW; r++)
#pragma unroll
      for (int k = 0; k < 2; k++) {
        const int m = wave + r * nwaves, b = lane + 64 * k;
        if (m < MT && b < nb) {
          xlo[(size_t)m * rs + b] = plo[r][k];
          xhi[(size_t)m * rs + b] = phi[r][k];
          xs[(size_t)m * nb + b] = u32x2{__float_as_uint(pd[r][k]), (uint32_t)pn[r][k]};
        }
      }
    for (int m = wave; m < MT; m += nwaves)  // rows longer than 128 blocks, rows beyond the first RW of this wave
      for (int b = lane; b < nb; b += 64) {
        if (b < 128 && m < wave + RW * nwaves) continue;
        const int it = m * nb + b;
        xlo[(size_t)m * rs + b] = img_lo[it];
        xhi[(size_t)m * rs + b] = img_hi[it];
        xs[(size_t)m * nb + b] = u32x2{__float_as_uint(img_d[it]), (uint32_t)img_n8[it]};
      }
  } else {
    const float inv_nb = 1.0f / (float)nb;
    auto put = [&](int it, const XRaw<XTT>& rw) {  // whole quads: nitems is a multiple of 4
      float v[8];
      x8_to_f32<XTT>(rw, v);
      if (it >= valid) {
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = 0.f;
      }
      uint32_t pk[2];
      float deff;
      int n8;
      quad_quantize(v, a.x86_scale, pk, deff, n8);
      const int blk = it >> 2, j = it & 3;  // block index over m * nb + b; lane j holds elements 8j .. 8j+7
      const int m = (int)(((float)blk + 0.5f) * inv_nb), b = blk - m * nb;  // blk / nb: below 2^12, far from rounding trouble
      u32x2* dst = reinterpret_cast<u32x2*>((j < 2 ? xlo : xhi) + (size_t)m * rs + b) + (j & 1);
      *dst = u32x2{pk[0], pk[1]};
      if (j == 0) xs[(size_t)m * nb + b] = u32x2{__float_as_uint(deff), (uint32_t)n8};
    };
#pragma unroll
    for (int k = 0; k < NPRE; k++)
      if (tid + k * nthreads < nitems) put(tid + k * nthreads, raw[k]);
    for (int base = tid + NPRE * nthreads; base < nitems; base += NPRE * nthreads) {  // whole quads stay together: nthreads % 4 == 0
#pragma unroll
      for (int k = 0; k < NPRE; k++) load_x8<XTT>(a.x, (int64_t)min(base + k * nthreads, valid - 1) * 8, raw[k]);
#pragma unroll
      for (int k = 0; k < NPRE; k++)
        if (base + k * nthreads < nitems) put(base + k * nthreads, raw[k]);
    }
  }
  for (int i = tid; i < nb + TRIP; i += nthreads) zrow[i] = u32x4{0u, 0u, 0u, 0u};
  for (int i = tid; i < TRIP; i += nthreads) {  // slack behind the last row
    xhi[(size_t)MT * rs + i] = u32x4{0u, 0u, 0u, 0u};
    xs[(size_t)MT * nb + i] = u32x2{0u, 0u};
  }
  // weight scales -> fp32 [block of the slice][row]; blocks past the row and the rest of the last trip are zero
#pragma unroll
  for (int k = 0; k < 2; k++) {
    const int ch = lane + 64 * k;
    const int r = ch / cps, cc = ch - r * cps;
    if (r < 16) {
      const uint32_t wds[4] = {sc[k].x, sc[k].y, sc[k].z, sc[k].w};
#pragma unroll
      for (int e = 0; e < 8; e++)
        ws[(8 * cc + e) * 16 + r] = (b0 + 8 * cc + e < nb) ? f16bits_to_f32((uint16_t)(wds[e >> 1] >> (16 * (e & 1)))) : 0.f;
    }
  }
  for (int i = nbs * 16 + lane; i < wsb * 16; i += 64) ws[i] = 0.f;
  __syncthreads();

  // ---- 5. block sums on the matrix cores, scaling on the vector ALU ----------------------------------------------------------
  // Software-pipelined over groups of four blocks: the operands of group j + 1 are requested and the instructions of group j
  // issued before the scaling of group j - 1 runs.  No branches inside a trip: blocks past the slice have zero codes
  // (out-of-range loads) and zero weight scales, and their activation scale is replaced by zero.
  const int q = (lane & 15) >> 2, tt = lane & 3;  // this lane's column: block 4j + q, activation row 4h + tt
  const bool mine = g == q;                      // the lane group that supplies this column's activation codes
  f32x4 acc[TH];
#pragma unroll
  for (int h = 0; h < TH; h++) acc[h] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int bb = b0; bb < b1; bb += TRIP) {
    if (bb != b0) load_groups(bb);
    const u32x4* xl[TH];
    const u32x4* xh[TH];
    const u32x2* xsl[TH];
#pragma unroll
    for (int h = 0; h < TH; h++) {
      xl[h] = mine ? xlo + (size_t)(4 * h + tt) * rs + bb + q : zrow + bb + q;
      xh[h] = mine ? xhi + (size_t)(4 * h + tt) * rs + bb + q : zrow + bb + q;
      xsl[h] = xs + (size_t)(4 * h + tt) * nb + bb + q;
    }
    const float* ws_l = ws + (bb - b0 + q) * 16 + 4 * g;
    u32x4 Bl[2][TH], Bh[2][TH];
    u32x2 sx[2][TH];
    f32x4 dw[2];
    v4i_t D[2][TH];
    auto fetch_b = [&](int set, int j) {
#pragma unroll
      for (int h = 0; h < TH; h++) {
        Bl[set][h] = xl[h][4 * j];
        Bh[set][h] = xh[h][4 * j];
      }
    };
    auto fetch_s = [&](int set, int j) {
#pragma unroll
      for (int h = 0; h < TH; h++) sx[set][h] = xsl[h][4 * j];
      dw[set] = *reinterpret_cast<const f32x4*>(ws_l + 4 * j * 16);
    };
    auto issue = [&](int set, int j) {
      v4i_t Al, Ah;
      if (WT == MLLM_HIP_Q4_0) {
        const u32x4 w = wq[j][0];
        Al = v4i_t{(int)(w.x & 0x0f0f0f0fu), (int)(w.y & 0x0f0f0f0fu), (int)(w.z & 0x0f0f0f0fu), (int)(w.w & 0x0f0f0f0fu)};
        Ah = v4i_t{(int)((w.x >> 4) & 0x0f0f0f0fu), (int)((w.y >> 4) & 0x0f0f0f0fu), (int)((w.z >> 4) & 0x0f0f0f0fu),
                   (int)((w.w >> 4) & 0x0f0f0f0fu)};
      } else {
        Al = __builtin_bit_cast(v4i_t, wq[j][0]);
        Ah = __builtin_bit_cast(v4i_t, wq[j][WT == MLLM_HIP_Q8_0 ? 1 : 0]);
      }
#pragma unroll
      for (int h = 0; h < TH; h++) {
        v4i_t d = __builtin_amdgcn_mfma_i32_16x16x64_i8(Al, __builtin_bit_cast(v4i_t, Bl[set][h]), v4i_t{0, 0, 0, 0}, 0, 0, 0);
        D[set][h] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Ah, __builtin_bit_cast(v4i_t, Bh[set][h]), d, 0, 0, 0);
      }
    };
    auto scale = [&](int set, int j) {
      const bool live = bb + 4 * j + q < b1;
#pragma unroll
      for (int h = 0; h < TH; h++) {
        const float dx = live ? __uint_as_float(sx[set][h].x) : 0.f;
        const int n8 = WT == MLLM_HIP_Q4_0 ? (int)sx[set][h].y : 0;  // nibbles are unsigned: sum((q - 8) x) = sum(q x) - 8 sum(x)
        acc[h].x = fmaf(dw[set].x * dx, (float)(D[set][h].x + n8), acc[h].x);
        acc[h].y = fmaf(dw[set].y * dx, (float)(D[set][h].y + n8), acc[h].y);
        acc[h].z = fmaf(dw[set].z * dx, (float)(D[set][h].z + n8), acc[h].z);
        acc[h].w = fmaf(dw[set].w * dx, (float)(D[set][h].w + n8), acc[h].w);
      }
    };
    fetch_b(0, 0);
#pragma unroll
    for (int j = 0; j < MF_NG; j++) {
      issue(j & 1, j);
      if (j + 1 < MF_NG) fetch_b((j + 1) & 1, j + 1);
      fetch_s(j & 1, j);
      __builtin_amdgcn_sched_barrier(0);
      if (j > 0) scale((j - 1) & 1, j - 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    scale((MF_NG - 1) & 1, MF_NG - 1);
  }
  // the four lanes of an activation row (blocks = 0, 1, 2, 3 mod 4): (0 + 1) + (2 + 3) on every lane
#pragma unroll
  for (int h = 0; h < TH; h++) {
    float v[4] = {acc[h].x, acc[h].y, acc[h].z, acc[h].w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
      v[e] += __shfl_xor(v[e], 4, 64);
      v[e] += __shfl_xor(v[e], 8, 64);
    }
    acc[h] = f32x4{v[0], v[1], v[2], v[3]};
  }

  // ---- 6. slices of a tile in slice order; bias, residual; PAIR: silu(gate) * up and its Q8_0 image ------------------------------
  if (S > 1 || PAIR) {
#pragma unroll
    for (int h = 0; h < TH; h++) red[h * 64 + lane] = acc[h];
    __syncthreads();
    if (slice == 0 && (!PAIR || pidx == 0)) {
      for (int s = 1; s < S; s++)
#pragma unroll
        for (int h = 0; h < TH; h++) {
          const f32x4 o = red[(size_t)s * TH * 64 + h * 64 + lane];
          acc[h].x += o.x; acc[h].y += o.y; acc[h].z += o.z; acc[h].w += o.w;
        }
    }
    if (!PAIR && slice != 0) return;
  }
  const int n = row0 + 4 * g;
  if constexpr (!PAIR) {
    if (!tile_ok || q != 0) return;
#pragma unroll
    for (int h = 0; h < TH; h++) {
      const int t = 4 * h + tt;
      if (t >= a.M) continue;
      const float v[4] = {acc[h].x, acc[h].y, acc[h].z, acc[h].w};
      float* yrow = pt.y + (int64_t)t * N;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if (n + e < N) {
          float o = v[e];
          if (pt.bias) o = pt.bias[n + e] + o;
          if (pt.residual) o = o + pt.residual[(int64_t)t * N + n + e];
          yrow[n + e] = o;
        }
      }
    }
  } else {
    // the gate wave of slice 0 adds up the up projection's slices (the S waves after its own S), forms h for its 16 channels and
    // puts it into LDS [MT][16 * tiles_wg] (over the activation codes: every wave is past them after the barrier above);
    // then one quad per (32-channel block, activation row) quantizes
    float* s_h = reinterpret_cast<float*>(smem);
    const int hw = 16 * tiles_wg;
    if (slice == 0 && pidx == 0 && q == 0) {
#pragma unroll
      for (int h = 0; h < TH; h++) {
        f32x4 u = red[(size_t)S * TH * 64 + h * 64 + lane];
        for (int s = 1; s < S; s++) {
          const f32x4 o = red[(size_t)(S + s) * TH * 64 + h * 64 + lane];
          u.x += o.x; u.y += o.y; u.z += o.z; u.w += o.w;
        }
        const int t = 4 * h + tt;
        const float gv[4] = {acc[h].x, acc[h].y, acc[h].z, acc[h].w};
        const float uv[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const bool ok = tile_ok && n + e < N && t < a.M;
          const float x = gv[e];
          const float hv = ok ? x * (1.0f / (1.0f + (mo.exp_accurate ? expf(-x) : exp_poly(-x)))) * uv[e] : 0.f;
          s_h[t * hw + tile_l * 16 + 4 * g + e] = hv;
          if (ok && mo.h) mo.h[(int64_t)t * N + n + e] = hv;
        }
      }
    }
    if (!mo.image) return;  // uniform
    __syncthreads();
    const int quads = MT * (tiles_wg / 2);
    if (tid < 4 * quads) {
      const int qd = tid >> 2, j = tid & 3;
      const int m = qd % MT, blk = qd / MT;  // 32-channel block within this workgroup
      const int gblk = ((int)blockIdx.x * tiles_wg) / 2 + blk;
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = s_h[m * hw + blk * 32 + 8 * j + i];
      if (gblk < N / QK) quad_quantize_to_image(v, QImage{mo.image, MT, N / QK, a.x86_scale}, m, gblk, j, true);
    }
  }
}

// bytes of LDS of a launch with `nwaves` waves per workgroup
template <int MT>
static size_t mf_lds_bytes(int nb, int nbs, int nwaves) {
  const int rs = mf_row_stride(nb), trip = 4 * MF_NG;
  const int wsb = (nbs + trip - 1) / trip * trip;
  return ((size_t)2 * MT * rs + trip + nb + trip) * 16 + ((size_t)MT * nb + trip) * 8 + (size_t)nwaves * wsb * 64 +
         (size_t)nwaves * (MT / 4) * 1024;
}

static int mf_slices(int nb) {
  int s = 1;
  while (s < 8 && nb > 40 * s) s *= 2;
  return s;
}

}  // namespace mllmhip
