// Q4_0 / Q8_0 decode GEMV for three to eight activation rows (and groups of such rows) on the matrix cores, K cut into slices that are separate
// WORKGROUPS (qgemv_mfma_kernel.h keeps the slices of a row tile inside one workgroup).
//
// Same arithmetic and the same order of additions as that kernel (block sums with v_mfma_i32_16x16x64_i8, one fused
// multiply-add per block into the lane that owns blocks = q mod 4, the four lanes as (0 + 1) + (2 + 3), then the slices
// in slice order), so both give the same bits.  What differs is who does which part:
//   * a workgroup holds `nwaves` row tiles of 16 weight rows and ONE K slice (rows that are cut: at most 64 blocks).  It
//     quantizes (or copies from the quantized image) only its slice of the activations: with eight rows of 9728 elements
//     that is 320 blocks per workgroup instead of 2432, and the LDS footprint no longer grows with K;
//   * a launch with enough row tiles to fill the chip by themselves keeps rows of up to 128 blocks whole (one slice, no
//     partial sums): the workgroup then sums the row in the chains the slices would have been and adds them in slice order;
//   * weight codes stream through a ring of chunk slots per wave (mfk_ring): a slot is requested again as soon as its chunk has
//     been staged, so a slice of any length keeps that many chunks of loads ahead of the arithmetic;
//   * weight codes are requested as 8 rows x 128 contiguous bytes per load instruction (the operand layout of the MFMA,
//     16 rows x 64 bytes per instruction, measured 25 % slower on the 4B shapes) and turned into the operand layout
//     through a 2 KB LDS stage that belongs to the wave (no barrier: LDS operations of one wave execute in order);
//   * the slices of a row tile meet in global memory: every workgroup stores its partial sums, the one that arrives last
//     at the tile's counter adds them up in slice order, applies bias / residual and stores y.  The counter goes back to
//     zero, so the counters are zero between launches;
//   * more than eight activation rows: groups of eight rows are further workgroups of the same launch (template parameter
//     GR), each with its own rows of x and y, partial sums and counters; the groups of a (workgroup column, slice) item are
//     neighbours on one XCD and read the same weights.
#pragma once
#include "qgemv_mfma_kernel.h"

namespace mllmhip {

// chunks of 8 blocks in flight per wave (a trip = one turn of the ring).  Measured on the 4B decode shapes (ms per step of 36
// layers at 3 / 4 / 8 rows, one row group; at 16 rows, two groups): four slots 0.999 / 1.001 / 1.280 and 1.765, three
// 0.972 / 0.975 / 1.264 and 1.773, two 0.979 / 0.984 / 1.297 and 1.746 (six and more were slower before that): what a launch
// asks for at its start delays the activations that every workgroup needs first.
// (Q8_0, two planes of codes per chunk: 1.265 / 1.509 -> 1.214 / 1.433 at four / eight rows with three slots, 2.075 -> 1.875 at 16
// rows with two; Q4_0 with several row groups is no faster with fewer than four.)
constexpr int mfk_ring(int wtype, bool groups) { return groups ? (wtype == MLLM_HIP_Q8_0 ? 2 : 4) : 3; }
constexpr int MR_CH = 2;  // the many-row kernel (qgemv_mr_kernel.h)
constexpr int MFK_STG = 16 * 9;       // 16-byte pieces of one stage: 16 rows, stride 9 (reads of 16 rows hit 16 bank groups)
constexpr int MFK_MAX_NBS = 128;      // blocks per slice (weight scales of a slice: four 16-byte loads per lane)

// Quantization of sixteen elements (half a block) by one lane of a pair; lanes 2 b and 2 b + 1 share block b.  The same
// operations on the same values as quad_quantize (maximum of 32 magnitudes, the two IEEE divisions, v * id rounded to
// nearest even, integer sums): same codes, same scale, half as many instructions per element.  `ok` false = an element past
// the row or a row past M: zeros (v then holds finite or non-finite values of the last valid row, whose codes a scale of
// zero multiplies away).
__device__ __forceinline__ void pair_quantize(const float (&v)[16], bool ok, int x86, u32x4& codes, float& deff, int& n8) {
  float amax = 0.f;
#pragma unroll
  for (int e = 0; e < 16; e++) amax = fmaxf(amax, fabsf(v[e]));
  amax = ok ? amax : 0.f;  // with amax = 0 the inverse scale is 0 and every code comes out 0, whatever v holds
  amax = fmaxf(amax, dpp_f<0xB1>(amax));
  float d, idv;
  q8_scales(amax, d, idv);
  codes = u32x4{q8_pack4(&v[0], idv), q8_pack4(&v[4], idv), q8_pack4(&v[8], idv), q8_pack4(&v[12], idv)};
  int sum = __builtin_amdgcn_sdot4((int)codes.x, 0x01010101, 0, false);
  sum = __builtin_amdgcn_sdot4((int)codes.y, 0x01010101, sum, false);
  sum = __builtin_amdgcn_sdot4((int)codes.z, 0x01010101, sum, false);
  sum = __builtin_amdgcn_sdot4((int)codes.w, 0x01010101, sum, false);
  sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xf, 0xf, true);
  uint16_t bits = f32_to_f16bits(d);
  if (x86) bits = x86_scale_bits(bits);
  deff = f16bits_to_f32(bits);
  n8 = -8 * sum;
}

struct MfkArgs {
  float* part;         // [row groups][S][MT][NP] partial sums (S > 1)
  unsigned* counters;  // one per (workgroup column, row group), zero between launches (S > 1)
  int NP;              // columns of a partial row: every part's rows rounded up to 16
  int S, nbs;          // K slices; blocks per slice (a multiple of 8, at most MFK_MAX_NBS)
  int vs;              // blocks per summation chain (a multiple of 8): S > 1: nbs; S == 1: the length the slices would have
                       // had -- the chains of a whole row are added in slice order, so the bits do not depend on S
  int col0[GEMV_MAX_PARTS];  // first column of each part within a partial row
  int gx, groups;            // groups > 1 (row groups of eight): a 1-D grid over (workgroup column < gx, slice, group), see the kernel
  int ipr_magic;             // ceil(2^20 / (2 nbs)): item / (items per row) as a multiply and a shift
  int cstride;               // counters from column to column: up to 32 (a cache line each) where the block has room, so that
                             // the arrivals of different columns do not queue on one line
};

// A wave's table of weight scales in LDS: fp32 [block of the slice][16 rows], with eight floats of padding after every eight
// blocks.  A lane writes the eight scales of one 16-byte piece (blocks 8 cc .. 8 cc + 7 of row r); without the padding the
// pieces of a row lie 128 dwords apart and all lanes of a row hit one bank (8 or 16 lanes per bank and instruction).
__host__ __device__ inline int mfk_ws_index(int lb) { return lb * 16 + (lb >> 3) * 8; }
__host__ __device__ inline int mfk_ws_floats(int nbs) { return nbs * 16 + (nbs + 7) / 8 * 8; }

template <int MT>
static size_t mfk_lds_bytes(int wtype, int nbs, int nwaves) {
  const int rs = mf_row_stride(nbs);
  return ((size_t)2 * MT * rs + nbs) * 16 + (size_t)MT * nbs * 8 +
         (size_t)nwaves * ((size_t)mfk_ws_floats(nbs) * 4 + (size_t)MFK_STG * 16 * (wtype == MLLM_HIP_Q8_0 ? 2 : 1)) + 16;
}

// blockDim = 64 x (row tiles per workgroup): three to eight waves, at least nbs / 16 (the threads hold one pass of
// quantization items per activation row).  Waves beyond the row tiles that only help to quantize were measured: slower
// (gate + up of the 4B layer at eight rows 11.6 -> 12.2 us with ten waves instead of five).
template <int WT, int XT, int MT, bool GR = false>  // GR: several row groups in the launch
__global__ __launch_bounds__(512) void gemv_mfk_kernel(GemvArgs a, MfkArgs k) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int TH = MT / 4;
  constexpr int NPL = WT == MLLM_HIP_Q8_0 ? 2 : 1;  // code planes
  constexpr int XTT = XT == GEMV_PREQ ? MLLM_HIP_BF16 : XT;
  const int nb = a.nb, nbp = a.nbp, nbs = k.nbs, S = k.S;
  const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Work item = (workgroup column bx, K slice, row group rg).  One row group: the grid is (columns, slices).  Several: a
  // 1-D grid in which the groups of one (column, slice) are neighbours ON ONE XCD (workgroup L runs on XCD L % 8, every XCD
  // has its own L2): they read the same weights at about the same time, so the weights come from memory once.  The grid is
  // padded to whole eights of (column, slice) items; the padding leaves at once.
  int bx = blockIdx.x, slice = blockIdx.y, rg = 0, gx = gridDim.x;
  if (GR) {
    const int L = blockIdx.x, seq = L >> 3;
    rg = seq % k.groups;
    const int item = (seq / k.groups) * 8 + (L & 7);
    if (item >= k.gx * S) return;
    gx = k.gx;
    slice = item / gx;
    bx = item - slice * gx;
  }
  int pidx = 0;  // uniform: which matrix this workgroup works on
#pragma unroll
  for (int p = 1; p < GEMV_MAX_PARTS; p++)
    if (p < a.nparts && bx >= a.wg_start[p]) pidx = p;
  const GemvPart& pt = a.part[pidx];
  const int wg0 = a.wg_start[pidx], pcol0 = k.col0[pidx];
  // rg: group of MT activation rows (raw activations; an image is always one group).  A group has its own rows of x and y,
  // its own partial sums and counters, and reads the same weights as its siblings.
  const void* const xptr =
      XT == GEMV_PREQ ? a.x : static_cast<const void*>(reinterpret_cast<const char*>(a.x) + (size_t)rg * MT * nb * QK * (XT == MLLM_HIP_F32 ? 4 : 2));
  const int aM = GR ? min(a.M - rg * MT, MT) : a.M, x86 = a.x86_scale;
  const int kNP = k.NP;
  float* const kpart = k.part + (size_t)rg * S * MT * kNP;
  unsigned* const kcnt = k.counters + (size_t)rg * gx * k.cstride;  // (column bx: kcnt[bx * k.cstride])
  const int N = pt.N;
  float* const ybase = pt.y + (int64_t)rg * MT * N;
  const float* const rbase = pt.residual ? pt.residual + (int64_t)rg * MT * N : nullptr;
  const int tile = (bx - wg0) * nwaves + wave;
  const int row0 = tile * 16;
  const bool tile_ok = row0 < N;
  const int b0 = slice * nbs, b1 = min(nb, b0 + nbs);  // this workgroup's blocks (possibly none: b1 <= b0)

  const int rs = mf_row_stride(nbs);
  u32x4* xlo = reinterpret_cast<u32x4*>(smem);  // [MT][rs] codes of elements 0..15 of (row, block of the slice)
  u32x4* xhi = xlo + (size_t)MT * rs;           // likewise elements 16..31
  u32x4* zrow = xhi + (size_t)MT * rs;          // [nbs] zeros: the operand of the lane groups that must not contribute
  u32x2* xs = reinterpret_cast<u32x2*>(zrow + nbs);  // [MT][nbs] {effective scale, -8 * sum of the codes (Q8_0: 0)}
  float* ws_all = reinterpret_cast<float*>(xs + (size_t)MT * nbs);
  float* ws = ws_all + (size_t)wave * mfk_ws_floats(nbs);  // per wave [block][16 rows], padded: mfk_ws_index
  u32x4* stg_all = reinterpret_cast<u32x4*>(ws_all + (size_t)nwaves * mfk_ws_floats(nbs));
  u32x4* stg = stg_all + (size_t)wave * MFK_STG * NPL;
  int* s_flag = reinterpret_cast<int*>(stg_all + (size_t)nwaves * MFK_STG * NPL);

  // ---- 1. activation requests (they return first; nothing here divides: the weight requests below must leave early) ------
  // raw activations: item it = tid + i * blockDim = sixteen elements, two neighbouring lanes share a block;
  // image: item it = tid + i * blockDim = (row it / 64, block it % 64) of the slice; slices of more than 64 blocks: 128
  const int ipr = nbs * 2;            // items of sixteen elements (half a block) per row of the slice
  const int nitems = MT * ipr;        // item it: row it / ipr, half block it % ipr (pairs of lanes stay whole: ipr % 2 == 0)
  constexpr int NXP = MT / 2;         // passes: the threads number at least 4 nbs (launcher), so MT * ipr / blockDim <= MT / 2
  XRaw<XTT> raw[NXP][2];
  const int mnb = MT * nb;
  const u32x4* img_lo = reinterpret_cast<const u32x4*>(xptr);
  const u32x4* img_hi = img_lo + mnb;
  const float* img_d = reinterpret_cast<const float*>(img_hi + mnb);
  const int* img_n8 = reinterpret_cast<const int*>(img_d + mnb);
  constexpr int NIMG = MT / 2;  // passes: at least three waves for up to 64 blocks, at least five for up to 128
  const int imsh = nbs > 64 ? 7 : 6, nimg = MT << imsh;  // uniform
  u32x4 plo[NIMG], phi[NIMG];
  float pd[NIMG];
  int pn[NIMG];
  if (XT == GEMV_PREQ) {
#pragma unroll
    for (int i = 0; i < NIMG; i++) {
      if (i * nthreads < nimg) {  // uniform
        const int item = tid + i * nthreads, im = item >> imsh, ib = item & ((1 << imsh) - 1);
        const int it = min(im, MT - 1) * nb + min(b0 + ib, nb - 1);
        plo[i] = img_lo[it]; phi[i] = img_hi[it]; pd[i] = img_d[it]; pn[i] = img_n8[it];
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < NXP; i++) {
      if (i * nthreads < nitems) {  // uniform
        const int it = min(tid + i * nthreads, nitems - 1);
        const int m = (int)(((uint32_t)it * (uint32_t)k.ipr_magic) >> 20), xc = it - m * ipr;
        // clamped addresses: validity is applied when the values are used
        const int64_t e0 = ((int64_t)min(m, aM - 1) * nb * 2 + min(b0 * 2 + xc, nb * 2 - 1)) * 16;
        load_x8<XTT>(xptr, e0, raw[i][0]);
        load_x8<XTT>(xptr, e0 + 8, raw[i][1]);
      }
    }
  }

  // ---- 2. weight scales of the tile and slice: 16-byte pieces of eight blocks, a row's pieces on neighbouring lanes ------
  const WRsrc wr = make_wrsrc(pt.w, WT, N, nb, nbp);
  // (slices of up to 64 blocks: 8 pieces per row, two loads; longer ones: 16 pieces per row, four loads)
  const int nsc = nbs > 64 ? 4 : 2;  // uniform
  u32x4 sc[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (i >= nsc) break;
    const int scsh = nbs > 64 ? 4 : 3;
    const int r = (lane >> scsh) + (64 >> scsh) * i, cc = lane & ((1 << scsh) - 1);
    const bool ok = tile_ok && row0 + r < N && 8 * cc < nbs && b0 + 8 * cc < nbp;
    sc[i] = __builtin_amdgcn_raw_buffer_load_b128(wr.d, ok ? (uint32_t)(((int64_t)(row0 + r) * nbp + b0 + 8 * cc) * 2) : BUF_OOB, 0, BUF_NT);
  }
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // ---- 3. weight codes of a trip: chunk ch = 8 blocks, instruction i of it = rows 8 i .. 8 i + 7, 128 bytes of each --------
  const int lr = lane >> 3, lp = lane & 7;
  constexpr int CH = mfk_ring(WT, GR), TRIP = 8 * CH;
  u32x4 wq[CH][2][NPL];
  auto load_chunk = [&](int ch, int cb) {  // chunk slot ch <- the eight blocks from cb on (nothing is fetched past the slice)
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int r = row0 + 8 * i + lr, b = cb + lp;
      const uint32_t off = (tile_ok && r < N && b < b1) ? ((uint32_t)r * (uint32_t)nb + (uint32_t)b) * 16u : BUF_OOB;
      wq[ch][i][0] = __builtin_amdgcn_raw_buffer_load_b128(wr.q0, off, 0, BUF_NT);
      if (WT == MLLM_HIP_Q8_0) wq[ch][i][NPL - 1] = __builtin_amdgcn_raw_buffer_load_b128(wr.q1, off, 0, BUF_NT);
    }
  };
  // (several row groups: only the first chunk is asked for here, the others of the ring behind the quantization of x -- the
  // step at 16 rows 1.749 -> 1.686 ms; with one row group it changes nothing, 0.971 -> 0.975 at three rows, 1.265 -> 1.266 at eight)
  constexpr int FIRST = GR ? 1 : CH;
#pragma unroll
  for (int ch = 0; ch < FIRST; ch++) load_chunk(ch, b0 + 8 * ch);
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // ---- 4. the slice of the activations into LDS ------------------------------------------------------------------------
  if (XT == GEMV_PREQ) {
#pragma unroll
    for (int i = 0; i < NIMG; i++) {
      const int item = tid + i * nthreads, m = item >> imsh, ib = item & ((1 << imsh) - 1);
      if (i * nthreads < nimg && m < MT && ib < nbs) {
        const bool live = b0 + ib < nb;  // the image has no blocks past the row
        xlo[(size_t)m * rs + ib] = live ? plo[i] : u32x4{0u, 0u, 0u, 0u};
        xhi[(size_t)m * rs + ib] = live ? phi[i] : u32x4{0u, 0u, 0u, 0u};
        const int n8 = (live && WT == MLLM_HIP_Q4_0) ? pn[i] : 0;
        xs[(size_t)m * nbs + ib] = u32x2{live ? __float_as_uint(pd[i]) : 0u, (uint32_t)n8};
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < NXP; i++) {
      const int it = tid + i * nthreads;
      if (it < nitems) {  // whole pairs: nitems and nthreads are even
        const int m = (int)(((uint32_t)it * (uint32_t)k.ipr_magic) >> 20), xc = it - m * ipr;
        float v[16], v1[8];
        {
          float v0[8];
          x8_to_f32<XTT>(raw[i][0], v0);
          x8_to_f32<XTT>(raw[i][1], v1);
#pragma unroll
          for (int e = 0; e < 8; e++) {
            v[e] = v0[e];
            v[8 + e] = v1[e];
          }
        }
        const int b = xc >> 1, j = xc & 1;
        u32x4 codes;
        float deff;
        int n8;
        pair_quantize(v, m < aM && b0 + b < nb, x86, codes, deff, n8);
        (j == 0 ? xlo : xhi)[(size_t)m * rs + b] = codes;
        if (j == 0) {
          if (WT != MLLM_HIP_Q4_0) n8 = 0;  // nibbles are unsigned: sum((q - 8) x) = sum(q x) - 8 sum(x); Q8_0 codes are signed
          xs[(size_t)m * nbs + b] = u32x2{__float_as_uint(deff), (uint32_t)n8};
        }
      }
    }
  }
#pragma unroll
  for (int ch = FIRST; ch < CH; ch++) load_chunk(ch, b0 + 8 * ch);
  for (int i = tid; i < nbs; i += nthreads) zrow[i] = u32x4{0u, 0u, 0u, 0u};
  // weight scales -> fp32 [block of the slice][row]; blocks past the row are zero
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (i >= nsc) break;
    const int scsh = nbs > 64 ? 4 : 3;
    const int r = (lane >> scsh) + (64 >> scsh) * i, cc = lane & ((1 << scsh) - 1);
    if (8 * cc < nbs) {
      const uint32_t wds[4] = {sc[i].x, sc[i].y, sc[i].z, sc[i].w};
#pragma unroll
      for (int e = 0; e < 8; e++)
        ws[mfk_ws_index(8 * cc + e) + r] = (b0 + 8 * cc + e < nb) ? f16bits_to_f32((uint16_t)(wds[e >> 1] >> (16 * (e & 1)))) : 0.f;
    }
  }
  __syncthreads();

  // ---- 5. block sums on the matrix cores, scaling on the vector ALU -----------------------------------------------------------
  // chunk by chunk as the weights arrive: its 8 blocks through the wave's LDS stage into the operand layout, then its two
  // groups of four blocks with all operands requested before the first instruction issues
  const int c = lane & 15, g = lane >> 4;        // operand layout: weight row c, block 4 j + g of a group of four
  const int q = (lane & 15) >> 2, tt = lane & 3;  // this lane's result column: block 4 j + q, activation row 4 h + tt
  const bool mine = g == q;                      // the lane group that supplies this column's activation codes
  f32x4 acc[TH];
#pragma unroll
  for (int h = 0; h < TH; h++) acc[h] = f32x4{0.f, 0.f, 0.f, 0.f};
  // the four lanes of an activation row (lane l + 4 j of a row of 16 lanes: blocks = j mod 4): (0 + 1) + (2 + 3), complete on
  // the lanes with j == 0, the ones that store.  Shifts within the row of 16 on the vector ALU (lane l takes lane l + 4, then
  // l + 8; a shuffle would be an LDS instruction in a loop that keeps LDS reads in flight)
  auto across_lanes = [&]() {
#pragma unroll
    for (int h = 0; h < TH; h++) {
      float v[4] = {acc[h].x, acc[h].y, acc[h].z, acc[h].w};
#pragma unroll
      for (int e = 0; e < 4; e++) {
        v[e] += dpp_f<0x104>(v[e]);  // row_shl:4
        v[e] += dpp_f<0x108>(v[e]);  // row_shl:8
      }
      acc[h] = f32x4{v[0], v[1], v[2], v[3]};
    }
  };
  f32x4 tot[TH];       // sum of the chains that are complete
  bool have_tot = false;
  int chain_end = b0 + k.vs;
  const int we = tile_ok ? b1 : b0;                    // a wave without a row tile has no chunks
  const int b1r = b0 + (max(we - b0, 0) + 7) / 8 * 8;  // the end of the wave's blocks rounded up to whole chunks
  // One chunk: slot ch of the ring holds blocks cb .. cb + 7.  The loop below runs whole trips with nothing conditional
  // between the requests, and the chunks of a last, partial trip follow as straight-line code: the compiler's wait counts have
  // to hold for every path that reaches a wait, and with an exit (or a skipped request) inside the loop body they came out as
  // "wait for all loads" at the head of every trip.
  auto chunk = [&](const int ch, const int cb, const bool refill) {
    if (cb == chain_end) {       // uniform; only whole rows (S == 1) get here
      across_lanes();
#pragma unroll
      for (int h = 0; h < TH; h++) {
        tot[h] = have_tot ? f32x4{tot[h].x + acc[h].x, tot[h].y + acc[h].y, tot[h].z + acc[h].z, tot[h].w + acc[h].w} : acc[h];
        acc[h] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      have_tot = true;
      chain_end += k.vs;
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int p = 0; p < NPL; p++) {
        stg[p * MFK_STG + (8 * i + lr) * 9 + lp] = wq[ch][i][p];
      }
    // the slot is free: the same chunk of the next trip takes it, CH chunks ahead of the arithmetic (past the slice the
    // offsets are out of range and nothing is fetched)
    if (refill) load_chunk(ch, cb + TRIP);
    u32x4 Aw[2][NPL], Bl[2][TH], Bh[2][TH];
    u32x2 sx[2][TH];
    f32x4 dw[2];
#pragma unroll
    for (int jj = 0; jj < 2; jj++) {
      const int lb = cb - b0 + 4 * jj + q;  // this lane's block within the slice (inside the slice's LDS rows even when dead)
#pragma unroll
      for (int p = 0; p < NPL; p++) Aw[jj][p] = stg[p * MFK_STG + c * 9 + 4 * jj + g];
      dw[jj] = *reinterpret_cast<const f32x4*>(ws + mfk_ws_index(lb) + 4 * g);
#pragma unroll
      for (int h = 0; h < TH; h++) {
        const int m = 4 * h + tt;
        // (selecting the address costs less than reading under a lane mask: the branches that takes cut the chunk into
        // pieces the instruction scheduler cannot mix; measured 3 % slower)
        Bl[jj][h] = mine ? xlo[(size_t)m * rs + lb] : zrow[lb];
        Bh[jj][h] = mine ? xhi[(size_t)m * rs + lb] : zrow[lb];
        sx[jj][h] = xs[(size_t)m * nbs + lb];
      }
    }
    v4i_t D[2][TH];
#pragma unroll
    for (int jj = 0; jj < 2; jj++) {
      v4i_t Al, Ah;
      if (WT == MLLM_HIP_Q4_0) {
        const u32x4 w = Aw[jj][0];
        Al = v4i_t{(int)(w.x & 0x0f0f0f0fu), (int)(w.y & 0x0f0f0f0fu), (int)(w.z & 0x0f0f0f0fu), (int)(w.w & 0x0f0f0f0fu)};
        Ah = v4i_t{(int)((w.x >> 4) & 0x0f0f0f0fu), (int)((w.y >> 4) & 0x0f0f0f0fu), (int)((w.z >> 4) & 0x0f0f0f0fu),
                   (int)((w.w >> 4) & 0x0f0f0f0fu)};
      } else {
        Al = __builtin_bit_cast(v4i_t, Aw[jj][0]);
        Ah = __builtin_bit_cast(v4i_t, Aw[jj][NPL - 1]);
      }
#pragma unroll
      for (int h = 0; h < TH; h++) {
        const int n8 = (int)sx[jj][h].y;  // nibbles are unsigned: sum((q - 8) x) = sum(q x) - 8 sum(x)
        const v4i_t d = __builtin_amdgcn_mfma_i32_16x16x64_i8(Al, __builtin_bit_cast(v4i_t, Bl[jj][h]), v4i_t{n8, n8, n8, n8}, 0, 0, 0);
        D[jj][h] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Ah, __builtin_bit_cast(v4i_t, Bh[jj][h]), d, 0, 0, 0);
      }
    }
#pragma unroll
    for (int jj = 0; jj < 2; jj++)
#pragma unroll
      for (int h = 0; h < TH; h++) {
        // blocks past the row carry zero scales on both sides (sections 4), blocks past the slice are never in a chunk
        const float dx = __uint_as_float(sx[jj][h].x);
        acc[h].x = fmaf(dw[jj].x * dx, (float)D[jj][h].x, acc[h].x);
        acc[h].y = fmaf(dw[jj].y * dx, (float)D[jj][h].y, acc[h].y);
        acc[h].z = fmaf(dw[jj].z * dx, (float)D[jj][h].z, acc[h].z);
        acc[h].w = fmaf(dw[jj].w * dx, (float)D[jj][h].w, acc[h].w);
      }
  };
  int cb0 = b0;
  for (; cb0 + TRIP <= b1r; cb0 += TRIP) {
#pragma unroll
    for (int ch = 0; ch < CH; ch++) chunk(ch, cb0 + 8 * ch, true);
  }
#pragma unroll
  for (int ch = 0; ch < CH - 1; ch++)
    if (cb0 + 8 * ch < we) chunk(ch, cb0 + 8 * ch, false);  // uniform
  across_lanes();
  if (have_tot) {
#pragma unroll
    for (int h = 0; h < TH; h++)
      acc[h] = f32x4{tot[h].x + acc[h].x, tot[h].y + acc[h].y, tot[h].z + acc[h].z, tot[h].w + acc[h].w};
  }

  const int n = row0 + 4 * g;  // lanes with q == 0 hold rows n .. n + 3 of activation row 4 h + tt
  if (S == 1) {
    if (!tile_ok || q != 0) return;
    // rows of a multiple of four outputs, 16-byte aligned pointers: 16 bytes per lane, the four lanes of an activation row
    // write one 64-byte line
    const bool vec = (N & 3) == 0 && ((reinterpret_cast<uintptr_t>(ybase) | reinterpret_cast<uintptr_t>(pt.bias) |
                                       reinterpret_cast<uintptr_t>(rbase)) & 15) == 0;  // uniform
#pragma unroll
    for (int h = 0; h < TH; h++) {
      const int t = 4 * h + tt;
      if (t >= aM) continue;
      if (vec) {
        if (n >= N) continue;  // (n and N are multiples of four: n < N means n + 3 < N)
        f32x4 o = acc[h];
        if (pt.bias) {
          const f32x4 bv = *reinterpret_cast<const f32x4*>(pt.bias + n);
          o = f32x4{bv.x + o.x, bv.y + o.y, bv.z + o.z, bv.w + o.w};
        }
        if (rbase) {
          const f32x4 rv = *reinterpret_cast<const f32x4*>(rbase + (int64_t)t * N + n);
          o = f32x4{o.x + rv.x, o.y + rv.y, o.z + rv.z, o.w + rv.w};
        }
        *reinterpret_cast<f32x4*>(ybase + (int64_t)t * N + n) = o;
        continue;
      }
      const float v[4] = {acc[h].x, acc[h].y, acc[h].z, acc[h].w};
      float* yrow = ybase + (int64_t)t * N;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if (n + e < N) {
          float o = v[e];
          if (pt.bias) o = pt.bias[n + e] + o;
          if (rbase) o = o + rbase[(int64_t)t * N + n + e];
          yrow[n + e] = o;
        }
      }
    }
    return;
  }

  // ---- 6. the slices of a tile meet in global memory ------------------------------------------------------------------------------
  // Ordering between workgroups, stated step by step (nothing here is left to what a barrier happens to wait for):
  //   producer  (a) partial sums leave with device-scope stores (written through this chip-let's L2 to where the other
  //                 chip-lets read them);
  //             (b) every wave waits until the memory system has acknowledged all its stores (s_waitcnt vmcnt(0): on this
  //                 chip stores count in vmcnt until they are acknowledged);
  //             (c) the workgroup barrier: all waves have passed (b);
  //             (d) thread 0 counts the workgroup in with a device-scope atomic add.
  //   consumer  (e) thread 0 of the workgroup that sees the last count tells its workgroup through LDS and a barrier;
  //             (f) its waves read the partial sums with device-scope loads, issued after that barrier.
  // A release fence in place of (b) (in every wave, or even one per workgroup) makes the hardware write back this
  // chip-let's whole L2 and cost 5 to 50 us per launch; nothing but these stores has to be visible to the consumer.
  const int col = pcol0 + n;
  if (tile_ok && q == 0) {
#pragma unroll
    for (int h = 0; h < TH; h++) {
      float* dst = kpart + ((size_t)slice * MT + 4 * h + tt) * kNP + col;
      __hip_atomic_store(dst + 0, acc[h].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + 1, acc[h].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + 2, acc[h].z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + 3, acc[h].w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (b)
  __syncthreads();                                       // (c)
  if (tid == 0) {
    const unsigned old = __hip_atomic_fetch_add(kcnt + bx * k.cstride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // (d)
    const int last = old == (unsigned)(S - 1);
    // every slice has arrived: ready for the next launch
    if (last) __hip_atomic_store(kcnt + bx * k.cstride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *s_flag = last;
  }
  __syncthreads();  // (e)
  if (!*s_flag || !tile_ok) return;
  // the workgroup that arrived last: lane l of a wave sums outputs (activation row l / 16 + 4 i, weight row l % 16) of its
  // tile over the slices, slice 0 first; the loads of up to eight slices are in flight together
  const int r = lane & 15;
#pragma unroll
  for (int i = 0; i < TH; i++) {
    const int t = (lane >> 4) + 4 * i;
    const float* src = kpart + (size_t)t * kNP + pcol0 + row0 + r;
    const size_t sstride = (size_t)MT * kNP;
    float sum = 0.f;
    for (int s0 = 0; s0 < S; s0 += 8) {
      float pv[8];
#pragma unroll
      for (int u = 0; u < 8; u++)
        pv[u] = __hip_atomic_load(src + (size_t)min(s0 + u, S - 1) * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int u = 0; u < 8; u++) {
        if (s0 + u == 0) sum = pv[0];
        else if (s0 + u < S) sum += pv[u];
      }
    }
    if (t < aM && row0 + r < N) {
      float o = sum;
      if (pt.bias) o = pt.bias[row0 + r] + o;
      if (rbase) o = o + rbase[(int64_t)t * N + row0 + r];
      ybase[(int64_t)t * N + row0 + r] = o;
    }
  }
}

}  // namespace mllmhip
