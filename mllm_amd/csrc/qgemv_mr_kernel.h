// Q4_0 / Q8_0 Linear for nine to a few dozen activation rows ("many rows" next to the decode kernels' one to eight): the
// weights are read ONCE for up to 32 rows of activations.
//
// The reference serves any number of rows with one tile kernel (llamafile_sgemm.cpp:588-695, mnpack; arithmetic :697-743:
// exact int32 block sums, acc = fma(fp32(dW * dX), float(isum), acc)).  The decode kernels of this library handle eight rows per
// pass (qgemv_mfk_kernel.h) and keep the blocks of an instruction apart with a block-diagonal activation operand; with more
// rows that form re-reads the weights and re-quantizes per group of eight.  Here one v_mfma_i32_16x16x32_i8 is exactly one
// block: K = 32, 16 weight rows against 16 activation rows, so a block's 16 x 16 sums come out of one instruction and
// a lane scales four of them: fma(dW[row] * dX[m], float(isum), acc) with its own accumulator per (weight row, activation
// row) -- no sums across lanes at all, every lane adds the blocks of its outputs in block order.
//
// Work split as in the K-slice decode kernel: a workgroup = `nwaves` row tiles of 16 weight rows x ONE K slice (at most 64
// blocks; whole rows of up to 128 blocks where the row tiles alone fill the chip) x one group of 16 AG activation rows; slices meet in memory (partial sums, arrival counter, the last one adds
// them in slice order); several activation-row groups are further workgroups of the same launch, neighbours on one XCD.
// Activations come as the quantized image a small kernel wrote once for all rows (quant_image_kernel), a workgroup copies
// its rows' slice of it into LDS.  Weight codes stream through the same ring of chunk slots and the same per-wave LDS
// stage as in that kernel (8 rows x 128 contiguous bytes per load instruction).
#pragma once
#include "qgemv_mfk_kernel.h"

namespace mllmhip {

typedef int64_t mr_i64;

struct MrArgs {
  float* part;         // [row groups][S][MT][NP] partial sums (S > 1)
  unsigned* counters;  // one per (workgroup column, row group), zero between launches (S > 1), cstride counters apart
  int cstride;
  int NP;              // columns of a partial row: every part's rows rounded up to 16
  int S, nbs;          // K slices; blocks per slice (a multiple of 8, at most MR_MAX_NBS)
  int col0[GEMV_MAX_PARTS];
  int gx, groups;      // workgroup columns; activation-row groups of MT rows
  int rows_img;        // rows of the image (groups * MT; rows past a.M are zero)
  int nbs_magic;       // ceil(2^20 / nbs): item / nbs as a multiply and a shift
};

// LDS row strides that keep the sixteen activation rows of one operand read on different banks: code planes in 16-byte units
// = 1 mod 16 (sixteen rows x 16 bytes cover the 64 banks once), scale records in 8-byte units = 1 mod 16
__host__ __device__ inline int mr_code_stride(int nbs) { return nbs + ((1 - nbs % 16) + 16) % 16; }
__host__ __device__ inline int mr_rec_stride(int nbs) { return nbs + ((1 - nbs % 16) + 16) % 16; }
constexpr int MR_MAX_NBS = 128;  // blocks per slice (weight scales of a slice: four 16-byte loads per lane)

template <int AG>
static size_t mr_lds_bytes(int wtype, int nbs, int nwaves) {
  const int rs = mr_code_stride(nbs), rx = mr_rec_stride(nbs), MT = 16 * AG;
  return (size_t)2 * MT * rs * 16 + (size_t)MT * rx * 8 + (size_t)nwaves * ((size_t)nbs * 64 + (size_t)MFK_STG * 16 * (wtype == MLLM_HIP_Q8_0 ? 2 : 1)) + 16;
}

// blockDim = 64 x (row tiles per workgroup); the threads number at least MT nbs / 8 (eight image items per thread at most).
// AG: groups of 16 activation rows per workgroup (1 or 2).
template <int WT, int AG>
__global__ __launch_bounds__(512) void gemv_mr_kernel(GemvArgs a, MrArgs k) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int MT = 16 * AG;
  constexpr int NPL = WT == MLLM_HIP_Q8_0 ? 2 : 1;
  const int nb = a.nb, nbp = a.nbp, nbs = k.nbs, S = k.S;
  const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // work item = (workgroup column bx, K slice, row group rg): a 1-D grid in which the row groups of one (column, slice) are
  // neighbours ON ONE XCD (workgroup L runs on XCD L % 8): they read the same weights at about the same time
  const int L = blockIdx.x, seq = L >> 3;
  const int rg = seq % k.groups;
  const int item = (seq / k.groups) * 8 + (L & 7);
  if (item >= k.gx * S) return;
  const int gx = k.gx;
  const int slice = item / gx, bx = item - slice * gx;
  int pidx = 0;
#pragma unroll
  for (int p = 1; p < GEMV_MAX_PARTS; p++)
    if (p < a.nparts && bx >= a.wg_start[p]) pidx = p;
  const GemvPart& pt = a.part[pidx];
  const int wg0 = a.wg_start[pidx], pcol0 = k.col0[pidx];
  const int N = pt.N, kNP = k.NP;
  const int m0 = rg * MT;                       // first activation row of this group
  const int aM = min(a.M - m0, MT);             // its valid rows (the image is zero past a.M)
  float* const kpart = k.part + (size_t)rg * S * MT * kNP;
  unsigned* const kcnt = k.counters + (size_t)rg * gx * k.cstride;
  float* const ybase = pt.y + (int64_t)m0 * N;
  const float* const rbase = pt.residual ? pt.residual + (int64_t)m0 * N : nullptr;
  const int tile = (bx - wg0) * nwaves + wave;
  const int row0 = tile * 16;
  const bool tile_ok = row0 < N;
  const int b0 = slice * nbs, b1 = min(nb, b0 + nbs);

  const int rs = mr_code_stride(nbs), rx = mr_rec_stride(nbs);
  u32x4* xlo = reinterpret_cast<u32x4*>(smem);           // [MT][rs] codes of elements 0..15 of (row, block of the slice)
  u32x4* xhi = xlo + (size_t)MT * rs;                    // likewise elements 16..31
  u32x2* xs = reinterpret_cast<u32x2*>(xhi + (size_t)MT * rs);  // [MT][rx] {effective scale, -8 * sum of the codes (Q8_0: 0)}
  float* ws_all = reinterpret_cast<float*>(xs + (size_t)MT * rx);
  float* ws = ws_all + (size_t)wave * nbs * 16;          // per wave [block][16 rows]
  u32x4* stg_all = reinterpret_cast<u32x4*>(ws_all + (size_t)nwaves * nbs * 16);
  u32x4* stg = stg_all + (size_t)wave * MFK_STG * NPL;
  int* s_flag = reinterpret_cast<int*>(stg_all + (size_t)nwaves * MFK_STG * NPL);

  // ---- 1. this group's rows of the image, the slice's blocks: requested first (they come from the caches and are needed first) ------
  // item it = tid + i * blockDim = (row it / nbs, block it % nbs of the slice); addresses clamped, validity applied at the store
  constexpr int NIMG = 8;
  const int nitems = MT * nbs;
  const int mnb = k.rows_img * nb;
  const u32x4* img_lo = reinterpret_cast<const u32x4*>(a.x);
  const u32x4* img_hi = img_lo + mnb;
  const float* img_d = reinterpret_cast<const float*>(img_hi + mnb);
  const int* img_n8 = reinterpret_cast<const int*>(img_d + mnb);
  u32x4 plo[NIMG], phi[NIMG];
  float pd[NIMG];
  int pn[NIMG];
#pragma unroll
  for (int i = 0; i < NIMG; i++) {
    if (i * nthreads < nitems) {  // uniform
      const int it = min(tid + i * nthreads, nitems - 1);
      const int m = (int)(((uint32_t)it * (uint32_t)k.nbs_magic) >> 20), ib = it - m * nbs;
      const int src = min(m0 + m, k.rows_img - 1) * nb + min(b0 + ib, nb - 1);
      plo[i] = img_lo[src]; phi[i] = img_hi[src]; pd[i] = img_d[src]; pn[i] = img_n8[src];
    }
  }
  // ---- 2. weight scales of the tile and slice (16-byte pieces of eight blocks, a row's pieces on neighbouring lanes) -------
  // (slices of up to 64 blocks: 8 pieces per row, two loads; longer ones: 16 pieces per row, four loads)
  const WRsrc wr = make_wrsrc(pt.w, WT, N, nb, nbp);
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
  // ---- 3. weight codes: the ring's first turn (chunk = 8 blocks; instruction i of it = rows 8 i .. 8 i + 7, 128 bytes of each) ----
  const int lr = lane >> 3, lp = lane & 7;
  u32x4 wq[MR_CH][2][NPL];
  auto load_chunk = [&](int ch, int cb) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int r = row0 + 8 * i + lr, b = cb + lp;
      const uint32_t off = (tile_ok && r < N && b < b1) ? ((uint32_t)r * (uint32_t)nb + (uint32_t)b) * 16u : BUF_OOB;
      wq[ch][i][0] = __builtin_amdgcn_raw_buffer_load_b128(wr.q0, off, 0, BUF_NT);
      if (WT == MLLM_HIP_Q8_0) wq[ch][i][NPL - 1] = __builtin_amdgcn_raw_buffer_load_b128(wr.q1, off, 0, BUF_NT);
    }
  };
  load_chunk(0, b0);  // (the other chunks of the ring: behind the image copy, see below)
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // ---- 4. the image items into LDS (rows past the image and blocks past the row: zeros) -----------------------------------------
#pragma unroll
  for (int i = 0; i < NIMG; i++) {
    const int it = tid + i * nthreads;
    if (i * nthreads < nitems && it < nitems) {
      const int m = (int)(((uint32_t)it * (uint32_t)k.nbs_magic) >> 20), ib = it - m * nbs;
      const bool live = b0 + ib < nb && m0 + m < k.rows_img;
      xlo[(size_t)m * rs + ib] = live ? plo[i] : u32x4{0u, 0u, 0u, 0u};
      xhi[(size_t)m * rs + ib] = live ? phi[i] : u32x4{0u, 0u, 0u, 0u};
      const int n8 = (live && WT == MLLM_HIP_Q4_0) ? pn[i] : 0;
      xs[(size_t)m * rx + ib] = u32x2{live ? __float_as_uint(pd[i]) : 0u, (uint32_t)n8};
    }
  }
#pragma unroll
  for (int ch = 1; ch < MR_CH; ch++) load_chunk(ch, b0 + 8 * ch);
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
        ws[(8 * cc + e) * 16 + r] = (b0 + 8 * cc + e < nb) ? f16bits_to_f32((uint16_t)(wds[e >> 1] >> (16 * (e & 1)))) : 0.f;
    }
  }
  __syncthreads();

  // ---- 5. one instruction per block and group of 16 activation rows ---------------------------------------------------------
  // operand layout of v_mfma_i32_16x16x32_i8: lane l supplies eight K elements 8 (l / 16) .. 8 (l / 16) + 7 of weight row (first
  // operand) or activation row (second operand) l % 16; result: lane l holds weight rows 4 (l / 16) + 0..3 of activation row l % 16
  const int c = lane & 15, g = lane >> 4;
  const int half = g & 1, plane = g >> 1;  // a block's 32 elements: plane 0 = elements 0..15 (Q4_0: low nibbles), plane 1 = 16..31
  f32x4 acc[AG];
#pragma unroll
  for (int h = 0; h < AG; h++) acc[h] = f32x4{0.f, 0.f, 0.f, 0.f};
  const unsigned char* xplane = reinterpret_cast<const unsigned char*>(plane ? xhi : xlo) + 8 * half;
  const int we = tile_ok ? b1 : b0;
  const int b1r = b0 + (max(we - b0, 0) + 7) / 8 * 8;
  auto chunk = [&](const int ch, const int cb, const bool refill) {
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int p = 0; p < NPL; p++) stg[p * MFK_STG + (8 * i + lr) * 9 + lp] = wq[ch][i][p];
    if (refill) load_chunk(ch, cb + (8 * MR_CH));
#pragma unroll
    for (int jb = 0; jb < 8; jb++) {
      const int lb = cb - b0 + jb;  // block within the slice (inside the slice's LDS rows even when past the row: zero scales)
      // weight operand: this lane's eight elements of (row c, block): bytes 8 half .. of the 16-byte record (Q8_0: of plane `plane`)
      const unsigned char* sp = reinterpret_cast<const unsigned char*>(stg + (WT == MLLM_HIP_Q8_0 ? plane * MFK_STG : 0) + c * 9 + jb) + 8 * half;
      u32x2 wv = *reinterpret_cast<const u32x2*>(sp);
      if (WT == MLLM_HIP_Q4_0) {
        const int sh = 4 * plane;
        wv = u32x2{(wv.x >> sh) & 0x0f0f0f0fu, (wv.y >> sh) & 0x0f0f0f0fu};
      }
      const f32x4 dw = *reinterpret_cast<const f32x4*>(ws + lb * 16 + 4 * g);
      const mr_i64 A = __builtin_bit_cast(mr_i64, wv);
#pragma unroll
      for (int h = 0; h < AG; h++) {
        const int m = 16 * h + c;
        const u32x2 xv = *reinterpret_cast<const u32x2*>(xplane + ((size_t)m * rs + lb) * 16);
        const u32x2 sx = xs[(size_t)m * rx + lb];
        const int n8 = (int)sx.y;  // nibbles are unsigned: sum((q - 8) x) = sum(q x) - 8 sum(x)
        const v4i_t D = __builtin_amdgcn_mfma_i32_16x16x32_i8(A, __builtin_bit_cast(mr_i64, xv), v4i_t{n8, n8, n8, n8}, 0, 0, 0);
        const float dx = __uint_as_float(sx.x);
        acc[h].x = fmaf(dw.x * dx, (float)D.x, acc[h].x);
        acc[h].y = fmaf(dw.y * dx, (float)D.y, acc[h].y);
        acc[h].z = fmaf(dw.z * dx, (float)D.z, acc[h].z);
        acc[h].w = fmaf(dw.w * dx, (float)D.w, acc[h].w);
      }
    }
  };
  int cb0 = b0;
  for (; cb0 + (8 * MR_CH) <= b1r; cb0 += (8 * MR_CH)) {
#pragma unroll
    for (int ch = 0; ch < MR_CH; ch++) chunk(ch, cb0 + 8 * ch, true);
  }
#pragma unroll
  for (int ch = 0; ch < MR_CH - 1; ch++)
    if (cb0 + 8 * ch < we) chunk(ch, cb0 + 8 * ch, false);  // uniform

  // lane: activation rows 16 h + c, weight rows n .. n + 3
  const int n = row0 + 4 * g;
  if (S == 1) {
    if (!tile_ok) return;
    const bool vec = (N & 3) == 0 && ((reinterpret_cast<uintptr_t>(ybase) | reinterpret_cast<uintptr_t>(pt.bias) |
                                       reinterpret_cast<uintptr_t>(rbase)) & 15) == 0;  // uniform
#pragma unroll
    for (int h = 0; h < AG; h++) {
      const int t = 16 * h + c;
      if (t >= aM) continue;
      if (vec) {
        if (n >= N) continue;
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
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if (n + e < N) {
          float o = v[e];
          if (pt.bias) o = pt.bias[n + e] + o;
          if (rbase) o = o + rbase[(int64_t)t * N + n + e];
          ybase[(int64_t)t * N + n + e] = o;
        }
      }
    }
    return;
  }

  // ---- 6. the slices of a tile meet in global memory (the protocol of the K-slice decode kernel) ---------------------------------
  //   (a) partial sums leave with device-scope stores; (b) every wave waits until all its stores are acknowledged; (c) workgroup
  //   barrier; (d) thread 0 counts the workgroup in with a device-scope atomic add; (e) the workgroup that sees the last count tells
  //   its waves through LDS and a barrier; (f) they read the partial sums with device-scope loads issued after that barrier.
  const int col = pcol0 + n;
  if (tile_ok) {
#pragma unroll
    for (int h = 0; h < AG; h++) {
      float* dst = kpart + ((size_t)slice * MT + 16 * h + c) * kNP + col;
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
    if (last) __hip_atomic_store(kcnt + bx * k.cstride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    *s_flag = last;
  }
  __syncthreads();  // (e)
  if (!*s_flag || !tile_ok) return;
  // the last workgroup: lane l of a wave sums outputs (activation row l / 16 + 4 i, weight row l % 16) of its tile over the
  // slices, slice 0 first.  Every load of up to eight slices of ALL its activation rows is requested before the first sum (a
  // load from another chip-let's stores takes about a microsecond: one round trip, not one per row)
  const int r = lane & 15;
  constexpr int NI = MT / 4;
  const size_t sstride = (size_t)MT * kNP;
  float sum[NI];
#pragma unroll
  for (int i = 0; i < NI; i++) sum[i] = 0.f;
  for (int s0 = 0; s0 < S; s0 += 8) {
    float pv[NI][8];
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const float* src = kpart + (size_t)((lane >> 4) + 4 * i) * kNP + pcol0 + row0 + r;
#pragma unroll
      for (int u = 0; u < 8; u++)
        pv[i][u] = __hip_atomic_load(src + (size_t)min(s0 + u, S - 1) * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
      for (int u = 0; u < 8; u++) {
        if (s0 + u == 0) sum[i] = pv[i][0];
        else if (s0 + u < S) sum[i] += pv[i][u];
      }
  }
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int t = (lane >> 4) + 4 * i;
    if (t < aM && row0 + r < N) {
      float o = sum[i];
      if (pt.bias) o = pt.bias[row0 + r] + o;
      if (rbase) o = o + rbase[(int64_t)t * N + row0 + r];
      ybase[(int64_t)t * N + row0 + r] = o;
    }
  }
}

}  // namespace mllmhip
