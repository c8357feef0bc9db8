// Q4_0 / Q8_0 decode GEMV kernel (M = 1..8) for gfx950 and its per-(weight type, activation type) launcher.
//
// Arithmetic follows the reference's x86 CPU path:
//   activation quantization  mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.cpp:106-190
//   block dot + scaling       mllm/backends/cpu/kernels/common/llamafile/llamafile_sgemm.cpp:697-743
// The int32 block sums are exact; the fp32 accumulation order differs from the CPU's 8-lane order.
//
// The kernel is HBM-bound.  A launch streams N*K/32 blocks of 18 (Q4_0) or 34 (Q8_0) algorithmic bytes exactly once,
// with 16-byte loads that are contiguous across the lanes of a group.  For matrices of a few MB the run time is
// dominated by latencies, so the kernel is organised around the ORDER in which memory requests are issued (vector
// memory returns in order): activations first, block scales second, then as many weight codes as the registers
// hold; all arithmetic that does not need the weights runs while they are in flight.
#pragma once
#include "qcommon.h"

namespace mllmhip {

// One launch serves up to four weight matrices that share the activations and K (sibling projections: q/k/v, gate/up):
// workgroups [wg_start[p], wg_start[p+1]) belong to part p.
constexpr int GEMV_MAX_PARTS = 4;
struct GemvPart {
  PackedView w;
  const float* bias;
  const float* residual;  // fp32 [M][N] added to the result (may be y itself), or null
  float* y;
  int N;
};
struct GemvArgs {
  GemvPart part[GEMV_MAX_PARTS];
  int wg_start[GEMV_MAX_PARTS + 1];
  int nparts;
  const void* x;
  int M;          // actual rows of x (<= MT)
  int nb;         // K / 32
  int nbp;        // scale row stride (nb rounded up to 8)
  int x86_scale;  // reproduce the x86 storage rounding of the activation scale
};
extern int g_gemv_defer;  // the deferred form of the one- and two-row kernel: -1 by the launch's size (default); 0 / 1: never / always (comparison runs)
struct GemvShape {
  int G, R, NW;  // lanes per weight row, rows per lane group, waves per workgroup
};

// exact int32 dot product of one weight block with one quantized activation block
template <int WT>
__device__ __forceinline__ int block_dot(const u32x4& w0, const u32x4& w1, const u32x4& xlo, const u32x4& xhi, int neg8sum) {
  if (WT == MLLM_HIP_Q4_0) {
    // dword j of the block: low nibbles = elements 4j..4j+3, high nibbles = elements 16+4j..16+4j+3.
    // nibbles stay unsigned (0..15); the -8 offset is folded in as -8 * sum(x codes), precomputed per activation block.
    const uint32_t m = 0x0f0f0f0fu;
    int acc = neg8sum;
    acc = __builtin_amdgcn_sdot4((int)(w0.x & m), (int)xlo.x, acc, false);
    acc = __builtin_amdgcn_sdot4((int)(w0.y & m), (int)xlo.y, acc, false);
    acc = __builtin_amdgcn_sdot4((int)(w0.z & m), (int)xlo.z, acc, false);
    acc = __builtin_amdgcn_sdot4((int)(w0.w & m), (int)xlo.w, acc, false);
    acc = __builtin_amdgcn_sdot4((int)((w0.x >> 4) & m), (int)xhi.x, acc, false);
    acc = __builtin_amdgcn_sdot4((int)((w0.y >> 4) & m), (int)xhi.y, acc, false);
    acc = __builtin_amdgcn_sdot4((int)((w0.z >> 4) & m), (int)xhi.z, acc, false);
    acc = __builtin_amdgcn_sdot4((int)((w0.w >> 4) & m), (int)xhi.w, acc, false);
    return acc;
  } else {
    int acc = 0;
    acc = __builtin_amdgcn_sdot4((int)w0.x, (int)xlo.x, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w0.y, (int)xlo.y, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w0.z, (int)xlo.z, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w0.w, (int)xlo.w, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w1.x, (int)xhi.x, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w1.y, (int)xhi.y, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w1.z, (int)xhi.z, acc, false);
    acc = __builtin_amdgcn_sdot4((int)w1.w, (int)xhi.w, acc, false);
    return acc;
  }
}

// One loop trip's worth of weight data of a lane: U block columns x R rows.
template <int WT, int R, int U, bool SCL>
struct WChunk {
  u32x4 w0[U][R];
  u32x4 w1[WT == MLLM_HIP_Q8_0 ? U : 1][R];
  uint16_t dw[SCL ? 1 : U][R];  // block scales, only when they are not staged through LDS
};

// Weight loads go through buffer descriptors: a lane whose block column lies past the end of the row (or whose row lies
// past N) gets an out-of-range offset, which returns zeros without touching memory and without a branch, so the
// number of loads in flight is the same on every path and the wait counters stay exact.
struct WRsrc {
  __amdgpu_buffer_rsrc_t q0, q1, d;
};
#define BUF_OOB 0xffffffffu
#define BUF_NT 2  // streamed once: non-temporal
__device__ __forceinline__ WRsrc make_wrsrc(const PackedView& w, int wtype, int64_t N, int nb, int nbp) {
  const uint32_t blocks = (uint32_t)(N * nb);
  WRsrc r;
  r.q0 = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(w.q0), 0, blocks * 16u, 0x00020000);
  r.q1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(wtype == MLLM_HIP_Q8_0 ? w.q1 : w.q0), 0, blocks * 16u, 0x00020000);
  r.d = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(w.d), 0, (uint32_t)(N * nbp) * 2u, 0x00020000);
  return r;
}

template <int WT, int G, int R, int U, bool SCL, int ULO = 0, int UHI = U>
__device__ __forceinline__ void load_chunk(WChunk<WT, R, U, SCL>& c, const WRsrc& w, const uint32_t (&rbase)[R],
                                           const uint32_t (&dbase)[R], int t0, int c0, int nb) {
#pragma unroll
  for (int u = ULO; u < UHI; u++) {
    const int col = t0 + u * G + c0;
#pragma unroll
    for (int r = 0; r < R; r++) {
      const bool ok = col < nb && rbase[r] != BUF_OOB;
      const uint32_t blk = rbase[r] + (uint32_t)col;
      c.w0[u][r] = __builtin_amdgcn_raw_buffer_load_b128(w.q0, ok ? blk * 16u : BUF_OOB, 0, BUF_NT);
      if (WT == MLLM_HIP_Q8_0) c.w1[u][r] = __builtin_amdgcn_raw_buffer_load_b128(w.q1, ok ? blk * 16u : BUF_OOB, 0, BUF_NT);
      if (!SCL) c.dw[u][r] = __builtin_amdgcn_raw_buffer_load_b16(w.d, ok ? (dbase[r] + (uint32_t)col) * 2u : BUF_OOB, 0, BUF_NT);
    }
  }
}

// XT == GEMV_PREQ: `x` is not the activations but their quantized image, laid out exactly like the kernel's LDS area
// (code planes, scales, -8*sums; rows m >= M zero), written once by quant_image_kernel; the kernel copies it instead of
// quantizing.  With several activation rows the quantization, which every workgroup would repeat, costs more than the
// weights take to arrive.
constexpr int GEMV_PREQ = 2;

// Eight consecutive activation elements of one lane, raw (bf16: 16 bytes, fp32: 32 bytes) and converted.
template <int XT>
struct XRaw {
  u32x4 r[XT == MLLM_HIP_F32 ? 2 : 1];
};
template <int XT>
__device__ __forceinline__ void load_x8(const void* x, int64_t elem, XRaw<XT>& raw) {
  if (XT == MLLM_HIP_F32) {
    const u32x4* p = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(x) + elem);
    raw.r[0] = p[0];
    raw.r[XT == MLLM_HIP_F32 ? 1 : 0] = p[1];
  } else {
    raw.r[0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(x) + elem);
  }
}
template <int XT>
__device__ __forceinline__ void x8_to_f32(const XRaw<XT>& raw, float (&v)[8]) {
  if (XT == MLLM_HIP_F32) {
    const u32x4 a = raw.r[0], b = raw.r[XT == MLLM_HIP_F32 ? 1 : 0];
    v[0] = __uint_as_float(a.x); v[1] = __uint_as_float(a.y); v[2] = __uint_as_float(a.z); v[3] = __uint_as_float(a.w);
    v[4] = __uint_as_float(b.x); v[5] = __uint_as_float(b.y); v[6] = __uint_as_float(b.z); v[7] = __uint_as_float(b.w);
  } else {  // bf16 -> fp32 is exact
    const uint32_t w[4] = {raw.r[0].x, raw.r[0].y, raw.r[0].z, raw.r[0].w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      v[2 * j + 0] = __uint_as_float(w[j] << 16);
      v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}

// Workgroup = NW waves.  Each wave is cut into 64/G groups of G lanes; a group owns R consecutive weight rows and its
// lanes stride over the row's blocks (lane c takes blocks c, c+G, ...), so one load instruction of a group reads G*16
// contiguous bytes.
// All of x is quantized once per workgroup into LDS, four lanes per 32-element block (quad reductions with DPP): codes
// in two 16-byte planes so that neighbouring lanes later read neighbouring 16-byte words, plus the fp32 scale and
// -8*sum(codes) per block.
// SCL: the fp16 scales of the wave's rows are fetched with (at most two) 16-byte loads per lane and handed out through
// LDS instead of one 2-byte load per block.
// U = how many block columns a lane keeps in flight per loop trip; later trips are double-buffered.
// Register budget: with four or eight activation rows the accumulators and the weights in flight need 140..215
// registers; the kernels are therefore built for at most eight waves per workgroup (under a 1024-thread bound the
// compiler has 128 and spills 40..330 bytes per lane).  For one or two rows 16 waves stay possible (long rows).
template <int WT, int XT, int MT, int G, int R, int U, bool SCL, bool DEFER = false>
__global__ __launch_bounds__(MT <= 2 ? 1024 : 512) void gemv_q_kernel(GemvArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int nb = a.nb, nbp = a.nbp;
  int pidx = 0;  // uniform: which matrix this workgroup works on
#pragma unroll
  for (int p = 1; p < GEMV_MAX_PARTS; p++)
    if (p < a.nparts && (int)blockIdx.x >= a.wg_start[p]) pidx = p;
  const GemvPart& pt = a.part[pidx];
  const int bid = blockIdx.x - a.wg_start[pidx];
  const int N = pt.N;
  const int mnb = MT * nb;
  u32x4* s_lo = reinterpret_cast<u32x4*>(smem);
  u32x4* s_hi = s_lo + mnb;
  float* s_d = reinterpret_cast<float*>(s_hi + mnb);
  int* s_n8 = reinterpret_cast<int*>(s_d + mnb);

  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int nwaves = nthreads >> 6;
  constexpr int GROUPS = 64 / G;
  constexpr int ROWS_W = GROUPS * R;  // weight rows of one wave
  const int grp = lane / G;
  const int c0 = lane % G;
  const int64_t wrow0 = ((int64_t)bid * nwaves + wave) * ROWS_W;
  const int64_t row0 = wrow0 + (int64_t)grp * R;
  uint16_t* s_ws = reinterpret_cast<uint16_t*>(smem + align_up((size_t)mnb * 40, 16)) + (size_t)wave * ROWS_W * nbp;

  // ---- 1. activation loads (two quantization items per thread are requested up front) -------------------------
  // item `it` = eight elements: block it/4, lanes of a quad share a block.  Addresses are clamped, validity is applied
  // when the values are used, so no branch separates these loads from the ones below.
  const int valid_items = a.M * nb * 4;
  const int img_chunks = (mnb * 5 + 1) / 2;  // 16-byte pieces of the quantized image (40 bytes per block; the buffer is sized for 8 rows)
  // (NPRE items per thread are requested here; an item requested in the quantization loop below comes back behind the
  // weights and costs a round trip to memory of its own.  Two rows of 2560 elements are 2.5 items per thread of a 256-thread
  // workgroup: with four requested here the step of the 4B layers at two rows goes 0.958 -> 0.876 ms.  One row keeps two:
  // a third -- used by rows of more than 4096 elements -- made the 4B step 1.5 % slower and 2 x 25600 x 5120 2 % slower.)
  constexpr int NPRE = MT == 1 ? 2 : 4;
  XRaw<XT> raw[NPRE];
#pragma unroll
  for (int i = 0; i < NPRE; i++) {
    if (i >= 2 && i * nthreads >= (XT == GEMV_PREQ ? img_chunks : mnb * 4)) break;  // uniform: nothing left for a third / fourth item
    if (XT == GEMV_PREQ) raw[i].r[0] = reinterpret_cast<const u32x4*>(a.x)[min(tid + i * nthreads, img_chunks - 1)];
    else load_x8<XT>(a.x, (int64_t)min(tid + i * nthreads, valid_items - 1) * 8, raw[i]);
  }

  // ---- 2. block scales of this wave's rows: chunks of 8 scales (16 bytes), lane L takes chunks L and L+64 ------
  const WRsrc wr = make_wrsrc(pt.w, WT, N, nb, nbp);
  const int cpr = nbp >> 3;  // chunks per row
  u32x4 sc[2];
  if (SCL) {
#pragma unroll
    for (int k = 0; k < 2; k++) {
      const int ch = lane + 64 * k;
      const int rw = ch / cpr, cc = ch - rw * cpr;
      const bool ok = rw < ROWS_W && wrow0 + rw < N;
      sc[k] = __builtin_amdgcn_raw_buffer_load_b128(wr.d, ok ? (uint32_t)(((wrow0 + rw) * nbp + cc * 8) * 2) : BUF_OOB, 0, BUF_NT);
    }
  }
  __asm__ volatile("" ::: "memory");  // keep the loads above ahead of the weight loads
  __builtin_amdgcn_sched_barrier(0);

  // ---- 3. first trip of weight loads ------------------------------------------------------------------------------
  // first block of each of the lane group's rows; rows past N load nothing and are dropped at the store
  uint32_t rbase[R], dbase[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    rbase[r] = (row0 + r < N) ? (uint32_t)((row0 + r) * nb) : BUF_OOB;
    dbase[r] = (uint32_t)((row0 + r) * nbp);
  }
  WChunk<WT, R, U, SCL> cur;
  // One or two rows: only the first block column of the trip is requested here, the others behind the quantization of x.
  // Every workgroup of a launch starts within a microsecond and needs its activations first; what all of them ask for at
  // that moment is in the way of exactly those answers (the step of the 4B layers: 0.698 -> 0.686 ms at one row, 0.981 ->
  // 0.960 at two; nothing here: 0.745; the others right after the activations have arrived: 0.697; behind the barrier: 0.729).
  constexpr int UFIRST = DEFER ? 1 : U;
  load_chunk<WT, G, R, U, SCL, 0, UFIRST>(cur, wr, rbase, dbase, 0, c0, nb);
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  // ---- 4. activation quantization into LDS (rows m >= M are zero-filled so the unrolled MT loop is harmless) -------
  auto quantize_item = [&](int it, const XRaw<XT>& rw) {
    const int id = it >> 2, j = it & 3;
    float v[8];
    x8_to_f32<XT>(rw, v);
    const bool valid = it < valid_items;
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      v[e] = valid ? v[e] : 0.f;
      amax = fmaxf(amax, fabsf(v[e]));
    }
    amax = fmaxf(amax, dpp_f<0xB1>(amax));  // over the quad that shares the block
    amax = fmaxf(amax, dpp_f<0x4E>(amax));
    const float d = amax / 127.f;
    const float idv = (amax != 0.f) ? 127.f / amax : 0.f;
    const uint32_t pk[2] = {q8_pack4(&v[0], idv), q8_pack4(&v[4], idv)};
    int sum = __builtin_amdgcn_sdot4((int)pk[0], 0x01010101, 0, false);
    sum = __builtin_amdgcn_sdot4((int)pk[1], 0x01010101, sum, false);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xf, 0xf, true);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xf, 0xf, true);
    if (it < mnb * 4) {
      uint2* dst = reinterpret_cast<uint2*>((j < 2 ? s_lo : s_hi) + id) + (j & 1);
      *dst = make_uint2(pk[0], pk[1]);
      if (j == 0) {
        uint16_t bits = f32_to_f16bits(d);
        if (a.x86_scale) bits = x86_scale_bits(bits);
        s_d[id] = f16bits_to_f32(bits);
        s_n8[id] = -8 * sum;
      }
    }
  };
  if (XT == GEMV_PREQ) {
    u32x4* s16 = reinterpret_cast<u32x4*>(smem);
#pragma unroll
    for (int i = 0; i < NPRE; i++)
      if (tid + i * nthreads < img_chunks) s16[tid + i * nthreads] = raw[i].r[0];
    for (int c = tid + NPRE * nthreads; c < img_chunks; c += nthreads) s16[c] = reinterpret_cast<const u32x4*>(a.x)[c];
  } else {
    quantize_item(tid, raw[0]);
    quantize_item(tid + nthreads, raw[1]);
#pragma unroll
    for (int i = 2; i < NPRE; i++)
      if ((i * nthreads) < mnb * 4) quantize_item(tid + i * nthreads, raw[i]);  // uniform
    for (int it = tid + NPRE * nthreads; it < mnb * 4; it += nthreads) {
      XRaw<XT> rw;
      load_x8<XT>(a.x, (int64_t)min(it, valid_items - 1) * 8, rw);
      quantize_item(it, rw);
    }
  }
  if (SCL) {
#pragma unroll
    for (int k = 0; k < 2; k++) {
      const int ch = lane + 64 * k;
      if (ch < ROWS_W * cpr) *reinterpret_cast<u32x4*>(s_ws + ch * 8) = sc[k];
    }
  }
  // the rest of the first trip's weights (see UFIRST above)
  load_chunk<WT, G, R, U, SCL, UFIRST, U>(cur, wr, rbase, dbase, 0, c0, nb);  // the rest of the first trip's weights (DEFER)
  __syncthreads();

  // ---- 5. block dots ------------------------------------------------------------------------------------------------
  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < MT; m++) acc[r][m] = 0.f;

  for (int t0 = 0; t0 < nb; t0 += G * U) {
    WChunk<WT, R, U, SCL> nxt;
    const bool more = t0 + G * U < nb;  // uniform
    if (more) load_chunk<WT, G, R, U, SCL>(nxt, wr, rbase, dbase, t0 + G * U, c0, nb);
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = t0 + u * G + c0;
      if (col < nb) {
        float dwf[R];
#pragma unroll
        for (int r = 0; r < R; r++)
          dwf[r] = f16bits_to_f32(SCL ? s_ws[(grp * R + r) * nbp + col] : cur.dw[SCL ? 0 : u][r]);
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const u32x4 xlo = s_lo[m * nb + col];
          const u32x4 xhi = s_hi[m * nb + col];
          const float dx = s_d[m * nb + col];
          const int n8 = s_n8[m * nb + col];
#pragma unroll
          for (int r = 0; r < R; r++) {
            const int isum = block_dot<WT>(cur.w0[u][r], cur.w1[WT == MLLM_HIP_Q8_0 ? u : 0][r], xlo, xhi, n8);
            acc[r][m] = fmaf(dwf[r] * dx, (float)isum, acc[r][m]);
          }
        }
      }
    }
    if (more) cur = nxt;
  }

#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < MT; m++) {
      float v = group_sum<G>(acc[r][m]);
      const int64_t row = row0 + r;
      if (c0 == 0 && row < N && m < a.M) {
        // Linear first (bias + dot), then the residual: the order of the two operators it replaces
        if (pt.bias) v = pt.bias[row] + v;
        if (pt.residual) v = v + pt.residual[(int64_t)m * N + row];
        pt.y[(int64_t)m * N + row] = v;
      }
    }
}

// ---- launchers ---------------------------------------------------------------------------------------------------
// U3: three block columns in flight instead of four.  Rows of up to 96 blocks (K = 2560: 80) are covered by one trip either
// way, and with three the kernel fits five waves per SIMD (81 registers instead of 97): 1280 resident workgroups, so the
// 1216 workgroups of the gate + up launch run in one round instead of 1024 + 192.
template <int WT, int XT, int MT, int G, int R, bool U3 = false>
static int launch_gemv_u(const GemvArgs& a_in, int NW, hipStream_t st) {
  constexpr int U0 = ((R >= 4) ? 1 : (R == 2 ? 2 : 4)) * (WT == MLLM_HIP_Q4_0 ? 2 : 1);
  constexpr int U = (U3 && U0 == 4) ? 3 : U0;
  constexpr int ROWS_W = (64 / G) * R;
  if (MT > 2 && NW > 8) NW = 8;  // see the register budget note at the kernel
  const int rows_per_wg = NW * ROWS_W;
  GemvArgs a = a_in;
  unsigned grid = 0;
  for (int p = 0; p < a.nparts; p++) {
    a.wg_start[p] = (int)grid;
    grid += (unsigned)((a.part[p].N + rows_per_wg - 1) / rows_per_wg);
  }
  a.wg_start[a.nparts] = (int)grid;
  const bool scl = ROWS_W * (a.nbp / 8) <= 128;
  const size_t lds = align_up((size_t)MT * a.nb * 40, 16) + (scl ? (size_t)NW * ROWS_W * a.nbp * 2 : 0);
  if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
  auto launch = [&](auto kern) -> int {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, st, a);
    return (int)hipGetLastError();
  };
  if constexpr (MT <= 2 && U >= 2) {
    // Measured per shape (us per launch, all at once -> deferred, one row, Q4_0): 1024 x 2560 3.23 -> 3.39, 2560 x 4096 3.61 -> 3.93,
    // 4096 x 2560 3.50 -> 3.68, 6144 x 2048 3.57 -> 3.90, 8192 x 2048 3.82 -> 4.08, q+k+v 6144 x 2560 4.15 -> 3.93, 9728 x 2560
    // 5.19 -> 4.68, 2560 x 9728 5.20 -> 4.80, gate + up 7.00 -> 6.92, 2 x 25600 x 5120 27.7 -> 26.9; Q8_0 wins from q+k+v
    // (15.9 MB) on.  So: launches of 8 MB (Q8_0: 14 MB) and more with rows of 80 blocks and more.
    int64_t blocks = 0;
    for (int p = 0; p < a.nparts; p++) blocks += (int64_t)a.part[p].N * a.nb;
    // (two rows: every shape with rows of 80 blocks and more wins, 2560 x 4096 5.50 -> 5.22, 4096 x 2560 4.75 -> 4.42)
    const bool big = a.nb >= 80 && (MT == 2 || blocks * (WT == MLLM_HIP_Q4_0 ? 18 : 34) >= (int64_t)(WT == MLLM_HIP_Q4_0 ? 8 : 14) << 20);
    if (g_gemv_defer < 0 ? big : g_gemv_defer != 0)
      return scl ? launch(gemv_q_kernel<WT, XT, MT, G, R, U, true, true>) : launch(gemv_q_kernel<WT, XT, MT, G, R, U, false, true>);
  }
  return scl ? launch(gemv_q_kernel<WT, XT, MT, G, R, U, true>) : launch(gemv_q_kernel<WT, XT, MT, G, R, U, false>);
}

// rows per lane group that are compiled for each activation-row tile: wider tiles reuse every LDS read for more rows
template <int MT> struct RowsFor;
template <> struct RowsFor<1> { static constexpr int lo = 1, hi = 2; };
template <> struct RowsFor<2> { static constexpr int lo = 1, hi = 2; };
template <> struct RowsFor<4> { static constexpr int lo = 2, hi = 4; };
template <> struct RowsFor<8> { static constexpr int lo = 2, hi = 4; };

template <int WT, int XT, int MT>
static int launch_gemv_m(const GemvArgs& a, GemvShape s, hipStream_t st) {
  constexpr int RL = RowsFor<MT>::lo, RH = RowsFor<MT>::hi;
#define CASE(G_)                                                                     \
  if (s.G == G_ && s.R == RL) return launch_gemv_u<WT, XT, MT, G_, RL>(a, s.NW, st); \
  if (s.G == G_ && s.R == RH) return launch_gemv_u<WT, XT, MT, G_, RH>(a, s.NW, st);
  if constexpr (WT == MLLM_HIP_Q4_0 && MT <= 2 && RH == 2) {
    if (s.G == 32 && s.R == 2 && a.nb <= 96) return launch_gemv_u<WT, XT, MT, 32, 2, true>(a, s.NW, st);
  }
  CASE(8) CASE(16) CASE(32) CASE(64)
#undef CASE
  return MLLM_HIP_E_BADARG;
}

// one instance per (weight type, activation type), each in its own translation unit (compiled in parallel)
template <int WT, int XT>
int launch_gemv(const GemvArgs& a, int MT, GemvShape s, hipStream_t st) {
  {
    switch (MT) {
      case 1: return launch_gemv_m<WT, XT, 1>(a, s, st);
      case 2: return launch_gemv_m<WT, XT, 2>(a, s, st);
      case 4: return launch_gemv_m<WT, XT, 4>(a, s, st);
      default: return launch_gemv_m<WT, XT, 8>(a, s, st);
    }
  }
}
// three to eight rows on the matrix cores (qgemv_mfma.hip); x_kind: MLLM_HIP_F32, MLLM_HIP_BF16 or GEMV_PREQ; MT: 4 or 8;
// waves per workgroup: 0 (by x_kind), 4 or 8; K slices per row tile: 0 (by row length), 1, 2 or 4 (sweeps)
int launch_gemv_mfma(int wtype, int x_kind, int MT, const GemvArgs& a, int waves, int slices, hipStream_t st);
bool gemv_mfma_fits(int MT, int nb);  // rows of nb blocks fit that kernel's LDS
// The matrix-core kernel with the K slices as separate workgroups.  image_ws: where a raw x could be quantized first (unused
// so far); part / part_bytes: room for the slices' partial sums (may be null / 0).  Returns MFK_NOT_TAKEN when the launch
// does not fit (no room for the partial sums, no counter block to be had under stream capture, slices too long): the caller
// takes another kernel.
constexpr int MFK_NOT_TAKEN = 1;
int launch_gemv_mfk(int wtype, int x_kind, int MT, const GemvArgs& a, const void* workspace, void* part, size_t part_bytes, int waves,
                    int slices, hipStream_t st, int groups = 1);
int gemv_mfk_slices(int nb);
// nine rows and more: the many-row kernel (qgemv_mr.hip).  a.x = the quantized image of gemv_mr_image_rows(a.M) rows; MFK_NOT_TAKEN
// where it does not fit (room for partial sums, counters)
int gemv_mr_image_rows(int M);
int gemv_mr_prepare_device();  // kernel attributes of the current device (mllm_hip_init)
size_t gemv_mr_part_bytes(int M, int nb, int64_t n_total_padded);
int launch_gemv_mr(int wtype, const GemvArgs& a, const void* workspace, void* part, size_t part_bytes, int waves, int slices, hipStream_t st,
                   bool dry = false);
int gemv_mfk_prepare_device();                 // counter table and kernel attributes of the current device (mllm_hip_init)
int gemv_mfk_release(const void* workspace);   // the workspace address gives its counter block back
void gemv_mfk_stats(int device, int* owned, int* capacity, long long* recycles, long long* refused);
int launch_gemv_q4_f32(const GemvArgs& a, int MT, GemvShape s, hipStream_t st);
int launch_gemv_q4_bf16(const GemvArgs& a, int MT, GemvShape s, hipStream_t st);
int launch_gemv_q8_f32(const GemvArgs& a, int MT, GemvShape s, hipStream_t st);
int launch_gemv_q8_bf16(const GemvArgs& a, int MT, GemvShape s, hipStream_t st);
int launch_gemv_q4_preq(const GemvArgs& a, int MT, GemvShape s, hipStream_t st);
int launch_gemv_q8_preq(const GemvArgs& a, int MT, GemvShape s, hipStream_t st);

}  // namespace mllmhip
