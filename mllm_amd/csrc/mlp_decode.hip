// Decode MLP front half in one launch: h = silu(gate(x)) * up(x) for up to eight activation rows, Q4_0 / Q8_0 weights.
//
//   reference: Qwen3MLP::forward, mllm/models/qwen3/modeling_qwen3_fa2.hpp:85-92 -- gate_proj (Linear), SiLU, up_proj
//   (Linear), elementwise product; each Linear = quantize_row_q8_0 + block dots (llamafile_sgemm.cpp:697-743).
//
// The gate row n and the up row n are the two rows of one lane group, so silu(g) * u is formed in the epilogue from two
// registers and g, u never go to memory.  A workgroup owns 32 consecutive channels, which is exactly one Q8_0 block of h:
// it can also write that block of the quantized image the down projection's GEMV reads (MLLM_HIP_Q8_IMAGE), without
// any exchange between workgroups.  x comes as activations (quantized here, once per workgroup) or as the image a
// producer (RMSNorm) wrote.  Same arithmetic as the stand-alone operators: results equal gate/up GEMV -> SiLU -> mul
// (-> quantization) bit for bit when the GEMV sums a row over the same 16 lanes, and agree to rounding otherwise.
#include <type_traits>
#include "qgemv_kernel.h"

namespace mllmhip {

int exp_mode_accurate();  // layer_ops.hip: the setting of mllm_hip_set_exp_mode
// three to eight rows of Q4_0: the matrix-core form (mlp_mfma.hip)
bool mlp_mfma_fits(int MT, int nb);
int launch_mlp_mfma(int x_kind, const PackedView& gate, const PackedView& up, const void* x, float* h, unsigned char* image, int M, int I,
                    int nb, int nbp, int x86_scale, int exp_accurate, hipStream_t st);

__device__ __forceinline__ float silu_sel(float x, int accurate) { return x * (1.0f / (1.0f + (accurate ? expf(-x) : exp_poly(-x)))); }

struct MlpArgs {
  PackedView gate, up;
  const void* x;          // activations [M][H] or their image
  float* h;               // [M][I] fp32 or null
  unsigned char* h_image; // image of h for MT rows or null
  int M, H, I, x86, exp_accurate;
};

// One weight matrix's share of a loop trip of a lane: U block columns.
template <int WT, int U, bool SCL>
struct PairChunk {
  u32x4 w0[U][2];
  u32x4 w1[WT == MLLM_HIP_Q8_0 ? U : 1][2];
  uint16_t dw[SCL ? 1 : U][2];
};

// 32 * G threads = 32 channels: wave w holds 64 / G lane groups, group grp -> channel n = n0 + (64 / G) w + grp; row 0 of
// the group is the gate row, row 1 the up row; lane c0 takes block columns c0, c0 + G, ...; U of them per trip, the next
// trip requested while the current one is multiplied.  Weight loads as in the GEMV kernel: buffer loads, streamed
// (non-temporal), out-of-range columns return zeros without a branch.
// SCL: the fp16 block scales of the wave's rows arrive as 16-byte pieces (one per lane and matrix) and are handed out
// through LDS instead of one 2-byte load per block.
template <int WT, int XT, int MT, int G, int U, bool SCL>
__global__ __launch_bounds__(32 * G) void mlp_gateup_kernel(MlpArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int GROUPS = 64 / G, NTHR = 32 * G;
  const int nb = a.H / QK, nbp = (int)scale_row_stride(a.H);
  const int mnb = MT * nb;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * 32;
  float* s_h = reinterpret_cast<float*>(smem + align_up((size_t)mnb * 40, 16));  // [MT][32]
  uint16_t* s_ws = reinterpret_cast<uint16_t*>(s_h + MT * 32) + (size_t)wave * 2 * GROUPS * nbp;  // [matrix][group][nbp]

  // requests return in order: activations first, then the scales, then the weights
  const int nitems = mnb * 4, valid = a.M * nb * 4;
  const int img_chunks = (mnb * 5 + 1) / 2;
  // (two rows: a second item per thread is requested here too -- one requested in the quantization loop comes back behind
  // the weights)
  constexpr int NPRE = MT == 1 ? 1 : 2;
  XRaw<XT> raw, raw2;
  if (XT == GEMV_PREQ) raw.r[0] = reinterpret_cast<const u32x4*>(a.x)[min(tid, img_chunks - 1)];
  else load_x8<XT>(a.x, (int64_t)min(tid, valid - 1) * 8, raw);
  if (NPRE > 1) {
    if (XT == GEMV_PREQ) raw2.r[0] = reinterpret_cast<const u32x4*>(a.x)[min(tid + NTHR, img_chunks - 1)];
    else load_x8<XT>(a.x, (int64_t)min(tid + NTHR, valid - 1) * 8, raw2);
  }

  const int grp = lane / G, c0 = lane % G;
  const int nw0 = n0 + GROUPS * wave;  // first channel of this wave
  const int n = nw0 + grp;
  const WRsrc wr[2] = {make_wrsrc(a.gate, WT, a.I, nb, nbp), make_wrsrc(a.up, WT, a.I, nb, nbp)};
  const int cpr = nbp >> 3;  // 16-byte pieces per row of scales
  u32x4 sc[2];
  if (SCL) {
    const int rw = lane / cpr, cc = lane - rw * cpr;
    const uint32_t off = rw < GROUPS ? (uint32_t)((((int64_t)nw0 + rw) * nbp + cc * 8) * 2) : BUF_OOB;
    sc[0] = __builtin_amdgcn_raw_buffer_load_b128(wr[0].d, off, 0, BUF_NT);
    sc[1] = __builtin_amdgcn_raw_buffer_load_b128(wr[1].d, off, 0, BUF_NT);
  }
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  const uint32_t rbase = (uint32_t)n * (uint32_t)nb, dbase = (uint32_t)n * (uint32_t)nbp;
  auto load_trip = [&](PairChunk<WT, U, SCL>& c, int t0, auto ulo, auto uhi) {
#pragma unroll
    for (int u = decltype(ulo)::value; u < decltype(uhi)::value; u++) {
      const int col = t0 + G * u + c0;
      const bool ok = col < nb;
#pragma unroll
      for (int r = 0; r < 2; r++) {
        const uint32_t off = ok ? (rbase + (uint32_t)col) * 16u : BUF_OOB;
        c.w0[u][r] = __builtin_amdgcn_raw_buffer_load_b128(wr[r].q0, off, 0, BUF_NT);
        if (WT == MLLM_HIP_Q8_0) c.w1[WT == MLLM_HIP_Q8_0 ? u : 0][r] = __builtin_amdgcn_raw_buffer_load_b128(wr[r].q1, off, 0, BUF_NT);
        if (!SCL) c.dw[SCL ? 0 : u][r] = __builtin_amdgcn_raw_buffer_load_b16(wr[r].d, ok ? (dbase + (uint32_t)col) * 2u : BUF_OOB, 0, BUF_NT);
      }
    }
  };
  // (only the first block column of the first trip here, the others behind the quantization of x: what every workgroup of
  // the launch asks for at its start delays the activations each of them needs first)
  PairChunk<WT, U, SCL> cur;
  constexpr int UFIRST = U >= 2 ? 1 : U;
  load_trip(cur, 0, std::integral_constant<int, 0>{}, std::integral_constant<int, UFIRST>{});
  __asm__ volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  if (XT == GEMV_PREQ) {
    u32x4* s16 = reinterpret_cast<u32x4*>(smem);
    if (tid < img_chunks) s16[tid] = raw.r[0];
    if (NPRE > 1 && tid + NTHR < img_chunks) s16[tid + NTHR] = raw2.r[0];
    for (int c = tid + NPRE * NTHR; c < img_chunks; c += NTHR) s16[c] = reinterpret_cast<const u32x4*>(a.x)[c];
  } else {
    const QImage xi{smem, MT, nb, a.x86};
    float v[8];
    x8_to_f32<XT>(raw, v);
    if (tid >= valid) {
#pragma unroll
      for (int e = 0; e < 8; e++) v[e] = 0.f;
    }
    if (tid < nitems) quad_quantize_to_image(v, xi, 0, tid >> 2, tid & 3, true);  // block index runs over m * nb + b
    if (NPRE > 1) {
      const int it = tid + NTHR;
      x8_to_f32<XT>(raw2, v);
      if (it >= valid) {
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = 0.f;
      }
      if (it < nitems) quad_quantize_to_image(v, xi, 0, it >> 2, it & 3, true);  // whole quads: nitems and NTHR are multiples of 4
    }
    for (int it = tid + NPRE * NTHR; it < nitems; it += NTHR) {
      XRaw<XT> rw;
      load_x8<XT>(a.x, (int64_t)min(it, valid - 1) * 8, rw);
      x8_to_f32<XT>(rw, v);
      if (it >= valid) {
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = 0.f;
      }
      quad_quantize_to_image(v, xi, 0, it >> 2, it & 3, true);
    }
  }
  if (SCL && lane < GROUPS * cpr) {
    *reinterpret_cast<u32x4*>(s_ws + lane * 8) = sc[0];
    *reinterpret_cast<u32x4*>(s_ws + (GROUPS * cpr + lane) * 8) = sc[1];
  }
  load_trip(cur, 0, std::integral_constant<int, UFIRST>{}, std::integral_constant<int, U>{});
  __syncthreads();
  const u32x4* s_lo = reinterpret_cast<const u32x4*>(smem);
  const u32x4* s_hi = s_lo + mnb;
  const float* s_d = reinterpret_cast<const float*>(s_hi + mnb);
  const int* s_n8 = reinterpret_cast<const int*>(s_d + mnb);

  float acc[2][MT];
#pragma unroll
  for (int r = 0; r < 2; r++)
#pragma unroll
    for (int m = 0; m < MT; m++) acc[r][m] = 0.f;
  for (int t0 = 0; t0 < nb; t0 += G * U) {
    PairChunk<WT, U, SCL> nxt;
    const bool more = t0 + G * U < nb;  // uniform
    if (more) load_trip(nxt, t0 + G * U, std::integral_constant<int, 0>{}, std::integral_constant<int, U>{});
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int col = t0 + G * u + c0;
      if (col < nb) {
        float dwf[2];
#pragma unroll
        for (int r = 0; r < 2; r++) dwf[r] = f16bits_to_f32(SCL ? s_ws[(r * GROUPS + grp) * nbp + col] : cur.dw[SCL ? 0 : u][r]);
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const u32x4 xlo = s_lo[m * nb + col], xhi = s_hi[m * nb + col];
          const float dx = s_d[m * nb + col];
          const int n8 = s_n8[m * nb + col];
#pragma unroll
          for (int r = 0; r < 2; r++)
            acc[r][m] = fmaf(dwf[r] * dx, (float)block_dot<WT>(cur.w0[u][r], cur.w1[WT == MLLM_HIP_Q8_0 ? u : 0][r], xlo, xhi, n8), acc[r][m]);
        }
      }
    }
    if (more) cur = nxt;
  }
#pragma unroll
  for (int m = 0; m < MT; m++) {
    const float g = group_sum<G>(acc[0][m]), u = group_sum<G>(acc[1][m]);
    if (c0 == 0) {
      const float hv = m < a.M ? silu_sel(g, a.exp_accurate) * u : 0.f;
      s_h[m * 32 + GROUPS * wave + grp] = hv;
      if (a.h && m < a.M) a.h[(size_t)m * a.I + n] = hv;
    }
  }
  if (!a.h_image) return;  // uniform
  __syncthreads();
  if (tid < 4 * MT) {  // one quad per activation row: the 32 values are exactly one Q8_0 block of h
    const int m = tid >> 2, j = tid & 3;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = s_h[m * 32 + 8 * j + i];
    quad_quantize_to_image(v, QImage{a.h_image, MT, a.I / QK, a.x86}, m, n0 / QK, j, true);
  }
}

static int g_mlp_U = 0;

template <int WT, int XT, int MT, int G, int U>
static int launch_mlp_gu(const MlpArgs& a, hipStream_t st) {
  const int nb = a.H / QK, nbp = (int)scale_row_stride(a.H);
  constexpr int GROUPS = 64 / G, NW = G / 2;
  const bool scl = GROUPS * (nbp / 8) <= 64;
  const size_t lds = align_up((size_t)MT * nb * 40, 16) + (size_t)MT * 32 * sizeof(float) + (scl ? (size_t)NW * 2 * GROUPS * nbp * 2 : 0);
  if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
  const dim3 grid((unsigned)(a.I / 32));
  auto go = [&](auto kern) -> int {
    if (lds > 64 * 1024)
      HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, grid, dim3(32 * G), lds, st, a);
    return (int)hipGetLastError();
  };
  return scl ? go(mlp_gateup_kernel<WT, XT, MT, G, U, true>) : go(mlp_gateup_kernel<WT, XT, MT, G, U, false>);
}
// 16 lanes per row, eight waves.  (32 lanes make 1024-thread workgroups, of which a CU holds one: the 304 workgroups of
// the 9728-channel MLP then run in two rounds, measured 11.2 us against 8.6.)
// Block columns per lane and trip, measured on 2 x [9728][2560]: Q8_0 (two 16-byte words per block) two; Q4_0 with one
// activation row the whole row in one trip (up to five), with more rows three.
template <int WT, int XT, int MT>
static int launch_mlp_u(const MlpArgs& a, hipStream_t st) {
  const int nb = a.H / QK;
  int U = WT == MLLM_HIP_Q8_0 ? 2 : 3;
  if (WT == MLLM_HIP_Q4_0 && MT == 1) {
    U = (nb + 15) / 16;
    if (U > 5) U = 4;
    if (U < 2) U = 2;
  }
  if (g_mlp_U) U = g_mlp_U;
  if (U == 2) return launch_mlp_gu<WT, XT, MT, 16, 2>(a, st);
  if (U == 3) return launch_mlp_gu<WT, XT, MT, 16, 3>(a, st);
  if (U == 5) return launch_mlp_gu<WT, XT, MT, 16, 5>(a, st);
  return launch_mlp_gu<WT, XT, MT, 16, 4>(a, st);
}
template <int WT, int XT>
static int launch_mlp_m(const MlpArgs& a, hipStream_t st) {
  if (a.M <= 1) return launch_mlp_u<WT, XT, 1>(a, st);
  if (a.M <= 2) return launch_mlp_u<WT, XT, 2>(a, st);
  if (a.M <= 4) return launch_mlp_u<WT, XT, 4>(a, st);
  return launch_mlp_u<WT, XT, 8>(a, st);
}

}  // namespace mllmhip

using namespace mllmhip;

// tuning override for sweeps: block columns per lane and trip (2..5); 0 = heuristic
MLLM_API int mllm_hip_mlp_set_tuning(int units_in_flight) {
  if (units_in_flight != 0 && (units_in_flight < 2 || units_in_flight > 5)) return MLLM_HIP_E_BADARG;
  g_mlp_U = units_in_flight;
  return 0;
}

MLLM_API int mllm_hip_mlp_gate_up_q(int wtype, const void* gate_packed, const void* up_packed, const void* x, int x_kind, float* h,
                                    void* h_image, int M, int64_t I, int64_t H, int act_scale_mode, void* stream) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || !gate_packed || !up_packed || !x || (!h && !h_image)) return MLLM_HIP_E_BADARG;
  if (x_kind != MLLM_HIP_F32 && x_kind != MLLM_HIP_BF16 && x_kind != MLLM_HIP_Q8_IMAGE) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (M < 1 || M > 8 || I <= 0 || H <= 0 || I % 32 || H % QK || I > INT32_MAX || H > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (I * (H / QK) * 16 >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(gate_packed) % 16 || reinterpret_cast<uintptr_t>(up_packed) % 16 || reinterpret_cast<uintptr_t>(x) % 16 ||
      reinterpret_cast<uintptr_t>(h_image) % 16)
    return MLLM_HIP_E_ALIGN;
  MlpArgs a{packed_view(wtype, gate_packed, I, H), packed_view(wtype, up_packed, I, H), x, h, reinterpret_cast<unsigned char*>(h_image),
            M, (int)H, (int)I, act_scale_mode == MLLM_HIP_SCALE_X86_REF, exp_mode_accurate()};
  hipStream_t st = (hipStream_t)stream;
  if (wtype == MLLM_HIP_Q4_0 && M >= 3 && g_mlp_U == 0 && mlp_mfma_fits(M <= 4 ? 4 : 8, (int)(H / QK)))
    return launch_mlp_mfma(x_kind, a.gate, a.up, x, h, a.h_image, M, (int)I, (int)(H / QK), (int)scale_row_stride(H), a.x86, a.exp_accurate, st);
  if (wtype == MLLM_HIP_Q4_0) {
    if (x_kind == MLLM_HIP_F32) return launch_mlp_m<MLLM_HIP_Q4_0, MLLM_HIP_F32>(a, st);
    if (x_kind == MLLM_HIP_BF16) return launch_mlp_m<MLLM_HIP_Q4_0, MLLM_HIP_BF16>(a, st);
    return launch_mlp_m<MLLM_HIP_Q4_0, GEMV_PREQ>(a, st);
  }
  if (x_kind == MLLM_HIP_F32) return launch_mlp_m<MLLM_HIP_Q8_0, MLLM_HIP_F32>(a, st);
  if (x_kind == MLLM_HIP_BF16) return launch_mlp_m<MLLM_HIP_Q8_0, MLLM_HIP_BF16>(a, st);
  return launch_mlp_m<MLLM_HIP_Q8_0, GEMV_PREQ>(a, st);
}
