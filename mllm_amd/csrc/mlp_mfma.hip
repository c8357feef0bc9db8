// The MLP front half h = silu(gate(x)) * up(x) for three to eight activation rows on the matrix cores (Q4_0): the decode GEMV
// kernel of qgemv_mfma_kernel.h in its paired mode, where the waves of the gate and of the up projection of the same 16
// channels sit in one workgroup and the epilogue forms h and its Q8_0 image.  Entry point: mllm_hip_mlp_gate_up_q
// (mlp_decode.hip).
#include "qgemv_mfma_kernel.h"

namespace mllmhip {

// A workgroup holds whole 32-channel blocks of h: two row tiles x two projections x S K-slices = 4 S waves, so at most four
// slices (rows of up to 160 blocks, K = 5120) under the 1024-thread bound
static int mlp_mfma_waves(int S) { return 4 * S; }

bool mlp_mfma_fits(int MT, int nb) {
  const int S = mf_slices(nb);
  if (S > 4) return false;
  const int nbs = ((nb + S - 1) / S + 7) / 8 * 8;
  return (MT == 4 ? mf_lds_bytes<4>(nb, nbs, 4 * S) : mf_lds_bytes<8>(nb, nbs, 4 * S)) <= 160 * 1024;
}

template <int XT, int MT>
static int launch_mlp_mfma_t(const GemvArgs& a, const MfmaMlpOut& mo, hipStream_t st) {
  const int S = mf_slices(a.nb);
  const int nbs = ((a.nb + S - 1) / S + 7) / 8 * 8;
  const int nwaves = mlp_mfma_waves(S);
  const int tiles_wg = nwaves / (2 * S);  // two
  const int tiles = (a.part[0].N + 15) / 16;
  const unsigned grid = (unsigned)((tiles + tiles_wg - 1) / tiles_wg);
  const size_t lds = mf_lds_bytes<MT>(a.nb, nbs, nwaves);
  if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
  auto kern = gemv_mfma_kernel<MLLM_HIP_Q4_0, XT, MT, true>;
  if (lds > 64 * 1024)
    HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(nwaves * 64), lds, st, a, S, nbs, mo);
  return (int)hipGetLastError();
}

// x_kind: MLLM_HIP_F32, MLLM_HIP_BF16 or GEMV_PREQ; 3 <= M <= 8; I % 32 == 0
int launch_mlp_mfma(int x_kind, const PackedView& gate, const PackedView& up, const void* x, float* h, unsigned char* image, int M, int I,
                    int nb, int nbp, int x86_scale, int exp_accurate, hipStream_t st) {
  GemvArgs a{};
  a.part[0].w = gate;
  a.part[1].w = up;
  a.part[0].N = a.part[1].N = I;
  a.nparts = 2;
  a.x = x;
  a.M = M;
  a.nb = nb;
  a.nbp = nbp;
  a.x86_scale = x86_scale;
  const MfmaMlpOut mo{h, image, exp_accurate};
  const bool four = M <= 4;
  if (x_kind == MLLM_HIP_F32) return four ? launch_mlp_mfma_t<MLLM_HIP_F32, 4>(a, mo, st) : launch_mlp_mfma_t<MLLM_HIP_F32, 8>(a, mo, st);
  if (x_kind == MLLM_HIP_BF16) return four ? launch_mlp_mfma_t<MLLM_HIP_BF16, 4>(a, mo, st) : launch_mlp_mfma_t<MLLM_HIP_BF16, 8>(a, mo, st);
  if (x_kind == GEMV_PREQ) return four ? launch_mlp_mfma_t<GEMV_PREQ, 4>(a, mo, st) : launch_mlp_mfma_t<GEMV_PREQ, 8>(a, mo, st);
  return MLLM_HIP_E_BADARG;
}

}  // namespace mllmhip
