// Launchers of the matrix-core decode GEMV (three to eight activation rows); the kernel is in qgemv_mfma_kernel.h.
#include "qgemv_mfma_kernel.h"

namespace mllmhip {

template <int WT, int XT, int MT>
static int launch_mfma_t(const GemvArgs& a_in, int waves, int slices, hipStream_t st) {
  GemvArgs a = a_in;
  int S = slices ? slices : mf_slices(a.nb);
  if (((a.nb + S - 1) / S + 7) / 8 * 8 > 64) S = mf_slices(a.nb);  // an override that leaves slices too long for the scale staging
  const int nbs = ((a.nb + S - 1) / S + 7) / 8 * 8;
  int nwaves = waves ? waves : (XT == GEMV_PREQ ? 4 : 8);
  if (nwaves < S) nwaves = S;
  const int tiles_wg = nwaves / S;
  unsigned grid = 0;
  for (int p = 0; p < a.nparts; p++) {
    a.wg_start[p] = (int)grid;
    const int tiles = (a.part[p].N + 15) / 16;
    grid += (unsigned)((tiles + tiles_wg - 1) / tiles_wg);
  }
  a.wg_start[a.nparts] = (int)grid;
  const size_t lds = mf_lds_bytes<MT>(a.nb, nbs, nwaves);
  if (lds > 160 * 1024) return MLLM_HIP_E_SHAPE;
  auto kern = gemv_mfma_kernel<WT, XT, MT, false>;
  if (lds > 64 * 1024)
    HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(nwaves * 64), lds, st, a, S, nbs, MfmaMlpOut{nullptr, nullptr, 0});
  return (int)hipGetLastError();
}

// whether rows of nb blocks fit the kernel's LDS (sized for eight waves, whatever the launch then uses: the answer must not
// depend on the kind of activations)
bool gemv_mfma_fits(int MT, int nb) {
  if (nb > 512) return false;  // weight scale pieces: at most 128 per wave
  const int S = mf_slices(nb);
  const int nbs = ((nb + S - 1) / S + 7) / 8 * 8;
  return (MT == 4 ? mf_lds_bytes<4>(nb, nbs, 8) : mf_lds_bytes<8>(nb, nbs, 8)) <= 160 * 1024;
}

// x_kind: MLLM_HIP_F32, MLLM_HIP_BF16 or GEMV_PREQ; MT: 4 or 8
int launch_gemv_mfma(int wtype, int x_kind, int MT, const GemvArgs& a, int waves, int slices, hipStream_t st) {
  if (waves != 0 && waves != 2 && waves != 4 && waves != 8) return MLLM_HIP_E_BADARG;
  if (slices != 0 && slices != 1 && slices != 2 && slices != 4) return MLLM_HIP_E_BADARG;
#define MF_CASE(WT_, XT_)                                                          \
  if (wtype == WT_ && x_kind == XT_)                                               \
    return MT == 4 ? launch_mfma_t<WT_, XT_, 4>(a, waves, slices, st) : launch_mfma_t<WT_, XT_, 8>(a, waves, slices, st);
  MF_CASE(MLLM_HIP_Q4_0, MLLM_HIP_F32)
  MF_CASE(MLLM_HIP_Q4_0, MLLM_HIP_BF16)
  MF_CASE(MLLM_HIP_Q4_0, GEMV_PREQ)
  MF_CASE(MLLM_HIP_Q8_0, MLLM_HIP_F32)
  MF_CASE(MLLM_HIP_Q8_0, MLLM_HIP_BF16)
  MF_CASE(MLLM_HIP_Q8_0, GEMV_PREQ)
#undef MF_CASE
  return MLLM_HIP_E_BADARG;
}

}  // namespace mllmhip
