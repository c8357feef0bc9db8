// GEMV kernel instances for one weight type reading pre-quantized activations; split out so that the sets compile in parallel.
#include "qgemv_kernel.h"

namespace mllmhip {
int launch_gemv_q8_preq(const GemvArgs& a, int MT, GemvShape s, hipStream_t st) { return launch_gemv<MLLM_HIP_Q8_0, GEMV_PREQ>(a, MT, s, st); }
}  // namespace mllmhip
