// GEMV kernel instances for one (weight type, activation type) pair; split out so that the pairs compile in parallel.
#include "qgemv_kernel.h"

namespace mllmhip {
int launch_gemv_q8_bf16(const GemvArgs& a, int MT, GemvShape s, hipStream_t st) { return launch_gemv<MLLM_HIP_Q8_0, MLLM_HIP_BF16>(a, MT, s, st); }
}  // namespace mllmhip
