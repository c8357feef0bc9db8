// Launcher of the many-row Q4_0 / Q8_0 kernel (nine rows and more per call; the kernel is in qgemv_mr_kernel.h).
#include <algorithm>

#include "qgemv_mr_kernel.h"

namespace mllmhip {

int gemv_counter_block(const void* workspace, hipStream_t st, unsigned** out);  // qgemv_mfma.hip

// activation rows of the quantized image a call with M rows needs (whole groups of 16 or 32 rows)
int gemv_mr_image_rows(int M) {
  const int MT = M <= 16 ? 16 : 32;
  return (M + MT - 1) / MT * MT;
}

// bytes of partial sums behind the image: every group's slices, each part's rows rounded up to 16
size_t gemv_mr_part_bytes(int M, int nb, int64_t n_total_padded) {
  const int S = gemv_mfk_slices(nb);
  return S > 1 ? (size_t)gemv_mr_image_rows(M) * S * (size_t)n_total_padded * 4 : 0;
}

// the limit of dynamic LDS is a per-device attribute of a kernel: set once per device for every instantiation (mllm_hip_init
// calls this, so that a launch under stream capture makes no other runtime call)
static bool g_mr_prepared[64];
int gemv_mr_prepare_device() {
  int dev = 0;
  HIP_RET(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return MLLM_HIP_E_NODEVICE;
  if (g_mr_prepared[dev]) return 0;
  HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_mr_kernel<MLLM_HIP_Q4_0, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_mr_kernel<MLLM_HIP_Q4_0, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_mr_kernel<MLLM_HIP_Q8_0, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_mr_kernel<MLLM_HIP_Q8_0, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  g_mr_prepared[dev] = true;
  return 0;
}

template <int WT, int AG>
static int launch_mr_t(const GemvArgs& a, const MrArgs& k, int nwaves, hipStream_t st) {
  const size_t lds = mr_lds_bytes<AG>(WT, k.nbs, nwaves);
  if (lds > 160 * 1024) return MFK_NOT_TAKEN;
  if (lds > 64 * 1024) RC_RET(gemv_mr_prepare_device());
  const unsigned grid = (unsigned)(((size_t)k.gx * k.S + 7) / 8 * 8 * k.groups);
  hipLaunchKernelGGL((gemv_mr_kernel<WT, AG>), dim3(grid), dim3(nwaves * 64), lds, st, a, k);
  return (int)hipGetLastError();
}

// a_in.x = the quantized image of gemv_mr_image_rows(a_in.M) rows (rows past a_in.M zero); part / part_bytes: room for the partial
// sums.  MFK_NOT_TAKEN where the launch does not fit (room, counters) or the kernel is not the faster one: the caller takes the
// eight-row kernels.  dry: decide only (0 = the launch would go out), so that the caller queues the quantization of x first.
int launch_gemv_mr(int wtype, const GemvArgs& a_in, const void* workspace, void* part, size_t part_bytes, int waves, int slices, hipStream_t st,
                   bool dry) {
  GemvArgs a = a_in;
  MrArgs k{};
  const int AG = a.M <= 16 ? 1 : 2, MT = 16 * AG;
  k.groups = (a.M + MT - 1) / MT;
  k.rows_img = k.groups * MT;
  int tiles_total = 0;
  for (int p = 0; p < a.nparts; p++) tiles_total += (a.part[p].N + 15) / 16;
  k.S = gemv_mfk_slices(a.nb);
  k.nbs = ((a.nb + k.S - 1) / k.S + 7) / 8 * 8;
  // Whole rows (one slice: no partial sums, no second pass) where the row tiles alone fill the chip and a row has at most
  // MR_MAX_NBS blocks: this is where the kernel is faster than groups of eight rows on the decode kernel (measured on the 4B
  // layer shapes, 16 / 32 / 64 rows, us: gate + up Q4_0 18.2 / 24.1 / 42.9 against 21.8 / 32.9 / 57.7, Q8_0 18.3 / 24.3 / 42.8
  // against 25.0 / 39.7 / 67.0; one 9728 x 2560 matrix Q8_0 at 32 rows 22.8 against 24.3).  Cut rows lose to that form (down
  // projection at 32 rows 20.4 against 19.0, q + k + v 18.6 against 13.3: a workgroup's dependent chain of image copy, block
  // loop and meeting in memory is longer than the decode kernel's and fewer waves share a CU) and are refused unless asked
  // for (slices == 2: tests and measurements).  The rule looks at the matrices only, never at the number of activation
  // rows: a row's bits must not depend on what else is in the call, so it also asks for the LDS of the taller build (32
  // activation rows) with the fewest waves that build may have.
  bool whole = false;
  if (a.nb <= MR_MAX_NBS && (slices == 1 || tiles_total >= (wtype == MLLM_HIP_Q8_0 ? 600 : 1024))) {
    const int nbs_w = (a.nb + 7) / 8 * 8;
    if (mr_lds_bytes<2>(wtype, nbs_w, std::max(4, (32 * nbs_w + 511) / 512)) <= 160 * 1024) {
      k.S = 1;
      k.nbs = nbs_w;
      whole = true;
    }
  }
  if (!whole && slices != 2) return MFK_NOT_TAKEN;
  if (k.nbs > MR_MAX_NBS || k.S > 65535 || k.groups > 4096) return MFK_NOT_TAKEN;
  k.nbs_magic = ((1 << 20) + k.nbs - 1) / k.nbs;
  // Row tiles (= waves) per workgroup: enough threads for the image items (at most eight per thread), then the count that makes
  // about one workgroup per CU and round (every workgroup copies its slice of the image: fewer, larger workgroups copy less)
  const int nw_min = std::max(4, (MT * k.nbs + 511) / 512);
  int nwaves = waves;
  if (nwaves < nw_min || nwaves > 8) {
    double best = 1e30;
    for (int nw = nw_min; nw <= 8; nw++) {
      if ((AG == 1 ? mr_lds_bytes<1>(wtype, k.nbs, nw) : mr_lds_bytes<2>(wtype, k.nbs, nw)) > 160 * 1024) break;
      int64_t wgs = 0;
      for (int p = 0; p < a.nparts; p++) wgs += ((a.part[p].N + 15) / 16 + nw - 1) / nw;
      wgs *= (int64_t)k.S * k.groups;
      const double cost = (double)((wgs + 255) / 256) * (nw + 2.0);
      if (cost < best - 1e-9) {
        best = cost;
        nwaves = nw;
      }
    }
    if (nwaves < nw_min) nwaves = nw_min;
  }
  unsigned grid = 0;
  int np = 0;
  for (int p = 0; p < a.nparts; p++) {
    a.wg_start[p] = (int)grid;
    const int tiles = (a.part[p].N + 15) / 16;
    grid += (unsigned)((tiles + nwaves - 1) / nwaves);
    k.col0[p] = np;
    np += tiles * 16;
  }
  a.wg_start[a.nparts] = (int)grid;
  k.NP = np;
  k.gx = (int)grid;
  if ((size_t)grid * k.S * k.groups > 0x7fffffffu / 8) return MFK_NOT_TAKEN;
  if (k.S > 1) {
    if (!workspace || !part || (size_t)k.groups * k.S * MT * np * 4 > part_bytes || (size_t)grid * k.groups > 1024) return MFK_NOT_TAKEN;
    if (!dry) RC_RET(gemv_counter_block(workspace, st, &k.counters));
    k.part = static_cast<float*>(part);
    k.cstride = 1;  // the columns' counters up to a cache line apart where the block of 1024 has room (see the K-slice kernel)
    while (k.cstride < 32 && (size_t)grid * k.groups * k.cstride * 2 <= 1024) k.cstride *= 2;
  }
  if (dry) return (wtype == MLLM_HIP_Q4_0 || wtype == MLLM_HIP_Q8_0) ? 0 : MLLM_HIP_E_BADARG;
  if (wtype == MLLM_HIP_Q4_0) return AG == 1 ? launch_mr_t<MLLM_HIP_Q4_0, 1>(a, k, nwaves, st) : launch_mr_t<MLLM_HIP_Q4_0, 2>(a, k, nwaves, st);
  if (wtype == MLLM_HIP_Q8_0) return AG == 1 ? launch_mr_t<MLLM_HIP_Q8_0, 1>(a, k, nwaves, st) : launch_mr_t<MLLM_HIP_Q8_0, 2>(a, k, nwaves, st);
  return MLLM_HIP_E_BADARG;
}

}  // namespace mllmhip
