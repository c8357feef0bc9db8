// Launchers of the matrix-core decode GEMV (three to eight activation rows); the kernel is in qgemv_mfma_kernel.h.
#include <stdio.h>

#include <algorithm>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "qgemv_mfk_kernel.h"

namespace mllmhip {

// ---- K slices as separate workgroups (qgemv_mfk_kernel.h) -----------------------------------------------------------------
// Arrival counters of the row tiles: device memory of the loaded code object, zero when the code object is loaded and put
// back to zero by every launch that uses them.  The name below is a host-side stand-in; kernels get the device address that
// hipGetSymbolAddress returned for the current device.  Launches that may run at the same time must not share counters:
// the array is cut into blocks and a block belongs to one workspace address (callers already keep one workspace per
// concurrent call) until that address is released (mllm_hip_gemv_workspace_release) or the table is recycled: when a new
// address finds every block taken, the device is synchronised -- after which no launch is in flight and every counter is
// zero -- and all blocks are handed out afresh.  A caller that walks through ever new workspace addresses therefore pays one
// device synchronisation per MFK_BLOCKS new addresses instead of losing this kernel.  Only a stream under capture cannot
// synchronise: that launch takes the other kernels (MFK_NOT_TAKEN) and the library says so once on stderr.
constexpr int MFK_BLOCKS = 1024, MFK_COUNTERS = 1024, MFK_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned mfk_counters[MFK_BLOCKS * MFK_COUNTERS];  // 4 MB per GPU
struct MfkTable {
  unsigned* base = nullptr;                     // device address of mfk_counters on this device
  std::unordered_map<const void*, int> block;   // workspace address -> block
  std::vector<int> free_blocks;
  bool prepared = false;                        // dynamic-LDS attributes of the kernels set on this device
  uint64_t recycles = 0, refused = 0;
};
static MfkTable g_mfk[MFK_MAX_DEVICES];
static std::mutex g_mfk_mutex;
static bool g_mfk_said_recycle = false, g_mfk_said_refused = false;

// every instantiation the launchers below can pick: the limit of dynamic LDS is a per-device attribute of a kernel and is
// set once here instead of in front of every launch (a launch under stream capture then makes no other runtime call)
template <int WT, int XT, int MT>
static int mfk_set_lds_attr() {
  HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_mfk_kernel<WT, XT, MT, false>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_mfma_kernel<WT, XT, MT, false>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  if constexpr (MT == 8 && XT != GEMV_PREQ)
    HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_mfk_kernel<WT, XT, MT, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  return 0;
}
template <int WT>
static int mfk_set_lds_attr_w() {
  RC_RET((mfk_set_lds_attr<WT, MLLM_HIP_F32, 4>()));
  RC_RET((mfk_set_lds_attr<WT, MLLM_HIP_F32, 8>()));
  RC_RET((mfk_set_lds_attr<WT, MLLM_HIP_BF16, 4>()));
  RC_RET((mfk_set_lds_attr<WT, MLLM_HIP_BF16, 8>()));
  RC_RET((mfk_set_lds_attr<WT, GEMV_PREQ, 4>()));
  RC_RET((mfk_set_lds_attr<WT, GEMV_PREQ, 8>()));
  return 0;
}

// the table of the current device, ready for launches (counter address looked up, kernel attributes set); g_mfk_mutex held
static int mfk_table_locked(MfkTable** out) {
  int dev = 0;
  HIP_RET(hipGetDevice(&dev));
  if (dev < 0 || dev >= MFK_MAX_DEVICES) return MLLM_HIP_E_NODEVICE;
  MfkTable& t = g_mfk[dev];
  if (!t.base) {
    void* p = nullptr;
    HIP_RET(hipGetSymbolAddress(&p, HIP_SYMBOL(mfk_counters)));
    if (!p) return MLLM_HIP_E_NODEVICE;
    t.base = static_cast<unsigned*>(p);
    t.free_blocks.reserve(MFK_BLOCKS);
    for (int b = MFK_BLOCKS - 1; b >= 0; b--) t.free_blocks.push_back(b);
  }
  if (!t.prepared) {
    RC_RET(mfk_set_lds_attr_w<MLLM_HIP_Q4_0>());
    RC_RET(mfk_set_lds_attr_w<MLLM_HIP_Q8_0>());
    t.prepared = true;
  }
  *out = &t;
  return 0;
}

// what mllm_hip_init does for these kernels on the device that is current
int gemv_mfk_prepare_device() {
  std::lock_guard<std::mutex> lock(g_mfk_mutex);
  MfkTable* t = nullptr;
  return mfk_table_locked(&t);
}

// 0 and *out = the counter block of `workspace` on the current device; MFK_NOT_TAKEN when every block has an owner and the
// device cannot be synchronised now (stream capture)
static int mfk_counter_block(const void* workspace, hipStream_t st, unsigned** out) {
  std::lock_guard<std::mutex> lock(g_mfk_mutex);
  MfkTable* t = nullptr;
  RC_RET(mfk_table_locked(&t));
  auto it = t->block.find(workspace);
  if (it == t->block.end()) {
    if (t->free_blocks.empty()) {
      // every block has an owner.  Once the device is idle no launch uses any counter and all of them are zero, so every
      // owner can lose its block (an owner that comes back simply takes a new one).
      hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
      const bool capturing = hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone;
      if (capturing || hipDeviceSynchronize() != hipSuccess) {
        (void)hipGetLastError();
        t->refused++;
        if (!g_mfk_said_refused) {
          g_mfk_said_refused = true;
          fprintf(stderr, "mllm_hip: all %d counter blocks of the K-slice decode GEMV belong to other workspaces and the device cannot be "
                          "synchronised during stream capture; this launch takes the slower kernels (release workspaces with "
                          "mllm_hip_gemv_workspace_release, or reuse them)\n", MFK_BLOCKS);
        }
        return MFK_NOT_TAKEN;
      }
      t->block.clear();
      t->free_blocks.clear();
      for (int b = MFK_BLOCKS - 1; b >= 0; b--) t->free_blocks.push_back(b);
      t->recycles++;
      if (!g_mfk_said_recycle) {
        g_mfk_said_recycle = true;
        fprintf(stderr, "mllm_hip: more than %d workspace addresses have used the K-slice decode GEMV; the device was synchronised to "
                        "hand its counter blocks out afresh (release workspaces with mllm_hip_gemv_workspace_release, or reuse them, "
                        "to avoid this)\n", MFK_BLOCKS);
      }
    }
    const int b = t->free_blocks.back();
    t->free_blocks.pop_back();
    it = t->block.emplace(workspace, b).first;
  }
  *out = t->base + (size_t)it->second * MFK_COUNTERS;
  return 0;
}

// the same blocks for the many-row kernel (qgemv_mr.hip): a workspace runs one launch at a time
int gemv_counter_block(const void* workspace, hipStream_t st, unsigned** out) { return mfk_counter_block(workspace, st, out); }

int gemv_mfk_release(const void* workspace) {
  std::lock_guard<std::mutex> lock(g_mfk_mutex);
  for (MfkTable& t : g_mfk) {
    auto it = t.block.find(workspace);
    if (it == t.block.end()) continue;
    t.free_blocks.push_back(it->second);
    t.block.erase(it);
  }
  return 0;
}

void gemv_mfk_stats(int device, int* owned, int* capacity, long long* recycles, long long* refused) {
  std::lock_guard<std::mutex> lock(g_mfk_mutex);
  const bool ok = device >= 0 && device < MFK_MAX_DEVICES;
  if (owned) *owned = ok ? (int)g_mfk[device].block.size() : 0;
  if (capacity) *capacity = MFK_BLOCKS;
  if (recycles) *recycles = ok ? (long long)g_mfk[device].recycles : 0;
  if (refused) *refused = ok ? (long long)g_mfk[device].refused : 0;
}

// slices of a row when it is cut: the ones of the one-workgroup kernel (at most eight) up to 512 blocks, then slices of 64
int gemv_mfk_slices(int nb) { return nb <= 8 * 64 ? mf_slices(nb) : (nb + 63) / 64; }

template <int WT, int XT, int MT>
static int launch_mfk_t(const GemvArgs& a_in, const MfkArgs& k_in, int nwaves, unsigned grid_x, unsigned groups, hipStream_t st) {
  MfkArgs k = k_in;
  k.gx = (int)grid_x;
  k.groups = (int)groups;
  const size_t lds = mfk_lds_bytes<MT>(WT, k.nbs, nwaves);
  if (lds > 160 * 1024) return MFK_NOT_TAKEN;
  constexpr bool CAN_GROUP = MT == 8 && XT != GEMV_PREQ;  // the only form the launcher lets through with several groups
  if (groups > 1 && !CAN_GROUP) return MFK_NOT_TAKEN;
  auto kern = groups > 1 ? gemv_mfk_kernel<WT, XT, MT, CAN_GROUP> : gemv_mfk_kernel<WT, XT, MT, false>;
  if (lds > 64 * 1024) RC_RET(gemv_mfk_prepare_device());  // (sets the kernels' dynamic-LDS limit once per device)
  // several row groups: a 1-D grid, (column, slice) items padded to whole eights, the groups of an item next to each other
  const dim3 grid = groups > 1 ? dim3((grid_x * (unsigned)k.S + 7) / 8 * 8 * groups) : dim3(grid_x, (unsigned)k.S);
  hipLaunchKernelGGL(kern, grid, dim3(nwaves * 64), lds, st, a_in, k);
  return (int)hipGetLastError();
}

// groups > 1: a_in.M rows of raw activations in groups of eight (the last may be shorter), every group a workgroup of its own per (row tiles, slice)
// in the same launch (the groups read the same weights: once from memory, then from the caches)
int launch_gemv_mfk(int wtype, int x_kind, int MT, const GemvArgs& a_in, const void* workspace, void* part, size_t part_bytes,
                    int waves, int slices, hipStream_t st, int groups) {
  if (groups < 1 || groups > 65535 || (groups > 1 && (MT != 8 || x_kind == GEMV_PREQ || a_in.M <= 8 * (groups - 1) || a_in.M > 8 * groups))) return MFK_NOT_TAKEN;
  GemvArgs a = a_in;
  MfkArgs k{};
  int tiles_total = 0;
  for (int p = 0; p < a.nparts; p++) tiles_total += (a.part[p].N + 15) / 16;
  k.S = gemv_mfk_slices(a.nb);
  k.nbs = ((a.nb + k.S - 1) / k.S + 7) / 8 * 8;
  k.vs = k.nbs;
  // a launch whose row tiles alone fill the chip keeps its rows whole where a slice may be that long: no partial sums, no
  // second pass (gate + up of the 4B layer, 1216 tiles x 80 blocks: 10.6 -> 9.3 us at four rows, 12.7 -> 12.3 at eight;
  // q+k+v, 384 tiles, is slower whole: 6.5 -> 8.6 / 8.2 -> 11.6).  The kernel still sums the row in chains of k.vs blocks
  // and adds the chains in slice order: the same bits either way.  (slices: 1 = whole rows, 2 = never, for measurements)
  // (Row groups count like more tiles, for matrices of at least 512 tiles: 9728 x 2560 with two groups 16.0 -> 12.3 us whole;
  // 4096 x 2560 with four groups is slower whole, 9.4 -> 12.1.)
  if (a.nb <= MFK_MAX_NBS && (slices == 1 || (slices <= 0 && (int64_t)tiles_total * groups >= 1024 && tiles_total >= 512))) {
    k.S = 1;
    k.nbs = (a.nb + 7) / 8 * 8;
  }
  if (k.nbs > MFK_MAX_NBS || k.S > 65535) return MFK_NOT_TAKEN;
  k.ipr_magic = ((1 << 20) + 2 * k.nbs - 1) / (2 * k.nbs);
  // Row tiles (= waves) per workgroup.  All workgroups are resident at once and every one costs vector-ALU time (its
  // quantization of the slice of x, then per tile the MFMA / scaling loop), so what counts is the work of the busiest CU:
  // rounds = ceil(workgroups / 256 CUs), each round costing (tiles per workgroup x loop + quantization).  Measured ratio of
  // the two on the 4B shapes at eight rows: quantization of a slice = about two tiles' loops.  E.g. gate + up (1216 tiles x 2
  // slices): four tiles per workgroup -> 608 workgroups, three on some CUs (12 tile loops + 3 quantizations), five -> 488
  // workgroups, two per CU (10 + 2); the down projection (160 tiles x 8 slices): five -> exactly 256 workgroups.
  const int nw_min = std::max(3, (k.nbs + 15) / 16);
  int nwaves = waves;
  // several row groups: four waves (measured over the 4B shapes with two to four groups against the model below, which counts
  // rounds of workgroups although all of them are resident: down 15.7 -> 12.6 us at 16 rows and 21.7 -> 17.8 at 32, o at 32
  // rows 13.5 -> 11.1, q+k+v at 24 rows 15.5 -> 12.2; q+k+v and o at 16 rows lose 0.8 us)
  // (cut rows only: whole rows want one workgroup per CU, which the model finds: 9728 x 2560 at 24 rows 13.6 us with eight
  // waves = 228 workgroups, 21.4 with five = 366)
  if ((nwaves < nw_min || nwaves > 8) && groups > 1 && k.S > 1) nwaves = std::max(nw_min, 4);
  if (nwaves < nw_min || nwaves > 8) {
    double best = 1e30;
    for (int nw = nw_min; nw <= 8; nw++) {
      int64_t wgs = 0;
      for (int p = 0; p < a.nparts; p++) wgs += ((a.part[p].N + 15) / 16 + nw - 1) / nw;
      wgs *= (int64_t)k.S * groups;
      const double cost = (double)((wgs + 255) / 256) * (nw + 2.0);
      if (cost < best - 1e-9) {
        best = cost;
        nwaves = nw;
      }
    }
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
  if (k.S > 1) {
    if (!workspace || !part || (size_t)groups * k.S * MT * np * 4 > part_bytes || (size_t)grid * groups > (size_t)MFK_COUNTERS) return MFK_NOT_TAKEN;
    RC_RET(mfk_counter_block(workspace, st, &k.counters));
    k.part = static_cast<float*>(part);
    // the columns' counters up to a cache line apart where the block has room: the workgroups of different columns arrive at
    // about the same time, and arrivals on one line queue behind each other (the step of the 4B layers at four rows
    // 1.078 -> 1.002 ms, at eight 1.351 -> 1.281; a block four times the size, a line per counter throughout: no further gain)
    k.cstride = 1;
    while (k.cstride < 32 && (size_t)grid * groups * k.cstride * 2 <= (size_t)MFK_COUNTERS) k.cstride *= 2;
  }
#define MFK_CASE(WT_, XT_)                                                         \
  if (wtype == WT_ && x_kind == XT_)                                               \
    return MT == 4 ? launch_mfk_t<WT_, XT_, 4>(a, k, nwaves, grid, (unsigned)groups, st) : launch_mfk_t<WT_, XT_, 8>(a, k, nwaves, grid, (unsigned)groups, st);
  MFK_CASE(MLLM_HIP_Q4_0, MLLM_HIP_F32)
  MFK_CASE(MLLM_HIP_Q4_0, MLLM_HIP_BF16)
  MFK_CASE(MLLM_HIP_Q4_0, GEMV_PREQ)
  MFK_CASE(MLLM_HIP_Q8_0, MLLM_HIP_F32)
  MFK_CASE(MLLM_HIP_Q8_0, MLLM_HIP_BF16)
  MFK_CASE(MLLM_HIP_Q8_0, GEMV_PREQ)
#undef MFK_CASE
  return MLLM_HIP_E_BADARG;
}

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
  if (lds > 64 * 1024) RC_RET(gemv_mfk_prepare_device());
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
