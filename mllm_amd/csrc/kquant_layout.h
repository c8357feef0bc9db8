// Packed layout of Q4_K / Q6_K weight matrices (written by mllm_hip_kq_prepack), shared by the decode GEMV kernels and the
// many-row tile kernels.
#pragma once
#include "qcommon.h"

#define QK_K 256

namespace mllmhip {

// ---- packed layout ---------------------------------------------------------------------------------------------------
// Q4_K: plane A = nibbles, 128 B per super-block (eight 16-byte chunks); plane S = the 6-bit scales and mins decoded to bytes
//       at load time, one dword per pair of sub-blocks {sc[2p], sc[2p+1], m[2p], m[2p+1]} = 16 B per super-block (a lane of
//       the GEMV needs exactly the dword of its chunk's pair: no bit shuffle per chunk); plane D = {fp16 d, fp16 dmin} as
//       IEEE patterns, 4 B per super-block.
// Q6_K: plane A = low nibbles (128 B per super-block), plane H = high bit pairs (64 B), plane S = 16 int8 scales, plane D =
//       fp16 d as IEEE pattern (2 B).
struct KView {
  const u32x4* a;
  const u32x4* h;
  const u32x4* s;
  const uint16_t* d;
};
__host__ __device__ inline size_t kq_plane(size_t bytes) { return align_up(bytes, 256); }
__host__ __device__ inline size_t kq_packed_bytes(int wtype, int64_t N, int64_t K) {
  const size_t sb = (size_t)N * (K / QK_K);
  if (wtype == MLLM_HIP_Q4_K) return kq_plane(sb * 128) + kq_plane(sb * 16) + kq_plane(sb * 4);
  return kq_plane(sb * 128) + kq_plane(sb * 64) + kq_plane(sb * 16) + kq_plane(sb * 2);
}
__host__ __device__ inline KView kq_view(int wtype, const void* packed, int64_t N, int64_t K) {
  const size_t sb = (size_t)N * (K / QK_K);
  const char* p = reinterpret_cast<const char*>(packed);
  KView v{};
  v.a = reinterpret_cast<const u32x4*>(p);
  p += kq_plane(sb * 128);
  if (wtype == MLLM_HIP_Q6_K) {
    v.h = reinterpret_cast<const u32x4*>(p);
    p += kq_plane(sb * 64);
  }
  v.s = reinterpret_cast<const u32x4*>(p);
  p += kq_plane(sb * 16);
  v.d = reinterpret_cast<const uint16_t*>(p);
  return v;
}

}  // namespace mllmhip
