// Q4_0 / Q8_0 Linear for decode (M = 1..8) on gfx950: weight pre-pack, fused Q8_0 activation quantization + block-dot
// GEMV, and the parity probes.  HBM-bound: every weight byte is read once with 16-byte fully coalesced loads.
//
// Arithmetic follows the reference's x86 CPU path:
//   activation quantization  mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.cpp:106-190
//   block dot + scaling       mllm/backends/cpu/kernels/common/llamafile/llamafile_sgemm.cpp:697-743
//   flow                      mllm/backends/cpu/kernels/common/ggml/matmul.cpp:148-206
// The int32 block sums are exact; the fp32 accumulation order differs from the CPU's 8-lane order (tolerance 1e-3 rel-L2).
#include <algorithm>

#include "qgemv_kernel.h"

#include <string.h>

#include <initializer_list>
#include <mutex>

namespace mllmhip {

// =========================================================================================================
// pre-pack: reference blocks (AoS) -> code planes + scale array
// =========================================================================================================
__global__ void prepack_kernel(int wtype, const uint8_t* __restrict__ blocks, int x86_scale, u32x4* __restrict__ q0,
                               u32x4* __restrict__ q1, uint16_t* __restrict__ d, int64_t nblocks, int nb, int nbp) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  const int bb = wtype == MLLM_HIP_Q4_0 ? 18 : 34;
  const uint8_t* b = blocks + i * bb;
  uint16_t raw = (uint16_t)b[0] | ((uint16_t)b[1] << 8);
  uint16_t bits = raw;
  if (x86_scale) {
    // the field holds the pattern as a half-precision NUMBER: number -> integer gives the pattern that is looked up
    float num = f16bits_to_f32(raw);
    bits = (num >= 0.f && num < 65536.f) ? (uint16_t)(uint32_t)num : (uint16_t)0;
  }
  const int64_t row = i / nb;
  const int col = (int)(i - row * nb);
  d[row * nbp + col] = bits;
  if (col == nb - 1)
    for (int c = nb; c < nbp; c++) d[row * nbp + c] = 0;  // padding of the scale row
  uint32_t w[8];
  const int nw = wtype == MLLM_HIP_Q4_0 ? 4 : 8;
  for (int j = 0; j < nw; j++) {
    const uint8_t* p = b + 2 + 4 * j;  // blocks are only 2-byte aligned: assemble from bytes
    w[j] = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
  }
  q0[i] = u32x4{w[0], w[1], w[2], w[3]};
  if (wtype == MLLM_HIP_Q8_0) q1[i] = u32x4{w[4], w[5], w[6], w[7]};
}

// =========================================================================================================
// stand-alone activation quantization, probes
// =========================================================================================================
__global__ void quantize_q8_0_kernel(const void* __restrict__ x, int x_dtype, int8_t* __restrict__ codes,
                                     uint16_t* __restrict__ d_bits, int64_t nblocks) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  float v[32];
  uint32_t q[8];
  int sum;
  load_block_f32(x, x_dtype, i * QK, v);
  d_bits[i] = quantize_block_q8_0(v, q, sum);
  u32x4* out = reinterpret_cast<u32x4*>(codes + i * QK);
  out[0] = u32x4{q[0], q[1], q[2], q[3]};
  out[1] = u32x4{q[4], q[5], q[6], q[7]};
}

__global__ void dequantize_kernel(int wtype, PackedView w, float* __restrict__ out, int64_t nblocks, int nb, int nbp) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  const float d = f16bits_to_f32(w.d[(i / nb) * nbp + i % nb]);
  const u32x4 a = w.q0[i];
  const uint32_t aw[4] = {a.x, a.y, a.z, a.w};
  float* o = out + i * QK;
  if (wtype == MLLM_HIP_Q4_0) {
    for (int j = 0; j < 16; j++) {
      const uint32_t byte = (aw[j >> 2] >> (8 * (j & 3))) & 0xffu;
      o[j] = (float)((int)(byte & 15u) - 8) * d;
      o[j + 16] = (float)((int)(byte >> 4) - 8) * d;
    }
  } else {
    const u32x4 b = w.q1[i];
    const uint32_t bw[4] = {b.x, b.y, b.z, b.w};
    for (int j = 0; j < 16; j++) {
      o[j] = (float)(int8_t)((aw[j >> 2] >> (8 * (j & 3))) & 0xffu) * d;
      o[j + 16] = (float)(int8_t)((bw[j >> 2] >> (8 * (j & 3))) & 0xffu) * d;
    }
  }
}

// one thread per (n, m, b)
__global__ void block_isums_kernel(int wtype, PackedView w, const int8_t* __restrict__ codes, int32_t* __restrict__ out,
                                   int64_t M, int64_t N, int64_t nb) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * M * nb) return;
  const int64_t b = i % nb, m = (i / nb) % M, n = i / (nb * M);
  const u32x4* xq = reinterpret_cast<const u32x4*>(codes + (m * nb + b) * QK);
  const u32x4 xlo = xq[0], xhi = xq[1];
  const u32x4 w0 = w.q0[n * nb + b];
  u32x4 w1 = w0;
  int isum;
  if (wtype == MLLM_HIP_Q4_0) {
    const uint32_t xs[8] = {xlo.x, xlo.y, xlo.z, xlo.w, xhi.x, xhi.y, xhi.z, xhi.w};
    int s = 0;
    for (int j = 0; j < 8; j++) s = __builtin_amdgcn_sdot4((int)xs[j], 0x01010101, s, false);
    isum = block_dot<MLLM_HIP_Q4_0>(w0, w1, xlo, xhi, -8 * s);
  } else {
    w1 = w.q1[n * nb + b];
    isum = block_dot<MLLM_HIP_Q8_0>(w0, w1, xlo, xhi, 0);
  }
  out[i] = isum;
}

// plain copy / read kernels of known size: the yardstick for HBM counters and for the per-launch floor of a stream
// (buffer loads / stores: an out-of-range lane needs no branch, so all eight loads of a thread are in flight together;
// with `if (i < n)` around each load the compiler waits for every load before the next block)
__global__ __launch_bounds__(256) void probe_copy_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, size_t n16) {
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(src), 0, (uint32_t)(n16 * 16), 0x00020000);
  const uint32_t base = (uint32_t)(((size_t)blockIdx.x * 256 * 8 + threadIdx.x) * 16);
  u32x4 v[8];
#pragma unroll
  for (int u = 0; u < 8; u++) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, base + (uint32_t)u * 4096u, 0, 2);
  if (dst) {
    const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(dst, 0, (uint32_t)(n16 * 16), 0x00020000);
#pragma unroll
    for (int u = 0; u < 8; u++) __builtin_amdgcn_raw_buffer_store_b128(v[u], rd, base + (uint32_t)u * 4096u, 0, 0);
  } else {  // read only: keep the loads alive without writing
    uint32_t a = 0;
#pragma unroll
    for (int u = 0; u < 8; u++) a ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    __asm__ volatile("" ::"v"(a));
  }
}

// =========================================================================================================
// offline weight quantizers: fp32 rows -> reference blocks (one thread per block)
//   Q4_0  quantize_row_q4_0_reference, ggml/quantize/quantize_q4.cpp:33-68
//   Q8_0  quantize_row_q8_0, ggml/quantize/quantize_q8.cpp:106-190
// x86_store: write the scale field as the x86 build of the reference leaves it in a file, the half-precision encoding
// of the NUMBER equal to the fp16 pattern (mllm/core/DataTypes.hpp:26 with quantize.hpp:108-134).
// =========================================================================================================
__global__ void quantize_weight_blocks_kernel(int wtype, const float* __restrict__ w, uint16_t* __restrict__ blocks,
                                              int64_t nblocks, int x86_store) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nblocks) return;
  float v[32];
  load_block_f32(w, MLLM_HIP_F32, i * QK, v);
  if (wtype == MLLM_HIP_Q4_0) {
    float amax = 0.f, mx = 0.f;
#pragma unroll
    for (int j = 0; j < 32; j++)
      if (amax < fabsf(v[j])) {
        amax = fabsf(v[j]);
        mx = v[j];
      }
    float d = mx / -8.f;
    asm("" : "+v"(d));  // keep the product and the fp16 conversion apart: fused (v_fma_mixlo_f16 with a +0 addend) an
                          // all-zero block would store +0 where the reference stores -0
    const float id = d != 0.f ? 1.0f / d : 0.0f;
    uint16_t field = f32_to_f16bits(d);
    if (x86_store) field = f32_to_f16bits((float)field);
    uint16_t* y = blocks + i * 9;  // 18 bytes
    y[0] = field;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      uint32_t pair = 0;
#pragma unroll
      for (int b = 0; b < 2; b++) {
        const int e = 2 * j + b;
        int q0 = (int)(int8_t)(int)(v[e] * id + 8.5f);       // truncation toward zero, as the C cast
        int q1 = (int)(int8_t)(int)(v[16 + e] * id + 8.5f);
        q0 = min(15, q0);
        q1 = min(15, q1);
        pair |= (((uint32_t)q0 & 0xffu) | (((uint32_t)q1 << 4) & 0xf0u)) << (8 * b);
      }
      y[1 + j] = (uint16_t)pair;
    }
  } else {
    uint32_t q[8];
    int sum;
    uint16_t field = quantize_block_q8_0(v, q, sum);
    if (x86_store) field = f32_to_f16bits((float)field);
    uint16_t* y = blocks + i * 17;  // 34 bytes
    y[0] = field;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      y[1 + 2 * j] = (uint16_t)(q[j] & 0xffffu);
      y[2 + 2 * j] = (uint16_t)(q[j] >> 16);
    }
  }
}

// The quantized image of x the GEMV kernel copies into LDS when it does not quantize itself: for MT rows (rows m >= M
// zero) of nb blocks: 16-byte planes of elements 0..15 and 16..31, fp32 effective scales, -8 * sum(codes).
__global__ void quant_image_kernel(const void* __restrict__ x, int x_dtype, unsigned char* __restrict__ img, int M, int MT, int nb,
                                   int x86_scale) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;  // block index m * nb + b
  const int mnb = MT * nb;
  if (i >= mnb) return;
  uint32_t q[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  float d = 0.f;
  int sum = 0;
  if (i < M * nb) {
    float v[32];
    load_block_f32(x, x_dtype, (int64_t)i * QK, v);
    uint16_t bits = quantize_block_q8_0(v, q, sum);
    if (x86_scale) bits = x86_scale_bits(bits);
    d = f16bits_to_f32(bits);
  }
  u32x4* lo = reinterpret_cast<u32x4*>(img);
  u32x4* hi = lo + mnb;
  float* sd = reinterpret_cast<float*>(hi + mnb);
  int* sn = reinterpret_cast<int*>(sd + mnb);
  lo[i] = u32x4{q[0], q[1], q[2], q[3]};
  hi[i] = u32x4{q[4], q[5], q[6], q[7]};
  sd[i] = d;
  sn[i] = -8 * sum;
}

static int g_tune_G = 0, g_tune_R = 0, g_tune_NW = 0;

static GemvShape pick_shape(int MT, int64_t N, int nb) {
  // Measured on MI355X over the Qwen3-4B projection shapes: groups of 32 lanes with two rows each (512 contiguous
  // bytes per row segment) suit rows of 65..255 blocks; very long rows want the whole wave on one row and, because
  // every workgroup quantizes all of x, many waves per workgroup to share that work.
  GemvShape s;
  s.R = 2;
  s.NW = 4;
  if (nb >= 256) {
    s.G = 64;
    if (MT <= 2) s.R = 1;
    s.NW = 16;
    // one row per wave: the waves per workgroup only decide how many workgroups there are (not the arithmetic).  With sixteen
    // the 2560 rows of a down projection make 160 workgroups on 256 CUs; about one workgroup per CU measured best
    // (N = 2560, 304 blocks: 16 waves 5.84 us, 11 waves 5.27 us, 8 waves 6.4 us)
    if (MT <= 2) s.NW = (int)std::min<int64_t>(16, std::max<int64_t>(8, (N + 239) / 240));
  } else if (nb > 64) {
    s.G = 32;
  } else if (nb >= 16) {
    // (rows of exactly 64 blocks, 6144 of them: 16 lanes per row 3.48 us, 32 lanes 3.80)
    s.G = 16;
  } else {
    s.G = 8;
  }
  // four or eight activation rows (kernels built for at most eight waves), measured over the projection shapes with and
  // without a pre-quantized image: eight waves, whole-wave rows from 128 blocks on.  (16 lanes per row would gain 10 % on
  // the gate + up launch and lose as much on q + k + v; the shape is kept a function of the row length alone, so that a
  // projection gives the same bits whether it is launched alone or with its siblings.)
  if (MT >= 4) {
    s.R = 2;
    s.NW = 8;
    if (nb >= 128) s.G = 64;
  }
  if (g_tune_G) s.G = g_tune_G;
  if (g_tune_R) s.R = g_tune_R;
  if (g_tune_NW) s.NW = g_tune_NW;
  if (MT >= 4 && s.R < 2) s.R = 2;  // only these row counts are compiled for the wide tiles
  if (MT <= 2 && s.R > 2) s.R = 2;
  return s;
}

}  // namespace mllmhip

using namespace mllmhip;

// =========================================================================================================
// C ABI
// =========================================================================================================
MLLM_API const char* mllm_hip_version(void) { return "mllm-hip-qlinear 0.1 (gfx950)"; }

// Scratch of mllm_hip_linear_q_gemv_multi_static: the quantized image of up to eight activation rows, in device memory
// that belongs to the loaded code object (one copy per GPU, held until the process ends).  The name below is a host-side
// stand-in only; the device address is looked up once per device (static_scratch) and only that pointer is ever handed
// to a kernel.
constexpr int64_t GEMV_STATIC_MAX_K = 32768;
constexpr size_t GEMV_STATIC_BYTES = (size_t)8 * (GEMV_STATIC_MAX_K / QK) * 40;  // 320 KB
static __device__ __align__(256) unsigned char scratch[GEMV_STATIC_BYTES];
constexpr int MAX_DEVICES = 64;
static void* g_scratch_ptr[MAX_DEVICES];
static std::mutex g_scratch_mutex;

// device address of the scratch array on `device`, which must be the current device; 0 + *out on success
static int static_scratch(int device, void** out) {
  if (device < 0 || device >= MAX_DEVICES) return MLLM_HIP_E_NODEVICE;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    HIP_RET(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return MLLM_HIP_E_NODEVICE;
    g_scratch_ptr[device] = p;
  }
  *out = g_scratch_ptr[device];
  return 0;
}

MLLM_API int mllm_hip_init(int device) {
  int count = 0;
  HIP_RET(hipGetDeviceCount(&count));
  if (device < 0 || device >= count) return MLLM_HIP_E_NODEVICE;
  hipDeviceProp_t prop;
  HIP_RET(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return MLLM_HIP_E_NODEVICE;
  // the per-device address of the static scratch array, looked up with that device current and put back afterwards
  int cur = 0;
  HIP_RET(hipGetDevice(&cur));
  if (cur != device) HIP_RET(hipSetDevice(device));
  // ... and everything else a first launch would otherwise look up or set: the arrival counters of the K-slice kernels and
  // the dynamic-LDS limits of the matrix-core GEMV kernels, so that a launch under stream capture makes no such call
  void* p = nullptr;
  int rc = static_scratch(device, &p);
  if (!rc) rc = gemv_mfk_prepare_device();
  if (!rc) rc = gemv_mr_prepare_device();
  if (cur != device) HIP_RET(hipSetDevice(cur));
  return rc;
}

MLLM_API int mllm_hip_gemv_workspace_release(const void* workspace) {
  if (!workspace) return MLLM_HIP_E_BADARG;
  return gemv_mfk_release(workspace);
}

MLLM_API int mllm_hip_gemv_workspace_stats(int device, int* owned, int* capacity, long long* recycles, long long* refused) {
  if (device < 0) return MLLM_HIP_E_BADARG;
  gemv_mfk_stats(device, owned, capacity, recycles, refused);
  return 0;
}

// every fp32 bit pattern in [first, last] as amax: the scale and inverse scale of q8_scales against IEEE division
__global__ void probe_q8_scales_kernel(uint32_t first, uint32_t last, unsigned long long* mismatches) {
  unsigned long long bad = 0;
  const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t b = (uint64_t)first + (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; b <= last; b += step) {
    const float amax = __uint_as_float((uint32_t)b);
    float d, id;
    q8_scales(amax, d, id);
    const float dref = amax / 127.f, iref = (amax != 0.f) ? 127.f / amax : 0.f;
    // (a NaN has no single pattern: both sides NaN counts as equal)
    bad += !((__float_as_uint(d) == __float_as_uint(dref) || (d != d && dref != dref)) &&
             (__float_as_uint(id) == __float_as_uint(iref) || (id != id && iref != iref)));
  }
  if (bad) atomicAdd(mismatches, bad);
}

MLLM_API int mllm_hip_probe_q8_scales(uint32_t first_bits, uint32_t last_bits, unsigned long long* mismatches, void* stream) {
  if (!mismatches || first_bits > last_bits) return MLLM_HIP_E_BADARG;
  hipLaunchKernelGGL(probe_q8_scales_kernel, dim3(4096), dim3(256), 0, (hipStream_t)stream, first_bits, last_bits, mismatches);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_probe_copy(void* dst, const void* src, size_t bytes, void* stream) {
  if (!src || bytes == 0 || bytes % 16) return MLLM_HIP_E_BADARG;
  if (bytes >= ((size_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(src) % 16 || reinterpret_cast<uintptr_t>(dst) % 16) return MLLM_HIP_E_ALIGN;
  const size_t n16 = bytes / 16;
  hipLaunchKernelGGL(probe_copy_kernel, dim3((unsigned)((n16 + 2047) / 2048)), dim3(256), 0, (hipStream_t)stream, (u32x4*)dst,
                     (const u32x4*)src, n16);
  return (int)hipGetLastError();
}

namespace mllmhip { int g_gemv_defer = -1; }
static int g_gemv_path = 0;
static int g_gemv_many_rows = 1;  // 0: nine rows and more as groups of eight (comparison runs and tests)
// 0: by the number of rows; 1: always the vector-ALU kernel; 2: as 0 without the K-slices-as-workgroups form of the
// matrix-core kernel (comparison runs and tests)
MLLM_API int mllm_hip_gemv_set_path(int path) {
  if (path != 0 && path != 1 && path != 2 && path != 3) return MLLM_HIP_E_BADARG;
  g_gemv_many_rows = path != 3;  // 3: as 0, nine rows and more as groups of eight rows (the form without the many-row kernel)
  g_gemv_path = path == 3 ? 0 : path;
  return 0;
}

MLLM_API int mllm_hip_gemv_set_request_order(int mode) {
  if (mode < -1 || mode > 1) return MLLM_HIP_E_BADARG;
  mllmhip::g_gemv_defer = mode;
  return 0;
}

MLLM_API int mllm_hip_gemv_set_tuning(int lanes_per_row, int rows_per_group, int waves_per_wg) {
  auto ok = [](int v, std::initializer_list<int> allowed) {
    for (int a : allowed)
      if (v == a) return true;
    return false;
  };
  if (!ok(lanes_per_row, {0, 8, 16, 32, 64}) || !ok(rows_per_group, {0, 1, 2, 4}) || waves_per_wg < 0 || waves_per_wg > 16)
    return MLLM_HIP_E_BADARG;
  g_tune_G = lanes_per_row;
  g_tune_R = rows_per_group;
  g_tune_NW = waves_per_wg;
  return 0;
}

MLLM_API size_t mllm_hip_q_packed_bytes(int wtype, int64_t N, int64_t K) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || N <= 0 || K <= 0 || K % QK) return 0;
  return packed_bytes(wtype, N, K);
}

static int check_w(int wtype, const void* packed, int64_t N, int64_t K) {
  if (wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) return MLLM_HIP_E_BADARG;
  if (!packed || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (K % QK) return MLLM_HIP_E_SHAPE;
  if (N > INT32_MAX || K > INT32_MAX) return MLLM_HIP_E_SHAPE;
  if (N * (K / QK) * 16 >= ((int64_t)1 << 32)) return MLLM_HIP_E_SHAPE;  // one code plane must stay below 4 GiB (32-bit buffer offsets)
  if (reinterpret_cast<uintptr_t>(packed) % 16) return MLLM_HIP_E_ALIGN;
  return 0;
}

MLLM_API int mllm_hip_q_prepack(int wtype, const void* blocks, int weight_scale_mode, void* packed, int64_t N, int64_t K,
                                void* stream) {
  int rc = check_w(wtype, packed, N, K);
  if (rc) return rc;
  if (!blocks || (weight_scale_mode != MLLM_HIP_SCALE_IEEE && weight_scale_mode != MLLM_HIP_SCALE_X86_REF))
    return MLLM_HIP_E_BADARG;
  const int64_t nblocks = N * (K / QK);
  PackedView v = packed_view(wtype, packed, N, K);
  hipLaunchKernelGGL(prepack_kernel, dim3((unsigned)((nblocks + 255) / 256)), dim3(256), 0, (hipStream_t)stream, wtype,
                     (const uint8_t*)blocks, weight_scale_mode == MLLM_HIP_SCALE_X86_REF, const_cast<u32x4*>(v.q0),
                     const_cast<u32x4*>(v.q1), const_cast<uint16_t*>(v.d), nblocks, (int)(K / QK),
                     (int)scale_row_stride(K));
  return (int)hipGetLastError();
}

// the quantized image of one pass of eight rows: 40 bytes per block
static size_t gemv_image_bytes(int64_t K) { return (size_t)8 * (K / QK) * 40; }
// ... of all rows of a call with nine rows or more (the many-row kernel reads whole groups of 16 or 32 rows)
static size_t gemv_mr_image_bytes(int M, int64_t K) { return (size_t)gemv_mr_image_rows(M) * (K / QK) * 40; }

MLLM_API size_t mllm_hip_gemv_workspace_bytes(int M, int64_t K) {
  if (M < 1 || K <= 0 || K % QK) return 0;
  return gemv_image_bytes(K);
}

// image, then the partial sums of the K slices of eight rows (each part's rows rounded up to 16), for every group of eight
// rows
MLLM_API size_t mllm_hip_gemv_splitk_workspace_bytes(int M, int64_t K, int64_t N_total) {
  if (M < 1 || K <= 0 || K % QK || N_total <= 0) return 0;
  const size_t groups = (size_t)(M + 7) / 8;  // the groups of eight rows share a launch
  const size_t eight = gemv_image_bytes(K) + groups * (size_t)gemv_mfk_slices((int)(K / QK)) * 8 * (size_t)(N_total + 16 * GEMV_MAX_PARTS) * 4;
  if (M <= 8) return eight;
  // nine rows and more: the image of all rows (whole groups of 16 or 32), then every group's partial sums
  const size_t many = gemv_mr_image_bytes(M, K) + gemv_mr_part_bytes(M, (int)(K / QK), N_total + 16 * GEMV_MAX_PARTS);
  return std::max(eight, many);
}

// x_kind: MLLM_HIP_F32 / MLLM_HIP_BF16 activations, or MLLM_HIP_Q8_IMAGE: their quantized image (act_scale_mode unused)
static int gemv_multi_pass(int wtype, int nparts, const mllm_hip_gemv_part* parts, const float* const* residual, const void* x,
                           int x_dtype, int M, int64_t K, int act_scale_mode, void* workspace, size_t ws_bytes, void* stream);

// everything that can be refused without touching the device
static int gemv_check_args(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype, int M, int64_t K,
                           int act_scale_mode, const void* workspace) {
  if (nparts < 1 || nparts > GEMV_MAX_PARTS || !parts) return MLLM_HIP_E_BADARG;
  if (!x || (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16 && x_dtype != MLLM_HIP_Q8_IMAGE)) return MLLM_HIP_E_BADARG;
  if (act_scale_mode != MLLM_HIP_SCALE_IEEE && act_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (M < 1) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(workspace) % 16) return MLLM_HIP_E_ALIGN;
  for (int p = 0; p < nparts; p++) {
    RC_RET(check_w(wtype, parts[p].packed, parts[p].N, K));
    if (!parts[p].y) return MLLM_HIP_E_BADARG;
  }
  return 0;
}

// `rows` rows of raw activations as `groups` groups of eight (the last one may be shorter) in one launch of the K-slice kernel; MFK_NOT_TAKEN where that kernel does
// not apply (the caller then runs passes)
static int gemv_multi_groups(int wtype, int nparts, const mllm_hip_gemv_part* parts, const float* const* residual, const void* x,
                             int x_dtype, int rows, int groups, int64_t K, int act_scale_mode, void* workspace, size_t ws_bytes,
                             void* stream) {
  RC_RET(gemv_check_args(wtype, nparts, parts, x, x_dtype, rows, K, act_scale_mode, workspace));
  if (g_gemv_path == 1 || g_gemv_path == 2 || !workspace) return MFK_NOT_TAKEN;
  const size_t img = gemv_image_bytes(K);
  if (ws_bytes <= img) return MFK_NOT_TAKEN;
  GemvArgs a{};
  for (int p = 0; p < nparts; p++) {
    a.part[p].w = packed_view(wtype, parts[p].packed, parts[p].N, K);
    a.part[p].bias = parts[p].bias;
    a.part[p].residual = residual ? residual[p] : nullptr;
    a.part[p].y = parts[p].y;
    a.part[p].N = (int)parts[p].N;
  }
  a.nparts = nparts;
  a.x = x;
  a.M = rows;
  a.nb = (int)(K / QK);
  a.nbp = (int)scale_row_stride(K);
  a.x86_scale = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  return launch_gemv_mfk(wtype, x_dtype, 8, a, workspace, reinterpret_cast<char*>(workspace) + img, ws_bytes - img, g_tune_NW, g_tune_R,
                         (hipStream_t)stream, groups);
}

// More than eight rows of raw activations: passes of eight rows, each streaming the weights again (the same arithmetic row by
// row; up to about 32 rows this is faster than the matrix-core GEMM path, whose 128-row tiles leave most of the chip idle).
static int gemv_multi_impl(int wtype, int nparts, const mllm_hip_gemv_part* parts, const mllm_hip_gemv_fusion* fu, const void* x,
                           int x_dtype, int M, int64_t K, int act_scale_mode, void* workspace, size_t ws_bytes, void* stream) {
  const float* const* residual = fu ? fu->residual : nullptr;
  if (M <= 8 || x_dtype == MLLM_HIP_Q8_IMAGE || nparts < 1 || nparts > GEMV_MAX_PARTS || !parts || !x)
    return gemv_multi_pass(wtype, nparts, parts, residual, x, x_dtype, M, K, act_scale_mode, workspace, ws_bytes, stream);
  if (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16) return MLLM_HIP_E_BADARG;
  // Nine rows and more with room in the workspace for the image of all rows and the partial sums: one small launch quantizes
  // x once, one launch of the many-row kernel reads the weights once for up to 32 rows (qgemv_mr_kernel.h).
  if (g_gemv_many_rows && g_gemv_path == 0 && workspace && K > 0 && K % QK == 0 && ws_bytes >= gemv_mr_image_bytes(M, K)) {
    RC_RET(gemv_check_args(wtype, nparts, parts, x, x_dtype, M, K, act_scale_mode, workspace));
    const size_t img = gemv_mr_image_bytes(M, K);
    GemvArgs a{};
    for (int p = 0; p < nparts; p++) {
      a.part[p].w = packed_view(wtype, parts[p].packed, parts[p].N, K);
      a.part[p].bias = parts[p].bias;
      a.part[p].residual = residual ? residual[p] : nullptr;
      a.part[p].y = parts[p].y;
      a.part[p].N = (int)parts[p].N;
    }
    a.nparts = nparts;
    a.x = workspace;
    a.M = M;
    a.nb = (int)(K / QK);
    a.nbp = (int)scale_row_stride(K);
    a.x86_scale = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
    // (refusals are decided before anything is queued: the quantization launch goes out only when the kernel will follow)
    const int rows_img = gemv_mr_image_rows(M);
    const int64_t mnb = (int64_t)rows_img * a.nb;
    if (mnb < ((int64_t)1 << 31)) {
      int np = 0;
      for (int p = 0; p < nparts; p++) np += ((int)parts[p].N + 15) / 16 * 16;
      const size_t need = gemv_mr_part_bytes(M, a.nb, np);
      char* part = reinterpret_cast<char*>(workspace) + img;
      if (ws_bytes - img >= need &&
          launch_gemv_mr(wtype, a, workspace, part, ws_bytes - img, g_tune_NW, g_tune_R, (hipStream_t)stream, true) == 0) {
        hipLaunchKernelGGL(quant_image_kernel, dim3((unsigned)((mnb + 127) / 128)), dim3(128), 0, (hipStream_t)stream, x, x_dtype,
                           reinterpret_cast<unsigned char*>(workspace), M, rows_img, a.nb, a.x86_scale);
        const int rc = launch_gemv_mr(wtype, a, workspace, part, ws_bytes - img, g_tune_NW, g_tune_R, (hipStream_t)stream);
        if (rc != MFK_NOT_TAKEN) return rc;
      }
    }
  }
  const size_t xrow = (size_t)K * (x_dtype == MLLM_HIP_F32 ? 4 : 2);
  int m_first = 0;
  // Groups of eight rows in one launch of the K-slice kernel where it applies (room for every group's partial sums): the
  // groups share one pass over the weights.  A last group of three to seven rows joins them (the kernel it would run alone,
  // with fewer rows filled); one or two remaining rows stay a pass of their own, on the kernel one or two rows always take.
  // Row by row the bits of a call with that group alone.  Where all groups together are refused (arrival counters or room
  // for partial sums), halves of them are tried, and so on down to two groups per launch.
  const int rem = M % 8, rows = rem >= 3 ? M : M - rem;
  auto offset_parts = [&](int m0, mllm_hip_gemv_part* pp, const float** rr) {
    for (int p = 0; p < nparts; p++) {
      pp[p] = parts[p];
      if (pp[p].y) pp[p].y += (size_t)m0 * parts[p].N;
      rr[p] = (residual && residual[p]) ? residual[p] + (size_t)m0 * parts[p].N : nullptr;
    }
  };
  for (int chunk = (rows + 7) / 8; chunk >= 2 && m_first == 0; chunk = chunk > 2 ? (chunk + 1) / 2 : 0) {
    while (rows - m_first > 8) {  // at least two groups left
      const int r = rows - m_first < chunk * 8 ? rows - m_first : chunk * 8;
      mllm_hip_gemv_part pp[GEMV_MAX_PARTS];
      const float* rr[GEMV_MAX_PARTS];
      offset_parts(m_first, pp, rr);
      const int rc = gemv_multi_groups(wtype, nparts, pp, residual ? rr : nullptr, reinterpret_cast<const char*>(x) + (size_t)m_first * xrow,
                                       x_dtype, r, (r + 7) / 8, K, act_scale_mode, workspace, ws_bytes, stream);
      if (rc == MFK_NOT_TAKEN) break;  // (the first launch of a chunk size decides: the later ones are no larger)
      if (rc) return rc;
      m_first += r;
    }
  }
  for (int m0 = m_first; m0 < M; m0 += 8) {
    mllm_hip_gemv_part pp[GEMV_MAX_PARTS];
    const float* rr[GEMV_MAX_PARTS];
    for (int p = 0; p < nparts; p++) {
      pp[p] = parts[p];
      if (pp[p].y) pp[p].y += (size_t)m0 * parts[p].N;
      rr[p] = (residual && residual[p]) ? residual[p] + (size_t)m0 * parts[p].N : nullptr;
    }
    const int rc = gemv_multi_pass(wtype, nparts, pp, residual ? rr : nullptr, reinterpret_cast<const char*>(x) + (size_t)m0 * xrow, x_dtype,
                                   M - m0 < 8 ? M - m0 : 8, K, act_scale_mode, workspace, ws_bytes, stream);
    if (rc) return rc;
  }
  return 0;
}

static int gemv_multi_pass(int wtype, int nparts, const mllm_hip_gemv_part* parts, const float* const* residual, const void* x,
                           int x_dtype, int M, int64_t K, int act_scale_mode, void* workspace, size_t ws_bytes, void* stream) {
  RC_RET(gemv_check_args(wtype, nparts, parts, x, x_dtype, M, K, act_scale_mode, workspace));
  if (M > 8) return MLLM_HIP_E_SHAPE;
  GemvArgs a{};
  int64_t nmax = 0;
  for (int p = 0; p < nparts; p++) {
    a.part[p].w = packed_view(wtype, parts[p].packed, parts[p].N, K);
    a.part[p].bias = parts[p].bias;
    a.part[p].residual = residual ? residual[p] : nullptr;
    a.part[p].y = parts[p].y;
    a.part[p].N = (int)parts[p].N;
    nmax += parts[p].N;
  }
  a.nparts = nparts;
  a.x = x;
  a.M = M;
  a.nb = (int)(K / QK);
  a.nbp = (int)scale_row_stride(K);
  a.x86_scale = act_scale_mode == MLLM_HIP_SCALE_X86_REF;
  const int MT = M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : 8));
  GemvShape s = pick_shape(MT, nmax, a.nb);
  hipStream_t st = (hipStream_t)stream;
  // three or more rows: block sums on the matrix cores.  The rule looks at the weight type, the number of rows and the row
  // length, never at the number of weight rows: a matrix takes the same kernel alone and in a multi launch.
  // The form with K slices as workgroups (below) is the fastest for both formats wherever it can run (Q8_0 at four rows, 4B
  // layer: gate + up 12.2 us against 16.6 on the vector ALU, down 9.2 / 13.0, q+k+v 7.5 / 7.9, o 6.9 / 7.5).  Where it cannot
  // (no room for partial sums), Q4_0 and Q8_0 at five rows or more take the one-workgroup matrix-core kernel (as long as the
  // rows fit its LDS: 8 rows of 11 000 elements), Q8_0 at three or four rows the vector-ALU kernel (down 13.0 against 15.4).
  const bool mfk_rows = MT >= 4 && g_gemv_path != 1;
  const bool mfma_rows = mfk_rows && (wtype == MLLM_HIP_Q4_0 || MT == 8);
  const int waves = (g_tune_NW == 2 || g_tune_NW == 4 || g_tune_NW == 8) ? g_tune_NW : 0;
  // K slices as separate workgroups, each quantizing only its slice of x (one launch, same bits, no limit on the row length
  // from LDS): needs room for the slices' partial sums behind the image area of the workspace; falls through where that
  // room is missing
  // (Q8_0 at three or four rows only when the caller has given that room, also for a launch that would not need it: its
  // other kernel, the vector-ALU one, adds the blocks in another order, and the bits of a matrix must not depend on what
  // else is in the launch)
  const size_t img = gemv_image_bytes(K);
  char* part = (workspace && ws_bytes > img) ? reinterpret_cast<char*>(workspace) + img : nullptr;
  if (mfk_rows && g_gemv_path != 2 && (mfma_rows || part)) {
    const int rc = launch_gemv_mfk(wtype, x_dtype == MLLM_HIP_Q8_IMAGE ? GEMV_PREQ : x_dtype, MT, a, workspace, part,
                                   part ? ws_bytes - img : 0, g_tune_NW, g_tune_R, st);
    if (rc != MFK_NOT_TAKEN) return rc;
  }
  if (mfma_rows && gemv_mfma_fits(MT, a.nb)) {
    // quantizing x in every workgroup costs more than one more small launch that quantizes it once: with five to eight rows
    // always (q+k+v of the 4B layer at eight rows: 11.2 us against 7.5 + 2.4), with three or four from about 600 000
    // block-rows on (gate + up, down).  Same bits either way.
    if (x_dtype != MLLM_HIP_Q8_IMAGE && workspace && (MT == 8 || nmax * a.nb >= 600000)) {
      hipLaunchKernelGGL(quant_image_kernel, dim3((unsigned)((MT * a.nb + 127) / 128)), dim3(128), 0, st, x, x_dtype,
                         reinterpret_cast<unsigned char*>(workspace), M, MT, a.nb, a.x86_scale);
      a.x = workspace;
      return launch_gemv_mfma(wtype, GEMV_PREQ, MT, a, waves, g_tune_R, st);
    }
    return launch_gemv_mfma(wtype, x_dtype, MT, a, waves, g_tune_R, st);
  }
  if (x_dtype == MLLM_HIP_Q8_IMAGE) {
    if (!g_tune_NW && MT <= 2) s.NW = a.nb >= 256 ? 8 : 4;
    return wtype == MLLM_HIP_Q4_0 ? launch_gemv_q4_preq(a, MT, s, st) : launch_gemv_q8_preq(a, MT, s, st);
  }
  // several rows and a large launch (measured: from about 600 000 block-rows, i.e. gate + up and down of the 4B shapes):
  // quantizing x in every workgroup costs more than one more small launch
  if (workspace && M >= 3 && nmax * a.nb >= 600000) {
    // several rows: quantize once for all workgroups, then the GEMV copies the quantized image instead of quantizing
    const int mnb = MT * a.nb;
    hipLaunchKernelGGL(quant_image_kernel, dim3((unsigned)((mnb + 127) / 128)), dim3(128), 0, st, x, x_dtype,
                       reinterpret_cast<unsigned char*>(workspace), M, MT, a.nb, a.x86_scale);
    a.x = workspace;

    return wtype == MLLM_HIP_Q4_0 ? launch_gemv_q4_preq(a, MT, s, st) : launch_gemv_q8_preq(a, MT, s, st);
  }
  if (wtype == MLLM_HIP_Q4_0)
    return x_dtype == MLLM_HIP_F32 ? launch_gemv_q4_f32(a, MT, s, st) : launch_gemv_q4_bf16(a, MT, s, st);
  return x_dtype == MLLM_HIP_F32 ? launch_gemv_q8_f32(a, MT, s, st) : launch_gemv_q8_bf16(a, MT, s, st);
}

MLLM_API int mllm_hip_linear_q_gemv_multi_ws(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype,
                                             int M, int64_t K, int act_scale_mode, void* workspace, void* stream) {
  if (x_dtype == MLLM_HIP_Q8_IMAGE) return MLLM_HIP_E_BADARG;
  return gemv_multi_impl(wtype, nparts, parts, nullptr, x, x_dtype, M, K, act_scale_mode, workspace,
                         workspace && K > 0 && K % QK == 0 ? gemv_image_bytes(K) : 0, stream);
}

MLLM_API int mllm_hip_linear_q_gemv_multi_wsn(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype,
                                              int M, int64_t K, int act_scale_mode, void* workspace, size_t workspace_bytes,
                                              void* stream) {
  if (x_dtype == MLLM_HIP_Q8_IMAGE) return MLLM_HIP_E_BADARG;
  if (workspace && K > 0 && K % QK == 0 && workspace_bytes < gemv_image_bytes(K)) return MLLM_HIP_E_SHAPE;
  return gemv_multi_impl(wtype, nparts, parts, nullptr, x, x_dtype, M, K, act_scale_mode, workspace, workspace ? workspace_bytes : 0,
                         stream);
}

// The call above for callers that cannot allocate or pass a workspace: the image lives in the static scratch array of the
// current device.  Calls that overlap on one GPU (two streams) would share it and race.
MLLM_API int mllm_hip_linear_q_gemv_multi_static(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype,
                                                 int M, int64_t K, int act_scale_mode, void* stream) {
  if (x_dtype == MLLM_HIP_Q8_IMAGE) return MLLM_HIP_E_BADARG;
  RC_RET(gemv_check_args(wtype, nparts, parts, x, x_dtype, M, K, act_scale_mode, nullptr));
  if (K > GEMV_STATIC_MAX_K) return MLLM_HIP_E_SHAPE;  // the image of eight rows would not fit the array
  int dev = 0;
  HIP_RET(hipGetDevice(&dev));
  void* ws = nullptr;
  RC_RET(static_scratch(dev, &ws));
  return gemv_multi_impl(wtype, nparts, parts, nullptr, x, x_dtype, M, K, act_scale_mode, ws, GEMV_STATIC_BYTES, stream);
}

MLLM_API int mllm_hip_linear_q_gemv_fused(int wtype, int nparts, const mllm_hip_gemv_part* parts, const mllm_hip_gemv_fusion* fusion,
                                          const void* x, int x_kind, int M, int64_t K, int act_scale_mode, void* stream) {
  void* ws = fusion ? fusion->workspace : nullptr;
  size_t ws_bytes = 0;
  if (ws && K > 0 && K % QK == 0) {
    ws_bytes = fusion->workspace_bytes ? fusion->workspace_bytes : gemv_image_bytes(K);
    if (ws_bytes < gemv_image_bytes(K)) return MLLM_HIP_E_SHAPE;
  }
  return gemv_multi_impl(wtype, nparts, parts, fusion, x, x_kind, M, K, act_scale_mode, ws, ws_bytes, stream);
}

MLLM_API int mllm_hip_linear_q_gemv_multi(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype,
                                          int M, int64_t K, int act_scale_mode, void* stream) {
  return mllm_hip_linear_q_gemv_multi_ws(wtype, nparts, parts, x, x_dtype, M, K, act_scale_mode, nullptr, stream);
}

MLLM_API int mllm_hip_linear_q_gemv(int wtype, const void* packed, const void* x, int x_dtype, const float* bias,
                                    float* y, int M, int64_t N, int64_t K, int act_scale_mode, void* stream) {
  if (!y) return MLLM_HIP_E_BADARG;
  mllm_hip_gemv_part part{packed, bias, y, N};
  return mllm_hip_linear_q_gemv_multi(wtype, 1, &part, x, x_dtype, M, K, act_scale_mode, stream);
}

MLLM_API int mllm_hip_quantize_q8_0(const void* x, int x_dtype, int8_t* codes, uint16_t* d_bits, int64_t M, int64_t K,
                                    void* stream) {
  if (!x || !codes || !d_bits || M <= 0 || K <= 0 || (x_dtype != MLLM_HIP_F32 && x_dtype != MLLM_HIP_BF16))
    return MLLM_HIP_E_BADARG;
  if (K % QK) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(codes) % 16) return MLLM_HIP_E_ALIGN;
  const int64_t nblocks = M * (K / QK);
  hipLaunchKernelGGL(quantize_q8_0_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, (hipStream_t)stream, x,
                     x_dtype, codes, d_bits, nblocks);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_quantize_weight_blocks(int wtype, const float* w, void* blocks, int weight_scale_mode, int64_t N,
                                             int64_t K, void* stream) {
  if ((wtype != MLLM_HIP_Q4_0 && wtype != MLLM_HIP_Q8_0) || !w || !blocks || N <= 0 || K <= 0) return MLLM_HIP_E_BADARG;
  if (weight_scale_mode != MLLM_HIP_SCALE_IEEE && weight_scale_mode != MLLM_HIP_SCALE_X86_REF) return MLLM_HIP_E_BADARG;
  if (K % QK) return MLLM_HIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(w) % 16 || reinterpret_cast<uintptr_t>(blocks) % 2) return MLLM_HIP_E_ALIGN;
  const int64_t nblocks = N * (K / QK);
  hipLaunchKernelGGL(quantize_weight_blocks_kernel, dim3((unsigned)((nblocks + 127) / 128)), dim3(128), 0, (hipStream_t)stream,
                     wtype, w, reinterpret_cast<uint16_t*>(blocks), nblocks, weight_scale_mode == MLLM_HIP_SCALE_X86_REF);
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_q_dequantize(int wtype, const void* packed, float* w, int64_t N, int64_t K, void* stream) {
  int rc = check_w(wtype, packed, N, K);
  if (rc) return rc;
  if (!w) return MLLM_HIP_E_BADARG;
  const int64_t nblocks = N * (K / QK);
  hipLaunchKernelGGL(dequantize_kernel, dim3((unsigned)((nblocks + 255) / 256)), dim3(256), 0, (hipStream_t)stream, wtype,
                     packed_view(wtype, packed, N, K), w, nblocks, (int)(K / QK), (int)scale_row_stride(K));
  return (int)hipGetLastError();
}

MLLM_API int mllm_hip_q_block_isums(int wtype, const void* packed, const int8_t* codes, int32_t* isums, int64_t M,
                                    int64_t N, int64_t K, void* stream) {
  int rc = check_w(wtype, packed, N, K);
  if (rc) return rc;
  if (!codes || !isums || M <= 0) return MLLM_HIP_E_BADARG;
  if (reinterpret_cast<uintptr_t>(codes) % 16) return MLLM_HIP_E_ALIGN;
  const int64_t total = N * M * (K / QK);
  hipLaunchKernelGGL(block_isums_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, wtype,
                     packed_view(wtype, packed, N, K), codes, isums, M, N, K / QK);
  return (int)hipGetLastError();
}
