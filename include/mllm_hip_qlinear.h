/*
 * mllm_hip_qlinear.h -- C ABI of the MI355X (gfx950) quantized-Linear kernels.
 *
 * This is the seam a HIP backend's Linear / MatMul ops call: plain pointers and sizes, no C++ or torch types.
 * The C++ ops that sit on top of it (HipLinearOp etc., mllm_amd/csrc/host) mirror the reference's
 * BaseOp::{load,reshape,setup,forward} contract; this header is what their forward()/load() bind.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the name ends in _host
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); calls are asynchronous on it
 *   - return value: 0 on success; a positive value is a hipError_t; a negative value is MLLM_HIP_E_* below
 *   - matrices are row-major; a Linear weight is [N out_channels][K in_channels] like the reference's
 *     `weight_.view({out_channels, in_channels})` (mllm/backends/cpu/ops/LinearOp.cpp:13-40)
 *   - nothing here allocates device memory: workspaces are sized by a *_bytes() call and passed in
 */
#ifndef MLLM_HIP_QLINEAR_H
#define MLLM_HIP_QLINEAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLLM_HIP_E_BADARG (-1)   /* null pointer, negative size, unknown enum            */
#define MLLM_HIP_E_SHAPE (-2)    /* K not a multiple of the block / group size, M too big */
#define MLLM_HIP_E_ALIGN (-3)    /* pointer not aligned as documented                     */
#define MLLM_HIP_E_NODEVICE (-4) /* no gfx950 device / kernel image not loadable          */

/* weight block formats: mllm/core/DataTypes.hpp:110-121 (block_q4_0, 18 B), :164-170 (block_q8_0, 34 B) */
enum { MLLM_HIP_Q4_0 = 0, MLLM_HIP_Q8_0 = 1 };
/* super-block formats of 256 weights: mllm/core/DataTypes.hpp:139-147 (block_q4_K, 144 B), :153-160 (block_q6_K, 210 B);
 * only the mllm_hip_kq_* / mllm_hip_linear_kq entry points take them */
enum { MLLM_HIP_Q4_K = 2, MLLM_HIP_Q6_K = 3 };
/* activation element types */
enum { MLLM_HIP_F32 = 0, MLLM_HIP_BF16 = 1 };
/* instead of activations: their Q8_0 image as the decode GEMV reads it (mllm_hip_gemv_workspace_bytes, written by
 * mllm_hip_rmsnorm / mllm_hip_silu_mul); only where an entry point says so */
enum { MLLM_HIP_Q8_IMAGE = 2 };
/* IEEE half precision; only where an entry point says so (mllm_hip_matmul_batched) */
enum { MLLM_HIP_F16 = 3 };
/* How a block scale is read.
 *   IEEE     the 2-byte `d` field is an IEEE fp16 bit pattern (ARM builds of the reference, GGUF files)
 *   X86_REF  the x86 build of the reference: the field is a half-precision NUMBER equal to the bit pattern
 *            (mllm/core/DataTypes.hpp:26 with quantize.hpp:108-134), i.e. the pattern rounded to 11 significant
 *            bits.  For weights this selects how prepack decodes the stored field; for the activation scale
 *            computed inside the GEMV it selects whether that rounding is reproduced. */
enum { MLLM_HIP_SCALE_IEEE = 0, MLLM_HIP_SCALE_X86_REF = 1 };

/* library / device ------------------------------------------------------------------------------------ */
const char* mllm_hip_version(void);
/* Selects nothing and allocates nothing; returns 0 when device `device` is a gfx950 part and the kernels load.  Also looks up
 * the per-device addresses of the library's own device arrays and sets the kernels' LDS limits, so that later launches
 * (e.g. under stream capture) make no such runtime call. */
int mllm_hip_init(int device);

/* ---------------------------------------------------------------------------------------------------------
 * Q4_0 / Q8_0 Linear  (decode GEMV: one launch per eight rows)
 * replaces: CPULinearOp::forward -> ggml::mat_mul -> quantize_row_q8_0 + llamafile_sgemm
 *           mllm/backends/cpu/ops/LinearOp.cpp:100-128,282-288 ; ggml/matmul.cpp:148-206 ;
 *           ggml/quantize/quantize_q8.cpp:106-190 ; llamafile/llamafile_sgemm.cpp:697-743
 * ------------------------------------------------------------------------------------------------------- */

/* Size of the pre-packed (structure-of-arrays) form of an [N][K] weight: 16-byte code vectors first, fp16 scales after. */
size_t mllm_hip_q_packed_bytes(int wtype, int64_t N, int64_t K);

/* load()-time repack of reference blocks (array of 18 / 34-byte structs, row-major [N][K/32], on the device) into the
 * coalesced layout the kernels read.  `weight_scale_mode` says how the stored `d` field is to be decoded.
 * replaces: CPULinearOp::load (LinearOp.cpp:13-98) + the X2X host->device copy of the weight. */
int mllm_hip_q_prepack(int wtype, const void* blocks, int weight_scale_mode, void* packed, int64_t N, int64_t K,
                       void* stream);

/* y[m][n] = bias[n] + sum_b fp32(dW[n][b] * dX[m][b]) * int32(sum_32 qW * qX),   qX,dX = Q8_0 quantization of x[m]
 * x: [M][K] fp32 or bf16 (x_dtype), y: fp32 [M][N], bias: fp32 [N] or NULL, M >= 1, K % 32 == 0.
 * The activation quantization is fused into the kernel.  One launch serves up to eight rows; more rows run as passes of
 * eight over the same weights (the reference arithmetic for any number of rows; from nine rows on
 * mllm_hip_linear_q_gemm_short is faster).  A quantized image (MLLM_HIP_Q8_IMAGE) holds at most eight rows. */
int mllm_hip_linear_q_gemv(int wtype, const void* packed, const void* x, int x_dtype, const float* bias, float* y,
                           int M, int64_t N, int64_t K, int act_scale_mode, void* stream);

/* Up to four Linears that share the activations and K in ONE launch (sibling projections: q/k/v, gate/up).  Per part the
 * result equals mllm_hip_linear_q_gemv on that part; the point is fewer, larger launches (a decode-size matrix is a few
 * MB, far below what hides the fixed cost of a launch).  `parts` is a host array, read during the call. */
typedef struct {
  const void* packed; /* pre-packed [N][K] weight                      */
  const float* bias;  /* fp32 [N] or NULL                              */
  float* y;           /* fp32 [M][N]                                   */
  int64_t N;
} mllm_hip_gemv_part;
int mllm_hip_linear_q_gemv_multi(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype, int M,
                                 int64_t K, int act_scale_mode, void* stream);

/* The same with a workspace (mllm_hip_gemv_workspace_bytes): from three activation rows on, x is quantized once by a small
 * kernel into the workspace and the GEMV copies that image instead of quantizing x again in every workgroup (two
 * launches; same results bit for bit).  workspace may be NULL: then it is the call above. */
size_t mllm_hip_gemv_workspace_bytes(int M, int64_t K);
int mllm_hip_linear_q_gemv_multi_ws(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype, int M,
                                    int64_t K, int act_scale_mode, void* workspace, void* stream);

/* The same with a workspace of stated size.  With room behind the image for the partial sums of the K slices
 * (mllm_hip_gemv_splitk_workspace_bytes; N_total = the rows of all parts together) three to eight activation rows take one
 * launch whose workgroups each quantize only their K slice of x and whose slices meet through the workspace: same results
 * bit for bit, about two thirds of the time at eight rows.  With less room it is the call above.  Calls that may overlap
 * on a GPU need workspaces of their own.  The library keeps a block of arrival counters per workspace ADDRESS (1024 blocks
 * per GPU, in its own device memory, zero between launches): give an address back with mllm_hip_gemv_workspace_release when
 * the workspace is freed.  A caller that never does and walks through more than 1024 addresses pays one device
 * synchronisation per 1024 new addresses (the blocks are then handed out afresh; said once on stderr); only under stream
 * capture, where the device cannot be synchronised, does such a launch take the slower kernels instead.
 * With more than eight rows the groups of eight rows run in ONE such launch when the workspace has room for every
 * group's partial sums (mllm_hip_gemv_splitk_workspace_bytes with the real M): the groups share one pass over the
 * weights.  A last group of three to seven rows joins them; one or two remaining rows run as a pass of their own.  Row
 * by row the bits of a call with that group of rows alone. */
size_t mllm_hip_gemv_splitk_workspace_bytes(int M, int64_t K, int64_t N_total);
int mllm_hip_linear_q_gemv_multi_wsn(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype, int M,
                                     int64_t K, int act_scale_mode, void* workspace, size_t workspace_bytes, void* stream);

/* Gives the counter block of a workspace address back (call it where the workspace is freed, after the work that used it has
 * finished -- the rule of hipFree).  Unknown addresses are fine.  No counterpart in the reference. */
int mllm_hip_gemv_workspace_release(const void* workspace);
/* Counter blocks in use on `device`, their number, how often they were handed out afresh and how many launches were
 * refused the K-slice kernel (any pointer may be NULL).  For tests and monitoring. */
int mllm_hip_gemv_workspace_stats(int device, int* owned, int* capacity, long long* recycles, long long* refused);

/* mllm_hip_linear_q_gemv_multi_wsn without a workspace argument and without any allocation.  No counterpart in the
 * reference; it exists for callers that cannot allocate device memory or carry a workspace around: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The workspace is a static device array of the library
 * (327 680 bytes per GPU, held until the process ends: the quantized image of the activations and, where they fit behind
 * it, the partial sums of the K slices), whose per-device address mllm_hip_init(device) looks up together with the arrival
 * counters and the LDS limits of the kernels (otherwise the first call on a device does, which is not allowed during
 * capture).  Same arguments otherwise, same results bit for bit as that call
 * with a workspace of 327 680 bytes.  K <= 32768, else MLLM_HIP_E_SHAPE.  Every call on a GPU shares that GPU's array:
 * calls that overlap on one GPU (different streams) race; calls on one stream are ordered and safe. */
int mllm_hip_linear_q_gemv_multi_static(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype,
                                        int M, int64_t K, int act_scale_mode, void* stream);

/* The decode GEMV with its neighbours folded in (fusion may be NULL: the plain call).
 *   residual     NULL, or nparts pointers (each NULL or fp32 [M][N], may be the part's y): y = (bias + W x) + residual, the
 *                order of Linear followed by the elementwise add it replaces (Qwen3 decoder block: x = x + attn(...),
 *                x = x + mlp(...), mllm/models/qwen3/modeling_qwen3_fa2.hpp, Qwen3Decoder::forward).
 * x_kind: MLLM_HIP_F32 / MLLM_HIP_BF16 activations [M][K], or MLLM_HIP_Q8_IMAGE: the image a producer kernel
 * (mllm_hip_rmsnorm, mllm_hip_silu_mul) wrote for these M rows (act_scale_mode was applied there); the results are those
 * of the plain call on the tensor the producer stored, bit for bit, and the launch is 0.2 .. 0.8 us shorter because no
 * workgroup quantizes. */
typedef struct {
  const float* const* residual;
  void* workspace; /* NULL, or mllm_hip_gemv_workspace_bytes(M, K) bytes for raw activations: as in
                      mllm_hip_linear_q_gemv_multi_ws (same results bit for bit) */
  size_t workspace_bytes; /* 0 = mllm_hip_gemv_workspace_bytes(M, K); more (mllm_hip_gemv_splitk_workspace_bytes): as in
                             mllm_hip_linear_q_gemv_multi_wsn, for raw activations and for images alike */
} mllm_hip_gemv_fusion;
int mllm_hip_linear_q_gemv_fused(int wtype, int nparts, const mllm_hip_gemv_part* parts, const mllm_hip_gemv_fusion* fusion,
                                 const void* x, int x_kind, int M, int64_t K, int act_scale_mode, void* stream);

/* Same for any M: quantizes the activations with a stand-alone kernel into `workspace`
 * (mllm_hip_linear_q_workspace_bytes) and runs the tiled block-dot kernel; up to 16 rows run as passes of the eight-row
 * GEMV above instead (the same block arithmetic, the weights streamed once per eight rows).  Used by prefill and by the
 * MoE path. */
size_t mllm_hip_linear_q_workspace_bytes(int64_t M, int64_t K);
int mllm_hip_linear_q(int wtype, const void* packed, const void* x, int x_dtype, const float* bias, float* y,
                      int64_t M, int64_t N, int64_t K, int act_scale_mode, void* workspace, void* stream);

/* Stand-alone Q8_0 activation quantization (quantize_row_q8_0, AVX2 branch, quantize_q8.cpp:106-190).
 * codes int8 [M][K]; d_bits uint16 [M][K/32] = the fp16 pattern of amax/127 (before any x86 storage rounding). */
int mllm_hip_quantize_q8_0(const void* x, int x_dtype, int8_t* codes, uint16_t* d_bits, int64_t M, int64_t K,
                           void* stream);

/* The step in front of the path: the offline weight quantizer (tools/mllm-quantizer -> quantize_row_q4_0 /
 * quantize_row_q8_0, ggml/quantize/quantize_q4.cpp:33-68, quantize_q8.cpp:106-190).  w: fp32 [N][K] -> `blocks`: the
 * reference's array of 18 / 34-byte structs, row-major [N][K/32] (2-byte aligned), ready for the prepack calls.
 * weight_scale_mode says how the 2-byte scale field is STORED: IEEE = the fp16 pattern of the scale; X86_REF = what the
 * x86 build of the reference writes (the pattern as a half-precision number; pass the same mode to prepack to read it). */
int mllm_hip_quantize_weight_blocks(int wtype, const float* w, void* blocks, int weight_scale_mode, int64_t N, int64_t K,
                                    void* stream);

/* Parity probes (used by the tests, cheap enough to ship):
 *   dequantize: w[n][k] = code * fp32(scale)       dequantize_row_q4_0 / _q8_0 (quantize_q4.cpp:74-93, quantize_q8.cpp:197-211)
 *   block_isums: exact int32 dot product of every weight block with every activation block, [N][M][K/32] */
int mllm_hip_q_dequantize(int wtype, const void* packed, float* w, int64_t N, int64_t K, void* stream);
int mllm_hip_q_block_isums(int wtype, const void* packed, const int8_t* codes, int32_t* isums, int64_t M, int64_t N,
                           int64_t K, void* stream);

/* Measurement yardstick: copies `bytes` (a multiple of 16) from src to dst with 16-byte accesses, or only reads src when
 * dst is NULL.  Used to calibrate HBM traffic counters and to measure the fixed cost of a launch of a given size. */
int mllm_hip_probe_copy(void* dst, const void* src, size_t bytes, void* stream);

/* Parity probe for the two divisions of quantize_row_q8_0 (d = amax / 127, id = 127 / amax,
 * mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q8.cpp:106-190): the kernels for three to eight activation rows
 * form them from short sequences; this runs those sequences on every fp32 bit pattern in [first_bits, last_bits] taken as
 * amax and ADDS to *mismatches (device memory, 8 bytes, set to zero by the caller) the number of patterns on which either
 * result differs from IEEE division.  Zero over 0 .. 0x7fffffff. */
int mllm_hip_probe_q8_scales(uint32_t first_bits, uint32_t last_bits, unsigned long long* mismatches, void* stream);

/* GEMV launch-shape override for tuning sweeps: lanes per weight row (8/16/32/64), rows per lane group (1/2/4; the
 * three- to eight-row kernel with K slices as workgroups reads it as: 1 = keep rows of up to 128 blocks whole, 2 = always cut
 * them; the result bits are the same either way), waves per workgroup (1..16; that kernel takes 3..8); 0 restores the
 * built-in heuristic. */
int mllm_hip_gemv_set_tuning(int lanes_per_row, int rows_per_group, int waves_per_wg);
/* Three to eight rows take their block sums from the matrix cores (v_mfma_i32_16x16x32_i8, same fp32 arithmetic around
 * them); path = 1 keeps every launch on the vector-ALU kernel, path = 2 keeps the K slices of a row tile in one workgroup
 * (comparison runs), 0 restores the default. */
int mllm_hip_gemv_set_path(int path);
/* One or two rows: the kernel asks for the first block column of its weights at once and for the others of its first trip
 * behind the quantization of x (what all workgroups of a launch ask for at their start delays the activations each of
 * them needs first).  mode = -1: launches of 8 MB (Q8_0: 14 MB) and more with rows of 80 blocks and more, at two rows every
 * launch with such rows (the default); 0: never; 1: always (comparison runs and tests; the bits are the same). */
int mllm_hip_gemv_set_request_order(int mode);

/* ---------------------------------------------------------------------------------------------------------
 * Q4_0 / Q8_0 Linear and MoE expert FFN for many rows on the matrix cores
 * replaces: the same reference calls as mllm_hip_linear_q / mllm_hip_moe_ffn_q (the tinyBLAS gemm branch of
 *           llamafile_sgemm.cpp:697-743 for M > 1, and Qwen3MoE::moeInfer, modeling_qwen3_moe_fa2.hpp:175-238)
 * Arithmetic: the activations' Q8_0 quantization is the bit-exact one; both operands then carry their block scale,
 *   xh = fp16(dX * qX), wh = fp16(dW * qW), each product exact before its single rounding to fp16, and
 *   y[m][n] = sum_k xh[m][k] * wh[n][k] accumulates in fp32 in v_mfma_f32_32x32x16_f16.  The two roundings (relative
 *   error <= 2^-12 each) keep y within about 3e-4 relative L2 of the reference's fp32 block arithmetic; the entry points
 *   above keep that arithmetic itself.  |dX*qX| and |dW*qW| must stay below 65504.
 * Weights: "gemm-packed" once at load time from the reference blocks (codes in matrix-core operand order, N padded to
 *   32 and K to 128; same bytes per element as the blocks).
 * ------------------------------------------------------------------------------------------------------- */
size_t mllm_hip_q_gemm_packed_bytes(int wtype, int64_t N, int64_t K);
int mllm_hip_q_gemm_prepack(int wtype, const void* blocks, int weight_scale_mode, void* gemm_packed, int64_t N, int64_t K,
                            void* stream);
size_t mllm_hip_linear_q_gemm_workspace_bytes(int64_t M, int64_t K);
int mllm_hip_linear_q_gemm(int wtype, const void* gemm_packed, const void* x, int x_dtype, const float* bias, float* y,
                           int64_t M, int64_t N, int64_t K, int act_scale_mode, void* workspace, void* stream);
/* The same Linear for short batches (a prompt of up to 1024 rows): its M/128 x N/256 tiles would occupy a fraction of the chip,
 * so K is cut into up to eight ranges that run as separate workgroups and a small second kernel adds their partial results
 * in range order (deterministic).  Same operands and arithmetic; the fp32 sum over K is grouped by range.  Any M is
 * accepted (where cutting K does not pay it is the call above).  workspace: 256-byte aligned. */
size_t mllm_hip_linear_q_gemm_short_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mllm_hip_linear_q_gemm_short(int wtype, const void* gemm_packed, const void* x, int x_dtype, const float* bias, float* y,
                                 int64_t M, int64_t N, int64_t K, int act_scale_mode, void* workspace, void* stream);
/* Same arguments as mllm_hip_moe_ffn_q; the three expert arrays are E gemm-packed matrices back to back
 * (stride mllm_hip_q_gemm_packed_bytes). */
size_t mllm_hip_moe_gemm_workspace_bytes(int64_t T, int64_t H, int64_t I, int E, int k);
int mllm_hip_moe_ffn_q_gemm(int wtype, const void* gate_packed, const void* up_packed, const void* down_packed,
                            const void* x, int x_dtype, const int32_t* topk_ids, const float* topk_w, float* y, int64_t T,
                            int64_t H, int64_t I, int E, int k, int act_scale_mode, void* workspace, void* stream);

/* mllm_hip_moe_ffn_q_gemm has two forms.  0 (default): the reference's block arithmetic itself on the matrix cores: the
 * exact integer sum of every 32-element block (fp16 MFMAs on the integer codes), the exact product dW * dX of its two
 * scales (a third MFMA), one fp32 fused multiply-add per block; only the order in which blocks are added differs from the
 * CPU path; an expert's last tile of at most sixteen rows takes instructions of 16 rows (half the matrix time, same
 * bits).  1: fp16 operands with the block scales folded in as in mllm_hip_linear_q_gemm (about 2e-4 relative L2).
 * 2: as 0 with every tile in the 32-row form (comparison runs and tests). */
int mllm_hip_moe_gemm_set_path(int path);

/* ---------------------------------------------------------------------------------------------------------
 * W8A8 Linear (prefill): per-token dynamic int8 activations x int8 weights with per-channel scales
 * replaces: CompressedTensorsW8A8Int8Scheme.apply = per_token_quant_int8 + int8_scaled_mm
 *           pymllm/quantization/methods/compressed_tensors.py:450-468
 *           pymllm/quantization/kernels/int8_activation_triton.py:13-42 (rounding rule of
 *           pymllm/tests/bench_w8a8_activation_quant.py:20-26: half to even)
 *           mllm-kernel/mllm_kernel/cuda/csrc/gemm/int8/int8_scaled_mm_cutlass.cu:40-154
 * ------------------------------------------------------------------------------------------------------- */

/* q[m][k] = clamp(round_half_even(x[m][k] / scale[m]), -128, 127), scale[m] = max(amax|x[m]|, 1e-10) / 127.
 * x: [M][K] fp32 or bf16; q: int8 [M][K]; scale: fp32 [M]. */
int mllm_hip_per_token_quant_int8(const void* x, int x_dtype, int8_t* q, float* scale, int64_t M, int64_t K,
                                  void* stream);

/* acc[m][n] = sum_k xq[m][k] * W[n][k] (int32, exact);  out = bf16( float(acc) * (w_scale[n] * x_scale[m]) + bias[n] ).
 * xq int8 [M][K]; W int8 [N][K] (the checkpoint's [out, in] layout); w_scale fp32 [N]; x_scale fp32 [M]; bias fp32 [N] or
 * NULL; out_bf16 [M][N] and/or acc_out int32 [M][N] (either may be NULL, not both).  K % 16 == 0. */
int mllm_hip_w8a8_gemm(const int8_t* xq, const float* x_scale, const int8_t* W, const float* w_scale, const float* bias,
                       void* out_bf16, int32_t* acc_out, int64_t M, int64_t N, int64_t K, void* stream);

/* The two steps back to back; `workspace` (mllm_hip_w8a8_workspace_bytes) holds the quantized activations. */
size_t mllm_hip_w8a8_workspace_bytes(int64_t M, int64_t K);
int mllm_hip_w8a8_linear(const void* x, int x_dtype, const int8_t* W, const float* w_scale, const float* bias,
                         void* out_bf16, int64_t M, int64_t N, int64_t K, void* workspace, void* stream);

/* Weights repacked once after loading (the step the reference does in process_weights_after_loading,
 * pymllm/quantization/methods/compressed_tensors.py:429-448, where it re-lays the matrix for its CUTLASS kernel): the
 * [N][K] int8 matrix in the operand order of v_mfma_i32_32x32x32_i8, N padded to 32 and K to 128 with zeros, so that the
 * GEMM's waves fetch their weight operands from global memory with fully contiguous 1 KB loads and skip LDS for them.
 * Same arithmetic and results as mllm_hip_w8a8_gemm / _linear; this is the fast path for prefill-sized M. */
size_t mllm_hip_w8a8_packed_bytes(int64_t N, int64_t K);
int mllm_hip_w8a8_prepack(const int8_t* W, int64_t N, int64_t K, void* packed, void* stream);
int mllm_hip_w8a8_gemm_packed(const int8_t* xq, const float* x_scale, const void* W_packed, const float* w_scale,
                              const float* bias, void* out_bf16, int32_t* acc_out, int64_t M, int64_t N, int64_t K,
                              void* stream);
int mllm_hip_w8a8_linear_packed(const void* x, int x_dtype, const void* W_packed, const float* w_scale, const float* bias,
                                void* out_bf16, int64_t M, int64_t N, int64_t K, void* workspace, void* stream);

/* GEMM tile override for tuning sweeps (plain-layout entry points): 0 heuristic, 1 = 256x192, 2 = 128x128, 3 = 64x64
 * workgroup tiles through LDS, 4 = weight operands fetched straight from global memory (K % 128 == 0, else 2). */
int mllm_hip_w8a8_set_tuning(int tile);
/* Up to 32 tokens against prepacked weights run as GEMV kernels (one block row of the packed matrix per workgroup, its
 * waves striding over K; dot instructions up to four tokens, the matrix cores from five, 17 to 32 tokens only where N <= 8192;
 * same integer sums and epilogue, so the same bits as the tile kernels).  0 keeps the tile kernels also there (comparison runs and tests), 1 restores the default. */
int mllm_hip_w8a8_set_decode(int gemv);
/* The token count from which the decode kernels use the matrix cores (1..33, 33 = never: then up to eight tokens take the dot
 * form; default 5): comparison runs and tests.  No counterpart in the reference. */
int mllm_hip_w8a8_set_decode_mfma_from(int tokens);
/* Tile override for the weights-from-global kernel (packed entry points and tile 4 above): 0 heuristic, 1 = 128x384,
 * 2 = 64x384, 3 = 128x128, 4 = 64x128, 5 = 128x256. */
int mllm_hip_w8a8_nsplit_set_tuning(int tile);

/* ---------------------------------------------------------------------------------------------------------
 * W4A16 Linear (prefill): bf16 activations x uint4 weights, per-group fp16 scale and uint4 zero-point
 * replaces: AWQMarlinLinearMethod.apply -> gptq_marlin_gemm with zero points
 *           pymllm/quantization/methods/awq_marlin.py:274-449
 *           mllm-kernel/mllm_kernel/cuda/csrc/gemm/marlin/marlin_template.h:255-... , dequant.h:18-26
 * ------------------------------------------------------------------------------------------------------- */

/* C[m][n] = bf16( sum_k A[m][k] * w[n][k] + bias[n] ),  w[n][k] = bf16( (q[n][k] - zp[n][k/group]) * scale[n][k/group] ).
 * a_bf16 [M][K]; qw uint8 [N][K/2] (element 2j in the low nibble of byte j); scales fp16 [N][K/group];
 * zeros uint8 [N][ceil(K/group/2)] (group 2i in the low nibble of byte i); bias_bf16 [N] or NULL; c_bf16 [M][N].
 * group % 64 == 0 and K % group == 0 (128 in the checkpoints). */
int mllm_hip_w4a16_gemm(const void* a_bf16, const uint8_t* qw, const uint16_t* scales, const uint8_t* zeros,
                        const void* bias_bf16, void* c_bf16, int64_t M, int64_t N, int64_t K, int group, void* stream);

/* Parity probe: the dequantized weight table w_bf16 [N][K] exactly as the GEMM forms it. */
int mllm_hip_w4a16_dequantize(const uint8_t* qw, const uint16_t* scales, const uint8_t* zeros, void* w_bf16, int64_t N,
                              int64_t K, int group, void* stream);

/* AWQ checkpoint tensors -> the row-major tensors mllm_hip_w4a16_gemm / mllm_hip_w4a16_prepack take.
 * replaces: the unpacking half of AWQMarlinLinearMethod.process_weights_after_loading
 *           pymllm/quantization/methods/awq_marlin.py:366-410 (awq_marlin_repack, awq_to_marlin_zero_points :237-259,
 *           unpack_cols :202-213), mllm-kernel/mllm_kernel/cuda/csrc/gemm/marlin/awq_marlin_repack.cuh:106-126
 * qweight int32 [K][N/8] and qzeros int32 [K/group][N/8] hold eight 4-bit codes per dword, nibble position p = output
 * column 8 j + {0,2,4,6,1,3,5,7}[p]; scales fp16 [K/group][N] (create_weights, awq_marlin.py:284-364).
 * Writes qw uint8 [N][K/2], scales_out fp16 [N][K/group], zeros_out uint8 [N][ceil(K/group/2)].
 * N % 8 == 0, K % 8 == 0, K % group == 0. */
int mllm_hip_w4a16_from_awq(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales, int64_t N, int64_t K,
                            int group, uint8_t* qw, uint16_t* scales_out, uint8_t* zeros_out, void* stream);

/* GEMM tile override for tuning sweeps: 0 heuristic, 1 = 256x192, 2 = 128x128, 3 = 64x64 workgroup tiles. */
int mllm_hip_w4a16_set_tuning(int tile);

/* Weights repacked once after loading (the step the reference does in AWQMarlinLinearMethod.process_weights_after_loading,
 * pymllm/quantization/methods/awq_marlin.py:366-410: awq_marlin_repack, marlin_permute_scales,
 * awq_to_marlin_zero_points): the 4-bit codes in the operand order of v_mfma_f32_32x32x16_bf16 (N padded to 32, K to 128),
 * followed by one (scale, -zero_point * scale) fp32 pair per row and group.  The GEMM's waves then fetch their weight
 * operands from global memory with contiguous 1 KB loads and dequantize them in registers; same arithmetic
 * (w = bf16(fma(q, scale, -zp*scale)) = bf16((q - zp) * scale), fp32 accumulation) as mllm_hip_w4a16_gemm.
 * This is the fast path for prefill-sized M. */
size_t mllm_hip_w4a16_packed_bytes(int64_t N, int64_t K, int group);
int mllm_hip_w4a16_prepack(const uint8_t* qw, const uint16_t* scales, const uint8_t* zeros, int64_t N, int64_t K, int group,
                           void* packed, void* stream);
int mllm_hip_w4a16_gemm_packed(const void* a_bf16, const void* packed, const void* bias_bf16, void* c_bf16, int64_t M,
                               int64_t N, int64_t K, int group, void* stream);
/* Parity probe: the dequantized weight table w_bf16 [N][K] exactly as the packed GEMM forms it. */
int mllm_hip_w4a16_dequantize_packed(const void* packed, void* w_bf16, int64_t N, int64_t K, int group, void* stream);
/* Up to 32 tokens against packed weights run as GEMV kernels (a block row of the packed matrix per workgroup, waves striding
 * over K; weights rounded to bf16 and the sum + bias rounded to bf16 as in the tile kernels, fp32 sums in another order): fp32
 * FMAs for one token, the matrix cores from two (17 to 32 tokens only where N <= 8192).
 * 0 keeps the tile kernels also there (comparison runs and tests), 1 restores the default. */
int mllm_hip_w4a16_set_decode(int gemv);
/* The token count from which the decode kernels use the matrix cores (1..33, 33 = never; default 2): comparison runs and tests.
 * No counterpart in the reference. */
int mllm_hip_w4a16_set_decode_mfma_from(int tokens);
/* Tile override for the packed GEMM: 0 heuristic, 1 = 128x384, 2 = 64x384, 3 = 128x128, 4 = 64x128, 5 = 128x256;
 * + 16 switches off the half-height tiles that shorten a partly filled last round. */
int mllm_hip_w4a16_packed_set_tuning(int tile);

/* ---------------------------------------------------------------------------------------------------------
 * MoE expert FFN over expert-sorted tokens, Q4_0 / Q8_0 expert weights
 * replaces: Qwen3MoE::moeInfer + Qwen3MoeMLP::forward (one CPULinearOp::forward per expert and projection)
 *           mllm/models/qwen3_moe/modeling_qwen3_moe_fa2.hpp:98-100,175-238
 * ------------------------------------------------------------------------------------------------------- */

/* y[t] = sum_j topk_w[t][j] * down_e( silu(gate_e(x[t])) * up_e(x[t]) ),  e = topk_ids[t][j], j ascending.
 * Every projection is the block-quantized Linear above (activations re-quantized to Q8_0 in front of each one).
 * gate_packed / up_packed: E pre-packed [I][H] matrices back to back, expert e at + e * mllm_hip_q_packed_bytes(wtype, I, H);
 * down_packed: E pre-packed [H][I] matrices, stride mllm_hip_q_packed_bytes(wtype, H, I).
 * x [T][H] fp32 or bf16; topk_ids int32 [T][k] (entries outside [0, E) contribute nothing); topk_w fp32 [T][k];
 * y fp32 [T][H], 16-byte aligned like x and the workspace.  H % 32 == 0, I % 32 == 0, E <= 3072 (more: MLLM_HIP_E_SHAPE).  workspace: mllm_hip_moe_workspace_bytes. */
size_t mllm_hip_moe_workspace_bytes(int64_t T, int64_t H, int64_t I, int E, int k);
int mllm_hip_moe_ffn_q(int wtype, const void* gate_packed, const void* up_packed, const void* down_packed, const void* x,
                       int x_dtype, const int32_t* topk_ids, const float* topk_w, float* y, int64_t T, int64_t H,
                       int64_t I, int E, int k, int act_scale_mode, void* workspace, void* stream);

/* The same expert FFN with the experts in the super-block formats (MLLM_HIP_Q4_K / MLLM_HIP_Q6_K, the formats the shipped
 * Qwen3-MoE recipe quantizes to; activations Q8_K in front of every projection): gate_packed / up_packed / down_packed are E
 * matrices packed by mllm_hip_kq_prepack back to back, mllm_hip_kq_packed_bytes(wtype, I, H) resp. (wtype, H, I) apart.
 * H % 256 == 0, I % 256 == 0, T * k <= 65535, E <= 3072.  Up to one (token, expert) pair per expert (Q6_K: half) every pair runs as one
 * GEMV row (three or four launches; the decode form, an expert's weights are read once per pair that uses it).  Beyond that
 * the pairs are sorted by expert and run as tiles of eight rows on the matrix cores (the grouped form: x and h quantized
 * to Q8_K once, an expert's weights read once per eight pairs; seven launches), same arithmetic; from four pairs per expert
 * on (Q4_K) as tiles of 32 rows, the weights as the second operand of 32 x 32 matrix instructions (an expert's weights read
 * and unpacked once per 32 pairs), the same integers.
 * replaces: the same loop over experts with Q4_K / Q6_K Linear ops, modeling_qwen3_moe_fa2.hpp:98-100,175-238 */
size_t mllm_hip_moe_kq_workspace_bytes(int64_t T, int64_t H, int64_t I, int E, int k);
/* 0: by the number of pairs per expert (default); 1: always pairs as GEMV rows; 2: always tiles of eight rows; 3: always tiles
 * of 32 rows where the format has them (comparison runs and tests) */
int mllm_hip_moe_kq_set_path(int path);
int mllm_hip_moe_ffn_kq(int wtype, const void* gate_packed, const void* up_packed, const void* down_packed, const void* x,
                        int x_dtype, const int32_t* topk_ids, const float* topk_w, float* y, int64_t T, int64_t H, int64_t I,
                        int E, int k, void* workspace, void* stream);
/* The same with the down projections in the other super-block format: wtype for gate and up, wtype_down for down (the shipped
 * recipe quantizes the experts' gate / up to Q4_K and down to Q6_K, examples/qwen3_moe/quant_cfg_30B_q4_k.json; down_packed then
 * holds E matrices mllm_hip_kq_packed_bytes(wtype_down, H, I) apart).  Same workspace. */
int mllm_hip_moe_ffn_kq2(int wtype, int wtype_down, const void* gate_packed, const void* up_packed, const void* down_packed,
                         const void* x, int x_dtype, const int32_t* topk_ids, const float* topk_w, float* y, int64_t T, int64_t H,
                         int64_t I, int E, int k, void* workspace, void* stream);

/* mllm_hip_moe_ffn_q has three forms: every (token, expert) pair as GEMV rows (up to eight tokens or one pair per
 * expert), the pairs sorted by expert in tiles of eight rows that share the expert's weights (up to ten pairs per expert), and
 * the grouped 64-row tiles.  Tuning override: token counts up to which the first and the second run (0 = the rule above; 1
 * keeps a form to single-token calls).  No counterpart in the reference (its loop over experts is the same for any T). */
int mllm_hip_moe_set_tuning(int pair_tokens, int row_tokens);

/* Routing probe: tokens per expert (counts [E]), exclusive prefix (offsets [E+1]) and the flat (t*k + j) index at every
 * expert-sorted position (sorted_idx [T*k]); any output may be NULL.  workspace as for mllm_hip_moe_ffn_q.
 * replaces: the histogram + argsort at modeling_qwen3_moe_fa2.hpp:178-197 */
int mllm_hip_moe_route(const int32_t* topk_ids, int64_t T, int E, int k, int32_t* counts, int32_t* offsets,
                       int32_t* sorted_idx, void* workspace, void* stream);

/* ---------------------------------------------------------------------------------------------------------
 * Q4_K / Q6_K Linear (weights in super-blocks of 256, activations quantized to Q8_K inside the kernel)
 * replaces: CPULinearOp::forward -> ggml::mat_mul generic branch -> quantize_row_q8_K + vec_dot_q4_K_q8_K / vec_dot_q6_K_q8_K
 *           mllm/backends/cpu/kernels/common/ggml/matmul.cpp:147-189,300-360, vec_dot.cpp:498-560,955-1044,
 *           quantize/quantize_q8.cpp:215-248
 * ------------------------------------------------------------------------------------------------------- */

/* Load-time repack of reference blocks [N][K/256] (144 / 210 bytes each, any alignment) into planes of 16-byte records.
 * weight_scale_mode as for mllm_hip_q_prepack (how the fp16 fields d / dmin are read).  packed: 256-byte aligned. */
size_t mllm_hip_kq_packed_bytes(int wtype, int64_t N, int64_t K);
int mllm_hip_kq_prepack(int wtype, const void* blocks, int weight_scale_mode, void* packed, int64_t N, int64_t K, void* stream);

/* Offline K-quant quantizers on the GPU: w fp32 [N][K] (K % 256 == 0) -> reference super-blocks [N][K/256] of 144 (Q4_K) or 210
 * (Q6_K) bytes, byte for byte what the reference's converter writes.  weight_scale_mode says how the fp16 fields d / dmin are
 * stored and read back inside the quantizer (IEEE pattern, or the x86 build's form; see MLLM_HIP_SCALE_*).  `blocks`: 16-byte
 * aligned for Q4_K, 2-byte aligned for Q6_K.
 * replaces: quantize_row_q4_K / quantize_row_q6_K, mllm/backends/cpu/kernels/common/ggml/quantize/quantize_q4.cpp:97-168,184-282,325 ;
 *           quantize_q6.cpp:34-106,153 with quantize.hpp:261-325 ; called from tools/mllm-quantizer/schema/gguf.cpp:211-250 */
int mllm_hip_kq_quantize_weight_blocks(int wtype, const float* w, void* blocks, int weight_scale_mode, int64_t N, int64_t K,
                                       void* stream);
/* y[M][N] fp32 = x[M][K] (fp32 or bf16) * W^T + bias.  K % 256 == 0.  Up to eight rows per launch (decode); more rows run
 * as groups of eight, each streaming the weights again.  workspace (mllm_hip_kq_workspace_bytes, may be NULL): from three
 * rows on x is quantized once by a small kernel and the GEMV copies that image instead of quantizing in every workgroup
 * (same results bit for bit). */
size_t mllm_hip_kq_workspace_bytes(int64_t M, int64_t K);
/* Up to four Linears that share the activations and K in one launch (q/k/v, gate/up), as mllm_hip_linear_q_gemv_multi. */
int mllm_hip_linear_kq_multi(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype, int64_t M, int64_t K,
                             void* workspace, void* stream);
/* The same with the size of the workspace stated.  A workspace of mllm_hip_kq_workspace_bytes_n(M, K, N_total) bytes (N_total =
 * the sum of the parts' N) also has room for partial sums: launches of three to eight rows on the matrix-core kernels whose
 * rows have more than 2560 elements (Q6_K: more than 5120) then give every K slice a workgroup of its own, which quantizes
 * just its part of x (no separate quantization launch), and the slices meet in that room.  Same results bit for bit.  The arrival counters
 * belong to the workspace address as for mllm_hip_linear_q_gemv_multi: one launch at a time per workspace, and
 * mllm_hip_gemv_workspace_release before the memory is freed.  A smaller workspace (at least mllm_hip_kq_workspace_bytes)
 * is used as by mllm_hip_linear_kq_multi; less than that is MLLM_HIP_E_BADARG.
 * replaces: the same call sites as mllm_hip_linear_kq (the workspace has no counterpart in the reference). */
size_t mllm_hip_kq_workspace_bytes_n(int64_t M, int64_t K, int64_t N_total);
int mllm_hip_linear_kq_multi_ws(int wtype, int nparts, const mllm_hip_gemv_part* parts, const void* x, int x_dtype, int64_t M, int64_t K,
                                void* workspace, size_t workspace_bytes, void* stream);
/* Comparison runs and tests: mode 0 keeps the K slices of every launch in one workgroup even where the workspace has room
 * for partial sums; -1 (the default) lets them meet in global memory where a row has at least four slices (more than
 * 2560 elements; Q6_K: eight slices, more than 5120 elements), 1 from two slices on; waves_per_wg = row tiles of a workgroup in that form (1..8, 0 = chosen per launch).
 * Same results bit for bit in every setting. */
int mllm_hip_kq_set_slice_meeting(int mode, int waves_per_wg);
/* Tuning override of the decode GEMV: lanes per weight row (8/16/32/64), waves per workgroup (1/2/4), units a lane keeps in
 * flight per row (1/2/4; more than one only for up to two activation rows); 0 = heuristic. */
int mllm_hip_kq_set_tuning(int lanes_per_row, int waves_per_wg, int units_in_flight);
/* Three to eight rows take their sub-block sums from the matrix cores as the Q4_0 kernel of that kind does (Q4_K always, Q6_K
 * with five to eight rows, and with three or four rows of more than 4096 elements, where it measured faster).  path = 1 keeps every launch on the dot4
 * kernel, 2 uses the matrix-core kernels wherever they fit (comparison runs, tests), 0 restores the default. */
int mllm_hip_kq_set_path(int path);
int mllm_hip_linear_kq(int wtype, const void* packed, const void* x, int x_dtype, const float* bias, float* y, int64_t M, int64_t N,
                       int64_t K, void* workspace, void* stream);
/* Many rows (prefill) on the matrix cores, as mllm_hip_linear_q_gemm: fp16 operands with the scales folded in
 * (activations: the Q8_K round trip fp16(d * q), codes and d bit-exact; weights: fma(q, fp16(d*sc), -fp16(dmin*m)) for
 * Q4_K, (q - 32) * fp16(d*sc) for Q6_K, each rounded once), fp32 accumulation; within about 5e-4 relative L2 of the
 * reference's arithmetic (mllm_hip_linear_kq keeps that arithmetic itself).  Weights "gemm-packed" once at load time from
 * the reference blocks: Q4_K 0.5 byte + Q6_K 1 byte per weight, plus 8 bytes of scales per 64 weights. */
size_t mllm_hip_kq_gemm_packed_bytes(int wtype, int64_t N, int64_t K);
int mllm_hip_kq_gemm_prepack(int wtype, const void* blocks, int weight_scale_mode, void* gemm_packed, int64_t N, int64_t K,
                             void* stream);
size_t mllm_hip_linear_kq_gemm_workspace_bytes(int64_t M, int64_t K);
int mllm_hip_linear_kq_gemm(int wtype, const void* gemm_packed, const void* x, int x_dtype, const float* bias, float* y,
                            int64_t M, int64_t N, int64_t K, void* workspace, void* stream);
/* The same for short batches, as mllm_hip_linear_q_gemm_short. */
size_t mllm_hip_linear_kq_gemm_short_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mllm_hip_linear_kq_gemm_short(int wtype, const void* gemm_packed, const void* x, int x_dtype, const float* bias, float* y,
                                  int64_t M, int64_t N, int64_t K, void* workspace, void* stream);
/* Parity probes.  Dequantized weights fp32 [N][K] (dequantize_row_q4_K / _q6_K, quantize_q4.cpp:284-312, quantize_q6.cpp:108-133);
 * Q8_K activation quantization: codes int8 [M][K], d fp32 [M][K/256], sums of 16 codes int16 [M][K/16]. */
int mllm_hip_kq_dequantize(int wtype, const void* packed, float* w, int64_t N, int64_t K, void* stream);
int mllm_hip_quantize_q8_K(const void* x, int x_dtype, int8_t* codes, float* d, int16_t* bsums, int64_t M, int64_t K, void* stream);

/* Decode MLP front half in ONE launch: h = silu(gate(x)) * up(x), M <= 8 rows, Q4_0 / Q8_0 weights [I][H].
 *   replaces: Qwen3MLP::forward, mllm/models/qwen3/modeling_qwen3_fa2.hpp:85-92 (gate_proj, SiLU, up_proj, product: two
 *             CPULinearOp::forward, CPUSiLUOp, CPUMulOp), fp32 tensors in between.
 * x_kind as for mllm_hip_linear_q_gemv_fused (F32 / BF16 activations [M][H], or the Q8_0 image of M rows).  h (fp32
 * [M][I], may be NULL) and/or h_image (may be NULL; the Q8_0 image of h for the down projection, size
 * mllm_hip_gemv_workspace_bytes(M, I)) receive the result.  I % 32 == 0, H % 32 == 0.  SiLU follows mllm_hip_set_exp_mode.
 * The gate and up values never reach memory; results agree with the separate calls to fp32 rounding of the row sums. */
int mllm_hip_mlp_gate_up_q(int wtype, const void* gate_packed, const void* up_packed, const void* x, int x_kind, float* h,
                           void* h_image, int M, int64_t I, int64_t H, int act_scale_mode, void* stream);
/* Tuning override of that launch: block columns of a weight row a lane keeps in flight (2..5); 0 = heuristic. */
int mllm_hip_mlp_set_tuning(int units_in_flight);

/* ---------------------------------------------------------------------------------------------------------
 * The operators either side of a quantized Linear in a decoder layer.  dtype: MLLM_HIP_F32 or MLLM_HIP_BF16 (arithmetic
 * in fp32, results rounded to the tensor's type).  All pointers 16-byte aligned, element counts multiples of 8.
 * q_image (may be NULL; rows <= 8, D % 32 == 0): also writes the Q8_0 image of the rows just stored, for
 * mllm_hip_linear_q_gemv_fused(..., MLLM_HIP_Q8_IMAGE, ...); size mllm_hip_gemv_workspace_bytes(rows, D).
 * ------------------------------------------------------------------------------------------------------- */

/* y = x * (w * rms) [x * ((w + 1) * rms) with add_unit_offset], rms = 1 / sqrt(mean(x^2) + epsilon); weight fp32 [D].
 * replaces: CPURMSNormOp::forward -> x86::rmsnorm_fp32  mllm/backends/cpu/ops/RMSNormOp.cpp:14-96,
 *           mllm/backends/cpu/kernels/x86/rmsnorm.cpp:17-52.  D <= 16384. */
int mllm_hip_rmsnorm(const void* x, int dtype, const float* weight, void* y, int64_t rows, int64_t D, float epsilon,
                     int add_unit_offset, void* q_image, int act_scale_mode, void* stream);

/* y = x * (1 / (1 + exp(-x))) with the reference's polynomial exp.
 * replaces: CPUSiLUOp::forward -> x86::silu_fp32  mllm/backends/cpu/kernels/x86/silu.cpp:16-56, math.hpp:19-72 */
int mllm_hip_silu(const void* x, void* y, int dtype, int64_t n, void* stream);
/* y = a + b, y = a * b over [rows][D] (same shapes, no broadcasting).
 * replaces: CPUAddOp / CPUMulOp::forward  mllm/backends/cpu/ops/ElewiseOps.cpp */
int mllm_hip_add(const void* a, const void* b, void* y, int dtype, int64_t rows, int64_t D, void* q_image, int act_scale_mode,
                 void* stream);
int mllm_hip_mul(const void* a, const void* b, void* y, int dtype, int64_t rows, int64_t D, void* q_image, int act_scale_mode,
                 void* stream);
/* y = silu(gate) * up in one pass (the SiLU result is rounded to the tensor's type before the product, as when the two
 * operators run one after the other).  replaces: silu_(gate) then x * y  mllm/models/qwen3/modeling_qwen3_fa2.hpp:87-90 */
int mllm_hip_silu_mul(const void* gate, const void* up, void* y, int dtype, int64_t rows, int64_t D, void* q_image,
                      int act_scale_mode, void* stream);
/* 0 (default): exp as the reference's x86 kernels compute it (math.hpp:19-72); 1: expf.  Process-wide; affects SiLU,
 * softmax and the MoE gate. */
int mllm_hip_set_exp_mode(int accurate);

/* softmax over the last axis of fp32 [rows][len].
 * replaces: CPUSoftmaxOp::forward -> x86::softmax_v1_fp32  mllm/backends/cpu/kernels/x86/softmax.cpp:18-76 */
int mllm_hip_softmax(const float* x, float* y, int64_t rows, int64_t len, void* stream);
/* k largest (or smallest) of every row of fp32 [rows][len]: values fp32 [rows][k], indices int32 [rows][k]; sorted != 0:
 * by value, else by index; equal values are taken lowest index first.
 * replaces: CPUTopKOp::forward  mllm/backends/cpu/ops/TopKOp.cpp:20-72 */
int mllm_hip_topk(const float* x, float* values, int32_t* indices, int64_t rows, int64_t len, int k, int largest, int sorted,
                  void* stream);
/* The MoE gate: scores = softmax(x . W^T) in fp32, the k largest per token in index order, weights divided by their sum
 * when norm_topk_prob.  x [M][H] fp32 or bf16; gate_weight fp32 [E][H]; topk_ids int32 [M][k]; topk_weights fp32 [M][k];
 * scores fp32 [M][E] or NULL.  H % 8 == 0.  With a scores buffer the call is two launches -- the logits with the experts
 * spread over the grid (the buffer holds them in between), then one wave per token for softmax and selection -- which is
 * what a decode token wants (1 MB of gate weights for 128 experts: 6 us against 26 through the single workgroup of the
 * one-launch form, which callers without a scores buffer get).  Same logits, scores and selection either way.
 * replaces: MoEGate::forward  mllm/models/qwen3_moe/modeling_qwen3_moe_fa2.hpp:121-139 */
int mllm_hip_moe_gate(const void* x, int x_dtype, const float* gate_weight, int32_t* topk_ids, float* topk_weights, float* scores,
                      int64_t M, int64_t H, int64_t E, int k, int norm_topk_prob, void* stream);
/* 0: the one-launch form also where a scores buffer is given (comparison runs and tests); 1: the default */
int mllm_hip_moe_gate_set_form(int two_launches);

/* ---------------------------------------------------------------------------------------------------------
 * Activation x activation MatMul on the matrix cores (the backend's kMatMul slot; not a quantized path)
 * replaces: CPUMatMulOp::forward  mllm/backends/cpu/ops/MatMulOp.cpp:19-90 (shapes :30-44, default kernel choice :47-61)
 * C[b][M][N] = op(A[b]) * op(B[b]), op(X) = X or X^T; A[b] is [M][K] ([K][M] when transposed), B[b] is [K][N] ([N][K]
 * when transposed).  dtype MLLM_HIP_F32, MLLM_HIP_BF16 or MLLM_HIP_F16 for all three tensors; products are exact and
 * summed in fp32, 16-bit results are rounded once to nearest even.  Batch entry b starts stride_x * b elements after
 * entry 0 (stride_b = 0 multiplies every A[b] by the same B); the whole batch is one launch.
 * ------------------------------------------------------------------------------------------------------- */
int mllm_hip_matmul_batched(const void* A, const void* B, void* C, int dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                            int64_t stride_a, int64_t stride_b, int64_t stride_c, int transpose_a, int transpose_b,
                            void* stream);
/* batch = 1, fp32 */
int mllm_hip_matmul_f32(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K, int transpose_a,
                        int transpose_b, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MLLM_HIP_QLINEAR_H */
