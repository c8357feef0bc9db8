// Q4_K / Q6_K experts with many rows each: tiles of 32 expert-sorted rows on the matrix cores, the reference's integer
// arithmetic kept exact.
//
// The decode kernels (kquant.hip) stream an expert's weights once per eight rows.  With tens of rows per expert the same
// weights would be streamed several times and every eight rows pay the whole unpacking, so here a workgroup takes 32 rows x
// 128 (two matrices) or 256 (one matrix) channels and walks K one super-block of 256 elements at a time:
//   * activations: the Q8_K image (codes, sums of 16, scale per super-block; bit-exact, written once per call by
//     quantize_q8k_kernel) goes through LDS, 32 rows x one super-block per stage, double-buffered;
//   * weights: from the packed planes of mllm_hip_kq_prepack into registers, one super-block ahead, as whole 128-byte
//     lines (a load instruction = 8 channels x the 128 bytes of their super-block; one channel per lane and 16 bytes of it,
//     the operand's own layout, touches 32 lines per instruction and was bound by the L1's tag rate: gate + up at 512 tokens
//     110 us), then through a 4.5 KB LDS patch that belongs to the wave into the operand layout.  The weights are the SECOND
//     operand of the matrix instruction, so a lane owns ONE channel (lane % 32) and sixteen rows: the channel's sub-block
//     scales are then per-lane values and scaling a sub-block's sums costs one integer multiply-add per output;
//   * Q4_K: per sub-block of 32 elements one v_mfma_i32_32x32x32_i8 (codes 0..15 as they are: the format's minimum is a
//     separate term), I += sc * T in int32; the minimum term sum_j m_j * bsum_j is one v_mfma_f32_32x32x16_f16 per super-block
//     on the sixteen sums of 16 as fp16 integers (at most 2048: exact) and the 6-bit minima (every product and sum below
//     2^24: exact); per super-block and output then y += (dX * d) * float(I) and y += -(dX * dmin) * float(M), the products
//     and the FMAs of vec_dot_q4_K_q8_K (mllm/backends/cpu/kernels/common/ggml/vec_dot.cpp:498-560).
//   * Q6_K: the scales belong to groups of 16 elements, so a group is one v_mfma_i32_32x32x16_i8; the 6-bit codes enter
//     unsigned (low nibble | two high bits << 4, three to four operations per four codes) and the format's offset of 32 leaves
//     through the sums of 16: I = sum_g sc_g * T_g - 32 * sum_g sc_g * bsum_g, the second sum again one fp16 instruction per
//     super-block (at most 128 * 2048 * 16: exact); y += (dX * d) * float(I), vec_dot_q6_K_q8_K (vec_dot.cpp:955-1044).
// What differs from the CPU path is the order of the fp32 additions only (the CPU keeps eight lanes per output and a
// separate accumulator for the minimum term; here one accumulator per output takes both terms super-block by super-block).
#include <type_traits>

#include "kquant_layout.h"

namespace mllmhip {

typedef int kx4i __attribute__((ext_vector_type(4)));
typedef int kx16i __attribute__((ext_vector_type(16)));
typedef float kx16f __attribute__((ext_vector_type(16)));
typedef _Float16 kxh8 __attribute__((ext_vector_type(8)));

struct KXArgs {
  const char* W[2];      // packed experts (mllm_hip_kq_prepack layout), expert e at W[w] + e * estride
  size_t estride;
  const char* image;     // Q8_K image of the activations: codes [img_rows][K], sums of 16 int16 [img_rows][K/16], d [img_rows][K/256]
  int img_rows;
  const int* row_ids;    // image row of sorted position pos: row_ids[pos] / row_div (null: pos)
  int row_div;
  const int* out_ids;    // output row of sorted position pos (null: pos)
  float* y[2];           // fp32 [..][N] per matrix
  const int* tile_expert;
  const int* tile_row0;
  const int* tile_rows;
  const int* ntiles;
  int N, K;
  int silu_mul;          // two matrices: write silu(y0) * y1 to y[0] instead of both results (the expert MLP's product)
  int exp_accurate;      // expf instead of the reference's polynomial (mllm_hip_set_exp_mode)
};

constexpr int KX_LDC = 256 + 16;                           // code row of a super-block, padded: 16-byte reads of 16 rows hit 16 bank groups
constexpr int KX_BS = 48;                                   // the row's sixteen sums of 16 as fp16, padded likewise
constexpr int KX_OFF_BS = 32 * KX_LDC;
constexpr int KX_OFF_DX = KX_OFF_BS + 32 * KX_BS;
constexpr int KX_STAGE = KX_OFF_DX + 32 * 4;
constexpr int KX_WROW = 128 + 16;                           // a channel's line in the wave's patch, padded likewise
constexpr int KX_PATCH = 32 * KX_WROW;
constexpr int KX6_WROW = 128 + 64 + 16;                     // Q6_K: low nibbles, high bit pairs, padding
constexpr int KX6_PATCH = 32 * KX6_WROW;
constexpr int KX_GROUP = 8;                                 // tiles per group of work items (see the kernel)

// NW matrices (gate and up share the activations) x TN column tiles of 32 channels per wave
template <int WT, int NW, int TN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void kx_kernel(KXArgs a) {
  constexpr bool K4 = WT == MLLM_HIP_Q4_K;
  extern __shared__ __align__(16) unsigned char smem[];
  // Work items in groups of KX_GROUP tiles (list order: an expert's tiles are neighbours) x all column blocks, inside a group
  // the tile index fastest.  Workgroup L runs on XCD L % 8, and every XCD has its own L2: XCD x takes a contiguous eighth of
  // the work items, so that the tiles of one expert and column block, which read the same weights, and the column blocks of
  // one tile, which read the same activation rows, run on one XCD at about the same time.
  const int nt = min(a.ntiles[0], (int)gridDim.x), ny = (int)gridDim.y;
  const int L = (int)(blockIdx.x + gridDim.x * blockIdx.y);
  const int nw = nt * ny, base = nw >> 3, rem = nw & 7;  // XCD x takes base + (x < rem) items
  const int xcd = L & 7, seq = L >> 3;
  if (seq >= base + (xcd < rem)) return;
  const int wi = xcd * base + min(xcd, rem) + seq;
  const int per = KX_GROUP * ny, grp = wi / per, r0 = wi - grp * per;
  const int gt = min(KX_GROUP, nt - grp * KX_GROUP);  // tiles in this group (the last one may be short)
  const int by = r0 / gt, t = grp * KX_GROUP + (r0 - by * gt);
  const int e = a.tile_expert[t], row0 = a.tile_row0[t], rows = a.tile_rows[t];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c32 = lane & 31, hi = lane >> 5;
  const int nsb = a.K / QK_K;
  const int n0 = by * (128 * TN) + wave * (32 * TN);

  // ---- the image: this thread's pieces of a stage ---------------------------------------------------------------------------
  const size_t img_codes = (size_t)a.img_rows * a.K, img_bs = (size_t)a.img_rows * (a.K / 16) * 2;
  const __amdgpu_buffer_rsrc_t rI = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a.image), 0,
                                                                    (uint32_t)(img_codes + img_bs + (size_t)a.img_rows * nsb * 4), 0x00020000);
  auto image_row = [&](int m) {  // rows past the tile repeat its last row; their results are dropped
    const int pos = row0 + min(m, rows - 1);
    return a.row_ids ? a.row_ids[pos] / a.row_div : pos;
  };
  // codes: chunk c = tid + 256 i of 16 bytes: row c / 16, column c % 16
  uint32_t offC[2];
#pragma unroll
  for (int i = 0; i < 2; i++) offC[i] = (uint32_t)((size_t)image_row((tid >> 4) + 16 * i) * a.K + (tid & 15) * 16);
  // sums of 16: threads 0..63, row tid / 2, eight sums each; scale: threads 64..95, one row each
  uint32_t offB = 0xffffffffu;
  if (tid < 64) offB = (uint32_t)(img_codes + ((size_t)image_row(tid >> 1) * (a.K / 16) + (tid & 1) * 8) * 2);
  else if (tid < 96) offB = (uint32_t)(img_codes + img_bs + (size_t)image_row(tid - 64) * nsb * 4);
  u32x4 gc[2], gb;
  auto load_stage = [&](int sb) {
    const bool ok = sb < nsb;
#pragma unroll
    for (int i = 0; i < 2; i++) gc[i] = __builtin_amdgcn_raw_buffer_load_b128(rI, ok ? offC[i] : 0xffffffffu, sb * 256, 0);
    if (tid < 64) gb = __builtin_amdgcn_raw_buffer_load_b128(rI, ok ? offB : 0xffffffffu, sb * 32, 0);
    else if (tid < 96) gb.x = __builtin_amdgcn_raw_buffer_load_b32(rI, ok ? offB : 0xffffffffu, sb * 4, 0);
  };
  auto store_stage = [&](int buf) {
    unsigned char* st = smem + buf * KX_STAGE;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      // Q6_K reads this stage (and its patch) 8 bytes per lane: rows r and r + 16 would meet in the same banks, so rows 16..31
      // keep the two halves of every 16-byte piece swapped (the reads swap them back by address)
      const u32x4 v = (!K4 && i == 1) ? u32x4{gc[i].z, gc[i].w, gc[i].x, gc[i].y} : gc[i];
      *reinterpret_cast<u32x4*>(st + ((tid >> 4) + 16 * i) * KX_LDC + (tid & 15) * 16) = v;
    }
    if (tid < 64) {
      // int16 sums (at most 16 * 128 in magnitude) as fp16 integers: exact
      const uint32_t w[4] = {gb.x, gb.y, gb.z, gb.w};
      uint32_t o[4];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const _Float16 lo = (_Float16)(short)(w[q] & 0xffffu), hi16 = (_Float16)(short)(w[q] >> 16);
        o[q] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi16) << 16);
      }
      *reinterpret_cast<u32x4*>(st + KX_OFF_BS + (tid >> 1) * KX_BS + (tid & 1) * 16) = u32x4{o[0], o[1], o[2], o[3]};
    } else if (tid < 96) {
      *reinterpret_cast<uint32_t*>(st + KX_OFF_DX + (tid - 64) * 4) = gb.x;
    }
  };

  // ---- the weights: lane (channel c32 of a column tile, K half hi) -----------------------------------------------------------
  const size_t sbt = (size_t)a.N * nsb;
  const uint32_t oH = (uint32_t)kq_plane(sbt * 128);                            // Q6_K: high bit pairs
  const uint32_t oS = K4 ? oH : oH + (uint32_t)kq_plane(sbt * 64), oD = oS + (uint32_t)kq_plane(sbt * 16);
  constexpr int DB = K4 ? 4 : 2;                                                // bytes of plane D per super-block
  __amdgpu_buffer_rsrc_t rW[NW];
#pragma unroll
  for (int w = 0; w < NW; w++)
    rW[w] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a.W[w] + (size_t)e * a.estride), 0, (uint32_t)a.estride, 0x00020000);
  uint32_t offS[TN], offD[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int n = n0 + 32 * j + c32;
    const bool ok = n < a.N;
    offS[j] = ok ? oS + (uint32_t)((size_t)n * nsb * 16) : 0xffffffffu;
    offD[j] = ok ? oD + (uint32_t)((size_t)n * nsb * DB) : 0xffffffffu;
  }
  // one register set: a chunk's registers are requested again for the next super-block as soon as the chunk is unpacked
  u32x4 wq[NW][TN][4], wh[NW][TN][K4 ? 1 : 2], ws[NW][TN];
  uint32_t wd[NW][TN];
  // request i of a column tile: channels 8 i .. 8 i + 7, lane l takes 16-byte chunk l % 8 of channel 8 i + l / 8
  const int lr = lane >> 3, lc = lane & 7;
  auto load_chunk = [&](int w, int j, int i, int sb) {
    const int n = n0 + 32 * j + 8 * i + lr;
    const uint32_t off = (n < a.N && sb < nsb) ? (uint32_t)(((size_t)n * nsb * 8 + lc) * 16) : 0xffffffffu;
    wq[w][j][i] = __builtin_amdgcn_raw_buffer_load_b128(rW[w], off, sb * 128, 0);
  };
  // Q6_K, high bit pairs: request i = channels 16 i .. 16 i + 15, lane l takes chunk l % 4 of channel 16 i + l / 4
  auto load_high = [&](int w, int j, int i, int sb) {
    const int n = n0 + 32 * j + 16 * i + (lane >> 2);
    const uint32_t off = (n < a.N && sb < nsb) ? oH + (uint32_t)(((size_t)n * nsb * 4 + (lane & 3)) * 16) : 0xffffffffu;
    wh[w][j][K4 ? 0 : i] = __builtin_amdgcn_raw_buffer_load_b128(rW[w], off, sb * 64, 0);
  };
  auto load_scales = [&](int w, int j, int sb) {
    ws[w][j] = __builtin_amdgcn_raw_buffer_load_b128(rW[w], sb < nsb ? offS[j] : 0xffffffffu, sb * 16, 0);
    if (K4) wd[w][j] = __builtin_amdgcn_raw_buffer_load_b32(rW[w], sb < nsb ? offD[j] : 0xffffffffu, sb * 4, 0);
    else wd[w][j] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rW[w], sb < nsb ? offD[j] : 0xffffffffu, sb * 2, 0);
  };

  float acc[NW][TN][16];
#pragma unroll
  for (int w = 0; w < NW; w++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[w][j][r] = 0.f;
  const kx16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const kx16f zf = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // one super-block from LDS buffer `buf`
  auto compute = [&](int sb, int buf) {
    const unsigned char* st = smem + buf * KX_STAGE;
    unsigned char* patch = smem + 2 * KX_STAGE + wave * (K4 ? KX_PATCH : KX6_PATCH);
    // output r of this lane = tile row 8 (r / 4) + 4 hi + r % 4
    f32x4 dxv[4];
#pragma unroll
    for (int g = 0; g < 4; g++) dxv[g] = *reinterpret_cast<const f32x4*>(st + KX_OFF_DX + (8 * g + 4 * hi) * 4);
    const kxh8 Am = *reinterpret_cast<const kxh8*>(st + KX_OFF_BS + c32 * KX_BS + hi * 16);
    if constexpr (K4) {
#pragma unroll
    for (int w = 0; w < NW; w++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        int I[16];
#pragma unroll
        for (int r = 0; r < 16; r++) I[r] = 0;
        const uint32_t srec[4] = {ws[w][j].x, ws[w][j].y, ws[w][j].z, ws[w][j].w};
        const uint32_t dd = wd[w][j];
        // into the operand layout through the wave's patch (LDS operations of one wave execute in order: no barrier); the
        // registers are then free for the next super-block, whose lines are requested in consecutive instructions
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<u32x4*>(patch + (8 * i + lr) * KX_WROW + lc * 16) = wq[w][j][i];
#pragma unroll
        for (int i = 0; i < 4; i++) load_chunk(w, j, i, sb + 1);
#pragma unroll
        for (int p = 0; p < 4; p++) {
          const kx4i A0 = *reinterpret_cast<const kx4i*>(st + c32 * KX_LDC + (2 * p) * 32 + hi * 16);
          const kx4i A1 = *reinterpret_cast<const kx4i*>(st + c32 * KX_LDC + (2 * p + 1) * 32 + hi * 16);
          // chunk 2 p + hi of the channel: low nibbles = elements 16 hi .. 16 hi + 15 of sub-block 2 p, high nibbles of 2 p + 1
          const u32x4 q = *reinterpret_cast<const u32x4*>(patch + c32 * KX_WROW + (2 * p + hi) * 16);
          const kx4i lo = {(int)(q.x & 0x0f0f0f0fu), (int)(q.y & 0x0f0f0f0fu), (int)(q.z & 0x0f0f0f0fu), (int)(q.w & 0x0f0f0f0fu)};
          const kx4i up = {(int)((q.x >> 4) & 0x0f0f0f0fu), (int)((q.y >> 4) & 0x0f0f0f0fu), (int)((q.z >> 4) & 0x0f0f0f0fu),
                           (int)((q.w >> 4) & 0x0f0f0f0fu)};
          const kx16i T0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(A0, lo, zi, 0, 0, 0);
          const kx16i T1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(A1, up, zi, 0, 0, 0);
          const int sc0 = (int)(srec[p] & 0xffu), sc1 = (int)((srec[p] >> 8) & 0xffu);
#pragma unroll
          for (int r = 0; r < 16; r++) {
            // one multiply-add per sub-block and output (|T| < 2^16, sc < 2^6), and one pair of sub-blocks at a time: written
            // as C the sums reassociate, the compiler forms all eight sub-block results (128 registers) before it scales the
            // first and adds with separate multiplies
            I[r] = __mul24(T0[r], sc0) + I[r];
            asm volatile("" : "+v"(I[r]));
            I[r] = __mul24(T1[r], sc1) + I[r];
            asm volatile("" : "+v"(I[r]));
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        load_scales(w, j, sb + 1);
        // the minimum term: K slot 8 hi + i of the instruction = sum of 16 number 8 hi + i, which belongs to sub-block 4 hi + i / 2
        const uint32_t sA = hi ? srec[2] : srec[0], sB = hi ? srec[3] : srec[1];
        const _Float16 m0 = (_Float16)(float)((sA >> 16) & 0xffu), m1 = (_Float16)(float)(sA >> 24);
        const _Float16 m2 = (_Float16)(float)((sB >> 16) & 0xffu), m3 = (_Float16)(float)(sB >> 24);
        const kxh8 Bm = {m0, m0, m1, m1, m2, m2, m3, m3};
        const kx16f Mn = __builtin_amdgcn_mfma_f32_32x32x16_f16(Am, Bm, zf, 0, 0, 0);
        const float dW = f16bits_to_f32((uint16_t)(dd & 0xffffu)), dmW = f16bits_to_f32((uint16_t)(dd >> 16));
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float dx = dxv[r >> 2][r & 3];
          acc[w][j][r] = fmaf(dx * dW, (float)I[r], acc[w][j][r]);
          acc[w][j][r] = fmaf(-dx * dmW, Mn[r], acc[w][j][r]);
        }
      }
      } else {
#pragma unroll
      for (int w = 0; w < NW; w++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
          int I[16];
#pragma unroll
          for (int r = 0; r < 16; r++) I[r] = 0;
          const uint32_t srec[4] = {ws[w][j].x, ws[w][j].y, ws[w][j].z, ws[w][j].w};
          const uint32_t dd = wd[w][j];
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const u32x4 v = i >= 2 ? u32x4{wq[w][j][i].z, wq[w][j][i].w, wq[w][j][i].x, wq[w][j][i].y} : wq[w][j][i];
            *reinterpret_cast<u32x4*>(patch + (8 * i + lr) * KX6_WROW + lc * 16) = v;
          }
#pragma unroll
          for (int i = 0; i < 2; i++) {
            const u32x4 v = i == 1 ? u32x4{wh[w][j][i].z, wh[w][j][i].w, wh[w][j][i].x, wh[w][j][i].y} : wh[w][j][i];
            *reinterpret_cast<u32x4*>(patch + (16 * i + (lane >> 2)) * KX6_WROW + 128 + (lane & 3) * 16) = v;
          }
          const int hs = hi ^ (c32 >> 4);  // which half of a 16-byte piece holds this lane's eight bytes
#pragma unroll
          for (int i = 0; i < 4; i++) load_chunk(w, j, i, sb + 1);
#pragma unroll
          for (int i = 0; i < 2; i++) load_high(w, j, i, sb + 1);
          // group g of 16 elements = half h = g / 8, quarter qd = g % 8 / 2, l = 16 (g % 2) + 8 hi + (0..7) (dequantize_row_q6_K,
          // quantize_q6.cpp:108-133): low nibbles from ql[64 h + 32 (qd % 2) + l] (high nibble for qd >= 2), bits 2 qd, 2 qd + 1 of qh[32 h + l]
#pragma unroll
          for (int h = 0; h < 2; h++)
#pragma unroll
            for (int par = 0; par < 2; par++) {
              const u32x2 QH = *reinterpret_cast<const u32x2*>(patch + c32 * KX6_WROW + 128 + 32 * h + 16 * par + 8 * hs);
#pragma unroll
              for (int ql01 = 0; ql01 < 2; ql01++) {
                const u32x2 QL = *reinterpret_cast<const u32x2*>(patch + c32 * KX6_WROW + 64 * h + 32 * ql01 + 16 * par + 8 * hs);
#pragma unroll
                for (int nib = 0; nib < 2; nib++) {
                  const int qd = 2 * nib + ql01, g = 8 * h + 2 * qd + par;
                  uint32_t b[2];
#pragma unroll
                  for (int d2 = 0; d2 < 2; d2++) {
                    const uint32_t lbits = nib ? (QL[d2] >> 4) & 0x0f0f0f0fu : QL[d2] & 0x0f0f0f0fu;
                    const uint32_t hs = qd == 0 ? QH[d2] << 4 : qd == 1 ? QH[d2] << 2 : qd == 2 ? QH[d2] : QH[d2] >> 2;
                    b[d2] = (hs & 0x30303030u) | lbits;
                  }
                  const long B = (long)(((unsigned long)b[1] << 32) | b[0]);
                  const long A = *reinterpret_cast<const long*>(st + c32 * KX_LDC + 16 * g + 8 * hs);
                  const kx16i T = __builtin_amdgcn_mfma_i32_32x32x16_i8(A, B, zi, 0, 0, 0);
                  const int sc = (int)(int8_t)(srec[g >> 2] >> (8 * (g & 3)));
#pragma unroll
                  for (int r = 0; r < 16; r++) {
                    I[r] = __mul24(T[r], sc) + I[r];
                    asm volatile("" : "+v"(I[r]));
                  }
                  __builtin_amdgcn_sched_barrier(0);
                }
              }
            }
          load_scales(w, j, sb + 1);
          // the offset of 32: K slot 8 hi + i of the instruction = sum of 16 number 8 hi + i = group 8 hi + i
          kxh8 Bs;
#pragma unroll
          for (int i = 0; i < 8; i++) Bs[i] = (_Float16)(float)(int)(int8_t)((hi ? srec[2 + (i >> 2)] : srec[i >> 2]) >> (8 * (i & 3)));
          const kx16f Mn = __builtin_amdgcn_mfma_f32_32x32x16_f16(Am, Bs, zf, 0, 0, 0);
          const float dW = f16bits_to_f32((uint16_t)dd);
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const float dx = dxv[r >> 2][r & 3];
            const int tot = I[r] - 32 * (int)Mn[r];
            acc[w][j][r] = fmaf(dx * dW, (float)tot, acc[w][j][r]);
          }
        }
    }
  };

  load_stage(0);
#pragma unroll
  for (int w = 0; w < NW; w++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int p = 0; p < 4; p++) load_chunk(w, j, p, 0);
      if (!K4) {
#pragma unroll
        for (int p = 0; p < 2; p++) load_high(w, j, p, 0);
      }
      load_scales(w, j, 0);
    }
  store_stage(0);
  __syncthreads();
  for (int sb = 0; sb < nsb; sb++) {
    load_stage(sb + 1);
    compute(sb, sb & 1);
    store_stage((sb + 1) & 1);  // free since the barrier that ended super-block sb - 1
    __syncthreads();
  }

#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int m = 8 * (r >> 2) + 4 * hi + (r & 3);
    if (m < rows) {
      const int pos = row0 + m;
      const int64_t orow = a.out_ids ? a.out_ids[pos] : pos;
      if (NW == 2 && a.silu_mul) {
        // SiLU as mllm/backends/cpu/kernels/x86/silu.cpp:16-27 (x * (1 / (1 + exp(-x)))), then the product with the up projection
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const int n = n0 + 32 * j + c32;
          const float gv = acc[0][j][r], uv = acc[NW - 1][j][r];
          if (n < a.N) a.y[0][orow * a.N + n] = gv * (1.0f / (1.0f + (a.exp_accurate ? expf(-gv) : exp_poly(-gv)))) * uv;
        }
        continue;
      }
#pragma unroll
      for (int w = 0; w < NW; w++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const int n = n0 + 32 * j + c32;
          if (n < a.N) a.y[w][orow * a.N + n] = acc[w][j][r];
        }
    }
  }
}

constexpr int KX_TILE = 32;
bool kx_moe_tiles_fit(int wtype, int64_t N, int64_t K) {
  return (wtype == MLLM_HIP_Q4_K || wtype == MLLM_HIP_Q6_K) && K % QK_K == 0 && kq_packed_bytes(wtype, N, K) < ((size_t)1 << 32);
}
int kx_tile_rows() { return KX_TILE; }
// MoE row tiles of up to 32 expert-sorted positions: tile t = rows tile_row0[t] .. of expert tile_expert[t]; its rows read
// image rows row_ids[pos] / row_div (null: pos) and write rows out_ids[pos] (null: pos) of ys[p].
// silu_mul (two matrices): ys[0] receives silu(first) * second, ys[1] is not written.
int exp_mode_accurate();  // layer_ops.hip: the setting of mllm_hip_set_exp_mode
int kx_moe_tiles(int wtype, int nparts, const void* const* packed0, float* const* ys, int64_t N, int64_t K, const void* image,
                 int64_t img_rows, const int* tile_expert, const int* tile_row0, const int* tile_rows, const int* ntiles,
                 unsigned max_tiles, const int* row_ids, int row_div, const int* out_ids, int silu_mul, hipStream_t st) {
  if (!kx_moe_tiles_fit(wtype, N, K) || nparts < 1 || nparts > 2 || max_tiles < 1) return MLLM_HIP_E_SHAPE;
  if ((size_t)img_rows * K + (size_t)img_rows * (K / 16) * 2 + (size_t)img_rows * (K / QK_K) * 4 >= ((size_t)1 << 32)) return MLLM_HIP_E_SHAPE;
  KXArgs a{};
  for (int p = 0; p < nparts; p++) {
    a.W[p] = reinterpret_cast<const char*>(packed0[p]);
    a.y[p] = ys[p];
  }
  a.estride = kq_packed_bytes(wtype, N, K);
  a.image = reinterpret_cast<const char*>(image);
  a.img_rows = (int)img_rows;
  a.row_ids = row_ids; a.row_div = row_div > 0 ? row_div : 1; a.out_ids = out_ids;
  a.tile_expert = tile_expert; a.tile_row0 = tile_row0; a.tile_rows = tile_rows; a.ntiles = ntiles;
  a.N = (int)N; a.K = (int)K;
  a.silu_mul = nparts == 2 && silu_mul;
  a.exp_accurate = exp_mode_accurate();
  const bool k4 = wtype == MLLM_HIP_Q4_K;
  const size_t lds = 2 * (size_t)KX_STAGE + 4 * (size_t)(k4 ? KX_PATCH : KX6_PATCH);
  const dim3 g2(max_tiles, (unsigned)((N + 127) / 128)), g1(max_tiles, (unsigned)((N + 255) / 256));
  if (nparts == 2) {
    if (k4) hipLaunchKernelGGL((kx_kernel<MLLM_HIP_Q4_K, 2, 1>), g2, dim3(256), lds, st, a);
    else hipLaunchKernelGGL((kx_kernel<MLLM_HIP_Q6_K, 2, 1>), g2, dim3(256), lds, st, a);
  } else {
    if (k4) hipLaunchKernelGGL((kx_kernel<MLLM_HIP_Q4_K, 1, 2>), g1, dim3(256), lds, st, a);
    else hipLaunchKernelGGL((kx_kernel<MLLM_HIP_Q6_K, 1, 2>), g1, dim3(256), lds, st, a);
  }
  return (int)hipGetLastError();
}

}  // namespace mllmhip
