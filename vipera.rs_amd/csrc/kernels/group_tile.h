// A 128 x 128 tile of a bfloat16 product on the matrix cores whose rows are found through the caller's functions:
// gathered activation rows (a mixture of experts' tokens, sorted by expert), a weight per group (expert, head),
// outputs scattered or strided.  Used by the grouped products of moe.hip and latent.hip.
//
// Workgroup: 256 threads, four waves as 2 x 2, each 64 activation rows x 64 weight rows: sixteen
// v_mfma_f32_16x16x32_bf16 per 32 k, the weight as the first operand, so that a lane ends up with four
// consecutive weight rows (outputs) of one activation row.  K runs in steps of 64 through two LDS stages (rows
// padded to 144 bytes); the next step's 16-byte chunks are on their way into registers while a step is
// multiplied; one barrier a step.  K must be a multiple of 8 and every row 16-byte aligned; chunks past K and
// rows that do not exist are zeros.  An output element is summed in k order whatever else the tile holds.
#pragma once
#include "common.h"

typedef __bf16 gt_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gt_f32x4 __attribute__((ext_vector_type(4)));

constexpr int GT_TILE = 128;     // rows of activations and of weights per workgroup
constexpr int GT_BK = 64;        // k per step
constexpr int GT_ROW = GT_BK * 2 + 16;   // bytes per LDS row
constexpr int GT_STAGE = 2 * GT_TILE * GT_ROW;
constexpr int GT_LDS_BYTES = 2 * GT_STAGE;

// a_row(r): pointer to activation row r of the tile (r < 128) or nullptr; w_row(r): pointer to weight row r of the
// tile or nullptr.  After the call acc[tn][tm] holds, for this lane, weight rows wn * 64 + tn * 16 + (lane / 16) * 4
// + 0..3 of activation row wm * 64 + tm * 16 + lane % 16.
// Chunks that do not exist are not loaded (measured against reading them at a fixed address and masking: a tile of a
// decode step, which is mostly empty rows, took 40 % longer that way).
template <typename ARow, typename WRow>
__device__ __forceinline__ void group_tile_mma(ARow a_row, WRow w_row, int K, unsigned char* lds,
                                               gt_f32x4 (&acc)[4][4]) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 15, lg = lane >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = gt_f32x4{0.f, 0.f, 0.f, 0.f};
  // a thread's eight chunks of a step: four of activations, four of weights; chunk c: row c / 8, k (c % 8) * 8
  const __bf16* src[8];
  unsigned dst[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + i * 256, row = c >> 3, kc = c & 7;
    const __bf16* pa = a_row(row);
    const __bf16* pw = w_row(row);
    src[i] = pa ? pa + kc * 8 : nullptr;
    src[4 + i] = pw ? pw + kc * 8 : nullptr;
    dst[i] = (unsigned)(row * GT_ROW + kc * 16);
    dst[4 + i] = (unsigned)((GT_TILE + row) * GT_ROW + kc * 16);
  }
  const int kc_of = tid & 7;      // the same for all of a thread's chunks (256 is a multiple of 8)
  gt_bf16x8 held[8];
  auto fetch = [&](int k0) {
    const bool in = k0 + kc_of * 8 < K;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      gt_bf16x8 zero = {};
      held[i] = (src[i] && in) ? *(const gt_bf16x8*)(src[i] + k0) : zero;
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int i = 0; i < 8; ++i) *(gt_bf16x8*)(lds + stage * GT_STAGE + dst[i]) = held[i];
  };
  const int steps = (K + GT_BK - 1) / GT_BK;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int stage = s & 1;
    if (s + 1 < steps) fetch((s + 1) * GT_BK);
    const unsigned char* base = lds + stage * GT_STAGE;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      gt_bf16x8 fa[4], fw[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        fa[t] = *(const gt_bf16x8*)(base + (wm * 64 + t * 16 + lr) * GT_ROW + half * 64 + lg * 16);
        fw[t] = *(const gt_bf16x8*)(base + (GT_TILE + wn * 64 + t * 16 + lr) * GT_ROW + half * 64 + lg * 16);
      }
#pragma unroll
      for (int tn = 0; tn < 4; ++tn)
#pragma unroll
        for (int tm = 0; tm < 4; ++tm)
          acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[tn], fa[tm], acc[tn][tm], 0, 0, 0);
    }
    if (s + 1 < steps) stash(stage ^ 1);
    __syncthreads();
  }
}
