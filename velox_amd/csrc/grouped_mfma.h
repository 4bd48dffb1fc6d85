// Many small bfloat16 products in one launch on the matrix cores of gfx950: a product per group (an expert, a head), each
// over its own rows, out[r, g, :] = W_g a[r, g, :].  Shared by the routed experts and by the per-head products of
// attention over a latent.
//
// A workgroup of four waves owns 64 rows and 128 output columns of one group (64 gate and the 64 up columns of the same
// outputs with the GLU epilogue); a wave owns 32 of the columns (two 16-row tiles of W; GLU: a gate tile and its up tile)
// and all 64 rows, eight 16x16 accumulators.  Operands come straight from global memory in the layout of
// v_mfma_f32_16x16x32_bf16 (lane = 16 g + i holds indices 8 g .. 8 g + 7 of row i: 16 bytes), W as the left operand, so
// acc[j] of lane (g, i) is out[row i][column 4 g + j]; the next step's operands are asked for before this step's matrix
// instructions.  The four waves read the same rows of `a`, which the compute unit's cache serves.  Rows and columns
// beyond a tile's own read a valid row again and are never stored.  A row's sum is built in the order of k whatever
// else is in the tile.
//
// Requirements (checked by the callers): K % 8 == 0, row strides and offsets of `a` multiples of 8 elements, 16-byte
// aligned bases.
#pragma once
#include "common.h"

typedef __bf16 gm_bf16x8_t __attribute__((ext_vector_type(8)));

#define GM_ROWS 64       // rows of a tile
#define GM_COLS 128      // output columns of a workgroup (GLU: 64)

enum { GM_PLAIN = 0, GM_GLU = 1, GM_GATE = 2, GM_ROW_SCALE = 3 };

struct GroupedArgs {
  const bf16_t* a;     // element (row r, group g, k) at a[r * a_ld + g * a_group + k]
  long long a_ld, a_group;
  const bf16_t* w;     // group g's matrix at w + g * w_group: [n (GLU: 2 n)][k]
  long long w_group;
  void* out;           // element (row r, group g, col) at out[r * out_ld + g * out_group + col]
  long long out_ld, out_group;
  int n, k;
  // rows: either every group runs rows [0, m) (plan == nullptr, blockIdx.y = row tile, blockIdx.z = group), or the plan's
  // tiles say which group runs which rows (blockIdx.y = tile)
  int m;
  const int* plan;
  int plan_pairs, plan_groups, plan_max_tiles;
  const bf16_t* gate;  // GM_GATE: times sigmoid(gate[r * gate_ld + g * n + col])
  long long gate_ld;
  const float* row_scale;  // GM_ROW_SCALE: times row_scale[order[r]]
};

__device__ __forceinline__ gm_bf16x8_t gm_load(const bf16_t* p, bool ok) {
  if (!ok) {
    const float4_t z = {0.f, 0.f, 0.f, 0.f};
    return __builtin_bit_cast(gm_bf16x8_t, z);
  }
  return __builtin_bit_cast(gm_bf16x8_t, *reinterpret_cast<const float4_t*>(p));
}

template <int EPI, typename TO>
__global__ void __launch_bounds__(256) grouped_mfma_kernel(const GroupedArgs args) {
  int group, row0, rows;
  const int* order = nullptr;
  if (args.plan != nullptr) {
    const int tile = blockIdx.y;
    if (tile >= args.plan[0]) return;  // (uniform over the workgroup)
    const int* starts = args.plan + 1;
    order = starts + args.plan_groups + 1;
    const int* tile_group = order + 2 * (size_t)args.plan_pairs;
    const int* tile_row = tile_group + args.plan_max_tiles;
    group = tile_group[tile];
    row0 = tile_row[tile];
    rows = min(GM_ROWS, starts[group + 1] - row0);
  } else {
    group = blockIdx.z;
    row0 = blockIdx.y * GM_ROWS;
    rows = min(GM_ROWS, args.m - row0);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane & 15, g4 = lane >> 4;
  const int n = args.n, k = args.k;
  // the two tiles of W this wave owns: their first columns
  int col0[2];
  if (EPI == GM_GLU) {
    col0[0] = blockIdx.x * (GM_COLS / 2) + wave * 16;
    col0[1] = col0[0];
  } else {
    col0[0] = blockIdx.x * GM_COLS + wave * 32;
    col0[1] = col0[0] + 16;
  }
  if (col0[0] >= n) return;  // (a wave without columns; no barrier follows)
  const bf16_t* w_base = args.w + (size_t)group * args.w_group;
  const bf16_t* w_row[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int col = min(col0[t] + i, n - 1);
    w_row[t] = w_base + (size_t)(EPI == GM_GLU && t == 1 ? n + col : col) * k + 8 * g4;
  }
  const bf16_t* a_row[4];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int r = min(mt * 16 + i, rows - 1);
    a_row[mt] = args.a + (size_t)(row0 + r) * args.a_ld + (size_t)group * args.a_group + 8 * g4;
  }
  float4_t acc[2][4];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) acc[t][mt] = float4_t{0.f, 0.f, 0.f, 0.f};

  gm_bf16x8_t w_cur[2], a_cur[4], w_next[2], a_next[4];
  bool ok = 8 * g4 < k;
#pragma unroll
  for (int t = 0; t < 2; ++t) w_cur[t] = gm_load(w_row[t], ok);
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) a_cur[mt] = gm_load(a_row[mt], ok);
  for (int k0 = 0; k0 < k; k0 += 32) {
    const bool more = k0 + 32 + 8 * g4 < k;
#pragma unroll
    for (int t = 0; t < 2; ++t) w_next[t] = gm_load(w_row[t] + k0 + 32, more);
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) a_next[mt] = gm_load(a_row[mt] + k0 + 32, more);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[t], a_cur[mt], acc[t][mt], 0, 0, 0);
#pragma unroll
    for (int t = 0; t < 2; ++t) w_cur[t] = w_next[t];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) a_cur[mt] = a_next[mt];
  }

  TO* out = reinterpret_cast<TO*>(args.out);
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int r = mt * 16 + i;
    if (r >= rows) continue;
    const size_t out_row = (size_t)(row0 + r) * args.out_ld + (size_t)group * args.out_group;
    float scale = 1.f;
    if (EPI == GM_ROW_SCALE) scale = args.row_scale[order[row0 + r]];
#pragma unroll
    for (int t = 0; t < (EPI == GM_GLU ? 1 : 2); ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = col0[t] + 4 * g4 + j;
        if (col >= n) continue;
        float v = acc[t][mt][j];
        if (EPI == GM_GLU) v = v / (1.f + expf(-v)) * acc[1][mt][j];
        if (EPI == GM_GATE) {
          const float z = to_f32(args.gate[(size_t)(row0 + r) * args.gate_ld + (size_t)group * n + col]);
          v *= 1.f / (1.f + expf(-z));
        }
        if (EPI == GM_ROW_SCALE) v *= scale;
        out[out_row + col] = from_f32<TO>(v);
      }
  }
}

// Whether the operands meet what the kernel's 16-byte loads need.
static inline bool grouped_mfma_fits(const void* a, long long a_ld, long long a_group, long long a_offset, const void* w, int k) {
  return k % 8 == 0 && a_ld % 8 == 0 && a_group % 8 == 0 && a_offset % 8 == 0 && ((uintptr_t)a) % 16 == 0 && ((uintptr_t)w) % 16 == 0;
}
