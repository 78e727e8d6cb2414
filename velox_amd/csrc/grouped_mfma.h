// Many small bfloat16 products in one launch on the matrix cores of gfx950: a product per group (an expert, a head), each
// over its own rows, out[r, g, :] = W_g a[r, g, :].  Shared by the routed experts and by the per-head products of
// attention over a latent.
//
// A workgroup of four waves owns 64 rows (128 for the large tiles of a plan) and 64 NT output columns of one group (NT = 2 or 4 tiles of W per wave; half as
// many gate columns and the up columns of the same outputs with the GLU epilogue); a wave owns 16 NT of the columns and all
// 64 rows: 4 NT 16x16 accumulators.  W comes straight from global memory in the layout of
// v_mfma_f32_16x16x32_bf16 (lane = 16 g + i holds indices 8 g .. 8 g + 7 of row i: 16 bytes) and is the left operand, so
// acc[j] of lane (g, i) is out[row i][column 4 g + j]; no two waves read the same W.  The rows of `a`, which all four
// waves need, pass through LDS: a step is 64 indices, 8 KB for the 64 rows, two 16-byte pieces per thread, laid out [piece][row] so
// that the 16 lanes of a lane group read 256 contiguous bytes (no bank conflicts on the reads, which are four times as many
// as the writes); two buffers, one barrier per step, the
// next step's pieces and W operands asked for before this step's matrix instructions.  Rows and columns beyond a tile's
// own read a valid row again and are never stored.  A row's sum is built in the order of k whatever else is in the tile.
//
// Requirements (checked by the callers): K % 8 == 0, row strides and offsets of `a` multiples of 8 elements, 16-byte
// aligned bases.
#pragma once
#include "common.h"

typedef __bf16 gm_bf16x8_t __attribute__((ext_vector_type(8)));

#define GM_ROWS 64       // rows of a tile without a plan (a plan's tiles hold 64 or 128)
#define GM_FEW_COLS 32   // output columns of a workgroup of the kernel for few rows (GLU: 16)

enum { GM_PLAIN = 0, GM_GLU = 1, GM_GATE = 2, GM_ROW_SCALE = 3, GM_ACT = 4 };

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
  const bf16_t* gate;  // GM_GATE: times sigmoid(gate[r * gate_ld + g * gate_group + col * gate_col]); (n, 1) is a number per output, (1, 0) one per group
  long long gate_ld, gate_group, gate_col;
  int act = 0;         // GM_ACT: the result goes through ungated_act(., act)
  const float* row_scale;  // GM_ROW_SCALE: times row_scale[order[r]]
  GluUnit unit = {1.f, INFINITY, 0.f};  // GM_GLU: the unit's middle (see glu_middle)
};

__device__ __forceinline__ gm_bf16x8_t gm_load(const bf16_t* p, bool ok) {
  if (!ok) {
    const float4_t z = {0.f, 0.f, 0.f, 0.f};
    return __builtin_bit_cast(gm_bf16x8_t, z);
  }
  return __builtin_bit_cast(gm_bf16x8_t, *reinterpret_cast<const float4_t*>(p));
}

template <int EPI, typename TO, int GM_NT, int MT>
__global__ void __launch_bounds__(256) grouped_mfma_kernel(const GroupedArgs args) {
  constexpr int GM_COLS = 64 * GM_NT;    // output columns of the workgroup (GLU: half as many)
  constexpr int ROWS = 16 * MT;          // rows of a tile: 64 or 128
  constexpr int HALVES = MT == 8 ? 1 : 2;  // 32-index halves per step (the larger tile takes shorter steps: registers)
  constexpr int STEP = 32 * HALVES;
  constexpr int PIECES = MT / 4;         // 16-byte pieces of `a` per thread and half
  __shared__ float4_t a_lds[2][HALVES][4 * ROWS];
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
    rows = min(ROWS, starts[group + 1] - row0);
  } else {
    group = blockIdx.z;
    row0 = blockIdx.y * ROWS;
    rows = min(ROWS, args.m - row0);
  }
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int i = lane & 15, g4 = lane >> 4;
  const int n = args.n, k = args.k;
  // the tiles of W this wave owns: their first output columns (GLU: the first half are gate rows, the others the up rows of the same)
  int col0[GM_NT];
#pragma unroll
  for (int t = 0; t < GM_NT; ++t) {
    if (EPI == GM_GLU) col0[t] = blockIdx.x * (GM_COLS / 2) + wave * (8 * GM_NT) + (t % (GM_NT / 2)) * 16;
    else col0[t] = blockIdx.x * GM_COLS + wave * (16 * GM_NT) + t * 16;
  }
  const bf16_t* w_base = args.w + (size_t)group * args.w_group;
  const bf16_t* w_row[GM_NT];
#pragma unroll
  for (int t = 0; t < GM_NT; ++t) {
    const int col = min(col0[t] + i, n - 1);
    w_row[t] = w_base + (size_t)(EPI == GM_GLU && t >= GM_NT / 2 ? n + col : col) * k + 8 * g4;
  }
  // this thread's pieces of the rows of `a`: piece q = tid + 256 p is row q / 4, indices 8 (q % 4) .. + 7 of a half; in LDS
  // [part][row], so that a row tile's operand reads are 256 contiguous bytes per 16 lanes
  const bf16_t* a_piece[PIECES];
  int a_slot[PIECES];
#pragma unroll
  for (int p = 0; p < PIECES; ++p) {
    const int q = tid + 256 * p;
    a_piece[p] = args.a + (size_t)(row0 + min(q >> 2, rows - 1)) * args.a_ld + (size_t)group * args.a_group + 8 * (q & 3);
    a_slot[p] = (q & 3) * ROWS + (q >> 2);
  }
  const int a_part = 8 * (tid & 3);  // (q % 4 is tid % 4 for every piece)
  float4_t acc[GM_NT][MT];
#pragma unroll
  for (int t = 0; t < GM_NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = float4_t{0.f, 0.f, 0.f, 0.f};

  gm_bf16x8_t w_cur[HALVES][GM_NT], w_next[HALVES][GM_NT];
#pragma unroll
  for (int u = 0; u < HALVES; ++u) {
#pragma unroll
    for (int t = 0; t < GM_NT; ++t) w_cur[u][t] = gm_load(w_row[t] + 32 * u, 32 * u + 8 * g4 < k);
#pragma unroll
    for (int p = 0; p < PIECES; ++p) a_lds[0][u][a_slot[p]] = __builtin_bit_cast(float4_t, gm_load(a_piece[p] + 32 * u, 32 * u + a_part < k));
  }
  __syncthreads();
  int buffer = 0;
  for (int k0 = 0; k0 < k; k0 += STEP) {
    gm_bf16x8_t a_next[HALVES][PIECES];
#pragma unroll
    for (int u = 0; u < HALVES; ++u) {
      const int at = k0 + STEP + 32 * u;
#pragma unroll
      for (int t = 0; t < GM_NT; ++t) w_next[u][t] = gm_load(w_row[t] + at, at + 8 * g4 < k);
#pragma unroll
      for (int p = 0; p < PIECES; ++p) a_next[u][p] = gm_load(a_piece[p] + at, at + a_part < k);
    }
#pragma unroll
    for (int u = 0; u < HALVES; ++u) {
#pragma unroll
      for (int mh = 0; mh < MT; mh += 4) {  // four row tiles at a time: their operands live in registers together
        gm_bf16x8_t a_cur[4];
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) a_cur[mt] = __builtin_bit_cast(gm_bf16x8_t, a_lds[buffer][u][g4 * ROWS + (mh + mt) * 16 + i]);
#pragma unroll
        for (int t = 0; t < GM_NT; ++t)
#pragma unroll
          for (int mt = 0; mt < 4; ++mt) acc[t][mh + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[u][t], a_cur[mt], acc[t][mh + mt], 0, 0, 0);
      }
    }
#pragma unroll
    for (int u = 0; u < HALVES; ++u)
#pragma unroll
      for (int p = 0; p < PIECES; ++p) a_lds[buffer ^ 1][u][a_slot[p]] = __builtin_bit_cast(float4_t, a_next[u][p]);
    __syncthreads();
    buffer ^= 1;
#pragma unroll
    for (int u = 0; u < HALVES; ++u)
#pragma unroll
      for (int t = 0; t < GM_NT; ++t) w_cur[u][t] = w_next[u][t];
  }

  TO* out = reinterpret_cast<TO*>(args.out);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int r = mt * 16 + i;
    if (r >= rows) continue;
    const size_t out_row = (size_t)(row0 + r) * args.out_ld + (size_t)group * args.out_group;
    float scale = 1.f;
    if (EPI == GM_ROW_SCALE) scale = args.row_scale[order[row0 + r]];
#pragma unroll
    for (int t = 0; t < (EPI == GM_GLU ? GM_NT / 2 : GM_NT); ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = col0[t] + 4 * g4 + j;
        if (col >= n) continue;
        float v = acc[t][mt][j];
        if (EPI == GM_GLU) v = glu_middle(v, acc[t + GM_NT / 2][mt][j], args.unit);
        if (EPI == GM_GATE) {
          const float z = to_f32(args.gate[(size_t)(row0 + r) * args.gate_ld + (size_t)group * args.gate_group + (size_t)col * args.gate_col]);
          v *= 1.f / (1.f + expf(-z));
        }
        if (EPI == GM_ROW_SCALE) v *= scale;
        if (EPI == GM_ACT) v = ungated_act(v, args.act);
        out[out_row + col] = from_f32<TO>(v);
      }
  }
}

// The same products when no tile has more than 16 MT rows (a decode step's pairs): then a product is bound by reading W
// once, and what counts is how many loads are in flight.  A workgroup owns 32 output columns (GLU: 16 gate columns and
// their up columns) of one tile; its four waves split K into quarters, each wave asks for four steps' operands at once,
// and the waves' sums are added through LDS in the order of the waves (no atomics: the same result on every run).
template <int EPI, typename TO, int MT>
__global__ void __launch_bounds__(256) grouped_mfma_few_rows_kernel(const GroupedArgs args) {
  __shared__ float4_t partial[3][2 * MT][64];
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
    rows = min(16 * MT, starts[group + 1] - row0);
  } else {
    group = blockIdx.z;
    row0 = blockIdx.y * 16 * MT;
    rows = min(16 * MT, args.m - row0);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane & 15, g4 = lane >> 4;
  const int n = args.n, k = args.k;
  int col0[2];
  col0[0] = blockIdx.x * (EPI == GM_GLU ? GM_FEW_COLS / 2 : GM_FEW_COLS);
  col0[1] = EPI == GM_GLU ? col0[0] : col0[0] + 16;
  const bf16_t* w_base = args.w + (size_t)group * args.w_group;
  const bf16_t* w_row[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int col = min(col0[t] + i, n - 1);
    w_row[t] = w_base + (size_t)(EPI == GM_GLU && t == 1 ? n + col : col) * k + 8 * g4;
  }
  const bf16_t* a_row[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) a_row[mt] = args.a + (size_t)(row0 + min(mt * 16 + i, rows - 1)) * args.a_ld + (size_t)group * args.a_group + 8 * g4;
  const int quarter = ((k + 127) / 128) * 32;  // indices per wave: a multiple of 32
  const int k_begin = wave * quarter, k_end = min(k, k_begin + quarter);
  float4_t acc[2][MT];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = float4_t{0.f, 0.f, 0.f, 0.f};
  for (int k0 = k_begin; k0 < k_end; k0 += 128) {
    gm_bf16x8_t wv[2][4], av[MT][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool ok = k0 + 32 * u + 8 * g4 < k_end;
#pragma unroll
      for (int t = 0; t < 2; ++t) wv[t][u] = gm_load(w_row[t] + k0 + 32 * u, ok);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) av[mt][u] = gm_load(a_row[mt] + k0 + 32 * u, ok);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[t][u], av[mt][u], acc[t][mt], 0, 0, 0);
  }
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) partial[wave - 1][t * MT + mt][lane] = acc[t][mt];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int other = 0; other < 3; ++other)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const float4_t p = partial[other][t * MT + mt][lane];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[t][mt][j] += p[j];
      }
  TO* out = reinterpret_cast<TO*>(args.out);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
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
        if (EPI == GM_GLU) v = glu_middle(v, acc[1][mt][j], args.unit);
        if (EPI == GM_GATE) {
          const float z = to_f32(args.gate[(size_t)(row0 + r) * args.gate_ld + (size_t)group * args.gate_group + (size_t)col * args.gate_col]);
          v *= 1.f / (1.f + expf(-z));
        }
        if (EPI == GM_ROW_SCALE) v *= scale;
        if (EPI == GM_ACT) v = ungated_act(v, args.act);
        out[out_row + col] = from_f32<TO>(v);
      }
  }
}

// Launches the kernel that fits: `most_rows` is the most rows any tile can have (the plan's pairs, or m), `tile_rows` the
// rows of the plan's tiles (64 or 128; without a plan rows come in tiles of 64), `tiles_y` and `tiles_z` the launch's other
// two dimensions.
template <int EPI, typename TO>
static void grouped_mfma_launch(const GroupedArgs& args, int most_rows, int tile_rows, int tiles_y, int tiles_z, hipStream_t stream) {
  const int n = args.n;
  if (most_rows <= 64 && args.plan != nullptr) {
    // (only with a plan: its tiles hold at most `most_rows` rows whatever their size; without one, rows come in tiles of the kernel's own size)
    dim3 grid((n + (EPI == GM_GLU ? GM_FEW_COLS / 2 : GM_FEW_COLS) - 1) / (EPI == GM_GLU ? GM_FEW_COLS / 2 : GM_FEW_COLS), tiles_y, tiles_z);
    if (most_rows <= 16) grouped_mfma_few_rows_kernel<EPI, TO, 1><<<grid, 256, 0, stream>>>(args);
    else if (most_rows <= 32) grouped_mfma_few_rows_kernel<EPI, TO, 2><<<grid, 256, 0, stream>>>(args);
    else grouped_mfma_few_rows_kernel<EPI, TO, 4><<<grid, 256, 0, stream>>>(args);
    return;
  }
  const int outputs = EPI == GM_GLU ? 2 * n : n;  // rows of W
  if (outputs <= 128) {
    const int cols = EPI == GM_GLU ? 64 : 128;
    grouped_mfma_kernel<EPI, TO, 2, 4><<<dim3((n + cols - 1) / cols, tiles_y, tiles_z), 256, 0, stream>>>(args);
  } else {
    const int cols = EPI == GM_GLU ? 128 : 256;
    if (tile_rows == 128) grouped_mfma_kernel<EPI, TO, 4, 8><<<dim3((n + cols - 1) / cols, tiles_y, tiles_z), 256, 0, stream>>>(args);
    else grouped_mfma_kernel<EPI, TO, 4, 4><<<dim3((n + cols - 1) / cols, tiles_y, tiles_z), 256, 0, stream>>>(args);
  }
}

// Whether the operands meet what the kernels' 16-byte loads need.
static inline bool grouped_mfma_fits(const void* a, long long a_ld, long long a_group, long long a_offset, const void* w, int k) {
  return k % 8 == 0 && a_ld % 8 == 0 && a_group % 8 == 0 && a_offset % 8 == 0 && ((uintptr_t)a) % 16 == 0 && ((uintptr_t)w) % 16 == 0;
}
