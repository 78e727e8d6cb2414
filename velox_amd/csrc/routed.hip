// Routed experts for gfx950: nothing about a step's routing is known to the host.
//
//   route_top:       scores of the router's float32 logits and the `top` largest per token
//   routed_plan:     the step's (token, choice) pairs sorted by expert, and the list of row tiles that the grouped products
//                    run: one workgroup, counters in LDS
//   grouped_glu:     act[p, :] = silu(Wgate_e a_p) * (Wup_e a_p) for every sorted pair p of expert e, a_p = x[token of p]
//                    (times the pair's weight when the weight scales the input)
//   grouped_down:    y[p, :] = Wdown_e act[p, :] (times the pair's weight when it scales the output), float32
//   routed_combine:  out[t, :] = sum_k y[place of pair (t, k), :] (+ shared[t, :]), the choices in order
//
// The grouped products are launched for the most tiles a step of its size can have; a workgroup beyond the step's own
// number of tiles (read from the plan) exits at once.  A row's result is summed over k in one fixed order by one thread,
// whatever other rows share its tile, so a token's output does not depend on which tokens go to the same experts or on
// the order in which the plan's atomic counters placed them.
#include "common.h"
#include "grouped_mfma.h"

#define RT_BM 64  // rows of a tile (sorted pairs of one expert)
#define RT_BN 64
#define RT_BK 16
#define RT_PAD 4
#define RT_FOLD 128

// ---------------------------------------------------------------------------------------------
// route_top: one wave per token, its lanes over the experts.  score = sigmoid(z) or softmax(z) over all experts; the `top`
// largest scores, ties to the lower index; weights are the chosen scores, divided by their sum when `renormalize`.
// Every round the wave takes the largest score that is not yet taken (value first, then the lower index), so the choices
// come out in descending order of score.  With `correction` (float32 [experts]) the choice goes by score + correction and
// the weights stay the scores themselves.  With `group_count` > 0 the experts form that many equal groups of neighbours; a
// group's score is the sum of its two largest choice scores (of its one, if it has one expert), and only experts of the
// `group_keep` best groups (ties to the lower index) can be chosen: the others' choice scores become minus infinity.
// `norm_floor` is added to the sum that renormalised weights are divided by.
// ---------------------------------------------------------------------------------------------
#define ROUTE_PER_LANE 32  // experts per lane held in registers: up to 2,048 experts

__global__ void __launch_bounds__(256) route_top_kernel(const float* __restrict__ logits, int* __restrict__ choice, float* __restrict__ weight, int tokens,
                                                        int experts, int top, int softmax, int renormalize, const float* __restrict__ correction,
                                                        int group_count, int group_keep, float norm_floor) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= tokens) return;  // (a whole wave; nothing below crosses waves)
  const float* z = logits + (size_t)t * experts;
  float shift = 0.f, denom = 1.f;
  if (softmax) {
    float m = -INFINITY;
    for (int e = lane; e < experts; e += 64) m = fmaxf(m, z[e]);
    shift = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < experts; e += 64) sum += expf(z[e] - shift);
    denom = wave_sum(sum);
  }
  const int used = (experts + 63) >> 6;  // registers of `score` that hold experts at all: the loops below stop there
  float score[ROUTE_PER_LANE];
#pragma unroll
  for (int u = 0; u < ROUTE_PER_LANE; ++u) {
    const int e = lane + 64 * u;
    score[u] = -INFINITY;  // ("no such expert" and "taken")
    if (e < experts) {
      score[u] = softmax ? expf(z[e] - shift) / denom : 1.f / (1.f + expf(-z[e]));
      if (correction) score[u] += correction[e];
    }
  }
  if (group_count > 0) {
    // lane g ends up with group g's score (group_count <= 64); every group's two largest by two rounds over the wave
    const int per = experts / group_count;
    float mine = -INFINITY;  // (lanes beyond the groups never win)
    if (used == 1 && (per & (per - 1)) == 0) {
      // one expert per lane and groups that are aligned runs of a power of two of lanes: all groups at once, the two
      // largest of a run by exchanges inside the run
      float first = score[0], second = -INFINITY;
      for (int offset = 1; offset < per; offset <<= 1) {
        const float of = __shfl_xor(first, offset, 64), os = __shfl_xor(second, offset, 64);
        second = fmaxf(fminf(first, of), fmaxf(second, os));
        first = fmaxf(first, of);
      }
      const float sum = per > 1 ? first + second : first;
      const float of_group = __shfl(sum, (lane * per) & 63, 64);
      if (lane < group_count) mine = of_group;
    } else
    for (int gidx = 0; gidx < group_count; ++gidx) {
      const int lo = gidx * per, hi = lo + per;
      float first = -INFINITY, second = -INFINITY;  // this lane's two largest inside the group
#pragma unroll
      for (int u = 0; u < ROUTE_PER_LANE; ++u) {
        if (u >= used) break;
        const int e = lane + 64 * u;
        if (e >= lo && e < hi) {
          const float v = score[u];
          if (v > first) { second = first; first = v; }
          else if (v > second) second = v;
        }
      }
      // the wave's two largest: merge (first, second) pairs
#pragma unroll
      for (int offset = 32; offset > 0; offset >>= 1) {
        const float of = __shfl_xor(first, offset, 64), os = __shfl_xor(second, offset, 64);
        const float hi1 = fmaxf(first, of);
        const float lo1 = fminf(first, of);
        second = fmaxf(lo1, fmaxf(second, os));
        first = hi1;
      }
      const float sum = per > 1 ? first + second : first;
      if (lane == gidx) mine = sum;
    }
    unsigned long long allowed = 0ull;
    for (int k = 0; k < group_keep; ++k) {
      float best = mine;
      int best_g = lane < group_count ? lane : 0x7fffffff;
      if (lane >= group_count || ((allowed >> lane) & 1ull)) { best = -INFINITY; best_g = 0x7fffffff; }
#pragma unroll
      for (int offset = 32; offset > 0; offset >>= 1) {
        const float other = __shfl_xor(best, offset, 64);
        const int other_g = __shfl_xor(best_g, offset, 64);
        if (other > best || (other == best && other_g < best_g)) { best = other; best_g = other_g; }
      }
      if (best_g < group_count) allowed |= 1ull << best_g;
      else {  // (every group left scores minus infinity or NaN: take the lowest group not yet taken)
        for (int gidx = 0; gidx < group_count; ++gidx)
          if (!((allowed >> gidx) & 1ull)) { allowed |= 1ull << gidx; break; }
      }
    }
#pragma unroll
    for (int u = 0; u < ROUTE_PER_LANE; ++u) {
      if (u >= used) break;
      const int e = lane + 64 * u;
      if (e < experts && !((allowed >> (e / per)) & 1ull)) score[u] = -INFINITY;
    }
  }
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int u = 0; u < ROUTE_PER_LANE; ++u) {
      if (u >= used) break;
      if (score[u] > best) { best = score[u]; best_e = lane + 64 * u; }  // (ascending e within a lane: the first of equals stays)
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
      const float other = __shfl_xor(best, offset, 64);
      const int other_e = __shfl_xor(best_e, offset, 64);
      if (other > best || (other == best && other_e < best_e)) { best = other; best_e = other_e; }
    }
#pragma unroll
    for (int u = 0; u < ROUTE_PER_LANE; ++u) {
      if (u >= used) break;
      if (lane + 64 * u == best_e) score[u] = -INFINITY;
    }
    // (the weight is the score without the correction: the same expression as above, so the same value)
    if (best_e >= experts) best_e = 0;  // (only when every score left is a NaN: stay inside the row)
    if (correction) best = softmax ? expf(z[best_e] - shift) / denom : 1.f / (1.f + expf(-z[best_e]));
    total += best;
    if (lane == 0) {
      choice[(size_t)t * top + k] = best_e;
      weight[(size_t)t * top + k] = best;
    }
  }
  if (renormalize && lane == 0)  // (the lane that wrote them)
    for (int k = 0; k < top; ++k) weight[(size_t)t * top + k] /= (total + norm_floor);
}

extern "C" int velox_route_top(const float* logits, int* choice, float* weight, int tokens, int experts, int top, int softmax, int renormalize,
                               const float* correction, int group_count, int group_keep, float norm_floor, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (experts < 1 || experts > 64 * ROUTE_PER_LANE || top < 1 || top > experts) return -1;
  if (group_count < 0 || group_count > 64 ||
      (group_count > 0 && (experts % group_count != 0 || group_keep < 1 || group_keep > group_count || group_keep * (experts / group_count) < top)))
    return -1;
  route_top_kernel<<<(tokens + 3) / 4, 256, 0, stream>>>(logits, choice, weight, tokens, experts, top, softmax, renormalize, correction, group_count,
                                                         group_keep, norm_floor);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// The plan, int32: [0] number of tiles, [1 .. 1 + E] first sorted row of every expert and the total, then order[P]
// (sorted row -> pair = token * top + k), place[P] (pair -> sorted row), tile_expert[max_tiles], tile_row[max_tiles]; a tile
// is up to tile_rows consecutive sorted rows of one expert.
// ---------------------------------------------------------------------------------------------
#define PLAN_MAX_EXPERTS 2048
#define PLAN_COPY_PAIRS 64  // up to this many pairs the plan kernel can copy the rows itself

// With `sorted` the kernel also copies the rows of x into the plan's order (scaled by the pair's weight when `scale`), what
// routed_gather_kernel does: for steps of few pairs, which then run one kernel less.
__global__ void __launch_bounds__(1024) routed_plan_kernel(const int* __restrict__ choice, int pairs, int experts, int max_tiles, int tile_rows,
                                                           int* __restrict__ plan, const bf16_t* __restrict__ x, bf16_t* __restrict__ sorted,
                                                           const float* __restrict__ pair_weight, int top, int hidden, int scale) {
  __shared__ int count[PLAN_MAX_EXPERTS];
  __shared__ int first[PLAN_MAX_EXPERTS + 1];
  __shared__ int order_s[PLAN_COPY_PAIRS];
  int* num_tiles = plan;
  int* starts = plan + 1;
  int* order = starts + experts + 1;
  int* place = order + pairs;
  int* tile_expert = place + pairs;
  int* tile_row = tile_expert + max_tiles;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = choice[p];
    if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = at;
      starts[e] = at;
      for (int r = 0; r < count[e] && tiles < max_tiles; r += tile_rows) {
        tile_expert[tiles] = e;
        tile_row[tiles] = at + r;
        ++tiles;
      }
      at += count[e];
      count[e] = 0;  // (from here on: how many of the expert's rows are placed)
    }
    first[experts] = at;
    starts[experts] = at;
    *num_tiles = tiles;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = choice[p];
    if (e < 0 || e >= experts) { place[p] = -1; continue; }
    const int row = first[e] + atomicAdd(&count[e], 1);
    order[row] = p;
    place[p] = row;
    if (sorted != nullptr) order_s[row] = p;
  }
  if (sorted == nullptr) return;  // (uniform over the workgroup)
  __syncthreads();
  // the rows of x in the plan's order, 16 bytes per thread at a time (the caller checked hidden % 8 == 0 and pairs <= PLAN_COPY_PAIRS)
  const int pieces = hidden / 8;
  for (int at = threadIdx.x; at < first[experts] * pieces; at += blockDim.x) {  // (first[experts]: the pairs that were placed)
    const int row = at / pieces, piece_at = at % pieces;
    const int p = order_s[row];
    float4_t piece = reinterpret_cast<const float4_t*>(x + (size_t)(p / top) * hidden)[piece_at];
    if (scale) {
      const float w = pair_weight[p];
      bf16_t* e8 = reinterpret_cast<bf16_t*>(&piece);
#pragma unroll
      for (int j = 0; j < 8; ++j) e8[j] = from_f32<bf16_t>(to_f32(e8[j]) * w);
    }
    reinterpret_cast<float4_t*>(sorted + (size_t)row * hidden)[piece_at] = piece;
  }
}

extern "C" long long velox_routed_plan_elems(int pairs, int experts) {
  const long long max_tiles = (pairs + RT_BM - 1) / RT_BM + experts;
  return 1 + (experts + 1) + 2LL * pairs + 2 * max_tiles;
}

extern "C" int velox_routed_max_tiles(int pairs, int experts) { return (pairs + RT_BM - 1) / RT_BM + experts; }

// tile_rows: 64, or 128 for the matrix-core products of a step with many rows per expert.  The plan's layout is that of
// 64-row tiles either way (the most tiles there can be).
// x, sorted, pair_weight, top, hidden, scale: see routed_plan_kernel (sorted == nullptr: the plan alone).
extern "C" int velox_routed_plan(const int* choice, int pairs, int experts, int* plan, int tile_rows, const void* x, void* sorted, const float* pair_weight,
                                 int top, int hidden, int scale, hipStream_t stream) {
  if (pairs <= 0) return 0;
  if (experts < 1 || experts > PLAN_MAX_EXPERTS || (tile_rows != RT_BM && tile_rows != 2 * RT_BM)) return -1;
  if (sorted != nullptr && (x == nullptr || pairs > PLAN_COPY_PAIRS || hidden % 8 != 0 || top < 1 || (((uintptr_t)x | (uintptr_t)sorted) & 15) != 0)) return -1;
  routed_plan_kernel<<<1, 1024, 0, stream>>>(choice, pairs, experts, velox_routed_max_tiles(pairs, experts), tile_rows, plan, (const bf16_t*)x, (bf16_t*)sorted,
                                             pair_weight, top, hidden, scale);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// The grouped products.  GLU: two tiles of W (gate rows and the up rows of the same columns), the activation as the
// epilogue.  Rows of A: GLU gathers x[token] (scaled by the pair's weight and rounded to T, as a product on T operands
// would read it); the down product reads the sorted rows of act.  FIRST = 2: a unit without a gate branch, one tile of
// W (the up rows), rows gathered as for GLU, ungated_act(., act_kind) as the epilogue.
// ---------------------------------------------------------------------------------------------
template <typename T, typename TO, int FIRST>
__global__ void __launch_bounds__(256) grouped_product_kernel(const T* __restrict__ a, const T* __restrict__ w, TO* __restrict__ out,
                                                              const int* __restrict__ plan, const float* __restrict__ pair_weight, int pairs, int experts,
                                                              int max_tiles, int top, int n, int k, int scale_rows, int a_vec, int w_vec, GluUnit unit,
                                                              int act_kind) {
  constexpr bool GLU = FIRST == 1;       // two tiles of W and the gated epilogue
  constexpr bool GATHERS = FIRST != 0;   // rows are x[token of the pair], not sorted rows
  __shared__ float a_tile[RT_BK][RT_BM + RT_PAD];
  __shared__ float w_tile[GLU ? 2 : 1][RT_BK][RT_BN + RT_PAD];
  __shared__ int row_pair[RT_BM];
  const int tile = blockIdx.y;
  if (tile >= plan[0]) return;  // (uniform over the workgroup)
  const int* starts = plan + 1;
  const int* order = starts + experts + 1;
  const int* tile_expert = order + 2 * (size_t)pairs;
  const int* tile_row = tile_expert + max_tiles;
  const int e = tile_expert[tile];
  const int row0 = tile_row[tile];
  const int rows = min(RT_BM, starts[e + 1] - row0);
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int n0 = blockIdx.x * RT_BN;
  const int load_row = tid / 4, load_k = (tid % 4) * 4;
  if (tid < RT_BM) row_pair[tid] = tid < rows ? order[row0 + tid] : -1;
  __syncthreads();
  const bool a_row_ok = load_row < rows;
  const int my_pair = row_pair[load_row];
  size_t a_off = 0;
  float a_scale = 1.f;
  if (a_row_ok) {
    if (GATHERS) {
      a_off = (size_t)(my_pair / top) * k;
      if (scale_rows) a_scale = pair_weight[my_pair];
    } else {
      a_off = (size_t)(row0 + load_row) * k;
    }
  }
  const bool w_row_ok = n0 + load_row < n;
  const size_t w_rows = GLU ? 2 * (size_t)n : (size_t)n;  // rows of one expert's matrix
  const size_t w_off = ((size_t)e * w_rows + n0 + load_row) * k;
  const size_t up_off = w_off + (size_t)n * k;

  constexpr int NW = GLU ? 2 : 1;
  float acc[NW][4][4], total[NW][4][4];
#pragma unroll
  for (int u = 0; u < NW; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[u][i][j] = total[u][i][j] = 0.f;

  for (int k0 = 0; k0 < k; k0 += RT_BK) {
    if (k0 % RT_FOLD == 0) {
#pragma unroll
      for (int u = 0; u < NW; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            total[u][i][j] += acc[u][i][j];
            acc[u][i][j] = 0.f;
          }
    }
    float av[4], wv[NW][4];
    load4<T>(a, a_off, k0 + load_k, k, a_row_ok, a_vec != 0, av);
    if (GATHERS && scale_rows) {
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = to_f32(from_f32<T>(av[i] * a_scale));
    }
    load4<T>(w, w_off, k0 + load_k, k, w_row_ok, w_vec != 0, wv[0]);
    if (GLU) load4<T>(w, up_off, k0 + load_k, k, w_row_ok, w_vec != 0, wv[NW - 1]);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a_tile[load_k + i][load_row] = av[i];
#pragma unroll
      for (int u = 0; u < NW; ++u) w_tile[u][load_k + i][load_row] = wv[u][i];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < RT_BK; ++kk) {
      const float4_t ar = *reinterpret_cast<const float4_t*>(&a_tile[kk][ty * 4]);
#pragma unroll
      for (int u = 0; u < NW; ++u) {
        const float4_t wr = *reinterpret_cast<const float4_t*>(&w_tile[u][kk][tx * 4]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[u][i][j] = fmaf(ar[i], wr[j], acc[u][i][j]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= rows) continue;
    const float row_scale = (!GATHERS && scale_rows) ? pair_weight[row_pair[r]] : 1.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= n) continue;
      float v = total[0][i][j] + acc[0][i][j];
      if (GLU) {
        const float up = total[NW - 1][i][j] + acc[NW - 1][i][j];
        v = glu_middle(v, up, unit);  // (float32 throughout, one rounding at the store)
      } else if (FIRST == 2) {
        v = ungated_act(v, act_kind);
      } else {
        v *= row_scale;
      }
      out[(size_t)(row0 + r) * n + col] = from_f32<TO>(v);
    }
  }
}

extern "C" int velox_grouped_glu(const void* x, const void* gate_up, void* act, const int* plan, const float* pair_weight, int pairs, int experts, int top,
                                 int inter, int hidden, int scale_input, int dtype, float alpha, float limit, float shift, int ungated, hipStream_t stream) {
  // `ungated` > 0: `gate_up` holds [experts * inter, hidden] (up rows only) and the unit is ungated_act(up, ungated)
  if (pairs <= 0) return 0;
  const GluUnit unit = {alpha, limit, shift};
  const int max_tiles = velox_routed_max_tiles(pairs, experts);
  dim3 grid((inter + RT_BN - 1) / RT_BN, max_tiles);
  if (grid.y > 65535) return -1;
  const int size = dtype == VELOX_BF16 ? 2 : 4;
  const int a_vec = hidden % 4 == 0 && ((uintptr_t)x) % (4 * size) == 0;
  const int w_vec = hidden % 4 == 0 && ((uintptr_t)gate_up) % (4 * size) == 0;
  if (ungated > 0) {
    if (dtype == VELOX_BF16)
      grouped_product_kernel<bf16_t, bf16_t, 2><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)gate_up, (bf16_t*)act, plan, pair_weight, pairs, experts,
                                                                          max_tiles, top, inter, hidden, scale_input, a_vec, w_vec, unit, ungated);
    else
      grouped_product_kernel<float, float, 2><<<grid, 256, 0, stream>>>((const float*)x, (const float*)gate_up, (float*)act, plan, pair_weight, pairs, experts,
                                                                        max_tiles, top, inter, hidden, scale_input, a_vec, w_vec, unit, ungated);
    VELOX_RETURN_LAUNCH_STATUS();
  }
  if (dtype == VELOX_BF16)
    grouped_product_kernel<bf16_t, bf16_t, 1><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)gate_up, (bf16_t*)act, plan, pair_weight, pairs, experts,
                                                                        max_tiles, top, inter, hidden, scale_input, a_vec, w_vec, unit, 0);
  else
    grouped_product_kernel<float, float, 1><<<grid, 256, 0, stream>>>((const float*)x, (const float*)gate_up, (float*)act, plan, pair_weight, pairs, experts,
                                                                      max_tiles, top, inter, hidden, scale_input, a_vec, w_vec, unit, 0);
  VELOX_RETURN_LAUNCH_STATUS();
}

extern "C" int velox_grouped_down(const void* act, const void* down, float* y, const int* plan, const float* pair_weight, int pairs, int experts, int top,
                                  int hidden, int inter, int scale_output, int dtype, hipStream_t stream) {
  if (pairs <= 0) return 0;
  const int max_tiles = velox_routed_max_tiles(pairs, experts);
  dim3 grid((hidden + RT_BN - 1) / RT_BN, max_tiles);
  if (grid.y > 65535) return -1;
  const int size = dtype == VELOX_BF16 ? 2 : 4;
  const int a_vec = inter % 4 == 0 && ((uintptr_t)act) % (4 * size) == 0;
  const int w_vec = inter % 4 == 0 && ((uintptr_t)down) % (4 * size) == 0;
  if (dtype == VELOX_BF16)
    grouped_product_kernel<bf16_t, float, 0><<<grid, 256, 0, stream>>>((const bf16_t*)act, (const bf16_t*)down, y, plan, pair_weight, pairs, experts, max_tiles,
                                                                       top, hidden, inter, scale_output, a_vec, w_vec, GluUnit{1.f, INFINITY, 0.f}, 0);
  else
    grouped_product_kernel<float, float, 0><<<grid, 256, 0, stream>>>((const float*)act, (const float*)down, y, plan, pair_weight, pairs, experts, max_tiles,
                                                                      top, hidden, inter, scale_output, a_vec, w_vec, GluUnit{1.f, INFINITY, 0.f}, 0);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// bfloat16 on the matrix cores: the rows of x are first copied into the order of the plan (and scaled, when the pair's
// weight scales the expert's input: float32 product, one rounding), then both grouped products read sorted rows.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) routed_gather_kernel(const bf16_t* __restrict__ x, const int* __restrict__ order, const float* __restrict__ pair_weight,
                                                            bf16_t* __restrict__ sorted, int top, int hidden, int scale, const int* __restrict__ placed) {
  const int row = blockIdx.x;
  if (row >= *placed) return;  // (pairs whose expert the plan leaves out have no row: `order` ends at the placed ones)
  const int pair = order[row];
  const bf16_t* src = x + (size_t)(pair / top) * hidden;
  bf16_t* dst = sorted + (size_t)row * hidden;
  const float w = scale ? pair_weight[pair] : 1.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = scale ? from_f32<bf16_t>(to_f32(src[i]) * w) : src[i];
}

static GroupedArgs routed_args(const void* a, const void* w, void* out, const int* plan, int pairs, int experts, int n, int k, int w_rows) {
  GroupedArgs args = {};
  args.a = (const bf16_t*)a;
  args.a_ld = k;
  args.w = (const bf16_t*)w;
  args.w_group = (long long)w_rows * k;
  args.out = out;
  args.out_ld = n;
  args.n = n;
  args.k = k;
  args.plan = plan;
  args.plan_pairs = pairs;
  args.plan_groups = experts;
  args.plan_max_tiles = velox_routed_max_tiles(pairs, experts);
  return args;
}

// x [T, hidden] -> sorted [pairs, hidden] -> act [pairs, inter] -> y [pairs, hidden] float32.  Needs hidden % 8 == 0 and
// inter % 8 == 0 (the caller checks).
extern "C" int velox_routed_products_bf16(const void* x, const void* gate_up, const void* down, void* sorted, void* act, float* y, const int* plan,
                                          const float* pair_weight, int pairs, int experts, int top, int inter, int hidden, int scale_input,
                                          int tile_rows, float alpha, float limit, float shift, int ungated, hipStream_t stream) {
  // `ungated` > 0: `gate_up` holds [experts * inter, hidden] (up rows only) and the unit is ungated_act(up, ungated)
  if (pairs <= 0) return 0;
  if (hidden % 8 != 0 || inter % 8 != 0) return -1;
  const int max_tiles = velox_routed_max_tiles(pairs, experts);
  if (max_tiles > 65535) return -1;
  const int* order = plan + 1 + (experts + 1);
  if (x != nullptr)  // (nullptr: the plan kernel has copied the rows already)
    routed_gather_kernel<<<pairs, 256, 0, stream>>>((const bf16_t*)x, order, pair_weight, (bf16_t*)sorted, top, hidden, scale_input, plan + 1 + experts);
  if (ungated > 0) {
    GroupedArgs first = routed_args(sorted, gate_up, act, plan, pairs, experts, inter, hidden, inter);
    first.act = ungated;
    grouped_mfma_launch<GM_ACT, bf16_t>(first, pairs, tile_rows, max_tiles, 1, stream);
  } else {
    GroupedArgs glu = routed_args(sorted, gate_up, act, plan, pairs, experts, inter, hidden, 2 * inter);
    glu.unit = GluUnit{alpha, limit, shift};
    grouped_mfma_launch<GM_GLU, bf16_t>(glu, pairs, tile_rows, max_tiles, 1, stream);
  }
  GroupedArgs last = routed_args(act, down, y, plan, pairs, experts, hidden, inter, hidden);
  // (a weight on the experts' OUTPUT is applied where the results are added up, routed_combine with scale_rows: the product
  // itself is the same kernel either way)
  grouped_mfma_launch<GM_PLAIN, float>(last, pairs, tile_rows, max_tiles, 1, stream);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// out[t, :] = (sum_k y[place[t * top + k], :]) + shared[t, :], the choices added in order, one rounding at the store.
// With `x`: a choice that the plan has not placed (an identity expert, whose index lies behind the real ones) adds
// pair_weight[t * top + k] * x[t, :] in its turn.  With `scale_rows` every row of y is multiplied with its pair's weight here
// (the products then left it out).
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) routed_combine_kernel(const float* __restrict__ y, const int* __restrict__ place, const T* __restrict__ shared,
                                                             T* __restrict__ out, int top, int hidden, const T* __restrict__ x,
                                                             const float* __restrict__ pair_weight, int scale_rows) {
  __shared__ int rows[64];  // the token's rows of y, looked up once (up to 64 choices; more are looked up as they are added)
  const int t = blockIdx.x;
  const int* mine = place + (size_t)t * top;
  if (top <= 64) {
    if (threadIdx.x < top) rows[threadIdx.x] = mine[threadIdx.x];
    __syncthreads();
    mine = rows;
  }
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = 0.f;
    for (int k = 0; k < top; ++k) {
      const int row = mine[k];
      if (row >= 0) v += scale_rows ? pair_weight[(size_t)t * top + k] * y[(size_t)row * hidden + i] : y[(size_t)row * hidden + i];
      else if (x) v += pair_weight[(size_t)t * top + k] * to_f32(x[(size_t)t * hidden + i]);
    }
    if (shared) v += to_f32(shared[(size_t)t * hidden + i]);
    out[(size_t)t * hidden + i] = from_f32<T>(v);
  }
}

// The same sum, handed straight to a norm on the experts' output: residual[t, :] += mult * v * rsqrt(mean(v^2) + eps) * w, with v the
// sum above in float32 (never rounded to T), and `copy` (nullable) the updated residual in T.  One workgroup per token holds
// the row in registers: hidden <= 16 * blockDim.x.
template <typename T>
__global__ void routed_combine_norm_kernel(const float* __restrict__ y, const int* __restrict__ place, const T* __restrict__ shared, int top, int hidden,
                                           const T* __restrict__ x, const float* __restrict__ pair_weight, int scale_rows, float* __restrict__ residual,
                                           const float* __restrict__ norm_weight, float eps, float mult, T* __restrict__ copy) {
  __shared__ int rows[64];
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int* mine = place + (size_t)t * top;
  if (top <= 64) {
    if (threadIdx.x < top) rows[threadIdx.x] = mine[threadIdx.x];
    __syncthreads();
    mine = rows;
  }
  float held[16];
  float sumsq = 0.f;
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    const int i = threadIdx.x + c * blockDim.x;
    float v = 0.f;
    if (i < hidden) {
      for (int k = 0; k < top; ++k) {
        const int row = mine[k];
        if (row >= 0) v += scale_rows ? pair_weight[(size_t)t * top + k] * y[(size_t)row * hidden + i] : y[(size_t)row * hidden + i];
        else if (x) v += pair_weight[(size_t)t * top + k] * to_f32(x[(size_t)t * hidden + i]);
      }
      if (shared) v += to_f32(shared[(size_t)t * hidden + i]);
    }
    held[c] = v;
    sumsq += v * v;
  }
  const float total = block_sum(sumsq, scratch);
  const float inv = 1.f / sqrtf(total / (float)hidden + eps);
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    const int i = threadIdx.x + c * blockDim.x;
    if (i < hidden) {
      const float r = residual[(size_t)t * hidden + i] + mult * (held[c] * inv * norm_weight[i]);
      residual[(size_t)t * hidden + i] = r;
      if (copy) copy[(size_t)t * hidden + i] = from_f32<T>(r);
    }
  }
}

// copy: nullptr in a float32 run (the residual is its own copy).  Returns -1 when the row does not fit the registers
// (hidden > 16,384): the caller then runs the two kernels one after the other.
extern "C" int velox_routed_combine_norm(const float* y, const int* plan, const void* shared, int tokens, int top, int experts, int hidden, int dtype,
                                         const void* x, const float* pair_weight, int scale_rows, float* residual, const float* norm_weight, float eps,
                                         float mult, void* copy, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden > 16 * 1024) return -1;
  const int* place = plan + 1 + (experts + 1) + (size_t)tokens * top;
  int threads = tokens <= 64 ? 512 : 256;  // (few rows: more threads each with less to do)
  while (16 * threads < hidden) threads *= 2;
  if (dtype == VELOX_BF16)
    routed_combine_norm_kernel<bf16_t><<<tokens, threads, 0, stream>>>(y, place, (const bf16_t*)shared, top, hidden, (const bf16_t*)x, pair_weight, scale_rows,
                                                                       residual, norm_weight, eps, mult, (bf16_t*)copy);
  else
    routed_combine_norm_kernel<float><<<tokens, threads, 0, stream>>>(y, place, (const float*)shared, top, hidden, (const float*)x, pair_weight, scale_rows,
                                                                      residual, norm_weight, eps, mult, (float*)copy);
  VELOX_RETURN_LAUNCH_STATUS();
}

extern "C" int velox_routed_combine(const float* y, const int* plan, const void* shared, void* out, int tokens, int top, int experts, int hidden, int dtype,
                                    const void* x, const float* pair_weight, int scale_rows, hipStream_t stream) {
  if (tokens <= 0) return 0;
  const int* place = plan + 1 + (experts + 1) + (size_t)tokens * top;
  if (dtype == VELOX_BF16)
    routed_combine_kernel<bf16_t><<<tokens, 256, 0, stream>>>(y, place, (const bf16_t*)shared, (bf16_t*)out, top, hidden, (const bf16_t*)x, pair_weight, scale_rows);
  else
    routed_combine_kernel<float><<<tokens, 256, 0, stream>>>(y, place, (const float*)shared, (float*)out, top, hidden, (const float*)x, pair_weight, scale_rows);
  VELOX_RETURN_LAUNCH_STATUS();
}
