// Kernels of attention over a cached latent, for gfx950.
//
//   latent_rotate_write: per token, the rotation of every head's rotated query part into the queries the attention
//     kernels read, and (for a layer that makes its own latent) the RMS norm of the latent, the rotation of the shared key
//     part and the write of both into the paged cache, as keys [page, 1, offset, D] and transposed as values
//     [page, 1, D, offset].  All arithmetic is float32; values are rounded once, at the store.
//   head_linear: one small product per head over the step's tokens, out[t, g] = maps[g] x[t, g], with heads at fixed
//     strides inside the rows of x and out, and optionally a sigmoid gate as its epilogue.
#include "common.h"
#include "grouped_mfma.h"

// ---------------------------------------------------------------------------------------------
// One block per token.  A row of `projected` holds [q: heads x (dim + rot) | ... | down: rank + rot at down_offset].
//   queries[t, h, rank + c]       = rotated(q[t, h, dim + c]),  c < rot
//   queries[t, h, rank + rot ..]  = 0 up to D (the first `rank` channels of a head are written by head_linear)
//   down_offset >= 0:  cached[0 .. rank) = latent / sqrt(mean(latent^2) + eps) * norm_weight
//                      cached[rank .. rank + rot) = rotated(shared key part), cached[rank + rot .. D) = 0
// The rotation turns the first 2 * half channels of a rotated part and passes the rest: pairs are (2i, 2i + 1) when
// `interleaved`, else (i, i + half); (u, v) -> (u cos - v sin, v cos + u sin) with cos/sin = table[position, i].
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float rotated_channel(float own, float partner, bool is_first, float c, float s) {
  return is_first ? own * c - partner * s : own * c + partner * s;
}

template <typename T>
__device__ __forceinline__ float rotate_at(const T* __restrict__ part, int ch, int half, bool interleaved, const float* __restrict__ cs,
                                           const float* __restrict__ sn) {
  const float own = to_f32(part[ch]);
  if (ch >= 2 * half) return own;
  int i, partner;
  bool first;
  if (interleaved) { i = ch >> 1; partner = ch ^ 1; first = (ch & 1) == 0; }
  else { first = ch < half; i = first ? ch : ch - half; partner = first ? ch + half : ch - half; }
  return rotated_channel(own, to_f32(part[partner]), first, cs[i], sn[i]);
}

template <typename T>
__global__ void __launch_bounds__(256) latent_rotate_write_kernel(const T* __restrict__ projected, int width, T* __restrict__ queries, int heads, int dim,
                                                                  int rot, int rank, int cached, int down_offset, const int* __restrict__ positions,
                                                                  const float* __restrict__ cos_table, const float* __restrict__ sin_table, int half,
                                                                  int interleaved, const float* __restrict__ norm_weight, float eps,
                                                                  const int* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                                  int page_size, int norm2_offset, int norm2_size, const float* __restrict__ norm2_weight,
                                                                  T* __restrict__ norm2_out) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = projected + (size_t)t * width;
  if (norm2_out != nullptr) {  // (uniform) a second slice of the row, RMS-normed with its own weight: the queries' latent
    const T* part = row + norm2_offset;
    float sq = 0.f;
    for (int i = threadIdx.x; i < norm2_size; i += blockDim.x) {
      const float x = to_f32(part[i]);
      sq += x * x;
    }
    const float inv2 = 1.0f / sqrtf(block_sum(sq, scratch) / (float)norm2_size + eps);
    T* dst = norm2_out + (size_t)t * norm2_size;
    for (int i = threadIdx.x; i < norm2_size; i += blockDim.x) dst[i] = from_f32<T>(to_f32(part[i]) * inv2 * norm2_weight[i]);
  }
  const int pos = positions[t];
  const float* cs = half ? cos_table + (size_t)pos * half : nullptr;
  const float* sn = half ? sin_table + (size_t)pos * half : nullptr;
  const int tail = cached - rank;  // channels of a head's query behind the room for the mapped plain part
  T* q_out = queries + (size_t)t * heads * cached;
  for (int item = threadIdx.x; item < heads * tail; item += blockDim.x) {
    const int h = item / tail, c = item % tail;
    float v = 0.f;
    if (c < rot) v = rotate_at<T>(row + h * (dim + rot) + dim, c, half, interleaved != 0, cs, sn);
    q_out[h * cached + rank + c] = from_f32<T>(v);
  }
  if (down_offset < 0) return;  // (uniform over the block)
  const T* down = row + down_offset;
  float sumsq = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float x = to_f32(down[i]);
    sumsq += x * x;
  }
  const float inv = 1.0f / sqrtf(block_sum(sumsq, scratch) / (float)rank + eps);
  const int slot = slots[t];
  const size_t page = (size_t)(slot / page_size);
  const int offset = slot % page_size;
  T* k_dst = k_cache + (page * page_size + offset) * cached;
  T* v_dst = v_cache + page * cached * page_size + offset;
  for (int i = threadIdx.x; i < cached; i += blockDim.x) {
    float v = 0.f;
    if (i < rank) v = to_f32(down[i]) * inv * norm_weight[i];
    else if (i < rank + rot) v = rotate_at<T>(down + rank, i - rank, half, interleaved != 0, cs, sn);
    const T stored = from_f32<T>(v);
    k_dst[i] = stored;
    v_dst[(size_t)i * page_size] = stored;
  }
}

extern "C" int velox_latent_rotate_write(const void* projected, int width, void* queries, int tokens, int heads, int dim, int rot, int rank, int cached,
                                         int down_offset, const int* positions, const float* cos_table, const float* sin_table, int half, int interleaved,
                                         const float* norm_weight, float eps, const int* slots, void* k_cache, void* v_cache, int page_size, int dtype,
                                         int norm2_offset, int norm2_size, const float* norm2_weight, void* norm2_out, hipStream_t stream) {
  if (tokens <= 0) return 0;
  // (heads == 0: no queries, only the cache write and the second norm)
  if (heads < 0 || dim < 0 || (heads > 0 && dim < 1) || rot < 0 || rank < 1 || cached < rank + rot || 2 * half > rot || page_size < 1) return -1;
  if (heads * (dim + rot) > width || (down_offset >= 0 && (down_offset + rank + rot > width || norm_weight == nullptr))) return -1;
  if (norm2_out != nullptr && (norm2_offset < 0 || norm2_size < 1 || norm2_offset + norm2_size > width || norm2_weight == nullptr)) return -1;
  if (dtype == VELOX_BF16)
    latent_rotate_write_kernel<bf16_t><<<tokens, 256, 0, stream>>>((const bf16_t*)projected, width, (bf16_t*)queries, heads, dim, rot, rank, cached, down_offset,
                                                                   positions, cos_table, sin_table, half, interleaved, norm_weight, eps, slots,
                                                                   (bf16_t*)k_cache, (bf16_t*)v_cache, page_size, norm2_offset, norm2_size, norm2_weight,
                                                                   (bf16_t*)norm2_out);
  else
    latent_rotate_write_kernel<float><<<tokens, 256, 0, stream>>>((const float*)projected, width, (float*)queries, heads, dim, rot, rank, cached, down_offset,
                                                                  positions, cos_table, sin_table, half, interleaved, norm_weight, eps, slots,
                                                                  (float*)k_cache, (float*)v_cache, page_size, norm2_offset, norm2_size, norm2_weight,
                                                                  (float*)norm2_out);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// head_linear: out[t, g * out_stride + out_offset + j] = sum_k x[t, g * x_stride + x_offset + k] * maps[g, j, k]
//   (* sigmoid(gate[t, gate_offset + g * n + j]) with a gate), for t < m, g < groups, j < n.
// bfloat16 operands whose rows start on 16-byte boundaries go to the matrix cores (grouped_mfma.h).  Everything else:
// exact float32 multiply-adds on 64 x 64 tiles through LDS, a head per blockIdx.z; every element is summed over k in one
// fixed order by one thread, in inner sums of 128 terms (as the framework's float32 product does), so a row's result
// depends on that row alone.
// ---------------------------------------------------------------------------------------------
#define HL_BM 64
#define HL_BN 64
#define HL_BK 16
#define HL_PAD 4
#define HL_FOLD 128

template <typename T>
__global__ void __launch_bounds__(256) head_linear_kernel(const T* __restrict__ x, int x_width, int x_stride, int x_offset, const T* __restrict__ maps,
                                                          T* __restrict__ out, int out_width, int out_stride, int out_offset,
                                                          const T* __restrict__ gate, int gate_width, int gate_offset, int m, int n, int k,
                                                          int x_vec, int w_vec, int gate_per_head) {
  __shared__ float a_tile[HL_BK][HL_BM + HL_PAD];
  __shared__ float w_tile[HL_BK][HL_BN + HL_PAD];
  const int g = blockIdx.z;
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * HL_BM, n0 = blockIdx.x * HL_BN;
  const int load_row = tid / 4, load_k = (tid % 4) * 4;
  const bool a_row_ok = m0 + load_row < m;
  const bool w_row_ok = n0 + load_row < n;
  const size_t a_off = (size_t)(m0 + load_row) * x_width + (size_t)g * x_stride + x_offset;
  const size_t w_off = ((size_t)g * n + n0 + load_row) * k;
  float acc[4][4], total[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = total[i][j] = 0.f;
  for (int k0 = 0; k0 < k; k0 += HL_BK) {
    if (k0 % HL_FOLD == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
    float av[4], wv[4];
    load4<T>(x, a_off, k0 + load_k, k, a_row_ok, x_vec != 0, av);
    load4<T>(maps, w_off, k0 + load_k, k, w_row_ok, w_vec != 0, wv);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a_tile[load_k + i][load_row] = av[i];
      w_tile[load_k + i][load_row] = wv[i];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HL_BK; ++kk) {
      const float4_t ar = *reinterpret_cast<const float4_t*>(&a_tile[kk][ty * 4]);
      const float4_t wr = *reinterpret_cast<const float4_t*>(&w_tile[kk][tx * 4]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(ar[i], wr[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + ty * 4 + i;
    if (row >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= n) continue;
      float v = total[i][j] + acc[i][j];
      if (gate) {
        const float z = to_f32(gate[(size_t)row * gate_width + gate_offset + (gate_per_head ? g : g * n + col)]);
        v *= 1.f / (1.f + expf(-z));
      }
      out[(size_t)row * out_width + (size_t)g * out_stride + out_offset + col] = from_f32<T>(v);
    }
  }
}

extern "C" int velox_head_linear(const void* x, int x_width, int x_stride, int x_offset, const void* maps, void* out, int out_width, int out_stride,
                                 int out_offset, const void* gate, int gate_width, int gate_offset, int m, int groups, int n, int k, int dtype,
                                 int gate_per_head, hipStream_t stream) {
  if (m <= 0 || groups <= 0 || n <= 0) return 0;
  if (k < 1 || groups > 65535 || (groups - 1) * x_stride + x_offset + k > x_width || (groups - 1) * out_stride + out_offset + n > out_width) return -1;
  // (gate_per_head: the gate holds one number per group, times every output of the group)
  if (gate != nullptr && gate_offset + (gate_per_head ? groups : groups * n) > gate_width) return -1;
  if (dtype == VELOX_BF16 && grouped_mfma_fits(x, x_width, x_stride, x_offset, maps, k)) {
    // bfloat16: the same sums on the matrix cores
    GroupedArgs args = {};
    args.a = (const bf16_t*)x + x_offset;
    args.a_ld = x_width;
    args.a_group = x_stride;
    args.w = (const bf16_t*)maps;
    args.w_group = (long long)n * k;
    args.out = (bf16_t*)out + out_offset;
    args.out_ld = out_width;
    args.out_group = out_stride;
    args.n = n;
    args.k = k;
    args.m = m;
    args.gate = gate ? (const bf16_t*)gate + gate_offset : nullptr;
    args.gate_ld = gate_width;
    args.gate_group = gate_per_head ? 1 : n;
    args.gate_col = gate_per_head ? 0 : 1;
    const int row_tiles = (m + GM_ROWS - 1) / GM_ROWS;
    if (row_tiles > 65535) return -1;
    if (gate) grouped_mfma_launch<GM_GATE, bf16_t>(args, m, GM_ROWS, row_tiles, groups, stream);
    else grouped_mfma_launch<GM_PLAIN, bf16_t>(args, m, GM_ROWS, row_tiles, groups, stream);
    VELOX_RETURN_LAUNCH_STATUS();
  }
  dim3 grid((n + HL_BN - 1) / HL_BN, (m + HL_BM - 1) / HL_BM, groups);
  if (grid.y > 65535) return -1;
  const int size = dtype == VELOX_BF16 ? 2 : 4;
  const int x_vec = k % 4 == 0 && x_width % 4 == 0 && x_stride % 4 == 0 && x_offset % 4 == 0 && ((uintptr_t)x) % (4 * size) == 0;
  const int w_vec = k % 4 == 0 && ((uintptr_t)maps) % (4 * size) == 0;
  if (dtype == VELOX_BF16)
    head_linear_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_width, x_stride, x_offset, (const bf16_t*)maps, (bf16_t*)out, out_width, out_stride,
                                                         out_offset, (const bf16_t*)gate, gate_width, gate_offset, m, n, k, x_vec, w_vec, gate_per_head);
  else
    head_linear_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_width, x_stride, x_offset, (const float*)maps, (float*)out, out_width, out_stride,
                                                        out_offset, (const float*)gate, gate_width, gate_offset, m, n, k, x_vec, w_vec, gate_per_head);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// Attention over the paged cache for head sizes beyond the tiled kernels' 256 channels (any size up to 1,024): one
// workgroup per (token, head), plain float32 arithmetic.  Keys [page, kv_head, offset, d], values transposed
// [page, kv_head, d, offset].  256 keys at a time: a thread takes one key's score (the query sits in LDS), the workgroup
// takes the maximum and the sum, and then every thread adds the 256 weighted values of its own channels; a running
// maximum rescales what was added before.  Probabilities stay float32.
// ---------------------------------------------------------------------------------------------
#define PLAIN_ATTENTION_MAX_D 1024

__device__ __forceinline__ float block_max_256(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  return fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
}

template <typename T>
__global__ void __launch_bounds__(256) plain_attention_kernel(const T* __restrict__ q, int q_width, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                                              const int* __restrict__ block_tables, int table_width, const int* __restrict__ cu_q,
                                                              const int* __restrict__ kv_lens, T* __restrict__ out, int num_seqs, int nh, int nkv, int d,
                                                              int page_shift, float scale, int window, const float* __restrict__ bias_table, int bias_len,
                                                              const float* __restrict__ sinks) {
  __shared__ float q_s[PLAIN_ATTENTION_MAX_D];
  __shared__ float p_s[256];
  __shared__ float scratch[16];
  __shared__ int seq_s;
  const int token = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  if (tid == 0) {
    int b = 0;
    while (b + 1 < num_seqs && cu_q[b + 1] <= token) ++b;
    seq_s = b;
  }
  for (int c = tid; c < d; c += 256) q_s[c] = to_f32(q[(size_t)token * q_width + (size_t)head * d + c]);
  __syncthreads();
  const int b = seq_s;
  const int kv_len = kv_lens[b];
  const int last = kv_len - (cu_q[b + 1] - cu_q[b]) + (token - cu_q[b]);  // this token's position: the last key it sees
  const int first = window > 0 ? max(0, last - window + 1) : 0;
  const int kvh = head / (nh / nkv);
  const int page_size = 1 << page_shift;
  const int* table = block_tables + (size_t)b * table_width;
  float running_max = -INFINITY, denom = 0.f;
  float acc[PLAIN_ATTENTION_MAX_D / 256];
#pragma unroll
  for (int u = 0; u < PLAIN_ATTENTION_MAX_D / 256; ++u) acc[u] = 0.f;
  for (int j0 = first; j0 <= last; j0 += 256) {
    const int j = j0 + tid;
    float s = -INFINITY;
    if (j <= last) {
      const T* key = k_cache + (((size_t)table[j >> page_shift] * nkv + kvh) * page_size + (j & (page_size - 1))) * d;
      float dot = 0.f;
      for (int c = 0; c < d; ++c) dot = fmaf(q_s[c], to_f32(key[c]), dot);
      s = dot * scale;
      // a bias by distance, float32 [nh, bias_len]: the key n positions behind the query reads column min(n, bias_len - 1)
      if (bias_table) s += bias_table[(size_t)head * bias_len + min(last - j, bias_len - 1)];
    }
    const float new_max = fmaxf(running_max, block_max_256(s, scratch));  // (finite: key j0 is always seen)
    const float p = j <= last ? expf(s - new_max) : 0.f;
    p_s[tid] = p;
    const float chunk_sum = block_sum(p, scratch);  // (its barriers also publish p_s)
    const float alpha = expf(running_max - new_max);
    denom = denom * alpha + chunk_sum;
    running_max = new_max;
    const int count = min(256, last - j0 + 1);
#pragma unroll
    for (int u = 0; u < PLAIN_ATTENTION_MAX_D / 256; ++u) {
      const int c = tid + 256 * u;
      if (c >= d) break;
      float sum = 0.f;
      for (int jj = 0; jj < count; ++jj) {
        const int key = j0 + jj;
        sum = fmaf(p_s[jj], to_f32(v_cache[(((size_t)table[key >> page_shift] * nkv + kvh) * d + c) * page_size + (key & (page_size - 1))]), sum);
      }
      acc[u] = acc[u] * alpha + sum;
    }
    __syncthreads();  // (p_s is written again in the next round)
  }
  // a sink: exp(sinks[head]) joins the denominator (it has no key and no value and is not scaled)
  if (sinks) denom += expf(sinks[head] - running_max);
#pragma unroll
  for (int u = 0; u < PLAIN_ATTENTION_MAX_D / 256; ++u) {
    const int c = tid + 256 * u;
    if (c < d) out[(size_t)token * nh * d + (size_t)head * d + c] = from_f32<T>(acc[u] / denom);
  }
}

extern "C" int velox_plain_attention(const void* q, int q_width, const void* k_cache, const void* v_cache, const int* block_tables, int table_width,
                                     const int* cu_q, const int* kv_lens, void* out, int num_seqs, int tokens, int nh, int nkv, int d, int page_shift,
                                     float scale, int window, int dtype, const float* bias_table, int bias_len, const float* sinks, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (bias_table != nullptr && bias_len < 1) return -1;
  if (d < 1 || d > PLAIN_ATTENTION_MAX_D || nh < 1 || nkv < 1 || nh % nkv != 0 || nh > 65535 || num_seqs < 1 || nh * d > q_width) return -1;
  dim3 grid(tokens, nh);
  if (dtype == VELOX_BF16)
    plain_attention_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)q, q_width, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, table_width,
                                                             cu_q, kv_lens, (bf16_t*)out, num_seqs, nh, nkv, d, page_shift, scale, window, bias_table, bias_len, sinks);
  else
    plain_attention_kernel<float><<<grid, 256, 0, stream>>>((const float*)q, q_width, (const float*)k_cache, (const float*)v_cache, block_tables, table_width,
                                                            cu_q, kv_lens, (float*)out, num_seqs, nh, nkv, d, page_shift, scale, window, bias_table, bias_len, sinks);
  VELOX_RETURN_LAUNCH_STATUS();
}
