// Kernels of the mixers that carry a state of fixed size from token to token, and of the blocks around them, for gfx950:
//   stream_norm         the residual streams' update (mix matrix, weighted sub-layer output) and the norm of their weighted sum
//   gated_act_mul       act(gate) * up with the tanh form of GELU or SiLU
//   short_conv          causal convolution over a few taps per channel, the inputs before a portion's start from the state slot
//   rotate_pad_write    partial rotation of q and k, q at the attention kernels' head size, k and v into the paged cache
//   recurrence_prepare  unit q and k, decay and beta of a linear recurrence, all float32
//   linear_scan         the recurrence itself, token by token from the state slot (portions of prompts staged through LDS)
//   gated_head_norm     RMS norm of each head's read-out, a shared weight, a gate
// Everything between a load and a store is float32; stores round once.  No result depends on how a sequence's tokens
// were cut into steps or on what else is in the batch: sums run in an order that only the sizes fix.
#include "common.h"

__device__ __forceinline__ float load_as_f32(const void* p, int is_bf16, size_t i) {
  return is_bf16 ? to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}
__device__ __forceinline__ void store_from_f32(void* p, int is_bf16, size_t i, float v) {
  if (is_bf16) ((bf16_t*)p)[i] = (bf16_t)v; else ((float*)p)[i] = v;
}
__device__ __forceinline__ float sigmoid_f32(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---------------------------------------------------------------------------------------------
// stream_norm.  One workgroup per output row.  residual float32 [T, S * H], stream after stream within a row.
//   With terms: y = scale0 * term0 (+ scale1 * term1); x_t <- sum_s mix[s, t] x_s + out[t] * y for all t (mix nullptr: the
//   identity, out nullptr: ones), written back unless `rows` picks rows.  Then u = sum_s in[s] x_s (in nullptr: ones) and
//   out = (u - mean(u)) / sqrt(mean((u - mean)^2) + eps) * w   (center)   or   u / sqrt(mean(u^2) + eps) * w.
//   u is kept in LDS between the passes (H floats).
// ---------------------------------------------------------------------------------------------
#define STREAMS_MAX 8
struct StreamNormArgs {
  float* residual;
  const void* term0;
  const void* term1;
  int term0_bf16, term1_bf16, num_terms;
  float scale0, scale1;
  const float* mix;
  const float* out_w;
  const float* in_w;
  const float* weight;
  const int* rows;
  void* out;
  int out_bf16, hidden, streams, center;
  float eps;
};

__global__ void __launch_bounds__(256) stream_norm_kernel(const StreamNormArgs a) {
  extern __shared__ float u_row[];
  __shared__ float scratch[16];
  __shared__ float coef[STREAMS_MAX * STREAMS_MAX + 2 * STREAMS_MAX];
  const int S = a.streams, H = a.hidden;
  float* mix = coef;
  float* ow = coef + STREAMS_MAX * STREAMS_MAX;
  float* iw = ow + STREAMS_MAX;
  if (threadIdx.x < S * S) {
    const int s = threadIdx.x / S, t = threadIdx.x % S;
    mix[s * STREAMS_MAX + t] = a.mix ? a.mix[s * S + t] : (s == t ? 1.f : 0.f);
  }
  if (threadIdx.x < S) {
    ow[threadIdx.x] = a.out_w ? a.out_w[threadIdx.x] : 1.f;
    iw[threadIdx.x] = a.in_w ? a.in_w[threadIdx.x] : 1.f;
  }
  __syncthreads();
  const int row = blockIdx.x;
  const size_t src = a.rows ? (size_t)a.rows[row] : (size_t)row;
  float* res = a.residual + src * (size_t)S * H;
  const bool update = a.num_terms > 0;
  const bool write_back = update && a.rows == nullptr;
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float x[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s) x[s] = s < S ? res[(size_t)s * H + i] : 0.f;
    float u = 0.f;
    if (update) {
      float y = a.scale0 * load_as_f32(a.term0, a.term0_bf16, src * H + i);
      if (a.num_terms > 1) y += a.scale1 * load_as_f32(a.term1, a.term1_bf16, src * H + i);
#pragma unroll
      for (int t = 0; t < STREAMS_MAX; ++t) {
        if (t < S) {
          float n = 0.f;
#pragma unroll
          for (int s = 0; s < STREAMS_MAX; ++s)
            if (s < S) n += mix[s * STREAMS_MAX + t] * x[s];
          n += ow[t] * y;
          if (write_back) res[(size_t)t * H + i] = n;
          u += iw[t] * n;
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < STREAMS_MAX; ++s)
        if (s < S) u += iw[s] * x[s];
    }
    u_row[i] = u;
    sum += u;
  }
  float mean = 0.f;
  if (a.center) mean = block_sum(sum, scratch) / (float)H;
  float sq = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {  // (each thread reads back what it wrote itself)
    const float d = u_row[i] - mean;
    sq += d * d;
  }
  const float inv = 1.f / sqrtf(block_sum(sq, scratch) / (float)H + a.eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    store_from_f32(a.out, a.out_bf16, (size_t)row * H + i, (u_row[i] - mean) * inv * a.weight[i]);
}

// The same for rows of a multiple of four floats: a lane owns pieces of four neighbours (16-byte loads and stores of the
// streams, 8-byte ones of bfloat16 terms and results), a workgroup is as wide as a row has pieces (1024 lanes at most), and
// u stays in registers between the passes: PIECES pieces per lane, which the launch picks from the row's length.
__device__ __forceinline__ float4_t load4_as_f32(const void* p, int is_bf16, size_t i) {
  if (!is_bf16) return *reinterpret_cast<const float4_t*>((const float*)p + i);
  const short4_t raw = *reinterpret_cast<const short4_t*>((const bf16_t*)p + i);
  float4_t out;
#pragma unroll
  for (int c = 0; c < 4; ++c) out[c] = __uint_as_float(((unsigned)(unsigned short)raw[c]) << 16);
  return out;
}
__device__ __forceinline__ void store4_from_f32(void* p, int is_bf16, size_t i, float4_t v) {
  if (!is_bf16) { *reinterpret_cast<float4_t*>((float*)p + i) = v; return; }
  short4_t raw;
#pragma unroll
  for (int c = 0; c < 4; ++c) raw[c] = bf16_bits(v[c]);
  *reinterpret_cast<short4_t*>((bf16_t*)p + i) = raw;
}

template <int PIECES>
__global__ void __launch_bounds__(1024) stream_norm_vec_kernel(const StreamNormArgs a) {
  __shared__ float scratch[16];
  __shared__ float coef[STREAMS_MAX * STREAMS_MAX + 2 * STREAMS_MAX];
  const int S = a.streams, H = a.hidden, pieces = H / 4;
  float* mix = coef;
  float* ow = coef + STREAMS_MAX * STREAMS_MAX;
  float* iw = ow + STREAMS_MAX;
  if (threadIdx.x < S * S) {
    const int s = threadIdx.x / S, t = threadIdx.x % S;
    mix[s * STREAMS_MAX + t] = a.mix ? a.mix[s * S + t] : (s == t ? 1.f : 0.f);
  }
  if (threadIdx.x < S) {
    ow[threadIdx.x] = a.out_w ? a.out_w[threadIdx.x] : 1.f;
    iw[threadIdx.x] = a.in_w ? a.in_w[threadIdx.x] : 1.f;
  }
  __syncthreads();
  const int row = blockIdx.x;
  const size_t src = a.rows ? (size_t)a.rows[row] : (size_t)row;
  float* res = a.residual + src * (size_t)S * H;
  const bool update = a.num_terms > 0;
  const bool write_back = update && a.rows == nullptr;
  float4_t u[PIECES];
  float sum = 0.f;
#pragma unroll
  for (int p = 0; p < PIECES; ++p) {
    const int piece = threadIdx.x + p * blockDim.x;
    u[p] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (piece >= pieces) continue;
    const int i = piece * 4;
    float4_t x[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < S) x[s] = *reinterpret_cast<const float4_t*>(res + (size_t)s * H + i);
    if (update) {
      float4_t y = a.scale0 * load4_as_f32(a.term0, a.term0_bf16, src * H + i);
      if (a.num_terms > 1) y += a.scale1 * load4_as_f32(a.term1, a.term1_bf16, src * H + i);
#pragma unroll
      for (int t = 0; t < STREAMS_MAX; ++t) {
        if (t < S) {
          float4_t n = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < STREAMS_MAX; ++s)
            if (s < S) n += mix[s * STREAMS_MAX + t] * x[s];
          n += ow[t] * y;
          if (write_back) *reinterpret_cast<float4_t*>(res + (size_t)t * H + i) = n;
          u[p] += iw[t] * n;
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < STREAMS_MAX; ++s)
        if (s < S) u[p] += iw[s] * x[s];
    }
    sum += (u[p][0] + u[p][1]) + (u[p][2] + u[p][3]);
  }
  float mean = 0.f;
  if (a.center) mean = block_sum(sum, scratch) / (float)H;
  float sq = 0.f;
#pragma unroll
  for (int p = 0; p < PIECES; ++p) {
    if (threadIdx.x + p * blockDim.x < pieces) {
      const float4_t d = u[p] - mean;
      sq += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
    }
  }
  const float inv = 1.f / sqrtf(block_sum(sq, scratch) / (float)H + a.eps);
#pragma unroll
  for (int p = 0; p < PIECES; ++p) {
    const int piece = threadIdx.x + p * blockDim.x;
    if (piece < pieces) {
      const float4_t w = *reinterpret_cast<const float4_t*>(a.weight + piece * 4);
      store4_from_f32(a.out, a.out_bf16, (size_t)row * H + piece * 4, (u[p] - mean) * inv * w);
    }
  }
}

extern "C" int velox_stream_norm(float* residual, const void* term0, int term0_dtype, float scale0, const void* term1, int term1_dtype, float scale1,
                                 int num_terms, const float* mix, const float* out_w, const float* in_w, const float* weight, const int* rows,
                                 void* out, int out_dtype, int count, int hidden, int streams, int center, float eps, hipStream_t stream) {
  if (count <= 0) return 0;
  if (streams < 1 || streams > STREAMS_MAX || hidden < 1 || hidden > 16384 || num_terms < 0 || num_terms > 2) return (int)hipErrorInvalidValue;
  StreamNormArgs a{residual, term0, term1, term0_dtype == VELOX_BF16, term1_dtype == VELOX_BF16, num_terms, scale0, scale1, mix, out_w, in_w, weight,
                   rows, out, out_dtype == VELOX_BF16, hidden, streams, center, eps};
  const uintptr_t addresses = (uintptr_t)residual | (uintptr_t)weight | (uintptr_t)out | (uintptr_t)term0 | (uintptr_t)term1;
  if (hidden % 4 == 0 && addresses % 16 == 0) {  // (rows are a multiple of four elements, so their pieces are as aligned as the tensors)
    const int pieces = hidden / 4;
    int lanes = (pieces + 63) / 64 * 64;
    if (lanes > 1024) lanes = 1024;
    const int per_lane = (pieces + lanes - 1) / lanes;
    if (per_lane == 1) stream_norm_vec_kernel<1><<<count, lanes, 0, stream>>>(a);
    else if (per_lane == 2) stream_norm_vec_kernel<2><<<count, lanes, 0, stream>>>(a);
    else stream_norm_vec_kernel<4><<<count, lanes, 0, stream>>>(a);
    VELOX_RETURN_LAUNCH_STATUS();
  }
  stream_norm_kernel<<<count, 256, (size_t)hidden * sizeof(float), stream>>>(a);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// embedding written `copies` times side by side: out[t, c * H + i] = table[ids[t], i] * scale.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) embed_copies_kernel(const int* __restrict__ ids, const void* __restrict__ table, int table_bf16, float* __restrict__ out,
                                                           int hidden, int vocab, float scale, int copies) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* dst = out + (size_t)t * hidden * copies;
  const bool ok = id >= 0 && id < vocab;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = ok ? load_as_f32(table, table_bf16, (size_t)id * hidden + i) * scale : __builtin_nanf("");
    for (int c = 0; c < copies; ++c) dst[(size_t)c * hidden + i] = v;
  }
}

extern "C" int velox_embed_copies(const int* ids, const void* table, int table_dtype, float* out, int tokens, int hidden, int vocab, float scale, int copies,
                                  hipStream_t stream) {
  if (tokens <= 0) return 0;
  embed_copies_kernel<<<tokens, 256, 0, stream>>>(ids, table, table_dtype == VELOX_BF16, out, hidden, vocab, scale, copies);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// gated_act_mul: out[t, i] = act(gate_up[t, i]) * gate_up[t, I + i]; kind 0: SiLU, 1: the tanh form of GELU.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float gelu_tanh_f32(float z) { return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

template <typename T>
__global__ void __launch_bounds__(256) gated_act_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter, int kind) {
  const size_t t = blockIdx.y;
  const T* row = gate_up + t * 2 * (size_t)inter;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < inter; i += gridDim.x * blockDim.x) {
    const float g = to_f32(row[i]), u = to_f32(row[inter + i]);
    const float act = kind == 1 ? gelu_tanh_f32(g) : g * sigmoid_f32(g);
    out[t * inter + i] = from_f32<T>(act * u);
  }
}

extern "C" int velox_gated_act_mul(const void* gate_up, void* out, int tokens, int inter, int dtype, int kind, hipStream_t stream) {
  if (tokens <= 0 || inter <= 0) return 0;
  if (tokens > 65535) return (int)hipErrorInvalidValue;
  int bx = (inter + 255) / 256;
  if (bx > 64) bx = 64;
  const dim3 grid(bx, tokens);
  if (dtype == VELOX_BF16) gated_act_mul_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, inter, kind);
  else gated_act_mul_kernel<float><<<grid, 256, 0, stream>>>((const float*)gate_up, (float*)out, inter, kind);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// short_conv.  x [T, ld]: the first C columns pass y_t = sum_j w[c, j] u_(t - taps + 1 + j), per sequence; the inputs before a
// portion's start are tail[slot] ([taps - 1, C], oldest first; nullptr: zeros).  Grid (channel blocks, token chunks, sequences);
// a thread owns one channel and walks CONV_CHUNK tokens with the last taps - 1 inputs in registers.
// The tail is brought up to date by the same thread when a sequence's portion is one chunk at most (decoding), else by
// short_conv_tail_kernel, which runs afterwards: no workgroup writes what another still reads.
// ---------------------------------------------------------------------------------------------
#define CONV_TAPS_MAX 8
#define CONV_CHUNK 16

template <typename T>
__global__ void __launch_bounds__(256) short_conv_kernel(const T* __restrict__ x, int ld, int C, const float* __restrict__ w, int taps, T* tail,
                                                         const int* __restrict__ slots, const int* __restrict__ cu_q, T* __restrict__ out, int silu,
                                                         int update_here) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int b = blockIdx.z;
  const int lo = cu_q[b], hi = cu_q[b + 1];
  const int first = lo + blockIdx.y * CONV_CHUNK;
  if (c >= C || first >= hi) return;
  const int last = first + CONV_CHUNK < hi ? first + CONV_CHUNK : hi;
  float wj[CONV_TAPS_MAX], u[CONV_TAPS_MAX];
#pragma unroll
  for (int j = 0; j < CONV_TAPS_MAX; ++j) wj[j] = j < taps ? w[(size_t)c * taps + j] : 0.f;
  T* my_tail = tail ? tail + (size_t)slots[b] * (taps - 1) * C + c : nullptr;
  // u[j] is the input `taps - 1 - j` tokens before the current one; u[taps - 1] the current
#pragma unroll
  for (int j = 0; j < CONV_TAPS_MAX; ++j) {
    u[j] = 0.f;
    if (j < taps - 1) {
      const int t = first - (taps - 1) + j;
      if (t >= lo) u[j] = to_f32(x[(size_t)t * ld + c]);
      else if (my_tail) u[j] = to_f32(my_tail[(size_t)(t - lo + taps - 1) * C]);
    }
  }
  for (int t = first; t < last; ++t) {
    const float now = to_f32(x[(size_t)t * ld + c]);
    float y = 0.f;
#pragma unroll
    for (int j = 0; j < CONV_TAPS_MAX; ++j)  // (oldest input first; the last column of the weights meets the current token)
      if (j < taps) y += wj[j] * (j == taps - 1 ? now : u[j]);
    if (silu) y = y * sigmoid_f32(y);
    out[(size_t)t * C + c] = from_f32<T>(y);
#pragma unroll
    for (int j = 0; j < CONV_TAPS_MAX; ++j) u[j] = j == taps - 2 ? now : (j + 1 < CONV_TAPS_MAX ? u[j + 1] : 0.f);
  }
  if (update_here && my_tail && taps > 1) {  // (then this thread has seen the whole portion: u[0 .. taps - 2] are the last inputs)
#pragma unroll
    for (int j = 0; j < CONV_TAPS_MAX; ++j)
      if (j < taps - 1) my_tail[(size_t)j * C] = from_f32<T>(u[j]);
  }
}

template <typename T>
__global__ void __launch_bounds__(256) short_conv_tail_kernel(const T* __restrict__ x, int ld, int C, int taps, T* tail, const int* __restrict__ slots,
                                                              const int* __restrict__ cu_q) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int b = blockIdx.y;
  const int lo = cu_q[b], hi = cu_q[b + 1];
  if (c >= C || hi <= lo) return;
  T* my_tail = tail + (size_t)slots[b] * (taps - 1) * C + c;
  float u[CONV_TAPS_MAX];
#pragma unroll
  for (int j = 0; j < CONV_TAPS_MAX; ++j) {
    u[j] = 0.f;
    if (j < taps - 1) {
      const int t = hi - (taps - 1) + j;
      u[j] = t >= lo ? to_f32(x[(size_t)t * ld + c]) : to_f32(my_tail[(size_t)(t - lo + taps - 1) * C]);
    }
  }
#pragma unroll
  for (int j = 0; j < CONV_TAPS_MAX; ++j)
    if (j < taps - 1) my_tail[(size_t)j * C] = from_f32<T>(u[j]);
}

extern "C" int velox_short_conv(const void* x, int ld, int channels, const float* w, int taps, void* tail, const int* slots, const int* cu_q, void* out,
                                int num_seqs, int max_q_len, int dtype, int silu, int update_state, hipStream_t stream) {
  if (num_seqs <= 0 || max_q_len <= 0) return 0;
  if (taps < 1 || taps > CONV_TAPS_MAX || num_seqs > 65535) return (int)hipErrorInvalidValue;
  const int chunks = (max_q_len + CONV_CHUNK - 1) / CONV_CHUNK;
  if (chunks > 65535) return (int)hipErrorInvalidValue;
  const dim3 grid((channels + 255) / 256, chunks, num_seqs);
  const int here = (update_state && chunks == 1) ? 1 : 0;
  if (dtype == VELOX_BF16)
    short_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ld, channels, w, taps, (bf16_t*)tail, slots, cu_q, (bf16_t*)out, silu, here);
  else
    short_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, ld, channels, w, taps, (float*)tail, slots, cu_q, (float*)out, silu, here);
  if (update_state && !here && tail && taps > 1) {
    const dim3 tail_grid((channels + 255) / 256, num_seqs);
    if (dtype == VELOX_BF16) short_conv_tail_kernel<bf16_t><<<tail_grid, 256, 0, stream>>>((const bf16_t*)x, ld, channels, taps, (bf16_t*)tail, slots, cu_q);
    else short_conv_tail_kernel<float><<<tail_grid, 256, 0, stream>>>((const float*)x, ld, channels, taps, (float*)tail, slots, cu_q);
  }
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// rotate_pad_write: workgroups take a token's heads in turn (queries, keys, then values; one head each in steps of few tokens).  A row
// of qkv holds `heads` queries and `kv_heads` keys of `dim` channels and `kv_heads` values of `vdim`.  The first 2 * half
// channels of every query and key head are rotated (channel i with i + half, or 2i with 2i + 1 when `interleaved`; cos/sin
// float32 [positions, half]; (u, v) -> (u cos - v sin, v cos + u sin)); queries go to
// q_out [T, heads * D], keys to k_cache [pages, kv_heads, page, D], values to v_cache [pages, kv_heads, D, page]; channels from
// dim (vdim) to D are zeros.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) rotate_pad_write_kernel(const T* __restrict__ qkv, int ld, T* __restrict__ q_out, const int* __restrict__ positions,
                                                               const float* __restrict__ cos_t, const float* __restrict__ sin_t, int half,
                                                               const int* __restrict__ slot_mapping, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                               int heads, int kv_heads, int dim, int vdim, int D, int page_shift, int write_kv,
                                                               int interleaved) {
  const int t = blockIdx.x;
  const T* row = qkv + (size_t)t * ld;
  const int q_size = heads * dim, k_size = kv_heads * dim;
  const int page_size = 1 << page_shift;
  int page = 0, offset = 0;
  if (write_kv) {
    const int slot = slot_mapping[t];
    page = slot >> page_shift;
    offset = slot & (page_size - 1);
  }
  const float* cs = half > 0 ? cos_t + (size_t)positions[t] * half : nullptr;
  const float* sn = half > 0 ? sin_t + (size_t)positions[t] * half : nullptr;
  const int all_heads = heads + (write_kv ? 2 * kv_heads : 0);
  for (int h = blockIdx.y; h < all_heads; h += gridDim.y) {  // (a step of few tokens has a workgroup per head, a long one a few per token)
    if (h >= heads + kv_heads) {  // a value head
      const int g = h - heads - kv_heads;
      const T* values = row + q_size + k_size + g * vdim;
      for (int c = threadIdx.x; c < D; c += blockDim.x)
        v_cache[(((size_t)page * kv_heads + g) * D + c) * page_size + offset] = c < vdim ? values[c] : from_f32<T>(0.f);
      continue;
    }
    const bool is_q = h < heads;
    const int g = is_q ? h : h - heads;
    const T* src = row + (is_q ? h * dim : q_size + g * dim);
    T* dst = is_q ? q_out + ((size_t)t * heads + h) * D : k_cache + (((size_t)page * kv_heads + g) * page_size + offset) * D;
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
      float v = 0.f;
      if (c < dim) {
        v = to_f32(src[c]);
        if (interleaved) {
          if (c < 2 * half) {
            const int i = c >> 1;
            v = (c & 1) ? v * cs[i] + to_f32(src[c - 1]) * sn[i] : v * cs[i] - to_f32(src[c + 1]) * sn[i];
          }
        } else if (c < half) v = v * cs[c] - to_f32(src[c + half]) * sn[c];
        else if (c < 2 * half) v = v * cs[c - half] + to_f32(src[c - half]) * sn[c - half];
      }
      dst[c] = from_f32<T>(v);
    }
  }
}

extern "C" int velox_rotate_pad_write(const void* qkv, int ld, void* q_out, const int* positions, const float* cos_t, const float* sin_t, int half,
                                      const int* slot_mapping, void* k_cache, void* v_cache, int tokens, int heads, int kv_heads, int dim, int vdim, int D,
                                      int page_size, int write_kv, int dtype, int interleaved, hipStream_t stream) {
  if (tokens <= 0) return 0;
  int shift = 0;
  while ((1 << shift) < page_size) ++shift;
  if ((1 << shift) != page_size || 2 * half > dim || dim > D || vdim > D) return (int)hipErrorInvalidValue;
  const int all_heads = heads + (write_kv ? 2 * kv_heads : 0);
  const dim3 grid(tokens, tokens <= 256 ? all_heads : (all_heads < 4 ? all_heads : 4));
  int lanes = (D + 63) / 64 * 64;
  if (lanes > 256) lanes = 256;
  if (dtype == VELOX_BF16)
    rotate_pad_write_kernel<bf16_t><<<grid, lanes, 0, stream>>>((const bf16_t*)qkv, ld, (bf16_t*)q_out, positions, cos_t, sin_t, half, slot_mapping,
                                                              (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, dim, vdim, D, shift, write_kv, interleaved);
  else
    rotate_pad_write_kernel<float><<<grid, lanes, 0, stream>>>((const float*)qkv, ld, (float*)q_out, positions, cos_t, sin_t, half, slot_mapping,
                                                             (float*)k_cache, (float*)v_cache, heads, kv_heads, dim, vdim, D, shift, write_kv, interleaved);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// recurrence_prepare: one workgroup per token (eight in steps of few tokens), waves take heads in turn.
//   qk float32 [T, kv_heads, 2, dim]: q (unit vector if `unit`, times q_scale), then k (unit vector if `unit`);
//   decay float32 [T, columns] = exp(-rate[h] * softplus(sign * (z + bias))), h = column / (columns / heads);
//   beta float32 [T, heads] = sigmoid(b).
// ---------------------------------------------------------------------------------------------
struct PrepareArgs {
  const void* qkv;
  int qkv_bf16, ld, q_at, k_at, kv_heads, dim, unit;
  float q_scale;
  const void* decay_src;
  int decay_bf16, decay_ld, decay_at, heads, columns;
  const float* rate;
  const float* bias;
  float sign;
  const void* beta_src;
  int beta_bf16, beta_ld, beta_at;
  float* qk;
  float* decay;
  float* beta;
};

__global__ void __launch_bounds__(256) recurrence_prepare_kernel(const PrepareArgs a) {
  const size_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int part = blockIdx.y, parts = gridDim.y;  // (a step of few tokens spreads each token over several workgroups)
  for (int h = wave + 4 * part; h < 2 * a.kv_heads; h += 4 * parts) {
    const int g = h >> 1, is_k = h & 1;
    const size_t at = t * a.ld + (is_k ? a.k_at : a.q_at) + (size_t)g * a.dim;
    float inv = 1.f;
    if (a.unit) {
      float s = 0.f;
      for (int c = lane; c < a.dim; c += 64) { const float v = load_as_f32(a.qkv, a.qkv_bf16, at + c); s += v * v; }
      s = wave_sum(s);
      inv = 1.f / sqrtf(s + 1e-6f);
    }
    const float factor = is_k ? 1.f : a.q_scale;
    float* dst = a.qk + ((t * a.kv_heads + g) * 2 + is_k) * a.dim;
    for (int c = lane; c < a.dim; c += 64) dst[c] = load_as_f32(a.qkv, a.qkv_bf16, at + c) * inv * factor;
  }
  const int per_head = a.columns / a.heads;
  for (int c = threadIdx.x + part * blockDim.x; c < a.columns; c += blockDim.x * parts) {
    float z = load_as_f32(a.decay_src, a.decay_bf16, t * a.decay_ld + a.decay_at + c);
    if (a.bias) z += a.bias[c];
    a.decay[t * a.columns + c] = expf(-a.rate[c / per_head] * softplus_f32(a.sign * z));
  }
  if (a.beta && part == 0)
    for (int h = threadIdx.x; h < a.heads; h += blockDim.x)
      a.beta[t * a.heads + h] = sigmoid_f32(load_as_f32(a.beta_src, a.beta_bf16, t * a.beta_ld + a.beta_at + h));
}

extern "C" int velox_recurrence_prepare(const void* qkv, int qkv_dtype, int ld, int q_at, int k_at, int kv_heads, int dim, int unit, float q_scale,
                                        const void* decay_src, int decay_dtype, int decay_ld, int decay_at, int heads, int columns, const float* rate,
                                        const float* bias, float sign, const void* beta_src, int beta_dtype, int beta_ld, int beta_at, float* qk,
                                        float* decay, float* beta, int tokens, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads < 1 || columns % heads != 0) return (int)hipErrorInvalidValue;
  PrepareArgs a{qkv, qkv_dtype == VELOX_BF16, ld, q_at, k_at, kv_heads, dim, unit, q_scale, decay_src, decay_dtype == VELOX_BF16, decay_ld, decay_at, heads,
                columns, rate, bias, sign, beta_src, beta_dtype == VELOX_BF16, beta_ld, beta_at, qk, decay, beta};
  const int parts = tokens <= 64 ? 8 : 1;
  recurrence_prepare_kernel<<<dim3(tokens, parts), 256, 0, stream>>>(a);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// linear_scan.  Per sequence and head a state S of dim x vdim float32 numbers (rows: key channels) in state[slot, head].
// Every column of S is a recurrence of its own:   s <- g * s;  u = beta (v_e - k . s)  (delta rule)  or  u = v_e;
// s <- s + k u;  o_e = q . s.   A column is held by R lanes of a wave, SCAN_ROWS consecutive rows each (R the smallest power of
// two with R * SCAN_ROWS >= dim: a function of dim alone, so the order of every sum is too); the two dot products are
// summed in four interleaved parts per lane and then over those lanes (scan_token, the one place where a token is worked).
// With eight rows to a lane a head of 128 key channels spreads over sixteen lanes, and a workgroup holds sixteen columns.
// Grid (column blocks, heads, sequences); a workgroup of 256 lanes holds 256 / R columns.
//   linear_scan_kernel         steps of single tokens: a token's q, k, decay, value and beta come straight from memory, the
//                              next token's while the current one is worked on.
//   linear_scan_staged_kernel  portions of prompts: the tokens are a dependent chain, so a token must cost no memory round
//                              trip.  The workgroup carries the next block of tokens (q, k, decay of the head, the values of its
//                              columns, beta) from memory into registers before it works through the current block out of
//                              LDS, and writes the registers to the other LDS buffer behind it: one barrier per block, the
//                              loads' latency lies behind a block's arithmetic.
//   linear_scan_wave_kernel    the same for dim = 64, 128, 256, 512, a column per wave (described at the kernel).
// The first two give the same bits: they differ in where the operands wait, not in what is done with them; the third sums in
// another order (which, like theirs, only the sizes fix).
// ---------------------------------------------------------------------------------------------
#define SCAN_ROWS 8

// Sum over the R lanes that hold a column (R a power of two, the lanes consecutive and aligned): pairs, quads, halves of a
// row of 16 and the row by data-parallel moves inside the vector unit, beyond a row through the cross-lane network.  Both
// partners of a step add the same two numbers, so every lane ends with the same bits.
template <int CTRL>
__device__ __forceinline__ float lanes_moved(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int R>
__device__ __forceinline__ float sum_over_lanes(float v) {
  if (R >= 2) v += lanes_moved<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  if (R >= 4) v += lanes_moved<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  if (R >= 8) v += lanes_moved<0x141>(v);   // row_half_mirror: lane i of eight with lane 7 - i, which holds the other quad's sum
  if (R >= 16) v += lanes_moved<0x140>(v);  // row_mirror: lane i of sixteen with lane 15 - i
#pragma unroll
  for (int off = 16; off < R; off <<= 1) v += __shfl_xor(v, off, VELOX_WAVE);
  return v;
}

struct ScanArgs {
  const float* qk;       // [T, kv_heads, 2, dim]
  const void* v;         // [T, v_ld], a token's values at v_at
  int v_bf16, v_ld, v_at;
  const float* decay;    // [T, heads * dim] or [T, heads]
  int decay_per_channel;
  const float* beta;     // [T, heads] or nullptr
  float* state;          // [slots, heads, dim, vdim]
  const int* slots;
  const int* cu_q;
  float* out;            // [T, heads * vdim]
  int heads, kv_heads, dim, vdim, delta;
};

__device__ __forceinline__ void scan_load_rows(const float* __restrict__ p, int d0, int dim, bool vec, float fill, float (&r)[SCAN_ROWS]) {
  if (vec && d0 + SCAN_ROWS <= dim) {
#pragma unroll
    for (int i = 0; i < SCAN_ROWS; i += 4) {
      const float4_t x = *reinterpret_cast<const float4_t*>(p + d0 + i);
      r[i] = x[0]; r[i + 1] = x[1]; r[i + 2] = x[2]; r[i + 3] = x[3];
    }
  } else {
#pragma unroll
    for (int i = 0; i < SCAN_ROWS; ++i) r[i] = d0 + i < dim ? p[d0 + i] : fill;
  }
}

// One token of one column: returns the read-out (complete in every lane of the column).
template <int R>
__device__ __forceinline__ float scan_token(float (&s)[SCAN_ROWS], const float (&q)[SCAN_ROWS], const float (&k)[SCAN_ROWS], const float (&dec)[SCAN_ROWS],
                                            float val, float bet, int delta) {
  float d[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < SCAN_ROWS; ++i) {
    s[i] *= dec[i];
    d[i & 3] += s[i] * k[i];
  }
  float u = val;
  if (delta) {
    const float dot = sum_over_lanes<R>((d[0] + d[1]) + (d[2] + d[3]));
    u = bet * (val - dot);
  }
  float p[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < SCAN_ROWS; ++i) {
    s[i] += k[i] * u;
    p[i & 3] += s[i] * q[i];
  }
  return sum_over_lanes<R>((p[0] + p[1]) + (p[2] + p[3]));
}

template <int R>
__global__ void __launch_bounds__(256) linear_scan_kernel(const ScanArgs a) {
  const int r = threadIdx.x % R;
  const int e = blockIdx.x * (256 / R) + threadIdx.x / R;
  const int h = blockIdx.y, b = blockIdx.z;
  const int lo = a.cu_q[b], hi = a.cu_q[b + 1];
  if (hi <= lo) return;
  const bool live = e < a.vdim;
  const int col = live ? e : a.vdim - 1;  // (lanes beyond the last column follow it and write nothing: the shuffles need every lane)
  const int dim = a.dim, vdim = a.vdim;
  const int d0 = r * SCAN_ROWS;
  const int g = h / (a.heads / a.kv_heads);
  const bool vec = (dim % 4) == 0;
  float* S = a.state + (((size_t)a.slots[b] * a.heads + h) * dim) * vdim + col;
  float s[SCAN_ROWS];
#pragma unroll
  for (int i = 0; i < SCAN_ROWS; ++i) s[i] = d0 + i < dim ? S[(size_t)(d0 + i) * vdim] : 0.f;

  float q[SCAN_ROWS], k[SCAN_ROWS], dec[SCAN_ROWS], qn[SCAN_ROWS], kn[SCAN_ROWS], decn[SCAN_ROWS];
  float val, bet, valn = 0.f, betn = 1.f;
  auto fetch = [&](int t, float (&fq)[SCAN_ROWS], float (&fk)[SCAN_ROWS], float (&fd)[SCAN_ROWS], float& fv, float& fb) {
    const float* base = a.qk + ((size_t)t * a.kv_heads + g) * 2 * dim;
    scan_load_rows(base, d0, dim, vec, 0.f, fq);
    scan_load_rows(base + dim, d0, dim, vec, 0.f, fk);
    if (a.decay_per_channel) {
      scan_load_rows(a.decay + ((size_t)t * a.heads + h) * dim, d0, dim, vec, 1.f, fd);
    } else {
      const float one = a.decay[(size_t)t * a.heads + h];
#pragma unroll
      for (int i = 0; i < SCAN_ROWS; ++i) fd[i] = one;
    }
    fv = load_as_f32(a.v, a.v_bf16, (size_t)t * a.v_ld + a.v_at + (size_t)h * vdim + col);
    fb = a.beta ? a.beta[(size_t)t * a.heads + h] : 1.f;
  };
  fetch(lo, q, k, dec, val, bet);
  for (int t = lo; t < hi; ++t) {
    if (t + 1 < hi) fetch(t + 1, qn, kn, decn, valn, betn);
    const float o = scan_token<R>(s, q, k, dec, val, bet, a.delta);
    if (live && r == 0) a.out[((size_t)t * a.heads + h) * vdim + e] = o;
#pragma unroll
    for (int i = 0; i < SCAN_ROWS; ++i) { q[i] = qn[i]; k[i] = kn[i]; dec[i] = decn[i]; }
    val = valn; bet = betn;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < SCAN_ROWS; ++i)
      if (d0 + i < dim) S[(size_t)(d0 + i) * vdim] = s[i];
  }
}

// A token's place in a staging buffer, in floats: q [dim], k [dim], the decay per channel [dim] if there is one, the values of
// the workgroup's columns [256 / R], then beta and the head's decay (and two floats that keep the next token 16-byte aligned).
#define STAGE_PIECES 8  // 16-byte pieces of q, k and decay that one lane carries per block of tokens, at most
#define STAGE_VALUES 4  // values that one lane carries per block, at most

template <int R>
__global__ void __launch_bounds__(256) linear_scan_staged_kernel(const ScanArgs a, const int block_tokens) {
  extern __shared__ float4_t stage_pieces[];
  float* stage = reinterpret_cast<float*>(stage_pieces);
  constexpr int COLS = 256 / R;
  const int tid = threadIdx.x;
  const int r = tid % R, c_local = tid / R;
  const int e = blockIdx.x * COLS + c_local;
  const int h = blockIdx.y, b = blockIdx.z;
  const int lo = a.cu_q[b], hi = a.cu_q[b + 1];
  if (hi <= lo) return;  // (the whole workgroup: no barrier is left waiting)
  const bool live = e < a.vdim;
  const int col = live ? e : a.vdim - 1;
  const int dim = a.dim, vdim = a.vdim, heads = a.heads;
  const int d0 = r * SCAN_ROWS;
  const int g = h / (heads / a.kv_heads);
  const int per_channel = a.decay_per_channel;
  const int qk_pieces = dim / 2;                                     // (2 * dim floats in pieces of 4)
  const int pieces_per_token = qk_pieces + (per_channel ? dim / 4 : 0);
  const int values_at = 2 * dim + (per_channel ? dim : 0);
  const int scalars_at = values_at + COLS;
  const int stride = scalars_at + 4;

  // what this lane carries from memory to LDS in every block: token within the block, offset within the token's row, place in LDS
  int piece_token[STAGE_PIECES], piece_from[STAGE_PIECES], piece_to[STAGE_PIECES];
#pragma unroll
  for (int p = 0; p < STAGE_PIECES; ++p) {
    const int index = tid + p * 256;
    const int token = index / pieces_per_token, piece = index - token * pieces_per_token;
    piece_token[p] = token < block_tokens ? token : -1;
    piece_from[p] = piece < qk_pieces ? piece * 4 : -1 - (piece - qk_pieces) * 4;  // (negative: a piece of the decay)
    piece_to[p] = token * stride + piece * 4;
  }
  float4_t carried[STAGE_PIECES];
  float carried_values[STAGE_VALUES];
  float carried_beta = 1.f, carried_decay = 1.f;
  auto load_block = [&](int t0) {
#pragma unroll
    for (int p = 0; p < STAGE_PIECES; ++p) {
      const int t = t0 + piece_token[p];
      if (piece_token[p] >= 0 && t < hi) {
        const float* from = piece_from[p] >= 0 ? a.qk + ((size_t)t * a.kv_heads + g) * 2 * dim + piece_from[p]
                                               : a.decay + ((size_t)t * heads + h) * dim + (-1 - piece_from[p]);
        carried[p] = *reinterpret_cast<const float4_t*>(from);
      }
    }
#pragma unroll
    for (int j = 0; j < STAGE_VALUES; ++j) {
      const int index = tid + j * 256;
      const int token = index / COLS, c = index % COLS;
      const int t = t0 + token, column = blockIdx.x * COLS + c;
      if (token < block_tokens && t < hi)
        carried_values[j] = column < vdim ? load_as_f32(a.v, a.v_bf16, (size_t)t * a.v_ld + a.v_at + (size_t)h * vdim + column) : 0.f;
    }
    if (tid < block_tokens && t0 + tid < hi) {
      carried_beta = a.beta ? a.beta[(size_t)(t0 + tid) * heads + h] : 1.f;
      carried_decay = per_channel ? 1.f : a.decay[(size_t)(t0 + tid) * heads + h];
    }
  };
  auto store_block = [&](int buffer) {  // (rows of tokens beyond the sequence's end keep what they held: nobody reads them)
    const int at = buffer * block_tokens * stride;
#pragma unroll
    for (int p = 0; p < STAGE_PIECES; ++p)
      if (piece_token[p] >= 0) *reinterpret_cast<float4_t*>(&stage[at + piece_to[p]]) = carried[p];
#pragma unroll
    for (int j = 0; j < STAGE_VALUES; ++j) {
      const int index = tid + j * 256;
      const int token = index / COLS, c = index % COLS;
      if (token < block_tokens) stage[at + token * stride + values_at + c] = carried_values[j];
    }
    if (tid < block_tokens) {
      stage[at + tid * stride + scalars_at] = carried_beta;
      stage[at + tid * stride + scalars_at + 1] = carried_decay;
    }
  };
#pragma unroll
  for (int p = 0; p < STAGE_PIECES; ++p) carried[p] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < STAGE_VALUES; ++j) carried_values[j] = 0.f;

  float* S = a.state + (((size_t)a.slots[b] * heads + h) * dim) * vdim + col;
  float s[SCAN_ROWS];
#pragma unroll
  for (int i = 0; i < SCAN_ROWS; ++i) s[i] = d0 + i < dim ? S[(size_t)(d0 + i) * vdim] : 0.f;

  float q[SCAN_ROWS], k[SCAN_ROWS], dec[SCAN_ROWS], qn[SCAN_ROWS], kn[SCAN_ROWS], decn[SCAN_ROWS];  // two sets of operands, used in turn
  float val, bet, valn = 0.f, betn = 1.f;
  auto fetch = [&](int at, float (&fq)[SCAN_ROWS], float (&fk)[SCAN_ROWS], float (&fd)[SCAN_ROWS], float& fv, float& fb) {
    const float one = stage[at + scalars_at + 1];
#pragma unroll
    for (int i = 0; i < SCAN_ROWS; i += 4) {
      if (d0 + i < dim) {  // (dim is a multiple of 4 here: a piece lies inside the head or outside)
        const float4_t x = *reinterpret_cast<const float4_t*>(&stage[at + d0 + i]);
        const float4_t y = *reinterpret_cast<const float4_t*>(&stage[at + dim + d0 + i]);
        fq[i] = x[0]; fq[i + 1] = x[1]; fq[i + 2] = x[2]; fq[i + 3] = x[3];
        fk[i] = y[0]; fk[i + 1] = y[1]; fk[i + 2] = y[2]; fk[i + 3] = y[3];
        if (per_channel) {
          const float4_t z = *reinterpret_cast<const float4_t*>(&stage[at + 2 * dim + d0 + i]);
          fd[i] = z[0]; fd[i + 1] = z[1]; fd[i + 2] = z[2]; fd[i + 3] = z[3];
        } else {
          fd[i] = fd[i + 1] = fd[i + 2] = fd[i + 3] = one;
        }
      } else {
        fq[i] = fq[i + 1] = fq[i + 2] = fq[i + 3] = 0.f;
        fk[i] = fk[i + 1] = fk[i + 2] = fk[i + 3] = 0.f;
        fd[i] = fd[i + 1] = fd[i + 2] = fd[i + 3] = 1.f;
      }
    }
    fv = stage[at + values_at + c_local];
    fb = stage[at + scalars_at];
  };

  load_block(lo);
  store_block(0);
  __syncthreads();
  int buffer = 0;
  for (int t0 = lo; t0 < hi; t0 += block_tokens, buffer ^= 1) {
    const bool more = t0 + block_tokens < hi;
    if (more) load_block(t0 + block_tokens);
    const int count = hi - t0 < block_tokens ? hi - t0 : block_tokens;
    const int at = buffer * block_tokens * stride;
    fetch(at, q, k, dec, val, bet);
    int j = 0;
    for (; j + 1 < count; j += 2) {  // (a token's operands are read from LDS while the token before it is worked)
      fetch(at + (j + 1) * stride, qn, kn, decn, valn, betn);
      const float o0 = scan_token<R>(s, q, k, dec, val, bet, a.delta);
      if (live && r == 0) a.out[((size_t)(t0 + j) * heads + h) * vdim + e] = o0;
      if (j + 2 < count) fetch(at + (j + 2) * stride, q, k, dec, val, bet);
      const float o1 = scan_token<R>(s, qn, kn, decn, valn, betn, a.delta);
      if (live && r == 0) a.out[((size_t)(t0 + j + 1) * heads + h) * vdim + e] = o1;
    }
    if (j < count) {
      const float o = scan_token<R>(s, q, k, dec, val, bet, a.delta);
      if (live && r == 0) a.out[((size_t)(t0 + j) * heads + h) * vdim + e] = o;
    }
    if (more) store_block(buffer ^ 1);  // (the buffer that the block before this one was worked from: everyone is past the barrier behind it)
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < SCAN_ROWS; ++i)
      if (d0 + i < dim) S[(size_t)(d0 + i) * vdim] = s[i];
  }
}

extern "C" int velox_linear_scan_lanes(int dim) {
  int lanes = 1;
  while (lanes * SCAN_ROWS < dim) lanes <<= 1;
  return lanes;
}

// The sum over a wave, the same bits in every lane: rows of 16 as in sum_over_lanes, then row 0's sum into row 1 and row 2's
// into row 3, the first half's into the second, and the last lane's total to everyone.
__device__ __forceinline__ float wave_total(float v) {
  v += lanes_moved<0xB1>(v);
  v += lanes_moved<0x4E>(v);
  v += lanes_moved<0x141>(v);
  v += lanes_moved<0x140>(v);
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xA, 0xF, false));  // row_bcast:15, rows 1 and 3 take it
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xC, 0xF, false));  // row_bcast:31, rows 2 and 3 take it
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// linear_scan_wave_kernel: portions of prompts where dim = 64 * RW.  A column of the state is one wave, lane l holds rows
// l * RW .. l * RW + RW - 1: a token costs a lane 3 RW multiply-adds and two sums over the wave, and a head of 128 x 128 is
// 128 waves, so that a long prompt of one request still reaches every compute unit.  A workgroup of 512 lanes holds eight
// columns and stages its head's tokens through LDS as linear_scan_staged_kernel does.  (It reads and writes a column of
// the state with a stride of vdim floats, once per portion; single tokens keep the kernel whose lanes lie along the rows.)
#define WAVE_COLS 8
// 16, 4 or 2 bytes per lane from global memory straight into LDS: lane l's piece lands at `to` + 16 l (4 l for the small
// ones; two bytes arrive as a zero-extended word).  `to` is the same for the whole wave and is taken from its first
// active lane.  Assembly, as load_to_lds_16 of common.h and for its reason: the compiler neither moves such a load nor
// waits for it; the caller waits (wait_for_loads) and places a barrier before anyone reads.
__device__ __forceinline__ uint32_t lds_address_of_wave(const void* to) {
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)to);
}
__device__ __forceinline__ void send_to_lds_16(const void* src, const void* to) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_address_of_wave(to)), "v"(src) : "memory", "m0");
}
__device__ __forceinline__ void send_to_lds_4(const void* src, const void* to) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(lds_address_of_wave(to)), "v"(src) : "memory", "m0");
}
__device__ __forceinline__ void send_to_lds_2(const void* src, const void* to) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ushort %1, off" : : "s"(lds_address_of_wave(to)), "v"(src) : "memory", "m0");
}

// A staging buffer of linear_scan_wave_kernel, in floats: q and k of the block's tokens [tokens, 2 dim], the decays per channel
// [tokens, dim] if there are such, the values of the workgroup's columns [tokens, 8] as they lie in memory (float32, or
// bfloat16 in the low half of a word), beta [tokens] and the head's decay [tokens].
__host__ __device__ __forceinline__ int wave_buffer_floats(int tokens, int dim, int per_channel) {
  return tokens * (2 * dim + (per_channel ? dim : 0) + WAVE_COLS + 2);
}

template <int RW>
__global__ void __launch_bounds__(512) linear_scan_wave_kernel(const ScanArgs a, const int block_tokens) {
  extern __shared__ float4_t stage_pieces[];
  float* stage = reinterpret_cast<float*>(stage_pieces);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int e = blockIdx.x * WAVE_COLS + wave;
  const int h = blockIdx.y, b = blockIdx.z;
  const int lo = a.cu_q[b], hi = a.cu_q[b + 1];
  if (hi <= lo) return;  // (the whole workgroup)
  const bool live = e < a.vdim;
  const int col = live ? e : a.vdim - 1;
  const int dim = 64 * RW, vdim = a.vdim, heads = a.heads;
  const int d0 = lane * RW;
  const int g = h / (heads / a.kv_heads);
  const int per_channel = a.decay_per_channel;
  const int qk_pieces = dim / 2, decay_pieces = dim / 4;  // 16-byte pieces of a token's q and k, of its decays
  const int decays_at = block_tokens * 2 * dim;
  const int values_at = decays_at + (per_channel ? block_tokens * dim : 0);
  const int betas_at = values_at + block_tokens * WAVE_COLS;
  const int head_decays_at = betas_at + block_tokens;
  const int buffer_floats = wave_buffer_floats(block_tokens, dim, per_channel);

  // Sends for the block of tokens from t0: every wave instruction fills 64 consecutive pieces of LDS, each lane from its own
  // place in memory.  Lanes whose token lies beyond the sequence's end send nothing (nobody reads those rows).
  auto send_block = [&](int which, int t0) {
    float* to = stage + which * buffer_floats;
    for (int first = wave * 64; first < block_tokens * qk_pieces; first += 512) {
      const int index = first + lane, token = index / qk_pieces, piece = index - token * qk_pieces;
      if (token < block_tokens && t0 + token < hi)
        send_to_lds_16(a.qk + ((size_t)(t0 + token) * a.kv_heads + g) * 2 * dim + piece * 4, to + first * 4);
    }
    if (per_channel) {
      for (int first = wave * 64; first < block_tokens * decay_pieces; first += 512) {
        const int index = first + lane, token = index / decay_pieces, piece = index - token * decay_pieces;
        if (token < block_tokens && t0 + token < hi)
          send_to_lds_16(a.decay + ((size_t)(t0 + token) * heads + h) * dim + piece * 4, to + decays_at + first * 4);
      }
    }
    for (int first = wave * 64; first < block_tokens * WAVE_COLS; first += 512) {
      const int index = first + lane, token = index / WAVE_COLS, column = blockIdx.x * WAVE_COLS + index % WAVE_COLS;
      if (token < block_tokens && t0 + token < hi && column < vdim) {
        const size_t at = (size_t)(t0 + token) * a.v_ld + a.v_at + (size_t)h * vdim + column;
        if (a.v_bf16) send_to_lds_2((const bf16_t*)a.v + at, to + values_at + first);
        else send_to_lds_4((const float*)a.v + at, to + values_at + first);
      }
    }
    if (wave == 7 && lane < block_tokens && t0 + lane < hi) {  // (at most 16 tokens to a block: one wave instruction each)
      if (a.beta) send_to_lds_4(a.beta + (size_t)(t0 + lane) * heads + h, to + betas_at);
      if (!per_channel) send_to_lds_4(a.decay + (size_t)(t0 + lane) * heads + h, to + head_decays_at);
    }
  };

  float* S = a.state + (((size_t)a.slots[b] * heads + h) * dim) * vdim + col;
  float s[RW];
#pragma unroll
  for (int i = 0; i < RW; ++i) s[i] = S[(size_t)(d0 + i) * vdim];

  float q[RW], k[RW], dec[RW], qn[RW], kn[RW], decn[RW];  // two sets of operands, used in turn
  float val, bet, valn = 0.f, betn = 1.f;
  const int has_beta = a.beta != nullptr, v_bf16 = a.v_bf16;
  auto fetch = [&](const float* from, int j, float (&fq)[RW], float (&fk)[RW], float (&fd)[RW], float& fv, float& fb) {
    const float one = per_channel ? 1.f : from[head_decays_at + j];
#pragma unroll
    for (int i = 0; i < RW; ++i) {
      fq[i] = from[j * 2 * dim + d0 + i];
      fk[i] = from[j * 2 * dim + dim + d0 + i];
      fd[i] = per_channel ? from[decays_at + j * dim + d0 + i] : one;
    }
    const float raw = from[values_at + j * WAVE_COLS + wave];
    fv = v_bf16 ? __uint_as_float(__float_as_uint(raw) << 16) : raw;
    fb = has_beta ? from[betas_at + j] : 1.f;
  };
  auto work = [&](const float (&wq)[RW], const float (&wk)[RW], const float (&wd)[RW], float wv, float wb) -> float {
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < RW; ++i) {
      s[i] *= wd[i];
      dot += s[i] * wk[i];
    }
    float u = wv;
    if (a.delta) u = wb * (wv - wave_total(dot));
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < RW; ++i) {
      s[i] += wk[i] * u;
      part += s[i] * wq[i];
    }
    return wave_total(part);
  };

  // Read-outs of a block wait in LDS and leave for memory at the start of the next block.
  const int outs_at = 2 * buffer_floats;
  auto flush = [&](int which, int t0, int count) {
    if (tid < count * WAVE_COLS) {
      const int token = tid / WAVE_COLS, c = tid % WAVE_COLS;
      const int column = blockIdx.x * WAVE_COLS + c;
      if (column < vdim) a.out[((size_t)(t0 + token) * heads + h) * vdim + column] = stage[outs_at + which * block_tokens * WAVE_COLS + tid];
    }
  };
  send_block(0, lo);
  wait_for_loads<0>();
  __syncthreads();
  int buffer = 0;
  for (int t0 = lo; t0 < hi; t0 += block_tokens, buffer ^= 1) {
    if (t0 > lo) flush(buffer ^ 1, t0 - block_tokens, block_tokens);
    if (t0 + block_tokens < hi) send_block(buffer ^ 1, t0 + block_tokens);  // (into the buffer that everyone left at the last barrier)
    const int count = hi - t0 < block_tokens ? hi - t0 : block_tokens;
    const float* from = stage + buffer * buffer_floats;
    float* outs = stage + outs_at + buffer * block_tokens * WAVE_COLS + wave;
    fetch(from, 0, q, k, dec, val, bet);
    int j = 0;
    for (; j + 1 < count; j += 2) {  // (a token's operands leave LDS while the token before it is worked)
      fetch(from, j + 1, qn, kn, decn, valn, betn);
      const float o0 = work(q, k, dec, val, bet);
      if (j + 2 < count) fetch(from, j + 2, q, k, dec, val, bet);
      const float o1 = work(qn, kn, decn, valn, betn);
      if (lane == 0) { outs[j * WAVE_COLS] = o0; outs[(j + 1) * WAVE_COLS] = o1; }
    }
    if (j < count) {
      const float o = work(q, k, dec, val, bet);
      if (lane == 0) outs[j * WAVE_COLS] = o;
    }
    wait_for_loads<0>();  // this wave's pieces of the next block have landed (and its stores of read-outs, long since)
    __syncthreads();
  }
  {
    const int blocks = (hi - lo + block_tokens - 1) / block_tokens;
    const int last = lo + (blocks - 1) * block_tokens;
    flush((blocks - 1) & 1, last, hi - last);
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < RW; ++i) S[(size_t)(d0 + i) * vdim] = s[i];
  }
}

// Tokens per staging block: as many as the lanes can carry and two buffers of LDS can hold, 16 at most; 0: no staging.
static int scan_block_tokens(int dim, int lanes, int per_channel) {
  if (dim % 4 != 0) return 0;
  const int cols = 256 / lanes;
  const int pieces = dim / 2 + (per_channel ? dim / 4 : 0);
  const int stride = 2 * dim + (per_channel ? dim : 0) + cols + 4;
  int tokens = 16;
  while (tokens >= 2 && (tokens * pieces > 256 * STAGE_PIECES || tokens * cols > 256 * STAGE_VALUES || 2 * tokens * stride * (int)sizeof(float) > 60 * 1024))
    tokens >>= 1;
  return tokens >= 2 ? tokens : 0;
}

extern "C" int velox_linear_scan(const float* qk, const void* v, int v_dtype, int v_ld, int v_at, const float* decay, int decay_per_channel, const float* beta,
                                 float* state, const int* slots, const int* cu_q, float* out, int num_seqs, int max_q_len, int heads, int kv_heads, int dim,
                                 int vdim, int delta, hipStream_t stream) {
  if (num_seqs <= 0) return 0;
  const int lanes = velox_linear_scan_lanes(dim);
  if (lanes > 64 || heads > 65535 || num_seqs > 65535 || kv_heads < 1 || heads % kv_heads != 0 || (delta && !beta)) return (int)hipErrorInvalidValue;
  ScanArgs a{qk, v, v_dtype == VELOX_BF16, v_ld, v_at, decay, decay_per_channel, beta, state, slots, cu_q, out, heads, kv_heads, dim, vdim, delta};
  const int cols = 256 / lanes;
  const dim3 grid((vdim + cols - 1) / cols, heads, num_seqs);
  if (max_q_len > 2 && (dim == 64 || dim == 128 || dim == 256 || dim == 512)) {
    int tokens = 16;
    while (2 * wave_buffer_floats(tokens, dim, decay_per_channel) * (int)sizeof(float) > 60 * 1024) tokens >>= 1;  // (dim = 512 with a decay per channel: 4)
    const size_t lds = (size_t)2 * (wave_buffer_floats(tokens, dim, decay_per_channel) + tokens * WAVE_COLS) * sizeof(float);  // (+ two blocks of read-outs)
    const dim3 wave_grid((vdim + WAVE_COLS - 1) / WAVE_COLS, heads, num_seqs);
    switch (dim) {
      case 64: linear_scan_wave_kernel<1><<<wave_grid, 512, lds, stream>>>(a, tokens); break;
      case 128: linear_scan_wave_kernel<2><<<wave_grid, 512, lds, stream>>>(a, tokens); break;
      case 256: linear_scan_wave_kernel<4><<<wave_grid, 512, lds, stream>>>(a, tokens); break;
      default: linear_scan_wave_kernel<8><<<wave_grid, 512, lds, stream>>>(a, tokens); break;
    }
    VELOX_RETURN_LAUNCH_STATUS();
  }
  const int block_tokens = max_q_len > 2 ? scan_block_tokens(dim, lanes, decay_per_channel) : 0;
  if (block_tokens > 0) {
    const int stride = 2 * dim + (decay_per_channel ? dim : 0) + cols + 4;
    const size_t lds = (size_t)2 * block_tokens * stride * sizeof(float);
    switch (lanes) {
      case 1: linear_scan_staged_kernel<1><<<grid, 256, lds, stream>>>(a, block_tokens); break;
      case 2: linear_scan_staged_kernel<2><<<grid, 256, lds, stream>>>(a, block_tokens); break;
      case 4: linear_scan_staged_kernel<4><<<grid, 256, lds, stream>>>(a, block_tokens); break;
      case 8: linear_scan_staged_kernel<8><<<grid, 256, lds, stream>>>(a, block_tokens); break;
      case 16: linear_scan_staged_kernel<16><<<grid, 256, lds, stream>>>(a, block_tokens); break;
      case 32: linear_scan_staged_kernel<32><<<grid, 256, lds, stream>>>(a, block_tokens); break;
      default: linear_scan_staged_kernel<64><<<grid, 256, lds, stream>>>(a, block_tokens); break;
    }
    VELOX_RETURN_LAUNCH_STATUS();
  }
  switch (lanes) {
    case 1: linear_scan_kernel<1><<<grid, 256, 0, stream>>>(a); break;
    case 2: linear_scan_kernel<2><<<grid, 256, 0, stream>>>(a); break;
    case 4: linear_scan_kernel<4><<<grid, 256, 0, stream>>>(a); break;
    case 8: linear_scan_kernel<8><<<grid, 256, 0, stream>>>(a); break;
    case 16: linear_scan_kernel<16><<<grid, 256, 0, stream>>>(a); break;
    case 32: linear_scan_kernel<32><<<grid, 256, 0, stream>>>(a); break;
    default: linear_scan_kernel<64><<<grid, 256, 0, stream>>>(a); break;
  }
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// gated_head_norm: one wave per (token, head): out = o / sqrt(mean(o^2) + eps) * w * gate, gate = silu(z) (kind 0) or
// sigmoid(z) (kind 1), z a token's row of gate_src at gate_at.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) gated_head_norm_kernel(const float* __restrict__ read, const float* __restrict__ weight, float eps,
                                                              const void* __restrict__ gate_src, int gate_bf16, int gate_ld, int gate_at, int kind,
                                                              void* __restrict__ out, int out_bf16, int heads, int vdim, size_t pairs) {
  const size_t pair = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const size_t t = pair / heads;
  const int h = (int)(pair % heads);
  const float* o = read + pair * vdim;
  float s = 0.f;
  for (int c = lane; c < vdim; c += 64) s += o[c] * o[c];
  s = wave_sum(s);
  const float inv = 1.f / sqrtf(s / (float)vdim + eps);
  for (int c = lane; c < vdim; c += 64) {
    const float z = load_as_f32(gate_src, gate_bf16, t * gate_ld + gate_at + (size_t)h * vdim + c);
    const float gate = kind == 0 ? z * sigmoid_f32(z) : sigmoid_f32(z);
    store_from_f32(out, out_bf16, pair * vdim + c, o[c] * inv * weight[c] * gate);
  }
}

extern "C" int velox_gated_head_norm(const float* read, const float* weight, float eps, const void* gate_src, int gate_dtype, int gate_ld, int gate_at,
                                     int kind, void* out, int out_dtype, int tokens, int heads, int vdim, hipStream_t stream) {
  if (tokens <= 0) return 0;
  const size_t pairs = (size_t)tokens * heads;
  gated_head_norm_kernel<<<(unsigned)((pairs + 3) / 4), 256, 0, stream>>>(read, weight, eps, gate_src, gate_dtype == VELOX_BF16, gate_ld, gate_at, kind, out,
                                                                         out_dtype == VELOX_BF16, heads, vdim, pairs);
  VELOX_RETURN_LAUNCH_STATUS();
}
