// Attention whose heads talk to each other before the softmax, with a sink in the softmax and a gate on every
// head's result: the step after the q|k|v|gate product, and the plain kernel.
//
//   raw_g[i, j] = (q_g[i] . k_c(g)[j]) * scale            c(g) = g / (heads / kv_heads)
//   s_h[i, j]   = sum_g talk[h, g] * raw_g[i, j]          (no talk matrix: s = raw)
//   p_h[i, j]   = exp(s_h[i, j]) / (exp(sink_h) + sum_{j' <= i} exp(s_h[i, j']))     (no sink: the usual softmax)
//   out_h[i]    = sigmoid(gate[i, h]) * sum_j p_h[i, j] v_c(h)[j]                     (no gate: factor 1)
//
// The sink is a score without key or value: the running maximum of a head starts at sink_h with a sum of one.
// Keys have `head_dim` numbers, values `value_dim`; keys are stored [page][kv_head][offset][head_dim], values
// [page][kv_head][value_dim][offset].  Scores, the mixing, exponentials and sums are float32.
#include "common.h"

// ---------------------------------------------------------------------------
// After the product: RMS norm over ALL of a token's query numbers at once (and over all of its key numbers),
// the values blended with the values that an earlier layer made for the same token, queries out, keys and
// values into the cache.  Three workgroups per token (blockIdx.y: queries, keys, values), so that what each has to
// wait for -- its own numbers, their sum of squares, the weights -- runs side by side.
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_append_kernel(const T* __restrict__ qkv, int64_t stride, const float* __restrict__ q_norm,
                      const float* __restrict__ k_norm, float eps, const T* __restrict__ v_first, float lambda,
                      T* __restrict__ v_out, const int32_t* __restrict__ slots, T* __restrict__ q_out,
                      T* __restrict__ k_cache, T* __restrict__ v_cache, int heads, int kv_heads, int head_dim,
                      int value_dim, int page_size) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int part = blockIdx.y;
  const int q_dim = heads * head_dim, k_dim = kv_heads * head_dim, v_dim = kv_heads * value_dim;
  const T* row = qkv + t * stride;
  if (part > 0 && !slots) return;
  const int64_t slot = slots ? slots[t] : 0;
  const int64_t page = slot / page_size, off = slot % page_size;
  if (part == 2) {
    for (int i = threadIdx.x; i < v_dim; i += blockDim.x) {
      const int c = i / value_dim, e = i - c * value_dim;
      float v = ix_load(row + q_dim + k_dim + i);
      if (v_first) v = (1.0f - lambda) * v + lambda * ix_load(v_first + t * v_dim + i);
      if (v_out) ix_store(v_out + t * v_dim + i, v);
      ix_store(v_cache + ((page * kv_heads + c) * value_dim + e) * page_size + off, v);
    }
    return;
  }
  const T* src = part == 0 ? row : row + q_dim;
  const float* weight = part == 0 ? q_norm : k_norm;
  const int n = part == 0 ? q_dim : k_dim;
  float inv = 1.f;
  if (weight) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const float v = ix_load(src + i);
      sq += v * v;
    }
    inv = 1.0f / sqrtf(ix_block_sum(sq, red) / static_cast<float>(n) + eps);
  }
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = ix_load(src + i) * inv * (weight ? weight[i] : 1.f);
    if (part == 0) {
      ix_store(q_out + t * q_dim + i, v);
    } else {
      const int c = i / head_dim, e = i - c * head_dim;
      ix_store(k_cache + ((page * kv_heads + c) * page_size + off) * head_dim + e, v);
    }
  }
}

extern "C" int ix_qk_norm_append(const void* qkv, int dtype, int64_t stride, const float* q_norm, const float* k_norm,
                                 float eps, const void* v_first, float lambda, void* v_out, const int32_t* slots,
                                 void* q_out, void* k_cache, void* v_cache, int64_t tokens, int heads, int kv_heads,
                                 int head_dim, int value_dim, int page_size, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && value_dim > 0 && page_size > 0,
             "sizes must be positive");
  IX_REQUIRE(stride >= static_cast<int64_t>(heads + kv_heads) * head_dim + static_cast<int64_t>(kv_heads) * value_dim,
             "a row of the product is shorter than q, k and v together");
  IX_REQUIRE(!slots || (k_cache && v_cache), "the cache is needed where slots are given");
  if (tokens == 0) return 0;
  dim3 grid(tokens, 3), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(qk_norm_append_kernel<float>, grid, block, 0, stream, (const float*)qkv, stride, q_norm, k_norm,
                       eps, (const float*)v_first, lambda, (float*)v_out, slots, (float*)q_out, (float*)k_cache,
                       (float*)v_cache, heads, kv_heads, head_dim, value_dim, page_size);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(qk_norm_append_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)qkv, stride, q_norm,
                       k_norm, eps, (const bf16_t*)v_first, lambda, (bf16_t*)v_out, slots, (bf16_t*)q_out,
                       (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, head_dim, value_dim, page_size);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_qk_norm_append");
}

// ---------------------------------------------------------------------------
// The plain kernel: one workgroup per query token serves all of its heads (each head's scores need every head's
// products), keys in chunks of 128 with the softmax kept online per head.  Any element type, page size, head and
// value size; the float32 run uses it throughout.
#define TALK_THREADS 128
#define TALK_CHUNK 128
#define TALK_MAX_ACC 32  // (head, value column) results per thread

template <typename T>
__global__ void __launch_bounds__(TALK_THREADS)
attn_talk_plain_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                       const int32_t* __restrict__ block_table, const int32_t* __restrict__ seq_of_token,
                       const int32_t* __restrict__ positions, T* __restrict__ out, const float* __restrict__ talk,
                       const float* __restrict__ sink, const T* __restrict__ gate, int64_t gate_stride, int heads,
                       int kv_heads, int head_dim, int value_dim, int page_size, int max_blocks, float scale,
                       int window) {
  extern __shared__ float smem[];
  float* qs = smem;                               // [heads * head_dim]
  float* raw = qs + heads * head_dim;             // [heads][chunk]
  float* mixed = talk ? raw + heads * TALK_CHUNK : raw;  // [heads][chunk]
  float* tk = mixed + heads * TALK_CHUNK;         // [heads * heads]
  float* m_run = tk + heads * heads;              // [heads]
  float* l_run = m_run + heads;
  float* a_run = l_run + heads;
  int32_t* pg = reinterpret_cast<int32_t*>(a_run + heads);  // [chunk]

  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & (IX_WAVE - 1), wave = tid / IX_WAVE;
  const int per_kv = heads / kv_heads;
  const int64_t seq = seq_of_token[t];
  const int pos = positions[t];
  const int start = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int32_t* table = block_table + seq * max_blocks;

  for (int i = tid; i < heads * head_dim; i += TALK_THREADS) qs[i] = ix_load(q + t * heads * head_dim + i);
  if (talk)
    for (int i = tid; i < heads * heads; i += TALK_THREADS) tk[i] = talk[i];
  for (int h = tid; h < heads; h += TALK_THREADS) {
    m_run[h] = sink ? sink[h] : -INFINITY;
    l_run[h] = sink ? 1.f : 0.f;
  }
  float acc[TALK_MAX_ACC];
#pragma unroll
  for (int k = 0; k < TALK_MAX_ACC; ++k) acc[k] = 0.f;
  const int n_out = heads * value_dim;
  __syncthreads();

  for (int base = start; base <= pos; base += TALK_CHUNK) {
    const int j = base + tid;
    const bool live = j <= pos;
    int32_t page = 0;
    if (live) {
      page = table[j / page_size];
      for (int c = 0; c < kv_heads; ++c) {
        const T* kr = k_cache + ((static_cast<int64_t>(page) * kv_heads + c) * page_size + j % page_size) * head_dim;
        for (int g = c * per_kv; g < (c + 1) * per_kv; ++g) {
          const float* qg = qs + g * head_dim;
          float dot = 0.f;
          for (int i = 0; i < head_dim; ++i) dot += qg[i] * ix_load(kr + i);
          raw[g * TALK_CHUNK + tid] = dot * scale;
        }
      }
      if (talk) {  // a thread mixes its own key's column: what it reads it wrote itself
        for (int h = 0; h < heads; ++h) {
          float s = 0.f;
          for (int g = 0; g < heads; ++g) s += tk[h * heads + g] * raw[g * TALK_CHUNK + tid];
          mixed[h * TALK_CHUNK + tid] = s;
        }
      }
    } else {
      for (int h = 0; h < heads; ++h) mixed[h * TALK_CHUNK + tid] = -INFINITY;
    }
    pg[tid] = page;
    __syncthreads();
    // every chunk holds at least one key, so a head's new maximum is finite
    for (int h = wave; h < heads; h += TALK_THREADS / IX_WAVE) {
      const float s0 = mixed[h * TALK_CHUNK + lane], s1 = mixed[h * TALK_CHUNK + IX_WAVE + lane];
      const float m_old = m_run[h];
      const float m_new = fmaxf(m_old, ix_wave_max(fmaxf(s0, s1)));
      const float p0 = expf(s0 - m_new), p1 = expf(s1 - m_new);
      mixed[h * TALK_CHUNK + lane] = p0;
      mixed[h * TALK_CHUNK + IX_WAVE + lane] = p1;
      const float sum = ix_wave_sum(p0 + p1);
      if (lane == 0) {
        const float alpha = expf(m_old - m_new);
        a_run[h] = alpha;
        l_run[h] = l_run[h] * alpha + sum;
        m_run[h] = m_new;
      }
    }
    __syncthreads();
    const int n = min(TALK_CHUNK, pos + 1 - base);
#pragma unroll
    for (int k = 0; k < TALK_MAX_ACC; ++k) {
      const int o = tid + k * TALK_THREADS;
      if (o < n_out) {
        const int h = o / value_dim, e = o - h * value_dim;
        const int c = h / per_kv;
        const float* ph = mixed + h * TALK_CHUNK;
        float a = acc[k] * a_run[h];
        for (int jj = 0; jj < n; ++jj) {
          const int key = base + jj;
          a += ph[jj] * ix_load(v_cache + ((static_cast<int64_t>(pg[jj]) * kv_heads + c) * value_dim + e) * page_size +
                                key % page_size);
        }
        acc[k] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int k = 0; k < TALK_MAX_ACC; ++k) {
    const int o = tid + k * TALK_THREADS;
    if (o < n_out) {
      const int h = o / value_dim;
      float v = acc[k] / l_run[h];
      if (gate) v *= 1.0f / (1.0f + expf(-ix_load(gate + t * gate_stride + h)));
      ix_store(out + t * n_out + o, v);
    }
  }
}

extern "C" int ix_attention_talk_plain(const void* q, const void* k_cache, const void* v_cache, int dtype,
                                       const int32_t* block_table, const int32_t* seq_of_token,
                                       const int32_t* positions, void* out, const float* talk, const float* sink,
                                       const void* gate, int64_t gate_stride, int64_t tokens, int heads, int kv_heads,
                                       int head_dim, int value_dim, int page_size, int max_blocks, float scale,
                                       int window, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && max_blocks > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(head_dim > 0 && value_dim > 0, "head and value sizes must be positive");
  IX_REQUIRE(heads * value_dim <= TALK_THREADS * TALK_MAX_ACC, "heads x value size is more than this kernel holds (4,096)");
  IX_REQUIRE(window >= 0, "window must not be negative");
  const size_t lds = (static_cast<size_t>(heads) * head_dim + static_cast<size_t>(talk ? 2 : 1) * heads * TALK_CHUNK +
                      static_cast<size_t>(heads) * heads + 3 * heads + TALK_CHUNK) * sizeof(float);
  IX_REQUIRE(lds <= 128 * 1024, "queries and scores of one token do not fit 128 KB of LDS");
  if (tokens == 0) return 0;
  dim3 grid(tokens), block(TALK_THREADS);
  if (lds > 64 * 1024) {  // more than 64 KB of LDS for a workgroup has to be allowed per kernel
    const void* fn = dtype == IX_F32 ? reinterpret_cast<const void*>(&attn_talk_plain_kernel<float>)
                                     : reinterpret_cast<const void*>(&attn_talk_plain_kernel<bf16_t>);
    IX_REQUIRE(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) == hipSuccess,
               "the kernel was refused more than 64 KB of LDS");
  }
  if (dtype == IX_F32)
    hipLaunchKernelGGL(attn_talk_plain_kernel<float>, grid, block, lds, stream, (const float*)q, (const float*)k_cache,
                       (const float*)v_cache, block_table, seq_of_token, positions, (float*)out, talk, sink,
                       (const float*)gate, gate_stride, heads, kv_heads, head_dim, value_dim, page_size, max_blocks,
                       scale, window);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(attn_talk_plain_kernel<bf16_t>, grid, block, lds, stream, (const bf16_t*)q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, seq_of_token, positions,
                       (bf16_t*)out, talk, sink, (const bf16_t*)gate, gate_stride, heads, kv_heads, head_dim,
                       value_dim, page_size, max_blocks, scale, window);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_attention_talk_plain");
}
