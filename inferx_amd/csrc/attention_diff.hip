// Differential attention over the paged cache, the plain kernel: one workgroup per (query token, query head).
//
// Every head has two score maps over one set of values: query head h holds maps 2h and 2h + 1 of `head_dim`
// numbers each, key/value head g = h / (heads / kv_heads) keys 2g and 2g + 1 and one value of `value_dim` numbers.
// Each map is a softmax attention of its own,
//
//   a_m = softmax_j(q_m . k_m[j] * scale) v[j],        o = a_0 - lambda a_1,
//   out = o / sqrt(mean(o^2) + eps) * mult             (no weight)
//
// over the keys that a query at position p sees: j <= p and (p - j < window or j < keep_first); window 0: all.
// Both softmaxes are kept online in float32 over chunks of 256 visible keys.  Keys are stored
// [page][2 kv_heads][offset][head_dim], values [page][kv_heads][value_dim][offset].  Any element type, head size up
// to 256, value size up to 256, any page size.
#include "common.h"

#define ATTN_DIFF_THREADS 256

template <typename T>
__global__ void __launch_bounds__(ATTN_DIFF_THREADS)
attn_diff_plain_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                       const int32_t* __restrict__ block_table, const int32_t* __restrict__ seq_of_token,
                       const int32_t* __restrict__ positions, T* __restrict__ out, int heads, int kv_heads,
                       int head_dim, int value_dim, int page_size, int max_blocks, float scale, int window,
                       int keep_first, float lambda, float eps, float mult) {
  __shared__ float qs[2][256];
  __shared__ float sc[2][ATTN_DIFF_THREADS];
  __shared__ int32_t pg[ATTN_DIFF_THREADS];
  __shared__ int32_t ky[ATTN_DIFF_THREADS];
  __shared__ float red[16];

  const int64_t t = blockIdx.x;
  const int head = blockIdx.y;
  const int g = head / (heads / kv_heads);
  const int tid = threadIdx.x;
  const int64_t seq = seq_of_token[t];
  const int pos = positions[t];
  const int start = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int kept = min(keep_first, start);           // kept first tokens that lie before the window
  const int visible = kept + pos + 1 - start;
  const int32_t* table = block_table + seq * max_blocks;

  for (int i = tid; i < 2 * head_dim; i += ATTN_DIFF_THREADS)
    qs[i / head_dim][i % head_dim] = ix_load(q + (t * heads + head) * 2 * head_dim + i);
  __syncthreads();

  float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f}, acc[2] = {0.f, 0.f};
  for (int base = 0; base < visible; base += ATTN_DIFF_THREADS) {
    const int idx = base + tid;
    const bool live = idx < visible;
    float s[2] = {-INFINITY, -INFINITY};
    int32_t page = 0, key = 0;
    if (live) {
      key = idx < kept ? idx : start + (idx - kept);
      page = table[key / page_size];
#pragma unroll
      for (int mp = 0; mp < 2; ++mp) {
        const T* kr = k_cache +
                      ((static_cast<int64_t>(page) * 2 * kv_heads + 2 * g + mp) * page_size + key % page_size) * head_dim;
        float dot = 0.f;
        for (int i = 0; i < head_dim; ++i) dot += qs[mp][i] * ix_load(kr + i);
        s[mp] = dot * scale;
      }
    }
    pg[tid] = page;
    ky[tid] = key;
    float alpha[2];
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      const float m_new = fmaxf(m[mp], ix_block_max(s[mp], red));
      const float p = live ? expf(s[mp] - m_new) : 0.f;
      sc[mp][tid] = p;
      const float chunk_sum = ix_block_sum(p, red);  // has the barriers that publish sc, pg and ky
      alpha[mp] = expf(m[mp] - m_new);               // exp(-inf) = 0 on the first chunk
      l[mp] = l[mp] * alpha[mp] + chunk_sum;
      m[mp] = m_new;
    }
    if (tid < value_dim) {
      acc[0] *= alpha[0];
      acc[1] *= alpha[1];
      const int n = min(ATTN_DIFF_THREADS, visible - base);
      for (int jj = 0; jj < n; ++jj) {
        const float v = ix_load(v_cache + ((static_cast<int64_t>(pg[jj]) * kv_heads + g) * value_dim + tid) * page_size +
                                ky[jj] % page_size);
        acc[0] += sc[0][jj] * v;
        acc[1] += sc[1][jj] * v;
      }
    }
    __syncthreads();
  }
  const float o = tid < value_dim ? acc[0] / l[0] - lambda * (acc[1] / l[1]) : 0.f;
  const float ss = ix_block_sum(o * o, red);
  if (tid < value_dim)
    ix_store(out + (t * heads + head) * value_dim + tid, o * (mult / sqrtf(ss / static_cast<float>(value_dim) + eps)));
}

extern "C" int ix_attention_diff_plain(const void* q, const void* k_cache, const void* v_cache, int dtype,
                                       const int32_t* block_table, const int32_t* seq_of_token,
                                       const int32_t* positions, void* out, int64_t tokens, int heads, int kv_heads,
                                       int head_dim, int value_dim, int page_size, int max_blocks, float scale,
                                       int window, int keep_first, float lambda, float eps, float mult,
                                       hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && max_blocks > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(head_dim > 0 && head_dim <= 256 && value_dim > 0 && value_dim <= 256,
             "head_dim and value_dim must be between 1 and 256");
  IX_REQUIRE(window >= 0 && keep_first >= 0, "window and keep_first must not be negative");
  IX_REQUIRE(heads <= 65535, "too many heads for one launch");
  if (tokens == 0) return 0;
  dim3 grid(tokens, heads), block(ATTN_DIFF_THREADS);
#define LAUNCH(TT)                                                                                                  \
  hipLaunchKernelGGL(attn_diff_plain_kernel<TT>, grid, block, 0, stream, (const TT*)q, (const TT*)k_cache,           \
                     (const TT*)v_cache, block_table, seq_of_token, positions, (TT*)out, heads, kv_heads, head_dim, \
                     value_dim, page_size, max_blocks, scale, window, keep_first, lambda, eps, mult)
  if (dtype == IX_F32) LAUNCH(float);
  else if (dtype == IX_BF16) LAUNCH(bf16_t);
  else IX_REQUIRE(false, "dtype must be float32 or bfloat16");
#undef LAUNCH
  return ix_check_launch("ix_attention_diff_plain");
}
