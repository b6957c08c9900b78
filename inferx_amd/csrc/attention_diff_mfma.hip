// Differential attention on the matrix cores (bfloat16), for prompt portions and for decoding alike.  Same
// arithmetic as the plain kernel (attention_diff.hip): per head two score maps over one set of values, a window
// with kept first tokens, softmax online in float32, then o = a_0 - lambda a_1, normalised per head.
//
// Unit of work = one wavefront: a tile of up to 16 consecutive queries of one request, one (query head, map)
// pair, one slice of the keys that the tile reads.  The operand layouts are those of attention_mfma.hip
// (S^T = K Q^T, O^T += V^T P^T with v_mfma_f32_16x16x32_bf16, nothing shuffled, no LDS, no barrier); keys are
// stored [page][2 kv_heads][offset][D] (key head 2 g + map), values [page][kv_heads][V][offset], and V may differ
// from D.  Every wavefront leaves (reference point, sum, unnormalised O) of its slice in the caller's workspace;
// a second kernel merges the slices of both maps of a (token, head), takes the difference and normalises.
//
// The keys that a tile reads are two runs: the kept first tokens that lie before the window of the tile's first
// query, [0, min(keep_first, lo)), and the window's keys up to the tile's last query, [lo, hi); rounds of 32 keys
// number both runs through, and a slice is a range of rounds.  Keys that a query of the tile does not see (before
// its own window and not kept, after its position) are masked per lane; values of keys that NO query of the tile
// may read (their pages may have been given back) are made zero before they are multiplied.
//
// GQ (grouped queries, for tiles of ONE token): the sixteen columns of a tile are the query heads that share a
// key/value head, all of the same map, so keys and values are read once per (key/value head, map); the next
// round's keys and values are asked for before the present round's are multiplied.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define DIFF_KEYS_PER_ROUND 32

template <int NB, int NBV, bool GQ>
__global__ void __launch_bounds__(256)
attn_diff_mfma_kernel(const __bf16* __restrict__ q, const __bf16* __restrict__ k_cache,
                      const __bf16* __restrict__ v_cache, const int32_t* __restrict__ block_table,
                      const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_q0,
                      const int32_t* __restrict__ tile_rows, const int32_t* __restrict__ positions,
                      float* __restrict__ part_o, float* __restrict__ part_ml, int n_tiles, int n_splits, int heads,
                      int kv_heads, int page_size, int max_blocks, float scale_log2, int window, int keep_first,
                      int page_shift) {
  constexpr int D = 16 * NB, V = 16 * NBV;
  constexpr int NC = (NB + 1) / 2;  // 32-wide chunks of the head dimension
  constexpr bool PF = GQ;
  const int lane = threadIdx.x & 63;
  const int unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= n_tiles * n_splits) return;
  const int tile = unit / n_splits, split = unit - tile * n_splits;
  const int group = heads / kv_heads;
  const int map = blockIdx.y & 1;
  const int kvh = GQ ? blockIdx.y >> 1 : (blockIdx.y >> 1) / group;
  const int n = lane & 15, g = lane >> 4;
  const int head = GQ ? kvh * group + min(n, group - 1) : blockIdx.y >> 1;
  const int key_head = 2 * kvh + map, key_heads = 2 * kv_heads;

  const int tq0 = tile_q0[tile];
  const int rows = GQ ? group : tile_rows[tile];  // columns of the tile that hold a query
  const int pos0 = positions[tq0];
  const int32_t* table = block_table + static_cast<int64_t>(tile_seq[tile]) * max_blocks;

  const int lo = (window > 0 && pos0 + 1 > window) ? pos0 + 1 - window : 0;
  const int hi = pos0 + (GQ ? 1 : rows);
  const int lo_al = lo & ~(DIFF_KEYS_PER_ROUND - 1);
  const int kept = min(keep_first, lo);  // kept first tokens before the window
  const int rounds_kept = min((kept + DIFF_KEYS_PER_ROUND - 1) & ~(DIFF_KEYS_PER_ROUND - 1), lo_al) / DIFF_KEYS_PER_ROUND;
  const int n_rounds = rounds_kept + (hi - lo_al + DIFF_KEYS_PER_ROUND - 1) / DIFF_KEYS_PER_ROUND;
  const int per = (n_rounds + n_splits - 1) / n_splits;
  const int r0 = split * per, r1 = min(n_rounds, r0 + per);
  auto first_key = [&](int r) {
    return r < rounds_kept ? r * DIFF_KEYS_PER_ROUND : lo_al + (r - rounds_kept) * DIFF_KEYS_PER_ROUND;
  };

  // Q as B operand: lane (n, g) holds Q[query n][32 c + 8 g .. +8]
  bf16x8 qf[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int d0 = 32 * c + 8 * g;
    if (n < rows && d0 < D)
      qf[c] = *reinterpret_cast<const bf16x8*>(
          q + ((static_cast<int64_t>(tq0 + (GQ ? 0 : n)) * heads + head) * 2 + map) * D + d0);
    else
      for (int j = 0; j < 8; ++j) qf[c][j] = (__bf16)0.f;
  }

  f32x4 o[NBV];
#pragma unroll
  for (int b = 0; b < NBV; ++b) o[b] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;

  auto page_of = [&](int key) { return page_shift >= 0 ? key >> page_shift : key / page_size; };
  // K fragments for the 32 keys from kb on (two blocks of 16 rows: row m of the first block is key 8 (m / 4) + m % 4,
  // of the second 8 (m / 4) + 4 + m % 4) and V^T fragments (lane (n, g) holds V^T[16 b + n][kb + 8 g .. +8])
  auto load_kv = [&](int kb, bf16x8 (&kf)[2][NC], bf16x8 (&vf)[NBV]) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int key = min(kb + 8 * (n >> 2) + 4 * b + (n & 3), hi - 1);  // rows past the end are masked below
      const int pi = page_of(key);
      const int page = max(table[pi], 0);  // a page that the window has passed: masked below
      const __bf16* kr =
          k_cache + ((static_cast<int64_t>(page) * key_heads + key_head) * page_size + (key - pi * page_size)) * D;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d0 = 32 * c + 8 * g;
        if (d0 < D)
          kf[b][c] = *reinterpret_cast<const bf16x8*>(kr + d0);
        else
          for (int j = 0; j < 8; ++j) kf[b][c][j] = (__bf16)0.f;
      }
    }
    const int key = min(kb + 8 * g, hi - 1) & ~7;
    const int pi = page_of(key);
    const int page = max(table[pi], 0);
    const __bf16* vr = v_cache + (static_cast<int64_t>(page) * kv_heads + kvh) * V * page_size + (key - pi * page_size);
#pragma unroll
    for (int b = 0; b < NBV; ++b)
      vf[b] = *reinterpret_cast<const bf16x8*>(vr + static_cast<int64_t>(16 * b + n) * page_size);
  };

  bf16x8 kf_next[PF ? 2 : 1][PF ? NC : 1], vf_next[PF ? NBV : 1];
  if constexpr (PF) {
    if (r0 < r1) load_kv(first_key(r0), kf_next, vf_next);
  }
  for (int r = r0; r < r1; ++r) {
    const int kb = first_key(r);
    bf16x8 kf[2][NC], vf[NBV];
    if constexpr (PF) {
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int c = 0; c < NC; ++c) kf[b][c] = kf_next[b][c];
#pragma unroll
      for (int b = 0; b < NBV; ++b) vf[b] = vf_next[b];
      if (r + 1 < r1) load_kv(first_key(r + 1), kf_next, vf_next);
    } else {
      load_kv(kb, kf, vf);
    }
    // values of keys that no query of the tile may read: zero (their probability is zero, but zero times whatever
    // lies there need not be)
    if (kb + DIFF_KEYS_PER_ROUND > hi || (kb < lo && kb + DIFF_KEYS_PER_ROUND > keep_first)) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = (min(kb + 8 * g, hi - 1) & ~7) + j;
        if (key >= hi || (key < lo && key >= keep_first)) {
#pragma unroll
          for (int b = 0; b < NBV; ++b) vf[b][j] = (__bf16)0.f;
        }
      }
    }
    // ---- S^T = K Q^T ----
    f32x4 s[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      s[b] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < NC; ++c) s[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[b][c], qf[c], s[b], 0, 0, 0);
    }
    // ---- mask, online softmax for this lane's query over its 8 keys ----
    const int my_pos = pos0 + (GQ ? 0 : n);
    const bool my_row = n < rows;
    const int my_lo = (window > 0 && my_pos + 1 > window) ? my_pos + 1 - window : 0;
    float sv[8];
    float mx = -INFINITY;
    // keys that every query of the tile sees need no mask (uniform over the wavefront)
    const int last_pos = pos0 + (GQ ? 0 : 15);
    const bool inner = (GQ || rows == 16) && kb + DIFF_KEYS_PER_ROUND - 1 <= pos0 &&
                       (window == 0 || kb > last_pos - window || kb + DIFF_KEYS_PER_ROUND <= keep_first);
    if (inner) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        sv[j] = s[j >> 2][j & 3];
        mx = fmaxf(mx, sv[j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = kb + 8 * g + j;
        const bool ok = my_row && key <= my_pos && key < hi && (key >= my_lo || key < keep_first);
        sv[j] = ok ? s[j >> 2][j & 3] : -INFINITY;
        mx = fmaxf(mx, sv[j]);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // the reference point of the exponentials (in units of log2) follows the running maximum lazily
    const float top = mx * scale_log2;
    if (__any(top > m + 8.f)) {
      const float m_new = fmaxf(m, top);
      const float alpha = __builtin_amdgcn_exp2f(m - ((m_new == -INFINITY) ? 0.f : m_new));
      lsum *= alpha;
#pragma unroll
      for (int b = 0; b < NBV; ++b) o[b] *= alpha;
      m = m_new;
    }
    const float m_safe = (m == -INFINITY) ? 0.f : m;
    float psum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float p = __builtin_amdgcn_exp2f(fmaf(sv[j], scale_log2, -m_safe));
      psum += p;
      pf[j] = (__bf16)p;
    }
    lsum += psum;
    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int b = 0; b < NBV; ++b) o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[b], pf, o[b], 0, 0, 0);
  }

  float l = lsum;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (n >= rows) return;
  // lane holds O^T rows 16 b + 4 g + i of column n
  const int64_t token = tq0 + (GQ ? 0 : n);
  const int64_t p = ((token * heads + head) * 2 + map) * n_splits + split;
  float* dst = part_o + p * V + 4 * g;
#pragma unroll
  for (int b = 0; b < NBV; ++b) *reinterpret_cast<f32x4*>(dst + 16 * b) = o[b];
  if (g == 0) {
    part_ml[2 * p] = m;
    part_ml[2 * p + 1] = l;
  }
}

// Per (token, head), one wavefront: both maps' slices merged (a_m = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M)),
// o = a_0 - lambda a_1, out = o / sqrt(mean(o^2) + eps) * mult.  At most 64 slices, value_dim at most 256.
// NS: the number of slices where it is 1, 2, 4 or 8 (the loop over them is then unrolled whole, so that every load of
// the launch is in flight at once), else 0.
template <int NS>
__global__ void __launch_bounds__(256)
attn_diff_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                         __bf16* __restrict__ out, int64_t pairs, int n_splits_any, int value_dim, float lambda,
                         float eps, float mult) {
  const int n_splits = NS > 0 ? NS : n_splits_any;
  const int64_t th = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);  // token * heads + head
  if (th >= pairs) return;
  const int lane = threadIdx.x & 63;
  // both maps' reference points and sums are asked for first, then all parts: the loads of a launch this small
  // should all be in flight together
  float a[2][4], w[2], inv_l[2];
  float m_s[2], l_s[2];
  const float* po = part_o + th * 2 * n_splits * value_dim;
  // (columns past the head's end read its last column again: every load is unconditional; what they sum is dropped)
  float parts[2][NS > 0 ? NS : 1][4];
  if constexpr (NS > 0) {  // the parts themselves first: they wait for nothing
#pragma unroll
    for (int mp = 0; mp < 2; ++mp)
#pragma unroll
      for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
          parts[mp][s][jj] = 64 * jj < value_dim
                                 ? po[static_cast<int64_t>(mp * NS + s) * value_dim + min(lane + 64 * jj, value_dim - 1)]
                                 : 0.f;
  }
#pragma unroll
  for (int mp = 0; mp < 2; ++mp) {
    const int64_t p0 = (th * 2 + mp) * n_splits;
    m_s[mp] = lane < n_splits ? part_ml[2 * (p0 + lane)] : -INFINITY;
    l_s[mp] = lane < n_splits ? part_ml[2 * (p0 + lane) + 1] : 0.f;
  }
#pragma unroll
  for (int mp = 0; mp < 2; ++mp) {
    const float M = ix_wave_max(m_s[mp]);
    w[mp] = (m_s[mp] == -INFINITY) ? 0.f : exp2f(m_s[mp] - M);
    inv_l[mp] = 1.0f / ix_wave_sum(w[mp] * l_s[mp]);
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) a[mp][jj] = 0.f;
  }
  auto take = [&](int s) {
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      const float ws = __shfl(w[mp], s, 64);
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
        if (64 * jj < value_dim)
          a[mp][jj] += ws * po[static_cast<int64_t>(mp * n_splits + s) * value_dim + min(lane + 64 * jj, value_dim - 1)];
    }
  };
  if constexpr (NS > 0) {
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int mp = 0; mp < 2; ++mp) {
        const float ws = __shfl(w[mp], s, 64);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) a[mp][jj] += ws * parts[mp][s][jj];
      }
  } else {
#pragma unroll 4
    for (int s = 0; s < n_splits; ++s) take(s);
  }
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) a[mp][jj] *= inv_l[mp];
  float ss = 0.f;
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    a[0][jj] = lane + 64 * jj < value_dim ? a[0][jj] - lambda * a[1][jj] : 0.f;
    ss += a[0][jj] * a[0][jj];
  }
  ss = ix_wave_sum(ss);
  const float f = mult / sqrtf(ss / static_cast<float>(value_dim) + eps);
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    const int j = lane + 64 * jj;
    if (j < value_dim) out[th * value_dim + j] = (__bf16)(a[0][jj] * f);
  }
}

template <int NB, int NBV, bool GQ>
static void launch_diff(dim3 grid, hipStream_t stream, const void* q, const void* k, const void* v,
                        const int32_t* table, const int32_t* tile_seq, const int32_t* tile_q0,
                        const int32_t* tile_rows, const int32_t* positions, float* part_o, float* part_ml, int n_tiles,
                        int n_splits, int heads, int kv_heads, int page_size, int max_blocks, float scale_log2,
                        int window, int keep_first) {
  int page_shift = -1;  // log2 of the page size if it is a power of two
  for (int b = 4; b < 31; ++b)
    if (page_size == (1 << b)) page_shift = b;
  // four wavefronts per workgroup, two or one while that makes fewer than two workgroups per compute unit
  const int64_t waves = static_cast<int64_t>(n_tiles) * n_splits * grid.y;
  const int per_group = waves >= 4 * 512 ? 4 : (waves >= 2 * 512 ? 2 : 1);
  grid.x = static_cast<unsigned>((static_cast<int64_t>(n_tiles) * n_splits + per_group - 1) / per_group);
  hipLaunchKernelGGL((attn_diff_mfma_kernel<NB, NBV, GQ>), grid, dim3(64 * per_group), 0, stream, (const __bf16*)q,
                     (const __bf16*)k, (const __bf16*)v, table, tile_seq, tile_q0, tile_rows, positions, part_o,
                     part_ml, n_tiles, n_splits, heads, kv_heads, page_size, max_blocks, scale_log2, window,
                     keep_first, page_shift);
}

// the sizes of heads (in sixteens) that the kernel is built for, keys and values alike
static bool diff_size_built(int sixteens) {
  return sixteens == 1 || sixteens == 2 || sixteens == 3 || sixteens == 4 || sixteens == 6 || sixteens == 8;
}

extern "C" int ix_attention_diff_mfma_fits(int head_dim, int value_dim, int page_size) {
  return head_dim % 16 == 0 && value_dim % 16 == 0 && diff_size_built(head_dim / 16) && diff_size_built(value_dim / 16) &&
         page_size > 0 && page_size % 16 == 0;
}

// q [tokens, heads, 2, head_dim]; k_cache [pages, 2 kv_heads, page, head_dim]; v_cache [pages, kv_heads, value_dim,
// page]; out [tokens, heads, value_dim]; tiles as for ix_attention_mfma (up to 16 queries each).  Workspace:
// part_o float32 [tokens * heads * 2 * n_splits * value_dim], part_ml float32 [tokens * heads * 2 * n_splits * 2].
// grouped: every tile is ONE token, and a wavefront serves the query heads of one key/value head together.
extern "C" int ix_attention_diff_mfma(const void* q, const void* k_cache, const void* v_cache,
                                      const int32_t* block_table, const int32_t* tile_seq, const int32_t* tile_q0,
                                      const int32_t* tile_rows, const int32_t* positions, void* out, float* part_o,
                                      float* part_ml, int64_t tokens, int n_tiles, int n_splits, int heads,
                                      int kv_heads, int head_dim, int value_dim, int page_size, int max_blocks,
                                      float scale, int window, int keep_first, float lambda, float eps, float mult,
                                      int grouped, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && n_tiles >= 0 && heads > 0 && kv_heads > 0 && max_blocks > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(ix_attention_diff_mfma_fits(head_dim, value_dim, page_size),
             "head_dim and value_dim must be 16, 32, 48, 64, 96 or 128, pages a multiple of 16");
  IX_REQUIRE(n_splits >= 1 && n_splits <= 64, "n_splits must be between 1 and 64");
  IX_REQUIRE(part_o != nullptr && part_ml != nullptr, "the workspace is needed");
  IX_REQUIRE(window >= 0 && keep_first >= 0, "window and keep_first must not be negative");
  IX_REQUIRE(2 * heads <= 65535, "too many heads");
  IX_REQUIRE(!grouped || heads / kv_heads <= 16, "grouped queries: at most 16 query heads per key/value head");
  if (n_tiles == 0 || tokens == 0) return 0;
  const int64_t units = static_cast<int64_t>(n_tiles) * n_splits;
  dim3 grid(static_cast<unsigned>((units + 3) / 4), 2 * (grouped ? kv_heads : heads));
  const float scale_log2 = scale * 1.4426950408889634f;
#define ARGS                                                                                                       \
  grid, stream, q, k_cache, v_cache, block_table, tile_seq, tile_q0, tile_rows, positions, part_o, part_ml, n_tiles, \
      n_splits, heads, kv_heads, page_size, max_blocks, scale_log2, window, keep_first
#define CASEV(NB, NBV)                                \
  case NBV:                                           \
    if (grouped) launch_diff<NB, NBV, true>(ARGS);    \
    else launch_diff<NB, NBV, false>(ARGS);           \
    break;
#define CASE(NB)                                                                  \
  case NB:                                                                        \
    switch (value_dim / 16) {                                                     \
      CASEV(NB, 1) CASEV(NB, 2) CASEV(NB, 3) CASEV(NB, 4) CASEV(NB, 6) CASEV(NB, 8) \
    }                                                                             \
    break;
  switch (head_dim / 16) { CASE(1) CASE(2) CASE(3) CASE(4) CASE(6) CASE(8) }
#undef CASE
#undef CASEV
#undef ARGS
  if (ix_check_launch("ix_attention_diff_mfma")) return 1;
  const int64_t pairs = tokens * heads;
#define MERGE(NS)                                                                                                   \
  hipLaunchKernelGGL(attn_diff_combine_kernel<NS>, dim3(static_cast<unsigned>((pairs + 3) / 4)), dim3(256), 0, stream, \
                     part_o, part_ml, (__bf16*)out, pairs, n_splits, value_dim, lambda, eps, mult)
  switch (n_splits) {
    case 1: MERGE(1); break;
    case 2: MERGE(2); break;
    case 4: MERGE(4); break;
    case 8: MERGE(8); break;
    default: MERGE(0); break;
  }
#undef MERGE
  return ix_check_launch("ix_attention_diff_mfma (merge)");
}
