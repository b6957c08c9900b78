// Attention whose heads talk to each other before the softmax (see attention_talk.hip for the arithmetic), on the
// matrix cores, bfloat16, for prompt portions and single tokens alike.
//
// A head's scores need every head's products, so the unit of work is a WORKGROUP: a tile of up to 16 consecutive
// queries of one request, over one slice of the tile's keys, for all heads.  Its wavefronts own HPW heads each (of
// one key/value head).  Per round of 32 keys a wavefront
//   1. forms the raw products of its heads,  S^T[key][query] = K[key][:] . Q[query][:]   (v_mfma_f32_16x16x32_bf16,
//      operand layouts as in attention_mfma.hip: a lane ends up with eight consecutive keys of its query),
//   2. leaves them in LDS, one 16-byte piece per lane, head and half (lanes side by side: no bank conflicts),
//   3. after one barrier reads the pieces of ALL heads at its own lane's place and mixes them into the scores of its
//      own heads in float32 (the mixing matrix is in LDS too),
//   4. keeps the softmax online per head and accumulates O^T += V^T P^T.
// The raw products are kept twice (rounds alternate between two buffers), so one barrier a round is enough; beyond
// sixteen heads there is one buffer and a second barrier.  Without a mixing matrix nothing goes through LDS.
//
// The sink is a score without key or value: slice 0 starts a head's running maximum at the sink with a sum of one.
// With several slices every workgroup writes (maximum, sum, unnormalised O) per head and a second kernel merges
// them; the sigmoid gate is applied where the result is written.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define TALK_KEYS_PER_ROUND 32
#define TALK_LOG2E 1.4426950408889634f

// A workgroup barrier that waits for this wavefront's LDS traffic only: `__syncthreads()` also waits for every load
// from memory that is on its way, which would undo the loads that run a round ahead.
__device__ __forceinline__ void talk_lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

struct TalkArgs {
  const __bf16* q;        // [tokens, heads, head_dim]
  const __bf16* k_cache;  // [pages, kv_heads, page_size, head_dim]
  const __bf16* v_cache;  // [pages, kv_heads, value_dim, page_size]
  const int32_t* block_table;
  const int32_t* tile_seq;
  const int32_t* tile_q0;
  const int32_t* tile_rows;
  const int32_t* positions;
  __bf16* out;            // [tokens, heads, value_dim]
  float* part_o;
  float* part_ml;
  const float* talk;      // [heads, heads] or null
  const float* sink;      // [heads] or null
  const __bf16* gate;     // [tokens] rows of `gate_stride`, heads numbers each, or null
  int64_t gate_stride;
  int n_tiles, n_splits, heads, kv_heads, head_dim, value_dim, page_size, max_blocks;
  float scale;
  int page_shift;  // log2 of the page size if it is a power of two (the usual case, which spares the divisions), else -1
};

// SZ: head_dim and value_dim are at most SZ (multiples of 16); HPW: heads per wavefront; MAXW: most wavefronts of a
// workgroup (which decides how many registers a wavefront may have); TALK: heads are mixed
template <int SZ, int HPW, int MAXW, bool TALK>
__global__ void __launch_bounds__(64 * MAXW)
talk_mfma_kernel(TalkArgs a) {
  constexpr int NC = SZ / 32 > 0 ? SZ / 32 : 1;  // 32-wide chunks of a key
  constexpr int NB = SZ / 16;                    // 16-wide blocks of a value
  extern __shared__ float smem[];
  const int H = a.heads, D = a.head_dim, E = a.value_dim;
  const int n_buffers = H > 16 ? 1 : 2;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = blockIdx.x;
  // (the last tiles of a prompt read the most keys: they start first)
  const int tile = a.n_tiles - 1 - unit / a.n_splits, split = unit % a.n_splits;
  const int group = H / a.kv_heads;
  const int h0 = wave * HPW;
  const int kvh = h0 / group;
  const int n = lane & 15, g = lane >> 4;

  const int tq0 = a.tile_q0[tile];
  const int rows = a.tile_rows[tile];
  const int pos0 = a.positions[tq0];
  const int32_t* table = a.block_table + static_cast<int64_t>(a.tile_seq[tile]) * a.max_blocks;
  const int hi = pos0 + rows;  // keys [0, hi)
  const int per = (((hi + a.n_splits - 1) / a.n_splits) + TALK_KEYS_PER_ROUND - 1) & ~(TALK_KEYS_PER_ROUND - 1);
  const int ks = split * per;
  const int ke = min(hi, ks + per);
  const float scale_log2 = a.scale * TALK_LOG2E;

  // the mixing matrix in LDS, its rows padded to a multiple of four (the scale and log2 e follow once, on the
  // mixed score).  Asking for four heads' pieces and weights at a time, and the weights as scalar operands through
  // the scalar cache, were both tried: the first spills registers at heads of 128, neither was faster.
  const int H4 = (H + 3) & ~3;
  float* tk = smem + static_cast<size_t>(n_buffers) * H * 2 * 64 * 4;  // [H][H4]
  if constexpr (TALK) {
    for (int i = threadIdx.x; i < H * H4; i += blockDim.x) {
      const int r = i / H4, c = i - r * H4;
      tk[i] = c < H ? a.talk[r * H + c] : 0.f;
    }
    __syncthreads();
  }

  // Q as B operand: lane (n, g) holds Q[query n][32 c + 8 g .. +8] of each of its heads
  bf16x8 qf[HPW][NC];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d0 = 32 * c + 8 * g;
      if (n < rows && d0 < D)
        qf[hh][c] = *reinterpret_cast<const bf16x8*>(a.q + (static_cast<int64_t>(tq0 + n) * H + h0 + hh) * D + d0);
      else
        for (int j = 0; j < 8; ++j) qf[hh][c][j] = (__bf16)0.f;
    }

  f32x4 o[HPW][NB];
  float m[HPW], lsum[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    const bool sunk = a.sink != nullptr && split == 0;
    m[hh] = sunk ? a.sink[h0 + hh] * TALK_LOG2E : -INFINITY;
    lsum[hh] = (sunk && g == 0) ? 1.f : 0.f;  // (a lane's sum is one of four that are added at the end)
#pragma unroll
    for (int b = 0; b < NB; ++b) o[hh][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // Loads run ahead of their use: the keys of round r + 1 are asked for at the start of round r, the values of round
  // r after its raw products (asked for earlier they cost registers that then spill: measured slower), and the
  // pages of both a round before that, so that no load in the loop waits for another one's result.  Every load is unconditional: keys past the tile's
  // last one are clamped onto it and masked.
  auto page_of = [&](int key) { return a.page_shift >= 0 ? key >> a.page_shift : key / a.page_size; };
  auto ask_pages = [&](int kb, int (&pk)[2], int& pv) {
#pragma unroll
    for (int b = 0; b < 2; ++b) pk[b] = table[page_of(min(kb + 8 * (n >> 2) + 4 * b + (n & 3), hi - 1))];
    pv = table[page_of(min(kb + 8 * g, hi - 1) & ~7)];
  };
  auto load_keys = [&](int kb, const int (&pk)[2], bf16x8 (&kf)[2][NC]) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int key = min(kb + 8 * (n >> 2) + 4 * b + (n & 3), hi - 1);  // rows past the end are masked below
      const int pi = page_of(key);
      const __bf16* kr = a.k_cache + ((static_cast<int64_t>(max(pk[b], 0)) * a.kv_heads + kvh) * a.page_size +
                                      (key - pi * a.page_size)) * D;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d0 = 32 * c + 8 * g;
        if (d0 < D)
          kf[b][c] = *reinterpret_cast<const bf16x8*>(kr + d0);
        else
          for (int j = 0; j < 8; ++j) kf[b][c][j] = (__bf16)0.f;
      }
    }
  };
  auto load_values = [&](int kb, int pv, bf16x8 (&vf)[NB]) {
    const int key = min(kb + 8 * g, hi - 1) & ~7;
    const int pi = page_of(key);
    const __bf16* vr = a.v_cache + (static_cast<int64_t>(max(pv, 0)) * a.kv_heads + kvh) * E * a.page_size +
                       (key - pi * a.page_size);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (16 * b < E)
        vf[b] = *reinterpret_cast<const bf16x8*>(vr + static_cast<int64_t>(16 * b + n) * a.page_size);
      else
        for (int j = 0; j < 8; ++j) vf[b][j] = (__bf16)0.f;
    }
  };

  bf16x8 kf[2][NC];
  int pk_next[2], pv_now = 0, pv_next = 0;
  if (ks < ke) {
    int pk_now[2];
    ask_pages(ks, pk_now, pv_now);
    ask_pages(ks + TALK_KEYS_PER_ROUND, pk_next, pv_next);
    load_keys(ks, pk_now, kf);
  }
  int round = 0;
  for (int kb = ks; kb < ke; kb += TALK_KEYS_PER_ROUND, ++round) {
    bf16x8 kf_next[2][NC], vf[NB];
    int pk_after[2], pv_after;
    load_keys(kb + TALK_KEYS_PER_ROUND, pk_next, kf_next);
    ask_pages(kb + 2 * TALK_KEYS_PER_ROUND, pk_after, pv_after);
    __builtin_amdgcn_sched_barrier(0);
    // ---- raw products of this wavefront's heads ----
    f32x4 s[HPW][2];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        s[hh][b] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NC; ++c)
          s[hh][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[b][c], qf[hh][c], s[hh][b], 0, 0, 0);
      }
    load_values(kb, pv_now, vf);  // (used at the round's end: the exchange and the mixing hide their way)
    __builtin_amdgcn_sched_barrier(0);
    // ---- the heads talk ----
    f32x4 mixed[HPW][2];
    if constexpr (TALK) {
      f32x4* buf = reinterpret_cast<f32x4*>(smem) + static_cast<size_t>(round & (n_buffers - 1)) * H * 2 * 64;
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int b = 0; b < 2; ++b) buf[((h0 + hh) * 2 + b) * 64 + lane] = s[hh][b];
      talk_lds_barrier();
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int b = 0; b < 2; ++b) mixed[hh][b] = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int o_head = 0; o_head < H; ++o_head) {
        const f32x4 r0 = buf[(o_head * 2) * 64 + lane], r1 = buf[(o_head * 2 + 1) * 64 + lane];
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
          const float w = tk[(h0 + hh) * H4 + o_head];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            mixed[hh][0][i] = fmaf(w, r0[i], mixed[hh][0][i]);
            mixed[hh][1][i] = fmaf(w, r1[i], mixed[hh][1][i]);
          }
        }
      }
      if (n_buffers == 1) talk_lds_barrier();
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int b = 0; b < 2; ++b) mixed[hh][b] *= scale_log2;
    } else {
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int b = 0; b < 2; ++b) mixed[hh][b] = s[hh][b] * scale_log2;
    }
    // values of keys past the tile's last one (whatever an earlier request left there) are made zero: their
    // probability is zero, but zero times not-a-number is not
    if (kb + TALK_KEYS_PER_ROUND > hi) {
      const int key = min(kb + 8 * g, hi - 1) & ~7;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (key + j >= hi) {
#pragma unroll
          for (int b = 0; b < NB; ++b) vf[b][j] = (__bf16)0.f;
        }
    }
    // ---- mask, online softmax per head (scores are in units of log2), O^T += V^T P^T ----
    const int my_pos = pos0 + n;
    const bool my_row = n < rows;
    // a round whose 32 keys every query of the tile sees needs no mask (columns without a query hold zeros for q:
    // what they sum is finite and is not stored)
    const bool inner = kb + TALK_KEYS_PER_ROUND <= ke && kb + TALK_KEYS_PER_ROUND - 1 <= pos0;
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      float sv[8];
      float mx = -INFINITY;
      if (inner) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          sv[j] = mixed[hh][j >> 2][j & 3];
          mx = fmaxf(mx, sv[j]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = kb + 8 * g + j;
          const bool ok = my_row && key <= my_pos && key < ke;
          sv[j] = ok ? mixed[hh][j >> 2][j & 3] : -INFINITY;
          mx = fmaxf(mx, sv[j]);
        }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      // The reference point m of the exponentials follows the running maximum lazily: it moves only when some
      // query's maximum has outgrown it by more than 2^8, so the accumulators are seldom rescaled.  Any m gives the
      // same quotient; probabilities up to 2^8 keep the relative precision of bfloat16.
      if (__any(mx > m[hh] + 8.f)) {
        const float m_new = fmaxf(m[hh], mx);
        const float alpha = __builtin_amdgcn_exp2f(m[hh] - ((m_new == -INFINITY) ? 0.f : m_new));
        lsum[hh] *= alpha;
#pragma unroll
        for (int b = 0; b < NB; ++b) o[hh][b] *= alpha;
        m[hh] = m_new;
      }
      const float m_safe = (m[hh] == -INFINITY) ? 0.f : m[hh];
      float psum = 0.f;
      bf16x8 pf;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float p = __builtin_amdgcn_exp2f(sv[j] - m_safe);
        psum += p;
        pf[j] = (__bf16)p;
      }
      lsum[hh] += psum;
#pragma unroll
      for (int b = 0; b < NB; ++b)
        if (16 * b < E) o[hh][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[b], pf, o[hh][b], 0, 0, 0);
    }
#pragma unroll
    for (int b = 0; b < 2; ++b) {
#pragma unroll
      for (int c = 0; c < NC; ++c) kf[b][c] = kf_next[b][c];
      pk_next[b] = pk_after[b];
    }
    pv_now = pv_next;
    pv_next = pv_after;
  }

#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    float l = lsum[hh];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (n >= rows) continue;
    const int head = h0 + hh;
    const int64_t token = tq0 + n;  // lane holds O^T rows 16 b + 4 g + i of column n
    if (a.n_splits == 1) {
      float f = 1.0f / l;
      if (a.gate) f *= 1.0f / (1.0f + expf(-static_cast<float>(a.gate[token * a.gate_stride + head])));
      __bf16* dst = a.out + (token * H + head) * E + 4 * g;
#pragma unroll
      for (int b = 0; b < NB; ++b)
        if (16 * b < E) {
          bf16x4 v;
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = (__bf16)(o[hh][b][i] * f);
          *reinterpret_cast<bf16x4*>(dst + 16 * b) = v;
        }
    } else {
      const int64_t p = (token * H + head) * a.n_splits + split;
      float* dst = a.part_o + p * E + 4 * g;
#pragma unroll
      for (int b = 0; b < NB; ++b)
        if (16 * b < E) *reinterpret_cast<f32x4*>(dst + 16 * b) = o[hh][b];
      if (g == 0) {
        a.part_ml[2 * p] = m[hh];
        a.part_ml[2 * p + 1] = l;
      }
    }
  }
}

// out[t, h, :] = gate * sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M),  M = max_s m_s.  A wavefront per (token,
// head): a lane per slice works out the slices' weights, then a lane per value column sums over the slices with
// independent loads.
__global__ void __launch_bounds__(256)
talk_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, __bf16* __restrict__ out,
                    const __bf16* __restrict__ gate, int64_t gate_stride, int64_t pairs, int heads, int n_splits,
                    int value_dim) {
  __shared__ float wgt[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t th = static_cast<int64_t>(blockIdx.x) * 4 + wave;  // token * heads + head
  if (th >= pairs) return;
  const float* ml = part_ml + th * n_splits * 2;
  const float m_s = lane < n_splits ? ml[2 * lane] : -INFINITY;
  const float M = ix_wave_max(m_s);
  const float w = (m_s == -INFINITY) ? 0.f : exp2f(m_s - M);
  wgt[wave][lane] = w;  // (a wavefront's own row: written and read in lockstep)
  const float L = ix_wave_sum(lane < n_splits ? w * ml[2 * lane + 1] : 0.f);
  float f = 1.0f / L;
  if (gate) f *= 1.0f / (1.0f + expf(-static_cast<float>(gate[(th / heads) * gate_stride + th % heads])));
  const float* po = part_o + th * n_splits * value_dim;
  for (int d = lane; d < value_dim; d += 64) {
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < n_splits; ++s) acc += wgt[wave][s] * po[s * value_dim + d];
    out[th * value_dim + d] = (__bf16)(acc * f);
  }
}

template <int SZ, int HPW, int MAXW>
static int launch_talk(const TalkArgs& a, size_t lds, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(a.n_tiles) * a.n_splits), block(64 * (a.heads / HPW));
  if (a.talk) {
    // more than 64 KB of LDS for a workgroup has to be allowed per kernel, once
    static bool allowed = false;
    if (lds > 64 * 1024 && !allowed) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&talk_mfma_kernel<SZ, HPW, MAXW, true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) != hipSuccess) {
        ix_set_error("ix_attention_talk_mfma: the kernel was refused more than 64 KB of LDS");
        return 1;
      }
      allowed = true;
    }
    hipLaunchKernelGGL((talk_mfma_kernel<SZ, HPW, MAXW, true>), grid, block, lds, stream, a);
  } else
    hipLaunchKernelGGL((talk_mfma_kernel<SZ, HPW, MAXW, false>), grid, block, 0, stream, a);
  return 0;
}

// Which forms of the kernel are built: heads per wavefront HPW, and the most wavefronts of a workgroup MAXW (4, 8 or
// 16, which leaves a wavefront 512, 256 or 128 registers).  The forms that keep their accumulators, queries, keys
// and values in registers without spilling, by the compiler's own count; a few that spill some are kept as a last
// resort for many heads, where the alternative is the plain kernel.
static bool talk_form_built(int sz, int hpw, int maxw) {
  switch (sz) {
    case 32:
    case 64: return hpw < 4 || maxw <= 8;
    case 128: return hpw == 1 || maxw <= 8;
    default: return hpw == 1 && maxw <= 8;
  }
}
static bool talk_form_spills(int sz, int hpw, int maxw) {
  return (sz == 64 && hpw == 2 && maxw == 16) || (sz == 128 && ((hpw == 1 && maxw == 16) || hpw == 4)) ||
         (sz == 256 && maxw == 8);
}

// How many heads a wavefront takes for these sizes (0: the kernel does not take them).  A wavefront's heads share
// a key/value head, and a workgroup holds at most sixteen wavefronts; of the forms that fit, the one with the most
// wavefronts that does not spill.
extern "C" int ix_attention_talk_mfma_heads_per_wave(int heads, int kv_heads, int head_dim, int value_dim,
                                                     int page_size) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads) return 0;
  if (head_dim <= 0 || value_dim <= 0 || head_dim % 16 || value_dim % 16 || page_size <= 0 || page_size % 16) return 0;
  const int big = std::max(head_dim, value_dim);
  if (big > 256 || heads > 32) return 0;
  const int sz = big <= 32 ? 32 : (big <= 64 ? 64 : (big <= 128 ? 128 : 256));
  const int group = heads / kv_heads;
  int spilling = 0;
  for (int hpw = 1; hpw <= 4; hpw *= 2) {
    if (group % hpw || heads / hpw > 16) continue;
    const int waves = heads / hpw, maxw = waves <= 4 ? 4 : (waves <= 8 ? 8 : 16);
    if (!talk_form_built(sz, hpw, maxw)) continue;
    if (!talk_form_spills(sz, hpw, maxw)) return hpw;
    if (!spilling) spilling = hpw;
  }
  return spilling;
}

extern "C" int ix_attention_talk_mfma(const void* q, const void* k_cache, const void* v_cache,
                                      const int32_t* block_table, const int32_t* tile_seq, const int32_t* tile_q0,
                                      const int32_t* tile_rows, const int32_t* positions, void* out, float* part_o,
                                      float* part_ml, const float* talk, const float* sink, const void* gate,
                                      int64_t gate_stride, int64_t tokens, int n_tiles, int n_splits, int heads,
                                      int kv_heads, int head_dim, int value_dim, int page_size, int max_blocks,
                                      float scale, int heads_per_wave, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && n_tiles >= 0 && max_blocks > 0, "sizes must be positive");
  IX_REQUIRE(n_splits >= 1 && n_splits <= 64, "between 1 and 64 slices of the keys");
  IX_REQUIRE(n_splits == 1 || (part_o && part_ml), "the slices' parts need a workspace");
  // heads_per_wave 0: the form that `ix_attention_talk_mfma_heads_per_wave` names; else the caller's choice
  const int hpw = heads_per_wave > 0 ? heads_per_wave
                                     : ix_attention_talk_mfma_heads_per_wave(heads, kv_heads, head_dim, value_dim, page_size);
  IX_REQUIRE(head_dim % 16 == 0 && value_dim % 16 == 0 && page_size % 16 == 0 && heads % kv_heads == 0 && heads <= 32,
             "heads and values in multiples of 16, pages in multiples of 16, at most 32 heads");
  IX_REQUIRE(hpw > 0 && heads % hpw == 0 && (heads / kv_heads) % hpw == 0 && heads / hpw <= 16,
             "a wavefront's heads must share a key/value head, in at most 16 wavefronts");
  IX_REQUIRE(hpw > 0, "sizes that the matrix-core kernel does not take (heads and values in multiples of 16 up to "
                      "256, pages in multiples of 16, at most 32 heads in at most 16 wavefronts)");
  if (tokens == 0 || n_tiles == 0) return 0;
  IX_REQUIRE(static_cast<int64_t>(n_tiles) * n_splits < (1ll << 31), "too many workgroups");
  TalkArgs a{(const __bf16*)q, (const __bf16*)k_cache, (const __bf16*)v_cache, block_table, tile_seq, tile_q0,
             tile_rows, positions, (__bf16*)out, part_o, part_ml, talk, sink, (const __bf16*)gate, gate_stride,
             n_tiles, n_splits, heads, kv_heads, head_dim, value_dim, page_size, max_blocks, scale, -1};
  for (int b = 4; b < 31; ++b)
    if (page_size == (1 << b)) a.page_shift = b;
  const size_t lds = (static_cast<size_t>(heads > 16 ? 1 : 2) * heads * 2 * 64 * 4 +
                      static_cast<size_t>(heads) * ((heads + 3) & ~3)) * sizeof(float);
  IX_REQUIRE(lds <= 128 * 1024, "the heads' products do not fit 128 KB of LDS");
  const int big = std::max(head_dim, value_dim);
  const int sz = big <= 32 ? 32 : (big <= 64 ? 64 : (big <= 128 ? 128 : 256));
#define TALK_FORM(SZ, HPW, MAXW)                                  \
  if (sz == SZ && hpw == HPW && maxw == MAXW) {                   \
    if (launch_talk<SZ, HPW, MAXW>(a, lds, stream)) return 1;     \
    launched = true;                                              \
  }
  const int waves = heads / hpw, maxw = waves <= 4 ? 4 : (waves <= 8 ? 8 : 16);
  bool launched = false;
  TALK_FORM(32, 1, 4) TALK_FORM(32, 1, 8) TALK_FORM(32, 1, 16) TALK_FORM(32, 2, 4) TALK_FORM(32, 2, 8) TALK_FORM(32, 2, 16)
  TALK_FORM(32, 4, 4) TALK_FORM(32, 4, 8)
  TALK_FORM(64, 1, 4) TALK_FORM(64, 1, 8) TALK_FORM(64, 1, 16) TALK_FORM(64, 2, 4) TALK_FORM(64, 2, 8) TALK_FORM(64, 2, 16)
  TALK_FORM(64, 4, 4) TALK_FORM(64, 4, 8)
  TALK_FORM(128, 1, 4) TALK_FORM(128, 1, 8) TALK_FORM(128, 1, 16) TALK_FORM(128, 2, 4) TALK_FORM(128, 2, 8)
  TALK_FORM(128, 4, 4) TALK_FORM(128, 4, 8)
  TALK_FORM(256, 1, 4) TALK_FORM(256, 1, 8)
#undef TALK_FORM
  IX_REQUIRE(launched, "no form of the kernel for these sizes");
  if (ix_check_launch("ix_attention_talk_mfma")) return 1;
  if (n_splits > 1) {
    const int64_t pairs = tokens * heads;
    hipLaunchKernelGGL(talk_combine_kernel, dim3(static_cast<unsigned>((pairs + 3) / 4)), dim3(256), 0, stream, part_o,
                       part_ml, (__bf16*)out, (const __bf16*)gate, gate_stride, pairs, heads, n_splits, value_dim);
    return ix_check_launch("ix_attention_talk_mfma (combine)");
  }
  return 0;
}
