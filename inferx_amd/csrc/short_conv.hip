// A short causal convolution over time, per channel, on the rows that a step brings, with what it needs of
// earlier steps kept per request:
//
//   y[t, c] = sum_j w[c, j] * u[t - taps + 1 + j, c],   u = projection (+ bias),   zeros before a sequence's start
//
// The rows of a step are the portions of several requests side by side (`q_start`); the taps - 1 inputs before a
// portion come from the request's state block, float32 [taps - 1, channels], oldest first, which the kernel
// brings up to date for the next step.
//
// The channels are three runs side by side, q | k | v: q and k in heads of `head_dim`, v in heads of `value_dim`.
// What follows the convolution is fused:
//   silu          y <- y * sigmoid(y)
//   rotation      the first `rot_dims` elements of every q and k head, element i paired with i + rot_dims / 2, by the
//                 (cos, sin) table of the step's tokens; computed in float32
//   destination   q always to `out_q` [T, q channels]; k and v either to `out_k`, `out_v` (plain rows) or into the
//                 paged cache at the token's slot: keys [pages, k heads, page, head_dim], values transposed within a
//                 page [pages, v heads, value_dim, page]
//
// A thread owns a unit: a rotated pair of channels, or one channel.  Whoever reads or writes the state of a
// channel is the ONE thread that has the request's last row of this step for that unit: it also forms the
// portion's first taps - 1 rows (the only ones that read the state), and then writes the new state, so the
// state is read before it is overwritten without any ordering between threads.
#include "common.h"

#define CONV_THREADS 256

struct ConvArgs {
  const void* in;          // [T, in_stride] of the run's type
  const void* bias;        // [channels] or null
  const void* w;           // [channels, taps]
  float* state;            // slot s at state + s * state_stride: [taps - 1, channels]
  const int32_t* seq_of_token;
  const int32_t* q_start;
  const int32_t* state_slots;
  const float* cos_sin;    // [T, rot_dims / 2, 2] or null
  const int32_t* slots;    // [T] flat cache index page * page_size + offset, or null (plain rows)
  void* out_q;
  void* out_k;             // plain rows, or the key cache
  void* out_v;             // plain rows, or the value cache
  int64_t in_stride, state_stride;
  int bias_dtype, w_dtype;
  int taps, channels;
  int q_channels, k_channels, v_channels, head_dim, value_dim;
  int rot_dims, silu, page_size;
  int units_qk_head;       // units of one q or k head: head_dim - rot_dims / 2
  int units;               // all units of a token
};

template <typename T>
__device__ __forceinline__ float conv_input(const ConvArgs& a, const T* in, const float* st, int64_t row0, int x, int c) {
  // input number x of the portion (negative: before it, from the state)
  if (x >= 0) {
    float u = ix_load(in + (row0 + x) * a.in_stride + c);
    if (a.bias) u += ix_load_rt(a.bias, a.bias_dtype, c);
    return u;
  }
  return st[static_cast<int64_t>(a.taps - 1 + x) * a.channels + c];
}

template <typename T>
__device__ __forceinline__ float conv_at(const ConvArgs& a, const T* in, const float* st, int64_t row0, int i, int c) {
  float y = 0.f;
  for (int j = 0; j < a.taps; ++j)
    y += ix_load_rt(a.w, a.w_dtype, static_cast<int64_t>(c) * a.taps + j) * conv_input(a, in, st, row0, i - a.taps + 1 + j, c);
  if (a.silu) y = y / (1.0f + expf(-y));
  return y;
}

// where channel c of row `row` goes
template <typename T>
__device__ __forceinline__ void conv_store(const ConvArgs& a, int64_t row, int c, float y) {
  if (c < a.q_channels) {
    ix_store(static_cast<T*>(a.out_q) + row * a.q_channels + c, y);
    return;
  }
  c -= a.q_channels;
  if (c < a.k_channels) {
    if (a.slots) {
      const int64_t slot = a.slots[row];
      const int64_t page = slot / a.page_size, off = slot % a.page_size;
      const int head = c / a.head_dim, e = c % a.head_dim;
      const int heads = a.k_channels / a.head_dim;
      ix_store(static_cast<T*>(a.out_k) + ((page * heads + head) * a.page_size + off) * a.head_dim + e, y);
    } else {
      ix_store(static_cast<T*>(a.out_k) + row * a.k_channels + c, y);
    }
    return;
  }
  c -= a.k_channels;
  if (a.slots) {
    const int64_t slot = a.slots[row];
    const int64_t page = slot / a.page_size, off = slot % a.page_size;
    const int head = c / a.value_dim, e = c % a.value_dim;
    const int heads = a.v_channels / a.value_dim;
    ix_store(static_cast<T*>(a.out_v) + ((page * heads + head) * a.value_dim + e) * a.page_size + off, y);
  } else {
    ix_store(static_cast<T*>(a.out_v) + row * a.v_channels + c, y);
  }
}

template <typename T>
__global__ void __launch_bounds__(CONV_THREADS) short_conv_kernel(ConvArgs a) {
  const int unit = blockIdx.y * CONV_THREADS + threadIdx.x;
  if (unit >= a.units) return;
  const int64_t t = blockIdx.x;
  const int seq = a.seq_of_token[t];
  const int64_t row0 = a.q_start[seq];
  const int n = a.q_start[seq + 1] - static_cast<int>(row0);
  const int i = static_cast<int>(t - row0);
  const bool last = i == n - 1;
  if (i < a.taps - 1 && !last) return;  // formed by the thread that has the portion's last row

  // the unit's channels: c0, and for a rotated pair c1 = c0 + rot_dims / 2
  const int qk_units = (a.q_channels + a.k_channels) / a.head_dim * a.units_qk_head;
  int c0, c1 = -1, pair = -1;
  if (unit < qk_units) {
    const int head = unit / a.units_qk_head, u = unit % a.units_qk_head;
    const int half = a.rot_dims / 2;
    if (u < half) {
      c0 = head * a.head_dim + u;
      c1 = c0 + half;
      pair = u;
    } else {
      c0 = head * a.head_dim + u + half;
    }
  } else {
    c0 = a.q_channels + a.k_channels + (unit - qk_units);
  }

  const T* in = static_cast<const T*>(a.in);
  float* st = a.state + static_cast<int64_t>(a.state_slots[seq]) * a.state_stride;
  const int first = last ? 0 : i;                       // the last row's thread starts with the portion's first rows
  const int head_rows = min(a.taps - 1, n - 1);         // rows 0 .. head_rows - 1 read the state
  for (int step = first;; ++step) {
    int ii = step;
    if (last) {
      if (step > head_rows) break;
      ii = step < head_rows ? step : n - 1;
    } else if (step > i) {
      break;
    }
    const int64_t row = row0 + ii;
    float y0 = conv_at(a, in, st, row0, ii, c0);
    if (c1 >= 0) {
      float y1 = conv_at(a, in, st, row0, ii, c1);
      if (a.cos_sin) {
        const float* cs = a.cos_sin + (row * (a.rot_dims / 2) + pair) * 2;
        const float c = cs[0], s = cs[1];
        const float r0 = y0 * c - y1 * s, r1 = y1 * c + y0 * s;
        y0 = r0;
        y1 = r1;
      }
      conv_store<T>(a, row, c1, y1);
    }
    conv_store<T>(a, row, c0, y0);
  }
  if (!last) return;
  // the state for the next step: the last taps - 1 inputs of what the request has seen so far
  for (int which = 0; which < 2; ++which) {
    const int c = which ? c1 : c0;
    if (c < 0) continue;
    for (int r = 0; r < a.taps - 1; ++r)  // ascending: an old entry is read (further on) before it is overwritten
      st[static_cast<int64_t>(r) * a.channels + c] = conv_input(a, in, st, row0, n - (a.taps - 1) + r, c);
  }
}

// The same for bfloat16 rows where everything comes in eights: a thread owns eight consecutive channels (and, if they
// are rotated, the eight they are paired with), reads its inputs in 16-byte pieces and the taps and the bias from
// float32 copies laid out for that (`wt` [taps, channels], `bias_f` [channels]).  Same sums in the same order.
typedef unsigned int conv_u32x4 __attribute__((ext_vector_type(4)));
typedef float conv_f32x4 __attribute__((ext_vector_type(4)));

struct Conv8 {
  float x[8];
};

__device__ __forceinline__ Conv8 conv_input8(const ConvArgs& a, const float* bias_f, const uint16_t* in, const float* st,
                                             int64_t row0, int x, int c) {
  Conv8 r;
  if (x >= 0) {
    const conv_u32x4 p = *reinterpret_cast<const conv_u32x4*>(in + (row0 + x) * a.in_stride + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r.x[2 * e] = __uint_as_float(p[e] << 16);
      r.x[2 * e + 1] = __uint_as_float(p[e] & 0xffff0000u);
    }
    if (bias_f) {
      const conv_f32x4 b0 = *reinterpret_cast<const conv_f32x4*>(bias_f + c), b1 = *reinterpret_cast<const conv_f32x4*>(bias_f + c + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        r.x[e] += b0[e];
        r.x[4 + e] += b1[e];
      }
    }
  } else {
    const float* sr = st + static_cast<int64_t>(a.taps - 1 + x) * a.channels + c;
    const conv_f32x4 s0 = *reinterpret_cast<const conv_f32x4*>(sr), s1 = *reinterpret_cast<const conv_f32x4*>(sr + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r.x[e] = s0[e];
      r.x[4 + e] = s1[e];
    }
  }
  return r;
}

__device__ __forceinline__ Conv8 conv_at8(const ConvArgs& a, const float* wt, const float* bias_f, const uint16_t* in,
                                          const float* st, int64_t row0, int i, int c) {
  Conv8 y;
#pragma unroll
  for (int e = 0; e < 8; ++e) y.x[e] = 0.f;
  if (a.taps <= 4) {
    // up to four taps: every input and every tap is asked for before the first is used (one trip to memory
    // instead of one per tap, which is what a step of few tokens waits for); the same sums in the same order
    Conv8 u[4];
    conv_f32x4 w0[4], w1[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int jj = min(j, a.taps - 1);
      u[j] = conv_input8(a, bias_f, in, st, row0, i - a.taps + 1 + jj, c);
      const float* wr = wt + static_cast<int64_t>(jj) * a.channels + c;
      w0[j] = *reinterpret_cast<const conv_f32x4*>(wr);
      w1[j] = *reinterpret_cast<const conv_f32x4*>(wr + 4);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (j < a.taps) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          y.x[e] += w0[j][e] * u[j].x[e];
          y.x[4 + e] += w1[j][e] * u[j].x[4 + e];
        }
      }
    }
  } else {
    for (int j = 0; j < a.taps; ++j) {
      const Conv8 u = conv_input8(a, bias_f, in, st, row0, i - a.taps + 1 + j, c);
      const float* wr = wt + static_cast<int64_t>(j) * a.channels + c;
      const conv_f32x4 w0 = *reinterpret_cast<const conv_f32x4*>(wr), w1 = *reinterpret_cast<const conv_f32x4*>(wr + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        y.x[e] += w0[e] * u.x[e];
        y.x[4 + e] += w1[e] * u.x[4 + e];
      }
    }
  }
  if (a.silu) {
#pragma unroll
    for (int e = 0; e < 8; ++e) y.x[e] = y.x[e] / (1.0f + expf(-y.x[e]));
  }
  return y;
}

__device__ __forceinline__ conv_u32x4 conv_pack8(const Conv8& y) {
  conv_u32x4 p;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    p[e] = ix_f32_to_bf16(y.x[2 * e]) | static_cast<uint32_t>(ix_f32_to_bf16(y.x[2 * e + 1])) << 16;
  return p;
}

// where channels c .. c + 7 of row `row` go (they lie within one head)
__device__ __forceinline__ void conv_store8(const ConvArgs& a, int64_t row, int c, const Conv8& y) {
  if (c < a.q_channels) {
    *reinterpret_cast<conv_u32x4*>(static_cast<uint16_t*>(a.out_q) + row * a.q_channels + c) = conv_pack8(y);
    return;
  }
  c -= a.q_channels;
  if (c < a.k_channels) {
    uint16_t* dst;
    if (a.slots) {
      const int64_t slot = a.slots[row];
      const int64_t page = slot / a.page_size, off = slot % a.page_size;
      const int head = c / a.head_dim, e = c % a.head_dim;
      dst = static_cast<uint16_t*>(a.out_k) + ((page * (a.k_channels / a.head_dim) + head) * a.page_size + off) * a.head_dim + e;
    } else {
      dst = static_cast<uint16_t*>(a.out_k) + row * a.k_channels + c;
    }
    *reinterpret_cast<conv_u32x4*>(dst) = conv_pack8(y);
    return;
  }
  c -= a.k_channels;
  if (a.slots) {
    const int64_t slot = a.slots[row];
    const int64_t page = slot / a.page_size, off = slot % a.page_size;
    const int head = c / a.value_dim, e0 = c % a.value_dim;
    uint16_t* dst = static_cast<uint16_t*>(a.out_v) + ((page * (a.v_channels / a.value_dim) + head) * a.value_dim + e0) * a.page_size + off;
#pragma unroll
    for (int e = 0; e < 8; ++e) dst[static_cast<int64_t>(e) * a.page_size] = ix_f32_to_bf16(y.x[e]);
  } else {
    *reinterpret_cast<conv_u32x4*>(static_cast<uint16_t*>(a.out_v) + row * a.v_channels + c) = conv_pack8(y);
  }
}

__global__ void __launch_bounds__(CONV_THREADS) short_conv_vec8_kernel(ConvArgs a, const float* __restrict__ wt,
                                                                       const float* __restrict__ bias_f, int vunits) {
  const int unit = blockIdx.y * CONV_THREADS + threadIdx.x;
  if (unit >= vunits) return;
  const int64_t t = blockIdx.x;
  const int seq = a.seq_of_token[t];
  const int64_t row0 = a.q_start[seq];
  const int n = a.q_start[seq + 1] - static_cast<int>(row0);
  const int i = static_cast<int>(t - row0);
  const bool last = i == n - 1;
  if (i < a.taps - 1 && !last) return;  // formed by the thread that has the portion's last row

  // the unit's channels: c0 .. c0 + 7, and for rotated ones their partners c1 = c0 + rot_dims / 2 ..
  const int half_blocks = a.rot_dims / 16, per_head = a.head_dim / 8 - half_blocks;
  const int qk_units = (a.q_channels + a.k_channels) / a.head_dim * per_head;
  int c0, c1 = -1, pair0 = 0;
  if (unit < qk_units) {
    const int head = unit / per_head, u = unit % per_head;
    if (u < half_blocks) {
      c0 = head * a.head_dim + 8 * u;
      c1 = c0 + a.rot_dims / 2;
      pair0 = 8 * u;
    } else {
      c0 = head * a.head_dim + 8 * (u + half_blocks);
    }
  } else {
    c0 = a.q_channels + a.k_channels + 8 * (unit - qk_units);
  }

  const uint16_t* in = static_cast<const uint16_t*>(a.in);
  float* st = a.state + static_cast<int64_t>(a.state_slots[seq]) * a.state_stride;
  const int first = last ? 0 : i;
  const int head_rows = min(a.taps - 1, n - 1);
  for (int step = first;; ++step) {
    int ii = step;
    if (last) {
      if (step > head_rows) break;
      ii = step < head_rows ? step : n - 1;
    } else if (step > i) {
      break;
    }
    const int64_t row = row0 + ii;
    Conv8 y0 = conv_at8(a, wt, bias_f, in, st, row0, ii, c0);
    if (c1 >= 0) {
      Conv8 y1 = conv_at8(a, wt, bias_f, in, st, row0, ii, c1);
      if (a.cos_sin) {
        const float* cs = a.cos_sin + (row * (a.rot_dims / 2) + pair0) * 2;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float c = cs[2 * e], s = cs[2 * e + 1];
          const float r0 = y0.x[e] * c - y1.x[e] * s, r1 = y1.x[e] * c + y0.x[e] * s;
          y0.x[e] = r0;
          y1.x[e] = r1;
        }
      }
      conv_store8(a, row, c1, y1);
    }
    conv_store8(a, row, c0, y0);
  }
  if (!last) return;
  for (int which = 0; which < 2; ++which) {
    const int c = which ? c1 : c0;
    if (c < 0) continue;
    for (int r = 0; r < a.taps - 1; ++r) {  // ascending: an old entry is read (further on) before it is overwritten
      const Conv8 u = conv_input8(a, bias_f, in, st, row0, n - (a.taps - 1) + r, c);
      float* dst = st + static_cast<int64_t>(r) * a.channels + c;
      *reinterpret_cast<conv_f32x4*>(dst) = conv_f32x4{u.x[0], u.x[1], u.x[2], u.x[3]};
      *reinterpret_cast<conv_f32x4*>(dst + 4) = conv_f32x4{u.x[4], u.x[5], u.x[6], u.x[7]};
    }
  }
}

// q_channels, k_channels: multiples of head_dim; v_channels: a multiple of value_dim.  `slots` null: k and v go to
// plain rows.  `dtype`: the type of in, out_q, out_k, out_v (and of the cache).  `wt` float32 [taps, channels] and
// `bias_f` float32 [channels]: copies of `w` and `bias` for the 16-byte form, or null.
extern "C" int ix_short_conv(const void* in, int dtype, int64_t in_stride, const void* bias, int bias_dtype,
                             const void* w, int w_dtype, int taps, float* state, int64_t state_stride,
                             const int32_t* seq_of_token, const int32_t* q_start, const int32_t* state_slots,
                             const float* cos_sin, int rot_dims, int silu, const int32_t* slots, int page_size,
                             void* out_q, void* out_k, void* out_v, int64_t tokens, int q_channels, int k_channels,
                             int v_channels, int head_dim, int value_dim, const float* wt, const float* bias_f,
                             hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && taps >= 1 && taps <= 64, "between 1 and 64 taps");
  IX_REQUIRE(head_dim > 0 && value_dim > 0 && q_channels >= 0 && k_channels >= 0 && v_channels >= 0,
             "sizes must be positive");
  IX_REQUIRE(q_channels % head_dim == 0 && k_channels % head_dim == 0 && v_channels % value_dim == 0,
             "channels must be whole heads");
  IX_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= head_dim, "an even number of rotated elements within a head");
  IX_REQUIRE(cos_sin != nullptr || rot_dims == 0, "a rotation needs its table");
  IX_REQUIRE(slots == nullptr || page_size > 0, "page_size must be positive");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  const int channels = q_channels + k_channels + v_channels;
  IX_REQUIRE(in_stride >= channels && state_stride >= static_cast<int64_t>(taps - 1) * channels, "strides too small");
  if (tokens == 0 || channels == 0) return 0;
  ConvArgs a;
  a.in = in; a.bias = bias; a.w = w; a.state = state; a.seq_of_token = seq_of_token; a.q_start = q_start;
  a.state_slots = state_slots; a.cos_sin = cos_sin; a.slots = slots; a.out_q = out_q; a.out_k = out_k; a.out_v = out_v;
  a.in_stride = in_stride; a.state_stride = state_stride; a.bias_dtype = bias_dtype; a.w_dtype = w_dtype;
  a.taps = taps; a.channels = channels; a.q_channels = q_channels; a.k_channels = k_channels; a.v_channels = v_channels;
  a.head_dim = head_dim; a.value_dim = value_dim; a.rot_dims = rot_dims; a.silu = silu; a.page_size = page_size;
  a.units_qk_head = head_dim - rot_dims / 2;
  a.units = (q_channels + k_channels) / head_dim * a.units_qk_head + v_channels;
  IX_REQUIRE(tokens < (1ll << 31) && a.units <= 65535 * CONV_THREADS, "too many tokens or channels for one launch");
  dim3 grid(static_cast<unsigned>(tokens), (a.units + CONV_THREADS - 1) / CONV_THREADS), block(CONV_THREADS);
  // everything in eights and 16-byte aligned, with the float32 copies of taps and bias: the 16-byte form
  const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool plain_rows_ok = slots != nullptr || (aligned(out_k) && aligned(out_v));
  if (dtype == IX_BF16 && wt != nullptr && (bias == nullptr || bias_f != nullptr) && head_dim % 8 == 0 &&
      value_dim % 8 == 0 && rot_dims % 16 == 0 && in_stride % 8 == 0 && state_stride % 4 == 0 && aligned(in) &&
      aligned(state) && aligned(wt) && aligned(bias_f) && aligned(out_q) && aligned(out_k) && plain_rows_ok &&
      (slots == nullptr || aligned(out_k))) {
    const int vunits = (q_channels + k_channels) / head_dim * (head_dim / 8 - rot_dims / 16) + v_channels / 8;
    dim3 vgrid(static_cast<unsigned>(tokens), (vunits + CONV_THREADS - 1) / CONV_THREADS);
    hipLaunchKernelGGL(short_conv_vec8_kernel, vgrid, block, 0, stream, a, wt, bias ? bias_f : nullptr, vunits);
    return ix_check_launch("ix_short_conv");
  }
  if (dtype == IX_F32) hipLaunchKernelGGL(short_conv_kernel<float>, grid, block, 0, stream, a);
  else hipLaunchKernelGGL(short_conv_kernel<bf16_t>, grid, block, 0, stream, a);
  return ix_check_launch("ix_short_conv");
}
