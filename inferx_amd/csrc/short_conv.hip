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

// q_channels, k_channels: multiples of head_dim; v_channels: a multiple of value_dim.  `slots` null: k and v go to
// plain rows.  `dtype`: the type of in, out_q, out_k, out_v (and of the cache).
extern "C" int ix_short_conv(const void* in, int dtype, int64_t in_stride, const void* bias, int bias_dtype,
                             const void* w, int w_dtype, int taps, float* state, int64_t state_stride,
                             const int32_t* seq_of_token, const int32_t* q_start, const int32_t* state_slots,
                             const float* cos_sin, int rot_dims, int silu, const int32_t* slots, int page_size,
                             void* out_q, void* out_k, void* out_v, int64_t tokens, int q_channels, int k_channels,
                             int v_channels, int head_dim, int value_dim, hipStream_t stream) {
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
  if (dtype == IX_F32) hipLaunchKernelGGL(short_conv_kernel<float>, grid, block, 0, stream, a);
  else hipLaunchKernelGGL(short_conv_kernel<bf16_t>, grid, block, 0, stream, a);
  return ix_check_launch("ix_short_conv");
}
