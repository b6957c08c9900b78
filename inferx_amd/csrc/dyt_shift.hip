// Dynamic Tanh norm fused with the residual add, a per-channel gain on the added branch and the token shift of
// the normalised rows; the token shift alone; the per-channel gain alone.
//
//   v[t]   = h_in[t] + gain * delta[t]                    (the residual sum, float32)
//   n[t]   = tanh(alpha * v[t]) * w + b                   (no mean, no variance)
//   out[t] = n[t] + (n[t-1] - n[t]) * mix                 (token shift; n[-1] = 0 at a sequence's first token)
//
// n[t-1] of a request's first row in a step is what the request's state slot holds from the step before; the
// thread that reads it also forms n of the request's last row of this step and leaves it there, so the slot is
// read before it is written by one and the same thread.  Inside a step n[t-1] is formed again from row t-1 of
// h_in and delta, which costs one more tanh per element and no trip through memory; that is why a shifted call
// does not update the stream in place: it writes v to h_out, which must be another buffer than h_in.
// Everything is float32; only `delta` and `out` have the run's type.
#include "common.h"

struct DytArgs {
  const float* h_in;
  float* h_out;        // may equal h_in when nothing is shifted; null: the stream is not written
  const void* delta;   // null: nothing to add
  const float* gain;   // null: delta is added as it is
  const float* w;
  const float* b;      // null: no bias
  float alpha;
  const int32_t* rows;  // null: row r of out is row r of the stream
  // token shift (mix null: none)
  const float* mix;
  float* state;         // [slots, width]
  const int32_t* seq_of_token;
  const int32_t* q_start;
  const int32_t* state_slots;
  const int32_t* positions;
};

template <typename TD>
__device__ __forceinline__ float dyt_sum(const DytArgs& a, int64_t row, int64_t width, int64_t i, float gain) {
  float v = a.h_in[row * width + i];
  if (a.delta) v += gain * ix_load(static_cast<const TD*>(a.delta) + row * width + i);
  return v;
}

template <typename TD, typename TO>
__global__ void __launch_bounds__(256)
add_dyt_kernel(DytArgs a, TO* __restrict__ out, int64_t width) {
  const int64_t r = blockIdx.x;
  const int64_t row = a.rows ? a.rows[r] : r;
  int64_t prev_row = -1, last_row = -1, slot = 0;
  bool first = false, from_state = false;
  if (a.mix) {
    const int64_t s = a.seq_of_token[row];
    first = row == a.q_start[s];
    if (first) {
      from_state = a.positions[row] > 0;
      last_row = a.q_start[s + 1] - 1;
      slot = a.state_slots[s];
    } else {
      prev_row = row - 1;
    }
  }
  for (int64_t i = static_cast<int64_t>(blockIdx.y) * blockDim.x + threadIdx.x; i < width;
       i += static_cast<int64_t>(gridDim.y) * blockDim.x) {
    const float gain = a.gain ? a.gain[i] : 1.0f;
    const float w = a.w[i], b = a.b ? a.b[i] : 0.f;
    const float v = dyt_sum<TD>(a, row, width, i, gain);
    if (a.h_out && !a.rows) a.h_out[row * width + i] = v;
    float n = tanhf(a.alpha * v) * w + b;
    if (a.mix) {
      float before;
      if (first) {
        before = from_state ? a.state[slot * width + i] : 0.f;
        const float n_last =
            last_row == row ? n : tanhf(a.alpha * dyt_sum<TD>(a, last_row, width, i, gain)) * w + b;
        a.state[slot * width + i] = n_last;
      } else {
        before = tanhf(a.alpha * dyt_sum<TD>(a, prev_row, width, i, gain)) * w + b;
      }
      n += (before - n) * a.mix[i];
    }
    ix_store(out + r * width + i, n);
  }
}

// bfloat16 delta and result with a width that is a multiple of 4: four columns per thread, 16-byte accesses to
// the stream, 8-byte ones to delta and result
struct Four {
  float v[4];
};
__device__ __forceinline__ Four dyt_sum4(const DytArgs& a, int64_t row, int64_t width, int64_t c, const Four& gain) {
  const float4 h = *reinterpret_cast<const float4*>(a.h_in + row * width + c);
  Four out{{h.x, h.y, h.z, h.w}};
  if (a.delta) {
    const uint2 d = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(a.delta) + row * width + c);
    out.v[0] += gain.v[0] * __uint_as_float(d.x << 16);
    out.v[1] += gain.v[1] * __uint_as_float(d.x & 0xffff0000u);
    out.v[2] += gain.v[2] * __uint_as_float(d.y << 16);
    out.v[3] += gain.v[3] * __uint_as_float(d.y & 0xffff0000u);
  }
  return out;
}

__global__ void __launch_bounds__(256)
add_dyt_vec4_kernel(DytArgs a, uint16_t* __restrict__ out, int64_t width) {
  const int64_t r = blockIdx.x;
  const int64_t row = a.rows ? a.rows[r] : r;
  int64_t prev_row = -1, last_row = -1, slot = 0;
  bool first = false, from_state = false;
  if (a.mix) {
    const int64_t s = a.seq_of_token[row];
    first = row == a.q_start[s];
    if (first) {
      from_state = a.positions[row] > 0;
      last_row = a.q_start[s + 1] - 1;
      slot = a.state_slots[s];
    } else {
      prev_row = row - 1;
    }
  }
  for (int64_t c = 4 * (static_cast<int64_t>(blockIdx.y) * blockDim.x + threadIdx.x); c < width;
       c += 4 * static_cast<int64_t>(gridDim.y) * blockDim.x) {
    Four gain{{1.f, 1.f, 1.f, 1.f}}, b{{0.f, 0.f, 0.f, 0.f}}, w, n;
    const float4 w4 = *reinterpret_cast<const float4*>(a.w + c);
    w = Four{{w4.x, w4.y, w4.z, w4.w}};
    if (a.gain) {
      const float4 g4 = *reinterpret_cast<const float4*>(a.gain + c);
      gain = Four{{g4.x, g4.y, g4.z, g4.w}};
    }
    if (a.b) {
      const float4 b4 = *reinterpret_cast<const float4*>(a.b + c);
      b = Four{{b4.x, b4.y, b4.z, b4.w}};
    }
    const Four v = dyt_sum4(a, row, width, c, gain);
    if (a.h_out && !a.rows) *reinterpret_cast<float4*>(a.h_out + row * width + c) = make_float4(v.v[0], v.v[1], v.v[2], v.v[3]);
#pragma unroll
    for (int i = 0; i < 4; ++i) n.v[i] = tanhf(a.alpha * v.v[i]) * w.v[i] + b.v[i];
    if (a.mix) {
      Four before{{0.f, 0.f, 0.f, 0.f}};
      if (first) {
        if (from_state) {
          const float4 s4 = *reinterpret_cast<const float4*>(a.state + slot * width + c);
          before = Four{{s4.x, s4.y, s4.z, s4.w}};
        }
        Four n_last = n;
        if (last_row != row) {
          const Four vl = dyt_sum4(a, last_row, width, c, gain);
#pragma unroll
          for (int i = 0; i < 4; ++i) n_last.v[i] = tanhf(a.alpha * vl.v[i]) * w.v[i] + b.v[i];
        }
        *reinterpret_cast<float4*>(a.state + slot * width + c) = make_float4(n_last.v[0], n_last.v[1], n_last.v[2], n_last.v[3]);
      } else {
        const Four vp = dyt_sum4(a, prev_row, width, c, gain);
#pragma unroll
        for (int i = 0; i < 4; ++i) before.v[i] = tanhf(a.alpha * vp.v[i]) * w.v[i] + b.v[i];
      }
      const float4 m4 = *reinterpret_cast<const float4*>(a.mix + c);
      const float m[4] = {m4.x, m4.y, m4.z, m4.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) n.v[i] += (before.v[i] - n.v[i]) * m[i];
    }
    uint2 o;
    o.x = ix_f32_to_bf16(n.v[0]) | static_cast<uint32_t>(ix_f32_to_bf16(n.v[1])) << 16;
    o.y = ix_f32_to_bf16(n.v[2]) | static_cast<uint32_t>(ix_f32_to_bf16(n.v[3])) << 16;
    *reinterpret_cast<uint2*>(out + r * width + c) = o;
  }
}

extern "C" int ix_add_dyt(const float* h_in, float* h_out, const void* delta, int delta_dtype, const float* gain,
                          const float* w, const float* b, float alpha, void* out, int out_dtype, const int32_t* rows,
                          int64_t n_out_rows, int64_t width, const float* mix, float* state,
                          const int32_t* seq_of_token, const int32_t* q_start, const int32_t* state_slots,
                          const int32_t* positions, hipStream_t stream) {
  IX_REQUIRE(width > 0 && n_out_rows >= 0, "sizes must be positive");
  IX_REQUIRE(h_in && w && out, "stream, weight and result are needed");
  IX_REQUIRE(!mix || (state && seq_of_token && q_start && state_slots && positions && !rows),
             "a shifted call needs the state and the step's index arrays, and takes all rows");
  IX_REQUIRE(!mix || h_out != h_in, "a shifted call reads the rows before it: the stream cannot be updated in place");
  if (n_out_rows == 0) return 0;
  DytArgs a{h_in, h_out, delta, gain, w, b, alpha, rows, mix, state, seq_of_token, q_start, state_slots, positions};
  const int threads = 256;
  const int chunks = static_cast<int>(std::min<int64_t>((width + threads - 1) / threads, 64));
  dim3 grid(n_out_rows, chunks), block(threads);
#define LAUNCH(TD, TO) hipLaunchKernelGGL((add_dyt_kernel<TD, TO>), grid, block, 0, stream, a, (TO*)out, width)
  const int dd = delta ? delta_dtype : IX_F32;
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (out_dtype == IX_BF16 && (!delta || delta_dtype == IX_BF16) && width % 4 == 0 && aligned(h_in) && aligned(h_out) &&
      aligned(delta) && aligned(out) && aligned(gain) && aligned(w) && aligned(b) && aligned(mix) && aligned(state)) {
    const int chunks4 = static_cast<int>(std::min<int64_t>((width / 4 + threads - 1) / threads, 64));
    hipLaunchKernelGGL(add_dyt_vec4_kernel, dim3(n_out_rows, chunks4), block, 0, stream, a, (uint16_t*)out, width);
    return ix_check_launch("ix_add_dyt");
  }
  if (dd == IX_F32 && out_dtype == IX_F32) LAUNCH(float, float);
  else if (dd == IX_F32 && out_dtype == IX_BF16) LAUNCH(float, bf16_t);
  else if (dd == IX_BF16 && out_dtype == IX_F32) LAUNCH(bf16_t, float);
  else if (dd == IX_BF16 && out_dtype == IX_BF16) LAUNCH(bf16_t, bf16_t);
  else IX_REQUIRE(false, "dtypes must be float32 or bfloat16");
#undef LAUNCH
  return ix_check_launch("ix_add_dyt");
}

// ---------------------------------------------------------------------------
// The token shift alone, for rows that some other norm made: out[t] = x[t] + (x[t-1] - x[t]) * mix, x[t-1] of a
// request's first row from its state slot (zero at position 0), the slot left holding x of its last row.
// `out` must not be `x`.
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(const T* __restrict__ x, T* __restrict__ out, const float* __restrict__ mix,
                   float* __restrict__ state, const int32_t* __restrict__ seq_of_token,
                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                   const int32_t* __restrict__ positions, int64_t width) {
  const int64_t row = blockIdx.x;
  const int64_t s = seq_of_token[row];
  const bool first = row == q_start[s];
  const bool from_state = first && positions[row] > 0;
  const int64_t last_row = q_start[s + 1] - 1;
  const int64_t slot = state_slots[s];
  for (int64_t i = static_cast<int64_t>(blockIdx.y) * blockDim.x + threadIdx.x; i < width;
       i += static_cast<int64_t>(gridDim.y) * blockDim.x) {
    const float n = ix_load(x + row * width + i);
    float before;
    if (first) {
      before = from_state ? state[slot * width + i] : 0.f;
      state[slot * width + i] = ix_load(x + last_row * width + i);
    } else {
      before = ix_load(x + (row - 1) * width + i);
    }
    ix_store(out + row * width + i, n + (before - n) * mix[i]);
  }
}

extern "C" int ix_token_shift(const void* x, void* out, int dtype, const float* mix, float* state,
                              const int32_t* seq_of_token, const int32_t* q_start, const int32_t* state_slots,
                              const int32_t* positions, int64_t tokens, int64_t width, hipStream_t stream) {
  IX_REQUIRE(width > 0 && tokens >= 0, "sizes must be positive");
  IX_REQUIRE(x && out && x != out && mix && state && seq_of_token && q_start && state_slots && positions,
             "operands are missing, or the result would overwrite its input");
  if (tokens == 0) return 0;
  const int chunks = static_cast<int>(std::min<int64_t>((width + 255) / 256, 64));
  dim3 grid(tokens, chunks), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(token_shift_kernel<float>, grid, block, 0, stream, (const float*)x, (float*)out, mix, state,
                       seq_of_token, q_start, state_slots, positions, width);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(token_shift_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x, (bf16_t*)out, mix, state,
                       seq_of_token, q_start, state_slots, positions, width);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_token_shift");
}

// ---------------------------------------------------------------------------
// out[t, i] = x[t, i] * gain[i]   (a branch's per-channel gain, for a consumer that cannot apply it on its way)
template <typename T>
__global__ void __launch_bounds__(256)
scale_columns_kernel(const T* __restrict__ x, T* __restrict__ out, const float* __restrict__ gain, int64_t n,
                     int64_t width) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    ix_store(out + i, ix_load(x + i) * gain[i % width]);
}

extern "C" int ix_scale_columns(const void* x, void* out, int dtype, const float* gain, int64_t tokens, int64_t width,
                                hipStream_t stream) {
  IX_REQUIRE(width > 0 && tokens >= 0, "sizes must be positive");
  if (tokens == 0) return 0;
  const int64_t n = tokens * width;
  const int blocks = static_cast<int>(std::min<int64_t>((n + 255) / 256, 65535));
  if (dtype == IX_F32)
    hipLaunchKernelGGL(scale_columns_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, (float*)out,
                       gain, n, width);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(scale_columns_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)x,
                       (bf16_t*)out, gain, n, width);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_scale_columns");
}
