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
