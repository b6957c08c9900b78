// The gated delta rule: a linear recurrence with a matrix of state per head,
//
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q          S [dim, vdim] float32 per head
//
// token after token, so that the read-out sees the token's own write.  q and k arrive as the short convolution left
// them and are made unit vectors here (x / sqrt(sum x^2 + 1e-6), q also times dim^(-1/2)); the decay and the step
// size come from two small projections a, b (float32):  g = exp(-exp(A_log) softplus(a + dt_bias)),  beta =
// sigmoid(b).  Everything but the loads of q, k, v is float32.
//
// The columns of S are independent recurrences (column j only ever meets v[j]), so the work is spread over
// (request, head, block of 16 value columns): one wavefront each, four lanes per column that own every fourth row
// of it (RPL rows a lane, in registers).  A wavefront walks its request's rows of this step in order, with the
// next row's operands asked for before the present row is worked; the state is read from the request's slot at the
// start and written back at the end.  Query head h reads the q/k head h / (heads / kv_heads).
#include "common.h"

#define DELTA_COLS 16   // value columns per wavefront
#define DELTA_SPLIT 4   // lanes per column

template <typename T, int RPL>
__global__ void __launch_bounds__(64)
delta_rule_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t q_stride,
                  int64_t k_stride, int64_t v_stride, const float* __restrict__ ab, const float* __restrict__ a_log,
                  const float* __restrict__ dt_bias, float* __restrict__ state, int64_t state_stride,
                  const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                  float* __restrict__ out, int heads, int kv_heads, int dim, int vdim) {
  const int lane = threadIdx.x;
  const int col = blockIdx.x * DELTA_COLS + lane / DELTA_SPLIT, part = lane % DELTA_SPLIT;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int kv = head / (heads / kv_heads);
  const int64_t row0 = q_start[seq];
  const int n = q_start[seq + 1] - static_cast<int>(row0);
  if (n <= 0) return;
  const bool live = col < vdim;
  const int cj = live ? col : vdim - 1;  // lanes past the last column repeat it and store nothing

  float* sp = state + static_cast<int64_t>(state_slots[seq]) * state_stride + static_cast<int64_t>(head) * dim * vdim;
  float S[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) {
    const int i = r * DELTA_SPLIT + part;
    S[r] = i < dim ? sp[static_cast<int64_t>(i) * vdim + cj] : 0.f;
  }
  const float rate = expf(a_log[head]), bias = dt_bias[head];
  const float q_scale = 1.0f / sqrtf(static_cast<float>(dim));

  float kc[RPL], qc[RPL], vc, ac, bc;  // the present row's operands
  auto fetch = [&](int64_t row, float* kk, float* qq, float& vv, float& aa, float& bb) {
    const T* qr = q + row * q_stride + kv * dim;
    const T* kr = k + row * k_stride + kv * dim;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = r * DELTA_SPLIT + part;
      kk[r] = i < dim ? ix_load(kr + i) : 0.f;
      qq[r] = i < dim ? ix_load(qr + i) : 0.f;
    }
    vv = ix_load(v + row * v_stride + head * vdim + cj);
    aa = ab[row * 2 * heads + head];
    bb = ab[row * 2 * heads + heads + head];
  };
  fetch(row0, kc, qc, vc, ac, bc);
  for (int i = 0; i < n; ++i) {
    float kn[RPL], qn[RPL], vn, an, bn;
    fetch(row0 + min(i + 1, n - 1), kn, qn, vn, an, bn);  // the next row's, on their way while this one is worked
    float kk = 0.f, qq = 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      kk += kc[r] * kc[r];
      qq += qc[r] * qc[r];
    }
    kk += ix_dpp<IX_DPP_XOR1>(kk);
    kk += ix_dpp<IX_DPP_XOR2>(kk);
    qq += ix_dpp<IX_DPP_XOR1>(qq);
    qq += ix_dpp<IX_DPP_XOR2>(qq);
    const float k_inv = 1.0f / sqrtf(kk + 1e-6f), q_inv = q_scale / sqrtf(qq + 1e-6f);
    const float x = ac + bias;
    const float softplus = x > 20.f ? x : log1pf(expf(x));
    const float g = expf(-rate * softplus);
    const float beta = 1.0f / (1.0f + expf(-bc));
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      S[r] *= g;
      dot += S[r] * (kc[r] * k_inv);
    }
    dot += ix_dpp<IX_DPP_XOR1>(dot);
    dot += ix_dpp<IX_DPP_XOR2>(dot);
    const float u = beta * (vc - dot);
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      S[r] += (kc[r] * k_inv) * u;
      o += S[r] * (qc[r] * q_inv);
    }
    o += ix_dpp<IX_DPP_XOR1>(o);
    o += ix_dpp<IX_DPP_XOR2>(o);
    if (live && part == 0) out[((row0 + i) * heads + head) * vdim + col] = o;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      kc[r] = kn[r];
      qc[r] = qn[r];
    }
    vc = vn;
    ac = an;
    bc = bn;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = r * DELTA_SPLIT + part;
      if (i < dim) sp[static_cast<int64_t>(i) * vdim + col] = S[r];
    }
  }
}

// q, k [T, kv_heads * dim] and v [T, heads * vdim] of the run's type with their row strides; ab float32 [T, 2 heads]
// (a then b); a_log, dt_bias float32 [heads]; state: slot s at state + s * state_stride, [heads, dim, vdim];
// out float32 [T, heads, vdim].
extern "C" int ix_delta_rule(const void* q, const void* k, const void* v, int dtype, int64_t q_stride,
                             int64_t k_stride, int64_t v_stride, const float* ab, const float* a_log,
                             const float* dt_bias, float* state, int64_t state_stride, const int32_t* q_start,
                             const int32_t* state_slots, float* out, int64_t tokens, int requests, int heads,
                             int kv_heads, int dim, int vdim, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && requests >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(dim <= 256, "at most 256 numbers per query and key head");
  IX_REQUIRE(state_stride >= static_cast<int64_t>(heads) * dim * vdim, "state blocks too small");
  IX_REQUIRE(heads <= 65535 && requests <= 65535, "too many heads or requests for one launch");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  if (tokens == 0 || requests == 0) return 0;
  dim3 grid((vdim + DELTA_COLS - 1) / DELTA_COLS, heads, requests), block(64);
  const int rpl = (dim + DELTA_SPLIT - 1) / DELTA_SPLIT;
#define LAUNCH(TT, RPL)                                                                                             \
  hipLaunchKernelGGL((delta_rule_kernel<TT, RPL>), grid, block, 0, stream, (const TT*)q, (const TT*)k, (const TT*)v, \
                     q_stride, k_stride, v_stride, ab, a_log, dt_bias, state, state_stride, q_start, state_slots, out, \
                     heads, kv_heads, dim, vdim)
#define PICK(TT)                      \
  if (rpl <= 8) LAUNCH(TT, 8);        \
  else if (rpl <= 16) LAUNCH(TT, 16); \
  else if (rpl <= 32) LAUNCH(TT, 32); \
  else LAUNCH(TT, 64);
  if (dtype == IX_F32) { PICK(float) } else { PICK(bf16_t) }
#undef PICK
#undef LAUNCH
  return ix_check_launch("ix_delta_rule");
}

// ---------------------------------------------------------------------------
// What follows a mixer whose heads are normalised one by one, a wavefront per (token, head):
//
//   o = x - lambda x2  (x2 optional);  y = o / sqrt(mean(o^2) + eps) * weight (optional) * silu(gate) (optional) * mult
//
// x, x2 float32 [T, heads, vdim]; weight [vdim], shared by the heads; gate of the run's type at
// gate[t * gate_stride + head * vdim + j]; out of the run's type [T, heads * vdim].
template <typename T>
__global__ void __launch_bounds__(256)
head_norm_gate_kernel(const float* __restrict__ x, const float* __restrict__ x2, float lambda,
                      const void* __restrict__ weight, int w_dtype, const T* __restrict__ gate, int64_t gate_stride,
                      T* __restrict__ out, int64_t pairs, int heads, int vdim, float eps, float mult) {
  const int64_t p = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (p >= pairs) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = p / heads;
  const int head = static_cast<int>(p % heads);
  const float* xr = x + p * vdim;
  const float* x2r = x2 ? x2 + p * vdim : nullptr;
  float ss = 0.f;
  for (int j = lane; j < vdim; j += 64) {
    const float o = x2r ? xr[j] - lambda * x2r[j] : xr[j];
    ss += o * o;
  }
  ss = ix_wave_sum(ss);
  const float inv = mult / sqrtf(ss / static_cast<float>(vdim) + eps);
  for (int j = lane; j < vdim; j += 64) {
    float y = (x2r ? xr[j] - lambda * x2r[j] : xr[j]) * inv;
    if (weight) y *= ix_load_rt(weight, w_dtype, j);
    if (gate) {
      const float gv = ix_load(gate + t * gate_stride + head * vdim + j);
      y *= gv / (1.0f + expf(-gv));
    }
    ix_store(out + p * vdim + j, y);
  }
}

extern "C" int ix_head_norm_gate(const float* x, const float* x2, float lambda, const void* weight, int w_dtype,
                                 const void* gate, int64_t gate_stride, void* out, int dtype, int64_t tokens,
                                 int heads, int vdim, float eps, float mult, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && vdim > 0, "sizes must be positive");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  if (tokens == 0) return 0;
  const int64_t pairs = tokens * heads;
  IX_REQUIRE((pairs + 3) / 4 < (1ll << 31), "too many rows for one launch");
  dim3 grid(static_cast<unsigned>((pairs + 3) / 4)), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, block, 0, stream, x, x2, lambda, weight, w_dtype,
                       (const float*)gate, gate_stride, (float*)out, pairs, heads, vdim, eps, mult);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, block, 0, stream, x, x2, lambda, weight, w_dtype,
                       (const bf16_t*)gate, gate_stride, (bf16_t*)out, pairs, heads, vdim, eps, mult);
  return ix_check_launch("ix_head_norm_gate");
}
