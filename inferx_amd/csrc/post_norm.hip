// A branch's result that is normalised before it joins the residual stream, fused with the norm that follows:
//
//   d = delta / sqrt(mean(delta^2) + eps_d) * w_d;   h += d;   out = h / sqrt(mean(h^2) + eps) * w
//
// for layers that norm both before and after each branch.  One workgroup per row, everything in float32; h is
// float32 [T, width] and updated in place, unless `rows` picks rows out (then out[r] comes from row rows[r] and h
// stays).  With w null only the first two steps are done (nothing follows).
#include "common.h"

template <typename TD, typename TO>
__global__ void add_normed_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                          const void* __restrict__ wd, int wd_dtype, float eps_d,
                                          const void* __restrict__ w, int w_dtype, float eps, TO* __restrict__ out,
                                          const int32_t* __restrict__ rows, int64_t width) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t row = rows ? rows[r] : r;
  float* hr = h + row * width;
  const TD* dr = delta + row * width;
  float ssd = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    const float d = ix_load(dr + i);
    ssd += d * d;
  }
  ssd = ix_block_sum(ssd, red);
  const float inv_d = 1.0f / sqrtf(ssd / static_cast<float>(width) + eps_d);
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = hr[i] + ix_load(dr + i) * inv_d * ix_load_rt(wd, wd_dtype, i);
    if (!rows) hr[i] = v;  // (read again below by the thread that wrote it)
    ss += v * v;
  }
  if (!w) return;
  ss = ix_block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(width) + eps);
  TO* outr = out + r * width;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = rows ? hr[i] + ix_load(dr + i) * inv_d * ix_load_rt(wd, wd_dtype, i) : hr[i];
    ix_store(outr + i, v * inv * ix_load_rt(w, w_dtype, i));
  }
}

extern "C" int ix_add_normed_rmsnorm(void* h, const void* delta, int delta_dtype, const void* wd, int wd_dtype,
                                     float eps_d, const void* w, int w_dtype, float eps, void* out, int out_dtype,
                                     const int32_t* rows, int64_t n_out_rows, int64_t width, hipStream_t stream) {
  IX_REQUIRE(width > 0 && n_out_rows >= 0, "sizes must be positive");
  IX_REQUIRE(delta != nullptr && wd != nullptr, "the branch's result and its norm's weight are needed");
  IX_REQUIRE((w == nullptr) == (out == nullptr), "a following norm and its output come together");
  if (n_out_rows == 0) return 0;
  dim3 grid(n_out_rows), block(width >= 4096 ? 1024 : (width >= 1024 ? 512 : 256));
#define LAUNCH(TD, TO)                                                                                             \
  hipLaunchKernelGGL((add_normed_rmsnorm_kernel<TD, TO>), grid, block, 0, stream, (float*)h, (const TD*)delta, wd, \
                     wd_dtype, eps_d, w, w_dtype, eps, (TO*)out, rows, width)
  if (delta_dtype == IX_F32 && out_dtype == IX_F32) LAUNCH(float, float);
  else if (delta_dtype == IX_F32 && out_dtype == IX_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == IX_BF16 && out_dtype == IX_F32) LAUNCH(bf16_t, float);
  else if (delta_dtype == IX_BF16 && out_dtype == IX_BF16) LAUNCH(bf16_t, bf16_t);
  else IX_REQUIRE(false, "dtypes must be float32 or bfloat16");
#undef LAUNCH
  return ix_check_launch("ix_add_normed_rmsnorm");
}
