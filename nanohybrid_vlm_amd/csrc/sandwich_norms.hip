// A layer whose sublayers are normed on both sides: x <- x + norm_b(sublayer(norm_a(x))) on a float stream x.
// nhv_sandwich_step is the one launch between two sublayers: it norms the result y of the sublayer before it
// (y / sqrt(mean(y^2) + eps) * wb), adds that to the stream, and norms the new stream for the sublayer after it
// (x / sqrt(mean(x^2) + eps) * wa, given as rows of the model's element type). Either half may be absent: the first
// launch of a model only reads, the last only adds. One block a token whose size depends on the width alone, so the
// order of a row's sums, and with it a token's result, does not depend on the batch. Statistics, weights and the
// stream are float.
#include "nhv_common.h"
#include <math.h>

template <typename TY, typename TH, int BLOCK>
__global__ __launch_bounds__(BLOCK) void sandwich_step_kernel(float* __restrict__ x, const TY* __restrict__ y,
                                                              const float* __restrict__ wb, float eps_b,
                                                              const float* __restrict__ wa, float eps_a,
                                                              TH* __restrict__ h, int W) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * W;
  float* xr = x + base;
  if (y) {
    const TY* yr = y + base;
    float ss = 0.f;
    for (int i = threadIdx.x; i < W; i += BLOCK) {
      const float v = to_f32(yr[i]);
      ss = fmaf(v, v, ss);
    }
    const float r = 1.0f / sqrtf(block_sum(ss, scratch) / (float)W + eps_b);
    if (!wa) {
      for (int i = threadIdx.x; i < W; i += BLOCK) xr[i] += to_f32(yr[i]) * r * wb[i];
      return;
    }
    float sx = 0.f;
    for (int i = threadIdx.x; i < W; i += BLOCK) {
      const float v = xr[i] + to_f32(yr[i]) * r * wb[i];
      xr[i] = v;                               // (a thread reads back only what it wrote itself)
      sx = fmaf(v, v, sx);
    }
    const float rx = 1.0f / sqrtf(block_sum(sx, scratch) / (float)W + eps_a);
    TH* hr = h + base;
    for (int i = threadIdx.x; i < W; i += BLOCK) hr[i] = from_f32<TH>(xr[i] * rx * wa[i]);
    return;
  }
  float sx = 0.f;
  for (int i = threadIdx.x; i < W; i += BLOCK) {
    const float v = xr[i];
    sx = fmaf(v, v, sx);
  }
  const float rx = 1.0f / sqrtf(block_sum(sx, scratch) / (float)W + eps_a);
  TH* hr = h + base;
  for (int i = threadIdx.x; i < W; i += BLOCK) hr[i] = from_f32<TH>(xr[i] * rx * wa[i]);
}

template <typename TY, typename TH>
static void sandwich_launch(hipStream_t s, int T, int W, float* x, const void* y, const float* wb, float eps_b,
                            const float* wa, float eps_a, void* h) {
#define LAUNCH(B) hipLaunchKernelGGL((sandwich_step_kernel<TY, TH, B>), dim3(T), dim3(B), 0, s, x, (const TY*)y, wb, eps_b, wa, eps_a, (TH*)h, W)
  if (W <= 1024) LAUNCH(256);
  else if (W <= 4096) LAUNCH(512);
  else LAUNCH(1024);
#undef LAUNCH
}

// x [T, W] float, rewritten if y is given. y [T, W] of y_dtype with wb [W] float, or null. wa [W] float with h [T, W] of
// h_dtype, or null.
extern "C" int nhv_sandwich_step(void* x, const void* y, int y_dtype, const void* wb, float eps_b, const void* wa,
                                 float eps_a, void* h, int h_dtype, int T, int W, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && x, "sandwich_step: bad sizes T=%d W=%d", T, W);
  NHV_REQUIRE(y || wa, "sandwich_step: nothing to add and nothing to read");
  NHV_REQUIRE(!y || wb, "sandwich_step: a result without the weight of its norm");
  NHV_REQUIRE(!wa || h, "sandwich_step: a norm to read through without rows for it");
  NHV_REQUIRE(eps_a >= 0.f && eps_b >= 0.f, "sandwich_step: eps %g, %g", (double)eps_a, (double)eps_b);
  hipStream_t s = (hipStream_t)stream;
  const bool yf = !y || y_dtype == NHV_F32, hf = !wa || h_dtype == NHV_F32;
  NHV_REQUIRE((yf || y_dtype == NHV_BF16) && (hf || h_dtype == NHV_BF16), "sandwich_step: unknown dtypes %d, %d", y_dtype, h_dtype);
  if (yf && hf) sandwich_launch<float, float>(s, T, W, (float*)x, y, (const float*)wb, eps_b, (const float*)wa, eps_a, h);
  else if (yf) sandwich_launch<float, bf16_t>(s, T, W, (float*)x, y, (const float*)wb, eps_b, (const float*)wa, eps_a, h);
  else if (hf) sandwich_launch<bf16_t, float>(s, T, W, (float*)x, y, (const float*)wb, eps_b, (const float*)wa, eps_a, h);
  else sandwich_launch<bf16_t, bf16_t>(s, T, W, (float*)x, y, (const float*)wb, eps_b, (const float*)wa, eps_a, h);
  NHV_LAUNCH_CHECK("sandwich_step");
  return 0;
}
