// Several residual streams side by side (hyper-connections), and the small kernels of models built on them.
//  - nhv_streams_step: one launch between two sublayers. The n streams X_1 .. X_n ([n, T, W] float) take the result y
//    of the sublayer that has just run, all at once from their old values,
//        X_t <- sum_s mix[s, t] X_s + out[t] y,         y = sa a (+ sb b)  (two mixers side by side, each with a scale),
//    and the next sublayer's input is read from the new values through its norm,
//        h = u / sqrt(mean(u^2) + eps) * w,             u = sum_s in[s] X_s.
//    Either half may be absent; at the start all streams equal one row (x0), at the end their sum is written
//    instead of the streams. With n = 1 and coefficients of 1 this is the plain residual addition and RMS norm
//    of a float stream. Everything is float but the rows a, b and h.
//  - nhv_embed_float: rows of the table times a scale, as floats (the start of a float stream).
//  - nhv_activation: an activation on rows, in place.  nhv_scale: float numbers times one number, in place.
//  - nhv_scaled_sum: sa a + sb b of two tensors of rows.
// One block per token, of 256, 512 or 1,024 threads by the width alone (a step of a few single tokens is a few blocks,
// and what it takes is the chain of loads and stores of one thread: at most four columns a thread from a width of
// 1,024 on); a thread owns columns i, i + threads, ...; the sum over a row's squares is taken in an order that
// depends on the width only, so a token's result does not depend on its batch.
#include "nhv_common.h"
#include <math.h>

#define NHV_MAX_STREAMS 16

template <typename TR, int NMAX, int THREADS>
__global__ __launch_bounds__(THREADS) void streams_step_kernel(
    float* __restrict__ X, long long stride, const float* __restrict__ x0, const float* __restrict__ mix,
    const float* __restrict__ out_w, const TR* __restrict__ a, const TR* __restrict__ b, float sa, float sb,
    const float* __restrict__ in_w, const float* __restrict__ norm_w, float eps, TR* __restrict__ h,
    float* __restrict__ total, int n, int W) {
  extern __shared__ float lds[];            // u: W floats; then 16 for the block's sum; then mix n n, out n, in n
  float* u_s = lds;
  float* scratch = lds + W;
  float* mix_s = scratch + 16;
  float* out_s = mix_s + n * n;
  float* in_s = out_s + n;
  const bool update = mix != nullptr;
  for (int i = threadIdx.x; i < n * n; i += blockDim.x) mix_s[i] = update ? mix[i] : 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    out_s[i] = update ? out_w[i] : 0.f;
    in_s[i] = in_w ? in_w[i] : 1.f;
  }
  __syncthreads();
  const size_t row = (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float xs[NMAX];
    if (x0) {
      const float v = x0[row + i];
#pragma unroll
      for (int s = 0; s < NMAX; ++s) xs[s] = v;
    } else {
#pragma unroll
      for (int s = 0; s < NMAX; ++s) xs[s] = s < n ? X[(size_t)s * stride + row + i] : 0.f;
    }
    float u = 0.f, sum = 0.f;
    if (update) {
      float y = sa * to_f32(a[row + i]);
      if (b) y = fmaf(sb, to_f32(b[row + i]), y);
#pragma unroll
      for (int t = 0; t < NMAX; ++t) {
        if (t < n) {
          float acc = out_s[t] * y;
#pragma unroll
          for (int s = 0; s < NMAX; ++s)
            if (s < n) acc = fmaf(mix_s[s * n + t], xs[s], acc);
          if (!total) X[(size_t)t * stride + row + i] = acc;
          u = fmaf(in_s[t], acc, u);
          sum += acc;
        }
      }
    } else {
#pragma unroll
      for (int t = 0; t < NMAX; ++t) {
        if (t < n) {
          if (x0 && !total) X[(size_t)t * stride + row + i] = xs[t];
          u = fmaf(in_s[t], xs[t], u);
          sum += xs[t];
        }
      }
    }
    if (total) total[row + i] = sum;
    if (h) {
      u_s[i] = u;
      ss = fmaf(u, u, ss);
    }
  }
  if (!h) return;
  const float r = 1.0f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) h[row + i] = from_f32<TR>(u_s[i] * r * norm_w[i]);
}

extern "C" int nhv_streams_step(void* X, long long stride, const void* x0, const void* mix, const void* out_w, const void* a,
                                const void* b, float sa, float sb, const void* in_w, const void* norm_w, float eps, void* h,
                                void* total, int n, int T, int W, int rows_dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && n >= 1 && n <= NHV_MAX_STREAMS, "streams_step: bad sizes T=%d W=%d streams=%d (1 to %d are taken)", T, W,
              n, NHV_MAX_STREAMS);
  NHV_REQUIRE(X || (x0 && total), "streams_step: no streams");
  NHV_REQUIRE((mix == nullptr) == (out_w == nullptr) && (mix == nullptr) == (a == nullptr), "streams_step: an update needs mix, out and a result");
  NHV_REQUIRE((h == nullptr) == (norm_w == nullptr), "streams_step: a read needs a norm weight and a place for its rows");
  NHV_REQUIRE(mix || h || total || x0, "streams_step: nothing to do");
  const size_t lds = ((size_t)W + 16 + (size_t)n * n + 2 * n) * sizeof(float);
  NHV_REQUIRE(lds <= 64 * 1024, "streams_step: a width of %d does not fit the kernel's 64 KB of LDS", W);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH_AS(TR, NMAX, THREADS)                                                                                  \
  hipLaunchKernelGGL((streams_step_kernel<TR, NMAX, THREADS>), dim3(T), dim3(THREADS), lds, s, (float*)X, stride,     \
                     (const float*)x0, (const float*)mix, (const float*)out_w, (const TR*)a, (const TR*)b, sa, sb,    \
                     (const float*)in_w, (const float*)norm_w, eps, (TR*)h, (float*)total, n, W)
#define LAUNCH(TR, NMAX)                             \
  do {                                               \
    if (W <= 1024) LAUNCH_AS(TR, NMAX, 256);         \
    else if (W <= 2048) LAUNCH_AS(TR, NMAX, 512);    \
    else LAUNCH_AS(TR, NMAX, 1024);                  \
  } while (0)
#define BY_N(TR)                                     \
  do {                                               \
    if (n == 1) LAUNCH(TR, 1);                       \
    else if (n == 2) LAUNCH(TR, 2);                  \
    else if (n <= 4) LAUNCH(TR, 4);                  \
    else if (n <= 8) LAUNCH(TR, 8);                  \
    else LAUNCH(TR, 16);                             \
  } while (0)
  if (rows_dtype == NHV_F32) BY_N(float);
  else if (rows_dtype == NHV_BF16) BY_N(bf16_t);
  else return nhv_fail("streams_step: unknown dtype %d", rows_dtype);
#undef BY_N
#undef LAUNCH
#undef LAUNCH_AS
  NHV_LAUNCH_CHECK("streams_step");
  return 0;
}

// ---------------------------------------------------------------- embedding rows as floats
template <typename T>
__global__ void embed_float_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out, int W,
                                   int V, float scale) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;   // the host checks ids; an id out of range gives a row of zeros, never a wild read
  const T* src = table + (size_t)(ok ? id : 0) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) out[(size_t)t * W + i] = ok ? to_f32(src[i]) * scale : 0.f;
}

extern "C" int nhv_embed_float(const void* ids, const void* table, void* out, int T, int W, int V, int dtype, float scale,
                               void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && V > 0, "embed_float: bad sizes T=%d W=%d V=%d", T, W, V);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(embed_float_kernel<float>, dim3(T), dim3(256), 0, s, (const int*)ids, (const float*)table, (float*)out, W, V, scale);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(embed_float_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (const int*)ids, (const bf16_t*)table, (float*)out, W, V, scale);
  else return nhv_fail("embed_float: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("embed_float");
  return 0;
}

// ---------------------------------------------------------------- an activation on rows, in place
// act 0: z sigmoid(z); 1: the tanh form of GELU; 2: max(z, 0)^2. Taken in float, rounded once.
__device__ __forceinline__ float activation_f(float z, int act) {
  if (act == 0) return z / (1.0f + expf(-z));
  if (act == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  const float r = fmaxf(z, 0.f);
  return r * r;
}

template <typename T>
__global__ void activation_kernel(T* __restrict__ x, size_t n, int act) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    x[i] = from_f32<T>(activation_f(to_f32(x[i]), act));
}

// the same, 16 bytes a thread and turn (counts that are a multiple of 8 from an address that is one of 16)
template <typename T>
__global__ void activation_vec_kernel(T* __restrict__ x, size_t n8, int act) {
  constexpr int PER = 16 / sizeof(T);       // entries in 16 bytes: 8 bfloat16 or 4 float
  typedef T vec_t __attribute__((ext_vector_type(PER)));
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8 * (8 / PER); i += (size_t)gridDim.x * blockDim.x) {
    vec_t v = reinterpret_cast<vec_t*>(x)[i];
#pragma unroll
    for (int e = 0; e < PER; ++e) v[e] = from_f32<T>(activation_f(to_f32((T)v[e]), act));
    reinterpret_cast<vec_t*>(x)[i] = v;
  }
}

extern "C" int nhv_activation(void* x, size_t n, int act, int dtype, void* stream) {
  NHV_REQUIRE(n > 0 && act >= 0 && act <= 2, "activation: %zu entries, activation %d", n, act);
  hipStream_t s = (hipStream_t)stream;
  if (n % 8 == 0 && (uintptr_t)x % 16 == 0) {
    const size_t turns = n / 8 * (dtype == NHV_F32 ? 2 : 1), want = (turns + 255) / 256;
    const dim3 grid((unsigned)(want > 65535 * 16 ? 65535 * 16 : want));
    if (dtype == NHV_F32) hipLaunchKernelGGL(activation_vec_kernel<float>, grid, dim3(256), 0, s, (float*)x, n / 8, act);
    else if (dtype == NHV_BF16) hipLaunchKernelGGL(activation_vec_kernel<bf16_t>, grid, dim3(256), 0, s, (bf16_t*)x, n / 8, act);
    else return nhv_fail("activation: unknown dtype %d", dtype);
    NHV_LAUNCH_CHECK("activation");
    return 0;
  }
  const size_t want = (n + 255) / 256;
  const dim3 grid((unsigned)(want > 65535 * 8 ? 65535 * 8 : want));
  if (dtype == NHV_F32) hipLaunchKernelGGL(activation_kernel<float>, grid, dim3(256), 0, s, (float*)x, n, act);
  else if (dtype == NHV_BF16) hipLaunchKernelGGL(activation_kernel<bf16_t>, grid, dim3(256), 0, s, (bf16_t*)x, n, act);
  else return nhv_fail("activation: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("activation");
  return 0;
}

// ---------------------------------------------------------------- float numbers times one number, in place
__global__ void scale_kernel(float* __restrict__ x, size_t n, float factor) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) x[i] *= factor;
}

extern "C" int nhv_scale(void* x, size_t n, float factor, void* stream) {
  NHV_REQUIRE(n > 0, "scale: nothing to scale");
  const size_t want = (n + 255) / 256;
  hipLaunchKernelGGL(scale_kernel, dim3((unsigned)(want > 65535 * 8 ? 65535 * 8 : want)), dim3(256), 0, (hipStream_t)stream,
                     (float*)x, n, factor);
  NHV_LAUNCH_CHECK("scale");
  return 0;
}

// ---------------------------------------------------------------- sa a + sb b, taken in float and rounded once
template <typename T>
__global__ void scaled_sum_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ y, size_t n, float sa, float sb) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    y[i] = from_f32<T>(fmaf(sb, to_f32(b[i]), sa * to_f32(a[i])));
}

extern "C" int nhv_scaled_sum(const void* a, const void* b, void* y, size_t n, float sa, float sb, int dtype, void* stream) {
  NHV_REQUIRE(n > 0, "scaled_sum: nothing to add");
  const size_t want = (n + 255) / 256;
  const dim3 grid((unsigned)(want > 65535 * 8 ? 65535 * 8 : want));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32) hipLaunchKernelGGL(scaled_sum_kernel<float>, grid, dim3(256), 0, s, (const float*)a, (const float*)b, (float*)y, n, sa, sb);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(scaled_sum_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)a, (const bf16_t*)b, (bf16_t*)y, n, sa, sb);
  else return nhv_fail("scaled_sum: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("scaled_sum");
  return 0;
}
