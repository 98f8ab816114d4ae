// What attention heads' results pass before the output projection, where a layer asks for more than the softmax:
//  - nhv_differential_combine: two softmax maps per head over the same values become one result,
//    o = a1 - lambda a2, divided by its root mean square over the head's value entries and multiplied by a constant
//    and, optionally, by the sigmoid of a gate per (token, head);
//  - nhv_gate_rows: rows multiplied entry by entry with the sigmoid of gates that lie in columns of another tensor;
//  - nhv_add_bias_rows: a bias added to the rows of a product that another routine has made.
// Everything is taken in float; rows are float or bfloat16.
#include "nhv_common.h"
#include <math.h>

// a [T, 2 H, E]: per head its map 1, then its map 2 ([head][map]); lambda [1] float; gate: null, or the gates of
// token t at gate[t * gate_ld + h]. out [T, H, E]. One wave per (token, head).
template <typename T>
__global__ void differential_combine_kernel(const T* __restrict__ a, const float* __restrict__ lambda, T* __restrict__ out,
                                            int H, int E, float eps, float post, const T* __restrict__ gate,
                                            long long gate_ld) {
  const int t = blockIdx.x / H, h = blockIdx.x % H;
  const T* a1 = a + ((size_t)t * H + h) * 2 * E;
  const T* a2 = a1 + E;
  const float lam = lambda[0];
  float ss = 0.f;
  for (int i = threadIdx.x; i < E; i += blockDim.x) {
    const float d = to_f32(a1[i]) - lam * to_f32(a2[i]);
    ss = fmaf(d, d, ss);
  }
  float r = post / sqrtf(wave_sum(ss) / (float)E + eps);
  if (gate) r /= 1.0f + expf(-to_f32(gate[(size_t)t * gate_ld + h]));
  T* o = out + ((size_t)t * H + h) * E;
  for (int i = threadIdx.x; i < E; i += blockDim.x) o[i] = from_f32<T>((to_f32(a1[i]) - lam * to_f32(a2[i])) * r);
}

extern "C" int nhv_differential_combine(const void* a, const void* lambda, void* out, int T, int H, int E, float eps,
                                        float post, const void* gate, long long gate_ld, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && H > 0 && E > 0 && eps >= 0.f, "differential_combine: bad sizes T=%d H=%d E=%d eps=%g", T, H, E, (double)eps);
  NHV_REQUIRE(!gate || gate_ld >= H, "differential_combine: gate rows %lld apart for %d heads", gate_ld, H);
  NHV_REQUIRE((long long)T * H < (1ll << 31), "differential_combine: too many tokens");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((size_t)T * H));
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(differential_combine_kernel<float>, grid, dim3(NHV_WAVE), 0, s, (const float*)a, (const float*)lambda,
                       (float*)out, H, E, eps, post, (const float*)gate, gate_ld);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(differential_combine_kernel<bf16_t>, grid, dim3(NHV_WAVE), 0, s, (const bf16_t*)a, (const float*)lambda,
                       (bf16_t*)out, H, E, eps, post, (const bf16_t*)gate, gate_ld);
  else return nhv_fail("differential_combine: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("differential_combine");
  return 0;
}

// bfloat16 rows whose entries come in whole groups of eight at 16-byte places: eight entries a thread
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 ho_bf16x8;

__global__ void gate_rows_bf16x8_kernel(bf16_t* __restrict__ x, const bf16_t* __restrict__ gate, long long gate_ld, int N8,
                                        size_t total8) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total8; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / N8, n = (i % N8) * 8;
    ho_bf16x8 v = *reinterpret_cast<const ho_bf16x8*>(x + i * 8);
    const ho_bf16x8 g = *reinterpret_cast<const ho_bf16x8*>(gate + t * gate_ld + n);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (__bf16)((float)v[e] / (1.0f + expf(-(float)g[e])));
    *reinterpret_cast<ho_bf16x8*>(x + i * 8) = v;
  }
}

__global__ void add_bias_rows_bf16x8_kernel(bf16_t* __restrict__ x, const bf16_t* __restrict__ bias, int N8, size_t total8) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total8; i += (size_t)gridDim.x * blockDim.x) {
    ho_bf16x8 v = *reinterpret_cast<const ho_bf16x8*>(x + i * 8);
    const ho_bf16x8 b = *reinterpret_cast<const ho_bf16x8*>(bias + (i % N8) * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (__bf16)((float)v[e] + (float)b[e]);
    *reinterpret_cast<ho_bf16x8*>(x + i * 8) = v;
  }
}

static bool ho_at_16_bytes(const void* p) { return ((uintptr_t)p & 15) == 0; }
static unsigned ho_blocks(size_t items) { return (unsigned)((items + 255) / 256 > 65535u * 16 ? 65535u * 16 : (items + 255) / 256); }

// x [T, N] in place: x[t, n] *= sigmoid(gate[t * gate_ld + n]).
template <typename T>
__global__ void gate_rows_kernel(T* __restrict__ x, const T* __restrict__ gate, long long gate_ld, int N, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / N, n = i % N;
    x[i] = from_f32<T>(to_f32(x[i]) / (1.0f + expf(-to_f32(gate[t * gate_ld + n]))));
  }
}

extern "C" int nhv_gate_rows(void* x, const void* gate, long long gate_ld, int T, int N, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && N > 0 && gate && gate_ld >= N, "gate_rows: bad sizes T=%d N=%d, gate rows %lld apart", T, N, gate_ld);
  const size_t total = (size_t)T * N;
  const unsigned blocks = ho_blocks(total);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_BF16 && N % 8 == 0 && gate_ld % 8 == 0 && ho_at_16_bytes(x) && ho_at_16_bytes(gate))
    hipLaunchKernelGGL(gate_rows_bf16x8_kernel, dim3(ho_blocks(total / 8)), dim3(256), 0, s, (bf16_t*)x, (const bf16_t*)gate,
                       gate_ld, N / 8, total / 8);
  else if (dtype == NHV_F32)
    hipLaunchKernelGGL(gate_rows_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)x, (const float*)gate, gate_ld, N, total);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(gate_rows_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (bf16_t*)x, (const bf16_t*)gate, gate_ld, N, total);
  else return nhv_fail("gate_rows: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("gate_rows");
  return 0;
}

// x [T, N] in place: x[t, n] += bias[n] (the sum is rounded to the rows' type once more).
template <typename T>
__global__ void add_bias_rows_kernel(T* __restrict__ x, const T* __restrict__ bias, int N, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
    x[i] = from_f32<T>(to_f32(x[i]) + to_f32(bias[i % N]));
}

extern "C" int nhv_add_bias_rows(void* x, const void* bias, int T, int N, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && N > 0 && bias, "add_bias_rows: bad sizes T=%d N=%d", T, N);
  const size_t total = (size_t)T * N;
  const unsigned blocks = ho_blocks(total);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_BF16 && N % 8 == 0 && ho_at_16_bytes(x) && ho_at_16_bytes(bias))
    hipLaunchKernelGGL(add_bias_rows_bf16x8_kernel, dim3(ho_blocks(total / 8)), dim3(256), 0, s, (bf16_t*)x, (const bf16_t*)bias,
                       N / 8, total / 8);
  else if (dtype == NHV_F32)
    hipLaunchKernelGGL(add_bias_rows_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)x, (const float*)bias, N, total);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(add_bias_rows_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (bf16_t*)x, (const bf16_t*)bias, N, total);
  else return nhv_fail("add_bias_rows: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("add_bias_rows");
  return 0;
}
