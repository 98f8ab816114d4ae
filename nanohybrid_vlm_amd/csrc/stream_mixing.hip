// Kernels around the residual stream and around attention for layers that are not the pre-norm kind:
//  - nhv_scalar_rmsnorm: RMS norm whose weight is one number;
//  - nhv_pair_norm_mean: half the sum of two rows, each RMS-normed with a weight vector of its own;
//  - nhv_depth_mix: a layer's result joins the list of all earlier results, and the stream that goes on is a
//    weighted sum over that list;
//  - nhv_rotary_split_write: splits a packed q | k | v projection whose value heads may have another size than
//    the key heads, adds biases, turns queries and keys (angles from the position and a list of frequencies,
//    taken in float here: no table, so no bound on positions) and optionally the values, and stores keys and
//    values at the step's slots.
// Statistics, angles and sums are float; rows are float or bfloat16.
#include "nhv_common.h"
#include <math.h>

// ---------------------------------------------------------------- norm with one number as its weight
template <typename TI, typename TO>
__global__ void scalar_rmsnorm_kernel(const TI* __restrict__ x, const float* __restrict__ gain, TO* __restrict__ y, int W,
                                      float eps) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = to_f32(x[base + i]);
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum(ss, scratch);
  const float r = gain[0] / sqrtf(total / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) y[base + i] = from_f32<TO>(to_f32(x[base + i]) * r);
}

extern "C" int nhv_scalar_rmsnorm(const void* x, int x_dtype, const void* gain, void* y, int y_dtype, int T, int W, float eps,
                                  void* stream) {
  NHV_REQUIRE(T > 0 && W > 0, "scalar_rmsnorm: bad sizes T=%d W=%d", T, W);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(TI, TO)                                                                                               \
  hipLaunchKernelGGL((scalar_rmsnorm_kernel<TI, TO>), dim3(T), dim3(256), 0, s, (const TI*)x, (const float*)gain, (TO*)y, \
                     W, eps)
  if (x_dtype == NHV_F32 && y_dtype == NHV_F32) LAUNCH(float, float);
  else if (x_dtype == NHV_F32 && y_dtype == NHV_BF16) LAUNCH(float, bf16_t);
  else if (x_dtype == NHV_BF16 && y_dtype == NHV_F32) LAUNCH(bf16_t, float);
  else if (x_dtype == NHV_BF16 && y_dtype == NHV_BF16) LAUNCH(bf16_t, bf16_t);
  else return nhv_fail("scalar_rmsnorm: unknown dtypes %d -> %d", x_dtype, y_dtype);
#undef LAUNCH
  NHV_LAUNCH_CHECK("scalar_rmsnorm");
  return 0;
}

// ---------------------------------------------------------------- two normed rows, half their sum
template <typename T>
__global__ void pair_norm_mean_kernel(const T* __restrict__ a, const float* __restrict__ wa, const T* __restrict__ b,
                                      const float* __restrict__ wb, T* __restrict__ y, int W, float eps) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * W;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float u = to_f32(a[base + i]), v = to_f32(b[base + i]);
    sa = fmaf(u, u, sa);
    sb = fmaf(v, v, sb);
  }
  const float ra = 1.0f / sqrtf(block_sum(sa, scratch) / (float)W + eps);
  const float rb = 1.0f / sqrtf(block_sum(sb, scratch) / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    y[base + i] = from_f32<T>(0.5f * (to_f32(a[base + i]) * ra * wa[i] + to_f32(b[base + i]) * rb * wb[i]));
}

extern "C" int nhv_pair_norm_mean(const void* a, const void* wa, const void* b, const void* wb, void* y, int T, int W,
                                  float eps, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0, "pair_norm_mean: bad sizes T=%d W=%d", T, W);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(pair_norm_mean_kernel<float>, dim3(T), dim3(256), 0, s, (const float*)a, (const float*)wa,
                       (const float*)b, (const float*)wb, (float*)y, W, eps);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(pair_norm_mean_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (const bf16_t*)a, (const float*)wa,
                       (const bf16_t*)b, (const float*)wb, (bf16_t*)y, W, eps);
  else return nhv_fail("pair_norm_mean: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("pair_norm_mean");
  return 0;
}

// ---------------------------------------------------------------- weighted sum over all results so far
// results[0 .. n) are [rows, W] float each, n = index + 2. results[index + 1] = x + (a + b) is written here (and
// results[0] = x when index is 0: the stream that enters the first layer is the first result); then
// out = sum over j < n of weights[j] * results[j], in rising j. With ``gain`` the RMS norm of out with that one number
// as its weight is written to ``normed`` as well (what the next layer reads). With ``a2`` the first addend is not a but
// half the sum of a and a2, each over its root mean square (pair_eps) times its weight vector wa, wb: what
// nhv_pair_norm_mean would have written, unrounded.
template <typename T>
__global__ void depth_mix_kernel(const float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b,
                                 float* __restrict__ results, size_t plane, int index, const float* __restrict__ weights,
                                 float* __restrict__ out, const float* __restrict__ gain, T* __restrict__ normed, int W,
                                 float eps, const T* __restrict__ a2, const float* __restrict__ wa,
                                 const float* __restrict__ wb, float pair_eps) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * W;
  const int n = index + 2;
  float ra = 1.f, rb = 0.f;
  if (a2 != nullptr) {
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float u = to_f32(a[base + i]), v = to_f32(a2[base + i]);
      sa = fmaf(u, u, sa);
      sb = fmaf(v, v, sb);
    }
    ra = 1.0f / sqrtf(block_sum(sa, scratch) / (float)W + pair_eps);
    rb = 1.0f / sqrtf(block_sum(sb, scratch) / (float)W + pair_eps);
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float xi = x[base + i];
    float add = a2 != nullptr ? 0.5f * (to_f32(a[base + i]) * ra * wa[i] + to_f32(a2[base + i]) * rb * wb[i]) : to_f32(a[base + i]);
    if (b != nullptr) add += to_f32(b[base + i]);
    const float mine = xi + add;
    results[(size_t)(index + 1) * plane + base + i] = mine;
    if (index == 0) results[base + i] = xi;
    float sum = 0.f;
    for (int j = 0; j + 1 < n; ++j) sum = fmaf(weights[j], j == 0 && index == 0 ? xi : results[(size_t)j * plane + base + i], sum);
    sum = fmaf(weights[n - 1], mine, sum);
    out[base + i] = sum;
    ss = fmaf(sum, sum, ss);
  }
  if (gain == nullptr) return;
  const float total = block_sum(ss, scratch);
  const float r = gain[0] / sqrtf(total / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) normed[base + i] = from_f32<T>(out[base + i] * r);
}

extern "C" int nhv_depth_mix(const void* x, const void* a, const void* b, void* results, long long plane, int index,
                             const void* weights, void* out, const void* gain, void* normed, int T, int W, float eps,
                             const void* a2, const void* wa, const void* wb, float pair_eps, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && index >= 0 && plane >= (long long)T * W, "depth_mix: bad sizes T=%d W=%d index=%d", T, W, index);
  NHV_REQUIRE(x != out, "depth_mix: the sum cannot be written over the stream it reads");
  NHV_REQUIRE(a2 == nullptr || (wa != nullptr && wb != nullptr), "depth_mix: a pair of addends without its weights");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(depth_mix_kernel<float>, dim3(T), dim3(256), 0, s, (const float*)x, (const float*)a, (const float*)b,
                       (float*)results, (size_t)plane, index, (const float*)weights, (float*)out, (const float*)gain,
                       (float*)normed, W, eps, (const float*)a2, (const float*)wa, (const float*)wb, pair_eps);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(depth_mix_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (const float*)x, (const bf16_t*)a, (const bf16_t*)b,
                       (float*)results, (size_t)plane, index, (const float*)weights, (float*)out, (const float*)gain,
                       (bf16_t*)normed, W, eps, (const bf16_t*)a2, (const float*)wa, (const float*)wb, pair_eps);
  else return nhv_fail("depth_mix: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("depth_mix");
  return 0;
}

// ---------------------------------------------------------------- split, bias, rotation, store
// qkv [T, ld]: q (Hq heads of D) | k (Hkv heads of D) | v (Hv heads of E) | further columns of another reader; one wave
// per (token, head). A query or key head at position p turns over its first ``rot`` coordinates by p * qk_freqs[i]:
// pair (i, i + rot / 2), or (2i, 2i + 1) where ``interleaved``; the coordinates from rot on pass. v_freqs [E / 2] or
// null: pair (m, m + E / 2) of a value head turns by p * v_freqs[m]. ``unit``: after the rotation every query and key
// head is divided by its root mean square (unit_eps under the root), in float before anything is rounded.
// ``v_from_k``: there are no value columns; value head g is key head g as projected (bias added, not turned, not
// normed). ``maps`` n > 1: every query and key head holds n maps of D entries, [map 1 | map 2 | ...], each turned (and
// normed) on its own; Hq and Hkv count maps. The n maps of a key head are stored side by side as one key of n D entries
// (there are Hkv / n key heads, and as many value heads); a query map goes out as a head of n D entries of its own
// with zeros in the other maps' places, so that its product with the stored key is its product with its own map.
template <typename T>
__global__ void rotary_split_write_kernel(const T* __restrict__ qkv, const T* __restrict__ bias,
                                          const float* __restrict__ qk_freqs, int rot, const float* __restrict__ v_freqs,
                                          const int* __restrict__ positions, const int* __restrict__ slot_mapping,
                                          T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int Hq,
                                          int Hkv, int Hv, int D, int E, int heads, int ld, int interleaved, int unit,
                                          float unit_eps, int v_from_k, int maps) {
  extern __shared__ float staged[];            // D floats where heads are normed: the head after bias and rotation
  const int t = blockIdx.x / heads, head = blockIdx.x % heads;
  const float p = (float)positions[t];
  int col, size, half;
  bool normed = false, pairs_adjacent = false;
  const float* freqs;
  T* dst;
  if (head < Hq) {
    col = head * D; size = D; half = rot / 2; freqs = qk_freqs; normed = unit; pairs_adjacent = interleaved;
    T* whole = q_out + ((size_t)t * Hq + head) * maps * D;
    dst = whole + (head % maps) * D;
    if (maps > 1)                              // the other maps' places
      for (int i = threadIdx.x; i < maps * D; i += blockDim.x)
        if (i / D != head % maps) whole[i] = from_f32<T>(0.f);
  } else {
    const int slot = slot_mapping[t];
    if (slot < 0) return;                      // a row that stores nothing (padding of a recorded step)
    if (head < Hq + Hkv) {
      const int g = head - Hq;
      col = Hq * D + g * D; size = D; half = rot / 2; freqs = qk_freqs; normed = unit; pairs_adjacent = interleaved;
      dst = k_cache + ((size_t)slot * Hkv + g) * D;          // (map g % maps of key head g / maps: the same place)
    } else {
      const int g = head - Hq - Hkv;
      col = v_from_k ? Hq * D + g * D : (Hq + Hkv) * D + g * E;
      size = E; half = v_freqs ? E / 2 : 0; freqs = v_freqs;
      dst = v_cache + ((size_t)slot * Hv + g) * E;
    }
  }
  const T* src = qkv + (size_t)t * ld + col;
  const T* bs = bias ? bias + col : nullptr;
  // the bias joins a projection that was rounded to the rows' type, and the sum is rounded again (the product's own result)
  auto value = [&](int i) { return bs ? to_f32(from_f32<T>(to_f32(src[i]) + to_f32(bs[i]))) : to_f32(src[i]); };
  if (!normed) {                               // nothing of the head depends on all of it: every entry goes out at once
    for (int i = threadIdx.x; i < size - half; i += blockDim.x) {
      if (i < half) {
        const int a = pairs_adjacent ? 2 * i : i, b = pairs_adjacent ? 2 * i + 1 : i + half;
        const float u = value(a), v = value(b);
        float sn, cs;
        sincosf(p * freqs[i], &sn, &cs);
        dst[a] = from_f32<T>(u * cs - v * sn);
        dst[b] = from_f32<T>(v * cs + u * sn);
      } else {
        dst[i + half] = from_f32<T>(value(i + half));
      }
    }
    return;
  }
  // the unit norm follows the rotation: the turned head waits in LDS as floats for its sum of squares
  float ss = 0.f;
  for (int i = threadIdx.x; i < size - half; i += blockDim.x) {
    if (i < half) {
      const int a = pairs_adjacent ? 2 * i : i, b = pairs_adjacent ? 2 * i + 1 : i + half;
      const float u = value(a), v = value(b);
      float sn, cs;
      sincosf(p * freqs[i], &sn, &cs);
      const float x = u * cs - v * sn, y = v * cs + u * sn;
      staged[a] = x;
      staged[b] = y;
      ss = fmaf(x, x, fmaf(y, y, ss));
    } else {
      const float x = value(i + half);
      staged[i + half] = x;
      ss = fmaf(x, x, ss);
    }
  }
  const float r = 1.0f / sqrtf(wave_sum(ss) / (float)size + unit_eps);
  __syncthreads();
  for (int i = threadIdx.x; i < size; i += blockDim.x) dst[i] = from_f32<T>(staged[i] * r);
}

extern "C" int nhv_rotary_split_write(const void* qkv, const void* bias, const void* qk_freqs, int rot, const void* v_freqs,
                                      const void* positions, const void* slot_mapping, void* q_out, void* k_cache,
                                      void* v_cache, int T, int Hq, int Hkv, int D, int E, int with_kv, int more_columns,
                                      int interleaved, int unit, float unit_eps, int v_from_k, int maps, int dtype,
                                      void* stream) {
  NHV_REQUIRE(more_columns >= 0, "rotary_split_write: %d columns after the projection", more_columns);
  NHV_REQUIRE(T > 0 && Hq > 0 && Hkv > 0 && D > 0 && E > 0, "rotary_split_write: bad sizes T=%d Hq=%d Hkv=%d D=%d E=%d", T, Hq, Hkv, D, E);
  NHV_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D, "rotary_split_write: rotary size %d with head size %d", rot, D);
  NHV_REQUIRE(rot == 0 || qk_freqs, "rotary_split_write: a rotary size without frequencies");
  NHV_REQUIRE(!v_freqs || E % 2 == 0, "rotary_split_write: value heads of odd size %d cannot be turned", E);
  NHV_REQUIRE(!with_kv || (slot_mapping && k_cache && v_cache), "rotary_split_write: cache write without cache");
  NHV_REQUIRE(maps >= 1 && Hq % maps == 0 && Hkv % maps == 0, "rotary_split_write: %d maps with %d and %d heads", maps, Hq, Hkv);
  NHV_REQUIRE(!v_from_k || (E == D && maps == 1), "rotary_split_write: values that are the keys as projected have the keys' size and one map");
  NHV_REQUIRE(!unit || unit_eps >= 0.f, "rotary_split_write: eps %g", (double)unit_eps);
  const int Hv = Hkv / maps;
  const int heads = with_kv ? Hq + Hkv + Hv : Hq;
  const int ld = (with_kv ? Hq * D + Hkv * D + (v_from_k ? 0 : Hv * E) : Hq * D) + more_columns;   // (columns that belong to another reader)
  NHV_REQUIRE((long long)T * heads < (1ll << 31), "rotary_split_write: too many tokens");
  const size_t lds = unit ? (size_t)D * sizeof(float) : 0;
  NHV_REQUIRE(lds <= 64 * 1024, "rotary_split_write: heads of %d entries are beyond this kernel's unit norm", D);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(TT)                                                                                                   \
  hipLaunchKernelGGL(rotary_split_write_kernel<TT>, dim3((unsigned)((size_t)T * heads)), dim3(NHV_WAVE), lds, s,     \
                     (const TT*)qkv, (const TT*)bias, (const float*)qk_freqs, rot, (const float*)v_freqs,            \
                     (const int*)positions, (const int*)slot_mapping, (TT*)q_out, (TT*)k_cache, (TT*)v_cache, Hq, Hkv, Hv, \
                     D, E, heads, ld, interleaved, unit, unit_eps, v_from_k, maps)
  if (dtype == NHV_F32) LAUNCH(float);
  else if (dtype == NHV_BF16) LAUNCH(bf16_t);
  else return nhv_fail("rotary_split_write: unknown dtype %d", dtype);
#undef LAUNCH
  NHV_LAUNCH_CHECK("rotary_split_write");
  return 0;
}

// ---------------------------------------------------------------- heads turned back by their position
// x[T, H, E] in place: pair (m, m + E / 2) of every head at position p turns by -p * freqs[m].
template <typename T>
__global__ void turn_back_kernel(T* __restrict__ x, const float* __restrict__ freqs, const int* __restrict__ positions, int H,
                                 int E) {
  const int t = blockIdx.x / H;
  const float p = (float)positions[t];
  T* row = x + (size_t)blockIdx.x * E;
  const int half = E / 2;
  for (int m = threadIdx.x; m < half; m += blockDim.x) {
    const float u = to_f32(row[m]), v = to_f32(row[m + half]);
    float sn, cs;
    sincosf(p * freqs[m], &sn, &cs);
    row[m] = from_f32<T>(u * cs + v * sn);
    row[m + half] = from_f32<T>(v * cs - u * sn);
  }
}

extern "C" int nhv_turn_back(void* x, const void* freqs, const void* positions, int T, int H, int E, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && H > 0 && E > 0 && E % 2 == 0, "turn_back: bad sizes T=%d H=%d E=%d", T, H, E);
  NHV_REQUIRE((long long)T * H < (1ll << 31), "turn_back: too many tokens");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(turn_back_kernel<float>, dim3((unsigned)((size_t)T * H)), dim3(NHV_WAVE), 0, s, (float*)x,
                       (const float*)freqs, (const int*)positions, H, E);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(turn_back_kernel<bf16_t>, dim3((unsigned)((size_t)T * H)), dim3(NHV_WAVE), 0, s, (bf16_t*)x,
                       (const float*)freqs, (const int*)positions, H, E);
  else return nhv_fail("turn_back: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("turn_back");
  return 0;
}
