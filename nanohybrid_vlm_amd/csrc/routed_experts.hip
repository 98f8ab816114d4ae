// A feed-forward made of many small gated feed-forwards of which every token uses a few.
//   nhv_route_topk        from a row's float router logits (plus an optional bias) the ``top`` largest: their numbers and
//                         scores (the sigmoid of each, or the softmax over the chosen logits alone)
//   nhv_experts_gate_up   for every (token, chosen expert): act(s G_e h) * (s U_e h), s the score: the expert's input is
//                         s h, and a product is linear in its rows, so the score multiplies the finished float sums
//                         (no scores: s = 1, for a design whose scores weigh the experts' outputs)
//   nhv_experts_down      out[t] = sum over the token's experts of [w[t, j]] D_e u[t, j] [+ one more row added to all]
// One wave per output: a sum runs over its inner index in an order that depends on the sizes only, so a row's result
// does not depend on its batch. Weights of all experts lie in one tensor, [experts, 2 ff, width] (gate rows, then up
// rows) and [experts, width, ff].
#include "nhv_common.h"
#include <math.h>

// z [T, E] float logits. One wave per token: the ``top`` largest in turn, the lower number among equals.
__global__ __launch_bounds__(256) void route_topk_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                         int* __restrict__ ids, float* __restrict__ scores, int T, int E,
                                                         int top, int mode) {
  extern __shared__ float z_all[];           // 4 waves x E logits
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  float* z = z_all + (size_t)wave * E;
  for (int e = lane; e < E; e += NHV_WAVE) z[e] = logits[(size_t)t * E + e] + (bias ? bias[e] : 0.f);
  __builtin_amdgcn_wave_barrier();
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += NHV_WAVE) {
      const float v = z[e];
      if (v > best) { best = v; at = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, NHV_WAVE);
      const int oa = __shfl_xor(at, o, NHV_WAVE);
      if (ov > best || (ov == best && oa < at)) { best = ov; at = oa; }
    }
    if (at == 0x7fffffff) at = 0;            // (every logit is no number: the first expert)
    if (lane == 0) {
      ids[(size_t)t * top + j] = at;
      scores[(size_t)t * top + j] = mode == 0 ? 1.0f / (1.0f + expf(-best)) : best;
      z[at] = -INFINITY;                     // a chosen expert is out of the next rounds
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (mode == 1 && lane == 0) {              // the softmax over the chosen logits alone; the first is the largest
    float* s = scores + (size_t)t * top;
    const float m = s[0];
    float sum = 0.f;
    for (int j = 0; j < top; ++j) {
      s[j] = expf(s[j] - m);
      sum += s[j];
    }
    for (int j = 0; j < top; ++j) s[j] /= sum;
  }
}

// mode 0: a score is the sigmoid of its logit; 1: the scores are the softmax over the chosen logits
extern "C" int nhv_route_topk(const void* logits, const void* bias, void* ids, void* scores, int T, int E, int top, int mode,
                              void* stream) {
  NHV_REQUIRE(T > 0 && E > 0 && top > 0 && top <= E && E <= 4096, "route_topk: bad sizes T=%d E=%d (up to 4096) top=%d", T, E, top);
  NHV_REQUIRE(mode == 0 || mode == 1, "route_topk: mode %d", mode);
  hipLaunchKernelGGL(route_topk_kernel, dim3((T + 3) / 4), dim3(256), 4 * (size_t)E * sizeof(float), (hipStream_t)stream,
                     (const float*)logits, (const float*)bias, (int*)ids, (float*)scores, T, E, top, mode);
  NHV_LAUNCH_CHECK("route_topk");
  return 0;
}

__device__ __forceinline__ float nhv_expert_act(float z, int act) {
  if (act == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z / (1.0f + expf(-z));
}

// eight consecutive entries as floats
template <typename V>
__device__ __forceinline__ void ex_load8f(const V* p, float* out) {
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = to_f32(p[e]);
}
template <>
__device__ __forceinline__ void ex_load8f<bf16_t>(const bf16_t* p, float* out) {
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 v8;
  const v8 v = *reinterpret_cast<const v8*>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (float)v[e];
}
template <>
__device__ __forceinline__ void ex_load8f<float>(const float* p, float* out) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w; out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
}

// u[t * top + j, f] for the pair (t, j): one wave per f.
template <typename T>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const T* __restrict__ h, const int* __restrict__ ids,
                                                              const float* __restrict__ scores,
                                                              const T* __restrict__ gate_up, T* __restrict__ u, int W,
                                                              int F, int top, int E, int act) {
  const int pair = blockIdx.x;
  const int f = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (f >= F) return;
  const int e = ids[pair];
  if (e < 0 || e >= E) return;
  const T* x = h + (size_t)(pair / top) * W;
  const T* g = gate_up + ((size_t)e * 2 * F + f) * W;
  const T* p = g + (size_t)F * W;
  float sg = 0.f, su = 0.f;
  if (W % 8 == 0) {                          // (rows then start at multiples of 16 or 32 bytes)
    for (int k = lane * 8; k < W; k += NHV_WAVE * 8) {
      float xv[8], gv[8], pv[8];
      ex_load8f(x + k, xv);
      ex_load8f(g + k, gv);
      ex_load8f(p + k, pv);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        sg = fmaf(gv[i], xv[i], sg);
        su = fmaf(pv[i], xv[i], su);
      }
    }
  } else {
    for (int k = lane; k < W; k += NHV_WAVE) {
      const float xv = to_f32(x[k]);
      sg = fmaf(to_f32(g[k]), xv, sg);
      su = fmaf(to_f32(p[k]), xv, su);
    }
  }
  sg = wave_sum(sg);
  su = wave_sum(su);
  if (lane == 0) {
    const float s = scores ? scores[pair] : 1.0f;
    u[(size_t)pair * F + f] = from_f32<T>(nhv_expert_act(s * sg, act) * (s * su));
  }
}

extern "C" int nhv_experts_gate_up(const void* h, const void* ids, const void* scores, const void* gate_up, void* u,
                                   int T, int W, int F, int top, int E, int act, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && F > 0 && top > 0 && E > 0, "experts_gate_up: bad sizes T=%d W=%d F=%d top=%d E=%d", T, W, F, top, E);
  NHV_REQUIRE((long long)T * top < (1ll << 31) && (F + 3) / 4 <= 65535, "experts_gate_up: T=%d top=%d F=%d are beyond this kernel's grid", T, top, F);
  const dim3 grid(T * top, (F + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(experts_gate_up_kernel<float>, grid, dim3(256), 0, s, (const float*)h, (const int*)ids,
                       (const float*)scores, (const float*)gate_up, (float*)u, W, F, top, E, act);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(experts_gate_up_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)h, (const int*)ids,
                       (const float*)scores, (const bf16_t*)gate_up, (bf16_t*)u, W, F, top, E, act);
  else
    return nhv_fail("experts_gate_up: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("experts_gate_up");
  return 0;
}

// out[t, n] = sum over j < top (rising), each a sum over f [times weights[t, j]], [plus add[t, n]]: one wave per n.
template <typename T>
__global__ __launch_bounds__(256) void experts_down_kernel(const T* __restrict__ u, const int* __restrict__ ids,
                                                           const T* __restrict__ down, T* __restrict__ out, int W, int F,
                                                           int top, int E, const float* __restrict__ weights,
                                                           const T* __restrict__ add) {
  const int t = blockIdx.x;
  const int n = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (n >= W) return;
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    const int e = ids[(size_t)t * top + j];
    if (e < 0 || e >= E) continue;
    const T* d = down + ((size_t)e * W + n) * F;
    const T* x = u + ((size_t)t * top + j) * F;
    float s = 0.f;
    if (F % 8 == 0) {
      for (int f = lane * 8; f < F; f += NHV_WAVE * 8) {
        float dv[8], xv[8];
        ex_load8f(d + f, dv);
        ex_load8f(x + f, xv);
#pragma unroll
        for (int i = 0; i < 8; ++i) s = fmaf(dv[i], xv[i], s);
      }
    } else {
      for (int f = lane; f < F; f += NHV_WAVE) s = fmaf(to_f32(d[f]), to_f32(x[f]), s);
    }
    total += weights ? weights[(size_t)t * top + j] * wave_sum(s) : wave_sum(s);
  }
  if (lane == 0) out[(size_t)t * W + n] = from_f32<T>(add ? total + to_f32(add[(size_t)t * W + n]) : total);
}

extern "C" int nhv_experts_down(const void* u, const void* ids, const void* down, void* out, int T, int W, int F, int top,
                                int E, const void* weights, const void* add, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && F > 0 && top > 0 && E > 0, "experts_down: bad sizes T=%d W=%d F=%d top=%d E=%d", T, W, F, top, E);
  NHV_REQUIRE((W + 3) / 4 <= 65535, "experts_down: width %d is beyond this kernel's grid", W);
  const dim3 grid(T, (W + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(experts_down_kernel<float>, grid, dim3(256), 0, s, (const float*)u, (const int*)ids,
                       (const float*)down, (float*)out, W, F, top, E, (const float*)weights, (const float*)add);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(experts_down_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)u, (const int*)ids,
                       (const bf16_t*)down, (bf16_t*)out, W, F, top, E, (const float*)weights, (const bf16_t*)add);
  else
    return nhv_fail("experts_down: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("experts_down");
  return 0;
}

// ---------------------------------------------------------------- many rows in bfloat16: the pairs sorted by expert
// The (token, expert) pairs of a step are put in the order of their experts, every expert's run filled up to whole
// tiles of TM pairs (-1 where there is none), so that a block meets one expert's matrices only: nhv_experts_sort.
// nhv_experts_grouped_gate_up and nhv_experts_grouped_down are then matrix products on the matrix cores. With tiles of
// 16 pairs (few pairs an expert) a block owns one tile of pairs and some tiles of 16 outputs; its waves share the
// inner dimension and their sums meet in LDS in the order of the waves. With tiles of 64 or 128 pairs the block's pieces of
// both operands go through LDS (experts_tiled_kernel). A pair's sums do not depend on where the sort has put it.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 ex_load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 ex_zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// One block. sorted [cap]: the pair at each place, -1 for none; tile_expert [tiles_cap]: the expert of each tile of
// TM places, -1 for a tile beyond the last.
__global__ __launch_bounds__(1024) void experts_sort_kernel(const int* __restrict__ ids, int P, int E, int TM,
                                                            int* __restrict__ sorted, int cap,
                                                            int* __restrict__ tile_expert, int tiles_cap) {
  extern __shared__ int sh[];                // counts [E], offsets [E], cursors [E]
  int* counts = sh;
  int* offsets = sh + E;
  int* cursors = sh + 2 * E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) { counts[e] = 0; cursors[e] = 0; }
  for (int i = threadIdx.x; i < cap; i += blockDim.x) sorted[i] = -1;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int tile = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = tile * TM;
      const int n = (counts[e] + TM - 1) / TM;
      for (int i = 0; i < n && tile < tiles_cap; ++i) tile_expert[tile++] = e;
    }
    for (; tile < tiles_cap; ++tile) tile_expert[tile] = -1;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < E) {
      const int at = offsets[e] + atomicAdd(&cursors[e], 1);
      if (at < cap) sorted[at] = p;
    }
  }
}

extern "C" int nhv_experts_sort(const void* ids, int P, int E, int TM, void* sorted, int cap, void* tile_expert,
                                int tiles_cap, void* stream) {
  NHV_REQUIRE(P > 0 && E > 0 && E <= 4096 && TM > 0, "experts_sort: bad sizes P=%d E=%d TM=%d", P, E, TM);
  NHV_REQUIRE(tiles_cap >= (P + TM - 1) / TM + E && cap >= tiles_cap * TM,
              "experts_sort: room for %d tiles and %d places is too little for %d pairs of %d experts", tiles_cap, cap, P, E);
  hipLaunchKernelGGL(experts_sort_kernel, dim3(1), dim3(1024), 3 * (size_t)E * sizeof(int), (hipStream_t)stream,
                     (const int*)ids, P, E, TM, (int*)sorted, cap, (int*)tile_expert, tiles_cap);
  NHV_LAUNCH_CHECK("experts_sort");
  return 0;
}

// x: GLU: the step's rows [tokens, K] (pair p reads row p / top); else one row per pair [pairs, K]. w: [experts, NA N, K].
// y: one row per pair [pairs, N]. GLU: y = act(s g) * (s u) with the pair's score s.
template <int MT, int NT, int WAVES, int UNROLL, bool GLU, typename TOut>
__global__ __launch_bounds__(64 * WAVES) void experts_grouped_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                     TOut* __restrict__ y, const int* __restrict__ sorted,
                                                                     const int* __restrict__ tile_expert,
                                                                     const float* __restrict__ scores, int top, int N, int K,
                                                                     int act) {
  constexpr int NA = GLU ? 2 : 1;
  constexpr int TILES = NA * NT;
  static_assert(MT <= WAVES, "each of the first MT waves finishes one tile of rows");
  __shared__ float red[WAVES][MT][4][64];
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;                         // the same for the whole block
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int n0 = blockIdx.y * 16 * NT;
  const bf16_t* wbase = w + (size_t)e * NA * N * K;
  const bf16_t* wrow[TILES];
  bool n_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = n0 + nt * 16 + col;
    n_ok[nt] = n < N;
#pragma unroll
    for (int na = 0; na < NA; ++na) wrow[na * NT + nt] = wbase + ((size_t)na * N + (n_ok[nt] ? n : 0)) * K;
  }
  const int* places = sorted + (size_t)blockIdx.x * 16 * MT;
  const bf16_t* xrow[MT];
  bool m_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int pair = places[mt * 16 + col];
    m_ok[mt] = pair >= 0;
    xrow[mt] = x + (size_t)(m_ok[mt] ? (GLU ? pair / top : pair) : 0) * K;
  }
  floatx4 acc[TILES][MT];
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int ksteps = (K + 31) / 32;
  for (int run = wave; run * UNROLL < ksteps; run += WAVES) {
    bf16x8 a[UNROLL][TILES], b[UNROLL][MT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k = (run * UNROLL + u) * 32 + grp * 8;
      const bool k_ok = k < K;
#pragma unroll
      for (int t = 0; t < TILES; ++t) a[u][t] = (n_ok[t % NT] && k_ok) ? ex_load8(wrow[t] + k) : ex_zero8();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = (m_ok[mt] && k_ok) ? ex_load8(xrow[mt] + k) : ex_zero8();
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][t], b[u][mt], acc[t][mt], 0, 0, 0);
  }
  // wave ``mt`` adds the waves' partial sums of tile (nt, mt) in the order of the waves and writes that tile
  const int my_pair = wave < MT ? places[wave * 16 + col] : -1;
  const float s = (GLU && scores && my_pair >= 0) ? scores[my_pair] : 1.0f;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float v[NA][4];
#pragma unroll
    for (int na = 0; na < NA; ++na) {
      __syncthreads();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j) red[wave][mt][j][lane] = acc[na * NT + nt][mt][j];
      __syncthreads();
      if (wave < MT) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float sum = 0.f;
#pragma unroll
          for (int wv = 0; wv < WAVES; ++wv) sum += red[wv][wave][j][lane];
          v[na][j] = sum;
        }
      }
    }
    if (wave < MT && my_pair >= 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + nt * 16 + grp * 4 + j;
        if (n < N) {
          float r = v[0][j];
          if (GLU) r = nhv_expert_act(s * r, act) * (s * v[NA - 1][j]);
          y[(size_t)my_pair * N + n] = (TOut)r;
        }
      }
    }
  }
}

// Tiles of 64 or 128 pairs (BM): a block of WM x WN waves owns BM pairs x BW rows of the expert's matrix (GLU: BW / 2 gate
// rows and their up rows, so BW / 2 outputs; else BW outputs) and walks over k in pieces of 64 that all its threads
// bring into LDS (the next piece is asked for, into registers, while this one is computed). A wave takes BM / 16 / WM
// tiles of pairs against BW / 16 / WN tiles of matrix rows (GLU: gate tiles and their up tiles). The larger the block's
// tile, the fewer bytes cross from L2 for a product: 64 x 128 asks for 24 KB per 2^20 multiply-adds, 128 x 256 for 48 KB
// per 2^22.
template <bool GLU, typename TOut, int BM, int BW, int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN) void experts_tiled_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                     TOut* __restrict__ y, const int* __restrict__ sorted,
                                                                     const int* __restrict__ tile_expert,
                                                                     const float* __restrict__ scores, int top, int N, int K,
                                                                     int act) {
  constexpr int THREADS = 64 * WM * WN, BK = 64, LD = BK + 8;  // (rows of 144 bytes: 16-byte pieces stay aligned, banks shift)
  constexpr int RP = THREADS / 8;            // rows that the threads bring in one pass
  constexpr int XI = BM / RP, WI = BW / RP;
  constexpr int MT = BM / 16 / WM, NT = BW / 16 / WN, NH = GLU ? NT / 2 : NT;
  constexpr int OUT = GLU ? BW / 2 : BW;     // outputs a block
  static_assert(XI >= 1 && WI >= 1 && MT >= 1 && NH >= 1, "tile sizes and waves do not fit");
  __shared__ __attribute__((aligned(16))) bf16_t xs[BM * LD];
  __shared__ __attribute__((aligned(16))) bf16_t ws[BW * LD];
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;                         // the same for the whole block
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 15, grp = lane >> 4;
  const int wm = wave / WN, wn = wave % WN;
  const int* places = sorted + (size_t)blockIdx.x * BM;
  const int n0 = blockIdx.y * OUT;
  const bf16_t* wbase = w + (size_t)e * (GLU ? 2 : 1) * N * K;
  // what this thread brings: 8 entries at k offset kc of rows r0 + RP i of x and of the matrix piece
  const int kc = (tid & 7) * 8, r0 = tid >> 3;
  const bf16_t* xp[XI];
  bool xok[XI];
#pragma unroll
  for (int i = 0; i < XI; ++i) {
    const int pair = places[r0 + RP * i];
    xok[i] = pair >= 0;
    xp[i] = x + (size_t)(xok[i] ? (GLU ? pair / top : pair) : 0) * K + kc;
  }
  const bf16_t* wp[WI];
  bool wok[WI];
#pragma unroll
  for (int i = 0; i < WI; ++i) {
    const int r = r0 + RP * i;
    const int n = GLU ? n0 + r % OUT : n0 + r;
    wok[i] = n < N;
    const size_t row = GLU ? (size_t)(r / OUT) * N + n : (size_t)n;
    wp[i] = wbase + (wok[i] ? row : 0) * K + kc;
  }
  bf16x8 xr[XI], wr[WI];
  auto ask = [&](int k0) {
    const bool k_ok = k0 + kc < K;
#pragma unroll
    for (int i = 0; i < XI; ++i) xr[i] = (xok[i] && k_ok) ? ex_load8(xp[i] + k0) : ex_zero8();
#pragma unroll
    for (int i = 0; i < WI; ++i) wr[i] = (wok[i] && k_ok) ? ex_load8(wp[i] + k0) : ex_zero8();
  };
  floatx4 acc[NT][MT];
#pragma unroll
  for (int a = 0; a < NT; ++a)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[a][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  // the rows of the matrix piece that this wave's tile a starts at: GLU: gate tiles first, then their up tiles
  auto tile_row = [&](int a) { return GLU ? (a / NH) * OUT + (wn * NH + a % NH) * 16 : (wn * NT + a) * 16; };
  ask(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();                         // the piece before is computed
#pragma unroll
    for (int i = 0; i < XI; ++i) *reinterpret_cast<bf16x8*>(&xs[(r0 + RP * i) * LD + kc]) = xr[i];
#pragma unroll
    for (int i = 0; i < WI; ++i) *reinterpret_cast<bf16x8*>(&ws[(r0 + RP * i) * LD + kc]) = wr[i];
    __syncthreads();
    if (k0 + BK < K) ask(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 32) {
      bf16x8 b[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        b[mt] = *reinterpret_cast<const bf16x8*>(&xs[((wm * MT + mt) * 16 + col) * LD + kk + grp * 8]);
#pragma unroll
      for (int a = 0; a < NT; ++a) {
        const bf16x8 af = *reinterpret_cast<const bf16x8*>(&ws[(tile_row(a) + col) * LD + kk + grp * 8]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[a][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, b[mt], acc[a][mt], 0, 0, 0);
      }
    }
  }
  // a lane holds, of every tile, four outputs (grp * 4 + j) of the pair at place (wm MT + mt) * 16 + col
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int pair = places[(wm * MT + mt) * 16 + col];
    if (pair < 0) continue;
    const float s = (GLU && scores) ? scores[pair] : 1.0f;
#pragma unroll
    for (int a = 0; a < NH; ++a)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + (wn * NH + a) * 16 + grp * 4 + j;
        if (n >= N) continue;
        if (GLU) y[(size_t)pair * N + n] = (TOut)(nhv_expert_act(s * acc[a][mt][j], act) * (s * acc[NH + a][mt][j]));
        else y[(size_t)pair * N + n] = (TOut)acc[a][mt][j];
      }
  }
}

template <bool GLU, typename TOut>
static void tiled_launch(hipStream_t s, const void* x, const void* w, void* y, const void* sorted, const void* tile_expert,
                         const void* scores, int top, int N, int K, int act, int tiles_cap, int TM) {
  const int out = GLU ? 64 : 128;
  const dim3 grid(tiles_cap, (N + out - 1) / out);
  if (TM == 128)
    hipLaunchKernelGGL((experts_tiled_kernel<GLU, TOut, 128, 128, 2, 4>), grid, dim3(512), 0, s, (const bf16_t*)x,
                       (const bf16_t*)w, (TOut*)y, (const int*)sorted, (const int*)tile_expert, (const float*)scores, top, N, K, act);
  else
    hipLaunchKernelGGL((experts_tiled_kernel<GLU, TOut, 64, 128, 1, 4>), grid, dim3(256), 0, s, (const bf16_t*)x,
                       (const bf16_t*)w, (TOut*)y, (const int*)sorted, (const int*)tile_expert, (const float*)scores, top, N, K, act);
}

template <int MT, bool GLU, typename TOut>
static void grouped_launch(hipStream_t s, const void* x, const void* w, void* y, const void* sorted, const void* tile_expert,
                           const void* scores, int top, int N, int K, int act, int tiles_cap) {
  constexpr int NT = GLU ? 2 : 4, WAVES = 8, UNROLL = 2;
  const dim3 grid(tiles_cap, (N + 16 * NT - 1) / (16 * NT));
  hipLaunchKernelGGL((experts_grouped_kernel<MT, NT, WAVES, UNROLL, GLU, TOut>), grid, dim3(64 * WAVES), 0, s,
                     (const bf16_t*)x, (const bf16_t*)w, (TOut*)y, (const int*)sorted, (const int*)tile_expert,
                     (const float*)scores, top, N, K, act);
}

// u [pairs, F] bfloat16 from the step's rows h [tokens, W]; TM: 16, 64 or 128 places a tile (as the sort was told).
extern "C" int nhv_experts_grouped_gate_up(const void* h, const void* gate_up, void* u, const void* sorted,
                                           const void* tile_expert, const void* scores, int top, int W, int F, int act,
                                           int TM, int tiles_cap, void* stream) {
  NHV_REQUIRE(W > 0 && F > 0 && W % 8 == 0 && top > 0 && tiles_cap > 0 && (TM == 16 || TM == 64 || TM == 128),
              "experts_grouped_gate_up: bad sizes W=%d (a multiple of 8) F=%d top=%d TM=%d", W, F, top, TM);
  NHV_REQUIRE((F + 31) / 32 <= 65535, "experts_grouped_gate_up: F=%d is beyond this kernel's grid", F);
  hipStream_t s = (hipStream_t)stream;
  if (TM >= 64) tiled_launch<true, bf16_t>(s, h, gate_up, u, sorted, tile_expert, scores, top, F, W, act, tiles_cap, TM);
  else grouped_launch<1, true, bf16_t>(s, h, gate_up, u, sorted, tile_expert, scores, top, F, W, act, tiles_cap);
  NHV_LAUNCH_CHECK("experts_grouped_gate_up");
  return 0;
}

// y [pairs, W] float from u [pairs, F] bfloat16.
extern "C" int nhv_experts_grouped_down(const void* u, const void* down, void* y, const void* sorted,
                                        const void* tile_expert, int W, int F, int TM, int tiles_cap, void* stream) {
  NHV_REQUIRE(W > 0 && F > 0 && F % 8 == 0 && tiles_cap > 0 && (TM == 16 || TM == 64 || TM == 128),
              "experts_grouped_down: bad sizes W=%d F=%d (a multiple of 8) TM=%d", W, F, TM);
  NHV_REQUIRE((W + 63) / 64 <= 65535, "experts_grouped_down: W=%d is beyond this kernel's grid", W);
  hipStream_t s = (hipStream_t)stream;
  if (TM >= 64) tiled_launch<false, float>(s, u, down, y, sorted, tile_expert, nullptr, 1, W, F, 0, tiles_cap, TM);
  else grouped_launch<1, false, float>(s, u, down, y, sorted, tile_expert, nullptr, 1, W, F, 0, tiles_cap);
  NHV_LAUNCH_CHECK("experts_grouped_down");
  return 0;
}

// out[t, n] = sum over j < top (rising) of [weights[t, j]] y[t * top + j, n], [plus add[t, n]]
__global__ void experts_combine_kernel(const float* __restrict__ y, bf16_t* __restrict__ out, int W, int top, size_t total,
                                       const float* __restrict__ weights, const bf16_t* __restrict__ add) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / W, n = i % W;
    float sum = 0.f;
    for (int j = 0; j < top; ++j) sum += weights ? weights[t * top + j] * y[(t * top + j) * W + n] : y[(t * top + j) * W + n];
    out[i] = (bf16_t)(add ? sum + (float)add[i] : sum);
  }
}

extern "C" int nhv_experts_combine(const void* y, void* out, int T, int W, int top, const void* weights, const void* add,
                                   void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && top > 0, "experts_combine: bad sizes T=%d W=%d top=%d", T, W, top);
  const size_t total = (size_t)T * W;
  const int blocks = (int)((total + 255) / 256 > 65535 * 4 ? 65535 * 4 : (total + 255) / 256);
  hipLaunchKernelGGL(experts_combine_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const float*)y, (bf16_t*)out,
                     W, top, total, (const float*)weights, (const bf16_t*)add);
  NHV_LAUNCH_CHECK("experts_combine");
  return 0;
}
