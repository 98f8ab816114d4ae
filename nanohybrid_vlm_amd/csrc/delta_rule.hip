// The gated delta rule: a recurrent mixer whose state is one matrix S[D, E] per head and request,
//   S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t,
// with a decay g_t per key channel (or one per head: ``Dd`` = 1 below), preceded by short causal convolutions over time
// on q, k and v.
// Four kernels, the same for prompt portions and for single decoded tokens:
//  - nhv_delta_prepare: per token, the convolutions (earlier inputs come from the step's own rows or from the
//    request's kept inputs), SiLU, unit length per head for q and k, the decays from their linear part, beta;
//  - nhv_conv_state_update: per request, the last taps - 1 inputs are kept for the next step;
//  - nhv_delta_rule: per (request, head, tile of value columns), the recurrence over the step's tokens in order,
//    from the request's state (zero for a request that starts at position 0) and back into it;
//  - nhv_gated_head_norm: per (token, head), o over its root mean square, times a weight, times sigmoid(gate) or
//    gate sigmoid(gate).
// Everything here is float: the state, the decays, the unit vectors, the sums. A column of S (one value channel)
// never meets another column, so a block owns a tile of columns, a column belongs to R adjacent lanes that hold D / R
// entries each, and the two sums over D per token are taken with lane shuffles; the tokens' vectors come through
// LDS a tile of tokens ahead. A request without tokens in the step is left alone.
#include "nhv_common.h"
#include <math.h>

#define NHV_MAX_TAPS 16

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---------------------------------------------------------------- per token: what enters the recurrence
// proj[T, ld]: q (G D) | k (G D) | v (H E) | beta (H) as the projection left them. taps[C, n], C = 2 G D + H E, last
// column for the token itself. kept[slots, C, n - 1]: the inputs at the n - 1 positions before the request's first
// token of this step. a_lin: the decays' linear part, rows of H Dd floats ``a_ld`` apart (a tensor of its own, or
// columns of a float projection); decay_out[T, H Dd]: the decays (it may be a_lin itself where that is dense); Dd = D
// (a decay per key channel) or 1 (one per head); dt_bias[H Dd].
// One wave per (token, unit); the units of a token are its 2 G query and key heads (D channels each), its H value
// heads (E channels), its H heads of decays (D channels) and its H betas (one unit).
template <typename TI>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    const TI* __restrict__ proj, int ld, const float* __restrict__ taps, int n_taps, const float* __restrict__ kept,
    const float* a_lin, long long a_ld, float* decay_out, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const int* __restrict__ token_req, const int* __restrict__ positions, const int* __restrict__ cu,
    const int* __restrict__ state_slots, float* __restrict__ q_out, float* __restrict__ k_out, float* __restrict__ v_out,
    float* __restrict__ beta_out, int H, int G, int D, int E, int Dd) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int unit = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int n_units = 2 * G + 2 * H + 1;
  if (unit >= n_units) return;
  const int C = 2 * G * D + H * E;
  if (unit == n_units - 1) {
    for (int h = lane; h < H; h += NHV_WAVE) beta_out[(size_t)t * H + h] = sigmoid_f(to_f32(proj[(size_t)t * ld + C + h]));
    return;
  }
  if (unit >= 2 * G + H) {
    const int h = unit - 2 * G - H;
    const float rate = expf(a_log[h]);
    for (int d = lane; d < Dd; d += NHV_WAVE) {
      decay_out[(size_t)t * H * Dd + h * Dd + d] = expf(-rate * softplus_f(a_lin[(size_t)t * a_ld + h * Dd + d] + dt_bias[h * Dd + d]));
    }
    return;
  }
  const int req = token_req[t];
  const int i_in_step = t - cu[req];         // tokens of this request before this one in the step
  const int pos = positions[t];
  const float* mine = kept + (size_t)state_slots[req] * C * (n_taps - 1);
  const bool is_v = unit >= 2 * G;
  const int size = is_v ? E : D;
  const int c0 = is_v ? 2 * G * D + (unit - 2 * G) * E : unit * D;
  float vals[16];                            // (heads of up to 1024 channels)
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int d = lane + i * NHV_WAVE;
    vals[i] = 0.f;
    if (d < size) {
      const int c = c0 + d;
      float sum = 0.f;
      for (int j = 0; j < n_taps; ++j) {     // the input j positions back meets the tap n - 1 - j
        if (pos - j < 0) break;
        const float x = j <= i_in_step ? to_f32(proj[(size_t)(t - j) * ld + c])
                                       : mine[(size_t)c * (n_taps - 1) + (n_taps - 1) + i_in_step - j];
        sum = fmaf(taps[(size_t)c * n_taps + n_taps - 1 - j], x, sum);
      }
      vals[i] = silu_f(sum);
      ss = fmaf(vals[i], vals[i], ss);
    }
  }
  float r = 1.0f;
  float* dst = v_out + (size_t)t * H * E + (c0 - 2 * G * D);
  if (!is_v) {
    // unit length (the sum of squares plus 1e-6 under the root); q also times D^(-1/2)
    r = (unit < G ? 1.0f / sqrtf((float)D) : 1.0f) / sqrtf(wave_sum(ss) + 1e-6f);
    dst = unit < G ? q_out + ((size_t)t * G + unit) * D : k_out + ((size_t)t * G + unit - G) * D;
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int d = lane + i * NHV_WAVE;
    if (d < size) dst[d] = vals[i] * r;
  }
}

extern "C" int nhv_delta_prepare(const void* proj, int proj_dtype, int ld, const void* taps, int n_taps, const void* kept,
                                 const void* a_lin, long long a_ld, void* decay_out, const void* dt_bias, const void* a_log, const void* token_req,
                                 const void* positions, const void* cu, const void* state_slots, void* q_out, void* k_out,
                                 void* v_out, void* beta_out, int T, int H, int G, int D, int E, int decay_dim, void* stream) {
  NHV_REQUIRE(T > 0 && H > 0 && G > 0 && D > 0 && E > 0 && H % G == 0, "delta_prepare: bad sizes T=%d H=%d G=%d D=%d E=%d", T, H, G, D, E);
  NHV_REQUIRE(decay_dim == D || decay_dim == 1, "delta_prepare: %d decays a head (one, or one per key channel: %d)", decay_dim, D);
  NHV_REQUIRE(n_taps >= 1 && n_taps <= NHV_MAX_TAPS, "delta_prepare: %d taps (1 to %d are taken)", n_taps, NHV_MAX_TAPS);
  NHV_REQUIRE(D <= 1024 && E <= 1024 && 2 * G + 2 * H + 1 <= 4 * 65535, "delta_prepare: D=%d, E=%d (up to 1024 each), %d heads", D, E, H);
  const int C = 2 * G * D + H * E;
  NHV_REQUIRE(ld >= C + H && a_ld >= (long long)H * decay_dim, "delta_prepare: rows of %d entries for %d, decays' rows of %lld for %d", ld, C + H,
              a_ld, H * decay_dim);
  const int n_units = 2 * G + 2 * H + 1;
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(TI)                                                                                                    \
  hipLaunchKernelGGL(delta_prepare_kernel<TI>, dim3(T, (n_units + 3) / 4), dim3(256), 0, s, (const TI*)proj, ld,      \
                     (const float*)taps, n_taps, (const float*)kept, (const float*)a_lin, a_ld, (float*)decay_out,    \
                     (const float*)dt_bias,                                                                           \
                     (const float*)a_log, (const int*)token_req, (const int*)positions, (const int*)cu,               \
                     (const int*)state_slots, (float*)q_out, (float*)k_out, (float*)v_out, (float*)beta_out, H, G, D, E,  \
                     decay_dim)
  if (proj_dtype == NHV_F32) LAUNCH(float);
  else if (proj_dtype == NHV_BF16) LAUNCH(bf16_t);
  else return nhv_fail("delta_prepare: unknown dtype %d", proj_dtype);
#undef LAUNCH
  NHV_LAUNCH_CHECK("delta_prepare");
  return 0;
}

// ---------------------------------------------------------------- per request: the inputs kept for the next step
// After a step that brought a request n tokens from position ``start`` on, kept[., c, s] is the input at position
// start + n - (taps - 1) + s: one of the step's rows, or what was kept before (nothing, i.e. zero, before position 0).
// A thread owns one channel of one request, reads all it needs and then writes.
template <typename TI>
__global__ void conv_state_update_kernel(const TI* __restrict__ proj, int ld, float* __restrict__ kept, int n_taps,
                                         const int* __restrict__ positions, const int* __restrict__ cu,
                                         const int* __restrict__ state_slots, int C) {
  const int req = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int first = cu[req], n = cu[req + 1] - first;
  if (n <= 0 || c >= C) return;
  const int start = positions[first];
  float* mine = kept + ((size_t)state_slots[req] * C + c) * (n_taps - 1);
  float next[NHV_MAX_TAPS];
  for (int s = 0; s < n_taps - 1; ++s) {
    const int rel = n - (n_taps - 1) + s;     // which of the step's tokens, if not negative
    if (rel >= 0) next[s] = to_f32(proj[(size_t)(first + rel) * ld + c]);
    else next[s] = start + rel >= 0 ? mine[n + s] : 0.f;
  }
  for (int s = 0; s < n_taps - 1; ++s) mine[s] = next[s];
}

extern "C" int nhv_conv_state_update(const void* proj, int proj_dtype, int ld, void* kept, int n_taps, const void* positions,
                                     const void* cu, const void* state_slots, int B, int C, void* stream) {
  NHV_REQUIRE(B > 0 && C > 0 && ld >= C && B <= 65535, "conv_state_update: bad sizes B=%d C=%d ld=%d", B, C, ld);
  NHV_REQUIRE(n_taps >= 1 && n_taps <= NHV_MAX_TAPS, "conv_state_update: %d taps (1 to %d are taken)", n_taps, NHV_MAX_TAPS);
  if (n_taps == 1) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((C + 255) / 256, B);
  if (proj_dtype == NHV_F32)
    hipLaunchKernelGGL(conv_state_update_kernel<float>, grid, dim3(256), 0, s, (const float*)proj, ld, (float*)kept, n_taps,
                       (const int*)positions, (const int*)cu, (const int*)state_slots, C);
  else if (proj_dtype == NHV_BF16)
    hipLaunchKernelGGL(conv_state_update_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)proj, ld, (float*)kept, n_taps,
                       (const int*)positions, (const int*)cu, (const int*)state_slots, C);
  else return nhv_fail("conv_state_update: unknown dtype %d", proj_dtype);
  NHV_LAUNCH_CHECK("conv_state_update");
  return 0;
}

// ---------------------------------------------------------------- the recurrence
// state[slots, H, E, D]: a column of S lies contiguous. Thread (column e, part r) of a block holds S[r DR .. r DR + DR, e];
// the R parts of a column are adjacent lanes (R a power of two, at most 64). Entries beyond D (where D is no multiple
// of R DR) are zeros that change nothing. The tokens' vectors (q, k, the decays: D floats each; the block's columns of
// v; beta) come through LDS in tiles of ``tile`` tokens, two buffers: the next tile's loads are under way in registers
// while this tile is computed, and are stored when it is done; one barrier a tile. A token then costs its
// arithmetic and two sums over R lanes, not a trip to memory.
#define NHV_DELTA_STAGE 24     // floats a thread can hold of the next tile (a tile has at most 256 * this many)

// The sum of x over the R adjacent lanes of a column (R a power of two, the groups aligned), in every one of them.
// Within a row of 16 lanes the partners are reached by lane permutations inside the instruction itself (the two
// exchanges inside a group of four; then, all four being equal, the mirror images within eight and within sixteen
// lanes); only beyond sixteen lanes do values cross through the permute unit.
template <int R>
__device__ __forceinline__ float column_sum(float x) {
#define NHV_DPP_ADD(ctrl) x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), ctrl, 0xf, 0xf, true))
  if (R > 1) NHV_DPP_ADD(0xB1);        // quad_perm [1, 0, 3, 2]
  if (R > 2) NHV_DPP_ADD(0x4E);        // quad_perm [2, 3, 0, 1]
  if (R > 4) NHV_DPP_ADD(0x141);       // row_half_mirror
  if (R > 8) NHV_DPP_ADD(0x140);       // row_mirror
#undef NHV_DPP_ADD
  if (R > 16) x += __shfl_xor(x, 16, NHV_WAVE);
  if (R > 32) x += __shfl_xor(x, 32, NHV_WAVE);
  return x;
}

template <int DR, int R, bool DIRECT>
__global__ __launch_bounds__(256) void delta_rule_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, const float* __restrict__ decay,
    const float* __restrict__ beta, float* __restrict__ state, float* __restrict__ out, const int* __restrict__ positions,
    const int* __restrict__ cu, const int* __restrict__ state_slots, int H, int G, int D, int E, int cols, int tile, int Dd) {
  extern __shared__ __attribute__((aligned(16))) float staged[];   // 2 buffers of tile * row floats, row = 3 Dp + cols + 1 (rounded up to 4), Dp = R DR
  const int req = blockIdx.z, h = blockIdx.y;
  const int first = cu[req], end = cu[req + 1];
  if (end <= first) return;                  // (the same for the whole block)
  const int e0 = blockIdx.x * cols;
  const int e = e0 + threadIdx.x / R;
  const int r = threadIdx.x % R;
  const int d0 = r * DR;
  const bool column = e < E;
  const int g = h / (H / G);
  const int Dp = R * DR;
  const int row = 3 * Dp + ((cols + 1 + 3) & ~3);       // (a multiple of four floats: every token's vectors can be read four at a time)
  const int n_threads = blockDim.x;
  const int my_col = threadIdx.x / R;
  const bool writes = r == 0 && column;
  float* out_col = out + (size_t)h * E + (column ? e : 0);
  float S[DR];
  float* mine = state + (((size_t)state_slots[req] * H + h) * E + (column ? e : 0)) * D;
  const bool fresh = positions[first] == 0;
  const bool whole4 = (D & 3) == 0;          // (then a lane's entries lie inside D four at a time, and aligned)
#pragma unroll
  for (int i = 0; i < DR; i += 4) {
    if (whole4) {
      const float4 s4 = (!fresh && column && d0 + i < D) ? *reinterpret_cast<const float4*>(mine + d0 + i) : float4{0.f, 0.f, 0.f, 0.f};
      S[i] = s4.x; S[i + 1] = s4.y; S[i + 2] = s4.z; S[i + 3] = s4.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) S[i + j] = (!fresh && column && d0 + i + j < D) ? mine[d0 + i + j] : 0.f;
    }
  }
  if (DIRECT) {
    // a step of one or two tokens a request (decoding): the token's vectors come straight from memory, this lane's
    // share of them; nothing goes through LDS and the block meets at no barrier
    for (int t = first; t < end; ++t) {
      const float* qr = q + ((size_t)t * G + g) * D;
      const float* kr = k + ((size_t)t * G + g) * D;
      const float* gr = decay + ((size_t)t * H + h) * Dd;
      const bool one_decay = Dd == 1;      // (one number a head: every key channel decays alike)
      float cq[DR], ck[DR];
      float k_s = 0.f, q_s = 0.f, q_k = 0.f;
#pragma unroll
      for (int i = 0; i < DR; i += 4) {
        float qv[4], kv[4], gv[4];
        if (whole4 && d0 + i < D) {
          const float4 q4 = *reinterpret_cast<const float4*>(qr + d0 + i), k4 = *reinterpret_cast<const float4*>(kr + d0 + i);
          const float g1 = one_decay ? gr[0] : 0.f;
          const float4 g4 = one_decay ? float4{g1, g1, g1, g1} : *reinterpret_cast<const float4*>(gr + d0 + i);
          qv[0] = q4.x; qv[1] = q4.y; qv[2] = q4.z; qv[3] = q4.w;
          kv[0] = k4.x; kv[1] = k4.y; kv[2] = k4.z; kv[3] = k4.w;
          gv[0] = g4.x; gv[1] = g4.y; gv[2] = g4.z; gv[3] = g4.w;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const bool ok = !whole4 && d0 + i + j < D;
            qv[j] = ok ? qr[d0 + i + j] : 0.f;
            kv[j] = ok ? kr[d0 + i + j] : 0.f;
            gv[j] = ok ? gr[one_decay ? 0 : d0 + i + j] : 0.f;
          }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          cq[i + j] = qv[j];
          ck[i + j] = kv[j];
          S[i + j] *= gv[j];
          k_s = fmaf(kv[j], S[i + j], k_s);
          q_s = fmaf(qv[j], S[i + j], q_s);
          q_k = fmaf(qv[j], kv[j], q_k);
        }
      }
      const float cv = column ? v[((size_t)t * H + h) * E + e] : 0.f, cb = beta[(size_t)t * H + h];
      k_s = column_sum<R>(k_s);
      q_s = column_sum<R>(q_s);
      q_k = column_sum<R>(q_k);
      const float u = cb * (cv - k_s);
      if (r == 0 && column) out[((size_t)t * H + h) * E + e] = fmaf(q_k, u, q_s);
#pragma unroll
      for (int i = 0; i < DR; ++i) S[i] = fmaf(ck[i], u, S[i]);
    }
  } else {

  // what this thread brings of a tile: entry x of the tile's tile * row floats, x = threadIdx.x + j * n_threads. Which
  // token of the tile and which number of it that is does not change from tile to tile: worked out once.
  float hold[NHV_DELTA_STAGE];
  const float* src[NHV_DELTA_STAGE];         // where entry j of the tile that begins at token 0 lies (null: a zero)
  int stride[NHV_DELTA_STAGE], tok_of[NHV_DELTA_STAGE];
#pragma unroll
  for (int j = 0; j < NHV_DELTA_STAGE; ++j) {
    const int x = threadIdx.x + j * n_threads;
    const int tt = x / row, c = x % row;
    tok_of[j] = tt;
    src[j] = nullptr;
    stride[j] = 0;
    if (tt < tile) {
      if (c < 3 * Dp) {
        const int which = c / Dp, d = c % Dp;
        if (d < D) {
          src[j] = which == 0 ? q + ((size_t)tt * G + g) * D + d : which == 1 ? k + ((size_t)tt * G + g) * D + d
                                                                              : decay + ((size_t)tt * H + h) * Dd + (Dd == 1 ? 0 : d);
          stride[j] = which == 2 ? H * Dd : G * D;
        }
      } else if (c < 3 * Dp + cols) {
        const int ee = e0 + c - 3 * Dp;
        if (ee < E) {
          src[j] = v + ((size_t)tt * H + h) * E + ee;
          stride[j] = H * E;
        }
      } else {
        src[j] = beta + (size_t)tt * H + h;
        stride[j] = H;
      }
    }
  }
  auto ask = [&](int t0, int n) {
#pragma unroll
    for (int j = 0; j < NHV_DELTA_STAGE; ++j)
      hold[j] = (src[j] != nullptr && tok_of[j] < n) ? src[j][(size_t)t0 * stride[j]] : 0.f;
  };
  // (LDS is always named through the array itself, so that the compiler knows every such access for what it is:
  // a read through a plain pointer would wait for the global loads that are under way as well)
  auto put = [&](int buf, int n) {
#pragma unroll
    for (int j = 0; j < NHV_DELTA_STAGE; ++j)
      if (tok_of[j] < n) staged[buf + threadIdx.x + j * n_threads] = hold[j];
  };
  int n_here = min(tile, end - first);
  ask(first, n_here);
  put(0, n_here);
  __syncthreads();
  int cur = 0;
  for (int t0 = first; t0 < end; t0 += tile) {
    const int n = min(tile, end - t0);
    const int n_next = min(tile, end - t0 - tile);
    if (n_next > 0) ask(t0 + tile, n_next);
    const int buf = cur * tile * row;
    // a token's vectors are read from LDS into registers while the token before it is computed
    float nq[DR], nk[DR], ng[DR], nv, nb;
    auto take = [&](int tok) {
#pragma unroll
      for (int i = 0; i < DR; i += 4) {
        const float4 q4 = *reinterpret_cast<const float4*>(&staged[tok + d0 + i]);
        const float4 k4 = *reinterpret_cast<const float4*>(&staged[tok + Dp + d0 + i]);
        const float4 g4 = *reinterpret_cast<const float4*>(&staged[tok + 2 * Dp + d0 + i]);
        nq[i] = q4.x; nq[i + 1] = q4.y; nq[i + 2] = q4.z; nq[i + 3] = q4.w;
        nk[i] = k4.x; nk[i + 1] = k4.y; nk[i + 2] = k4.z; nk[i + 3] = k4.w;
        ng[i] = g4.x; ng[i + 1] = g4.y; ng[i + 2] = g4.z; ng[i + 3] = g4.w;
      }
      nv = staged[tok + 3 * Dp + my_col];
      nb = staged[tok + 3 * Dp + cols];
    };
    take(buf);
    for (int i_t = 0; i_t < n; ++i_t) {
      // with S' = diag(g) S:  u = beta (v - k . S'),  o = q . (S' + k u) = q . S' + (q . k) u: the three sums over D are
      // taken together, so a token waits for one exchange between the lanes of its column, not two. (The read-out's
      // share joined in the lane first and summed after u, one sum fewer: 798 against 756 us for 2,048 tokens; a wave
      // alone waits for the second exchange as it does for the first.)
      float ck[DR];
      float k_s = 0.f, q_s = 0.f, q_k = 0.f;
      const float cv = nv, cb = nb;
#pragma unroll
      for (int i = 0; i < DR; ++i) {
        ck[i] = nk[i];
        S[i] *= ng[i];
        k_s = fmaf(nk[i], S[i], k_s);
        q_s = fmaf(nq[i], S[i], q_s);
        q_k = fmaf(nq[i], nk[i], q_k);
      }
      if (i_t + 1 < n) take(buf + (i_t + 1) * row);
      k_s = column_sum<R>(k_s);
      q_s = column_sum<R>(q_s);
      q_k = column_sum<R>(q_k);
      const float u = cb * (cv - k_s);
      const float read = fmaf(q_k, u, q_s);
#pragma unroll
      for (int i = 0; i < DR; ++i) S[i] = fmaf(ck[i], u, S[i]);
      if (writes) out_col[(size_t)(t0 + i_t) * H * E] = read;
    }
    if (n_next > 0) put((cur ^ 1) * tile * row, n_next);
    __syncthreads();
    cur ^= 1;
  }
  }
  if (column) {
#pragma unroll
    for (int i = 0; i < DR; i += 4) {
      if (whole4) {
        if (d0 + i < D) *reinterpret_cast<float4*>(mine + d0 + i) = float4{S[i], S[i + 1], S[i + 2], S[i + 3]};
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (d0 + i + j < D) mine[d0 + i + j] = S[i + j];
      }
    }
  }
}

extern "C" int nhv_delta_rule(const void* q, const void* k, const void* v, const void* decay, const void* beta, void* state,
                              void* out, const void* positions, const void* cu, const void* state_slots, int B, int H, int G,
                              int D, int E, int max_q_len, int decay_dim, void* stream) {
  NHV_REQUIRE(B > 0 && H > 0 && G > 0 && D > 0 && E > 0 && H % G == 0, "delta_rule: bad sizes B=%d H=%d G=%d D=%d E=%d", B, H, G, D, E);
  NHV_REQUIRE(decay_dim == D || decay_dim == 1, "delta_rule: %d decays a head (one, or one per key channel: %d)", decay_dim, D);
  NHV_REQUIRE(D <= 1024 && B <= 65535 && H <= 65535, "delta_rule: D=%d (up to 1024), B=%d, H=%d (up to 65535)", D, B, H);
  // entries a lane: 4, or what keeps a column within the 64 lanes of a wave. (A token's time is what a wave has to
  // issue for it, not its arithmetic: 2,048 tokens of 16 heads of 128 x 128 took 890 us with 8 entries a lane and 700 us
  // with 4, which have one exchange more between the lanes and half the reads from LDS a lane.)
  // With few requests and heads the chip is far from full and 4 entries a lane are the faster; from about two waves a
  // SIMD on (4 requests of 2,048 tokens: 1,040 us with 8 entries a lane, 1,450 us with 4) the lanes' own work counts.
  const long long lanes_at_8 = (long long)B * H * E * ((D + 7) / 8);
  const int dr = D > 512 ? 16 : ((D > 256 || (D >= 64 && lanes_at_8 >= 100000)) ? 8 : 4);
  int R = 1;
  while (R * dr < D) R <<= 1;
  int cols = 256 / R;
  if (cols < 1) cols = 1;
  if (cols > E) cols = E;
  const int n_threads = cols * R;
  const int row = 3 * R * dr + ((cols + 1 + 3) & ~3);
  // tokens a tile: what the threads can hold of the next tile, at most 16, no more than the longest portion
  int tile = n_threads * NHV_DELTA_STAGE / row;
  if (tile > 16) tile = 16;
  if (tile > max_q_len) tile = max_q_len;
  if (tile < 1) tile = 1;
  NHV_REQUIRE(row <= n_threads * NHV_DELTA_STAGE, "delta_rule: a token's %d floats do not fit the block's staging", row);
  const bool direct = max_q_len <= 2;
  const size_t lds = direct ? 0 : 2 * (size_t)tile * row * sizeof(float);
  const dim3 grid((E + cols - 1) / cols, H, B), block(n_threads);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH_AS(DRV, RV, DIR)                                                                                       \
  hipLaunchKernelGGL((delta_rule_kernel<DRV, RV, DIR>), grid, block, lds, s, (const float*)q, (const float*)k,        \
                     (const float*)v, (const float*)decay, (const float*)beta, (float*)state, (float*)out,            \
                     (const int*)positions, (const int*)cu, (const int*)state_slots, H, G, D, E, cols, tile, decay_dim)
#define LAUNCH(DRV, RV)               \
  do {                                \
    if (direct) LAUNCH_AS(DRV, RV, true); \
    else LAUNCH_AS(DRV, RV, false);   \
  } while (0)
#define BY_R(DRV)                          \
  switch (R) {                             \
    case 1: LAUNCH(DRV, 1); break;         \
    case 2: LAUNCH(DRV, 2); break;         \
    case 4: LAUNCH(DRV, 4); break;         \
    case 8: LAUNCH(DRV, 8); break;         \
    case 16: LAUNCH(DRV, 16); break;       \
    case 32: LAUNCH(DRV, 32); break;       \
    default: LAUNCH(DRV, 64); break;       \
  }
  if (dr == 16) { BY_R(16) } else if (dr == 8) { BY_R(8) } else { BY_R(4) }
#undef BY_R
#undef LAUNCH
#undef LAUNCH_AS
  NHV_LAUNCH_CHECK("delta_rule");
  return 0;
}

// ---------------------------------------------------------------- the read-out's norm and gate
// y[t, h, e] = o[t, h, e] / sqrt(mean over e of o^2 + eps) * w[e] * f(gate[t, h, e]) (the gates' rows ``gate_ld`` floats apart), f the sigmoid (gate_act 0) or
// z sigmoid(z) (1); one wave per (t, h).
template <typename TO>
__global__ void gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate, long long gate_ld, int H,
                                       const float* __restrict__ w,
                                       TO* __restrict__ y, int E, float eps, int n_items, int gate_act) {
  const int item = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= n_items) return;
  const int lane = threadIdx.x & 63;
  const float* src = o + (size_t)item * E;
  float ss = 0.f;
  for (int e = lane; e < E; e += NHV_WAVE) ss = fmaf(src[e], src[e], ss);
  const float r = 1.0f / sqrtf(wave_sum(ss) / (float)E + eps);
  for (int e = lane; e < E; e += NHV_WAVE)
  {
    const float z = gate[(size_t)(item / H) * gate_ld + (size_t)(item % H) * E + e];
    y[(size_t)item * E + e] = from_f32<TO>(src[e] * r * w[e] * (gate_act == 1 ? silu_f(z) : sigmoid_f(z)));
  }
}

extern "C" int nhv_gated_head_norm(const void* o, const void* gate, long long gate_ld, const void* w, void* y, int T, int H, int E, float eps,
                                   int y_dtype, int gate_act, void* stream) {
  NHV_REQUIRE(gate_ld >= (long long)H * E, "gated_head_norm: gate rows %lld apart for %d entries", gate_ld, H * E);
  NHV_REQUIRE(gate_act == 0 || gate_act == 1, "gated_head_norm: gate activation %d (0: sigmoid, 1: SiLU)", gate_act);
  NHV_REQUIRE(T > 0 && H > 0 && E > 0 && (long long)T * H < (1ll << 31), "gated_head_norm: bad sizes T=%d H=%d E=%d", T, H, E);
  const int n_items = T * H;
  const unsigned blocks = (unsigned)((n_items + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (y_dtype == NHV_F32)
    hipLaunchKernelGGL(gated_head_norm_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)o, (const float*)gate,
                       gate_ld, H, (const float*)w, (float*)y, E, eps, n_items, gate_act);
  else if (y_dtype == NHV_BF16)
    hipLaunchKernelGGL(gated_head_norm_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (const float*)o, (const float*)gate,
                       gate_ld, H, (const float*)w, (bf16_t*)y, E, eps, n_items, gate_act);
  else return nhv_fail("gated_head_norm: unknown dtype %d", y_dtype);
  NHV_LAUNCH_CHECK("gated_head_norm");
  return 0;
}
