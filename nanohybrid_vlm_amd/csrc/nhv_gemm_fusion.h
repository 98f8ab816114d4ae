// What a few-rows matrix product may take over from the kernels around it (all null: a plain product).
//
// After the product: its result is added to the residual stream in the product's own kernel. The kernel reads
// and rewrites `residual`; every tile of 16 outputs leaves its share of each row's sum of squares in
// `ss_out[row][tile]` (added up in a fixed order by whoever norms the rows); and `sum_out` gets the sum times the
// weight of the norm that follows (`next_w`, by column), rounded to bfloat16: the norm's product with its weight is
// done here, its scaling of the rows is left to the reader.
// Before the product: x is such a sum (already times the norm's weight) whose rows still lack their scales
// r[m] = 1 / sqrt(sum over tiles of ss_in[m][.] / K + eps). The product is linear in x, so the scale is applied to
// the finished sums: y[m][n] = r[m] * (x[m] . w[n]) (+ bias), in float.
#pragma once
#include "nhv_common.h"

struct NhvGemmFusion {
  void* residual;        // [M, N] float or bfloat16, read and rewritten
  int residual_f32;
  bf16_t* sum_out;       // [M, N]: (residual + product) * next_w, rounded
  float* ss_out;         // [M, tiles of N]
  const void* next_w;    // [N] float or bfloat16; null: the sum goes out as it is
  int next_w_f32;
  const float* ss_in;    // [M, tiles_in]
  int tiles_in;
  float eps;
  int glu_act;           // what a gated product passes its gate through: 0 SiLU, 1 the tanh form of GELU
  int plain_act;         // what a product without a gate passes its result through (after the bias): 0 nothing, 1 SiLU,
                         // 2 the tanh form of GELU, 3 the square of max(z, 0)
};

__device__ __forceinline__ float nhv_plain_act(float z, int act) {
  if (act == 3) {
    const float r = fmaxf(z, 0.f);
    return r * r;
  }
  if (act == 2) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  if (act == 1) return z / (1.0f + expf(-z));
  return z;
}

__device__ __forceinline__ float nhv_glu_gate(float z, int act) {
  if (act == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z / (1.0f + expf(-z));
}
