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
};
