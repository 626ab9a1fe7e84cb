// Adam update shared by the optimiser kernels (optim.hip) and the decoder weight-gradient kernel that
// applies it in place (backward.hip).  torch.optim.Adam semantics: bias-corrected first / second moments,
// no weight decay, no amsgrad (the reference builds its optimizer in clt/training/trainer.py:290-312):
//   m = b1 m + (1 - b1) g;  v = b2 v + (1 - b2) g^2
//   p -= (lr / (1 - b1^step)) * m / (sqrt(v) / sqrt(1 - b2^step) + eps)
// computed in fp32 and rounded once to the parameter dtype.
#pragma once
#include <cmath>
#include "clt_common.h"

struct AdamCoef { float b1, b2, step_size, inv_sqrt_bc2, eps; };

// The sequence of roundings is spelled out with fmaf so that every kernel that inlines this produces
// the same bits for the same inputs.
__device__ __forceinline__ float adam_update(float p, float g, float &m, float &v, const AdamCoef &c) {
  m = fmaf(c.b1, m, __fmul_rn(1.0f - c.b1, g));
  v = fmaf(c.b2, v, __fmul_rn(__fmul_rn(1.0f - c.b2, g), g));
  const float denom = fmaf(sqrtf(v), c.inv_sqrt_bc2, c.eps);
  return fmaf(-c.step_size, __fdiv_rn(m, denom), p);
}

static inline AdamCoef adam_coef(double lr, double b1, double b2, double eps, int64_t step) {
  AdamCoef c;
  c.b1 = (float)b1; c.b2 = (float)b2; c.eps = (float)eps;
  c.step_size = (float)(lr / (1.0 - pow(b1, (double)step)));
  c.inv_sqrt_bc2 = (float)(1.0 / sqrt(1.0 - pow(b2, (double)step)));
  return c;
}
