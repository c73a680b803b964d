// Optimiser steps on device arrays: SGD (momentum, dampening, Nesterov, weight decay) and
// Adam / AdamW (optionally AMSGrad), one fused HBM-bound kernel per parameter.
//
// The reference evaluates these updates as chains of NumPy array expressions
// (src/tortto/optim/_functional.py:4-119).  Every product and sum there is rounded to float32
// on its own, and Adam's denominator is formed in float64 (a float32 array divided by the
// float64 scalar sqrt(bias_correction2), :58-63, :108-113); the kernels keep exactly those
// roundings (one operation per rounding, no contraction into FMA) so that a long training
// run follows the reference's trajectory bit for bit.
#include "tt_common.h"

#include <math.h>

// The compiler would fuse a product and the sum that follows it into one FMA (one rounding
// instead of two) -- also through the __fmul_rn / __fadd_rn intrinsics, which are plain operators
// defined in a header.  Contraction is switched off for this file and the arithmetic below goes
// through these two helpers, which are compiled under that setting.
#pragma clang fp contract(off)

namespace {

__device__ __forceinline__ float mul(float a, float b) { return a * b; }
__device__ __forceinline__ float add(float a, float b) { return a + b; }

constexpr int kThreads = 256;

struct Sgd {
  float neg_lr, momentum, one_minus_dampening, weight_decay;
  int nesterov, first, has_buf;
};

__global__ __launch_bounds__(kThreads) void sgd_step(float* __restrict__ param, const float* __restrict__ grad,
                                                     float* __restrict__ buf, size_t n, Sgd a) {
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    const float p = param[i];
    float d = grad[i];
    if (a.weight_decay != 0.f) d = add(d, mul(p, a.weight_decay));          // :8
    if (a.has_buf) {
      float b;
      if (a.first) {
        b = d;                                                                          // :12-13
      } else {
        b = mul(buf[i], a.momentum);                                              // :15
        b = add(b, mul(d, a.one_minus_dampening));                          // :16
      }
      buf[i] = b;
      d = a.nesterov ? add(d, mul(b, a.momentum)) : b;                      // :17-20
    }
    param[i] = add(p, mul(d, a.neg_lr));                                    // :22
  }
}

struct Adam {
  float beta1, beta2, one_minus_beta1, one_minus_beta2, weight_decay, neg_step_size, decay_factor;
  double sqrt_bias_correction2, eps;
  int amsgrad, decoupled;
};

__global__ __launch_bounds__(kThreads) void adam_step(float* __restrict__ param, const float* __restrict__ grad,
                                                      float* __restrict__ exp_avg, float* __restrict__ exp_avg_sq,
                                                      float* __restrict__ max_exp_avg_sq, size_t n, Adam a) {
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    float p = param[i];
    float g = grad[i];
    if (a.decoupled) {
      p = mul(p, a.decay_factor);                                                 // :94
    } else if (a.weight_decay != 0.f) {
      g = add(g, mul(p, a.weight_decay));                                   // :46
    }
    float m = mul(exp_avg[i], a.beta1);                                           // :49
    m = add(m, mul(a.one_minus_beta1, g));                                  // :50
    float v = mul(exp_avg_sq[i], a.beta2);                                        // :52
    v = add(v, mul(mul(g, g), a.one_minus_beta2));                    // :53
    exp_avg[i] = m;
    exp_avg_sq[i] = v;
    float s = v;
    if (a.amsgrad) {
      const float old = max_exp_avg_sq[i];
      s = (old >= v || old != old) ? old : v;                                           // :57 maximum(out=)
      max_exp_avg_sq[i] = s;
    }
    // float32 square root, correctly rounded as NumPy's is: the hardware's single-precision
    // instruction is good to 1 ulp only, so it is taken in float64 and rounded once more
    const float root = (float)sqrt((double)s);
    const double denom = (double)root / a.sqrt_bias_correction2 + a.eps;                // :59 / :61
    const double update = (double)mul(a.neg_step_size, m) / denom;                // :64
    param[i] = (float)((double)p + update);
  }
}

unsigned blocks_for(size_t n) {
  size_t b = (n + kThreads - 1) / kThreads;
  return (unsigned)(b < 256 * 16 ? b : 256 * 16);
}

}  // namespace

extern "C" {

int tt_sgd_step_f32(float* param, const float* grad, float* momentum_buf, size_t n, double lr, double momentum,
                    double dampening, double weight_decay, int nesterov, int first_step) {
  TT_REQUIRE_INIT();
  if (n == 0) return 0;
  TT_REQUIRE(param && grad, "tt_sgd_step_f32: null pointer");
  TT_REQUIRE(momentum == 0.0 || momentum_buf, "tt_sgd_step_f32: momentum needs a buffer");
  Sgd a;
  a.neg_lr = (float)(-lr);
  a.momentum = (float)momentum;
  a.one_minus_dampening = (float)(1.0 - dampening);
  a.weight_decay = (float)weight_decay;
  a.nesterov = nesterov;
  a.first = first_step;
  a.has_buf = momentum != 0.0;
  sgd_step<<<blocks_for(n), kThreads, 0, tt::stream()>>>(param, grad, momentum_buf, n, a);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_adam_step_f32(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, float* max_exp_avg_sq,
                     size_t n, int step, double lr, double beta1, double beta2, double eps, double weight_decay,
                     int amsgrad, int decoupled_weight_decay) {
  TT_REQUIRE_INIT();
  if (n == 0) return 0;
  TT_REQUIRE(param && grad && exp_avg && exp_avg_sq, "tt_adam_step_f32: null pointer");
  TT_REQUIRE(!amsgrad || max_exp_avg_sq, "tt_adam_step_f32: amsgrad needs max_exp_avg_sq");
  TT_REQUIRE(step >= 1, "tt_adam_step_f32: step counts from 1");
  const double bias_correction1 = 1.0 - pow(beta1, (double)step);
  const double bias_correction2 = 1.0 - pow(beta2, (double)step);
  Adam a;
  a.beta1 = (float)beta1;
  a.beta2 = (float)beta2;
  a.one_minus_beta1 = (float)(1.0 - beta1);
  a.one_minus_beta2 = (float)(1.0 - beta2);
  a.weight_decay = (float)weight_decay;
  a.neg_step_size = (float)(-(lr / bias_correction1));
  a.decay_factor = (float)(1.0 - lr * weight_decay);
  a.sqrt_bias_correction2 = sqrt(bias_correction2);
  a.eps = eps;
  a.amsgrad = amsgrad;
  a.decoupled = decoupled_weight_decay;
  adam_step<<<blocks_for(n), kThreads, 0, tt::stream()>>>(param, grad, exp_avg, exp_avg_sq, max_exp_avg_sq, n, a);
  TT_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
