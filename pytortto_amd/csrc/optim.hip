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

__device__ __forceinline__ void sgd_range(float* __restrict__ param, const float* __restrict__ grad,
                                          float* __restrict__ buf, size_t n, size_t start, size_t stride,
                                          const Sgd& a) {
  for (size_t i = start; i < n; i += stride) {
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

__global__ __launch_bounds__(kThreads) void sgd_step(float* __restrict__ param, const float* __restrict__ grad,
                                                     float* __restrict__ buf, size_t n, Sgd a) {
  sgd_range(param, grad, buf, n, (size_t)blockIdx.x * kThreads + threadIdx.x, (size_t)gridDim.x * kThreads, a);
}

// Several parameters in one launch: blocks [first_block[t], first_block[t+1]) work on tensor t.
// A network has one launch-bound update per parameter otherwise (161 for ResNet-50).
constexpr int kMultiMax = 24;
struct Tensors {
  float* param[kMultiMax];
  const float* grad[kMultiMax];
  float* buf[kMultiMax];
  unsigned long long n[kMultiMax];
  unsigned first_block[kMultiMax + 1];
  unsigned first_step_mask;      // bit t: tensor t takes its first momentum step
  int count;
};

__global__ __launch_bounds__(kThreads) void sgd_step_multi(Tensors ts, Sgd a) {
  int t = 0;
  while (t + 1 < ts.count && blockIdx.x >= ts.first_block[t + 1]) ++t;
  const unsigned blocks = ts.first_block[t + 1] - ts.first_block[t];
  a.first = (ts.first_step_mask >> t) & 1;
  sgd_range(ts.param[t], ts.grad[t], ts.buf[t], (size_t)ts.n[t],
            (size_t)(blockIdx.x - ts.first_block[t]) * kThreads + threadIdx.x, (size_t)blocks * kThreads, a);
}

struct Adam {
  float beta1, beta2, one_minus_beta1, one_minus_beta2, weight_decay, neg_step_size, decay_factor;
  double sqrt_bias_correction2, eps;
  int amsgrad, decoupled;
};

__device__ __forceinline__ void adam_range(float* __restrict__ param, const float* __restrict__ grad,
                                           float* __restrict__ exp_avg, float* __restrict__ exp_avg_sq,
                                           float* __restrict__ max_exp_avg_sq, size_t n, size_t start,
                                           size_t stride, const Adam& a) {
  for (size_t i = start; i < n; i += stride) {
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

__global__ __launch_bounds__(kThreads) void adam_step(float* __restrict__ param, const float* __restrict__ grad,
                                                      float* __restrict__ exp_avg, float* __restrict__ exp_avg_sq,
                                                      float* __restrict__ max_exp_avg_sq, size_t n, Adam a) {
  adam_range(param, grad, exp_avg, exp_avg_sq, max_exp_avg_sq, n, (size_t)blockIdx.x * kThreads + threadIdx.x,
             (size_t)gridDim.x * kThreads, a);
}

struct AdamTensors {
  float* param[kMultiMax];
  const float* grad[kMultiMax];
  float* exp_avg[kMultiMax];
  float* exp_avg_sq[kMultiMax];
  float* max_exp_avg_sq[kMultiMax];
  unsigned long long n[kMultiMax];
  double sqrt_bias_correction2[kMultiMax];   // the step count, and with it the corrections, is per parameter
  float neg_step_size[kMultiMax];
  unsigned first_block[kMultiMax + 1];
  int count;
};

__global__ __launch_bounds__(kThreads) void adam_step_multi(AdamTensors ts, Adam a) {
  int t = 0;
  while (t + 1 < ts.count && blockIdx.x >= ts.first_block[t + 1]) ++t;
  const unsigned blocks = ts.first_block[t + 1] - ts.first_block[t];
  a.neg_step_size = ts.neg_step_size[t];
  a.sqrt_bias_correction2 = ts.sqrt_bias_correction2[t];
  adam_range(ts.param[t], ts.grad[t], ts.exp_avg[t], ts.exp_avg_sq[t], ts.max_exp_avg_sq[t], (size_t)ts.n[t],
             (size_t)(blockIdx.x - ts.first_block[t]) * kThreads + threadIdx.x, (size_t)blocks * kThreads, a);
}

unsigned blocks_for(size_t n) {
  size_t b = (n + kThreads - 1) / kThreads;
  const size_t cap = (size_t)tt::compute_units() * 16;
  return (unsigned)(b < cap ? b : cap);
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

int tt_sgd_step_multi_f32(int count, float* const* params, const float* const* grads, float* const* momentum_bufs,
                          const size_t* sizes, const int* first_steps, double lr, double momentum, double dampening,
                          double weight_decay, int nesterov) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(count >= 0, "tt_sgd_step_multi_f32: negative count");
  TT_REQUIRE(count == 0 || (params && grads && sizes), "tt_sgd_step_multi_f32: null table");
  TT_REQUIRE(momentum == 0.0 || (momentum_bufs && first_steps), "tt_sgd_step_multi_f32: momentum needs buffers");
  Sgd a;
  a.neg_lr = (float)(-lr);
  a.momentum = (float)momentum;
  a.one_minus_dampening = (float)(1.0 - dampening);
  a.weight_decay = (float)weight_decay;
  a.nesterov = nesterov;
  a.first = 0;
  a.has_buf = momentum != 0.0;
  for (int i = 0; i < count; ++i) {
    TT_REQUIRE(sizes[i] == 0 || (params[i] && grads[i]), "tt_sgd_step_multi_f32: null pointer for tensor %d", i);
    TT_REQUIRE(!a.has_buf || sizes[i] == 0 || momentum_bufs[i], "tt_sgd_step_multi_f32: tensor %d has no buffer", i);
  }
  int done = 0;
  while (done < count) {
    Tensors ts;
    ts.count = 0;
    ts.first_step_mask = 0;
    unsigned blocks = 0;
    for (; done < count && ts.count < kMultiMax; ++done) {
      if (sizes[done] == 0) continue;
      const int t = ts.count++;
      ts.param[t] = params[done];
      ts.grad[t] = grads[done];
      ts.buf[t] = a.has_buf ? momentum_bufs[done] : nullptr;
      ts.n[t] = sizes[done];
      ts.first_block[t] = blocks;
      if (a.has_buf && first_steps[done]) ts.first_step_mask |= 1u << t;
      const size_t want = (sizes[done] + 4 * kThreads - 1) / (4 * kThreads);     // about four elements per thread
      blocks += (unsigned)(want < 2048 ? want : 2048);
    }
    if (ts.count == 0) break;
    ts.first_block[ts.count] = blocks;
    sgd_step_multi<<<blocks, kThreads, 0, tt::stream()>>>(ts, a);
    TT_LAUNCH_CHECK();
  }
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

int tt_adam_step_multi_f32(int count, float* const* params, const float* const* grads, float* const* exp_avgs,
                           float* const* exp_avg_sqs, float* const* max_exp_avg_sqs, const size_t* sizes,
                           const int* steps, double lr, double beta1, double beta2, double eps, double weight_decay,
                           int amsgrad, int decoupled_weight_decay) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(count >= 0, "tt_adam_step_multi_f32: negative count");
  TT_REQUIRE(count == 0 || (params && grads && exp_avgs && exp_avg_sqs && sizes && steps),
             "tt_adam_step_multi_f32: null table");
  TT_REQUIRE(!amsgrad || max_exp_avg_sqs, "tt_adam_step_multi_f32: amsgrad needs max_exp_avg_sq");
  Adam a;
  a.beta1 = (float)beta1;
  a.beta2 = (float)beta2;
  a.one_minus_beta1 = (float)(1.0 - beta1);
  a.one_minus_beta2 = (float)(1.0 - beta2);
  a.weight_decay = (float)weight_decay;
  a.neg_step_size = 0.f;
  a.decay_factor = (float)(1.0 - lr * weight_decay);
  a.sqrt_bias_correction2 = 1.0;
  a.eps = eps;
  a.amsgrad = amsgrad;
  a.decoupled = decoupled_weight_decay;
  for (int i = 0; i < count; ++i) {
    if (sizes[i] == 0) continue;
    TT_REQUIRE(params[i] && grads[i] && exp_avgs[i] && exp_avg_sqs[i] && (!amsgrad || max_exp_avg_sqs[i]),
               "tt_adam_step_multi_f32: null pointer for tensor %d", i);
    TT_REQUIRE(steps[i] >= 1, "tt_adam_step_multi_f32: step counts from 1 (tensor %d)", i);
  }
  int done = 0;
  while (done < count) {
    AdamTensors ts;
    ts.count = 0;
    unsigned blocks = 0;
    for (; done < count && ts.count < kMultiMax; ++done) {
      if (sizes[done] == 0) continue;
      const int t = ts.count++;
      ts.param[t] = params[done];
      ts.grad[t] = grads[done];
      ts.exp_avg[t] = exp_avgs[done];
      ts.exp_avg_sq[t] = exp_avg_sqs[done];
      ts.max_exp_avg_sq[t] = amsgrad ? max_exp_avg_sqs[done] : nullptr;
      ts.n[t] = sizes[done];
      ts.neg_step_size[t] = (float)(-(lr / (1.0 - pow(beta1, (double)steps[done]))));
      ts.sqrt_bias_correction2[t] = sqrt(1.0 - pow(beta2, (double)steps[done]));
      ts.first_block[t] = blocks;
      const size_t want = (sizes[done] + 4 * kThreads - 1) / (4 * kThreads);
      blocks += (unsigned)(want < 2048 ? want : 2048);
    }
    if (ts.count == 0) break;
    ts.first_block[ts.count] = blocks;
    adam_step_multi<<<blocks, kThreads, 0, tt::stream()>>>(ts, a);
    TT_LAUNCH_CHECK();
  }
  return 0;
}

}  // extern "C"
