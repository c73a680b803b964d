// Elementwise glue kernels (ReLU, LeakyReLU, residual add, gradient accumulation, fill): HBM-bound,
// float4 grid-stride loops with a scalar tail.
#include "tt_common.h"

namespace {

constexpr int kThreads = 256;

enum Op { kRelu, kReluBwd, kAdd, kAxpy, kFill, kLeakyRelu, kLeakyReluBwd, kAddScalar, kAddRelu };

template <int OP>
__device__ __forceinline__ float apply1(float a, float b, float alpha) {
  // NumPy's maximum propagates NaN (src/tortto/autograd/grad_nn.py:56), fmaxf would drop it
  if (OP == kRelu) return (a > 0.f || a != a) ? a : 0.f;
  if (OP == kLeakyRelu) {                         // maximum(x * slope, x), grad_nn.py:85
    const float t = a * alpha;
    return (t > a || t != t) ? t : a;
  }
  if (OP == kLeakyReluBwd) return b < 0.f ? a * alpha : a;   // a = dy, b = x: g[x < 0] *= slope, grad_nn.py:94
  // a = dy, b = y: the reference multiplies by the mask, gd0 * (yd0 > 0) (grad_nn.py:67), so a
  // non-finite gradient at a masked element gives NaN and a negative one -0, not +0
  if (OP == kReluBwd) return a * (b > 0.f ? 1.f : 0.f);
  if (OP == kAdd) return a + b;
  if (OP == kAddRelu) {                           // maximum(a + b, 0): the sum rounded as by kAdd, NaN kept as by kRelu
    const float t = a + b;
    return (t > 0.f || t != t) ? t : 0.f;
  }
  if (OP == kAxpy) return fmaf(alpha, a, b);      // a = v, b = acc
  if (OP == kAddScalar) return a + alpha;
  return alpha;                                    // kFill
}

template <int OP>
__global__ __launch_bounds__(kThreads) void eltwise(const float* __restrict__ a, const float* __restrict__ b,
                                                    float* __restrict__ out, float alpha, size_t n) {
  constexpr bool kUseA = OP != kFill;
  // results that are not accumulated in place stream out past the caches
  constexpr bool kStreamOut = OP == kRelu || OP == kReluBwd || OP == kAdd || OP == kLeakyRelu || OP == kLeakyReluBwd || OP == kAddRelu;
  constexpr bool kUseB = OP == kReluBwd || OP == kAdd || OP == kAxpy || OP == kLeakyReluBwd || OP == kAddRelu;
  // two-input kernels whose inputs are read for the last time here (a gradient and the saved
  // activation, the two branches of a residual add) stream them in past the caches too: 8-9 %
  // faster than allocating loads at 200 MB per tensor; one-input kernels are faster with plain loads
  constexpr bool kStreamIn = kStreamOut && kUseB;
  const size_t n4 = n >> 2;
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n4; i += stride) {
    float4 va = make_float4(0.f, 0.f, 0.f, 0.f), vb = va, o;
    typedef float fx4 __attribute__((ext_vector_type(4)));
    if (kUseA) {
      // (the increment of a gradient accumulation is read for the last time as well)
      if (kStreamIn || OP == kAxpy) { const fx4 t = __builtin_nontemporal_load(reinterpret_cast<const fx4*>(a) + i); va = make_float4(t.x, t.y, t.z, t.w); }
      else va = reinterpret_cast<const float4*>(a)[i];
    }
    if (kUseB) {
      if (kStreamIn) { const fx4 t = __builtin_nontemporal_load(reinterpret_cast<const fx4*>(b) + i); vb = make_float4(t.x, t.y, t.z, t.w); }
      else vb = reinterpret_cast<const float4*>(b)[i];
    }
    o.x = apply1<OP>(va.x, vb.x, alpha);
    o.y = apply1<OP>(va.y, vb.y, alpha);
    o.z = apply1<OP>(va.z, vb.z, alpha);
    o.w = apply1<OP>(va.w, vb.w, alpha);
    if (kStreamOut) {
      const fx4 ov = {o.x, o.y, o.z, o.w};
      __builtin_nontemporal_store(ov, reinterpret_cast<fx4*>(out) + i);
    } else {
      reinterpret_cast<float4*>(out)[i] = o;
    }
  }
  // tail (n % 4 elements)
  const size_t t = (n4 << 2) + (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (t < n) out[t] = apply1<OP>(kUseA ? a[t] : 0.f, kUseB ? b[t] : 0.f, alpha);
}

template <int OP>
int run(const char* fn, const float* a, const float* b, float* out, float alpha, size_t n) {
  TT_REQUIRE_INIT();
  if (n == 0) return 0;
  TT_REQUIRE(out != nullptr, "%s: null output pointer", fn);
  TT_REQUIRE_ALIGNED(fn, a, b, out);
  size_t blocks = ((n >> 2) + kThreads - 1) / kThreads;
  const size_t cap = (size_t)tt::compute_units() * 16;   // grid-stride beyond 16 blocks per CU
  if (blocks < 1) blocks = 1;
  if (blocks > cap) blocks = cap;
  eltwise<OP><<<(unsigned)blocks, kThreads, 0, tt::stream()>>>(a, b, out, alpha, n);
  TT_LAUNCH_CHECK();
  return 0;
}

}  // namespace

extern "C" {

int tt_relu_fwd_f32(const float* x, float* y, size_t n) { return run<kRelu>("tt_relu_fwd_f32", x, nullptr, y, 0.f, n); }
int tt_relu_bwd_f32(const float* dy, const float* y, float* dx, size_t n) {
  return run<kReluBwd>("tt_relu_bwd_f32", dy, y, dx, 0.f, n);
}
int tt_leaky_relu_fwd_f32(const float* x, float* y, float negative_slope, size_t n) {
  return run<kLeakyRelu>("tt_leaky_relu_fwd_f32", x, nullptr, y, negative_slope, n);
}
int tt_leaky_relu_bwd_f32(const float* dy, const float* x, float* dx, float negative_slope, size_t n) {
  return run<kLeakyReluBwd>("tt_leaky_relu_bwd_f32", dy, x, dx, negative_slope, n);
}
int tt_add_f32(const float* a, const float* b, float* out, size_t n) { return run<kAdd>("tt_add_f32", a, b, out, 0.f, n); }
int tt_add_relu_f32(const float* a, const float* b, float* out, size_t n) {
  return run<kAddRelu>("tt_add_relu_f32", a, b, out, 0.f, n);
}
int tt_axpy_f32(float alpha, const float* v, float* acc, size_t n) {
  return run<kAxpy>("tt_axpy_f32", v, acc, acc, alpha, n);
}
int tt_add_scalar_f32(float* acc, float value, size_t n) {
  return run<kAddScalar>("tt_add_scalar_f32", acc, nullptr, acc, value, n);
}
int tt_fill_f32(float* dst, float value, size_t n) { return run<kFill>("tt_fill_f32", nullptr, nullptr, dst, value, n); }

}  // extern "C"
