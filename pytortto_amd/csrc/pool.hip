// MaxPool2d forward / backward on NCHW float32 planes (HBM-bound gather kernels).
//
// Follows src/tortto/autograd/grad_nn.py:784-824: windows are taken over the input padded with
// -inf (also below/right for ceil_mode), the maximum ignores NaN and ties go to the first tap in
// (row, column) order; the backward ASSIGNS each output gradient to its window's arg-max pixel
// (`expanded[pos] = grad`, :818), so where overlapping windows pick the same pixel the window
// that comes last in (p, q) order wins -- gradients are not summed.
#include "tt_common.h"

#include <math.h>

namespace {

constexpr int kThreads = 256;

struct Pool {
  int NC, H, W, P, Q;
  int kh, kw, sh, sw, ph, pw, dh, dw;
  tt::FastDiv divQ, divP, divW, divH;
};

// One thread per output element; `tap` receives the arg-max as kernel-row * kw + kernel-column.
__global__ __launch_bounds__(kThreads) void maxpool_fwd(const float* __restrict__ x, float* __restrict__ y,
                                                        int* __restrict__ tap, Pool g, uint32_t total) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t o = blockIdx.x * kThreads + threadIdx.x; o < total; o += stride) {
    const uint32_t t = tt::fd_div(o, g.divQ);
    const int q = (int)(o - t * (uint32_t)g.Q);
    const uint32_t nc = tt::fd_div(t, g.divP);
    const int p = (int)(t - nc * (uint32_t)g.P);
    const float* __restrict__ plane = x + (size_t)nc * g.H * g.W;
    const int h0 = p * g.sh - g.ph, w0 = q * g.sw - g.pw;
    float best = -INFINITY;
    int arg = 0;
    for (int i = 0; i < g.kh; ++i) {
      const int h = h0 + i * g.dh;
      const bool row_ok = (unsigned)h < (unsigned)g.H;
      for (int j = 0; j < g.kw; ++j) {
        const int w = w0 + j * g.dw;
        float v = -INFINITY;
        if (row_ok && (unsigned)w < (unsigned)g.W) v = plane[h * g.W + w];
        if (v > best) {   // false for NaN: ignored, as nanargmax does; strict: first maximum wins
          best = v;
          arg = i * g.kw + j;
        }
      }
    }
    y[o] = best;
    tap[o] = arg;
  }
}

// One thread per input pixel: of the windows that cover it, the last in (p, q) order whose
// arg-max is this pixel supplies the gradient; none -> 0.
__global__ __launch_bounds__(kThreads) void maxpool_bwd(const float* __restrict__ dy, const int* __restrict__ tap,
                                                        float* __restrict__ dx, Pool g, uint32_t total) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t e = blockIdx.x * kThreads + threadIdx.x; e < total; e += stride) {
    const uint32_t t = tt::fd_div(e, g.divW);
    const int w = (int)(e - t * (uint32_t)g.W);
    const uint32_t nc = tt::fd_div(t, g.divH);
    const int h = (int)(t - nc * (uint32_t)g.H);
    const int hh = h + g.ph, ww = w + g.pw;
    // windows with p*sh <= hh <= p*sh + (kh-1)*dh
    const int p_hi = min(g.P - 1, hh / g.sh);
    const int q_hi = min(g.Q - 1, ww / g.sw);
    const int reach_h = (g.kh - 1) * g.dh, reach_w = (g.kw - 1) * g.dw;
    const int p_lo = hh > reach_h ? (hh - reach_h + g.sh - 1) / g.sh : 0;
    const int q_lo = ww > reach_w ? (ww - reach_w + g.sw - 1) / g.sw : 0;
    const size_t obase = (size_t)nc * g.P * g.Q;
    float out = 0.f;
    bool found = false;
    for (int p = p_hi; p >= p_lo && !found; --p) {
      const int r = hh - p * g.sh;
      const int i = r / g.dh;
      if (i * g.dh != r) continue;
      for (int q = q_hi; q >= q_lo; --q) {
        const int c = ww - q * g.sw;
        const int j = c / g.dw;
        if (j * g.dw != c) continue;
        const size_t o = obase + (size_t)p * g.Q + q;
        if (tap[o] == i * g.kw + j) {
          out = dy[o];
          found = true;
          break;
        }
      }
    }
    dx[e] = out;
  }
}

int fill(const char* fn, Pool* g, int NC, int H, int W, int P, int Q, int kh, int kw, int sh, int sw, int ph,
         int pw, int dh, int dw) {
  TT_REQUIRE(NC > 0 && H > 0 && W > 0 && P > 0 && Q > 0, "%s: sizes must be positive", fn);
  TT_REQUIRE(kh > 0 && kw > 0 && sh > 0 && sw > 0 && dh > 0 && dw > 0 && ph >= 0 && pw >= 0,
             "%s: kernel, stride, dilation must be positive and padding non-negative", fn);
  TT_REQUIRE(H < 32768 && W < 32768 && kh < 32768 && kw < 32768 && (long long)kh * kw < 2147483647LL,
             "%s: extents above 32767 are not supported", fn);
  TT_REQUIRE(tt::fits_i32((long long)NC * H * W) && tt::fits_i32((long long)NC * P * Q),
             "%s: tensor exceeds 2^31-1 elements", fn);
  // every window starts inside the input or its top/left padding
  TT_REQUIRE((long long)(P - 1) * sh < (long long)H + ph && (long long)(Q - 1) * sw < (long long)W + pw,
             "%s: output size (%d, %d) does not fit the input (%d, %d)", fn, P, Q, H, W);
  *g = Pool{NC, H, W, P, Q, kh, kw, sh, sw, ph, pw, dh, dw,
            tt::make_fastdiv((uint32_t)Q), tt::make_fastdiv((uint32_t)P), tt::make_fastdiv((uint32_t)W),
            tt::make_fastdiv((uint32_t)H)};
  return 0;
}

unsigned grid_for(uint32_t total) {
  uint32_t blocks = (total + kThreads - 1) / kThreads;
  const uint32_t cap = 256 * 32;
  return blocks < cap ? blocks : cap;
}

}  // namespace

extern "C" {

int tt_maxpool2d_fwd_f32(const float* x, float* y, int* tap, int NC, int H, int W, int P, int Q, int kh, int kw,
                         int sh, int sw, int ph, int pw, int dh, int dw) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(x && y && tap, "tt_maxpool2d_fwd_f32: null pointer");
  Pool g;
  if (int rc = fill("tt_maxpool2d_fwd_f32", &g, NC, H, W, P, Q, kh, kw, sh, sw, ph, pw, dh, dw)) return rc;
  const uint32_t total = (uint32_t)NC * P * Q;
  tt::ProfScope prof(TT_PROF_MAXPOOL_FWD);
  maxpool_fwd<<<grid_for(total), kThreads, 0, tt::stream()>>>(x, y, tap, g, total);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_maxpool2d_bwd_f32(const float* dy, const int* tap, float* dx, int NC, int H, int W, int P, int Q, int kh,
                         int kw, int sh, int sw, int ph, int pw, int dh, int dw) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(dy && tap && dx, "tt_maxpool2d_bwd_f32: null pointer");
  Pool g;
  if (int rc = fill("tt_maxpool2d_bwd_f32", &g, NC, H, W, P, Q, kh, kw, sh, sw, ph, pw, dh, dw)) return rc;
  const uint32_t total = (uint32_t)NC * H * W;
  tt::ProfScope prof(TT_PROF_MAXPOOL_BWD);
  maxpool_bwd<<<grid_for(total), kThreads, 0, tt::stream()>>>(dy, tap, dx, g, total);
  TT_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
