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

// ---- LDS-staged variants -------------------------------------------------------------------------
// Forward: a block owns a band of output rows of one plane.  The input rows the band depends on
// are one contiguous span of memory: it is fetched once with 16-byte loads into LDS, and the
// per-window gather then runs out of LDS.

constexpr int kStageFloats = 4096;   // 16 KiB of LDS per block

// Copies the span [s0, s0 + len) of `src` (element indices) to lds[(s0 & 3) + k]; 16-byte loads
// where the aligned quad lies inside the span, single elements at its two ends.
template <typename T>
__device__ __forceinline__ void stage_span(const T* __restrict__ src, size_t s0, int len, T* lds) {
  const size_t a0 = s0 & ~(size_t)3;
  const int head = (int)(s0 - a0);
  const int quads = (head + len + 3) >> 2;
  for (int k = threadIdx.x; k < quads; k += kThreads) {
    const int lo = 4 * k - head;             // span-relative index of the quad's first element
    if (lo >= 0 && lo + 4 <= len) {
      const int4 v = *reinterpret_cast<const int4*>(src + a0 + 4 * (size_t)k);
      *reinterpret_cast<int4*>(lds + 4 * k) = v;
    } else {
      for (int e = 0; e < 4; ++e)
        if (lo + e >= 0 && lo + e < len) lds[4 * k + e] = src[s0 + lo + e];
    }
  }
}

struct Band {
  int rows;             // output rows (forward) / input rows (backward) per block
  tt::FastDiv divSh, divKw;
};

// K > 0: square K x K kernel known at compile time; K == 0: run-time extents.
template <int K>
__global__ __launch_bounds__(kThreads) void maxpool_fwd_staged(const float* __restrict__ x, float* __restrict__ y,
                                                               int* __restrict__ tap, Pool g, Band b) {
  __shared__ __align__(16) float lds[kStageFloats + 8];
  const int nc = blockIdx.x;
  const int p0 = blockIdx.y * b.rows;
  const int p1 = min(g.P, p0 + b.rows);
  const int kh = K ? K : g.kh, kw = K ? K : g.kw;
  const int h_lo = max(0, p0 * g.sh - g.ph);
  const int h_hi = min(g.H, (p1 - 1) * g.sh - g.ph + (kh - 1) * g.dh + 1);   // exclusive
  const size_t s0 = (size_t)nc * g.H * g.W + (size_t)h_lo * g.W;
  if (h_hi > h_lo) stage_span(x, s0, (h_hi - h_lo) * g.W, lds);
  __syncthreads();
  const int shift = (int)(s0 & 3) - h_lo * g.W;            // lds[shift + h * W + w] for staged rows
  const int count = (p1 - p0) * g.Q;
  const size_t obase = ((size_t)nc * g.P + p0) * g.Q;
  for (int o = threadIdx.x; o < count; o += kThreads) {
    const int pl = (int)tt::fd_div((uint32_t)o, g.divQ);
    const int q = o - pl * g.Q;
    const int h0 = (p0 + pl) * g.sh - g.ph, w0 = q * g.sw - g.pw;
    float best = -INFINITY;
    int arg = 0;
    for (int i = 0; i < kh; ++i) {
      const int h = h0 + i * g.dh;
      const bool row_ok = (unsigned)h < (unsigned)g.H;
      for (int j = 0; j < kw; ++j) {
        const int w = w0 + j * g.dw;
        float v = -INFINITY;
        if (row_ok && (unsigned)w < (unsigned)g.W) v = lds[shift + h * g.W + w];
        if (v > best) {
          best = v;
          arg = i * kw + j;
        }
      }
    }
    __builtin_nontemporal_store(best, y + obase + o);
    __builtin_nontemporal_store(arg, tap + obase + o);
  }
}

// Backward as an ordered scatter inside LDS.  A block owns a band of input rows of one plane and
// keeps one 64-bit slot per pixel: (window order + 1) in the high half, the gradient's bits in the
// low half.  Every window that can reach the band offers its gradient to its arg-max pixel with a
// 64-bit maximum, so the window that is last in (p, q) order stays -- the same pixel the
// reference's indexed assignment leaves -- and untouched slots keep 0, whose low half is 0.0f.
constexpr int kScatterSlots = 4096;   // 32 KiB of LDS per block

__global__ __launch_bounds__(kThreads) void maxpool_bwd_scatter(const float* __restrict__ dy,
                                                                const int* __restrict__ tap,
                                                                float* __restrict__ dx, Pool g, Band b) {
  __shared__ __align__(16) unsigned long long slot[kScatterSlots];
  const int nc = blockIdx.x;
  const int h0 = blockIdx.y * b.rows;
  const int h1 = min(g.H, h0 + b.rows);
  const int rows = h1 - h0;
  const int count = rows * g.W;
  // output rows whose windows touch input rows [h0, h1)
  const int reach_h = (g.kh - 1) * g.dh;
  const int lo_num = h0 + g.ph - reach_h;
  const int p_first = lo_num > 0 ? (int)tt::fd_div((uint32_t)(lo_num + g.sh - 1), b.divSh) : 0;
  const int p_last = min(g.P - 1, (int)tt::fd_div((uint32_t)(h1 - 1 + g.ph), b.divSh));
  const int windows = (p_last - p_first + 1) * g.Q;
  const size_t obase = ((size_t)nc * g.P + p_first) * g.Q;
  // the first windows of every thread are fetched before the slots are cleared
  constexpr int kAhead = 4;
  int t_ahead[kAhead];
  float g_ahead[kAhead];
#pragma unroll
  for (int u = 0; u < kAhead; ++u) {
    const int o = min((int)threadIdx.x + u * kThreads, max(windows - 1, 0));
    t_ahead[u] = windows > 0 ? tap[obase + o] : 0;
    g_ahead[u] = windows > 0 ? dy[obase + o] : 0.f;
  }
  for (int k = threadIdx.x; 2 * k < count; k += kThreads)
    *reinterpret_cast<ulonglong2*>(&slot[2 * k]) = make_ulonglong2(0ull, 0ull);   // count <= kScatterSlots, even size
  __syncthreads();
  auto offer = [&](int o, int t, float gv) {
    const int pl = (int)tt::fd_div((uint32_t)o, g.divQ);
    const int q = o - pl * g.Q;
    const int i = (int)tt::fd_div((uint32_t)t, b.divKw);
    const int j = t - i * g.kw;
    const int h = (p_first + pl) * g.sh - g.ph + i * g.dh - h0;
    const int w = q * g.sw - g.pw + j * g.dw;
    if ((unsigned)h < (unsigned)rows && (unsigned)w < (unsigned)g.W) {
      const unsigned long long v =
          ((unsigned long long)(uint32_t)(p_first * g.Q + o + 1) << 32) | (unsigned long long)__float_as_uint(gv);
      atomicMax(&slot[h * g.W + w], v);
    }
  };
#pragma unroll
  for (int u = 0; u < kAhead; ++u) {
    const int o = (int)threadIdx.x + u * kThreads;
    if (o < windows) offer(o, t_ahead[u], g_ahead[u]);
  }
  for (int o = threadIdx.x + kAhead * kThreads; o < windows; o += kThreads) offer(o, tap[obase + o], dy[obase + o]);
  __syncthreads();
  const size_t ibase = ((size_t)nc * g.H + h0) * g.W;
  if (((ibase | (size_t)count) & 3) == 0) {
    for (int k = threadIdx.x; 4 * k < count; k += kThreads) {
      const ulonglong2 a = *reinterpret_cast<const ulonglong2*>(&slot[4 * k]);
      const ulonglong2 c = *reinterpret_cast<const ulonglong2*>(&slot[4 * k + 2]);
      float4 v;
      v.x = __uint_as_float((uint32_t)a.x);
      v.y = __uint_as_float((uint32_t)a.y);
      v.z = __uint_as_float((uint32_t)c.x);
      v.w = __uint_as_float((uint32_t)c.y);
      typedef float fx4 __attribute__((ext_vector_type(4)));
      const fx4 ov = {v.x, v.y, v.z, v.w};
      __builtin_nontemporal_store(ov, reinterpret_cast<fx4*>(dx + ibase) + k);
    }
  } else {
    for (int e = threadIdx.x; e < count; e += kThreads) dx[ibase + e] = __uint_as_float((uint32_t)slot[e]);
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

// Rows per block: what fits the stage, capped so that a plane still yields several blocks.
Band make_band(const Pool& g, int rows_fit, int cap) {
  Band b;
  b.rows = rows_fit < cap ? rows_fit : cap;
  b.divSh = tt::make_fastdiv((uint32_t)g.sh);
  b.divKw = tt::make_fastdiv((uint32_t)g.kw);
  return b;
}

unsigned grid_for(uint32_t total) {
  uint32_t blocks = (total + kThreads - 1) / kThreads;
  const uint32_t cap = (uint32_t)tt::compute_units() * 32;
  return blocks < cap ? blocks : cap;
}

}  // namespace

extern "C" {

int tt_maxpool2d_fwd_f32(const float* x, float* y, int* tap, int NC, int H, int W, int P, int Q, int kh, int kw,
                         int sh, int sw, int ph, int pw, int dh, int dw) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(x && y && tap, "tt_maxpool2d_fwd_f32: null pointer");
  TT_REQUIRE_ALIGNED("tt_maxpool2d_fwd_f32", x, y, tap);
  Pool g;
  if (int rc = fill("tt_maxpool2d_fwd_f32", &g, NC, H, W, P, Q, kh, kw, sh, sw, ph, pw, dh, dw)) return rc;
  const uint32_t total = (uint32_t)NC * P * Q;
  tt::ProfScope prof(TT_PROF_MAXPOOL_FWD);
  // output rows per block: as many as keep the input rows they need within the LDS stage
  const long long first = (long long)(kh - 1) * dh + 1;          // input rows of one output row
  const long long fit = ((long long)kStageFloats / W - first) / sh + 1;
  if ((long long)first * W <= kStageFloats && fit >= 1) {
    Band b = make_band(g, (int)(fit < P ? fit : P), 32);
    const dim3 grid(NC, (P + b.rows - 1) / b.rows);       // planes on x: their number has no 16-bit limit
    if (kh == 3 && kw == 3) maxpool_fwd_staged<3><<<grid, kThreads, 0, tt::stream()>>>(x, y, tap, g, b);
    else if (kh == 2 && kw == 2) maxpool_fwd_staged<2><<<grid, kThreads, 0, tt::stream()>>>(x, y, tap, g, b);
    else maxpool_fwd_staged<0><<<grid, kThreads, 0, tt::stream()>>>(x, y, tap, g, b);
  } else {
    maxpool_fwd<<<grid_for(total), kThreads, 0, tt::stream()>>>(x, y, tap, g, total);
  }
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_maxpool2d_bwd_f32(const float* dy, const int* tap, float* dx, int NC, int H, int W, int P, int Q, int kh,
                         int kw, int sh, int sw, int ph, int pw, int dh, int dw) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(dy && tap && dx, "tt_maxpool2d_bwd_f32: null pointer");
  TT_REQUIRE_ALIGNED("tt_maxpool2d_bwd_f32", dy, tap, dx);
  Pool g;
  if (int rc = fill("tt_maxpool2d_bwd_f32", &g, NC, H, W, P, Q, kh, kw, sh, sw, ph, pw, dh, dw)) return rc;
  const uint32_t total = (uint32_t)NC * H * W;
  tt::ProfScope prof(TT_PROF_MAXPOOL_BWD);
  // input rows per block: one 8-byte LDS slot per pixel of the band
  const int fit = kScatterSlots / W;
  if (fit >= 1) {
    Band b = make_band(g, fit < H ? fit : H, 32);
    const dim3 grid(NC, (H + b.rows - 1) / b.rows);
    maxpool_bwd_scatter<<<grid, kThreads, 0, tt::stream()>>>(dy, tap, dx, g, b);
  } else {
    maxpool_bwd<<<grid_for(total), kThreads, 0, tt::stream()>>>(dy, tap, dx, g, total);
  }
  TT_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
