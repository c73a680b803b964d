// The classifier head either side of the convolution stack: spatial mean, 2-D transpose, bias
// broadcast, LogSoftmax and NLLLoss (forward and backward).  All tensors here are small next to
// the feature maps (a batch of logits, one value per plane), so the kernels are plain: one wave
// per row with shuffle reductions, float64 accumulation where a sum feeds a statistic.
#include "tt_common.h"

#include <math.h>

namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / tt::kWave;

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int off = tt::kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, tt::kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = tt::kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, tt::kWave));
  return v;
}

// y[r] = mean(x[r, 0..L)): one wave per row.
__global__ __launch_bounds__(kThreads) void mean_rows(const float* __restrict__ x, float* __restrict__ y, int R,
                                                      int L) {
  const int lane = threadIdx.x & (tt::kWave - 1);
  const int row = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (row >= R) return;
  const float* __restrict__ p = x + (size_t)row * L;
  double s = 0.0;
  for (int i = lane; i < L; i += tt::kWave) s += (double)p[i];
  s = wave_sum(s);
  if (lane == 0) y[row] = (float)(s / (double)L);
}

// dx[r, i] = g[r] / L  (the reference divides the gradient in its own dtype, then repeats it)
__global__ __launch_bounds__(kThreads) void mean_rows_bwd(const float* __restrict__ g, float* __restrict__ dx,
                                                          size_t total, tt::FastDiv divL, float L) {
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x; e < total; e += stride)
    dx[e] = __fdiv_rn(g[tt::fd_div((uint32_t)e, divL)], L);
}

// y[c, r] = x[r, c] through a padded 32x32 LDS tile; block = 32 x 8 threads.
__global__ __launch_bounds__(kThreads) void transpose2d(const float* __restrict__ x, float* __restrict__ y, int R,
                                                        int C) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  for (int j = ty; j < 32; j += 8)
    if (r0 + j < R && c0 + tx < C) tile[j][tx] = x[(size_t)(r0 + j) * C + c0 + tx];
  __syncthreads();
  for (int j = ty; j < 32; j += 8)
    if (c0 + j < C && r0 + tx < R) y[(size_t)(c0 + j) * R + r0 + tx] = tile[tx][j];
}

// out[r, c] = a[r, c] + v[c]
__global__ __launch_bounds__(kThreads) void add_rowvec(const float* __restrict__ a, const float* __restrict__ v,
                                                       float* __restrict__ out, size_t total, tt::FastDiv divC,
                                                       int C) {
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x; e < total; e += stride) {
    const uint32_t r = tt::fd_div((uint32_t)e, divC);
    out[e] = a[e] + v[(uint32_t)e - r * (uint32_t)C];
  }
}

// y = (x - max) - log(sum(exp(x - max))) along each row: one wave per row.
__global__ __launch_bounds__(kThreads) void log_softmax_rows(const float* __restrict__ x, float* __restrict__ y,
                                                             int R, int C) {
  const int lane = threadIdx.x & (tt::kWave - 1);
  const int row = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (row >= R) return;
  const float* __restrict__ p = x + (size_t)row * C;
  float* __restrict__ o = y + (size_t)row * C;
  float m = -INFINITY;
  bool nan = false;
  for (int i = lane; i < C; i += tt::kWave) {
    const float v = p[i];
    nan |= v != v;
    m = fmaxf(m, v);
  }
  m = wave_max(m);
  if (__any(nan)) m = NAN;                      // NumPy's max propagates NaN: the whole row turns NaN
  float s = 0.f;
  for (int i = lane; i < C; i += tt::kWave) s += expf(p[i] - m);
  const float lse = logf(wave_sum(s));
  for (int i = lane; i < C; i += tt::kWave) o[i] = (p[i] - m) - lse;
}

// dx = g - sum(g) * exp(y)
__global__ __launch_bounds__(kThreads) void log_softmax_rows_bwd(const float* __restrict__ g,
                                                                 const float* __restrict__ y,
                                                                 float* __restrict__ dx, int R, int C) {
  const int lane = threadIdx.x & (tt::kWave - 1);
  const int row = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (row >= R) return;
  const size_t base = (size_t)row * C;
  float s = 0.f;
  for (int i = lane; i < C; i += tt::kWave) s += g[base + i];
  s = wave_sum(s);
  for (int i = lane; i < C; i += tt::kWave) dx[base + i] = g[base + i] - s * expf(y[base + i]);
}

// One block.  per_row[n] = -logp[n, t[n]] * w[n]; w[n] = weight[t[n]] (or 1), zeroed where
// t[n] == ignore_index >= 0.  reduction: 0 none (per_row is the result), 1 sum, 2 mean.
// count_out receives the divisor of the mean: the number of rows without weights, else the
// number of rows whose weight is non-zero.
__global__ __launch_bounds__(kThreads) void nll_loss_fwd(const float* __restrict__ logp,
                                                         const long long* __restrict__ target,
                                                         const float* __restrict__ weight, float* __restrict__ out,
                                                         float* __restrict__ count_out, int R, int C,
                                                         long long ignore_index, int reduction) {
  __shared__ double part[2][kWavesPerBlock];
  const bool weighted = weight != nullptr || ignore_index >= 0;
  double s = 0.0, cnt = 0.0;
  for (int n = threadIdx.x; n < R; n += kThreads) {
    const long long t0 = target[n];
    const long long t = t0 < 0 ? t0 + C : t0;      // -C..-1 count from the end, as NumPy indexing does (:300, :309)
    float w = 1.f, v = 0.f;
    if (t >= 0 && t < C) {
      if (weight) w = weight[t];
      v = -logp[(size_t)n * C + t];
    } else {
      // a class outside [-C, C): the reference's indexing raises IndexError; a kernel cannot raise,
      // so the row's loss -- and with it a summed or averaged loss -- becomes NaN
      v = __builtin_nanf("");
    }
    if (ignore_index >= 0 && t0 == ignore_index) w = 0.f;
    if (weighted) v = v * w;
    if (reduction == 0) out[n] = v;
    s += (double)v;
    cnt += weighted ? (w != 0.f ? 1.0 : 0.0) : 1.0;
  }
  s = wave_sum(s);
  cnt = wave_sum(cnt);
  const int lane = threadIdx.x & (tt::kWave - 1), wv = threadIdx.x >> 6;
  if (lane == 0) {
    part[0][wv] = s;
    part[1][wv] = cnt;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double ts = 0.0, tc = 0.0;
    for (int i = 0; i < kWavesPerBlock; ++i) {
      ts += part[0][i];
      tc += part[1][i];
    }
    count_out[0] = (float)tc;
    if (reduction == 1) out[0] = (float)ts;
    if (reduction == 2) out[0] = (float)(ts / tc);
  }
}

// dlogp[n, c] = (c == t[n]) ? -g * w[n] / divisor : 0;  g is per row for reduction none, else g[0].
__global__ __launch_bounds__(kThreads) void nll_loss_bwd(const float* __restrict__ g,
                                                         const long long* __restrict__ target,
                                                         const float* __restrict__ weight,
                                                         const float* __restrict__ count, float* __restrict__ dlogp,
                                                         size_t total, tt::FastDiv divC, int C,
                                                         long long ignore_index, int reduction) {
  const size_t stride = (size_t)gridDim.x * kThreads;
  const float div = reduction == 2 ? count[0] : 1.f;
  for (size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x; e < total; e += stride) {
    const uint32_t n = tt::fd_div((uint32_t)e, divC);
    const long long c = (long long)((uint32_t)e - n * (uint32_t)C);
    const long long t0 = target[n];
    const long long t = t0 < 0 ? t0 + C : t0;      // negative classes count from the end, as in the forward
    float v = 0.f;
    if (c == t) {
      float w = weight ? weight[t] : 1.f;
      if (ignore_index >= 0 && t0 == ignore_index) w = 0.f;
      float gv = reduction == 0 ? g[n] : g[0];
      if (reduction == 2) gv = __fdiv_rn(gv, div);
      v = -gv * w;
    }
    dlogp[e] = v;
  }
}

unsigned blocks_for(size_t total) {
  size_t b = (total + kThreads - 1) / kThreads;
  if (b < 1) b = 1;
  const size_t cap = (size_t)tt::compute_units() * 16;
  return (unsigned)(b < cap ? b : cap);
}

int check_rows(const char* fn, int R, int C) {
  TT_REQUIRE(R > 0 && C > 0, "%s: rows and columns must be positive (got %d, %d)", fn, R, C);
  TT_REQUIRE(tt::fits_i32((long long)R * C), "%s: tensor exceeds 2^31-1 elements", fn);
  return 0;
}

}  // namespace

extern "C" {

int tt_mean_rows_f32(const float* x, float* y, int R, int L) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(x && y, "tt_mean_rows_f32: null pointer");
  if (int rc = check_rows("tt_mean_rows_f32", R, L)) return rc;
  mean_rows<<<(R + kWavesPerBlock - 1) / kWavesPerBlock, kThreads, 0, tt::stream()>>>(x, y, R, L);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_mean_rows_bwd_f32(const float* g, float* dx, int R, int L) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(g && dx, "tt_mean_rows_bwd_f32: null pointer");
  if (int rc = check_rows("tt_mean_rows_bwd_f32", R, L)) return rc;
  const size_t total = (size_t)R * L;
  mean_rows_bwd<<<blocks_for(total), kThreads, 0, tt::stream()>>>(g, dx, total, tt::make_fastdiv((uint32_t)L),
                                                                 (float)L);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_transpose2d_f32(const float* x, float* y, int R, int C) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(x && y && x != y, "tt_transpose2d_f32: null or aliased pointers");
  if (int rc = check_rows("tt_transpose2d_f32", R, C)) return rc;
  TT_REQUIRE((R + 31) / 32 <= 65535, "tt_transpose2d_f32: more than 2097120 rows are not supported");
  transpose2d<<<dim3((C + 31) / 32, (R + 31) / 32), kThreads, 0, tt::stream()>>>(x, y, R, C);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_add_rowvec_f32(const float* a, const float* v, float* out, int R, int C) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(a && v && out, "tt_add_rowvec_f32: null pointer");
  if (int rc = check_rows("tt_add_rowvec_f32", R, C)) return rc;
  const size_t total = (size_t)R * C;
  add_rowvec<<<blocks_for(total), kThreads, 0, tt::stream()>>>(a, v, out, total, tt::make_fastdiv((uint32_t)C), C);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_log_softmax_fwd_f32(const float* x, float* y, int R, int C) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(x && y, "tt_log_softmax_fwd_f32: null pointer");
  if (int rc = check_rows("tt_log_softmax_fwd_f32", R, C)) return rc;
  log_softmax_rows<<<(R + kWavesPerBlock - 1) / kWavesPerBlock, kThreads, 0, tt::stream()>>>(x, y, R, C);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_log_softmax_bwd_f32(const float* g, const float* y, float* dx, int R, int C) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(g && y && dx, "tt_log_softmax_bwd_f32: null pointer");
  if (int rc = check_rows("tt_log_softmax_bwd_f32", R, C)) return rc;
  log_softmax_rows_bwd<<<(R + kWavesPerBlock - 1) / kWavesPerBlock, kThreads, 0, tt::stream()>>>(g, y, dx, R, C);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_nll_loss_fwd_f32(const float* logp, const long long* target, const float* weight, float* out,
                        float* count, int R, int C, long long ignore_index, int reduction) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(logp && target && out && count, "tt_nll_loss_fwd_f32: null pointer");
  TT_REQUIRE(reduction >= 0 && reduction <= 2, "tt_nll_loss_fwd_f32: reduction must be 0 (none), 1 (sum) or 2 (mean)");
  if (int rc = check_rows("tt_nll_loss_fwd_f32", R, C)) return rc;
  nll_loss_fwd<<<1, kThreads, 0, tt::stream()>>>(logp, target, weight, out, count, R, C, ignore_index, reduction);
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_nll_loss_bwd_f32(const float* g, const long long* target, const float* weight, const float* count,
                        float* dlogp, int R, int C, long long ignore_index, int reduction) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(g && target && count && dlogp, "tt_nll_loss_bwd_f32: null pointer");
  TT_REQUIRE(reduction >= 0 && reduction <= 2, "tt_nll_loss_bwd_f32: reduction must be 0 (none), 1 (sum) or 2 (mean)");
  if (int rc = check_rows("tt_nll_loss_bwd_f32", R, C)) return rc;
  const size_t total = (size_t)R * C;
  nll_loss_bwd<<<blocks_for(total), kThreads, 0, tt::stream()>>>(g, target, weight, count, dlogp, total,
                                                                tt::make_fastdiv((uint32_t)C), C, ignore_index,
                                                                reduction);
  TT_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
