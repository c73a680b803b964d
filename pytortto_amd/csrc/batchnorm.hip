// BatchNorm2d training forward/backward for NCHW float32 on gfx950 -- HBM-bound kernels.
//
// x is viewed as [N, C, HW]: channel c owns N planes of HW contiguous floats, C*HW apart.
// Forward  = sweep 1 (read x: per-channel shifted moments)  + sweep 2 (read x, write y).
// Backward = sweep 1 (read x, dy: sum dy, sum dy*(x-mean))  + sweep 2 (read x, dy, write dx).
// Algorithmic traffic: 3*S forward, 5*S backward, S = 4*N*C*HW bytes.
//
// Grid is (splits, C): one block column per channel, `splits` blocks share a channel's planes
// so that even C = 64 fills 256 CUs.  Each block leaves an fp64 partial; the second sweep's
// blocks each re-reduce their channel's <= 64 partials in their prologue (cheaper than a
// separate finalize launch), and the block with split 0 writes the per-channel outputs.
// The second sweep walks channels, splits and planes in the opposite order of the first one,
// so what the first sweep touched last -- still resident in the memory-side cache -- is read
// first.
//
// Numerics: moments are taken about shift = x[0,c,0,0] (a sample of the channel, so within a
// few sigma of its mean): float32 accumulation inside one plane per lane, float64 across
// planes, lanes, waves and blocks; var = E[d^2] - E[d]^2 in float64.  This keeps the
// cancellation that a raw one-pass E[x^2]-E[x]^2 suffers for inputs with |mean| >> sigma away.
#include "tt_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / tt::kWave;
constexpr int kMaxSplits = 64;

// ---- wave64 all-reduce (sum) with DPP + ds_swizzle ------------------------------------------

template <int kCtrl>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, false));
}
template <int kCtrl>
__device__ __forceinline__ double dpp_d(double v) {
  int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), kCtrl, 0xf, 0xf, false);
  int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), kCtrl, 0xf, 0xf, false);
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double swz16_d(double v) {  // lane ^ 16 inside each 32-lane half
  int lo = __builtin_amdgcn_ds_swizzle(__double2loint(v), 0x401f);
  int hi = __builtin_amdgcn_ds_swizzle(__double2hiint(v), 0x401f);
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double readlane_d(double v, int lane) {
  int lo = __builtin_amdgcn_readlane(__double2loint(v), lane);
  int hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
  return __hiloint2double(hi, lo);
}

// Sum over the 64 lanes of a wave; every lane gets the (wave-uniform) result.
__device__ __forceinline__ double wave_sum(double v) {
  v += dpp_d<0xB1>(v);   // quad_perm [1,0,3,2]   : lane ^ 1
  v += dpp_d<0x4E>(v);   // quad_perm [2,3,0,1]   : lane ^ 2
  v += dpp_d<0x141>(v);  // row_half_mirror       : joins the two quads of each 8
  v += dpp_d<0x140>(v);  // row_mirror            : joins the two 8s of each row of 16
  v += swz16_d(v);       // joins the two rows of each 32-lane half
  return readlane_d(v, 0) + readlane_d(v, 32);
}

// Two sums per block: wave_sum, then the waves through LDS in wave order.  Result valid in all threads.
template <int WAVES = kWaves>
__device__ __forceinline__ void block_sum2(double& a, double& b, double* lds /* 2*WAVES */) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    lds[2 * wave] = a;
    lds[2 * wave + 1] = b;
  }
  __syncthreads();
  a = 0;
  b = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    a += lds[2 * w];
    b += lds[2 * w + 1];
  }
  __syncthreads();
}

// Re-reduce one channel's partials (<= 64, one per lane) -- wave-uniform result.
__device__ __forceinline__ void load_partials(const double2* __restrict__ partial, int c, int splits,
                                              double& a, double& b) {
  const int lane = threadIdx.x & 63;
  double2 p = make_double2(0.0, 0.0);
  if (lane < splits) p = partial[(size_t)c * splits + lane];
  a = wave_sum(p.x);
  b = wave_sum(p.y);
}

typedef float fx4 __attribute__((ext_vector_type(4)));
// Streaming accesses: data that is not read again soon should not displace what is (the input x is
// swept twice per pass) from the L2 and the memory-side cache.
__device__ __forceinline__ float4 load_stream(const float4* p) {
  const fx4 v = __builtin_nontemporal_load(reinterpret_cast<const fx4*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store_stream(float4* p, const float4 o) {
  const fx4 v = {o.x, o.y, o.z, o.w};
  __builtin_nontemporal_store(v, reinterpret_cast<fx4*>(p));
}

// ReLU fused behind the normalisation (tt_bn_relu_*): forward y = max(bn(x), 0) keeping NaN, as
// NumPy's maximum does (autograd/grad_nn.py:56); backward g = dy * (y > 0) as a product (:67), so
// that a non-finite dy at a masked element gives NaN like the unfused pair of kernels.
__device__ __forceinline__ float relu1(float v) { return (v > 0.f || v != v) ? v : 0.f; }
__device__ __forceinline__ float4 relu4(float4 v) { return make_float4(relu1(v.x), relu1(v.y), relu1(v.z), relu1(v.w)); }
__device__ __forceinline__ float mask1(float g, float y) { return g * (y > 0.f ? 1.f : 0.f); }
__device__ __forceinline__ float4 mask4(float4 g, float4 y) {
  return make_float4(mask1(g.x, y.x), mask1(g.y, y.y), mask1(g.z, y.z), mask1(g.w, y.w));
}

constexpr int kStreamU = 8;   // float4 loads in flight per thread in the stream reduce kernel

struct Geometry {
  int N, C, HW;         // HW in floats
  int splits;           // gridDim.x
  int per_block;        // planes (plane kernels) or vectors (flat kernels) per block
  tt::FastDiv hwv_div;  // flat kernels: divisor HW / VEC
};

// ---- sweep 1: partial sums ---------------------------------------------------------------------
// kKind 0: a = sum (x - shift),  b = sum (x - shift)^2         (shift = x[0,c,0,0])
// kKind 1: a = sum dy,           b = sum dy * (x - mean[c])
// kKind 2: a = sum x,            b unused                        (bias gradient)

// Plane kernel: HW % 4 == 0 and HW/4 >= 32.  Each wave streams whole planes with float4 loads.
template <int kKind>
__global__ __launch_bounds__(kThreads) void bn_reduce_planes(const float* __restrict__ x,
                                                             const float* __restrict__ dy,
                                                             const float* __restrict__ mean,
                                                             double2* __restrict__ partial, Geometry g) {
  __shared__ double lds[2 * kWaves];
  const int c = blockIdx.y, split = blockIdx.x;
  constexpr bool kBwd = kKind == 1;
  const int hw4 = g.HW >> 2;
  const float ref = kKind == 1 ? mean[c] : (kKind == 0 ? x[(size_t)c * g.HW] : 0.f);
  const int n0 = split * g.per_block;
  const int n1 = min(g.N, n0 + g.per_block);
  double sa = 0.0, sb = 0.0;
  // The whole block streams one plane at a time (a contiguous HW*4-byte region): batches of kU
  // float4 loads per thread, all issued before the first is consumed; threads past the end of
  // the plane take `ref` (a zero contribution) instead of branching out.
  constexpr int kU = kBwd ? 2 : 4;
  const float4 fill = make_float4(ref, ref, ref, ref);
  for (int n = n0; n < n1; ++n) {
    const size_t off = ((size_t)n * g.C + c) * g.HW;
    const float4* __restrict__ px = reinterpret_cast<const float4*>(x + off);
    const float4* __restrict__ pg = reinterpret_cast<const float4*>(dy + (kBwd ? off : 0));
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
    for (int i0 = threadIdx.x; i0 < hw4; i0 += kThreads * kU) {
      float4 v[kU], gq[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int i = i0 + kThreads * u;
        v[u] = i < hw4 ? px[i] : fill;
        if (kBwd) gq[u] = i < hw4 ? pg[i] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        float4 d = v[u];
        d.x -= ref; d.y -= ref; d.z -= ref; d.w -= ref;
        if (kBwd) {
          a.x += gq[u].x; a.y += gq[u].y; a.z += gq[u].z; a.w += gq[u].w;
          b.x = fmaf(gq[u].x, d.x, b.x); b.y = fmaf(gq[u].y, d.y, b.y);
          b.z = fmaf(gq[u].z, d.z, b.z); b.w = fmaf(gq[u].w, d.w, b.w);
        } else {
          a.x += d.x; a.y += d.y; a.z += d.z; a.w += d.w;
          if (kKind == 0) {
            b.x = fmaf(d.x, d.x, b.x); b.y = fmaf(d.y, d.y, b.y);
            b.z = fmaf(d.z, d.z, b.z); b.w = fmaf(d.w, d.w, b.w);
          }
        }
      }
    }
    sa += ((double)a.x + (double)a.y) + ((double)a.z + (double)a.w);
    sb += ((double)b.x + (double)b.y) + ((double)b.z + (double)b.w);
  }
  block_sum2(sa, sb, lds);
  if (threadIdx.x == 0) partial[(size_t)c * g.splits + split] = make_double2(sa, sb);
}

// Stream kernel: HW % 4 == 0.  A block takes a contiguous range of the channel's N*HW/4 float4
// vectors (flattened over planes, so no batch is cut short at a plane end) and issues kU loads
// per tensor and thread before it consumes the first: enough bytes in flight per block that the
// reduction tails of other blocks do not leave the memory system idle.
template <int kKind, bool kRelu = false>
__global__ __launch_bounds__(kThreads) void bn_reduce_stream(const float* __restrict__ x,
                                                             const float* __restrict__ dy,
                                                             const float* __restrict__ mean,
                                                             double2* __restrict__ partial, Geometry g,
                                                             const float* __restrict__ ry = nullptr) {
  __shared__ double lds[2 * kWaves];
  const int c = blockIdx.y, split = blockIdx.x;
  constexpr bool kBwd = kKind == 1;
  constexpr int kU = kBwd ? kStreamU / 2 : kStreamU;
  const uint32_t hwv = (uint32_t)g.HW >> 2;
  const uint32_t total = (uint32_t)g.N * hwv;
  const float ref = kKind == 1 ? mean[c] : (kKind == 0 ? x[(size_t)c * g.HW] : 0.f);
  const uint32_t e0 = (uint32_t)split * (uint32_t)g.per_block;
  const uint32_t e1 = min(total, e0 + (uint32_t)g.per_block);
  const float4 fill = make_float4(ref, ref, ref, ref);
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  double sa = 0.0, sb = 0.0;
  for (uint32_t base = e0; base < e1; base += kThreads * kU) {
    float4 v[kU], gq[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const uint32_t e = base + threadIdx.x + kThreads * u;
      const bool ok = e < e1;
      const uint32_t ee = ok ? e : e0;   // past the end: re-read a valid vector, use the neutral value
      const uint32_t n = tt::fd_div(ee, g.hwv_div);
      const size_t off = ((size_t)n * g.C + c) * g.HW + (size_t)(ee - n * hwv) * 4;
      const float4 t = *reinterpret_cast<const float4*>(x + off);
      v[u] = ok ? t : fill;
      if constexpr (kBwd) {
        // dy is streamed in both backward sweeps: x is read four times per training pass, dy twice,
        // and at these sizes the memory-side cache cannot hold both
        float4 q = load_stream(reinterpret_cast<const float4*>(dy + off));
        if constexpr (kRelu) q = mask4(q, load_stream(reinterpret_cast<const float4*>(ry + off)));
        gq[u] = ok ? q : zero;
      }
    }
    float4 a = zero, b = zero;
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      float4 d = v[u];
      d.x -= ref; d.y -= ref; d.z -= ref; d.w -= ref;
      if (kBwd) {
        a.x += gq[u].x; a.y += gq[u].y; a.z += gq[u].z; a.w += gq[u].w;
        b.x = fmaf(gq[u].x, d.x, b.x); b.y = fmaf(gq[u].y, d.y, b.y);
        b.z = fmaf(gq[u].z, d.z, b.z); b.w = fmaf(gq[u].w, d.w, b.w);
      } else {
        a.x += d.x; a.y += d.y; a.z += d.z; a.w += d.w;
        if (kKind == 0) {
          b.x = fmaf(d.x, d.x, b.x); b.y = fmaf(d.y, d.y, b.y);
          b.z = fmaf(d.z, d.z, b.z); b.w = fmaf(d.w, d.w, b.w);
        }
      }
    }
    sa += ((double)a.x + (double)a.y) + ((double)a.z + (double)a.w);
    sb += ((double)b.x + (double)b.y) + ((double)b.z + (double)b.w);
  }
  block_sum2(sa, sb, lds);
  if (threadIdx.x == 0) partial[(size_t)c * g.splits + split] = make_double2(sa, sb);
}

// Flat kernel: any HW.  Vector index e over the channel's N*HW/VEC vectors, n = e / (HW/VEC).
template <int kKind, int VEC, bool kRelu = false>
__global__ __launch_bounds__(kThreads) void bn_reduce_flat(const float* __restrict__ x,
                                                           const float* __restrict__ dy,
                                                           const float* __restrict__ mean,
                                                           double2* __restrict__ partial, Geometry g,
                                                           const float* __restrict__ ry = nullptr) {
  __shared__ double lds[2 * kWaves];
  const int c = blockIdx.y, split = blockIdx.x;
  const uint32_t hwv = (uint32_t)g.HW / VEC;
  constexpr bool kBwd = kKind == 1;
  const uint32_t total = (uint32_t)g.N * hwv;
  const float ref = kKind == 1 ? mean[c] : (kKind == 0 ? x[(size_t)c * g.HW] : 0.f);
  const uint32_t e0 = (uint32_t)split * (uint32_t)g.per_block;
  const uint32_t e1 = min(total, e0 + (uint32_t)g.per_block);
  double sa = 0.0, sb = 0.0;
  for (uint32_t e = e0 + threadIdx.x; e < e1; e += kThreads) {
    const uint32_t n = tt::fd_div(e, g.hwv_div);
    const uint32_t r = e - n * hwv;
    const size_t off = ((size_t)n * g.C + c) * g.HW + (size_t)r * VEC;
    float v[VEC], gq[VEC] = {};
    if constexpr (VEC == 4) {
      const float4 t = *reinterpret_cast<const float4*>(x + off);
      v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
      if constexpr (kBwd) {
        float4 u = *reinterpret_cast<const float4*>(dy + off);
        if constexpr (kRelu) u = mask4(u, *reinterpret_cast<const float4*>(ry + off));
        gq[0] = u.x; gq[1] = u.y; gq[2] = u.z; gq[3] = u.w;
      }
    } else {
      v[0] = x[off];
      if constexpr (kBwd) gq[0] = kRelu ? mask1(dy[off], ry[off]) : dy[off];
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float d = v[j] - ref;
      if (kBwd) {
        sa += (double)gq[j];
        sb += (double)gq[j] * (double)d;
      } else {
        sa += (double)d;
        if (kKind == 0) sb += (double)d * (double)d;
      }
    }
  }
  block_sum2(sa, sb, lds);
  if (threadIdx.x == 0) partial[(size_t)c * g.splits + split] = make_double2(sa, sb);
}

// ---- sweep 2: y = (x - m) * k1 + k0      (forward)
//               dx = dy * k1 + (x - m) * k2 + k0   (backward)
struct Coef {
  float m, k0, k1, k2;
};

template <bool kBwd>
__device__ __forceinline__ float4 apply4(const float4 v, const float4 gq, const Coef k) {
  float4 o;
  if (kBwd) {
    o.x = fmaf(gq.x, k.k1, fmaf(v.x - k.m, k.k2, k.k0));
    o.y = fmaf(gq.y, k.k1, fmaf(v.y - k.m, k.k2, k.k0));
    o.z = fmaf(gq.z, k.k1, fmaf(v.z - k.m, k.k2, k.k0));
    o.w = fmaf(gq.w, k.k1, fmaf(v.w - k.m, k.k2, k.k0));
  } else {
    o.x = fmaf(v.x - k.m, k.k1, k.k0);
    o.y = fmaf(v.y - k.m, k.k1, k.k0);
    o.z = fmaf(v.z - k.m, k.k1, k.k0);
    o.w = fmaf(v.w - k.m, k.k1, k.k0);
  }
  return o;
}

template <bool kBwd, bool kRelu>
__device__ __forceinline__ void sweep2_planes(const float* __restrict__ x, const float* __restrict__ dy,
                                              float* __restrict__ out, const Geometry& g, int c, int split,
                                              const Coef k, const float* __restrict__ ry) {
  const int hw4 = g.HW >> 2;
  const int n0 = split * g.per_block;
  const int n1 = min(g.N, n0 + g.per_block);
  constexpr int kU = kBwd ? 2 : 4;
  for (int n = n1 - 1; n >= n0; --n) {
    const size_t off = ((size_t)n * g.C + c) * g.HW;
    const float4* __restrict__ px = reinterpret_cast<const float4*>(x + off);
    const float4* __restrict__ pg = reinterpret_cast<const float4*>(dy + (kBwd ? off : 0));
    float4* __restrict__ po = reinterpret_cast<float4*>(out + off);
    const float4* __restrict__ pr = reinterpret_cast<const float4*>(ry + (kBwd && kRelu ? off : 0));
    for (int i0 = threadIdx.x; i0 < hw4; i0 += kThreads * kU) {
      float4 v[kU], gq[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int i = min(i0 + kThreads * u, hw4 - 1);   // clamped: out-of-range threads re-read, never store
        // backward: the last use of x and dy in the pass; forward: x is read again by the backward
        v[u] = kBwd ? load_stream(px + i) : px[i];
        gq[u] = kBwd ? load_stream(pg + i) : v[u];
        if constexpr (kBwd && kRelu) gq[u] = mask4(gq[u], load_stream(pr + i));
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int i = i0 + kThreads * u;
        if (i < hw4) {
          const float4 o = apply4<kBwd>(v[u], gq[u], k);
          store_stream(po + i, (!kBwd && kRelu) ? relu4(o) : o);
        }
      }
    }
  }
}

template <bool kBwd, int VEC, bool kRelu>
__device__ __forceinline__ void sweep2_flat(const float* __restrict__ x, const float* __restrict__ dy,
                                            float* __restrict__ out, const Geometry& g, int c, int split,
                                            const Coef k, const float* __restrict__ ry) {
  const uint32_t hwv = (uint32_t)g.HW / VEC;
  const uint32_t total = (uint32_t)g.N * hwv;
  const uint32_t e0 = (uint32_t)split * (uint32_t)g.per_block;
  const uint32_t e1 = min(total, e0 + (uint32_t)g.per_block);
  for (uint32_t e = e0 + threadIdx.x; e < e1; e += kThreads) {
    const uint32_t n = tt::fd_div(e, g.hwv_div);
    const uint32_t r = e - n * hwv;
    const size_t off = ((size_t)n * g.C + c) * g.HW + (size_t)r * VEC;
    if constexpr (VEC == 4) {
      const float4* px = reinterpret_cast<const float4*>(x + off);
      const float4 v = kBwd ? load_stream(px) : *px;
      float4 gq = v;
      if (kBwd) gq = load_stream(reinterpret_cast<const float4*>(dy + off));
      if constexpr (kBwd && kRelu) gq = mask4(gq, load_stream(reinterpret_cast<const float4*>(ry + off)));
      const float4 o = apply4<kBwd>(v, gq, k);
      store_stream(reinterpret_cast<float4*>(out + off), (!kBwd && kRelu) ? relu4(o) : o);
    } else {
      const float v = kBwd ? __builtin_nontemporal_load(x + off) : x[off];
      float o;
      if (kBwd) {
        float gv = __builtin_nontemporal_load(dy + off);
        if constexpr (kRelu) gv = mask1(gv, __builtin_nontemporal_load(ry + off));
        o = fmaf(gv, k.k1, fmaf(v - k.m, k.k2, k.k0));
      } else {
        o = fmaf(v - k.m, k.k1, k.k0);
        if constexpr (kRelu) o = relu1(o);
      }
      __builtin_nontemporal_store(o, out + off);
    }
  }
}

struct FwdArgs {
  const float* x;
  const float* gamma;
  const float* beta;
  float* y;
  float* save_mean;
  float* save_var_eps;
  float* save_sd;
  const float* rm_in;
  const float* rv_in;
  float* rm_out;
  float* rv_out;
  const float* given_mean;  // eval mode: statistics are inputs, no partials
  const float* given_var;
  const double2* partial;
  int partial_splits;       // partials per channel written by the first sweep
  float one_minus_mom, mom, unbias, eps;
  float* nbt;               // training: the module's batch counter, incremented by one (may be null)
};

// kMode: 0 planes, 1 flat VEC=4, 2 flat VEC=1
template <int kMode, bool kRelu = false>
__global__ __launch_bounds__(kThreads) void bn_fwd_apply(FwdArgs a, Geometry g) {
  __shared__ Coef sk;
  const int c = g.C - 1 - (int)blockIdx.y;
  const int split = g.splits - 1 - (int)blockIdx.x;
  if (threadIdx.x < tt::kWave) {
    float mean, var;
    if (a.given_mean) {
      mean = a.given_mean[c];
      var = a.given_var[c];
    } else {
      double s1, s2;
      load_partials(a.partial, c, a.partial_splits, s1, s2);
      const double m = (double)g.N * (double)g.HW;
      const double shift = (double)a.x[(size_t)c * g.HW];
      const double d1 = s1 / m;
      mean = (float)(shift + d1);
      var = (float)fmax(s2 / m - d1 * d1, 0.0);
    }
    const float var_eps = __fadd_rn(var, a.eps);
    const float sd = __fsqrt_rn(var_eps);
    const float gam = a.gamma ? a.gamma[c] : 1.0f;
    const float bet = a.beta ? a.beta[c] : 0.0f;
    if (threadIdx.x == 0) {
      sk.m = mean;
      sk.k1 = __fdiv_rn(gam, sd);
      sk.k0 = bet;
      sk.k2 = 0.f;
      if (split == 0) {
        a.save_mean[c] = mean;
        a.save_var_eps[c] = var_eps;
        a.save_sd[c] = sd;
        if (a.rm_in && !a.given_mean) {
          // separate roundings, as NumPy evaluates (1-m)*rm + m*mean on float32 arrays
          a.rm_out[c] = __fadd_rn(__fmul_rn(a.one_minus_mom, a.rm_in[c]), __fmul_rn(a.mom, mean));
          a.rv_out[c] =
              __fadd_rn(__fmul_rn(a.one_minus_mom, a.rv_in[c]), __fmul_rn(a.mom, __fmul_rn(var, a.unbias)));
        }
        if (a.nbt && c == 0) *a.nbt = __fadd_rn(*a.nbt, 1.0f);   // one thread of the whole grid
      }
    }
  }
  __syncthreads();
  const Coef k = sk;
  if (kMode == 0) sweep2_planes<false, kRelu>(a.x, a.x, a.y, g, c, split, k, a.x);
  if (kMode == 1) sweep2_flat<false, 4, kRelu>(a.x, a.x, a.y, g, c, split, k, a.x);
  if (kMode == 2) sweep2_flat<false, 1, kRelu>(a.x, a.x, a.y, g, c, split, k, a.x);
}

struct BwdArgs {
  const float* x;
  const float* dy;
  const float* gamma;
  const float* save_mean;
  const float* save_var_eps;
  const float* save_sd;
  float* dx;
  float* dgamma;
  float* dbeta;
  const double2* partial;
  int partial_splits;
  const float* ry;   // fused ReLU backward: the ReLU's output; dy is masked by (ry > 0) on the fly
};

template <int kMode, bool kRelu = false>
__global__ __launch_bounds__(kThreads) void bn_bwd_apply(BwdArgs a, Geometry g) {
  __shared__ Coef sk;
  const int c = g.C - 1 - (int)blockIdx.y;
  const int split = g.splits - 1 - (int)blockIdx.x;
  if (threadIdx.x < tt::kWave) {
    double s_dy, s_dyxmu;
    load_partials(a.partial, c, a.partial_splits, s_dy, s_dyxmu);
    if (threadIdx.x == 0) {
      const double m = (double)g.N * (double)g.HW;
      const double sd = (double)a.save_sd[c];
      const double var_eps = (double)a.save_var_eps[c];
      const double k1 = (a.gamma ? (double)a.gamma[c] : 1.0) / sd;
      sk.m = a.save_mean[c];
      sk.k1 = (float)k1;
      sk.k0 = (float)(-k1 * s_dy / m);
      sk.k2 = (float)(-k1 * s_dyxmu / (m * var_eps));
      if (split == 0) {
        if (a.dbeta) a.dbeta[c] = (float)s_dy;
        if (a.dgamma) a.dgamma[c] = (float)(s_dyxmu / sd);
      }
    }
  }
  if (a.dx == nullptr) return;
  __syncthreads();
  const Coef k = sk;
  if (kMode == 0) sweep2_planes<true, kRelu>(a.x, a.dy, a.dx, g, c, split, k, a.ry);
  if (kMode == 1) sweep2_flat<true, 4, kRelu>(a.x, a.dy, a.dx, g, c, split, k, a.ry);
  if (kMode == 2) sweep2_flat<true, 1, kRelu>(a.x, a.dy, a.dx, g, c, split, k, a.ry);
}

// ---- small channels: one kernel per pass ---------------------------------------------------------
// When a channel's N*HW values fit the registers of one block (<= BT * EMAX, BT threads), the block
// reads them once, reduces, and applies from registers: S read + S written forward, 2S + S
// backward instead of 3S and 5S, and one launch instead of two.  Grid = C blocks; g.hwv_div
// divides by HW.  The deep layers of a network (7x7 to 16x16 planes, hundreds of channels) are
// of this kind.  Statistics and coefficients follow the two-sweep kernels' formulas exactly.
// Larger channels take 64 values per thread, or -- when there are so few channels that a CU gets
// two blocks at most -- blocks of 1024 threads with 16 values each: more waves on a CU keep loads
// in flight while others reduce or store (measured, 256 channels of 64 x 14 x 14 values: backward
// 32 -> 15 us, forward 12.5 -> 10 us; 1024 such channels are 10 % slower that way and keep 256 threads).

template <int EMAX, int BT, typename F>
__device__ __forceinline__ void for_channel_elements(const Geometry& g, F&& f) {
  const int total = g.N * g.HW;
  const size_t image = (size_t)g.C * g.HW;
#pragma unroll
  for (int k = 0; k < EMAX; ++k) {
    const int e = (int)threadIdx.x + k * BT;
    if (e < total) {
      const uint32_t n = tt::fd_div((uint32_t)e, g.hwv_div);
      f(k, (size_t)n * image + ((uint32_t)e - n * (uint32_t)g.HW));
    }
  }
}

template <int EMAX, int BT, bool kRelu = false>
__global__ __launch_bounds__(BT) void bn_fwd_small(FwdArgs a, Geometry g) {
  __shared__ double red[2 * BT / tt::kWave];
  __shared__ Coef sk;
  // neighbouring channels share cache lines wherever a plane is not a whole number of lines (7x7: 196
  // bytes): blocks of one die (every eighth block of the grid) take a contiguous run of channels
  const int c = tt::xcd_remap((int)blockIdx.x, (int)gridDim.x);
  const float* __restrict__ xc = a.x + (size_t)c * g.HW;
  float* __restrict__ yc = a.y + (size_t)c * g.HW;
  const float shift = xc[0];
  float v[EMAX];
  for_channel_elements<EMAX, BT>(g, [&](int k, size_t off) { v[k] = xc[off]; });
  double s1 = 0.0, s2 = 0.0;
  for_channel_elements<EMAX, BT>(g, [&](int k, size_t) {
    const double d = (double)(v[k] - shift);
    s1 += d;
    s2 += d * d;
  });
  block_sum2<BT / tt::kWave>(s1, s2, red);
  if (threadIdx.x == 0) {
    const double m = (double)g.N * (double)g.HW;
    const double d1 = s1 / m;
    const float mean = (float)((double)shift + d1);
    const float var = (float)fmax(s2 / m - d1 * d1, 0.0);
    const float var_eps = __fadd_rn(var, a.eps);
    const float sd = __fsqrt_rn(var_eps);
    sk.m = mean;
    sk.k1 = __fdiv_rn(a.gamma ? a.gamma[c] : 1.0f, sd);
    sk.k0 = a.beta ? a.beta[c] : 0.0f;
    sk.k2 = 0.f;
    a.save_mean[c] = mean;
    a.save_var_eps[c] = var_eps;
    a.save_sd[c] = sd;
    if (a.rm_in) {   // separate roundings, as NumPy evaluates (1-m)*rm + m*mean on float32 arrays
      a.rm_out[c] = __fadd_rn(__fmul_rn(a.one_minus_mom, a.rm_in[c]), __fmul_rn(a.mom, mean));
      a.rv_out[c] = __fadd_rn(__fmul_rn(a.one_minus_mom, a.rv_in[c]), __fmul_rn(a.mom, __fmul_rn(var, a.unbias)));
    }
    if (a.nbt && c == 0) *a.nbt = __fadd_rn(*a.nbt, 1.0f);
  }
  __syncthreads();
  const Coef k = sk;
  for_channel_elements<EMAX, BT>(g, [&](int kk, size_t off) {
    const float o = fmaf(v[kk] - k.m, k.k1, k.k0);
    __builtin_nontemporal_store(kRelu ? relu1(o) : o, yc + off);
  });
}

template <int EMAX, int BT, bool kRelu = false>
__global__ __launch_bounds__(BT) void bn_bwd_small(BwdArgs a, Geometry g) {
  __shared__ double red[2 * BT / tt::kWave];
  __shared__ Coef sk;
  // neighbouring channels share cache lines wherever a plane is not a whole number of lines (7x7: 196
  // bytes): blocks of one die (every eighth block of the grid) take a contiguous run of channels
  const int c = tt::xcd_remap((int)blockIdx.x, (int)gridDim.x);
  const float* __restrict__ xc = a.x + (size_t)c * g.HW;
  const float* __restrict__ dyc = a.dy + (size_t)c * g.HW;
  const float mean = a.save_mean[c];
  float v[EMAX], gq[EMAX];
  for_channel_elements<EMAX, BT>(g, [&](int k, size_t off) {
    v[k] = __builtin_nontemporal_load(xc + off);
    gq[k] = __builtin_nontemporal_load(dyc + off);
    if constexpr (kRelu) gq[k] = mask1(gq[k], __builtin_nontemporal_load(a.ry + (size_t)c * g.HW + off));
  });
  double s_dy = 0.0, s_dyxmu = 0.0;
  for_channel_elements<EMAX, BT>(g, [&](int k, size_t) {
    s_dy += (double)gq[k];
    s_dyxmu += (double)gq[k] * (double)(v[k] - mean);
  });
  block_sum2<BT / tt::kWave>(s_dy, s_dyxmu, red);
  if (threadIdx.x == 0) {
    const double m = (double)g.N * (double)g.HW;
    const double sd = (double)a.save_sd[c];
    const double var_eps = (double)a.save_var_eps[c];
    const double k1 = (a.gamma ? (double)a.gamma[c] : 1.0) / sd;
    sk.m = mean;
    sk.k1 = (float)k1;
    sk.k0 = (float)(-k1 * s_dy / m);
    sk.k2 = (float)(-k1 * s_dyxmu / (m * var_eps));
    if (a.dbeta) a.dbeta[c] = (float)s_dy;
    if (a.dgamma) a.dgamma[c] = (float)(s_dyxmu / sd);
  }
  if (a.dx == nullptr) return;
  __syncthreads();
  const Coef k = sk;
  float* __restrict__ dxc = a.dx + (size_t)c * g.HW;
  for_channel_elements<EMAX, BT>(g, [&](int kk, size_t off) {
    __builtin_nontemporal_store(fmaf(gq[kk], k.k1, fmaf(v[kk] - k.m, k.k2, k.k0)), dxc + off);
  });
}

// ---- host side -------------------------------------------------------------------------------------

int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

// Channels small enough for the single-kernel passes, and enough of them to fill the device.
constexpr int kSmallValues = 16, kSmallValuesMax = 64;   // values per thread
constexpr int kSmallThreads = 1024;                     // threads of the larger block size
// 0: two-sweep kernels; 1: 256 threads x 16 values; 2: 256 x 64; 3: 1024 x 16
int small_channel_config(int N, int C, int HW) {
  const long long total = (long long)N * HW;
  if (C < 128 || total > (long long)kThreads * kSmallValuesMax) return 0;
  if (total <= (long long)kThreads * kSmallValues) return 1;
  return C <= 2 * tt::compute_units() ? 3 : 2;
}
Geometry small_geometry(int N, int C, int HW) {
  Geometry g{};
  g.N = N; g.C = C; g.HW = HW;
  g.splits = 1;
  g.per_block = 0;
  g.hwv_div = tt::make_fastdiv((uint32_t)HW);
  return g;
}

// Picks the kernel flavour and how a channel is shared between blocks.
constexpr int kStreamBatches = 4;
int plan(int N, int C, int HW, Geometry* g, int* mode) {
  g->N = N;
  g->C = C;
  g->HW = HW;
  const int target_blocks = 16384;  // many short-lived blocks: their start-up and reduction tails overlap other blocks' streaming
  int want = target_blocks / C;
  if (want < 1) want = 1;
  if (want > kMaxSplits) want = kMaxSplits;
  if (HW % 4 == 0 && HW / 4 >= 32) {
    *mode = 0;
    int ppb = ceil_div(N, want);
    g->per_block = ppb;
    g->splits = ceil_div(N, ppb);
    g->hwv_div = tt::make_fastdiv(1);
  } else {
    const int vec = (HW % 4 == 0) ? 4 : 1;
    *mode = vec == 4 ? 1 : 2;
    const long long vectors = (long long)N * (HW / vec);
    long long per = (vectors + want - 1) / want;
    per = (per + kThreads - 1) / kThreads * kThreads;
    g->per_block = (int)per;
    g->splits = ceil_div(vectors, per);
    g->hwv_div = tt::make_fastdiv((uint32_t)(HW / vec));
  }
  return 0;
}

int check_shape(const char* fn, int N, int C, int HW) {
  TT_REQUIRE(N > 0 && C > 0 && HW > 0, "%s: N, C, HW must be positive (got %d, %d, %d)", fn, N, C, HW);
  // element offsets are 64-bit; what must fit 32 bits are a channel's N*HW values (the index the
  // blocks split) and one image's C*HW
  TT_REQUIRE(tt::fits_i32((long long)N * HW) && tt::fits_i32((long long)C * HW),
             "%s: a channel (%lld values) or an image (%lld) exceeds 2^31-1 elements", fn, (long long)N * HW,
             (long long)C * HW);
  TT_REQUIRE(C <= 65535, "%s: more than 65535 channels are not supported", fn);
  return 0;
}

template <int kKind>
void launch_reduce(int mode, dim3 grid, const float* x, const float* dy, const float* mean, double2* partial,
                   const Geometry& g, const float* ry = nullptr) {
  hipStream_t st = tt::stream();
  if constexpr (kKind == 1) {
    if (ry) {   // backward behind a fused ReLU: dy is masked by (ry > 0) as it is read
      if (mode == 3) bn_reduce_stream<1, true><<<grid, kThreads, 0, st>>>(x, dy, mean, partial, g, ry);
      if (mode == 1) bn_reduce_flat<1, 4, true><<<grid, kThreads, 0, st>>>(x, dy, mean, partial, g, ry);
      if (mode == 2) bn_reduce_flat<1, 1, true><<<grid, kThreads, 0, st>>>(x, dy, mean, partial, g, ry);
      return;
    }
  }
  if (mode == 0) bn_reduce_planes<kKind><<<grid, kThreads, 0, st>>>(x, dy, mean, partial, g);
  if (mode == 3) bn_reduce_stream<kKind><<<grid, kThreads, 0, st>>>(x, dy, mean, partial, g);
  if (mode == 1) bn_reduce_flat<kKind, 4><<<grid, kThreads, 0, st>>>(x, dy, mean, partial, g);
  if (mode == 2) bn_reduce_flat<kKind, 1><<<grid, kThreads, 0, st>>>(x, dy, mean, partial, g);
}

// Geometry of the first sweep: the stream kernel when planes are float4-aligned, else as plan().
int plan_reduce(int N, int C, int HW, Geometry* g, int* mode) {
  plan(N, C, HW, g, mode);
  if (HW % 4 != 0) return 0;
  *mode = 3;
  const long long vectors = (long long)N * (HW / 4);
  const long long batch = (long long)kThreads * kStreamU;
  long long per = kStreamBatches * batch;                 // a few batches per block ...
  const long long min_per = (vectors + kMaxSplits - 1) / kMaxSplits;   // ... but at most kMaxSplits partials
  if (per < min_per) per = min_per;
  per = (per + batch - 1) / batch * batch;
  g->per_block = (int)per;
  g->splits = ceil_div(vectors, per);
  g->hwv_div = tt::make_fastdiv((uint32_t)(HW / 4));
  return 0;
}

// out[c] = sum of channel c's partials (bias gradient).
__global__ __launch_bounds__(tt::kWave) void channel_sum_finish(const double2* __restrict__ partial,
                                                               float* __restrict__ out, int splits) {
  double a, b;
  load_partials(partial, blockIdx.x, splits, a, b);
  if (threadIdx.x == 0) out[blockIdx.x] = (float)a;
}

// ---- fixed scratch for the entry point that allocates nothing -----------------------------------
// tt_bn_fwd_train_noalloc_f32 keeps the first sweep's partial moments here instead of in the
// library workspace: one double2 per (channel, reduction split), 256 KiB per device for the life
// of the process (enough for every tensor of at most 2^29 elements).  The array's name is only a host-side handle; its device address is looked up once
// per device (tt::bn_scratch_init, called by tt_init with that device current) and everything on
// the host uses that address.  Every slot a launch reads was written by the reduce kernel of the
// same call, so nothing needs clearing between calls; calls that overlap on one device would race.
constexpr int kScratchPartials = 16384;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) double2 scratch[kScratchPartials];
double2* g_scratch_ptr[kMaxDevices] = {};

}  // namespace

namespace tt {

int bn_scratch_init(int device) {
  TT_REQUIRE(device >= 0 && device < kMaxDevices, "device index %d beyond the %d the scratch table covers", device,
             kMaxDevices);
  if (g_scratch_ptr[device]) return 0;
  double2* ptr = nullptr;
  TT_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
  TT_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned a null address for the BatchNorm scratch array");
  g_scratch_ptr[device] = ptr;
  return 0;
}

}  // namespace tt

extern "C" {

// Training forward behind both entry points.  `fixed_partials` == nullptr: the partial moments of
// the first sweep go to the library workspace (grown on demand) and launches are bracketed for
// tt_profile_read.  Otherwise they go to that buffer of `fixed_capacity` entries and the call makes
// no allocation of any kind (no workspace growth, no event creation).
static int bn_fwd_train(const char* fn, const float* x, const float* gamma, const float* beta, float* y,
                        float* save_mean, float* save_var_eps, float* save_sd, const float* running_mean_in,
                        const float* running_var_in, float* running_mean_out, float* running_var_out,
                        float* num_batches_tracked, double momentum, double eps, int N, int C, int HW,
                        double2* fixed_partials, size_t fixed_capacity, bool relu = false) {
  TT_REQUIRE_INIT();
  if (check_shape(fn, N, C, HW)) return -1;
  TT_REQUIRE(x && y && save_mean && save_var_eps && save_sd, "%s: null tensor pointer", fn);
  TT_REQUIRE_ALIGNED(fn, x, y);
  const long long m = (long long)N * HW;
  TT_REQUIRE(m > 1, "Expected more than 1 value per channel when training, got input size [%d, %d, %d]", N, C, HW);
  const bool track = running_mean_in && running_var_in;
  TT_REQUIRE(!track || (running_mean_out && running_var_out), "%s: running statistics given without output buffers",
             fn);
  const bool timed = fixed_partials == nullptr;
  FwdArgs a{};
  a.x = x; a.gamma = gamma; a.beta = beta; a.y = y;
  a.save_mean = save_mean; a.save_var_eps = save_var_eps; a.save_sd = save_sd;
  a.rm_in = track ? running_mean_in : nullptr; a.rv_in = track ? running_var_in : nullptr;
  a.rm_out = running_mean_out; a.rv_out = running_var_out;
  a.given_mean = nullptr; a.given_var = nullptr;
  a.nbt = num_batches_tracked;
  a.one_minus_mom = (float)(1.0 - momentum);
  a.mom = (float)momentum;
  a.unbias = (float)((double)m / (double)(m - 1));
  a.eps = (float)eps;
  hipStream_t st = tt::stream();
  if (const int cfg = small_channel_config(N, C, HW)) {
    tt::ProfScope prof(timed ? TT_PROF_BN_FWD_APPLY : -1);
    const Geometry gs = small_geometry(N, C, HW);
    if (relu) {
      if (cfg == 1) bn_fwd_small<kSmallValues, kThreads, true><<<C, kThreads, 0, st>>>(a, gs);
      else if (cfg == 2) bn_fwd_small<kSmallValuesMax, kThreads, true><<<C, kThreads, 0, st>>>(a, gs);
      else bn_fwd_small<kSmallValues, kSmallThreads, true><<<C, kSmallThreads, 0, st>>>(a, gs);
    } else {
      if (cfg == 1) bn_fwd_small<kSmallValues, kThreads><<<C, kThreads, 0, st>>>(a, gs);
      else if (cfg == 2) bn_fwd_small<kSmallValuesMax, kThreads><<<C, kThreads, 0, st>>>(a, gs);
      else bn_fwd_small<kSmallValues, kSmallThreads><<<C, kSmallThreads, 0, st>>>(a, gs);
    }
    TT_LAUNCH_CHECK();
    return 0;
  }
  Geometry g, gr;
  int mode, rmode;
  plan(N, C, HW, &g, &mode);
  plan_reduce(N, C, HW, &gr, &rmode);
  const size_t partials = (size_t)C * gr.splits;
  double2* part = fixed_partials;
  if (part) {
    TT_REQUIRE(partials <= fixed_capacity,
               "%s: [%d, %d, %d] needs %zu partial moments, the fixed scratch array holds %zu "
               "(use tt_bn_fwd_train_f32, whose workspace grows)",
               fn, N, C, HW, partials, fixed_capacity);
  } else {
    void* ws;
    if (tt::workspace(sizeof(double2) * partials, &ws)) return -1;
    part = (double2*)ws;
  }
  dim3 grid(g.splits, C);
  {
    tt::ProfScope prof(timed ? TT_PROF_BN_FWD_REDUCE : -1);
    launch_reduce<0>(rmode, dim3(gr.splits, C), x, x, nullptr, part, gr);
  }
  TT_LAUNCH_CHECK();
  a.partial = part;
  a.partial_splits = gr.splits;
  {
    tt::ProfScope prof(timed ? TT_PROF_BN_FWD_APPLY : -1);
    if (relu) {
      if (mode == 0) bn_fwd_apply<0, true><<<grid, kThreads, 0, st>>>(a, g);
      if (mode == 1) bn_fwd_apply<1, true><<<grid, kThreads, 0, st>>>(a, g);
      if (mode == 2) bn_fwd_apply<2, true><<<grid, kThreads, 0, st>>>(a, g);
    } else {
      if (mode == 0) bn_fwd_apply<0><<<grid, kThreads, 0, st>>>(a, g);
      if (mode == 1) bn_fwd_apply<1><<<grid, kThreads, 0, st>>>(a, g);
      if (mode == 2) bn_fwd_apply<2><<<grid, kThreads, 0, st>>>(a, g);
    }
  }
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_bn_fwd_train_f32(const float* x, const float* gamma, const float* beta, float* y, float* save_mean,
                        float* save_var_eps, float* save_sd, const float* running_mean_in,
                        const float* running_var_in, float* running_mean_out, float* running_var_out,
                        float* num_batches_tracked, double momentum, double eps, int N, int C, int HW) {
  return bn_fwd_train("tt_bn_fwd_train_f32", x, gamma, beta, y, save_mean, save_var_eps, save_sd, running_mean_in,
                      running_var_in, running_mean_out, running_var_out, num_batches_tracked, momentum, eps, N, C, HW,
                      nullptr, 0);
}

int tt_bn_relu_fwd_train_f32(const float* x, const float* gamma, const float* beta, float* y, float* save_mean,
                             float* save_var_eps, float* save_sd, const float* running_mean_in,
                             const float* running_var_in, float* running_mean_out, float* running_var_out,
                             float* num_batches_tracked, double momentum, double eps, int N, int C, int HW) {
  return bn_fwd_train("tt_bn_relu_fwd_train_f32", x, gamma, beta, y, save_mean, save_var_eps, save_sd, running_mean_in,
                      running_var_in, running_mean_out, running_var_out, num_batches_tracked, momentum, eps, N, C, HW,
                      nullptr, 0, true);
}

int tt_bn_fwd_train_noalloc_f32(const float* x, const float* gamma, const float* beta, float* y, float* save_mean,
                                float* save_var_eps, float* save_sd, const float* running_mean_in,
                                const float* running_var_in, float* running_mean_out, float* running_var_out,
                                float* num_batches_tracked, double momentum, double eps, int N, int C, int HW) {
  TT_REQUIRE_INIT();
  int dev = -1;
  TT_HIP(hipGetDevice(&dev));
  TT_REQUIRE(dev >= 0 && dev < kMaxDevices && g_scratch_ptr[dev] != nullptr,
             "tt_bn_fwd_train_noalloc_f32: the scratch array of device %d was not set up by tt_init", dev);
  return bn_fwd_train("tt_bn_fwd_train_noalloc_f32", x, gamma, beta, y, save_mean, save_var_eps, save_sd,
                      running_mean_in, running_var_in, running_mean_out, running_var_out, num_batches_tracked, momentum,
                      eps, N, C, HW, g_scratch_ptr[dev], (size_t)kScratchPartials);
}

int tt_bn_fwd_eval_f32(const float* x, const float* gamma, const float* beta, float* y, const float* mean,
                       const float* var, float* save_mean, float* save_var_eps, float* save_sd, double eps, int N,
                       int C, int HW) {
  TT_REQUIRE_INIT();
  if (check_shape("tt_bn_fwd_eval_f32", N, C, HW)) return -1;
  TT_REQUIRE(x && y && mean && var && save_mean && save_var_eps && save_sd,
             "tt_bn_fwd_eval_f32: null tensor pointer");
  TT_REQUIRE_ALIGNED("tt_bn_fwd_eval_f32", x, y);
  Geometry g;
  int mode;
  plan(N, C, HW, &g, &mode);
  dim3 grid(g.splits, C);
  FwdArgs a{};
  a.x = x; a.gamma = gamma; a.beta = beta; a.y = y;
  a.save_mean = save_mean; a.save_var_eps = save_var_eps; a.save_sd = save_sd;
  a.given_mean = mean; a.given_var = var;
  a.eps = (float)eps;
  hipStream_t st = tt::stream();
  {
    tt::ProfScope prof(TT_PROF_BN_FWD_APPLY);
    if (mode == 0) bn_fwd_apply<0><<<grid, kThreads, 0, st>>>(a, g);
    if (mode == 1) bn_fwd_apply<1><<<grid, kThreads, 0, st>>>(a, g);
    if (mode == 2) bn_fwd_apply<2><<<grid, kThreads, 0, st>>>(a, g);
  }
  TT_LAUNCH_CHECK();
  return 0;
}

// Backward behind tt_bn_bwd_f32 (ry == nullptr) and tt_bn_relu_bwd_f32 (ry = the fused ReLU's output).
static int bn_bwd(const char* fn, const float* x, const float* dy, const float* ry, const float* gamma,
                  const float* save_mean, const float* save_var_eps, const float* save_sd, float* dx, float* dgamma,
                  float* dbeta, int N, int C, int HW) {
  TT_REQUIRE_INIT();
  if (check_shape(fn, N, C, HW)) return -1;
  TT_REQUIRE(x && dy && save_mean && save_var_eps && save_sd, "%s: null tensor pointer", fn);
  TT_REQUIRE_ALIGNED(fn, x, dy, dx, ry);
  if (!dx && !dgamma && !dbeta) return 0;
  if (const int cfg = small_channel_config(N, C, HW)) {
    tt::ProfScope prof(TT_PROF_BN_BWD_APPLY);
    const Geometry gs = small_geometry(N, C, HW);
    BwdArgs b{x, dy, gamma, save_mean, save_var_eps, save_sd, dx, dgamma, dbeta, nullptr, 0, ry};
    hipStream_t st = tt::stream();
    if (ry) {
      if (cfg == 1) bn_bwd_small<kSmallValues, kThreads, true><<<C, kThreads, 0, st>>>(b, gs);
      else if (cfg == 2) bn_bwd_small<kSmallValuesMax, kThreads, true><<<C, kThreads, 0, st>>>(b, gs);
      else bn_bwd_small<kSmallValues, kSmallThreads, true><<<C, kSmallThreads, 0, st>>>(b, gs);
    } else {
      if (cfg == 1) bn_bwd_small<kSmallValues, kThreads><<<C, kThreads, 0, st>>>(b, gs);
      else if (cfg == 2) bn_bwd_small<kSmallValuesMax, kThreads><<<C, kThreads, 0, st>>>(b, gs);
      else bn_bwd_small<kSmallValues, kSmallThreads><<<C, kSmallThreads, 0, st>>>(b, gs);
    }
    TT_LAUNCH_CHECK();
    return 0;
  }
  Geometry g, gr;
  int mode, rmode;
  plan(N, C, HW, &g, &mode);
  plan_reduce(N, C, HW, &gr, &rmode);
  void* ws;
  if (tt::workspace(sizeof(double2) * (size_t)C * gr.splits, &ws)) return -1;
  dim3 grid(g.splits, C);
  {
    tt::ProfScope prof(TT_PROF_BN_BWD_REDUCE);
    launch_reduce<1>(rmode, dim3(gr.splits, C), x, dy, save_mean, (double2*)ws, gr, ry);
  }
  TT_LAUNCH_CHECK();
  BwdArgs a{x, dy, gamma, save_mean, save_var_eps, save_sd, dx, dgamma, dbeta, (const double2*)ws, gr.splits, ry};
  hipStream_t st = tt::stream();
  {
    tt::ProfScope prof(TT_PROF_BN_BWD_APPLY);
    if (ry) {
      if (mode == 0) bn_bwd_apply<0, true><<<grid, kThreads, 0, st>>>(a, g);
      if (mode == 1) bn_bwd_apply<1, true><<<grid, kThreads, 0, st>>>(a, g);
      if (mode == 2) bn_bwd_apply<2, true><<<grid, kThreads, 0, st>>>(a, g);
    } else {
      if (mode == 0) bn_bwd_apply<0><<<grid, kThreads, 0, st>>>(a, g);
      if (mode == 1) bn_bwd_apply<1><<<grid, kThreads, 0, st>>>(a, g);
      if (mode == 2) bn_bwd_apply<2><<<grid, kThreads, 0, st>>>(a, g);
    }
  }
  TT_LAUNCH_CHECK();
  return 0;
}

int tt_bn_bwd_f32(const float* x, const float* dy, const float* gamma, const float* save_mean,
                  const float* save_var_eps, const float* save_sd, float* dx, float* dgamma, float* dbeta, int N,
                  int C, int HW) {
  return bn_bwd("tt_bn_bwd_f32", x, dy, nullptr, gamma, save_mean, save_var_eps, save_sd, dx, dgamma, dbeta, N, C, HW);
}

int tt_bn_relu_bwd_f32(const float* x, const float* dy, const float* relu_y, const float* gamma, const float* save_mean,
                       const float* save_var_eps, const float* save_sd, float* dx, float* dgamma, float* dbeta, int N,
                       int C, int HW) {
  TT_REQUIRE(relu_y != nullptr, "tt_bn_relu_bwd_f32: null ReLU output");
  return bn_bwd("tt_bn_relu_bwd_f32", x, dy, relu_y, gamma, save_mean, save_var_eps, save_sd, dx, dgamma, dbeta, N, C,
                HW);
}

int tt_channel_sum_f32(const float* t, float* out, int N, int K, int HW) {
  TT_REQUIRE_INIT();
  if (check_shape("tt_channel_sum_f32", N, K, HW)) return -1;
  TT_REQUIRE(t && out, "tt_channel_sum_f32: null tensor pointer");
  TT_REQUIRE_ALIGNED("tt_channel_sum_f32", t);
  Geometry g;
  int mode;
  plan_reduce(N, K, HW, &g, &mode);
  void* ws;
  if (tt::workspace(sizeof(double2) * (size_t)K * g.splits, &ws)) return -1;
  launch_reduce<2>(mode, dim3(g.splits, K), t, t, nullptr, (double2*)ws, g);
  TT_LAUNCH_CHECK();
  channel_sum_finish<<<K, tt::kWave, 0, tt::stream()>>>((const double2*)ws, out, g.splits);
  TT_LAUNCH_CHECK();
  return 0;
}

// Workspace of tt_bn_fwd_train_f32 and tt_bn_bwd_f32 alike: one double2 partial per channel and
// reduction split of the first sweep.
int tt_workspace_size_bn_f32(size_t* bytes, int N, int C, int HW) {
  TT_REQUIRE(bytes, "tt_workspace_size_bn_f32: null result pointer");
  if (check_shape("tt_workspace_size_bn_f32", N, C, HW)) return -1;
  if (small_channel_config(N, C, HW)) {   // single-kernel passes: no partials
    *bytes = 0;
    return 0;
  }
  Geometry gr;
  int rmode;
  plan_reduce(N, C, HW, &gr, &rmode);
  *bytes = sizeof(double2) * (size_t)C * gr.splits;
  return 0;
}

}  // extern "C"
