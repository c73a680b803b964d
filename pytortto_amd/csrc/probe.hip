// Hardware calibration probes: what this GPU sustains on the two resources the path is bound
// by, measured with nothing else in the way.  bench.py reports them next to the published
// peaks so that a roofline fraction can be read against both.
#include "tt_common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Back-to-back v_mfma_f32_32x32x2_f32 on four accumulators with operands that differ per lane
// and per step (constant operands toggle fewer bits, draw less power and clock higher).
__global__ __launch_bounds__(256) void probe_mfma(const float* __restrict__ rnd, float* __restrict__ out, int iters) {
  floatx16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  float a[8], b[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    a[u] = rnd[(threadIdx.x * 16 + u) & 4095];
    b[u] = rnd[(threadIdx.x * 16 + 8 + u + blockIdx.x) & 4095];
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[(u + i) & 7], b[(u + 2 * i) & 7], acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void probe_fill_random(float* __restrict__ p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) {
    uint32_t h = (uint32_t)i * 2654435761u;
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
    p[i] = ((float)(h & 0xffff) / 65536.f - 0.5f) * 4.f;
  }
}

// Each block copies (kCopy) or reads (!kCopy) one contiguous 16 KiB chunk.
template <bool kCopy>
__global__ __launch_bounds__(256) void probe_stream(const floatx4* __restrict__ a, floatx4* __restrict__ b, float* sink) {
  const size_t base = (size_t)blockIdx.x * 1024;
  floatx4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) v[u] = a[base + threadIdx.x + 256 * u];
  if (kCopy) {
#pragma unroll
    for (int u = 0; u < 4; ++u) b[base + threadIdx.x + 256 * u] = v[u];
  } else {
    const float s = (v[0][0] + v[1][1]) + (v[2][2] + v[3][3]);
    if (s == 12345.678f) sink[0] = s;
  }
}

}  // namespace

extern "C" {

int tt_probe_mfma_f32(int launches, double* tflops_mean, double* tflops_min, double* tflops_max) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(launches > 0 && launches <= 1000, "tt_probe_mfma_f32: launches must be in 1..1000");
  const int blocks = 1024, iters = 500;   // about 1.3 ms per launch at 100 TFLOP/s
  void* ws;
  const size_t out_bytes = (size_t)blocks * 256 * sizeof(float);
  if (tt::workspace(out_bytes + 4096 * sizeof(float), &ws)) return -1;
  float* out = (float*)ws;
  float* rnd = (float*)((char*)ws + out_bytes);
  hipStream_t st = tt::stream();
  probe_fill_random<<<16, 256, 0, st>>>(rnd, 4096);
  probe_mfma<<<blocks, 256, 0, st>>>(rnd, out, iters);   // warm-up
  TT_LAUNCH_CHECK();
  hipEvent_t e0, e1;
  TT_HIP(hipEventCreate(&e0));
  TT_HIP(hipEventCreate(&e1));
  const double flops = (double)blocks * 4 * iters * 32 * 4096.0;
  double sum = 0, lo = 1e30, hi = 0;
  for (int i = 0; i < launches; ++i) {
    TT_HIP(hipEventRecord(e0, st));
    probe_mfma<<<blocks, 256, 0, st>>>(rnd, out, iters);
    TT_HIP(hipEventRecord(e1, st));
    TT_HIP(hipEventSynchronize(e1));
    float ms = 0.f;
    TT_HIP(hipEventElapsedTime(&ms, e0, e1));
    const double tf = flops / ((double)ms * 1e-3) / 1e12;
    sum += tf;
    lo = tf < lo ? tf : lo;
    hi = tf > hi ? tf : hi;
  }
  TT_HIP(hipEventDestroy(e0));
  TT_HIP(hipEventDestroy(e1));
  if (tflops_mean) *tflops_mean = sum / launches;
  if (tflops_min) *tflops_min = lo;
  if (tflops_max) *tflops_max = hi;
  return 0;
}

int tt_probe_hbm_f32(size_t bytes, double* read_gbs, double* copy_gbs) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(bytes >= ((size_t)64 << 20), "tt_probe_hbm_f32: use at least 64 MiB (far beyond the caches)");
  bytes = bytes / 16384 * 16384;
  void *a = nullptr, *b = nullptr;
  TT_HIP(hipMalloc(&a, bytes));
  if (hipMalloc(&b, bytes) != hipSuccess) {
    (void)hipFree(a);
    return tt::fail(-1, "tt_probe_hbm_f32: out of device memory");
  }
  hipStream_t st = tt::stream();
  TT_HIP(hipMemsetAsync(a, 1, bytes, st));
  TT_HIP(hipMemsetAsync(b, 0, bytes, st));
  void* ws;
  if (tt::workspace(256, &ws)) return -1;
  const unsigned blocks = (unsigned)(bytes / 16384);
  hipEvent_t e0, e1;
  TT_HIP(hipEventCreate(&e0));
  TT_HIP(hipEventCreate(&e1));
  float ms_r = 0.f, ms_c = 0.f;
  for (int rep = 0; rep < 2; ++rep) {   // second repetition is the measurement
    TT_HIP(hipEventRecord(e0, st));
    probe_stream<false><<<blocks, 256, 0, st>>>((const floatx4*)a, (floatx4*)b, (float*)ws);
    TT_HIP(hipEventRecord(e1, st));
    TT_HIP(hipEventSynchronize(e1));
    TT_HIP(hipEventElapsedTime(&ms_r, e0, e1));
    TT_HIP(hipEventRecord(e0, st));
    probe_stream<true><<<blocks, 256, 0, st>>>((const floatx4*)a, (floatx4*)b, (float*)ws);
    TT_HIP(hipEventRecord(e1, st));
    TT_HIP(hipEventSynchronize(e1));
    TT_HIP(hipEventElapsedTime(&ms_c, e0, e1));
  }
  TT_HIP(hipEventDestroy(e0));
  TT_HIP(hipEventDestroy(e1));
  TT_HIP(hipFree(a));
  TT_HIP(hipFree(b));
  if (read_gbs) *read_gbs = (double)bytes / ((double)ms_r * 1e-3) / 1e9;
  if (copy_gbs) *copy_gbs = 2.0 * (double)bytes / ((double)ms_c * 1e-3) / 1e9;
  return 0;
}

}  // extern "C"
