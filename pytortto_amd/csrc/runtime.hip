// Runtime of libtortto_hip.so: device selection, the library stream, a pooling allocator for
// the device arrays the Python side owns, the grow-only workspace, copies and events.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <unordered_map>
#include <vector>

#include "tt_common.h"

namespace {

thread_local char g_err[512] = "";

struct State {
  bool ready = false;
  int device = -1;
  int compute_units = 256;
  hipStream_t stream = nullptr;
  // pooling allocator: freed blocks are kept per rounded size and handed out again, so the
  // autograd loop does not pay hipMalloc/hipFree (which synchronises the device) per tensor
  std::unordered_map<void*, size_t> live;            // ptr -> rounded size
  std::map<size_t, std::vector<void*>> pool;         // rounded size -> free blocks
  size_t bytes_live = 0;
  size_t bytes_pooled = 0;
  void* ws = nullptr;
  size_t ws_bytes = 0;
  int conv_math = TT_CONV_MATH_F32;
  // per-kernel timing
  bool profiling = false;
  std::vector<hipEvent_t> event_pool;
  struct Pending {
    int id;
    hipEvent_t start, stop;
  };
  std::vector<Pending> pending;
  long long prof_launches[TT_PROF_COUNT] = {};
  double prof_ms[TT_PROF_COUNT] = {};
};

State& S() {
  static State s;
  return s;
}

size_t round_size(size_t bytes) {
  if (bytes == 0) bytes = 1;
  const size_t small = 512, big = (size_t)2 << 20;
  if (bytes <= ((size_t)1 << 20)) return (bytes + small - 1) / small * small;
  return (bytes + big - 1) / big * big;
}

int release_pool() {
  State& s = S();
  for (auto& kv : s.pool)
    for (void* p : kv.second) TT_HIP(hipFree(p));
  s.pool.clear();
  s.bytes_pooled = 0;
  return 0;
}

}  // namespace

namespace tt {

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code == 0 ? -1 : code;
}

int fail_hip(hipError_t e, const char* what, const char* file, int line) {
  const char* base = strrchr(file, '/');
  snprintf(g_err, sizeof(g_err), "HIP error %d (%s) in %s at %s:%d", (int)e, hipGetErrorString(e), what,
           base ? base + 1 : file, line);
  return (int)e;
}

std::recursive_mutex& api_mutex() {
  static std::recursive_mutex m;
  return m;
}

hipStream_t stream() { return S().stream; }
int compute_units() { return S().compute_units; }
int conv_math() { return S().conv_math; }
bool initialised() { return S().ready; }

int workspace(size_t bytes, void** out) {
  State& s = S();
  if (bytes > s.ws_bytes) {
    // kernels that still read the old block were enqueued earlier on the same stream
    TT_HIP(hipStreamSynchronize(s.stream));
    if (s.ws) TT_HIP(hipFree(s.ws));
    s.ws = nullptr;
    s.ws_bytes = 0;
    size_t want = round_size(bytes + bytes / 4);
    hipError_t e = hipMalloc(&s.ws, want);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      if (release_pool() != 0) return -1;
      TT_HIP(hipMalloc(&s.ws, want));
    }
    s.ws_bytes = want;
  }
  *out = s.ws;
  return 0;
}

ProfScope::ProfScope(int kernel_id) : id(kernel_id), start(nullptr) {
  State& s = S();
  if (!s.profiling || kernel_id < 0) return;   // a negative id: this launch is never timed
  hipEvent_t e = nullptr;
  if (!s.event_pool.empty()) {
    e = s.event_pool.back();
    s.event_pool.pop_back();
  } else if (hipEventCreate(&e) != hipSuccess) {
    return;
  }
  if (hipEventRecord(e, s.stream) != hipSuccess) {
    s.event_pool.push_back(e);
    return;
  }
  start = (void*)e;
}

ProfScope::~ProfScope() {
  if (!start) return;
  State& s = S();
  hipEvent_t e = nullptr;
  if (!s.event_pool.empty()) {
    e = s.event_pool.back();
    s.event_pool.pop_back();
  } else if (hipEventCreate(&e) != hipSuccess) {
    s.event_pool.push_back((hipEvent_t)start);
    return;
  }
  (void)hipEventRecord(e, s.stream);
  s.pending.push_back({id, (hipEvent_t)start, e});
}

FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d;
  uint32_t l = 0;
  while (((uint64_t)1 << l) < d) ++l;
  f.mul = (uint32_t)((((uint64_t)1 << 32) * (((uint64_t)1 << l) - d)) / d + 1);
  f.shift = l;
  return f;
}

}  // namespace tt

extern "C" {

const char* tt_last_error(void) { return g_err; }

int tt_init(int device) {
  TT_API_LOCK();
  State& s = S();
  if (s.ready) {
    TT_REQUIRE(device == s.device, "tt_init(%d): library already initialised on device %d", device, s.device);
    return 0;
  }
  int count = 0;
  TT_HIP(hipGetDeviceCount(&count));
  TT_REQUIRE(device >= 0 && device < count, "tt_init(%d): %d HIP device(s) visible", device, count);
  TT_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  TT_HIP(hipGetDeviceProperties(&prop, device));
  TT_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0,
             "libtortto_hip is built for gfx950 (MI355X) only; device %d is %s", device, prop.gcnArchName);
  TT_HIP(hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking));
  if (tt::bn_scratch_init(device)) return -1;   // device address of the fixed scratch array, once per device
  s.device = device;
  s.compute_units = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  s.ready = true;
  return 0;
}

int tt_device_info(char* name, int name_len, int* compute_units, int* clock_khz, int* lds_bytes_per_block,
                   size_t* total_mem_bytes) {
  TT_REQUIRE_INIT();
  hipDeviceProp_t prop;
  TT_HIP(hipGetDeviceProperties(&prop, S().device));
  if (name && name_len > 0) snprintf(name, (size_t)name_len, "%s (%s)", prop.name, prop.gcnArchName);
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (clock_khz) *clock_khz = prop.clockRate;
  if (lds_bytes_per_block) *lds_bytes_per_block = (int)prop.sharedMemPerBlock;
  if (total_mem_bytes) *total_mem_bytes = prop.totalGlobalMem;
  return 0;
}

int tt_malloc(void** ptr, size_t bytes) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(ptr != nullptr, "tt_malloc: null output pointer");
  State& s = S();
  size_t r = round_size(bytes);
  auto it = s.pool.find(r);
  void* p = nullptr;
  if (it != s.pool.end() && !it->second.empty()) {
    p = it->second.back();
    it->second.pop_back();
    s.bytes_pooled -= r;
  } else {
    hipError_t e = hipMalloc(&p, r);
    if (e != hipSuccess) {  // out of memory: give pooled blocks back and try once more
      (void)hipGetLastError();
      TT_HIP(hipStreamSynchronize(s.stream));
      if (release_pool() != 0) return -1;
      TT_HIP(hipMalloc(&p, r));
    }
  }
  s.live[p] = r;
  s.bytes_live += r;
  *ptr = p;
  return 0;
}

int tt_free(void* ptr) {
  if (ptr == nullptr) return 0;
  TT_REQUIRE_INIT();
  State& s = S();
  auto it = s.live.find(ptr);
  TT_REQUIRE(it != s.live.end(), "tt_free: %p was not allocated by tt_malloc (or freed twice)", ptr);
  size_t r = it->second;
  s.live.erase(it);
  s.bytes_live -= r;
  // Reuse is safe without waiting: every consumer of the old contents and every producer of
  // the new ones is ordered on the single library stream.
  s.pool[r].push_back(ptr);
  s.bytes_pooled += r;
  return 0;
}

int tt_empty_cache(void) {
  TT_REQUIRE_INIT();
  State& s = S();
  TT_HIP(hipStreamSynchronize(s.stream));
  if (release_pool() != 0) return -1;
  if (s.ws) TT_HIP(hipFree(s.ws));
  s.ws = nullptr;
  s.ws_bytes = 0;
  if (tt::conv_release_tables() || tt::wgrad_release_tables()) return -1;
  return 0;
}

int tt_mem_stats(size_t* bytes_in_use, size_t* bytes_pooled, size_t* workspace_bytes) {
  TT_REQUIRE_INIT();
  if (bytes_in_use) *bytes_in_use = S().bytes_live;
  if (bytes_pooled) *bytes_pooled = S().bytes_pooled;
  if (workspace_bytes) *workspace_bytes = S().ws_bytes;
  return 0;
}

int tt_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes) {
  TT_REQUIRE_INIT();
  if (bytes == 0) return 0;
  TT_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, S().stream));
  TT_HIP(hipStreamSynchronize(S().stream));
  return 0;
}

int tt_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes) {
  TT_REQUIRE_INIT();
  if (bytes == 0) return 0;
  TT_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, S().stream));
  TT_HIP(hipStreamSynchronize(S().stream));
  return tt::conv_check_async_error();
}

int tt_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes) {
  TT_REQUIRE_INIT();
  if (bytes == 0) return 0;
  TT_HIP(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, S().stream));
  return 0;
}

int tt_memset(void* dst_dev, int byte_value, size_t bytes) {
  TT_REQUIRE_INIT();
  if (bytes == 0) return 0;
  TT_HIP(hipMemsetAsync(dst_dev, byte_value, bytes, S().stream));
  return 0;
}

int tt_set_conv_math(int mode) {
  TT_API_LOCK();
  TT_REQUIRE(mode == TT_CONV_MATH_F32 || mode == TT_CONV_MATH_BF16 || mode == TT_CONV_MATH_BF16X3, "tt_set_conv_math: unknown mode %d", mode);
  S().conv_math = mode;
  return 0;
}

int tt_get_conv_math(int* mode) {
  TT_API_LOCK();
  TT_REQUIRE(mode != nullptr, "tt_get_conv_math: null output pointer");
  *mode = S().conv_math;
  return 0;
}

// The three convolution passes with another matrix arithmetic for this call only, whatever the
// process-wide mode is: the mode is switched under the API lock, which this thread holds for the
// whole call, so no other caller can see the switch.
namespace {
struct ScopedMath {
  int saved;
  explicit ScopedMath(int mode) : saved(S().conv_math) { S().conv_math = mode; }
  ~ScopedMath() { S().conv_math = saved; }
};
struct ScopedBf16 : ScopedMath {
  ScopedBf16() : ScopedMath(TT_CONV_MATH_BF16) {}
};
}  // namespace

int tt_conv2d_fwd_bf16(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K,
                       int R, int S_, int sh, int sw, int ph, int pw, int dh, int dw, int groups) {
  TT_API_LOCK();
  ScopedBf16 mode;
  return tt_conv2d_fwd_f32(x, w, bias, y, N, C, H, W, K, R, S_, sh, sw, ph, pw, dh, dw, groups);
}

int tt_conv2d_dgrad_bf16(const float* dy, const float* w, const float* bias, float* dx, int N, int C, int Hx, int Wx,
                         int K, int R, int S_, int sh, int sw, int ph, int pw, int dh, int dw, int groups, int P, int Q) {
  TT_API_LOCK();
  ScopedBf16 mode;
  return tt_conv2d_dgrad_f32(dy, w, bias, dx, N, C, Hx, Wx, K, R, S_, sh, sw, ph, pw, dh, dw, groups, P, Q);
}

int tt_conv2d_wgrad_bf16(const float* x, const float* dy, float* dw, int N, int C, int H, int W, int K, int R, int S_,
                         int sh, int sw, int ph, int pw, int dh, int dw_, int groups, int P, int Q) {
  TT_API_LOCK();
  ScopedBf16 mode;
  return tt_conv2d_wgrad_f32(x, dy, dw, N, C, H, W, K, R, S_, sh, sw, ph, pw, dh, dw_, groups, P, Q);
}

int tt_conv2d_fwd_bf16x3(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K,
                         int R, int S_, int sh, int sw, int ph, int pw, int dh, int dw, int groups) {
  TT_API_LOCK();
  ScopedMath mode(TT_CONV_MATH_BF16X3);
  return tt_conv2d_fwd_f32(x, w, bias, y, N, C, H, W, K, R, S_, sh, sw, ph, pw, dh, dw, groups);
}

int tt_conv2d_dgrad_bf16x3(const float* dy, const float* w, const float* bias, float* dx, int N, int C, int Hx, int Wx,
                           int K, int R, int S_, int sh, int sw, int ph, int pw, int dh, int dw, int groups, int P, int Q) {
  TT_API_LOCK();
  ScopedMath mode(TT_CONV_MATH_BF16X3);
  return tt_conv2d_dgrad_f32(dy, w, bias, dx, N, C, Hx, Wx, K, R, S_, sh, sw, ph, pw, dh, dw, groups, P, Q);
}

int tt_sync(void) {
  TT_REQUIRE_INIT();
  TT_HIP(hipStreamSynchronize(S().stream));
  return tt::conv_check_async_error();
}

int tt_profile_enable(int on) {
  TT_REQUIRE_INIT();
  State& s = S();
  TT_HIP(hipStreamSynchronize(s.stream));
  for (auto& p : s.pending) {
    s.event_pool.push_back(p.start);
    s.event_pool.push_back(p.stop);
  }
  s.pending.clear();
  for (int i = 0; i < TT_PROF_COUNT; ++i) {
    s.prof_launches[i] = 0;
    s.prof_ms[i] = 0.0;
  }
  s.profiling = on != 0;
  return 0;
}

int tt_profile_read(int kernel_id, long long* launches, double* total_ms) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(kernel_id >= 0 && kernel_id < TT_PROF_COUNT, "tt_profile_read: unknown kernel id %d", kernel_id);
  State& s = S();
  TT_HIP(hipStreamSynchronize(s.stream));
  for (auto& p : s.pending) {
    float ms = 0.f;
    TT_HIP(hipEventElapsedTime(&ms, p.start, p.stop));
    s.prof_launches[p.id] += 1;
    s.prof_ms[p.id] += (double)ms;
    s.event_pool.push_back(p.start);
    s.event_pool.push_back(p.stop);
  }
  s.pending.clear();
  if (launches) *launches = s.prof_launches[kernel_id];
  if (total_ms) *total_ms = s.prof_ms[kernel_id];
  return 0;
}

int tt_event_create(void** event) {
  TT_REQUIRE_INIT();
  hipEvent_t e;
  TT_HIP(hipEventCreate(&e));
  *event = (void*)e;
  return 0;
}

int tt_event_record(void* event) {
  TT_REQUIRE_INIT();
  TT_HIP(hipEventRecord((hipEvent_t)event, S().stream));
  return 0;
}

int tt_event_elapsed_ms(void* start, void* stop, float* ms) {
  TT_REQUIRE_INIT();
  TT_HIP(hipEventSynchronize((hipEvent_t)stop));
  TT_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return 0;
}

int tt_event_destroy(void* event) {
  TT_REQUIRE_INIT();
  TT_HIP(hipEventDestroy((hipEvent_t)event));
  return 0;
}

}  // extern "C"
