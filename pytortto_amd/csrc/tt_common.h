// Internal declarations shared by the translation units of libtortto_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <mutex>

#include "../../include/tortto_hip.h"

namespace tt {

// Records a message for tt_last_error() and returns a non-zero status.
int fail(int code, const char* fmt, ...);
int fail_hip(hipError_t e, const char* what, const char* file, int line);

// One lock serialises the C ABI: the allocator's maps, the workspace, the table caches and the
// profiling state are shared, and callers such as a Python process (ctypes releases the GIL
// during a call; a device array may be finalised on another thread) reach them from several
// threads.  Every entry point that touches that state holds the lock for its duration (calls only
// enqueue work, so it is held for microseconds; tt_sync and the synchronous copies hold it while
// they wait).  Recursive: entry points call each other.
std::recursive_mutex& api_mutex();

// The one stream every kernel of the library is enqueued on.
hipStream_t stream();
bool initialised();
// Compute units of the device tt_init() selected (256 on an MI355X): persistent grids, tile-count
// thresholds and the caps on grid-stride launches scale with it.
int compute_units();

// Grow-only scratch memory owned by the library (split-K partial sums, repacked weights,
// per-channel partial moments).  The pointer stays valid until the next call that asks for
// more; work on the stream is ordered, so consecutive launches may reuse it.
int workspace(size_t bytes, void** out);

// Looks up the device address of the fixed scratch array behind tt_bn_fwd_train_noalloc_f32 for
// `device`, which must be the current device (batchnorm.hip).  Called once per device by tt_init.
int bn_scratch_init(int device);

// Frees the per-geometry index tables of the convolution kernels (conv_igemm.hip) and the pixel
// tables of the weight gradient (conv_wgrad.hip); the caller has synchronised the stream.
int conv_release_tables();
int wgrad_release_tables();
// After a stream sync: reports (once) a convolution launch whose blocks gave up waiting for each other.
int conv_check_async_error();
// Device pointer of the one word (pinned host memory) that such a block sets; shared by the
// forward / input-gradient kernels and the weight gradient.
int conv_async_error_word(unsigned** device_pointer);

// Brackets the launches made during its lifetime with events when profiling is enabled
// (a negative kernel id switches it off for that scope).
struct ProfScope {
  explicit ProfScope(int kernel_id);
  ~ProfScope();
  int id;
  void* start;
};

constexpr int kWave = 64;

// Matrix arithmetic of the convolution kernels: TT_CONV_MATH_F32, _BF16 or _BF16X3 (tt_set_conv_math).
int conv_math();

inline bool fits_i32(long long elems) { return elems >= 0 && elems < 2147483647LL; }

// Unsigned division by a run-time constant without a divide instruction:
// q = (umulhi(n, mul) + n) >> shift, valid for n < 2^31.
struct FastDiv {
  uint32_t mul;
  uint32_t shift;
  uint32_t d;
};
FastDiv make_fastdiv(uint32_t d);

__device__ __forceinline__ uint32_t fd_div(uint32_t n, const FastDiv& f) {
  return (uint32_t)(((uint64_t)__umulhi(n, f.mul) + n) >> f.shift);
}

// Blocks are dealt round-robin to the 8 XCDs (each with its own L2) in launch order.  Maps block b
// of nb to a work index such that every XCD receives one contiguous range of work indices.
__device__ __forceinline__ int xcd_remap(int b, int nb) {
  const int q = nb >> 3, rem = nb & 7;
  const int xcd = b & 7, idx = b >> 3;
  return (xcd < rem ? xcd * (q + 1) : rem * (q + 1) + (xcd - rem) * q) + idx;
}

}  // namespace tt

#define TT_HIP(expr)                                                      \
  do {                                                                    \
    hipError_t _e = (expr);                                               \
    if (_e != hipSuccess) return tt::fail_hip(_e, #expr, __FILE__, __LINE__); \
  } while (0)

#define TT_REQUIRE(cond, ...)                     \
  do {                                            \
    if (!(cond)) return tt::fail(-1, __VA_ARGS__); \
  } while (0)

// Tensor pointers at the C ABI are 16-byte aligned (the kernels use 16-byte vector accesses);
// null pointers (optional arguments) pass.
namespace tt {
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
template <typename... P>
inline bool all_aligned16(P... ptrs) { return (aligned16(ptrs) && ...); }
}  // namespace tt
#define TT_REQUIRE_ALIGNED(fn, ...) \
  TT_REQUIRE(tt::all_aligned16(__VA_ARGS__), "%s: tensor pointers must be 16-byte aligned", fn)

#define TT_CAT2(a, b) a##b
#define TT_CAT(a, b) TT_CAT2(a, b)
#define TT_API_LOCK() std::lock_guard<std::recursive_mutex> TT_CAT(tt_api_lock_, __LINE__)(tt::api_mutex())
// Takes the API lock for the rest of the enclosing scope and refuses calls before tt_init().
#define TT_REQUIRE_INIT() \
  TT_API_LOCK();          \
  TT_REQUIRE(tt::initialised(), "tt_init() has not been called")

#define TT_LAUNCH_CHECK() TT_HIP(hipGetLastError())
