// Float32 convolution arithmetic on the bf16 matrix instructions of gfx950
// (tt_set_conv_math(TT_CONV_MATH_BF16X3)): the implicit-GEMM kernel body of conv_igemm_kernel.h with
// its three-term matrix step -- every operand value as three bfloat16 terms that add up to it exactly,
// six v_mfma_f32_32x32x16_bf16 per accumulator and 16-deep step -- for Conv2d forward and the input
// gradient.  Same tiles, stream-K grid, addressing modes and epilogues as the float32 kernels; the
// launch planning stays in conv_igemm.hip, which calls in here with the tile shape it chose.
#include "conv_igemm_kernel.h"

namespace {

using namespace ttc;

// The same launch in float32 arithmetic carried out on the bf16 matrix instructions; two blocks per CU.
template <int WM, int WN, int MT, int NT, bool SK, int MODE, bool AT>
__global__ __launch_bounds__(kThreads, 2) void igemm_bf16x3(const Igemm p) {
  igemm_body<WM, WN, MT, NT, SK, MODE, AT, 3>(p, (int)blockIdx.x);
}

template <int WM, int WN, int MT, int NT, int MODE>
__global__ __launch_bounds__(kThreads, 2) void igemm_multi_bf16x3(const IgemmMulti m) {
  int ci = 0;
  while (ci + 1 < m.n && (int)blockIdx.x >= m.first[ci + 1]) ++ci;
  igemm_body<WM, WN, MT, NT, false, MODE, false, 3>(m.c[ci], (int)blockIdx.x - m.first[ci]);
}

// Blocks of one stream-K instantiation a compute unit holds (asked once: registers and LDS of the
// compiled kernel decide it).
template <int WM, int WN, int MT, int NT, int MODE, bool AT>
int resident_blocks_per_cu() {
  static int cached = -1;
  if (cached < 0) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, igemm_bf16x3<WM, WN, MT, NT, true, MODE, AT>, kThreads, 0) != hipSuccess) {
      (void)hipGetLastError();
      n = 0;
    }
    cached = n;
  }
  return cached;
}

template <int WM, int WN, int MT, int NT, int MODE, bool AT>
bool launch_mode(const Igemm& p, int groups, int sk_blocks, int forced_occupancy, hipStream_t st) {
  if (sk_blocks > 0) {
    const int held = forced_occupancy >= 0 ? forced_occupancy : resident_blocks_per_cu<WM, WN, MT, NT, MODE, AT>();
    if ((long long)held * tt::compute_units() < sk_blocks) sk_blocks = 0;   // one tile per block instead: never a stalled wait
  }
  if (sk_blocks > 0) igemm_bf16x3<WM, WN, MT, NT, true, MODE, AT><<<dim3(sk_blocks, 1), kThreads, 0, st>>>(p);
  else igemm_bf16x3<WM, WN, MT, NT, false, MODE, AT><<<dim3(p.tiles, groups), kThreads, 0, st>>>(p);
  return sk_blocks > 0;
}

template <int WM, int WN, int MT, int NT>
bool launch_config(const Igemm& p, int groups, int sk_blocks, int forced, hipStream_t st) {
  const bool at = p.wTransStride > 0;
  if (p.mode == kModeGemm && at) return launch_mode<WM, WN, MT, NT, kModeGemm, true>(p, groups, sk_blocks, forced, st);
  if (p.mode == kModeGemm) return launch_mode<WM, WN, MT, NT, kModeGemm, false>(p, groups, sk_blocks, forced, st);
  if (p.mode == kModeTapMask && at) return launch_mode<WM, WN, MT, NT, kModeTapMask, true>(p, groups, sk_blocks, forced, st);
  if (p.mode == kModeTapMask) return launch_mode<WM, WN, MT, NT, kModeTapMask, false>(p, groups, sk_blocks, forced, st);
  if (p.mode == kModeTapMask64) return launch_mode<WM, WN, MT, NT, kModeTapMask64, false>(p, groups, sk_blocks, forced, st);
  return launch_mode<WM, WN, MT, NT, kModeCompare, false>(p, groups, sk_blocks, forced, st);
}

template <int WM, int WN, int MT, int NT>
int min_resident() {
  const int all[] = {resident_blocks_per_cu<WM, WN, MT, NT, kModeGemm, true>(),    resident_blocks_per_cu<WM, WN, MT, NT, kModeGemm, false>(),
                     resident_blocks_per_cu<WM, WN, MT, NT, kModeTapMask, true>(), resident_blocks_per_cu<WM, WN, MT, NT, kModeTapMask, false>(),
                     resident_blocks_per_cu<WM, WN, MT, NT, kModeTapMask64, false>(), resident_blocks_per_cu<WM, WN, MT, NT, kModeCompare, false>()};
  int lo = all[0];
  for (int v : all) lo = v < lo ? v : lo;
  return lo;
}

template <int WM, int WN, int MT, int NT>
void launch_multi_config(const IgemmMulti& m, int groups, hipStream_t st) {
  const dim3 grid(m.first[m.n], groups);
  if (m.c[0].mode == kModeTapMask) igemm_multi_bf16x3<WM, WN, MT, NT, kModeTapMask><<<grid, kThreads, 0, st>>>(m);
  else igemm_multi_bf16x3<WM, WN, MT, NT, kModeCompare><<<grid, kThreads, 0, st>>>(m);
}

}  // namespace

namespace ttc {

bool x3_launch(const Igemm& p, int groups, int sk_blocks, int bm, int bn, int forced_occupancy, hipStream_t st) {
  if (bm == 128 && bn == 128) return launch_config<2, 2, 2, 2>(p, groups, sk_blocks, forced_occupancy, st);
  if (bm == 64 && bn == 256) return launch_config<1, 4, 2, 2>(p, groups, sk_blocks, forced_occupancy, st);
  if (bm == 32 && bn == 256) return launch_config<1, 4, 1, 2>(p, groups, sk_blocks, forced_occupancy, st);
  return launch_config<2, 2, 1, 1>(p, groups, sk_blocks, forced_occupancy, st);
}

void x3_launch_multi(const IgemmMulti& m, int groups, int bm, int bn, hipStream_t st) {
  if (bm == 128 && bn == 128) launch_multi_config<2, 2, 2, 2>(m, groups, st);
  else if (bm == 64 && bn == 256) launch_multi_config<1, 4, 2, 2>(m, groups, st);
  else if (bm == 32 && bn == 256) launch_multi_config<1, 4, 1, 2>(m, groups, st);
  else launch_multi_config<2, 2, 1, 1>(m, groups, st);
}

int x3_min_resident_blocks() {
  const int all[] = {min_resident<2, 2, 2, 2>(), min_resident<1, 4, 2, 2>(), min_resident<1, 4, 1, 2>(), min_resident<2, 2, 1, 1>()};
  int lo = all[0];
  for (int v : all) lo = v < lo ? v : lo;
  return lo;
}

}  // namespace ttc
