// Implicit-GEMM convolution on fp32 MFMA for gfx950: Conv2d forward, and the gather-form input
// gradient that also serves as ConvTranspose2d forward.  NCHW float32, no im2col buffer in HBM.
// (This file: launch planning, index tables, weight repacks and the float32 / bf16 instantiations; the
// kernel body itself is conv_igemm_kernel.h, shared with conv_igemm_x3.hip.)
//
// Per group the kernel computes   D[i, m] = sum_k  Wp[i, k] * G[k, m]   (+ bias[i])
//   forward: i = output channel, m = (n, p, q) output pixel, k = (c, r, s),
//            G[k, m] = x[n, c, p*sh + r*dh - ph, q*sw + s*dw - pw]  (0 outside the image)
//   dgrad  : dx pixels are split into sh*sw stride-parity classes; inside a class every pixel
//            has the same set of valid taps, so a class is again a dense GEMM with
//            i = input channel, m = (n, h', w') with h = h'*sh + class_h, k = (ko, tr, ts),
//            G[k, m] = dy[n, ko, ih_base(h') - tr*eh, iw_base(w') - ts*ew]
//            (no zero-insertion, no wasted MACs at stride > 1; classes without a tap get bias/0).
// Both are the same kernel: a pixel decomposes as (n, u, v), a reduction index k looks up
// {element offset, row step, column step} in a small table read with scalar loads.
//
// Tiling: 256 threads = 4 waves; block tile BM x BN with BK = 16; each wave owns MT x NT
// v_mfma_f32_32x32x2_f32 accumulators (rows = i from the weights, columns = pixels, so a
// lane's 32 consecutive pixels store as 128 contiguous bytes of NCHW output).  Weights are
// repacked once per call into k-quad-major float4 tiles [k/4][i][k%4]; the gathered operand is
// written to LDS in the same layout, so every MFMA operand fetch is one ds_read_b128 that
// yields four k-steps.  Global loads for chunk c+1 are issued before the MFMAs of chunk c
// (register prefetch) and land in the other LDS buffer: one barrier per chunk.
//
// Vector-ALU instructions are not free next to MFMAs on this part (measured: every VALU
// instruction in the loop costs matrix-pipe time), so the loop keeps them to a minimum:
// operands are fetched with buffer loads whose per-lane offset is fixed for a whole tile, the
// reduction index only moves a scalar offset, and padding is left to the buffer range check
// (a lane whose tap falls outside the image gets bit 31 of its offset set, two VALU
// instructions per element, and reads 0).
//
// Optional reduced-precision variant (tt_set_conv_math(TT_CONV_MATH_BF16)): the same kernels with
// the operands rounded to bfloat16 after the LDS read and contracted by v_mfma_f32_32x32x16_bf16,
// float32 accumulation, float32 tensors in memory.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <type_traits>
#include <vector>

#include "conv_igemm_common.h"

namespace {

using namespace ttc;

// ---- preparation kernels (tiny) --------------------------------------------------------------

// k -> {offset, steps}.  k = (a*TB + b)*TC + c:  off = a*sa + b*sb + c*sc, steps (b*stepH, c*stepW).
// Tables are built on the host (host_ktab), checked there against the tensor they index
// (check_ktab) and kept in device buffers of their own, one per geometry: no kernel writes them
// and they never share memory with per-call scratch data.
struct KTabArgs {
  int Kred, Kpad, TB, TC, sa, sb, sc, stepH, stepW;
  int tapMask;   // 1 / 2: entries are {4*(off + offBias), tap number b*TC + c}; padding tap 31 / 63
  int offBias;
};
KEntry ktab_entry(const KTabArgs& a, int k) {
  KEntry e;
  if (k < a.Kred) {
    const int c = k % a.TC, t = k / a.TC;
    const int b = t % a.TB, aa = t / a.TB;
    e.off = aa * a.sa + b * a.sb + c * a.sc;
    e.dhw = ((b * a.stepH) & 0xffff) | ((c * a.stepW) << 16);
    if (a.tapMask) {
      e.off = 4 * (e.off + a.offBias);
      e.dhw = b * a.TC + c;
    }
  } else {
    e.off = 0;
    e.dhw = a.tapMask == 2 ? 63 : a.tapMask ? 31 : (-16384) & 0xffff;   // the mask's top tap / a row far above the image: never valid
  }
  return e;
}

// Forward: Wp[g][kq][i][j] = w[g*I + i][4*kq + j]  (w rows are Kred = Cg*R*S long, 0 beyond).
__global__ void pack_w_fwd(const float* __restrict__ w, floatx4* __restrict__ wp, int I, int Ipad, int Kred, int KQ) {
  const int g = blockIdx.z, kq = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= Ipad) return;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (i < I) {
    const float* row = w + ((size_t)g * I + i) * Kred;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (4 * kq + j < Kred) v[j] = row[4 * kq + j];
  }
  wp[((size_t)g * KQ + kq) * Ipad + i] = floatx4{v[0], v[1], v[2], v[3]};
}

// Input gradient, one stride-parity class: k = (ko*nTr + tr)*nTs + ts,
// Wp[g][kq][c][j] = w[g*Kg + ko][c][r0 + tr*rstep][s0 + ts*sstep].
// Up to kMaxMulti classes (the classes of one strided layer that have taps) are repacked by one
// launch: blockIdx.z = class * groups + group, blockIdx.y runs to the longest class's KQ.
struct PackDgrad {
  int Kg, Cg, R, S, Ipad, Kred, KQ;
  int nTr, nTs, r0, rstep, s0, sstep;
  floatx4* wp;
};
struct PackDgradMulti {
  PackDgrad c[kMaxMulti];
  int groups;
};
__global__ void pack_w_dgrad(const float* __restrict__ w, const PackDgradMulti m) {
  const int cls = blockIdx.z / m.groups, g = blockIdx.z % m.groups, kq = blockIdx.y;
  const PackDgrad& a = m.c[cls];
  if (kq >= a.KQ) return;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= a.Ipad) return;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < a.Cg) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = 4 * kq + j;
      if (k < a.Kred) {
        const int ts = k % a.nTs, t = k / a.nTs;
        const int tr = t % a.nTr, ko = t / a.nTr;
        v[j] = w[((((size_t)g * a.Kg + ko) * a.Cg + c) * a.R + a.r0 + tr * a.rstep) * a.S + a.s0 + ts * a.sstep];
      }
    }
  }
  a.wp[((size_t)g * a.KQ + kq) * a.Ipad + c] = floatx4{v[0], v[1], v[2], v[3]};
}

// Dense input gradient: every stride-parity class becomes Cg rows of one GEMM over the union
// of the classes' tap windows.  Row i = (class, c), k = (ko*Na + ia)*Nb + ib reads dy at row
// offset a = amin + ia from the cell's base row; the weight is w[ko][c][r][s] with
// r = (ch + ph - a*sh)/dh when that is an integer inside the kernel, else 0 (the class does
// not have that tap).  Worth it only when Cg is tiny: the zero taps are wasted MACs.
struct PackDense {
  int Kg, Cg, R, S, sh, sw, ph, pw, dh, dw, Na, Nb, amin, bmin, I, Ipad, Kred, KQ, HxWx, Wx;
  int cellW;   // pixel classes per cell row (a multiple of sw)
};
__global__ void pack_w_dgrad_dense(const float* __restrict__ w, floatx4* __restrict__ wp, PackDense a) {
  const int kq = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= a.Ipad) return;
  const int cls = i / a.Cg, c = i % a.Cg;
  const int ch = cls / a.cellW, cw = cls % a.cellW;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (i < a.I) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = 4 * kq + j;
      if (k >= a.Kred) continue;
      const int ib = k % a.Nb, t = k / a.Nb;
      const int ia = t % a.Na, ko = t / a.Na;
      const int rn = ch + a.ph - (a.amin + ia) * a.sh, sn = cw + a.pw - (a.bmin + ib) * a.sw;
      if (rn < 0 || sn < 0 || rn % a.dh != 0 || sn % a.dw != 0) continue;
      const int r = rn / a.dh, ss = sn / a.dw;
      if (r >= a.R || ss >= a.S) continue;
      v[j] = w[(((size_t)ko * a.Cg + c) * a.R + r) * a.S + ss];
    }
  }
  wp[(size_t)kq * a.Ipad + i] = floatx4{v[0], v[1], v[2], v[3]};
}

}  // namespace

#include "conv_igemm_kernel.h"

namespace {

using namespace ttc;

template <int WM, int WN, int MT, int NT, bool SK, int MODE, bool AT>
__global__ __launch_bounds__(kThreads, 2) void igemm_f32(const Igemm p) {
  igemm_body<WM, WN, MT, NT, SK, MODE, AT, 0>(p, (int)blockIdx.x);
}
// The same launch on bf16 matrix instructions (tt_set_conv_math); three blocks per CU.
template <int WM, int WN, int MT, int NT, bool SK, int MODE, bool AT>
__global__ __launch_bounds__(kThreads, 3) void igemm_bf16(const Igemm p) {
  igemm_body<WM, WN, MT, NT, SK, MODE, AT, 1>(p, (int)blockIdx.x);
}

template <int WM, int WN, int MT, int NT, int MODE>
__global__ __launch_bounds__(kThreads, 2) void igemm_multi_f32(const IgemmMulti m) {
  int ci = 0;
  while (ci + 1 < m.n && (int)blockIdx.x >= m.first[ci + 1]) ++ci;
  igemm_body<WM, WN, MT, NT, false, MODE, false, 0>(m.c[ci], (int)blockIdx.x - m.first[ci]);
}
template <int WM, int WN, int MT, int NT, int MODE>
__global__ __launch_bounds__(kThreads, 3) void igemm_multi_bf16(const IgemmMulti m) {
  int ci = 0;
  while (ci + 1 < m.n && (int)blockIdx.x >= m.first[ci + 1]) ++ci;
  igemm_body<WM, WN, MT, NT, false, MODE, false, 1>(m.c[ci], (int)blockIdx.x - m.first[ci]);
}

// ---- host side -------------------------------------------------------------------------------------

int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }
int gcd(int a, int b) { return b == 0 ? a : gcd(b, a % b); }

struct TileChoice {
  int bm, bn;
  int sk_blocks;   // > 0: persistent launch with this many blocks, left-over tiles split stream-K fashion
};

// Compute units of the device (256 on an MI355X), and the blocks of a persistent launch: two per
// CU (three or four measured slower).
int cus() { return tt::compute_units(); }
int sk_blocks_f32() { return 2 * cus(); }

// Stream-K pays (partial tiles through memory, a wait at the end) and only helps when the
// tiles do not spread evenly over the CUs; it needs a reduction long enough to split.
bool wants_stream_k(long long tiles, int chunks, int groups) {
  if (groups != 1 || chunks < 8) return false;
  // many tiles and a short reduction: hardware block scheduling balances better than fixed rounds
  if (tiles >= 3LL * sk_blocks_f32() && chunks < 64) return false;
  if (tiles * chunks < 4LL * sk_blocks_f32()) return false;
  const long long rounds = (tiles + cus() - 1) / cus();
  return (double)tiles / (double)(rounds * cus()) < 0.93;
}

// The bf16 kernels are bound by their fetch path, not by the matrix pipe: smaller tiles fetch more
// per FLOP and lose there.
bool bf16_math() { return tt::conv_math() == TT_CONV_MATH_BF16; }
// float32 arithmetic on the bf16 matrix pipe (three bf16 terms per operand element): launches the
// bf16-first kernels take run there, every other launch on the float32 kernels.
bool split_math() { return tt::conv_math() == TT_CONV_MATH_BF16X3; }
// bf16 terms per operand element of the matrix instructions in use (0: float32 instructions)
int math_terms() { return bf16_math() ? 1 : split_math() ? 3 : 0; }

// Blocks of a persistent launch: the bf16 kernels hide their loads with a third block per CU
// (measured: 3 % faster than two, four do not fit the register file).
int sk_launch_blocks() { return bf16_math() ? 3 * cus() : sk_blocks_f32(); }

// 128x128 by default, 64 rows when a group has no more than 64 of them.  When that leaves
// CUs idle or unevenly loaded the reduction is split stream-K fashion; if it is too short for
// that, 64x64 tiles raise the block count instead.  `small` asks for 64x64 tiles outright: many
// light blocks (four or five resident per CU) balance better and exchange no partial sums where a
// tile's reduction is short (plain matrix products with at most 32 chunks) or where several
// short launches share a grid (the stride-parity classes of an input gradient).
TileChoice choose_tile(int I, int M, int groups, int chunks, bool allow_stream_k = true, bool small = false) {
  TileChoice t;
  t.bm = I <= 64 ? 64 : 128;
  t.bn = I <= 64 ? 256 : 128;
  if (small && groups == 1) { t.bm = 64; t.bn = 64; }
  t.sk_blocks = 0;
  const long long tiles = (long long)ceil_div(I, t.bm) * ceil_div(M, t.bn);
  if (allow_stream_k && wants_stream_k(tiles, chunks, groups)) {
    t.sk_blocks = sk_launch_blocks();
  } else if (tiles * groups < cus()) {
    t.bm = 64;
    t.bn = 64;
    const long long small = (long long)ceil_div(I, 64) * ceil_div(M, 64);
    if (allow_stream_k && wants_stream_k(small, chunks, groups)) t.sk_blocks = sk_launch_blocks();
  }
  return t;
}

// bytes of stream-K partial accumulators for the largest tile: one slot per block
size_t sk_workspace_bytes() { return (size_t)sk_launch_blocks() * 128 * 128 * sizeof(float); }

// The stream-K wait is safe only while every block of the persistent grid is resident at once
// (sk_launch_blocks() = 2 per CU, 3 for the bf16 kernels).  What the device can hold of one
// instantiation is asked once (registers and LDS of the compiled kernel decide it); an
// instantiation that cannot hold that many is launched data-parallel instead, one tile per block:
// a register-count regression then costs speed, never a stalled launch.
template <int WM, int WN, int MT, int NT, int MODE, bool AT, int BFK>
int sk_resident_blocks_per_cu() {
  static int cached = -1;
  if (cached < 0) {
    int n = 0;
    hipError_t e;
    if constexpr (BFK == 1) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, igemm_bf16<WM, WN, MT, NT, true, MODE, AT>, kThreads, 0);
    else e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, igemm_f32<WM, WN, MT, NT, true, MODE, AT>, kThreads, 0);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      n = 0;
    }
    cached = n;
  }
  return cached;
}
int g_sk_forced_occupancy = -1;   // >= 0: pretend every instantiation holds this many blocks per CU (tests of the fallback)

// Returns whether the persistent (stream-K) grid was launched.
template <int WM, int WN, int MT, int NT, int MODE, bool AT>
bool launch_mode(const Igemm& p, int groups, int sk_blocks, hipStream_t st) {
  const bool bf = tt::conv_math() == TT_CONV_MATH_BF16;
  if (sk_blocks > 0) {
    int held = bf ? sk_resident_blocks_per_cu<WM, WN, MT, NT, MODE, AT, 1>() : sk_resident_blocks_per_cu<WM, WN, MT, NT, MODE, AT, 0>();
    if (g_sk_forced_occupancy >= 0) held = g_sk_forced_occupancy;
    if ((long long)held * cus() < sk_blocks) sk_blocks = 0;   // the data-parallel launch ignores the stream-K fields
  }
  if (sk_blocks > 0) {
    if (bf) igemm_bf16<WM, WN, MT, NT, true, MODE, AT><<<dim3(sk_blocks, 1), kThreads, 0, st>>>(p);
    else igemm_f32<WM, WN, MT, NT, true, MODE, AT><<<dim3(sk_blocks, 1), kThreads, 0, st>>>(p);
  } else if (bf) {
    igemm_bf16<WM, WN, MT, NT, false, MODE, AT><<<dim3(p.tiles, groups), kThreads, 0, st>>>(p);
  } else {
    igemm_f32<WM, WN, MT, NT, false, MODE, AT><<<dim3(p.tiles, groups), kThreads, 0, st>>>(p);
  }
  return sk_blocks > 0;
}
// smallest number of resident blocks per CU over every stream-K instantiation of one tile shape
template <int WM, int WN, int MT, int NT, int BFK>
int sk_min_resident() {
  const int all[] = {sk_resident_blocks_per_cu<WM, WN, MT, NT, kModeGemm, true, BFK>(),
                     sk_resident_blocks_per_cu<WM, WN, MT, NT, kModeGemm, false, BFK>(),
                     sk_resident_blocks_per_cu<WM, WN, MT, NT, kModeTapMask, true, BFK>(),
                     sk_resident_blocks_per_cu<WM, WN, MT, NT, kModeTapMask, false, BFK>(),
                     sk_resident_blocks_per_cu<WM, WN, MT, NT, kModeTapMask64, false, BFK>(),
                     sk_resident_blocks_per_cu<WM, WN, MT, NT, kModeCompare, false, BFK>()};
  int lo = all[0];
  for (int v : all) lo = v < lo ? v : lo;
  return lo;
}
template <int BFK>
int sk_min_resident_all() {
  const int all[] = {sk_min_resident<2, 2, 2, 2, BFK>(), sk_min_resident<1, 4, 2, 2, BFK>(),
                     sk_min_resident<1, 4, 1, 2, BFK>(), sk_min_resident<2, 2, 1, 1, BFK>()};
  int lo = all[0];
  for (int v : all) lo = v < lo ? v : lo;
  return lo;
}
template <int WM, int WN, int MT, int NT>
bool launch_config(const Igemm& p, int groups, int sk_blocks, hipStream_t st) {
  const bool at = p.wTransStride > 0;
  if (p.mode == kModeGemm && at) return launch_mode<WM, WN, MT, NT, kModeGemm, true>(p, groups, sk_blocks, st);
  if (p.mode == kModeGemm) return launch_mode<WM, WN, MT, NT, kModeGemm, false>(p, groups, sk_blocks, st);
  if (p.mode == kModeTapMask && at) return launch_mode<WM, WN, MT, NT, kModeTapMask, true>(p, groups, sk_blocks, st);
  if (p.mode == kModeTapMask) return launch_mode<WM, WN, MT, NT, kModeTapMask, false>(p, groups, sk_blocks, st);
  if (p.mode == kModeTapMask64) return launch_mode<WM, WN, MT, NT, kModeTapMask64, false>(p, groups, sk_blocks, st);
  return launch_mode<WM, WN, MT, NT, kModeCompare, false>(p, groups, sk_blocks, st);
}

// Picks how the kernel addresses the gathered operand (see Igemm::mode) and completes the table
// arguments accordingly.  Needs the source geometry fields of `p`; `pixels` = U*V pixels per
// image, `gemm_geometry` = 1x1 / stride 1 / unpadded / pixel count a multiple of 4.
// `wide_masks`: the launch may use the 64-bit tap mask (single launches only: the shared grids of
// an input gradient's stride-parity classes are built for the other modes).
void choose_mode(Igemm& p, KTabArgs& ka, bool gemm_geometry, int N, int U, int V, long long weight_bytes,
                 bool wide_masks = false) {
  p.mode = kModeCompare;
  p.TB = ka.TB; p.TC = ka.TC; p.stepH = ka.stepH; p.stepW = ka.stepW;
  const long long b1 = (long long)(p.bh < 0 ? -p.bh : 0) * p.srcRow + (p.bw < 0 ? -p.bw : 0);
  const long long lo_b = (long long)(ka.TB - 1) * ka.sb, lo_c = (long long)(ka.TC - 1) * ka.sc;
  const long long b2 = -((lo_b < 0 ? lo_b : 0) + (lo_c < 0 ? lo_c : 0));
  // byte offsets a lane can reach: the images one 256-pixel tile spans, one more for the
  // reduction offset, the rows and columns its taps may overshoot, and the biases
  const long long span = (long long)(255 / ((long long)U * V) + 2 < N ? 255 / ((long long)U * V) + 2 : N);
  const long long reach = 4 * ((span + 1) * p.srcStrideN + 2 * (b1 + b2) +
                               ((long long)U * p.su + (p.bh < 0 ? -p.bh : p.bh) + 2) * p.srcRow + (long long)V * p.sv +
                               (p.bw < 0 ? -p.bw : p.bw));
  const long long limit = (1LL << 31) - (1LL << 20);
  if (reach >= limit || weight_bytes >= limit) return;
  if (gemm_geometry && ka.Kred % (4 * kBKQ) == 0) {
    p.mode = kModeGemm;
  } else if (ka.TB * ka.TC <= 31 || (wide_masks && ka.TB * ka.TC <= 63)) {
    p.mode = ka.TB * ka.TC <= 31 ? kModeTapMask : kModeTapMask64;
    p.voffBias = (int)b1;
    p.srdBias = b1 + b2;
    ka.tapMask = ka.TB * ka.TC <= 31 ? 1 : 2;
    ka.offBias = (int)b2;
  }
}

// Flags of the stream-K launches: zeroed once; every launch publishes with a new epoch (never 0),
// so the words never need clearing again.
unsigned g_sk_epoch = 0;
unsigned* g_sk_flags = nullptr;
// The word a block sets when its wait ran out: pinned host memory mapped into the device's address
// space, so the host reads it directly once the stream has drained.
volatile unsigned* g_sk_error_host = nullptr;
unsigned* g_sk_error_dev = nullptr;
int sk_error_word(unsigned** out) {
  if (g_sk_error_host == nullptr) {
    void* host = nullptr;
    TT_HIP(hipHostMalloc(&host, sizeof(unsigned), hipHostMallocMapped));
    *(volatile unsigned*)host = 0u;
    void* dev = nullptr;
    if (hipError_t e = hipHostGetDevicePointer(&dev, host, 0); e != hipSuccess) {
      (void)hipHostFree(host);
      return tt::fail_hip(e, "hipHostGetDevicePointer", __FILE__, __LINE__);
    }
    g_sk_error_host = (volatile unsigned*)host;
    g_sk_error_dev = (unsigned*)dev;
  }
  *out = g_sk_error_dev;
  return 0;
}
int sk_flags(unsigned** out) {
  if (g_sk_flags == nullptr) {
    const size_t bytes = sizeof(unsigned) * kSkFlagWords;
    TT_HIP(hipMalloc((void**)&g_sk_flags, bytes));
    TT_HIP(hipMemsetAsync(g_sk_flags, 0, bytes, tt::stream()));
  }
  *out = g_sk_flags;
  return 0;
}

// Sets the error word from the device, exactly as a block whose wait ran out does.
__global__ void sk_raise_error(unsigned* word) {
  __hip_atomic_store(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// What the last single launch looked like (instrumentation: tests pick the images to compare from it).
int g_last_launch[8] = {};
// bf16 arithmetic: launches that the bf16-first kernels support go to them (tests switch this off to
// reach the float32 kernels' bf16 instantiations on the same shapes)
bool g_bf16_first = true;
bool g_bf16_first_always = false;   // tests: also where the tile-count rule would keep the other kernels

int launch_igemm(Igemm& p, int groups, TileChoice t, int prof_id, floatx4* sk_partial) {
  tt::ProfScope prof(prof_id);
  p.tilesI = p.Ipad / t.bm;
  p.tiles = p.tilesI * ceil_div(p.M, t.bn);
  if (t.sk_blocks > 0) {
    const int chunks = p.KQ / kBKQ;
    const int rem = p.tiles % t.sk_blocks;
    if (rem == 0) {
      t.sk_blocks = 0;   // whole rounds only: nothing to split
    } else {
      p.skDpTiles = p.tiles - rem;
      p.skIters = (long long)rem * chunks;
      // every sharing block gets at least 8 reduction steps of work for the partial tile it leaves
      long long share = p.skIters / 8;
      if (share < rem) share = rem;
      p.skBlocks = (int)(share < t.sk_blocks ? share : t.sk_blocks);
      p.skPartial = sk_partial;
      if (sk_flags(&p.skFlags) || sk_error_word(&p.skError)) return -1;
      if (++g_sk_epoch == 0) ++g_sk_epoch;
      p.skEpoch = g_sk_epoch;
    }
  }
  hipStream_t st = tt::stream();
  // The reduced-precision mode's own kernels: 128-pixel tiles, one tile per block, nothing shared.
  // They share no reduction between blocks, so launches with fewer tiles than compute units and a
  // long reduction stay on the stream-K instantiations (measured per layer: 1.2-1.8 times faster
  // where taken, up to 2 times slower on 100 tiles of 144 chunks).
  const int bf_tiles = (p.Ipad / t.bm) * ceil_div(p.M, 128);
  int bf_bm = 0;   // tile rows of the launch they take (0: not taken)
  if (bf16_math() && g_bf16_first && bf16_first_supported(p, groups, t.bm) &&
      ((long long)bf_tiles * groups >= cus() || p.Kred <= 1024 || g_bf16_first_always)) {
    bf_bm = t.bm;
  }
  if (bf_bm > 0) {
    const int tiles = (p.Ipad / bf_bm) * ceil_div(p.M, 128);
    const int plan[8] = {bf_bm, 128, tiles, p.Ipad / bf_bm, -1, tiles, 0, p.mode | 1 << 8};   // -1: the bf16-first kernels
    std::copy(plan, plan + 8, g_last_launch);
    bf16_first_launch(p, groups, bf_bm, st);
    TT_LAUNCH_CHECK();
    return 0;
  }
  const int plan[8] = {t.bm, t.bn, p.tiles, p.tilesI, t.sk_blocks, t.sk_blocks > 0 ? p.skDpTiles : p.tiles,
                       t.sk_blocks > 0 ? p.skBlocks : 0, p.mode | math_terms() << 8};
  std::copy(plan, plan + 8, g_last_launch);
  bool persistent;
  if (split_math())
    persistent = x3_launch(p, groups, t.sk_blocks, t.bm, t.bn, g_sk_forced_occupancy, st);
  else if (t.bm == 128 && t.bn == 128)
    persistent = launch_config<2, 2, 2, 2>(p, groups, t.sk_blocks, st);
  else if (t.bm == 64 && t.bn == 256)
    persistent = launch_config<1, 4, 2, 2>(p, groups, t.sk_blocks, st);
  else if (t.bm == 32 && t.bn == 256)
    persistent = launch_config<1, 4, 1, 2>(p, groups, t.sk_blocks, st);
  else
    persistent = launch_config<2, 2, 1, 1>(p, groups, t.sk_blocks, st);
  if (!persistent) {   // also when the device could not hold the persistent grid: one tile per block
    g_last_launch[4] = 0;
    g_last_launch[5] = p.tiles;
    g_last_launch[6] = 0;
  }
  TT_LAUNCH_CHECK();
  return 0;
}

// Launches the data-parallel GEMMs in `list` (same tile shape, same addressing mode, no stream-K,
// no transposed weights) as one grid.
template <int WM, int WN, int MT, int NT>
void launch_multi_config(const IgemmMulti& m, int groups, hipStream_t st) {
  const dim3 grid(m.first[m.n], groups);
  const bool bf = bf16_math();
  if (m.c[0].mode == kModeTapMask) {
    if (bf) igemm_multi_bf16<WM, WN, MT, NT, kModeTapMask><<<grid, kThreads, 0, st>>>(m);
    else igemm_multi_f32<WM, WN, MT, NT, kModeTapMask><<<grid, kThreads, 0, st>>>(m);
  } else {
    if (bf) igemm_multi_bf16<WM, WN, MT, NT, kModeCompare><<<grid, kThreads, 0, st>>>(m);
    else igemm_multi_f32<WM, WN, MT, NT, kModeCompare><<<grid, kThreads, 0, st>>>(m);
  }
}
int launch_igemm_multi(IgemmMulti& m, int groups, TileChoice t, int prof_id) {
  tt::ProfScope prof(prof_id);
  m.first[0] = 0;
  for (int i = 0; i < m.n; ++i) {
    Igemm& p = m.c[i];
    p.tilesI = p.Ipad / t.bm;
    p.tiles = p.tilesI * ceil_div(p.M, t.bn);
    m.first[i + 1] = m.first[i] + p.tiles;
  }
  const int plan[8] = {t.bm, t.bn, m.first[m.n], 0, 0, m.first[m.n], 0, m.c[0].mode | math_terms() << 8};   // several launches in one grid
  std::copy(plan, plan + 8, g_last_launch);
  hipStream_t st = tt::stream();
  if (split_math())
    x3_launch_multi(m, groups, t.bm, t.bn, st);
  else if (t.bm == 128 && t.bn == 128)
    launch_multi_config<2, 2, 2, 2>(m, groups, st);
  else if (t.bm == 64 && t.bn == 256)
    launch_multi_config<1, 4, 2, 2>(m, groups, st);
  else if (t.bm == 32 && t.bn == 256)
    launch_multi_config<1, 4, 1, 2>(m, groups, st);
  else
    launch_multi_config<2, 2, 1, 1>(m, groups, st);
  TT_LAUNCH_CHECK();
  return 0;
}

// ---- index tables ----------------------------------------------------------------------------------
// Reduction-index tables (and the row tables of dense input gradients) depend only on the layer
// geometry.  They are built on the host, checked there against the tensor they address, uploaded
// once into a device buffer of their own and kept per geometry: nothing on the device ever writes
// them, and they share no memory with the per-call workspace.  At kMaxTables geometries the cache
// is dropped and rebuilt (after a stream sync); tt_empty_cache drops it too.
constexpr size_t kMaxTables = 1024;
struct DeviceTable {
  void* dev = nullptr;
  std::vector<char> host;   // stays alive while the upload may still be reading it
};
std::map<std::vector<int>, DeviceTable>& table_cache() {
  static std::map<std::vector<int>, DeviceTable> cache;
  return cache;
}
int release_tables() {   // the caller has synchronised the stream
  auto& cache = table_cache();
  for (auto& kv : cache)
    if (kv.second.dev) TT_HIP(hipFree(kv.second.dev));
  cache.clear();
  return 0;
}
// Looks `key` up; on a miss uploads `bytes` from `host` (already checked by the caller).
int cached_table(const std::vector<int>& key, const void* host, size_t bytes, const void** out) {
  auto& cache = table_cache();
  auto it = cache.find(key);
  if (it == cache.end()) {
    hipStream_t st = tt::stream();
    if (cache.size() >= kMaxTables) {
      TT_HIP(hipStreamSynchronize(st));
      if (release_tables()) return -1;
    }
    DeviceTable t;
    t.host.assign((const char*)host, (const char*)host + bytes);
    TT_HIP(hipMalloc(&t.dev, bytes));
    it = cache.emplace(key, std::move(t)).first;   // the vector's storage moves with it
    hipError_t e = hipMemcpyAsync(it->second.dev, it->second.host.data(), bytes, hipMemcpyHostToDevice, st);
    if (e != hipSuccess) {
      (void)hipFree(it->second.dev);
      cache.erase(it);
      return tt::fail_hip(e, "hipMemcpyAsync(index table)", __FILE__, __LINE__);
    }
  }
  *out = it->second.dev;
  return 0;
}

// What the kernel will do with entry k of `tab` for launch `p`, replayed on the host for the
// extreme pixels of every tap: wherever the kernel's own bounds rule calls a tap valid, the
// element it would fetch must be the element (n, group, plane a, row, column) of the source
// tensor that the reduction index stands for, and lie inside the tensor; padding entries must
// never be valid; the 32-bit byte offsets of the buffer mode must stay in [0, 2^31).
// `planes` = channels of the source per group, `src_elems` = elements of the whole source tensor.
int check_ktab(const char* fn, const Igemm& p, const KTabArgs& ka, const std::vector<KEntry>& tab, int N, int groups,
               int U, int V, int planes, long long src_elems) {
  if (p.mode == kModeGemm) return 0;   // plain matrix product: no table is read
  const bool mask = p.mode == kModeTapMask || p.mode == kModeTapMask64;
  const int top_tap = p.mode == kModeTapMask64 ? 63 : 31;
  TT_REQUIRE((int)tab.size() == ka.Kpad && ka.Kpad % (4 * kBKQ) == 0 && ka.Kred <= ka.Kpad,
             "%s: index table of %zu entries for a reduction of %d (%d padded)", fn, tab.size(), ka.Kred, ka.Kpad);
  TT_REQUIRE(p.srcRow == p.Wlim && (long long)p.srcStrideG == (long long)planes * p.Hlim * p.Wlim &&
                 (long long)N * p.srcStrideN <= src_elems,
             "%s: source geometry of the launch does not describe an [N, C, %d, %d] tensor", fn, p.Hlim, p.Wlim);
  TT_REQUIRE(!mask || (ka.TB * ka.TC <= top_tap && ka.tapMask == (top_tap == 63 ? 2 : 1)),
             "%s: %d x %d taps do not fit the %d-bit tap mask", fn, ka.TB, ka.TC, top_tap);
  const long long plane = (long long)p.Hlim * p.Wlim;
  // images a 256-pixel tile can span beyond its first one (buffer offsets are relative to that)
  const long long span = std::min<long long>(N - 1, 255 / ((long long)U * V) + 1);
  for (int k = 0; k < ka.Kpad; ++k) {
    const KEntry e = tab[k];
    long long off;
    int th, tw;
    if (mask) {
      const int tap = e.dhw;
      if (k >= ka.Kred) {
        TT_REQUIRE(tap == top_tap, "%s: padding entry %d of the index table names tap %d", fn, k, tap);
        continue;
      }
      TT_REQUIRE(tap >= 0 && tap < ka.TB * ka.TC && e.off >= 0 && e.off % 4 == 0,
                 "%s: index table entry %d: tap %d, byte offset %d", fn, k, tap, e.off);
      off = e.off / 4 - ka.offBias;
      th = (tap / ka.TC) * p.stepH;
      tw = (tap % ka.TC) * p.stepW;
    } else {
      off = e.off;
      th = (int)(short)(e.dhw & 0xffff);
      tw = e.dhw >> 16;
      if (k >= ka.Kred) {
        TT_REQUIRE(th <= -16384, "%s: padding entry %d of the index table can be valid (row step %d)", fn, k, th);
        continue;
      }
    }
    const int a = k / (ka.TB * ka.TC), b = (k / ka.TC) % ka.TB, c = k % ka.TC;
    TT_REQUIRE(th == b * p.stepH && tw == c * p.stepW, "%s: index table entry %d steps (%d, %d), tap (%d, %d)", fn, k, th,
               tw, b, c);
    // pixels u with 0 <= u*su + bh + th < Hlim, likewise v
    auto range = [](int n, int stride, int base, int lim, int* lo, int* hi) {
      *lo = base >= 0 ? 0 : (-base + stride - 1) / stride;
      *hi = lim - 1 - base < 0 ? -1 : std::min(n - 1, (lim - 1 - base) / stride);
    };
    int ulo, uhi, vlo, vhi;
    range(U, p.su, p.bh + th, p.Hlim, &ulo, &uhi);
    range(V, p.sv, p.bw + tw, p.Wlim, &vlo, &vhi);
    if (ulo > uhi || vlo > vhi) continue;   // no pixel uses this tap
    TT_REQUIRE(a < planes, "%s: index table entry %d addresses plane %d of %d", fn, k, a, planes);
    for (int iu = 0; iu < 2; ++iu)
      for (int iv = 0; iv < 2; ++iv)
        for (int in = 0; in < 2; ++in)
          for (int ig = 0; ig < 2; ++ig) {
            const long long u = iu ? uhi : ulo, v = iv ? vhi : vlo, n = in ? N - 1 : 0, g = ig ? groups - 1 : 0;
            const long long ih0 = u * p.su + p.bh, iw0 = v * p.sv + p.bw;
            const long long at = n * p.srcStrideN + g * p.srcStrideG + ih0 * p.srcRow + iw0 + off;
            const long long want = n * p.srcStrideN + g * p.srcStrideG + a * plane + (ih0 + th) * p.srcRow + (iw0 + tw);
            TT_REQUIRE(at == want && at >= 0 && at < src_elems,
                       "%s: index table entry %d reaches element %lld of the source (expected %lld of %lld)", fn, k, at,
                       want, src_elems);
            if (mask) {
              const long long lane = 4 * (std::min<long long>(n, span) * p.srcStrideN + ih0 * p.srcRow + iw0 + p.voffBias);
              TT_REQUIRE(lane >= 0 && lane + e.off < (1LL << 31),
                         "%s: index table entry %d: byte offset %lld + %d leaves the buffer range", fn, k, lane, e.off);
            }
          }
  }
  return 0;
}

// Set only inside tt_conv2d_check_tables_selftest (host-only checks): damages one entry of the
// next tables built, to show that check_ktab refuses them.
int g_selftest_fault_entry = -1, g_selftest_fault_delta = 0;

// Builds the table for `ka`, checks it against launch `p`, and (unless `host_only`) returns the
// device copy kept for this geometry.
int make_ktab(const char* fn, const Igemm& p, const KTabArgs& ka, int N, int groups, int U, int V, int planes,
              long long src_elems, bool host_only, const KEntry** out) {
  if (p.mode == kModeGemm) {   // plain matrix product: the kernel reads no table
    *out = nullptr;
    return 0;
  }
  std::vector<int> key{0, ka.Kred, ka.Kpad, ka.TB, ka.TC, ka.sa, ka.sb, ka.sc, ka.stepH, ka.stepW, ka.tapMask, ka.offBias,
                       p.mode, N, groups, U, V, planes, p.su, p.bh, p.sv, p.bw, p.Hlim, p.Wlim, p.voffBias};
  if (!host_only) {
    auto it = table_cache().find(key);
    if (it != table_cache().end()) {   // checked when it was built
      *out = (const KEntry*)it->second.dev;
      return 0;
    }
  }
  std::vector<KEntry> tab((size_t)ka.Kpad);
  for (int k = 0; k < ka.Kpad; ++k) tab[(size_t)k] = ktab_entry(ka, k);
  if (g_selftest_fault_entry >= 0 && g_selftest_fault_entry < ka.Kpad)   // tt_conv2d_check_tables_selftest only
    tab[(size_t)g_selftest_fault_entry].off += g_selftest_fault_delta;
  if (check_ktab(fn, p, ka, tab, N, groups, U, V, planes, src_elems)) return -1;
  if (host_only) return 0;
  return cached_table(key, tab.data(), sizeof(KEntry) * tab.size(), (const void**)out);
}

// Row table of a dense input gradient: GEMM row i = (pixel class (ch, cw) of the cell, channel c)
// -> {element offset c*Hx*Wx + ch*Wx + cw inside an image, ch, cw, c}.  Checked: every row of
// every cell that the kernel's bounds rule (oh + ch < Hx, ow + cw < Wx) lets through lands inside
// the output tensor.
int make_rowtab(const char* fn, int I, int Cg, int cellH, int cellW, int Hx, int Wx, int N, int U, int V,
                bool host_only, const int4** out) {
  std::vector<int> key{1, I, Cg, cellH, cellW, Hx, Wx, N, U, V};
  if (!host_only) {
    auto it = table_cache().find(key);
    if (it != table_cache().end()) {
      *out = (const int4*)it->second.dev;
      return 0;
    }
  }
  TT_REQUIRE(I == cellH * cellW * Cg, "%s: %d rows for a %d x %d cell of %d channels", fn, I, cellH, cellW, Cg);
  std::vector<int4> tab((size_t)I);
  const long long out_elems = (long long)N * Cg * Hx * Wx;
  for (int i = 0; i < I; ++i) {
    const int cls = i / Cg, c = i % Cg;
    const int ch = cls / cellW, cw = cls % cellW;
    tab[(size_t)i] = make_int4(c * Hx * Wx + ch * Wx + cw, ch, cw, c);
    // last cell row / column that still holds this class, last image
    const long long u = (Hx - 1 - ch) / cellH, v = (Wx - 1 - cw) / cellW;
    if (Hx - 1 - ch < 0 || Wx - 1 - cw < 0) continue;
    TT_REQUIRE(u < U && v < V, "%s: row table: class (%d, %d) needs cell (%lld, %lld) of %d x %d", fn, ch, cw, u, v, U, V);
    const long long at = (long long)(N - 1) * Cg * Hx * Wx + (u * cellH) * Wx + v * cellW + tab[(size_t)i].x;
    TT_REQUIRE(at >= 0 && at < out_elems && u * cellH + ch < Hx && v * cellW + cw < Wx,
               "%s: row table entry %d reaches element %lld of %lld", fn, i, at, out_elems);
  }
  if (host_only) return 0;
  return cached_table(key, tab.data(), sizeof(int4) * tab.size(), (const void**)out);
}

int check_common(const char* fn, int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int ph, int pw,
                 int dh, int dw, int groups, int P, int Q) {
  TT_REQUIRE(N > 0 && C > 0 && H > 0 && W > 0 && K > 0 && R > 0 && S > 0, "%s: sizes must be positive", fn);
  TT_REQUIRE(sh > 0 && sw > 0 && dh > 0 && dw > 0 && ph >= 0 && pw >= 0, "%s: stride/dilation must be positive, padding non-negative", fn);
  TT_REQUIRE(groups > 0 && C % groups == 0 && K % groups == 0, "%s: channels (%d, %d) not divisible by groups=%d", fn, C, K, groups);
  TT_REQUIRE(P > 0 && Q > 0, "%s: empty output (%d x %d)", fn, P, Q);
  TT_REQUIRE(groups <= 65535, "%s: more than 65535 groups are not supported", fn);
  TT_REQUIRE((long long)H + 2 * ph + (long long)R * dh < 16384 && (long long)W + 2 * pw + (long long)S * dw < 16384 &&
                 P < 16384 && Q < 16384,
             "%s: spatial extents must stay below 16384", fn);
  TT_REQUIRE(tt::fits_i32((long long)N * C * H * W) && tt::fits_i32((long long)N * K * P * Q) &&
                 tt::fits_i32((long long)K * (C / groups) * R * S),
             "%s: one image or the weights exceed 2^31-1 elements", fn);
  return 0;
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// tt_set_conv_dense_cell_min_tiles: 256-pixel tiles a larger dense input-gradient cell must leave
// (< 0: not set, 1.5 per compute unit)
int g_dense_cell_min_tiles = -1;
int dense_cell_min_tiles() { return g_dense_cell_min_tiles >= 0 ? g_dense_cell_min_tiles : 3 * cus() / 2; }

}  // namespace

namespace tt {
int conv_release_tables() { return release_tables(); }
int conv_async_error_word(unsigned** device_pointer) { return sk_error_word(device_pointer); }

// After a stream sync: has a stream-K block given up waiting for another block's partial sums since
// the last check?  The convolution results since then are invalid in that case.
int conv_check_async_error() {
  if (g_sk_error_host == nullptr || *g_sk_error_host == 0u) return 0;
  *g_sk_error_host = 0u;   // the stream has drained: no kernel that could set it is running
  return tt::fail(-1, "a convolution launch timed out waiting for another block's partial sums (the device could not "
                      "hold its grid of resident blocks); convolution results since the last "
                      "synchronisation are invalid");
}
}  // namespace tt

extern "C" {

int tt_set_conv_dense_cell_min_tiles(int tiles) {
  TT_API_LOCK();
  TT_REQUIRE(tiles >= -1 && tiles <= (1 << 20), "tt_set_conv_dense_cell_min_tiles: %d is out of range (-1..2^20)", tiles);
  g_dense_cell_min_tiles = tiles;   // -1: back to the default, 1.5 tiles per compute unit
  return 0;
}

// Instrumentation (tests): resident blocks per compute unit of the stream-K kernels, the smallest
// over every instantiation, float32 (bf16 == 0) or bf16 ones.  The launches need 2 resp. 3.
int tt_conv2d_stream_k_blocks_per_cu(int bf16, int* blocks) {
  TT_REQUIRE_INIT();
  TT_REQUIRE(blocks != nullptr, "tt_conv2d_stream_k_blocks_per_cu: null result pointer");
  *blocks = bf16 == 3 ? x3_min_resident_blocks() : bf16 ? sk_min_resident_all<1>() : sk_min_resident_all<0>();
  return 0;
}

// Instrumentation (tests): the plan of the last single matrix-product launch of a forward or input
// gradient call: {tile rows, tile columns (pixels), tiles, row tiles, blocks of the persistent grid
// (0: one tile per block; -1: one tile per block on the bf16-first kernels), tiles computed whole (the rest share their reduction between blocks),
// blocks sharing them, addressing mode | bf16 terms per operand element << 8 (0: float32 matrix instructions)}.  Pixel tile t starts at pixel (t / row tiles) * tile columns.
int tt_conv2d_last_launch(int* plan8) {
  TT_API_LOCK();
  TT_REQUIRE(plan8 != nullptr, "tt_conv2d_last_launch: null result pointer");
  std::copy(g_last_launch, g_last_launch + 8, plan8);
  return 0;
}

// Instrumentation (tests): with bf16 arithmetic selected, route the launches the bf16-first kernels
// support to them (1, the default) or keep everything on the float32 kernels' bf16 instantiations (0).
int tt_conv2d_bf16_first_enable(int on) {
  TT_API_LOCK();
  g_bf16_first = on != 0;
  g_bf16_first_always = on == 2;   // 2: every supported launch, whatever its tile count (small test shapes)
  return 0;
}

// Instrumentation (tests): pretend that every stream-K instantiation holds `blocks` blocks per
// compute unit (-1: ask the device again), so that the data-parallel fallback can be exercised.
int tt_conv2d_stream_k_force_occupancy(int blocks) {
  TT_API_LOCK();
  TT_REQUIRE(blocks >= -1 && blocks <= 64, "tt_conv2d_stream_k_force_occupancy: %d is out of range (-1..64)", blocks);
  g_sk_forced_occupancy = blocks;
  return 0;
}

// Instrumentation (tests): a one-thread kernel sets the word that a stream-K block sets when its
// wait for another block runs out.  The next tt_sync() / tt_memcpy_d2h() must report it, once.
int tt_conv2d_selftest_raise_async_error(void) {
  TT_REQUIRE_INIT();
  unsigned* word = nullptr;
  if (sk_error_word(&word)) return -1;
  sk_raise_error<<<1, 1, 0, tt::stream()>>>(word);
  TT_LAUNCH_CHECK();
  return 0;
}

// `size_only`: report the workspace bytes this call would ask the library for and do nothing else.
// `check_only`: build and check every index table the call would use, on the host alone (no
// device is touched, tensor pointers are not looked at).
static int conv2d_fwd(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K,
                      int R, int S, int sh, int sw, int ph, int pw, int dh, int dw, int groups, size_t* size_only,
                      bool check_only = false) {
  const char* fn = "tt_conv2d_fwd_f32";
  TT_API_LOCK();
  if (!check_only) {
    TT_REQUIRE_INIT();
    TT_REQUIRE(x && w && y, "tt_conv2d_fwd_f32: null tensor pointer");
    TT_REQUIRE_ALIGNED("tt_conv2d_fwd_f32", x, w, y);
  }
  const int P = (H + 2 * ph - dh * (R - 1) - 1) / sh + 1;
  const int Q = (W + 2 * pw - dw * (S - 1) - 1) / sw + 1;
  TT_REQUIRE(H + 2 * ph - dh * (R - 1) - 1 >= 0 && W + 2 * pw - dw * (S - 1) - 1 >= 0,
             "tt_conv2d_fwd_f32: kernel (%d x %d, dilation %d x %d) larger than padded input (%d x %d)", R, S, dh, dw,
             H + 2 * ph, W + 2 * pw);
  if (check_common(fn, N, C, H, W, K, R, S, sh, sw, ph, pw, dh, dw, groups, P, Q)) return -1;
  const int Cg = C / groups, Kg = K / groups;
  const int Kred = Cg * R * S;
  const int M = N * P * Q;
  const int KQ = ceil_div(Kred, 4 * kBKQ) * kBKQ;
  const bool plain = R == 1 && S == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0;
  const TileChoice t = choose_tile(Kg, M, groups, KQ / kBKQ, true, plain && KQ / kBKQ <= 32 && !bf16_math() && !split_math());
  const int Ipad = ceil_div(Kg, t.bm) * t.bm;

  const size_t wp_bytes = align_up(sizeof(floatx4) * (size_t)groups * KQ * Ipad, 256);
  if (size_only) {
    *size_only = wp_bytes + sk_workspace_bytes();
    return 0;
  }
  void* ws = nullptr;
  if (!check_only && tt::workspace(wp_bytes + sk_workspace_bytes(), &ws)) return -1;
  floatx4* wp = (floatx4*)ws;
  // weight rows that are a whole number of chunks long are k-major 16-byte quads already
  const bool in_place = Kred % (4 * kBKQ) == 0;

  Igemm p{};
  p.src = x; p.wp = wp; p.bias = bias; p.out = y;
  if (in_place) {
    p.wraw = w;
    p.wRowStride = Kred;
  }
  p.wbuf = in_place ? (const void*)w : (const void*)wp;
  p.I = Kg; p.Ipad = Ipad; p.KQ = KQ; p.M = M;
  p.divUV = tt::make_fastdiv((uint32_t)(P * Q));
  p.divV = tt::make_fastdiv((uint32_t)Q);
  p.su = sh; p.bh = -ph; p.sv = sw; p.bw = -pw;
  p.Hlim = H; p.Wlim = W; p.srcRow = W;
  p.srcStrideN = C * H * W; p.srcStrideG = Cg * H * W;
  p.outStrideN = K * P * Q; p.outStrideG = Kg * P * Q; p.outStrideI = P * Q; p.outRow = Q;
  p.ou = 1; p.ouh = 0; p.ov = 1; p.ovw = 0;
  // y[k][n,hw] = sum_c w[k][c] * x[n][c][hw]: for 1x1 layers the gathered operand is x itself
  p.kStride = H * W;
  p.Kred = Kred;
  KTabArgs ka{Kred, KQ * 4, R, S, H * W, dh * W, dw, dh, dw, 0, 0};
  choose_mode(p, ka, plain && (H * W) % 4 == 0, N, P, Q,
              in_place ? (long long)sizeof(float) * K * Kred : (long long)wp_bytes, true);
  if (make_ktab(fn, p, ka, N, groups, P, Q, Cg, (long long)N * C * H * W, check_only, &p.ktab)) return -1;
  if (check_only) return 0;
  if (!in_place) {
    tt::ProfScope prof(TT_PROF_CONV_PREP);
    pack_w_fwd<<<dim3(ceil_div(Ipad, 64), KQ, groups), 64, 0, tt::stream()>>>(w, wp, Kg, Ipad, Kred, KQ);
    TT_LAUNCH_CHECK();
  }
  return launch_igemm(p, groups, t, TT_PROF_CONV_IGEMM_FWD, (floatx4*)((char*)ws + wp_bytes));
}

static int conv2d_dgrad(const float* dy, const float* w, const float* bias, float* dx, int N, int C, int Hx, int Wx,
                        int K, int R, int S, int sh, int sw, int ph, int pw, int dh, int dw, int groups, int P,
                        int Q, size_t* size_only, bool check_only = false) {
  const char* fn = "tt_conv2d_dgrad_f32";
  TT_API_LOCK();
  if (!check_only) {
    TT_REQUIRE_INIT();
    TT_REQUIRE(dy && w && dx, "tt_conv2d_dgrad_f32: null tensor pointer");
    TT_REQUIRE_ALIGNED("tt_conv2d_dgrad_f32", dy, w, dx);
  }
  if (check_common(fn, N, C, Hx, Wx, K, R, S, sh, sw, ph, pw, dh, dw, groups, P, Q)) return -1;
  const long long dy_elems = (long long)N * K * P * Q;
  // One dy pixel per image spread over a whole R x S kernel (the first layer of a transposed
  // generator: latent vector -> R x S map): every dx pixel has exactly one tap, tap (h, w), so
  // dx[n][(c,h,w)] = sum_k dy[n][k] * w[k][(c,h,w)] is the input gradient of a 1x1 convolution
  // with C*R*S channels on 1x1 images.  As R x S taps it would run R*S times the products.
  if (P == 1 && Q == 1 && R * S > 1 && ph == 0 && pw == 0 && dh == 1 && dw == 1 && Hx == R && Wx == S && groups == 1 &&
      bias == nullptr && tt::fits_i32((long long)C * R * S))
    return conv2d_dgrad(dy, w, nullptr, dx, N, C * R * S, 1, 1, K, 1, 1, 1, 1, 0, 0, 1, 1, 1, 1, 1, size_only,
                        check_only);
  const int Cg = C / groups, Kg = K / groups;
  const int gh = gcd(sh, dh), gw = gcd(sw, dw);
  const int rstep = sh / gh, sstep = sw / gw;   // valid taps of a class: r0, r0+rstep, ...
  const int eh = dh / gh, ew = dw / gw;          // dy row/column step per tap

  const int classes = sh * sw;
  TT_REQUIRE(classes <= 4096, "tt_conv2d_dgrad_f32: stride %d x %d not supported", sh, sw);
  hipStream_t st = check_only ? nullptr : tt::stream();

  if (groups == 1 && classes > 1 && classes * Cg <= 64 && Hx >= sh && Wx >= sw) {
    // tiny Cg: per-class GEMMs would fill 3 of 32 MFMA rows; stack all classes as rows instead
    // A cell of the output is one period of the stride pattern, or a few of them side by side:
    // fh x fw periods make sh*fh x sw*fw pixel classes, each Cg rows of the GEMM.  More classes
    // fill more of the 32 or 64 tile rows, at the price of a union tap window one dy pixel
    // larger per added period; the cell with the fewest tile MACs per output pixel is taken.
    auto window = [](int cell, int stride, int pad, int taps, int dil, int* lo, int* hi) {
      *lo = 1 << 30;
      *hi = -(1 << 30);
      for (int cc = 0; cc < cell; ++cc)
        for (int r = 0; r < taps; ++r)
          if (((cc + pad - r * dil) % stride + stride) % stride == 0) {
            const int a = (cc + pad - r * dil) / stride;   // exact
            *lo = a < *lo ? a : *lo;
            *hi = a > *hi ? a : *hi;
          }
    };
    int fh = 1, fw = 1;
    {
      // equal costs: the taller cell first (its stores keep the narrower column stride)
      static const int kCells[6][2] = {{1, 1}, {2, 1}, {1, 2}, {2, 2}, {1, 4}, {2, 4}};
      long long best = -1;
      for (const auto& cell : kCells) {
        const int th = cell[0], tw = cell[1];
        const int rows = sh * th * sw * tw * Cg;
        if (rows > 64 || Hx < sh * th || Wx < sw * tw) continue;
        int lo, hi, lo2, hi2;
        window(sh * th, sh, ph, R, dh, &lo, &hi);
        window(sw * tw, sw, pw, S, dw, &lo2, &hi2);
        if (lo > hi || lo2 > hi2) continue;
        const long long taps = (long long)(hi - lo + 1) * (hi2 - lo2 + 1);
        if (th > 1 || tw > 1) {
          if (taps > 31) continue;   // larger cells only while the tap-mask mode holds their window
          // and only while about 1.5 tiles per CU remain: with fewer, too few blocks are resident to
          // cover each other's load latency and the saved MACs are lost again (measured)
          const long long cells = (long long)N * ceil_div(Hx, sh * th) * ceil_div(Wx, sw * tw);
          if (cells < 256LL * dense_cell_min_tiles()) continue;
        }
        // tile MACs per output pixel, scaled by 8 so that the division by the cell size is exact
        const long long cost = (rows <= 32 ? 32 : 64) * taps * (8 / (th * tw));
        if (best < 0 || cost < best) { best = cost; fh = th; fw = tw; }
      }
    }
    const int cellH = sh * fh, cellW = sw * fw;
    int amin, amax, bmin, bmax;
    window(cellH, sh, ph, R, dh, &amin, &amax);
    window(cellW, sw, pw, S, dw, &bmin, &bmax);
    if (amin <= amax && bmin <= bmax) {
      const int Na = amax - amin + 1, Nb = bmax - bmin + 1;
      const int I = cellH * cellW * Cg;
      const int Kred = Kg * Na * Nb;
      const int KQ = ceil_div(Kred, 4 * kBKQ) * kBKQ;
      const int U = ceil_div(Hx, cellH), V = ceil_div(Wx, cellW);
      const int M = N * U * V;
      TileChoice t;
      t.bm = I <= 32 ? 32 : 64;
      t.bn = 256;
      t.sk_blocks = 0;
      const int Ipad = t.bm;
      const size_t wp_bytes = align_up(sizeof(floatx4) * (size_t)KQ * Ipad, 256);
      if (size_only) {
        *size_only = wp_bytes;
        return 0;
      }
      void* ws = nullptr;
      if (!check_only && tt::workspace(wp_bytes, &ws)) return -1;
      floatx4* wp = (floatx4*)ws;
      Igemm p{};
      p.src = dy; p.wp = wp; p.wbuf = wp; p.bias = bias; p.out = dx;
      p.I = I; p.Ipad = Ipad; p.KQ = KQ; p.M = M;
      p.divUV = tt::make_fastdiv((uint32_t)(U * V));
      p.divV = tt::make_fastdiv((uint32_t)V);
      p.su = fh; p.bh = amin; p.sv = fw; p.bw = bmin;
      p.Hlim = P; p.Wlim = Q; p.srcRow = Q;
      p.srcStrideN = K * P * Q; p.srcStrideG = 0;
      p.outStrideN = C * Hx * Wx; p.outStrideG = 0; p.outStrideI = 0; p.outRow = Wx;
      p.ou = cellH; p.ouh = 0; p.ov = cellW; p.ovw = 0;
      p.outH = Hx; p.outW = Wx;
      KTabArgs ka{Kred, KQ * 4, Na, Nb, P * Q, Q, 1, 1, 1, 0, 0};
      choose_mode(p, ka, false, N, U, V, (long long)wp_bytes, true);
      // (one group: the launch's group stride is 0, the check takes the whole of dy as one group)
      Igemm pc = p;
      pc.srcStrideG = K * P * Q;
      if (make_ktab(fn, pc, ka, N, 1, U, V, Kg, dy_elems, check_only, &p.ktab)) return -1;
      if (make_rowtab(fn, I, Cg, cellH, cellW, Hx, Wx, N, U, V, check_only, &p.rowtab)) return -1;
      if (check_only) return 0;
      {
        tt::ProfScope prof(TT_PROF_CONV_PREP);
        PackDense pa{Kg, Cg, R, S, sh, sw, ph, pw, dh, dw, Na, Nb, amin, bmin, I, Ipad, Kred, KQ, Hx * Wx, Wx, cellW};
        pack_w_dgrad_dense<<<dim3(ceil_div(Ipad, 64), KQ), 64, 0, st>>>(w, wp, pa);
        TT_LAUNCH_CHECK();
      }
      return launch_igemm(p, 1, t, TT_PROF_CONV_IGEMM_DGRAD, nullptr);
    }
  }

  // workspace: the largest class (all taps at stride 1) bounds every class
  int max_taps_r = ceil_div(R, rstep), max_taps_s = ceil_div(S, sstep);
  const int KQmax = ceil_div((long long)Kg * max_taps_r * max_taps_s, 4 * kBKQ) * kBKQ;
  const int IpadMax = ceil_div(Cg, 128) * 128;
  const size_t wp_bytes = align_up(sizeof(floatx4) * (size_t)groups * KQmax * IpadMax, 256);
  if (size_only) {
    *size_only = wp_bytes * classes + sk_workspace_bytes();
    return 0;
  }
  void* ws = nullptr;
  if (!check_only && tt::workspace(wp_bytes * classes + sk_workspace_bytes(), &ws)) return -1;
  floatx4* sk_partial = (floatx4*)((char*)ws + wp_bytes * classes);

  // Parity classes without a tap hold only bias (or zero).  Without a bias it is cheaper to
  // clear dx once with a streaming fill than to launch a strided store kernel per empty class.
  bool prefilled = false;
  // 1x1 kernels with a stride two wide: the one class that has a tap stores whole cells instead
  const int cell_fill = (bias == nullptr && R == 1 && S == 1 && ph == 0 && pw == 0 && sw == 2 && sh <= 4 &&
                         Hx == P * sh && Wx == Q * sw && Cg % 8 == 0 && (reinterpret_cast<uintptr_t>(dx) & 7) == 0)
                            ? sh : 0;
  if (cell_fill > 0) {
    prefilled = true;   // the classes without a tap have nothing left to do
  } else if (bias == nullptr) {
    bool any_empty = false;
    for (int ch = 0; ch < sh && ch < Hx; ++ch) {
      bool has = false;
      for (int r = 0; r < R; ++r) has |= ((ch + ph - r * dh) % sh + sh) % sh == 0;
      any_empty |= !has;
    }
    for (int cw = 0; cw < sw && cw < Wx; ++cw) {
      bool has = false;
      for (int s2 = 0; s2 < S; ++s2) has |= ((cw + pw - s2 * dw) % sw + sw) % sw == 0;
      any_empty |= !has;
    }
    if (any_empty) {
      if (!check_only) TT_HIP(hipMemsetAsync(dx, 0, sizeof(float) * (size_t)N * C * Hx * Wx, st));
      prefilled = true;
    }
  }

  // Several classes with taps mean several short launches in a row; splitting the reduction of
  // each costs more than the imbalance it removes (measured on 3x3 stride-2 layers, also with
  // the partial sums added inside the kernel: 0.19-0.21 ms against 0.15-0.17 ms for one shared grid).
  int tap_rows = 0, tap_cols = 0;
  for (int ch = 0; ch < sh && ch < Hx; ++ch)
    for (int r = 0; r < R; ++r)
      if (((ch + ph - r * dh) % sh + sh) % sh == 0) { ++tap_rows; break; }
  for (int cw = 0; cw < sw && cw < Wx; ++cw)
    for (int s2 = 0; s2 < S; ++s2)
      if (((cw + pw - s2 * dw) % sw + sw) % sw == 0) { ++tap_cols; break; }
  const bool allow_stream_k = tap_rows * tap_cols <= 1;

  // Classes that have taps and agree on tile shape and addressing mode go into one grid when
  // there are 2..kMaxMulti of them; anything else is launched on its own.
  IgemmMulti multi{};
  TileChoice multi_tile{};
  bool multi_ok = !allow_stream_k && tap_rows * tap_cols <= kMaxMulti;

  // First every class is planned (launch descriptor, index table, repack descriptor), then the
  // repacks run, then the matrix products.
  std::vector<PackDgradMulti> packs;
  std::vector<int> pack_kq, pack_ipad;
  int pack_n = 0;
  const int pack_limit = groups * kMaxMulti <= 65535 ? kMaxMulti : 1;   // grid.z = classes * groups
  std::vector<std::pair<Igemm, TileChoice>> singles;
  int slot = 0;
  for (int ch = 0; ch < sh && ch < Hx; ++ch) {
    // taps r with (ch + ph - r*dh) % sh == 0
    int r0 = -1;
    for (int r = 0; r < R && r < rstep; ++r)
      if (((ch + ph - r * dh) % sh + sh) % sh == 0) { r0 = r; break; }
    const int nTr = r0 < 0 ? 0 : ceil_div(R - r0, rstep);
    const int U = ceil_div(Hx - ch, sh);
    for (int cw = 0; cw < sw && cw < Wx; ++cw, ++slot) {
      int s0 = -1;
      for (int s = 0; s < S && s < sstep; ++s)
        if (((cw + pw - s * dw) % sw + sw) % sw == 0) { s0 = s; break; }
      const int nTs = s0 < 0 ? 0 : ceil_div(S - s0, sstep);
      const int V = ceil_div(Wx - cw, sw);
      const int Kred = Kg * nTr * nTs;
      if (Kred == 0 && prefilled) continue;
      const int M = N * U * V;
      const int KQ = ceil_div(Kred, 4 * kBKQ) * kBKQ;
      const bool plain = R == 1 && S == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0;
      const TileChoice t = choose_tile(Cg, M, groups, KQ / kBKQ, allow_stream_k,
                                       (plain && KQ / kBKQ <= 32 && !bf16_math() && !split_math()) || !allow_stream_k);
      const int Ipad = ceil_div(Cg, t.bm) * t.bm;
      floatx4* wp = (floatx4*)((char*)ws + wp_bytes * slot);
      Igemm p{};
      p.src = dy; p.wp = wp; p.wbuf = wp; p.bias = bias; p.out = dx;
      p.I = Cg; p.Ipad = Ipad; p.KQ = KQ; p.M = M;
      p.divUV = tt::make_fastdiv((uint32_t)(U * V));
      p.divV = tt::make_fastdiv((uint32_t)V);
      p.su = 1; p.sv = 1;
      p.Hlim = P; p.Wlim = Q; p.srcRow = Q;
      p.srcStrideN = K * P * Q; p.srcStrideG = Kg * P * Q;
      p.outStrideN = C * Hx * Wx; p.outStrideG = Cg * Hx * Wx; p.outStrideI = Hx * Wx; p.outRow = Wx;
      p.ou = sh; p.ouh = ch; p.ov = sw; p.ovw = cw;
      p.kStride = P * Q;   // 1x1 layers: dx[c][n,hw] = sum_k w[k][c] * dy[n][k][hw]
      p.cellFill = cell_fill;
      p.Kred = Kred;
      if (KQ > 0) {
        // h = u*sh + ch reads dy row (h + ph - r0*dh)/sh = u + (ch + ph - r0*dh)/sh  (exact)
        p.bh = (ch + ph - r0 * dh) / sh;   // numerator is a multiple of sh by choice of r0
        p.bw = (cw + pw - s0 * dw) / sw;
        KTabArgs ka{Kred, KQ * 4, nTr, nTs, P * Q, -eh * Q, -ew, -eh, -ew, 0, 0};
        // 1x1 layers with whole chunks of output channels: w[k][c] is read in place, transposed
        const bool in_place = R == 1 && S == 1 && Kred % (4 * kBKQ) == 0;
        choose_mode(p, ka,
                    R == 1 && S == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0 && Hx == P && Wx == Q && (P * Q) % 4 == 0,
                    N, U, V, in_place ? (long long)sizeof(float) * K * Cg : (long long)wp_bytes);
        if (make_ktab(fn, p, ka, N, groups, U, V, Kg, dy_elems, check_only, &p.ktab)) return -1;
        if (in_place && p.mode != kModeCompare) {
          p.wbuf = w;
          p.wTransStride = Cg;
        } else {
          // the classes' repacks are collected and launched together, kMaxMulti classes per launch
          if (packs.empty() || pack_n == pack_limit) {
            packs.push_back(PackDgradMulti{});
            packs.back().groups = groups;
            pack_n = 0;
            pack_kq.push_back(0);
            pack_ipad.push_back(0);
          }
          packs.back().c[pack_n++] = PackDgrad{Kg, Cg, R, S, Ipad, Kred, KQ, nTr, nTs, r0, rstep, s0, sstep, wp};
          pack_kq.back() = KQ > pack_kq.back() ? KQ : pack_kq.back();
          pack_ipad.back() = Ipad > pack_ipad.back() ? Ipad : pack_ipad.back();
        }
      }
      if (multi_ok && KQ > 0 && t.sk_blocks == 0 && p.wTransStride == 0 && p.mode != kModeGemm &&
          (multi.n == 0 || (t.bm == multi_tile.bm && t.bn == multi_tile.bn && p.mode == multi.c[0].mode))) {
        // longest reduction first: the heavy blocks start early, the light ones fill the tail
        int at = multi.n;
        while (at > 0 && multi.c[at - 1].KQ < p.KQ) {
          multi.c[at] = multi.c[at - 1];
          --at;
        }
        multi.c[at] = p;
        ++multi.n;
        multi_tile = t;
        continue;
      }
      singles.push_back({p, t});
    }
  }
  if (check_only) return 0;
  if (!packs.empty()) {
    tt::ProfScope prof(TT_PROF_CONV_PREP);
    for (size_t i = 0; i < packs.size(); ++i) {
      const int n = i + 1 < packs.size() ? pack_limit : pack_n;
      pack_w_dgrad<<<dim3(ceil_div(pack_ipad[i], 64), pack_kq[i], groups * n), 64, 0, st>>>(w, packs[i]);
      TT_LAUNCH_CHECK();
    }
  }
  for (auto& one : singles)
    if (launch_igemm(one.first, groups, one.second, TT_PROF_CONV_IGEMM_DGRAD, sk_partial)) return -1;
  if (multi.n == 1) {
    if (launch_igemm(multi.c[0], groups, multi_tile, TT_PROF_CONV_IGEMM_DGRAD, sk_partial)) return -1;
  } else if (multi.n > 1) {
    if (launch_igemm_multi(multi, groups, multi_tile, TT_PROF_CONV_IGEMM_DGRAD)) return -1;
  }
  return 0;
}

// The kernels index with 32-bit element offsets.  Forward and input gradient are independent per
// image, so a batch whose tensors have 2^31 elements or more runs as several calls over runs of
// images that stay below that (one image and the weights must fit on their own).
// Every run but the first starts `per` images into the tensors, and the kernels need 16-byte
// aligned pointers: `per` is rounded down until both tensors' runs are whole float4s long (one of
// four consecutive counts always is).  0: not even one image per run can be kept aligned.
static int images_per_call(int N, long long image_a, long long image_b) {
  const long long image = image_a > image_b ? image_a : image_b;
  if (N <= 0 || image <= 0 || (long long)N * image < 2147483647LL) return N;
  long long per = 2147483646LL / image;
  if (per < 1) per = 1;
  for (long long cand = per; cand >= 1 && cand > per - 4; --cand)
    if ((cand * image_a) % 4 == 0 && (cand * image_b) % 4 == 0) return (int)cand;
  return 0;
}
static long long out_size(long long in, int k, int s, int p, int d) { return (in + 2LL * p - (long long)d * (k - 1) - 1) / s + 1; }

int tt_conv2d_fwd_f32(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K,
                      int R, int S, int sh, int sw, int ph, int pw, int dh, int dw, int groups) {
  const long long xi = (long long)C * H * W;
  const long long yi = sh > 0 && sw > 0 ? (long long)K * out_size(H, R, sh, ph, dh) * out_size(W, S, sw, pw, dw) : 0;
  const int per = images_per_call(N, xi, yi);
  TT_REQUIRE(per > 0, "tt_conv2d_fwd_f32: a batch of 2^31 elements or more is cut into runs of images, and images of "
                      "%lld and %lld elements leave no run 16-byte aligned", xi, yi);
  if (per >= N) return conv2d_fwd(x, w, bias, y, N, C, H, W, K, R, S, sh, sw, ph, pw, dh, dw, groups, nullptr);
  for (int n0 = 0; n0 < N; n0 += per) {
    const int n = N - n0 < per ? N - n0 : per;
    if (int rc = conv2d_fwd(x + (size_t)n0 * xi, w, bias, y + (size_t)n0 * yi, n, C, H, W, K, R, S, sh, sw, ph, pw, dh,
                            dw, groups, nullptr))
      return rc;
  }
  return 0;
}

int tt_conv2d_dgrad_f32(const float* dy, const float* w, const float* bias, float* dx, int N, int C, int Hx, int Wx,
                        int K, int R, int S, int sh, int sw, int ph, int pw, int dh, int dw, int groups, int P,
                        int Q) {
  const long long xi = (long long)C * Hx * Wx, yi = (long long)K * P * Q;
  const int per = images_per_call(N, xi, yi);
  TT_REQUIRE(per > 0, "tt_conv2d_dgrad_f32: a batch of 2^31 elements or more is cut into runs of images, and images of "
                      "%lld and %lld elements leave no run 16-byte aligned", xi, yi);
  if (per >= N) return conv2d_dgrad(dy, w, bias, dx, N, C, Hx, Wx, K, R, S, sh, sw, ph, pw, dh, dw, groups, P, Q, nullptr);
  for (int n0 = 0; n0 < N; n0 += per) {
    const int n = N - n0 < per ? N - n0 : per;
    if (int rc = conv2d_dgrad(dy + (size_t)n0 * yi, w, bias, dx + (size_t)n0 * xi, n, C, Hx, Wx, K, R, S, sh, sw, ph, pw,
                              dh, dw, groups, P, Q, nullptr))
      return rc;
  }
  return 0;
}

// Instrumentation (tests, host-only): images per run for a batch of N images of `image_a` and
// `image_b` elements (input and output of a forward or input-gradient call); 0 = no aligned run.
int tt_conv2d_images_per_run(int N, long long image_a, long long image_b, int* per) {
  TT_REQUIRE(per != nullptr, "tt_conv2d_images_per_run: null result pointer");
  *per = images_per_call(N, image_a, image_b);
  return 0;
}

// Host-only: builds every index table the corresponding call would use for this geometry and checks
// each entry's reach against the tensors, as the calls themselves do once per new geometry.
int tt_conv2d_check_tables_fwd_f32(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int ph, int pw,
                                   int dh, int dw, int groups) {
  const long long yi = sh > 0 && sw > 0 ? (long long)K * out_size(H, R, sh, ph, dh) * out_size(W, S, sw, pw, dw) : 0;
  N = std::max(1, images_per_call(N, (long long)C * H * W, yi));
  return conv2d_fwd(nullptr, nullptr, nullptr, nullptr, N, C, H, W, K, R, S, sh, sw, ph, pw, dh, dw, groups, nullptr,
                    true);
}

int tt_conv2d_check_tables_dgrad_f32(int N, int C, int Hx, int Wx, int K, int R, int S, int sh, int sw, int ph, int pw,
                                     int dh, int dw, int groups, int P, int Q) {
  N = std::max(1, images_per_call(N, (long long)C * Hx * Wx, (long long)K * P * Q));
  return conv2d_dgrad(nullptr, nullptr, nullptr, nullptr, N, C, Hx, Wx, K, R, S, sh, sw, ph, pw, dh, dw, groups, P, Q,
                      nullptr, true);
}

// Host-only: damages single table entries of a few geometries (an offset one row, one element or
// one image off, in both addressing modes, forward and input gradient) and returns 0 when the
// table check refuses every damaged table and accepts the undamaged ones.
int tt_conv2d_check_tables_selftest(void) {
  TT_API_LOCK();
  struct Case { int R, pad, stride, entry, delta; };
  // 3x3 pad 1 (tap-mask tables: byte offsets), 6x6 pad 2 (compare-mode tables: element offsets)
  const Case cases[] = {{3, 1, 1, 0, 4}, {3, 1, 1, 5, 4 * 9}, {3, 1, 2, 17, -4 * 9 * 9}, {6, 2, 1, 3, 1}, {6, 2, 1, 40, -14}};
  int bad = 0;
  for (const Case& c : cases) {
    const int H = 9 + c.R, P = (H + 2 * c.pad - c.R) / c.stride + 1;
    for (int pass = 0; pass < 2; ++pass) {
      for (int damaged = 0; damaged < 2; ++damaged) {
        g_selftest_fault_entry = damaged ? c.entry : -1;
        g_selftest_fault_delta = c.delta;
        const int rc = pass == 0 ? conv2d_fwd(nullptr, nullptr, nullptr, nullptr, 3, 8, H, H, 16, c.R, c.R, c.stride, c.stride,
                                              c.pad, c.pad, 1, 1, 1, nullptr, true)
                                 : conv2d_dgrad(nullptr, nullptr, nullptr, nullptr, 3, 8, H, H, 16, c.R, c.R, c.stride,
                                                c.stride, c.pad, c.pad, 1, 1, 1, P, P, nullptr, true);
        g_selftest_fault_entry = -1;
        if ((rc != 0) != (damaged != 0)) ++bad;
      }
    }
  }
  TT_REQUIRE(bad == 0, "tt_conv2d_check_tables_selftest: %d of 20 table checks gave the wrong verdict", bad);
  return 0;
}

// The queries run the same argument checks and planning as the calls themselves, with placeholder
// tensor pointers that are never dereferenced, and stop where the call would ask for the workspace.
int tt_workspace_size_conv2d_fwd_f32(size_t* bytes, int N, int C, int H, int W, int K, int R, int S, int sh, int sw,
                                     int ph, int pw, int dh, int dw, int groups) {
  TT_REQUIRE(bytes, "tt_workspace_size_conv2d_fwd_f32: null result pointer");
  const float* in = reinterpret_cast<const float*>(uintptr_t(256));
  const long long yi = sh > 0 && sw > 0 ? (long long)K * out_size(H, R, sh, ph, dh) * out_size(W, S, sw, pw, dw) : 0;
  N = std::max(1, images_per_call(N, (long long)C * H * W, yi));   // the largest of the calls a long batch is cut into
  return conv2d_fwd(in, in, nullptr, const_cast<float*>(in), N, C, H, W, K, R, S, sh, sw, ph, pw, dh, dw, groups,
                    bytes);
}

int tt_workspace_size_conv2d_dgrad_f32(size_t* bytes, int N, int C, int Hx, int Wx, int K, int R, int S, int sh,
                                       int sw, int ph, int pw, int dh, int dw, int groups, int P, int Q) {
  TT_REQUIRE(bytes, "tt_workspace_size_conv2d_dgrad_f32: null result pointer");
  const float* in = reinterpret_cast<const float*>(uintptr_t(256));
  N = std::max(1, images_per_call(N, (long long)C * Hx * Wx, (long long)K * P * Q));
  return conv2d_dgrad(in, in, nullptr, const_cast<float*>(in), N, C, Hx, Wx, K, R, S, sh, sw, ph, pw, dh, dw, groups,
                      P, Q, bytes);
}

}  // extern "C"
