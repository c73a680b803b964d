// Implicit-GEMM convolution on fp32 MFMA for gfx950: Conv2d forward, and the gather-form input
// gradient that also serves as ConvTranspose2d forward.  NCHW float32, no im2col buffer in HBM.
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
constexpr int kMaxMulti = 4;
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

// ---- the GEMM kernel -----------------------------------------------------------------------------

// Blocks are dealt round-robin to the 8 XCDs; tt::xcd_remap gives each XCD a contiguous range of
// tiles, row tiles fastest, so blocks that share a pixel tile (same gathered operand) share an L2.
using tt::xcd_remap;

typedef float floatx2 __attribute__((ext_vector_type(2)));

// s_waitcnt vmcnt(0) in straight-line code.  Stores share the counter with loads, and the
// compiler, unsure after a branch whether an earlier load has been waited for, repeats the wait
// in every conditional store block -- which then waits for the stores before it.  One explicit
// wait before the first store lets it drop those.
__device__ __forceinline__ void wait_loads() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0), expcnt and lgkmcnt left alone
  __builtin_amdgcn_sched_barrier(0);
}

// 16-byte buffer accesses at system scope (cache-policy bits sc0 | sc1): the store is written
// through to memory and the load is served from memory, past the per-XCD L2s, which do not snoop
// each other.  The stream-K partial accumulators travel between blocks on different XCDs this way,
// without the cache-wide write-back and invalidate that a release / acquire fence at device scope
// costs.  Ordering is by completion: the writer waits for its stores (vmcnt) before the flag goes
// up, the reader issues its loads after it has seen the flag.
constexpr int kSystemScope = 1 | 16;   // sc0, sc1
// stream-K flags: one word per block.  A wait that runs out (about four seconds of polling: a block
// that was never scheduled, i.e. a grid that does not fit the device at two blocks per CU next to
// foreign work) is reported through a word in pinned host memory, which the host reads after its
// next stream synchronisation without any device operation.
constexpr int kSkFlagWords = 4096, kSkSpinLimit = 1 << 22;
__device__ __forceinline__ void store_coherent(__amdgpu_buffer_rsrc_t rsrc, int byte_off, floatx4 v) {
  typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uintx4, v), rsrc, byte_off, 0, kSystemScope);
}
__device__ __forceinline__ floatx4 load_coherent(__amdgpu_buffer_rsrc_t rsrc, int byte_off) {
  return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off, 0, kSystemScope));
}

// Eight float32 values (a lane's k values of one 16-deep matrix step) as three vectors of bfloat16
// terms that add up to them exactly: term i of value v is the bf16 nearest to v minus the terms
// before it.
__device__ __forceinline__ void three_terms(const floatx4 lo, const floatx4 hi, bf16x8 (&out)[3]) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
  const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  unsigned t[3][4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    float e = v[2 * q], o = v[2 * q + 1];   // the pair shares a register of every term
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      const bf16x2 pair = {(__bf16)e, (__bf16)o};
      t[i][q] = __builtin_bit_cast(unsigned, pair);
      if (i < 2) {
        e -= as_float(t[i][q] << 16);
        o -= as_float(t[i][q] & 0xffff0000u);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 3; ++i) out[i] = __builtin_bit_cast(bf16x8, uintx4{t[i][0], t[i][1], t[i][2], t[i][3]});
}

// The kernel body: `block_x` is the block's index among the blocks of launch `p` (a launch may
// be one of several that share a grid, see igemm_multi_f32).
// BF: 0 = float32 matrix instructions; 1 = operands rounded to bfloat16; 3 = float32 arithmetic on the
// bf16 matrix instructions (three bf16 terms per operand element, six products per step).
template <int WM, int WN, int MT, int NT, bool SK, int MODE, bool AT, int BF>
__device__ __forceinline__ void igemm_body(const Igemm& p, const int block_x) {
  static_assert(WM * WN == 4, "four waves per block");
  constexpr bool GEMM = MODE == kModeGemm, BUF = MODE != kModeCompare;
  constexpr bool MASK = MODE == kModeTapMask || MODE == kModeTapMask64;
  using TapBits = std::conditional_t<MODE == kModeTapMask64, uint64_t, uint32_t>;
  constexpr int BM = WM * MT * 32, BN = WN * NT * 32;
  constexpr int A_ITEMS = (kBKQ * BM + kThreads - 1) / kThreads, B_ITEMS = kBKQ * BN / kThreads;
  static_assert(B_ITEMS >= 1 && kThreads % BM == 0 && kThreads % BN == 0, "tile shape");
  __shared__ floatx4 As[2][kBKQ][BM];
  __shared__ floatx4 Bs[2][kBKQ][BN];

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int g = blockIdx.y;

  // gathered operand: within a tile this thread always loads the same pixel, for B_ITEMS
  // k-quads per chunk
  const int pix = tid % BN;
  const int bq0 = __builtin_amdgcn_readfirstlane(tid / BN);   // first k-quad (wave-uniform)
  const int arow = tid % BM, aq0 = tid / BM;
  const ConstKTab ktab = (ConstKTab)(uintptr_t)p.ktab;
  constexpr int GPQ = BN / 4, GR = BN / 64;
  const int gpq = tid % GPQ, gkr = (tid / GPQ) * GR;
  int i0 = 0, m0 = 0, ih0 = kInvalid, iw0 = 0, base = 0;
  const floatx4* __restrict__ wsrc = p.wp;
  const float* __restrict__ wrow = p.wraw;
  // buffer modes: resource descriptors (scalar), per-lane byte offsets fixed for the tile, and
  // the scalar byte offset of the tile's weight rows
  __amdgpu_buffer_rsrc_t srcSrd = __builtin_amdgcn_make_buffer_rsrc((void*)p.src, 0, kSrdRecords, kSrdFlags);
  const __amdgpu_buffer_rsrc_t wSrd = __builtin_amdgcn_make_buffer_rsrc((void*)p.wbuf, 0, kSrdRecords, kSrdFlags);
  int bvoff = 0, avoff = 0, asoff = 0;
  TapBits nmask = ~(TapBits)0;   // bit t set: tap t lies outside the image for this lane's pixel
  constexpr int AQ = kThreads / BM;   // k-quads between a thread's weight items
  auto set_tile = [&](int tile) __attribute__((always_inline)) {
    i0 = (tile % p.tilesI) * BM;
    m0 = (tile / p.tilesI) * BN;
    if constexpr (BUF) {
      const uint32_t n0 = tt::fd_div((uint32_t)__builtin_amdgcn_readfirstlane(m0), p.divUV);   // first image of the tile
      const long long rebase = (long long)n0 * p.srcStrideN + (long long)g * p.srcStrideG - p.srdBias;
      srcSrd = __builtin_amdgcn_make_buffer_rsrc((void*)(p.src + rebase), 0, kSrdRecords, kSrdFlags);
      if constexpr (GEMM) {
        // four consecutive pixels per thread: m % 4 == 0 and (U*V) % 4 == 0, so they share n
        const int mq = min(m0 + 4 * gpq, p.M - 4);   // past-the-end quads re-read the last one; never stored
        const uint32_t n = tt::fd_div((uint32_t)mq, p.divUV);
        bvoff = 4 * ((int)(n - n0) * p.srcStrideN + (int)((uint32_t)mq - n * p.divUV.d) + gkr * p.kStride);
      } else {
        const int m = m0 + pix;
        bvoff = 0;
        nmask = ~(TapBits)0;
        if (m < p.M) {
          const uint32_t n = tt::fd_div((uint32_t)m, p.divUV);
          const uint32_t rem = (uint32_t)m - n * p.divUV.d;
          const uint32_t u = tt::fd_div(rem, p.divV);
          const uint32_t v = rem - u * p.divV.d;
          const int ih = (int)u * p.su + p.bh, iw = (int)v * p.sv + p.bw;
          bvoff = 4 * ((int)(n - n0) * p.srcStrideN + ih * p.srcRow + iw + p.voffBias);
          TapBits cols = 0, inside = 0;
          for (int c = 0; c < p.TC; ++c) cols |= (TapBits)((unsigned)(iw + c * p.stepW) < (unsigned)p.Wlim) << c;
          for (int b = 0; b < p.TB; ++b)
            if ((unsigned)(ih + b * p.stepH) < (unsigned)p.Hlim) inside |= cols << (b * p.TC);
          nmask = ~inside;   // the top bit (the padding entries' tap) always stays set: TB*TC <= 31 or 63
        }
      }
      if constexpr (AT) {   // w[k][c] in place: k = Kred rows of I = C/groups columns per group
        avoff = 4 * (min(i0 + arow, p.I - 1) + 4 * aq0 * p.wTransStride);
        asoff = 4 * g * p.Kred * p.wTransStride;
      } else if (p.wRowStride) {   // in place; rows past I are never stored
        avoff = 4 * (min(i0 + arow, p.I - 1) * p.wRowStride + 4 * aq0);
        asoff = 4 * g * p.I * p.wRowStride;
      } else {
        avoff = 16 * (aq0 * p.Ipad + arow);
        asoff = 16 * (g * p.KQ * p.Ipad + i0);
      }
    } else {
      ih0 = kInvalid;
      iw0 = 0;
      base = 0;
      const int m = m0 + pix;
      if (m < p.M) {
        const uint32_t n = tt::fd_div((uint32_t)m, p.divUV);
        const uint32_t rem = (uint32_t)m - n * p.divUV.d;
        const uint32_t u = tt::fd_div(rem, p.divV);
        const uint32_t v = rem - u * p.divV.d;
        ih0 = (int)u * p.su + p.bh;
        iw0 = (int)v * p.sv + p.bw;
        base = (int)n * p.srcStrideN + g * p.srcStrideG + ih0 * p.srcRow + iw0;
      }
      wsrc = p.wp + (size_t)g * p.KQ * p.Ipad + i0;
      if (p.wRowStride) wrow = p.wraw + (size_t)(g * p.I + min(i0 + arow, p.I - 1)) * p.wRowStride;   // rows past I: never stored
    }
  };

  // plain-GEMM mode: thread (gpq, gkr) loads rows gkr .. gkr+GR-1 of the chunk's 16 k rows for
  // pixel quad gpq with one 16-byte load per row; no bounds tests, no table (the reduction is a
  // whole number of chunks in this mode), and only the scalar offset moves with k
  floatx4 greg[GR];
  auto load_g_row = [&](int chunk, int j) __attribute__((always_inline)) {
    const int soff = 4 * (chunk * (4 * kBKQ) + j) * p.kStride;
    greg[j] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(srcSrd, bvoff, soff, 0));
  };
  // In this mode the gathered tile lies in LDS as it lies in memory, [k][pixel]: a fetched
  // 16-byte vector is written as it is (consecutive lanes, consecutive addresses: no bank
  // conflicts, where scattering its four pixels into the k-quad layout cost up to eight-way
  // ones), and read_ops picks a lane's four k values with four dword reads off one address.
  auto store_g = [&](int buf) __attribute__((always_inline)) {
    float* tile = reinterpret_cast<float*>(&Bs[buf][0][0]);
#pragma unroll
    for (int j = 0; j < GR; ++j) *reinterpret_cast<floatx4*>(tile + (gkr + j) * BN + 4 * gpq) = greg[j];
  };

  floatx4 areg[A_ITEMS];
  floatx4 breg[B_ITEMS];
  bool bok[B_ITEMS][4];   // applied when the values are written to LDS
  constexpr int nB = 4 * B_ITEMS;
  intx2 tab_e[nB];        // table entries {off, dhw} of the chunk being fetched (SGPRs)

  auto load_tab = [&](int chunk) __attribute__((always_inline)) {
    if constexpr (GEMM) return;
#pragma unroll
    for (int it = 0; it < B_ITEMS; ++it) {
      const int kq = chunk * kBKQ + bq0 + it * (kThreads / BN);
#pragma unroll
      for (int j = 0; j < 4; ++j) tab_e[it * 4 + j] = ktab[kq * 4 + j];
    }
  };
  auto load_a_item = [&](int chunk, int it) __attribute__((always_inline)) {
    const int q = aq0 + it * (kThreads / BM);   // always < kBKQ unless the tile has fewer than 64 rows
    if (BM >= 64 || q < kBKQ) {   // (the compile-time half keeps the load out of a divergent branch)
      const int kq = chunk * kBKQ + q;
      if constexpr (AT) {
        // four k values of this row: one coalesced dword load each (whole chunks only)
        const int soff = asoff + 16 * (chunk * kBKQ + it * AQ) * p.wTransStride;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          areg[it][j] = as_float(__builtin_amdgcn_raw_buffer_load_b32(wSrd, avoff, soff + 4 * j * p.wTransStride, 0));
      } else if constexpr (BUF) {
        // in place only when rows are a whole number of chunks long: nothing to zero
        const int soff = asoff + (p.wRowStride ? 16 * (chunk * kBKQ + it * AQ) : 16 * (chunk * kBKQ + it * AQ) * p.Ipad);
        areg[it] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(wSrd, avoff, soff, 0));
      } else if (p.wRowStride) {   // in place; quads past the end of the row must be zero, not garbage
        areg[it] = 4 * kq < p.wRowStride ? *reinterpret_cast<const floatx4*>(wrow + 4 * kq) : floatx4{0.f, 0.f, 0.f, 0.f};
      } else {
        areg[it] = wsrc[(size_t)kq * p.Ipad + arow];
      }
    }
  };
  auto load_b_elem = [&](int e) __attribute__((always_inline)) {   // uses tab_e: must follow load_tab() of the same chunk
    const intx2 t = tab_e[e];
    if constexpr (MASK) {
      // {byte offset, tap}: shift the lane's "outside" bit for this tap into bit 31 of its offset
      const uint32_t vo = ((uint32_t)(nmask >> t.y) << 31) | (uint32_t)bvoff;
      breg[e >> 2][e & 3] = as_float(__builtin_amdgcn_raw_buffer_load_b32(srcSrd, (int)vo, t.x, 0));
      return;
    }
    const int ih = ih0 + (int)(short)(t.y & 0xffff);
    const int iw = iw0 + (t.y >> 16);
    const bool ok = (unsigned)ih < (unsigned)p.Hlim && (unsigned)iw < (unsigned)p.Wlim;
    const uint32_t off = ok ? (uint32_t)(base + t.x) : 0u;
    breg[e >> 2][e & 3] = p.src[off];
    bok[e >> 2][e & 3] = ok;
  };
  auto store_a_item = [&](int buf, int it) __attribute__((always_inline)) {
    const int q = aq0 + it * (kThreads / BM);
    if (BM >= 64 || q < kBKQ) As[buf][q][arow] = areg[it];
  };
  auto store_b_item = [&](int buf, int it) __attribute__((always_inline)) {
    floatx4 v = breg[it];
    if constexpr (MODE == kModeCompare) {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = bok[it][j] ? breg[it][j] : 0.f;
    }
    Bs[buf][bq0 + it * (kThreads / BN)][pix] = v;
  };

  // MFMA operands of one chunk: [kk][tile] float4 = four k-steps each.  Lanes 0-31 take quad
  // 2*kk, lanes 32-63 quad 2*kk+1, so MFMA step j of half kk contracts k = 4*(2*kk + h) + j.
  floatx4 opA[2][2][MT], opB[2][2][NT];
  auto read_ops = [&](int set, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
      for (int x = 0; x < MT; ++x) opA[set][kk][x] = As[buf][kk * 2 + h][(wm * MT + x) * 32 + l32];
#pragma unroll
      for (int y = 0; y < NT; ++y) {
        if constexpr (GEMM) {
          const float* tile = reinterpret_cast<const float*>(&Bs[buf][0][0]);
#pragma unroll
          for (int j = 0; j < 4; ++j) opB[set][kk][y][j] = tile[(4 * (kk * 2 + h) + j) * BN + (wn * NT + y) * 32 + l32];
        } else {
          opB[set][kk][y] = Bs[buf][kk * 2 + h][(wn * NT + y) * 32 + l32];
        }
      }
    }
  };

  floatx16 acc[MT][NT];

  auto load_all = [&](int chunk) __attribute__((always_inline)) {   // tab_e must hold `chunk`'s entries
    if constexpr (GEMM) {
#pragma unroll
      for (int j = 0; j < GR; ++j) load_g_row(chunk, j);
    } else {
#pragma unroll
      for (int e = 0; e < nB; ++e) load_b_elem(e);
    }
#pragma unroll
    for (int it = 0; it < A_ITEMS; ++it) load_a_item(chunk, it);
  };
  auto store_all = [&](int buf) __attribute__((always_inline)) {
    if constexpr (GEMM) {
      store_g(buf);
    } else {
#pragma unroll
      for (int it = 0; it < B_ITEMS; ++it) store_b_item(buf, it);
    }
#pragma unroll
    for (int it = 0; it < A_ITEMS; ++it) store_a_item(buf, it);
  };

  // One chunk of MFMAs (operand set `set`, read from LDS buffer `set` earlier) with the work for
  // the following chunks woven in between them, one small step per MFMA, so that it executes in
  // the shadow of the 64-cycle matrix instructions:
  //   slots 0..      : global loads of chunk `nchunk` (gathered elements, then weight quads)
  //   slots T-8..    : write them to the other LDS buffer
  //   slot  T-4      : barrier, fetch the operands of the next chunk from LDS, and start the
  //                    scalar loads of the table entries of chunk `nnchunk`
  // sched_barrier pins this order; the compiler otherwise sinks the loads below the MFMAs.
  constexpr int T = 8 * MT * NT;
  auto chunk_body = [&](const int set, const int nchunk, const int nnchunk) __attribute__((always_inline)) {
    if constexpr (BF == 3) {
      // float32 arithmetic on the bf16 matrix instructions.  Every operand value v read from LDS
      // becomes three bfloat16 terms, t0 = bf16(v), t1 = bf16(v - t0), t2 = bf16(v - t0 - t1) (nearest
      // even; both differences are exact in float32), so that v = t0 + t1 + t2 exactly, and six
      // v_mfma_f32_32x32x16_bf16 per accumulator add up every product of terms except (t1,t2), (t2,t1)
      // and (t2,t2), which together stay below 2^-24 of the product: half an ulp of it, what rounding
      // it to float32 once would cost.  bf16 x bf16 is exact in float32; accumulation is float32.
      // Six instructions of 32 cycles replace eight of 64; the price is the conversion, about 5.5
      // vector instructions per value, which issue next to the matrix instructions of the other
      // wave on the SIMD.
      load_all(nchunk);
      __builtin_amdgcn_sched_barrier(0);
      bf16x8 a[MT][3], b[NT][3];
#pragma unroll
      for (int x = 0; x < MT; ++x) three_terms(opA[set][0][x], opA[set][1][x], a[x]);
#pragma unroll
      for (int y = 0; y < NT; ++y) three_terms(opB[set][0][y], opB[set][1][y], b[y]);
      constexpr int ta[6] = {2, 0, 1, 1, 0, 0}, tb[6] = {0, 2, 1, 0, 1, 0};   // smallest products first
#pragma unroll
      for (int o = 0; o < 6; ++o)
#pragma unroll
        for (int x = 0; x < MT; ++x)
#pragma unroll
          for (int y = 0; y < NT; ++y)
            acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[x][ta[o]], b[y][tb[o]], acc[x][y], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      store_all(set ^ 1);
      __syncthreads();
      read_ops(set ^ 1, set ^ 1);
      load_tab(nnchunk);
    } else if constexpr (BF == 1) {
      // bf16 matrix instructions: one v_mfma_f32_32x32x16_bf16 per accumulator contracts the whole
      // chunk (a lane's two quads are its eight k values, the same ones for both operands), so a
      // chunk's matrix time is a sixteenth of the fp32 one and there is no shadow to weave the
      // loads into; more resident blocks hide them instead.  Operands are rounded to bf16
      // (nearest even) after the LDS read; accumulation stays fp32.
      load_all(nchunk);
      __builtin_amdgcn_sched_barrier(0);
      bf16x8 a[MT], b[NT];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int x = 0; x < MT; ++x) {
          a[x][j] = (__bf16)opA[set][0][x][j];
          a[x][4 + j] = (__bf16)opA[set][1][x][j];
        }
#pragma unroll
        for (int y = 0; y < NT; ++y) {
          b[y][j] = (__bf16)opB[set][0][y][j];
          b[y][4 + j] = (__bf16)opB[set][1][y][j];
        }
      }
#pragma unroll
      for (int x = 0; x < MT; ++x)
#pragma unroll
        for (int y = 0; y < NT; ++y)
          acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[x], b[y], acc[x][y], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      store_all(set ^ 1);
      __syncthreads();
      read_ops(set ^ 1, set ^ 1);
      load_tab(nnchunk);
    } else if constexpr (T >= 32) {
      constexpr int kStore = T - 8, kSync = T - 4;
      constexpr int nL = GEMM ? GR : nB;   // load steps of the gathered operand
      static_assert(nL + A_ITEMS <= kStore && kStore + B_ITEMS + A_ITEMS - 1 <= kSync, "schedule does not fit");
#pragma unroll
      for (int s = 0; s < T; ++s) {
        const int kk = s / (4 * MT * NT), rem = s % (4 * MT * NT);
        const int j = rem / (MT * NT), x = (rem % (MT * NT)) / NT, y = rem % NT;
        acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x2f32(opA[set][kk][x][j], opB[set][kk][y][j], acc[x][y], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (GEMM) {
          if (s < nL) load_g_row(nchunk, s);
          else if (s < nL + A_ITEMS) load_a_item(nchunk, s - nL);
          if (s == kStore) store_g(set ^ 1);
          else if (s > kStore && s <= kStore + A_ITEMS) store_a_item(set ^ 1, s - kStore - 1);
        } else {
          if (s < nB) load_b_elem(s);
          else if (s < nB + A_ITEMS) load_a_item(nchunk, s - nB);
          if (s >= kStore && s < kStore + B_ITEMS) store_b_item(set ^ 1, s - kStore);
          else if (s >= kStore + B_ITEMS && s < kStore + B_ITEMS + A_ITEMS) store_a_item(set ^ 1, s - kStore - B_ITEMS);
        }
        if (s == kSync) {
          __syncthreads();
          read_ops(set ^ 1, set ^ 1);
          load_tab(nnchunk);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      load_all(nchunk);
      __builtin_amdgcn_sched_barrier(0);
      // the burst of MFMAs runs at raised wave priority: with five to seven light blocks on a CU
      // some wave is always in its prologue or epilogue, and its vector instructions would
      // otherwise take issue slots from the matrix pipe (measured: -0.5 % on these launches;
      // keeping the whole reduction loop of every tile size at raised priority measured 2.5 % slower)
      __builtin_amdgcn_s_setprio(2);
#pragma unroll
      for (int s = 0; s < T; ++s) {
        const int kk = s / (4 * MT * NT), rem = s % (4 * MT * NT);
        const int j = rem / (MT * NT), x = (rem % (MT * NT)) / NT, y = rem % NT;
        acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x2f32(opA[set][kk][x][j], opB[set][kk][y][j], acc[x][y], 0, 0, 0);
      }
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      store_all(set ^ 1);
      __syncthreads();
      read_ops(set ^ 1, set ^ 1);
      load_tab(nnchunk);
    }
  };

  // Reduction chunks [c0, c1) of the current tile into acc (zeroed first).
  auto run_segment = [&](const int c0, const int c1) __attribute__((always_inline)) {
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
      for (int b = 0; b < NT; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
    if (c0 >= c1) return;
    const int last = c1 - 1;
    load_tab(c0);
    load_all(c0);
    store_all(0);
    __syncthreads();
    read_ops(0, 0);
    load_tab(min(c0 + 1, last));
    // the final chunks re-fetch the last chunk (cache hits) instead of branching: a loop body
    // free of conditions keeps the prefetch registers in registers
    int c = c0;
    for (; c + 1 < c1; c += 2) {
      chunk_body(0, c + 1, min(c + 2, last));
      chunk_body(1, min(c + 2, last), min(c + 3, last));
    }
    if (c < c1) chunk_body(0, c, c);
  };

  // epilogue: accumulator register r of a 32x32 tile holds row 8*(r/4) + 4*h + r%4, column l32
  auto epilogue = [&]() __attribute__((always_inline)) {
    uint32_t obase[NT];
    bool mok[NT];
#pragma unroll
    for (int y = 0; y < NT; ++y) {
      const int m = m0 + (wn * NT + y) * 32 + l32;
      mok[y] = m < p.M;
      const uint32_t mm = mok[y] ? (uint32_t)m : 0u;
      const uint32_t n = tt::fd_div(mm, p.divUV);
      const uint32_t rem = mm - n * p.divUV.d;
      const uint32_t u = tt::fd_div(rem, p.divV);
      const uint32_t v = rem - u * p.divV.d;
      obase[y] = (uint32_t)((int)n * p.outStrideN + g * p.outStrideG + ((int)u * p.ou + p.ouh) * p.outRow +
                            (int)v * p.ov + p.ovw);
    }
    if (p.rowtab == nullptr && p.bias == nullptr && (p.I & 7) == 0) {
      // The common case, without bias and with rows in whole groups of eight: a group is inside the
      // matrix or not for the whole wave (scalar test), a row's address is a scalar base plus the
      // lane's 32-bit pixel offset, and nothing is left to compute per store.  Short reductions
      // (1x1 layers) spend a noticeable share of their time here otherwise.
      const int i0u = __builtin_amdgcn_readfirstlane(i0);
      const uint32_t hoff = (uint32_t)(4 * h * p.outStrideI);
      if (p.cellFill > 0) {
#pragma unroll
        for (int y = 0; y < NT; ++y) {
          if (mok[y]) {
            const uint32_t vo = obase[y] + hoff;
#pragma unroll
            for (int x = 0; x < MT; ++x) {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const int srow = i0u + (wm * MT + x) * 32 + 8 * q;
                if (srow < p.I) {
#pragma unroll
                  for (int j = 0; j < 4; ++j) {
                    float* __restrict__ rowp = p.out + (size_t)(srow + j) * (size_t)p.outStrideI;
                    *reinterpret_cast<floatx2*>(rowp + vo) = floatx2{acc[x][y][4 * q + j], 0.f};
                    for (int f = 1; f < p.cellFill; ++f)
                      *reinterpret_cast<floatx2*>(rowp + vo + (uint32_t)(f * p.outRow)) = floatx2{0.f, 0.f};
                  }
                }
              }
            }
          }
        }
        return;
      }
#pragma unroll
      for (int y = 0; y < NT; ++y) {
        if (mok[y]) {
          const uint32_t vo = obase[y] + hoff;
#pragma unroll
          for (int x = 0; x < MT; ++x) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int srow = i0u + (wm * MT + x) * 32 + 8 * q;
              if (srow < p.I) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  float* __restrict__ rowp = p.out + (size_t)(srow + j) * (size_t)p.outStrideI;
                  rowp[vo] = acc[x][y][4 * q + j];
                }
              }
            }
          }
        }
      }
      return;
    }
    // Everything the stores need is fetched before the first store: a wait for a load issued
    // between stores would also wait for every store before it (one counter covers both), and
    // the epilogue would run at one store round trip per row.
    if (p.rowtab == nullptr) {
      float bz[MT][16];
#pragma unroll
      for (int x = 0; x < MT; ++x)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = i0 + (wm * MT + x) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
          bz[x][r] = p.bias ? p.bias[g * p.I + min(i, p.I - 1)] : 0.f;
        }
      wait_loads();
#pragma unroll
      for (int x = 0; x < MT; ++x) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = i0 + (wm * MT + x) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
          if (i < p.I) {
            const uint32_t ioff = (uint32_t)(i * p.outStrideI);
#pragma unroll
            for (int y = 0; y < NT; ++y)
              if (mok[y]) p.out[obase[y] + ioff] = acc[x][y][r] + bz[x][r];
          }
        }
      }
    } else {
      // rows are (parity class, channel): each row has its own offset inside the sh x sw cell
      // anchored at the pixel, and cells at the bottom/right edge may be cut off
      int oh[NT], ow[NT];
#pragma unroll
      for (int y = 0; y < NT; ++y) {
        const int m = m0 + (wn * NT + y) * 32 + l32;
        const uint32_t mm = mok[y] ? (uint32_t)m : 0u;
        const uint32_t rem = mm - tt::fd_div(mm, p.divUV) * p.divUV.d;
        const uint32_t u = tt::fd_div(rem, p.divV);
        oh[y] = (int)u * p.ou;
        ow[y] = (int)(rem - u * p.divV.d) * p.ov;
      }
      // eight rows at a time: their table entries and biases are loaded, then stored to
#pragma unroll
      for (int x = 0; x < MT; ++x) {
#pragma unroll
        for (int r0 = 0; r0 < 16; r0 += 8) {
          int4 row[8];
          float bz[8];
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            const int i = i0 + (wm * MT + x) * 32 + 8 * ((r0 + r) >> 2) + 4 * h + (r & 3);
            row[r] = p.rowtab[min(i, p.I - 1)];
          }
#pragma unroll
          for (int r = 0; r < 8; ++r) bz[r] = p.bias ? p.bias[row[r].w] : 0.f;
          wait_loads();
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            const int i = i0 + (wm * MT + x) * 32 + 8 * ((r0 + r) >> 2) + 4 * h + (r & 3);
            if (i < p.I) {
              const int4 e = row[r];
#pragma unroll
              for (int y = 0; y < NT; ++y)
                if (mok[y] && oh[y] + e.y < p.outH && ow[y] + e.z < p.outW)
                  p.out[obase[y] + (uint32_t)e.x] = acc[x][y][r0 + r] + bz[r];
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };

  const int chunks = p.KQ / kBKQ;
  if constexpr (!SK) {
    set_tile(xcd_remap(block_x, p.tiles));
    run_segment(0, chunks);
    epilogue();
  } else {
    // Whole rounds of tiles are computed one tile per block as usual.  The tiles left over would
    // load the CUs unevenly, so their reduction steps (tile-major sequence of T = tiles*chunks
    // steps) are dealt evenly instead: block b owns steps [b*T/P, (b+1)*T/P).
    // That share covers, in tile order: at most one segment that finishes a tile somebody else
    // started (the first), whole tiles, and at most one segment that does not reach its tile's end
    // (the last).  The last one is computed FIRST and published: partial accumulators into the
    // block's slot, written through to memory, then the block's flag raised to this launch's epoch.
    // The first one is computed LAST: the block then waits for the flags of the blocks holding the
    // tile's earlier steps -- set long before, as the first thing those blocks did --, adds their
    // partials in block order (a fixed order: results do not depend on timing) and stores the tile
    // through the ordinary epilogue.  No second kernel, one partial slot per block.
    // A block only ever waits for blocks that publish before they do anything else, so no wait
    // depends on another wait; the wait is bounded all the same, and a wait that runs out raises an
    // error word that tt_sync() and the device-to-host copy report.
    // (A release / acquire fence pair at device scope instead of write-through accesses was measured
    // 11 % slower on the whole step: the fences write back and invalidate whole L2s on this multi-die
    // part.  A second kernel that added the partials, the earlier design, cost 0.3 ms per step more.)
    constexpr int kAccQ = MT * NT * 4;
    const int b = xcd_remap(blockIdx.x, gridDim.x);
    {
      long long it = 0, end = 0;
      if (b < p.skBlocks) {
        it = (long long)b * p.skIters / p.skBlocks;
        end = (long long)(b + 1) * p.skIters / p.skBlocks;
      }
      int t_first = 0, t_last = -1, c0f = 0, endc = chunks;
      if (it < end) {
        t_first = (int)(it / chunks);
        c0f = (int)(it - (long long)t_first * chunks);
        t_last = (int)((end - 1) / chunks);
        endc = (int)(end - (long long)t_last * chunks);
      }
      const bool has_open = it < end && endc < chunks;                                  // last segment, unfinished
      const bool has_closing = it < end && c0f > 0 && (t_first < t_last || endc == chunks);   // first segment, finishes its tile
      if (has_open) {
        set_tile(p.skDpTiles + t_last);
        run_segment(t_last == t_first ? c0f : 0, endc);
        const __amdgpu_buffer_rsrc_t part =
            __builtin_amdgcn_make_buffer_rsrc((void*)(p.skPartial + (size_t)b * kAccQ * kThreads), 0, kSrdRecords, kSrdFlags);
#pragma unroll
        for (int x = 0; x < MT; ++x)
#pragma unroll
          for (int y = 0; y < NT; ++y)
#pragma unroll
            for (int q = 0; q < 4; ++q)
              store_coherent(part, 16 * (((x * NT + y) * 4 + q) * kThreads + tid),
                             floatx4{acc[x][y][4 * q], acc[x][y][4 * q + 1], acc[x][y][4 * q + 2], acc[x][y][4 * q + 3]});
        // every wave waits until its write-through stores are acknowledged, then one thread raises the flag
        __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
        __syncthreads();
        if (tid == 0) __hip_atomic_store(&p.skFlags[b], p.skEpoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
      for (int tile = b; tile < p.skDpTiles; tile += (int)gridDim.x) {
        set_tile(tile);
        run_segment(0, chunks);
        epilogue();
        __syncthreads();
      }
      for (int t = t_first; t <= t_last; ++t) {
        const bool whole = (t > t_first || c0f == 0) && (t < t_last || endc == chunks);
        if (!whole) continue;
        set_tile(p.skDpTiles + t);
        run_segment(0, chunks);
        epilogue();
        __syncthreads();
      }
      if (has_closing) {
        set_tile(p.skDpTiles + t_first);
        run_segment(c0f, chunks);
        // blocks that hold the earlier steps of this tile: the one containing its first step ... b - 1
        const long long t0 = (long long)t_first * chunks;
        const int b_first = (int)(((t0 + 1) * p.skBlocks - 1) / p.skIters);
        if (tid == 0) {
          bool lost = false;
          for (int j = b_first; j < b && !lost; ++j) {
            int spins = 0;
            while (__hip_atomic_load(&p.skFlags[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != p.skEpoch) {
              if (++spins >= kSkSpinLimit) {
                // never hang: give up, report the launch as failed, and do not wait for the
                // remaining predecessors either (one spin budget per block, not one per predecessor)
                __hip_atomic_store(p.skError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                lost = true;
                break;
              }
              __builtin_amdgcn_s_sleep(4);
            }
          }
        }
        __syncthreads();
        for (int j = b_first; j < b; ++j) {
          const __amdgpu_buffer_rsrc_t part =
              __builtin_amdgcn_make_buffer_rsrc((void*)(p.skPartial + (size_t)j * kAccQ * kThreads), 0, kSrdRecords, kSrdFlags);
#pragma unroll
          for (int x = 0; x < MT; ++x)
#pragma unroll
            for (int y = 0; y < NT; ++y) {
              floatx4 v[4];
#pragma unroll
              for (int q = 0; q < 4; ++q) v[q] = load_coherent(part, 16 * (((x * NT + y) * 4 + q) * kThreads + tid));
#pragma unroll
              for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[x][y][4 * q + e] += v[q][e];
            }
        }
        epilogue();
      }
    }
  }
}

template <int WM, int WN, int MT, int NT, bool SK, int MODE, bool AT>
__global__ __launch_bounds__(kThreads, 2) void igemm_f32(const Igemm p) {
  igemm_body<WM, WN, MT, NT, SK, MODE, AT, 0>(p, (int)blockIdx.x);
}
// The same launch on bf16 matrix instructions (tt_set_conv_math); three blocks per CU.
template <int WM, int WN, int MT, int NT, bool SK, int MODE, bool AT>
__global__ __launch_bounds__(kThreads, 3) void igemm_bf16(const Igemm p) {
  igemm_body<WM, WN, MT, NT, SK, MODE, AT, 1>(p, (int)blockIdx.x);
}
// The same launch in float32 arithmetic carried out on the bf16 matrix instructions; two blocks per CU.
template <int WM, int WN, int MT, int NT, bool SK, int MODE, bool AT>
__global__ __launch_bounds__(kThreads, 2) void igemm_bf16x3(const Igemm p) {
  igemm_body<WM, WN, MT, NT, SK, MODE, AT, 3>(p, (int)blockIdx.x);
}

// Several data-parallel launches in one grid (the stride-parity classes of a strided input
// gradient): blocks [first[i], first[i+1]) belong to launch i.  One grid instead of a short
// launch per class, each with its own ramp-up and tail.
struct IgemmMulti {
  Igemm c[kMaxMulti];
  int first[kMaxMulti + 1];
  int n;
};
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
template <int WM, int WN, int MT, int NT, int MODE>
__global__ __launch_bounds__(kThreads, 2) void igemm_multi_bf16x3(const IgemmMulti m) {
  int ci = 0;
  while (ci + 1 < m.n && (int)blockIdx.x >= m.first[ci + 1]) ++ci;
  igemm_body<WM, WN, MT, NT, false, MODE, false, 3>(m.c[ci], (int)blockIdx.x - m.first[ci]);
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
    else if constexpr (BFK == 3) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, igemm_bf16x3<WM, WN, MT, NT, true, MODE, AT>, kThreads, 0);
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
  const int math = tt::conv_math();
  const bool bf = math == TT_CONV_MATH_BF16, x3 = math == TT_CONV_MATH_BF16X3;
  if (sk_blocks > 0) {
    int held = bf   ? sk_resident_blocks_per_cu<WM, WN, MT, NT, MODE, AT, 1>()
               : x3 ? sk_resident_blocks_per_cu<WM, WN, MT, NT, MODE, AT, 3>()
                    : sk_resident_blocks_per_cu<WM, WN, MT, NT, MODE, AT, 0>();
    if (g_sk_forced_occupancy >= 0) held = g_sk_forced_occupancy;
    if ((long long)held * cus() < sk_blocks) sk_blocks = 0;   // the data-parallel launch ignores the stream-K fields
  }
  if (sk_blocks > 0) {
    if (bf) igemm_bf16<WM, WN, MT, NT, true, MODE, AT><<<dim3(sk_blocks, 1), kThreads, 0, st>>>(p);
    else if (x3) igemm_bf16x3<WM, WN, MT, NT, true, MODE, AT><<<dim3(sk_blocks, 1), kThreads, 0, st>>>(p);
    else igemm_f32<WM, WN, MT, NT, true, MODE, AT><<<dim3(sk_blocks, 1), kThreads, 0, st>>>(p);
  } else if (bf) {
    igemm_bf16<WM, WN, MT, NT, false, MODE, AT><<<dim3(p.tiles, groups), kThreads, 0, st>>>(p);
  } else if (x3) {
    igemm_bf16x3<WM, WN, MT, NT, false, MODE, AT><<<dim3(p.tiles, groups), kThreads, 0, st>>>(p);
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
  if (t.bm == 128 && t.bn == 128)
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
  const bool bf = bf16_math(), x3 = split_math();
  if (m.c[0].mode == kModeTapMask) {
    if (bf) igemm_multi_bf16<WM, WN, MT, NT, kModeTapMask><<<grid, kThreads, 0, st>>>(m);
    else if (x3) igemm_multi_bf16x3<WM, WN, MT, NT, kModeTapMask><<<grid, kThreads, 0, st>>>(m);
    else igemm_multi_f32<WM, WN, MT, NT, kModeTapMask><<<grid, kThreads, 0, st>>>(m);
  } else {
    if (bf) igemm_multi_bf16<WM, WN, MT, NT, kModeCompare><<<grid, kThreads, 0, st>>>(m);
    else if (x3) igemm_multi_bf16x3<WM, WN, MT, NT, kModeCompare><<<grid, kThreads, 0, st>>>(m);
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
  if (t.bm == 128 && t.bn == 128)
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
  *blocks = bf16 == 3 ? sk_min_resident_all<3>() : bf16 ? sk_min_resident_all<1>() : sk_min_resident_all<0>();
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
