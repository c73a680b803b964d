// bf16-first implicit-GEMM convolution for gfx950: the kernels behind the optional reduced-precision
// mode (tt_set_conv_math(TT_CONV_MATH_BF16)) of Conv2d forward and the stride-1 input gradient.
//
// Same product as the float32 kernels,  D[i, m] = sum_k  A[i, k] * G[k, m]  (+ bias[i]),  with both
// operands rounded to bfloat16 (nearest even) and contracted by v_mfma_f32_32x32x16_bf16 into float32
// accumulators; tensors stay float32 in memory.  What differs from running the float32 kernel's
// schedule on bf16 instructions is everything around the matrix instruction, which is sixteen times
// shorter here and leaves nothing to hide work behind:
//   * operands are converted once, on their way INTO LDS (v_cvt_pk_bf16_f32 on the fetched
//     registers), not after every LDS read: half the LDS bytes, no conversion next to the MFMAs;
//   * LDS holds 16-byte units of eight consecutive k of one row / pixel, [k/8][row][8 bf16]: one
//     ds_read_b128 is a lane's whole operand of a 16-deep MFMA step;
//   * a chunk is 32 deep (two MFMA steps per accumulator), one barrier per chunk, double-buffered
//     LDS, the next chunk's global loads in flight across the MFMAs of the current one;
//   * plain matrix products (1x1 layers) fetch 16 bytes per lane along pixels and transpose four
//     k x four pixels in registers; gathered taps reuse the float32 kernels' per-lane tap masks and
//     scalar index tables;
//   * no reduction is shared between blocks: one tile per block, three blocks per compute unit.
// Launches it does not take (few-channel dense input gradients, strided input gradients, kernels
// beyond 31 taps, reductions that are not whole chunks) stay on the float32 kernels' bf16
// instantiations.
#include "conv_igemm_common.h"

namespace {

using namespace ttc;

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));

constexpr int kBK = 32;    // reduction depth of a chunk
constexpr int kK8 = kBK / 8;

__device__ __forceinline__ unsigned pack2(float lo, float hi) {
  const bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(unsigned, v);
}

// Column of a row / pixel inside an LDS line: one empty 16-byte unit after every sixteen, so that the
// 8-byte writes of the transposing fetch (lanes four pixels apart) spread over the banks while reads
// of 32 consecutive rows stay conflict-free.
__device__ __forceinline__ int pos(int i) { return i + (i >> 4); }
constexpr int line_units(int n) { return n + n / 16 + 2; }

// How the weight operand is fetched:
//   kRows : rows of w are contiguous along k (forward, Kred a whole number of chunks): in place
//   kCols : w[k][c] read in place for the input gradient of a 1x1 layer: rows of the product are
//           columns of w, fetched 16 bytes along c and transposed in registers
//   kQuads: the repacked copy wp[k/4][row][4] of the float32 kernels
constexpr int kRows = 0, kCols = 1, kQuads = 2;

template <int WM, int WN, int MT, int NT, bool GEMM, int AMODE>
__global__ __launch_bounds__(kThreads, 3) void igemm_bf16_first(const Igemm p, const int tilesM) {
  static_assert(WM * WN == 4, "four waves per block");
  constexpr int BM = WM * MT * 32, BN = WN * NT * 32;
  static_assert(BN == 128 && (BM == 128 || BM == 64), "tile shape");
  constexpr int ALINE = line_units(BM), BLINE = line_units(BN);
  __shared__ uintx4 As[2][kK8][ALINE];
  __shared__ uintx4 Bs[2][kK8][BLINE];

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int g = blockIdx.y;
  const int tile = tt::xcd_remap((int)blockIdx.x, (int)gridDim.x);
  const int tilesI = p.Ipad / BM;
  const int i0 = (tile % tilesI) * BM;
  const int m0 = (tile / tilesI) * BN;
  (void)tilesM;

  // ---- gathered operand: per-lane offsets fixed for the tile ---------------------------------------
  const uint32_t n0 = tt::fd_div((uint32_t)__builtin_amdgcn_readfirstlane(m0), p.divUV);   // first image of the tile
  const long long rebase = (long long)n0 * p.srcStrideN + (long long)g * p.srcStrideG - p.srdBias;
  const __amdgpu_buffer_rsrc_t srcSrd = __builtin_amdgcn_make_buffer_rsrc((void*)(p.src + rebase), 0, kSrdRecords, kSrdFlags);
  const __amdgpu_buffer_rsrc_t wSrd = __builtin_amdgcn_make_buffer_rsrc((void*)p.wbuf, 0, kSrdRecords, kSrdFlags);
  const ConstKTab ktab = (ConstKTab)(uintptr_t)p.ktab;
  int bvoff = 0;
  uint32_t nmask = ~0u;   // tap-mask mode: bit t set = tap t lies outside the image for this lane's pixel
  // plain matrix product: thread = (pixel quad, group of four k rows); taps: thread = (pixel, group of 16 k)
  const int gpq = tid % 32, gkg = tid / 32;
  const int tpx = tid % BN;
  const int tkg = __builtin_amdgcn_readfirstlane(tid / BN);
  if constexpr (GEMM) {
    const int mq = min(m0 + 4 * gpq, p.M - 4);   // quads past the end re-read the last one; never stored
    const uint32_t n = tt::fd_div((uint32_t)mq, p.divUV);
    bvoff = 4 * ((int)(n - n0) * p.srcStrideN + (int)((uint32_t)mq - n * p.divUV.d) + 4 * gkg * p.kStride);
  } else {
    const int m = m0 + tpx;
    if (m < p.M) {
      const uint32_t n = tt::fd_div((uint32_t)m, p.divUV);
      const uint32_t rem = (uint32_t)m - n * p.divUV.d;
      const uint32_t u = tt::fd_div(rem, p.divV);
      const uint32_t v = rem - u * p.divV.d;
      const int ih = (int)u * p.su + p.bh, iw = (int)v * p.sv + p.bw;
      bvoff = 4 * ((int)(n - n0) * p.srcStrideN + ih * p.srcRow + iw + p.voffBias);
      uint32_t cols = 0, inside = 0;
      for (int c = 0; c < p.TC; ++c) cols |= (uint32_t)((unsigned)(iw + c * p.stepW) < (unsigned)p.Wlim) << c;
      for (int b = 0; b < p.TB; ++b)
        if ((unsigned)(ih + b * p.stepH) < (unsigned)p.Hlim) inside |= cols << (b * p.TC);
      nmask = ~inside;   // the top bit (the padding entries' tap) always stays set: TB*TC <= 31
    }
  }

  // ---- weight operand: per-lane offsets fixed for the tile -----------------------------------------
  constexpr int A_PASSES = BM / 64;                 // kRows: rows per thread
  constexpr int A_KPT = BM / 32;                    // kCols: k rows per thread (4 or 2)
  constexpr int A_QPT = BM / 32;                    // kQuads: k-quads per thread (4 or 2)
  int avoff[A_PASSES > 0 ? A_PASSES : 1];
  int asoff = 0;
  const int rko = tid % 4, rrow = tid / 4;                  // kRows: k-octet of the chunk, row (+ 64 per pass)
  const int ccq = tid % (BM / 4), ckg = tid / (BM / 4);     // kCols: row quad, k group
  const int qrow = tid % BM, qkg = tid / BM;                // kQuads: row, group of A_QPT quads
  if constexpr (AMODE == kRows) {
#pragma unroll
    for (int ps = 0; ps < A_PASSES; ++ps)   // rows past I are never stored
      avoff[ps] = 4 * (min(i0 + rrow + 64 * ps, p.I - 1) * p.wRowStride + 8 * rko);
    asoff = 4 * g * p.I * p.wRowStride;
  } else if constexpr (AMODE == kCols) {
    avoff[0] = 4 * (min(i0 + 4 * ccq, p.I - 4) + A_KPT * ckg * p.wTransStride);
    asoff = 4 * g * p.Kred * p.wTransStride;
  } else {
    avoff[0] = 16 * (A_QPT * qkg * p.Ipad + qrow);
    asoff = 16 * (g * p.KQ * p.Ipad + i0);
  }

  // ---- staging registers of the chunk being fetched --------------------------------------------------
  floatx4 breg[4];                 // GEMM: [k row][4 pixels];  taps: 16 k of one pixel
  floatx4 areg[AMODE == kRows ? 2 * A_PASSES : (AMODE == kCols ? A_KPT : A_QPT)];

  auto fetch = [&](const int chunk) __attribute__((always_inline)) {
    if constexpr (GEMM) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        breg[j] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(srcSrd, bvoff, 4 * (chunk * kBK + j) * p.kStride, 0));
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const intx2 t = ktab[chunk * kBK + tkg * 16 + e];   // {byte offset, tap}: wave-uniform, scalar loads
        const uint32_t vo = ((nmask >> t.y) << 31) | (uint32_t)bvoff;
        breg[e >> 2][e & 3] = as_float(__builtin_amdgcn_raw_buffer_load_b32(srcSrd, (int)vo, t.x, 0));
      }
    }
    if constexpr (AMODE == kRows) {
#pragma unroll
      for (int ps = 0; ps < A_PASSES; ++ps) {
        areg[2 * ps] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(wSrd, avoff[ps], asoff + 4 * chunk * kBK, 0));
        areg[2 * ps + 1] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(wSrd, avoff[ps], asoff + 4 * chunk * kBK + 16, 0));
      }
    } else if constexpr (AMODE == kCols) {
#pragma unroll
      for (int j = 0; j < A_KPT; ++j)
        areg[j] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(wSrd, avoff[0], asoff + 4 * (chunk * kBK + j) * p.wTransStride, 0));
    } else {
#pragma unroll
      for (int j = 0; j < A_QPT; ++j)
        areg[j] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(wSrd, avoff[0], asoff + 16 * (chunk * (kBK / 4) + j) * p.Ipad, 0));
    }
  };

  // Round to bf16 and write the staged chunk into LDS buffer `buf`.
  auto stage = [&](const int buf) __attribute__((always_inline)) {
    if constexpr (GEMM) {
      // four k rows x four pixels: per pixel the four k as 8 bytes, half of a unit
      char* line = reinterpret_cast<char*>(&Bs[buf][gkg >> 1][0]) + 8 * (gkg & 1);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *reinterpret_cast<uintx2*>(line + 16 * pos(4 * gpq + j)) =
            uintx2{pack2(breg[0][j], breg[1][j]), pack2(breg[2][j], breg[3][j])};
    } else {
      Bs[buf][2 * tkg][pos(tpx)] = uintx4{pack2(breg[0][0], breg[0][1]), pack2(breg[0][2], breg[0][3]),
                                         pack2(breg[1][0], breg[1][1]), pack2(breg[1][2], breg[1][3])};
      Bs[buf][2 * tkg + 1][pos(tpx)] = uintx4{pack2(breg[2][0], breg[2][1]), pack2(breg[2][2], breg[2][3]),
                                             pack2(breg[3][0], breg[3][1]), pack2(breg[3][2], breg[3][3])};
    }
    if constexpr (AMODE == kRows) {
#pragma unroll
      for (int ps = 0; ps < A_PASSES; ++ps)
        As[buf][rko][pos(rrow + 64 * ps)] =
            uintx4{pack2(areg[2 * ps][0], areg[2 * ps][1]), pack2(areg[2 * ps][2], areg[2 * ps][3]),
                   pack2(areg[2 * ps + 1][0], areg[2 * ps + 1][1]), pack2(areg[2 * ps + 1][2], areg[2 * ps + 1][3])};
    } else if constexpr (AMODE == kCols) {
      // A_KPT k rows x four rows of the product: per row its A_KPT consecutive k
      const int k0 = A_KPT * ckg;   // first k of this thread inside the chunk
      char* line = reinterpret_cast<char*>(&As[buf][k0 >> 3][0]) + 2 * (k0 & 7);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        char* at = line + 16 * pos(4 * ccq + j);
        if constexpr (A_KPT == 4)
          *reinterpret_cast<uintx2*>(at) = uintx2{pack2(areg[0][j], areg[1][j]), pack2(areg[2][j], areg[3][j])};
        else
          *reinterpret_cast<unsigned*>(at) = pack2(areg[0][j], areg[1][j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < A_QPT; j += 2)
        As[buf][(A_QPT * qkg + j) >> 1][pos(qrow)] = uintx4{pack2(areg[j][0], areg[j][1]), pack2(areg[j][2], areg[j][3]),
                                                          pack2(areg[j + 1][0], areg[j + 1][1]), pack2(areg[j + 1][2], areg[j + 1][3])};
    }
  };

  floatx16 acc[MT][NT];
#pragma unroll
  for (int a = 0; a < MT; ++a)
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // MFMA step kk of a chunk contracts k8-blocks 2*kk (lanes 0-31) and 2*kk + 1 (lanes 32-63): a lane's
  // 16 bytes are its eight k of that block, the same eight for both operands.
  auto multiply = [&](const int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int kk = 0; kk < kK8 / 2; ++kk) {
      bf16x8 a[MT], b[NT];
#pragma unroll
      for (int x = 0; x < MT; ++x) a[x] = __builtin_bit_cast(bf16x8, As[buf][2 * kk + h][pos((wm * MT + x) * 32 + l32)]);
#pragma unroll
      for (int y = 0; y < NT; ++y) b[y] = __builtin_bit_cast(bf16x8, Bs[buf][2 * kk + h][pos((wn * NT + y) * 32 + l32)]);
#pragma unroll
      for (int x = 0; x < MT; ++x)
#pragma unroll
        for (int y = 0; y < NT; ++y) acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[x], b[y], acc[x][y], 0, 0, 0);
    }
  };

  const int chunks = p.Kred / kBK;
  fetch(0);
  stage(0);
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    const int buf = c & 1;
    if (c + 1 < chunks) fetch(c + 1);     // in flight across this chunk's MFMAs
    multiply(buf);
    if (c + 1 < chunks) stage(buf ^ 1);   // the other buffer was last read before the previous barrier
    __syncthreads();
  }

  // ---- epilogue: accumulator register r of a 32x32 tile holds row 8*(r/4) + 4*h + r%4, column l32 ----
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
    obase[y] = (uint32_t)((int)n * p.outStrideN + g * p.outStrideG + ((int)u * p.ou + p.ouh) * p.outRow + (int)v * p.ov + p.ovw);
  }
  if (p.bias == nullptr && (p.I & 7) == 0) {
    // rows in whole groups of eight: one scalar test per group, a row's address is a scalar base plus
    // the lane's pixel offset
    const int i0u = __builtin_amdgcn_readfirstlane(i0);
    const uint32_t hoff = (uint32_t)(4 * h * p.outStrideI);
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
  float bz[MT][16];
#pragma unroll
  for (int x = 0; x < MT; ++x)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = i0 + (wm * MT + x) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
      bz[x][r] = p.bias ? p.bias[g * p.I + min(i, p.I - 1)] : 0.f;
    }
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0x0f70);   // every load done before the first store: they share one counter
  __builtin_amdgcn_sched_barrier(0);
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
}

template <int WM, int WN, int MT, int NT>
void launch_shape(const Igemm& p, dim3 grid, int tilesM, hipStream_t st) {
  const bool gemm = p.mode == kModeGemm;
  const int amode = p.wTransStride > 0 ? kCols : (p.wRowStride > 0 ? kRows : kQuads);
  if (gemm && amode == kRows) igemm_bf16_first<WM, WN, MT, NT, true, kRows><<<grid, kThreads, 0, st>>>(p, tilesM);
  else if (gemm && amode == kCols) igemm_bf16_first<WM, WN, MT, NT, true, kCols><<<grid, kThreads, 0, st>>>(p, tilesM);
  else if (gemm) igemm_bf16_first<WM, WN, MT, NT, true, kQuads><<<grid, kThreads, 0, st>>>(p, tilesM);
  else if (amode == kRows) igemm_bf16_first<WM, WN, MT, NT, false, kRows><<<grid, kThreads, 0, st>>>(p, tilesM);
  else if (amode == kCols) igemm_bf16_first<WM, WN, MT, NT, false, kCols><<<grid, kThreads, 0, st>>>(p, tilesM);
  else igemm_bf16_first<WM, WN, MT, NT, false, kQuads><<<grid, kThreads, 0, st>>>(p, tilesM);
}

}  // namespace

namespace ttc {

bool bf16_first_supported(const Igemm& p, int groups, int bm) {
  if (bm != 64 && bm != 128) return false;
  if (p.rowtab != nullptr || p.cellFill != 0) return false;              // dense and whole-cell input gradients
  if (p.mode != kModeGemm && p.mode != kModeTapMask) return false;       // 64-bit masks, compared bounds
  if (p.Kred <= 0 || p.Kred % kBK != 0) return false;                    // whole chunks only
  if (p.wTransStride > 0 && (p.I % 4 != 0)) return false;                // transposed in-place weights: 16 bytes along rows
  if (p.wTransStride == 0 && p.wRowStride == 0 && p.Ipad % bm != 0) return false;
  if (groups > 65535) return false;
  return true;
}

void bf16_first_launch(const Igemm& p, int groups, int bm, hipStream_t st) {
  const int tilesM = (p.M + 127) / 128;
  const int tilesI = p.Ipad / bm;
  const dim3 grid((unsigned)(tilesI * tilesM), (unsigned)groups);
  if (bm == 128) launch_shape<2, 2, 2, 2>(p, grid, tilesM, st);
  else launch_shape<1, 4, 2, 1>(p, grid, tilesM, st);
}

}  // namespace ttc
