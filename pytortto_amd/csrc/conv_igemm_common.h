// Types shared by the translation units of the implicit-GEMM convolution (conv_igemm.hip: the float32
// kernels and the launch planning; conv_igemm_bf16.hip: the bf16-first kernels of the optional
// reduced-precision mode).
#pragma once
#include "tt_common.h"

namespace ttc {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kBKQ = 4;          // k-quads per chunk (BK = 16)
constexpr int kInvalid = -(1 << 20);

// One entry per reduction index k (padded with never-valid entries to a whole chunk).
struct KEntry {
  int off;   // element offset added to the pixel's base offset (tap-mask tables: byte offset, biased to be >= 0)
  int dhw;   // (row step & 0xffff) | (column step << 16), both signed 16 bit (tap-mask tables: tap number; 31, or 63 with the 64-bit mask, = padding)
};

typedef int intx2 __attribute__((ext_vector_type(2)));
typedef const intx2 __attribute__((address_space(4))) * ConstKTab;   // constant address space: scalar (s_load) access

struct Igemm {
  const float* src;
  const floatx4* wp;     // [G][KQ][Ipad] x 4 floats
  const KEntry* ktab;    // [KQ*4]
  const float* bias;     // [G*I] or null
  float* out;
  int I, Ipad, KQ, M;
  tt::FastDiv divUV, divV;   // m -> (n, u, v)
  int su, bh, sv, bw;        // ih0 = u*su + bh, iw0 = v*sv + bw
  int Hlim, Wlim, srcRow;
  int srcStrideN, srcStrideG;
  int outStrideN, outStrideG, outStrideI, outRow;
  int ou, ouh, ov, ovw;      // output row = u*ou + ouh, column = v*ov + ovw
  int tilesI;                // row tiles per group
  int tiles;                 // tilesI * pixel tiles
  // forward launches whose weight rows are a multiple of 4 long read the weights in place (a
  // row of w is already k-major): row stride in floats, 0 = use the repacked copy in wp
  const float* wraw;
  int wRowStride;
  // How the gathered operand is addressed:
  //   kModeCompare: 64-bit addresses, bounds compared per element (any geometry, any size)
  //   kModeGemm   : 1x1, stride 1, no padding: the operand is the [k][pixel] matrix of each image
  //                 itself; 16-byte buffer loads along pixels, kStride elements between k rows
  //   kModeTapMask: buffer loads; per tile every lane keeps one bit per tap (TB x TC <= 31 taps)
  //                 telling whether that tap falls outside the image for its pixel
  //   kModeTapMask64: the same with a 64-bit mask (32 .. 63 taps: 7x7 kernels), one 64-bit shift
  //                 per element instead of a 32-bit one
  // The two buffer modes address relative to the first image of the tile with 32-bit byte
  // offsets; the host selects them only when those stay below 2 GiB.
  int mode;
  int kStride, Kred;
  int TB, TC, stepH, stepW;  // tap window and steps of the table (tap-mask mode)
  int voffBias;              // elements added to every lane offset so that it is never negative
  long long srdBias;         // elements subtracted from the buffer base to make up for all biases
  const void* wbuf;          // buffer modes: base of the weight operand (wp or wraw)
  // buffer-mode input gradients of 1x1 layers read w[k][c] in place, transposed: row i of the
  // GEMM is column c of w, so lanes (rows) are contiguous and k strides by wTransStride = C/groups
  int wTransStride;
  // dense input-gradient launches only (all stride-parity classes as rows of one GEMM):
  // row i -> {element offset c*Hx*Wx + ch*Wx + cw, ch, cw, c}; output bounds outH x outW
  const int4* rowtab;
  int outH, outW;
  // strided 1x1 input gradients: only one pixel of every sh x 2 cell of dx has a tap.  > 0: the
  // launch stores each value together with the zero to its right (one 8-byte store) and zero
  // pairs into the cellFill - 1 rows below, so dx needs no clearing beforehand
  int cellFill;
  // stream-K launches only: the tiles*chunks reduction steps are dealt evenly to the blocks
  int skDpTiles;             // tiles [0, skDpTiles) are computed whole, block b takes b, b+blocks, ...
  int skBlocks;              // blocks that share the remaining tiles' reduction steps
  long long skIters;         // (tiles - skDpTiles) * (KQ / kBKQ)
  floatx4* skPartial;        // [skBlocks][acc float4s per thread][256] partial accumulators, one slot per block
  unsigned* skFlags;         // [block] = skEpoch once the block's partial is in memory
  unsigned skEpoch;          // differs from launch to launch, so the flags never need clearing
  unsigned* skError;         // one word in pinned host memory: set when a wait for a flag ran out
};


// Several data-parallel launches in one grid (the stride-parity classes of a strided input
// gradient): blocks [first[i], first[i+1]) belong to launch i.  One grid instead of a short
// launch per class, each with its own ramp-up and tail.
constexpr int kMaxMulti = 4;
struct IgemmMulti {
  Igemm c[kMaxMulti];
  int first[kMaxMulti + 1];
  int n;
};

constexpr int kModeCompare = 0, kModeGemm = 1, kModeTapMask = 2, kModeTapMask64 = 3;
constexpr int kSrdFlags = 0x00020000;        // raw buffer, 32-bit data format
constexpr int kSrdRecords = 0x7fffffff;      // offsets with bit 31 set are out of range and read 0

__device__ __forceinline__ float as_float(unsigned v) { return __builtin_bit_cast(float, v); }

// The bf16-first kernels (conv_igemm_bf16.hip).  `supported` tells whether they take launch `p`
// (tile rows `bm` as planned by the caller); `launch` enqueues it on the library stream.
bool bf16_first_supported(const Igemm& p, int groups, int bm);
void bf16_first_launch(const Igemm& p, int groups, int bm, hipStream_t st);


// Float32 arithmetic in three bf16 terms (conv_igemm_x3.hip: the kernel body of conv_igemm_kernel.h
// instantiated on six v_mfma_f32_32x32x16_bf16 per product step).  `bm` x `bn` is the tile the caller
// planned; `sk_blocks` > 0 asks for the persistent (stream-K) grid, which is launched only if the
// device holds that many blocks at once (`forced_occupancy` >= 0 replaces what the device says:
// tests); returns whether the persistent grid was launched.
bool x3_launch(const Igemm& p, int groups, int sk_blocks, int bm, int bn, int forced_occupancy, hipStream_t st);
void x3_launch_multi(const IgemmMulti& m, int groups, int bm, int bn, hipStream_t st);
// resident blocks per compute unit of its stream-K kernels, the smallest over every instantiation
int x3_min_resident_blocks();

}  // namespace ttc
