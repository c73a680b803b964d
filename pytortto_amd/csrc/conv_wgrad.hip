// Weight gradient of Conv2d on fp32 MFMA for gfx950 (NCHW float32).
//
// Per group:  dw[i, j] = sum_m  dy[m, i] * x~[m, j],   i = output channel, j = (c, r, s),
// m = (n, p, q) running over all N*P*Q output pixels (the reduction).  The output is small and
// the reduction long (up to ~8e5), so the reduction is split over blockIdx.z into `splits`
// contiguous ranges of 32-pixel chunks; each split writes an fp32 partial tile to the
// workspace and the partials are added in a fixed order in float64 (deterministic, and more
// accurate than one long fp32 accumulation).  When the whole grid is resident at once -- one round
// of two blocks per compute unit, which is what the split count aims for -- the adding happens
// inside the kernel: every block publishes its partial tile (write-through stores, then a flag),
// waits for the flags of the other splits of its tile, and adds 1/splits of the tile's elements
// over all splits.  Otherwise a second kernel (wgrad_reduce) adds them.
//
// Both operands are contiguous along the reduction index in NCHW memory, so lanes run along
// pixels for coalesced loads and the LDS tiles are [row][pixel] with a 4-float pad: an MFMA
// operand fetch is one ds_read_b128 holding four reduction steps, conflict-free because
// consecutive rows start 36 floats apart.  v_mfma_f32_32x32x2_f32 rows = output channels,
// columns = (c,r,s), so 32 lanes store 128 contiguous bytes of dw.
//
// Vector-ALU instructions cost matrix-pipe time on this part, so the usual launch (BUF) fetches
// with buffer loads: per chunk a lane computes one byte offset for its pixel in dy and one in x,
// each load adds a per-lane constant (row / column offset), padding taps set bit 31 of the
// offset from a per-chunk tap mask and read 0 through the buffer range check, and nothing is
// masked when the values are written to LDS.  Offsets are relative to the first image of the
// chunk.  Kernels of 32 to 63 taps (7x7) keep a 64-bit mask (WIDE: its upper half comes from a second
// table); geometries whose offsets could reach 2 GiB, or with more than 63 taps, take the
// compare-and-select path instead.
#include <algorithm>
#include <map>
#include <type_traits>
#include <vector>

#include "tt_common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kBK = 32;        // pixels per chunk
constexpr int kLd = kBK + 4;   // padded LDS row (floats)
constexpr int kInvalid = -(1 << 20);

struct Wgrad {
  const float* x;
  const float* dy;
  float* out;            // dw (splits == 1) or workspace [splits][G][Kg][J]
  int Kg, J, M;          // rows, columns (Cg*R*S), reduction length
  int chunks, chunksPerSplit;
  tt::FastDiv divPQ, divQ, divRS, divS;
  int sh, sw, ph, pw, dh, dw;
  int H, W, HW;
  int xStrideN, xStrideG;     // C*H*W, Cg*H*W
  int dyStrideN, dyStrideG;   // K*P*Q, Kg*P*Q
  int PQ;
  int tilesI;
  size_t outStrideSplit;      // G*Kg*J
  int R, S;                   // buffer path: taps, one bit each in the per-chunk mask
  int xBias;                  // buffer path: ph*W + pw, keeps lane offsets non-negative
  // buffer path: per output pixel m {image n, 4*(p*Q + q), 4*(ih*W + iw + xBias), tap mask};
  // entries from M to chunks*32 hold {N-1, bit 31, 0, all ones}.  Built once per geometry.
  const int4* pixtab;
  const int* pixhi;   // kernels of 32 .. 63 taps: bits 32 .. 63 of every pixel's tap mask
  // partial sums added inside the kernel (fuse != 0; the grid is one round of resident blocks):
  // `out` is dw itself, partial tiles go to fusePartial[group * tiles + tile][split] in the
  // accumulators' own register order, 16 bytes per lane
  int fuse;
  floatx4* fusePartial;
  unsigned* fuseFlags;    // [(group * tiles + tile) * splits + split] = fuseEpoch once the partial is in memory
  unsigned fuseEpoch;     // differs from launch to launch: the flags never need clearing
  unsigned* fuseError;    // pinned host word, set when a wait for a flag ran out
  int fuseKL, fuseNf;     // lanes along the splits, and float4s per pass, of the adding stage (KL * Nf = 256)
};

constexpr int kSrdFlags = 0x00020000;     // raw buffer, 32-bit data format
constexpr int kSrdRecords = 0x7fffffff;   // offsets with bit 31 set are out of range and read 0
__device__ __forceinline__ float as_float(unsigned v) { return __builtin_bit_cast(float, v); }

// 16-byte buffer accesses at system scope (cache-policy bits sc0 | sc1): written through to memory,
// read from memory, past the per-XCD L2s, which do not snoop each other.  Partial tiles travel
// between blocks on different XCDs this way; ordering is by completion (the writer waits for its
// stores before its flag goes up, the reader loads after it has seen the flag).
constexpr int kSystemScope = 1 | 16;
constexpr int kFuseFlagWords = 4096, kFuseSpinLimit = 1 << 22;
__device__ __forceinline__ void store_coherent(__amdgpu_buffer_rsrc_t rsrc, int byte_off, floatx4 v) {
  typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uintx4, v), rsrc, byte_off, 0, kSystemScope);
}
__device__ __forceinline__ floatx4 load_coherent(__amdgpu_buffer_rsrc_t rsrc, int byte_off) {
  return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off, 0, kSystemScope));
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned pack2(float lo, float hi) {   // two floats -> two bf16 (nearest even), lo in the low half
  const bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(unsigned, v);
}
__device__ __forceinline__ int pos16(int i) { return i + (i >> 4); }   // unit of row i in a bf16 LDS line
// The value the next lane holds (lanes 0, 2 of every quad get lanes 1, 3; odd lanes get their own).
__device__ __forceinline__ float next_lane(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xF5 /* quad_perm [1,1,3,3] */, 0xf, 0xf, false));
}

// Two blocks per CU is all the LDS tiles allow: tell the compiler not to squeeze registers (and
// spill) for a third wave per SIMD.
// VA / VB (buffer path only): dy / x are fetched as 16-byte vectors of four consecutive pixels
// (thread = (row group of 32, pixel quad) instead of (row group of 8, pixel)).  VA needs P*Q to be
// a multiple of 4 so that a quad never straddles two images, VB in addition a 1x1, stride-1,
// unpadded layer, where x is indexed by the output pixel like dy and has no padding to mask.
// BF: the optional bf16 variant (tt_set_conv_math): operands rounded to bfloat16 after the LDS
// read, v_mfma_f32_32x32x16_bf16, float32 accumulation.
template <int WM, int WN, int MT, int NT, bool BUF, bool VA, bool VB, bool BF, bool WIDE = false>
__device__ __forceinline__ void wgrad_body(const Wgrad& p) {
  static_assert(WM * WN == 4, "four waves per block");
  static_assert(BUF || (!VA && !VB), "vector fetches belong to the buffer path");
  static_assert(!WIDE || (BUF && !VB), "64-bit tap masks belong to the buffer path of kernels larger than 1x1");
  using TapBits = std::conditional_t<WIDE, uint64_t, uint32_t>;
  constexpr int BM = WM * MT * 32, BN = WN * NT * 32;
  constexpr int A_ROWS = VA ? BM / 32 : BM / 8, B_ROWS = VB ? BN / 32 : BN / 8;   // fetches per thread and chunk
  // float32 arithmetic: [row][32 pixels + pad] floats.  bf16 arithmetic: operands are rounded on their
  // way INTO LDS and lie as 16-byte units of eight consecutive pixels of one row, [pixel / 8][row][8
  // bf16] (one ds_read_b128 is a lane's operand of a 16-deep MFMA step; rows padded by one unit per
  // sixteen, lines 12 or 4 units past a multiple of sixteen so that the four lines of a chunk spread
  // over the banks): half the LDS bytes and no conversion next to the matrix instructions.
  constexpr int ALINE = BM == 128 ? 140 : 68, BLINE = BN == 128 ? 140 : 68;
  constexpr size_t kBytesA = BF ? sizeof(uintx4) * 2 * 4 * ALINE : sizeof(float) * 2 * BM * kLd;
  constexpr size_t kBytesB = BF ? sizeof(uintx4) * 2 * 4 * BLINE : sizeof(float) * 2 * BN * kLd;
  __shared__ __attribute__((aligned(16))) char lds[kBytesA + kBytesB];
  char* const ldsA = lds;
  char* const ldsB = lds + kBytesA;
  float (*As)[BM][kLd] = reinterpret_cast<float (*)[BM][kLd]>(ldsA);
  float (*Bs)[BN][kLd] = reinterpret_cast<float (*)[BN][kLd]>(ldsB);
  uintx4 (*As16)[4][ALINE] = reinterpret_cast<uintx4 (*)[4][ALINE]>(ldsA);
  uintx4 (*Bs16)[4][BLINE] = reinterpret_cast<uintx4 (*)[4][BLINE]>(ldsB);
  // per column j: {x offset c*HW + r*dh*W + s*dw, (r*dh) | (s*dw) << 16}; buffer path: {4 * offset, tap r*S + s}
  __shared__ int2 jtab[BN];

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  // The tiles of one reduction split read the same pixels of x and dy: with one group, splits are
  // dealt to the XCDs in contiguous runs so that those tiles share an L2 instead of each XCD
  // fetching every split's pixels.
  const int g = blockIdx.y;
  int tile = blockIdx.x, split = blockIdx.z;
  if (gridDim.y == 1) {
    const int v = tt::xcd_remap((int)(blockIdx.x + gridDim.x * blockIdx.z), (int)(gridDim.x * gridDim.z));
    split = v / (int)gridDim.x;
    tile = v - split * (int)gridDim.x;
  }
  const int i0 = (tile % p.tilesI) * BM;
  const int j0 = (tile / p.tilesI) * BN;

  if (tid < BN) {
    const int j = j0 + tid;
    int2 e = make_int2(0, WIDE ? 63 : BUF ? 31 : (-16384) & 0xffff);   // column beyond J: never valid
    if (j < p.J) {
      const uint32_t c = tt::fd_div((uint32_t)j, p.divRS);
      const uint32_t rs = (uint32_t)j - c * p.divRS.d;
      const uint32_t r = tt::fd_div(rs, p.divS);
      const uint32_t s = rs - r * p.divS.d;
      e.x = (int)c * p.HW + (int)r * p.dh * p.W + (int)s * p.dw;
      e.y = (((int)r * p.dh) & 0xffff) | (((int)s * p.dw) << 16);
      if (BUF) {
        e.x *= 4;
        e.y = (int)rs;
      }
    }
    jtab[tid] = e;
  }

  const int px = tid & 31, rg = tid >> 5;   // this thread's pixel inside a chunk, and row group
  const int qpx = tid & 7, rgq = tid >> 3;   // vector fetches: pixel quad inside a chunk, and row group
  const float* __restrict__ dyg = p.dy + (size_t)g * p.dyStrideG;
  const float* __restrict__ xg = p.x + (size_t)g * p.xStrideG;

  // staging registers of the chunk being fetched, and what its loads need
  // (bf16 arithmetic keeps two sets: the loads of the chunk after next are issued while the next
  // chunk's values still wait in the other set for their turn to be written to LDS)
  constexpr int SETS = BF ? 2 : 1;
  float areg[SETS][A_ROWS], breg[SETS][B_ROWS];
  int amask[SETS] = {};        // all ones if this thread's pixel is inside the reduction range
  uint32_t bok[SETS] = {};     // bit t: breg[set][t] is inside the image (applied when written to LDS)
  int2 jreg[B_ROWS];
  int ih0 = kInvalid, iw0 = 0, xbase = 0, dybase = 0, alim = 0;
  const int arow = i0 + rg;

  const int c_begin = split * p.chunksPerSplit;
  const int c_end = min(p.chunks, c_begin + p.chunksPerSplit);

  // buffer path: descriptors re-based to the chunk's first image, this lane's pixel offsets in
  // dy and x (bit 31 of the dy offset set for pixels past the end), its tap mask (bit t set: tap
  // t is outside the image), and the per-lane constants added per load
  __amdgpu_buffer_rsrc_t dySrd = __builtin_amdgcn_make_buffer_rsrc((void*)p.dy, 0, kSrdRecords, kSrdFlags);
  __amdgpu_buffer_rsrc_t xSrd = __builtin_amdgcn_make_buffer_rsrc((void*)p.x, 0, kSrdRecords, kSrdFlags);
  uint32_t dyvoff = 0x80000000u, xvoff = 0;
  TapBits nmask = ~(TapBits)0;
  int aoff[A_ROWS];
  if constexpr (BUF) {
#pragma unroll
    for (int t = 0; t < A_ROWS; ++t)   // rows past Kg are never stored
      aoff[t] = 4 * min(VA ? i0 + rgq + 32 * t : arow + 8 * t, p.Kg - 1) * p.PQ;
  }
  // vector fetches: offsets of the quad's first pixel, staging vectors, per-row x offsets
  uint32_t qvoff = 0x80000000u, qxvoff = 0x80000000u;
  floatx4 aregv[SETS][VA ? A_ROWS : 1], bregv[SETS][VB ? B_ROWS : 1];
  int boffv[VB ? B_ROWS : 1];
  if constexpr (VB) {
#pragma unroll
    for (int t = 0; t < B_ROWS; ++t) boffv[t] = 4 * min(j0 + rgq + 32 * t, p.J - 1) * p.HW;   // column j = channel
  }

  // table entry of this lane's pixel in the chunk after the one being decomposed: fetched one
  // chunk ahead so that its latency is covered
  int4 pixnext = make_int4(0, 0, 0, 0);
  int2 pixnextq = make_int2(0, 0);
  int pixnexthi = 0;
  auto fetch_pix = [&](int chunk) __attribute__((always_inline)) {
    if constexpr (BUF && !(VA && VB)) pixnext = p.pixtab[chunk * kBK + px];
    if constexpr (WIDE) pixnexthi = p.pixhi[chunk * kBK + px];
    if constexpr (VA || VB) pixnextq = *reinterpret_cast<const int2*>(&p.pixtab[chunk * kBK + 4 * qpx]);
  };
  auto decompose = [&](int chunk, int following, const int set = 0) __attribute__((always_inline)) {
    if constexpr (BUF) {
      const int4 e = pixnext;   // entry of `chunk`
      const int2 eq = pixnextq;
      const int ehi = pixnexthi;
      fetch_pix(following);
      const int n0 = __builtin_amdgcn_readfirstlane((VA && VB) ? eq.x : e.x);   // lane 0 holds the chunk's first pixel
      if constexpr (VA || VB) {
        qvoff = (uint32_t)(4 * (eq.x - n0) * p.dyStrideN) + (uint32_t)eq.y;   // bit 31 of eq.y: quad past the end
        qxvoff = (uint32_t)(4 * (eq.x - n0) * p.xStrideN) + (uint32_t)eq.y;   // 1x1: x is indexed like dy
      }
      dySrd = __builtin_amdgcn_make_buffer_rsrc((void*)(p.dy + ((size_t)n0 * p.dyStrideN + (size_t)g * p.dyStrideG)), 0,
                                                kSrdRecords, kSrdFlags);
      xSrd = __builtin_amdgcn_make_buffer_rsrc(
          (void*)(p.x + ((long long)n0 * p.xStrideN + (long long)g * p.xStrideG - p.xBias)), 0, kSrdRecords, kSrdFlags);
      dyvoff = (uint32_t)(4 * (e.x - n0) * p.dyStrideN) + (uint32_t)e.y;   // bit 31 of e.y survives: pixel past the end
      xvoff = (uint32_t)(4 * (e.x - n0) * p.xStrideN) + (uint32_t)e.z;
      if constexpr (WIDE) nmask = (TapBits)(((uint64_t)(uint32_t)ehi << 32) | (uint32_t)e.w);
      else nmask = (uint32_t)e.w;
      return;
    }
    const int m = chunk * kBK + px;
    const bool mok = m < p.M;
    const uint32_t mm = mok ? (uint32_t)m : 0u;
    const uint32_t n = tt::fd_div(mm, p.divPQ);
    const uint32_t pq = mm - n * p.divPQ.d;
    const uint32_t pp = tt::fd_div(pq, p.divQ);
    const uint32_t qq = pq - pp * p.divQ.d;
    ih0 = mok ? (int)pp * p.sh - p.ph : kInvalid;
    iw0 = (int)qq * p.sw - p.pw;
    xbase = (int)n * p.xStrideN + ((int)pp * p.sh - p.ph) * p.W + iw0;
    dybase = (int)n * p.dyStrideN + (int)pq + arow * p.PQ;
    amask[set] = mok ? -1 : 0;
    alim = mok ? p.Kg : 0;   // rows at or beyond it are not read (they are never stored either)
    bok[set] = 0;
  };
  auto load_step = [&](int li, const int set = 0) __attribute__((always_inline)) {
    if constexpr (BUF) {
      if (li < A_ROWS) {
        if constexpr (VA)
          aregv[set][li] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(dySrd, (int)(qvoff + (uint32_t)aoff[li]), 0, 0));
        else
          areg[set][li] = as_float(__builtin_amdgcn_raw_buffer_load_b32(dySrd, (int)(dyvoff + (uint32_t)aoff[li]), 0, 0));
      } else {
        const int t = li - A_ROWS;
        if constexpr (VB) {
          bregv[set][t] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(xSrd, (int)(qxvoff + (uint32_t)boffv[t]), 0, 0));
        } else {
          const int2 e = jreg[t];
          const uint32_t vo = ((uint32_t)(nmask >> e.y) << 31) | (xvoff + (uint32_t)e.x);
          breg[set][t] = as_float(__builtin_amdgcn_raw_buffer_load_b32(xSrd, (int)vo, 0, 0));
        }
      }
      return;
    }
    if (li < A_ROWS) {
      const int t = li;
      const bool ok = arow + 8 * t < alim;
      areg[set][t] = dyg[ok ? (uint32_t)(dybase + 8 * t * p.PQ) : 0u];
    } else {
      const int t = li - A_ROWS;
      const int2 e = jreg[t];
      const int ih = ih0 + (int)(short)(e.y & 0xffff);
      const int iw = iw0 + (e.y >> 16);
      const bool ok = (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
      breg[set][t] = xg[ok ? (uint32_t)(xbase + e.x) : 0u];
      bok[set] |= ok ? (1u << t) : 0u;
    }
  };
  // Rows beyond Kg / columns beyond J may hold anything (never stored); pixels beyond M and taps
  // outside the image must be exactly zero: AND with an all-ones / all-zeros word.
  auto store_step = [&](int buf, int li, const int set = 0) __attribute__((always_inline)) {
    if constexpr (BF) {
      // Round to bf16 and write pixel-major units.  Vector fetches hold four consecutive pixels of a
      // row: 8 bytes, half a unit.  Scalar fetches hold one pixel per lane: every even lane takes its
      // neighbour's value too and writes the pair.  (Masks of the compare path apply first.)
      if (li < A_ROWS) {
        if constexpr (VA) {
          const floatx4 v = aregv[set][li];
          *reinterpret_cast<uintx2*>(reinterpret_cast<char*>(&As16[buf][qpx >> 1][pos16(rgq + 32 * li)]) + 8 * (qpx & 1)) =
              uintx2{pack2(v[0], v[1]), pack2(v[2], v[3])};
        } else {
          const float v = BUF ? areg[set][li] : __int_as_float(__float_as_int(areg[set][li]) & amask[set]);
          const unsigned pair = pack2(v, next_lane(v));
          if ((px & 1) == 0)
            *reinterpret_cast<unsigned*>(reinterpret_cast<char*>(&As16[buf][px >> 3][pos16(rg + 8 * li)]) + 2 * (px & 7)) = pair;
        }
      } else {
        const int t = li - A_ROWS;
        if constexpr (VB) {
          const floatx4 v = bregv[set][t];
          *reinterpret_cast<uintx2*>(reinterpret_cast<char*>(&Bs16[buf][qpx >> 1][pos16(rgq + 32 * t)]) + 8 * (qpx & 1)) =
              uintx2{pack2(v[0], v[1]), pack2(v[2], v[3])};
        } else {
          const int bmask = ((int)(bok[set] << (31 - t))) >> 31;
          const float v = BUF ? breg[set][t] : __int_as_float(__float_as_int(breg[set][t]) & bmask);
          const unsigned pair = pack2(v, next_lane(v));
          if ((px & 1) == 0)
            *reinterpret_cast<unsigned*>(reinterpret_cast<char*>(&Bs16[buf][px >> 3][pos16(rg + 8 * t)]) + 2 * (px & 7)) = pair;
        }
      }
      return;
    }
    if constexpr (BUF) {   // padding and pixels past the end were read as zeros
      if (li < A_ROWS) {
        if constexpr (VA) *reinterpret_cast<floatx4*>(&As[buf][rgq + 32 * li][4 * qpx]) = aregv[set][li];
        else As[buf][rg + 8 * li][px] = areg[set][li];
      } else {
        const int t = li - A_ROWS;
        if constexpr (VB) *reinterpret_cast<floatx4*>(&Bs[buf][rgq + 32 * t][4 * qpx]) = bregv[set][t];
        else Bs[buf][rg + 8 * t][px] = breg[set][t];
      }
      return;
    }
    if (li < A_ROWS) {
      As[buf][rg + 8 * li][px] = __int_as_float(__float_as_int(areg[set][li]) & amask[set]);
    } else {
      const int t = li - A_ROWS;
      const int bmask = ((int)(bok[set] << (31 - t))) >> 31;
      Bs[buf][rg + 8 * t][px] = __int_as_float(__float_as_int(breg[set][t]) & bmask);
    }
  };

  floatx16 acc[MT][NT];
#pragma unroll
  for (int a = 0; a < MT; ++a)
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // MFMA operands of one eighth-of-a-chunk (8 pixels): two register sets, the next one is read
  // from LDS while the current one is consumed
  floatx4 opA[2][MT], opB[2][NT];
  auto read_ops = [&](int set, int buf, int kk) __attribute__((always_inline)) {
#pragma unroll
    for (int xx = 0; xx < MT; ++xx)
      opA[set][xx] = *reinterpret_cast<const floatx4*>(&As[buf][(wm * MT + xx) * 32 + l32][kk * 8 + 4 * h]);
#pragma unroll
    for (int yy = 0; yy < NT; ++yy)
      opB[set][yy] = *reinterpret_cast<const floatx4*>(&Bs[buf][(wn * NT + yy) * 32 + l32][kk * 8 + 4 * h]);
  };

  // One chunk (32 pixels of the reduction) of MFMAs out of LDS buffer `buf`, with the next
  // chunk's work woven in between them, one small step per MFMA, so that it runs in the shadow
  // of the 64-cycle matrix instructions: pixel decomposition and global loads in the first half,
  // masked LDS writes into the other buffer from 5/8 on, then the one barrier and the first
  // operand fetch of the next chunk.  sched_barrier pins the order.
  constexpr int T = 16 * MT * NT;            // MFMAs per chunk
  constexpr int PK = 4 * MT * NT;            // MFMAs per 8-pixel operand set
  constexpr int L = A_ROWS + B_ROWS;         // loads (and LDS writes) per thread per chunk
  constexpr int LPS = (L + T / 2 - 2) / (T / 2 - 1);       // loads per slot, slots 1 .. T/2-1
  constexpr int kStore = 5 * T / 8, kSync = T - 4;
  constexpr int SPS = (L + (kSync - kStore) - 1) / (kSync - kStore);   // LDS writes per slot
  auto chunk_body = [&](const int buf, const int nchunk, const int nnchunk) __attribute__((always_inline)) {
    if constexpr (BF) {
      // Two bf16 MFMAs per accumulator contract the chunk's 32 pixels: step t takes pixel blocks 2t
      // (lanes 0-31) and 2t + 1 (lanes 32-63), a lane's 16 bytes being its eight pixels, the same
      // eight for both operands.  A sixteenth of the fp32 matrix time: nothing to weave the loads
      // into and too short to cover their latency, so this chunk issues the loads of the chunk AFTER
      // NEXT (`nchunk`) into staging set `buf`.
      decompose(nchunk, nnchunk, buf);
#pragma unroll
      for (int li = 0; li < L; ++li) load_step(li, buf);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        bf16x8 a[MT], b[NT];
#pragma unroll
        for (int xx = 0; xx < MT; ++xx)
          a[xx] = __builtin_bit_cast(bf16x8, As16[buf][2 * t + h][pos16((wm * MT + xx) * 32 + l32)]);
#pragma unroll
        for (int yy = 0; yy < NT; ++yy)
          b[yy] = __builtin_bit_cast(bf16x8, Bs16[buf][2 * t + h][pos16((wn * NT + yy) * 32 + l32)]);
#pragma unroll
        for (int xx = 0; xx < MT; ++xx)
#pragma unroll
          for (int yy = 0; yy < NT; ++yy)
            acc[xx][yy] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[xx], b[yy], acc[xx][yy], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      // the chunk after this one was fetched during the previous chunk: it has had a whole chunk's
      // time to arrive and goes to the other LDS buffer now
#pragma unroll
      for (int li = 0; li < L; ++li) store_step(buf ^ 1, li, buf ^ 1);
      __syncthreads();
      return;
    }
#pragma unroll
    for (int s = 0; s < T; ++s) {
      const int kk = s / PK, rem = s % PK;
      const int j = rem / (MT * NT), xx = (rem % (MT * NT)) / NT, yy = rem % NT;
      acc[xx][yy] = __builtin_amdgcn_mfma_f32_32x32x2f32(opA[kk & 1][xx][j], opB[kk & 1][yy][j], acc[xx][yy], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (rem == 0 && kk < 3) read_ops((kk + 1) & 1, buf, kk + 1);
      if (s == 0) decompose(nchunk, nnchunk);
#pragma unroll
      for (int u = 0; u < LPS; ++u) {
        const int li = (s - 1) * LPS + u;
        if (s >= 1 && li < L) load_step(li);
      }
#pragma unroll
      for (int u = 0; u < SPS; ++u) {
        const int li = (s - kStore) * SPS + u;
        if (s >= kStore && s < kSync && li < L) store_step(buf ^ 1, li);
      }
      if (s == kSync) {
        __syncthreads();
        read_ops(0, buf ^ 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  __syncthreads();   // jtab
  if constexpr (!VB) {
#pragma unroll
    for (int t = 0; t < B_ROWS; ++t) jreg[t] = jtab[rg + 8 * t];
  }

  if (c_begin < c_end) {
    const int last = c_end - 1;
    fetch_pix(c_begin);
    decompose(c_begin, min(c_begin + 1, last));
#pragma unroll
    for (int li = 0; li < L; ++li) load_step(li);
#pragma unroll
    for (int li = 0; li < L; ++li) store_step(0, li);
    // past the end the last chunk is fetched again (cache hits) instead of branching
    int c = c_begin;
    if constexpr (BF) {
      // two chunks ahead: the second chunk waits in staging set 1 while the loop starts
      decompose(min(c_begin + 1, last), min(c_begin + 2, last), 1);
#pragma unroll
      for (int li = 0; li < L; ++li) load_step(li, 1);
      __syncthreads();
      for (; c + 1 < c_end; c += 2) {
        chunk_body(0, min(c + 2, last), min(c + 3, last));
        chunk_body(1, min(c + 3, last), min(c + 4, last));
      }
      if (c < c_end) chunk_body(0, last, last);
    } else {
      __syncthreads();
      read_ops(0, 0, 0);
      for (; c + 1 < c_end; c += 2) {
        chunk_body(0, c + 1, min(c + 2, last));
        chunk_body(1, min(c + 2, last), min(c + 3, last));
      }
      if (c < c_end) chunk_body(0, last, last);
    }
  }

  if (p.fuse) {
    // ---- partial sums added inside the kernel --------------------------------------------------
    // Publish: the accumulators as they lie in registers, one coalesced 16-byte store per lane and
    // quad, written through to memory; every wave waits for its stores, then one thread raises the
    // block's flag to this launch's epoch.
    constexpr int F4 = MT * NT * 4 * kThreads;   // float4s of one tile
    const int S = (int)gridDim.z;
    const int tl = g * (int)gridDim.x + tile;
    const __amdgpu_buffer_rsrc_t part =
        __builtin_amdgcn_make_buffer_rsrc((void*)(p.fusePartial + (size_t)tl * S * F4), 0, kSrdRecords, kSrdFlags);
#pragma unroll
    for (int xx = 0; xx < MT; ++xx)
#pragma unroll
      for (int yy = 0; yy < NT; ++yy)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          store_coherent(part, 16 * (split * F4 + ((xx * NT + yy) * 4 + q) * kThreads + tid),
                         floatx4{acc[xx][yy][4 * q], acc[xx][yy][4 * q + 1], acc[xx][yy][4 * q + 2], acc[xx][yy][4 * q + 3]});
    __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
    __syncthreads();
    unsigned* flags = p.fuseFlags + (size_t)tl * S;
    if (tid == 0) __hip_atomic_store(&flags[split], p.fuseEpoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    // Wait for every split of this tile (all blocks of the grid are resident and publish as soon as
    // their reduction range is done, so nobody waits on somebody who waits).  Bounded all the same:
    // a wait that runs out raises the error word that the host reports at its next synchronisation.
    for (int j = tid; j < S; j += kThreads) {
      int spins = 0;
      while (__hip_atomic_load(&flags[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != p.fuseEpoch) {
        if (++spins >= kFuseSpinLimit) {
          __hip_atomic_store(p.fuseError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          break;
        }
        __builtin_amdgcn_s_sleep(4);
      }
    }
    __syncthreads();
    // Add: this block owns float4s [split * nf, (split + 1) * nf) of the tile, nf = ceil(F4 / S).
    // Thread (kl, fi) adds splits kl, kl + KL, ... of float4 fi in float64; the KL sums of a float4
    // are then added in kl order.  The order is fixed by the geometry alone: results are
    // bit-reproducible.
    const int nf = (F4 + S - 1) / S;
    const int lo = split * nf, hi = min(F4, lo + nf);
    const int KL = p.fuseKL, NF = p.fuseNf;
    const int fi = tid % NF, kl = tid / NF;
    double* comb = reinterpret_cast<double*>(lds);   // [KL][NF][4] (8 KiB); the tiles are no longer read
    float* __restrict__ dwg = p.out + (size_t)g * p.Kg * p.J;
    for (int base = lo; base < hi; base += NF) {
      const int f = base + fi;
      double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
      if (f < hi) {
#pragma unroll 4
        for (int k = kl; k < S; k += KL) {
          const floatx4 v = load_coherent(part, 16 * (k * F4 + f));
          s0 += (double)v[0]; s1 += (double)v[1]; s2 += (double)v[2]; s3 += (double)v[3];
        }
      }
      if (kl > 0) {
        double* c = comb + ((size_t)kl * NF + fi) * 4;
        c[0] = s0; c[1] = s1; c[2] = s2; c[3] = s3;
      }
      __syncthreads();
      if (kl == 0 && f < hi) {
        for (int l = 1; l < KL; ++l) {
          const double* c = comb + ((size_t)l * NF + fi) * 4;
          s0 += c[0]; s1 += c[1]; s2 += c[2]; s3 += c[3];
        }
        // float4 f of the tile = accumulator quad (xx, yy, q) of thread t: rows 8q + 4h .. +3, one column
        const int t = f % kThreads, idx = f / kThreads;
        const int q = idx & 3, yy = (idx >> 2) % NT, xx = (idx >> 2) / NT;
        const int tw = t >> 6, tl32 = t & 31, th = (t >> 5) & 1;
        const int i = i0 + ((tw / WN) * MT + xx) * 32 + 8 * q + 4 * th;
        const int j = j0 + ((tw % WN) * NT + yy) * 32 + tl32;
        if (j < p.J) {
          if (i < p.Kg) dwg[(size_t)i * p.J + j] = (float)s0;
          if (i + 1 < p.Kg) dwg[(size_t)(i + 1) * p.J + j] = (float)s1;
          if (i + 2 < p.Kg) dwg[(size_t)(i + 2) * p.J + j] = (float)s2;
          if (i + 3 < p.Kg) dwg[(size_t)(i + 3) * p.J + j] = (float)s3;
        }
      }
      __syncthreads();
    }
    return;
  }

  float* __restrict__ out = p.out + (size_t)split * p.outStrideSplit + (size_t)g * p.Kg * p.J;
#pragma unroll
  for (int yy = 0; yy < NT; ++yy) {
    const int j = j0 + (wn * NT + yy) * 32 + l32;
    if (j >= p.J) continue;
#pragma unroll
    for (int xx = 0; xx < MT; ++xx)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = i0 + (wm * MT + xx) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
        if (i < p.Kg) out[(size_t)i * p.J + j] = acc[xx][yy][r];
      }
  }
}

template <int WM, int WN, int MT, int NT, bool BUF, bool VA, bool VB>
__global__ __launch_bounds__(kThreads, 2) __attribute__((amdgpu_waves_per_eu(2, 2))) void wgrad_f32(const Wgrad p) {
  wgrad_body<WM, WN, MT, NT, BUF, VA, VB, false>(p);
}
template <int WM, int WN, int MT, int NT, bool BUF, bool VA, bool VB>
__global__ __launch_bounds__(kThreads, 2) __attribute__((amdgpu_waves_per_eu(2, 2))) void wgrad_bf16(const Wgrad p) {
  wgrad_body<WM, WN, MT, NT, BUF, VA, VB, true>(p);
}
// kernels of 32 .. 63 taps: buffer path with 64-bit tap masks
template <int WM, int WN, int MT, int NT, bool VA>
__global__ __launch_bounds__(kThreads, 2) __attribute__((amdgpu_waves_per_eu(2, 2))) void wgrad_wide_f32(const Wgrad p) {
  wgrad_body<WM, WN, MT, NT, true, VA, false, false, true>(p);
}
template <int WM, int WN, int MT, int NT, bool VA>
__global__ __launch_bounds__(kThreads, 2) __attribute__((amdgpu_waves_per_eu(2, 2))) void wgrad_wide_bf16(const Wgrad p) {
  wgrad_body<WM, WN, MT, NT, true, VA, false, true, true>(p);
}

// dw[e] = sum over splits of partial[s][e] in float64.  A block covers 64 float4 columns with
// 4 lanes per column; lane l adds splits l, l+4, ... in order, the four lane sums are added in
// lane order: the summation order is fixed, so the result is deterministic.
__global__ __launch_bounds__(kThreads) void wgrad_reduce(const float* __restrict__ partial, float* __restrict__ dw,
                                                         size_t elems, int splits) {
  __shared__ double lds[3][64][4];
  const int col = threadIdx.x & 63, lane = threadIdx.x >> 6;
  const size_t e = ((size_t)blockIdx.x * 64 + col) * 4;
  double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
  const bool vec = (elems & 3) == 0;   // partial rows stay 16-byte aligned
  if (vec && e < elems) {
#pragma unroll 2
    for (int k = lane; k < splits; k += 4) {
      const floatx4 v = *reinterpret_cast<const floatx4*>(partial + (size_t)k * elems + e);
      s0 += (double)v[0]; s1 += (double)v[1]; s2 += (double)v[2]; s3 += (double)v[3];
    }
  } else if (e < elems) {
    for (int k = lane; k < splits; k += 4) {
      const float* q = partial + (size_t)k * elems + e;
      s0 += (double)q[0];
      if (e + 1 < elems) s1 += (double)q[1];
      if (e + 2 < elems) s2 += (double)q[2];
      if (e + 3 < elems) s3 += (double)q[3];
    }
  }
  if (lane > 0) {
    lds[lane - 1][col][0] = s0; lds[lane - 1][col][1] = s1; lds[lane - 1][col][2] = s2; lds[lane - 1][col][3] = s3;
  }
  __syncthreads();
  if (lane == 0 && e < elems) {
#pragma unroll
    for (int l = 0; l < 3; ++l) {
      s0 += lds[l][col][0]; s1 += lds[l][col][1]; s2 += lds[l][col][2]; s3 += lds[l][col][3];
    }
    if (vec) {
      *reinterpret_cast<floatx4*>(dw + e) = floatx4{(float)s0, (float)s1, (float)s2, (float)s3};
    } else {
      dw[e] = (float)s0;
      if (e + 1 < elems) dw[e + 1] = (float)s1;
      if (e + 2 < elems) dw[e + 2] = (float)s2;
      if (e + 3 < elems) dw[e + 3] = (float)s3;
    }
  }
}

int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

// ---- pixel table -------------------------------------------------------------------------------------
// What the main loop would otherwise recompute for every chunk in every block (two divisions, the
// tap ranges) depends only on the geometry: per output pixel m = (n, p, q)
//   {image n, byte offset 4*(p*Q + q) of the pixel in a dy plane,
//    byte offset 4*(ih*W + iw + xBias) of the window's first tap in an x plane, tap mask}
// (bit t of the mask set: tap t = r*S + s lies outside the image for this pixel; kernels of
// 32 .. 63 taps keep bits 32 .. 63 in a second array).  Entries from M to chunks*32 hold
// {N-1, bit 31, 0, all ones}: a pixel past the end reads zeros everywhere.
// The table is built on the host, checked there against the two tensors it indexes, uploaded once
// into a device buffer of its own and kept per geometry: no kernel writes it.
struct PixGeom {
  int N, C, K, groups, P, Q, H, W, R, S, sh, sw, ph, pw, dh, dw, chunks;
};
struct HostPixTab {
  std::vector<int4> tab;
  std::vector<int> hi;   // empty unless the kernel has 32 .. 63 taps
};

// Floor and ceiling of a / b for b > 0 and any a.
long long floor_div(long long a, long long b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }
long long ceil_div_s(long long a, long long b) { return -floor_div(-a, b); }

// Taps t = 0 .. n-1 at pos + t*step: bits [lo*unit, (hi+1)*unit) for the range [lo, hi] of taps that
// fall inside [0, lim) (closed form, as the lanes used to compute it).
uint64_t tap_range_bits_host(int pos, int lim, int n, int unit, int step) {
  long long lo = std::max<long long>(0, ceil_div_s(-(long long)pos, step));
  long long hi = std::min<long long>(n - 1, floor_div((long long)lim - 1 - pos, step));
  if (lo > hi) return 0;
  const uint64_t upto = (hi + 1) * unit >= 64 ? ~0ull : (1ull << ((hi + 1) * unit)) - 1ull;
  const uint64_t below = (1ull << (lo * unit)) - 1ull;
  return upto & ~below;
}

void build_pixtab(const PixGeom& g, bool wide, HostPixTab* out) {
  const int PQ = g.P * g.Q, M = g.N * PQ, entries = g.chunks * kBK;
  const int xBias = g.ph * g.W + g.pw;
  out->tab.assign((size_t)entries, make_int4(g.N - 1, (int)0x80000000u, 0, -1));
  out->hi.assign(wide ? (size_t)entries : 0, -1);
  uint64_t row_ones = 0;
  for (int r = 0; r < g.R; ++r) row_ones |= 1ull << (r * g.S);
  // the part that depends on (p, q) only, once; then one entry per image
  std::vector<int4> plane((size_t)PQ);
  std::vector<int> plane_hi(wide ? (size_t)PQ : 0);
  for (int pq = 0; pq < PQ; ++pq) {
    const int pp = pq / g.Q, qq = pq % g.Q;
    const int ih = pp * g.sh - g.ph, iw = qq * g.sw - g.pw;
    // valid tap columns, replicated into every valid tap row (fields of S bits: no carries)
    const uint64_t cols = tap_range_bits_host(iw, g.W, g.S, 1, g.dw);
    const uint64_t rows = tap_range_bits_host(ih, g.H, g.R, g.S, g.dh) & row_ones;
    const uint64_t outside = ~(cols * rows);   // the top bit stays set: R*S <= 31 (63)
    plane[(size_t)pq] = make_int4(0, 4 * pq, 4 * (ih * g.W + iw + xBias), (int)(uint32_t)outside);
    if (wide) plane_hi[(size_t)pq] = (int)(uint32_t)(outside >> 32);
  }
  for (int m = 0; m < M; ++m) {
    int4 e = plane[(size_t)(m % PQ)];
    e.x = m / PQ;
    out->tab[(size_t)m] = e;
    if (wide) out->hi[(size_t)m] = plane_hi[(size_t)(m % PQ)];
  }
}

// What the kernel will do with every entry, replayed on the host: the dy element a lane fetches for
// the entry's pixel must be pixel (n, p, q) of the row's plane and lie inside dy; for every tap the
// mask lets through, the x element must be (n, c, p*sh - ph + r*dh, q*sw - pw + s*dw), inside its
// image -- and every tap the mask blocks must really fall outside, or a product would be lost
// silently; 32-bit byte offsets relative to the first image of a chunk (at most 33 images back)
// must stay in [0, 2^31); entries past the end must read zeros.
int check_pixtab(const char* fn, const PixGeom& g, bool wide, const HostPixTab& t) {
  const int PQ = g.P * g.Q, M = g.N * PQ, entries = g.chunks * kBK;
  const int taps = g.R * g.S, top = wide ? 63 : 31;
  const int Cg = g.C / g.groups, Kg = g.K / g.groups;
  const long long xImg = (long long)g.C * g.H * g.W, dyImg = (long long)g.K * PQ;
  const long long xBias = (long long)g.ph * g.W + g.pw;
  TT_REQUIRE((int)t.tab.size() == entries && (wide ? (int)t.hi.size() == entries : t.hi.empty()) && entries >= M &&
                 taps <= top,
             "%s: pixel table of %zu entries for %d pixels in %d chunks, %d taps", fn, t.tab.size(), M, g.chunks, taps);
  auto mask_of = [&](int m) {
    return wide ? ((uint64_t)(uint32_t)t.hi[(size_t)m] << 32) | (uint32_t)t.tab[(size_t)m].w
                : (uint64_t)(uint32_t)t.tab[(size_t)m].w;
  };
  // the (p, q)-dependent fields, pixel by pixel of the first image
  for (int pq = 0; pq < std::min(PQ, M); ++pq) {
    const int4 e = t.tab[(size_t)pq];
    const int pp = pq / g.Q, qq = pq % g.Q;
    TT_REQUIRE(e.y == 4 * pq, "%s: pixel table entry %d: dy byte offset %d for pixel (%d, %d)", fn, pq, e.y, pp, qq);
    const uint64_t outside = mask_of(pq);
    TT_REQUIRE((outside >> top) & 1, "%s: pixel table entry %d: the padding tap %d is not blocked", fn, pq, top);
    const long long first = e.z / 4 - xBias;   // element offset of tap (0, 0) in an x plane; may be negative (padding)
    TT_REQUIRE(e.z % 4 == 0 && e.z >= 0, "%s: pixel table entry %d: x byte offset %d", fn, pq, e.z);
    for (int r = 0; r < g.R; ++r)
      for (int s2 = 0; s2 < g.S; ++s2) {
        const int ih = pp * g.sh - g.ph + r * g.dh, iw = qq * g.sw - g.pw + s2 * g.dw;
        const bool inside = ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
        const bool blocked = (outside >> (r * g.S + s2)) & 1;
        TT_REQUIRE(inside != blocked, "%s: pixel table entry %d: tap (%d, %d) at (%d, %d) of a %d x %d image is %s", fn,
                   pq, r, s2, ih, iw, g.H, g.W, blocked ? "blocked" : "let through");
        if (!inside) continue;
        // per column j = (c, r, s) the kernel adds c*H*W + r*dh*W + s*dw elements (jtab)
        const long long at = first + (long long)r * g.dh * g.W + (long long)s2 * g.dw;
        TT_REQUIRE(at == (long long)ih * g.W + iw && at + (long long)(Cg - 1) * g.H * g.W < (long long)Cg * g.H * g.W,
                   "%s: pixel table entry %d: tap (%d, %d) reaches element %lld of its plane (expected %lld)", fn, pq, r, s2,
                   at, (long long)ih * g.W + iw);
      }
  }
  // per entry: image, sameness with the first image's fields, reach inside both tensors, 31-bit offsets
  for (int m = 0; m < entries; ++m) {
    const int4 e = t.tab[(size_t)m];
    if (m >= M) {
      TT_REQUIRE(e.x == g.N - 1 && e.y < 0 && mask_of(m) == (wide ? ~0ull : 0xffffffffull),
                 "%s: pixel table entry %d (past the last pixel) does not read zeros", fn, m);
      continue;
    }
    const int n = m / PQ, pq = m % PQ;
    const int4 e0 = t.tab[(size_t)pq];
    TT_REQUIRE(e.x == n && e.y == e0.y && e.z == e0.z && mask_of(m) == mask_of(pq), "%s: pixel table entry %d: image %d, fields differ from pixel %d of image 0", fn, m, e.x, pq);
    // the chunk's first pixel decides the base image n0 of the descriptors
    const int n0 = ((m / kBK) * kBK) / PQ;
    const long long dy_lane = 4LL * (n - n0) * dyImg + e.y + 4LL * (Kg - 1) * PQ;            // last row of a group
    const long long x_lane = 4LL * (n - n0) * xImg + e.z + 4LL * ((long long)(Cg - 1) * g.H * g.W + (long long)(g.R - 1) * g.dh * g.W + (long long)(g.S - 1) * g.dw);
    TT_REQUIRE(n >= n0 && dy_lane < (1LL << 31) && x_lane < (1LL << 31),
               "%s: pixel table entry %d: byte offsets %lld / %lld leave the buffer range", fn, m, dy_lane, x_lane);
    const long long dy_at = (long long)n * dyImg + (long long)(g.groups - 1) * Kg * PQ + (long long)(Kg - 1) * PQ + pq;
    TT_REQUIRE(dy_at < (long long)g.N * dyImg, "%s: pixel table entry %d reaches element %lld of dy (%lld)", fn, m, dy_at,
               (long long)g.N * dyImg);
  }
  return 0;
}

// Set only inside tt_conv2d_check_tables_selftest_wgrad (host-only): damages one field of one
// entry of the next table built, to show that check_pixtab refuses it.
int g_pix_fault_entry = -1, g_pix_fault_field = 0, g_pix_fault_delta = 0;

struct PixKey {
  int v[17];
  bool operator<(const PixKey& o) const {
    for (int i = 0; i < 17; ++i)
      if (v[i] != o.v[i]) return v[i] < o.v[i];
    return false;
  }
};
// At most kMaxPixTables geometries (16 bytes per output pixel, 20 with a 64-bit mask), then all are dropped.
constexpr size_t kMaxPixTables = 256;
struct PixTables {
  int4* tab = nullptr;
  int* hi = nullptr;   // null unless the kernel has 32 .. 63 taps
  HostPixTab host;     // stays alive while the upload may still be reading it
};
std::map<PixKey, PixTables>& pixtab_cache() {
  static std::map<PixKey, PixTables> cache;
  return cache;
}
int drop_pixtabs() {
  auto& cache = pixtab_cache();
  for (auto& kv : cache) {
    TT_HIP(hipFree(kv.second.tab));
    if (kv.second.hi) TT_HIP(hipFree(kv.second.hi));
  }
  cache.clear();
  return 0;
}
// Builds and checks the table of geometry `g`; unless `host_only`, returns the device copy kept for it.
int cached_pixtab(const char* fn, const PixGeom& g, bool wide, bool host_only, const int4** out, const int** out_hi) {
  auto& cache = pixtab_cache();
  const PixKey key{{g.N, g.C, g.K, g.groups, g.P, g.Q, g.H, g.W, g.R, g.S, g.sh, g.sw, g.ph, g.pw, g.dh, g.dw, g.chunks}};
  auto it = host_only ? cache.end() : cache.find(key);
  if (it == cache.end()) {
    PixTables t;
    build_pixtab(g, wide, &t.host);
    if (g_pix_fault_entry >= 0 && g_pix_fault_entry < (int)t.host.tab.size()) {   // self-test only
      int4& e = t.host.tab[(size_t)g_pix_fault_entry];
      (g_pix_fault_field == 0 ? e.x : g_pix_fault_field == 1 ? e.y : g_pix_fault_field == 2 ? e.z : e.w) ^= g_pix_fault_delta;
    }
    if (check_pixtab(fn, g, wide, t.host)) return -1;
    if (host_only) return 0;
    hipStream_t st = tt::stream();
    if (cache.size() >= kMaxPixTables) {
      TT_HIP(hipStreamSynchronize(st));
      if (drop_pixtabs()) return -1;
    }
    const size_t entries = t.host.tab.size();
    TT_HIP(hipMalloc((void**)&t.tab, sizeof(int4) * entries));
    if (wide) {
      if (hipError_t e = hipMalloc((void**)&t.hi, sizeof(int) * entries); e != hipSuccess) {
        (void)hipFree(t.tab);
        return tt::fail_hip(e, "hipMalloc", __FILE__, __LINE__);
      }
    }
    it = cache.emplace(key, std::move(t)).first;   // the vectors' storage moves with it
    PixTables& kept = it->second;
    hipError_t e = hipMemcpyAsync(kept.tab, kept.host.tab.data(), sizeof(int4) * entries, hipMemcpyHostToDevice, st);
    if (e == hipSuccess && wide)
      e = hipMemcpyAsync(kept.hi, kept.host.hi.data(), sizeof(int) * entries, hipMemcpyHostToDevice, st);
    if (e != hipSuccess) {
      (void)hipStreamSynchronize(st);
      (void)hipFree(kept.tab);
      if (kept.hi) (void)hipFree(kept.hi);
      cache.erase(it);
      return tt::fail_hip(e, "hipMemcpyAsync(pixel table)", __FILE__, __LINE__);
    }
  }
  *out = it->second.tab;
  *out_hi = it->second.hi;
  return 0;
}

typedef void (*WgradKernel)(const Wgrad);
template <int WM, int WN, int MT, int NT>
WgradKernel pick_wgrad(bool buf, bool va, bool vb, bool wide) {
  if (wide) {   // implies buf and not vb
    const bool bf = tt::conv_math() == TT_CONV_MATH_BF16;
    if (bf && va) return wgrad_wide_bf16<WM, WN, MT, NT, true>;
    if (bf) return wgrad_wide_bf16<WM, WN, MT, NT, false>;
    if (va) return wgrad_wide_f32<WM, WN, MT, NT, true>;
    return wgrad_wide_f32<WM, WN, MT, NT, false>;
  }
  if (tt::conv_math() == TT_CONV_MATH_BF16) {
    if (buf && va && vb) return wgrad_bf16<WM, WN, MT, NT, true, true, true>;
    if (buf && va) return wgrad_bf16<WM, WN, MT, NT, true, true, false>;
    if (buf) return wgrad_bf16<WM, WN, MT, NT, true, false, false>;
    return wgrad_bf16<WM, WN, MT, NT, false, false, false>;
  }
  if (buf && va && vb) return wgrad_f32<WM, WN, MT, NT, true, true, true>;
  if (buf && va) return wgrad_f32<WM, WN, MT, NT, true, true, false>;
  if (buf) return wgrad_f32<WM, WN, MT, NT, true, false, false>;
  return wgrad_f32<WM, WN, MT, NT, false, false, false>;
}

// Blocks of `kernel` that the device holds at once (asked once per kernel: registers and LDS of the
// compiled code decide it).  The in-kernel adding of the partial sums is used only for grids that
// fit: all blocks of a tile wait for each other.
int g_wgrad_forced_occupancy = -1;   // >= 0: pretend this many blocks per compute unit (tests of the fallback)
long long resident_blocks(WgradKernel kernel) {
  static std::map<WgradKernel, int> cache;
  auto it = cache.find(kernel);
  if (it == cache.end()) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, kThreads, 0) != hipSuccess) {
      (void)hipGetLastError();
      n = 0;
    }
    it = cache.emplace(kernel, n).first;
  }
  const int per_cu = g_wgrad_forced_occupancy >= 0 ? g_wgrad_forced_occupancy : it->second;
  return (long long)per_cu * tt::compute_units();
}

unsigned g_fuse_epoch = 0;
unsigned* g_fuse_flags = nullptr;
int fuse_flags(unsigned** out) {
  if (g_fuse_flags == nullptr) {
    const size_t bytes = sizeof(unsigned) * kFuseFlagWords;
    TT_HIP(hipMalloc((void**)&g_fuse_flags, bytes));
    TT_HIP(hipMemsetAsync(g_fuse_flags, 0, bytes, tt::stream()));
  }
  *out = g_fuse_flags;
  return 0;
}
int g_last_wgrad[4] = {};   // instrumentation: {tiles * groups, splits, partial sums added in the kernel, slots}

}  // namespace

namespace tt {
int wgrad_release_tables() {   // the caller has synchronised the stream
  return drop_pixtabs();
}
}  // namespace tt

extern "C" {

// `size_only`: report the workspace bytes this call would ask the library for and do nothing else.
// `check_only`: build and check the pixel tables the call would use, on the host alone (no device
// is touched, tensor pointers are not looked at).
static int conv2d_wgrad(const float* x, const float* dy, float* dw, int N, int C, int H, int W, int K, int R, int S,
                        int sh, int sw, int ph, int pw, int dh, int dw_, int groups, int P, int Q, size_t* size_only,
                        bool check_only = false) {
  TT_API_LOCK();
  const char* fn = "tt_conv2d_wgrad_f32";
  if (!check_only) {
    TT_REQUIRE(tt::initialised(), "tt_init() has not been called");
    TT_REQUIRE(x && dy && dw, "%s: null tensor pointer", fn);
    TT_REQUIRE_ALIGNED(fn, dw);
  }
  TT_REQUIRE(N > 0 && C > 0 && H > 0 && W > 0 && K > 0 && R > 0 && S > 0 && P > 0 && Q > 0, "%s: sizes must be positive", fn);
  TT_REQUIRE(sh > 0 && sw > 0 && dh > 0 && dw_ > 0 && ph >= 0 && pw >= 0, "%s: stride/dilation must be positive, padding non-negative", fn);
  TT_REQUIRE(groups > 0 && groups <= 65535 && C % groups == 0 && K % groups == 0, "%s: channels (%d, %d) not divisible by groups=%d", fn, C, K, groups);
  TT_REQUIRE(H + 2 * ph + R * dh < 16384 && W + 2 * pw + S * dw_ < 16384, "%s: spatial extents must stay below 16384", fn);
  // dy is [N, K, P, Q]: P x Q windows must exist in the padded input.  Fewer than the geometry allows
  // is legitimate (a transposed convolution with output_padding hands over a cropped problem, as the
  // reference crops x~ to the rows the windows cover, grad_nn.py:653-655); more is a caller's mix-up
  // of the roles of x and dy, which would read dy with a wrong pitch and return a plausible dw.
  {
    const long long span_h = (long long)H + 2 * ph - (long long)dh * (R - 1) - 1, span_w = (long long)W + 2 * pw - (long long)dw_ * (S - 1) - 1;
    TT_REQUIRE(span_h >= 0 && span_w >= 0, "%s: kernel (%d x %d, dilation %d x %d) larger than padded input (%d x %d)", fn, R,
               S, dh, dw_, H + 2 * ph, W + 2 * pw);
    TT_REQUIRE(P <= span_h / sh + 1 && Q <= span_w / sw + 1,
               "%s: dy of %d x %d does not belong to this geometry (input %d x %d, kernel %d x %d, stride %d x %d, padding "
               "%d x %d, dilation %d x %d give at most %lld x %lld)",
               fn, P, Q, H, W, R, S, sh, sw, ph, pw, dh, dw_, span_h / sh + 1, span_w / sw + 1);
  }
  // The kernels index with 32-bit element offsets.  A batch whose tensors have 2^31 elements or
  // more is cut into runs of images that stay below that; every run writes its own partial sums
  // and the reduce kernel adds the partials of all runs, still in a fixed order.
  const long long image = std::max((long long)C * H * W, (long long)K * P * Q);
  TT_REQUIRE(tt::fits_i32(image) && tt::fits_i32((long long)K * (C / groups) * R * S),
             "%s: one image or the weights exceed 2^31-1 elements", fn);
  int per_run = (int)std::min<long long>(N, std::max<long long>(1, 2147483646LL / image));
  if (per_run < N && per_run >= 4) per_run -= per_run % 4;   // later runs start 16-byte aligned: vector fetches stay on
  const int Cg = C / groups, Kg = K / groups;
  const int J = Cg * R * S;

  int bm = 128, bn = 128;
  if (Kg <= 64) bm = 64;
  if (J <= 64) bn = 64;
  // 64 columns where 128 would be badly filled (the 7x7 stem: J = 147), and for 1x1 layers: twice
  // the tiles means half the reduction splits, so half the partial sums to write and add up
  // (measured on the ResNet-50 shapes: 4-7 % faster there, slower for 3x3 layers).
  if (J % 128 != 0 && J % 128 <= 64) bn = 64;
  if (R == 1 && S == 1 && Kg >= 128) bn = 64;
  const int tilesI = ceil_div(Kg, bm), tilesJ = ceil_div(J, bn);
  const long long tiles = (long long)tilesI * tilesJ * groups;
  // Two blocks fit a CU (LDS), so 2 x CUs (512 on an MI355X) run at a time and all take equally
  // long: fill one such round as well as possible, or two rounds if that fills them clearly better;
  // at least 8 chunks (256 pixels) of work per split.
  const int kSlots = 2 * tt::compute_units();
  struct Run { int n0, n, chunks, cps, splits, slot0; };
  std::vector<Run> runs;
  int slots = 0;
  for (int n0 = 0; n0 < N; n0 += per_run) {
    Run r{};
    r.n0 = n0;
    r.n = std::min(per_run, N - n0);
    r.chunks = ceil_div((long long)r.n * P * Q, kBK);
    int splits = (int)(kSlots / tiles);
    const int two = (int)(2 * kSlots / tiles);
    if ((double)tiles * two / (2.0 * kSlots) > (double)tiles * splits / kSlots + 0.08) splits = two;
    if (splits > r.chunks / 8) splits = r.chunks / 8;
    if (splits < 1) splits = 1;
    if (splits > 4096) splits = 4096;
    r.cps = ceil_div(r.chunks, splits);
    r.splits = ceil_div(r.chunks, r.cps);
    r.slot0 = slots;
    slots += r.splits;
    runs.push_back(r);
  }

  const size_t elems = (size_t)groups * Kg * J;
  // Partial sums added inside the kernel: one run, several splits, and every partial tile of the
  // grid (padded to whole tiles, 16 bytes per lane) addressable with 32-bit byte offsets per tile.
  const size_t fuse_bytes = sizeof(float) * (size_t)bm * bn * (size_t)tiles * (size_t)slots;
  const bool fuse_shape = runs.size() == 1 && slots > 1 && tiles * slots <= kFuseFlagWords &&
                          (long long)slots * bm * bn * 4 < (1LL << 31);
  if (size_only) {
    const size_t plain = slots > 1 ? sizeof(float) * elems * slots : 0;
    *size_only = fuse_shape && fuse_bytes > plain ? fuse_bytes : plain;
    return 0;
  }
  hipStream_t st = check_only ? nullptr : tt::stream();
  float* target = dw;
  void* ws = nullptr;
  bool fused = false;
  for (const Run& r : runs) {
    Wgrad p{};
    p.x = x + (size_t)r.n0 * C * H * W;
    p.dy = dy + (size_t)r.n0 * K * P * Q;
    p.Kg = Kg; p.J = J; p.M = r.n * P * Q;
    p.chunks = r.chunks; p.chunksPerSplit = r.cps;
    p.divPQ = tt::make_fastdiv((uint32_t)(P * Q));
    p.divQ = tt::make_fastdiv((uint32_t)Q);
    p.divRS = tt::make_fastdiv((uint32_t)(R * S));
    p.divS = tt::make_fastdiv((uint32_t)S);
    p.sh = sh; p.sw = sw; p.ph = ph; p.pw = pw; p.dh = dh; p.dw = dw_;
    p.H = H; p.W = W; p.HW = H * W;
    p.xStrideN = C * H * W; p.xStrideG = Cg * H * W;
    p.dyStrideN = K * P * Q; p.dyStrideG = Kg * P * Q;
    p.PQ = P * Q;
    p.tilesI = tilesI;
    p.outStrideSplit = elems;
    p.R = R; p.S = S;
    p.xBias = ph * W + pw;
    // buffer path: byte offsets relative to the first image of a 32-pixel chunk stay below 2 GiB
    // (a chunk spans at most 33 images; x offsets also carry the column's tap and channel offset)
    const long long reach = 4 * (34LL * (p.xStrideN > p.dyStrideN ? p.xStrideN : p.dyStrideN) +
                                 ((long long)H + ph + (long long)R * dh + 2) * W + pw + (long long)S * dw_ + p.xBias);
    const bool buf = R * S <= 63 && reach < (1LL << 31) - (1LL << 20);
    const bool wide = buf && R * S > 31;
    if (buf) {
      const PixGeom geom{r.n, C, K, groups, P, Q, H, W, R, S, sh, sw, ph, pw, dh, dw_, r.chunks};
      if (cached_pixtab(fn, geom, wide, check_only, &p.pixtab, &p.pixhi)) return -1;
    }
    if (check_only) continue;
    // 16-byte fetches along the reduction: whole pixel quads inside one image, aligned tensors
    const bool va = buf && (P * Q) % 4 == 0 && ((uintptr_t)p.dy & 15) == 0;
    const bool vb = va && R == 1 && S == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0 && ((uintptr_t)p.x & 15) == 0;
    WgradKernel kernel;
    if (bm == 128 && bn == 128) kernel = pick_wgrad<2, 2, 2, 2>(buf, va, vb, wide);
    else if (bm == 64 && bn == 128) kernel = pick_wgrad<2, 2, 1, 2>(buf, va, vb, wide);
    else if (bm == 128 && bn == 64) kernel = pick_wgrad<2, 2, 2, 1>(buf, va, vb, wide);
    else kernel = pick_wgrad<2, 2, 1, 1>(buf, va, vb, wide);
    if (ws == nullptr && slots > 1) {   // first run: now the kernel is known, and with it what the device holds of it
      fused = fuse_shape && tiles * r.splits <= resident_blocks(kernel);
      if (tt::workspace(fused ? fuse_bytes : sizeof(float) * elems * slots, &ws)) return -1;
      target = (float*)ws;
    }
    p.out = target + (size_t)r.slot0 * elems;
    if (fused) {
      p.out = dw;
      p.fuse = 1;
      p.fusePartial = (floatx4*)ws;
      if (fuse_flags(&p.fuseFlags) || tt::conv_async_error_word(&p.fuseError)) return -1;
      if (++g_fuse_epoch == 0) ++g_fuse_epoch;
      p.fuseEpoch = g_fuse_epoch;
      // adding stage: nf float4s per block; KL lanes along the splits for each, KL * NF = 256
      const int nf = ceil_div((long long)bm * bn / 4, r.splits);
      int KL = 1;
      while (KL < 32 && 2 * KL * nf <= kThreads && 2 * KL <= r.splits) KL *= 2;
      p.fuseKL = KL;
      p.fuseNf = kThreads / KL;
    }
    const int plan[4] = {(int)tiles, r.splits, fused ? 1 : 0, slots};
    std::copy(plan, plan + 4, g_last_wgrad);
    dim3 grid(tilesI * tilesJ, groups, r.splits);
    {
      tt::ProfScope prof(TT_PROF_CONV_WGRAD);
      hipLaunchKernelGGL(kernel, grid, dim3(kThreads), 0, st, p);
    }
    TT_LAUNCH_CHECK();
  }
  if (check_only) return 0;
  if (slots > 1 && !fused) {
    tt::ProfScope prof(TT_PROF_CONV_WGRAD_REDUCE);
    wgrad_reduce<<<ceil_div((long long)elems, 256), kThreads, 0, st>>>(target, dw, elems, slots);
    TT_LAUNCH_CHECK();
  }
  return 0;
}

// Instrumentation (tests): {tiles, reduction splits, 1 if the partial sums were added inside the
// kernel, partial-sum slots} of the last weight-gradient launch.
int tt_conv2d_last_wgrad_launch(int* plan4) {
  TT_API_LOCK();
  TT_REQUIRE(plan4 != nullptr, "tt_conv2d_last_wgrad_launch: null result pointer");
  std::copy(g_last_wgrad, g_last_wgrad + 4, plan4);
  return 0;
}

// Instrumentation (tests): pretend the device holds `blocks` blocks of every weight-gradient kernel
// per compute unit (-1: ask the device), so that the separate reduce kernel can be exercised on
// shapes that would otherwise add their partial sums inside the kernel.
int tt_conv2d_wgrad_force_occupancy(int blocks) {
  TT_API_LOCK();
  TT_REQUIRE(blocks >= -1 && blocks <= 64, "tt_conv2d_wgrad_force_occupancy: %d is out of range (-1..64)", blocks);
  g_wgrad_forced_occupancy = blocks;
  return 0;
}

int tt_conv2d_wgrad_f32(const float* x, const float* dy, float* dw, int N, int C, int H, int W, int K, int R, int S,
                        int sh, int sw, int ph, int pw, int dh, int dw_, int groups, int P, int Q) {
  return conv2d_wgrad(x, dy, dw, N, C, H, W, K, R, S, sh, sw, ph, pw, dh, dw_, groups, P, Q, nullptr);
}

// Host-only: builds the pixel tables the call would use for this geometry and checks every entry's
// reach against x and dy, as the call itself does once per new geometry.
int tt_conv2d_check_tables_wgrad_f32(int N, int C, int H, int W, int K, int R, int S, int sh, int sw, int ph, int pw,
                                     int dh, int dw_, int groups, int P, int Q) {
  return conv2d_wgrad(nullptr, nullptr, nullptr, N, C, H, W, K, R, S, sh, sw, ph, pw, dh, dw_, groups, P, Q, nullptr, true);
}

// Host-only: damages single fields of single pixel-table entries (image, dy offset, x offset, a tap
// bit; 32-bit and 64-bit masks) and returns 0 when the check refuses every damaged table and
// accepts the undamaged ones.
int tt_conv2d_check_tables_selftest_wgrad(void) {
  TT_API_LOCK();
  struct Case { int R, pad, stride, entry, field, delta; };
  const Case cases[] = {{3, 1, 1, 7, 0, 1},   {3, 1, 1, 40, 1, 4},  {3, 1, 2, 5, 2, 4},      {3, 1, 1, 0, 3, 1},
                        {3, 1, 1, 13, 3, 16}, {7, 3, 2, 9, 2, 64},  {7, 3, 2, 30, 3, 1 << 20}, {3, 1, 1, 3 * 144 - 1, 0, 2}};
  int bad = 0;
  for (const Case& c : cases) {
    const int H = 9 + c.R, P = (H + 2 * c.pad - c.R) / c.stride + 1;
    for (int damaged = 0; damaged < 2; ++damaged) {
      g_pix_fault_entry = damaged ? c.entry : -1;
      g_pix_fault_field = c.field;
      g_pix_fault_delta = c.delta;
      const int rc = conv2d_wgrad(nullptr, nullptr, nullptr, 3, 8, H, H, 16, c.R, c.R, c.stride, c.stride, c.pad, c.pad, 1, 1, 1,
                                  P, P, nullptr, true);
      g_pix_fault_entry = -1;
      if ((rc != 0) != (damaged != 0)) ++bad;
    }
  }
  TT_REQUIRE(bad == 0, "tt_conv2d_check_tables_selftest_wgrad: %d of 16 table checks gave the wrong verdict", bad);
  return 0;
}

int tt_workspace_size_conv2d_wgrad_f32(size_t* bytes, int N, int C, int H, int W, int K, int R, int S, int sh, int sw,
                                       int ph, int pw, int dh, int dw_, int groups, int P, int Q) {
  TT_REQUIRE(bytes, "tt_workspace_size_conv2d_wgrad_f32: null result pointer");
  const float* in = reinterpret_cast<const float*>(uintptr_t(256));   // placeholder, never dereferenced
  return conv2d_wgrad(in, in, const_cast<float*>(in), N, C, H, W, K, R, S, sh, sw, ph, pw, dh, dw_, groups, P, Q,
                      bytes);
}

}  // extern "C"
