// The implicit-GEMM convolution kernel body for gfx950, shared by the translation units that
// instantiate it: conv_igemm.hip (float32 and bf16 matrix instructions) and conv_igemm_x3.hip (float32
// arithmetic in three bf16 terms).  Everything here is device code in an unnamed namespace: each unit
// gets its own copy.
#pragma once
#include <type_traits>

#include "conv_igemm_common.h"

namespace {

using namespace ttc;

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


}  // namespace
