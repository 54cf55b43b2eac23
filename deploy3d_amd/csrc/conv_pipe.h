// Software-pipelined MFMA convolution for gfx950 (fp16 / bf16 storage with fp32 accumulation; int8 storage with
// int32 accumulation and a requantizing store, for rows of 64 or 128 bytes).
//
// Same mathematics and data layouts as convStaged (conv_kernels.h): output-stationary tiles, rows of a tap
// gathered through the neighbour table into an XOR-swizzled LDS stage, weights in fragment-major order streamed
// through LDS, one plain store per output element.  What differs is the schedule.  convStaged runs 8 wavefronts
// that a barrier re-aligns every tap, each with its phases back to back (weight fragments from LDS, MFMAs,
// gather issue, row fragments from LDS), so the LDS pipe, the vector-memory path and the matrix pipe take turns,
// and every tile pays for a prologue of two dependent memory round trips.  Here
//  * a wavefront multiplies its 16*MT rows one 16-row group after the other and keeps two register sets of
//    fragments: while group m multiplies, the row fragments of group m+1 and one weight fragment of the NEXT step
//    are read from LDS, the stage rows of group m (already in registers) are refilled with the rows of the step
//    after next, and the index and weight loads of later steps are issued - each piece placed behind an MFMA in
//    program order, so all of it runs in the shadow of the matrix pipe;
//  * workgroups are persistent and the pipeline runs ACROSS tiles: a workgroup's tiles form one stream of steps
//    (tile, tap, channel part); when the multiplying end of the pipeline finishes a tile it stores the tile's rows
//    and clears the accumulators, while the loading end is already several steps into the next tile.  Only the
//    first tile of a workgroup pays for a prologue;
//  * a step exists only for taps that some row of the workgroup's tile has (tile masks written with the table).
//
// Gathers and index loads are buffer loads: an absent neighbour (-1) or a row past the input produces an
// out-of-range offset, for which the hardware delivers zeros - no zero row, no select, one VALU per gather.
#pragma once
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "conv_kernels.h"

namespace d3d {
namespace convk {

typedef __attribute__((address_space(3))) void* LdsVoidPtr;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t makeRawBuffer(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(bytes), 0x00020000);
}

// tileMasks: one 64-bit tap mask per 64 output rows, padded with zero entries to a multiple of 8 entries past
// ceil(outRows / 64) (a workgroup reads the masks of a whole tile at once); null = every tap of every tile.
template <class T, int CIN, int COUT, int MT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
convPipe(const T* __restrict__ in, T* __restrict__ out, const T* __restrict__ wf, const float* __restrict__ bias,
         const float* __restrict__ requantM, const int32_t* __restrict__ nbr, int64_t nbrPitch, int tapMirror,
         const unsigned long long* __restrict__ tileMasks, int kVol, int64_t inRows, int64_t outRows, int relu,
         int tileBlocks, int xcdShift, const int32_t* __restrict__ numActOut) {
  constexpr int THREADS = 64 * WAVES;
  constexpr int ES = static_cast<int>(sizeof(T));
  constexpr int CS = CIN * ES > 128 ? 128 / ES : CIN;          // input channels per step (at most 128 bytes of a row); a tap takes KS steps
  constexpr int KS = CIN / CS;
  constexpr int CH = CS * ES / 16;                             // 16-byte chunks of a row staged per step
  constexpr int RPI = 64 / CH;                                 // rows one gather instruction covers
  constexpr int WM = 16 * MT, TM = WAVES * WM;
  constexpr int GL = WM / RPI;                                 // gather instructions per step
  constexpr int GPM = 16 / RPI;                                // gathers that cover the 16 rows of one row group
  constexpr int NT = COUT / 16;
  constexpr int KK = CS * ES / 64;                             // MFMAs along K per step: 64 bytes of a row each
  constexpr int NQ = KK * NT;                                  // MFMAs per row group and step
  constexpr int WCH = CS * COUT * ES / 16;                     // 16-byte chunks of one step's weights
  constexpr int WL = (WCH + THREADS - 1) / THREADS;            // weight loads per wavefront and step
  constexpr int NWB = 3;                                       // weight buffers
  constexpr int NI = 4;                                        // index ring depth (steps)
  constexpr int IL = (WM + 63) / 64;                           // index loads per step
  constexpr int SLOTS = WM * CH;                               // 16-byte slots of one stage
  constexpr int PER = TM / 64;                                 // tile masks per workgroup tile
  constexpr int ROWSHIFT = CIN * ES == 64 ? 6 : (CIN * ES == 128 ? 7 : 8);
  static_assert((ES == 2 || ES == 1) && (CS * ES == 64 || CS * ES == 128) && CIN % CS == 0 && WM % RPI == 0 && TM % 64 == 0, "shape");
  static_assert((1 << ROWSHIFT) == CIN * ES && WCH % 64 == 0 && MT >= 2 && MT * NT * 4 <= 128, "shape");
  static_assert(WM < 64 || WM % 64 == 0, "an index load covers 64 rows: a wavefront tile is below 64 rows or whole multiples");
  using F = u32x4;
  using Acc = typename Mfma<T>::Acc;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kgrp = lane >> 4;
  u32x4* wLds = reinterpret_cast<u32x4*>(smem);                                      // [NWB][WCH]
  u32x4* stage = reinterpret_cast<u32x4*>(smem + static_cast<size_t>(NWB) * WCH * 16) + wave * 2 * SLOTS;  // [2][SLOTS]
  // ring of NI steps' neighbour indices, per wavefront, stored so that the GL indices one lane needs for its
  // gathers are consecutive: position (lane / CH) * GL + j holds the index of tile row j * RPI + lane / CH
  int32_t* idxLds = reinterpret_cast<int32_t*>(smem + static_cast<size_t>(NWB) * WCH * 16 +
                                               static_cast<size_t>(WAVES) * 2 * SLOTS * 16) + wave * NI * WM;

  // the 16-byte chunk of a row this lane gathers: logical chunk (lane % CH) of stage row (j * RPI + lane / CH)
  // lands in physical chunk lane % CH, so the lane fetches the chunk that the swizzle maps there (the swizzle of
  // a stage row does not depend on j)
  const uint32_t chunkOff = static_cast<uint32_t>(((lane % CH) ^ stageSwizzle<CH>(lane / CH)) * 16);
  const __amdgpu_buffer_rsrc_t inBuf = makeRawBuffer(in, static_cast<uint32_t>(inRows * (CIN * ES)));
  const __amdgpu_buffer_rsrc_t nbrBuf = makeRawBuffer(nbr, static_cast<uint32_t>(kVol * nbrPitch * 4));
  // Row of the tile (counted from the workgroup's first row) whose index sits at ring position i * 64 + lane:
  // position p belongs to the wavefront's row (p % GL) * RPI + p / GL.
  uint32_t idxRow[IL];
#pragma unroll
  for (int i = 0; i < IL; ++i) {
    const int p = i * 64 + lane;
    idxRow[i] = static_cast<uint32_t>(wave * WM + (p % GL) * RPI + p / GL);
  }

  // ---- this workgroup's tiles: XCD x serves the x-th contiguous part of the tiles that hold live rows
  // (neighbouring tiles gather many of the same rows: they should meet behind one L2) and its share of the tiles
  // past the live rows; inside an XCD, workgroups take tiles round robin ----
  const TileOrder order(tileBlocks, static_cast<int>((liveOutRows(numActOut, outRows) + TM - 1) / TM), xcdShift,
                        blockIdx.x & ((1 << xcdShift) - 1));
  const int firstLocal = blockIdx.x >> xcdShift, strideLocal = gridDim.x >> xcdShift;
  const int nMine = firstLocal < order.count() ? (order.count() - 1 - firstLocal) / strideLocal + 1 : 0;
  if (nMine <= 0) return;                                // workgroup-uniform
  auto tileAt = [&](int pos) __attribute__((always_inline)) { return order.tile(firstLocal + pos * strideLocal); };
  const unsigned long long allTaps = kVol >= 64 ? ~0ull : ((1ull << kVol) - 1ull);
  // taps of the workgroup's pos-th tile; a tile without any tap still takes one step (tap 0: all rows absent)
  auto maskAt = [&](int pos) __attribute__((always_inline)) -> unsigned long long {
    if (pos >= nMine) return 0ull;
    if (!order.live(firstLocal + pos * strideLocal)) return 1ull;   // no live row: one step of absent neighbours
    unsigned long long m = allTaps;
    if (tileMasks) {
      const unsigned long long* p = tileMasks + static_cast<int64_t>(tileAt(pos)) * PER;
      m = 0;
#pragma unroll
      for (int e = 0; e < PER; ++e) m |= p[e];
      m &= allTaps;
    }
    return m ? m : 1ull;
  };

  // A walk over the workgroup's steps (tile, tap, part), one per consumer; each consumer asks for its steps in
  // order.  Past the last step a walk stays on it: the loads issued for steps that do not exist repeat valid
  // addresses and nothing in the loop has to branch on "is there such a step".
  struct Walk {
    int pos;                       // ordinal of the tile among this workgroup's
    unsigned long long rem, next;  // taps of this tile still to walk; taps of the following tile
    int tap, part;
  };
  auto walkInit = [&]() __attribute__((always_inline)) { return Walk{0, maskAt(0), maskAt(1), 0, 0}; };
  // moves to the walk's next step; returns its step id (tap * KS + part).  *newTile = the step opens a tile.
  auto walkNext = [&](Walk& w, bool* newTile) __attribute__((always_inline)) -> int {
    *newTile = false;
    if (w.part == 0) {
      if (w.rem == 0 && w.pos + 1 < nMine) {
        ++w.pos;
        w.rem = w.next;
        w.next = maskAt(w.pos + 1);
        *newTile = true;
      }
      if (w.rem) {
        w.tap = __builtin_ctzll(w.rem);
        w.rem &= w.rem - 1;
      }
    }
    const int s = w.tap * KS + w.part;
    w.part = w.part + 1 == KS ? 0 : w.part + 1;
    return s;
  };
  Walk walkIndex = walkInit(), walkWeights = walkInit(), walkRows = walkInit(), walkMul = walkInit();

  F rowBuf[2][KK];                                   // row fragments of the group that multiplies / of the next
  int32_t ixBuf[2][GPM];                             // neighbour indices for the gathers of this group / the next
  F wtsA[KK][NT], wtsB[KK][NT];                      // weight fragments of this step / of the next
  Acc acc[MT][NT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[m][n] = Acc{0, 0, 0, 0};

  // indices of the index walk's next step -> ring slot `seq % NI` (asynchronous, straight into LDS); rows past
  // the table read as 0 and are never stored
  uint32_t idxOff[IL];
  auto loadIndex = [&](int seq) __attribute__((always_inline)) {
    bool newTile;
    const int tap = walkNext(walkIndex, &newTile) / KS;
    if (newTile || seq == 0) {
      const uint32_t rowBase = static_cast<uint32_t>(tileAt(walkIndex.pos)) * TM;
#pragma unroll
      for (int i = 0; i < IL; ++i) idxOff[i] = (rowBase + idxRow[i]) * 4u;
    }
    const uint32_t base = static_cast<uint32_t>((tapMirror ? kVol - 1 - tap : tap) * nbrPitch * 4);
#pragma unroll
    for (int i = 0; i < IL; ++i) {
      if (WM >= 64 || lane < WM)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(nbrBuf, (LdsVoidPtr)(idxLds + (seq & (NI - 1)) * WM + i * 64), 4,
                                                 base + idxOff[i], 0, 0, 0);
    }
  };
  // the GPM indices of row group m of ring slot `seq % NI`, for this lane's gathers
  auto readIndex = [&](int seq, int m, int32_t (&dst)[GPM]) __attribute__((always_inline)) {
    const int32_t* p = idxLds + (seq & (NI - 1)) * WM + (lane / CH) * GL + m * GPM;
    if constexpr (GPM == 2) {
      const u32x2 v = *reinterpret_cast<const u32x2*>(p);
      dst[0] = static_cast<int32_t>(v[0]);
      dst[1] = static_cast<int32_t>(v[1]);
    } else {
      dst[0] = *p;
    }
  };
  auto gatherOne = [&](int j, int32_t idx, uint32_t partOff, int slot) __attribute__((always_inline)) {
    const uint32_t off = (static_cast<uint32_t>(idx) << ROWSHIFT) + partOff;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(inBuf, (LdsVoidPtr)(stage + slot * SLOTS + j * 64), 16, off, 0, 0, 0);
  };
  auto weightLoad = [&](int q, int s, int buf) __attribute__((always_inline)) {
    const u32x4* wk = reinterpret_cast<const u32x4*>(wf) + static_cast<size_t>(s) * WCH;
    const int base = (q * THREADS + wave * 64) % WCH;  // wavefronts past the slice repeat a part of it: same bytes
    __builtin_amdgcn_global_load_lds(wk + base + lane, wLds + buf * WCH + base, 16, 0, 0);
  };
  auto readRowGroup = [&](F (&dst)[KK], int m, int slot) __attribute__((always_inline)) {
    const int n = m * 16 + r16;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) dst[kk] = stage[slot * SLOTS + n * CH + ((kk * 4 + kgrp) ^ stageSwizzle<CH>(n))];
  };
  auto readWeight = [&](F (&dst)[KK][NT], int e, int buf) __attribute__((always_inline)) {
    dst[e / NT][e % NT] = wLds[buf * WCH + e * 64 + lane];
  };
  // Stores the finished tile (bias, ReLU, one rounding) and clears the accumulators for the next one.  After the
  // MFMAs a lane holds, per channel tile n, 4 consecutive channels (8 bytes) of one row; two 16-lane row swaps
  // per pair of channel tiles hand every lane 8 consecutive channels instead, so a store instruction writes
  // 16 bytes per lane and 64 contiguous bytes per row.
  static_assert(NT % 2 == 0, "channel tiles are stored in pairs");
  auto storeTile = [&](int pos) __attribute__((always_inline)) {
    const int64_t row0 = static_cast<int64_t>(tileAt(pos)) * TM + wave * WM;
#pragma unroll
    for (int n = 0; n < NT; n += 2) {
      const int col0 = n * 16 + kgrp * 4, col1 = col0 + 16;
      const float4v b0 = bias ? *reinterpret_cast<const float4v*>(bias + col0) : float4v{0.f, 0.f, 0.f, 0.f};
      const float4v b1 = bias ? *reinterpret_cast<const float4v*>(bias + col1) : float4v{0.f, 0.f, 0.f, 0.f};
      // channels this lane stores after the swaps: tile n for even 16-lane rows, tile n+1 for odd ones; the
      // first or second half of the tile's 16 channels by lane row / 2
      const int outCol = (n + (kgrp & 1)) * 16 + (kgrp >> 1) * 8;
      if constexpr (ES == 1) {
        // int8: q = clamp(rint(float(acc) * m[c] + bq[c])), lower bound 0 with the fused ReLU; a lane's 4 channels
        // are one dword, and one swap hands every lane 8 consecutive channels.  One channel tile at a time, so that
        // only one set of scales is live beside the accumulators.
        const float lo = relu ? 0.f : -128.f;
        uint32_t packed[2][MT];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int col = h ? col1 : col0;
          const float4v mq = *reinterpret_cast<const float4v*>(requantM + col);
          const float4v bq = h ? b1 : b0;
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float t = static_cast<float>(acc[m][n + h][j]) * mq[j];
              t = t + bq[j];
              const float q = __builtin_fminf(127.f, __builtin_fmaxf(lo, __builtin_rintf(t)));
              w |= (static_cast<uint32_t>(static_cast<int>(q)) & 0xFFu) << (8 * j);
            }
            packed[h][m] = w;
            acc[m][n + h] = Acc{0, 0, 0, 0};
          }
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const auto sw = __builtin_amdgcn_permlane16_swap(packed[0][m], packed[1][m], false, false);
          const u32x2 line = {sw[0], sw[1]};
          const int64_t row = row0 + m * 16 + r16;
          if (row < outRows) *reinterpret_cast<u32x2*>(out + static_cast<size_t>(row) * COUT + outCol) = line;
        }
        __builtin_amdgcn_sched_barrier(0);
      } else {
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        float v0[4], v1[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v0[j] = acc[m][n][j] + b0[j];
          v1[j] = acc[m][n + 1][j] + b1[j];
          if (relu) {
            v0[j] = v0[j] > 0.f ? v0[j] : 0.f;
            v1[j] = v1[j] > 0.f ? v1[j] : 0.f;
          }
        }
        acc[m][n] = Acc{0, 0, 0, 0};
        acc[m][n + 1] = Acc{0, 0, 0, 0};
        T p0[4] = {static_cast<T>(v0[0]), static_cast<T>(v0[1]), static_cast<T>(v0[2]), static_cast<T>(v0[3])};
        T p1[4] = {static_cast<T>(v1[0]), static_cast<T>(v1[1]), static_cast<T>(v1[2]), static_cast<T>(v1[3])};
        const u32x2 a = __builtin_bit_cast(u32x2, p0), c = __builtin_bit_cast(u32x2, p1);
        // swap the odd 16-lane rows of `a` with the even ones of `c`: lane rows then hold
        //   (tile n, ch 0-3 | 4-7), (tile n+1, ch 0-3 | 4-7), (tile n, ch 8-11 | 12-15), (tile n+1, ch 8-11 | 12-15)
        const auto s0 = __builtin_amdgcn_permlane16_swap(a[0], c[0], false, false);
        const auto s1 = __builtin_amdgcn_permlane16_swap(a[1], c[1], false, false);
        const u32x4 line = {s0[0], s1[0], s0[1], s1[1]};
        const int64_t row = row0 + m * 16 + r16;
        if (row < outRows) *reinterpret_cast<u32x4*>(out + static_cast<size_t>(row) * COUT + outCol) = line;
      }
      }
    }
  };

  // ---- prologue: indices of steps 0..3, weights of steps 0..2, rows of steps 0 and 1 in flight ----
  bool opened;
  loadIndex(0);
  loadIndex(1);
  loadIndex(2);
  loadIndex(3);
  for (int wseq = 0; wseq < 3; ++wseq) {
    const int s = walkNext(walkWeights, &opened);
#pragma unroll
    for (int q = 0; q < WL; ++q) weightLoad(q, s, wseq);
  }
  waitVmcnt<0>();
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int s0 = walkNext(walkRows, &opened);
    const uint32_t p0 = chunkOff + static_cast<uint32_t>((s0 % KS) * CS * ES);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      int32_t ix[GPM];
      readIndex(t, m, ix);
#pragma unroll
      for (int g = 0; g < GPM; ++g) gatherOne(m * GPM + g, ix[g], p0, t);
    }
  }
  waitVmcnt<0>();
  __syncthreads();                                  // the weight slices are whole
  readRowGroup(rowBuf[0], 0, 0);
  readIndex(2, 0, ixBuf[0]);
#pragma unroll
  for (int e = 0; e < NQ; ++e) readWeight(wtsA, e, 0);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();                     // buffer 0 has been read by everyone: step 0 refills it

  // One step = one (tile, tap, channel part).  Row groups of 16 rows multiply one after the other; while group m
  // multiplies, the fragments of group m+1 are read (of group 0 of the next step at the end, once its rows have
  // landed), the stage rows of group m - their fragments are in registers - are refilled with the rows of the
  // step after next, one of the next step's weight fragments is read, and the indices four steps on and the
  // weight slice three steps on are requested.
  // SLOT = a % 2 is the stage being multiplied, wbuf = a % 3 the weight buffer whose fragments are in curW.
  // Returns true when the step was the last of its tile.
  int wbuf = 0;
  auto step = [&](int a, auto slotTag, F (&curW)[KK][NT], F (&nxtW)[KK][NT]) __attribute__((always_inline)) -> bool {
    constexpr int SLOT = decltype(slotTag)::value;
    // The two register sets alternate from group to group, across steps as well: with an odd number of groups
    // per step the set a group uses flips with the parity of the step (SLOT is that parity).
    constexpr int PAR = (MT & 1) ? SLOT : 0;
    constexpr int WREADS = (NQ + MT - 1) / MT;      // weight fragment reads per group
    // Loads ride behind MFMAs: the GPM gathers of a group behind its first GPM MFMAs, and the remaining
    // ("free") MFMA slots of the step, in order, carry the index load and then the WL weight loads.
    constexpr int FREE = NQ - GPM;                  // free slots per group
    static_assert(FREE >= 0 && MT * FREE >= 1 + WL, "a step has too few MFMAs to carry its loads");
    constexpr int freeBeforeWait = (MT - 1) * FREE; // free slots ahead of the wait (which opens the last group)
    constexpr int extraBeforeWait = (freeBeforeWait >= 1 ? IL : 0) +
                                    (freeBeforeWait - 1 > WL ? WL : (freeBeforeWait - 1 > 0 ? freeBeforeWait - 1 : 0));
    bool open;
    walkNext(walkMul, &open);
    const bool lastOfTile = walkMul.rem == 0 && walkMul.part == 0;
    const int sRows = walkNext(walkRows, &open);
    const uint32_t partOff = chunkOff + static_cast<uint32_t>((sRows % KS) * CS * ES);
    const int sW = walkNext(walkWeights, &open);
    const int nextBuf = wbuf + 1 == NWB ? 0 : wbuf + 1;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      F(&cur)[KK] = rowBuf[(m + PAR) & 1];
      F(&nxt)[KK] = rowBuf[(m + 1 + PAR) & 1];
      int32_t(&ix)[GPM] = ixBuf[(m + PAR) & 1];
      if (m + 1 < MT) {
        readRowGroup(nxt, m + 1, SLOT);
        readIndex(a + 2, m + 1, ixBuf[(m + 1 + PAR) & 1]);
      } else {
        // everything issued before this step has landed: the rows of the next step, this wavefront's part of
        // the weight slice of the step after next, the indices of the step after that
        waitVmcnt<(MT - 1) * GPM + extraBeforeWait>();
        readRowGroup(nxt, 0, SLOT ^ 1);
        readIndex(a + 3, 0, ixBuf[(m + 1 + PAR) & 1]);
      }
#pragma unroll
      for (int e = m * WREADS; e < (m + 1) * WREADS && e < NQ; ++e)
        readWeight(nxtW, e, nextBuf);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        acc[m][q % NT] = Mfma<T>::k32(curW[q / NT][q % NT], cur[q / NT], acc[m][q % NT]);
        __builtin_amdgcn_sched_barrier(0);
        // the fragments of group m have left LDS (the MFMA above waited for them): refill its stage rows
        if (q < GPM) gatherOne(m * GPM + q, ix[q], partOff, SLOT);
        if (q >= GPM) {
          const int u = m * FREE + q - GPM;         // ordinal of this free slot within the step
          if (u == 0) loadIndex(a + 4);
          if (u >= 1 && u <= WL) weightLoad(u - 1, sW, wbuf);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    wbuf = nextBuf;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    return lastOfTile;
  };

  for (int a = 0;; a += 2) {
    if (step(a, std::integral_constant<int, 0>{}, wtsA, wtsB)) {
      storeTile(walkMul.pos);
      if (walkMul.pos + 1 >= nMine) break;
    }
    if (step(a + 1, std::integral_constant<int, 1>{}, wtsB, wtsA)) {
      storeTile(walkMul.pos);
      if (walkMul.pos + 1 >= nMine) break;
    }
  }
  waitVmcnt<0>();                                   // loads issued for steps that do not exist, and the stores
}

template <class T, int CIN, int COUT, int MT, int WAVES>
int32_t launchPipeCfg(const ConvArgs& a, hipStream_t stream) {
  constexpr int CS = CIN * static_cast<int>(sizeof(T)) > 128 ? 128 / static_cast<int>(sizeof(T)) : CIN;
  constexpr int WM = 16 * MT, TM = WM * WAVES;
  constexpr int WCH = CS * COUT * static_cast<int>(sizeof(T)) / 16;
  const size_t lds = static_cast<size_t>(3) * WCH * 16 + static_cast<size_t>(WAVES) * 2 * WM * (CS * sizeof(T)) +
                     static_cast<size_t>(WAVES) * 4 * WM * 4;
  const int64_t pitch = a.nbrPitch > 0 ? a.nbrPitch : a.outRows;
  if (lds > kLdsLimit || a.kVol > 64) return D3D_ERR_UNSUPPORTED;
  if (static_cast<uint64_t>(a.inRows) * CIN * sizeof(T) >= 0xFFFF0000ull ||
      static_cast<uint64_t>(a.kVol) * static_cast<uint64_t>(pitch) * 4 >= 0xFFFF0000ull ||
      static_cast<uint64_t>(a.outRows) + TM >= 0x3FFFFFFFull)
    return D3D_ERR_UNSUPPORTED;                         // 32-bit buffer offsets
  static std::atomic<size_t> granted{64 * 1024};
  const int32_t rc = grantLds(&convPipe<T, CIN, COUT, MT, WAVES>, lds, &granted);
  if (rc != D3D_OK) return rc;
  const int tiles = static_cast<int>((a.outRows + TM - 1) / TM);
  // persistent workgroups: as many as the CUs can hold at this LDS footprint, never more than there are tiles
  int perCu = static_cast<int>(kLdsLimit / lds);
  if (perCu > 2) perCu = 2;
  if (perCu < 1) perCu = 1;
  const ChipLayout chip = chipLayout();
  const int nXcd = 1 << chip.xcdShift;
  int blocks = (tiles + nXcd - 1) / nXcd * nXcd;
  if (blocks > chip.cus / nXcd * nXcd * perCu) blocks = chip.cus / nXcd * nXcd * perCu;
  hipLaunchKernelGGL((convPipe<T, CIN, COUT, MT, WAVES>), dim3(static_cast<unsigned>(blocks)), dim3(64 * WAVES),
                     lds, stream, static_cast<const T*>(a.in), static_cast<T*>(a.out),
                     static_cast<const T*>(a.weightsMfma), a.bias, a.requantM, a.nbr, pitch, a.tapMirror, a.tileMasks,
                     a.kVol, a.inRows, a.outRows, a.relu, tiles, chip.xcdShift, a.numActOut);
  return D3D_OK;
}

// Configuration per layer shape, measured on the layers of a VoxelNet backbone (120k voxels): rows per wavefront
// 16 * MT, wavefronts per workgroup.  64 x 64 and narrower tiles afford 8 wavefronts (4 wavefronts of 128 rows,
// which read half the weight fragments per MFMA, measured slower on a 64 -> 64 layer: 68 us against 58 - one
// wavefront per SIMD has nobody to hide its waits); 128 output channels double the accumulators, so the wavefront
// tile halves.  32 -> 32 takes 8 wavefronts as well (two workgroups of 78 KB per CU, 16 wavefronts): 38 us against
// 41 with 4, 40 with three 4-wavefront workgroups per CU, 41 with 128-row and 42 with 48-row wavefront tiles; with gathers and MFMAs
// both taken out of it the kernel still runs 27 us on that layer (25 with the table reads served from cache), so
// what is left is the per-step bookkeeping of a 32-channel step, not a memory or matrix limit.  Two taps per step
// (a stage row holding the neighbours under two taps side by side, the step of a 64-channel layer) measured slower
// on both 32-channel layers in every tile shape tried (32 -> 32: 44-58 us against 37.5; 32 -> 64: 45-57 against
// 36): the stage doubles, one workgroup fits a CU instead of two, and the layer needs the wavefronts more than
// the longer steps.  Smaller tiles for the sake of balance do not pay either: 351 000 rows are 686 tiles of 512 rows
// on 512 workgroup slots (the busiest workgroup takes two), yet 384-row tiles (busiest: 768 rows) run the layer in
// 43 us and 256-row tiles in 49 - a step costs about the same whatever its rows, because a CU's 16 wavefronts
// move about 168 KB through LDS per step (gathered rows in and out, weight fragments) at 128 bytes per clock.
// Layers with few
// rows (the 128-channel stages: 47 000 rows are 186 tiles of 256 rows for 256 CUs) pick the workgroup shape by
// tile count: the time of a layer that fits one round is that of ONE tile, so 248 tiles of 192 rows beat 186 of
// 256 (48 us against 55), and there four wavefronts of 48 rows - one per SIMD, three 16-row groups each - beat
// six of 32 rows (45 us against 48).
template <class T, int CIN, int COUT>
int32_t launchPipeShape(const ConvArgs& a, hipStream_t stream) {
  // shapes go by the bytes of an input row (the stage) and by the output channels (the accumulators): an int8 layer
  // takes the shape of the two-byte layer with half its input channels
  constexpr int RB = CIN * static_cast<int>(sizeof(T));
  if constexpr (RB == 128 && COUT == 64) {
    return launchPipeCfg<T, CIN, COUT, 4, 8>(a, stream);
  } else if constexpr (COUT >= 128) {
    // 8, 6 or 4 wavefronts of 32 rows: the workgroup size whose tiles load the busiest CU least (rounds of tiles
    // over the 256 CUs x rows per tile).  A layer that fits ONE round of 192-row tiles takes them as four
    // wavefronts of 48 rows - one per SIMD - instead of six of 32, which load two SIMDs twice as much as the
    // others (conv4_x: 45 us against 48); over several rounds the eight-wavefront shapes hide their waits better
    // (a 64 -> 128 layer of 10 rounds: 105 us with 8 x 32 rows, 138 us with 4 x 48).
    static const int kCand[4][2] = {{32, 8}, {32, 6}, {32, 4}, {48, 4}};
    // int8 128 -> 128: the wider workgroups (two wavefronts per SIMD, 256 registers each) spill - 84-97 us against
    // 33-44 on a 47 000-row layer - so only the four-wavefront shapes are candidates, the larger tile winning ties
    constexpr bool FOUR_ONLY = sizeof(T) == 1 && CIN == 128;
    int best = FOUR_ONLY ? 3 : 0;
    int64_t bestCost = 0;
    const int64_t cus = chipLayout().cus;
    auto costOf = [&](int c) {
      const int64_t tm = kCand[c][0] * kCand[c][1], tiles = (a.outRows + tm - 1) / tm;
      return (tiles + cus - 1) / cus * tm;              // rows the busiest CU multiplies
    };
    if (FOUR_ONLY) {
      if (costOf(2) < costOf(3)) best = 2;
    } else {
      for (int c = 0; c < 3; ++c) {
        const int64_t cost = costOf(c);
        if (c == 0 || cost < bestCost) {
          best = c;
          bestCost = cost;
        }
      }
      if (best == 1 && (a.outRows + 191) / 192 <= cus) best = 3;
    }
    if (const char* force = debugEnv("D3D_CONV_PIPE_SHAPE")) {  // "rows,wavefronts" of one candidate (tests)
      for (int c = FOUR_ONLY ? 2 : 0; c < 4; ++c)
        if (std::atoi(force) == kCand[c][0] && std::strchr(force, ',') &&
            std::atoi(std::strchr(force, ',') + 1) == kCand[c][1])
          best = c;
    }
    if (best == 2) return launchPipeCfg<T, CIN, COUT, 2, 4>(a, stream);
    if (best == 3) return launchPipeCfg<T, CIN, COUT, 3, 4>(a, stream);
    if constexpr (!FOUR_ONLY) {
      if (best == 1) return launchPipeCfg<T, CIN, COUT, 2, 6>(a, stream);
      return launchPipeCfg<T, CIN, COUT, 2, 8>(a, stream);
    }
    return D3D_ERR_UNSUPPORTED;
  } else if constexpr (RB == 64 && COUT == 32) {
    return launchPipeCfg<T, CIN, COUT, 4, 8>(a, stream);
  } else {
    return launchPipeCfg<T, CIN, COUT, 4, 4>(a, stream);
  }
}

template <class T>
int32_t launchPipe(const ConvArgs& a, hipStream_t stream) {
#define D3D_PIPE_CASE(CI, CO) \
  if (a.cin == CI && a.cout == CO) return launchPipeShape<T, CI, CO>(a, stream);
  if constexpr (sizeof(T) == 2) {  // rows of 64 bytes at least
    D3D_PIPE_CASE(32, 32)
    D3D_PIPE_CASE(32, 64)
    D3D_PIPE_CASE(32, 128)
  }
  D3D_PIPE_CASE(64, 32)
  D3D_PIPE_CASE(64, 64)
  D3D_PIPE_CASE(64, 128)
  D3D_PIPE_CASE(128, 32)
  D3D_PIPE_CASE(128, 64)
  D3D_PIPE_CASE(128, 128)
#undef D3D_PIPE_CASE
  return D3D_ERR_UNSUPPORTED;
}

}  // namespace convk
}  // namespace d3d
