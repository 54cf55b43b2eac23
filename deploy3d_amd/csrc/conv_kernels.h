// MFMA convolution kernels of the sparse-convolution engine for gfx950 and their launchers, as templates: one
// translation unit per storage type instantiates them (conv_half.hip, conv_bf16.hip, conv_int8.hip), so the types
// compile side by side.
#pragma once
#include <hip/hip_fp16.h>

#include <atomic>
#include <type_traits>

#include "common.h"

namespace d3d {
namespace convk {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int32_t int4v __attribute__((ext_vector_type(4)));


// ---------------------------------------------------------------------------
// MFMA implicit GEMM, fp16 / bf16 storage, fp32 accumulation.
//
// A wavefront owns 16*MT consecutive output rows and all COUT channels; a
// workgroup is 4 such wavefronts.  Per tap
//   * each lane gathers its own operand fragments of the input rows straight
//     from global memory into registers (16 bytes per load; the four lanes of
//     a row cover 64 contiguous bytes), zero for rows without this tap, and
//     the gathers of the next two taps are already in flight while the MFMAs
//     of the current tap run;
//   * the weight slice comes from LDS, in the fragment-major order of the
//     device copy (Wf[tap][kk][n][lane]), so weight reads and row gathers are
//     tracked by different hardware counters and overlap freely.
// The product is formed transposed, D^T = W[tap]^T-tile x rows^T, so a lane
// ends up with 4 consecutive output channels of one row and the epilogue
// (bias, ReLU, one rounding) stores 8 bytes per lane.
//
// Operand layout of v_mfma_f32_16x16x32 (and 16x16x16): lane l supplies row
// (first operand) or column (second operand) l%16 and the (l/16)-th group of
// 8 (4) consecutive K values; it receives column l%16, rows 4*(l/16)..+3.
// ---------------------------------------------------------------------------
template <class T> struct Mfma;
template <> struct Mfma<_Float16> {
  using Acc = float4v;
  __device__ static float4v k32(const u32x4& a, const u32x4& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0,
                                                  0);
  }
  __device__ static float4v k16(const u32x2& a, const u32x2& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, a), __builtin_bit_cast(half4, b), c, 0, 0,
                                                 0);
  }
};
template <> struct Mfma<__bf16> {
  using Acc = float4v;
  __device__ static float4v k32(const u32x4& a, const u32x4& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  }
  __device__ static float4v k16(const u32x2& a, const u32x2& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4v, a), __builtin_bit_cast(short4v, b), c,
                                                     0, 0, 0);
  }
};

// int8 operands, int32 accumulators: 16x16x64 takes 16 bytes per lane, 16x16x32 takes 8.
template <> struct Mfma<int8_t> {
  using Acc = int4v;
  __device__ static int4v k32(const u32x4& a, const u32x4& b, const int4v& c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(int4v, a), __builtin_bit_cast(int4v, b), c, 0, 0, 0);
  }
  __device__ static int4v k16(const u32x2& a, const u32x2& b, const int4v& c) {
    return __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b), c, 0, 0, 0);
  }
};

// Which tiles (or row groups) a persistent workgroup serves, in which order.  Workgroups are dealt to the XCDs
// round-robin; XCD x serves the x-th contiguous part of the tiles that hold LIVE rows (neighbouring tiles gather
// many of the same rows: they meet behind one L2), and every n-th of the tiles past the live rows, which only
// take their bias.  With capacities above the live count the XCDs still share the real work evenly (a partition
// of all tiles gave the last XCDs nothing but empty ones: 45 -> 85 us on a layer at 1.5 x capacity).
struct TileOrder {
  int liveTiles, liveLocal, lx, dx, nXcd, xcd;
  __device__ __forceinline__ TileOrder(int tiles, int live, int xcdShift, int xcdOfBlock) {
    nXcd = 1 << xcdShift;
    xcd = xcdOfBlock;
    liveTiles = live < tiles ? live : tiles;
    liveLocal = (liveTiles + nXcd - 1) >> xcdShift;
    int hi = (xcd + 1) * liveLocal;
    if (hi > liveTiles) hi = liveTiles;
    lx = hi - xcd * liveLocal;
    if (lx < 0) lx = 0;
    const int dead = tiles - liveTiles;
    dx = xcd < dead ? (dead - xcd + nXcd - 1) >> xcdShift : 0;
  }
  __device__ __forceinline__ int count() const { return lx + dx; }          // tiles of this XCD
  __device__ __forceinline__ bool live(int local) const { return local < lx; }
  __device__ __forceinline__ int tile(int local) const {
    return local < lx ? xcd * liveLocal + local : liveTiles + (local - lx) * nXcd + xcd;
  }
};

// Live rows of the output (device count clamped to the capacity; the capacity when no count is passed).
__device__ __forceinline__ int64_t liveOutRows(const int32_t* numActOut, int64_t outRows) {
  if (!numActOut) return outRows;
  const int64_t n = *numActOut;
  return n < 0 ? 0 : (n > outRows ? outRows : n);
}

// Fragment type per K step: 8 elements (16 bytes) when CIN >= 32, else 4.
template <int CIN> struct Frag { using type = u32x4; };
template <> struct Frag<16> { using type = u32x2; };

// Weights live in LDS in the same fragment-major order as in global memory:
// fragment (kk, n) of a tap is 64 consecutive lanes' worth of data, so a
// wavefront read is one contiguous, conflict-free sweep.
//
// RESIDENT = true : the weights of ALL taps fit in LDS.  They are loaded once
//   in the prologue and shared by up to 16 wavefronts; after that every
//   wavefront runs alone (its own list of the taps that occur among its rows,
//   no barriers).
// RESIDENT = false: one tap's weights at a time, double-buffered.  The slice of
//   tap t+1 travels global -> registers -> idle LDS buffer while tap t
//   multiplies; one barrier per tap.  The weights are requested before the
//   rows, because the vector-memory counter retires in order: waiting for a
//   weight slice must not drain the younger gathers behind it.
// Either way three register sets of gathered rows rotate, so the gathers of
// taps t+1 and t+2 are in flight while tap t multiplies.  The rotation is
// written out as three pipeline steps per loop iteration, with no branch
// between them (the tap list is padded to a multiple of three with null taps
// whose rows all come from the zero row), so that the compiler can neither
// sink a gather towards its use nor has to copy a register set that is still
// being loaded.
template <class T, int CIN, int COUT, int MT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
convMfma(const T* __restrict__ in, T* __restrict__ out, const T* __restrict__ wf, const float* __restrict__ bias,
         const int32_t* __restrict__ nbr, int64_t nbrPitch, int tapMirror, const T* __restrict__ zeros, int kVol,
         int64_t inRows, int64_t outRows, int relu, int tileBlocks, int xcdShift) {
  constexpr int THREADS = 64 * WAVES;
  constexpr int WM = 16 * MT;            // rows per wavefront
  constexpr int TM = WAVES * WM;         // rows per workgroup
  constexpr int NT = COUT / 16;          // output-channel tiles
  constexpr int KSTEP = CIN >= 32 ? 32 : 16;
  constexpr int KK = CIN / KSTEP;        // K steps per tap
  constexpr int KG = KSTEP / 4;          // elements per lane per K step
  constexpr int WFRAGS = KK * NT * 64;   // fragments (lane granules) per tap
  constexpr int WCHUNKS = CIN * COUT / 8;  // 16-byte chunks per tap
  constexpr int WPT = (WCHUNKS + THREADS - 1) / THREADS;
  using F = typename Frag<CIN>::type;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  F* wLds = reinterpret_cast<F*>(smem);  // [2][WFRAGS]
  int32_t* nbT = reinterpret_cast<int32_t*>(smem + static_cast<size_t>(2) * CIN * COUT * sizeof(T));
  int32_t* tapList = nbT + kVol * TM;    // active taps of the tile padded with -1, then their count

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kgrp = lane >> 4;
  // Workgroups are dealt to the XCDs round-robin; handing XCD x the x-th contiguous part of the tiles
  // keeps neighbouring tiles, which gather many of the same rows, behind the same L2.
  const int nXcd = 1 << xcdShift;
  const int perXcd = (tileBlocks + nXcd - 1) >> xcdShift;
  const int tile = (blockIdx.x & (nXcd - 1)) * perXcd + (blockIdx.x >> xcdShift);
  if (tile >= tileBlocks) return;        // workgroup-uniform, before any barrier
  const int64_t row0 = static_cast<int64_t>(tile) * TM;
  const int32_t* nb = nbT + wave * WM;   // this wavefront's columns of the [kVol][TM] neighbour tile

  for (int t = tid; t < kVol + 4; t += THREADS) tapList[t] = 0;
  __syncthreads();
  // neighbour tile: requests first, LDS writes after, four taps at a time
  for (int e0 = 0; e0 < kVol * TM; e0 += 4 * THREADS) {
    int32_t v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = e0 + q * THREADS + tid;
      const int tap = e / TM, r = e % TM;
      const int64_t row = row0 + r;
      const bool ok = e < kVol * TM && row < outRows;
      v[q] = nbr[ok ? static_cast<int64_t>(tapMirror ? kVol - 1 - tap : tap) * nbrPitch + row : 0];
      if (!ok || v[q] >= inRows) v[q] = -1;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = e0 + q * THREADS + tid;
      if (e < kVol * TM) {
        nbT[e] = v[q];
        if (v[q] >= 0) tapList[e / TM] = 1;
      }
    }
  }
  __syncthreads();

  float4v acc[MT][NT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[m][n] = float4v{0.f, 0.f, 0.f, 0.f};

  // Rows without this tap (and every row of a null tap, tap < 0) read a row of zeros (one cached line for the
  // whole device) instead of branching or selecting afterwards: nothing touches the gathered registers until
  // the MFMAs that consume them, so the loads of a tap issue back to back and stay in flight.
  auto gatherRows = [&](int tap, F (&dst)[MT][KK]) __attribute__((always_inline)) {
    int32_t src[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) src[m] = tap < 0 ? -1 : nb[tap * TM + m * 16 + r16];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const T* rowPtr = (src[m] < 0 ? zeros : in + static_cast<size_t>(src[m]) * CIN) + kgrp * KG;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) dst[m][kk] = *reinterpret_cast<const F*>(rowPtr + kk * KSTEP);
    }
  };
  auto multiply = [&](const F* wTap, const F (&rows)[MT][KK]) __attribute__((always_inline)) {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const F wfrag = wTap[(kk * NT + n) * 64 + lane];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          if constexpr (CIN >= 32) {
            acc[m][n] = Mfma<T>::k32(wfrag, rows[m][kk], acc[m][n]);
          } else {
            acc[m][n] = Mfma<T>::k16(wfrag, rows[m][kk], acc[m][n]);
          }
        }
      }
    }
  };

  F bufA[MT][KK], bufB[MT][KK], bufC[MT][KK];

  {
    if (tid == 0) {  // compact the flags into a list in place (slot n <= t is written after flag t was read)
      int n = 0;
      for (int t = 0; t < kVol; ++t)
        if (tapList[t]) tapList[n++] = t;
      const int count = n;
      while (n < kVol + 3) tapList[n++] = -1;  // null taps pad the list
      tapList[kVol + 3] = count;
    }
    __syncthreads();
    const int nActive = tapList[kVol + 3];
    if (nActive > 0) {
      auto tapAt = [&](int a) __attribute__((always_inline)) { return tapList[a < kVol + 3 ? a : kVol + 2]; };
      auto loadWeights = [&](int a, u32x4 (&dst)[WPT]) __attribute__((always_inline)) {
        const int t = tapAt(a);
        const u32x4* wk = reinterpret_cast<const u32x4*>(wf + static_cast<size_t>(t < 0 ? 0 : t) * CIN * COUT);
#pragma unroll
        for (int q = 0; q < WPT; ++q) {
          const int e = tid + q * THREADS;
          dst[q] = wk[(WCHUNKS % THREADS == 0 || e < WCHUNKS) ? e : 0];
        }
      };
      auto storeWeights = [&](int buf, const u32x4 (&src)[WPT]) __attribute__((always_inline)) {
        u32x4* dst = reinterpret_cast<u32x4*>(wLds + buf * WFRAGS);
#pragma unroll
        for (int q = 0; q < WPT; ++q) {
          const int e = tid + q * THREADS;
          if (WCHUNKS % THREADS == 0 || e < WCHUNKS) dst[e] = src[q];
        }
      };
      // one pipeline step: tap a multiplies while the weights of a+1 and the rows of a+2 are requested
      auto step = [&](int a, const F (&rowsNow)[MT][KK], F (&rowsFuture)[MT][KK]) __attribute__((always_inline)) {
        u32x4 wreg[WPT];
        loadWeights(a + 1, wreg);
        gatherRows(tapAt(a + 2), rowsFuture);
        __builtin_amdgcn_sched_barrier(0);  // keep the requests ahead of the MFMAs they are meant to overlap
        multiply(wLds + (a & 1) * WFRAGS, rowsNow);
        __builtin_amdgcn_sched_barrier(0);
        storeWeights((a + 1) & 1, wreg);
        __syncthreads();
      };
      {
        u32x4 wreg[WPT];
        loadWeights(0, wreg);
        gatherRows(tapAt(0), bufA);
        gatherRows(tapAt(1), bufB);
        storeWeights(0, wreg);
      }
      __syncthreads();
      for (int a = 0; a < nActive; a += 3) {  // steps past nActive work on null taps: zero rows, no effect
        step(a, bufA, bufC);
        step(a + 1, bufB, bufA);
        step(a + 2, bufC, bufB);
      }
    }
  }

  // epilogue: lane holds channels n*16 + 4*kgrp .. +3 of row (m*16 + r16)
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int64_t row = row0 + wave * WM + m * 16 + r16;
    if (row >= outRows) continue;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      const int col = n * 16 + kgrp * 4;
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] = acc[m][n][j] + (bias ? bias[col + j] : 0.f);
        if (relu) v[j] = v[j] > 0.f ? v[j] : 0.f;
      }
      T packed[4] = {static_cast<T>(v[0]), static_cast<T>(v[1]), static_cast<T>(v[2]), static_cast<T>(v[3])};
      *reinterpret_cast<u32x2*>(out + static_cast<size_t>(row) * COUT + col) = __builtin_bit_cast(u32x2, packed);
    }
  }
}

// Small layers: the weights of ALL taps fit in LDS.  A workgroup loads them once and then lives on: each of
// its wavefronts walks, on its own, over groups of 16 output rows (group index strided by the number of
// wavefronts in the grid), with a private slice of the neighbour table, its own list of the taps that occur
// in the group, and no barrier after the weight load.  CROW < CIN: the rows of `in` store CROW channels only and
// the lanes that would read the others multiply zeros (their weights are zero rows as well); CROW < 0: the rows
// store `rowCh` channels, any number below CIN, and are read element by element (a 5-channel input: no widened
// copy, and the few bytes of such rows do not need vector loads).
template <class T, int CIN, int COUT, int WAVES, int CROW = CIN>
__global__ void __launch_bounds__(64 * WAVES)
convMfmaResident(const T* __restrict__ in, T* __restrict__ out, const T* __restrict__ wf,
                 const float* __restrict__ bias, const float* __restrict__ requantM, const int32_t* __restrict__ nbr,
                 int64_t nbrPitch, int tapMirror, const T* __restrict__ zeros, int kVol, int64_t inRows,
                 int64_t outRows, int relu, int groups, int xcdShift, const int32_t* __restrict__ numActOut,
                 int rowCh) {
  constexpr int THREADS = 64 * WAVES;
  constexpr int MT = 1;
  constexpr int NT = COUT / 16;
  constexpr int ES = static_cast<int>(sizeof(T));              // 2: fp16 / bf16, 1: int8
  constexpr bool WIDE = CIN * ES >= 64;                        // 16-byte operand fragments (else 8-byte)
  constexpr int KSTEP = (WIDE ? 64 : 32) / ES;                 // channels one MFMA contracts
  constexpr int KK = CIN / KSTEP;
  constexpr int KG = KSTEP / 4;
  constexpr int WFRAGS = KK * NT * 64;
  constexpr int WCHUNKS = CIN * COUT * ES / 16;
  using F = typename std::conditional<WIDE, u32x4, u32x2>::type;
  using Acc = typename Mfma<T>::Acc;
  static_assert(CIN % KSTEP == 0 && (CROW == CIN || (KK == 1 && !WIDE && (CROW < 0 || CROW % KG == 0))), "whole MFMA steps");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  F* wLds = reinterpret_cast<F*>(smem);                                              // [kVol][WFRAGS]
  int32_t* nbAll = reinterpret_cast<int32_t*>(smem + static_cast<size_t>(kVol) * CIN * COUT * sizeof(T));
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kgrp = lane >> 4;
  int32_t* nb = nbAll + wave * kVol * 16;                                            // [kVol][16], private

  {
    const u32x4* src = reinterpret_cast<const u32x4*>(wf);
    u32x4* dst = reinterpret_cast<u32x4*>(wLds);
    for (int e = tid; e < kVol * WCHUNKS; e += THREADS) dst[e] = src[e];
  }
  __syncthreads();

  auto gatherRows = [&](int tap, F (&dst)[MT][KK]) __attribute__((always_inline)) {
    const int32_t src = tap < 0 ? -1 : nb[tap * 16 + r16];
    if constexpr (CROW < 0) {
      T v[KG];
#pragma unroll
      for (int j = 0; j < KG; ++j) {
        const int ch = kgrp * KG + j;
        v[j] = (src >= 0 && ch < rowCh) ? in[static_cast<size_t>(src) * rowCh + ch] : static_cast<T>(0);
      }
      dst[0][0] = __builtin_bit_cast(F, v);
    } else {
      const T* rowPtr = (src < 0 || kgrp * KG >= CROW ? zeros : in + static_cast<size_t>(src) * CROW + kgrp * KG);
      if constexpr (CROW == CIN) rowPtr = (src < 0 ? zeros : in + static_cast<size_t>(src) * CIN) + kgrp * KG;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) dst[0][kk] = *reinterpret_cast<const F*>(rowPtr + kk * KSTEP);
    }
  };

  // Workgroups are dealt to the XCDs round-robin; XCD x takes the x-th contiguous part of the row groups,
  // so neighbouring groups, which gather many of the same rows, meet behind the same L2.
  const int wavesPerXcd = (gridDim.x >> xcdShift) * WAVES;
  const TileOrder order(groups, static_cast<int>((liveOutRows(numActOut, outRows) + 15) / 16), xcdShift,
                        blockIdx.x & ((1 << xcdShift) - 1));
  for (int local = (blockIdx.x >> xcdShift) * WAVES + wave; local < order.count(); local += wavesPerXcd) {
    const int group = order.tile(local);
    const int64_t row0 = static_cast<int64_t>(group) * 16;

    // private neighbour slice and the taps that occur in it (wavefront-uniform masks)
    unsigned long long active[2] = {0ull, 0ull};
    for (int t0 = 0; t0 < kVol; t0 += 4) {
      const int tap = t0 + kgrp;
      const int64_t row = row0 + r16;
      const bool ok = tap < kVol && row < outRows;
      int32_t v = nbr[ok ? static_cast<int64_t>(tapMirror ? kVol - 1 - tap : tap) * nbrPitch + row : 0];
      if (!ok || v >= inRows) v = -1;
      if (tap < kVol) nb[tap * 16 + r16] = v;
      const unsigned long long hit = __ballot(v >= 0);
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if ((hit >> (16 * q)) & 0xFFFFull) active[(t0 + q) >> 6] |= 1ull << ((t0 + q) & 63);
    }
    auto nextTap = [&]() __attribute__((always_inline)) -> int {  // -1 once the list is exhausted
      if (active[0]) {
        const int t = __builtin_ctzll(active[0]);
        active[0] &= active[0] - 1;
        return t;
      }
      if (active[1]) {
        const int t = __builtin_ctzll(active[1]);
        active[1] &= active[1] - 1;
        return 64 + t;
      }
      return -1;
    };
    auto weightsOf = [&](int tap) __attribute__((always_inline)) {
      return wLds + static_cast<size_t>(tap < 0 ? 0 : tap) * WFRAGS;  // a null tap multiplies zero rows
    };

    Acc acc[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[n] = Acc{0, 0, 0, 0};
    auto multiply = [&](const F* wTap, const F (&rows)[MT][KK]) __attribute__((always_inline)) {
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          const F wfrag = wTap[(kk * NT + n) * 64 + lane];
          if constexpr (WIDE) {
            acc[n] = Mfma<T>::k32(wfrag, rows[0][kk], acc[n]);
          } else {
            acc[n] = Mfma<T>::k16(wfrag, rows[0][kk], acc[n]);
          }
        }
      }
    };

    F bufA[MT][KK], bufB[MT][KK], bufC[MT][KK];
    int tA = nextTap(), tB = nextTap(), tC;
    gatherRows(tA, bufA);
    gatherRows(tB, bufB);
    while (tA >= 0) {  // three steps per iteration, no branch between them (see convMfma)
      tC = nextTap();
      gatherRows(tC, bufC);
      __builtin_amdgcn_sched_barrier(0);
      multiply(weightsOf(tA), bufA);
      __builtin_amdgcn_sched_barrier(0);
      tA = nextTap();
      gatherRows(tA, bufA);
      __builtin_amdgcn_sched_barrier(0);
      multiply(weightsOf(tB), bufB);
      __builtin_amdgcn_sched_barrier(0);
      tB = nextTap();
      gatherRows(tB, bufB);
      __builtin_amdgcn_sched_barrier(0);
      multiply(weightsOf(tC), bufC);
      __builtin_amdgcn_sched_barrier(0);
    }

    const int64_t row = row0 + r16;
    if (row < outRows) {
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const int col = n * 16 + kgrp * 4;
        if constexpr (ES == 1) {
          // int8: t = float(acc) * m[c]; t += bq[c]; round to nearest even; clamp (lo = 0 with the fused ReLU)
          uint32_t packed = 0;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            float t = static_cast<float>(acc[n][j]) * requantM[col + j];
            t = t + (bias ? bias[col + j] : 0.f);
            float q = __builtin_rintf(t);
            q = __builtin_fminf(127.f, __builtin_fmaxf(relu ? 0.f : -128.f, q));
            packed |= (static_cast<uint32_t>(static_cast<int>(q)) & 0xFFu) << (8 * j);
          }
          *reinterpret_cast<uint32_t*>(out + static_cast<size_t>(row) * COUT + col) = packed;
        } else {
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[j] = acc[n][j] + (bias ? bias[col + j] : 0.f);
            if (relu) v[j] = v[j] > 0.f ? v[j] : 0.f;
          }
          T packed[4] = {static_cast<T>(v[0]), static_cast<T>(v[1]), static_cast<T>(v[2]), static_cast<T>(v[3])};
          *reinterpret_cast<u32x2*>(out + static_cast<size_t>(row) * COUT + col) = __builtin_bit_cast(u32x2, packed);
        }
      }
    }
  }
}


// ---------------------------------------------------------------------------
// Staged MFMA convolution.
//
// A lane of the MFMA operand layout owns ONE row (lane % 16), so gathering rows
// straight into operand registers makes adjacent lanes touch different rows, and
// the texture path then serves 16 bytes per clock per CU.  It serves 64 when
// the lanes of a quad read 64 contiguous bytes.  Here the gather therefore uses
// the memory-friendly mapping (consecutive lanes sweep one row, 16 bytes each)
// and lands in LDS without passing through registers (global_load_lds); the
// MFMA fragments are then read from LDS in operand layout.  The 16-byte chunks
// of a staged row are XOR-swizzled by row so both sides are conflict-free.
//
// Per wavefront: WM = 16*MT output rows, NS stage slots (rows of tap a+NS are
// in flight while tap a multiplies), the neighbour indices of a tap arrive in
// LDS the same way three taps earlier.  All vector-memory traffic of the loop
// is asynchronous and retires in order, so one s_waitcnt vmcnt(X) per tap, X =
// the loads that may stay in flight, is the only wait.
//
// Weights: RESIDENT = every tap's fragments stay in LDS (small layers, no
// barrier at all); otherwise three tap buffers rotate (tap a multiplies, a+1
// has landed, a+2 is landing) with one barrier per tap.
// The result goes back through the wavefront's stage area so that rows leave
// as whole contiguous lines.
// ---------------------------------------------------------------------------
template <int CH> __device__ __forceinline__ int stageSwizzle(int n) {
  if (CH == 2) return (n >> 2) & 1;
  if (CH == 4) return (n >> 1) & 3;
  if (CH == 8) return n & 7;
  return n & 15;
}

template <int N> __device__ __forceinline__ void waitVmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

constexpr int cmin(int a, int b) { return a < b ? a : b; }

template <class T, int CIN, int COUT, int KS, int MT, int WAVES, int NS, bool RESIDENT>
__global__ void __launch_bounds__(64 * WAVES)
convStaged(const T* __restrict__ in, T* __restrict__ out, const T* __restrict__ wf, const float* __restrict__ bias,
           const float* __restrict__ requantM, const int32_t* __restrict__ nbr, int64_t nbrPitch, int tapMirror,
           const unsigned long long* __restrict__ tileMasks, const T* __restrict__ zeros, int kVol, int64_t inRows,
           int64_t outRows, int relu, int tileBlocks, int xcdShift, const int32_t* __restrict__ numActOut) {
  constexpr int THREADS = 64 * WAVES;
  constexpr int ES = static_cast<int>(sizeof(T));              // 2: fp16 / bf16, 1: int8
  constexpr int CS = CIN / KS;                                 // input channels per step (a tap takes KS steps)
  constexpr int CH = CS * ES / 16;                             // 16-byte chunks of a row staged per step
  constexpr bool WIDE = CS * ES >= 64;                         // 16-byte operand fragments (else 8-byte)
  constexpr int RPI = 64 / CH;                                 // rows one gather instruction covers
  constexpr int WM = 16 * MT, TM = WAVES * WM;
  constexpr int GL = WM / RPI;                                 // gather instructions per tap
  static_assert(WM % RPI == 0 && WM <= 64 && 64 % WM == 0 && TM % 64 == 0, "wavefront tile");
  constexpr int NT = COUT / 16;
  constexpr int KSTEP = (WIDE ? 64 : 32) / ES;                 // channels one MFMA contracts
  constexpr int KK = CS / KSTEP;
  constexpr int WCH = CS * COUT * ES / 16;                     // 16-byte chunks of one step's weights
  static_assert(WCH % 64 == 0 && KK >= 1, "weights per step");
  constexpr int WL = RESIDENT ? 0 : (WCH + THREADS - 1) / THREADS;
  constexpr int NWB = 3, NI = 4;
  constexpr int SLOTS = WM * CH;                               // 16-byte slots per stage
  constexpr int OCH = COUT * ES / 16;                          // chunks per output row
  constexpr bool LDS_EPILOGUE = ES == 2 && WM * OCH <= NS * SLOTS;
  // Issue order inside step a: indices of step a+NS+3, weights of step a+2, rows of step a+NS.  X = loads that
  // may still be in flight when the step ends, behind the rows and the weights of step a+1.
  constexpr int PER_STEP = 1 + WL + GL;
  constexpr int X_ROWS = (NS - 1) * PER_STEP;
  constexpr int X_WEIGHTS = RESIDENT ? 63 : GL + PER_STEP;
  constexpr int X_INDEX = WL + GL + 2 * PER_STEP;
  constexpr int X = cmin(cmin(X_ROWS, X_WEIGHTS), cmin(X_INDEX, 63));
  using F = typename Frag<WIDE ? 32 : 16>::type;
  using Acc = typename Mfma<T>::Acc;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kgrp = lane >> 4;
  const int allSteps = kVol * KS;                              // step id s = tap s / KS, channel part s % KS
  const int wChunks = (RESIDENT ? allSteps : NWB) * WCH;
  u32x4* wLds = reinterpret_cast<u32x4*>(smem);
  int32_t* idxLds = reinterpret_cast<int32_t*>(smem + static_cast<size_t>(wChunks) * 16) + wave * NI * 64;
  u32x4* stage = reinterpret_cast<u32x4*>(smem + static_cast<size_t>(wChunks) * 16 + WAVES * NI * 256) + wave * NS * SLOTS;

  if (RESIDENT) {
    const u32x4* src = reinterpret_cast<const u32x4*>(wf);
    for (int e = tid; e < allSteps * WCH; e += THREADS) wLds[e] = src[e];
    __syncthreads();
  }

  // per-lane constants of the gathers: byte offset of this lane's (swizzled) chunk inside a row
  uint32_t chunkOff[GL];
#pragma unroll
  for (int j = 0; j < GL; ++j)
    chunkOff[j] = static_cast<uint32_t>(((lane % CH) ^ stageSwizzle<CH>(j * RPI + lane / CH)) * 16);
  const uint32_t rowLimit = static_cast<uint32_t>(inRows);   // the launcher keeps inRows * row bytes below 4 GiB
  const uintptr_t zeroBase = reinterpret_cast<uintptr_t>(zeros);

  const TileOrder order(tileBlocks, static_cast<int>((liveOutRows(numActOut, outRows) + TM - 1) / TM), xcdShift,
                        blockIdx.x & ((1 << xcdShift) - 1));
  for (int local = blockIdx.x >> xcdShift; local < order.count(); local += gridDim.x >> xcdShift) {
    const int tile = order.tile(local);
    const int64_t row0 = static_cast<int64_t>(tile) * TM + wave * WM;
    auto nbrOfTap = [&](int tap) __attribute__((always_inline)) {
      return nbr + static_cast<int64_t>(tapMirror ? kVol - 1 - tap : tap) * nbrPitch;
    };

    // Taps that occur among the rows this pipeline serves: the workgroup's tile when the weights stream through
    // shared buffers (every wavefront then walks the same steps, barrier by barrier), the wavefront's own rows
    // when the weights are resident.  A tap none of those rows has is not walked at all: no index load, no
    // weight slice, no gather, no MFMA.  Kernel volumes beyond 64 walk every tap.
    const bool sparseTaps = kVol <= 64;
    unsigned long long present = 0;
    if (sparseTaps) {
      if (tileMasks) {  // one mask per 64 output rows, written next to the table
        constexpr int PER = RESIDENT ? 1 : TM / 64;
        const int64_t firstMask = RESIDENT ? row0 / 64 : static_cast<int64_t>(tile) * PER;
        const int64_t nMasks = (outRows + 63) / 64;
        unsigned long long m = (lane < PER && firstMask + lane < nMasks) ? tileMasks[firstMask + lane] : 0ull;
#pragma unroll
        for (int off = 1; off < PER; off <<= 1) m |= __shfl_xor(m, off, 64);
        present = m;
      } else {
        int64_t row = row0 + (lane & (WM - 1));
        if (row >= outRows) row = outRows - 1;
        unsigned long long mine = 0;
        for (int t0 = 0; t0 < kVol; t0 += 8) {
          uint32_t v[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) v[q] = static_cast<uint32_t>(nbrOfTap(t0 + q < kVol ? t0 + q : kVol - 1)[row]);
#pragma unroll
          for (int q = 0; q < 8; ++q)
            if (t0 + q < kVol && __ballot(v[q] < rowLimit) != 0ull) mine |= 1ull << (t0 + q);
        }
        present = mine;
        if (!RESIDENT) {  // union over the workgroup, through each wavefront's (still idle) index slots
          if (lane == 0) {
            idxLds[0] = static_cast<int32_t>(mine);
            idxLds[1] = static_cast<int32_t>(mine >> 32);
          }
          __syncthreads();
          const int32_t* all = idxLds - wave * NI * 64;
          unsigned long long u = 0;
#pragma unroll
          for (int w = 0; w < WAVES; ++w)
            u |= static_cast<uint32_t>(all[w * NI * 64]) |
                 (static_cast<unsigned long long>(static_cast<uint32_t>(all[w * NI * 64 + 1])) << 32);
          present = u;
          __syncthreads();  // every wavefront has read the masks before the first index load overwrites them
        }
      }
      present = static_cast<unsigned long long>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(present))) |
                (static_cast<unsigned long long>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(present >> 32)))
                 << 32);
    }
    const int steps = (sparseTaps ? __popcll(present) : kVol) * KS;
    // Four walks over the present taps, one per consumer (index loads, weight loads, row gathers, resident weight
    // reads); each consumer asks for its steps in order, so a walk only ever moves forward.
    struct Walk {
      unsigned long long rem;
      int tap, part;
    };
    auto walkNext = [&](Walk& w) __attribute__((always_inline)) -> int {  // step id of the walk's next step
      if (w.part == 0) {
        if (sparseTaps) {
          w.tap = __builtin_ctzll(w.rem);
          w.rem &= w.rem - 1;
        } else {
          ++w.tap;
        }
      }
      const int s = w.tap * KS + w.part;
      w.part = w.part + 1 == KS ? 0 : w.part + 1;
      return s;
    };
    Walk walkIndex{present, -1, 0}, walkWeights{present, -1, 0}, walkRows{present, -1, 0}, walkMul{present, -1, 0};

    // `seq` counts the steps actually walked (it picks the ring slots), `s` is the step id (it picks the data)
    auto issueIndex = [&](int seq) __attribute__((always_inline)) {
      const int s = walkNext(walkIndex);
      int64_t row = row0 + lane;
      if (row >= outRows) row = outRows - 1;
      __builtin_amdgcn_global_load_lds(nbrOfTap(s / KS) + row, idxLds + (seq & (NI - 1)) * 64, 4, 0, 0);
    };
    auto issueWeights = [&](int seq) __attribute__((always_inline)) {
      const int t = walkNext(walkWeights);
      const u32x4* wk = reinterpret_cast<const u32x4*>(wf) + static_cast<size_t>(t) * WCH;
      const int buf = seq % NWB;
#pragma unroll
      for (int q = 0; q < WL; ++q) {
        const int base = (q * THREADS + wave * 64) % WCH;  // wavefronts past the slice repeat a part of it: same bytes
        __builtin_amdgcn_global_load_lds(wk + base + lane, wLds + buf * WCH + base, 16, 0, 0);
      }
    };
    // Branch-free addresses: an absent neighbour (-1) or a row index past the input compares as a huge unsigned
    // number and selects the zero row; rows past outRows repeat the last row's neighbours and are never stored.
    auto issueRows = [&](int seq, int slot) __attribute__((always_inline)) {
      const int t = walkNext(walkRows);
      const int32_t* ix = idxLds + (seq & (NI - 1)) * 64;
      uint32_t src[GL];
#pragma unroll
      for (int j = 0; j < GL; ++j) src[j] = static_cast<uint32_t>(ix[j * RPI + lane / CH]);
      const uintptr_t inBase = reinterpret_cast<uintptr_t>(in) + static_cast<uint32_t>((t % KS) * CS * ES);
#pragma unroll
      for (int j = 0; j < GL; ++j) {
        const uintptr_t row = inBase + static_cast<uint64_t>(src[j] * static_cast<uint32_t>(CIN * ES));
        const uintptr_t a = (src[j] < rowLimit ? row : zeroBase) + chunkOff[j];
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(a), stage + slot * SLOTS + j * 64, 16, 0, 0);
      }
    };

    // prologue: indices and rows of the first NS steps, the first two weight slices, indices of the next three steps
    for (int t = 0; t < NS && t < steps; ++t) issueIndex(t);
    if (!RESIDENT) {
      if (steps > 0) issueWeights(0);
      if (steps > 1) issueWeights(1);
    }
    waitVmcnt<0>();
    for (int t = 0; t < NS && t < steps; ++t) issueRows(t, t);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // index slots are reused by the next three steps
    for (int t = NS; t < NS + 3 && t < steps; ++t) issueIndex(t);
    waitVmcnt<0>();
    if (!RESIDENT) __syncthreads();

    Acc acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int n = 0; n < NT; ++n) acc[m][n] = Acc{0, 0, 0, 0};

    // Row fragments of a step are read from LDS at the end of the step before (its rows have landed by then and
    // belong to this wavefront alone), so those reads overlap the tail of the MFMAs and the barrier instead of
    // standing in front of the next step's MFMAs.
    F rows[MT][KK], rowsNext[MT][KK];
    auto readRows = [&](F (&dst)[MT][KK], int fromSlot) __attribute__((always_inline)) {
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int n = m * 16 + r16;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          if constexpr (WIDE) {
            dst[m][kk] = stage[fromSlot * SLOTS + n * CH + ((kk * 4 + kgrp) ^ stageSwizzle<CH>(n))];
          } else {
            const u32x2* s2 = reinterpret_cast<const u32x2*>(stage + fromSlot * SLOTS + n * CH + ((kgrp >> 1) ^ stageSwizzle<CH>(n)));
            dst[m][kk] = s2[kgrp & 1];
          }
        }
      }
    };
    readRows(rows, 0);
    asm volatile("" ::: "memory");

    int slot = 0, wbuf = 0;
    // one step; `cur` holds its row fragments, `nxt` receives those of the step after (the caller swaps the two
    // from step to step, so no fragment is ever copied)
    auto step = [&](int a, F (&cur)[MT][KK], F (&nxt)[MT][KK]) __attribute__((always_inline)) {
      const bool steady = a + NS + 3 < steps;
      if (steady) issueIndex(a + NS + 3);
      if (!RESIDENT && a + 2 < steps) issueWeights(a + 2);
      // every fragment of the step - rows, then weights - is requested before the first MFMA, so the LDS pipe
      // works from the first cycle of the step and the MFMAs start as the fragments arrive
      const F* wTap = reinterpret_cast<const F*>(wLds + (RESIDENT ? walkNext(walkMul) : wbuf) * WCH);
      F wts[KK][NT];
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
#pragma unroll
        for (int n = 0; n < NT; ++n) wts[kk][n] = wTap[(kk * NT + n) * 64 + lane];
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
        for (int n = 0; n < NT; ++n) {
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            if constexpr (WIDE) {
              acc[m][n] = Mfma<T>::k32(wts[kk][n], cur[m][kk], acc[m][n]);
            } else {
              acc[m][n] = Mfma<T>::k16(wts[kk][n], cur[m][kk], acc[m][n]);
            }
          }
          if (kk == 0 && n == 0 && a + NS < steps) {
            // the row fragments of this slot were read a step ago and have just been multiplied: refill it
            issueRows(a + NS, slot);
          }
        }
      }
      if (steady) {
        waitVmcnt<X>();
      } else {
        // the last steps issue fewer loads: count what may stay in flight behind the ones step a+1 needs
        auto issued = [&](int s_) __attribute__((always_inline)) {
          return (s_ + NS + 3 < steps ? 1 : 0) + (s_ + 2 < steps ? WL : 0) + (s_ + NS < steps ? GL : 0);
        };
        int allowed = 0;
        if (a + 1 < steps) {
          allowed = 63;
          if (a + 1 >= NS) {  // rows of step a+1 left in step a+1-NS, the last loads of that step
            int r = 0;
            for (int s_ = a + 2 - NS; s_ <= a; ++s_) r += issued(s_);
            allowed = r < allowed ? r : allowed;
          }
          if (!RESIDENT && a >= 1) {  // weights of step a+1 left in step a-1, before that step's rows
            const int w = (a - 1 + NS < steps ? GL : 0) + issued(a);
            allowed = w < allowed ? w : allowed;
          }
          if (a + 1 + NS < steps && a >= 2) {  // indices of step a+1+NS left first in step a-2
            const int i_ = issued(a - 2) - 1 + issued(a - 1) + issued(a);
            allowed = i_ < allowed ? i_ : allowed;
          }
        }
        if (allowed >= X) waitVmcnt<X>();
        else if (allowed >= PER_STEP - 1) waitVmcnt<cmin(PER_STEP - 1, 63)>();
        else if (allowed >= GL) waitVmcnt<cmin(GL, 63)>();
        else waitVmcnt<0>();
      }
      slot = slot + 1 == NS ? 0 : slot + 1;
      wbuf = wbuf + 1 == NWB ? 0 : wbuf + 1;
      if (a + 1 < steps) readRows(nxt, slot);
      // Compiler fence: the weight-fragment reads of the next step stay behind these reads in program order.  LDS
      // reads return in order, so the first MFMA of a step (which waits for a weight fragment) then implies that
      // every row fragment of the slot has left LDS, and the slot may be refilled right after it.
      asm volatile("" ::: "memory");
      // a bare barrier: __syncthreads() would also drain every load in flight, i.e. the whole prefetch
      if (!RESIDENT) __builtin_amdgcn_s_barrier();
    };
    for (int a = 0; a < steps; a += 2) {
      step(a, rows, rowsNext);
      if (a + 1 < steps) step(a + 1, rowsNext, rows);
    }

    // epilogue: bias, ReLU, rounding; rows leave through the stage area as contiguous lines
    const float* biasRow = bias ? bias : reinterpret_cast<const float*>(zeros);  // the zero row doubles as "no bias"
    float4v biasV[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) biasV[n] = *reinterpret_cast<const float4v*>(biasRow + n * 16 + kgrp * 4);
    if constexpr (LDS_EPILOGUE) {
      unsigned char* sb = reinterpret_cast<unsigned char*>(stage);
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int n_ = m * 16 + r16;
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          const int col = n * 16 + kgrp * 4;
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[j] = acc[m][n][j] + biasV[n][j];
            if (relu) v[j] = v[j] > 0.f ? v[j] : 0.f;
          }
          T packed[4] = {static_cast<T>(v[0]), static_cast<T>(v[1]), static_cast<T>(v[2]), static_cast<T>(v[3])};
          const int oc = (col >> 3) ^ stageSwizzle<OCH>(n_);
          *reinterpret_cast<u32x2*>(sb + (n_ * OCH + oc) * 16 + (kgrp & 1) * 8) = __builtin_bit_cast(u32x2, packed);
        }
      }
      constexpr int ORPI = 64 / OCH;
#pragma unroll
      for (int j = 0; j < WM / ORPI; ++j) {
        const int n_ = j * ORPI + lane / OCH;
        const int c = lane % OCH;
        const u32x4 v = stage[n_ * OCH + (c ^ stageSwizzle<OCH>(n_))];
        const int64_t row = row0 + n_;
        if (row < outRows) *reinterpret_cast<u32x4*>(out + static_cast<size_t>(row) * COUT + c * 8) = v;
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the stage is free again before the next tile's rows land
    } else if constexpr (ES == 1) {
      // int8: t = float(acc) * m[c]; t += bq[c]; round to nearest even; clamp (lo = 0 with the fused ReLU)
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int64_t row = row0 + m * 16 + r16;
        if (row >= outRows) continue;
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          const int col = n * 16 + kgrp * 4;
          uint32_t packed = 0;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            float t = static_cast<float>(acc[m][n][j]) * requantM[col + j];
            t = t + biasV[n][j];
            float q = __builtin_rintf(t);
            q = __builtin_fminf(127.f, __builtin_fmaxf(relu ? 0.f : -128.f, q));
            packed |= (static_cast<uint32_t>(static_cast<int>(q)) & 0xFFu) << (8 * j);
          }
          *reinterpret_cast<uint32_t*>(out + static_cast<size_t>(row) * COUT + col) = packed;
        }
      }
    } else {
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int64_t row = row0 + m * 16 + r16;
        if (row >= outRows) continue;
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          const int col = n * 16 + kgrp * 4;
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[j] = acc[m][n][j] + biasV[n][j];
            if (relu) v[j] = v[j] > 0.f ? v[j] : 0.f;
          }
          T packed[4] = {static_cast<T>(v[0]), static_cast<T>(v[1]), static_cast<T>(v[2]), static_cast<T>(v[3])};
          *reinterpret_cast<u32x2*>(out + static_cast<size_t>(row) * COUT + col) = __builtin_bit_cast(u32x2, packed);
        }
      }
    }
  }
}

constexpr size_t kLdsLimit = 160 * 1024;

// Compute units of the device the process runs on and log2 of the number of XCDs they are spread over, read once
// from the runtime.  Workgroups are dealt to the XCDs of a partition round-robin, and the tile orders of the
// kernels above follow that: a gfx950 XCD has 32 active compute units, so a whole MI355X reports 256 = 8 XCDs and
// its partition modes 128 / 64 / 32 = 4 / 2 / 1.
struct ChipLayout {
  int cus;
  int xcdShift;
};
inline ChipLayout chipLayout() {
  static const ChipLayout layout = [] {
    int dev = 0, cus = 256;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
      cus = prop.multiProcessorCount;
    const int xcds = cus / 32;
    return ChipLayout{cus, xcds >= 8 ? 3 : (xcds >= 4 ? 2 : (xcds >= 2 ? 1 : 0))};
  }();
  return layout;
}

template <int CIN, int COUT>
constexpr size_t mfmaLds(int kVol, int rows, size_t elem) {
  return static_cast<size_t>(2) * CIN * COUT * elem + static_cast<size_t>(kVol) * rows * 4 +
         (static_cast<size_t>(kVol) + 4) * 4;
}

template <class K>
int32_t grantLds(K kernel, size_t lds, std::atomic<size_t>* granted) {
  // dynamic LDS beyond 64 KiB has to be requested per kernel; two threads that both find it not yet granted both
  // request it, which is harmless
  if (lds > granted->load(std::memory_order_acquire)) {
    D3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(kLdsLimit)));
    granted->store(kLdsLimit, std::memory_order_release);
  }
  return D3D_OK;
}

template <class T, int CIN, int COUT, int MT, int WAVES>
int32_t launchMfmaTile(const ConvArgs& a, hipStream_t stream) {
  constexpr int TM = 16 * MT * WAVES;
  const size_t lds = mfmaLds<CIN, COUT>(a.kVol, TM, sizeof(T));
  if (lds > kLdsLimit) {
    setError("conv: kernel volume %d too large for the MFMA kernel", a.kVol);
    return D3D_ERR_UNSUPPORTED;
  }
  static std::atomic<size_t> granted{64 * 1024};
  const int32_t rc = grantLds(&convMfma<T, CIN, COUT, MT, WAVES>, lds, &granted);
  if (rc != D3D_OK) return rc;
  const int tiles = static_cast<int>((a.outRows + TM - 1) / TM);
  const ChipLayout chip = chipLayout();
  const int nXcd = 1 << chip.xcdShift;
  const int perXcd = (tiles + nXcd - 1) / nXcd;
  hipLaunchKernelGGL((convMfma<T, CIN, COUT, MT, WAVES>), dim3(static_cast<unsigned>(perXcd * nXcd)), dim3(64 * WAVES),
                     lds, stream, static_cast<const T*>(a.in), static_cast<T*>(a.out),
                     static_cast<const T*>(a.weightsMfma), a.bias, a.nbr, a.nbrPitch > 0 ? a.nbrPitch : a.outRows,
                     a.tapMirror, static_cast<const T*>(a.zeros), a.kVol, a.inRows, a.outRows, a.relu, tiles,
                     chip.xcdShift);
  return D3D_OK;
}

template <class T, int CIN, int COUT, int CROW = CIN>
int32_t launchMfmaResident(const ConvArgs& a, hipStream_t stream) {
  constexpr int WAVES = 16;
  const size_t lds = static_cast<size_t>(a.kVol) * CIN * COUT * sizeof(T) + static_cast<size_t>(WAVES) * a.kVol * 16 * 4;
  static std::atomic<size_t> granted{64 * 1024};
  const int32_t rc = grantLds(&convMfmaResident<T, CIN, COUT, WAVES, CROW>, lds, &granted);
  if (rc != D3D_OK) return rc;
  const int groups = static_cast<int>((a.outRows + 15) / 16);
  // persistent workgroups: as many as fit on the CUs at this LDS footprint, but no more than there is work
  const ChipLayout chip = chipLayout();
  const int nXcd = 1 << chip.xcdShift;
  int perCu = static_cast<int>(kLdsLimit / (lds + 1024));
  if (perCu < 1) perCu = 1;
  if (perCu > 2) perCu = 2;  // 16 wavefronts each
  int blocks = chip.cus / nXcd * nXcd * perCu;
  const int needed = (groups + WAVES - 1) / WAVES;
  if (blocks > needed) blocks = (needed + nXcd - 1) / nXcd * nXcd;
  if (blocks < nXcd) blocks = nXcd;
  hipLaunchKernelGGL((convMfmaResident<T, CIN, COUT, WAVES, CROW>), dim3(static_cast<unsigned>(blocks)), dim3(64 * WAVES),
                     lds, stream, static_cast<const T*>(a.in), static_cast<T*>(a.out),
                     static_cast<const T*>(a.weightsMfma), a.bias, a.requantM, a.nbr,
                     a.nbrPitch > 0 ? a.nbrPitch : a.outRows, a.tapMirror, static_cast<const T*>(a.zeros), a.kVol,
                     a.inRows, a.outRows, a.relu, groups, chip.xcdShift, a.numActOut, a.rowChannels);
  return D3D_OK;
}

template <class T, int CIN, int COUT, int KS, int MT, int WAVES, int NS, bool RESIDENT>
int32_t launchStagedCfg(const ConvArgs& a, hipStream_t stream) {
  constexpr int CH = CIN / KS * static_cast<int>(sizeof(T)) / 16;
  constexpr int WM = 16 * MT, TM = WM * WAVES;
  constexpr int WCH = CIN / KS * COUT * static_cast<int>(sizeof(T)) / 16;
  const size_t lds = static_cast<size_t>(RESIDENT ? a.kVol * KS : 3) * WCH * 16 + static_cast<size_t>(WAVES) * 4 * 256 +
                     static_cast<size_t>(WAVES) * NS * WM * CH * 16;
  if (lds > kLdsLimit) return D3D_ERR_UNSUPPORTED;  // the caller falls back
  if (static_cast<uint64_t>(a.inRows) * CIN * sizeof(T) >= (1ull << 32)) return D3D_ERR_UNSUPPORTED;  // 32-bit row offsets
  static std::atomic<size_t> granted{64 * 1024};
  const int32_t rc = grantLds(&convStaged<T, CIN, COUT, KS, MT, WAVES, NS, RESIDENT>, lds, &granted);
  if (rc != D3D_OK) return rc;
  const int tiles = static_cast<int>((a.outRows + TM - 1) / TM);
  const ChipLayout chip = chipLayout();
  const int nXcd = 1 << chip.xcdShift;
  int blocks = (tiles + nXcd - 1) / nXcd * nXcd;
  if (RESIDENT) {  // persistent workgroups share one weight load
    int perCu = static_cast<int>(kLdsLimit / lds);
    if (perCu > 2) perCu = 2;
    if (blocks > chip.cus / nXcd * nXcd * perCu) blocks = chip.cus / nXcd * nXcd * perCu;
  }
  hipLaunchKernelGGL((convStaged<T, CIN, COUT, KS, MT, WAVES, NS, RESIDENT>), dim3(static_cast<unsigned>(blocks)),
                     dim3(64 * WAVES), lds, stream, static_cast<const T*>(a.in), static_cast<T*>(a.out),
                     static_cast<const T*>(a.weightsMfma), a.bias, a.requantM, a.nbr,
                     a.nbrPitch > 0 ? a.nbrPitch : a.outRows, a.tapMirror, a.tileMasks, static_cast<const T*>(a.zeros),
                     a.kVol, a.inRows, a.outRows, a.relu, tiles, chip.xcdShift, a.numActOut);
  return D3D_OK;
}

// Configuration of the staged kernel: rows per wavefront (16*MT), wavefronts, stage depth, weights resident or
// streamed.  `a.staged` (tests, tuning) = MT | WAVES << 8 | NS << 16 | resident << 24; 0 = choose here.
template <class T, int CIN, int COUT>
int32_t launchStaged(const ConvArgs& a, hipStream_t stream) {
  constexpr bool SMALL = CIN * COUT <= 1024;  // 27 taps of weights fit beside the stages
  constexpr int ROWB = CIN * static_cast<int>(sizeof(T));
  constexpr int KS = ROWB > 128 ? ROWB / 128 : 1;  // at most 128 bytes of a row are staged per step
  int cfg = a.staged;
  if (cfg == 0) {  // measured on the layers of a VoxelNet backbone (120k voxels)
    if (CIN == 16 && sizeof(T) == 2) return D3D_ERR_UNSUPPORTED;  // 32-byte rows: the register-gather kernels are faster
    if (CIN * COUT >= 16384) cfg = 2 | 8 << 8 | 3 << 16;
    else if (CIN * COUT >= 8192 || CIN * COUT == 2048) cfg = 2 | 8 << 8 | 2 << 16;
    else cfg = 4 | 8 << 8 | 2 << 16;
  }
  switch (cfg) {
    case 4 | 8 << 8 | 2 << 16: if constexpr (CIN * COUT < 8192) return launchStagedCfg<T, CIN, COUT, KS, 4, 8, 2, false>(a, stream); break;
    case 2 | 8 << 8 | 3 << 16: return launchStagedCfg<T, CIN, COUT, KS, 2, 8, 3, false>(a, stream);
    case 2 | 8 << 8 | 2 << 16: return launchStagedCfg<T, CIN, COUT, KS, 2, 8, 2, false>(a, stream);
    case 4 | 4 << 8 | 2 << 16: return launchStagedCfg<T, CIN, COUT, KS, 4, 4, 2, false>(a, stream);
    case 4 | 4 << 8 | 3 << 16: return launchStagedCfg<T, CIN, COUT, KS, 4, 4, 3, false>(a, stream);
    case 4 | 8 << 8 | 3 << 16 | 1 << 24: if constexpr (SMALL) return launchStagedCfg<T, CIN, COUT, KS, 4, 8, 3, true>(a, stream); break;
    case 2 | 8 << 8 | 3 << 16 | 1 << 24: if constexpr (SMALL) return launchStagedCfg<T, CIN, COUT, KS, 2, 8, 3, true>(a, stream); break;
  }
  return D3D_ERR_UNSUPPORTED;
}

// Does the resident-weight kernel take the layer: every tap's weights and 16 wavefronts' table slices in LDS,
// two workgroups per CU.
inline bool residentFits(int kVol, int cin, int cout, size_t elemBytes) {
  const size_t allTaps = static_cast<size_t>(kVol) * cin * cout * elemBytes;
  return allTaps <= 56 * 1024 && kVol <= 128 && allTaps + static_cast<size_t>(16) * kVol * 16 * 4 <= kLdsLimit;
}

// Small layers keep every tap's weights in LDS (convMfmaResident).  Large layers stream one tap's weights at a
// time through LDS for 8 (or 4) wavefronts; more rows per wavefront (MT) amortise that stream.
template <class T, int CIN, int COUT>
int32_t launchMfmaOne(const ConvArgs& a, hipStream_t stream) {
  if (a.rowChannels > 0 && a.rowChannels < CIN) {  // narrow rows read as stored: the resident kernel only
    if constexpr (CIN == 16 && (COUT == 16 || COUT == 32)) {
      if (residentFits(a.kVol, CIN, COUT, sizeof(T))) return launchMfmaResident<T, CIN, COUT, -1>(a, stream);
    }
    return D3D_ERR_UNSUPPORTED;
  }
  if constexpr (CIN * COUT >= 512) {
    if (a.staged >= 0) {
      const int32_t rc = launchStaged<T, CIN, COUT>(a, stream);
      if (rc != D3D_ERR_UNSUPPORTED) return rc;
    }
  }
  if (residentFits(a.kVol, CIN, COUT, sizeof(T))) return launchMfmaResident<T, CIN, COUT>(a, stream);
  // rows per workgroup = 16 * MT * WAVES
  int mt = 2;
  int waves = 8;
  if (a.tileRows > 0) {  // tuning / test override: tileRows = 16 * MT * WAVES, waves encoded in bit 30
    waves = (a.tileRows & (1 << 30)) ? 4 : 8;
    mt = (a.tileRows & 0xFFFF) / (16 * waves);
    if (mt < 1) mt = 1;
    if (mt > 4) mt = 4;
    if (mt == 3) mt = 2;
    if (mt == 4 && CIN * COUT >= 64 * 128) mt = 2;  // would spill registers
  } else {
    // keep at least two workgroups per CU when the layer is small
    while (mt > 1 && (a.outRows + 16 * mt * waves - 1) / (16 * mt * waves) < 512) mt >>= 1;
  }
  while (mt > 1 && mfmaLds<CIN, COUT>(a.kVol, 16 * mt * waves, sizeof(T)) > kLdsLimit) mt >>= 1;
  if (waves == 4) {
    switch (mt) {
      case 4: return launchMfmaTile<T, CIN, COUT, 4, 4>(a, stream);
      case 2: return launchMfmaTile<T, CIN, COUT, 2, 4>(a, stream);
      default: return launchMfmaTile<T, CIN, COUT, 1, 4>(a, stream);
    }
  }
  switch (mt) {
    case 4: return launchMfmaTile<T, CIN, COUT, 4, 8>(a, stream);
    case 2: return launchMfmaTile<T, CIN, COUT, 2, 8>(a, stream);
    default: return launchMfmaTile<T, CIN, COUT, 1, 8>(a, stream);
  }
}

template <class T, int CIN>
int32_t launchMfmaCout(const ConvArgs& a, hipStream_t stream) {
  switch (a.cout) {
    case 16: return launchMfmaOne<T, CIN, 16>(a, stream);
    case 32: return launchMfmaOne<T, CIN, 32>(a, stream);
    case 64: return launchMfmaOne<T, CIN, 64>(a, stream);
    case 128: return launchMfmaOne<T, CIN, 128>(a, stream);
  }
  return D3D_ERR_UNSUPPORTED;
}

template <class T>
int32_t launchMfma(const ConvArgs& a, hipStream_t stream) {
  switch (a.cin) {
    case 16: return launchMfmaCout<T, 16>(a, stream);
    case 32: return launchMfmaCout<T, 32>(a, stream);
    case 64: return launchMfmaCout<T, 64>(a, stream);
    case 128: return launchMfmaCout<T, 128>(a, stream);
  }
  return D3D_ERR_UNSUPPORTED;
}

// Weights of every tap resident in LDS (register gathers, no barriers): what the 32-channel int8 layers of few
// output channels run, like the 16-channel layers in two-byte types - their rows are as many bytes.
inline bool int8ResidentFits(int kVol, int cin, int cout) { return residentFits(kVol, cin, cout, 1); }

template <int CIN, int COUT, int CROW = CIN>
int32_t launchInt8Resident(const ConvArgs& a, hipStream_t stream) {
  if (int8ResidentFits(a.kVol, CIN, COUT)) return launchMfmaResident<int8_t, CIN, COUT, CROW>(a, stream);
  return D3D_ERR_UNSUPPORTED;
}

template <int CIN>
int32_t launchInt8Cout(const ConvArgs& a, hipStream_t stream) {
  if constexpr (CIN == 32) {
    int32_t rc = D3D_ERR_UNSUPPORTED;
    if (a.rowChannels == 16) {  // rows of 16 stored channels: only the resident kernel reads them as they are
      if (a.cout == 16) return launchInt8Resident<32, 16, 16>(a, stream);
      if (a.cout == 32) return launchInt8Resident<32, 32, 16>(a, stream);
      return D3D_ERR_UNSUPPORTED;
    }
    if (a.rowChannels > 0) return D3D_ERR_UNSUPPORTED;
    if (a.staged == 0) {
      if (a.cout == 16) rc = launchInt8Resident<32, 16>(a, stream);
      if (a.cout == 32 && a.tileMasks == nullptr) rc = launchInt8Resident<32, 32>(a, stream);
      if (a.cout == 64 && a.tileMasks == nullptr) rc = launchInt8Resident<32, 64>(a, stream);
    }
    if (rc != D3D_ERR_UNSUPPORTED) return rc;
  }
  switch (a.cout) {
    case 16: if constexpr (CIN * 16 >= 1024) return launchStaged<int8_t, CIN, 16>(a, stream); break;
    case 32: return launchStaged<int8_t, CIN, 32>(a, stream);
    case 64: return launchStaged<int8_t, CIN, 64>(a, stream);
    case 128: return launchStaged<int8_t, CIN, 128>(a, stream);
  }
  return D3D_ERR_UNSUPPORTED;
}

// (a template so that only the translation unit that calls it instantiates the int8 kernels)
template <class T = int8_t>
int32_t launchInt8(const ConvArgs& a, hipStream_t stream) {
  switch (a.cin) {
    case 32: return launchInt8Cout<32>(a, stream);
    case 64: return launchInt8Cout<64>(a, stream);
    case 128: return launchInt8Cout<128>(a, stream);
  }
  return D3D_ERR_UNSUPPORTED;
}

}  // namespace convk
}  // namespace d3d
