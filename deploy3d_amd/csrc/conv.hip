// Sparse convolution kernels for gfx950: neighbour-table build, the MFMA
// implicit GEMM for fp16/bf16 channel counts in {16,32,64,128}, and the
// narrow-channel kernel for everything else (odd channel counts, fp32).
//
// The reference computes out = bias, then one tap-major gather-GEMM whose
// epilogue scatter-adds fp16 atomics (trt/spconv/mm.h:35-71,
// trt/spconv/mm/kernel.h:84-179, trt/spconv/mm/output_iterator.h:19-49).
// Here the computation is output-stationary: a workgroup owns a tile of output
// rows, walks the taps that any row of the tile has, gathers the input rows of
// that tap into LDS and accumulates in fp32 registers, so bias, ReLU and the
// final rounding are fused into one plain store per output element: no
// atomics, and a bit-reproducible result.
#include <hip/hip_fp16.h>

#include "common.h"

namespace d3d {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kConvThreads = 256;
constexpr int kTileRows = 64;

// ---------------------------------------------------------------------------
// neighbour table: nbr[tap, out row] = input row or -1
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) nbrFill(int32_t* nbr, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) nbr[i] = -1;
}

__global__ void __launch_bounds__(256)
nbrScatter(const int32_t* __restrict__ gather, const int32_t* __restrict__ scatter, const int32_t* __restrict__ tapRow,
           const int32_t* __restrict__ numIndex, int64_t rowLen, int kVol, int64_t outRows, int32_t* __restrict__ nbr) {
  int64_t n = *numIndex;
  if (n > rowLen) n = rowLen;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; j < n; j += stride) {
    const int32_t t = tapRow[j];
    if (t < 0 || t >= kVol) continue;  // padding slot
    const int32_t o = scatter[j];
    if (o < 0 || o >= outRows) continue;
    nbr[static_cast<int64_t>(t) * outRows + o] = gather[j];
  }
}

// ---------------------------------------------------------------------------
// element helpers
// ---------------------------------------------------------------------------
template <class T> struct Elem;
template <> struct Elem<float> {
  __device__ static float load(const float* p) { return *p; }
  __device__ static void store(float* p, float v) { *p = v; }
};
template <> struct Elem<_Float16> {
  __device__ static float load(const _Float16* p) { return static_cast<float>(*p); }
  __device__ static void store(_Float16* p, float v) { *p = static_cast<_Float16>(v); }  // round-to-nearest-even
};
template <> struct Elem<__bf16> {
  __device__ static float load(const __bf16* p) { return static_cast<float>(*p); }
  __device__ static void store(__bf16* p, float v) { *p = static_cast<__bf16>(v); }
};

// ---------------------------------------------------------------------------
// Narrow-channel / generic kernel.  Workgroup = 64 output rows x up to 64
// output channels; fp32 math on values widened from the storage type; weights
// fp32 [kVol, cin, cout].  Each thread owns 4 adjacent output channels of up to
// 4 rows.  Per tap the gathered rows and the weight slice pass through LDS in
// K chunks of 32.
// ---------------------------------------------------------------------------
constexpr int kNarrowCols = 64;
constexpr int kNarrowK = 32;

template <class T>
__global__ void __launch_bounds__(kConvThreads)
convNarrow(const T* __restrict__ in, T* __restrict__ out, const float* __restrict__ w, const float* __restrict__ bias,
           const int32_t* __restrict__ nbr, int kVol, int cin, int cout, int64_t inRows, int64_t outRows, int relu) {
  __shared__ float xs[kTileRows][kNarrowK + 1];
  __shared__ float ws[kNarrowK][kNarrowCols];
  __shared__ int32_t nb[kTileRows];

  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kTileRows;
  const int col0 = blockIdx.y * kNarrowCols;
  const int colsHere = cout - col0 < kNarrowCols ? cout - col0 : kNarrowCols;
  const int groups = (colsHere + 3) / 4 > 4 ? 16 : 4;  // column groups of 4 channels: 4 or 16
  const int rowsPerPass = kConvThreads / groups;        // 64 or 16
  const int rt = kTileRows / rowsPerPass;               // rows per thread: 1 or 4
  const int tcol = threadIdx.x % groups;
  const int trow = threadIdx.x / groups;

  float acc[4][4];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int col = col0 + tcol * 4 + c;
      acc[r][c] = (bias && col < cout) ? bias[col] : 0.f;
    }

  for (int tap = 0; tap < kVol; ++tap) {
    int32_t mine = -1;
    if (threadIdx.x < kTileRows) {
      const int64_t row = row0 + threadIdx.x;
      if (row < outRows) mine = nbr[static_cast<int64_t>(tap) * outRows + row];
      if (mine >= inRows) mine = -1;
      nb[threadIdx.x] = mine;
    }
    if (!__syncthreads_or(mine >= 0)) continue;  // no row of the tile has this tap
    const float* wt = w + static_cast<size_t>(tap) * cin * cout;
    for (int k0 = 0; k0 < cin; k0 += kNarrowK) {
      const int kc = cin - k0 < kNarrowK ? cin - k0 : kNarrowK;
      for (int e = threadIdx.x; e < kTileRows * kNarrowK; e += kConvThreads) {
        const int r = e / kNarrowK, c = e % kNarrowK;
        const int32_t src = nb[r];
        xs[r][c] = (src >= 0 && c < kc) ? Elem<T>::load(in + static_cast<size_t>(src) * cin + k0 + c) : 0.f;
      }
      for (int e = threadIdx.x; e < kNarrowK * kNarrowCols; e += kConvThreads) {
        const int c = e / kNarrowCols, o = e % kNarrowCols;
        ws[c][o] = (c < kc && o < colsHere) ? wt[static_cast<size_t>(k0 + c) * cout + col0 + o] : 0.f;
      }
      __syncthreads();
      if (tcol * 4 < colsHere) {
        for (int c = 0; c < kc; ++c) {
          const float4v w4 = *reinterpret_cast<const float4v*>(&ws[c][tcol * 4]);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            if (r < rt) {
              const float x = xs[trow + r * rowsPerPass][c];
              acc[r][0] = __builtin_fmaf(x, w4[0], acc[r][0]);
              acc[r][1] = __builtin_fmaf(x, w4[1], acc[r][1]);
              acc[r][2] = __builtin_fmaf(x, w4[2], acc[r][2]);
              acc[r][3] = __builtin_fmaf(x, w4[3], acc[r][3]);
            }
          }
        }
      }
      __syncthreads();
    }
  }

#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (r >= rt) continue;
    const int64_t row = row0 + trow + r * rowsPerPass;
    if (row >= outRows) continue;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int col = col0 + tcol * 4 + c;
      if (col >= cout || tcol * 4 + c >= colsHere) continue;
      float v = acc[r][c];
      if (relu) v = v > 0.f ? v : 0.f;
      Elem<T>::store(out + static_cast<size_t>(row) * cout + col, v);
    }
  }
}

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
  __device__ static float4v k32(const u32x4& a, const u32x4& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  }
  __device__ static float4v k16(const u32x2& a, const u32x2& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4v, a), __builtin_bit_cast(short4v, b), c,
                                                     0, 0, 0);
  }
};

// Fragment type per K step: 8 elements (16 bytes) when CIN >= 32, else 4.
template <int CIN> struct Frag { using type = u32x4; };
template <> struct Frag<16> { using type = u32x2; };

// Weights live in LDS in the same fragment-major order as in global memory:
// fragment (kk, n) of a tap is 64 consecutive lanes' worth of data, so a
// wavefront read is one contiguous, conflict-free sweep.
//
// RESIDENT = true : the weights of ALL taps fit in LDS.  They are loaded once
//   in the prologue; after that every wavefront runs alone (its own active-tap
//   list, no barriers), with the gathers of the next two taps in flight.
// RESIDENT = false: one tap's weights at a time, double-buffered.  The slice of
//   tap t+1 travels global -> registers -> idle LDS buffer while tap t
//   multiplies; one barrier per tap.  Loads are issued oldest-needed-first, because the
//   vector-memory counter retires in order: waiting for a weight slice must
//   not drain the younger gathers behind it.
template <class T, int CIN, int COUT, int MT, bool RESIDENT>
__global__ void __launch_bounds__(kConvThreads)
convMfma(const T* __restrict__ in, T* __restrict__ out, const T* __restrict__ wf, const float* __restrict__ bias,
         const int32_t* __restrict__ nbr, const T* __restrict__ zeros, int kVol, int64_t inRows, int64_t outRows,
         int relu) {
  constexpr int WM = 16 * MT;            // rows per wavefront
  constexpr int TM = 4 * WM;             // rows per workgroup
  constexpr int NT = COUT / 16;          // output-channel tiles
  constexpr int KSTEP = CIN >= 32 ? 32 : 16;
  constexpr int KK = CIN / KSTEP;        // K steps per tap
  constexpr int KG = KSTEP / 4;          // elements per lane per K step
  constexpr int WFRAGS = KK * NT * 64;   // fragments (lane granules) per tap
  constexpr int WCHUNKS = CIN * COUT / 8;  // 16-byte chunks per tap
  constexpr int WPT = (WCHUNKS + kConvThreads - 1) / kConvThreads;
  using F = typename Frag<CIN>::type;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  F* wLds = reinterpret_cast<F*>(smem);  // RESIDENT: [kVol][WFRAGS]; else [2][WFRAGS]
  int32_t* nbT = reinterpret_cast<int32_t*>(smem + static_cast<size_t>(RESIDENT ? kVol : 2) * CIN * COUT * sizeof(T));
  int32_t* tapList = nbT + kVol * TM;    // (!RESIDENT) active taps of the tile, then their count

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kgrp = lane >> 4;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * TM;
  const int32_t* nb = nbT + wave * WM;   // this wavefront's columns of the [kVol][TM] neighbour tile

  // neighbour tile
  if (!RESIDENT)
    for (int t = tid; t <= kVol; t += kConvThreads) tapList[t] = 0;
  if (RESIDENT) {  // all weights, once
    const u32x4* src = reinterpret_cast<const u32x4*>(wf);
    u32x4* dst = reinterpret_cast<u32x4*>(wLds);
    for (int e = tid; e < kVol * WCHUNKS; e += kConvThreads) dst[e] = src[e];
  } else {
    __syncthreads();
  }
  for (int e = tid; e < kVol * TM; e += kConvThreads) {
    const int tap = e / TM, r = e % TM;
    const int64_t row = row0 + r;
    int32_t src = row < outRows ? nbr[static_cast<int64_t>(tap) * outRows + row] : -1;
    if (src >= inRows) src = -1;
    nbT[e] = src;
    if (!RESIDENT && src >= 0) tapList[tap] = 1;
  }
  __syncthreads();

  float4v acc[MT][NT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[m][n] = float4v{0.f, 0.f, 0.f, 0.f};

  // Rows without this tap read a row of zeros (one cached line for the whole device) instead of branching
  // or selecting afterwards: nothing touches the gathered registers until the MFMAs that consume them, so
  // the loads of a tap issue back to back and stay in flight across the MFMAs of the taps before it.
  auto gatherRows = [&](int tap, F (&dst)[MT][KK]) __attribute__((always_inline)) {
    int32_t src[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) src[m] = nb[tap * TM + m * 16 + r16];
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

  if constexpr (RESIDENT) {
    // taps that occur among this wavefront's rows (wavefront-uniform masks)
    unsigned long long active[2] = {0ull, 0ull};
    for (int tap = 0; tap < kVol; ++tap) {
      bool any = false;
      for (int r = lane; r < WM; r += 64) any = any || nb[tap * TM + r] >= 0;
      if (__ballot(any)) active[tap >> 6] |= 1ull << (tap & 63);
    }
    auto nextTap = [&]() __attribute__((always_inline)) -> int {
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
    // Three register sets: while tap t multiplies, the gathers of t+1 and t+2 are in flight.  The sets
    // rotate through loop-carried copies, which pins each gather to the iteration that issues it.  Past
    // the last tap the pipeline re-gathers the last tap (harmless, cached) instead of branching.
    int tNow = nextTap();
    if (tNow >= 0) {
      int last = tNow;
      int tNext = nextTap();
      gatherRows(tNow, bufA);
      gatherRows(tNext >= 0 ? (last = tNext) : last, bufB);
      while (tNow >= 0) {
        const int tFuture = nextTap();
        gatherRows(tFuture >= 0 ? (last = tFuture) : last, bufC);
        __builtin_amdgcn_sched_barrier(0);  // keep the requests ahead of the MFMAs they are meant to overlap
        multiply(wLds + static_cast<size_t>(tNow) * WFRAGS, bufA);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) {
            bufA[m][kk] = bufB[m][kk];
            bufB[m][kk] = bufC[m][kk];
          }
        tNow = tNext;
        tNext = tFuture;
      }
    }
  } else {
    if (tid == 0) {  // compact the flags into a list in place (slot n <= t is written after flag t was read)
      int n = 0;
      for (int t = 0; t < kVol; ++t)
        if (tapList[t]) tapList[n++] = t;
      tapList[kVol] = n;
    }
    __syncthreads();
    const int nActive = tapList[kVol];
    if (nActive > 0) {
      // indices past the end of the list are clamped to the last tap: the pipeline then re-requests data it
      // already has (cache hits) instead of branching around loads, which keeps every load unconditional
      auto tapAt = [&](int a) __attribute__((always_inline)) { return tapList[a < nActive ? a : nActive - 1]; };
      auto loadWeights = [&](int a, u32x4 (&dst)[WPT]) __attribute__((always_inline)) {
        const u32x4* wk = reinterpret_cast<const u32x4*>(wf + static_cast<size_t>(tapAt(a)) * CIN * COUT);
#pragma unroll
        for (int q = 0; q < WPT; ++q) {
          const int e = tid + q * kConvThreads;
          dst[q] = wk[(WCHUNKS % kConvThreads == 0 || e < WCHUNKS) ? e : 0];
        }
      };
      auto storeWeights = [&](int buf, const u32x4 (&src)[WPT]) __attribute__((always_inline)) {
        u32x4* dst = reinterpret_cast<u32x4*>(wLds + buf * WFRAGS);
#pragma unroll
        for (int q = 0; q < WPT; ++q) {
          const int e = tid + q * kConvThreads;
          if (WCHUNKS % kConvThreads == 0 || e < WCHUNKS) dst[e] = src[q];
        }
      };
      {
        u32x4 wreg[WPT];
        loadWeights(0, wreg);
        gatherRows(tapAt(0), bufA);
        gatherRows(tapAt(1), bufB);
        storeWeights(0, wreg);
      }
      __syncthreads();
      // One tap per iteration: tap a multiplies while the weights of a+1 and the rows of a+2 are requested.
      // The weights are requested first, so waiting for them leaves the younger gathers in flight; the row
      // sets rotate through loop-carried copies, which pins each gather to the iteration that issues it.
      for (int a = 0; a < nActive; ++a) {
        u32x4 wreg[WPT];
        loadWeights(a + 1, wreg);
        gatherRows(tapAt(a + 2), bufC);
        __builtin_amdgcn_sched_barrier(0);  // keep the requests ahead of the MFMAs they are meant to overlap
        multiply(wLds + (a & 1) * WFRAGS, bufA);
        __builtin_amdgcn_sched_barrier(0);
        storeWeights((a + 1) & 1, wreg);
        __syncthreads();
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) {
            bufA[m][kk] = bufB[m][kk];
            bufB[m][kk] = bufC[m][kk];
          }
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

constexpr size_t kLdsLimit = 160 * 1024;

template <class T, int CIN, int COUT, int MT, bool RESIDENT>
int32_t launchMfmaTile(const ConvArgs& a, hipStream_t stream) {
  constexpr int TM = 64 * MT;
  const size_t lds = static_cast<size_t>(RESIDENT ? a.kVol : 2) * CIN * COUT * sizeof(T) +
                     static_cast<size_t>(a.kVol) * TM * sizeof(int32_t) + (static_cast<size_t>(a.kVol) + 1) * 4;
  if (lds > kLdsLimit) {
    setError("conv: kernel volume %d too large for the MFMA kernel", a.kVol);
    return D3D_ERR_UNSUPPORTED;
  }
  static size_t granted = 64 * 1024;  // dynamic LDS beyond 64 KiB has to be requested per kernel
  if (lds > granted) {
    D3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&convMfma<T, CIN, COUT, MT, RESIDENT>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kLdsLimit)));
    granted = kLdsLimit;
  }
  const dim3 grid(static_cast<unsigned>((a.outRows + TM - 1) / TM));
  hipLaunchKernelGGL((convMfma<T, CIN, COUT, MT, RESIDENT>), grid, dim3(kConvThreads), lds, stream,
                     static_cast<const T*>(a.in), static_cast<T*>(a.out), static_cast<const T*>(a.weightsMfma), a.bias,
                     a.nbr, static_cast<const T*>(a.zeros), a.kVol, a.inRows, a.outRows, a.relu);
  return D3D_OK;
}

// Rows per wavefront (16*MT): more rows amortise the weight fragments over more MFMAs; fewer rows give
// more workgroups per CU to hide the gather latency and to fill 256 CUs.
template <class T, int CIN, int COUT>
int32_t launchMfmaOne(const ConvArgs& a, hipStream_t stream) {
  const size_t allTaps = static_cast<size_t>(a.kVol) * CIN * COUT * sizeof(T);
  const bool resident = allTaps <= 56 * 1024 && a.kVol <= 128;
  int mt = resident ? 2 : 4;
  if (a.tileRows > 0) {
    mt = a.tileRows / 64;
  } else {
    while (mt > 1 && (a.outRows + 64 * mt - 1) / (64 * mt) < 512) mt >>= 1;
  }
  auto ldsFor = [&](int m) {
    return (resident ? allTaps : 2 * static_cast<size_t>(CIN) * COUT * sizeof(T)) +
           static_cast<size_t>(a.kVol) * 64 * m * 4 + (static_cast<size_t>(a.kVol) + 1) * 4;
  };
  while (mt > 1 && ldsFor(mt) > kLdsLimit) mt >>= 1;
  if (resident) {
    switch (mt) {
      case 4: return launchMfmaTile<T, CIN, COUT, 4, true>(a, stream);
      case 2: return launchMfmaTile<T, CIN, COUT, 2, true>(a, stream);
      default: return launchMfmaTile<T, CIN, COUT, 1, true>(a, stream);
    }
  }
  switch (mt) {
    case 4: return launchMfmaTile<T, CIN, COUT, 4, false>(a, stream);
    case 2: return launchMfmaTile<T, CIN, COUT, 2, false>(a, stream);
    default: return launchMfmaTile<T, CIN, COUT, 1, false>(a, stream);
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

template <class T>
int32_t launchNarrow(const ConvArgs& a, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>((a.outRows + kTileRows - 1) / kTileRows),
                  static_cast<unsigned>((a.cout + kNarrowCols - 1) / kNarrowCols));
  hipLaunchKernelGGL(convNarrow<T>, grid, dim3(kConvThreads), 0, stream, static_cast<const T*>(a.in),
                     static_cast<T*>(a.out), a.weightsF32, a.bias, a.nbr, a.kVol, a.cin,
                     a.cout, a.inRows, a.outRows, a.relu);
  return D3D_OK;
}

bool isMfmaChannels(int c) { return c == 16 || c == 32 || c == 64 || c == 128; }

}  // namespace

bool convUsesMfma(int32_t dtype, int cin, int cout) {
  return (dtype == D3D_HALF || dtype == D3D_BF16) && isMfmaChannels(cin) && isMfmaChannels(cout);
}

int32_t launchBuildNeighbours(const int32_t* index, int64_t rowLen, const int32_t* numIndex, bool inverse, int kVol,
                              int64_t outRows, int32_t* nbr, hipStream_t stream) {
  const int64_t n = static_cast<int64_t>(kVol) * outRows;
  if (n <= 0) return D3D_OK;
  int fillBlocks = static_cast<int>((n + 255) / 256);
  if (fillBlocks > 4096) fillBlocks = 4096;
  hipLaunchKernelGGL(nbrFill, dim3(fillBlocks), dim3(256), 0, stream, nbr, n);
  const int32_t* gather = inverse ? index + rowLen : index;
  const int32_t* scatter = inverse ? index : index + rowLen;
  int blocks = static_cast<int>((rowLen + 255) / 256);
  if (blocks > 4096) blocks = 4096;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(nbrScatter, dim3(blocks), dim3(256), 0, stream, gather, scatter, index + 2 * rowLen, numIndex,
                     rowLen, kVol, outRows, nbr);
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

int32_t launchConv(const ConvArgs& a, hipStream_t stream) {
  if (a.outRows <= 0) return D3D_OK;
  int32_t rc = D3D_ERR_UNSUPPORTED;
  const bool aligned = ((reinterpret_cast<uintptr_t>(a.in) | reinterpret_cast<uintptr_t>(a.out)) & 15) == 0;
  if (convUsesMfma(a.dtype, a.cin, a.cout) && aligned && a.weightsMfma && a.zeros) {
    rc = a.dtype == D3D_HALF ? launchMfma<_Float16>(a, stream) : launchMfma<__bf16>(a, stream);
  } else {
    switch (a.dtype) {
      case D3D_FLOAT: rc = launchNarrow<float>(a, stream); break;
      case D3D_HALF: rc = launchNarrow<_Float16>(a, stream); break;
      case D3D_BF16: rc = launchNarrow<__bf16>(a, stream); break;
      default: setError("conv: dtype %d not implemented", a.dtype); return D3D_ERR_UNSUPPORTED;
    }
  }
  if (rc != D3D_OK) return rc;
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

}  // namespace d3d
