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
//   weights: [kVol, COUT, CIN] (reduction dim contiguous), storage type T
//   tile   : 64 output rows x COUT, 4 wavefronts arranged WAVES_M x WAVES_N
//   LDS    : gathered rows As[64][CIN+8], weight slice Bs[COUT][CIN+8],
//            neighbour tile nbT[kVol][64]
// Operand layout of v_mfma_f32_16x16x32 (and 16x16x16): lane l supplies row
// (A) or column (B) l%16 and the (l/16)-th group of 8 (4) consecutive K
// values; it receives column l%16, rows 4*(l/16)..+3 of the 16x16 result.
// ---------------------------------------------------------------------------
template <class T> struct Mfma;
template <> struct Mfma<_Float16> {
  using Vec8 = half8;
  __device__ static float4v k32(const Vec8& a, const Vec8& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  __device__ static float4v k16(const uint2& a, const uint2& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, a), __builtin_bit_cast(half4, b), c, 0, 0,
                                                 0);
  }
};
template <> struct Mfma<__bf16> {
  using Vec8 = bf16x8;
  __device__ static float4v k32(const Vec8& a, const Vec8& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static float4v k16(const uint2& a, const uint2& b, const float4v& c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4v, a), __builtin_bit_cast(short4v, b), c,
                                                     0, 0, 0);
  }
};

template <class T, int CIN, int COUT, int WAVES_M>
__global__ void __launch_bounds__(kConvThreads)
convMfma(const T* __restrict__ in, T* __restrict__ out, const T* __restrict__ wt, const float* __restrict__ bias,
         const int32_t* __restrict__ nbr, int kVol, int64_t inRows, int64_t outRows, int relu) {
  constexpr int TM = kTileRows;
  constexpr int WAVES_N = 4 / WAVES_M;
  constexpr int WM = TM / WAVES_M, WN = COUT / WAVES_N;
  constexpr int MT = WM / 16, NT = WN / 16;
  constexpr int PITCH = CIN + 8;         // elements; 16 bytes of padding staggers LDS banks
  constexpr int CHUNKS = CIN / 8;        // 16-byte chunks per row
  static_assert(MT >= 1 && NT >= 1, "tile split");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* As = reinterpret_cast<T*>(smem);
  T* Bs = As + TM * PITCH;
  int32_t* nbT = reinterpret_cast<int32_t*>(Bs + COUT * PITCH);
  uint32_t* tapAny = reinterpret_cast<uint32_t*>(nbT + kVol * TM);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int waveM = wave % WAVES_M, waveN = wave / WAVES_M;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * TM;

  // neighbour tile + which taps occur in it
  for (int t = tid; t < kVol; t += kConvThreads) tapAny[t] = 0;
  __syncthreads();
  for (int e = tid; e < kVol * TM; e += kConvThreads) {
    const int tap = e / TM, r = e % TM;
    const int64_t row = row0 + r;
    int32_t src = row < outRows ? nbr[static_cast<int64_t>(tap) * outRows + row] : -1;
    if (src >= inRows) src = -1;
    nbT[e] = src;
    if (src >= 0) tapAny[tap] = 1;
  }
  __syncthreads();

  float4v acc[MT][NT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[m][n] = float4v{0.f, 0.f, 0.f, 0.f};

  const int arow = lane & 15, kgrp = lane >> 4;

  for (int tap = 0; tap < kVol; ++tap) {
    if (!tapAny[tap]) continue;  // workgroup-uniform
    __syncthreads();             // previous tap's MFMA reads are done
    for (int e = tid; e < TM * CHUNKS; e += kConvThreads) {
      const int r = e / CHUNKS, c = e % CHUNKS;
      const int32_t src = nbT[tap * TM + r];
      uint4 v = make_uint4(0, 0, 0, 0);
      if (src >= 0) v = *reinterpret_cast<const uint4*>(in + static_cast<size_t>(src) * CIN + c * 8);
      *reinterpret_cast<uint4*>(As + r * PITCH + c * 8) = v;
    }
    const T* wk = wt + static_cast<size_t>(tap) * COUT * CIN;
    for (int e = tid; e < COUT * CHUNKS; e += kConvThreads) {
      const int r = e / CHUNKS, c = e % CHUNKS;
      *reinterpret_cast<uint4*>(Bs + r * PITCH + c * 8) = *reinterpret_cast<const uint4*>(wk + r * CIN + c * 8);
    }
    __syncthreads();
    if constexpr (CIN >= 32) {
#pragma unroll
      for (int kk = 0; kk < CIN / 32; ++kk) {
        typename Mfma<T>::Vec8 a[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
          a[m] = *reinterpret_cast<const typename Mfma<T>::Vec8*>(As + (waveM * WM + m * 16 + arow) * PITCH + kk * 32 +
                                                                  kgrp * 8);
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          const auto b = *reinterpret_cast<const typename Mfma<T>::Vec8*>(Bs + (waveN * WN + n * 16 + arow) * PITCH +
                                                                          kk * 32 + kgrp * 8);
#pragma unroll
          for (int m = 0; m < MT; ++m) acc[m][n] = Mfma<T>::k32(a[m], b, acc[m][n]);
        }
      }
    } else {
      uint2 a[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m)
        a[m] = *reinterpret_cast<const uint2*>(As + (waveM * WM + m * 16 + arow) * PITCH + kgrp * 4);
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const uint2 b = *reinterpret_cast<const uint2*>(Bs + (waveN * WN + n * 16 + arow) * PITCH + kgrp * 4);
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m][n] = Mfma<T>::k16(a[m], b, acc[m][n]);
      }
    }
  }

  // epilogue: bias, ReLU, one rounding to the storage type
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    const int col = waveN * WN + n * 16 + arow;
    const float bv = bias ? bias[col] : 0.f;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t row = row0 + waveM * WM + m * 16 + kgrp * 4 + j;
        if (row >= outRows) continue;
        float v = acc[m][n][j] + bv;
        if (relu) v = v > 0.f ? v : 0.f;
        Elem<T>::store(out + static_cast<size_t>(row) * COUT + col, v);
      }
    }
  }
}

template <class T, int CIN, int COUT>
int32_t launchMfmaOne(const ConvArgs& a, hipStream_t stream) {
  constexpr int WAVES_M = COUT >= 64 ? 2 : 4;
  const size_t lds = static_cast<size_t>(kTileRows + COUT) * (CIN + 8) * sizeof(T) +
                     static_cast<size_t>(a.kVol) * kTileRows * 4 + static_cast<size_t>(a.kVol) * 4;
  if (lds > 160 * 1024) {
    setError("conv: %zu bytes of LDS needed (kVol %d too large for the MFMA kernel)", lds, a.kVol);
    return D3D_ERR_UNSUPPORTED;
  }
  if (lds > 64 * 1024) {  // beyond the default dynamic-LDS limit: raise it for this instantiation
    D3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&convMfma<T, CIN, COUT, WAVES_M>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
  }
  const dim3 grid(static_cast<unsigned>((a.outRows + kTileRows - 1) / kTileRows));
  hipLaunchKernelGGL((convMfma<T, CIN, COUT, WAVES_M>), grid, dim3(kConvThreads), lds, stream,
                     static_cast<const T*>(a.in), static_cast<T*>(a.out), static_cast<const T*>(a.weightsMfma), a.bias,
                     a.nbr, a.kVol, a.inRows, a.outRows, a.relu);
  return D3D_OK;
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
  if (convUsesMfma(a.dtype, a.cin, a.cout) && aligned && a.weightsMfma) {
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
