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

#include <type_traits>

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
typedef int32_t int4v __attribute__((ext_vector_type(4)));

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
           const int32_t* __restrict__ numIndex, int64_t rowLen, int kVol, int64_t outRows, int64_t inRows,
           int32_t* __restrict__ nbr) {
  int64_t n = *numIndex;
  if (n > rowLen) n = rowLen;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; j < n; j += stride) {
    const int32_t t = tapRow[j];
    if (t < 0 || t >= kVol) continue;  // padding slot
    const int32_t o = scatter[j];
    if (o < 0 || o >= outRows) continue;
    // a gather row outside the input is no neighbour: the table holds -1 or rows that exist, nothing else (the
    // kernels that turn an entry into a buffer offset rely on that)
    const int32_t i = gather[j];
    if (i < 0 || i >= inRows) continue;
    // An index tensor that names two inputs for one (tap, output) - duplicate coordinates, a tensor of other
    // origin - keeps the higher input row: one neighbour per (tap, output), the same one on every run.
    atomicMax(&nbr[static_cast<int64_t>(t) * outRows + o], i);
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
           const int32_t* __restrict__ nbr, int64_t nbrPitch, int tapMirror, int kVol, int cin, int cout,
           int64_t inRows, int64_t outRows, int relu) {
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
      if (row < outRows) mine = nbr[static_cast<int64_t>(tapMirror ? kVol - 1 - tap : tap) * nbrPitch + row];
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

template <class T>
int32_t launchNarrow(const ConvArgs& a, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>((a.outRows + kTileRows - 1) / kTileRows),
                  static_cast<unsigned>((a.cout + kNarrowCols - 1) / kNarrowCols));
  hipLaunchKernelGGL(convNarrow<T>, grid, dim3(kConvThreads), 0, stream, static_cast<const T*>(a.in),
                     static_cast<T*>(a.out), a.weightsF32, a.bias, a.nbr, a.nbrPitch > 0 ? a.nbrPitch : a.outRows,
                     a.tapMirror, a.kVol, a.cin, a.cout, a.inRows, a.outRows, a.relu);
  return D3D_OK;
}

// ---------------------------------------------------------------------------
// Narrow layers proper (at most 32 input and 32 output channels, any storage type; fp32 math): lanes across the
// output channels, several rows per wavefront.  A wavefront holds 64 / CP rows at a time (CP = 16 or 32 lanes per
// row); lane (r, co) accumulates channel co of row r over all taps and input channels.  The 16 or 32 lanes of a
// row read the same input values - one address per row, served as a broadcast, 128 bits at a time when the rows
// allow it - and consecutive LDS words of the weight slice W[tap][ci][:], which every row shares; a tap that none
// of the wavefront's rows has is skipped after one ballot, and the table entries of 27 taps are requested
// together so that their latencies overlap.  Nothing is staged per tap and there is no barrier after the weights
// have landed: such a layer moves a few megabytes, and what it costs is the chain of dependent loads.
// ---------------------------------------------------------------------------
template <class T, int CP>
__global__ void __launch_bounds__(kConvThreads)
convNarrowRows(const T* __restrict__ in, T* __restrict__ out, const float* __restrict__ w, const float* __restrict__ bias,
               const int32_t* __restrict__ nbr, int64_t nbrPitch, int tapMirror, int kVol, int cin, int cout,
               int64_t inRows, int64_t outRows, int relu, int rowsPerWave) {
  extern __shared__ __attribute__((aligned(16))) float wl[];  // [kVol][cin][CP], channels past cout zero
  const int total = kVol * cin * CP;
  for (int e = threadIdx.x; e < total; e += kConvThreads) {
    const int co = e % CP, tc = e / CP;
    wl[e] = co < cout ? w[static_cast<size_t>(tc) * cout + co] : 0.f;
  }
  __syncthreads();
  constexpr int RP = 64 / CP;
  constexpr int kBatch = 27;  // table entries requested together: a whole 3x3x3 kernel
  const int lane = threadIdx.x & 63, r = lane / CP, co = lane % CP;
  const int64_t first = (static_cast<int64_t>(blockIdx.x) * (kConvThreads / 64) + (threadIdx.x >> 6)) * rowsPerWave;
  const float b = (bias && co < cout) ? bias[co] : 0.f;
  const bool wide = std::is_same<T, float>::value && (cin & 3) == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0;
  for (int64_t row0 = first; row0 < first + rowsPerWave && row0 < outRows; row0 += RP) {
    const int64_t row = row0 + r;
    const bool valid = row < outRows;
    float acc = b;
    for (int tap0 = 0; tap0 < kVol; tap0 += kBatch) {
      int32_t ids[kBatch];
#pragma unroll
      for (int q = 0; q < kBatch; ++q) {
        const int tap = tap0 + q;
        ids[q] = (valid && tap < kVol) ? nbr[static_cast<int64_t>(tapMirror ? kVol - 1 - tap : tap) * nbrPitch + row] : -1;
      }
#pragma unroll
      for (int q = 0; q < kBatch; ++q) {
        const int32_t idx = ids[q];
        const bool has = idx >= 0 && idx < inRows;
        if (__ballot(has) == 0ull) continue;  // wavefront-uniform
        if (has) {
          const float* wt = wl + static_cast<size_t>(tap0 + q) * cin * CP + co;
          const T* x = in + static_cast<size_t>(idx) * cin;
          if (wide) {
            for (int ci = 0; ci < cin; ci += 4) {
              const float4v v = *reinterpret_cast<const float4v*>(reinterpret_cast<const float*>(x) + ci);
              acc = __builtin_fmaf(v[0], wt[(ci + 0) * CP], acc);
              acc = __builtin_fmaf(v[1], wt[(ci + 1) * CP], acc);
              acc = __builtin_fmaf(v[2], wt[(ci + 2) * CP], acc);
              acc = __builtin_fmaf(v[3], wt[(ci + 3) * CP], acc);
            }
          } else {
            for (int ci = 0; ci < cin; ++ci) acc = __builtin_fmaf(Elem<T>::load(x + ci), wt[ci * CP], acc);
          }
        }
      }
    }
    if (relu) acc = acc > 0.f ? acc : 0.f;
    if (valid && co < cout) Elem<T>::store(out + static_cast<size_t>(row) * cout + co, acc);
  }
}

template <class T>
int32_t launchNarrowRows(const ConvArgs& a, hipStream_t stream) {
  const int cp = a.cout <= 16 ? 16 : 32;
  const size_t lds = static_cast<size_t>(a.kVol) * a.cin * cp * sizeof(float);
  if (a.cin > 32 || a.cout > 32 || lds > 64 * 1024) return D3D_ERR_UNSUPPORTED;
  // Small layers: one group of rows per wavefront - the layer is a chain of dependent loads per row, and only many
  // wavefronts hide it (20 000 rows: 22 us at 16 rows per wavefront, 14 us at 4).  Large ones: 16 rows per
  // wavefront, so that the copy of the weights into LDS is shared by more rows.
  const bool large = a.outRows > (1 << 16);
  const int rowsPerWave = large ? 16 : 64 / cp;
  const int64_t rowsPerBlock = static_cast<int64_t>(rowsPerWave) * (kConvThreads / 64);
  const dim3 grid(static_cast<unsigned>((a.outRows + rowsPerBlock - 1) / rowsPerBlock));
  const int64_t pitch = a.nbrPitch > 0 ? a.nbrPitch : a.outRows;
  if (cp == 16)
    hipLaunchKernelGGL((convNarrowRows<T, 16>), grid, dim3(kConvThreads), lds, stream,
                       static_cast<const T*>(a.in), static_cast<T*>(a.out), a.weightsF32, a.bias, a.nbr, pitch,
                       a.tapMirror, a.kVol, a.cin, a.cout, a.inRows, a.outRows, a.relu, rowsPerWave);
  else
    hipLaunchKernelGGL((convNarrowRows<T, 32>), grid, dim3(kConvThreads), lds, stream,
                       static_cast<const T*>(a.in), static_cast<T*>(a.out), a.weightsF32, a.bias, a.nbr, pitch,
                       a.tapMirror, a.kVol, a.cin, a.cout, a.inRows, a.outRows, a.relu, rowsPerWave);
  return D3D_OK;
}

bool isMfmaChannels(int c) { return c == 16 || c == 32 || c == 64 || c == 128; }

// rows of `inBytes` bytes widened to `outBytes` (a multiple of 16) with zeros, so that a narrow first layer
// (5 input channels, say) can run on the MFMA path
__global__ void __launch_bounds__(256)
padRows(const uint8_t* __restrict__ in, int64_t rows, int inBytes, int outBytes, uint8_t* __restrict__ out) {
  const int chunks = outBytes / 16;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; e < rows * chunks; e += stride) {
    const int64_t row = e / chunks;
    const int c0 = static_cast<int>(e % chunks) * 16;
    uint8_t v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) v[j] = c0 + j < inBytes ? in[row * inBytes + c0 + j] : static_cast<uint8_t>(0);
    *reinterpret_cast<u32x4*>(out + row * outBytes + c0) = __builtin_bit_cast(u32x4, v);
  }
}

}  // namespace

bool convUsesMfma(int32_t dtype, int cin, int cout) {
  if (dtype == D3D_INT8) return (cin == 32 || cin == 64 || cin == 128) && isMfmaChannels(cout);
  return (dtype == D3D_HALF || dtype == D3D_BF16) && isMfmaChannels(cin) && isMfmaChannels(cout);
}

int paddedMfmaChannels(int32_t dtype, int cin, int cout) {
  if (!isMfmaChannels(cout) || cin < 1 || cin > 128) return cin;
  if (dtype == D3D_HALF || dtype == D3D_BF16) {
    int c = 16;
    while (c < cin) c *= 2;
    return c;
  }
  if (dtype == D3D_INT8) {  // the int8 MFMA contracts at least 32 channels
    int c = 32;
    while (c < cin) c *= 2;
    return c <= 128 ? c : cin;
  }
  return cin;
}

int32_t launchPadRows(const void* in, int64_t rows, int inBytes, int outBytes, void* out, hipStream_t stream) {
  if (rows <= 0) return D3D_OK;
  int64_t blocks = (rows * (outBytes / 16) + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(padRows, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                     static_cast<const uint8_t*>(in), rows, inBytes, outBytes, static_cast<uint8_t*>(out));
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

int32_t launchBuildNeighbours(const int32_t* index, int64_t rowLen, const int32_t* numIndex, bool inverse, int kVol,
                              int64_t outRows, int64_t inRows, int32_t* nbr, hipStream_t stream) {
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
                     rowLen, kVol, outRows, inRows, nbr);
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

int32_t launchConv(const ConvArgs& a, hipStream_t stream) {
  if (a.outRows <= 0) return D3D_OK;
  int32_t rc = D3D_ERR_UNSUPPORTED;
  const bool aligned = ((reinterpret_cast<uintptr_t>(a.in) | reinterpret_cast<uintptr_t>(a.out)) & 15) == 0;
  if (a.dtype == D3D_INT8) {
    if (!convUsesMfma(a.dtype, a.cin, a.cout) || !aligned || !a.weightsMfma || !a.zeros || !a.requantM) {
      setError("conv: int8 needs 32/64/128 (widened) input channels, 16/32/64/128 output channels, 16-byte aligned "
               "tensors and requantize scales");
      return D3D_ERR_UNSUPPORTED;
    }
    rc = D3D_ERR_UNSUPPORTED;
    if (a.pipe >= 0 && a.staged == 0 && a.tileRows == 0 && a.rowChannels == 0) rc = launchPipeInt8(a, stream);
    if (rc == D3D_ERR_UNSUPPORTED) rc = launchMfmaInt8(a, stream);
    if (rc == D3D_ERR_UNSUPPORTED) setError("conv: int8 layer does not fit the staged kernel (kernel volume %d)", a.kVol);
  } else if (convUsesMfma(a.dtype, a.cin, a.cout) && aligned && a.weightsMfma && a.zeros) {
    rc = D3D_ERR_UNSUPPORTED;
    if (a.pipe >= 0 && a.staged == 0 && a.tileRows == 0)
      rc = a.dtype == D3D_HALF ? launchPipeHalf(a, stream) : launchPipeBf16(a, stream);
    if (rc == D3D_ERR_UNSUPPORTED) rc = a.dtype == D3D_HALF ? launchMfmaHalf(a, stream) : launchMfmaBf16(a, stream);
    if (rc == D3D_ERR_UNSUPPORTED && a.weightsF32 && a.inNarrow) {
      // no MFMA instantiation fits (a kernel volume whose index rows exceed LDS, 7x7x7 at 128 channels say): the
      // narrow kernel takes any kernel volume (the reference accepts any, trt/spconv/mm.h:35-71)
      ConvArgs b = a;
      b.in = a.inNarrow;
      b.cin = a.cinNarrow;
      rc = a.dtype == D3D_HALF ? launchNarrow<_Float16>(b, stream) : launchNarrow<__bf16>(b, stream);
    }
  } else {
    const char* rowsEnv = debugEnv("D3D_CONV_NARROW_ROWS");  // =0: keep the tile kernel (tests)
    const bool rows = !(rowsEnv && rowsEnv[0] == '0');
    switch (a.dtype) {
      case D3D_FLOAT:
        rc = rows ? launchNarrowRows<float>(a, stream) : D3D_ERR_UNSUPPORTED;
        if (rc == D3D_ERR_UNSUPPORTED) rc = launchNarrow<float>(a, stream);
        break;
      case D3D_HALF:
        rc = rows ? launchNarrowRows<_Float16>(a, stream) : D3D_ERR_UNSUPPORTED;
        if (rc == D3D_ERR_UNSUPPORTED) rc = launchNarrow<_Float16>(a, stream);
        break;
      case D3D_BF16:
        rc = rows ? launchNarrowRows<__bf16>(a, stream) : D3D_ERR_UNSUPPORTED;
        if (rc == D3D_ERR_UNSUPPORTED) rc = launchNarrow<__bf16>(a, stream);
        break;
      default: setError("conv: dtype %d not implemented", a.dtype); return D3D_ERR_UNSUPPORTED;
    }
  }
  if (rc != D3D_OK) return rc;
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

}  // namespace d3d
