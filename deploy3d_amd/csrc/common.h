// Shared host-side declarations of the sparse-convolution engine: status
// plumbing, the geometry record handed to the rulebook kernels, and the
// launcher entry points implemented in rulebook.hip and conv.hip.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "d3d_spconv.h"

namespace d3d {

constexpr int kMaxSpatial = 4;    // SPConvIdx1d .. SPConvIdx4d
constexpr int kSegment = 128;     // tap segments of the index tensor start on multiples of 128
                                  // (reference: TBSegment, trt/spconv/index.cu:21)
constexpr int kRbThreads = 256;   // rulebook kernels: 4 wavefronts per workgroup

void setError(const char* fmt, ...);
const char* lastError();

#define D3D_HIP_CHECK(expr)                                                              \
  do {                                                                                   \
    hipError_t e_ = (expr);                                                              \
    if (e_ != hipSuccess) {                                                              \
      ::d3d::setError("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
      return D3D_ERR_DEVICE;                                                             \
    }                                                                                    \
  } while (0)

// Geometry of one rulebook, always widened to four spatial dims: missing
// leading dims get kernel 1, stride 1, padding 0, dilation 1 and extent 1, so
// the tap index stays row-major over the real kernel dims
// (reference: kernelOffsetStride, trt/spconv/geometry.h:106-109).
struct RbGeom {
  int nd;                       // real spatial dims (1..4); coordinate rows hold nd+1 ints
  int k[kMaxSpatial];
  int s[kMaxSpatial];
  int p[kMaxSpatial];
  int d[kMaxSpatial];
  int shape[kMaxSpatial + 1];   // output grid: batch, then 4 spatial extents
  int kVol;
  int transpose;
};

// Workspace carve-up of one rulebook build; all offsets in bytes, 256-aligned.
struct RbWorkspace {
  uint32_t slots;         // hash slots (power of two)
  uint32_t nBlocks;       // ceil(cap / kRbThreads)
  size_t table;           // u64 [slots]   key<<32 | value
  size_t ids;             // u32 [slots]   output row of an occupied slot (strided conv only)
  size_t staging;         // u32 [kVol, cap] per (tap, input): slot, then output row, or ~0
  size_t ownPrefix;       // u32 [cap]     (strided conv only)
  size_t blockOwn;        // u32 [nBlocks] (strided conv only)
  size_t cnt;             // u32 [kVol, nBlocks] valid pairs per (tap, workgroup)
  size_t totals;          // u32 [kVol]    valid pairs per tap
  size_t total;           // bytes
};

RbWorkspace planRulebookWorkspace(const RbGeom& g, int64_t cap, bool subM);

// Builds one rulebook on `stream`.  coors [cap, nd+1]; numActIn device int32.
// index [3, rowLen] with rowLen = kVol * (cap + 128).  outCoors / numActOut are
// null for SubM.  Returns a D3D status.
int32_t launchRulebook(const RbGeom& g, bool subM, const int32_t* coors, const int32_t* numActIn, int64_t cap,
                       int32_t maxNumActOut, int32_t* index, int32_t* numIndex, int32_t* outCoors, int32_t* numActOut,
                       void* workspace, size_t workspaceBytes, hipStream_t stream);

// Out-major neighbour table of one rulebook: nbr[tap, row] = gathered input row
// or -1, rows = maxNumActOut.  Built from the index tensor (optionally with the
// gather and scatter rows swapped for an inverse convolution).
int32_t launchBuildNeighbours(const int32_t* index, int64_t rowLen, const int32_t* numIndex, bool inverse, int kVol,
                              int64_t outRows, int32_t* nbr, hipStream_t stream);

struct ConvArgs {
  int32_t dtype;          // D3D_FLOAT / D3D_HALF / D3D_BF16 / D3D_INT8
  int kVol, cin, cout;
  int64_t inRows;         // capacity rows of inFeats
  int64_t outRows;        // maxNumActOut
  const void* in;
  void* out;
  const float* weightsF32;  // device fp32 [kVol, cin, cout], values already rounded to the storage type
  const void* weightsMfma;  // device storage-type [kVol, cout, cin] (reduction dim contiguous) or null
  const float* bias;      // device fp32 [cout] or null
  const float* requantM;  // int8: per-channel multiplier
  const float* requantB;  // int8: per-channel bias in output quanta
  const int32_t* nbr;     // [kVol, outRows]
  int relu;
};

int32_t launchConv(const ConvArgs& a, hipStream_t stream);

// True if the MFMA kernel family covers (dtype, cin, cout); otherwise the
// narrow-channel kernel runs.
bool convUsesMfma(int32_t dtype, int cin, int cout);

}  // namespace d3d
