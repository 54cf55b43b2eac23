// Sparse rows -> dense bird's-eye-view feature map.
//
// The dense map is [B, C, Z, Y, X] (handed on as [B, C*Z, Y, X]); voxel row i
// with coordinate (b, z, y, x) fills out[b, :, z, y, x] and every other cell is
// zero (reference: kernel::densify and the memset before it,
// trt/spconv/bev_densify_trt.cu:22-35, :160-174).
//
// The reference clears the map and then scatters one channel at a time, so a
// row of C values lands in C different cache lines.  Here the map is produced
// output-stationary instead: a cell -> row table is built first (4 bytes per
// cell), then every workgroup owns 64 consecutive cells of one (b, z) plane,
// pulls the rows of its occupied cells through LDS and writes whole runs of
// 64 cells per channel, zeros included.  Each output byte is written exactly
// once and no clearing pass is needed.
#include "common.h"

namespace d3d {
namespace {

constexpr int kTile = 64;          // cells per workgroup, consecutive in y*X + x
constexpr int kChunkBytes = 128;   // bytes of a feature row handled by one workgroup
constexpr int kPitch = kChunkBytes + 4;  // LDS bytes per cell: an odd number of dwords

__global__ __launch_bounds__(256) void dzMapClear(int32_t* __restrict__ map, int64_t cells) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < cells) map[i] = -1;
}

// The highest row wins a cell named twice, which is what a serial pass over
// the rows leaves behind.  Rows outside the grid are dropped.
__global__ __launch_bounds__(256) void dzMapRows(const int32_t* __restrict__ coors,
                                                 const int32_t* __restrict__ numAct, int32_t cap, int B, int Z, int Y,
                                                 int X, int32_t* __restrict__ map) {
  const int32_t n = min(max(*numAct, 0), cap);
  const int32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int4 c = reinterpret_cast<const int4*>(coors)[i];
  if (static_cast<unsigned>(c.x) >= static_cast<unsigned>(B) || static_cast<unsigned>(c.y) >= static_cast<unsigned>(Z) ||
      static_cast<unsigned>(c.z) >= static_cast<unsigned>(Y) || static_cast<unsigned>(c.w) >= static_cast<unsigned>(X))
    return;
  const int64_t cell = ((static_cast<int64_t>(c.x) * Z + c.y) * Y + c.z) * X + c.w;
  atomicMax(map + cell, i);
}

// grid: (tiles of a plane, B*Z planes, channel chunks).  E = bytes per element,
// PACK = cells written by one store (PACK*E == 4, or PACK == 1), VEC = rows are
// fetched in 16-byte pieces.
template <int E, int PACK, bool VEC>
__global__ __launch_bounds__(256) void dzGather(const uint8_t* __restrict__ feats, const int32_t* __restrict__ map,
                                                uint8_t* __restrict__ out, int C, int Z, int64_t YX) {
  __shared__ int32_t rows[kTile];
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTile * kPitch];

  const int t = threadIdx.x;
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kTile;
  const int plane = blockIdx.y;
  const int b = plane / Z, z = plane % Z;
  const int c0 = blockIdx.z * (kChunkBytes / E);          // first channel of this chunk
  const int cc = min(kChunkBytes / E, C - c0);            // channels in this chunk
  const int ccBytes = cc * E;
  const size_t rowBytes = static_cast<size_t>(C) * E;

  if (t < kTile) rows[t] = (p0 + t < YX) ? map[static_cast<int64_t>(plane) * YX + p0 + t] : -1;
  __syncthreads();

  if constexpr (VEC) {
    // 8 lanes x 16 bytes per cell, 32 cells per sweep
    for (int u = t; u < kTile * (kChunkBytes / 16); u += 256) {
      const int cell = u / (kChunkBytes / 16), q = u % (kChunkBytes / 16);
      if (q * 16 >= ccBytes) continue;
      const int r = rows[cell];
      uint4 v = make_uint4(0, 0, 0, 0);
      if (r >= 0) v = *reinterpret_cast<const uint4*>(feats + r * rowBytes + static_cast<size_t>(c0) * E + q * 16);
      uint32_t* dst = reinterpret_cast<uint32_t*>(tile + cell * kPitch + q * 16);
      dst[0] = v.x;
      dst[1] = v.y;
      dst[2] = v.z;
      dst[3] = v.w;
    }
  } else {
    for (int u = t; u < kTile * ccBytes; u += 256) {
      const int cell = u / ccBytes, q = u % ccBytes;
      const int r = rows[cell];
      tile[cell * kPitch + q] = r >= 0 ? feats[r * rowBytes + static_cast<size_t>(c0) * E + q] : uint8_t(0);
    }
  }
  __syncthreads();

  constexpr int kGroups = kTile / PACK;  // stores per channel
  for (int u = t; u < cc * kGroups; u += 256) {
    const int ch = u / kGroups, cell0 = (u % kGroups) * PACK;
    const int64_t p = p0 + cell0;
    if (p >= YX) continue;
    const size_t at = (((static_cast<size_t>(b) * C + c0 + ch) * Z + z) * YX + p) * E;
    const uint8_t* src = tile + cell0 * kPitch + ch * E;
    if constexpr (E == 4) {
      *reinterpret_cast<uint32_t*>(out + at) = *reinterpret_cast<const uint32_t*>(src);
    } else if constexpr (E == 2) {
      if constexpr (PACK == 2) {
        const uint32_t lo = *reinterpret_cast<const uint16_t*>(src);
        const uint32_t hi = *reinterpret_cast<const uint16_t*>(src + kPitch);
        *reinterpret_cast<uint32_t*>(out + at) = lo | (hi << 16);
      } else {
        *reinterpret_cast<uint16_t*>(out + at) = *reinterpret_cast<const uint16_t*>(src);
      }
    } else {
      if constexpr (PACK == 4) {
        const uint32_t v = uint32_t(src[0]) | (uint32_t(src[kPitch]) << 8) | (uint32_t(src[2 * kPitch]) << 16) |
                           (uint32_t(src[3 * kPitch]) << 24);
        *reinterpret_cast<uint32_t*>(out + at) = v;
      } else {
        out[at] = src[0];
      }
    }
  }
}

template <int E>
void launchGather(const DensifyArgs& a, const int32_t* map, dim3 grid, hipStream_t stream) {
  const int64_t yx = static_cast<int64_t>(a.Y) * a.X;
  const bool vec = (static_cast<size_t>(a.C) * E) % 16 == 0 && reinterpret_cast<uintptr_t>(a.feats) % 16 == 0;
  constexpr int kPack = 4 / E;
  const bool pack = kPack > 1 && yx % kPack == 0 && reinterpret_cast<uintptr_t>(a.out) % 4 == 0;
  const uint8_t* f = static_cast<const uint8_t*>(a.feats);
  uint8_t* o = static_cast<uint8_t*>(a.out);
#define D3D_DZ(P, V) hipLaunchKernelGGL((dzGather<E, P, V>), grid, dim3(256), 0, stream, f, map, o, a.C, a.Z, yx)
  if (pack) {
    if (vec) D3D_DZ(kPack, true); else D3D_DZ(kPack, false);
  } else {
    if (vec) D3D_DZ(1, true); else D3D_DZ(1, false);
  }
#undef D3D_DZ
}

}  // namespace

size_t densifyWorkspaceBytes(int64_t B, int64_t Z, int64_t Y, int64_t X) {
  return static_cast<size_t>(B * Z * Y * X) * sizeof(int32_t);
}

int32_t launchDensify(const DensifyArgs& a, hipStream_t stream) {
  const int64_t cells = static_cast<int64_t>(a.B) * a.Z * a.Y * a.X;
  if (cells == 0 || a.C == 0) return D3D_OK;  // nothing to write
  const int64_t yx = static_cast<int64_t>(a.Y) * a.X;
  const int64_t tiles = (yx + kTile - 1) / kTile;
  const int64_t planes = static_cast<int64_t>(a.B) * a.Z;
  const int E = a.elemBytes;
  const int64_t chunks = (static_cast<int64_t>(a.C) * E + kChunkBytes - 1) / kChunkBytes;
  if (E != 1 && E != 2 && E != 4) {
    setError("BEVDensify: elements of %d bytes not implemented", E);
    return D3D_ERR_UNSUPPORTED;
  }
  if (planes > 65535 || chunks > 65535 || cells >= (int64_t(1) << 31)) {
    setError("BEVDensify: grid [%d, %d, %d, %d] x %d channels exceeds the launch limits", a.B, a.Z, a.Y, a.X, a.C);
    return D3D_ERR_BAD_ARG;
  }
  if (a.workspaceBytes < static_cast<size_t>(cells) * 4 || !a.workspace) {
    setError("BEVDensify: workspace of %zu bytes, %zu needed", a.workspaceBytes, static_cast<size_t>(cells) * 4);
    return D3D_ERR_WORKSPACE;
  }
  if (reinterpret_cast<uintptr_t>(a.coors) % 16 != 0) {
    setError("BEVDensify: coordinate rows must start on a 16-byte boundary");
    return D3D_ERR_BAD_ARG;
  }
  int32_t* map = static_cast<int32_t*>(a.workspace);
  hipLaunchKernelGGL(dzMapClear, dim3(static_cast<unsigned>((cells + 255) / 256)), dim3(256), 0, stream, map, cells);
  if (a.cap > 0)
    hipLaunchKernelGGL(dzMapRows, dim3(static_cast<unsigned>((a.cap + 255) / 256)), dim3(256), 0, stream, a.coors,
                       a.numAct, a.cap, a.B, a.Z, a.Y, a.X, map);
  const dim3 grid(static_cast<unsigned>(tiles), static_cast<unsigned>(planes), static_cast<unsigned>(chunks));
  if (E == 4) launchGather<4>(a, map, grid, stream);
  else if (E == 2) launchGather<2>(a, map, grid, stream);
  else launchGather<1>(a, map, grid, stream);
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

}  // namespace d3d
