// Points -> voxels with mean features (the step in front of a sparse backbone).
//
// Reference: voxel_encoder::func::simpleMeanEncoder and its kernels,
// trt/voxel_encoder/simple_mean_trt.cu:26-168.  A point is kept when all its
// features are finite, its batch index is not negative and its cell
//   (b, int((z - zMin) / zSize), int((y - yMin) / ySize), int((x - xMin) / xSize))
// (fp32 arithmetic, conversion truncating toward zero) lies in the grid; every
// occupied cell becomes one output row holding the mean of its points' features,
// its coordinate, and numActOut = min(occupied cells, maxNumActOut).
//
// The reference numbers the voxels in hash-slot order, which depends on the
// races of its insertions.  Here a voxel is represented by the lowest index
// among its points (a 64-bit atomic min on key<<32 | index, so the table's
// races cannot show), and voxels are numbered by a prefix sum over the points
// of "I am my voxel's representative": rows come out in order of first
// appearance, the same on every run, and truncation keeps the voxels that
// appear first.  Sums use fp32 atomic adds like the reference's, so the means
// can differ in the last bits from run to run; coordinates and counts cannot.
#include "common.h"

namespace d3d {
namespace {

constexpr int kVxThreads = 256;
constexpr int kVxItems = 4;
constexpr int kVxChunk = kVxThreads * kVxItems;  // points per workgroup of the ranking pass
constexpr uint32_t kVxNone = 0xFFFFFFFFu;
constexpr unsigned long long kVxEmpty = ~0ull;

// trt/include/common/hash32.h:23-33 (MurmurHash3 finaliser)
__device__ __forceinline__ uint32_t vxMix(uint32_t k) {
  k ^= k >> 16;
  k *= 0x85ebca6bu;
  k ^= k >> 13;
  k *= 0xc2b2ae35u;
  k ^= k >> 16;
  return k;
}

struct VxGeom {
  int B, Z, Y, X;
};

// table = empty, outFeats = 0 (simple_mean_trt.cu:139-143), counts = 0, ticket = 0
__global__ void __launch_bounds__(kVxThreads)
vxReset(unsigned long long* table, int64_t slots, float* outFeats, int64_t nFeats, uint32_t* counts, int64_t nCounts,
        int32_t* numActOut) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  for (int64_t i = tid; i < slots; i += stride) table[i] = kVxEmpty;
  for (int64_t i = tid; i < nFeats; i += stride) outFeats[i] = 0.f;
  for (int64_t i = tid; i < nCounts; i += stride) counts[i] = 0;
  if (tid == 0) *numActOut = 0;
}

// kernel::voxelize (simple_mean_trt.cu:28-60).  pointSlot[i] = the slot of point i's voxel, or none.
__global__ void __launch_bounds__(kVxThreads)
vxInsert(const float* __restrict__ feats, const int32_t* __restrict__ batchIdx, const float* __restrict__ config, int32_t n,
         int C, VxGeom g, unsigned long long* table, uint32_t mask, uint32_t* __restrict__ pointSlot) {
  const int32_t i = blockIdx.x * kVxThreads + threadIdx.x;
  if (i >= n) return;
  const float* f = feats + static_cast<size_t>(i) * C;
  bool ok = true;
  for (int c = 0; c < C; ++c) ok = ok && isfinite(f[c]);
  const int b = batchIdx[i];
  uint32_t slot = kVxNone;
  if (ok && b >= 0 && b < g.B) {
    const int x = static_cast<int>((f[0] - config[0]) / config[3]);
    const int y = static_cast<int>((f[1] - config[1]) / config[4]);
    const int z = static_cast<int>((f[2] - config[2]) / config[5]);
    if (x >= 0 && x < g.X && y >= 0 && y < g.Y && z >= 0 && z < g.Z) {
      const uint32_t key = ((static_cast<uint32_t>(b) * g.Z + z) * g.Y + y) * g.X + x;
      const unsigned long long mine = (static_cast<unsigned long long>(key) << 32) | static_cast<uint32_t>(i);
      uint32_t s = vxMix(key) & mask;
      for (uint32_t tries = 0; tries <= mask; ++tries) {  // at most half the slots are ever taken
        const unsigned long long old = atomicCAS(&table[s], kVxEmpty, mine);
        if (old == kVxEmpty) {
          slot = s;
          break;
        }
        if (static_cast<uint32_t>(old >> 32) == key) {
          if (old > mine) atomicMin(&table[s], mine);
          slot = s;
          break;
        }
        s = (s + 1) & mask;
      }
    }
  }
  pointSlot[i] = slot;
}

// Numbers the voxels: a point that is the lowest of its voxel counts 1.  local[i] = how many such points
// precede i inside its chunk of 1024 points; chunk totals become exclusive chunk bases in the workgroup that
// finishes last (ticket counter, no waiting), which also writes numActOut (simple_mean_trt.cu:149-150, :87).
__global__ void __launch_bounds__(kVxThreads)
vxRank(const unsigned long long* __restrict__ table, const uint32_t* __restrict__ pointSlot, int32_t n,
       uint32_t* __restrict__ local, uint32_t* chunkBase, uint32_t nChunks, uint32_t* ticket, int32_t* numActOut,
       int32_t maxNumActOut) {
  __shared__ uint32_t scratch[kVxThreads / 64];
  __shared__ uint32_t isLast;
  const int32_t first = blockIdx.x * kVxChunk + threadIdx.x * kVxItems;
  uint32_t flag[kVxItems];
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < kVxItems; ++j) {
    const int32_t i = first + j;
    flag[j] = 0;
    if (i < n) {
      const uint32_t s = pointSlot[i];
      if (s != kVxNone && static_cast<uint32_t>(table[s]) == static_cast<uint32_t>(i)) flag[j] = 1;
    }
    mine += flag[j];
  }
  // exclusive prefix over the workgroup
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  uint32_t rank = incl - mine, total = 0;
#pragma unroll
  for (int w = 0; w < kVxThreads / 64; ++w) {
    if (w < wave) rank += scratch[w];
    total += scratch[w];
  }
#pragma unroll
  for (int j = 0; j < kVxItems; ++j) {
    if (flag[j]) local[first + j] = rank;
    rank += flag[j];
  }
  if (threadIdx.x == 0) {
    // the total is published with a returning device-scope atomic (performed where every XCD sees it once the
    // result is back); only then is the ticket taken.  An acquire-release ticket instead (a device-scope release
    // per workgroup) measured 8.2 -> 13.8 us for this kernel on 100 000 points.
    uint32_t old = __hip_atomic_exchange(&chunkBase[blockIdx.x], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(old)::"memory");
    isLast = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nChunks - 1 ? 1u : 0u;
  }
  __syncthreads();
  if (!isLast) return;
  uint32_t running = 0;
  for (uint32_t base = 0; base < nChunks; base += kVxThreads) {
    const uint32_t q = base + threadIdx.x;
    const uint32_t v = q < nChunks ? __hip_atomic_load(&chunkBase[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    uint32_t inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(inc, off, 64);
      if (lane >= off) inc += up;
    }
    __syncthreads();
    if (lane == 63) scratch[wave] = inc;
    __syncthreads();
    uint32_t before = running, sum = 0;
#pragma unroll
    for (int w = 0; w < kVxThreads / 64; ++w) {
      if (w < wave) before += scratch[w];
      sum += scratch[w];
    }
    if (q < nChunks) chunkBase[q] = before + inc - v;
    running += sum;
  }
  if (threadIdx.x == 0)
    *numActOut = static_cast<int32_t>(running < static_cast<uint32_t>(maxNumActOut) ? running : maxNumActOut);
}

// kernel::scatterAddFeats (simple_mean_trt.cu:62-91): sums, point counts, and the coordinate row, written by the
// voxel's representative (refnd.h:56-64 turns the cell offset back into (b, z, y, x)).
__global__ void __launch_bounds__(kVxThreads)
vxAccumulate(const float* __restrict__ feats, int32_t n, int C, VxGeom g, const unsigned long long* __restrict__ table,
             const uint32_t* __restrict__ pointSlot, const uint32_t* __restrict__ local,
             const uint32_t* __restrict__ chunkBase, int32_t maxNumActOut, float* outFeats, uint32_t* counts,
             int32_t* __restrict__ outCoors) {
  const int32_t i = blockIdx.x * kVxThreads + threadIdx.x;
  if (i >= n) return;
  const uint32_t s = pointSlot[i];
  if (s == kVxNone) return;
  const unsigned long long entry = table[s];
  const uint32_t rep = static_cast<uint32_t>(entry);
  const uint32_t id = chunkBase[rep / kVxChunk] + local[rep];
  if (id >= static_cast<uint32_t>(maxNumActOut)) return;
  const float* f = feats + static_cast<size_t>(i) * C;
  float* row = outFeats + static_cast<size_t>(id) * C;
  for (int c = 0; c < C; ++c) unsafeAtomicAdd(row + c, f[c]);
  atomicAdd(counts + id, 1u);
  if (rep == static_cast<uint32_t>(i)) {
    uint32_t off = static_cast<uint32_t>(entry >> 32);
    const uint32_t x = off % g.X;
    off /= g.X;
    const uint32_t y = off % g.Y;
    off /= g.Y;
    const uint32_t z = off % g.Z;
    off /= g.Z;
    reinterpret_cast<int4*>(outCoors)[id] = make_int4(static_cast<int>(off), static_cast<int>(z), static_cast<int>(y),
                                                      static_cast<int>(x));
  }
}

// kernel::meanFeats (simple_mean_trt.cu:93-101)
__global__ void __launch_bounds__(kVxThreads)
vxMean(float* outFeats, const uint32_t* __restrict__ counts, const int32_t* __restrict__ numActOut, int C) {
  const int64_t total = static_cast<int64_t>(*numActOut) * C;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t q = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; q < total; q += stride)
    outFeats[q] = outFeats[q] / static_cast<float>(counts[q / C]);
}

uint32_t pow2AtLeast(uint64_t v) {
  uint32_t p = 1024;
  while (p < v && p < 0x80000000u) p <<= 1;
  return p;
}

size_t alignUp256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

struct VxPlan {
  uint32_t slots, nChunks;
  size_t table, pointSlot, local, chunkBase, counts, ticket, total;
};

VxPlan planVoxelize(int64_t numPts, int64_t maxNumActOut) {
  VxPlan p{};
  const int64_t n = numPts < 1 ? 1 : numPts;
  p.slots = pow2AtLeast(static_cast<uint64_t>(n) * 2);  // the reference's hashSpace = 2 (simple_mean_trt.cu:110)
  p.nChunks = static_cast<uint32_t>((n + kVxChunk - 1) / kVxChunk);
  size_t off = 0;
  p.table = off;
  off = alignUp256(off + static_cast<size_t>(p.slots) * 8);
  p.pointSlot = off;
  off = alignUp256(off + static_cast<size_t>(n) * 4);
  p.local = off;
  off = alignUp256(off + static_cast<size_t>(n) * 4);
  p.chunkBase = off;
  off = alignUp256(off + static_cast<size_t>(p.nChunks) * 4);
  p.counts = off;  // [maxNumActOut] point counts, directly followed by the ticket
  off += static_cast<size_t>(maxNumActOut < 0 ? 0 : maxNumActOut) * 4;
  p.ticket = off;
  off = alignUp256(off + 4);
  p.total = off;
  return p;
}

}  // namespace

size_t voxelizeWorkspaceBytes(int64_t numPts, int64_t maxNumActOut) { return planVoxelize(numPts, maxNumActOut).total; }

int32_t launchVoxelize(const VoxelizeArgs& a, hipStream_t stream) {
  const VxPlan p = planVoxelize(a.numPts, a.maxNumActOut);
  if (!a.workspace || a.workspaceBytes < p.total) {
    setError("SimpleMeanEncoder: workspace of %zu bytes, %zu needed", a.workspaceBytes, p.total);
    return D3D_ERR_WORKSPACE;
  }
  if (reinterpret_cast<uintptr_t>(a.workspace) % 16 != 0 || reinterpret_cast<uintptr_t>(a.outCoors) % 16 != 0) {
    setError("SimpleMeanEncoder: workspace and outCoors must start on 16-byte boundaries");
    return D3D_ERR_BAD_ARG;
  }
  const uint64_t cells = static_cast<uint64_t>(a.B) * a.Z * a.Y * a.X;
  if (cells >= 0xFFFFFFFFull) {
    setError("SimpleMeanEncoder: grid [%d, %d, %d, %d] has more cells than a 32-bit key can name", a.B, a.Z, a.Y, a.X);
    return D3D_ERR_UNSUPPORTED;
  }
  char* ws = static_cast<char*>(a.workspace);
  auto* table = reinterpret_cast<unsigned long long*>(ws + p.table);
  auto* pointSlot = reinterpret_cast<uint32_t*>(ws + p.pointSlot);
  auto* local = reinterpret_cast<uint32_t*>(ws + p.local);
  auto* chunkBase = reinterpret_cast<uint32_t*>(ws + p.chunkBase);
  auto* counts = reinterpret_cast<uint32_t*>(ws + p.counts);
  auto* ticket = reinterpret_cast<uint32_t*>(ws + p.ticket);
  const VxGeom g{a.B, a.Z, a.Y, a.X};
  const int64_t nFeats = static_cast<int64_t>(a.maxNumActOut) * a.C;
  const int64_t resetItems = static_cast<int64_t>(p.slots) + nFeats;
  int64_t resetBlocks = (resetItems + kVxThreads - 1) / kVxThreads;
  if (resetBlocks > 4096) resetBlocks = 4096;
  hipLaunchKernelGGL(vxReset, dim3(static_cast<unsigned>(resetBlocks < 1 ? 1 : resetBlocks)), dim3(kVxThreads), 0, stream,
                     table, static_cast<int64_t>(p.slots), a.outFeats, nFeats, counts,
                     static_cast<int64_t>(a.maxNumActOut) + 1, a.numActOut);
  if (a.numPts > 0 && a.maxNumActOut > 0 && cells > 0) {
    const dim3 perPoint(static_cast<unsigned>((a.numPts + kVxThreads - 1) / kVxThreads));
    hipLaunchKernelGGL(vxInsert, perPoint, dim3(kVxThreads), 0, stream, a.feats, a.batchIdx, a.config,
                       static_cast<int32_t>(a.numPts), a.C, g, table, p.slots - 1, pointSlot);
    hipLaunchKernelGGL(vxRank, dim3(p.nChunks), dim3(kVxThreads), 0, stream, table, pointSlot,
                       static_cast<int32_t>(a.numPts), local, chunkBase, p.nChunks, ticket, a.numActOut, a.maxNumActOut);
    hipLaunchKernelGGL(vxAccumulate, perPoint, dim3(kVxThreads), 0, stream, a.feats, static_cast<int32_t>(a.numPts), a.C,
                       g, table, pointSlot, local, chunkBase, a.maxNumActOut, a.outFeats, counts, a.outCoors);
    int64_t meanBlocks = (nFeats + kVxThreads - 1) / kVxThreads;
    if (meanBlocks > 2048) meanBlocks = 2048;
    hipLaunchKernelGGL(vxMean, dim3(static_cast<unsigned>(meanBlocks)), dim3(kVxThreads), 0, stream, a.outFeats, counts,
                       a.numActOut, a.C);
  }
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

}  // namespace d3d
