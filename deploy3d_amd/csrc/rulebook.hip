// Rulebook (index-pair) builder for gfx950.
//
// Produces the index tensor contract of deploy3d's SPConvIdx{N}d plugin
// (reference: trt/spconv/index.cu:253-476): rows gather / scatter / tap of
// length kVol*(cap+128), pairs laid out tap-major and input-row ascending,
// every tap segment starting on a multiple of 128, every unused slot -1,
// numIndex = end rounded up to 128.
//
// Differences in HOW, all deliberate:
//  * no host read-back of numActIn (index_trt.cu:207-209): grids are sized on
//    the static capacity and every kernel reads the live count on the device;
//  * two occupancy structures.  The default is a dense map of 64-cell bricks of the output grid (second half of
//    this file): voxels are ranked in brick-major order by popcounts and a prefix over the bricks, a probe is a
//    handful of neighbouring 16-byte records, strided outputs need no election and come out sorted.  Grids too
//    large or too sparse for it take the coordinate hash (first half): one 64-bit slot per entry (key<<32 | value)
//    in HBM, claimed with a single 64-bit CAS, so a probe is one 8-byte load;
//  * the per-pair passes run one workgroup per (chunk of 1024 inputs, tap), so all kVol*N probes or inserts of a
//    pass are independent and in flight together;
//  * compaction is a prefix inside the workgroup plus per-(tap, chunk) counts;
//    each workgroup sums the counts of its predecessors itself, so there are
//    no device-wide scan kernels;
//  * hash path: a strided output belongs to the contributing pair with the smallest
//    (input row, tap) code (atomicMin) and outputs are numbered in (tap, input
//    row) order of their owners, which makes the output order deterministic
//    (the reference numbers them by hash-slot order, which depends on CAS races); the
//    strided hash is sized by the real bound on distinct outputs per input
//    (product over dims of the largest number of stride-compatible taps), not
//    by 2*kVol*N slots;
//  * besides the index tensor a build can write what the convolutions read - the pairs in output-major form and
//    the tap masks of 64-row tiles (RbSide) - and can reuse the index tensor and the occupancy map of an earlier
//    build (incremental fill, shared map).
#include <cstdlib>
#include <cstring>

#include "common.h"

namespace d3d {
namespace {

constexpr unsigned long long kEmptySlot = ~0ull;
constexpr uint32_t kNone = 0xFFFFFFFFu;

// MurmurHash3 finaliser, the reference's slot hash (trt/include/common/hash32.h:23-33).
__device__ __forceinline__ uint32_t fmix32(uint32_t k) {
  k ^= k >> 16;
  k *= 0x85ebca6bu;
  k ^= k >> 13;
  k *= 0xc2b2ae35u;
  k ^= k >> 16;
  return k;
}

// Inserts (key, value); on a key that is already present keeps the smaller
// value.  Returns the slot, or kNone if the table is full (cannot happen at
// load factor <= 1/2).  At most `mask + 1` probes, so every lane terminates.
__device__ __forceinline__ uint32_t hashInsertMin(unsigned long long* table, uint32_t mask, uint32_t key,
                                                  uint32_t value) {
  const unsigned long long packed = (static_cast<unsigned long long>(key) << 32) | value;
  uint32_t slot = fmix32(key) & mask;
  for (uint32_t probe = 0; probe <= mask; ++probe) {
    unsigned long long cur = __builtin_nontemporal_load(table + slot);
    if (cur == kEmptySlot) {
      cur = atomicCAS(table + slot, kEmptySlot, packed);
      if (cur == kEmptySlot) return slot;
    }
    if (static_cast<uint32_t>(cur >> 32) == key) {
      // values only ever decrease, so a (possibly stale) smaller value settles it
      if (packed < cur) atomicMin(table + slot, packed);
      return slot;
    }
    slot = (slot + 1) & mask;
  }
  return kNone;
}

__device__ __forceinline__ uint32_t hashLookup(const unsigned long long* table, uint32_t mask, uint32_t key) {
  uint32_t slot = fmix32(key) & mask;
  for (uint32_t probe = 0; probe <= mask; ++probe) {
    const unsigned long long cur = table[slot];
    if (static_cast<uint32_t>(cur >> 32) == key) return static_cast<uint32_t>(cur);
    if (cur == kEmptySlot) return kNone;
    slot = (slot + 1) & mask;
  }
  return kNone;
}

// Loads coordinate row `i` widened to (batch, 4 spatial).
__device__ __forceinline__ void loadCoord(const int32_t* coors, int nd, int64_t i, int c[5]) {
  const int32_t* row = coors + i * (nd + 1);
  if (nd == 3 && (reinterpret_cast<uintptr_t>(coors) & 15) == 0) {  // the common case: one 16-byte load
    const int4 v = *reinterpret_cast<const int4*>(row);
    c[0] = v.x; c[1] = 0; c[2] = v.y; c[3] = v.z; c[4] = v.w;
    return;
  }
  const int pad = kMaxSpatial - nd;
  c[0] = row[0];
#pragma unroll
  for (int dim = 0; dim < kMaxSpatial; ++dim) c[dim + 1] = dim >= pad ? row[1 + dim - pad] : 0;
}

// Loads input row `i`; false if its coordinate lies outside the input grid.  Such a row takes part in no pair, on
// every structure (the reference hashes its linear offset unchecked, so it aliases into another cell there:
// trt/spconv/index.cu:174-182).
__device__ __forceinline__ bool loadInput(const RbGeom& g, const int32_t* coors, int64_t i, int c[5]) {
  loadCoord(coors, g.nd, i, c);
  bool ok = true;
#pragma unroll
  for (int dim = 0; dim <= kMaxSpatial; ++dim) ok = ok && c[dim] >= 0 && c[dim] < g.inShape[dim];
  return ok;
}

__device__ __forceinline__ bool coordInGrid(const RbGeom& g, const int c[5]) {
  bool ok = true;
#pragma unroll
  for (int dim = 0; dim <= kMaxSpatial; ++dim) ok = ok && c[dim] >= 0 && c[dim] < g.shape[dim];
  return ok;
}

__device__ __forceinline__ uint32_t coordOffset(const RbGeom& g, const int c[5]) {
  uint32_t off = static_cast<uint32_t>(c[0]);
#pragma unroll
  for (int dim = 1; dim <= kMaxSpatial; ++dim) off = off * static_cast<uint32_t>(g.shape[dim]) + c[dim];
  return off;
}

// One kernel dim of the tap walk (reference: dimLoop, trt/spconv/geometry.h:28-74).
// Forward: c = in + p - i*d must divide by the stride (C remainder semantics,
// so negative odd numerators drop out); transposed: out = in*s - p + i*d.
__device__ __forceinline__ bool tapDim(const RbGeom& g, int dim, int in, int i, int& out) {
  if (g.transpose) {
    out = in * g.s[dim] - g.p[dim] + i * g.d[dim];
  } else {
    const int c = in + g.p[dim] - i * g.d[dim];
    const int st = g.s[dim];  // uniform: the branches below are scalar
    if (st == 1) {
      out = c;
    } else if (st == 2) {  // an arithmetic shift keeps negative even numerators negative, so the range test drops them
      if (c & 1) return false;
      out = c >> 1;
    } else {
      if (c % st != 0) return false;
      out = c / st;
    }
  }
  return out >= 0 && out < g.shape[dim + 1];
}

__device__ __forceinline__ int liveCount(const int32_t* numActIn, int64_t cap) {
  const int n = *numActIn;
  return n < 0 ? 0 : (n > cap ? static_cast<int>(cap) : n);
}

// Sum over the whole workgroup (kRbThreads threads); every thread gets the result.
__device__ __forceinline__ uint32_t blockSum(uint32_t v, uint32_t* scratch) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  uint32_t total = 0;
#pragma unroll
  for (int w = 0; w < kRbThreads / 64; ++w) total += scratch[w];
  return total;
}

// Exclusive prefix of v over the workgroup in thread order; *total gets the sum.
__device__ __forceinline__ uint32_t blockExclusiveScan(uint32_t v, uint32_t* scratch, uint32_t* total) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  uint32_t incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  __syncthreads();
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  uint32_t waveBase = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < kRbThreads / 64; ++w) {
    if (w < wave) waveBase += scratch[w];
    sum += scratch[w];
  }
  *total = sum;
  return waveBase + incl - v;
}

// Both at once behind one pair of barriers: *sum gets the workgroup sum of `a`, the return value is the exclusive
// prefix of `v` in thread order.  scratch: 2 * kRbThreads / 64 words.
__device__ __forceinline__ uint32_t blockSumAndScan(uint32_t a, uint32_t v, uint32_t* scratch, uint32_t* sum) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  uint32_t incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) a += __shfl_down(a, off, 64);
  __syncthreads();
  if (lane == 63) scratch[wave] = incl;
  if (lane == 0) scratch[kRbThreads / 64 + wave] = a;
  __syncthreads();
  uint32_t waveBase = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kRbThreads / 64; ++w) {
    if (w < wave) waveBase += scratch[w];
    total += scratch[kRbThreads / 64 + w];
  }
  *sum = total;
  return waveBase + incl - v;
}

// ---------------------------------------------------------------------------
// reset: hash slots = EMPTY, index tensor = -1, tap totals = 0.  One streaming
// pass of 16-byte stores (replaces resetHashKernel + the cudaMemsetAsync calls
// of trt/spconv/index.cu:309-314, :352-354).
// ---------------------------------------------------------------------------
// Every pass starts with one of the two reset kernels; besides their own clearing they zero the tile masks of
// the pass and hand the fill state over: fillState[0] (the end of what the previous pass used of the index
// tensor) takes the value the previous pass left in fillState[1].
__device__ __forceinline__ void resetShared(int64_t tid, int64_t stride, unsigned long long* masks, int64_t nMasks,
                                            uint32_t* fillState) {
  for (int64_t i = tid; i < nMasks; i += stride) masks[i] = 0ull;
  if (tid == 0 && fillState) fillState[0] = fillState[1];
}

__global__ void __launch_bounds__(kRbThreads)
rbReset(uint4* table16, int64_t nTable16, int32_t* index, int64_t nIndex, uint32_t* totals, int kVol,
        int32_t* numIndex, unsigned long long* masks, int64_t nMasks, uint32_t* fillState) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  resetShared(tid, stride, masks, nMasks, fillState);
  const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
  for (int64_t i = tid; i < nTable16; i += stride) table16[i] = ones;
  // index tensor: 16-byte body when the base is aligned, scalar head/tail otherwise
  const uintptr_t base = reinterpret_cast<uintptr_t>(index);
  int64_t head = ((16 - (base & 15)) & 15) >> 2;
  if (head > nIndex) head = nIndex;
  const int64_t body16 = index ? (nIndex - head) >> 2 : 0;
  uint4* body = reinterpret_cast<uint4*>(index + head);
  for (int64_t i = tid; i < body16; i += stride) body[i] = ones;
  const int64_t tailStart = head + (body16 << 2);
  if (index) {
    if (tid < head) index[tid] = -1;
    if (tid < nIndex - tailStart) index[tailStart + tid] = -1;
  }
  for (int64_t q = tid; q < kVol; q += stride) totals[q] = 0;
  if (tid == 0) *numIndex = 0;
}

// ---------------------------------------------------------------------------
// All passes below run one workgroup per (input chunk, tap): blockIdx.y is the
// tap, blockIdx.x a chunk of kRbChunk consecutive inputs, 4 per thread.  Every
// (tap, input) item is independent, so the probes and inserts of a pass are all
// in flight together instead of one voxel walking its taps serially.
// ---------------------------------------------------------------------------
constexpr int kRbItems = 4;
constexpr int kRbChunk = kRbThreads * kRbItems;

// Tap index -> per-dim kernel positions (row-major over the kernel dims;
// reference: kernelOffsetStride, trt/spconv/geometry.h:106-109).
__device__ __forceinline__ void tapPositions(const RbGeom& g, int tap, int idx[kMaxSpatial]) {
#pragma unroll
  for (int dim = kMaxSpatial - 1; dim >= 0; --dim) {
    idx[dim] = tap % g.k[dim];
    tap /= g.k[dim];
  }
}

// Output voxel of (input coordinate, tap); false if the tap does not land on
// the output lattice or falls outside the output grid.
__device__ __forceinline__ bool tapTarget(const RbGeom& g, const int c[5], const int idx[kMaxSpatial], uint32_t* off) {
  bool ok = c[0] >= 0 && c[0] < g.shape[0];
  uint32_t o = static_cast<uint32_t>(c[0]);
#pragma unroll
  for (int dim = 0; dim < kMaxSpatial; ++dim) {
    int v = 0;
    ok = tapDim(g, dim, c[dim + 1], idx[dim], v) && ok;
    o = o * static_cast<uint32_t>(g.shape[dim + 1]) + static_cast<uint32_t>(v);
  }
  *off = o;
  return ok;
}

// Words per tap of the workspace area behind the pair counts (the hash path keeps its owned-output counts per
// tap there; the pair counts themselves need no per-tap totals: the compaction sums the rows of counts).  Atomics
// on one address are performed one after the other (about 18 ns each across the XCDs), device-wide atomics run
// at a few per nanosecond in all: passes that every workgroup ended with a handful of them spent more time there
// than on their loads and stores.
constexpr int kTotalSlots = 8;

// Pairs per (tap, block of 256 or 512 inputs), kept in 16 bits so that a row of counts is short.
typedef uint16_t RbCount;

// Publishes the number of flagged items of this workgroup for its tap in cnt (row pitch nBlocks) and, when `totals` is
// given, adds it to the per-tap sums there (`slots` partial sums per tap).
template <class Count>
__device__ __forceinline__ void publishCount(uint32_t mine, uint32_t* scratch, Count* cnt, uint32_t nBlocks,
                                             uint32_t* totals, int slots) {
  const uint32_t total = blockSum(mine, scratch);
  if (threadIdx.x == 0) {
    cnt[static_cast<size_t>(blockIdx.y) * nBlocks + blockIdx.x] = static_cast<Count>(total);
    if (total && totals) atomicAdd(&totals[blockIdx.y * slots + blockIdx.x % slots], total);
  }
}

// Pairs per (tap, 256 inputs) of the passes that run one workgroup per (chunk of 1024 inputs, tap): a wavefront's
// lanes hold 256 consecutive inputs, so every wavefront stores the count of its own block (row pitch `pitch`).
__device__ __forceinline__ void publishWaveCounts(uint32_t mine, RbCount* cnt, uint32_t pitch) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mine += __shfl_down(mine, off, 64);
  if ((threadIdx.x & 63) == 0)
    cnt[static_cast<size_t>(blockIdx.y) * pitch + blockIdx.x * (kRbThreads / 64) + (threadIdx.x >> 6)] =
        static_cast<RbCount>(mine);
}

// SubM: coordinate -> row map (reference: setSubMHashKernel, index.cu:174-182)
__global__ void __launch_bounds__(kRbThreads)
rbSubmInsert(RbGeom g, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
             unsigned long long* table, uint32_t mask) {
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int c[5];
  if (!loadInput(g, coors, i, c) || !coordInGrid(g, c)) return;
  hashInsertMin(table, mask, coordOffset(g, c), static_cast<uint32_t>(i));
}

// SubM probe (reference: subMGeometryKernel + SubMHashWriter, index.cu:48-84):
// staging[tap, i] = row of the voxel at (coord_i + p - tap*d), or ~0.
__global__ void __launch_bounds__(kRbThreads)
rbSubmProbe(RbGeom g, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
            int64_t pitch, const unsigned long long* __restrict__ table, uint32_t mask, uint32_t* __restrict__ staging,
            RbCount* __restrict__ cnt, uint32_t nBlocks, uint32_t* totals) {
  const int n = liveCount(numActIn, cap);
  const int tap = blockIdx.y;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kRbChunk + threadIdx.x * kRbItems;
  uint32_t found = 0;
  if (static_cast<int64_t>(blockIdx.x) * kRbChunk < n) {  // workgroup-uniform
    int idx[kMaxSpatial];
    tapPositions(g, tap, idx);
    uint32_t row[kRbItems];
#pragma unroll
    for (int j = 0; j < kRbItems; ++j) {
      row[j] = kNone;
      const int64_t i = first + j;
      if (i < n) {
        int c[5];
        uint32_t off;
        if (loadInput(g, coors, i, c) && tapTarget(g, c, idx, &off)) row[j] = hashLookup(table, mask, off);
      }
      found += row[j] != kNone;
    }
    if (first < n) *reinterpret_cast<uint4*>(staging + static_cast<int64_t>(tap) * pitch + first) =
        make_uint4(row[0], row[1], row[2], row[3]);
  }
  publishWaveCounts(found, cnt, nBlocks);
}

// ---------------------------------------------------------------------------
// Strided / transposed convolution (reference: convGeometryKernel, index.cu:86-102)
// ---------------------------------------------------------------------------
// Pass 1: every candidate output is inserted with value = i*kVol + tap, the
// smallest value per key surviving; staging[tap, i] = slot.
__global__ void __launch_bounds__(kRbThreads)
rbConvInsert(RbGeom g, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
             int64_t pitch, unsigned long long* table, uint32_t mask, uint32_t* __restrict__ staging) {
  const int n = liveCount(numActIn, cap);
  const int tap = blockIdx.y;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kRbChunk + threadIdx.x * kRbItems;
  if (first >= n) return;
  int idx[kMaxSpatial];
  tapPositions(g, tap, idx);
  uint32_t slot[kRbItems];
#pragma unroll
  for (int j = 0; j < kRbItems; ++j) {
    slot[j] = kNone;
    const int64_t i = first + j;
    if (i < n) {
      int c[5];
      uint32_t off;
      if (loadInput(g, coors, i, c) && tapTarget(g, c, idx, &off))
        slot[j] = hashInsertMin(table, mask, off, static_cast<uint32_t>(i) * static_cast<uint32_t>(g.kVol) + tap);
    }
  }
  *reinterpret_cast<uint4*>(staging + static_cast<int64_t>(tap) * pitch + first) =
      make_uint4(slot[0], slot[1], slot[2], slot[3]);
}

// A pair owns its output iff its code is the value that survived in the slot.
__device__ __forceinline__ void loadOwned(const RbGeom& g, int n, int tap, int64_t first, int64_t pitch,
                                          const unsigned long long* __restrict__ table,
                                          const uint32_t* __restrict__ staging, uint32_t slot[kRbItems],
                                          unsigned long long entry[kRbItems], bool own[kRbItems]) {
  uint4 s4 = make_uint4(kNone, kNone, kNone, kNone);
  if (first < n) s4 = *reinterpret_cast<const uint4*>(staging + static_cast<int64_t>(tap) * pitch + first);
  slot[0] = s4.x; slot[1] = s4.y; slot[2] = s4.z; slot[3] = s4.w;
#pragma unroll
  for (int j = 0; j < kRbItems; ++j) {
    const int64_t i = first + j;
    own[j] = false;
    entry[j] = 0;
    if (i < n && slot[j] != kNone) {
      entry[j] = table[slot[j]];
      own[j] = static_cast<uint32_t>(entry[j]) == static_cast<uint32_t>(i) * static_cast<uint32_t>(g.kVol) + tap;
    }
  }
}

// Pass 2: owners per (tap, chunk).
__global__ void __launch_bounds__(kRbThreads)
rbConvOwner(RbGeom g, const int32_t* __restrict__ numActIn, int64_t cap, int64_t pitch,
            const unsigned long long* __restrict__ table, const uint32_t* __restrict__ staging,
            uint32_t* __restrict__ ownCnt, uint32_t nBlocks, uint32_t* ownTotals) {
  __shared__ uint32_t scratch[kRbThreads / 64];
  const int n = liveCount(numActIn, cap);
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kRbChunk + threadIdx.x * kRbItems;
  uint32_t mine = 0;
  if (static_cast<int64_t>(blockIdx.x) * kRbChunk < n) {
    uint32_t slot[kRbItems];
    unsigned long long entry[kRbItems];
    bool own[kRbItems];
    loadOwned(g, n, blockIdx.y, first, pitch, table, staging, slot, entry, own);
#pragma unroll
    for (int j = 0; j < kRbItems; ++j) mine += own[j];
  }
  publishCount(mine, scratch, ownCnt, nBlocks, ownTotals, 1);
}

// Pass 3: output rows are numbered in (tap, owner input row) order; writes the
// output coordinates (reference: coorsOutOrganizeKernel, index.cu:104-121) and
// numActOut = min(total, maxNumActOut).
__global__ void __launch_bounds__(kRbThreads)
rbConvAssign(RbGeom g, const int32_t* __restrict__ numActIn, int64_t cap, int64_t pitch,
             const unsigned long long* __restrict__ table, const uint32_t* __restrict__ staging,
             const uint32_t* __restrict__ ownCnt, uint32_t nBlocks, const uint32_t* __restrict__ ownTotals,
             uint32_t* __restrict__ ids, int32_t* __restrict__ outCoors, int32_t* numActOut, int32_t maxNumActOut) {
  __shared__ uint32_t scratch[kRbThreads / 64];
  const int tap = blockIdx.y;
  if (blockIdx.x == 0 && tap == 0 && threadIdx.x == 0) {
    uint32_t total = 0;
    for (int t = 0; t < g.kVol; ++t) total += ownTotals[t];
    *numActOut = static_cast<int32_t>(total < static_cast<uint32_t>(maxNumActOut) ? total : maxNumActOut);
  }
  const int n = liveCount(numActIn, cap);
  if (static_cast<int64_t>(blockIdx.x) * kRbChunk >= n) return;  // workgroup-uniform
  if (ownCnt[static_cast<size_t>(tap) * nBlocks + blockIdx.x] == 0) return;
  uint32_t before = 0;
  for (uint32_t q = threadIdx.x; q < blockIdx.x; q += blockDim.x) before += ownCnt[static_cast<size_t>(tap) * nBlocks + q];
  uint32_t base = blockSum(before, scratch);
  for (int t = 0; t < tap; ++t) base += ownTotals[t];

  const int64_t first = static_cast<int64_t>(blockIdx.x) * kRbChunk + threadIdx.x * kRbItems;
  uint32_t slot[kRbItems];
  unsigned long long entry[kRbItems];
  bool own[kRbItems];
  loadOwned(g, n, tap, first, pitch, table, staging, slot, entry, own);
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < kRbItems; ++j) mine += own[j];
  uint32_t total;
  uint32_t next = base + blockExclusiveScan(mine, scratch, &total);
  const int cw = g.nd + 1;
  const int pad = kMaxSpatial - g.nd;
#pragma unroll
  for (int j = 0; j < kRbItems; ++j) {
    if (!own[j]) continue;
    ids[slot[j]] = next;
    if (next < static_cast<uint32_t>(maxNumActOut)) {
      // reference: Size::deserialize, trt/include/common/refnd.h:56-64
      uint32_t off = static_cast<uint32_t>(entry[j] >> 32);
      int32_t* row = outCoors + static_cast<size_t>(next) * cw;
#pragma unroll
      for (int dim = kMaxSpatial; dim >= 1; --dim) {
        const uint32_t extent = static_cast<uint32_t>(g.shape[dim]);
        const uint32_t q = off / extent;
        if (dim - 1 >= pad) row[dim - pad] = static_cast<int32_t>(off - q * extent);
        off = q;
      }
      row[0] = static_cast<int32_t>(off);
    }
    ++next;
  }
}

// Pass 4: slot -> output row, dropping outputs beyond maxNumActOut
// (reference: hashOutIndexKernel, index.cu:158-172), plus per-(tap, chunk) counts.
__global__ void __launch_bounds__(kRbThreads)
rbConvResolve(const int32_t* __restrict__ numActIn, int64_t cap, int64_t pitch, const uint32_t* __restrict__ ids,
              uint32_t* __restrict__ staging, int32_t maxNumActOut, RbCount* __restrict__ cnt, uint32_t nBlocks,
              uint32_t* totals) {
  const int n = liveCount(numActIn, cap);
  const int tap = blockIdx.y;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kRbChunk + threadIdx.x * kRbItems;
  uint32_t found = 0;
  if (first < n) {
    uint4* cell = reinterpret_cast<uint4*>(staging + static_cast<int64_t>(tap) * pitch + first);
    const uint4 s4 = *cell;
    uint32_t v[kRbItems] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
    for (int j = 0; j < kRbItems; ++j) {
      uint32_t row = kNone;
      if (first + j < n && v[j] != kNone) {
        const uint32_t id = ids[v[j]];
        if (id < static_cast<uint32_t>(maxNumActOut)) row = id;
      }
      v[j] = row;
      found += row != kNone;
    }
    *cell = make_uint4(v[0], v[1], v[2], v[3]);
  }
  publishWaveCounts(found, cnt, nBlocks);
}

// ---------------------------------------------------------------------------
// Compaction (reference: Valid_Counter scan + outputIndexPadOrganizeKernel +
// indexOrganizeKernel, index.cu:123-156, :352-366).  Workgroup (span, tap)
// writes the valid pairs of its inputs at
//   segment start of the tap  +  pairs of that tap in earlier spans  +  rank.
// Both sums come from the per-(tap, block) counts the probe pass left in `cnt` with plain stores
// (cnt[tap * cntPitch + b] = pairs of inputs [b << cntShift, (b + 1) << cntShift) under the tap): the sixteen
// wavefronts of a workgroup sum the rows of the taps up to their own, one row per wavefront at a time, so no pass
// keeps per-tap totals with device-wide atomics and nothing has to be zeroed before a build.  A workgroup covers
// `iters` runs of 4096 inputs, which keeps the number of workgroups that repeat these sums small.
// ---------------------------------------------------------------------------
constexpr int kCompactThreads = 1024;
constexpr int kCompactWaves = kCompactThreads / 64;

// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves (no LDS traffic, no index registers):
// four shifts inside each row of 16 lanes, then the total of row 0 (2) is added to row 1 (3), then that of rows
// 0-1 to rows 2-3.
__device__ __forceinline__ uint32_t waveInclusiveScan(uint32_t v) {
  v += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x111, 0xF, 0xF, false));  // row_shr:1
  v += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x112, 0xF, 0xF, false));  // row_shr:2
  v += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x114, 0xF, 0xF, false));  // row_shr:4
  v += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x118, 0xF, 0xF, false));  // row_shr:8
  v += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x142, 0xA, 0xF, false));  // row_bcast:15
  v += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x143, 0xC, 0xF, false));  // row_bcast:31
  return v;
}

// Sum over the 64 lanes, the same value in every lane.
__device__ __forceinline__ uint32_t waveSum(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(waveInclusiveScan(v)), 63));
}

__device__ __forceinline__ uint32_t alignSegment(uint32_t v) {
  return (v + (kSegment - 1)) & ~static_cast<uint32_t>(kSegment - 1);
}

// Sum of the eight 16-bit counts of `v` whose block index (b0 .. b0 + 7) lies below `limit`.
__device__ __forceinline__ uint32_t countsBelow(const uint4& v, uint32_t b0, uint32_t limit) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t sum = 0;
  if (b0 + 8 <= limit) {  // the common case: all eight (sad_u16 against 0 adds both halves of a word)
#pragma unroll
    for (int j = 0; j < 4; ++j) sum = __builtin_amdgcn_sad_u16(w[j], 0u, sum);
    return sum;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (b0 + 2 * j < limit) sum += w[j] & 0xFFFFu;
    if (b0 + 2 * j + 1 < limit) sum += w[j] >> 16;
  }
  return sum;
}

// MIRROR: the table is that of a SubM rulebook with "same" padding (see below).  SKIP: the index tensor is left
// unwritten (nothing reads it): what remains is numIndex and, where inputs were not in rank order, the ranks in
// the mirrored table turned into rows.  SHIFT: log2 of the inputs per entry of cnt (8 or 9); a wavefront
// compacts exactly one such block, 1 << (SHIFT - 6) consecutive inputs per lane, so its write position is the
// workgroup's plus the counts of the workgroup's earlier blocks - after the one barrier behind the sums the
// wavefronts run on their own, each as soon as its own staging entries have arrived.
template <bool MIRROR, bool SKIP, int SHIFT>
__global__ void __launch_bounds__(kCompactThreads) __attribute__((amdgpu_waves_per_eu(8, 8)))
rbCompact(const int32_t* __restrict__ numActIn, int64_t cap, int64_t pitch, int kVol, const uint32_t* staging,
          const RbCount* __restrict__ cnt, uint32_t cntPitch, int32_t* __restrict__ gather,
          int32_t* __restrict__ scatter, int32_t* __restrict__ tapRow, int32_t* numIndex, int32_t* nbr, int64_t nbrRows,
          const uint32_t* __restrict__ perm, const uint32_t* __restrict__ permShuffled, int inPlace,
          unsigned long long* __restrict__ masks, uint32_t* fillState, int incrementalFill) {
  constexpr int ITEMS = 1 << (SHIFT - 6);           // consecutive inputs per lane
  constexpr int RUN = kCompactThreads * ITEMS;      // inputs per workgroup
  extern __shared__ uint32_t tapTotal[];           // [kVol] pairs per tap (the taps this workgroup needs)
  __shared__ uint32_t partBefore;                   // pairs of this tap in the blocks before this workgroup's
  const int tap = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = liveCount(numActIn, cap);
  const int64_t run0 = static_cast<int64_t>(blockIdx.x) * RUN;
  const int64_t first = run0 + tid * ITEMS;
  const bool lastTap = tap == kVol - 1;
  const bool lastSpan = blockIdx.x == gridDim.x - 1;
  const bool shuffled = perm && *permShuffled;

  if (SKIP) {
    if (MIRROR && inPlace && shuffled) {
#pragma unroll
      for (int q = 0; q < ITEMS / 4; ++q) {
        if (first + 4 * q >= n) break;
        uint4* cell = reinterpret_cast<uint4*>(const_cast<uint32_t*>(staging) + static_cast<int64_t>(tap) * pitch + first) + q;
        uint4 v = *cell;
        if (v.x != kNone) v.x = perm[v.x];
        if (v.y != kNone) v.y = perm[v.y];
        if (v.z != kNone) v.z = perm[v.z];
        if (v.w != kNone) v.w = perm[v.w];
        *cell = v;
      }
    }
    if (blockIdx.x != 0 || tap != 0) return;  // workgroup-uniform
  }

  // ---- pairs per tap (rows of cnt), pairs of this tap before this workgroup's blocks ----
  const uint32_t liveBlocks = static_cast<uint32_t>((static_cast<int64_t>(n) + (1 << SHIFT) - 1) >> SHIFT);
  uint32_t firstBlock = blockIdx.x * kCompactWaves;
  if (firstBlock > liveBlocks) firstBlock = liveBlocks;
  // pairs of this tap in the workgroup's blocks before this wavefront's: read now, summed behind the barrier
  uint32_t earlier = 0;
  if (!SKIP && lane < wave && blockIdx.x * kCompactWaves + lane < liveBlocks)
    earlier = cnt[static_cast<size_t>(tap) * cntPitch + blockIdx.x * kCompactWaves + lane];
  // workgroups of the last tap also need that tap's total (the end of the used part of the tensor); the one
  // workgroup of a build that leaves the tensor unwritten needs every tap's
  const bool wantAll = SKIP || lastTap;
  const int lastRow = wantAll ? kVol - 1 : tap;
  // A wavefront sums rows wave, wave + 16, ..., two rows at a time with the loads of both in flight together
  // (three loads cover 1536 blocks of a row).  Loads return in the order of their issue: the rows (L2) are
  // requested before the staging entries (HBM), so that the sums do not wait for those.
  auto rowLimit = [&](int row) -> uint32_t {
    return row > lastRow ? 0u : ((row < tap || wantAll) ? liveBlocks : firstBlock);
  };
  auto loadRows = [&](int row0, uint32_t base, uint4 (&a)[3], uint4 (&b)[3]) {
    const int row1 = row0 + kCompactWaves;
    const uint32_t limit0 = rowLimit(row0), limit1 = rowLimit(row1);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const uint32_t b0 = base + static_cast<uint32_t>(k * 64 + lane) * 8;
      a[k] = make_uint4(0, 0, 0, 0);
      b[k] = make_uint4(0, 0, 0, 0);
      if (b0 < limit0) a[k] = *reinterpret_cast<const uint4*>(cnt + static_cast<size_t>(row0) * cntPitch + b0);
      if (b0 < limit1) b[k] = *reinterpret_cast<const uint4*>(cnt + static_cast<size_t>(row1) * cntPitch + b0);
    }
  };
  auto sumRows = [&](int row0, uint32_t base, const uint4 (&a)[3], const uint4 (&b)[3], uint32_t* full0,
                     uint32_t* full1, uint32_t* part) {
    const int row1 = row0 + kCompactWaves;
    const uint32_t limit0 = rowLimit(row0), limit1 = rowLimit(row1);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const uint32_t b0 = base + static_cast<uint32_t>(k * 64 + lane) * 8;
      *full0 += countsBelow(a[k], b0, limit0);
      *full1 += countsBelow(b[k], b0, limit1);
      if (row0 == tap) *part += countsBelow(a[k], b0, firstBlock);
      if (row1 == tap) *part += countsBelow(b[k], b0, firstBlock);
    }
  };
  auto publishRows = [&](int row0, uint32_t full0, uint32_t full1, uint32_t part) {
    const int row1 = row0 + kCompactWaves;
    full0 = waveSum(full0);
    full1 = waveSum(full1);
    if (row0 == tap || row1 == tap) part = waveSum(part);
    if (lane == 0) {
      if (row0 <= lastRow) tapTotal[row0] = full0;
      if (row1 <= lastRow) tapTotal[row1] = full1;
      if (row0 == tap || row1 == tap) partBefore = part;
    }
  };
  uint4 headA[3], headB[3];
  loadRows(wave, 0, headA, headB);
  // the staging entries: their latency (HBM) covers the sums below
  uint4 s4[ITEMS / 4];
#pragma unroll
  for (int q = 0; q < ITEMS / 4; ++q) {
    s4[q] = make_uint4(kNone, kNone, kNone, kNone);
    if (!SKIP && first + 4 * q < n)
      s4[q] = *(reinterpret_cast<const uint4*>(staging + static_cast<int64_t>(tap) * pitch + first) + q);
  }
  {
    uint32_t full0 = 0, full1 = 0, part = 0;
    sumRows(wave, 0, headA, headB, &full0, &full1, &part);
    for (uint32_t base = 3 * 512; base < liveBlocks; base += 3 * 512) {  // more than 1536 blocks in a row
      uint4 a[3], b[3];
      loadRows(wave, base, a, b);
      sumRows(wave, base, a, b, &full0, &full1, &part);
    }
    publishRows(wave, full0, full1, part);
  }
  for (int row0 = wave + 2 * kCompactWaves; row0 <= lastRow; row0 += 2 * kCompactWaves) {  // more than 32 taps
    uint32_t full0 = 0, full1 = 0, part = 0;
    for (uint32_t base = 0; base < liveBlocks; base += 3 * 512) {
      uint4 a[3], b[3];
      loadRows(row0, base, a, b);
      sumRows(row0, base, a, b, &full0, &full1, &part);
    }
    publishRows(row0, full0, full1, part);
  }
  __syncthreads();
  uint32_t segs = 0;  // segments of the earlier taps
  for (int t = lane; t < tap; t += 64) segs += alignSegment(tapTotal[t]);
  const uint32_t segStart = waveSum(segs);
  uint32_t end = 0;   // end of the used part of the index tensor (workgroups that summed every row)
  if (wantAll) {
    uint32_t all = 0;
    for (int t = lane; t < kVol; t += 64) all += alignSegment(tapTotal[t]);
    end = waveSum(all);
  }
  if (SKIP) {
    if (tid == 0) {
      *numIndex = static_cast<int32_t>(end);
      if (fillState) fillState[1] = end;
    }
    return;
  }
  const uint32_t at0 = segStart + partBefore + waveSum(earlier);  // where this wavefront's first pair goes

  // ---- rank of this lane's pairs among the wavefront's ----
  uint32_t v[ITEMS];
#pragma unroll
  for (int q = 0; q < ITEMS / 4; ++q) {
    v[4 * q] = s4[q].x;
    v[4 * q + 1] = s4[q].y;
    v[4 * q + 2] = s4[q].z;
    v[4 * q + 3] = s4[q].w;
  }
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    if (first + j >= n) v[j] = kNone;
    mine += (v[j] != kNone);
  }
  const uint32_t incl = waveInclusiveScan(mine);
  uint32_t at = at0 + incl - mine;

  // Mirror mode (SubM with "same" padding): the pair (tap, in i -> out o) has the twin (kVol-1-tap, in o -> out i),
  // so row i of the neighbour table under the mirrored tap is simply o - this thread's own staging entry.  The
  // table is then written here in whole coalesced rows, -1 included: no fill pass, no scatter.  With inPlace the
  // probe pass already used the table rows as its staging rows (staging + tap * pitch IS the row below): only
  // what the probe did not leave right is stored - entries of rows past the live count, and rows where ranks have
  // to become row numbers.
  int32_t* nbrRow = (MIRROR && nbr) ? nbr + static_cast<int64_t>(kVol - 1 - tap) * nbrRows : nullptr;
  auto mirrorStore = [&](const uint32_t (&o)[ITEMS]) {
    if (!nbrRow) return;
    if (first + ITEMS <= nbrRows && ((reinterpret_cast<uintptr_t>(nbrRow + first) & 15) == 0)) {
#pragma unroll
      for (int q = 0; q < ITEMS / 4; ++q)
        reinterpret_cast<uint4*>(nbrRow + first)[q] = make_uint4(o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]);
    } else {
#pragma unroll
      for (int j = 0; j < ITEMS; ++j)
        if (first + j < nbrRows) nbrRow[first + j] = static_cast<int32_t>(o[j]);
    }
  };
  if (shuffled) {  // block-map SubM: the probe stored ranks; rows are perm[rank]
#pragma unroll
    for (int j = 0; j < ITEMS; ++j)
      if (v[j] != kNone) v[j] = perm[v[j]];
  }
  if (!inPlace || shuffled || first + ITEMS > n) mirrorStore(v);
  if (masks && MIRROR && kVol <= 64) {
    // tile masks of the convolution (bit t of masks[r / 64]: some output row of 64-row tile r / 64 has tap t).
    // Mirrored table: this thread's consecutive INPUT rows are output rows under tap kVol-1-tap; kTileLanes
    // lanes cover exactly one tile.
    constexpr int kTileLanes = 64 / ITEMS;
    const unsigned long long any = __ballot(mine != 0);
    if ((lane & (kTileLanes - 1)) == 0 && ((any >> lane) & ((1ull << kTileLanes) - 1ull)) && first < nbrRows)
      atomicOr(&masks[first >> 6], 1ull << (kVol - 1 - tap));
  }
  if constexpr (ITEMS <= 8) {
    // The wavefront's pairs are packed in LDS first (a lane's pairs start at its exclusive rank) and stored from
    // there: lane l writes pairs l, l + 64, ... of the wavefront, so every store instruction covers 256
    // consecutive bytes of a row instead of 64 runs of a few entries.  The buffer is the wavefront's own: LDS
    // accesses of one wavefront are performed in order, no workgroup barrier is involved.
    __shared__ uint2 packed[kCompactWaves][64 * ITEMS];
    uint32_t slot = incl - mine;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      if (v[j] != kNone) {
        packed[wave][slot++] = make_uint2(static_cast<uint32_t>(first + j), v[j]);
        // the same pair in output-major form, for the convolution: nbr[tap][output row] = input row
        if (nbr && !MIRROR && v[j] < static_cast<uint64_t>(nbrRows))
          nbr[static_cast<int64_t>(tap) * nbrRows + v[j]] = static_cast<int32_t>(first + j);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint32_t pairs = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), 63));
    for (uint32_t k = lane; k < pairs; k += 64) {
      const uint2 e = packed[wave][k];
      gather[at0 + k] = static_cast<int32_t>(e.x);
      scatter[at0 + k] = static_cast<int32_t>(e.y);
      tapRow[at0 + k] = tap;
    }
    (void)at;
  } else {
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      if (v[j] != kNone) {
        gather[at] = static_cast<int32_t>(first + j);
        scatter[at] = static_cast<int32_t>(v[j]);
        tapRow[at] = tap;
        ++at;
        if (nbr && !MIRROR && v[j] < static_cast<uint64_t>(nbrRows))
          nbr[static_cast<int64_t>(tap) * nbrRows + v[j]] = static_cast<int32_t>(first + j);
      }
    }
  }
  if (lastTap && lastSpan && tid == 0) {
    *numIndex = static_cast<int32_t>(end);
    if (fillState) fillState[1] = end;  // what this pass uses of the index tensor: the next pass clears from here
  }
  // The index tensor still holds the previous pass (of this operator, at this address): instead of clearing it at
  // capacity, write -1 where that pass had entries and this one has none - in the gap that rounds this tap's
  // segment up to 128 (the wavefront that holds the tap's last pairs), and behind the new end up to the old one
  // (the workgroups of the last tap, which know the new end; short unless the scene changed a lot).
  if (!incrementalFill) return;
  if (lastSpan && wave == kCompactWaves - 1) {
    const uint32_t pairsEnd = at0 + static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), 63));
    const uint32_t segEnd = alignSegment(pairsEnd);
    for (uint32_t i = pairsEnd + lane; i < segEnd; i += 64) {
      gather[i] = -1;
      scatter[i] = -1;
      tapRow[i] = -1;
    }
  }
  if (lastTap) {
    const uint32_t oldEnd = fillState[0];
    const uint32_t gid = blockIdx.x * kCompactThreads + tid, nThreads = gridDim.x * kCompactThreads;
    // segment ends are multiples of 128 entries: 16-byte stores when the three rows are 16-byte aligned
    if (((reinterpret_cast<uintptr_t>(gather) | reinterpret_cast<uintptr_t>(scatter) |
          reinterpret_cast<uintptr_t>(tapRow)) & 15) == 0) {
      const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
      for (uint32_t i = end / 4 + gid; i < oldEnd / 4; i += nThreads) {
        reinterpret_cast<uint4*>(gather)[i] = ones;
        reinterpret_cast<uint4*>(scatter)[i] = ones;
        reinterpret_cast<uint4*>(tapRow)[i] = ones;
      }
    } else {
      for (uint32_t i = end + gid; i < oldEnd; i += nThreads) {
        gather[i] = -1;
        scatter[i] = -1;
        tapRow[i] = -1;
      }
    }
  }
}


// ===========================================================================
// Block-map path.  When the grid is small enough to afford 16 bytes per 64
// cells, occupancy is kept in a dense table of records instead of the hash:
//   record = { u64 bits; u32 prefix; u32 pad }   one per block of 64 cells
// A block is a small brick of the grid (1x8x8 cells in 3-D: one level of the
// outermost dim), so a 3x3x3 neighbourhood touches at most 12 records, close
// in memory and resident in L2, where a hash probe costs one random cache
// line per tap.  A voxel's rank is prefix + popcount(bits below its own), i.e.
// voxels are ranked in brick-major order.  SubM looks rows up through
// perm[rank]; strided outputs are numbered by their rank directly, which
// needs no CAS, no owner election, and leaves output rows sorted level by
// level of the outermost dim and in 8x8 patches inside a level.  Rows that
// follow each other then share most of their neighbourhood pattern (on a
// LiDAR grid: which of the levels above and below exist), which lets the
// convolution skip the taps a whole tile of rows lacks, and their neighbours
// sit in runs of consecutive feature rows for its gathers.
// ===========================================================================
struct __attribute__((aligned(16))) BmRecord {
  unsigned long long bits;
  uint32_t prefix;
  uint32_t pad;
};

// The records a kernel works on.  A build whose caller keeps the map between passes alternates between two maps
// (`stride` records apart): `*epoch` counts the scans performed so far, the scan pass of a build clears the
// occupancy bits of the map the NEXT build will mark and then advances the count, so no pass has to zero a map
// before marking it.  Kernels before (and including) the scan use bias 0, kernels behind it bias 1 (the count
// has moved on by then).  epoch == nullptr: one map at `base`, zeroed by a reset pass.
struct RecRef {
  BmRecord* base;
  uint32_t* epoch;
  uint32_t stride;
  uint32_t bias;
  __device__ __forceinline__ BmRecord* get() const {
    return epoch ? base + static_cast<size_t>((*epoch + bias) & 1u) * stride : base;
  }
};

struct BlockMap {
  int shift[kMaxSpatial];  // log2 brick extent per spatial dim (extents multiply to 64)
  int nb[kMaxSpatial];     // bricks per dim
  uint32_t records;        // batch * product of nb
};

__device__ __forceinline__ void bmLocate(const BlockMap& m, const int c[5], uint32_t* rec, uint32_t* bit) {
  uint32_t r = static_cast<uint32_t>(c[0]);
  uint32_t b = 0;
#pragma unroll
  for (int dim = 0; dim < kMaxSpatial; ++dim) {
    const uint32_t v = static_cast<uint32_t>(c[dim + 1]);
    r = r * static_cast<uint32_t>(m.nb[dim]) + (v >> m.shift[dim]);
    b = (b << m.shift[dim]) | (v & ((1u << m.shift[dim]) - 1));
  }
  *rec = r;
  *bit = b;
}

// Output voxel of (input coordinate, tap) as a coordinate; false if off-lattice or outside the grid.
__device__ __forceinline__ bool tapTargetCoord(const RbGeom& g, const int c[5], const int idx[kMaxSpatial], int o[5]) {
  bool ok = c[0] >= 0 && c[0] < g.shape[0];
  o[0] = c[0];
#pragma unroll
  for (int dim = 0; dim < kMaxSpatial; ++dim) {
    int v = 0;
    ok = tapDim(g, dim, c[dim + 1], idx[dim], v) && ok;
    o[dim + 1] = v;
  }
  return ok;
}

// rank = occupied cells in earlier chunks of 1024 records + in earlier records of the chunk + below the bit
__device__ __forceinline__ uint32_t bmRank(const BmRecord& r, uint32_t bit, const uint32_t* __restrict__ chunkBase,
                                           uint32_t rec) {
  return chunkBase[rec / kRbChunk] + r.prefix + static_cast<uint32_t>(__popcll(r.bits & ((1ull << bit) - 1ull)));
}

// reset for the block-map path: records = 0, index tensor = -1, counters = 0
// -1 over p[0..n) by the threads tid, tid+stride, ...: 16-byte stores over the aligned body
__device__ __forceinline__ void fillMinusOneRange(int32_t* p, int64_t n, int64_t tid, int64_t stride) {
  if (!p || n <= 0) return;
  const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
  const uintptr_t base = reinterpret_cast<uintptr_t>(p);
  int64_t head = ((16 - (base & 15)) & 15) >> 2;
  if (head > n) head = n;
  const int64_t body16 = (n - head) >> 2;
  uint4* body = reinterpret_cast<uint4*>(p + head);
  for (int64_t i = tid; i < body16; i += stride) body[i] = ones;
  const int64_t tailStart = head + (body16 << 2);
  if (tid < head) p[tid] = -1;
  if (tid < n - tailStart) p[tailStart + tid] = -1;
}

__global__ void __launch_bounds__(kRbThreads)
bmReset(uint4* records16, int64_t nRecords, int32_t* index, int64_t nIndex, uint32_t* counters, int64_t nCounters,
        int32_t* numIndex, unsigned long long* masks, int64_t nMasks, uint32_t* fillState) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  resetShared(tid, stride, masks, nMasks, fillState);
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (int64_t i = tid; i < nRecords; i += stride) records16[i] = zero;
  fillMinusOneRange(index, nIndex, tid, stride);  // index == nullptr: a later pass fills it
  for (int64_t q = tid; q < nCounters; q += stride) counters[q] = 0;
  if (tid == 0) *numIndex = 0;
}

__global__ void __launch_bounds__(kRbThreads) rbFillMinusOne(int32_t* p, int64_t n) {
  fillMinusOneRange(p, n, static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x,
                    static_cast<int64_t>(gridDim.x) * blockDim.x);
}

// Lanes of a 16-lane row that target the same record merge their bits before the atomic: inputs usually arrive
// in brick order, so neighbouring lanes hit the same record and device-wide atomic throughput (the bound of the
// marking passes) is spent on one operation per run instead of one per voxel.  `rec` = kNone for lanes with
// nothing to mark.  Bits only accumulate with OR, so merging any equal-record lanes is valid; the last lane of
// each run of equal records issues the atomic.
__device__ __forceinline__ void orRuns(BmRecord* records, uint32_t rec, unsigned long long bits) {
  uint32_t lo = static_cast<uint32_t>(bits), hi = static_cast<uint32_t>(bits >> 32);
  const int key = static_cast<int>(rec);
#define D3D_ROW_SHR_STEP(N)                                                                        \
  {                                                                                                \
    const int k2 = __builtin_amdgcn_update_dpp(-2, key, 0x110 + N, 0xF, 0xF, false);               \
    const uint32_t lo2 = __builtin_amdgcn_update_dpp(0, static_cast<int>(lo), 0x110 + N, 0xF, 0xF, false); \
    const uint32_t hi2 = __builtin_amdgcn_update_dpp(0, static_cast<int>(hi), 0x110 + N, 0xF, 0xF, false); \
    if (k2 == key) {                                                                               \
      lo |= lo2;                                                                                   \
      hi |= hi2;                                                                                   \
    }                                                                                              \
  }
  D3D_ROW_SHR_STEP(1)
  D3D_ROW_SHR_STEP(2)
  D3D_ROW_SHR_STEP(4)
  D3D_ROW_SHR_STEP(8)
#undef D3D_ROW_SHR_STEP
  const int next = __builtin_amdgcn_update_dpp(-2, key, 0x101, 0xF, 0xF, false);  // row_shl:1 = the next lane's record
  if (rec != kNone && next != key && (lo | hi))
    atomicOr(&records[rec].bits, (static_cast<unsigned long long>(hi) << 32) | lo);
}

// SubM: mark the input voxels.
__global__ void __launch_bounds__(kRbThreads)
bmMarkInputs(RbGeom g, BlockMap m, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
             RecRef recRef, uint32_t* clearFlag) {
  BmRecord* records = recRef.get();
  // a build without a reset pass: the "rows not in rank order" flag of the previous pass goes here (the pass that
  // raises it comes behind the scan)
  if (clearFlag && blockIdx.x == 0 && threadIdx.x == 0) *clearFlag = 0u;
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  uint32_t rec = kNone, bit = 0;
  if (i < n) {
    int c[5];
    if (loadInput(g, coors, i, c) && coordInGrid(g, c)) bmLocate(m, c, &rec, &bit);
  }
  orRuns(records, rec, 1ull << bit);  // every lane takes part in the cross-lane merge
}

// Strided / transposed: mark every candidate output (reference: convGeometryKernel, index.cu:86-102).
// A bit that a plain read already shows set needs no atomic; bits are only ever set.
__global__ void __launch_bounds__(kRbThreads)
bmMarkCandidates(RbGeom g, BlockMap m, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn,
                 int64_t cap, RecRef recRef) {
  BmRecord* records = recRef.get();
  const int n = liveCount(numActIn, cap);
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kRbChunk + threadIdx.x * kRbItems;
  if (first >= n) return;
  int idx[kMaxSpatial];
  tapPositions(g, blockIdx.y, idx);
#pragma unroll
  for (int j = 0; j < kRbItems; ++j) {
    const int64_t i = first + j;
    if (i >= n) break;
    int c[5], o[5];
    if (!loadInput(g, coors, i, c) || !tapTargetCoord(g, c, idx, o)) continue;
    uint32_t rec, bit;
    bmLocate(m, o, &rec, &bit);
    const unsigned long long mask = 1ull << bit;
    if ((__builtin_nontemporal_load(&records[rec].bits) & mask) == 0) atomicOr(&records[rec].bits, mask);
  }
}

// c ? a : b on values: the operands are made opaque first, so that a choice between two elements of a local array
// stays a register select instead of becoming a dynamically indexed (memory-resident) array.
__device__ __forceinline__ uint32_t pick(bool c, uint32_t a, uint32_t b) {
  asm("" : "+v"(a));
  asm("" : "+v"(b));
  return c ? a : b;
}

constexpr uint32_t kScanGroup = 32;  // workgroups of the scan pass that share one first-level ticket

// What a scan that derives its occupancy from the map of the input grid needs (bmScan<.., GATHER>).
struct GatherArgs {
  RecRef src;                      // finished map of the input grid (rows of the input = ranks in it)
  const uint32_t* srcChunkBase;
  BlockMap mo, mi;                 // bricks of the output grid / of the input grid
  const int32_t* numActIn;
  uint32_t inCap;                  // row capacity of the input: a live count below it rules truncation out
  int shapeY, shapeX;              // output extents of the two in-brick dims
  int padZ;                        // GATHER 1: padding of the level dim, 0 or 1
  float rcpX, rcpY, rcpZ;          // 1 / mo.nb[3], 1 / mo.nb[2], 1 / mo.nb[1] (record indices stay below 2^24)
};

// x / d for x < 2^24 with rcp = 1.0f / d: the float quotient is off by one at most.
__device__ __forceinline__ uint32_t divSmall(uint32_t x, uint32_t d, float rcp) {
  uint32_t q = static_cast<uint32_t>(static_cast<float>(x) * rcp);
  const int32_t r = static_cast<int32_t>(x - q * d);
  if (r < 0) --q;
  else if (r >= static_cast<int32_t>(d)) ++q;
  return q;
}

// Cells of an input-map record (bits, rank `first` of its lowest cell) that are rows of the input: cells ranked at
// or past nLive were cut off when the build that wrote the map truncated its outputs.
__device__ __forceinline__ unsigned long long cutToLive(unsigned long long bits, uint32_t first, uint32_t nLive) {
  if (first >= nLive) return 0ull;
  uint32_t n = static_cast<uint32_t>(__popcll(bits));
  while (first + n > nLive) {  // at most one record of the map is cut inside
    bits &= ~(1ull << (63 - __builtin_clzll(bits)));
    --n;
  }
  return bits;
}

// Three consecutive cells OR-ed, every second one kept: with the 8 cells of byte k of `mid` at positions 1..8 of a
// row of 17, the last cell of byte k of `left` at position 0 and the cells of byte k of `right` at 9..16, byte k
// of the result holds cell j = OR of positions 2j, 2j+1, 2j+2 - for all 8 bytes at once.
__device__ __forceinline__ unsigned long long foldCells(unsigned long long left, unsigned long long mid,
                                                        unsigned long long right) {
  constexpr unsigned long long k01 = 0x0101010101010101ull;
  const unsigned long long tm = mid | ((mid >> 1) & (k01 * 0x7F)) | ((mid >> 2) & (k01 * 0x3F));        // bit i: m_i|m_i+1|m_i+2
  const unsigned long long tr = right | ((right >> 1) & (k01 * 0x7F)) | ((right >> 2) & (k01 * 0x3F));
  unsigned long long out = (((left >> 7) | mid | (mid >> 1)) & k01);                                     // l7|m0|m1
  out |= (tm & (k01 * 0x02)) | ((tm >> 1) & (k01 * 0x04)) | ((tm >> 2) & (k01 * 0x08));                  // m1.., m3.., m5..
  out |= (((mid >> 7) | right | (right >> 1)) & k01) << 4;                                               // m7|r0|r1
  out |= ((tr & (k01 * 0x02)) << 4) | ((tr & (k01 * 0x08)) << 3) | ((tr & (k01 * 0x20)) << 2);           // r1.., r3.., r5..
  return out;
}

// The same fold one level up: rows instead of cells.  `above`, `here`, `below` hold 8 rows of 8 cells each (a byte
// per row); row k of the result = OR of rows 2k, 2k+1, 2k+2 of the 17 rows (last of above, 8 of here, 8 of below).
__device__ __forceinline__ unsigned long long foldRows(unsigned long long above, unsigned long long here,
                                                       unsigned long long below) {
  const unsigned long long th = here | (here >> 8) | (here >> 16);    // byte i: rows i, i+1, i+2 of here
  const unsigned long long tb = below | (below >> 8) | (below >> 16);
  const unsigned long long r0 = ((above >> 56) | here | (here >> 8)) & 0xFFull;
  const unsigned long long r4 = ((here >> 56) | below | (below >> 8)) & 0xFFull;
  return r0 | (((th >> 8) & 0xFFull) << 8) | (((th >> 24) & 0xFFull) << 16) | (((th >> 40) & 0xFFull) << 24) |
         (r4 << 32) | (((tb >> 8) & 0xFFull) << 40) | (((tb >> 24) & 0xFFull) << 48) | (((tb >> 40) & 0xFFull) << 56);
}

// Occupancy of output record `rec` (a brick of 1 x 8 x 8 cells) from the input map.
//   GATHER 1: 3x3x3, stride 2, padding (pz, 1, 1) with pz 0 or 1: output (z, y, x) has a pair when any input cell of
//             (2z-pz..2z-pz+2, 2y-1..2y+1, 2x-1..2x+1) is a row: 3 levels of 3 x 3 input bricks.
//   GATHER 2: 3x1x1, stride (2,1,1), padding 0: input levels 2z..2z+2 of the same brick.
template <int GATHER>
__device__ __forceinline__ unsigned long long gatherOccupancy(const GatherArgs& ga, const BmRecord* __restrict__ src,
                                                              uint32_t rec, uint32_t nLive, bool checkRanks) {
  const uint32_t q1 = divSmall(rec, static_cast<uint32_t>(ga.mo.nb[3]), ga.rcpX);
  const int obx = static_cast<int>(rec - q1 * static_cast<uint32_t>(ga.mo.nb[3]));
  const uint32_t q2 = divSmall(q1, static_cast<uint32_t>(ga.mo.nb[2]), ga.rcpY);
  const int oby = static_cast<int>(q1 - q2 * static_cast<uint32_t>(ga.mo.nb[2]));
  const uint32_t batch = divSmall(q2, static_cast<uint32_t>(ga.mo.nb[1]), ga.rcpZ);  // (the leading spatial dim of a 3-D grid has extent 1)
  const int oz = static_cast<int>(q2 - batch * static_cast<uint32_t>(ga.mo.nb[1]));
  const int nz = ga.mi.nb[1], ny = ga.mi.nb[2], nx = ga.mi.nb[3];
  constexpr int NA = GATHER == 1 ? 3 : 1;           // input bricks under the output brick per in-brick dim
  constexpr int N = 3 * NA * NA;
  // Every record underneath is requested before the first is looked at - the loads are independent - and only
  // its occupancy bits are (8 bytes; 27 whole records would not fit the registers of a 1024-thread workgroup).
  // A brick outside the grid reads record 0 and counts as empty.
  auto recordAt = [&](int e, bool* inside) -> uint32_t {
    const int dz = e / (NA * NA), a = (e / NA) % NA, c = e % NA;
    const int iz = GATHER == 1 ? 2 * oz + dz - ga.padZ : 2 * oz + dz;
    const int iby = GATHER == 1 ? 2 * oby + a - 1 : oby;
    const int ibx = GATHER == 1 ? 2 * obx + c - 1 : obx;
    *inside = iz >= 0 && iz < nz && iby >= 0 && iby < ny && ibx >= 0 && ibx < nx;
    return *inside ? ((batch * static_cast<uint32_t>(nz) + static_cast<uint32_t>(iz)) * static_cast<uint32_t>(ny) +
                      static_cast<uint32_t>(iby)) * static_cast<uint32_t>(nx) + static_cast<uint32_t>(ibx)
                   : 0u;
  };
  uint2 got[N];
#pragma unroll
  for (int e = 0; e < N; ++e) {
    bool inside;
    const uint32_t at = recordAt(e, &inside);
    got[e] = *reinterpret_cast<const uint2*>(src + at);
    if (!inside) got[e] = make_uint2(0u, 0u);
  }
  unsigned long long under[NA][NA];  // [brick row][brick column] of the input bricks, the three levels merged
#pragma unroll
  for (int a = 0; a < NA; ++a)
#pragma unroll
    for (int c = 0; c < NA; ++c) under[a][c] = 0ull;
  if (!checkRanks) {  // grid-uniform
#pragma unroll
    for (int e = 0; e < N; ++e) under[(e / NA) % NA][e % NA] |= (static_cast<unsigned long long>(got[e].y) << 32) | got[e].x;
  } else {
#pragma unroll 1
    for (int e = 0; e < N; ++e) {
      bool inside;
      const uint32_t at = recordAt(e, &inside);
      if (!inside) continue;
      const uint4 r = *reinterpret_cast<const uint4*>(src + at);
      unsigned long long bits = (static_cast<unsigned long long>(r.y) << 32) | r.x;
      if (bits) bits = cutToLive(bits, ga.srcChunkBase[at / kRbChunk] + r.z, nLive);
      // (a loop that is not unrolled: the brick is chosen by arithmetic, not by a constant index)
      const int a = (e / NA) % NA, c = e % NA;
#pragma unroll
      for (int aa = 0; aa < NA; ++aa)
#pragma unroll
        for (int cc = 0; cc < NA; ++cc)
          if (aa == a && cc == c) under[aa][cc] |= bits;
    }
  }
  if constexpr (GATHER == 2) {
    return under[0][0];
  } else {
    // 17 x 17 input cells under the 8 x 8 outputs: rows folded first (per brick column), then cells
    return foldCells(foldRows(under[0][0], under[1][0], under[2][0]), foldRows(under[0][1], under[1][1], under[2][1]),
                     foldRows(under[0][2], under[1][2], under[2][2]));
  }
}

// GATHER != 0: the occupancy bits are not in the map yet (no marking pass ran) - they are derived here from the
// map of the input grid (gatherOccupancy) and stored with the prefix.
// That variant runs 1024 threads per workgroup: one thread per record of the chunk gathers (27 independent loads),
// the bits pass through LDS, and the first 256 threads go on with the scan as always.
template <bool ORDERED, int GATHER>
__global__ void __launch_bounds__(GATHER ? kRbChunk : kRbThreads)
bmScan(RecRef recRef, uint32_t nRecords, uint32_t* chunkBase, uint32_t nChunks, uint32_t* ticket,
       uint32_t* groupTickets, int32_t* numActOut, int32_t maxNumActOut, GatherArgs ga) {
  __shared__ uint32_t scratch[kRbThreads / 64];
  __shared__ uint32_t isLast;
  const uint32_t epoch = recRef.epoch ? *recRef.epoch : 0u;
  BmRecord* __restrict__ records = recRef.base + static_cast<size_t>(epoch & 1u) * (recRef.epoch ? recRef.stride : 0u);
  // two maps: the occupancy bits of the one the next build marks are cleared here, record by record
  BmRecord* __restrict__ other = recRef.epoch ? recRef.base + static_cast<size_t>((epoch + 1u) & 1u) * recRef.stride : nullptr;
  // A wavefront takes 256 consecutive records as 4 rows of 64: lane l reads records l, 64 + l, 128 + l, 192 + l of
  // them, so every load instruction covers 1 KB of consecutive memory.  Counts are at most 64 and a row's running
  // sum at most 4096, so two rows share one 32-bit lane scan (16 bits each).
  static_assert(kRbItems == 4 && kRbChunk == 4 * 256, "bmScan assumes 4 wavefronts of 4 x 64 records");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t first = blockIdx.x * kRbChunk + wave * 256 + lane;
  uint32_t count[kRbItems];
  unsigned long long gathered[GATHER ? kRbItems : 1];
  if constexpr (GATHER != 0) {
    __shared__ unsigned long long chunkBits[kRbChunk];
    {
      const BmRecord* __restrict__ src = ga.src.get();
      const int32_t live = *ga.numActIn;
      const uint32_t nLive = live < 0 ? 0u : (static_cast<uint32_t>(live) < ga.inCap ? static_cast<uint32_t>(live) : ga.inCap);
      const bool checkRanks = nLive >= ga.inCap;  // fewer rows than the capacity: nothing was cut off
      const uint32_t rec = blockIdx.x * kRbChunk + threadIdx.x;
      unsigned long long bits = rec < nRecords ? gatherOccupancy<GATHER>(ga, src, rec, nLive, checkRanks) : 0ull;
      if (bits) {  // cells of the brick past the edge of the output grid are no outputs
        const uint32_t q1 = divSmall(rec, static_cast<uint32_t>(ga.mo.nb[3]), ga.rcpX);
        const int bx = static_cast<int>(rec - q1 * static_cast<uint32_t>(ga.mo.nb[3]));
        const int by = static_cast<int>(q1 - divSmall(q1, static_cast<uint32_t>(ga.mo.nb[2]), ga.rcpY) * static_cast<uint32_t>(ga.mo.nb[2]));
        const int rows = ga.shapeY - 8 * by, cols = ga.shapeX - 8 * bx;
        if (rows < 8) bits &= (1ull << (8 * rows)) - 1ull;
        if (cols < 8) bits &= 0x0101010101010101ull * ((1ull << cols) - 1ull);
      }
      chunkBits[threadIdx.x] = bits;
    }
    __syncthreads();
    if (threadIdx.x >= kRbThreads) return;  // (a wavefront that has ended no longer counts at a barrier)
#pragma unroll
    for (int j = 0; j < kRbItems; ++j) {
      gathered[j] = chunkBits[wave * 256 + j * 64 + lane];
      count[j] = static_cast<uint32_t>(__popcll(gathered[j]));
    }
  }
#pragma unroll
  for (int j = 0; j < kRbItems; ++j) {
    if constexpr (GATHER == 0)
      count[j] = first + j * 64 < nRecords ? static_cast<uint32_t>(__popcll(records[first + j * 64].bits)) : 0u;
    if (other && first + j * 64 < nRecords) other[first + j * 64].bits = 0ull;
  }
  uint32_t inclA = count[0] | (count[1] << 16), inclB = count[2] | (count[3] << 16);
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t upA = __shfl_up(inclA, off, 64), upB = __shfl_up(inclB, off, 64);
    if (lane >= off) {
      inclA += upA;
      inclB += upB;
    }
  }
  const uint32_t endA = __shfl(inclA, 63, 64), endB = __shfl(inclB, 63, 64);
  const uint32_t rowSum[kRbItems] = {endA & 0xFFFFu, endA >> 16, endB & 0xFFFFu, endB >> 16};
  const uint32_t incl[kRbItems] = {inclA & 0xFFFFu, inclA >> 16, inclB & 0xFFFFu, inclB >> 16};
  if (lane == 0) scratch[wave] = rowSum[0] + rowSum[1] + rowSum[2] + rowSum[3];
  __syncthreads();
  uint32_t rank = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kRbThreads / 64; ++w) {
    if (w < wave) rank += scratch[w];
    total += scratch[w];
  }
#pragma unroll
  for (int j = 0; j < kRbItems; ++j) {
    // an empty record is never ranked: on sparse grids most are
    if constexpr (GATHER != 0) {
      if (count[j]) {
        const unsigned long long bits = gathered[j];
        *reinterpret_cast<uint4*>(records + first + j * 64) =
            make_uint4(static_cast<uint32_t>(bits), static_cast<uint32_t>(bits >> 32), rank + incl[j] - count[j], 0u);
      }
    } else {
      if (count[j]) records[first + j * 64].prefix = rank + incl[j] - count[j];
    }
    rank += rowSum[j];
  }
  if (threadIdx.x == 0) {
    // The chunk totals are the only data that passes between workgroups inside this kernel, and every access to
    // them is a device-scope atomic.  ORDERED makes the hand-off formal: acquire-release tickets, i.e. a
    // device-scope release per workgroup, which on this part writes the L2 back - measured 6.3 -> 10.9 us per
    // launch on average and 17 -> 50 us on a 1.3 M-record grid, 37 us per pass of eight rulebooks.  The default
    // does without: the total is published with a RETURNING device-scope atomic, which has been performed where
    // every XCD sees it once its result is back (the s_waitcnt below), and only then is the ticket taken, so the
    // workgroup that draws the last ticket cannot read an older total.
    uint32_t old = __hip_atomic_exchange(&chunkBase[blockIdx.x], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(old)::"memory");
    // Atomics on one address are performed one after the other (about 18 ns each across the XCDs), so the
    // tickets are taken in two levels: one counter per kScanGroup workgroups, and only the last of each group
    // goes on to the counter of the whole grid.
    const uint32_t group = blockIdx.x / kScanGroup;
    const uint32_t groupSize = min(kScanGroup, nChunks - group * kScanGroup);
    const uint32_t nGroups = (nChunks + kScanGroup - 1) / kScanGroup;
    uint32_t last = 0;
    constexpr int kOrder = ORDERED ? __ATOMIC_ACQ_REL : __ATOMIC_RELAXED;
    if (__hip_atomic_fetch_add(&groupTickets[group], 1u, kOrder, __HIP_MEMORY_SCOPE_AGENT) == groupSize - 1)
      last = __hip_atomic_fetch_add(ticket, 1u, kOrder, __HIP_MEMORY_SCOPE_AGENT) == nGroups - 1 ? 1u : 0u;
    isLast = last;
  }
  __syncthreads();
  if (!isLast) return;
  // one exclusive scan over all chunk totals: thread t takes a contiguous run of them (all loads in flight at
  // once), scans it in registers, and a single workgroup scan of the run sums supplies the offsets
  constexpr uint32_t kRun = 8;
  uint32_t running = 0;
  for (uint32_t base = 0; base < nChunks; base += kRun * kRbThreads) {
    const uint32_t q0 = base + threadIdx.x * kRun;
    uint32_t v[kRun];
#pragma unroll
    for (uint32_t j = 0; j < kRun; ++j)
      v[j] = q0 + j < nChunks ? __hip_atomic_load(&chunkBase[q0 + j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    uint32_t mineSum = 0;
#pragma unroll
    for (uint32_t j = 0; j < kRun; ++j) mineSum += v[j];
    uint32_t sum;
    uint32_t at = running + blockExclusiveScan(mineSum, scratch, &sum);
#pragma unroll
    for (uint32_t j = 0; j < kRun; ++j) {
      if (q0 + j < nChunks) chunkBase[q0 + j] = at;
      at += v[j];
    }
    running += sum;
    __syncthreads();
  }
  if (threadIdx.x == 0 && numActOut)
    *numActOut = static_cast<int32_t>(running < static_cast<uint32_t>(maxNumActOut) ? running : maxNumActOut);
  // Every other workgroup has drawn its tickets (and read the scan count before that): the counters go back to
  // zero for the next pass, and with two maps the count moves on - the passes behind this one see this map as
  // the finished one, the next build marks the other.
  if (recRef.epoch) {
    const uint32_t nGroups = (nChunks + kScanGroup - 1) / kScanGroup;
    for (uint32_t q = threadIdx.x; q < nGroups; q += kRbThreads) groupTickets[q] = 0u;
    if (threadIdx.x == 0) {
      *ticket = 0u;
      *recRef.epoch = epoch + 1u;
    }
  }
}


constexpr uint32_t kEmitGroup = 8;  // records per wavefront of the coordinate pass

// One cell per lane of an occupied record (bits, global prefix of record `rec`): outCoors[rank] = its coordinate.
__device__ __forceinline__ void emitCells(const RbGeom& g, const BlockMap& m, unsigned long long bits, uint32_t prefix,
                                          uint32_t rec, int32_t* __restrict__ outCoors, int32_t maxNumActOut) {
  uint32_t bit = threadIdx.x & 63;
  if (!((bits >> bit) & 1ull)) return;
  const uint32_t id = prefix + static_cast<uint32_t>(__popcll(bits & ((1ull << bit) - 1ull)));
  if (id >= static_cast<uint32_t>(maxNumActOut)) return;
  const int pad = kMaxSpatial - g.nd;
  int32_t* row = outCoors + static_cast<size_t>(id) * (g.nd + 1);
  uint32_t q = rec;
#pragma unroll
  for (int dim = kMaxSpatial - 1; dim >= 0; --dim) {
    const uint32_t nb = static_cast<uint32_t>(m.nb[dim]);
    const uint32_t brick = q % nb;
    q /= nb;
    const int v = static_cast<int>((brick << m.shift[dim]) + (bit & ((1u << m.shift[dim]) - 1)));
    bit >>= m.shift[dim];
    if (dim >= pad) row[1 + dim - pad] = v;
  }
  row[0] = static_cast<int32_t>(q);
}

// Strided convolutions: output coordinates in rank order (reference: coorsOutOrganizeKernel,
// index.cu:104-121).  A wavefront takes kEmitGroup consecutive records, one per lane, and then walks the occupied
// ones among them with one cell per lane: on a sparse grid most records are empty and cost one load between
// several (a wavefront per 64 records measured 16 -> 41 us on a small dense grid, where every record is a turn of
// the loop; a wavefront per record 42 -> 36 us on a large sparse one).
__device__ __forceinline__ void emitRecordCoords(const RbGeom& g, const BlockMap& m, const BmRecord* __restrict__ records,
                                                 const uint32_t* __restrict__ chunkBase, uint32_t nRecords,
                                                 uint32_t group, int32_t* __restrict__ outCoors, int32_t maxNumActOut) {
  const uint32_t rec0 = group * kEmitGroup;
  if (rec0 >= nRecords) return;  // wavefront-uniform
  const uint32_t lane = threadIdx.x & 63;
  uint32_t lo = 0, hi = 0, prefix = 0;
  if (lane < kEmitGroup && rec0 + lane < nRecords) {
    const uint4 r = *reinterpret_cast<const uint4*>(records + rec0 + lane);
    lo = r.x;
    hi = r.y;
    prefix = r.z;
  }
  unsigned long long occupied = __ballot((lo | hi) != 0u);
  if (occupied == 0ull) return;
  prefix += chunkBase[((lane < kEmitGroup && rec0 + lane < nRecords) ? rec0 + lane : rec0) / kRbChunk];
  while (occupied) {
    const int r = __builtin_ctzll(occupied);
    occupied &= occupied - 1ull;
    const unsigned long long bits =
        (static_cast<unsigned long long>(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(hi), r))) << 32) |
        static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(lo), r));
    const uint32_t pre = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(prefix), r));
    emitCells(g, m, bits, pre, rec0 + static_cast<uint32_t>(r), outCoors, maxNumActOut);
  }
}

__global__ void __launch_bounds__(kRbThreads)
bmEmitCoords(RbGeom g, BlockMap m, RecRef recRef, const uint32_t* __restrict__ chunkBase,
             uint32_t nRecords, int32_t* __restrict__ outCoors, int32_t maxNumActOut) {
  const BmRecord* __restrict__ records = recRef.get();
  emitRecordCoords(g, m, records, chunkBase, nRecords, blockIdx.x * (kRbThreads / 64) + (threadIdx.x >> 6), outCoors,
                   maxNumActOut);
}

// SubM: perm[rank of voxel i] = i (reference: the value side of setSubMHashKernel, index.cu:174-182).
// perm[rank] = input row i (SubM).  Rows that already sit in rank order (the outputs of a strided rulebook of
// this engine do) need no permutation afterwards; any mismatch raises the flag.
__device__ __forceinline__ void permuteRow(const RbGeom& g, const BlockMap& m, const int32_t* __restrict__ coors, int n,
                                           int64_t i, const BmRecord* __restrict__ records,
                                           const uint32_t* __restrict__ chunkBase, uint32_t* __restrict__ perm,
                                           uint32_t* permShuffled) {
  if (i >= n) return;
  int c[5];
  if (!loadInput(g, coors, i, c) || !coordInGrid(g, c)) return;
  uint32_t rec, bit;
  bmLocate(m, c, &rec, &bit);
  const uint32_t rank = bmRank(records[rec], bit, chunkBase, rec);
  perm[rank] = static_cast<uint32_t>(i);
  if (rank != static_cast<uint32_t>(i)) *permShuffled = 1u;
}

__global__ void __launch_bounds__(kRbThreads)
bmPermutation(RbGeom g, BlockMap m, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn,
              int64_t cap, RecRef recRef, const uint32_t* __restrict__ chunkBase,
              uint32_t* __restrict__ perm, uint32_t* permShuffled) {
  const BmRecord* __restrict__ records = recRef.get();
  permuteRow(g, m, coors, liveCount(numActIn, cap), static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x, records,
             chunkBase, perm, permShuffled);
}

// SubM probe / strided resolve on the block map: staging[tap, i] = output row of
// pair (tap, i) or ~0, plus per-(tap, chunk) counts.  For SubM the output row is
// perm[rank]; for strided convolutions it is the rank itself, dropped when it
// falls beyond maxNumActOut (reference: hashOutIndexKernel, index.cu:158-172).
template <bool SUBM>
__global__ void __launch_bounds__(kRbThreads)
bmProbe(RbGeom g, BlockMap m, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
        int64_t pitch, RecRef recRef, const uint32_t* __restrict__ chunkBase,
        const uint32_t* __restrict__ perm, const uint32_t* __restrict__ permShuffled, int32_t maxNumActOut,
        uint32_t* __restrict__ staging, RbCount* __restrict__ cnt, uint32_t nBlocks, uint32_t* totals) {
  const BmRecord* __restrict__ records = recRef.get();
  const int n = liveCount(numActIn, cap);
  const int tap = blockIdx.y;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kRbChunk + threadIdx.x * kRbItems;
  uint32_t found = 0;
  if (static_cast<int64_t>(blockIdx.x) * kRbChunk < n) {  // workgroup-uniform
    int idx[kMaxSpatial];
    tapPositions(g, tap, idx);
    uint32_t row[kRbItems];
#pragma unroll
    for (int j = 0; j < kRbItems; ++j) {
      row[j] = kNone;
      const int64_t i = first + j;
      if (i < n) {
        int c[5], o[5];
        if (loadInput(g, coors, i, c) && tapTargetCoord(g, c, idx, o)) {
          uint32_t rec, bit;
          bmLocate(m, o, &rec, &bit);
          const BmRecord r = records[rec];
          if ((r.bits >> bit) & 1ull) {
            const uint32_t rank = bmRank(r, bit, chunkBase, rec);
            if (SUBM ? rank < static_cast<uint32_t>(n) : rank < static_cast<uint32_t>(maxNumActOut))
              row[j] = rank;  // SubM: the compaction turns ranks into rows through perm[] when rows are shuffled
          }
        }
      }
      found += row[j] != kNone;
    }
    if (first < n) *reinterpret_cast<uint4*>(staging + static_cast<int64_t>(tap) * pitch + first) =
        make_uint4(row[0], row[1], row[2], row[3]);
  }
  publishWaveCounts(found, cnt, nBlocks);
}

// ---------------------------------------------------------------------------
// "Near" passes of the block-map path.  When the taps of one input reach at
// most 2E+1 consecutive output cells in dim 1 and E+1 in dims 2 and 3 (E =
// brick extent of the dim), all targets of that input lie in a 3x2x2 group of
// bricks.  One thread then serves one input: it fetches that group once (12
// independent 16-byte loads, neighbours in memory) and resolves all kVol taps
// from it, instead of one random record access per (tap, input) pair.  A wavefront's memory requests
// drop from 64 lines per tap to a handful per input, which is what bounds
// these passes: the request rate of scattered accesses, not bandwidth.
// Requires the outermost of the four dims to be degenerate (always true for
// 1-D..3-D rulebooks).
// ---------------------------------------------------------------------------
constexpr int kNearGroup = 12;          // members e = e1 * 4 + e2 * 2 + e3 with e1 in 0..2, e2 and e3 in 0..1
constexpr int kNearMembers[kMaxSpatial] = {1, 3, 2, 2};

// Lowest output cell (clamped to 0) any tap of input coordinate `in` can reach in `dim`.
__device__ __forceinline__ int nearBaseCell(const RbGeom& g, int dim, int in) {
  if (g.transpose) {
    const int lo = in * g.s[dim] - g.p[dim];
    return lo > 0 ? lo : 0;
  }
  const int lo = in + g.p[dim] - (g.k[dim] - 1) * g.d[dim];
  if (lo <= 0) return 0;
  const int st = g.s[dim];
  return st == 1 ? lo : (st == 2 ? (lo + 1) >> 1 : (lo + st - 1) / st);
}

struct NearBase {
  int brick[kMaxSpatial];   // lower brick of the group per dim
  uint32_t rec0;            // record index of (brick[0..3])
  bool ok;                  // batch and dim-0 in range
};

__device__ __forceinline__ NearBase nearBase(const RbGeom& g, const BlockMap& m, const int c[5]) {
  NearBase b;
  b.ok = c[0] >= 0 && c[0] < g.shape[0];
  uint32_t r = static_cast<uint32_t>(c[0]);
#pragma unroll
  for (int dim = 0; dim < kMaxSpatial; ++dim) {
    b.brick[dim] = nearBaseCell(g, dim, c[dim + 1]) >> m.shift[dim];
    r = r * static_cast<uint32_t>(m.nb[dim]) + static_cast<uint32_t>(b.brick[dim]);
  }
  b.rec0 = r;
  return b;
}

// Record index offset and validity of group member e = (e1, e2, e3) in {0,1,2} x {0,1}^2.
__device__ __forceinline__ bool nearMember(const BlockMap& m, const NearBase& b, int e, uint32_t* rec) {
  const int e1 = e >> 2, e2 = (e >> 1) & 1, e3 = e & 1;
  *rec = b.rec0 + static_cast<uint32_t>((e1 * m.nb[2] + e2) * m.nb[3] + e3);
  return b.ok && b.brick[0] < m.nb[0] && b.brick[1] + e1 < m.nb[1] && b.brick[2] + e2 < m.nb[2] &&
         b.brick[3] + e3 < m.nb[3];
}

// Calls f(tap, valid, member, bit) for every tap of one input (dim 0 degenerate: k[0] == 1).
template <class Fn>
__device__ __forceinline__ void nearForEachTap(const RbGeom& g, const BlockMap& m, const int c[5], const NearBase& b,
                                               Fn&& f) {
  int o0;
  const bool ok0 = b.ok && tapDim(g, 0, c[1], 0, o0);
  int tap = 0;
  for (int i1 = 0; i1 < g.k[1]; ++i1) {
    int o1;
    const bool ok1 = tapDim(g, 1, c[2], i1, o1) && ok0;
    int e1 = (o1 >> m.shift[1]) - b.brick[1];
    e1 = e1 < 0 ? 0 : (e1 > 2 ? 2 : e1);  // in range by construction when the tap is valid
    for (int i2 = 0; i2 < g.k[2]; ++i2) {
      int o2;
      const bool ok2 = tapDim(g, 2, c[3], i2, o2) && ok1;
      const int e2 = (o2 >> m.shift[2]) - b.brick[2];
      for (int i3 = 0; i3 < g.k[3]; ++i3) {
        int o3;
        const bool ok3 = tapDim(g, 3, c[4], i3, o3) && ok2;
        const int e3 = (o3 >> m.shift[3]) - b.brick[3];
        uint32_t bit = static_cast<uint32_t>(o0) & ((1u << m.shift[0]) - 1);
        bit = (bit << m.shift[1]) | (static_cast<uint32_t>(o1) & ((1u << m.shift[1]) - 1));
        bit = (bit << m.shift[2]) | (static_cast<uint32_t>(o2) & ((1u << m.shift[2]) - 1));
        bit = (bit << m.shift[3]) | (static_cast<uint32_t>(o3) & ((1u << m.shift[3]) - 1));
        f(tap, ok3, (e1 << 2) | ((e2 & 1) << 1) | (e3 & 1), bit);
        ++tap;
      }
    }
  }
}

// The same enumeration for the shapes that matter (3-D, dilation 1, not transposed, kernel sizes known at compile
// time, strides powers of two): everything that depends on one dim only - validity, output cell, brick of the
// group, bit part - is computed once per dim and tap position, the K1*K2*K3 taps are fully unrolled, and a tap
// costs a handful of instructions instead of three calls of the general per-dim routine.
template <int K1, int K2, int K3, class Fn>
__device__ __forceinline__ void nearForEachTapFixed(const RbGeom& g, const BlockMap& m, const int c[5],
                                                    const NearBase& b, Fn&& f) {
  constexpr int KS[3] = {K1, K2, K3};
  bool ok[3][3];
  int member[3][3];
  uint32_t part[3][3];
#pragma unroll
  for (int q = 0; q < 3; ++q) {
    const int dim = q + 1;
    const int st = g.s[dim];                  // 1, 2 or 4
    const int ls = st >> 1 > 1 ? 2 : st >> 1; // log2
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      if (i < KS[q]) {
        const int num = c[dim + 1] + g.p[dim] - i;
        const int o = num >> ls;
        ok[q][i] = num >= 0 && (num & (st - 1)) == 0 && o < g.shape[dim + 1];
        const int mem = (o >> m.shift[dim]) - b.brick[dim];
        member[q][i] = q == 0 ? (mem < 0 ? 0 : (mem > 2 ? 2 : mem)) : (mem & 1);
        part[q][i] = static_cast<uint32_t>(o) & ((1u << m.shift[dim]) - 1);
      } else {
        ok[q][i] = false;
        member[q][i] = 0;
        part[q][i] = 0;
      }
    }
  }
  const bool ok0 = b.ok && c[1] == 0;  // dim 0 is degenerate: extent 1, kernel 1
#pragma unroll
  for (int i1 = 0; i1 < K1; ++i1)
#pragma unroll
    for (int i2 = 0; i2 < K2; ++i2)
#pragma unroll
      for (int i3 = 0; i3 < K3; ++i3) {
        const uint32_t bit = (((part[0][i1] << m.shift[2]) | part[1][i2]) << m.shift[3]) | part[2][i3];
        f((i1 * K2 + i2) * K3 + i3, ok0 && ok[0][i1] && ok[1][i2] && ok[2][i3],
          (member[0][i1] << 2) | (member[1][i2] << 1) | member[2][i3], bit);
      }
}

// KSEL picks the enumeration: 0 = general, else a fixed kernel shape.
template <int KSEL, class Fn>
__device__ __forceinline__ void nearTaps(const RbGeom& g, const BlockMap& m, const int c[5], const NearBase& b, Fn&& f) {
  if constexpr (KSEL == 1) nearForEachTapFixed<3, 3, 3>(g, m, c, b, f);
  else if constexpr (KSEL == 2) nearForEachTapFixed<3, 1, 1>(g, m, c, b, f);
  else if constexpr (KSEL == 3) nearForEachTapFixed<3, 1, 3>(g, m, c, b, f);
  else if constexpr (KSEL == 4) nearForEachTapFixed<1, 3, 3>(g, m, c, b, f);
  else nearForEachTap(g, m, c, b, f);
}

// Record indices of the group members; members outside the grid are clamped to record 0 (so that every
// load is unconditional and all eight issue back to back) and reported absent in the returned mask.
__device__ __forceinline__ uint32_t nearMembers(const BlockMap& m, const NearBase& b, uint32_t rec[kNearGroup]) {
  uint32_t present = 0;
#pragma unroll
  for (int e = 0; e < kNearGroup; ++e) {
    uint32_t r;
    const bool ok = nearMember(m, b, e, &r);
    rec[e] = ok ? r : 0u;
    present |= (ok ? 1u : 0u) << e;
  }
  return present;
}

// Strided / transposed: one thread marks all candidate outputs of one input: per brick of its group one
// atomicOr for each run of neighbouring lanes that target the same brick.
template <int KSEL>
__global__ void __launch_bounds__(kRbThreads)
bmMarkNear(RbGeom g, BlockMap m, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
           RecRef recRef) {
  BmRecord* records = recRef.get();
  __shared__ unsigned long long masks[kNearGroup][kRbThreads];
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kRbThreads + threadIdx.x;
  bool live = i < n;
  int c[5] = {0, 0, 0, 0, 0};
  if (live && !loadInput(g, coors, i, c)) {
    live = false;
    c[0] = c[1] = c[2] = c[3] = c[4] = 0;
  }
  const NearBase b = nearBase(g, m, c);
  uint32_t rec[kNearGroup];
  const uint32_t present = live ? nearMembers(m, b, rec) : (nearMembers(m, b, rec), 0u);
#pragma unroll
  for (int e = 0; e < kNearGroup; ++e) masks[e][threadIdx.x] = 0ull;
  if (live)
    nearTaps<KSEL>(g, m, c, b, [&](int, bool ok, int member, uint32_t bit) {
      if (ok) masks[member][threadIdx.x] |= 1ull << bit;
    });
#pragma unroll
  for (int e = 0; e < kNearGroup; ++e) {
    const unsigned long long want = masks[e][threadIdx.x];
    const bool any = ((present >> e) & 1u) && want;
    // wavefront-uniform: most of the twelve group members get no candidate from any of a wavefront's 64 inputs
    // (a strided kernel reaches two of the three levels, and neighbouring inputs share their bricks)
    if (__ballot(any) == 0ull) continue;
    orRuns(records, any ? rec[e] : kNone, want);
  }
}

// SubM probe / strided resolve, one thread per input (see bmProbe for the per-pair form).
// cnt takes one entry per (tap, 256 inputs).
template <bool SUBM, int KSEL>
__global__ void __launch_bounds__(kRbThreads)
bmProbeNear(RbGeom g, BlockMap m, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
            int64_t pitch, RecRef recRef, const uint32_t* __restrict__ chunkBase,
            uint32_t* __restrict__ perm, uint32_t* permShuffled, int32_t maxNumActOut, uint32_t* __restrict__ staging,
            RbCount* __restrict__ cnt, uint32_t nBlocks, uint32_t* totals, int32_t* fillA, int64_t nFillA, int32_t* fillB,
            int64_t nFillB, uint32_t fillBlocks, int32_t* __restrict__ outCoors, uint32_t nRecords) {
  const BmRecord* __restrict__ records = recRef.get();
  extern __shared__ __attribute__((aligned(16))) unsigned char nearSmem[];
  uint4* group = reinterpret_cast<uint4*>(nearSmem);                                   // [8][kRbThreads] records
  uint32_t* ldsCnt = reinterpret_cast<uint32_t*>(group + kNearGroup * kRbThreads);    // [kVol]
  // Every second workgroup is a fill workgroup: the -1 fill of the index tensor and of the neighbour table is
  // bandwidth-bound, this pass latency-bound, and neither depends on the other, so they share one launch.
  // Workgroups past the interleaved range carry the pass that only the compaction waits for: the rank -> row
  // permutation (SubM) or the output coordinates (strided).
  if (blockIdx.x >= fillBlocks * 2) {
    const uint32_t e = blockIdx.x - fillBlocks * 2;
    if (SUBM) {
      permuteRow(g, m, coors, liveCount(numActIn, cap), static_cast<int64_t>(e) * kRbThreads + threadIdx.x, records,
                 chunkBase, perm, permShuffled);
    } else {
      emitRecordCoords(g, m, records, chunkBase, nRecords, e * (kRbThreads / 64) + (threadIdx.x >> 6), outCoors,
                       maxNumActOut);
    }
    return;
  }
  const uint32_t quad = blockIdx.x >> 1, part = blockIdx.x & 1;
  if (part == 1) {
    if (quad < fillBlocks) {
      const int64_t tid = static_cast<int64_t>(quad) * kRbThreads + threadIdx.x;
      const int64_t stride = static_cast<int64_t>(fillBlocks) * kRbThreads;
      fillMinusOneRange(fillA, nFillA, tid, stride);
      fillMinusOneRange(fillB, nFillB, tid, stride);
    }
    return;
  }
  const uint32_t probeBlock = quad;
  const int n = liveCount(numActIn, cap);
  const int64_t i0 = static_cast<int64_t>(probeBlock) * kRbThreads;
  if (i0 >= n) return;  // workgroup-uniform
  for (int t = threadIdx.x; t < g.kVol; t += blockDim.x) ldsCnt[t] = 0;
  const int64_t i = i0 + threadIdx.x;
  const bool inRange = i < n;   // rows below the live count get a staging entry, in the grid or not
  bool live = inRange;
  int c[5] = {0, 0, 0, 0, 0};
  if (live && !loadInput(g, coors, i, c)) {
    live = false;
    c[0] = c[1] = c[2] = c[3] = c[4] = 0;
  }
  const NearBase b = nearBase(g, m, c);
  uint32_t rec[kNearGroup];
  const uint32_t present = live ? nearMembers(m, b, rec) : (nearMembers(m, b, rec), 0u);
  uint4 loaded[kNearGroup];
  uint32_t base[kNearGroup];
#pragma unroll
  for (int e = 0; e < kNearGroup; ++e) {
    loaded[e] = *reinterpret_cast<const uint4*>(records + (live ? rec[e] : 0u));
    base[e] = chunkBase[(live ? rec[e] : 0u) / kRbChunk];
  }
#pragma unroll
  for (int e = 0; e < kNearGroup; ++e) {
    loaded[e].z += base[e];  // in-chunk prefix -> global prefix
    group[e * kRbThreads + threadIdx.x] = ((present >> e) & 1u) ? loaded[e] : make_uint4(0, 0, 0, 0);
  }
  __syncthreads();  // ldsCnt zeroed
  uint32_t mine = 0;  // lane t of a wavefront counts the wavefront's pairs of tap t (t + 64 for more than 64 taps)
  const int lane = threadIdx.x & 63;
  nearTaps<KSEL>(g, m, c, b, [&](int tap, bool ok, int member, uint32_t bit) {
    uint32_t row = kNone;
    if (live && ok) {
      const uint4 v = group[member * kRbThreads + threadIdx.x];
      const unsigned long long bits = (static_cast<unsigned long long>(v.y) << 32) | v.x;
      if ((bits >> bit) & 1ull) {
        const uint32_t rank = v.z + static_cast<uint32_t>(__popcll(bits & ((1ull << bit) - 1ull)));
        if (SUBM ? rank < static_cast<uint32_t>(n) : rank < static_cast<uint32_t>(maxNumActOut))
          row = rank;  // SubM: the compaction turns ranks into rows through perm[] when rows are shuffled
      }
    }
    if (inRange) staging[static_cast<int64_t>(tap) * pitch + i] = row;
    const uint32_t hits = static_cast<uint32_t>(__popcll(__ballot(row != kNone)));
    if (KSEL != 0) {
      if (lane == tap) mine += hits;           // tap is a compile-time constant below 64 here
    } else if ((threadIdx.x & 63) == 0 && hits) {
      atomicAdd(&ldsCnt[tap], hits);
    }
  });
  if (KSEL != 0 && mine) atomicAdd(&ldsCnt[lane], mine);
  __syncthreads();
  // this workgroup's 256 inputs are one block of counts: plain stores
  for (int t = threadIdx.x; t < g.kVol; t += blockDim.x)
    cnt[static_cast<size_t>(t) * nBlocks + probeBlock] = static_cast<RbCount>(ldsCnt[t]);
}

// The same pass for the kernel shapes of fixedKernelShape (3-D, dilation 1, strides 1 / 2 / 4, not transposed):
// one thread per input resolves all K1*K2*K3 taps.  A brick is one level of the outermost dim, so the taps of
// kernel position i1 along that dim look into the 2x2 bricks of ONE level: 4 record loads per position, all
// K1*4 of them issued before the first is used.  Nothing in the pass is accumulated across workgroups: a
// workgroup owns 256 consecutive inputs, so the pairs per (tap, 256 inputs) go to `cnt` with plain stores, and a
// wavefront owns one 64-row tile, so the tile masks do too (device-wide atomics run at a few per nanosecond on
// this part: the 22 per workgroup of an earlier form of this pass cost more than all its loads and stores).
// Workgroup roles by block index: first the fill workgroups (-1 over the neighbour table, bandwidth-bound work
// beside latency-bound work), then the probing workgroups, then the pass only the compaction waits for
// (rank -> row permutation, or the output coordinates).
constexpr int kProbeThreads = 512;   // inputs per workgroup of the fixed-shape probe = inputs per entry of its counts
constexpr int kProbeShift = 9;
static_assert(1 << kProbeShift == kProbeThreads, "counts per workgroup");

template <bool SUBM, int K1, int K2, int K3>
__global__ void __launch_bounds__(kProbeThreads)
bmProbeFixed(RbGeom g, BlockMap m, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
             int64_t pitch, RecRef recRef, const uint32_t* __restrict__ chunkBase,
             uint32_t* __restrict__ perm, uint32_t* permShuffled, int32_t maxNumActOut, uint32_t* __restrict__ staging,
             RbCount* __restrict__ cnt, uint32_t cntPitch, int32_t* fillA, int64_t nFillA, int32_t* fillB,
             int64_t nFillB, uint32_t fillBlocks, uint32_t probeBlocks, int32_t* __restrict__ outCoors,
             uint32_t nRecords, unsigned long long* __restrict__ maskOut, int64_t nMasks, int fixTail,
             int32_t* __restrict__ nbrDirect, int64_t nbrRows, uint32_t* fillState, int handOver) {
  const BmRecord* __restrict__ records = recRef.get();
  // Besides the staging entries the pass writes what a linked convolution reads: maskOut (SubM, staging rows =
  // rows of the mirrored table) takes the tile masks - a wavefront's 64 inputs are one 64-row tile - and fixTail
  // has the rows between the live count and the capacity set to -1; nbrDirect (strided, index tensor unread)
  // takes the pairs straight into the scattered table nbrDirect[tap][output row] = input row, filled with -1 by
  // the reset pass; staging may then be null.
  constexpr int KP = K2 * K3, KV = K1 * KP;
  static_assert(KV <= 64, "one lane per tap keeps the wavefront's pair counts");
  __shared__ uint32_t ldsCnt[KV];
  if (blockIdx.x < fillBlocks) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * kProbeThreads + threadIdx.x;
    const int64_t stride = static_cast<int64_t>(fillBlocks) * kProbeThreads;
    fillMinusOneRange(fillA, nFillA, tid, stride);
    fillMinusOneRange(fillB, nFillB, tid, stride);
    return;
  }
  const uint32_t probeBlock = blockIdx.x - fillBlocks;
  if (probeBlock >= probeBlocks) {
    const uint32_t e = probeBlock - probeBlocks;
    if (SUBM) {
      permuteRow(g, m, coors, liveCount(numActIn, cap), static_cast<int64_t>(e) * kProbeThreads + threadIdx.x, records,
                 chunkBase, perm, permShuffled);
    } else {
      emitRecordCoords(g, m, records, chunkBase, nRecords, e * (kProbeThreads / 64) + (threadIdx.x >> 6), outCoors,
                       maxNumActOut);
    }
    return;
  }
  const int n = liveCount(numActIn, cap);
  const int64_t i0 = static_cast<int64_t>(probeBlock) * kProbeThreads;
  const int64_t i = i0 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  // a build without a reset pass hands the fill state over itself: the end of what the previous pass used
  if (handOver && probeBlock == 0 && threadIdx.x == 0 && fillState) fillState[0] = fillState[1];
  if (maskOut && probeBlock == probeBlocks - 1) {  // the entries past the last tile that a convolution reads with it
    for (int64_t q = (static_cast<int64_t>(probeBlocks) * kProbeThreads >> 6) + threadIdx.x; q < nMasks; q += kProbeThreads)
      maskOut[q] = 0ull;
  }
  if (i0 >= n) {  // workgroup-uniform: no live input here
    if (fixTail && i < cap) {
#pragma unroll
      for (int q = 0; q < KV; ++q) staging[static_cast<int64_t>(q) * pitch + i] = kNone;
    }
    if (maskOut && lane == 0 && (i >> 6) < nMasks) maskOut[i >> 6] = 0ull;
    return;
  }
  if (threadIdx.x < KV) ldsCnt[threadIdx.x] = 0;
  // rows below the live count get a staging entry, in the grid or not (fixTail: every row below the capacity)
  const bool inRange = i < n || (fixTail && i < cap);
  bool live = i < n;
  int c[5] = {0, 0, 0, 0, 0};   // (b, z, y, x) in c[0], c[2..4]; c[1] is the degenerate dim
  if (live && !loadInput(g, coors, i, c)) {
    live = false;
    c[0] = c[1] = c[2] = c[3] = c[4] = 0;
  }
  live = live && c[0] >= 0 && c[0] < g.shape[0] && c[1] == 0;
  // per dim and kernel position: validity, brick, cell inside the brick
  auto along = [&](int dim, int pos, int* brick, uint32_t* part) {
    const int st = g.s[dim];
    const int ls = st >> 1 > 1 ? 2 : st >> 1;
    const int num = c[dim + 1] + g.p[dim] - pos;
    const int o = num >> ls;
    *brick = o >> m.shift[dim];
    *part = static_cast<uint32_t>(o) & ((1u << m.shift[dim]) - 1);
    return num >= 0 && (num & (st - 1)) == 0 && o < g.shape[dim + 1];
  };
  bool ok1[K1], ok2[K2], ok3[K3];
  int b1[K1], b2[K2], b3[K3];
  uint32_t part1[K1], part2[K2], part3[K3];
#pragma unroll
  for (int q = 0; q < K1; ++q) ok1[q] = along(1, q, &b1[q], &part1[q]) && live;
#pragma unroll
  for (int q = 0; q < K2; ++q) ok2[q] = along(2, q, &b2[q], &part2[q]);
#pragma unroll
  for (int q = 0; q < K3; ++q) ok3[q] = along(3, q, &b3[q], &part3[q]);
  // lower brick of the 2x2 group per dim: that of the highest kernel position (the lowest cell), clamped to 0
  const int base2 = b2[K2 - 1] > 0 ? b2[K2 - 1] : 0, base3 = b3[K3 - 1] > 0 ? b3[K3 - 1] : 0;
  const uint32_t levelRecords = static_cast<uint32_t>(m.nb[2]) * static_cast<uint32_t>(m.nb[3]);
  const uint32_t inLevel = static_cast<uint32_t>(base2 * m.nb[3] + base3);
  // the records of every level first (independent loads), then the taps
  uint32_t lo[K1][4], hi[K1][4], pre[K1][4];
#pragma unroll
  for (int q1 = 0; q1 < K1; ++q1) {
    const uint32_t rec0 = (static_cast<uint32_t>(ok1[q1] ? c[0] : 0) * static_cast<uint32_t>(m.nb[0]) *
                               static_cast<uint32_t>(m.nb[1]) + static_cast<uint32_t>(ok1[q1] ? b1[q1] : 0)) * levelRecords + inLevel;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool present = ok1[q1] && base2 + (e >> 1) < m.nb[2] && base3 + (e & 1) < m.nb[3];
      const uint32_t rec = present ? rec0 + static_cast<uint32_t>((e >> 1) * m.nb[3] + (e & 1)) : 0u;
      const uint4 r = *reinterpret_cast<const uint4*>(records + rec);
      const uint32_t base = chunkBase[rec / kRbChunk];
      lo[q1][e] = present ? r.x : 0u;
      hi[q1][e] = present ? r.y : 0u;
      pre[q1][e] = r.z + base;  // in-chunk prefix -> global prefix
    }
  }
  uint32_t mine = 0;  // lane t of a wavefront counts the wavefront's pairs of tap t
  unsigned long long tileBits = 0;  // wavefront-uniform: (mirrored) taps that some input of the wavefront has
  const uint32_t rankLimit = SUBM ? static_cast<uint32_t>(n) : static_cast<uint32_t>(maxNumActOut);
#pragma unroll
  for (int q1 = 0; q1 < K1; ++q1)
#pragma unroll
    for (int q2 = 0; q2 < K2; ++q2) {
      // the two records of this brick row
      const bool up = ((b2[q2] - base2) & 1) != 0;
      const uint32_t lo0 = pick(up, lo[q1][2], lo[q1][0]), hi0 = pick(up, hi[q1][2], hi[q1][0]), pre0 = pick(up, pre[q1][2], pre[q1][0]);
      const uint32_t lo1 = pick(up, lo[q1][3], lo[q1][1]), hi1 = pick(up, hi[q1][3], hi[q1][1]), pre1 = pick(up, pre[q1][3], pre[q1][1]);
#pragma unroll
      for (int q3 = 0; q3 < K3; ++q3) {
        const bool right = ((b3[q3] - base3) & 1) != 0;
        const unsigned long long bits = (static_cast<unsigned long long>(pick(right, hi1, hi0)) << 32) | pick(right, lo1, lo0);
        const uint32_t prefix = pick(right, pre1, pre0);
        uint32_t row = kNone;
        const uint32_t bit = (((part1[q1] << m.shift[2]) | part2[q2]) << m.shift[3]) | part3[q3];
        if (ok1[q1] && ok2[q2] && ok3[q3] && ((bits >> bit) & 1ull)) {
          const uint32_t rank = prefix + static_cast<uint32_t>(__popcll(bits & ((1ull << bit) - 1ull)));
          // SubM: a rank past the live rows is a cell of a shared map whose row a truncated strided build dropped
          if (rank < rankLimit) row = rank;
        }
        const int tap = (q1 * K2 + q2) * K3 + q3;
        if (nbrDirect && row != kNone && row < static_cast<uint64_t>(nbrRows))
          nbrDirect[static_cast<int64_t>(tap) * nbrRows + row] = static_cast<int32_t>(i);
        if (staging && inRange) staging[static_cast<int64_t>(tap) * pitch + i] = row;
        const uint32_t hits = static_cast<uint32_t>(__popcll(__ballot(row != kNone)));
        if (lane == tap) mine += hits;
        if (hits) tileBits |= 1ull << (KV - 1 - tap);
      }
    }
  if (maskOut && lane == 0 && (i >> 6) < nMasks) maskOut[i >> 6] = tileBits;
  __syncthreads();  // ldsCnt zeroed
  if (mine) atomicAdd(&ldsCnt[lane], mine);
  __syncthreads();
  if (threadIdx.x < KV) cnt[static_cast<size_t>(threadIdx.x) * cntPitch + probeBlock] = static_cast<RbCount>(ldsCnt[threadIdx.x]);
}

size_t alignUp(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

// workgroups of `threads` threads that give every kEmitGroup records a wavefront
uint32_t emitBlocks(uint32_t nRecords, int threads) {
  const uint32_t perBlock = static_cast<uint32_t>(threads / 64) * kEmitGroup;
  return (nRecords + perBlock - 1) / perBlock;
}

uint32_t nextPow2(uint64_t v) {
  uint64_t p = 1;
  while (p < v) p <<= 1;
  return static_cast<uint32_t>(p);
}

// Largest number of taps of one kernel dim that can hit the output lattice
// from a single input coordinate: max over residues r of #{i : (r - i*d) % s == 0}.
int maxCompatibleTaps(int k, int s, int d) {
  int best = 0;
  for (int r = 0; r < s; ++r) {
    int c = 0;
    for (int i = 0; i < k; ++i)
      if (((r - i * d) % s + s) % s == 0) ++c;
    best = c > best ? c : best;
  }
  return best;
}

}  // namespace

namespace {

// Brick shape per number of real spatial dims (extents multiply to 64).
BlockMap makeBlockMap(const RbGeom& g, uint64_t* records) {
  static const int kShifts[kMaxSpatial + 1][kMaxSpatial] = {
      {0, 0, 0, 6}, {0, 0, 0, 6}, {0, 0, 3, 3}, {0, 0, 3, 3}, {1, 1, 2, 2}};
  BlockMap m{};
  uint64_t n = static_cast<uint64_t>(g.shape[0] > 0 ? g.shape[0] : 0);
  for (int dim = 0; dim < kMaxSpatial; ++dim) {
    m.shift[dim] = kShifts[g.nd][dim];
    const int extent = g.shape[dim + 1] > 0 ? g.shape[dim + 1] : 0;
    m.nb[dim] = (extent + (1 << m.shift[dim]) - 1) >> m.shift[dim];
    n *= static_cast<uint64_t>(m.nb[dim]);
  }
  *records = n;
  m.records = static_cast<uint32_t>(n < 0xFFFFFFFFull ? n : 0xFFFFFFFFull);
  return m;
}

constexpr uint64_t kMaxBlockMapBytes = 256ull << 20;

// D3D_RULEBOOK=hash or =blockmap pins the occupancy structure (tests, tuning);
// otherwise the block map is used whenever its records fit kMaxBlockMapBytes.
int structureOverride() {
  const char* e = debugEnv("D3D_RULEBOOK");
  if (!e) return 0;
  if (std::strcmp(e, "hash") == 0) return 1;
  if (std::strcmp(e, "blockmap") == 0) return 2;
  return 0;
}

size_t scanGroups(uint32_t nChunks) { return (static_cast<size_t>(nChunks) + kScanGroup - 1) / kScanGroup; }
size_t totalsWords(int kVol, uint32_t nChunks) {
  return static_cast<size_t>(kVol) * (kTotalSlots + 1) + 2 + scanGroups(nChunks);
}

RbWorkspace planWith(const RbGeom& g, int64_t cap, bool subM, bool blockMap) {
  RbWorkspace w{};
  if (cap < 1) cap = 1;
  w.blockMap = blockMap;
  w.nBlocks = static_cast<uint32_t>((cap + kRbChunk - 1) / kRbChunk);
  w.pitch = static_cast<int64_t>(w.nBlocks) * kRbChunk;
  size_t off = 0;
  if (blockMap) {
    uint64_t records;
    makeBlockMap(g, &records);
    w.nRecords = static_cast<uint32_t>(records);
    w.nChunks = static_cast<uint32_t>((records + kRbChunk - 1) / kRbChunk);
    w.table = off;  // BmRecord [nRecords]
    off = alignUp(off + static_cast<size_t>(records) * sizeof(BmRecord));
    w.ids = off;    // SubM: perm u32 [cap]
    if (subM) off = alignUp(off + static_cast<size_t>(cap) * 4);
    w.ownCnt = off;  // chunk totals u32 [nChunks]
    off = alignUp(off + static_cast<size_t>(w.nChunks > 0 ? w.nChunks : 1) * 4);
  } else {
    uint64_t bound;
    if (subM) {
      bound = static_cast<uint64_t>(cap);
    } else {
      uint64_t perInput = 1;
      for (int dim = 0; dim < kMaxSpatial; ++dim)
        perInput *= g.transpose ? g.k[dim] : maxCompatibleTaps(g.k[dim], g.s[dim], g.d[dim]);
      bound = perInput * static_cast<uint64_t>(cap);
      uint64_t cells = 1;
      for (int dim = 0; dim <= kMaxSpatial; ++dim)
        cells *= static_cast<uint64_t>(g.shape[dim] > 0 ? g.shape[dim] : 1);
      if (cells < bound) bound = cells;
    }
    w.slots = nextPow2(bound * 2 < 1024 ? 1024 : bound * 2);
    w.table = off;
    off = alignUp(off + static_cast<size_t>(w.slots) * 8);
    w.ids = off;
    if (!subM) off = alignUp(off + static_cast<size_t>(w.slots) * 4);
    w.ownCnt = off;
    if (!subM) off = alignUp(off + static_cast<size_t>(g.kVol) * w.nBlocks * 4);
  }
  w.staging = off;
  off = alignUp(off + static_cast<size_t>(g.kVol) * w.pitch * 4);
  // pairs per (tap, block of inputs): rows of cntPitch words, one per 256 inputs (the fixed-shape probe) or per
  // 1024 (the others, which use the head of each row)
  w.cntPitch = static_cast<uint32_t>(((cap + kRbThreads - 1) / kRbThreads + 7) / 8 * 8);
  w.cnt = off;     // RbCount [kVol, cntPitch], followed (the counters are cleared as one range) by
  off = alignUp(off + static_cast<size_t>(g.kVol) * w.cntPitch * sizeof(RbCount), 16);
  w.totals = off;  // [kVol, kTotalSlots] valid pairs per tap in partial sums, [kVol] owned outputs per tap, "rows not
                   // in rank order" flag, scan ticket, first-level scan tickets
  off = alignUp(off + totalsWords(g.kVol, w.nChunks) * 4);
  w.total = off;
  return w;
}

// True if every input's targets fall in one 3x2x2 group of bricks (see the "near" passes).
bool nearEligible(const RbGeom& g, const BlockMap& m) {
  if (g.k[0] != 1) return false;
  for (int dim = 1; dim < kMaxSpatial; ++dim) {
    const int reach = g.transpose ? (g.k[dim] - 1) * g.d[dim] : ((g.k[dim] - 1) * g.d[dim]) / g.s[dim];
    if (reach > ((kNearMembers[dim] - 1) << m.shift[dim])) return false;
  }
  const char* e = debugEnv("D3D_RULEBOOK_NEAR");
  return !(e && e[0] == '0');
}

// 1: 3x3x3, 2: 3x1x1, 3: 3x1x3, 4: 1x3x3 (3-D, dilation 1, strides 1/2/4, not transposed), else 0 = general code.
// D3D_RULEBOOK_FIXED=0 forces the general enumeration (tests).
int fixedKernelShape(const RbGeom& g) {
  const char* e = debugEnv("D3D_RULEBOOK_FIXED");
  if (e && e[0] == '0') return 0;
  if (g.nd != 3 || g.transpose || g.k[0] != 1) return 0;
  for (int dim = 1; dim < kMaxSpatial; ++dim)
    if (g.d[dim] != 1 || (g.s[dim] != 1 && g.s[dim] != 2 && g.s[dim] != 4)) return 0;
  const int k1 = g.k[1], k2 = g.k[2], k3 = g.k[3];
  if (k1 == 3 && k2 == 3 && k3 == 3) return 1;
  if (k1 == 3 && k2 == 1 && k3 == 1) return 2;
  if (k1 == 3 && k2 == 1 && k3 == 3) return 3;
  if (k1 == 1 && k2 == 3 && k3 == 3) return 4;
  return 0;
}

bool blockMapFits(const RbGeom& g) {
  uint64_t records;
  makeBlockMap(g, &records);
  return records > 0 && records * sizeof(BmRecord) <= kMaxBlockMapBytes;
}

}  // namespace

size_t mapStateWords(size_t chunkBaseBytes) { return 4 + scanGroups(static_cast<uint32_t>(chunkBaseBytes / 4)) + 1; }

void blockMapBytes(const RbGeom& g, int64_t cap, size_t* records, size_t* chunkBase) {
  *records = *chunkBase = 0;
  const RbWorkspace w = planRulebookWorkspace(g, cap, false, ~static_cast<size_t>(0));
  if (!w.blockMap) return;
  *records = static_cast<size_t>(w.nRecords) * sizeof(BmRecord);
  *chunkBase = static_cast<size_t>(w.nChunks > 0 ? w.nChunks : 1) * 4;
}

size_t rulebookWorkspaceBytes(const RbGeom& g, int64_t cap, bool subM, bool gridKnown) {
  // enough for either structure, so the choice at enqueue time is free
  size_t need = planWith(g, cap, subM, false).total;
  if (gridKnown && blockMapFits(g)) {
    const size_t bm = planWith(g, cap, subM, true).total;
    if (bm > need) need = bm;
  }
  return need;
}

// The block map pays for every record of the grid (cleared and scanned on each pass) whatever the number of
// voxels; with more than kMaxRecordsPerRow records per row of capacity that costs more than the hash saves
// (measured: 20 000 voxels uniform in a [41,1600,1408] grid, 1.44 M records, 72 per row: 50 us against 36 us on
// the hash; 120 000 LiDAR voxels in [41,1440,1440], 1.33 M records, 11 per row: 63 us against 93 us).
constexpr uint64_t kMaxRecordsPerRow = 32;

RbWorkspace planRulebookWorkspace(const RbGeom& g, int64_t cap, bool subM, size_t workspaceBytes) {
  const int pin = structureOverride();
  if (pin != 1 && blockMapFits(g)) {
    uint64_t records;
    makeBlockMap(g, &records);
    const RbWorkspace w = planWith(g, cap, subM, true);
    if (pin == 2 || (w.total <= workspaceBytes && records <= kMaxRecordsPerRow * static_cast<uint64_t>(cap < 1 ? 1 : cap)))
      return w;
  }
  return planWith(g, cap, subM, false);
}

int32_t launchRulebook(const RbGeom& g, bool subM, const int32_t* coors, const int32_t* numActIn, int64_t cap,
                       int32_t maxNumActOut, int32_t* index, int32_t* numIndex, int32_t* outCoors, int32_t* numActOut,
                       void* workspace, size_t workspaceBytes, RbSide& side, hipStream_t stream) {
  side.masksWritten = false;
  int32_t* const nbrOut = side.nbrRows > 0 ? side.nbr : nullptr;
  const int64_t nbrRows = nbrOut ? side.nbrRows : 0;
  // tile masks go with the table; the fill state lets this pass clear only what the previous one left behind
  unsigned long long* masks = (nbrOut && g.kVol <= 64) ? side.masks : nullptr;
  uint32_t* const fillState = side.fillState;
  const bool incremental = side.incrementalFill && fillState;
  int32_t* const fillIndex = incremental ? nullptr : index;
  if (!coors || !numActIn || !index || !numIndex || (!subM && (!outCoors || !numActOut))) {
    setError("rulebook: null tensor pointer");
    return D3D_ERR_BAD_ARG;
  }
  // 32-bit keys and pair codes: the grid and kVol*cap must stay below 2^31
  uint64_t cells = 1;
  for (int dim = 0; dim <= kMaxSpatial; ++dim) {
    if (g.shape[dim] <= 0) {  // empty grid: nothing can be active
      cells = 0;
      break;
    }
    cells *= static_cast<uint64_t>(g.shape[dim]);
  }
  if (cells >= 0x7FFFFFFFull || static_cast<uint64_t>(g.kVol) * static_cast<uint64_t>(cap) >= 0x7FFFFFFFull) {
    setError("rulebook: grid (%llu cells) or kVol*capacity exceeds the 32-bit key range",
             static_cast<unsigned long long>(cells));
    return D3D_ERR_UNSUPPORTED;
  }
  for (int dim = 0; dim < kMaxSpatial; ++dim) {
    if (g.k[dim] < 1 || g.s[dim] < 1 || g.d[dim] < 1) {
      setError("rulebook: kernel size, stride and dilation must be positive");
      return D3D_ERR_UNSUPPORTED;
    }
  }
  const RbWorkspace w = planRulebookWorkspace(g, cap, subM, workspaceBytes);
  if (!workspace || workspaceBytes < w.total) {
    setError("rulebook: workspace of %zu bytes, %zu needed", workspaceBytes, w.total);
    return D3D_ERR_WORKSPACE;
  }
  if (reinterpret_cast<uintptr_t>(workspace) & 15) {
    setError("rulebook: workspace must be 16-byte aligned");
    return D3D_ERR_BAD_ARG;
  }
  char* ws = static_cast<char*>(workspace);
  uint32_t* staging = reinterpret_cast<uint32_t*>(ws + w.staging);
  int64_t pitch = w.pitch;
  auto* cnt = reinterpret_cast<RbCount*>(ws + w.cnt);
  auto* totals = reinterpret_cast<uint32_t*>(ws + w.totals);
  uint32_t* ownTotals = totals + g.kVol * kTotalSlots;
  const int64_t rowLen = static_cast<int64_t>(g.kVol) * (cap + kSegment);
  const int64_t nIndex = 3 * rowLen;
  const dim3 block(kRbThreads);
  const int64_t inputBlocks = (cap + kRbThreads - 1) / kRbThreads;
  const dim3 perInput(static_cast<unsigned>(inputBlocks > 0 ? inputBlocks : 1));
  const dim3 perTap(w.nBlocks > 0 ? w.nBlocks : 1, g.kVol);
  auto fillGrid = [](int64_t items) {
    int64_t blocks = (items + kRbThreads - 1) / kRbThreads;
    if (blocks > 256 * 16) blocks = 256 * 16;  // streaming fill: cover the CUs several times over
    return dim3(static_cast<unsigned>(blocks < 1 ? 1 : blocks));
  };

  // SubM with stride 1 and padding (k-1)*d/2 in every dim: pairs come in mirrored twins, and the compaction
  // writes the neighbour table row by row (see rbCompact).  D3D_RULEBOOK_MIRROR=0 switches it off (tests).
  bool mirror = subM && nbrOut && nbrRows == cap && !g.transpose;
  for (int dim = 0; dim < kMaxSpatial; ++dim)
    if (g.s[dim] != 1 || 2 * g.p[dim] != (g.k[dim] - 1) * g.d[dim]) mirror = false;
  {
    const char* e = debugEnv("D3D_RULEBOOK_MIRROR");
    if (e && e[0] == '0') mirror = false;
  }
  // Tile masks come with the mirrored table, whose rows are written whole by the lanes that hold them; a scattered
  // table would need an atomic per pair for them (measured: 18 us on a 640k-pair rulebook, more than the
  // convolution saves by skipping taps).
  // The mirrored table's rows are what the probe pass stages (row kVol-1-tap = the output rows of tap's pairs):
  // with 16-byte aligned rows the probe writes them straight into the table - a base at its last row and a
  // negative pitch make staging[tap * pitch + i] that entry - and the compaction reads them from there.
  const bool inPlace = mirror && cap % 4 == 0 && (reinterpret_cast<uintptr_t>(nbrOut) & 15) == 0;
  if (inPlace) {
    staging = reinterpret_cast<uint32_t*>(nbrOut) + static_cast<int64_t>(g.kVol - 1) * nbrRows;
    pitch = -nbrRows;
  }
  if (!mirror) masks = nullptr;
  const int64_t nMasks = masks ? side.nMasks : 0;
  side.masksWritten = masks != nullptr;
  bool nbrFilled = mirror;
  bool skipIndex = false;                     // set below when side.skipIndex can be honoured
  bool directScatter = false;                 // the probe pass writes the scattered table itself
  bool needReset = true;                      // a reset pass opens the build
  int cntShift = 8;                           // log2 of the inputs one entry of cnt covers
  unsigned long long* compactMasks = masks;   // null when the probe pass writes the masks itself
  const uint32_t* compactPerm = nullptr;      // block-map SubM: staging holds ranks, rows = perm[rank] when shuffled
  const uint32_t* compactPermFlag = nullptr;
  if (w.blockMap) {
    uint64_t nRecords64;
    const BlockMap m = makeBlockMap(g, &nRecords64);
    // the map lives in the workspace, or in the caller's buffers that carry it from a strided build to the SubM
    // builds on its outputs
    const bool mapOutside = side.mapRecords && side.mapChunkBase;
    const bool sharedMap = subM && mapOutside && side.useSharedMap;
    auto* records = mapOutside ? static_cast<BmRecord*>(side.mapRecords) : reinterpret_cast<BmRecord*>(ws + w.table);
    auto* perm = reinterpret_cast<uint32_t*>(ws + w.ids);
    auto* chunkBase = mapOutside ? side.mapChunkBase : reinterpret_cast<uint32_t*>(ws + w.ownCnt);
    side.mapWritten = !subM && mapOutside;
    const dim3 perChunk(w.nChunks > 0 ? w.nChunks : 1);
    const bool near = nearEligible(g, m);
    const int ksel = near ? fixedKernelShape(g) : 0;
    // Two maps in turn (no reset pass) when the caller keeps the map and its state between passes and the probe
    // is the fixed-shape one, which leaves nothing else to zero; a SubM build on a shared map follows the build
    // that wrote it.
    const bool twoMaps = mapOutside && side.mapState && side.mapStride > 0 &&
                         (sharedMap ? side.mapDouble
                                    : (side.mapStride == static_cast<int64_t>(w.nRecords) && near && ksel != 0 &&
                                       !side.skipIndex && !side.mapDirty));
    side.mapDouble = twoMaps;
    uint32_t* const epochPtr = twoMaps ? side.mapState : nullptr;
    const uint32_t recStride = twoMaps ? static_cast<uint32_t>(side.mapStride) : 0u;
    const RecRef recBefore{records, epochPtr, recStride, 0u};  // mark and scan
    const RecRef recBehind{records, epochPtr, recStride, 1u};  // behind the scan: probe, coordinates, SubM builds on it
    uint32_t* scanTicket = (twoMaps && !sharedMap) ? side.mapState + 2 : ownTotals + g.kVol + 1;
    uint32_t* permShuffled = (twoMaps && !sharedMap) ? side.mapState + 1 : ownTotals + g.kVol;
    if (subM && !sharedMap) {
      compactPerm = perm;
      compactPermFlag = permShuffled;
    }
    const size_t nearLds = static_cast<size_t>(kNearGroup) * kRbThreads * sizeof(uint4) + static_cast<size_t>(g.kVol) * 4;
    // A build whose index tensor nobody reads (side.skipIndex) writes table and masks in the probe pass and skips
    // the compaction: for the kernel shapes of the plane probe, a SubM build with the mirrored table staged in
    // place, or a strided build with a table to scatter into (which the reset pass then fills with -1, since the
    // probe pass writes entries into it).
    skipIndex = side.skipIndex && near && ksel != 0 && nbrOut && (subM ? (mirror && inPlace) : true);
    // (with the index tensor written it does not pay: the fill, moved into the reset pass, is no longer hidden
    // beside the probe - measured 1-2 us slower per strided build)
    directScatter = skipIndex && !subM;
    const bool probeMasks = subM && mirror && masks && near && ksel != 0;
    if (probeMasks) compactMasks = nullptr;
    side.indexWritten = !skipIndex;
    int32_t* const resetFill = directScatter ? nbrOut : ((near || skipIndex) ? nullptr : fillIndex);
    const int64_t resetFillN = directScatter ? static_cast<int64_t>(g.kVol) * nbrRows : nIndex;
    const int64_t clearRecords = sharedMap ? 0 : static_cast<int64_t>(w.nRecords);
    // A build on a shared map with the fixed-shape probe leaves nothing to zero: the probe writes counts and tile
    // masks with plain stores, the compaction sums the counts itself, numIndex is written last.
    needReset = !((sharedMap || twoMaps) && near && ksel != 0 && !directScatter && !resetFill && compactMasks == nullptr);
    if (needReset)
      hipLaunchKernelGGL(bmReset, fillGrid(clearRecords + (resetFill ? resetFillN / 4 : 0) + 1), block, 0,
                         stream, reinterpret_cast<uint4*>(records), clearRecords,
                         resetFill, resetFillN, reinterpret_cast<uint32_t*>(cnt),
                         static_cast<int64_t>((w.totals - w.cnt) / 4 + totalsWords(g.kVol, w.nChunks)),
                         numIndex, masks, nMasks, fillState);
    // A strided build on the outputs of another strided build, handed that build's finished map: the occupancy of
    // its own map is derived from it inside the scan (bmScan<.., GATHER>), the marking pass and its atomics go.
    int gather = 0;
    GatherArgs ga{};
    if (!subM && !g.transpose && near && side.srcRecords && side.srcChunkBase && g.nd == 3 && ksel != 0) {
      const bool cube = ksel == 1 && g.s[1] == 2 && g.s[2] == 2 && g.s[3] == 2 && (g.p[1] == 0 || g.p[1] == 1) &&
                        g.p[2] == 1 && g.p[3] == 1;
      const bool column = ksel == 2 && g.s[1] == 2 && g.s[2] == 1 && g.s[3] == 1 && g.p[1] == 0 && g.p[2] == 0 && g.p[3] == 0;
      RbGeom gi = g;
      for (int dim = 0; dim <= kMaxSpatial; ++dim) gi.shape[dim] = g.inShape[dim];
      uint64_t inRecords64 = 0;
      const BlockMap mi = makeBlockMap(gi, &inRecords64);
      const char* e = debugEnv("D3D_RULEBOOK_GATHER");
      if ((cube || column) && inRecords64 > 0 && inRecords64 < 0xFFFFFFFFull && w.nRecords < (1u << 24) &&
          !(e && e[0] == '0')) {
        gather = cube ? 1 : 2;
        ga.src = RecRef{const_cast<BmRecord*>(static_cast<const BmRecord*>(side.srcRecords)),
                        side.srcDouble ? side.srcState : nullptr,
                        side.srcDouble ? static_cast<uint32_t>(side.srcStride) : 0u, 1u};
        ga.srcChunkBase = side.srcChunkBase;
        ga.mo = m;
        ga.mi = mi;
        ga.numActIn = numActIn;
        ga.inCap = static_cast<uint32_t>(cap);
        ga.shapeY = g.shape[3];
        ga.shapeX = g.shape[4];
        ga.padZ = g.p[1];
        ga.rcpX = 1.0f / static_cast<float>(m.nb[3]);
        ga.rcpY = 1.0f / static_cast<float>(m.nb[2]);
        ga.rcpZ = 1.0f / static_cast<float>(m.nb[1]);
      }
    }
    side.sourceMapUsed = gather != 0;
    if (sharedMap) {
      // the strided build that wrote these coordinates marked and scanned this very grid
    } else if (gather) {
      // marked inside the scan
    } else if (subM) {
      hipLaunchKernelGGL(bmMarkInputs, perInput, block, 0, stream, g, m, coors, numActIn, cap, recBefore,
                         needReset ? nullptr : permShuffled);
    } else if (near) {
      switch (ksel) {
        case 1: hipLaunchKernelGGL(bmMarkNear<1>, perInput, block, 0, stream, g, m, coors, numActIn, cap, recBefore); break;
        case 2: hipLaunchKernelGGL(bmMarkNear<2>, perInput, block, 0, stream, g, m, coors, numActIn, cap, recBefore); break;
        case 3: hipLaunchKernelGGL(bmMarkNear<3>, perInput, block, 0, stream, g, m, coors, numActIn, cap, recBefore); break;
        case 4: hipLaunchKernelGGL(bmMarkNear<4>, perInput, block, 0, stream, g, m, coors, numActIn, cap, recBefore); break;
        default: hipLaunchKernelGGL(bmMarkNear<0>, perInput, block, 0, stream, g, m, coors, numActIn, cap, recBefore);
      }
    } else {
      hipLaunchKernelGGL(bmMarkCandidates, perTap, block, 0, stream, g, m, coors, numActIn, cap, recBefore);
    }
    // D3D_RULEBOOK_ORDERED_SCAN=1: acquire-release tickets (see bmScan)
#define D3D_LAUNCH_SCAN(ORDERED, GATHER)                                                                          \
  hipLaunchKernelGGL((bmScan<ORDERED, GATHER>), perChunk, dim3(GATHER ? kRbChunk : kRbThreads), 0, stream, recBefore, w.nRecords, chunkBase, \
                     w.nChunks, scanTicket, scanTicket + 1, subM ? nullptr : numActOut, maxNumActOut, ga)
    const bool ordered = debugEnv("D3D_RULEBOOK_ORDERED_SCAN") != nullptr;
    if (sharedMap) {
    } else if (gather == 1) {
      if (ordered) D3D_LAUNCH_SCAN(true, 1); else D3D_LAUNCH_SCAN(false, 1);
    } else if (gather == 2) {
      if (ordered) D3D_LAUNCH_SCAN(true, 2); else D3D_LAUNCH_SCAN(false, 2);
    } else {
      if (ordered) D3D_LAUNCH_SCAN(true, 0); else D3D_LAUNCH_SCAN(false, 0);
    }
#undef D3D_LAUNCH_SCAN
    if (!near) {  // the near probe launch carries these passes itself
      if (!subM)
        hipLaunchKernelGGL(bmEmitCoords, dim3(emitBlocks(w.nRecords, kRbThreads)), block, 0, stream,
                           g, m, recBehind, chunkBase, w.nRecords, outCoors, maxNumActOut);
      if (subM && !sharedMap)
        hipLaunchKernelGGL(bmPermutation, perInput, block, 0, stream, g, m, coors, numActIn, cap, recBehind, chunkBase,
                           perm, permShuffled);
    }
    if (near) {  // probe workgroups interleaved 1:1 with fill workgroups (index tensor, neighbour table)
      const uint32_t probeBlocks = perInput.x;
      const uint32_t quads = probeBlocks;
      const uint32_t extra = sharedMap ? 0u : (subM ? probeBlocks : emitBlocks(w.nRecords, kRbThreads));
      const dim3 fused(quads * 2 + extra);
      int32_t* fillB = (nbrOut && nbrRows > 0 && !mirror && !directScatter) ? nbrOut : nullptr;
      int32_t* const probeFillIndex = skipIndex ? nullptr : fillIndex;
      const int64_t nFillB = fillB ? static_cast<int64_t>(g.kVol) * nbrRows : 0;
      nbrFilled = true;
#define D3D_LAUNCH_PROBE_NEAR(SUBM, KSEL)                                                                          \
  hipLaunchKernelGGL((bmProbeNear<SUBM, KSEL>), fused, block, nearLds, stream, g, m, coors, numActIn, cap, pitch,   \
                     recBehind, chunkBase, perm, permShuffled, maxNumActOut, staging, cnt, w.cntPitch, nullptr, fillIndex, \
                     nIndex, fillB, nFillB, quads, outCoors, w.nRecords)
      // fixed kernel shapes: K1 threads per input; fill workgroups only for what there is to fill
      const int64_t fillItems = (probeFillIndex ? nIndex : 0) + nFillB;
      uint32_t planeFill = static_cast<uint32_t>((fillItems / 4 + kRbThreads - 1) / kRbThreads);
      if (planeFill > 1024) planeFill = 1024;
      // the fixed-shape probe runs workgroups of kProbeThreads inputs
      const uint32_t fixedBlocks = static_cast<uint32_t>((cap + kProbeThreads - 1) / kProbeThreads > 0 ? (cap + kProbeThreads - 1) / kProbeThreads : 1);
      const uint32_t fixedExtra = sharedMap ? 0u : (subM ? fixedBlocks : emitBlocks(w.nRecords, kProbeThreads));
      planeFill = (planeFill * kRbThreads + kProbeThreads - 1) / kProbeThreads;
#define D3D_LAUNCH_PROBE_PLANE(SUBM, K1, K2, K3)                                                                    \
  hipLaunchKernelGGL((bmProbeFixed<SUBM, K1, K2, K3>), dim3(planeFill + fixedBlocks + fixedExtra), dim3(kProbeThreads), 0, stream, \
                     g, m, coors, numActIn, cap, pitch, recBehind, chunkBase, perm, permShuffled, maxNumActOut,   \
                     (directScatter && skipIndex) ? nullptr : staging, cnt, w.cntPitch, probeFillIndex,             \
                     nIndex, fillB, nFillB, planeFill,                                                               \
                     fixedBlocks, outCoors, w.nRecords, probeMasks ? masks : nullptr, nMasks,                        \
                     (subM && inPlace) ? 1 : 0, directScatter ? nbrOut : nullptr, nbrRows, fillState,               \
                     needReset ? 0 : 1)
      cntShift = ksel != 0 ? kProbeShift : 8;  // the one-thread-per-input probes count per workgroup
      if (subM) {
        switch (ksel) {
          case 1: D3D_LAUNCH_PROBE_PLANE(true, 3, 3, 3); break;
          case 2: D3D_LAUNCH_PROBE_PLANE(true, 3, 1, 1); break;
          case 3: D3D_LAUNCH_PROBE_PLANE(true, 3, 1, 3); break;
          case 4: D3D_LAUNCH_PROBE_PLANE(true, 1, 3, 3); break;
          default: D3D_LAUNCH_PROBE_NEAR(true, 0);
        }
      } else {
        switch (ksel) {
          case 1: D3D_LAUNCH_PROBE_PLANE(false, 3, 3, 3); break;
          case 2: D3D_LAUNCH_PROBE_PLANE(false, 3, 1, 1); break;
          case 3: D3D_LAUNCH_PROBE_PLANE(false, 3, 1, 3); break;
          case 4: D3D_LAUNCH_PROBE_PLANE(false, 1, 3, 3); break;
          default: D3D_LAUNCH_PROBE_NEAR(false, 0);
        }
      }
#undef D3D_LAUNCH_PROBE_PLANE
#undef D3D_LAUNCH_PROBE_NEAR
    } else if (subM) {
      hipLaunchKernelGGL(bmProbe<true>, perTap, block, 0, stream, g, m, coors, numActIn, cap, pitch, recBehind, chunkBase, perm,
                         permShuffled, maxNumActOut, staging, cnt, w.cntPitch, nullptr);
    } else {
      hipLaunchKernelGGL(bmProbe<false>, perTap, block, 0, stream, g, m, coors, numActIn, cap, pitch, recBehind, chunkBase, perm,
                         permShuffled, maxNumActOut, staging, cnt, w.cntPitch, nullptr);
    }
  } else {
    auto* table = reinterpret_cast<unsigned long long*>(ws + w.table);
    auto* ids = reinterpret_cast<uint32_t*>(ws + w.ids);
    auto* ownCnt = reinterpret_cast<uint32_t*>(ws + w.ownCnt);
    const uint32_t mask = w.slots - 1;
    const int64_t nTable16 = static_cast<int64_t>(w.slots) / 2;
    hipLaunchKernelGGL(rbReset, fillGrid(nTable16 + (incremental ? 0 : nIndex / 4) + 1), block, 0, stream,
                       reinterpret_cast<uint4*>(table), nTable16, fillIndex, nIndex, totals, g.kVol * (kTotalSlots + 1), numIndex, masks,
                       nMasks, fillState);
    if (subM) {
      hipLaunchKernelGGL(rbSubmInsert, perInput, block, 0, stream, g, coors, numActIn, cap, table, mask);
      hipLaunchKernelGGL(rbSubmProbe, perTap, block, 0, stream, g, coors, numActIn, cap, pitch, table, mask,
                         staging, cnt, w.cntPitch, nullptr);
    } else {
      hipLaunchKernelGGL(rbConvInsert, perTap, block, 0, stream, g, coors, numActIn, cap, pitch, table, mask,
                         staging);
      hipLaunchKernelGGL(rbConvOwner, perTap, block, 0, stream, g, numActIn, cap, pitch, table, staging, ownCnt,
                         w.nBlocks, ownTotals);
      hipLaunchKernelGGL(rbConvAssign, perTap, block, 0, stream, g, numActIn, cap, pitch, table, staging, ownCnt,
                         w.nBlocks, ownTotals, ids, outCoors, numActOut, maxNumActOut);
      hipLaunchKernelGGL(rbConvResolve, perTap, block, 0, stream, numActIn, cap, pitch, ids, staging, maxNumActOut,
                         cnt, w.cntPitch, nullptr);
    }
  }
  if (nbrOut && nbrRows > 0 && !nbrFilled)
    hipLaunchKernelGGL(rbFillMinusOne, fillGrid(static_cast<int64_t>(g.kVol) * nbrRows / 4 + 1), block, 0, stream, nbrOut,
                       static_cast<int64_t>(g.kVol) * nbrRows);
  // with the index tensor unwritten only a build that may have to turn ranks into rows needs the whole grid; the
  // others launch the one workgroup that writes numIndex
  const int64_t compactRun = static_cast<int64_t>(kCompactWaves) << cntShift;  // a wavefront per block of counts
  const dim3 allSpans(static_cast<unsigned>((cap + compactRun - 1) / compactRun > 0 ? (cap + compactRun - 1) / compactRun : 1),
                      g.kVol);
  const dim3 compactGrid = (skipIndex && !compactPerm) ? dim3(1, 1) : allSpans;
#define D3D_LAUNCH_COMPACT(MIRROR, SKIP, SHIFT)                                                                       \
  hipLaunchKernelGGL((rbCompact<MIRROR, SKIP, SHIFT>), compactGrid, dim3(kCompactThreads),                            \
                     static_cast<size_t>(g.kVol) * 4, stream, numActIn, cap, pitch, g.kVol, staging, cnt, w.cntPitch,  \
                     index, index + rowLen, index + 2 * rowLen, numIndex,                                             \
                     (nbrRows > 0 && !directScatter) ? nbrOut : nullptr, nbrRows, compactPerm, compactPermFlag,        \
                     inPlace ? 1 : 0, compactMasks, fillState, incremental ? 1 : 0)
#define D3D_LAUNCH_COMPACT_SHIFT(MIRROR, SKIP)                        \
  do {                                                                \
    if (cntShift == 8) D3D_LAUNCH_COMPACT(MIRROR, SKIP, 8);           \
    else D3D_LAUNCH_COMPACT(MIRROR, SKIP, 9);                         \
  } while (0)
  if (skipIndex) {
    if (mirror) D3D_LAUNCH_COMPACT_SHIFT(true, true); else D3D_LAUNCH_COMPACT_SHIFT(false, true);
  } else {
    if (mirror) D3D_LAUNCH_COMPACT_SHIFT(true, false); else D3D_LAUNCH_COMPACT_SHIFT(false, false);
  }
#undef D3D_LAUNCH_COMPACT_SHIFT
#undef D3D_LAUNCH_COMPACT
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

}  // namespace d3d
