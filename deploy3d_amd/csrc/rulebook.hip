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
//  * the coordinate hash is one 64-bit slot per entry (key<<32 | value) in
//    HBM, claimed with a single 64-bit CAS, so a probe is one 8-byte load;
//  * compaction is ballot/popcount inside a wavefront plus per-workgroup tap
//    counts; each workgroup sums the counts of its predecessors itself, so no
//    device-wide scan kernels and no full-capacity staging passes are needed;
//  * strided outputs are numbered by their first contributing (input row, tap)
//    via atomicMin, which makes the output order deterministic (the reference
//    numbers them by hash-slot order, which depends on CAS races);
//  * the strided hash is sized by the real bound on distinct outputs per input
//    (product over dims of the largest number of stride-compatible taps), not
//    by 2*kVol*N slots.
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
      atomicMin(table + slot, packed);
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
  const int pad = kMaxSpatial - nd;
  c[0] = row[0];
#pragma unroll
  for (int dim = 0; dim < kMaxSpatial; ++dim) c[dim + 1] = dim >= pad ? row[1 + dim - pad] : 0;
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
    if (c % g.s[dim] != 0) return false;
    out = c / g.s[dim];
  }
  return out >= 0 && out < g.shape[dim + 1];
}

// Calls f(tap, valid, offset) for the kVol taps of one input voxel in
// row-major tap order; offset is the linear offset of the output voxel in the
// output grid and only meaningful when valid.
template <class F>
__device__ __forceinline__ void forEachTap(const RbGeom& g, const int c[5], F&& f) {
  const bool batchOk = c[0] >= 0 && c[0] < g.shape[0];
  int tap = 0;
  for (int i0 = 0; i0 < g.k[0]; ++i0) {
    int o0;
    const bool ok0 = tapDim(g, 0, c[1], i0, o0) && batchOk;
    const uint32_t off0 = static_cast<uint32_t>(c[0]) * g.shape[1] + o0;
    for (int i1 = 0; i1 < g.k[1]; ++i1) {
      int o1;
      const bool ok1 = tapDim(g, 1, c[2], i1, o1) && ok0;
      const uint32_t off1 = off0 * g.shape[2] + o1;
      for (int i2 = 0; i2 < g.k[2]; ++i2) {
        int o2;
        const bool ok2 = tapDim(g, 2, c[3], i2, o2) && ok1;
        const uint32_t off2 = off1 * g.shape[3] + o2;
        for (int i3 = 0; i3 < g.k[3]; ++i3) {
          int o3;
          const bool ok3 = tapDim(g, 3, c[4], i3, o3) && ok2;
          f(tap, ok3, off2 * g.shape[4] + o3);
          ++tap;
        }
      }
    }
  }
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

// ---------------------------------------------------------------------------
// reset: hash slots = EMPTY, index tensor = -1, tap totals = 0.  One streaming
// pass of 16-byte stores (replaces resetHashKernel + the cudaMemsetAsync calls
// of trt/spconv/index.cu:309-314, :352-354).
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kRbThreads)
rbReset(uint4* table16, int64_t nTable16, int32_t* index, int64_t nIndex, uint32_t* totals, int kVol,
        int32_t* numIndex) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
  for (int64_t i = tid; i < nTable16; i += stride) table16[i] = ones;
  // index tensor: 16-byte body when the base is aligned, scalar head/tail otherwise
  const uintptr_t base = reinterpret_cast<uintptr_t>(index);
  int64_t head = ((16 - (base & 15)) & 15) >> 2;
  if (head > nIndex) head = nIndex;
  const int64_t body16 = (nIndex - head) >> 2;
  uint4* body = reinterpret_cast<uint4*>(index + head);
  for (int64_t i = tid; i < body16; i += stride) body[i] = ones;
  const int64_t tailStart = head + (body16 << 2);
  if (tid < head) index[tid] = -1;
  if (tid < nIndex - tailStart) index[tailStart + tid] = -1;
  if (tid < kVol) totals[tid] = 0;
  if (tid == 0) *numIndex = 0;
}

// ---------------------------------------------------------------------------
// SubM: coordinate -> row map (reference: setSubMHashKernel, index.cu:174-182)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kRbThreads)
rbSubmInsert(RbGeom g, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
             unsigned long long* table, uint32_t mask) {
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int c[5];
  loadCoord(coors, g.nd, i, c);
  if (!coordInGrid(g, c)) return;
  hashInsertMin(table, mask, coordOffset(g, c), static_cast<uint32_t>(i));
}

// Shared tail of the probe / resolve kernels: per-tap valid counts of this
// workgroup, accumulated in LDS by one lane per wavefront.
__device__ __forceinline__ void countTap(uint32_t* ldsCnt, int tap, bool valid) {
  const unsigned long long m = __ballot(valid);
  if ((threadIdx.x & 63) == 0 && m) atomicAdd(&ldsCnt[tap], static_cast<uint32_t>(__popcll(m)));
}

__device__ __forceinline__ void publishCounts(const uint32_t* ldsCnt, int kVol, uint32_t* cnt, uint32_t nBlocks,
                                              uint32_t* totals) {
  __syncthreads();
  for (int t = threadIdx.x; t < kVol; t += blockDim.x) {
    const uint32_t v = ldsCnt[t];
    cnt[static_cast<size_t>(t) * nBlocks + blockIdx.x] = v;
    if (v) atomicAdd(&totals[t], v);
  }
}

// SubM probe (reference: subMGeometryKernel + SubMHashWriter, index.cu:48-84):
// staging[tap, i] = row of the voxel at (coord_i + p - tap*d), or ~0.
__global__ void __launch_bounds__(kRbThreads)
rbSubmProbe(RbGeom g, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
            const unsigned long long* __restrict__ table, uint32_t mask, uint32_t* __restrict__ staging,
            uint32_t* __restrict__ cnt, uint32_t nBlocks, uint32_t* totals) {
  extern __shared__ uint32_t ldsCnt[];
  for (int t = threadIdx.x; t < g.kVol; t += blockDim.x) ldsCnt[t] = 0;
  __syncthreads();
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const bool live = i < n;
  int c[5] = {0, 0, 0, 0, 0};
  if (live) loadCoord(coors, g.nd, i, c);
  if (static_cast<int64_t>(blockIdx.x) * blockDim.x < n) {  // workgroup-uniform
    forEachTap(g, c, [&](int tap, bool ok, uint32_t off) {
      uint32_t row = kNone;
      if (live && ok) row = hashLookup(table, mask, off);
      if (live) staging[static_cast<size_t>(tap) * cap + i] = row;
      countTap(ldsCnt, tap, row != kNone);
    });
  }
  publishCounts(ldsCnt, g.kVol, cnt, nBlocks, totals);
}

// ---------------------------------------------------------------------------
// Strided / transposed convolution (reference: convGeometryKernel, index.cu:86-102)
// ---------------------------------------------------------------------------
// Pass 1: every candidate output is inserted with value = i*kVol + tap, the
// smallest value per key surviving; staging[tap, i] = slot.
__global__ void __launch_bounds__(kRbThreads)
rbConvInsert(RbGeom g, const int32_t* __restrict__ coors, const int32_t* __restrict__ numActIn, int64_t cap,
             unsigned long long* table, uint32_t mask, uint32_t* __restrict__ staging) {
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int c[5];
  loadCoord(coors, g.nd, i, c);
  const uint32_t codeBase = static_cast<uint32_t>(i) * static_cast<uint32_t>(g.kVol);
  forEachTap(g, c, [&](int tap, bool ok, uint32_t off) {
    uint32_t slot = kNone;
    if (ok) slot = hashInsertMin(table, mask, off, codeBase + tap);
    staging[static_cast<size_t>(tap) * cap + i] = slot;
  });
}

// Pass 2: a pair owns its output iff its code is the surviving value.  Counts
// owned outputs per input and scans them inside the workgroup.
__global__ void __launch_bounds__(kRbThreads)
rbConvOwner(RbGeom g, const int32_t* __restrict__ numActIn, int64_t cap, const unsigned long long* __restrict__ table,
            const uint32_t* __restrict__ staging, uint32_t* __restrict__ ownPrefix, uint32_t* __restrict__ blockOwn) {
  __shared__ uint32_t scratch[kRbThreads / 64];
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  uint32_t own = 0;
  if (i < n) {
    const uint32_t codeBase = static_cast<uint32_t>(i) * static_cast<uint32_t>(g.kVol);
    for (int tap = 0; tap < g.kVol; ++tap) {
      const uint32_t slot = staging[static_cast<size_t>(tap) * cap + i];
      if (slot != kNone && static_cast<uint32_t>(table[slot]) == codeBase + tap) ++own;
    }
  }
  uint32_t total;
  const uint32_t prefix = blockExclusiveScan(own, scratch, &total);
  if (i < n) ownPrefix[i] = prefix;
  if (threadIdx.x == 0) blockOwn[blockIdx.x] = total;
}

// Pass 3: output rows are numbered in (owner input row, tap) order; writes the
// output coordinates (reference: coorsOutOrganizeKernel, index.cu:104-121) and
// numActOut = min(total, maxNumActOut).
__global__ void __launch_bounds__(kRbThreads)
rbConvAssign(RbGeom g, const int32_t* __restrict__ numActIn, int64_t cap, const unsigned long long* __restrict__ table,
             const uint32_t* __restrict__ staging, const uint32_t* __restrict__ ownPrefix,
             const uint32_t* __restrict__ blockOwn, uint32_t nBlocks, uint32_t* __restrict__ ids,
             int32_t* __restrict__ outCoors, int32_t* numActOut, int32_t maxNumActOut) {
  __shared__ uint32_t scratch[kRbThreads / 64];
  uint32_t before = 0, all = 0;
  for (uint32_t b = threadIdx.x; b < nBlocks; b += blockDim.x) {
    const uint32_t v = blockOwn[b];
    all += v;
    if (b < blockIdx.x) before += v;
  }
  const uint32_t base = blockSum(before, scratch);
  if (blockIdx.x == 0) {
    const uint32_t total = blockSum(all, scratch);
    if (threadIdx.x == 0)
      *numActOut = static_cast<int32_t>(total < static_cast<uint32_t>(maxNumActOut) ? total : maxNumActOut);
  }
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  uint32_t next = base + ownPrefix[i];
  const uint32_t codeBase = static_cast<uint32_t>(i) * static_cast<uint32_t>(g.kVol);
  const int cw = g.nd + 1;
  const int pad = kMaxSpatial - g.nd;
  for (int tap = 0; tap < g.kVol; ++tap) {
    const uint32_t slot = staging[static_cast<size_t>(tap) * cap + i];
    if (slot == kNone) continue;
    const unsigned long long entry = table[slot];
    if (static_cast<uint32_t>(entry) != codeBase + tap) continue;
    ids[slot] = next;
    if (next < static_cast<uint32_t>(maxNumActOut)) {
      // reference: Size::deserialize, trt/include/common/refnd.h:56-64
      uint32_t off = static_cast<uint32_t>(entry >> 32);
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
// (reference: hashOutIndexKernel, index.cu:158-172), plus per-tap counts.
__global__ void __launch_bounds__(kRbThreads)
rbConvResolve(RbGeom g, const int32_t* __restrict__ numActIn, int64_t cap, const uint32_t* __restrict__ ids,
              uint32_t* __restrict__ staging, int32_t maxNumActOut, uint32_t* __restrict__ cnt, uint32_t nBlocks,
              uint32_t* totals) {
  extern __shared__ uint32_t ldsCnt[];
  for (int t = threadIdx.x; t < g.kVol; t += blockDim.x) ldsCnt[t] = 0;
  __syncthreads();
  const int n = liveCount(numActIn, cap);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const bool live = i < n;
  if (static_cast<int64_t>(blockIdx.x) * blockDim.x < n) {  // workgroup-uniform
    for (int tap = 0; tap < g.kVol; ++tap) {
      uint32_t row = kNone;
      if (live) {
        const uint32_t slot = staging[static_cast<size_t>(tap) * cap + i];
        if (slot != kNone) {
          const uint32_t id = ids[slot];
          if (id < static_cast<uint32_t>(maxNumActOut)) row = id;
        }
        staging[static_cast<size_t>(tap) * cap + i] = row;
      }
      countTap(ldsCnt, tap, row != kNone);
    }
  }
  publishCounts(ldsCnt, g.kVol, cnt, nBlocks, totals);
}

// ---------------------------------------------------------------------------
// Compaction (reference: Valid_Counter scan + outputIndexPadOrganizeKernel +
// indexOrganizeKernel, index.cu:123-156, :352-366).  Workgroup (b, tap) writes
// the valid pairs of inputs [256b, 256b+256) of one tap at
//   segment start of the tap  +  pairs of that tap in earlier workgroups  +  rank.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kRbThreads)
rbCompact(const int32_t* __restrict__ numActIn, int64_t cap, int kVol, const uint32_t* __restrict__ staging,
          const uint32_t* __restrict__ cnt, uint32_t nBlocks, const uint32_t* __restrict__ totals,
          int32_t* __restrict__ gather, int32_t* __restrict__ scatter, int32_t* __restrict__ tapRow,
          int32_t* numIndex) {
  __shared__ uint32_t scratch[kRbThreads / 64];
  const int tap = blockIdx.y;
  const uint32_t b = blockIdx.x;
  if (b == 0 && tap == 0 && threadIdx.x == 0) {
    uint32_t end = 0;
    for (int t = 0; t < kVol; ++t) end += (totals[t] + (kSegment - 1)) & ~static_cast<uint32_t>(kSegment - 1);
    *numIndex = static_cast<int32_t>(end);
  }
  const int n = liveCount(numActIn, cap);
  if (static_cast<int64_t>(b) * blockDim.x >= n) return;  // workgroup-uniform
  if (cnt[static_cast<size_t>(tap) * nBlocks + b] == 0) return;  // workgroup-uniform

  uint32_t before = 0;
  for (uint32_t q = threadIdx.x; q < b; q += blockDim.x) before += cnt[static_cast<size_t>(tap) * nBlocks + q];
  uint32_t pos = blockSum(before, scratch);
  for (int t = 0; t < tap; ++t) pos += (totals[t] + (kSegment - 1)) & ~static_cast<uint32_t>(kSegment - 1);

  const int64_t i = static_cast<int64_t>(b) * blockDim.x + threadIdx.x;
  const uint32_t row = i < n ? staging[static_cast<size_t>(tap) * cap + i] : kNone;
  const bool valid = row != kNone;
  uint32_t total;
  const uint32_t rank = blockExclusiveScan(valid ? 1u : 0u, scratch, &total);
  if (valid) {
    gather[pos + rank] = static_cast<int32_t>(i);
    scatter[pos + rank] = static_cast<int32_t>(row);
    tapRow[pos + rank] = tap;
  }
}

size_t alignUp(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

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

RbWorkspace planRulebookWorkspace(const RbGeom& g, int64_t cap, bool subM) {
  RbWorkspace w{};
  if (cap < 1) cap = 1;
  uint64_t bound;
  if (subM) {
    bound = static_cast<uint64_t>(cap);
  } else {
    uint64_t perInput = 1;
    for (int dim = 0; dim < kMaxSpatial; ++dim)
      perInput *= g.transpose ? g.k[dim] : maxCompatibleTaps(g.k[dim], g.s[dim], g.d[dim]);
    bound = perInput * static_cast<uint64_t>(cap);
    uint64_t cells = 1;
    for (int dim = 0; dim <= kMaxSpatial; ++dim) cells *= static_cast<uint64_t>(g.shape[dim] > 0 ? g.shape[dim] : 1);
    if (cells < bound) bound = cells;
  }
  w.slots = nextPow2(bound * 2 < 1024 ? 1024 : bound * 2);
  w.nBlocks = static_cast<uint32_t>((cap + kRbThreads - 1) / kRbThreads);
  size_t off = 0;
  w.table = off;
  off = alignUp(off + static_cast<size_t>(w.slots) * 8);
  w.ids = off;
  if (!subM) off = alignUp(off + static_cast<size_t>(w.slots) * 4);
  w.staging = off;
  off = alignUp(off + static_cast<size_t>(g.kVol) * cap * 4);
  w.ownPrefix = off;
  if (!subM) off = alignUp(off + static_cast<size_t>(cap) * 4);
  w.blockOwn = off;
  if (!subM) off = alignUp(off + static_cast<size_t>(w.nBlocks) * 4);
  w.cnt = off;
  off = alignUp(off + static_cast<size_t>(g.kVol) * w.nBlocks * 4);
  w.totals = off;
  off = alignUp(off + static_cast<size_t>(g.kVol) * 4);
  w.total = off;
  return w;
}

int32_t launchRulebook(const RbGeom& g, bool subM, const int32_t* coors, const int32_t* numActIn, int64_t cap,
                       int32_t maxNumActOut, int32_t* index, int32_t* numIndex, int32_t* outCoors, int32_t* numActOut,
                       void* workspace, size_t workspaceBytes, hipStream_t stream) {
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
  const RbWorkspace w = planRulebookWorkspace(g, cap, subM);
  if (!workspace || workspaceBytes < w.total) {
    setError("rulebook: workspace of %zu bytes, %zu needed", workspaceBytes, w.total);
    return D3D_ERR_WORKSPACE;
  }
  if (reinterpret_cast<uintptr_t>(workspace) & 15) {
    setError("rulebook: workspace must be 16-byte aligned");
    return D3D_ERR_BAD_ARG;
  }
  char* ws = static_cast<char*>(workspace);
  auto* table = reinterpret_cast<unsigned long long*>(ws + w.table);
  auto* ids = reinterpret_cast<uint32_t*>(ws + w.ids);
  auto* staging = reinterpret_cast<uint32_t*>(ws + w.staging);
  auto* ownPrefix = reinterpret_cast<uint32_t*>(ws + w.ownPrefix);
  auto* blockOwn = reinterpret_cast<uint32_t*>(ws + w.blockOwn);
  auto* cnt = reinterpret_cast<uint32_t*>(ws + w.cnt);
  auto* totals = reinterpret_cast<uint32_t*>(ws + w.totals);
  const uint32_t mask = w.slots - 1;
  const int64_t rowLen = static_cast<int64_t>(g.kVol) * (cap + kSegment);
  const int64_t nIndex = 3 * rowLen;
  const int64_t nTable16 = static_cast<int64_t>(w.slots) / 2;

  // streaming fill: enough workgroups to cover the CUs several times over
  const int64_t fillItems = nTable16 + nIndex / 4 + 1;
  int fillBlocks = static_cast<int>((fillItems + kRbThreads - 1) / kRbThreads);
  if (fillBlocks > 256 * 16) fillBlocks = 256 * 16;
  if (fillBlocks < 1) fillBlocks = 1;
  hipLaunchKernelGGL(rbReset, dim3(fillBlocks), dim3(kRbThreads), 0, stream, reinterpret_cast<uint4*>(table), nTable16,
                     index, nIndex, totals, g.kVol, numIndex);

  const dim3 grid(w.nBlocks > 0 ? w.nBlocks : 1);
  const dim3 block(kRbThreads);
  const size_t ldsCnt = static_cast<size_t>(g.kVol) * sizeof(uint32_t);
  if (subM) {
    hipLaunchKernelGGL(rbSubmInsert, grid, block, 0, stream, g, coors, numActIn, cap, table, mask);
    hipLaunchKernelGGL(rbSubmProbe, grid, block, ldsCnt, stream, g, coors, numActIn, cap, table, mask, staging, cnt,
                       w.nBlocks, totals);
  } else {
    hipLaunchKernelGGL(rbConvInsert, grid, block, 0, stream, g, coors, numActIn, cap, table, mask, staging);
    hipLaunchKernelGGL(rbConvOwner, grid, block, 0, stream, g, numActIn, cap, table, staging, ownPrefix, blockOwn);
    hipLaunchKernelGGL(rbConvAssign, grid, block, 0, stream, g, numActIn, cap, table, staging, ownPrefix, blockOwn,
                       w.nBlocks, ids, outCoors, numActOut, maxNumActOut);
    hipLaunchKernelGGL(rbConvResolve, grid, block, ldsCnt, stream, g, numActIn, cap, ids, staging, maxNumActOut, cnt,
                       w.nBlocks, totals);
  }
  hipLaunchKernelGGL(rbCompact, dim3(grid.x, g.kVol), block, 0, stream, numActIn, cap, g.kVol, staging, cnt, w.nBlocks,
                     totals, index, index + rowLen, index + 2 * rowLen, numIndex);
  D3D_HIP_CHECK(hipGetLastError());
  return D3D_OK;
}

}  // namespace d3d
