// Host side of the engine: the two plugin objects behind the C ABI of
// include/d3d_spconv.h, attribute-blob parsing, weight preparation, and the
// per-index-tensor cache of neighbour tables that implements indice-key reuse.
//
// Reference life cycle being mirrored: SPConvIdxPlugin (trt/spconv/index_trt.cu:52-249)
// and SPConvMMPlugin (trt/spconv/mm_trt.cu:39-206).
#include <dlfcn.h>

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace d3d {

// ---------------------------------------------------------------------------
// error text (thread local)
// ---------------------------------------------------------------------------
namespace {
thread_local char g_error[512] = "";
thread_local bool g_noAlloc = false;  // set for the duration of d3d_enqueue_static: no device allocation allowed
}

void setError(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
const char* lastError() { return g_error; }

namespace {

// ---------------------------------------------------------------------------
// device memory
// ---------------------------------------------------------------------------
struct DeviceBuffer {
  void* ptr = nullptr;
  size_t bytes = 0;
  DeviceBuffer() = default;
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  ~DeviceBuffer() {
    if (ptr) (void)hipFree(ptr);
  }
  int32_t reserve(size_t n) {
    if (n <= bytes) return D3D_OK;
    if (ptr) {
      D3D_HIP_CHECK(hipFree(ptr));
      ptr = nullptr;
      bytes = 0;
    }
    D3D_HIP_CHECK(hipMalloc(&ptr, n));
    bytes = n;
    return D3D_OK;
  }
  // a fresh, zeroed allocation of n bytes, whatever was held before
  int32_t reallocZeroed(size_t n) {
    if (ptr) {
      D3D_HIP_CHECK(hipFree(ptr));
      ptr = nullptr;
      bytes = 0;
    }
    D3D_HIP_CHECK(hipMalloc(&ptr, n));
    bytes = n;
    D3D_HIP_CHECK(hipMemset(ptr, 0, n));
    return D3D_OK;
  }
  int32_t upload(const void* src, size_t n) {
    int32_t rc = reserve(n);
    if (rc != D3D_OK) return rc;
    D3D_HIP_CHECK(hipMemcpy(ptr, src, n, hipMemcpyHostToDevice));
    return D3D_OK;
  }
};

// ---------------------------------------------------------------------------
// IEEE conversions on the host (round-to-nearest-even), written out so the
// library does not depend on the host compiler's _Float16 runtime support.
// ---------------------------------------------------------------------------
uint16_t floatToHalfBits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7FFFFFFFu;
  if (x >= 0x7F800000u) return static_cast<uint16_t>(sign | 0x7C00u | (x > 0x7F800000u ? 0x200u : 0));  // inf / nan
  if (x >= 0x477FF000u) return static_cast<uint16_t>(sign | 0x7C00u);  // rounds to >= 65520 -> inf
  if (x < 0x33000001u) return static_cast<uint16_t>(sign);             // below half of the smallest subnormal
  int exp = static_cast<int>(x >> 23) - 127;
  uint32_t man = (x & 0x7FFFFFu) | 0x800000u;
  int shift;
  uint32_t base;
  if (exp < -14) {  // subnormal half
    shift = 13 + (-14 - exp);
    base = 0;
  } else {
    shift = 13;
    base = static_cast<uint32_t>(exp + 15) << 10;
    man &= 0x7FFFFFu;
  }
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) ++q;
  return static_cast<uint16_t>(sign | (base + q));  // a mantissa carry correctly bumps the exponent
}

float halfBitsToFloat(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1F, man = h & 0x3FFu;
  uint32_t x;
  if (exp == 0) {
    if (man == 0) {
      x = sign;
    } else {
      float v = std::ldexp(static_cast<float>(man), -24);
      std::memcpy(&x, &v, 4);
      x |= sign;
    }
  } else if (exp == 31) {
    x = sign | 0x7F800000u | (man << 13);
  } else {
    x = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &x, 4);
  return f;
}

uint16_t floatToBf16Bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((x >> 16) | 0x40u);  // quiet nan
  x += 0x7FFFu + ((x >> 16) & 1u);
  return static_cast<uint16_t>(x >> 16);
}

float bf16BitsToFloat(uint16_t b) {
  const uint32_t x = static_cast<uint32_t>(b) << 16;
  float f;
  std::memcpy(&f, &x, 4);
  return f;
}

int dtypeBytes(int32_t dtype) {
  switch (dtype) {
    case D3D_FLOAT:
    case D3D_INT32: return 4;
    case D3D_HALF:
    case D3D_BF16: return 2;
    case D3D_INT8:
    case D3D_BOOL: return 1;
  }
  return 0;
}

// ---------------------------------------------------------------------------
// Rulebook by-products.  A rulebook operator that convolutions have been linked to (d3d_link_rulebook) writes,
// besides the index tensor, the pairs in output-major form (the neighbour table the convolution kernels read) and
// the tap masks of 64-row tiles, into device memory this record owns.  The record belongs to the operator handle
// and to the convolutions linked to it (shared ownership: it is freed when the last of them is destroyed), and a
// convolution uses it only for the index tensor the operator wrote last, at the shapes it wrote it for; any other
// index tensor has its table derived from its contents on every enqueue, as the reference re-reads the index on
// every enqueue (trt/spconv/mm_trt.cu:166-170).
// ---------------------------------------------------------------------------
struct RulebookLink {
  std::mutex mutex;
  bool wanted = false;            // some convolution is linked: the operator writes the table
  bool wantMasks = false;         // ... and one of them runs a kernel that reads tile masks
  DeviceBuffer table, masks, fillState;
  // what the table describes (set by the operator's enqueue)
  const void* index = nullptr;    // index tensor the by-products belong to
  const void* numIndex = nullptr;
  int kVol = 0;
  int64_t outRows = 0, rowLen = 0;
  bool tableValid = false, masksValid = false;
  bool indexWritten = true;       // false: the last enqueue left the index tensor unwritten (D3D_OPT_INDEX_UNUSED)
  // incremental fill: index tensor that holds a complete earlier pass of this operator
  const void* primedIndex = nullptr;
  int64_t primedRowLen = 0;
  // block map of the output grid, kept for the SubM operators that run on this (strided) operator's outputs
  bool shareMap = false;          // some SubM operator is linked to these coordinates
  DeviceBuffer mapRecords, mapChunkBase;
  // an operator that keeps its map between passes holds two of them (mapStride records apart) and the state
  // words of RbSide::mapState: its builds then need no reset pass
  DeviceBuffer mapState;
  int64_t mapStride = 0;
  bool mapDouble = false;         // the last build alternated between the two maps
  bool mapDirty = false;          // a build with a reset pass has used the first map since the allocation: the
                                  // two no longer alternate cleanly, builds keep their reset pass from then on
  bool mapValid = false;
  const void* mapCoors = nullptr;     // outCoors / numActOut the map belongs to
  const void* mapNumAct = nullptr;
  int32_t mapGrid[kMaxSpatial + 1] = {0, 0, 0, 0, 0};
  int mapNd = 0;
  int64_t mapRows = 0;
};

size_t maskEntries(int64_t outRows) { return static_cast<size_t>((outRows + 63) / 64 + 8); }

// Profiler ranges around an operator's enqueue (reference analogue: the per-layer profiler of
// deploy3d/symfun/trt_utils/trt_module.py:20-44).  Off unless D3D_ROCTX is set in a process that enabled the
// debug switches; the tracing library is looked up at run time, so the engine does not link against it.
struct RoctxRange {
  typedef int (*PushFn)(const char*);
  typedef int (*PopFn)();
  static void lookup(PushFn* push, PopFn* pop) {
    static PushFn pushFn = nullptr;
    static PopFn popFn = nullptr;
    static const bool tried = [] {
      if (!debugEnv("D3D_ROCTX")) return true;
      void* lib = dlopen("libroctx64.so", RTLD_NOW | RTLD_GLOBAL);
      if (!lib) lib = dlopen("librocprofiler-sdk-roctx.so", RTLD_NOW | RTLD_GLOBAL);
      if (lib) {
        pushFn = reinterpret_cast<PushFn>(dlsym(lib, "roctxRangePushA"));
        popFn = reinterpret_cast<PopFn>(dlsym(lib, "roctxRangePop"));
      }
      return true;
    }();
    (void)tried;
    *push = pushFn;
    *pop = popFn;
  }
  PopFn pop = nullptr;
  explicit RoctxRange(const char* name) {
    PushFn push = nullptr;
    lookup(&push, &pop);
    if (push && pop) push(name); else pop = nullptr;
  }
  ~RoctxRange() {
    if (pop) pop();
  }
};

bool streamIsCapturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
}

// ---------------------------------------------------------------------------
// packed little-endian blob reader
// (reference: SerializeStream, trt/include/common/refnd.h:258-294)
// ---------------------------------------------------------------------------
struct BlobReader {
  const uint8_t* p;
  size_t len, pos = 0;
  BlobReader(const void* data, size_t n) : p(static_cast<const uint8_t*>(data)), len(n) {}
  bool i32(int32_t* v) {
    if (pos + 4 > len) return false;
    std::memcpy(v, p + pos, 4);
    pos += 4;
    return true;
  }
  bool u8(uint8_t* v) {
    if (pos + 1 > len) return false;
    *v = p[pos++];
    return true;
  }
};

}  // namespace
}  // namespace d3d

// ---------------------------------------------------------------------------
// plugin objects
// ---------------------------------------------------------------------------
struct d3d_plugin {
  std::string type;
  std::vector<uint8_t> blob;  // kept verbatim: serialize() is a byte-exact round trip
  virtual ~d3d_plugin() = default;
  virtual d3d_plugin* clone() const = 0;
  virtual int32_t numOutputs() const = 0;
  virtual int32_t outputDims(int32_t idx, const d3d_tensor_desc* in, int32_t nbIn, d3d_tensor_desc* out) const = 0;
  virtual int32_t outputDtype(int32_t idx, const int32_t* inTypes, int32_t nbIn) const = 0;
  virtual int32_t supportsFormat(int32_t pos, const d3d_tensor_desc* io, int32_t nbIn, int32_t nbOut) const = 0;
  virtual int32_t configure(const d3d_tensor_desc* in, int32_t nbIn, const d3d_tensor_desc* out, int32_t nbOut) = 0;
  virtual size_t workspaceSize(const d3d_tensor_desc* in, int32_t nbIn) const = 0;
  virtual int32_t enqueue(const d3d_tensor_desc* inDesc, const d3d_tensor_desc* outDesc, const void* const* inputs,
                          void* const* outputs, void* workspace, size_t workspaceBytes, hipStream_t stream) = 0;
  virtual int32_t setOption(int32_t option, int64_t) {
    d3d::setError("%s: option %d not known to this operator", type.c_str(), option);
    return D3D_ERR_UNSUPPORTED;
  }
};

namespace d3d {
namespace {

// --- SPConvIdx{N}d -----------------------------------------------------------
// Attribute layout: SPConvIdxPluginParam<NDim>, trt/spconv/index_trt.cu:39-50.
struct IdxPlugin final : d3d_plugin {
  int nd = 3;
  int32_t kernel[kMaxSpatial], stride[kMaxSpatial], padding[kMaxSpatial], dilation[kMaxSpatial],
      outPadding[kMaxSpatial];
  int32_t maxNumActOut = 0;
  bool subM = false, transpose = false;
  bool persistentIndex = false;                  // D3D_OPT_PERSISTENT_INDEX
  bool indexUnused = false;                      // D3D_OPT_INDEX_UNUSED
  std::shared_ptr<RulebookLink> link = std::make_shared<RulebookLink>();  // by-products for linked convolutions
  std::shared_ptr<RulebookLink> coordSource;     // record of the strided operator that writes inCoors (d3d_link_coords)

  int kVol() const {
    int v = 1;
    for (int i = 0; i < nd; ++i) v *= kernel[i];
    return v;
  }

  static int32_t parse(int nd, const void* data, size_t len, IdxPlugin** out) {
    const size_t need = static_cast<size_t>(nd) * 5 * 4 + 4 + 2;
    if (!data || len < need) {
      setError("SPConvIdx%dd: attribute blob of %zu bytes, %zu expected", nd, len, need);
      return D3D_ERR_BAD_BLOB;
    }
    auto p = std::unique_ptr<IdxPlugin>(new IdxPlugin());
    p->nd = nd;
    p->type = "SPConvIdx" + std::to_string(nd) + "d";
    BlobReader r(data, len);
    int32_t* fields[5] = {p->kernel, p->stride, p->padding, p->dilation, p->outPadding};
    for (auto* f : fields)
      for (int i = 0; i < nd; ++i) r.i32(&f[i]);
    r.i32(&p->maxNumActOut);
    uint8_t b0 = 0, b1 = 0;
    r.u8(&b0);
    r.u8(&b1);
    p->subM = b0 != 0;
    p->transpose = b1 != 0;
    for (int i = 0; i < nd; ++i) {
      if (p->kernel[i] < 1 || p->stride[i] < 1 || p->dilation[i] < 1 || p->padding[i] < 0) {
        setError("%s: kernel/stride/dilation must be positive and padding non-negative", p->type.c_str());
        return D3D_ERR_BAD_BLOB;
      }
    }
    if (p->maxNumActOut < 0) {
      setError("%s: negative maxNumActOut", p->type.c_str());
      return D3D_ERR_BAD_BLOB;
    }
    p->blob.assign(static_cast<const uint8_t*>(data), static_cast<const uint8_t*>(data) + need);
    *out = p.release();
    return D3D_OK;
  }

  d3d_plugin* clone() const override {
    auto* c = new IdxPlugin(*this);
    c->link = std::make_shared<RulebookLink>();  // a clone is another node: its own by-products, no links yet
    c->coordSource.reset();
    c->persistentIndex = false;
    c->indexUnused = false;
    return c;
  }
  int32_t numOutputs() const override { return subM ? 2 : 5; }  // index_trt.cu:98-101

  // Called when a convolution is linked: from now on enqueue also writes the neighbour table and the tile masks.
  int32_t wantByProducts(bool masks) {
    std::lock_guard<std::mutex> lock(link->mutex);
    link->wantMasks = link->wantMasks || (masks && kVol() <= 64);
    if (maxNumActOut > 0) {
      int32_t rc = link->table.reserve(static_cast<size_t>(kVol()) * static_cast<size_t>(maxNumActOut) * sizeof(int32_t));
      if (rc != D3D_OK) return rc;
      rc = link->masks.reserve(maskEntries(maxNumActOut) * sizeof(unsigned long long));
      if (rc != D3D_OK) return rc;
    }
    link->wanted = true;
    return D3D_OK;
  }

  int32_t setOption(int32_t option, int64_t value) override {
    if (option == D3D_OPT_INDEX_UNUSED) {
      std::lock_guard<std::mutex> lock(link->mutex);
      indexUnused = value != 0;
      link->primedIndex = nullptr;
      return D3D_OK;
    }
    if (option != D3D_OPT_PERSISTENT_INDEX) return d3d_plugin::setOption(option, value);
    std::lock_guard<std::mutex> lock(link->mutex);
    if (value && !link->fillState.ptr) {
      int32_t rc = link->fillState.reallocZeroed(256);
      if (rc != D3D_OK) return rc;
    }
    persistentIndex = value != 0;
    link->primedIndex = nullptr;
    return D3D_OK;
  }

  // spatial extents of the output grid from those of the input grid
  void outSpatial(const int32_t* in, int32_t* out) const {
    for (int i = 0; i < nd; ++i) {
      if (transpose) {  // geometry.h:138-156
        out[i] = (in[i] - 1) * stride[i] - 2 * padding[i] + (kernel[i] - 1) * dilation[i] + outPadding[i] + 1;
      } else {  // geometry.h:118-136
        out[i] = (in[i] + 2 * padding[i] - dilation[i] * (kernel[i] - 1) - 1) / stride[i] + 1;
      }
    }
  }

  int32_t outputDims(int32_t idx, const d3d_tensor_desc* in, int32_t nbIn, d3d_tensor_desc* out) const override {
    if (!in || nbIn < 3 || !out || idx < 0 || idx >= numOutputs()) {
      setError("%s: output %d of %d, %d inputs", type.c_str(), idx, numOutputs(), nbIn);
      return D3D_ERR_BAD_ARG;
    }
    std::memset(out, 0, sizeof(*out));
    out->dtype = D3D_INT32;
    out->format = D3D_LINEAR;
    switch (idx) {
      case 0:  // index_trt.cu:107-119
        out->nb_dims = 2;
        out->dims[0] = 3;
        out->dims[1] = kVol() * (in[0].dims[0] + kSegment);
        break;
      case 1:
      case 3:
        out->nb_dims = 1;
        out->dims[0] = 1;
        break;
      case 2:  // index_trt.cu:123-126
        out->nb_dims = 2;
        out->dims[0] = maxNumActOut;
        out->dims[1] = nd + 1;
        break;
      default: {  // index_trt.cu:131-150: [B, 0, spatial...]
        if (in[2].nb_dims != nd + 2) {
          setError("%s: spatial-shape tensor must have %d dims", type.c_str(), nd + 2);
          return D3D_ERR_BAD_ARG;
        }
        *out = in[2];
        out->dtype = D3D_INT32;
        outSpatial(in[2].dims + 2, out->dims + 2);
      }
    }
    return D3D_OK;
  }
  int32_t outputDtype(int32_t, const int32_t*, int32_t) const override { return D3D_INT32; }  // index_trt.cu:153-155
  int32_t supportsFormat(int32_t pos, const d3d_tensor_desc* io, int32_t nbIn, int32_t nbOut) const override {
    if (!io || pos < 0 || pos >= nbIn + nbOut) return 0;
    return io[pos].format == D3D_LINEAR && io[pos].dtype == D3D_INT32;  // index_trt.cu:156-161
  }
  // The operator-owned pair of block maps (and their state words) for this grid and capacity: kept between passes
  // for the SubM operators linked to this one's outputs, and - two maps in turn - so that a build needs no reset
  // pass.  The two alternate cleanly only among builds on one grid size: another size takes a new, zeroed
  // allocation.  `mayAllocate` false (a stream under capture): only says whether they are there.  Caller holds
  // link->mutex.
  bool mapsReady(const RbGeom& g, int64_t cap, bool mayAllocate) {
    size_t recBytes = 0, chunkBytes = 0;
    blockMapBytes(g, cap, &recBytes, &chunkBytes);
    if (!recBytes) return false;
    const size_t stateBytes = mapStateWords(chunkBytes) * 4;
    auto have = [&]() {
      return link->mapRecords.bytes >= 2 * recBytes && link->mapChunkBase.bytes >= chunkBytes &&
             link->mapState.bytes >= stateBytes && link->mapStride * 16 == static_cast<int64_t>(recBytes);
    };
    if (!have() && mayAllocate) {
      link->mapStride = 0;
      if (link->mapRecords.reallocZeroed(2 * recBytes) == D3D_OK && link->mapChunkBase.reserve(chunkBytes) == D3D_OK &&
          link->mapState.reallocZeroed(stateBytes) == D3D_OK) {
        link->mapStride = static_cast<int64_t>(recBytes / 16);
        link->mapDirty = false;
      }
    }
    return have();
  }
  bool keepsItsMap() const { return (!subM && link->shareMap) || persistentIndex; }

  // configurePlugin (index_trt.cu:153-159 does nothing): capacities and grid are known here, so the maps an
  // operator keeps are reserved now and an enqueue - under capture or not - finds them.
  int32_t configure(const d3d_tensor_desc* in, int32_t nbIn, const d3d_tensor_desc*, int32_t) override {
    if (!in || nbIn < 3 || in[0].nb_dims != 2 || in[0].dims[1] != nd + 1 || in[2].nb_dims != nd + 2) return D3D_OK;
    int32_t grid[kMaxSpatial + 1], inGrid[kMaxSpatial + 1];
    outputGrid(in[2], grid);
    inGrid[0] = in[2].dims[0];
    for (int i = 0; i < nd; ++i) inGrid[1 + i] = in[2].dims[2 + i];
    std::lock_guard<std::mutex> lock(link->mutex);
    if (keepsItsMap()) (void)mapsReady(geometry(grid, inGrid), in[0].dims[0], true);
    return D3D_OK;
  }

  RbGeom geometry(const int32_t* outGrid /* [B, spatial...] */, const int32_t* inGrid = nullptr) const {
    RbGeom g{};
    if (!inGrid) inGrid = outGrid;
    g.nd = nd;
    const int pad = kMaxSpatial - nd;
    for (int i = 0; i < kMaxSpatial; ++i) {
      const bool real = i >= pad;
      g.k[i] = real ? kernel[i - pad] : 1;
      g.s[i] = real ? stride[i - pad] : 1;
      g.p[i] = real ? padding[i - pad] : 0;
      g.d[i] = real ? dilation[i - pad] : 1;
      g.shape[i + 1] = real ? outGrid[1 + i - pad] : 1;
      g.inShape[i + 1] = real ? inGrid[1 + i - pad] : 1;
    }
    g.shape[0] = outGrid[0];
    g.inShape[0] = inGrid[0];
    g.kVol = kVol();
    g.transpose = transpose ? 1 : 0;
    return g;
  }

  // output grid [B, spatial...] from the descriptor of the spatial-shape input
  void outputGrid(const d3d_tensor_desc& shape, int32_t* grid) const {
    grid[0] = shape.dims[0];
    if (subM) {  // index_trt.cu:218-219: SubM works on the input grid
      for (int i = 0; i < nd; ++i) grid[1 + i] = shape.dims[2 + i];
    } else {
      outSpatial(shape.dims + 2, grid + 1);
    }
  }

  // getWorkspaceSize (index_trt.cu:178-187): from the row capacity, and from the grid when the caller passes it
  size_t workspaceSize(const d3d_tensor_desc* in, int32_t nbIn) const override {
    if (!in || nbIn < 1) return 0;
    const bool gridKnown = nbIn >= 3 && in[2].nb_dims == nd + 2;
    int32_t grid[kMaxSpatial + 1] = {1 << 6, 1 << 6, 1 << 6, 1 << 6, 1 << 6};  // only caps the strided hash
    if (gridKnown) outputGrid(in[2], grid);
    return rulebookWorkspaceBytes(geometry(grid), in[0].dims[0], subM, gridKnown);
  }

  int32_t enqueue(const d3d_tensor_desc* inDesc, const d3d_tensor_desc* outDesc, const void* const* inputs,
                  void* const* outputs, void* workspace, size_t workspaceBytes, hipStream_t stream) override {
    if (!inDesc || !outDesc || !inputs || !outputs) {
      setError("%s: null descriptor or tensor array", type.c_str());
      return D3D_ERR_BAD_ARG;
    }
    if (inDesc[0].nb_dims != 2 || inDesc[0].dims[1] != nd + 1 || inDesc[2].nb_dims != nd + 2) {
      setError("%s: inCoors must be [cap, %d] and the spatial shape [B, 0, %d extents]", type.c_str(), nd + 1, nd);
      return D3D_ERR_BAD_ARG;
    }
    const int64_t cap = inDesc[0].dims[0];
    const int64_t rowLen = static_cast<int64_t>(kVol()) * (cap + kSegment);
    if (outDesc[0].nb_dims != 2 || outDesc[0].dims[0] != 3 || outDesc[0].dims[1] != rowLen) {
      setError("%s: index tensor must be [3, %lld]", type.c_str(), static_cast<long long>(rowLen));
      return D3D_ERR_BAD_ARG;
    }
    // output grid: the input's for SubM (index_trt.cu:218-219), else derived from it
    int32_t grid[kMaxSpatial + 1];
    outputGrid(inDesc[2], grid);
    if (!subM) {
      if (outDesc[2].nb_dims != 2 || outDesc[2].dims[0] != maxNumActOut || outDesc[2].dims[1] != nd + 1) {
        setError("%s: outCoors must be [%d, %d]", type.c_str(), maxNumActOut, nd + 1);
        return D3D_ERR_BAD_ARG;
      }
    }
    int32_t inGrid[kMaxSpatial + 1];
    inGrid[0] = inDesc[2].dims[0];
    for (int i = 0; i < nd; ++i) inGrid[1 + i] = inDesc[2].dims[2 + i];
    const RbGeom g = geometry(grid, inGrid);
    const RoctxRange range(subM ? "d3d rulebook (submanifold)" : "d3d rulebook (strided)");
    std::lock_guard<std::mutex> lock(link->mutex);
    RbSide side{};
    const size_t tableBytes = static_cast<size_t>(kVol()) * static_cast<size_t>(maxNumActOut) * sizeof(int32_t);
    const bool withTable = link->wanted && maxNumActOut > 0 && link->table.bytes >= tableBytes &&
                           link->masks.bytes >= maskEntries(maxNumActOut) * sizeof(unsigned long long);
    if (withTable) {
      side.nbr = static_cast<int32_t*>(link->table.ptr);
      side.nbrRows = maxNumActOut;
      if (link->wantMasks) {
        side.masks = static_cast<unsigned long long*>(link->masks.ptr);
        side.nMasks = static_cast<int64_t>(maskEntries(maxNumActOut));
      }
    }
    side.skipIndex = indexUnused && withTable;
    if (persistentIndex && link->fillState.ptr) {
      side.fillState = static_cast<uint32_t*>(link->fillState.ptr);
      side.incrementalFill = link->primedIndex == outputs[0] && link->primedRowLen == rowLen;
    }
    // one block map per stage (d3d_link_coords): a strided operator keeps its map for the SubM operators on its
    // outputs, a SubM operator takes the map of the operator that wrote the coordinates it is handed
    std::shared_ptr<RulebookLink> source = coordSource;
    std::unique_lock<std::mutex> sourceLock;
    if (keepsItsMap() && !g_noAlloc) {
      // allocated (and zeroed) on first use unless configure did it, or when the grid grows; never while the stream
      // is being captured
      hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
      (void)hipStreamIsCapturing(stream, &capturing);
      if (mapsReady(g, cap, capturing == hipStreamCaptureStatusNone)) {
        side.mapRecords = link->mapRecords.ptr;
        side.mapChunkBase = static_cast<uint32_t*>(link->mapChunkBase.ptr);
        side.mapState = static_cast<uint32_t*>(link->mapState.ptr);
        side.mapStride = link->mapStride;
        side.mapDirty = link->mapDirty;
      }
    }
    link->mapValid = false;
    if (source && source != link) {
      sourceLock = std::unique_lock<std::mutex>(source->mutex);
      bool same = source->mapValid && source->mapCoors == inputs[0] && source->mapNumAct == inputs[1] &&
                  source->mapNd == nd && source->mapRows == cap;
      for (int i = 0; same && i <= nd; ++i) same = source->mapGrid[i] == inGrid[i];  // (SubM: the output grid too)
      if (same && subM) {
        side.mapRecords = source->mapRecords.ptr;
        side.mapChunkBase = static_cast<uint32_t*>(source->mapChunkBase.ptr);
        side.mapState = static_cast<uint32_t*>(source->mapState.ptr);
        side.mapStride = source->mapStride;
        side.mapDouble = source->mapDouble;
        side.useSharedMap = true;
      } else if (same) {
        // a strided operator on another's outputs: that operator's map is the map of THIS one's input cells
        side.srcRecords = source->mapRecords.ptr;
        side.srcChunkBase = static_cast<const uint32_t*>(source->mapChunkBase.ptr);
        side.srcState = static_cast<uint32_t*>(source->mapState.ptr);
        side.srcStride = source->mapStride;
        side.srcDouble = source->mapDouble;
      }
    }
    link->tableValid = link->masksValid = false;
    // An enqueue on a stream that is being captured runs later, if ever: it must not make the tensor count as
    // holding a complete pass unless an executed enqueue had already made it so.
    hipStreamCaptureStatus captureNow = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(stream, &captureNow);
    const bool wasPrimed = side.incrementalFill;
    link->primedIndex = nullptr;
    int32_t rc = launchRulebook(g, subM, static_cast<const int32_t*>(inputs[0]),
                                static_cast<const int32_t*>(inputs[1]), cap, maxNumActOut,
                                static_cast<int32_t*>(outputs[0]), static_cast<int32_t*>(outputs[1]),
                                subM ? nullptr : static_cast<int32_t*>(outputs[2]),
                                subM ? nullptr : static_cast<int32_t*>(outputs[3]), workspace, workspaceBytes, side,
                                stream);
    if (rc == D3D_OK) {
      link->index = outputs[0];
      link->numIndex = outputs[1];
      link->kVol = kVol();
      link->outRows = maxNumActOut;
      link->rowLen = rowLen;
      link->tableValid = withTable;
      link->indexWritten = side.indexWritten;
      link->masksValid = withTable && side.masksWritten;
      if (side.fillState && side.indexWritten && (captureNow == hipStreamCaptureStatusNone || wasPrimed)) {
        link->primedIndex = outputs[0];
        link->primedRowLen = rowLen;
      }
      if (!side.useSharedMap) {
        link->mapDouble = side.mapDouble;
        if (side.mapRecords && !side.mapDouble) link->mapDirty = true;
      }
      if (side.mapWritten) {
        link->mapValid = true;
        link->mapCoors = outputs[2];
        link->mapNumAct = outputs[3];
        link->mapNd = nd;
        link->mapRows = maxNumActOut;
        for (int i = 0; i <= nd; ++i) link->mapGrid[i] = grid[i];
      }
    }
    return rc;
  }
};

// One zero-filled device row shared by every convolution: the source of gathers for absent neighbours.
const void* zeroRow() {
  static std::mutex m;
  static DeviceBuffer* buf = nullptr;  // lives until the process ends
  std::lock_guard<std::mutex> lock(m);
  if (!buf) {
    auto* b = new DeviceBuffer();
    if (b->reserve(1024) != D3D_OK || hipMemset(b->ptr, 0, 1024) != hipSuccess) {
      delete b;
      return nullptr;
    }
    buf = b;
  }
  return buf->ptr;
}

// Tuning / test hook: D3D_CONV_TILE_ROWS = rows per workgroup of the weight-streaming MFMA convolution
// (64 .. 512, a multiple of 64), D3D_CONV_WAVES = 4 or 8 wavefronts per workgroup; unset = heuristic.
int tileRowsOverride() {
  const char* e = debugEnv("D3D_CONV_TILE_ROWS");
  if (!e) return 0;
  const int v = std::atoi(e);
  if (v < 64 || v > 512 || v % 64) return 0;
  const char* w = debugEnv("D3D_CONV_WAVES");
  return v | ((w && std::atoi(w) == 4) ? (1 << 30) : 0);
}

// Tuning / test hook: D3D_CONV_STAGED = "off" keeps the register-gather kernels; "MT,WAVES,NS[,1]" picks a
// configuration of the staged kernel (trailing 1 = weights resident in LDS); unset = heuristic.
int stagedOverride() {
  const char* e = debugEnv("D3D_CONV_STAGED");
  if (!e || !*e) return 0;
  if (std::strcmp(e, "off") == 0) return -1;
  int mt = 0, waves = 0, ns = 0, res = 0;
  if (std::sscanf(e, "%d,%d,%d,%d", &mt, &waves, &ns, &res) < 3) return 0;
  return mt | waves << 8 | ns << 16 | (res ? 1 << 24 : 0);
}

// --- SPConvMM ----------------------------------------------------------------
// Attribute layout: SPConvMMPluginParam + fp32 payload, trt/spconv/mm_trt.cu:27-37, :61-68.
constexpr uint32_t kExtMagic = 0x58443344u;  // "D3DX"
constexpr size_t kMMHeader = 19;

struct MMDeviceWeights {
  int32_t dtype = -1;
  int cinMfma = 0;  // input channels of the packed MFMA weights (cin widened with zero rows), 0 = no MFMA copy
  DeviceBuffer f32, mfma, bias, requantM;  // int8: bias holds bias / s_out, requantM holds s_in * s_w[c] / s_out
};

struct MMPlugin final : d3d_plugin {
  int32_t kernelVol = 0, cin = 0, cout = 0, maxNumActOut = 0;
  bool inverse = false, withBias = false, relu = false;
  float actScaleIn = 1.f, actScaleOut = 1.f;
  size_t weightOffset = kMMHeader;             // byte offset of W in blob
  std::shared_ptr<MMDeviceWeights> dev;        // shared by clones (mm_trt.cu:43-45, :75-79)
  std::shared_ptr<std::mutex> devMutex;
  std::shared_ptr<RulebookLink> linked;        // by-products of the rulebook operator this node is linked to
  std::shared_ptr<DeviceBuffer> derived;       // neighbour table derived from the index tensor (no link, foreign
                                               // tensor, inverse)
  std::shared_ptr<DeviceBuffer> widened;       // input rows widened to the MFMA channel count (narrow layers)

  static int32_t parse(const void* data, size_t len, MMPlugin** out) {
    if (!data || len < kMMHeader) {
      setError("SPConvMM: attribute blob of %zu bytes, at least %zu expected", len, kMMHeader);
      return D3D_ERR_BAD_BLOB;
    }
    auto p = std::unique_ptr<MMPlugin>(new MMPlugin());
    p->type = "SPConvMM";
    BlobReader r(data, len);
    r.i32(&p->kernelVol);
    r.i32(&p->cin);
    r.i32(&p->cout);
    r.i32(&p->maxNumActOut);
    uint8_t subM = 0, inv = 0, wb = 0;
    r.u8(&subM);  // deprecated, ignored (mm_trt.cu:33)
    r.u8(&inv);
    r.u8(&wb);
    p->inverse = inv != 0;
    p->withBias = wb != 0;
    if (p->kernelVol < 1 || p->cin < 1 || p->cout < 1 || p->maxNumActOut < 0) {
      setError("SPConvMM: kernelVol/inChannels/outChannels must be positive");
      return D3D_ERR_BAD_BLOB;
    }
    const size_t floats = static_cast<size_t>(p->kernelVol) * p->cin * p->cout + (p->withBias ? p->cout : 0);
    const size_t payloadEnd = kMMHeader + floats * 4;
    if (len < payloadEnd) {
      setError("SPConvMM: blob holds %zu payload bytes, %zu needed for W[%d,%d,%d]%s", len - kMMHeader, floats * 4,
               p->kernelVol, p->cin, p->cout, p->withBias ? " + bias" : "");
      return D3D_ERR_BAD_BLOB;
    }
    if (len >= payloadEnd + 20) {  // optional extension record
      const uint8_t* e = static_cast<const uint8_t*>(data) + payloadEnd;
      uint32_t magic, version, flags;
      std::memcpy(&magic, e, 4);
      std::memcpy(&version, e + 4, 4);
      std::memcpy(&flags, e + 8, 4);
      if (magic == kExtMagic) {
        if (version != 1) {
          setError("SPConvMM: extension record version %u not understood", version);
          return D3D_ERR_BAD_BLOB;
        }
        p->relu = (flags & 1u) != 0;
        std::memcpy(&p->actScaleIn, e + 12, 4);
        std::memcpy(&p->actScaleOut, e + 16, 4);
      }
    }
    p->blob.assign(static_cast<const uint8_t*>(data), static_cast<const uint8_t*>(data) + len);
    p->dev = std::make_shared<MMDeviceWeights>();
    p->devMutex = std::make_shared<std::mutex>();
    *out = p.release();
    return D3D_OK;
  }

  d3d_plugin* clone() const override {
    auto* c = new MMPlugin(*this);  // weights are shared (mm_trt.cu:75-79); per-enqueue buffers are not
    c->linked.reset();
    c->derived.reset();
    c->widened.reset();
    return c;
  }
  int32_t numOutputs() const override { return 1; }
  int32_t outputDims(int32_t idx, const d3d_tensor_desc*, int32_t, d3d_tensor_desc* out) const override {
    if (idx != 0 || !out) return D3D_ERR_BAD_ARG;
    std::memset(out, 0, sizeof(*out));  // mm_trt.cu:98-103
    out->format = D3D_LINEAR;
    out->nb_dims = 2;
    out->dims[0] = maxNumActOut;
    out->dims[1] = cout;
    return D3D_OK;
  }
  int32_t outputDtype(int32_t, const int32_t* inTypes, int32_t nbIn) const override {
    return (inTypes && nbIn > 0) ? inTypes[0] : D3D_ERR_BAD_ARG;  // mm_trt.cu:104-106
  }
  static bool featureType(int32_t t) { return t == D3D_HALF || t == D3D_FLOAT || t == D3D_BF16 || t == D3D_INT8; }
  int32_t supportsFormat(int32_t pos, const d3d_tensor_desc* io, int32_t nbIn, int32_t nbOut) const override {
    if (!io || pos < 0 || pos >= nbIn + nbOut || io[pos].format != D3D_LINEAR) return 0;
    if (pos == 0) return featureType(io[0].dtype);
    if (pos == 5) return io[5].dtype == io[0].dtype;  // mm_trt.cu:113
    return io[pos].dtype == D3D_INT32;
  }

  // configurePlugin (mm_trt.cu:127-142): weights and bias are rounded to the
  // feature type exactly as the reference's static_cast<half> does, then
  // uploaded; the fp32 copy holds the rounded values.
  int32_t configure(const d3d_tensor_desc* in, int32_t nbIn, const d3d_tensor_desc*, int32_t) override {
    if (!in || nbIn < 1) return D3D_ERR_BAD_ARG;
    const int32_t dtype = in[0].dtype;
    if (!featureType(dtype)) {
      setError("SPConvMM: feature dtype %d not implemented", dtype);
      return D3D_ERR_UNSUPPORTED;
    }
    {
      std::lock_guard<std::mutex> lock(*devMutex);
      if (dev->dtype != dtype) {
        const int32_t rc = dtype == D3D_INT8 ? configureInt8() : configureFloat(dtype);
        if (rc != D3D_OK) return rc;
      }
    }
    // Capacities are known here: reserve what enqueue would otherwise have to allocate on first use - the rows of a
    // narrow layer widened to the MFMA channel count, and the derived table of a node that has no link (or is an
    // inverse convolution, whose table is always derived).
    if (in[0].nb_dims == 2 && in[0].dims[0] > 0 && dev->cinMfma > cin &&
        !convReadsNarrowRows(dtype, kernelVol, cin, cout)) {
      if (!widened) widened = std::make_shared<DeviceBuffer>();
      const int32_t rc = widened->reserve(static_cast<size_t>(in[0].dims[0]) * dev->cinMfma * dtypeBytes(dtype));
      if (rc != D3D_OK) return rc;
    }
    if ((!linked || inverse) && maxNumActOut > 0) {
      if (!derived) derived = std::make_shared<DeviceBuffer>();
      const int32_t rc = derived->reserve(static_cast<size_t>(kernelVol) * static_cast<size_t>(maxNumActOut) * sizeof(int32_t));
      if (rc != D3D_OK) return rc;
    }
    return D3D_OK;
  }

  int32_t configureFloat(int32_t dtype) {
    const size_t nW = static_cast<size_t>(kernelVol) * cin * cout;
    std::vector<float> w(nW), b(withBias ? cout : 0);
    std::memcpy(w.data(), blob.data() + weightOffset, nW * 4);
    if (withBias) std::memcpy(b.data(), blob.data() + weightOffset + nW * 4, static_cast<size_t>(cout) * 4);
    std::vector<uint16_t> packed;
    int cinMfma = 0;
    if (dtype == D3D_HALF || dtype == D3D_BF16) {
      const bool half = dtype == D3D_HALF;
      auto rnd = [&](float v, uint16_t* bits) {
        *bits = half ? floatToHalfBits(v) : floatToBf16Bits(v);
        return half ? halfBitsToFloat(*bits) : bf16BitsToFloat(*bits);
      };
      const int cinP = paddedMfmaChannels(dtype, cin, cout);
      const bool mfma = convUsesMfma(dtype, cinP, cout);
      if (mfma) packed.assign(static_cast<size_t>(kernelVol) * cinP * cout, 0);
      cinMfma = mfma ? cinP : 0;
      // fragment-major copy for the MFMA kernel: Wf[tap][kk][n][lane][j] = W[tap][kk*KS + (lane/16)*KG + j][n*16 + lane%16]
      // with KS = 32 (16 when cin == 16) and KG = KS/4, so one wavefront load fetches one whole operand fragment;
      // rows past cin (a narrow layer widened to 16 channels) stay zero
      const int ks = cinP >= 32 ? 32 : 16, kg = ks / 4, nt = cout / 16, kkN = cinP / ks;
      for (int k = 0; k < kernelVol; ++k)
        for (int ci = 0; ci < cin; ++ci)
          for (int co = 0; co < cout; ++co) {
            const size_t src = (static_cast<size_t>(k) * cin + ci) * cout + co;
            uint16_t bits;
            w[src] = rnd(w[src], &bits);
            if (mfma) {
              const int kk = ci / ks, within = ci % ks, lane = (within / kg) * 16 + co % 16, j = within % kg;
              const size_t dst = (((static_cast<size_t>(k) * kkN + kk) * nt + co / 16) * 64 + lane) * kg + j;
              packed[dst] = bits;
            }
          }
      for (auto& v : b) {
        uint16_t bits;
        v = rnd(v, &bits);
      }
    }
    int32_t rc = dev->f32.upload(w.data(), nW * 4);
    if (rc != D3D_OK) return rc;
    if (!packed.empty()) {
      rc = dev->mfma.upload(packed.data(), packed.size() * 2);
      if (rc != D3D_OK) return rc;
    }
    if (withBias) {
      rc = dev->bias.upload(b.data(), b.size() * 4);
      if (rc != D3D_OK) return rc;
    }
    if (!zeroRow()) {
      setError("SPConvMM: could not allocate the zero row");
      return D3D_ERR_DEVICE;
    }
    dev->cinMfma = cinMfma;
    dev->dtype = dtype;
    return D3D_OK;
  }

  // int8 (no counterpart in the reference): symmetric per-output-channel weights, s_w[c] = max|W[:,:,c]| / 127,
  // q = clamp(rint(w / s_w)); the epilogue computes clamp(rint(float(acc) * m[c] + bq[c])) with
  // m[c] = float(s_in * s_w[c] / s_out) and bq[c] = float(bias[c] / s_out), all three quotients in double.
  int32_t configureInt8() {
    if (!(actScaleIn > 0.f) || !(actScaleOut > 0.f)) {
      setError("SPConvMM: int8 needs positive activation scales in the extension record");
      return D3D_ERR_UNSUPPORTED;
    }
    const int cinP = paddedMfmaChannels(D3D_INT8, cin, cout);
    if (!convUsesMfma(D3D_INT8, cinP, cout)) {
      setError("SPConvMM: int8 is implemented for up to 128 input channels and 16/32/64/128 output channels");
      return D3D_ERR_UNSUPPORTED;
    }
    const size_t nW = static_cast<size_t>(kernelVol) * cin * cout;
    std::vector<float> w(nW), b(cout, 0.f);
    std::memcpy(w.data(), blob.data() + weightOffset, nW * 4);
    if (withBias) std::memcpy(b.data(), blob.data() + weightOffset + nW * 4, static_cast<size_t>(cout) * 4);
    std::vector<double> sw(cout, 0.0);
    for (size_t i = 0; i < nW; ++i) {
      const double v = std::fabs(static_cast<double>(w[i]));
      if (v > sw[i % cout]) sw[i % cout] = v;
    }
    std::vector<float> m(cout), bq(cout);
    for (int c = 0; c < cout; ++c) {
      sw[c] = sw[c] / 127.0;
      if (sw[c] == 0.0) sw[c] = 1.0;
      m[c] = static_cast<float>(static_cast<double>(actScaleIn) * sw[c] / static_cast<double>(actScaleOut));
      bq[c] = static_cast<float>(static_cast<double>(b[c]) / static_cast<double>(actScaleOut));
    }
    // fragment-major: Wf[tap][kk][n][lane][j] = q[tap][kk*KS + (lane/16)*KG + j][n*16 + lane%16], KS = 64 (32), KG = KS/4
    const int ks = cinP >= 64 ? 64 : 32, kg = ks / 4, nt = cout / 16, kkN = cinP / ks;
    std::vector<int8_t> packed(static_cast<size_t>(kernelVol) * cinP * cout, 0);
    for (int k = 0; k < kernelVol; ++k)
      for (int ci = 0; ci < cin; ++ci)
        for (int co = 0; co < cout; ++co) {
          const size_t src = (static_cast<size_t>(k) * cin + ci) * cout + co;
          double q = std::nearbyint(static_cast<double>(w[src]) / sw[co]);
          q = q > 127.0 ? 127.0 : (q < -127.0 ? -127.0 : q);
          const int kk = ci / ks, within = ci % ks, lane = (within / kg) * 16 + co % 16, j = within % kg;
          const size_t dst = (((static_cast<size_t>(k) * kkN + kk) * nt + co / 16) * 64 + lane) * kg + j;
          packed[dst] = static_cast<int8_t>(q);
        }
    int32_t rc = dev->mfma.upload(packed.data(), packed.size());
    if (rc == D3D_OK) rc = dev->requantM.upload(m.data(), m.size() * 4);
    if (rc == D3D_OK) rc = dev->bias.upload(bq.data(), bq.size() * 4);
    if (rc != D3D_OK) return rc;
    if (!zeroRow()) {
      setError("SPConvMM: could not allocate the zero row");
      return D3D_ERR_DEVICE;
    }
    dev->cinMfma = cinP;
    dev->dtype = D3D_INT8;
    return D3D_OK;
  }

  size_t workspaceSize(const d3d_tensor_desc*, int32_t) const override { return 0; }  // mm_trt.cu:143-148

  int32_t enqueue(const d3d_tensor_desc* inDesc, const d3d_tensor_desc* outDesc, const void* const* inputs,
                  void* const* outputs, void*, size_t, hipStream_t stream) override {
    if (!inDesc || !outDesc || !inputs || !outputs || !inputs[0] || !inputs[3] || !inputs[4] || !outputs[0]) {
      setError("SPConvMM: null descriptor or tensor");
      return D3D_ERR_BAD_ARG;
    }
    if (g_noAlloc) {
      setError("SPConvMM keeps its neighbour table in library-allocated memory: use d3d_enqueue");
      return D3D_ERR_UNSUPPORTED;
    }
    const int32_t dtype = inDesc[0].dtype;
    if (!featureType(dtype) || outDesc[0].dtype != dtype) {
      setError("SPConvMM: feature dtype %d / output dtype %d not implemented", dtype, outDesc[0].dtype);
      return D3D_ERR_UNSUPPORTED;  // the reference returns -1 here too (mm_trt.cu:204)
    }
    if (inDesc[0].nb_dims != 2 || inDesc[0].dims[1] != cin || outDesc[0].nb_dims != 2 ||
        outDesc[0].dims[1] != cout || inDesc[3].nb_dims != 2 || inDesc[3].dims[0] != 3) {
      setError("SPConvMM: expected inFeats [*, %d], index [3, *], outFeats [*, %d]", cin, cout);
      return D3D_ERR_BAD_ARG;
    }
    if (dev->dtype != dtype) {  // a plugin enqueued without configurePlugin, or with another dtype
      if (streamIsCapturing(stream)) {  // converting and uploading the weights allocates and synchronises
        setError("SPConvMM: the node was not configured for this feature type before the capture (call "
                 "d3d_configure, or enqueue it once, first)");
        return D3D_ERR_UNSUPPORTED;
      }
      int32_t rc = configure(inDesc, 1, nullptr, 0);
      if (rc != D3D_OK) return rc;
    }
    const RoctxRange range("d3d convolution");
    const int64_t rowLen = inDesc[3].dims[1];  // numIndicesMax, mm_trt.cu:169
    const int64_t outRows = outDesc[0].dims[0];
    const int32_t* nbr = nullptr;
    const unsigned long long* masks = nullptr;
    std::shared_ptr<RulebookLink> held = linked;  // by-products are read by the kernels launched below
    if (held && !inverse) {
      std::lock_guard<std::mutex> lock(held->mutex);
      if (held->tableValid && held->index == inputs[3] && held->numIndex == inputs[4] && held->kVol == kernelVol &&
          held->outRows == outRows && held->rowLen == rowLen) {
        nbr = static_cast<const int32_t*>(held->table.ptr);
        if (held->masksValid) masks = static_cast<const unsigned long long*>(held->masks.ptr);
      }
    }
    int32_t rc = D3D_OK;
    if (!nbr && held) {
      // the table cannot be used (other shapes, an inverse convolution): the index tensor is all there is to go
      // by - unless the operator it is linked to left exactly that tensor unwritten on its last enqueue
      std::lock_guard<std::mutex> lock(held->mutex);
      if (!held->indexWritten && held->index == inputs[3]) {
        setError("SPConvMM: the linked rulebook operator left this index tensor unwritten (D3D_OPT_INDEX_UNUSED) "
                 "and its table does not fit this convolution");
        return D3D_ERR_UNSUPPORTED;
      }
    }
    if (!nbr) {  // the index tensor is all there is to go by: derive the table from it
      if (!derived) derived = std::make_shared<DeviceBuffer>();
      const size_t bytes = static_cast<size_t>(kernelVol) * static_cast<size_t>(outRows > 0 ? outRows : 1) * sizeof(int32_t);
      if (derived->bytes < bytes && streamIsCapturing(stream)) {
        setError("SPConvMM: the table derived from the index tensor needs %zu bytes that were not reserved before the "
                 "capture (configure the node at these shapes, or enqueue it once, first)", bytes);
        return D3D_ERR_UNSUPPORTED;
      }
      rc = derived->reserve(bytes);
      if (rc != D3D_OK) return rc;
      rc = launchBuildNeighbours(static_cast<const int32_t*>(inputs[3]), rowLen, static_cast<const int32_t*>(inputs[4]),
                                 inverse, kernelVol, outRows, inDesc[0].dims[0], static_cast<int32_t*>(derived->ptr), stream);
      if (rc != D3D_OK) return rc;
      nbr = static_cast<const int32_t*>(derived->ptr);
    }
    const void* zeros = zeroRow();
    ConvArgs a{};
    a.dtype = dtype;
    a.kVol = kernelVol;
    a.cin = cin;
    a.cout = cout;
    a.inRows = inDesc[0].dims[0];
    a.outRows = outRows;
    a.in = inputs[0];
    a.inNarrow = inputs[0];
    a.cinNarrow = cin;
    a.staged = stagedOverride();
    if (dev->cinMfma > cin && a.staged == 0 && convReadsNarrowRows(dtype, kernelVol, cin, cout) &&
        ((reinterpret_cast<uintptr_t>(inputs[0]) | reinterpret_cast<uintptr_t>(outputs[0])) & 15) == 0 &&
        (dtype == D3D_INT8 || debugEnv("D3D_CONV_NO_PAD") == nullptr) && tileRowsOverride() == 0) {
      a.cin = dev->cinMfma;       // the kernel reads the rows as they are and multiplies zeros for the rest
      a.rowChannels = cin;
    } else if (dev->cinMfma > cin && (dtype == D3D_INT8 || ((reinterpret_cast<uintptr_t>(outputs[0]) & 15) == 0 &&
                                                     debugEnv("D3D_CONV_NO_PAD") == nullptr))) {  // narrow layer: widen the rows, then MFMA
      if (!widened) widened = std::make_shared<DeviceBuffer>();
      const int es = dtypeBytes(dtype);
      const size_t wideBytes = static_cast<size_t>(a.inRows > 0 ? a.inRows : 1) * dev->cinMfma * es;
      if (widened->bytes < wideBytes && streamIsCapturing(stream)) {
        setError("SPConvMM: %zu bytes for the widened input rows were not reserved before the capture", wideBytes);
        return D3D_ERR_UNSUPPORTED;
      }
      rc = widened->reserve(wideBytes);
      if (rc != D3D_OK) return rc;
      rc = launchPadRows(inputs[0], a.inRows, cin * es, dev->cinMfma * es, widened->ptr, stream);
      if (rc != D3D_OK) return rc;
      a.in = widened->ptr;
      a.cin = dev->cinMfma;
    }
    a.out = outputs[0];
    a.weightsF32 = static_cast<const float*>(dev->f32.ptr);
    a.weightsMfma = dev->mfma.ptr;
    a.bias = (withBias || dtype == D3D_INT8) ? static_cast<const float*>(dev->bias.ptr) : nullptr;
    a.requantM = dtype == D3D_INT8 ? static_cast<const float*>(dev->requantM.ptr) : nullptr;
    a.nbr = nbr;
    a.tileMasks = masks;
    a.numActOut = static_cast<const int32_t*>(inputs[2]);
    a.relu = relu ? 1 : 0;
    a.zeros = zeros;
    if (const char* e = debugEnv("D3D_CONV_PIPE")) a.pipe = e[0] == '0' ? -1 : 0;
    a.tileRows = tileRowsOverride();
    return launchConv(a, stream);
  }
};

// --- BEVDensify --------------------------------------------------------------
// Attribute layout: BEVDensifyPluginParam, one int32 outChannels
// (trt/spconv/bev_densify_trt.cu:43-47; written by
// deploy3d/symfun/ops/spconv/bev_densify.py:38).
struct DensifyPlugin final : d3d_plugin {
  int32_t outChannels = 0;

  static int32_t parse(const void* data, size_t len, DensifyPlugin** out) {
    if (!data || len < 4) {
      setError("BEVDensify: attribute blob of %zu bytes, 4 expected", len);
      return D3D_ERR_BAD_BLOB;
    }
    auto p = std::unique_ptr<DensifyPlugin>(new DensifyPlugin());
    p->type = "BEVDensify";
    std::memcpy(&p->outChannels, data, 4);
    if (p->outChannels < 0) {
      setError("BEVDensify: outChannels %d", p->outChannels);
      return D3D_ERR_BAD_BLOB;
    }
    p->blob.assign(static_cast<const uint8_t*>(data), static_cast<const uint8_t*>(data) + len);
    *out = p.release();
    return D3D_OK;
  }

  d3d_plugin* clone() const override { return new DensifyPlugin(*this); }
  int32_t numOutputs() const override { return 1; }
  // [B, outChannels, Y, X] from inSpatialShape [B, 0, Z, Y, X] (bev_densify_trt.cu:86-97)
  int32_t outputDims(int32_t idx, const d3d_tensor_desc* in, int32_t nbIn, d3d_tensor_desc* out) const override {
    if (idx != 0 || !out || !in || nbIn < 4 || in[3].nb_dims != 5) return D3D_ERR_BAD_ARG;
    std::memset(out, 0, sizeof(*out));
    out->format = D3D_LINEAR;
    out->nb_dims = 4;
    out->dims[0] = in[3].dims[0];
    out->dims[1] = outChannels;
    out->dims[2] = in[3].dims[3];
    out->dims[3] = in[3].dims[4];
    return D3D_OK;
  }
  int32_t outputDtype(int32_t, const int32_t* inTypes, int32_t nbIn) const override {
    return (inTypes && nbIn > 0) ? inTypes[0] : D3D_ERR_BAD_ARG;  // bev_densify_trt.cu:98-100
  }
  // The reference takes float and half features (bev_densify_trt.cu:101-115); bf16 and int8 rows move the same way.
  static bool featureType(int32_t t) { return t == D3D_HALF || t == D3D_FLOAT || t == D3D_BF16 || t == D3D_INT8; }
  int32_t supportsFormat(int32_t pos, const d3d_tensor_desc* io, int32_t nbIn, int32_t nbOut) const override {
    if (!io || pos < 0 || pos >= nbIn + nbOut || io[pos].format != D3D_LINEAR) return 0;
    if (pos == 0) return featureType(io[0].dtype);
    if (pos <= 3) return io[pos].dtype == D3D_INT32;
    return io[pos].dtype == io[0].dtype;
  }
  int32_t configure(const d3d_tensor_desc*, int32_t, const d3d_tensor_desc*, int32_t) override { return D3D_OK; }
  // One int32 per cell of the grid: the cell -> row table.  (The reference needs none, bev_densify_trt.cu:130-135;
  // it pays with a clearing pass and channel-strided stores instead.)
  size_t workspaceSize(const d3d_tensor_desc* in, int32_t nbIn) const override {
    if (!in || nbIn < 4 || in[3].nb_dims != 5) return 0;
    return densifyWorkspaceBytes(in[3].dims[0], in[3].dims[2], in[3].dims[3], in[3].dims[4]);
  }
  int32_t enqueue(const d3d_tensor_desc* inDesc, const d3d_tensor_desc* outDesc, const void* const* inputs,
                  void* const* outputs, void* workspace, size_t workspaceBytes, hipStream_t stream) override {
    if (!inDesc || !outDesc || !inputs || !outputs) return D3D_ERR_BAD_ARG;
    if (inDesc[0].nb_dims != 2 || inDesc[1].nb_dims != 2 || inDesc[1].dims[1] != 4 || inDesc[3].nb_dims != 5 ||
        inDesc[1].dims[0] < inDesc[0].dims[0]) {
      setError("BEVDensify: expects inFeats [cap, C], inCoors [cap, 4], numActIn [1], inSpatialShape [B, 0, Z, Y, X]");
      return D3D_ERR_BAD_ARG;
    }
    const int32_t dtype = inDesc[0].dtype;
    if (!featureType(dtype)) {
      setError("BEVDensify: feature dtype %d not implemented", dtype);
      return D3D_ERR_UNSUPPORTED;
    }
    const int64_t cap = inDesc[0].dims[0], C = inDesc[0].dims[1];
    const int64_t B = inDesc[3].dims[0], Z = inDesc[3].dims[2], Y = inDesc[3].dims[3], X = inDesc[3].dims[4];
    if (B < 0 || Z < 0 || Y < 0 || X < 0 || cap > 0x7fffffff || C > 0x7fffffff || B > 0x7fffffff || Z > 0x7fffffff ||
        Y > 0x7fffffff || X > 0x7fffffff) {
      setError("BEVDensify: tensor extents out of range");
      return D3D_ERR_BAD_ARG;
    }
    // The map is addressed as [B, C, Z, Y, X] and handed on as [B, outChannels, Y, X] (bev_densify_trt.cu:160-163).
    if (C * Z != outChannels) {
      setError("BEVDensify: outChannels %d but the input has %lld channels on %lld levels", outChannels,
               static_cast<long long>(C), static_cast<long long>(Z));
      return D3D_ERR_BAD_ARG;
    }
    if (outDesc[0].nb_dims != 4 || outDesc[0].dims[0] != B || outDesc[0].dims[1] != outChannels ||
        outDesc[0].dims[2] != Y || outDesc[0].dims[3] != X || outDesc[0].dtype != dtype) {
      setError("BEVDensify: output must be [B, outChannels, Y, X] of the feature type");
      return D3D_ERR_BAD_ARG;
    }
    if (B * C * Z * Y * X == 0) return D3D_OK;
    if (!outputs[0] || !inputs[2] || (cap > 0 && (!inputs[0] || !inputs[1]))) {
      setError("BEVDensify: null tensor pointer");
      return D3D_ERR_BAD_ARG;
    }
    DensifyArgs a{};
    a.feats = inputs[0];
    a.coors = static_cast<const int32_t*>(inputs[1]);
    a.numAct = static_cast<const int32_t*>(inputs[2]);
    a.cap = static_cast<int32_t>(cap);
    a.C = static_cast<int>(C);
    a.elemBytes = dtypeBytes(dtype);
    a.B = static_cast<int>(B);
    a.Z = static_cast<int>(Z);
    a.Y = static_cast<int>(Y);
    a.X = static_cast<int>(X);
    a.out = outputs[0];
    a.workspace = workspace;
    a.workspaceBytes = workspaceBytes;
    return launchDensify(a, stream);
  }
};

// --- SimpleMeanEncoder -------------------------------------------------------
// Attribute layout: SimpleMeanEncoderPluginParam, one int32 maxNumActOut
// (trt/voxel_encoder/simple_mean_trt.cu:176-180; written by
// deploy3d/symfun/ops/voxel_encoder/simple_mean.py:44).
struct VoxelizePlugin final : d3d_plugin {
  int32_t maxNumActOut = 0;

  static int32_t parse(const void* data, size_t len, VoxelizePlugin** out) {
    if (!data || len < 4) {
      setError("SimpleMeanEncoder: attribute blob of %zu bytes, 4 expected", len);
      return D3D_ERR_BAD_BLOB;
    }
    auto p = std::unique_ptr<VoxelizePlugin>(new VoxelizePlugin());
    p->type = "SimpleMeanEncoder";
    std::memcpy(&p->maxNumActOut, data, 4);
    if (p->maxNumActOut < 0) {
      setError("SimpleMeanEncoder: maxNumActOut %d", p->maxNumActOut);
      return D3D_ERR_BAD_BLOB;
    }
    p->blob.assign(static_cast<const uint8_t*>(data), static_cast<const uint8_t*>(data) + len);
    *out = p.release();
    return D3D_OK;
  }

  d3d_plugin* clone() const override { return new VoxelizePlugin(*this); }
  int32_t numOutputs() const override { return 3; }
  // outFeats [maxNumActOut, C], outCoors [maxNumActOut, 4], numActOut [1] (simple_mean_trt.cu:221-238)
  int32_t outputDims(int32_t idx, const d3d_tensor_desc* in, int32_t nbIn, d3d_tensor_desc* out) const override {
    if (idx < 0 || idx > 2 || !out || !in || nbIn < 1 || in[0].nb_dims != 2) return D3D_ERR_BAD_ARG;
    std::memset(out, 0, sizeof(*out));
    out->format = D3D_LINEAR;
    if (idx == 2) {
      out->nb_dims = 1;
      out->dims[0] = 1;
      return D3D_OK;
    }
    out->nb_dims = 2;
    out->dims[0] = maxNumActOut;
    out->dims[1] = idx == 0 ? in[0].dims[1] : 4;
    return D3D_OK;
  }
  int32_t outputDtype(int32_t idx, const int32_t* inTypes, int32_t nbIn) const override {
    if (!inTypes || nbIn < 1) return D3D_ERR_BAD_ARG;
    return idx == 0 ? inTypes[0] : D3D_INT32;  // simple_mean_trt.cu:239-244
  }
  // simple_mean_trt.cu:245-258: point features, voxel config and voxel features float; the rest int32
  int32_t supportsFormat(int32_t pos, const d3d_tensor_desc* io, int32_t nbIn, int32_t nbOut) const override {
    if (!io || pos < 0 || pos >= nbIn + nbOut || io[pos].format != D3D_LINEAR) return 0;
    if (pos == 0) return io[0].dtype == D3D_FLOAT;
    if (pos == 1 || pos == 3 || pos == 5 || pos == 6) return io[pos].dtype == D3D_INT32;
    return io[pos].dtype == io[0].dtype;
  }
  int32_t configure(const d3d_tensor_desc*, int32_t, const d3d_tensor_desc*, int32_t) override { return D3D_OK; }
  size_t workspaceSize(const d3d_tensor_desc* in, int32_t nbIn) const override {  // simple_mean_trt.cu:273-278
    if (!in || nbIn < 1 || in[0].nb_dims != 2) return 0;
    return voxelizeWorkspaceBytes(in[0].dims[0], maxNumActOut);
  }
  int32_t enqueue(const d3d_tensor_desc* inDesc, const d3d_tensor_desc* outDesc, const void* const* inputs,
                  void* const* outputs, void* workspace, size_t workspaceBytes, hipStream_t stream) override {
    if (!inDesc || !outDesc || !inputs || !outputs) return D3D_ERR_BAD_ARG;
    if (inDesc[0].nb_dims != 2 || inDesc[0].dims[1] < 3 || inDesc[1].nb_dims != 1 ||
        inDesc[1].dims[0] != inDesc[0].dims[0] || inDesc[2].nb_dims != 1 || inDesc[2].dims[0] != 6 ||
        inDesc[3].nb_dims != 5) {
      setError("SimpleMeanEncoder: expects batchPointFeats [N, C >= 3], batchIndices [N], voxelConfig [6], "
               "inSpatialShape [B, 0, Z, Y, X]");
      return D3D_ERR_BAD_ARG;
    }
    if (inDesc[0].dtype != D3D_FLOAT || inDesc[2].dtype != D3D_FLOAT || inDesc[1].dtype != D3D_INT32) {
      setError("SimpleMeanEncoder: point features and voxel config must be float, batch indices int32");
      return D3D_ERR_UNSUPPORTED;
    }
    const int64_t n = inDesc[0].dims[0], C = inDesc[0].dims[1];
    const int64_t B = inDesc[3].dims[0], Z = inDesc[3].dims[2], Y = inDesc[3].dims[3], X = inDesc[3].dims[4];
    if (n < 0 || n > 0x7fffffff || C > 4096 || B < 0 || Z < 0 || Y < 0 || X < 0 || B > 0x7fffffff || Z > 0x7fffffff ||
        Y > 0x7fffffff || X > 0x7fffffff) {
      setError("SimpleMeanEncoder: tensor extents out of range");
      return D3D_ERR_BAD_ARG;
    }
    if (outDesc[0].nb_dims != 2 || outDesc[0].dims[0] != maxNumActOut || outDesc[0].dims[1] != C ||
        outDesc[1].nb_dims != 2 || outDesc[1].dims[0] != maxNumActOut || outDesc[1].dims[1] != 4) {
      setError("SimpleMeanEncoder: outputs must be [maxNumActOut, C] and [maxNumActOut, 4]");
      return D3D_ERR_BAD_ARG;
    }
    if (!outputs[2] || (maxNumActOut > 0 && (!outputs[0] || !outputs[1])) ||
        (n > 0 && (!inputs[0] || !inputs[1] || !inputs[2]))) {
      setError("SimpleMeanEncoder: null tensor pointer");
      return D3D_ERR_BAD_ARG;
    }
    VoxelizeArgs a{};
    a.feats = static_cast<const float*>(inputs[0]);
    a.batchIdx = static_cast<const int32_t*>(inputs[1]);
    a.config = static_cast<const float*>(inputs[2]);
    a.numPts = n;
    a.C = static_cast<int>(C);
    a.B = static_cast<int>(B);
    a.Z = static_cast<int>(Z);
    a.Y = static_cast<int>(Y);
    a.X = static_cast<int>(X);
    a.maxNumActOut = maxNumActOut;
    a.outFeats = static_cast<float*>(outputs[0]);
    a.outCoors = static_cast<int32_t*>(outputs[1]);
    a.numActOut = static_cast<int32_t*>(outputs[2]);
    a.workspace = workspace;
    a.workspaceBytes = workspaceBytes;
    return launchVoxelize(a, stream);
  }
};

struct OpEntry {
  const char* name;
  int nd;  // 0 = SPConvMM, -1 = BEVDensify, -2 = SimpleMeanEncoder
};
constexpr OpEntry kOps[] = {{"SPConvIdx1d", 1}, {"SPConvIdx2d", 2}, {"SPConvIdx3d", 3}, {"SPConvIdx4d", 4},
                            {"SPConvMM", 0},    {"BEVDensify", -1},  {"SimpleMeanEncoder", -2}};
constexpr const char* kVersion = "2.0";

}  // namespace
}  // namespace d3d

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
using namespace d3d;

#define D3D_GUARD_BEGIN try {
#define D3D_GUARD_END(ret)                         \
  }                                                \
  catch (const std::bad_alloc&) {                  \
    setError("out of host memory");                \
    return ret;                                    \
  }                                                \
  catch (...) {                                    \
    setError("unexpected C++ exception");          \
    return ret;                                    \
  }

extern "C" {

int32_t d3d_create(const char* name, const char* version, const void* blob, size_t len, d3d_plugin** out) {
  D3D_GUARD_BEGIN
  if (!name || !out) {
    setError("d3d_create: null name or output pointer");
    return D3D_ERR_BAD_ARG;
  }
  *out = nullptr;
  if (version && std::strcmp(version, kVersion) != 0) {
    setError("operator %s version %s not registered (have %s)", name, version, kVersion);
    return D3D_ERR_UNKNOWN_OP;
  }
  for (const OpEntry& op : kOps) {
    if (std::strcmp(name, op.name) != 0) continue;
    if (op.nd == -2) {
      VoxelizePlugin* p = nullptr;
      int32_t rc = VoxelizePlugin::parse(blob, len, &p);
      *out = p;
      return rc;
    }
    if (op.nd == -1) {
      DensifyPlugin* p = nullptr;
      int32_t rc = DensifyPlugin::parse(blob, len, &p);
      *out = p;
      return rc;
    }
    if (op.nd == 0) {
      MMPlugin* p = nullptr;
      int32_t rc = MMPlugin::parse(blob, len, &p);
      *out = p;
      return rc;
    }
    IdxPlugin* p = nullptr;
    int32_t rc = IdxPlugin::parse(op.nd, blob, len, &p);
    *out = p;
    return rc;
  }
  setError("operator %s not registered", name);
  return D3D_ERR_UNKNOWN_OP;
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

int32_t d3d_clone(const d3d_plugin* p, d3d_plugin** out) {
  D3D_GUARD_BEGIN
  if (!p || !out) return D3D_ERR_BAD_ARG;
  *out = p->clone();
  return D3D_OK;
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

void d3d_destroy(d3d_plugin* p) { delete p; }

const char* d3d_plugin_type(const d3d_plugin* p) { return p ? p->type.c_str() : ""; }
const char* d3d_plugin_version(const d3d_plugin*) { return kVersion; }

size_t d3d_serialize_size(const d3d_plugin* p) { return p ? p->blob.size() : 0; }

int32_t d3d_serialize(const d3d_plugin* p, void* buffer, size_t len) {
  if (!p || !buffer) return D3D_ERR_BAD_ARG;
  if (len < p->blob.size()) {
    setError("serialize: buffer of %zu bytes, %zu needed", len, p->blob.size());
    return D3D_ERR_BAD_ARG;
  }
  std::memcpy(buffer, p->blob.data(), p->blob.size());
  return D3D_OK;
}

int32_t d3d_num_outputs(const d3d_plugin* p) { return p ? p->numOutputs() : D3D_ERR_BAD_ARG; }

int32_t d3d_output_dims(const d3d_plugin* p, int32_t output_index, const d3d_tensor_desc* in, int32_t nb_in,
                        d3d_tensor_desc* out) {
  D3D_GUARD_BEGIN
  if (!p) return D3D_ERR_BAD_ARG;
  return p->outputDims(output_index, in, nb_in, out);
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

int32_t d3d_output_dtype(const d3d_plugin* p, int32_t output_index, const int32_t* in_dtypes, int32_t nb_in) {
  if (!p) return D3D_ERR_BAD_ARG;
  return p->outputDtype(output_index, in_dtypes, nb_in);
}

int32_t d3d_supports_format(const d3d_plugin* p, int32_t pos, const d3d_tensor_desc* in_out, int32_t nb_in,
                            int32_t nb_out) {
  if (!p) return 0;
  return p->supportsFormat(pos, in_out, nb_in, nb_out);
}

int32_t d3d_configure(d3d_plugin* p, const d3d_tensor_desc* in, int32_t nb_in, const d3d_tensor_desc* out,
                      int32_t nb_out) {
  D3D_GUARD_BEGIN
  if (!p) return D3D_ERR_BAD_ARG;
  return p->configure(in, nb_in, out, nb_out);
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

size_t d3d_workspace_size(const d3d_plugin* p, const d3d_tensor_desc* in, int32_t nb_in, const d3d_tensor_desc*,
                          int32_t) {
  if (!p) return 0;
  return p->workspaceSize(in, nb_in);
}

int32_t d3d_enqueue(d3d_plugin* p, const d3d_tensor_desc* in_desc, const d3d_tensor_desc* out_desc,
                    const void* const* inputs, void* const* outputs, void* workspace, size_t workspace_bytes,
                    void* stream) {
  D3D_GUARD_BEGIN
  if (!p) return D3D_ERR_BAD_ARG;
  return p->enqueue(in_desc, out_desc, inputs, outputs, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

int32_t d3d_enqueue_static(d3d_plugin* p, const d3d_tensor_desc* in_desc, const d3d_tensor_desc* out_desc,
                           const void* const* inputs, void* const* outputs, void* stream) {
  D3D_GUARD_BEGIN
  if (!p) return D3D_ERR_BAD_ARG;
  void* ws = nullptr;
  size_t wsBytes = 0;
  int32_t rc = staticScratch(&ws, &wsBytes);
  if (rc != D3D_OK) return rc;
  struct Scope {
    Scope() { g_noAlloc = true; }
    ~Scope() { g_noAlloc = false; }
  } scope;
  return p->enqueue(in_desc, out_desc, inputs, outputs, ws, wsBytes, static_cast<hipStream_t>(stream));
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

const char* d3d_last_error(void) { return lastError(); }

int32_t d3d_num_ops(void) { return static_cast<int32_t>(sizeof(kOps) / sizeof(kOps[0])); }
const char* d3d_op_name(int32_t i) { return (i >= 0 && i < d3d_num_ops()) ? kOps[i].name : ""; }

int32_t d3d_link_rulebook(d3d_plugin* mm, d3d_plugin* idx) {
  D3D_GUARD_BEGIN
  auto* m = dynamic_cast<MMPlugin*>(mm);
  if (!m) {
    setError("d3d_link_rulebook: the first handle must be an SPConvMM");
    return D3D_ERR_BAD_ARG;
  }
  if (!idx) {
    m->linked.reset();
    return D3D_OK;
  }
  auto* r = dynamic_cast<IdxPlugin*>(idx);
  if (!r) {
    setError("d3d_link_rulebook: the second handle must be an SPConvIdx{N}d");
    return D3D_ERR_BAD_ARG;
  }
  if (r->kVol() != m->kernelVol) {
    setError("d3d_link_rulebook: kernel volume %d of the convolution, %d of the rulebook", m->kernelVol, r->kVol());
    return D3D_ERR_BAD_ARG;
  }
  // The table the rulebook operator writes has maxNumActOut rows of ITS blob; a forward convolution whose own
  // maxNumActOut differs could never use it (and, were the index tensor left unwritten for its sake, would have
  // nothing to work from).  An inverse convolution derives its table from the index tensor whatever the sizes.
  if (!m->inverse && r->maxNumActOut != m->maxNumActOut) {
    setError("d3d_link_rulebook: maxNumActOut %d of the convolution, %d of the rulebook", m->maxNumActOut,
             r->maxNumActOut);
    return D3D_ERR_BAD_ARG;
  }
  // tile masks are read by the kernels of layers with at least 32 (widened) input channels
  int32_t rc = r->wantByProducts(m->cin > 16);
  if (rc != D3D_OK) return rc;
  m->linked = r->link;
  return D3D_OK;
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

int32_t d3d_link_coords(d3d_plugin* subm, d3d_plugin* producer) {
  D3D_GUARD_BEGIN
  auto* s = dynamic_cast<IdxPlugin*>(subm);
  if (!s) {
    setError("d3d_link_coords: the first handle must be an SPConvIdx{N}d");
    return D3D_ERR_BAD_ARG;
  }
  if (!producer) {
    s->coordSource.reset();
    return D3D_OK;
  }
  auto* r = dynamic_cast<IdxPlugin*>(producer);
  if (!r || r->subM || r->nd != s->nd) {
    setError("d3d_link_coords: the second handle must be a strided or transposed SPConvIdx%dd", s->nd);
    return D3D_ERR_BAD_ARG;
  }
  {
    std::lock_guard<std::mutex> lock(r->link->mutex);
    r->link->shareMap = true;
  }
  s->coordSource = r->link;
  return D3D_OK;
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

int32_t d3d_set_option(d3d_plugin* p, int32_t option, int64_t value) {
  D3D_GUARD_BEGIN
  if (!p) return D3D_ERR_BAD_ARG;
  return p->setOption(option, value);
  D3D_GUARD_END(D3D_ERR_BAD_ARG)
}

}  // extern "C"
