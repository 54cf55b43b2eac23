// Shared host-side declarations of the sparse-convolution engine: status
// plumbing, the geometry record handed to the rulebook kernels, and the
// launcher entry points implemented in rulebook.hip and conv.hip.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "d3d_spconv.h"

namespace d3d {

constexpr int kMaxSpatial = 4;    // SPConvIdx1d .. SPConvIdx4d
constexpr int kSegment = 128;     // tap segments of the index tensor start on multiples of 128
                                  // (reference: TBSegment, trt/spconv/index.cu:21)
constexpr int kRbThreads = 256;   // rulebook kernels: 4 wavefronts per workgroup

// Size of the scratch array of d3d_enqueue_static (scratch.hip); D3D_STATIC_SCRATCH_BYTES in the public header.
constexpr size_t kStaticScratchBytes = static_cast<size_t>(D3D_STATIC_SCRATCH_BYTES);
int32_t staticScratch(void** ptr, size_t* bytes);

// Tuning and test switches (D3D_RULEBOOK, D3D_CONV_STAGED, ...) are honoured only in a process that had
// D3D_DEBUG_ENV set when the library first looked; otherwise a query costs one cached flag, not a getenv.
inline const char* debugEnv(const char* name) {
  static const bool enabled = std::getenv("D3D_DEBUG_ENV") != nullptr;
  return enabled ? std::getenv(name) : nullptr;
}

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
  int inShape[kMaxSpatial + 1]; // input grid, same layout: a live row outside it takes part in no pair
  int kVol;
  int transpose;
};

// Workspace carve-up of one rulebook build; all offsets in bytes, 256-aligned.
struct RbWorkspace {
  bool blockMap;          // dense block map (records) instead of the hash
  uint32_t nRecords;      // block map: records; nChunks = chunks of 1024 records
  uint32_t nChunks;
  uint32_t slots;         // hash slots (power of two)
  uint32_t nBlocks;       // input chunks per tap
  uint32_t cntPitch;      // 16-bit entries per tap row of cnt (a multiple of 8)
  int64_t pitch;          // row pitch of staging, a multiple of the chunk size
  size_t table;           // hash: u64 [slots] key<<32 | value;  block map: records [nRecords]
  size_t ids;             // hash: u32 [slots] output row of an occupied slot (strided only);  block map: perm [cap] (SubM)
  size_t staging;         // u32 [kVol, pitch] per (tap, input): slot, then output row, or ~0
  size_t ownCnt;          // hash: u32 [kVol, nBlocks] owned outputs per (tap, chunk) (strided only);  block map: chunk totals
  size_t cnt;             // u16 [kVol, cntPitch] valid pairs per (tap, block of 256 or 1024 inputs)
  size_t totals;          // u32 [2, kVol]  valid pairs per tap; owned outputs per tap
  size_t total;           // bytes
};

// Plan for the structure that will be used given `workspaceBytes` of workspace.
RbWorkspace planRulebookWorkspace(const RbGeom& g, int64_t cap, bool subM, size_t workspaceBytes);
// Workspace that is enough for whichever structure gets chosen.  gridKnown = g.shape holds the real output grid.
size_t rulebookWorkspaceBytes(const RbGeom& g, int64_t cap, bool subM, bool gridKnown);

// By-products of a rulebook build for the convolutions that follow it, and the state that lets a pass reuse the
// index tensor of the pass before it.  All pointers are device memory owned by the caller of launchRulebook.
struct RbSide {
  int32_t* nbr = nullptr;               // [kVol, nbrRows] pairs in output-major form: nbr[tap][output row] = input
                                        // row, -1 elsewhere; 16-byte aligned; null = not wanted
  int64_t nbrRows = 0;
  unsigned long long* masks = nullptr;  // [nMasks] bit t of masks[r / 64]: some output row of 64r..64r+63 has tap t;
                                        // written with the table of a SubM rulebook when kVol <= 64 (entries past
                                        // the rows read 0), see masksWritten
  int64_t nMasks = 0;
  uint32_t* fillState = nullptr;        // 2 words: end of the used part of the index tensor after the previous
                                        // pass / after this pass
  bool incrementalFill = false;         // the index tensor still holds the previous pass that used this fillState:
                                        // only the slots that pass used and this one does not are set to -1
  bool masksWritten = false;            // out: this build wrote `masks` (SubM rulebooks with a mirrored table)
  bool skipIndex = false;               // nothing reads the index tensor but convolutions that read nbr: where the
                                        // build can write nbr (and masks) without compacting, it leaves the index
                                        // tensor unwritten (numIndex is still written)
  bool indexWritten = true;             // out: false when skipIndex was honoured
  // One block map per stage: a strided build whose caller passes mapRecords (blockMapBytes() of them) keeps its
  // finished map of the OUTPUT grid there instead of in the workspace; a SubM build on those outputs (same grid,
  // rows in rank order, which is how a strided build numbers them) that gets the map back with useSharedMap
  // skips clearing, marking and scanning a map of its own, and the rank -> row permutation.
  void* mapRecords = nullptr;
  uint32_t* mapChunkBase = nullptr;
  bool useSharedMap = false;
  bool mapWritten = false;              // out: a strided build left its finished map in mapRecords / mapChunkBase
  // Two maps in turn: with mapState (zeroed when allocated, kept between passes: [0] scans performed so far, [1]
  // "rows not in rank order", [2] scan ticket, [3..] first-level scan tickets) and mapStride (records from the
  // first map to the second; mapRecords holds both, zeroed when allocated) a build needs no reset pass: the scan of
  // one build clears the map the next one marks.  Any build (SubM on its own inputs too) may be given its map
  // this way.  A SubM build on a shared map passes what the build that wrote it used.
  uint32_t* mapState = nullptr;
  int64_t mapStride = 0;
  bool mapDouble = false;               // out: the build alternated between the two maps (in, with useSharedMap:
                                        // the build that wrote the shared map did)
  bool mapDirty = false;                // a build with a reset pass has used these maps: keep the reset pass
  // A strided build whose input rows are the outputs of another strided build (rows in rank order of that
  // build's map, srcRows of them at capacity) may be handed that finished map of its INPUT grid: for the kernel
  // shapes it knows (3x3x3 stride 2 padding 1; 3x1x1 stride (2,1,1) padding 0) it then derives the occupancy of
  // every output brick from the input bricks underneath, inside the scan pass - no marking pass, no atomics.
  const void* srcRecords = nullptr;
  const uint32_t* srcChunkBase = nullptr;
  uint32_t* srcState = nullptr;         // with srcDouble: the source's mapState (which of its two maps is finished)
  int64_t srcStride = 0;
  bool srcDouble = false;
  bool sourceMapUsed = false;           // out
};

// 32-bit words of RbSide::mapState for a map of `chunkBaseBytes` bytes of chunk bases.
size_t mapStateWords(size_t chunkBaseBytes);

// Bytes of the block map of g's output grid (records, chunk bases); 0 when the grid takes the hash instead.
void blockMapBytes(const RbGeom& g, int64_t cap, size_t* records, size_t* chunkBase);

// Builds one rulebook on `stream`.  coors [cap, nd+1]; numActIn device int32.
// index [3, rowLen] with rowLen = kVol * (cap + 128).  outCoors / numActOut are
// null for SubM.  Returns a D3D status.
int32_t launchRulebook(const RbGeom& g, bool subM, const int32_t* coors, const int32_t* numActIn, int64_t cap,
                       int32_t maxNumActOut, int32_t* index, int32_t* numIndex, int32_t* outCoors, int32_t* numActOut,
                       void* workspace, size_t workspaceBytes, RbSide& side, hipStream_t stream);

// Out-major neighbour table of one rulebook: nbr[tap, row] = gathered input row
// or -1, rows = maxNumActOut.  Built from the index tensor (optionally with the
// gather and scatter rows swapped for an inverse convolution); pairs whose gather row lies outside [0, inRows) are dropped.
int32_t launchBuildNeighbours(const int32_t* index, int64_t rowLen, const int32_t* numIndex, bool inverse, int kVol,
                              int64_t outRows, int64_t inRows, int32_t* nbr, hipStream_t stream);

struct ConvArgs {
  int32_t dtype;          // D3D_FLOAT / D3D_HALF / D3D_BF16 / D3D_INT8
  int kVol, cin, cout;
  int64_t inRows;         // capacity rows of inFeats
  int64_t outRows;        // maxNumActOut
  const void* in;
  const void* inNarrow;   // the rows as the caller passed them, cinNarrow channels wide (in may be a widened copy)
  int cinNarrow;
  int rowChannels;        // channels a row of `in` stores when fewer than cin (the kernel reads the rest as zeros); 0 = cin
  void* out;
  const float* weightsF32;  // device fp32 [kVol, cin, cout], values already rounded to the storage type
  const void* weightsMfma;  // device storage-type, MFMA fragment-major (see MMPlugin::configure) or null
  const float* bias;      // device fp32 [cout] or null
  const float* requantM;  // int8: per-channel multiplier
  const int32_t* nbr;     // [kVol, nbrPitch]: input row that feeds output row r through tap t, at nbr[t' * nbrPitch + r]
                          // with t' = tapMirror ? kVol - 1 - t : t; -1 (or any value >= inRows) = no neighbour
  int64_t nbrPitch;       // row pitch of nbr in elements; 0 = outRows
  int tapMirror;          // the table is indexed by the mirrored tap (a SubM rulebook's input-major table, see rbCompact)
  const unsigned long long* tileMasks;  // optional [ceil(outRows / 64)]: bit t set iff any of rows 64i..64i+63 has tap t
  const int32_t* numActOut;  // device int32 or null: live output rows (tiles past them only take their bias; the
                          // kernels balance the live ones over the chip)
  const void* zeros;      // device, >= 512 zero bytes: the row that absent neighbours gather
  int relu;
  int tileRows;           // 0 = choose; else rows per workgroup of the weight-streaming MFMA kernel (128, 256, 512)
  int staged;             // staged MFMA kernel: 0 = choose, -1 = do not use it, else MT | WAVES << 8 | NS << 16 | resident << 24
  int pipe;               // software-pipelined kernel: 0 = use it where it applies, -1 = do not
};

int32_t launchConv(const ConvArgs& a, hipStream_t stream);
// The MFMA kernel family, one translation unit per storage type (conv_half.hip, conv_bf16.hip, conv_int8.hip);
// D3D_ERR_UNSUPPORTED when no instantiation fits the layer.
int32_t launchMfmaHalf(const ConvArgs& a, hipStream_t stream);
int32_t launchMfmaBf16(const ConvArgs& a, hipStream_t stream);
int32_t launchMfmaInt8(const ConvArgs& a, hipStream_t stream);
// The software-pipelined kernel (conv_pipe.h): 32 / 64 / 128 channels, kernel volumes up to 64.
int32_t launchPipeHalf(const ConvArgs& a, hipStream_t stream);
int32_t launchPipeBf16(const ConvArgs& a, hipStream_t stream);
int32_t launchPipeInt8(const ConvArgs& a, hipStream_t stream);

// True if the MFMA kernel family covers (dtype, cin, cout); otherwise the
// narrow-channel kernel runs.
bool convUsesMfma(int32_t dtype, int cin, int cout);
// Input-channel count the MFMA path would run a layer at (the next of 16/32/64/128 for 2-byte types when the
// output channels qualify), else cin itself; and the kernel that widens rows to it with zero channels.
int paddedMfmaChannels(int32_t dtype, int cin, int cout);
// True when the layer's kernel reads rows of `cin` stored channels as they are although its MFMA contracts
// paddedMfmaChannels() of them (ConvArgs::rowChannels): no widened copy of the input is needed.
bool convReadsNarrowRows(int32_t dtype, int kVol, int cin, int cout);
int32_t launchPadRows(const void* in, int64_t rows, int inBytes, int outBytes, void* out, hipStream_t stream);

// Sparse rows -> dense [B, C, Z, Y, X] map (densify.hip).  The workspace holds one int32 per cell.
struct DensifyArgs {
  const void* feats;      // [cap, C] elements of elemBytes bytes
  const int32_t* coors;   // [cap, 4] (b, z, y, x)
  const int32_t* numAct;  // device int32[1], live rows
  int32_t cap;
  int C, elemBytes;
  int B, Z, Y, X;
  void* out;
  void* workspace;
  size_t workspaceBytes;
};
// Points -> voxels with mean features (voxelize.hip).
struct VoxelizeArgs {
  const float* feats;       // [numPts, C], x y z first
  const int32_t* batchIdx;  // [numPts], negative = skip
  const float* config;      // device float[6]: xMin yMin zMin xSize ySize zSize
  int64_t numPts;
  int C;
  int B, Z, Y, X;
  int32_t maxNumActOut;
  float* outFeats;          // [maxNumActOut, C]
  int32_t* outCoors;        // [maxNumActOut, 4]
  int32_t* numActOut;       // [1]
  void* workspace;
  size_t workspaceBytes;
};
size_t voxelizeWorkspaceBytes(int64_t numPts, int64_t maxNumActOut);
int32_t launchVoxelize(const VoxelizeArgs& a, hipStream_t stream);

size_t densifyWorkspaceBytes(int64_t B, int64_t Z, int64_t Y, int64_t X);
int32_t launchDensify(const DensifyArgs& a, hipStream_t stream);

}  // namespace d3d
