/* C ABI of the MI355X sparse-convolution engine.
 *
 * The library exposes the operators of deploy3d's sparse-convolution path (the
 * rulebook builder, the gather-GEMM-scatter, and the sparse-to-dense step that
 * ends the sparse part of a network, and the voxeliser in front of it) as
 * opaque plugin objects with the life cycle TensorRT drives on the
 * reference's IPluginV2DynamicExt classes: deserialize -> clone -> configure
 * -> workspace size -> enqueue (stream-ordered) -> destroy.  Every function is
 * noexcept, takes plain pointers and sizes, and returns an int32 status.
 *
 * Operator names, version and the packed attribute blobs are the reference's:
 *   "SPConvIdx1d" .. "SPConvIdx4d", version "2.0"   (trt/spconv/index_trt.cu:20-50, :287-290)
 *   "SPConvMM",                     version "2.0"   (trt/spconv/mm_trt.cu:22-37, :239)
 *   "BEVDensify",                   version "2.0"   (trt/spconv/bev_densify_trt.cu:37-47, :209)
 *   "SimpleMeanEncoder",            version "2.0"   (trt/voxel_encoder/simple_mean_trt.cu:170-180, :346)
 */
#ifndef D3D_SPCONV_H_
#define D3D_SPCONV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  0 and -1 are the reference's enqueue() results
 * (trt/spconv/mm_trt.cu:204); the others replace its print-and-continue. */
enum {
  D3D_OK = 0,
  D3D_ERR_UNSUPPORTED = -1, /* dtype / format / alignment not implemented */
  D3D_ERR_BAD_BLOB = -2,    /* attribute blob too short or inconsistent */
  D3D_ERR_BAD_ARG = -3,     /* null pointer, wrong tensor count, wrong dims */
  D3D_ERR_UNKNOWN_OP = -4,  /* (name, version) not registered */
  D3D_ERR_WORKSPACE = -5,   /* caller's workspace smaller than d3d_workspace_size() */
  D3D_ERR_DEVICE = -6       /* a HIP runtime call failed; see d3d_last_error() */
};

/* Element types; the first five values are nvinfer1::DataType's. */
enum { D3D_FLOAT = 0, D3D_HALF = 1, D3D_INT8 = 2, D3D_INT32 = 3, D3D_BOOL = 4, D3D_BF16 = 7 };

/* Tensor formats: only row-major linear (nvinfer1::TensorFormat::kLINEAR = 0). */
enum { D3D_LINEAR = 0 };

#define D3D_MAX_DIMS 8

/* Plain counterpart of nvinfer1::PluginTensorDesc. */
typedef struct d3d_tensor_desc {
  int32_t dtype;
  int32_t format;
  int32_t nb_dims;
  int32_t dims[D3D_MAX_DIMS];
} d3d_tensor_desc;

typedef struct d3d_plugin d3d_plugin;

/* IPluginCreator::deserializePlugin (trt/spconv/index_trt.cu:270-275,
 * trt/spconv/mm_trt.cu:222-227): the only constructor.  The blob is
 *   SPConvIdx{N}d: int32 kernelSize[N], stride[N], padding[N], dilation[N],
 *                  outPadding[N]; int32 maxNumActOut; u8 subM; u8 transpose
 *                  (packed; trt/spconv/index_trt.cu:39-50).  Kernel sizes, strides and
 *                  dilations must be positive: the reference's kernelSize == -1
 *                  ("the whole extent", output extent 1: trt/spconv/geometry.h:129-131),
 *                  which none of its own operators or tests produce, is refused with
 *                  D3D_ERR_BAD_BLOB.
 *   SPConvMM:      int32 kernelVol, inChannels, outChannels, maxNumActOut;
 *                  u8 subM(ignored), inverse, withBias; fp32 W[kVol*Cin*Cout];
 *                  fp32 bias[Cout] iff withBias  (trt/spconv/mm_trt.cu:27-37, :61-68)
 *                  optionally followed by a 20-byte extension record
 *                  {u32 magic 'D3DX'; u32 version 1; u32 flags (bit0 fused ReLU);
 *                   f32 actScaleIn; f32 actScaleOut} that the reference's parser
 *                  skips as trailing floats.
 *   BEVDensify:    int32 outChannels  (trt/spconv/bev_densify_trt.cu:43-47, :199-204)
 *   SimpleMeanEncoder: int32 maxNumActOut  (trt/voxel_encoder/simple_mean_trt.cu:176-180, :335-339) */
int32_t d3d_create(const char* name, const char* version, const void* blob, size_t len, d3d_plugin** out);

/* IPluginV2DynamicExt::clone (index_trt.cu:75-79, mm_trt.cu:75-79): clones share device weights. */
int32_t d3d_clone(const d3d_plugin* p, d3d_plugin** out);

/* destroy() (index_trt.cu:82, mm_trt.cu:82). */
void d3d_destroy(d3d_plugin* p);

/* getPluginType / getPluginVersion / getPluginNamespace (index_trt.cu:165-168). */
const char* d3d_plugin_type(const d3d_plugin* p);
const char* d3d_plugin_version(const d3d_plugin* p);

/* getSerializationSize / serialize (index_trt.cu:70-74, mm_trt.cu:69-74): byte-exact round trip. */
size_t d3d_serialize_size(const d3d_plugin* p);
int32_t d3d_serialize(const d3d_plugin* p, void* buffer, size_t len);

/* getNbOutputs (index_trt.cu:98-101: 2 for SubM, 5 otherwise; mm_trt.cu:97). */
int32_t d3d_num_outputs(const d3d_plugin* p);

/* getOutputDimensions (index_trt.cu:102-151, mm_trt.cu:98-103).  `in` holds the
 * operator's input descriptors; only their dims are read. */
int32_t d3d_output_dims(const d3d_plugin* p, int32_t output_index, const d3d_tensor_desc* in, int32_t nb_in,
                        d3d_tensor_desc* out);

/* getOutputDataType (index_trt.cu:153-155: int32; mm_trt.cu:104-106: type of input 0). */
int32_t d3d_output_dtype(const d3d_plugin* p, int32_t output_index, const int32_t* in_dtypes, int32_t nb_in);

/* supportsFormatCombination (index_trt.cu:156-161, mm_trt.cu:107-117).  Returns 1 or 0.
 * Beyond the reference's fp16, SPConvMM also accepts fp32, bf16 and int8 features. */
int32_t d3d_supports_format(const d3d_plugin* p, int32_t pos, const d3d_tensor_desc* in_out, int32_t nb_in,
                            int32_t nb_out);

/* configurePlugin (mm_trt.cu:127-142): converts the fp32 weights of the blob to
 * the feature dtype of in[0] and uploads them (synchronous, default stream). */
int32_t d3d_configure(d3d_plugin* p, const d3d_tensor_desc* in, int32_t nb_in, const d3d_tensor_desc* out,
                      int32_t nb_out);

/* getWorkspaceSize (index_trt.cu:178-187, mm_trt.cu:143-148), from capacities only. */
size_t d3d_workspace_size(const d3d_plugin* p, const d3d_tensor_desc* in, int32_t nb_in, const d3d_tensor_desc* out,
                          int32_t nb_out);

/* enqueue (index_trt.cu:188-248, mm_trt.cu:149-205).  `stream` is a hipStream_t.
 * Stream-ordered, no host synchronisation: live counts are read on the device.
 *
 * SPConvIdx{N}d  inputs : 0 inCoors int32 [cap, N+1] (b, spatial...), 1 numActIn int32 [1],
 *                         2 inSpatialShape (dims [B, 0, spatial...] only; pointer unused)
 *                outputs: 0 index int32 [3, kVol*(cap+128)], 1 numIndex int32 [1],
 *                         (non-SubM) 2 outCoors int32 [maxNumActOut, N+1], 3 numActOut int32 [1],
 *                         4 outSpatialShape (dims only)
 * SPConvMM       inputs : 0 inFeats [capIn, Cin], 1 numActIn [1], 2 numActOut [1],
 *                         3 index int32 [3, L], 4 numIndex int32 [1]
 *                outputs: 0 outFeats [maxNumActOut, Cout], dtype of input 0
 * BEVDensify     (bev_densify_trt.cu:136-176; float, half, and also bf16 / int8 rows)
 *                inputs : 0 inFeats [cap, C], 1 inCoors int32 [cap, 4] (b, z, y, x), 2 numActIn int32 [1],
 *                         3 inSpatialShape (dims [B, 0, Z, Y, X] only; pointer unused)
 *                outputs: 0 outFeatMaps [B, outChannels = C*Z, Y, X], dtype of input 0: zero except
 *                         out[b, c*Z + z, y, x] = inFeats[i, c] for live row i at (b, z, y, x)
 *                workspace: one int32 per grid cell (the reference needs none); rows outside the grid
 *                         are skipped, and of rows naming one cell the highest stays
 * SimpleMeanEncoder (simple_mean_trt.cu:279-311; float features only, as in the reference)
 *                inputs : 0 batchPointFeats float [N, C >= 3] (x y z first), 1 batchIndices int32 [N]
 *                         (negative = skip), 2 voxelConfig float [6] on the device (xMin yMin zMin xSize ySize
 *                         zSize), 3 inSpatialShape (dims [B, 0, Z, Y, X] only; pointer unused)
 *                outputs: 0 outFeats float [maxNumActOut, C] (mean per voxel; zero past numActOut),
 *                         1 outCoors int32 [maxNumActOut, 4] (b, z, y, x), 2 numActOut int32 [1]
 *                         = min(occupied cells, maxNumActOut); voxels in order of first appearance */
int32_t d3d_enqueue(d3d_plugin* p, const d3d_tensor_desc* in_desc, const d3d_tensor_desc* out_desc,
                    const void* const* inputs, void* const* outputs, void* workspace, size_t workspace_bytes,
                    void* stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory or hand over a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  d3d_enqueue for SPConvIdx{N}d,
 * BEVDensify and SimpleMeanEncoder with the workspace taken from a fixed array of D3D_STATIC_SCRATCH_BYTES that is
 * part of the library's device image (each GPU the library runs on holds it until the process ends).  Calls no
 * hipMalloc / hipFree; an operator whose d3d_workspace_size() exceeds the array returns D3D_ERR_WORKSPACE, and
 * SPConvMM (which may have to derive a table into library-allocated memory) returns D3D_ERR_UNSUPPORTED.  All calls on one
 * GPU share the array: calls that overlap in time on one GPU (two streams, two threads) race; calls ordered on
 * one stream do not, since every operator clears what it needs zeroed itself. */
#define D3D_STATIC_SCRATCH_BYTES (64u << 20)
int32_t d3d_enqueue_static(d3d_plugin* p, const d3d_tensor_desc* in_desc, const d3d_tensor_desc* out_desc,
                           const void* const* inputs, void* const* outputs, void* stream);

/* Text of the last error on the calling thread ("" if none).  Replaces the
 * reference's std::cout reporting (trt/include/common/macros.h:14-34). */
const char* d3d_last_error(void);

/* Library-wide queries used by loaders: number of registered operators and their names. */
int32_t d3d_num_ops(void);
const char* d3d_op_name(int32_t i);

/* No counterpart in the reference, whose SPConvMM re-reads the index tensor on every enqueue
 * (trt/spconv/mm_trt.cu:166-170) and so does an SPConvMM of this library that nobody linked: it derives the
 * output-major neighbour table its kernels read from the index tensor it is handed, every time.
 * d3d_link_rulebook(mm, idx) tells the convolution `mm` that its index tensor (inputs 3 and 4) is output 0 and 1 of
 * the rulebook operator `idx` - the edge an engine builder sees in the graph.  From then on `idx` writes the
 * table (and the tap masks of 64-row tiles) itself while it compacts the pairs, into device memory that the two
 * handles own together (allocated here, freed when the last of them is destroyed), and `mm` uses it whenever the
 * index tensor it is handed is the one `idx` wrote last, at the same shapes; any other tensor is still derived.
 * Several convolutions may be linked to one rulebook operator (the reference's indice_key sharing);
 * idx = NULL removes the link.  What the link cannot see: a caller that edits the index tensor in place between
 * the two enqueues - do not link such graphs.  A convolution accumulates one input per (tap, output row): an
 * index tensor that names several (duplicate input coordinates) keeps the highest input row. */
int32_t d3d_link_rulebook(d3d_plugin* mm, d3d_plugin* idx);

/* No counterpart in the reference.  d3d_link_coords(consumer, producer) tells the rulebook operator `consumer`
 * that its inCoors / numActIn (inputs 0 and 1) are outCoors / numActOut (outputs 2 and 3) of the strided or
 * transposed operator `producer` - again an edge of the graph.  `producer` then keeps the occupancy map of its
 * output grid in memory the two handles own together (allocated at its next configure or enqueue, freed with the
 * last handle).  A submanifold `consumer` uses that map instead of clearing, marking and scanning a map of the same
 * grid itself; a strided one (3x3x3 with stride 2 and padding 1, or 3x1x1 with stride (2,1,1) and padding 0)
 * derives the occupancy of its own output grid from it instead of marking it input by input - whenever the tensors
 * it is handed are the ones `producer` wrote last, on the same grid and capacity; otherwise it works from the
 * coordinates alone, as an operator nobody linked does.  Several operators may be linked to one producer;
 * producer = NULL removes the link.  As with d3d_link_rulebook: do not link when something edits the coordinates
 * between the two enqueues. */
int32_t d3d_link_coords(d3d_plugin* consumer, d3d_plugin* producer);

/* Options, none of which the reference has.
 * D3D_OPT_PERSISTENT_INDEX (SPConvIdx{N}d; value 0 / 1): the caller promises that the index tensor this handle
 * writes (output 0) is the same buffer on every enqueue and that nothing else writes to it in between - true for
 * a runner that owns its buffers, not for a buffer an executor recycles for other tensors.  The operator then sets
 * to -1 only the slots its previous pass used and the new one does not, instead of the whole tensor at capacity
 * (reference: cudaMemsetAsync of the whole tensor, trt/spconv/index.cu:352-354); after every enqueue the tensor
 * still reads -1 in every unused slot.  The first enqueue on a buffer, and the first after the buffer or its shape
 * changed, fill it whole.
 * D3D_OPT_INDEX_UNUSED (SPConvIdx{N}d; value 0 / 1): the caller promises that nothing reads the index tensor
 * (output 0) except forward convolutions linked to this operator with d3d_link_rulebook - the situation of an
 * engine in which the tensor is an edge between these nodes only.  Where the operator can write what those
 * convolutions read without compacting the pairs (3-D kernels 3x3x3, 3x1x1, 3x1x3, 1x3x3 at dilation 1 on the
 * occupancy map), it then leaves output 0 unwritten: its content is unspecified, numIndex (output 1) and the
 * coordinate outputs are written as always.  Without linked convolutions, and for every other geometry, the
 * option changes nothing.  An inverse convolution, an unlinked one, or any other reader of output 0 needs it off. */
enum { D3D_OPT_PERSISTENT_INDEX = 1, D3D_OPT_INDEX_UNUSED = 2 };
int32_t d3d_set_option(d3d_plugin* p, int32_t option, int64_t value);

/* ---- a pass as one native call -------------------------------------------------------------------------------
 * Replaces, for a chain of these operators, what TensorRT's execution context does in the reference
 * (IExecutionContext::enqueueV3 walking the engine's layers; the reference drives it from
 * deploy3d/symfun/trt_utils/trt_onnx_module.py:186-250): the caller describes the pass once, step by step, and a run
 * then enqueues every step from native code, on several HIP streams where the steps allow it.
 *
 * d3d_schedule_create: `n_lanes` streams (1..8).  Lane 0 is the stream handed to d3d_schedule_run; the others are
 *   streams the schedule creates (default priority) and owns.
 * d3d_schedule_add: appends one d3d_enqueue call - operator, descriptors, device pointers, workspace - to run on
 *   `lane`, after the earlier steps listed in `after` (their return values).  Steps of one lane run in the order
 *   added.  Descriptors and pointer arrays are copied; the operator, the tensors and the workspace must outlive the
 *   schedule's runs, and the operator must be configured as for d3d_enqueue.  Returns the step's index (>= 0) or a
 *   negative status.
 * d3d_schedule_run: enqueues all steps; the owned lanes start behind what `stream` holds at the call and `stream`
 *   continues behind all of them, so for the caller the run is stream-ordered work on `stream`.  No host
 *   synchronisation.  Returns the first failing status; steps behind a failed one are not enqueued.  Refused with
 *   D3D_ERR_UNSUPPORTED while `stream` is capturing (capture the operators' own enqueues instead).  One thread at
 *   a time per schedule.
 * d3d_schedule_destroy: waits for the owned lanes, then frees them; the operators stay the caller's. */
typedef struct d3d_schedule d3d_schedule;
int32_t d3d_schedule_create(int32_t n_lanes, d3d_schedule** out);
int32_t d3d_schedule_add(d3d_schedule* s, d3d_plugin* plugin, const d3d_tensor_desc* in_desc, int32_t nb_in,
                         const d3d_tensor_desc* out_desc, int32_t nb_out, const void* const* inputs,
                         void* const* outputs, void* workspace, size_t workspace_bytes, int32_t lane,
                         const int32_t* after, int32_t nb_after);
int32_t d3d_schedule_size(const d3d_schedule* s);
int32_t d3d_schedule_run(d3d_schedule* s, void* stream);
void d3d_schedule_destroy(d3d_schedule* s);

#ifdef __cplusplus
}
#endif
#endif /* D3D_SPCONV_H_ */
