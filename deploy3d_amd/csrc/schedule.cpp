// A schedule: a recorded sequence of operator enqueues, replayed from native code on several HIP streams.
//
// What TensorRT's execution context does for the reference (IExecutionContext::enqueueV3 walking the engine's
// layers; deploy3d/symfun/trt_utils/trt_onnx_module.py:186-250 drives it): the caller describes a pass once -
// operator, descriptors, device pointers, workspace per step, the lane (stream) it runs on and the earlier
// steps it has to wait for - and `d3d_schedule_run` then enqueues the whole pass without going back to the
// caller's language between operators.  Lane 0 is the stream passed to run; the other lanes are streams the
// schedule owns.  Steps of one lane run in the order they were added; a step waits for the steps named in `after`
// through events, recorded only behind steps that somebody on another lane waits for.  All lanes fork from
// lane 0 when a run starts and join it when the run ends, so for the caller a run is ordinary stream-ordered work
// on its stream.  Built on the public entry point d3d_enqueue only.
#include <hip/hip_runtime.h>

#include <cstring>
#include <vector>

#include "common.h"
#include "d3d_spconv.h"

struct d3d_schedule {
  struct Step {
    d3d_plugin* plugin;
    std::vector<d3d_tensor_desc> in, out;
    std::vector<const void*> inputs;
    std::vector<void*> outputs;
    void* workspace;
    size_t workspaceBytes;
    int lane;
    std::vector<int> after;
    hipEvent_t done = nullptr;  // recorded behind the step if a step of another lane waits for it
  };
  std::vector<hipStream_t> lanes;  // [0] unused: lane 0 is the caller's stream
  std::vector<hipEvent_t> joined;  // per owned lane: its tail, for the join
  hipEvent_t fork = nullptr;
  std::vector<Step> steps;
};

namespace {

int32_t hipFail(hipError_t e, const char* what) {
  d3d::setError("schedule: %s failed: %s", what, hipGetErrorString(e));
  return D3D_ERR_DEVICE;
}

}  // namespace

extern "C" {

int32_t d3d_schedule_create(int32_t n_lanes, d3d_schedule** out) {
  if (!out || n_lanes < 1 || n_lanes > 8) {
    d3d::setError("schedule: 1 to 8 lanes");
    return D3D_ERR_BAD_ARG;
  }
  *out = nullptr;
  auto* s = new d3d_schedule();
  hipError_t e = hipSuccess;
  if (n_lanes > 1) e = hipEventCreateWithFlags(&s->fork, hipEventDisableTiming);  // one lane: no HIP object at all
  s->lanes.assign(static_cast<size_t>(n_lanes), nullptr);
  s->joined.assign(static_cast<size_t>(n_lanes), nullptr);
  for (int l = 1; l < n_lanes && e == hipSuccess; ++l) {
    e = hipStreamCreateWithFlags(&s->lanes[l], hipStreamNonBlocking);  // default priority
    if (e == hipSuccess) e = hipEventCreateWithFlags(&s->joined[l], hipEventDisableTiming);
  }
  if (e != hipSuccess) {
    d3d_schedule_destroy(s);
    return hipFail(e, "creating streams and events");
  }
  *out = s;
  return D3D_OK;
}

void d3d_schedule_destroy(d3d_schedule* s) {
  if (!s) return;
  for (auto& st : s->steps)
    if (st.done) (void)hipEventDestroy(st.done);
  for (size_t l = 1; l < s->lanes.size(); ++l) {
    if (s->lanes[l]) {
      (void)hipStreamSynchronize(s->lanes[l]);
      (void)hipStreamDestroy(s->lanes[l]);
    }
    if (s->joined[l]) (void)hipEventDestroy(s->joined[l]);
  }
  if (s->fork) (void)hipEventDestroy(s->fork);
  delete s;
}

int32_t d3d_schedule_add(d3d_schedule* s, d3d_plugin* plugin, const d3d_tensor_desc* in_desc, int32_t nb_in,
                         const d3d_tensor_desc* out_desc, int32_t nb_out, const void* const* inputs,
                         void* const* outputs, void* workspace, size_t workspace_bytes, int32_t lane,
                         const int32_t* after, int32_t nb_after) {
  if (!s || !plugin || nb_in < 0 || nb_out < 0 || nb_after < 0 || (nb_in && (!in_desc || !inputs)) ||
      (nb_out && (!out_desc || !outputs)) || (nb_after && !after) || lane < 0 ||
      lane >= static_cast<int32_t>(s->lanes.size())) {
    d3d::setError("schedule: bad step (null array, negative count or lane outside the schedule)");
    return D3D_ERR_BAD_ARG;
  }
  {
    // the operators read fixed positions of the input arrays: a shorter array is a host out-of-bounds read
    const char* type = d3d_plugin_type(plugin);
    const int32_t need = !type ? 0 : (std::strncmp(type, "SPConvIdx", 9) == 0 ? 3 : (std::strcmp(type, "SPConvMM") == 0 ? 5 : 4));
    if (nb_in < need) {
      d3d::setError("schedule: %s reads %d inputs, step names %d", type ? type : "?", need, nb_in);
      return D3D_ERR_BAD_ARG;
    }
  }
  if (nb_out != d3d_num_outputs(plugin)) {
    d3d::setError("schedule: %s has %d outputs, step names %d", d3d_plugin_type(plugin), d3d_num_outputs(plugin), nb_out);
    return D3D_ERR_BAD_ARG;
  }
  const int me = static_cast<int>(s->steps.size());
  for (int32_t i = 0; i < nb_after; ++i)
    if (after[i] < 0 || after[i] >= me) {
      d3d::setError("schedule: step %d waits for step %d, which does not precede it", me, after[i]);
      return D3D_ERR_BAD_ARG;
    }
  d3d_schedule::Step st;
  st.plugin = plugin;
  st.in.assign(in_desc, in_desc + nb_in);
  st.out.assign(out_desc, out_desc + nb_out);
  st.inputs.assign(inputs, inputs + nb_in);
  st.outputs.assign(outputs, outputs + nb_out);
  st.workspace = workspace;
  st.workspaceBytes = workspace_bytes;
  st.lane = lane;
  for (int32_t i = 0; i < nb_after; ++i) {
    d3d_schedule::Step& dep = s->steps[static_cast<size_t>(after[i])];
    if (dep.lane == lane) continue;  // stream order already holds
    if (!dep.done) {
      const hipError_t e = hipEventCreateWithFlags(&dep.done, hipEventDisableTiming);
      if (e != hipSuccess) return hipFail(e, "hipEventCreateWithFlags");
    }
    st.after.push_back(after[i]);
  }
  s->steps.push_back(std::move(st));
  return me;
}

int32_t d3d_schedule_run(d3d_schedule* s, void* stream) {
  if (!s) return D3D_ERR_BAD_ARG;
  hipStream_t main = static_cast<hipStream_t>(stream);
  // A run puts event edges between streams that are not the caller's; under stream capture that is a topology
  // this runtime has crashed on at the end of the capture.  Capture the operators' own enqueues instead.
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(main, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) {
    d3d::setError("schedule: the stream is capturing; a schedule runs eagerly");
    return D3D_ERR_UNSUPPORTED;
  }
  hipError_t e = hipSuccess;
  auto laneStream = [&](int lane) { return lane == 0 ? main : s->lanes[static_cast<size_t>(lane)]; };
  if (s->lanes.size() > 1) {
    e = hipEventRecord(s->fork, main);
    for (size_t l = 1; l < s->lanes.size() && e == hipSuccess; ++l) e = hipStreamWaitEvent(s->lanes[l], s->fork, 0);
    if (e != hipSuccess) return hipFail(e, "fork");
  }
  int32_t rc = D3D_OK;
  for (auto& st : s->steps) {
    hipStream_t q = laneStream(st.lane);
    for (int dep : st.after) {
      e = hipStreamWaitEvent(q, s->steps[static_cast<size_t>(dep)].done, 0);
      if (e != hipSuccess && rc == D3D_OK) rc = hipFail(e, "hipStreamWaitEvent");
    }
    if (rc == D3D_OK)  // after a failure nothing more is enqueued, but the lanes still join below
      rc = d3d_enqueue(st.plugin, st.in.data(), st.out.data(), st.inputs.data(), st.outputs.data(), st.workspace,
                       st.workspaceBytes, q);
    if (st.done) {
      e = hipEventRecord(st.done, q);
      if (e != hipSuccess && rc == D3D_OK) rc = hipFail(e, "hipEventRecord");
    }
  }
  for (size_t l = 1; l < s->lanes.size(); ++l) {
    e = hipEventRecord(s->joined[l], s->lanes[l]);
    if (e == hipSuccess) e = hipStreamWaitEvent(main, s->joined[l], 0);
    if (e != hipSuccess && rc == D3D_OK) rc = hipFail(e, "join");
  }
  return rc;
}

int32_t d3d_schedule_size(const d3d_schedule* s) { return s ? static_cast<int32_t>(s->steps.size()) : D3D_ERR_BAD_ARG; }

}  // extern "C"
