// The scratch array behind d3d_enqueue_static: a fixed block of device memory that is part of the library's
// device image, for callers that may not allocate (HIP graph capture, serving loops, harnesses that forbid
// hipMalloc).  Every GPU the library runs on holds its own copy until the process ends.
#include <mutex>

#include "common.h"

namespace d3d {
namespace {

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratchMutex;
void* g_scratchPtr[kMaxDevices] = {};  // device address of `scratch` on each device, resolved on first use

}  // namespace

// Device address and size of the scratch array on the CURRENT device.  In host code the array's name is only a
// handle for the runtime: the address a kernel can use comes from hipGetSymbolAddress, once per device.
int32_t staticScratch(void** ptr, size_t* bytes) {
  int dev = -1;
  D3D_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) {
    setError("static scratch: device ordinal %d out of range", dev);
    return D3D_ERR_DEVICE;
  }
  std::lock_guard<std::mutex> lock(g_scratchMutex);
  if (!g_scratchPtr[dev]) {
    void* p = nullptr;
    D3D_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) {
      setError("static scratch: hipGetSymbolAddress returned a null address");
      return D3D_ERR_DEVICE;
    }
    g_scratchPtr[dev] = p;
  }
  *ptr = g_scratchPtr[dev];
  *bytes = kStaticScratchBytes;
  return D3D_OK;
}

}  // namespace d3d
