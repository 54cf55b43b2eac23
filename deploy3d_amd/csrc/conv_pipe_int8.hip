// Instantiates the software-pipelined MFMA convolution (conv_pipe.h) for int8 storage (int32 accumulation,
// requantizing store).  Built with -mllvm -amdgpu-mfma-vgpr-form like the two-byte instantiations: the kernel
// keeps its accumulators in ordinary VGPRs.
#include "conv_pipe.h"

namespace d3d {

int32_t launchPipeInt8(const ConvArgs& a, hipStream_t stream) { return convk::launchPipe<int8_t>(a, stream); }

}  // namespace d3d
