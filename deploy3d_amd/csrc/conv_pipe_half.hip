// Instantiates the software-pipelined MFMA convolution (conv_pipe.h) for one storage type.  Built with
// -mllvm -amdgpu-mfma-vgpr-form: the kernel keeps its accumulators in ordinary VGPRs (it fits 256 of them), and
// without the switch the compiler moves them through AGPRs with four copies per MFMA.
#include "conv_pipe.h"

namespace d3d {

int32_t launchPipeHalf(const ConvArgs& a, hipStream_t stream) { return convk::launchPipe<_Float16>(a, stream); }

}  // namespace d3d
