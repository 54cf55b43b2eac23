// Instantiates the MFMA convolution kernels (conv_kernels.h) for one storage type.
#include "conv_kernels.h"

namespace d3d {

int32_t launchMfmaBf16(const ConvArgs& a, hipStream_t stream) { return convk::launchMfma<__bf16>(a, stream); }

}  // namespace d3d
