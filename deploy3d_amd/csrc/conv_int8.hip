// Instantiates the MFMA convolution kernels (conv_kernels.h) for one storage type.
#include "conv_kernels.h"

namespace d3d {

int32_t launchMfmaInt8(const ConvArgs& a, hipStream_t stream) { return convk::launchInt8<>(a, stream); }

bool convReadsNarrowRows(int32_t dtype, int kVol, int cin, int cout) {
  return dtype == D3D_INT8 && cin == 16 && (cout == 16 || cout == 32) && convk::int8ResidentFits(kVol, 32, cout);
}

}  // namespace d3d
