// Instantiates the MFMA convolution kernels (conv_kernels.h) for one storage type.
#include "conv_kernels.h"

namespace d3d {

int32_t launchMfmaInt8(const ConvArgs& a, hipStream_t stream) { return convk::launchInt8<>(a, stream); }

bool convReadsNarrowRows(int32_t dtype, int kVol, int cin, int cout) {
  if (cout != 16 && cout != 32) return false;
  // int8: rows of 16 channels as two 8-byte loads; narrower rows read byte by byte measured slower than widening
  // them first (a 5 -> 16 layer on 120 000 rows: 19 us against 17)
  if (dtype == D3D_INT8) return cin == 16 && convk::residentFits(kVol, 32, cout, 1);
  // two-byte types: rows below 16 channels read element by element (16.3 us against 17.6 with the widening pass
  // on that layer, and no widened copy to keep)
  if (dtype == D3D_HALF || dtype == D3D_BF16) return cin < 16 && convk::residentFits(kVol, 16, cout, 2);
  return false;
}

}  // namespace d3d
