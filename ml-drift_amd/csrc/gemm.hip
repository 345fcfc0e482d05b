// MFMA kernels of the prefill side (placeholder translation unit until the kernels land).
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mldhip {

bool FcW4MfmaSupported(const FcArgs&) { return false; }
hipError_t LaunchFcW4Mfma(const FcArgs&, hipStream_t, const char**) { return hipErrorNotSupported; }
hipError_t LaunchConvInt8(const ConvInt8Args&, hipStream_t, const char**) { return hipErrorNotSupported; }

}  // namespace mldhip
