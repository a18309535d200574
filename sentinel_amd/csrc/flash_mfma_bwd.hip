#include "flash_common.h"
namespace sentinel_hip {
hipError_t launch_bwd_mfma(Elem, const void*, const void*, const void*, const void*, const float*, RowMap, const void*, void*,
                           void*, void*, float*, AttnGeom, hipStream_t) {
    return hipErrorNotSupported;
}
}  // namespace sentinel_hip
