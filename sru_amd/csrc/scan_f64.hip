// Forward and backward scan kernels and their launchers for double streams (the general kernels,
// computing in double).
#include "sru_dispatch.h"

namespace sru_amd {
template hipError_t launch_forward<double>(const sru_amd_shape &, const FwdParams &, hipStream_t);
template hipError_t launch_backward<double>(const sru_amd_shape &, const BwdParams &, hipStream_t);
}  // namespace sru_amd
