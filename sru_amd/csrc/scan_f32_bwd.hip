// Backward scan kernels and their launcher for float streams.
#include "sru_dispatch.h"

namespace sru_amd {
template hipError_t launch_backward<float>(const sru_amd_shape &, const BwdParams &, hipStream_t);
}  // namespace sru_amd
