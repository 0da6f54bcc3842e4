// Forward scan kernels and their launcher for half_bits streams.
#include "sru_dispatch.h"

namespace sru_amd {
template hipError_t launch_forward<half_bits>(const sru_amd_shape &, const FwdParams &, hipStream_t);
}  // namespace sru_amd
