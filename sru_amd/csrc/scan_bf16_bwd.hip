// Backward scan kernels and their launcher for bf16_bits streams.
#include "sru_dispatch.h"

namespace sru_amd {
template hipError_t launch_backward<bf16_bits>(const sru_amd_shape &, const BwdParams &, hipStream_t);
}  // namespace sru_amd
