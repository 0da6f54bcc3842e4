// Forward scan kernels and their launcher for bf16_bits streams.
#include "sru_dispatch.h"

namespace sru_amd {
template hipError_t launch_forward<bf16_bits>(const sru_amd_shape &, const FwdParams &, hipStream_t);
}  // namespace sru_amd
