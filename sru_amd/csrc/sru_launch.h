// Host-side launchers of the scan kernels, one explicit instantiation per stream element
// type (scan_f32.hip, scan_f16.hip, scan_bf16.hip) so the three compile in parallel.
#pragma once

#include <hip/hip_runtime.h>

#include "sru_amd.h"
#include "sru_scan.h"

namespace sru_amd {

template <typename T>
void launch_forward(const sru_amd_shape &s, const FwdParams &p, hipStream_t stream);

template <typename T>
void launch_backward(const sru_amd_shape &s, const BwdParams &p, hipStream_t stream);

}  // namespace sru_amd
