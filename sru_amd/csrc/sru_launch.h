// Host-side launchers of the scan kernels, one explicit instantiation per stream element
// type and pass (scan_f32_fwd.hip, scan_f32_bwd.hip, ... scan_bf16_bwd.hip; scan_f64.hip holds both passes)
// so that they compile in parallel.
#pragma once

#include <hip/hip_runtime.h>

#include "sru_amd.h"
#include "sru_scan.h"

namespace sru_amd {

// Both return the status of the launch itself (hipSuccess = enqueued).
template <typename T>
hipError_t launch_forward(const sru_amd_shape &s, const FwdParams &p, hipStream_t stream);

template <typename T>
hipError_t launch_backward(const sru_amd_shape &s, const BwdParams &p, hipStream_t stream);

}  // namespace sru_amd
