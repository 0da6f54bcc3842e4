// Batch reduction of the backward scan's per-column partial sums (one definition: included
// by the translation unit that launches it).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sru_amd {

// ================================================================= batch reduction
// partial (4, B, D') -> grad_wc (2, D'), grad_bias (2, D'). One workgroup per 64 hidden
// indices and per quantity; its 16 wavefronts take every 16th batch row each (loads of
// a wavefront are 256 contiguous bytes), accumulate in double and are combined through
// LDS in a fixed order, so the result does not depend on scheduling.
// A: float, or double for double streams (partial sums and results in one type).
constexpr int kReduceSlices = 16;

template <typename A>
__global__ void __launch_bounds__(64 * kReduceSlices)
reduce_partials(const A *partial, A *grad_wc, A *grad_bias, int64_t B, int32_t Dp) {
    __shared__ double acc[kReduceSlices][64];
    const int lane = threadIdx.x & 63;
    const int slice = threadIdx.x >> 6;
    const int j = blockIdx.x * 64 + lane;
    const int q = blockIdx.y;  // 0 gwc1, 1 gwc2, 2 gbias1, 3 gbias2
    double sum = 0.0;
    if (j < Dp) {
        const A *src = partial + ((int64_t)q * B) * Dp + j;
        int64_t b = slice;
        for (; b + 3 * kReduceSlices < B; b += 4 * kReduceSlices) {  // 4 loads in flight
            const A v0 = src[b * Dp], v1 = src[(b + kReduceSlices) * Dp];
            const A v2 = src[(b + 2 * kReduceSlices) * Dp], v3 = src[(b + 3 * kReduceSlices) * Dp];
            sum += (double)v0;
            sum += (double)v1;
            sum += (double)v2;
            sum += (double)v3;
        }
        for (; b < B; b += kReduceSlices) sum += (double)src[b * Dp];
    }
    acc[slice][lane] = sum;
    __syncthreads();
    if (slice == 0 && j < Dp) {
        double total = acc[0][lane];
#pragma unroll
        for (int s = 1; s < kReduceSlices; ++s) total += acc[s][lane];
        A *dst = (q < 2) ? grad_wc : grad_bias;
        if (dst) dst[(q & 1) * Dp + j] = (A)total;
    }
}

template <typename A>
inline hipError_t launch_reduce(const A *partial, A *grad_wc, A *grad_bias, int64_t B, int32_t Dp,
                                hipStream_t st) {
    void *args[] = {&partial, &grad_wc, &grad_bias, &B, &Dp};
    return hipLaunchKernel(reinterpret_cast<const void *>(reduce_partials<A>), dim3((unsigned)((Dp + 63) / 64), 4),
                           dim3(64 * kReduceSlices), args, 0, st);
}

}  // namespace sru_amd
