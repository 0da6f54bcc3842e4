// Layer normalisation next to the recurrence: the reference normalises a layer's input before the
// projection (sru/modules.py:250-253) or its output after the recurrence (:278-279) with
// torch.nn.LayerNorm over the feature dimension (created at :155-162, eps 1e-5, affine).
// These kernels read the tensor once in the dtype it has and write the normalised rows in the dtype
// the consumer wants (the 16-bit operand of the projection under autocast), which replaces the
// chain "cast to float, normalise, cast to 16 bits" that autocast builds around torch's kernel.
//
// Mapping: one wavefront per row (a row = the D features of one (t, b) position); a lane holds
// 8 consecutive features per pass of 512, so rows of float move as two 16-byte vectors per lane
// and pass, 16-bit rows as one. Statistics are float: mean first, then the variance of the
// centred values (both wavefront reductions). The backward kernel walks rows with a stride of the
// grid's wavefront count, keeps its share of the weight / bias gradient sums in registers,
// combines the block's wavefronts through LDS in a fixed order and leaves one partial row per
// block; reduce_rows() then adds the blocks in index order, in double: bit-reproducible.
#include "sru_amd.h"

#include <hip/hip_runtime.h>

#include "sru_scan.h"

namespace {

using namespace sru_amd;

constexpr int kLanes = 64;
constexpr int kPer = 8;                       // features per lane and pass
constexpr int kPass = kLanes * kPer;          // features per pass of a wavefront
constexpr int kNormWaves = 4;                 // wavefronts (rows in flight) per workgroup

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ void load8(const T *p, float (&v)[kPer]);
template <> __device__ __forceinline__ void load8<float>(const float *p, float (&v)[kPer]) {
    const f32x4 a = *reinterpret_cast<const f32x4 *>(p), b = *reinterpret_cast<const f32x4 *>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
}
template <typename T> __device__ __forceinline__ void load8(const T *p, float (&v)[kPer]) {
    const u32x4 a = *reinterpret_cast<const u32x4 *>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = bits_to_float<T>(a[i] & 0xffffu);
        v[2 * i + 1] = bits_to_float<T>(a[i] >> 16);
    }
}
template <typename T> __device__ __forceinline__ void store8(T *p, const float (&v)[kPer]);
template <> __device__ __forceinline__ void store8<float>(float *p, const float (&v)[kPer]) {
    f32x4 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) { a[i] = v[i]; b[i] = v[4 + i]; }
    *reinterpret_cast<f32x4 *>(p) = a;
    *reinterpret_cast<f32x4 *>(p + 4) = b;
}
template <typename T> __device__ __forceinline__ void store8(T *p, const float (&v)[kPer]) {
    u32x4 a;
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = pack_pair<T>(v[2 * i], v[2 * i + 1]);
    *reinterpret_cast<u32x4 *>(p) = a;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kLanes);
    return v;
}

// y = (x - mean) * rstd * gamma + beta per row; mean and rstd (float, one per row) are kept for
// the backward pass. MAXP: passes of 512 features a lane can hold (D <= 512 * MAXP).
template <typename TI, typename TO, int MAXP>
__global__ void __launch_bounds__(kLanes * kNormWaves)
layer_norm_forward(const TI *x, const float *gamma, const float *beta, TO *y, float *mean, float *rstd,
                   int64_t rows, int32_t D, float eps) {
    const int lane = threadIdx.x & (kLanes - 1);
    const int64_t first = (int64_t)blockIdx.x * kNormWaves + (threadIdx.x >> 6);
    const int64_t stride = (int64_t)gridDim.x * kNormWaves;
    float g[MAXP][kPer], b[MAXP][kPer];
#pragma unroll
    for (int p = 0; p < MAXP; ++p) {
        const int e = p * kPass + lane * kPer;
        if (e < D) {
            load8<float>(gamma + e, g[p]);
            load8<float>(beta + e, b[p]);
        }
    }
    const float inv_d = 1.0f / (float)D;
    for (int64_t row = first; row < rows; row += stride) {
        float v[MAXP][kPer];
        float s = 0.f;
#pragma unroll
        for (int p = 0; p < MAXP; ++p) {
            const int e = p * kPass + lane * kPer;
            if (e < D) {
                load8<TI>(x + row * D + e, v[p]);
#pragma unroll
                for (int i = 0; i < kPer; ++i) s += v[p][i];
            }
        }
        const float mu = wave_sum(s) * inv_d;
        float q = 0.f;
#pragma unroll
        for (int p = 0; p < MAXP; ++p) {
            if (p * kPass + lane * kPer < D) {
#pragma unroll
                for (int i = 0; i < kPer; ++i) {
                    v[p][i] -= mu;
                    q += v[p][i] * v[p][i];
                }
            }
        }
        const float rs = 1.0f / sqrtf(wave_sum(q) * inv_d + eps);
#pragma unroll
        for (int p = 0; p < MAXP; ++p) {
            const int e = p * kPass + lane * kPer;
            if (e < D) {
                float o[kPer];
#pragma unroll
                for (int i = 0; i < kPer; ++i) o[i] = v[p][i] * rs * g[p][i] + b[p][i];
                store8<TO>(y + row * D + e, o);
            }
        }
        if (lane == 0) {
            mean[row] = mu;
            rstd[row] = rs;
        }
    }
}

// dx = rstd * (g - mean(g) - xhat * mean(g * xhat)) with g = dy * gamma, xhat = (x - mean) * rstd;
// partial[block] = (sum over the block's rows of dy * xhat, sum of dy), each D floats.
template <typename TI, typename TG, typename TD, int MAXP>
__global__ void __launch_bounds__(kLanes * kNormWaves)
layer_norm_backward(const TI *x, const float *gamma, const float *mean, const float *rstd, const TG *dy, TD *dx,
                    float *partial, int64_t rows, int32_t D) {
    extern __shared__ float acc[];   // (2, D): the block's sums
    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t first = (int64_t)blockIdx.x * kNormWaves + wave;
    const int64_t stride = (int64_t)gridDim.x * kNormWaves;
    float g[MAXP][kPer], dg[MAXP][kPer], db[MAXP][kPer];
#pragma unroll
    for (int p = 0; p < MAXP; ++p) {
        const int e = p * kPass + lane * kPer;
        if (e < D) load8<float>(gamma + e, g[p]);
#pragma unroll
        for (int i = 0; i < kPer; ++i) dg[p][i] = db[p][i] = 0.f;
    }
    const float inv_d = 1.0f / (float)D;
    for (int64_t row = first; row < rows; row += stride) {
        const float mu = mean[row], rs = rstd[row];
        float xh[MAXP][kPer], gy[MAXP][kPer];
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int p = 0; p < MAXP; ++p) {
            const int e = p * kPass + lane * kPer;
            if (e < D) {
                float d[kPer];
                load8<TI>(x + row * D + e, xh[p]);
                load8<TG>(dy + row * D + e, d);
#pragma unroll
                for (int i = 0; i < kPer; ++i) {
                    xh[p][i] = (xh[p][i] - mu) * rs;
                    gy[p][i] = d[i] * g[p][i];
                    s1 += gy[p][i];
                    s2 += gy[p][i] * xh[p][i];
                    dg[p][i] += d[i] * xh[p][i];
                    db[p][i] += d[i];
                }
            }
        }
        const float c1 = wave_sum(s1) * inv_d, c2 = wave_sum(s2) * inv_d;
#pragma unroll
        for (int p = 0; p < MAXP; ++p) {
            const int e = p * kPass + lane * kPer;
            if (e < D) {
                float o[kPer];
#pragma unroll
                for (int i = 0; i < kPer; ++i) o[i] = rs * (gy[p][i] - c1 - xh[p][i] * c2);
                store8<TD>(dx + row * D + e, o);
            }
        }
    }
    // the block's wavefronts add their sums one after the other: a fixed order
    for (int w = 0; w < kNormWaves; ++w) {
        if (wave == w) {
#pragma unroll
            for (int p = 0; p < MAXP; ++p) {
                const int e = p * kPass + lane * kPer;
                if (e < D) {
#pragma unroll
                    for (int i = 0; i < kPer; ++i) {
                        acc[e + i] = (w == 0 ? 0.f : acc[e + i]) + dg[p][i];
                        acc[D + e + i] = (w == 0 ? 0.f : acc[D + e + i]) + db[p][i];
                    }
                }
            }
        }
        __syncthreads();
    }
    float *out = partial + (int64_t)blockIdx.x * 2 * D;
    for (int e = threadIdx.x; e < 2 * D; e += blockDim.x) out[e] = acc[e];
}

// out[e] = sum over r of partial[r][e]. One workgroup per 64 columns; its 16 wavefronts take every
// 16th row each, accumulate in double and are combined through LDS in a fixed order.
constexpr int kRowSlices = 16;
__global__ void __launch_bounds__(kLanes * kRowSlices)
reduce_rows(const float *partial, float *out, int32_t nrows, int32_t width) {
    __shared__ double part[kRowSlices][kLanes];
    const int lane = threadIdx.x & (kLanes - 1), slice = threadIdx.x >> 6;
    const int e = blockIdx.x * kLanes + lane;
    double s = 0.0;
    if (e < width)
        for (int r = slice; r < nrows; r += kRowSlices) s += (double)partial[(int64_t)r * width + e];
    part[slice][lane] = s;
    __syncthreads();
    if (slice == 0 && e < width) {
        double total = part[0][lane];
#pragma unroll
        for (int i = 1; i < kRowSlices; ++i) total += part[i][lane];
        out[e] = (float)total;
    }
}

int norm_blocks(int64_t rows) {
    const int64_t want = (rows + kNormWaves - 1) / kNormWaves;
    return (int)(want < 1024 ? want : 1024);   // 4096 wavefronts at most: 4 per SIMD
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) % 16) == 0; }

int check_norm(int64_t rows, int64_t cols, int dt_a, int dt_b) {
    if (rows < 1 || cols < 1 || cols % kPer != 0 || cols > SRU_AMD_NORM_MAX_FEATURES || rows > (INT64_C(1) << 40))
        return SRU_AMD_ERR_BAD_SHAPE;
    for (int dt : {dt_a, dt_b})
        if (dt != SRU_AMD_F32 && dt != SRU_AMD_F16 && dt != SRU_AMD_BF16) return SRU_AMD_ERR_BAD_DTYPE;
    return SRU_AMD_OK;
}

template <typename TI, typename TO>
hipError_t launch_norm_forward(const void *x, const float *gamma, const float *beta, void *y, float *mean,
                               float *rstd, int64_t rows, int32_t D, float eps, hipStream_t st) {
    const TI *xi = static_cast<const TI *>(x);
    TO *yo = static_cast<TO *>(y);
    void *args[] = {&xi, &gamma, &beta, &yo, &mean, &rstd, &rows, &D, &eps};
    const dim3 grid(norm_blocks(rows)), block(kLanes * kNormWaves);
    const int passes = (D + kPass - 1) / kPass;
    const void *k = passes <= 1   ? reinterpret_cast<const void *>(layer_norm_forward<TI, TO, 1>)
                    : passes <= 2 ? reinterpret_cast<const void *>(layer_norm_forward<TI, TO, 2>)
                    : passes <= 4 ? reinterpret_cast<const void *>(layer_norm_forward<TI, TO, 4>)
                                  : reinterpret_cast<const void *>(layer_norm_forward<TI, TO, 8>);
    return hipLaunchKernel(k, grid, block, args, 0, st);
}

template <typename TI, typename TG, typename TD>
hipError_t launch_norm_backward(const void *x, const float *gamma, const float *mean, const float *rstd,
                                const void *dy, void *dx, float *partial, int64_t rows, int32_t D, hipStream_t st) {
    const TI *xi = static_cast<const TI *>(x);
    const TG *gi = static_cast<const TG *>(dy);
    TD *di = static_cast<TD *>(dx);
    void *args[] = {&xi, &gamma, &mean, &rstd, &gi, &di, &partial, &rows, &D};
    const dim3 grid(norm_blocks(rows)), block(kLanes * kNormWaves);
    const size_t lds = (size_t)2 * D * sizeof(float);
    const int passes = (D + kPass - 1) / kPass;
    const void *k = passes <= 1   ? reinterpret_cast<const void *>(layer_norm_backward<TI, TG, TD, 1>)
                    : passes <= 2 ? reinterpret_cast<const void *>(layer_norm_backward<TI, TG, TD, 2>)
                    : passes <= 4 ? reinterpret_cast<const void *>(layer_norm_backward<TI, TG, TD, 4>)
                                  : reinterpret_cast<const void *>(layer_norm_backward<TI, TG, TD, 8>);
    return hipLaunchKernel(k, grid, block, args, lds, st);
}

// run F<A, B>(...) for the two runtime dtypes
template <typename A>
hipError_t forward_by_out(int dt_y, const void *x, const float *gamma, const float *beta, void *y, float *mean,
                          float *rstd, int64_t rows, int32_t D, float eps, hipStream_t st) {
    if (dt_y == SRU_AMD_F32) return launch_norm_forward<A, float>(x, gamma, beta, y, mean, rstd, rows, D, eps, st);
    if (dt_y == SRU_AMD_F16) return launch_norm_forward<A, half_bits>(x, gamma, beta, y, mean, rstd, rows, D, eps, st);
    return launch_norm_forward<A, bf16_bits>(x, gamma, beta, y, mean, rstd, rows, D, eps, st);
}

// the gradient of x has x's dtype
template <typename A>
hipError_t backward_by_grad(int dt_y, const void *x, const float *gamma, const float *mean, const float *rstd,
                            const void *dy, void *dx, float *partial, int64_t rows, int32_t D, hipStream_t st) {
    if (dt_y == SRU_AMD_F32) return launch_norm_backward<A, float, A>(x, gamma, mean, rstd, dy, dx, partial, rows, D, st);
    if (dt_y == SRU_AMD_F16) return launch_norm_backward<A, half_bits, A>(x, gamma, mean, rstd, dy, dx, partial, rows, D, st);
    return launch_norm_backward<A, bf16_bits, A>(x, gamma, mean, rstd, dy, dx, partial, rows, D, st);
}

}  // namespace

extern "C" {

int sru_amd_layer_norm_forward(int64_t rows, int64_t cols, const void *x, int x_dtype, const float *weight,
                               const float *bias, float eps, void *y, int y_dtype, float *mean, float *rstd,
                               void *stream) {
    if (const int rc = check_norm(rows, cols, x_dtype, y_dtype)) return rc;
    if (!x || !weight || !bias || !y || !mean || !rstd) return SRU_AMD_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(y) || !aligned16(weight) || !aligned16(bias)) return SRU_AMD_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t D = (int32_t)cols;
    const hipError_t err =
        x_dtype == SRU_AMD_F32   ? forward_by_out<float>(y_dtype, x, weight, bias, y, mean, rstd, rows, D, eps, st)
        : x_dtype == SRU_AMD_F16 ? forward_by_out<half_bits>(y_dtype, x, weight, bias, y, mean, rstd, rows, D, eps, st)
                                 : forward_by_out<bf16_bits>(y_dtype, x, weight, bias, y, mean, rstd, rows, D, eps, st);
    return err == hipSuccess ? SRU_AMD_OK : SRU_AMD_ERR_LAUNCH;
}

size_t sru_amd_layer_norm_backward_workspace_bytes(int64_t rows, int64_t cols) {
    if (check_norm(rows, cols, SRU_AMD_F32, SRU_AMD_F32) != SRU_AMD_OK) return 0;
    return (size_t)norm_blocks(rows) * 2 * (size_t)cols * sizeof(float);
}

int sru_amd_layer_norm_backward(int64_t rows, int64_t cols, const void *x, int x_dtype, const float *weight,
                                const float *mean, const float *rstd, const void *grad_y, int y_dtype,
                                void *grad_x, float *grad_weight, float *grad_bias, void *workspace,
                                size_t workspace_bytes, void *stream) {
    if (const int rc = check_norm(rows, cols, x_dtype, y_dtype)) return rc;
    if (!x || !weight || !mean || !rstd || !grad_y || !grad_x || !grad_weight || !grad_bias)
        return SRU_AMD_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(grad_y) || !aligned16(grad_x) || !aligned16(weight)) return SRU_AMD_ERR_MISALIGNED;
    if (!workspace || !aligned16(workspace) || workspace_bytes < sru_amd_layer_norm_backward_workspace_bytes(rows, cols))
        return SRU_AMD_ERR_WORKSPACE;
    // the two sums must be contiguous for the single reduction launch: (grad_weight, grad_bias) = out[0:D], out[D:2D]
    if (grad_bias != grad_weight + cols) return SRU_AMD_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t D = (int32_t)cols;
    float *partial = static_cast<float *>(workspace);
    const hipError_t err =
        x_dtype == SRU_AMD_F32   ? backward_by_grad<float>(y_dtype, x, weight, mean, rstd, grad_y, grad_x, partial, rows, D, st)
        : x_dtype == SRU_AMD_F16 ? backward_by_grad<half_bits>(y_dtype, x, weight, mean, rstd, grad_y, grad_x, partial, rows, D, st)
                                 : backward_by_grad<bf16_bits>(y_dtype, x, weight, mean, rstd, grad_y, grad_x, partial, rows, D, st);
    if (err != hipSuccess) return SRU_AMD_ERR_LAUNCH;
    int32_t nrows = norm_blocks(rows), width = 2 * D;
    const float *src = partial;
    void *args[] = {&src, &grad_weight, &nrows, &width};
    return hipLaunchKernel(reinterpret_cast<const void *>(reduce_rows), dim3((width + kLanes - 1) / kLanes),
                           dim3(kLanes * kRowSlices), args, 0, st) == hipSuccess ? SRU_AMD_OK : SRU_AMD_ERR_LAUNCH;
}

}  // extern "C"
