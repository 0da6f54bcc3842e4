// C ABI of the SRU recurrence library: argument validation, kernel selection, launch.
// Everything before the launch is plain host logic, so bad arguments are rejected
// without touching the GPU.
#include "sru_amd.h"

#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "sru_scan.h"

namespace {

using namespace sru_amd;

size_t elem_size(int dtype) { return dtype == SRU_AMD_F32 ? 4 : 2; }

bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Shape and flag rules; those on k / skip_type are the device-side asserts of the
// reference's general kernels (sru/csrc/sru_cuda_kernel.cu:397-399).
int check_shape(const sru_amd_shape *s) {
    if (!s) return SRU_AMD_ERR_NULL_POINTER;
    if (s->length < 1 || s->batch < 1 || s->hidden < 1) return SRU_AMD_ERR_BAD_SHAPE;
    if (s->dirs != 1 && s->dirs != 2) return SRU_AMD_ERR_BAD_FLAGS;
    if (s->k != 3 && s->k != 4) return SRU_AMD_ERR_BAD_FLAGS;
    if (s->activation_type != 0 && s->activation_type != 1) return SRU_AMD_ERR_BAD_FLAGS;
    if (s->skip_type < 0 || s->skip_type > 2) return SRU_AMD_ERR_BAD_FLAGS;
    if (s->skip_type == 1 && s->k != 3) return SRU_AMD_ERR_BAD_FLAGS;
    if (s->skip_type == 2 && s->k != 4) return SRU_AMD_ERR_BAD_FLAGS;
    if (s->is_custom != 0 && s->is_custom != 1) return SRU_AMD_ERR_BAD_FLAGS;
    if (s->dtype != SRU_AMD_F32 && s->dtype != SRU_AMD_F16 && s->dtype != SRU_AMD_BF16)
        return SRU_AMD_ERR_BAD_DTYPE;
    // D' must fit an int, the grid must fit 2^31-1 workgroups and the largest stream
    // (L*B*D'*k elements) must stay far inside the 64-bit byte offsets the kernels use.
    const int64_t lim = INT64_C(1) << 31;
    if (s->hidden >= lim / 2) return SRU_AMD_ERR_BAD_SHAPE;
    const int64_t Dp = s->hidden * s->dirs;
    if (s->batch > (INT64_C(1) << 36) / Dp) return SRU_AMD_ERR_BAD_SHAPE;
    const int64_t ncols = s->batch * Dp;
    if (s->length > (INT64_C(1) << 56) / (ncols * 4)) return SRU_AMD_ERR_BAD_SHAPE;
    return SRU_AMD_OK;
}

int ring_depth(const char *var, int fallback) {
    const char *e = std::getenv(var);
    if (!e) return fallback;
    const int v = std::atoi(e);
    return (v == 4 || v == 8 || v == 12 || v == 16) ? v : fallback;
}

// Fast kernels exist for the two layouts the SRU layer produces with a skip term and no
// tanh / per-step weight_c: (k=3, skip from x) and (k=4, skip from U[..., 3]); whether a
// padding mask is given and whether c is stored are compiled in. Everything else runs
// the general kernels. Only the float (k=3, skip from x) fast kernels are built at more
// than one ring depth.
template <typename T, int K, int SKIP, int MODE>
void launch_forward(const FwdParams &p, dim3 grid, hipStream_t st, int depth) {
    if constexpr (std::is_same<T, float>::value && K == 3 && !(MODE & kGeneral)) {
        switch (depth) {
        case 4: hipLaunchKernelGGL((forward_scan<T, K, SKIP, MODE, 4>), grid, dim3(kBlock), 0, st, p); return;
        case 12: hipLaunchKernelGGL((forward_scan<T, K, SKIP, MODE, 12>), grid, dim3(kBlock), 0, st, p); return;
        case 16: hipLaunchKernelGGL((forward_scan<T, K, SKIP, MODE, 16>), grid, dim3(kBlock), 0, st, p); return;
        default: break;
        }
    }
    hipLaunchKernelGGL((forward_scan<T, K, SKIP, MODE, 8>), grid, dim3(kBlock), 0, st, p);
}

template <typename T, int K, int SKIP, int MODE>
void launch_backward(const BwdParams &p, dim3 grid, hipStream_t st, int depth) {
    if constexpr (std::is_same<T, float>::value && K == 3 && !(MODE & kGeneral)) {
        switch (depth) {
        case 4: hipLaunchKernelGGL((backward_scan<T, K, SKIP, MODE, 4>), grid, dim3(kBlock), 0, st, p); return;
        case 12: hipLaunchKernelGGL((backward_scan<T, K, SKIP, MODE, 12>), grid, dim3(kBlock), 0, st, p); return;
        case 16: hipLaunchKernelGGL((backward_scan<T, K, SKIP, MODE, 16>), grid, dim3(kBlock), 0, st, p); return;
        default: break;
        }
    }
    hipLaunchKernelGGL((backward_scan<T, K, SKIP, MODE, 8>), grid, dim3(kBlock), 0, st, p);
}

template <typename T, int K, int SKIP>
void fast_forward(const FwdParams &p, dim3 grid, hipStream_t st, int depth) {
    const int mode = (p.pad ? kHasPad : 0) | (p.c ? kKeepC : 0);
    switch (mode) {
    case 0: launch_forward<T, K, SKIP, 0>(p, grid, st, depth); break;
    case kHasPad: launch_forward<T, K, SKIP, kHasPad>(p, grid, st, depth); break;
    case kKeepC: launch_forward<T, K, SKIP, kKeepC>(p, grid, st, depth); break;
    default: launch_forward<T, K, SKIP, kHasPad | kKeepC>(p, grid, st, depth); break;
    }
}

template <typename T, int K, int SKIP>
void fast_backward(const BwdParams &p, dim3 grid, hipStream_t st, int depth) {
    if (p.pad) launch_backward<T, K, SKIP, kHasPad>(p, grid, st, depth);
    else launch_backward<T, K, SKIP, 0>(p, grid, st, depth);
}

// (k, skip_type) pairs that pass check_shape: (3,0) (3,1) (4,0) (4,2).
template <typename T>
void dispatch_forward(const sru_amd_shape &s, const FwdParams &p, dim3 grid, hipStream_t st, int depth) {
    const bool general = s.activation_type != 0 || s.is_custom != 0 || s.skip_type == 0;
    if (!general) {
        if (s.k == 3) fast_forward<T, 3, 1>(p, grid, st, depth);
        else fast_forward<T, 4, 2>(p, grid, st, depth);
    } else if (s.k == 3 && s.skip_type == 1) launch_forward<T, 3, 1, kGeneral>(p, grid, st, 8);
    else if (s.k == 3) launch_forward<T, 3, 0, kGeneral>(p, grid, st, 8);
    else if (s.skip_type == 2) launch_forward<T, 4, 2, kGeneral>(p, grid, st, 8);
    else launch_forward<T, 4, 0, kGeneral>(p, grid, st, 8);
}

template <typename T>
void dispatch_backward(const sru_amd_shape &s, const BwdParams &p, dim3 grid, hipStream_t st, int depth) {
    const bool general = s.activation_type != 0 || s.is_custom != 0 || s.skip_type == 0;
    if (!general) {
        if (s.k == 3) fast_backward<T, 3, 1>(p, grid, st, depth);
        else fast_backward<T, 4, 2>(p, grid, st, depth);
    } else if (s.k == 3 && s.skip_type == 1) launch_backward<T, 3, 1, kGeneral>(p, grid, st, 8);
    else if (s.k == 3) launch_backward<T, 3, 0, kGeneral>(p, grid, st, 8);
    else if (s.skip_type == 2) launch_backward<T, 4, 2, kGeneral>(p, grid, st, 8);
    else launch_backward<T, 4, 0, kGeneral>(p, grid, st, 8);
}

}  // namespace

extern "C" {

int sru_amd_abi_version(void) { return SRU_AMD_ABI_VERSION; }

const char *sru_amd_status_string(int status) {
    switch (status) {
    case SRU_AMD_OK: return "ok";
    case SRU_AMD_ERR_NULL_POINTER: return "a required pointer is NULL";
    case SRU_AMD_ERR_BAD_SHAPE: return "length, batch or hidden is not positive, or the problem is too large";
    case SRU_AMD_ERR_BAD_FLAGS: return "inconsistent dirs / k / activation_type / skip_type / is_custom";
    case SRU_AMD_ERR_BAD_DTYPE: return "unknown dtype";
    case SRU_AMD_ERR_MISALIGNED: return "a stream pointer is not aligned to its element group";
    case SRU_AMD_ERR_WORKSPACE: return "workspace is NULL, misaligned or too small";
    case SRU_AMD_ERR_LAUNCH: return "the HIP runtime refused the kernel launch";
    default: return "unknown status";
    }
}

int sru_amd_forward(const sru_amd_shape *shape, const void *u, const void *x, const void *weight_c,
                    const float *bias, const float *c_init, const float *mask_c,
                    const uint8_t *mask_pad, const float *scale_x, void *h, void *c, float *c_last,
                    void *stream) {
    if (const int rc = check_shape(shape)) return rc;
    const sru_amd_shape &s = *shape;
    if (!u || !weight_c || !bias || !c_init || !h || !c_last) return SRU_AMD_ERR_NULL_POINTER;
    if (s.skip_type == 1 && !x) return SRU_AMD_ERR_NULL_POINTER;
    const size_t es = elem_size(s.dtype);
    const size_t group = (s.k == 4) ? 4 * es : es;  // a k=4 group moves as one vector
    if (!aligned(u, group) || !aligned(h, es) || (c && !aligned(c, es)) ||
        (s.skip_type == 1 && !aligned(x, es)) || !aligned(weight_c, s.is_custom ? 2 * es : 4) ||
        !aligned(bias, 4) || !aligned(c_init, 4) || !aligned(c_last, 4) ||
        (mask_c && !aligned(mask_c, 4)) || (scale_x && !aligned(scale_x, 4)))
        return SRU_AMD_ERR_MISALIGNED;

    FwdParams p{};
    p.u = u; p.x = x; p.wc = weight_c; p.bias = bias; p.c0 = c_init; p.mask_c = mask_c;
    p.pad = mask_pad; p.scale_x = scale_x; p.h = h; p.c = c; p.c_last = c_last;
    p.L = s.length; p.B = s.batch; p.d = (int32_t)s.hidden; p.Dp = (int32_t)(s.hidden * s.dirs);
    p.ncols = s.batch * p.Dp; p.act = s.activation_type; p.custom = s.is_custom;

    const dim3 grid((unsigned)((p.ncols + kBlock - 1) / kBlock));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int depth = ring_depth("SRU_AMD_FWD_DEPTH", 8);
    (void)hipGetLastError();
    if (s.dtype == SRU_AMD_F32) dispatch_forward<float>(s, p, grid, st, depth);
    else if (s.dtype == SRU_AMD_F16) dispatch_forward<half_bits>(s, p, grid, st, depth);
    else dispatch_forward<bf16_bits>(s, p, grid, st, depth);
    return hipGetLastError() == hipSuccess ? SRU_AMD_OK : SRU_AMD_ERR_LAUNCH;
}

size_t sru_amd_backward_workspace_bytes(const sru_amd_shape *shape) {
    if (check_shape(shape) != SRU_AMD_OK) return 0;
    return (size_t)4 * sizeof(float) * (size_t)(shape->batch * shape->hidden * shape->dirs);
}

int sru_amd_backward(const sru_amd_shape *shape, const void *u, const void *x, const void *weight_c,
                     const float *bias, const float *c_init, const float *mask_c,
                     const uint8_t *mask_pad, const float *scale_x, const void *c,
                     const void *grad_h, const float *grad_last, void *grad_u, void *grad_x,
                     void *grad_wc, float *grad_bias, float *grad_init, void *workspace,
                     size_t workspace_bytes, void *stream) {
    if (const int rc = check_shape(shape)) return rc;
    const sru_amd_shape &s = *shape;
    if (!u || !weight_c || !bias || !c_init || !c || !grad_h || !grad_last || !grad_u || !grad_wc ||
        !grad_bias || !grad_init)
        return SRU_AMD_ERR_NULL_POINTER;
    if (s.skip_type == 1 && (!x || !grad_x)) return SRU_AMD_ERR_NULL_POINTER;
    const size_t es = elem_size(s.dtype);
    const size_t group = (s.k == 4) ? 4 * es : es;
    if (!aligned(u, group) || !aligned(grad_u, group) || !aligned(c, es) || !aligned(grad_h, es) ||
        (s.skip_type == 1 && (!aligned(x, es) || !aligned(grad_x, es))) ||
        !aligned(weight_c, s.is_custom ? 2 * es : 4) || !aligned(grad_wc, s.is_custom ? 2 * es : 4) ||
        !aligned(bias, 4) || !aligned(c_init, 4) || !aligned(grad_last, 4) || !aligned(grad_bias, 4) ||
        !aligned(grad_init, 4) || (mask_c && !aligned(mask_c, 4)) || (scale_x && !aligned(scale_x, 4)))
        return SRU_AMD_ERR_MISALIGNED;
    if (!workspace || !aligned(workspace, 16) ||
        workspace_bytes < sru_amd_backward_workspace_bytes(shape))
        return SRU_AMD_ERR_WORKSPACE;

    BwdParams p{};
    p.u = u; p.x = x; p.wc = weight_c; p.bias = bias; p.c0 = c_init; p.mask_c = mask_c;
    p.pad = mask_pad; p.scale_x = scale_x; p.c = c; p.gh = grad_h; p.glast = grad_last;
    p.gu = grad_u; p.gx = grad_x; p.gwc_steps = s.is_custom ? grad_wc : nullptr;
    p.ginit = grad_init; p.partial = static_cast<float *>(workspace);
    p.L = s.length; p.B = s.batch; p.d = (int32_t)s.hidden; p.Dp = (int32_t)(s.hidden * s.dirs);
    p.ncols = s.batch * p.Dp; p.act = s.activation_type; p.custom = s.is_custom;

    const dim3 grid((unsigned)((p.ncols + kBlock - 1) / kBlock));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int depth = ring_depth("SRU_AMD_BWD_DEPTH", 8);
    (void)hipGetLastError();
    if (s.dtype == SRU_AMD_F32) dispatch_backward<float>(s, p, grid, st, depth);
    else if (s.dtype == SRU_AMD_F16) dispatch_backward<half_bits>(s, p, grid, st, depth);
    else dispatch_backward<bf16_bits>(s, p, grid, st, depth);
    if (hipGetLastError() != hipSuccess) return SRU_AMD_ERR_LAUNCH;

    const dim3 rgrid((unsigned)((p.Dp + 63) / 64), 4);
    hipLaunchKernelGGL(reduce_partials, rgrid, dim3(64 * kReduceSlices), 0, st, p.partial,
                       s.is_custom ? nullptr : static_cast<float *>(grad_wc), grad_bias, p.B, p.Dp);
    return hipGetLastError() == hipSuccess ? SRU_AMD_OK : SRU_AMD_ERR_LAUNCH;
}

}  // extern "C"
