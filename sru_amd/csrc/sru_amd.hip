// C ABI of the SRU recurrence library: argument validation, kernel selection, launch.
// Everything before the launch is plain host logic, so bad arguments are rejected
// without touching the GPU.
#include "sru_amd.h"

#include <hip/hip_runtime.h>

#include "sru_launch.h"
#include "sru_reduce.h"

#include <mutex>

namespace {

using namespace sru_amd;

// Scratch of sru_amd_backward_static: the per-column partial sums (4 floats per column) of at most
// SRU_AMD_STATIC_MAX_COLUMNS columns. One copy of the array exists on every device the library runs
// on, at that device's own address, for the life of the process. In host code the array's name is
// only a handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) float scratch[4 * SRU_AMD_STATIC_MAX_COLUMNS];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float *g_scratch_ptr[kMaxDevices] = {};   // device address of `scratch`, per device ordinal

// Address of the current device's copy of `scratch`; resolved once per device, on the first
// call made with that device current. NULL if the runtime cannot tell.
float *static_scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = static_cast<float *>(ptr);
    }
    return g_scratch_ptr[dev];
}

static_assert(SRU_AMD_STATE_INTERVAL == kCkptInterval, "header and kernels disagree");

size_t elem_size(int dtype) { return dtype == SRU_AMD_F64 ? 8 : dtype == SRU_AMD_F32 ? 4 : 2; }
// element size of the small tensors and of the partial sums: float, or double with double streams
size_t small_size(int dtype) { return dtype == SRU_AMD_F64 ? 8 : 4; }

bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// x (and grad_x) is float while the other streams are 16-bit
bool x_is_float_beside_16bit(const sru_amd_shape &s) {
    return (s.dtype == SRU_AMD_F16 || s.dtype == SRU_AMD_BF16) && s.x_dtype == SRU_AMD_X_F32 && s.skip_type == 1;
}

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
    if (s->dtype != SRU_AMD_F32 && s->dtype != SRU_AMD_F16 && s->dtype != SRU_AMD_BF16 && s->dtype != SRU_AMD_F64)
        return SRU_AMD_ERR_BAD_DTYPE;
    if (s->state_interval != 0 && s->state_interval != 1 && s->state_interval != SRU_AMD_STATE_INTERVAL)
        return SRU_AMD_ERR_BAD_FLAGS;
    // checkpointed state exists only for the chunked kernels: not for four streams without a skip
    // term, not for a per-step weight_c together with tanh, and 16-bit streams need an even d
    // (their chunked kernels move two columns at a time); double streams run the general kernels
    if (s->state_interval == SRU_AMD_STATE_INTERVAL) {
        if (s->dtype == SRU_AMD_F64) return SRU_AMD_ERR_BAD_FLAGS;
        if (s->skip_type == 0 && s->k == 4) return SRU_AMD_ERR_BAD_FLAGS;
        if (s->is_custom != 0 && s->activation_type != 0) return SRU_AMD_ERR_BAD_FLAGS;
        if (elem_size(s->dtype) == 2 && s->hidden % 2 != 0) return SRU_AMD_ERR_BAD_FLAGS;
    }
    if (s->x_dtype != SRU_AMD_X_AS_STREAMS && s->x_dtype != SRU_AMD_X_F32) return SRU_AMD_ERR_BAD_DTYPE;
    // a float x next to 16-bit streams exists in the chunked kernels for the plain layer only
    // (and for the state as checkpoints or not at all, which the entry points check)
    if (x_is_float_beside_16bit(*s) && (s->is_custom != 0 || s->activation_type != 0 || s->hidden % 2 != 0))
        return SRU_AMD_ERR_BAD_FLAGS;
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

// Everything sru_amd_backward and sru_amd_backward_static share: pointer checks, then the
// scan and the batch reduction enqueued on `stream`, with the per-column partial sums in
// `partial` (4 * B * D' floats of device memory).
int backward_core(const sru_amd_shape *shape, const void *u, const void *x, const void *weight_c,
                  const void *bias, const void *c_init, const void *mask_c, const uint8_t *mask_pad,
                  const void *scale_x, const void *c, const void *grad_h, const void *grad_last,
                  void *grad_u, void *grad_x, void *grad_wc, void *grad_bias, void *grad_init,
                  void *partial, void *stream) {
    const sru_amd_shape &s = *shape;
    if (!u || !weight_c || !bias || !c || !grad_h || !grad_u || !grad_wc || !grad_bias || !grad_init)
        return SRU_AMD_ERR_NULL_POINTER;
    if (s.skip_type == 1 && (!x || !grad_x)) return SRU_AMD_ERR_NULL_POINTER;
    const size_t es = elem_size(s.dtype), ss = small_size(s.dtype);
    const size_t group = (s.k == 4) ? (es == 8 ? 16 : 4 * es) : es;
    const bool ckpt = s.state_interval == SRU_AMD_STATE_INTERVAL;
    const bool x_float = x_is_float_beside_16bit(s);
    if (x_float && !ckpt) return SRU_AMD_ERR_BAD_FLAGS;
    const size_t xs = x_float ? 4 : es;
    if (!aligned(u, group) || !aligned(grad_u, group) || !aligned(c, ckpt ? 4 : es) || !aligned(grad_h, es) ||
        (s.skip_type == 1 && (!aligned(x, xs) || !aligned(grad_x, xs))) ||
        !aligned(weight_c, s.is_custom ? 2 * es : ss) || !aligned(grad_wc, s.is_custom ? 2 * es : ss) ||
        !aligned(bias, ss) || (c_init && !aligned(c_init, ss)) || (grad_last && !aligned(grad_last, ss)) || !aligned(grad_bias, ss) ||
        !aligned(grad_init, ss) || (mask_c && !aligned(mask_c, ss)) || (scale_x && !aligned(scale_x, ss)))
        return SRU_AMD_ERR_MISALIGNED;

    if (ckpt && es == 2 &&
        (!aligned(u, s.k == 4 ? 16 : 4) || !aligned(grad_u, s.k == 4 ? 16 : 4) ||
         (s.is_custom && (!aligned(weight_c, 8) || !aligned(grad_wc, 8))) || !aligned(grad_h, 4) ||
         (s.skip_type == 1 && (!aligned(x, 4) || !aligned(grad_x, 4)))))
        return SRU_AMD_ERR_MISALIGNED;

    // (the parameter block types the small tensors as float; the double kernels know better)
    auto small = [](const void *q) { return static_cast<const float *>(q); };
    BwdParams p{};
    p.u = u; p.x = x; p.wc = weight_c; p.bias = small(bias); p.c0 = small(c_init); p.mask_c = small(mask_c);
    p.pad = mask_pad; p.scale_x = small(scale_x); p.gh = grad_h; p.glast = small(grad_last);
    p.c = ckpt ? nullptr : c;
    p.ckpt = ckpt ? static_cast<const float *>(c) : nullptr;
    p.gu = grad_u; p.gx = grad_x; p.gwc_steps = s.is_custom ? grad_wc : nullptr;
    p.ginit = static_cast<float *>(grad_init); p.partial = static_cast<float *>(partial);
    p.L = s.length; p.B = s.batch; p.d = (int32_t)s.hidden; p.Dp = (int32_t)(s.hidden * s.dirs);
    p.ncols = s.batch * p.Dp; p.act = s.activation_type; p.custom = s.is_custom; p.x_float = x_float;

    hipStream_t st = static_cast<hipStream_t>(stream);
    const hipError_t err = s.dtype == SRU_AMD_F32    ? launch_backward<float>(s, p, st)
                           : s.dtype == SRU_AMD_F16  ? launch_backward<half_bits>(s, p, st)
                           : s.dtype == SRU_AMD_BF16 ? launch_backward<bf16_bits>(s, p, st)
                                                     : launch_backward<double>(s, p, st);
    if (err != hipSuccess) return SRU_AMD_ERR_LAUNCH;
    const hipError_t red =
        s.dtype == SRU_AMD_F64
            ? launch_reduce(static_cast<const double *>(partial), s.is_custom ? nullptr : static_cast<double *>(grad_wc),
                            static_cast<double *>(grad_bias), p.B, p.Dp, st)
            : launch_reduce(static_cast<const float *>(partial), s.is_custom ? nullptr : static_cast<float *>(grad_wc),
                            static_cast<float *>(grad_bias), p.B, p.Dp, st);
    return red == hipSuccess ? SRU_AMD_OK : SRU_AMD_ERR_LAUNCH;
}

}  // namespace

extern "C" {

int sru_amd_abi_version(void) { return SRU_AMD_ABI_VERSION; }

const char *sru_amd_status_string(int status) {
    switch (status) {
    case SRU_AMD_OK: return "ok";
    case SRU_AMD_ERR_NULL_POINTER: return "a required pointer is NULL";
    case SRU_AMD_ERR_BAD_SHAPE: return "length, batch or hidden is not positive, or the problem is too large";
    case SRU_AMD_ERR_BAD_FLAGS:
        return "inconsistent dirs / k / activation_type / skip_type / is_custom, or checkpointed state asked for a combination it does not exist for";
    case SRU_AMD_ERR_BAD_DTYPE: return "unknown dtype";
    case SRU_AMD_ERR_MISALIGNED: return "a pointer is not aligned as the header's alignment rules ask";
    case SRU_AMD_ERR_WORKSPACE: return "workspace is NULL, misaligned or too small";
    case SRU_AMD_ERR_LAUNCH: return "the HIP runtime refused the kernel launch";
    case SRU_AMD_ERR_STATIC_LIMIT:
        return "more than SRU_AMD_STATIC_MAX_COLUMNS (262144; half as many for double streams) columns: use sru_amd_backward with a workspace";
    default: return "unknown status";
    }
}

int sru_amd_forward(const sru_amd_shape *shape, const void *u, const void *x, const void *weight_c,
                    const void *bias, const void *c_init, const void *mask_c,
                    const uint8_t *mask_pad, const void *scale_x, void *h, void *c, void *c_last,
                    void *stream) {
    if (const int rc = check_shape(shape)) return rc;
    const sru_amd_shape &s = *shape;
    if (!u || !weight_c || !bias || !h || !c_last) return SRU_AMD_ERR_NULL_POINTER;
    if (s.skip_type == 1 && !x) return SRU_AMD_ERR_NULL_POINTER;
    const size_t es = elem_size(s.dtype), ss = small_size(s.dtype);
    const size_t group = (s.k == 4) ? (es == 8 ? 16 : 4 * es) : es;  // a k=4 group moves as one vector (doubles: as two)
    const bool ckpt = s.state_interval == SRU_AMD_STATE_INTERVAL;
    const bool x_float = x_is_float_beside_16bit(s);
    if (x_float && c && !ckpt) return SRU_AMD_ERR_BAD_FLAGS;
    // (a float x still travels with 16-bit streams that move two columns at a time)
    if (x_float && (!aligned(u, s.k == 4 ? 16 : 4) || !aligned(h, 4))) return SRU_AMD_ERR_MISALIGNED;
    if (!aligned(u, group) || !aligned(h, es) || (c && !aligned(c, ckpt ? 4 : es)) ||
        (s.skip_type == 1 && !aligned(x, x_float ? 4 : es)) || !aligned(weight_c, s.is_custom ? 2 * es : ss) ||
        !aligned(bias, ss) || (c_init && !aligned(c_init, ss)) || !aligned(c_last, ss) ||
        (mask_c && !aligned(mask_c, ss)) || (scale_x && !aligned(scale_x, ss)))
        return SRU_AMD_ERR_MISALIGNED;

    // 16-bit streams with checkpoints move two columns at a time
    if (ckpt && es == 2 &&
        (!aligned(u, s.k == 4 ? 16 : 4) || (s.is_custom && !aligned(weight_c, 8)) || !aligned(h, 4) ||
         (s.skip_type == 1 && !aligned(x, 4))))
        return SRU_AMD_ERR_MISALIGNED;

    // (the parameter block types the small tensors as float; the double kernels know better)
    auto small = [](const void *q) { return static_cast<const float *>(q); };
    FwdParams p{};
    p.u = u; p.x = x; p.wc = weight_c; p.bias = small(bias); p.c0 = small(c_init); p.mask_c = small(mask_c);
    p.pad = mask_pad; p.scale_x = small(scale_x); p.h = h; p.c_last = static_cast<float *>(c_last);
    p.c = ckpt ? nullptr : c;
    p.ckpt = ckpt ? static_cast<float *>(c) : nullptr;
    p.L = s.length; p.B = s.batch; p.d = (int32_t)s.hidden; p.Dp = (int32_t)(s.hidden * s.dirs);
    p.ncols = s.batch * p.Dp; p.act = s.activation_type; p.custom = s.is_custom; p.x_float = x_float;

    hipStream_t st = static_cast<hipStream_t>(stream);
    const hipError_t err = s.dtype == SRU_AMD_F32    ? launch_forward<float>(s, p, st)
                           : s.dtype == SRU_AMD_F16  ? launch_forward<half_bits>(s, p, st)
                           : s.dtype == SRU_AMD_BF16 ? launch_forward<bf16_bits>(s, p, st)
                                                     : launch_forward<double>(s, p, st);
    return err == hipSuccess ? SRU_AMD_OK : SRU_AMD_ERR_LAUNCH;
}

size_t sru_amd_state_bytes(const sru_amd_shape *shape) {
    if (check_shape(shape) != SRU_AMD_OK) return 0;
    const size_t ncols = (size_t)(shape->batch * shape->hidden * shape->dirs);
    if (shape->state_interval == SRU_AMD_STATE_INTERVAL) {
        const size_t rows = (size_t)(shape->length / SRU_AMD_STATE_INTERVAL);
        return (rows ? rows : 1) * ncols * sizeof(float);
    }
    return (size_t)shape->length * ncols * elem_size(shape->dtype);
}

size_t sru_amd_backward_workspace_bytes(const sru_amd_shape *shape) {
    if (check_shape(shape) != SRU_AMD_OK) return 0;
    return (size_t)4 * small_size(shape->dtype) * (size_t)(shape->batch * shape->hidden * shape->dirs);
}

int sru_amd_backward(const sru_amd_shape *shape, const void *u, const void *x, const void *weight_c,
                     const void *bias, const void *c_init, const void *mask_c,
                     const uint8_t *mask_pad, const void *scale_x, const void *c,
                     const void *grad_h, const void *grad_last, void *grad_u, void *grad_x,
                     void *grad_wc, void *grad_bias, void *grad_init, void *workspace,
                     size_t workspace_bytes, void *stream) {
    if (const int rc = check_shape(shape)) return rc;
    if (!workspace || !aligned(workspace, 16) ||
        workspace_bytes < sru_amd_backward_workspace_bytes(shape))
        return SRU_AMD_ERR_WORKSPACE;
    return backward_core(shape, u, x, weight_c, bias, c_init, mask_c, mask_pad, scale_x, c, grad_h, grad_last,
                         grad_u, grad_x, grad_wc, grad_bias, grad_init, workspace, stream);
}

int sru_amd_backward_static(const sru_amd_shape *shape, const void *u, const void *x, const void *weight_c,
                            const void *bias, const void *c_init, const void *mask_c,
                            const uint8_t *mask_pad, const void *scale_x, const void *c,
                            const void *grad_h, const void *grad_last, void *grad_u, void *grad_x,
                            void *grad_wc, void *grad_bias, void *grad_init, void *stream) {
    if (const int rc = check_shape(shape)) return rc;
    // the array holds 4 floats for SRU_AMD_STATIC_MAX_COLUMNS columns; double partial sums fill it with half as many
    if (sru_amd_backward_workspace_bytes(shape) > sizeof(float) * 4 * SRU_AMD_STATIC_MAX_COLUMNS) return SRU_AMD_ERR_STATIC_LIMIT;
    float *partial = static_scratch_of_current_device();
    if (!partial) return SRU_AMD_ERR_LAUNCH;
    return backward_core(shape, u, x, weight_c, bias, c_init, mask_c, mask_pad, scale_x, c, grad_h, grad_last,
                         grad_u, grad_x, grad_wc, grad_bias, grad_init, partial, stream);
}

}  // extern "C"
