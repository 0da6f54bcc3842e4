/*
 * sru_amd: the SRU elementwise recurrence (forward scan and backward scan over
 * time) as hand-written HIP kernels for gfx950, behind a C ABI.
 *
 * These entry points stand where the reference binds its eight TorchScript
 * operators sru_cuda::sru_[bi_]forward[_simple] and
 * sru_cuda::sru_[bi_]backward[_simple]
 * (sru/csrc/sru_cuda_impl.cpp:177-518, registered at :531-546, called from
 * sru/cuda_functional.py:85-144 and :213-251). One forward and one backward
 * entry cover all eight: direction count, k, activation, skip type and the
 * per-step weight_c variant are fields of sru_amd_shape.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless said otherwise; the library never
 *     allocates, frees or retains memory; the caller owns all buffers;
 *   - every output cell is written, zeros at padded cells included, so outputs
 *     may be uninitialised memory (the reference relies on zero-filled
 *     allocations instead, sru_cuda_impl.cpp:189-190,:225-229);
 *   - kernels are enqueued on `stream` (a hipStream_t; NULL = the null stream)
 *     and the call returns without waiting;
 *   - return value 0 = enqueued, anything else = nothing was launched; no
 *     exception ever crosses this boundary.
 *
 * Layouts (those of the reference)
 *   U        (L, B, D', k)      k innermost; D' = dirs * hidden
 *   x, h, c, grad_h, grad_x     (L, B, D')            (x, grad_x: see shape->x_dtype)
 *   weight_c (2, D') small, or, when is_custom, (L, B, D', 2) in `dtype`
 *   bias     (2, D') small
 *   c_init, mask_c, c_last, grad_last, grad_init   (B, D') small
 *   mask_pad (L, B) one byte per cell, non-zero = padded
 *   scale_x  one small value on the device, or NULL for 1
 * `dtype` is the element type of the large streams U, x, h, c, grad_h, grad_u,
 * grad_x and of a per-step weight_c / its gradient. With SRU_AMD_F32, SRU_AMD_F16 and
 * SRU_AMD_BF16 the recurrence state and all arithmetic are float, and so is every tensor
 * marked "small" below. With SRU_AMD_F64 everything is double: the streams, the small
 * tensors (weight_c, bias, c_init, mask_c, scale_x, c_last, grad_last, grad_wc, grad_bias,
 * grad_init), the state and the arithmetic, as in the reference's double kernels
 * (sru/csrc/sru_cuda_kernel.cu:845, AT_DISPATCH_FLOATING_TYPES_AND_HALF); the backward
 * workspace doubles with it. The small tensors are therefore declared `void *`: float
 * unless `dtype` is SRU_AMD_F64.
 *
 * Alignment (SRU_AMD_ERR_MISALIGNED otherwise)
 *   - small tensors: their element size; U and grad_u with k = 4: four elements (one group; 16 bytes
 *     are enough for double streams);
 *   - every stream: its element size; a per-step weight_c and its gradient: two elements;
 *   - 16-bit streams with state_interval == SRU_AMD_STATE_INTERVAL move two columns at a
 *     time: x, h, grad_h, grad_x 4 bytes; U and grad_u 4 bytes (k = 3) or 16 bytes (k = 4);
 *     a per-step weight_c and its gradient 8 bytes.
 *   Memory from hipMalloc or a torch allocation satisfies all of these; a view that starts at
 *   an odd element may not.
 */
#ifndef SRU_AMD_H
#define SRU_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SRU_AMD_ABI_VERSION 6

enum sru_amd_dtype {
    SRU_AMD_F32 = 0,
    SRU_AMD_F16 = 1,
    SRU_AMD_BF16 = 2,
    SRU_AMD_F64 = 3     /* double streams, small tensors, state and arithmetic; state_interval 0 / 1 only */
};

enum sru_amd_status {
    SRU_AMD_OK = 0,
    SRU_AMD_ERR_NULL_POINTER = 1,   /* a required pointer is NULL */
    SRU_AMD_ERR_BAD_SHAPE = 2,      /* a size is <= 0 or the problem exceeds the index range */
    SRU_AMD_ERR_BAD_FLAGS = 3,      /* dirs, k, activation_type, skip_type, is_custom inconsistent, or a
                                     * combination that checkpointed state does not exist for (see
                                     * state_interval below) */
    SRU_AMD_ERR_BAD_DTYPE = 4,
    SRU_AMD_ERR_MISALIGNED = 5,     /* a pointer is not aligned as "Alignment" below asks */
    SRU_AMD_ERR_WORKSPACE = 6,      /* workspace missing or smaller than required */
    SRU_AMD_ERR_LAUNCH = 7,         /* the HIP runtime refused the launch */
    SRU_AMD_ERR_STATIC_LIMIT = 8    /* sru_amd_backward_static: more columns than its built-in scratch holds */
};

/* Problem description; the fields are the integer arguments of the reference's
 * general operators (sru/csrc/sru_cuda_impl.cpp:333-347: length, batch_size,
 * hidden_size, k, activation_type, skip_type, is_custom) plus the direction
 * count that the reference encodes in the operator name. */
typedef struct sru_amd_shape {
    int64_t length;          /* L >= 1 */
    int64_t batch;           /* B >= 1 */
    int64_t hidden;          /* d >= 1, per direction */
    int32_t dirs;            /* 1, or 2: columns with (col % 2d) >= d walk time backwards */
    int32_t k;               /* 3 or 4 streams per column in U */
    int32_t activation_type; /* 0 identity, 1 tanh */
    int32_t skip_type;       /* 0 none; 1 from x (k == 3); 2 from U[..., 3] (k == 4) */
    int32_t is_custom;       /* 0: weight_c (2, D'); 1: per step (L, B, D', 2) */
    int32_t dtype;           /* enum sru_amd_dtype */
    int32_t state_interval;  /* what `c` holds between forward and backward:
                              * 0 or 1: the state after every step, (L, B, D') in `dtype`, as
                              *   the reference keeps it (sru_cuda_kernel.cu:72,:436);
                              * SRU_AMD_STATE_INTERVAL: float checkpoints only, one row per
                              *   SRU_AMD_STATE_INTERVAL steps of each column's walk,
                              *   (max(1, L / SRU_AMD_STATE_INTERVAL), B, D') float; the backward
                              *   call rebuilds the states in between. Refused (BAD_FLAGS) for
                              *   k = 4 without a skip term, for is_custom together with tanh, for
                              *   16-bit streams with an odd `hidden`, and for double streams. This is the mode the fast
                              *   kernels of every shape are built for; with 0 / 1 the 16-bit
                              *   kernels for few columns and the checkpoint backward kernels are
                              *   not available. No counterpart in the reference. */
    int32_t x_dtype;         /* element type of x and grad_x: SRU_AMD_X_AS_STREAMS (0): `dtype`, like
                              * every other stream; SRU_AMD_X_F32: float, next to 16-bit streams -
                              * under autocast the reference hands the recurrence a float32 x beside
                              * the 16-bit U (sru/ops.py:116-127 casts both to float32; here neither
                              * is cast). Needs skip_type 1 (otherwise x is not read and the field is
                              * ignored), is_custom 0, activation_type 0, an even `hidden`, and the
                              * state as checkpoints or not at all (BAD_FLAGS otherwise). With dtype
                              * SRU_AMD_F32 both values mean the same; with SRU_AMD_F64 the field is
                              * ignored (x is double). */
} sru_amd_shape;

#define SRU_AMD_X_AS_STREAMS 0
#define SRU_AMD_X_F32 1

#define SRU_AMD_STATE_INTERVAL 8

/* Forward scan. Replaces sru_cuda::sru_forward_simple, sru_bi_forward_simple,
 * sru_forward and sru_bi_forward (sru/csrc/sru_cuda_impl.cpp:177-207,:255-285,
 * :333-412) together with the x * scale_x pass and the gather of the last state
 * that sru/cuda_functional.py:73-78 and :146-153 run around them.
 *   x        required iff skip_type == 1
 *   c_init   NULL = zeros (what the reference allocates when the caller gives no c0,
 *            sru/modules.py:241-243)
 *   mask_c   NULL = no dropout mask
 *   mask_pad NULL = no padding
 *   c        state kept for the backward pass, sru_amd_state_bytes() bytes laid out as
 *            shape->state_interval says; NULL = do not store it (inference)
 *   c_last   state after the last step of each column's walk: what the
 *            reference assembles as cat(c[-1, :, :d], c[0, :, d:]) */
int sru_amd_forward(const sru_amd_shape *shape,
                    const void *u, const void *x, const void *weight_c,
                    const void *bias, const void *c_init, const void *mask_c,
                    const uint8_t *mask_pad, const void *scale_x,
                    void *h, void *c, void *c_last, void *stream);

/* Bytes of the state buffer `c` that sru_amd_forward fills and sru_amd_backward reads for
 * `shape`, according to shape->state_interval (0 on a bad shape). */
size_t sru_amd_state_bytes(const sru_amd_shape *shape);

/* Bytes of device scratch sru_amd_backward needs for `shape` (0 on a bad
 * shape). The scratch holds per-column partial sums of the weight_c and bias
 * gradients between the scan kernel and the batch reduction. */
size_t sru_amd_backward_workspace_bytes(const sru_amd_shape *shape);

/* Backward scan. Replaces sru_cuda::sru_backward_simple, sru_bi_backward_simple,
 * sru_backward and sru_bi_backward (sru/csrc/sru_cuda_impl.cpp:210-252,:288-330,
 * :415-518) together with what sru/cuda_functional.py:204-207 and :253-260 run
 * around them: the x * scale_x pass, grad_x *= scale_x and the batch sums of
 * the weight_c / bias gradients.
 *   c         the state buffer the forward call filled (same shape->state_interval)
 *   c_init    as given to the forward call (NULL = zeros)
 *   grad_last gradient of c_last; NULL = zeros (the usual case: the last state is not part of
 *             the loss)
 *   grad_x    required iff skip_type == 1; already multiplied by scale_x
 *   grad_wc   (2, D') small, summed over time and batch, or, when is_custom,
 *             (L, B, D', 2) in `dtype`
 *   grad_bias (2, D') small, summed over time and batch
 *   workspace device scratch of at least sru_amd_backward_workspace_bytes()
 *             bytes, 16-byte aligned; contents before and after are undefined
 * The batch sums are formed in a fixed order: results are bit-reproducible. */
int sru_amd_backward(const sru_amd_shape *shape,
                     const void *u, const void *x, const void *weight_c,
                     const void *bias, const void *c_init, const void *mask_c,
                     const uint8_t *mask_pad, const void *scale_x,
                     const void *c, const void *grad_h, const void *grad_last,
                     void *grad_u, void *grad_x, void *grad_wc, void *grad_bias,
                     void *grad_init, void *workspace, size_t workspace_bytes,
                     void *stream);

/* sru_amd_backward without the workspace argument, for callers that cannot allocate device
 * memory at all: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc. It has no counterpart in the reference (whose operators allocate every output,
 * sru/csrc/sru_cuda_impl.cpp:225-229). The per-column partial sums live in an array built into
 * the library's device code (4 floats per column, 4 MiB, one copy per GPU for the life of the
 * process), so the call allocates nothing and asks for nothing beyond inputs and outputs.
 *   - at most SRU_AMD_STATIC_MAX_COLUMNS columns (B * D'; half as many with SRU_AMD_F64, whose
 *     partial sums are doubles); more returns SRU_AMD_ERR_STATIC_LIMIT and launches nothing;
 *   - results are bit-identical to sru_amd_backward's (same kernels);
 *   - all calls on one GPU share that GPU's array: two calls that overlap in time on one GPU
 *     (different streams, or two host threads) race; calls on one stream are safe back to back;
 *   - the first call on a device resolves the array's address (hipGetSymbolAddress); make that
 *     call outside a stream capture. */
#define SRU_AMD_STATIC_MAX_COLUMNS 262144
int sru_amd_backward_static(const sru_amd_shape *shape,
                            const void *u, const void *x, const void *weight_c,
                            const void *bias, const void *c_init, const void *mask_c,
                            const uint8_t *mask_pad, const void *scale_x,
                            const void *c, const void *grad_h, const void *grad_last,
                            void *grad_u, void *grad_x, void *grad_wc, void *grad_bias,
                            void *grad_init, void *stream);

/* Layer normalisation of the rows of a (rows, cols) matrix, the operation the reference applies to a
 * layer's input before the projection or to its output after the recurrence with
 * torch.nn.LayerNorm (sru/modules.py:155-162 created, :250-253 and :278-279 applied):
 *   y = (x - mean(x)) / sqrt(var(x) + eps) * weight + bias,   statistics per row, biased variance.
 * x and y may have different element types (enum sru_amd_dtype): the row is read once as it is
 * and written in the type its consumer wants, which under autocast replaces a chain of three
 * kernels (cast to float, normalise, cast to 16 bits). weight, bias, mean, rstd are float;
 * mean and rstd (one value per row) are what the backward call needs.
 *   cols must be a multiple of 8 and at most SRU_AMD_NORM_MAX_FEATURES; x, y, weight, bias
 *   16-byte aligned. */
#define SRU_AMD_NORM_MAX_FEATURES 4096
int sru_amd_layer_norm_forward(int64_t rows, int64_t cols, const void *x, int x_dtype,
                               const float *weight, const float *bias, float eps,
                               void *y, int y_dtype, float *mean, float *rstd, void *stream);

/* Bytes of device scratch sru_amd_layer_norm_backward needs (0 on a bad shape). */
size_t sru_amd_layer_norm_backward_workspace_bytes(int64_t rows, int64_t cols);

/* Backward of the above: grad_x (in x's element type) from grad_y (in y's element type), and the
 * weight / bias gradients summed over rows in a fixed order (bit-reproducible). grad_weight and
 * grad_bias must be the two halves of one (2, cols) float array: grad_bias == grad_weight + cols. */
int sru_amd_layer_norm_backward(int64_t rows, int64_t cols, const void *x, int x_dtype,
                                const float *weight, const float *mean, const float *rstd,
                                const void *grad_y, int y_dtype, void *grad_x,
                                float *grad_weight, float *grad_bias,
                                void *workspace, size_t workspace_bytes, void *stream);

/* Static, NUL-terminated description of a status code (never NULL). The
 * reference has no counterpart: its operators throw (sru_cuda_impl_dummy.cpp:19)
 * or fail inside data_ptr<T>(). */
const char *sru_amd_status_string(int status);

/* SRU_AMD_ABI_VERSION the library was built with. */
int sru_amd_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* SRU_AMD_H */
