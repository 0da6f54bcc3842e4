"""Host side of the recurrence: the autograd boundary.

`ElementwiseRecurrence.apply` and `elementwise_recurrence_forward` keep the
argument lists and return values of the reference's
sru/cuda_functional.py:37-153 (forward helper) and :156-261 (autograd
Function), so a caller such as SRUCell.apply_recurrence (sru/modules.py:296-304)
can switch over without change. Behind them sits the C ABI of
include/sru_amd.h instead of the eight torch.ops.sru_cuda operators.

What moves into the kernels compared with the reference's Python:
  * x * scale_x (sru/cuda_functional.py:73-78, :204-207) and grad_x *= scale_x
    (:253-255): scale_x is handed over as a device pointer, never read on the host;
  * last_hidden (:146-153): the kernel writes the final state of every column;
  * the batch sums of grad_wc / grad_bias (:258-260);
  * zero filling of outputs (sru/csrc/sru_cuda_impl.cpp:189-190,:225-229): the
    kernels write every cell.

The large streams (U, x, h, c and their gradients) are consumed in the dtype of
`u` (float32, float16 or bfloat16); state and arithmetic are float32. A float32 x
beside a 16-bit U (the layer's input under autocast, which the reference keeps in
float32 too, sru/ops.py:121) is read as it is, and grad_x comes back in float32,
wherever the kernels take it (plain layer: vector weight_c, identity activation, even
d); elsewhere x is rounded to u's dtype first. A float64 U runs the double kernels:
streams, small tensors, state and arithmetic in double, as the reference's kernels
dispatched for double do (sru/csrc/sru_cuda_kernel.cu:845).
"""
from typing import Optional, Tuple

import ctypes
import functools

import torch
from torch import Tensor
from torch.autograd import Function

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float64: _lib.F64}


def _ptr(t: Optional[Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


class _on_device:
    """`with _on_device(dev) as stream:` makes `dev` the current device when it is not already (the
    launch goes to the current device) and yields the handle of torch's current stream on it. Same
    effect as torch.cuda.device() + torch.cuda.current_stream(), without their per-call bookkeeping,
    which is a quarter of the host time of a short call."""
    __slots__ = ("index", "guard")

    def __init__(self, dev: torch.device):
        self.index = dev.index if dev.index is not None else torch.cuda.current_device()
        self.guard = None

    def __enter__(self):
        if _raw_device is None or _raw_device() != self.index:
            self.guard = torch.cuda.device(self.index)
            self.guard.__enter__()
        if _raw_stream is not None:
            return ctypes.c_void_p(_raw_stream(self.index))
        return ctypes.c_void_p(torch.cuda.current_stream(self.index).cuda_stream)

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def _aligned(t: Tensor, nbytes: int) -> Tensor:
    """Contiguous tensor whose first byte sits on an nbytes boundary."""
    t = t.contiguous()
    if t.data_ptr() % nbytes:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def _small(t: Optional[Tensor], dtype: torch.dtype) -> Optional[Tensor]:
    """A small tensor (weight_c vector, bias, initial state, mask, scale, last-state gradient) as the
    kernels read it: float32, or float64 beside double streams."""
    if t is None:
        return None
    return _aligned(t if t.dtype == dtype else t.to(dtype), 8)


class _Problem:
    """Sizes and flags derived the way sru/cuda_functional.py:54-65 derives them. Instances are
    immutable and shared: `_problem()` keeps one per distinct (shape, dtype, flags)."""

    def __init__(self, dtype, x_dim, length, batch, u_numel, u_last, is_custom, d_out,
                 bidirectional, has_skip_term, activation_type, checkpoint_state, x_is_float, state_kept):
        if dtype not in _DTYPES:
            raise ValueError(f"U must be float32, float64, float16 or bfloat16, not {dtype}")
        if x_dim not in (2, 3):
            raise ValueError("x must be 2 or 3 dimensional")
        self.batch = batch
        self.d = d_out
        self.length = length
        self.dirs = 2 if bidirectional else 1
        k = u_last // d_out
        self.k = k // 2 if bidirectional else k
        self.Dp = d_out * self.dirs
        if u_numel != self.length * self.batch * self.Dp * self.k:
            raise ValueError(f"U has {u_numel} elements, expected length*batch*{self.Dp}*{self.k}")
        self.is_custom = is_custom
        self.skip_type = 0 if not has_skip_term else (1 if self.k == 3 else 2)
        self.activation_type = activation_type
        self.dtype = dtype
        self.small_dtype = torch.float64 if dtype == torch.float64 else torch.float32
        self.squeeze = x_dim == 2
        # Between forward and backward keep float checkpoints of the state instead of the
        # state after every step wherever the kernels support it (with four streams, a skip
        # term): the backward kernel rebuilds what lies in between.
        # 16-bit streams need an even d for that; a per-step weight_c must not come with tanh;
        # double streams run the general kernels, which read the state after every step.
        ok = (dtype == torch.float32 or d_out % 2 == 0) and not (self.is_custom and activation_type != 0) \
            and dtype != torch.float64
        self.checkpointed = bool(checkpoint_state and ok and not (self.skip_type == 0 and self.k == 4))
        # A float32 x beside 16-bit streams (the layer's input under autocast) is read as it is by
        # the chunked kernels of the plain layer; everywhere else x is rounded to the stream dtype.
        self.x_float = bool(x_is_float and dtype in (torch.float16, torch.bfloat16) and self.skip_type == 1 and not self.is_custom
                            and activation_type == 0 and d_out % 2 == 0 and (self.checkpointed or not state_kept))
        self.x_dtype = torch.float32 if self.x_float else dtype
        self.shape = _lib.Shape(self.length, self.batch, self.d, self.dirs, self.k,
                                activation_type, self.skip_type, self.is_custom,
                                _DTYPES[dtype],
                                _lib.STATE_INTERVAL if self.checkpointed else 1,
                                _lib.X_F32 if self.x_float else _lib.X_AS_STREAMS)
        lib = _lib.load()
        self.state_rows = lib.sru_amd_state_bytes(ctypes.byref(self.shape)) // (4 * self.batch * self.Dp) \
            if self.checkpointed else self.length
        self.workspace_bytes = lib.sru_amd_backward_workspace_bytes(ctypes.byref(self.shape))


_problem_cached = functools.lru_cache(maxsize=256)(_Problem)


def _problem(u: Tensor, x: Tensor, weight_c: Tensor, d_out: int, bidirectional: bool,
             has_skip_term: bool, activation_type: int, checkpoint_state: bool = False,
             state_kept: bool = True) -> _Problem:
    if not u.is_cuda:
        raise RuntimeError("the SRU recurrence kernels need device tensors (got a CPU tensor)")
    if x.dim() not in (2, 3):
        raise ValueError("x must be 2 or 3 dimensional")
    return _problem_cached(u.dtype, x.dim(), x.size(0) if x.dim() == 3 else 1, x.size(-2), u.numel(),
                           u.size(-1), 1 if weight_c.dim() > 1 else 0, d_out, bool(bidirectional),
                           bool(has_skip_term), int(activation_type), bool(checkpoint_state),
                           x.dtype == torch.float32, bool(state_kept))


def _prepare_inputs(pb: _Problem, u, x, weight_c, bias, init, scale_x, mask_c, mask_pad):
    # (16-bit k=4 groups of two columns move as one 16-byte vector in the checkpointed kernels)
    u_ = _aligned(u, 16)
    x_ = None
    if pb.skip_type == 1:
        x_ = _aligned(x if x.dtype == pb.x_dtype else x.to(pb.x_dtype), 4)
        if x_.numel() != pb.length * pb.batch * pb.Dp:
            raise ValueError("x must have length*batch*output_size elements when it is the skip term")
    if pb.is_custom:
        wc_ = _aligned(weight_c if weight_c.dtype == pb.dtype else weight_c.to(pb.dtype), 8)
        if wc_.numel() != pb.length * pb.batch * pb.Dp * 2:
            raise ValueError("per-step weight_c must have length*batch*output_size*2 elements")
    else:
        wc_ = _small(weight_c, pb.small_dtype)
        if wc_.numel() != 2 * pb.Dp:
            raise ValueError("weight_c must have 2*output_size elements")
    bias_ = _small(bias, pb.small_dtype)
    init_ = _small(init, pb.small_dtype)         # None: the kernels start from zeros
    if bias_.numel() != 2 * pb.Dp or (init_ is not None and init_.numel() != pb.batch * pb.Dp):
        raise ValueError("bias must have 2*output_size and init batch*output_size elements")
    mask_c_ = _small(mask_c, pb.small_dtype)
    if mask_c_ is not None and mask_c_.numel() != pb.batch * pb.Dp:
        raise ValueError("mask_c must have batch*output_size elements")
    scale_ = None
    if scale_x is not None and pb.skip_type == 1:
        scale_ = _small(scale_x.reshape(-1)[:1], pb.small_dtype)
    pad_ = None
    if mask_pad is not None:
        pad_ = mask_pad.contiguous()
        # same two checks as sru/cuda_functional.py:70-71
        assert pad_.size(0) == pb.length
        assert pad_.size(1) == pb.batch
        pad_ = (pad_ if pad_.dtype == torch.bool else pad_.bool()).view(torch.uint8)
    return u_, x_, wc_, bias_, init_, scale_, mask_c_, pad_


def _run_forward(pb, u_, x_, wc_, bias_, init_, scale_, mask_c_, pad_, keep_c: bool):
    dev = u_.device
    lib = _lib.load()
    h = torch.empty(pb.length, pb.batch, pb.Dp, dtype=pb.dtype, device=dev)
    c = None
    if keep_c and pb.checkpointed:
        c = torch.empty(pb.state_rows, pb.batch, pb.Dp, dtype=torch.float32, device=dev)
    elif keep_c:
        c = torch.empty(pb.length, pb.batch, pb.Dp, dtype=pb.dtype, device=dev)
    c_last = torch.empty(pb.batch, pb.Dp, dtype=pb.small_dtype, device=dev)
    with _on_device(dev) as stream:
        rc = lib.sru_amd_forward(ctypes.byref(pb.shape), _ptr(u_), _ptr(x_), _ptr(wc_), _ptr(bias_),
                                 _ptr(init_), _ptr(mask_c_), _ptr(pad_), _ptr(scale_), _ptr(h),
                                 _ptr(c), _ptr(c_last), stream)
    _lib.check(rc, "sru_amd_forward")
    return h, c, c_last


def _kernel_dtype(u: Tensor) -> torch.dtype:
    """Stream dtype the kernels run in for a U of this dtype: the four the kernels exist for as
    they are, anything else float32."""
    return u.dtype if u.dtype in _DTYPES else torch.float32


def elementwise_recurrence_forward(
        u: Tensor, x: Tensor, weight_c: Tensor, bias: Tensor, init: Optional[Tensor],
        activation_type: int, d_out: int, bidirectional: bool, has_skip_term: bool,
        scale_x: Optional[Tensor] = None, mask_c: Optional[Tensor] = None,
        mask_pad: Optional[Tensor] = None, keep_c: bool = True
) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
    """Forward scan; returns (h, last_hidden, c) as sru/cuda_functional.py:37-153 does, in U's dtype.

    `keep_c=False` (no counterpart in the reference) skips storing the per-step
    state and returns None for it: the inference variant. `init=None` stands for zeros.
    """
    out_dtype = u.dtype
    if u.dtype != _kernel_dtype(u):
        u = u.to(_kernel_dtype(u))
    pb = _problem(u, x, weight_c, d_out, bidirectional, has_skip_term, activation_type, state_kept=keep_c)
    prepared = _prepare_inputs(pb, u, x, weight_c, bias, init, scale_x, mask_c, mask_pad)
    h, c, c_last = _run_forward(pb, *prepared, keep_c=keep_c)
    last_hidden = c_last if out_dtype == c_last.dtype else c_last.to(out_dtype)
    if out_dtype != pb.dtype:
        h = h.to(out_dtype)
        c = c.to(out_dtype) if c is not None else None
    if pb.squeeze:
        h = h.squeeze(0)
        c = c.squeeze(0) if c is not None else None
    return h, last_hidden, c


class ElementwiseRecurrence(Function):
    """Drop-in for sru/cuda_functional.py:156-261.

    Beyond the reference's argument list: `init` may be None (zeros, and no gradient for it).
    Outputs come back in U's dtype and gradients in the dtypes of the inputs; a float64 U is
    computed in double, so torch.autograd.gradcheck applies to this Function as it is."""

    @staticmethod
    def forward(ctx, u, x, weight_c, bias, init, activation_type, d_out, bidirectional,
                has_skip_term, scale_x, mask_c=None, mask_pad=None):
        # gradients that autograd does not have stay None instead of becoming zero tensors (one
        # fill kernel per layer for the usually unused gradient of the last state)
        ctx.set_materialize_grads(False)
        u_dtype = u.dtype
        if u.dtype != _kernel_dtype(u):
            u = u.to(_kernel_dtype(u))
        pb = _problem(u, x, weight_c, d_out, bidirectional, has_skip_term, activation_type,
                      checkpoint_state=True)
        prepared = _prepare_inputs(pb, u, x, weight_c, bias, init, scale_x, mask_c, mask_pad)
        h, c, c_last = _run_forward(pb, *prepared, keep_c=True)
        ctx.problem = pb
        ctx.in_dtypes = (u_dtype, x.dtype, weight_c.dtype, bias.dtype, None if init is None else init.dtype)
        ctx.in_shapes = (u.shape, x.shape, weight_c.shape, bias.shape, None if init is None else init.shape)
        ctx.save_for_backward(*[t for t in prepared if t is not None], c)
        ctx.present = [t is not None for t in prepared]
        last_hidden = c_last if u_dtype == c_last.dtype else c_last.to(u_dtype)
        if u_dtype != pb.dtype:
            h = h.to(u_dtype)
        if pb.squeeze:
            h = h.squeeze(0)
        return h, last_hidden

    @staticmethod
    def backward(ctx, grad_h, grad_last):
        pb = ctx.problem
        saved = list(ctx.saved_tensors)
        c = saved.pop()
        it = iter(saved)
        u_, x_, wc_, bias_, init_, scale_, mask_c_, pad_ = [next(it) if p else None for p in ctx.present]
        dev = u_.device
        if grad_h is None:     # only last_hidden was used downstream
            gh = torch.zeros(pb.length, pb.batch, pb.Dp, dtype=pb.dtype, device=dev)
        else:
            gh = _aligned(grad_h if grad_h.dtype == pb.dtype else grad_h.to(pb.dtype), 4)
        gl = _small(grad_last, pb.small_dtype)   # None: the kernels start from a zero state gradient
        grad_u = torch.empty_like(u_)
        grad_x = torch.empty_like(x_) if pb.skip_type == 1 else None
        grad_wc = torch.empty_like(wc_) if pb.is_custom else \
            torch.empty(2 * pb.Dp, dtype=pb.small_dtype, device=dev)
        # grad_bias (2, D') and grad_init (B, D') share one allocation
        small = torch.empty((2 + pb.batch) * pb.Dp, dtype=pb.small_dtype, device=dev)
        grad_bias, grad_init = small[:2 * pb.Dp], small[2 * pb.Dp:]
        ws_bytes = pb.workspace_bytes
        workspace = torch.empty(ws_bytes // 4, dtype=torch.float32, device=dev)
        with _on_device(dev) as stream:
            rc = _lib.load().sru_amd_backward(
                ctypes.byref(pb.shape), _ptr(u_), _ptr(x_), _ptr(wc_), _ptr(bias_), _ptr(init_),
                _ptr(mask_c_), _ptr(pad_), _ptr(scale_), _ptr(c), _ptr(gh), _ptr(gl),
                _ptr(grad_u), _ptr(grad_x), _ptr(grad_wc), _ptr(grad_bias), _ptr(grad_init),
                _ptr(workspace), ctypes.c_size_t(ws_bytes), stream)
        _lib.check(rc, "sru_amd_backward")
        u_dt, x_dt, wc_dt, bias_dt, init_dt = ctx.in_dtypes
        u_sh, x_sh, wc_sh, bias_sh, init_sh = ctx.in_shapes
        grad_u = grad_u.view(u_sh).to(u_dt)
        if grad_x is not None:
            grad_x = grad_x.view(x_sh).to(x_dt)
        grad_wc = grad_wc.view(wc_sh).to(wc_dt)
        grad_bias = grad_bias.view(bias_sh).to(bias_dt)
        grad_init = None if init_sh is None else grad_init.view(init_sh).to(init_dt)
        return grad_u, grad_x, grad_wc, grad_bias, grad_init, \
            None, None, None, None, None, None, None
