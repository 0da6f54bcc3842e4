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
`u` (float32, float16 or bfloat16); state and arithmetic are float32.
"""
from typing import Optional, Tuple

import ctypes

import torch
from torch import Tensor
from torch.autograd import Function

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


def _ptr(t: Optional[Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _aligned(t: Tensor, nbytes: int) -> Tensor:
    """Contiguous tensor whose first byte sits on an nbytes boundary."""
    t = t.contiguous()
    if t.data_ptr() % nbytes:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def _f32(t: Optional[Tensor]) -> Optional[Tensor]:
    if t is None:
        return None
    return _aligned(t if t.dtype == torch.float32 else t.float(), 4)


class _Problem:
    """Sizes and flags derived the way sru/cuda_functional.py:54-65 derives them."""

    def __init__(self, u: Tensor, x: Tensor, weight_c: Tensor, d_out: int,
                 bidirectional: bool, has_skip_term: bool, activation_type: int,
                 checkpoint_state: bool = False):
        if u.dtype not in _DTYPES:
            raise ValueError(f"U must be float32, float16 or bfloat16, not {u.dtype}")
        if not u.is_cuda:
            raise RuntimeError("the SRU recurrence kernels need device tensors (got a CPU tensor)")
        if x.dim() not in (2, 3):
            raise ValueError("x must be 2 or 3 dimensional")
        self.batch = x.size(-2)
        self.d = d_out
        self.length = x.size(0) if x.dim() == 3 else 1
        self.dirs = 2 if bidirectional else 1
        k = u.size(-1) // d_out
        self.k = k // 2 if bidirectional else k
        self.Dp = d_out * self.dirs
        if u.numel() != self.length * self.batch * self.Dp * self.k:
            raise ValueError(f"U has {u.numel()} elements, expected length*batch*{self.Dp}*{self.k}")
        self.is_custom = 1 if weight_c.dim() > 1 else 0
        self.skip_type = 0 if not has_skip_term else (1 if self.k == 3 else 2)
        self.activation_type = activation_type
        self.dtype = u.dtype
        self.squeeze = x.dim() == 2
        # Between forward and backward keep float checkpoints of the state instead of the
        # state after every step wherever the kernels support it (with four streams, a skip
        # term): the backward kernel rebuilds what lies in between.
        # 16-bit streams need an even d for that; a per-step weight_c must not come with tanh.
        ok = (u.dtype == torch.float32 or d_out % 2 == 0) and not (self.is_custom and activation_type != 0)
        self.checkpointed = bool(checkpoint_state and ok and not (self.skip_type == 0 and self.k == 4))
        self.shape = _lib.Shape(self.length, self.batch, self.d, self.dirs, self.k,
                                activation_type, self.skip_type, self.is_custom,
                                _DTYPES[u.dtype],
                                _lib.STATE_INTERVAL if self.checkpointed else 1)

    def group_bytes(self):
        es = 4 if self.dtype == torch.float32 else 2
        return es * (4 if self.k == 4 else 1)


def _prepare_inputs(pb: _Problem, u, x, weight_c, bias, init, scale_x, mask_c, mask_pad):
    u_ = _aligned(u, max(4, pb.group_bytes()))
    x_ = None
    if pb.skip_type == 1:
        x_ = _aligned(x if x.dtype == pb.dtype else x.to(pb.dtype), 4)
        if x_.numel() != pb.length * pb.batch * pb.Dp:
            raise ValueError("x must have length*batch*output_size elements when it is the skip term")
    if pb.is_custom:
        wc_ = _aligned(weight_c if weight_c.dtype == pb.dtype else weight_c.to(pb.dtype), 8)
        if wc_.numel() != pb.length * pb.batch * pb.Dp * 2:
            raise ValueError("per-step weight_c must have length*batch*output_size*2 elements")
    else:
        wc_ = _f32(weight_c)
        if wc_.numel() != 2 * pb.Dp:
            raise ValueError("weight_c must have 2*output_size elements")
    bias_ = _f32(bias)
    init_ = _f32(init)
    if bias_.numel() != 2 * pb.Dp or init_.numel() != pb.batch * pb.Dp:
        raise ValueError("bias must have 2*output_size and init batch*output_size elements")
    mask_c_ = _f32(mask_c)
    if mask_c_ is not None and mask_c_.numel() != pb.batch * pb.Dp:
        raise ValueError("mask_c must have batch*output_size elements")
    scale_ = None
    if scale_x is not None and pb.skip_type == 1:
        scale_ = _f32(scale_x.reshape(-1)[:1])
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
        rows = lib.sru_amd_state_bytes(ctypes.byref(pb.shape)) // (4 * pb.batch * pb.Dp)
        c = torch.empty(rows, pb.batch, pb.Dp, dtype=torch.float32, device=dev)
    elif keep_c:
        c = torch.empty(pb.length, pb.batch, pb.Dp, dtype=pb.dtype, device=dev)
    c_last = torch.empty(pb.batch, pb.Dp, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        rc = lib.sru_amd_forward(ctypes.byref(pb.shape), _ptr(u_), _ptr(x_), _ptr(wc_), _ptr(bias_),
                                 _ptr(init_), _ptr(mask_c_), _ptr(pad_), _ptr(scale_), _ptr(h),
                                 _ptr(c), _ptr(c_last), stream)
    _lib.check(rc, "sru_amd_forward")
    return h, c, c_last


def elementwise_recurrence_forward(
        u: Tensor, x: Tensor, weight_c: Tensor, bias: Tensor, init: Tensor,
        activation_type: int, d_out: int, bidirectional: bool, has_skip_term: bool,
        scale_x: Optional[Tensor] = None, mask_c: Optional[Tensor] = None,
        mask_pad: Optional[Tensor] = None, keep_c: bool = True
) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
    """Forward scan; returns (h, last_hidden, c) as sru/cuda_functional.py:37-153 does.

    `keep_c=False` (no counterpart in the reference) skips storing the per-step
    state and returns None for it: the inference variant.
    """
    pb = _Problem(u, x, weight_c, d_out, bidirectional, has_skip_term, activation_type)
    prepared = _prepare_inputs(pb, u, x, weight_c, bias, init, scale_x, mask_c, mask_pad)
    h, c, c_last = _run_forward(pb, *prepared, keep_c=keep_c)
    last_hidden = c_last if pb.dtype == torch.float32 else c_last.to(pb.dtype)
    if pb.squeeze:
        h = h.squeeze(0)
        c = c.squeeze(0) if c is not None else None
    return h, last_hidden, c


class ElementwiseRecurrence(Function):
    """Drop-in for sru/cuda_functional.py:156-261."""

    @staticmethod
    def forward(ctx, u, x, weight_c, bias, init, activation_type, d_out, bidirectional,
                has_skip_term, scale_x, mask_c=None, mask_pad=None):
        pb = _Problem(u, x, weight_c, d_out, bidirectional, has_skip_term, activation_type,
                      checkpoint_state=True)
        prepared = _prepare_inputs(pb, u, x, weight_c, bias, init, scale_x, mask_c, mask_pad)
        h, c, c_last = _run_forward(pb, *prepared, keep_c=True)
        ctx.problem = pb
        ctx.in_dtypes = (x.dtype, weight_c.dtype, bias.dtype, init.dtype)
        ctx.in_shapes = (u.shape, x.shape, weight_c.shape, bias.shape, init.shape)
        ctx.save_for_backward(*[t for t in prepared if t is not None], c)
        ctx.present = [t is not None for t in prepared]
        last_hidden = c_last if pb.dtype == torch.float32 else c_last.to(pb.dtype)
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
        gh = _aligned(grad_h if grad_h.dtype == pb.dtype else grad_h.to(pb.dtype), 4)
        gl = _f32(grad_last)
        grad_u = torch.empty_like(u_)
        grad_x = torch.empty_like(x_) if pb.skip_type == 1 else None
        grad_wc = torch.empty_like(wc_) if pb.is_custom else \
            torch.empty(2 * pb.Dp, dtype=torch.float32, device=dev)
        grad_bias = torch.empty(2 * pb.Dp, dtype=torch.float32, device=dev)
        grad_init = torch.empty(pb.batch, pb.Dp, dtype=torch.float32, device=dev)
        lib = _lib.load()
        ws_bytes = lib.sru_amd_backward_workspace_bytes(ctypes.byref(pb.shape))
        workspace = torch.empty(ws_bytes // 4, dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
            rc = lib.sru_amd_backward(
                ctypes.byref(pb.shape), _ptr(u_), _ptr(x_), _ptr(wc_), _ptr(bias_), _ptr(init_),
                _ptr(mask_c_), _ptr(pad_), _ptr(scale_), _ptr(c), _ptr(gh), _ptr(gl),
                _ptr(grad_u), _ptr(grad_x), _ptr(grad_wc), _ptr(grad_bias), _ptr(grad_init),
                _ptr(workspace), ctypes.c_size_t(ws_bytes), stream)
        _lib.check(rc, "sru_amd_backward")
        x_dt, wc_dt, bias_dt, init_dt = ctx.in_dtypes
        u_sh, x_sh, wc_sh, bias_sh, init_sh = ctx.in_shapes
        grad_u = grad_u.view(u_sh)
        if grad_x is not None:
            grad_x = grad_x.view(x_sh).to(x_dt)
        grad_wc = grad_wc.view(wc_sh).to(wc_dt)
        grad_bias = grad_bias.view(bias_sh).to(bias_dt)
        grad_init = grad_init.view(init_sh).to(init_dt)
        return grad_u, grad_x, grad_wc, grad_bias, grad_init, \
            None, None, None, None, None, None, None
