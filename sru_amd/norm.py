"""Layer normalisation next to the recurrence (sru/modules.py:155-162, :250-253, :278-279).

`layer_norm(x, weight, bias, eps, out_dtype)` is torch.nn.functional.layer_norm over the last
dimension with one difference: the output dtype can be chosen, so that under autocast the
normalised rows leave the kernel already in the 16-bit dtype the projection consumes. It runs the
HIP kernels of csrc/sru_norm.hip through the C ABI (include/sru_amd.h); `supported()` says whether
a tensor can take that path (device tensor, feature count a multiple of 8 and at most
SRU_AMD_NORM_MAX_FEATURES) - anything else is torch's own layer_norm, which is the operation the
reference itself calls; `layer_norm` says so with a warning (or raises with `strict=True`).
"""
import ctypes
import warnings
from typing import Optional

import torch
from torch import Tensor
from torch.autograd import Function

from . import _lib
from .functional import _aligned, _on_device, _ptr, _small

# element types the layer-norm kernels read and write (no double rows)
_DTYPES = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


def supported(x: Tensor) -> bool:
    d = x.size(-1)
    return bool(x.is_cuda and x.dtype in _DTYPES and x.numel() > 0 and d % 8 == 0 and d <= _lib.NORM_MAX_FEATURES)


class LayerNormFunction(Function):
    @staticmethod
    def forward(ctx, x, weight, bias, eps, out_dtype):
        D = x.size(-1)
        if weight.numel() != D or bias.numel() != D:
            raise ValueError(f"layer norm over {D} features needs weight and bias of {D} elements, "
                             f"not {weight.numel()} and {bias.numel()}")
        x_ = _aligned(x, 16)
        w_, b_ = _aligned(_small(weight, torch.float32), 16), _aligned(_small(bias, torch.float32), 16)
        rows = x_.numel() // D
        y = torch.empty(x_.shape, dtype=out_dtype, device=x.device)
        mean = torch.empty(rows, dtype=torch.float32, device=x.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
        with _on_device(x.device) as stream:
            rc = _lib.load().sru_amd_layer_norm_forward(rows, D, _ptr(x_), _DTYPES[x_.dtype], _ptr(w_), _ptr(b_),
                                                        ctypes.c_float(eps), _ptr(y), _DTYPES[out_dtype],
                                                        _ptr(mean), _ptr(rstd), stream)
        _lib.check(rc, "sru_amd_layer_norm_forward")
        ctx.save_for_backward(x_, w_, mean, rstd)
        ctx.param_dtypes = (weight.dtype, bias.dtype)
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x_, w_, mean, rstd = ctx.saved_tensors
        D = x_.size(-1)
        rows = x_.numel() // D
        gy = _aligned(grad_y if grad_y.dtype in _DTYPES else grad_y.float(), 16)
        if gy.shape != x_.shape:
            raise ValueError(f"grad_y has shape {tuple(gy.shape)}, expected {tuple(x_.shape)}")
        grad_x = torch.empty_like(x_)
        grad_wb = torch.empty(2, D, dtype=torch.float32, device=x_.device)
        lib = _lib.load()
        nbytes = lib.sru_amd_layer_norm_backward_workspace_bytes(rows, D)
        workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=x_.device)
        with _on_device(x_.device) as stream:
            rc = lib.sru_amd_layer_norm_backward(rows, D, _ptr(x_), _DTYPES[x_.dtype], _ptr(w_), _ptr(mean),
                                                 _ptr(rstd), _ptr(gy), _DTYPES[gy.dtype], _ptr(grad_x),
                                                 _ptr(grad_wb[0]), _ptr(grad_wb[1]), _ptr(workspace),
                                                 ctypes.c_size_t(nbytes), stream)
        _lib.check(rc, "sru_amd_layer_norm_backward")
        wdt, bdt = ctx.param_dtypes
        return grad_x, grad_wb[0].to(wdt), grad_wb[1].to(bdt), None, None


_warned_widths = set()


def layer_norm(x: Tensor, weight: Tensor, bias: Tensor, eps: float = 1e-5,
               out_dtype: Optional[torch.dtype] = None, strict: bool = False) -> Tensor:
    """Normalises over the last dimension; `out_dtype` defaults to x's dtype.

    A tensor the kernels do not take (see `supported`) goes through torch's own layer_norm, once
    per feature count with a warning; `strict=True` raises instead."""
    out_dtype = out_dtype or x.dtype
    if out_dtype not in _DTYPES and x.dtype in _DTYPES:
        raise ValueError(f"out_dtype must be float32, float16 or bfloat16, not {out_dtype}")
    if not supported(x):
        why = (f"sru_amd.norm.layer_norm: no kernel for a {x.dtype} {'device' if x.is_cuda else 'CPU'} tensor with "
               f"{x.size(-1)} features (needs a device tensor, a multiple of 8 and at most {_lib.NORM_MAX_FEATURES})")
        if strict:
            raise ValueError(why)
        key = (x.size(-1), x.dtype, x.is_cuda)
        if key not in _warned_widths:
            _warned_widths.add(key)
            warnings.warn(why + "; using torch.nn.functional.layer_norm")
        wide = torch.float64 if x.dtype == torch.float64 else torch.float32
        y = torch.nn.functional.layer_norm(x.to(wide), (x.size(-1),), weight.to(wide), bias.to(wide), eps)
        return y.to(out_dtype)
    return LayerNormFunction.apply(x, weight, bias, eps, out_dtype)
