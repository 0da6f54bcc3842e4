"""Replaying a stack from a HIP graph.

Short sequences are bound by launches, not by kernels: the README example (2 layers, L=20, B=32,
d=128) spends about 90 us of host time per forward around 15 us of kernels. Nothing in this
package allocates device memory behind torch's back, synchronises or reads a device value on the
host, so a whole `SRU` forward (and backward) records into a HIP graph as it is; a replay costs one
launch.

    fast = sru_amd.graphed(model, x_example, mask_pad=mask_example)
    h, c = fast(x, mask_pad=mask)            # same call, same results as model(x, mask_pad=mask)

* Shapes, dtypes, and which optional arguments are given are fixed at recording time; call
  `graphed` again for another shape.
* In eval mode, or when nothing requires a gradient, the forward pass alone is recorded
  (`torch.cuda.CUDAGraph`); the returned tensors are the graph's own output buffers and are
  overwritten by the next call: clone what must survive.
* In training mode forward and backward are recorded with torch's
  `torch.cuda.make_graphed_callables`; its rules apply (no double backward, parameters must not be
  replaced afterwards).
* Packed sequences are not supported: hand over the padded tensor and `mask_pad`.

The reference has no counterpart; it is the caller-side answer to the launch gaps that its own
per-call Python leaves between kernels as well (sru/modules.py:617-652).
"""
from typing import Optional

import torch
from torch import Tensor, nn


class _Positional(nn.Module):
    """model(x, c0, mask_pad) behind a signature of tensors only, which graph capture asks for."""

    def __init__(self, model: nn.Module, has_c0: bool, has_mask: bool, autocast_dtype):
        super().__init__()
        self.model = model
        self.has_c0, self.has_mask, self.autocast_dtype = has_c0, has_mask, autocast_dtype

    def forward(self, *tensors):
        it = iter(tensors)
        x = next(it)
        c0 = next(it) if self.has_c0 else None
        mask_pad = next(it) if self.has_mask else None
        if self.autocast_dtype is None:
            return self.model(x, c0, mask_pad=mask_pad)
        # (the cast cache would keep tensors of the recording alive across replays)
        with torch.autocast("cuda", dtype=self.autocast_dtype, cache_enabled=False):
            return self.model(x, c0, mask_pad=mask_pad)


class GraphedSRU:
    """Callable with the signature of `SRU.forward` that replays recorded graphs."""

    def __init__(self, model: nn.Module, x: Tensor, c0: Optional[Tensor] = None,
                 mask_pad: Optional[Tensor] = None, autocast_dtype: Optional[torch.dtype] = None,
                 warmup: int = 3):
        if not isinstance(x, Tensor) or x.dim() != 3 or not x.is_cuda:
            raise ValueError("graphed() records a (length, batch, input_size) device tensor; unpack packed "
                             "sequences and pass mask_pad")
        self.has_c0, self.has_mask = c0 is not None, mask_pad is not None
        self.module = _Positional(model, self.has_c0, self.has_mask, autocast_dtype)
        example = [t for t in (x, c0, mask_pad) if t is not None]
        self.shapes = [(t.shape, t.dtype) for t in example]
        wants_grad = torch.is_grad_enabled() and model.training and (
            x.requires_grad or any(p.requires_grad for p in model.parameters()))
        self.training = wants_grad
        if wants_grad:
            self._callable = torch.cuda.make_graphed_callables(
                self.module, tuple(t.detach().clone().requires_grad_(t.requires_grad) for t in example),
                num_warmup_iters=warmup)
            return
        # forward only: static input buffers, the recorded graph, static outputs
        self.static_in = [t.detach().clone() for t in example]
        side = torch.cuda.Stream(device=x.device)
        side.wait_stream(torch.cuda.current_stream(x.device))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):
                self.module(*self.static_in)
        torch.cuda.current_stream(x.device).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph), torch.no_grad():
            self.static_out = self.module(*self.static_in)

    def __call__(self, x: Tensor, c0: Optional[Tensor] = None, mask_pad: Optional[Tensor] = None):
        given = [t for t in (x, c0, mask_pad) if t is not None]
        if (c0 is not None) != self.has_c0 or (mask_pad is not None) != self.has_mask or \
                [(t.shape, t.dtype) for t in given] != self.shapes:
            raise ValueError("arguments differ from the recording (shapes, dtypes and which optional "
                             "arguments are given are fixed): record another graph with graphed()")
        if self.training:
            return self._callable(*given)
        for dst, src in zip(self.static_in, given):
            if dst.data_ptr() != src.data_ptr():
                dst.copy_(src)
        self.graph.replay()
        return self.static_out


def graphed(model: nn.Module, x: Tensor, c0: Optional[Tensor] = None, mask_pad: Optional[Tensor] = None,
            autocast_dtype: Optional[torch.dtype] = None, warmup: int = 3) -> GraphedSRU:
    """Records `model(x, c0, mask_pad=mask_pad)` (an `sru_amd.SRU` or `SRUCell`) and returns a callable
    that replays it. Recording happens in the model's current mode (train / eval) and under the
    current grad mode; `autocast_dtype` records the stack under autocast."""
    return GraphedSRU(model, x, c0, mask_pad, autocast_dtype, warmup)
