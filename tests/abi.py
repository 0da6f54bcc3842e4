"""Drives the C ABI (include/sru_amd.h) from a tests.cases.Case: torch is used only to
own device memory and the stream."""
import ctypes

import numpy as np
import torch

from sru_amd import _lib

TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "f64": torch.float64}
CODE = {"f32": _lib.F32, "f16": _lib.F16, "bf16": _lib.BF16, "f64": _lib.F64}


def p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


class DeviceProblem:
    """Device copies of a Case in stream dtype `dt`; float32 for the small tensors (float64 with
    double streams)."""

    def __init__(self, case, dt="f32", device="cuda:0", checkpointed=False, x_f32=False):
        """checkpointed: keep float state checkpoints between forward and backward
        (shape.state_interval = SRU_AMD_STATE_INTERVAL) instead of the state after every step.
        x_f32: x and grad_x are float32 beside 16-bit streams (shape.x_dtype = SRU_AMD_X_F32)."""
        self.case, self.dt, self.checkpointed, self.x_f32 = case, dt, checkpointed, x_f32
        tdt = TORCH_DT[dt]
        sdt = self.sdt = torch.float64 if dt == "f64" else torch.float32
        dev = torch.device(device)
        big = lambda a: torch.tensor(a, dtype=tdt, device=dev).contiguous()
        small = lambda a: None if a is None else torch.tensor(a, dtype=sdt, device=dev).contiguous()
        c = case
        self.U, self.x, self.gh = big(c.U), big(c.x), big(c.gh)
        if x_f32:
            self.x = torch.tensor(c.x, dtype=torch.float32, device=dev).contiguous()
        self.wc = big(c.wc) if c.custom else small(c.wc)
        self.bias, self.c0, self.gl, self.mask_c = small(c.bias), small(c.c0), small(c.gl), small(c.mask_c)
        self.scale = torch.tensor([c.scale], dtype=sdt, device=dev)
        self.pad = None if c.pad is None else torch.tensor(c.pad, dtype=torch.bool, device=dev).view(torch.uint8)
        self.shape = _lib.Shape(c.L, c.B, c.d, c.dirs, c.k, c.act, c.skip_type, c.custom, CODE[dt],
                                _lib.STATE_INTERVAL if checkpointed else 1, _lib.X_F32 if x_f32 else _lib.X_AS_STREAMS)
        self.dev, self.tdt = dev, tdt

    def rounded_case(self):
        """The Case holding exactly the values the device sees (after rounding to dt)."""
        import copy
        c = copy.copy(self.case)
        up = lambda t: t.double().cpu().numpy()
        c.U, c.x, c.gh = up(self.U), up(self.x), up(self.gh)
        c.wc, c.bias, c.c0, c.gl = up(self.wc), up(self.bias), up(self.c0), up(self.gl)
        c.mask_c = None if self.mask_c is None else up(self.mask_c)
        c.scale = float(self.scale.item())
        return c

    def forward(self, keep_c=True, poison=True):
        c = self.case
        mk = (lambda *s, dtype: torch.full(s, float("nan"), dtype=dtype, device=self.dev)) if poison else \
            (lambda *s, dtype: torch.empty(s, dtype=dtype, device=self.dev))
        self.h = mk(c.L, c.B, c.Dp, dtype=self.tdt)
        if keep_c and self.checkpointed:
            nbytes = _lib.load().sru_amd_state_bytes(ctypes.byref(self.shape))
            self.c = mk(nbytes // (4 * c.B * c.Dp), c.B, c.Dp, dtype=torch.float32)
        else:
            self.c = mk(c.L, c.B, c.Dp, dtype=self.tdt) if keep_c else None
        self.c_last = mk(c.B, c.Dp, dtype=self.sdt)
        stream = ctypes.c_void_p(torch.cuda.current_stream(self.dev).cuda_stream)
        rc = _lib.load().sru_amd_forward(
            ctypes.byref(self.shape), p(self.U), p(self.x) if c.skip_type == 1 else None, p(self.wc),
            p(self.bias), p(self.c0), p(self.mask_c), p(self.pad),
            p(self.scale) if c.skip_type == 1 else None, p(self.h), p(self.c), p(self.c_last), stream)
        assert rc == 0, _lib.status_string(rc)
        return self.h, self.c, self.c_last

    def backward(self, c_state=None, poison=True):
        c = self.case
        mk = (lambda *s, dtype: torch.full(s, float("nan"), dtype=dtype, device=self.dev)) if poison else \
            (lambda *s, dtype: torch.empty(s, dtype=dtype, device=self.dev))
        self.gu = mk(c.L, c.B, c.Dp * c.k, dtype=self.tdt)
        self.gx = mk(c.L, c.B, c.Dp, dtype=torch.float32 if self.x_f32 else self.tdt) if c.skip_type == 1 else None
        self.gwc = mk(c.L, c.B, c.Dp * 2, dtype=self.tdt) if c.custom else mk(2 * c.Dp, dtype=self.sdt)
        self.gb = mk(2 * c.Dp, dtype=self.sdt)
        self.gi = mk(c.B, c.Dp, dtype=self.sdt)
        lib = _lib.load()
        nbytes = lib.sru_amd_backward_workspace_bytes(ctypes.byref(self.shape))
        self.ws = mk(nbytes // 4, dtype=torch.float32)
        stream = ctypes.c_void_p(torch.cuda.current_stream(self.dev).cuda_stream)
        rc = lib.sru_amd_backward(
            ctypes.byref(self.shape), p(self.U), p(self.x) if c.skip_type == 1 else None, p(self.wc),
            p(self.bias), p(self.c0), p(self.mask_c), p(self.pad),
            p(self.scale) if c.skip_type == 1 else None, p(self.c if c_state is None else c_state),
            p(self.gh), p(self.gl), p(self.gu), p(self.gx), p(self.gwc), p(self.gb), p(self.gi),
            p(self.ws), ctypes.c_size_t(nbytes), stream)
        assert rc == 0, _lib.status_string(rc)
        return self.gu, self.gx, self.gwc, self.gb, self.gi


def to_np(t):
    return None if t is None else t.double().cpu().numpy()
