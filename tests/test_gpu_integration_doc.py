"""The binding INTEGRATION.md shows to a maintainer of the reference (section B) is executed here as
it stands: the first fenced python block of that section is extracted from the file, run, and its
two functions are called the way the text says sru/cuda_functional.py would call them (variable
names derived as at sru/cuda_functional.py:54-65). Results are checked against the CPU oracle to
the tolerances of tests/test_gpu_parity.py.
"""
import os
import re

import numpy as np
import pytest
import torch

from oracle import sru_oracle as so
from sru_amd import _lib
from tests.abi import to_np
from tests.cases import Case

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


def _binding():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    section = text[text.index("## B. Bind the C ABI directly"):text.index("## C. Layer norm")]
    block = re.search(r"```python\n(.*?)```", section, re.S).group(1)
    os.environ["SRU_AMD_SO"] = _lib.LIB_PATH
    ns = {}
    exec(compile(block, "INTEGRATION.md section B", "exec"), ns)
    return ns


def _reference_side_call(ns, case, dt, reference_state):
    """What the doc's two call sites do, from the tensors cuda_functional.py has in hand."""
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dt]
    t = lambda a, d=torch.float32: None if a is None else torch.tensor(a, dtype=d, device=DEV)
    c = case
    u, x = t(c.U, tdt), t(c.x, tdt)
    weight_c = t(c.wc, tdt if c.custom else torch.float32)
    bias, init, mask_c = t(c.bias), t(c.c0), t(c.mask_c)
    scale_x = torch.tensor([c.scale], device=DEV)
    mask_pad = None if c.pad is None else torch.tensor(c.pad, device=DEV)
    bidirectional, d, activation_type, has_skip_term = c.dirs == 2, c.d, c.act, c.skip_type != 0
    # sru/cuda_functional.py:54-71
    length = x.size(0) if x.dim() == 3 else 1
    batch = x.size(-2)
    k = u.size(-1) // d
    k_ = k // 2 if bidirectional else k
    is_custom = weight_c.dim() > 1
    skip_type = 0 if not has_skip_term else (1 if k_ == 3 else 2)
    mask_pad_ = None if mask_pad is None else mask_pad.to(torch.bool).contiguous()
    # the doc's forward call site
    shape = ns["sru_amd_shape_of"](u, length, batch, d, bidirectional, k_, activation_type, skip_type,
                                   is_custom, reference_state=reference_state)
    h, cs, last_hidden, saved = ns["sru_amd_forward"](shape, u, x, weight_c, bias, init, mask_c, mask_pad_,
                                                      scale_x if skip_type == 1 else None)
    # the doc's backward call site
    grad_h, grad_last = t(c.gh, tdt), t(c.gl)
    grads = ns["sru_amd_backward"](shape, saved, grad_h, grad_last)
    rounded = Case.__new__(Case)
    rounded.__dict__.update(c.__dict__)
    up = lambda v: v.double().cpu().numpy()
    rounded.U, rounded.x, rounded.gh, rounded.wc = up(u), up(x), up(grad_h), up(weight_c)
    return shape, h, cs, last_hidden, grads, rounded


@pytest.mark.parametrize("reference_state", [False, True], ids=["checkpoints", "reference_state"])
@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("cfg", [
    dict(L=40, B=6, d=128, dirs=2, pad="right", scale=1.7, mask_c=True),
    dict(L=33, B=4, d=64, dirs=2, k=4, pad="right"),
    dict(L=24, B=3, d=64, custom=True),
], ids=["bi_k3_padded", "bi_k4", "per_step_weight_c"])
def test_section_b_binding_against_oracle(cfg, dt, reference_state):
    ns = _binding()
    case = Case(seed=91, **cfg).f32()
    shape, h, cs, last_hidden, grads, rc = _reference_side_call(ns, case, dt, reference_state)
    assert shape.state_interval == (1 if reference_state else ns["SRU_AMD_STATE_INTERVAL"])
    h_ref, c_ref, cl_ref = so.forward(*rc.fwd_args(), **rc.kw())
    big = lambda ref: max(1.0, float(np.abs(ref).max()))
    tol = (lambda ref: 1e-5) if dt == "f32" else (lambda ref: 2e-2 * big(ref))
    err = lambda got, ref: float(np.abs(to_np(got).reshape(-1) - ref.reshape(-1)).max())
    assert err(h, h_ref) <= tol(h_ref)
    assert err(last_hidden, cl_ref) <= tol(cl_ref)
    if reference_state:
        assert tuple(cs.shape) == h_ref.shape and err(cs, c_ref) <= tol(c_ref)
        c_used = to_np(cs)
    else:
        c_used = c_ref
    g_ref = so.backward(*rc.fwd_args(), c_used, rc.gh, rc.gl, **rc.kw())
    for name, got, ref in zip(("grad_u", "grad_x", "grad_wc", "grad_bias", "grad_init"), grads, g_ref):
        if got is None:
            assert name == "grad_x" and case.skip_type != 1
            continue
        cell = float((np.abs(to_np(got).reshape(-1) - ref.reshape(-1)) / np.maximum(1.0, np.abs(ref.reshape(-1)))).max())
        assert cell <= (1e-5 * (big(ref) if name in ("grad_wc", "grad_bias") else 1.0) if dt == "f32"
                        else 2e-2 * (big(ref) if name in ("grad_wc", "grad_bias") else 1.0)), (name, cell)


def test_section_b_binding_without_initial_state_and_last_state_gradient():
    # init = None and grad_last = None stand for zeros
    ns = _binding()
    case = Case(seed=92, L=20, B=3, d=64, dirs=2, zero_c0=True).f32()
    case.gl = np.zeros_like(case.gl)
    t = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    u, x = t(case.U), t(case.x)
    shape = ns["sru_amd_shape_of"](u, case.L, case.B, case.d, True, 3, 0, 1, False)
    h, cs, last_hidden, saved = ns["sru_amd_forward"](shape, u, x, t(case.wc), t(case.bias), None, None, None, None)
    grads = ns["sru_amd_backward"](shape, saved, t(case.gh), None)
    h_ref, c_ref, cl_ref = so.forward(*case.fwd_args(), **case.kw())
    g_ref = so.backward(*case.fwd_args(), c_ref, case.gh, case.gl, **case.kw())
    assert float(np.abs(to_np(h) - h_ref).max()) <= 1e-5
    for got, ref in zip(grads, g_ref):
        assert float(np.abs(to_np(got).reshape(-1) - ref.reshape(-1)).max()) <= 1e-5 * max(1.0, float(np.abs(ref).max()))
