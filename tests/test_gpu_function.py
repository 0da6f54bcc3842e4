"""The autograd boundary on the GPU: sru_amd.ElementwiseRecurrence.apply with the
reference's argument list (sru/cuda_functional.py:159-167) against the oracle's
differentiable restatement, in the manner of the reference's own CPU-vs-GPU gradient test
(test/sru/test_sru.py:128-162; tolerance there 1e-4, here 1e-5)."""
import numpy as np
import pytest
import torch

from oracle import sru_torch as st
from tests.cases import Case

pytestmark = pytest.mark.gpu


def _apply(fn, c, device, dtype):
    t = lambda a, rg=True: torch.tensor(a, dtype=dtype, device=device, requires_grad=rg)
    u, x, wc, bias, c0 = t(c.U), t(c.x), t(c.wc), t(c.bias), t(c.c0)
    sx = torch.tensor([c.scale], dtype=dtype, device=device)
    mc = None if c.mask_c is None else torch.tensor(c.mask_c, dtype=dtype, device=device)
    pad = None if c.pad is None else torch.tensor(c.pad, device=device)
    h, last = fn(u, x, wc, bias, c0, c.act, c.d, c.dirs == 2, c.skip_type != 0, sx, mc, pad)
    gh = torch.tensor(c.gh, dtype=dtype, device=device)
    gl = torch.tensor(c.gl, dtype=dtype, device=device)
    ((h * gh).sum() + (last * gl).sum()).backward()
    grads = [None if v.grad is None else v.grad.double().cpu().numpy() for v in (u, x, wc, bias, c0)]
    return h.detach().double().cpu().numpy(), last.detach().double().cpu().numpy(), grads


@pytest.mark.parametrize("cfg", [
    dict(L=12, B=3, d=64, dirs=2, pad="right", scale=1.7, mask_c=True),
    dict(L=9, B=4, d=7, dirs=2, k=4),
    dict(L=5, B=2, d=3, skip=False),
    dict(L=6, B=2, d=8, custom=True, act=1),
    dict(L=3, B=5, d=2, dirs=2),
])
def test_function_matches_restatement(cfg):
    from sru_amd import ElementwiseRecurrence
    c = Case(seed=41, **cfg).f32()
    h, last, g = _apply(ElementwiseRecurrence.apply, c, "cuda:0", torch.float32)
    h_ref, last_ref, g_ref = _apply(st.recurrence, c, "cpu", torch.float64)
    assert np.abs(h - h_ref).max() <= 1e-5 and np.abs(last - last_ref).max() <= 1e-5
    for a, b in zip(g, g_ref):
        if b is None or (c.skip_type != 1 and a is None):
            continue
        assert a is not None
        assert np.abs(a - b).max() <= 1e-5 * max(1.0, np.abs(b).max())
    if c.skip_type != 1:
        assert g[1] is None


def test_single_step_2d_input_and_inference_entry():
    from sru_amd import elementwise_recurrence_forward, elementwise_recurrence_inference
    c = Case(L=1, B=4, d=64, dirs=2, seed=42).f32()
    dev = "cuda:0"
    t = lambda a: torch.tensor(a, dtype=torch.float32, device=dev)
    h, last, cc = elementwise_recurrence_forward(t(c.U[0]), t(c.x[0]), t(c.wc), t(c.bias), t(c.c0),
                                                 0, c.d, True, True, None)
    assert h.shape == (4, 128) and cc.shape == (4, 128) and torch.equal(last, cc)
    h3, last3 = elementwise_recurrence_inference(t(c.U), t(c.x), t(c.wc), t(c.bias), t(c.c0),
                                                 0, c.d, True, True, None, None, None)
    assert torch.equal(h3[0], h) and torch.equal(last3, last)
    with pytest.raises(AssertionError):
        elementwise_recurrence_inference(t(c.U), t(c.x), t(c.wc), t(c.bias), t(c.c0), 0, c.d, True, True,
                                         None, t(c.c0), None)
    with pytest.raises(AssertionError):   # mask_pad shape, as sru/cuda_functional.py:70-71
        elementwise_recurrence_forward(t(c.U), t(c.x), t(c.wc), t(c.bias), t(c.c0), 0, c.d, True, True,
                                       None, None, torch.zeros(2, 4, device=dev))


def test_amp_style_bf16_streams_against_fp32_run():
    # U and x arrive in bfloat16 (autocast GEMM output); the reference would cast them to
    # float32 (sru/ops.py:116-127) and run there. Tolerance: 2e-2 relative to that run.
    from sru_amd import elementwise_recurrence_gpu
    c = Case(L=32, B=4, d=128, dirs=2, seed=43, pad="right", scale=1.7)
    dev = "cuda:0"
    outs = {}
    for native in (True, False):
        t = lambda a, dt=torch.float32: torch.tensor(a, dtype=dt, device=dev, requires_grad=True)
        u, x = t(c.U, torch.bfloat16), t(c.x, torch.bfloat16)
        wc, bias, c0 = t(c.wc), t(c.bias), t(c.c0)
        h, last = elementwise_recurrence_gpu(u, x, wc, bias, c0, 0, c.d, True, True,
                                             torch.tensor([c.scale], device=dev), None,
                                             torch.tensor(c.pad, device=dev), native_16bit=native)
        assert h.dtype == (torch.bfloat16 if native else torch.float32)
        (h.float() * torch.tensor(c.gh, dtype=torch.float32, device=dev)).sum().backward()
        outs[native] = [h.float()] + [v.grad.float() for v in (u, x, wc, bias, c0)]
    for a, b in zip(outs[True], outs[False]):
        assert float((a - b).detach().abs().max()) <= 2e-2 * max(1.0, float(b.detach().abs().max()))


def test_float64_function_runs_in_double_and_training_entry_casts_to_float32():
    # the reference's autograd Function, called directly, keeps the dtype of U and its kernels exist
    # for double (sru/csrc/sru_cuda_kernel.cu:845); its training entry casts float64 to float32 and
    # returns float32 (sru/ops.py:116-127). Same here.
    from sru_amd import ElementwiseRecurrence, elementwise_recurrence_gpu
    c = Case(L=14, B=3, d=64, dirs=2, seed=44, pad="right", scale=1.7, mask_c=True)
    h64, last64, g64 = _apply(ElementwiseRecurrence.apply, c, "cuda:0", torch.float64)
    h_ref, last_ref, g_ref = _apply(st.recurrence, c, "cpu", torch.float64)
    assert np.abs(h64 - h_ref).max() <= 1e-12 and np.abs(last64 - last_ref).max() <= 1e-12
    for a, b in zip(g64, g_ref):
        assert a is not None and np.abs(a - b).max() <= 1e-12 * max(1.0, np.abs(b).max())
    dev = "cuda:0"
    t = lambda a: torch.tensor(a, dtype=torch.float64, device=dev, requires_grad=True)
    u, x, wc, bias, c0 = t(c.U), t(c.x), t(c.wc), t(c.bias), t(c.c0)
    h, last = ElementwiseRecurrence.apply(u, x, wc, bias, c0, 0, c.d, True, True, None, None, None)
    assert h.dtype == torch.float64 and last.dtype == torch.float64
    h.sum().backward()
    assert all(v.grad is not None and v.grad.dtype == torch.float64 for v in (u, x, wc, bias, c0))
    h, last = elementwise_recurrence_gpu(u, x, wc, bias, c0, 0, c.d, True, True)
    assert h.dtype == torch.float32 and last.dtype == torch.float32
    with torch.no_grad():
        h, last = elementwise_recurrence_gpu(u, x, wc, bias, c0, 0, c.d, True, True)
    assert h.dtype == torch.float32


@pytest.mark.parametrize("cfg", [
    dict(L=6, B=2, d=5, dirs=2, pad="right", scale=1.7, mask_c=True),
    dict(L=5, B=2, d=3, dirs=2, k=4, act=1),
    dict(L=4, B=2, d=3, skip=False, pad="random"),
    dict(L=4, B=2, d=4, custom=True, act=1),
])
def test_gradcheck_of_the_function_in_double(cfg):
    # finite differences of the forward kernels against the backward kernels, both in double: a check
    # of the analytic backward pass that does not go through the oracle
    from sru_amd import ElementwiseRecurrence
    c = Case(seed=46, **cfg)
    dev = "cuda:0"
    t = lambda a: torch.tensor(a, dtype=torch.float64, device=dev, requires_grad=True)
    u, x, wc, bias, c0 = t(c.U), t(c.x), t(c.wc), t(c.bias), t(c.c0)
    sx = torch.tensor([c.scale], dtype=torch.float64, device=dev)
    mc = None if c.mask_c is None else torch.tensor(c.mask_c, dtype=torch.float64, device=dev)
    pad = None if c.pad is None else torch.tensor(c.pad, device=dev)
    fn = lambda u, x, wc, bias, c0: ElementwiseRecurrence.apply(
        u, x, wc, bias, c0, c.act, c.d, c.dirs == 2, c.skip_type != 0, sx, mc, pad)
    inputs = (u, x, wc, bias, c0) if c.skip_type == 1 else (u, x.detach(), wc, bias, c0)
    assert torch.autograd.gradcheck(fn, inputs, eps=1e-6, atol=1e-7, rtol=1e-6, nondet_tol=0.0)


def test_no_initial_state_no_last_state_gradient_and_last_state_only():
    # init = None stands for zeros (no zero tensor is built); a loss that does not use last_hidden
    # hands the backward kernel no grad_last; a loss that uses only last_hidden hands it no grad_h
    from sru_amd import ElementwiseRecurrence
    c = Case(L=21, B=3, d=64, dirs=2, seed=45, scale=1.3, zero_c0=True).f32()
    dev = "cuda:0"
    t = lambda a: torch.tensor(a, dtype=torch.float32, device=dev, requires_grad=True)
    sx = torch.tensor([c.scale], device=dev)
    gh = torch.tensor(c.gh, dtype=torch.float32, device=dev)
    gl = torch.tensor(c.gl, dtype=torch.float32, device=dev)
    results = {}
    for name, init_none, loss in (("zeros", False, "both"), ("none", True, "both"), ("h_only", True, "h"),
                                  ("h_only_ref", False, "h"), ("last_only", True, "last"), ("last_only_ref", False, "last")):
        u, x, wc, bias = t(c.U), t(c.x), t(c.wc), t(c.bias)
        c0 = None if init_none else t(c.c0)
        h, last = ElementwiseRecurrence.apply(u, x, wc, bias, c0, 0, c.d, True, True, sx, None, None)
        total = 0
        if loss in ("both", "h"):
            total = total + (h * gh).sum()
        if loss in ("both", "last"):
            total = total + (last * gl).sum()
        total.backward()
        results[name] = [h.detach(), last.detach()] + [v.grad for v in (u, x, wc, bias)]
    for a, b in (("none", "zeros"), ("h_only", "h_only_ref"), ("last_only", "last_only_ref")):
        for got, ref in zip(results[a], results[b]):
            assert torch.equal(got, ref), (a, b)


def test_u_view_at_an_unaligned_offset_is_copied_not_refused():
    # a contiguous U whose storage offset is 8 bytes: the 16-bit k=4 checkpoint kernels need 16
    from sru_amd import ElementwiseRecurrence
    c = Case(L=16, B=2, d=64, dirs=2, k=4, seed=46)
    dev = "cuda:0"
    flat = torch.zeros(c.U.size + 4, dtype=torch.bfloat16, device=dev)
    flat[4:] = torch.tensor(c.U, dtype=torch.bfloat16, device=dev).reshape(-1)
    u_view = flat[4:].view(c.L, c.B, -1).requires_grad_(True)
    assert u_view.data_ptr() % 16 == 8 and u_view.is_contiguous()
    u_own = u_view.detach().clone().requires_grad_(True)
    t = lambda a: torch.tensor(a, dtype=torch.float32, device=dev)
    x = torch.tensor(c.x, dtype=torch.bfloat16, device=dev)
    outs = []
    for u in (u_view, u_own):
        h, last = ElementwiseRecurrence.apply(u, x, t(c.wc), t(c.bias), t(c.c0), 0, c.d, True, True, None, None, None)
        h.float().sum().backward()
        outs.append((h.detach(), u.grad))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


def test_float32_x_beside_bf16_u_is_not_rounded():
    """Under autocast the layer's input stays float32 while U is 16-bit: x goes to the kernels as it
    is (no cast pass, no rounding) and grad_x comes back in float32. Checked against a run whose x was
    rounded to bfloat16 first (must differ, and by no more than that rounding) and against the float64
    restatement fed the same values."""
    from sru_amd import ElementwiseRecurrence
    from sru_amd.functional import _problem
    c = Case(L=24, B=4, d=128, dirs=2, seed=48, scale=1.7, pad="right")
    dev = "cuda:0"
    t = lambda a, dt=torch.float32, rg=True: torch.tensor(a, dtype=dt, device=dev, requires_grad=rg)
    u = t(c.U, torch.bfloat16)
    x = t(c.x)
    wc, bias, c0 = t(c.wc), t(c.bias), t(c.c0)
    sx = torch.tensor([c.scale], device=dev)
    pad = torch.tensor(c.pad, device=dev)
    assert _problem(u, x, wc, c.d, True, True, 0, checkpoint_state=True).x_float
    h, last = ElementwiseRecurrence.apply(u, x, wc, bias, c0, 0, c.d, True, True, sx, None, pad)
    gh = torch.tensor(c.gh, dtype=torch.bfloat16, device=dev)
    (h * gh).sum().backward()
    assert h.dtype == torch.bfloat16 and x.grad.dtype == torch.float32
    # float64 restatement on the values the kernels saw
    import copy
    c64 = copy.copy(c)
    c64.U, c64.gh = u.detach().double().cpu().numpy(), gh.double().cpu().numpy()
    c64.x = x.detach().double().cpu().numpy()
    c64.gl = np.zeros_like(c.gl)
    for n in ("wc", "bias", "c0"):
        setattr(c64, n, getattr(c, n).astype(np.float32).astype(np.float64))
    c64.scale = float(np.float32(c.scale))
    h_ref, _, g_ref = _apply(st.recurrence, c64, "cpu", torch.float64)
    assert np.abs(h.detach().double().cpu().numpy() - h_ref).max() <= 2e-2 * max(1.0, np.abs(h_ref).max())
    gx = x.grad.double().cpu().numpy()
    assert (np.abs(gx - g_ref[1]) / np.maximum(1.0, np.abs(g_ref[1]))).max() <= 2e-2
    # against the rounded-x run: different, but only by the rounding of x
    x16 = t(c.x, torch.bfloat16)
    h16, _ = ElementwiseRecurrence.apply(u.detach(), x16, wc.detach(), bias.detach(), c0.detach(), 0, c.d, True, True,
                                         sx, None, pad)
    assert not torch.equal(h16, h.detach())
    assert float((h16.float() - h.detach().float()).abs().max()) <= 2e-2 * max(1.0, float(h.detach().float().abs().max()))
