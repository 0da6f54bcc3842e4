"""Pins the oracle's analytic backward (nothing in the reference holds a golden
vector for it).

* torch.autograd.gradcheck (float64) on the differentiable restatement of the
  forward equations, whose forward is itself tied to the C oracle here;
* the C backward equals autograd of that restatement for every flag combination
  -- the cross-check the reference's own test_sru_backward performs between its
  CPU autograd path and its GPU kernels (test/sru/test_sru.py:128-162, 1e-4);
* central finite differences of the C forward on tiny problems, so a mistake
  shared by both restatements would still show.
"""
import numpy as np
import pytest
import torch

from oracle import sru_oracle as so
from oracle import sru_torch as st
from tests.cases import GRID, Case


def _torch_inputs(c, requires_grad=True):
    t = lambda a: torch.tensor(a, dtype=torch.float64, requires_grad=requires_grad)
    wc = t(c.wc)
    args = [t(c.U), t(c.x), wc, t(c.bias), t(c.c0)]
    sx = torch.tensor([c.scale], dtype=torch.float64)
    mc = None if c.mask_c is None else torch.tensor(c.mask_c, dtype=torch.float64)
    pad = None if c.pad is None else torch.tensor(c.pad)
    return args, (c.act, c.d, c.dirs == 2, c.skip_type != 0, sx, mc, pad)


@pytest.mark.parametrize("cfg", GRID, ids=lambda g: "-".join(f"{k}{v}" for k, v in g.items()))
def test_c_backward_equals_autograd(cfg):
    c = Case(seed=11, **cfg)
    args, rest = _torch_inputs(c)
    h, last = st.recurrence(*args, *rest)
    hn, c_all, cl = so.forward(*c.fwd_args(), **c.kw())
    assert np.abs(hn - h.detach().numpy().reshape(hn.shape)).max() < 1e-12
    assert np.abs(cl - last.detach().numpy()).max() < 1e-12
    ((h.reshape(c.L, c.B, c.Dp) * torch.tensor(c.gh)).sum() + (last * torch.tensor(c.gl)).sum()).backward()
    gu, gx, gwc, gb, gi = so.backward(*c.fwd_args(), c_all, c.gh, c.gl, **c.kw())
    assert np.abs(gu - args[0].grad.numpy()).max() < 1e-11
    if c.skip_type == 1:
        assert np.abs(gx - args[1].grad.numpy()).max() < 1e-11
    else:
        assert gx is None
        assert args[1].grad is None or float(args[1].grad.abs().max()) == 0.0
    assert np.abs(gwc - args[2].grad.numpy().reshape(gwc.shape)).max() < 1e-11
    assert np.abs(gb - args[3].grad.numpy()).max() < 1e-11
    assert np.abs(gi - args[4].grad.numpy()).max() < 1e-11


@pytest.mark.parametrize("cfg", [
    dict(L=3, B=2, d=2, dirs=2, pad="random", mask_c=True, scale=1.4),
    dict(L=3, B=2, d=2, k=4, act=1),
    dict(L=3, B=1, d=2, custom=True, dirs=2),
    dict(L=2, B=2, d=2, skip=False, act=1),
])
def test_gradcheck_of_restatement(cfg):
    c = Case(seed=5, **cfg)
    args, rest = _torch_inputs(c)
    if c.skip_type != 1:
        args[1] = args[1].detach()
    assert torch.autograd.gradcheck(lambda *a: st.recurrence(*a, *rest), args, eps=1e-6, atol=1e-7)


@pytest.mark.parametrize("cfg", [
    dict(L=4, B=2, d=3, dirs=2, pad="random", mask_c=True, scale=1.4),
    dict(L=3, B=2, d=2, k=4, dirs=2, act=1),
    dict(L=3, B=1, d=2, custom=True),
])
def test_c_backward_equals_finite_differences_of_c_forward(cfg):
    c = Case(seed=9, **cfg)
    kw = c.kw()

    def loss(U, x, wc, bias, c0):
        h, _, cl = so.forward(U, x, wc, bias, c0, **kw)
        return float((h * c.gh).sum() + (cl * c.gl).sum())

    _, c_all, _ = so.forward(*c.fwd_args(), **kw)
    grads = so.backward(*c.fwd_args(), c_all, c.gh, c.gl, **kw)
    base = [a.copy() for a in c.fwd_args()]
    eps = 1e-6
    for idx, g in enumerate(grads):
        if g is None:
            continue
        flat = base[idx].reshape(-1)
        gflat = g.reshape(-1) if idx != 0 else g.reshape(-1)
        rng = np.random.default_rng(idx)
        for pos in rng.choice(flat.size, size=min(12, flat.size), replace=False):
            keep = flat[pos]
            flat[pos] = keep + eps
            up = loss(*base)
            flat[pos] = keep - eps
            dn = loss(*base)
            flat[pos] = keep
            assert abs((up - dn) / (2 * eps) - gflat[pos]) < 1e-6, (idx, pos)
