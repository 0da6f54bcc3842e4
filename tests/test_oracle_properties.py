"""Closed forms and invariants that fix the oracle where no stored vector does.

Each one is chosen so that a plausible slip (a dropped term, a swapped gate, a
wrong time index for the second direction, a pad that leaks) breaks it.
"""
import numpy as np
import pytest

from oracle import sru_oracle as so
from tests.cases import Case


def test_weight_c_zero_closed_form():
    # With weight_c = 0 (the reference's v1 mode, sru/modules.py:231-233) the gates do not
    # depend on the state: c_t = c0*prod_{r<=t} f_r + sum_s (1-f_s) u0_s prod_{s<r<=t} f_r.
    c = Case(L=11, B=3, d=4, seed=3)
    c.wc[:] = 0
    h, c_all, _ = so.forward(*c.fwd_args(), **c.kw())
    U = c.U.reshape(c.L, c.B, c.Dp, 3)
    f = 1 / (1 + np.exp(-(U[..., 1] + c.bias[:c.Dp])))
    r = 1 / (1 + np.exp(-(U[..., 2] + c.bias[c.Dp:])))
    P = np.cumprod(f, 0)
    expect = c.c0 * P + P * np.cumsum((1 - f) * U[..., 0] / P, 0)
    assert np.abs(c_all - expect).max() < 1e-10
    assert np.abs(h - (r * expect + (1 - r) * c.x)).max() < 1e-10


def test_saturated_gates():
    c = Case(L=6, B=2, d=3, seed=4, scale=1.5)
    U = c.U.reshape(c.L, c.B, c.Dp, 3)
    big = 200.0
    U[..., 1] = -big  # forget gate 0: c_t = u0_t
    U[..., 2] = -big  # output gate 0: h = x * scale
    h, c_all, _ = so.forward(*c.fwd_args(), **c.kw())
    assert np.abs(c_all - U[..., 0]).max() < 1e-12
    assert np.abs(h - c.x * 1.5).max() < 1e-12
    U[..., 1] = big   # forget gate 1: state frozen at c0
    U[..., 2] = big   # output gate 1: h = c
    h, c_all, cl = so.forward(*c.fwd_args(), **c.kw())
    assert np.abs(c_all - c.c0[None]).max() < 1e-12 and np.abs(cl - c.c0).max() < 1e-12
    assert np.abs(h - c.c0[None]).max() < 1e-12


@pytest.mark.parametrize("k", [3, 4])
def test_bidirectional_is_two_unidirectional_runs(k):
    c = Case(L=9, B=3, d=4, dirs=2, k=k, seed=6, pad="random", mask_c=True, scale=1.2)
    h, c_all, cl = so.forward(*c.fwd_args(), **c.kw())
    gu, gx, gwc, gb, gi = so.backward(*c.fwd_args(), c_all, c.gh, c.gl, **c.kw())
    d = c.d
    U5 = c.U.reshape(c.L, c.B, 2, d, k)
    for di in range(2):
        flip = (lambda a: a[::-1].copy()) if di else (lambda a: a)
        sel = slice(di * d, (di + 1) * d)
        kw = dict(c.kw(), dirs=1, mask_c=c.mask_c[:, sel], mask_pad=flip(c.pad))
        wc = c.wc.reshape(2, 2, d)[:, di].reshape(-1)
        bias = c.bias.reshape(2, 2, d)[:, di].reshape(-1)
        args = (flip(U5[:, :, di].reshape(c.L, c.B, d * k)), flip(c.x[..., sel]), wc, bias, c.c0[:, sel])
        h1, c1, cl1 = so.forward(*args, **kw)
        assert np.array_equal(flip(h1), h[..., sel])
        assert np.array_equal(cl1, cl[:, sel])
        g1 = so.backward(*args, c1, flip(c.gh[..., sel]), c.gl[:, sel], **kw)
        assert np.allclose(flip(g1[0]).reshape(c.L, c.B, d, k), gu.reshape(c.L, c.B, 2, d, k)[:, :, di], atol=1e-13)
        if k == 3:
            assert np.allclose(flip(g1[1]), gx[..., sel], atol=1e-13)
        assert np.allclose(g1[2].reshape(2, d), gwc.reshape(2, 2, d)[:, di], atol=1e-12)
        assert np.allclose(g1[3].reshape(2, d), gb.reshape(2, 2, d)[:, di], atol=1e-12)
        assert np.allclose(g1[4], gi[:, sel], atol=1e-13)


@pytest.mark.parametrize("dirs", [1, 2])
def test_right_padding_equals_truncated_sequences(dirs):
    # sru/csrc/sru_cuda_kernel.cu:61,:72 and sru/ops.py:230-231,:245-246
    c = Case(L=10, B=4, d=3, dirs=dirs, seed=8, pad="right", scale=1.3)
    h, c_all, cl = so.forward(*c.fwd_args(), **c.kw())
    gu, gx, gwc, gb, gi = so.backward(*c.fwd_args(), c_all, c.gh, c.gl, **c.kw())
    gwc_sum, gb_sum = np.zeros_like(gwc), np.zeros_like(gb)
    for b in range(c.B):
        n = int(c.lens[b])
        kw = dict(c.kw(), mask_pad=None)
        args = (c.U[:n, b:b + 1], c.x[:n, b:b + 1], c.wc, c.bias, c.c0[b:b + 1])
        h1, c1, cl1 = so.forward(*args, **kw)
        assert np.array_equal(h1[:, 0], h[:n, b])
        assert np.all(h[n:, b] == 0)
        assert np.array_equal(cl1[0], cl[b])
        g1 = so.backward(*args, c1, c.gh[:n, b:b + 1], c.gl[b:b + 1], **kw)
        assert np.array_equal(g1[0][:, 0], gu[:n, b]) and np.all(gu[n:, b] == 0)
        assert np.array_equal(g1[1][:, 0], gx[:n, b]) and np.all(gx[n:, b] == 0)
        assert np.array_equal(g1[4][0], gi[b])
        gwc_sum += g1[2]
        gb_sum += g1[3]
    assert np.allclose(gwc_sum, gwc, atol=1e-12) and np.allclose(gb_sum, gb, atol=1e-12)


def test_padded_inputs_do_not_leak_and_empty_mask_is_no_mask():
    # misc/test_sru.py:34-42: changing a padded token leaves the output bit-identical
    c = Case(L=8, B=3, d=4, dirs=2, seed=10, pad="random", mask_c=True)
    out = so.forward(*c.fwd_args(), **c.kw())
    grads = so.backward(*c.fwd_args(), out[1], c.gh, c.gl, **c.kw())
    U2, x2, gh2 = c.U.copy(), c.x.copy(), c.gh.copy()
    U2[c.pad] = np.nan
    x2[c.pad] = 1e30
    gh2[c.pad] = np.inf
    out2 = so.forward(U2, x2, c.wc, c.bias, c.c0, **c.kw())
    grads2 = so.backward(U2, x2, c.wc, c.bias, c.c0, out2[1], gh2, c.gl, **c.kw())
    for a, b in zip(out + grads, out2 + grads2):
        assert np.array_equal(a, b)
    for g in (grads[0], grads[1]):
        assert np.all(g[c.pad] == 0)
    e = Case(L=8, B=3, d=4, dirs=2, seed=10, pad="none_mask")
    a = so.forward(*e.fwd_args(), **e.kw())
    b = so.forward(*e.fwd_args(), **dict(e.kw(), mask_pad=None))
    assert all(np.array_equal(p, q) for p, q in zip(a, b))


@pytest.mark.parametrize("dirs", [1, 2])
def test_k4_with_scaled_x_in_fourth_stream_equals_k3(dirs):
    c = Case(L=7, B=2, d=3, dirs=dirs, seed=12, scale=1.6, mask_c=True, pad="random")
    U4 = np.concatenate([c.U.reshape(c.L, c.B, c.Dp, 3), (c.x * c.scale)[..., None]], -1).reshape(c.L, c.B, -1)
    kw4 = dict(c.kw(), k=4, skip_type=2)
    h3, c3, cl3 = so.forward(*c.fwd_args(), **c.kw())
    h4, c4, cl4 = so.forward(U4, c.x, c.wc, c.bias, c.c0, **kw4)
    assert np.array_equal(h3, h4) and np.array_equal(c3, c4)
    g3 = so.backward(*c.fwd_args(), c3, c.gh, c.gl, **c.kw())
    g4 = so.backward(U4, c.x, c.wc, c.bias, c.c0, c4, c.gh, c.gl, **kw4)
    gu4 = g4[0].reshape(c.L, c.B, c.Dp, 4)
    assert np.array_equal(gu4[..., :3].reshape(g3[0].shape), g3[0])
    assert np.allclose(gu4[..., 3] * c.scale, g3[1], atol=1e-14)
    assert g4[1] is None
    for i in (2, 3, 4):
        assert np.array_equal(g3[i], g4[i])


def test_broadcast_per_step_v_equals_vector_weight_c():
    # misc/test_impl.py:85-96: layout (2, dirs, d) -> (dirs, d, 2)
    c = Case(L=6, B=3, d=4, dirs=2, seed=13, pad="random")
    V = np.broadcast_to(c.wc.reshape(2, c.Dp).T[None, None], (c.L, c.B, c.Dp, 2)).copy()
    a = so.forward(*c.fwd_args(), **c.kw())
    b = so.forward(c.U, c.x, V, c.bias, c.c0, **dict(c.kw(), is_custom=1))
    assert all(np.array_equal(p, q) for p, q in zip(a, b))
    ga = so.backward(*c.fwd_args(), a[1], c.gh, c.gl, **c.kw())
    gb = so.backward(c.U, c.x, V, c.bias, c.c0, b[1], c.gh, c.gl, **dict(c.kw(), is_custom=1))
    assert np.allclose(gb[2].sum((0, 1)).T.reshape(-1), ga[2], atol=1e-12)
    for i in (0, 1, 3, 4):
        assert np.array_equal(ga[i], gb[i])


def test_batch_independence_and_scale_mask_linearity():
    # test/sru/test_sru.py:68-72: a batched run equals per-sample runs
    c = Case(L=6, B=4, d=3, dirs=2, seed=14, mask_c=True, scale=1.25)
    h, c_all, cl = so.forward(*c.fwd_args(), **c.kw())
    for b in range(c.B):
        kw = dict(c.kw(), mask_c=c.mask_c[b:b + 1])
        h1, _, cl1 = so.forward(c.U[:, b:b + 1], c.x[:, b:b + 1], c.wc, c.bias, c.c0[b:b + 1], **kw)
        assert np.array_equal(h1[:, 0], h[:, b]) and np.array_equal(cl1[0], cl[b])
    # scale_x only ever multiplies x (sru/cuda_functional.py:76)
    h2, _, _ = so.forward(c.U, c.x * c.scale, c.wc, c.bias, c.c0, **dict(c.kw(), scale_x=1.0))
    assert np.allclose(h, h2, atol=1e-14)
    # the state never sees mask_c (sru/csrc/sru_cuda_kernel.cu:69-70)
    _, c_nomask, _ = so.forward(*c.fwd_args(), **dict(c.kw(), mask_c=None))
    assert np.array_equal(c_all, c_nomask)
