"""Parity at the headline shape (bidirectional, d=1024, L=256, B=64, k=3, float32): the
kernels, through the C ABI, against the float64 oracle on identical inputs, plus
size-independent properties of the domain checked at that size on the GPU alone.

Tolerances: forward outputs 1e-5 absolute; gradient cells 1e-5 * max(1, |reference cell|)
(absolute 1e-5 for every cell of magnitude up to 1, relative 1e-5 for the few larger ones);
the sums over L*B = 16384 terms (grad_wc, grad_bias) 1e-6 * max(1, max|reference|). The test
prints, beside each figure, how far the float32 serial CPU loop itself lands from float64.
"""
import numpy as np
import pytest
import torch

from oracle import sru_oracle as so
from tests.abi import DeviceProblem, to_np
from tests.cases import Case

pytestmark = pytest.mark.gpu

HEADLINE = dict(L=256, B=64, d=1024, dirs=2, k=3)


def _maxerr(a, b):
    d = np.abs(a.reshape(-1) - b.reshape(-1))
    assert not np.isnan(d).any()
    return float(d.max())


def _check_cells(name, got, ref, ref32=None):
    """Per-cell bound: |got - ref| <= 1e-5 * max(1, |ref|). Cells of magnitude <= 1 are held
    to the absolute 1e-5; float32 cannot hold larger values (a few of the 10^8 gradient cells
    reach magnitudes of tens) to an absolute 1e-5, so those are held to 1e-5 relative."""
    got, ref = got.reshape(-1), ref.reshape(-1)
    err = np.abs(got - ref)
    assert not np.isnan(err).any(), name
    worst = float((err / np.maximum(1.0, np.abs(ref))).max())
    line = f"{name}: max abs err {err.max():.3g} (max |ref| {np.abs(ref).max():.3g}), worst scaled {worst:.3g}"
    if ref32 is not None:
        line += f"; float32 CPU loop max abs err {np.abs(ref32.reshape(-1) - ref).max():.3g}"
    print(line)
    assert worst <= 1e-5, line


@pytest.mark.parametrize("checkpointed", [False, True], ids=["state_every_step", "state_checkpoints"])
def test_headline_shape_against_float64_oracle(checkpointed):
    c = Case(seed=51, scale=3 ** 0.5, zero_c0=True, **HEADLINE).f32()
    dp = DeviceProblem(c, checkpointed=checkpointed)
    h, cs, cl = dp.forward()
    h_ref, c_ref, cl_ref = so.forward(*c.fwd_args(), **c.kw())
    print()
    _check_cells("h", to_np(h), h_ref)
    _check_cells("c_last", to_np(cl), cl_ref)
    assert _maxerr(to_np(h), h_ref) <= 1e-5
    if checkpointed:      # rows = states after walk steps 7, 15, ...; second direction walks time backwards
        rows = np.arange(7, c.L, 8)
        expect = np.concatenate([c_ref[rows][..., :c.d], c_ref[c.L - 1 - rows][..., c.d:]], -1)
        _check_cells("state checkpoints", to_np(cs), expect)
        c_used = c_ref
    else:
        _check_cells("c", to_np(cs), c_ref)
        assert _maxerr(to_np(cs), c_ref) <= 1e-5
        c_used = to_np(cs)
    gu, gx, gwc, gb, gi = dp.backward()
    g_ref = so.backward(*c.fwd_args(), c_used, c.gh, c.gl, **c.kw())
    # context: the float32 serial CPU loop (the reference's own arithmetic, forward and backward,
    # working from its own float32 states) against the same float64 result
    kw32 = dict(c.kw(), precision="f32")
    h32, c32, _ = so.forward(*c.fwd_args(), **kw32)
    print(f"float32 CPU loop forward: h max abs err {_maxerr(h32, h_ref):.3g}, c {_maxerr(c32, c_ref):.3g}")
    g32 = so.backward(*c.fwd_args(), c32, c.gh, c.gl, **kw32)
    _check_cells("grad_u", to_np(gu), g_ref[0], g32[0])
    _check_cells("grad_x", to_np(gx), g_ref[1], g32[1])
    _check_cells("grad_init", to_np(gi), g_ref[4], g32[4])
    e_wc, e_b = _maxerr(to_np(gwc), g_ref[2]), _maxerr(to_np(gb), g_ref[3])
    print(f"summed gradients vs float64: kernels grad_wc {e_wc:.3g} grad_bias {e_b:.3g}; "
          f"float32 CPU loop grad_wc {_maxerr(g32[2], g_ref[2]):.3g} grad_bias {_maxerr(g32[3], g_ref[3]):.3g}; "
          f"max|grad_wc| {np.abs(g_ref[2]).max():.3g} max|grad_bias| {np.abs(g_ref[3]).max():.3g}")
    # sums of 16 384 terms reaching magnitudes above 100 (one float32 ulp there is 7.6e-6): held to
    # 1e-6 of the largest sum, ten times tighter than the per-cell rule, which is where the float32
    # CPU loop lands as well
    assert e_wc <= 1e-6 * max(1.0, np.abs(g_ref[2]).max())
    assert e_b <= 1e-6 * max(1.0, np.abs(g_ref[3]).max())


@pytest.mark.parametrize("checkpointed", [False, True], ids=["state_every_step", "state_checkpoints"])
def test_headline_shape_bf16_streams(checkpointed):
    # the two-columns-per-lane kernels (16-bit streams, 65 536 lanes); tolerance 2e-2 * max(1, max|ref|)
    c = Case(seed=55, scale=3 ** 0.5, pad="right", **HEADLINE)
    dp = DeviceProblem(c, "bf16", checkpointed=checkpointed)
    rc = dp.rounded_case()
    h, cs, cl = dp.forward()
    h_ref, c_ref, cl_ref = so.forward(*rc.fwd_args(), **rc.kw())
    rel = lambda got, ref: _maxerr(got, ref) / max(1.0, float(np.abs(ref).max()))
    assert rel(to_np(h), h_ref) <= 2e-2 and rel(to_np(cl), cl_ref) <= 1e-3
    gu, gx, gwc, gb, gi = dp.backward()
    c_used = c_ref if checkpointed else to_np(cs)
    g_ref = so.backward(*rc.fwd_args(), c_used, rc.gh, rc.gl, **rc.kw())
    for got, ref in zip((gu, gx, gwc, gb, gi), g_ref):
        assert rel(to_np(got), ref) <= 2e-2


def _device_case(seed=52, **over):
    kw = dict(HEADLINE, seed=seed, scale=3 ** 0.5, pad="right", mask_c=True)
    kw.update(over)
    return Case(**kw)


def test_headline_shape_properties_on_device():
    c = _device_case()
    dp = DeviceProblem(c)
    h, cs, cl = [t.clone() for t in dp.forward()]
    grads = [t.clone() for t in dp.backward()]
    pad = torch.tensor(c.pad, device=h.device)
    # padded cells: zero output, zero gradient, state carried through
    assert float(h[pad].abs().max()) == 0.0
    assert float(grads[0][pad].abs().max()) == 0.0 and float(grads[1][pad].abs().max()) == 0.0
    lens = torch.tensor(c.lens, device=h.device)
    d = c.d
    last_fwd = cs[(lens - 1), torch.arange(c.B, device=h.device), :d]   # forward direction stops at len-1
    assert torch.equal(last_fwd, cl[:, :d])
    assert torch.equal(cs[0, :, d:], cl[:, d:])                          # backward direction ends at t=0
    # k=4 with U[..., 3] = x * scale must reproduce k=3 (same h, c; grad_u[..., 3] * scale = grad_x)
    c4 = _device_case(k=4)
    c4.U = np.concatenate([c.U.reshape(c.L, c.B, c.Dp, 3), (c.x * np.float32(c.scale))[..., None]], -1)
    c4.U = c4.U.reshape(c.L, c.B, -1)
    for n in ("x", "wc", "bias", "c0", "gh", "gl", "mask_c", "pad", "lens"):
        setattr(c4, n, getattr(c, n))
    dp4 = DeviceProblem(c4)
    h4, cs4, cl4 = dp4.forward()
    # (x * scale is rounded to float32 once in U[..., 3] but stays fused in the k=3 kernel, so
    # h and the gradients agree to rounding, not bit for bit; the state never sees the skip term)
    close = lambda a, b: float(((a - b).abs() / b.abs().clamp(min=1.0)).max()) <= 1e-5
    assert close(h4, h) and float((cs4 - cs).abs().max()) == 0.0
    g4 = dp4.backward()
    gu4 = g4[0].view(c.L, c.B, c.Dp, 4)
    assert close(gu4[..., :3].reshape(grads[0].shape), grads[0])
    assert close(gu4[..., 3] * dp.scale, grads[1])
    assert float((g4[3] - grads[3]).abs().max()) <= 1e-5 * max(1.0, float(grads[3].abs().max()))


def test_headline_shape_bidirectional_equals_two_unidirectional_runs():
    c = _device_case(seed=53)
    dp = DeviceProblem(c)
    h, cs, cl = dp.forward()
    gu, gx, gwc, gb, gi = dp.backward()
    d, L, B = c.d, c.L, c.B
    for di in range(2):
        sel = slice(di * d, (di + 1) * d)
        flip = (lambda a: a[::-1].copy()) if di else (lambda a: a)
        u = Case(L=L, B=B, d=d, dirs=1, k=3, seed=0, scale=c.scale)
        u.U = flip(c.U.reshape(L, B, 2, d, 3)[:, :, di].reshape(L, B, d * 3))
        u.x, u.gh = flip(c.x[..., sel]), flip(c.gh[..., sel])
        u.wc = c.wc.reshape(2, 2, d)[:, di].reshape(-1)
        u.bias = c.bias.reshape(2, 2, d)[:, di].reshape(-1)
        u.c0, u.gl, u.mask_c = c.c0[:, sel], c.gl[:, sel], c.mask_c[:, sel]
        u.pad = flip(c.pad)
        du = DeviceProblem(u)
        h1, c1, cl1 = du.forward()
        g1 = du.backward()
        fl = (lambda t: t.flip(0)) if di else (lambda t: t)
        assert torch.equal(fl(h1), h[..., sel]) and torch.equal(cl1, cl[:, sel])
        assert torch.equal(fl(g1[0]).view(L, B, d, 3), gu.view(L, B, 2, d, 3)[:, :, di])
        assert torch.equal(fl(g1[1]), gx[..., sel])
        assert torch.equal(g1[2].view(2, d), gwc.view(2, 2, d)[:, di])
        assert torch.equal(g1[3].view(2, d), gb.view(2, 2, d)[:, di])
        assert torch.equal(g1[4], gi[:, sel])


def test_long_sequence_inference_shape_fp16():
    # config 5 at reduced batch: bi d=256, L=4096, fp16 streams, forward only, lengths in
    # [1024, 4096], c0 ~ N(0,1); state not stored
    c = Case(L=4096, B=8, d=256, dirs=2, k=3, seed=54, pad="right", scale=1.0)
    dp = DeviceProblem(c, "f16")
    rc = dp.rounded_case()
    h, _, cl = dp.forward(keep_c=False)
    h_ref, _, cl_ref = so.forward(*rc.fwd_args(), **rc.kw())
    assert _maxerr(to_np(h), h_ref) <= 2e-2 * max(1.0, np.abs(h_ref).max())
    assert _maxerr(to_np(cl), cl_ref) <= 1e-3 * max(1.0, np.abs(cl_ref).max())


def test_offsets_beyond_32_bits_long_sequence_k4():
    # config-5 scale with k=4: U has exactly 2^31 elements (4.3 GB in float16), so element and
    # byte offsets leave the 32-bit range. Checked through batch independence: the first and the
    # last batch row of the big run must equal a run on those two rows alone.
    import ctypes
    from sru_amd import _lib
    L, B, d, dirs, k = 4096, 256, 256, 2, 4
    Dp = d * dirs
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(77)
    U = torch.empty(L, B, Dp * k, dtype=torch.float16, device=dev)
    for t0 in range(0, L, 512):
        U[t0:t0 + 512] = torch.randn(512, B, Dp * k, device=dev, generator=g).half()
    assert U.numel() == 2 ** 31
    wc = (torch.rand(2 * Dp, device=dev, generator=g) * 2 - 1)
    bias = torch.randn(2 * Dp, device=dev, generator=g) * 0.3
    c0 = torch.randn(B, Dp, device=dev, generator=g)
    lens = torch.randint(1024, L + 1, (B,), device=dev, generator=g)
    pad = (torch.arange(L, device=dev)[:, None] >= lens[None, :])
    lib = _lib.load()
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())

    def run(U_, c0_, pad_, batch):
        shape = _lib.Shape(L, batch, d, dirs, k, 0, 2, 0, _lib.F16, 1)
        h = torch.full((L, batch, Dp), float("nan"), dtype=torch.float16, device=dev)
        cl = torch.full((batch, Dp), float("nan"), device=dev)
        padb = pad_.contiguous().view(torch.uint8)
        rc = lib.sru_amd_forward(ctypes.byref(shape), p(U_), None, p(wc), p(bias), p(c0_), None, p(padb),
                                 None, p(h), None, p(cl), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, _lib.status_string(rc)
        torch.cuda.synchronize()
        return h, cl

    h_big, cl_big = run(U, c0, pad, B)
    assert not torch.isnan(h_big[-1]).any() and not torch.isnan(h_big[0]).any()
    rows = torch.tensor([0, B - 1], device=dev)
    h_small, cl_small = run(U[:, rows].contiguous(), c0[rows].contiguous(), pad[:, rows], 2)
    # the two runs select different kernels (two columns per lane for the wide one, lane pairs for
    # the narrow one) whose float arithmetic is the same up to the compiler's choice of fused
    # multiply-adds: the final states agree to 1e-6, the float16 outputs to one unit in the last place
    a, b = h_big[:, rows].float(), h_small.float()
    assert float(((a - b).abs() / b.abs().clamp(min=1.0)).max()) <= 2.0 ** -10
    assert float((a != b).float().mean()) <= 1e-3
    assert float((cl_big[rows] - cl_small).abs().max()) <= 1e-6 * max(1.0, float(cl_small.abs().max()))
    assert float(h_big[pad].abs().max()) == 0.0


def test_long_sequence_inference_full_size_k3_fp16():
    """The long-sequence inference workload at its real size: bidirectional, d=256, L=4096, B=256,
    float16 streams, k=3 with the skip term read from x, lengths in [1024, 4096], c0 ~ N(0,1), state
    not stored. Inputs are drawn on the device (as float64 host arrays they would not fit). Checked
    three ways: padded cells are zero; the first and the last batch row equal a run on those two rows
    alone (another kernel: the lane-pair one); and those two rows equal the float64 oracle fed the
    same rounded values."""
    import ctypes
    from sru_amd import _lib
    L, B, d, dirs, k = 4096, 256, 256, 2, 3
    Dp = d * dirs
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(78)
    U = torch.empty(L, B, Dp * k, dtype=torch.float16, device=dev)
    x = torch.empty(L, B, Dp, dtype=torch.float16, device=dev)
    for t0 in range(0, L, 512):
        U[t0:t0 + 512] = torch.randn(512, B, Dp * k, device=dev, generator=g).half()
        x[t0:t0 + 512] = torch.randn(512, B, Dp, device=dev, generator=g).half()
    wc = (torch.rand(2 * Dp, device=dev, generator=g) * 2 - 1)
    bias = torch.randn(2 * Dp, device=dev, generator=g) * 0.3
    c0 = torch.randn(B, Dp, device=dev, generator=g)
    scale = torch.tensor([1.7], device=dev)
    lens = torch.randint(1024, L + 1, (B,), device=dev, generator=g)
    lens[0], lens[B - 1] = L, 1024          # the two rows looked at closely: the longest and the shortest
    pad = (torch.arange(L, device=dev)[:, None] >= lens[None, :])
    lib = _lib.load()
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())

    def run(U_, x_, c0_, pad_, batch):
        shape = _lib.Shape(L, batch, d, dirs, k, 0, 1, 0, _lib.F16, 1)
        h = torch.full((L, batch, Dp), float("nan"), dtype=torch.float16, device=dev)
        cl = torch.full((batch, Dp), float("nan"), device=dev)
        padb = pad_.contiguous().view(torch.uint8)
        rc = lib.sru_amd_forward(ctypes.byref(shape), p(U_), p(x_), p(wc), p(bias), p(c0_), None, p(padb),
                                 p(scale), p(h), None, p(cl), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, _lib.status_string(rc)
        torch.cuda.synchronize()
        return h, cl

    h_big, cl_big = run(U, x, c0, pad, B)
    assert not torch.isnan(h_big).any() and not torch.isnan(cl_big).any()
    assert float(h_big[pad].abs().max()) == 0.0
    rows = torch.tensor([0, B - 1], device=dev)
    U2, x2, c02, pad2 = U[:, rows].contiguous(), x[:, rows].contiguous(), c0[rows].contiguous(), pad[:, rows]
    h_small, cl_small = run(U2, x2, c02, pad2, 2)
    # two kernels whose float arithmetic agrees up to the compiler's choice of fused multiply-adds:
    # final states to 1e-6, float16 outputs to one unit in the last place in a few cells
    a, b = h_big[:, rows].float(), h_small.float()
    assert float(((a - b).abs() / b.abs().clamp(min=1.0)).max()) <= 2.0 ** -10
    assert float((a != b).float().mean()) <= 5e-3
    assert float((cl_big[rows] - cl_small).abs().max()) <= 1e-6 * max(1.0, float(cl_small.abs().max()))
    # the same two rows against the float64 oracle
    n = lambda t: t.double().cpu().numpy()
    h_ref, _, cl_ref = so.forward(n(U2), n(x2), n(wc), n(bias), n(c02), d=d, dirs=dirs, k=k, activation_type=0,
                                  skip_type=1, is_custom=0, scale_x=float(scale.item()), mask_c=None,
                                  mask_pad=pad2.cpu().numpy())
    assert _maxerr(n(h_big[:, rows]), h_ref) <= 2e-2 * max(1.0, np.abs(h_ref).max())
    assert _maxerr(n(cl_big[rows]), cl_ref) <= 1e-3 * max(1.0, np.abs(cl_ref).max())


@pytest.mark.parametrize("checkpointed", [False, True], ids=["state_every_step", "state_checkpoints"])
@pytest.mark.parametrize("k", [3, 4])
def test_long_sequence_training_against_float64_oracle(checkpointed, k):
    """2048 steps (256 checkpoint chunks, plus a ragged tail of 5): errors of the recomputed
    states must not build up along the walk. Same per-cell bounds as at the headline shape."""
    c = Case(L=2053, B=3, d=96, dirs=2, k=k, seed=61, scale=1.7 if k == 3 else None, pad="right",
             mask_c=True).f32()
    dp = DeviceProblem(c, checkpointed=checkpointed)
    h, cs, cl = dp.forward()
    h_ref, c_ref, cl_ref = so.forward(*c.fwd_args(), **c.kw())
    print()
    _check_cells("h", to_np(h), h_ref)
    _check_cells("c_last", to_np(cl), cl_ref)
    gu, gx, gwc, gb, gi = dp.backward()
    c_used = c_ref if checkpointed else to_np(cs)
    g_ref = so.backward(*c.fwd_args(), c_used, c.gh, c.gl, **c.kw())
    _check_cells("grad_u", to_np(gu), g_ref[0])
    if k == 3:
        _check_cells("grad_x", to_np(gx), g_ref[1])
    _check_cells("grad_init", to_np(gi), g_ref[4])
    assert _maxerr(to_np(gwc), g_ref[2]) <= 1e-5 * max(1.0, np.abs(g_ref[2]).max())
    assert _maxerr(to_np(gb), g_ref[3]) <= 1e-5 * max(1.0, np.abs(g_ref[3]).max())
