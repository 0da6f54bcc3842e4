"""The layer-norm kernels (csrc/sru_norm.hip) through sru_amd.norm against
torch.nn.functional.layer_norm in float64 on the same (rounded) inputs.

Tolerances: float32 in and out: 2e-6 * max(1, |cell|) on y, 1e-5 * max(1, |cell|) on grad_x, the
row-summed weight / bias gradients 1e-6 * max(1, max|ref|) per 1000 rows summed; a 16-bit output
or input adds its own rounding: 2^-8 (bfloat16) or 2^-11 (float16) relative per cell."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from sru_amd.norm import LayerNormFunction, layer_norm, supported

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ULP = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


def _check(rows_shape, D, in_dt, out_dt, seed=0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = (torch.randn(*rows_shape, D, device=DEV, generator=g) * 1.7 + 0.4).to(in_dt)
    w = torch.randn(D, device=DEV, generator=g)
    b = torch.randn(D, device=DEV, generator=g)
    x.requires_grad_(True), w.requires_grad_(True), b.requires_grad_(True)
    y = layer_norm(x, w, b, 1e-5, out_dt)
    assert y.dtype == out_dt and y.shape == x.shape
    probe = torch.randn(y.shape, device=DEV, generator=g).to(out_dt)
    y.backward(probe)
    xr = x.detach().double().requires_grad_(True)
    wr, br = w.detach().double().requires_grad_(True), b.detach().double().requires_grad_(True)
    yr = F.layer_norm(xr, (D,), wr, br, 1e-5)
    yr.backward(probe.double())
    cell = lambda a, r: float(((a.double() - r).abs() / r.abs().clamp(min=1.0)).max())
    assert cell(y.detach(), yr.detach()) <= 2e-6 + ULP[out_dt]
    assert x.grad.dtype == in_dt
    assert cell(x.grad, xr.grad) <= 1e-5 + ULP[in_dt]
    rows = x.numel() // D
    for got, ref in ((w.grad, wr.grad), (b.grad, br.grad)):
        assert got.dtype == torch.float32
        tol = 1e-6 * max(1.0, rows / 1000) * max(1.0, float(ref.abs().max()))
        assert float((got.double() - ref).abs().max()) <= tol


@pytest.mark.parametrize("in_dt", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("out_dt", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [8, 64, 520, 1024, 2048])
def test_against_float64_layer_norm(D, in_dt, out_dt):
    _check((7, 5), D, in_dt, out_dt, seed=D)


@pytest.mark.parametrize("shape,D", [((1,), 512), ((3, 1), 776), ((4099,), 1024), ((2, 3), 4096), ((5000,), 2048)])
def test_row_counts_and_feature_counts(shape, D):
    _check(shape, D, torch.float32, torch.float32, seed=3)
    _check(shape, D, torch.bfloat16, torch.bfloat16, seed=4)


def test_config_3_rows_bf16_in_and_out_and_float_in_bf16_out():
    # what the layers of the classification-scale stack see under bf16 autocast: 16 384 rows of 2048
    _check((256, 64), 2048, torch.bfloat16, torch.bfloat16, seed=5)
    _check((256, 64), 1024, torch.float32, torch.bfloat16, seed=6)


def test_backward_is_bit_reproducible_and_padded_rows_are_independent():
    g = torch.Generator(device=DEV).manual_seed(9)
    x = torch.randn(3000, 1024, device=DEV, generator=g, requires_grad=True)
    w = torch.randn(1024, device=DEV, generator=g, requires_grad=True)
    b = torch.randn(1024, device=DEV, generator=g, requires_grad=True)
    probe = torch.randn(3000, 1024, device=DEV, generator=g)
    outs = []
    for _ in range(3):
        for t in (x, w, b):
            t.grad = None
        y = layer_norm(x, w, b)
        y.backward(probe)
        outs.append([y.detach().clone(), x.grad.clone(), w.grad.clone(), b.grad.clone()])
    for later in outs[1:]:
        assert all(torch.equal(p, q) for p, q in zip(outs[0], later))
    # a row's output depends on that row only
    y1 = layer_norm(x[5:6].detach(), w.detach(), b.detach())
    assert torch.equal(y1[0], outs[0][0][5])


def test_unsupported_shapes_take_torch_layer_norm():
    x = torch.randn(4, 6, 7, device=DEV)          # 7 features: not a multiple of 8
    assert not supported(x) and supported(torch.randn(4, 16, device=DEV))
    w, b = torch.randn(7, device=DEV), torch.randn(7, device=DEV)
    with pytest.warns(UserWarning, match="no kernel for"):       # the second path is never silent
        y = layer_norm(x, w, b)
    assert torch.allclose(y, F.layer_norm(x, (7,), w, b), atol=1e-6)
    with pytest.raises(ValueError, match="no kernel for"):
        layer_norm(x, w, b, strict=True)
    with pytest.raises(ValueError):
        layer_norm(torch.randn(4, 16, device=DEV), torch.randn(16, device=DEV), torch.randn(16, device=DEV),
                   out_dtype=torch.float64)
    # float64 rows: torch's kernel in double; parameters of the wrong size never reach a kernel
    xd = torch.randn(4, 16, device=DEV, dtype=torch.float64)
    wd, bd = torch.randn(16, device=DEV, dtype=torch.float64), torch.randn(16, device=DEV, dtype=torch.float64)
    with pytest.warns(UserWarning, match="no kernel for"):
        yd = layer_norm(xd, wd, bd)
    assert yd.dtype == torch.float64 and torch.allclose(yd, F.layer_norm(xd, (16,), wd, bd), atol=1e-12)
    with pytest.raises(ValueError, match="needs weight and bias"):
        layer_norm(torch.randn(4, 16, device=DEV), torch.randn(8, device=DEV), torch.randn(16, device=DEV))


def test_module_uses_the_kernels_and_emits_the_autocast_dtype_before_the_projection(monkeypatch):
    from sru_amd.modules import SRUCell
    calls = []
    real = LayerNormFunction.apply
    monkeypatch.setattr(LayerNormFunction, "apply", staticmethod(lambda *a: (calls.append(a[-1]), real(*a))[1]))
    torch.manual_seed(2)
    cell = SRUCell(64, 64, layer_norm=True).to(DEV)
    x = torch.randn(9, 3, 64, device=DEV)
    h32, _ = cell(x)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        h16, _ = cell(x)
    assert calls == [torch.float32, torch.bfloat16]
    assert float((h16.float() - h32).abs().max()) <= 2e-2 * max(1.0, float(h32.abs().max()))
    ref = F.layer_norm(x, (64,), cell.layer_norm.weight, cell.layer_norm.bias)
    assert torch.allclose(layer_norm(x, cell.layer_norm.weight, cell.layer_norm.bias), ref, atol=2e-6)
