"""CPU-only checks of the layer wrapper: constructor rules, parameter names and shapes
(state_dict compatibility with the reference), the initialisation recipe, error behaviour."""
import math
import os

import numpy as np
import pytest
import torch

from sru_amd.modules import SRU, SRUCell

HERE = os.path.dirname(os.path.abspath(__file__))


def test_loads_the_reference_state_dict_of_the_regression_artifact():
    z = np.load(os.path.join(HERE, "golden", "regression_2.3.5.npz"))
    kwargs = {k.split("/", 1)[1]: z[k].item() for k in z.files if k.startswith("kwargs/")}
    model = SRU(**kwargs)
    state = {k.split("/", 1)[1]: torch.tensor(z[k]) for k in z.files if k.startswith("state/")}
    assert set(model.state_dict()) == set(state)
    model.load_state_dict(state, strict=True)
    assert model.rnn_lst[0].num_matrices == 4 and model.rnn_lst[1].num_matrices == 3
    assert model.rnn_lst[0].dropout == pytest.approx(0.1) and model.rnn_lst[1].dropout == 0


@pytest.mark.parametrize("kw,keys", [
    (dict(input_size=8, hidden_size=8), {"weight", "weight_c", "bias", "scale_x"}),
    (dict(input_size=16, hidden_size=8, n_proj=4),
     {"weight", "weight_proj", "weight_c", "bias", "scale_x"}),
    (dict(input_size=8, hidden_size=8, layer_norm=True),
     {"weight", "weight_c", "bias", "scale_x", "layer_norm.weight", "layer_norm.bias"}),
])
def test_cell_parameter_names(kw, keys):
    assert set(SRUCell(**kw).state_dict()) == keys


def test_shape_rules():
    # k = 4 only when there is a skip term that cannot be the input itself (sru/modules.py:131-133)
    assert SRUCell(8, 8).num_matrices == 3
    assert SRUCell(8, 4, bidirectional=True).num_matrices == 3
    assert SRUCell(8, 8, bidirectional=True).num_matrices == 4
    assert SRUCell(6, 8, has_skip_term=False).num_matrices == 3
    # projection only when it is a bottleneck (sru/modules.py:126-128)
    assert SRUCell(16, 8, n_proj=8).projection_size == 0
    assert SRUCell(16, 8, n_proj=4).weight.shape == (4, 32)   # 16 != 8: four streams
    assert SRUCell(16, 8, n_proj=4).weight_proj.shape == (16, 4)
    cell = SRUCell(6, 5, bidirectional=True)
    assert cell.weight.shape == (6, 40) and cell.weight_c.shape == (20,) and cell.bias.shape == (20,)
    stack = SRU(6, 5, num_layers=3, bidirectional=True, dropout=0.2, proj_input_to_hidden_first=True)
    assert stack.input_to_hidden.weight.shape == (10, 6)
    assert [c.input_size for c in stack.rnn_lst] == [10, 10, 10]
    assert [c.dropout for c in stack.rnn_lst] == [0.2, 0.2, 0.0]
    # defaults differ between the two classes (sru/modules.py:41 vs :444)
    assert SRUCell(4, 4).rescale is True and SRU(4, 4).rnn_lst[0].rescale is False


def test_initialisation_recipe():
    torch.manual_seed(0)
    d = 256
    cell = SRUCell(d, d, highway_bias=-2.0, rescale=True)
    w = cell.weight.detach().view(d, 1, d, 3)
    assert abs(float(w[..., 0].var()) * d - 1.0) < 0.05          # Var = 1/d
    assert abs(float(w[..., 1].var()) * d - 0.5) < 0.03          # gate columns * sqrt(0.5)
    assert abs(float(w[..., 2].var()) * d - 0.5) < 0.03
    assert abs(float(cell.weight_c.var()) - 0.5) < 0.08          # Var = 1 then * 0.5
    assert torch.all(cell.bias[:d] == 0) and torch.all(cell.bias[d:] == -2.0)
    assert float(cell.scale_x) == pytest.approx(math.sqrt(1 + 2 * math.exp(-2.0)))
    assert float(SRUCell(d, d, rescale=False).scale_x) == 1.0
    # k = 4 with rescale: the fourth stream carries the scale (sru/modules.py:208-210)
    c4 = SRUCell(d, 2 * d, highway_bias=0.0, rescale=True)
    w4 = c4.weight.detach().view(d, 1, 2 * d, 4)
    assert abs(float(w4[..., 3].var()) * d - 3.0) < 0.15
    # layer norm shrinks the weights, dropout rescales the candidate stream
    cl = SRUCell(d, d, layer_norm=True, dropout=0.5)
    wl = cl.weight.detach().view(d, 1, d, 3)
    assert abs(float(wl[..., 0].var()) * d - 0.01 * 0.5) < 0.001
    v1 = SRUCell(d, d, v1=True)
    assert torch.all(v1.weight_c == 0) and not v1.weight_c.requires_grad
    assert float(SRUCell(d, d, weight_c_init=0.01).weight_c.abs().max()) <= 0.01


def test_error_behaviour():
    cell, stack = SRUCell(4, 4), SRU(4, 4)
    with pytest.raises(ValueError):
        cell(torch.zeros(2, 2, 2, 4))
    with pytest.raises(ValueError):
        stack(torch.zeros(3, 4))
    with pytest.raises(ValueError):
        stack(torch.zeros(3, 2, 4), c0=torch.zeros(2, 4))
    with pytest.raises(RuntimeError):          # no CPU path for the recurrence
        stack(torch.zeros(3, 2, 4))

    class Bad(torch.nn.Module):
        def forward(self, x):
            return x
    with pytest.raises(ValueError):
        SRUCell(4, 4, custom_m=Bad()).compute_UV(torch.zeros(3, 2, 4), None, None)


def test_repr_follows_the_reference_format():
    # sru/modules.py:384-419
    assert repr(SRUCell(8, 8)) == "SRUCell(8, 8, rescale=True)"
    cell = SRUCell(16, 8, dropout=0.1, rnn_dropout=0.2, bidirectional=True, n_proj=4, use_tanh=True,
                   highway_bias=-1.0, has_skip_term=False, layer_norm=True, rescale=False, v1=True)
    assert repr(cell) == ("SRUCell(16, 8, projection_size=4, dropout=0.1, rnn_dropout=0.2, bidirectional=True, "
                          "highway_bias=-1.0, activation=tanh, v1=True, rescale=False, has_skip_term=False, "
                          "layer_norm=True)")
    with_m = SRUCell(4, 4, custom_m=torch.nn.Linear(4, 12, bias=False))
    assert repr(with_m) == ("SRUCell(4, 4, rescale=True,\n  custom_m=Linear(in_features=4, out_features=12, "
                            "bias=False)\n)")
    assert "SRUCell(4, 4, rescale=False)" in repr(SRU(4, 4))


def _drop(module, name):
    """Removes an attribute wherever nn.Module keeps it (plain attribute or sub-module slot)."""
    if name in module._modules:
        del module._modules[name]
    else:
        module.__dict__.pop(name, None)


def test_make_backward_compatible():
    # sru/modules.py:660-689: attribute names of releases <= 2.1.7 and <= 2.1.9
    model = SRU(6, 5, num_layers=2, bidirectional=True, projection_size=2)
    # an object as release 2.1.7 pickled it: old names only
    old = SRU(6, 5, num_layers=2, bidirectional=True, projection_size=2)
    old.n_in, old.n_out, old.out_size, old.depth, old.n_proj = 6, 5, 10, 2, 2
    old.ln_lst, old.use_weight_norm = [], False
    for name in ("input_size", "hidden_size", "output_size", "num_layers", "projection_size", "use_layer_norm",
                 "nn_rnn_compatible_return"):
        delattr(old, name)
    _drop(old, "input_to_hidden")
    for cell in old.rnn_lst:
        cell.n_in, cell.n_out, cell.k, cell.n_proj = cell.input_size, cell.hidden_size, cell.num_matrices, 2
        for name in ("input_size", "hidden_size", "output_size", "num_matrices", "projection_size", "custom_m",
                     "layer_norm"):
            _drop(cell, name)
    old.make_backward_compatible()
    for name in ("input_size", "hidden_size", "output_size", "num_layers", "projection_size"):
        assert getattr(old, name) == getattr(model, name), name
    assert old.use_layer_norm is False and old.nn_rnn_compatible_return is False
    assert old.input_to_hidden is None
    for cell, new in zip(old.rnn_lst, model.rnn_lst):
        for name in ("input_size", "hidden_size", "output_size", "num_matrices", "projection_size"):
            assert getattr(cell, name) == getattr(new, name), name
        assert cell.layer_norm is None and cell.custom_m is None
    # what cannot be carried over is refused
    old.use_weight_norm = True
    with pytest.raises(Exception, match="Weight norm"):
        old.make_backward_compatible()
    old.use_weight_norm, old.ln_lst = False, [1]
    with pytest.raises(Exception, match="Layer norm"):
        old.make_backward_compatible()
    old.ln_lst = []
    old.rnn_lst[0].activation_type = 2
    with pytest.raises(Exception, match="ReLU or SeLU"):
        old.make_backward_compatible()
    # a current object passes through unchanged
    before = dict(model.__dict__)
    model.make_backward_compatible()
    assert {k: v for k, v in model.__dict__.items() if k != "_modules"} == \
        {k: v for k, v in before.items() if k != "_modules"}


def test_large_stack_restatement_equals_the_python_loop_restatement():
    # tests/stack_ref.py: the float64 stack built on the C oracle (used at sizes where the Python
    # loop is too slow) must agree with the one built on the differentiable torch loop
    from tests.stack_ref import stack_forward, stack_forward_large
    torch.manual_seed(4)
    model = SRU(6, 8, num_layers=3, bidirectional=True, layer_norm=True, rescale=True, projection_size=3,
                dropout=0.2)
    x = torch.randn(9, 4, 6)
    pad = torch.arange(9)[:, None] >= torch.tensor([9, 4, 7, 1])[None, :]
    h1, c1, p1 = stack_forward(model, x, mask_pad=pad)
    h2, c2, p2 = stack_forward_large(model, x, mask_pad=pad, device="cpu")
    probe = torch.randn(h1.shape, dtype=torch.float64)
    (h1 * probe).sum().backward()
    (h2 * probe).sum().backward()
    assert float((h1 - h2).abs().max()) <= 1e-12 and float((c1 - c2).abs().max()) <= 1e-12
    for n in p1:
        assert float((p1[n].grad - p2[n].grad).abs().max()) <= 1e-10 * max(1.0, float(p1[n].grad.abs().max())), n
