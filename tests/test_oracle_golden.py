"""Pins the oracle's forward against what the reference itself holds.

* the reference's only golden vector, test/regression/artifacts/2.3.5.pt
  (tolerance 1e-6 as in test/regression/test_regression.py:13,:50-51), replayed
  as U = x @ weight -> recurrence for two bidirectional layers (k=4 then k=3);
* vectors produced by the reference's CPU routine compiled from its source
  (sru/csrc/sru_cpu_impl.cpp), committed under tests/golden/ and, where
  oracle/_ref is present, recomputed live at other seeds and sizes.
"""
import os

import numpy as np
import pytest
import torch

from oracle import sru_oracle as so

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SO = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "libsru_cpu_ref.so")


@pytest.mark.parametrize("precision", ["f32", "f64"])
def test_regression_artifact_2_3_5(precision):
    z = np.load(os.path.join(HERE, "golden", "regression_2.3.5.npz"))
    assert str(z["version"]) == "2.3.5"
    d = int(z["kwargs/hidden_size"])
    assert bool(z["kwargs/bidirectional"]) and int(z["kwargs/num_layers"]) == 2
    x = z["inputs"]
    L, B, _ = x.shape
    c_fin = []
    for layer in range(2):
        w = z[f"state/rnn_lst.{layer}.weight"]
        k = w.shape[1] // (2 * d)
        assert k == (4 if layer == 0 else 3)
        U = (x.reshape(L * B, -1) @ w).astype(np.float32).reshape(L, B, -1)
        # rescale=False: the module passes scale_x=None (sru/modules.py:262)
        h, _, cl = so.forward(U, x, z[f"state/rnn_lst.{layer}.weight_c"],
                              z[f"state/rnn_lst.{layer}.bias"], np.zeros((B, 2 * d), np.float32),
                              d=d, dirs=2, k=k, skip_type=1 if k == 3 else 2, precision=precision)
        x = h.astype(np.float32)
        c_fin.append(cl)
    assert np.abs(x - z["out_h"]).max() <= 1e-6
    assert np.abs(np.stack(c_fin) - z["out_c"]).max() <= 1e-6


def _fixture_cases():
    z = np.load(os.path.join(HERE, "golden", "cpu_ref_vectors.npz"))
    return z, [str(n) for n in z["names"]]


@pytest.mark.parametrize("name", _fixture_cases()[1])
def test_cpu_routine_vectors(name):
    z, _ = _fixture_cases()
    L, B, d, dirs, k, act, skip, custom = [int(v) for v in z[name + "/cfg"]]
    pad = z[name + "/pad"] if name + "/pad" in z.files else None
    skip_type = 0 if not skip else (1 if k == 3 else 2)
    for precision, tol in (("f32", 2e-6), ("f64", 2e-6)):
        h, _, cl = so.forward(z[name + "/U"], z[name + "/x"], z[name + "/wc"], z[name + "/bias"],
                              z[name + "/c0"], d=d, dirs=dirs, k=k, activation_type=act,
                              skip_type=skip_type, is_custom=custom, scale_x=float(z[name + "/scale"]),
                              mask_pad=pad, precision=precision)
        assert np.abs(h - z[name + "/h"]).max() <= tol, precision
        assert np.abs(cl - z[name + "/c"]).max() <= tol, precision


@pytest.mark.skipif(not os.path.exists(REF_SO), reason="oracle/_ref not built")
@pytest.mark.parametrize("dirs", [1, 2])
@pytest.mark.parametrize("k", [3, 4])
@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("pad", [False, True])
def test_live_against_compiled_reference_cpu_routine(dirs, k, act, pad):
    torch.ops.load_library(REF_SO)
    g = torch.Generator().manual_seed(7 + dirs * 8 + k * 2 + act)
    L, B, d = 33, 5, 37
    Dp = d * dirs
    U = torch.randn(L, B, Dp * k, generator=g)
    x = torch.randn(L, B, Dp, generator=g)
    wc = torch.randn(2 * Dp, generator=g)
    bias = torch.randn(2 * Dp, generator=g)
    c0 = torch.randn(B, Dp, generator=g)
    mask = (torch.rand(L, B, generator=g) < 0.25) if pad else None
    fn = torch.ops.sru_cpu.cpu_bi_forward if dirs == 2 else torch.ops.sru_cpu.cpu_forward
    h_ref, c_ref = fn(U, x, wc, bias, c0, mask, L, B, d, k, act, True, 1.25, False)
    h, _, cl = so.forward(U.numpy(), x.numpy(), wc.numpy(), bias.numpy(), c0.numpy(), d=d, dirs=dirs,
                          k=k, activation_type=act, skip_type=1 if k == 3 else 2, scale_x=1.25,
                          mask_pad=None if mask is None else mask.numpy(), precision="f32")
    assert np.abs(h - h_ref.numpy()).max() <= 2e-6
    assert np.abs(cl - c_ref.numpy()).max() <= 2e-6
