"""One hop from the HIP kernels to what the reference itself holds: the committed vectors are
fed to sru_amd_forward through the C ABI and its output is compared with the stored reference
output directly, at the reference's own tolerance (no oracle in between).

* tests/golden/cpu_ref_vectors.npz: outputs of the reference's CPU routine
  (sru/csrc/sru_cpu_impl.cpp compiled from its source), float32, bound 2e-6;
* tests/golden/regression_2.3.5.npz: the reference's golden vector
  test/regression/artifacts/2.3.5.pt, bound 1e-6 as in
  test/regression/test_regression.py:13,:50-51. U = x @ weight is formed on the CPU in
  float32, as the artifact was, so only the recurrence runs on the GPU.
"""
import os

import numpy as np
import pytest

from tests.abi import DeviceProblem, to_np
from tests.cases import Case

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def _names():
    z = np.load(os.path.join(HERE, "golden", "cpu_ref_vectors.npz"))
    return [str(n) for n in z["names"]]


def _case(L, B, d, dirs, k, act, skip, custom, U, x, wc, bias, c0, scale, pad):
    c = Case(L=L, B=B, d=d, dirs=dirs, k=k, act=act, skip=bool(skip), custom=bool(custom))
    f = lambda a: np.asarray(a, np.float64)
    c.U, c.x, c.wc, c.bias, c.c0 = f(U), f(x), f(wc), f(bias), f(c0)
    c.scale, c.pad, c.mask_c = float(scale), pad, None
    return c


@pytest.mark.parametrize("state", ["every_step", "checkpoints", "none"])
@pytest.mark.parametrize("name", _names())
def test_cpu_routine_vectors_on_the_kernels(name, state):
    z = np.load(os.path.join(HERE, "golden", "cpu_ref_vectors.npz"))
    L, B, d, dirs, k, act, skip, custom = [int(v) for v in z[name + "/cfg"]]
    fast = (skip or k == 3) and not (custom and act)
    if state == "checkpoints" and not fast:
        pytest.skip("checkpointed state exists for the fast layouts only")
    pad = z[name + "/pad"] if name + "/pad" in z.files else None
    c = _case(L, B, d, dirs, k, act, skip, custom, z[name + "/U"], z[name + "/x"], z[name + "/wc"],
              z[name + "/bias"], z[name + "/c0"], z[name + "/scale"], pad)
    dp = DeviceProblem(c, "f32", checkpointed=(state == "checkpoints"))
    h, _, c_last = dp.forward(keep_c=(state != "none"))
    assert np.abs(to_np(h) - z[name + "/h"]).max() <= 2e-6
    assert np.abs(to_np(c_last) - z[name + "/c"]).max() <= 2e-6


@pytest.mark.parametrize("state", ["every_step", "checkpoints", "none"])
def test_regression_artifact_2_3_5_recurrence_on_the_kernels(state):
    z = np.load(os.path.join(HERE, "golden", "regression_2.3.5.npz"))
    d = int(z["kwargs/hidden_size"])
    x = z["inputs"]
    L, B, _ = x.shape
    finals = []
    for layer in range(2):
        w = z[f"state/rnn_lst.{layer}.weight"]
        k = w.shape[1] // (2 * d)
        U = (x.reshape(L * B, -1) @ w).astype(np.float32).reshape(L, B, -1)
        c = _case(L, B, d, 2, k, 0, True, False, U, x if k == 3 else np.zeros((L, B, 2 * d)),
                  z[f"state/rnn_lst.{layer}.weight_c"], z[f"state/rnn_lst.{layer}.bias"],
                  np.zeros((B, 2 * d)), 1.0, None)
        dp = DeviceProblem(c, "f32", checkpointed=(state == "checkpoints"))
        h, _, c_last = dp.forward(keep_c=(state != "none"))
        x = to_np(h).astype(np.float32)
        finals.append(to_np(c_last))
    assert np.abs(x - z["out_h"]).max() <= 1e-6
    assert np.abs(np.stack(finals) - z["out_c"]).max() <= 1e-6
