"""sru_amd_backward_static, the backward entry point that takes no workspace and allocates
nothing (its partial sums live in an array built into the library's device code), against
sru_amd_backward on the same inputs: the two run the same kernels, so every output must be
bit-identical. Two calls in a row share the built-in array; the second is smaller, so it finds
the first call's leftovers there."""
import ctypes

import pytest
import torch

from sru_amd import _lib
from tests.abi import DeviceProblem, p
from tests.cases import Case

pytestmark = pytest.mark.gpu


def _static_backward(dp):
    c = dp.case
    nan = lambda *s, dtype: torch.full(s, float("nan"), dtype=dtype, device=dp.dev)
    gu = nan(c.L, c.B, c.Dp * c.k, dtype=dp.tdt)
    gx = nan(c.L, c.B, c.Dp, dtype=dp.tdt) if c.skip_type == 1 else None
    gwc = nan(c.L, c.B, c.Dp * 2, dtype=dp.tdt) if c.custom else nan(2 * c.Dp, dtype=dp.sdt)
    gb = nan(2 * c.Dp, dtype=dp.sdt)
    gi = nan(c.B, c.Dp, dtype=dp.sdt)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dp.dev).cuda_stream)
    rc = _lib.load().sru_amd_backward_static(
        ctypes.byref(dp.shape), p(dp.U), p(dp.x) if c.skip_type == 1 else None, p(dp.wc), p(dp.bias),
        p(dp.c0), p(dp.mask_c), p(dp.pad), p(dp.scale) if c.skip_type == 1 else None, p(dp.c), p(dp.gh),
        p(dp.gl), p(gu), p(gx), p(gwc), p(gb), p(gi), stream)
    assert rc == 0, _lib.status_string(rc)
    return gu, gx, gwc, gb, gi


@pytest.mark.parametrize("dt,checkpointed", [("f32", True), ("f32", False), ("bf16", True), ("f64", False)])
def test_static_backward_equals_workspace_backward_on_two_calls_in_a_row(dt, checkpointed):
    big = Case(L=40, B=16, d=256, dirs=2, seed=91, pad="right", scale=1.7, mask_c=True)
    small = Case(L=19, B=3, d=70, dirs=2, k=4, seed=92, pad="random")
    for case in (big, small):     # the second, smaller call reuses the array the first one filled
        dp = DeviceProblem(case, dt, checkpointed=checkpointed)
        dp.forward()
        expect = [None if t is None else t.clone() for t in dp.backward()]
        got = _static_backward(dp)
        torch.cuda.synchronize()
        for a, b in zip(got, expect):
            assert (a is None) == (b is None)
            if a is not None:
                assert not torch.isnan(a.float()).any()
                assert torch.equal(a, b)


def test_static_backward_per_step_weight_c_and_headline_width():
    # the general kernels, and the widest reference shape (131 072 columns) at a short length
    for case in (Case(L=12, B=3, d=64, dirs=2, custom=True, seed=93, pad="right"),
                 Case(L=9, B=64, d=1024, dirs=2, seed=94, scale=1.7)):
        dp = DeviceProblem(case, "f32", checkpointed=not case.custom)
        dp.forward()
        expect = [None if t is None else t.clone() for t in dp.backward()]
        for a, b in zip(_static_backward(dp), expect):
            if a is not None:
                assert torch.equal(a, b)


def test_static_backward_rejects_more_columns_than_its_array_holds():
    lib = _lib.load()
    fake = ctypes.c_void_p(0x1000)      # never dereferenced: the size check comes first
    cols = _lib.STATIC_MAX_COLUMNS
    too_wide = _lib.Shape(4, cols // 1024 + 1, 1024, 1, 3, 0, 1, 0, _lib.F32, 8)
    assert lib.sru_amd_backward_static(ctypes.byref(too_wide), *([fake] * 16), None) == 8
    assert "262144" in _lib.status_string(8)
    # double partial sums fill the array with half as many columns
    half = _lib.Shape(4, cols // 2048 + 1, 1024, 1, 3, 0, 1, 0, _lib.F64, 1)
    assert lib.sru_amd_backward_static(ctypes.byref(half), *([fake] * 16), None) == 8
    bad = _lib.Shape(0, 1, 8, 1, 3, 0, 1, 0, _lib.F32, 8)
    assert lib.sru_amd_backward_static(ctypes.byref(bad), *([fake] * 16), None) == 2
