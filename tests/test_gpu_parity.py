"""GPU parity of the HIP kernels, called through the C ABI, against the CPU oracle.

Tolerances (the bar the build is held to):
  float32 streams : max abs error <= 1e-5 for h, c, c_last against the float64 oracle on
                    identical inputs; gradient cells (grad_u, grad_x, grad_init)
                    <= 1e-5 * max(1, |reference cell|), i.e. absolute 1e-5 up to magnitude 1
                    and relative 1e-5 for the few larger cells; the batch/time-summed
                    grad_wc and grad_bias <= 1e-5 * max(1, max|reference|) (float32 cannot
                    hold a large value or a sum of L*B terms to an absolute 1e-5; the
                    float32 CPU loop itself does not at the large shapes).
  float16 / bfloat16 streams : against the float64 oracle fed the same rounded inputs: h, c
                    max abs error <= 2e-2 * max(1, max|reference|); gradient cells
                    <= 2e-2 * max(1, |reference cell|) (per cell, so a wrong small cell cannot hide
                    behind a large one); the summed grad_wc / grad_bias <= 2e-2 * max(1, max|reference|).
  float64 streams : everything is computed in double; the same comparisons with 1e-12 in the place
                    of 1e-5 (the double exp of the device library against the host's).
Outputs are pre-filled with NaN: a cell the kernels do not write fails the comparison.
"""
import os

import numpy as np
import pytest
import torch

from oracle import sru_oracle as so
from tests.abi import DeviceProblem, to_np
from tests.cases import GRID, Case

pytestmark = pytest.mark.gpu

F32_ABS = 1e-5
F64_ABS = 1e-12
HALF_REL = 2e-2


def _err(a, b):
    assert a.shape == b.shape or a.size == b.size
    d = np.abs(a.reshape(-1) - b.reshape(-1))
    assert not np.isnan(d).any(), "unwritten or NaN cells"
    return float(d.max()) if d.size else 0.0


def _scale(ref):
    return max(1.0, float(np.abs(ref).max()))


def _cell_err(a, b):
    """max over cells of |a - b| / max(1, |b|)"""
    a, b = a.reshape(-1), b.reshape(-1)
    d = np.abs(a - b) / np.maximum(1.0, np.abs(b))
    assert not np.isnan(d).any(), "unwritten or NaN cells"
    return float(d.max()) if d.size else 0.0


def check_against_oracle(case, dt="f32", keep_c=True, checkpointed=False, x_f32=False):
    """checkpointed: the state travels from forward to backward as float checkpoints every
    SRU_AMD_STATE_INTERVAL steps and the backward kernel rebuilds the rest.
    x_f32: x and grad_x are float32 beside the 16-bit streams."""
    dp = DeviceProblem(case, dt, checkpointed=checkpointed, x_f32=x_f32)
    rc = dp.rounded_case()
    h, c, c_last = dp.forward(keep_c=keep_c)
    h_ref, c_ref, cl_ref = so.forward(*rc.fwd_args(), **rc.kw())
    exact = {"f32": F32_ABS, "f64": F64_ABS}.get(dt)   # absolute bar of the float and double streams
    tol = (lambda ref: exact) if exact else (lambda ref: HALF_REL * _scale(ref))
    assert _err(to_np(h), h_ref) <= tol(h_ref)
    assert _err(to_np(c_last), cl_ref) <= (exact or 1e-3 * _scale(cl_ref))
    if not keep_c:
        return
    if checkpointed:
        # rows of the checkpoint array are states after walk steps 7, 15, ... (second direction: walk
        # step s is time L-1-s); the backward kernel works from the exact float states
        T, d = 8, case.d
        for r in range(case.L // T):
            s_ = (r + 1) * T - 1
            expect = np.concatenate([c_ref[s_, :, :d], c_ref[case.L - 1 - s_, :, d:]], -1) if case.dirs == 2 \
                else c_ref[s_]
            assert _err(to_np(c[r]), expect) <= (exact or 1e-3 * _scale(expect))
        c_used = c_ref
    else:
        assert _err(to_np(c), c_ref) <= tol(c_ref)
        c_used = to_np(c)
    # backward from the state the device stored (what a training step does)
    gu, gx, gwc, gb, gi = dp.backward()
    g_ref = so.backward(*rc.fwd_args(), c_used, rc.gh, rc.gl, **rc.kw())
    # gradient cells, every stream type: error relative to max(1, |that cell|)
    cell_tol = exact or HALF_REL
    assert _cell_err(to_np(gu), g_ref[0]) <= cell_tol
    if case.skip_type == 1:
        assert _cell_err(to_np(gx), g_ref[1]) <= cell_tol
    sum_tol = (lambda ref: (exact or HALF_REL) * _scale(ref))
    if case.custom:
        assert _cell_err(to_np(gwc), g_ref[2]) <= cell_tol
    else:
        assert _err(to_np(gwc), g_ref[2]) <= sum_tol(g_ref[2])
    assert _err(to_np(gb), g_ref[3]) <= sum_tol(g_ref[3])
    assert _cell_err(to_np(gi), g_ref[4]) <= cell_tol


_ids = lambda g: "-".join(f"{k}{v}" for k, v in g.items())


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("cfg", GRID, ids=_ids)
def test_small_grid(cfg, dt):
    check_against_oracle(Case(seed=21, **cfg), dt)


# shapes that exercise whole wavefronts, ragged tails, both loop phases and odd ring fills
MID = [
    dict(L=1, B=3, d=64, dirs=2),
    dict(L=7, B=2, d=128, dirs=2, pad="right", scale=1.7),
    dict(L=8, B=2, d=64),
    dict(L=15, B=3, d=64, dirs=2, pad="random", mask_c=True),
    dict(L=16, B=2, d=96, dirs=2, k=4, pad="right"),
    dict(L=17, B=5, d=50, dirs=2, scale=1.3, pad="right"),
    dict(L=33, B=4, d=192, k=4),
    dict(L=40, B=3, d=130, pad="random"),
    dict(L=64, B=8, d=256, dirs=2, pad="right", scale=1.7, mask_c=True),
    dict(L=25, B=2, d=64, dirs=2, custom=True, pad="right"),
    dict(L=25, B=2, d=64, dirs=2, act=1, k=4),
    dict(L=19, B=3, d=128, dirs=2, act=1, pad="right", scale=1.3, mask_c=True),
    dict(L=33, B=2, d=70, act=1, pad="random"),
    dict(L=25, B=2, d=64, skip=False, pad="random"),
]


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("cfg", MID, ids=_ids)
def test_mid_shapes(cfg, dt):
    check_against_oracle(Case(seed=22, **cfg), dt)


@pytest.mark.parametrize("cfg", GRID + MID, ids=_ids)
def test_double_streams(cfg):
    # the general kernels computing in double: streams, small tensors, state, sums
    check_against_oracle(Case(seed=23, **cfg), "f64")


def test_double_streams_without_state_store():
    # the inference variant (c == NULL) of the double kernels: same h and last state, bit for bit
    c = Case(L=19, B=3, d=70, dirs=2, seed=27, pad="right", scale=1.3, mask_c=True)
    dp = DeviceProblem(c, "f64")
    h, _, c_last = [t.clone() if t is not None else None for t in dp.forward(keep_c=True)]
    h2, none, c_last2 = dp.forward(keep_c=False)
    assert none is None and torch.equal(h, h2) and torch.equal(c_last, c_last2)


def test_double_streams_refuse_checkpoints():
    dp = DeviceProblem(Case(L=9, B=2, d=8, seed=1), "f64", checkpointed=True)
    import ctypes
    from sru_amd import _lib
    assert _lib.load().sru_amd_state_bytes(ctypes.byref(dp.shape)) == 0   # bad flags: no size


# every layout that can keep its state as checkpoints: all but four streams without a skip term and
# a per-step weight_c together with tanh
FAST = [g for g in GRID + MID if (g.get("skip", True) or g.get("k", 3) == 3)
        and not (g.get("custom") and g.get("act"))]
FAST += [dict(L=21, B=3, d=64, dirs=2, custom=True, k=4, pad="right"),
         dict(L=33, B=2, d=70, custom=True, pad="random", mask_c=True, scale=1.3),
         dict(L=17, B=4, d=128, dirs=2, custom=True, skip=False),
         dict(L=40, B=2, d=192, custom=True, scale=0.7)]


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("cfg", FAST, ids=_ids)
def test_checkpointed_state(cfg, dt):
    if dt != "f32" and cfg["d"] % 2:
        pytest.skip("16-bit streams keep checkpoints for an even d only")
    check_against_oracle(Case(seed=24, **cfg), dt, checkpointed=True)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("checkpointed", [False, True])
def test_two_columns_per_lane_without_wave_uniformity(dt, checkpointed):
    # 16-bit streams, >= 65 536 lanes at two columns per lane, d not a multiple of 128: the
    # two-column kernels with per-lane direction / row arithmetic
    c = Case(L=21, B=70, d=992, dirs=2, seed=25, pad="right", scale=1.7, mask_c=True)
    assert c.B * c.Dp // 2 >= 65536 and c.d % 128 != 0
    check_against_oracle(c, dt, checkpointed=checkpointed)


# 16-bit streams, two columns per lane, every fast layout and activation, with per-lane
# direction / row arithmetic (d % 128 != 0) and at least 65 536 lanes, both passes
WIDE = [
    dict(k=3), dict(k=3, pad="right"), dict(k=4), dict(k=4, pad="random"), dict(k=3, act=1, pad="right"),
    dict(k=4, act=1), dict(k=3, skip=False), dict(k=3, skip=False, act=1, pad="random"),
]


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("cfg", WIDE, ids=_ids)
def test_two_columns_per_lane_every_fast_layout(cfg, dt):
    kw = dict(L=9, B=128, d=1030, dirs=1, seed=26, mask_c=True)
    kw.update(cfg)
    if kw["k"] == 3 and kw.get("skip", True):
        kw["scale"] = 1.7
    c = Case(**kw)
    assert c.B * c.Dp // 2 >= 65536 and c.d % 128 != 0
    for checkpointed in (False, True):
        check_against_oracle(c, dt, checkpointed=checkpointed)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_inference_variant_without_state_store(dt):
    check_against_oracle(Case(L=40, B=4, d=128, dirs=2, seed=23, pad="right", scale=1.7), dt, keep_c=False)
    check_against_oracle(Case(L=9, B=2, d=5, dirs=2, k=4, seed=23), dt, keep_c=False)


def test_reference_config_1_readme_example_layer():
    # 2-layer uni SRU, input=hidden=128, L=20, B=32, highway_bias=-2 (README.md example)
    c = Case(L=20, B=32, d=128, seed=31, zero_c0=True, gate_bias=-2.0)
    check_against_oracle(c.f32(), "f32")


def test_reference_config_2_shape_with_lengths():
    # bi d=512, L=128, B=32, right-padded lengths; layer 0 is k=4, the others k=3
    check_against_oracle(Case(L=128, B=32, d=512, dirs=2, k=4, seed=32, pad="right", zero_c0=True).f32())
    check_against_oracle(Case(L=128, B=32, d=512, dirs=2, k=3, seed=33, pad="right", zero_c0=True).f32())
    check_against_oracle(Case(L=128, B=32, d=512, dirs=2, k=4, seed=32, pad="right", zero_c0=True).f32(),
                         checkpointed=True)
    check_against_oracle(Case(L=128, B=32, d=512, dirs=2, k=3, seed=33, pad="right", zero_c0=True).f32(),
                         checkpointed=True)


def test_padded_cells_cannot_leak_bit_identical():
    # misc/test_sru.py:34-42 at kernel level, forward and backward
    c = Case(L=24, B=4, d=128, dirs=2, seed=34, pad="random", mask_c=True, scale=1.7)
    a = DeviceProblem(c)
    out_a = [t.clone() for t in a.forward()] + [t.clone() for t in a.backward()]
    c2 = Case(L=24, B=4, d=128, dirs=2, seed=34, pad="random", mask_c=True, scale=1.7)
    c2.U[c2.pad] = np.nan
    c2.x[c2.pad] = 1e30
    c2.gh[c2.pad] = np.inf
    b = DeviceProblem(c2)
    out_b = list(b.forward()) + list(b.backward())
    for p, q in zip(out_a, out_b):
        assert torch.equal(p, q)
    pad = torch.tensor(c.pad, device="cuda:0")
    assert float(out_a[0][pad].abs().max()) == 0.0      # h
    assert float(out_a[3][pad].abs().max()) == 0.0      # grad_u
    assert float(out_a[4][pad].abs().max()) == 0.0      # grad_x


@pytest.mark.parametrize("dt,checkpointed", [("f32", False), ("f32", True), ("bf16", True), ("f16", True)])
def test_backward_is_bit_reproducible(dt, checkpointed):
    # repeated backward calls on one state buffer: the batch sums are added in a fixed order, and the
    # backward call leaves the state buffer as it found it
    for cfg in (dict(L=50, B=16, d=256, dirs=2, pad="right"), dict(L=23, B=5, d=96, dirs=1, k=4),
                dict(L=9, B=1, d=64, dirs=2, mask_c=True)):
        c = Case(seed=35, **cfg)
        a = DeviceProblem(c, dt, checkpointed=checkpointed)
        a.forward()
        first = [None if t is None else t.clone() for t in a.backward()]
        for _ in range(3):
            again = a.backward()
            assert all(p is None or torch.equal(p, q) for p, q in zip(first, again))


def _random_cases(n, seed):
    """Seeded draw over everything the boundary accepts: sizes around the wavefront, pair and
    chunk boundaries, both directions, every flag combination the shape check allows."""
    rng = np.random.default_rng(seed)
    to_double = np.random.default_rng(seed + 1)   # (its own stream: the other draws stay what they were)
    out = []
    for i in range(n):
        k = int(rng.choice([3, 4]))
        skip = bool(rng.random() < 0.85)
        cfg = dict(L=int(rng.choice([1, 2, 7, 8, 9, 15, 16, 17, 23, 24, 31, 40])),
                   B=int(rng.integers(1, 6)),
                   d=int(rng.choice([1, 2, 3, 31, 32, 33, 63, 64, 65, 96, 127, 128, 130, 192])),
                   dirs=int(rng.choice([1, 2])), k=k, skip=skip,
                   act=int(rng.random() < 0.2), custom=bool(rng.random() < 0.15),
                   pad=[None, "right", "random"][int(rng.integers(0, 3))],
                   mask_c=bool(rng.random() < 0.4),
                   scale=float(rng.choice([1.0, 0.6, 1.7])) if (k == 3 and skip) else None,
                   zero_c0=bool(rng.random() < 0.3))
        dt = ["f32", "f16", "bf16"][int(rng.integers(0, 3))]
        ckpt = bool(rng.random() < 0.5)
        if to_double.random() < 0.15:     # double streams: state after every step only
            dt, ckpt = "f64", False
        out.append((cfg, dt, ckpt, 1000 + i))
    return out


# SRU_AMD_RANDOM_CASES / SRU_AMD_RANDOM_SEED widen or move the draw for a one-off sweep
@pytest.mark.parametrize("cfg,dt,checkpointed,seed",
                         _random_cases(int(os.environ.get("SRU_AMD_RANDOM_CASES", "60")),
                                       int(os.environ.get("SRU_AMD_RANDOM_SEED", "2024"))),
                         ids=lambda v: _ids(v) if isinstance(v, dict) else str(v))
def test_random_draws_over_shapes_and_flags(cfg, dt, checkpointed, seed):
    fast = (cfg["skip"] or cfg["k"] == 3) and not (cfg["custom"] and cfg["act"]) and not (dt != "f32" and cfg["d"] % 2)
    check_against_oracle(Case(seed=seed, **cfg), dt, checkpointed=checkpointed and fast)


@pytest.mark.parametrize("checkpointed", [False, True])
@pytest.mark.parametrize("act", [0, 1])
def test_saturated_gates_stay_finite(checkpointed, act):
    """Gate inputs of magnitude up to 1e4: the sigmoids are exactly 0 or 1 in float, exp2
    overflows to infinity inside them, and neither pass may turn that into NaN."""
    c = Case(L=24, B=3, d=64, dirs=2, seed=88, scale=1.3, pad="right", act=act)
    rng = np.random.default_rng(5)
    big = rng.choice([-1e4, -100.0, 100.0, 1e4], size=c.U.shape)
    hit = rng.random(c.U.shape) < 0.3
    hit.reshape(c.L, c.B, c.Dp, c.k)[..., 0] = False      # gate streams only; u0 stays moderate
    c.U = np.where(hit, big, c.U)
    check_against_oracle(c.f32(), "f32", checkpointed=checkpointed)


def _windowed_mask(L, B, kind, rng):
    """Masks whose padding sits at the ends of the sequences, where the wave-uniform kernels skip
    whole chunks of 8 steps: every batch row gets a live span [lo, hi) of its own."""
    pad = np.ones((L, B), bool)
    for b in range(B):
        if kind == "right":
            lo, hi = 0, int(rng.integers(1, L + 1))
        elif kind == "left":
            lo, hi = int(rng.integers(0, L)), L
        elif kind == "both":
            lo = int(rng.integers(0, L - 1))
            hi = int(rng.integers(lo + 1, L + 1))
        elif kind == "chunk_edges":            # spans that start and end on multiples of 8
            lo = 8 * int(rng.integers(0, L // 8))
            hi = min(L, lo + 8 * int(rng.integers(1, L // 8 + 1)))
        else:                                  # "holes": live ends, padding inside the span too
            lo, hi = int(rng.integers(0, L // 2)), int(rng.integers(L // 2 + 1, L + 1))
        pad[lo:hi, b] = False
        if kind == "holes":
            inner = rng.random(hi - lo) < 0.4
            inner[0] = inner[-1] = False
            pad[lo:hi, b] |= inner
    if kind in ("both", "holes"):
        pad[:, B - 1] = True                   # one batch row with no live step at all
    return pad


@pytest.mark.parametrize("dt,checkpointed", [("f32", False), ("f32", True), ("bf16", True), ("f16", False)])
@pytest.mark.parametrize("kind", ["right", "left", "both", "chunk_edges", "holes"])
@pytest.mark.parametrize("L", [64, 45])
def test_padding_at_the_ends_of_sequences_is_skipped_exactly(L, kind, dt, checkpointed):
    rng = np.random.default_rng(L + len(kind))
    for cfg in (dict(B=5, d=128, dirs=2), dict(B=3, d=256, dirs=1, k=4), dict(B=4, d=128, dirs=2, mask_c=True, scale=1.7)):
        c = Case(L=L, seed=61, **cfg)
        c.pad = _windowed_mask(L, c.B, kind, rng)
        check_against_oracle(c, dt, checkpointed=checkpointed)
    c = Case(L=L, B=4, d=128, dirs=2, seed=62)
    c.pad = _windowed_mask(L, 4, kind, rng)
    check_against_oracle(c, dt, keep_c=False)


@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_long_right_padded_rows_forward_only_and_training(dt):
    """Many chunks per row, lengths spread over a wide range (the shape class of the L=4096
    inference configuration, shortened): most wavefronts skip a long tail or head of padding."""
    rng = np.random.default_rng(77)
    c = Case(L=523, B=6, d=128, dirs=2, seed=63, scale=1.7)
    lens = rng.integers(131, 524, c.B)
    lens[0], lens[1] = 523, 1
    c.pad = np.arange(c.L)[:, None] >= lens[None, :]
    check_against_oracle(c, dt, keep_c=False)
    check_against_oracle(c, dt, checkpointed=True)



FLOAT_X = [
    dict(L=21, B=3, d=64, dirs=2, scale=1.7),                             # lane pairs, wave-uniform
    dict(L=40, B=4, d=70, dirs=2, pad="right", scale=1.3, mask_c=True),   # lane pairs, wavefronts straddle rows
    dict(L=17, B=2, d=6, pad="random"),                                   # less than a wavefront
    dict(L=19, B=64, d=1024, dirs=2, pad="right", scale=1.7),             # two columns per lane (131 072 columns)
    dict(L=12, B=1100, d=70, dirs=2, pad="random", scale=0.8),            # two columns per lane, straddling rows
]


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("cfg", FLOAT_X, ids=_ids)
def test_float_x_beside_16bit_streams(cfg, dt):
    """x stays float32 while U, h and grad_h are 16-bit (shape.x_dtype = SRU_AMD_X_F32): training with
    checkpoints, and inference without a state store. Same bounds as the 16-bit runs; grad_x comes
    back in float32 and is held per cell."""
    c = Case(seed=47, **cfg)
    check_against_oracle(c, dt, checkpointed=True, x_f32=True)
    check_against_oracle(c, dt, keep_c=False, x_f32=True)
