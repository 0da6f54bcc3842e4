"""Seeded op-level inputs shared by the oracle tests and the GPU parity tests."""
import numpy as np


class Case:
    """One recurrence problem in the reference's layouts, as float64 numpy arrays."""

    def __init__(self, L, B, d, dirs=1, k=3, act=0, skip=True, custom=False, pad=None,
                 mask_c=False, scale=None, zero_c0=False, seed=0, gate_bias=0.0):
        rng = np.random.default_rng(seed)
        self.L, self.B, self.d, self.dirs, self.k = L, B, d, dirs, k
        self.act, self.custom = act, int(custom)
        self.skip_type = 0 if not skip else (1 if k == 3 else 2)
        Dp = d * dirs
        self.Dp = Dp
        self.U = rng.standard_normal((L, B, Dp * k))
        self.x = rng.standard_normal((L, B, Dp))
        self.wc = (rng.standard_normal((L, B, Dp * 2)) if custom
                   else rng.uniform(-1.5 ** 0.5, 1.5 ** 0.5, 2 * Dp))
        self.bias = rng.standard_normal(2 * Dp) * 0.5
        self.bias[Dp:] += gate_bias
        self.c0 = np.zeros((B, Dp)) if zero_c0 else rng.standard_normal((B, Dp))
        self.scale = 1.0 if scale is None else float(scale)
        self.mask_c = None
        if mask_c:
            self.mask_c = (rng.random((B, Dp)) < 0.8) / 0.8
        self.pad = None
        if pad == "right":
            lens = rng.integers(max(1, L // 4), L + 1, B)
            self.lens = lens
            self.pad = np.arange(L)[:, None] >= lens[None, :]
        elif pad == "random":
            self.pad = rng.random((L, B)) < 0.3
        elif pad == "none_mask":
            self.pad = np.zeros((L, B), bool)
        self.gh = rng.standard_normal((L, B, Dp))
        self.gl = rng.standard_normal((B, Dp))

    def kw(self):
        return dict(d=self.d, dirs=self.dirs, k=self.k, activation_type=self.act,
                    skip_type=self.skip_type, is_custom=self.custom, scale_x=self.scale,
                    mask_c=self.mask_c, mask_pad=self.pad)

    def fwd_args(self):
        return (self.U, self.x, self.wc, self.bias, self.c0)

    def f32(self):
        """Round every real input to float32 in place (values stay float64 arrays)."""
        for n in ("U", "x", "wc", "bias", "c0", "gh", "gl"):
            setattr(self, n, getattr(self, n).astype(np.float32).astype(np.float64))
        if self.mask_c is not None:
            self.mask_c = self.mask_c.astype(np.float32).astype(np.float64)
        self.scale = float(np.float32(self.scale))
        return self


GRID = [
    dict(L=1, B=1, d=1),
    dict(L=7, B=3, d=5),
    dict(L=7, B=3, d=5, dirs=2),
    dict(L=6, B=2, d=4, k=4),
    dict(L=6, B=2, d=4, k=4, dirs=2, pad="random"),
    dict(L=9, B=4, d=3, dirs=2, pad="right", scale=1.7, mask_c=True),
    dict(L=8, B=3, d=4, pad="random", mask_c=True, scale=0.6),
    dict(L=5, B=2, d=3, skip=False),
    dict(L=5, B=2, d=3, skip=False, dirs=2, act=1, pad="random"),
    dict(L=6, B=3, d=4, act=1, scale=1.3, mask_c=True),
    dict(L=6, B=3, d=4, k=4, act=1, dirs=2),
    dict(L=6, B=3, d=4, custom=True),
    dict(L=6, B=3, d=4, custom=True, dirs=2, pad="random", mask_c=True, scale=1.1),
    dict(L=5, B=2, d=3, custom=True, k=4, act=1, dirs=2),
    dict(L=12, B=2, d=70, dirs=2, pad="right", scale=1.7),
]
