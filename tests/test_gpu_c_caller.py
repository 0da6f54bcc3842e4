"""The C ABI called from a program with no Python and no torch in it.

sru_amd/serve_forward (csrc/serve_forward.cpp, the role sru/csrc/main_test_cpp.cpp plays
for the reference's operators) builds its inputs from a fixed integer recipe, runs one
forward scan without state store and writes h and c_last to a file. Here the same inputs
are rebuilt in numpy and the file is compared with the CPU oracle: float32, max abs error
<= 1e-5.
"""
import os
import subprocess

import numpy as np
import pytest

from oracle import sru_oracle as so

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAM = os.path.join(ROOT, "sru_amd", "serve_forward")

pytestmark = pytest.mark.gpu


def value(n, salt):
    i = np.arange(n, dtype=np.uint64)
    h = (i * np.uint64(2654435761) + np.uint64(salt * 40503)) & np.uint64(0xFFFFFFFF)
    return (((h >> np.uint64(8)) & np.uint64(0xFFFF)).astype(np.float32) / np.float32(65536.0)
            - np.float32(0.5))


@pytest.mark.parametrize("L,B,d,dirs,k,padded", [
    (20, 32, 128, 1, 3, 0),      # the README example's layer shape
    (37, 5, 96, 2, 3, 1),
    (16, 3, 50, 2, 4, 1),
    (64, 8, 256, 2, 4, 0),
])
def test_forward_from_a_plain_c_caller(tmp_path, L, B, d, dirs, k, padded):
    if not os.path.exists(PROGRAM):
        pytest.fail("sru_amd/serve_forward is not built: run python -m sru_amd.build")
    out = tmp_path / "h.bin"
    print(f"serve_forward L={L} B={B} d={d} dirs={dirs} k={k} padded={padded}", flush=True)
    proc = subprocess.run([PROGRAM, str(L), str(B), str(d), str(dirs), str(k), str(padded), str(out)],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout
    Dp = d * dirs
    cells = L * B * Dp
    got = np.fromfile(out, dtype=np.float32)
    assert got.size == cells + B * Dp
    h, c_last = got[:cells].reshape(L, B, Dp), got[cells:].reshape(B, Dp)

    U = (2 * value(cells * k, 1)).reshape(L, B, Dp * k)
    x = (2 * value(cells, 2)).reshape(L, B, Dp)
    pad = None
    if padded:
        pad = np.zeros((L, B), bool)
        for b in range(B):
            pad[L - (b * 3) % (L // 2):, b] = True
    h_ref, _, cl_ref = so.forward(U, x, value(2 * Dp, 3), value(2 * Dp, 4), value(B * Dp, 5).reshape(B, Dp),
                                  d=d, dirs=dirs, k=k, skip_type=1 if k == 3 else 2, scale_x=1.5,
                                  mask_pad=pad, precision="f64")
    assert np.abs(h - h_ref).max() <= 1e-5
    assert np.abs(c_last - cl_ref).max() <= 1e-5
    if padded:
        assert not h[pad].any()          # padded cells are exact zeros
