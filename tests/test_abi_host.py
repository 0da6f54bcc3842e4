"""CPU-only checks of the boundary: the library loads, exports every symbol the header
declares, and rejects bad arguments before anything reaches a GPU."""
import ctypes
import os
import re

import pytest

from sru_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "sru_amd.h")).read()
    code = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(sru_amd_[a-z_]+)\s*\(", code))
    assert declared == set(_lib.SIGNATURES), (declared, set(_lib.SIGNATURES))
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert _lib.load().sru_amd_abi_version() == int(re.search(r"SRU_AMD_ABI_VERSION\s+(\d+)", header).group(1))


def test_struct_layout_matches_header():
    assert ctypes.sizeof(_lib.Shape) == 56
    assert _lib.Shape.dirs.offset == 24 and _lib.Shape.dtype.offset == 44
    assert _lib.Shape.state_interval.offset == 48 and _lib.Shape.x_dtype.offset == 52


def _shape(**kw):
    base = dict(length=4, batch=2, hidden=8, dirs=2, k=3, activation_type=0, skip_type=1,
                is_custom=0, dtype=0, state_interval=0, x_dtype=0)
    base.update(kw)
    return _lib.Shape(*[base[f[0]] for f in _lib.Shape._fields_])


FAKE = ctypes.c_void_p(0x1000)  # never dereferenced: validation fails first


@pytest.mark.parametrize("kw,code", [
    (dict(length=0), 2), (dict(batch=-1), 2), (dict(hidden=0), 2), (dict(hidden=1 << 31), 2),
    (dict(length=1 << 60), 2), (dict(dirs=3), 3), (dict(k=5), 3), (dict(k=2), 3),
    (dict(activation_type=2), 3), (dict(skip_type=3), 3), (dict(skip_type=1, k=4), 3),
    (dict(skip_type=2, k=3), 3), (dict(is_custom=2), 3), (dict(dtype=7), 4),
    (dict(state_interval=4), 3), (dict(state_interval=8, dtype=3), 3),   # double streams: no checkpoints
    (dict(state_interval=8, is_custom=1, activation_type=1), 3), (dict(state_interval=8, skip_type=0, k=4), 3),
    (dict(state_interval=8, dtype=2, hidden=7), 3), (dict(state_interval=8, dtype=1, hidden=1), 3),
    # a float x beside 16-bit streams: plain layer only, even hidden; with float streams the field changes nothing
    (dict(x_dtype=2), 4), (dict(x_dtype=1, dtype=2, state_interval=8, is_custom=1), 3),
    (dict(x_dtype=1, dtype=1, state_interval=8, activation_type=1), 3), (dict(x_dtype=1, dtype=2, hidden=7), 3),
])
def test_forward_rejects_bad_shapes(kw, code):
    lib = _lib.load()
    s = _shape(**kw)
    assert lib.sru_amd_forward(ctypes.byref(s), *([FAKE] * 11), None) == code
    assert lib.sru_amd_backward_workspace_bytes(ctypes.byref(s)) == 0
    assert lib.sru_amd_state_bytes(ctypes.byref(s)) == 0
    assert lib.sru_amd_backward(ctypes.byref(s), *([FAKE] * 17), 1 << 20, None) == code


def test_null_and_misaligned_pointers_and_workspace():
    lib = _lib.load()
    s = _shape()
    assert lib.sru_amd_forward(None, *([FAKE] * 11), None) == 1
    args = [FAKE] * 11
    for required in (0, 1, 2, 3, 8, 10):   # u, x (skip from x), weight_c, bias, h, c_last (c_init may be NULL: zeros)
        bad = list(args)
        bad[required] = None
        assert lib.sru_amd_forward(ctypes.byref(s), *bad, None) == 1, required
    odd = ctypes.c_void_p(0x1002)
    bad = list(args)
    bad[0] = odd
    assert lib.sru_amd_forward(ctypes.byref(s), *bad, None) == 5
    s4 = _shape(k=4, skip_type=2)
    bad = list(args)
    bad[0] = ctypes.c_void_p(0x1008)            # k=4 float groups move as 16-byte vectors
    assert lib.sru_amd_forward(ctypes.byref(s4), *bad, None) == 5
    need = lib.sru_amd_backward_workspace_bytes(ctypes.byref(s))
    assert need == 4 * 4 * 2 * 16
    assert lib.sru_amd_state_bytes(ctypes.byref(s)) == 4 * 2 * 16 * 4           # (L, B, D') floats
    assert lib.sru_amd_state_bytes(ctypes.byref(_shape(dtype=2))) == 4 * 2 * 16 * 2
    assert lib.sru_amd_state_bytes(ctypes.byref(_shape(state_interval=8))) == 1 * 2 * 16 * 4
    assert lib.sru_amd_state_bytes(ctypes.byref(_shape(length=33, state_interval=8, dtype=1))) == 4 * 2 * 16 * 4
    # double streams: the state after every step in double, and double partial sums
    assert lib.sru_amd_state_bytes(ctypes.byref(_shape(dtype=3))) == 4 * 2 * 16 * 8
    assert lib.sru_amd_backward_workspace_bytes(ctypes.byref(_shape(dtype=3))) == 4 * 8 * 2 * 16
    bad = list(args)
    bad[3] = ctypes.c_void_p(0x1004)            # with double streams the small tensors are doubles too
    assert lib.sru_amd_forward(ctypes.byref(_shape(dtype=3)), *bad, None) == 5
    assert lib.sru_amd_backward(ctypes.byref(s), *([FAKE] * 16), None, need, None) == 6
    assert lib.sru_amd_backward(ctypes.byref(s), *([FAKE] * 17), need - 1, None) == 6
    # u, x, weight_c, bias, c, grad_h, grad_u, grad_x, grad_wc, grad_bias, grad_init
    # (c_init = 4 and grad_last = 10 may be NULL: zeros)
    for required in (0, 1, 2, 3, 8, 9, 11, 12, 13, 14, 15):
        bad = [FAKE] * 17                        # e.g. 12: grad_x is required when the skip term is x
        bad[required] = None
        assert lib.sru_amd_backward(ctypes.byref(s), *bad, need, None) == 1, required


def test_float_x_beside_16bit_streams_needs_checkpoints_or_no_state():
    lib = _lib.load()
    s = _shape(dtype=2, x_dtype=1, state_interval=1)
    assert lib.sru_amd_forward(ctypes.byref(s), *([FAKE] * 11), None) == 3       # c given, state after every step
    assert lib.sru_amd_backward(ctypes.byref(s), *([FAKE] * 17), 1 << 20, None) == 3
    s = _shape(dtype=2, x_dtype=1, state_interval=8)
    bad = [FAKE] * 11
    bad[1] = ctypes.c_void_p(0x1002)             # the float x must be 4-byte aligned
    assert lib.sru_amd_forward(ctypes.byref(s), *bad, None) == 5


def test_static_backward_checks_sizes_before_anything_else():
    # the allocation-free entry point refuses more columns than its built-in array holds
    lib = _lib.load()
    wide = _shape(batch=_lib.STATIC_MAX_COLUMNS // 16 + 1)
    assert lib.sru_amd_backward_static(ctypes.byref(wide), *([FAKE] * 16), None) == 8
    half = _shape(batch=_lib.STATIC_MAX_COLUMNS // 32 + 1, dtype=3)   # double partial sums: half the columns
    assert lib.sru_amd_backward_static(ctypes.byref(half), *([FAKE] * 16), None) == 8
    assert lib.sru_amd_backward_static(ctypes.byref(_shape(k=5)), *([FAKE] * 16), None) == 3
    assert lib.sru_amd_backward_static(None, *([FAKE] * 16), None) == 1


def test_layer_norm_entry_points_validate_before_launching():
    lib = _lib.load()
    f32 = 0
    fwd = lambda rows, cols, x=FAKE, dx=f32, dy=f32: lib.sru_amd_layer_norm_forward(
        rows, cols, x, dx, FAKE, FAKE, ctypes.c_float(1e-5), FAKE, dy, FAKE, FAKE, None)
    assert fwd(0, 64) == 2 and fwd(4, 0) == 2 and fwd(4, 12) == 2          # cols must be a multiple of 8
    assert fwd(4, _lib.NORM_MAX_FEATURES + 8) == 2
    assert fwd(4, 64, dx=9) == 4 and fwd(4, 64, dy=5) == 4 and fwd(4, 64, dx=3) == 4   # no double rows
    assert fwd(4, 64, x=None) == 1
    assert fwd(4, 64, x=ctypes.c_void_p(0x1004)) == 5
    need = lib.sru_amd_layer_norm_backward_workspace_bytes(4, 64)
    # one (2, cols) float row per workgroup of the backward kernel: one workgroup here, 512 at most
    assert need == 2 * 64 * 4 and lib.sru_amd_layer_norm_backward_workspace_bytes(4, 12) == 0
    assert lib.sru_amd_layer_norm_backward_workspace_bytes(16384, 2048) == 512 * 2 * 2048 * 4
    assert lib.sru_amd_layer_norm_backward_workspace_bytes(10 ** 6, 4096) == 512 * 2 * 4096 * 4   # 8 wavefronts per row
    gw = ctypes.c_void_p(0x2000)
    gb = ctypes.c_void_p(0x2000 + 64 * 4)
    bwd = lambda ws, nbytes, gbias=gb: lib.sru_amd_layer_norm_backward(
        4, 64, FAKE, f32, FAKE, FAKE, FAKE, FAKE, f32, FAKE, gw, gbias, ws, nbytes, None)
    assert bwd(None, need) == 6 and bwd(FAKE, need - 1) == 6
    assert bwd(FAKE, need, gbias=ctypes.c_void_p(0x3000)) == 5          # the two sums must be adjacent


def test_status_strings_and_python_error_mapping():
    for code in range(0, 9):
        assert _lib.status_string(code)
    with pytest.raises(ValueError):
        _lib.check(3, "x")
    with pytest.raises(RuntimeError):
        _lib.check(7, "x")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libsru_amd.so"))
    with pytest.raises(_lib.LibraryError):
        _lib.load()


def test_function_refuses_cpu_tensors():
    import torch
    from sru_amd import ElementwiseRecurrence
    L, B, d = 3, 2, 4
    with pytest.raises(RuntimeError):
        ElementwiseRecurrence.apply(torch.randn(L, B, 3 * d), torch.randn(L, B, d), torch.randn(2 * d),
                                    torch.randn(2 * d), torch.zeros(B, d), 0, d, False, True, None)


def test_plain_c_caller_is_built_and_links_against_the_library():
    """sru_amd/serve_forward (no Python, no torch) starts, i.e. finds libsru_amd.so and the HIP
    runtime next to it, and refuses a wrong argument list before it touches any device."""
    import subprocess
    program = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "sru_amd", "serve_forward")
    assert os.path.exists(program), "run python -m sru_amd.build"
    proc = subprocess.run([program], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert proc.returncode == 64 and "usage:" in proc.stderr
