"""ctypes front end of the C oracle (liboracle.so): TEST INFRASTRUCTURE ONLY.

`forward` / `backward` take and return numpy arrays in the reference's layouts
(see sru_oracle_impl.h). `precision` picks the float ("f32", the serial CPU loop
of sru/csrc/sru_cpu_impl.cpp:56-226 in its own arithmetic) or the double
("f64", the checker) instantiation.

Argument derivation mirrors sru/cuda_functional.py:54-65: `k` streams per
column, skip_type 0 (no skip), 1 (skip from x, k == 3) or 2 (skip from
U[..., 3], k == 4), is_custom when weight_c has more than one dimension.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build():
    """Compile liboracle.so (and oracle/_ref when the reference is present)."""
    subprocess.check_call(["make", "-C", _HERE, "all"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            subprocess.check_call(["make", "-C", _HERE, "liboracle.so"])
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


_CT = {"f32": (np.float32, ctypes.c_float), "f64": (np.float64, ctypes.c_double)}


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _prep(a, npdt):
    return None if a is None else np.ascontiguousarray(np.asarray(a), dtype=npdt)


def derive(U_last, d, dirs, has_skip_term, weight_c_ndim):
    """k, skip_type, is_custom as sru/cuda_functional.py:57-65 derives them."""
    k = U_last // (d * dirs)
    skip_type = 0 if not has_skip_term else (1 if k == 3 else 2)
    return k, skip_type, int(weight_c_ndim > 1)


def forward(U, x, weight_c, bias, c_init, *, d, dirs, k, activation_type=0, skip_type=1,
            is_custom=0, scale_x=1.0, mask_c=None, mask_pad=None, precision="f64"):
    """Returns (h (L,B,D'), c_all (L,B,D'), c_last (B,D'))."""
    npdt, cdt = _CT[precision]
    U = _prep(U, npdt)
    B = c_init.shape[0]
    Dp = d * dirs
    L = U.size // (B * Dp * k)
    assert U.size == L * B * Dp * k
    x = _prep(x, npdt) if skip_type == 1 else None
    if skip_type == 1:
        assert x.size == L * B * Dp
    weight_c = _prep(weight_c, npdt)
    assert weight_c.size == (L * B * Dp * 2 if is_custom else 2 * Dp)
    bias = _prep(bias, npdt)
    assert bias.size == 2 * Dp
    c_init = _prep(c_init, npdt)
    assert c_init.size == B * Dp
    mask_c = _prep(mask_c, npdt)
    mask_pad = None if mask_pad is None else np.ascontiguousarray(np.asarray(mask_pad) != 0, dtype=np.uint8)
    if mask_pad is not None:
        assert mask_pad.shape == (L, B)
    h = np.empty((L, B, Dp), npdt)
    c_all = np.empty((L, B, Dp), npdt)
    c_last = np.empty((B, Dp), npdt)
    fn = getattr(lib(), "sru_oracle_forward_" + precision)
    fn.restype = None
    fn(_ptr(U), _ptr(x), _ptr(weight_c), _ptr(bias), _ptr(c_init), _ptr(mask_c), _ptr(mask_pad),
       ctypes.c_int64(L), ctypes.c_int64(B), ctypes.c_int64(d), ctypes.c_int(dirs), ctypes.c_int(k),
       ctypes.c_int(activation_type), ctypes.c_int(skip_type), ctypes.c_int(is_custom), cdt(scale_x),
       _ptr(h), _ptr(c_all), _ptr(c_last))
    return h, c_all, c_last


def backward(U, x, weight_c, bias, c_init, c_all, grad_h, grad_last, *, d, dirs, k,
             activation_type=0, skip_type=1, is_custom=0, scale_x=1.0, mask_c=None,
             mask_pad=None, precision="f64"):
    """Returns (grad_u, grad_x or None, grad_wc, grad_bias, grad_init).

    grad_wc is (2*D',) summed over batch and time, or (L,B,D',2) with is_custom.
    """
    npdt, cdt = _CT[precision]
    U = _prep(U, npdt)
    B = c_init.shape[0]
    Dp = d * dirs
    L = U.size // (B * Dp * k)
    x = _prep(x, npdt) if skip_type == 1 else None
    weight_c = _prep(weight_c, npdt)
    bias = _prep(bias, npdt)
    c_init = _prep(c_init, npdt)
    mask_c = _prep(mask_c, npdt)
    mask_pad = None if mask_pad is None else np.ascontiguousarray(np.asarray(mask_pad) != 0, dtype=np.uint8)
    c_all = _prep(c_all, npdt)
    grad_h = _prep(grad_h, npdt)
    grad_last = _prep(grad_last, npdt)
    assert c_all.size == grad_h.size == L * B * Dp and grad_last.size == B * Dp
    grad_u = np.empty((L, B, Dp * k), npdt)
    grad_x = np.empty((L, B, Dp), npdt) if skip_type == 1 else None
    grad_wc = np.empty((L, B, Dp, 2) if is_custom else (2 * Dp,), npdt)
    grad_bias = np.empty((2 * Dp,), npdt)
    grad_init = np.empty((B, Dp), npdt)
    fn = getattr(lib(), "sru_oracle_backward_" + precision)
    fn.restype = None
    fn(_ptr(U), _ptr(x), _ptr(weight_c), _ptr(bias), _ptr(c_init), _ptr(mask_c), _ptr(mask_pad),
       _ptr(c_all), _ptr(grad_h), _ptr(grad_last),
       ctypes.c_int64(L), ctypes.c_int64(B), ctypes.c_int64(d), ctypes.c_int(dirs), ctypes.c_int(k),
       ctypes.c_int(activation_type), ctypes.c_int(skip_type), ctypes.c_int(is_custom), cdt(scale_x),
       _ptr(grad_u), _ptr(grad_x), _ptr(grad_wc), _ptr(grad_bias), _ptr(grad_init))
    return grad_u, grad_x, grad_wc, grad_bias, grad_init
