"""Writes the committed golden fixtures under tests/golden/.

1. regression_2.3.5.npz: the reference's own regression artifact
   (test/regression/artifacts/2.3.5.pt: inputs, state_dict and outputs of a
   2-layer bidirectional SRU(5, 7) saved by v2.3.5 in eval mode,
   test/regression/build_artifact.py:17-48), re-encoded as plain arrays. It is
   read with torch.load(weights_only=True); no reference code runs.
2. cpu_ref_vectors.npz: seeded inputs pushed through the reference's CPU
   routine compiled from its source (oracle/_ref, sru/csrc/sru_cpu_impl.cpp:
   cpu_forward / cpu_bi_forward): uni/bi, k=3/4, tanh, padding, no-skip,
   per-step V (unidirectional only: the reference's bidirectional CPU routine
   indexes V by loop counter, :202-203, unlike its GPU kernels).

Run from the repo root where /root/reference exists:
    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REFERENCE = os.environ.get("SRU_REFERENCE", "/root/reference")


def regression_artifact():
    art = torch.load(os.path.join(REFERENCE, "test/regression/artifacts/2.3.5.pt"),
                     weights_only=True)
    out = {"inputs": art["inputs"].numpy(),
           "out_h": art["outputs"][0].numpy(),
           "out_c": art["outputs"][1].numpy()}
    for key, val in art["model_state"].items():
        out["state/" + key] = val.numpy()
    for key, val in art["sru_kwargs"].items():
        out["kwargs/" + key] = np.asarray(val)
    out["version"] = np.asarray(art["sru.__version__"])
    np.savez(os.path.join(HERE, "regression_2.3.5.npz"), **out)
    print("regression_2.3.5.npz:", sorted(out))


CASES = [
    # name, L, B, d, dirs, k, act, skip, custom, pad, scale
    ("uni_k3", 6, 3, 5, 1, 3, 0, True, False, False, 1.0),
    ("uni_k3_scale_pad", 7, 4, 5, 1, 3, 0, True, False, True, 1.7320508),
    ("uni_k4", 6, 3, 5, 1, 4, 0, True, False, False, 1.0),
    ("uni_k3_noskip_tanh", 5, 2, 4, 1, 3, 1, False, False, True, 1.0),
    ("uni_k4_tanh", 5, 2, 4, 1, 4, 1, True, False, False, 1.0),
    ("uni_k3_custom", 6, 3, 4, 1, 3, 0, True, True, True, 1.5),
    ("bi_k3", 6, 3, 5, 2, 3, 0, True, False, False, 1.0),
    ("bi_k3_scale_pad", 9, 4, 3, 2, 3, 0, True, False, True, 1.2),
    ("bi_k4_pad", 8, 3, 4, 2, 4, 0, True, False, True, 1.0),
    ("bi_k3_noskip", 5, 2, 4, 2, 3, 0, False, False, False, 1.0),
    ("bi_k4_tanh_pad", 6, 3, 3, 2, 4, 1, True, False, True, 1.0),
]


def cpu_ref_vectors():
    so = os.path.join(ROOT, "oracle", "_ref", "libsru_cpu_ref.so")
    torch.ops.load_library(so)
    out = {}
    names = []
    for i, (name, L, B, d, dirs, k, act, skip, custom, pad, scale) in enumerate(CASES):
        g = torch.Generator().manual_seed(1000 + i)
        Dp = d * dirs
        U = torch.randn(L, B, Dp * k, generator=g)
        x = torch.randn(L, B, Dp, generator=g)
        wc = torch.randn(L, B, Dp * 2, generator=g) if custom else torch.randn(2 * Dp, generator=g)
        bias = torch.randn(2 * Dp, generator=g)
        c0 = torch.randn(B, Dp, generator=g)
        mask = None
        if pad:
            mask = torch.rand(L, B, generator=g) < 0.3
        fn = torch.ops.sru_cpu.cpu_bi_forward if dirs == 2 else torch.ops.sru_cpu.cpu_forward
        h, c = fn(U, x, wc, bias, c0, mask, L, B, d, k, act, skip, float(scale), custom)
        names.append(name)
        out[name + "/cfg"] = np.asarray([L, B, d, dirs, k, act, int(skip), int(custom)], np.int64)
        out[name + "/scale"] = np.asarray(scale, np.float64)
        out[name + "/U"] = U.numpy()
        out[name + "/x"] = x.numpy()
        out[name + "/wc"] = wc.numpy()
        out[name + "/bias"] = bias.numpy()
        out[name + "/c0"] = c0.numpy()
        if mask is not None:
            out[name + "/pad"] = mask.numpy()
        out[name + "/h"] = h.numpy()
        out[name + "/c"] = c.numpy()
    out["names"] = np.asarray(names)
    np.savez(os.path.join(HERE, "cpu_ref_vectors.npz"), **out)
    print("cpu_ref_vectors.npz:", names)


if __name__ == "__main__":
    if not os.path.isdir(REFERENCE):
        sys.exit("reference checkout not found at " + REFERENCE)
    regression_artifact()
    cpu_ref_vectors()
