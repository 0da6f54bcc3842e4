#!/usr/bin/env python3
"""Benchmark of the SRU recurrence hot path on one MI355X.

A step = one forward scan + one backward scan of ONE layer's recurrence, called
through the C ABI (include/sru_amd.h) on synthetic inputs already resident in HBM.
Workload = the headline configuration: bidirectional, d=1024 per direction
(D'=2048), L=256, B=64, k=3 with the skip term read from x, scale_x=sqrt(3), c0=0,
float32 streams. Inputs rotate over several buffer sets, and the backward call of a
step uses another set than its forward call, so that no kernel finds its operands in
the last-level cache.

Prints ONE JSON line: tokens/s (tokens = L*B per step), per-kernel HIP-event timings,
the HBM roofline of the dominant kernel (the backward scan) on algorithmic bytes, and
a single-core CPU baseline timed on this host with the CPU oracle (reported only).
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
WORKLOADS = {
    # key: (name, L, B, d, dirs, k, forward_only, padded). "headline" is the configuration the
    # metric is quoted on; the others are the reference's remaining GPU configurations at
    # one layer, kept for side measurements (--workload).
    "headline": ("bi-SRU d=1024 L=256 B=64 k=3", 256, 64, 1024, 2, 3, False, False),
    "headline-uni": ("uni-SRU d=2048 L=256 B=64 k=3 (the headline's columns in one direction)", 256, 64, 2048, 1, 3, False, False),
    "headline-k4": ("bi-SRU d=1024 L=256 B=64 k=4", 256, 64, 1024, 2, 4, False, False),
    "config1": ("uni-SRU d=128 L=20 B=32 k=3 forward only (README example)", 20, 32, 128, 1, 3, True, False),
    "config2": ("bi-SRU d=512 L=128 B=32 k=3, right-padded lengths in [32,128]", 128, 32, 512, 2, 3, False, True),
    "config4": ("uni-SRU d=2048 L=512 B=16 k=3", 512, 16, 2048, 1, 3, False, False),
    "config5": ("bi-SRU d=256 L=4096 B=256 k=3 forward only, lengths in [1024,4096]", 4096, 256, 256, 2, 3, True, True),
    "config5-nopad": ("bi-SRU d=256 L=4096 B=256 k=3 forward only", 4096, 256, 256, 2, 3, True, False),
    "headline-infer": ("bi-SRU d=1024 L=256 B=64 k=3 forward only", 256, 64, 1024, 2, 3, True, False),
    "headline-pad": ("bi-SRU d=1024 L=256 B=64 k=3, right-padded lengths in [64,256]", 256, 64, 1024, 2, 3, False, True),
}
DT_BYTES = {"f32": 4, "f16": 2, "bf16": 2, "f64": 8}


def cpu_baseline(L, B, d, dirs, k, budget_s=12.0):
    """Times the float32 CPU oracle (serial loop, 1 core) on a slice of the batch."""
    from oracle import sru_oracle as so
    Bc = B
    Dp = d * dirs
    rng = np.random.default_rng(0)
    U = rng.standard_normal((L, Bc, Dp * k), dtype=np.float32)
    x = rng.standard_normal((L, Bc, Dp), dtype=np.float32)
    wc = rng.uniform(-1.2, 1.2, 2 * Dp).astype(np.float32)
    bias = np.zeros(2 * Dp, np.float32)
    c0 = np.zeros((Bc, Dp), np.float32)
    gh = rng.standard_normal((L, Bc, Dp), dtype=np.float32)
    gl = np.zeros((Bc, Dp), np.float32)
    kw = dict(d=d, dirs=dirs, k=k, skip_type=1 if k == 3 else 2, scale_x=3 ** 0.5, precision="f32")
    so.lib()
    reps, spent = 0, 0.0
    while reps < 1 or spent < budget_s:
        t0 = time.perf_counter()
        _, c_all, _ = so.forward(U, x, wc, bias, c0, **kw)
        so.backward(U, x, wc, bias, c0, c_all, gh, gl, **kw)
        spent += time.perf_counter() - t0
        reps += 1
    tokens = L * Bc * reps
    out = {"value": tokens / spent, "unit": "tokens/s", "cores": 1, "kind": "port",
           "sample": f"{reps} x (forward+backward) of the same layer at batch {Bc} of {B} "
                     f"(L={L}, D'={Dp}, k={k}, float32 serial C loop), {spent:.1f} s",
           "host_cores": os.cpu_count()}
    # Beside it, where the build made it: the reference's own CPU routine compiled from its
    # source file (forward only, it has no backward), on the same arrays, one thread.
    ref_so = os.path.join(ROOT, "oracle", "_ref", "libsru_cpu_ref.so")
    if os.path.exists(ref_so):
        try:
            import torch
            torch.ops.load_library(ref_so)
            fn = torch.ops.sru_cpu.cpu_bi_forward if dirs == 2 else torch.ops.sru_cpu.cpu_forward
            tU, tx, twc, tb, tc0 = (torch.from_numpy(a) for a in (U, x, wc, bias, c0))
            threads = torch.get_num_threads()
            torch.set_num_threads(1)
            reps, spent = 0, 0.0
            while reps < 1 or spent < budget_s / 3:
                t0 = time.perf_counter()
                fn(tU, tx, twc, tb, tc0, None, L, Bc, d, k, 0, True, 3 ** 0.5, False)
                spent += time.perf_counter() - t0
                reps += 1
            torch.set_num_threads(threads)
            out["reference_forward_only"] = {
                "value": L * Bc * reps / spent, "unit": "tokens/s", "cores": 1, "kind": "reference",
                "sample": f"{reps} x forward of the same layer (sru/csrc/sru_cpu_impl.cpp compiled "
                          f"as oracle/_ref), {spent:.1f} s"}
        except Exception as e:   # a baseline that cannot load is reported, never fatal
            out["reference_forward_only"] = {"error": repr(e)[:200]}
    out["python_autograd_loop"] = cpu_autograd_loop()
    return out


def cpu_autograd_loop(budget_s=3.0):
    """The reference's other CPU path, the Python loop over time under autograd
    (sru/ops.py:145-250), as restated in oracle/sru_torch.py: forward + backward at the small
    shapes it is practical for (configs 1 and 2, one layer), float32, torch's default threads."""
    import torch
    from oracle import sru_torch as st
    res = {"unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port"}
    for key, (L, B, d, bi) in {"config1": (20, 32, 128, False), "config2": (128, 32, 512, True)}.items():
        g = torch.Generator().manual_seed(0)
        Dp = d * (2 if bi else 1)
        u = torch.randn(L, B, Dp * 3, generator=g, requires_grad=True)
        x = torch.randn(L, B, Dp, generator=g, requires_grad=True)
        wc = torch.randn(2 * Dp, generator=g, requires_grad=True)
        bias = torch.zeros(2 * Dp, requires_grad=True)
        c0 = torch.zeros(B, Dp, requires_grad=True)
        probe = torch.randn(L, B, Dp, generator=g)
        reps, spent = 0, 0.0
        while reps < 1 or spent < budget_s:
            t0 = time.perf_counter()
            h, last = st.recurrence(u, x, wc, bias, c0, 0, d, bi, True, torch.tensor([3 ** 0.5]))
            (h * probe).sum().backward()
            spent += time.perf_counter() - t0
            reps += 1
        res[key] = {"value": L * B * reps / spent, "sample": f"{reps} x (forward+backward), L={L} B={B} D'={Dp}, {spent:.1f} s"}
    return res


STACKS = {
    # key: (name, constructor arguments of sru_amd.SRU, L, B, input size, autocast dtype or None)
    "stack1": ("README example: 2-layer uni-SRU d=128 L=20 B=32 highway_bias=-2, forward only, module level",
               dict(input_size=128, hidden_size=128, num_layers=2, highway_bias=-2.0), 20, 32, 128),
    "stack2": ("4-layer bi-SRU d=512 L=128 B=32, right-padded lengths in [32,128], module level",
               dict(input_size=512, hidden_size=512, num_layers=4, bidirectional=True), 128, 32, 512),
    "stack3": ("4-layer bi-SRU d=1024 L=256 B=64 layer_norm rescale, module level",
               dict(input_size=1024, hidden_size=1024, num_layers=4, bidirectional=True, layer_norm=True,
                    rescale=True), 256, 64, 1024),
    "stack4": ("10-layer uni-SRU hidden=2048 projection=512 L=512 B=16 dropout=0.1, module level",
               dict(input_size=2048, hidden_size=2048, num_layers=10, projection_size=512, dropout=0.1),
               512, 16, 2048),
}


def run_stack(args):
    """Side measurement: the whole layer stack (GEMM, recurrence, layer norm, autograd) through
    sru_amd.SRU, forward + backward per step. Not the headline metric: it shows what share of a
    training step the recurrence kernels are and what the Python layer adds around them."""
    import torch
    import sru_amd
    name, kw, L, B, n_in = STACKS[args.workload]
    if args.torch_layer_norm:   # comparison run: torch's layer norm (and autocast's casts around it)
        import sru_amd.modules
        sru_amd.modules.fused_layer_norm_supported = lambda x: False
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    model = sru_amd.SRU(**kw).to(dev)
    amp = {"f32": None, "bf16": torch.bfloat16, "f16": torch.float16}[args.dtype]
    x = torch.randn(L, B, n_in, device=dev)
    probe = torch.randn(L, B, model.output_size, device=dev)

    forward_only = args.workload == "stack1"
    mask_pad = None
    if args.workload == "stack2":
        lens = torch.randint(32, L + 1, (B,), device=dev)
        mask_pad = (torch.arange(L, device=dev)[:, None] >= lens[None, :])

    def step():
        if forward_only:
            with torch.no_grad(), torch.autocast("cuda", dtype=amp, enabled=amp is not None):
                return model(x)
        with torch.autocast("cuda", dtype=amp, enabled=amp is not None):
            h, _ = model(x, mask_pad=mask_pad)
        (h.float() * probe).sum().backward()
        model.zero_grad(set_to_none=True)

    if args.graph:      # record once with sru_amd.graphed, replay per step (launch-bound shapes)
        if forward_only:
            model.eval()
            with torch.no_grad():
                fast = sru_amd.graphed(model, x, autocast_dtype=amp)

            def step():
                return fast(x)
        else:
            fast = sru_amd.graphed(model, x, mask_pad=mask_pad, autocast_dtype=amp)

            def step():
                h, _ = fast(x, mask_pad=mask_pad)
                (h.float() * probe).sum().backward()
                model.zero_grad(set_to_none=True)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    print(json.dumps({
        "metric": "module-level step (side measurement)", "value": L * B / (ms_step * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype if amp is None else args.dtype + " autocast", "data": "synthetic",
        "config": {"workload": name, "length": L, "batch": B, "layers": kw["num_layers"],
                   "pass": "forward only" if forward_only else "forward+backward",
                   "replayed_from_graph": bool(args.graph),
                   "layer_norm": "torch" if args.torch_layer_norm else "sru_amd kernels"}}), flush=True)


def run_layer_norm(args):
    """Side measurement: the layer-norm kernels next to the recurrence, through the C ABI, at the
    row count and width of the headline layer (16 384 rows of 2 048 features). Forward and backward
    (the backward call includes the launch that adds the workgroups' weight / bias sums) are
    timed with HIP events on rotating buffer sets; the roofline is HBM, bytes = rows read + written,
    plus, for the backward call, the workgroups' partial sums written once and read once."""
    import torch
    from sru_amd import _lib
    rows, D = 256 * 64, 2048
    dev = torch.device("cuda:0")
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    code = {"f32": _lib.F32, "f16": _lib.F16, "bf16": _lib.BF16}[args.dtype]
    es = DT_BYTES[args.dtype]
    lib = _lib.load()
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    g = torch.Generator(device=dev).manual_seed(0)
    w = torch.rand(D, device=dev, generator=g) + 0.5
    b = torch.randn(D, device=dev, generator=g)
    nbytes = lib.sru_amd_layer_norm_backward_workspace_bytes(rows, D)
    sets = []
    for _ in range(args.sets):
        sets.append(dict(x=torch.randn(rows, D, device=dev, generator=g).to(tdt), y=torch.empty(rows, D, device=dev, dtype=tdt),
                         dy=torch.randn(rows, D, device=dev, generator=g).to(tdt), dx=torch.empty(rows, D, device=dev, dtype=tdt),
                         mean=torch.empty(rows, device=dev), rstd=torch.empty(rows, device=dev),
                         gwb=torch.empty(2, D, device=dev), ws=torch.empty(nbytes // 4, device=dev)))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def fwd(s):
        _lib.check(lib.sru_amd_layer_norm_forward(rows, D, p(s["x"]), code, p(w), p(b), ctypes.c_float(1e-5), p(s["y"]), code,
                                                  p(s["mean"]), p(s["rstd"]), stream), "sru_amd_layer_norm_forward")

    def bwd(s):
        _lib.check(lib.sru_amd_layer_norm_backward(rows, D, p(s["x"]), code, p(w), p(s["mean"]), p(s["rstd"]), p(s["dy"]), code,
                                                   p(s["dx"]), p(s["gwb"][0]), p(s["gwb"][1]), p(s["ws"]),
                                                   ctypes.c_size_t(nbytes), stream), "sru_amd_layer_norm_backward")

    for s in sets:
        fwd(s)
    ev = lambda: torch.cuda.Event(enable_timing=True)
    n = args.warmup + args.steps
    marks = [(ev(), ev(), ev()) for _ in range(n)]
    torch.cuda.synchronize()
    t0 = None
    for i in range(n):
        if i == args.warmup:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
        a, m, e = marks[i]
        a.record()
        fwd(sets[i % args.sets])
        m.record()
        bwd(sets[(i + 2) % args.sets])   # a set whose forward ran earlier: operands cache-cold
        e.record()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    f_us = sum(a.elapsed_time(m) for a, m, _ in marks[args.warmup:]) * 1e3 / args.steps
    b_us = sum(m.elapsed_time(e) for _, m, e in marks[args.warmup:]) * 1e3 / args.steps
    f_bytes, b_bytes = 2 * es * rows * D, 3 * es * rows * D + 2 * nbytes
    gbs = lambda nb, us: nb / (us * 1e-6) / 1e9
    print(json.dumps({
        "metric": "layer norm rows/s (side measurement)", "value": rows / (ms_step * 1e-3), "unit": "rows/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": f"layer norm forward + backward, {rows} rows of {D} features, {args.dtype} in and out"},
        "roofline": {"bound": "hbm", "kernel": "layer_norm_backward (+ reduce_rows)", "achieved": gbs(b_bytes, b_us),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs(b_bytes, b_us) / HBM_PEAK_GBS, "traffic": None,
                     "avg_us": b_us},
        "kernels": {"layer_norm_forward": {"avg_us": f_us, "algorithmic_GBps": gbs(f_bytes, f_us),
                                           "frac_of_hbm_peak": gbs(f_bytes, f_us) / HBM_PEAK_GBS},
                    "layer_norm_backward+reduce": {"avg_us": b_us, "algorithmic_GBps": gbs(b_bytes, b_us),
                                                   "frac_of_hbm_peak": gbs(b_bytes, b_us) / HBM_PEAK_GBS}}}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--dtype", default="f32", choices=sorted(DT_BYTES))
    ap.add_argument("--sets", type=int, default=4, help="rotating buffer sets")
    ap.add_argument("--workload", default="headline", choices=sorted(WORKLOADS) + sorted(STACKS) + ["layernorm"])
    ap.add_argument("--full-state", action="store_true",
                    help="keep the state after every step between forward and backward, as the "
                         "reference does, instead of float checkpoints every 8 steps (the path "
                         "the autograd Function of this package takes)")
    ap.add_argument("--no-skip", action="store_true",
                    help="side measurement: no skip term (has_skip_term=False); with a k=4 workload this "
                         "runs the general kernels, which keep the state after every step")
    ap.add_argument("--tanh", action="store_true",
                    help="side measurement: activation_type = tanh (the reference's deprecated use_tanh)")
    ap.add_argument("--graph", action="store_true",
                    help="side measurement: record the calls into a HIP graph and time replays (recurrence "
                         "workloads: one rotation of forward + backward calls; stack1: the forward-only stack)")
    ap.add_argument("--per-step-weight-c", action="store_true",
                    help="side measurement: weight_c given per step, (L, B, D', 2) in the stream dtype (the "
                         "reference's custom_m returning V)")
    ap.add_argument("--torch-layer-norm", action="store_true",
                    help="with a stack workload: use torch.nn.LayerNorm's kernels instead of this package's")
    ap.add_argument("--shape", default=None, metavar="L,B,d,dirs",
                    help="side measurement at another shape (k=3 forward + backward, no padding); replaces --workload")
    ap.add_argument("--x-f32", action="store_true",
                    help="side measurement with 16-bit streams: x and grad_x stay float32 (shape.x_dtype = "
                         "SRU_AMD_X_F32), as the layer's input does under autocast")
    ap.add_argument("--fixed-length", type=int, default=0,
                    help="side measurement with a padded workload: every sequence has this length (default: "
                         "lengths uniform in [L/4, L])")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also time a plain device copy of 1 GiB (context for the roofline figures "
                         "and the known-size kernel that scales the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures the recurrence on ONE GPU only "
                 "(columns are independent; no multi-GPU path exists): run with --gpus 1")
    if args.dtype == "f64" and (args.workload in STACKS or args.workload == "layernorm"):
        sys.exit("bench.py: --dtype f64 is a side measurement of the recurrence calls only (the layer stacks "
                 "cast float64 to float32 as the reference's training entry does; layer norm has no double rows)")
    if args.workload in STACKS:
        return run_stack(args)
    if args.workload == "layernorm":
        return run_layer_norm(args)

    import torch
    from sru_amd import _lib

    TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "f64": torch.float64}
    CODE = {"f32": _lib.F32, "f16": _lib.F16, "bf16": _lib.BF16, "f64": _lib.F64}

    def p(t):   # device pointer for the C ABI
        return None if t is None else ctypes.c_void_p(t.data_ptr())

    name, L, B, d, dirs, k, fwd_only, padded = WORKLOADS[args.workload]
    if args.shape:
        L, B, d, dirs = (int(v) for v in args.shape.split(","))
        name, k, fwd_only, padded = f"{'bi' if dirs == 2 else 'uni'}-SRU d={d} L={L} B={B} k=3", 3, False, False
    name += " " + args.dtype
    Dp = d * dirs
    ncols, cells = B * Dp, L * B * Dp
    dev = torch.device("cuda:0")
    tdt = TORCH_DT[args.dtype]
    es = DT_BYTES[args.dtype]
    lib = _lib.load()
    custom = args.per_step_weight_c
    # (double streams: the general kernels, state after every step, small tensors in double too)
    ckpt = not args.full_state and not fwd_only and not (args.no_skip and k == 4) and not (custom and args.tanh) \
        and args.dtype != "f64"
    sdt = torch.float64 if args.dtype == "f64" else torch.float32
    use_x = k == 3 and not args.no_skip      # the skip term is read from x
    if args.tanh:
        name += " tanh"
    if args.no_skip:
        name += " no skip term"
    if custom:
        name += " per-step weight_c"
    x_f32 = args.x_f32 and es == 2 and use_x
    if x_f32:
        name += " float32 x"
    shape = _lib.Shape(L, B, d, dirs, k, 1 if args.tanh else 0,
                       0 if args.no_skip else (1 if k == 3 else 2), 1 if custom else 0, CODE[args.dtype],
                       _lib.STATE_INTERVAL if ckpt else 1, _lib.X_F32 if x_f32 else _lib.X_AS_STREAMS)
    xdt = torch.float32 if x_f32 else tdt
    xs = 4 if x_f32 else es   # bytes per element of x and grad_x
    state_rows = lib.sru_amd_state_bytes(ctypes.byref(shape)) // (B * Dp * (4 if ckpt else DT_BYTES[args.dtype]))

    g = torch.Generator(device=dev).manual_seed(1234)
    sets = []
    for _ in range(args.sets):
        s = dict(
            U=torch.randn(L, B, Dp * k, device=dev, generator=g).to(tdt),
            x=torch.randn(L, B, Dp, device=dev, generator=g).to(xdt),
            gh=torch.randn(L, B, Dp, device=dev, generator=g).to(tdt),
            h=torch.empty(L, B, Dp, device=dev, dtype=tdt),
            c=torch.empty(state_rows, B, Dp, device=dev, dtype=torch.float32 if ckpt else tdt),
            gu=torch.empty(L, B, Dp * k, device=dev, dtype=tdt),
            gx=torch.empty(L, B, Dp, device=dev, dtype=xdt),
        )
        sets.append(s)
    wc = ((torch.rand(2 * Dp, device=dev, generator=g) * 2 - 1) * 1.5 ** 0.5).to(sdt)
    if custom:
        wc = (wc.view(2, Dp).t().reshape(1, 1, 2 * Dp) + 0.1 * torch.randn(L, B, 2 * Dp, device=dev, generator=g)).to(tdt)
    bias = torch.zeros(2 * Dp, device=dev, dtype=sdt)
    c0 = torch.zeros(B, Dp, device=dev, dtype=sdt)
    gl = torch.zeros(B, Dp, device=dev, dtype=sdt)
    scale = torch.tensor([3 ** 0.5], device=dev, dtype=sdt)
    c_last = torch.empty(B, Dp, device=dev, dtype=sdt)
    pad = None
    if padded:
        lens = torch.randint(L // 4, L + 1, (B,), device=dev, generator=g)
        if args.fixed_length:
            lens = torch.full((B,), args.fixed_length, device=dev)
        pad = (torch.arange(L, device=dev)[:, None] >= lens[None, :]).view(torch.uint8).contiguous()
    gwc = torch.empty(L, B, 2 * Dp, device=dev, dtype=tdt) if custom else torch.empty(2 * Dp, device=dev, dtype=sdt)
    gb = torch.empty(2 * Dp, device=dev, dtype=sdt)
    gi = torch.empty(B, Dp, device=dev, dtype=sdt)
    ws_bytes = lib.sru_amd_backward_workspace_bytes(ctypes.byref(shape))
    ws = torch.empty(ws_bytes // 4, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    on = [stream]   # the stream the calls are issued on (the capture stream while a graph is recorded)

    def fwd(s):
        rc = lib.sru_amd_forward(ctypes.byref(shape), p(s["U"]), p(s["x"]) if use_x else None, p(wc), p(bias),
                                 p(c0), None, p(pad), p(scale) if use_x else None, p(s["h"]),
                                 None if fwd_only else p(s["c"]), p(c_last), on[0])
        assert rc == 0, _lib.status_string(rc)

    def bwd(s):
        if fwd_only:
            return
        rc = lib.sru_amd_backward(ctypes.byref(shape), p(s["U"]), p(s["x"]) if use_x else None, p(wc), p(bias),
                                  p(c0), None, p(pad), p(scale) if use_x else None, p(s["c"]), p(s["gh"]),
                                  p(gl), p(s["gu"]), p(s["gx"]) if use_x else None,
                                  p(gwc), p(gb), p(gi), p(ws), ctypes.c_size_t(ws_bytes), on[0])
        assert rc == 0, _lib.status_string(rc)

    copy_cal = None
    if args.calibrate_copy:
        n = 1 << 28                                    # 2^28 floats = 1 GiB read + 1 GiB written
        src = torch.randn(n, device=dev)
        dst = torch.empty_like(src)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        dst.copy_(src)
        e0.record()
        for _ in range(5):
            dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / 5
        copy_cal = {"bytes_read": 4 * n, "bytes_written": 4 * n, "avg_us": us,
                    "GBps": 8 * n / (us * 1e-6) / 1e9, "frac_of_hbm_peak": 8 * n / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
        del src, dst

    # The backward call of a step works on the buffer set whose forward call ran half a
    # rotation earlier, so it cannot find operands the forward call just left in the caches.
    lag = args.sets // 2
    for s in sets:
        fwd(s)              # every set holds a valid per-step state before any backward call
    for i in range(args.warmup):
        fwd(sets[i % args.sets])
        bwd(sets[(i + lag) % args.sets])
    if args.graph:
        # Side measurement: one rotation of the buffer sets (forward + backward calls) recorded into
        # a HIP graph and replayed. The entry points neither allocate nor synchronise, so the calls
        # record as they are; what the replay removes is the host-side gap between dependent launches.
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            on[0] = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
            for i in range(args.sets):
                fwd(sets[i])
                bwd(sets[(i + lag) % args.sets])
        on[0] = stream
        replays = max(1, args.steps // args.sets)
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        ms_step = (time.perf_counter() - t0) * 1e3 / (replays * args.sets)
        print(json.dumps({"metric": "recurrence tokens/s, calls replayed from a HIP graph (side measurement)",
                          "value": L * B / (ms_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": replays * args.sets,
                          "warmup": args.warmup, "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak",
                          "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
                          "config": {"workload": name, "pass": "forward only" if fwd_only else "forward+backward, one layer",
                                     "replayed_from_graph": True, "calls_per_graph": args.sets}}), flush=True)
        return
    # events live on the stream the kernels are launched on (torch's current stream)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        ev[i][0].record()
        fwd(sets[i % args.sets])
        ev[i][1].record()
        bwd(sets[(i + lag) % args.sets])
        ev[i][2].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    ms_step = (t1 - t0) * 1e3 / args.steps
    fwd_us = 1e3 * sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    bwd_us = 1e3 * sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    # spread of the timed region: per-step times between the events that open consecutive steps
    # (the last step: from its own first to its last event)
    per_step = [ev[i][0].elapsed_time(ev[i + 1][0]) for i in range(args.steps - 1)] + [ev[-1][0].elapsed_time(ev[-1][2])]
    spread = {"min": min(per_step), "median": float(np.median(per_step)), "max": max(per_step),
              "source": "HIP events on the launch stream, one value per timed step"}
    # HBM bytes per backward launch as the hardware counters saw them: NOT measured by this run
    # (counters need a rocprofv3 --pmc session) but replayed from the committed summary of such
    # sessions on this same command; the file is named in the output
    traffic, traffic_source = None, None
    tfile = os.path.join(ROOT, "profiles", "traffic_bi_d1024_L256_B64_%s.json" % args.dtype)
    if args.workload == "headline" and ckpt and not args.tanh and not args.no_skip and not custom \
            and os.path.exists(tfile):
        rec = json.load(open(tfile))
        traffic = rec["backward_scan"]["traffic_bytes"]
        traffic_source = ("replayed from profiles/%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, %s); "
                          "not measured in this run" % (os.path.basename(tfile), rec.get("measured", "date not recorded")))
    # Reference algorithm (what `achieved` and `frac` are priced on): forward reads U (k) and x (k=3
    # with a skip term), writes h and (training) the state c after every step; backward reads U (k),
    # x, c, grad_h and writes grad_u (k), grad_x.
    # (a per-step weight_c is one more stream of 2 elements per cell: read by both passes, its
    # gradient written by the backward pass)
    fwd_bytes = (k + (1 if fwd_only else 2) + (2 if custom else 0)) * es * cells + (xs * cells if use_x else 0)
    bwd_bytes = (2 * k + 2 + (4 if custom else 0)) * es * cells + (2 * xs * cells if use_x else 0)
    # What the selected kernels are built to move: with checkpoints the per-step state (es bytes per
    # cell each way) shrinks to one float per 8 steps.
    state_bytes = (4 * cells // 8) if ckpt else es * cells
    # Padding at the ends of a batch row's sequence is skipped in chunks of 8 steps by the kernels
    # whose wavefronts lie inside one batch row: those cells cost their output bytes only.
    live_f = live_b = 1.0
    if padded:
        walked = torch.clamp((lens + 7) // 8 * 8, max=L).sum().item() / float(L * B)
        sixteen = es == 2
        lane_pairs = sixteen and d % 32 == 0 and ncols // 32 <= 1024 and (ckpt or fwd_only)   # those kernels walk every step
        cols = 2 if sixteen and ncols // 2 >= 65536 else 1
        uniform = d % (64 * cols) == 0 and not lane_pairs and not (custom and args.tanh)
        live_f = walked if uniform else 1.0
        live_b = walked if uniform and ckpt else 1.0   # (the state-after-every-step backward kernel walks every step)
    fwd_in = (k + (2 if custom else 0)) * es * cells + (xs * cells if use_x else 0)
    bwd_in = (k + 1 + (2 if custom else 0)) * es * cells + (xs * cells if use_x else 0) + state_bytes
    fwd_moved = int(fwd_in * live_f) + es * cells + (0 if fwd_only else state_bytes)
    bwd_moved = int(bwd_in * live_b) + (k + (2 if custom else 0)) * es * cells + (xs * cells if use_x else 0)
    if fwd_only:
        bwd_us = float("nan")
    bwd_gbs = bwd_bytes / (bwd_us * 1e-6) / 1e9
    gbs = lambda nbytes, us: nbytes / (us * 1e-6) / 1e9
    out = {
        "metric": "recurrence tokens/sec & HBM GB/s (%peak), bi-SRU d=1024 L=256 B=64",
        "value": L * B / (ms_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "ms_per_step_spread": spread,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": name, "length": L, "batch": B, "hidden_per_direction": d,
                   "directions": dirs, "k": k, "pass": "forward only, one layer" if fwd_only else "forward+backward, one layer",
                   "state_between_passes": "float checkpoints every 8 steps" if ckpt else "every step",
                   "buffer_sets": args.sets},
        "roofline": {"bound": "hbm", "kernel": ("backward_scan_ckpt" if ckpt else "backward_scan") + " (+ reduce_partials)",
                     "achieved": bwd_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": bwd_gbs / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_source": traffic_source,
                     "traffic_GBps": None if traffic is None else gbs(traffic, bwd_us),
                     "actual_frac": None if traffic is None else gbs(traffic, bwd_us) / HBM_PEAK_GBS,
                     "algorithmic_bytes_per_launch": bwd_bytes,
                     "moved_bytes_per_launch": bwd_moved,
                     "moved_frac": gbs(bwd_moved, bwd_us) / HBM_PEAK_GBS,
                     "walked_cell_fraction": {"forward": live_f, "backward": live_b},
                     "note": "achieved / frac price the reference algorithm's bytes (state after every step written "
                             "and read); moved_* price what the selected kernels move (state checkpoints), "
                             "actual_frac the counter-measured traffic",
                     "avg_us": bwd_us},
        "kernels": {
            "forward_scan": {"avg_us": fwd_us, "algorithmic_GBps": gbs(fwd_bytes, fwd_us),
                             "frac_of_hbm_peak": gbs(fwd_bytes, fwd_us) / HBM_PEAK_GBS,
                             "moved_frac_of_hbm_peak": gbs(fwd_moved, fwd_us) / HBM_PEAK_GBS},
            "backward_scan+reduce": {"avg_us": bwd_us, "algorithmic_GBps": bwd_gbs,
                                     "frac_of_hbm_peak": bwd_gbs / HBM_PEAK_GBS,
                                     "moved_frac_of_hbm_peak": gbs(bwd_moved, bwd_us) / HBM_PEAK_GBS},
            "forward+backward": {"avg_us": fwd_us + bwd_us,
                                 "algorithmic_GBps": gbs(fwd_bytes + bwd_bytes, fwd_us + bwd_us),
                                 "frac_of_hbm_peak": gbs(fwd_bytes + bwd_bytes, fwd_us + bwd_us) / HBM_PEAK_GBS,
                                 "moved_frac_of_hbm_peak": gbs(fwd_moved + bwd_moved, fwd_us + bwd_us) / HBM_PEAK_GBS},
        },
    }
    if copy_cal is not None:
        out["copy_calibration"] = copy_cal
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(L, B, d, dirs, k)
    if fwd_only:   # side measurement: the forward scan is the only kernel
        out["roofline"].update(kernel="forward_scan (inference, no state store)",
                               achieved=out["kernels"]["forward_scan"]["algorithmic_GBps"],
                               frac=out["kernels"]["forward_scan"]["frac_of_hbm_peak"],
                               algorithmic_bytes_per_launch=fwd_bytes, moved_bytes_per_launch=fwd_moved,
                               moved_frac=gbs(fwd_moved, fwd_us) / HBM_PEAK_GBS, avg_us=fwd_us)
        for key in ("backward_scan+reduce", "forward+backward"):
            out["kernels"].pop(key)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
