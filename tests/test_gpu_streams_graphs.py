"""The entry points only enqueue kernels on the stream they are given: they can run on a
side stream and be recorded into a HIP graph (no allocation, no memset, no host sync)."""
import ctypes

import pytest
import torch

from sru_amd import _lib, ElementwiseRecurrence
from tests.abi import DeviceProblem
from tests.cases import Case

pytestmark = pytest.mark.gpu


def test_side_stream_matches_default_stream():
    c = Case(L=40, B=4, d=128, dirs=2, seed=61, pad="right", scale=1.7)
    dp = DeviceProblem(c, checkpointed=True)
    ref = [t.clone() for t in dp.forward()] + [t.clone() for t in dp.backward()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        got = list(dp.forward()) + list(dp.backward())
    side.synchronize()
    for a, b in zip(ref, got):
        assert torch.equal(a, b)


def test_forward_and_backward_replay_from_a_graph():
    c = Case(L=33, B=4, d=128, dirs=2, seed=62, pad="right", scale=1.7, mask_c=True)
    dp = DeviceProblem(c, checkpointed=True)
    eager = [t.clone() for t in dp.forward(poison=False)] + [t.clone() for t in dp.backward(poison=False)]
    torch.cuda.synchronize()
    # static buffers: the graph replays the same pointers
    outs = [dp.h, dp.c, dp.c_last, dp.gu, dp.gx, dp.gwc, dp.gb, dp.gi]
    lib = _lib.load()
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    nbytes = lib.sru_amd_backward_workspace_bytes(ctypes.byref(dp.shape))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.sru_amd_forward(ctypes.byref(dp.shape), p(dp.U), p(dp.x), p(dp.wc), p(dp.bias), p(dp.c0),
                                 p(dp.mask_c), p(dp.pad), p(dp.scale), p(dp.h), p(dp.c), p(dp.c_last), stream)
        assert rc == 0
        rc = lib.sru_amd_backward(ctypes.byref(dp.shape), p(dp.U), p(dp.x), p(dp.wc), p(dp.bias), p(dp.c0),
                                  p(dp.mask_c), p(dp.pad), p(dp.scale), p(dp.c), p(dp.gh), p(dp.gl),
                                  p(dp.gu), p(dp.gx), p(dp.gwc), p(dp.gb), p(dp.gi), p(dp.ws),
                                  ctypes.c_size_t(nbytes), stream)
        assert rc == 0
    for replay in range(3):
        for t in outs:
            t.fill_(float("nan"))          # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager, outs):
            assert torch.equal(a, b), replay
    # new inputs in the same buffers: the replay follows them
    dp.U.mul_(0.5)
    graph.replay()
    torch.cuda.synchronize()
    replayed = [t.clone() for t in outs]
    again = [t.clone() for t in dp.forward(poison=False)] + [t.clone() for t in dp.backward(poison=False)]
    for a, b in zip(again, replayed):
        assert torch.equal(a, b)


def test_autograd_function_on_second_device_stream_and_noncontiguous_inputs():
    c = Case(L=12, B=3, d=64, dirs=2, seed=63, scale=1.3).f32()
    dev = "cuda:0"
    t = lambda a: torch.tensor(a, dtype=torch.float32, device=dev)
    u, x, wc, bias, c0 = t(c.U), t(c.x), t(c.wc), t(c.bias), t(c.c0)
    sx = torch.tensor([c.scale], device=dev)
    h_ref, last_ref = ElementwiseRecurrence.apply(u, x, wc, bias, c0, 0, c.d, True, True, sx)
    # U as a transposed view, x with a storage offset: the wrapper makes them contiguous / aligned
    u_view = u.transpose(0, 1).contiguous().transpose(0, 1)
    x_off = torch.cat([torch.zeros(1, device=dev), x.reshape(-1)])[1:].view_as(x)
    assert not u_view.is_contiguous() and x_off.data_ptr() % 16 != 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        h, last = ElementwiseRecurrence.apply(u_view, x_off, wc, bias, c0, 0, c.d, True, True, sx)
    side.synchronize()
    assert torch.equal(h, h_ref) and torch.equal(last, last_ref)


def test_module_forward_replays_from_a_graph():
    """The README-example stack (2 layers, d=128, L=20, B=32) is launch-bound; the whole
    forward (GEMMs + recurrence) can be recorded once and replayed. Every replay is checked
    against the eager result for the input it is given."""
    import sru_amd
    torch.manual_seed(5)
    model = sru_amd.SRU(128, 128, num_layers=2, highway_bias=-2.0).cuda().eval()
    static_x = torch.randn(20, 32, 128, device="cuda")
    with torch.no_grad():
        side = torch.cuda.Stream()          # warm-up on a side stream, as torch asks before a capture
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                model(static_x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_h, static_c = model(static_x)
        for replay in range(3):
            x = torch.randn(20, 32, 128, device="cuda")
            h_eager, c_eager = model(x)          # eager work and a sync between replays
            torch.cuda.synchronize()
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_h, h_eager), replay
            assert torch.equal(static_c, c_eager), replay


def test_two_host_threads_on_two_streams():
    """The library keeps no state between calls: two host threads, each with its own stream and
    buffers, run forward + backward at the same time and get what they get alone."""
    import threading
    cases = [Case(L=48, B=4, d=128, dirs=2, seed=71, pad="right", scale=1.7),
             Case(L=40, B=3, d=192, dirs=1, k=4, seed=72, mask_c=True)]
    problems = [DeviceProblem(c, checkpointed=True) for c in cases]
    alone = []
    for dp in problems:
        alone.append([t.clone() for t in dp.forward()] + [t.clone() for t in dp.backward() if t is not None])
    torch.cuda.synchronize()
    together = [None, None]
    errors = []

    def work(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(20):
                    out = list(problems[i].forward()) + [t for t in problems[i].backward() if t is not None]
            stream.synchronize()
            together[i] = out
        except Exception as e:      # surfaced below, in the test's own thread
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for a, b in zip(alone, together):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


def _timed(fn, n=200):
    import time
    for _ in range(10):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e6 / n


def test_graphed_helper_forward_only_readme_example():
    """sru_amd.graphed on the README-example stack in eval mode: every replay equals the eager result
    for the input it is given (with eager work and a sync in between), and a replay is faster than
    the eager call it replaces (the eager call is all host-side launch work at this size)."""
    import sru_amd
    torch.manual_seed(6)
    model = sru_amd.SRU(128, 128, num_layers=2, highway_bias=-2.0).cuda().eval()
    x0 = torch.randn(20, 32, 128, device="cuda")
    with torch.no_grad():
        fast = sru_amd.graphed(model, x0)
        assert not fast.training
        for replay in range(3):
            x = torch.randn(20, 32, 128, device="cuda")
            h_eager, c_eager = model(x)
            torch.cuda.synchronize()
            h, c = fast(x)
            torch.cuda.synchronize()
            assert torch.equal(h, h_eager) and torch.equal(c, c_eager), replay
        eager_us = _timed(lambda: model(x0))
        replay_us = _timed(lambda: fast(x0))
    print(f"\nREADME-example stack, forward: eager {eager_us:.1f} us per call, graph replay {replay_us:.1f} us")
    assert replay_us < eager_us
    with pytest.raises(ValueError):
        fast(torch.randn(21, 32, 128, device="cuda"))
    with pytest.raises(ValueError):
        fast(x0, mask_pad=torch.zeros(20, 32, dtype=torch.bool, device="cuda"))


def test_graphed_helper_training_step_padded_stack():
    """Forward and backward of a padded bidirectional stack (the 4-layer d=512 L=128 B=32
    configuration at half its depth and batch) recorded with sru_amd.graphed in training mode:
    outputs and every parameter gradient of three replays on fresh inputs against eager runs."""
    import sru_amd
    torch.manual_seed(8)
    L, B = 128, 16
    model = sru_amd.SRU(512, 512, num_layers=2, bidirectional=True).cuda().train()
    mk_mask = lambda: torch.arange(L, device="cuda")[:, None] >= torch.randint(32, L + 1, (B,), device="cuda")[None, :]
    x0, m0 = torch.randn(L, B, 512, device="cuda"), mk_mask()
    fast = sru_amd.graphed(model, x0, mask_pad=m0)
    assert fast.training
    for replay in range(3):
        x, m = torch.randn(L, B, 512, device="cuda"), mk_mask()
        probe = torch.randn(L, B, 1024, device="cuda")
        model.zero_grad(set_to_none=True)
        h, c = model(x, mask_pad=m)
        ((h * probe).sum() + c.sum()).backward()
        eager = [h.detach().clone(), c.detach().clone()] + [p.grad.clone() for p in model.parameters()]
        model.zero_grad(set_to_none=True)
        torch.cuda.synchronize()
        h, c = fast(x, mask_pad=m)
        ((h * probe).sum() + c.sum()).backward()
        torch.cuda.synchronize()
        got = [h.detach(), c.detach()] + [p.grad for p in model.parameters()]
        for a, b in zip(got, eager):
            assert float((a - b).abs().max()) <= 1e-6 * max(1.0, float(b.abs().max())), replay
