"""The reference workloads at their real sizes (the long-sequence one at a reduced batch).

* "config 4": language-model-scale stack, 10 unidirectional layers, hidden 2048, projection 512,
  L=512, B=16, bf16 autocast, dropout 0.1 (a per-layer mask_c), inputs = embedding rows N(0, 0.02).
  One layer's recurrence is 32 768 columns = 512 wavefronts: the shape where 16-bit streams run
  the lane-pairing kernels.
* "config 3": classification-scale stack, 4 bidirectional layers, d=1024, L=256, B=64, layer norm,
  rescale, fp32 and bf16 autocast.
* "config 1": the README example, 2 unidirectional layers, input = hidden = 128, L=20, B=32, fp32,
  highway_bias=-2, forward only.
* "config 2": 4 bidirectional layers, input = hidden = 512, L=128, B=32, fp32, forward + backward,
  right-padded batch with lengths in [32, 128], loss = sum(h * probe).
* "config 5": long-sequence inference, 2 bidirectional layers, d=256, L=4096, fp16 weights and
  inputs, no_grad, lengths in [1024, 4096], c0 ~ N(0,1); batch 16 instead of 256 so that the
  float64 host oracle finishes in seconds (the one-layer recurrence runs at B=256 in
  tests/test_gpu_fullsize.py).

Op level: the kernels through the C ABI against the float64 oracle on identical (rounded) inputs.
Module level: the whole stack against a float64 restatement (dense products in float64 on the
GPU by torch, recurrence by the C oracle on the host). Bound for 16-bit runs: 2e-2 * max|ref|,
the bar the build states for bf16 / fp16 AMP; the measured figures are printed.
"""
import numpy as np
import pytest
import torch

from sru_amd.modules import SRU
from tests.cases import Case
from tests.stack_ref import record_dropout_masks, stack_forward_large
from tests.test_gpu_parity import check_against_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("checkpointed", [False, True], ids=["state_every_step", "state_checkpoints"])
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_config_4_layer_recurrence_against_float64_oracle(dt, checkpointed):
    c = Case(L=512, B=16, d=2048, dirs=1, k=3, seed=41, mask_c=True, zero_c0=True)
    check_against_oracle(c.f32() if dt == "f32" else c, dt, checkpointed=checkpointed)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_config_4_last_layer_without_dropout_mask_and_k4_first_layer(dt):
    # the last layer of a stack draws no mask (sru/modules.py:554); a first layer fed by a
    # narrower embedding has four streams
    check_against_oracle(Case(L=512, B=16, d=2048, dirs=1, k=3, seed=42, zero_c0=True), dt, checkpointed=True)
    check_against_oracle(Case(L=512, B=16, d=2048, dirs=1, k=4, seed=43, mask_c=True, zero_c0=True), dt,
                         checkpointed=True)


def _rel(got, ref):
    ref = ref.detach().double().cpu()
    return float((got.detach().double().cpu() - ref).abs().max()) / max(float(ref.abs().max()), 1e-30)


def _config_4_model(native_16bit):
    torch.manual_seed(404)
    model = SRU(2048, 2048, num_layers=10, projection_size=512, dropout=0.1,
                native_16bit=native_16bit).to(DEV)
    table = torch.randn(50000, 2048, device=DEV) * 0.02
    ids = torch.randint(0, 50000, (512, 16), device=DEV)
    return model, table[ids]


@pytest.mark.parametrize("native_16bit", [True, False], ids=["native_16bit", "reference_casts"])
def test_config_4_stack_eval_bf16_drift_over_10_layers(native_16bit):
    model, x = _config_4_model(native_16bit)
    model.eval()
    with torch.no_grad():
        h_ref, c_ref, _ = stack_forward_large(model, x, device=DEV)
        h32, c32 = model(x)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            h16, c16 = model(x)
    assert h16.dtype == (torch.bfloat16 if native_16bit else torch.float32)
    e32, e16, ec = _rel(h32, h_ref), _rel(h16, h_ref), _rel(c16, c_ref)
    print(f"\nconfig 4, eval, 10 layers, native_16bit={native_16bit}: max|h - float64| / max|float64| "
          f"float32 run {e32:.3g}, bf16 autocast run {e16:.3g} (final states {ec:.3g}); "
          f"bf16 run vs float32 run {_rel(h16, h32):.3g}")
    assert e32 <= 1e-4
    assert e16 <= 2e-2 and ec <= 2e-2 and _rel(h16, h32) <= 2e-2


def test_config_4_stack_training_step_bf16_against_float64_with_the_same_masks():
    model, x = _config_4_model(True)
    model.train()
    undo = record_dropout_masks(model)
    torch.manual_seed(1)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        h16, _ = model(x)
    probe = torch.randn(h16.shape, device=DEV)
    (h16.float() * probe).sum().backward()
    undo()
    masks = [cell.drawn_masks[0] if cell.drawn_masks else None for cell in model.rnn_lst]
    assert all(m is not None for m in masks[:-1]) and masks[-1] is None
    h_ref, _, params = stack_forward_large(model, x, masks=masks, device=DEV)
    (h_ref * probe.double()).sum().backward()
    print(f"\nconfig 4, training step, bf16 autocast vs float64: h {_rel(h16, h_ref):.3g}")
    assert _rel(h16, h_ref) <= 2e-2
    worst = 0.0
    for name, p in model.named_parameters():
        e = _rel(p.grad, params[name].grad)
        worst = max(worst, e)
        assert e <= 3e-2, (name, e)
    print(f"parameter gradients, worst max-abs error / max|ref| over {len(params)} tensors: {worst:.3g}")


@pytest.mark.parametrize("amp", [None, torch.bfloat16], ids=["fp32", "bf16_autocast"])
def test_config_3_stack_with_layer_norm_and_rescale(amp):
    torch.manual_seed(303)
    model = SRU(1024, 1024, num_layers=4, bidirectional=True, layer_norm=True, rescale=True).to(DEV)
    # input width 1024 against output width 2048: the first layer carries four streams
    x = torch.randn(256, 64, 1024, device=DEV)
    if amp is None:
        h, c = model(x)
    else:
        with torch.autocast("cuda", dtype=amp):
            h, c = model(x)
    probe = torch.randn(h.shape, device=DEV)
    (h.float() * probe).sum().backward()
    h_ref, c_ref, params = stack_forward_large(model, x, device=DEV)
    (h_ref * probe.double()).sum().backward()
    eh, ec = _rel(h, h_ref), _rel(c, c_ref)
    worst = max(_rel(p.grad, params[n].grad) for n, p in model.named_parameters())
    print(f"\nconfig 3 stack ({'fp32' if amp is None else 'bf16 autocast'}): h {eh:.3g}, final states {ec:.3g}, "
          f"worst parameter gradient {worst:.3g} (max-abs error / max|ref|)")
    if amp is None:
        assert eh <= 1e-4 and ec <= 1e-4 and worst <= 1e-3
    else:
        assert eh <= 2e-2 and ec <= 2e-2 and worst <= 3e-2


def test_config_1_readme_example_forward():
    torch.manual_seed(101)
    model = SRU(128, 128, num_layers=2, highway_bias=-2.0).to(DEV).eval()
    x = torch.randn(20, 32, 128, device=DEV)
    with torch.no_grad():
        h, c = model(x)
        h_ref, c_ref, _ = stack_forward_large(model, x, device=DEV)
    eh = float((h.double() - h_ref).abs().max())
    ec = float((c.double() - c_ref).abs().max())
    print(f"\nconfig 1 stack (fp32, forward): max abs error h {eh:.3g}, final states {ec:.3g}")
    assert h.shape == (20, 32, 128) and c.shape == (2, 32, 128)
    assert eh <= 1e-5 and ec <= 1e-5


def test_config_2_stack_padded_batch_forward_and_backward():
    torch.manual_seed(202)
    L, B = 128, 32
    model = SRU(512, 512, num_layers=4, bidirectional=True).to(DEV)
    x = torch.randn(L, B, 512, device=DEV)
    lens = torch.randint(32, L + 1, (B,), device=DEV)
    lens[0] = L
    mask_pad = torch.arange(L, device=DEV)[:, None] >= lens[None, :]
    h, c = model(x, mask_pad=mask_pad)
    probe = torch.randn(h.shape, device=DEV)
    (h * probe).sum().backward()
    h_ref, c_ref, params = stack_forward_large(model, x, mask_pad=mask_pad, device=DEV)
    (h_ref * probe.double()).sum().backward()
    eh, ec = _rel(h, h_ref), _rel(c, c_ref)
    worst = max(_rel(p.grad, params[n].grad) for n, p in model.named_parameters())
    print(f"\nconfig 2 stack (fp32, lengths in [32, 128]): h {eh:.3g}, final states {ec:.3g}, "
          f"worst parameter gradient {worst:.3g} (max-abs error / max|ref|)")
    # every layer zeroes its padded outputs
    assert float(h[mask_pad].abs().max()) == 0.0
    assert eh <= 1e-5 and ec <= 1e-5 and worst <= 1e-4


def test_config_5_stack_long_sequence_fp16_inference():
    torch.manual_seed(505)
    L, B = 4096, 16
    model = SRU(256, 256, num_layers=2, bidirectional=True).to(DEV).half().eval()
    x = torch.randn(L, B, 256, device=DEV).half()
    c0 = torch.randn(2, B, 512, device=DEV).half()
    lens = torch.randint(1024, L + 1, (B,), device=DEV)
    lens[0] = L
    mask_pad = torch.arange(L, device=DEV)[:, None] >= lens[None, :]
    with torch.no_grad():
        h, c = model(x, c0, mask_pad=mask_pad)
        h_ref, c_ref, _ = stack_forward_large(model, x, mask_pad=mask_pad, device=DEV, c0=c0)
    assert h.dtype == torch.float16 and c.dtype == torch.float16
    eh, ec = _rel(h, h_ref), _rel(c, c_ref)
    print(f"\nconfig 5 stack (fp16, L=4096, B={B}): h {eh:.3g}, final states {ec:.3g} (max-abs error / max|ref|)")
    assert float(h[mask_pad].abs().max()) == 0.0
    assert eh <= 2e-2 and ec <= 2e-2
