"""CPU restatement of a stack of SRU layers on top of the oracle's differentiable recurrence
(test infrastructure). Runs a sru_amd.modules.SRU's parameters through
x -> [pre-LN] -> U = x @ W -> recurrence -> [post-LN], layer by layer, in float64, following
sru/modules.py:235-281 and :617-652 (eval mode: no dropout masks)."""
import torch
import torch.nn.functional as F

from oracle import sru_torch as st


def stack_forward(model, x, c0=None, mask_pad=None, dtype=torch.float64):
    """Returns (h, c_stack) and leaves autograd history on copies of the parameters, which are
    returned as a dict name -> tensor (requires_grad) for gradient comparison."""
    params = {n: p.detach().to("cpu", dtype).requires_grad_(True) for n, p in model.named_parameters()}
    x = x.detach().to("cpu", dtype)
    if model.input_to_hidden is not None:
        x = x @ params["input_to_hidden.weight"].t()
    finals = []
    for i, cell in enumerate(model.rnn_lst):
        g = lambda n: params[f"rnn_lst.{i}.{n}"]
        residual = x
        inp = x
        if cell.layer_norm is not None and not cell.normalize_after:
            inp = F.layer_norm(inp, (inp.size(-1),), g("layer_norm.weight"), g("layer_norm.bias"))
        L, B = inp.shape[0], inp.shape[1]
        flat = inp.reshape(L * B, -1)
        if cell.projection_size:
            flat = flat @ g("weight_proj")
        U = (flat @ g("weight")).reshape(L, B, -1)
        init = torch.zeros(B, cell.output_size, dtype=dtype) if c0 is None else c0[i].detach().to("cpu", dtype)
        scale = cell.scale_x.detach().to("cpu", dtype) if cell.rescale else None
        h, c = st.recurrence(U, residual, g("weight_c"), g("bias"), init, cell.activation_type,
                             cell.hidden_size, cell.bidirectional, cell.has_skip_term, scale, None,
                             None if mask_pad is None else mask_pad.cpu())
        if cell.layer_norm is not None and cell.normalize_after:
            h = F.layer_norm(h, (h.size(-1),), g("layer_norm.weight"), g("layer_norm.bias"))
        x = h
        finals.append(c)
    return x, torch.stack(finals), params
