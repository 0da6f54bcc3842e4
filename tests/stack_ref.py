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


class OracleRecurrence(torch.autograd.Function):
    """The C oracle (float64, on the host) as an autograd node, for stacks too large for the
    Python loop of oracle/sru_torch.py. Tensors may live on any device; vector weight_c only."""

    @staticmethod
    def forward(ctx, u, x, weight_c, bias, init, activation_type, d, bidirectional, has_skip_term,
                scale_x, mask_c, mask_pad):
        from oracle import sru_oracle as so
        dirs = 2 if bidirectional else 1
        k, skip_type, custom = so.derive(u.size(-1), d, dirs, has_skip_term, weight_c.dim())
        assert not custom
        n = lambda t: None if t is None else t.detach().double().cpu().numpy()
        kw = dict(d=d, dirs=dirs, k=k, activation_type=activation_type, skip_type=skip_type,
                  scale_x=1.0 if scale_x is None else float(scale_x), mask_c=n(mask_c), mask_pad=n(mask_pad))
        args = (n(u), n(x), n(weight_c), n(bias), n(init))
        h, c_all, c_last = so.forward(*args, **kw)
        ctx.args, ctx.kw, ctx.c_all = args, kw, c_all
        ctx.dev, ctx.u_shape, ctx.x_shape = u.device, u.shape, x.shape
        t = lambda a: torch.from_numpy(a).to(u.device)
        return t(h), t(c_last)

    @staticmethod
    def backward(ctx, grad_h, grad_last):
        from oracle import sru_oracle as so
        n = lambda t: t.detach().double().cpu().numpy()
        gu, gx, gwc, gb, gi = so.backward(*ctx.args, ctx.c_all, n(grad_h), n(grad_last), **ctx.kw)
        t = lambda a: None if a is None else torch.from_numpy(a).to(ctx.dev)
        gx = t(gx)
        return (t(gu).view(ctx.u_shape), None if gx is None else gx.view(ctx.x_shape), t(gwc), t(gb), t(gi),
                None, None, None, None, None, None, None)


def record_dropout_masks(model):
    """Makes every layer of `model` remember the dropout masks it draws (in call order) in
    `cell.drawn_masks`; returns a function that removes the hooks again."""
    originals = []
    for cell in model.rnn_lst:
        cell.drawn_masks = []
        orig = cell._dropout_mask

        def wrapped(size, p, _orig=orig, _cell=cell):
            m = _orig(size, p)
            _cell.drawn_masks.append(m)
            return m
        cell._dropout_mask = wrapped
        originals.append((cell, orig))

    def undo():
        for cell, orig in originals:
            cell._dropout_mask = orig
    return undo


def stack_forward_large(model, x, mask_pad=None, masks=None, device="cuda:0", c0=None):
    """Float64 restatement of a whole stack at sizes where stack_forward is too slow: the dense
    products run in float64 on `device` (torch), the recurrence in the C oracle on the host.
    `masks`: per layer, the mask_c that layer drew in the run being checked (None = eval mode;
    rnn_dropout is not supported). `c0`: (layers, B, D') initial states or None for zeros.
    Returns (h, c_stack, params) like stack_forward."""
    dt = torch.float64
    params = {n: p.detach().to(device, dt).requires_grad_(True) for n, p in model.named_parameters()}
    x = x.detach().to(device, dt)
    if model.input_to_hidden is not None:
        x = x @ params["input_to_hidden.weight"].t()
    finals = []
    for i, cell in enumerate(model.rnn_lst):
        assert cell.custom_m is None and cell.rnn_dropout == 0
        g = lambda n: params[f"rnn_lst.{i}.{n}"]
        residual, inp = x, x
        if cell.layer_norm is not None and not cell.normalize_after:
            inp = F.layer_norm(inp, (inp.size(-1),), g("layer_norm.weight"), g("layer_norm.bias"))
        L, B = inp.shape[0], inp.shape[1]
        flat = inp.reshape(L * B, -1)
        if cell.projection_size:
            flat = flat @ g("weight_proj")
        U = (flat @ g("weight")).reshape(L, B, -1)
        init = torch.zeros(B, cell.output_size, dtype=dt, device=device) if c0 is None \
            else c0[i].detach().to(device, dt)
        scale = float(cell.scale_x.item()) if cell.rescale else None
        mask_c = None if masks is None or masks[i] is None else masks[i].detach().to(device, dt)
        h, c = OracleRecurrence.apply(U, residual, g("weight_c"), g("bias"), init, cell.activation_type,
                                      cell.hidden_size, cell.bidirectional, cell.has_skip_term, scale,
                                      mask_c, mask_pad)
        if cell.layer_norm is not None and cell.normalize_after:
            h = F.layer_norm(h, (h.size(-1),), g("layer_norm.weight"), g("layer_norm.bias"))
        x = h
        finals.append(c)
    return x, torch.stack(finals), params
