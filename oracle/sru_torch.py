"""Differentiable torch restatement of the recurrence: TEST INFRASTRUCTURE ONLY.

Same argument list and return as the reference's autograd entry
(sru/cuda_functional.py:159-167 -> (h, last_hidden)); the arithmetic is the
definitional CPU path of sru/ops.py:145-250 (view U as (L,B,dirs,d,k), second
direction walks time backwards, a padded step keeps the previous state and
emits h = 0). It exists so that autograd and torch.autograd.gradcheck can pin
the analytic backward of the C oracle; it runs in whatever dtype it is given
(float64 in the tests).
"""
from typing import Optional, Tuple

import torch
from torch import Tensor


def recurrence(u: Tensor, x: Tensor, weight_c: Tensor, bias: Tensor, init: Tensor,
               activation_type: int, d_out: int, bidirectional: bool, has_skip_term: bool,
               scale_x: Optional[Tensor] = None, mask_c: Optional[Tensor] = None,
               mask_pad: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    dirs = 2 if bidirectional else 1
    d = d_out
    B = x.size(-2)
    L = x.size(0) if x.dim() == 3 else 1
    k = u.size(-1) // (d * dirs)
    custom = weight_c.dim() > 1
    u = u.reshape(L, B, dirs, d, k)
    if custom:
        v = weight_c.reshape(L, B, dirs, d, 2)
    else:
        wc = weight_c.reshape(2, dirs, d)
    bs = bias.reshape(2, dirs, d)
    if not has_skip_term:
        skip = None
    elif k == 3:
        skip = x.reshape(L, B, dirs, d)
        if scale_x is not None:
            skip = skip * scale_x
    else:
        skip = u[..., 3]
    m = None if mask_c is None else mask_c.reshape(B, dirs, d)
    pad = None if mask_pad is None else (mask_pad != 0).reshape(L, B, 1)

    h_rows = [[None] * L for _ in range(dirs)]
    finals = []
    for di in range(dirs):
        state = init.reshape(B, dirs, d)[:, di]
        order = range(L) if di == 0 else range(L - 1, -1, -1)
        for t in order:
            w1 = v[t, :, di, :, 0] if custom else wc[0, di]
            w2 = v[t, :, di, :, 1] if custom else wc[1, di]
            f = torch.sigmoid(u[t, :, di, :, 1] + w1 * state + bs[0, di])
            r = torch.sigmoid(u[t, :, di, :, 2] + w2 * state + bs[1, di])
            new = (state - u[t, :, di, :, 0]) * f + u[t, :, di, :, 0]
            val = torch.tanh(new) if activation_type == 1 else new
            if m is not None:
                r = r * m[:, di]
            out = (val - skip[t, :, di]) * r + skip[t, :, di] if skip is not None else val * r
            if pad is not None:
                new = torch.where(pad[t], state, new)
                out = torch.where(pad[t], torch.zeros_like(out), out)
            state = new
            h_rows[di][t] = out
        finals.append(state)
    h = torch.stack([torch.stack(rows, 0) for rows in h_rows], 2).reshape(L, B, dirs * d)
    last = torch.stack(finals, 1).reshape(B, dirs * d)
    if x.dim() == 2:
        h = h.squeeze(0)
    return h, last
