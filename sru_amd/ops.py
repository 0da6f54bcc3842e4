"""Call sites of the recurrence, mirroring sru/ops.py.

* elementwise_recurrence_gpu   (sru/ops.py:97-142): training entry under autograd.
* elementwise_recurrence_inference (sru/ops.py:22-94): forward only; here it
  also skips storing the per-step state, which the reference still writes.

Dtype policy. The reference casts every tensor to float32 unless
amp_recurrence_fp16 is set and U is float16 (sru/ops.py:116-127), because its
kernels compute in the tensor dtype. These kernels always compute in float32
whatever the stream dtype, so the `.float()` copies of U and x are not needed:
with `native_16bit=True` (default) a float16 / bfloat16 U is read as is and h
comes back in that dtype; `native_16bit=False` reproduces the reference's
float32 casts (h is then float32, as in the reference). Any other dtype (float64)
is cast to float32 as in the reference, and h is float32; double kernels exist
behind `ElementwiseRecurrence.apply` called directly, as in the reference.

`c_init` may be None (no counterpart in the reference): the kernels then start from zeros
without a zero tensor being allocated and filled.
"""
from typing import List, Optional

import torch
from torch import Tensor

from .functional import ElementwiseRecurrence, elementwise_recurrence_forward


def elementwise_recurrence_gpu(U: Tensor, x: Tensor, weight_c: Tensor, bias: Tensor,
                               c_init: Optional[Tensor], activation_type: int, hidden_size: int,
                               bidirectional: bool, has_skip_term: bool,
                               scale_x: Optional[Tensor] = None,
                               dropout_mask_c: Optional[Tensor] = None,
                               mask_pad: Optional[Tensor] = None,
                               amp_recurrence_fp16: bool = False,
                               native_16bit: bool = True) -> List[Tensor]:
    keep_16bit = native_16bit and U.dtype in (torch.float16, torch.bfloat16)
    if not keep_16bit and not (amp_recurrence_fp16 and U.dtype == torch.float16):
        # the reference's cast (sru/ops.py:116-127): everything to float32, float64 included, and
        # a float32 h comes back
        U, x = U.float(), x.float()
        if weight_c.dim() > 1:
            weight_c = weight_c.float()
    wants_grad = torch.is_grad_enabled() and any(
        t.requires_grad for t in (U, x, weight_c, bias, c_init) if t is not None)
    if not wants_grad:
        # Nothing will be differentiated (torch.no_grad(), or no input requires grad): same
        # results as the autograd Function, dropout mask included (the reference takes this
        # branch of sru/modules.py:296-304 for training-mode modules under no_grad as well),
        # without storing the state for a backward pass that cannot come.
        h, last_hidden, _ = elementwise_recurrence_forward(
            U, x, weight_c, bias, c_init, activation_type, hidden_size, bidirectional,
            has_skip_term, scale_x, dropout_mask_c, mask_pad, keep_c=False)
        return h, last_hidden
    return ElementwiseRecurrence.apply(U, x, weight_c, bias, c_init, activation_type,
                                       hidden_size, bidirectional, has_skip_term, scale_x,
                                       dropout_mask_c, mask_pad)


def elementwise_recurrence_inference(U: Tensor, x: Tensor, weight_c: Tensor, bias: Tensor,
                                     c_init: Tensor, activation_type: int, hidden_size: int,
                                     bidirectional: bool, has_skip_term: bool,
                                     scale_x: Optional[Tensor] = None,
                                     dropout_mask_c: Optional[Tensor] = None,
                                     mask_pad: Optional[Tensor] = None) -> List[Tensor]:
    # same refusal as sru/ops.py:38
    assert dropout_mask_c is None, "Dropout mask cannot be set during inference"
    with torch.no_grad():
        h, last_hidden, _ = elementwise_recurrence_forward(
            U, x, weight_c, bias, c_init, activation_type, hidden_size, bidirectional,
            has_skip_term, scale_x, None, mask_pad, keep_c=False)
    return h, last_hidden
