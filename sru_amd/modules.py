"""Layer wrapper around the recurrence: minimal counterparts of the reference's
`SRUCell` (sru/modules.py:16-419) and `SRU` (sru/modules.py:422-689).

Constructor arguments, parameter / buffer names (`weight`, `weight_proj`, `weight_c`,
`bias`, `scale_x`, `layer_norm.*`, `rnn_lst.{i}.*`, `input_to_hidden.weight`), the
initialisation recipe and the forward semantics follow the reference, so a state_dict
saved by it loads here and the same inputs give the same outputs. What differs is
below the layer: the projection stays `torch.mm` (hipBLASLt) and the recurrence always
runs the HIP kernels of this package; there is no CPU path (CPU tensors are refused).
"""
import copy
import math
import warnings
from typing import List, Optional, Tuple, Union

import torch
import torch.nn as nn
from torch import Tensor
from torch.nn.utils.rnn import PackedSequence, pad_packed_sequence, pack_padded_sequence

from .norm import layer_norm as fused_layer_norm, supported as fused_layer_norm_supported
from .ops import elementwise_recurrence_gpu


class SRUCell(nn.Module):
    """One SRU layer: [layer norm] -> U = x @ W -> elementwise recurrence -> [layer norm]."""

    def __init__(self, input_size: int, hidden_size: int, dropout: float = 0.0,
                 rnn_dropout: float = 0.0, bidirectional: bool = False, n_proj: int = 0,
                 use_tanh: bool = False, highway_bias: float = 0.0, has_skip_term: bool = True,
                 layer_norm: bool = False, rescale: bool = True, v1: bool = False,
                 custom_m: Optional[nn.Module] = None, amp_recurrence_fp16: bool = False,
                 normalize_after: bool = False, weight_c_init: Optional[float] = None,
                 native_16bit: bool = True):
        """Arguments as sru/modules.py:32-50. `native_16bit` (no counterpart there): under
        autocast, or with 16-bit inputs, the kernels read a float16 / bfloat16 U as it is and
        return h in that dtype (state and arithmetic stay float32); False restores the
        reference's policy of casting U and x to float32 first and returning a float32 h
        (sru/ops.py:116-127)."""
        super().__init__()
        self.native_16bit = native_16bit
        self.input_size = input_size
        self.hidden_size = hidden_size                       # per direction
        self.bidirectional = bidirectional
        self.output_size = hidden_size * (2 if bidirectional else 1)
        self.dropout = float(dropout)
        self.rnn_dropout = float(rnn_dropout)
        self.has_skip_term = has_skip_term
        self.highway_bias = highway_bias
        self.rescale = rescale
        self.v1 = v1
        self.activation_type = 1 if use_tanh else 0          # sru/modules.py:115-120
        self.activation = "tanh" if use_tanh else "none"
        self.custom_m = custom_m
        self.amp_recurrence_fp16 = amp_recurrence_fp16
        self.normalize_after = normalize_after
        self.weight_c_init = weight_c_init

        # a projection is only used when it is a real bottleneck (sru/modules.py:126-128)
        self.projection_size = n_proj if 0 < n_proj < min(input_size, self.output_size) else 0
        # the skip term needs a fourth stream when it cannot be the input itself (:131-133)
        self.num_matrices = 4 if (has_skip_term and input_size != self.output_size) else 3

        if custom_m is None:
            inner = self.projection_size or input_size
            self.weight_proj = (nn.Parameter(torch.empty(input_size, self.projection_size))
                                if self.projection_size else None)
            self.weight = nn.Parameter(torch.empty(inner, self.output_size * self.num_matrices))
        self.weight_c = nn.Parameter(torch.empty(2 * self.output_size))
        self.bias = nn.Parameter(torch.empty(2 * self.output_size))
        self.register_buffer("scale_x", torch.zeros(1))
        self.layer_norm = None
        if layer_norm:
            self.layer_norm = nn.LayerNorm(self.output_size if normalize_after else input_size)
        self.reset_parameters()

    # ------------------------------------------------------------------ initialisation
    def reset_parameters(self):
        """The reference's recipe (sru/modules.py:164-233): unit-variance uniform weights,
        gate columns and weight_c scaled by sqrt(0.5), the dropout / layer-norm / rescale
        corrections, highway bias on the output gate, scale_x = sqrt(1 + 2 exp(bias))."""
        out = self.output_size
        with torch.no_grad():
            self.bias.zero_()
            self.bias[out:] += self.highway_bias
            scale = math.sqrt(1.0 + 2.0 * math.exp(self.highway_bias))
            self.scale_x[0] = scale if (self.rescale and self.has_skip_term) else 1.0

            if self.custom_m is None:
                bound = math.sqrt(3.0 / self.weight.size(0))
                self.weight.uniform_(-bound, bound)
                if self.weight_proj is not None:
                    bound = math.sqrt(3.0 / self.weight_proj.size(0))
                    self.weight_proj.uniform_(-bound, bound)
                # (in, direction, hidden, stream) view of the projection
                w = self.weight.view(self.weight.size(0), -1, self.hidden_size, self.num_matrices)
                if self.dropout > 0:
                    w[..., 0] *= math.sqrt(1.0 - self.dropout)
                if self.rnn_dropout > 0:
                    w *= math.sqrt(1.0 - self.rnn_dropout)
                if self.layer_norm is not None:
                    w *= 0.1
                if self.rescale and self.has_skip_term and self.num_matrices == 4:
                    w[..., 3] *= scale
            elif hasattr(self.custom_m, "reset_parameters"):
                self.custom_m.reset_parameters()
            else:
                warnings.warn("Unable to reset parameters for custom module. reset_parameters() "
                              "method not found for custom module. " + type(self.custom_m).__name__)

            if self.v1:
                self.weight_c.zero_()
                self.weight_c.requires_grad = False
            else:
                if self.weight_c_init is None:
                    self.weight_c.uniform_(-math.sqrt(3.0), math.sqrt(3.0))
                    self.weight_c *= math.sqrt(0.5)
                else:
                    self.weight_c.uniform_(-self.weight_c_init, self.weight_c_init)
                if self.custom_m is None:
                    w[..., 1] *= math.sqrt(0.5)
                    w[..., 2] *= math.sqrt(0.5)

    # ------------------------------------------------------------------ forward
    def forward(self, input: Tensor, c0: Optional[Tensor] = None,
                mask_pad: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
        if input.dim() not in (2, 3):
            raise ValueError("Input must be 2 or 3 dimensional")
        batch = input.size(-2)
        # (c0 = None goes down to the kernels as it is: they start from zeros, and no zero tensor is
        # allocated and filled per layer as at sru/modules.py:241-243)

        residual = input                                   # the skip term is the un-normalised input
        if self.layer_norm is not None and not self.normalize_after:
            input = self._normalise(input, feeds_projection=True)
        if self.training and self.rnn_dropout > 0:
            input = input * self._dropout_mask((batch, input.size(-1)), self.rnn_dropout)
        mask_c = None
        if self.training and self.dropout > 0:
            mask_c = self._dropout_mask((batch, self.output_size), self.dropout)
        scale_val = self.scale_x if self.rescale else None

        U, V = self.compute_UV(input, c0, mask_pad)
        h, c = self.apply_recurrence(U, V, residual, c0, scale_val, mask_c, mask_pad)
        if self.layer_norm is not None and self.normalize_after:
            h = self._normalise(h, feeds_projection=False)
        return h, c

    def _normalise(self, x: Tensor, feeds_projection: bool) -> Tensor:
        """self.layer_norm(x) (sru/modules.py:250-253, :278-279) through the layer-norm kernels of
        this package where they apply. Before the projection under autocast the rows leave the
        kernel in the autocast dtype, i.e. as the operand the dense product would otherwise obtain
        by casting a float32 result; everywhere else the output keeps x's dtype."""
        ln = self.layer_norm
        if not fused_layer_norm_supported(x) or ln.weight is None or ln.bias is None:
            return ln(x)
        out_dtype = x.dtype
        # (only when the dense product is the direct consumer: a custom module or the rnn_dropout
        # multiply in between sees what nn.LayerNorm would have given them, rows in x's dtype)
        direct = self.custom_m is None and not (self.training and self.rnn_dropout > 0)
        if feeds_projection and direct and torch.is_autocast_enabled("cuda"):
            out_dtype = torch.get_autocast_dtype("cuda")
        return fused_layer_norm(x, ln.weight, ln.bias, ln.eps, out_dtype)

    def apply_recurrence(self, U: Tensor, V: Tensor, residual: Tensor, c0: Optional[Tensor],
                         scale_val: Optional[Tensor], mask_c: Optional[Tensor],
                         mask_pad: Optional[Tensor]) -> List[Tensor]:
        """The call of sru/modules.py:296-304: always the training entry, which itself skips the
        state store when nothing can be differentiated. There are no CPU branches."""
        return elementwise_recurrence_gpu(
            U, residual, V, self.bias, c0, self.activation_type, self.hidden_size,
            self.bidirectional, self.has_skip_term, scale_val, mask_c, mask_pad,
            self.amp_recurrence_fp16, getattr(self, "native_16bit", True))

    def compute_UV(self, input: Tensor, c0: Optional[Tensor],
                   mask_pad: Optional[Tensor]) -> Tuple[Tensor, Tensor]:
        if self.custom_m is None:
            return self.compute_U(input), self.weight_c
        ret = self.custom_m(input)
        if isinstance(ret, (tuple, list)):
            if len(ret) > 2:
                raise Exception("Custom module must return 1 or 2 tensors but got {}.".format(len(ret)))
            U, V = ret[0], ret[1] + self.weight_c          # per-step V added to the vector
        else:
            U, V = ret, self.weight_c
        if U.size(-1) != self.output_size * self.num_matrices:
            raise ValueError("U must have a last dimension of {} but got {}.".format(
                self.output_size * self.num_matrices, U.size(-1)))
        if V.size(-1) != self.output_size * 2:
            raise ValueError("V must have a last dimension of {} but got {}.".format(
                self.output_size * 2, V.size(-1)))
        return U, V

    def compute_U(self, input: Tensor) -> Tensor:
        """(length*batch, output_size*num_matrices): one dense GEMM (two with a projection)."""
        x = input if input.dim() == 2 else input.contiguous().view(-1, self.input_size)
        if self.weight_proj is not None:
            x = x.mm(self.weight_proj)
        return x.mm(self.weight)

    def _dropout_mask(self, size: Tuple[int, int], p: float) -> Tensor:
        return self.bias.new_empty(size).bernoulli_(1 - p).div_(1 - p)

    def extra_repr(self):
        # the fields and order of sru/modules.py:388-413
        parts = [f"{self.input_size}, {self.hidden_size}"]
        if self.projection_size > 0:
            parts.append(f"projection_size={self.projection_size}")
        if self.dropout > 0:
            parts.append(f"dropout={self.dropout}")
        if self.rnn_dropout > 0:
            parts.append(f"rnn_dropout={self.rnn_dropout}")
        if self.bidirectional:
            parts.append(f"bidirectional={self.bidirectional}")
        if self.highway_bias != 0:
            parts.append(f"highway_bias={self.highway_bias}")
        if self.activation_type != 0:
            parts.append(f"activation={self.activation}")
        if self.v1:
            parts.append(f"v1={self.v1}")
        parts.append(f"rescale={self.rescale}")
        if not self.has_skip_term:
            parts.append(f"has_skip_term={self.has_skip_term}")
        if self.layer_norm is not None:
            parts.append("layer_norm=True")
        s = ", ".join(parts)
        if self.custom_m is not None:
            s += ",\n  custom_m=" + str(self.custom_m)
        return s

    def __repr__(self):
        s = self.extra_repr()
        if len(s.split("\n")) == 1:
            return "{}({})".format(self.__class__.__name__, s)
        return "{}({}\n)".format(self.__class__.__name__, s)


class SRU(nn.Module):
    """Stack of SRUCell layers with the reference's interface (sru/modules.py:422-652)."""

    def __init__(self, input_size: int, hidden_size: int, num_layers: int = 2, dropout: float = 0.0,
                 rnn_dropout: float = 0.0, bidirectional: bool = False, projection_size: int = 0,
                 use_tanh: bool = False, layer_norm: bool = False, highway_bias: float = 0.0,
                 has_skip_term: bool = True, rescale: bool = False, v1: bool = False,
                 nn_rnn_compatible_return: bool = False,
                 custom_m: Optional[Union[nn.Module, List[nn.Module]]] = None,
                 proj_input_to_hidden_first: bool = False, amp_recurrence_fp16: bool = False,
                 normalize_after: bool = False, weight_c_init: Optional[float] = None,
                 native_16bit: bool = True):
        """Arguments as sru/modules.py:437-457; `native_16bit` as in SRUCell."""
        super().__init__()
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.num_directions = 2 if bidirectional else 1
        self.output_size = hidden_size * self.num_directions
        self.num_layers = num_layers
        self.dropout = dropout
        self.rnn_dropout = rnn_dropout
        self.projection_size = projection_size
        self.bidirectional = bidirectional
        self.use_layer_norm = layer_norm
        self.has_skip_term = has_skip_term
        self.nn_rnn_compatible_return = nn_rnn_compatible_return
        self.amp_recurrence_fp16 = amp_recurrence_fp16
        if rnn_dropout > 0:
            warnings.warn("rnn_dropout > 0 is deprecated and will be removed in "
                          "next major version of SRU. Please use dropout instead.")
        if use_tanh:
            warnings.warn("use_tanh = True is deprecated and will be removed in "
                          "next major version of SRU.")

        self.input_to_hidden = None
        first_in = input_size
        if proj_input_to_hidden_first and input_size != self.output_size:
            self.input_to_hidden = nn.Linear(input_size, self.output_size, bias=False)
            first_in = self.output_size

        self.rnn_lst = nn.ModuleList()
        for i in range(num_layers):
            m_i = None
            if custom_m is not None:
                m_i = custom_m[i] if isinstance(custom_m, list) else copy.deepcopy(custom_m)
            self.rnn_lst.append(SRUCell(
                first_in if i == 0 else self.output_size, hidden_size,
                dropout=dropout if i + 1 != num_layers else 0,     # no dropout after the last layer
                rnn_dropout=rnn_dropout, bidirectional=bidirectional, n_proj=projection_size,
                use_tanh=use_tanh, layer_norm=layer_norm, highway_bias=highway_bias,
                has_skip_term=has_skip_term, rescale=rescale, v1=v1, custom_m=m_i,
                amp_recurrence_fp16=amp_recurrence_fp16, normalize_after=normalize_after,
                weight_c_init=weight_c_init, native_16bit=native_16bit))

    def forward(self, input: Union[Tensor, PackedSequence], c0: Optional[Tensor] = None,
                mask_pad: Optional[Tensor] = None) -> Tuple[Union[Tensor, PackedSequence], Tensor]:
        packed = isinstance(input, PackedSequence)
        if packed:
            # lengths -> (length, batch) mask, 1 where padded (sru/modules.py:606-611)
            input, lengths = pad_packed_sequence(input)
            steps = torch.arange(input.size(0), device=lengths.device)
            mask_pad = (steps[:, None] >= lengths[None, :]).to(input.device)
        if input.dim() != 3:
            raise ValueError("There must be 3 dimensions for (length, batch_size, input_size)")
        if c0 is None:
            states = [None] * self.num_layers      # the kernels start from zeros (sru/modules.py:617-620)
        else:
            if c0.dim() != 3:
                raise ValueError("c0 must be 3 dim (num_layers, batch_size, output_size)")
            states = list(c0.unbind(0))

        x = input if self.input_to_hidden is None else self.input_to_hidden(input)
        finals = []
        for layer, state in zip(self.rnn_lst, states):
            x, c = layer(x, state, mask_pad=mask_pad)
            finals.append(c)
        c_stack = torch.stack(finals)
        if self.nn_rnn_compatible_return:
            # (layers, batch, dirs*hidden) -> (layers*dirs, batch, hidden), as nn.RNN returns it
            b = input.size(1)
            c_stack = c_stack.view(self.num_layers, b, self.num_directions, self.hidden_size)
            c_stack = c_stack.transpose(1, 2).reshape(self.num_layers * self.num_directions, b,
                                                      self.hidden_size)
        if packed:
            x = pack_padded_sequence(x, lengths, enforce_sorted=False)
        return x, c_stack

    def reset_parameters(self):
        for layer in self.rnn_lst:
            layer.reset_parameters()
        if self.input_to_hidden is not None:
            self.input_to_hidden.reset_parameters()

    def make_backward_compatible(self):
        """Brings a module object unpickled from an older release up to the current attribute
        names (sru/modules.py:660-689): releases up to 2.1.7 called the sizes n_in / n_out /
        out_size / depth / n_proj and the stream count k, had no layer norm that can be carried
        over, and knew weight norm and relu / selu, which no longer exist; releases up to 2.1.9
        had neither `input_to_hidden` nor `custom_m`."""
        self.nn_rnn_compatible_return = getattr(self, "nn_rnn_compatible_return", False)
        if hasattr(self, "n_in"):
            if len(self.ln_lst):
                raise Exception("Layer norm is not backward compatible for sru<=2.1.7")
            if self.use_weight_norm:
                raise Exception("Weight norm removed in sru>=2.1.9")
            self.input_size, self.hidden_size = self.n_in, self.n_out
            self.output_size, self.num_layers = self.out_size, self.depth
            self.projection_size = self.n_proj
            self.use_layer_norm = False
            for cell in self.rnn_lst:
                cell.input_size, cell.hidden_size = cell.n_in, cell.n_out
                cell.output_size = cell.n_out * (2 if cell.bidirectional else 1)
                cell.num_matrices = cell.k
                cell.projection_size = cell.n_proj
                cell.layer_norm = None
                if cell.activation_type > 1:
                    raise Exception("ReLU or SeLU activation removed in sru>=2.1.9")
        if not hasattr(self, "input_to_hidden"):
            self.input_to_hidden = None
            for cell in self.rnn_lst:
                cell.custom_m = None
