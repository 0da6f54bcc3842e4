"""SRU elementwise recurrence for MI355X (gfx950): hand-written HIP kernels behind a C ABI,
with the host-side interface of the reference's sru/cuda_functional.py and sru/ops.py."""
from .functional import ElementwiseRecurrence, elementwise_recurrence_forward
from .ops import elementwise_recurrence_gpu, elementwise_recurrence_inference
from .modules import SRU, SRUCell
from .graphs import graphed

__all__ = ["ElementwiseRecurrence", "elementwise_recurrence_forward",
           "elementwise_recurrence_gpu", "elementwise_recurrence_inference", "SRU", "SRUCell", "graphed"]
