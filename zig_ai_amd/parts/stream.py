"""Parts that add to the residual stream between two run-order entries (family
``stream``).  A run-order entry names one with ``LayerCall.before`` and the keywords its
``forward`` takes; the model hands it the stream, what is still pending for it, and the
embedding's output as it was before the first layer (``origin``).

``pass_offset``: for models that run a span of layers several times with the same weights.
Before pass ``row`` of the span the stream takes the row ``row`` of a table ``[passes,
width]`` and, with ``add_origin``, the embedding's output once more:

    x <- x (+ pending) (+ origin) + table[row]
"""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Part, Runtime, TensorRule, register_stream_step


class PassOffset(Part):
    kind = "pass_offset"
    graph_safe = True
    kernel_sources = ("norm",)

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        return {"table": TensorRule(((int(params["passes"]), int(params["width"])),), role="bias")}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.passes = int(params["passes"])
        self.table = tensors["table"]          # 32-bit [passes, width]

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor],
                origin: Optional[torch.Tensor], step, row: int = 0, add_origin: bool = False):
        if not 0 <= int(row) < self.passes:
            raise ValueError(f"pass {row} of {self.passes}")
        if add_origin and origin is None:
            raise ValueError("the embedding's output was not kept for this model")
        ops.stream_add_(residual, pending, origin if add_origin else None, self.table[int(row)])
        return residual, None


register_stream_step(PassOffset.kind, PassOffset)
