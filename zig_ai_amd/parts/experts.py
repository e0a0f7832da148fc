"""A feed-forward of many small experts of which every token uses a few.

``table_experts``: no router.  A table ``[vocab, top]`` of integers names, for each
token id, the ``top`` experts its tokens use (the entries of a row differ); each counts
``1 / top``:

    y[t] = (1 / top) * sum_j  down[e_j] act(up[e_j] x[t]),   e_j = table[token_id[t], j]

``act`` is ``relu2`` (the square of relu); experts have no gate and no biases.  Sizes and
the activation come from ``params``: ``hidden_size``, ``intermediate_size`` (of one expert),
``experts``, ``top``, ``vocab_size``, ``activation``.

The step's tokens are listed per expert on the device (``ops.expert_lists``), two grouped
products run every expert's rows against its own weights in one launch each, and the
second leaves a token's ``top`` results as a stack of 32-bit partial sums that the next
norm adds up: nothing is looked at on the host, so steps can be recorded.
"""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from ..kernels import ops
from .base import FeedForward, Runtime, TensorRule, register_feed_forward


class TableExperts(FeedForward):
    kind = "table_experts"
    graph_safe = True
    kernel_sources = ("experts",)

    @staticmethod
    def _sizes(params):
        return tuple(int(params[k]) for k in ("hidden_size", "intermediate_size", "experts", "top",
                                              "vocab_size"))

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, I, E, top, V = cls._sizes(params)
        rules = {"table": TensorRule(((V, top),), role="choice", bound=E)}
        for e in range(E):
            rules[f"experts.{e}.up.weight"] = TensorRule(((I, H),))
            rules[f"experts.{e}.down.weight"] = TensorRule(((H, I),))
        return rules

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        H, I, E, top, V = self._sizes(params)
        if not 0 < top <= E or E > ops.EXPERTS_MAX:
            raise ValueError(f"{top} of {E} experts: top must be within 1..experts, experts at "
                             f"most {ops.EXPERTS_MAX}")
        self.experts, self.top = E, top
        self.activation = str(params.get("activation", "relu2"))
        if self.activation not in ops.EXPERT_ACTIVATIONS:
            raise ValueError(f"expert activation must be relu2, got {self.activation!r}")
        self.table = tensors["table"]
        if self.table.dtype != torch.int32:
            raise ValueError(f"the experts' table must hold integers, got {self.table.dtype}")
        self.up = self._stack([tensors[f"experts.{e}.up.weight"] for e in range(E)])
        self.down = self._stack([tensors[f"experts.{e}.down.weight"] for e in range(E)])

    @staticmethod
    def _stack(mats) -> torch.Tensor:
        w = torch.stack(list(mats), dim=0)
        # (rows of a bfloat16 weight start on 16-byte boundaries, or it is kept in 32-bit)
        if w.dtype == torch.bfloat16 and w.shape[2] % 8:
            w = w.float()
        return w.contiguous()

    def forward(self, x, step):
        T = x.shape[0]
        lists, counts = ops.expert_lists(step.token_ids, self.table, T, self.experts)
        a = ops.grouped_linear(x, self.up, lists, counts, T, per_token=True,
                               activation=self.activation, out_dtype=x.dtype)
        # a stack [top, T, width] of 32-bit partial results, already times 1 / top
        return ops.grouped_linear(a, self.down, lists, counts, T, per_token=False, stacked=True,
                                  out_scale=1.0 / self.top)


register_feed_forward(TableExperts.kind, TableExperts)
