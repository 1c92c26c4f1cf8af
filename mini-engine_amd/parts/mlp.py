"""Dense gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases
(reference: ``src/mini_engine/model.py:122-131``). Gate and up weights are stacked at load time so
that one product feeds the activation, which is the epilogue of that product where a kernel of this
package computes it (silu as in the reference, or the tanh form of gelu)."""

from __future__ import annotations

import torch

from ..ops import kernels as K
from ..weights.loader import TensorWant
from .base import FEED_FORWARDS, FeedForward


class GatedMlp(FeedForward):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation not in K.GATE_ACTIVATIONS:
            raise ValueError(f"gated_mlp knows the activations {sorted(K.GATE_ACTIVATIONS)}, got {spec.activation!r}")
        self.w_gate_up = self.w_down = None

    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s = self.spec
        return {
            f"{prefix}.gate_proj.weight": TensorWant((s.intermediate_size, s.hidden_size)),
            f"{prefix}.up_proj.weight": TensorWant((s.intermediate_size, s.hidden_size)),
            f"{prefix}.down_proj.weight": TensorWant((s.hidden_size, s.intermediate_size)),
        }

    def load(self, tensors, prefix: str) -> None:
        self.w_gate_up = torch.cat((tensors[f"{prefix}.gate_proj.weight"], tensors[f"{prefix}.up_proj.weight"]), dim=0)
        self.w_down = tensors[f"{prefix}.down_proj.weight"]

    takes_normed_input = True

    def forward(self, h, batch=None) -> torch.Tensor:
        act = K.linear(h, self.w_gate_up, gated=self.spec.activation)
        return K.linear(act, self.w_down, as_delta=True)

    def emit(self, program, h) -> None:
        act = program.linear(h, self.w_gate_up, gated=self.spec.activation)
        program.linear_delta(act, self.w_down)


FEED_FORWARDS.register("gated_mlp", GatedMlp)
