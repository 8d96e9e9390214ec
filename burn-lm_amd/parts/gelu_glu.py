"""Dense gated feed-forward with the tanh form of GELU: ``W_down (gelu_tanh(W_gate x) * (W_up x))`` without biases,
``gelu_tanh(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))``.  Gate and up run as one product on the stacked
weight; the activation and the product are float32, in the epilogue of the hand-written products (few rows, and
prompts of the sizes the runtime gives to its tiled kernel) and in a kernel of their own behind the library's product."""
from __future__ import annotations

import torch

from .base import FeedForward, TensorSpec


class GeluGLU(FeedForward):
    """params: width, inner.  names: gate, up, down."""
    graph_safe = True

    def tensor_specs(self):
        d, i = self.params["width"], self.params["inner"]
        return {self.names["gate"]: TensorSpec((i, d)), self.names["up"]: TensorSpec((i, d)),
                self.names["down"]: TensorSpec((d, i))}

    def bind(self, tensors, rt):
        self.rt = rt
        g, u = tensors[self.names["gate"]], tensors[self.names["up"]]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gate_up = rt.weight(torch.cat([g, u], dim=0), gated=True)
        self.w_down = rt.weight(tensors[self.names["down"]])
        self.inner = self.params["inner"]

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_gate_up, self.w_down))

    def step_flops(self, rows):
        return 2 * rows * (self.w_gate_up.w.numel() + self.w_down.w.numel())

    def forward(self, x, step):
        rt = self.rt
        return rt.linear(rt.gated_linear(x, self.w_gate_up, activation="gelu_tanh"), self.w_down, partials=True)
