"""A pre-norm layer whose sublayers join the residual behind gates.

``n1 = norm1(x)``; ``x <- x + m * mixer(n1) * sigmoid(W_1 n1 + b_1)``; ``n2 = norm2(x)``;
``x <- x + m * feed_forward(n2) * sigmoid(W_2 n2 + b_2)``: each gate is projected from the very rows its sublayer
reads, and ``m`` is one residual multiplier for the model.  The gate's projection runs beside the sublayer; the
gating, the add into the float32 residual and the next norm are one kernel (the norm takes a ``Gated`` delta), so a
block takes the pending gated result of the block before it and hands on its own."""
from __future__ import annotations

from .base import Block, Gated, Part, TensorSpec


class ResidualGate(Part):
    """The gates of a layer.  params: width, mult (default 1), roles (the sublayers that have a gate; default mixer and
    feed_forward).  names: per role ``<role>`` ([width, width]) and ``<role>_bias`` ([width])."""
    graph_safe = True

    def _roles(self):
        return tuple(self.params.get("roles", ("mixer", "feed_forward")))

    def tensor_specs(self):
        d = self.params["width"]
        specs = {}
        for r in self._roles():
            specs[self.names[r]] = TensorSpec((d, d))
            specs[self.names[r + "_bias"]] = TensorSpec((d,))
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        self.mult = float(self.params.get("mult", 1.0))
        self.weights = {r: rt.weight(tensors[self.names[r]]) for r in self._roles()}
        self.biases = {r: tensors[self.names[r + "_bias"]].float().contiguous() for r in self._roles()}

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in self.weights.values()) + sum(4 * b.numel() for b in self.biases.values())

    def step_flops(self, rows):
        return 2 * rows * sum(w.w.numel() for w in self.weights.values())

    def gated(self, role, x, y):
        """The sublayer's result y (of the rows x it read) with its gate, for the next norm's add."""
        return Gated(y, self.rt.linear(x, self.weights[role]), self.biases[role], self.mult)


class GatedPreNormBlock(Block):
    roles = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "feed_forward": "feed_forward",
             "gate": "connection"}

    def forward(self, h, delta, step, view):
        x = self.mixer_norm.add_norm(h, delta)
        a = self.gate.gated("mixer", x, self.mixer.forward(x, step, view))
        x = self.ffn_norm.add_norm(h, a)
        return self.gate.gated("feed_forward", x, self.feed_forward.forward(x, step))


class GatedPreNormMixerBlock(Block):
    """The same without a feed-forward."""
    roles = {"mixer_norm": "norm", "mixer": "mixer", "gate": "connection"}

    def forward(self, h, delta, step, view):
        x = self.mixer_norm.add_norm(h, delta)
        return self.gate.gated("mixer", x, self.mixer.forward(x, step, view))
