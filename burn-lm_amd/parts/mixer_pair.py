"""Two mixers side by side on the same rows: ``left_scale * left(x) + right_scale * right(x)``.

Each of the two is a mixer of any registered kind with its own tensors and its own place in the cache (the pair asks
for both needs and gets both views).  A block that adds summands itself gets the two results apart, each with its
factor (`forward_terms`); for any other block the pair adds them up in float32."""
from __future__ import annotations

import torch

from .. import registry
from .base import Mixer, PartSpec, Term


def _flat(need):
    return [] if need is None else (list(need) if isinstance(need, (tuple, list)) else [need])


class MixerPair(Mixer):
    """params: left, right (each a PartSpec of a mixer), left_scale, right_scale, position (handed to both)."""

    def __init__(self, params, names):
        super().__init__(params, names)
        self.sides = []
        for side in ("left", "right"):
            spec = params[side]
            if not isinstance(spec, PartSpec):
                raise TypeError(f"mixer pair: '{side}' must be a PartSpec, got {type(spec).__name__}")
            inner = dict(spec.params)
            if params.get("position") is not None:
                inner["position"] = params["position"]
            self.sides.append(registry.part("mixer", spec.kind)(inner, spec.names))
        self.scales = (float(params["left_scale"]), float(params["right_scale"]))

    @property
    def graph_safe(self):
        return all(m.graph_safe for m in self.sides)

    def tensor_specs(self):
        specs = {}
        for m in self.sides:
            specs.update(m.tensor_specs())
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        for m in self.sides:
            m.bind(tensors, rt)

    def cache_need(self):
        needs = [n for m in self.sides for n in _flat(m.cache_need())]
        return tuple(needs) if needs else None

    def step_bytes(self, rows):
        return sum(m.step_bytes(rows) for m in self.sides)

    def step_flops(self, rows):
        return sum(m.step_flops(rows) for m in self.sides)

    def mixing_flops(self, past, new):
        return sum(m.mixing_flops(past, new) for m in self.sides)

    def _views(self, view):
        views = list(view) if isinstance(view, (tuple, list)) else [view]
        out, at = [], 0
        for m in self.sides:
            need = m.cache_need()
            n = len(_flat(need))
            part = views[at:at + n]
            at += n
            out.append(tuple(part) if isinstance(need, (tuple, list)) else (part[0] if part else None))
        return out

    def forward_terms(self, x, step, view):
        terms = []
        for m, scale, v in zip(self.sides, self.scales, self._views(view)):
            terms += [Term(t.y, t.scale * scale, t.row) for t in m.forward_terms(x, step, v)]
        return terms

    def forward(self, x, step, view):
        out = torch.zeros(1, x.shape[0], self.params["width"], dtype=torch.float32, device=x.device)
        terms = self.forward_terms(x, step, view)
        chans = [torch.full((out.shape[2],), t.scale, dtype=torch.float32, device=x.device) for t in terms]
        self.rt.ops.scaled_add(out[0], [(t.y, c, t.row) for t, c in zip(terms, chans)])
        return out
