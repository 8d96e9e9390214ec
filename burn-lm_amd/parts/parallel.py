"""A layer whose mixer and feed-forward run side by side on the same normalised rows, and what surrounds them.

``n = norm(x)``; the mixer reads ``n + conv_1(n)`` and the feed-forward ``n + conv_2(n)`` (short causal
convolutions over time, one set of taps per channel and reader; the last taps - 1 rows ``n`` of a sequence are
its state); ``x <- x + mixer + feed_forward`` in float32; then a side input per token: a row ``e`` of a second
embedding table (this layer's columns of it), ``g = gelu_tanh(W_gate x) * e``, ``y = W_proj g``,
``x <- x + y / rms(y) * w``.  The last add is handed to the next norm as a float32 delta."""
from __future__ import annotations

import torch

from .base import Block, Part, StateNeed, TensorSpec


class CausalConvInput(Part):
    """The convolution in front of the sublayers.  params: width, taps, readers (how many sublayers read: 1 or 2).
    names: w0, w1 (each [width, taps])."""
    graph_safe = True

    def tensor_specs(self):
        p = self.params
        return {self.names[f"w{r}"]: TensorSpec((p["width"], p["taps"])) for r in range(p["readers"])}

    def bind(self, tensors, rt):
        self.rt = rt
        self.taps = int(self.params["taps"])
        self.weights = [tensors[self.names[f"w{r}"]].float().contiguous() for r in range(self.params["readers"])]

    def step_bytes(self, rows):
        return sum(w.numel() * 4 for w in self.weights)

    def cache_need(self):
        return StateNeed((self.params["taps"] - 1, self.params["width"]), torch.float32) if self.params["taps"] > 1 else None

    def read(self, n, step, view):
        """n: float32 normalised rows -> one tensor per reader in the activation dtype; moves the history on."""
        outs = [torch.empty(n.shape, dtype=self.rt.dtype, device=n.device) for _ in self.weights]
        self.rt.ops.input_conv(n, view.tensor if view is not None else None, self.weights, outs, step)
        return outs


class TokenSide(Part):
    """The side input per token.  params: width, dim, vocab, columns (width of the side table), column (this layer's
    first column in it), eps.  names: table, gate, proj, norm."""
    graph_safe = True

    def tensor_specs(self):
        p, n = self.params, self.names
        return {n["table"]: TensorSpec((p["vocab"], p["columns"])), n["gate"]: TensorSpec((p["dim"], p["width"])),
                n["proj"]: TensorSpec((p["width"], p["dim"])), n["norm"]: TensorSpec((p["width"],))}

    def bind(self, tensors, rt):
        self.rt = rt
        n = self.names
        self.table = tensors[n["table"]].contiguous()
        self.w_gate, self.w_proj = rt.weight(tensors[n["gate"]]), rt.weight(tensors[n["proj"]])
        self.norm_w = tensors[n["norm"]].float().contiguous()
        self.column, self.eps = int(self.params["column"]), float(self.params["eps"])

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_gate, self.w_proj)) \
            + rows * self.params["dim"] * self.table.element_size()

    def step_flops(self, rows):
        return 2 * rows * (self.w_gate.w.numel() + self.w_proj.w.numel())

    def forward(self, x, step):
        """x: the residual rows in the activation dtype -> the float32 delta [1, tokens, width]."""
        rt = self.rt
        z = rt.linear(x, self.w_gate)
        g = rt.ops.side_gate(z, self.table, self.column, step.token_ids, torch.empty_like(z), step.token_source)
        y = rt.linear(g, self.w_proj, partials=True)
        out = torch.empty(1, x.shape[0], x.shape[1], dtype=torch.float32, device=x.device)
        rt.ops.rms_scale(y, self.norm_w, self.eps, out[0])
        return out


class ParallelBlock(Block):
    roles = {"norm": "norm", "input": "connection", "mixer": "mixer", "feed_forward": "feed_forward",
             "side": "connection"}

    def cache_need(self):
        need = self.mixer.cache_need()
        mine = [self.input.cache_need()]
        return tuple(mine + (list(need) if isinstance(need, (tuple, list)) else [need]))

    def _mixer_view(self, view):
        rest = view[1:]
        return tuple(rest) if isinstance(self.mixer.cache_need(), (tuple, list)) else rest[0]

    def _feed_forward(self, xs, step):
        return self.feed_forward.forward(xs[1], step)

    def forward(self, h, delta, step, view):
        rt = self.norm.rt
        n = self.norm.add_norm(h, delta, out_dtype=torch.float32)
        xs = self.input.read(n, step, view[0])
        if hasattr(self.mixer, "forward_unbiased"):
            a, bias = self.mixer.forward_unbiased(xs[0], step, self._mixer_view(view))
        else:
            a, bias = self.mixer.forward(xs[0], step, self._mixer_view(view)), None
        f = self._feed_forward(xs, step)
        rows = h.view(h.shape[0], h.shape[-1])
        copy = torch.empty(rows.shape, dtype=rt.dtype, device=h.device)
        rt.ops.residual_add(rows, a, f, bias, copy)
        return self.side.forward(copy, step)


class ParallelMixerBlock(ParallelBlock):
    """The same without a feed-forward."""
    roles = {"norm": "norm", "input": "connection", "mixer": "mixer", "side": "connection"}

    def _feed_forward(self, xs, step):
        return None


class LayerScale(Part):
    """What a layer with layer scale multiplies its sublayers' results by before they join the residual: a stored
    vector per sublayer, element by element, and one number for the whole layer (a residual multiplier).
    params: width, mult (default 1), roles (which sublayers have a vector; default mixer and feed_forward).
    names: one tensor [width] per role."""
    graph_safe = True

    def _roles(self):
        return tuple(self.params.get("roles", ("mixer", "feed_forward")))

    def tensor_specs(self):
        return {self.names[r]: TensorSpec((self.params["width"],)) for r in self._roles()}

    def bind(self, tensors, rt):
        self.rt = rt
        self.mult = float(self.params.get("mult", 1.0))
        self.vectors = {r: tensors[self.names[r]].float().contiguous() for r in self._roles()}
        self._scaled = {}

    def step_bytes(self, rows):
        return sum(4 * v.numel() for v in self.vectors.values())

    def coefficient(self, role, factor):
        """float32 [width]: the role's vector times the layer's multiplier times a summand's own factor."""
        key = (role, float(factor))
        if key not in self._scaled:
            self._scaled[key] = (self.vectors[role].double() * (self.mult * float(factor))).float().contiguous()
        return self._scaled[key]

    def add(self, h, by_role):
        """h += sum over roles and their terms of coefficient(role, term.scale) * term.row * term.y, in float32."""
        terms = [(t.y, self.coefficient(role, t.scale), t.row) for role, ts in by_role for t in ts]
        limit = self.rt.ops.MAX_ADD_TERMS
        for at in range(0, len(terms), limit):
            self.rt.ops.scaled_add(h, terms[at:at + limit])
        return h


class ScaledParallelBlock(Block):
    """``n = norm(x)``; ``x <- x + mult * (scale_1 * mixer(n) + scale_2 * feed_forward(n))``: one norm, both sublayers
    read its output, and each result is multiplied element by element by a stored vector before the sum.  The add is
    one float32 kernel over the sublayers' summands, which arrive apart with their own factors."""
    roles = {"norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward", "scale": "connection"}

    def _feed_forward(self, x, step):
        return [("feed_forward", self.feed_forward.forward_terms(x, step))]

    def forward(self, h, delta, step, view):
        x = self.norm.add_norm(h, delta)
        terms = [("mixer", self.mixer.forward_terms(x, step, view))] + self._feed_forward(x, step)
        self.scale.add(h.view(h.shape[0], h.shape[-1]), terms)
        return None


class ScaledParallelMixerBlock(ScaledParallelBlock):
    """The same without a feed-forward."""
    roles = {"norm": "norm", "mixer": "mixer", "scale": "connection"}

    def _feed_forward(self, x, step):
        return []
