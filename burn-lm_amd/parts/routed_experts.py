"""Mixture of experts: ``experts`` small SwiGLU feed-forwards without biases, of which every token uses the ``top``
with the largest router logits ``W_router x + b``, weighted by the softmax over the chosen logits only; a shared
expert of the same form may run for every token, times ``sigmoid(W_sg x)`` (one number per token).

The router's logits, the choice and the weights are float32.  All experts run as ONE stacked product: their gate
and up projections are the rows of one matrix, their down projections the columns of another, and every expert's
gated activations are multiplied by the token's weight for that expert (zero for experts it did not choose)
before the one down projection, which so adds the chosen experts' outputs up.  That computes every expert for
every token: the same weights are read as in a batch that uses every expert, nothing depends on which tokens
share a step, and no step shape depends on the routing, so steps replay from recorded graphs."""
from __future__ import annotations

import torch

from .base import FeedForward, TensorSpec, Term


class RoutedExperts(FeedForward):
    """params: width, experts, top, expert_inner, shared_inner (0: no shared expert).
    names: router, router_bias, e<i>.gate / e<i>.up / e<i>.down for every expert, and with a shared expert
    shared.gate, shared.up, shared.down, shared.sg."""
    graph_safe = True

    def tensor_specs(self):
        p, n = self.params, self.names
        d, E, f, s = p["width"], p["experts"], p["expert_inner"], int(p.get("shared_inner", 0))
        specs = {n["router"]: TensorSpec((E, d)), n["router_bias"]: TensorSpec((E,))}
        for e in range(E):
            specs[n[f"e{e}.gate"]] = TensorSpec((f, d))
            specs[n[f"e{e}.up"]] = TensorSpec((f, d))
            specs[n[f"e{e}.down"]] = TensorSpec((d, f))
        if s:
            specs.update({n["shared.gate"]: TensorSpec((s, d)), n["shared.up"]: TensorSpec((s, d)),
                          n["shared.down"]: TensorSpec((d, s)), n["shared.sg"]: TensorSpec((1, d))})
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.E, self.top, self.f, self.s = p["experts"], p["top"], p["expert_inner"], int(p.get("shared_inner", 0))
        if not 1 <= self.top <= self.E:
            raise ValueError(f"top = {self.top} of {self.E} experts")
        t = lambda name: tensors[n[name]]
        gates = [t(f"e{e}.gate") for e in range(self.E)] + ([t("shared.gate")] if self.s else [])
        ups = [t(f"e{e}.up") for e in range(self.E)] + ([t("shared.up")] if self.s else [])
        downs = [t(f"e{e}.down") for e in range(self.E)] + ([t("shared.down")] if self.s else [])
        ws = gates + ups + downs
        if len({w.dtype for w in ws}) != 1:
            gates, ups, downs = ([w.float() for w in group] for group in (gates, ups, downs))
        self.inner = self.E * self.f + self.s
        self.w_gate_up = rt.weight(torch.cat(gates + ups, dim=0))
        self.w_down = rt.weight(torch.cat(downs, dim=1).contiguous())
        router = [t("router")] + ([t("shared.sg")] if self.s else [])
        if len({w.dtype for w in router}) != 1:
            router = [w.float() for w in router]
        rows = sum(w.shape[0] for w in router)
        pad = (-rows) % 16
        if pad:
            router.append(torch.zeros(pad, router[0].shape[1], dtype=router[0].dtype, device=router[0].device))
        self.w_router = rt.weight(torch.cat(router, dim=0))
        self.router_bias = t("router_bias").float().contiguous()

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_gate_up, self.w_down, self.w_router))

    def step_flops(self, rows):
        return 2 * rows * sum(w.w.numel() for w in (self.w_gate_up, self.w_down, self.w_router))

    def route(self, x):
        """float32 [tokens, experts + 1]: every expert's weight for every token (zero if not chosen), and the shared
        expert's gate."""
        rt = self.rt
        logits = rt.linear(x, self.w_router, out_dtype=torch.float32)
        weights = torch.empty(x.shape[0], self.E + 1, dtype=torch.float32, device=x.device)
        return rt.ops.moe_route(logits, self.router_bias, self.E, self.top, self.E if self.s else -1, weights)

    def forward(self, x, step):
        rt = self.rt
        weights = self.route(x)
        gu = rt.linear(x, self.w_gate_up)
        act = torch.empty(x.shape[0], self.inner, dtype=gu.dtype, device=x.device)
        return rt.linear(rt.ops.moe_gate(gu, weights, act, self.E, self.f), self.w_down, partials=True)


class GroupedRoutedExperts(RoutedExperts):
    """The same stacked experts behind another router: the scores are the softmax of ``W_router x`` over all experts;
    the choice goes by ``score + correction`` (a stored vector), only among the experts of the ``keep`` best of
    ``groups`` equal groups of neighbouring experts (a group ranks by its largest corrected score); the ``top`` chosen
    experts' weights are their scores (without the correction) over the sum of the chosen scores.  The last
    ``identity`` of the router's outputs belong to experts without tensors that hand their input on unchanged; they
    count like the others in softmax, groups and choice, and their share of the result is ``weight * x``.

    params: width, experts (those with tensors), identity (default 0), top, groups (default 1), keep (default 1),
    expert_inner, correction (whether the checkpoint has one; default True).
    names: router [experts + identity, width], correction [experts + identity], e<i>.gate / e<i>.up / e<i>.down."""

    def _counts(self):
        p = self.params
        E, I = int(p["experts"]), int(p.get("identity", 0))
        groups, keep = int(p.get("groups", 1)), int(p.get("keep", 1))
        if E < 1 or I < 0 or groups < 1 or (E + I) % groups or not 1 <= keep <= groups:
            raise ValueError(f"grouped experts: {E} + {I} experts do not form {groups} equal groups of which {keep} stay")
        if not 1 <= p["top"] <= keep * ((E + I) // groups):
            raise ValueError(f"grouped experts: top = {p['top']} is more than {keep} groups of {(E + I) // groups} hold")
        return E, I, groups, keep

    def tensor_specs(self):
        p, n = self.params, self.names
        d, f = p["width"], p["expert_inner"]
        E, I, _, _ = self._counts()
        specs = {n["router"]: TensorSpec((E + I, d))}
        if p.get("correction", True):
            specs[n["correction"]] = TensorSpec((E + I,))
        for e in range(E):
            specs[n[f"e{e}.gate"]] = TensorSpec((f, d))
            specs[n[f"e{e}.up"]] = TensorSpec((f, d))
            specs[n[f"e{e}.down"]] = TensorSpec((d, f))
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.E, self.I, self.groups, self.keep = self._counts()
        self.top, self.f, self.s = int(p["top"]), p["expert_inner"], 0
        t = lambda name: tensors[n[name]]
        gates, ups = [t(f"e{e}.gate") for e in range(self.E)], [t(f"e{e}.up") for e in range(self.E)]
        downs = [t(f"e{e}.down") for e in range(self.E)]
        if len({w.dtype for w in gates + ups + downs}) != 1:
            gates, ups, downs = ([w.float() for w in group] for group in (gates, ups, downs))
        self.inner = self.E * self.f
        self.w_gate_up = rt.weight(torch.cat(gates + ups, dim=0))
        self.w_down = rt.weight(torch.cat(downs, dim=1).contiguous())
        router = t("router")
        pad = (-router.shape[0]) % 16
        if pad:
            router = torch.cat([router, torch.zeros(pad, router.shape[1], dtype=router.dtype, device=router.device)], dim=0)
        self.w_router = rt.weight(router.contiguous())
        self.correction = t("correction").float().contiguous() if p.get("correction", True) else None

    def route(self, x):
        """float32 [tokens, experts + 1]: every expert's weight for every token (zero if not chosen), and behind them
        the weight of the token's pass-through experts together."""
        rt = self.rt
        logits = rt.linear(x, self.w_router, out_dtype=torch.float32)
        weights = torch.empty(x.shape[0], self.E + 1, dtype=torch.float32, device=x.device)
        return rt.ops.moe_route_grouped(logits, self.correction, self.E, self.I, self.groups, self.keep, self.top, weights)

    def forward_terms(self, x, step):
        rt = self.rt
        weights = self.route(x)
        gu = rt.linear(x, self.w_gate_up)
        act = torch.empty(x.shape[0], self.inner, dtype=gu.dtype, device=x.device)
        terms = [Term(rt.linear(rt.ops.moe_gate(gu, weights, act, self.E, self.f), self.w_down, partials=True))]
        if self.I:
            terms.append(Term(x, 1.0, weights[:, self.E]))
        return terms

    def forward(self, x, step):
        terms = self.forward_terms(x, step)
        if len(terms) == 1:
            return terms[0].y
        out = torch.zeros(1, x.shape[0], x.shape[1], dtype=torch.float32, device=x.device)
        self.rt.ops.scaled_add(out[0], [(t.y, None, t.row) for t in terms])
        return out
