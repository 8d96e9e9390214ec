"""Lightning attention: linear attention whose matrix state per head fades by a constant of the model.

``q = silu(W_q x)``, ``k = silu(W_k x)`` (heads x dim), ``v = silu(W_v x)`` (heads x vdim); per head
``S_t = decay_h S_{t-1} + k_t v_t^T`` and ``o_t = S_t^T q_t`` with one fixed ``decay_h`` per head and no other scale.
The heads' ``o`` are concatenated and RMS-normed together (one weight per lane of the concatenation), multiplied by
``sigmoid(W_g x)`` and projected.  ``S`` starts at zero, is float32 and is carried per sequence as fixed-size state;
the recurrence, the decays and the norm are float32 in every mode.  Steps of few tokens per sequence (decoding) run on
the scan of the gated linear attention, whose per-channel decays are here a constant vector; prompts run chunk by
chunk as float32 matrix products, which a constant decay allows (heads of up to 128 x 128 channels; larger ones take
the scan there too)."""
from __future__ import annotations

import torch

from .base import Mixer, StateNeed, TensorSpec


class LightningAttention(Mixer):
    """params: width, heads, dim, vdim, decay (one number in (0, 1] per head), eps.  names: q, k, v, g, norm, o."""
    graph_safe = True
    CHUNKS_FROM = 8      # a step whose longest sequence brings at least this many tokens runs in chunks

    def tensor_specs(self):
        p, n = self.params, self.names
        d, H, dk, dv = p["width"], p["heads"], p["dim"], p["vdim"]
        return {n["q"]: TensorSpec((H * dk, d)), n["k"]: TensorSpec((H * dk, d)), n["v"]: TensorSpec((H * dv, d)),
                n["g"]: TensorSpec((H * dv, d)), n["norm"]: TensorSpec((H * dv,)), n["o"]: TensorSpec((d, H * dv))}

    def cache_need(self):
        p = self.params
        return StateNeed((p["heads"], p["dim"], p["vdim"]), torch.float32)

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.H, self.dk, self.dv, self.eps = p["heads"], p["dim"], p["vdim"], float(p["eps"])
        decay = [float(a) for a in p["decay"]]
        if len(decay) != self.H or not all(0.0 < a <= 1.0 for a in decay):
            raise ValueError(f"lightning attention: {self.H} heads need as many decays in (0, 1], got {decay}")
        # the scan takes a decay per key channel: each head's constant, once for every channel of the head
        self.decay = torch.tensor(decay, dtype=torch.float64).to(torch.float32).repeat_interleave(self.dk).to(rt.device)
        ws = [tensors[n[r]] for r in ("q", "k", "v", "g")]
        if len({w.dtype for w in ws}) != 1:
            ws = [w.float() for w in ws]
        rows = sum(w.shape[0] for w in ws)
        if rows % 8:
            ws.append(torch.zeros(8 - rows % 8, ws[0].shape[1], dtype=ws[0].dtype, device=ws[0].device))
        self.w_in = rt.weight(torch.cat(ws, dim=0))
        self.w_o = rt.weight(tensors[n["o"]])
        self.norm_w = tensors[n["norm"]].float().contiguous()
        self.in_chunks = rt.ops.lightning_chunks_supported(self.dk, self.dv)
        if self.in_chunks:
            rt.ops.lightning_chunks_init(rt.device)      # the kernels' shared memory, before any step is recorded
            self.powers = rt.ops.decay_powers(decay, rt.device)

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_in, self.w_o))

    def step_flops(self, rows):
        return 2 * rows * (self.w_in.w.numel() + self.w_o.w.numel())

    def mixing_flops(self, past, new):
        return 5 * self.H * self.dk * self.dv * new

    def forward(self, x, step, view):
        return self.output(self.scan(self.project(x), step, view))

    def project(self, x):
        """The stacked projection [q | k | v | g]."""
        return self.rt.linear(x, self.w_in)

    def scan(self, proj, step, view):
        """The recurrence over the step's tokens, each sequence from its own state -> [tokens, heads * vdim]."""
        rt = self.rt
        T = proj.shape[0]
        o_raw = torch.zeros(T, self.H * self.dv, dtype=torch.float32, device=proj.device)
        out = torch.empty(T, self.H * self.dv, dtype=rt.dtype, device=proj.device)
        if self.in_chunks and step.max_new >= self.CHUNKS_FROM and T > 4 * step.n_seqs:
            return rt.ops.lightning_chunks(proj, self.powers, self.norm_w, self.eps, view.tensor, o_raw, out, step, self.H,
                                           self.dk, self.dv, activation="silu", norm_all=True, gate="sigmoid")
        return rt.ops.gla_scan(proj, None, None, None, self.norm_w, self.eps, view.tensor, o_raw, out, step, self.H, self.dk,
                               self.dv, fixed_decay=self.decay, activation="silu", q_scale=1.0, norm_all=True, gate="sigmoid")

    def output(self, mixed):
        return self.rt.linear(mixed, self.w_o, partials=True)
