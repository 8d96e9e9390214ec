"""RMS norm with the residual add fused in front of it.

``y = x / sqrt(mean(x^2) + eps) * gamma`` (crates/burn-lm-llama/src/nn/transformer.rs:60-62,
vector at :278-297).  The sum of squares, the root and the scaling are float32; the add that
precedes the norm in a block (transformer.rs:248-255) is done here, on the float32 residual.
"""
from __future__ import annotations

import torch

from .base import Gated, Norm, TensorSpec


class RMSNorm(Norm):
    """params: width, eps, single (default False; True: the stored weight is one number for all lanes, a tensor without
    dimensions).  names: weight."""
    graph_safe = True


    def tensor_specs(self):
        return {self.names["weight"]: TensorSpec(() if self.params.get("single") else (self.params["width"],))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.gamma = tensors[self.names["weight"]]
        if self.params.get("single"):      # the kernels read a weight per lane: the one number, once for each
            self.gamma = self.gamma.reshape(1).expand(self.params["width"])
        self.gamma = self.gamma.contiguous()
        self.eps = float(self.params["eps"])

    def step_bytes(self, rows):
        return self.gamma.numel() * self.gamma.element_size()

    def rms_constants(self):
        return self.gamma, self.eps

    def add_norm(self, h, delta, rows=None, write_h=True):
        n = h.shape[0] if rows is None else rows.shape[0]
        out = torch.empty(n, h.shape[1], dtype=self.rt.dtype, device=h.device)
        if isinstance(delta, Gated):
            return self.rt.ops.add_rmsnorm(h, delta.y, self.gamma, self.eps, out, rows=rows, write_h=write_h,
                                           gate=delta.z, gate_bias=delta.bias, mult=delta.mult)
        return self.rt.ops.add_rmsnorm(h, delta, self.gamma, self.eps, out, rows=rows, write_h=write_h)
