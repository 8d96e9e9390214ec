"""Token embedding and output head.

``h = table[ids]`` with no scaling (crates/burn-lm-llama/src/nn/transformer.rs:95) into the
float32 residual stream; ``logits = x W_out^T`` without bias in float32 (transformer.rs:102).
A tied head uses the embedding table itself: the ``[vocab, width]`` table is the head's
``[d_out, d_in]`` matrix (the reference leaves tying as a TODO, transformer.rs:82-84)."""
from __future__ import annotations

import torch

from .base import Part, TensorSpec


class Embedding(Part):
    """params: vocab, width, copies (default 1; more: the residual starts as that many equal streams,
    [tokens, copies, width]), scale (default 1: every row is multiplied by it).  names: weight."""
    graph_safe = True

    def tensor_specs(self):
        return {self.names["weight"]: TensorSpec((self.params["vocab"], self.params["width"]))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.table = tensors[self.names["weight"]].contiguous()
        self.scale = float(self.params.get("scale", 1.0))

    def step_bytes(self, rows):
        return rows * self.params["width"] * self.table.element_size()      # the rows that are looked up

    def _rows(self, ids):
        copies = int(self.params.get("copies", 1))
        shape = (ids.shape[0], self.params["width"]) if copies == 1 else (ids.shape[0], copies, self.params["width"])
        return torch.empty(shape, dtype=torch.float32, device=ids.device)

    def forward(self, ids):
        h = self._rows(ids)
        return self.rt.ops.embed_gather(self.table, ids, h, self.scale)

    def forward_from(self, ids, source_rows, source_cell):
        """The same where some tokens are still on the device: row t is element source_rows[t] of the
        array whose address is in source_cell, where source_rows[t] >= 0.  An embedding without this
        method gets its tokens gathered by a separate launch before the step."""
        h = self._rows(ids)
        return self.rt.ops.embed_gather_from(self.table, ids, source_rows, source_cell, h, self.scale)


class LMHead(Part):
    """params: vocab, width, softcap (optional; a positive number c: logits <- c * tanh(logits / c)).
    names: weight (the embedding's name when tied)."""
    graph_safe = True

    def tensor_specs(self):
        return {self.names["weight"]: TensorSpec((self.params["vocab"], self.params["width"]))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.weight = rt.weight(tensors[self.names["weight"]])
        self.softcap = float(self.params.get("softcap") or 0.0)

    def step_bytes(self, rows):
        return self.weight.w.numel() * self.weight.w.element_size() if rows else 0

    def step_flops(self, rows):
        return 2 * rows * self.weight.w.numel()

    def forward(self, x):
        logits = self.rt.linear(x, self.weight, out_dtype=torch.float32)
        return self.rt.ops.softcap(logits, self.softcap) if self.softcap > 0 else logits
