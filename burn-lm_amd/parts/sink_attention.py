"""Grouped-query attention with projection biases, a sliding window, a softmax sink and head mixing.

``q, k, v = W x + b``; the first ``rot_dims`` lanes of every query and key head are turned by the token's position
(lane i with lane i + rot_dims/2, angle ``p * base^(-2i/rot_dims)``), the rest pass; rotated keys and the values
go into the paged cache.  ``score = q . k * scale``; query i sees key j while ``0 <= i - j < window`` (window 0:
every earlier key).  The softmax's denominator also holds ``exp(sink_h)``, a learned logit per head without key
or value.  The heads' weights are then mixed, ``w'_h = sum_g talk[h, g] w_g``, and head h applies its mixed
weights to the values of its own key-value head.  Keys and values may differ in head size.  A layer that
borrows (``borrows=True``) has no key and value projections and reads the keys (as cached, rotated) and values
that an earlier layer keeps, with queries, window, sink and mixing of its own.  Scores, softmax and the mixing
are float32 in every mode.

Variants by parameter: no biases at all (``bias=False``); turning pairs of adjacent lanes ``(2i, 2i + 1)``
(``pairing="adjacent"``); values that are the keys as projected, before the rotation, with no value projection
(``values="keys"``; then ``vdim = dim``); a stored temperature per head that multiplies the head's scores
(``temperature=True``; it rides on the queries, which the scores are linear in, applied in float32 behind their
rotation); an output gate (``gate=True``): the concatenated heads are multiplied element by element by
``sigmoid(W_g x)`` of the mixer's own input before the output projection (``W_g`` runs with the other projections)."""
from __future__ import annotations

import os

import torch

from .base import KVNeed, Mixer, TensorSpec, Term


class SinkAttention(Mixer):
    """params: width, heads, kv_heads, dim, vdim, scale, window (0: all keys), cache_window (what the cache keeps:
    the largest window of this layer and of the layers that borrow from it; default window), rot_dims, position
    (a rotary encoding whose table has rot_dims/2 pairs; given by the model builder), borrows, sink, talk (whether
    the layer has them; default True), bias (whether the projections have biases; default True), pairing ("half",
    the default: lane i turns with lane i + rot_dims/2; "adjacent": lane 2i with 2i + 1), values ("projected", the
    default, or "keys": the unrotated keys are the values and there is no value projection), temperature (whether a
    number per head multiplies its scores; default False), gate (whether the heads pass a sigmoid gate projected from
    the input; default False).
    names: q, q_bias, o, o_bias, sink, talk, temp, g and, unless the layer borrows, k, k_bias, v, v_bias (those the
    parameters leave)."""
    graph_safe = True

    def _flags(self):
        p = self.params
        return bool(p.get("borrows")), p.get("sink", True), p.get("talk", True)

    def _variant(self):
        """(projections have biases, values are the keys, pairs are adjacent lanes)"""
        p = self.params
        values, pairing = p.get("values", "projected"), p.get("pairing", "half")
        if values not in ("projected", "keys") or pairing not in ("half", "adjacent"):
            raise ValueError(f"sink attention: values={values!r} (projected, keys) or pairing={pairing!r} (half, adjacent) unknown")
        if values == "keys" and (p["vdim"] != p["dim"] or p.get("borrows")):
            raise ValueError("values that are the keys have the keys' head size, and their layer keeps its own")
        return bool(p.get("bias", True)), values == "keys", pairing == "adjacent"

    def tensor_specs(self):
        p, n = self.params, self.names
        d, H, G, dk, dv = p["width"], p["heads"], p["kv_heads"], p["dim"], p["vdim"]
        borrows, sink, talk = self._flags()
        bias, values_are_keys, _ = self._variant()
        specs = {n["q"]: TensorSpec((H * dk, d)), n["o"]: TensorSpec((d, H * dv))}
        if sink:
            specs[n["sink"]] = TensorSpec((H,))
        if talk:
            specs[n["talk"]] = TensorSpec((H, H))
        if p.get("temperature"):
            specs[n["temp"]] = TensorSpec((H,))
        if p.get("gate"):
            specs[n["g"]] = TensorSpec((H * dv, d))
        if not borrows:
            specs[n["k"]] = TensorSpec((G * dk, d))
            if not values_are_keys:
                specs[n["v"]] = TensorSpec((G * dv, d))
        if bias:
            specs.update({n[r + "_bias"]: TensorSpec(specs[n[r]].shape[:1]) for r in ("q", "o", "k", "v") if n.get(r) in specs})
        return specs

    def cache_need(self):
        p = self.params
        return KVNeed(p["kv_heads"], p["dim"], int(p.get("cache_window", p.get("window", 0))), value_dim=p["vdim"])

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.H, self.G, self.dk, self.dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
        if self.H % self.G:
            raise ValueError(f"{self.H} heads are no multiple of {self.G} key-value heads")
        self.scale, self.window, self.rot = float(p["scale"]), int(p.get("window", 0)), int(p.get("rot_dims", 0))
        self.borrows, sink, talk = self._flags()
        bias, self.values_are_keys, self.adjacent = self._variant()
        self.position = p.get("position")
        if self.rot and (self.position is None or self.rot % 2 or self.rot > self.dk):
            raise ValueError("rot_dims must be even, at most the key head size, and come with a rotary encoding")
        roles = ("q",) if self.borrows else ("q", "k") if self.values_are_keys else ("q", "k", "v")
        ws = [tensors[n[r]] for r in roles]
        self.gated = bool(p.get("gate"))
        if self.gated and bias:
            raise ValueError("sink attention: an output gate comes without projection biases")
        if self.gated:
            # the gate's columns start at a multiple of eight, so that rows of eight can be read from them at once
            rows = sum(w.shape[0] for w in ws)
            if rows % 8:
                ws.append(torch.zeros(8 - rows % 8, ws[0].shape[1], dtype=ws[0].dtype, device=ws[0].device))
            self.gate_at = sum(w.shape[0] for w in ws)
            ws.append(tensors[n["g"]])
        if len({w.dtype for w in ws}) != 1:
            ws = [w.float() for w in ws]
        rows = sum(w.shape[0] for w in ws)
        if rows % 8:
            ws.append(torch.zeros(8 - rows % 8, ws[0].shape[1], dtype=ws[0].dtype, device=ws[0].device))
        self.w_in = rt.weight(torch.cat(ws, dim=0))
        self.bias_in = torch.cat([tensors[n[r + "_bias"]].float() for r in roles]).contiguous() if bias else None
        self.w_o = rt.weight(tensors[n["o"]])
        self.output_bias = tensors[n["o_bias"]].float().contiguous() if bias else None
        self.on_matrix_cores = rt.ops.sink_attn_mfma_supported(rt.dtype, self.dk, self.dv) and self.scale > 0 \
            and os.environ.get("BURN_LM_AMD_SINK_ATTENTION") != "generic"
        # without head mixing and with values of the keys' size this is the plain attention's arithmetic plus a share of
        # the denominator: the plain attention's matrix-core kernels take the sink
        self.on_plain_kernels = self.on_matrix_cores and not talk and self.dk == self.dv \
            and rt.ops.attn_decode_supported(rt.dtype, self.dk) and rt.ops.attn_prefill_mfma_supported(rt.dtype, self.dk) \
            and os.environ.get("BURN_LM_AMD_SINK_ATTENTION") != "own"
        if self.on_matrix_cores:
            rt.ops.latent_attn_init(rt.device)     # the pieces' workspace, before any step is recorded
            rt.ops.sink_attn_mfma_init(rt.device)  # likewise: the shared memory of the form that stages pages
        self.temperature = tensors[n["temp"]].float().contiguous() if p.get("temperature") else None
        self.sinks = tensors[n["sink"]].float().contiguous() if sink else None
        self.talk = tensors[n["talk"]].float().contiguous() if talk else None

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_in, self.w_o))

    def step_flops(self, rows):
        return 2 * rows * (self.w_in.w.numel() + self.w_o.w.numel())

    def mixing_flops(self, past, new):
        """Scores once, weighted values once for every key-value head (the mixing is done behind the sum over keys)."""
        keys = sum(min(past + t + 1, self.window) if self.window else past + t + 1 for t in range(new)) if self.window \
            else new * past + new * (new + 1) // 2
        return 2 * self.H * (self.dk + self.dv * (self.G if self.talk is not None else 1)) * keys

    def forward(self, x, step, view):
        """The whole mixer, its output bias added."""
        out = self.rt.linear(self.attend(self.project(x, step, view), step, view), self.w_o)
        return out.add_(self.output_bias.to(out.dtype)) if self.output_bias is not None else out

    def forward_unbiased(self, x, step, view):
        """(result without the output projection's bias, possibly as partial planes; that bias in float32): for a
        block that adds both to the residual stream itself."""
        return self.output(self.attend(self.project(x, step, view), step, view)), self.output_bias

    def forward_terms(self, x, step, view):
        if self.output_bias is not None:
            return super().forward_terms(x, step, view)
        return [Term(self.forward_unbiased(x, step, view)[0])]

    def project(self, x, step, view):
        """q (and k, v) of the step's tokens with their biases, q and k turned by position, k and v stored."""
        rt = self.rt
        if view.need.head_dim != self.dk or view.need.v_dim != self.dv or view.need.n_kv_heads != self.G:
            raise ValueError("the cache's pages do not have this layer's head counts and sizes")
        qkv = rt.linear(x, self.w_in)
        if self.rot and step.max_position >= self.position.n_positions:
            raise ValueError(f"position {step.max_position} is past the rotary table of {self.position.n_positions}")
        store = not self.borrows
        if store != bool(view.store):
            raise ValueError("a layer with key and value projections keeps its own pages, a borrowing layer reads another's")
        rt.ops.qkv_prepare(qkv, self.bias_in, self.position.table if self.rot else None, self.rot, step,
                           view.block_table(step), view.k, view.v, view.page_size, self.H, self.G, self.dk, self.dv,
                           write_kv=store, adjacent=self.adjacent, values_are_keys=self.values_are_keys,
                           q_scale=self.temperature)
        return qkv

    def attend(self, qkv, step, view):
        """What the output projection reads: the heads' results, behind the output gate where the layer has one."""
        out = self._attend(qkv, step, view)
        if self.gated:
            n = self.H * self.dv
            self.rt.ops.sigmoid_gate(out, qkv[:, self.gate_at:self.gate_at + n])
        return out

    def _attend(self, qkv, step, view):
        """Every token's queries over its sequence's visible keys -> [tokens, heads * vdim].  bfloat16 with pages of
        64 keys and head sizes the matrix-core kernel takes: that kernel, its pages cut into pieces when a step
        brings so few tiles (decoding) that they would leave most of the chip idle; else the generic kernel."""
        rt = self.rt
        out = torch.empty(qkv.shape[0], self.H * self.dv, dtype=rt.dtype, device=qkv.device)
        if self.on_plain_kernels and view.page_size == 64 and qkv.stride(0) % 8 == 0 and qkv.data_ptr() % 16 == 0:
            return self._attend_plain(qkv, out, step, view)
        if self.on_matrix_cores and view.page_size == 64 and qkv.stride(0) % 8 == 0 and qkv.data_ptr() % 16 == 0 \
                and hasattr(step, "lens_after"):
            n_splits, group_batch = 1, 0
            if step.max_new == 1:
                span = step.max_len_after if not self.window else min(step.max_len_after, self.window + view.page_size)
                pages = (span + view.page_size - 1) // view.page_size
                group_batch = int(os.environ.get("BURN_LM_AMD_SINK_GROUP_BATCH", "1"))
                batches = -(-self.G // max(1, min(4, group_batch or 4))) if self.talk is not None else 1
                tiles = step.n_seqs * self.G * -(-(self.H // self.G) // 16) * batches
                n_splits = max(1, min(pages, (4 * rt.compute_units) // max(1, tiles),
                                      rt.ops.sink_attn_mfma_max_splits(step.n_seqs, 1, self.H, self.G, self.dv,
                                                                       self.talk is not None)))
            return rt.ops.sink_attn_mfma(qkv, out, self.sinks, self.talk, step, view.block_table(step), view.k, view.v,
                                         view.page_size, self.H, self.G, self.dk, self.dv, self.scale, self.window,
                                         n_splits=n_splits, group_batch=group_batch)
        return rt.ops.sink_attn(qkv, out, self.sinks, self.talk, step, view.block_table(step), view.k, view.v,
                                view.page_size, self.H, self.G, self.dk, self.dv, self.scale, self.window)

    def _attend_plain(self, qkv, out, step, view):
        """The plain attention's kernels (decode: key ranges cut as that mixer cuts them), with the sink."""
        from .attention import decode_splits
        rt, table = self.rt, view.block_table(step)
        H, G, hd = self.H, self.G, self.dk
        if step.max_new == 1:
            span = step.max_len_after if not self.window else min(step.max_len_after, self.window + view.page_size)
            pages = (span + view.page_size - 1) // view.page_size
            blocks = qkv.shape[0] * G * ((H // G + 15) // 16)
            rt.ops.attn_decode(qkv, qkv.stride(0), out, step.positions, step.token_seq, table, view.k, view.v, view.page_size,
                               H, G, hd, self.scale, self.window, decode_splits(pages, blocks, hd, rt.compute_units),
                               sinks=self.sinks)
        else:
            queries = rt.prefill_queries or rt.ops.attn_prefill_queries(step.n_seqs, step.max_new, H, G, hd, rt.compute_units)
            if queries == 32 and (hd % 32 or hd > 128):
                queries = 16
            rt.ops.attn_prefill_mfma(qkv, qkv.stride(0), out, step.positions, step.cu_seqlens, table, view.k, view.v,
                                     view.page_size, step.n_seqs, step.max_new, H, G, hd, self.scale, self.window,
                                     queries=queries, sinks=self.sinks)
        return out

    def output(self, attended):
        return self.rt.linear(attended, self.w_o, partials=True)
