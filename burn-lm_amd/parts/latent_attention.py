"""Attention whose keys and values are expanded from one low-rank latent per token (latent attention).

``q = W_q x`` per head as ``[dim plain lanes | rot_dim lanes turned by position]``; ``W_dkv x`` gives the latent
``c`` (kv_rank lanes, RMS-normed with a weight) and one turned key part shared by all heads (rot_dim lanes).
A head's plain key is ``W_uk c`` and its value ``W_uv c``; score = (q_plain . k_plain + q_rot . k_rot) * scale,
causal softmax, output projection over the concatenated heads.  Only ``[c | k_rot]`` is cached: the scores are
computed as ``(W_uk^T q_plain) . c`` and the values applied as ``W_uv (sum_j p_j c_j)``, which is the same
function, so the cache holds one row of kv_rank + rot_dim lanes per token for all heads and no value pages.
Rotation: lane i of the first ``rot_dims`` turned lanes pairs with lane i + rot_dims/2 (``pairing="half"``, the
default), or lane 2i with lane 2i + 1 (``pairing="adjacent"``).

Variants by parameter: queries through a latent of their own (``q_rank``): ``c_q = rmsnorm(W_dq x)`` with a stored
weight, ``q = W_uq c_q``; a layer that borrows (``borrows=True``) has no ``W_dkv``: it reads the rows
``[c | k_rot]`` that an earlier layer keeps, as cached, and expands them with its own ``W_uk`` and ``W_uv``."""
from __future__ import annotations

import os

import torch

from .base import KVNeed, Mixer, TensorSpec

DECODE_BLOCKS_PER_UNIT = 2     # blocks of four (token, head) wavefronts the split decode aims for per compute unit
MFMA_MAX_PIECES = 64           # most pieces the matrix-core decode cuts a sequence's pages into


class LatentAttention(Mixer):
    """params: width, heads, dim, rot_dim, vdim, kv_rank, scale, rot_dims, eps, position (the rotary table's
    owner, given by the model builder), pairing ("half", the default, or "adjacent"), q_rank (0, the default: queries
    projected directly; else the size of the queries' latent), borrows (default False).
    names: q (or dq, dq_norm, uq with a query latent), uk, uv, o and, unless the layer borrows, dkv, dkv_norm."""
    graph_safe = True

    def tensor_specs(self):
        p, n = self.params, self.names
        d, H, dn, dr, dv, R = p["width"], p["heads"], p["dim"], p["rot_dim"], p["vdim"], p["kv_rank"]
        specs = {n["uk"]: TensorSpec((H * dn, R)), n["uv"]: TensorSpec((H * dv, R)), n["o"]: TensorSpec((d, H * dv))}
        qr = int(p.get("q_rank", 0))
        if qr:
            specs.update({n["dq"]: TensorSpec((qr, d)), n["dq_norm"]: TensorSpec((qr,)),
                          n["uq"]: TensorSpec((H * (dn + dr), qr))})
        else:
            specs[n["q"]] = TensorSpec((H * (dn + dr), d))
        if not p.get("borrows"):
            specs.update({n["dkv"]: TensorSpec((R + dr, d)), n["dkv_norm"]: TensorSpec((R,))})
        return specs

    def cache_need(self):
        """One row [latent | turned key part] per token for all heads.  Where the matrix-core attention runs
        (bfloat16, sizes it is built for) the latent is kept a second time, transposed, as the value pages."""
        p = self.params
        if getattr(self, "use_mfma", False):
            return KVNeed(1, p["kv_rank"] + p["rot_dim"], 0, value_dim=p["kv_rank"])
        return KVNeed(1, p["kv_rank"] + p["rot_dim"], 0, no_values=True)

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.H, self.dn, self.dr, self.dv, self.R = p["heads"], p["dim"], p["rot_dim"], p["vdim"], p["kv_rank"]
        self.scale, self.eps, self.rot = float(p["scale"]), float(p["eps"]), int(p["rot_dims"])
        if self.rot % 2 or not 0 <= self.rot <= self.dr:
            raise ValueError(f"{self.rot} turning lanes do not fit a turned part of {self.dr} lanes")
        self.position = p["position"]
        pairing = p.get("pairing", "half")
        if pairing not in ("half", "adjacent"):
            raise ValueError(f"latent attention: pairing={pairing!r} unknown (half, adjacent)")
        self.adjacent, self.borrows, self.q_rank = pairing == "adjacent", bool(p.get("borrows")), int(p.get("q_rank", 0))
        ws = [tensors[n["dq"] if self.q_rank else n["q"]]] + ([] if self.borrows else [tensors[n["dkv"]]])
        if len({w.dtype for w in ws}) != 1:
            ws = [w.float() for w in ws]
        self.n_q = ws[0].shape[0]
        if len(ws) > 1 and self.n_q % 8:      # the down-projection's columns start at a multiple of eight
            ws.insert(1, torch.zeros(8 - self.n_q % 8, ws[0].shape[1], dtype=ws[0].dtype, device=ws[0].device))
        self.down_at = sum(w.shape[0] for w in ws[:-1]) if not self.borrows else 0
        self.w_in = rt.weight(torch.cat(ws, dim=0))
        # (a reading layer writes no rows and has no weight for their norm; the kernel's check wants one of its size)
        self.norm_w = torch.ones(self.R, dtype=torch.float32, device=rt.device) if self.borrows \
            else tensors[n["dkv_norm"]].float().contiguous()
        if self.q_rank:
            self.q_norm_w = tensors[n["dq_norm"]].float().contiguous()
            self.w_uq = rt.weight(tensors[n["uq"]])
        H, dn, dv, R = self.H, self.dn, self.dv, self.R
        self.w_uk_t = tensors[n["uk"]].view(H, dn, R).transpose(1, 2).contiguous()   # [H, R, dn]: q_plain -> latent lanes
        self.w_uv = tensors[n["uv"]].view(H, dv, R).contiguous()
        self.w_o = rt.weight(tensors[n["o"]])
        rt.ops.latent_attn_init(rt.device)
        self.use_mfma = (os.environ.get("BURN_LM_AMD_LATENT_MFMA") != "0" and self.w_uk_t.dtype == torch.bfloat16
                         and rt.ops.latent_attn_mfma_supported(rt.dtype, R, self.dr))

    def _matrices(self):
        return [self.w_in.w, self.w_o.w, self.w_uk_t, self.w_uv] + ([self.w_uq.w] if self.q_rank else [])

    def step_bytes(self, rows):
        return sum(w.numel() * w.element_size() for w in self._matrices())

    def step_flops(self, rows):
        return 2 * rows * sum(w.numel() for w in self._matrices())

    def mixing_flops(self, past, new):
        """Scores over kv_rank + rot_dim lanes and weighted latents over kv_rank lanes, per (query, visible row, head)."""
        pairs = new * past + new * (new + 1) // 2
        return 2 * self.H * (2 * self.R + self.dr) * pairs

    def forward(self, x, step, view):
        return self.output(self.attend(self.project(x, step, view), step, view))

    def project(self, x, step, view):
        """The absorbed queries [tokens, heads, kv_rank + rot_dim] (float32) of the step's tokens; their latents and
        turned key parts are in the cache afterwards."""
        rt, ops = self.rt, self.rt.ops
        H, dn, dr, R = self.H, self.dn, self.dr, self.R
        T = x.shape[0]
        if self.borrows == bool(view.store):
            raise ValueError("a layer with a down-projection keeps its own rows, a borrowing layer reads another's")
        qd = rt.linear(x, self.w_in)                         # [T, H (dn + dr) or q_rank | R + dr]
        q, down = qd[:, :self.n_q], (None if self.borrows else qd[:, self.down_at:])
        if self.q_rank:
            cq = rt.ops.rmsnorm_rows(q, self.q_norm_w, self.eps, torch.empty(T, self.q_rank, dtype=qd.dtype, device=x.device))
            q = rt.linear(cq, self.w_uq)
        mfma = self.use_mfma and view.v.numel() > 0 and view.page_size == 64
        qabs = torch.empty(T, H, R + dr, dtype=rt.dtype if mfma else torch.float32, device=x.device)
        ops.latent_write(down, q, self.norm_w, self.eps,
                         self.position.table, self.rot, qabs, view.k, step, view.block_table(step), view.page_size, H, dn,
                         R, dr, write_kv=view.store, vcache=view.v if mfma and view.store else None,
                         adjacent=self.adjacent)
        ops.head_project(q, dn + dr, self.w_uk_t, qabs.view(T, H * (R + dr)), R + dr)
        return qabs

    def attend(self, qabs, step, view):
        """Every (token, head)'s weighted sum of the latents it sees -> float32 [tokens, heads, kv_rank]."""
        rt, ops = self.rt, self.rt.ops
        H, dr, R = self.H, self.dr, self.R
        T = qabs.shape[0]
        olat = torch.empty(T, H, R, dtype=torch.float32, device=qabs.device)
        n_splits = 1
        if qabs.dtype == torch.bfloat16:        # the matrix-core form: one wavefront per 16 (token, head) pairs
            if step.max_new == 1:
                waves = step.n_seqs * ((H + 15) // 16)
                pages = (step.max_len_after + 63) // 64
                # up to a wavefront for every vector unit of the chip: a wavefront waits out a page's trip from memory
                # with nothing else to do, so short pieces are what shortens the step
                n_splits = max(1, min(pages, (4 * rt.compute_units) // waves, MFMA_MAX_PIECES,
                                      ops.latent_attn_mfma_max_splits(step.n_seqs, 1, H, R)))
            return ops.latent_attn_mfma(qabs, olat, view.k, view.v, step, view.block_table(step), view.page_size, H, R,
                                        dr, self.scale, n_splits)
        if step.max_new == 1:
            chunks = (step.max_len_after + 63) // 64
            blocks = (T * H + 3) // 4
            n_splits = max(1, min(chunks, (DECODE_BLOCKS_PER_UNIT * rt.compute_units) // blocks,
                                  ops.latent_attn_max_splits(T, H, R)))
        return ops.latent_attn(qabs, olat, view.k, step, view.block_table(step), view.page_size, H, R, dr, self.scale,
                               n_splits)

    def output(self, olat):
        rt = self.rt
        T = olat.shape[0]
        o = torch.empty(T, self.H * self.dv, dtype=rt.dtype, device=olat.device)
        rt.ops.head_project(olat.view(T, self.H * self.R), self.R, self.w_uv, o, self.dv)
        return rt.linear(o, self.w_o, partials=True)
