"""The Bitonex design as a plan of parts.

A pre-norm decoder whose norms hold one number each and whose sublayers join the residual behind gates projected
from the sublayer's own input, times one residual multiplier.  Mixers, chosen layer by layer: softmax attention
(grouped queries, partial rotation of pairs half the turning lanes apart, a temperature per head, a sigmoid output
gate), lightning attention (a matrix state per head that fades by a constant), and latent attention (queries through
a normed latent, keys and values expanded from a cached latent with one turned key part for all heads, adjacent
pairs; a layer may read the rows an earlier layer keeps).  Feed-forward: dense, gated, tanh GELU; a layer may have
none.  Output: the norm, a head matrix of its own, a soft cap on the logits.

Checkpoint tensor names: ``embed``, ``head``, ``final.norm``; per layer i ``l<i>.norm1|norm2`` (no dimensions),
``l<i>.rg1|rg2`` with ``.b``, ``l<i>.mix.*`` (attention: ``q k v temp g o``; lightning: ``q k v g norm o``; latent
attention: ``dq dq.norm uq dkv dkv.norm uk uv o``), ``l<i>.mlp.gate|up|down``."""
from __future__ import annotations

from ..config.bitonex import MAX_POSITIONS, BitonexConfig
from ..errors import ConfigError
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from ..weights.random_init import Normal, Ones, Uniform
from .plan import LayerPlan, ModelPlan, Place


def _rope(positions, dims, base):
    """Key of the table of angles for `dims` turning lanes (made once per distinct (dims, base)); None without."""
    if not dims:
        return None
    key = f"rope_{dims}_{base!r}"
    positions.setdefault(key, PartSpec("rope", dict(head_dim=dims, theta=base, pairing="interleaved", scaling=None)))
    return key


def _q_rank(m, prefix, checkpoint):
    shape = checkpoint.get(prefix + "dq") if isinstance(checkpoint, dict) else None
    if shape is not None:
        return int(tuple(shape)[0])
    if m.q_rank is None:
        raise ConfigError(f"the size of the queries' latent of {prefix[:-1]} is neither in config.json (q_rank) nor in a "
                          f"checkpoint's shapes")
    return m.q_rank


def _mixer(cfg, i, positions, checkpoint):
    m, p, D = cfg.layers[i].mixer, f"l{i}.mix.", cfg.width
    if m.type == "attention":
        spec = PartSpec("sink_attention",
                        dict(width=D, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale, window=0,
                             rot_dims=m.rot_dims, sink=False, talk=False, bias=False, pairing="half", temperature=True,
                             gate=True),
                        {r: p + r for r in ("q", "k", "v", "temp", "g", "o")})
        return spec, _rope(positions, m.rot_dims, m.rot_base)
    if m.type == "lightning":
        return PartSpec("lightning_attention", dict(width=D, heads=m.heads, dim=m.dim, vdim=m.vdim, decay=m.decay, eps=cfg.eps),
                        {r: p + r for r in ("q", "k", "v", "g", "norm", "o")}), None
    names = dict(dq=p + "dq", dq_norm=p + "dq.norm", uq=p + "uq", uk=p + "uk", uv=p + "uv", o=p + "o")
    if m.kv_from is None:
        names.update(dkv=p + "dkv", dkv_norm=p + "dkv.norm")
    spec = PartSpec("latent_attention",
                    dict(width=D, heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim, kv_rank=m.kv_rank, scale=m.scale,
                         rot_dims=m.rot_dims, eps=cfg.eps, pairing="adjacent", q_rank=_q_rank(m, p, checkpoint),
                         borrows=m.kv_from is not None), names)
    return spec, _rope(positions, m.rot_dims, m.rot_base) or _rope(positions, 2, 1.0)


def plan(cfg: BitonexConfig, checkpoint=None) -> ModelPlan:
    D = cfg.width
    positions, layers = {}, []
    norm = lambda name: PartSpec("rmsnorm", dict(width=D, eps=cfg.eps, single=True), dict(weight=name))
    for i, layer in enumerate(cfg.layers):
        l = f"l{i}."
        mixer, position = _mixer(cfg, i, positions, checkpoint)
        parts = dict(mixer_norm=norm(l + "norm1"), mixer=mixer)
        gates = dict(mixer=l + "rg1", mixer_bias=l + "rg1.b")
        if layer.mlp is None:
            parts["gate"] = PartSpec("residual_gate", dict(width=D, mult=cfg.residual_mult, roles=("mixer",)), gates)
            layers.append(LayerPlan("pre_norm_gated_mixer_only", parts, position=position))
        else:
            parts["ffn_norm"] = norm(l + "norm2")
            parts["feed_forward"] = PartSpec("gelu_glu", dict(width=D, inner=layer.mlp.ff),
                                             {r: f"{l}mlp.{r}" for r in ("gate", "up", "down")})
            gates.update(feed_forward=l + "rg2", feed_forward_bias=l + "rg2.b")
            parts["gate"] = PartSpec("residual_gate", dict(width=D, mult=cfg.residual_mult), gates)
            layers.append(LayerPlan("pre_norm_gated", parts, position=position))
    order = [Place(i, reads_cache_of=getattr(layer.mixer, "kv_from", None)) for i, layer in enumerate(cfg.layers)]
    return ModelPlan(
        vocab_size=cfg.vocab, width=D, max_positions=MAX_POSITIONS,
        embedding=PartSpec("table", dict(vocab=cfg.vocab, width=D), dict(weight="embed")),
        layers=layers, order=order, final_norm=norm("final.norm"),
        head=PartSpec("linear", dict(vocab=cfg.vocab, width=D, softcap=cfg.logit_softcap), dict(weight="head")),
        positions=positions, stop_ids=())


def checkpoint_tensors(cfg: BitonexConfig):
    """Name -> (shape, initialiser) of a fresh checkpoint: matrices N(0, 1/sqrt(fan-in)), norms near one, temperatures
    around one, gate biases of a size that matters."""
    D = cfg.width
    lin = lambda n_out, n_in: ((n_out, n_in), Normal(n_in ** -0.5))
    out = {"embed": ((cfg.vocab, D), Normal(1.0, layout="table")), "head": lin(cfg.vocab, D), "final.norm": ((), Ones(0.1))}
    for i, layer in enumerate(cfg.layers):
        l, m, f = f"l{i}.", layer.mixer, layer.mlp
        out[l + "norm1"] = ((), Ones(0.1))
        out[l + "rg1"], out[l + "rg1.b"] = lin(D, D), ((D,), Normal(0.5))
        p = l + "mix."
        if m.type == "attention":
            out[p + "q"], out[p + "k"], out[p + "v"] = lin(m.heads * m.dim, D), lin(m.kv_heads * m.dim, D), lin(m.kv_heads * m.vdim, D)
            out[p + "temp"] = ((m.heads,), Uniform(0.5, 1.5))
            out[p + "g"], out[p + "o"] = lin(m.heads * m.vdim, D), lin(D, m.heads * m.vdim)
        elif m.type == "lightning":
            out[p + "q"], out[p + "k"] = lin(m.heads * m.dim, D), lin(m.heads * m.dim, D)
            out[p + "v"], out[p + "g"] = lin(m.heads * m.vdim, D), lin(m.heads * m.vdim, D)
            out[p + "norm"] = ((m.heads * m.vdim,), Ones(0.1))
            out[p + "o"] = lin(D, m.heads * m.vdim)
        else:
            qr = m.q_rank if m.q_rank is not None else max(8, D // 2)
            out[p + "dq"], out[p + "dq.norm"] = lin(qr, D), ((qr,), Ones(0.1))
            out[p + "uq"] = lin(m.heads * (m.dim + m.rot_dim), qr)
            if m.kv_from is None:
                out[p + "dkv"], out[p + "dkv.norm"] = lin(m.kv_rank + m.rot_dim, D), ((m.kv_rank,), Ones(0.1))
            out[p + "uk"], out[p + "uv"] = lin(m.heads * m.dim, m.kv_rank), lin(m.heads * m.vdim, m.kv_rank)
            out[p + "o"] = lin(D, m.heads * m.vdim)
        if f is None:
            continue
        out[l + "norm2"] = ((), Ones(0.1))
        out[l + "rg2"], out[l + "rg2.b"] = lin(D, D), ((D,), Normal(0.5))
        p = l + "mlp."
        out[p + "gate"], out[p + "up"], out[p + "down"] = lin(f.ff, D), lin(f.ff, D), lin(D, f.ff)
    return out


BITONEX = Architecture(name="Bitonex", read_config=BitonexConfig.from_dict, plan=plan,
                       checkpoint_tensors=checkpoint_tensors, display_name="Bitonex", created_by="")
register_architecture(BITONEX, "bitonex")
