"""The Girelix design as a plan of parts.

A decoder whose layers run their mixer and their feed-forward side by side behind one RMS norm, each result
multiplied by a stored vector (layer scale) and the sum by a residual multiplier.  The mixer is a pair: softmax
attention (grouped queries, rotation of adjacent lanes, a softmax sink, values that are the unrotated keys) beside
lightning attention (a matrix state per head that fades by a constant), added with two factors.  The feed-forward is
a mixture of experts routed by corrected scores within the best groups, some of whose experts pass their input
through; a layer may have none.  Output: RMS norm, then a head matrix of its own.

Checkpoint tensor names: ``embed``, ``head``, ``final.norm``; per layer i ``l<i>.norm1``, ``l<i>.ls1``, ``l<i>.ls2``,
``l<i>.mix.left.q|k|sink|o``, ``l<i>.mix.right.q|k|v|g|norm|o``, ``l<i>.mlp.router|correction|e<j>.gate|up|down``."""
from __future__ import annotations

from ..config.girelix import MAX_POSITIONS, GirelixConfig
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from ..weights.random_init import Normal, Ones, Uniform
from .plan import LayerPlan, ModelPlan, Place


def _mixer(cfg, i, positions):
    m, p, D = cfg.layers[i].mixer, f"l{i}.mix.", cfg.width
    a, b = m.left, m.right
    key = None
    if a.rot_dims:
        key = f"rope_{a.rot_dims}_{a.rot_base!r}"
        positions.setdefault(key, PartSpec("rope", dict(head_dim=a.rot_dims, theta=a.rot_base, pairing="interleaved",
                                                        scaling=None)))
    left = PartSpec("sink_attention",
                    dict(width=D, heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim, scale=a.scale, window=0,
                         rot_dims=a.rot_dims, talk=False, bias=False, pairing="adjacent", values="keys"),
                    dict(q=p + "left.q", k=p + "left.k", o=p + "left.o", sink=p + "left.sink"))
    right = PartSpec("lightning_attention",
                     dict(width=D, heads=b.heads, dim=b.dim, vdim=b.vdim, decay=b.decay, eps=cfg.eps),
                     {r: f"{p}right.{r}" for r in ("q", "k", "v", "g", "norm", "o")})
    return PartSpec("mixer_pair", dict(width=D, left=left, right=right, left_scale=m.left_scale,
                                       right_scale=m.right_scale)), key


def _feed_forward(cfg, i):
    f, p = cfg.layers[i].mlp, f"l{i}.mlp."
    names = dict(router=p + "router", correction=p + "correction")
    for e in range(f.experts):
        names.update({f"e{e}.{r}": f"{p}e{e}.{r}" for r in ("gate", "up", "down")})
    return PartSpec("grouped_experts", dict(width=cfg.width, experts=f.experts, identity=f.identity, top=f.top,
                                            groups=f.groups, keep=f.keep, expert_inner=f.ff), names)


def plan(cfg: GirelixConfig, checkpoint=None) -> ModelPlan:
    D = cfg.width
    positions, layers = {}, []
    norm = lambda name: PartSpec("rmsnorm", dict(width=D, eps=cfg.eps), dict(weight=name))
    for i, layer in enumerate(cfg.layers):
        l = f"l{i}."
        mixer, position = _mixer(cfg, i, positions)
        parts = dict(norm=norm(l + "norm1"), mixer=mixer)
        if layer.mlp is None:
            parts["scale"] = PartSpec("layer_scale", dict(width=D, mult=cfg.residual_mult, roles=("mixer",)),
                                      dict(mixer=l + "ls1"))
            layers.append(LayerPlan("parallel_scaled_mixer_only", parts, position=position))
        else:
            parts["feed_forward"] = _feed_forward(cfg, i)
            parts["scale"] = PartSpec("layer_scale", dict(width=D, mult=cfg.residual_mult),
                                      dict(mixer=l + "ls1", feed_forward=l + "ls2"))
            layers.append(LayerPlan("parallel_scaled", parts, position=position))
    ignorable = [rf"^l{i}\.ls2$" for i, layer in enumerate(cfg.layers) if layer.mlp is None]
    return ModelPlan(
        vocab_size=cfg.vocab, width=D, max_positions=MAX_POSITIONS,
        embedding=PartSpec("table", dict(vocab=cfg.vocab, width=D), dict(weight="embed")),
        layers=layers, order=[Place(i) for i in range(len(cfg.layers))], final_norm=norm("final.norm"),
        head=PartSpec("linear", dict(vocab=cfg.vocab, width=D), dict(weight="head")),
        positions=positions, stop_ids=(), ignorable_tensors=tuple(ignorable))


def checkpoint_tensors(cfg: GirelixConfig):
    """Name -> (shape, initialiser) of a fresh checkpoint: matrices N(0, 1/sqrt(fan-in)), norms near one, layer scales
    of a size that matters, sinks and corrections large enough to change what is chosen."""
    D = cfg.width
    lin = lambda n_out, n_in: ((n_out, n_in), Normal(n_in ** -0.5))
    out = {"embed": ((cfg.vocab, D), Normal(1.0, layout="table")), "head": lin(cfg.vocab, D),
           "final.norm": ((D,), Ones(0.1))}
    for i, layer in enumerate(cfg.layers):
        l, a, b, f = f"l{i}.", layer.mixer.left, layer.mixer.right, layer.mlp
        out[l + "norm1"] = ((D,), Ones(0.1))
        out[l + "ls1"] = ((D,), Uniform(0.5, 1.0))
        p = l + "mix.left."
        out[p + "q"], out[p + "k"] = lin(a.heads * a.dim, D), lin(a.kv_heads * a.dim, D)
        out[p + "sink"] = ((a.heads,), Normal(1.0))
        out[p + "o"] = lin(D, a.heads * a.vdim)
        p = l + "mix.right."
        out[p + "q"], out[p + "k"] = lin(b.heads * b.dim, D), lin(b.heads * b.dim, D)
        out[p + "v"], out[p + "g"] = lin(b.heads * b.vdim, D), lin(b.heads * b.vdim, D)
        out[p + "norm"] = ((b.heads * b.vdim,), Ones(0.1))
        out[p + "o"] = lin(D, b.heads * b.vdim)
        if f is None:
            continue
        out[l + "ls2"] = ((D,), Uniform(0.5, 1.0))
        p = l + "mlp."
        n = f.experts + f.identity
        out[p + "router"], out[p + "correction"] = lin(n, D), ((n,), Normal(0.5 / n))
        for e in range(f.experts):
            out[f"{p}e{e}.gate"], out[f"{p}e{e}.up"], out[f"{p}e{e}.down"] = lin(f.ff, D), lin(f.ff, D), lin(D, f.ff)
    return out


GIRELIX = Architecture(name="Girelix", read_config=GirelixConfig.from_dict, plan=plan,
                       checkpoint_tensors=checkpoint_tensors, display_name="Girelix", created_by="")
register_architecture(GIRELIX, "girelix")
