"""Typed configuration of the Girelix design, read from the keys of its ``config.json``.

Top level: ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` and ``layers``: a list of ``{type, mixer, mlp}``.
``type`` is ``parallel``: one norm whose output the mixer and the feed-forward both read.  ``mixer`` holds two mixers
side by side, ``left`` (softmax attention: ``heads, kv_heads, dim, vdim, scale, rot: {dims, base}``) and ``right``
(lightning attention: ``heads, dim, vdim, decay`` with one decay per head, or one number for all), and their factors
``left_scale`` and ``right_scale``.  ``mlp`` is ``null`` (none) or ``{kind: moe, expert: {ff}, router: {experts, top, identity,
groups: {count, keep}}}`` (``identity`` and ``groups`` may be missing: no pass-through experts, one group).  Every
size is a required key."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError

MAX_POSITIONS = 1 << 20     # the design has no limit of its own; the cache's size decides


def _get(d, key, kind, where):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing in {where}")
    v = d[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
            raise ConfigError(f"config.json: '{key}' in {where} must be a positive integer, got {v!r}")
        return v
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: '{key}' in {where} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class SoftmaxSide:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int         # 0: no rotation
    rot_base: float


@dataclass(frozen=True)
class LightningSide:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]


@dataclass(frozen=True)
class PairConfig:
    left: SoftmaxSide
    right: LightningSide
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class MoeConfig:
    experts: int          # those with tensors
    identity: int         # pass-through experts behind them in the router's outputs
    top: int
    groups: int
    keep: int
    ff: int
    kind: str = "moe"


@dataclass(frozen=True)
class LayerConfig:
    mixer: PairConfig
    mlp: Optional[MoeConfig]


@dataclass(frozen=True)
class GirelixConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    layers: Tuple[LayerConfig, ...]

    @property
    def vocab_size(self):
        return self.vocab

    @property
    def max_positions(self):
        return MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "GirelixConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        out = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            if kind != "parallel":
                raise ConfigError(f"config.json: {where}.type is {kind!r}; known: parallel")
            m, mw = entry.get("mixer"), where + ".mixer"
            l, lw = (m or {}).get("left"), mw + ".left"
            heads, kv_heads = _get(l, "heads", int, lw), _get(l, "kv_heads", int, lw)
            if heads % kv_heads:
                raise ConfigError(f"config.json: {lw}.heads must be a multiple of kv_heads")
            dim, vdim = _get(l, "dim", int, lw), _get(l, "vdim", int, lw)
            if vdim != dim:
                raise ConfigError(f"config.json: {lw}.vdim must equal dim: the values of this attention are its keys")
            rot = l.get("rot")
            if isinstance(rot, dict) and rot.get("dims") == 0 and not isinstance(rot.get("dims"), bool):
                rot = None      # no lanes turn
            rot_dims = _get(rot, "dims", int, lw + ".rot") if rot is not None else 0
            if rot_dims % 2 or rot_dims > dim:
                raise ConfigError(f"config.json: {lw}.rot.dims must be even and at most dim")
            left = SoftmaxSide(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=_get(l, "scale", float, lw),
                               rot_dims=rot_dims, rot_base=_get(rot, "base", float, lw + ".rot") if rot is not None else 0.0)
            r, rw = m.get("right"), mw + ".right"
            r_heads = _get(r, "heads", int, rw)
            decay = r.get("decay")
            if isinstance(decay, (int, float)) and not isinstance(decay, bool):
                decay = [decay] * r_heads      # one number for all heads
            if not isinstance(decay, list) or len(decay) != r_heads \
                    or not all(isinstance(a, (int, float)) and not isinstance(a, bool) and 0.0 < a <= 1.0 for a in decay):
                raise ConfigError(f"config.json: {rw}.decay must list one number in (0, 1] for each of the {r_heads} heads")
            right = LightningSide(heads=r_heads, dim=_get(r, "dim", int, rw), vdim=_get(r, "vdim", int, rw),
                                  decay=tuple(float(a) for a in decay))
            pair = PairConfig(left, right, _get(m, "left_scale", float, mw), _get(m, "right_scale", float, mw))
            mlp, fw = entry.get("mlp"), where + ".mlp"
            if mlp is None:
                ff = None
            elif mlp.get("kind") == "moe":
                router, tw = mlp.get("router"), fw + ".router"
                experts, top = _get(router, "experts", int, tw), _get(router, "top", int, tw)
                identity = _get(router, "identity", int, tw) if router.get("identity") else 0
                groups = router.get("groups")
                count = _get(groups, "count", int, tw + ".groups") if groups is not None else 1
                keep = _get(groups, "keep", int, tw + ".groups") if groups is not None else 1
                if (experts + identity) % count or keep > count:
                    raise ConfigError(f"config.json: {tw}: {experts} + {identity} experts do not form {count} equal "
                                      f"groups of which {keep} stay")
                if top > keep * ((experts + identity) // count):
                    raise ConfigError(f"config.json: {tw}.top is more than the kept groups hold")
                ff = MoeConfig(experts=experts, identity=identity, top=top, groups=count, keep=keep,
                               ff=_get(mlp.get("expert"), "ff", int, fw + ".expert"))
            else:
                raise ConfigError(f"config.json: {fw}.kind is {mlp.get('kind')!r}; known: moe")
            out.append(LayerConfig(pair, ff))
        top_level = "the top level"
        return cls(vocab=_get(d, "vocab", int, top_level), width=_get(d, "width", int, top_level),
                   eps=_get(d.get("norm"), "eps", float, "norm"),
                   residual_mult=_get(d, "residual_mult", float, top_level), layers=tuple(out))
