"""Typed configuration of the Bitonex design, read from the keys of its ``config.json``.

Top level: ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``logit_softcap`` (missing or null: none) and
``layers``: a list of ``{type, mixer, mlp}``.  ``type`` names the mixer: ``attention`` (``heads, kv_heads, dim, vdim,
scale, rot: {dims, base}``), ``lightning`` (``heads, dim, vdim, decay`` with one decay per head, or one number for
all) or ``latent_attention`` (``heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot: {dims, base}`` and
optionally ``kv_from: j``: the layer has no down-projection of its own and reads the rows layer j keeps).  ``mlp`` is
``null`` (none) or ``{kind: dense, ff}``.  Every size is a required key; ``q_rank`` may instead be read from the
checkpoint's shapes by the plan."""
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


def _rot(m, where, most):
    """(turning lanes, base) of a mixer's ``rot``; missing, null or zero lanes: no rotation."""
    rot = m.get("rot")
    if rot is None or (isinstance(rot, dict) and rot.get("dims") == 0 and not isinstance(rot.get("dims"), bool)):
        return 0, 0.0
    dims = _get(rot, "dims", int, where + ".rot")
    if dims % 2 or dims > most:
        raise ConfigError(f"config.json: {where}.rot.dims must be even and at most {most}")
    return dims, _get(rot, "base", float, where + ".rot")


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int         # 0: no rotation
    rot_base: float
    type: str = "attention"


@dataclass(frozen=True)
class LightningConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    type: str = "lightning"


@dataclass(frozen=True)
class LatentConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: Optional[int]       # None: in the checkpoint's shapes only
    scale: float
    rot_dims: int
    rot_base: float
    kv_from: Optional[int]
    type: str = "latent_attention"


@dataclass(frozen=True)
class DenseConfig:
    ff: int
    kind: str = "dense"


@dataclass(frozen=True)
class LayerConfig:
    mixer: object
    mlp: Optional[DenseConfig]


@dataclass(frozen=True)
class BitonexConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    logit_softcap: float        # 0: none
    layers: Tuple[LayerConfig, ...]

    @property
    def vocab_size(self):
        return self.vocab

    @property
    def max_positions(self):
        return MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "BitonexConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        out = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            m, mw = (entry.get("mixer") if isinstance(entry, dict) else None), where + ".mixer"
            if kind == "attention":
                heads, kv_heads = _get(m, "heads", int, mw), _get(m, "kv_heads", int, mw)
                if heads % kv_heads:
                    raise ConfigError(f"config.json: {mw}.heads must be a multiple of kv_heads")
                dim = _get(m, "dim", int, mw)
                rot_dims, rot_base = _rot(m, mw, dim)
                mixer = AttentionConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=_get(m, "vdim", int, mw),
                                        scale=_get(m, "scale", float, mw), rot_dims=rot_dims, rot_base=rot_base)
            elif kind == "lightning":
                heads = _get(m, "heads", int, mw)
                decay = m.get("decay")
                if isinstance(decay, (int, float)) and not isinstance(decay, bool):
                    decay = [decay] * heads      # one number for all heads
                if not isinstance(decay, list) or len(decay) != heads \
                        or not all(isinstance(a, (int, float)) and not isinstance(a, bool) and 0.0 < a <= 1.0 for a in decay):
                    raise ConfigError(f"config.json: {mw}.decay must list one number in (0, 1] for each of the {heads} heads")
                mixer = LightningConfig(heads=heads, dim=_get(m, "dim", int, mw), vdim=_get(m, "vdim", int, mw),
                                        decay=tuple(float(a) for a in decay))
            elif kind == "latent_attention":
                kv_from = m.get("kv_from") if isinstance(m, dict) else None
                src = None
                if kv_from is not None:
                    if isinstance(kv_from, bool) or not isinstance(kv_from, int) or not 0 <= kv_from < i:
                        raise ConfigError(f"config.json: {mw}.kv_from must name an earlier layer, got {kv_from!r}")
                    src = out[kv_from].mixer
                    if src.type != "latent_attention" or src.kv_from is not None:
                        raise ConfigError(f"config.json: {mw}.kv_from names layer {kv_from}, which keeps no latent rows of its own")
                    # what the rows' shape decides may be left to the layer that keeps them
                    m = dict(m)
                    m.setdefault("kv_rank", src.kv_rank)
                    m.setdefault("rot_dim", src.rot_dim)
                    if m.get("rot") is None and src.rot_dims:
                        m["rot"] = dict(dims=src.rot_dims, base=src.rot_base)
                rot_dim = _get(m, "rot_dim", int, mw)
                rot_dims, rot_base = _rot(m, mw, rot_dim)
                mixer = LatentConfig(heads=_get(m, "heads", int, mw), dim=_get(m, "dim", int, mw), rot_dim=rot_dim,
                                     vdim=_get(m, "vdim", int, mw), kv_rank=_get(m, "kv_rank", int, mw),
                                     q_rank=_get(m, "q_rank", int, mw) if m.get("q_rank") is not None else None,
                                     scale=_get(m, "scale", float, mw), rot_dims=rot_dims, rot_base=rot_base, kv_from=kv_from)
                if src is not None and (src.kv_rank, src.rot_dim, src.rot_dims, src.rot_base) != \
                        (mixer.kv_rank, mixer.rot_dim, mixer.rot_dims, mixer.rot_base):
                    raise ConfigError(f"config.json: {mw} reads layer {kv_from}'s rows but differs from it in kv_rank, "
                                      f"rot_dim or rotation")
            else:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; known: attention, lightning, latent_attention")
            mlp, fw = entry.get("mlp"), where + ".mlp"
            if mlp is None:
                ff = None
            elif isinstance(mlp, dict) and mlp.get("kind") == "dense":
                ff = DenseConfig(ff=_get(mlp, "ff", int, fw))
            else:
                raise ConfigError(f"config.json: {fw}.kind is {mlp.get('kind') if isinstance(mlp, dict) else mlp!r}; known: dense")
            out.append(LayerConfig(mixer, ff))
        top_level = "the top level"
        cap = d.get("logit_softcap")
        if cap is not None and (isinstance(cap, bool) or not isinstance(cap, (int, float)) or cap < 0):
            raise ConfigError(f"config.json: 'logit_softcap' must be a positive number or null, got {cap!r}")
        return cls(vocab=_get(d, "vocab", int, top_level), width=_get(d, "width", int, top_level),
                   eps=_get(d.get("norm"), "eps", float, "norm"),
                   residual_mult=_get(d, "residual_mult", float, top_level) if d.get("residual_mult") is not None else 1.0,
                   logit_softcap=float(cap or 0.0), layers=tuple(out))
