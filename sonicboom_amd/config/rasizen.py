"""Typed configuration of the Rasizen decoder, read from config.json.

The file lists the layers one by one; each names its mixer (``type``), the mixer's sizes
(``mixer``) and its feed-forward (``mlp``, or null for a layer without one):

    {"architecture": "Rasizen", "vocab": V, "width": D, "residual_mult": m,
     "norm": {"eps": e, "groups": G},
     "layers": [{"type": "mingru", "mixer": {"width": W}, "mlp": null},
                {"type": "latent_attention",
                 "mixer": {"heads": H, "dim": d, "rot_dim": r, "vdim": v, "kv_rank": c, "scale": s,
                           "mask": {"size": w}, "rot": {"base": b, "dims": n}, "kv_from": j},
                 "mlp": {"kind": "dense", "ff": F}}, ...]}

Every size and constant of the model is read here and handed to the parts as a parameter;
no part knows a number of its own.  A key that is missing or of the wrong kind is reported by
its path (``layers[3].mixer.heads``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, read_key

MIXERS = ("mingru", "latent_attention")
FEED_FORWARDS = ("dense",)


def _at(path: str, fn, *a):
    """``fn(*a)`` with the path of the object in front of the key a ConfigError names."""
    try:
        return fn(*a)
    except ConfigError as e:
        raise ConfigError(str(e).replace("config key: ", f"config key: {path}.", 1)) from None


def _obj(d: Mapping, key: str, path: str, optional: bool = False):
    v = d.get(key)
    if v is None and optional:
        return None
    if not isinstance(v, Mapping):
        raise ConfigError(f"missing/invalid config key: {path}{key} (want an object)")
    return v


@dataclass(frozen=True)
class MinGRUConfig:
    """The gated recurrence's inner width."""
    width: int


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int            # plain (not rotated) query/key numbers per head
    rot_dim: int        # rotated query/key numbers per head; the rotated key part is shared by the heads
    vdim: int           # value numbers per head
    kv_rank: int        # size of the latent that is kept per token
    scale: float
    window: int         # a position sees itself and the window - 1 before it; 0: all before it
    rot_base: float
    rot_dims: int       # how many of the rot_dim numbers turn (the rest pass)
    kv_from: Optional[int] = None   # the earlier layer whose latent and rotated key this layer reads


@dataclass(frozen=True)
class DenseFFConfig:
    kind: str
    ff: int


@dataclass(frozen=True)
class RasizenLayer:
    type: str
    mixer: object                       # MinGRUConfig or LatentAttentionConfig
    mlp: Optional[DenseFFConfig]


@dataclass(frozen=True)
class RasizenConfig:
    architecture: str
    vocab: int
    width: int
    residual_mult: float
    norm_eps: float
    norm_groups: int
    layers: Tuple[RasizenLayer, ...]
    eos_token_ids: Tuple[int, ...] = ()
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "RasizenConfig":
        norm = _obj(d, "norm", "")
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("missing/invalid config key: layers (want a list of layers)")
        layers = []
        for i, layer in enumerate(raw_layers):
            path = f"layers[{i}]"
            if not isinstance(layer, Mapping):
                raise ConfigError(f"missing/invalid config key: {path} (want an object)")
            kind = _at(path, read_key, layer, "type", str)
            mx = _obj(layer, "mixer", path + ".")
            mp = path + ".mixer"
            if kind == "mingru":
                mixer = MinGRUConfig(width=_at(mp, read_key, mx, "width", int))
            elif kind == "latent_attention":
                mask = _obj(mx, "mask", mp + ".", optional=True)
                rot = _obj(mx, "rot", mp + ".")
                rot_dim = _at(mp, read_key, mx, "rot_dim", int)
                mixer = LatentAttentionConfig(
                    heads=_at(mp, read_key, mx, "heads", int), dim=_at(mp, read_key, mx, "dim", int),
                    rot_dim=rot_dim, vdim=_at(mp, read_key, mx, "vdim", int),
                    kv_rank=_at(mp, read_key, mx, "kv_rank", int), scale=_at(mp, read_key, mx, "scale", float),
                    window=0 if mask is None else _at(mp + ".mask", read_key, mask, "size", int, 0),
                    rot_base=_at(mp + ".rot", read_key, rot, "base", float),
                    rot_dims=_at(mp + ".rot", read_key, rot, "dims", int, rot_dim),
                    kv_from=_at(mp, read_key, mx, "kv_from", int, None))
            else:
                raise ConfigError(f"unknown layer type: {path}.type = {kind!r} (known: {', '.join(MIXERS)})")
            mlp = _obj(layer, "mlp", path + ".", optional=True)
            ff = None
            if mlp is not None:
                ff = DenseFFConfig(kind=_at(path + ".mlp", read_key, mlp, "kind", str, "dense"),
                                   ff=_at(path + ".mlp", read_key, mlp, "ff", int))
                if ff.kind not in FEED_FORWARDS:
                    raise ConfigError(f"unknown feed-forward kind: {path}.mlp.kind = {ff.kind!r} "
                                      f"(known: {', '.join(FEED_FORWARDS)})")
            layers.append(RasizenLayer(kind, mixer, ff))
        from .base import token_id_list
        known = {"architecture", "architectures", "vocab", "width", "residual_mult", "norm", "layers", "eos_token_id"}
        cfg = cls(
            architecture="Rasizen",
            vocab=read_key(d, "vocab", int), width=read_key(d, "width", int),
            residual_mult=read_key(d, "residual_mult", float, 1.0),
            norm_eps=_at("norm", read_key, norm, "eps", float),
            norm_groups=_at("norm", read_key, norm, "groups", int, 1),
            layers=tuple(layers),
            eos_token_ids=token_id_list(d.get("eos_token_id"), "eos_token_id"),
            extra={k: v for k, v in d.items() if k not in known})
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if self.norm_groups <= 0 or self.width % self.norm_groups:
            raise ConfigError(f"norm.groups = {self.norm_groups} does not divide the width {self.width}")
        if self.norm_eps < 0:
            raise ConfigError("norm.eps must not be negative")
        for i, layer in enumerate(self.layers):
            m, path = layer.mixer, f"layers[{i}].mixer"
            if isinstance(m, MinGRUConfig):
                if m.width <= 0:
                    raise ConfigError(f"{path}.width must be positive")
            else:
                for key in ("heads", "dim", "vdim", "kv_rank"):
                    if getattr(m, key) <= 0:
                        raise ConfigError(f"{path}.{key} must be positive")
                if m.rot_dim < 0 or m.window < 0:
                    raise ConfigError(f"{path}: rot_dim and mask.size must not be negative")
                if m.rot_dims < 0 or m.rot_dims % 2 or m.rot_dims > m.rot_dim:
                    raise ConfigError(f"{path}.rot.dims = {m.rot_dims} must be even and at most rot_dim = {m.rot_dim}")
                if m.rot_dims and m.rot_base <= 0:
                    raise ConfigError(f"{path}.rot.base must be positive")
                if m.kv_from is not None:
                    src = self.layers[m.kv_from].mixer if 0 <= m.kv_from < i else None
                    if not isinstance(src, LatentAttentionConfig) or src.kv_from is not None:
                        raise ConfigError(f"{path}.kv_from = {m.kv_from} must name an earlier latent_attention layer "
                                          f"that keeps a latent of its own")
                    if (src.kv_rank, src.rot_dim, src.rot_dims, src.rot_base) != (m.kv_rank, m.rot_dim, m.rot_dims, m.rot_base):
                        raise ConfigError(f"{path}: kv_rank, rot_dim and rot differ from those of layer {m.kv_from}, "
                                          f"whose latent it reads")
            if layer.mlp is not None and layer.mlp.ff <= 0:
                raise ConfigError(f"layers[{i}].mlp.ff must be positive")

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, MinGRUConfig):
                mx = {"width": m.width}
            else:
                mx = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                      "scale": m.scale, "rot": {"base": m.rot_base, "dims": m.rot_dims}}
                if m.window:
                    mx["mask"] = {"size": m.window}
                if m.kv_from is not None:
                    mx["kv_from"] = m.kv_from
            layers.append({"type": layer.type, "mixer": mx,
                           "mlp": None if layer.mlp is None else {"kind": layer.mlp.kind, "ff": layer.mlp.ff}})
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
             "residual_mult": self.residual_mult, "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
             "layers": layers}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        d.update(self.extra)
        return d
