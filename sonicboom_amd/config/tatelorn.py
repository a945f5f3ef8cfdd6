"""Typed configuration of the Tatelorn decoder, read from config.json.

The file lists the layers one by one; each names its mixer (``type``), the mixer's sizes and
constants (``mixer``) and its feed-forward (``mlp``, or null for a layer without one):

    {"architecture": "Tatelorn", "vocab": V, "width": D, "max_positions": P, "logit_scale": s,
     "embedding": {"scale": a}, "norm": {"eps": e},
     "layers": [{"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": c, "softcap": t, "v_mix": true},
                 "mlp": {"kind": "dense", "ff": F}},
                {"type": "attention", "mixer": {...},
                 "mlp": {"kind": "moe", "router": {"experts": E, "top": k}, "expert": {"ff": F, "limit": l},
                         "shared": {"ff": F2, "limit": l2}}}, ...]}

Every size and constant of the model is read here and handed to the parts as a parameter.  A key
that is missing or of the wrong kind is reported by its path (``layers[3].mixer.heads``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, read_key, token_id_list

MIXERS = ("attention",)
FEED_FORWARDS = ("dense", "moe")


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
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int            # query/key numbers per head
    vdim: int           # value numbers per head
    scale: float        # multiplies q . k
    softcap: float      # scores become softcap * tanh(score / softcap); 0: no cap
    v_mix: bool         # values are mixed with those of the first layer that says so


@dataclass(frozen=True)
class DenseFFConfig:
    ff: int
    kind: str = "dense"


@dataclass(frozen=True)
class MoEFFConfig:
    experts: int
    top: int
    ff: int
    limit: float
    shared_ff: int = 0          # 0: no expert that every token takes
    shared_limit: float = 0.0
    kind: str = "moe"


@dataclass(frozen=True)
class TatelornLayer:
    type: str
    mixer: AttentionConfig
    mlp: object                 # DenseFFConfig, MoEFFConfig or None


@dataclass(frozen=True)
class TatelornConfig:
    architecture: str
    vocab: int
    width: int
    max_positions: int
    embedding_scale: float
    logit_scale: float
    norm_eps: float
    layers: Tuple[TatelornLayer, ...]
    eos_token_ids: Tuple[int, ...] = ()
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "TatelornConfig":
        norm = _obj(d, "norm", "")
        emb = _obj(d, "embedding", "", optional=True) or {}
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("missing/invalid config key: layers (want a list of layers)")
        layers = []
        for i, layer in enumerate(raw_layers):
            path = f"layers[{i}]"
            if not isinstance(layer, Mapping):
                raise ConfigError(f"missing/invalid config key: {path} (want an object)")
            kind = _at(path, read_key, layer, "type", str)
            if kind not in MIXERS:
                raise ConfigError(f"unknown layer type: {path}.type = {kind!r} (known: {', '.join(MIXERS)})")
            mx, mp = _obj(layer, "mixer", path + "."), path + ".mixer"
            heads = _at(mp, read_key, mx, "heads", int)
            dim = _at(mp, read_key, mx, "dim", int)
            mixer = AttentionConfig(
                heads=heads, kv_heads=_at(mp, read_key, mx, "kv_heads", int, heads), dim=dim,
                vdim=_at(mp, read_key, mx, "vdim", int, dim), scale=_at(mp, read_key, mx, "scale", float),
                softcap=_at(mp, read_key, mx, "softcap", float, 0.0), v_mix=_at(mp, read_key, mx, "v_mix", bool, False))
            mlp, fp = _obj(layer, "mlp", path + ".", optional=True), path + ".mlp"
            ff = None
            if mlp is not None:
                ff_kind = _at(fp, read_key, mlp, "kind", str, "dense")
                if ff_kind == "dense":
                    ff = DenseFFConfig(ff=_at(fp, read_key, mlp, "ff", int))
                elif ff_kind == "moe":
                    router, expert = _obj(mlp, "router", fp + "."), _obj(mlp, "expert", fp + ".")
                    shared = _obj(mlp, "shared", fp + ".", optional=True)
                    ff = MoEFFConfig(
                        experts=_at(fp + ".router", read_key, router, "experts", int),
                        top=_at(fp + ".router", read_key, router, "top", int),
                        ff=_at(fp + ".expert", read_key, expert, "ff", int),
                        limit=_at(fp + ".expert", read_key, expert, "limit", float),
                        shared_ff=0 if shared is None else _at(fp + ".shared", read_key, shared, "ff", int),
                        shared_limit=0.0 if shared is None else _at(fp + ".shared", read_key, shared, "limit", float))
                else:
                    raise ConfigError(f"unknown feed-forward kind: {fp}.kind = {ff_kind!r} "
                                      f"(known: {', '.join(FEED_FORWARDS)})")
            layers.append(TatelornLayer(kind, mixer, ff))
        known = {"architecture", "architectures", "vocab", "width", "max_positions", "embedding", "logit_scale", "norm",
                 "layers", "eos_token_id"}
        cfg = cls(
            architecture="Tatelorn",
            vocab=read_key(d, "vocab", int), width=read_key(d, "width", int),
            max_positions=read_key(d, "max_positions", int),
            embedding_scale=_at("embedding", read_key, emb, "scale", float, 1.0),
            logit_scale=read_key(d, "logit_scale", float, 1.0),
            norm_eps=_at("norm", read_key, norm, "eps", float),
            layers=tuple(layers),
            eos_token_ids=token_id_list(d.get("eos_token_id"), "eos_token_id"),
            extra={k: v for k, v in d.items() if k not in known})
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.max_positions <= 0:
            raise ConfigError("vocab, width and max_positions must be positive")
        if self.norm_eps < 0:
            raise ConfigError("norm.eps must not be negative")
        mixed = None
        for i, layer in enumerate(self.layers):
            m, path = layer.mixer, f"layers[{i}].mixer"
            for key in ("heads", "kv_heads", "dim", "vdim"):
                if getattr(m, key) <= 0:
                    raise ConfigError(f"{path}.{key} must be positive")
            if m.heads % m.kv_heads:
                raise ConfigError(f"{path}: {m.heads} heads are not a multiple of {m.kv_heads} kv_heads")
            if m.softcap < 0:
                raise ConfigError(f"{path}.softcap must not be negative")
            if m.v_mix:
                if mixed is not None and mixed[1] != (m.kv_heads, m.vdim):
                    raise ConfigError(f"{path}: kv_heads and vdim differ from those of layer {mixed[0]}, whose values it mixes in")
                mixed = mixed or (i, (m.kv_heads, m.vdim))
            f, fp = layer.mlp, f"layers[{i}].mlp"
            if isinstance(f, DenseFFConfig) and f.ff <= 0:
                raise ConfigError(f"{fp}.ff must be positive")
            if isinstance(f, MoEFFConfig):
                if f.experts <= 0 or not 0 < f.top <= f.experts:
                    raise ConfigError(f"{fp}.router: top = {f.top} must be between 1 and experts = {f.experts}")
                if f.ff <= 0 or f.shared_ff < 0:
                    raise ConfigError(f"{fp}: the experts' ff must be positive")

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            m, f = layer.mixer, layer.mlp
            mx = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                  "softcap": m.softcap, "v_mix": m.v_mix}
            if f is None:
                mlp = None
            elif isinstance(f, DenseFFConfig):
                mlp = {"kind": "dense", "ff": f.ff}
            else:
                mlp = {"kind": "moe", "router": {"experts": f.experts, "top": f.top},
                       "expert": {"ff": f.ff, "limit": f.limit},
                       "shared": {"ff": f.shared_ff, "limit": f.shared_limit} if f.shared_ff else None}
            layers.append({"type": layer.type, "mixer": mx, "mlp": mlp})
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
             "max_positions": self.max_positions, "embedding": {"scale": self.embedding_scale},
             "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        d.update(self.extra)
        return d
