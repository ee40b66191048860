"""Typed configuration of the Fitatar decoder, read from config.json.

The file lists the layers one by one; each names its mixer (``type``), the mixer's sizes and
constants (``mixer``) and its feed-forward (``mlp``, or null for a layer without one):

    {"architecture": "Fitatar", "vocab": V, "width": D, "logit_softcap": c,
     "embedding": {"scale": a}, "norm": {"eps": e},
     "layers": [{"type": "latent_attention",
                 "mixer": {"heads": H, "dim": d, "rot_dim": r, "vdim": v, "kv_rank": c, "q_rank": q, "scale": s,
                           "rot": {"base": b, "dims": n, "scaling": {"factor": f, "original": L, "fast": x, "slow": y}},
                           "kv_from": j},
                 "mlp": {"kind": "dense", "ff": F}},
                {"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": s,
                           "rot": {"base": b, "dims": n, "scaling": {"factor": f}}},
                 "mlp": {"kind": "moe", "router": {"experts": E, "top": k, "groups": {"count": g, "keep": m}},
                         "expert": {"ff": F}, "shared": {"ff": F2}}}, ...]}

Every size and constant of the model is read here and handed to the parts as a parameter.  A key
that is missing or of the wrong kind is reported by its path (``layers[3].mixer.heads``).  The
rotation of a ``latent_attention`` layer stretches its slow pairs with a ramp between two wavelengths
(``factor``, ``original``, ``fast``, ``slow``); that of an ``attention`` layer divides every frequency
by ``factor``.  A ``rot`` without ``scaling`` rotates by the plain frequencies.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, read_key, token_id_list

MIXERS = ("latent_attention", "attention")
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
class RotationConfig:
    base: float
    dims: int                   # how many numbers of a head (or of the rotated part) turn
    factor: float = 0.0         # 0: the frequencies as they are
    original: float = 0.0       # the ramp's length of reference (latent attention)
    fast: float = 32.0          # turns over that length of the pair where the ramp starts
    slow: float = 1.0           # and of the pair where it ends


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int            # plain (not rotated) query/key numbers per head
    rot_dim: int        # rotated query/key numbers per head; the rotated key part is shared by the heads
    vdim: int           # value numbers per head
    kv_rank: int        # size of the latent that is kept per token
    q_rank: int         # size of the queries' latent
    scale: float
    rot: RotationConfig
    kv_from: Optional[int] = None   # the earlier layer whose latent and rotated key this layer reads


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int            # query/key numbers per head
    vdim: int           # value numbers per head
    scale: float
    rot: RotationConfig


@dataclass(frozen=True)
class DenseFFConfig:
    ff: int
    kind: str = "dense"


@dataclass(frozen=True)
class MoEFFConfig:
    experts: int
    top: int
    ff: int
    groups: int = 1             # equal groups of neighbouring experts
    keep: int = 1               # groups whose experts can be chosen
    shared_ff: int = 0          # 0: no expert that every token takes
    kind: str = "moe"


@dataclass(frozen=True)
class FitatarLayer:
    type: str
    mixer: object               # LatentAttentionConfig or AttentionConfig
    mlp: object                 # DenseFFConfig, MoEFFConfig or None


def _rotation(mx: Mapping, mp: str, default_dims: int, ramp: bool) -> RotationConfig:
    rot = _obj(mx, "rot", mp + ".")
    rp = mp + ".rot"
    sc = _obj(rot, "scaling", rp + ".", optional=True)
    kw = {}
    if sc is not None:
        kw["factor"] = _at(rp + ".scaling", read_key, sc, "factor", float)
        if ramp:
            kw["original"] = _at(rp + ".scaling", read_key, sc, "original", float)
            kw["fast"] = _at(rp + ".scaling", read_key, sc, "fast", float)
            kw["slow"] = _at(rp + ".scaling", read_key, sc, "slow", float)
    return RotationConfig(base=_at(rp, read_key, rot, "base", float), dims=_at(rp, read_key, rot, "dims", int, default_dims), **kw)


def _rotation_dict(r: RotationConfig, ramp: bool) -> dict:
    d = {"base": r.base, "dims": r.dims}
    if r.factor:
        d["scaling"] = {"factor": r.factor}
        if ramp:
            d["scaling"].update(original=r.original, fast=r.fast, slow=r.slow)
    return d


@dataclass(frozen=True)
class FitatarConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    logit_softcap: float        # 0: logits as they are
    norm_eps: float
    layers: Tuple[FitatarLayer, ...]
    eos_token_ids: Tuple[int, ...] = ()
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "FitatarConfig":
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
            mx, mp = _obj(layer, "mixer", path + "."), path + ".mixer"
            if kind == "latent_attention":
                rot_dim = _at(mp, read_key, mx, "rot_dim", int)
                mixer = LatentAttentionConfig(
                    heads=_at(mp, read_key, mx, "heads", int), dim=_at(mp, read_key, mx, "dim", int), rot_dim=rot_dim,
                    vdim=_at(mp, read_key, mx, "vdim", int), kv_rank=_at(mp, read_key, mx, "kv_rank", int),
                    q_rank=_at(mp, read_key, mx, "q_rank", int), scale=_at(mp, read_key, mx, "scale", float),
                    rot=_rotation(mx, mp, rot_dim, ramp=True), kv_from=_at(mp, read_key, mx, "kv_from", int, None))
            elif kind == "attention":
                heads, dim = _at(mp, read_key, mx, "heads", int), _at(mp, read_key, mx, "dim", int)
                mixer = AttentionConfig(
                    heads=heads, kv_heads=_at(mp, read_key, mx, "kv_heads", int, heads), dim=dim,
                    vdim=_at(mp, read_key, mx, "vdim", int, dim), scale=_at(mp, read_key, mx, "scale", float),
                    rot=_rotation(mx, mp, dim, ramp=False))
            else:
                raise ConfigError(f"unknown layer type: {path}.type = {kind!r} (known: {', '.join(MIXERS)})")
            mlp, fp = _obj(layer, "mlp", path + ".", optional=True), path + ".mlp"
            ff = None
            if mlp is not None:
                ff_kind = _at(fp, read_key, mlp, "kind", str, "dense")
                if ff_kind == "dense":
                    ff = DenseFFConfig(ff=_at(fp, read_key, mlp, "ff", int))
                elif ff_kind == "moe":
                    router, expert = _obj(mlp, "router", fp + "."), _obj(mlp, "expert", fp + ".")
                    groups = _obj(router, "groups", fp + ".router.", optional=True)
                    shared = _obj(mlp, "shared", fp + ".", optional=True)
                    ff = MoEFFConfig(
                        experts=_at(fp + ".router", read_key, router, "experts", int),
                        top=_at(fp + ".router", read_key, router, "top", int),
                        ff=_at(fp + ".expert", read_key, expert, "ff", int),
                        groups=1 if groups is None else _at(fp + ".router.groups", read_key, groups, "count", int),
                        keep=1 if groups is None else _at(fp + ".router.groups", read_key, groups, "keep", int),
                        shared_ff=0 if shared is None else _at(fp + ".shared", read_key, shared, "ff", int))
                else:
                    raise ConfigError(f"unknown feed-forward kind: {fp}.kind = {ff_kind!r} "
                                      f"(known: {', '.join(FEED_FORWARDS)})")
            layers.append(FitatarLayer(kind, mixer, ff))
        known = {"architecture", "architectures", "vocab", "width", "embedding", "logit_softcap", "norm", "layers",
                 "eos_token_id"}
        cfg = cls(
            architecture="Fitatar",
            vocab=read_key(d, "vocab", int), width=read_key(d, "width", int),
            embedding_scale=_at("embedding", read_key, emb, "scale", float, 1.0),
            logit_softcap=read_key(d, "logit_softcap", float, 0.0),
            norm_eps=_at("norm", read_key, norm, "eps", float),
            layers=tuple(layers),
            eos_token_ids=token_id_list(d.get("eos_token_id"), "eos_token_id"),
            extra={k: v for k, v in d.items() if k not in known})
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if self.norm_eps < 0 or self.logit_softcap < 0:
            raise ConfigError("norm.eps and logit_softcap must not be negative")
        for i, layer in enumerate(self.layers):
            m, path = layer.mixer, f"layers[{i}].mixer"
            keys = ("heads", "dim", "vdim", "kv_rank", "q_rank") if isinstance(m, LatentAttentionConfig) \
                else ("heads", "kv_heads", "dim", "vdim")
            for key in keys:
                if getattr(m, key) <= 0:
                    raise ConfigError(f"{path}.{key} must be positive")
            r = m.rot
            room = m.rot_dim if isinstance(m, LatentAttentionConfig) else m.dim
            if r.dims < 0 or r.dims % 2 or r.dims > room:
                raise ConfigError(f"{path}.rot.dims = {r.dims} must be even and at most {room}")
            if r.dims and r.base <= 0:
                raise ConfigError(f"{path}.rot.base must be positive")
            if r.factor < 0 or (r.factor and isinstance(m, LatentAttentionConfig) and (r.original <= 0 or r.fast <= 0 or r.slow <= 0)):
                raise ConfigError(f"{path}.rot.scaling: factor, original, fast and slow must be positive")
            if isinstance(m, LatentAttentionConfig):
                if m.rot_dim < 0:
                    raise ConfigError(f"{path}.rot_dim must not be negative")
                if m.kv_from is not None:
                    src = self.layers[m.kv_from].mixer if 0 <= m.kv_from < i else None
                    if not isinstance(src, LatentAttentionConfig) or src.kv_from is not None:
                        raise ConfigError(f"{path}.kv_from = {m.kv_from} must name an earlier latent_attention layer "
                                          f"that keeps a latent of its own")
                    if (src.kv_rank, src.rot_dim, src.rot) != (m.kv_rank, m.rot_dim, m.rot):
                        raise ConfigError(f"{path}: kv_rank, rot_dim and rot differ from those of layer {m.kv_from}, "
                                          f"whose latent it reads")
            elif m.heads % m.kv_heads:
                raise ConfigError(f"{path}: {m.heads} heads are not a multiple of {m.kv_heads} kv_heads")
            f, fp = layer.mlp, f"layers[{i}].mlp"
            if isinstance(f, DenseFFConfig) and f.ff <= 0:
                raise ConfigError(f"{fp}.ff must be positive")
            if isinstance(f, MoEFFConfig):
                if f.experts <= 0 or not 0 < f.top <= f.experts:
                    raise ConfigError(f"{fp}.router: top = {f.top} must be between 1 and experts = {f.experts}")
                if f.ff <= 0 or f.shared_ff < 0:
                    raise ConfigError(f"{fp}: the experts' ff must be positive")
                if f.groups <= 0 or f.experts % f.groups or not 0 < f.keep <= f.groups:
                    raise ConfigError(f"{fp}.router.groups: keep = {f.keep} of count = {f.groups} groups do not fit "
                                      f"{f.experts} experts")
                if f.keep * (f.experts // f.groups) < f.top:
                    raise ConfigError(f"{fp}.router.groups: {f.keep} groups of {f.experts // f.groups} experts hold fewer "
                                      f"than top = {f.top}")

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            m, f = layer.mixer, layer.mlp
            if isinstance(m, LatentAttentionConfig):
                mx = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                      "q_rank": m.q_rank, "scale": m.scale, "rot": _rotation_dict(m.rot, True)}
                if m.kv_from is not None:
                    mx["kv_from"] = m.kv_from
            else:
                mx = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                      "rot": _rotation_dict(m.rot, False)}
            if f is None:
                mlp = None
            elif isinstance(f, DenseFFConfig):
                mlp = {"kind": "dense", "ff": f.ff}
            else:
                mlp = {"kind": "moe", "router": {"experts": f.experts, "top": f.top}, "expert": {"ff": f.ff}}
                if f.groups > 1:
                    mlp["router"]["groups"] = {"count": f.groups, "keep": f.keep}
                if f.shared_ff:
                    mlp["shared"] = {"ff": f.shared_ff}
            layers.append({"type": layer.type, "mixer": mx, "mlp": mlp})
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
             "embedding": {"scale": self.embedding_scale}, "logit_softcap": self.logit_softcap,
             "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        d.update(self.extra)
        return d
