"""Typed configuration of the Nalasun decoder, read from config.json.

The file lists the layers one by one; each names its mixer (``type``), the mixer's sizes and
constants (``mixer``) and its feed-forward (``mlp``, or null for a layer without one):

    {"architecture": "Nalasun", "vocab": V, "width": D, "max_positions": P, "norm": {"eps": e},
     "canon": {"taps": t},
     "layers": [{"type": "mamba2",
                 "mixer": {"heads": H, "vdim": P, "state": N, "groups": G, "conv": taps, "norm_groups": g},
                 "mlp": {"kind": "moe", "router": {"experts": E, "top": k, "scale": s}, "expert": {"ff": F},
                         "shared": {"ff": F2}}},
                {"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": dk, "vdim": dk, "scale": c,
                           "q_temp": {"coef": a, "every": n}}, "mlp": ...},
                {"type": "channel_delta",
                 "mixer": {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "conv": taps}, "mlp": null}, ...]}

Every size and constant of the model is read here and handed to the parts as a parameter.  A key
that is missing or of the wrong kind is reported by its path (``layers[3].mixer.heads``).  The
inner sizes of the delta rule's two-step projections are not in the file (its tensors tell them);
``decay_rank`` and ``gate_rank`` may name them for models of seeded random weights.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, read_key, token_id_list
from .tatelorn import _at, _obj

MIXERS = ("mamba2", "channel_delta", "attention")
FEED_FORWARDS = ("moe",)


@dataclass(frozen=True)
class Mamba2Config:
    heads: int
    vdim: int           # channels per head
    state: int          # rows of a head's state matrix
    groups: int         # B and C are shared by the heads of a group
    conv: int           # taps of the short convolution
    norm_groups: int    # parts of the gated output that are normed on their own


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    kv_heads: int       # heads of queries and keys
    dim: int            # query/key numbers per head
    vdim: int           # value numbers per head
    conv: int           # taps of the short convolutions
    decay_rank: int = -1    # -1: what the file's tensors have
    gate_rank: int = -1


@dataclass(frozen=True)
class SharedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int            # query/key numbers per head
    vdim: int           # value numbers per head (the values are the keys: equal to dim)
    scale: float        # multiplies q . k
    temp_coef: float    # q times 1 + coef ln(floor((p + 1) / every) + 1)
    temp_every: int


@dataclass(frozen=True)
class MoEConfig:
    experts: int
    top: int
    scale: float        # multiplies the chosen experts' scores
    ff: int
    shared_ff: int = 0  # 0: no expert that every token takes
    kind: str = "moe"


@dataclass(frozen=True)
class NalasunLayer:
    type: str
    mixer: object               # Mamba2Config, ChannelDeltaConfig or SharedAttentionConfig
    mlp: Optional[MoEConfig]


def _mixer(kind: str, mx: Mapping, mp: str):
    def key(name, typ, *default):
        return _at(mp, read_key, mx, name, typ, *default)
    if kind == "mamba2":
        return Mamba2Config(heads=key("heads", int), vdim=key("vdim", int), state=key("state", int),
                            groups=key("groups", int, 1), conv=key("conv", int), norm_groups=key("norm_groups", int, 1))
    heads, dim = key("heads", int), key("dim", int)
    if kind == "channel_delta":
        return ChannelDeltaConfig(heads=heads, kv_heads=key("kv_heads", int, heads), dim=dim, vdim=key("vdim", int, dim),
                                  conv=key("conv", int), decay_rank=key("decay_rank", int, -1),
                                  gate_rank=key("gate_rank", int, -1))
    temp = _obj(mx, "q_temp", mp + ".", optional=True)
    return SharedAttentionConfig(
        heads=heads, kv_heads=key("kv_heads", int, heads), dim=dim, vdim=key("vdim", int, dim), scale=key("scale", float),
        temp_coef=0.0 if temp is None else _at(mp + ".q_temp", read_key, temp, "coef", float),
        temp_every=1 if temp is None else _at(mp + ".q_temp", read_key, temp, "every", int))


@dataclass(frozen=True)
class NalasunConfig:
    architecture: str
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    canon_taps: int
    layers: Tuple[NalasunLayer, ...]
    eos_token_ids: Tuple[int, ...] = ()
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "NalasunConfig":
        norm = _obj(d, "norm", "")
        canon = _obj(d, "canon", "")
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
            mixer = _mixer(kind, _obj(layer, "mixer", path + "."), path + ".mixer")
            mlp, fp = _obj(layer, "mlp", path + ".", optional=True), path + ".mlp"
            ff = None
            if mlp is not None:
                ff_kind = _at(fp, read_key, mlp, "kind", str, "moe")
                if ff_kind != "moe":
                    raise ConfigError(f"unknown feed-forward kind: {fp}.kind = {ff_kind!r} (known: {', '.join(FEED_FORWARDS)})")
                router, expert = _obj(mlp, "router", fp + "."), _obj(mlp, "expert", fp + ".")
                shared = _obj(mlp, "shared", fp + ".", optional=True)
                ff = MoEConfig(experts=_at(fp + ".router", read_key, router, "experts", int),
                               top=_at(fp + ".router", read_key, router, "top", int),
                               scale=_at(fp + ".router", read_key, router, "scale", float, 1.0),
                               ff=_at(fp + ".expert", read_key, expert, "ff", int),
                               shared_ff=0 if shared is None else _at(fp + ".shared", read_key, shared, "ff", int))
            layers.append(NalasunLayer(kind, mixer, ff))
        known = {"architecture", "architectures", "vocab", "width", "max_positions", "norm", "canon", "layers", "eos_token_id"}
        cfg = cls(architecture="Nalasun", vocab=read_key(d, "vocab", int), width=read_key(d, "width", int),
                  max_positions=read_key(d, "max_positions", int), norm_eps=_at("norm", read_key, norm, "eps", float),
                  canon_taps=_at("canon", read_key, canon, "taps", int), layers=tuple(layers),
                  eos_token_ids=token_id_list(d.get("eos_token_id"), "eos_token_id"),
                  extra={k: v for k, v in d.items() if k not in known})
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.max_positions <= 0:
            raise ConfigError("vocab, width and max_positions must be positive")
        if self.norm_eps < 0:
            raise ConfigError("norm.eps must not be negative")
        if self.canon_taps < 2:
            raise ConfigError("canon.taps must be at least 2")
        for i, layer in enumerate(self.layers):
            m, path = layer.mixer, f"layers[{i}].mixer"
            sizes = {"mamba2": ("heads", "vdim", "state", "groups", "norm_groups"),
                     "channel_delta": ("heads", "kv_heads", "dim", "vdim"),
                     "attention": ("heads", "kv_heads", "dim", "vdim", "temp_every")}[layer.type]
            for key in sizes:
                if getattr(m, key) <= 0:
                    raise ConfigError(f"{path}.{key} must be positive")
            if layer.type == "mamba2":
                if m.heads % m.groups:
                    raise ConfigError(f"{path}: {m.heads} heads are not a multiple of {m.groups} groups")
                if (m.heads * m.vdim) % m.norm_groups:
                    raise ConfigError(f"{path}: {m.norm_groups} norm_groups do not divide heads * vdim = {m.heads * m.vdim}")
            else:
                if m.heads % m.kv_heads:
                    raise ConfigError(f"{path}: {m.heads} heads are not a multiple of {m.kv_heads} kv_heads")
            if layer.type != "attention" and m.conv < 2:
                raise ConfigError(f"{path}.conv must be at least 2")
            if layer.type == "attention" and m.vdim != m.dim:
                raise ConfigError(f"{path}: the values are the keys, so vdim = {m.vdim} must equal dim = {m.dim}")
            f, fp = layer.mlp, f"layers[{i}].mlp"
            if f is not None:
                if f.experts <= 0 or not 0 < f.top <= f.experts:
                    raise ConfigError(f"{fp}.router: top = {f.top} must be between 1 and experts = {f.experts}")
                if f.ff <= 0 or f.shared_ff < 0:
                    raise ConfigError(f"{fp}: the experts' ff must be positive")

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            m, f = layer.mixer, layer.mlp
            if layer.type == "mamba2":
                mx = {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "conv": m.conv,
                      "norm_groups": m.norm_groups}
            elif layer.type == "channel_delta":
                mx = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
                if m.decay_rank > 0:
                    mx["decay_rank"] = m.decay_rank
                if m.gate_rank > 0:
                    mx["gate_rank"] = m.gate_rank
            else:
                mx = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                      "q_temp": {"coef": m.temp_coef, "every": m.temp_every}}
            mlp = None
            if f is not None:
                mlp = {"kind": "moe", "router": {"experts": f.experts, "top": f.top, "scale": f.scale}, "expert": {"ff": f.ff},
                       "shared": {"ff": f.shared_ff} if f.shared_ff else None}
            layers.append({"type": layer.type, "mixer": mx, "mlp": mlp})
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
             "norm": {"eps": self.norm_eps}, "canon": {"taps": self.canon_taps}, "layers": layers}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        d.update(self.extra)
        return d
