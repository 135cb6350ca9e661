"""Typed configuration of the Kapanex decoder, read from its config.json.

Keys: ``architecture`` ("Kapanex"), ``vocab``, ``width``, ``embedding.scale``, ``norm.eps``,
``max_positions`` (optional: the design itself sets no limit) and ``layers``: a list with one entry
a layer, ``{"type": "attention" | "delta", "mixer": {...}, "mlp": {...} or null}``, and optionally
``"weights_of": j``: the layer has no tensors of its own and runs with those of layer j (of equal
sizes), keeping a cache or state of its own.

An attention mixer gives ``heads``, ``kv_heads``, ``dim`` (of a query and a key head), ``vdim`` (of
a value head), ``scale`` (of the scores), ``rot.dims`` and ``rot.base`` (the rotated part of a head
and the base of its frequencies) and ``mask.size`` (a row sees itself and the size - 1 before it).
A delta mixer gives ``heads`` (value heads), ``kv_heads`` (query/key heads), ``dim``, ``vdim`` and
``conv`` (taps of the short convolution over time).  A feed-forward gives ``kind`` ("moe"),
``expert.ff``, ``router.experts|top|scale``, ``router.groups.count|keep`` and optionally ``shared.ff``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple, Union

from .base import ConfigError, JsonReader

ARCHITECTURE = "Kapanex"
NO_POSITION_LIMIT = 1 << 20          # what a config.json without ``max_positions`` is taken to allow


@dataclass(frozen=True)
class KapanexAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    rot_dims: int
    rot_base: float

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                "scale": self.scale, "mask": {"size": self.window},
                "rot": {"dims": self.rot_dims, "base": self.rot_base}}


@dataclass(frozen=True)
class KapanexDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class KapanexExperts:
    experts: int
    top: int
    groups: int
    keep: int
    scale: float
    ff: int
    shared_ff: Optional[int]          # None: no shared expert

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff},
                               "router": {"experts": self.experts, "top": self.top, "scale": self.scale,
                                          "groups": {"count": self.groups, "keep": self.keep}}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class KapanexLayer:
    kind: str                                         # "attention" or "delta"
    mixer: Union[KapanexAttention, KapanexDelta]
    mlp: Optional[KapanexExperts]
    weights_of: Optional[int] = None

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"type": self.kind, "mixer": self.mixer.to_dict(),
                               "mlp": None if self.mlp is None else self.mlp.to_dict()}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out


def _attention(m: JsonReader, where: str) -> KapanexAttention:
    heads = m.integer("heads", minimum=1)
    kv_heads = m.integer("kv_heads", heads, minimum=1)
    dim = m.integer("dim", minimum=1)
    vdim = m.integer("vdim", dim, minimum=1)
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads {heads} must be a multiple of kv_heads {kv_heads}")
    mask = JsonReader(m.raw("mask") or {}, where + ".mask")
    rot = JsonReader(m.raw("rot") or {}, where + ".rot")
    dims = rot.integer("dims", minimum=2)
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}: rot.dims {dims} must be even and at most dim {dim}")
    return KapanexAttention(heads, kv_heads, dim, vdim, m.number("scale"), mask.integer("size", minimum=1),
                            dims, rot.number("base"))


def _delta(m: JsonReader, where: str) -> KapanexDelta:
    heads = m.integer("heads", minimum=1)
    kv_heads = m.integer("kv_heads", heads, minimum=1)
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads {heads} must be a multiple of kv_heads {kv_heads}")
    dim = m.integer("dim", minimum=1)
    return KapanexDelta(heads, kv_heads, dim, m.integer("vdim", dim, minimum=1), m.integer("conv", minimum=1))


def _experts(f: JsonReader, where: str) -> KapanexExperts:
    kind = f.string("kind")
    if kind != "moe":
        raise ConfigError(f"{where}: feed-forward kind '{kind}' is not known; known: moe")
    r = JsonReader(f.raw("router") or {}, where + ".router")
    g = JsonReader(r.raw("groups") or {}, where + ".router.groups")
    experts = r.integer("experts", minimum=1)
    top = r.integer("top", minimum=1)
    groups = g.integer("count", 1, minimum=1)
    keep = g.integer("keep", groups, minimum=1)
    if experts % groups:
        raise ConfigError(f"{where}: {experts} experts do not form {groups} equal groups")
    if keep > groups or keep * (experts // groups) < top:
        raise ConfigError(f"{where}: {keep} of {groups} groups of {experts // groups} cannot give {top} experts")
    ff = JsonReader(f.raw("expert") or {}, where + ".expert").integer("ff", minimum=1)
    shared = f.raw("shared")
    shared_ff = None if shared is None else JsonReader(shared, where + ".shared").integer("ff", minimum=1)
    return KapanexExperts(experts, top, groups, keep, r.number("scale", 1.0), ff, shared_ff)


@dataclass(frozen=True)
class KapanexConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[KapanexLayer, ...]
    max_positions: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()

    @staticmethod
    def from_dict(data: Dict[str, Any], origin: str = "config.json") -> "KapanexConfig":
        r = JsonReader(data, origin)
        name = r.string("architecture")
        if name != ARCHITECTURE:
            raise ConfigError(f"{origin}: architecture '{name}' is not '{ARCHITECTURE}'")
        vocab = r.integer("vocab", minimum=1)
        width = r.integer("width", minimum=1)
        scale = JsonReader(r.raw("embedding") or {}, origin + ": embedding").number("scale", 1.0)
        eps = JsonReader(r.raw("norm") or {}, origin + ": norm").number("eps")
        if eps <= 0.0:
            raise ConfigError(f"{origin}: norm.eps must be positive")
        raw_layers = r.raw("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError(f"{origin}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            where = f"{origin}: layers[{i}]"
            lr = JsonReader(entry, where)
            kind = lr.string("type")
            m = JsonReader(lr.raw("mixer") or {}, where + ".mixer")
            if kind == "attention":
                mixer = _attention(m, where + ".mixer")
            elif kind == "delta":
                mixer = _delta(m, where + ".mixer")
            else:
                raise ConfigError(f"{where}: layer type '{kind}' is not known; known: attention, delta")
            mlp = lr.raw("mlp")
            mlp = None if mlp is None else _experts(JsonReader(mlp, where + ".mlp"), where + ".mlp")
            of = lr.integer("weights_of", None)
            layers.append(KapanexLayer(kind, mixer, mlp, of))
        for i, layer in enumerate(layers):
            of, hops = layer.weights_of, 0
            while of is not None:                       # (a layer may name one that itself names another)
                if not 0 <= of < len(layers) or of == i or hops > len(layers):
                    raise ConfigError(f"{origin}: layers[{i}]: weights_of must name another layer with tensors of its own")
                owner = layers[of]
                if owner.weights_of is None:
                    break
                of, hops = owner.weights_of, hops + 1
            if of is not None:
                if (owner.kind, owner.mixer, owner.mlp) != (layer.kind, layer.mixer, layer.mlp):
                    raise ConfigError(f"{origin}: layers[{i}] runs with the weights of layer {of} but has other sizes")
                layers[i] = KapanexLayer(layer.kind, layer.mixer, layer.mlp, of)
        return KapanexConfig(vocab=vocab, width=width, embedding_scale=scale, norm_eps=eps, layers=tuple(layers),
                             max_positions=r.integer("max_positions", None, minimum=1),
                             eos_token_ids=tuple(r.int_list("eos_token_id", [])))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json this configuration is read back from."""
        out: Dict[str, Any] = {
            "architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width,
            "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.max_positions is not None:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
