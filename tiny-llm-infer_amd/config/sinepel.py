"""Typed configuration of the Sinepel decoder, read from its config.json.

Keys: ``architecture`` ("Sinepel"), ``vocab``, ``width``, ``max_positions``,
``streams`` (copies of the residual stream that the hyper-connections mix),
``embedding.scale``, ``norm.eps``, ``logit_softcap`` and ``layers``: a list with one
entry a layer, ``{"type": "attention", "mixer": {...}, "mlp": {...} or null}``.  A
mixer gives ``heads``, ``kv_heads``, ``dim`` (of a query and a key head), ``vdim`` (of
a value head: the values are the keys, so it equals ``dim``), ``conv`` (taps of the
short convolution over time on q and k), ``scale`` (of the scores) and
``mask.size`` (positions see each other only inside blocks of that many positions).
A feed-forward gives ``kind`` ("dense") and ``ff``.  Layers may differ in every size.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, JsonReader

ARCHITECTURE = "Sinepel"


@dataclass(frozen=True)
class SinepelMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    scale: float
    chunk: int

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                "conv": self.conv, "scale": self.scale, "mask": {"size": self.chunk}}


@dataclass(frozen=True)
class SinepelLayer:
    mixer: SinepelMixer
    ff: Optional[int]              # None: the layer has no feed-forward

    def to_dict(self) -> Dict[str, Any]:
        return {"type": "attention", "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class SinepelConfig:
    vocab: int
    width: int
    max_positions: int
    streams: int
    embedding_scale: float
    norm_eps: float
    logit_softcap: float
    layers: Tuple[SinepelLayer, ...]
    eos_token_ids: Tuple[int, ...] = ()

    @staticmethod
    def from_dict(data: Dict[str, Any], origin: str = "config.json") -> "SinepelConfig":
        r = JsonReader(data, origin)
        name = r.string("architecture")
        if name != ARCHITECTURE:
            raise ConfigError(f"{origin}: architecture '{name}' is not '{ARCHITECTURE}'")
        vocab = r.integer("vocab", minimum=1)
        width = r.integer("width", minimum=1)
        max_pos = r.integer("max_positions", minimum=1)
        streams = r.integer("streams", minimum=1)
        emb = JsonReader(r.raw("embedding") or {}, origin + ": embedding")
        norm = JsonReader(r.raw("norm") or {}, origin + ": norm")
        scale = emb.number("scale")
        eps = norm.number("eps")
        cap = r.number("logit_softcap")
        if eps <= 0.0:
            raise ConfigError(f"{origin}: norm.eps must be positive")
        if cap <= 0.0:
            raise ConfigError(f"{origin}: logit_softcap must be positive")
        raw_layers = r.raw("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError(f"{origin}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            where = f"{origin}: layers[{i}]"
            lr = JsonReader(entry, where)
            kind = lr.string("type")
            if kind != "attention":
                raise ConfigError(f"{where}: layer type '{kind}' is not known; known: attention")
            m = JsonReader(lr.raw("mixer") or {}, where + ".mixer")
            heads = m.integer("heads", minimum=1)
            kv_heads = m.integer("kv_heads", heads, minimum=1)
            dim = m.integer("dim", minimum=1)
            vdim = m.integer("vdim", dim, minimum=1)
            conv = m.integer("conv", minimum=1)
            mask = JsonReader(m.raw("mask") or {}, where + ".mixer.mask")
            chunk = mask.integer("size", minimum=1)
            if heads % kv_heads:
                raise ConfigError(f"{where}: heads {heads} must be a multiple of kv_heads {kv_heads}")
            if vdim != dim:
                raise ConfigError(f"{where}: the values are the keys, so vdim {vdim} must equal dim {dim}")
            mixer = SinepelMixer(heads, kv_heads, dim, vdim, conv, m.number("scale"), chunk)
            ff = None
            mlp = lr.raw("mlp")
            if mlp is not None:
                f = JsonReader(mlp, where + ".mlp")
                fk = f.string("kind")
                if fk != "dense":
                    raise ConfigError(f"{where}: feed-forward kind '{fk}' is not known; known: dense")
                ff = f.integer("ff", minimum=1)
            layers.append(SinepelLayer(mixer, ff))
        eos = tuple(r.int_list("eos_token_id", []))
        return SinepelConfig(vocab=vocab, width=width, max_positions=max_pos, streams=streams,
                             embedding_scale=scale, norm_eps=eps, logit_softcap=cap,
                             layers=tuple(layers), eos_token_ids=eos)

    def to_dict(self) -> Dict[str, Any]:
        """The config.json this configuration is read back from."""
        out: Dict[str, Any] = {
            "architecture": ARCHITECTURE,
            "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
            "streams": self.streams, "embedding": {"scale": self.embedding_scale},
            "norm": {"eps": self.norm_eps}, "logit_softcap": self.logit_softcap,
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
