"""Sinepel: from its typed configuration to a ``ModelSpec``.

A decoder of hyper-connected pre-norm blocks.  Embedding: scale * E[token] plus a
learned vector for the position.  Every block: RMS norm, token shift, an attention
whose queries and keys pass a short convolution and whose values are its keys, with
a temperature and a log-distance penalty a head, over the positions of the row's own
block of ``mask.size`` positions; then (unless the layer has none) RMS norm and a
dense feed-forward with relu(z)^2.  After the blocks the streams are added up, normed,
multiplied by the head and soft-capped.

Tensor names: ``embed``, ``pos``, ``final.norm``, ``head``, and for layer i
``l<i>.norm1|norm2|shift``, ``l<i>.hc1|hc2.in|out|mix``, ``l<i>.mix.q|k`` (with
``.b`` bias and ``.conv``), ``l<i>.mix.o|temp|r1|r2``, ``l<i>.mlp.up|down``.
"""
from __future__ import annotations

from ..config.base import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..config.sinepel import ARCHITECTURE, SinepelConfig
from ..registry import register_architecture


def sinepel_spec(cfg: SinepelConfig) -> ModelSpec:
    def rms(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps}, {"weight": name})

    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer.mixer
        mixer = PartSpec(
            "conv_key_attention",
            {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
             "scale": m.scale, "conv_taps": m.conv, "mask": ("chunk", m.chunk)},
            {"q": p + "mix.q", "q_bias": p + "mix.q.b", "q_conv": p + "mix.q.conv",
             "k": p + "mix.k", "k_bias": p + "mix.k.b", "k_conv": p + "mix.k.conv",
             "o": p + "mix.o", "temp": p + "mix.temp", "r1": p + "mix.r1", "r2": p + "mix.r2"})
        ffn, norms = None, {"mixer": rms(p + "norm1")}
        names = {"in1": p + "hc1.in", "out1": p + "hc1.out", "mix1": p + "hc1.mix"}
        if layer.ff is not None:
            ffn = PartSpec("dense_act", {"hidden_size": cfg.width, "intermediate_size": layer.ff,
                                         "activation": "relu2"},
                           {"up": p + "mlp.up", "down": p + "mlp.down"})
            norms["ffn"] = rms(p + "norm2")
            names.update({"in2": p + "hc2.in", "out2": p + "hc2.out", "mix2": p + "hc2.mix"})
        blocks.append(BlockSpec(
            "hyper_prenorm", mixer, ffn, norms,
            params={"streams": cfg.streams, "width": cfg.width}, names=names,
            parts={"shift": PartSpec("token_shift", {"size": cfg.width}, {"weight": p + "shift"})}))
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=cfg.max_positions,
        embedding=PartSpec("token_embedding",
                           {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "scale": cfg.embedding_scale,
                            "max_positions": cfg.max_positions},
                           {"weight": "embed", "positions": "pos"}),
        blocks=tuple(blocks),
        schedule=tuple(LayerCall(block=i, cache=i, writes_cache=True) for i in range(len(cfg.layers))),
        final_norm=rms("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied": False,
                                      "softcap": cfg.logit_softcap}, {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids)


register_architecture(ARCHITECTURE, SinepelConfig.from_dict, sinepel_spec)
