"""Kapanex: from its typed configuration to a ``ModelSpec``.

A decoder whose blocks run their two branches side by side: with n1, n2 two layer norms (a
weight, no bias) of the same x,  x <- x + (mixer(n1(x)) + ff(n2(x))).  Embedding: scale *
E[token].  A layer's mixer is either attention over a sliding window (rotation of a part of every
head, then an RMS norm without weights of q and k per head, grouped heads, value heads of a size
of their own) or the gated delta rule (a recurrent state a head, short convolutions in front).
Its feed-forward, if it has one, is a set of routed experts (sigmoid scores, the best groups of
neighbouring experts first, then the best experts of those) beside a gated shared expert.  A
layer may run with another layer's weights and keeps a cache or state of its own all the same.
After the blocks: layer norm and the head (a matrix of its own).

Tensor names: ``embed``, ``final.norm``, ``head``, and for layer i ``l<i>.norm1|norm2``,
``l<i>.mix.q|k|v|o`` (a delta mixer also ``.q.conv|.k.conv|.v.conv``, ``.b``, ``.a``, ``.A_log``,
``.dt_bias``, ``.g``, ``.norm``), ``l<i>.mlp.router``, ``l<i>.mlp.e<j>.gate|up|down``,
``l<i>.mlp.shared.gate|up|down|sg``.
"""
from __future__ import annotations

from ..config.base import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..config.kapanex import ARCHITECTURE, NO_POSITION_LIMIT, KapanexConfig
from ..registry import register_architecture


def kapanex_spec(cfg: KapanexConfig) -> ModelSpec:
    limit = cfg.max_positions or NO_POSITION_LIMIT

    def layer_norm(name: str) -> PartSpec:
        return PartSpec("layernorm", {"size": cfg.width, "eps": cfg.norm_eps}, {"weight": name})

    blocks, block_of = [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p = f"l{i}."
        m = layer.mixer
        if layer.kind == "attention":
            head_norm = PartSpec("rmsnorm", {"size": m.dim, "eps": cfg.norm_eps})        # no weights
            mixer = PartSpec(
                "paged_attention",
                {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                 "value_dim": m.vdim, "scale": m.scale, "window": m.window, "norm_after_rotation": True},
                {"q": p + "mix.q", "k": p + "mix.k", "v": p + "mix.v", "o": p + "mix.o"},
                {"position": PartSpec("rope_neox", {"head_dim": m.dim, "rotary_dim": m.rot_dims,
                                                    "theta": m.rot_base, "max_positions": limit}),
                 "q_norm": head_norm, "k_norm": head_norm})
        else:
            mixer = PartSpec(
                "gated_delta",
                {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
                 "value_dim": m.vdim, "conv_taps": m.conv, "norm_eps": cfg.norm_eps},
                {"q": p + "mix.q", "k": p + "mix.k", "v": p + "mix.v", "q_conv": p + "mix.q.conv",
                 "k_conv": p + "mix.k.conv", "v_conv": p + "mix.v.conv", "b": p + "mix.b", "a": p + "mix.a",
                 "a_log": p + "mix.A_log", "dt_bias": p + "mix.dt_bias", "gate": p + "mix.g",
                 "norm": p + "mix.norm", "o": p + "mix.o"})
        ffn, norms = None, {"mixer": layer_norm(p + "norm1")}
        if layer.mlp is not None:
            f = layer.mlp
            names = {"router": p + "mlp.router", "experts": p + "mlp.e{}."}
            if f.shared_ff is not None:
                names.update({"shared_gate": p + "mlp.shared.gate", "shared_up": p + "mlp.shared.up",
                              "shared_down": p + "mlp.shared.down", "shared_scale": p + "mlp.shared.sg"})
            ffn = PartSpec("routed_experts",
                           {"hidden_size": cfg.width, "experts": f.experts, "top": f.top, "groups": f.groups,
                            "keep": f.keep, "scale": f.scale, "intermediate_size": f.ff,
                            "shared_intermediate_size": f.shared_ff}, names)
            norms["ffn"] = layer_norm(p + "norm2")
        block_of[i] = len(blocks)
        blocks.append(BlockSpec("parallel_prenorm", mixer, ffn, norms))
    schedule = []
    for i, layer in enumerate(cfg.layers):
        owner = i if layer.weights_of is None else layer.weights_of
        schedule.append(LayerCall(block=block_of[owner], cache=i if layer.kind == "attention" else -1))
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=limit,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                               "scale": cfg.embedding_scale}, {"weight": "embed"}),
        blocks=tuple(blocks),
        schedule=tuple(schedule),
        final_norm=layer_norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied": False},
                      {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids)


register_architecture(ARCHITECTURE, KapanexConfig.from_dict, kapanex_spec)
