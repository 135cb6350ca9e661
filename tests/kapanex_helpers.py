"""Shared by the Kapanex tests: small configurations that differ in every size and option,
weights drawn so that every mechanism matters, and model folders of them."""
from __future__ import annotations

import json
import os
from typing import Dict, List

import numpy as np
import torch


def _attention(heads, kv_heads, dim, vdim, window, rot, base=10000.0, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": float(dim ** -0.5 if scale is None else scale),
            "mask": {"size": window}, "rot": {"dims": rot, "base": base}}


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _moe(experts, top, groups, keep, ff, shared, scale=1.0):
    out = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": groups, "keep": keep}}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def _layer(kind, mixer, mlp, weights_of=None):
    out = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def _config(vocab, width, layers, emb_scale=4.0, eps=1e-5):
    return {"architecture": "Kapanex", "vocab": vocab, "width": width, "embedding": {"scale": emb_scale},
            "norm": {"eps": eps}, "layers": layers}


_A_DELTA, _A_ATT, _A_MOE = _delta(4, 2, 16, 24, 4), _attention(4, 2, 32, 16, 20, 16), _moe(6, 2, 3, 2, 32, 48, scale=1.5)
_C_ATT, _C_MOE = _attention(6, 1, 24, 40, 100, 8, base=500.0, scale=0.3), _moe(8, 3, 8, 3, 24, 16, scale=2.5)
# name -> (config.json, page size of the engine in its tests, seed)
SMALL = {
    # the recurrent layer first; value heads smaller than key heads in the attention, larger in the delta rule; half of
    # every head turned; a window that is no multiple of the page; layers 2 and 3 run with the weights of 0 and 1
    "A": (_config(160, 64, [_layer("delta", _A_DELTA, _A_MOE), _layer("attention", _A_ATT, _A_MOE),
                            _layer("delta", _A_DELTA, _A_MOE, 0), _layer("attention", _A_ATT, _A_MOE, 1)]), 16, 3),
    # as many key heads as query heads, whole heads turned, a window shorter than a page, one tap (no convolution),
    # one group of experts with one chosen and no shared expert, a layer without feed-forward, embedding scale 1
    "B": (_config(211, 96, [_layer("attention", _attention(2, 2, 16, 16, 7, 16), _moe(4, 1, 1, 1, 40, None)),
                            _layer("delta", _delta(2, 2, 16, 16, 1), None)], emb_scale=1.0, eps=3e-6), 8, 5),
    # a width that is no multiple of 8, value heads larger than key heads and no multiple of 16, six query heads on one
    # key head, a window longer than every test sequence, groups of one expert, a key size of 40, two taps
    "C": (_config(257, 100, [_layer("attention", _C_ATT, _C_MOE), _layer("delta", _delta(3, 1, 40, 20, 2), _C_MOE),
                             _layer("attention", _C_ATT, _C_MOE, 0)], emb_scale=2.0, eps=1e-6), 16, 11),
    # whole heads of 64 turned (the attention kernels that norm, turn and write the cache themselves), four query heads
    # on one key head, key heads of 128 on value heads of 32 in the delta rule, every group of experts kept
    "F": (_config(300, 128, [_layer("delta", _delta(2, 1, 128, 32, 3), _moe(4, 2, 2, 2, 48, 64)),
                             _layer("attention", _attention(4, 1, 64, 64, 40, 64), _moe(4, 2, 2, 2, 48, 64))], emb_scale=3.0), 16, 13),
    # heads of 64 (the matrix-core attention kernels), a delta state of 64 x 64, sixteen experts in four groups
    "R": (_config(320, 128, [_layer("attention", _attention(4, 2, 64, 64, 48, 32, base=50000.0), _moe(16, 4, 4, 2, 64, 128, scale=2.0)),
                             _layer("delta", _delta(4, 2, 64, 64, 4), _moe(16, 4, 4, 2, 64, 128, scale=2.0))]), 32, 7),
}


def make_weights(cfg: dict, seed: int, long_memory: bool = False, clear_routing: bool = False) -> Dict[str, torch.Tensor]:
    """bfloat16 weights of a size that makes every mechanism show in the logits.  ``long_memory``: the delta
    rule's decays lie near 1, so that what a token wrote hundreds of positions back still counts.
    ``clear_routing``: no router ever has a close call, so that rounding in bfloat16 cannot turn one (a row
    that goes to another expert is another computation, and so are the rows behind it).  The last E elements
    of the width are set aside: a token's embedding has one of them set (which one: its id modulo E), no layer
    writes to them, and the routers read nothing else, expert e taking element j with the weight
    3 / E (((p(e) + j) mod E) - (E - 1) / 2) for a permutation p a layer: for every token the experts' logits are E
    different levels, and since a row of the router adds up to 0 for every expert, the layer norm's mean shifts none.
    (The choice among groups is a sum of sigmoids and has close calls all the same: configurations that take
    such weights keep all their groups.)"""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g) * std + mean

    def uniform(*shape, lo=0.0, hi=1.0):
        return torch.rand(*shape, generator=g) * (hi - lo) + lo

    w = {"embed": normal(cfg["vocab"], D, std=0.5), "final.norm": normal(D, std=0.1, mean=1.0),
         "head": normal(cfg["vocab"], D, std=D ** -0.5 * 4)}
    for i, layer in enumerate(cfg["layers"]):
        if "weights_of" in layer:
            continue
        p, m = f"l{i}.", layer["mixer"]
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        w[p + "norm1"] = normal(D, std=0.1, mean=1.0)
        if layer["type"] == "attention":
            w[p + "mix.q"] = normal(H * d, D, std=D ** -0.5 * 2)
            w[p + "mix.k"] = normal(G * d, D, std=D ** -0.5 * 2)
            w[p + "mix.v"] = normal(G * e, D, std=D ** -0.5 * 1.5)
            w[p + "mix.o"] = normal(D, H * e, std=(H * e) ** -0.5 * 1.5)
        else:
            taps = m["conv"]
            for r, n in (("q", G * d), ("k", G * d), ("v", H * e)):
                w[p + "mix." + r] = normal(n, D, std=D ** -0.5 * 2)
                w[p + "mix." + r + ".conv"] = normal(n, taps, std=0.6)
            w[p + "mix.b"] = normal(H, D, std=D ** -0.5 * 2)
            w[p + "mix.a"] = normal(H, D, std=D ** -0.5 * 2)
            w[p + "mix.A_log"] = uniform(H, lo=-7.0, hi=-5.0) if long_memory else uniform(H, lo=-2.0, hi=0.5)
            w[p + "mix.dt_bias"] = normal(H, std=0.5)
            w[p + "mix.norm"] = normal(e, std=0.1, mean=1.0)
            w[p + "mix.g"] = normal(H * e, D, std=D ** -0.5 * 2)
            w[p + "mix.o"] = normal(D, H * e, std=(H * e) ** -0.5 * 2)
        f = layer["mlp"]
        if f is not None:
            ff = f["expert"]["ff"]
            w[p + "norm2"] = normal(D, std=0.1, mean=1.0)
            w[p + "mlp.router"] = normal(f["router"]["experts"], D, std=D ** -0.5 * 3)
            for j in range(f["router"]["experts"]):
                w[f"{p}mlp.e{j}.gate"] = normal(ff, D, std=D ** -0.5 * 1.5)
                w[f"{p}mlp.e{j}.up"] = normal(ff, D, std=D ** -0.5 * 1.5)
                w[f"{p}mlp.e{j}.down"] = normal(D, ff, std=ff ** -0.5 * 1.5)
            if f.get("shared") is not None:
                sf = f["shared"]["ff"]
                w[p + "mlp.shared.gate"] = normal(sf, D, std=D ** -0.5 * 1.5)
                w[p + "mlp.shared.up"] = normal(sf, D, std=D ** -0.5 * 1.5)
                w[p + "mlp.shared.down"] = normal(D, sf, std=sf ** -0.5 * 1.5)
                w[p + "mlp.shared.sg"] = normal(1, D, std=D ** -0.5 * 2)
    if clear_routing:
        sizes = {layer["mlp"]["router"]["experts"] for layer in cfg["layers"] if layer["mlp"] is not None}
        assert len(sizes) == 1, "one number of experts in all layers"
        E = sizes.pop()
        w["embed"][:, D - E:] = 0.0
        w["embed"][torch.arange(cfg["vocab"]), D - E + torch.arange(cfg["vocab"]) % E] = 6.0 / cfg["embedding"]["scale"]
        for name in w:
            if name.endswith(("mix.o", ".down")):
                w[name][D - E:] = 0.0                            # nothing is written where the routers read
            if name.endswith("mlp.router"):
                order = torch.randperm(E, generator=g)
                w[name] = torch.zeros(E, D)
                w[name][:, D - E:] = (((order[:, None] + torch.arange(E)[None, :]) % E) - (E - 1) / 2) * (3.0 / E)
                w[name.replace("mlp.router", "norm2")][D - E:] = 1.0
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


def write_folder(folder: str, cfg: dict, weights: Dict[str, torch.Tensor]) -> str:
    from tiny_llm_infer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(folder, "model.safetensors"), list(weights.items()))
    return folder


def make_folder(folder: str, name: str, clear_routing: bool = False) -> str:
    cfg, _, seed = SMALL[name]
    if clear_routing:                     # (all groups are kept: see make_weights)
        cfg = json.loads(json.dumps(cfg))
        for layer in cfg["layers"]:
            if layer["mlp"] is not None:
                layer["mlp"]["router"]["groups"]["keep"] = layer["mlp"]["router"]["groups"]["count"]
    return write_folder(folder, cfg, make_weights(cfg, seed, clear_routing=clear_routing))


def plain_logits(folder: str, reqs: Dict[str, List[int]]) -> Dict[str, np.ndarray]:
    import plain_kapanex
    cfg, w = plain_kapanex.read_model(folder)
    return {rid: plain_kapanex.forward(cfg, w, toks).numpy() for rid, toks in reqs.items()}


def rows_with_a_clear_choice(folder: str, reqs: Dict[str, List[int]], margin: float = 0.05) -> Dict[str, int]:
    """For every request, the number of leading rows whose routers all choose by more than ``margin``
    (``plain_kapanex.route_margin``).  Rounding in bfloat16 can turn a closer call, after which that row and
    the rows behind it (which read it through the mixers) are another computation; a comparison in bfloat16
    takes the rows before."""
    import plain_kapanex
    cfg, w = plain_kapanex.read_model(folder)
    out = {}
    for rid, toks in reqs.items():
        margins = []
        plain_kapanex.forward(cfg, w, toks, margins=margins)
        close = torch.zeros(len(toks), dtype=torch.bool)
        for m in margins:
            close |= m < margin
        out[rid] = int(close.nonzero()[0]) if close.any() else len(toks)
    return out


def plain_greedy(folder: str, prompt: List[int], new_tokens: int) -> List[int]:
    import plain_kapanex
    cfg, w = plain_kapanex.read_model(folder)
    toks = list(prompt)
    for _ in range(new_tokens):
        toks.append(int(plain_kapanex.forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]
