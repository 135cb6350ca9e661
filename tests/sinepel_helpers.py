"""Shared by the Sinepel tests: small configurations that differ in every size and
option, weights drawn so that every mechanism matters, and model folders of them."""
from __future__ import annotations

import json
import os
from typing import Dict, List

import numpy as np
import torch


def _layer(heads, kv_heads, dim, conv, chunk, ff, scale=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "conv": conv,
                      "scale": float(dim ** -0.5 if scale is None else scale), "mask": {"size": chunk}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _config(vocab, width, streams, layers, max_positions=256, emb_scale=2.5, eps=1e-5, cap=20.0):
    return {"architecture": "Sinepel", "vocab": vocab, "width": width, "max_positions": max_positions,
            "streams": streams, "embedding": {"scale": emb_scale}, "norm": {"eps": eps},
            "logit_softcap": cap, "layers": layers}


# name -> (config.json, page size of the engine in its tests, seed)
SMALL = {
    # two streams; layers of different sizes; a block of positions that is no multiple of the page;
    # the second layer has no feed-forward
    "P": (_config(200, 64, 2, [_layer(4, 2, 16, 3, 24, 96), _layer(2, 1, 32, 2, 16, None)]), 16, 3),
    # one stream, embedding scale 1, no convolution in the first layer (one tap), as many key heads as
    # query heads, heads of 8 and of 48, a block of 7 positions and one longer than every test sequence
    "Q": (_config(131, 48, 1, [_layer(3, 3, 16, 1, 7, 80), _layer(6, 2, 8, 5, 40, 64), _layer(1, 1, 48, 4, 200, 64, scale=0.2)],
                  emb_scale=1.0, eps=3e-6, cap=8.0), 8, 5),
    # four streams, heads of 64 (the matrix-core kernels), one key head for all query heads
    # three streams, a width that is no multiple of 8, heads of 24 and 20 (no matrix-core attention), eight query
    # heads on one key head, six taps, blocks of 96, 33 and 50 positions
    "T": (_config(257, 100, 3, [_layer(6, 3, 24, 6, 96, 144), _layer(2, 2, 20, 2, 33, None), _layer(8, 1, 16, 3, 50, 72)],
                  emb_scale=0.7, eps=1e-4, cap=30.0), 16, 11),
    "R": (_config(320, 128, 4, [_layer(4, 1, 64, 2, 32, 192), _layer(2, 2, 64, 3, 128, 160)], max_positions=384, cap=12.0), 32, 7),
}


def make_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bfloat16 weights, of a size that makes every mechanism show in the logits: shifts in (0, 1),
    temperatures around 1, positive distance penalties, stream weights near (not at) the identity."""
    g = torch.Generator().manual_seed(seed)
    D, S = cfg["width"], cfg["streams"]

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g) * std + mean

    def uniform(*shape, lo=0.0, hi=1.0):
        return torch.rand(*shape, generator=g) * (hi - lo) + lo

    w = {"embed": normal(cfg["vocab"], D, std=0.5), "pos": normal(cfg["max_positions"], D, std=0.3),
         "final.norm": normal(D, std=0.1, mean=1.0), "head": normal(cfg["vocab"], D, std=D ** -0.5 * 4)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, G, d, taps = m["heads"], m["kv_heads"], m["dim"], m["conv"]
        w[p + "norm1"] = normal(D, std=0.1, mean=1.0)
        w[p + "shift"] = uniform(D, lo=0.05, hi=0.9)
        w[p + "mix.q"] = normal(H * d, D, std=D ** -0.5 * 1.5)
        w[p + "mix.q.b"] = normal(H * d, std=0.2)
        w[p + "mix.k"] = normal(G * d, D, std=D ** -0.5 * 1.5)
        w[p + "mix.k.b"] = normal(G * d, std=0.2)
        w[p + "mix.q.conv"] = normal(H * d, taps, std=0.5)
        w[p + "mix.k.conv"] = normal(G * d, taps, std=0.5)
        w[p + "mix.temp"] = uniform(H, lo=0.6, hi=1.6)
        w[p + "mix.r1"] = uniform(H, lo=0.2, hi=1.5)
        w[p + "mix.r2"] = uniform(H, lo=0.1, hi=2.0)
        w[p + "mix.o"] = normal(D, H * d, std=(H * d) ** -0.5)
        for q in ("hc1", "hc2") if layer["mlp"] is not None else ("hc1",):
            w[p + q + ".in"] = normal(S, std=0.2, mean=1.0 / S)
            w[p + q + ".out"] = normal(S, std=0.2, mean=1.0)
            w[p + q + ".mix"] = torch.eye(S) * 0.8 + normal(S, S, std=0.15)
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            w[p + "norm2"] = normal(D, std=0.1, mean=1.0)
            w[p + "mlp.up"] = normal(ff, D, std=D ** -0.5)
            w[p + "mlp.down"] = normal(D, ff, std=ff ** -0.5)
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


def write_folder(folder: str, cfg: dict, weights: Dict[str, torch.Tensor]) -> str:
    from tiny_llm_infer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(folder, "model.safetensors"), list(weights.items()))
    return folder


def make_folder(folder: str, name: str) -> str:
    cfg, _, seed = SMALL[name]
    return write_folder(folder, cfg, make_weights(cfg, seed))


def plain_logits(folder: str, reqs: Dict[str, List[int]]) -> Dict[str, np.ndarray]:
    import plain_sinepel
    cfg, w = plain_sinepel.read_model(folder)
    return {rid: plain_sinepel.forward(cfg, w, toks).numpy() for rid, toks in reqs.items()}


def plain_greedy(folder: str, prompt: List[int], new_tokens: int) -> List[int]:
    import plain_sinepel
    cfg, w = plain_sinepel.read_model(folder)
    toks = list(prompt)
    for _ in range(new_tokens):
        toks.append(int(plain_sinepel.forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]
