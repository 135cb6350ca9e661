"""A plain, slow implementation of the Sinepel decoder: whole sequences, no
cache, no state, one function for each mechanism, float64 arithmetic.  It
shares no code with the engine: it reads config.json as a plain dict and the
weights as a name -> tensor dict.

Notation: T tokens of one sequence at positions 0..T-1, width D, S residual
streams, H query heads and G key heads of size d.
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch

F64 = torch.float64


# ---------------------------------------------------------------- weights ----
def read_safetensors(path):
    kinds = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "I32": torch.int32}
    with open(path, "rb") as fh:
        raw = fh.read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        data = bytearray(raw[8 + hlen + b:8 + hlen + e])
        t = torch.frombuffer(data, dtype=kinds[info["dtype"]]).reshape(info["shape"])
        out[name] = t.to(F64) if t.dtype.is_floating_point else t.clone()
    return out


def read_model(folder):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ------------------------------------------------------------- mechanisms ----
def embed(table, positions_table, scale, tokens):
    """x_p = scale * E[token_p] + P[p]."""
    idx = torch.as_tensor(tokens, dtype=torch.long)
    return table[idx] * scale + positions_table[:len(tokens)]


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def token_shift(h, mu):
    """h_p + (h_{p-1} - h_p) * mu, with h_{-1} = 0; h_{p-1} is taken before the replacement."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (prev - h) * mu


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_p = sum_j w[:, j] * u_{p - taps + 1 + j}, zeros before position 0."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for p in range(T):
        for j in range(taps):
            src = p - taps + 1 + j
            if src >= 0:
                y[p] += w[:, j] * u[src]
    return y


def chunk_visible(i, j, size):
    """Position i sees j: not later, and in the same block of ``size`` positions counted from 0."""
    return j <= i and i // size == j // size


def attention_scores(q, k, scale, temp, r1, r2, size):
    """One head.  q, k [T, d].  score_ij = (q_i . k_j) * scale * temp - r1 * ln(1 + r2 * (i - j));
    softmax over the visible j.  Returns the weights [T, T] (zero where not visible)."""
    T = q.shape[0]
    w = torch.zeros(T, T, dtype=q.dtype)
    for i in range(T):
        js = [j for j in range(T) if chunk_visible(i, j, size)]
        s = torch.stack([(q[i] @ k[j]) * scale * temp - r1 * math.log(1.0 + r2 * (i - j)) for j in js])
        e = torch.exp(s - s.max())
        w[i, js] = e / e.sum()
    return w


def attention_mixer(h, W, pre, m):
    """The whole mixer on its (already shifted) input h [T, D].  ``m``: the layer's 'mixer' sizes."""
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = h @ W[pre + "q"].t() + W[pre + "q.b"]
    k = h @ W[pre + "k"].t() + W[pre + "k.b"]
    q = causal_conv(q, W[pre + "q.conv"])
    k = causal_conv(k, W[pre + "k.conv"])
    v = k                                   # the values are the keys as they leave the convolution
    T = h.shape[0]
    out = torch.zeros(T, H * d, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        w = attention_scores(q[:, head * d:(head + 1) * d], k[:, g * d:(g + 1) * d], m["scale"],
                             float(W[pre + "temp"][head]), float(W[pre + "r1"][head]), float(W[pre + "r2"][head]),
                             m["mask"]["size"])
        out[:, head * d:(head + 1) * d] = w @ v[:, g * d:(g + 1) * d]
    return out @ W[pre + "o"].t()


def dense_ff(h, up, down):
    """down( relu(up h)^2 )."""
    a = torch.relu(h @ up.t())
    return (a * a) @ down.t()


def hyper_read(x, w_in):
    """x [S, T, D] -> u = sum_s in[s] x_s."""
    return torch.einsum("s,std->td", w_in, x)


def hyper_write(x, y, w_mix, w_out):
    """x_t <- sum_s mix[s, t] x_s + out[t] y, every stream from the old ones."""
    return torch.einsum("st,sld->tld", w_mix, x) + w_out[:, None, None] * y[None]


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


# ------------------------------------------------------------------ model ----
def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] for one whole sequence.  ``layers_out``: a list that receives the sum of the
    streams after every layer."""
    eps = cfg["norm"]["eps"]
    x0 = embed(W["embed"], W["pos"], cfg["embedding"]["scale"], tokens)
    x = torch.stack([x0] * cfg["streams"])
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        assert layer["type"] == "attention"
        u = hyper_read(x, W[p + "hc1.in"])
        h = token_shift(rms_norm(u, W[p + "norm1"], eps), W[p + "shift"])
        x = hyper_write(x, attention_mixer(h, W, p + "mix.", layer["mixer"]), W[p + "hc1.mix"], W[p + "hc1.out"])
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            u = hyper_read(x, W[p + "hc2.in"])
            y = dense_ff(rms_norm(u, W[p + "norm2"], eps), W[p + "mlp.up"], W[p + "mlp.down"])
            x = hyper_write(x, y, W[p + "hc2.mix"], W[p + "hc2.out"])
        if layers_out is not None:
            layers_out.append(x.sum(dim=0))
    z = rms_norm(x.sum(dim=0), W["final.norm"], eps) @ W["head"].t()
    return soft_cap(z, cfg["logit_softcap"])
