"""A plain, slow implementation of the Kapanex decoder: whole sequences, no cache, no
carried state, one function for each mechanism, float64 arithmetic.  It shares no code with
the engine: it reads config.json as a plain dict and the weights as a name -> tensor dict.

Notation: T tokens of one sequence at positions 0..T-1, width D; attention with H query heads
and G key/value heads, query/key size d and value size e; the delta rule with H value heads of
size e and G query/key heads of size d.
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
        t = torch.frombuffer(bytearray(raw[8 + hlen + b:8 + hlen + e]), dtype=kinds[info["dtype"]]).reshape(info["shape"])
        out[name] = t.to(F64) if t.dtype.is_floating_point else t.clone()
    return out


def read_model(folder):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ------------------------------------------------------------- small parts ---
def silu(z):
    return z / (1.0 + torch.exp(-z))


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * w, no bias."""
    dev = x - x.mean(dim=-1, keepdim=True)
    return dev / torch.sqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * w


def rms_unit(x, eps):
    """x over its root mean square (eps inside the root), no weight."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rotate_part(x, dims, base):
    """x [T, heads, d]: the first ``dims`` elements of every head are turned, element i paired with
    i + dims/2, by the angle position * base^(-2i/dims); the rest passes."""
    T, half = x.shape[0], dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    ang = torch.arange(T, dtype=F64)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def window_weights(q, k, scale, size):
    """softmax over the keys j with 0 <= i - j < size of (q_i . k_j) * scale;  q, k [T, d] -> [T, T]."""
    T = q.shape[0]
    i = torch.arange(T)
    seen = (i[:, None] >= i[None, :]) & (i[:, None] - i[None, :] < size)
    s = (q @ k.T) * scale
    return torch.softmax(s.masked_fill(~seen, -math.inf), dim=-1)


def causal_conv(x, w):
    """x [T, C], w [C, taps] (last column: the current row): y_t = sum_j w[:, j] x_{t - taps + 1 + j}."""
    T, taps = x.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x], dim=0)
    return sum(padded[j:j + T] * w[:, j] for j in range(taps))


def delta_recurrence(q, k, v, beta, decay):
    """One head: q, k [T, d], v [T, e], beta, decay [T].  S starts at zero;
    S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, d, e = q.shape[0], q.shape[1], v.shape[1]
    S = torch.zeros(d, e, dtype=F64)
    out = torch.zeros(T, e, dtype=F64)
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def route(z, top, groups, keep, scale):
    """z [T, E] router logits -> (chosen experts [T, top], their weights [T, top])."""
    T, E = z.shape
    s = torch.sigmoid(z)
    per = E // groups
    ids = torch.zeros(T, top, dtype=torch.long)
    wts = torch.zeros(T, top, dtype=F64)
    for t in range(T):
        score = [sum(sorted(s[t, g * per:(g + 1) * per].tolist(), reverse=True)[:2]) for g in range(groups)]
        kept = sorted(range(groups), key=lambda g: (-score[g], g))[:keep]
        allowed = [e for e in range(E) if e // per in kept]
        chosen = sorted(allowed, key=lambda e: (-float(s[t, e]), e))[:top]
        total = sum(float(s[t, e]) for e in chosen)
        for j, e in enumerate(chosen):
            ids[t, j] = e
            wts[t, j] = s[t, e] / (total + 1e-20) * scale
    return ids, wts


def gated_ff(x, w_gate, w_up, w_down):
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


# ------------------------------------------------------------------ mixers ---
def attention_mixer(w, p, m, h, eps):
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, d)
    k = (h @ w[p + "k"].T).view(T, G, d)
    v = (h @ w[p + "v"].T).view(T, G, e)
    q = rms_unit(rotate_part(q, m["rot"]["dims"], m["rot"]["base"]), eps)
    k = rms_unit(rotate_part(k, m["rot"]["dims"], m["rot"]["base"]), eps)
    out = torch.zeros(T, H, e, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        out[:, a] = window_weights(q[:, a], k[:, g], m["scale"], m["mask"]["size"]) @ v[:, g]
    return out.reshape(T, H * e) @ w[p + "o"].T


def delta_mixer(w, p, m, h, eps):
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, e)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * torch.nn.functional.softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    gate = silu(h @ w[p + "g"].T).view(T, H, e)
    o = torch.stack([delta_recurrence(q[:, a // (H // G)], k[:, a // (H // G)], v[:, a], beta[:, a], decay[:, a])
                     for a in range(H)], dim=1)
    y = rms_unit(o, eps) * w[p + "norm"] * gate
    return y.reshape(T, H * e) @ w[p + "o"].T


def route_margin(z, top, groups, keep):
    """How far each row of z [T, E] is from another choice: the smaller of (a) the gap between the last group kept
    and the first one left out, in units of group score, and (b) the gap in z between the last expert chosen and
    the first one left out among the kept groups, over the spread of the row's logits.  Infinite where there
    is no choice to make."""
    T, E = z.shape
    s = torch.sigmoid(z)
    per = E // groups
    out = torch.full((T,), math.inf, dtype=F64)
    for t in range(T):
        score = [sum(sorted(s[t, g * per:(g + 1) * per].tolist(), reverse=True)[:2]) for g in range(groups)]
        order = sorted(range(groups), key=lambda g: (-score[g], g))
        if keep < groups:
            out[t] = min(float(out[t]), score[order[keep - 1]] - score[order[keep]])
        allowed = sorted((float(z[t, e]) for e in range(E) if e // per in order[:keep]), reverse=True)
        if top < len(allowed):
            out[t] = min(float(out[t]), (allowed[top - 1] - allowed[top]) / max(float(z[t].std()), 1e-9))
    return out


def experts_ff(w, p, f, h, margins=None):
    r = f["router"]
    groups = r.get("groups", {})
    z = h @ w[p + "router"].T
    ids, wts = route(z, r["top"], groups.get("count", 1), groups.get("keep", groups.get("count", 1)), r.get("scale", 1.0))
    if margins is not None:
        margins.append(route_margin(z, r["top"], groups.get("count", 1), groups.get("keep", groups.get("count", 1))))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            q = f"{p}e{int(ids[t, j])}."
            out[t] += wts[t, j] * gated_ff(h[t], w[q + "gate"], w[q + "up"], w[q + "down"])
    if f.get("shared") is not None:
        q = p + "shared."
        out = out + torch.sigmoid(h @ w[q + "sg"].T) * gated_ff(h, w[q + "gate"], w[q + "up"], w[q + "down"])
    return out


# ------------------------------------------------------------------- model ---
def forward(cfg, w, tokens, residuals=None, margins=None):
    """Logits [T, vocab] of one whole sequence (``residuals``: a list that takes x after every layer;
    ``margins``: a list that takes, for every layer with a router, ``route_margin`` of its rows)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)] * cfg.get("embedding", {}).get("scale", 1.0)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{layer.get('weights_of', i)}."
        h = layer_norm(x, w[p + "norm1"], eps)
        mixer = attention_mixer if layer["type"] == "attention" else delta_mixer
        both = mixer(w, p + "mix.", layer["mixer"], h, eps)
        if layer["mlp"] is not None:
            both = both + experts_ff(w, p + "mlp.", layer["mlp"], layer_norm(x, w[p + "norm2"], eps), margins)
        x = x + both
        if residuals is not None:
            residuals.append(x.clone())
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T
