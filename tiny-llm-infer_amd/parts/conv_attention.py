"""Attention whose queries and keys pass a short causal convolution over time and
whose values are its keys.

For the rows h_p of one sequence (H query heads, G key heads of size d, query
head a reads key head a // (H / G)):

    q_p = Wq h_p + bq,  k_p = Wk h_p + bk                      (projections with bias)
    q'_p = sum_j cq[:, j] * q_{p - taps + 1 + j}               (per channel, zeros before position 0;
    k'_p = sum_j ck[:, j] * k_{p - taps + 1 + j}                the same for k)
    v_p = k'_p                                                  (no value projection)
    s_ij = (q'_i . k'_j) * scale * temp_a - r1_a * ln(1 + r2_a * (i - j))
    j is visible to i if j <= i and, with ``mask`` ("chunk", n), i // n == j // n
                                  with ("window", n), i - j < n;  None: every j <= i
    out_i = sum_j softmax_j(s_ij) v_j,  then Wo on the heads side by side.

``temp``, ``r1`` and ``r2`` are one number a query head each; any of them may be
left out of ``names`` (a temperature of 1, no penalty).  k' goes into the paged
cache (one record: the values are read from it too).  The last ``taps - 1``
projected rows of q and k, before bias and convolution, are per-request state.
Scores, softmax, the penalty and the convolution's sums are float32.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import PAGE, CacheNeed, CacheRecord, StateNeed
from ..weights.loader import TensorDecl
from .base import BuildEnv, Mixer, StepView, register_part
from .linear import as_matrix, fuse_rows

MASKS = ("chunk", "window")


class ConvKeyAttention(Mixer):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.scale = float(p["scale"])
        self.taps = int(p["conv_taps"])
        mask = p.get("mask")
        self.mask = None if mask is None else (str(mask[0]), int(mask[1]))
        if self.mask is not None and (self.mask[0] not in MASKS or self.mask[1] <= 0):
            raise ValueError(f"mask {mask!r}: one of {', '.join(MASKS)} with a positive size")
        if self.heads % self.kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if self.taps <= 0:
            raise ValueError("conv_taps must be positive")
        self.q_dim = self.heads * self.head_dim
        self.kv_dim = self.kv_heads * self.head_dim

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        qd, kd = self.q_dim, self.kv_dim
        out = [TensorDecl(n["q"], (qd, self.hidden)), TensorDecl(n["q_bias"], (qd,)),
               TensorDecl(n["k"], (kd, self.hidden)), TensorDecl(n["k_bias"], (kd,)),
               TensorDecl(n["q_conv"], (qd, self.taps), f"normal({1.0 / self.taps},0.1)"),
               TensorDecl(n["k_conv"], (kd, self.taps), f"normal({1.0 / self.taps},0.1)"),
               TensorDecl(n["o"], (self.hidden, qd))]
        if "temp" in n:
            out.append(TensorDecl(n["temp"], (self.heads,), "ones_normal"))
        if "r1" in n or "r2" in n:
            out += [TensorDecl(n["r1"], (self.heads,), "abs_normal(0.5,0.2)"),
                    TensorDecl(n["r2"], (self.heads,), "abs_normal(0.5,0.2)")]
        return out

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        env.ops.check_conv_attention_sizes(self.heads, self.kv_heads, self.head_dim, self.taps)

        def f32(*roles):
            return torch.cat([weights[n[r]].to(torch.float32) for r in roles], dim=0).contiguous()
        self.w_qk = fuse_rows([weights[n["q"]], weights[n["k"]]], env)
        self.bias = f32("q_bias", "k_bias")                     # [q_dim + kv_dim]
        self.conv = f32("q_conv", "k_conv").t().contiguous()    # [taps, q_dim + kv_dim]: tap by tap, as the kernels read it
        self.temp = f32("temp") if "temp" in n else None
        self.penalty = (f32("r1"), f32("r2")) if "r1" in n else None
        self.w_o = as_matrix(weights[n["o"]], env)

    def cache_need(self) -> Optional[CacheNeed]:
        kind, size = self.mask if self.mask is not None else (None, None)
        return CacheNeed((CacheRecord("k", (self.kv_heads, PAGE, self.head_dim)),),
                         window=size if kind == "window" else None, chunk=size if kind == "chunk" else None)

    def state_need(self) -> Optional[StateNeed]:
        if self.taps == 1:
            return None
        return StateNeed((self.taps - 1, self.q_dim + self.kv_dim), None)

    def workspace_elems(self, rows: int) -> int:
        return rows * (2 * (self.q_dim + self.kv_dim) + 2 * self.q_dim)

    def forward(self, x: torch.Tensor, step: StepView) -> torch.Tensor:
        ops = self.env.ops
        qk = ops.linear(x, self.w_qk)
        o = ops.conv_key_attention(qk, self.bias, self.conv, step.state, step, step.cache, self.heads,
                                   self.kv_heads, self.head_dim, self.taps, self.scale, self.temp,
                                   self.penalty, self.mask)
        return ops.linear(o, self.w_o, deferred=True)


register_part("mixer", "conv_key_attention", ConvKeyAttention)
