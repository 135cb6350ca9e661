"""The gated delta rule: a recurrent mixer that keeps a matrix of state a head instead of keys
and values a token.

For the rows h_t of one sequence (G key heads of size dk, H value heads of size dv, value head a
reads key head a // (H / G)):

    q, k = Wq h, Wk h  [G dk],   v = Wv h  [H dv]                  (no biases)
    each channel of q, k, v: causal convolution over time with ``taps`` taps (the last tap is
        the current row's; zeros before position 0), then silu
    q <- unit(q) / sqrt(dk),  k <- unit(k)  per head,  unit(x) = x / sqrt(sum(x^2) + 1e-6)
    beta = sigmoid(Wb h)  [H],   decay = exp(-exp(A_log) * softplus(Wa h + dt_bias))  [H]
    per value head:  S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    y = o / sqrt(mean(o^2) + eps) * w * silu(Wg h)   per head (w [dv] is shared by the heads)
    out = Wo y

S [dk, dv] starts at zero and is per-request state in float32, as are the last ``taps - 1`` raw
rows of q, k, v (in the run's storage type: they are the projection's own outputs, so a prompt cut
into portions convolves the same numbers as one that is not).  Everything between the
projections and the output projection is float32; b and a leave their projection in float32.
Nothing is kept in the paged cache.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import StateNeed
from ..weights.loader import TensorDecl
from .base import BuildEnv, Mixer, StepView, register_part
from .linear import as_matrix, fuse_rows


class GatedDeltaRule(Mixer):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.dk = int(p["key_dim"])
        self.dv = int(p["value_dim"])
        self.taps = int(p["conv_taps"])
        self.eps = float(p["norm_eps"])
        if self.heads % self.kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if self.taps <= 0:
            raise ValueError("conv_taps must be positive")
        self.qk_dim = self.kv_heads * self.dk
        self.v_dim = self.heads * self.dv
        self.channels = 2 * self.qk_dim + self.v_dim          # what the convolution runs over

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        conv = f"normal({1.0 / self.taps},0.2)"
        return [TensorDecl(n["q"], (self.qk_dim, self.hidden)), TensorDecl(n["q_conv"], (self.qk_dim, self.taps), conv),
                TensorDecl(n["k"], (self.qk_dim, self.hidden)), TensorDecl(n["k_conv"], (self.qk_dim, self.taps), conv),
                TensorDecl(n["v"], (self.v_dim, self.hidden)), TensorDecl(n["v_conv"], (self.v_dim, self.taps), conv),
                TensorDecl(n["b"], (self.heads, self.hidden)), TensorDecl(n["a_log"], (self.heads,), "normal(0.0,0.5)"),
                TensorDecl(n["norm"], (self.dv,), "ones_normal"), TensorDecl(n["a"], (self.heads, self.hidden)),
                TensorDecl(n["dt_bias"], (self.heads,), "normal(0.0,0.5)"), TensorDecl(n["gate"], (self.v_dim, self.hidden)),
                TensorDecl(n["o"], (self.hidden, self.v_dim))]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        env.ops.check_delta_sizes(self.heads, self.kv_heads, self.dk, self.dv, self.taps)

        def f32(*roles):
            return torch.cat([weights[n[r]].to(torch.float32) for r in roles], dim=0).contiguous()
        # one product for everything that stays in the run's type (q, k, v, then the output gate),
        # one for the two numbers a head that the recurrence wants in float32 (b, then a)
        self.w_main = fuse_rows([weights[n[r]] for r in ("q", "k", "v", "gate")], env)
        self.w_gates = torch.cat([weights[n["b"]].to(env.dtype), weights[n["a"]].to(env.dtype)], dim=0).contiguous()   # few rows: kept row-major
        self.conv = f32("q_conv", "k_conv", "v_conv").t().contiguous()      # [taps, channels]: tap by tap
        self.a_log, self.dt_bias, self.norm = f32("a_log"), f32("dt_bias"), f32("norm")
        self.w_o = as_matrix(weights[n["o"]], env)

    def state_need(self):
        # (the kernel library says in which order, and padded how, it keeps a head's matrix)
        needs = {"S": StateNeed(tuple(self.env.ops.delta_state_shape(self.heads, self.dk, self.dv)), torch.float32)}
        if self.taps > 1:
            needs["conv"] = StateNeed((self.taps - 1, self.channels), None)
        return needs

    def workspace_elems(self, rows: int) -> int:
        # the projections, then q, k, v, o in float32 (two elements of the run's type each at worst)
        return rows * (self.channels + self.v_dim + 2 * (2 * self.qk_dim + 2 * self.v_dim) + self.v_dim)

    def forward(self, x: torch.Tensor, step: StepView):
        ops = self.env.ops
        main = ops.linear(x, self.w_main)
        gates, transposed = ops.small_product(x, self.w_gates)
        states = step.state
        o = ops.delta_rule(main, gates, self.conv, self.a_log, self.dt_bias, states.get("conv"), states["S"], step,
                           self.heads, self.kv_heads, self.dk, self.dv, self.taps, gates_transposed=transposed)
        y = ops.gated_rmsnorm(o, main, self.channels, self.norm, self.eps, self.heads, self.dv, self.env.dtype)
        return ops.linear(y, self.w_o, deferred=True)


register_part("mixer", "gated_delta", GatedDeltaRule)
