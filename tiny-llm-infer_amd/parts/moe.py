"""Routed experts: a feed-forward of E small gated feed-forwards of which every row uses ``top``,
beside an optional shared one that every row uses.

    s = sigmoid(W_router h)                                   [E], float32
    the experts form ``groups`` equal groups of neighbours; a group's score is the sum of its two
        largest s; experts outside the ``keep`` best groups cannot be chosen
    chosen = the ``top`` largest s among the rest;  weight_j = s_j / (sum of the chosen s + 1e-20) * scale
    out = sum_j weight_j expert_j(h)  +  sigmoid(w_sg . h) * shared(h)
    expert(h) = W_down (silu(W_gate h) * (W_up h))

The router's product gives float32 (the row of the shared expert's gate rides along as one more
row of that matrix); scores, choice and weights are float32.  A row's chosen experts are added
in the order of the choice, whatever else is in the step.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorDecl
from .base import BuildEnv, FeedForward, StepView, register_part
from .linear import GatedMatrix, as_matrix


class RoutedExperts(FeedForward):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.experts = int(p["experts"])
        self.top = int(p["top"])
        self.groups = int(p.get("groups") or 1)
        self.keep = int(p.get("keep") or self.groups)
        self.scale = float(p.get("scale", 1.0))
        self.inter = int(p["intermediate_size"])
        shared = p.get("shared_intermediate_size")
        self.shared_inter = None if shared is None else int(shared)
        if self.experts % self.groups or not 1 <= self.keep <= self.groups \
                or not 1 <= self.top <= self.keep * (self.experts // self.groups):
            raise ValueError(f"{self.experts} experts in {self.groups} groups, {self.keep} kept, cannot give {self.top}")

    def _expert(self, j: int, role: str) -> str:
        return self.spec.names["experts"].format(j) + role

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        out = [TensorDecl(n["router"], (self.experts, self.hidden))]
        for j in range(self.experts):
            out += [TensorDecl(self._expert(j, "gate"), (self.inter, self.hidden)),
                    TensorDecl(self._expert(j, "up"), (self.inter, self.hidden)),
                    TensorDecl(self._expert(j, "down"), (self.hidden, self.inter))]
        if self.shared_inter is not None:
            out += [TensorDecl(n["shared_gate"], (self.shared_inter, self.hidden)),
                    TensorDecl(n["shared_up"], (self.shared_inter, self.hidden)),
                    TensorDecl(n["shared_down"], (self.hidden, self.shared_inter)),
                    TensorDecl(n["shared_scale"], (1, self.hidden))]
        return out

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        env.ops.check_expert_sizes(self.experts, self.top, self.groups, self.keep, self.hidden, self.inter)
        rows = [weights[n["router"]]] + ([weights[n["shared_scale"]]] if self.shared_inter is not None else [])
        self.w_router = torch.cat([r.to(env.dtype) for r in rows], dim=0).contiguous()       # few rows: kept row-major
        # the experts' matrices side by side: [E, 2 ff, hidden] (an expert's gate rows, then its up rows), [E, hidden, ff]
        self.w_gate_up = torch.stack([torch.cat([weights[self._expert(j, "gate")], weights[self._expert(j, "up")]], dim=0)
                                      for j in range(self.experts)]).to(env.dtype).contiguous()
        self.w_down = torch.stack([weights[self._expert(j, "down")] for j in range(self.experts)]).to(env.dtype).contiguous()
        # (where the kernels for the matrix cores apply they read a layout of their own, and the row-major
        # matrices are not kept beside it)
        self.packed = env.ops.pack_experts(self.w_gate_up, self.w_down)
        if self.packed is not None:
            self.w_gate_up = self.w_down = None
        self.shared_gate_up = self.shared_down = None
        if self.shared_inter is not None:
            self.shared_gate_up = GatedMatrix(weights[n["shared_gate"]], weights[n["shared_up"]], env)
            self.shared_down = as_matrix(weights[n["shared_down"]], env)

    def workspace_elems(self, rows: int) -> int:
        return rows * (self.top * (3 * self.inter + self.hidden) + 3 * (self.shared_inter or 0) + 2 * self.experts)

    def forward(self, x: torch.Tensor, step: StepView):
        ops = self.env.ops
        z, transposed = ops.small_product(x, self.w_router)
        ids, weights, shared_gate = ops.route_experts(z, self.experts, self.top, self.groups, self.keep, self.scale,
                                                      self.shared_inter is not None, transposed)
        shared = None
        if self.shared_inter is not None:
            shared = ops.linear(ops.linear_swiglu(x, self.shared_gate_up), self.shared_down)
        return ops.apply_experts(x, ids, weights, self.w_gate_up, self.w_down, self.packed, shared, shared_gate)


register_part("ffn", "routed_experts", RoutedExperts)
