"""Hyper-connections: a pre-norm block over S copies of the residual stream, and
the token shift that can stand in front of a mixer.

The residual is float32 [T, S, n], every stream equal to the embedding's rows
at the start.  Sublayer q of a block (1: the mixer, 2: the feed-forward) has
three small weights: ``in`` [S], ``out`` [S], ``mix`` [S, S] (indexed [from, to]):

    u   = sum_s in[s] x_s                       what the sublayer reads
    y   = sublayer(norm(u))
    x_t = sum_s mix[s, t] x_s + out[t] y        every stream at once, from the old ones

and after the last block the streams are added up.  As in the single-stream
block, a sublayer's write is left to whoever reads the residual next: one
kernel writes the streams, reads u from the new ones and norms it.  The final
sum is that same kernel with in = 1.  All of it is float32.

Token shift: the rows h_p that a mixer is about to read become
h_p + (h_{p-1} - h_p) * mu, element by element, h_{p-1} the row before as it was
before this replacement (zeros at position 0).  The last row of every sequence
is kept as per-request state, so that a prompt cut into portions, and decoding,
find it.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import StateNeed
from ..weights.loader import TensorDecl
from .base import Block, BuildEnv, Part, StepView, build_part, register_part


class StreamDelta:
    """What a sublayer of a hyper-connected block still owes the streams: its output ``y``
    (a tensor, or an unfinished product) and the ``mix`` and ``out`` weights it is written with."""

    def __init__(self, y, mix: torch.Tensor, out: torch.Tensor):
        self.y, self.mix, self.out = y, mix, out


class TokenShift(Part):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        self.size = int(spec.params["size"])
        self.name = spec.names["weight"]

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.size,), "normal(0.3,0.1)")]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        self.mu = weights[self.name].to(torch.float32).contiguous()

    def state_need(self) -> StateNeed:
        return StateNeed((self.size,), torch.float32)

    def forward(self, h: torch.Tensor, step: StepView, state: torch.Tensor) -> torch.Tensor:
        """h: float32 [T, size], the rows before the shift; returns the shifted rows in the run
        dtype and leaves every sequence's last row of h in ``state``."""
        return self.env.ops.token_shift(h, self.mu, state, step, self.env.dtype)


class HyperBlock(Block):
    def __init__(self, spec, mixer, ffn, norms):
        super().__init__(spec)
        self.streams = int(spec.params["streams"])
        self.width = int(spec.params["width"])
        if self.streams <= 0:
            raise ValueError("a hyper-connected block needs at least one stream")
        self.mixer = mixer
        self.ffn = ffn
        self.norm_mixer = norms["mixer"]
        self.norm_ffn = norms["ffn"] if ffn is not None else None
        self.shift = build_part("shift", spec.parts["shift"]) if "shift" in spec.parts else None
        self.replayable = all(p.replayable for p in self._parts())

    def _parts(self):
        return [p for p in (self.norm_mixer, self.shift, self.mixer, self.norm_ffn, self.ffn) if p is not None]

    def _own(self) -> List[str]:
        return ["in1", "out1", "mix1"] + (["in2", "out2", "mix2"] if self.ffn is not None else [])

    def tensors(self) -> List[TensorDecl]:
        s = self.streams
        # (random weights: reads and writes near 1 / S and 1, a mix near the identity)
        init = {"in": f"normal({1.0 / s},0.05)", "out": "normal(1.0,0.05)", "mix": f"normal({1.0 / s},0.1)"}
        out = [TensorDecl(self.spec.names[r], (s, s) if r.startswith("mix") else (s,), init[r[:-1]]) for r in self._own()]
        return out + [d for p in self._parts() for d in p.tensors()]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        for part in self._parts():
            part.load(weights, env)
        self.w = {r: weights[self.spec.names[r]].to(torch.float32).contiguous() for r in self._own()}
        self.rms = []
        for norm in (self.norm_mixer, self.norm_ffn):
            rms = None if norm is None else norm.as_rms()
            if norm is not None and rms is None:
                raise ValueError(f"a hyper-connected block norms with the RMS norm that its kernel has built in, "
                                 f"not with '{norm.spec.kind}'")
            self.rms.append(rms)
        env.ops.check_streams(self.streams, self.width)
        self.ones = torch.ones(self.streams, dtype=torch.float32, device=env.device)

    def state_need(self):
        needs = {}
        if self.shift is not None:
            needs["shift"] = self.shift.state_need()
        mixer = self.mixer.state_need()
        if mixer is not None:
            needs["mixer"] = mixer
        return needs or None

    def open(self, x: torch.Tensor) -> torch.Tensor:
        return self.env.ops.streams_open(x, self.streams)

    def close(self, resid, pending, final_norm, rows=None, num_rows=None):
        rms = final_norm.as_rms()
        if rms is None:
            raise ValueError("the norm after hyper-connected blocks must be an RMS norm")
        return self.env.ops.streams_norm(resid, pending, self.ones, rms[0], rms[1], self.env.dtype,
                                         rows=rows, num_rows=num_rows)

    def forward(self, resid: torch.Tensor, pending: Optional[StreamDelta], step: StepView) -> StreamDelta:
        ops = self.env.ops
        states = step.state or {}
        mixer_state = states.get("mixer")
        weight, eps = self.rms[0]
        if self.shift is not None:
            h = ops.streams_norm(resid, pending, self.w["in1"], weight, eps, self.env.dtype,
                                 shift=(self.shift.mu, states["shift"], step))
        else:
            h = ops.streams_norm(resid, pending, self.w["in1"], weight, eps, self.env.dtype)
        step.state = mixer_state
        a = self.mixer.forward(h, step)
        step.state = states
        owed = StreamDelta(a, self.w["mix1"], self.w["out1"])
        if self.ffn is None:
            return owed
        weight, eps = self.rms[1]
        m = ops.streams_norm(resid, owed, self.w["in2"], weight, eps, self.env.dtype)
        return StreamDelta(self.ffn.forward(m, step), self.w["mix2"], self.w["out2"])


register_part("shift", "token_shift", TokenShift)
register_part("block", "hyper_prenorm", HyperBlock)
