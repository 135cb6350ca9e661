"""Parallel residual block: the mixer and the feed-forward read two norms of the same x and their
outputs are added together,  x <- x + (mixer(n1(x)) + ff(n2(x))).  Both sums are left to whoever
normalises next (the following block or the final norm), which adds them in float32 in the same
pass as its norm; where both norms are layer norms with equal eps, one pass over the row gives the
rows of both (they share the mean and the variance).  Without a feed-forward the block is
x <- x + mixer(n1(x))."""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..weights.loader import TensorDecl
from .base import Block, BuildEnv, StepView, register_part, run_norm


class ParallelBlock(Block):
    def __init__(self, spec, mixer, ffn, norms):
        super().__init__(spec)
        self.mixer = mixer
        self.ffn = ffn
        self.norm_mixer = norms["mixer"]
        self.norm_ffn = norms["ffn"] if ffn is not None else None
        self.replayable = all(p.replayable for p in self._parts())

    def _parts(self):
        return [p for p in (self.norm_mixer, self.mixer, self.norm_ffn, self.ffn) if p is not None]

    def tensors(self) -> List[TensorDecl]:
        return [d for p in self._parts() for d in p.tensors()]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        for part in self._parts():
            part.load(weights, env)
        # two layer norms of one row in one pass, where that is what the norms are
        self.pair = None
        if self.norm_ffn is not None:
            a = getattr(self.norm_mixer, "as_layer_norm", lambda: None)()
            b = getattr(self.norm_ffn, "as_layer_norm", lambda: None)()
            if a is not None and b is not None and a[1] == b[1]:
                self.pair = ((a[0], b[0]), a[1])

    def _owed(self, pending) -> Tuple[torch.Tensor, ...]:
        ops = self.env.ops
        return tuple(ops.resolve(y) for y in (pending or ()) if y is not None)

    def _one(self, owed: Tuple[torch.Tensor, ...]) -> Optional[torch.Tensor]:
        """What is owed as one tensor, for a norm of another kind, which takes one."""
        if not owed:
            return None
        return owed[0] if len(owed) == 1 else (owed[0].to(torch.float32) + owed[1].to(torch.float32)).to(owed[0].dtype)

    def forward(self, resid: torch.Tensor, pending, step: StepView):
        owed = self._owed(pending)
        if self.pair is not None:
            (w1, w2), eps = self.pair
            n1, n2 = self.env.ops.add_layernorm(resid, owed, (w1, w2), eps, self.env.dtype)
        else:
            n1 = run_norm(self.norm_mixer, resid, self._one(owed))
            n2 = run_norm(self.norm_ffn, resid, None) if self.norm_ffn is not None else None
        a = self.mixer.forward(n1, step)
        if self.ffn is None:
            return (a,)
        return (a, self.ffn.forward(n2, step))

    def close(self, resid, pending, final_norm, rows=None, num_rows=None):
        owed = self._owed(pending)
        ln = getattr(final_norm, "as_layer_norm", lambda: None)()
        if ln is not None:
            return self.env.ops.add_layernorm(resid, owed, (ln[0],), ln[1], self.env.dtype, rows=rows, num_rows=num_rows)[0]
        return run_norm(final_norm, resid, self._one(owed), rows=rows, num_rows=num_rows)


register_part("block", "parallel_prenorm", ParallelBlock)
