"""Token embedding (x_t = E[token_t], no scaling; layers/src/embedding.cpp:37-44;
with ``scale`` and a table of learned position vectors, x_t = scale * E[token_t] + P[position_t],
computed in float32) and the head that turns final hidden rows into float32 logits
(model/src/qwen3_paged_batch.cpp:343-346; with ``softcap`` c, logits z become c * tanh(z / c)).  The reference always uses the
embedding matrix as the head (model/src/qwen3_layers.cpp:246-265) and rounds
logits to half precision; here a head has its own matrix unless the model ties
it, and logits leave the product in float32."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..weights.loader import TensorDecl
from .base import BuildEnv, Part, register_part
from .linear import as_matrix


class TokenEmbedding(Part):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        self.vocab = int(spec.params["vocab_size"])
        self.hidden = int(spec.params["hidden_size"])
        self.name = spec.names["weight"]
        self.scale = float(spec.params.get("scale", 1.0))
        self.pos_name = spec.names.get("positions")              # a learned vector for every position, or none
        self.max_positions = int(spec.params.get("max_positions", 0))
        self.pos_table = None

    def tensors(self) -> List[TensorDecl]:
        out = [TensorDecl(self.name, (self.vocab, self.hidden))]
        if self.pos_name is not None:
            out.append(TensorDecl(self.pos_name, (self.max_positions, self.hidden)))
        return out

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        self.table = weights[self.name].to(env.dtype).contiguous()      # rows are gathered: row-major only
        if self.pos_name is not None:
            self.pos_table = weights[self.pos_name].to(env.dtype).contiguous()

    def forward(self, token_ids: torch.Tensor, num_rows: int, positions: torch.Tensor = None) -> torch.Tensor:
        """Rows of the table as a float32 residual stream [rows, hidden]."""
        if self.pos_table is None and self.scale == 1.0:
            return self.env.ops.embed(self.table, token_ids, num_rows)
        if self.pos_table is not None and positions is None:
            raise ValueError("an embedding with learned positions needs the rows' positions")
        return self.env.ops.embed(self.table, token_ids, num_rows, scale=self.scale,
                                  positions=positions, pos_table=self.pos_table)


class LinearHead(Part):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        self.vocab = int(spec.params["vocab_size"])
        self.hidden = int(spec.params["hidden_size"])
        self.name = spec.names["weight"]
        cap = spec.params.get("softcap")
        self.softcap = None if cap is None else float(cap)
        if self.softcap is not None and self.softcap <= 0.0:
            raise ValueError("a head's softcap must be positive")

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.vocab, self.hidden))]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv, share_with=None) -> None:
        super().load(weights, env)
        if share_with is not None and share_with.name == self.name:
            self.weight = as_matrix(share_with.table, env)     # tied: the row-major copy is shared
        else:
            self.weight = as_matrix(weights[self.name], env)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = self.env.ops.linear(x, self.weight, out_dtype=torch.float32)
        return logits if self.softcap is None else self.env.ops.softcap(logits, self.softcap)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
