"""What a layer adds to the residual stream from the token itself, after its sublayers:

  e = columns [first, first + dim) of the token's row of a second embedding table (one table for the model, a slice a layer)
  g = gelu_tanh(W_gate x) * e           x: the stream as it stands
  y = W_proj g                          x += y / rms(y) * weight      (a plain RMS norm, eps inside the root)

The product reads the stream itself, so everything that is due to the stream is summed first (`ResidualStream.rows`); the
normed result is left with the stream (`push_normed`) and joins it inside the next norm's kernel.
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import kernels
from .base import BuildContext, Param, Part, ResidualStream
from .linear import Linear
from .norm import RMSNorm


class TokenSideInput(Part):
    records_mixed_steps = True

    def __init__(self, hidden_size: int, dim: int, first_column: int, table: str, eps: float, ctx: BuildContext,
                 names=("gate", "proj", "norm")):
        self.dim, self.first, self.table_name = int(dim), int(first_column), table
        self.dtype = ctx.dtype
        self.gate = Linear(hidden_size, self.dim, names[0], False, ctx, suffix="")
        self.proj = Linear(self.dim, hidden_size, names[1], False, ctx, suffix="")
        self.norm = RMSNorm(hidden_size, eps, ctx, param_name=names[2])
        self.table = None

    def bind_shared(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.table_name]
        if self.table.dim() != 2 or self.first + self.dim > self.table.shape[1]:
            raise ValueError(f"columns {self.first} .. {self.first + self.dim} are not in a table of {tuple(self.table.shape)}")

    def named_parameters(self) -> Dict[str, Param]:
        out = dict(self.gate.named_parameters())
        out.update(self.proj.named_parameters())
        for name, p in self.norm.named_parameters().items():
            out[name] = Param(p.tensor, neutral=1.0)     # (stays in the activations' dtype: it is read beside other weights)
        return out

    def forward(self, stream: ResidualStream, batch) -> None:
        x = stream.rows(self.dtype)
        g = kernels.embed_gate(self.gate.forward(x), batch.token_ids, self.table, self.first)
        stream.push_normed(self.proj.forward(g), self.norm, 1.0)
