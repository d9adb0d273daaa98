"""Dense projections y = alpha * (x W^T + b), W [out, in].

Reference: csrc/layers/linear/base_linear.{hpp,cpp} (alpha, weight layout) and fused_linear.cpp
(:62-71 the q|k|v split, :90-111 and :163-185 the named row-slices of one fused weight): several
checkpoint tensors are row ranges of one allocation, so loading by name fills the fused weight and
one product computes all of them.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from .. import kernels
from .base import BuildContext, DeferredNorm, NormTail, Param, join_name


class FusedLinear:
    """`out_sizes[i]` rows of the weight belong to the checkpoint tensor `names[i]`.

    `suffix`: a tensor's name is `names[i]` + "." + suffix ("": the bare name).
    `out_heads[i]` = (heads, size, padded size): the rows of piece i are heads of `size` rows in a checkpoint, held here
    as heads of `padded size` rows whose last rows are zeros and stay zeros (`out_sizes[i]` = heads * padded size), so
    that heads of a size the kernels do not take run as the next size they do.  `in_heads` = (heads, size, padded
    size): the same for the columns."""

    def __init__(self, in_features: int, out_sizes: Sequence[int], names: Sequence[str], bias: bool,
                 ctx: BuildContext, suffix: str = "weight", out_heads: Optional[Sequence] = None,
                 in_heads: Optional[tuple] = None, bias_suffix: str = "bias"):
        self.in_features = int(in_features)
        self.bias_suffix = bias_suffix      # a bias's name is `names[i]` + "." + bias_suffix
        self.out_sizes = [int(s) for s in out_sizes]
        self.names = list(names)
        self.suffix = suffix
        self.out_heads = list(out_heads) if out_heads is not None else [None] * len(self.names)
        self.in_heads = tuple(in_heads) if in_heads is not None and in_heads[1] != in_heads[2] else None
        for size, oh in zip(self.out_sizes, self.out_heads):
            if oh is not None and (oh[0] * oh[2] != size or oh[1] > oh[2]):
                raise ValueError(f"{oh[0]} heads of {oh[1]} filled up to {oh[2]} are not {size} rows")
        if self.in_heads is not None and self.in_heads[0] * self.in_heads[2] != self.in_features:
            raise ValueError("filled-up columns must make up the whole input")
        n = sum(self.out_sizes)
        padded = self.in_heads is not None or any(oh is not None and oh[1] != oh[2] for oh in self.out_heads)
        make = torch.zeros if padded else torch.empty
        self.weight = make((n, self.in_features), dtype=ctx.dtype, device=ctx.device)
        self.bias = make((n,), dtype=ctx.dtype, device=ctx.device) if bias else None
        self._frag = {}   # layout -> (version of the weight it was packed from, the weight in fragment order)

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        row = 0
        for name, size, oh in zip(self.names, self.out_sizes, self.out_heads):
            w = self.weight[row:row + size]
            b = self.bias[row:row + size] if self.bias is not None else None
            if oh is not None and oh[1] != oh[2]:
                heads, real, pad = oh
                out[join_name(name, self.suffix)] = Param(w.view(heads, pad, self.in_features)[:, :real], shape=(heads * real, self.in_features))
                if b is not None:
                    out[join_name(name, self.bias_suffix)] = Param(b.view(heads, pad)[:, :real], shape=(heads * real,))
            elif self.in_heads is not None:
                heads, real, pad = self.in_heads
                out[join_name(name, self.suffix)] = Param(w.view(size, heads, pad)[:, :, :real], shape=(size, heads * real))
                if b is not None:
                    out[join_name(name, self.bias_suffix)] = Param(b)
            else:
                out[join_name(name, self.suffix)] = Param(w)
                if b is not None:
                    out[join_name(name, self.bias_suffix)] = Param(b)
            row += size
        return out

    def frag_weight(self, kind: str = "plain", **layout):
        """The weight in fragment order (`kernels.pack_weight`), packed at its first use and again when the weight
        has been written since (a second copy of the weight: the many-rows products keep the plain rows)."""
        key = (kind, tuple(sorted(layout.items())))
        held = self._frag.get(key)
        if held is None or held[0] != self.weight._version or held[2] != self.weight.data_ptr():
            held = (self.weight._version, kernels.pack_weight(self.weight, kind, **layout), self.weight.data_ptr())
            self._frag[key] = held
        return held[1]

    def forward(self, x: torch.Tensor, alpha: float = 1.0, out_dtype: Optional[torch.dtype] = None,
                allow_parts: bool = False) -> torch.Tensor:
        """`allow_parts`: the result may come as float32 parts [P, T, out] still to be summed; only for a
        result that goes straight into `ResidualStream.push` (the next norm's kernel sums them)."""
        frag = self.frag_weight if kernels.frag_weight_ok(self.weight) and x.shape[0] <= max(kernels.FRAG_MAX_ROWS, kernels.TALL_MAX_ROWS) else None
        return kernels.gemm(x, self.weight, self.bias, alpha, out_dtype, allow_parts=allow_parts, frag_w=frag)


    def forward_tail(self, x: torch.Tensor, tail: NormTail) -> Optional[DeferredNorm]:
        """The projection with the residual sum and the first half of the following norm in its epilogue
        (`kernels.gemm_tail`), or None where that kernel does not take the shapes."""
        if not kernels.tail_ok(x.shape[0], self.weight, self.bias, tail.weight, x.dtype):
            return None
        xw, ss = kernels.gemm_tail(x, self.weight, self.bias, tail.scale, tail.residual, tail.weight)
        return DeferredNorm(xw, ss, tail.eps)


class Linear(FusedLinear):
    def __init__(self, in_features: int, out_features: int, name: str, bias: bool, ctx: BuildContext,
                 suffix: str = "weight", in_heads: Optional[tuple] = None, bias_suffix: str = "bias"):
        super().__init__(in_features, [out_features], [name], bias, ctx, suffix=suffix, in_heads=in_heads, bias_suffix=bias_suffix)
