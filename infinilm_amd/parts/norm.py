"""RMS norm fused with the residual add.

Reference: `RMSNorm::forward_inplace(h, residual)` as used in
csrc/models/minicpm4/minicpm4_for_causal_lm.cpp:52,54,99: residual = h + residual, h = norm(residual).
Here the residual stream is float32 and the branch's scale (the reference's GEMM alpha on o_proj
and down_proj, :23-34) is applied in the same kernel: residual += scale * branch.
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import kernels
from .base import BuildContext, Norm, NormTail, Param, ResidualStream
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    takes_frag_request = True

    def __init__(self, size: int, eps: float, ctx: BuildContext, param_name: str = "weight"):
        self.size = int(size)
        self.eps = float(eps)
        self.dtype = ctx.dtype
        self.param_name = param_name    # "": the weight lies under the norm's own name in a checkpoint
        self.weight = torch.empty((self.size,), dtype=ctx.dtype, device=ctx.device)

    def _set_weight(self, t: torch.Tensor) -> None:
        self.weight = t

    def named_parameters(self) -> Dict[str, Param]:
        return {self.param_name: Param(self.weight, keep_f32=True, replace=self._set_weight, neutral=1.0)}

    def apply(self, x: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """The norm of rows that are not the residual stream (a branch's output normed before it is added): sums in
        float32, the result in `out_dtype`."""
        return kernels.group_norm_gate(x, self.weight, self.eps, 1, out_dtype=out_dtype)

    def tail(self, stream: ResidualStream, scale: float, rows: int):
        stream.settle()
        if stream.pending is not None or self.dtype != torch.bfloat16 or rows > kernels.TAIL_MAX_ROWS:
            return None
        return NormTail(stream.residual, float(scale), self.weight, self.eps)

    def forward(self, stream: ResidualStream, frag: bool = False):
        """`frag`: the consumer takes its rows in fragment order (`kernels.FragRows`)."""
        if stream.more:
            stream.settle()
        post = stream.pending_norm
        if post is not None and not frag and isinstance(post, RMSNorm):
            # the branch's own norm, the sum and this norm in one kernel
            x = kernels.norm_add_norm(stream.residual, stream.pending, post.weight, post.eps, stream.pending_scale, self.weight,
                                      self.eps, self.dtype)
            stream.pending, stream.pending_scale, stream.pending_norm = None, 1.0, None
            return x
        stream.settle()
        x = kernels.add_rmsnorm(stream.residual, stream.pending, self.weight, stream.pending_scale, self.eps,
                                self.dtype, frag=frag)
        stream.pending = None
        stream.pending_scale = 1.0
        return x


@register_norm("group_rmsnorm")
class GroupRMSNorm(Norm):
    """RMS norm in `groups` consecutive equal parts of a row: each part is divided by its own sqrt(mean square + eps), the whole
    row is multiplied by one weight.  Fused with what is due to the residual stream: a plain branch, a branch times
    sigmoid(gate) (`ResidualStream.push_gated`) or a branch with an RMS norm of its own (`push_normed`) is added in the
    same kernel (`kernels.stream_update`)."""

    def __init__(self, size: int, eps: float, groups: int, ctx: BuildContext, param_name: str = "weight"):
        self.size, self.eps, self.groups = int(size), float(eps), int(groups)
        if self.groups < 1 or self.size % self.groups:
            raise ValueError(f"rows of {self.size} do not divide into {self.groups} groups")
        self.dtype = ctx.dtype
        self.param_name = param_name
        self.weight = torch.empty((self.size,), dtype=ctx.dtype, device=ctx.device)

    def named_parameters(self) -> Dict[str, Param]:
        return {self.param_name: Param(self.weight, neutral=1.0)}

    def apply(self, x: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        return kernels.group_norm_gate(x, self.weight, self.eps, self.groups, out_dtype=out_dtype)

    def forward(self, stream: ResidualStream, frag: bool = False):
        if stream.more:
            stream.settle()
        post = stream.pending_norm
        if post is not None and not (isinstance(post, RMSNorm) and post.weight.dtype == self.weight.dtype):
            stream.settle()      # a branch norm of another kind: applied by itself
            post = None
        gate, bias = stream.pending_gate if stream.pending_gate is not None else (None, None)
        x = kernels.stream_update(stream.residual, stream.pending, stream.pending_scale, gate=gate, gate_bias=bias,
                                  branch_weight=post.weight if post is not None else None,
                                  branch_eps=post.eps if post is not None else 0.0,
                                  weight=self.weight, eps=self.eps, groups=self.groups, out_dtype=self.dtype)
        stream.pending, stream.pending_scale, stream.pending_norm, stream.pending_gate = None, 1.0, None, None
        return x


@register_norm("layernorm")
class LayerNorm(Norm):
    """(x - mean) / sqrt(mean of squared deviations + eps) * weight + bias, fused with the sums that are due to the residual
    stream: the pending branch and every further addend (`ResidualStream.more`) are added in the same kernel.
    `param_name` / `bias_name`: the tensors' names under the norm's own name ("": the norm's name itself)."""

    def __init__(self, size: int, eps: float, ctx: BuildContext, bias: bool = True, param_name: str = "weight",
                 bias_name: str = "bias"):
        self.size, self.eps, self.dtype = int(size), float(eps), ctx.dtype
        self.param_name, self.bias_name = param_name, bias_name
        self.weight = torch.empty((self.size,), dtype=ctx.dtype, device=ctx.device)
        self.bias = torch.empty((self.size,), dtype=ctx.dtype, device=ctx.device) if bias else None

    def named_parameters(self) -> Dict[str, Param]:
        out = {self.param_name: Param(self.weight, neutral=1.0)}
        if self.bias is not None:
            out[self.bias_name] = Param(self.bias)
        return out

    def forward(self, stream: ResidualStream, frag: bool = False):
        if stream.pending_gate is not None:
            stream.settle()
        if stream.pending_norm is not None:
            norm, stream.pending_norm = stream.pending_norm, None
            stream.pending = norm.apply(stream.pending)
        addends = ([(stream.pending, stream.pending_scale)] if stream.pending is not None else []) + stream.more
        x = kernels.add_layernorm(stream.residual, addends, self.weight, self.bias, self.eps, self.dtype)
        stream.pending, stream.pending_scale, stream.more = None, 1.0, []
        return x
