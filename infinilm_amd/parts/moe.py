"""A feed-forward of many small experts of which every token uses a few, with an optional expert that every token uses.

  z = W_router h (float32)          s = sigmoid(z)         the `top` experts with the largest s are chosen
  y = sum over the chosen e of expert_e(s_e * h)           the score multiplies the expert's input; scores are not renormalised
    + sigmoid(w_sg . h) * expert_shared(h)                 one number a token weighs the shared expert
  expert(x): g = min(W_gate x, limit), u = clamp(W_up x, -limit, limit), W_down (g * sigmoid(alpha g) * (u + 1))

The experts' matrices lie stacked in two tensors ([experts, 2 ff, hidden]: gate rows, then up rows; [experts, hidden, ff]); a
checkpoint's tensors `e<j>.gate`, `e<j>.up`, `e<j>.down` are views into them.  The router's rows and the shared expert's
weighing row are one float32-result product.  A step's (token, slot) pairs are ordered by expert on the device
(`kernels.moe_route`) and the experts' products walk that order tile by tile (`kernels.moe_gemm`), so nothing depends on
the host's view of the batch and a token's result does not depend on what else is in the step.  The shared expert is a
dense feed-forward and takes the dense products.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import kernels
from .base import BuildContext, FeedForward, Param
from .linear import FusedLinear, Linear
from .registry import register_feed_forward


@register_feed_forward("routed_experts")
class RoutedExperts(FeedForward):
    records_mixed_steps = True
    # a look into the routing: a list put here receives every call's chosen experts, int32 [tokens, top] (a copy a call)
    trace: Optional[list] = None

    def __init__(self, hidden_size: int, experts: int, top: int, expert_ff: int, limit: float, ctx: BuildContext,
                 shared_ff: int = 0, shared_limit: Optional[float] = None, alpha: float = 1.702,
                 names=("router", "e{}", "gate", "up", "down", "shared", "sg"), whole_output: bool = True):
        self.W, self.E, self.top, self.ff = int(hidden_size), int(experts), int(top), int(expert_ff)
        if not 1 <= self.top <= self.E:
            raise ValueError(f"{self.top} of {self.E} experts a token")
        self.limit, self.alpha = float(limit), float(alpha)
        self.shared_ff = int(shared_ff or 0)
        self.shared_limit = float(shared_limit if shared_limit is not None else limit)
        self.names = tuple(names)
        rn, en, gn, un, dn, sn, sgn = self.names
        self.dtype = ctx.dtype
        rows, rnames = [self.E], [rn]
        if self.shared_ff:
            rows.append(1)
            rnames.append(f"{sn}.{sgn}")
        self.router = FusedLinear(self.W, rows, rnames, False, ctx, suffix="")
        self.w_gate_up = torch.empty((self.E, 2 * self.ff, self.W), dtype=ctx.dtype, device=ctx.device)
        self.w_down = torch.empty((self.E, self.W, self.ff), dtype=ctx.dtype, device=ctx.device)
        self.shared_gate_up = self.shared_down = None
        if self.shared_ff:
            self.shared_gate_up = FusedLinear(self.W, [self.shared_ff, self.shared_ff], [f"{sn}.{gn}", f"{sn}.{un}"], False, ctx, suffix="")
            self.shared_down = Linear(self.shared_ff, self.W, f"{sn}.{dn}", False, ctx, suffix="")

    def named_parameters(self) -> Dict[str, Param]:
        rn, en, gn, un, dn, sn, sgn = self.names
        out = dict(self.router.named_parameters())
        for e in range(self.E):
            pre = en.format(e)
            out[f"{pre}.{gn}"] = Param(self.w_gate_up[e, :self.ff])
            out[f"{pre}.{un}"] = Param(self.w_gate_up[e, self.ff:])
            out[f"{pre}.{dn}"] = Param(self.w_down[e])
        if self.shared_ff:
            out.update(self.shared_gate_up.named_parameters())
            out.update(self.shared_down.named_parameters())
        return out

    def forward(self, x, batch) -> torch.Tensor:
        logits = kernels.gemm(x, self.router.weight, None, 1.0, torch.float32)          # [T, experts (+ 1)]
        plan = kernels.moe_route(logits, self.E, self.top,
                                 big_tiles_ok=x.dtype == torch.bfloat16 and self.W % 8 == 0 and self.ff % 8 == 0 and x.stride(0) % 8 == 0)
        if RoutedExperts.trace is not None:
            RoutedExperts.trace.append(plan.ids.clone())
        act = kernels.moe_gemm(x, self.w_gate_up, plan, True, self.limit, self.alpha)   # [pairs, ff], ordered by expert
        pair_out = kernels.moe_gemm(act, self.w_down, plan, False)                      # [pairs, hidden]
        shared = gate = None
        if self.shared_ff:
            shared = self.shared_down.forward(kernels.glu_clamp(self.shared_gate_up.forward(x), self.shared_limit, self.alpha))
            gate = logits[:, self.E:]
        return kernels.moe_combine(pair_out, plan, shared, gate)


@register_feed_forward("routed_activation_experts")
class RoutedActivationExperts(FeedForward):
    """Experts without a gate, weighed on their way out:

      z = W_router h (float32)      s = softmax(z) over all experts (`router` = "softmax") or sigmoid(z) ("sigmoid")
      y = sum over the `top` experts e with the largest s of  weight_scale * s_e * W_down,e act(W_up,e h)   (not renormalised)
        + W_down,shared act(W_up,shared h)                                                           (if `shared_ff`)

    `activation`: "relu2" (the square of relu) for the experts (the kernels' epilogue) and any of the kernels' activations
    for the shared expert.  The experts' matrices lie stacked ([experts, ff, hidden], [experts, hidden, ff]); a checkpoint's
    `e<j>.up`, `e<j>.down` are views into them.  Routing, ordering and the experts' products run on the device alone, as for
    `routed_experts`; a pair's weight multiplies its expert's result in float32 when the token's results are summed."""
    records_mixed_steps = True
    trace: Optional[list] = None     # as `RoutedExperts.trace`

    def __init__(self, hidden_size: int, experts: int, top: int, expert_ff: int, ctx: BuildContext, router: str = "softmax",
                 weight_scale: float = 1.0, activation: str = "relu2", shared_ff: int = 0,
                 names=("router", "e{}", "up", "down", "shared")):
        self.W, self.E, self.top, self.ff = int(hidden_size), int(experts), int(top), int(expert_ff)
        if not 1 <= self.top <= self.E:
            raise ValueError(f"{self.top} of {self.E} experts a token")
        if router not in ("softmax", "sigmoid"):
            raise ValueError(f"unknown router {router!r} (softmax, sigmoid)")
        if activation != "relu2":
            raise ValueError(f"the experts' products take relu2 as their activation, got {activation!r}")
        self.softmax, self.weight_scale, self.activation = router == "softmax", float(weight_scale), activation
        self.shared_ff = int(shared_ff or 0)
        self.names = tuple(names)
        rn, en, un, dn, sn = self.names
        self.dtype = ctx.dtype
        self.router = Linear(self.W, self.E, rn, False, ctx, suffix="")
        self.w_up = torch.empty((self.E, self.ff, self.W), dtype=ctx.dtype, device=ctx.device)
        self.w_down = torch.empty((self.E, self.W, self.ff), dtype=ctx.dtype, device=ctx.device)
        self.shared_up = self.shared_down = None
        if self.shared_ff:
            self.shared_up = Linear(self.W, self.shared_ff, f"{sn}.{un}", False, ctx, suffix="")
            self.shared_down = Linear(self.shared_ff, self.W, f"{sn}.{dn}", False, ctx, suffix="")

    def named_parameters(self) -> Dict[str, Param]:
        rn, en, un, dn, sn = self.names
        out = dict(self.router.named_parameters())
        for e in range(self.E):
            pre = en.format(e)
            out[f"{pre}.{un}"] = Param(self.w_up[e])
            out[f"{pre}.{dn}"] = Param(self.w_down[e])
        if self.shared_ff:
            out.update(self.shared_up.named_parameters())
            out.update(self.shared_down.named_parameters())
        return out

    def forward(self, x, batch) -> torch.Tensor:
        logits = kernels.gemm(x, self.router.weight, None, 1.0, torch.float32)          # [T, experts]
        plan = kernels.moe_route(logits, self.E, self.top, softmax=self.softmax, weight_scale=self.weight_scale,
                                 big_tiles_ok=x.dtype == torch.bfloat16 and self.W % 8 == 0 and self.ff % 8 == 0 and x.stride(0) % 8 == 0)
        if RoutedActivationExperts.trace is not None:
            RoutedActivationExperts.trace.append(plan.ids.clone())
        act = kernels.moe_gemm(x, self.w_up, plan, False, gather=True, act=self.activation)   # [pairs, ff], ordered by expert
        pair_out = kernels.moe_gemm(act, self.w_down, plan, False)                            # [pairs, hidden]
        shared = None
        if self.shared_ff:
            shared = self.shared_down.forward(kernels.activation(self.shared_up.forward(x), self.activation))
        return kernels.moe_combine(pair_out, plan, shared, None, weighted=True)
