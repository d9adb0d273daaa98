"""A selective scan whose every channel keeps a state vector of its own (the matrix-decay form).

  W_in h = [x: inner | z: inner];  x passes a causal convolution per channel (`conv_taps` inputs, the last the token's own,
  zeros before a sequence's start) with a bias, then silu;
  W_x x = [dt: dt_rank | B: state | C: state];  dt <- softplus(W_dt dt + dt_bias), one step size a channel;  A = -exp(A_log);
  S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,   y_c = sum_n S[c, n] C_n + D_c x_c      (S from zero, per sequence)
  y * silu(z), the output projection.

Two states a request: the recurrence's [inner, state] and the convolution's last conv_taps - 1 inputs [conv_taps - 1, inner],
both float32 rows of the cache manager's pools.  Step sizes, softplus, exponentials, the state and its sums are float32
whatever the activations' dtype; the projections run in the activations' dtype.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from .. import kernels
from ..cache.needs import FixedState
from .base import BuildContext, Mixer, Param
from .linear import Linear
from .registry import register_mixer


@register_mixer("selective_scan")
class SelectiveScan(Mixer):
    records_mixed_steps = True

    def __init__(self, hidden_size: int, inner: int, state: int, dt_rank: int, conv_taps: int, ctx: BuildContext,
                 names: Sequence[str] = ("in", "conv", "conv.b", "x", "dt", "dt.b", "A_log", "D", "o")):
        self.inner, self.state, self.dt_rank, self.taps = int(inner), int(state), int(dt_rank), int(conv_taps)
        if not 1 <= self.taps <= kernels.CONV_MAX_TAPS:
            raise ValueError(f"{self.taps} taps: the convolution kernel takes 1 to {kernels.CONV_MAX_TAPS}")
        if not 1 <= self.state <= kernels.SELECTIVE_SCAN_MAX_STATE:
            raise ValueError(f"state size {self.state}: the scan kernel takes 1 to {kernels.SELECTIVE_SCAN_MAX_STATE}")
        self.names = tuple(names)
        n = self.names
        self.dtype = ctx.dtype
        dev = ctx.device
        self.in_proj = Linear(hidden_size, 2 * self.inner, n[0], False, ctx, suffix="")
        self.x_proj = Linear(self.inner, self.dt_rank + 2 * self.state, n[3], False, ctx, suffix="")
        self.dt_proj = Linear(self.dt_rank, self.inner, n[4], False, ctx, suffix="")
        self.o_proj = Linear(self.inner, hidden_size, n[8], False, ctx, suffix="")
        self.conv_w = torch.empty((self.inner, self.taps), dtype=ctx.dtype, device=dev)
        self.conv_b = torch.empty((self.inner,), dtype=ctx.dtype, device=dev)
        self.dt_bias = torch.empty((self.inner,), dtype=torch.float32, device=dev)
        self.a_log = torch.empty((self.inner, self.state), dtype=torch.float32, device=dev)
        self.skip = torch.empty((self.inner,), dtype=torch.float32, device=dev)

    def named_parameters(self) -> Dict[str, Param]:
        n = self.names
        out = dict(self.in_proj.named_parameters())
        for lin in (self.x_proj, self.dt_proj, self.o_proj):
            out.update(lin.named_parameters())
        out.update({n[1]: Param(self.conv_w), n[2]: Param(self.conv_b), n[5]: Param(self.dt_bias), n[6]: Param(self.a_log),
                    n[7]: Param(self.skip)})
        return out

    def cache_need(self):
        return (FixedState((self.taps - 1, self.inner), torch.float32), FixedState((self.inner, self.state), torch.float32))

    def forward(self, x, batch, view):
        conv, scan = view
        inner, R, N = self.inner, self.dt_rank, self.state
        segments = scan.state_in.numel()
        u = self.in_proj.forward(x)                                       # [T, x | z]
        xc = kernels.causal_conv(u[:, :inner], self.conv_w, self.conv_b, conv.pool, conv.state_in, conv.state_out,
                                 batch.seg_of_token, batch.seg_offsets, segments, "silu")          # float32 [T, inner]
        xa = xc if self.dtype == torch.float32 else kernels.activation(xc, "none", out_dtype=self.dtype)
        r = self.x_proj.forward(xa)                                       # [T, dt | B | C]
        raw = self.dt_proj.forward(r[:, :R])                              # [T, inner], before bias and softplus
        y = kernels.selective_scan(xc, raw, self.dt_bias, r[:, R:R + N], r[:, R + N:], u[:, inner:], self.a_log, self.skip,
                                   scan.pool, scan.state_in, scan.state_out, batch.seg_offsets, segments, max_len=batch.max_q_len)
        return self.o_proj.forward(y, allow_parts=True)
