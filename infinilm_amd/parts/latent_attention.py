"""Attention whose keys and values are made from a small latent row a token.

  q = W_q h                      heads x [dim unrotated | rot_dim rotated]
  W_dkv h                        kv_rank + rot_dim rows: c = RMS norm of the first kv_rank (times a weight), the last
                                 rot_dim are one rotated key part shared by all heads
  key_h = [W_uk,h c | rotated part],  value_h = W_uv,h c
  score = (q_unrotated . key_unrotated + q_rotated . key_rotated) * scale,  causal softmax,  W_o on the heads' results

The cache holds c and the rotated key part only.  The step runs the absorbed form: a head's unrotated query is carried
into the latent space (W_uk,h^T q_h, a product per head), so the scores are dot products of rows of kv_rank + rot_dim
entries against one cached key row per token, the attention's values are the latent rows themselves, and W_uv,h is
applied to the head's result afterwards.  That makes it an attention with one key/value head of
d = kv_rank + rot_dim (rounded up to a multiple of 32, of 16 beyond 128) entries: the key row is [c | rotated part | zeros],
the value row [c | zeros], and the attention is the kernels' that keep the softmax weights in float32 (the matrix-core kernel
of `kernels.headmix_attention` without mixing and sink, or the plain paged kernel).  Rotation: entry pairs (2i, 2i + 1), angle p * theta^(-2i/rot_dim),
formed in float32 in the kernel.

`q_rank` > 0: the queries pass a small row of their own first, q = W_uq RMSnorm(W_dq h) (weight, the layer's eps); the two
down projections are one product.  `sink`: every head's softmax denominator holds one more term exp(sink_h), a learned number
with no key and no value (float32).  `window` > 0: a query sees itself and the window - 1 tokens before it.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from .. import kernels
from ..cache.needs import PagedKV
from .base import BuildContext, Mixer, Param
from .linear import FusedLinear, Linear
from .registry import register_mixer
from .rotary import pair_frequencies


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    records_mixed_steps = True    # every index comes from the batch's device tensors

    def __init__(self, hidden_size: int, heads: int, head_dim: int, rotary_dim: int, value_dim: int, kv_rank: int, scale: float,
                 theta: float, eps: float, ctx: BuildContext, window: int = 0,
                 names: Sequence[str] = ("q", "dkv", "dkv.norm", "uk", "uv", "o"), suffix: str = "", whole_output: bool = False,
                 q_rank: int = 0, q_names: Sequence[str] = ("dq", "dq.norm", "uq"), sink: bool = False, sink_name: str = "sink"):
        self.H, self.dn, self.dr, self.dv, self.rank = int(heads), int(head_dim), int(rotary_dim), int(value_dim), int(kv_rank)
        if self.dr % 2:
            raise ValueError(f"{self.dr} rotated entries must be even")
        # the head size the attention runs: the next multiple of 32 up to 128 (the matrix-core kernel with float weights), of
        # 16 beyond
        need = self.rank + self.dr
        self.d = -(-need // 32) * 32 if need <= 128 else -(-need // 16) * 16
        self.scale, self.eps, self.window = float(scale), float(eps), int(window)
        self.whole_output = bool(whole_output)
        self.dtype = ctx.dtype
        qn, dn_, self.norm_name, ukn, uvn, on = names
        self.q_rank = int(q_rank)
        if self.q_rank:
            if self.dr:
                raise ValueError("queries through a low-rank row take no rotated entries")
            # [query row | latent row] from one product; the queries' second projection follows the row's norm
            self.proj = FusedLinear(hidden_size, [self.q_rank, self.rank], [q_names[0], dn_], False, ctx, suffix=suffix)
            self.q_norm_name = q_names[1]
            self.q_norm_w = torch.empty((self.q_rank,), dtype=ctx.dtype, device=ctx.device)
            self.uq = Linear(self.q_rank, self.H * self.dn, q_names[2], False, ctx, suffix=suffix)
        else:
            self.proj = FusedLinear(hidden_size, [self.H * (self.dn + self.dr), self.rank + self.dr], [qn, dn_], False, ctx, suffix=suffix)
        self.sink_name = sink_name
        self.sink = torch.empty((self.H,), dtype=torch.float32, device=ctx.device) if sink else None
        self.uk = Linear(self.rank, self.H * self.dn, ukn, False, ctx, suffix=suffix)    # [heads * dim, kv_rank]
        self.uv = Linear(self.rank, self.H * self.dv, uvn, False, ctx, suffix=suffix)    # [heads * vdim, kv_rank]
        self.o_proj = Linear(self.H * self.dv, hidden_size, on, False, ctx, suffix=suffix)
        self.norm_w = torch.empty((self.rank,), dtype=ctx.dtype, device=ctx.device)
        self.freq = pair_frequencies(self.dr, theta, ctx.device)

    def named_parameters(self) -> Dict[str, Param]:
        out = dict(self.proj.named_parameters())
        for part in (self.uk, self.uv, self.o_proj):
            out.update(part.named_parameters())
        out[self.norm_name] = Param(self.norm_w, neutral=1.0)
        if self.q_rank:
            out.update(self.uq.named_parameters())
            out[self.q_norm_name] = Param(self.q_norm_w, neutral=1.0)
        if self.sink is not None:
            out[self.sink_name] = Param(self.sink)
        return out

    def cache_need(self):
        return PagedKV(1, self.d, self.window)

    def forward(self, x, batch, view):
        H, dn, dr, dv, rank, d = self.H, self.dn, self.dr, self.dv, self.rank, self.d
        rows = self.proj.forward(x)                                         # [T, q heads | down]
        T = rows.shape[0]
        qx = torch.empty((T, H, d), dtype=rows.dtype, device=rows.device)   # the attention's queries [absorbed | rotated | zeros]
        if self.q_rank:
            kernels.latent_prep(rows, qx, batch.positions, None, self.norm_w, view.k, view.v, view.slots, H, dn, 0, rank, d, self.eps,
                                down_offset=self.q_rank)
            cq = kernels.group_norm_gate(rows[:, :self.q_rank], self.q_norm_w, self.eps, 1)
            q_plain = self.uq.forward(cq).view(T, H, dn)
        else:
            kernels.latent_prep(rows, qx, batch.positions, self.freq, self.norm_w, view.k, view.v, view.slots, H, dn, dr, rank, d, self.eps)
            q_plain = rows[:, :H * (dn + dr)].view(T, H, dn + dr)[:, :, :dn]
        kernels.head_gemm(q_plain, self.uk.weight.view(H, dn, rank), qx[:, :, :rank])          # q_h^T W_uk,h
        # bfloat16: the kernels that keep the softmax weights float32 up to the second product (the matrix-core kernel with
        # its two-term weights where the sizes fit, else the plain one); float32: everything is float anyway
        q2 = qx.view(T, H * d)
        if self.sink is not None or (rows.dtype == torch.bfloat16 and kernels.headmix_mfma_ok(H, 1, d, view.page_size, rows.dtype)):
            # (with a sink the plain kernel of this entry point serves what the matrix-core kernel does not: float32, other sizes)
            o = kernels.headmix_attention(q2, view.k, view.v, view.block_tables, batch.seg_of_token, batch.positions, H, 1, d, rank,
                                          self.scale, self.window, sink=self.sink, tiles=batch.att_tiles, single_rows=batch.att_single_rows,
                                          max_total_len=batch.max_total_len, seg_offsets=batch.seg_offsets)
        else:
            o = kernels.paged_attention(q2, view.k, view.v, view.block_tables, batch.seg_of_token, batch.positions, H, 1, d,
                                        self.scale, self.window, batch.max_total_len, batch.att_tiles, batch.att_single_rows,
                                        float_weights=True)
        y = torch.empty((T, H, dv), dtype=rows.dtype, device=rows.device)
        kernels.head_gemm(o.view(T, H, d)[:, :, :rank], self.uv.weight.view(H, dv, rank).transpose(1, 2), y)   # W_uv,h (sum_j p_j c_j)
        return self.o_proj.forward(y.view(T, H * dv), allow_parts=not self.whole_output)
