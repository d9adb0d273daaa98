"""Grouped-query attention over the paged cache.

Reference: csrc/layers/attention/attention.cpp:96-137 (fused qkv projection -> heads -> rotation
of q and k in place -> backend -> o_proj), backends/paged_attn.cpp:20-84 (write k, v by slot, then
attention over the pages), backends/static_attn.cpp:82-99 (the formula: head h uses kv head
h // (nh/nkv), scores * scale, causal softmax, P V).  One contract serves prompts, portions of
prompts and single decoded tokens: a token at position p sees its request's keys [lo, p].
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from .. import kernels
from ..cache.needs import PagedKV
from ..config.spec import PartSpec
from .base import BuildContext, Mixer, Param, join_name
from .linear import FusedLinear, Linear
from .registry import build_position_encoding, register_mixer


@register_mixer("gqa_attention")
class GQAttention(Mixer):
    """`value_dim`: the size of a value head where it differs from the query and key heads'; `softcap` > 0: scaled
    scores pass through softcap * tanh(score / softcap); `names`, `suffix`: the projections' tensor names in a
    checkpoint; `whole_output`: the result comes as one [T, hidden] tensor in the activations' dtype (never as float32
    parts still to be summed), for an arrangement that does more with it than add it to the residual stream.

    The cache and the attention kernels know one head size: query/key heads and value heads of different sizes (or
    of a size that is no multiple of 16) are filled up with zeros to the next multiple of 16 that holds both, in the
    projections' weights: zero entries add nothing to a score, and the output entries they make meet zero columns
    of the output projection.

    `head_mix`: the scaled scores are mixed over the heads before the softmax, s_h = sum_g M[h, g] raw_g, with a tensor
    M [heads, heads]; `sink`: every head's softmax denominator holds one more term exp(sink_h), a tensor [heads] with no
    key and no value.  Both are float32 whatever the activations' dtype; `mix_names` are their tensor names.
    `position_prefix`: the sub-name under which the position encoding's own tensors lie ("": directly under the mixer's)."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, qkv_bias: bool,
                 out_bias: bool, scale: float, window: int, position: PartSpec, ctx: BuildContext,
                 value_dim: Optional[int] = None, softcap: float = 0.0,
                 names: Sequence[str] = ("q_proj", "k_proj", "v_proj", "o_proj"), suffix: str = "weight",
                 whole_output: bool = False, head_mix: bool = False, sink: bool = False,
                 mix_names: Sequence[str] = ("head_mix", "sink"), position_prefix: str = "position", bias_suffix: str = "bias",
                 keep_first: int = 0, fixed_sink: Optional[float] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} groups")
        self.nh, self.nkv = int(num_heads), int(num_kv_heads)
        self.dn = int(head_dim)                                       # entries of a query or key head that count
        self.dv = int(value_dim) if value_dim is not None else self.dn
        self.d = self.dn if self.dv == self.dn else -(-max(self.dn, self.dv) // 16) * 16   # the head size that runs
        self.scale = float(scale)
        self.softcap = float(softcap)
        self.window = int(window)
        self.whole_output = bool(whole_output)
        qn, kn, vn, on = names
        self.qkv = FusedLinear(hidden_size, [self.nh * self.d, self.nkv * self.d, self.nkv * self.d], [qn, kn, vn],
                               qkv_bias, ctx, suffix=suffix, bias_suffix=bias_suffix,
                               out_heads=[(self.nh, self.dn, self.d), (self.nkv, self.dn, self.d), (self.nkv, self.dv, self.d)])
        self.o_proj = Linear(self.nh * self.d, hidden_size, on, out_bias, ctx, suffix=suffix, bias_suffix=bias_suffix,
                             in_heads=(self.nh, self.dv, self.d))
        self.position = build_position_encoding(position, ctx)
        self.position_prefix = position_prefix
        self.mix_names = tuple(mix_names)
        self.head_mix = torch.empty((self.nh, self.nh), dtype=torch.float32, device=ctx.device) if head_mix else None
        self.sink = torch.empty((self.nh,), dtype=torch.float32, device=ctx.device) if sink else None
        # `fixed_sink`: the denominators' extra term is exp(fixed_sink) for every head, a constant of the design and no tensor
        # of a checkpoint (0.0: one is added to every denominator); `keep_first`: with a window, the sequence's first
        # that many tokens stay seen at their true positions however far the window has moved
        self.fixed_sink = None
        if fixed_sink is not None:
            if sink:
                raise ValueError("the denominators' extra term is learned or fixed, not both")
            self.fixed_sink = torch.full((self.nh,), float(fixed_sink), dtype=torch.float32, device=ctx.device)
        self.keep_first = int(keep_first) if self.window > 0 else 0
        if self.keep_first < 0:
            raise ValueError(f"{keep_first} kept first tokens")
        if getattr(self.position, "head_dim", self.d) not in (0, self.d):
            raise ValueError(f"the position encoding is made for heads of {self.position.head_dim}, the mixer's have {self.d}")

    def named_parameters(self) -> Dict[str, Param]:
        out = dict(self.qkv.named_parameters())
        out.update(self.o_proj.named_parameters())
        for name, p in self.position.named_parameters().items():   # an encoding may bring tensors of its own
            out[join_name(self.position_prefix, name)] = p
        if self.head_mix is not None:
            out[self.mix_names[0]] = Param(self.head_mix)
        if self.sink is not None:
            out[self.mix_names[1]] = Param(self.sink)
        return out

    def cache_need(self):
        return PagedKV(self.nkv, self.d, self.window, self.keep_first)

    takes_tail = True
    records_mixed_steps = True

    def takes_frag(self, rows: int) -> bool:
        fn = getattr(self.position, "takes_frag", None)
        return bool(fn is not None and fn(rows, self.qkv, self.nh, self.nkv, self.d))

    def forward(self, x, batch, cache_view, tail=None):
        pe = self.position
        pe.check(batch)
        qkv = None
        if batch.taps is None:   # (a dump of the rotated rows needs them in one piece)
            qkv = pe.project_encode_store(x, self.qkv, batch, cache_view, self.nh, self.nkv, self.d)
        if qkv is None:
            qkv = self.qkv.forward(x)
            pe.encode_and_store(qkv, batch, cache_view, self.nh, self.nkv, self.d)
            if batch.taps is not None:
                batch.taps.setdefault("qkv_rotated", []).append(qkv.clone())
        sink = self.sink if self.sink is not None else self.fixed_sink
        if self.head_mix is not None or sink is not None or self.keep_first:
            if self.softcap:
                raise ValueError("scores mixed over the heads take no cap")
            o = kernels.headmix_attention(qkv, cache_view.k, cache_view.v, cache_view.block_tables, batch.seg_of_token,
                                          batch.positions, self.nh, self.nkv, self.d, self.dv, self.scale, self.window,
                                          mix=self.head_mix, sink=sink, tiles=batch.att_tiles,
                                          single_rows=batch.att_single_rows, max_total_len=batch.max_total_len,
                                          seg_offsets=batch.seg_offsets, keep_first=self.keep_first)
        else:
            o = self._plain_attention(qkv, batch, cache_view)
        if tail is not None:   # the output projection adds into the residual stream itself, where its kernel can
            deferred = self.o_proj.forward_tail(o, tail)
            if deferred is not None:
                return deferred
        return self.o_proj.forward(o, allow_parts=not self.whole_output)

    def _plain_attention(self, qkv, batch, cache_view):
        o = kernels.paged_attention(qkv, cache_view.k, cache_view.v, cache_view.block_tables, batch.seg_of_token,
                                    batch.positions, self.nh, self.nkv, self.d, self.scale, self.window,
                                    batch.max_total_len, batch.att_tiles, batch.att_single_rows, softcap=self.softcap)
        return o
