"""Differential attention: every query head asks twice, and the second answer is taken off the first.

  q = W_q h + b_q  [heads x 2 x dim],  k = W_k h + b_k  [kv_heads x 2 x dim],  v = W_v h + b_v  [kv_heads x vdim]
        (head by head as [map 1 | map 2]; query head h reads key/value head h // (heads / kv_heads))
  a short causal convolution per channel of q, k and v (`conv_taps` inputs, the last the token's own, zeros before a
        sequence's start; no bias), whose last conv_taps - 1 inputs are part of the request's state
  q and k RMS-normed per head and map with one weight [dim] each, then the first `rotary_dim` entries of every map turned in
        the pairs (i, i + rotary_dim/2) by position x frequency_i
  a_m = softmax(scale q_m k_m^T over the last `window` positions, or all) v           both maps over the same values
  lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff;  o = a_1 - lambda a_2;  o / sqrt(mean(o^2) + eps) * (1 - diff) per head
  W_o on the heads side by side.

The cache holds a key/value head's two maps side by side as one key row of 2 dim entries, and its values once
(`PagedKV(kv_heads, d)`, d the next multiple of 16 that holds both).  A layer with `own_kv` false has no key and value tensors:
its run borrows the cache entry another layer's run writes (`LayerRun.borrows`) and attends over it with its own queries.
`cache_window`: the positions the cache keeps (the widest window of all layers that read it; 0: all).  Scores, softmax
weights, lambda and the norms are float32 whatever the activations' dtype.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from .. import kernels
from ..cache.manager import KVView, Lent
from ..cache.needs import FixedState, PagedKV
from .base import BuildContext, Mixer, Param
from .linear import FusedLinear, Linear
from .registry import register_mixer


@register_mixer("differential_attention")
class DifferentialAttention(Mixer):
    records_mixed_steps = True

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, diff: float, eps: float,
                 ctx: BuildContext, window: int = 0, cache_window: Optional[int] = None, conv_taps: int = 0, rotary_dim: int = 0,
                 frequencies: Optional[Sequence[float]] = None, own_kv: bool = True, qk_norm: bool = True,
                 names: Sequence[str] = ("q", "k", "v", "o", "conv", "norm", "lq1", "lk1", "lq2", "lk2"), bias_suffix: str = "b"):
        self.H, self.G, self.dim, self.vdim = int(heads), int(kv_heads), int(dim), int(vdim)
        if self.G <= 0 or self.H % self.G:
            raise ValueError(f"{heads} query heads do not divide into {kv_heads} groups")
        self.scale, self.diff, self.eps = float(scale), float(diff), float(eps)
        self.window = int(window)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        if self.cache_window and (self.window == 0 or self.window > self.cache_window):
            raise ValueError(f"a cache that keeps {self.cache_window} positions cannot serve a window of {self.window or 'all'}")
        self.taps = int(conv_taps)
        if self.taps < 0 or self.taps > kernels.CONV_MAX_TAPS:
            raise ValueError(f"{self.taps} taps: the convolution kernel takes up to {kernels.CONV_MAX_TAPS}")
        self.rd = int(rotary_dim)
        if self.rd % 2 or not 0 <= self.rd <= self.dim:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and at most the maps' size {dim}")
        if self.rd and (frequencies is None or len(frequencies) != self.rd // 2):
            raise ValueError(f"{self.rd // 2} frequencies are needed for {self.rd} turned entries")
        self.own_kv = bool(own_kv)
        self.d = -(-max(2 * self.dim, self.vdim) // 16) * 16            # the cache's head size
        self.names = tuple(names)
        qn, kn, vn, on, cn, nn = self.names[:6]
        self.dtype = ctx.dtype
        dev = ctx.device
        self.Cq, self.Ck, self.Cv = self.H * 2 * self.dim, self.G * 2 * self.dim, self.G * self.vdim
        sizes, pnames = [self.Cq], [qn]
        if self.own_kv:
            sizes += [self.Ck, self.Cv]
            pnames += [kn, vn]
        self.C = sum(sizes)
        self.proj_names = pnames
        self.qkv = FusedLinear(hidden_size, sizes, pnames, True, ctx, suffix="", bias_suffix=bias_suffix)
        self.o_proj = Linear(self.H * self.vdim, hidden_size, on, False, ctx, suffix="")
        self.conv_w = torch.empty((self.C, self.taps), dtype=ctx.dtype, device=dev) if self.taps else None
        self.q_norm = torch.empty((self.dim,), dtype=ctx.dtype, device=dev) if qk_norm else None
        self.k_norm = torch.empty((self.dim,), dtype=ctx.dtype, device=dev) if qk_norm and self.own_kv else None
        self.lam = [torch.empty((self.dim,), dtype=ctx.dtype, device=dev) for _ in range(4)]
        self.freq = (torch.tensor(list(frequencies), dtype=torch.float64).to(torch.float32).to(dev) if self.rd else None)

    def named_parameters(self) -> Dict[str, Param]:
        qn, kn, vn, on, cn, nn = self.names[:6]
        out = dict(self.qkv.named_parameters())
        out.update(self.o_proj.named_parameters())
        if self.taps:
            row = 0
            for name, size in zip(self.proj_names, self.qkv.out_sizes):
                out[f"{name}.{cn}"] = Param(self.conv_w[row:row + size])
                row += size
        if self.q_norm is not None:
            out[f"{qn}.{nn}"] = Param(self.q_norm, neutral=1.0)
        if self.k_norm is not None:
            out[f"{kn}.{nn}"] = Param(self.k_norm, neutral=1.0)
        for name, t in zip(self.names[6:10], self.lam):
            out[name] = Param(t)
        return out

    def _conv_state(self):
        return FixedState((self.taps - 1, self.C), torch.float32) if self.taps >= 1 else None

    def borrowed_need(self):
        """What a layer without keys and values of its own reads of the cache entry it borrows."""
        return None if self.own_kv else PagedKV(self.G, self.d, self.cache_window)

    def cache_need(self):
        state = self._conv_state()
        if not self.own_kv:
            return state
        kv = PagedKV(self.G, self.d, self.cache_window)
        return kv if state is None else (kv, state)

    def forward(self, x, batch, view):
        lent = None
        if isinstance(view, Lent):
            view, lent = view.own, view.lent
        members = view if isinstance(view, tuple) else (view,)
        kv = next((m for m in members if isinstance(m, KVView)), None)
        conv = next((m for m in members if m is not None and not isinstance(m, KVView)), None)
        if not self.own_kv:
            borrowed = lent if isinstance(lent, tuple) else (lent,)
            kv = next((m for m in borrowed if isinstance(m, KVView)), None)
        if kv is None:
            raise RuntimeError("the differential attention got no keys and values to attend over")
        u = self.qkv.forward(x)                                   # [T, q | k | v]
        if self.taps >= 1:
            u = kernels.causal_conv(u, self.conv_w, None, conv.pool, conv.state_in, conv.state_out, batch.seg_of_token,
                                    batch.seg_offsets, conv.state_in.numel(), "none")       # float32
        k_off = self.Cq if self.own_kv else -1
        slots = kv.slots if self.own_kv else None
        has_runs = batch.att_tiles is not None and batch.att_tiles.numel() > 0
        if has_runs and kernels.maps_mfma_ok(self.H, self.G, self.dim, self.vdim, self.d, kv.k.shape[2], self.dtype):
            # bfloat16, portions of prompts, at the two-maps matrix-core kernel's sizes: both maps of a head in one pass over
            # the keys, combined and normed in the kernel's epilogue
            q = kernels.maps_norm_rope_kvwrite(u, 0, k_off, self.Cq + self.Ck, batch.positions, self.freq, self.q_norm, self.k_norm,
                                               kv.k, kv.v, slots, self.H, self.G, 2, self.dim, self.vdim, self.rd, self.eps, self.dtype)
            o = kernels.maps_attention_tiles(q, kv.k, kv.v, kv.block_tables, batch.seg_of_token, batch.positions, self.H, self.G,
                                             self.dim, self.vdim, self.scale, self.window, self.lam, self.diff, self.eps,
                                             1.0 - self.diff, tiles=batch.att_tiles, single_rows=batch.att_single_rows,
                                             seg_offsets=batch.seg_offsets)
        elif kernels.headmix_mfma_ok(2 * self.H, self.G, self.d, kv.k.shape[2], self.dtype):
            # bfloat16 at the matrix-core kernel's sizes: every (head, map) asks as a head of its own, with a query that is zeros
            # outside its map's part of the key row; the two results come back in float32 and are combined and normed there
            qx = kernels.maps_norm_rope_kvwrite(u, 0, k_off, self.Cq + self.Ck, batch.positions, self.freq, self.q_norm, self.k_norm,
                                                kv.k, kv.v, slots, self.H, self.G, 2, self.dim, self.vdim, self.rd, self.eps, self.dtype,
                                                spread=True)
            a = kernels.headmix_attention(qx, kv.k, kv.v, kv.block_tables, batch.seg_of_token, batch.positions, 2 * self.H, self.G,
                                          self.d, self.vdim, self.scale, self.window, tiles=batch.att_tiles,
                                          single_rows=batch.att_single_rows, max_total_len=batch.max_total_len,
                                          seg_offsets=batch.seg_offsets, spread_queries=True, out_dtype=torch.float32)
            o = kernels.maps_combine(a, self.H, self.vdim, self.dim, self.lam, self.diff, self.eps, 1.0 - self.diff, self.dtype)
        else:
            q = kernels.maps_norm_rope_kvwrite(u, 0, k_off, self.Cq + self.Ck, batch.positions, self.freq, self.q_norm, self.k_norm,
                                               kv.k, kv.v, slots, self.H, self.G, 2, self.dim, self.vdim, self.rd, self.eps, self.dtype)
            o = kernels.maps_attention(q, kv.k, kv.v, kv.block_tables, batch.seg_of_token, batch.positions, self.H, self.G, 2, self.dim,
                                       self.vdim, self.scale, self.window, 0, None, self.lam, self.diff, self.eps, 1.0 - self.diff)
        return self.o_proj.forward(o, allow_parts=True)
