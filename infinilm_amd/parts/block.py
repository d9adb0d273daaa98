"""Arrangements: how a layer's parts are wired around the residual stream.

`pre_norm`: x += s * mixer(norm1(x)); x += s * ffn(norm2(x)), the reference's decoder layer
(csrc/models/minicpm4/minicpm4_for_causal_lm.cpp:49-71, csrc/layers/causal_lm_templates/
text_decoder_layer.hpp:39-61).  The adds are deferred into the next norm's kernel.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import LayerSpec
from .base import BuildContext, DeferredNorm, Param, ResidualStream, join_name
from .registry import ARRANGEMENTS, build_feed_forward, build_mixer, build_norm, register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock:
    slots = ("norm1", "mixer", "norm2", "ffn")

    def __init__(self, spec: LayerSpec, ctx: BuildContext):
        self.spec = spec
        self.norm1 = build_norm(spec.parts["norm1"], ctx)
        self.mixer = build_mixer(spec.parts["mixer"], ctx)
        self.norm2 = build_norm(spec.parts["norm2"], ctx)
        self.ffn = build_feed_forward(spec.parts["ffn"], ctx)
        self.residual_scale = float(spec.residual_scale)

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        for slot in self.slots:
            sub = self.spec.names[slot]
            for name, p in getattr(self, slot).named_parameters().items():
                out[join_name(self.spec.prefix, sub, name)] = p
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def records_mixed_steps(self) -> bool:
        return bool(getattr(self.mixer, "records_mixed_steps", False) and getattr(self.ffn, "records_mixed_steps", False))

    def forward(self, stream: ResidualStream, batch, cache_view) -> None:
        # a decode step of many rows: the mixer may take its rows in fragment order, which the norm then writes
        rows = stream.residual.shape[0]
        if (batch.taps is None and getattr(self.norm1, "takes_frag_request", False)
                and getattr(self.mixer, "takes_frag", lambda rows: False)(rows)):
            x = self.norm1.forward(stream, frag=True)
        else:
            x = self.norm1.forward(stream)
        # Few rows (decoded tokens): where the mixer's last projection, the second norm and the feed-forward
        # all can, the projection adds into the residual stream itself and the norm's kernel is not run
        # (see NormTail).  Not while intermediate values are dumped: they are taken between the kernels.
        tail = None
        if self.mixer.takes_tail and batch.taps is None:
            tail = self.norm2.tail(stream, self.residual_scale, x.shape[0])
            if tail is not None and not self.ffn.takes_deferred(x.shape[0]):
                tail = None
        y = self.mixer.forward(x, batch, cache_view) if tail is None else self.mixer.forward(x, batch, cache_view, tail=tail)
        if isinstance(y, DeferredNorm):
            x = y
        else:
            stream.push(y, self.residual_scale)
            x = self.norm2.forward(stream)
        stream.push(self.ffn.forward(x, batch), self.residual_scale)


@register_arrangement("sandwich_norm")
class SandwichNormBlock:
    """x += s * norm1b(mixer(norm1(x))); x += s * norm2b(ffn(norm2(x))): a norm before every sublayer and another on
    its output before the sum.  A layer may have no feed-forward (no `ffn`, `norm2`, `norm2b` among its parts).  A
    sublayer's output is left with the stream together with its norm (`ResidualStream.push_normed`): the next norm's
    kernel norms it, adds it to the float32 residual stream and norms the stream, in one pass."""

    def __init__(self, spec: LayerSpec, ctx: BuildContext):
        self.spec = spec
        self.slots = tuple(s for s in ("norm1", "mixer", "norm1b", "norm2", "ffn", "norm2b") if s in spec.parts)
        if not {"norm1", "mixer", "norm1b"} <= set(self.slots) or (("ffn" in self.slots) != ("norm2" in self.slots)) \
                or (("ffn" in self.slots) != ("norm2b" in self.slots)):
            raise ValueError(f"layer {spec.prefix}: a sandwich layer has norm1, mixer, norm1b and, with a feed-forward, norm2 and norm2b")
        self.norm1 = build_norm(spec.parts["norm1"], ctx)
        self.mixer = build_mixer(spec.parts["mixer"], ctx)
        self.norm1b = build_norm(spec.parts["norm1b"], ctx)
        self.ffn = self.norm2 = self.norm2b = None
        if "ffn" in self.slots:
            self.norm2 = build_norm(spec.parts["norm2"], ctx)
            self.ffn = build_feed_forward(spec.parts["ffn"], ctx)
            self.norm2b = build_norm(spec.parts["norm2b"], ctx)
        self.residual_scale = float(spec.residual_scale)

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        for slot in self.slots:
            for name, p in getattr(self, slot).named_parameters().items():
                out[join_name(self.spec.prefix, self.spec.names[slot], name)] = p
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def records_mixed_steps(self) -> bool:
        return bool(getattr(self.mixer, "records_mixed_steps", False)
                    and (self.ffn is None or getattr(self.ffn, "records_mixed_steps", False)))

    def forward(self, stream: ResidualStream, batch, cache_view) -> None:
        y = self.mixer.forward(self.norm1.forward(stream), batch, cache_view)
        stream.push_normed(y, self.norm1b, self.residual_scale)      # (normed and added inside the next norm's kernel)
        if self.ffn is not None:
            y = self.ffn.forward(self.norm2.forward(stream), batch)
            stream.push_normed(y, self.norm2b, self.residual_scale)


@register_arrangement("parallel_residual")
class ParallelResidualBlock:
    """x += s * (mixer(h) + ffn(h)) with h = norm1(x): one norm, and both sublayers read its output.  A layer may have no
    feed-forward.  Both outputs are left with the stream and summed into it inside the next norm's kernel."""

    def __init__(self, spec: LayerSpec, ctx: BuildContext):
        self.spec = spec
        self.slots = tuple(s for s in ("norm1", "mixer", "ffn") if s in spec.parts)
        if not {"norm1", "mixer"} <= set(self.slots):
            raise ValueError(f"layer {spec.prefix}: a parallel layer has norm1, mixer and, if any, ffn")
        self.norm1 = build_norm(spec.parts["norm1"], ctx)
        self.mixer = build_mixer(spec.parts["mixer"], ctx)
        self.ffn = build_feed_forward(spec.parts["ffn"], ctx) if "ffn" in self.slots else None
        self.residual_scale = float(spec.residual_scale)

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        for slot in self.slots:
            for name, p in getattr(self, slot).named_parameters().items():
                out[join_name(self.spec.prefix, self.spec.names[slot], name)] = p
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def records_mixed_steps(self) -> bool:
        return bool(getattr(self.mixer, "records_mixed_steps", False)
                    and (self.ffn is None or getattr(self.ffn, "records_mixed_steps", False)))

    def forward(self, stream: ResidualStream, batch, cache_view) -> None:
        h = self.norm1.forward(stream)
        stream.push(self.mixer.forward(h, batch, cache_view), self.residual_scale)
        if self.ffn is not None:
            stream.push_more(self.ffn.forward(h, batch), self.residual_scale)


@register_arrangement("gated_pre_norm")
class GatedPreNormBlock:
    """x += mixer(h) * sigmoid(W_g1 h + b_g1), h = norm1(x); x += ffn(h2) * sigmoid(W_g2 h2 + b_g2), h2 = norm2(x); then, if the
    layer has one, a side input from the token itself (`side_input.TokenSideInput`).  The gates read what their sublayer
    reads.  A layer may have no feed-forward (then no norm2 and no second gate), no gates, no side input.  A gated branch is
    left with the stream together with its gate rows (`ResidualStream.push_gated`): the next norm's kernel multiplies, adds
    and norms in one pass.  `gate1`, `gate2`: PartSpec("sigmoid_gate", {hidden_size, bias, bias_suffix}); `side`:
    PartSpec("token_side_input", {...})."""

    def __init__(self, spec: LayerSpec, ctx: BuildContext):
        from .linear import Linear
        from .side_input import TokenSideInput
        self.spec = spec
        self.slots = tuple(s for s in ("norm1", "mixer", "gate1", "norm2", "ffn", "gate2", "side") if s in spec.parts)
        if not {"norm1", "mixer"} <= set(self.slots) or (("ffn" in self.slots) != ("norm2" in self.slots)) \
                or ("gate2" in self.slots and "ffn" not in self.slots):
            raise ValueError(f"layer {spec.prefix}: a gated layer has norm1, mixer and, with a feed-forward, norm2")
        self.norm1 = build_norm(spec.parts["norm1"], ctx)
        self.mixer = build_mixer(spec.parts["mixer"], ctx)
        self.norm2 = build_norm(spec.parts["norm2"], ctx) if "norm2" in self.slots else None
        self.ffn = build_feed_forward(spec.parts["ffn"], ctx) if "ffn" in self.slots else None
        self.gates = {}
        for slot in ("gate1", "gate2"):
            if slot in self.slots:
                p = dict(spec.parts[slot].params)
                size = int(p["hidden_size"])
                lin = Linear(size, size, "", False, ctx, suffix="")
                bias = torch.empty((size,), dtype=ctx.dtype, device=ctx.device) if p.get("bias", True) else None
                self.gates[slot] = (lin, bias, p.get("bias_suffix", "bias"))
        self.side = TokenSideInput(ctx=ctx, **spec.parts["side"].params) if "side" in self.slots else None
        self.residual_scale = float(spec.residual_scale)

    def bind_shared(self, tensors) -> None:
        if self.side is not None:
            self.side.bind_shared(tensors)

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        for slot in self.slots:
            sub = self.spec.names[slot]
            if slot in self.gates:
                lin, bias, suffix = self.gates[slot]
                for name, p in lin.named_parameters().items():
                    out[join_name(self.spec.prefix, sub, name)] = p
                if bias is not None:
                    out[join_name(self.spec.prefix, sub, suffix)] = Param(bias)
                continue
            for name, p in getattr(self, slot).named_parameters().items():
                out[join_name(self.spec.prefix, sub, name)] = p
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def records_mixed_steps(self) -> bool:
        return bool(getattr(self.mixer, "records_mixed_steps", False)
                    and (self.ffn is None or getattr(self.ffn, "records_mixed_steps", False)))

    def _push(self, stream: ResidualStream, slot: str, h, y) -> None:
        if slot in self.gates:
            lin, bias, _ = self.gates[slot]
            stream.push_gated(y, lin.forward(h), bias, self.residual_scale)
        else:
            stream.push(y, self.residual_scale)

    def forward(self, stream: ResidualStream, batch, cache_view) -> None:
        h = self.norm1.forward(stream)
        self._push(stream, "gate1", h, self.mixer.forward(h, batch, cache_view))
        if self.ffn is not None:
            h = self.norm2.forward(stream)
            self._push(stream, "gate2", h, self.ffn.forward(h, batch))
        if self.side is not None:
            self.side.forward(stream, batch)


@register_arrangement("branch_norm")
class BranchNormBlock:
    """x += s * norm1(mixer(x)); x += s * norm2(ffn(x)): the sublayers read the residual stream itself (its rows in the
    activations' dtype), and the only norms stand on the sublayers' outputs.  A layer may have no feed-forward (then no
    `ffn` and no `norm2`).  A sublayer's output is left with the stream together with its norm (`push_normed`); the kernel that
    next reads the stream norms it, adds it and hands out the rows (`ResidualStream.rows`), in one pass."""

    def __init__(self, spec: LayerSpec, ctx: BuildContext):
        self.spec = spec
        self.slots = tuple(s for s in ("mixer", "norm1", "ffn", "norm2") if s in spec.parts)
        if not {"mixer", "norm1"} <= set(self.slots) or (("ffn" in self.slots) != ("norm2" in self.slots)):
            raise ValueError(f"layer {spec.prefix}: a layer with normed branches has mixer, norm1 and, with a feed-forward, norm2")
        self.mixer = build_mixer(spec.parts["mixer"], ctx)
        self.norm1 = build_norm(spec.parts["norm1"], ctx)
        self.ffn = build_feed_forward(spec.parts["ffn"], ctx) if "ffn" in self.slots else None
        self.norm2 = build_norm(spec.parts["norm2"], ctx) if "ffn" in self.slots else None
        self.residual_scale = float(spec.residual_scale)
        self.dtype = ctx.dtype

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        for slot in self.slots:
            for name, p in getattr(self, slot).named_parameters().items():
                out[join_name(self.spec.prefix, self.spec.names[slot], name)] = p
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def records_mixed_steps(self) -> bool:
        return bool(getattr(self.mixer, "records_mixed_steps", False)
                    and (self.ffn is None or getattr(self.ffn, "records_mixed_steps", False)))

    def forward(self, stream: ResidualStream, batch, cache_view) -> None:
        y = self.mixer.forward(stream.rows(self.dtype), batch, cache_view)
        stream.push_normed(y, self.norm1, self.residual_scale)
        if self.ffn is not None:
            y = self.ffn.forward(stream.rows(self.dtype), batch)
            stream.push_normed(y, self.norm2, self.residual_scale)


def build_block(spec: LayerSpec, ctx: BuildContext):
    try:
        cls = ARRANGEMENTS[spec.arrangement]
    except KeyError:
        raise KeyError(f"unknown arrangement {spec.arrangement!r}; registered: {sorted(ARRANGEMENTS)}") from None
    return cls(spec, ctx)
