"""Interfaces of the parts a layer is put together from.

A part is built from its `PartSpec.params` (sizes and constants) and a `BuildContext` (dtype and
device); it owns its tensors and says under which names they lie in a checkpoint.  No part knows
which model it is in.

  Norm             forward(stream)                 folds the pending branch into the residual
                                                   stream and returns the normed activations
  Mixer            cache_need() -> PagedKV | FixedState | None
                   forward(x, batch, cache_view)   x [T, hidden] -> [T, hidden]; reads what it
                                                   needs of the batch (segments, positions) and
                                                   of its cache view
  FeedForward      forward(x, batch)               x [T, hidden] -> [T, hidden]
  PositionEncoding encode_and_store(qkv, batch, view, nh, nkv, d)   called by mixers: positions into
                                                   q and k, encoded k and v into the cache
  Arrangement      forward(stream, batch, cache_view)  wires the slots around the residual stream
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Optional

import torch


@dataclass
class BuildContext:
    dtype: torch.dtype
    device: torch.device


class Param:
    """A named tensor of a part.  `tensor` is where the loader copies to (it may be a view into a
    fused buffer).  `keep_f32`: a tensor stored in 32-bit in the checkpoint stays 32-bit even when
    the model runs in bfloat16 (the part's kernels take both).  `neutral`: the value at which the
    tensor does nothing (1.0 for a norm's gain, 0.0 for matrices and biases); random weights may be
    drawn around it."""

    def __init__(self, tensor: torch.Tensor, keep_f32: bool = False,
                 replace: Optional[Callable[[torch.Tensor], None]] = None, neutral: float = 0.0,
                 shape: Optional[tuple] = None):
        self.tensor = tensor
        self.keep_f32 = keep_f32 and replace is not None
        self._replace = replace
        self.neutral = float(neutral)
        # the tensor's shape in a checkpoint; `tensor` may be a strided view of the same elements in another shape
        # (heads filled up with zeros to a size the kernels take)
        self.shape = tuple(shape) if shape is not None else tuple(tensor.shape)
        if shape is not None and self.keep_f32:
            raise ValueError("a parameter stored through a view cannot be replaced")

    def replace(self, t: torch.Tensor) -> None:
        self._replace(t)
        self.tensor = t

    def store(self, t: torch.Tensor) -> None:
        """Copies a checkpoint's tensor (of shape `shape`) into the parameter."""
        self.tensor.copy_(t.to(self.tensor.dtype).reshape(self.tensor.shape))


def join_name(*pieces: str) -> str:
    """Pieces of a tensor's name joined by dots; empty pieces are left out (a part whose one tensor carries the
    part's own name gives it the name "")."""
    return ".".join(p for p in pieces if p)


class Part:
    def named_parameters(self) -> Dict[str, Param]:
        return {}


class ResidualStream:
    """The residual stream in float32 and the branch output that is still to be added to it.
    The sum `residual += scale * pending` happens inside the next norm's kernel.  `pending` is
    [T, hidden] or, from a product that was split over K, float32 parts [P, T, hidden]."""

    def __init__(self, residual: torch.Tensor):
        self.residual = residual
        self.pending: Optional[torch.Tensor] = None
        self.pending_scale: float = 1.0
        # a branch that is still to be normed by `pending_norm` before it is added (an arrangement with a norm on every
        # sublayer's output): a norm that knows how does both in its own kernel, anybody else calls `settle()` first
        self.pending_norm = None
        # further addends (tensor, scale) that are due to the stream beside `pending`: a second branch that read the same
        # norm's output, a copy of the embedding's output, one row for all tokens.  A norm that knows how sums them in its
        # own kernel; anybody else calls `settle()` first
        self.more: list = []
        # a branch that is still to be multiplied element by element by sigmoid(gate rows + bias) before it is added:
        # (gate rows [T, hidden], bias [hidden] or None); a norm that knows how does it in its own kernel, `settle()` for
        # anybody else
        self.pending_gate = None

    def push_gated(self, branch: torch.Tensor, gate: torch.Tensor, gate_bias, scale: float = 1.0) -> None:
        """`branch` joins the stream as branch * sigmoid(gate + gate_bias) * scale when the stream is next read."""
        self.push(branch, scale)
        self.pending_gate = (gate, gate_bias)

    def rows(self, dtype: torch.dtype) -> torch.Tensor:
        """Everything that is due summed into the stream, and its rows as `dtype` (float32: the stream's own tensor) for a
        part that reads the stream itself and not a norm's output."""
        from .. import kernels
        if self.more:
            self.settle()
        out_dtype = None if dtype == torch.float32 else dtype
        if self.pending is None:
            x = kernels.stream_update(self.residual, out_dtype=out_dtype)
        elif self.pending_gate is not None:
            x = kernels.stream_update(self.residual, self.pending, self.pending_scale, gate=self.pending_gate[0],
                                      gate_bias=self.pending_gate[1], out_dtype=out_dtype)
        elif self.pending_norm is not None and hasattr(self.pending_norm, "weight") and getattr(self.pending_norm, "groups", 1) == 1:
            x = kernels.stream_update(self.residual, self.pending, self.pending_scale, branch_weight=self.pending_norm.weight,
                                      branch_eps=self.pending_norm.eps, out_dtype=out_dtype)
        else:
            self.settle()
            x = kernels.stream_update(self.residual, self.pending, self.pending_scale, out_dtype=out_dtype)
        self.pending, self.pending_scale, self.pending_norm, self.pending_gate = None, 1.0, None, None
        return self.residual if x is None else x

    def push_more(self, addend: torch.Tensor, scale: float = 1.0) -> None:
        """`addend` ([T, hidden], float32 parts [P, T, hidden], or one row [hidden] for every token) times `scale` joins
        the stream when it is next read."""
        self.more.append((addend, float(scale)))

    def push(self, branch: torch.Tensor, scale: float) -> None:
        if self.pending is not None:
            raise RuntimeError("a branch is already pending; a norm must fold it first")
        self.pending = branch
        self.pending_scale = scale

    def push_normed(self, branch: torch.Tensor, norm, scale: float) -> None:
        """`branch` ([T, hidden], or float32 parts [P, T, hidden] of a product split over K) joins the stream as
        norm(branch) * scale; the norm is applied when the stream is next read."""
        self.push(branch, scale)
        self.pending_norm = norm

    def settle(self) -> None:
        """Applies a norm that is still due to the pending branch, so that `pending` is what is added."""
        if self.pending_norm is not None:
            norm, self.pending_norm = self.pending_norm, None
            self.pending = norm.apply(self.pending)
        if self.pending_gate is not None:     # the gated branch goes into the stream now
            from .. import kernels
            (gate, bias), self.pending_gate = self.pending_gate, None
            kernels.stream_update(self.residual, self.pending, self.pending_scale, gate=gate, gate_bias=bias)
            self.pending, self.pending_scale = None, 1.0
        if self.more:
            from .. import kernels
            more, self.more = self.more, []
            kernels.add_layernorm(self.residual, more, None, None, 0.0, torch.float32)


@dataclass
class NormTail:
    """An offer to the part before a norm (an arrangement makes it when the norm, the part before and
    the part after all can): add your branch into `residual` yourself (times `scale`) and return a
    `DeferredNorm` instead of the branch; the norm's kernel is then not run."""
    residual: torch.Tensor      # float32 [T, hidden], updated in place
    scale: float
    weight: torch.Tensor        # the norm's weight
    eps: float


@dataclass
class DeferredNorm:
    """A norm's output up to one number a row: `x` = residual * weight in the activations' dtype, and
    partial sums of squares of the residual's rows (`sumsq` [tiles, 32]), from which the consumer
    forms 1 / sqrt(mean square + eps) and applies it to its own sums."""
    x: torch.Tensor
    sumsq: torch.Tensor
    eps: float


class Norm(Part):
    """`takes_frag_request`: forward accepts `frag=True` and then returns its rows in fragment order
    (`kernels.FragRows`) for a consumer that said `takes_frag(rows)`."""
    takes_frag_request = False

    def forward(self, stream: ResidualStream) -> torch.Tensor:
        raise NotImplementedError

    def tail(self, stream: ResidualStream, scale: float, rows: int) -> Optional[NormTail]:
        """The offer for the part before this norm, or None (see NormTail)."""
        return None


class Mixer(Part):
    """`takes_tail`: forward accepts `tail=NormTail` and may answer with a DeferredNorm."""
    takes_tail = False
    # True: forward takes every index from the batch's device tensors also in steps that hold portions of prompts
    # (never from the host copies `h_*`), so that such steps can be recorded and replayed for other requests
    records_mixed_steps = False

    def takes_frag(self, rows: int) -> bool:
        """Whether forward accepts x as `kernels.FragRows` (rows in fragment order) for a step of `rows` rows."""
        return False

    def cache_need(self):
        return None

    def forward(self, x: torch.Tensor, batch, cache_view) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    records_mixed_steps = False   # as for a mixer: nothing in forward depends on the host's view of the batch

    def takes_deferred(self, rows: int) -> bool:
        """Whether forward accepts a DeferredNorm of `rows` rows as x."""
        return False

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions enter a mixer's queries and keys.  A mixer holds one, calls the three methods
    below and never looks inside (tables, angles and kernels are the encoding's own), so another
    encoding is a class of its own and no change to a mixer.

      max_positions   positions from here on are refused (`check`)
      encode_and_store(qkv, batch, view, nh, nkv, d)
                      encodes `batch.positions` (or whatever of `batch` it reads) into the q and k heads
                      of the fused projection rows qkv [T, (nh + 2 nkv) d], in place, and writes the
                      encoded k and the v into the cache view (`view.k`, `view.v` at `view.slots`;
                      nothing is written when `view.slots` is None).  The write belongs here because
                      the kernel that touches k anyway does it in the same pass.
      project_encode_store(x, proj, batch, view, nh, nkv, d) -> q or None
                      optional short cut: projection, encoding and cache write in one kernel for the
                      shapes an encoding has one for; returns the encoded queries [T, nh d], or None,
                      after which the mixer runs `proj.forward(x)` and `encode_and_store`.
    An encoding that cannot be written as a change of q and k (a bias on the scores) needs a mixer
    that asks for it; the mixers here do not."""

    max_positions: int = 1 << 30

    def check(self, batch) -> None:
        if batch.max_position >= self.max_positions:
            raise ValueError(f"position {batch.max_position} is beyond the position encoding's {self.max_positions}")

    def project_encode_store(self, x, proj, batch, view, nh: int, nkv: int, d: int):
        return None

    def encode_and_store(self, qkv, batch, view, nh: int, nkv: int, d: int) -> None:
        raise NotImplementedError
