"""Bebuzen: a decoder-only model whose sublayers read the residual stream itself and are RMS-normed on their way back into
it (x += m * norm1(mixer(x)); x += m * norm2(ff(x))), with three mixers a layer may pick (a differential attention with short
convolutions on q, k and v, rotate-half positions with scaled frequencies and a sliding window, which may read another
layer's keys and values; a selective scan with a state vector a channel; an attention with interleaved rotary pairs, a window
that keeps the sequence's first tokens and a unit term in every softmax denominator) and two feed-forwards (SwiGLU; routed
squared-relu experts with a softmax router beside a shared expert).  This file holds everything that is specific to the
design: config.json's keys, their validation, the tensor names and the description of the model as parts.  No part and no
kernel knows of it.

config.json:  architecture "Bebuzen"; vocab, width; norm {eps}; residual_mult (absent: 1);
  layers: a list of {type, mixer, mlp}
    type "attention":    mixer {heads, kv_heads, dim, vdim, scale, diff, conv (taps; absent: no convolution),
                                rot {base, dims, scaling {factor, low, high, original} | absent} | absent,
                                mask {size} | absent, kv_from: j | absent}
    type "attention_2":  mixer {heads, kv_heads, dim, vdim, scale, rot {base, dims, scaling | absent} | absent,
                                mask {size, keep_first | absent} | absent}
    type "mamba1":       mixer {inner, state, dt_rank, conv}
    mlp: null | {kind: "dense", ff} | {kind: "moe", router {experts, top, scale | absent}, expert {ff}, shared {ff} | absent}
Tensors (matrices stored [out, in]): embed, head, final.norm; l<i>.norm1, l<i>.norm2;
  attention:   l<i>.mix.{q, k, v} with .b and .conv, q.norm, k.norm, lq1, lk1, lq2, lk2, o   (no k, v tensors with kv_from)
  attention_2: l<i>.mix.{q, k, v, o} with .b, q.norm, k.norm
  mamba1:      l<i>.mix.{in, conv, conv.b, x, dt, dt.b, A_log, D, o}
  dense:       l<i>.mlp.{gate, up, down};   moe: l<i>.mlp.{router, e<j>.up, e<j>.down, shared.up, shared.down}
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.errors import ConfigError
from ..config.registry import register_architecture
from ..config.spec import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec
from .kekevik import _need

MAX_POSITIONS = 1 << 30      # the design sets no limit: angles are formed from the position in the kernels, no table


def rotary_frequencies(rot: Optional[Dict[str, Any]]) -> List[float]:
    """The turning rates f_i = base^(-2i/dims), i < dims / 2, in float64; with `scaling` (wavelength l = 2 pi / f): kept
    where l < original / high, divided by `factor` where l > original / low, and in between blended by
    s = (original / l - low) / (high - low) as (1 - s) f / factor + s f."""
    if not rot or not rot["dims"]:
        return []
    dims, base, sc = rot["dims"], rot["base"], rot.get("scaling")
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc is not None:
            wavelength = 2.0 * math.pi / f
            if wavelength > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            elif not wavelength < sc["original"] / sc["high"]:
                s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                f = (1.0 - s) * f / sc["factor"] + s * f
        out.append(f)
    return out


@dataclass
class BebuzenLayer:
    kind: str                        # attention | attention_2 | mamba1
    mixer: Dict[str, Any]            # the checked sizes and constants of its mixer
    mlp: Optional[Dict[str, Any]]    # None: no feed-forward; {"kind": "dense", "ff"} or {"kind": "moe", experts, top, scale, ff, shared_ff}


@dataclass
class BebuzenConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    layers: List[BebuzenLayer]
    dtype: Optional[str] = "bfloat16"
    eos_token_ids: List[int] = field(default_factory=list)
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "BebuzenConfig":
        vocab, width = _need(raw, "vocab", "config", int), _need(raw, "width", "config", int)
        eps = _need(raw.get("norm"), "eps", "config 'norm'")
        if eps < 0:
            raise ConfigError(f"norm.eps must not be negative, got {eps}")
        mult = _need(raw, "residual_mult", "config") if raw.get("residual_mult") is not None else 1.0
        entries = _need(raw, "layers", "config", list)
        if not entries:
            raise ConfigError("config 'layers' is empty")
        layers: List[BebuzenLayer] = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(e, "type", where, str)
            m = _need(e, "mixer", where, dict)
            mw = where + ".mixer"
            if kind in ("attention", "attention_2"):
                mixer = {k: _need(m, k, mw, int) for k in ("heads", "kv_heads", "dim", "vdim")}
                if mixer["heads"] % mixer["kv_heads"]:
                    raise ConfigError(f"{mw}: {mixer['heads']} query heads do not divide into {mixer['kv_heads']} key/value heads")
                mixer["scale"] = _need(m, "scale", mw)
                mixer["rot"] = _rot(m.get("rot"), mixer["dim"], mw + ".rot")
                mask = m.get("mask")
                mixer["window"] = _need(mask, "size", mw + ".mask", int) if mask is not None and mask.get("size") is not None else 0
                mixer["keep_first"] = 0
                if kind == "attention":
                    mixer["diff"] = _need(m, "diff", mw)
                    mixer["conv"] = _need(m, "conv", mw, int) if m.get("conv") is not None else 0
                    src = m.get("kv_from")
                    if src is not None:
                        if isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < i:
                            raise ConfigError(f"{mw}: kv_from must name an earlier layer, got {src!r}")
                        other = layers[src]
                        if other.kind != "attention" or other.mixer.get("kv_from") is not None:
                            raise ConfigError(f"{mw}: kv_from names layer {src}, which has no keys and values of this kind of its own")
                        for k in ("heads", "kv_heads", "dim", "vdim"):
                            if other.mixer[k] != mixer[k]:
                                raise ConfigError(f"{mw}: '{k}' is {mixer[k]}, but layer {src}, whose keys and values it reads, has {other.mixer[k]}")
                    mixer["kv_from"] = src
                elif mask is not None and mask.get("keep_first") is not None:
                    kf = mask["keep_first"]
                    if isinstance(kf, bool) or not isinstance(kf, int) or kf < 0:
                        raise ConfigError(f"Key 'keep_first' in {mw}.mask must be a non-negative integer, got {kf!r}")
                    mixer["keep_first"] = kf if mixer["window"] else 0
            elif kind == "mamba1":
                mixer = {k: _need(m, k, mw, int) for k in ("inner", "state", "dt_rank", "conv")}
            else:
                raise ConfigError(f"{where}: unknown layer type {kind!r} (attention, attention_2, mamba1)")
            mlp = e.get("mlp")
            ff = None
            if mlp is not None:
                fw = where + ".mlp"
                fkind = _need(mlp, "kind", fw, str)
                if fkind == "dense":
                    ff = {"kind": "dense", "ff": _need(mlp, "ff", fw, int)}
                elif fkind == "moe":
                    router, expert = _need(mlp, "router", fw, dict), _need(mlp, "expert", fw, dict)
                    ff = {"kind": "moe", "experts": _need(router, "experts", fw + ".router", int),
                          "top": _need(router, "top", fw + ".router", int),
                          "scale": _need(router, "scale", fw + ".router") if router.get("scale") is not None else 1.0,
                          "ff": _need(expert, "ff", fw + ".expert", int), "shared_ff": 0}
                    if ff["top"] > ff["experts"]:
                        raise ConfigError(f"{fw}.router: top {ff['top']} of {ff['experts']} experts")
                    if mlp.get("shared") is not None:
                        ff["shared_ff"] = _need(mlp["shared"], "ff", fw + ".shared", int)
                else:
                    raise ConfigError(f"{fw}: unknown kind {fkind!r} (dense, moe)")
            layers.append(BebuzenLayer(kind, mixer, ff))
        return cls(vocab=vocab, width=width, eps=eps, residual_mult=mult, layers=layers, raw=dict(raw))


def _rot(rot, dim: int, where: str) -> Optional[Dict[str, Any]]:
    if rot is None:
        return None
    dims = rot.get("dims")
    if isinstance(dims, bool) or not isinstance(dims, int) or dims < 0 or dims % 2 or dims > dim:
        raise ConfigError(f"Key 'dims' in {where} must be an even number of at most the head's {dim} entries, got {dims!r}")
    out = {"dims": dims, "base": _need(rot, "base", where), "scaling": None}
    sc = rot.get("scaling")
    if sc is not None:
        out["scaling"] = {k: _need(sc, k, where + ".scaling") for k in ("factor", "low", "high", "original")}
        if out["scaling"]["high"] == out["scaling"]["low"]:
            raise ConfigError(f"{where}.scaling: 'low' and 'high' must differ")
    return out


def build_spec(cfg: BebuzenConfig) -> ModelSpec:
    """embed[token] -> layers (x += m * norm1(mixer(x)), x += m * norm2(ff(x))) -> final norm -> head."""
    W = cfg.width

    def norm():
        return PartSpec("rmsnorm", {"size": W, "eps": cfg.eps, "param_name": ""})

    # the positions a differential layer's cache keeps: the widest window of the layers that read it (0: all)
    readers: Dict[int, List[int]] = {}
    for i, layer in enumerate(cfg.layers):
        if layer.kind == "attention":
            src = layer.mixer["kv_from"]
            readers.setdefault(i if src is None else src, []).append(layer.mixer["window"])
    layers, order, entry_of = [], [], {}
    n_entries = 0
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        borrows = None
        if layer.kind == "attention":
            src = m["kv_from"]
            windows = readers[i if src is None else src]
            mixer = PartSpec("differential_attention", {
                "hidden_size": W, "heads": m["heads"], "kv_heads": m["kv_heads"], "dim": m["dim"], "vdim": m["vdim"],
                "scale": m["scale"], "diff": m["diff"], "eps": cfg.eps, "window": m["window"],
                "cache_window": 0 if 0 in windows else max(windows), "conv_taps": m["conv"],
                "rotary_dim": m["rot"]["dims"] if m["rot"] else 0, "frequencies": rotary_frequencies(m["rot"]),
                "own_kv": src is None})
            has_cache = src is None or m["conv"] >= 1
            if src is not None:
                borrows = entry_of[src]
        elif layer.kind == "attention_2":
            rot = m["rot"]
            position = PartSpec("normed_pair_rotary", {"dim": m["dim"], "value_dim": m["vdim"], "rotary_dim": rot["dims"] if rot else 0,
                                                       "theta": rot["base"] if rot else 1.0, "eps": cfg.eps, "qk_norm": True,
                                                       "v_norm": False, "names": ("q.norm", "k.norm"),
                                                       "frequencies": rotary_frequencies(rot) if rot else None})
            mixer = PartSpec("gqa_attention", {
                "hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"], "qkv_bias": True,
                "out_bias": True, "scale": m["scale"], "window": m["window"], "position": position, "value_dim": m["vdim"],
                "names": ("q", "k", "v", "o"), "suffix": "", "bias_suffix": "b", "position_prefix": "",
                "keep_first": m["keep_first"], "fixed_sink": 0.0})
            has_cache = True
        else:
            mixer = PartSpec("selective_scan", {"hidden_size": W, "inner": m["inner"], "state": m["state"], "dt_rank": m["dt_rank"],
                                                "conv_taps": m["conv"]})
            has_cache = True
        parts = {"mixer": mixer, "norm1": norm()}
        names = {"mixer": "mix", "norm1": "norm1"}
        f = layer.mlp
        if f is not None:
            if f["kind"] == "dense":
                parts["ffn"] = PartSpec("swiglu", {"hidden_size": W, "intermediate_size": f["ff"], "bias": False,
                                                   "names": ("gate", "up", "down"), "suffix": ""})
            else:
                parts["ffn"] = PartSpec("routed_activation_experts", {
                    "hidden_size": W, "experts": f["experts"], "top": f["top"], "expert_ff": f["ff"], "router": "softmax",
                    "weight_scale": f["scale"], "activation": "relu2", "shared_ff": f["shared_ff"]})
            parts["norm2"] = norm()
            names.update({"ffn": "mlp", "norm2": "norm2"})
        layers.append(LayerSpec(prefix=f"l{i}", arrangement="branch_norm", parts=parts, names=names,
                                residual_scale=cfg.residual_mult))
        entry = None
        if has_cache:
            entry = entry_of[i] = n_entries
            n_entries += 1
        order.append(LayerRun(layer=i, cache=entry, writes_cache=True, borrows=borrows))
    spec = ModelSpec(architecture="Bebuzen", vocab_size=cfg.vocab, hidden_size=W, max_positions=MAX_POSITIONS, embed_name="",
                     embed_scale=1.0, layers=layers, order=order, final_norm=norm(), final_norm_name="final.norm",
                     head=HeadSpec(name="head", scale=1.0, tie_to_embedding_when_missing=False, params={"param_name": ""}),
                     eos_token_ids=list(cfg.eos_token_ids), embed_params={"param_name": "embed"})
    spec.validate()
    return spec


register_architecture(["Bebuzen", "bebuzen"], BebuzenConfig.from_dict, build_spec)
