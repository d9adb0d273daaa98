"""Patadra: a decoder-only model with learned position rows, pre-norm layers whose sublayers' results pass a sigmoid
gate on their way into the residual stream, an attention over latent rows (queries through a normed low-rank row, a
sliding window, a learned term in every head's softmax denominator), a feed-forward of many small experts with a
sigmoid router and a shared expert, a per-layer input from a second embedding table, RMS norms in groups, capped
logits, and a stretch of layers that may run several times in a row with the same weights.  This file holds everything
that is specific to the design: config.json's keys, their validation, the tensor names and the description of the model
as parts.  No part and no kernel knows of it.

config.json:  architecture "Patadra"; vocab, width, max_positions; norm {eps, groups}; logit_softcap (absent: no cap);
  token_side {dim} (absent: no per-layer token input);
  layers: a list of {type: "latent_attention",
                     mixer: {heads, dim, vdim, kv_rank, q_rank, scale, mask: {size} (absent: every earlier token is seen)},
                     mlp: null | {kind: "moe", router: {experts, top}, expert: {ff, limit}, shared: {ff, limit} | absent}}
  loop: {start, stop, times} or absent: layers start .. stop-1 run `times` times in a row, each pass with a cache of its own.
Tensors: embed, pos, side.embed, head, final.norm; l<i>.norm1, l<i>.norm2, l<i>.rg1, l<i>.rg1.b, l<i>.rg2, l<i>.rg2.b,
l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv, sink, o}, l<i>.mlp.{router, e<j>.gate, e<j>.up, e<j>.down,
shared.gate, shared.up, shared.down, shared.sg}, l<i>.side.{gate, proj, norm} (matrices stored [out, in]).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.errors import ConfigError
from ..config.registry import register_architecture
from ..config.spec import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec
from .kekevik import _need

EXPERT_SIGMOID_SLOPE = 1.702     # the experts' activation is g * sigmoid(1.702 g): fixed by the design


@dataclass
class PatadraLayer:
    mixer: Dict[str, Any]            # heads, dim, vdim, kv_rank, q_rank, scale, window (0: none)
    mlp: Optional[Dict[str, Any]]    # experts, top, ff, limit, shared_ff (0: none), shared_limit; None: no feed-forward


@dataclass
class PatadraConfig:
    vocab: int
    width: int
    max_positions: int
    eps: float
    groups: int
    layers: List[PatadraLayer]
    side_dim: int = 0                          # 0: no per-layer token input
    softcap: Optional[float] = None
    loop: Optional[Dict[str, int]] = None      # {start, stop, times}
    dtype: Optional[str] = "bfloat16"
    eos_token_ids: List[int] = field(default_factory=list)
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "PatadraConfig":
        vocab, width = _need(raw, "vocab", "config", int), _need(raw, "width", "config", int)
        max_positions = _need(raw, "max_positions", "config", int)
        norm = raw.get("norm")
        eps = _need(norm, "eps", "config 'norm'")
        if eps < 0:
            raise ConfigError(f"norm.eps must not be negative, got {eps}")
        groups = _need(norm, "groups", "config 'norm'", int) if norm.get("groups") is not None else 1
        if width % groups:
            raise ConfigError(f"norm.groups: rows of {width} do not divide into {groups} equal parts")
        entries = _need(raw, "layers", "config", list)
        if not entries:
            raise ConfigError("config 'layers' is empty")
        layers = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(e, "type", where, str)
            if kind != "latent_attention":
                raise ConfigError(f"{where}: unknown layer type {kind!r} (latent_attention)")
            m = _need(e, "mixer", where, dict)
            mw = where + ".mixer"
            mixer = {k: _need(m, k, mw, int) for k in ("heads", "dim", "vdim", "kv_rank", "q_rank")}
            mixer["scale"] = _need(m, "scale", mw)
            mask = m.get("mask")
            mixer["window"] = _need(mask, "size", mw + ".mask", int) if mask is not None and mask.get("size") is not None else 0
            mlp = e.get("mlp")
            ff = None
            if mlp is not None:
                fw = where + ".mlp"
                if mlp.get("kind", "moe") != "moe":
                    raise ConfigError(f"{fw}: unknown kind {mlp.get('kind')!r} (moe)")
                router, expert = _need(mlp, "router", fw, dict), _need(mlp, "expert", fw, dict)
                ff = {"experts": _need(router, "experts", fw + ".router", int), "top": _need(router, "top", fw + ".router", int),
                      "ff": _need(expert, "ff", fw + ".expert", int), "limit": _need(expert, "limit", fw + ".expert"),
                      "shared_ff": 0, "shared_limit": None}
                if ff["top"] > ff["experts"]:
                    raise ConfigError(f"{fw}.router: top {ff['top']} of {ff['experts']} experts")
                shared = mlp.get("shared")
                if shared is not None:
                    ff["shared_ff"] = _need(shared, "ff", fw + ".shared", int)
                    ff["shared_limit"] = _need(shared, "limit", fw + ".shared")
                for k in ("limit", "shared_limit"):
                    if ff[k] is not None and ff[k] <= 0:
                        raise ConfigError(f"{fw}: a limit must be positive, got {ff[k]}")
            layers.append(PatadraLayer(mixer, ff))
        side = raw.get("token_side")
        side_dim = _need(side, "dim", "config 'token_side'", int) if side is not None else 0
        cap = raw.get("logit_softcap")
        if cap is not None:
            cap = _need(raw, "logit_softcap", "config")
            if cap <= 0:
                raise ConfigError(f"logit_softcap must be positive, got {cap}")
        loop = raw.get("loop")
        if loop is not None:
            lw = "config 'loop'"
            times = _need(loop, "times", lw, int)
            start, stop = loop.get("start"), loop.get("stop")
            for k, v in (("start", start), ("stop", stop)):
                if isinstance(v, bool) or not isinstance(v, int):
                    raise ConfigError(f"Key '{k}' in {lw} must be an integer, got {v!r}")
            if not 0 <= start < stop <= len(layers):
                raise ConfigError(f"{lw}: layers {start} .. {stop - 1} are not a stretch of the {len(layers)} layers")
            loop = {"start": start, "stop": stop, "times": times}
        return cls(vocab=vocab, width=width, max_positions=max_positions, eps=eps, groups=groups, layers=layers,
                   side_dim=side_dim, softcap=cap, loop=loop, raw=dict(raw))


def run_order(n_layers: int, loop: Optional[Dict[str, int]]) -> List[int]:
    """The layers in the order they run: a looped stretch `times` times in a row."""
    if not loop:
        return list(range(n_layers))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n_layers))


def build_spec(cfg: PatadraConfig) -> ModelSpec:
    """embed[token] + pos[p] -> runs (x += mixer(h1) * sigmoid(gate1 h1), x += ff(h2) * sigmoid(gate2 h2), x += side(x, token))
    -> norm -> head -> cap."""
    W = cfg.width

    def norm():
        return PartSpec("group_rmsnorm", {"size": W, "eps": cfg.eps, "groups": cfg.groups, "param_name": ""})

    gate = PartSpec("sigmoid_gate", {"hidden_size": W, "bias": True, "bias_suffix": "b"})
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        parts = {"norm1": norm(),
                 "mixer": PartSpec("latent_attention", {"hidden_size": W, "heads": m["heads"], "head_dim": m["dim"], "rotary_dim": 0,
                                                        "value_dim": m["vdim"], "kv_rank": m["kv_rank"], "scale": m["scale"],
                                                        "theta": 1.0, "eps": cfg.eps, "window": m["window"], "q_rank": m["q_rank"],
                                                        "sink": True}),
                 "gate1": gate}
        names = {"norm1": "norm1", "mixer": "mix", "gate1": "rg1"}
        f = layer.mlp
        if f is not None:
            parts["norm2"] = norm()
            parts["ffn"] = PartSpec("routed_experts", {"hidden_size": W, "experts": f["experts"], "top": f["top"], "expert_ff": f["ff"],
                                                       "limit": f["limit"], "shared_ff": f["shared_ff"], "shared_limit": f["shared_limit"],
                                                       "alpha": EXPERT_SIGMOID_SLOPE})
            parts["gate2"] = gate
            names.update({"norm2": "norm2", "ffn": "mlp", "gate2": "rg2"})
        if cfg.side_dim:
            parts["side"] = PartSpec("token_side_input", {"hidden_size": W, "dim": cfg.side_dim, "first_column": i * cfg.side_dim,
                                                          "table": "side.embed", "eps": cfg.eps})
            names["side"] = "side"
        layers.append(LayerSpec(prefix=f"l{i}", arrangement="gated_pre_norm", parts=parts, names=names))
    # every run of a layer has a cache entry of its own
    order = [LayerRun(layer=i, cache=c, writes_cache=True) for c, i in enumerate(run_order(len(layers), cfg.loop))]
    head = HeadSpec(name="head", scale=1.0, tie_to_embedding_when_missing=False, params={"param_name": ""})
    if cfg.softcap is not None:
        head = HeadSpec(name="head", scale=1.0, tie_to_embedding_when_missing=False, kind="capped_linear",
                        params={"param_name": "", "cap": cfg.softcap})
    spec = ModelSpec(architecture="Patadra", vocab_size=cfg.vocab, hidden_size=W, max_positions=cfg.max_positions,
                     embed_name="", embed_scale=1.0, layers=layers, order=order, final_norm=norm(),
                     final_norm_name="final.norm", head=head, eos_token_ids=list(cfg.eos_token_ids),
                     embed_kind="positioned_lookup",
                     embed_params={"param_name": "embed", "position_name": "pos", "max_positions": cfg.max_positions},
                     shared_tensors={"side.embed": (cfg.vocab, len(layers) * cfg.side_dim)} if cfg.side_dim else None)
    spec.validate()
    return spec


register_architecture(["Patadra", "patadra"], PatadraConfig.from_dict, build_spec)
