"""A plain, slow implementation of the Patadra design: whole sequences at once, one function per mechanism, in torch on
the CPU (float64 unless told otherwise).  It shares no code with the engine and is what the tests compare the engine with.

Notation: h is a sublayer's input row, p a token's position in its sequence (from 0), W x a stored [out, in] matrix
applied to a column.  `cfg` is config.json as a dict, `w` the tensors by name.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


_ROUND = [None]    # the dtype that projections round their operands and results to (`forward(round_to=...)`)


def _r(x: torch.Tensor) -> torch.Tensor:
    return x if _ROUND[0] is None else x.to(_ROUND[0]).to(x.dtype)


def proj(h: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None, exact: bool = False) -> torch.Tensor:
    """W h (+ b).  Under `round_to` the operands and the result are rounded (`exact`: only the operands, for a product whose
    result stays in 32-bit, as a router's)."""
    y = _r(h) @ _r(w).T
    if b is not None:
        y = y + b
    return y if exact else _r(y)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * weight


def grouped_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, groups: int) -> torch.Tensor:
    """Every row in `groups` consecutive equal parts, each of unit root mean square by itself; then the weight."""
    T, n = x.shape
    return (unit_rms(x.reshape(T, groups, n // groups), eps).reshape(T, n)) * weight


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def model_norm(cfg: dict, x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    return grouped_rms_norm(x, weight, cfg["norm"]["eps"], int(cfg["norm"].get("groups", 1)))


def visible(T: int, window: Optional[int]) -> torch.Tensor:
    """[T, T] True where query i may look at key j: j <= i, and with a window i - j < window."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok &= (i - j) < window
    return ok


def latent_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    """Queries through a normed low-rank row, keys and values made per head from one normed latent row a token, a
    sliding window, and a learned term exp(sink) of every head in the softmax's denominator that has no value."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    cq = rms_norm(proj(h, w[pre + ".dq"]), w[pre + ".dq.norm"], eps)
    q = proj(cq, w[pre + ".uq"]).view(T, H, dk)
    c = rms_norm(proj(h, w[pre + ".dkv"]), w[pre + ".dkv.norm"], eps)
    k = proj(c, w[pre + ".uk"]).view(T, H, dk)
    v = proj(c, w[pre + ".uv"]).view(T, H, dv)
    window = (m.get("mask") or {}).get("size")
    ok = visible(T, window)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    s = s.masked_fill(~ok[None], float("-inf"))
    sink = w[pre + ".sink"].to(h.dtype)                       # [H]
    top = torch.maximum(s.max(-1).values, sink[:, None])      # [H, T]
    e = torch.exp(s - top[..., None])
    den = e.sum(-1) + torch.exp(sink[:, None] - top)
    o = torch.einsum("hij,jhd->ihd", e / den[..., None], v)
    return proj(o.reshape(T, H * dv), w[pre + ".o"])


def expert(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, limit: float) -> torch.Tensor:
    g = torch.clamp(proj(h, w[pre + ".gate"]), max=limit)
    u = torch.clamp(proj(h, w[pre + ".up"]), min=-limit, max=limit)
    return proj(g * sigmoid(1.702 * g) * (u + 1.0), w[pre + ".down"])


def routed_feed_forward(h: torch.Tensor, mlp: dict, w: Dict[str, torch.Tensor], pre: str, chosen: Optional[list] = None,
                        forced: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Each token goes to the `top` experts with the largest sigmoid(router) scores; an expert sees the token's row times
    its score (not renormalised) and the outputs are summed.  A shared expert, if any, sees every row and is weighed by
    one sigmoid number a token.  `chosen` receives (the experts picked here [T, top], the scores [T, n]); `forced` [T, top]
    replaces the pick (for a comparison with a computation that rounds, where two nearly equal scores may change places)."""
    n, top = mlp["router"]["experts"], mlp["router"]["top"]
    score = sigmoid(proj(h, w[pre + ".router"], exact=True))    # [T, n]
    pick = torch.topk(score, top, dim=-1).indices               # [T, top]
    if chosen is not None:
        chosen.append((pick, score))
    if forced is not None:
        pick = torch.as_tensor(forced, dtype=torch.long)
    y = torch.zeros_like(h)
    for e in range(n):
        for slot in range(top):
            rows = (pick[:, slot] == e).nonzero().flatten()
            if rows.numel():
                y[rows] += expert(h[rows] * score[rows, e][:, None], w, f"{pre}.e{e}", mlp["expert"]["limit"])
    if mlp.get("shared"):
        y = y + expert(h, w, pre + ".shared", mlp["shared"]["limit"]) * sigmoid(proj(h, w[pre + ".shared.sg"], exact=True))
    return y


def token_side(x: torch.Tensor, tokens: torch.Tensor, w: Dict[str, torch.Tensor], layer: int, dim: int, eps: float) -> torch.Tensor:
    """What a layer adds to the stream from the token itself: a slice of a second embedding table, gated by the stream."""
    e = w["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(proj(x, w[f"l{layer}.side.gate"])) * e
    y = proj(g, w[f"l{layer}.side.proj"])
    return rms_norm(y, w[f"l{layer}.side.norm"], eps)


def run_order(cfg: dict) -> List[int]:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def layer(cfg: dict, w: Dict[str, torch.Tensor], i: int, x: torch.Tensor, tokens: torch.Tensor, chosen: Optional[list] = None,
          forced: Optional[torch.Tensor] = None) -> torch.Tensor:
    L = cfg["layers"][i]
    eps = cfg["norm"]["eps"]
    h = model_norm(cfg, x, w[f"l{i}.norm1"])
    y = latent_attention(h, L["mixer"], w, f"l{i}.mix", eps)
    x = x + y * sigmoid(proj(h, w[f"l{i}.rg1"], w[f"l{i}.rg1.b"]))
    if L.get("mlp"):
        h = model_norm(cfg, x, w[f"l{i}.norm2"])
        y = routed_feed_forward(h, L["mlp"], w, f"l{i}.mlp", chosen=chosen, forced=forced)
        x = x + y * sigmoid(proj(h, w[f"l{i}.rg2"], w[f"l{i}.rg2.b"]))
    side = cfg.get("token_side")
    if side:
        x = x + token_side(x, tokens, w, i, side["dim"], eps)
    return x


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens, dtype=torch.float64, round_to=None,
            layers_out: Optional[list] = None, chosen: Optional[list] = None, forced: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  `round_to`: projections take operands and give results rounded to that dtype
    (what a bfloat16 engine does at its matrix products), everything else stays in `dtype`.  `chosen` receives, for every run
    of a layer with experts in the order of the runs, (picked experts, scores); `forced`: the picks to use instead, one
    [T, top] tensor for each such run."""
    _ROUND[0] = round_to
    try:
        return _forward(cfg, w, tokens, dtype, layers_out, chosen, forced)
    finally:
        _ROUND[0] = None


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt, n: int) -> List[int]:
    """The n tokens greedy decoding appends to `prompt` (the whole sequence is run again for every token)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]


def _forward(cfg, w, tokens, dtype, layers_out, chosen=None, forced=None):
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.numel()
    x = w["embed"][tokens] + w["pos"][:T]
    forced = list(forced) if forced is not None else None
    for i in run_order(cfg):
        f = forced.pop(0) if forced is not None and cfg["layers"][i].get("mlp") else None
        x = layer(cfg, w, i, x, tokens, chosen=chosen, forced=f)
        if layers_out is not None:
            layers_out.append(x.clone())
    z = proj(model_norm(cfg, x, w["final.norm"]), w["head"], exact=True)
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * torch.tanh(z / cap)
    return z


# ---- shapes and random weights ---------------------------------------------------------------------------------------
def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    V, W = cfg["vocab"], cfg["width"]
    out = {"embed": (V, W), "pos": (cfg["max_positions"], W), "final.norm": (W,), "head": (V, W)}
    side = cfg.get("token_side")
    if side:
        out["side.embed"] = (V, len(cfg["layers"]) * side["dim"])
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        H, dk, dv, r, rq = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        p = f"l{i}."
        out.update({p + "norm1": (W,), p + "mix.dq": (rq, W), p + "mix.dq.norm": (rq,), p + "mix.uq": (H * dk, rq),
                    p + "mix.dkv": (r, W), p + "mix.dkv.norm": (r,), p + "mix.uk": (H * dk, r), p + "mix.uv": (H * dv, r),
                    p + "mix.sink": (H,), p + "mix.o": (W, H * dv), p + "rg1": (W, W), p + "rg1.b": (W,)})
        mlp = L.get("mlp")
        if mlp:
            out.update({p + "norm2": (W,), p + "rg2": (W, W), p + "rg2.b": (W,), p + "mlp.router": (mlp["router"]["experts"], W)})
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                out.update({f"{p}mlp.e{e}.gate": (ff, W), f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (fs, W), p + "mlp.shared.up": (fs, W), p + "mlp.shared.down": (W, fs),
                            p + "mlp.shared.sg": (1, W)})
        if side:
            out.update({p + "side.gate": (side["dim"], W), p + "side.proj": (W, side["dim"]), p + "side.norm": (W,)})
    return out


def random_weights(cfg: dict, seed: int, store: torch.dtype = torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors (rounded to `store`, returned as float32): matrices of about unit gain, norm weights around 1,
    sinks and biases of order 1, so that every mechanism moves the logits."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm", "norm1", "norm2"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last in ("sink", "b"):
            t = torch.randn(shape, generator=g)
        elif name in ("embed", "pos", "side.embed"):
            t = torch.randn(shape, generator=g)
        elif last == "router":
            t = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[1])
        else:
            t = 1.3 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        out[name] = t.to(store).to(torch.float32)
    return out


def tiny_config(width=64, vocab=97, heads=3, dim=16, vdim=24, kv_rank=32, q_rank=40, window=12, layers=3, experts=4, top=2,
                ff=48, shared_ff=40, groups=2, side_dim=8, loop=None, softcap=20.0, limit=1.5, max_positions=512,
                scale=None, mlp_at=None, windows=None, mixers=None) -> dict:
    """A small configuration; `mlp_at`: the layers that have a feed-forward (None: all); `windows`: a window a layer
    (None in the list: that layer sees every earlier token); `mixers`: a dict a layer of mixer sizes that differ from the
    common ones."""
    ls = []
    for i in range(layers):
        win = window if windows is None else windows[i]
        mixer = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale or dim ** -0.5, "vdim": vdim}
        if mixers is not None and mixers[i]:
            mixer.update(mixers[i])
        if win:
            mixer["mask"] = {"size": win}
        mlp = None
        if mlp_at is None or i in mlp_at:
            mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
            if shared_ff:
                mlp["shared"] = {"ff": shared_ff, "limit": limit + 0.5}
        ls.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Patadra", "vocab": vocab, "width": width, "max_positions": max_positions,
           "norm": {"eps": 1e-5, "groups": groups}, "layers": ls}
    if softcap:
        cfg["logit_softcap"] = softcap
    if side_dim:
        cfg["token_side"] = {"dim": side_dim}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def config_a() -> dict:
    """Three layers, no loop, two experts a token of four, a shared expert, norms in two parts, every layer alike."""
    return tiny_config()


def config_b() -> dict:
    """Four layers of which two run twice, one without a feed-forward, one that sees every earlier token, windows of 70, 5
    and 33, one expert a token of five, no shared expert, norms of the whole row, no cap, a token input of 12 columns, latent
    rows of 48 (filled up to 64 in the cache), layers of unequal head counts and sizes."""
    return tiny_config(width=96, vocab=131, heads=4, dim=32, vdim=16, kv_rank=48, q_rank=24, layers=4, experts=5, top=1, ff=40,
                       shared_ff=0, groups=1, side_dim=12, loop=(1, 3, 2), softcap=None, limit=2.5, mlp_at=[0, 2, 3],
                       windows=[None, 70, 5, 33], scale=0.2,
                       mixers=[None, {"heads": 2, "dim": 16, "vdim": 32, "scale": 0.3}, {"kv_rank": 24, "q_rank": 56}, None])


def config_c() -> dict:
    """Three layers of which the first two run three times, eight heads over latent rows of 136 (beyond the matrix-core
    attention's head sizes), a window longer than most prompts, three experts a token of eight, no token input."""
    return tiny_config(width=128, vocab=300, heads=8, dim=24, vdim=40, kv_rank=136, q_rank=64, window=200, layers=3, experts=8,
                       top=3, ff=72, shared_ff=24, groups=4, side_dim=0, loop=(0, 2, 3), softcap=8.0, limit=1.0)


CONFIGS = {"A": config_a, "B": config_b, "C": config_c}
