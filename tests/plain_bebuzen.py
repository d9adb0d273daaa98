"""The Bebuzen design written plainly: one function a mechanism, whole sequences at once, float64 on the CPU.

Nothing here is shared with the engine: the functions take a dict of tensors by checkpoint name and the parsed
config.json, and follow the design's equations directly.  A layer is

    x <- x + m * rms(mixer(x)) * w1,   x <- x + m * rms(ff(x)) * w2          (the sublayers read x itself)

with three mixers (a two-map "differential" attention with short convolutions on q, k, v; a selective scan; an
attention with a window that keeps the first tokens and a unit term in the softmax denominator) and two feed-forwards
(SwiGLU; routed squared-relu experts beside a shared one).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64
_ROUND = None      # a dtype: `forward(..., round_to=)` rounds what an engine in that dtype rounds (see `_r`)


def _r(x: torch.Tensor) -> torch.Tensor:
    """x as it is, or rounded to the dtype a run of `forward` asked for: the rows a projection reads, its result, the normed
    and turned queries and keys, an attention's result.  What the design computes in 32-bit is never rounded."""
    return x if _ROUND is None else x.to(_ROUND).to(F64)


def rms(x: torch.Tensor, eps: float, w: Optional[torch.Tensor] = None) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(x):
    return x * torch.sigmoid(x)


def short_conv(u: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros((taps - 1, C), dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j]
    return y if bias is None else y + bias


def rotary_frequencies(rot: dict) -> torch.Tensor:
    dims = int(rot["dims"])
    i = torch.arange(dims // 2, dtype=F64)
    f = float(rot["base"]) ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for fi in f.tolist():
            wl = 2.0 * math.pi / fi
            if wl < orig / high:
                out.append(fi)
            elif wl > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=F64)
    return f


def rotate(x: torch.Tensor, pos: torch.Tensor, rot: Optional[dict], layout: str) -> torch.Tensor:
    """x [T, heads, dim]; the first rot.dims entries of every head are turned.  layout 'half': entry i with i + dims/2;
    'pairs': entry 2i with 2i + 1."""
    if not rot or int(rot["dims"]) == 0:
        return x
    dims = int(rot["dims"])
    f = rotary_frequencies(rot)
    ang = pos.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if layout == "half":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    return out


def visible(T: int, size: Optional[int], keep_first: int = 0) -> torch.Tensor:
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if size is not None:
        ok = ok & ((i - j < size) | (j < keep_first))
    return ok


def softmax_attention(q, k, v, scale: float, mask: torch.Tensor, extra_one: bool) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; head h reads group h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    per = H // G
    out = torch.zeros((T, H, v.shape[-1]), dtype=q.dtype)
    for h in range(H):
        g = h // per
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, -math.inf)
        m = s.max(-1, keepdim=True).values
        if extra_one:
            m = torch.clamp(m, min=0.0)
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if extra_one:
            den = den + torch.exp(-m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def differential_keys_values(W: Dict[str, torch.Tensor], p: str, mx: dict, h: torch.Tensor, pos: torch.Tensor, eps: float):
    """The keys (after convolution, norm and rotation) [T, G, 2, dim] and values (after convolution) [T, G, vdim]."""
    G, dim, vdim = int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    T = h.shape[0]
    k = _r(h @ W[p + "k"].T + W[p + "k.b"])
    v = _r(h @ W[p + "v"].T + W[p + "v.b"])
    if mx.get("conv"):
        k = short_conv(k, W[p + "k.conv"])
        v = short_conv(v, W[p + "v.conv"])
    k = rms(k.view(T, G * 2, dim), eps, W[p + "k.norm"])
    k = _r(rotate(k, pos, mx.get("rot"), "half"))
    return k.view(T, G, 2, dim), _r(v).view(T, G, vdim)


def differential_attention(W, p: str, mx: dict, h, pos, eps: float, kv=None):
    """Returns (output [T, width], (k, v)); `kv`: another layer's keys and values to read instead of one's own."""
    H, G, dim, vdim = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    T = h.shape[0]
    q = _r(h @ W[p + "q"].T + W[p + "q.b"])
    if mx.get("conv"):
        q = short_conv(q, W[p + "q.conv"])
    q = rms(q.view(T, H * 2, dim), eps, W[p + "q.norm"])
    q = _r(rotate(q, pos, mx.get("rot"), "half")).view(T, H, 2, dim)
    if kv is None:
        kv = differential_keys_values(W, p, mx, h, pos, eps)
    k, v = kv
    size = mx["mask"]["size"] if mx.get("mask") else None
    mask = visible(T, size)
    a1 = softmax_attention(q[:, :, 0], k[:, :, 0], v, float(mx["scale"]), mask, False)
    a2 = softmax_attention(q[:, :, 1], k[:, :, 1], v, float(mx["scale"]), mask, False)
    diff = float(mx["diff"])
    lam = torch.exp((W[p + "lq1"] * W[p + "lk1"]).sum()) - torch.exp((W[p + "lq2"] * W[p + "lk2"]).sum()) + diff
    o = _r(rms(a1 - lam * a2, eps) * (1.0 - diff))
    return _r(o.reshape(T, H * vdim) @ W[p + "o"].T), kv


def sink_window_attention(W, p: str, mx: dict, h, pos, eps: float):
    H, G, dim, vdim = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    T = h.shape[0]
    q = _r(h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, dim)
    k = _r(h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, dim)
    v = _r(h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, vdim)
    q = _r(rotate(rms(q, eps, W[p + "q.norm"]), pos, mx.get("rot"), "pairs"))
    k = _r(rotate(rms(k, eps, W[p + "k.norm"]), pos, mx.get("rot"), "pairs"))
    mk = mx.get("mask")
    mask = visible(T, mk["size"] if mk else None, int(mk.get("keep_first", 0)) if mk else 0)
    o = _r(softmax_attention(q, k, v, float(mx["scale"]), mask, True))
    return _r(o.reshape(T, H * vdim) @ W[p + "o"].T + W[p + "o.b"])


def selective_scan(W, p: str, mx: dict, h):
    inner, state, dt_rank = int(mx["inner"]), int(mx["state"]), int(mx["dt_rank"])
    T = h.shape[0]
    xz = _r(h @ W[p + "in"].T)
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(short_conv(x, W[p + "conv"], W[p + "conv.b"]))
    r = _r(_r(x) @ W[p + "x"].T)
    dt, B, C = r[:, :dt_rank], r[:, dt_rank:dt_rank + state], r[:, dt_rank + state:]
    dt = torch.nn.functional.softplus(_r(dt @ W[p + "dt"].T) + W[p + "dt.b"])
    A = -torch.exp(W[p + "A_log"])
    S = torch.zeros((inner, state), dtype=h.dtype)
    ys = []
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        ys.append(S @ C[t] + W[p + "D"] * x[t])
    y = _r(torch.stack(ys) * silu(z))
    return _r(y @ W[p + "o"].T)


def relu2_mlp(W, p: str, h):
    return _r(_r(torch.relu(_r(h @ W[p + "up"].T)) ** 2) @ W[p + "down"].T)


def feed_forward(W, p: str, ml: dict, h, forced: Optional[torch.Tensor] = None, chosen: Optional[list] = None):
    """`forced` [T, top]: expert choices to use instead of the router's own (the weights still come from the scores);
    `chosen`: a list that receives (the router's own choices [T, top], the scores [T, experts])."""
    if ml["kind"] == "dense":
        return _r(_r(silu(_r(h @ W[p + "gate"].T)) * _r(h @ W[p + "up"].T)) @ W[p + "down"].T)
    r = ml["router"]
    E, top = int(r["experts"]), int(r["top"])
    s = torch.softmax(h @ W[p + "router"].T, -1)
    own = torch.topk(s, top, dim=-1).indices
    if chosen is not None:
        chosen.append((own, s))
    idx = forced if forced is not None else own
    out = torch.zeros_like(h)
    for e in range(E):
        rows = (idx == e).any(-1).nonzero().flatten()
        if rows.numel():
            out[rows] += relu2_mlp(W, p + f"e{e}.", h[rows]) * (s[rows, e] * float(r.get("scale", 1.0)))[:, None]
    if ml.get("shared"):
        out = out + relu2_mlp(W, p + "shared.", h)
    return out


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], return_layers: bool = False, forced: Optional[dict] = None,
            chosen: Optional[dict] = None, round_to: Optional[torch.dtype] = None):
    """Logits [T, vocab] of one sequence from its start (and the stream after every layer).  `forced` {layer: [T, top]}: expert
    choices to use; `chosen`: a dict that receives {layer: (the router's own choices, the scores)}; `round_to`: a dtype to which
    the rows a projection reads and what it gives are rounded, as an engine in that dtype does (the stream, norms, scores,
    states and routers stay exact)."""
    global _ROUND
    _ROUND = round_to
    try:
        return _forward(cfg, W, tokens, return_layers, forced, chosen)
    finally:
        _ROUND = None


def _forward(cfg, W, tokens, return_layers, forced, chosen):
    W = {k: v.to(F64) for k, v in W.items()}
    eps, m = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    x = W["embed"][torch.tensor(tokens)]
    pos = torch.arange(len(tokens))
    kvs, layers = {}, []
    for i, ly in enumerate(cfg["layers"]):
        p, mx = f"l{i}.mix.", ly["mixer"]
        if ly["type"] == "attention":
            src = mx.get("kv_from")
            y, kv = differential_attention(W, p, mx, _r(x), pos, eps, kvs[src] if src is not None else None)
            kvs[i] = kv
        elif ly["type"] == "attention_2":
            y = sink_window_attention(W, p, mx, _r(x), pos, eps)
        elif ly["type"] == "mamba1":
            y = selective_scan(W, p, mx, _r(x))
        else:
            raise ValueError(ly["type"])
        x = x + m * rms(y, eps, W[f"l{i}.norm1"])
        if ly.get("mlp"):
            got = [] if chosen is not None else None
            y = feed_forward(W, f"l{i}.mlp.", ly["mlp"], _r(x), None if forced is None else forced.get(i), got)
            if got:
                chosen[i] = got[0]
            x = x + m * rms(y, eps, W[f"l{i}.norm2"])
        layers.append(x.clone())
    logits = _r(rms(x, eps, W["final.norm"])) @ W["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    """Every tensor of a model of this configuration with its shape, as a checkpoint holds them."""
    Wd, out = int(cfg["width"]), {}
    out["embed"] = (int(cfg["vocab"]), Wd)
    for i, ly in enumerate(cfg["layers"]):
        p, mx = f"l{i}.mix.", ly["mixer"]
        out[f"l{i}.norm1"] = (Wd,)
        if ly["type"] in ("attention", "attention_2"):
            H, G, dim, vdim = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
            maps = 2 if ly["type"] == "attention" else 1
            own_kv = mx.get("kv_from") is None
            sizes = {"q": H * maps * dim}
            if own_kv:
                sizes.update(k=G * maps * dim, v=G * vdim)
            for n, rows in sizes.items():
                out[p + n] = (rows, Wd)
                out[p + n + ".b"] = (rows,)
                if ly["type"] == "attention" and mx.get("conv"):
                    out[p + n + ".conv"] = (rows, int(mx["conv"]))
            out[p + "q.norm"] = (dim,)
            if own_kv:
                out[p + "k.norm"] = (dim,)
            out[p + "o"] = (Wd, H * vdim)
            if ly["type"] == "attention":
                for n in ("lq1", "lk1", "lq2", "lk2"):
                    out[p + n] = (dim,)
            else:
                out[p + "o.b"] = (Wd,)
        else:
            inner, state, dt_rank, taps = int(mx["inner"]), int(mx["state"]), int(mx["dt_rank"]), int(mx["conv"])
            out.update({p + "in": (2 * inner, Wd), p + "conv": (inner, taps), p + "conv.b": (inner,),
                        p + "x": (dt_rank + 2 * state, inner), p + "dt": (inner, dt_rank), p + "dt.b": (inner,),
                        p + "A_log": (inner, state), p + "D": (inner,), p + "o": (Wd, inner)})
        ml = ly.get("mlp")
        if ml:
            out[f"l{i}.norm2"] = (Wd,)
            q = f"l{i}.mlp."
            if ml["kind"] == "dense":
                ff = int(ml["ff"])
                out.update({q + "gate": (ff, Wd), q + "up": (ff, Wd), q + "down": (Wd, ff)})
            else:
                ff = int(ml["expert"]["ff"])
                for e in range(int(ml["router"]["experts"])):
                    out[q + f"e{e}.up"] = (ff, Wd)
                    out[q + f"e{e}.down"] = (Wd, ff)
                out[q + "router"] = (int(ml["router"]["experts"]), Wd)
                if ml.get("shared"):
                    sf = int(ml["shared"]["ff"])
                    out[q + "shared.up"] = (sf, Wd)
                    out[q + "shared.down"] = (Wd, sf)
    out["final.norm"] = (Wd,)
    out["head"] = (int(cfg["vocab"]), Wd)
    return out


# ---- configurations and weights for tests --------------------------------------------------------------------------------
def _scaling():
    return {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 64}


def config_a():
    moe = {"kind": "moe", "router": {"experts": 4, "top": 2, "scale": 1.5}, "expert": {"ff": 24}, "shared": {"ff": 16}}
    return {"architecture": "Bebuzen", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.5, "layers": [
        {"type": "attention_2", "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3, "rot": {"base": 100.0, "dims": 8},
                                          "mask": {"size": 20, "keep_first": 3}}, "mlp": {"kind": "dense", "ff": 48}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 12, "scale": 0.4, "diff": 0.3, "conv": 2,
                                        "rot": {"base": 50.0, "dims": 8, "scaling": _scaling()}, "mask": {"size": 33}}, "mlp": moe},
        {"type": "mamba1", "mixer": {"inner": 48, "state": 5, "dt_rank": 3, "conv": 4}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 12, "scale": 0.4, "diff": 0.3, "conv": 2,
                                        "rot": {"base": 50.0, "dims": 8, "scaling": _scaling()}, "mask": {"size": 50}, "kv_from": 1}, "mlp": moe}]}


def config_b():
    moe = {"kind": "moe", "router": {"experts": 3, "top": 1}, "expert": {"ff": 20}}
    return {"architecture": "Bebuzen", "vocab": 130, "width": 96, "norm": {"eps": 1e-6}, "layers": [
        {"type": "mamba1", "mixer": {"inner": 160, "state": 20, "dt_rank": 7, "conv": 2}, "mlp": {"kind": "dense", "ff": 72}},
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 6, "dim": 12, "vdim": 8, "scale": 0.25, "diff": 0.7, "conv": 4,
                                        "rot": {"base": 1000.0, "dims": 4}}, "mlp": moe},
        {"type": "attention_2", "mixer": {"heads": 3, "kv_heads": 1, "dim": 32, "vdim": 32, "scale": 0.2, "mask": {"size": 64}}, "mlp": moe},
        {"type": "attention_2", "mixer": {"heads": 2, "kv_heads": 2, "dim": 20, "vdim": 36, "scale": 0.2, "rot": {"base": 10000.0, "dims": 20}},
         "mlp": None},
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 6, "dim": 12, "vdim": 8, "scale": 0.25, "diff": 0.7, "conv": 4,
                                        "rot": {"base": 1000.0, "dims": 4}, "kv_from": 1}, "mlp": {"kind": "dense", "ff": 40}}]}


def config_c():
    """Sizes the matrix-core kernels take."""
    moe = {"kind": "moe", "router": {"experts": 8, "top": 3, "scale": 2.0}, "expert": {"ff": 64}, "shared": {"ff": 64}}
    rot = {"base": 5000.0, "dims": 32, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 128}}
    return {"architecture": "Bebuzen", "vocab": 200, "width": 128, "norm": {"eps": 1e-5}, "residual_mult": 0.8, "layers": [
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 64, "scale": 0.18, "diff": 0.5, "conv": 3,
                                        "rot": rot, "mask": {"size": 70}}, "mlp": {"kind": "dense", "ff": 256}},
        {"type": "attention_2", "mixer": {"heads": 4, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.125, "rot": {"base": 10000.0, "dims": 32},
                                          "mask": {"size": 40, "keep_first": 5}}, "mlp": moe},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 64, "scale": 0.18, "diff": 0.5, "conv": 3,
                                        "rot": rot, "mask": {"size": 70}, "kv_from": 0}, "mlp": moe},
        {"type": "mamba1", "mixer": {"inner": 256, "state": 16, "dt_rank": 8, "conv": 4}, "mlp": {"kind": "dense", "ff": 128}}]}


CONFIGS = {"A": config_a, "B": config_b, "C": config_c}


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors of a size that keeps every mechanism at work: norms near one, decays spread over (0, 1), routers sharp
    enough that the chosen experts seldom hang on a rounding."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        r = torch.randn(shape, generator=g)
        if leaf in ("norm1", "norm2", "norm") or name == "final.norm":
            t = 1.0 + 0.2 * r
        elif name.endswith("A_log"):
            t = torch.log(0.3 + 3.0 * torch.rand(shape, generator=g))
        elif name.endswith("dt.b"):
            t = -2.5 + 0.8 * r
        elif leaf == "D":
            t = 1.0 + 0.3 * r
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.3 * r
        elif leaf == "b":
            t = 0.2 * r
        elif leaf == "conv":
            t = 0.6 * r
        elif leaf == "router":
            t = 3.0 * r / math.sqrt(shape[1])
        elif name == "embed":
            t = r
        elif len(shape) == 2:
            t = r * (1.3 / math.sqrt(shape[1]))
        else:
            t = r
        out[name] = t
    return out
