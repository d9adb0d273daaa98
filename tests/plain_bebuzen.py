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
    k = h @ W[p + "k"].T + W[p + "k.b"]
    v = h @ W[p + "v"].T + W[p + "v.b"]
    if mx.get("conv"):
        k = short_conv(k, W[p + "k.conv"])
        v = short_conv(v, W[p + "v.conv"])
    k = rms(k.view(T, G * 2, dim), eps, W[p + "k.norm"])
    k = rotate(k, pos, mx.get("rot"), "half")
    return k.view(T, G, 2, dim), v.view(T, G, vdim)


def differential_attention(W, p: str, mx: dict, h, pos, eps: float, kv=None):
    """Returns (output [T, width], (k, v)); `kv`: another layer's keys and values to read instead of one's own."""
    H, G, dim, vdim = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    T = h.shape[0]
    q = h @ W[p + "q"].T + W[p + "q.b"]
    if mx.get("conv"):
        q = short_conv(q, W[p + "q.conv"])
    q = rms(q.view(T, H * 2, dim), eps, W[p + "q.norm"])
    q = rotate(q, pos, mx.get("rot"), "half").view(T, H, 2, dim)
    if kv is None:
        kv = differential_keys_values(W, p, mx, h, pos, eps)
    k, v = kv
    size = mx["mask"]["size"] if mx.get("mask") else None
    mask = visible(T, size)
    a1 = softmax_attention(q[:, :, 0], k[:, :, 0], v, float(mx["scale"]), mask, False)
    a2 = softmax_attention(q[:, :, 1], k[:, :, 1], v, float(mx["scale"]), mask, False)
    diff = float(mx["diff"])
    lam = torch.exp((W[p + "lq1"] * W[p + "lk1"]).sum()) - torch.exp((W[p + "lq2"] * W[p + "lk2"]).sum()) + diff
    o = rms(a1 - lam * a2, eps) * (1.0 - diff)
    return o.reshape(T, H * vdim) @ W[p + "o"].T, kv


def sink_window_attention(W, p: str, mx: dict, h, pos, eps: float):
    H, G, dim, vdim = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, dim)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, dim)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, vdim)
    q = rotate(rms(q, eps, W[p + "q.norm"]), pos, mx.get("rot"), "pairs")
    k = rotate(rms(k, eps, W[p + "k.norm"]), pos, mx.get("rot"), "pairs")
    mk = mx.get("mask")
    mask = visible(T, mk["size"] if mk else None, int(mk.get("keep_first", 0)) if mk else 0)
    o = softmax_attention(q, k, v, float(mx["scale"]), mask, True)
    return o.reshape(T, H * vdim) @ W[p + "o"].T + W[p + "o.b"]


def selective_scan(W, p: str, mx: dict, h):
    inner, state, dt_rank = int(mx["inner"]), int(mx["state"]), int(mx["dt_rank"])
    T = h.shape[0]
    xz = h @ W[p + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(short_conv(x, W[p + "conv"], W[p + "conv.b"]))
    r = x @ W[p + "x"].T
    dt, B, C = r[:, :dt_rank], r[:, dt_rank:dt_rank + state], r[:, dt_rank + state:]
    dt = torch.nn.functional.softplus(dt @ W[p + "dt"].T + W[p + "dt.b"])
    A = -torch.exp(W[p + "A_log"])
    S = torch.zeros((inner, state), dtype=h.dtype)
    ys = []
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        ys.append(S @ C[t] + W[p + "D"] * x[t])
    y = torch.stack(ys) * silu(z)
    return y @ W[p + "o"].T


def relu2_mlp(W, p: str, h):
    return torch.relu(h @ W[p + "up"].T) ** 2 @ W[p + "down"].T


def feed_forward(W, p: str, ml: dict, h, forced: Optional[torch.Tensor] = None):
    """`forced` [T, top]: expert choices to use instead of the router's own (the weights still come from the scores)."""
    if ml["kind"] == "dense":
        return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T
    r = ml["router"]
    E, top = int(r["experts"]), int(r["top"])
    s = torch.softmax(h @ W[p + "router"].T, -1)
    idx = forced if forced is not None else torch.topk(s, top, dim=-1).indices
    out = torch.zeros_like(h)
    for e in range(E):
        rows = (idx == e).any(-1).nonzero().flatten()
        if rows.numel():
            out[rows] += relu2_mlp(W, p + f"e{e}.", h[rows]) * (s[rows, e] * float(r.get("scale", 1.0)))[:, None]
    if ml.get("shared"):
        out = out + relu2_mlp(W, p + "shared.", h)
    return out


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], return_layers: bool = False, forced: Optional[dict] = None):
    """Logits [T, vocab] of one sequence from its start (and the stream after every layer)."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps, m = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    x = W["embed"][torch.tensor(tokens)]
    pos = torch.arange(len(tokens))
    kvs, layers = {}, []
    for i, ly in enumerate(cfg["layers"]):
        p, mx = f"l{i}.mix.", ly["mixer"]
        if ly["type"] == "attention":
            src = mx.get("kv_from")
            y, kv = differential_attention(W, p, mx, x, pos, eps, kvs[src] if src is not None else None)
            kvs[i] = kv
        elif ly["type"] == "attention_2":
            y = sink_window_attention(W, p, mx, x, pos, eps)
        elif ly["type"] == "mamba1":
            y = selective_scan(W, p, mx, x)
        else:
            raise ValueError(ly["type"])
        x = x + m * rms(y, eps, W[f"l{i}.norm1"])
        if ly.get("mlp"):
            y = feed_forward(W, f"l{i}.mlp.", ly["mlp"], x, None if forced is None else forced.get(i))
            x = x + m * rms(y, eps, W[f"l{i}.norm2"])
        layers.append(x.clone())
    logits = rms(x, eps, W["final.norm"]) @ W["head"].T
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
