"""config.json contents of the model shapes the benchmarks run with random weights: the MiniCPM4-8B,
MiniCPM4-0.5B and MiniCPM-2B-family layer sizes.  LongRoPE factors are drawn from a fixed seed
(uniform in [1, 4]); nothing else is random."""
from __future__ import annotations


def _factors(n: int, seed: int):
    import torch
    g = torch.Generator().manual_seed(seed)
    short = (1.0 + 3.0 * torch.rand(n, generator=g)).tolist()
    long = (1.0 + 3.0 * torch.rand(n, generator=g)).tolist()
    return short, long


def shape_config(name: str, layers: int = 0) -> dict:
    """`name`: "8b", "0.5b", "2b" (MiniCPM4 family), "kekevik-<width>", "pugavik-<width>", "patadra-<width>" or "bebuzen-<width>" (those designs at
    that width, 8 layers unless told otherwise); `layers` > 0 overrides the number of layers."""
    if name.startswith("bebuzen-"):
        width = int(name.split("-", 1)[1])
        return bebuzen_shape(width, width // 128, 128, 2, layers or 8, 32768)
    if name.startswith("patadra-"):
        width = int(name.split("-")[1])
        return patadra_shape(width, width // 128, 128, layers or 8, 32768)
    if name.startswith("kekevik-"):
        width = int(name.split("-")[1])
        return kekevik_shape(width, width // 128, 128, 2, layers or 8, 32768, 6 * width)
    if name.startswith("pugavik-"):
        width = int(name.split("-")[1])
        return pugavik_shape(width, width // 128, 128, 2, layers or 8, 32768, 6 * width)
    base = {"architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm", "torch_dtype": "bfloat16", "rope_theta": 10000.0,
            "scale_emb": 12, "scale_depth": 1.4, "dim_model_base": 256}
    if name == "8b":
        short, long = _factors(64, 1234)
        cfg = dict(base, num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=2, head_dim=128,
                   intermediate_size=16384, vocab_size=73448, max_position_embeddings=32768, rms_norm_eps=1e-6,
                   tie_word_embeddings=False,
                   rope_scaling={"type": "longrope", "short_factor": short, "long_factor": long,
                                 "original_max_position_embeddings": 32768})
    elif name == "0.5b":
        short, long = _factors(32, 1235)
        cfg = dict(base, num_hidden_layers=24, hidden_size=1024, num_attention_heads=16, num_key_value_heads=2, head_dim=64,
                   intermediate_size=4096, vocab_size=73448, max_position_embeddings=32768, rms_norm_eps=1e-6,
                   tie_word_embeddings=True,
                   rope_scaling={"type": "longrope", "short_factor": short, "long_factor": long,
                                 "original_max_position_embeddings": 32768})
    elif name == "2b":
        cfg = dict(base, num_hidden_layers=40, hidden_size=2304, num_attention_heads=36, num_key_value_heads=36, head_dim=64,
                   intermediate_size=5760, vocab_size=122753, max_position_embeddings=4096, rms_norm_eps=1e-5,
                   tie_word_embeddings=True)
    else:
        raise KeyError(f"unknown shape {name!r}; there are 8b, 0.5b and 2b")
    if layers > 0:
        cfg["num_hidden_layers"] = int(layers)
    return cfg


def kekevik_shape(width: int, heads: int, head_dim: int, kv_heads: int, layers: int, vocab: int, ff: int) -> dict:
    """A Kekevik configuration with the layer sizes of a transformer of this width: the four layer kinds in turn
    (retention, lightning, two side-by-side layers), `heads` heads of `head_dim` everywhere, a state space of
    heads * head_dim channels with 128 state entries a head, `ff` inner units of the feed-forward."""
    decay = [1.0 - 2.0 ** -(5 + (7 * h) // max(heads, 1)) for h in range(heads)]
    lin = {"heads": heads, "dim": head_dim, "vdim": head_dim, "decay": decay}
    par = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": head_dim, "vdim": head_dim, "scale": head_dim ** -0.5,
                    "softcap": 50.0, "q_temp": {"coef": 0.1, "every": 1024}},
           "right": {"heads": heads, "vdim": head_dim, "state": 128, "groups": 1, "conv": 4, "norm_groups": 1},
           "left_scale": 1.0, "right_scale": 1.0}
    kinds = [("retention", dict(lin, rot={"dims": head_dim, "base": 10000.0})), ("lightning", lin), ("parallel", par), ("parallel", par)]
    return {"architecture": "Kekevik", "vocab": vocab, "width": width, "embedding": {"scale": 12.0}, "norm": {"eps": 1e-6},
            "layers": [{"type": kinds[i % 4][0], "mixer": kinds[i % 4][1], "mlp": {"kind": "dense", "ff": ff}} for i in range(layers)]}


def pugavik_shape(width: int, heads: int, head_dim: int, kv_heads: int, layers: int, vocab: int, ff: int, window: int = 1024,
                  loop: dict = None) -> dict:
    """A Pugavik configuration with the layer sizes of a transformer of this width: the three layer kinds in turn (latent
    attention, windowed attention with mixed scores, gated linear attention), `heads` heads everywhere: query/key heads of
    `head_dim` (the latent layers': three quarters unrotated, a quarter rotated; latent rows of three quarters of `head_dim`,
    so that a cached row with its rotated part has `head_dim` entries), value heads of `head_dim`, gated layers with keys of
    half of it; `ff` inner units of the feed-forward; no loop unless one is given."""
    rot = head_dim // 4
    latent = {"heads": heads, "dim": head_dim - rot, "rot_dim": rot, "vdim": head_dim, "kv_rank": head_dim - rot,
              "scale": head_dim ** -0.5, "rot": {"dims": rot, "base": 10000.0}}
    att = {"heads": heads, "kv_heads": kv_heads, "dim": head_dim, "vdim": head_dim, "scale": head_dim ** -0.5,
           "mask": {"size": window}, "rot": {"dims": head_dim // 2, "base": 500000.0}}
    gla = {"heads": heads, "dim": head_dim // 2, "vdim": head_dim, "tau": 16.0, "decay_rank": 16}
    kinds = [("latent_attention", latent), ("attention", att), ("gla", gla)]
    cfg = {"architecture": "Pugavik", "vocab": vocab, "width": width, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
           "layers": [{"type": kinds[i % 3][0], "mixer": kinds[i % 3][1], "mlp": {"kind": "dense", "ff": ff}} for i in range(layers)]}
    if loop:
        cfg["loop"] = dict(loop)
    return cfg


def patadra_shape(width: int, heads: int, head_dim: int, layers: int, vocab: int, experts: int = 16, top: int = 2, window: int = 1024,
                  max_positions: int = 4096, loop: dict = None) -> dict:
    """A Patadra configuration with the layer sizes of a transformer of this width: `heads` heads with queries, keys and values
    of `head_dim`, latent rows of `head_dim` (one cached row a token), queries through a row of a quarter of the width; `experts`
    experts with `width` inner units each, of which a token uses `top`, and a shared expert of the same size (three times the
    width of inner units at work for a token); norms in four parts, a token input of 256 columns a layer, capped logits."""
    mixer = {"heads": heads, "dim": head_dim, "vdim": head_dim, "kv_rank": head_dim, "q_rank": width // 4, "scale": head_dim ** -0.5,
             "mask": {"size": window}}
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": width, "limit": 7.0},
           "shared": {"ff": width, "limit": 7.0}}
    cfg = {"architecture": "Patadra", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": 1e-5, "groups": 4},
           "logit_softcap": 30.0, "token_side": {"dim": 256},
           "layers": [{"type": "latent_attention", "mixer": dict(mixer), "mlp": dict(mlp)} for _ in range(layers)]}
    if loop:
        cfg["loop"] = dict(loop)
    return cfg


def bebuzen_shape(width: int, heads: int, head_dim: int, kv_heads: int, layers: int, vocab: int, window: int = 1024, experts: int = 8,
                  top: int = 2) -> dict:
    """A Bebuzen configuration with the layer sizes of a transformer of this width: four layer kinds in turn (an attention with a
    window that keeps eight first tokens and a dense feed-forward of 4 x width; a differential attention with two maps of half
    of `head_dim` each, a convolution of four taps and scaled frequencies; a selective scan over 2 x width channels with 16
    state entries each; a differential attention that reads the second layer's keys and values), the last three with `experts`
    experts of 2 x width inner units of which a token uses `top`, beside a shared expert of the same size (as many feed-forward
    weights at work for a token as in the dense layers)."""
    half = head_dim // 2
    att2 = {"heads": heads, "kv_heads": kv_heads, "dim": head_dim, "vdim": head_dim, "scale": head_dim ** -0.5,
            "rot": {"base": 10000.0, "dims": head_dim}, "mask": {"size": window, "keep_first": 8}}
    diff = {"heads": heads, "kv_heads": kv_heads, "dim": half, "vdim": head_dim, "scale": half ** -0.5, "diff": 0.5, "conv": 4,
            "rot": {"base": 500000.0, "dims": half, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}},
            "mask": {"size": window}}
    scan = {"inner": 2 * width, "state": 16, "dt_rank": max(width // 16, 1), "conv": 4}
    dense = {"kind": "dense", "ff": 4 * width}
    moe = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": 2.0}, "expert": {"ff": 2 * width}, "shared": {"ff": 2 * width}}
    out = []
    for i in range(layers):
        k = i % 4
        if k == 0:
            out.append({"type": "attention_2", "mixer": dict(att2), "mlp": dict(dense)})
        elif k == 1:
            out.append({"type": "attention", "mixer": dict(diff), "mlp": dict(moe)})
        elif k == 2:
            out.append({"type": "mamba1", "mixer": dict(scan), "mlp": dict(moe)})
        else:
            out.append({"type": "attention", "mixer": dict(diff, kv_from=i - 2), "mlp": dict(moe)})
    return {"architecture": "Bebuzen", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "residual_mult": 0.5, "layers": out}
