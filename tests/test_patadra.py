"""Patadra without a GPU: config.json's keys and their checks, the order of layer runs, tensor names against the plain
implementation's own list, the experts' stacked tensors, the cache entries of a looped model with several windows, and the
plain implementation's own consistency (a prefix's logits do not depend on what follows; a window's edge; the sink takes
weight from every key; scores that are not renormalised; norms in parts)."""
import copy
import os

import pytest
import torch

import plain_patadra as P
from infinilm_amd.cache import CacheManager
from infinilm_amd.cache.needs import PagedKV
from infinilm_amd.config import ConfigError, load_model_config
from infinilm_amd.engine.model import CausalLM


def _latent_rows(rank):
    return -(-rank // 32) * 32 if rank <= 128 else -(-rank // 16) * 16


@pytest.mark.parametrize("name", sorted(P.CONFIGS))
def test_description_names_every_tensor(name):
    cfg = P.CONFIGS[name]()
    arch, typed = load_model_config(cfg)
    assert arch.name == "Patadra"
    spec = arch.build_spec(typed)
    model = CausalLM(spec, torch.float32, "meta")
    assert {k: tuple(p.shape) for k, p in model.named_parameters().items()} == P.tensor_shapes(cfg)
    assert not model.head_is_tied
    want = P.run_order(cfg)
    assert [r.layer for r in spec.order] == want
    assert [r.cache for r in spec.order] == list(range(len(want)))
    assert all(r.start is None for r in spec.order)            # nothing happens between the passes of a loop
    for run, need in zip(spec.order, model.cache_needs):
        m = cfg["layers"][run.layer]["mixer"]
        assert need == PagedKV(1, _latent_rows(m["kv_rank"]), (m.get("mask") or {}).get("size", 0))


def test_a_looped_model_keeps_a_cache_for_every_pass():
    cfg = P.config_b()
    arch, typed = load_model_config(cfg)
    model = CausalLM(arch.build_spec(typed), torch.float32, "meta")
    assert len(model.cache_needs) == 1 + 2 * 2 + 1
    cache = CacheManager(model.cache_needs, page_size=8, num_pages=12, max_requests=2, dtype=torch.float32, device="meta")
    assert sorted({g.window for g in cache.groups}) == [0, 5, 33, 70]
    cache.admit("a")
    cache.reserve("a", 90)
    cache.commit("a", 90)
    held = {}
    for g, t in zip(cache.groups, cache.requests["a"].tables):
        held.setdefault(g.window, [p >= 0 for p in t])
    assert held[0] == [True] * 12
    assert held[5] == [False] * 10 + [True] * 2                # the next token sees positions 86 .. 90
    assert held[33] == [False] * 7 + [True] * 5                # 58 ..
    assert held[70] == [False] * 2 + [True] * 10               # 21 ..
    cache.release("a")
    cache.check()


def test_experts_lie_stacked_and_the_router_holds_the_shared_gate():
    from infinilm_amd.weights.loader import load_state_dict
    cfg = P.config_a()
    arch, typed = load_model_config(cfg)
    model = CausalLM(arch.build_spec(typed), torch.float32, "cpu")
    W = P.random_weights(cfg, 1)
    load_state_dict(model, W)
    ff = model.blocks[1].ffn
    assert (ff.E, ff.top, ff.ff, ff.shared_ff, ff.limit, ff.shared_limit, ff.alpha) == (4, 2, 48, 40, 1.5, 2.0, 1.702)
    for e in range(4):
        assert torch.equal(ff.w_gate_up[e, :48], W[f"l1.mlp.e{e}.gate"]) and torch.equal(ff.w_gate_up[e, 48:], W[f"l1.mlp.e{e}.up"])
        assert torch.equal(ff.w_down[e], W[f"l1.mlp.e{e}.down"])
    assert torch.equal(ff.router.weight[:4], W["l1.mlp.router"]) and torch.equal(ff.router.weight[4:], W["l1.mlp.shared.sg"])
    att = model.blocks[2].mixer
    assert (att.H, att.dn, att.dr, att.dv, att.rank, att.q_rank, att.window, att.d) == (3, 16, 0, 24, 32, 40, 12, 32)
    assert att.sink.dtype == torch.float32 and torch.equal(att.sink, W["l2.mix.sink"])
    assert torch.equal(att.proj.weight[:40], W["l2.mix.dq"]) and torch.equal(att.proj.weight[40:], W["l2.mix.dkv"])
    side = model.blocks[2].side
    assert side.first == 16 and side.dim == 8 and side.table is model.shared_tensors["side.embed"]
    assert torch.equal(model.shared_tensors["side.embed"], W["side.embed"])
    assert torch.equal(model.embedding.position_table, W["pos"]) and model.output_head.cap == 20.0
    assert model.blocks[0].norm1.groups == 2 and model.final_norm.groups == 2


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("max_positions"), "max_positions"),
    (lambda c: c["layers"][0].update(type="retention"), "unknown layer type"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][1]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "unknown kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c["layers"][2]["mlp"]["expert"].update(limit=-1.0), "limit"),
    (lambda c: c["loop"].update(stop=9), "stretch"),
    (lambda c: c["loop"].pop("times"), "times"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["norm"].update(groups=7), "groups"),
    (lambda c: c["token_side"].pop("dim"), "dim"),
    (lambda c: c.update(logit_softcap=0.0), "logit_softcap"),
])
def test_config_errors_name_the_key(change, message):
    cfg = copy.deepcopy(P.config_b())
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        load_model_config(cfg)


def test_what_config_leaves_out_does_not_exist():
    cfg = P.tiny_config(side_dim=0, softcap=None, shared_ff=0, windows=[None, None, None], mlp_at=[])
    cfg["norm"].pop("groups")
    arch, typed = load_model_config(cfg)
    spec = arch.build_spec(typed)
    model = CausalLM(spec, torch.float32, "meta")
    assert typed.groups == 1 and typed.side_dim == 0 and typed.softcap is None and typed.loop is None
    assert all(b.ffn is None and b.side is None for b in model.blocks) and not model.shared_tensors
    assert type(model.output_head).__name__ == "LinearHead"
    assert {k: tuple(p.shape) for k, p in model.named_parameters().items()} == P.tensor_shapes(cfg)


def test_random_weights_writer_knows_the_design(tmp_path):
    from infinilm_amd.weights.loader import checkpoint_shapes
    from infinilm_amd.weights.random_init import write_random_model
    cfg = P.config_c()
    write_random_model(cfg, 3, str(tmp_path), dtype="bfloat16")
    assert checkpoint_shapes(str(tmp_path)) == P.tensor_shapes(cfg)
    assert os.path.isfile(tmp_path / "config.json")


# ---- the plain implementation's own consistency -----------------------------------------------------------------------------
@pytest.mark.parametrize("name", sorted(P.CONFIGS))
def test_plain_prefix_logits_do_not_depend_on_what_follows(name):
    cfg = P.CONFIGS[name]()
    W = P.random_weights(cfg, 5)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, cfg["vocab"], (50,), generator=g).tolist()
    whole = P.forward(cfg, W, toks)
    for n in (1, 2, 9, 33):
        assert torch.allclose(P.forward(cfg, W, toks[:n]), whole[:n], atol=1e-9)


def test_plain_window_edge_and_sink():
    cfg = P.tiny_config(layers=1, window=4, mlp_at=[], side_dim=0)
    W = P.random_weights(cfg, 1)
    toks = [3, 4, 5, 6, 7, 8, 9]
    base = P.forward(cfg, W, toks)[-1]
    inside = P.forward(cfg, W, toks[:3] + [11] + toks[4:])[-1]      # position 3 = 6 - 4 + 1: the window's last place
    outside = P.forward(cfg, W, toks[:2] + [11] + toks[3:])[-1]     # position 2: one too far
    assert not torch.allclose(inside, base, atol=1e-6) and torch.allclose(outside, base, atol=1e-12)
    # a very large sink takes all the weight: the mixer adds nothing, whatever the tokens before
    W2 = dict(W, **{"l0.mix.sink": torch.full((3,), 80.0)})
    a = P.forward(cfg, W2, toks)[-1]
    b = P.forward(cfg, W2, [1, 2, 1, 2, 1, 2, 9])[-1]
    assert torch.allclose(a, b, atol=1e-9)
    # and a sink far below every score is as good as none: a plain softmax
    h = torch.randn(5, 64, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    Wd = {k: v.double() for k, v in W.items()}
    m = dict(cfg["layers"][0]["mixer"])
    m.pop("mask")
    low = P.latent_attention(h, m, dict(Wd, **{"l0.mix.sink": torch.full((3,), -200.0, dtype=torch.float64)}), "l0.mix", 1e-5)
    T, H, dk, dv = 5, 3, 16, 24
    cq = P.rms_norm(h @ Wd["l0.mix.dq"].T, Wd["l0.mix.dq.norm"], 1e-5)
    c = P.rms_norm(h @ Wd["l0.mix.dkv"].T, Wd["l0.mix.dkv.norm"], 1e-5)
    q, k, v = (cq @ Wd["l0.mix.uq"].T).view(T, H, dk), (c @ Wd["l0.mix.uk"].T).view(T, H, dk), (c @ Wd["l0.mix.uv"].T).view(T, H, dv)
    rows = []
    for i in range(T):
        p = torch.softmax(torch.einsum("hd,jhd->hj", q[i], k[:i + 1]) * m["scale"], -1)
        rows.append(torch.einsum("hj,jhd->hd", p, v[:i + 1]).reshape(-1))
    assert torch.allclose(low, torch.stack(rows) @ Wd["l0.mix.o"].T, atol=1e-10)


def test_plain_norm_in_parts():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 24, dtype=torch.float64, generator=g) * torch.tensor([1.0] * 12 + [30.0] * 12, dtype=torch.float64)
    w = torch.randn(24, dtype=torch.float64, generator=g)
    whole, halves = P.grouped_rms_norm(x, w, 1e-6, 1), P.grouped_rms_norm(x, w, 1e-6, 2)
    assert torch.allclose(whole, P.rms_norm(x, w, 1e-6))
    assert torch.allclose(halves[:, :12], P.rms_norm(x[:, :12], w[:12], 1e-6)) and torch.allclose(halves[:, 12:], P.rms_norm(x[:, 12:], w[12:], 1e-6))
    assert not torch.allclose(whole, halves, atol=1e-2)


def test_plain_experts_take_their_score_at_the_input():
    cfg = P.tiny_config(layers=1, experts=3, top=2, shared_ff=0)
    W = {k: v.double() for k, v in P.random_weights(cfg, 4).items()}
    h = torch.randn(6, 64, dtype=torch.float64, generator=torch.Generator().manual_seed(5))
    mlp = cfg["layers"][0]["mlp"]
    picks = []
    y = P.routed_feed_forward(h, mlp, W, "l0.mlp", chosen=picks)
    s = P.sigmoid(h @ W["l0.mlp.router"].T)
    for t in range(6):
        order = sorted(range(3), key=lambda e: -float(s[t, e]))[:2]
        assert sorted(picks[0][0][t].tolist()) == sorted(order)
        want = sum(P.expert((h[t] * s[t, e])[None], W, f"l0.mlp.e{e}", mlp["expert"]["limit"])[0] for e in order)
        assert torch.allclose(y[t], want, atol=1e-12)
        at_output = sum(s[t, e] * P.expert(h[t][None], W, f"l0.mlp.e{e}", mlp["expert"]["limit"])[0] for e in order)
        assert not torch.allclose(y[t], at_output, atol=1e-4)     # (the activation is not linear: the place of the score shows)
    # the limits bind: a gate far above the limit gives what the limit gives
    g = torch.tensor([[50.0]], dtype=torch.float64)
    one = {"x.gate": torch.ones(1, 1, dtype=torch.float64), "x.up": torch.ones(1, 1, dtype=torch.float64), "x.down": torch.ones(1, 1, dtype=torch.float64)}
    assert torch.allclose(P.expert(g, one, "x", 2.0), 2.0 * P.sigmoid(torch.tensor(3.404, dtype=torch.float64)) * 3.0)
    assert torch.allclose(P.expert(-g, one, "x", 2.0), -50.0 * P.sigmoid(torch.tensor(-85.1, dtype=torch.float64)) * -1.0)
