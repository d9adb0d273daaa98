"""Bebuzen without a GPU: config.json's keys and their errors, the tensor names against the plain list, the cache entries a
model asks for (a reader of another layer's keys, kept first tokens), the pages a window with kept tokens holds on to, and
the plain implementation's own consistency."""
import copy

import pytest
import torch

import plain_bebuzen as P
from infinilm_amd.cache import CacheManager, FixedState, PagedKV
from infinilm_amd.config.errors import ConfigError
from infinilm_amd.config.registry import load_model_config
from infinilm_amd.engine.model import CausalLM


def _build(cfg):
    arch, c = load_model_config(cfg)
    spec = arch.build_spec(c)
    return spec, CausalLM(spec, torch.bfloat16, "meta")


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_tensor_names_and_shapes(name):
    cfg = P.CONFIGS[name]()
    spec, model = _build(cfg)
    assert {k: tuple(p.shape) for k, p in model.named_parameters().items()} == P.tensor_shapes(cfg)
    assert spec.architecture == "Bebuzen"


def test_cache_entries_of_a_reader_and_its_writer():
    spec, model = _build(P.config_a())
    runs = [(r.layer, r.cache, r.borrows) for r in spec.order]
    assert runs == [(0, 0, None), (1, 1, None), (2, 2, None), (3, 3, 1)]
    # the writer's cache keeps the wider of the two windows (33 and the reader's 50); the reader has its convolution's state alone
    assert model.cache_needs[0] == PagedKV(2, 32, 20, 3)
    assert model.cache_needs[1] == (PagedKV(1, 16, 50), FixedState((1, 2 * 2 * 8 + 1 * 2 * 8 + 12), torch.float32))
    assert model.cache_needs[3] == FixedState((1, 2 * 2 * 8), torch.float32)
    assert model.blocks[3].mixer.window == 50 and model.blocks[1].mixer.window == 33
    # a reader without a window makes the writer keep everything
    spec, model = _build(P.config_b())
    assert model.cache_needs[1][0] == PagedKV(6, 32, 0)
    assert [r.borrows for r in spec.order] == [None, None, None, None, 1]


def test_a_reader_without_a_convolution_has_no_entry_of_its_own():
    cfg = P.config_a()
    for i in (1, 3):
        del cfg["layers"][i]["mixer"]["conv"]
    spec, model = _build(cfg)
    assert [(r.cache, r.borrows) for r in spec.order] == [(0, None), (1, None), (2, None), (None, 1)]
    assert model.cache_needs[1] == PagedKV(1, 16, 50)
    assert {k: tuple(p.shape) for k, p in model.named_parameters().items()} == P.tensor_shapes(cfg)


def test_what_config_leaves_out_does_not_exist():
    cfg = P.config_b()
    _, model = _build(cfg)
    m2, m3 = model.blocks[2].mixer, model.blocks[3].mixer
    assert m2.position.rotary_dim == 0 and m2.window == 64 and m2.keep_first == 0
    assert m3.window == 0 and m3.keep_first == 0 and m3.position.rotary_dim == 20
    assert model.blocks[3].ffn is None and model.blocks[0].residual_scale == 1.0
    assert model.blocks[1].ffn.shared_ff == 0 and model.blocks[1].ffn.weight_scale == 1.0


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].__setitem__("type", "attention_3"), "attention_3"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("heads", 3), "heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 18), "dims"),
    (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("keep_first", -1), "keep_first"),
    (lambda c: c["layers"][1]["mixer"].pop("diff"), "diff"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 3), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 0), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("dim", 16), "dim"),
    (lambda c: c["layers"][2]["mixer"].pop("state"), "state"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 9), "top"),
    (lambda c: c["layers"][1]["mlp"].__setitem__("kind", "sparse"), "sparse"),
    (lambda c: c["layers"][0]["mlp"].pop("ff"), "ff"),
])
def test_config_errors_name_the_key(change, word):
    cfg = copy.deepcopy(P.config_a())
    change(cfg)
    with pytest.raises(ConfigError) as e:
        load_model_config(cfg)
    assert word in str(e.value)


def test_scaled_frequencies_against_their_definition():
    from infinilm_amd.models.bebuzen import rotary_frequencies
    rot = {"base": 5000.0, "dims": 32, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 128}}
    got = torch.tensor(rotary_frequencies(rot), dtype=torch.float64)
    assert torch.allclose(got, P.rotary_frequencies(rot), rtol=1e-14, atol=0)
    plain = torch.tensor(rotary_frequencies(dict(rot, scaling=None)), dtype=torch.float64)
    ratio = plain / got
    assert ratio[0] == 1.0 and abs(float(ratio[-1]) - 8.0) < 1e-12 and 1.0 < float(ratio[len(ratio) // 2 + 1]) <= 8.0
    assert (ratio[1:] >= ratio[:-1] - 1e-12).all()          # slower pairs are stretched more
    assert rotary_frequencies(None) == []


def test_pages_of_kept_first_tokens_stay():
    """Window 20 and 5 kept tokens on pages of 4: the pages of positions 0 .. 7 stay (the second one holds position 4), the
    window's pages come and go."""
    cm = CacheManager([PagedKV(1, 16, 20, 5), PagedKV(1, 16, 20)], page_size=4, num_pages=40, max_requests=2, dtype=torch.float32, device="cpu")
    assert len(cm.groups) == 2
    cm.admit("a")
    for n in (30, 1, 1, 17, 2):
        cm.reserve("a", n)
        cm.commit("a", n)
    length = cm.length("a")
    first = (length - 20 + 1) // 4
    kept, plain = cm.table("a", 0), cm.table("a", 1)
    assert [p >= 0 for p in kept[:first]] == [True, True] + [False] * (first - 2)
    assert all(p < 0 for p in plain[:first]) and all(p >= 0 for p in plain[first:]) and all(p >= 0 for p in kept[first:])
    cm.check()
    cm.release("a")
    assert cm.free_pages(0) == 40 and cm.free_pages(1) == 40


def test_the_plain_implementation_agrees_with_itself():
    """Logits of a prefix do not depend on what follows; a window wider than the sequence is no window; kept tokens beyond the
    sequence keep everything; the second map's weight vanishes where lambda does."""
    cfg = P.config_a()
    W = P.random_weights(cfg, 1)
    toks = list(range(60))
    full = P.forward(cfg, W, toks)
    assert torch.allclose(P.forward(cfg, W, toks[:41]), full[:41], atol=1e-10)
    wide = copy.deepcopy(cfg)
    wide["layers"][0]["mixer"]["mask"] = {"size": 1000}
    none = copy.deepcopy(cfg)
    del none["layers"][0]["mixer"]["mask"]
    kept = copy.deepcopy(cfg)
    kept["layers"][0]["mixer"]["mask"] = {"size": 2, "keep_first": 100}
    a, b, c = (P.forward(x, W, toks) for x in (wide, none, kept))
    assert torch.allclose(a, b, atol=1e-12) and torch.allclose(a, c, atol=1e-12) and not torch.allclose(a, full, atol=1e-6)
    assert bool(P.visible(5, 2, 1)[4].tolist() == [True, False, False, True, True])
