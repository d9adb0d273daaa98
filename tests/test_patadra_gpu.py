"""The Patadra design in the engine against the plain implementation (`plain_patadra.py`): the new kernels alone, every
mechanism alone in a one-layer model (with keys made to stand out far back, at page borders and on either side of a window's
edge), then whole models through the engine's own step function (whole prompts, decoding token by token, portions down to
two tokens, mixed batches with pages and slots used again, recorded decode steps) and through the entry point with its
scheduler (greedy generation).  Configurations A, B and C differ from each other in every size and switch: with and without a
loop (of two layers, two and three times), layers without a feed-forward, one, two and three experts a token, with and
without a shared expert, a token input and a cap, norms in one, two and four parts, windows shorter and longer than the
prompts and none at all, latent rows below and above the matrix-core kernels' head size, layers of unequal sizes.

bfloat16 and the routing: two experts whose scores are nearly equal may change places under rounding, and the token then
takes another expert.  Where whole models are compared in bfloat16 the plain implementation is therefore told which experts
the engine chose (`forced`), and the choice itself is checked apart: it may differ from the plain one only where the plain
scores of the exchanged experts are close."""
import json
import os

import pytest
import torch

import plain_patadra as P
from helpers import TOL, Driver, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, F32 = torch.bfloat16, torch.float32


def make_dir(path, cfg, W, store):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    save_file({k: v.to(getattr(torch, store)).contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return {k: v.to(getattr(torch, store)).to(torch.float32) for k, v in W.items()}


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def _close(got, want, tol, what):
    err = rel_err(got, want)
    assert err < tol, f"{what}: error {err:.3e}"


# ---- the kernels alone ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("H,groups", [(24, 1), (24, 3), (250, 5), (256, 4), (1000, 8), (4100, 2), (96, 96)])
def test_stream_update_adds_gates_norms(H, groups):
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(H + groups)
    T = 5
    r = torch.randn(T, H, generator=g)
    y = torch.randn(T, H, generator=g)
    z = 2.0 * torch.randn(T, H, generator=g)
    zb, bw, w = torch.randn(H, generator=g), 1.0 + 0.3 * torch.randn(H, generator=g), 1.0 + 0.3 * torch.randn(H, generator=g)
    parts = torch.randn(3, T, H, generator=g)
    eps = 1e-5
    # a gated branch, then the norm in parts
    want_r = r.double() + 0.5 * y.double() * P.sigmoid(z.double() + zb.double())
    rd = r.clone().to(DEV)
    x = kernels.stream_update(rd, y.to(DEV), 0.5, gate=z.to(DEV), gate_bias=zb.to(DEV), weight=w.to(DEV), eps=eps, groups=groups, out_dtype=F32)
    _close(rd.cpu(), want_r, 1e-6, "gated branch, residual")
    _close(x.cpu(), P.grouped_rms_norm(want_r, w.double(), eps, groups), 1e-5, "gated branch, normed rows")
    # a gate without a bias, bfloat16 branch, gate and result
    yb, zbf = y.to(BF), z.to(BF)
    want_r = r.double() + yb.double() * P.sigmoid(zbf.double())
    rd = r.clone().to(DEV)
    x = kernels.stream_update(rd, yb.to(DEV), 1.0, gate=zbf.to(DEV), weight=w.to(BF).to(DEV), eps=eps, groups=groups, out_dtype=BF)
    _close(rd.cpu(), want_r, 1e-6, "bfloat16 gated branch, residual")
    _close(x.cpu(), P.grouped_rms_norm(want_r, w.to(BF).double(), eps, groups), 1e-2, "bfloat16 gated branch, normed rows")
    # a branch with a norm of its own, arriving in parts
    want_r = r.double() - 2.0 * P.rms_norm(parts.double().sum(0), bw.double(), 1e-3)
    rd = r.clone().to(DEV)
    x = kernels.stream_update(rd, parts.to(DEV), -2.0, branch_weight=bw.to(DEV), branch_eps=1e-3, weight=w.to(DEV), eps=eps, groups=groups, out_dtype=F32)
    _close(rd.cpu(), want_r, 1e-5, "normed branch in parts, residual")
    _close(x.cpu(), P.grouped_rms_norm(want_r, w.double(), eps, groups), 1e-5, "normed branch in parts, normed rows")
    # a plain branch and the rows themselves as bfloat16; nothing to add and a norm alone; a sum alone
    rd = r.clone().to(DEV)
    x = kernels.stream_update(rd, y.to(DEV), 1.0, out_dtype=BF)
    _close(rd.cpu(), r.double() + y.double(), 1e-6, "plain branch")
    assert torch.equal(x.cpu(), rd.cpu().to(BF))
    x = kernels.stream_update(rd, weight=w.to(DEV), eps=eps, groups=groups, out_dtype=F32)
    _close(x.cpu(), P.grouped_rms_norm(rd.cpu().double(), w.double(), eps, groups), 1e-5, "norm alone")
    before = rd.cpu().double()
    assert kernels.stream_update(rd, y.to(DEV), 3.0) is None
    _close(rd.cpu(), before + 3.0 * y.double(), 1e-6, "sum alone")


def test_position_rows_token_gate_and_cap():
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(1)
    for dtype, tol in ((F32, 1e-6), (BF, 1e-6)):
        table, ptable = torch.randn(30, 72, generator=g).to(dtype), torch.randn(50, 72, generator=g).to(dtype)
        ids = torch.tensor([3, 29, 0, 3], dtype=torch.int32)
        pos = torch.tensor([0, 49, 7, 8], dtype=torch.int32)
        got = kernels.embed_positions(ids.to(DEV), pos.to(DEV), table.to(DEV), ptable.to(DEV), 1.5)
        assert got.dtype == F32
        _close(got.cpu(), 1.5 * table.double()[ids.long()] + ptable.double()[pos.long()], tol, "token rows plus position rows")
        side = torch.randn(30, 40, generator=g).to(dtype)
        z = (2.0 * torch.randn(4, 10, generator=g)).to(dtype)
        got = kernels.embed_gate(z.to(DEV), ids.to(DEV), side.to(DEV), 20)
        _close(got.cpu(), P.gelu_tanh(z.double()) * side.double()[ids.long()][:, 20:30], 1e-6 if dtype == F32 else 1e-2, "gated slice of a table")
    x = torch.tensor([[-300.0, -30.0, -1.0, 0.0, 0.5, 29.0, 1e4]])
    got = kernels.softcap_(x.clone().to(DEV), 30.0)
    _close(got.cpu(), 30.0 * torch.tanh(x.double() / 30.0), 1e-6, "capped numbers")
    gu = (3.0 * torch.randn(7, 26, generator=g))
    got = kernels.glu_clamp(gu.to(DEV), 2.0, 1.702)
    gg, uu = gu[:, :13].double().clamp(max=2.0), gu[:, 13:].double().clamp(-2.0, 2.0)
    _close(got.cpu(), gg * P.sigmoid(1.702 * gg) * (uu + 1.0), 1e-6, "the experts' activation")


@pytest.mark.parametrize("E,top", [(1, 1), (3, 1), (4, 2), (8, 3), (70, 4), (130, 130)])
def test_routing_takes_the_largest_scores(E, top):
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(E)
    T = 37
    z = torch.randn(T, E + 2, generator=g)
    if E > 2:
        z[0, :E] = 0.25                      # all equal: the lowest indices win
        z[1, 1], z[1, E - 1] = 9.0, 9.0      # a tie at the top
    plan = kernels.moe_route(z.to(DEV), E, top)
    ids, wts = plan.ids.cpu().long(), plan.weights.cpu()
    order = torch.sort(z[:, :E], dim=-1, descending=True, stable=True).indices[:, :top]
    assert torch.equal(ids, order)
    _close(wts, P.sigmoid(z[:, :E].double()).gather(1, order), 1e-6, "scores of the chosen experts")
    # every pair has one place in the order by expert, and the places of an expert lie together
    perm, inv, offs = plan.perm.cpu().long(), plan.inv.cpu().long(), plan.offsets.cpu().long()
    assert sorted(perm.tolist()) == list(range(T * top)) and torch.equal(perm[inv], torch.arange(T * top))
    flat = ids.reshape(-1)
    for e in range(E):
        assert (flat[perm[offs[e]:offs[e + 1]]] == e).all()
    assert int(offs[E]) == T * top


@pytest.mark.parametrize("T,H,K,N", [(1, 2, 8, 20), (5, 3, 16, 40), (40, 4, 64, 96), (64, 6, 32, 48), (100, 2, 136, 24), (128, 8, 128, 128),
                                     (7, 32, 128, 64), (17, 5, 72, 17)])
def test_product_per_head_for_few_rows_on_the_matrix_cores(T, H, K, N):
    """Rows whose strides allow 16-byte loads take the kernel without LDS: both layouts of W, outputs that end inside a tile of
    16, K that ends inside a step of 32, more rows than one workgroup's 64, columns beside the result left alone, and a row's
    result the same bits whatever rows lie beside it."""
    from infinilm_amd import kernels
    assert T <= kernels.HEAD_GEMM_MFMA_MAX_ROWS
    g = torch.Generator().manual_seed(T + K)
    x = torch.randn(T, H * (K + 8), generator=g).to(BF)
    w_kn = (torch.randn(H, K, N, generator=g) / K ** 0.5).to(BF)
    w_nk = (torch.randn(H, N, K, generator=g) / K ** 0.5).to(BF)
    xv = x.to(DEV).view(T, H, K + 8)[:, :, :K]
    kernels.enable_timing(True)
    try:
        kernels.timing_report()
        out = torch.zeros(T, H, N + 3, dtype=BF, device=DEV)
        kernels.head_gemm(xv, w_kn.to(DEV), out[:, :, :N])
        out2 = torch.empty(T, H, N, dtype=BF, device=DEV)
        kernels.head_gemm(xv, w_nk.to(DEV).transpose(1, 2), out2)
        assert set(kernels.timing_report()) == {"ilm_head_gemm_mfma"}, "the matrix-core kernel did not run"
    finally:
        kernels.enable_timing(False)
    _close(out[:, :, :N].cpu(), torch.einsum("thk,hkn->thn", xv.cpu().double(), w_kn.double()), 1e-2, "W with the outputs dense")
    assert float(out[:, :, N:].abs().max()) == 0.0
    _close(out2.cpu(), torch.einsum("thk,hnk->thn", xv.cpu().double(), w_nk.double()), 1e-2, "W with the inputs dense")
    one = torch.empty(1, H, N, dtype=BF, device=DEV)
    kernels.head_gemm(xv[T - 1:], w_nk.to(DEV).transpose(1, 2), one)
    assert torch.equal(one[0], out2[T - 1])


def test_routing_of_rows_without_numbers_stays_in_range():
    """A row of NaNs compares larger nowhere: it still gets valid experts, and every pair keeps its place in the order."""
    from infinilm_amd import kernels
    E, top, T = 6, 2, 9
    z = torch.randn(T, E, generator=torch.Generator().manual_seed(3))
    z[2] = float("nan")
    z[5, 1:] = float("nan")
    z[7] = float("-inf")
    plan = kernels.moe_route(z.to(DEV), E, top)
    ids = plan.ids.cpu().long()
    assert int(ids.min()) >= 0 and int(ids.max()) < E
    perm, inv = plan.perm.cpu().long(), plan.inv.cpu().long()
    assert sorted(perm.tolist()) == list(range(T * top)) and torch.equal(perm[inv], torch.arange(T * top))
    assert int(plan.offsets.cpu()[E]) == T * top
    assert ids[5, 0] == 0


def _experts(dtype, W, E, top, ff, limit, shared_ff, shared_limit, width):
    from infinilm_amd.config.spec import PartSpec
    from infinilm_amd.parts import BuildContext
    from infinilm_amd.parts.registry import build_feed_forward
    part = build_feed_forward(PartSpec("routed_experts", {"hidden_size": width, "experts": E, "top": top, "expert_ff": ff, "limit": limit,
                                                          "shared_ff": shared_ff, "shared_limit": shared_limit}),
                              BuildContext(dtype=dtype, device=torch.device(DEV)))
    for name, p in part.named_parameters().items():
        p.tensor.copy_(W["l0.mlp." + name].to(dtype))
    return part


@pytest.mark.parametrize("dtype", [F32, BF])
@pytest.mark.parametrize("T,width,E,top,ff,shared_ff", [(1, 64, 4, 2, 48, 40), (5, 96, 3, 1, 40, 0), (200, 64, 3, 2, 100, 24), (70, 100, 8, 3, 36, 20),
                                                        (300, 128, 2, 2, 64, 0), (33, 72, 16, 1, 8, 8), (150, 256, 8, 2, 192, 64), (700, 256, 4, 2, 136, 0), (1000, 192, 3, 3, 200, 64)])
def test_routed_experts_against_the_formula(T, width, E, top, ff, shared_ff, dtype):
    """The feed-forward alone: one token, few, and so many that an expert's rows fill several tiles; widths and inner sizes
    that are no multiples of 8 or 64 (the plain products in bfloat16 too); the score at the expert's input, limits that bind."""
    from infinilm_amd.parts.moe import RoutedExperts
    cfg = P.tiny_config(width=width, layers=1, experts=E, top=top, ff=ff, shared_ff=shared_ff, limit=0.8, side_dim=0)
    W = P.random_weights(cfg, T + E)
    W = {k: (v.to(dtype).float() if k.startswith("l0.mlp.") else v) for k, v in W.items()}
    mlp = cfg["layers"][0]["mlp"]
    h = (1.5 * torch.randn(T, width, generator=torch.Generator().manual_seed(7))).to(dtype)
    part = _experts(dtype, W, E, top, ff, 0.8, shared_ff, 1.3 if shared_ff else None, width)
    RoutedExperts.trace = []
    try:
        got = part.forward(h.to(DEV), None)
        picks = RoutedExperts.trace[0].cpu().long()
    finally:
        RoutedExperts.trace = None
    Wd = {k: v.double() for k, v in W.items()}
    chosen = []
    want = P.routed_feed_forward(h.double(), mlp, Wd, "l0.mlp", chosen=chosen)
    free, score = chosen[0]
    if dtype == BF:      # nearly equal scores may change places: checked apart, and the plain result follows the engine's choice
        differ = (torch.sort(picks, -1).values != torch.sort(free, -1).values).any(-1)
        for t in differ.nonzero().flatten().tolist():
            a, b = set(picks[t].tolist()), set(free[t].tolist())
            assert max(abs(float(score[t, i] - score[t, j])) for i in a - b for j in b - a) < 0.02, f"token {t}: experts {a} for {b}"
        assert differ.sum() <= max(1, T // 20)
        want = P.routed_feed_forward(h.double(), mlp, Wd, "l0.mlp", forced=picks)
        _close(got.cpu(), want, 2e-2, "bfloat16 experts")
    else:
        assert torch.equal(torch.sort(picks, -1).values, torch.sort(free, -1).values)
        _close(got.cpu(), want, 1e-5, "float32 experts")
    g_all = torch.einsum("tk,enk->ten", h.double(), torch.stack([Wd[f"l0.mlp.e{e}.gate"] for e in range(E)]))
    assert float(g_all.max()) > 0.8, "no gate reaches the limit: it would show nothing"


@pytest.mark.parametrize("T,width,E,top,ff,shared_ff", [(700, 256, 4, 2, 136, 0), (900, 320, 3, 2, 264, 0), (1000, 192, 3, 3, 200, 64)])
def test_routed_experts_in_wide_tiles(T, width, E, top, ff, shared_ff, monkeypatch):
    """The many-rows kernel with 256 rows of W a tile (an option): output slices that end inside a tile, experts with more and
    fewer rows than a tile."""
    from infinilm_amd import kernels
    monkeypatch.setattr(kernels, "MOE_WIDE", 1)
    test_routed_experts_against_the_formula(T, width, E, top, ff, shared_ff, BF)


# ---- the attention alone, with one key made to stand out ----------------------------------------------------------------
def _normed_row(cfg, W, token):
    return P.model_norm(cfg, W["embed"][token].double()[None], W["l0.norm1"].double())[0]


def _attention_with_a_marked_key(window, rank=40, heads=2, dim=16, vdim=12, q_rank=20):
    """One layer without a feed-forward.  Token 47's keys and token 48's queries point the same way in every head: that one
    score stands far above the others.  Position rows are small, so a token's normed row is nearly the same everywhere."""
    cfg = P.tiny_config(width=32, vocab=50, heads=heads, dim=dim, vdim=vdim, kv_rank=rank, q_rank=q_rank, window=window, layers=1,
                        mlp_at=[], side_dim=0, groups=2, scale=1.0, softcap=None, max_positions=1024)
    W = P.random_weights(cfg, 9)
    W["pos"] *= 0.02
    W["embed"][47], W["embed"][48] = (torch.eye(32)[0] + torch.eye(32)[16]) * 4, (torch.eye(32)[1] + torch.eye(32)[17]) * 4
    hk, hq = _normed_row(cfg, W, 47), _normed_row(cfg, W, 48)
    c = P.rms_norm((W["l0.mix.dkv"].double() @ hk)[None], W["l0.mix.dkv.norm"].double(), 1e-5)[0]
    cq = P.rms_norm((W["l0.mix.dq"].double() @ hq)[None], W["l0.mix.dq.norm"].double(), 1e-5)[0]
    key = (W["l0.mix.uk"].double() @ c).view(heads, dim)
    key = key / key.norm(dim=-1, keepdim=True) * 6.0
    uq = W["l0.mix.uq"].double()
    for h in range(heads):
        rows = slice(h * dim, (h + 1) * dim)
        uq[rows] -= torch.outer(uq[rows] @ cq - key[h], cq) / (cq @ cq)      # now W_uq,h c_q(48) = that key
    W["l0.mix.uq"] = uq.float()
    return cfg, W


def _run_last_tokens(tmp_path, cfg, W, toks, dtype, decoded=5, page=64):
    Wr = make_dir(str(tmp_path), cfg, W, dtype)
    want = P.forward(cfg, Wr, toks)
    drv = Driver(str(tmp_path), dtype, num_pages=-(-len(toks) // page) + 1, page_size=page, max_requests=2)
    if decoded < len(toks):
        drv.step([("a", toks[:len(toks) - decoded])])
    for t in toks[len(toks) - decoded:]:
        drv.step([("a", [t])])
    return drv.request_logits("a", len(toks)), want, Wr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decoded", [5, 0])
@pytest.mark.parametrize("back", [1, 63, 64, 65, 127, 128, 299, 300])
def test_window_finds_one_key_up_to_its_edge(dtype, decoded, back, tmp_path):
    """A window of 300 positions: the marked key lies `back` positions before the last query, next to it, on either side of a
    page border, and at the window's last place (299); one place further (300) it is outside and must not count.  In a
    prompt's portion and with the last tokens decoded one by one."""
    window, n = 300, 420
    cfg, W = _attention_with_a_marked_key(window)
    toks = [1 + (i % 40) for i in range(n)]
    toks[n - 1 - back], toks[-1] = 47, 48
    got, want, Wr = _run_last_tokens(tmp_path, cfg, W, toks, dtype, decoded=decoded if decoded else n)
    err = rel_err(got[-1], want[-1])
    assert err < TOL[dtype], f"key {back} back: {err:.3e}"
    moved = P.forward(cfg, Wr, toks[:n - 1 - back] + [2] + toks[n - back:])
    if back < window:
        assert rel_err(moved[-1], want[-1]) > 0.2, "the test's key does not matter: it would show nothing"
    else:
        assert rel_err(moved[-1], want[-1]) < 1e-9, "a key outside the window matters to the plain implementation"
        wider = json.loads(json.dumps(cfg))
        wider["layers"][0]["mixer"]["mask"]["size"] = window + 1
        assert rel_err(P.forward(wider, Wr, toks)[-1], want[-1]) > 0.2, "a window one too long would not show"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key_at", [0, 3, 63, 64, 127, 128, 640])
@pytest.mark.parametrize("rank", [40, 150])
def test_no_window_finds_a_key_far_back(dtype, key_at, rank, tmp_path):
    """A layer that sees every earlier token: the marked key is one among 700, at the very start, far back, or on either side
    of a page border.  Latent rows of 40 entries (64 in the cache: the matrix-core kernels in bfloat16) and of 150 (beyond
    them)."""
    cfg, W = _attention_with_a_marked_key(0, rank=rank)
    n = 700
    toks = [1 + (i % 40) for i in range(n)]
    toks[key_at], toks[-1] = 47, 48
    got, want, Wr = _run_last_tokens(tmp_path, cfg, W, toks, dtype)
    err = rel_err(got[-1], want[-1])
    assert err < TOL[dtype], f"key at {key_at}: {err:.3e}"
    moved = P.forward(cfg, Wr, toks[:key_at] + [2] + toks[key_at + 1:])
    assert rel_err(moved[-1], want[-1]) > 0.2, "the test's key does not matter: it would show nothing"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [1, 2, 3])
def test_first_tokens_and_short_windows(dtype, window, tmp_path):
    """Windows of one to three positions, pages of four: every token of a short sequence, decoded one by one from the first,
    and the same sequence as one prompt."""
    cfg, W = _attention_with_a_marked_key(window)
    toks = [47, 48, 47, 48, 3, 47, 9, 48, 48, 47, 2, 48]
    got, want, _ = _run_last_tokens(tmp_path / "d", cfg, W, toks, dtype, decoded=len(toks), page=4)
    _close(got, want, TOL[dtype], "every token of a short sequence, decoded")
    got, want, _ = _run_last_tokens(tmp_path / "p", cfg, W, toks, dtype, decoded=0, page=4)
    _close(got, want, TOL[dtype], "every token of a short sequence, as a prompt")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_sink_matters(dtype, tmp_path):
    """Sinks far from zero, positive and negative: the engine follows the plain implementation, whose result depends on them."""
    cfg, W = _attention_with_a_marked_key(50, heads=4, q_rank=24)
    W["l0.mix.sink"] = torch.tensor([3.0, -2.0, 6.0, 0.5])
    toks = tokens(cfg, 90, 4)
    got, want, Wr = _run_last_tokens(tmp_path, cfg, W, toks, dtype, decoded=30)
    _close(got, want, TOL[dtype], "sinks")
    no_sink = dict(Wr, **{"l0.mix.sink": torch.full((4,), -60.0)})
    assert rel_err(P.forward(cfg, no_sink, toks), want) > 0.05
    scaled = dict(Wr, **{"l0.mix.sink": Wr["l0.mix.sink"] * cfg["layers"][0]["mixer"]["scale"] * 0.5})
    assert rel_err(P.forward(cfg, scaled, toks), want) > 0.01


# ---- whole models through the step function -----------------------------------------------------------------------------
class RoutedDriver(Driver):
    """The helper's driver, which also files the experts the engine chose under (request, position)."""

    def __init__(self, *a, **k):
        super().__init__(*a, **k)
        self.picks = {}

    def step(self, entries, want_all=True, end=()):
        from infinilm_amd.parts.moe import RoutedExperts
        starts = [self.runner.cache.length(rid) if self.runner.cache.has(rid) else 0 for rid, _ in entries]
        RoutedExperts.trace = []
        try:
            super().step(entries, want_all=want_all, end=end)
            calls = [t.cpu().long() for t in RoutedExperts.trace]
        finally:
            RoutedExperts.trace = None
        row = 0
        for (rid, toks), s in zip(entries, starts):
            for i in range(len(toks)):
                self.picks[(rid, s + i)] = [c[row] for c in calls]
                row += 1

    def request_picks(self, rid, n):
        runs = len(self.picks[(rid, 0)])
        return [torch.stack([self.picks[(rid, i)][r] for i in range(n)]) for r in range(runs)]


CASES = [(c, d, p) for d in ("float32", "bfloat16") for c, p in (("A", 16), ("B", 64), ("C", 64), ("C", 16))]


@pytest.fixture(scope="module", params=CASES, ids=[f"{c}-{d}-p{p}" for c, d, p in CASES])
def case(request, tmp_path_factory):
    name, dtype, page = request.param
    cfg = P.CONFIGS[name]()
    d = tmp_path_factory.mktemp(f"patadra_{name}_{dtype}")
    W = make_dir(str(d), cfg, P.random_weights(cfg, 40 + ord(name)), dtype)
    toks = {r: tokens(cfg, n, 11 * i + 3) for i, (r, n) in
            enumerate([("r0", 300), ("r1", 1), ("r2", 45), ("r3", 70), ("r4", 2), ("r5", 131)])}
    free = {r: [] for r in toks}
    oracle = {r: P.forward(cfg, W, t, chosen=free[r]) for r, t in toks.items()}
    return {"cfg": cfg, "dir": str(d), "dtype": dtype, "toks": toks, "oracle": oracle, "free": free, "name": name, "page": page, "W": W}


def _check(case, drv, rid):
    """float32: every logit and every choice of experts as the plain implementation's.  bfloat16: the choices may differ where
    the plain scores are close (few of them), the logits follow the plain implementation run with the engine's choices, within
    the tolerance or twice what the plain implementation loses when it rounds at its projections."""
    cfg, W, toks = case["cfg"], case["W"], case["toks"][rid]
    n = len(toks)
    got = drv.request_logits(rid, n)
    picks = drv.request_picks(rid, n)
    free = case["free"][rid]
    assert len(picks) == len(free)
    want, tol = case["oracle"][rid], TOL[case["dtype"]]
    if case["dtype"] == "float32":
        for mine, (theirs, _) in zip(picks, free):
            assert torch.equal(torch.sort(mine, -1).values, torch.sort(theirs, -1).values), "another expert in float32"
    else:
        chosen = []
        want = P.forward(cfg, W, toks, forced=picks, chosen=chosen)
        changed = 0
        for mine, (theirs, score) in zip(picks, chosen):        # (scores as they are on the engine's own path)
            differ = (torch.sort(mine, -1).values != torch.sort(theirs, -1).values).any(-1)
            changed += int(differ.sum())
            for t in differ.nonzero().flatten().tolist():
                a, b = set(mine[t].tolist()), set(theirs[t].tolist())
                gap = max(abs(float(score[t, i] - score[t, j])) for i in a - b for j in b - a)
                assert gap < 0.03, f"{rid} token {t}: experts {sorted(a)} for {sorted(b)}, scores {gap:.3f} apart"
        assert changed <= max(2, len(picks) * n // 25), f"{changed} choices of {len(picks) * n} differ"
        tol = max(tol, 2.0 * rel_err(P.forward(cfg, W, toks, forced=picks, round_to=BF), want))
    err = rel_err(got, want)
    print(f"[err] {case['name']} {case['dtype']} {rid} n={n}: {err:.3e} (bound {tol:.3e})")
    assert err < tol, f"{case['name']} {case['dtype']} request {rid}: error {err:.3e} (bound {tol:.3e})"


def _pages(n, page):
    return -(-n // page)


def test_whole_requests(case):
    page = case["page"]
    drv = RoutedDriver(case["dir"], case["dtype"], num_pages=_pages(300, page) + 1, page_size=page, max_requests=2)
    for rid, t in case["toks"].items():
        drv.step([(rid, t)], end=[rid])
        _check(case, drv, rid)


def test_last_tokens_one_by_one(case):
    """The last 140 tokens decoded one by one (longer than any window but one, so windows pass over decoded tokens)."""
    page = case["page"]
    drv = RoutedDriver(case["dir"], case["dtype"], num_pages=_pages(300, page) + 1, page_size=page, max_requests=2)
    for rid, t in case["toks"].items():
        head = max(len(t) - 140, 0)
        if head:
            drv.step([(rid, t[:head])])
        for i in range(head, len(t)):
            drv.step([(rid, [t[i]])], end=[rid] if i == len(t) - 1 else [])
        _check(case, drv, rid)


def test_portions_of_changing_size(case):
    page = case["page"]
    drv = RoutedDriver(case["dir"], case["dtype"], num_pages=_pages(300, page) + 1, page_size=page, max_requests=2)
    sizes = [2, 5, page, 3, 2 * page + 1, 2, 17, page - 1, 1, 64]
    for rid, t in case["toks"].items():
        at, i = 0, 0
        while at < len(t):
            n = min(sizes[i % len(sizes)], len(t) - at)
            drv.step([(rid, t[at:at + n])], end=[rid] if at + n == len(t) else [])
            at, i = at + n, i + 1
        _check(case, drv, rid)


def test_mixed_steps_reuse_pages_and_slots(case):
    """Four request slots and pages for about two long requests serve six requests: portions of some beside single tokens of
    others; a request that ends frees its slot and pages for the next."""
    page, toks = case["page"], case["toks"]
    drv = RoutedDriver(case["dir"], case["dtype"], num_pages=_pages(300, page) + _pages(131, page) + 3, page_size=page, max_requests=4)
    at = {r: 0 for r in toks}

    def take(rid, n):
        a = at[rid]
        at[rid] = min(a + n, len(toks[rid]))
        return (rid, toks[rid][a:at[rid]])

    def run(plan):
        entries = [take(r, n) for r, n in plan if at[r] < len(toks[r])]
        if entries:
            drv.step(entries, end=[r for r, _ in entries if at[r] == len(toks[r])])

    run([("r1", 1), ("r0", 100), ("r2", 3)])
    run([("r0", 2), ("r2", 40), ("r4", 1)])
    run([("r0", 50), ("r2", 2), ("r4", 1), ("r3", 33)])       # r2 and r4 end: two slots free
    run([("r0", 1), ("r3", 1), ("r5", 64)])
    while any(at[r] < len(toks[r]) for r in ("r0", "r3", "r5")):
        run([("r0", 1), ("r3", 7), ("r5", 2)])
        run([("r0", 37), ("r3", 1), ("r5", 1)])
    for rid in toks:
        _check(case, drv, rid)
    assert drv.runner.cache.stats()["state_slots_free"] == 4


def test_recorded_decode_steps_equal_eager_ones(case):
    """Three requests decode side by side for 70 steps, once step by step and once with recorded steps switched on (one
    request ends on the way, so the recorded size changes): the same logits (32-bit: the same bits)."""
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    if case["page"] != 64:
        pytest.skip("one page size is enough here")
    toks = case["toks"]
    model = load_model(case["dir"], case["dtype"], DEV)
    ids = ["r0", "r3", "r5"]
    start = {"r0": 200, "r3": 20, "r5": 61}
    got = {}
    for graph in (False, True):
        runner = make_runner(model, num_pages=12, page_size=64, max_requests=4, enable_graph=graph)
        for r in ids:
            runner.cache.admit(r)
        runner.step([StepEntry(r, toks[r][:start[r]], []) for r in ids])
        rows = {r: [] for r in ids}
        for i in range(70):
            live = [r for r in ids if start[r] + i < len(toks[r])]
            out = runner.step([StepEntry(r, [toks[r][start[r] + i]], [0]) for r in live]).cpu()
            for j, r in enumerate(live):
                rows[r].append(out[j].clone())
            for r in live:
                if start[r] + i + 1 == len(toks[r]):
                    runner.cache.release(r)
        if graph:
            assert runner._graphs, "no step was recorded"
        got[graph] = {r: torch.stack(rows[r]) for r in ids}
    for r in ids:
        if case["dtype"] == "float32":
            assert torch.equal(got[True][r], got[False][r]), f"{r}: a recorded step differs from the eager one"
            _close(got[True][r], case["oracle"][r][start[r]:start[r] + len(got[True][r])], TOL["float32"], f"{r} against the plain implementation")
        else:
            _close(got[True][r], got[False][r], TOL["bfloat16"], f"{r}: recorded against eager")


def test_logits_do_not_depend_on_the_cut_in_32_bit(case):
    """float32: a request alone in one step, and the same request in portions beside another request, give the same logits
    up to the rounding of sums in another order."""
    if case["dtype"] != "float32":
        pytest.skip("the 32-bit path")
    page, toks = case["page"], case["toks"]
    a = Driver(case["dir"], "float32", num_pages=_pages(131, page) + 1, page_size=page, max_requests=2)
    a.step([("r5", toks["r5"])])
    b = Driver(case["dir"], "float32", num_pages=_pages(131, page) + _pages(70, page) + 2, page_size=page, max_requests=2)
    b.step([("r3", toks["r3"][:9]), ("r5", toks["r5"][:50])])
    b.step([("r5", toks["r5"][50:52]), ("r3", toks["r3"][9:])])
    b.step([("r5", toks["r5"][52:130])])
    b.step([("r5", toks["r5"][130:])])
    _close(b.request_logits("r5", 131), a.request_logits("r5", 131), 2e-6, "cut and batched against whole")


# ---- random configurations -----------------------------------------------------------------------------------------------
def _random_config(seed):
    """Two to four layers whose every size is drawn from a short list, layer by layer; a loop over a random stretch (or none);
    layers without a feed-forward, without a window, models without a token input, a cap or a shared expert now and then."""
    import random
    rnd = random.Random(seed)
    n = rnd.randint(2, 4)
    width = rnd.choice([48, 64, 96, 120, 128, 200])
    groups = rnd.choice([g for g in (1, 2, 3, 4, 8) if width % g == 0])
    mixers = [{"heads": rnd.choice([1, 2, 3, 5, 8, 16]), "dim": rnd.choice([8, 16, 24, 32, 64]), "vdim": rnd.choice([8, 20, 32, 48]),
               "kv_rank": rnd.choice([16, 24, 32, 64, 96, 112, 136]), "q_rank": rnd.choice([8, 20, 64]), "scale": rnd.choice([0.1, 0.25, 0.5])}
              for _ in range(n)]
    cfg = P.tiny_config(width=width, vocab=rnd.choice([50, 131, 640]), layers=n, experts=rnd.choice([1, 2, 4, 7, 8]), top=1,
                        ff=rnd.choice([8, 36, 64, 100]), shared_ff=rnd.choice([0, 16, 72]), groups=groups, side_dim=rnd.choice([0, 4, 12, 16]),
                        softcap=rnd.choice([None, 5.0, 30.0]), limit=rnd.choice([0.7, 2.0, 7.0]),
                        windows=[rnd.choice([None, 1, 2, 9, 31, 64, 65, 500]) for _ in range(n)], mixers=mixers,
                        mlp_at=[i for i in range(n) if rnd.random() < 0.8])
    for layer in cfg["layers"]:
        if layer["mlp"]:
            layer["mlp"]["router"]["top"] = rnd.randint(1, min(3, layer["mlp"]["router"]["experts"]))
            layer["mlp"]["expert"]["ff"] = rnd.choice([8, 36, 64, 100])
    if rnd.random() < 0.7:
        a = rnd.randrange(n)
        cfg["loop"] = {"start": a, "stop": rnd.randint(a + 1, n), "times": rnd.choice([1, 2, 3])}
    return cfg


@pytest.mark.parametrize("seed", range(16))
def test_random_configurations(seed, tmp_path):
    """A random configuration in 32-bit, two requests: one in portions beside the other's decoded tokens, on pages of 16 or 64
    with four slots; every logit against the plain implementation."""
    cfg = _random_config(seed)
    W = make_dir(str(tmp_path), cfg, P.random_weights(cfg, 100 + seed), "float32")
    ta, tb = tokens(cfg, 75, seed), tokens(cfg, 40, seed + 50)
    want_a, want_b = P.forward(cfg, W, ta), P.forward(cfg, W, tb)
    page = 16 if seed % 2 else 64
    drv = Driver(str(tmp_path), "float32", num_pages=-(-75 // page) + -(-40 // page) + 1, page_size=page, max_requests=4)
    drv.step([("a", ta[:33])])
    drv.step([("a", ta[33:35]), ("b", tb[:19])])
    drv.step([("a", ta[35:70]), ("b", tb[19:20])])
    for i in range(5):
        drv.step([("a", ta[70 + i:71 + i]), ("b", tb[20 + 4 * i:24 + 4 * i])])
    ea, eb = rel_err(drv.request_logits("a", 75), want_a), rel_err(drv.request_logits("b", 40), want_b)
    assert ea < TOL["float32"] and eb < TOL["float32"], f"seed {seed}: {ea:.3e}, {eb:.3e}; {json.dumps(cfg)}"


@pytest.mark.parametrize("seed", range(16, 24))
def test_random_configurations_in_bfloat16(seed, tmp_path):
    """The same in bfloat16, the plain implementation following the engine's choice of experts."""
    cfg = _random_config(seed)
    W = make_dir(str(tmp_path), cfg, P.random_weights(cfg, 100 + seed), "bfloat16")
    ta, tb = tokens(cfg, 75, seed), tokens(cfg, 40, seed + 50)
    page = 16 if seed % 2 else 64
    drv = RoutedDriver(str(tmp_path), "bfloat16", num_pages=-(-75 // page) + -(-40 // page) + 1, page_size=page, max_requests=4)
    drv.step([("a", ta[:33])])
    drv.step([("a", ta[33:35]), ("b", tb[:19])])
    drv.step([("a", ta[35:70]), ("b", tb[19:20])])
    for i in range(5):
        drv.step([("a", ta[70 + i:71 + i]), ("b", tb[20 + 4 * i:24 + 4 * i])])
    for rid, t in (("a", ta), ("b", tb)):
        picks = drv.request_picks(rid, len(t)) if any(layer["mlp"] for layer in cfg["layers"]) else None
        want = P.forward(cfg, W, t, forced=picks)
        lossy = P.forward(cfg, W, t, forced=picks, round_to=BF)
        # A branch that is divided by its own root mean square (the token input, a few numbers wide here) multiplies a rounding
        # error many times at the positions where that root mean square happens to be small, so single positions err several
        # times more than most, in the plain implementation with rounded products too, at positions of its own.  The engine is
        # held to that implementation's errors: at most positions (the median) closely, at the worst position loosely.
        top = max(1.0, float(want.abs().max()))
        e = (drv.request_logits(rid, len(t)).double() - want).abs().amax(-1) / top
        l = (lossy - want).abs().amax(-1) / top
        what = f"seed {seed} request {rid}: median {float(e.median()):.3e} (plain, rounded: {float(l.median()):.3e}), " \
               f"worst {float(e.max()):.3e} ({float(l.max()):.3e}); {json.dumps(cfg)}"
        assert float(e.median()) < max(TOL["bfloat16"] / 8, 1.5 * float(l.median())), what
        assert float(e.max()) < max(TOL["bfloat16"], 5.0 * float(l.max())), what


# ---- the entry point and its scheduler ------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,graph", [("A", False), ("B", False), ("B", True), ("C", True)])
def test_greedy_generation_through_the_entry_point(name, graph, tmp_path):
    """Five prompts through `LLM.generate` with three request slots, prompts cut into portions of five tokens under a token
    budget, and few pages: every request's greedy tokens are the plain implementation's (32-bit)."""
    from infinilm_amd import LLM, SamplingParams
    cfg = P.CONFIGS[name]()
    W = make_dir(str(tmp_path), cfg, P.random_weights(cfg, 7), "float32")
    prompts = [tokens(cfg, n, 50 + n) for n in (9, 1, 23, 4, 40)]
    llm = LLM(str(tmp_path), dtype="float32", num_blocks=10, block_size=16, max_batch_size=3, chunk_size=5,
              max_num_batched_tokens=11, enable_graph=graph)
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(top_k=1, max_tokens=12))
    for p, o in zip(prompts, outs):
        assert o.outputs[0].token_ids == P.greedy(cfg, W, p, 12), f"prompt of {len(p)} tokens"
    llm.close()


def test_long_decoding(tmp_path):
    """460 tokens decoded one by one after a prompt of 40 on few pages (windows pass, pages are given back and used again):
    the logits along the way against the plain implementation."""
    cfg = P.config_a()
    W = make_dir(str(tmp_path), cfg, P.random_weights(cfg, 12), "float32")
    toks = tokens(cfg, 500, 8)
    want = P.forward(cfg, W, toks)
    drv = Driver(str(tmp_path), "float32", num_pages=3, page_size=16, max_requests=2)
    drv.step([("a", toks[:40])])
    for t in toks[40:]:
        drv.step([("a", [t])])
    _close(drv.request_logits("a", 500), want, TOL["float32"], "long decoding")
