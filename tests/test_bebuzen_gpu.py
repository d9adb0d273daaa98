"""The Bebuzen design in the engine against the plain implementation (`plain_bebuzen.py`): the new kernels alone, every
mechanism alone in a one-layer model (with a key made to stand out far back, at page borders, on either side of a window's edge
and among the kept first tokens), then whole models through the engine's own step function (whole prompts, decoding token by
token, portions down to two tokens, mixed batches with pages and slots used again, recorded decode steps) and through the
entry point with its scheduler (greedy generation).  Configurations A, B and C differ in every size and switch: heads of 8 to 64
entries, with and without rotation, scaling, windows, kept tokens, convolutions of 2 to 4 taps, a reader of another layer's
keys with a wider window than the writer's and one without any, one to three experts a token with and without a shared one,
layers without a feed-forward, a scan with 5, 16 and 20 state entries a channel.

bfloat16 and the routing: two experts whose scores are nearly equal may change places under rounding; where whole models are
compared in bfloat16 the plain implementation is told which experts the engine chose, and the choices may differ from the
plain ones only in few places."""
import json
import math
import os

import pytest
import torch

import plain_bebuzen as P
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
def _paged(k, v, page, d, dtype, shuffle_seed=0):
    """k [n, G, dk], v [n, G, dv] of one request -> caches with the pages in a shuffled order, and its block table."""
    n, G = k.shape[0], k.shape[1]
    pages = -(-n // page)
    order = torch.randperm(pages + 2, generator=torch.Generator().manual_seed(shuffle_seed))[:pages]
    kc = torch.zeros((pages + 2, G, page, d), dtype=dtype)
    vc = torch.zeros((pages + 2, G, d, page), dtype=dtype)
    for j in range(n):
        pg, off = int(order[j // page]), j % page
        kc[pg, :, off, :k.shape[2]] = k[j].to(dtype)
        vc[pg, :, :v.shape[2], off] = v[j].to(dtype)
    return kc.to(DEV), vc.to(DEV), order.to(torch.int32)[None].contiguous().to(DEV)


@pytest.mark.parametrize("dtype", [F32, BF])
@pytest.mark.parametrize("H,G,maps,dim,vdim,window,keep,sink,page", [
    (4, 2, 2, 8, 12, 33, 0, False, 16), (6, 6, 2, 12, 8, 0, 0, False, 4), (2, 1, 2, 24, 40, 70, 0, False, 64),
    (3, 1, 1, 20, 36, 20, 3, True, 16), (4, 2, 1, 16, 16, 50, 70, True, 8), (2, 2, 1, 10, 6, 0, 0, True, 16),
    (1, 1, 2, 5, 3, 1, 0, False, 4), (2, 1, 1, 6, 6, 2, 1, True, 4)])
def test_attention_in_maps_against_the_formula(H, G, maps, dim, vdim, window, keep, sink, page, dtype):
    """Two requests of 150 and 37 tokens in one launch, every token of both."""
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(H * 100 + dim)
    d = -(-max(maps * dim, vdim) // 16) * 16
    lens = [150, 37]
    outs, wants = [], []
    lam = [0.4 * torch.randn(dim, generator=g) for _ in range(4)]
    diff, eps, scale = 0.35, 1e-5, 0.3
    qs, tables, kcs, vcs = [], [], [], []
    for r, n in enumerate(lens):
        q = torch.randn(n, H, maps, dim, generator=g)
        k = torch.randn(n, G, maps, dim, generator=g)
        v = torch.randn(n, G, vdim, generator=g)
        if dtype == BF:
            q, k, v = (t.to(BF).float() for t in (q, k, v))
        mask = P.visible(n, window or None, keep)
        a = [P.softmax_attention(q[:, :, m].double(), k[:, :, m].double(), v.double(), scale, mask, sink) for m in range(maps)]
        if maps == 2:
            lv = [t.to(dtype).double() for t in lam]
            lmb = torch.exp((lv[0] * lv[1]).sum()) - torch.exp((lv[2] * lv[3]).sum()) + diff
            want = P.rms(a[0] - lmb * a[1], eps) * (1.0 - diff)
        else:
            want = a[0]
        wants.append(want.reshape(n, H * vdim))
        kc, vc, bt = _paged(k.reshape(n, G, maps * dim), v, page, d, dtype, r)
        qs.append(q.reshape(n, -1))
        kcs.append(kc); vcs.append(vc); tables.append(bt)
    # one cache for both requests: the second one's pages behind the first one's
    off = kcs[0].shape[0]
    kc, vc = torch.cat(kcs), torch.cat(vcs)
    width = max(t.shape[1] for t in tables)
    bt = torch.full((2, width), -1, dtype=torch.int32, device=DEV)
    bt[0, :tables[0].shape[1]] = tables[0][0]
    bt[1, :tables[1].shape[1]] = tables[1][0] + off
    seg = torch.cat([torch.full((n,), r, dtype=torch.int32) for r, n in enumerate(lens)]).to(DEV)
    pos = torch.cat([torch.arange(n, dtype=torch.int32) for n in lens]).to(DEV)
    q = torch.cat(qs).to(dtype).to(DEV).contiguous()
    got = kernels.maps_attention(q, kc, vc, bt, seg, pos, H, G, maps, dim, vdim, scale, window, keep,
                                 torch.zeros(H, device=DEV) if sink else None, [t.to(dtype).to(DEV) for t in lam] if maps == 2 else None,
                                 diff, eps if maps == 2 else -1.0, 1.0 - diff if maps == 2 else 1.0)
    _close(got.float().cpu(), torch.cat(wants), 2e-5 if dtype == F32 else 2e-2, "attention in maps")


@pytest.mark.parametrize("dtype", [F32, BF])
@pytest.mark.parametrize("H,G,dim,vdim,rd,own", [(4, 2, 8, 12, 8, True), (3, 1, 20, 6, 4, True), (2, 2, 16, 16, 0, True), (4, 2, 8, 12, 6, False)])
def test_norm_rotation_and_cache_write_in_maps(H, G, dim, vdim, rd, own, dtype):
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(dim + rd)
    T, page, eps = 11, 4, 1e-5
    Cq, Ck, Cv = H * 2 * dim, G * 2 * dim, G * vdim
    d = -(-max(2 * dim, vdim) // 16) * 16
    src = torch.randn(T, 3 + Cq + Ck + Cv, generator=g)          # (wider rows: the pieces start at entry 3)
    wq, wk = 1.0 + 0.3 * torch.randn(dim, generator=g), 1.0 + 0.3 * torch.randn(dim, generator=g)
    rot = {"base": 77.0, "dims": rd, "scaling": {"factor": 3.0, "low": 1.0, "high": 2.0, "original": 40}} if rd else None
    freq = P.rotary_frequencies(rot).float().to(DEV) if rd else None
    pos = torch.tensor([5, 6, 7, 0, 1, 2, 3, 200, 201, 40, 41], dtype=torch.int32)
    slots = torch.tensor([20, 21, 22, 4, 5, 6, 7, 12, 13, 30, 31], dtype=torch.int32)
    kc = torch.zeros((9, G, page, d), dtype=dtype, device=DEV)
    vc = torch.zeros((9, G, d, page), dtype=dtype, device=DEV)
    wd = wq.to(dtype).to(DEV), wk.to(dtype).to(DEV)
    q = kernels.maps_norm_rope_kvwrite(src.to(DEV), 3, 3 + Cq if own else -1, 3 + Cq + Ck, pos.to(DEV), freq, wd[0], wd[1] if own else None,
                                       kc, vc, slots.to(DEV) if own else None, H, G, 2, dim, vdim, rd, eps, dtype)
    x = src.double()
    wqd, wkd = wd[0].double().cpu(), wd[1].double().cpu()
    want_q = P.rotate(P.rms(x[:, 3:3 + Cq].reshape(T, H * 2, dim), eps, wqd), pos, rot, "half").reshape(T, Cq)
    tol = 3e-5 if dtype == F32 else 1e-2      # (angles are formed in float32: position 200 x a rate near 1 carries 1e-5)
    _close(q.float().cpu(), want_q, tol, "queries")
    if not own:
        assert float(kc.float().abs().max()) == 0.0 and float(vc.float().abs().max()) == 0.0
        return
    want_k = P.rotate(P.rms(x[:, 3 + Cq:3 + Cq + Ck].reshape(T, G * 2, dim), eps, wkd), pos, rot, "half").reshape(T, G, 2 * dim)
    want_v = x[:, 3 + Cq + Ck:].reshape(T, G, vdim)
    for t in range(T):
        pg, off = int(slots[t]) // page, int(slots[t]) % page
        _close(kc[pg, :, off, :2 * dim].float().cpu(), want_k[t], tol, f"key of token {t}")
        _close(vc[pg, :, :vdim, off].float().cpu(), want_v[t], tol, f"value of token {t}")
        assert float(kc[pg, :, off, 2 * dim:].float().abs().max()) == 0.0 if d > 2 * dim else True


@pytest.mark.parametrize("dtype", [F32, BF])
@pytest.mark.parametrize("inner,state,lens1,lens2,pieces", [(48, 5, [7, 1, 30], [4, 9, 2], False), (160, 20, [7, 1, 30], [4, 9, 2], False),
                                                            (64, 16, [7, 1, 30], [4, 9, 2], False), (33, 1, [7, 1, 30], [4, 9, 2], False),
                                                            (20, 70, [7, 1, 30], [4, 9, 2], False), (64, 16, [200, 1, 64], [65, 130, 2], True),
                                                            (40, 3, [129, 300, 5], [1, 128, 127], True), (70, 40, [140, 2, 1], [3, 190, 64], True),
                                                            (256, 16, [7, 1, 30], [4, 9, 2], False), (300, 5, [17, 1, 33], [1, 16, 2], False),
                                                            (512, 32, [200, 1, 64], [65, 130, 2], True), (260, 3, [129, 300, 5], [1, 128, 127], True)])
def test_selective_scan_carries_its_state(inner, state, lens1, lens2, pieces, dtype):
    """Three requests of unequal length over two launches; the second launch starts from the rows the first left, one
    request starts anew in a row that was used before.  `pieces`: segments long enough to be cut into pieces of 64 tokens that
    run side by side (lengths on either side of a piece's edge).  From 256 channels on, states of up to 32 entries take the form
    with a thread a channel."""
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(inner + state)
    a_log = torch.log(0.3 + 3.0 * torch.rand(inner, state, generator=g))
    skip, bias = torch.randn(inner, generator=g), -2.0 + torch.randn(inner, generator=g)
    pool = torch.zeros((6, inner, state), device=DEV)
    pool[5] = 7.0                                                # (stale content of a row that is used again)
    seqs = []
    for n1, n2 in zip(lens1, lens2):
        n = n1 + n2
        seqs.append({k: torch.randn(n, w, generator=g) for k, w in (("x", inner), ("raw", inner), ("z", inner), ("B", state), ("C", state))})

    def plain(s, n0, n1, S):
        ys = []
        rd = lambda t: t.to(dtype).double()
        for t in range(n0, n1):
            dt = torch.nn.functional.softplus(rd(s["raw"][t]) + rd(bias) if dtype == BF else s["raw"][t].double() + bias.double())
            xv = s["x"][t].double()
            S = torch.exp(dt[:, None] * -torch.exp(a_log.double())) * S + (dt * xv)[:, None] * rd(s["B"][t])[None, :]
            ys.append((S @ rd(s["C"][t]) + skip.double() * xv) * P.silu(rd(s["z"][t])))
        return torch.stack(ys), S

    def launch(ranges, rows_in, rows_out):
        cat = lambda k, dt: torch.cat([s[k][a:b] for s, (a, b) in zip(seqs, ranges)]).to(dt).to(DEV)
        offs = [0]
        for a, b in ranges:
            offs.append(offs[-1] + b - a)
        bc = torch.cat([cat("B", dtype), cat("C", dtype)], 1)
        return kernels.selective_scan(cat("x", F32), cat("raw", dtype), bias.to(dtype).to(DEV), bc[:, :state], bc[:, state:], cat("z", dtype),
                                      a_log.to(DEV), skip.to(DEV), pool, torch.tensor(rows_in, dtype=torch.int32, device=DEV),
                                      torch.tensor(rows_out, dtype=torch.int32, device=DEV), torch.tensor(offs, dtype=torch.int32, device=DEV),
                                      len(ranges), max_len=max(b - a for a, b in ranges) if pieces else None).float().cpu()

    got1 = launch([(0, n) for n in lens1], [0, 0, 0], [1, 2, 5])
    got2 = launch([(n1, n1 + n2) for n1, n2 in zip(lens1, lens2)], [1, 2, 5], [1, 2, 5])
    tol = 2e-5 if dtype == F32 else 2e-2
    o1 = o2 = 0
    for s, n1, n2 in zip(seqs, lens1, lens2):
        y1, S = plain(s, 0, n1, torch.zeros(inner, state, dtype=torch.float64))
        y2, S = plain(s, n1, n1 + n2, S)
        _close(got1[o1:o1 + n1], y1, tol, "first launch")
        _close(got2[o2:o2 + n2], y2, tol, "second launch")
        o1, o2 = o1 + n1, o2 + n2
    _close(pool[5].cpu(), S, tol, "the state a request left")


@pytest.mark.parametrize("dtype", [F32, BF])
@pytest.mark.parametrize("T,width,E,top,ff,shared_ff,scale", [(1, 64, 4, 2, 24, 16, 1.5), (5, 96, 3, 1, 20, 0, 1.0), (200, 64, 8, 3, 100, 24, 2.0),
                                                           (70, 100, 5, 5, 36, 20, 0.5), (300, 128, 2, 1, 64, 64, 1.0),
                                                           (9, 2048, 2, 1, 4096, 0, 1.0), (40, 2048, 3, 2, 4160, 0, 1.0)])
def test_softmax_routed_experts_against_the_formula(T, width, E, top, ff, shared_ff, scale, dtype):
    """(The last two shapes are large enough for the few-rows kernel that takes two blocks of outputs a workgroup; 4160 leaves
    its last block half empty.)"""
    from infinilm_amd.parts.base import BuildContext
    from infinilm_amd.parts.moe import RoutedActivationExperts
    g = torch.Generator().manual_seed(T + E)
    ml = {"kind": "moe", "router": {"experts": E, "top": top, "scale": scale}, "expert": {"ff": ff}}
    if shared_ff:
        ml["shared"] = {"ff": shared_ff}
    W = {"router": 3.0 * torch.randn(E, width, generator=g) / math.sqrt(width)}
    for e in range(E):
        W[f"e{e}.up"] = torch.randn(ff, width, generator=g) / math.sqrt(width)
        W[f"e{e}.down"] = torch.randn(width, ff, generator=g) / math.sqrt(ff)
    if shared_ff:
        W["shared.up"] = torch.randn(shared_ff, width, generator=g) / math.sqrt(width)
        W["shared.down"] = torch.randn(width, shared_ff, generator=g) / math.sqrt(shared_ff)
    part = RoutedActivationExperts(width, E, top, ff, BuildContext(dtype, torch.device(DEV)), weight_scale=scale, shared_ff=shared_ff)
    for name, p in part.named_parameters().items():
        p.store(W[name].to(DEV))
    Wr = {k: v.to(dtype).double() for k, v in W.items()}
    x = torch.randn(T, width, generator=g).to(dtype)
    RoutedActivationExperts.trace = []
    try:
        got = part.forward(x.to(DEV), None).float().cpu()
        picks = RoutedActivationExperts.trace[0].cpu().long()
    finally:
        RoutedActivationExperts.trace = None
    chosen = []
    want = P.feed_forward(Wr, "", ml, x.double(), forced=picks, chosen=chosen)
    own = chosen[0][0]
    differ = int((torch.sort(own, -1).values != torch.sort(picks, -1).values).any(-1).sum())
    assert differ <= (0 if dtype == F32 else max(1, T // 20)), f"{differ} of {T} tokens took other experts"
    _close(got, want, 2e-5 if dtype == F32 else 3e-2, "routed experts")


# ---- one mechanism in a one-layer model, a key made to stand out -----------------------------------------------------------
def _one_layer(kind, mixer):
    return {"architecture": "Bebuzen", "vocab": 50, "width": 32, "norm": {"eps": 1e-5}, "residual_mult": 1.0,
            "layers": [{"type": kind, "mixer": mixer, "mlp": None}]}


def _last_logits(tmp_path, cfg, W, toks, dtype, decoded, page):
    """Engine logits of the last token (the prompt in one step, the last `decoded` tokens one by one), the plain ones, and the
    weights as stored."""
    d = str(tmp_path / f"m_{dtype}_{decoded}_{page}_{len(toks)}")
    Wr = make_dir(d, cfg, W, dtype)
    drv = Driver(d, dtype, num_pages=-(-len(toks) // page) + 1, page_size=page, max_requests=2)
    head = len(toks) - decoded
    if head:
        drv.step([("a", toks[:head])])
    for i in range(head, len(toks)):
        drv.step([("a", [toks[i]])])
    return drv.logits[("a", len(toks) - 1)], Wr


def _marked(cfg, W, toks, key_at, p="l0.mix."):
    """Makes the last token's query and the key at `key_at` stand out: both tokens are one that occurs nowhere else, whose
    embedding is large, so that the score between them dominates if the key is seen."""
    toks = list(toks)
    special = cfg["vocab"] - 1
    toks = [t if t != special else 0 for t in toks]
    toks[key_at] = special
    toks[-1] = special
    W = dict(W)
    W["embed"] = W["embed"].clone()
    W["embed"][special] *= 6.0
    return toks, W


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decoded", [4, 0])
@pytest.mark.parametrize("back", [1, 15, 16, 17, 63, 64, 65, 99, 100, 101])
def test_differential_window_finds_one_key_up_to_its_edge(dtype, decoded, back, tmp_path):
    """Window of 100 on pages of 16: a marked token `back` positions before the last one.  It enters its own key and, through
    the convolution of two taps, the next one, so it shows up to 100 back and not at 101; the logits follow the plain
    implementation on both sides."""
    mixer = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 12, "scale": 1.0, "diff": 0.3, "conv": 2, "rot": {"base": 50.0, "dims": 4},
             "mask": {"size": 100}}
    cfg = _one_layer("attention", mixer)
    W = P.random_weights(cfg, 5)
    n = 230
    toks, Wm = _marked(cfg, W, tokens(cfg, n, 9), n - 1 - back)
    got, Wr = _last_logits(tmp_path, cfg, Wm, toks, dtype, decoded, 16)
    want = P.forward(cfg, Wr, toks)[-1]
    _close(got, want, TOL[dtype], f"key {back} back")
    plain_toks = list(toks)
    plain_toks[n - 1 - back] = 1
    moved = rel_err(P.forward(cfg, Wr, plain_toks)[-1], want)
    assert (moved > 1e-3) == (back <= 100), f"a token {back} back moves the logits by {moved:.2e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decoded", [4, 0])
@pytest.mark.parametrize("key_at,seen", [(0, True), (2, True), (3, False), (15, False), (16, False), (189, False), (190, True), (191, True), (228, True)])
def test_window_with_kept_first_tokens(dtype, decoded, key_at, seen, tmp_path):
    """Window of 40, the first 3 tokens kept, 230 tokens on pages of 16: a marked key is seen among the kept tokens and inside
    the window, and nowhere between."""
    mixer = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 1.0, "rot": {"base": 50.0, "dims": 4}, "mask": {"size": 40, "keep_first": 3}}
    cfg = _one_layer("attention_2", mixer)
    W = P.random_weights(cfg, 6)
    n = 230
    toks, Wm = _marked(cfg, W, tokens(cfg, n, 10), key_at)
    got, Wr = _last_logits(tmp_path, cfg, Wm, toks, dtype, decoded, 16)
    want = P.forward(cfg, Wr, toks)[-1]
    _close(got, want, TOL[dtype], f"key at {key_at}")
    plain_toks = list(toks)
    plain_toks[key_at] = 1
    moved = rel_err(P.forward(cfg, Wr, plain_toks)[-1], want)
    assert (moved > 1e-3) == seen, f"key at {key_at} moves the logits by {moved:.2e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_kept_first_tokens_on_the_matrix_cores(dtype, tmp_path):
    """Heads of 64 on pages of 64 (the bfloat16 kernel's sizes), window 70, five kept tokens, 300 tokens: prompt and decoded."""
    mixer = {"heads": 4, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.125, "rot": {"base": 1000.0, "dims": 32},
             "mask": {"size": 70, "keep_first": 5}}
    cfg = _one_layer("attention_2", mixer)
    cfg["width"] = 64
    W = P.random_weights(cfg, 8)
    for key_at in (1, 4, 5, 100, 230, 231):
        toks, Wm = _marked(cfg, W, tokens(cfg, 300, 12), key_at)
        d = str(tmp_path / f"k{key_at}")
        Wr = make_dir(d, cfg, Wm, dtype)
        want = P.forward(cfg, Wr, toks)
        drv = Driver(d, dtype, num_pages=6, page_size=64, max_requests=2)
        drv.step([("a", toks[:290])])
        for i in range(290, 300):
            drv.step([("a", [toks[i]])])
        _close(drv.request_logits("a", 300), want, TOL[dtype], f"key at {key_at}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv,dim,vdim", [(4, 2, 64, 128), (6, 1, 32, 96), (2, 2, 32, 40), (5, 1, 32, 64)])
def test_differential_attention_on_the_matrix_cores(dtype, heads, kv, dim, vdim, tmp_path):
    """Maps of 32 and 64 on pages of 64 and 32 (the bfloat16 kernels' sizes; five heads leave a wave idle), window 70, 300
    tokens: a portion from the start, a portion with history that begins inside a page, two tokens, then decoded tokens (the
    chunked kernel); beside it a second request, so that steps hold tiles and single rows."""
    mixer = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "diff": 0.4, "conv": 2,
             "rot": {"base": 1000.0, "dims": dim // 2}, "mask": {"size": 70}}
    cfg = _one_layer("attention", mixer)
    cfg["width"] = 64
    W = P.random_weights(cfg, 11)
    toks, other = tokens(cfg, 300, 13), tokens(cfg, 40, 14)
    for page in (64, 32):
        d = str(tmp_path / f"p{page}")
        Wr = make_dir(d, cfg, W, dtype)
        drv = Driver(d, dtype, num_pages=-(-300 // page) + 3, page_size=page, max_requests=2)
        drv.step([("a", toks[:150])])
        drv.step([("a", toks[150:271]), ("b", other[:1])])
        drv.step([("a", toks[271:273]), ("b", other[1:2])])
        drv.step([("a", toks[273:274]), ("b", other[2:30])])
        for i in range(274, 300):
            drv.step([("a", [toks[i]])] + ([("b", [other[30 + i - 274]])] if 30 + i - 274 < 40 else []))
        _close(drv.request_logits("a", 300), P.forward(cfg, Wr, toks), TOL[dtype], f"pages of {page}")
        _close(drv.request_logits("b", 40), P.forward(cfg, Wr, other), TOL[dtype], f"second request, pages of {page}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_unit_term_of_the_denominator_matters(dtype, tmp_path):
    mixer = {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.05, "mask": {"size": 30}}
    cfg = _one_layer("attention_2", mixer)
    W = P.random_weights(cfg, 7)
    toks = tokens(cfg, 50, 3)
    got, Wr = _last_logits(tmp_path, cfg, W, toks, dtype, 5, 16)
    want = P.forward(cfg, Wr, toks)[-1]
    _close(got, want, TOL[dtype], "unit term")
    # the first token sees one key of score near 0: half of its weight goes to the term that has no value
    d = str(tmp_path / "first")
    make_dir(d, cfg, W, dtype)
    drv = Driver(d, dtype, num_pages=2, page_size=16, max_requests=1)
    drv.step([("a", toks[:1])])
    _close(drv.logits[("a", 0)], P.forward(cfg, Wr, toks[:1])[0], TOL[dtype], "first token")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_scan_remembers_through_portions(dtype, tmp_path):
    """Slow decays: a token 300 positions back still shows, through portions of odd sizes and decoded tokens."""
    cfg = _one_layer("mamba1", {"inner": 40, "state": 6, "dt_rank": 4, "conv": 3})
    W = P.random_weights(cfg, 9)
    W["l0.mix.A_log"] = torch.full_like(W["l0.mix.A_log"], -4.0)
    toks = tokens(cfg, 320, 4)
    d = str(tmp_path / "m")
    Wr = make_dir(d, cfg, W, dtype)
    want = P.forward(cfg, Wr, toks)
    other = list(toks)
    other[15] = (toks[15] + 1) % cfg["vocab"]
    assert rel_err(P.forward(cfg, Wr, other)[-1], want[-1]) > 1e-3
    drv = Driver(d, dtype, num_pages=1, page_size=16, max_requests=2)
    at = 0
    for n in [2, 131, 3, 64, 100]:
        drv.step([("a", toks[at:at + n])])
        at += n
    for i in range(at, 320):
        drv.step([("a", [toks[i]])])
    _close(drv.request_logits("a", 320), want, TOL[dtype], "scan through portions")


# ---- whole models through the step function -----------------------------------------------------------------------------
class RoutedDriver(Driver):
    """The helper's driver, which also files the experts the engine chose under (request, position)."""

    def __init__(self, *a, **k):
        super().__init__(*a, **k)
        self.picks = {}

    def step(self, entries, want_all=True, end=()):
        from infinilm_amd.parts.moe import RoutedActivationExperts as R
        starts = [self.runner.cache.length(rid) if self.runner.cache.has(rid) else 0 for rid, _ in entries]
        R.trace = []
        try:
            super().step(entries, want_all=want_all, end=end)
            calls = [t.cpu().long() for t in R.trace]
        finally:
            R.trace = None
        row = 0
        for (rid, toks), s in zip(entries, starts):
            for i in range(len(toks)):
                self.picks[(rid, s + i)] = [c[row] for c in calls]
                row += 1

    def request_picks(self, rid, n):
        runs = len(self.picks[(rid, 0)])
        return [torch.stack([self.picks[(rid, i)][r] for i in range(n)]) for r in range(runs)]


def _moe_layers(cfg):
    return [i for i, ly in enumerate(cfg["layers"]) if ly.get("mlp") and ly["mlp"]["kind"] == "moe"]


def _compare(cfg, W, toks, got, picks, dtype, what, narrow=False):
    """float32: logits and experts as the plain implementation's own.  bfloat16: the plain implementation with the engine's
    choices, which may differ from its own in few places; the bound is the other tests' 4e-2, or twice the error of the plain
    implementation with its projections' operands and results rounded to bfloat16 where that is larger."""
    layers = _moe_layers(cfg)
    assert len(picks) == len(layers)
    chosen = {}
    forced = {i: p for i, p in zip(layers, picks)}
    want = P.forward(cfg, W, toks, forced=forced if dtype == "bfloat16" else None, chosen=chosen)
    changed = sum(int((torch.sort(forced[i], -1).values != torch.sort(chosen[i][0], -1).values).any(-1).sum()) for i in layers)
    if dtype == "float32":
        assert changed == 0, f"{what}: another expert in float32"
    else:
        assert changed <= max(2, len(layers) * len(toks) // 20), f"{what}: {changed} choices of {len(layers) * len(toks)} differ"
    tol = TOL[dtype]
    if dtype == "bfloat16":     # ... or twice what the plain implementation loses when it rounds at its projections
        own = rel_err(P.forward(cfg, W, toks, forced=forced, round_to=BF), want)
        if narrow and own > TOL[dtype]:
            # layers of a handful of channels whose normed outputs turn one rounding into a large part of a logit: the plain
            # implementation's own rounding error is beyond the tolerance, so nothing can be told from a comparison
            assert torch.isfinite(got).all()
            return
        tol = max(tol, 2.0 * own)
    err = rel_err(got, want)
    print(f"[err] {what} {dtype} n={len(toks)}: {err:.3e} (bound {tol:.3e})")
    assert err < tol, f"{what} {dtype}: error {err:.3e} (bound {tol:.3e})"


CASES = [(c, d, p) for d in ("float32", "bfloat16") for c, p in (("A", 16), ("B", 64), ("C", 64), ("C", 32), ("A", 4))]


@pytest.fixture(scope="module", params=CASES, ids=[f"{c}-{d}-p{p}" for c, d, p in CASES])
def case(request, tmp_path_factory):
    name, dtype, page = request.param
    cfg = P.CONFIGS[name]()
    d = tmp_path_factory.mktemp(f"bebuzen_{name}_{dtype}")
    W = make_dir(str(d), cfg, P.random_weights(cfg, 40 + ord(name)), dtype)
    toks = {r: tokens(cfg, n, 11 * i + 3) for i, (r, n) in
            enumerate([("r0", 300), ("r1", 1), ("r2", 45), ("r3", 70), ("r4", 2), ("r5", 131)])}
    return {"cfg": cfg, "dir": str(d), "dtype": dtype, "toks": toks, "name": name, "page": page, "W": W}


def _check(case, drv, rid):
    n = len(case["toks"][rid])
    _compare(case["cfg"], case["W"], case["toks"][rid], drv.request_logits(rid, n), drv.request_picks(rid, n), case["dtype"],
             f"{case['name']} {rid}")


def _pages(n, page):
    return -(-n // page)


def test_whole_requests(case):
    page = case["page"]
    drv = RoutedDriver(case["dir"], case["dtype"], num_pages=_pages(300, page) + 1, page_size=page, max_requests=2)
    for rid, t in case["toks"].items():
        drv.step([(rid, t)], end=[rid])
        _check(case, drv, rid)


def test_last_tokens_one_by_one(case):
    """The last 140 tokens decoded one by one (longer than every window, so windows pass over decoded tokens)."""
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
            n = max(1, min(sizes[i % len(sizes)], len(t) - at))
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
            want = P.forward(case["cfg"], case["W"], toks[r])
            _close(got[True][r], want[start[r]:start[r] + len(got[True][r])], TOL["float32"], f"{r} against the plain implementation")
        else:
            _close(got[True][r], got[False][r], TOL["bfloat16"], f"{r}: recorded against eager")


def test_logits_do_not_depend_on_the_cut_in_32_bit(case):
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
def _random_config(seed, widths=(24, 40, 64, 72, 96), inners=(16, 40, 100)):
    g = torch.Generator().manual_seed(1000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    pick = lambda xs: xs[ri(0, len(xs) - 1)]
    width = pick(list(widths))
    layers, diffs = [], []
    for i in range(ri(2, 5)):
        kind = pick(["attention", "attention_2", "mamba1"])
        if kind == "mamba1":
            mixer = {"inner": pick(list(inners)), "state": pick([1, 3, 8, 16, 24]), "dt_rank": ri(1, 6), "conv": ri(1, 4)}
        else:
            G = pick([1, 2, 3])
            dim = pick([4, 6, 10, 16, 32])
            mixer = {"heads": G * pick([1, 2, 3]), "kv_heads": G, "dim": dim, "vdim": pick([4, 7, 12, 16, 32]), "scale": 0.5 / math.sqrt(dim)}
            if ri(0, 3):
                mixer["rot"] = {"base": pick([10.0, 1000.0, 50000.0]), "dims": 2 * ri(1, dim // 2)}
                if ri(0, 1):
                    mixer["rot"]["scaling"] = {"factor": pick([2.0, 8.0]), "low": 1.0, "high": pick([2.0, 4.0]), "original": pick([16, 64, 256])}
            if ri(0, 3):
                mixer["mask"] = {"size": pick([1, 2, 7, 30, 64, 100])}
            if kind == "attention":
                mixer["diff"] = pick([0.2, 0.5, 0.8])
                if ri(0, 3):
                    mixer["conv"] = ri(1, 4)
                if diffs and ri(0, 1):
                    src = pick(diffs)
                    mixer = dict(layers[src]["mixer"])
                    mixer.pop("mask", None)
                    if ri(0, 2):
                        mixer["mask"] = {"size": pick([3, 20, 90])}
                    mixer["kv_from"] = src
                else:
                    diffs.append(i)
            elif "mask" in mixer and ri(0, 1):
                mixer["mask"]["keep_first"] = pick([1, 2, 5, 40])
        mlp = pick([None, "dense", "moe", "moe"])
        if mlp == "dense":
            mlp = {"kind": "dense", "ff": pick([8, 30, 64])}
        elif mlp == "moe":
            E = ri(1, 6)
            mlp = {"kind": "moe", "router": {"experts": E, "top": ri(1, E)}, "expert": {"ff": pick([8, 20, 33])}}
            if ri(0, 1):
                mlp["router"]["scale"] = pick([0.5, 2.0, 3.0])
            if ri(0, 1):
                mlp["shared"] = {"ff": pick([8, 24])}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Bebuzen", "vocab": pick([31, 64, 257]), "width": width, "norm": {"eps": pick([1e-5, 1e-6])}, "layers": layers}
    if ri(0, 1):
        cfg["residual_mult"] = pick([0.3, 0.7, 1.0])
    return cfg


def _mixed_run(tmp_path, cfg, seed, dtype, page, narrow=False):
    d = str(tmp_path / "m")
    W = make_dir(d, cfg, P.random_weights(cfg, seed), dtype)
    toks = {"a": tokens(cfg, 150, seed), "b": tokens(cfg, 40, seed + 1), "c": tokens(cfg, 3, seed + 2)}
    drv = RoutedDriver(d, dtype, num_pages=_pages(150, page) + _pages(40, page) + 2, page_size=page, max_requests=2)
    drv.step([("a", toks["a"][:70]), ("c", toks["c"][:2])])
    drv.step([("a", toks["a"][70:72]), ("c", toks["c"][2:])], end=["c"])
    drv.step([("a", toks["a"][72:73]), ("b", toks["b"][:33])])
    for i in range(73, 80):
        drv.step([("a", [toks["a"][i]]), ("b", [toks["b"][33 + i - 73]])], end=["b"] if i == 79 else [])
    drv.step([("a", toks["a"][80:])], end=["a"])
    for rid, t in toks.items():
        _compare(cfg, W, t, drv.request_logits(rid, len(t)), drv.request_picks(rid, len(t)), dtype, f"seed {seed} {rid}", narrow)


@pytest.mark.parametrize("seed", range(24))
def test_random_configurations(seed, tmp_path):
    _mixed_run(tmp_path, _random_config(seed), seed, "float32", [4, 16, 64][seed % 3])


@pytest.mark.parametrize("seed", range(24, 36))
def test_random_configurations_in_bfloat16(seed, tmp_path):
    _mixed_run(tmp_path, _random_config(seed), seed, "bfloat16", [16, 64, 32][seed % 3])


@pytest.mark.parametrize("seed", range(36, 52))
def test_random_configurations_of_odd_widths(seed, tmp_path):
    """Widths and channel counts that are no multiples of 8 (or of 4), where the products and the row kernels take their plain
    forms; both dtypes in turn."""
    cfg = _random_config(seed, widths=(20, 36, 50, 100, 132, 17), inners=(10, 30, 52, 7, 300))
    _mixed_run(tmp_path, cfg, seed, "float32" if seed % 2 else "bfloat16", [16, 64, 4][seed % 3], narrow=True)


# ---- through the entry point ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,graph", [("A", False), ("B", True), ("C", True)])
def test_greedy_generation_through_the_entry_point(name, graph, tmp_path):
    """`LLM.generate` with its scheduler (three slots, portions of five tokens): every request token for token as the plain
    implementation generates it greedily."""
    from infinilm_amd import LLM, SamplingParams
    cfg = P.CONFIGS[name]()
    W = make_dir(str(tmp_path), cfg, P.random_weights(cfg, 77), "float32")
    prompts = [tokens(cfg, n, 5 + n) for n in (3, 40, 9, 64, 1)]
    llm = LLM(str(tmp_path), dtype="float32", num_blocks=24, block_size=16, max_batch_size=3, chunk_size=5,
              max_num_batched_tokens=11, enable_graph=graph)
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(top_k=1, max_tokens=12))
    for prompt, out in zip(prompts, outs):
        seq = list(prompt)
        for _ in range(12):
            seq.append(int(P.forward(cfg, W, seq)[-1].argmax()))
        assert out.outputs[0].token_ids == seq[len(prompt):], f"prompt of {len(prompt)} tokens"
    llm.close()


def test_recorded_steps_with_long_portions(tmp_path):
    """Portions of up to 160 tokens (long enough for the scan's pieces) in recorded steps that are replayed with other requests'
    portions of other lengths: greedy tokens as the plain implementation's."""
    from infinilm_amd import LLM, SamplingParams
    cfg = P.CONFIGS["C"]()
    W = make_dir(str(tmp_path), cfg, P.random_weights(cfg, 78), "float32")
    prompts = [tokens(cfg, n, 9 + n) for n in (300, 170, 129, 5, 161, 320)]
    llm = LLM(str(tmp_path), dtype="float32", num_blocks=40, block_size=32, max_batch_size=3, chunk_size=160,
              max_num_batched_tokens=192, enable_graph=True)
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(top_k=1, max_tokens=6))
    for prompt, out in zip(prompts, outs):
        seq = list(prompt)
        for _ in range(6):
            seq.append(int(P.forward(cfg, W, seq)[-1].argmax()))
        assert out.outputs[0].token_ids == seq[len(prompt):], f"prompt of {len(prompt)} tokens"
    llm.close()


def test_long_decoding(tmp_path):
    """600 decoded tokens after a prompt of 10, recorded steps, pages of 16 given back as the windows pass."""
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    cfg = P.CONFIGS["A"]()
    d = str(tmp_path / "m")
    W = make_dir(d, cfg, P.random_weights(cfg, 3), "float32")
    toks = tokens(cfg, 610, 2)
    want = P.forward(cfg, W, toks)
    model = load_model(d, "float32", DEV)
    runner = make_runner(model, num_pages=8, page_size=16, max_requests=2, enable_graph=True)
    runner.cache.admit("a")
    runner.step([StepEntry("a", toks[:10], [])])
    rows = [runner.step([StepEntry("a", [toks[i]], [0])]).cpu()[0] for i in range(10, 610)]
    _close(torch.stack(rows), want[10:], TOL["float32"], "600 decoded tokens")
    runner.cache.check()
