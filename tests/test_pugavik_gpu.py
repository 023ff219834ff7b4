"""The Pugavik design in the engine against the plain implementation (`plain_pugavik.py`): the new kernels alone, every
mixer alone in a one-layer model (with keys made to stand out far back, at page borders and on either side of a
window's edge), then whole models through the engine's own step function (whole prompts, decoding token by token,
portions down to two tokens, mixed batches with pages and state slots used again, recorded decode steps) and through the
entry point with its scheduler (greedy generation).  Configurations A, B and C differ from each other in every size and
switch: with and without a loop (of one layer, of two, two and three times), layers without a feed-forward, key and value
heads of equal and unequal sizes, one, some and as many key/value heads as heads, heads turned partly, wholly and not at
all, windows shorter and longer than the prompts, latent rows below and above the matrix-core kernels' head size."""
import json
import os

import pytest
import torch

import plain_pugavik as P
from helpers import TOL, Driver, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_dir(path, cfg, W, store):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    cfg = json.loads(json.dumps(cfg))
    for layer in cfg["layers"]:           # (the low rank is read from the checkpoint's tensor, as for a model from elsewhere)
        layer["mixer"].pop("decay_rank", None)
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
def test_add_layernorm_sums_every_kind_of_addend():
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(3)
    for H in (24, 250, 256, 1000, 4100):
        r = torch.randn(5, H, generator=g)
        a = torch.randn(5, H, generator=g).to(torch.bfloat16)
        parts = torch.randn(3, 5, H, generator=g)
        row = torch.randn(H, generator=g)
        extra = [torch.randn(5, H, generator=g) for _ in range(3)]
        w, b = torch.randn(H, generator=g), torch.randn(H, generator=g)
        want_r = r.double() + 0.5 * a.double() + parts.double().sum(0) + row.double() - 2.0 * extra[0].double() + extra[1].double() + extra[2].double()
        rd = r.clone().to(DEV)
        adds = [(a.to(DEV), 0.5), (parts.to(DEV), 1.0), (row.to(DEV), 1.0), (extra[0].to(DEV), -2.0), (extra[1].to(DEV), 1.0), (extra[2].to(DEV), 1.0)]
        x = kernels.add_layernorm(rd, adds, w.to(DEV), b.to(DEV), 1e-5, torch.float32)
        _close(rd.cpu(), want_r, 1e-5, f"residual, width {H}")
        _close(x.cpu(), P.layer_norm(want_r, w.double(), b.double(), 1e-5), 1e-5, f"normed rows, width {H}")
        # nothing to add, bfloat16 result and weights; a sum alone
        rd2 = want_r.float().to(DEV)
        x = kernels.add_layernorm(rd2, [], w.to(torch.bfloat16).to(DEV), b.to(torch.bfloat16).to(DEV), 1e-5, torch.bfloat16)
        _close(x.cpu(), P.layer_norm(want_r.float().double(), w.to(torch.bfloat16).double(), b.to(torch.bfloat16).double(), 1e-5), 1e-2, f"bfloat16, width {H}")
        assert kernels.add_layernorm(rd2, [(row.to(DEV), 3.0)], None, None, 0.0, torch.float32) is None
        _close(rd2.cpu(), want_r.float().double() + 3.0 * row.double(), 1e-5, f"sum alone, width {H}")


def test_a_large_mean_does_not_spoil_the_variance():
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(4)
    r = 1000.0 + 0.01 * torch.randn(3, 512, generator=g)
    w, b = torch.ones(512), torch.zeros(512)
    x = kernels.add_layernorm(r.clone().to(DEV), [], w.to(DEV), b.to(DEV), 1e-8, torch.float32)
    _close(x.cpu(), P.layer_norm(r.double(), w.double(), b.double(), 1e-8), 2e-3, "rows far from zero")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,K,N", [(1, 2, 8, 20), (5, 3, 16, 40), (40, 4, 64, 96), (70, 2, 33, 17)])
def test_product_per_head(T, H, K, N, dtype):
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(T + K)
    x = torch.randn(T, H * (K + 5), generator=g).to(dtype)
    w_kn = (torch.randn(H, K, N, generator=g) / K ** 0.5).to(dtype)
    w_nk = (torch.randn(H, N, K, generator=g) / K ** 0.5).to(dtype)
    xv = x.to(DEV).view(T, H, K + 5)[:, :, :K]
    want = torch.einsum("thk,hkn->thn", xv.cpu().double(), w_kn.double())
    out = torch.zeros(T, H, N + 3, dtype=dtype, device=DEV)
    kernels.head_gemm(xv, w_kn.to(DEV), out[:, :, :N])
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    _close(out[:, :, :N].cpu(), want, tol, "W with the outputs dense")
    assert float(out[:, :, N:].abs().max()) == 0.0
    want = torch.einsum("thk,hnk->thn", xv.cpu().double(), w_nk.double())
    out2 = torch.empty(T, H, N, dtype=dtype, device=DEV)
    kernels.head_gemm(xv, w_nk.to(DEV).transpose(1, 2), out2)
    _close(out2.cpu(), want, tol, "W with the inputs dense")


def test_sigmoid_root_is_stable_at_both_ends():
    from infinilm_amd import kernels
    z = torch.tensor([[-90.0, -20.0, -3.0, -0.1, 0.0, 0.2, 4.0, 30.0, 90.0]])
    for tau in (1.0, 3.0, 16.0):
        got = kernels.sigmoid_root(z.to(DEV), tau).cpu().double()
        want = torch.exp(-torch.nn.functional.softplus(-z.double()) / tau)
        assert torch.isfinite(got).all()
        _close(got, want, 1e-6, f"tau {tau}")
    got = kernels.sigmoid_root(z.to(torch.bfloat16).to(DEV), 2.0).cpu().double()
    _close(got, torch.exp(-torch.nn.functional.softplus(-z.to(torch.bfloat16).double()) / 2.0), 1e-6, "bfloat16 rows")
    bias = torch.linspace(-2.0, 2.0, 9)
    got = kernels.sigmoid_root(z.to(DEV), 4.0, bias=bias.to(DEV)).cpu().double()
    _close(got, torch.exp(-torch.nn.functional.softplus(-(z + bias).double()) / 4.0), 1e-6, "with a bias")


@pytest.mark.parametrize("page", [32, 64])
@pytest.mark.parametrize("window", [0, 5, 40, 1000])
@pytest.mark.parametrize("nh,nkv,d,dv", [(8, 2, 64, 32), (4, 1, 128, 128), (8, 4, 32, 20), (32, 2, 128, 96), (6, 2, 96, 96), (20, 4, 128, 128),
                                         (16, 1, 64, 48), (48, 1, 32, 32), (64, 4, 64, 64)])
def test_matrix_core_headmix_attention_equals_the_plain_kernel(nh, nkv, d, dv, window, page):
    """A step with a portion of 19 tokens after 70 cached ones (tiles of 8, 8 and 3 tokens), a decoded token at position 130
    of another request (pages the window has passed are gone) and a first token of a third: the matrix-core kernel against
    the plain one on the same cache, and the plain one against the formula.  Served by tiles and token by token (where the
    heads come in groups of 16, 48 or 64 the latter puts heads side by side as the products' columns)."""
    from infinilm_amd import kernels
    g = torch.Generator().manual_seed(nh * 7 + d + window)
    pages = 12
    bf = torch.bfloat16
    kc = torch.randn(pages + 1, nkv, page, d, generator=g).to(bf)
    vc = torch.randn(pages + 1, nkv, d, page, generator=g).to(bf)
    vc[:, :, dv:] = 0
    lens = [89, 131, 1]                                    # keys of each request after this step
    ids = [3, 7, 1, 9, 2, 10, 4, 6, 5]
    width = -(-131 // page)
    tables, at = [], 0
    for n in lens:
        k = -(-n // page)
        tables.append(ids[at:at + k] + [-1] * (width - k))
        at += k
    if 0 < window <= 40:                                   # pages the decoded token's window has passed are given back
        tables[1][:(131 - window) // page] = [-1] * ((131 - window) // page)
    rows_pos = [(0, 70 + i) for i in range(19)] + [(1, 130), (2, 0)]
    T = len(rows_pos)
    q = torch.randn(T, nh * d, generator=g).to(bf)
    mix = (torch.eye(nh) + 0.3 * torch.randn(nh, nh, generator=g)).float()
    sink = torch.randn(nh, generator=g).float()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    args = (q.to(DEV), kc.to(DEV), vc.to(DEV), i32(tables), i32([r for r, _ in rows_pos]), i32([p for _, p in rows_pos]), nh, nkv, d, dv,
            d ** -0.5, window)
    tiles, singles = i32([[0, 8], [8, 8], [16, 3], [0, 0]]), i32([19, -1, 20])
    fast = kernels.headmix_attention(*args, mix=mix.to(DEV), sink=sink.to(DEV), tiles=tiles, single_rows=singles).cpu()
    paired = kernels.headmix_attention(*args, mix=mix.to(DEV), sink=sink.to(DEV), tiles=tiles, single_rows=singles,
                                       seg_offsets=i32([0, 19, 20, 21])).cpu()
    each = kernels.headmix_attention(*args, mix=mix.to(DEV), sink=sink.to(DEV)).cpu()
    old = kernels.USE_HEADMIX_MFMA
    kernels.USE_HEADMIX_MFMA = False
    try:
        plain = kernels.headmix_attention(*args, mix=mix.to(DEV), sink=sink.to(DEV)).cpu()
    finally:
        kernels.USE_HEADMIX_MFMA = old
    # the formula, request by request
    want = torch.zeros(T, nh, d, dtype=torch.float64)
    per = nh // nkv
    for t, (r, p) in enumerate(rows_pos):
        lo = max(0, p - window + 1) if window > 0 else 0
        keys = torch.stack([kc[tables[r][j // page], :, j % page, :] for j in range(lo, p + 1)]).double()      # [n, nkv, d]
        vals = torch.stack([vc[tables[r][j // page], :, :, j % page] for j in range(lo, p + 1)]).double()
        raw = torch.stack([keys[:, h // per] @ q[t].double().view(nh, d)[h] for h in range(nh)]) * d ** -0.5       # [nh, n]
        s = mix.double() @ raw
        top = torch.maximum(s.max(-1).values, sink.double())
        e = torch.exp(s - top[:, None])
        prob = e / (e.sum(-1) + torch.exp(sink.double() - top))[:, None]
        want[t] = torch.stack([prob[h] @ vals[:, h // per] for h in range(nh)])
    _close(plain.view(T, nh, d), want, 1e-2, "the plain kernel against the formula")
    _close(fast.view(T, nh, d), want, 2e-2, "the matrix-core kernel, by tiles")
    _close(paired.view(T, nh, d), want, 2e-2, "the matrix-core kernel, tiles two at a time")
    _close(each.view(T, nh, d), want, 2e-2, "the matrix-core kernel, token by token")


@pytest.mark.parametrize("piece", [0, 4, 7])
@pytest.mark.parametrize("heads,dk,dv", [(2, 16, 24), (3, 5, 3), (2, 128, 64), (1, 200, 40), (4, 64, 8)])
def test_decay_per_channel_carries_states_over_launches(heads, dk, dv, piece, monkeypatch):
    """Three segments of unequal length in one launch, one from a zero state, two from the states an earlier launch left
    in rows that are used again; every key channel with a decay of its own.  In one pass (`piece` 0) and with the segments
    cut into pieces of 4 and of 7 tokens that run side by side."""
    from infinilm_amd import kernels
    monkeypatch.setattr(kernels, "SCAN_PIECE", piece)
    monkeypatch.setattr(kernels, "SCAN_PIECE_FROM", 1)
    g = torch.Generator().manual_seed(heads * 100 + dk)
    lens_a, lens_b = [7, 1, 19], [8, 33, 2]
    pool = torch.zeros((6, heads, dv, dk), device=DEV)
    data, want = {}, {}
    for r, n in enumerate([a + b for a, b in zip(lens_a, lens_b)]):
        q, k = torch.randn(n, heads, dk, generator=g), torch.randn(n, heads, dk, generator=g)
        v = torch.randn(n, heads, dv, generator=g)
        alpha = torch.rand(n, heads, dk, generator=g) * 0.5 + 0.5
        data[r] = (q, k, v, alpha)
        want[r] = P.channel_decay_scan(q.double(), k.double(), v.double(), alpha.double())

    def launch(spans, rows_in, rows_out):
        cat = lambda i: torch.cat([data[r][i][a:b].reshape(b - a, -1) for r, a, b in spans]).to(DEV)
        offs = [0]
        for _, a, b in spans:
            offs.append(offs[-1] + b - a)
        i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
        return kernels.decay_scan(cat(0), cat(1), cat(2), heads, dk, dv, heads, pool, i32(rows_in), i32(rows_out), i32(offs), len(spans),
                                  decay_c=cat(3), max_len=max(b - a for _, a, b in spans)).cpu(), offs

    o1, offs = launch([(r, 0, lens_a[r]) for r in range(3)], [0, 0, 0], [2, 4, 1])
    for r in range(3):
        _close(o1[offs[r]:offs[r + 1]].view(-1, heads, dv), want[r][:lens_a[r]], 1e-5, f"first launch, segment {r}")
    # segment 1 ends; its row goes to a new segment that starts from zero, beside the two that go on
    o2, offs = launch([(0, lens_a[0], lens_a[0] + lens_b[0]), (1, 0, lens_a[1] + lens_b[1]), (2, lens_a[2], lens_a[2] + lens_b[2])],
                      [2, 0, 1], [2, 4, 1])
    _close(o2[offs[0]:offs[1]].view(-1, heads, dv), want[0][lens_a[0]:], 1e-5, "a state carried on")
    _close(o2[offs[1]:offs[2]].view(-1, heads, dv), want[1], 1e-5, "a row used again from zero")
    _close(o2[offs[2]:offs[3]].view(-1, heads, dv), want[2][lens_a[2]:], 1e-5, "a state carried on beside it")


# ---- every mixer alone, with one key made to stand out ------------------------------------------------------------------
def _one_layer(kind, mixer, width=32, vocab=50):
    return {"architecture": "Pugavik", "vocab": vocab, "width": width, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
            "layers": [P._layer(kind, mixer, None)]}


def _normed_row(W, token):
    return P.layer_norm(W["embed"][token].double(), W["l0.norm1"].double(), W["l0.norm1.b"].double(), 1e-6)


def _run_last_tokens(tmp_path, cfg, W, toks, dtype, decoded=5, page=64):
    Wr = make_dir(str(tmp_path), cfg, W, dtype)
    want = P.forward(cfg, Wr, toks)
    drv = Driver(str(tmp_path), dtype, num_pages=-(-len(toks) // page) + 1, page_size=page, max_requests=2)
    if decoded < len(toks):
        drv.step([("a", toks[:len(toks) - decoded])])
    for t in toks[len(toks) - decoded:]:
        drv.step([("a", [t])])
    return drv.request_logits("a", len(toks)), want, Wr


def _attention_with_a_marked_key(window, rot_dims=4):
    """Token 47's key and token 48's queries point the same way in every head: that one score stands far above the others."""
    cfg = _one_layer("attention", P._attention(4, 2, 64, 24, window, rot_dims, scale=1.0))
    W = P.random_weights(cfg, 9)
    W["embed"][47], W["embed"][48] = torch.eye(32)[0] * 4, torch.eye(32)[1] * 4
    W["l0.mix.q.b"].zero_(), W["l0.mix.k.b"].zero_()
    W["l0.mix.q.norm"].fill_(1.0), W["l0.mix.k.norm"].fill_(1.0)
    hk, hq = _normed_row(W, 47).float(), _normed_row(W, 48).float()
    key = (W["l0.mix.k"] @ hk).view(2, 64)                              # token 47's keys before the norm
    key[:, :rot_dims] = 0                                              # (the turned entries would turn away with the distance)
    for h in range(4):
        want_q = key[h // 2]
        rows = slice(h * 64, (h + 1) * 64)
        W["l0.mix.q"][rows] -= torch.outer(W["l0.mix.q"][rows] @ hq - want_q, hq) / (hq @ hq)   # now W_q h_48 = that key
    W["l0.mix.talk"] = torch.eye(4) + 0.1 * torch.randn(4, 4, generator=torch.Generator().manual_seed(1))
    return cfg, W


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decoded", [5, 0])
@pytest.mark.parametrize("back", [1, 63, 64, 65, 127, 128, 299, 300])
def test_window_attention_finds_one_key_up_to_its_edge(dtype, decoded, back, tmp_path):
    """A window of 300 positions: the marked key lies `back` positions before the last query, next to it, on either side
    of a page border, and at the window's last place (299); one place further (300) it is outside and must not count.  In a
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
def test_first_tokens_and_short_windows(dtype, tmp_path):
    """A window of three positions, pages of four: every token of a short sequence, decoded one by one from the first."""
    cfg, W = _attention_with_a_marked_key(3, rot_dims=16)
    toks = [47, 48, 47, 48, 3, 47, 9, 48, 48, 47, 2, 48]
    got, want, _ = _run_last_tokens(tmp_path, cfg, W, toks, dtype, decoded=len(toks), page=4)
    _close(got, want, TOL[dtype], "every token of a short sequence")


def test_sink_and_head_mixing_matter(tmp_path):
    """The engine follows the plain implementation when the sinks are large and the mixing matrix is far from the identity,
    and the plain implementation's result depends on both."""
    cfg, W = _attention_with_a_marked_key(50)
    W["l0.mix.sink"] = torch.tensor([3.0, -2.0, 6.0, 0.5])
    W["l0.mix.talk"] = torch.tensor([[0.2, 1.0, 0.0, -0.5], [1.0, 0.0, 0.3, 0.0], [0.0, -1.0, 1.0, 0.6], [0.5, 0.5, 0.5, 0.5]])
    toks = tokens(cfg, 90, 4)
    got, want, Wr = _run_last_tokens(tmp_path, cfg, W, toks, "float32", decoded=30)
    _close(got, want, TOL["float32"], "sinks and mixing")
    no_sink = dict(Wr, **{"l0.mix.sink": torch.full((4,), -60.0)})
    assert rel_err(P.forward(cfg, no_sink, toks), want) > 0.05
    plain_mix = dict(Wr, **{"l0.mix.talk": torch.eye(4)})
    assert rel_err(P.forward(cfg, plain_mix, toks), want) > 0.05


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key_at", [3, 63, 64, 127, 128, 640])
@pytest.mark.parametrize("rank", [40, 150])
def test_latent_attention_finds_one_key(dtype, key_at, rank, tmp_path):
    """The key at `key_at` (far back among 700, or on either side of a page border) is the only one that matches the last
    query's unrotated part.  Latent rows of 48 entries (the matrix-core kernels in bfloat16) and of 160 (beyond them)."""
    cfg = _one_layer("latent_attention", P._latent(2, 16, 8, 12, rank, scale=1.0))
    W = P.random_weights(cfg, 5)
    W["embed"][47], W["embed"][48] = torch.eye(32)[0] * 4, torch.eye(32)[1] * 4
    hk, hq = _normed_row(W, 47).float(), _normed_row(W, 48).float()
    c = P.rms_unit(W["l0.mix.dkv"][:rank] @ hk, 1e-6) * W["l0.mix.dkv.norm"]
    key = (W["l0.mix.uk"] @ c).view(2, 16)
    key = key / key.norm(dim=-1, keepdim=True) * 6.0
    for h in range(2):
        rows = slice(h * 24, h * 24 + 16)
        W["l0.mix.q"][rows] -= torch.outer(W["l0.mix.q"][rows] @ hq - key[h], hq) / (hq @ hq)
    n = 700
    toks = [1 + (i % 40) for i in range(n)]
    toks[key_at], toks[-1] = 47, 48
    got, want, Wr = _run_last_tokens(tmp_path, cfg, W, toks, dtype)
    err = rel_err(got[-1], want[-1])
    assert err < TOL[dtype], f"key at {key_at}: {err:.3e}"
    moved = P.forward(cfg, Wr, toks[:key_at] + [2] + toks[key_at + 1:])
    assert rel_err(moved[-1], want[-1]) > 0.2, "the test's key does not matter: it would show nothing"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_state_remembers_a_far_token(dtype, tmp_path):
    """Decays near one: a token 600 positions back still shapes the last output, through portions and decoded tokens."""
    cfg = _one_layer("gla", P._gla(2, 16, 20, 16.0, 4))
    W = P.random_weights(cfg, 6)
    W["l0.mix.a2.b"].fill_(7.0)
    W["l0.mix.a2"].mul_(0.1)
    # the other tokens are three kinds only; token 48's query is made to point along the part of token 47's key that is
    # orthogonal to every other key (its own too), head by head: the last output is token 47's value alone
    W["embed"][47], W["embed"][48] = torch.eye(32)[0] * 4, torch.eye(32)[1] * 4
    hq = _normed_row(W, 48).float()
    for h in range(2):
        rows = slice(h * 16, (h + 1) * 16)
        others = torch.stack([W["l0.mix.k"][rows] @ _normed_row(W, t).float() for t in (1, 2, 3, 48)])
        key = W["l0.mix.k"][rows] @ _normed_row(W, 47).float()
        basis = torch.linalg.qr(others.T).Q                               # [16, 4]
        aim = key - basis @ (basis.T @ key)
        W["l0.mix.q"][rows] -= torch.outer(W["l0.mix.q"][rows] @ hq - aim / aim.norm() * 8.0, hq) / (hq @ hq)
    n = 700
    toks = [1 + (i % 3) for i in range(n)]
    toks[100], toks[-1] = 47, 48
    Wr = make_dir(str(tmp_path), cfg, W, dtype)
    want = P.forward(cfg, Wr, toks)
    drv = Driver(str(tmp_path), dtype, num_pages=2, page_size=64, max_requests=2)
    drv.step([("a", toks[:300])])
    drv.step([("a", toks[300:302])])
    drv.step([("a", toks[302:680])])
    for t in toks[680:]:
        drv.step([("a", [t])])
    err = rel_err(drv.request_logits("a", n)[-20:], want[-20:])
    # (the query is orthogonal to all keys but one, so every rounding is a large share of what remains of the sums: the
    # bound is twice what the plain implementation loses when it rounds alike: float32 arithmetic, or bfloat16 products)
    lossy = P.forward(cfg, Wr, toks, dtype=torch.float32) if dtype == "float32" else P.forward(cfg, Wr, toks, round_to=torch.bfloat16)
    bound = max(TOL[dtype], 2.0 * rel_err(lossy[-20:], want[-20:]))
    assert err < bound, f"{err:.3e} (bound {bound:.3e})"
    moved = P.forward(cfg, Wr, toks[:100] + [2] + toks[101:])
    assert rel_err(moved[-1], want[-1]) > 0.2, "the far token does not matter: it would show nothing"


# ---- whole models through the step function -----------------------------------------------------------------------------
CASES = [(c, d, p) for d in ("float32", "bfloat16") for c, p in (("A", 16), ("B", 64), ("C", 64), ("C", 16))]


@pytest.fixture(scope="module", params=CASES, ids=[f"{c}-{d}-p{p}" for c, d, p in CASES])
def case(request, tmp_path_factory):
    name, dtype, page = request.param
    cfg = P.CONFIGS[name]()
    d = tmp_path_factory.mktemp(f"pugavik_{name}_{dtype}")
    W = make_dir(str(d), cfg, P.random_weights(cfg, 40 + ord(name)), dtype)
    toks = {r: tokens(cfg, n, 11 * i + 3) for i, (r, n) in
            enumerate([("r0", 300), ("r1", 1), ("r2", 45), ("r3", 70), ("r4", 2), ("r5", 131)])}
    oracle = {r: P.forward(cfg, W, t) for r, t in toks.items()}
    # bfloat16: the bound is the tolerance of the other models' tests or, where it is larger, twice the error of the plain
    # implementation with every projection's operands and result rounded to bfloat16
    tol = {r: TOL[dtype] for r in toks}
    if dtype == "bfloat16":
        tol = {r: max(TOL[dtype], 2.0 * rel_err(P.forward(cfg, W, t, round_to=torch.bfloat16), oracle[r])) for r, t in toks.items()}
    return {"cfg": cfg, "dir": str(d), "dtype": dtype, "toks": toks, "oracle": oracle, "name": name, "page": page, "tol": tol, "W": W}


def _check(case, drv, rid):
    n = len(case["toks"][rid])
    err = rel_err(drv.request_logits(rid, n), case["oracle"][rid])
    print(f"[err] {case['name']} {case['dtype']} {rid} n={n}: {err:.3e} (bound {case['tol'][rid]:.3e})")
    assert err < case["tol"][rid], f"{case['name']} {case['dtype']} request {rid}: error {err:.3e}"


def _pages(n, page):
    return -(-n // page)


def test_whole_requests(case):
    page = case["page"]
    drv = Driver(case["dir"], case["dtype"], num_pages=_pages(300, page) + 1, page_size=page, max_requests=2)
    for rid, t in case["toks"].items():
        drv.step([(rid, t)], end=[rid])
        _check(case, drv, rid)


def test_last_tokens_one_by_one(case):
    """The last 140 tokens decoded one by one (longer than any window but one, so windows pass over decoded tokens)."""
    page = case["page"]
    drv = Driver(case["dir"], case["dtype"], num_pages=_pages(300, page) + 1, page_size=page, max_requests=2)
    for rid, t in case["toks"].items():
        head = max(len(t) - 140, 0)
        if head:
            drv.step([(rid, t[:head])])
        for i in range(head, len(t)):
            drv.step([(rid, [t[i]])], end=[rid] if i == len(t) - 1 else [])
        _check(case, drv, rid)


def test_portions_of_changing_size(case):
    page = case["page"]
    drv = Driver(case["dir"], case["dtype"], num_pages=_pages(300, page) + 1, page_size=page, max_requests=2)
    sizes = [2, 5, page, 3, 2 * page + 1, 2, 17, page - 1, 1, 64]
    for rid, t in case["toks"].items():
        at, i = 0, 0
        while at < len(t):
            n = min(sizes[i % len(sizes)], len(t) - at)
            drv.step([(rid, t[at:at + n])], end=[rid] if at + n == len(t) else [])
            at, i = at + n, i + 1
        _check(case, drv, rid)


def test_mixed_steps_reuse_pages_and_slots(case):
    """Four state slots and pages for about two long requests serve six requests: portions of some beside single
    tokens of others; a request that ends frees its slot and pages for the next, which must start from zero state."""
    page, toks = case["page"], case["toks"]
    drv = Driver(case["dir"], case["dtype"], num_pages=_pages(300, page) + _pages(131, page) + 3, page_size=page, max_requests=4)
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
    """Three requests decode side by side for 70 steps with recorded steps switched on (one ends on the way, so the
    recorded size changes): every logit as the plain implementation gives it."""
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    if case["page"] != 64:
        pytest.skip("one page size is enough here")
    toks = case["toks"]
    model = load_model(case["dir"], case["dtype"], DEV)
    runner = make_runner(model, num_pages=12, page_size=64, max_requests=4, enable_graph=True)
    ids = ["r0", "r3", "r5"]
    start = {"r0": 200, "r3": 20, "r5": 61}
    for r in ids:
        runner.cache.admit(r)
    runner.step([StepEntry(r, toks[r][:start[r]], []) for r in ids])
    got = {r: [] for r in ids}
    for i in range(70):
        live = [r for r in ids if start[r] + i < len(toks[r])]
        out = runner.step([StepEntry(r, [toks[r][start[r] + i]], [0]) for r in live]).cpu()
        for j, r in enumerate(live):
            got[r].append(out[j].clone())
        for r in live:
            if start[r] + i + 1 == len(toks[r]):
                runner.cache.release(r)
    assert runner._graphs, "no step was recorded"
    for r in ids:
        err = rel_err(torch.stack(got[r]), case["oracle"][r][start[r]:start[r] + len(got[r])])
        assert err < case["tol"][r], f"{r}: {err:.3e}"


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
    """Three to five layers of the three kinds in a random order, every size drawn from a short list, a loop over a random
    stretch (or none), layers without a feed-forward now and then."""
    import random
    rnd = random.Random(seed)
    width = rnd.choice([48, 64, 96, 120, 128])
    layers = []
    for _ in range(rnd.randint(3, 5)):
        kind = rnd.choice(["attention", "latent_attention", "gla"])
        if kind == "attention":
            kv = rnd.choice([1, 2, 3, 4])
            heads = kv * rnd.choice([1, 2, 3])
            dim = rnd.choice([8, 12, 16, 32, 40, 64])
            m = P._attention(heads, kv, dim, rnd.choice([dim, 8, 24, 32, 64]), rnd.choice([1, 2, 9, 31, 64, 65, 500]),
                             rnd.choice([0, 2, dim // 2 // 2 * 2, dim]), base=rnd.choice([100.0, 10000.0, 500000.0]), scale=rnd.choice([0.1, 0.25, dim ** -0.5]))
        elif kind == "latent_attention":
            rot = rnd.choice([0, 4, 8, 16, 32])
            m = P._latent(rnd.choice([1, 2, 3, 4, 8]), rnd.choice([8, 16, 24, 32]), rot, rnd.choice([8, 16, 20, 32]), rnd.choice([16, 24, 48, 96, 112, 136]),
                          base=rnd.choice([1000.0, 10000.0]))
        else:
            m = P._gla(rnd.choice([1, 2, 4]), rnd.choice([8, 16, 20, 32, 64]), rnd.choice([8, 16, 24, 64]), rnd.choice([1.0, 4.0, 16.0]), rnd.choice([2, 4, 7, 16]))
        layers.append(P._layer(kind, m, rnd.choice([None, 32, 100, 2 * width])))
    cfg = {"architecture": "Pugavik", "vocab": rnd.choice([50, 131, 640]), "width": width, "embedding": {"scale": rnd.choice([0.5, 1.0, 3.0])},
           "norm": {"eps": rnd.choice([1e-6, 1e-5])}, "layers": layers}
    if rnd.random() < 0.7:
        a = rnd.randrange(len(layers))
        cfg["loop"] = {"start": a, "stop": rnd.randint(a + 1, len(layers)), "times": rnd.choice([1, 2, 3])}
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(seed, dtype, tmp_path):
    """A random configuration, two requests: one whole, one in portions beside the other's decoded tokens, on pages of 16 or
    64 with four slots; every logit against the plain implementation."""
    cfg = _random_config(seed)
    W = make_dir(str(tmp_path), cfg, P.random_weights(cfg, 100 + seed), dtype)
    ta, tb = tokens(cfg, 75, seed), tokens(cfg, 40, seed + 50)
    want_a, want_b = P.forward(cfg, W, ta), P.forward(cfg, W, tb)
    page = 16 if seed % 2 else 64
    drv = Driver(str(tmp_path), dtype, num_pages=-(-75 // page) + -(-40 // page) + 1, page_size=page, max_requests=4)
    drv.step([("a", ta[:33])])
    drv.step([("a", ta[33:35]), ("b", tb[:19])])
    drv.step([("a", ta[35:70]), ("b", tb[19:20])])
    for i in range(5):
        drv.step([("a", ta[70 + i:71 + i]), ("b", tb[20 + 4 * i:24 + 4 * i])])
    tol = lambda t, want: TOL[dtype] if dtype == "float32" else max(TOL[dtype], 2.0 * rel_err(P.forward(cfg, W, t, round_to=torch.bfloat16), want))
    ea, eb = rel_err(drv.request_logits("a", 75), want_a), rel_err(drv.request_logits("b", 40), want_b)
    assert ea < tol(ta, want_a) and eb < tol(tb, want_b), f"seed {seed}: {ea:.3e}, {eb:.3e}; {json.dumps(cfg)}"


# ---- the entry point and its scheduler ------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,graph", [("A", False), ("B", False), ("B", True), ("C", True)])
def test_greedy_generation_through_the_entry_point(name, graph, tmp_path):
    """Five prompts through `LLM.generate` with three state slots, prompts cut into portions of five tokens under a
    token budget, and few pages: every request's greedy tokens are the plain implementation's (32-bit)."""
    from infinilm_amd import LLM, SamplingParams
    cfg = P.CONFIGS[name]()
    W = make_dir(str(tmp_path), cfg, P.random_weights(cfg, 7), "float32")
    prompts = [tokens(cfg, n, 50 + n) for n in (9, 1, 23, 4, 40)]
    llm = LLM(str(tmp_path), dtype="float32", num_blocks=10, block_size=16, max_batch_size=3, chunk_size=5,
              max_num_batched_tokens=11, enable_graph=graph)
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(top_k=1, max_tokens=12))
    for p, o in zip(prompts, outs):
        assert o.outputs[0].token_ids == P.greedy(cfg, W, p, 12), f"prompt of {len(p)} tokens"
    assert llm.engine.runner.cache.stats()["state_slots_free"] == 3
    llm.close()
