"""Madipel on the GPU against the plain fp64 oracle (tests/madipel_oracle.py): each mechanism alone, then the
model through the engine — whole prompts, token-by-token decoding, portions, unequal batches, page reuse, window
edges, far keys, long decoding and greedy generation through the scheduler.  Small configurations with random
weights, sizes chosen so that nothing the design allows to differ happens to be equal or 1."""
import json
import math

import pytest
import torch

import madipel_oracle as O

pytestmark = pytest.mark.gpu

F64 = torch.float64


def _dev(t, dtype):
    return t.to("cuda", dtype=dtype).contiguous()


# ------------------------------------------------------------------ mechanisms, one by one
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_sinpos(gpu, dtype):
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(1)
    V, d = 37, 22
    table = torch.randn(V, d, generator=g).to(torch.bfloat16)
    toks = [0, 36, 5, 5, 17, 1]
    pos = [0, 1, 2, 4093, 100000, 7]
    out = res32.embed_sinpos(_dev(table, dtype), torch.tensor(toks, dtype=torch.int32, device=gpu),
                             torch.tensor(pos, dtype=torch.int32, device=gpu), res32.sinpos_inv_freq(d, device=gpu))
    ref = table.to(F64)[torch.tensor(toks)] + O.sin_positions(pos, d)
    assert out.dtype == torch.float32
    assert (out.cpu().double() - ref).abs().max() < 2e-6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 2e-2)])
def test_layernorm_rows(gpu, dtype, tol):
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(2)
    x = torch.randn(9, 300, generator=g) * 3 + 1.5
    w, b = torch.randn(300, generator=g).to(torch.bfloat16), torch.randn(300, generator=g).to(torch.bfloat16)
    ref = O.layer_norm(x.double(), w.double(), b.double(), 1e-3)
    out = res32.layernorm(x.to(gpu), _dev(w, dtype), _dev(b, dtype), 1e-3)
    assert (out.cpu().double() - ref).abs().max() < tol * 4
    rows = torch.tensor([7, 0, 7, 3], device=gpu)
    out = res32.layernorm(x.to(gpu), _dev(w, dtype), _dev(b, dtype), 1e-3, rows=rows)
    assert (out.cpu().double() - ref[rows.cpu()]).abs().max() < tol * 4
    # a width that is a multiple of 8 (the 16-byte path in bf16), more than one chunk per thread
    x8, w8, b8 = torch.randn(5, 2312, generator=g) * 2 - 0.7, torch.randn(2312, generator=g).to(torch.bfloat16), torch.randn(2312, generator=g).to(torch.bfloat16)
    ref8 = O.layer_norm(x8.double(), w8.double(), b8.double(), 1e-3)
    out = res32.layernorm(x8.to(gpu), _dev(w8, dtype), _dev(b8, dtype), 1e-3, rows=torch.tensor([4, 1], device=gpu))
    assert (out.cpu().double() - ref8[[4, 1]]).abs().max() < tol * 6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
def test_xielu_and_residual(gpu, dtype, tol):
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(3)
    z = (torch.randn(5, 64, generator=g) * 3).to(torch.bfloat16)
    pq = torch.tensor([0.3, -1.2]).to(torch.bfloat16)
    wide = torch.zeros(5, 100, dtype=dtype, device=gpu)
    wide[:, 10:74] = _dev(z, dtype)
    out = torch.zeros(5, 90, dtype=dtype, device=gpu)
    res32.xielu(wide[:, 10:74], _dev(pq, dtype), out[:, 20:84])
    ref = O.xielu(z.double(), float(pq[0]), float(pq[1]))
    assert (z > 0).any() and (z < 0).any()
    got = out.cpu().double()
    assert ((got[:, 20:84] - ref).abs() / (1 + ref.abs())).max() < tol
    assert got[:, :20].abs().max() == 0 and got[:, 84:].abs().max() == 0
    # rows whose width and leading dimensions are multiples of 8 (the 16-byte path in bf16)
    wide2, out2 = torch.zeros(5, 128, dtype=dtype, device=gpu), torch.zeros(5, 96, dtype=dtype, device=gpu)
    wide2[:, 16:80] = _dev(z, dtype)
    res32.xielu(wide2[:, 16:80], _dev(pq, dtype), out2[:, 32:96])
    assert ((out2.cpu().double()[:, 32:96] - ref).abs() / (1 + ref.abs())).max() < tol
    assert out2[:, :32].abs().max() == 0
    x = torch.randn(5, 64, generator=g)
    xd = x.to(gpu)
    res32.residual_add_scaled(xd, _dev(z, dtype), 0.37)
    assert (xd.cpu().double() - (x.double() + 0.37 * z.double())).abs().max() < 1e-5


def _paged(n_tokens, bs, nk, nv, dtype, perm_seed=0):
    """A cache of one layer with shuffled pages and a table for one sequence of n_tokens."""
    from llm_weighted_consensus_amd.models.cache import PagedLayerCache

    nb = -(-n_tokens // bs) + 3
    cache = PagedLayerCache([(nk, nv)], nb, bs, "cuda", dtype)
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(perm_seed)).tolist()
    table = perm[: -(-n_tokens // bs)]
    slots = [table[p // bs] * bs + p % bs for p in range(n_tokens)]
    return cache, table, slots


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("H,G,D,Dv,window", [(4, 2, 16, 8, 5), (3, 3, 12, 20, 33), (6, 1, 8, 72, 200), (2, 2, 24, 4, 1)])
def test_proj_norm_write_and_window_attention(gpu, dtype, tol, H, G, D, Dv, window):
    """q/k whole-projection norms, value blending, the cache write and the attention, against the oracle, with
    the sequence's pages shuffled and its rows cut into a portion and single decode rows."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(H * 100 + D)
    n, bs, eps = 70, 16, 1e-4
    nq, nk, nv = H * D, G * D, G * Dv
    pad = 8 if D % 8 == 0 and Dv % 8 == 0 else 5  # (rows of 8-element multiples take the 16-byte path in bf16)
    proj = (torch.randn(n, nq + nk + nv + pad, generator=g) * 2).to(torch.bfloat16)
    wq, wk = (1 + 0.3 * torch.randn(nq, generator=g)).to(torch.bfloat16), (1 + 0.3 * torch.randn(nk, generator=g)).to(torch.bfloat16)
    temp = (1 + torch.rand(H, generator=g)).to(torch.bfloat16)
    r1, r2 = (0.2 + torch.rand(H, generator=g)).to(torch.bfloat16), (0.2 + torch.rand(H, generator=g)).to(torch.bfloat16)
    lam = torch.tensor([0.3]).to(torch.bfloat16)
    v_first = torch.randn(n, nv, generator=g)
    scale = 0.21
    pd = proj.double()
    q = O.rms_norm_whole(pd[:, :nq], wq.double(), eps)
    k = O.rms_norm_whole(pd[:, nq:nq + nk], wk.double(), eps)
    v = (1 - float(lam)) * pd[:, nq + nk:nq + nk + nv] + float(lam) * v_first.double()
    ref = O.window_attention(q.view(n, H, D), k.view(n, G, D), v.view(n, G, Dv), H, G, window, scale, temp.double(),
                             r1.double(), r2.double())
    cache, table, slots = _paged(n, bs, nk, nv, dtype, perm_seed=D)
    head_scale = (temp.float() * scale).to(gpu)
    q_dev = res32.proj_norm_kv_write(_dev(proj, dtype), _dev(wq, dtype), _dev(wk, dtype), head_scale,
                                     torch.tensor(slots, dtype=torch.int32, device=gpu), cache.k[0], cache.v[0], H, D, eps,
                                     lam=_dev(lam, dtype), v0=v_first.to(gpu), vmode=2)
    kc, vc = (t.cpu().double() for t in cache.rows(0, torch.tensor(slots, device=gpu)))
    assert (kc - k).abs().max() < tol and (vc - v).abs().max() < tol * 3
    pos = torch.arange(n, dtype=torch.int32, device=gpu)
    out = torch.zeros(n, H * Dv + 3, dtype=dtype, device=gpu)
    cut = 41  # rows [0, cut) as one portion, the rest as single decode rows of the same sequence
    tab = torch.tensor([table], dtype=torch.int32, device=gpu)
    res32.window_attn(q_dev[:cut], cache.k[0], cache.v[0], pos[:cut], tab, r1.float().to(gpu), r2.float().to(gpu), window,
                      out[:cut, :H * Dv], H, G, cu_q=torch.tensor([0, cut], dtype=torch.int32, device=gpu))
    res32.window_attn(q_dev[cut:], cache.k[0], cache.v[0], pos[cut:], tab.repeat(n - cut, 1), r1.float().to(gpu),
                      r2.float().to(gpu), window, out[cut:, :H * Dv], H, G)
    got = out.cpu().double()
    assert (got[:, :H * Dv] - ref).abs().max() < tol * 2
    assert got[:, H * Dv:].abs().max() == 0


@pytest.mark.parametrize("H,G,D,Dv,window,bs", [(4, 2, 32, 64, 37, 16), (2, 1, 128, 32, 500, 16), (6, 3, 64, 128, 64, 8),
                                                 (2, 2, 32, 32, 1, 32)])
def test_matrix_core_portions(gpu, H, G, D, Dv, window, bs):
    """Prompt portions on the matrix-core kernel (bf16 cache): several items of unequal length, each the tail of a
    longer sequence whose head is already cached, tiles cut by item ends, window edges inside and across tiles;
    against the oracle on the cache's own (bf16) keys and values, and against the general kernel."""
    from llm_weighted_consensus_amd.models.cache import PagedLayerCache
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(D + Dv)
    k_lens, q_lens = [150, 64, 209, 3], [150, 1, 70, 2]
    nk, nv = G * D, G * Dv
    nb = sum(-(-n // bs) for n in k_lens) + 2
    cache = PagedLayerCache([(nk, nv)], nb, bs, "cuda", torch.bfloat16)
    pages = torch.randperm(nb, generator=g).tolist()
    temp, r1, r2 = 1 + torch.rand(H, generator=g), 0.3 + torch.rand(H, generator=g), 0.3 + torch.rand(H, generator=g)
    scale = 0.3
    width = max(-(-n // bs) for n in k_lens)
    tables, refs, qs, pos, cu = [], [], [], [], [0]
    for n, nq_ in zip(k_lens, q_lens):
        tab = [pages.pop() for _ in range(-(-n // bs))]
        tables.append(tab + [0] * (width - len(tab)))
        k = (torch.randn(n, nk, generator=g)).to(torch.bfloat16)
        v = (torch.randn(n, nv, generator=g)).to(torch.bfloat16)
        sl = torch.tensor([tab[p // bs] * bs + p % bs for p in range(n)], device=gpu)
        cache.set_rows(0, sl, k.to(gpu), v.to(gpu))
        q = torch.randn(n, H * D, generator=g) * 2
        ref = O.window_attention(q.double().view(n, H, D), k.double().view(n, G, D), v.double().view(n, G, Dv), H, G, window,
                                 scale, temp.double(), r1.double(), r2.double())
        refs.append(ref[n - nq_:])
        qs.append((q.view(n, H, D) * (temp * scale)[None, :, None]).reshape(n, H * D)[n - nq_:])
        pos.extend(range(n - nq_, n))
        cu.append(cu[-1] + nq_)
    ref = torch.cat(refs)
    qd = torch.cat(qs).float().to(gpu).contiguous()
    T = qd.shape[0]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    r1d, r2d = r1.to(gpu), r2.to(gpu)
    out_m = torch.zeros(T, H * Dv, dtype=torch.bfloat16, device=gpu)
    out_g = torch.zeros_like(out_m)
    assert res32.kernels().window_attn_mfma_ok(D, Dv)
    res32.window_attn(qd, cache.k[0], cache.v[0], i32(pos), i32(tables), r1d, r2d, window, out_m, H, G, cu_q=i32(cu),
                      k_lens=i32(k_lens), max_q=max(q_lens), bias=res32.distance_bias(r1d, r2d, window))
    res32.window_attn(qd, cache.k[0], cache.v[0], i32(pos), i32(tables), r1d, r2d, window, out_g, H, G, cu_q=i32(cu))
    tol = 0.02  # the outputs are rounded to bf16
    assert (out_g.cpu().double() - ref).abs().max() < tol
    assert (out_m.cpu().double() - ref).abs().max() < tol
    assert (out_m.float() - out_g.float()).abs().max() < tol
    # the last token of every item as a decode row (split over the keys when the window is long)
    last = [c - 1 for c in cu[1:]]
    out_d = torch.zeros(len(last), H * Dv, dtype=torch.bfloat16, device=gpu)
    res32.window_attn(qd[last].contiguous(), cache.k[0], cache.v[0], i32([pos[r] for r in last]), i32(tables), r1d, r2d,
                      window, out_d, H, G, bias=res32.distance_bias(r1d, r2d, window))
    assert (out_d.cpu().double() - ref[last]).abs().max() < tol


def test_value_publish_and_plain_modes(gpu):
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(5)
    n, H, D, nk, nv = 6, 2, 8, 8, 12
    proj = torch.randn(n, H * D + nk + nv, generator=g)
    cache, table, slots = _paged(n, 4, nk, nv, torch.float32)
    slots[2] = -1  # a padding row: nothing written
    before = cache.pool.clone()
    v0 = torch.zeros(n, nv, device=gpu)
    ones = torch.ones(H * D, device=gpu)
    res32.proj_norm_kv_write(proj.to(gpu), ones, torch.ones(nk, device=gpu), torch.ones(H, device=gpu),
                             torch.tensor(slots, dtype=torch.int32, device=gpu), cache.k[0], cache.v[0], H, D, 1e-6, v0=v0, vmode=1)
    assert torch.equal(v0.cpu(), proj[:, H * D + nk:])
    rows = [s for s in slots if s >= 0]
    kc, vc = cache.rows(0, torch.tensor(rows, device=gpu))
    assert torch.equal(vc.cpu(), proj[[0, 1, 3, 4, 5], H * D + nk:])
    rest = torch.tensor([s for s in range(cache.num_blocks * 4) if s not in rows], device=gpu)
    for a, b in zip(cache.rows(0, rest), (before[:, :4 * nk].reshape(-1, nk)[rest], torch.zeros(len(rest), nv, device=gpu))):
        assert torch.equal(a, b)


@pytest.mark.parametrize("decode", [False, True])
def test_window_edge_and_far_key_stand_out(gpu, decode):
    """One key gets a score far above all others; the value it carries must dominate the output exactly while the
    key is inside the window (distance window - 1, across several pages) and vanish one position later."""
    from llm_weighted_consensus_amd.ops import res32

    H = G = 1
    D, Dv, window, bs, n = 8, 4, 300, 16, 700
    special = 250
    k = torch.zeros(n, D)
    k[:, 0] = 0.01
    k[special, 1] = 50.0
    v = torch.zeros(n, Dv)
    v[:, 0] = 1.0
    v[special] = torch.tensor([0.0, 7.0, 0.0, 0.0])
    cache, table, slots = _paged(n, bs, D, Dv, torch.float32, perm_seed=3)
    sl = torch.tensor(slots, device=gpu)
    cache.set_rows(0, sl, k.to(gpu), v.to(gpu))
    rows = [special, special + 1, special + window - 1, special + window, n - 1]
    q = torch.zeros(len(rows), D, device=gpu)
    q[:, 1] = 1.0
    pos = torch.tensor(rows, dtype=torch.int32, device=gpu)
    out = torch.zeros(len(rows), Dv, device=gpu)
    tab = torch.tensor([table], dtype=torch.int32, device=gpu)
    zero = torch.zeros(1, device=gpu)
    if decode:
        res32.window_attn(q, cache.k[0], cache.v[0], pos, tab.repeat(len(rows), 1), zero, zero, window, out, H, G)
    else:
        # (rows of one portion need not be consecutive positions for the kernel: each carries its own)
        res32.window_attn(q, cache.k[0], cache.v[0], pos, tab, zero, zero, window, out, H, G,
                          cu_q=torch.tensor([0, len(rows)], dtype=torch.int32, device=gpu))
    got = out.cpu()
    for r in range(3):  # the special key is visible: its value wins
        assert got[r, 1] > 6.99 and got[r, 0] < 0.01, (r, got[r])
    for r in (3, 4):    # one past the window's edge, and far past: gone
        assert got[r, 1] == 0 and abs(got[r, 0] - 1) < 1e-6, (r, got[r])


# ------------------------------------------------------------------ the model through the engine
CONFIGS = {
    # heads != kv_heads != 1, dim != vdim, a layer without feed-forward, blending that starts in the second layer
    "mixed": dict(width=48, vocab=300, layers=[
        dict(heads=4, kv_heads=2, dim=16, vdim=8, window=6, v_mix=False, ff=64),
        dict(heads=4, kv_heads=2, dim=16, vdim=8, window=6, v_mix=True, ff=None),
        dict(heads=2, kv_heads=1, dim=8, vdim=16, window=19, v_mix=True, ff=40),
        dict(heads=8, kv_heads=4, dim=4, vdim=4, window=3, v_mix=True, ff=72)]),
    # sizes the matrix-core kernels take (bf16): dim != vdim, one window shorter than a key tile, one longer
    "cores": dict(width=64, vocab=320, layers=[
        dict(heads=4, kv_heads=2, dim=32, vdim=64, window=40, v_mix=True, ff=64),
        dict(heads=2, kv_heads=1, dim=128, vdim=32, window=7, v_mix=False, ff=None),
        dict(heads=4, kv_heads=2, dim=32, vdim=64, window=90, v_mix=True, ff=48)]),
    # odd sizes, heads == kv_heads, a window longer than any test prompt and a window of one
    "odd": dict(width=40, vocab=97, layers=[
        dict(heads=3, kv_heads=3, dim=12, vdim=20, window=1000, v_mix=True, ff=50),
        dict(heads=3, kv_heads=3, dim=12, vdim=20, window=1, v_mix=True, ff=30)]),
}


def _build(tmp_path, name, dtype, seed=0, **engine_kw):
    from safetensors.torch import save_file

    from llm_weighted_consensus_amd.engine.engine import LLMEngine
    from llm_weighted_consensus_amd.engine.tokenizer import load_tokenizer
    from llm_weighted_consensus_amd.models.registry import load_model

    c = CONFIGS[name]
    cfg = O.make_config(c["width"], c["vocab"], c["layers"])
    W = O.make_weights(cfg, seed)
    d = tmp_path / f"{name}-{seed}"
    d.mkdir(exist_ok=True)
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(d / "model.safetensors"))
    model = load_model(str(d), dtype=dtype)
    kw = dict(block_size=16, num_blocks=24, max_batch=4, max_model_len=256, use_graphs=False, prefix_sharing=False,
              tune_gc=False)
    kw.update(engine_kw)
    return cfg, W, model, LLMEngine(model, load_tokenizer({}, cfg["vocab"]), **kw)


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _err(got, ref):
    return float((got.cpu().double() - ref).abs().max())


TOL = {torch.float32: 2e-4, torch.bfloat16: 0.25}


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt_and_layers(gpu, tmp_path, name, dtype):
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(45, cfg["vocab"], 1)
    layers, ref_layers = [], []
    model.on_layer = lambda li, x: layers.append(x.detach().cpu().double().clone())
    got = eng.step_tokens([("a", toks, list(range(len(toks))))], ["a"])
    model.on_layer = None
    ref = O.forward(cfg, W, toks, ref_layers)
    if dtype == torch.float32:
        for a, b in zip(layers, ref_layers):
            assert (a - b).abs().max() < 1e-4
    assert _err(got, ref) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("cores", torch.bfloat16), ("odd", torch.bfloat16)])
def test_few_wanted_rows_and_the_cache_they_leave(gpu, tmp_path, name, dtype):
    """Portions of which few logits are wanted run their last layer on those rows only; the logits match, and so do
    the tokens decoded afterwards from the cache those steps left (every row's keys and values were written)."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    a, b = _tokens(64, cfg["vocab"], 5), _tokens(37, cfg["vocab"], 6)
    ra, rb = O.forward(cfg, W, a), O.forward(cfg, W, b)
    got = eng.step_tokens([("a", a[:50], [49, 3]), ("b", b[:30], [29])])
    assert _err(got, torch.cat([ra[[49, 3]], rb[[29]]])) < TOL[dtype]
    got = eng.step_tokens([("a", a[50:60], []), ("b", b[30:], [6])], ["b"])
    assert _err(got, rb[[36]]) < TOL[dtype]
    for i in range(60, 64):
        got = eng.step_tokens([("a", [a[i]], [0])], ["a"] if i == 63 else [])
        assert _err(got, ra[[i]]) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("odd", torch.float32), ("cores", torch.float32),
                                        ("cores", torch.bfloat16)])
def test_decode_token_by_token_and_portions(gpu, tmp_path, name, dtype):
    """The same logits whether a prompt comes whole, token by token from the first token on, or in portions of
    changing sizes (down to two tokens, cut inside pages and windows)."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(75, cfg["vocab"], 2)
    ref = O.forward(cfg, W, toks)
    rows = []
    for i, t in enumerate(toks):
        rows.append(eng.step_tokens([("d", [t], [0])], ["d"] if i + 1 == len(toks) else []))
    assert _err(torch.cat(rows), ref) < TOL[dtype]
    for sizes in ([2, 2, 13, 3, 16, 2, 30, 7], [17, 16, 15, 2, 25], [1, 2, 5, 67]):
        assert sum(sizes) == len(toks)
        rows, a = [], 0
        for n in sizes:
            rows.append(eng.step_tokens([("p", toks[a:a + n], list(range(n)))], ["p"] if a + n == len(toks) else []))
            a += n
        assert _err(torch.cat(rows), ref) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("mixed", torch.bfloat16), ("cores", torch.bfloat16)])
def test_unequal_batches_and_page_reuse(gpu, tmp_path, name, dtype):
    """Up to four live sequences of unequal lengths, portions beside single tokens, in a pool so small that pages
    are freed and taken again; every position equals the sequence run alone."""
    cfg, W, model, eng = _build(tmp_path, name, dtype, num_blocks=14)
    seqs = {k: _tokens(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate([("a", 70), ("b", 9), ("c", 40), ("d", 33), ("e", 58), ("f", 1)])}
    ref = {k: O.forward(cfg, W, t) for k, t in seqs.items()}
    at = {k: 0 for k in seqs}
    plan = [[("a", 30), ("b", 2)], [("a", 1), ("b", 7), ("c", 17)], [("a", 1), ("c", 1), ("d", 33)], [("a", 2), ("c", 22)],
            [("a", 36), ("d", 0)], [("e", 20), ("f", 1)], [("e", 1)], [("e", 37)]]
    worst = 0.0
    for step in plan:
        entries, end, spans = [], [], []
        for k, n in step:
            if n == 0:
                continue
            a = at[k]
            entries.append((k, seqs[k][a:a + n], list(range(n))))
            spans.append((k, a, n))
            at[k] = a + n
            if at[k] == len(seqs[k]):
                end.append(k)
        got = eng.step_tokens(entries, end)
        o = 0
        for k, a, n in spans:
            worst = max(worst, _err(got[o:o + n], ref[k][a:a + n]))
            o += n
    assert all(at[k] == len(seqs[k]) for k in seqs)
    assert worst < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks
    with pytest.raises(RuntimeError):  # more than the pool holds: refused before anything runs
        eng.step_tokens([("x", _tokens(250, cfg["vocab"], 3), [0])])


def test_window_edge_through_the_model(gpu, tmp_path):
    """A token's logits change with a token exactly window - 1 back and not with one a position farther, in a
    prompt portion and in single-token decoding (one-layer model: no second hop)."""
    from llm_weighted_consensus_amd.engine.engine import LLMEngine  # noqa: F401

    CONFIGS["edge"] = dict(width=32, vocab=260, layers=[dict(heads=2, kv_heads=1, dim=8, vdim=8, window=21, v_mix=True, ff=None)])
    cfg, W, model, eng = _build(tmp_path, "edge", torch.float32)
    base = _tokens(60, 260, 7)
    i, w = 50, 21

    def last_logits(toks, decode_from):
        out = eng.step_tokens([("s", toks[:decode_from], [decode_from - 1] if decode_from == i + 1 else [])],
                              ["s"] if decode_from == i + 1 else [])
        for p in range(decode_from, i + 1):
            out = eng.step_tokens([("s", [toks[p]], [0])], ["s"] if p == i else [])
        return out[0].cpu()

    for decode_from in (i + 1, i - 30):
        ref = last_logits(base, decode_from)
        inside, outside = list(base), list(base)
        inside[i - w + 1] = (base[i - w + 1] + 1) % 260
        outside[i - w] = (base[i - w] + 1) % 260
        assert (last_logits(inside, decode_from) - ref).abs().max() > 1e-4
        assert (last_logits(outside, decode_from) - ref).abs().max() < 1e-6


def _check_greedy(cfg, W, prompt, got, slack=0.04):
    """Every generated token is the oracle's best next token GIVEN the engine's own tokens so far, up to near-ties
    (the sampler reads bf16 logits: two logits closer than their rounding may swap); most are the exact argmax."""
    lg = O.forward(cfg, W, list(prompt) + list(got[:-1]))[len(prompt) - 1:]
    exact = 0
    for t, tok in enumerate(got):
        assert 0 <= tok < cfg["vocab"]
        assert float(lg[t].max() - lg[t, tok]) < slack, f"token {t}: {tok} is {float(lg[t].max() - lg[t, tok])} below the best"
        exact += int(lg[t].argmax()) == tok
    assert exact >= 0.8 * len(got)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_scheduler(gpu, tmp_path, graphs):
    """engine.generate (admission, paged prefill, batched decode steps, the fused sampler at temperature 0; with
    hipGraph replay of the decode step when ``graphs``) against the oracle's greedy continuation: two prompts of
    unequal length, a long decode that crosses pages and leaves the first window."""
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, use_graphs=graphs, num_blocks=40)
    prompts = [_tokens(23, 250, 21), _tokens(5, 250, 22)]
    n_new = 60
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True))
    for p, o in zip(prompts, out):
        assert len(o[0]) == n_new
        _check_greedy(cfg, W, p, o[0])
    assert eng.bm.num_free == eng.bm.num_blocks


def test_generation_chunked_prefill_and_forks(gpu, tmp_path):
    """Chunked prefill (prompt portions beside running decodes) and n > 1 (forked sequences sharing prompt pages,
    copy-on-write of the last page) give the greedy continuation too."""
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, num_blocks=48, chunked_prefill=8, max_batch=8)
    prompts = [_tokens(37, 250, 31), _tokens(12, 250, 32)]
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True), n=2)
    for p, o in zip(prompts, out):
        assert len(o) == 2 and o[0] == o[1]  # greedy forks of one prompt agree
        _check_greedy(cfg, W, p, o[0])
    assert eng.bm.num_free == eng.bm.num_blocks


def test_split_reduction_output_projection(gpu, tmp_path):
    """A model whose [o | down] reduction is long enough for the decode step's split-K path (few rows): decode rows
    (split) and a long portion (one GEMM) both match the oracle."""
    CONFIGS["wide"] = dict(width=32, vocab=288, layers=[dict(heads=2, kv_heads=1, dim=32, vdim=64, window=50, v_mix=True, ff=4096 - 128)])
    cfg, W, model, eng = _build(tmp_path, "wide", torch.bfloat16, num_blocks=40, max_model_len=512)
    assert model._split_ok
    toks = _tokens(300, 288, 5)
    ref = O.forward(cfg, W, toks)
    got = [eng.step_tokens([("w", toks[:290], list(range(290)))])]
    for i in range(290, 300):
        got.append(eng.step_tokens([("w", [toks[i]], [0])], ["w"] if i == 299 else []))
    assert _err(torch.cat(got), ref) < TOL[torch.bfloat16]


def test_trace_replay_command_line(gpu, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, ``done <step>`` lines and <step>.f32 files out; two sequences
    interleaved (portions beside single tokens, one sitting a step out), pages given back at ``end``."""
    import os
    import subprocess
    import sys

    import numpy as np
    from safetensors.torch import save_file

    c = CONFIGS["odd"]
    cfg = O.make_config(c["width"], c["vocab"], c["layers"])
    W = O.make_weights(cfg, 4)
    mdir, out = tmp_path / "model", tmp_path / "out"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(mdir / "model.safetensors"))
    a, b = _tokens(40, cfg["vocab"], 1), _tokens(21, cfg["vocab"], 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:20], "want": []}, {"id": "a", "tokens": a[30:31], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[31:], "want": [8, 2]}], "end": ["a"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(mdir), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    ra, rb = O.forward(cfg, W, a), O.forward(cfg, W, b)
    want = {0: ra[[0, 29]], 2: rb[[20]], 3: ra[[39, 33]], 1: ra[[30]]}
    for step, ref in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4")).view(-1, cfg["vocab"])
        assert _err(got, ref) < TOL[torch.float32]
    assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "2.f32", "3.f32"]


def test_loader_refuses_wrong_shapes(gpu, tmp_path):
    from safetensors.torch import save_file

    from llm_weighted_consensus_amd.models.registry import load_model

    c = CONFIGS["odd"]
    cfg = O.make_config(c["width"], c["vocab"], c["layers"])
    W = O.make_weights(cfg, 0)
    W["l1.mix.k"] = W["l1.mix.k"][:-1]
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError):
        load_model(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(dict(cfg, architecture="Nope")))
    with pytest.raises(ValueError):
        load_model(str(tmp_path))
