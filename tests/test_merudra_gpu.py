"""Merudra on the GPU against the plain fp64 oracle (tests/merudra_oracle.py): each mechanism alone, then the model
through the engine — whole prompts, token-by-token decoding, portions, unequal batches, pages and state slots used
again, the first tokens of a sequence, keys far away and at page borders, the temperature's steps, long decoding
and greedy generation through the scheduler.  Small configurations with random weights, sizes chosen so that
nothing the design allows to differ happens to be equal or 1."""
import json
import math

import pytest
import torch

import merudra_oracle as O

pytestmark = pytest.mark.gpu

F64 = torch.float64


def _dev(t, dtype):
    return t.to("cuda", dtype=dtype).contiguous()


def _items(lens, slots, starts, gpu):
    """StepItems of portions with ``lens`` rows starting at positions ``starts`` in state slots ``slots``."""
    from llm_weighted_consensus_amd.ops import res32

    cu, row_item, pos = [0], [], []
    for i, (n, p0) in enumerate(zip(lens, starts)):
        cu.append(cu[-1] + n)
        row_item += [i] * n
        pos += list(range(p0, p0 + n))
    t = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu)  # noqa: E731
    return res32.StepItems(t(row_item), t(cu), t(slots), t(pos))


# ------------------------------------------------------------------ mechanisms, one by one
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("taps,C,tap_major", [(1, 37, False), (2, 37, False), (4, 37, True), (4, 40, True), (3, 264, True)])
def test_conv_with_history_in_portions(gpu, dtype, tol, taps, C, tap_major):
    """x + conv(x) and silu(conv(x)): two sequences cut into portions (one shorter than the history, single rows,
    the two interleaved in one step) in slots that held other data before, against the whole-sequence oracle."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(taps)
    na, nb = 23, 9
    xa, xb = torch.randn(na, C, generator=g).to(dtype), torch.randn(nb, C, generator=g).to(dtype)
    w = torch.randn(C, taps, generator=g)
    # tap-major storage with a width that is a multiple of four takes the 16-byte kernel
    wg = w.to(gpu).t().contiguous().t() if tap_major else w.to(gpu)
    hist = torch.randn(4, taps - 1, C, generator=g).to(gpu) * 50  # stale contents of earlier sequences
    for mode in (0, 1):
        ya, yb = O.causal_conv(xa.double(), w.double()), O.causal_conv(xb.double(), w.double())
        ra, rb = (xa.double() + ya, xb.double() + yb) if mode == 0 else (O.silu(ya), O.silu(yb))
        plan = [[("a", 1)], [("a", 2), ("b", 1)], [("b", 2), ("a", 1)], [("a", 7)], [("b", 6), ("a", 12)]]
        at, got = {"a": 0, "b": 0}, {"a": [], "b": []}
        src, slot = {"a": xa, "b": xb}, {"a": 2, "b": 0}
        for step in plan:
            x = torch.cat([src[k][at[k]:at[k] + n] for k, n in step]).to(gpu)
            items = _items([n for _, n in step], [slot[k] for k, _ in step], [at[k] for k, _ in step], gpu)
            out = torch.empty(x.shape[0], C, dtype=dtype, device=gpu)
            out2 = torch.empty_like(out) if mode == 0 and dtype == torch.bfloat16 else None
            res32.conv_hist(x, wg, hist, items, out, mode=mode, out2=out2)
            if out2 is not None:
                assert torch.equal(out2, x)
            o = 0
            for k, n in step:
                got[k].append(out[o:o + n].cpu())
                o, at[k] = o + n, at[k] + n
        assert at == {"a": na, "b": nb}
        assert (torch.cat(got["a"]).double() - ra).abs().max() < tol * 8
        assert (torch.cat(got["b"]).double() - rb).abs().max() < tol * 8


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("taps,C", [(4, 40), (2, 264), (8, 12), (9, 12)])
def test_conv_many_rows_of_several_sequences(gpu, dtype, tol, taps, C):
    """A step of 128 rows of three sequences that each continue behind a short first portion (the kernel that keeps a
    row's earlier inputs in registers takes it for up to 8 taps): item borders inside a thread's rows, histories
    read at the borders, against the oracle."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(taps * 7 + C)
    lens, first = [60, 45, 33], [7, 2, 1]
    xs = [torch.randn(n, C, generator=g).to(dtype) for n in lens]
    w = torch.randn(C, taps, generator=g)
    wg = w.to(gpu).t().contiguous().t()
    hist = torch.randn(4, taps - 1, C, generator=g).to(gpu) * 50
    slots = [1, 3, 0]
    for mode in (0, 1):
        refs = [O.causal_conv(x.double(), w.double()) for x in xs]
        refs = [x.double() + y if mode == 0 else O.silu(y) for x, y in zip(xs, refs)]
        x1 = torch.cat([x[:f] for x, f in zip(xs, first)]).to(gpu)
        o1 = torch.empty(x1.shape[0], C, dtype=dtype, device=gpu)
        res32.conv_hist(x1, wg, hist, _items(first, slots, [0, 0, 0], gpu), o1, mode=mode)
        x2 = torch.cat([x[f:] for x, f in zip(xs, first)]).to(gpu)
        o2 = torch.empty(x2.shape[0], C, dtype=dtype, device=gpu)
        res32.conv_hist(x2, wg, hist, _items([n - f for n, f in zip(lens, first)], slots, first, gpu), o2, mode=mode)
        a1 = a2 = 0
        for k, (n, f) in enumerate(zip(lens, first)):
            got = torch.cat([o1[a1:a1 + f], o2[a2:a2 + n - f]]).cpu().double()
            assert (got - refs[k]).abs().max() < tol * 10, (mode, k)
            a1, a2 = a1 + f, a2 + n - f


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("taps,C,tap_major", [(1, 10, False), (3, 37, False), (4, 40, True)])
def test_conv_decode_steps_advance_the_history_themselves(gpu, dtype, tol, taps, C, tap_major):
    """Decode steps (every row its own sequence) compute and move the history on in ONE kernel: three sequences side
    by side, one joining later behind a portion, against the oracle."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(taps + C)
    n = 12
    xs = [torch.randn(n, C, generator=g).to(dtype) for _ in range(3)]
    w = torch.randn(C, taps, generator=g)
    wg = w.to(gpu).t().contiguous().t() if tap_major else w.to(gpu)
    refs = [x.double() + O.causal_conv(x.double(), w.double()) for x in xs]
    hist = torch.randn(5, taps - 1, C, generator=g).to(gpu) * 50
    slots = [3, 0, 4]
    got = [[], [], []]
    # sequence 2 starts with a portion of 5 rows (separate history update), then joins the decode steps
    out = torch.empty(5, C, dtype=dtype, device=gpu)
    res32.conv_hist(xs[2][:5].to(gpu), wg, hist, _items([5], [slots[2]], [0], gpu), out)
    got[2].append(out.cpu())
    for t in range(n):
        who = [0, 1] + ([2] if t >= 5 else [])
        x = torch.stack([xs[k][t] for k in who]).to(gpu)
        items = res32.StepItems.rows(torch.tensor([slots[k] for k in who], dtype=torch.int32, device=gpu),
                                     torch.full((len(who),), t, dtype=torch.int32, device=gpu))
        out = torch.empty(len(who), C, dtype=dtype, device=gpu)
        res32.conv_hist(x, wg, hist, items, out)
        for j, k in enumerate(who):
            got[k].append(out[j:j + 1].cpu())
    for k in range(3):
        assert (torch.cat(got[k]).double() - refs[k]).abs().max() < tol * 8


@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 12, 20), (2, 2, 64, 64), (3, 1, 80, 72), (2, 1, 130, 8)])
def test_delta_rule_whole_portions_and_single_tokens(gpu, H, G, D, Dv):
    """The gated delta rule of the kernel (unit q / k, decay, beta, state carried in a slot) against the oracle's
    recurrence: one portion, portions of 1..5 rows and single rows; a second sequence in the same step; the slot
    held another sequence's state before."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(H * 100 + D)
    n, nq = 21, G * D
    qkv = torch.randn(n, 2 * nq + H * Dv, generator=g)
    ba = torch.randn(n, 5 + 2 * H, generator=g)
    A_log, dtb = torch.randn(H, generator=g) * 0.5, torch.randn(H, generator=g)
    ref = torch.zeros(n, H, Dv, dtype=F64)
    q, k, v = qkv[:, :nq].double().view(n, G, D), qkv[:, nq:2 * nq].double().view(n, G, D), qkv[:, 2 * nq:].double().view(n, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(ba[:, 2:2 + H].double())
    dec = torch.exp(-torch.exp(A_log.double()) * torch.nn.functional.softplus(ba[:, 5 + H:].double() + dtb.double()))
    S_ref = []
    for h in range(H):
        ref[:, h], S = O.delta_rule(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], beta[:, h], dec[:, h])
        S_ref.append(S)
    for cuts in ([n], [1, 2, 5, 1, 1, 4, 3, 4], [1] * n):
        state = torch.randn(3, H, D, Dv, generator=g).to(gpu) * 7  # stale
        outs, a = [], 0
        for c in cuts:
            rows = slice(a, a + c)
            # a second, unrelated sequence beside it in the step (slot 0), started fresh every time
            x = torch.cat([qkv[rows], qkv[:2]]).to(gpu)
            b = torch.cat([ba[rows], ba[:2]]).to(gpu)
            items = _items([c, 2], [2, 0], [a, 0], gpu)
            o = res32.delta_rule(x, b, 2, 5 + H, A_log.to(gpu), dtb.to(gpu), state, items, H, G)
            outs.append(o[:c].cpu())
            assert (o[c:].cpu().double().view(2, H, Dv) - ref[:2]).abs().max() < 2e-5
            a += c
        assert (torch.cat(outs).double().view(n, H, Dv) - ref).abs().max() < 5e-5
        assert (state[2].cpu().double() - torch.stack(S_ref)).abs().max() < 5e-5


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("H,Dv", [(3, 20), (5, 32), (9, 128), (2, 7)])
def test_head_norm_gate_and_gated_norm_residual(gpu, dtype, tol, H, Dv):
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(5)
    T, d = 7, 52
    o = torch.randn(T, H * Dv, generator=g) * 3
    gate = torch.randn(T, H * Dv + 6, generator=g).to(dtype)
    w = 1 + 0.2 * torch.randn(Dv, generator=g)
    out = torch.empty(T, H * Dv, dtype=dtype, device=gpu)
    res32.head_norm_gate(o.to(gpu), out, H, 1e-3, w=w.to(gpu), gate=gate.to(gpu)[:, 6:], mode="silu")
    ref = (O.rms_unit(o.double().view(T, H, Dv), 1e-3) * w.double()).reshape(T, -1) * O.silu(gate[:, 6:].double())
    assert (out.cpu().double() - ref).abs().max() < tol * 8
    gate8 = torch.randn(T, H * Dv + 8, generator=g).to(dtype)  # an offset the 16-byte kernel takes
    res32.head_norm_gate(o.to(gpu), out, H, 1e-3, w=w.to(gpu), gate=gate8.to(gpu)[:, 8:], mode="sigmoid")
    ref = (O.rms_unit(o.double().view(T, H, Dv), 1e-3) * w.double()).reshape(T, -1) * torch.sigmoid(gate8[:, 8:].double())
    assert (out.cpu().double() - ref).abs().max() < tol * 8
    res32.head_norm_gate(o.to(gpu), out, H, 1e-3)
    assert (out.cpu().double() - O.rms_unit(o.double().view(T, H, Dv), 1e-3).reshape(T, -1)).abs().max() < tol * 4
    x = torch.randn(T, d, generator=g) * 4
    y, r = torch.randn(T, d, generator=g).to(dtype), torch.randn(T, d, generator=g).to(dtype)
    wn = 1 + 0.2 * torch.randn(d, generator=g)
    xg = x.to(gpu)
    cast = torch.empty(T, d, dtype=torch.bfloat16, device=gpu)
    res32.gated_norm_residual(xg, y.to(gpu), wn.to(gpu), 1e-4, gate_logits=r.to(gpu), x_cast=cast)
    ref = x.double() + O.rms_unit(y.double() * torch.sigmoid(r.double()), 1e-4) * wn.double()
    assert (xg.cpu().double() - ref).abs().max() < 1e-5
    assert torch.equal(cast, xg.to(torch.bfloat16))
    xg = x.to(gpu)
    res32.gated_norm_residual(xg, y.float().to(gpu), wn.to(gpu), 1e-4)  # fp32 result, no gate
    assert (xg.cpu().double() - (x.double() + O.rms_unit(y.double(), 1e-4) * wn.double())).abs().max() < 1e-5
    for dw in (2320, 1030):  # several 16-byte chunks per thread; a width the 16-byte kernel does not take
        xw, yw, rw = torch.randn(3, dw, generator=g), torch.randn(3, dw, generator=g).to(dtype), torch.randn(3, dw, generator=g).to(dtype)
        ww = 1 + 0.2 * torch.randn(dw, generator=g)
        xg = xw.to(gpu)
        res32.gated_norm_residual(xg, yw.to(gpu), ww.to(gpu), 1e-4, gate_logits=rw.to(gpu))
        ref = xw.double() + O.rms_unit(yw.double() * torch.sigmoid(rw.double()), 1e-4) * ww.double()
        assert (xg.cpu().double() - ref).abs().max() < 1e-5
    rows = torch.tensor([6, 0, 6, 2], device=gpu)
    n = res32.rmsnorm_rows(x.to(gpu), wn.to(gpu), 1e-4, dtype, rows=rows)
    assert (n.cpu().double() - (O.rms_unit(x.double(), 1e-4) * wn.double())[rows.cpu()]).abs().max() < tol * 6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
def test_embed_side_input_gate_mul_and_stack_mix(gpu, dtype, tol):
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(6)
    V, d, sd, T = 19, 28, 5, 6
    table, side = torch.randn(V, d, generator=g).to(dtype), torch.randn(V, 3 * sd, generator=g).to(dtype)
    toks = torch.tensor([0, 18, 4, 4, 9, 1], dtype=torch.int32)
    x = res32.embed_rows(table.to(gpu), toks.to(gpu))
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), table.float()[toks.long()])
    z = torch.randn(T, sd, generator=g).to(dtype)
    out = res32.gelu_mul_rows(z.to(gpu), side.to(gpu), 2 * sd, toks.to(gpu))
    ref = O.gelu_tanh(z.double()) * side.double()[toks.long()][:, 2 * sd:3 * sd]
    assert (out.cpu().double() - ref).abs().max() < tol * 4
    a, gt = torch.randn(T, 11, generator=g).to(dtype), torch.randn(T, 30, generator=g).to(dtype)
    ag = a.to(gpu)
    res32.gate_mul(ag, gt.to(gpu)[:, 19:], "sigmoid")
    assert (ag.cpu().double() - a.double() * torch.sigmoid(gt[:, 19:].double())).abs().max() < tol * 4
    a, gt = torch.randn(T, 12, generator=g).to(dtype), torch.randn(T, 28, generator=g).to(dtype)  # the 16-byte kernel
    ag = a.to(gpu)
    res32.gate_mul(ag, gt.to(gpu)[:, 16:], "silu")
    assert (ag.cpu().double() - a.double() * O.silu(gt[:, 16:].double())).abs().max() < tol * 4
    X = torch.randn(5, T, d, generator=g)
    coef = torch.randn(4, generator=g)
    Xg = X.to(gpu)
    res32.stack_mix(Xg, coef.to(gpu), 3, Xg[4])  # into a later plane of the stack itself
    assert (Xg[4].cpu().double() - sum(coef[j].double() * X[j].double() for j in range(3))).abs().max() < 1e-5


def _paged(n_tokens, bs, nk, nv, dtype, perm_seed=0):
    from llm_weighted_consensus_amd.models.cache import PagedLayerCache

    nb = -(-n_tokens // bs) + 3
    cache = PagedLayerCache([(nk, nv)], nb, bs, "cuda", dtype)
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(perm_seed))[: -(-n_tokens // bs)]
    slots = torch.tensor([int(perm[t // bs]) * bs + t % bs for t in range(n_tokens)], dtype=torch.int32)
    return cache, perm.to(torch.int32), slots


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 4e-2)])
@pytest.mark.parametrize("H,G,D,every", [(4, 2, 12, 5), (6, 6, 64, 16), (2, 1, 128, 3), (3, 3, 20, 1)])
def test_head_norm_cache_write_and_attention(gpu, dtype, tol, H, G, D, every):
    """q / k unit-RMS per head, the temperature's steps (positions around every multiple of ``every``), the keys as
    projected stored as values, causal attention over shuffled pages: portions and single rows, against the oracle."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(H + D)
    n, bs, scale, coef, eps = 45, 16, 0.37, 0.6, 1e-4
    nq, nk = H * D, G * D
    proj = (torch.randn(n, nq + nk + (4 if D % 16 == 0 else 3), generator=g) * 2).to(dtype)  # (row stride: both kernels)
    q, k = proj[:, :nq].double().view(n, H, D), proj[:, nq:nq + nk].double().view(n, G, D)
    qn = O.rms_unit(q, eps) * O.query_temperature(range(n), coef, every)[:, None, None]
    ref = O.softmax_attention(qn, O.rms_unit(k, eps), k, H, G, scale)
    cache, table, slots = _paged(n, bs, nk, nk, dtype, 3)
    pos = torch.arange(n, dtype=torch.int32)
    z = torch.zeros(H, device=gpu)
    table_g = table.to(gpu)[None]
    cuts = [17, 2, 1, 1, 9, 15]
    outs, a = [], 0
    for c in cuts:
        rows = slice(a, a + c)
        qo = res32.head_norm_kv_write(proj[rows].to(gpu), nq, nq, pos[rows].to(gpu), slots[rows].to(gpu), cache.k[0], cache.v[0],
                                      H, G, eps, scale, coef, every)
        out = torch.empty(c, nq, dtype=dtype, device=gpu)
        if c == 1:  # a decode row: table row = row
            res32.window_attn(qo, cache.k[0], cache.v[0], pos[rows].to(gpu), table_g, z, z, 1 << 30, out, H, G)
        else:
            res32.window_attn(qo, cache.k[0], cache.v[0], pos[rows].to(gpu), table_g, z, z, 1 << 30, out, H, G,
                              cu_q=torch.tensor([0, c], dtype=torch.int32, device=gpu),
                              k_lens=torch.tensor([a + c], dtype=torch.int32, device=gpu), max_q=c)
        outs.append(out.cpu())
        a += c
    assert (torch.cat(outs).double() - ref).abs().max() < tol * 6
    kc, vc = cache.rows(0, slots.long().to(gpu))
    assert (kc.cpu().double() - O.rms_unit(k, eps).reshape(n, nk)).abs().max() < tol
    assert (vc.cpu().double() - k.reshape(n, nk)).abs().max() < tol * 4


@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_far_key_and_page_borders_stand_out(gpu, decode, dtype):
    """Among 300 keys over 19 shuffled pages, the query is made to match ONE key (at the sequence's first token, at
    both sides of page borders, far back, and itself): the output must be that key's value."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(11)
    n, bs, H, G, D = 300, 16, 2, 1, 32
    k = torch.randn(n, D, generator=g).to(torch.bfloat16)
    cache, table, slots = _paged(n, bs, D, D, dtype, 5)
    cache.set_rows(0, slots.long().to(gpu), O.rms_unit(k.double(), 1e-5).to(dtype).to(gpu), k.to(dtype).to(gpu))
    z = torch.zeros(H, device=gpu)
    for j in (0, 1, 15, 16, 17, 143, 144, 255, 256, 298, 299):
        q = torch.zeros(1, H * D)
        q[0, :D] = O.rms_unit(k[j].double(), 1e-5).float() * 40  # head 0 looks for key j; head 1 sees a flat softmax
        out = torch.empty(1, H * D, dtype=dtype, device=gpu)
        pos = torch.tensor([n - 1], dtype=torch.int32, device=gpu)
        kw = {} if decode else dict(cu_q=torch.tensor([0, 1], dtype=torch.int32, device=gpu),
                                    k_lens=torch.tensor([n], dtype=torch.int32, device=gpu), max_q=1)
        res32.window_attn(q.to(gpu), cache.k[0], cache.v[0], pos, table.to(gpu)[None], z, z, 1 << 30, out, H, G, **kw)
        assert (out[0, :D].cpu().double() - k[j].double()).abs().max() < 0.05, j
        assert (out[0, D:].cpu().double() - k.double().mean(0)).abs().max() < 0.05


@pytest.mark.parametrize("E,I,top,d", [(5, 3, 3, 24), (30, 10, 4, 24), (90, 10, 6, 23)])
def test_router_identity_experts_and_correction(gpu, E, I, top, d):
    """The correction moves the choice and not the weight; identity experts return the input; weights are the
    softmax over ALL router outputs, not renormalised; expert-major rows cover every real choice exactly once."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(8)
    T, ff = 50, 10
    h = torch.randn(T, d, generator=g)
    W = {"r.router": torch.randn(E + I, d, generator=g) * 0.6, "r.correction": torch.randn(E + I, generator=g) * 0.3 / (E + I) * 8}
    for e in range(E):
        W.update({f"r.e{e}.gate": torch.randn(ff, d, generator=g) * 0.3, f"r.e{e}.up": torch.randn(ff, d, generator=g) * 0.3,
                  f"r.e{e}.down": torch.randn(d, ff, generator=g) * 0.3})
    Wd = {k: v.double() for k, v in W.items()}
    ids_ref, w_ref = O.route(h.double(), Wd, "r.", {"top": top})
    z = torch.nn.functional.linear(h, W["r.router"]).to(gpu)
    ids, w, row_off, src, row_expert, inv = res32.router(z, W["r.correction"].to(gpu), E, top)
    assert torch.equal(ids.cpu().long().sort(1).values, ids_ref.sort(1).values)
    order = ids.cpu().long().argsort(1), ids_ref.argsort(1)
    assert (torch.gather(w.cpu().double(), 1, order[0]) - torch.gather(w_ref, 1, order[1])).abs().max() < 1e-6
    assert not torch.equal(ids_ref.sort(1).values, torch.topk(torch.softmax(h.double() @ Wd["r.router"].T, -1), top).indices.sort(1).values)
    n_real = int((ids.cpu() < E).sum())
    assert int(row_off[-1]) == n_real and int((inv.cpu() >= 0).sum()) == n_real
    assert sorted(inv.cpu()[inv.cpu() >= 0].tolist()) == list(range(n_real))
    w_gu = torch.stack([torch.cat([W[f"r.e{e}.gate"], W[f"r.e{e}.up"]]) for e in range(E)]).to(gpu)
    w_down = torch.stack([W[f"r.e{e}.down"] for e in range(E)]).to(gpu)
    Y = res32.expert_rows(h.to(gpu), src, row_expert, row_off, w_gu, w_down)
    out = res32.moe_combine(Y, inv, w, h.to(gpu))
    ref = O.moe(h.double(), Wd, "r.", {"router": {"experts": E, "identity": I, "top": top}})
    assert (out.cpu().double() - ref).abs().max() < 2e-5


# ------------------------------------------------------------------ the model through the engine
A = dict(type="attention", heads=4, kv_heads=2, dim=12, every=7, mlp=dict(experts=5, identity=2, top=3, ff=24))
CONFIGS = {
    # delta and attention layers of different sizes; a layer without feed-forward; GQA; conv taps != canon taps
    "mixed": dict(width=40, vocab=250, taps=3, side=5, layers=[
        dict(type="delta", heads=4, kv_heads=2, dim=12, vdim=20, conv=2, mlp=dict(experts=3, identity=2, top=2, ff=24)),
        A, dict(type="attention", heads=2, kv_heads=1, dim=16, every=3, coef=0.9, mlp=None),
        dict(type="delta", heads=2, kv_heads=2, dim=8, vdim=8, conv=4, mlp=dict(experts=4, identity=0, top=1, ff=16))]),
    # odd sizes; one tap (no history); no identity experts anywhere; top = all experts
    "odd": dict(width=34, vocab=131, taps=1, side=3, layers=[
        dict(type="attention", heads=3, kv_heads=3, dim=10, every=4, mlp=dict(experts=2, identity=0, top=2, ff=9)),
        dict(type="delta", heads=3, kv_heads=1, dim=70, vdim=66, conv=1, mlp=None)]),
    # sizes the matrix-core kernels take; delta first and last
    "cores": dict(width=64, vocab=320, taps=4, side=8, layers=[
        dict(type="delta", heads=2, kv_heads=1, dim=64, vdim=64, conv=3, mlp=dict(experts=4, identity=1, top=2, ff=64)),
        dict(type="attention", heads=4, kv_heads=2, dim=64, every=16, mlp=dict(experts=2, identity=2, top=2, ff=32)),
        dict(type="attention", heads=2, kv_heads=2, dim=32, every=9, mlp=None),
        dict(type="delta", heads=4, kv_heads=4, dim=32, vdim=32, conv=4, mlp=None)]),
}


CONFIGS["recurrent"] = dict(width=36, vocab=90, taps=2, side=4, layers=[  # no attention layer: the paged cache is empty
    dict(type="delta", heads=2, kv_heads=1, dim=16, vdim=24, conv=2, mlp=None),
    dict(type="delta", heads=3, kv_heads=3, dim=8, vdim=12, conv=3, mlp=dict(experts=0, identity=3, top=2, ff=8))])
CONFIGS["attentive"] = dict(width=36, vocab=90, taps=5, side=4, layers=[  # no recurrent layer but the convolutions
    dict(type="attention", heads=2, kv_heads=1, dim=16, every=2, mlp=dict(experts=6, identity=1, top=6, ff=8)),
    dict(type="attention", heads=6, kv_heads=3, dim=8, every=50, mlp=None)])
# experts large enough for the grouped matrix-core GEMMs of the full kernel extension (bf16)
CONFIGS["grouped"] = dict(width=512, vocab=300, taps=3, side=16, layers=[
    dict(type="attention", heads=4, kv_heads=2, dim=64, every=16, mlp=dict(experts=4, identity=1, top=2, ff=512))])


def _build(tmp_path, name, dtype, seed=0, **engine_kw):
    from safetensors.torch import save_file

    from llm_weighted_consensus_amd.engine.engine import LLMEngine
    from llm_weighted_consensus_amd.engine.tokenizer import load_tokenizer
    from llm_weighted_consensus_amd.models.registry import load_model

    c = CONFIGS[name]
    cfg = O.make_config(c["width"], c["vocab"], c["layers"], taps=c["taps"], side=c["side"])
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


def _err(got, ref, dtype=torch.float32):
    """fp32: the largest difference.  bf16: the row-wise relative RMS difference that 90 % of the rows stay under,
    times 4 (a routing choice or an argmax that rounding flips changes single rows; that is not what is tested),
    and no row may be off by more than its own size."""
    d, ref = got.cpu().double() - ref, ref.double()
    if dtype == torch.float32:
        return float(d.abs().max())
    rel = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-3)
    assert float(rel.max()) < 1.0
    return 4 * float(rel.flatten().quantile(0.9))


TOL = {torch.float32: 3e-4, torch.bfloat16: 0.5}


def test_grouped_expert_path(gpu, tmp_path):
    """Experts past the size threshold run through the framework's grouped GEMMs (bf16): a prompt portion and
    single tokens against the oracle; identity choices and the rows no expert owns do not disturb them."""
    from llm_weighted_consensus_amd import ops

    assert ops.available()
    cfg, W, model, eng = _build(tmp_path, "grouped", torch.bfloat16)
    assert cfg["width"] * cfg["layers"][0]["mlp"]["expert"]["ff"] >= model.GROUPED_MIN
    toks = _tokens(48, cfg["vocab"], 3)
    ref = O.forward(cfg, W, toks)
    got = [eng.step_tokens([("g", toks[:40], list(range(40)))])]
    for i in range(40, 48):
        got.append(eng.step_tokens([("g", [toks[i]], [0])], ["g"] if i == 47 else []))
    assert _err(torch.cat(got), ref, torch.bfloat16) < TOL[torch.bfloat16]


@pytest.mark.parametrize("name", ["mixed", "odd", "cores", "recurrent", "attentive"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt_and_layers(gpu, tmp_path, name, dtype):
    """A whole prompt in one step: the stream after every layer and the logits against the oracle."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(70, cfg["vocab"], 1)
    layers_ref, seen = [], []
    ref = O.forward(cfg, W, toks, layers_ref)
    model.on_layer = lambda li, x: seen.append(x.detach().cpu().double())
    got = eng.step_tokens([("w", toks, list(range(len(toks))))], ["w"])
    model.on_layer = None
    assert len(seen) == len(layers_ref)
    for a, b in zip(seen, layers_ref):
        assert _err(a, b, dtype) < TOL[dtype] * max(1.0, float(b.abs().max()) / 8)
    assert _err(got, ref, dtype) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("cores", torch.float32), ("odd", torch.float32)])
def test_few_wanted_rows_and_what_they_leave(gpu, tmp_path, name, dtype):
    """Portions of which few logits are wanted run the last layer's feed-forward side on those rows only; the logits
    match, and so do the tokens decoded afterwards from the pages, histories and states those steps left."""
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
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("odd", torch.float32), ("cores", torch.float32),
                                        ("cores", torch.bfloat16)])
def test_decode_token_by_token_and_portions(gpu, tmp_path, name, dtype):
    """The same logits whether a prompt comes whole, token by token from the first token on, or in portions of
    changing sizes (down to two tokens: shorter than the convolutions' histories; cut inside pages)."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(75, cfg["vocab"], 2)
    ref = O.forward(cfg, W, toks)
    rows = []
    for i, t in enumerate(toks):
        rows.append(eng.step_tokens([("d", [t], [0])], ["d"] if i + 1 == len(toks) else []))
    assert _err(torch.cat(rows), ref, dtype) < TOL[dtype]
    for sizes in ([2, 2, 13, 3, 16, 2, 30, 7], [17, 16, 15, 2, 25], [1, 2, 5, 67]):
        assert sum(sizes) == len(toks)
        rows, a = [], 0
        for n in sizes:
            rows.append(eng.step_tokens([("p", toks[a:a + n], list(range(n)))], ["p"] if a + n == len(toks) else []))
            a += n
        assert _err(torch.cat(rows), ref, dtype) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("mixed", torch.bfloat16), ("cores", torch.bfloat16)])
def test_unequal_batches_pages_and_slots_used_again(gpu, tmp_path, name, dtype):
    """Up to four live sequences of unequal lengths, portions beside single tokens, one sitting steps out, in a pool
    so small that pages and state slots are freed and taken again; every position equals the sequence run alone."""
    cfg, W, model, eng = _build(tmp_path, name, dtype, num_blocks=14)
    seqs = {k: _tokens(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate([("a", 70), ("b", 12), ("c", 40), ("d", 33), ("e", 58), ("f", 1)])}
    ref = {k: O.forward(cfg, W, t) for k, t in seqs.items()}
    at = {k: 0 for k in seqs}
    plan = [[("a", 30), ("b", 2)], [("a", 1), ("b", 7), ("c", 17)], [("a", 1), ("c", 1), ("d", 33), ("b", 3)], [("a", 2), ("c", 22)],
            [("a", 36)], [("e", 20), ("f", 1)], [("e", 1)], [("e", 37)]]
    gots, refs, used = [], [], set()
    for step in plan:
        entries, end, spans = [], [], []
        for k, n in step:
            a = at[k]
            entries.append((k, seqs[k][a:a + n], list(range(n))))
            spans.append((k, a, n))
            at[k] = a + n
            if at[k] == len(seqs[k]):
                end.append(k)
        got = eng.step_tokens(entries, end)
        o = 0
        for k, a, n in spans:
            gots.append(got[o:o + n].cpu())
            refs.append(ref[k][a:a + n])
            o += n
        used.add(eng.bm.num_free_state_slots)
    assert all(at[k] == len(seqs[k]) for k in seqs)
    assert _err(torch.cat(gots), torch.cat(refs), dtype) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4 and min(used) == 1
    with pytest.raises(RuntimeError):  # a fifth live sequence: no state slot
        eng.step_tokens([(k, [1, 2], []) for k in "vwxyz"])


def test_temperature_steps_in_prompt_and_decoding(gpu, tmp_path):
    """A one-layer attention model whose temperature steps at every multiple of ``every``: positions just below and
    at each step match the oracle, in a portion and decoded one by one; with the coefficient set to zero in the
    oracle they do not (the temperature matters at those positions)."""
    CONFIGS["temp"] = dict(width=32, vocab=140, taps=2, side=4, layers=[
        dict(type="attention", heads=2, kv_heads=1, dim=16, every=11, coef=1.5, scale=0.9, mlp=None)])
    cfg, W, model, eng = _build(tmp_path, "temp", torch.float32)
    toks = _tokens(50, 140, 4)
    ref = O.forward(cfg, W, toks)
    flat = json.loads(json.dumps(cfg))
    flat["layers"][0]["mixer"]["q_temp"]["coef"] = 0.0
    ref0 = O.forward(flat, W, toks)
    edge = [9, 10, 11, 20, 21, 22, 31, 32, 33, 42, 43, 44]
    assert float((ref[edge] - ref0[edge]).abs().max()) > 0.01 and float((ref[:9] - ref0[:9]).abs().max()) < 1e-9
    got = eng.step_tokens([("t", toks[:25], list(range(25)))])
    assert _err(got, ref[:25]) < TOL[torch.float32]
    for i in range(25, 50):
        got = eng.step_tokens([("t", [toks[i]], [0])], ["t"] if i == 49 else [])
        assert _err(got, ref[[i]]) < TOL[torch.float32]


def test_long_decoding_against_the_recurrence(gpu, tmp_path):
    """220 tokens decoded one by one after a short prompt (pages cross, the delta state runs long): fp32 stays at
    rounding distance from the oracle."""
    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, num_blocks=20, max_model_len=320)
    toks = _tokens(230, cfg["vocab"], 9)
    ref = O.forward(cfg, W, toks)
    got = [eng.step_tokens([("l", toks[:10], list(range(10)))])]
    for i in range(10, 230):
        got.append(eng.step_tokens([("l", [toks[i]], [0])], ["l"] if i == 229 else []))
    assert _err(torch.cat(got), ref) < TOL[torch.float32]


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
    """engine.generate (admission, paged prefill, state slots from the block manager, batched decode steps, the
    fused sampler at temperature 0; with hipGraph replay of the decode step when ``graphs``: its warm-up run must
    not advance the sequences' states) against the oracle's greedy continuation, twice on one engine so that slots
    and pages come back dirty."""
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, use_graphs=graphs, num_blocks=40)
    for seeds in ((21, 22), (23, 24)):
        prompts = [_tokens(23, 250, seeds[0]), _tokens(5, 250, seeds[1])]
        n_new = 40
        out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True))
        for p, o in zip(prompts, out):
            assert len(o[0]) == n_new
            _check_greedy(cfg, W, p, o[0])
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


def test_generation_chunked_prefill_and_forks(gpu, tmp_path):
    """Chunked prefill (prompt portions beside running decodes) and n > 1 (forked sequences: shared prompt pages, the
    prompt's recurrent state copied to every child) give the greedy continuation too."""
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, num_blocks=48, chunked_prefill=8, max_batch=8)
    prompts = [_tokens(37, 250, 31), _tokens(12, 250, 32)]
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True), n=2)
    for p, o in zip(prompts, out):
        assert len(o) == 2 and o[0] == o[1]  # greedy forks of one prompt agree
        _check_greedy(cfg, W, p, o[0])
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 8


def test_preemption_keeps_the_recurrent_state(gpu, tmp_path):
    """A pool too small for both sequences' growth: one is swapped out and back in (its pages and its state slot's
    contents travel through host memory) and still continues greedily."""
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, num_blocks=11, kv_reserve_tokens=8, max_model_len=128)
    prompts = [_tokens(30, 250, 41), _tokens(28, 250, 42)]
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=90, ignore_eos=True))
    assert eng.stats["preemptions"] >= 1
    for p, o in zip(prompts, out):
        _check_greedy(cfg, W, p, o[0])
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


def test_server_worker_factory_builds_the_design(gpu, tmp_path):
    """The server's worker factory (`engine.group.build_engine`) on a model folder of the design: prefix caching is
    switched off for it (a cached head brings no recurrent state), the state pool is there, generation works."""
    from safetensors.torch import save_file

    from llm_weighted_consensus_amd.engine.group import build_engine
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    c = CONFIGS["cores"]
    cfg = O.make_config(c["width"], c["vocab"], c["layers"], taps=c["taps"], side=c["side"])
    W = O.make_weights(cfg, 2)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    eng = build_engine({"model_dir": str(tmp_path), "dtype": "float32", "max_batch": 4, "max_model_len": 128,
                        "kv_fraction": 0.001}, 0)
    assert eng.state is not None and not eng.prefix_caching and eng.bm.num_state_slots == 4
    prompt = _tokens(20, cfg["vocab"], 8)
    out = eng.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    _check_greedy(cfg, W, prompt, out[0][0])


def test_trace_replay_command_line(gpu, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, ``done <step>`` lines and <step>.f32 files out; two sequences
    interleaved (portions beside single tokens, one sitting a step out), pages and slots given back at ``end``."""
    import os
    import subprocess
    import sys

    import numpy as np
    from safetensors.torch import save_file

    c = CONFIGS["mixed"]
    cfg = O.make_config(c["width"], c["vocab"], c["layers"], taps=c["taps"], side=c["side"])
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
    cfg = O.make_config(c["width"], c["vocab"], c["layers"], taps=c["taps"], side=c["side"])
    W = O.make_weights(cfg, 0)
    d = tmp_path / "bad"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    bad = dict(W)
    bad["l1.mix.A_log"] = torch.zeros(5, dtype=torch.bfloat16)
    save_file(bad, str(d / "model.safetensors"))
    with pytest.raises(ValueError):
        load_model(str(d))
    del bad["l0.mix.q.b"]
    bad["l1.mix.A_log"] = W["l1.mix.A_log"]
    save_file(bad, str(d / "model.safetensors"))
    with pytest.raises(KeyError):
        load_model(str(d))
