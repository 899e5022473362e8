"""CPU-side pieces of the Madipel decoder: config parsing, the paged layer cache's layout, the registry, the id
tokenizer and the oracle's own consistency (no GPU)."""
import json

import pytest
import torch

import madipel_oracle as O


def _cfg():
    return O.make_config(48, 300, [dict(heads=4, kv_heads=2, dim=16, vdim=8, window=6, v_mix=False, ff=64),
                                   dict(heads=2, kv_heads=1, dim=8, vdim=24, window=19, v_mix=True, ff=None)],
                         eps=1e-4, residual_mult=0.7, logit_scale=0.3)


def test_config_reads_every_size_and_constant(tmp_path):
    from llm_weighted_consensus_amd.models.config import MadipelConfig, load_model_config
    from llm_weighted_consensus_amd.models.registry import model_class, resolve_config

    (tmp_path / "config.json").write_text(json.dumps(_cfg()))
    cfg = load_model_config(tmp_path)
    assert isinstance(cfg, MadipelConfig) and cfg.layers == 2
    assert (cfg.vocab_size, cfg.hidden, cfg.norm_eps, cfg.residual_mult, cfg.logit_scale) == (300, 48, 1e-4, 0.7, 0.3)
    a, b = cfg.layer_specs
    assert (a.mixer.heads, a.mixer.kv_heads, a.mixer.dim, a.mixer.vdim, a.mixer.window, a.mixer.v_mix, a.ff) == (4, 2, 16, 8, 6, False, 64)
    assert (b.mixer.nq, b.mixer.nk, b.mixer.nv, b.mlp_kind, b.ff, b.mixer.v_mix) == (16, 8, 24, None, 0, True)
    assert a.mixer.scale == pytest.approx(0.25)
    assert (cfg.heads, cfg.kv_heads, cfg.head_dim) == (4, 2, 16)
    assert resolve_config({"model_dir": str(tmp_path)}) == cfg
    assert model_class(cfg).__name__ == "MadipelModel"
    assert resolve_config({"arch": "llama-tiny"}).name == "llama-tiny"
    n = sum(t.numel() for t in O.make_weights(_cfg(), 0).values())
    assert cfg.params() == n


@pytest.mark.parametrize("bad", [{"architecture": "Other"}, {"layers": [{"type": "recurrent", "mixer": {}, "mlp": None}]}])
def test_config_refuses_what_it_does_not_know(tmp_path, bad):
    from llm_weighted_consensus_amd.models.config import load_model_config

    (tmp_path / "config.json").write_text(json.dumps(dict(_cfg(), **bad)))
    with pytest.raises(ValueError):
        load_model_config(tmp_path)


def test_paged_layer_cache_layout_and_block_moves():
    from llm_weighted_consensus_amd.models.cache import PagedLayerCache

    dims = [(32, 16), (8, 24)]
    c = PagedLayerCache(dims, 6, 8, "cpu", torch.float32)
    assert c.block_elems == PagedLayerCache.elems_per_block(dims, 8) == 8 * (32 + 16 + 8 + 24)
    assert c.k[1].shape == (6, 8, 8) and c.v[1].shape == (6, 2, 24, 4)
    g = torch.Generator().manual_seed(0)
    slots = torch.tensor([3, 8, 9, 10, 11, 47])
    for li, (nk, nv) in enumerate(dims):
        k, v = torch.randn(len(slots), nk, generator=g), torch.randn(len(slots), nv, generator=g)
        c.set_rows(li, slots, k, v)
        kk, vv = c.rows(li, slots)
        assert torch.equal(kk, k) and torch.equal(vv, v)
        # four consecutive tokens of one value column are adjacent in memory
        blk, col = 1, 5
        base = c.v[li][blk, 0, col]
        assert base.stride(0) == 1 and torch.equal(base, torch.stack([c.rows(li, torch.tensor([8 + t]))[1][0, col] for t in range(4)]))
    with pytest.raises(ValueError):
        PagedLayerCache(dims, 2, 6, "cpu")
    before = c.pool.clone()
    c.copy_blocks(torch.tensor([[1, 4], [0, 2]], dtype=torch.int32))
    assert torch.equal(c.pool[4], before[1]) and torch.equal(c.pool[2], before[0]) and torch.equal(c.pool[5], before[5])
    out = c.take_blocks(torch.tensor([5, 1]))
    assert c.num_exported(out) == 2 and c.num_exported(torch.empty(0)) == 0
    c.put_blocks(torch.tensor([0, 3]), out)
    assert torch.equal(c.pool[0], before[5]) and torch.equal(c.pool[3], before[1])


def test_id_tokenizer_for_tiny_vocabularies():
    from llm_weighted_consensus_amd.engine.tokenizer import ByteTokenizer, IdTokenizer, IncrementalDecoder, load_tokenizer

    t = load_tokenizer({}, 97)
    assert isinstance(t, IdTokenizer) and (t.bos_token_id, t.eos_token_id) == (95, 96)
    assert all(0 <= i < 95 for i in t.encode("any text at all")) and t.decode([3, 96, 4]) == " w3 w4"
    d = IncrementalDecoder(t)
    assert d.push(7) + d.push(96) == " w7"
    assert isinstance(load_tokenizer({}, 300), ByteTokenizer)


def test_oracle_mechanisms_agree_with_each_other():
    """The oracle's window attention with a window past the sequence and no bias is plain causal softmax attention;
    xIELU is continuous at 0 and its two branches meet in slope; the sinusoid has the stated entries."""
    g = torch.Generator().manual_seed(1)
    n, H, G, D, Dv = 9, 4, 2, 6, 5
    q, k, v = (torch.randn(n, h, d, generator=g, dtype=torch.float64) for h, d in ((H, D), (G, D), (G, Dv)))
    zero, one = torch.zeros(H, dtype=torch.float64), torch.ones(H, dtype=torch.float64)
    out = O.window_attention(q, k, v, H, G, 100, 0.5, one, zero, one).view(n, H, Dv)
    for h in range(H):
        s = (q[:, h] @ k[:, h // 2].T) * 0.5
        s = s.masked_fill(torch.triu(torch.ones(n, n, dtype=torch.bool), 1), float("-inf"))
        assert torch.allclose(out[:, h], torch.softmax(s, -1) @ v[:, h // 2])
    one_key = O.window_attention(q, k, v, H, G, 1, 0.5, one, one, one).view(n, H, Dv)
    assert torch.allclose(one_key[:, 3], v[:, 1])
    z = torch.tensor([-1e-7, 0.0, 1e-7], dtype=torch.float64)
    y = O.xielu(z, 0.3, -0.4)
    assert abs(float(y[1])) == 0 and abs(float(y[2] - y[1]) - float(y[1] - y[0])) < 1e-12
    s = O.sin_positions([0, 3], 6)
    assert torch.allclose(s[0], torch.tensor([0, 1, 0, 1, 0, 1], dtype=torch.float64))
    assert float(s[1, 0]) == pytest.approx(0.1411200080598672) and float(s[1, 1]) == pytest.approx(-0.9899924966004454)
