"""Merudra on the CPU: config parsing, registry, the recurrent-state pool's layout and the block manager's state
slots (the GPU tests cover the kernels and the model)."""
import json

import pytest
import torch

import merudra_oracle as O

LAYERS = [dict(type="delta", heads=4, kv_heads=2, dim=12, vdim=20, conv=2, mlp=dict(experts=3, identity=2, top=2, ff=24)),
          dict(type="attention", heads=4, kv_heads=2, dim=8, every=5, mlp=None)]


def test_config_from_json_and_registry(tmp_path):
    from llm_weighted_consensus_amd.models.config import MerudraConfig, load_model_config
    from llm_weighted_consensus_amd.models.registry import model_class

    cfg = O.make_config(40, 77, LAYERS, taps=3, side=5)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    c = load_model_config(tmp_path)
    assert isinstance(c, MerudraConfig) and c.layers == 2 and c.attention_layers == (1,)
    assert c.canon_taps == 3 and c.side_dim == 5 and c.vocab_size == 77 and c.hidden == 40
    d, a = c.layer_specs[0], c.layer_specs[1]
    assert (d.type, d.mixer.conv, d.mixer.nq, d.mixer.nv, d.mlp.identity, d.mlp.top) == ("delta", 2, 24, 80, 2, 2)
    assert (a.type, a.mixer.temp_every, a.mixer.nq, a.mixer.nk, a.mlp) == ("attention", 5, 32, 16, None)
    assert model_class(c).__name__ == "MerudraModel"
    W = O.make_weights(cfg, 0)
    assert c.params() == sum(t.numel() for t in W.values())
    bad = json.loads(json.dumps(cfg))
    bad["layers"][1]["mixer"]["vdim"] = 9
    with pytest.raises(ValueError):
        MerudraConfig.from_dict(bad)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][0]["type"] = "other"
    with pytest.raises(ValueError):
        MerudraConfig.from_dict(bad)


def test_state_pool_layout_copy_and_swap():
    from llm_weighted_consensus_amd.models.state import RecurrentStatePool

    fields = [("c", (2, 5)), ("S", (3, 4, 6)), ("e", (0, 7))]
    pool = RecurrentStatePool(fields, 4, "cpu")
    assert pool.scratch == 4 and pool["c"].shape == (5, 2, 5) and pool["S"].shape == (5, 3, 4, 6) and pool["e"].shape == (5, 0, 7)
    assert RecurrentStatePool.bytes_per_slot(fields) == 4 * pool.slot_elems
    pool["c"][1] = 1.0
    pool["S"][1] = 2.0
    assert float(pool.pool[0].abs().sum()) == 0 and float(pool.pool[2].abs().sum()) == 0  # views do not overlap slots
    assert float(pool.pool[1].sum()) == 10 + 2 * 72
    pool.copy_slots([(1, 3)])
    assert torch.equal(pool.pool[3], pool.pool[1])
    saved = pool.take([1, 3])
    pool.pool.zero_()
    pool.put([0, 2], saved)
    assert torch.equal(pool["S"][2], torch.full((3, 4, 6), 2.0)) and float(pool.pool[1].abs().sum()) == 0


def test_block_manager_state_slots():
    from llm_weighted_consensus_amd._runtime import BlockManager

    bm = BlockManager(16, 16)
    bm.add_sequence(1, 5)
    assert bm.state_slot(1) == -1  # off by default
    bm.free_sequence(1)
    bm.set_state_slots(3)
    bm.add_sequence(1, 5)
    bm.add_sequence(2, 20)
    assert {bm.state_slot(1), bm.state_slot(2)} == {0, 1} and bm.num_free_state_slots == 1
    bm.fork(1, 3)
    assert bm.state_slot(3) == 2 and bm.take_state_copies() == [(bm.state_slot(1), 2)] and bm.take_state_copies() == []
    with pytest.raises(RuntimeError):
        bm.add_sequence(4, 1)
    assert not bm.has_sequence(4) and bm.num_free == 16 - 1 - 2
    bm.free_sequence(2)
    bm.fork(1, 5, True)  # the last child takes the parent's slot: no copy, no new slot
    assert bm.state_slot(5) == 0 and bm.state_slot(1) == -1 and bm.take_state_copies() == [] and bm.num_free_state_slots == 1
    bm.free_sequence(1)
    assert bm.num_free_state_slots == 1
    blocks, tables, lens = bm.swap_out([3, 5])
    assert bm.num_free_state_slots == 3
    bm.swap_in([3, 5], len(blocks), tables, lens)
    assert bm.num_free_state_slots == 1 and {bm.state_slot(3), bm.state_slot(5)} <= {0, 1, 2}
    with pytest.raises(Exception):
        bm.set_state_slots(2)  # only while no sequence exists
