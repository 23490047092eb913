"""The Puguzen decoder without a GPU: configuration, tensor names, what a request keeps, the cache manager with rows that
stand for blocks of positions, and the plain statement's mechanisms on hand-made cases."""
import json
import math

import numpy as np
import pytest
import torch

import plain_puguzen as pp
from ginfer_amd import config_from_dict
from ginfer_amd.cache import CacheManager
from ginfer_amd.config import ConfigError
from ginfer_amd.parts.base import PagedSpec, StateSpec
from ginfer_amd.parts.model import build_model


def GLA(heads, dim, vdim, tau, rank=None):
    m = dict(heads=heads, dim=dim, vdim=vdim, tau=tau)
    if rank is not None:
        m["rank"] = rank
    return "gla", m


def RET(heads, dim, vdim, decay, rot=None):
    m = dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay))
    if rot is not None:
        m["rot"] = dict(base=rot[0], dims=rot[1])
    return "retention", m


def ATT(heads, kv_heads, dim, vdim, scale, size, pool, rot=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, mask=dict(size=size, pool=pool))
    if rot is not None:
        m["rot"] = dict(base=rot[0], dims=rot[1])
    return "attention", m


def config(width, vocab, layers, eps=1e-6):
    return dict(architecture="Puguzen", vocab=vocab, width=width, norm=dict(eps=eps),
                layers=[dict(type=t, mixer=m, mlp=None if ff is None else dict(kind="dense", ff=ff)) for (t, m), ff in layers])


SMALL = config(48, 90, [
    (GLA(3, 8, 12, 4.0, rank=5), 40),
    (ATT(4, 2, 12, 20, 0.4, 9, 4, rot=(100.0, 8)), None),
    (RET(2, 16, 8, (0.9, 0.99), rot=(50.0, 6)), 24),
    (ATT(3, 3, 8, 8, 0.3, 5, 7), 16),
], eps=2e-6)


def test_configuration_round_trip_and_names():
    cfg = config_from_dict(SMALL)
    assert json.loads(json.dumps(cfg.to_dict())) == cfg.to_dict()
    again = config_from_dict(cfg.to_dict())
    assert again.to_dict() == cfg.to_dict()
    model = build_model(cfg.model_spec(), torch.float32, None)
    specs = model.weight_specs()
    assert tuple(specs["embed"].shape) == (90, 48) and tuple(specs["final.norm"].shape) == (48,)
    assert tuple(specs["l0.mix.a1"].shape) == (5, 48) and tuple(specs["l0.mix.a2"].shape) == (24, 5)
    assert tuple(specs["l0.mix.a2.b"].shape) == (24,) and tuple(specs["l0.mix.norm"].shape) == (12,)
    assert tuple(specs["l0.mix.g"].shape) == (36, 48) and tuple(specs["l0.mix.o"].shape) == (48, 36)
    assert tuple(specs["l1.mix.q"].shape) == (48, 48) and tuple(specs["l1.mix.k"].shape) == (24, 48)
    assert tuple(specs["l1.mix.v"].shape) == (40, 48) and tuple(specs["l1.mix.pb"].shape) == (4,)
    assert tuple(specs["l1.mix.g"].shape) == (80, 48) and tuple(specs["l1.mix.o"].shape) == (48, 80)
    assert tuple(specs["l2.mix.q"].shape) == (32, 48) and "l2.mix.norm" not in specs and "l2.mix.a1" not in specs
    for i in range(4):
        assert tuple(specs["l%d.norm1" % i].shape) == (48,)
        assert tuple(specs["l%d.rg1" % i].shape) == (48, 48) and tuple(specs["l%d.rg1.b" % i].shape) == (48,)
    # a layer without a feed-forward has neither its tensors nor its gate
    assert "l1.rg2" not in specs and "l1.mlp.gate" not in specs
    assert tuple(specs["l0.rg2"].shape) == (48, 48) and tuple(specs["l0.mlp.gate"].shape) == (40, 48)
    assert tuple(specs["l0.mlp.down"].shape) == (48, 40)
    assert not any(n.startswith("head") for n in specs)          # the head is the embedding table
    assert model.capturable()


def test_what_a_request_keeps():
    model = build_model(config_from_dict(SMALL).model_spec(), torch.bfloat16, None)
    gla, att, ret, att2 = model.cache_specs()
    assert gla == StateSpec((3, 8, 12), torch.float32) and ret == StateSpec((2, 16, 8), torch.float32)
    near, means = att
    assert near == PagedSpec((("k", 24), ("v", 40)), window=9) and means == PagedSpec((("k", 24), ("v", 40)), every=4, dtype=torch.float32)
    # blocks longer than the window: the tokens stay until their block's mean is made
    assert att2[0].window == 7 and att2[1].every == 7


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="mamba"), "unknown mixer type"),
    (lambda c: c["layers"][0]["mixer"].pop("tau"), "'tau'"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5]), "one number per head"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "not a multiple"),
    (lambda c: c["layers"][1]["mixer"]["mask"].pop("pool"), "'pool'"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=14), "at most dim"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=5), "even"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "unknown feed-forward"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.update(layers=[]), "at least one layer"),
])
def test_configuration_errors(change, message):
    c = json.loads(json.dumps(SMALL))
    change(c)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(c)


def test_rank_of_the_decay_projection_comes_from_the_checkpoint(tmp_path):
    from ginfer_amd import write_random_model, config_from_folder
    folder = write_random_model(str(tmp_path / "m"), config_from_dict(SMALL), 3, "bfloat16")
    d = json.load(open(tmp_path / "m" / "config.json"))
    del d["layers"][0]["mixer"]["rank"]                # as this design's checkpoints come: the tensor's shape says it
    json.dump(d, open(tmp_path / "m" / "config.json", "w"))
    assert config_from_dict(d).layers[0].mixer["rank"] is None
    assert config_from_folder(folder).layers[0].mixer["rank"] == 5


def test_manager_with_rows_that_stand_for_blocks_of_positions():
    """A windowed group of tokens beside a group with a row per 4 positions and state: pages follow the tokens, rows of
    blocks are never given back while the request runs, and everything returns at the end."""
    near = PagedSpec((("k", 8), ("v", 8)), window=9)
    means = PagedSpec((("k", 8), ("v", 8)), every=4, dtype=torch.float32)
    m = CacheManager([StateSpec((2, 2)), [near, means]], page_size=4, num_pages=[16, 6], max_requests=2)
    gi_near, gi_means = m.group_of[(1, 0)][0], m.group_of[(1, 1)][0]
    assert m.groups[gi_means].every == 4 and m.groups[gi_near].every == 1
    m.admit("a")
    m.append("a", 21)
    m.commit("a")
    m.check()
    # 21 tokens: 6 rows of blocks -> 2 pages; the window of 9 before token 21 starts at 13: the pages of 12.. stay
    assert len([p for p in m.table("a", gi_means) if p >= 0]) == 2
    assert [p >= 0 for p in m.table("a", gi_near)] == [False, False, False, True, True, True]
    for _ in range(30):                                # decoding: one token at a time, also over page and block borders
        m.append("a", 1)
        m.commit("a")
        m.check()
    assert m.length("a") == 51
    assert len([p for p in m.table("a", gi_means) if p >= 0]) == 4          # 13 rows
    assert sum(p >= 0 for p in m.table("a", gi_near)) <= 4
    free_before = m.groups[gi_means].pool.num_free
    assert m.free_tokens("a") == min((4 + free_before) * 16 - 51, m.free_tokens("a"))
    m.admit("b")
    m.append("b", 30)                                  # 8 rows -> 2 pages: the pool of 6 is full now
    m.commit("b")
    assert m.groups[gi_means].pool.num_free == 0
    assert m.pages_short("a", 14) > 0 and m.pages_short("a", 13) == 0       # 64 positions fit 4 pages of 4 rows of 4
    m.release("a")
    m.check()
    assert m.groups[gi_means].pool.num_free == 4
    m.release("b")
    m.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups)


def test_pool_planned_for_a_group_of_rows_per_block():
    """From a number of bytes: the windowed group gets what a window can hold, the group of rows per block of 4 positions a
    quarter of the pages a group of tokens would get for the same tokens (and one page more per request), at 4 bytes an
    element whatever the model's format."""
    near = PagedSpec((("k", 8), ("v", 8)), window=9)
    means = PagedSpec((("k", 8), ("v", 8)), every=4, dtype=torch.float32)
    full = PagedSpec((("c", 16),))
    specs = [StateSpec((2, 2)), [near, means], full]
    counts = CacheManager.plan_pages(specs, 4, 2, 1 << 20, max_requests=3, max_step_tokens=64, max_model_len=512)
    by = dict(zip(CacheManager.group_specs(specs), counts))
    assert by[near] == CacheManager.window_pages(9, 4, 3, 64, 512)
    assert by[means] == by[full] // 4 + 3 + 1
    used = by[near] * 16 * 4 * 2 + by[means] * 16 * 4 * 4 + by[full] * 16 * 4 * 2
    assert 0.9 * (1 << 20) < used <= (1 << 20)
    m = CacheManager(specs, 4, counts, 3)
    assert m.pool_bytes(2) == used


def test_what_a_token_sees():
    # window of 5, blocks of 3: token 9 sees tokens 5..9 and the block 0..2 (ends at 2 <= 4); block 3..5 ends at 5 > 4
    assert pp.visible(9, 20, 5, 3) == ([0], [5, 6, 7, 8, 9])
    assert pp.visible(10, 20, 5, 3) == ([0, 1], [6, 7, 8, 9, 10])           # 5 <= 10 - 5
    assert pp.visible(3, 20, 5, 3) == ([], [0, 1, 2, 3])
    # tokens 3 and 4 at token 9: behind the window, their block not yet seen -> not seen at all
    blocks, tokens = pp.visible(9, 20, 5, 3)
    assert 3 not in tokens and 4 not in tokens and 1 not in blocks
    # blocks longer than the window
    assert pp.visible(8, 20, 2, 7) == ([0], [7, 8]) and pp.visible(7, 20, 2, 7) == ([], [6, 7])


def test_plain_recurrence_and_rotations_by_hand():
    q = torch.ones((3, 1, 2), dtype=torch.float64)
    k = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]], [[1.0, 1.0]]], dtype=torch.float64)
    v = torch.tensor([[[2.0]], [[3.0]], [[5.0]]], dtype=torch.float64)
    decay = torch.tensor([0.5, 0.25], dtype=torch.float64).expand(3, 1, 2)
    o = pp.decayed_outer_recurrence(q, k, v, decay)
    # S after t0: [2, 0]; t1: [1, 3]; t2: [0.5 + 5, 0.75 + 5]
    assert o.flatten().tolist() == [2.0, 4.0, 11.25]
    u = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 9.0]]], dtype=torch.float64).repeat(2, 1, 1)
    rot = dict(base=1.0, dims=4)                       # every angle is the position itself
    h = pp.turn_halves(u, rot)
    n = pp.turn_neighbours(u, rot)
    assert torch.equal(h[0], u[0]) and torch.equal(n[0], u[0])              # position 0
    c, s = math.cos(1.0), math.sin(1.0)
    assert np.allclose(h[1, 0].tolist(), [1 * c - 3 * s, 2 * c - 4 * s, 3 * c + 1 * s, 4 * c + 2 * s, 9.0])
    assert np.allclose(n[1, 0].tolist(), [1 * c - 2 * s, 2 * c + 1 * s, 3 * c - 4 * s, 4 * c + 3 * s, 9.0])


def test_plain_attention_by_hand():
    # one head, keys and values of one number: weights sigmoid(q k), values summed without a denominator
    q = torch.ones((6, 1, 1), dtype=torch.float64)
    k = torch.tensor([0.0, 1.0, 2.0, 3.0, 4.0, 5.0], dtype=torch.float64).view(6, 1, 1)
    v = torch.tensor([1.0, 10.0, 100.0, 1e3, 1e4, 1e5], dtype=torch.float64).view(6, 1, 1)
    out = pp.sigmoid_attention(q, k, v, torch.zeros(1, dtype=torch.float64), 1.0, 2, 2).flatten()
    sig = lambda z: 1.0 / (1.0 + math.exp(-z))
    assert math.isclose(out[0], sig(0) * 1) and math.isclose(out[1], sig(0) * 1 + sig(1) * 10)
    assert math.isclose(out[2], sig(1) * 10 + sig(2) * 100)                  # token 0 is gone, its block ends at 1 > 0
    assert math.isclose(out[3], sig(0.5) * 5.5 + sig(2) * 100 + sig(3) * 1e3)       # block 0 (mean key 0.5, mean value 5.5)
    assert math.isclose(out[5], sig(0.5) * 5.5 + sig(2.5) * 550 + sig(4) * 1e4 + sig(5) * 1e5)
