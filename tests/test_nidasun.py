"""The Nidasun architecture without a GPU: its configuration, the order of runs under a loop, the model's tensors and what a
request keeps, the manager with pages beside several state tensors, and the plain statement's own mechanisms against hand-made
cases."""
import copy
import math

import pytest
import torch

import plain_nidasun as pn
from ginfer_amd import config_from_dict
from ginfer_amd.cache import CacheManager
from ginfer_amd.config import ConfigError
from ginfer_amd.parts import KVCacheSpec, StateSpec
from ginfer_amd.parts.model import build_model
from ginfer_amd.parts.rope import RotaryNeoX


def ATT(heads, kv_heads, dim, vdim, scale, size=None, rot=None, factor=None):
    """Sizes of a softmax attention: rot = (base, dims); size: the chunk's (or, as a left mixer, the window's) length."""
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot is not None:
        m["rot"] = dict(base=rot[0], dims=rot[1])
        if factor is not None:
            m["rot"]["scaling"] = dict(factor=factor)
    if size is not None:
        m["mask"] = dict(size=size)
    return "attention", m


def LIT(heads, dim, vdim, decay):
    return "lightning", dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay))


def PAR(left, width, blocks, conv, left_scale=1.0, right_scale=1.0):
    return "parallel", dict(left=left[1], right=dict(width=width, blocks=blocks, conv=conv), left_scale=left_scale,
                            right_scale=right_scale)


def DENSE(ff):
    return dict(kind="dense", ff=ff)


def MOE(experts, top, ff, scale=1.0, groups=None):
    router = dict(experts=experts, top=top, scale=scale)
    if groups is not None:
        router["groups"] = dict(count=groups[0], keep=groups[1])
    return dict(kind="moe", router=router, expert=dict(ff=ff))


def config(width, vocab, layers, eps=1e-5, streams=None, loop=None):
    """layers: (mixer, mlp) pairs, the mixer from ATT / LIT / PAR."""
    d = dict(architecture="Nidasun", vocab=vocab, width=width, norm=dict(eps=eps),
             layers=[dict(type=m[0], mixer=m[1], mlp=f) for m, f in layers])
    if streams is not None:
        d["streams"] = streams
    if loop is not None:
        d["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return d


CFG = config(48, 101, [
    (ATT(4, 2, 12, 20, 0.3, 10, rot=(5000.0, 8)), DENSE(56)),
    (LIT(3, 8, 12, (0.5, 0.9, 0.99)), MOE(6, 2, 24, scale=1.5, groups=(3, 2))),
    (PAR(ATT(3, 3, 16, 8, 0.2, 7, rot=(100.0, 16), factor=2.0), 40, 5, 3, 0.7, 1.3), None),
    (PAR(ATT(2, 1, 8, 8, 0.5), 24, 1, 1), MOE(3, 3, 16)),
], eps=2e-6, streams=3, loop=(1, 3, 2))


def test_configuration_reads_every_size_and_round_trips():
    cfg = config_from_dict(CFG)
    assert type(cfg).__name__ == "NidasunConfig" and cfg.to_dict() == CFG
    spec = cfg.model_spec()
    assert [l.arrangement for l in spec.layers] == ["hyper_prenorm"] * 4 and spec.stream.params["streams"] == 3
    m0 = spec.layers[0].parts["mixer"]
    assert m0.kind == "conv_attention"
    p = m0.params
    assert (p["num_heads"], p["num_kv_heads"], p["head_dim"], p["value_dim"], p["scale"], p["chunk"], p["sink"], p["bias"]) == \
        (4, 2, 12, 20, 0.3, 10, "learned", True)
    assert p.get("window") is None and p.get("qk_norm_eps") is None and p["taps"] is None
    assert p["position"].params["rotary_dim"] == 8 and p["position"].params["linear_factor"] is None
    m1 = spec.layers[1].parts["mixer"]
    assert m1.kind == "lightning" and m1.params["decay"] == [0.5, 0.9, 0.99] and m1.params["eps"] == 2e-6
    m2 = spec.layers[2].parts["mixer"]
    assert m2.kind == "parallel_sum" and m2.params["scales"] == [0.7, 1.3] and m2.params["names"] == ["left", "right"]
    left, right = m2.params["branches"]
    assert (left.params["window"], left.params["sink"], left.params["bias"], left.params["qk_norm_eps"]) == (7, None, False, 2e-6)
    assert left.params.get("chunk") is None and left.params["position"].params["linear_factor"] == 2.0
    assert right.kind == "rglru" and (right.params["width"], right.params["blocks"], right.params["taps"], right.params["rate"]) == (40, 5, 3, 8.0)
    assert spec.layers[3].parts["mixer"].params["branches"][0].params["position"] is None
    assert "feed_forward" not in spec.layers[2].parts and "feed_forward_link" not in spec.layers[2].parts
    ff = spec.layers[1].parts["feed_forward"].params
    assert (ff["num_experts"], ff["top_k"], ff["expert_size"], ff["groups"], ff["keep_groups"], ff["weight_scale"], ff["scoring"]) == \
        (6, 2, 24, 3, 2, 1.5, "sigmoid")
    assert ff["group_top"] == 2 and ff["weight_floor"] == 1e-20 and ff["correction"] and not ff["router_bias"]
    ff3 = spec.layers[3].parts["feed_forward"].params
    assert (ff3["groups"], ff3["keep_groups"], ff3["weight_scale"]) == (1, 1, 1.0)
    assert spec.layers[0].parts["feed_forward"].kind == "squared_relu" and not spec.head.params["tied"]


def test_the_loop_orders_the_runs():
    assert [e.layer for e in config_from_dict(CFG).model_spec().schedule] == [0, 1, 2, 1, 2, 3] == pn.run_order(CFG)
    c = copy.deepcopy(CFG)
    c.pop("loop")
    assert [e.layer for e in config_from_dict(c).model_spec().schedule] == [0, 1, 2, 3] == pn.run_order(c)
    for loop, want in ((dict(start=0, stop=4, times=1), [0, 1, 2, 3]), (dict(start=3, stop=4, times=3), [0, 1, 2, 3, 3, 3]),
                       (dict(start=0, stop=2, times=2), [0, 1, 0, 1, 2, 3]), (dict(start=2, stop=2, times=5), [0, 1, 2, 3])):
        c["loop"] = loop
        assert [e.layer for e in config_from_dict(c).model_spec().schedule] == want == pn.run_order(c)
    assert all(e.cache_of is None and e.enter == () for e in config_from_dict(CFG).model_spec().schedule)


def test_without_streams_the_block_runs_around_one_plain_stream():
    c = copy.deepcopy(CFG)
    c.pop("streams")
    spec = config_from_dict(c).model_spec()
    assert spec.stream.params["streams"] == 1
    assert all(l.parts["mixer_link"].params == dict(streams=1, learned=False) for l in spec.layers)
    shapes = build_model(spec, torch.float32, None).weight_specs()
    assert not [n for n in shapes if ".hc" in n]


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][0].update(type="lstm"), "unknown mixer type"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "feed-forward kind"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "top"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=14), "dims"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][2]["mixer"]["right"].update(blocks=3), "blocks"),
    (lambda c: c["layers"][2]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c.update(streams=0), "streams"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_configuration_errors_name_the_key(change, word):
    c = copy.deepcopy(CFG)
    change(c)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(c)


def test_tensor_names_shapes_and_caches():
    model = build_model(config_from_dict(CFG).model_spec(), torch.float32, None)
    shapes = {n: tuple(s.shape) for n, s in model.weight_specs().items()}
    assert shapes["embed"] == (101, 48) and shapes["final.norm"] == (48,) and shapes["head"] == (101, 48)
    for i in range(4):
        assert shapes["l%d.norm1" % i] == (48,) and shapes["l%d.hc1.in" % i] == (3,) and shapes["l%d.hc1.mix" % i] == (3, 3)
    assert shapes["l0.hc2.out"] == (3,) and "l2.norm2" not in shapes and "l2.hc2.in" not in shapes
    assert shapes["l0.mix.q"] == (48, 48) and shapes["l0.mix.k"] == (24, 48) and shapes["l0.mix.v"] == (40, 48)
    assert shapes["l0.mix.q.b"] == (48,) and shapes["l0.mix.v.b"] == (40,) and shapes["l0.mix.o"] == (48, 80)
    assert shapes["l0.mix.o.b"] == (48,) and shapes["l0.mix.sink"] == (4,)
    assert shapes["l1.mix.q"] == (24, 48) and shapes["l1.mix.v"] == (36, 48) and shapes["l1.mix.g"] == (36, 48)
    assert shapes["l1.mix.norm"] == (36,) and shapes["l1.mix.o"] == (48, 36)
    assert shapes["l2.mix.left.q"] == (48, 48) and shapes["l2.mix.left.q.norm"] == (48,) and shapes["l2.mix.left.k.norm"] == (48,)
    assert shapes["l2.mix.left.v"] == (24, 48) and shapes["l2.mix.left.o"] == (48, 24)
    assert "l2.mix.left.q.b" not in shapes and "l2.mix.left.sink" not in shapes
    assert shapes["l2.mix.right.y"] == (40, 48) and shapes["l2.mix.right.x.b"] == (40,) and shapes["l2.mix.right.conv"] == (40, 3)
    assert shapes["l2.mix.right.conv.b"] == (40,) and shapes["l2.mix.right.ra"] == (5, 8, 8) and shapes["l2.mix.right.ri.b"] == (5, 8)
    assert shapes["l2.mix.right.lam"] == (40,) and shapes["l2.mix.right.o"] == (48, 40) and shapes["l3.mix.right.conv"] == (24, 1)
    assert shapes["l0.mlp.up"] == (56, 48) and shapes["l0.mlp.down"] == (48, 56)
    assert shapes["l1.mlp.router"] == (6, 48) and shapes["l1.mlp.correction"] == (6,) and "l1.mlp.router.b" not in shapes
    assert shapes["l1.mlp.e5.gate"] == (24, 48) and shapes["l1.mlp.e0.down"] == (48, 24) and "l1.mlp.e6.gate" not in shapes
    specs = model.cache_specs()
    assert len(specs) == 6                              # six runs: the looped layers keep a cache per pass
    none, kv = specs[0]
    assert none is None and isinstance(kv, KVCacheSpec) and (kv.num_kv_heads, kv.head_dim, kv.window) == (2, 32, 10)   # a chunk's length
    assert specs[1] == specs[3] == StateSpec((3, 8, 12), torch.float32)
    none, kv, state, conv = specs[2]
    assert none is None and (kv.num_kv_heads, kv.head_dim, kv.window) == (3, 16, 7)
    assert state == StateSpec((40,), torch.float32) and conv == StateSpec((2, 40), torch.float32)
    assert specs[5][3] is None and specs[5][1].window is None          # one tap: no convolution state; no mask: every key


def test_cache_manager_with_pages_and_state_of_every_run():
    model = build_model(config_from_dict(CFG).model_spec(), torch.float32, None)
    cm = CacheManager(model.cache_specs(), page_size=8, num_pages=6, max_requests=2)
    cm.admit("a")
    cm.append("a", 20)
    cm.commit("a")
    cm.admit("b")
    assert cm.can_append("b", 24) and not cm.can_append("b", 25)
    assert not cm.can_admit()
    cm.release("a")
    assert cm.can_append("b", 48) and cm.can_admit()
    cm.check()
    # the two passes of the windowed layer hold places of their own in one group; the chunked layer's keys are another
    assert cm.group_of[(2, 1)][0] == cm.group_of[(4, 1)][0] and cm.group_of[(2, 1)] != cm.group_of[(4, 1)]
    assert cm.group_of[(0, 1)][0] != cm.group_of[(2, 1)][0]


def test_the_kernels_mask_parameter_sees_what_the_plain_statement_sees():
    """One signed number tells the attention kernels what a token sees; its host twin bounds the key splits."""
    from ginfer_amd.kernels import ops
    assert (ops.mask_parameter(), ops.mask_parameter(window=7), ops.mask_parameter(chunk=7)) == (0, 7, -7)
    with pytest.raises(ops.KernelError):
        ops.mask_parameter(window=3, chunk=3)
    pos = torch.arange(40)
    for kind, size, mask in (("chunk", 1, -1), ("chunk", 7, -7), ("chunk", 64, -64), ("window", 1, 1), ("window", 7, 7), ("all", 0, 0)):
        seen = pn.visible(pos, kind, size)
        for i in range(40):
            first = ops.first_visible_key(i, mask)
            assert seen[i].tolist() == [first <= j <= i for j in range(40)], (kind, size, i)


def test_stretched_frequencies():
    part = RotaryNeoX(theta=100.0, rotary_dim=16, max_positions=32, linear_factor=2.0, device="cpu")
    cos, sin = part.tables()
    f = torch.tensor([100.0 ** (-2.0 * i / 16) / 2.0 for i in range(8)], dtype=torch.float64).to(torch.float32)
    ang = torch.arange(32, dtype=torch.float32)[:, None] * f[None, :]
    assert torch.equal(cos, torch.cos(ang)) and torch.equal(sin, torch.sin(ang))
    with pytest.raises(ValueError):
        RotaryNeoX(theta=100.0, rotary_dim=16, max_positions=32, linear_factor=0.0)


def test_plain_mechanisms_on_hand_made_cases():
    f64 = torch.float64
    # what a token sees: its own chunk up to itself; the last `size` tokens
    pos = torch.arange(7)
    chunk = pn.visible(pos, "chunk", 3)
    assert chunk[5].tolist() == [False, False, False, True, True, True, False] and chunk[3].tolist() == [False] * 3 + [True] + [False] * 3
    window = pn.visible(pos, "window", 3)
    assert window[5].tolist() == [False, False, False, True, True, True, False] and window[3].tolist() == [False, True, True, True, False, False, False]
    assert pn.visible(pos, "all", 0)[6].all()
    # the sink: one key with score 0 and a sink of 0 share the weight
    q = torch.zeros((1, 1, 4), dtype=f64)
    v = torch.tensor([[[3.0, 5.0]]], dtype=f64)
    assert pn.softmax_attention(q, q.clone(), v, 1.0, "all", 0, sink=torch.zeros(1, dtype=f64)).tolist() == [[1.5, 2.5]]
    assert pn.softmax_attention(q, q.clone(), v, 1.0, "all", 0).tolist() == [[3.0, 5.0]]
    # convolution: zeros before the start, the last tap on the token itself, the bias on top
    u = torch.tensor([[1.0], [2.0], [4.0]], dtype=f64)
    w = torch.tensor([[100.0, 10.0, 1.0]], dtype=f64)
    assert pn.causal_convolution(u, w, torch.tensor([0.5], dtype=f64)).flatten().tolist() == [1.5, 12.5, 124.5]
    # rotation: the pair (i, i + dims / 2) turns by the position's angle; the rest passes
    x = torch.tensor([[[1.0, 0.0, 7.0]]], dtype=f64).repeat(2, 1, 1)
    got = pn.turn(x, torch.arange(2), 1.0, 2, factor=2.0)
    assert torch.allclose(got[1, 0], torch.tensor([math.cos(0.5), math.sin(0.5), 7.0], dtype=f64)) and got[0, 0].tolist() == [1.0, 0.0, 7.0]
    # routing: the better group by its two largest choice scores; inside it the largest; weights from the plain scores
    z = torch.tensor([[4.0, -4.0, -4.0, 1.0, 1.1, 0.9]], dtype=f64)            # group 0 holds the single best expert
    w = {"r.router": torch.eye(6, dtype=f64), "r.correction": torch.zeros(6, dtype=f64)}
    ids, weights = pn.route(z, w, "r.", dict(experts=6, top=2, scale=2.0, groups=dict(count=2, keep=1)))
    assert ids == [[4, 3]]                                                     # 0.75 + 0.73 beats 0.98 + 0.02
    s = torch.sigmoid(z[0])
    assert abs(float(weights[0][0]) - float(s[4] / (s[4] + s[3]) * 2.0)) < 1e-12
    w["r.correction"] = torch.tensor([0.0, 0.0, 0.0, 0.0, -5.0, 0.0], dtype=f64)  # the correction moves the choice, not the weight
    ids, weights = pn.route(z, w, "r.", dict(experts=6, top=2, scale=1.0, groups=dict(count=2, keep=2)))
    assert ids == [[0, 3]] and abs(float(sum(weights[0])) - 1.0) < 1e-12
    # the recurrence: one channel, constants that can be followed by hand
    w = {"m.ra": torch.zeros((1, 1, 1), dtype=f64), "m.ra.b": torch.zeros((1, 1), dtype=f64), "m.ri": torch.zeros((1, 1, 1), dtype=f64),
         "m.ri.b": torch.full((1, 1), 50.0, dtype=f64), "m.lam": torch.tensor([math.log(math.e - 1.0)], dtype=f64)}
    a = math.exp(-8.0 * 0.5 * 1.0)                                             # r = 1/2, softplus(lam) = 1, i = 1
    S = pn.gated_linear_recurrence(torch.tensor([[1.0], [1.0]], dtype=f64), w, "m.", 1)
    b = math.sqrt(1 - a * a)
    assert torch.allclose(S.flatten(), torch.tensor([b, a * b + b], dtype=f64))
    # lightning attention: S_1 = k_1 v_1^T, S_2 = d S_1 + k_2 v_2^T
    q = torch.tensor([[[1.0]], [[1.0]]], dtype=f64)
    o = pn.decayed_outer_products(q, q.clone(), torch.tensor([[[2.0]], [[3.0]]], dtype=f64), torch.tensor([0.5], dtype=f64))
    assert o.flatten().tolist() == [2.0, 4.0]
