"""The Nidasun decoder in the engine against its plain statement (plain_nidasun.py), on the GPU: each mechanism alone, then
whole models under every way of cutting and batching, in 32-bit and in bfloat16, at sizes of the tests' own."""
import json
import os

import numpy as np
import pytest
import torch

import helpers as H
import plain_nidasun as pn
from test_nidasun import ATT, LIT, PAR, DENSE, MOE, config

pytestmark = pytest.mark.gpu

# Sizes that differ from one another wherever the design allows it: keys wider and narrower than values and as wide; one kv
# head for all, one per head, groups; the rotation on a part of a head, on all of it and absent, stretched or not; chunks and
# windows of 1 to 70 tokens; 1 to 5 streams and none; 1 to 4 taps; 1 to 5 blocks; groups of experts, none, top = all; loops
# from the first layer, in the middle, once, thrice, absent; layers without a feed-forward; every order of the mixers.
MIX = config(96, 211, [
    (ATT(4, 2, 12, 20, 0.4, 9, rot=(100.0, 8)), DENSE(136)),
    (LIT(3, 8, 12, (0.5, 0.9, 0.995)), MOE(6, 2, 24, scale=1.5, groups=(3, 2))),
    (PAR(ATT(3, 3, 16, 8, 0.3, 11, rot=(50.0, 16), factor=2.0), 40, 5, 3, 0.7, 1.3), None),
    (PAR(ATT(2, 1, 8, 8, 0.5, 5), 24, 1, 1), MOE(3, 3, 16)),
], eps=2e-6, streams=3, loop=(1, 3, 2))
WIDE = config(64, 150, [
    (PAR(ATT(6, 1, 16, 24, 0.25, 33, rot=(1e4, 16), factor=8.0), 72, 3, 4, 1.2, 0.9), MOE(8, 1, 20, scale=2.5, groups=(4, 1))),
    (ATT(5, 5, 20, 12, 0.2, 70, rot=(5e5, 20)), None),
    (LIT(2, 40, 8, (0.97, 1.0)), DENSE(72)),
], eps=1e-5, streams=5)
TINY = config(40, 64, [(ATT(1, 1, 16, 16, 0.5, 1, rot=(50.0, 2)), DENSE(8))], streams=1)
DEEP = config(48, 97, [
    (LIT(4, 4, 4, (0.3, 0.6, 0.9, 0.99)), DENSE(40)),
    (PAR(ATT(8, 4, 8, 12, 0.35, 20), 48, 2, 2, 1.0, 1.0), MOE(12, 4, 8, scale=0.5, groups=(2, 2))),
    (ATT(2, 2, 24, 8, 0.2, rot=(10.0, 24), factor=4.0), None),
    (LIT(1, 32, 48, (0.97,)), None),
], eps=1e-4, loop=(0, 2, 3))
CONFIGS = {"mix": (MIX, 8), "wide": (WIDE, 16), "tiny": (TINY, 16), "deep": (DEEP, 32)}
STD = 5.0


def make_folder(path, cfg, seed, std_scale=STD, edit=None):
    """A model folder with random weights, stored in bfloat16 as this design's checkpoints are (so the 32-bit engine, the
    bfloat16 engine and the plain statement all start from the same numbers); `edit(tensors)` may change them before they
    are written."""
    folder = H.make_model_folder(path, cfg, seed, "bfloat16", std_scale=std_scale)
    from safetensors.torch import load_file, save_file
    file = os.path.join(folder, "model.safetensors")
    tensors = {k: v.clone() for k, v in load_file(file).items()}
    (edit or sharpen)(tensors)
    save_file(tensors, file)
    return folder


def sharpen(tensors, std_scale=STD):
    """What the folder's wider draw would saturate keeps the spread its spec names: the streams' mixing, the router and its
    correction, the recurrence's gates and decay."""
    for name, t in tensors.items():
        if name.endswith((".router", ".correction", ".lam", ".ra.b", ".ri.b", ".sink", ".conv.b", "hc1.mix", "hc2.mix")):
            t /= std_scale


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: make_folder(tmp_path_factory.mktemp(name), cfg, seed=i) for i, (name, (cfg, _)) in enumerate(CONFIGS.items())}


def runner_for(folder, name, dtype, tokens=1024, max_requests=4, **kw):
    from ginfer_amd import ModelRunner
    ps = CONFIGS[name][1]
    return ModelRunner(folder, dtype=dtype, page_size=ps, num_pages=-(-tokens // ps), max_requests=max_requests,
                       max_model_len=2048, **kw)


def requests_for(name, lengths, seed=20):
    return {"q%d" % i: H.random_tokens(n, CONFIGS[name][0]["vocab"], seed + i) for i, n in enumerate(lengths)}


_plain = {}


def plain(folder, ids):
    key = (folder, tuple(ids))
    if key not in _plain:
        _plain[key] = pn.forward(pn.read_config(folder), pn.read_weights(folder), list(ids)).numpy()
    return _plain[key]


def compare(got, requests, folder, tol, what, close_calls=0.0, median=0.5):
    """Every row against the plain statement.  close_calls: the share of rows that may miss the tolerance."""
    over, first, errors = 0, None, []
    for (rid, p), row in sorted(got.items()):
        ref = plain(folder, requests[rid])
        assert np.isfinite(row).all(), "%s: request %s position %d: non-finite logits" % (what, rid, p)
        err = float(np.abs(row.astype(np.float64) - ref[p]).max() / np.abs(ref).max())
        errors.append(err)
        if err > tol:
            over += 1
            first = first or "%s: first wrong place is request %s position %d of %d: error %.3g > %.3g" % (
                what, rid, p, len(requests[rid]), err, tol)
    assert over <= close_calls * len(got), "%s (%d of %d rows)" % (first, over, len(got))
    assert float(np.median(errors)) <= tol * median, "%s: the median row is off by %.3g" % (what, float(np.median(errors)))
    for rid, ids in requests.items():
        missing = [p for p in range(len(ids)) if (rid, p) not in got]
        assert not missing, "%s: request %s lacks logits at %s" % (what, rid, missing[:8])


# 32-bit differs from the 64-bit plain statement by the rounding of sums of a few hundred terms; bfloat16 rounds every stored
# activation to 8 bits, and where two experts' choice scores lie within that rounding the engine may take the other one; the
# rows that see that token through a window or a chunk follow (measured on these models: the same rows miss the tolerance
# when a request runs alone and whole, up to one in eight).  So in bfloat16 the median row must stay within half the
# tolerance and a share of the rows may miss it; a mechanism that is wrong moves nearly every row, and in 32-bit, where no
# row may miss, every cutting and batching must give the whole request's bits.
TOL = {"float32": 1e-4, "bfloat16": 6e-2}
CLOSE = {"float32": 0.0, "bfloat16": 0.2}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


class _Step:
    """The few arrays of a step that the kernels under test read."""

    def __init__(self, q_len, q_start):
        dev = torch.device("cuda")
        cu = np.concatenate([[0], np.cumsum(q_len)]).astype(np.int32)
        self.cu_tokens = torch.tensor(cu, device=dev)
        self.q_start = torch.tensor(q_start, dtype=torch.int32, device=dev)
        self.token_entry = torch.tensor(np.repeat(np.arange(len(q_len)), q_len), dtype=torch.int32, device=dev)
        self.positions = torch.tensor(np.concatenate([np.arange(s, s + n) for s, n in zip(q_start, q_len)]), dtype=torch.int32,
                                      device=dev)
        self.num_entries = len(q_len)
        self.host_q_len, self.host_q_start = list(q_len), list(q_start)
        self.extra = {}

    @property
    def max_q_len(self):
        return max(self.host_q_len)

    @property
    def max_kv_len(self):
        return max(s + n for s, n in zip(self.host_q_start, self.host_q_len))


# ----------------------------------------------------------------------------------------------- mechanisms alone

def test_streams_opened_read_written_and_summed():
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(0)
    for streams, width in ((1, 7), (2, 96), (3, 328), (4, 1000), (8, 4100), (16, 72)):
        x = torch.randn((5, width), generator=g) * 3
        X = ops.hyper_open(x.cuda(), streams)
        assert X.shape == (5, streams, width) and all(torch.equal(X[:, s].cpu(), x) for s in range(streams))
        X = (torch.randn((5, streams, width), generator=g) * 2)
        w_in, w_out = torch.randn((streams,), generator=g), torch.randn((streams,), generator=g)
        mix, nin = torch.randn((streams, streams), generator=g), torch.randn((streams,), generator=g)
        gain, ngain = torch.randn((width,), generator=g), torch.randn((width,), generator=g)
        u = torch.einsum("s,tsw->tw", w_in.double(), X.double())
        for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 1e-2)):
            rows = ops.hyper_read(X.cuda(), w_in.cuda(), gain.cuda(), 3e-6, dtype)
            assert H.rel_err(rows.float().cpu(), pn.rms(u, 3e-6) * gain.double()) < tol
            y = torch.randn((5, width), generator=g).to(dtype)
            want = torch.einsum("sj,tsw->tjw", mix.double(), X.double()) + w_out.double()[None, :, None] * y.double()[:, None, :]
            Xd = X.cuda().clone()
            assert ops.hyper_write(Xd, mix.cuda(), w_out.cuda(), y.cuda()) is None
            assert H.rel_err(Xd.cpu(), want) < 2e-6
            Xn = X.cuda().clone()
            rows = ops.hyper_write(Xn, mix.cuda(), w_out.cuda(), y.cuda(), nin.cuda(), ngain.cuda(), 1e-5, dtype)
            assert torch.equal(Xn, Xd)
            un = torch.einsum("s,tsw->tw", nin.double(), want)
            assert H.rel_err(rows.float().cpu(), pn.rms(un, 1e-5) * ngain.double()) < tol
        parts = torch.randn((3, 5, width), generator=g)
        Xp = X.cuda().clone()
        ops.hyper_write(Xp, mix.cuda(), w_out.cuda(), parts.cuda())
        want = torch.einsum("sj,tsw->tjw", mix.double(), X.double()) + w_out.double()[None, :, None] * parts.double().sum(0)[:, None, :]
        assert H.rel_err(Xp.cpu(), want) < 2e-6
        rows = torch.tensor([4, 0, 0, 2], dtype=torch.int32)
        assert H.rel_err(ops.hyper_sum(X.cuda(), rows.cuda()).cpu(), X.double().sum(1)[rows.long()]) < 2e-6
        assert H.rel_err(ops.hyper_sum(X.cuda()).cpu(), X.double().sum(1)) < 2e-6


def test_routing_by_sigmoid_scores_in_groups():
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    for experts, top, count, keep, scale in ((6, 2, 3, 2, 1.5), (12, 4, 2, 2, 0.5), (8, 1, 4, 1, 2.5), (3, 3, 1, 1, 1.0),
                                              (256, 8, 8, 3, 1.0), (10, 2, 10, 2, 1.0), (7, 3, 1, 1, 3.0)):
        z = torch.randn((40, experts), generator=g) * 1.5
        z[1] = 0.0                                         # equal scores: the lowest indices
        z[2, : experts // 2] = z[2, experts // 2: 2 * (experts // 2)]
        corr = torch.randn((experts,), generator=g) * 0.3
        corr[0] = -3.0                                     # negative choice scores count as they are, not as zero
        w = {"r.router": torch.eye(experts, dtype=torch.float64), "r.correction": corr.double()}
        router = dict(experts=experts, top=top, scale=scale)
        if count > 1:
            router["groups"] = dict(count=count, keep=keep)
        ids_want, w_want = pn.route(z.double(), w, "r.", router)
        ids, weights, dense = ops.route_sigmoid_groups(z.cuda(), top, corr.cuda(), count, keep, 2, True, 1e-20, scale)
        assert ids.cpu().tolist() == ids_want, (experts, top, count, keep)
        assert H.rel_err(weights.cpu(), torch.tensor([[float(x) for x in row] for row in w_want])) < 2e-6
        d = dense.cpu()
        for t in range(40):
            assert torch.count_nonzero(d[t]) == top and torch.equal(d[t][ids[t].long().cpu()], weights[t].cpu())
    z = torch.full((3, 9), float("nan"))
    z[1, 4] = 1.0
    for count in (1, 3):                                   # rows that hold no numbers (the padding of a recorded step) stay inside
        ids, weights, dense = ops.route_sigmoid_groups(z.cuda(), 2, None, count, 1, 2, True, 1e-20, 1.0)
        assert ((ids >= 0) & (ids < 9)).all()
        assert count > 1 or ids[1].cpu().tolist() == [4, 0]


def test_recurrent_block_across_cuts_and_slots():
    """The convolution with its bias, the gates by block and the recurrence: whole against cuts of 1 to 31 tokens, through a
    slot that holds another request's state, beside a second request."""
    from ginfer_amd.parts.model import StateView
    from ginfer_amd.parts.rglru import RecurrentBlock
    g = torch.Generator().manual_seed(2)
    W, T = 56, 61
    cuts = [1, 1, 2, 5, 3, 16, 1, 31, 1]
    for width, blocks, taps in ((40, 5, 3), (24, 1, 1), (64, 2, 4), (300, 3, 2), (1200, 1, 2), (4000, 1, 3)):
        bw = width // blocks
        shapes = {"y": (width, W), "y.b": (width,), "x": (width, W), "x.b": (width,), "conv": (width, taps), "conv.b": (width,),
                  "ra": (blocks, bw, bw), "ra.b": (blocks, bw), "ri": (blocks, bw, bw), "ri.b": (blocks, bw), "lam": (width,),
                  "o": (W, width)}
        w = {n: (torch.randn(s, generator=g) * (0.3 if n in ("y", "x", "o", "ra", "ri") else 0.7)).to(torch.bfloat16) for n, s in shapes.items()}
        x = torch.randn((T, W), generator=g).to(torch.bfloat16)
        other = torch.randn((9, W), generator=g).to(torch.bfloat16)
        ref = pn.recurrent_mixer(x.double(), {"m." + n: t.double() for n, t in w.items()}, "m.", dict(blocks=blocks))
        for dtype, tol in (("float32", 2e-5), ("bfloat16", 3e-2)):
            dt = DT[dtype]
            part = RecurrentBlock(W, width, blocks, taps, dt, "cuda")
            part.bind_weights({n: t.cuda().to(dt) for n, t in w.items()})
            specs = part.cache_spec()
            outs = []
            for c in ([T], cuts):
                states = [None if s is None else torch.full((3,) + tuple(s.shape), 1e4, dtype=torch.float32, device="cuda") for s in specs]
                got, at = [], 0
                for i, n in enumerate(c):
                    slots = torch.tensor([1, 2], dtype=torch.int64, device="cuda")
                    views = [None if s is None else StateView(s, slots, True) for s in states]
                    # a second request's first tokens ride beside: its state lies in another slot
                    rows = torch.cat([x[at:at + n], other[:2 + i % 3]]).cuda().to(dt)
                    out = part.forward(rows, _Step([n, 2 + i % 3], [at, 0]), views)
                    if out.dim() == 3:               # partial sums of a product whose K was split
                        out = out.sum(0)
                    got.append(out[:n].float().cpu())
                    at += n
                outs.append(torch.cat(got))
                assert H.rel_err(outs[-1], ref) < tol, (width, blocks, taps, dtype, c)
            if dtype == "float32":
                assert torch.equal(outs[0], outs[1])


def test_lightning_attention_across_cuts():
    from ginfer_amd.parts.model import StateView
    from ginfer_amd.parts.linear_attention import LightningAttention
    g = torch.Generator().manual_seed(3)
    W, T, eps = 56, 61, 3e-6
    cuts = [1, 1, 2, 5, 3, 16, 1, 31, 1]
    for heads, dim, vdim, decay in ((3, 8, 12, (0.5, 0.9, 0.995)), (1, 40, 8, (1.0,)), (2, 100, 33, (0.97, 0.2))):
        shapes = {"q": (heads * dim, W), "k": (heads * dim, W), "v": (heads * vdim, W), "g": (heads * vdim, W),
                  "o": (W, heads * vdim), "norm": (heads * vdim,)}
        w = {n: (torch.randn(s, generator=g) * (1.0 if n == "norm" else 0.3)).to(torch.bfloat16) for n, s in shapes.items()}
        x = torch.randn((T, W), generator=g).to(torch.bfloat16)
        ref = pn.lightning_mixer(x.double(), {"m." + n: t.double() for n, t in w.items()}, "m.",
                                 dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)), eps)
        for dtype, tol in (("float32", 2e-5), ("bfloat16", 3e-2)):
            dt = DT[dtype]
            part = LightningAttention(W, heads, dim, vdim, decay, eps, dt, "cuda")
            part.bind_weights({n: t.cuda().to(dt) for n, t in w.items()})
            outs = []
            for c in ([T], cuts):
                state = torch.full((3,) + tuple(part.cache_spec().shape), 1e4, dtype=torch.float32, device="cuda")
                got, at = [], 0
                for n in c:
                    sv = StateView(state, torch.tensor([1], dtype=torch.int64, device="cuda"), True)
                    out = part.forward(x[at:at + n].cuda().to(dt), _Step([n], [at]), sv)
                    if out.dim() == 3:
                        out = out.sum(0)
                    got.append(out.float().cpu())
                    at += n
                outs.append(torch.cat(got))
                assert H.rel_err(outs[-1], ref) < tol, (heads, dim, vdim, dtype, c)
            if dtype == "float32":
                assert torch.equal(outs[0], outs[1])


def test_norm_over_the_whole_projection_before_the_rotation():
    """q and k divided by the root mean square of the token's whole projection, times a gain per channel, then turned; values
    as they are; heads padded to the width the attention kernels take."""
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    for nh, nkv, hd, vd, rot in ((3, 3, 16, 8, 16), (6, 1, 12, 20, 8), (2, 2, 40, 40, 0)):
        T, ps, padded = 9, 8, -(-max(hd, vd) // 16) * 16
        C = (nh + nkv) * hd + nkv * vd
        proj = torch.randn((T, C), generator=g) * 2
        gain = torch.randn(((nh + nkv) * hd,), generator=g)
        step = _Step([T], [3])
        cos = sin = None
        if rot:
            f = torch.tensor([77.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64).float()
            ang = torch.arange(32, dtype=torch.float32)[:, None] * f[None, :]
            cos, sin = torch.cos(ang).cuda(), torch.sin(ang).cuda()
        k_pages = torch.zeros((4, nkv, ps, padded), dtype=torch.float32, device="cuda")
        v_pages = torch.zeros((4, nkv, padded, ps), dtype=torch.float32, device="cuda")
        slots = torch.arange(8, 8 + T, dtype=torch.int64, device="cuda")
        q = ops.conv_rope_kv(proj.cuda(), None, None, None, step, cos, sin, slots, k_pages, v_pages, nh, nkv, hd, vd, padded,
                             torch.float32, qk_gain=gain.cuda(), qk_eps=2e-6)
        p = proj.double()
        qn = (pn.rms(p[:, :nh * hd], 2e-6) * gain[:nh * hd].double()).reshape(T, nh, hd)
        kn = (pn.rms(p[:, nh * hd:(nh + nkv) * hd], 2e-6) * gain[nh * hd:].double()).reshape(T, nkv, hd)
        if rot:
            qn, kn = pn.turn(qn, torch.arange(3, 3 + T), 77.0, rot), pn.turn(kn, torch.arange(3, 3 + T), 77.0, rot)
        got_q = q.cpu().reshape(T, nh, padded)
        assert H.rel_err(got_q[:, :, :hd], qn) < 2e-6 and not got_q[:, :, hd:].any()
        for t in range(T):
            page, off = (8 + t) // ps, (8 + t) % ps
            assert H.rel_err(k_pages[page, :, off, :hd].cpu(), kn[t]) < 2e-6
            assert H.rel_err(v_pages[page, :, :vd, off].cpu(), p[t, (nh + nkv) * hd:].reshape(nkv, vd)) < 1e-7


# ----------------------------------------------------------------------------------------------- whole models

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_decoded_and_in_portions(folders, name, dtype):
    """Every request whole; then most of it in one step and the rest token by token; then in portions of 1 to 64 tokens, and
    in pairs.  In 32-bit the four agree to the bit."""
    reqs = requests_for(name, [1, 2, 5, 44, 131])
    runner = runner_for(folders[name], name, dtype)
    got = {}
    for what, steps in (("whole", H.steps_whole(reqs)), ("decoded", H.steps_last_decoded(reqs, last=48)),
                        ("portions", H.steps_portions(reqs)), ("pairs", H.steps_portions(reqs, sizes=(2,)))):
        got[what] = H.run_steps(runner, steps)
        runner.cache.check()
        compare(got[what], reqs, folders[name], TOL[dtype], "%s %s %s" % (name, dtype, what), CLOSE[dtype])
    if dtype == "float32":
        for what in ("decoded", "portions", "pairs"):
            for key, row in got["whole"].items():
                assert np.array_equal(row, got[what][key]), "%s: %s differs from whole at %s" % (name, what, key)
    assert not runner.cache.requests and all(g.pool.num_free == g.pool.num_pages for g in runner.cache.groups)


def test_the_streams_sum_after_every_run(folders):
    name = "mix"
    ids = H.random_tokens(37, CONFIGS[name][0]["vocab"], 5)
    runner = runner_for(folders[name], name, "float32", use_graphs=False)
    seen = []
    for block in runner.model.blocks:
        def wrapped(residual, delta, step, cache, inner=block.forward, **kw):
            out = inner(residual, delta, step, cache, **kw)
            seen.append(residual.sum(dim=1).cpu())
            return out
        block.forward = wrapped
    from ginfer_amd import StepEntry
    runner.step([StepEntry("a", ids, [0])])
    want = []
    pn.forward(pn.read_config(folders[name]), pn.read_weights(folders[name]), ids, want)
    assert len(seen) == len(want) == 6
    for i, s in enumerate(seen):
        assert H.rel_err(s, want[i]) < 1e-5, "after run %d" % i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mix", "wide", "deep"])
def test_unequal_requests_together_with_pages_and_slots_used_again(folders, name, dtype):
    """Seven requests through three state slots and a pool that holds three of them: portions of some beside single tokens
    of others, requests that sit a step out, and every page and slot used several times."""
    reqs = requests_for(name, [70, 3, 120, 33, 64, 17, 90], seed=50)
    steps = H.steps_mixed(reqs, max_live=3, seed=4)
    ps = CONFIGS[name][1]
    tokens = H.max_live_tokens(steps, round_to=ps)
    runner = runner_for(folders[name], name, dtype, tokens=tokens, max_requests=3)
    alone = H.run_steps(runner_for(folders[name], name, dtype), H.steps_whole(reqs)) if dtype == "float32" else None
    for rounds in range(2):                      # the second time the steps' shapes are known and recorded
        got = H.run_steps(runner, steps)
        runner.cache.check()
        compare(got, reqs, folders[name], TOL[dtype], "%s %s mixed, pass %d" % (name, dtype, rounds), CLOSE[dtype])
        if alone is not None:
            for key, row in alone.items():
                assert np.array_equal(row, got[key]), "%s: in a batch, %s differs from the request alone" % (name, key)
    assert not runner.cache.requests


def drawn_config(seed):
    """A configuration drawn at random."""
    rng = np.random.RandomState(seed)
    pick = lambda *xs: xs[rng.randint(len(xs))]
    width = int(pick(24, 40, 50, 52, 64, 66, 96, 136, 75))

    def attention(left):
        heads = int(pick(1, 2, 3, 4, 6))
        kv = int(pick(*[d for d in (1, 2, 3, 4, 6) if heads % d == 0]))
        dim, vdim = int(pick(2, 4, 7, 8, 12, 16, 32, 56, 72)), int(pick(1, 4, 5, 8, 20, 32, 48, 80))
        dims = int(pick(2, 4, dim - dim % 2)) if dim >= 4 else 2
        rot = pick(None, (float(pick(10.0, 1e3, 2.5e5)), min(dims, dim - dim % 2)))
        return ATT(heads, kv, dim, vdim, float(pick(0.1, 0.25, 0.5)), pick(None, 1, 2, 7, 16, 40, 100), rot=rot,
                   factor=pick(None, 1.0, 4.0) if rot else None)
    layers = []
    for _ in range(int(rng.randint(1, 5))):
        ff = pick(None, "dense", "moe")
        if ff == "dense":
            ff = DENSE(int(pick(16, 36, 37, 64, 100)))
        elif ff == "moe":
            count = int(pick(1, 2, 3))
            per = int(pick(1, 2, 4))
            keep = int(rng.randint(1, count + 1))
            ff = MOE(count * per, int(rng.randint(1, keep * per + 1)), int(pick(8, 20, 33)), scale=float(pick(1.0, 2.5)),
                     groups=(count, keep) if count > 1 or rng.rand() < 0.5 else None)
        kind = pick("attention", "lightning", "parallel")
        if kind == "attention":
            layers.append((attention(False), ff))
        elif kind == "lightning":
            heads = int(pick(1, 2, 3, 5))
            layers.append((LIT(heads, int(pick(2, 7, 8, 16, 40)), int(pick(1, 4, 5, 20, 48)),
                               [float(1 - 2.0 ** -rng.randint(1, 9)) for _ in range(heads)]), ff))
        else:
            blocks = int(pick(1, 2, 3, 4))
            layers.append((PAR(attention(True), blocks * int(pick(1, 5, 8, 20)), blocks, int(pick(1, 2, 4, 7)),
                               float(pick(1.0, 0.5, 1.3)), float(pick(1.0, 0.8, 2.0))), ff))
    n = len(layers)
    loop = None
    if rng.rand() < 0.6:
        start = int(rng.randint(0, n))
        loop = (start, int(rng.randint(start, n + 1)), int(rng.randint(1, 4)))
    return config(width, int(pick(50, 128, 301)), layers, eps=float(pick(1e-6, 1e-5, 1e-4)), streams=pick(None, 1, 2, 4, 7), loop=loop)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(tmp_path, seed, dtype):
    cfg = drawn_config(seed)
    folder = make_folder(tmp_path / "m", cfg, seed=seed)
    reqs = {"q%d" % i: H.random_tokens(n, cfg["vocab"], 200 + seed + i) for i, n in enumerate([1, 23, 70])}
    from ginfer_amd import ModelRunner
    page = [8, 16, 32][seed % 3]
    runner = ModelRunner(folder, dtype=dtype, page_size=page, num_pages=-(-256 // page), max_requests=3, max_model_len=512)
    for what, steps in (("whole", H.steps_whole(reqs)), ("decoded", H.steps_last_decoded(reqs, last=20)),
                        ("mixed", H.steps_mixed(reqs, max_live=3, seed=seed))):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        compare(got, reqs, folder, TOL[dtype], "drawn configuration %d (%s) %s %s" % (seed, json.dumps(cfg), dtype, what),
                1.5 * CLOSE[dtype], median=1.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """A short prompt and 400 decoded tokens, recorded steps replayed throughout: windows and chunk borders pass over decoded
    tokens, pages behind the window go back."""
    reqs = requests_for("mix", [420], seed=70)
    runner = runner_for(folders["mix"], "mix", dtype)
    got = H.run_steps(runner, H.steps_last_decoded(reqs, last=400))
    compare(got, reqs, folders["mix"], TOL[dtype], "long decoding " + dtype, CLOSE[dtype])
    if runner.use_graphs:
        assert runner.counts["replayed_decode"] > 300


def _marked(cfg_layer, kind):
    """Edits that make one layer's attention read the tokens themselves: token 7 is the marked key, token 8 (the last) the
    query that matches it; every other score is 0."""
    def edit(t):
        for n in t:
            if n.endswith(("norm1", "norm2")) or n == "final.norm":
                t[n].fill_(1.0)
            if n.endswith(("hc1.mix", "hc2.mix")):
                t[n].copy_(torch.eye(t[n].shape[0]).to(t[n].dtype))
            if n.endswith(("hc1.in", "hc2.in", "hc1.out", "hc2.out")):
                t[n].fill_(0.5)
        e = t["embed"]
        e.copy_((torch.randn(e.shape, generator=torch.Generator().manual_seed(1)) * 0.2).to(e.dtype))
        e[:, :2] = 0
        e[7].zero_()
        e[8].zero_()
        e[7, 1] = 4.0                              # token 7: the marked key (keys read coordinate 1)
        e[8, 0] = 4.0                              # token 8, the last: the query that matches it (queries read coordinate 0)
        p = "l0.mix." + ("left." if kind == "window" else "")
        for n in ("q", "k"):
            t[p + n].zero_()
        dim = cfg_layer["dim"]
        t[p + "q"][0::dim, 0] = 1.0                # coordinate 0 of each head's query
        t[p + "k"][0, 1] = 1.0
        if kind == "window":
            t[p + "q.norm"].fill_(1.0)
            t[p + "k.norm"].fill_(1.0)
        else:
            for n in ("q.b", "k.b"):
                t[p + n].zero_()
            t[p + "sink"].fill_(0.0)
        t[p + "v"] *= 30                           # what the marked token brings is as large as the stream itself
        t[p + "o"] *= 30
    return edit


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_marked_key_at_the_edges_of_a_chunk(tmp_path, dtype):
    """One chunked attention whose keys are the tokens themselves.  The last token's query matches the key of one marked
    token: at its chunk's first place and later it decides the last logits, one place earlier (the chunk before) it must not
    show; whole and decoded, the chunk's border in the prompt and among the decoded tokens."""
    size, T = 24, 260                               # the last token, 259, sees 240 .. 259
    att = ATT(2, 1, 16, 16, 4.0, size)
    cfg = config(32, 40, [(att, None)], streams=2)
    for place, seen in ((0, False), (215, False), (239, False), (240, True), (241, True), (258, True)):
        folder = make_folder(tmp_path / ("m%d" % place), cfg, seed=3, std_scale=1.0, edit=_marked(att[1], "chunk"))
        ids = [int(x) % 6 for x in H.random_tokens(T, 40, place)]
        ids[place] = 7
        ids[-1] = 8
        reqs = {"a": ids}
        runner = runner_for(folder, "wide", dtype, tokens=512)
        for what, steps in (("whole", H.steps_whole(reqs)), ("decoded", H.steps_last_decoded(reqs, last=30)),
                            ("portions", H.steps_portions(reqs, sizes=(7, 2, 33)))):
            got = H.run_steps(runner, steps)
            compare(got, reqs, folder, TOL[dtype], "marked token at %d, %s, %s" % (place, what, dtype))
        moved = list(ids)
        moved[place] = 1
        changed = H.rel_err(plain(folder, moved)[-1], plain(folder, ids)[-1])
        assert (changed > 0.02) == seen, (place, changed)       # the plain statement sees the token, or rightly not


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_marked_key_at_the_edges_of_a_window(tmp_path, dtype):
    """The same with a sliding window beside a recurrent block that is switched off (factor 0): the window's first place and
    the place before it, in prompts and in decoding; pages behind the window have gone back by then."""
    size, T = 40, 300                               # the last token, 299, sees 260 .. 299
    att = ATT(2, 2, 16, 16, 4.0, size)
    cfg = config(32, 40, [(PAR(att, 16, 2, 3, 1.0, 0.0), None)], streams=3)
    for place, seen in ((0, False), (63, False), (259, False), (260, True), (261, True), (298, True)):
        folder = make_folder(tmp_path / ("m%d" % place), cfg, seed=3, std_scale=1.0, edit=_marked(att[1], "window"))
        ids = [int(x) % 6 for x in H.random_tokens(T, 40, place)]
        ids[place] = 7
        ids[-1] = 8
        reqs = {"a": ids}
        runner = runner_for(folder, "wide", dtype, tokens=512)
        for what, steps in (("whole", H.steps_whole(reqs)), ("decoded", H.steps_last_decoded(reqs, last=50)),
                            ("portions", H.steps_portions(reqs, sizes=(7, 2, 33)))):
            got = H.run_steps(runner, steps)
            compare(got, reqs, folder, TOL[dtype], "marked token at %d, %s, %s" % (place, what, dtype))
        moved = list(ids)
        moved[place] = 1
        changed = H.rel_err(plain(folder, moved)[-1], plain(folder, ids)[-1])
        assert (changed > 0.02) == seen, (place, changed)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_decides_the_last_token(tmp_path, dtype):
    """No mask: one marked key among 600, at the first place, at page borders and in the middle, whole and decoded; and a sink
    that takes most of the weight where nothing is marked."""
    T = 600
    att = ATT(2, 1, 16, 16, 4.0)
    cfg = config(32, 40, [(att, DENSE(24))], streams=2)
    for place in (0, 15, 16, 63, 64, 301):
        folder = make_folder(tmp_path / ("m%d" % place), cfg, seed=3, std_scale=1.0, edit=_marked(att[1], "chunk"))
        ids = [int(x) % 6 for x in H.random_tokens(T, 40, place)]
        ids[place] = 7
        ids[-1] = 8
        reqs = {"a": ids}
        runner = runner_for(folder, "wide", dtype, tokens=1024)
        for what, steps in (("whole", H.steps_whole(reqs)), ("decoded", H.steps_last_decoded(reqs, last=30))):
            got = H.run_steps(runner, steps)
            compare(got, reqs, folder, TOL[dtype], "marked token at %d, %s, %s" % (place, what, dtype))
        moved = list(ids)
        moved[place] = 1
        assert H.rel_err(plain(folder, moved)[-1], plain(folder, ids)[-1]) > 0.02


def test_the_sink_takes_its_share(tmp_path):
    """A large sink leaves the attention nearly nothing to add; without it the logits differ: the engine follows both."""
    att = ATT(2, 1, 16, 16, 0.5, 30)
    cfg = config(32, 40, [(att, None)], streams=2)
    reqs = {"a": H.random_tokens(50, 40, 9)}
    rows = []
    for sink in (-20.0, 6.0):
        def edit(t, sink=sink):
            sharpen(t, 1.0)
            t["l0.mix.sink"].fill_(sink)
            t["l0.mix.v"] *= 20
        folder = make_folder(tmp_path / ("s%d" % int(sink)), cfg, seed=5, std_scale=1.0, edit=edit)
        for dtype in ("float32", "bfloat16"):
            got = H.run_steps(runner_for(folder, "wide", dtype), H.steps_last_decoded(reqs, last=5))
            compare(got, reqs, folder, TOL[dtype], "sink %g %s" % (sink, dtype))
        rows.append(plain(folder, reqs["a"])[-1])
    assert H.rel_err(rows[0], rows[1]) > 0.05


LARGER = config(384, 1000, [
    (ATT(12, 4, 128, 64, 0.12, 500, rot=(250000.0, 64)), MOE(16, 2, 96, scale=2.0, groups=(4, 2))),
    (LIT(6, 64, 128, (0.6, 0.9, 0.97, 0.99, 0.995, 0.999)), DENSE(512)),
    (PAR(ATT(6, 6, 48, 80, 0.2, 300, rot=(500.0, 16), factor=4.0), 512, 4, 4, 1.2, 1.1), DENSE(640)),
], eps=1e-6, streams=4, loop=(1, 3, 2))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_at_larger_sizes(tmp_path, dtype):
    """1,300 tokens at once (products of many rows, many chunks and windows), then 30 decoded tokens and a second request in
    portions beside them."""
    folder = make_folder(tmp_path / "m", LARGER, seed=11, std_scale=2.0, edit=lambda t: sharpen(t, 2.0))
    reqs = {"long": H.random_tokens(1330, 1000, 1), "short": H.random_tokens(150, 1000, 2)}
    from ginfer_amd import ModelRunner, StepEntry
    runner = ModelRunner(folder, dtype=dtype, page_size=16, num_pages=-(-1600 // 16), max_requests=4, max_model_len=1600)
    got = {}
    logits = runner.step([StepEntry("long", reqs["long"][:1300], [0, 1, 640, 1299])]).cpu().numpy()
    got.update({("long", p): row for p, row in zip([0, 1, 640, 1299], logits)})
    at = 0
    for k in range(30):
        n = min(7, 150 - at)
        entries = [StepEntry("long", reqs["long"][1300 + k:1301 + k], [0])] + ([StepEntry("short", reqs["short"][at:at + n], [n - 1])] if n else [])
        logits = runner.step(entries).cpu().numpy()
        got[("long", 1300 + k)] = logits[0]
        if n:
            got[("short", at + n - 1)] = logits[1]
            at += n
    runner.cache.check()
    worst = []
    for (rid, p), row in sorted(got.items()):
        ref = plain(folder, reqs[rid])
        worst.append(float(np.abs(row.astype(np.float64) - ref[p]).max() / np.abs(ref).max()))
    assert np.isfinite(worst).all()
    if dtype == "float32":
        assert max(worst) < TOL[dtype], worst
    else:
        assert float(np.median(worst)) < TOL[dtype] / 2 and sum(w > TOL[dtype] for w in worst) <= CLOSE[dtype] * len(worst), worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_steps_equal_launched_ones(folders, dtype):
    reqs = requests_for("mix", [60, 25, 41], seed=80)
    steps = H.steps_mixed(reqs, max_live=3, seed=9)
    outs = []
    for graphs in (True, False):
        runner = runner_for(folders["mix"], "mix", dtype, use_graphs=graphs)
        for rounds in range(3):
            got = H.run_steps(runner, steps)
        outs.append(got)
        if graphs:
            assert runner.use_graphs and runner.counts["replayed_decode"] + runner.counts["replayed_padded"] > 0
    for key, row in outs[0].items():
        if dtype == "float32":
            assert np.array_equal(row, outs[1][key]), key
    if dtype == "bfloat16":
        compare(outs[0], reqs, folders["mix"], TOL[dtype], "recorded", CLOSE[dtype])
        compare(outs[1], reqs, folders["mix"], TOL[dtype], "launched", CLOSE[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(folders, tmp_path, dtype):
    reqs = requests_for("mix", [40, 9, 77], seed=90)
    steps = H.steps_mixed(reqs, max_live=2, seed=2)
    cfg_vocab = CONFIGS["mix"][0]["vocab"]
    import plain_model
    orig = plain_model.read_config
    plain_model.read_config = lambda folder: {"vocab_size": cfg_vocab}          # the helper only asks for the vocabulary
    try:
        got = H.run_trace(folders["mix"], dtype, steps, tmp_path / "out", H.max_live_tokens(steps), page_size=16)
    finally:
        plain_model.read_config = orig
    compare(got, reqs, folders["mix"], TOL[dtype], "trace replay " + dtype, CLOSE[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    """Engine.generate with its scheduler: five prompts through three slots under a budget of 48 tokens a step.  Every token is
    the plain statement's greedy choice after the engine's own tokens so far (in bfloat16: or within rounding of it)."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    name = "mix"
    folder = folders[name]
    prompts = list(requests_for(name, [3, 30, 11, 64, 1], seed=100).values())
    eng = Engine(EngineConfig(model_path=folder, dtype=dtype, max_num_batched_tokens=48, max_num_seqs=3, max_seq_len=256,
                              kvcache_block_size=8, num_kvcache_blocks=96))
    outs = eng.generate(prompts, SamplingParams(max_tokens=24, ignore_eos=True))
    cfg, w = pn.read_config(folder), pn.read_weights(folder)
    far = 0
    for p, o in zip(prompts, outs):
        assert len(o.token_ids) == 24
        logits = pn.forward(cfg, w, (p + o.token_ids)[:-1])
        for k, tok in enumerate(o.token_ids):
            row = logits[len(p) - 1 + k]
            best = int(torch.argmax(row))
            gap = float(row[best] - row[tok]) / float(row.abs().max())
            if dtype == "float32":
                assert tok == best or gap <= 1e-5, "token %d after a prompt of %d: engine %d, plain %d (gap %.3g)" % (k, len(p), tok, best, gap)
            else:
                far += not (tok == best or gap <= 6e-2)
    assert far <= 0.08 * 24 * len(prompts)      # bfloat16: where an expert's choice is a close call, a token and those behind it
    eng.runner.cache.check()


def test_pool_planned_from_the_device_memory(folders):
    """No page counts given: the engine sizes the groups itself (the keys behind a window or inside a chunk, state slots) and
    generates what the plain statement generates."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    folder = folders["mix"]
    eng = Engine(EngineConfig(model_path=folder, dtype="float32", max_num_batched_tokens=64, max_num_seqs=4, max_seq_len=512,
                              kvcache_block_size=8, gpu_memory_utilization=0.05))
    groups = {g.spec: g.pool.num_pages for g in eng.runner.cache.groups}
    assert len(groups) == 3 and all(n >= 1 for n in groups.values())
    for spec, n in groups.items():
        if spec.window is not None:
            assert n == eng.runner.cache.window_pages(spec.window, 8, 4, 64, 512)
    prompts = list(requests_for("mix", [150, 9], seed=300).values())
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    cfg, w = pn.read_config(folder), pn.read_weights(folder)
    for p, o in zip(prompts, outs):
        logits = pn.forward(cfg, w, (p + o.token_ids)[:-1])
        for k, tok in enumerate(o.token_ids):
            row = logits[len(p) - 1 + k]
            assert tok == int(torch.argmax(row)) or float(row.max() - row[tok]) / float(row.abs().max()) <= 1e-5
    eng.runner.cache.check()


def test_command_line_generates(folders):
    import subprocess
    import sys
    folder = folders["deep"]
    cmd = [sys.executable, os.path.join(H.ROOT, "bin", "ginfer"), "generate", "--model-path", folder, "--dtype", "float32",
           "--prompt-ids", "1,2,3,4,5", "--max-tokens", "6", "--ignore-eos", "--max-num-seqs", "2", "--max-seq-len", "64",
           "--num-kvcache-blocks", "16"]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    cfg, w = pn.read_config(folder), pn.read_weights(folder)
    ids = [1, 2, 3, 4, 5]
    for _ in range(6):
        ids.append(int(torch.argmax(pn.forward(cfg, w, ids)[-1])))
    assert json.loads(out.stdout.strip().splitlines()[0])["token_ids"] == ids[5:]
