"""Typed configuration of the Nidasun decoder, read from its own config.json keys.

config.json names the architecture under `architecture` and gives: `vocab`, `width`, `norm.eps`, optionally `streams` (the
number of residual streams of the hyper-connections; absent: one plain residual stream), optionally `loop` ({start, stop,
times}: the layers start .. stop - 1 run `times` times in a row with the same weights, each pass with a cache and state of
its own, and nothing else happens between passes) and `layers`, a list whose entries name the mixer (`type`), its sizes
(`mixer`) and the feed-forward (`mlp`, or null for a layer without one):

  type "attention"   mixer: heads, kv_heads, dim, vdim, scale, optionally rot = {base, dims, optionally scaling = {factor}},
                     optionally mask = {size}: chunks of that many positions
  type "lightning"   mixer: heads, dim, vdim, decay (one per head)
  type "parallel"    mixer: left (as "attention"; its mask.size is a sliding window), right = {width, blocks, conv},
                     left_scale, right_scale
  mlp                {kind: "dense", ff} or {kind: "moe", router: {experts, top, scale, optionally groups = {count, keep}},
                     expert: {ff}}

What the design fixes (no key of config.json): the "attention" mixer has biases, a learned sink per head and chunks; the left
mixer of "parallel" has none of these but a norm over the whole projection of q and of k and a sliding window; lightning
attention reads silu(q), silu(k), silu(v) and gates its normed output with a sigmoid; the recurrence's decay rate 8; the dense
feed-forward squares a relu, the experts gate with silu; the router scores with a sigmoid, a group is scored by its two largest
choice scores, and the chosen weights are divided by their sum + 1e-20.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .registry import register_architecture, ConfigError
from .spec import PartSpec, LayerSpec, ScheduleEntry, ModelSpec
from .potupel import _int, _number

RECURRENCE_RATE = 8.0            # log a = -RECURRENCE_RATE * r * softplus(lam)
GROUP_SCORE_TOP = 2              # a group of experts is scored by this many of its largest choice scores
WEIGHT_FLOOR = 1e-20             # added to the sum of the chosen scores before the division
# positions are counted in 32-bit floats where angles are made; the rotation's tables are as long as the longest sequence
# the engine is set up for, never longer than this
MAX_POSITIONS = 1 << 20
MIXER_TYPES = ("attention", "lightning", "parallel")

# how the checkpoints spell things: layer i is "l<i>", its sublayers' connections to the streams "hc1" and "hc2"
LAYER_TENSOR_NAMES = dict(mixer="mix", feed_forward="mlp", mixer_norm="norm1", feed_forward_norm="norm2",
                          mixer_link="hc1", feed_forward_link="hc2")
MODEL_TENSOR_NAMES = dict(embedding="embed", final_norm="final.norm", head="head")


@dataclass
class NidasunLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


def _read_attention(m, where):
    if not isinstance(m, dict):
        raise ConfigError("config.json: %s has no mixer sizes" % where)
    out = {k: _int(m, k, where + " mixer") for k in ("heads", "kv_heads", "dim", "vdim")}
    if out["heads"] % out["kv_heads"]:
        raise ConfigError("config.json: %s: heads %d is not a multiple of kv_heads %d" % (where, out["heads"], out["kv_heads"]))
    out["scale"] = _number(m, "scale", where + " mixer")
    rot = m.get("rot")
    if rot is not None:
        r = dict(base=_number(rot, "base", where + " rot", positive=True), dims=_int(rot, "dims", where + " rot", minimum=2))
        if r["dims"] % 2 or r["dims"] > out["dim"]:
            raise ConfigError("config.json: %s rot 'dims' must be even and at most dim %d, got %d" % (where, out["dim"], r["dims"]))
        sc = rot.get("scaling")
        r["factor"] = None if sc is None else _number(sc, "factor", where + " rot scaling", positive=True)
        rot = r
    out["rot"] = rot
    mask = m.get("mask")
    out["mask"] = None if mask is None else _int(mask, "size", where + " mask")
    return out


def _read_mixer(kind, m, where):
    if kind == "attention":
        return _read_attention(m, where)
    if not isinstance(m, dict):
        raise ConfigError("config.json: %s has no mixer sizes" % where)
    if kind == "lightning":
        out = {k: _int(m, k, where + " mixer") for k in ("heads", "dim", "vdim")}
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != out["heads"] or \
                any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError("config.json: %s mixer 'decay' must list one number per head (%d), got %r" % (where, out["heads"], decay))
        out["decay"] = [float(d) for d in decay]
        return out
    right = m.get("right")
    if not isinstance(right, dict):
        raise ConfigError("config.json: %s has no right mixer" % where)
    r = dict(width=_int(right, "width", where + " right"), blocks=_int(right, "blocks", where + " right"),
             conv=_int(right, "conv", where + " right"))
    if r["width"] % r["blocks"]:
        raise ConfigError("config.json: %s right: width %d is not a multiple of blocks %d" % (where, r["width"], r["blocks"]))
    return dict(left=_read_attention(m.get("left"), where + " left"), right=r,
                left_scale=_number(m, "left_scale", where + " mixer"), right_scale=_number(m, "right_scale", where + " mixer"))


def _read_mlp(mlp, where):
    if mlp is None:
        return None
    kind = mlp.get("kind") if isinstance(mlp, dict) else None
    if kind == "dense":
        return dict(kind="dense", ff=_int(mlp, "ff", where + " mlp"))
    if kind == "moe":
        router = mlp.get("router")
        r = dict(experts=_int(router, "experts", where + " mlp router"), top=_int(router, "top", where + " mlp router"),
                 scale=_number(router, "scale", where + " mlp router") if "scale" in router else 1.0)
        groups = router.get("groups")
        r["groups"] = None if groups is None else dict(count=_int(groups, "count", where + " mlp router groups"),
                                                       keep=_int(groups, "keep", where + " mlp router groups"))
        count, keep = (r["groups"]["count"], r["groups"]["keep"]) if r["groups"] else (1, 1)
        if r["experts"] % count or keep > count or r["top"] > keep * (r["experts"] // count):
            raise ConfigError("config.json: %s mlp router: %d experts in %d groups of which %d are kept cannot give top %d"
                              % (where, r["experts"], count, keep, r["top"]))
        return dict(kind="moe", router=r, expert=dict(ff=_int(mlp.get("expert"), "ff", where + " mlp expert")))
    raise ConfigError("config.json: %s has the unknown feed-forward kind %r (known: dense, moe)" % (where, kind))


@register_architecture("Nidasun", "nidasun")
@dataclass
class NidasunConfig:
    vocab: int
    width: int
    eps: float
    layers: List[NidasunLayer] = field(default_factory=list)
    streams: Optional[int] = None
    loop: Optional[Dict[str, int]] = None
    eos_token_ids: List[int] = field(default_factory=list)

    architecture = "Nidasun"

    @classmethod
    def from_dict(cls, d):
        missing = [k for k in ("vocab", "width", "norm", "layers") if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): %s" % ", ".join(missing))
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, l in enumerate(d["layers"]):
            where = "layer %d" % i
            kind = l.get("type") if isinstance(l, dict) else l
            if kind not in MIXER_TYPES:
                raise ConfigError("config.json: %s has the unknown mixer type %r (known: %s)" % (where, kind, ", ".join(MIXER_TYPES)))
            layers.append(NidasunLayer(kind, _read_mixer(kind, l.get("mixer"), where), _read_mlp(l.get("mlp"), where)))
        loop = d.get("loop")
        if loop is not None:
            loop = dict(start=_int(loop, "start", "loop", minimum=0), stop=_int(loop, "stop", "loop", minimum=0),
                        times=_int(loop, "times", "loop", minimum=0))
            if not loop["start"] <= loop["stop"] <= len(layers):
                raise ConfigError("config.json: loop needs 0 <= start <= stop <= %d layers, got %d .. %d"
                                  % (len(layers), loop["start"], loop["stop"]))
        eos = d.get("eos_token_id")
        eos = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, (list, tuple)) else [int(eos)])
        return cls(vocab=_int(d, "vocab", ""), width=_int(d, "width", ""), eps=_number(d["norm"], "eps", "norm", positive=True),
                   layers=layers, streams=None if d.get("streams") is None else _int(d, "streams", ""), loop=loop,
                   eos_token_ids=eos)

    def to_dict(self):
        def attention(m):
            out = {k: m[k] for k in ("heads", "kv_heads", "dim", "vdim", "scale")}
            if m["rot"] is not None:
                out["rot"] = dict(base=m["rot"]["base"], dims=m["rot"]["dims"])
                if m["rot"]["factor"] is not None:
                    out["rot"]["scaling"] = dict(factor=m["rot"]["factor"])
            if m["mask"] is not None:
                out["mask"] = dict(size=m["mask"])
            return out

        def mixer(l):
            if l.type == "attention":
                return attention(l.mixer)
            if l.type == "lightning":
                return dict(l.mixer)
            return dict(left=attention(l.mixer["left"]), right=dict(l.mixer["right"]), left_scale=l.mixer["left_scale"],
                        right_scale=l.mixer["right_scale"])

        def mlp(f):
            if f is None or f["kind"] == "dense":
                return None if f is None else dict(f)
            router = dict(experts=f["router"]["experts"], top=f["router"]["top"], scale=f["router"]["scale"])
            if f["router"]["groups"] is not None:
                router["groups"] = dict(f["router"]["groups"])
            return dict(kind="moe", router=router, expert=dict(f["expert"]))
        d = dict(architecture=self.architecture, vocab=self.vocab, width=self.width, norm=dict(eps=self.eps),
                 layers=[dict(type=l.type, mixer=mixer(l), mlp=mlp(l.mlp)) for l in self.layers])
        if self.streams is not None:
            d["streams"] = self.streams
        if self.loop is not None:
            d["loop"] = dict(self.loop)
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    def run_order(self):
        """The layers in the order they run (a looped layer once per pass)."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        return (list(range(self.loop["start"])) + list(range(self.loop["start"], self.loop["stop"])) * self.loop["times"]
                + list(range(self.loop["stop"], n)))

    def _attention(self, m, left):
        """The softmax attention of a layer: the "attention" mixer (biases, learned sink, chunks) or the left mixer of a
        "parallel" one (a norm over the whole projection of q and k, a sliding window)."""
        position = None
        if m["rot"] is not None:
            position = PartSpec("rope_neox", dict(theta=m["rot"]["base"], rotary_dim=m["rot"]["dims"], max_positions=MAX_POSITIONS,
                                                  wide_frequencies=True, linear_factor=m["rot"]["factor"]))
        params = dict(hidden_size=self.width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"],
                      value_dim=m["vdim"], scale=m["scale"], taps=None, position=position)
        if left:
            params.update(sink=None, window=m["mask"], bias=False, qk_norm_eps=self.eps)
        else:
            params.update(sink="learned", chunk=m["mask"], bias=True)
        return PartSpec("conv_attention", params)

    def _mixer(self, l):
        m = l.mixer
        if l.type == "attention":
            return self._attention(m, left=False)
        if l.type == "lightning":
            return PartSpec("lightning", dict(hidden_size=self.width, num_heads=m["heads"], key_dim=m["dim"], value_dim=m["vdim"],
                                              decay=list(m["decay"]), eps=self.eps))
        right = PartSpec("rglru", dict(hidden_size=self.width, width=m["right"]["width"], blocks=m["right"]["blocks"],
                                       taps=m["right"]["conv"], rate=RECURRENCE_RATE))
        return PartSpec("parallel_sum", dict(branches=[self._attention(m["left"], left=True), right], names=["left", "right"],
                                             scales=[m["left_scale"], m["right_scale"]]))

    def _feed_forward(self, f):
        if f["kind"] == "dense":
            return PartSpec("squared_relu", dict(hidden_size=self.width, intermediate_size=f["ff"]))
        r = f["router"]
        groups = r["groups"] or dict(count=1, keep=1)
        return PartSpec("routed_glu", dict(
            hidden_size=self.width, num_experts=r["experts"], top_k=r["top"], expert_size=f["expert"]["ff"], shared_size=None,
            router_bias=False, scoring="sigmoid", correction=True, groups=groups["count"], keep_groups=groups["keep"],
            group_top=GROUP_SCORE_TOP, weight_scale=r["scale"], weight_floor=WEIGHT_FLOOR))

    def model_spec(self):
        W, S = self.width, self.streams

        def norm():
            return PartSpec("rmsnorm", dict(size=W, eps=self.eps, weight_name=""))
        layers = []
        for i, l in enumerate(self.layers):
            parts = dict(mixer=self._mixer(l), mixer_norm=norm())
            if l.mlp is not None:
                parts.update(feed_forward=self._feed_forward(l.mlp), feed_forward_norm=norm())
            # without `streams` the same block runs around one stream with every weight 1: the plain residual sum
            link = PartSpec("hyper_connection", dict(streams=S or 1, learned=S is not None))
            parts["mixer_link"] = link
            if l.mlp is not None:
                parts["feed_forward_link"] = link
            layers.append(LayerSpec(prefix="l%d" % i, parts=parts, arrangement="hyper_prenorm", names=dict(LAYER_TENSOR_NAMES)))
        spec = ModelSpec(
            hidden_size=W, vocab_size=self.vocab, layers=layers, schedule=[ScheduleEntry(i) for i in self.run_order()],
            embedding=PartSpec("embedding", dict(vocab_size=self.vocab, hidden_size=W, weight_name="")),
            final_norm=norm(),
            head=PartSpec("lm_head", dict(vocab_size=self.vocab, hidden_size=W, tied=False, weight_name="")),
            max_positions=MAX_POSITIONS, eos_token_ids=list(self.eos_token_ids), names=dict(MODEL_TENSOR_NAMES),
            stream=PartSpec("hyper_streams", dict(streams=S or 1)))
        spec.validate()
        return spec
