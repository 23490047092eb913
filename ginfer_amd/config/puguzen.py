"""Typed configuration of the Puguzen decoder, read from its own config.json keys.

config.json names the architecture under `architecture` and gives `vocab`, `width`, `norm.eps` and `layers`, a list whose
entries name the mixer (`type`: "gla", "retention" or "attention"), the mixer's sizes (`mixer`) and the feed-forward (`mlp`:
{kind: "dense", ff}, or null for a layer without one):
  gla        heads, dim, vdim, tau (the decay is sigmoid(.)^(1 / tau)); the rank of the decay's narrow projection is the shape
             of the tensor `a1`, which the configuration reads from the checkpoint's header or is told (`rank`)
  retention  heads, dim, vdim, decay (one constant per head), optionally rot = {base, dims}
  attention  heads, kv_heads, dim, vdim, scale, mask = {size, pool}, optionally rot = {base, dims}
Layers may differ from one another in kind and in every size.

What the design fixes (no key of config.json): gains of norms are stored around zero (g = 1 + stored); the head is the
embedding table; a layer has one norm, its sublayers run side by side and each passes a gate sigmoid(R n + r); the
feed-forward is relu(gate) * up; gla scales q and retention scales k by 1 / sqrt(dim); retention pairs the coordinates
(i, i + dims / 2), the attention (2i, 2i + 1); the attention norms q and k per head, weighs keys by a sigmoid with a bias
per head and gates its output with a sigmoid; gla and retention gate theirs with silu.
"""
import json
import os
import struct
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .registry import register_architecture, ConfigError
from .spec import PartSpec, LayerSpec, ScheduleEntry, ModelSpec

NORM_GAIN_OFFSET = 1.0
# the gated feed-forward of clamped_glu with no bound, a step for the gate's sigmoid and no shift: relu(gate) * up
FF_LIMIT, FF_ALPHA, FF_SHIFT = float("inf"), float("inf"), 0.0
DEFAULT_DECAY_RANK = 16
# positions are counted in 32-bit floats where angles are made: whole numbers are exact far beyond this; the rotation's
# tables are as long as the longest sequence the engine is set up for, never longer than this
MAX_POSITIONS = 1 << 20

# how the checkpoints spell things: layer i is "l<i>"; the one norm is the tensor l<i>.norm1 itself, the gates' tensors
# stand in the layer (l<i>.rg1, l<i>.rg1.b, l<i>.rg2, l<i>.rg2.b)
LAYER_TENSOR_NAMES = dict(mixer="mix", feed_forward="mlp", norm="norm1", gate="")
GATE_NAMES = ("rg1", "rg2")
MODEL_TENSOR_NAMES = dict(embedding="embed", final_norm="final.norm", head="head")
MIXER_TYPES = ("gla", "retention", "attention")


def _int(d, key, where, minimum=1):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, int) or v < minimum:
        raise ConfigError("config.json: %s %r must be an integer >= %d, got %r" % (where, key, minimum, v))
    return v


def _number(d, key, where, positive=False):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0):
        raise ConfigError("config.json: %s %r must be a %snumber, got %r" % (where, key, "positive " if positive else "", v))
    return float(v)


def _read_rot(m, dim, where):
    rot = m.get("rot")
    if rot is None:
        return None
    r = dict(base=_number(rot, "base", where + " rot", positive=True), dims=_int(rot, "dims", where + " rot", minimum=2))
    if r["dims"] % 2 or r["dims"] > dim:
        raise ConfigError("config.json: %s rot 'dims' must be even and at most dim %d, got %d" % (where, dim, r["dims"]))
    return r


def _read_mixer(kind, m, where):
    if not isinstance(m, dict):
        raise ConfigError("config.json: %s has no mixer sizes" % where)
    w = where + " mixer"
    out = {k: _int(m, k, w) for k in ("heads", "dim", "vdim")}
    if kind == "gla":
        out["tau"] = _number(m, "tau", w, positive=True)
        out["rank"] = None if m.get("rank") is None else _int(m, "rank", w)
    elif kind == "retention":
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != out["heads"] or any(
                isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError("config.json: %s 'decay' must list one number per head (%d), got %r" % (w, out["heads"], decay))
        out["decay"] = [float(d) for d in decay]
        out["rot"] = _read_rot(m, out["dim"], where)
    else:
        out["kv_heads"] = _int(m, "kv_heads", w)
        if out["heads"] % out["kv_heads"]:
            raise ConfigError("config.json: %s: heads %d is not a multiple of kv_heads %d" % (where, out["heads"], out["kv_heads"]))
        out["scale"] = _number(m, "scale", w)
        mask = m.get("mask")
        out["mask"] = dict(size=_int(mask, "size", where + " mask"), pool=_int(mask, "pool", where + " mask"))
        out["rot"] = _read_rot(m, out["dim"], where)
    return out


def _read_mlp(mlp, where):
    if mlp is None:
        return None
    kind = mlp.get("kind") if isinstance(mlp, dict) else None
    if kind == "dense":
        return dict(kind="dense", ff=_int(mlp, "ff", where + " mlp"))
    raise ConfigError("config.json: %s has the unknown feed-forward kind %r (known: dense)" % (where, kind))


def _shapes_in_header(folder):
    """{tensor name: shape} from the header of folder/model.safetensors (8 bytes of length, then JSON), or {}."""
    path = os.path.join(folder, "model.safetensors")
    try:
        with open(path, "rb") as f:
            n = struct.unpack("<Q", f.read(8))[0]
            head = json.loads(f.read(n))
    except (OSError, ValueError, struct.error):
        return {}
    return {k: tuple(v["shape"]) for k, v in head.items() if isinstance(v, dict) and "shape" in v}


@dataclass
class PuguzenLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


@register_architecture("Puguzen", "puguzen")
@dataclass
class PuguzenConfig:
    vocab: int
    width: int
    eps: float
    layers: List[PuguzenLayer] = field(default_factory=list)
    eos_token_ids: List[int] = field(default_factory=list)

    architecture = "Puguzen"

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
            kind = l.get("type") if isinstance(l, dict) else None
            if kind not in MIXER_TYPES:
                raise ConfigError("config.json: %s has the unknown mixer type %r (known: %s)" % (where, kind, ", ".join(MIXER_TYPES)))
            layers.append(PuguzenLayer(kind, _read_mixer(kind, l.get("mixer"), where), _read_mlp(l.get("mlp"), where)))
        eos = d.get("eos_token_id")
        eos = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, (list, tuple)) else [int(eos)])
        return cls(vocab=_int(d, "vocab", ""), width=_int(d, "width", ""), eps=_number(d["norm"], "eps", "norm", positive=True),
                   layers=layers, eos_token_ids=eos)

    def read_folder(self, folder):
        """What config.json leaves to the tensors' shapes: the rank of every gla layer's narrow decay projection, from the
        checkpoint's header."""
        shapes = _shapes_in_header(folder)
        for i, l in enumerate(self.layers):
            if l.type == "gla" and l.mixer.get("rank") is None:
                shape = shapes.get("l%d.mix.a1" % i)
                if shape is not None and len(shape) == 2:
                    l.mixer["rank"] = int(shape[0])
        return self

    def to_dict(self):
        def mixer(l):
            m = l.mixer
            out = {k: m[k] for k in ("heads", "dim", "vdim")}
            if l.type == "gla":
                out["tau"] = m["tau"]
                if m.get("rank") is not None:
                    out["rank"] = m["rank"]
            elif l.type == "retention":
                out["decay"] = list(m["decay"])
            else:
                out.update(kv_heads=m["kv_heads"], scale=m["scale"], mask=dict(m["mask"]))
            if m.get("rot") is not None:
                out["rot"] = dict(m["rot"])
            return out
        d = dict(architecture=self.architecture, vocab=self.vocab, width=self.width, norm=dict(eps=self.eps),
                 layers=[dict(type=l.type, mixer=mixer(l), mlp=None if l.mlp is None else dict(l.mlp)) for l in self.layers])
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    def _mixer_spec(self, l):
        W, m = self.width, l.mixer

        def position(kind):
            if m.get("rot") is None:
                return None
            return PartSpec(kind, dict(theta=m["rot"]["base"], rotary_dim=m["rot"]["dims"], max_positions=MAX_POSITIONS,
                                       wide_frequencies=True))
        if l.type == "gla":
            return PartSpec("gla", dict(hidden_size=W, num_heads=m["heads"], key_dim=m["dim"], value_dim=m["vdim"],
                                        decay_rank=m["rank"] if m.get("rank") is not None else DEFAULT_DECAY_RANK,
                                        tau=m["tau"], eps=self.eps))
        if l.type == "retention":
            return PartSpec("retention", dict(hidden_size=W, num_heads=m["heads"], key_dim=m["dim"], value_dim=m["vdim"],
                                              decay=tuple(m["decay"]), eps=self.eps, position=position("rope_neox")))
        return PartSpec("pooled_window_attention", dict(
            hidden_size=W, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"],
            scale=m["scale"], window=m["mask"]["size"], pool=m["mask"]["pool"], eps=self.eps,
            position=position("rope_interleaved"), unit_norm=True, head_bias=True, gated=True))

    def model_spec(self):
        W = self.width

        def norm():
            return PartSpec("rmsnorm", dict(size=W, eps=self.eps, gain_offset=NORM_GAIN_OFFSET, weight_name=""))
        layers = []
        for i, l in enumerate(self.layers):
            parts = dict(norm=norm(), mixer=self._mixer_spec(l))
            if l.mlp is not None:
                parts["feed_forward"] = PartSpec("clamped_glu", dict(hidden_size=W, intermediate_size=l.mlp["ff"], limit=FF_LIMIT,
                                                                     alpha=FF_ALPHA, shift=FF_SHIFT))
            parts["gate"] = PartSpec("sigmoid_projection", dict(hidden_size=W, names=GATE_NAMES[:1 if l.mlp is None else 2]))
            layers.append(LayerSpec(prefix="l%d" % i, parts=parts, arrangement="parallel_gated", names=dict(LAYER_TENSOR_NAMES)))
        spec = ModelSpec(
            hidden_size=W, vocab_size=self.vocab, layers=layers, schedule=[ScheduleEntry(i) for i in range(len(layers))],
            embedding=PartSpec("embedding", dict(vocab_size=self.vocab, hidden_size=W, weight_name="")),
            final_norm=norm(),
            head=PartSpec("lm_head", dict(vocab_size=self.vocab, hidden_size=W, tied=True)),
            max_positions=MAX_POSITIONS, eos_token_ids=list(self.eos_token_ids), names=dict(MODEL_TENSOR_NAMES))
        spec.validate()
        return spec
