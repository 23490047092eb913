"""Linear attention with a decay, as a recurrence over per-request state: gated linear attention (a decay per token and key
channel) and retention (a constant decay per head, rotary positions)."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, StateSpec
from .linear import linear
from .registry import register_mixer


class _DecayedLinearAttention(Part):
    """What the two kinds share: per head S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with a 32-bit state of one slot
    per request (zeros at a request's start); each head's o divided by its root mean square over the value columns (times
    a weight shared by the heads, where the kind has one), the heads side by side times silu(Wg x), then Wo.  All
    projections that read x are one product over the stacked weights, left in 32-bit; decays, rotation, state, output sum
    and norm are 32-bit."""

    capturable = True

    def __init__(self, hidden_size, num_heads, key_dim, value_dim, eps, dtype, device):
        if not 0 < key_dim <= ops.DECAY_SCAN_MAX_DIM:
            raise ValueError("key_dim %d is not supported: the recurrence kernel takes up to %d channels per head"
                             % (key_dim, ops.DECAY_SCAN_MAX_DIM))
        self.hidden_size, self.nh, self.dk, self.dv = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        self.eps, self.dtype, self.device = float(eps), dtype, device
        self.w_in = self.w_o = self.b_in = self._extra = self.extra_columns = None

    def cache_spec(self):
        return StateSpec((self.nh, self.dk, self.dv), torch.float32)

    # Columns that someone else wants of the same rows (a block's gates read what the mixer reads): their matrix is
    # stacked behind the mixer's own, so that ONE product makes both; forward leaves them in `extra_columns`.
    def append_columns(self, weight, bias):
        own = self.w_in.shape[0]
        self._extra = (own, own + weight.shape[0])
        self.w_in = torch.cat([self.w_in, weight], dim=0).contiguous()
        self.b_in = torch.cat([torch.zeros((own,), dtype=bias.dtype, device=bias.device), bias]).contiguous()
        return True

    def _project(self, x):
        proj = linear(x, self.w_in, self.b_in, out_dtype=torch.float32)
        self.extra_columns = proj[:, self._extra[0]:self._extra[1]] if self._extra is not None else None
        return proj

    def _projection_specs(self):
        H, k, v = self.hidden_size, self.nh * self.dk, self.nh * self.dv
        return {"q": WeightSpec((k, H)), "k": WeightSpec((k, H)), "v": WeightSpec((v, H)), "g": WeightSpec((v, H)),
                "o": WeightSpec((H, v))}

    def kernel_modules(self):
        return ["decay_scan", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    # column blocks of the stacked projection
    @property
    def _k0(self):
        return self.nh * self.dk

    @property
    def _v0(self):
        return 2 * self.nh * self.dk

    @property
    def _g0(self):
        return 2 * self.nh * self.dk + self.nh * self.dv

    @property
    def _rest0(self):
        return 2 * self.nh * self.dk + 2 * self.nh * self.dv


@register_mixer("gla")
class GatedLinearAttention(_DecayedLinearAttention):
    """q = Wq x / sqrt(key_dim), k = Wk x, v = Wv x; the decay of key channel c at token t is a = sigmoid(z)^(1 / tau) with z =
    Wa2 (Wa1 x) + b, a narrow projection and its widening (`decay_rank` between them), computed as exp(log sigmoid(z) / tau);
    the heads' outputs are normed with a weight over the value columns.  Tensors: q, k, v, g, o, norm, a1, a2, a2.b."""

    def __init__(self, hidden_size, num_heads, key_dim, value_dim, decay_rank, tau, eps, dtype, device):
        super().__init__(hidden_size, num_heads, key_dim, value_dim, eps, dtype, device)
        self.rank, self.tau = int(decay_rank), float(tau)
        if not 1 <= self.rank <= ops.GLA_DECAY_MAX_RANK or not self.tau > 0:
            raise ValueError("the decay needs a rank of 1 to %d and tau > 0, got %r and %r" % (ops.GLA_DECAY_MAX_RANK, decay_rank, tau))
        self.w_a2 = self.b_a2 = self.norm_weight = None

    def weight_specs(self):
        specs = self._projection_specs()
        k = self.nh * self.dk
        specs.update({"norm": WeightSpec((self.dv,), init="one_plus_normal"), "a1": WeightSpec((self.rank, self.hidden_size)),
                      "a2": WeightSpec((k, self.rank), std=0.5), "a2.b": WeightSpec((k,), std=2.0)})
        return specs

    def bind_weights(self, t):
        self.w_in = torch.cat([t["q"], t["k"], t["v"], t["g"], t["a1"]], dim=0).contiguous()
        self.w_a2 = t["a2"].float().t().contiguous()        # [rank, channels]: the kernel reads neighbouring channels
        self.b_a2 = t["a2.b"].float().contiguous()
        self.norm_weight = t["norm"].float().contiguous()
        self.w_o = t["o"]

    def forward(self, x, step, cache):
        proj = self._project(x)
        decay = ops.gla_decay(proj, self._rest0, self.w_a2, self.b_a2, self.tau)
        o = ops.decay_scan(proj, 0, self._k0, self._v0, cache.state, cache.slots, step, self.nh, self.dk, self.dv,
                           decay=decay, q_scale=self.dk ** -0.5)
        o = ops.head_norm_gate(o, self.norm_weight, self.eps, self.dtype, proj=proj, gate_start=self._g0)
        return linear(o, self.w_o)


@register_mixer("retention")
class Retention(_DecayedLinearAttention):
    """q = Wq x, k = Wk x, both turned by position on the rotary part's first coordinates (`position`: a rotary part whose pairs
    are (i, i + r / 2), or None), then k / sqrt(key_dim); head h decays by the constant decay[h]; the heads' outputs are divided
    by their root mean square, without a weight.  Tensors: q, k, v, g, o."""

    def __init__(self, hidden_size, num_heads, key_dim, value_dim, decay, eps, dtype, device, position=None):
        super().__init__(hidden_size, num_heads, key_dim, value_dim, eps, dtype, device)
        self.decay = [float(d) for d in decay]
        if len(self.decay) != self.nh:
            raise ValueError("%d decays for %d heads" % (len(self.decay), self.nh))
        if position is not None and (getattr(position, "style", None) != "neox" or position.rotary_dim > self.dk):
            raise ValueError("retention turns the pairs (i, i + r / 2) of at most key_dim coordinates")
        self.position = position
        self.head_decay = None

    def weight_specs(self):
        return self._projection_specs()

    def bind_weights(self, t):
        self.w_in = torch.cat([t["q"], t["k"], t["v"], t["g"]], dim=0).contiguous()
        self.w_o = t["o"]
        self.head_decay = torch.tensor(self.decay, dtype=torch.float32, device=self.w_in.device)

    def forward(self, x, step, cache):
        proj = self._project(x)
        cos, sin = self.position.tables() if self.position is not None else (None, None)
        o = ops.decay_scan(proj, 0, self._k0, self._v0, cache.state, cache.slots, step, self.nh, self.dk, self.dv,
                           head_decay=self.head_decay, cos=cos, sin=sin, k_scale=self.dk ** -0.5)
        o = ops.head_norm_gate(o, None, self.eps, self.dtype, proj=proj, gate_start=self._g0)
        return linear(o, self.w_o)


@register_mixer("lightning")
class LightningAttention(_DecayedLinearAttention):
    """q = silu(Wq x), k = silu(Wk x), v = silu(Wv x); head h decays by the constant decay[h] and nothing else scales; the
    heads' outputs side by side are divided by the root mean square over ALL of them at once, times a weight per channel,
    times sigmoid(Wg x); then Wo.  Tensors: q, k, v, g, o, norm."""

    def __init__(self, hidden_size, num_heads, key_dim, value_dim, decay, eps, dtype, device):
        super().__init__(hidden_size, num_heads, key_dim, value_dim, eps, dtype, device)
        self.decay = [float(d) for d in decay]
        if len(self.decay) != self.nh:
            raise ValueError("%d decays for %d heads" % (len(self.decay), self.nh))
        self.head_decay = self.norm_weight = None

    def weight_specs(self):
        specs = self._projection_specs()
        specs["norm"] = WeightSpec((self.nh * self.dv,), init="one_plus_normal", keep_32bit=True)
        return specs

    def bind_weights(self, t):
        self.w_in = torch.cat([t["q"], t["k"], t["v"], t["g"]], dim=0).contiguous()
        self.w_o = t["o"]
        self.norm_weight = t["norm"].float().contiguous()
        self.head_decay = torch.tensor(self.decay, dtype=torch.float32, device=self.w_in.device)

    def forward(self, x, step, cache):
        proj = self._project(x)
        o = ops.decay_scan(proj, 0, self._k0, self._v0, cache.state, cache.slots, step, self.nh, self.dk, self.dv,
                           head_decay=self.head_decay, silu_inputs=True)
        # the norm runs over the heads together: one "head" as wide as all of them
        o = ops.head_norm_gate(o.view(o.shape[0], 1, self.nh * self.dv), self.norm_weight, self.eps, self.dtype, proj=proj,
                               gate_start=self._g0, sigmoid_gate=True)
        return linear(o, self.w_o, parts_ok=True)
