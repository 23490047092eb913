"""Griffin's recurrent block: a gated branch beside a short convolution and a real-gated linear recurrent unit."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, StateSpec
from .linear import linear
from .registry import register_mixer


@register_mixer("rglru")
class RecurrentBlock(Part):
    """Two branches of `width` channels: y = gelu_tanh(Wy x + by) and u = conv(Wx x + bx) + bc, a causal convolution of `taps`
    taps over time on every channel (zeros before the sequence; the last taps - 1 rows of Wx x + bx are state).  The
    channels of u fall into `blocks` equal parts; in part b: r = sigmoid(Ra[b] u_b + ra[b]), i = sigmoid(Ri[b] u_b + ri[b]);
    a = exp(-rate * r * softplus(lam)); S_t = a S_(t-1) + sqrt(1 - a^2) * i * u from S = 0 (the first token has no special
    case); out = Wo (S * y).  Both branches are one product whose result stays 32-bit; convolution, gates, decay and state
    are 32-bit.  Tensors: y, y.b, x, x.b, conv [width, taps], conv.b, ra [blocks, out, in], ra.b [blocks, out], ri, ri.b,
    lam, o."""

    capturable = True

    def __init__(self, hidden_size, width, blocks, taps, dtype, device, rate=8.0):
        self.hidden_size, self.width, self.blocks, self.taps = int(hidden_size), int(width), int(blocks), int(taps)
        self.rate = float(rate)
        if self.blocks < 1 or self.width % self.blocks or self.width // self.blocks > ops.RGLRU_MAX_BLOCK:
            raise ValueError("%d channels in %d blocks (a block may hold up to %d)" % (self.width, self.blocks, ops.RGLRU_MAX_BLOCK))
        if not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError("the short convolution takes 1 to %d taps, got %r" % (ops.SHORT_CONV_MAX_TAPS, taps))
        self.dtype, self.device = dtype, device
        self.w_in = self.b_in = self.w_conv = self.b_conv = self.ra_t = self.ra_b = self.ri_t = self.ri_b = self.lam = self.w_o = None

    def cache_spec(self):
        """[the recurrence's state, the convolution's last inputs (None for one tap)]."""
        conv = StateSpec((self.taps - 1, self.width), torch.float32) if self.taps > 1 else None
        return [StateSpec((self.width,), torch.float32), conv]

    def weight_specs(self):
        H, C, B = self.hidden_size, self.width, self.blocks
        bw = C // B
        return {"y": WeightSpec((C, H)), "y.b": WeightSpec((C,), std=0.1), "x": WeightSpec((C, H)), "x.b": WeightSpec((C,), std=0.1),
                "conv": WeightSpec((C, self.taps), std=0.5, keep_32bit=True), "conv.b": WeightSpec((C,), std=0.1, keep_32bit=True),
                "ra": WeightSpec((B, bw, bw), keep_32bit=True), "ra.b": WeightSpec((B, bw), std=0.5, keep_32bit=True),
                "ri": WeightSpec((B, bw, bw), keep_32bit=True), "ri.b": WeightSpec((B, bw), std=0.5, keep_32bit=True),
                "lam": WeightSpec((C,), std=1.0, keep_32bit=True), "o": WeightSpec((H, C))}

    def bind_weights(self, t):
        self.w_in = torch.cat([t["y"], t["x"]], dim=0).contiguous()
        self.b_in = torch.cat([t["y.b"], t["x.b"]], dim=0).contiguous()
        self.w_conv = t["conv"].float().contiguous()
        self.b_conv = t["conv.b"].float().contiguous()
        # the gates' matrices [block][out][in] transposed: the kernel's neighbouring threads read neighbouring outputs
        self.ra_t = t["ra"].float().transpose(1, 2).contiguous()
        self.ri_t = t["ri"].float().transpose(1, 2).contiguous()
        self.ra_b = t["ra.b"].float().reshape(-1).contiguous()
        self.ri_b = t["ri.b"].float().reshape(-1).contiguous()
        self.lam = t["lam"].float().contiguous()
        self.w_o = t["o"]

    def kernel_modules(self):
        return ["rglru", "short_conv", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x, step, cache):
        state, conv = cache
        C = self.width
        proj = linear(x, self.w_in, self.b_in, out_dtype=torch.float32)
        u = ops.short_conv(proj[:, C:], self.w_conv, None if conv is None else conv.state, None if conv is None else conv.slots,
                           step, torch.float32, add_input=False, update=conv is not None and conv.owner, bias=self.b_conv)
        a, b, g = ops.rglru_gates(u, self.ra_t, self.ra_b, self.ri_t, self.ri_b, self.lam, self.blocks, self.rate, proj[:, :C])
        h = ops.rglru_scan(a, b, g, state.state, state.slots, step, self.dtype)
        return linear(h, self.w_o, parts_ok=True)
