"""Attention with values of their own width: optionally a short convolution over time behind the projections, a norm over
the whole projection of q and of k, biases, a sink (one score for all heads, or a learned one per head), a window or chunks."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, KVCacheSpec, StateSpec
from .linear import linear
from .registry import register_mixer


def _ceil16(n):
    return -(-int(n) // 16) * 16


@register_mixer("conv_attention")
class ConvAttention(Part):
    """q = Wq x, k = Wk x, v = Wv x (no biases); each channel of q, k and v then passes a causal convolution of `taps`
    taps over time (zeros before the sequence; the last taps - 1 projected rows of a request are its state); q and k are
    rotated by position (the rotary part may cover only the first coordinates of a head); grouped queries over the
    paged cache, scores times `scale`; `sink`: a score that every query sees beside its keys' and that has no value
    (None: a plain softmax); Wo on the heads' results.  Keys are head_dim wide, values value_dim.

    The attention kernels take one head size, so behind the projection every head is `padded` = the wider of the two
    widths, rounded up to 16: one kernel convolves, rotates and lays q out so, and writes keys and values so into their
    pages, with zeros where a head is narrower; Wo has columns of zeros there.  What the zeros add to a score or a
    result is exactly nothing."""

    capturable = True

    LEARNED = "learned"

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, value_dim, scale, dtype, device, taps=None,
                 position=None, sink=None, window=None, names=None, chunk=None, bias=False, qk_norm_eps=None):
        """Beyond the class's text: sink = ConvAttention.LEARNED reads one score per head from the tensor `sink`; chunk: a
        token sees the earlier tokens of its own chunk of `chunk` positions, counted from position 0 (in place of a
        window); bias: q, k, v and o have biases (`<name>.b`); qk_norm_eps: q and k are divided by the root mean square of
        the token's whole q (k) projection, all heads at once, and multiplied by the gains `q.norm`, `k.norm`, before the
        rotation (no convolution then)."""
        if num_heads % num_kv_heads:
            raise ValueError("num_heads %d is not a multiple of num_kv_heads %d" % (num_heads, num_kv_heads))
        self.hidden_size, self.nh, self.nkv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.hd, self.vd = int(head_dim), int(value_dim)
        self.padded = _ceil16(max(self.hd, self.vd))
        if not 0 < self.padded <= 256:
            raise ValueError("heads of %d / %d are not supported: the attention kernels take head sizes up to 256"
                             % (self.hd, self.vd))
        self.taps = int(taps) if taps else 1
        if not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError("the short convolution takes 1 to %d taps, got %r" % (ops.SHORT_CONV_MAX_TAPS, taps))
        self.has_conv = bool(taps)
        self.position = position
        if position is not None and position.rotary_dim > self.hd:
            raise ValueError("the rotation covers %d coordinates of a head of %d" % (position.rotary_dim, self.hd))
        self.scale = float(scale)
        self.learned_sink = sink == self.LEARNED
        self.sink = None if sink is None or self.learned_sink else float(sink)
        self.window = int(window) if window else None
        self.chunk = int(chunk) if chunk else None
        if self.window and self.chunk:
            raise ValueError("a window and chunks at once: %r, %r" % (window, chunk))
        self.bias = bool(bias)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        if self.qk_norm_eps is not None and taps:
            raise ValueError("the norm over the whole projection stands in front of no convolution")
        self.names = dict(q="q", k="k", v="v", o="o", conv="conv", sink="sink", bias="b", norm="norm")
        self.names.update(names or {})
        self.dtype, self.device = dtype, device
        self.width = (self.nh + self.nkv) * self.hd + self.nkv * self.vd        # the projection's channels
        self.w_qkv = self.w_conv = self.w_o = self.sinks = self.b_qkv = self.b_o = self.qk_gain = None

    def cache_spec(self):
        """[the convolution's state (or None), the pages of keys and values].  With chunks the cache keeps what a window of
        the chunk's length keeps: a token's own chunk starts inside that window, so every key it sees is held, and the
        pages before it go back to the pool while the request runs."""
        state = StateSpec((self.taps - 1, self.width), torch.float32) if self.taps > 1 else None
        return [state, KVCacheSpec(self.nkv, self.padded, self.window or self.chunk)]

    def weight_specs(self):
        n, H = self.names, self.hidden_size
        rows = {"q": self.nh * self.hd, "k": self.nkv * self.hd, "v": self.nkv * self.vd}
        specs = {n[r]: WeightSpec((rows[r], H)) for r in ("q", "k", "v")}
        specs[n["o"]] = WeightSpec((H, self.nh * self.vd))
        if self.has_conv:
            for r in ("q", "k", "v"):
                specs[n[r] + "." + n["conv"]] = WeightSpec((rows[r], self.taps), std=0.5, keep_32bit=True)
        if self.bias:
            for r in ("q", "k", "v"):
                specs[n[r] + "." + n["bias"]] = WeightSpec((rows[r],), std=0.1)
            specs[n["o"] + "." + n["bias"]] = WeightSpec((H,), std=0.1)
        if self.learned_sink:
            specs[n["sink"]] = WeightSpec((self.nh,), std=1.0, keep_32bit=True)
        if self.qk_norm_eps is not None:
            for r in ("q", "k"):
                specs[n[r] + "." + n["norm"]] = WeightSpec((rows[r],), init="one_plus_normal", keep_32bit=True)
        return specs

    def _padded_rows(self, t, heads, width):
        """t [heads * width, ...] -> [heads * padded, ...] with zeros behind every head's rows."""
        if width == self.padded:
            return t
        out = torch.zeros((heads, self.padded) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
        out[:, :width] = t.reshape((heads, width) + tuple(t.shape[1:]))
        return out.reshape((heads * self.padded,) + tuple(t.shape[1:]))

    def bind_weights(self, t):
        n = self.names
        self.w_qkv = torch.cat([t[n[r]] for r in ("q", "k", "v")], dim=0).contiguous()
        if self.has_conv:
            self.w_conv = torch.cat([t[n[r] + "." + n["conv"]].float() for r in ("q", "k", "v")], dim=0).contiguous()
        w_o = t[n["o"]]
        self.w_o = self._padded_rows(w_o.t().contiguous(), self.nh, self.vd).t().contiguous()
        dev = self.w_qkv.device
        self.sinks = None if self.sink is None else torch.full((self.nh,), self.sink, dtype=torch.float32, device=dev)
        if self.learned_sink:
            self.sinks = t[n["sink"]].float().contiguous()
        if self.bias:
            self.b_qkv = torch.cat([t[n[r] + "." + n["bias"]] for r in ("q", "k", "v")], dim=0).contiguous()
            self.b_o = t[n["o"] + "." + n["bias"]].contiguous()
        if self.qk_norm_eps is not None:
            self.qk_gain = torch.cat([t[n[r] + "." + n["norm"]].float() for r in ("q", "k")], dim=0).contiguous()

    def kernel_modules(self):
        mods = ["conv_rope_kv", "attention_generic", "gemm"]
        if self.dtype == torch.bfloat16:
            mods += ["gemm_skinny"]
            if self.padded in ops.MFMA_HEAD_DIMS:
                mods += [("attention_mfma", {"HEAD_DIM": self.padded})]
        return mods

    def forward(self, x, step, cache):
        state, kv = cache
        cos, sin = self.position.tables() if self.position is not None else (None, None)
        # the projection's rows stay 32-bit until they are convolved and rotated: what is cached is rounded once
        q = ops.conv_rope_kv(linear(x, self.w_qkv, self.b_qkv, out_dtype=torch.float32), self.w_conv,
                             None if state is None else state.state,
                             None if state is None else state.slots, step, cos, sin, kv.slot_mapping, kv.k_pages, kv.v_pages,
                             self.nh, self.nkv, self.hd, self.vd, self.padded, self.dtype, write_kv=kv.owner,
                             update_state=state is not None and state.owner, qk_gain=self.qk_gain,
                             qk_eps=self.qk_norm_eps or 0.0)
        a = ops.paged_attention(q, kv.k_pages, kv.v_pages, kv.block_table, step, self.nh, self.nkv, self.padded,
                                self.scale, self.window, sinks=self.sinks, chunk=self.chunk)
        return linear(a, self.w_o, self.b_o, parts_ok=self.b_o is None)
