"""Attention over a sliding window and, before it, over the means of whole blocks of tokens, with sigmoid weights."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, PagedSpec
from .linear import linear
from .registry import register_mixer


@register_mixer("pooled_window_attention")
class PooledWindowAttention(Part):
    """q = Wq x, k = Wk x, v = Wv x (no biases); grouped queries (query head h reads kv head h // (heads / kv heads)); q and k
    turned by position (`position`: a rotary part whose pairs are (2i, 2i + 1), over the first coordinates of a head, or
    None), then divided by their root mean square per head (`unit_norm`, eps).  Token i sees the tokens j with 0 <= i - j <
    `window`, and for every block of `pool` tokens that ends before them one key and one value: the means of the block's keys
    and values as the cache holds them.  The weight of a key is sigmoid(scale q . k + b_head), not normalised over keys
    (`head_bias`: whether there is a b).  The heads' results side by side, times sigmoid(Wg x) (`gated`), through Wo.
    Tensors: q, k, v, o, and pb (the b), g where the part has them.

    What a request keeps: the keys and values of the last max(window, pool) tokens, a token a row (pages behind that go
    back to the pool while the request runs), and a row per block of `pool` tokens with the block's means in 32-bit, made
    when the block's last token is written.  Scores, weights and sums are 32-bit."""

    capturable = True

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, value_dim, scale, window, pool, eps, dtype, device,
                 position=None, unit_norm=True, head_bias=True, gated=True):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads %d is not a multiple of num_kv_heads %d" % (num_heads, num_kv_heads))
        self.hidden_size, self.nh, self.nkv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.hd, self.vd = int(head_dim), int(value_dim)
        if not (0 < self.hd <= ops.POOLED_ATTENTION_MAX_DIM and 0 < self.vd <= ops.POOLED_ATTENTION_MAX_DIM):
            raise ValueError("heads of %d / %d are not supported: the kernel takes up to %d"
                             % (self.hd, self.vd, ops.POOLED_ATTENTION_MAX_DIM))
        self.window, self.pool = int(window), int(pool)
        if self.window < 1 or self.pool < 1:
            raise ValueError("window and pool must be positive, got %r and %r" % (window, pool))
        if position is not None and (getattr(position, "style", None) != "interleaved" or position.rotary_dim > self.hd):
            raise ValueError("this attention turns the pairs (2i, 2i + 1) of at most head_dim coordinates")
        self.position = position
        self.scale, self.eps = float(scale), float(eps)
        self.unit_norm, self.has_bias, self.gated = bool(unit_norm), bool(head_bias), bool(gated)
        self.dtype, self.device = dtype, device
        self.w_in = self.w_o = self.head_bias = self.b_in = self._extra = self.extra_columns = None

    def cache_spec(self):
        """[keys and values of the tokens a query or a block's mean can still need, the blocks' means]."""
        widths = (("k", self.nkv * self.hd), ("v", self.nkv * self.vd))
        return [PagedSpec(widths, window=max(self.window, self.pool)),
                PagedSpec(widths, every=self.pool, dtype=torch.float32)]

    def weight_specs(self):
        H = self.hidden_size
        specs = {"q": WeightSpec((self.nh * self.hd, H)), "k": WeightSpec((self.nkv * self.hd, H)),
                 "v": WeightSpec((self.nkv * self.vd, H)), "o": WeightSpec((H, self.nh * self.vd))}
        if self.has_bias:
            specs["pb"] = WeightSpec((self.nh,), std=1.0)
        if self.gated:
            specs["g"] = WeightSpec((self.nh * self.vd, H))
        return specs

    def bind_weights(self, t):
        self.w_in = torch.cat([t["q"], t["k"], t["v"]] + ([t["g"]] if self.gated else []), dim=0).contiguous()
        self.head_bias = t["pb"].float().contiguous() if self.has_bias else None
        self.w_o = t["o"]

    def append_columns(self, weight, bias):
        """Columns that someone else wants of the same rows (a block's gates): stacked behind the part's own matrix, so that
        one product makes both; forward leaves them in `extra_columns`."""
        own = self.w_in.shape[0]
        self._extra = (own, own + weight.shape[0])
        self.w_in = torch.cat([self.w_in, weight], dim=0).contiguous()
        self.b_in = torch.cat([torch.zeros((own,), dtype=bias.dtype, device=bias.device), bias]).contiguous()
        return True

    def kernel_modules(self):
        return ["pooled_attention", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x, step, cache):
        near, means = cache
        k_rows, v_rows = near.pages["k"], near.pages["v"]
        pk_rows, pv_rows = means.pages["k"], means.pages["v"]
        proj = linear(x, self.w_in, self.b_in, out_dtype=torch.float32)
        self.extra_columns = proj[:, self._extra[0]:self._extra[1]] if self._extra is not None else None
        cos, sin = self.position.tables() if self.position is not None else (None, None)
        q = ops.pooled_attention_prepare(proj, step.positions, cos, sin, near.slot_mapping, k_rows, v_rows, self.nh, self.nkv,
                                         self.hd, self.vd, self.eps, near.page_size, unit_norm=self.unit_norm, write=near.owner)
        if means.owner:
            ops.pooled_attention_pool(pk_rows, pv_rows, k_rows, v_rows, step, near.block_table, means.slot_mapping, self.nkv,
                                      self.hd, self.vd, self.pool, near.page_size)
        a = ops.pooled_attention(q, k_rows, v_rows, pk_rows, pv_rows, step, near.block_table, means.block_table,
                                 self.head_bias, self.nh, self.nkv, self.hd, self.vd, self.window, self.pool, near.page_size,
                                 self.scale, self.dtype, proj=proj if self.gated else None,
                                 gate_start=(self.nh + self.nkv) * self.hd + self.nkv * self.vd)
        return linear(a, self.w_o)
